"""CPU oracle for the block-sparse attention path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this
directory; only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may use it, and only as the checker.

Modules
-------
layout_oracle   block-index tables (bit-exact contract), to_sparse / to_dense
matmul_oracle   SDD / DSD / DDS dense semantics in float64 + backward algebra
softmax_oracle  block-sparse softmax forward / backward in float64
configs         seeded synthetic inputs of the five benchmark configurations
cpu_baseline    masked-dense torch-CPU timing used as the reported CPU baseline
bsa_oracle.c    plain-C block-walk restatement (second, independent checker)
"""
