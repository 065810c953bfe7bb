"""Benchmark of the block-sparse attention hot path on one MI355X.

Workload (BASELINE.json's metric): fp16, seq 4096, block 32, 16 batch*heads, head
dim 64, causal local-4 + every-8th-column mask (1530 of 16384 blocks, 9.3 %).
A step is one pass of the three products over that batch:

    SDD  scores = q @ k^T on the stored blocks       (reads q, k; writes 1530 blocks/head)
    DSD  out    = probs @ v                           (reads 1530 blocks/head, v)
    DDS  grad   = dy^T @ w  -> [16, 64, 4096]         (reads 1530 blocks/head, dy)

`value` = nnz-block TFLOP/s = 3 * 2 * nnz * 32 * 32 * 64 * 16 flop / step time.
The softmax (scale 1/8, causal) is timed in its own loop and reported in GB/s, and the
attention forward q, k, v -> out as one fused launch next to the chain of three.
Consecutive launches take the next of several resident operand sets (`--sets`, default 6), so the
blocks -- 88 % of a step's bytes, moved with non-temporal loads and stores -- come from and go to HBM on
every launch.  The dense operands and dense results (42 MB per step, not streamed) are another matter: over
6 sets they add up to 252 MB and can stay in the 256 MB last-level cache from one replay to the next, over 8
sets or more they cannot, and the step then takes 57 us instead of 48 (the SDD product, whose only reads
are q and k, goes from 12.5 to 19.9 us).  `step_regimes` reports the step over 3 sets (dense operands
cache-resident for certain, as behind the kernel that produced them) and over 16 (every operand from HBM)
beside the headline; `--sets 1` shows everything cache-resident.  Launches are replayed
from HIP graphs (the Python call path costs more than a 10 us kernel).

The K timed steps are run `--repeats` times (default 7); `ms_per_step` / `value` are the median of those
runs, the fastest and slowest are reported beside it.  A streaming copy of the softmax's byte count
(non-temporal 16-byte loads and stores, csrc/bench_yardstick.hip) is timed the same way in the same run:
`yardstick` says what a plain copy reaches on this box in this minute, and every kernel carries
`vs_copy` = its algorithmic GB/s over the copy's.  `torch.Tensor.copy_` over the same buffers (`torch_copy_us`,
`vs_torch_copy`) is the same yardstick from a kernel that is not this repository's.  The same bytes as a read
alone, as a write alone, and a launch that moves nothing are timed beside it (`read_us`, `write_us`, `empty_launch_us`).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--repeats R] [--sets S] [--no-cpu] [--no-attention] [--no-dense] [--no-configs]
    python bench.py --traffic-from FETCH_CSV WRITE_CSV      (summarises two counter runs, see profiles/)
"""
import argparse
import json
import os
import sys

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "experiments-pytorch-cuda-extension-for-sparse-matmul_amd"))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
# The per-kernel loops (not the headline step, whose K and W are the caller's) time at least this many graph
# replays of 12 launches after at least this many untimed ones: with fewer a kernel's figure moves by 3-5 %
# from run to run (clocks and caches have not settled after the 3 ms the loop then lasts).
KERNEL_LOOP_MIN_REPLAYS = 40
KERNEL_LOOP_MIN_WARMUP = 8
MFMA_F16_PEAK_TFLOPS = 2500.0  # dense fp16 MFMA


def kernel_sources_sha256() -> str:
    """One hash over the sources libbsa_hip.so is built from (csrc/build.py lists them)."""
    import hashlib
    csrc = os.path.join(ROOT, "experiments-pytorch-cuda-extension-for-sparse-matmul_amd", "csrc")
    sys.path.insert(0, csrc)
    import build as csrc_build
    h = hashlib.sha256()
    for name in sorted(csrc_build.SOURCES + [x for x in csrc_build.HEADERS if x.endswith(".hpp")]):
        with open(os.path.join(csrc, name), "rb") as f:
            h.update(name.encode() + b"\0" + f.read())
    return h.hexdigest()


# kernel name fragment -> row of the traffic table (rocprofv3 --pmc, one counter per run)
TRAFFIC_KERNELS = [("sdd_f16_kernel", "sdd"), ("dsd_runs_f16_kernel", "dsd"), ("gw_f16_kernel", "dds"),
                   ("softmax_fwd_kernel", "softmax"), ("attention_fwd", "attn"), ("attention_bwd_scores", "bwd_rows"),
                   ("attention_bwd_dkdv", "bwd_cols")]
CALIBRATION_KIB = 65536.0          # what the cold 64 MiB torch.neg in front of the timed loops reads, and writes


def summarise_traffic(fetch_csv: str, write_csv: str) -> None:
    """Turns the counter_collection.csv of a FETCH_SIZE run and of a WRITE_SIZE run of this script into
    profiles/bench_seq4096_hbm_traffic.json: bytes per launch of every kernel, each counter scaled by what it
    reads for the calibration kernel of known size, stamped with the kernel sources they were measured on."""
    import collections
    import csv

    def averages(path, counter):
        acc = collections.defaultdict(list)
        for row in csv.DictReader(open(path)):
            if row["Counter_Name"] != counter:
                continue
            name = row["Kernel_Name"]
            if "neg" in name and int(row.get("Grid_Size", "0")) >= (16 << 20) // 4:
                acc["calibration"].append(float(row["Counter_Value"]))
            for frag, op in TRAFFIC_KERNELS:
                if frag in name:
                    acc[op].append(float(row["Counter_Value"]))
                    break
        return {k: sum(v) / len(v) for k, v in acc.items()}

    fetch, write = averages(fetch_csv, "FETCH_SIZE"), averages(write_csv, "WRITE_SIZE")
    fetch_scale = CALIBRATION_KIB / fetch["calibration"]
    write_scale = CALIBRATION_KIB / write["calibration"]
    traffic = {op: int(round(1024 * (fetch[op] * fetch_scale + write.get(op, 0.0) * write_scale)))
               for _, op in TRAFFIC_KERNELS if op in fetch}
    out = {"workload": "seq4096_block32_causal-local4-stride8_nnz1530_bh16_d64", "unit": "bytes per launch",
           "fetch_scale": round(fetch_scale, 4), "write_scale": round(write_scale, 4),
           "kernel_sources_sha256": kernel_sources_sha256(), "traffic": traffic}
    with open(os.path.join(ROOT, "profiles", "bench_seq4096_hbm_traffic.json"), "w") as f:
        json.dump(out, f, indent=1)
    print("kernel    FETCH_SIZE raw   scaled MB   WRITE_SIZE raw   scaled MB   total MB")
    for _, op in TRAFFIC_KERNELS:
        if op in fetch:
            print(f"{op:9s} {fetch[op]:12.1f} {fetch[op] * fetch_scale * 1024 / 1e6:11.2f} {write.get(op, 0.0):16.1f} "
                  f"{write.get(op, 0.0) * write_scale * 1024 / 1e6:11.2f} {traffic[op] / 1e6:10.2f}")
    print(f"calibration: FETCH_SIZE {fetch['calibration']:.1f}, WRITE_SIZE {write['calibration']:.1f} KiB for "
          f"{CALIBRATION_KIB:.0f} KiB each way: scale factors {fetch_scale:.3f}, {write_scale:.3f}")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--repeats", type=int, default=7, help="times the K timed steps are run; the median is reported")
    ap.add_argument("--sets", type=int, default=6,
                    help="operand sets to rotate over (1 = the same operands every launch, which the 256 MB "
                         "infinity cache then serves)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-attention", action="store_true",
                    help="skip the fused attention legs (kernel traces of the hot path alone)")
    ap.add_argument("--no-dense", action="store_true", help="skip the dense torch.matmul yardstick")
    ap.add_argument("--no-configs", action="store_true", help="skip the per-configuration table")
    ap.add_argument("--no-graph", action="store_true", help="launch eagerly instead of replaying HIP graphs")
    ap.add_argument("--no-regimes", action="store_true",
                    help="skip the step over 3 and over 16 operand sets (dense operands cache-resident / from HBM)")
    ap.add_argument("--traffic-from", nargs=2, metavar=("FETCH_CSV", "WRITE_CSV"),
                    help="no GPU work: summarise two rocprofv3 --pmc runs of this script (FETCH_SIZE, WRITE_SIZE) into "
                         "profiles/bench_seq4096_hbm_traffic.json")
    args = ap.parse_args()
    if args.traffic_from:
        summarise_traffic(*args.traffic_from)
        return
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU; the path shards over batch*heads with no "
                 "communication, so --gpus N > 1 is not implemented.")

    import torch
    import __graft_entry__
    __graft_entry__.ensure_built()          # loads what is built; compiles only when nothing is
    import sparse
    import workloads as wl

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    B, D = 16, 64
    sets = []
    for s in range(args.sets):
        wk = wl.seq4096(batch=B, head_dim=D, seed=1004 + s)
        sets.append({k: (v.to(dev) if hasattr(v, "to") else v) for k, v in wk.items()})
    cpu_workload = wl.seq4096(batch=B, head_dim=D, seed=1004)
    layout = sparse.SparseLayout(sets[0]["mask"])
    nnz = layout.num_blocks
    es = 2

    flops_one = 2.0 * nnz * 32 * 32 * D * B
    seq = 4096
    bytes_alg = {
        "sdd": (seq * D + seq * D) * B * es + nnz * 1024 * B * es,
        "dsd": nnz * 1024 * B * es + seq * D * B * es + seq * D * B * es,
        "dds": seq * D * B * es + nnz * 1024 * B * es + D * seq * B * es,
        "softmax": 2 * nnz * 1024 * B * es,
    }

    ops = {
        "sdd": lambda w: sparse.matmul(w["q"], w["k"], "sdd", layout, False, True),
        "dsd": lambda w: sparse.matmul(w["scores"], w["v"], "dsd", layout, False, False),
        "dds": lambda w: sparse.matmul(w["v"], w["w"], "dds", layout, True, False),
        "softmax": lambda w: sparse.softmax(w["scores"], layout, 0.125, True),
    }

    def step(w):
        return ops["sdd"](w), ops["dsd"](w), ops["dds"](w)

    # parity spot check before timing: a fast wrong kernel is not a result
    with torch.no_grad():
        w0 = sets[0]
        o = ops["dsd"](w0)
        ref = torch.matmul(layout.to_dense(w0["scores"][:2]).float(), w0["v"][:2].float())
        err = ((o[:2].float() - ref).abs().max() / ref.abs().max()).item()
        assert err <= 2e-3, f"DSD parity check failed: {err}"

    # plain streaming kernel of known size (reads 64 MiB, writes 64 MiB, 16 bytes per lane), run on
    # cold caches: the yardstick for the FETCH_SIZE / WRITE_SIZE counters of a profiler run
    cal_src = torch.randn(16 << 20, dtype=torch.float32, device=dev)
    cal_dst = torch.empty_like(cal_src)
    flush = torch.zeros(256 << 20, dtype=torch.float32, device=dev)   # 1 GiB: evicts L2 and the 256 MB MALL
    flush.add_(1.0)
    torch.neg(cal_src, out=cal_dst)
    torch.cuda.synchronize()
    del cal_src, cal_dst, flush

    stream = torch.cuda.Stream()

    def make_runner(fn, reps=1, pool=None):
        """Callables that each run `reps` launches of fn; consecutive launches always take the next
        operand set of `pool` (default: all of them), inside a graph as well as from one graph to the next."""
        pool = sets if pool is None else pool
        with torch.cuda.stream(stream), torch.no_grad():
            for w in pool:
                fn(w)                          # build schedules / workspaces outside capture
            stream.synchronize()
        n_graphs = len(pool) if reps % len(pool) else 1
        runners = []
        for gi in range(n_graphs):
            order = [pool[(gi * reps + i) % len(pool)] for i in range(reps)]
            if args.no_graph:
                runners.append(lambda order=order: [fn(w) for w in order])
                continue
            g = torch.cuda.CUDAGraph()
            with torch.cuda.stream(stream), torch.no_grad():
                with torch.cuda.graph(g, stream=stream):
                    keep = [fn(w) for w in order]
            runners.append(lambda g=g, keep=keep: g.replay())
        return runners

    def timed(runners, n, warmup):
        """ms per call of n calls, between two events on the stream, synchronised before and after.  One more
        untimed call is queued between the synchronisation and the first event: the GPU is then still busy
        when the timed calls are submitted, so the interval between the events holds exactly the n calls and
        not the time the host needs to submit the first of them to an idle GPU (20-40 us, 2-4 % of 20 steps)."""
        with torch.cuda.stream(stream), torch.no_grad():
            for i in range(warmup):
                runners[i % len(runners)]()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            runners[(warmup - 1) % len(runners)]()
            e0.record(stream)
            for i in range(n):
                runners[(warmup + i) % len(runners)]()
            e1.record(stream)
            torch.cuda.synchronize()
        return e0.elapsed_time(e1) / n    # ms per call

    # headline: exactly K steps of the three products, several steps per graph replay (the largest of
    # these counts that divides K: a replay of one step spends 4 us between graphs that a training loop,
    # which captures whole iterations, does not)
    per_graph = next(g for g in (12, 10, 8, 6, 5, 4, 3, 2, 1) if args.steps % g == 0)
    step_runners = make_runner(step, per_graph)
    step_runs = sorted(timed(step_runners, args.steps // per_graph, -(-args.warmup // per_graph) if r == 0 else 1) / per_graph
                       for r in range(max(args.repeats, 1)))
    step_ms = step_runs[len(step_runs) // 2]
    value = 3 * flops_one / (step_ms * 1e-3) / 1e12

    # The two regimes either side of the default rotation.  Non-temporal streams (the blocks, 88 % of the bytes)
    # come from and go to HBM whatever the rotation; what does not stream -- per step 25 MB of dense operands
    # and 17 MB of dense results -- stays in the 256 MB last-level cache from one replay to the next while the
    # sets together hold less than that (up to 6 sets, and 6 is the edge), as it would behind the kernel that
    # produced it in a model.  Few sets: dense operands cache-resident for certain; many: everything from HBM.
    def step_regime(pool):
        runs = sorted(timed(make_runner(step, per_graph, pool), max(args.steps // per_graph, 1),
                            -(-args.warmup // per_graph) if r == 0 else 1) / per_graph for r in range(3))
        ms = runs[len(runs) // 2]
        return {"operand_sets": len(pool), "ms_per_step": round(ms, 5),
                "value": round(3 * flops_one / (ms * 1e-3) / 1e12, 2),
                "dense_MB_per_replay_cycle": round(len(pool) * 5 * seq * D * B * es / 1e6, 1)}

    regimes = {}
    if not args.no_regimes:
        regimes["dense_operands_cache_resident"] = step_regime(sets[:3])
        extra = []
        for s in range(len(sets), 16):
            wk = wl.seq4096(batch=B, head_dim=D, seed=1004 + s)
            extra.append({k: (v.to(dev) if hasattr(v, "to") else v) for k, v in wk.items()})
        regimes["every_operand_from_hbm"] = step_regime(sets + extra)
        del extra

    # yardstick: a non-temporal streaming copy of the softmax's bytes (50 MB in, 50 MB out), rotating over
    # as many buffer pairs as there are operand sets, from a HIP graph like every kernel below
    import ctypes
    bench_lib = ctypes.CDLL(os.path.join(ROOT, "experiments-pytorch-cuda-extension-for-sparse-matmul_amd", "csrc",
                                         "libbsa_bench.so"))
    bench_lib.bsa_bench_copy_nt.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
    copy_bytes = nnz * 1024 * B * es
    copy_dst = [torch.empty_like(w["scores"]) for w in sets]

    def copy_fn(w):
        i = next(k for k, v in enumerate(sets) if v is w)
        rc = bench_lib.bsa_bench_copy_nt(w["scores"].data_ptr(), copy_dst[i].data_ptr(), copy_bytes,
                                         torch.cuda.current_stream().cuda_stream)
        assert rc == 0, rc
        return copy_dst[i]

    REPS = 2 * len(sets)
    copy_ms = timed(make_runner(copy_fn, REPS), max(args.steps // REPS, KERNEL_LOOP_MIN_REPLAYS), max(args.warmup // REPS, KERNEL_LOOP_MIN_WARMUP)) / REPS
    assert torch.equal(copy_dst[0], sets[0]["scores"])
    copy_gbs = 2 * copy_bytes / (copy_ms * 1e-3) / 1e9
    yardstick = {"what": "non-temporal copy, 16 B per lane, 4 loads in flight", "bytes_in": copy_bytes, "bytes_out": copy_bytes,
                 "us": round(copy_ms * 1e3, 3), "GBps": round(copy_gbs, 1), "hbm_frac": round(copy_gbs / HBM_PEAK_GBS, 4)}
    # an independent yardstick: the same bytes moved by torch's own device-to-device copy (not a kernel of this
    # repository), in the same graph harness over the same rotating buffers
    def torch_copy_fn(w):
        i = next(k for k, v in enumerate(sets) if v is w)
        copy_dst[i].copy_(w["scores"])
        return copy_dst[i]

    tc_ms = timed(make_runner(torch_copy_fn, REPS), max(args.steps // REPS, KERNEL_LOOP_MIN_REPLAYS), max(args.warmup // REPS, KERNEL_LOOP_MIN_WARMUP)) / REPS
    yardstick["torch_copy_us"] = round(tc_ms * 1e3, 3)
    yardstick["torch_copy_GBps"] = round(2 * copy_bytes / (tc_ms * 1e-3) / 1e9, 1)
    yardstick["torch_copy_hbm_frac"] = round(2 * copy_bytes / (tc_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)
    # the same stream as a read alone and as a write alone, and a launch that moves nothing: what the hardware
    # does with 50 MB in one direction, and what a launch costs before its first byte
    bench_lib.bsa_bench_read_nt.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
    bench_lib.bsa_bench_write_nt.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
    bench_lib.bsa_bench_empty.argtypes = [ctypes.c_uint, ctypes.c_void_p]
    sink = torch.zeros(1, dtype=torch.int32, device=dev)

    def checked(rc):
        assert rc == 0, rc
        return sink

    def index_of(w):
        return next(k for k, v in enumerate(sets) if v is w)

    for key, fn in (("read", lambda w: checked(bench_lib.bsa_bench_read_nt(w["scores"].data_ptr(), sink.data_ptr(), copy_bytes,
                                                                             torch.cuda.current_stream().cuda_stream))),
                    ("write", lambda w: checked(bench_lib.bsa_bench_write_nt(copy_dst[index_of(w)].data_ptr(), copy_bytes,
                                                                               torch.cuda.current_stream().cuda_stream))),
                    ("empty_launch", lambda w: checked(bench_lib.bsa_bench_empty(2048, torch.cuda.current_stream().cuda_stream)))):
        ms = timed(make_runner(fn, REPS), max(args.steps // REPS, KERNEL_LOOP_MIN_REPLAYS), max(args.warmup // REPS, KERNEL_LOOP_MIN_WARMUP)) / REPS
        yardstick[key + "_us"] = round(ms * 1e3, 3)
        if key != "empty_launch":
            yardstick[key + "_GBps"] = round(copy_bytes / (ms * 1e-3) / 1e9, 1)
    del copy_dst

    # per-kernel average launch duration: REPS launches per graph, events around the replays; like the headline,
    # the median of `--repeats` runs (a launch's time depends on what the last-level cache holds when it starts,
    # which shifts from run to run), fastest and slowest beside it
    per_op = {}
    for name, fn in ops.items():
        runners = make_runner(fn, REPS)
        runs = sorted(timed(runners, max(args.steps // REPS, KERNEL_LOOP_MIN_REPLAYS), max(args.warmup // REPS, KERNEL_LOOP_MIN_WARMUP) if r == 0 else 1) / REPS
                      for r in range(max(args.repeats, 1)))
        ms = runs[len(runs) // 2]
        gbs = bytes_alg[name] / (ms * 1e-3) / 1e9
        per_op[name] = {"us": round(ms * 1e3, 3), "GBps": round(gbs, 1), "hbm_frac": round(gbs / HBM_PEAK_GBS, 4),
                        "vs_copy": round(gbs / copy_gbs, 3), "vs_torch_copy": round(gbs / yardstick["torch_copy_GBps"], 3),
                        "algorithmic_MB": round(bytes_alg[name] / 1e6, 3),
                        "us_min": round(runs[0] * 1e3, 3), "us_max": round(runs[-1] * 1e3, 3)}
        if name != "softmax":
            tf = flops_one / (ms * 1e-3) / 1e12
            per_op[name]["nnz_TFLOPs"] = round(tf, 2)
            per_op[name]["mfma_frac"] = round(tf / MFMA_F16_PEAK_TFLOPS, 4)

    attention = None
    if not args.no_attention:
        # attention forward as a whole, q k v -> out: one fused launch against the chain of three launches
        # (the two products of a forward pass are 2 * flops_one); not part of `value`
        def chain(w):
            s = sparse.matmul(w["q"], w["k"], "sdd", layout, False, True)
            return sparse.matmul(sparse.softmax(s, layout, 0.125, True), w["v"], "dsd", layout)

        def fused(w):
            return sparse.attention(w["q"], w["k"], w["v"], layout, 0.125, True)

        with torch.no_grad():
            a, b = fused(sets[0]), chain(sets[0])
            err = ((a.float() - b.float()).abs().max() / b.float().abs().max()).item()
            assert err <= 2e-3, f"fused attention differs from the chain: {err}"
        attention = {}
        for name, fn in (("fused", fused), ("chain", chain)):
            ms = timed(make_runner(fn, REPS), max(args.steps // REPS, KERNEL_LOOP_MIN_REPLAYS), max(args.warmup // REPS, KERNEL_LOOP_MIN_WARMUP)) / REPS
            attention[name + "_us"] = round(ms * 1e3, 3)
            attention[name + "_nnz_TFLOPs"] = round(2 * flops_one / (ms * 1e-3) / 1e12, 2)
        attention["speedup"] = round(attention["chain_us"] / attention["fused_us"], 2)

        # the backward pass of the same attention: a walk over the rows (dq) and one over the columns (dk, dv)
        # that keep the probabilities and score gradients in registers, against the seven launches of the
        # unfused chain (gradients of q, k, v from dout)
        from sparse.kernel import sparse_ops
        rows, cols = layout.row_layout, layout.col_layout
        for w in sets:
            w["dout"] = torch.randn_like(w["q"])
            w["out"], w["lse"] = sparse_ops.sparse_attention_forward(w["q"], w["k"], w["v"], rows[0], rows[1], 0.125, True,
                                                                     cols, return_lse=True)

        def products(p, ds, w):
            return (sparse.matmul(ds, w["k"], "dsd", layout), sparse.matmul(ds, w["q"], "dsd", layout, True, False),
                    sparse.matmul(p, w["dout"], "dsd", layout, True, False))

        def backward_fused(w):
            return sparse_ops.sparse_attention_backward(w["q"], w["k"], w["v"], w["dout"], w["out"], w["lse"],
                                                        rows[0], rows[1], cols[0], cols[1], 0.125, True)

        def backward_chain(w):
            p = sparse.softmax(sparse.matmul(w["q"], w["k"], "sdd", layout, False, True), layout, 0.125, True)
            dp = sparse.matmul(w["dout"], w["v"], "sdd", layout, False, True)
            ds = sparse_ops.sparse_softmax_backward(p, dp, rows[0], rows[1], 0.125, cols)
            return products(p, ds, w)

        with torch.no_grad():
            for a, b in zip(backward_fused(sets[0]), backward_chain(sets[0])):
                err = ((a.float() - b.float()).abs().max() / b.float().abs().max()).item()
                assert err <= 4e-3, f"attention backward differs from the chain: {err}"
        for name, fn in (("backward_us", backward_fused), ("backward_chain_us", backward_chain)):
            ms = timed(make_runner(fn, REPS), max(args.steps // REPS, KERNEL_LOOP_MIN_REPLAYS), max(args.warmup // REPS, KERNEL_LOOP_MIN_WARMUP)) / REPS
            attention[name] = round(ms * 1e3, 3)

    def graph_time_us(fn, reps, iters=10):
        """Average duration of one call of fn(), `reps` calls per HIP graph, on its own operands."""
        with torch.cuda.stream(stream), torch.no_grad():
            fn()
            stream.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=stream):
                keep = [fn() for _ in range(reps)]
            for _ in range(2):
                g.replay()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            e0.record(stream)
            for _ in range(iters):
                g.replay()
            e1.record(stream)
            torch.cuda.synchronize()
            del keep
        return e0.elapsed_time(e1) / (iters * reps) * 1e3

    # The same three products as DENSE fp16 matmuls at the full M, N, K (torch.matmul: rocBLAS / hipBLASLt),
    # the "dense-MFMA-equivalent" yardstick: what the library reaches when it multiplies all 16384 blocks
    # of a head, against what these kernels reach on the 1530 stored ones.
    dense_equivalent = None
    if not args.no_dense:
        w = sets[0]
        with torch.no_grad():
            p_dense = layout.to_dense(w["scores"])                  # [16, 4096, 4096]
            w_dense = layout.to_dense(w["w"])
            kt, dyt = w["k"].transpose(-1, -2), w["v"].transpose(-1, -2)
        dense_flops = 2.0 * seq * seq * D * B
        dense_equivalent = {}
        for name, fn in (("sdd", lambda: torch.matmul(w["q"], kt)), ("dsd", lambda: torch.matmul(p_dense, w["v"])),
                         ("dds", lambda: torch.matmul(dyt, w_dense))):
            us = graph_time_us(fn, 4)
            dtf = dense_flops / (us * 1e-6) / 1e12
            dense_equivalent[name] = {
                "dense_us": round(us, 2), "dense_TFLOPs": round(dtf, 1),
                "dense_mfma_frac": round(dtf / MFMA_F16_PEAK_TFLOPS, 4),
                "nnz_TFLOPs_over_dense_TFLOPs": round(per_op[name]["nnz_TFLOPs"] / dtf, 3),
                "time_dense_over_sparse": round(us / per_op[name]["us"], 2)}
        del p_dense, w_dense

    # the five configurations of the coverage table, each on its own operands (one set: the small ones are
    # cache-resident), per launch from a HIP graph and eagerly (Python call path included)
    configs = None
    if not args.no_configs:
        import time
        configs = {}

        def run_config(name, fn, reps, flops=None, nbytes=None, cache_resident=False):
            us = graph_time_us(fn, reps)
            with torch.no_grad():
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for _ in range(50):
                    fn()
                torch.cuda.synchronize()
                eager = (time.perf_counter() - t0) / 50 * 1e6
            row = {"us": round(us, 2), "eager_us": round(eager, 1)}
            if cache_resident:      # one small operand set, replayed: served by the 256 MB last-level cache, and
                row["cache_resident"] = True    # the figure moves by up to 2x from run to run
            if flops:
                row["nnz_TFLOPs"] = round(flops / (us * 1e-6) / 1e12, 2)
            if nbytes:
                row["GBps"] = round(nbytes / (us * 1e-6) / 1e9, 1)
                row["hbm_frac"] = round(row["GBps"] / HBM_PEAK_GBS, 4)
            configs[name] = row

        def on_gpu(c):
            return {k: (v.to(dev) if hasattr(v, "to") else v) for k, v in c.items()}

        c = on_gpu(wl.config1())
        l1 = sparse.SparseLayout(c["mask"])
        run_config("config1_sdd_fp32_16x16", lambda: sparse.matmul(c["a"], c["b"], "sdd", l1, False, True), 20,
                   flops=2.0 * l1.num_blocks * 32 * 32 * 64,
                   nbytes=(2 * 512 * 64 + l1.num_blocks * 1024) * 4, cache_resident=True)
        c2 = on_gpu(wl.config2())
        l2 = sparse.SparseLayout(c2["mask"])
        run_config("config2_dsd_fp16_64x64_local", lambda: sparse.matmul(c2["a"], c2["b"], "dsd", l2), 20,
                   flops=2.0 * l2.num_blocks * 32 * 32 * 64 * 16,
                   nbytes=(l2.num_blocks * 1024 + 2 * 2048 * 64) * 16 * 2, cache_resident=True)
        c3 = on_gpu(wl.config3())
        run_config("config3_softmax_fp16_causal", lambda: sparse.softmax(c3["x"], layout, 0.125, True), 12,
                   nbytes=2 * nnz * 1024 * 16 * 2)
        c4 = on_gpu(wl.config4())
        run_config("config4_dds_fp16", lambda: sparse.matmul(c4["a"], c4["b"], "dds", layout, True, False), 12,
                   flops=flops_one, nbytes=bytes_alg["dds"])
        run_config("config4_as_dsd_TF", lambda: sparse.matmul(c4["b"], c4["a"], "dsd", layout, True, False), 12,
                   flops=flops_one, nbytes=bytes_alg["dds"])
        del c, c2, c3, c4

        # The headline mask coarsened to blocks of 64 (causal, window of 2 blocks, every 8th block column: 399
        # blocks = 1596 tiles, 9.7 %): the DSD product through the kernel that owns whole 64x64 blocks and through
        # the walk over the same layout's 32x32 tiles, on rotating operand sets like the headline.
        from sparse import _ops as ops64
        ci, cj = torch.arange(64)[:, None], torch.arange(64)[None, :]
        l64 = sparse.SparseLayout(((cj <= ci) & ((ci - cj < 2) | (cj % 8 == 0))).long(), block=64)
        g64 = torch.Generator().manual_seed(1064)
        sets64 = [(torch.rand(B, l64.num_blocks, 32, 32, generator=g64).half().to(dev),
                   torch.randn(B, 4096, D, generator=g64).half().to(dev)) for _ in range(len(sets))]
        turn = [0]

        def dsd64():
            p64, v64 = sets64[turn[0] % len(sets64)]
            turn[0] += 1
            return sparse.matmul(p64, v64, "dsd", l64)

        f64 = 2.0 * l64.num_blocks * 32 * 32 * D * B
        b64 = (l64.num_blocks * 1024 + 2 * 4096 * D) * B * es
        run_config("block64_mask_dsd_as_32x32_tiles", dsd64, 2 * len(sets64), flops=f64, nbytes=b64)
        ops64.USE_BLOCK64_KERNEL = True
        try:
            run_config("block64_mask_dsd_block_kernel", dsd64, 2 * len(sets64), flops=f64, nbytes=b64)
        finally:
            ops64.USE_BLOCK64_KERNEL = False
        configs["block64_mask_tiles"] = l64.num_blocks
        del sets64

        # The headline products in fp32 (v_mfma_f32_32x32x2_f32: 157 TFLOP/s bounds them before HBM does), on
        # rotating operand sets (three: an fp32 set is twice the bytes).
        sets32 = [{k: w[k].float() for k in ("q", "k", "v", "scores", "w")} for w in sets[:3]]
        turn32 = [0]

        def next32():
            turn32[0] += 1
            return sets32[turn32[0] % len(sets32)]

        b32 = (nnz * 1024 + 2 * seq * D) * B * 4
        for name, fn in (("sdd", lambda: (lambda w: sparse.matmul(w["q"], w["k"], "sdd", layout, False, True))(next32())),
                         ("dsd", lambda: (lambda w: sparse.matmul(w["scores"], w["v"], "dsd", layout))(next32())),
                         ("dds", lambda: (lambda w: sparse.matmul(w["v"], w["w"], "dds", layout, True, False))(next32()))):
            run_config(f"seq4096_{name}_fp32", fn, 2 * len(sets32), flops=flops_one, nbytes=b32)
            configs[f"seq4096_{name}_fp32"]["mfma_f32_frac"] = round(
                configs[f"seq4096_{name}_fp32"]["nnz_TFLOPs"] / 157.3, 4)
        # SDD in fp32 at head dim 128 (four k-blocks: the widest the tiled kernel keeps resident, 78 KB of LDS per
        # workgroup with the package's schedule)
        g128 = torch.Generator().manual_seed(1128)
        qk128 = [(torch.randn(B, seq, 128, generator=g128).to(dev), torch.randn(B, seq, 128, generator=g128).to(dev))
                 for _ in range(2)]
        turn128 = [0]

        def sdd128():
            turn128[0] += 1
            q128, k128 = qk128[turn128[0] % 2]
            return sparse.matmul(q128, k128, "sdd", layout, False, True)

        run_config("seq4096_sdd_fp32_k128", sdd128, 4, flops=2 * flops_one, nbytes=(nnz * 1024 + 2 * seq * 128) * B * 4)
        configs["seq4096_sdd_fp32_k128"]["mfma_f32_frac"] = round(configs["seq4096_sdd_fp32_k128"]["nnz_TFLOPs"] / 157.3, 4)
        del sets32, qk128
        c5 = on_gpu(wl.config5())
        l5 = sparse.SparseLayout(c5["mask"])
        n5, b5 = l5.num_blocks, 48

        def chain5():
            sc = sparse.matmul(c5["q"], c5["k"], "sdd", l5, False, True)
            return sparse.matmul(sparse.softmax(sc, l5, 0.125, False), c5["v"], "dsd", l5)

        f5 = 2 * 2.0 * n5 * 32 * 32 * 64 * b5
        run_config("config5_chain_sdd_softmax_dsd_fp16_8192", chain5, 4, flops=f5,
                   nbytes=(4 * 8192 * 64 + 4 * n5 * 1024) * b5 * 2)
        run_config("config5_fused_attention", lambda: sparse.attention(c5["q"], c5["k"], c5["v"], l5, 0.125, False), 4,
                   flops=f5, nbytes=4 * 8192 * 64 * b5 * 2)
        with torch.no_grad():
            from sparse.kernel import sparse_ops as ops5
            rl5, cl5 = l5.row_layout, l5.col_layout
            out5, lse5 = ops5.sparse_attention_forward(c5["q"], c5["k"], c5["v"], rl5[0], rl5[1], 0.125, False, cl5,
                                                       return_lse=True)
            dout5 = torch.randn_like(c5["q"])
        # the two-launch backward of the fused attention: five block products per stored block
        run_config("config5_fused_attention_backward",
                   lambda: ops5.sparse_attention_backward(c5["q"], c5["k"], c5["v"], dout5, out5, lse5, rl5[0], rl5[1],
                                                          cl5[0], cl5[1], 0.125, False), 4,
                   flops=2.5 * f5, nbytes=(8 * 8192 * 64) * b5 * 2)
        del out5, lse5, dout5
        with torch.no_grad():
            sc5 = sparse.matmul(c5["q"], c5["k"], "sdd", l5, False, True)
            p5 = sparse.softmax(sc5, l5, 0.125, False)
        blk5, dense5 = n5 * 1024 * b5 * 2, 8192 * 64 * b5 * 2
        run_config("config5_sdd_alone", lambda: sparse.matmul(c5["q"], c5["k"], "sdd", l5, False, True), 4,
                   flops=f5 / 2, nbytes=2 * dense5 + blk5)
        run_config("config5_softmax_alone", lambda: sparse.softmax(sc5, l5, 0.125, False), 4, nbytes=2 * blk5)
        run_config("config5_dsd_alone", lambda: sparse.matmul(p5, c5["v"], "dsd", l5), 4,
                   flops=f5 / 2, nbytes=blk5 + 2 * dense5)
        configs["config5_nnz"] = n5
        del c5, sc5, p5

    # HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (profiles/): same
    # workload, same kernels.  The file names the kernel sources it was measured on; when they have
    # changed since (or the file is absent) the figure is stale and null is reported instead.
    traffic = {}
    try:
        with open(os.path.join(ROOT, "profiles", "bench_seq4096_hbm_traffic.json")) as f:
            measured = json.load(f)
        if measured.get("kernel_sources_sha256") == kernel_sources_sha256():
            traffic = measured["traffic"]
    except (OSError, ValueError, KeyError):
        pass
    for name in per_op:
        per_op[name]["traffic_bytes"] = traffic.get(name)

    dominant = max(("sdd", "dsd", "dds"), key=lambda n: per_op[n]["us"])
    roofline = {"kernel": dominant, "bound": "hbm", "achieved": per_op[dominant]["GBps"], "peak": HBM_PEAK_GBS,
                "unit": "GB/s", "frac": per_op[dominant]["hbm_frac"], "traffic": traffic.get(dominant)}

    result = {
        "metric": "nnz-block TFLOP/s SDD/DSD/DDS fp16 @seq4096; softmax GB/s; % of roofline",
        "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(step_ms, 5), "ms_per_step_min": round(step_runs[0], 5), "ms_per_step_max": round(step_runs[-1], 5),
        "repeats": len(step_runs), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": "seq4096_block32_causal-local4-stride8_nnz1530_bh16_d64: SDD(q,k^T)+DSD(p,v)+DDS(dy^T,w) per step",
                   "operand_sets": args.sets, "launch": "eager" if args.no_graph else f"hip-graph replay, {per_graph} steps per graph"},
        "roofline": roofline,
        "step_regimes": regimes,
        "yardstick": yardstick,
        "softmax": {"GBps": per_op["softmax"]["GBps"], "us": per_op["softmax"]["us"],
                    "roofline": {"bound": "hbm", "achieved": per_op["softmax"]["GBps"], "peak": HBM_PEAK_GBS,
                                 "unit": "GB/s", "frac": per_op["softmax"]["hbm_frac"],
                                 "traffic": traffic.get("softmax")}},
        "kernels": per_op,
        "attention": attention,
        "dense_equivalent": dense_equivalent,
        "configs": configs,
    }

    if not args.no_cpu:
        from oracle import cpu_baseline
        heads = 2
        cb = cpu_baseline.time_seq4096(cpu_workload, heads=heads, repeats=5)
        cpu_tf = 3 * (flops_one / B * heads) / cb["matmul"] / 1e12
        result["cpu_baseline"] = {
            "value": round(cpu_tf, 5), "unit": "TFLOP/s", "cores": cb["cores"], "kind": "port",
            "sample": f"{heads} of {B} heads of the same workload, masked-dense torch fp32 on the host, median of 5; "
                      f"softmax on the same sample: {bytes_alg['softmax'] / B * heads / cb['softmax'] / 1e9:.3f} GB/s"}
    print(json.dumps(result))


if __name__ == "__main__":
    main()
