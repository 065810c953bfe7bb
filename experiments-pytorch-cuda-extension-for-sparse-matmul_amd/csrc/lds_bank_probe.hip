// Timing probe of the LDS banks of gfx950, the measurement behind lds_bank_model.py.
//
//   hipcc --offload-arch=gfx950 -O3 -o lds_bank_probe lds_bank_probe.hip && ./lds_bank_probe
//
// One workgroup of 4 wavefronts (one per SIMD) issues batches of 16 independent LDS
// reads per lane pattern and reports clocks per wave-instruction.  The patterns come
// in pairs that two bank geometries tell apart:
//   linear        lane l -> 16 l                       conflict-free everywhere
//   stride32      lane l -> 32 l                       two-way conflict everywhere
//   halfwin       lane l -> 16 (l % 8) + 256 (l / 8)   two-way with 64 banks and 16-lane phases,
//                                                      conflict-free with 32 banks and 8-lane phases
//   rows64 / rows64x: one 16-byte piece of 64-byte rows, lane l -> 64 l (+ XOR swizzles)
#include <hip/hip_runtime.h>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#define CK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("HIP error %s line %d\n", hipGetErrorString(e_), __LINE__); exit(1); } } while (0)

typedef unsigned int u4 __attribute__((ext_vector_type(4)));
typedef unsigned int u2 __attribute__((ext_vector_type(2)));

template <int WIDTH>
__global__ __launch_bounds__(256) void probe(const int *offs, unsigned long long *out, int iters)
{
    extern __shared__ __align__(16) unsigned char lds[];
    const int l = threadIdx.x & 63;
    for (int i = threadIdx.x; i < 16384; i += 256) ((uint32_t *)lds)[i] = i;
    __syncthreads();
    const unsigned addr = (unsigned)(uintptr_t)lds + offs[l];
    unsigned acc = 0;
    __syncthreads();
    unsigned long long t0 = __builtin_readcyclecounter();
    for (int it = 0; it < iters; ++it) {
        if (WIDTH == 16) {
            u4 v[16];
#pragma unroll
            for (int u = 0; u < 16; ++u) asm volatile("ds_read_b128 %0, %1" : "=v"(v[u]) : "v"(addr));
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
            for (int u = 0; u < 16; ++u) acc ^= v[u].x;
        } else if (WIDTH == 8) {
            u2 v[16];
#pragma unroll
            for (int u = 0; u < 16; ++u) asm volatile("ds_read_b64 %0, %1" : "=v"(v[u]) : "v"(addr));
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
            for (int u = 0; u < 16; ++u) acc ^= v[u].x;
        } else if (WIDTH == 4) {
            unsigned v[16];
#pragma unroll
            for (int u = 0; u < 16; ++u) asm volatile("ds_read_b32 %0, %1" : "=v"(v[u]) : "v"(addr));
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
            for (int u = 0; u < 16; ++u) acc ^= v[u];
        } else if (WIDTH == -16) {   // ds_write_b128
            u4 w = {acc, acc + 1, acc + 2, acc + 3};
#pragma unroll
            for (int u = 0; u < 16; ++u) asm volatile("ds_write_b128 %0, %1" ::"v"(addr), "v"(w) : "memory");
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            acc += 1;
        } else if (WIDTH == -64) {   // ds_write_b64
            u2 w = {acc, acc + 1};
#pragma unroll
            for (int u = 0; u < 16; ++u) asm volatile("ds_write_b64 %0, %1" ::"v"(addr), "v"(w) : "memory");
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            acc += 1;
        } else if (WIDTH == -32) {   // ds_write_b32
#pragma unroll
            for (int u = 0; u < 16; ++u) asm volatile("ds_write_b32 %0, %1" ::"v"(addr), "v"(acc) : "memory");
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            acc += 1;
        } else {                     // ds_read_b64_tr_b16
            u2 v[16];
#pragma unroll
            for (int u = 0; u < 16; ++u) asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(v[u]) : "v"(addr));
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
            for (int u = 0; u < 16; ++u) acc ^= v[u].x;
        }
    }
    unsigned long long t1 = __builtin_readcyclecounter();
    if (threadIdx.x == 0) out[0] = t1 - t0;
    if (acc == 0x12345u) out[1] = acc;
}

template <int WIDTH>
static double run(const std::vector<int> &offs)
{
    int *d;
    unsigned long long *o;
    CK(hipMalloc(&d, 256));
    CK(hipMalloc(&o, 16));
    CK(hipMemcpy(d, offs.data(), 256, hipMemcpyHostToDevice));
    const int iters = 400;
    probe<WIDTH><<<1, 256, 65536>>>(d, o, iters);
    probe<WIDTH><<<1, 256, 65536>>>(d, o, iters);
    CK(hipDeviceSynchronize());
    unsigned long long c;
    CK(hipMemcpy(&c, o, 8, hipMemcpyDeviceToHost));
    CK(hipFree(d));
    CK(hipFree(o));
    return (double)c / (iters * 16.0 * 4.0);   // per wave-instruction, 4 waves share the LDS
}

static std::vector<int> pattern(int (*f)(int))
{
    std::vector<int> v(64);
    for (int l = 0; l < 64; ++l) v[l] = f(l) % 65536;
    return v;
}

// `./lds_bank_probe OP a0,a1,...,a63 [label]` times one caller-supplied pattern (byte offsets per
// lane); OP is b128, b64, b32 (reads), w128, w64, w32 (ds_write_b128 / _b64 / _b32) or tr64
// (ds_read_b64_tr_b16).
static int custom(int argc, char **argv)
{
    std::vector<int> v;
    for (char *tok = strtok(argv[2], ","); tok; tok = strtok(nullptr, ",")) v.push_back(atoi(tok));
    if (v.size() != 64) { printf("need 64 offsets\n"); return 1; }
    double t = !strcmp(argv[1], "b128") ? run<16>(v) : !strcmp(argv[1], "b64") ? run<8>(v)
             : !strcmp(argv[1], "w128") ? run<-16>(v) : !strcmp(argv[1], "w64") ? run<-64>(v)
             : !strcmp(argv[1], "w32") ? run<-32>(v) : !strcmp(argv[1], "tr64") ? run<-8>(v) : run<4>(v);
    printf("%s %7.2f\n", argc > 3 ? argv[3] : "custom", t);
    return 0;
}

int main(int argc, char **argv)
{
    if (argc >= 3) return custom(argc, argv);
    struct P { const char *name; int (*f)(int); };
    const P b128[] = {
        {"linear", [](int l) { return 16 * l; }},
        {"stride32", [](int l) { return 32 * l; }},
        {"halfwin", [](int l) { return 16 * (l % 8) + 256 * (l / 8); }},
        {"rows64 (one piece of 64-byte rows)", [](int l) { return 64 * (l % 32) + 16 * (l / 32); }},
        {"rows64 ^ (row>>1)&3", [](int l) { int r = l % 32; return 64 * r + 16 * ((l / 32) ^ ((r >> 1) & 3)); }},
        {"rows64 ^ ((row>>1)^(row>>3))&3", [](int l) { int r = l % 32; return 64 * r + 16 * ((l / 32) ^ (((r >> 1) ^ (r >> 3)) & 3)); }},
        {"rows128 (one piece of 128-byte rows)", [](int l) { return 128 * (l % 32) + 16 * (l / 32); }},
        {"same address (broadcast)", [](int) { return 0; }},
    };
    printf("clock ticks per wave-instruction (relative scale; compare within a width)\n");
    for (const P &p : b128) printf("b128 %-40s %7.2f\n", p.name, run<16>(pattern(p.f)));
    const P b64[] = {
        {"linear", [](int l) { return 8 * l; }},
        {"stride16", [](int l) { return 16 * l; }},
        {"halfwin (16 lanes per 128 B, next 16 at +256)", [](int l) { return 8 * (l % 16) + 256 * (l / 16); }},
        {"stride64", [](int l) { return 64 * l; }},
    };
    for (const P &p : b64) printf("b64  %-40s %7.2f\n", p.name, run<8>(pattern(p.f)));
    const P b32[] = {
        {"linear", [](int l) { return 4 * l; }},
        {"stride8", [](int l) { return 8 * l; }},
        {"halfwin (32 lanes per 128 B, next 32 at +256)", [](int l) { return 4 * (l % 32) + 256 * (l / 32); }},
        {"stride128", [](int l) { return 128 * l; }},
    };
    for (const P &p : b32) printf("b32  %-40s %7.2f\n", p.name, run<4>(pattern(p.f)));
    printf("w128 %-40s %7.2f\n", "linear", run<-16>(pattern([](int l) { return 16 * l; })));
    printf("w64  %-40s %7.2f\n", "linear", run<-64>(pattern([](int l) { return 8 * l; })));
    printf("w64  %-40s %7.2f\n", "stride16 (half of a b128 pattern)", run<-64>(pattern([](int l) { return 16 * l; })));
    printf("w32  %-40s %7.2f\n", "linear", run<-32>(pattern([](int l) { return 4 * l; })));
    return 0;
}
