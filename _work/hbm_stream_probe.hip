// What a plain streaming kernel reaches on this GPU: the yardstick the softmax and the SDD
// kernel are held against.  Copies 50 MB to 50 MB (the softmax's bytes at seq 4096 x 16 heads)
// with 16-byte accesses, over six rotating buffer pairs so that the 256 MB last-level cache
// cannot serve it, and prints microseconds per launch for
//   - the cache-policy bits of loads and stores (none, nt, sc0, sc1 and their unions),
//   - the number of loads a lane keeps in flight (1 to 16) and one-shot against persistent grids,
//   - reading alone and writing alone.
// Launches are timed inside HIP graphs of 60, best of 4 replays.
//
//   hipcc --offload-arch=gfx950 -O3 -std=c++17 -Xclang -target-feature -Xclang -packed-fp32-ops \
//         hbm_stream_probe.hip -o hbm_stream_probe && ./hbm_stream_probe
#include <hip/hip_runtime.h>
#include <cstdio>
#include <vector>

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
#define CK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); return 1; } } while (0)

#define LOAD_ASM(POL) asm volatile("global_load_dwordx4 %0, %1, off " POL : "=v"(v[k]) : "v"(in + i) : "memory")
#define STORE_ASM(POL) asm volatile("global_store_dwordx4 %0, %1, off " POL :: "v"(out + i), "v"(v[k]) : "memory")

// K loads, one wait, K stores per lane; the element count is a multiple of 256 * K, so no bounds
template <int LP, int SP>
__global__ __launch_bounds__(256) void copy_policy(const u32x4 *__restrict__ in, u32x4 *__restrict__ out)
{
    constexpr int K = 4;
    const size_t base = (size_t)blockIdx.x * (256 * K) + threadIdx.x;
    u32x4 v[K];
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const size_t i = base + (size_t)k * 256;
        if (LP == 0) LOAD_ASM("");
        if (LP == 1) LOAD_ASM("nt");
        if (LP == 2) LOAD_ASM("sc0");
        if (LP == 3) LOAD_ASM("sc1");
        if (LP == 4) LOAD_ASM("sc0 sc1");
        if (LP == 5) LOAD_ASM("sc0 sc1 nt");
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
    for (int k = 0; k < K; ++k) {
        const size_t i = base + (size_t)k * 256;
        if (SP == 0) STORE_ASM("");
        if (SP == 1) STORE_ASM("nt");
        if (SP == 2) STORE_ASM("sc0");
        if (SP == 3) STORE_ASM("sc1");
        if (SP == 4) STORE_ASM("sc0 sc1");
        if (SP == 5) STORE_ASM("sc0 sc1 nt");
    }
}

// MODE 0 copy, 1 read only, 2 write only; non-temporal; a grid-stride loop when the grid is smaller than the work
template <int K, int MODE>
__global__ __launch_bounds__(256) void stream_nt(const u32x4 *__restrict__ in, u32x4 *__restrict__ out, size_t n)
{
    const size_t step = (size_t)gridDim.x * 256 * K;
    u32x4 acc = {0, 0, 0, 0};
    for (size_t base = (size_t)blockIdx.x * (256 * K) + threadIdx.x; base < n; base += step) {
        u32x4 v[K];
#pragma unroll
        for (int k = 0; k < K; ++k)
            v[k] = MODE == 2 ? u32x4{1u, 2u, 3u, (unsigned)k} : __builtin_nontemporal_load(in + base + (size_t)k * 256);
#pragma unroll
        for (int k = 0; k < K; ++k) {
            if (MODE == 1) acc ^= v[k];
            else __builtin_nontemporal_store(v[k], out + base + (size_t)k * 256);
        }
    }
    if (MODE == 1 && acc.x == 0x12345678u && acc.y == 0x9abcdef0u) out[0] = acc;   // keeps the loads alive
}

int main()
{
    const size_t bytes = 16ull * 1536 * 1024 * 2;      // 50.3 MB, a multiple of every 256 * K * 16 used below
    const size_t n = bytes / 16;
    const int SETS = 6, REP = 60;
    std::vector<u32x4 *> a(SETS), b(SETS);
    for (int s = 0; s < SETS; ++s) {
        CK(hipMalloc(&a[s], bytes)); CK(hipMalloc(&b[s], bytes));
        CK(hipMemset(a[s], 1, bytes)); CK(hipMemset(b[s], 2, bytes));
    }
    hipStream_t st; CK(hipStreamCreate(&st));
    hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
    auto timeit = [&](auto launch, float &out_us) -> int {
        for (int i = 0; i < 12; ++i) launch(i % SETS);
        CK(hipStreamSynchronize(st));
        hipGraph_t g; hipGraphExec_t ge;
        CK(hipStreamBeginCapture(st, hipStreamCaptureModeGlobal));
        for (int i = 0; i < REP; ++i) launch(i % SETS);
        CK(hipStreamEndCapture(st, &g)); CK(hipGraphInstantiate(&ge, g, nullptr, nullptr, 0));
        CK(hipGraphLaunch(ge, st)); CK(hipStreamSynchronize(st));
        float best = 1e9f;
        for (int r = 0; r < 4; ++r) {
            CK(hipEventRecord(e0, st)); CK(hipGraphLaunch(ge, st)); CK(hipEventRecord(e1, st)); CK(hipStreamSynchronize(st));
            float ms; CK(hipEventElapsedTime(&ms, e0, e1)); if (ms < best) best = ms;
        }
        out_us = best * 1000.0f / REP;
        CK(hipGraphExecDestroy(ge)); CK(hipGraphDestroy(g));
        return 0;
    };

    static const char *NAMES[6] = {"-", "nt", "sc0", "sc1", "sc0 sc1", "sc0 sc1 nt"};
    float res[6][6];
    const int grid4 = (int)(n / (256 * 4));
#define RUN(LP, SP) if (timeit([&](int s) { hipLaunchKernelGGL((copy_policy<LP, SP>), dim3(grid4), dim3(256), 0, st, a[s], b[s]); }, res[LP][SP])) return 1;
#define ROW(LP) RUN(LP, 0) RUN(LP, 1) RUN(LP, 2) RUN(LP, 3) RUN(LP, 4) RUN(LP, 5)
    ROW(0) ROW(1) ROW(2) ROW(3) ROW(4) ROW(5)
    printf("copy %.1f MB -> %.1f MB, us per launch (x2 bytes / us = TB/s); rows = load policy, columns = store policy\n%-12s",
           bytes / 1e6, bytes / 1e6, "");
    for (int s = 0; s < 6; ++s) printf("%11s", NAMES[s]);
    printf("\n");
    for (int l = 0; l < 6; ++l) {
        printf("%-12s", NAMES[l]);
        for (int s = 0; s < 6; ++s) printf("%11.2f", res[l][s]);
        printf("\n");
    }

    printf("\nnon-temporal, by loads in flight per lane (K) and grid\n");
    float us;
#define SHAPE(K, MODE, GRID, LABEL) { const int g_ = (GRID) ? (GRID) : (int)(n / (256 * K)); \
        if (timeit([&](int s) { hipLaunchKernelGGL((stream_nt<K, MODE>), dim3(g_), dim3(256), 0, st, a[s], b[s], n); }, us)) return 1; \
        printf("%-10s K=%-2d grid=%-6d %7.2f us  %5.2f TB/s\n", LABEL, K, g_, us, (MODE == 0 ? 2.0 : 1.0) * bytes / 1e6 / us); }
    SHAPE(1, 0, 0, "copy") SHAPE(2, 0, 0, "copy") SHAPE(4, 0, 0, "copy") SHAPE(8, 0, 0, "copy") SHAPE(16, 0, 0, "copy")
    SHAPE(4, 0, 2048, "persistent") SHAPE(8, 0, 1024, "persistent") SHAPE(8, 0, 512, "persistent")
    SHAPE(4, 1, 0, "read") SHAPE(8, 1, 0, "read") SHAPE(4, 2, 0, "write") SHAPE(8, 2, 0, "write")
    if (timeit([&](int s) { hipLaunchKernelGGL((stream_nt<1, 2>), dim3(1), dim3(256), 0, st, a[s], b[s], (size_t)256); }, us)) return 1;
    printf("one workgroup writing 4 KB (the floor of a launch inside a graph): %.2f us\n", us);
    return 0;
}
