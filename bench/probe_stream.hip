// Benchmark instrument, not part of the product: how fast ONE kernel launch can pull a given number of
// bytes out of HBM on this GPU, as a function of how the loads are spread over workgroups, waves and
// loads in flight per lane.  The decode-size kernels of the library read 9 to 50 MB per launch, where
// dispatch, first-byte latency and the depth of the memory pipeline decide, not the HBM peak.
//
//   probe_stream <MiB per launch> [buffers] [row bytes of the strip shape, a multiple of 256]
//
// Every variant reads the same bytes (rotating over `buffers` distinct buffers so that no cache serves
// them), 16 bytes per lane per load, and folds them into a value it never stores.  Shapes:
//   flat    : every wave reads LOADS KB once and ends (many short workgroups)
//   deep    : 256 workgroups-ish of 512 threads; a wave issues LOADS loads, then loops (ROUNDS rounds), the
//             next round's loads issued before the current round is consumed
//   strip   : as deep, but a wave instruction reads four 256-byte segments `row_bytes` apart (a column
//             strip of a row-major matrix) instead of 1 KB contiguous
//   -nt     : the same with the non-temporal hint on every load
// Times are per launch, replayed from a HIP graph of `buffers` launches.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#include <vector>

#define CHECK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_)); exit(1); } } while (0)

__device__ __forceinline__ uint32_t fold(uint4 v) { return v.x ^ v.y ^ v.z ^ v.w; }

// NT: the load carries the non-temporal hint (data used once)
typedef uint32_t u4v __attribute__((ext_vector_type(4)));
template <bool NT>
__device__ __forceinline__ uint4 ld(const uint4* p) {
    if (NT) {
        const u4v v = __builtin_nontemporal_load(reinterpret_cast<const u4v*>(p));
        return make_uint4(v.x, v.y, v.z, v.w);
    }
    return *p;
}

// flat: workgroup b reads LOADS * threads * 16 contiguous bytes
template <int LOADS, bool NT = false>
__global__ __launch_bounds__(512) void flat_kernel(const uint4* __restrict__ p, uint32_t* sink) {
    const uint4* q = p + (size_t)blockIdx.x * LOADS * blockDim.x + threadIdx.x;
    uint4 v[LOADS];
#pragma unroll
    for (int i = 0; i < LOADS; i++) v[i] = ld<NT>(q + (size_t)i * blockDim.x);
    uint32_t s = 0;
#pragma unroll
    for (int i = 0; i < LOADS; i++) s |= fold(v[i]);
    if (s == 0x12345678u) sink[threadIdx.x] = s;
}

// deep: a wave owns rounds * LOADS KB, contiguous; double-buffered rounds
template <int LOADS, bool STRIP, bool NT = false>
__global__ __launch_bounds__(512) void deep_kernel(const uint4* __restrict__ p, uint32_t* sink, uint32_t rounds,
                                                   uint32_t row_vec /* uint4 per matrix row, strip only */) {
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
    const size_t wave_id = (size_t)blockIdx.x * waves + wave;
    uint4 v[2][LOADS];
    auto issue = [&](int slot, uint32_t r) {
#pragma unroll
        for (int i = 0; i < LOADS; i++) {
            if (STRIP) {
                // workgroup = a strip of 16 uint4 (256 bytes) columns; wave = rounds * LOADS * 4 rows of it;
                // lane (c = lane % 16, b = lane / 16) reads row 4 * (r * LOADS + i) + b
                const size_t row = (size_t)wave * rounds * LOADS * 4 + (size_t)(r * LOADS + i) * 4 + (lane >> 4);
                v[slot][i] = ld<NT>(p + row * row_vec + (size_t)blockIdx.x * 16 + (lane & 15));
            } else {
                v[slot][i] = ld<NT>(p + (wave_id * rounds + r) * LOADS * 64 + (size_t)i * 64 + lane);
            }
        }
    };
    uint32_t s = 0;
    issue(0, 0);
    for (uint32_t r = 0; r < rounds; r += 2) {
        if (r + 1 < rounds) issue(1, r + 1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < LOADS; i++) s |= fold(v[0][i]);
        if (r + 2 < rounds) issue(0, r + 2);
        __builtin_amdgcn_sched_barrier(0);
        if (r + 1 < rounds) {
#pragma unroll
            for (int i = 0; i < LOADS; i++) s |= fold(v[1][i]);
        }
    }
    if (s == 0x12345678u) sink[threadIdx.x] = s;
}

struct Timer {
    hipStream_t stream;
    hipEvent_t e0, e1;
    Timer() { CHECK(hipStreamCreate(&stream)); CHECK(hipEventCreate(&e0)); CHECK(hipEventCreate(&e1)); }
    template <typename F>
    double per_launch_us(int launches, F&& launch_one) {
        hipGraph_t graph;
        hipGraphExec_t exec;
        CHECK(hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal));
        for (int i = 0; i < launches; i++) launch_one(i, stream);
        CHECK(hipStreamEndCapture(stream, &graph));
        CHECK(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0));
        for (int w = 0; w < 3; w++) CHECK(hipGraphLaunch(exec, stream));
        const int replays = 20;
        CHECK(hipEventRecord(e0, stream));
        for (int r = 0; r < replays; r++) CHECK(hipGraphLaunch(exec, stream));
        CHECK(hipEventRecord(e1, stream));
        CHECK(hipEventSynchronize(e1));
        float ms = 0;
        CHECK(hipEventElapsedTime(&ms, e0, e1));
        CHECK(hipGraphExecDestroy(exec));
        CHECK(hipGraphDestroy(graph));
        return (double)ms * 1e3 / ((double)replays * launches);
    }
};

int main(int argc, char** argv) {
    const double mib = argc > 1 ? atof(argv[1]) : 22.0;
    const int buffers = argc > 2 && atoi(argv[2]) > 0 ? atoi(argv[2]) : (int)(640.0 / mib) + 1;
    // a matrix of 1024-byte-per-wave-instruction pieces: rows of `row_bytes` for the strip shape
    const uint32_t row_bytes = argc > 3 ? (uint32_t)atoi(argv[3]) / 256 * 256 : 44032;   // 11008 packed words
    const size_t want = (size_t)(mib * 1048576.0);
    size_t rows = want / row_bytes / 64 * 64;               // whole strips of 64 rows: every shape below divides them
    if (rows == 0) rows = 64;
    const size_t bytes = rows * row_bytes;
    std::vector<uint4*> bufs(buffers);
    for (auto& b : bufs) { CHECK(hipMalloc(&b, bytes + 65536)); CHECK(hipMemset(b, 1, bytes + 65536)); }
    uint32_t* sink;
    CHECK(hipMalloc(&sink, 4096));
    CHECK(hipDeviceSynchronize());
    Timer t;
    printf("bytes per launch %zu (%.2f MiB), %d buffers\n", bytes, bytes / 1048576.0, buffers);
    auto report = [&](const char* name, uint32_t wgs, uint32_t threads, int loads, uint32_t rounds, double us) {
        printf("%-8s wgs %5u x %4u threads, %2d loads/lane/round, %3u rounds: %7.2f us  %6.0f GB/s\n", name, wgs, threads,
               loads, rounds, us, bytes / us / 1e3);
        fflush(stdout);
    };
    const double empty = t.per_launch_us(64, [&](int, hipStream_t s) {
        hipLaunchKernelGGL(flat_kernel<1>, dim3(1), dim3(64), 0, s, bufs[0], sink); });
    printf("one-wave kernel: %.2f us per launch\n", empty);

#define FLAT(L, T) do { const uint32_t wgs = (uint32_t)(bytes / ((size_t)(L) * (T) * 16)); \
        if (wgs >= 1 && (size_t)wgs * (L) * (T) * 16 == bytes) report("flat", wgs, T, L, 1, t.per_launch_us(buffers, [&](int i, hipStream_t s) { \
            hipLaunchKernelGGL(flat_kernel<L>, dim3(wgs), dim3(T), 0, s, bufs[i], sink); })); } while (0)
    FLAT(1, 256); FLAT(2, 256); FLAT(4, 256); FLAT(8, 256);
    FLAT(1, 512); FLAT(2, 512); FLAT(4, 512); FLAT(8, 512); FLAT(16, 512);
#define FLAT_NT(L, T) do { const uint32_t wgs = (uint32_t)(bytes / ((size_t)(L) * (T) * 16)); \
        if (wgs >= 1 && (size_t)wgs * (L) * (T) * 16 == bytes) report("flat-nt", wgs, T, L, 1, t.per_launch_us(buffers, [&](int i, hipStream_t s) { \
            hipLaunchKernelGGL((flat_kernel<L, true>), dim3(wgs), dim3(T), 0, s, bufs[i], sink); })); } while (0)
    FLAT_NT(1, 512); FLAT_NT(4, 512); FLAT_NT(8, 512);

#define DEEP(L, T, WGS) do { const uint32_t waves = (WGS) * ((T) / 64); \
        const uint32_t rounds = (uint32_t)(bytes / ((size_t)waves * (L) * 1024)); \
        if (rounds >= 1 && (size_t)rounds * waves * (L) * 1024 == bytes) report("deep", WGS, T, L, rounds, t.per_launch_us(buffers, [&](int i, hipStream_t s) { \
            hipLaunchKernelGGL((deep_kernel<L, false>), dim3(WGS), dim3(T), 0, s, bufs[i], sink, rounds, 0u); })); } while (0)
    DEEP(2, 512, 256); DEEP(4, 512, 256); DEEP(8, 512, 256); DEEP(16, 512, 256);
    DEEP(2, 512, 512); DEEP(4, 512, 512); DEEP(8, 512, 512);
    DEEP(2, 512, 1024); DEEP(4, 512, 1024);
    DEEP(4, 256, 512); DEEP(4, 256, 1024);

    // strips: row_bytes / 256 workgroups, each a 256-byte column strip over all rows
#define STRIPS(L, T) do { const uint32_t wgs = row_bytes / 256, waves = (T) / 64; \
        const uint32_t rounds = (uint32_t)(rows / ((size_t)waves * (L) * 4)); \
        if (rounds >= 1 && (size_t)rounds * waves * (L) * 4 == rows) report("strip", wgs, T, L, rounds, t.per_launch_us(buffers, [&](int i, hipStream_t s) { \
            hipLaunchKernelGGL((deep_kernel<L, true>), dim3(wgs), dim3(T), 0, s, bufs[i], sink, rounds, row_bytes / 16); })); } while (0)
    STRIPS(1, 256); STRIPS(2, 256); STRIPS(1, 512); STRIPS(2, 512); STRIPS(4, 512); STRIPS(8, 512);
#define STRIPS_NT(L, T) do { const uint32_t wgs = row_bytes / 256, waves = (T) / 64; \
        const uint32_t rounds = (uint32_t)(rows / ((size_t)waves * (L) * 4)); \
        if (rounds >= 1 && (size_t)rounds * waves * (L) * 4 == rows) report("strip-nt", wgs, T, L, rounds, t.per_launch_us(buffers, [&](int i, hipStream_t s) { \
            hipLaunchKernelGGL((deep_kernel<L, true, true>), dim3(wgs), dim3(T), 0, s, bufs[i], sink, rounds, row_bytes / 16); })); } while (0)
    STRIPS_NT(4, 512); STRIPS_NT(8, 512);
    return 0;
}
