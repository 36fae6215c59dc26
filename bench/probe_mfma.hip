// Benchmark instrument, not part of the product ABI (built into its own
// librumus_probe.so): how many int8 operations per second the matrix cores of
// this device sustain when nothing else happens, i.e. v_mfma_i32_32x32x32_i8
// back to back from registers in every SIMD, no memory traffic.  With zero or
// constant operands the chip holds ~2.1-2.3 GHz; with random operand bits the
// power limit pulls the clock down, and that rate, not the datasheet figure,
// is what a GEMM on real data can approach on this board.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <vector>

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

static __device__ uint32_t mix(uint32_t x) {
    x ^= x >> 16; x *= 0x7feb352dU; x ^= x >> 15; x *= 0x846ca68bU; x ^= x >> 16;
    return x;
}

__global__ __launch_bounds__(256) void probe_i8_mfma_kernel(int* out, long long* ticks, int iters, int random_bits) {
    v4i a = {1, 1, 1, 1}, b = {1, 1, 1, 1};
    if (random_bits) {
        const uint32_t t = threadIdx.x * 977u + blockIdx.x * 131071u;
        for (int q = 0; q < 4; q++) { a[q] = (int)mix(t + q); b[q] = (int)mix(t + 17 + q); }
    }
    v16i c0 = {0}, c1 = {0}, c2 = {0}, c3 = {0};
    const long long t0 = clock64(), w0 = wall_clock64();
    for (int i = 0; i < iters; i++) {
        c0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c0, 0, 0, 0);
        c1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c1, 0, 0, 0);
        c2 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c2, 0, 0, 0);
        c3 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c3, 0, 0, 0);
    }
    const long long t1 = clock64(), w1 = wall_clock64();
    if (threadIdx.x == 0 && blockIdx.x == 0) { ticks[0] = t1 - t0; ticks[1] = w1 - w0; }
    int s = 0;
    for (int r = 0; r < 16; r++) s += c0[r] + c1[r] + c2[r] + c3[r];
    out[blockIdx.x * 256 + threadIdx.x] = s;
}

// Returns 0 on success.  tops: int8 TOP/s over the whole device (2 ops per MAC);
// mhz: shader clock during the run (clock64 ticks per 100 MHz wall tick).
extern "C" int rumus_probe_i8_mfma(int random_bits, double* tops, double* mhz) {
    hipDeviceProp_t prop;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return 1;
    const int wgs = prop.multiProcessorCount * 2;      // 8 waves per CU, 2 per SIMD
    const int iters = 20000;
    int* out = nullptr;
    long long* ticks = nullptr;
    if (hipMalloc(&out, (size_t)wgs * 256 * 4) != hipSuccess) return 1;
    if (hipMalloc(&ticks, 16) != hipSuccess) { (void)hipFree(out); return 1; }
    hipEvent_t e0, e1;
    (void)hipEventCreate(&e0);
    (void)hipEventCreate(&e1);
    float best_ms = 1e30f;
    long long h[2] = {0, 1};
    for (int rep = 0; rep < 4; rep++) {                 // the first run ramps the clock
        (void)hipEventRecord(e0, 0);
        hipLaunchKernelGGL(probe_i8_mfma_kernel, dim3(wgs), dim3(256), 0, 0, out, ticks, iters, random_bits);
        (void)hipEventRecord(e1, 0);
        if (hipEventSynchronize(e1) != hipSuccess) { best_ms = -1; break; }
        float ms = 0;
        (void)hipEventElapsedTime(&ms, e0, e1);
        if (rep > 0 && ms < best_ms) {
            best_ms = ms;
            (void)hipMemcpy(h, ticks, 16, hipMemcpyDeviceToHost);
        }
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    (void)hipFree(out);
    (void)hipFree(ticks);
    if (best_ms <= 0) return 1;
    // 4 waves per workgroup, 4 MFMAs per iteration, 32*32*32 MACs each
    const double ops = (double)wgs * 4 * iters * 4 * 2.0 * 32768.0;
    *tops = ops / (best_ms * 1e-3) / 1e12;
    *mhz = (double)h[0] / (double)h[1] * 100.0;
    return 0;
}

// The same for the f16 matrix instruction of the W4 GEMM kernels, v_mfma_f32_32x32x16_f16.  random_bits = 1: both
// operands random f16 values of magnitude 2^-3 .. 2^4 (random sign and mantissa); 2: A random like that, B small
// integers 0..15 (what a packed nibble becomes); 0: ones.
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));

__global__ __launch_bounds__(256) void probe_f16_mfma_kernel(float* out, long long* ticks, int iters, int random_bits) {
    v8h a, b;
    for (int q = 0; q < 8; q++) { a[q] = (_Float16)1.0f; b[q] = (_Float16)1.0f; }
    if (random_bits) {
        const uint32_t t = threadIdx.x * 977u + blockIdx.x * 131071u;
        for (int q = 0; q < 8; q++) {
            const uint32_t ra = mix(t + q), rb = mix(t + 29 + q);
            // sign | exponent 12..19 (2^-3 .. 2^4) | 10 mantissa bits
            const uint16_t ha = (uint16_t)(((ra >> 16) & 0x8000u) | ((12u + (ra & 7u)) << 10) | ((ra >> 3) & 0x3ffu));
            const uint16_t hb = (uint16_t)(((rb >> 16) & 0x8000u) | ((12u + (rb & 7u)) << 10) | ((rb >> 3) & 0x3ffu));
            a[q] = __builtin_bit_cast(_Float16, ha);
            b[q] = random_bits == 2 ? (_Float16)(float)(rb & 15u) : __builtin_bit_cast(_Float16, hb);
        }
    }
    v16f c0 = {0}, c1 = {0}, c2 = {0}, c3 = {0};
    const long long t0 = clock64(), w0 = wall_clock64();
    for (int i = 0; i < iters; i++) {
        c0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c0, 0, 0, 0);
        c1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c1, 0, 0, 0);
        c2 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c2, 0, 0, 0);
        c3 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c3, 0, 0, 0);
    }
    const long long t1 = clock64(), w1 = wall_clock64();
    if (threadIdx.x == 0 && blockIdx.x == 0) { ticks[0] = t1 - t0; ticks[1] = w1 - w0; }
    float s = 0;
    for (int r = 0; r < 16; r++) s += c0[r] + c1[r] + c2[r] + c3[r];
    out[blockIdx.x * 256 + threadIdx.x] = s;
}

// Returns 0 on success.  tflops: f16 TFLOP/s over the whole device (2 flop per multiply-add); mhz as above.
extern "C" int rumus_probe_f16_mfma(int random_bits, double* tflops, double* mhz) {
    hipDeviceProp_t prop;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return 1;
    const int wgs = prop.multiProcessorCount * 2;      // 8 waves per CU, 2 per SIMD
    const int iters = 20000;
    float* out = nullptr;
    long long* ticks = nullptr;
    if (hipMalloc(&out, (size_t)wgs * 256 * 4) != hipSuccess) return 1;
    if (hipMalloc(&ticks, 16) != hipSuccess) { (void)hipFree(out); return 1; }
    hipEvent_t e0, e1;
    (void)hipEventCreate(&e0);
    (void)hipEventCreate(&e1);
    float best_ms = 1e30f;
    long long h[2] = {0, 1};
    for (int rep = 0; rep < 4; rep++) {                 // the first run ramps the clock
        (void)hipEventRecord(e0, 0);
        hipLaunchKernelGGL(probe_f16_mfma_kernel, dim3(wgs), dim3(256), 0, 0, out, ticks, iters, random_bits);
        (void)hipEventRecord(e1, 0);
        if (hipEventSynchronize(e1) != hipSuccess) { best_ms = -1; break; }
        float ms = 0;
        (void)hipEventElapsedTime(&ms, e0, e1);
        if (rep > 0 && ms < best_ms) {
            best_ms = ms;
            (void)hipMemcpy(h, ticks, 16, hipMemcpyDeviceToHost);
        }
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    (void)hipFree(out);
    (void)hipFree(ticks);
    if (best_ms <= 0) return 1;
    // 4 waves per workgroup, 4 MFMAs per iteration, 32*32*16 multiply-adds each
    const double flop = (double)wgs * 4 * iters * 4 * 2.0 * 16384.0;
    *tflops = flop / (best_ms * 1e-3) / 1e12;
    *mhz = (double)h[0] / (double)h[1] * 100.0;
    return 0;
}

// ---- what one small memory-bound launch can reach -----------------------------------------
// A kernel that only reads `bytes` (64 bytes per thread, four 128-bit loads issued at once,
// one XCD-contiguous slab per workgroup) and folds them into a value it never stores, launched
// back to back from a graph over `buffers` distinct buffers so that no cache can serve it.
// bytes = 0 times an empty kernel.  This is the floor for any single launch that must read
// that many bytes (a decode GEMV reads 9.4 MB): dispatch, first-byte latency and drain included.
__global__ __launch_bounds__(512) void probe_read_kernel(const uint4* __restrict__ p, uint32_t* sink, uint32_t wgs) {
    if (!p) {
        if (threadIdx.x == 9999) sink[0] = 1;
        return;
    }
    const uint32_t b = blockIdx.x, slab = (b % 8) * (wgs / 8) + b / 8;     // one contiguous range per XCD
    const uint4* q = p + (size_t)slab * 2048 + threadIdx.x;
    const uint4 a = q[0], c = q[512], d = q[1024], e = q[1536];
    const uint32_t v = (a.x ^ c.x ^ d.x ^ e.x) | (a.y ^ c.y ^ d.y ^ e.y) | (a.z ^ c.z ^ d.z ^ e.z) | (a.w ^ c.w ^ d.w ^ e.w);
    if (v == 0x12345678u) sink[threadIdx.x] = v;
}

extern "C" int rumus_probe_read_launch(uint64_t bytes, int buffers, double* us_per_launch) {
    const uint32_t wgs = (uint32_t)(bytes / (512 * 64)) / 8 * 8;
    if (bytes && wgs == 0) return 1;
    if (buffers < 1 || buffers > 256) return 1;
    std::vector<uint4*> bufs(bytes ? buffers : 0, nullptr);
    uint32_t* sink = nullptr;
    int rc = 1;
    hipStream_t stream = nullptr;
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    do {
        if (hipMalloc(&sink, 4096) != hipSuccess) break;
        bool ok = true;
        for (auto& b : bufs) {
            if (hipMalloc(&b, (size_t)wgs * 512 * 64) != hipSuccess) { ok = false; break; }
            (void)hipMemset(b, 1, (size_t)wgs * 512 * 64);
        }
        if (!ok) break;
        if (hipStreamCreate(&stream) != hipSuccess) break;
        if (hipDeviceSynchronize() != hipSuccess) break;
        const int launches = bytes ? buffers : 64;
        if (hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal) != hipSuccess) break;
        for (int i = 0; i < launches; i++)
            hipLaunchKernelGGL(probe_read_kernel, dim3(bytes ? wgs : 256), dim3(512), 0, stream,
                               bytes ? bufs[i] : nullptr, sink, wgs);
        if (hipStreamEndCapture(stream, &graph) != hipSuccess) break;
        if (hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0) != hipSuccess) break;
        (void)hipEventCreate(&e0);
        (void)hipEventCreate(&e1);
        const int replays = 20;
        for (int w = 0; w < 3; w++) (void)hipGraphLaunch(exec, stream);
        (void)hipEventRecord(e0, stream);
        for (int r = 0; r < replays; r++) (void)hipGraphLaunch(exec, stream);
        (void)hipEventRecord(e1, stream);
        if (hipEventSynchronize(e1) != hipSuccess) break;
        float ms = 0;
        (void)hipEventElapsedTime(&ms, e0, e1);
        *us_per_launch = (double)ms * 1e3 / ((double)replays * launches);
        rc = 0;
    } while (0);
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    if (exec) (void)hipGraphExecDestroy(exec);
    if (graph) (void)hipGraphDestroy(graph);
    if (stream) (void)hipStreamDestroy(stream);
    for (auto b : bufs)
        if (b) (void)hipFree(b);
    if (sink) (void)hipFree(sink);
    return rc;
}
