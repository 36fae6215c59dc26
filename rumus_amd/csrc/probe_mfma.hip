// Benchmark instrument, not part of the product ABI (built into its own
// librumus_probe.so): how many int8 operations per second the matrix cores of
// this device sustain when nothing else happens, i.e. v_mfma_i32_32x32x32_i8
// back to back from registers in every SIMD, no memory traffic.  With zero or
// constant operands the chip holds ~2.1-2.3 GHz; with random operand bits the
// power limit pulls the clock down, and that rate, not the datasheet figure,
// is what a GEMM on real data can approach on this board.
#include <hip/hip_runtime.h>
#include <stdint.h>

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
