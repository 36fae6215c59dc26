// INT4 dequant-matmul for small batches (a few to about a hundred rows) on the int8 matrix cores.
//
//   y[m,n] = sum_g scale[g,n] * ( sum_{k in g} x[m,k] q[k,n]  -  zp[g,n] * sum_{k in g} x[m,k] )
//
// Inside a group only x and the raw nibbles meet, and a nibble is already an int8 operand: a packed
// word becomes two operand registers with three instructions (w & 0x0f0f0f0f, (w >> 4) & 0x0f0f0f0f),
// where the f16 path spends nine per word.  The f32 activations cannot enter an integer MFMA, so a
// small kernel first writes them as fixed point: X = rint(x * 2^e) with |X| < 2^22 relative to the
// largest magnitude of the row's eighth of K (the part one wave of the matmul multiplies), split into
// three signed digits X = d0 + 256 d1 + 65536 d2 (|d0|, |d1| <= 128, |d2| <= 64), one int8 plane each,
// stored in the order the MFMA's A operand wants, plus the sum of X over every chunk of 64 or 128 k; a
// gather through `perm` (act-order) happens there too.  Every product and every sum over a chunk is then
// an exact integer (v_mfma_i32_16x16x64_i8, three per weight fragment); the two low tiles are put
// together with a shift-add (below 2^26), the high one joins them in f32 (its weight, 2^16 times up to
// 64 * 15 * 128, does not fit 32 bits) -- one rounding of 2^-24 of the chunk's sum -- and one
// multiply-add applies the group's scale.  The zero-point term is a small matrix product of its own, chunk sums of X times
// -scale * zero-point, on v_mfma_f32_16x16x4_f32 once per round of chunks.
//
// A workgroup owns 16*Q columns over all of K for one block of 16*RT rows; its eight waves take an
// eighth of K each and meet in LDS at the end, so nothing crosses workgroups: no partial sums in
// memory, no atomics, the same bits on every run.  Lane (c = lane % 16, b = lane / 16) reads Q
// adjacent columns of packed word rows 8*step + 2b and + 2b+1 with one load each (the 16 lanes of a
// k block read 64*Q contiguous bytes); word j of those loads is the B operand of MFMA j, whose 16
// columns are therefore n0 + Q*c + j: the output tile comes out with the Q columns of a lane side
// by side.  Weights go global -> registers -> MFMA, a wave's whole share in flight when it is four
// chunks or fewer; the activation planes come out of the L2 (every workgroup reads all of them, 3 bytes
// per element).
#include <algorithm>

#include "w4.h"

namespace rumus {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef uint32_t u3a4 __attribute__((ext_vector_type(3), aligned(4)));

constexpr int kI8WK = 8;                   // waves of a workgroup = shares of K
constexpr uint32_t kI8AlwaysRows = 128;    // batches up to here always come here ...
constexpr uint32_t kI8MaxRows = 1024;      // ... up to here where an estimate says this kernel is the faster one (weights of at
                                           // least 2048 x 4096); beyond, the larger tiles of the f16 kernel win ...
constexpr uint32_t kI8FilledRows = 512;    // ... and for smaller weights up to here where the rounds of workgroups are well filled
constexpr int kI8Outliers = 16;            // elements per (row, share of K) that may leave the fixed point

struct W4I8Args {
    const uint32_t* packed;
    const float* scales;
    const float* zp;
    const uint32_t* zp4;
    const float* bias;
    const uint8_t* planes;    // [row tile][step][digit][64 lanes x 16 bytes]
    const float* rscale;      // [row tile][share][16 rows]: 2^-e (NaN: that part of the row holds a NaN or an infinity)
    const int32_t* csum;      // [row tile][chunk][16 rows]: sum of the chunk's X
    const uint8_t* out_n;     // [row tile][share][16 rows]: elements of that part of the row that are multiplied on their own
    const int32_t* out_k;     // [row][share][kI8Outliers]: their positions (rows of the packed matrix) ...
    const float* out_x;       // ... and values
    float* y;
    uint32_t m, n, steps, chunks, steps_per_group, per;   // per: chunks per share
};


// low bytes of a, b, c, d -> one word
__device__ __forceinline__ uint32_t pack4(int a, int b, int c, int d) {
    const uint32_t lo = __builtin_amdgcn_perm((uint32_t)b, (uint32_t)a, 0x0c0c0400u);
    const uint32_t hi = __builtin_amdgcn_perm((uint32_t)d, (uint32_t)c, 0x0c0c0400u);
    return __builtin_amdgcn_perm(hi, lo, 0x05040100u);
}

// ---- lane exchanges without a trip through the LDS crossbar (integers: any order of the operands) --------
// value of the lane's partner under the DPP pattern `ctrl`
template <int CTRL>
__device__ __forceinline__ int dpp_move(int v) { return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, true); }
constexpr int kDppQuadXor1 = 0xB1, kDppQuadXor2 = 0x4E;        // quad_perm [1,0,3,2], [2,3,0,1]
constexpr int kDppHalfMirror = 0x141, kDppRowMirror = 0x140;   // lane i <-> 7 - i of its 8, 15 - i of its 16

// sum over aligned groups of LANES = 8 or 16 lanes, in every lane of the group
template <uint32_t LANES>
__device__ __forceinline__ int group_sum(int v) {
    static_assert(LANES == 8 || LANES == 16, "half a row or a row of lanes");
    v += dpp_move<kDppQuadXor1>(v);
    v += dpp_move<kDppQuadXor2>(v);
    v += dpp_move<kDppHalfMirror>(v);          // the other quad of the 8
    if (LANES == 16) v += dpp_move<kDppRowMirror>(v);   // the other 8 of the row
    return v;
}

// ---- activations -> digit planes ------------------------------------------------------------------
// One wave per (row, share of K); a lane takes 8 consecutive k at a time: half of a lane's operand bytes of
// one step (its even elements fill one word - a packed word's even nibbles -, its odd elements the next).
// f = 2^e; 1.5 * 2^23 + x * f has rint(x * f) in its low mantissa bits (round to nearest even by the addition
// itself).  Rows past m are written as zeros: the matmul reads whole row tiles.  The first four groups of a
// lane (shares up to 2048 k) stay in registers between the pass that finds the maximum and the pass that
// writes the digits.
// STAGED (act-order, x[row][perm[j]]): the eight waves of a row are one workgroup that first copies the row
// into LDS (k floats of dynamic LDS) with contiguous reads and gathers from there; gathered from global
// memory a wave instruction touches 64 cache lines for 256 bytes, behind the load of perm itself.
template <int CS, bool VEC, bool STAGED>
__global__ __launch_bounds__(STAGED ? 64 * kI8WK : 64) void w4_i8_prepare_kernel(
    const float* __restrict__ x, const int32_t* __restrict__ perm, uint8_t* __restrict__ planes,
    float* __restrict__ rscale, int32_t* __restrict__ csum, uint8_t* __restrict__ out_n, int32_t* __restrict__ out_k,
    float* __restrict__ out_x, uint32_t m, uint32_t k, uint32_t steps, uint32_t chunks, uint32_t per) {
    static_assert(!(VEC && STAGED), "staging is for the gather");
    extern __shared__ __attribute__((aligned(16))) float lds_row[];
    constexpr int CACHE = 4;
    constexpr uint32_t SUBS = 8 * CS;                               // lanes per chunk
    const uint32_t lane = threadIdx.x & 63, share = STAGED ? threadIdx.x >> 6 : blockIdx.x;
    const uint32_t row = STAGED ? blockIdx.x : blockIdx.y, rt = row >> 4, row_l = row & 15;
    const uint32_t k_begin = min(share * per, chunks) * CS * 64, k_end = min((share + 1) * per, chunks) * CS * 64;
    const bool live = row < m;
    const float* xr = x + (uint64_t)(live ? row : 0) * k;
    // STAGED (the launcher sends k % 8 == 0 and 16-byte aligned x and perm here): where a lane's 8 values come
    // from, then the values themselves.  Straight-line code with clamped addresses: a load under a branch
    // would make the wave wait for it at the end of the branch, one trip to memory after the other.
    auto index8 = [&](uint32_t k0, int4 (&ix)[2]) {
        const bool in = live && k0 < k_end && k0 < k;              // whole groups of 8 are in or out
        const int4* src = reinterpret_cast<const int4*>(perm + (in ? k0 : 0));
        ix[0] = src[0];
        ix[1] = src[1];
        return in;
    };
    auto gather8 = [&](const int4 (&ix)[2], bool in, float (&v)[8]) {
        const uint32_t j[8] = {(uint32_t)ix[0].x, (uint32_t)ix[0].y, (uint32_t)ix[0].z, (uint32_t)ix[0].w,
                               (uint32_t)ix[1].x, (uint32_t)ix[1].y, (uint32_t)ix[1].z, (uint32_t)ix[1].w};
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const float f = lds_row[j[e]];
            v[e] = in ? f : 0.0f;
        }
    };
    // the indices of the groups kept in registers are fetched while the row is on its way into LDS
    int4 cix[STAGED ? CACHE : 1][2];
    bool cin[STAGED ? CACHE : 1];
    if (STAGED) {
#pragma unroll
        for (int i = 0; i < CACHE; i++) cin[i] = index8(k_begin + (lane + 64 * i) * 8, cix[i]);
        constexpr uint32_t T = 64 * kI8WK;
        const uint32_t vecs = k / 4;
        const float4* src = reinterpret_cast<const float4*>(xr);
        for (uint32_t i0 = threadIdx.x; i0 < vecs; i0 += 4 * T) {      // four loads in flight: one trip up to 8192 k
            float4 t[4];
#pragma unroll
            for (int u = 0; u < 4; u++) t[u] = src[min(i0 + u * T, vecs - 1)];
            __builtin_amdgcn_sched_barrier(0);                     // all issued before the first is waited for
#pragma unroll
            for (int u = 0; u < 4; u++)
                if (i0 + u * T < vecs) reinterpret_cast<float4*>(lds_row)[i0 + u * T] = t[u];
        }
        __syncthreads();
    }

    auto load8 = [&](uint32_t k0, float (&v)[8]) {
#pragma unroll
        for (int j4 = 0; j4 < 2; j4++) {
            const uint32_t kk = k0 + 4 * j4;
            if (VEC) {                                             // k % 4 == 0: a float4 is all in or all out
                float4 f = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                if (live && k0 < k_end && kk < k) f = *reinterpret_cast<const float4*>(xr + kk);
                v[4 * j4] = f.x; v[4 * j4 + 1] = f.y; v[4 * j4 + 2] = f.z; v[4 * j4 + 3] = f.w;
            } else if (STAGED) {
                if (j4 == 0) {
                    int4 ix[2];
                    const bool in = index8(k0, ix);
                    gather8(ix, in, v);
                }
            } else {
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const bool in = live && k0 < k_end && kk + j < k;
                    const uint32_t src = in ? (perm ? (uint32_t)perm[kk + j] : kk + j) : 0;
                    const float f = xr[src];
                    v[4 * j4 + j] = in ? f : 0.0f;
                }
            }
        }
    };
    auto max_bits = [](const float (&v)[8]) {
        uint32_t mb = 0;
#pragma unroll
        for (int j = 0; j < 8; j++) mb = max(mb, __float_as_uint(v[j]) & 0x7fffffffu);
        return mb;
    };

    // pass 1: the largest magnitude, on the bit patterns: a NaN or an infinity sorts highest
    float cache[CACHE][8];
    uint32_t mb = 0;
#pragma unroll
    for (int i = 0; i < CACHE; i++) {
        if (STAGED) gather8(cix[i], cin[i], cache[i]);
        else load8(k_begin + (lane + 64 * i) * 8, cache[i]);
        mb = max(mb, max_bits(cache[i]));
    }
    for (uint32_t k0 = k_begin + (lane + 64 * CACHE) * 8; k0 < k_end; k0 += 512) {
        float v[8];
        load8(k0, v);
        mb = max(mb, max_bits(v));
    }
    const uint32_t lane_top = mb;                                  // this lane's largest
    mb = wave_max(mb);
    // Elements that tower over the rest of their part would set the fixed point for all of it and cost the others
    // their low bits (22 bits below the LARGEST magnitude).  When only a few elements lie within 2^-8 of the largest
    // - few enough for the slots left - they leave the fixed point: position and value go to the matmul, which
    // multiplies them in f32 on their own, x * ((q - zp) * scale) as the reference's loop does with every element,
    // and the part is scaled by what remains (looked at once more: towers of two heights).  Ordinary data has
    // hundreds of elements that close to the largest and passes with one count.  Only where the whole part sits
    // in registers (shares up to 2048 k).
    uint32_t n_out = 0;
    if (k_end - k_begin <= 64 * 8 * CACHE) {
        // first a test that ordinary data fails at once: does any lane hold nothing within 2^-8 of the largest?  (If
        // every lane does, 64 elements are that close: more than the slots.)
        const uint32_t lowest_top = ~wave_max(~lane_top);
        if (lowest_top + (8u << 23) < mb && mb < 0x7f800000u) {
            for (int level = 0; level < 2; level++) {
                if (mb == 0 || mb >= 0x7f800000u) break;               // nothing there, or a NaN / an infinity: poisoned below
                const uint32_t near_top = mb > (8u << 23) ? mb - (8u << 23) : 1u;   // the largest / 256, on the bit patterns
                int near = 0;
#pragma unroll
                for (int i = 0; i < CACHE; i++)
#pragma unroll
                    for (int j = 0; j < 8; j++) near += (__float_as_uint(cache[i][j]) & 0x7fffffffu) >= near_top ? 1 : 0;
                int left = wave_sum(near);
                if ((uint32_t)left > (uint32_t)kI8Outliers - n_out) break;
                // one element at a time: the first lane that still has one hands over its first
                while (left > 0) {
                    int at = -1;
#pragma unroll
                    for (int i = CACHE - 1; i >= 0; i--)
#pragma unroll
                        for (int j = 7; j >= 0; j--)
                            if ((__float_as_uint(cache[i][j]) & 0x7fffffffu) >= near_top) at = i * 8 + j;
                    const uint32_t owner = (uint32_t)__builtin_ctzll(__ballot(at >= 0));
                    if (lane == owner) {
                        float v = 0.0f;
#pragma unroll
                        for (int i = 0; i < CACHE; i++)
#pragma unroll
                            for (int j = 0; j < 8; j++)
                                if (at == i * 8 + j) { v = cache[i][j]; cache[i][j] = 0.0f; }
                        const uint64_t slot = ((uint64_t)row * kI8WK + share) * kI8Outliers + n_out;
                        out_k[slot] = (int32_t)(k_begin + (lane + 64 * (at >> 3)) * 8 + (at & 7));
                        out_x[slot] = v;
                    }
                    n_out++;
                    left--;
                }
                mb = 0;
#pragma unroll
                for (int i = 0; i < CACHE; i++) mb = max(mb, max_bits(cache[i]));
                mb = wave_max(mb);
            }
        }
    }
    if (lane == 0) out_n[((uint64_t)rt * kI8WK + share) * 16 + row_l] = (uint8_t)n_out;
    // 2^e with max * 2^e in [2^21, 2^22); e stops at 126, where 2^-e is the smallest normal number, so parts whose
    // largest magnitude lies below 2^-107 keep fewer than 20 bits.  A
    // non-finite activation poisons its row: the scale becomes NaN (the digits are then whatever the
    // conversion gives; they only ever meet the NaN)
    const bool finite = mb < 0x7f800000u;
    int e = 21 - ((int)(mb >> 23) - 127);
    e = mb == 0 ? 0 : min(e, 126);
    const float f = finite ? __uint_as_float((uint32_t)(e + 127) << 23) : 0.0f;
    if (lane == 0)
        rscale[((uint64_t)rt * kI8WK + share) * 16 + row_l] =
            finite ? __uint_as_float((uint32_t)(127 - e) << 23) : __uint_as_float(0x7fc00000u);

    // pass 2: digits and chunk sums
    auto emit = [&](uint32_t k0, const float (&v)[8]) {
        int d[3][8], sum = 0;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int X = (int)__float_as_uint(fmaf(v[j], f, 12582912.0f)) - 0x4b400000;   // |X| < 2^22
            const int X1 = (X + 128) >> 8;
            d[0][j] = __builtin_amdgcn_sbfe(X, 0, 8);              // X - 256 * X1
            d[1][j] = __builtin_amdgcn_sbfe(X1, 0, 8);             // X1 - 256 * d2
            d[2][j] = (X1 + 128) >> 8;                             // |d2| <= 64
            sum += X;
        }
        sum = group_sum<SUBS>(sum);                                  // whole chunks are in or out together
        const uint32_t piece = k0 >> 4, step = piece >> 2, b = piece & 3, half = (k0 >> 3) & 1;
#pragma unroll
        for (int p = 0; p < 3; p++)
            *reinterpret_cast<uint2*>(planes + (((uint64_t)rt * steps + step) * 3 + p) * 1024 + (b * 16 + row_l) * 16 + half * 8) =
                make_uint2(pack4(d[p][0], d[p][2], d[p][4], d[p][6]), pack4(d[p][1], d[p][3], d[p][5], d[p][7]));
        if ((k0 >> 3) % SUBS == 0) csum[((uint64_t)rt * chunks + (k0 >> 3) / SUBS) * 16 + row_l] = sum;
    };
#pragma unroll
    for (int i = 0; i < CACHE; i++) {
        const uint32_t k0 = k_begin + (lane + 64 * i) * 8;
        if (k0 < k_end) emit(k0, cache[i]);
    }
    for (uint32_t k0 = k_begin + (lane + 64 * CACHE) * 8; k0 < k_end; k0 += 512) {
        float v[8];
        load8(k0, v);
        emit(k0, v);
    }
}

// ---- the matmul -------------------------------------------------------------------------------------
template <int Q>
__device__ __forceinline__ void load_q(const uint32_t* p, uint32_t (&o)[Q]) {
    if constexpr (Q == 4) {
        const uint4 v = *reinterpret_cast<const uint4*>(p);
        o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
    } else if constexpr (Q == 3) {
        const u3a4 v = *reinterpret_cast<const u3a4*>(p);
        o[0] = v.x; o[1] = v.y; o[2] = v.z;
    } else if constexpr (Q == 2) {
        const uint2 v = *reinterpret_cast<const uint2*>(p);
        o[0] = v.x; o[1] = v.y;
    } else {
        o[0] = *p;
    }
}

// Q: columns per lane (16*Q per workgroup).  RT: row tiles of 16 per workgroup.  CS: steps of 64 k per
// chunk (1 or 2).  U: chunks per round = chunks of weight loads in flight per lane.
template <int Q, int RT, int CS, int U, bool ZP4>
__global__ __launch_bounds__(512) void w4_gemm_i8_kernel(W4I8Args a) {
    constexpr int WK = kI8WK;
    static_assert((U * RT) % 2 == 0, "the two activation slots alternate with a fixed phase per unrolled position");
    static_assert(U <= 4, "a round's chunks are the four k slots of the zero-point MFMA");
    constexpr int RP = RT % 2 == 0 ? 2 : 1;                        // row tiles per round of the final sum over the shares
    static_assert(RT % RP == 0, "whole rounds");
    __shared__ float red[WK][RP * Q * 4][64];
    const uint32_t lane = threadIdx.x & 63, wk = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t c = lane & 15, b = lane >> 4;
    const uint32_t n0 = xcd_contiguous(blockIdx.x, gridDim.x) * (16 * Q), rb = blockIdx.y;
    // past the edge: the last Q columns again (computed twice, stored twice with the same values)
    const uint32_t colc = min(n0 + Q * c, a.n - Q);
    const uint32_t f0 = min(wk * a.per, a.chunks), f1 = min(f0 + a.per, a.chunks);
    const uint32_t flast = f1 > f0 ? f1 - 1 : f0 ? f0 - 1 : 0;
    const uint32_t lane_w = 2 * b * a.n + colc;                    // lane part of a packed-word address

    uint32_t braw[U][CS][2][Q], msc[U][Q], mzp[U][Q];
    auto fetch_b = [&](int slot, uint32_t chunk) {
        const uint32_t fc = min(chunk, flast);                       // past the wave's share: fetched again, adds 0
#pragma unroll
        for (int s = 0; s < CS; s++)
#pragma unroll
            for (int h = 0; h < 2; h++)
                load_q<Q>(a.packed + (uint64_t)((fc * CS + s) * 8 + h) * a.n + lane_w, braw[slot][s][h]);
        const uint32_t g = fc * CS / a.steps_per_group;
        load_q<Q>(reinterpret_cast<const uint32_t*>(a.scales) + (uint64_t)g * a.n + colc, msc[slot]);
        if (ZP4) mzp[slot][0] = a.zp4[(uint64_t)g * (a.n / 8) + colc / 8];
        else load_q<Q>(reinterpret_cast<const uint32_t*>(a.zp) + (uint64_t)g * a.n + colc, mzp[slot]);
    };
    // A lane of a row past m reads the last real row's fragment instead of its own zeros (the same address as
    // that row's lane: no extra traffic); what it computes is never stored.  With 8 of a tile's 16 rows real the
    // planes cost half the bytes out of L2.
    uint32_t a_lane[RT];
#pragma unroll
    for (int t = 0; t < RT; t++) {
        const uint32_t first = (rb * RT + t) * 16, real = a.m > first ? min(a.m - first, 16u) : 1u;
        a_lane[t] = (b * 16 + min(c, real - 1)) * 16;
    }
    v4i afr[2][CS][3];
    auto fetch_a = [&](int slot, uint32_t chunk, uint32_t rt) {
        const uint32_t fc = min(chunk, flast), rtg = rb * RT + rt;
#pragma unroll
        for (int s = 0; s < CS; s++)
#pragma unroll
            for (int p = 0; p < 3; p++)
                afr[slot][s][p] = *reinterpret_cast<const v4i*>(
                    a.planes + (((uint64_t)rtg * a.steps + fc * CS + s) * 3 + p) * 1024 + a_lane[rt]);
    };

    v4f accf[RT][Q];
#pragma unroll
    for (int t = 0; t < RT; t++)
#pragma unroll
        for (int q = 0; q < Q; q++) accf[t][q] = v4f{0.0f, 0.0f, 0.0f, 0.0f};

    // whether any element of this share of the rows of each tile left the fixed point (see the end of the kernel):
    // sixteen byte counts at a wave-uniform address, a scalar load asked for now and looked at when the loop is done
    uint4 out_bytes[RT];
#pragma unroll
    for (int t = 0; t < RT; t++)
        out_bytes[t] = *reinterpret_cast<const uint4*>(a.out_n + ((uint64_t)(rb * RT + t) * WK + wk) * 16);

    // Loads retire in order, so what is issued last is waited for last: activation fragments (needed
    // first, they come out of the L2) always go ahead of the weight loads that are needed later.
    fetch_a(0, f0, 0);
#pragma unroll
    for (int u = 0; u < U; u++) fetch_b(u, f0 + u);

    // Whole rounds of U chunks, straight-line code: a chunk past the wave's share is computed on the last
    // chunk's data again (addresses are clamped) with its scale and zero-point set to 0, so it adds 0.
    for (uint32_t base = f0; base < f1; base += U) {
        // chunk sums of the round for the zero-point product: lane (row c, k slot b) holds chunk base + b
        float sm[RT];
#pragma unroll
        for (int t = 0; t < RT; t++)
            sm[t] = (float)a.csum[((uint64_t)(rb * RT + t) * a.chunks + min(base + b, flast)) * 16 + c];
        float szq[Q];
#pragma unroll
        for (int q = 0; q < Q; q++) szq[q] = 0.0f;
#pragma unroll
        for (int u = 0; u < U; u++) {
            const uint32_t chunk = base + u;
            const bool alive = chunk < f1;                             // wave-uniform
            v4i bf[CS][Q];
#pragma unroll
            for (int s = 0; s < CS; s++)
#pragma unroll
                for (int q = 0; q < Q; q++) {
                    const uint32_t w0 = braw[u][s][0][q], w1 = braw[u][s][1][q];
                    bf[s][q] = v4i{(int)(w0 & 0x0f0f0f0fu), (int)((w0 >> 4) & 0x0f0f0f0fu),
                                   (int)(w1 & 0x0f0f0f0fu), (int)((w1 >> 4) & 0x0f0f0f0fu)};
                }
            float sc[Q];
#pragma unroll
            for (int q = 0; q < Q; q++) {
                sc[q] = alive ? __uint_as_float(msc[u][q]) : 0.0f;
                const float zq = ZP4 ? (float)((mzp[u][0] >> (4 * ((colc & 7u) + q))) & 15u) : __uint_as_float(mzp[u][q]);
                // this chunk is k slot u of the round's zero-point product: -(scale * zp), 0 for a dead chunk
                szq[q] = (alive && b == (uint32_t)u) ? -(sc[q] * zq) : szq[q];
            }
#pragma unroll
            for (int t = 0; t < RT; t++) {
                const int cur = (u * RT + t) & 1;
                if (t + 1 < RT) {
                    fetch_a(cur ^ 1, chunk, t + 1);
                } else {
                    fetch_a(cur ^ 1, chunk + 1, 0);
                    fetch_b(u, chunk + U);                             // this slot's words are in bf by now
                }
                // the prefetches stay here: the scheduler would sink them to their first use to save registers
                __builtin_amdgcn_sched_barrier(0);
                v4i acc[Q][3];
#pragma unroll
                for (int q = 0; q < Q; q++)
#pragma unroll
                    for (int p = 0; p < 3; p++) acc[q][p] = v4i{0, 0, 0, 0};
#pragma unroll
                for (int s = 0; s < CS; s++)
#pragma unroll
                    for (int q = 0; q < Q; q++)
#pragma unroll
                        for (int p = 0; p < 3; p++)
                            acc[q][p] = __builtin_amdgcn_mfma_i32_16x16x64_i8(afr[cur][s][p], bf[s][q], acc[q][p], 0, 0, 0);
#pragma unroll
                for (int q = 0; q < Q; q++)
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        // |low| <= 128 * 15 * 128 * 257 < 2^26 is exact; the high digits' tile times 2^16 passes 2^31,
                        // so it joins in f32: exact by itself, one rounding in the sum
                        const int low = (acc[q][1][i] << 8) + acc[q][0][i];
                        const float tot = fmaf((float)acc[q][2][i], 65536.0f, (float)low);
                        accf[t][q][i] = fmaf(sc[q], tot, accf[t][q][i]);
                    }
            }
        }
        // - scale * zp * (sum of X over the chunk), the round's chunks at once: [16 rows x 4 chunks] x [4 chunks x 16 columns]
#pragma unroll
        for (int t = 0; t < RT; t++)
#pragma unroll
            for (int q = 0; q < Q; q++) accf[t][q] = __builtin_amdgcn_mfma_f32_16x16x4f32(sm[t], szq[q], accf[t][q], 0, 0, 0);
    }

    // Elements that left the fixed point (w4_i8_prepare_kernel): x * ((q - zp) * scale) in f32, the reference's own
    // expression, added in the accumulators' units (x / rscale: a power of two, exact).  Lane (c, b) holds rows
    // 4b .. 4b + 3 and columns colc .. colc + Q - 1 of a tile.
#pragma unroll
    for (int t = 0; t < RT; t++) {
        // (the words stay opaque until the loop's results exist: looked at earlier, the wait for them would stand at
        // the top of the kernel)
        uint32_t any = out_bytes[t].x | out_bytes[t].y | out_bytes[t].z | out_bytes[t].w;
        asm volatile("" : "+s"(any) : "v"(accf[t][0][0]));
        if (any == 0) continue;                                        // wave-uniform; ordinary data ends here
        const uint32_t row0 = (rb * RT + t) * 16;
        const int cnt = a.out_n[((uint64_t)(rb * RT + t) * WK + wk) * 16 + c];
        uint32_t rows_with = (uint32_t)(__ballot(cnt > 0) & 0xFFFFu);
        while (rows_with) {
            const uint32_t r = (uint32_t)__builtin_ctz(rows_with);
            rows_with &= rows_with - 1;
            const uint32_t n_r = (uint32_t)__builtin_amdgcn_readlane(cnt, r);
            const float unit = 1.0f / a.rscale[((uint64_t)(rb * RT + t) * WK + wk) * 16 + r];
            for (uint32_t o = 0; o < n_r; o++) {
                const uint64_t slot = ((uint64_t)(row0 + r) * WK + wk) * kI8Outliers + o;
                const uint32_t ko = (uint32_t)a.out_k[slot];
                const float xo = a.out_x[slot] * unit;
                const uint32_t g = (ko / 64) / a.steps_per_group;
                uint32_t wq[Q], sq[Q], zq[Q];
                load_q<Q>(a.packed + (uint64_t)(ko / 8) * a.n + colc, wq);
                load_q<Q>(reinterpret_cast<const uint32_t*>(a.scales) + (uint64_t)g * a.n + colc, sq);
                if (ZP4) zq[0] = a.zp4[(uint64_t)g * (a.n / 8) + colc / 8];
                else load_q<Q>(reinterpret_cast<const uint32_t*>(a.zp) + (uint64_t)g * a.n + colc, zq);
#pragma unroll
                for (int q = 0; q < Q; q++) {
                    const float nib = (float)((wq[q] >> (4 * (ko & 7u))) & 15u);
                    const float z = ZP4 ? (float)((zq[0] >> (4 * ((colc & 7u) + q))) & 15u) : __uint_as_float(zq[q]);
                    const float w = (nib - z) * __uint_as_float(sq[q]);
#pragma unroll
                    for (int i = 0; i < 4; i++)
                        accf[t][q][i] = (b == r / 4 && (uint32_t)i == r % 4) ? fmaf(xo, w, accf[t][q][i]) : accf[t][q][i];
                }
            }
        }
    }

    // back to the activations' scale (this wave's share of K has its own), then the eight shares meet in LDS, two
    // row tiles per round; wave w adds them up, in a fixed order, for rows 4b + w % 4 of the round's row tile w / 4
    // and stores
#pragma unroll
    for (int t0 = 0; t0 < RT; t0 += RP) {
        if (t0) __syncthreads();                               // the round before has been read
#pragma unroll
        for (int tt = 0; tt < RP; tt++) {
            const int t = t0 + tt;
            const float4 rs = *reinterpret_cast<const float4*>(a.rscale + ((uint64_t)(rb * RT + t) * WK + wk) * 16 + 4 * b);
            const float r4[4] = {rs.x, rs.y, rs.z, rs.w};
#pragma unroll
            for (int q = 0; q < Q; q++)
#pragma unroll
                for (int i = 0; i < 4; i++) red[wk][(tt * Q + q) * 4 + i][lane] = f1 > f0 ? accf[t][q][i] * r4[i] : 0.0f;
        }
        __syncthreads();
        const uint32_t tt = wk >> 2, i = wk & 3;
        const uint32_t row = (rb * RT + t0 + tt) * 16 + 4 * b + i;
        if (wk < RP * 4 && row < a.m) {
            float* dst = a.y + (uint64_t)row * a.n + colc;
            float o[Q];
#pragma unroll
            for (int q = 0; q < Q; q++) {
                float v = red[0][(tt * Q + q) * 4 + i][lane];
#pragma unroll
                for (int w = 1; w < WK; w++) v += red[w][(tt * Q + q) * 4 + i][lane];
                if (a.bias) v += a.bias[colc + q];
                o[q] = v;
            }
            if constexpr (Q == 4) *reinterpret_cast<float4*>(dst) = make_float4(o[0], o[1], o[2], o[3]);
            else if constexpr (Q == 2) *reinterpret_cast<float2*>(dst) = make_float2(o[0], o[1]);
            else {
#pragma unroll
                for (int q = 0; q < Q; q++) dst[q] = o[q];
            }
        }
    }
}

static int pick_q(uint32_t n, uint32_t row_blocks, bool zp4);

// 129 to 512 rows on weights outside the range of the estimates below: the workgroups (a block of 64 rows by 16 Q columns each) run one per compute unit, in rounds of 256
// that last the same full or not.  Where the rounds are at least three quarters full, with three or four columns per
// lane, this kernel beats the f16 tiles (4096 -> 11008: 129 rows 55.8 -> 47.8 us, 256 rows 75.4 -> 60.1, 384 rows 118 -> 98,
// 512 rows 120 -> 118; 4096 -> 4096 at 512 rows 56.2 -> 45.6; 8192 -> 8192 at 384 rows 132 -> 107); where the column count
// only fills the rounds with two columns per lane it loses (11008 -> 4096 at 384 rows 91 -> 101 us, 8192 -> 8192 at 160
// rows 68 -> 72) and the f16 tiles keep the batch.
static bool i8_rounds_filled(uint32_t m, uint32_t n, bool zp4) {
    const uint32_t row_blocks = ceil_div(m, 64);
    const uint32_t q = (uint32_t)pick_q(n, row_blocks, zp4);
    const uint64_t wgs = (uint64_t)ceil_div(n, 16 * q) * row_blocks;
    const uint64_t rounds = (wgs + 255) / 256;
    return q >= 3 && wgs * 4 >= rounds * 256 * 3;
}

// 129 to 1024 rows, n >= 4096 and k >= 2048: both kernels run in rounds of workgroups over the 256 CUs, and which one
// is faster depends on how the shape fills them.  Two estimates in microseconds, fitted to both kernels forced over ten
// weight shapes (2048 x 8192 to 8192 x 28672) at nine batches each (within 8 % rms of this kernel's times and 6 % of the
// f16 tiles'); the faster estimate takes the batch.  Measured against the better of the two on those 90 cases the
// choice costs 1 % on average and 12 % at worst (the rules it replaced: 2 % and 30 %).
//   here: W workgroups / 256 rounds of 3.4 + 3.9 Q each (Q columns per lane), less what the first round overlaps;
//   f16 tiles: from 192 tiles of 64 x 512 on, rounds as w4_launch_gemm prices its two shapes, 109 per round; below,
//       K is split over the workgroups and the time follows the tile count.
// Both scale with K; 16 and 24 are what a call costs besides (activation planes, launches).
static bool i8_beats_f16_estimate(uint32_t m, uint32_t k, uint32_t n, bool zp4) {
    const uint32_t row_blocks = ceil_div(m, 64);
    const uint32_t q = (uint32_t)pick_q(n, row_blocks, zp4);
    const double kf = (double)k / 4096.0;
    const double wgs = (double)ceil_div(n, 16 * q) * row_blocks;
    const double est_i8 = (wgs / 256.0 - 0.14) * (3.4 + 3.9 * q) * kf + 16.0;
    const uint64_t tiles = (uint64_t)row_blocks * ceil_div(n, 512), full = (tiles + 255) / 256;
    const uint64_t halves = ((uint64_t)row_blocks * ceil_div(n, 256) + 255) / 256;
    double est_f16;
    if (tiles >= 192) {
        double units = 0.97 * (double)full;
        units = std::min(units, (double)(halves / 2) * 1.05 + (double)(halves % 2) * 0.75);
        est_f16 = units * 109.0 * kf + 24.0;
    } else {
        est_f16 = (156.0 * (double)tiles / 256.0 - 3.0) * kf + 24.0;
    }
    return est_i8 < 0.97 * est_f16;                           // ties go to the f16 tiles (slightly fewer wrong choices on the fitted cases)
}

bool w4_gemm_i8_supported(const W4Args& a) {
    const uintptr_t bits = reinterpret_cast<uintptr_t>(a.packed) | reinterpret_cast<uintptr_t>(a.scales) |
                           reinterpret_cast<uintptr_t>(a.zp) | reinterpret_cast<uintptr_t>(a.y) |
                           (a.bias ? reinterpret_cast<uintptr_t>(a.bias) : 0);
    if (!(a.m > 0 && a.m <= kI8MaxRows && a.group_size % 64 == 0 && a.n % 4 == 0 && a.n >= 4 && (bits & 15) == 0 &&
          !a.g_idx && !a.tiled && !a.glu && (!a.zp4 || a.n % 8 == 0)))
        return false;
    if (a.m <= kI8AlwaysRows) return true;
    if (a.n >= 4096 && a.k >= 2048) return i8_beats_f16_estimate(a.m, a.k, a.n, a.zp4 != nullptr);
    return a.m <= kI8FilledRows && i8_rounds_filled(a.m, a.n, a.zp4 != nullptr);
}

template <int Q, int RT, int CS, int U>
static int launch_i8(const W4I8Args& k, bool zp4, uint32_t row_blocks, hipStream_t s) {
    const dim3 grid(ceil_div(k.n, 16 * Q), row_blocks);
    if (zp4) hipLaunchKernelGGL((w4_gemm_i8_kernel<Q, RT, CS, U, true>), grid, dim3(512), 0, s, k);
    else hipLaunchKernelGGL((w4_gemm_i8_kernel<Q, RT, CS, U, false>), grid, dim3(512), 0, s, k);
    return check_launch("w4_gemm_i8_kernel");
}

// Columns per lane.  Workgroups run one per compute unit, in rounds of 256, and a workgroup's time grows
// with its columns on top of a fixed part (its share of the activation planes): the cheapest
// rounds * (Q + 1.5) wins.  u4 zero-points come eight to a word: Q = 3 would straddle words.
static int pick_q(uint32_t n, uint32_t row_blocks, bool zp4) {
    int best = 4;
    double best_cost = 1e30;
    for (int q = 4; q >= 1; q--) {
        if (q == 3 && zp4) continue;
        const uint64_t wgs = (uint64_t)ceil_div(n, 16 * q) * row_blocks;
        const double cost = (double)((wgs + 255) / 256) * (q + 1.5);
        if (cost < best_cost) { best_cost = cost; best = q; }
    }
    return best;
}

template <int RT, int CS, int U>
static int launch_i8_q(const W4I8Args& k, bool zp4, uint32_t row_blocks, hipStream_t s) {
    switch (pick_q(k.n, row_blocks, zp4)) {
        case 4: return launch_i8<4, RT, CS, U>(k, zp4, row_blocks, s);
        case 3: return launch_i8<3, RT, CS, U>(k, zp4, row_blocks, s);
        case 2: return launch_i8<2, RT, CS, U>(k, zp4, row_blocks, s);
        default: return launch_i8<1, RT, CS, U>(k, zp4, row_blocks, s);
    }
}

int w4_launch_gemm_i8(const W4Args& a, hipStream_t s) {
    const uint32_t cs = a.group_size % 128 == 0 ? 2 : 1;             // chunk = 128 or 64 k: never across a group end
    const uint32_t steps = a.padded_k / 64, chunks = steps / cs, per = ceil_div(chunks, (uint32_t)kI8WK);
    // Rows per workgroup.  The weights are streamed once per block of rows, so the blocks are as tall as the registers
    // allow (four row tiles: 64 rows 26.7 -> 22.8 us, 128 rows 40.8 -> 36.8 us against blocks of 32) but not taller than
    // the rows that exist: 33 to 48 rows take one block of 48 (40 rows 21.7 -> 19.8 us against a block of 64 with an
    // empty tile), 65 to 96 rows two blocks of 48 (80 rows 34.2 -> 31.7 us against three blocks of 32).  Eight row tiles
    // per workgroup spill registers and run one long round (128 rows 43.8 us).
    const uint32_t rt_per = a.m <= 16 ? 1 : a.m <= 32 ? 2 : a.m <= 48 || (a.m > 64 && a.m <= 96) ? 3 : 4;
    const uint32_t row_blocks = ceil_div(a.m, 16 * rt_per), rts = row_blocks * rt_per;
    RUMUS_REQUIRE(row_blocks <= 65535, "qmatmul_int4: m %u is beyond the grid limit", a.m);
    auto up = [](size_t v) { return (v + 255) & ~size_t(255); };
    const size_t planes_bytes = (size_t)rts * steps * 3 * 1024;
    const size_t csum_bytes = up((size_t)rts * chunks * 16 * sizeof(int32_t)), rscale_bytes = up((size_t)rts * kI8WK * 16 * sizeof(float));
    const size_t outn_bytes = up((size_t)rts * 16 * kI8WK), outk_bytes = up((size_t)rts * 16 * kI8WK * kI8Outliers * sizeof(int32_t));
    void* ws = nullptr;
    WorkspaceLease lease;                                            // until both kernels are queued
    if (int rc = workspace_get(s, planes_bytes + csum_bytes + rscale_bytes + outn_bytes + 2 * outk_bytes, &ws, lease)) return rc;
    uint8_t* planes = static_cast<uint8_t*>(ws);
    int32_t* csum = reinterpret_cast<int32_t*>(planes + planes_bytes);
    float* rscale = reinterpret_cast<float*>(planes + planes_bytes + csum_bytes);
    uint8_t* out_n = planes + planes_bytes + csum_bytes + rscale_bytes;
    int32_t* out_k = reinterpret_cast<int32_t*>(planes + planes_bytes + csum_bytes + rscale_bytes + outn_bytes);
    float* out_x = reinterpret_cast<float*>(planes + planes_bytes + csum_bytes + rscale_bytes + outn_bytes + outk_bytes);
    const bool vec = !a.perm && a.k % 4 == 0 && (reinterpret_cast<uintptr_t>(a.x) & 15) == 0;
    const bool staged = a.perm && (size_t)a.k * sizeof(float) <= 64 * 1024 && a.k % 8 == 0 &&
                        ((reinterpret_cast<uintptr_t>(a.x) | reinterpret_cast<uintptr_t>(a.perm)) & 15) == 0;
    const dim3 pgrid(kI8WK, rts * 16);
    const size_t row_bytes = (size_t)a.k * sizeof(float);
#define RUMUS_I8_PREPARE(CS)                                                                                           \
    do {                                                                                                               \
        if (staged)                                                                                                    \
            hipLaunchKernelGGL((w4_i8_prepare_kernel<CS, false, true>), dim3(rts * 16), dim3(64 * kI8WK), row_bytes, s, \
                               a.x, a.perm, planes, rscale, csum, out_n, out_k, out_x, a.m, a.k, steps, chunks, per); \
        else if (vec)                                                                                                  \
            hipLaunchKernelGGL((w4_i8_prepare_kernel<CS, true, false>), pgrid, dim3(64), 0, s, a.x, a.perm, planes,    \
                               rscale, csum, out_n, out_k, out_x, a.m, a.k, steps, chunks, per);                      \
        else                                                                                                           \
            hipLaunchKernelGGL((w4_i8_prepare_kernel<CS, false, false>), pgrid, dim3(64), 0, s, a.x, a.perm, planes,   \
                               rscale, csum, out_n, out_k, out_x, a.m, a.k, steps, chunks, per);                      \
    } while (0)
    if (cs == 2) RUMUS_I8_PREPARE(2);
    else RUMUS_I8_PREPARE(1);
#undef RUMUS_I8_PREPARE
    if (int rc = check_launch("w4_i8_prepare_kernel")) return rc;
    const W4I8Args k{a.packed, a.scales, a.zp, a.zp4, a.bias, planes, rscale, csum, out_n, out_k, out_x, a.y,
                     a.m, a.n, steps, chunks, a.group_size / 64, per};
    const bool zp4 = a.zp4 != nullptr;
    // a wave's whole share in flight when it is up to four chunks (two for two row tiles: registers)
    if (rt_per == 1) return cs == 2 ? launch_i8_q<1, 2, 4>(k, zp4, row_blocks, s) : launch_i8_q<1, 1, 4>(k, zp4, row_blocks, s);
    if (rt_per == 2) return cs == 2 ? launch_i8_q<2, 2, 2>(k, zp4, row_blocks, s) : launch_i8_q<2, 1, 2>(k, zp4, row_blocks, s);
    if (rt_per == 3) return cs == 2 ? launch_i8_q<3, 2, 2>(k, zp4, row_blocks, s) : launch_i8_q<3, 1, 2>(k, zp4, row_blocks, s);
    return cs == 2 ? launch_i8_q<4, 2, 2>(k, zp4, row_blocks, s) : launch_i8_q<4, 1, 2>(k, zp4, row_blocks, s);
}

}  // namespace rumus
