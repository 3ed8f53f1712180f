// Residual add + RMSNorm of one row by 256 threads, in pieces shared by the stand-alone kernel
// and by the matmul kernels that normalise their own input (NORM variants): the same thread owns
// the same 8-value chunks (tid, tid + 256, ...), adds its squares in the same order and the four
// wave sums meet in the same order, so both paths produce the same bits.
//   s = x (+ delta, one fp16 add);  inv = rsqrt(mean(s^2) + eps) in fp32;
//   y = weight * fp16(s * inv)      (the rounding order of the LLaMA RMSNorm module).
#pragma once

#include "gptq4_common.h"

__device__ __forceinline__ float norm_wave_sum(float v) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) v += __shfl_xor(v, o);
    return v;
}

// one chunk: s = x (+ d); the squares of its 8 values are added to ss
template <bool ADD>
__device__ __forceinline__ uint4 norm_take(uint4 v, uint4 d, float &ss) {
    if (ADD) {
        v.x = as_u32(as_h2(v.x) + as_h2(d.x));
        v.y = as_u32(as_h2(v.y) + as_h2(d.y));
        v.z = as_u32(as_h2(v.z) + as_h2(d.z));
        v.w = as_u32(as_h2(v.w) + as_h2(d.w));
    }
    const h2_t p[4] = {as_h2(v.x), as_h2(v.y), as_h2(v.z), as_h2(v.w)};
#pragma unroll
    for (int i = 0; i < 4; ++i) ss += (float)p[i].x * (float)p[i].x + (float)p[i].y * (float)p[i].y;
    return v;
}

// 1/rms of the row from the per-thread sums of squares; part4 = 4 floats of LDS.  Contains a
// workgroup barrier: every thread of the workgroup calls it; `active` marks the 256 that hold sums.
__device__ __forceinline__ float norm_inv_rms(float ss, float *part4, int tid, int H, float eps, bool active = true) {
    ss = norm_wave_sum(ss);
    if (active && (tid & 63) == 0) part4[tid >> 6] = ss;
    __syncthreads();
    return rsqrtf((part4[0] + part4[1] + part4[2] + part4[3]) / (float)H + eps);
}

// one chunk of the result: weight * fp16(s * inv)
__device__ __forceinline__ uint4 norm_put(uint4 v, uint4 g, float inv) {
    const uint32_t vi[4] = {v.x, v.y, v.z, v.w}, gi[4] = {g.x, g.y, g.z, g.w};
    uint32_t o[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const h2_t p = as_h2(vi[i]);
        const h2_t nrm = {(half_t)((float)p.x * inv), (half_t)((float)p.y * inv)};
        o[i] = as_u32(as_h2(gi[i]) * nrm);
    }
    return make_uint4(o[0], o[1], o[2], o[3]);
}

constexpr int NORM_KEEP = 4;      // chunks per thread held in registers: covers rows of up to 8192 values
constexpr int NORM_MAX_H = 8192;  // longest row a matmul kernel normalises itself
constexpr int NORM_MAX_M = 4;     // most rows

// The loads of row 0, issued early (before the kernel's first weight loads, so that the row
// can be normalised while those are still in flight): KEEP chunks of x, delta and the weight
// per thread, H <= 2048 * KEEP.
template <int KEEP>
struct NormLoads {
    uint4 x[KEEP], d[KEEP], g[KEEP];
};

template <bool ADD, int KEEP>
__device__ __forceinline__ void norm_issue_row0(const half_t *x, const half_t *delta, const half_t *w, int H, int tid,
                                                NormLoads<KEEP> &r) {
    const int chunks = H >> 3;
#pragma unroll
    for (int n = 0; n < KEEP; ++n) {
        const int c = min(tid + 256 * n, chunks - 1);  // clamped: always a valid load, unused past the row
        r.x[n] = reinterpret_cast<const uint4 *>(x)[c];
        r.d[n] = ADD ? reinterpret_cast<const uint4 *>(delta)[c] : r.x[n];
        r.g[n] = reinterpret_cast<const uint4 *>(w)[c];
    }
}

// Rows 0..M-1 of weight * rmsnorm(x (+ delta)) into xs[row * (H/8) + chunk] (LDS, natural k order);
// row 0 from the registers norm_issue_row0 filled, further rows loaded here.  If sum_out is not
// null the sums x + delta are written there as well (one workgroup of the launch does that).
// 256 threads, part = NORM_MAX_M * 4 floats of LDS.  Ends with a barrier.  In a workgroup of more than 256
// threads all of them call it (the barriers are the workgroup's) and `active` is true for threads 0..255 only.
// (`put(row, chunk, value)` places a normalised chunk: natural order into an LDS array for most callers, straight into
// the k order of the decoded weights for the kernel that keeps its activations that way)
template <bool ADD, int KEEP, typename Put>
__device__ __forceinline__ void norm_rows_put(const half_t *x, const half_t *delta, const half_t *w, half_t *sum_out, Put put,
                                              float *part, int M, int H, float eps, int tid, const NormLoads<KEEP> &r0,
                                              bool active = true) {
    const int chunks = H >> 3;
    for (int row = 0; row < M; ++row) {
        const uint4 *xr = reinterpret_cast<const uint4 *>(x + (size_t)row * H);
        const uint4 *dr = reinterpret_cast<const uint4 *>(ADD ? delta + (size_t)row * H : x);
        uint4 held[KEEP];
        float ss = 0.f;
#pragma unroll
        for (int n = 0; n < KEEP; ++n) {
            const int c = tid + 256 * n;
            if (active && c < chunks) {
                const uint4 v = (row == 0) ? r0.x[n] : xr[c];
                const uint4 d = (row == 0) ? r0.d[n] : (ADD ? dr[c] : v);
                held[n] = norm_take<ADD>(v, d, ss);
                if (ADD && sum_out != nullptr) reinterpret_cast<uint4 *>(sum_out + (size_t)row * H)[c] = held[n];
            }
        }
        const float inv = norm_inv_rms(ss, part + 4 * row, tid, H, eps, active);
#pragma unroll
        for (int n = 0; n < KEEP; ++n) {
            const int c = tid + 256 * n;
            if (active && c < chunks) put(row, c, norm_put(held[n], r0.g[n], inv));
        }
    }
    __syncthreads();
}

template <bool ADD, int KEEP>
__device__ __forceinline__ void norm_rows_to_lds(const half_t *x, const half_t *delta, const half_t *w, half_t *sum_out,
                                                 uint4 *xs, float *part, int M, int H, float eps, int tid,
                                                 const NormLoads<KEEP> &r0, bool active = true) {
    const int chunks = H >> 3;
    norm_rows_put<ADD, KEEP>(x, delta, w, sum_out, [&](int row, int c, uint4 v) { xs[row * chunks + c] = v; }, part, M, H, eps, tid, r0,
                             active);
}
