// The two non-matmul operators a decode step runs between the quantised linears, so that a
// whole step is a short chain of HIP launches: RMSNorm and single-query attention over a
// preallocated KV cache.  Both are HBM/L2-bound elementwise-and-reduce kernels.
#include "gptq4_internal.h"
#include "gptq4_norm.h"

namespace {

// y[row] = weight * fp16( s[row] * rsqrt(mean(s[row]^2) + eps) ) with s = x (ADD false) or
// s = fp16(x + delta), also written to sum_out (ADD true: the residual add that precedes
// every RMSNorm of a decoder layer).  Statistics and the normalisation in fp32, rounded to
// fp16, then an fp16 multiply by the weight - the rounding order of the LLaMA RMSNorm
// module.  One workgroup per row, H % 8 == 0; sum_out may alias x.  The arithmetic lives in
// gptq4_norm.h, shared with the matmul kernels that normalise their own input.
// y_index (nullable): value f of a row is stored at y[row][y_index[f]] - the order in which an
// act-order projection reads its input, so that it needs no gather.
template <bool ADD>
__global__ __launch_bounds__(256) void gptq4_rmsnorm_kernel(const half_t *x, const half_t *delta, const half_t *__restrict__ w,
                                                            half_t *sum_out, half_t *__restrict__ y,
                                                            const int32_t *__restrict__ y_index, int H, float eps) {
    __shared__ float part[4];
    const int tid = threadIdx.x;
    const size_t row = (size_t)blockIdx.x * H;
    const uint4 *xr = reinterpret_cast<const uint4 *>(x + row);
    const uint4 *dr = reinterpret_cast<const uint4 *>(delta + (ADD ? row : 0));
    const uint4 *wr = reinterpret_cast<const uint4 *>(w);
    uint4 *sr = reinterpret_cast<uint4 *>(sum_out + (ADD ? row : 0));
    uint4 *yr = reinterpret_cast<uint4 *>(y + row);
    const int chunks = H >> 3;
    constexpr int KEEP = NORM_KEEP;  // chunks per thread held in registers (covers H <= 8192); beyond that re-read
    uint4 held[KEEP];
    float ss = 0.f;
    auto take = [&](int c) {
        const uint4 v0 = xr[c];
        const uint4 v = norm_take<ADD>(v0, ADD ? dr[c] : v0, ss);
        if (ADD) sr[c] = v;
        return v;
    };
#pragma unroll
    for (int n = 0; n < KEEP; ++n)
        if (tid + 256 * n < chunks) held[n] = take(tid + 256 * n);
    for (int c = tid + 256 * KEEP; c < chunks; c += 256) take(c);
    const float inv = norm_inv_rms(ss, part, tid, H, eps);
    uint16_t *yh = reinterpret_cast<uint16_t *>(y + row);
    auto put = [&](int c, uint4 v) {
        const uint4 o = norm_put(v, wr[c], inv);
        if (y_index == nullptr) {
            yr[c] = o;
            return;
        }
        const int4 i0 = *reinterpret_cast<const int4 *>(y_index + 8 * c);
        const int4 i1 = *reinterpret_cast<const int4 *>(y_index + 8 * c + 4);
        yh[i0.x] = (uint16_t)o.x, yh[i0.y] = (uint16_t)(o.x >> 16);
        yh[i0.z] = (uint16_t)o.y, yh[i0.w] = (uint16_t)(o.y >> 16);
        yh[i1.x] = (uint16_t)o.z, yh[i1.y] = (uint16_t)(o.z >> 16);
        yh[i1.z] = (uint16_t)o.w, yh[i1.w] = (uint16_t)(o.w >> 16);
    };
#pragma unroll
    for (int n = 0; n < KEEP; ++n)
        if (tid + 256 * n < chunks) put(tid + 256 * n, held[n]);
    // chunks past the held ones: this thread wrote sr[c] itself (ADD), or x is unchanged
    for (int c = tid + 256 * KEEP; c < chunks; c += 256) put(c, ADD ? sr[c] : xr[c]);
}

// Single-query attention, split over the valid prefix 0..positions[b] of the cache.  Workgroup (split, b*H + h) takes
// an equal share of its rows (at most `chunk`, the share at full capacity); 16 lanes share a row (8
// head dimensions each, one 16-byte load of K and of V per lane), 16 rows per pass,
// running (max, sum, weighted V) per thread in fp32; the 16 row slots are merged through
// LDS and the partial [max, sum, acc[128]] goes to the workspace.  The splits of one (b, h)
// meet through an arrival counter (agent-scope stores, completion wait, atomic count, as
// in the matmul kernels); the last one merges the partials in split order and writes
// out[b, h*128 + d] - or, with out_index, out[b, out_index[h*128 + d]]: the order in which an act-order
// o_proj reads its input, so that it needs no gather.
constexpr int ATT_PART = 130;  // floats per partial: max, sum, 128 accumulators

__global__ __launch_bounds__(256) void gptq4_attn_decode_kernel(const half_t *__restrict__ q, const half_t *__restrict__ kc,
                                                                const half_t *__restrict__ vc, const int *__restrict__ positions,
                                                                float *part, int *counters, half_t *__restrict__ out,
                                                                const int32_t *__restrict__ out_index, int H,
                                                                int capacity, int chunk, float scale) {
    __shared__ float s_m[16], s_l[16];
    __shared__ float s_acc[16][128];
    __shared__ int s_is_last;
    const int tid = threadIdx.x;
    const int slot = tid >> 4, sub = tid & 15;
    const int bh = blockIdx.y, split = blockIdx.x, nsplit = gridDim.x;
    const int b = bh / H;
    const int len = min(max(positions[b], 0), capacity - 1) + 1;
    // the valid prefix, not the capacity, is dealt to the splits (in multiples of the 16 rows of a pass): a short
    // context in a long cache still spreads over all of them
    const int mine = min(chunk, (((len + nsplit - 1) / nsplit) + 15) & ~15);
    const int r0 = split * mine, r1 = min(r0 + mine, len);

    float qf[8];
    {
        const uint4 v = *reinterpret_cast<const uint4 *>(q + (size_t)bh * 128 + 8 * sub);
        const h2_t p[4] = {as_h2(v.x), as_h2(v.y), as_h2(v.z), as_h2(v.w)};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            qf[2 * i] = (float)p[i].x * scale;
            qf[2 * i + 1] = (float)p[i].y * scale;
        }
    }
    const half_t *kb = kc + (size_t)bh * capacity * 128 + 8 * sub;
    const half_t *vb = vc + (size_t)bh * capacity * 128 + 8 * sub;
    float m = -INFINITY, l = 0.f, acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.f;

    constexpr int U = 4;  // rows in flight per thread
    for (int r = r0 + slot; r < r1; r += 16 * U) {
        uint4 kv[U], vv[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int rr = min(r + 16 * u, r1 - 1);  // clamped: the load is always valid
            kv[u] = *reinterpret_cast<const uint4 *>(kb + (size_t)rr * 128);
            vv[u] = *reinterpret_cast<const uint4 *>(vb + (size_t)rr * 128);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const h2_t kp[4] = {as_h2(kv[u].x), as_h2(kv[u].y), as_h2(kv[u].z), as_h2(kv[u].w)};
            float s = 0.f;
#pragma unroll
            for (int i = 0; i < 4; ++i) s += qf[2 * i] * (float)kp[i].x + qf[2 * i + 1] * (float)kp[i].y;
            s += __shfl_xor(s, 1);
            s += __shfl_xor(s, 2);
            s += __shfl_xor(s, 4);
            s += __shfl_xor(s, 8);
            if (r + 16 * u < r1) {  // uniform over the 16 lanes of a row
                const float mn = fmaxf(m, s);
                const float corr = __expf(m - mn), pw = __expf(s - mn);
                const h2_t vp[4] = {as_h2(vv[u].x), as_h2(vv[u].y), as_h2(vv[u].z), as_h2(vv[u].w)};
                l = l * corr + pw;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    acc[2 * i] = acc[2 * i] * corr + pw * (float)vp[i].x;
                    acc[2 * i + 1] = acc[2 * i + 1] * corr + pw * (float)vp[i].y;
                }
                m = mn;
            }
        }
    }
    if (sub == 0) {
        s_m[slot] = m;
        s_l[slot] = l;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) s_acc[slot][8 * sub + i] = acc[i];
    __syncthreads();
    float mw = -INFINITY, lw = 0.f, a = 0.f;  // threads 0..127: this workgroup's partial for dimension tid
    if (tid < 128) {
#pragma unroll
        for (int s = 0; s < 16; ++s) mw = fmaxf(mw, s_m[s]);
#pragma unroll
        for (int s = 0; s < 16; ++s) {
            const float f = (s_m[s] == -INFINITY) ? 0.f : __expf(s_m[s] - mw);
            lw += s_l[s] * f;
            a += s_acc[s][tid] * f;
        }
    }
    if (nsplit > 1) {
        float *base = part + (size_t)bh * nsplit * ATT_PART;
        if (tid < 128) {
            float *dst = base + (size_t)split * ATT_PART;
            if (tid == 0) {
                __hip_atomic_store(dst, mw, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(dst + 1, lw, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            __hip_atomic_store(dst + 2 + tid, a, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (tid == 0) {
            const int old = __hip_atomic_fetch_add(&counters[bh * COUNTER_STRIDE], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            s_is_last = (old == nsplit - 1);
        }
        __syncthreads();
        if (!s_is_last) return;
        if (tid == 0) __hip_atomic_store(&counters[bh * COUNTER_STRIDE], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        // Both halves of the workgroup merge: threads 0..127 take splits 0..7, 16..23, ..., threads 128..255 splits 8..15,
        // 24..31, ... - dimension tid % 128 each, 8 splits per round trip and thread - so the 16 partials of a one-sequence
        // step are one round trip, not two (0.3 us of 12.6; 24 more registers for a single round of 16 cost the streaming
        // loop of the batched steps 1 - 2 %).  The halves meet through LDS, the lower one first: a fixed order.
        const int half = tid >> 7, d = tid & 127;
        mw = -INFINITY, lw = 0.f, a = 0.f;
        for (int s0 = 8 * half; s0 < nsplit; s0 += 16) {
            float ms[8], ls[8], as[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) {  // all loads issued together; slots past the end re-read the last
                const float *src = base + (size_t)min(s0 + k, nsplit - 1) * ATT_PART;
                ms[k] = __hip_atomic_load(src, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                ls[k] = __hip_atomic_load(src + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                as[k] = __hip_atomic_load(src + 2 + d, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                if (s0 + k < nsplit && ms[k] != -INFINITY) {
                    const float mn = fmaxf(mw, ms[k]);
                    const float f0 = __expf(mw - mn), f1 = __expf(ms[k] - mn);
                    lw = lw * f0 + ls[k] * f1;
                    a = a * f0 + as[k] * f1;
                    mw = mn;
                }
            }
        }
        if (half == 1) {
            s_acc[0][d] = mw;
            s_acc[1][d] = lw;
            s_acc[2][d] = a;
        }
        __syncthreads();  // (the whole workgroup is here: s_is_last is uniform)
        if (half == 0) {
            const float m1 = s_acc[0][d], l1 = s_acc[1][d], a1 = s_acc[2][d];
            if (m1 != -INFINITY) {
                const float mn = fmaxf(mw, m1);
                const float f0 = __expf(mw - mn), f1 = __expf(m1 - mn);
                lw = lw * f0 + l1 * f1;
                a = a * f0 + a1 * f1;
                mw = mn;
            }
        }
    }
    if (tid < 128) {
        const int b = bh / H;
        const int col = (bh - b * H) * 128 + tid;
        out[(size_t)b * H * 128 + (out_index ? out_index[col] : col)] = (half_t)(a / lw);
    }
}

}  // namespace

int launch_rmsnorm(const half_t *x, const half_t *delta, const half_t *w, half_t *sum_out, half_t *y, const int32_t *y_index,
                   int M, int H, float eps, hipStream_t stream) {
    if (delta != nullptr)
        hipLaunchKernelGGL(gptq4_rmsnorm_kernel<true>, dim3((unsigned)M), dim3(256), 0, stream, x, delta, w, sum_out, y, y_index, H,
                           eps);
    else
        hipLaunchKernelGGL(gptq4_rmsnorm_kernel<false>, dim3((unsigned)M), dim3(256), 0, stream, x, x, w, y, y, y_index, H, eps);
    return (int)hipGetLastError();
}

// Splits per (sequence, head): as many as fill the chip's 2 x CUs places once without spilling into a second round (40
// heads: 12 splits = 480 workgroups, not 13 = 520), at least 64 rows each; with many heads still shares of about 256
// rows, so that the workgroups come in several rounds and the last one is a small part (416 heads x 2048 rows: 83 us
// with 8 splits against 88 with 2; 128 heads: 16.6 against 17.6).
int attn_decode_splits(int BH, int capacity) {
    const int want = 2 * device_shape().cus;  // 512 workgroups on MI355X
    int nsplit = want / BH;
    if (nsplit < capacity / 256) nsplit = capacity / 256;
    const int max_split = (capacity + 63) / 64;
    if (nsplit > max_split) nsplit = max_split;
    if (nsplit < 1) nsplit = 1;
    return nsplit;
}

size_t attn_decode_partial_bytes(int BH, int capacity) {
    return (size_t)BH * attn_decode_splits(BH, capacity) * ATT_PART * sizeof(float);
}

int launch_attn_decode(const half_t *q, const half_t *kc, const half_t *vc, const int *positions, half_t *out,
                       const int32_t *out_index, int B, int H, int capacity, float scale, int *counters, float *partials, hipStream_t stream) {
    const int BH = B * H;
    const int nsplit = attn_decode_splits(BH, capacity);
    int chunk = (capacity + nsplit - 1) / nsplit;
    chunk = (chunk + 15) & ~15;
    hipLaunchKernelGGL(gptq4_attn_decode_kernel, dim3((unsigned)nsplit, (unsigned)BH), dim3(256), 0, stream, q, kc, vc,
                       positions, partials, counters, out, out_index, H, capacity, chunk, scale);
    return (int)hipGetLastError();
}
