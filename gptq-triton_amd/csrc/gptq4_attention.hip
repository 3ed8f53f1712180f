// Causal attention over a prompt for gfx950 (head dimension 128): the pass between the fused QKV + rotary projection,
// whose q and KV-cache rows it reads where they lie, and o_proj, whose input [B, S, H * 128] it writes directly.
// (The reference hands this step to torch's scaled_dot_product_attention and transposes the result,
// fused_attention.py:117-141; with a 2048-token prompt it is a sixth of the prompt pass.)
//
// One workgroup of four waves per 128 queries of one head, a wave per 32 queries; the keys come in blocks of 64
// through LDS, shared by the four waves.  Both products run on v_mfma_f32_32x32x16_f16 in their TRANSPOSED form, so
// that what one produces is what the next consumes without leaving the lane:
//   S^T = K Q^T   A = 32 keys x 16 dims out of LDS (rows 256 bytes apart, 16-byte chunks XOR-swizzled by the key),
//                 B = the wave's queries, in registers for the whole kernel; lane (h, q) then holds, for its query
//                 column q, the scores of keys 8 * i + 4 * h + j of each half block (register 4 * i + j);
//   O^T = V^T P^T A = 32 dims x 16 keys, B = 16 keys x 32 queries: the lane's own probabilities, registers 8 * u .. 8 * u + 7
//                 of a half block for step u.  That fixes which key sits in which of the 16 contraction slots of a
//                 step - slot 8 * h + t is key 4 * h + t (t < 4) or 8 + 4 * h + t - 4 - and V^T is written to LDS with
//                 its keys in that order (the two middle groups of four swapped), rows of 64 keys = 128 bytes apart,
//                 chunks swizzled by the dimension.
// The softmax runs per lane on its own query column (one exchange per block with the other half-wave for the running
// maximum; the row sums meet once, at the end), in base 2 with the scale folded in.  Blocks beyond a wave's last
// visible key are skipped by that wave; heavy and light query blocks are paired up by workgroup id (see the kernel).
#include "../../include/gptq4.h"
#include "gptq4_internal.h"

namespace {

typedef float f16x_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

// (fmaxf makes the compiler quiet possible signalling NaNs first, one more instruction per operand; the scores are
// matrix-core outputs or -inf)
__device__ __forceinline__ float max3(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

__device__ __forceinline__ int key_slot(int key) {  // position of a key of a 64-key block in V^T's row
    const int o = key & 15;
    return (key & ~15) | (o < 4 ? o : o < 8 ? o + 4 : o < 12 ? o - 4 : o);
}

__global__ __launch_bounds__(256, 2) void gptq4_attn_prefill_kernel(const half_t *__restrict__ q, const half_t *__restrict__ kc,
                                                                    const half_t *__restrict__ vc, half_t *__restrict__ out, int H,
                                                                    int S, int capacity, int past, float scale_log2e, int nq, int nbh) {
    // (the LDS serves a 16-byte read of 16 lanes at a time from 64 banks: the 16 chunks must fall into different 16-byte slots of 256)
    __shared__ uint4 k_s[2 * 64 * 16];  // two buffers of [key][16 chunks of 8 dims], chunk c of key k at c ^ (k & 15)
    __shared__ uint4 v_s[2 * 128 * 8];  // two buffers of [dim][8 chunks of 8 key slots], chunk c of dim d at c ^ ((d >> 1) & 7)
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int h = lane >> 5, c32 = lane & 31;
    // Workgroup id -> (head, query block).  A query block's work grows with its index, and the grid's first half lands
    // one workgroup per CU, the second half beside them: ids i and i + T/2 take blocks nq - 1 - j and j of the same head, so
    // that the two a CU holds together add up to the same work everywhere (and share the head's keys in L2).
    int qb, bh;
    {
        const int id = blockIdx.x, half = (nq + 1) >> 1, first = nbh * half;
        if (id < first) {
            bh = id / half;
            qb = nq - 1 - (id - bh * half);
        } else {
            const int k = id - first, low = nq - half;
            bh = k / low;
            qb = k - bh * low;
        }
    }
    const int q0 = qb * 128 + wave * 32;  // first query of the wave
    const int kv_len = past + S;

    // ---- the wave's queries: B operand of S^T, lane (h, q): dims 16 * ks + 8 * h .. + 7
    h8_t qf[8];
    {
        const int row = min(q0 + c32, S - 1);
        const uint4 *qp = reinterpret_cast<const uint4 *>(q + ((size_t)bh * S + row) * 128);
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) qf[ks] = __builtin_bit_cast(h8_t, qp[2 * ks + h]);
    }
    f16x_t o[4];
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[db][i] = 0.f;
    float m = -INFINITY, l = 0.f;

    const int kmax = min(kv_len, past + (qb + 1) * 128);  // keys any query of the workgroup sees
    const int nblk = (kmax + 63) >> 6;
    const int my_last = past + min(q0 + 31, S - 1);      // last key the wave's last query sees
    const int my_first = past + q0;                      // last key its first query sees
    const half_t *kb = kc + (size_t)bh * capacity * 128;
    const half_t *vb = vc + (size_t)bh * capacity * 128;

    // ---- staging, two LDS buffers: while block i is multiplied, block i + 1 goes from registers into the other buffer
    //      and block i + 2 is on its way from memory; one barrier per block.
    //      K chunk id = tid + 256 * n -> (key id / 16, chunk id % 16): whole rows per 16 lanes.
    //      V: thread (pair p = tid % 32, dc = tid / 32 + 8 * n) holds chunk dc of keys 2p and 2p + 1 - neighbours in V^T's
    //      slot order too - and writes, per dimension, one dword {key 2p, key 2p + 1}: half a wave fills 128 bytes of a row.
    u32x4_t kr[4], vr[2][2];
#define FETCH_BLOCK(blk)                                                                                             \
    _Pragma("unroll") for (int n = 0; n < 4; ++n) {                                                                  \
        const int id = tid + 256 * n;                                                                                \
        const int key = min((blk) * 64 + (id >> 4), kv_len - 1);                                                     \
        kr[n] = *reinterpret_cast<const u32x4_t *>(kb + (size_t)key * 128 + 8 * (id & 15));                          \
    }                                                                                                                \
    _Pragma("unroll") for (int n = 0; n < 2; ++n) _Pragma("unroll") for (int kk = 0; kk < 2; ++kk) {                 \
        const int vkey = min((blk) * 64 + 2 * (tid & 31) + kk, kv_len - 1);                                          \
        vr[n][kk] = *reinterpret_cast<const u32x4_t *>(vb + (size_t)vkey * 128 + 8 * ((tid >> 5) + 8 * n));          \
    }
    const int vslot = key_slot(2 * (tid & 31));  // even: the pair's dword
    auto stage = [&](int buf) {
        uint4 *const kd = k_s + buf * (64 * 16);
        uint32_t *const vd = reinterpret_cast<uint32_t *>(v_s + buf * (128 * 8));
#pragma unroll
        for (int n = 0; n < 4; ++n) {
            const int id = tid + 256 * n;
            const int key = id >> 4, c = id & 15;
            kd[key * 16 + (c ^ (key & 15))] = __builtin_bit_cast(uint4, kr[n]);
        }
#pragma unroll
        for (int n = 0; n < 2; ++n) {
            const int dc = (tid >> 5) + 8 * n;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int d = 8 * dc + e;
                const uint32_t lo = vr[n][0][e >> 1], hi = vr[n][1][e >> 1];
                // halves e of the two keys: bytes (0, 1) or (2, 3) of each word
                const uint32_t w = (e & 1) ? __builtin_amdgcn_perm(hi, lo, 0x07060302u) : __builtin_amdgcn_perm(hi, lo, 0x05040100u);
                vd[d * 32 + ((((vslot >> 3) ^ ((d >> 1) & 7)) << 3) + (vslot & 7)) / 2] = w;
            }
        }
    };
    FETCH_BLOCK(0)
    stage(0);
    if (nblk > 1) {
        FETCH_BLOCK(1)
    }
    for (int blk = 0; blk < nblk; ++blk) {
        const int buf = blk & 1;
        __syncthreads();  // block blk is in its buffer; the other buffer (block blk - 1) has been read by every wave
        if (blk + 1 < nblk) {
            stage(buf ^ 1);
            if (blk + 2 < nblk) {
                FETCH_BLOCK(blk + 2)
            }
        }
        const uint4 *const kt = k_s + buf * (64 * 16);
        const uint4 *const vt = v_s + buf * (128 * 8);
        const int key0 = blk * 64;
        if (key0 > my_last) continue;  // nothing in this block is visible to the wave (it still takes part in the staging)

        // ---- S^T = K Q^T for the two half blocks of 32 keys
        f16x_t s[2];
#pragma unroll
        for (int rb = 0; rb < 2; ++rb) {
#pragma unroll
            for (int i = 0; i < 16; ++i) s[rb][i] = 0.f;
#pragma unroll
            for (int ks = 0; ks < 8; ++ks) {
                const int key = 32 * rb + c32;
                const h8_t a = __builtin_bit_cast(h8_t, kt[key * 16 + ((2 * ks + h) ^ (key & 15))]);
                s[rb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, qf[ks], s[rb], 0, 0, 0);
            }
        }
        // ---- masking (only a block that reaches past the wave's first query's last key), running maximum,
        //      probabilities; the accumulators are rescaled only when some lane's maximum moved
        if (key0 + 63 > my_first) {
            const int limit = past + q0 + c32 - key0 - 4 * h;  // last visible key of this lane's query, in the lane's numbering
#pragma unroll
            for (int rb = 0; rb < 2; ++rb)
#pragma unroll
                for (int i = 0; i < 16; ++i)
                    if (32 * rb + 8 * (i >> 2) + (i & 3) > limit) s[rb][i] = -INFINITY;
        }
        float mx = -INFINITY;
#pragma unroll
        for (int i = 0; i < 16; ++i) mx = max3(mx, s[0][i], s[1][i]);
        mx = fmaxf(mx, __shfl_xor(mx, 32)) * scale_log2e;  // (the scale is positive: the maximum commutes with it)
        const float m_new = fmaxf(m, mx);
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;  // (a query beyond S in a clamped row: nothing visible yet)
        float sum = 0.f;
        h8_t pf[2][2];
#pragma unroll
        for (int rb = 0; rb < 2; ++rb)
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int t = 0; t < 8; ++t) {
                    const float pv = __builtin_amdgcn_exp2f(__builtin_fmaf(s[rb][8 * u + t], scale_log2e, -m_use));
                    sum += pv;
                    pf[rb][u][t] = (_Float16)pv;
                }
        if (__any(m_new != m)) {
            const float corr = __builtin_amdgcn_exp2f(m - m_use);
            l *= corr;
#pragma unroll
            for (int db = 0; db < 4; ++db)
#pragma unroll
                for (int i = 0; i < 16; ++i) o[db][i] *= corr;
            m = m_new;
        }
        l += sum;
        // ---- O^T += V^T P^T: per step of 16 keys four independent products (the four blocks of 32 dims), the V^T
        //      fragments of the next step requested before this step's products are issued
        h8_t va[2][4];
        auto read_v = [&](int step, int slot) {
#pragma unroll
            for (int db = 0; db < 4; ++db) {
                const int d = 32 * db + c32;
                va[slot][db] = __builtin_bit_cast(h8_t, vt[d * 8 + ((2 * step + h) ^ ((d >> 1) & 7))]);
            }
        };
        read_v(0, 0);
#pragma unroll
        for (int step = 0; step < 4; ++step) {
            if (step < 3) read_v(step + 1, (step + 1) & 1);
#pragma unroll
            for (int db = 0; db < 4; ++db)
                o[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(va[step & 1][db], pf[step >> 1][step & 1], o[db], 0, 0, 0);
        }
    }

    // ---- out[b, s, head * 128 + d] = O[s, d] / l: lane (h, q) holds dims 32 * db + 8 * i + 4 * h + j of its query
    l += __shfl_xor(l, 32);
    const int row = q0 + c32;
    if (row < S) {
        const float inv = 1.0f / l;
        const int b = bh / H, head = bh - b * H;
        half_t *dst = out + (((size_t)b * S + row) * H + head) * 128;
#pragma unroll
        for (int db = 0; db < 4; ++db)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                h2_t lo, hi;
                lo.x = (half_t)(o[db][4 * i] * inv);
                lo.y = (half_t)(o[db][4 * i + 1] * inv);
                hi.x = (half_t)(o[db][4 * i + 2] * inv);
                hi.y = (half_t)(o[db][4 * i + 3] * inv);
                uint2 w;
                w.x = __builtin_bit_cast(uint32_t, lo);
                w.y = __builtin_bit_cast(uint32_t, hi);
                *reinterpret_cast<uint2 *>(dst + 32 * db + 8 * i + 4 * h) = w;
            }
    }
}

#undef FETCH_BLOCK

}  // namespace

int launch_attn_prefill(const half_t *q, const half_t *kc, const half_t *vc, half_t *out, int B, int H, int S, int capacity, int past,
                        float scale, hipStream_t stream) {
    const int qblocks = (S + 127) / 128;
    hipLaunchKernelGGL(gptq4_attn_prefill_kernel, dim3((unsigned)(qblocks * B * H)), dim3(256), 0, stream, q, kc, vc, out, H, S, capacity,
                       past, scale * 1.4426950408889634f, qblocks, B * H);
    return (int)hipGetLastError();
}
