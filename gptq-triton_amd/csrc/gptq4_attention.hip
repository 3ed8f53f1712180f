// Causal attention over a prompt for gfx950 (head dimension 128): the pass between the fused QKV + rotary projection,
// whose q and KV-cache rows it reads where they lie, and o_proj, whose input [B, S, H * 128] it writes directly.
// (The reference hands this step to torch's scaled_dot_product_attention and transposes the result,
// fused_attention.py:117-141; with a 2048-token prompt it is a sixth of the prompt pass.)
//
// One workgroup of four waves per 128 queries of one head, a wave per 32 queries; the keys come in blocks of 64
// through LDS, shared by the four waves.  Both products run on v_mfma_f32_32x32x16_f16 in their TRANSPOSED form, so
// that what one produces is what the next consumes without leaving the lane:
//   S^T = K Q^T   A = 32 keys x 16 dims out of LDS (rows of 256 bytes, 272 apart),
//                 B = the wave's queries, in registers for the whole kernel; lane (h, q) then holds, for its query
//                 column q, the scores of keys 8 * i + 4 * h + j of each half block (register 4 * i + j);
//   O^T = V^T P^T A = 32 dims x 16 keys, B = 16 keys x 32 queries: the lane's own probabilities, registers 8 * u .. 8 * u + 7
//                 of a half block for step u.  That fixes which key sits in which of the 16 contraction slots of a
//                 step - slot 8 * h + t is key 4 * h + t (t < 4) or 8 + 4 * h + t - 4 - and V^T is written to LDS with
//                 its keys in that order (the two middle groups of four swapped), rows of 64 keys = 128 bytes, 144 apart.
// The softmax runs per lane on its own query column (one exchange per block with the other half-wave for the running
// maximum; the row sums meet once, at the end), in base 2 with the scale folded in.  Blocks beyond a wave's last
// visible key are skipped by that wave; heavy and light query blocks are paired up by workgroup id (see the kernel).
#include "../../include/gptq4.h"
#include "gptq4_internal.h"

#include <mutex>

namespace {

typedef float f16x_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
constexpr int FA_K_BUF = 64 * 17, FA_V_BUF = 128 * 9;                      // 16-byte chunks per buffer
constexpr size_t FA_LDS_BYTES = (size_t)2 * (FA_K_BUF + FA_V_BUF) * 16;  // 71,680
constexpr int FA_GROUP = 4;  // heads of an XCD worked on together when it has many (1 MiB of keys and values each at 2048 tokens; 4 MiB of L2)

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
    // Two buffers of K [64 keys][16 chunks of 8 dims] and V^T [128 dims][8 chunks of 8 key slots], every row one chunk longer
    // than its data (17 and 9 chunks): the LDS serves a 16-byte read of 16 lanes at a time from 64 banks, and rows 272 /
    // 144 bytes apart put the 16 chunks into 16 different 16-byte slots of 256 - with plain strides, so that every address
    // below is a lane constant plus an immediate.
    extern __shared__ uint4 fa_smem[];
    uint4 *const k_s = fa_smem;                  // 2 x 64 x 17 chunks
    uint4 *const v_s = fa_smem + 2 * FA_K_BUF;   // 2 x 128 x 9 chunks
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int h = lane >> 5, c32 = lane & 31;
    // Workgroup id -> (head, query block).  Consecutive ids go to the eight XCDs in turn, each with an L2 of its own:
    // id % 8 picks the XCD and all query blocks of a head are given to one XCD (head % 8, for the heads up to the last
    // multiple of eight; the rest are dealt as if there were one XCD), so that a head's keys and values are fetched into
    // one L2 only.  Within an XCD the heavy halves of all its heads come first (a query block's work grows with its
    // index), then the light halves in the matching order: when the whole grid is resident at once, a CU's two workgroups
    // are blocks nq - 1 - j and j of one head and add up to the same work everywhere; when it is not, long work goes first.
    int qb, bh;
    {
        const int nb8 = nbh & ~7, cut = nb8 * nq;
        int y = blockIdx.x, heads = nbh, head_step = 1, head0 = 0;
        if (y < cut) {
            head0 = y & 7, head_step = 8, heads = nb8 >> 3, y >>= 3;
        } else {
            y -= cut, heads = nbh - nb8, head0 = nb8;
        }
        // (more than eight heads to an XCD: in groups of FA_GROUP heads, each group in the order above, so that the keys and
        // values in use stay within the L2)
        int group0 = 0;
        if (heads > 8) {
            const int per = FA_GROUP * nq, g = y / per;
            group0 = g * FA_GROUP, y -= g * per, heads = min(FA_GROUP, heads - group0);
        }
        const int half = (nq + 1) >> 1, first = heads * half;
        int hl;
        if (y < first) {
            hl = y / half;
            qb = nq - 1 - (y - hl * half);
        } else {
            const int k = y - first, low = nq - half;
            hl = k / low;
            qb = k - hl * low;
        }
        hl += group0;
        bh = head0 + hl * head_step;
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
    // (buffer loads: rows from kv_len on come back as zeros - they are masked.  The block's offset is part of the lane
    // offset: the range check does not see a scalar offset)
    const __amdgpu_buffer_rsrc_t k_rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t *>(kb), 0, (int)((uint32_t)kv_len * 256u), 0x00020000);
    const __amdgpu_buffer_rsrc_t v_rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t *>(vb), 0, (int)((uint32_t)kv_len * 256u), 0x00020000);
    const uint32_t k_voff = (uint32_t)(tid >> 4) * 256u + (uint32_t)(tid & 15) * 16u;  // + 16 keys per n
    const uint32_t v_voff = (uint32_t)(2 * (tid & 31)) * 256u + (uint32_t)(tid >> 5) * 16u;  // + 1 key per kk, + 8 chunks per n
    u32x4_t kr[4], vr[2][2];
#define FETCH_K(blk)                                                                                                      \
    _Pragma("unroll") for (int n = 0; n < 4; ++n)                                                                         \
        kr[n] = __builtin_amdgcn_raw_buffer_load_b128(k_rs, k_voff + 16u * 256u * n + (uint32_t)(blk) * (64u * 256u), 0, 0);
#define FETCH_V(blk)                                                                                                      \
    _Pragma("unroll") for (int n = 0; n < 2; ++n) _Pragma("unroll") for (int kk = 0; kk < 2; ++kk)                        \
        vr[n][kk] = __builtin_amdgcn_raw_buffer_load_b128(v_rs, v_voff + 256u * kk + 128u * n + (uint32_t)(blk) * (64u * 256u), 0, 0);
    const int vslot = key_slot(2 * (tid & 31));  // even: the pair's dword
    uint4 *const k_put = k_s + (tid >> 4) * 17 + (tid & 15);                                          // + 16 rows per n
    uint32_t *const v_put = reinterpret_cast<uint32_t *>(v_s) + (8 * (tid >> 5)) * 36 + (vslot >> 1);  // + 36 dwords per dim
    auto stage_k = [&](int buf) {
#pragma unroll
        for (int n = 0; n < 4; ++n) k_put[buf * FA_K_BUF + n * (16 * 17)] = __builtin_bit_cast(uint4, kr[n]);
    };
    auto stage_v = [&](int buf) {
#pragma unroll
        for (int n = 0; n < 2; ++n)
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const uint32_t lo = vr[n][0][e >> 1], hi = vr[n][1][e >> 1];
                // halves e of the two keys: bytes (0, 1) or (2, 3) of each word
                const uint32_t w = (e & 1) ? __builtin_amdgcn_perm(hi, lo, 0x07060302u) : __builtin_amdgcn_perm(hi, lo, 0x05040100u);
                v_put[buf * (FA_V_BUF * 4) + (64 * n + e) * 36] = w;
            }
    };
    // ---- S^T = K Q^T for the two half blocks of 32 keys of the block in K buffer `buf`
    auto scores = [&](int buf, f16x_t(&s)[2]) {
        const uint4 *const kt = k_s + buf * FA_K_BUF + c32 * 17 + h;  // the lane's key row of a half block, chunk h
#pragma unroll
        for (int rb = 0; rb < 2; ++rb) {
#pragma unroll
            for (int i = 0; i < 16; ++i) s[rb][i] = 0.f;
#pragma unroll
            for (int ks = 0; ks < 8; ++ks) {
                const h8_t a = __builtin_bit_cast(h8_t, kt[rb * (32 * 17) + 2 * ks]);
                s[rb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, qf[ks], s[rb], 0, 0, 0);
            }
        }
    };

    // ---- The order of work.  K is staged two blocks ahead of the block whose probabilities are being made and V one, in two
    //      buffers each, with one barrier per block: in step i the wave takes the scores of block i, made in step i - 1,
    //      issues the products for the scores of block i + 1, and turns block i's scores into probabilities while the matrix
    //      cores work on those; then O^T += V^T P^T for block i.  Step i writes K block i + 2 over block i (last read in
    //      step i - 1) and V block i + 1 over block i - 1.
    {
        FETCH_K(0)
        FETCH_V(0)
        u32x4_t k1[4];  // (block 1 of K asked for together with block 0: one round trip to memory before the first product)
        if (nblk > 1) {
#pragma unroll
            for (int n = 0; n < 4; ++n) k1[n] = __builtin_amdgcn_raw_buffer_load_b128(k_rs, k_voff + 16u * 256u * n + 64u * 256u, 0, 0);
        }
        stage_k(0);
        stage_v(0);
        if (nblk > 1) {
#pragma unroll
            for (int n = 0; n < 4; ++n) k_put[FA_K_BUF + n * (16 * 17)] = __builtin_bit_cast(uint4, k1[n]);
            FETCH_V(1)
            if (nblk > 2) {
                FETCH_K(2)
            }
        }
    }
    __syncthreads();
    f16x_t sa[2], sb[2];
    scores(0, sa);
    auto step = [&](int blk, f16x_t(&s)[2], f16x_t(&sn)[2]) {
        const int buf = blk & 1;
        __syncthreads();  // K block blk + 1 and V block blk are in their buffers; the buffers written below have been read
        if (blk + 1 < nblk) {
            stage_v(buf ^ 1);
            if (blk + 2 < nblk) {
                FETCH_V(blk + 2)
                stage_k(buf);
                if (blk + 3 < nblk) {
                    FETCH_K(blk + 3)
                }
            }
        }
        const uint4 *const vt = v_s + buf * FA_V_BUF + c32 * 9 + h;  // the lane's dim row of a block of 32, chunk h
        const int key0 = blk * 64;
        if (key0 > my_last) return;  // nothing in this block is visible to the wave (it still takes part in the staging)

        // ---- masking (only a block that reaches past the wave's first query's last key)
        if (key0 + 63 > my_first) {
            asm volatile("" ::: "memory");  // (keeps this a branch: turned into selects the masking would run for every block)
            const int limit = past + q0 + c32 - key0 - 4 * h;  // last visible key of this lane's query, in the lane's numbering
#pragma unroll
            for (int rb = 0; rb < 2; ++rb)
#pragma unroll
                for (int i = 0; i < 16; ++i)
                    if (32 * rb + 8 * (i >> 2) + (i & 3) > limit) s[rb][i] = -INFINITY;
        }
        // ---- the next block's scores (whatever the buffer holds after the last block: nobody reads them), then the
        //      running maximum and the probabilities of this one; the accumulators are rescaled only when some lane's
        //      maximum moved
        // (ahead of the other workgroup's wave on this SIMD while that one is staging or waiting at its barrier: 656 -> 622 us
        // at 416 heads, 84.6 -> 80.1 at 40)
        __builtin_amdgcn_s_setprio(1);
        scores(buf ^ 1, sn);
        float mx = -INFINITY;
#pragma unroll
        for (int i = 0; i < 16; ++i) mx = max3(mx, s[0][i], s[1][i]);
        mx = fmaxf(mx, __shfl_xor(mx, 32)) * scale_log2e;  // (the scale is positive: the maximum commutes with it)
        const float m_new = fmaxf(m, mx);
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;  // (a query beyond S in a clamped row: nothing visible yet)
        float sum = 0.f;
        const h2_t ones = {(_Float16)1.0f, (_Float16)1.0f};
        h8_t pf[2][2];
#pragma unroll
        for (int rb = 0; rb < 2; ++rb)
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int t = 0; t < 8; t += 2) {
                    // (the row sum takes the probabilities as the product takes them: rounded to fp16, two per instruction)
                    h2_t pp;
                    pp.x = (_Float16)__builtin_amdgcn_exp2f(__builtin_fmaf(s[rb][8 * u + t], scale_log2e, -m_use));
                    pp.y = (_Float16)__builtin_amdgcn_exp2f(__builtin_fmaf(s[rb][8 * u + t + 1], scale_log2e, -m_use));
                    sum = __builtin_amdgcn_fdot2(pp, ones, sum, false);
                    pf[rb][u][t] = pp.x;
                    pf[rb][u][t + 1] = pp.y;
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
        auto read_v = [&](int st, int slot) {
#pragma unroll
            for (int db = 0; db < 4; ++db) va[slot][db] = __builtin_bit_cast(h8_t, vt[db * (32 * 9) + 2 * st]);
        };
        read_v(0, 0);
#pragma unroll
        for (int st = 0; st < 4; ++st) {
            if (st < 3) read_v(st + 1, (st + 1) & 1);
#pragma unroll
            for (int db = 0; db < 4; ++db)
                o[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(va[st & 1][db], pf[st >> 1][st & 1], o[db], 0, 0, 0);
        }
        __builtin_amdgcn_s_setprio(0);
    };
    for (int blk = 0; blk < nblk; blk += 2) {
        step(blk, sa, sb);
        if (blk + 1 < nblk) step(blk + 1, sb, sa);
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

#undef FETCH_K
#undef FETCH_V

}  // namespace

int launch_attn_prefill(const half_t *q, const half_t *kc, const half_t *vc, half_t *out, int B, int H, int S, int capacity, int past,
                        float scale, hipStream_t stream) {
    const int qblocks = (S + 127) / 128;
    static bool prepared[64] = {};  // per device: the attribute belongs to the kernel as loaded on one device
    static std::mutex lock;
    {
        int device = 0;
        if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return (int)hipErrorInvalidDevice;
        std::lock_guard<std::mutex> guard(lock);
        if (!prepared[device]) {  // more than the 64 KiB a launch may ask for unless the kernel is marked for it
            const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&gptq4_attn_prefill_kernel),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)FA_LDS_BYTES);
            if (e != hipSuccess) return (int)e;
            prepared[device] = true;
        }
    }
    hipLaunchKernelGGL(gptq4_attn_prefill_kernel, dim3((unsigned)(qblocks * B * H)), dim3(256), FA_LDS_BYTES, stream, q, kc, vc, out, H, S,
                       capacity, past, scale * 1.4426950408889634f, qblocks, B * H);
    return (int)hipGetLastError();
}
