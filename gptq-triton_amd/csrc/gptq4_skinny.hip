// Small-M (1..16 rows) dequant-fused matmul for gfx950: the decode GEMV / skinny GEMM.
//
// Memory-bound by design: the packed weights are streamed from HBM exactly once with
// 128-bit loads, decoded in registers and fed to v_mfma_f32_16x16x32_f16 (the 16-row
// matrix-core tile holds all of x even at M = 16; at M = 1 the unused rows cost
// nothing because the matrix pipe is otherwise idle and the decode, not the MFMA, is
// the VALU work).
//
// Work decomposition
//   strip  = 64 output columns.  A wave-wide 128-bit load covers 4 qweight rows
//            (= 32 values of k, one MFMA K step) x 64 columns: lane l reads row
//            l/16 and columns 4*(l%16) .. +3.  Word t of the lane is the complete B
//            operand of MFMA t, whose 16 columns are {4j + t}: no transposition
//            between the checkpoint layout and the matrix-core register layout.
//   batch  = 128 values of k (4 K steps): the unit of K distribution.
//   tile   = the strips one workgroup owns: 1 strip (plain), the same strip of the
//            gate and up matrices (SiLU*mul), or the 2 strips of one 128-wide head
//            (rotary: column d and its partner d + 64 meet in one workgroup).
//   The 4 waves of a workgroup take disjoint contiguous batch ranges and are summed
//   through LDS; `splitk` workgroups share a tile and are summed, in fixed order, by
//   the workgroup that arrives last (arrival counter in global memory), which also
//   runs the epilogue.  Results are therefore deterministic.
//   blockIdx -> (tile, split) keeps all splits of a tile on one XCD (blockIdx % 8),
//   so the partial sums it re-reads are in that XCD's L2.
#include "gptq4_internal.h"

namespace {

template <int NV>
struct Batch {
    uint4 w[NV][4];   // packed weights: [loaded strip][K step]
    uint4 a[4];       // activations for row lane%16, natural k order, per K step
    uint2 raw_s[NV];  // 4 fp16 scales of the lane's columns
    uint32_t raw_z[NV];
    int group;
};

template <int EPI>
__global__ __launch_bounds__(256) void gptq4_skinny_kernel(MatmulArgs p) {
    constexpr int NV = (EPI == EPI_PLAIN) ? 1 : 2;       // strips loaded per K step
    constexpr int NSTRIP = (EPI == EPI_ROPE) ? 2 : 1;    // distinct column strips per tile
    constexpr int TILE_COLS = 64 * NV;                    // columns of the LDS tile

    __shared__ float red[4][SKINNY_MAX_M][TILE_COLS];
    __shared__ int s_is_last;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int lrow = lane >> 4;  // k-block inside a K step; also output row group
    const int lcol = lane & 15;

    const int xcd = blockIdx.x & 7;
    const int j = blockIdx.x >> 3;
    const int split = j % p.splitk;
    const int tile = (j / p.splitk) * 8 + xcd;
    if (tile >= p.tiles) return;

    const int M = p.M, K = p.K, N = p.N;
    const int nbatches = K >> 7;
    const int slots = p.splitk * 4;
    const int slot = split * 4 + wave;
    const int b0 = (int)(((long)slot * nbatches) / slots);
    const int b1 = (int)(((long)(slot + 1) * nbatches) / slots);
    const int n0 = tile * 64 * NSTRIP;
    const int gs = p.groupsize;

    const uint32_t *qw[NV];
    const uint32_t *qz[NV];
    const half_t *sc[NV];
    int ncol[NV];
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int m = (EPI == EPI_SILU_MUL) ? v : 0;
        ncol[v] = n0 + ((EPI == EPI_ROPE) ? 64 * v : 0) + 4 * lcol;
        qw[v] = p.w[m].qweight + ncol[v];
        qz[v] = p.w[m].qzeros;
        sc[v] = p.w[m].scales;
    }

    f4_t acc[NV][4];
#pragma unroll
    for (int v = 0; v < NV; ++v)
#pragma unroll
        for (int t = 0; t < 4; ++t) acc[v][t] = (f4_t){0.f, 0.f, 0.f, 0.f};

    ColDecode cd[NV][4];
    int cur_group = -1;

    auto load_batch = [&](Batch<NV> &B, int b, int prev_group) {
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const uint32_t *base = qw[v] + (size_t)(b * 16 + lrow) * N;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                B.w[v][i] = *reinterpret_cast<const uint4 *>(base + (size_t)(4 * i) * N);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int k = b * 128 + 32 * i + 8 * lrow;
            uint4 a = make_uint4(0u, 0u, 0u, 0u);
            if (lcol < M) {
                const half_t *xr = p.x + (size_t)lcol * K;
                if (p.perm == nullptr) {
                    a = *reinterpret_cast<const uint4 *>(xr + k);
                } else {
                    const int4 i0 = *reinterpret_cast<const int4 *>(p.perm + k);
                    const int4 i1 = *reinterpret_cast<const int4 *>(p.perm + k + 4);
                    const uint16_t *xs = reinterpret_cast<const uint16_t *>(xr);
                    a.x = (uint32_t)xs[i0.x] | ((uint32_t)xs[i0.y] << 16);
                    a.y = (uint32_t)xs[i0.z] | ((uint32_t)xs[i0.w] << 16);
                    a.z = (uint32_t)xs[i1.x] | ((uint32_t)xs[i1.y] << 16);
                    a.w = (uint32_t)xs[i1.z] | ((uint32_t)xs[i1.w] << 16);
                }
            }
            B.a[i] = a;
        }
        B.group = (b * 128) / gs;
        if (B.group != prev_group) {
#pragma unroll
            for (int v = 0; v < NV; ++v) {
                B.raw_s[v] = *reinterpret_cast<const uint2 *>(sc[v] + (size_t)B.group * N + ncol[v]);
                B.raw_z[v] = qz[v][(size_t)B.group * (N >> 3) + (ncol[v] >> 3)];
            }
        }
    };

    auto compute_batch = [&](const Batch<NV> &B) {
        if (B.group != cur_group) {
            cur_group = B.group;
#pragma unroll
            for (int v = 0; v < NV; ++v) {
                // the lane's 4 columns are nibbles (4*lcol % 8) .. +3 of the zero word
                const uint32_t z4 = B.raw_z[v] >> ((lcol & 1) * 16);
                const h2_t s01 = as_h2(B.raw_s[v].x), s23 = as_h2(B.raw_s[v].y);
                cd[v][0] = make_col_decode(z4 & 0xFu, s01.x);
                cd[v][1] = make_col_decode((z4 >> 4) & 0xFu, s01.y);
                cd[v][2] = make_col_decode((z4 >> 8) & 0xFu, s23.x);
                cd[v][3] = make_col_decode((z4 >> 12) & 0xFu, s23.y);
            }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const h8_t a = pair_order_a(B.a[i]);
#pragma unroll
            for (int v = 0; v < NV; ++v) {
                const uint32_t ww[4] = {B.w[v][i].x, B.w[v][i].y, B.w[v][i].z, B.w[v][i].w};
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const h8_t bf = decode_word_h8(ww[t], cd[v][t]);
                    acc[v][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, bf, acc[v][t], 0, 0, 0);
                }
            }
        }
    };

    if (b0 < b1) {
        Batch<NV> cur, nxt;
        load_batch(cur, b0, -1);
        for (int b = b0; b < b1; ++b) {
            if (b + 1 < b1) load_batch(nxt, b + 1, cur.group);
            compute_batch(cur);
            if (b + 1 < b1) {
                // when the group did not change, the decode constants stay valid and
                // nxt.raw_* were not loaded
                cur = nxt;
            }
        }
    }

    // ---- sum the 4 waves through LDS: lane holds rows 4*lrow+i, columns 4*lcol+t
#pragma unroll
    for (int v = 0; v < NV; ++v)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int row = 4 * lrow + i;
            if (row < M) {
                const float4 q4 = make_float4(acc[v][0][i], acc[v][1][i], acc[v][2][i], acc[v][3][i]);
                *reinterpret_cast<float4 *>(&red[wave][row][v * 64 + 4 * lcol]) = q4;
            }
        }
    __syncthreads();

    // thread owns elements (row = 4*q + tid/64, c = tid%64), each with NV values
    const int c = tid & 63;
    const int rbase = tid >> 6;
    float val[4][NV];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const int row = 4 * q + rbase;
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            float s = 0.f;
            if (row < M) s = ((red[0][row][v * 64 + c] + red[1][row][v * 64 + c]) + red[2][row][v * 64 + c]) + red[3][row][v * 64 + c];
            val[q][v] = s;
        }
    }

    if (p.splitk > 1) {
        const size_t tile_elems = (size_t)M * TILE_COLS;
        float *mine = p.partials + ((size_t)tile * p.splitk + split) * tile_elems;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int row = 4 * q + rbase;
            if (row < M) {
#pragma unroll
                for (int v = 0; v < NV; ++v) mine[(size_t)row * TILE_COLS + v * 64 + c] = val[q][v];
            }
        }
        __threadfence();
        __syncthreads();
        if (tid == 0) {
            const int old = atomicAdd(&p.counters[tile], 1);
            s_is_last = (old == p.splitk - 1);
        }
        __syncthreads();
        if (!s_is_last) return;
        __threadfence();
        const float *all = p.partials + (size_t)tile * p.splitk * tile_elems;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int row = 4 * q + rbase;
            if (row < M) {
#pragma unroll
                for (int v = 0; v < NV; ++v) {
                    float s = 0.f;
                    for (int sp = 0; sp < p.splitk; ++sp)
                        s += all[(size_t)sp * tile_elems + (size_t)row * TILE_COLS + v * 64 + c];
                    val[q][v] = s;
                }
            }
        }
        if (tid == 0) p.counters[tile] = 0;
    }

    // ---- epilogue
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const int row = 4 * q + rbase;
        if (row >= M) continue;
        if (EPI == EPI_PLAIN) {
            const int n = n0 + c;
            half_t o = (half_t)val[q][0];
            if (p.bias != nullptr) o = o + p.bias[n];
            p.y[(size_t)row * N + n] = o;
        } else if (EPI == EPI_SILU_MUL) {
            const int n = n0 + c;
            p.y[(size_t)row * N + n] = (half_t)(silu_f32(val[q][0]) * val[q][NV - 1]);
        } else {
            // tile = one 128-wide head of q, k or v; c = d < 64, partner d + 64
            const RopeArgs &r = p.rope;
            const int which = tile / r.H;
            const int head = tile - which * r.H;
            const int bb = row / r.S;
            const int ss = row - bb * r.S;
            float o1 = val[q][0], o2 = val[q][NV - 1];
            if (which < 2) {
                const int pos = min(max(r.position_ids[row], 0), r.max_pos - 1);
                const float cs = r.cos_table[(size_t)pos * 64 + c];
                const float sn = r.sin_table[(size_t)pos * 64 + c];
                const float x1 = o1, x2 = o2;
                o1 = x1 * cs - x2 * sn;
                o2 = x2 * cs + x1 * sn;
            }
            half_t *dst;
            size_t off;
            if (which == 0) {
                dst = r.q;
                off = ((size_t)(bb * r.H + head) * r.S + ss) * 128;
            } else {
                dst = (which == 1) ? r.k : r.v;
                off = ((size_t)(bb * r.H + head) * r.kv_capacity + r.kv_offset + ss) * 128;
            }
            dst[off + c] = (half_t)o1;
            dst[off + 64 + c] = (half_t)o2;
        }
    }
}

}  // namespace

int g_forced_splitk = 0;

int skinny_pick_splitk(int tiles, int k_batches) {
    int s;
    if (g_forced_splitk > 0) {
        s = g_forced_splitk;
    } else {
        // aim for ~1024 workgroups (4 per CU) so every CU has loads in flight
        s = (1024 + tiles - 1) / tiles;
    }
    const int by_k = k_batches / 4;  // at least one batch per wave
    if (s > by_k) s = by_k;
    if (s > SKINNY_MAX_SPLITK) s = SKINNY_MAX_SPLITK;
    if (s < 1) s = 1;
    return s;
}

int launch_skinny(int epi, MatmulArgs a, hipStream_t stream) {
    const int groups = ((a.tiles + 7) / 8) * 8;
    dim3 grid((unsigned)(groups * a.splitk)), block(256);
    switch (epi) {
        case EPI_PLAIN:
            hipLaunchKernelGGL(gptq4_skinny_kernel<EPI_PLAIN>, grid, block, 0, stream, a);
            break;
        case EPI_SILU_MUL:
            hipLaunchKernelGGL(gptq4_skinny_kernel<EPI_SILU_MUL>, grid, block, 0, stream, a);
            break;
        default:
            hipLaunchKernelGGL(gptq4_skinny_kernel<EPI_ROPE>, grid, block, 0, stream, a);
            break;
    }
    return (int)hipGetLastError();
}
