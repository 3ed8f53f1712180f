// Tiled dequant-fused matmul for gfx950 (prefill and any M > 16).
//
// v_mfma_f32_32x32x16_f16 with fp32 accumulation.  The checkpoint layout already IS
// the matrix-core B layout: one packed word = 8 consecutive k of one column = one
// lane's B operand for a 16-deep K step.  So the weights never touch LDS: every lane
// loads 128 bits (4 adjacent columns x 8 k) straight from global memory, decodes the
// 4 words in registers and uses word t as the B operand of column tile t, whose 32
// columns are {4j + t}.  Each decoded operand is reused by all M tiles of the wave.
// Only the activations go through LDS (stored in pair order, rows padded to 144 B).
//
// Workgroup = 4 waves as 2 (M) x 2 (N).  Wave tile = (32*MT) rows x 128 columns.
//   plain / rotary : workgroup tile (64*MT) x 256; a wave's 128 columns are one head,
//                    so the rotary partner d +- 64 is lane ^ 16 of the same register.
//   SiLU*mul       : the two N waves take the SAME 128 columns of the gate and of the
//                    up matrix; the up accumulators are handed over through LDS.
// blockIdx is remapped so each XCD (blockIdx % 8) owns a contiguous range of tiles:
// the M tiles that share a weight panel then share one L2.
#include "gptq4_internal.h"

namespace {

constexpr int BK = 64;
constexpr int LDS_ROW = BK + 8;  // halves; 144-byte rows keep 128-bit reads conflict-free

template <int EPI, int MT>
__global__ __launch_bounds__(256) void gptq4_gemm_kernel(MatmulArgs p) {
    constexpr int BM = 64 * MT;
    constexpr int BN = (EPI == EPI_SILU_MUL) ? 128 : 256;
    constexpr int A_UNITS = BM * (BK / 8) / 256;  // 16-byte units each thread stages per K tile

    __shared__ __attribute__((aligned(16))) half_t As[2][BM][LDS_ROW];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave & 1;
    const int wn = wave >> 1;
    const int l32 = lane & 31;
    const int lhi = lane >> 5;

    const int M = p.M, K = p.K, N = p.N;
    const int tiles_m = (M + BM - 1) / BM;

    // XCD-contiguous logical tile index
    const int total = gridDim.x;
    const int per = total >> 3, rem = total & 7;
    const int xcd = blockIdx.x & 7;
    const int logical = xcd * per + (xcd < rem ? xcd : rem) + (blockIdx.x >> 3);
    const int tile_n = logical / tiles_m;
    const int tile_m = logical - tile_n * tiles_m;
    const int m0 = tile_m * BM;
    const int n0 = tile_n * BN;

    const int mat = (EPI == EPI_SILU_MUL) ? wn : 0;
    const int nw0 = n0 + ((EPI == EPI_SILU_MUL) ? 0 : wn * 128);  // first column of the wave
    const int ncol = nw0 + 4 * l32;                                // lane's 4 columns
    const uint32_t *qw = p.w[mat].qweight + ncol;
    const uint32_t *qz = p.w[mat].qzeros;
    const half_t *sc = p.w[mat].scales;
    const int gs = p.groupsize;

    f16_t acc[MT][4];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[mt][t][i] = 0.f;

    uint4 a_stage[A_UNITS];
    uint4 b_cur[4], b_nxt[4];
    uint2 raw_s = make_uint2(0u, 0u);
    uint32_t raw_z = 0;
    int grp_loaded = -1, grp_decoded = -1;
    ColDecode cd[4];

    auto load_a = [&](int kt) {
#pragma unroll
        for (int u = 0; u < A_UNITS; ++u) {
            const int unit = tid + 256 * u;
            const int row = unit >> 3, ku = unit & 7;
            const int gm = m0 + row;
            const int k = kt * BK + 8 * ku;
            uint4 a = make_uint4(0u, 0u, 0u, 0u);
            if (gm < M) {
                const half_t *xr = p.x + (size_t)gm * K;
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
            a_stage[u] = a;
        }
    };
    auto store_a = [&](int buf) {
#pragma unroll
        for (int u = 0; u < A_UNITS; ++u) {
            const int unit = tid + 256 * u;
            const int row = unit >> 3, ku = unit & 7;
            *reinterpret_cast<uint4 *>(&As[buf][row][8 * ku]) = pair_order_u4(a_stage[u]);
        }
    };
    auto load_b = [&](uint4 (&b)[4], int kt) {
        const uint32_t *base = qw + (size_t)(kt * (BK / 8) + lhi) * N;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) b[ks] = *reinterpret_cast<const uint4 *>(base + (size_t)(2 * ks) * N);
        const int g = (kt * BK) / gs;
        if (g != grp_loaded) {
            grp_loaded = g;
            raw_s = *reinterpret_cast<const uint2 *>(sc + (size_t)g * N + ncol);
            raw_z = qz[(size_t)g * (N >> 3) + (ncol >> 3)];
        }
    };

    const int nk = K / BK;
    load_a(0);
    load_b(b_cur, 0);

    for (int kt = 0; kt < nk; ++kt) {
        const int buf = kt & 1;
        store_a(buf);
        // decode constants of the group this K tile belongs to (raw_* were fetched
        // together with b_cur)
        const int g = (kt * BK) / gs;
        if (g != grp_decoded) {
            grp_decoded = g;
            const uint32_t z4 = raw_z >> ((l32 & 1) * 16);
            cd[0] = make_col_decode(z4 & 0xFu, raw_s.x);
            cd[1] = make_col_decode((z4 >> 4) & 0xFu, raw_s.x >> 16);
            cd[2] = make_col_decode((z4 >> 8) & 0xFu, raw_s.y);
            cd[3] = make_col_decode((z4 >> 12) & 0xFu, raw_s.y >> 16);
        }
        __syncthreads();
        if (kt + 1 < nk) {
            load_a(kt + 1);
            load_b(b_nxt, kt + 1);
        }
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            h8_t af[MT];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const int row = wm * (32 * MT) + mt * 32 + l32;
                af[mt] = *reinterpret_cast<const h8_t *>(&As[buf][row][8 * (2 * ks + lhi)]);
            }
            const uint32_t ww[4] = {b_cur[ks].x, b_cur[ks].y, b_cur[ks].z, b_cur[ks].w};
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const h8_t bf = decode_word_h8(ww[t], cd[t]);
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    acc[mt][t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[mt], bf, acc[mt][t], 0, 0, 0);
            }
        }
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) b_cur[ks] = b_nxt[ks];
    }

    // ---- epilogue.  acc[mt][t][i]: row = 32*mt + 8*(i/4) + 4*lhi + i%4 of the wave,
    //      column = 4*l32 + t of the wave.
    const int wrow0 = m0 + wm * (32 * MT);
    if (EPI == EPI_PLAIN) {
        h2_t bias01 = {(half_t)0.f, (half_t)0.f}, bias23 = bias01;
        if (p.bias != nullptr) {
            const uint2 braw = *reinterpret_cast<const uint2 *>(p.bias + ncol);
            bias01 = as_h2(braw.x);
            bias23 = as_h2(braw.y);
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int row = wrow0 + mt * 32 + 8 * (i >> 2) + 4 * lhi + (i & 3);
                if (row < M) {
                    h2_t o01 = {(half_t)acc[mt][0][i], (half_t)acc[mt][1][i]};
                    h2_t o23 = {(half_t)acc[mt][2][i], (half_t)acc[mt][3][i]};
                    if (p.bias != nullptr) {
                        o01 = o01 + bias01;
                        o23 = o23 + bias23;
                    }
                    *reinterpret_cast<uint2 *>(p.y + (size_t)row * N + ncol) = make_uint2(as_u32(o01), as_u32(o23));
                }
            }
    } else if (EPI == EPI_SILU_MUL) {
        // hand the up accumulators (wn == 1) to the gate wave (wn == 0) with the same wm
        float *ex = reinterpret_cast<float *>(&As[0][0][0]) + wm * (64 * 64);
        static_assert(sizeof(As) >= 2 * 64 * 64 * sizeof(float), "exchange buffer does not fit");
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            __syncthreads();
            if (wn == 1) {
#pragma unroll
                for (int t = 0; t < 4; ++t)
#pragma unroll
                    for (int i = 0; i < 16; ++i) ex[(t * 16 + i) * 64 + lane] = acc[mt][t][i];
            }
            __syncthreads();
            if (wn == 0) {
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int row = wrow0 + mt * 32 + 8 * (i >> 2) + 4 * lhi + (i & 3);
                    float o[4];
#pragma unroll
                    for (int t = 0; t < 4; ++t) o[t] = silu_f32(acc[mt][t][i]) * ex[(t * 16 + i) * 64 + lane];
                    if (row < M) {
                        const h2_t o01 = {(half_t)o[0], (half_t)o[1]};
                        const h2_t o23 = {(half_t)o[2], (half_t)o[3]};
                        *reinterpret_cast<uint2 *>(p.y + (size_t)row * N + ncol) = make_uint2(as_u32(o01), as_u32(o23));
                    }
                }
            }
        }
    } else {
        const RopeArgs &r = p.rope;
        const int head_col = nw0 >> 7;  // 128-wide head index over q | k | v
        const int which = head_col / r.H;
        const int head = head_col - which * r.H;
        const int c0 = 4 * (lane & 15);  // column of the cos/sin row shared by d and d +- 64
        const bool upper = (lane & 16) != 0;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int row = wrow0 + mt * 32 + 8 * (i >> 2) + 4 * lhi + (i & 3);
                float o[4];
#pragma unroll
                for (int t = 0; t < 4; ++t) o[t] = acc[mt][t][i];
                if (which < 2) {
                    float partner[4];
#pragma unroll
                    for (int t = 0; t < 4; ++t) partner[t] = __shfl_xor(o[t], 16, 64);
                    float4 cs = make_float4(1.f, 1.f, 1.f, 1.f), sn = make_float4(0.f, 0.f, 0.f, 0.f);
                    if (row < M) {
                        const int pos = min(max(r.position_ids[row], 0), r.max_pos - 1);
                        cs = *reinterpret_cast<const float4 *>(r.cos_table + (size_t)pos * 64 + c0);
                        sn = *reinterpret_cast<const float4 *>(r.sin_table + (size_t)pos * 64 + c0);
                    }
                    const float cc[4] = {cs.x, cs.y, cs.z, cs.w};
                    const float ss[4] = {sn.x, sn.y, sn.z, sn.w};
#pragma unroll
                    for (int t = 0; t < 4; ++t)
                        o[t] = upper ? (o[t] * cc[t] + partner[t] * ss[t]) : (o[t] * cc[t] - partner[t] * ss[t]);
                }
                if (row < M) {
                    const int bb = row / r.S;
                    const int srow = row - bb * r.S;
                    half_t *dst;
                    size_t off;
                    if (which == 0) {
                        dst = r.q;
                        off = ((size_t)(bb * r.H + head) * r.S + srow) * 128;
                    } else {
                        dst = (which == 1) ? r.k : r.v;
                        off = ((size_t)(bb * r.H + head) * r.kv_capacity + r.kv_offset + srow) * 128;
                    }
                    const h2_t o01 = {(half_t)o[0], (half_t)o[1]};
                    const h2_t o23 = {(half_t)o[2], (half_t)o[3]};
                    *reinterpret_cast<uint2 *>(dst + off + 4 * l32) = make_uint2(as_u32(o01), as_u32(o23));
                }
            }
    }
}

template <int EPI, int MT>
int launch_one(const MatmulArgs &a, hipStream_t stream) {
    constexpr int BM = 64 * MT;
    constexpr int BN = (EPI == EPI_SILU_MUL) ? 128 : 256;
    const int tiles = ((a.M + BM - 1) / BM) * (a.N / BN);
    hipLaunchKernelGGL((gptq4_gemm_kernel<EPI, MT>), dim3((unsigned)tiles), dim3(256), 0, stream, a);
    return (int)hipGetLastError();
}

}  // namespace

int launch_gemm(int epi, const MatmulArgs &a, hipStream_t stream) {
    switch (epi) {
        case EPI_PLAIN:
            return launch_one<EPI_PLAIN, 2>(a, stream);
        case EPI_SILU_MUL:
            return launch_one<EPI_SILU_MUL, 2>(a, stream);
        default:
            return launch_one<EPI_ROPE, 2>(a, stream);
    }
}
