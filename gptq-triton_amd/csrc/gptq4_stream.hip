// Small-M (1..16 rows) dequant-fused matmul for gfx950, streaming form: the decode GEMV.
//
// The packed weights are read from HBM exactly once and are the only long-latency
// traffic; everything else is arranged so that a wave spends its instructions on
// weights:
//   * x is staged ONCE per workgroup into LDS, already in the k order the decoded
//     weights come out in ("pair order", and gathered through `perm` for act-order
//     checkpoints), so the loop reads its matrix-core A operand with one ds_read_b128
//     per K step and holds no activation registers across the HBM latency.
//   * the weights are decoded to the same fp16 values the dequantisation kernel writes
//     (one rounding, after the multiply by the scale), so the result is the matmul with
//     the fp16 weights accumulated in fp32.
//   * the loop body is branch-free around its loads (indices are clamped instead), so
//     the compiler's s_waitcnt counters stay exact and DEPTH batches really are in
//     flight per wave.
//
// Work decomposition (as in the register-operand kernel next door)
//   K step = 32 values of k = 4 qweight rows; lane l reads row l/16 and W adjacent
//            words; word t is the B operand of MFMA t (columns {W*j + t}).
//   batch  = 128 k (4 K steps), never straddles a quantisation group.
//   tile   = one strip of 16*W columns (plain), the same strip of gate and up
//            (SiLU*mul), or strips d and d+64 of one head (rotary).
//   A workgroup has NW waves, each with its own contiguous batch range; they are summed
//   through LDS.  With splitk > 1 that many workgroups share a tile and the last to
//   arrive adds the partial sums in fixed order (deterministic).
#include "gptq4_internal.h"

namespace {

template <int W>
struct WordVec;
template <>
struct WordVec<1> {
    typedef uint32_t type;
};
template <>
struct WordVec<2> {
    typedef uint2 type;
};
template <>
struct WordVec<4> {
    typedef uint4 type;
};

__device__ __forceinline__ uint32_t word_of(uint32_t v, int) { return v; }
__device__ __forceinline__ uint32_t word_of(uint2 v, int t) { return t == 0 ? v.x : v.y; }
__device__ __forceinline__ uint32_t word_of(uint4 v, int t) { return t == 0 ? v.x : (t == 1 ? v.y : (t == 2 ? v.z : v.w)); }

template <int NV, int W>
struct WBatch {
    typename WordVec<W>::type w[NV][4];  // packed weights: [strip][K step]
    uint2 raw_s[NV];                     // W fp16 scales of the lane's columns
    uint32_t raw_z[NV];                  // the zero-point word holding the lane's columns
};

template <int EPI, int W, int DEPTH, bool PERM, int NW>
__global__ __launch_bounds__(64 * NW) void gptq4_stream_kernel(MatmulArgs p) {
    constexpr int NV = (EPI == EPI_PLAIN) ? 1 : 2;
    constexpr int SW = 16 * W;
    constexpr int TILE_COLS = SW * NV;
    constexpr int Q = SW / 16;
    constexpr int LINE_TILES = (SW >= 32) ? 1 : 32 / SW;
    constexpr int NT = 64 * NW;
    constexpr int LOG_NT = (NW == 4) ? 8 : (NW == 8 ? 9 : 10);
    constexpr int XU = 6;  // x chunks per thread loaded ahead of the weights

    extern __shared__ uint4 smem[];  // x slice [M][xs_stride] (16-byte chunks, pair order), then red[NW][M][TILE_COLS]
    __shared__ int s_is_last;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lrow = lane >> 4;
    const int lcol = lane & 15;

    const int xcd = blockIdx.x & 7;
    const int j = blockIdx.x >> 3;
    const int split = blockIdx.y;
    const int sub = j % LINE_TILES;
    const int tile = ((j / LINE_TILES) * 8 + xcd) * LINE_TILES + sub;
    if (tile >= p.tiles) return;

    const int M = p.M, K = p.K, N = p.N;
    // batches [B0, B1) belong to this workgroup, [b0, b1) to this wave
    const int slot0 = split * NW;
    const int B0 = slot0 * p.slot_q + min(slot0, p.slot_rem);
    const int B1 = (slot0 + NW) * p.slot_q + min(slot0 + NW, p.slot_rem);
    const int slot = slot0 + wave;
    const int b0 = slot * p.slot_q + min(slot, p.slot_rem);
    const int b1 = b0 + p.slot_q + (slot < p.slot_rem ? 1 : 0);
    const int nchunks = (B1 - B0) * 16;  // 16-byte chunks of x per row in this workgroup's K range
    const int xs_stride = nchunks + 1;   // +1: rows start in different LDS banks
    float *red = reinterpret_cast<float *>(smem + M * xs_stride);

    // ---- x: thread -> (row, chunk) with a power-of-two number of threads per row
    const int cpr = NT >> p.m_shift;  // threads per row; 1 << m_shift >= M rows are dealt
    const int xr = tid >> (LOG_NT - p.m_shift);
    const int xc = tid & (cpr - 1);
    const half_t *xsrc = p.x + (size_t)min(xr, M - 1) * K + (size_t)B0 * 128;
    uint4 xv[XU];
    if (!PERM) {
#pragma unroll
        for (int u = 0; u < XU; ++u) {
            const int c = min(xc + u * cpr, nchunks - 1);
            xv[u] = *reinterpret_cast<const uint4 *>(xsrc + 8 * c);
        }
    }

    int n0;
    if (EPI == EPI_ROPE) {
        constexpr int per_head = 64 / SW;
        n0 = (tile / per_head) * 128 + (tile % per_head) * SW;
    } else {
        n0 = tile * SW;
    }
    const uint32_t *qw[NV];
    const uint32_t *qz[NV];
    const half_t *sc[NV];
    int ncol[NV];
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int m = (EPI == EPI_SILU_MUL) ? v : 0;
        ncol[v] = n0 + ((EPI == EPI_ROPE) ? 64 * v : 0) + W * lcol;
        qw[v] = p.w[m].qweight + ncol[v] + (size_t)lrow * N;
        qz[v] = p.w[m].qzeros + (ncol[v] >> 3);
        sc[v] = p.w[m].scales + ncol[v];
    }

    typedef typename WordVec<W>::type wvec_t;
    typedef WBatch<NV, W> batch_t;
    const bool one_per_group = p.batches_per_group == 1;

    // `valid` false: a load past the wave's range, issued only to keep the loop free of
    // branches around loads (so the wait counters stay exact); every lane then reads the
    // first bytes of the matrix - one cache line per instruction - and nobody uses them.
    auto load_batch = [&](batch_t &B, int b, bool valid) {
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const uint32_t *base = valid ? qw[v] + (size_t)(b * 16) * N : p.w[(EPI == EPI_SILU_MUL) ? v : 0].qweight;
            const size_t step = valid ? (size_t)4 * N : 0;
#pragma unroll
            for (int i = 0; i < 4; ++i) B.w[v][i] = *reinterpret_cast<const wvec_t *>(base + i * step);
        }
        const int g = one_per_group ? b : (int)__umulhi((unsigned)b, p.group_magic);
#if defined(GPTQ4_EXP) && GPTQ4_EXP >= 4
        for (int v = 0; v < NV; ++v) { B.raw_s[v] = make_uint2(0x3c003c00u, 0x3c003c00u); B.raw_z[v] = 0x77777777u; }
        return;
#endif
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const half_t *sp = sc[v] + (size_t)g * N;
            if (W == 1)
                B.raw_s[v] = make_uint2(*reinterpret_cast<const uint16_t *>(sp), 0u);
            else if (W == 2)
                B.raw_s[v] = make_uint2(*reinterpret_cast<const uint32_t *>(sp), 0u);
            else
                B.raw_s[v] = *reinterpret_cast<const uint2 *>(sp);
            B.raw_z[v] = qz[v][(size_t)g * (N >> 3)];
        }
    };

    batch_t ring[DEPTH];
    const int blast = max(b1 - 1, 0);  // always a valid batch, for the clamped loads
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) load_batch(ring[d], min(b0 + d, blast), b0 + d < b1);

    // ---- x into LDS
    if (!PERM) {
#pragma unroll
        for (int u = 0; u < XU; ++u) {
            const int c = xc + u * cpr;
            if (xr < M && c < nchunks) smem[xr * xs_stride + c] = pair_order_u4(xv[u]);
        }
        for (int c = xc + XU * cpr; c < nchunks; c += cpr) {
            const uint4 v = *reinterpret_cast<const uint4 *>(xsrc + 8 * c);
            if (xr < M) smem[xr * xs_stride + c] = pair_order_u4(v);
        }
    } else {
        // act-order: x_sorted[k] = x[perm[k]]
        const uint16_t *xs = reinterpret_cast<const uint16_t *>(p.x + (size_t)min(xr, M - 1) * K);
        for (int c = xc; c < nchunks; c += cpr) {
            const int k = B0 * 128 + 8 * c;
            const int4 i0 = *reinterpret_cast<const int4 *>(p.perm + k);
            const int4 i1 = *reinterpret_cast<const int4 *>(p.perm + k + 4);
            uint4 v;  // written directly in pair order: (0,4) (1,5) (2,6) (3,7)
            v.x = (uint32_t)xs[i0.x] | ((uint32_t)xs[i1.x] << 16);
            v.y = (uint32_t)xs[i0.y] | ((uint32_t)xs[i1.y] << 16);
            v.z = (uint32_t)xs[i0.z] | ((uint32_t)xs[i1.z] << 16);
            v.w = (uint32_t)xs[i0.w] | ((uint32_t)xs[i1.w] << 16);
            if (xr < M) smem[xr * xs_stride + c] = v;
        }
    }
    __syncthreads();

    f4_t acc[NV][W];
#pragma unroll
    for (int v = 0; v < NV; ++v)
#pragma unroll
        for (int t = 0; t < W; ++t) acc[v][t] = (f4_t){0.f, 0.f, 0.f, 0.f};

    // A operand of lane (lrow, lcol): row lcol (rows >= M alias row M-1; their outputs
    // are never stored), chunk 4*kstep + lrow of the batch
    const uint4 *xs_lane = smem + min(lcol, M - 1) * xs_stride + lrow - B0 * 16;

    auto compute_batch = [&](const batch_t &B, int b) {
        const uint4 *ap = xs_lane + b * 16;
        h8_t a[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) a[i] = __builtin_bit_cast(h8_t, ap[4 * i]);
        // decode constants of the batch's group, rebuilt every batch (a few integer ops)
        // rather than behind a "group changed" branch
        ColDecode cd[NV][W];
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const uint32_t zs = B.raw_z[v] >> (((W * lcol) & 7) * 4);
#pragma unroll
            for (int t = 0; t < W; ++t) {
                const uint32_t sw = (t >> 1) ? B.raw_s[v].y : B.raw_s[v].x;
                cd[v][t] = make_col_decode((zs >> (4 * t)) & 0xFu, sw >> (16 * (t & 1)));
            }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int v = 0; v < NV; ++v)
#pragma unroll
                for (int t = 0; t < W; ++t)
#if defined(GPTQ4_EXP) && GPTQ4_EXP >= 5
                    acc[v][t][0] += __builtin_bit_cast(float, word_of(B.w[v][i], t)) + (float)a[i][0];
#else
                    acc[v][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[i], decode_word_h8(word_of(B.w[v][i], t), cd[v][t]), acc[v][t], 0, 0, 0);
#endif
    };

    for (int b = b0; b < b1; b += DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            if (b + d < b1) compute_batch(ring[d], b + d);
            load_batch(ring[d], min(b + d + DEPTH, blast), b + d + DEPTH < b1);
        }
    }

#if defined(GPTQ4_EXP) && GPTQ4_EXP >= 7
    { float t = 0; for (int v = 0; v < NV; ++v) for (int w = 0; w < W; ++w) t += acc[v][w][0] + acc[v][w][1] + acc[v][w][2] + acc[v][w][3];
      if (t == 12345.678f) p.y[tid] = (half_t)t; return; }
#endif
    // ---- sum the waves through LDS: lane holds rows 4*lrow+i, columns W*lcol+t
#pragma unroll
    for (int v = 0; v < NV; ++v)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int row = 4 * lrow + i;
            if (row < M) {
#pragma unroll
                for (int t = 0; t < W; ++t) red[(wave * M + row) * TILE_COLS + v * SW + W * lcol + t] = acc[v][t][i];
            }
        }
    __syncthreads();

    // the first 256 threads finish the tile: thread owns elements (row = (256/SW)*q + tid/SW,
    // c = tid%SW), each with NV values; the other waves stay for the barriers only
    const int Mf = (NW > 4 && tid >= 256) ? 0 : M;
    constexpr int ROWS_PER_PASS = 256 / SW;
    const int c = tid % SW;
    const int rbase = tid / SW;
    float val[Q][NV];
#pragma unroll
    for (int q = 0; q < Q; ++q) {
        const int row = ROWS_PER_PASS * q + rbase;
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            float s = 0.f;
            if (row < Mf) {
#pragma unroll
                for (int w = 0; w < NW; ++w) s += red[(w * M + row) * TILE_COLS + v * SW + c];
            }
            val[q][v] = s;
        }
    }

    if (p.splitk > 1) {
        // Cross-workgroup exchange without cache maintenance: partial sums are written
        // and read with agent-scope relaxed atomics, which are coherent across the XCDs'
        // L2s by themselves; a release/acquire fence would add an L2 write-back and
        // invalidate per workgroup.  Ordering is by completion: every wave waits until
        // its stores are acknowledged before the barrier that precedes the arrival count.
        const size_t tile_elems = (size_t)M * TILE_COLS;
        float *mine = p.partials + ((size_t)tile * p.splitk + split) * tile_elems;
#pragma unroll
        for (int q = 0; q < Q; ++q) {
            const int row = ROWS_PER_PASS * q + rbase;
            if (row < Mf) {
#pragma unroll
                for (int v = 0; v < NV; ++v)
                    __hip_atomic_store(&mine[(size_t)row * TILE_COLS + v * SW + c], val[q][v], __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (tid == 0) {
            const int old = __hip_atomic_fetch_add(&p.counters[tile * COUNTER_STRIDE], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            s_is_last = (old == p.splitk - 1);
        }
        __syncthreads();
        if (!s_is_last) return;
        const float *all = p.partials + (size_t)tile * p.splitk * tile_elems;
#pragma unroll
        for (int q = 0; q < Q; ++q) {
            const int row = ROWS_PER_PASS * q + rbase;
            if (row < Mf) {
#pragma unroll
                for (int v = 0; v < NV; ++v) {
                    const float *src = all + (size_t)row * TILE_COLS + v * SW + c;
                    float part[SKINNY_MAX_SPLITK];
#pragma unroll
                    for (int sp = 0; sp < SKINNY_MAX_SPLITK; ++sp)
                        part[sp] = (sp < p.splitk) ? __hip_atomic_load(src + (size_t)sp * tile_elems, __ATOMIC_RELAXED,
                                                                       __HIP_MEMORY_SCOPE_AGENT)
                                                   : 0.f;
                    float s = 0.f;
#pragma unroll
                    for (int sp = 0; sp < SKINNY_MAX_SPLITK; ++sp) s += part[sp];
                    val[q][v] = s;
                }
            }
        }
        if (tid == 0) __hip_atomic_store(&p.counters[tile * COUNTER_STRIDE], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }

    // ---- epilogue
#pragma unroll
    for (int q = 0; q < Q; ++q) {
        const int row = ROWS_PER_PASS * q + rbase;
        if (row >= Mf) continue;
        if (EPI == EPI_PLAIN) {
            const int n = n0 + c;
            half_t o = (half_t)val[q][0];
            if (p.bias != nullptr) o = o + p.bias[n];
            p.y[(size_t)row * N + n] = o;
        } else if (EPI == EPI_SILU_MUL) {
            const int n = n0 + c;
            p.y[(size_t)row * N + n] = (half_t)(silu_f32(val[q][0]) * val[q][NV - 1]);
        } else {
            // columns n0 + c (d < 64) and n0 + 64 + c (its partner) of one head of q, k or v
            const RopeArgs &r = p.rope;
            const int head_col = n0 >> 7;
            const int d = (n0 & 127) + c;
            const int which = head_col / r.H;
            const int head = head_col - which * r.H;
            const int bb = row / r.S;
            const int ss = row - bb * r.S;
            float o1 = val[q][0], o2 = val[q][NV - 1];
            if (which < 2) {
                const int pos = min(max(r.position_ids[row], 0), r.max_pos - 1);
                const float cs = r.cos_table[(size_t)pos * 64 + d];
                const float sn = r.sin_table[(size_t)pos * 64 + d];
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
            dst[off + d] = (half_t)o1;
            dst[off + 64 + d] = (half_t)o2;
        }
    }
}

template <int EPI, int W, int DEPTH, int NW>
int launch_variant(const MatmulArgs &a, size_t lds_bytes, hipStream_t stream) {
    constexpr int SW = 16 * W;
    constexpr int LINE_TILES = (SW >= 32) ? 1 : 32 / SW;
    const int per_xcd = 8 * LINE_TILES;
    const int groups = (a.tiles + per_xcd - 1) / per_xcd;
    dim3 grid((unsigned)(groups * per_xcd), (unsigned)a.splitk), block(64 * NW);
    if (a.perm == nullptr)
        hipLaunchKernelGGL((gptq4_stream_kernel<EPI, W, DEPTH, false, NW>), grid, block, lds_bytes, stream, a);
    else
        hipLaunchKernelGGL((gptq4_stream_kernel<EPI, W, DEPTH, true, NW>), grid, block, lds_bytes, stream, a);
    return (int)hipGetLastError();
}

template <int EPI>
int launch_epi(const MatmulArgs &a, const SkinnyPlan &pl, size_t lds, hipStream_t stream) {
    const int key = pl.waves * 100 + pl.words * 10 + pl.depth;
    switch (key) {
        case 422: return launch_variant<EPI, 2, 2, 4>(a, lds, stream);
        case 423: return launch_variant<EPI, 2, 3, 4>(a, lds, stream);
        case 424: return launch_variant<EPI, 2, 4, 4>(a, lds, stream);
        case 442: return launch_variant<EPI, 4, 2, 4>(a, lds, stream);
        case 822: return launch_variant<EPI, 2, 2, 8>(a, lds, stream);
        case 823: return launch_variant<EPI, 2, 3, 8>(a, lds, stream);
        case 824: return launch_variant<EPI, 2, 4, 8>(a, lds, stream);
        case 842: return launch_variant<EPI, 4, 2, 8>(a, lds, stream);
        case 1622: return launch_variant<EPI, 2, 2, 16>(a, lds, stream);
        case 1623: return launch_variant<EPI, 2, 3, 16>(a, lds, stream);
        default: return -1;
    }
}

}  // namespace

// LDS the streaming kernel needs for a plan: the x slice of the workgroup with the most
// batches plus the cross-wave reduction buffer.
size_t stream_lds_bytes(int epi, int M, int K, const SkinnyPlan &pl) {
    const int nbatches = K / 128, slots = pl.splitk * pl.waves;
    const int q = nbatches / slots, rem = nbatches % slots;
    const int max_batches = pl.waves * q + (rem < pl.waves ? rem : pl.waves);
    const int tile_cols = 16 * pl.words * (epi == EPI_PLAIN ? 1 : 2);
    return (size_t)M * (max_batches * 16 + 1) * 16 + (size_t)pl.waves * M * tile_cols * sizeof(float);
}

int g_stream_enabled = 1;

// Launch shape: 32-column strips (full 128-byte lines per row).  splitk = 0 in the
// result means "no streaming variant fits" (the x slice would not fit in LDS).
SkinnyPlan stream_plan(int epi, int M, int N, int K) {
    SkinnyPlan pl;
    pl.words = g_skinny_tuning.words > 0 ? g_skinny_tuning.words : 2;
    pl.depth = g_skinny_tuning.depth > 0 ? g_skinny_tuning.depth : 2;
    pl.waves = g_skinny_tuning.waves > 0 ? g_skinny_tuning.waves : 8;
    const int sw = 16 * pl.words;
    pl.tiles = (epi == EPI_ROPE) ? (N / 128) * (64 / sw) : N / sw;
    const int k_batches = K / 128;
    int s = g_skinny_tuning.splitk > 0 ? g_skinny_tuning.splitk : 1;
    if (s > k_batches / pl.waves) s = k_batches / pl.waves;  // every wave gets a batch
    if (s > SKINNY_MAX_SPLITK) s = SKINNY_MAX_SPLITK;
    if (s < 1) s = 1;
    pl.splitk = s;
    if (!stream_has_variant(pl)) {
        pl.splitk = 0;
        return pl;
    }
    // split further until the x slice fits in 64 KiB of LDS
    while (stream_lds_bytes(epi, M, K, pl) > 65536) {
        if (pl.splitk >= SKINNY_MAX_SPLITK || (pl.splitk + 1) * pl.waves > k_batches) {
            pl.splitk = 0;
            return pl;
        }
        ++pl.splitk;
    }
    return pl;
}

bool stream_has_variant(const SkinnyPlan &pl) {
    if (pl.waves != 4 && pl.waves != 8 && pl.waves != 16) return false;
    if (pl.waves == 16) return pl.words == 2 && (pl.depth == 2 || pl.depth == 3);  // 128 VGPRs per wave
    if (pl.words == 2) return pl.depth >= 2 && pl.depth <= 4;
    return pl.words == 4 && pl.depth == 2;
}

int launch_stream(int epi, const MatmulArgs &a, const SkinnyPlan &pl, hipStream_t stream) {
    const size_t lds = stream_lds_bytes(epi, a.M, a.K, pl);
    switch (epi) {
        case EPI_PLAIN: return launch_epi<EPI_PLAIN>(a, pl, lds, stream);
        case EPI_SILU_MUL: return launch_epi<EPI_SILU_MUL>(a, pl, lds, stream);
        default: return launch_epi<EPI_ROPE>(a, pl, lds, stream);
    }
}
