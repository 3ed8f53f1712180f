// Dequant-fused matmul for mid-sized M (17 .. a few hundred rows) on gfx950.
//
// With so few rows there is one row tile (or a handful), so the tiled kernel's tile count
// - N / 256 - leaves most CUs idle unless K is split across workgroups, and every split
// costs a round trip of fp32 partial sums through memory.  Here the split along K happens
// inside the workgroup: a workgroup owns a strip of only 64 output columns (128 for a
// rotary head), and its four waves each run the tiled kernel's wave loop over their own
// contiguous quarter of K.  The waves share nothing while they stream: each has its own
// double-buffered activation tile in LDS, filled by its own LDS-direct loads, so the loop
// has no barrier at all.  At the end the four accumulator sets meet in LDS: row block mt
// is summed and finished by wave mt.
//
// Wave tile: (32*MT) rows x NB blocks of 64 columns.
//   plain   : NB = 1, one 64-column strip; or (WIDE, long K and many rows) NB = 2, two adjacent strips.
//   SiLU*mul: NB = 2, the same 64 columns of the gate and of the up matrix.
//   rotary  : NB = 2, columns [0, 64) and [64, 128) of one head, so the wave that finishes
//             a row block holds d and d + 64 itself; or (PAIRED, few rows) NB = 1: 32 columns of a head and their
//             32 rotation partners, the two columns of a lane being d and d + 64.
// With NB = 2 every activation fragment read from LDS feeds twice as many MFMAs.
//
// Weights are decoded exactly once per row tile.  K can still be split across workgroups
// on top (last-arriver protocol of the other kernels) when the strips do not fill the
// chip; the partial sums exchanged are the workgroup's already reduced tile.
#include "gptq4_internal.h"

// Development aid, compiled out of the product build: per-workgroup stamps of the 100 MHz clock at the
// phase boundaries of the kernel, written 32 MiB into the workspace (size it so).
#ifdef GPTQ4_PHASE_TIMERS
#define KS_STAMP(i)                                                                                             \
    do {                                                                                                        \
        if (threadIdx.x == 0 && p.counters != nullptr)                                                          \
            reinterpret_cast<unsigned long long *>(reinterpret_cast<char *>(p.counters) + (32 << 20))[(blockIdx.y * gridDim.x + blockIdx.x) * 8 + (i)] = \
                wall_clock64();                                                                                 \
    } while (0)
#else
#define KS_STAMP(i)
#endif

namespace {

constexpr int BK = 64;

// WIDE (plain epilogue only): two adjacent 64-column blocks per wave tile, like a rotary head.
// KS: waves of the workgroup, each with its own slice of K (4 or 8).  A wave spends about half of its life
// waiting (first loads, the exchanges at the end) and the other half issuing ~20 instructions per MFMA, one wave
// per SIMD; the matrix cores are busy 15 % of the time (SQ counters at 128 rows, 4096 x 4096).  A second wave
// per SIMD overlaps the two.  8 waves with 64-row tiles are 128 KiB of LDS: one workgroup per CU.
// PAIRED (rotary epilogue only): the workgroup owns 32 columns of a head and their 32 rotation partners (d, d + 64)
// instead of the whole head.  The two columns of a lane are then d and d + 64 - two 4-byte loads per row instead of one
// 8-byte load of adjacent columns - so the wave tile has ONE column block, like a plain strip, twice as many workgroups
// share the projection without splitting K, and the lane that finishes a value holds its rotation partner itself.
// SB: the packed words are in streaming order and w[].qzeros holds the {scale, zero} words, as in the tiled kernel's
// variant of the same name: per column one 8-byte load of rows 2 * lhi, 2 * lhi + 1 of a four-row chunk, K step ks
// multiplies packed row 4 * (ks / 2) + 2 * lhi + ks % 2 of the tile.
template <int EPI, int MT, bool WIDE, int KS, bool PAIRED = false, bool SB = false>
// (eight waves: one workgroup per CU - all its registers - wherever the wave tile has two column blocks or two row blocks)
__global__ __launch_bounds__(64 * KS, KS == 8 && (MT == 2 || (EPI != EPI_PLAIN && !PAIRED) || WIDE) ? 1 : 2) void gptq4_kslice_kernel(MatmulArgs p) {
    static_assert(KS == 4 || KS == 8, "four or eight waves");
    static_assert(!WIDE || EPI == EPI_PLAIN, "the other epilogues have two blocks already");
    static_assert(!PAIRED || EPI == EPI_ROPE, "paired columns are a rotary head's");
    constexpr bool ADJ = (EPI == EPI_ROPE && !PAIRED) || WIDE;  // the second block is columns + 64 of the same matrix
    constexpr int BM = 32 * MT;
    constexpr int NB = ((EPI == EPI_PLAIN && !WIDE) || PAIRED) ? 1 : 2;  // 64-column blocks of the wave tile
    constexpr int BN = ADJ ? 128 : 64;                  // output columns of the workgroup
    constexpr int NSET = NB;                            // value sets the finishing wave combines
    constexpr int A_HALVES = BM * BK;                   // one wave's K tile of activations
    constexpr int A_UNITS = BM / 8;                     // LDS-direct loads per wave and K tile (8 rows each)

    // Per-wave activation tiles (two objects, so that the compiler can tell the loads into one
    // from the reads of the other).  Afterwards the same memory is MT * 4 exchange regions of
    // 8 KiB: region (mt, w) = accumulators of row block mt from wave w.
    __shared__ __attribute__((aligned(16))) half_t As0[KS * A_HALVES];
    __shared__ __attribute__((aligned(16))) half_t As1[KS * A_HALVES];
    static_assert(2 * KS * A_HALVES * sizeof(half_t) >= (size_t)MT * KS * 32 * 64 * sizeof(float), "exchange regions do not fit");
    auto region = [&](int mt, int w) -> float * {
        const int r = mt * KS + w;
        constexpr int HALF = MT * KS / 2;
        return reinterpret_cast<float *>(r < HALF ? As0 : As1) + (r < HALF ? r : r - HALF) * (32 * 64);
    };

    KS_STAMP(0);
    GPTQ4_FETCH_MATMUL_ARGS(p);
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ksl = wave;
    const int l32 = lane & 31;
    const int lhi = lane >> 5;

    const int M = p.M, K = p.K, N = p.N;
    const int tiles_m = (M + BM - 1) / BM;

    // XCD-contiguous logical tile index, row tiles fastest; the workgroup's K tiles [wg_begin, wg_begin + wg_len), its
    // rank `split` among the `nsplit` workgroups that share the tile, and the tile's index `xtile` among those that
    // exchange partial sums
    int logical, split, nsplit, wg_begin, wg_len, xtile;
    {
        const bool tail = p.tail_split > 1;  // one-dimensional grid: whole tiles first, then the parts of the shared ones
        const int total = tail ? p.tail_first : (int)gridDim.x;
        const int per = total >> 3, rem = total & 7;
        const int xcd = blockIdx.x & 7;
        logical = xcd * per + (xcd < rem ? xcd : rem) + (blockIdx.x >> 3);
        if (!tail) {
            split = blockIdx.y;
            nsplit = p.splitk;
            wg_begin = split * p.slot_q + min(split, p.slot_rem);
            wg_len = p.slot_q + (split < p.slot_rem ? 1 : 0);
            xtile = logical;
        } else if ((int)blockIdx.x < total) {
            split = 0, nsplit = 1, wg_begin = 0, wg_len = p.K / BK, xtile = 0;
        } else {
            const int s = p.tail_split, w = (int)blockIdx.x - total;
            xtile = w / s;
            split = w - xtile * s;
            logical = total + xtile;
            nsplit = s;
            const int nkt = p.K / BK, q = nkt / s, r = nkt - q * s;
            wg_begin = split * q + min(split, r);
            wg_len = q + (split < r ? 1 : 0);
        }
    }
    const int tile_n = logical / tiles_m;
    const int tile_m = logical - tile_n * tiles_m;
    const int m0 = tile_m * BM;
    // the launch covers columns [n_begin, n_begin + n_count) of the N; PAIRED: tile_n counts quarter heads,
    // n0 = the first of the tile's 32 low columns
    const int n0 = PAIRED ? p.n_begin + (tile_n >> 1) * 128 + (tile_n & 1) * 32 : p.n_begin + tile_n * BN;

    // block j of the wave tile: matrix j at the strip's columns (SiLU*mul), or columns
    // 64*j .. 64*j + 63 of the head (rotary); the lane's 2 columns of it (PAIRED: ncol and ncol + 64)
    const int ncol = PAIRED ? n0 + l32 : n0 + 2 * l32;
    // (for rotary the second block is a constant offset from the first: no second set of pointers)
    constexpr int NPTR = (EPI == EPI_SILU_MUL) ? 2 : 1;
    const uint32_t *bptr_[NPTR];
    const uint32_t *qz_[NPTR];
    const half_t *sc_[NPTR];
#pragma unroll
    for (int j = 0; j < NPTR; ++j) {
        bptr_[j] = p.w[j].qweight + (size_t)lhi * N + ncol;  // row lhi of K tile 0
        qz_[j] = p.w[j].qzeros + (ncol >> 3);
        sc_[j] = p.w[j].scales + ncol;
    }
    auto bptr = [&](int j) { return ADJ ? bptr_[0] + 64 * j : bptr_[j < NPTR ? j : 0]; };
    // SB: word offset of the lane's rows 2 * lhi, 2 * lhi + 1 of chunk 0 of column ncol, and of its {scale, zero} word of
    // group 0; 64 columns on are four strips on
    const uint32_t sb_strip = (uint32_t)(K >> 7) * 256u;            // words of a strip
    const uint32_t sb_groups16 = (uint32_t)(K / p.groupsize) * 16u;  // {scale, zero} words of a strip
    const uint32_t sb_off = (uint32_t)(ncol >> 4) * sb_strip + (uint32_t)(ncol & 15) * 4u + 2u * lhi;
    const uint32_t sb_moff = (uint32_t)(ncol >> 4) * sb_groups16 + (uint32_t)(ncol & 15);
    auto sb_words = [&](int j) { return p.w[(EPI == EPI_SILU_MUL) ? j : 0].qweight + ((ADJ && j) ? 4 * sb_strip : 0u); };
    auto sb_meta = [&](int j) { return p.w[(EPI == EPI_SILU_MUL) ? j : 0].qzeros + ((ADJ && j) ? 4 * sb_groups16 : 0u); };
    auto qz = [&](int j) { return ADJ ? qz_[0] + 8 * j : qz_[j < NPTR ? j : 0]; };
    auto sc = [&](int j) { return ADJ ? sc_[0] + 64 * j : sc_[j < NPTR ? j : 0]; };
    const int tiles_per_group = p.groupsize / BK;
    const int last_group = K / p.groupsize - 1;

    f16_t acc[NB][MT][2];
#pragma unroll
    for (int j = 0; j < NB; ++j)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int i = 0; i < 16; ++i) acc[j][mt][t][i] = 0.f;

    // K tiles of the workgroup (split across workgroups), then of this wave
    const int wq = wg_len / KS, wr = wg_len % KS;
    const int k_begin = wg_begin + ksl * wq + min(ksl, wr);
    const int nk = k_begin + wq + (ksl < wr ? 1 : 0);

    if (nk > k_begin) {
        half_t *const buf0 = As0 + wave * A_HALVES;
        half_t *const buf1 = As1 + wave * A_HALVES;
        // Activations global -> LDS directly.  One instruction fills 8 rows x 8 chunks of 16
        // bytes; the chunk that lands at position c of row r is global chunk c ^ ((r >> 1) & 7),
        // which makes the 128-bit fragment reads conflict-free without padding.  Rows of a
        // unit are 8u + lane / 8, so the swizzle term is (lane >> 4) for even u and that ^ 4
        // for odd u: two per-lane offsets, everything else is a scalar offset.
        const int valid = min(BM, M - m0);
        const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(
            (void *)(p.x + (size_t)m0 * K), 0, (int)((uint32_t)valid * (uint32_t)K * 2u), 0x00020000);
        const int r8 = lane >> 3, c8 = lane & 7;
        const int voff_even = (r8 * K + 8 * (c8 ^ (r8 >> 1))) * 2;
        const int voff_odd = (r8 * K + 8 * (c8 ^ (r8 >> 1) ^ 4)) * 2;
        const bool full = (valid == BM);
        auto dma_a = [&](half_t *dst, int kt) {
            if (full) {
#pragma unroll
                for (int u = 0; u < A_UNITS; ++u)
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, (__attribute__((address_space(3))) void *)(dst + u * 512), 16,
                                                             (u & 1) ? voff_odd : voff_even, (8 * u * K + kt * BK) * 2, 0, 0);
            } else {
                // last row tile: rows beyond M load row M-1 instead (the scalar offset is not
                // covered by the buffer's range check, so the row has to be clamped per lane)
#pragma unroll
                for (int u = 0; u < A_UNITS; ++u) {
                    const int row = min(8 * u + r8, valid - 1);
                    const int chunk = c8 ^ (r8 >> 1) ^ ((u & 1) ? 4 : 0);
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, (__attribute__((address_space(3))) void *)(dst + u * 512), 16,
                                                             (row * K + 8 * chunk) * 2, kt * (BK * 2), 0, 0);
                }
            }
            asm volatile("" ::: "memory");  // the loads that follow stay behind these
        };
        const int sw = (l32 >> 1) & 7;  // (row >> 1) & 7 for every row this lane reads (rows = 32*j + l32)

        // Packed words of two K tiles: slot [par][ks] holds step ks of a tile of parity par.  It
        // is decoded during step ks - 1 and refilled during step ks - once its old contents
        // are dead, so the load can land in place - with the same step two tiles on.
        uint2 b2[NB][2][4];
        // (SB: slot [par][2 * m + t] holds, for column t, the words of steps 2 * m and 2 * m + 1; both are refilled during step
        // 2 * m + 1)
        auto load_b2 = [&](int par, int kt, int ks) {
            if constexpr (SB) {
                if (ks & 1) {
                    const uint32_t off = sb_off + (uint32_t)(2 * min(kt, nk - 1) + (ks >> 1)) * 64u;
#pragma unroll
                    for (int j = 0; j < NB; ++j) {
                        const uint32_t *src = sb_words(j) + off;
                        b2[j][par][ks - 1] = *reinterpret_cast<const uint2 *>(src);
                        b2[j][par][ks] = *reinterpret_cast<const uint2 *>(src + (PAIRED ? 4 * sb_strip : 4u));
                    }
                }
                return;
            }
            const size_t off = ((size_t)min(kt, nk - 1) * (BK / 8) + 2 * ks) * N;
            if constexpr (PAIRED) {
                b2[0][par][ks].x = bptr_[0][off];
                b2[0][par][ks].y = bptr_[0][off + 64];
            } else {
#pragma unroll
                for (int j = 0; j < NB; ++j) b2[j][par][ks] = *reinterpret_cast<const uint2 *>(bptr(j) + off);
            }
        };
        // Scale and zero words two tiles ahead as well; the group of the look-ahead tile is
        // tracked by counting.
        int group2 = k_begin / tiles_per_group;
        int left2 = tiles_per_group - (k_begin - group2 * tiles_per_group);
        uint32_t g_s[NB][2], g_z[NB][2];
        uint32_t g_s_hi[2], g_z_hi[2];  // PAIRED: scale and zero word of the lane's second column
        auto word_of = [&](int j, int par, int step, int t) -> uint32_t {
            if constexpr (SB) {
                const uint2 w = b2[j][par][(step & ~1) + t];
                return (step & 1) ? w.y : w.x;
            } else {
                return t ? b2[j][par][step].y : b2[j][par][step].x;
            }
        };
        auto load_group2 = [&](int par) {
            const int g = min(group2, last_group);
            if constexpr (SB) {
                // {scale | zero << 16} of the lane's two columns of each block, in g_s and g_z
#pragma unroll
                for (int j = 0; j < NB; ++j) {
                    const uint32_t *src = sb_meta(j) + sb_moff + (uint32_t)g * 16u;
                    if constexpr (PAIRED) {
                        g_s[j][par] = src[0];
                        g_z[j][par] = src[4 * sb_groups16];
                    } else {
                        const uint2 m2 = *reinterpret_cast<const uint2 *>(src);
                        g_s[j][par] = m2.x;
                        g_z[j][par] = m2.y;
                    }
                }
            } else if constexpr (PAIRED) {
                const uint16_t *const sp = reinterpret_cast<const uint16_t *>(sc_[0] + (size_t)g * N);
                g_s[0][par] = sp[0];
                g_s_hi[par] = sp[64];
                g_z[0][par] = qz_[0][(size_t)g * (N >> 3)];
                g_z_hi[par] = qz_[0][(size_t)g * (N >> 3) + 8];
            } else {
#pragma unroll
                for (int j = 0; j < NB; ++j) {
                    g_s[j][par] = *reinterpret_cast<const uint32_t *>(sc(j) + (size_t)g * N);
                    g_z[j][par] = qz(j)[(size_t)g * (N >> 3)];
                }
            }
            if (left2 == 1) {
                ++group2;
                left2 = tiles_per_group;
            } else {
                --left2;
            }
        };
        ColDecodeNat cn[NB][2];
        auto make_cn = [&](int par) {
            if constexpr (SB) {
#pragma unroll
                for (int j = 0; j < NB; ++j) {
                    cn[j][0] = make_col_decode_nat((g_s[j][par] >> 16) & 0xFu, g_s[j][par]);
                    cn[j][1] = make_col_decode_nat((g_z[j][par] >> 16) & 0xFu, g_z[j][par]);
                }
                return;
            }
            if constexpr (PAIRED) {
                const int sh = (l32 & 7) * 4;
                cn[0][0] = make_col_decode_nat((g_z[0][par] >> sh) & 0xFu, g_s[0][par]);
                cn[0][1] = make_col_decode_nat((g_z_hi[par] >> sh) & 0xFu, g_s_hi[par]);
                return;
            }
#pragma unroll
            for (int j = 0; j < NB; ++j) {
                const uint32_t z2 = g_z[j][par] >> (((2 * l32) & 7) * 4);
                cn[j][0] = make_col_decode_nat(z2 & 0xFu, g_s[j][par]);
                cn[j][1] = make_col_decode_nat((z2 >> 4) & 0xFu, g_s[j][par] >> 16);
            }
        };

        dma_a(buf0, k_begin);
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) load_b2(0, k_begin, ks);
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) load_b2(1, k_begin + 1, ks);
        load_group2(0);  // group of tile k_begin
        make_cn(0);
        load_group2(1);  // group of tile k_begin + 1, made into constants at the end of tile k_begin
        h8_t bf[NB][2];
#pragma unroll
        for (int j = 0; j < NB; ++j) {
            bf[j][0] = decode_word_natural(word_of(j, 0, 0, 0), cn[j][0]);
            bf[j][1] = decode_word_natural(word_of(j, 0, 0, 1), cn[j][1]);
        }

        // one K tile (of parity `par` counted from k_begin) from buffer `cur`, while the next
        // tile streams into `nxt`
        auto k_tile = [&](const half_t *cur, half_t *nxt, int kt, int par) {
            // Loads complete in order and this wave issued 4 * NB packed-word loads after the
            // scale/zero words that followed its LDS-direct loads of this tile: at most that
            // many outstanding means the tile has landed.  It is this wave's own tile: no barrier.
            // (tests/test_wait_counts.py counts the loads behind the tile's in the compiled code of every variant.)
            // (lgkmcnt: the fragment reads of the tile before are done before its buffer is requested again.)
            asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(4 * NB * ((PAIRED && !SB) ? 2 : 1)) : "memory");
            dma_a(nxt, min(kt + 1, nk - 1));
            load_group2(par);
            h8_t araw[MT];
            auto read_a = [&](int ks) {
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    araw[mt] = *reinterpret_cast<const h8_t *>(cur + (mt * 32 + l32) * BK +
                                                               8 * ((SB ? 4 * (ks >> 1) + 2 * lhi + (ks & 1) : 2 * ks + lhi) ^ sw));
            };
            read_a(0);
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
                h8_t af[MT];
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) af[mt] = araw[mt];
                if (ks < 3) read_a(ks + 1);
                if (ks == 3) make_cn(par ^ 1);
                load_b2(par, kt + 2, ks);           // this step's words were decoded during the previous step
                __builtin_amdgcn_sched_barrier(0);  // keep the loads above the MFMAs that hide them
#pragma unroll
                for (int j = 0; j < NB; ++j) {
                    const uint32_t next0 = (ks < 3) ? word_of(j, par, ks + 1, 0) : word_of(j, par ^ 1, 0, 0);
                    const uint32_t next1 = (ks < 3) ? word_of(j, par, ks + 1, 1) : word_of(j, par ^ 1, 0, 1);
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt)
                        acc[j][mt][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[mt], bf[j][0], acc[j][mt][0], 0, 0, 0);
                    bf[j][0] = decode_word_natural(next0, cn[j][0]);
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt)
                        acc[j][mt][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[mt], bf[j][1], acc[j][mt][1], 0, 0, 0);
                    bf[j][1] = decode_word_natural(next1, cn[j][1]);
                }
            }
        };
        KS_STAMP(1);
        int kt = k_begin;
        for (; kt + 1 < nk; kt += 2) {
            k_tile(buf0, buf1, kt, 0);
            k_tile(buf1, buf0, kt + 1, 1);
        }
        if (kt < nk) k_tile(buf0, buf1, kt, 0);
    }
    // every LDS-direct load has landed and every wave is done reading before the tiles are
    // reused for the exchange
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    KS_STAMP(3);
    __syncthreads();
    KS_STAMP(2);

    // ---- the KS accumulator sets meet, one column block at a time.  Row block mt is finished by PARTS waves
    // (one with four waves, two with eight): wave mt * PARTS + part takes registers i = part * IW .. + IW - 1.
    // acc[j][mt][t][i]: row = 32*mt + 8*(i/4) + 4*lhi + i%4 of the tile, column = 2*l32 + t of block j.
    // vals[j][t][ii], i = part * IW + ii: the sums the epilogue combines - plain: the strip; SiLU*mul: gate and
    // up; rotary: columns d < 64 and d >= 64 of the head.  Only waves < MT * PARTS hold any.
    constexpr int PARTS = KS / 4;
    constexpr int IW = 16 / PARTS;
    float vals[NSET][2][IW];
    const bool owner = wave < MT * PARTS;
    const int own_mt = wave / PARTS, part = wave % PARTS;
    const int i0 = part * IW;
#pragma unroll
    for (int j = 0; j < NB; ++j) {
        if (j > 0) __syncthreads();  // the owners are done reading the previous block
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            float *const dst = region(mt, wave);
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int i = 0; i < 16; ++i) dst[(t * 16 + i) * 64 + lane] = acc[j][mt][t][i];
        }
        __syncthreads();
#ifdef GPTQ4_PHASE_TIMERS
        if (j == 0 && nsplit == 1) KS_STAMP(6);
#endif
        if (owner) {
            const float *src[KS];
#pragma unroll
            for (int w = 0; w < KS; ++w) src[w] = region(own_mt, w) + i0 * 64 + lane;
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int ii = 0; ii < IW; ++ii) {
                    float v[KS];
#pragma unroll
                    for (int w = 0; w < KS; ++w) v[w] = src[w][(t * 16 + ii) * 64];
                    float sum = v[0];
#pragma unroll
                    for (int w = 1; w < KS; ++w) sum += v[w];
                    vals[j][t][ii] = sum;
                }
        }
    }

    KS_STAMP(4);
    constexpr int NREG = NSET * 2 * IW;  // values per lane of an owner wave
    if (nsplit > 1) {
        // K split across workgroups as well: each publishes its reduced tile (agent-scope
        // atomics, no cache maintenance), the last one to arrive sums them in split order.
        __shared__ int s_is_last;
        const int tile = xtile;
        const size_t per_split = (size_t)MT * PARTS * NREG * 64;
        float *const mine = p.partials + ((size_t)tile * nsplit + split) * per_split + (size_t)wave * NREG * 64 + lane;
        if (owner) {
#pragma unroll
            for (int s = 0; s < NSET; ++s)
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int ii = 0; ii < IW; ++ii)
                        __hip_atomic_store(mine + ((s * 2 + t) * IW + ii) * 64, vals[s][t][ii], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        KS_STAMP(5);
        __syncthreads();
        if (tid == 0) {
            const int old = __hip_atomic_fetch_add(&p.counters[tile * COUNTER_STRIDE], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            s_is_last = (old == nsplit - 1);
        }
        __syncthreads();
        KS_STAMP(6);
        if (!s_is_last) return;
        if (owner) {
            // E of the lane's values from SPR splits per round, 32 loads in flight per lane: a round is one round trip
            constexpr int E = NREG < 32 ? NREG : 32;
            constexpr int SPR = 32 / E;
            const float *const all = p.partials + (size_t)tile * nsplit * per_split + (size_t)wave * NREG * 64 + lane;
#pragma unroll
            for (int e0 = 0; e0 < NREG; e0 += E) {
                float sum[E];
#pragma unroll
                for (int e = 0; e < E; ++e) sum[e] = 0.f;
#pragma unroll 1
                for (int c0 = 0; c0 < nsplit; c0 += SPR) {
                    float got[SPR][E];
#pragma unroll
                    for (int k = 0; k < SPR; ++k)
#pragma unroll
                        for (int e = 0; e < E; ++e)  // (past the last split: the last one again, not added)
                            got[k][e] = __hip_atomic_load(all + (size_t)min(c0 + k, nsplit - 1) * per_split + (e0 + e) * 64, __ATOMIC_RELAXED,
                                                          __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
                    for (int k = 0; k < SPR; ++k)
#pragma unroll
                        for (int e = 0; e < E; ++e) sum[e] += (c0 + k < nsplit) ? got[k][e] : 0.f;
                }
#pragma unroll
                for (int e = 0; e < E; ++e) {
                    const int f = e0 + e;  // = (s * 2 + t) * IW + ii
                    vals[f / (2 * IW)][(f / IW) & 1][f % IW] = sum[e];
                }
            }
        }
        if (tid == 0) __hip_atomic_store(&p.counters[tile * COUNTER_STRIDE], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if (!owner) return;

    // ---- epilogue of registers i0 .. i0 + IW - 1 of row block own_mt
    const int row0 = m0 + own_mt * 32 + 4 * lhi;
    auto row_of = [&](int ii) { return row0 + 8 * ((i0 + ii) >> 2) + ((i0 + ii) & 3); };
    if (EPI == EPI_PLAIN) {
        // Stores go out 16 bytes per lane (store_block_rows), turned through the part of this wave's exchange region
        // that only this wave read: its own registers' slots of the first column, 64 floats per register.
        uint32_t *const tr = reinterpret_cast<uint32_t *>(region(own_mt, wave)) + i0 * 64;
        const int block_row0 = m0 + own_mt * 32 + 2 * i0;  // first row of the 2 * IW rows this wave finishes
#pragma unroll
        for (int j = 0; j < NSET; ++j) {
            h2_t bias2 = {(half_t)0.f, (half_t)0.f};
            if (p.bias != nullptr) bias2 = as_h2(*reinterpret_cast<const uint32_t *>(p.bias + ncol + 64 * j));
            uint32_t w[IW];
#pragma unroll
            for (int ii = 0; ii < IW; ++ii) {
                h2_t o = {(half_t)vals[j][0][ii], (half_t)vals[j][1][ii]};
                if (p.bias != nullptr) o = o + bias2;
                w[ii] = as_u32(o);
            }
            store_block_rows<IW>(tr, w, lane, [&](int, int rr) -> half_t * {
                const int row = block_row0 + rr;
                return row < M ? p.y + (size_t)row * N + n0 + 64 * j : nullptr;
            });
        }
    } else if (EPI == EPI_SILU_MUL) {
        // (4 bytes per lane: the output is half as wide as the tile, the wider stores gain nothing here and their
        // registers cost the loop of the 64-row variants five more spilled values)
#pragma unroll
        for (int ii = 0; ii < IW; ++ii) {
            const int row = row_of(ii);
            if (row < M) {
                const h2_t o = {(half_t)(silu_f32(vals[0][0][ii]) * vals[NSET - 1][0][ii]),
                                (half_t)(silu_f32(vals[0][1][ii]) * vals[NSET - 1][1][ii])};
                *reinterpret_cast<uint32_t *>(p.y + (size_t)row * N + n0 + 2 * l32) = as_u32(o);
            }
        }
    } else {
        // the workgroup's 128 columns are one head of q, k or v
        const RopeArgs &r = p.rope;
        const int head_col = n0 >> 7;
        const int which = head_col / r.H;
        const int head = head_col - which * r.H;
        const int cap = (which == 0) ? r.S : r.kv_capacity;
        half_t *const dst = ((which == 0) ? r.q : (which == 1) ? r.k : r.v) + (size_t)head * cap * 128 + 2 * l32;
        const size_t seq_stride = (size_t)r.H * cap * 128;
        const bool at_position = (which != 0) && r.kv_offset < 0;  // cache row = the token's position
        const int row_shift = (which == 0 || r.kv_offset < 0) ? 0 : r.kv_offset;
        int pos[IW];
        if (which < 2 || at_position) {
#pragma unroll
            for (int ii = 0; ii < IW; ++ii) pos[ii] = max(r.position_ids[min(row_of(ii), M - 1)], 0);
        }
        if constexpr (PAIRED) {
            // the lane's two values are columns d and d + 64 of the head: the same products and sums as below
            const int d = (n0 & 127) + l32;
            float c1[IW], s1[IW];
            if (which < 2) {
#pragma unroll
                for (int ii = 0; ii < IW; ++ii) {
                    const int tp = min(pos[ii], r.max_pos - 1);
                    c1[ii] = r.cos_table[(size_t)tp * 64 + d];
                    s1[ii] = r.sin_table[(size_t)tp * 64 + d];
                }
            }
#pragma unroll
            for (int ii = 0; ii < IW; ++ii) {
                const int row = row_of(ii);
                float lo = vals[0][0][ii], hi = vals[0][1][ii];
                if (which < 2) {
                    const float a = lo * c1[ii] - hi * s1[ii];
                    const float b = hi * c1[ii] + lo * s1[ii];
                    lo = a, hi = b;
                }
                if (row < M) {
                    int bb, srow;
                    split_row(r, row, bb, srow);
                    const int crow = at_position ? min(pos[ii], r.kv_capacity - 1) : srow + row_shift;
                    half_t *const at = dst - 2 * l32 + d + (size_t)bb * seq_stride + (size_t)crow * 128;
                    at[0] = (half_t)lo;
                    at[64] = (half_t)hi;
                }
            }
            KS_STAMP(7);
            return;
        }
        float2 cs[IW], sn[IW];
        if (which < 2) {
#pragma unroll
            for (int ii = 0; ii < IW; ++ii) {
                const int tp = min(pos[ii], r.max_pos - 1);
                cs[ii] = *reinterpret_cast<const float2 *>(r.cos_table + (size_t)tp * 64 + 2 * l32);
                sn[ii] = *reinterpret_cast<const float2 *>(r.sin_table + (size_t)tp * 64 + 2 * l32);
            }
        }
#pragma unroll
        for (int ii = 0; ii < IW; ++ii) {
            const int row = row_of(ii);
            float lo0 = vals[0][0][ii], lo1 = vals[0][1][ii], hi0 = vals[NSET - 1][0][ii], hi1 = vals[NSET - 1][1][ii];
            if (which < 2) {
                const float a0 = lo0 * cs[ii].x - hi0 * sn[ii].x, a1 = lo1 * cs[ii].y - hi1 * sn[ii].y;
                const float b0 = hi0 * cs[ii].x + lo0 * sn[ii].x, b1 = hi1 * cs[ii].y + lo1 * sn[ii].y;
                lo0 = a0, lo1 = a1, hi0 = b0, hi1 = b1;
            }
            // (4 bytes per lane, as for gate/up: with 16-byte stores this epilogue was 2 - 6 % slower at 256 and 512 rows
            // with the weights from HBM, and the 64-row variants spilled two more values)
            if (row < M) {
                int bb, srow;
                split_row(r, row, bb, srow);
                const int crow = at_position ? min(pos[ii], r.kv_capacity - 1) : srow + row_shift;
                half_t *const at = dst + (size_t)bb * seq_stride + (size_t)crow * 128;
                const h2_t olo = {(half_t)lo0, (half_t)lo1}, ohi = {(half_t)hi0, (half_t)hi1};
                *reinterpret_cast<uint32_t *>(at) = as_u32(olo);
                *reinterpret_cast<uint32_t *>(at + 64) = as_u32(ohi);
            }
        }
    }
    KS_STAMP(7);
}

template <int EPI, int MT, bool WIDE, int KS, bool PAIRED = false>
int launch_one(const MatmulArgs &a, int tiles, hipStream_t stream) {
    dim3 grid((unsigned)tiles, (unsigned)a.splitk), block(64 * KS);
    if (a.tail_split > 1) grid = dim3((unsigned)(a.tail_first + (tiles - a.tail_first) * a.tail_split), 1u);
    if (a.stream_b)
        hipLaunchKernelGGL((gptq4_kslice_kernel<EPI, MT, WIDE, KS, PAIRED, true>), grid, block, 0, stream, a);
    else
        hipLaunchKernelGGL((gptq4_kslice_kernel<EPI, MT, WIDE, KS, PAIRED>), grid, block, 0, stream, a);
    return (int)hipGetLastError();
}

template <int EPI, int KS>
int launch_waves(const MatmulArgs &a, const KslicePlan &pl, hipStream_t stream) {
    if constexpr (EPI == EPI_ROPE) {
        if (pl.paired)
            return pl.mt == 1 ? launch_one<EPI_ROPE, 1, false, KS, true>(a, pl.tiles, stream)
                              : launch_one<EPI_ROPE, 2, false, KS, true>(a, pl.tiles, stream);
    }
    if constexpr (KS == 8) {
        // 32-row tiles with two column blocks per wave tile are never planned with eight waves (kslice_plan)
        if (EPI == EPI_PLAIN && !pl.wide)
            return pl.mt == 1 ? launch_one<EPI_PLAIN, 1, false, 8>(a, pl.tiles, stream) : launch_one<EPI_PLAIN, 2, false, 8>(a, pl.tiles, stream);
        // (128-column strips of a plain projection on 32-row tiles are never planned with eight waves)
        if (EPI == EPI_PLAIN) return pl.mt == 1 ? (int)hipErrorInvalidValue : launch_one<EPI_PLAIN, 2, true, 8>(a, pl.tiles, stream);
        return pl.mt == 1 ? launch_one<EPI, 1, false, 8>(a, pl.tiles, stream) : launch_one<EPI, 2, false, 8>(a, pl.tiles, stream);
    } else {
        if (EPI == EPI_PLAIN && pl.wide)
            return pl.mt == 1 ? launch_one<EPI_PLAIN, 1, true, KS>(a, pl.tiles, stream) : launch_one<EPI_PLAIN, 2, true, KS>(a, pl.tiles, stream);
        return pl.mt == 1 ? launch_one<EPI, 1, false, KS>(a, pl.tiles, stream) : launch_one<EPI, 2, false, KS>(a, pl.tiles, stream);
    }
}

template <int EPI>
int launch_epi(const MatmulArgs &a, const KslicePlan &pl, hipStream_t stream) {
    return pl.waves == 8 ? launch_waves<EPI, 8>(a, pl, stream) : launch_waves<EPI, 4>(a, pl, stream);
}

}  // namespace

KsliceTuning g_kslice_tuning = {1, 0, 0, 0, 0, 0};

// Row tile: 32 rows up to M = 32, else 64 - or 32 for plain projections where that scores higher, see below.  (128-row tiles decode each weight once instead of twice at M = 128 and
// halve the instructions per MFMA, but came out no faster: 17.3 against 15.1 us on 4096 x 4096, level on
// 11008 x 4096.  Four activation tiles per wave instead of two - the tile three K tiles on requested while one is
// multiplied - gained nothing that eight waves do not gain as well.)  How far K is split across workgroups on top is
// scored below.
// One variant of the plan: the rotary epilogue on whole heads or on paired quarter heads.  *score: that of the split it
// chose (0 with a forced split).
static KslicePlan plan_variant(int epi, int M, int N, int K, bool has_perm, bool paired, double *score) {
    KslicePlan pl = {};
    // eight waves for plain projections wherever they fit (checked below): ahead of four waves by 4 - 18 % at
    // LLaMA-7B / 30B shapes from 17 to 256 rows, level at 512; the gate/up pair and the rotary epilogue take eight up to
    // 32 rows (one workgroup per CU then: two column blocks per wave tile need the registers of a whole SIMD; 7B QKV
    // 16.9 -> 15.6 us, gate/up 19.6 -> 18.6, 13B QKV 19.3 -> 18.0) and stay at four beyond (level or 3 % behind)
    // (paired quarter heads: one column block per wave tile like a plain strip, so eight waves fit as they do there)
    pl.paired = paired;
    pl.waves = g_kslice_tuning.waves ? g_kslice_tuning.waves : ((epi == EPI_PLAIN || pl.paired || M <= 32) ? 8 : 4);
    int ks = pl.waves;
    // plain projections: 128-column strips (half the activation traffic per weight byte, half the tiles) pay
    // from 256 rows on when K is long (LLaMA-7B down_proj: 39.8 -> 37.3 us at 256 rows, 66.2 -> 61.1 at 512;
    // o_proj with K = 4096 loses below 512 rows)
    pl.wide = epi == EPI_PLAIN && (g_kslice_tuning.wide > 0 || (g_kslice_tuning.wide == 0 && M >= 256 && K >= 8192));
    const int bn = ((epi == EPI_ROPE && !pl.paired) || pl.wide) ? 128 : 64;
    const int nk = K / 64;
    pl.mt = g_kslice_tuning.mt ? g_kslice_tuning.mt : (M <= 32 ? 1 : 2);
    int bm = 32 * pl.mt;
    pl.tiles = ((M + bm - 1) / bm) * (N / bn);
    const long cus = device_shape().cus;  // 256 on MI355X
    double split_score = 0.0;  // of the split choose_split returned last (automatic choice only)
    auto choose_split = [&](int ks) {
        int s = 1;
        split_score = 0.0;
        if (g_kslice_tuning.splitk > 0) {
            s = g_kslice_tuning.splitk;
        } else {
            // Score 1..8 splits by how evenly tiles * s workgroups fill 256 CUs holding two each (w / 256 up to 256,
            // else w / (512 * ceil(w / 512)), never below 0.8 from 512 workgroups on: with several rounds the
            // scheduler evens things out), every extra split at 4 % + 15 / (K tiles) of the time, at least 4 K
            // tiles per wave.  Fitted to sweeps at LLaMA-7B / 13B / 30B shapes, 32..256 rows: on average 1 % off
            // the best split (a fixed target of 512 workgroups: 2.3 %, worst case 17 %).
            const double pen = 0.04 + 15.0 / (double)nk;
            double best = -1.0;
            for (int c = 1; c <= 8 && c <= nk / (4 * ks); ++c) {
                const long w = (long)pl.tiles * c;
                double e = (w <= cus) ? (double)w / (double)cus : (double)w / ((double)(2 * cus) * (double)((w + 2 * cus - 1) / (2 * cus)));
                if (w >= 2 * cus && e < 0.8) e = 0.8;
                const double score = e / (1.0 + pen * (c - 1));
                if (score > best + 1e-9) {
                    best = score;
                    s = c;
                }
            }
            split_score = best;
        }
        if (s > GEMM_MAX_SPLITK) s = GEMM_MAX_SPLITK;
        if (s < 1 || pl.tiles > SKINNY_MAX_TILES) s = 1;
        return s;
    };
    int s = choose_split(ks);
    // Plain projections on 64-column strips, 33 rows and more: 32-row tiles as well, where twice as many tiles fill
    // the chip without a split across workgroups (or with a smaller one) - each weight is then decoded once per 32
    // rows instead of once per 64, priced at 0.85 of the rate, but the exchange through memory goes.  Same score as
    // for the splits.  4096 x 4096 at 128 rows: 256 tiles of 32 rows, 12.8 -> 11.5 us; 5120 x 5120 at 96 rows 16.2 ->
    // 12.9, 13824 x 5120 at 96 rows 32.3 -> 28.8; 64-row tiles stay where they score higher (11008 x 4096 at 128
    // rows, 5120 x 5120 at 128 rows: 320 tiles of 32 rows would not fit one round).
    if (epi == EPI_PLAIN && !pl.wide && M > 32 && g_kslice_tuning.mt == 0 && g_kslice_tuning.splitk == 0) {
        const double score2 = split_score;
        const int tiles2 = pl.tiles;
        pl.tiles = ((M + 31) / 32) * (N / bn);
        const int s1 = choose_split(ks);
        if (score2 > 0.0 && 0.85 * split_score > score2 + 1e-9 && pl.tiles <= SKINNY_MAX_TILES) {
            pl.mt = 1;
            bm = 32;
            s = s1;
        } else {
            pl.tiles = tiles2;
        }
    }
    // eight waves: 128 KiB of LDS with 64-row tiles, so only in launches of at most one workgroup per CU; with 32-row
    // tiles two workgroups share a CU and four waves a SIMD, which leaves each 128 registers - enough for one
    // column block per wave tile only, so two blocks also need the CU to themselves; and every wave needs a K tile
    // or two
    if (pl.waves == 8) {
        const int nb = ((epi == EPI_PLAIN && !pl.wide) || pl.paired) ? 1 : 2;
        if (((pl.mt == 2 || nb == 2) && (long)pl.tiles * s > cus) || (pl.mt == 1 && nb == 2 && epi == EPI_PLAIN) || nk / s < 16) {
            pl.waves = ks = 4;
            s = choose_split(ks);
        }
    }
    pl.splitk = s;
    // Unsplit tiles past a whole number of rounds (one per CU and round; two workgroups of four waves are resident
    // per CU, and two that share a CU take 1.6 times what one takes alone): up to half a round of them - whole column
    // strips, every row tile, so that a row's summation order does not depend on its place in the batch - are cut along
    // K into as many parts as spread them over the chip, and the parts run beside the whole tiles.  LLaMA-7B gate/up
    // at 128 rows: 344 tiles, 88 of them in two parts each.
    pl.tail_first = 0;
    pl.tail_split = 1;
    if (s == 1 && pl.waves == 4 && g_kslice_tuning.splitk == 0 && g_gemm_tuning.tail != 1 && pl.tiles > cus && pl.tiles <= SKINNY_MAX_TILES) {
        const long tiles_m = (M + bm - 1) / bm, strips = N / bn;
        const long rest = pl.tiles % cus;
        const long cut_strips = (rest + tiles_m - 1) / tiles_m, cut = cut_strips * tiles_m;
        if (rest > 0 && 2 * cut <= cus && cut_strips < strips) {
            long parts = cus / cut;
            if (parts > nk / (4 * ks)) parts = nk / (4 * ks);  // at least 4 K tiles per wave
            if (parts > GEMM_MAX_SPLITK) parts = GEMM_MAX_SPLITK;
            if (parts >= 2) {
                pl.tail_first = (int)(pl.tiles - cut);
                pl.tail_split = (int)parts;
            }
        }
    }
    // the wave loop needs the activations unpermuted and at least one K tile per wave
    pl.ok = !has_perm && (N % bn) == 0 && nk / s >= ks;
    *score = split_score;
    return pl;
}

// Rotary epilogue: whole heads (tiles of 128 columns) or tiles of 32 columns of a head and their 32 rotation partners -
// twice as many tiles, so that few rows fill the chip without splitting K across workgroups (an exchange of partial
// sums through memory, 3 us), at the price of two 4-byte loads per row and lane instead of one 8-byte load and half as
// many MFMAs per activation fragment (priced at 0.85 of the rate).  Each variant is planned by itself and the better
// split score wins (never with a larger split than whole heads take).  LLaMA-7B QKV: 15.7 -> 13.0 us at 17 rows, 16.2 -> 13.4 at 32 (16 rows: 12.4), 21.1 -> 16.9 at 64,
// 42.4 -> 37.0 at 192; 13B 18.7 -> 16.2 at 32, 24.6 -> 20.6 at 64; 30B 60 -> 54 at 96 rows and whole heads below that
// (312 paired tiles do not fit one round of 256 CUs).
KslicePlan kslice_plan(int epi, int M, int N, int K, bool has_perm) {
    double score = 0.0;
    if (epi != EPI_ROPE || g_kslice_tuning.paired == 2) return plan_variant(epi, M, N, K, has_perm, false, &score);
    if (g_kslice_tuning.paired == 1) return plan_variant(epi, M, N, K, has_perm, true, &score);
    double score_p = 0.0;
    const KslicePlan heads = plan_variant(epi, M, N, K, has_perm, false, &score);
    const KslicePlan pairs = plan_variant(epi, M, N, K, has_perm, true, &score_p);
    // (only where whole heads leave the chip short of two workgroups per CU: beyond that the score's steps at whole
    // rounds say nothing about twice as many, smaller tiles - 7B QKV at 512 rows: 768 whole heads 72.6 us, 1536 paired
    // tiles 87.8)
    const bool few = (long)heads.tiles < 2 * device_shape().cus;
    return (pairs.ok && few && score > 0.0 && pairs.splitk <= heads.splitk && 0.85 * score_p > score + 1e-9) ? pairs : heads;
}

size_t kslice_partial_bytes(int epi, const KslicePlan &pl) {
    // (the same with four or eight waves: eight split the 32 values per lane and block over two owner waves)
    const int nset = ((epi == EPI_PLAIN && !pl.wide) || pl.paired) ? 1 : 2;
    if (pl.tail_split > 1) return (size_t)(pl.tiles - pl.tail_first) * pl.tail_split * pl.mt * nset * 32 * 64 * sizeof(float);
    return pl.splitk > 1 ? (size_t)pl.tiles * pl.splitk * pl.mt * nset * 32 * 64 * sizeof(float) : 0;
}

int launch_kslice(int epi, const MatmulArgs &a, const KslicePlan &pl, hipStream_t stream) {
    switch (epi) {
        case EPI_PLAIN: return launch_epi<EPI_PLAIN>(a, pl, stream);
        case EPI_SILU_MUL: return launch_epi<EPI_SILU_MUL>(a, pl, stream);
        default: return launch_epi<EPI_ROPE>(a, pl, stream);
    }
}
