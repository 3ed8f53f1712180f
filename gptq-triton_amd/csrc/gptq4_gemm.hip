// Tiled dequant-fused matmul for gfx950 (prefill and any M > 16).
//
// v_mfma_f32_32x32x16_f16 with fp32 accumulation.  The checkpoint layout already IS
// the matrix-core B layout: one packed word = 8 consecutive k of one column = one
// lane's B operand for a 16-deep K step.  So the weights never touch LDS: every lane
// loads 2 adjacent words (8 bytes; a wave covers 2 qweight rows x 64 columns = one K
// step) straight from global memory, decodes them in registers and uses word t as the
// B operand of column tile t, whose 32 columns are {2j + t}.
//
// The decode is VALU work that has to hide under the MFMAs, and each decoded operand is
// reused only by the row tiles of its own wave.  The wave tile is therefore tall and
// narrow: (32*MT) rows x 64 columns, MT = 4 by default - 8 MFMAs per pair of decoded
// words, 128 accumulator registers, two waves per SIMD.  The decode of K step s+1 is
// written between the MFMAs of step s.  Packed words and scale/zero words are loaded two
// K tiles ahead into register slots that are refilled in place; every load in the loop is
// unconditional (clamped indices), so the waits are exact vmcnt(N) and none of them
// waits for a load younger than a whole K tile.
//
// Only the activations go through LDS, double buffered, one barrier per K tile of 64.
// They are 4x the bytes of the 4-bit weights they meet, so the workgroup tile is wide:
// one tile of 128 rows serves 4 waves side by side (256 columns).  They travel
// global -> LDS directly (buffer_load ... lds: no staging registers, and - unlike the
// flat form - counted in order by the compiler's wait insertion); rows are unpadded and
// the 16-byte chunks of a row are XOR-swizzled for conflict-free fragment reads.  The
// fragments come out in natural k order, so the weights are decoded in natural order too
// (16 ops per word instead of 13, none per fragment).  With an act-order permutation the
// activations are gathered through registers instead and stored in pair order.
//
// Workgroup = 4 waves.  MT = 4: 1 (M) x 4 (N), tile 128 x 256; MT = 2: 2 x 2, tile 128 x 128
// (more tiles for mid-sized M).  N waves work in pairs:
//   plain   : every N wave takes its own 64 columns.
//   rotary  : a pair's 128 columns are one head; column d and its partner d + 64 sit in
//             the two waves at the same lane and register, and are swapped through LDS.
//   SiLU*mul: a pair takes the SAME 64 columns of the gate and of the up matrix (the
//             output tile is half as wide); up is handed over through LDS.
// blockIdx is remapped so each XCD (blockIdx % 8) owns a contiguous range of tiles, ordered
// so that the workgroups resident on it at one time share both activation tiles and weight
// panels in its L2.
#include "gptq4_internal.h"

// Development aid, compiled out of the product build: per-workgroup stamps of the 100 MHz clock at the phase
// boundaries of the kernel, written 32 MiB into the workspace (size it so).
#ifdef GPTQ4_PHASE_TIMERS
#define GM_STAMP(i)                                                                                             \
    do {                                                                                                        \
        if (threadIdx.x == 0 && p.counters != nullptr)                                                          \
            reinterpret_cast<unsigned long long *>(reinterpret_cast<char *>(p.counters) + (32 << 20))[(blockIdx.y * gridDim.x + blockIdx.x) * 8 + (i)] = \
                wall_clock64();                                                                                 \
    } while (0)
#else
#define GM_STAMP(i)
#endif

namespace {

constexpr int BK = 64;
constexpr int LDS_ROW = BK + 8;  // halves; 144-byte rows keep 128-bit reads conflict-free

// STREAM: the workgroups do not own tiles.  The K tiles of all output tiles form one sequence (in the tile order
// described below), and workgroup g of the resident grid takes the g-th of gridDim.x equal ranges of it: the
// end of one tile, whole tiles, the beginning of another.  Every CU slot then has the same amount of work whatever
// the tile count - with tiles dealt whole, 344 tiles on 512 slots leave a third of the slots idle while the CUs
// that got two set the pace, and 768 tiles are a pair and then a single one per CU.  A tile cut by a range
// boundary is finished like a split-K tile: its parts are exchanged through the workspace, the last to arrive
// adds them in K order and runs the epilogue; nobody waits for anybody.  (Measured slower than whole tiles at the
// shapes of the plan's comment, so only the tuning hook selects it.)
// SB: the packed words are in streaming order (see gptq4_stream.hip): the 8 packed rows of a K tile are two 64-byte
// chunks of four rows per column, so a lane fetches, per column, rows 2 * lhi and 2 * lhi + 1 of a chunk with one 8-byte
// load - as many loads of the same width as from the checkpoint order - and K step ks multiplies packed row
// 4 * (ks / 2) + 2 * lhi + ks % 2 of the tile instead of 2 * ks + lhi (the activation fragments follow: only an index).
template <int EPI, int MT, bool PERM, bool STREAM = false, bool SB = false>
__global__ __launch_bounds__(256, 2) void gptq4_gemm_kernel(MatmulArgs p) {
    static_assert(!STREAM || !PERM, "act-order calls reach the streamed schedule with gathered activations");
    static_assert(!SB || (!PERM && !STREAM), "streaming-order words: plain path only");
    constexpr int NW = 4;        // waves
    constexpr int NT = 64 * NW;  // threads
    constexpr int WM = (MT == 4) ? 1 : 2;  // waves along M
    constexpr int WN = NW / WM;            // waves along N
    constexpr int BM = 32 * MT * WM;
    constexpr int BN = ((EPI == EPI_SILU_MUL) ? 32 : 64) * WN;
    constexpr int A_UNITS = BM * (BK / 8) / NT;  // 16-byte units each thread stages per K tile
    constexpr int A_ROWS = NT / 8;               // rows one pass of the workgroup stages (act-order path)

    // Activation tiles.  Plain path: two unpadded buffers of BM x 64 halves filled by
    // LDS-direct loads (two separate objects, so that the compiler can tell a load into one
    // from the reads of the other); act-order path: one padded double buffer filled through
    // registers.  The epilogues reuse them as four 8 KiB exchange regions.
    constexpr int REGIONS = NW;                        // 8 KiB each
    constexpr int EX_HALVES = REGIONS * 32 * 64 * 2;          // all regions, in halves
    constexpr int A_HALVES = BM * BK;
    constexpr int S0 = PERM ? (2 * BM * LDS_ROW > EX_HALVES ? 2 * BM * LDS_ROW : EX_HALVES)
                            : (A_HALVES > EX_HALVES / 2 ? A_HALVES : EX_HALVES / 2);
    constexpr int S1 = PERM ? 8 : S0;
    __shared__ __attribute__((aligned(16))) half_t As0[S0];
    __shared__ __attribute__((aligned(16))) half_t As1[S1];
    auto region = [&](int w) -> float * {
        if (PERM) return reinterpret_cast<float *>(As0) + w * (32 * 64);
        constexpr int HALF = (REGIONS + 1) / 2;
        return reinterpret_cast<float *>(w < HALF ? As0 : As1) + (w < HALF ? w : w - HALF) * (32 * 64);
    };

    GPTQ4_FETCH_MATMUL_ARGS(p);
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = (WM == 2) ? (wave & 1) : 0;
    const int wn = (WM == 2) ? (wave >> 1) : wave;
    const int wn_pair = wn >> 1, wn_odd = wn & 1;  // SiLU*mul and rotary work on pairs of N waves
    const int l32 = lane & 31;
    const int lhi = lane >> 5;

    const int M = p.M, K = p.K, N = p.N;
    const int tiles_m = (M + BM - 1) / BM;
    __shared__ int s_is_last;
    constexpr bool ROPE_TAB = (EPI == EPI_ROPE) && (MT == 4);
    extern __shared__ __attribute__((aligned(16))) float rope_tab[];  // ROPE_TAB: [2 buffers][cos, sin][32 tokens][64]

    // One (part of a) tile: K tiles [k_begin, nk) of tile `logical`, which `nsplit` workgroups share; this one is
    // number `idx` of them in K order.  part_slot(c): where sharer c keeps its partial sums.
    auto run_part = [&](const int logical, const int k_begin, const int nk, const int nsplit, const int idx, auto part_slot) {
    GM_STAMP(0);
    // XCD-contiguous logical tile index: workgroups that run at the same time on one XCD (one
    // L2) have consecutive logical indices.  These walk GROUP_M row tiles, then move to the
    // next column panel, and only after the last panel to the next GROUP_M row tiles: the
    // ~64 workgroups resident on an XCD then cover about 8 row tiles x 8 column panels, so
    // every activation tile and every weight panel they stream is shared by 8 of them in
    // the L2 (row tiles fastest over all of M left a weight panel shared by many but an
    // activation tile by two, and the activation tiles are the larger stream).
    constexpr int GROUP_M = 8;
    const int tiles_n = p.n_count / BN;  // the tiles in this order cover columns [n_begin, n_begin + n_count) of the N
    int tile_m, tile_n;
    if (logical < tiles_m * tiles_n) {
        const int band = logical / (GROUP_M * tiles_n);  // band of GROUP_M row tiles
        const int in_band = logical - band * (GROUP_M * tiles_n);
        const int band_rows = min(GROUP_M, tiles_m - band * GROUP_M);
        tile_n = in_band / band_rows;
        tile_m = band * GROUP_M + (in_band - tile_n * band_rows);
    } else {
        // tiles cut along K: whole column panels behind those columns, row tiles fastest
        const int t = logical - tiles_m * tiles_n;
        tile_n = tiles_n + t / tiles_m;
        tile_m = t - (t / tiles_m) * tiles_m;
    }
    const int m0 = tile_m * BM;
    const int n0 = p.n_begin + tile_n * BN;

    const int mat = (EPI == EPI_SILU_MUL) ? wn_odd : 0;
    const int nw0 = n0 + ((EPI == EPI_SILU_MUL) ? wn_pair : wn) * 64;  // first column of the wave
    const int ncol = nw0 + 2 * l32;                               // lane's 2 columns
    const uint32_t *bptr = p.w[mat].qweight + (size_t)lhi * N + ncol;  // row lhi of K tile 0
    const uint32_t *qz = p.w[mat].qzeros + (ncol >> 3);
    const half_t *sc = p.w[mat].scales + ncol;
    const int tiles_per_group = p.groupsize / BK;
    const int last_group = K / p.groupsize - 1;

    f16_t acc[MT][2];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[mt][t][i] = 0.f;

    const half_t *a_base = p.x + (size_t)m0 * K;

    // Rotary epilogue of the wide tile: the cos / sin rows of the tile's 128 tokens come through LDS, a block of
    // 32 tokens (8 KiB per table) at a time in two buffers, filled by LDS-direct loads that all four waves share
    // (they need the same values: both heads of the tile, and d and d + 64 of a head, turn by the same angles).
    // Blocks 0 and 1 are asked for here, ahead of the K loop; 2 and 3 follow in the epilogue as the buffers
    // become free.  Read from memory per lane instead (16 tokens x 2 tables in registers, after the positions
    // they depend on, once per block of 32 rows), the epilogue is four round trips to memory long with the
    // matrix cores idle: the two workgroups of a CU start together and so reach it together.
    bool need_tab = false;
    int tab_voff[4][2];  // per block and unit of 4 tokens: byte offset of the lane's 16-byte chunk in the tables
    __amdgpu_buffer_rsrc_t cos_rsrc, sin_rsrc;
    if constexpr (ROPE_TAB) {
        const RopeArgs &r = p.rope;
        need_tab = (n0 >> 7) / r.H < 2;  // the tile's first head is of q or k (else both are heads of v)
        if (need_tab) {
#pragma unroll
            for (int blk = 0; blk < 4; ++blk)
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const int row = min(m0 + 32 * blk + 4 * (2 * wave + j) + (lane >> 4), M - 1);
                    const int tp = min(max(r.position_ids[row], 0), r.max_pos - 1);
                    tab_voff[blk][j] = tp * 256 + (lane & 15) * 16;
                }
        }
        cos_rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)r.cos_table, 0, (int)((uint32_t)r.max_pos * 256u), 0x00020000);
        sin_rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)r.sin_table, 0, (int)((uint32_t)r.max_pos * 256u), 0x00020000);
    }
    // wave w brings tokens 8w .. 8w + 7 of the block: one load = 4 table rows of 256 bytes = 1 KiB of LDS
    auto dma_table = [&](int blk, int buf) {
        if constexpr (ROPE_TAB) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                float *const dst = rope_tab + buf * (2 * 32 * 64) + (2 * wave + j) * 256;
                __builtin_amdgcn_raw_ptr_buffer_load_lds(cos_rsrc, (__attribute__((address_space(3))) void *)dst, 16, tab_voff[blk][j], 0, 0, 0);
                __builtin_amdgcn_raw_ptr_buffer_load_lds(sin_rsrc, (__attribute__((address_space(3))) void *)(dst + 32 * 64), 16,
                                                         tab_voff[blk][j], 0, 0, 0);
            }
            asm volatile("" ::: "memory");
        }
    };

    int group = (k_begin > 0) ? k_begin / tiles_per_group : 0;
    int left_in_group = tiles_per_group - (k_begin - group * tiles_per_group);  // K tiles left in the group
    if constexpr (PERM) {
        // ---- act-order path: the activations are gathered through registers (x_sorted[k] =
        // x[perm[k]]) and stored to LDS in pair order, rows padded to 144 bytes; the weights are
        // decoded in pair order.  Each thread owns A_UNITS 16-byte units (row, 8 k) of the tile;
        // rows beyond M read row M-1 instead of branching (A row m only feeds output row m and
        // rows >= M are never stored).
        uint32_t a_rowoff[A_UNITS];
        const int a_row = tid >> 3, a_ku = tid & 7;  // unit u of this thread: row a_row + A_ROWS*u, k-unit a_ku
#pragma unroll
        for (int u = 0; u < A_UNITS; ++u) a_rowoff[u] = (uint32_t)min(a_row + A_ROWS * u, M - 1 - m0) * (uint32_t)K;
        half_t *const a_lds = As0 + a_row * LDS_ROW + 8 * a_ku;

        uint4 a_stage[A_UNITS];
        uint2 bw[4];  // packed B words of the 4 K steps; refilled in place for the next K tile
        uint32_t raw_s, raw_z;
        ColDecode cd[2];

        auto load_a = [&](int kt) {
#pragma unroll
            for (int u = 0; u < A_UNITS; ++u) {
                const int k = kt * BK + 8 * a_ku;
                const int4 i0 = *reinterpret_cast<const int4 *>(p.perm + k);
                const int4 i1 = *reinterpret_cast<const int4 *>(p.perm + k + 4);
                const uint16_t *xs = reinterpret_cast<const uint16_t *>(a_base + a_rowoff[u]);
                uint4 a;
                a.x = (uint32_t)xs[i0.x] | ((uint32_t)xs[i0.y] << 16);
                a.y = (uint32_t)xs[i0.z] | ((uint32_t)xs[i0.w] << 16);
                a.z = (uint32_t)xs[i1.x] | ((uint32_t)xs[i1.y] << 16);
                a.w = (uint32_t)xs[i1.z] | ((uint32_t)xs[i1.w] << 16);
                a_stage[u] = a;
            }
        };
        auto store_a = [&](int buf) {
#pragma unroll
            for (int u = 0; u < A_UNITS; ++u)
                *reinterpret_cast<uint4 *>(a_lds + buf * (BM * LDS_ROW) + u * (A_ROWS * LDS_ROW)) = pair_order_u4(a_stage[u]);
        };
        auto load_b_step = [&](int kt, int ks) {
            bw[ks] = *reinterpret_cast<const uint2 *>(bptr + ((size_t)kt * (BK / 8) + 2 * ks) * N);
        };
        auto load_group = [&](int g) {
            raw_s = *reinterpret_cast<const uint32_t *>(sc + (size_t)g * N);
            raw_z = qz[(size_t)g * (N >> 3)];
        };
        // Decode constants from the raw scale / zero words.  Recomputed for every K tile from
        // that tile's own group (a few integer ops) rather than only at group boundaries:
        // with no branch around the loads that feed them, every wait in the loop is exact.
        auto make_cd = [&]() {
            const uint32_t z2 = raw_z >> (((2 * l32) & 7) * 4);
            cd[0] = make_col_decode(z2 & 0xFu, raw_s);
            cd[1] = make_col_decode((z2 >> 4) & 0xFu, raw_s >> 16);
        };

        load_a(k_begin);
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) load_b_step(k_begin, ks);
        load_group(group);
        make_cd();

        // B operands of the K step about to be multiplied.  They are decoded one step ahead,
        // in place, right after the MFMAs that consumed the previous contents were issued, so
        // the decode (VALU) of step s+1 runs under the MFMAs of step s.
        h8_t bf[2];
        bf[0] = decode_word_h8(bw[0].x, cd[0]);
        bf[1] = decode_word_h8(bw[0].y, cd[1]);
        load_b_step(min(k_begin + 1, nk - 1), 0);
        if (need_tab) {
            dma_table(0, 0);
            dma_table(1, 1);
        }

        for (int kt = k_begin; kt < nk; ++kt) {
            const int buf = kt & 1;
            store_a(buf);
            __syncthreads();
            const int kn = min(kt + 1, nk - 1), kn2 = min(kt + 2, nk - 1);
            const bool new_group = (left_in_group == 1);
            load_a(kn);
            load_group(min(group + (new_group ? 1 : 0), last_group));
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
                h8_t af[MT];
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    const int row = wm * (32 * MT) + mt * 32 + l32;
                    af[mt] = *reinterpret_cast<const h8_t *>(As0 + (buf * BM + row) * LDS_ROW + 8 * (2 * ks + lhi));
                }
                if (ks == 3) make_cd();  // constants of the next K tile; this tile's decodes are all done
                const uint2 nw = bw[(ks + 1) & 3];  // words of the next step (step 0 of the next tile when ks == 3)
                // refill: step ks+1 of the next tile (step 0 of tile kt+2 when ks == 3)
                if (ks < 3)
                    load_b_step(kn, ks + 1);
                else
                    load_b_step(kn2, 0);
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) acc[mt][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[mt], bf[0], acc[mt][0], 0, 0, 0);
                bf[0] = decode_word_h8(nw.x, cd[0]);
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) acc[mt][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[mt], bf[1], acc[mt][1], 0, 0, 0);
                bf[1] = decode_word_h8(nw.y, cd[1]);
            }
            if (new_group) {
                ++group;
                left_in_group = tiles_per_group;
            } else {
                --left_in_group;
            }
        }
    } else {
        // ---- plain path: activations go global -> LDS directly (no staging registers, so the
        // loads of tile kt+1 are in flight under the MFMAs of tile kt).  A wave instruction
        // fills 64 consecutive 16-byte chunks = 8 rows x 8 chunks; chunk c of row r sits at
        // position c ^ ((r >> 1) & 7) of its row, which makes the 128-bit fragment reads
        // (16 lanes = 16 rows, one position each) conflict-free without padding.  The lane
        // picks the global chunk that belongs at its fixed LDS slot.
        uint32_t a_goff[A_UNITS];
#pragma unroll
        for (int u = 0; u < A_UNITS; ++u) {
            const int slot = (u * NW + wave) * 64 + lane;
            const int row = slot >> 3;
            const int c = (slot & 7) ^ ((row >> 1) & 7);
            a_goff[u] = (uint32_t)min(row, M - 1 - m0) * (uint32_t)K + 8u * c;
        }
        // Buffer-addressed form of the LDS-direct load: unlike the flat/global form the compiler
        // counts it in order with the other vector-memory loads, so its waits for the packed
        // words stay exact while activation tiles are in flight.
        const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(
            (void *)a_base, 0, (int)((uint32_t)min(BM, M - m0) * (uint32_t)K * 2u), 0x00020000);
        auto dma_a = [&](half_t *dst, int kt) {
#pragma unroll
            for (int u = 0; u < A_UNITS; ++u)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, (__attribute__((address_space(3))) void *)(dst + (u * NW + wave) * 512),
                                                         16, (int)(a_goff[u] * 2u), kt * (BK * 2), 0, 0);
            asm volatile("" ::: "memory");  // the loads that follow stay behind these
        };
        const int sw = (l32 >> 1) & 7;  // (row >> 1) & 7 for every row this lane reads (rows = 32*j + l32)

        // Packed words of two K tiles: slot [par][ks] holds step ks of a tile of parity par.  It
        // is decoded during step ks - 1 and refilled during step ks - once its old contents
        // are dead, so the load can land in place - with the same step two tiles on.
        // (SB: slot [par][2 * m + t] holds, for column t, the words of steps 2 * m and 2 * m + 1; both are refilled during
        // step 2 * m + 1, when the later of the two has been decoded)
        uint2 b2[2][4];
        const uint32_t *sbptr = nullptr, *sb_meta = nullptr;
        if constexpr (SB) {
            sbptr = p.w[mat].qweight + ((size_t)(ncol >> 4) * (size_t)(K >> 7)) * 256 + (ncol & 15) * 4 + 2 * lhi;
            sb_meta = p.w[mat].qzeros + (size_t)(ncol >> 4) * (size_t)(K / p.groupsize) * 16 + (ncol & 15);  // (the meta words travel in the qzeros field)
        }
        auto load_b2 = [&](int par, int kt, int ks) {
            if constexpr (SB) {
                if (ks & 1) {
                    const uint32_t *src = sbptr + ((size_t)(2 * min(kt, nk - 1) + (ks >> 1))) * 64;
                    b2[par][ks - 1] = *reinterpret_cast<const uint2 *>(src);
                    b2[par][ks] = *reinterpret_cast<const uint2 *>(src + 4);
                }
            } else {
                b2[par][ks] = *reinterpret_cast<const uint2 *>(bptr + ((size_t)min(kt, nk - 1) * (BK / 8) + 2 * ks) * N);
            }
        };
        // the packed word of column t for step `step` of the tile of parity par
        auto word_of = [&](int par, int step, int t) -> uint32_t {
            if constexpr (SB) {
                const uint2 w = b2[par][(step & ~1) + t];
                return (step & 1) ? w.y : w.x;
            } else {
                return t ? b2[par][step].y : b2[par][step].x;
            }
        };
        dma_a(As0, k_begin);
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) load_b2(0, k_begin, ks);
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) load_b2(1, k_begin + 1, ks);
        // Scale and zero words run two tiles ahead as well: slot [par] is loaded at the top of a
        // tile of parity par with the group of the tile two on, and turned into the decode
        // constants of that tile during the last step of the tile in between.  The group of
        // the look-ahead tile is tracked by counting, like the current one.
        uint32_t g_s[2], g_z[2];
        int group2 = group, left2 = left_in_group;
        auto load_group2 = [&](int par) {
            const int g = min(group2, last_group);
            if constexpr (SB) {
                // {scale | zero << 16} of the lane's two columns: neighbours in the strip's row of the group
                const uint2 m2 = *reinterpret_cast<const uint2 *>(sb_meta + (size_t)g * 16);
                g_s[par] = m2.x;
                g_z[par] = m2.y;
            } else {
                g_s[par] = *reinterpret_cast<const uint32_t *>(sc + (size_t)g * N);
                g_z[par] = qz[(size_t)g * (N >> 3)];
            }
            if (left2 == 1) {
                ++group2;
                left2 = tiles_per_group;
            } else {
                --left2;
            }
        };
        // the activation fragments come out of LDS in natural k order, so the weights are
        // decoded in natural order too
        ColDecodeNat cn[2];
        auto make_cn = [&](int par) {
            if constexpr (SB) {
                cn[0] = make_col_decode_nat((g_s[par] >> 16) & 0xFu, g_s[par]);
                cn[1] = make_col_decode_nat((g_z[par] >> 16) & 0xFu, g_z[par]);
            } else {
                const uint32_t z2 = g_z[par] >> (((2 * l32) & 7) * 4);
                cn[0] = make_col_decode_nat(z2 & 0xFu, g_s[par]);
                cn[1] = make_col_decode_nat((z2 >> 4) & 0xFu, g_s[par] >> 16);
            }
        };
        load_group2(0);  // group of tile k_begin
        make_cn(0);
        load_group2(1);  // group of tile k_begin + 1, made into constants at the end of tile k_begin
        h8_t bf[2];
        bf[0] = decode_word_natural(word_of(0, 0, 0), cn[0]);
        bf[1] = decode_word_natural(word_of(0, 0, 1), cn[1]);

        // one K tile (of parity `par` counted from k_begin) from buffer `cur`, while the next
        // tile streams into `nxt`
        auto k_tile = [&](const half_t *cur, half_t *nxt, int kt, int par) {
            // Every wave has issued at least 4 vector-memory loads after its LDS-direct loads
            // of this tile (the scale/zero words and the packed words of 4 K steps), and
            // loads complete in order: at most 4 outstanding means the tile has landed.
            // (tests/test_wait_counts.py counts the loads behind the tile's in the compiled code of every variant.)
            asm volatile("s_waitcnt vmcnt(4) lgkmcnt(0)\n\ts_barrier" ::: "memory");
            dma_a(nxt, min(kt + 1, nk - 1));
            load_group2(par);
            // fragments of K step ks+1 are read from LDS before the MFMAs of step ks are issued
            h8_t araw[MT];
            auto read_a = [&](int ks) {
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    const int row = wm * (32 * MT) + mt * 32 + l32;
                    const int chunk = SB ? 4 * (ks >> 1) + 2 * lhi + (ks & 1) : 2 * ks + lhi;
                    araw[mt] = *reinterpret_cast<const h8_t *>(cur + row * BK + 8 * (chunk ^ sw));
                }
            };
            read_a(0);
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
                h8_t af[MT];
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    af[mt] = araw[mt];
                }
                if (ks < 3) read_a(ks + 1);
                if (ks == 3) make_cn(par ^ 1);
                load_b2(par, kt + 2, ks);  // this step's words were decoded during the previous step
                __builtin_amdgcn_sched_barrier(0);  // keep the loads above the MFMAs that hide them
                // words of the next step (step 0 of the next tile when ks == 3)
                const uint32_t next0 = (ks < 3) ? word_of(par, ks + 1, 0) : word_of(par ^ 1, 0, 0);
                const uint32_t next1 = (ks < 3) ? word_of(par, ks + 1, 1) : word_of(par ^ 1, 0, 1);
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) acc[mt][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[mt], bf[0], acc[mt][0], 0, 0, 0);
                bf[0] = decode_word_natural(next0, cn[0]);
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) acc[mt][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[mt], bf[1], acc[mt][1], 0, 0, 0);
                bf[1] = decode_word_natural(next1, cn[1]);
                // The decode of the next step's words (32 VALU instructions) spread between this step's MFMAs, three
                // after each of the wide tile's eight (six after each of the narrow tile's four), instead of four MFMAs
                // back to back and the decode behind them: 1 - 4 % (LLaMA-7B down_proj at 2048 rows 184 -> 177 us,
                // o_proj 76.8 -> 74.5, gate/up 353 -> 347; narrow tile: 13B o_proj at 640 rows 57.4 -> 53.8 with six,
                // 30B o_proj at 512 rows 70.5 -> 65.8).
#pragma unroll
                for (int i = 0; i < 2 * MT; ++i) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x002, MT == 4 ? 3 : 6, 0);
                }
            }
        };
        // the first two blocks of the rotary tables: older than every load the waits below count, so landed
        // long before the epilogue
        if (need_tab) {
            dma_table(0, 0);
            dma_table(1, 1);
        }
        // pairs of tiles without a branch between them (a join there would make the compiler
        // move packed words that are still in flight, and wait for them), then the odd one
        GM_STAMP(1);
#ifdef GPTQ4_PHASE_TIMERS
        if (threadIdx.x == 0 && p.counters != nullptr)
            reinterpret_cast<unsigned long long *>(reinterpret_cast<char *>(p.counters) + (32 << 20))[(blockIdx.y * gridDim.x + blockIdx.x) * 8 + 5] = __builtin_readcyclecounter();
#endif
        int kt = k_begin;
        for (; kt + 1 < nk; kt += 2) {
            k_tile(As0, As1, kt, 0);
            k_tile(As1, As0, kt + 1, 1);
        }
        if (kt < nk) k_tile(As0, As1, kt, 0);
        // all LDS-direct loads have landed and every wave is done reading before the
        // epilogues reuse the buffers
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    }

    GM_STAMP(2);
#ifdef GPTQ4_PHASE_TIMERS
    if (threadIdx.x == 0 && p.counters != nullptr)
        reinterpret_cast<unsigned long long *>(reinterpret_cast<char *>(p.counters) + (32 << 20))[(blockIdx.y * gridDim.x + blockIdx.x) * 8 + 6] = __builtin_readcyclecounter();
#endif
    if (nsplit > 1) {
        // Split-K for problems with too few tiles to fill the chip (or a tile cut by the streamed schedule): every
        // sharer publishes its fp32 accumulators (agent-scope atomics, no cache maintenance - see the small-M
        // kernel), the last one to arrive sums them in K order and runs the epilogue.
        constexpr int NREG = MT * 32;
        const int tile = logical;
        float *const mine = p.partials + part_slot(idx) * (NREG * NT) + tid;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int i = 0; i < 16; ++i)
                    __hip_atomic_store(mine + ((mt * 2 + t) * 16 + i) * NT, acc[mt][t][i], __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (tid == 0) {
            const int old = __hip_atomic_fetch_add(&p.counters[tile * COUNTER_STRIDE], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            s_is_last = (old == nsplit - 1);
        }
        __syncthreads();
        if (!s_is_last) return;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int i = 0; i < 16; ++i) acc[mt][t][i] = 0.f;
        for (int sp = 0; sp < nsplit; ++sp) {
            const float *const theirs = p.partials + part_slot(sp) * (NREG * NT) + tid;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    // 16 loads in flight, then 16 adds (added as they are loaded, each would
                    // wait for its own round trip)
                    float got[16];
#pragma unroll
                    for (int i = 0; i < 16; ++i)
                        got[i] = __hip_atomic_load(theirs + ((mt * 2 + t) * 16 + i) * NT, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
                    for (int i = 0; i < 16; ++i) acc[mt][t][i] += got[i];
                }
        }
        if (tid == 0) __hip_atomic_store(&p.counters[tile * COUNTER_STRIDE], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }

    // ---- epilogue.  acc[mt][t][i]: row = 32*mt + 8*(i/4) + 4*lhi + i%4 of the wave,
    //      column = 2*l32 + t of the wave.
    const int wrow0 = m0 + wm * (32 * MT);
    // exchange buffer: [wave][t*16 + i][lane], reusing the activation tiles
    if (EPI == EPI_PLAIN) {
        h2_t bias2 = {(half_t)0.f, (half_t)0.f};
        if (p.bias != nullptr) bias2 = as_h2(*reinterpret_cast<const uint32_t *>(p.bias + ncol));
        if (PERM) __syncthreads();  // (the plain K loop ends with a barrier; here the last tile may still be read)
        uint32_t *const tr = reinterpret_cast<uint32_t *>(region(wave));
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            uint32_t w[16];
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                h2_t o = {(half_t)acc[mt][0][i], (half_t)acc[mt][1][i]};
                if (p.bias != nullptr) o = o + bias2;
                w[i] = as_u32(o);
            }
            store_block_rows<16>(tr, w, lane, [&](int, int rr) -> half_t * {
                const int row = wrow0 + mt * 32 + rr;
                return row < M ? p.y + (size_t)row * N + nw0 : nullptr;
            });
        }
    } else if (EPI == EPI_SILU_MUL) {
        // The gate wave (even) and the up wave (odd) of a pair hold the same output tile.
        // They split it by row blocks: in round r the up wave hands over block r and the
        // gate wave block MT/2 + r, then each finishes the block it received a half of.
        const int pair = (WM == 2) ? wm : wn_pair;
        float *const to_gate = region(2 * pair), *const to_up = region(2 * pair + 1);
#pragma unroll
        for (int r = 0; r < MT / 2; ++r) {
            const int mt = wn_odd ? MT / 2 + r : r;  // the block this wave finishes
            __syncthreads();
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    if (wn_odd)
                        to_gate[(t * 16 + i) * 64 + lane] = acc[r][t][i];
                    else
                        to_up[(t * 16 + i) * 64 + lane] = acc[MT / 2 + r][t][i];
                }
            __syncthreads();
            uint32_t w[16];
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                float o0, o1;
                if (wn_odd) {
                    o0 = silu_f32(to_up[(0 * 16 + i) * 64 + lane]) * acc[MT / 2 + r][0][i];
                    o1 = silu_f32(to_up[(1 * 16 + i) * 64 + lane]) * acc[MT / 2 + r][1][i];
                } else {
                    o0 = silu_f32(acc[r][0][i]) * to_gate[(0 * 16 + i) * 64 + lane];
                    o1 = silu_f32(acc[r][1][i]) * to_gate[(1 * 16 + i) * 64 + lane];
                }
                const h2_t o = {(half_t)o0, (half_t)o1};
                w[i] = as_u32(o);
            }
            // turned through the region this wave has just read (the partner writes there again behind the next barrier)
            store_block_rows<16>(reinterpret_cast<uint32_t *>(wn_odd ? to_up : to_gate), w, lane, [&](int, int rr) -> half_t * {
                const int row = wrow0 + mt * 32 + rr;
                return row < M ? p.y + (size_t)row * N + nw0 : nullptr;
            });
        }
    } else {
        // the workgroup's 128 columns are one head of q, k or v; this wave holds d in
        // [64*wn, 64*wn + 64), the partner d +- 64 is the same lane and register of the
        // other N wave
        const RopeArgs &r = p.rope;
        const int head_col = (n0 >> 7) + wn_pair;
        const int which = head_col / r.H;
        const int head = head_col - which * r.H;
        float *const mine = region(wave);
        const float *const theirs = region(WM == 2 ? (wave ^ 2) : (wave ^ 1));
        // destination of this wave's head: q [B,H,S,128], k and v [B,H,kv_capacity,128]
        const int cap = (which == 0) ? r.S : r.kv_capacity;
        half_t *const dst = ((which == 0) ? r.q : (which == 1) ? r.k : r.v) + (size_t)head * cap * 128 + 64 * wn_odd;  // the wave's 64 values of cache row 0
        const size_t seq_stride = (size_t)r.H * cap * 128;
        const bool at_position = (which != 0) && r.kv_offset < 0;  // cache row = the token's position
        const int row_shift = (which == 0 || r.kv_offset < 0) ? 0 : r.kv_offset;
        // The rotated values of all row blocks are kept in registers and stored at the end, 16 bytes per lane
        // (store_block_rows): behind the last wait for table values - loads and stores share one counter, so a wait
        // for a block's table loads would wait for the stores of the blocks before it as well (LLaMA-7B QKV at 1024
        // rows 118.6 -> 113.5 us, at 2048 rows 204.9 -> 198.2) - and behind a barrier, since the LDS they are turned
        // through is the region the partner wave read this wave's sums from.
        uint32_t outw[MT][16];
        int crow_at[MT][16];  // (cache rows, when they are the tokens' positions)
        auto store_all = [&]() {
            __syncthreads();
            uint32_t *const tr = reinterpret_cast<uint32_t *>(mine);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
                store_block_rows<16>(tr, outw[mt], lane, [&](int j, int rr) -> half_t * {
                    const int row = wrow0 + mt * 32 + rr;
                    if (row >= M) return nullptr;
                    int bb, srow;
                    split_row(r, row, bb, srow);
                    // the lane that stores row 8*j + 4*lhi + q holds that row's cache row itself, in word 4*j + q
                    int crow = srow + row_shift;
                    if (at_position) {
                        const int q = (lane >> 3) & 3;
                        crow = q == 0 ? crow_at[mt][4 * j] : q == 1 ? crow_at[mt][4 * j + 1] : q == 2 ? crow_at[mt][4 * j + 2] : crow_at[mt][4 * j + 3];
                    }
                    return dst + (size_t)bb * seq_stride + (size_t)crow * 128;
                });
        };
        if constexpr (ROPE_TAB) {
            if (PERM) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // table blocks 0 and 1 (the plain path has waited already)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                if (need_tab) {
                    // the block of this step was asked for a step ago: wait for this wave's share of it before
                    // the barrier, and before asking for the next one
                    if (mt >= 2) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                    __syncthreads();  // the step before is finished: its exchange regions and table buffer are free
                    if (mt >= 1 && mt + 1 < MT) dma_table(mt + 1, (mt + 1) & 1);
                    if (which < 2) {
#pragma unroll
                        for (int t = 0; t < 2; ++t)
#pragma unroll
                            for (int i = 0; i < 16; ++i) mine[(t * 16 + i) * 64 + lane] = acc[mt][t][i];
                    }
                    __syncthreads();
                }
                int pos[16];
                if (at_position) {
#pragma unroll
                    for (int i = 0; i < 16; ++i) {
                        const int row = min(wrow0 + mt * 32 + 8 * (i >> 2) + 4 * lhi + (i & 3), M - 1);
                        pos[i] = max(r.position_ids[row], 0);
                    }
                }
                const float *const tcos = rope_tab + (mt & 1) * (2 * 32 * 64) + (4 * lhi) * 64 + 2 * l32;
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    float o0 = acc[mt][0][i], o1 = acc[mt][1][i];
                    if (which < 2) {
                        const float2 cs = *reinterpret_cast<const float2 *>(tcos + (8 * (i >> 2) + (i & 3)) * 64);
                        const float2 sn = *reinterpret_cast<const float2 *>(tcos + 32 * 64 + (8 * (i >> 2) + (i & 3)) * 64);
                        const float p0 = theirs[(0 * 16 + i) * 64 + lane], p1 = theirs[(1 * 16 + i) * 64 + lane];
                        if (wn_odd == 0) {
                            o0 = o0 * cs.x - p0 * sn.x;
                            o1 = o1 * cs.y - p1 * sn.y;
                        } else {
                            o0 = o0 * cs.x + p0 * sn.x;
                            o1 = o1 * cs.y + p1 * sn.y;
                        }
                    }
                    const h2_t o = {(half_t)o0, (half_t)o1};
                    outw[mt][i] = as_u32(o);
                    if (at_position) crow_at[mt][i] = min(pos[i], r.kv_capacity - 1);
                }
            }
            store_all();
            return;
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            if (which < 2) {
                __syncthreads();
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int i = 0; i < 16; ++i) mine[(t * 16 + i) * 64 + lane] = acc[mt][t][i];
                __syncthreads();
            }
            // positions and table rows of the 16 rows this lane holds: all loads are
            // unconditional (rows beyond M read row M-1) and issued together, so their
            // latencies overlap instead of forming 16 dependent chains
            float2 cs[16], sn[16];
            int pos[16];
            if (which < 2 || at_position) {
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int row = min(wrow0 + mt * 32 + 8 * (i >> 2) + 4 * lhi + (i & 3), M - 1);
                    pos[i] = max(r.position_ids[row], 0);
                }
            }
            if (which < 2) {
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int tp = min(pos[i], r.max_pos - 1);
                    cs[i] = *reinterpret_cast<const float2 *>(r.cos_table + (size_t)tp * 64 + 2 * l32);
                    sn[i] = *reinterpret_cast<const float2 *>(r.sin_table + (size_t)tp * 64 + 2 * l32);
                }
            }
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                float o0 = acc[mt][0][i], o1 = acc[mt][1][i];
                if (which < 2) {
                    const float p0 = theirs[(0 * 16 + i) * 64 + lane], p1 = theirs[(1 * 16 + i) * 64 + lane];
                    if (wn_odd == 0) {
                        o0 = o0 * cs[i].x - p0 * sn[i].x;
                        o1 = o1 * cs[i].y - p1 * sn[i].y;
                    } else {
                        o0 = o0 * cs[i].x + p0 * sn[i].x;
                        o1 = o1 * cs[i].y + p1 * sn[i].y;
                    }
                }
                const h2_t o = {(half_t)o0, (half_t)o1};
                outw[mt][i] = as_u32(o);
                if (at_position) crow_at[mt][i] = min(pos[i], r.kv_capacity - 1);
            }
        }
        store_all();
    }
#ifdef GPTQ4_PHASE_TIMERS
    GM_STAMP(3);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    GM_STAMP(4);
#endif
    };  // run_part

    if constexpr (!STREAM) {
        if (p.tail_split > 1) {
            // Tiles [0, tail_first) whole, one workgroup each; every tile from tail_first on - the last column
            // panels, all their row tiles, so that a row is summed in the same order wherever it sits in the
            // batch - cut into tail_split parts along K with a workgroup each.  The parts come last in the grid:
            // they are dispatched onto CUs that are working on a whole tile already and run beside it, so the few
            // tiles past a whole number of rounds cost a fraction of a round instead of one.
            const int full = p.tail_first;
            if ((int)blockIdx.x < full) {
                const int per = full >> 3, rem = full & 7;
                const int xcd = blockIdx.x & 7;
                const int logical = xcd * per + (xcd < rem ? xcd : rem) + (blockIdx.x >> 3);
                run_part(logical, 0, K / BK, 1, 0, [&](int c) { return (size_t)c; });
            } else {
                const int s = p.tail_split;
                const int w = blockIdx.x - full;
                const int t = w / s, idx = w - t * s;
                const int nkt = K / BK, q = nkt / s, r = nkt % s;
                const int kb = idx * q + min(idx, r);
                run_part(full + t, kb, kb + q + (idx < r ? 1 : 0), s, idx, [&](int c) { return (size_t)t * s + c; });
            }
            return;
        }
        // one tile (or one K split of it) per workgroup; K tiles of the split by host-side quotient / remainder
        const int total = gridDim.x;
        const int per = total >> 3, rem = total & 7;
        const int xcd = blockIdx.x & 7;
        const int logical = xcd * per + (xcd < rem ? xcd : rem) + (blockIdx.x >> 3);
        const int split = blockIdx.y;
        const int k_begin = split * p.slot_q + min(split, p.slot_rem);
        const int nk = k_begin + p.slot_q + (split < p.slot_rem ? 1 : 0);
        const int nsplit = p.splitk;
        run_part(logical, k_begin, nk, nsplit, split, [&](int c) { return (size_t)logical * nsplit + c; });
    } else {
        // Range of this workgroup in the sequence of all K tiles.  g: its rank with the workgroups of one XCD
        // (blockIdx.x % 8) adjacent, so that an XCD works on one stretch of the tile order, as it does unstreamed.
        const int S = gridDim.x;  // a multiple of 8
        const int nkt = K / BK;
        const long U = (long)p.tiles * nkt;
        const int g = (blockIdx.x & 7) * (S >> 3) + (blockIdx.x >> 3);
        auto start_of = [&](int w) { return (int)((long)w * U / S); };
        const int u1 = start_of(g + 1);
        for (int u = start_of(g); u < u1;) {
            const int tile = u / nkt;
            const int kb = u - tile * nkt;
            const int ke = min(nkt, kb + (u1 - u));
            // the sharers of this tile: workgroups whose ranges meet [tile * nkt, (tile + 1) * nkt)
            const long x0 = (long)tile * nkt, x1 = x0 + nkt;
            const int g_first = (int)(((x0 + 1) * S + U - 1) / U) - 1;  // the last workgroup that starts at or before x0
            const int g_last = (int)((x1 * S + U - 1) / U) - 1;         // the last one that starts before x1
            // a sharer keeps the part with which its range begins in slot 0 and the one with which it ends in
            // slot 1: only the first sharer of a tile can hold the tile at the end of its range
            const bool first_ends_here = start_of(g_first) < (int)x0;
            run_part(tile, kb, ke, g_last - g_first + 1, g - g_first,
                     [&](int c) { return (size_t)(g_first + c) * 2 + ((c == 0 && first_ends_here) ? 1 : 0); });
            u += ke - kb;
            // the epilogue's exchange regions (and table buffers) are the next part's activation tiles
            asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
            __syncthreads();
        }
    }
}

template <int EPI, int MT>
int launch_one(const MatmulArgs &a, int tiles, hipStream_t stream) {
    dim3 grid((unsigned)tiles, (unsigned)a.splitk), block(256);
    const bool perm = a.perm != nullptr;
    // the wide rotary tile stages its cos / sin rows in 32 KiB of LDS on top of the activation tiles: more than
    // the 64 KiB a launch may ask for unless the kernel is marked for it (once per variant)
    const size_t lds = (EPI == EPI_ROPE && MT == 4) ? 2 * 2 * 32 * 64 * sizeof(float) : 0;
    if (a.stream_b && perm) return (int)hipErrorInvalidValue;  // (the entry points gather beforehand)
    const int variant = a.stream_b ? 2 : (perm ? 1 : 0);
    if (lds) {
        static bool allowed[3] = {false, false, false};
        if (!allowed[variant]) {
            const void *fn = variant == 2   ? reinterpret_cast<const void *>(&gptq4_gemm_kernel<EPI, MT, false, false, true>)
                             : variant == 1 ? reinterpret_cast<const void *>(&gptq4_gemm_kernel<EPI, MT, true>)
                                            : reinterpret_cast<const void *>(&gptq4_gemm_kernel<EPI, MT, false>);
            const hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return (int)e;
            allowed[variant] = true;
        }
    }
    if (variant == 2)
        hipLaunchKernelGGL((gptq4_gemm_kernel<EPI, MT, false, false, true>), grid, block, lds, stream, a);
    else if (variant == 0)
        hipLaunchKernelGGL((gptq4_gemm_kernel<EPI, MT, false>), grid, block, lds, stream, a);
    else
        hipLaunchKernelGGL((gptq4_gemm_kernel<EPI, MT, true>), grid, block, lds, stream, a);
    return (int)hipGetLastError();
}

// The streamed schedule: wide tiles only, a grid of exactly the workgroups that are resident at one time.
template <int EPI>
int launch_streamed(const MatmulArgs &a, int workgroups, hipStream_t stream) {
    dim3 grid((unsigned)workgroups), block(256);
    const size_t lds = (EPI == EPI_ROPE) ? 2 * 2 * 32 * 64 * sizeof(float) : 0;
    if (a.perm != nullptr) return (int)hipErrorInvalidValue;
    if (lds) {
        static bool allowed = false;
        if (!allowed) {
            const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&gptq4_gemm_kernel<EPI, 4, false, true>),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return (int)e;
            allowed = true;
        }
    }
    hipLaunchKernelGGL((gptq4_gemm_kernel<EPI, 4, false, true>), grid, block, lds, stream, a);
    return (int)hipGetLastError();
}

template <int EPI>
int launch_epi(const MatmulArgs &a, const GemmPlan &pl, hipStream_t stream) {
    if (pl.streamed) return launch_streamed<EPI>(a, pl.streamed, stream);
    if (pl.tail_split > 1) return launch_one<EPI, 4>(a, pl.tail_first + (pl.tiles - pl.tail_first) * pl.tail_split, stream);
    return pl.mt == 4 ? launch_one<EPI, 4>(a, pl.tiles, stream) : launch_one<EPI, 2>(a, pl.tiles, stream);
}

}  // namespace

GemmTuning g_gemm_tuning = {0, 0, 0, 0, 0, 0};

// Tile shape and split-K factor of the tiled kernel.  The wide tile (128 x 256, half as
// wide for SiLU*mul) is the faster one as soon as there are enough of them to give three
// CUs out of four a workgroup; from half the CUs on it still wins with K split in two.
// Below that, 128 x 128 tiles, with K split when even those leave most CUs idle (the
// M = 17..255 range on narrow layers).
// How evenly `w` workgroups of equal work fill the device's CUs (256 on MI355X) that hold two of them each: up to
// one per CU every workgroup has a CU to itself, beyond that they run in rounds of two per CU.  What this captures is the
// cliff just above a multiple of the CU count (a few CUs run one workgroup more than the rest and
// set the pace).
static double fill_efficiency(long w) {
    const long cus = device_shape().cus;
    if (w <= cus) return (double)w / (double)cus;
    return (double)w / ((double)(2 * cus) * (double)((w + 2 * cus - 1) / (2 * cus)));
}

GemmPlan gemm_plan(int epi, int M, int N, int K, bool has_perm, bool allow_streamed) {
    GemmPlan pl;
    pl.score = 1.0;
    pl.streamed = 0;
    pl.tail_first = 0;
    pl.tail_split = 1;
    const int bn2 = (epi == EPI_SILU_MUL) ? 64 : 128;  // tile width at MT = 2; twice that at MT = 4
    const int nk = K / 64;
    const long wide = (long)((M + 127) / 128) * (N / (2 * bn2));
    int s = 1;
    bool scored = false;
    const long cus = device_shape().cus;  // the thresholds below are 512, 96 and 384 workgroups on MI355X's 256 CUs
    if (g_gemm_tuning.mt) {
        pl.mt = g_gemm_tuning.mt;
    } else if (wide >= 2 * cus) {
        pl.mt = 4;
    } else if (wide >= 3 * cus / 8 && nk >= 32) {
        // Few enough tiles for their count to matter: score (tile, split) candidates by how evenly they fill
        // the chip, the narrow tile at 0.85 of the wide one's rate, every extra split at 5 % + 20 / (K tiles)
        // of the time (the exchange of partial sums weighs more on a short K).  Fitted to LLaMA-7B / 13B /
        // 30B shapes at 896..2048 rows; e.g. 13824 x 5120: 337 -> 297 us at 2048 rows and 193 -> 163 at 1024,
        // 17920 x 6656 at 1536 rows: 435 -> 367 (three splits each); 4096 x 4096 at 1024 rows: 59 -> 50 us
        // (256 narrow tiles, no split).
        const double pen = 0.05 + 20.0 / (double)nk;
        double best = -1.0;
        for (int mt = 4; mt >= 2; mt -= 2) {
            const long tiles = (mt == 4) ? wide : 2 * wide;
            for (int c = 1; c <= 4 && c <= nk / 8; ++c) {
                const double score = fill_efficiency(tiles * c) * (mt == 4 ? 1.0 : 0.85) / (1.0 + pen * (c - 1));
                if (score > best + 1e-9) {
                    best = score;
                    pl.mt = mt;
                    pl.score = score;
                    s = c;
                }
            }
        }
        scored = true;
    } else {
        pl.mt = 2;
    }
    pl.tiles = ((M + 127) / 128) * (N / (pl.mt == 4 ? 2 * bn2 : bn2));
    if (g_gemm_tuning.splitk > 0) {
        s = g_gemm_tuning.splitk;
    } else if (pl.mt == 2 && pl.tiles < 3 * cus / 2 && !scored) {
        s = (int)((2 * cus + pl.tiles / 2) / pl.tiles);  // aim for ~2 workgroups per CU
        if (s > nk / 8) s = nk / 8;            // keep at least 8 K tiles (512 k) per split
    }
    if (s > GEMM_MAX_SPLITK) s = GEMM_MAX_SPLITK;
    if (s > nk) s = nk;
    if (s < 1 || pl.tiles > SKINNY_MAX_TILES) s = 1;
    pl.splitk = s;
    // Wide unsplit tiles past a whole number of rounds (one tile per CU and round): up to half a round of them is cut
    // along K, each into as many parts as spread the left-over tiles over the chip, and the parts run beside the whole
    // tiles of the last round instead of after them.
    if (pl.mt == 4 && s == 1 && g_gemm_tuning.tail != 1 && g_gemm_tuning.mt == 0 && g_gemm_tuning.splitk == 0 && wide > cus &&
        wide <= SKINNY_MAX_TILES) {
        const long rest = wide % cus;
        // (after an even number of rounds every CU holds its two workgroups and the parts have to wait for a free
        // place: a small remainder is then better off as a launch of its own, see tiled_parts)
        const bool own_launch = ((wide - rest) / cus) % 2 == 0 && 8 * rest <= cus && K >= 2048 && g_gemm_tuning.parts != 1;
        // whole column panels are cut: at least `rest` tiles
        const long tiles_m = (M + 127) / 128, tiles_n = wide / tiles_m;
        const long panels = (rest + tiles_m - 1) / tiles_m, cut = panels * tiles_m;
        if (rest > 0 && 2 * cut <= cus && panels < tiles_n && !own_launch) {
            long parts = cus / cut;
            if (parts > nk / 8) parts = nk / 8;  // at least 8 K tiles (512 k) per part
            if (parts > GEMM_MAX_SPLITK) parts = GEMM_MAX_SPLITK;
            if (parts >= 2) {
                pl.tail_first = (int)(wide - cut);
                pl.tail_split = (int)parts;
            }
        }
    }
    // The streamed schedule (wide tiles; the K tiles of all of them dealt evenly to the 2 x CUs workgroups that are
    // resident at one time) is never chosen automatically: it evens out the work - 344 tiles on 512 slots, or 768 (a
    // pair and then a single one per CU) - but every workgroup then exchanges a 128 KiB tile of fp32 partial sums,
    // 128 MB per launch, at the moment all of them finish, and that costs more than the idle slots did.  Measured at
    // LLaMA-7B / 13B / 30B shapes, 512 .. 4096 rows: 0 - 25 % slower (7B gate/up at 512 rows 122 -> 133 us, QKV at
    // 2048 rows 216 -> 240), ahead only where K is long and the tile count large (30B down_proj at 4096 rows
    // 970 -> 942 us).  gptq4_set_gemm_tuning(200, 0) runs it wherever it can run.
    const long slots = 2 * cus;
    const bool can_stream = !has_perm && allow_streamed && g_gemm_tuning.streamed == 2 && g_gemm_tuning.mt == 0 && g_gemm_tuning.splitk == 0 &&
                            wide >= 1 && wide <= SKINNY_MAX_TILES;
    if (can_stream) {
        // every workgroup of the grid needs at least one K tile (the sharers of a tile are counted from the
        // ranges), and the grid is a multiple of 8 (the XCDs)
        const long grid = (wide * nk < slots ? wide * nk : slots) & ~7L;
        if (grid >= 8) {
            pl.mt = 4;
            pl.tiles = (int)wide;
            pl.splitk = 1;
            pl.streamed = (int)grid;
            pl.tail_split = 1;
        }
    }
    return pl;
}

size_t gemm_partial_bytes(const GemmPlan &pl) {
    // streamed: two slots of a whole wide tile per workgroup (the part that begins its range, the part that ends it)
    if (pl.streamed) return (size_t)pl.streamed * 2 * (4 * 32 * 256) * sizeof(float);
    if (pl.tail_split > 1) return (size_t)(pl.tiles - pl.tail_first) * pl.tail_split * (4 * 32 * 256) * sizeof(float);
    return pl.splitk > 1 ? (size_t)pl.tiles * pl.splitk * (pl.mt * 32 * 256) * sizeof(float) : 0;
}

int launch_gemm(int epi, const MatmulArgs &a, const GemmPlan &pl, hipStream_t stream) {
    switch (epi) {
        case EPI_PLAIN: return launch_epi<EPI_PLAIN>(a, pl, stream);
        case EPI_SILU_MUL: return launch_epi<EPI_SILU_MUL>(a, pl, stream);
        default: return launch_epi<EPI_ROPE>(a, pl, stream);
    }
}
