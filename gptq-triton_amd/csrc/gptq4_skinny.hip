// Small-M (1..16 rows) dequant-fused matmul for gfx950: the decode GEMV / skinny GEMM.
//
// Memory-bound by design: the packed weights are streamed from HBM exactly once,
// decoded in registers and fed to v_mfma_f32_16x16x32_f16 (the 16-row matrix-core tile
// holds all of x even at M = 16; at M = 1 the unused rows cost nothing because the
// matrix pipe is otherwise idle - the decode is the VALU work either way).
//
// Work decomposition
//   K step = 32 values of k = 4 qweight rows.  Lane l of a wave reads row l/16 and
//            W adjacent columns W*(l%16) .. +W-1 (W = 1, 2 or 4 words = 4/8/16-byte
//            loads).  Word t of the lane is the complete B operand of MFMA t, whose
//            16 columns are {W*j + t}: no transposition between the checkpoint layout
//            and the matrix-core register layout.
//   strip  = 16*W output columns.
//   batch  = 128 values of k (4 K steps): the unit of K distribution; a quantisation
//            group is a whole number of batches.
//   tile   = what one workgroup owns: 1 strip (plain), the same strip of the gate and
//            of the up matrix (SiLU*mul), or a strip of head columns d and the strip
//            d + 64 of the same head (rotary: partners meet in one workgroup).
//   The 4 waves of a workgroup take disjoint contiguous batch ranges, keep DEPTH
//   batches of loads in flight, and are summed through LDS.  With splitk > 1, that many
//   workgroups share a tile; each publishes its partial sums and the one that arrives
//   last (arrival counter) adds them in fixed order and runs the epilogue, so results
//   are deterministic.
//   blockIdx -> (tile, split): all splits of a tile, and tiles that share a 128-byte
//   line of a qweight row, land on one XCD (blockIdx % 8) and hence one L2.
#include "gptq4_internal.h"
#include "gptq4_norm.h"

// Development aid, compiled out of the product build: per-workgroup cycle stamps at
// the phase boundaries of the kernel, written 32 MiB into the workspace (size it so).
#ifdef GPTQ4_PHASE_TIMERS
#define PHASE_STAMP(i)                                                                     \
    do {                                                                                   \
        if (threadIdx.x == 0)                                                              \
            reinterpret_cast<unsigned long long *>(reinterpret_cast<char *>(p.counters) + (32 << 20))[(blockIdx.y * gridDim.x + blockIdx.x) * 8 + (i)] = \
                wall_clock64();                                                            \
    } while (0)
#else
#define PHASE_STAMP(i)
#endif

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
struct Batch {
    typename WordVec<W>::type w[NV][4];  // packed weights: [loaded strip][K step]
    uint4 a[4];                          // activations of row lane%16, natural k order, per K step
    uint2 raw_s[NV];                     // W fp16 scales of the lane's columns (low halves first)
    uint32_t raw_z[NV];
    int group;
    int b;                               // the batch (uniform over the wave)
};

// NORM: p.x is the residual stream; the workgroup first computes weight * rmsnorm(x (+ delta)) of
// all M rows into LDS (gptq4_norm.h; the workgroup of tile 0, split 0 also writes the sums out)
// and takes its A operand from there instead of from memory.
// NORM = chunks of 8 values per thread that cover a row (2: K <= 4096, 4: K <= 8192), 0 = off.
// PERM (with NORM only): act-order - the rows in LDS are then put into the order of the sorted weight
// rows, xs[j] <- xs[perm[j]].  Without NORM the caller passes activations that are gathered already.
template <int EPI, int W, int DEPTH, bool PERM, int NW, int NORM>
__global__ __launch_bounds__(64 * NW) void gptq4_skinny_kernel(MatmulArgs p) {
    static_assert(!NORM || NW == 4, "the fused norm is written for 256 threads");
    static_assert(!PERM || NORM, "act-order inside the kernel needs the rows in LDS");
    constexpr int NV = (EPI == EPI_PLAIN) ? 1 : 2;  // strips loaded per K step
    constexpr int SW = 16 * W;                      // strip width in columns
    constexpr int TILE_COLS = SW * NV;              // columns of the LDS tile
    constexpr int Q = SW / 16;                      // output elements per thread and row block
    constexpr int LINE_TILES = (SW >= 32) ? 1 : 32 / SW;  // tiles sharing a 128-byte row segment

    __shared__ float red[NW][SKINNY_MAX_M][TILE_COLS];
    __shared__ int s_is_last;
    __shared__ float norm_part[NORM ? NORM_MAX_M * 4 : 1];
    extern __shared__ uint4 xs[];  // NORM: [M][K / 8] normalised activations

    GPTQ4_FETCH_MATMUL_ARGS(p);
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    // the wave index is uniform: keep it (and everything derived from it - batch range,
    // group index, row base addresses) in scalar registers
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lrow = lane >> 4;  // k-block inside a K step; also output row group
    const int lcol = lane & 15;

    // grid: x = 8 * (tiles per XCD, rounded up), y = split.  grid.x is a multiple of 8,
    // so blockIdx.x % 8 is the XCD for every y.  No runtime divisions here: the host
    // precomputes how the K batches are dealt to the splitk * 4 wave slots.
    const int xcd = blockIdx.x & 7;
    const int j = blockIdx.x >> 3;
    const int split = blockIdx.y;
    const int sub = j % LINE_TILES;
    const int tile = ((j / LINE_TILES) * 8 + xcd) * LINE_TILES + sub;
    if (tile >= p.tiles) return;

    PHASE_STAMP(0);
    const int M = p.M, K = p.K, N = p.N;
    const int slot = split * NW + wave;
    const int b0 = slot * p.slot_q + min(slot, p.slot_rem);
    const int b1 = b0 + p.slot_q + (slot < p.slot_rem ? 1 : 0);
    const int bpg = p.batches_per_group;

    // first column of the tile's strip(s)
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
        qw[v] = p.w[m].qweight + ncol[v];
        qz[v] = p.w[m].qzeros;
        sc[v] = p.w[m].scales;
    }

    // Lanes of rows >= M read row M-1 instead of branching: A row m only feeds output row
    // m, and output rows >= M are never stored.
    const half_t *xrow = p.x + (size_t)(lcol < M ? lcol : M - 1) * K;

    f4_t acc[NV][W];
#pragma unroll
    for (int v = 0; v < NV; ++v)
#pragma unroll
        for (int t = 0; t < W; ++t) acc[v][t] = (f4_t){0.f, 0.f, 0.f, 0.f};

    ColDecode cd[NV][W];
    int cur_group = -1;
    // group of the next batch to be loaded (loads are issued in increasing batch order)
    int ld_group = (bpg >= (K >> 7)) ? 0 : b0 / bpg;
    int ld_left = (bpg >= (K >> 7)) ? 0x7fffffff : bpg - (b0 - ld_group * bpg);

    typedef typename WordVec<W>::type wvec_t;
    typedef Batch<NV, W> batch_t;

    auto load_batch = [&](batch_t &B, int b) {
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const uint32_t *base = qw[v] + (size_t)(b * 16 + lrow) * N;
#pragma unroll
            for (int i = 0; i < 4; ++i) B.w[v][i] = *reinterpret_cast<const wvec_t *>(base + (size_t)(4 * i) * N);
        }
        B.b = b;
        if (!NORM) {
            // NORM takes the A operand from LDS at compute time
#pragma unroll
            for (int i = 0; i < 4; ++i) B.a[i] = *reinterpret_cast<const uint4 *>(xrow + b * 128 + 32 * i + 8 * lrow);
        }
        B.group = ld_group;
        if (--ld_left == 0) {
            ld_left = bpg;
            ++ld_group;
        }
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const half_t *sp = sc[v] + (size_t)B.group * N + ncol[v];
            if (W == 1)
                B.raw_s[v] = make_uint2(*reinterpret_cast<const uint16_t *>(sp), 0u);
            else if (W == 2)
                B.raw_s[v] = make_uint2(*reinterpret_cast<const uint32_t *>(sp), 0u);
            else
                B.raw_s[v] = *reinterpret_cast<const uint2 *>(sp);
            B.raw_z[v] = qz[v][(size_t)B.group * (N >> 3) + (ncol[v] >> 3)];
        }
    };

    const int xs_row = (lcol < M ? lcol : M - 1) * (K >> 3);  // NORM: the lane's row of xs
    auto compute_batch = [&](const batch_t &B) {
        if (B.group != cur_group) {
            cur_group = B.group;
#pragma unroll
            for (int v = 0; v < NV; ++v) {
                // the lane's W columns are nibbles (ncol % 8) .. +W-1 of the zero word
                const uint32_t zs = B.raw_z[v] >> (((W * lcol) & 7) * 4);
#pragma unroll
                for (int t = 0; t < W; ++t) {
                    const uint32_t sw = (t >> 1) ? B.raw_s[v].y : B.raw_s[v].x;
                    cd[v][t] = make_col_decode((zs >> (4 * t)) & 0xFu, sw >> (16 * (t & 1)));
                }
            }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint4 av = NORM ? xs[xs_row + B.b * 16 + 4 * i + lrow] : B.a[i];
            const h8_t a = pair_order_a(av);
#pragma unroll
            for (int v = 0; v < NV; ++v) {
#pragma unroll
                for (int t = 0; t < W; ++t) {
                    const h8_t bf = decode_word_h8(word_of(B.w[v][i], t), cd[v][t]);
                    acc[v][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, bf, acc[v][t], 0, 0, 0);
                }
            }
        }
    };

    // software pipeline: DEPTH batches of loads in flight per wave
    {
        // NORM: the loads of the first row go out ahead of the weights, so that the row is
        // normalised while the weights are still on their way
        NormLoads<NORM ? NORM : 1> nl;
        if (NORM) {
            if (p.nrm_delta != nullptr)
                norm_issue_row0<true>(p.x, p.nrm_delta, p.nrm_weight, K, tid, nl);
            else
                norm_issue_row0<false>(p.x, p.x, p.nrm_weight, K, tid, nl);
        }
        batch_t ring[DEPTH];
#pragma unroll
        for (int d = 0; d < DEPTH; ++d)
            if (b0 + d < b1) load_batch(ring[d], b0 + d);
#ifdef GPTQ4_PHASE_TIMERS
        PHASE_STAMP(7);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        PHASE_STAMP(5);
#endif
        if (NORM) {
            half_t *const sums = (tile == 0 && split == 0) ? p.nrm_sum_out : nullptr;
            if (p.nrm_delta != nullptr)
                norm_rows_to_lds<true>(p.x, p.nrm_delta, p.nrm_weight, sums, xs, norm_part, M, K, p.nrm_eps, tid, nl);
            else
                norm_rows_to_lds<false>(p.x, p.x, p.nrm_weight, nullptr, xs, norm_part, M, K, p.nrm_eps, tid, nl);
        }
        if (NORM && PERM) {
            // act-order: put each row into the order of the sorted weight rows, xs[j] <- xs[perm[j]], in
            // place: every thread gathers its chunks into registers, all wait, then the chunks go back.  (The
            // source positions are only asked for here, in registers that the norm has just given up: held
            // from before the weight loads they would cost a wave per SIMD.)
            int4 src[NORM ? NORM : 1][2];
#pragma unroll
            for (int c = 0; c < NORM; ++c) {
                const int chunk = min(tid + 256 * c, (K >> 3) - 1);
                src[c][0] = *reinterpret_cast<const int4 *>(p.perm + 8 * chunk);
                src[c][1] = *reinterpret_cast<const int4 *>(p.perm + 8 * chunk + 4);
            }
            for (int m = 0; m < M; ++m) {
                const uint16_t *xh = reinterpret_cast<const uint16_t *>(xs + m * (K >> 3));
                uint4 g[NORM ? NORM : 1];
#pragma unroll
                for (int c = 0; c < NORM; ++c) {
                    const int4 i0 = src[c][0], i1 = src[c][1];
                    g[c].x = (uint32_t)xh[i0.x] | ((uint32_t)xh[i0.y] << 16);
                    g[c].y = (uint32_t)xh[i0.z] | ((uint32_t)xh[i0.w] << 16);
                    g[c].z = (uint32_t)xh[i1.x] | ((uint32_t)xh[i1.y] << 16);
                    g[c].w = (uint32_t)xh[i1.z] | ((uint32_t)xh[i1.w] << 16);
                }
                __syncthreads();
#pragma unroll
                for (int c = 0; c < NORM; ++c)
                    if (tid + 256 * c < (K >> 3)) xs[m * (K >> 3) + tid + 256 * c] = g[c];
            }
            __syncthreads();
        }
        for (int b = b0; b < b1; b += DEPTH) {
#pragma unroll
            for (int d = 0; d < DEPTH; ++d) {
                if (b + d < b1) {
                    compute_batch(ring[d]);
                    if (b + d + DEPTH < b1) load_batch(ring[d], b + d + DEPTH);
                }
            }
        }
    }

    PHASE_STAMP(1);
    // ---- sum the 4 waves through LDS: lane holds rows 4*lrow+i, columns W*lcol+t
#pragma unroll
    for (int v = 0; v < NV; ++v)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int row = 4 * lrow + i;
            if (row < M) {
#pragma unroll
                for (int t = 0; t < W; ++t) red[wave][row][v * SW + W * lcol + t] = acc[v][t][i];
            }
        }
    __syncthreads();

    // the first 256 threads finish the tile: thread owns elements (row = (256/SW)*q + tid/SW,
    // c = tid%SW), each with NV values
    // (the other waves stay for the barriers below but own no rows)
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
                for (int w = 0; w < NW; ++w) s += red[w][row][v * SW + c];
            }
            val[q][v] = s;
        }
    }

    PHASE_STAMP(2);
    if (p.splitk > 1 && p.tagged != nullptr) {
        // Cross-workgroup exchange through marked values: every partial sum travels as one 8-byte
        // {fp32 bits, 1} store (value and mark arrive together) into a region of the workspace that is zero
        // whenever no call runs.  The workgroups of splits 0 .. splitk-2 store theirs and leave - no wait for
        // the stores' completion, no arrival counter; the workgroup of the last split keeps its own sums in
        // registers, polls the others' slots until every value it needs carries its mark, adds them in split
        // order and writes the slots back to zero.  It waits only for workgroups with a lower blockIdx.y,
        // dispatched before it, which never wait themselves; the wait is bounded all the same.
        constexpr uint64_t MARK = 1ull << 32;
        const size_t tile_elems = (size_t)M * TILE_COLS;
        uint64_t *const slots = p.tagged + (size_t)tile * p.splitk * tile_elems;
        if (split != p.splitk - 1) {
            uint64_t *const mine = slots + (size_t)split * tile_elems;
#pragma unroll
            for (int q = 0; q < Q; ++q) {
                const int row = ROWS_PER_PASS * q + rbase;
                if (row < Mf) {
#pragma unroll
                    for (int v = 0; v < NV; ++v)
                        __hip_atomic_store(&mine[(size_t)row * TILE_COLS + v * SW + c], MARK | (uint64_t)__float_as_uint(val[q][v]),
                                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
            PHASE_STAMP(3);
            return;
        }
        // CH splits per round of polls, every element of the thread at once: 16 loads in flight per thread (more
        // would cost the streaming loop a wave per SIMD in registers), and a round is one round trip however
        // many elements and splits it covers
        const int others = p.splitk - 1;
        constexpr int CH = (Q * NV >= 8) ? 2 : (Q * NV >= 4) ? 4 : 8;
        float sum[Q][NV];
#pragma unroll
        for (int q = 0; q < Q; ++q)
#pragma unroll
            for (int v = 0; v < NV; ++v) sum[q][v] = 0.f;
        uint32_t tries = p.spin_limit;
#pragma unroll 1
        for (int c0 = 0; c0 < others; c0 += CH) {
            uint64_t part[Q][NV][CH];
            for (;;) {
                uint64_t got = MARK;
#pragma unroll
                for (int q = 0; q < Q; ++q) {
                    const int row = ROWS_PER_PASS * q + rbase;
                    const uint64_t *const src = slots + (row < Mf ? (size_t)row * TILE_COLS + c : 0);
#pragma unroll
                    for (int v = 0; v < NV; ++v)
#pragma unroll
                        for (int k = 0; k < CH; ++k)  // (splits past the last one re-read the last slot)
                            part[q][v][k] = __hip_atomic_load(src + v * SW + (size_t)min(c0 + k, others - 1) * tile_elems, __ATOMIC_RELAXED,
                                                              __HIP_MEMORY_SCOPE_AGENT);
                }
#pragma unroll
                for (int q = 0; q < Q; ++q)
#pragma unroll
                    for (int v = 0; v < NV; ++v)
#pragma unroll
                        for (int k = 0; k < CH; ++k) got &= (ROWS_PER_PASS * q + rbase < Mf) ? part[q][v][k] : MARK;
                // (a limit of 0xFFFFFFFF is the test hook: give up even though everything has arrived)
                if (p.spin_limit != 0xFFFFFFFFu && __builtin_amdgcn_ballot_w64(got == 0) == 0) break;
                if (p.spin_limit == 0xFFFFFFFFu || --tries == 0) {
                    // gave up: the call's result is not valid; the word stays set for the host to find
                    if (lane == 0) __hip_atomic_store(&p.counters[EXCHANGE_ERROR_WORD], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    tries = 1;
                    break;
                }
                __builtin_amdgcn_s_sleep(4);
            }
#pragma unroll
            for (int q = 0; q < Q; ++q) {
                const int row = ROWS_PER_PASS * q + rbase;
                if (row < Mf) {
                    uint64_t *const src = slots + (size_t)row * TILE_COLS + c;
#pragma unroll
                    for (int v = 0; v < NV; ++v)
#pragma unroll
                        for (int k = 0; k < CH; ++k)
                            if (c0 + k < others) {
                                // a fixed-order sum: splits 0 .. splitk-2, then this workgroup's own
                                sum[q][v] += __uint_as_float((uint32_t)part[q][v][k]);
                                // back to zero for the next call
                                __hip_atomic_store(src + v * SW + (size_t)(c0 + k) * tile_elems, (uint64_t)0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                            }
                }
            }
        }
#pragma unroll
        for (int q = 0; q < Q; ++q)
#pragma unroll
            for (int v = 0; v < NV; ++v) val[q][v] = sum[q][v] + val[q][v];
        PHASE_STAMP(5);
    } else if (p.splitk > 1) {
        // Cross-workgroup exchange without cache maintenance: partial sums are written
        // and read with agent-scope (sc1) relaxed atomics, which are coherent across the
        // XCDs' L2s by themselves.  A release/acquire fence would add an L2 write-back
        // and invalidate per workgroup, which serialises the whole grid.  Ordering is
        // by completion: every wave waits until its stores are acknowledged
        // (s_waitcnt vmcnt(0)) before the barrier that precedes the arrival count.
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
        PHASE_STAMP(3);
        __syncthreads();
        if (tid == 0) {
            const int old = __hip_atomic_fetch_add(&p.counters[tile * COUNTER_STRIDE], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            s_is_last = (old == p.splitk - 1);
        }
        __syncthreads();
        PHASE_STAMP(4);
        if (!s_is_last) return;
        const float *all = p.partials + (size_t)tile * p.splitk * tile_elems;
#pragma unroll
        for (int q = 0; q < Q; ++q) {
            const int row = ROWS_PER_PASS * q + rbase;
            if (row < Mf) {
#pragma unroll
                for (int v = 0; v < NV; ++v) {
                    // all loads in flight at once, then a fixed-order sum
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
        PHASE_STAMP(5);
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
            int bb, ss;
            split_row(r, row, bb, ss);
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
                // kv_offset < 0: the cache row is the token's position
                const int crow = r.kv_offset >= 0 ? r.kv_offset + ss : min(max(r.position_ids[row], 0), r.kv_capacity - 1);
                off = ((size_t)(bb * r.H + head) * r.kv_capacity + crow) * 128;
            }
            dst[off + d] = (half_t)o1;
            dst[off + 64 + d] = (half_t)o2;
        }
    }
    PHASE_STAMP(6);
}

template <int EPI, int W, int DEPTH, int NW>
int launch_variant(const MatmulArgs &a, hipStream_t stream) {
    constexpr int SW = 16 * W;
    constexpr int LINE_TILES = (SW >= 32) ? 1 : 32 / SW;
    const int per_xcd = 8 * LINE_TILES;
    const int groups = (a.tiles + per_xcd - 1) / per_xcd;
    dim3 grid((unsigned)(groups * per_xcd), (unsigned)a.splitk), block(64 * NW);
    // act-order: the caller hands over the activations already gathered (launch_gather_cols)
    if (a.perm != nullptr) return (int)hipErrorInvalidValue;
    hipLaunchKernelGGL((gptq4_skinny_kernel<EPI, W, DEPTH, false, NW, 0>), grid, block, 0, stream, a);
    return (int)hipGetLastError();
}

// The variant that normalises its own input: the automatic launch shape only.
template <int EPI, int DEPTH>
int launch_norm_variant(const MatmulArgs &a, hipStream_t stream) {
    const int groups = (a.tiles + 7) / 8;
    dim3 grid((unsigned)(groups * 8), (unsigned)a.splitk), block(256);
    const size_t lds = (size_t)a.M * a.K * sizeof(half_t);
    const bool perm = a.perm != nullptr;
    if (a.K <= 4096 && !perm)
        hipLaunchKernelGGL((gptq4_skinny_kernel<EPI, 2, DEPTH, false, 4, 2>), grid, block, lds, stream, a);
    else if (a.K <= 4096)
        hipLaunchKernelGGL((gptq4_skinny_kernel<EPI, 2, DEPTH, true, 4, 2>), grid, block, lds, stream, a);
    else {
        // rows of more than 4096 values: up to 64 KiB of rows on top of the 16 KiB reduction buffer - more than
        // the 64 KiB a launch may ask for unless the kernel is marked for it (once per variant)
        static bool allowed[2] = {false, false};
        if (!allowed[perm]) {
            const void *fn = perm ? reinterpret_cast<const void *>(&gptq4_skinny_kernel<EPI, 2, DEPTH, true, 4, 4>)
                                  : reinterpret_cast<const void *>(&gptq4_skinny_kernel<EPI, 2, DEPTH, false, 4, 4>);
            const hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, NORM_MAX_M * NORM_MAX_H * (int)sizeof(half_t));
            if (e != hipSuccess) return (int)e;
            allowed[perm] = true;
        }
        if (!perm)
            hipLaunchKernelGGL((gptq4_skinny_kernel<EPI, 2, DEPTH, false, 4, 4>), grid, block, lds, stream, a);
        else
            hipLaunchKernelGGL((gptq4_skinny_kernel<EPI, 2, DEPTH, true, 4, 4>), grid, block, lds, stream, a);
    }
    return (int)hipGetLastError();
}

template <int EPI>
int launch_epi(const MatmulArgs &a, const SkinnyPlan &pl, hipStream_t stream) {
    const int key = pl.waves * 100 + pl.words * 10 + pl.depth;
    switch (key) {
        case 412: return launch_variant<EPI, 1, 2, 4>(a, stream);
        case 414: return launch_variant<EPI, 1, 4, 4>(a, stream);
        case 421: return launch_variant<EPI, 2, 1, 4>(a, stream);
        case 422: return launch_variant<EPI, 2, 2, 4>(a, stream);
        case 424: return launch_variant<EPI, 2, 4, 4>(a, stream);
        case 441: return launch_variant<EPI, 4, 1, 4>(a, stream);
        case 442: return launch_variant<EPI, 4, 2, 4>(a, stream);
        default: return (int)hipErrorInvalidValue;  // skinny_plan only makes the pairs above
    }
}

}  // namespace

SkinnyTuning g_skinny_tuning = {0, 0, 0, 0, 0};

// Launch shape for a small-M problem, from sweeps on MI355X at LLaMA-7B / 13B / 30B shapes: split K until
// there are ~1024 workgroups (4 per CU) but keep >= 2 batches per wave.  8-byte loads (32-column strips,
// full 128-byte lines per row) with two batches in flight per wave (one for the gate/up pair: register
// budget) unless 16-byte loads (64-column strips, half the tiles, one batch in flight) still reach ~900
// workgroups: then those are 10-18 % faster (13B / 30B down_proj and gate/up; never at 7B shapes, where the
// split is capped first).  The rotary epilogue keeps 8-byte loads (two strips per head either way).
static int split_for(int tiles, int k_batches, int waves) {
    const int want = 4 * device_shape().cus;  // 1024 workgroups on MI355X
    int s = (want + tiles - 1) / tiles;
    if (s > k_batches / (2 * waves)) s = k_batches / (2 * waves);
    if (s > SKINNY_MAX_SPLITK) s = SKINNY_MAX_SPLITK;
    return s < 1 ? 1 : s;
}

SkinnyPlan skinny_plan(int epi, int M, int N, int K, bool standard_shape) {
    SkinnyPlan pl;
    const bool tuned = !standard_shape;
    const int k_batches = K / 128;
    pl.waves = (tuned && g_skinny_tuning.waves > 0) ? g_skinny_tuning.waves : 4;
    pl.words = 2;
    // Batches of loads in flight per wave: two, but one for the gate/up pair (two matrices' worth of registers) and for
    // plain projections of up to 4 rows - measured at LLaMA-7B / 13B / 30B shapes with the weights coming from HBM:
    // 7B o_proj 6.2 -> 5.9 us and down_proj 9.6 -> 8.6 at one row, 13B down_proj 12.5 -> 11.4, 30B o_proj 9.5 -> 8.6,
    // level elsewhere; from 8 rows on and with the rotary epilogue two are level or ahead.
    pl.depth = (epi == EPI_SILU_MUL || (epi == EPI_PLAIN && M <= 4)) ? 1 : 2;
    if (tuned && epi != EPI_ROPE && (long)(N / 64) * split_for(N / 64, k_batches, pl.waves) >= 900) {
        pl.words = 4;
        pl.depth = 1;
    }
    if (tuned && g_skinny_tuning.words > 0) {
        pl.words = g_skinny_tuning.words;
        pl.depth = (epi == EPI_SILU_MUL || (epi == EPI_PLAIN && M <= 4)) ? 1 : 2;
    }
    if (tuned && g_skinny_tuning.depth > 0) pl.depth = g_skinny_tuning.depth;
    // the instantiated (width, depth) pairs: 4 bytes x {2, 4}, 8 bytes x {1, 2, 4}, 16 bytes x {1, 2}
    if (pl.words == 1) pl.depth = (pl.depth <= 2) ? 2 : 4;
    if (pl.words == 2 && pl.depth == 3) pl.depth = 2;
    if (pl.words == 4 && pl.depth > 2) pl.depth = 2;
    const int sw = 16 * pl.words;
    pl.tiles = (epi == EPI_ROPE) ? (N / 128) * (64 / sw) : N / sw;
    int s;
    if (g_skinny_tuning.splitk > 0) {
        s = g_skinny_tuning.splitk;
        if (s > k_batches / pl.waves) s = k_batches / pl.waves;  // at least one batch per wave
        if (s > SKINNY_MAX_SPLITK) s = SKINNY_MAX_SPLITK;
        if (s < 1) s = 1;
    } else {
        s = split_for(pl.tiles, k_batches, pl.waves);
    }
    pl.splitk = s;
    return pl;
}

int launch_skinny(int epi, const MatmulArgs &a, const SkinnyPlan &pl, hipStream_t stream) {
    if (a.nrm_weight != nullptr) {
        // checked by the caller: automatic plan (8-byte loads, 4 waves), M <= NORM_MAX_M, K <= NORM_MAX_H
        if (epi == EPI_SILU_MUL) return launch_norm_variant<EPI_SILU_MUL, 1>(a, stream);
        if (epi == EPI_ROPE) return launch_norm_variant<EPI_ROPE, 2>(a, stream);
        return (int)hipErrorInvalidValue;  // no entry point asks a plain projection to normalise its input
    }
    switch (epi) {
        case EPI_PLAIN: return launch_epi<EPI_PLAIN>(a, pl, stream);
        case EPI_SILU_MUL: return launch_epi<EPI_SILU_MUL>(a, pl, stream);
        default: return launch_epi<EPI_ROPE>(a, pl, stream);
    }
}
