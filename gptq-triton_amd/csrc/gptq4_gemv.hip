// Decode GEMV (1..4 rows) for gfx950 with wave-granular, evenly dealt work.
//
// Why another decomposition: one CU pulls ~24 GB/s from HBM and decodes at a fixed VALU
// rate, so a decode GEMV is as fast as its most loaded CU.  Column tiles rarely divide
// by 256 CUs (a LLaMA-7B gate/up pair has 344 of them), so here the unit of work is not
// a tile but a (tile, 128-k batch) pair, and the U = tiles * K/128 units are dealt as one
// flat, contiguous range per WAVE: wave v of the grid owns units [v*q + min(v,r), ...),
// q = U / waves, r = U % waves.  The grid is sized to fill every SIMD of the chip exactly
// once (the host also requests enough LDS per workgroup that no CU takes more than its
// share), so every SIMD decodes the same number of units +-1.
//
// A wave's range lies in one tile or crosses into the next one.  There is no
// workgroup-level cooperation at all (no barrier, no LDS reduction):
//   * the wave stages the x values of its own units into its private slice of LDS, in
//     the k order the decoded weights come out in ("pair order"; gathered through `perm`
//     for act-order checkpoints), and reads its matrix-core A operand from there;
//   * per unit: 4 K steps of v_mfma_f32_16x16x32_f16 on weights decoded in registers to
//     the exact fp16 values of the dequantisation kernel;
//   * at the end of a tile segment the wave publishes its partial sums
//     [rows][tile columns] in its slot of the workspace (slot = its rank among the waves
//     that touch the tile) as 8-byte {fp32 bits, 1} pairs with agent-scope stores, and goes
//     on: no wait for their completion, no counter.  The wave that owns the tile's last unit
//     finishes the tile: it polls the slots until every pair carries its 1 (a pair is one
//     store, so value and mark arrive together), sums them in rank order (deterministic),
//     runs the epilogue (bias / SiLU*mul / rotary + head-major q,k,v store) and writes the
//     slots back to zero for the next call.  The region of the workspace that holds the
//     slots is zero whenever no call is running; nothing else is ever written there.
//     A finisher only waits for waves of lower rank, which sit in workgroups dispatched no
//     later than its own and never wait themselves unless they finish a lower tile - so the
//     waits end even when the grid does not fit the chip at once.  They are bounded all the
//     same: a wave that gives up sets the error word of the workspace and moves on.
// The loop is free of branches around loads: loads past the end of the range are
// redirected to the first bytes of the matrix (one cache line) and never used, so the
// compiler's wait counters stay exact and DEPTH units are really in flight.
#include "../../include/gptq4.h"
#include "gptq4_internal.h"
#include "gptq4_norm.h"

#ifdef GPTQ4_PHASE_TIMERS
#define WSTAMP(i)                                                                                          \
    do {                                                                                                   \
        if (lane == 0)                                                                                     \
            reinterpret_cast<unsigned long long *>(reinterpret_cast<char *>(p.counters) + (32 << 20))[v * 8 + (i)] = wall_clock64(); \
    } while (0)
#else
#define WSTAMP(i)
#endif

namespace {

typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

// n / d through the host-made reciprocal (floor(2^32 / d) + 1); exact while n * d < 2^32.
__device__ __forceinline__ int div_magic(int n, int d, uint32_t magic) {
    return d == 1 ? n : (int)__umulhi((unsigned)n, magic);
}

// Raw buffer descriptor over `bytes` bytes at p.  Loads go through it so that an address
// is a 32-bit lane offset plus a 32-bit scalar offset (no 64-bit vector arithmetic), and
// so that a lane offset of 0x80000000 or more - out of range - returns zeros without
// touching memory: that is how loads past the end of a wave's range are switched off.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *p, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, (int)bytes, 0x00020000);
}
constexpr uint32_t OFF_RANGE = 0x80000000u;

struct UnitRegs {
    u32x2_t w[2][4];    // packed weights: [strip][K step], 2 adjacent columns per lane
    uint32_t raw_s[2];  // the 2 fp16 scales of the lane's columns
    uint32_t raw_z[2];  // the zero-point word holding the lane's columns
};

constexpr int XROW = 17;  // 16-byte chunks per (unit, row) of the x slice: 16 + 1 pad

// NORM (2 or 4 chunks of 8 values per thread cover a row; 0 = off): p.x is the residual stream; the
// workgroup first writes weight * rmsnorm(x (+ delta)) of all rows to LDS (gptq4_norm.h; workgroup 0
// also writes the sums out) and its waves stage their x slices from there instead of from memory.
template <int EPI, int DEPTH, bool PERM, int NW, int NORM>
__global__ __launch_bounds__(64 * NW) void gptq4_gemv_kernel(MatmulArgs p) {
    static_assert(!NORM || NW == 4, "the fused norm is written for 256 threads");
    __shared__ float norm_part[NORM ? NORM_MAX_M * 4 : 1];
    constexpr int NV = (EPI == EPI_PLAIN) ? 1 : 2;
    constexpr int W = 2;
    constexpr int SW = 32;
    constexpr int TILE_COLS = SW * NV;
    constexpr int LOG_TC = (NV == 1) ? 5 : 6;

    extern __shared__ uint4 smem[];

    GPTQ4_FETCH_MATMUL_ARGS(p);
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lrow = lane >> 4;
    const int lcol = lane & 15;

    const int M = p.M, K = p.K, N = p.N;
    const int NB = p.nb;
    const int q = p.slot_q, r = p.slot_rem;
    const int v = blockIdx.x * NW + wave;  // this wave's rank in the grid
    const int u0 = v * q + min(v, r);      // first unit
    const int n = q + (v < r ? 1 : 0);     // units of this wave
    if (n == 0 && !NORM) return;           // (waves never wait for each other; with NORM they share the row first)
    WSTAMP(0);
    const int t0 = div_magic(u0, NB, p.nb_magic);
    const int bs = u0 - t0 * NB;  // first batch inside tile t0

    // unit i of this wave -> (tile, batch)
    auto batch_of = [&](int i) { return bs + i - (bs + i >= NB ? NB : 0); };
    auto col0_of = [&](int tile) { return (EPI == EPI_ROPE) ? (tile >> 1) * 128 + (tile & 1) * SW : tile * SW; };

    // ---- x of this wave's units -> private LDS slice [(unit * Mp + row) * XROW + chunk];
    //      chunk c = lane + 64 * u of the slice is (unit, row, 16-byte piece j)
    const int mshift = p.m_shift;
    uint4 *xw = smem + wave * p.lds_wave_chunks;
    const __amdgpu_buffer_rsrc_t rs_x = make_rsrc(p.x, (uint32_t)M * K * 2);
    auto x_chunk = [&](int c, int &dst, uint32_t &off) -> bool {
        const int j = c & 15;
        const int t = c >> 4;
        const int rr = t & ((1 << mshift) - 1);
        const int i = t >> mshift;
        const bool ok = (i < n) && (rr < M);
        dst = t * XROW + j;
        off = ok ? (uint32_t)(rr * K + batch_of(i) * 128 + 8 * j) * 2u : OFF_RANGE;
        return ok;
    };
    uint4 *const xs = smem + NW * p.lds_wave_chunks;  // NORM: [M][K / 8] normalised activations, behind the slices
    NormLoads<NORM ? NORM : 1> nl;
    if (NORM) {
        if (p.nrm_delta != nullptr)
            norm_issue_row0<true>(p.x, p.nrm_delta, p.nrm_weight, K, (int)threadIdx.x, nl);
        else
            norm_issue_row0<false>(p.x, p.x, p.nrm_weight, K, (int)threadIdx.x, nl);
    }
    u32x4_t xv0, xv1;
    if (!PERM && !NORM) {
        int dst;
        uint32_t off;
        x_chunk(lane, dst, off);
        xv0 = __builtin_amdgcn_raw_buffer_load_b128(rs_x, off, 0, 0);
        x_chunk(lane + 64, dst, off);
        xv1 = __builtin_amdgcn_raw_buffer_load_b128(rs_x, off, 0, 0);
    }

    // ---- weights
    const uint32_t wbytes = (uint32_t)(K >> 3) * N * 4u;
    const int G = p.groups;
    const __amdgpu_buffer_rsrc_t rs_w0 = make_rsrc(p.w[0].qweight, wbytes);
    const __amdgpu_buffer_rsrc_t rs_s0 = make_rsrc(p.w[0].scales, (uint32_t)G * N * 2u);
    const __amdgpu_buffer_rsrc_t rs_z0 = make_rsrc(p.w[0].qzeros, (uint32_t)G * (N >> 3) * 4u);
    const int m1 = (EPI == EPI_SILU_MUL) ? 1 : 0;
    const __amdgpu_buffer_rsrc_t rs_w1 = make_rsrc(p.w[m1].qweight, wbytes);
    const __amdgpu_buffer_rsrc_t rs_s1 = make_rsrc(p.w[m1].scales, (uint32_t)G * N * 2u);
    const __amdgpu_buffer_rsrc_t rs_z1 = make_rsrc(p.w[m1].qzeros, (uint32_t)G * (N >> 3) * 4u);
    constexpr int STRIP1 = (EPI == EPI_ROPE) ? 64 : 0;  // column distance of the second strip
    const uint32_t voff_w = ((uint32_t)lrow * N + W * lcol) * 4u;
    const uint32_t voff_s = (uint32_t)(W * lcol) * 2u;
    const uint32_t voff_z = (uint32_t)((W * lcol) >> 3) * 4u;
    const uint32_t kstep = 16u * N;  // bytes between K steps (4 qweight rows)
    const bool one_per_group = p.batches_per_group == 1;

    auto load_unit = [&](UnitRegs &U, int i) {
        const uint32_t dead = (i < n) ? 0u : OFF_RANGE;
        const int ic = min(i, n - 1);
        const int wrap = (bs + ic >= NB) ? 1 : 0;
        const int col0 = col0_of(t0 + wrap);
        const int b = bs + ic - (wrap ? NB : 0);
        const uint32_t vw = voff_w | dead, vs = voff_s | dead, vz = voff_z | dead;
        const uint32_t sw = ((uint32_t)(b * 16) * N + col0) * 4u;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            U.w[0][k] = __builtin_amdgcn_raw_buffer_load_b64(rs_w0, vw, sw + k * kstep, 0);
            if (NV == 2) U.w[1][k] = __builtin_amdgcn_raw_buffer_load_b64(rs_w1, vw + STRIP1 * 4, sw + k * kstep, 0);
        }
        const int g = one_per_group ? b : (int)__umulhi((unsigned)b, p.group_magic);
        const uint32_t ss = ((uint32_t)g * N + col0) * 2u;
        const uint32_t sz = ((uint32_t)g * (N >> 3) + (col0 >> 3)) * 4u;
        U.raw_s[0] = __builtin_amdgcn_raw_buffer_load_b32(rs_s0, vs, ss, 0);
        U.raw_z[0] = __builtin_amdgcn_raw_buffer_load_b32(rs_z0, vz, sz, 0);
        if (NV == 2) {
            U.raw_s[1] = __builtin_amdgcn_raw_buffer_load_b32(rs_s1, vs + STRIP1 * 2, ss, 0);
            U.raw_z[1] = __builtin_amdgcn_raw_buffer_load_b32(rs_z1, vz + (STRIP1 >> 3) * 4, sz, 0);
        }
    };

    UnitRegs ring[DEPTH];
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) load_unit(ring[d], d);
    WSTAMP(1);

    if (NORM) {
        half_t *const sums = (blockIdx.x == 0) ? p.nrm_sum_out : nullptr;
        if (p.nrm_delta != nullptr)
            norm_rows_to_lds<true>(p.x, p.nrm_delta, p.nrm_weight, sums, xs, norm_part, M, K, p.nrm_eps, (int)threadIdx.x, nl);
        else
            norm_rows_to_lds<false>(p.x, p.x, p.nrm_weight, nullptr, xs, norm_part, M, K, p.nrm_eps, (int)threadIdx.x, nl);
        if (n == 0) return;
        for (int c = lane; c < p.x_chunks_max; c += 64) {
            int dst;
            uint32_t off;
            if (x_chunk(c, dst, off)) {
                if (!PERM) {
                    xw[dst] = pair_order_u4(xs[off >> 4]);
                } else {
                    // act-order: x_sorted[k] = x[perm[k]], gathered from the row in LDS, directly in pair order
                    const int rowk = (int)(off >> 1);
                    const int row = (c >> 4) & ((1 << mshift) - 1);
                    const int k = rowk - row * K;
                    const uint16_t *xh = reinterpret_cast<const uint16_t *>(xs) + (size_t)row * K;
                    const int4 i0 = *reinterpret_cast<const int4 *>(p.perm + k);
                    const int4 i1 = *reinterpret_cast<const int4 *>(p.perm + k + 4);
                    uint4 val;
                    val.x = (uint32_t)xh[i0.x] | ((uint32_t)xh[i1.x] << 16);
                    val.y = (uint32_t)xh[i0.y] | ((uint32_t)xh[i1.y] << 16);
                    val.z = (uint32_t)xh[i0.z] | ((uint32_t)xh[i1.z] << 16);
                    val.w = (uint32_t)xh[i0.w] | ((uint32_t)xh[i1.w] << 16);
                    xw[dst] = val;
                }
            }
        }
    } else
    // ---- finish the x slice (its first loads were issued before the weights, so they
    //      arrive first)
    if (!PERM) {
        int dst;
        uint32_t off;
        if (x_chunk(lane, dst, off)) xw[dst] = pair_order_u4(__builtin_bit_cast(uint4, xv0));
        if (x_chunk(lane + 64, dst, off)) xw[dst] = pair_order_u4(__builtin_bit_cast(uint4, xv1));
        for (int c = lane + 128; c < p.x_chunks_max; c += 64) {
            const bool ok = x_chunk(c, dst, off);
            const u32x4_t val = __builtin_amdgcn_raw_buffer_load_b128(rs_x, off, 0, 0);
            if (ok) xw[dst] = pair_order_u4(__builtin_bit_cast(uint4, val));
        }
    } else {
        // act-order: x_sorted[k] = x[perm[k]]
        for (int c = lane; c < p.x_chunks_max; c += 64) {
            int dst;
            uint32_t off;
            if (x_chunk(c, dst, off)) {
                const int rowk = (int)(off >> 1);  // row * K + k
                const int row = (c >> 4) & ((1 << mshift) - 1);
                const int k = rowk - row * K;
                const uint16_t *xs = reinterpret_cast<const uint16_t *>(p.x + (size_t)row * K);
                const int4 i0 = *reinterpret_cast<const int4 *>(p.perm + k);
                const int4 i1 = *reinterpret_cast<const int4 *>(p.perm + k + 4);
                uint4 val;  // directly in pair order: (0,4) (1,5) (2,6) (3,7)
                val.x = (uint32_t)xs[i0.x] | ((uint32_t)xs[i1.x] << 16);
                val.y = (uint32_t)xs[i0.y] | ((uint32_t)xs[i1.y] << 16);
                val.z = (uint32_t)xs[i0.z] | ((uint32_t)xs[i1.z] << 16);
                val.w = (uint32_t)xs[i0.w] | ((uint32_t)xs[i1.w] << 16);
                xw[dst] = val;
            }
        }
    }
    WSTAMP(2);
#ifdef GPTQ4_PHASE_TIMERS
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    WSTAMP(3);
#endif

    f4_t acc[NV][W];
#pragma unroll
    for (int vv = 0; vv < NV; ++vv)
#pragma unroll
        for (int t = 0; t < W; ++t) acc[vv][t] = (f4_t){0.f, 0.f, 0.f, 0.f};

    // A operand of lane (lrow, lcol): row lcol (rows >= M alias row M-1, their outputs are
    // never stored), chunk 4*kstep + lrow of the unit
    const uint4 *xa = xw + min(lcol, M - 1) * XROW + lrow;
    const int xunit = XROW << mshift;

    auto compute_unit = [&](const UnitRegs &U, int i) {
        const uint4 *ap = xa + i * xunit;
        h8_t a[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) a[k] = __builtin_bit_cast(h8_t, ap[4 * k]);
        ColDecode cd[NV][W];
#pragma unroll
        for (int vv = 0; vv < NV; ++vv) {
            const uint32_t zs = U.raw_z[vv] >> (((W * lcol) & 7) * 4);
#pragma unroll
            for (int t = 0; t < W; ++t) cd[vv][t] = make_col_decode((zs >> (4 * t)) & 0xFu, U.raw_s[vv] >> (16 * t));
        }
#pragma unroll
        for (int k = 0; k < 4; ++k)
#pragma unroll
            for (int vv = 0; vv < NV; ++vv)
#pragma unroll
                for (int t = 0; t < W; ++t)
                    acc[vv][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[k], decode_word_h8(t == 0 ? U.w[vv][k].x : U.w[vv][k].y, cd[vv][t]), acc[vv][t], 0, 0, 0);
    };

    // waves owning q+1 units come first: the owner of unit u
    auto wave_of_unit = [&](int u) {
        const int big = r * (q + 1);
        return u < big ? div_magic(u, q + 1, p.q1_magic) : r + div_magic(u - big, q, p.q_magic);
    };
    // partial sums of one tile segment -> this wave's slot (its rank among the waves that
    // touch the tile; the owner of the tile's first unit has rank 0).  Rows 0..3 of the
    // accumulators live in lanes 0..15.
    const size_t tile_elems = (size_t)M * TILE_COLS;
    constexpr uint64_t MARK = 1ull << 32;
    auto publish = [&](int tile) {
        const int rank = v - wave_of_unit(tile * NB);
        uint64_t *mine = p.tagged + ((size_t)tile * p.max_contrib + rank) * tile_elems;
        if (lane < 16) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if (e < M) {
#pragma unroll
                    for (int vv = 0; vv < NV; ++vv)
#pragma unroll
                        for (int t = 0; t < W; ++t)
                            __hip_atomic_store(&mine[(size_t)e * TILE_COLS + vv * SW + W * lcol + t],
                                               MARK | (uint64_t)__float_as_uint(acc[vv][t][e]), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
        }
    };

    const int first_len = min(n, NB - bs);  // units of this wave in tile t0
    for (int i = 0; i < n; i += DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            if (i + d < n) {
                if (i + d == first_len) {  // the range crosses into tile t0 + 1 here
                    publish(t0);
#pragma unroll
                    for (int vv = 0; vv < NV; ++vv)
#pragma unroll
                        for (int t = 0; t < W; ++t) acc[vv][t] = (f4_t){0.f, 0.f, 0.f, 0.f};
                }
                compute_unit(ring[d], i + d);
            }
            load_unit(ring[d], i + d + DEPTH);
        }
    }
    WSTAMP(4);
    const bool crossed = n > first_len;
    publish(crossed ? t0 + 1 : t0);
    WSTAMP(5);

    // ---- the owner of a tile's last unit finishes it: that can only be tile t0 (a range is at most one tile long)
    if (bs + n < NB) return;
    {
        const int tile = t0;
        const int w_first = wave_of_unit(tile * NB);
        const int ncontrib = v - w_first + 1;
        uint64_t *const all = p.tagged + (size_t)tile * p.max_contrib * tile_elems;
        const int col0 = col0_of(tile);
        const int total = M << LOG_TC;
        // lane <-> element (row, tile column); with two strips the partner (same row and
        // column of the other strip) sits 32 lanes away
#pragma unroll 1
        for (int e0 = 0; e0 < total; e0 += 64) {
            const int e = e0 + lane;
            const bool live = e < total;
            uint64_t *const src = all + (live ? e : 0);
            float s = 0.f;
            // every load is issued (contributors past the last one re-read the last slot),
            // so one round trip covers 16 slots
#pragma unroll 1
            for (int c0 = 0; c0 < ncontrib; c0 += 16) {
                uint64_t part[16];
                uint32_t tries = p.spin_limit;
                for (;;) {
#pragma unroll
                    for (int k = 0; k < 16; ++k)
                        part[k] = __hip_atomic_load(src + (size_t)min(c0 + k, ncontrib - 1) * tile_elems, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    uint64_t got = MARK;
#pragma unroll
                    for (int k = 0; k < 16; ++k) got &= part[k];
                    // (a limit of 0xFFFFFFFF is the test hook: give up even though everything has arrived)
                    if (p.spin_limit != 0xFFFFFFFFu && __builtin_amdgcn_ballot_w64(live && got == 0) == 0) break;
                    if (p.spin_limit == 0xFFFFFFFFu || --tries == 0) {
                        // gave up: the call's result is not valid; the word stays set for the host to find
                        if (lane == 0) __hip_atomic_store(&p.counters[EXCHANGE_ERROR_WORD], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        break;
                    }
                    __builtin_amdgcn_s_sleep(1);
                }
#pragma unroll
                for (int k = 0; k < 16; ++k) s += (c0 + k < ncontrib) ? __uint_as_float((uint32_t)part[k]) : 0.f;
                // back to zero for the next call
                if (live) {
#pragma unroll
                    for (int k = 0; k < 16; ++k)
                        if (c0 + k < ncontrib)
                            __hip_atomic_store(src + (size_t)(c0 + k) * tile_elems, (uint64_t)0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
            const int row = e >> LOG_TC;
            const int c = e & (SW - 1);
            if (EPI == EPI_PLAIN) {
                if (live) {
                    const int nn = col0 + c;
                    half_t o = (half_t)s;
                    if (p.bias != nullptr) o = o + p.bias[nn];
                    p.y[(size_t)row * N + nn] = o;
                }
            } else {
                const float other = __shfl_xor(s, 32);  // strip 1 for lanes < 32
                const bool mine = live && ((e & SW) == 0);
                if (EPI == EPI_SILU_MUL) {
                    if (mine) p.y[(size_t)row * N + col0 + c] = (half_t)(silu_f32(s) * other);
                } else if (mine) {
                    const RopeArgs &ra = p.rope;
                    const int head_col = col0 >> 7;
                    const int dd = (col0 & 127) + c;
                    const int which = head_col / ra.H;
                    const int head = head_col - which * ra.H;
                    const int bb = row / ra.S;
                    const int ss = row - bb * ra.S;
                    float o1 = s, o2 = other;
                    if (which < 2) {
                        const int pos = min(max(ra.position_ids[row], 0), ra.max_pos - 1);
                        const float cs = ra.cos_table[(size_t)pos * 64 + dd];
                        const float sn = ra.sin_table[(size_t)pos * 64 + dd];
                        o1 = s * cs - other * sn;
                        o2 = other * cs + s * sn;
                    }
                    half_t *dst;
                    size_t off;
                    if (which == 0) {
                        dst = ra.q;
                        off = ((size_t)(bb * ra.H + head) * ra.S + ss) * 128;
                    } else {
                        dst = (which == 1) ? ra.k : ra.v;
                        // kv_offset < 0: the cache row is the token's position
                        const int crow = ra.kv_offset >= 0 ? ra.kv_offset + ss : min(max(ra.position_ids[row], 0), ra.kv_capacity - 1);
                        off = ((size_t)(bb * ra.H + head) * ra.kv_capacity + crow) * 128;
                    }
                    dst[off + dd] = (half_t)o1;
                    dst[off + 64 + dd] = (half_t)o2;
                }
            }
        }
        WSTAMP(7);
    }
}

template <int EPI, int DEPTH, int NW>
int launch_variant(const MatmulArgs &a, const GemvPlan &pl, hipStream_t stream) {
    dim3 grid((unsigned)pl.workgroups), block(64 * NW);
    if (a.perm == nullptr)
        hipLaunchKernelGGL((gptq4_gemv_kernel<EPI, DEPTH, false, NW, 0>), grid, block, pl.lds_bytes, stream, a);
    else
        hipLaunchKernelGGL((gptq4_gemv_kernel<EPI, DEPTH, true, NW, 0>), grid, block, pl.lds_bytes, stream, a);
    return (int)hipGetLastError();
}

// The variant that normalises its own input: 4 waves, one unit in flight.
template <int EPI>
int launch_norm_variant(const MatmulArgs &a, const GemvPlan &pl, hipStream_t stream) {
    dim3 grid((unsigned)pl.workgroups), block(256);
    const bool perm = a.perm != nullptr;
    if (a.K <= 4096 && !perm)
        hipLaunchKernelGGL((gptq4_gemv_kernel<EPI, 1, false, 4, 2>), grid, block, pl.lds_bytes, stream, a);
    else if (a.K <= 4096)
        hipLaunchKernelGGL((gptq4_gemv_kernel<EPI, 1, true, 4, 2>), grid, block, pl.lds_bytes, stream, a);
    else if (!perm)
        hipLaunchKernelGGL((gptq4_gemv_kernel<EPI, 1, false, 4, 4>), grid, block, pl.lds_bytes, stream, a);
    else
        hipLaunchKernelGGL((gptq4_gemv_kernel<EPI, 1, true, 4, 4>), grid, block, pl.lds_bytes, stream, a);
    return (int)hipGetLastError();
}

template <int EPI>
int launch_epi(const MatmulArgs &a, const GemvPlan &pl, hipStream_t stream) {
    if (a.nrm_weight != nullptr) {
        if (EPI == EPI_PLAIN) return (int)hipErrorInvalidValue;  // no entry point asks a plain projection for it
        return launch_norm_variant<(EPI == EPI_PLAIN) ? EPI_SILU_MUL : EPI>(a, pl, stream);
    }
    const int key = pl.waves * 10 + pl.depth;
    switch (key) {
        case 41: return launch_variant<EPI, 1, 4>(a, pl, stream);
        case 81: return launch_variant<EPI, 1, 8>(a, pl, stream);
        case 42: return launch_variant<EPI, 2, 4>(a, pl, stream);
        case 43: return launch_variant<EPI, 3, 4>(a, pl, stream);
        case 82: return launch_variant<EPI, 2, 8>(a, pl, stream);
        case 83: return launch_variant<EPI, 3, 8>(a, pl, stream);
        case 162: return launch_variant<EPI, 2, 16>(a, pl, stream);
        default: return launch_variant<EPI, 1, 4>(a, pl, stream);
    }
}

uint32_t magic_of(int d) { return d > 1 ? (uint32_t)(0x100000000ull / (unsigned)d + 1) : 0u; }

}  // namespace

GemvTuning g_gemv_tuning = {1, 0, 0, 0, 0};

// Launch shape: the grid holds `waves_per_cu` waves per CU on all CUs of the device (or fewer
// waves when there are fewer units than that), each wave owning q or q+1 units.
GemvPlan gemv_plan(int epi, int M, int N, int K, bool norm) {
    GemvPlan pl = {};
    // one unit in flight per wave: with 8 waves per CU a deeper ring only queues requests the CU cannot
    // have outstanding anyway (measured 15.2 us against 15.9 at two units for the LLaMA-7B gate/up pair).
    // The variant that normalises its own input exists for the automatic shape only.
    pl.depth = (!norm && g_gemv_tuning.depth > 0) ? g_gemv_tuning.depth : 1;
    pl.waves = (!norm && g_gemv_tuning.waves > 0) ? g_gemv_tuning.waves : 4;
    const int waves_per_cu = (!norm && g_gemv_tuning.waves_per_cu > 0) ? g_gemv_tuning.waves_per_cu : 8;
    const int sw = 32;
    pl.tiles = (epi == EPI_ROPE) ? (N / 128) * (64 / sw) : N / sw;
    pl.nb = K / 128;
    const long units = (long)pl.tiles * pl.nb;
    long total_waves = (long)device_shape().cus * waves_per_cu;
    if (total_waves > units) total_waves = units;
    pl.workgroups = (int)((total_waves + pl.waves - 1) / pl.waves);
    total_waves = (long)pl.workgroups * pl.waves;
    pl.q = (int)(units / total_waves);
    pl.r = (int)(units % total_waves);
    // measured on MI355X at LLaMA-7B / 13B / 30B shapes, one row: ahead of the split-K kernel for the gate/up
    // pair (15.0 against 17.6 us, 20.3 / 23.8, 32.2 / 32.4) and, from 13B on, for QKV with the rotary epilogue
    // (7B 12.1 against 11.1 us, 13B 14.5 / 15.8, 30B 20.2 / 23.4: the crossover is put at 8192 units); within
    // 3 % either way for o_proj, behind for down_proj (7B 12.6 against 10.8 us) and everywhere from 2 rows on
    const bool wanted = g_gemv_tuning.mode == 2 ||
                        (g_gemv_tuning.mode == 1 && M == 1 && (epi == EPI_SILU_MUL || (epi == EPI_ROPE && units >= 8192)));
    pl.ok = wanted && M >= 1 && M <= GEMV_MAX_M && pl.tiles <= SKINNY_MAX_TILES && pl.q + 1 <= pl.nb &&
            units < (1L << 24) && (long)K * N < (1L << 32) && (long)M * K < (1L << 30);
    int mshift = 0;
    while ((1 << mshift) < M) ++mshift;
    pl.m_shift = mshift;
    const int max_units = pl.q + (pl.r ? 1 : 0);
    pl.lds_wave_chunks = (max_units << mshift) * XROW;
    size_t lds = (size_t)pl.waves * pl.lds_wave_chunks * 16;
    if (norm) lds += (size_t)M * K * sizeof(half_t);  // the normalised rows, shared by the workgroup
    // no CU may take more than its share of workgroups: ask for so much LDS (160 KiB per
    // CU) that one more workgroup would not fit
    const int wgs_per_cu = (waves_per_cu + pl.waves - 1) / pl.waves;
    size_t want = (size_t)(160 * 1024) / (size_t)wgs_per_cu;
    if (want > 65536) want = 65536;
    want &= ~(size_t)1023;
    if (lds > 65536) pl.ok = false;
    if (lds < want) lds = want;
    pl.lds_bytes = lds;
    // waves touching one tile: its NB units are owned by consecutive waves of >= q units
    // (fewer units than waves: every unit has a wave of its own, a tile as many contributors as batches)
    pl.max_contrib = (pl.q > 0) ? (pl.nb + pl.q - 1) / pl.q + 1 : pl.nb;
    if (pl.max_contrib > pl.nb) pl.max_contrib = pl.nb;
    if (gemv_tagged_bytes(pl, M, epi) > GPTQ4_WS_TAGGED_BYTES) pl.ok = false;
    return pl;
}

size_t gemv_tagged_bytes(const GemvPlan &pl, int M, int epi) {
    const int tile_cols = 32 * (epi == EPI_PLAIN ? 1 : 2);
    return (size_t)pl.tiles * pl.max_contrib * M * tile_cols * sizeof(uint64_t);
}

int launch_gemv(int epi, MatmulArgs &a, const GemvPlan &pl, hipStream_t stream) {
    a.tiles = pl.tiles;
    a.nb = pl.nb;
    a.slot_q = pl.q;
    a.slot_rem = pl.r;
    a.m_shift = pl.m_shift;
    a.lds_wave_chunks = pl.lds_wave_chunks;
    a.x_chunks_max = (pl.q + 1) << (4 + pl.m_shift);
    a.max_contrib = pl.max_contrib;
    a.spin_limit = g_gemv_tuning.spin_limit ? g_gemv_tuning.spin_limit : (1u << 22);
    a.batches_per_group = a.groupsize / 128;
    a.groups = a.K / a.groupsize;
    a.group_magic = magic_of(a.batches_per_group);
    a.nb_magic = magic_of(pl.nb);
    a.q_magic = magic_of(pl.q);
    a.q1_magic = magic_of(pl.q + 1);
    switch (epi) {
        case EPI_PLAIN: return launch_epi<EPI_PLAIN>(a, pl, stream);
        case EPI_SILU_MUL: return launch_epi<EPI_SILU_MUL>(a, pl, stream);
        default: return launch_epi<EPI_ROPE>(a, pl, stream);
    }
}
