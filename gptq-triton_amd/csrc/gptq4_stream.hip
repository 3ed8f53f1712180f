// Decode GEMV (1..4 rows; a variant for 5..16 follows it) for gfx950 on weights in streaming order.
//
// What bounds a decode GEMV on this chip is not arithmetic and not the memory's rate but how many bytes a CU can
// have in flight and how long a launch runs with nothing in flight: its start (arguments, addresses, first-load
// latency) and its end (partial sums handed from one workgroup to another, a last pass over them).  This kernel is
// built around those two:
//   * Layout.  Per strip of 16 output columns and unit of 128 input rows the packed words form one contiguous
//     1 KiB block in matrix-core operand order (see SMat): a wave fetches a unit with ONE 16-byte load per lane and
//     one 4-byte load of {scale, zero}; consecutive units of a strip are consecutive in memory.
//   * Work.  A tile is a strip (plain projection), the same strip of gate and up (SiLU*mul) or a strip and the
//     strip of its rotation partners 64 columns on (rotary).  The tiles * K/128 units form one sequence that is cut
//     into equal contiguous ranges, one per workgroup, one workgroup of 8 or 16 waves per CU: every CU streams the
//     same number of bytes, whatever the number of columns.  Inside the workgroup the range is dealt to the waves
//     unit by unit, from its top end down; a wave keeps DEPTH units of loads in flight.
//   * Start.  A wave needs blockIdx, its wave number and a handful of scalars for the address of its first unit;
//     the activations (all M rows: every wave needs all of K) are requested just before, land in LDS - in the k
//     order the decoded weights come out in - while the first weights are on their way, and are the A operand of
//     v_mfma_f32_16x16x32_f16 from there.
//   * End.  The waves leave their sums, per strip, in LDS and the workgroup adds them in wave order and stores its
//     own columns.  Only a strip that the cut between two workgroups runs through needs memory: a range is walked
//     from its top end down, so the part of such a strip that belongs to the LOWER workgroup (the top of its range)
//     is finished within the first few units; the last of its waves to get there adds the waves' sums and publishes
//     them as marked 8-byte values {fp32 bits, 1} in the workgroup's slot of the workspace - one aligned store
//     each, so value and mark arrive together - and streams on.  The UPPER workgroup meets its part of the strip
//     (the bottom of its range) last and finds the other part waiting: nobody waits for a neighbour that has the
//     same amount of work.  A finishing workgroup polls slots of lower-numbered workgroups only, which never wait
//     themselves, so the waits end even if the grid is not resident as a whole; they are bounded anyway (error
//     word of the workspace).  Sums are added in a fixed order: results do not change from run to run.
#include "../../include/gptq4.h"
#include "gptq4_internal.h"
#include "gptq4_norm.h"

#include <mutex>

namespace {

typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ int sdiv_magic(int n, int d, uint32_t magic) { return d == 1 ? n : (int)__umulhi((unsigned)n, magic); }

__device__ __forceinline__ __amdgpu_buffer_rsrc_t srsrc(const void *p, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, (int)bytes, 0x00020000);
}
// a lane offset that is out of range for every buffer here: the load returns zeros and touches no memory
constexpr uint32_t S_OFF_RANGE = 0x80000000u;
constexpr uint64_t S_MARK = 1ull << 32;

// What a wave needs for the address of its first loads, as kernel arguments of their own in front of the struct, and
// buffer sizes that do not wait for K and N: LLaMA-7B QKV + rotary at one row 8.49 -> 8.03 us, down_proj 7.88 -> 7.59
// (having the compiler ask for these arguments in registers at wave start, -amdgpu-kernarg-preload-count, measured
// no further gain: 7.98 / 7.54)
#define STREAM_HOT_PARAMS                                                                                                   \
    const uint32_t *hw0, const uint32_t *hm0, const uint32_t *hw1, const uint32_t *hm1, int hq, int hr, int hnb, uint32_t hnb_magic, \
        int hgroups, int hbpg, uint32_t hgroup_magic
#define STREAM_HOT_ARGS(a) (a).m[0].w, (a).m[0].meta, (a).m[1].w, (a).m[1].meta, (a).q, (a).r, (a).nb, (a).nb_magic, (a).groups, (a).batches_per_group, (a).group_magic

template <int NV>
struct SUnit {
    u32x4_t w[NV];      // the lane's four packed words of the unit, per matrix
    uint32_t meta[NV];  // scale | zero << 16 of the lane's column
};

// EPI: epilogue; NW waves per workgroup; DEPTH units in flight per wave; PERM: x is gathered through p.perm on its
// way into LDS (act-order); NORM (0, or chunks of 8 values per thread of the first four waves that cover a row): x is
// the residual stream and the workgroup multiplies with weight * rmsnorm(x (+ delta)); NOMATH: the same loads, waits
// and stores with the decode and the matrix-core instructions left out (measurement only).
template <int EPI, int NW, int DEPTH, bool PERM, int NORM, bool NOMATH>
__global__ __launch_bounds__(64 * NW) void gptq4_stream_kernel(STREAM_HOT_PARAMS, StreamArgs p) {
    constexpr int NV = (EPI == EPI_PLAIN) ? 1 : 2;
    constexpr int NT = 64 * NW;
    extern __shared__ uint4 smem[];
    __shared__ float norm_part[NORM ? NORM_MAX_M * 4 : 1];
    __shared__ int arrivals;

    // (the compiler fetches kernel arguments where it first needs them, in dependent round trips of 0.2 - 0.3 us each
    // with nothing else in flight: naming them here makes it one)
    asm volatile("" ::"s"(p.x), "s"(p.M), "s"(p.K), "s"(p.N), "s"(p.xrow), "s"(p.red_off), "s"(p.m_magic), "s"(p.tagged));
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r4 = lane >> 4;
    const int c = lane & 15;

    const int M = p.M, K = p.K, N = p.N, nb = hnb, G = hgroups;
    const int wg = blockIdx.x;
    const int a0 = wg * hq + min(wg, hr);      // first unit of this workgroup
    const int L = hq + (wg < hr ? 1 : 0);      // its units
    const int b0 = a0 + L;
    const int tile_hi = sdiv_magic(b0 - 1, nb, hnb_magic);
    const int n = wave < L ? (L - wave + NW - 1) / NW : 0;   // units of this wave: positions wave, wave + NW, ...

    // ---- which output element this thread finishes, if any: e = (piece from the bottom, row, column) belongs to
    //      thread NT - 1 - e.  Its row's position (rotary) is requested here, ahead of everything else.
    const int e_mine = NT - 1 - tid;
    const int e_col = e_mine & 15;
    const int e_t = e_mine >> 4;
    const int e_pb = (e_t * p.m_magic) >> 16;  // e_t / M (m_magic = ceil(2^16 / M), exact for e_t < 2^10)
    const int e_row = e_t - e_pb * M;
    int rope_pos = 0;
    if (EPI == EPI_ROPE) rope_pos = p.rope.position_ids[e_row];

    // ---- activations: requested first (two instructions), so that they arrive first
    const int chunks = K >> 3;  // 16-byte chunks per row
    uint4 *const xs = smem;     // [M][xrow] in pair order
    const __amdgpu_buffer_rsrc_t rs_x = srsrc(p.x, (uint32_t)M * K * 2u);
    constexpr int XPRE = 2;
    u32x4_t xv[XPRE];
    NormLoads<NORM ? NORM : 1> nl;
    if (NORM) {
        if (wave < 4) {
            if (p.nrm_delta != nullptr)
                norm_issue_row0<true>(p.x, p.nrm_delta, p.nrm_weight, K, tid, nl);
            else
                norm_issue_row0<false>(p.x, p.x, p.nrm_weight, K, tid, nl);
        }
    } else if (!PERM) {
#pragma unroll
        for (int u = 0; u < XPRE; ++u) {
            const int ch = tid + u * NT;  // chunk of the [M][chunks] array
            xv[u] = __builtin_amdgcn_raw_buffer_load_b128(rs_x, ch < M * chunks ? (uint32_t)ch * 16u : S_OFF_RANGE, 0, 0);
        }
    }

    // ---- weights: the unit the next load / the next multiplication is for, (tile, 128-k batch), walking down from
    //      the top of the range
    // (both below the plan's limit of 2 GiB and below the offset that switches a load off; exact sizes would wait for K and N)
    constexpr uint32_t wbytes = 0x7FFFFFF0u, mbytes = 0x7FFFFFF0u;
    __amdgpu_buffer_rsrc_t rs_w[NV], rs_m[NV];
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        rs_w[v] = srsrc(v ? hw1 : hw0, wbytes);
        rs_m[v] = srsrc(v ? hm1 : hm0, mbytes);
    }
    const int bpg = hbpg;
    int ld_tile = tile_hi, ld_batch = 0;
    if (n > 0) {
        const int u = b0 - 1 - wave;
        ld_tile = sdiv_magic(u, nb, hnb_magic);
        ld_batch = u - ld_tile * nb;
    }
    int cp_tile = ld_tile, cp_batch = ld_batch;
    auto strip_of = [&](int tile, int v) { return (EPI == EPI_ROPE) ? ((tile >> 2) << 3) + (tile & 3) + 4 * v : tile; };
    auto issue = [&](SUnit<NV> &U, bool live) {
        const uint32_t dead = live ? 0u : S_OFF_RANGE;
        const int g = (bpg == 1) ? ld_batch : (int)__umulhi((unsigned)ld_batch, hgroup_magic);
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const int strip = strip_of(ld_tile, v);
            // (streamed once: the hint keeps the lines from displacing what the caches hold)
            U.w[v] = __builtin_amdgcn_raw_buffer_load_b128(rs_w[v], ((uint32_t)lane * 16u) | dead, (uint32_t)(strip * nb + ld_batch) * 1024u, 2);
            U.meta[v] = __builtin_amdgcn_raw_buffer_load_b32(rs_m[v], ((uint32_t)c * 4u) | dead, (uint32_t)(strip * G + g) * 64u, 0);
        }
        ld_batch -= NW;
        if (ld_batch < 0) {  // (the plan keeps NW <= nb: one strip down at most)
            ld_batch += nb;
            ld_tile -= 1;
        }
    };
    SUnit<NV> ring[DEPTH];
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) issue(ring[d], d < n);

    const int tile_lo = sdiv_magic(a0, nb, hnb_magic);
    const int npieces = tile_hi - tile_lo + 1;
    const int top_len = min(L, b0 - tile_hi * nb);           // units of the top piece
    const bool publishes = (b0 - tile_hi * nb) != nb;        // its strip goes on in the next workgroup
    const bool shared_lo = (a0 - tile_lo * nb) != 0;         // lower workgroups hold the rest of the bottom strip

    // ---- the pieces this workgroup finishes: all but a published top piece (the plan keeps the number of their
    //      elements within NT).  The bottom piece, whose other part comes from memory, falls to lanes of the last
    //      wave, which is never the one with the most units.
    const int fin0 = publishes ? 1 : 0;
    const int total = (npieces - fin0) * M * 16;
    const bool gets_partials = shared_lo && total > 0;
    const bool owner = e_mine < total;
    const int e_tile = tile_lo + e_pb;
    // what its epilogue reads is requested now: the token's position (rotary), the bias
    const int rope_head_col = e_tile >> 2;                  // head among the 3 * H heads of q, k, v
    const int rope_dd = ((e_tile & 3) << 4) + e_col;        // column of the head, < 64; the second sum is column dd + 64
    int rope_which = 0, rope_head = 0;
    float rope_cs = 1.f, rope_sn = 0.f;
    half_t bias_v = (half_t)0.f;
    if (EPI == EPI_ROPE) {
        rope_which = rope_head_col / p.rope.H;
        rope_head = rope_head_col - rope_which * p.rope.H;
    }
    if (EPI == EPI_PLAIN && owner && p.bias != nullptr) bias_v = p.bias[e_tile * 16 + e_col];

    // ---- partial-sum slots of the waves, per piece: zero, so that a piece a wave never enters adds nothing
    f4_t *const red = reinterpret_cast<f4_t *>(smem + p.red_off);  // [piece][wave][NV][16 columns] x 4 rows
    const float *const redf = reinterpret_cast<const float *>(red);
    if (lane < 16) {
        for (int pc = 0; pc < npieces; ++pc)
#pragma unroll
            for (int v = 0; v < NV; ++v) red[((pc * NW + wave) * NV + v) * 16 + c] = (f4_t){0.f, 0.f, 0.f, 0.f};
    }
    if (tid == 0) arrivals = 0;

    // ---- the activations reach LDS
    auto put_x = [&](int ch, uint4 val) {  // chunk ch of [M][chunks], natural order in, pair order out
        const int row = (M == 1) ? 0 : ch / chunks;
        xs[row * p.xrow + (ch - row * chunks)] = pair_order_u4(val);
    };
    auto gather_x = [&](const uint16_t *src, int ch) {  // act-order: x_sorted[k] = x[perm[k]], directly in pair order
        const int row = (M == 1) ? 0 : ch / chunks;
        const int k = (ch - row * chunks) * 8;
        const uint16_t *xh = src + (size_t)row * K;
        const int4 i0 = *reinterpret_cast<const int4 *>(p.perm + k);
        const int4 i1 = *reinterpret_cast<const int4 *>(p.perm + k + 4);
        uint4 val;  // (0,4) (1,5) (2,6) (3,7)
        val.x = (uint32_t)xh[i0.x] | ((uint32_t)xh[i1.x] << 16);
        val.y = (uint32_t)xh[i0.y] | ((uint32_t)xh[i1.y] << 16);
        val.z = (uint32_t)xh[i0.z] | ((uint32_t)xh[i1.z] << 16);
        val.w = (uint32_t)xh[i0.w] | ((uint32_t)xh[i1.w] << 16);
        xs[row * p.xrow + (ch - row * chunks)] = val;
    };
    if (NORM) {
        half_t *const sums = (wg == 0) ? p.nrm_sum_out : nullptr;
        if (!PERM) {
            // the normalised chunks go straight into the k order of the decoded weights
            auto put = [&](int row, int c, uint4 v) { xs[row * p.xrow + c] = pair_order_u4(v); };
            if (p.nrm_delta != nullptr)
                norm_rows_put<true>(p.x, p.nrm_delta, p.nrm_weight, sums, put, norm_part, M, K, p.nrm_eps, tid, nl, wave < 4);
            else
                norm_rows_put<false>(p.x, p.x, p.nrm_weight, nullptr, put, norm_part, M, K, p.nrm_eps, tid, nl, wave < 4);
        } else {
            uint4 *const xn = smem + p.nat_off;  // [M][chunks], natural order: the gather reads single values of it
            if (p.nrm_delta != nullptr)
                norm_rows_to_lds<true>(p.x, p.nrm_delta, p.nrm_weight, sums, xn, norm_part, M, K, p.nrm_eps, tid, nl, wave < 4);
            else
                norm_rows_to_lds<false>(p.x, p.x, p.nrm_weight, nullptr, xn, norm_part, M, K, p.nrm_eps, tid, nl, wave < 4);
            for (int ch = tid; ch < M * chunks; ch += NT) gather_x(reinterpret_cast<const uint16_t *>(xn), ch);
        }
    } else if (!PERM) {
#pragma unroll
        for (int u = 0; u < XPRE; ++u) {
            const int ch = tid + u * NT;
            if (ch < M * chunks) put_x(ch, __builtin_bit_cast(uint4, xv[u]));
        }
        for (int ch = tid + XPRE * NT; ch < M * chunks; ch += NT)
            put_x(ch, __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(rs_x, (uint32_t)ch * 16u, 0, 0)));
    } else {
        for (int ch = tid; ch < M * chunks; ch += NT) gather_x(reinterpret_cast<const uint16_t *>(p.x), ch);
    }
    if (EPI == EPI_ROPE && owner && rope_which < 2) {
        const int pos = min(max(rope_pos, 0), p.rope.max_pos - 1);
        rope_cs = p.rope.cos_table[(size_t)pos * 64 + rope_dd];
        rope_sn = p.rope.sin_table[(size_t)pos * 64 + rope_dd];
    }
    __syncthreads();

    // ---- a wave's sums of a piece -> its slot; the top piece of a range whose strip goes on in the next workgroup
    //      is added up and published by the last wave to leave it
    const int slot_elems = NV * 16 * M;  // marked values a workgroup publishes
    auto arrive_top = [&]() {
        int old = 0;
        if (lane == 0) old = __hip_atomic_fetch_add(&arrivals, 1, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_WORKGROUP);
        old = __builtin_amdgcn_readfirstlane(old);
        if (old != NW - 1) return;
        uint64_t *const mine = p.tagged + (size_t)wg * slot_elems;
        for (int e = lane; e < slot_elems; e += 64) {  // e = (v * M + row) * 16 + column
            const int col = e & 15, t = e >> 4;
            const int v = (t >= M) ? 1 : 0;
            const int row = t - v * M;
            float s = 0.f;
#pragma unroll
            for (int w = 0; w < NW; ++w) s += redf[((w * NV + v) * 16 + col) * 4 + row];
            __hip_atomic_store(&mine[e], S_MARK | (uint64_t)__float_as_uint(s), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    };
    f4_t acc[NV];
#pragma unroll
    for (int v = 0; v < NV; ++v) acc[v] = (f4_t){0.f, 0.f, 0.f, 0.f};
    auto dump = [&](int pc) {
        if (lane < 16) {
#pragma unroll
            for (int v = 0; v < NV; ++v) red[((pc * NW + wave) * NV + v) * 16 + c] = acc[v];
        }
        if (pc == 0 && publishes) arrive_top();
    };
    if (publishes && wave >= top_len) arrive_top();  // no unit of the top piece is this wave's: its slot stays zero

    // A operand of lane (r4, c): row min(c, M - 1) (rows >= M alias row M - 1, their outputs are never stored), the
    // chunks 4 * r4 + j of the unit for the steps j = 0..3
    const uint4 *const xa = xs + min(c, M - 1) * p.xrow + 4 * r4;
    int cur_tile = cp_tile;

    auto compute = [&](const SUnit<NV> &U) {
        if (cp_tile != cur_tile) {  // the range crosses into the next strip down
            dump(tile_hi - cur_tile);
            cur_tile = cp_tile;
#pragma unroll
            for (int v = 0; v < NV; ++v) acc[v] = (f4_t){0.f, 0.f, 0.f, 0.f};
        }
        const uint4 *ap = xa + cp_batch * 16;
        if (NOMATH) {
            uint32_t xo = ap[0].x ^ ap[1].y ^ ap[2].z ^ ap[3].w;
#pragma unroll
            for (int v = 0; v < NV; ++v) xo ^= U.w[v].x ^ U.w[v].y ^ U.w[v].z ^ U.w[v].w ^ U.meta[v];
            acc[0][0] += __builtin_bit_cast(float, xo & 0x3fffffffu);
        } else {
            h8_t a[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) a[j] = __builtin_bit_cast(h8_t, ap[j]);
            ColDecode cd[NV];
#pragma unroll
            for (int v = 0; v < NV; ++v) cd[v] = make_col_decode(U.meta[v] >> 16, U.meta[v]);
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int v = 0; v < NV; ++v)
                    acc[v] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[j], decode_word_h8(U.w[v][j], cd[v]), acc[v], 0, 0, 0);
        }
        cp_batch -= NW;
        if (cp_batch < 0) {
            cp_batch += nb;
            cp_tile -= 1;
        }
    };

    // ---- the loop: loads past the end of the range are switched off through their offset, not branched around, so
    //      that the compiler's counts of loads in flight stay exact
    for (int i = 0; i < n; i += DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            if (i + d < n) compute(ring[d]);
            issue(ring[d], i + d + DEPTH < n);
        }
    }
    if (n > 0) dump(tile_hi - cur_tile);

    // ---- the lower workgroups' sums of the bottom strip, published when they were a few units into their ranges:
    //      workgroups first .. wg - 1, one slot each
    float part[NV];
#pragma unroll
    for (int v = 0; v < NV; ++v) part[v] = 0.f;
    if (gets_partials && owner && e_pb == 0) {
        const int u_first = tile_lo * nb;
        const int big = hr * (hq + 1);
        const int first = u_first < big ? sdiv_magic(u_first, hq + 1, p.q1_magic) : hr + sdiv_magic(u_first - big, hq, p.q_magic);
        for (int src = first; src < wg; ++src) {
            uint64_t *const slot = p.tagged + (size_t)src * slot_elems;
            uint64_t got[NV];
            uint32_t tries = p.spin_limit;
            for (;;) {
                uint64_t all = S_MARK;
#pragma unroll
                for (int v = 0; v < NV; ++v) {
                    got[v] = __hip_atomic_load(&slot[(v * M + e_row) * 16 + e_col], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    all &= got[v];
                }
                // (a limit of 0xFFFFFFFF is the test hook: give up even though everything has arrived)
                if (p.spin_limit != 0xFFFFFFFFu && all != 0) break;
                if (p.spin_limit == 0xFFFFFFFFu || --tries == 0) {
                    // gave up: the call's result is not valid; the word stays set for the host to find
                    __hip_atomic_store(&p.counters[EXCHANGE_ERROR_WORD], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    break;
                }
                __builtin_amdgcn_s_sleep(1);
            }
#pragma unroll
            for (int v = 0; v < NV; ++v) {
                part[v] += __uint_as_float((uint32_t)got[v]);
                // back to zero for the next call
                __hip_atomic_store(&slot[(v * M + e_row) * 16 + e_col], (uint64_t)0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    }
    __syncthreads();

    if (owner) {
        const int pc = npieces - 1 - e_pb;
        float s[NV];
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            s[v] = part[v];
#pragma unroll
            for (int w = 0; w < NW; ++w) s[v] += redf[(((pc * NW + w) * NV + v) * 16 + e_col) * 4 + e_row];
        }
        if (EPI == EPI_PLAIN) {
            half_t o = (half_t)s[0];
            if (p.bias != nullptr) o = o + bias_v;
            p.y[(size_t)e_row * N + e_tile * 16 + e_col] = o;
        } else if (EPI == EPI_SILU_MUL) {
            p.y[(size_t)e_row * N + e_tile * 16 + e_col] = NOMATH ? (half_t)(s[0] + s[NV - 1]) : (half_t)(silu_f32(s[0]) * s[NV - 1]);
        } else {
            const RopeArgs &ra = p.rope;
            int bb, ss;
            split_row(ra, e_row, bb, ss);
            float o1 = s[0], o2 = s[NV - 1];
            if (rope_which < 2) {
                o1 = s[0] * rope_cs - s[NV - 1] * rope_sn;
                o2 = s[NV - 1] * rope_cs + s[0] * rope_sn;
            }
            half_t *dst;
            size_t off;
            if (rope_which == 0) {
                dst = ra.q;
                off = ((size_t)(bb * ra.H + rope_head) * ra.S + ss) * 128;
            } else {
                dst = (rope_which == 1) ? ra.k : ra.v;
                // kv_offset < 0: the cache row is the token's position
                const int crow = ra.kv_offset >= 0 ? ra.kv_offset + ss : min(max(rope_pos, 0), ra.kv_capacity - 1);
                off = ((size_t)(bb * ra.H + rope_head) * ra.kv_capacity + crow) * 128;
            }
            dst[off + rope_dd] = (half_t)o1;
            dst[off + 64 + rope_dd] = (half_t)o2;
        }
    }
}

// ---- 5 .. 16 rows ------------------------------------------------------------------------------------------------
// The same walk over the same layout for more rows than fit LDS with all of K (16 rows of K = 11008 are 344 KiB): a
// wave fetches the rows' values of a unit WITH the unit, from memory (the rows are a few hundred KiB that every
// workgroup reads: they live in L2) - four loads of four rows each, 256 contiguous bytes per row, so that a load
// touches eight cache lines and uses all of them (fetching the A operand as the matrix core wants it - lane (r4, c):
// row c, chunks 4 * r4 + j - would touch 32 lines per load and use a quarter of each; measured, that made the time grow
// with the number of rows: 14.4 us at 5 rows, 20.6 at 16 for the LLaMA-7B gate/up pair).  The wave turns the block
// into operand order through a 4.25 KiB LDS slot of its own (rows 17 chunks apart: both directions free of bank
// conflicts; no barrier, a wave's LDS accesses are in order), in the k order of the decoded weights.  All 64 lanes of
// an accumulator hold rows below M now (lane (r4, c): rows 4 * r4 .. 4 * r4 + 3 of column c), so a wave's slot of
// partial sums is 1 KiB per strip, and a thread may finish several output elements.  No variant with the norm inside
// or with the act-order gather: callers with more than four rows run the norm launch (which can store in the
// projection's row order) and the entry points gather beforehand.
template <int NV>
struct TUnit {
    u32x4_t w[NV];
    uint32_t meta[NV];
    u32x4_t a[4];
};

template <int EPI, int NW, int DEPTH, int NS>
__global__ __launch_bounds__(64 * NW) void gptq4_stream_tall_kernel(STREAM_HOT_PARAMS, StreamArgs p) {
    constexpr int NV = (EPI == EPI_PLAIN) ? 1 : 2;
    constexpr int NV2 = NV * NS;  // weight blocks per unit: NS adjacent tiles (strips; quarter-head pairs for the rotary epilogue) of NV matrices
    constexpr int NT = 64 * NW;
    constexpr int RE = (16 * 64 + NT - 1) / NT;  // (row, column of a head's half) pairs of the rotary table per thread
    extern __shared__ uint4 smem[];
    __shared__ int arrivals;
    __shared__ int pos_s[16];

    asm volatile("" ::"s"(p.x), "s"(p.M), "s"(p.K), "s"(p.N), "s"(p.red_off), "s"(p.nat_off), "s"(p.m_magic), "s"(p.tagged));
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r4 = lane >> 4;
    const int c = lane & 15;

    const int M = p.M, K = p.K, N = p.N, nb = hnb, G = hgroups;
    const int wg = blockIdx.x;
    const int a0 = wg * hq + min(wg, hr);
    const int L = hq + (wg < hr ? 1 : 0);
    const int b0 = a0 + L;
    const int tile_hi = sdiv_magic(b0 - 1, nb, hnb_magic);
    const int n = wave < L ? (L - wave + NW - 1) / NW : 0;

    // ---- rotary: the table rows of the M tokens, requested ahead of everything (two dependent loads), parked in
    //      registers until the loop is done
    int rp_pos[RE];
    float rp_cs[RE], rp_sn[RE];
    if (EPI == EPI_ROPE) {
#pragma unroll
        for (int i = 0; i < RE; ++i) {
            const int idx = tid + i * NT;
            rp_pos[i] = idx < M * 64 ? p.rope.position_ids[idx >> 6] : 0;
        }
    }

    const __amdgpu_buffer_rsrc_t rs_x = srsrc(p.x, (uint32_t)M * K * 2u);
    // load i of a unit: row 4 * i + r4, chunk c of the unit's sixteen; rows from M on are never read
    uint32_t xoff[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) xoff[i] = (4 * i + r4 < M) ? (uint32_t)(4 * i + r4) * (uint32_t)K * 2u + (uint32_t)c * 16u : S_OFF_RANGE;
    constexpr uint32_t wbytes = 0x7FFFFFF0u, mbytes = 0x7FFFFFF0u;  // (see the kernel above)
    __amdgpu_buffer_rsrc_t rs_w[NV], rs_m[NV];
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        rs_w[v] = srsrc(v ? hw1 : hw0, wbytes);
        rs_m[v] = srsrc(v ? hm1 : hm0, mbytes);
    }
    const int bpg = hbpg;
    int ld_tile = tile_hi, ld_batch = 0;
    if (n > 0) {
        const int u = b0 - 1 - wave;
        ld_tile = sdiv_magic(u, nb, hnb_magic);
        ld_batch = u - ld_tile * nb;
    }
    int cp_tile = ld_tile, cp_batch = ld_batch;
    auto strip_of = [&](int tile, int v) { return (EPI == EPI_ROPE) ? ((tile >> 2) << 3) + (tile & 3) + 4 * v : tile; };
    auto issue = [&](TUnit<NV2> &U, bool live) {
        const uint32_t dead = live ? 0u : S_OFF_RANGE;
        const int g = (bpg == 1) ? ld_batch : (int)__umulhi((unsigned)ld_batch, hgroup_magic);
#pragma unroll
        for (int s = 0; s < NS; ++s)
#pragma unroll
            for (int v = 0; v < NV; ++v) {
                const int strip = strip_of(ld_tile * NS + s, v);
                U.w[s * NV + v] =
                    __builtin_amdgcn_raw_buffer_load_b128(rs_w[v], ((uint32_t)lane * 16u) | dead, (uint32_t)(strip * nb + ld_batch) * 1024u, 2);
                U.meta[s * NV + v] = __builtin_amdgcn_raw_buffer_load_b32(rs_m[v], ((uint32_t)c * 4u) | dead, (uint32_t)(strip * G + g) * 64u, 0);
            }
#pragma unroll
        for (int i = 0; i < 4; ++i) U.a[i] = __builtin_amdgcn_raw_buffer_load_b128(rs_x, xoff[i] | dead, (uint32_t)ld_batch * 256u, 0);
        ld_batch -= NW;
        if (ld_batch < 0) {
            ld_batch += nb;
            ld_tile -= 1;
        }
    };
    TUnit<NV2> ring[DEPTH];
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) issue(ring[d], d < n);

    if (EPI == EPI_ROPE) {
#pragma unroll
        for (int i = 0; i < RE; ++i) {
            const int idx = tid + i * NT;
            const int pos = min(max(rp_pos[i], 0), p.rope.max_pos - 1);
            rp_cs[i] = idx < M * 64 ? p.rope.cos_table[(size_t)pos * 64 + (idx & 63)] : 1.f;
            rp_sn[i] = idx < M * 64 ? p.rope.sin_table[(size_t)pos * 64 + (idx & 63)] : 0.f;
        }
    }

    const int tile_lo = sdiv_magic(a0, nb, hnb_magic);
    const int npieces = tile_hi - tile_lo + 1;
    const int top_len = min(L, b0 - tile_hi * nb);
    const bool publishes = (b0 - tile_hi * nb) != nb;
    const bool shared_lo = (a0 - tile_lo * nb) != 0;
    const int fin0 = publishes ? 1 : 0;
    const int total = (npieces - fin0) * NS * M * 16;

    // element e = (piece from the bottom, tile of the piece's NS, row, column); thread t finishes e = NT - 1 - t, + NT, ...: the bottom piece,
    // whose other part comes from memory, falls to lanes of the last wave, which never has the most units
    const int e_mine = NT - 1 - tid;
    const bool gets_partials = shared_lo && e_mine < min(total, NS * M * 16);

    f4_t *const red = reinterpret_cast<f4_t *>(smem);  // [piece][wave][NV2][lane]
    const float *const redf = reinterpret_cast<const float *>(red);
    for (int pc = 0; pc < npieces; ++pc)
#pragma unroll
        for (int v = 0; v < NV2; ++v) red[((pc * NW + wave) * NV2 + v) * 64 + lane] = (f4_t){0.f, 0.f, 0.f, 0.f};
    if (tid == 0) arrivals = 0;
    __syncthreads();

    const int slot_elems = NV2 * 16 * M;
    auto arrive_top = [&]() {
        int old = 0;
        if (lane == 0) old = __hip_atomic_fetch_add(&arrivals, 1, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_WORKGROUP);
        old = __builtin_amdgcn_readfirstlane(old);
        if (old != NW - 1) return;
        uint64_t *const mine = p.tagged + (size_t)wg * slot_elems;
        for (int e = lane; e < slot_elems; e += 64) {  // e = (block * M + row) * 16 + column, block = tile of the NS * NV + matrix
            const int col = e & 15, t = e >> 4;
            const int v = (t * p.m_magic) >> 16;
            const int row = t - v * M;
            float s = 0.f;
#pragma unroll
            for (int w = 0; w < NW; ++w) s += redf[((w * NV2 + v) * 64 + (row >> 2) * 16 + col) * 4 + (row & 3)];
            __hip_atomic_store(&mine[e], S_MARK | (uint64_t)__float_as_uint(s), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    };
    f4_t acc[NV2];
#pragma unroll
    for (int v = 0; v < NV2; ++v) acc[v] = (f4_t){0.f, 0.f, 0.f, 0.f};
    auto dump = [&](int pc) {
#pragma unroll
        for (int v = 0; v < NV2; ++v) red[((pc * NW + wave) * NV2 + v) * 64 + lane] = acc[v];
        if (pc == 0 && publishes) arrive_top();
    };
    if (publishes && wave >= top_len) arrive_top();

    int cur_tile = cp_tile;
    uint4 *const turn = smem + p.nat_off + wave * (16 * 17);  // the wave's own 16 x 17 chunks
    auto compute = [&](const TUnit<NV2> &U) {
        if (cp_tile != cur_tile) {
            dump(tile_hi - cur_tile);
            cur_tile = cp_tile;
#pragma unroll
            for (int v = 0; v < NV2; ++v) acc[v] = (f4_t){0.f, 0.f, 0.f, 0.f};
        }
        // rows x chunks in, (row c, chunks 4 * r4 + j) out
#pragma unroll
        for (int i = 0; i < 4; ++i) turn[(4 * i + r4) * 17 + c] = pair_order_u4(__builtin_bit_cast(uint4, U.a[i]));
        h8_t a[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) a[j] = __builtin_bit_cast(h8_t, turn[c * 17 + 4 * r4 + j]);
        ColDecode cd[NV2];
#pragma unroll
        for (int v = 0; v < NV2; ++v) cd[v] = make_col_decode(U.meta[v] >> 16, U.meta[v]);
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int v = 0; v < NV2; ++v)
                acc[v] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[j], decode_word_h8(U.w[v][j], cd[v]), acc[v], 0, 0, 0);
        cp_batch -= NW;
        if (cp_batch < 0) {
            cp_batch += nb;
            cp_tile -= 1;
        }
    };

    for (int i = 0; i < n; i += DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            if (i + d < n) compute(ring[d]);
            issue(ring[d], i + d + DEPTH < n);
        }
    }
    if (n > 0) dump(tile_hi - cur_tile);

    // ---- the rotary table rows reach LDS (behind the partial sums)
    float *const cs_s = reinterpret_cast<float *>(smem + p.red_off);  // [M][64], then the sines
    float *const sn_s = cs_s + 16 * 64;
    if (EPI == EPI_ROPE) {
#pragma unroll
        for (int i = 0; i < RE; ++i) {
            const int idx = tid + i * NT;
            if (idx < M * 64) {
                cs_s[idx] = rp_cs[i];
                sn_s[idx] = rp_sn[i];
                if ((idx & 63) == 0) pos_s[idx >> 6] = rp_pos[i];
            }
        }
    }

    // ---- the lower workgroups' sums of the bottom strip
    float part[NV];
#pragma unroll
    for (int v = 0; v < NV; ++v) part[v] = 0.f;
    if (gets_partials) {
        const int e_col = e_mine & 15, e_s = ((e_mine >> 4) * p.m_magic) >> 16, e_row = (e_mine >> 4) - e_s * M;  // piece 0: e = (tile * M + row) * 16 + column
        const int u_first = tile_lo * nb;
        const int big = hr * (hq + 1);
        const int first = u_first < big ? sdiv_magic(u_first, hq + 1, p.q1_magic) : hr + sdiv_magic(u_first - big, hq, p.q_magic);
        for (int src = first; src < wg; ++src) {
            uint64_t *const slot = p.tagged + (size_t)src * slot_elems;
            uint64_t got[NV];
            uint32_t tries = p.spin_limit;
            for (;;) {
                uint64_t all = S_MARK;
#pragma unroll
                for (int v = 0; v < NV; ++v) {
                    got[v] = __hip_atomic_load(&slot[((e_s * NV + v) * M + e_row) * 16 + e_col], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    all &= got[v];
                }
                if (p.spin_limit != 0xFFFFFFFFu && all != 0) break;
                if (p.spin_limit == 0xFFFFFFFFu || --tries == 0) {
                    __hip_atomic_store(&p.counters[EXCHANGE_ERROR_WORD], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    break;
                }
                __builtin_amdgcn_s_sleep(1);
            }
#pragma unroll
            for (int v = 0; v < NV; ++v) {
                part[v] += __uint_as_float((uint32_t)got[v]);
                __hip_atomic_store(&slot[((e_s * NV + v) * M + e_row) * 16 + e_col], (uint64_t)0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    }
    __syncthreads();

    for (int e = e_mine; e < total; e += NT) {
        const int e_col = e & 15;
        const int e_t = e >> 4;
        const int e_ps = (e_t * p.m_magic) >> 16;  // (piece, tile of the piece)
        const int e_row = e_t - e_ps * M;
        const int e_pb = e_ps / NS, e_s = e_ps - e_pb * NS;
        const int e_tile = (tile_lo + e_pb) * NS + e_s;
        const int pc = npieces - 1 - e_pb;
        float s[NV];
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            s[v] = (e == e_mine) ? part[v] : 0.f;
#pragma unroll
            for (int w = 0; w < NW; ++w) s[v] += redf[(((pc * NW + w) * NV2 + e_s * NV + v) * 64 + (e_row >> 2) * 16 + e_col) * 4 + (e_row & 3)];
        }
        if (EPI == EPI_PLAIN) {
            half_t o = (half_t)s[0];
            if (p.bias != nullptr) o = o + p.bias[e_tile * 16 + e_col];
            p.y[(size_t)e_row * N + e_tile * 16 + e_col] = o;
        } else if (EPI == EPI_SILU_MUL) {
            p.y[(size_t)e_row * N + e_tile * 16 + e_col] = (half_t)(silu_f32(s[0]) * s[NV - 1]);
        } else {
            const RopeArgs &ra = p.rope;
            const int head_col = e_tile >> 2;
            const int dd = ((e_tile & 3) << 4) + e_col;
            const int which = head_col / ra.H;
            const int head = head_col - which * ra.H;
            int bb, ss;
            split_row(ra, e_row, bb, ss);
            float o1 = s[0], o2 = s[NV - 1];
            if (which < 2) {
                const float cs = cs_s[e_row * 64 + dd], sn = sn_s[e_row * 64 + dd];
                o1 = s[0] * cs - s[NV - 1] * sn;
                o2 = s[NV - 1] * cs + s[0] * sn;
            }
            half_t *dst;
            size_t off;
            if (which == 0) {
                dst = ra.q;
                off = ((size_t)(bb * ra.H + head) * ra.S + ss) * 128;
            } else {
                dst = (which == 1) ? ra.k : ra.v;
                const int crow = ra.kv_offset >= 0 ? ra.kv_offset + ss : min(max(pos_s[e_row], 0), ra.kv_capacity - 1);
                off = ((size_t)(bb * ra.H + head) * ra.kv_capacity + crow) * 128;
            }
            dst[off + dd] = (half_t)o1;
            dst[off + 64 + dd] = (half_t)o2;
        }
    }
}

// ---- layout conversion ------------------------------------------------------------------------------------------
// word o of the streaming order <-> (8-row block kb, column n) of the checkpoint order
__device__ __forceinline__ void stream_coords(size_t o, int nb, int &kb, int &n) {
    const int j = (int)(o & 3);
    const int lane = (int)((o >> 2) & 63);
    const size_t blk = o >> 8;  // strip * nb + unit
    const int strip = (int)(blk / (size_t)nb);
    const int unit = (int)(blk - (size_t)strip * nb);
    kb = unit * 16 + 4 * (lane >> 4) + j;
    n = strip * 16 + (lane & 15);
}

__global__ __launch_bounds__(256) void gptq4_stream_pack_kernel(const uint32_t *__restrict__ qweight, uint32_t *__restrict__ sw,
                                                                int K, int N) {
    const size_t o = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (o >= (size_t)(K >> 3) * N) return;
    int kb, n;
    stream_coords(o, K >> 7, kb, n);
    sw[o] = qweight[(size_t)kb * N + n];
}

// (whole lines both ways: a wave moves the packed rows 4 * r .. 4 * r + 3 of one unit for 64 columns - it reads one
// 16-byte chunk per lane, 256 contiguous bytes per strip, and writes 256 contiguous bytes of each of the four rows)
__global__ __launch_bounds__(256) void gptq4_stream_unpack_kernel(const uint32_t *__restrict__ sw, uint32_t *__restrict__ qweight,
                                                                  int K, int N) {
    const int nb = K >> 7;
    const int r = threadIdx.x >> 6, cc = threadIdx.x & 63;
    const int col = blockIdx.x * 64 + cc;  // N % 64 == 0
    const int unit = blockIdx.y;
    const uint4 w = reinterpret_cast<const uint4 *>(sw)[((size_t)(col >> 4) * nb + unit) * 64 + r * 16 + (col & 15)];
    uint32_t *dst = qweight + (size_t)(unit * 16 + 4 * r) * N + col;
    dst[0] = w.x;
    dst[(size_t)N] = w.y;
    dst[2 * (size_t)N] = w.z;
    dst[3 * (size_t)N] = w.w;
}

// meta[(strip * G + g) * 16 + c] = scale bits | stored zero << 16 of column 16 * strip + c in group g
__global__ __launch_bounds__(256) void gptq4_stream_meta_kernel(const uint32_t *__restrict__ qzeros, const half_t *__restrict__ scales,
                                                                uint32_t *__restrict__ meta, int G, int N) {
    const size_t o = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (o >= (size_t)G * N) return;
    const int c = (int)(o & 15);
    const size_t sg = o >> 4;
    const int strip = (int)(sg / (size_t)G);
    const int g = (int)(sg - (size_t)strip * G);
    const int n = strip * 16 + c;
    const uint32_t z = (qzeros[(size_t)g * (N >> 3) + (n >> 3)] >> ((n & 7) * 4)) & 0xFu;
    meta[o] = (uint32_t)reinterpret_cast<const uint16_t *>(scales)[(size_t)g * N + n] | (z << 16);
}

// one thread per (group, 8 columns): a word of qzeros and eight scales
__global__ __launch_bounds__(256) void gptq4_stream_unmeta_kernel(const uint32_t *__restrict__ meta, uint32_t *__restrict__ qzeros,
                                                                  half_t *__restrict__ scales, int G, int N) {
    const size_t o = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (o >= (size_t)G * (N >> 3)) return;
    const int g = (int)(o / (size_t)(N >> 3));
    const int n0 = (int)(o - (size_t)g * (N >> 3)) * 8;
    uint32_t zw = 0;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        const int n = n0 + t;
        const uint32_t m = meta[((size_t)(n >> 4) * G + g) * 16 + (n & 15)];
        reinterpret_cast<uint16_t *>(scales)[(size_t)g * N + n] = (uint16_t)(m & 0xFFFFu);
        zw |= ((m >> 16) & 0xFu) << (4 * t);
    }
    qzeros[o] = zw;
}

// One thread per word of the streaming order, decoded with the matmul kernel's own decode_word.
__global__ __launch_bounds__(256) void gptq4_stream_dequant_kernel(const uint32_t *__restrict__ sw, const uint32_t *__restrict__ meta,
                                                                   half_t *__restrict__ out, int K, int N, int groupsize) {
    const size_t o = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (o >= (size_t)(K >> 3) * N) return;
    int kb, n;
    stream_coords(o, K >> 7, kb, n);
    const int G = K / groupsize;
    const int g = (8 * kb) / groupsize;
    const uint32_t m = meta[((size_t)(n >> 4) * G + g) * 16 + (n & 15)];
    const ColDecode cd = make_col_decode(m >> 16, m);
    h2_t pr[4];
    decode_word(sw[o], cd, pr);
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {
        out[(size_t)(8 * kb + jj) * N + n] = pr[jj].x;
        out[(size_t)(8 * kb + jj + 4) * N + n] = pr[jj].y;
    }
}

// ---- launch ------------------------------------------------------------------------------------------------------
constexpr size_t STREAM_LDS_BUDGET = 160 * 1024 - 512;  // dynamic LDS a workgroup may ask for (the rest: the kernel's static words)

template <int EPI, int NW, int DEPTH, bool PERM, int NORM, bool NOMATH>
int launch_kernel(const StreamArgs &a, const StreamPlan &pl, hipStream_t stream) {
    static bool prepared = false;
    static std::mutex lock;
    {
        std::lock_guard<std::mutex> guard(lock);
        if (!prepared) {
            const void *fn = reinterpret_cast<const void *>(&gptq4_stream_kernel<EPI, NW, DEPTH, PERM, NORM, NOMATH>);
            const hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)STREAM_LDS_BUDGET);
            if (e != hipSuccess) return (int)e;
            prepared = true;
        }
    }
    hipLaunchKernelGGL((gptq4_stream_kernel<EPI, NW, DEPTH, PERM, NORM, NOMATH>), dim3((unsigned)pl.workgroups), dim3(64 * NW), pl.lds_bytes,
                       stream, STREAM_HOT_ARGS(a), a);
    return (int)hipGetLastError();
}

template <int EPI, int NW, int DEPTH>
int launch_shape(const StreamArgs &a, const StreamPlan &pl, bool nomath, hipStream_t stream) {
    const bool perm = a.perm != nullptr;
    if (nomath) return perm || a.nrm_weight ? (int)hipErrorInvalidValue : launch_kernel<EPI, NW, DEPTH, false, 0, true>(a, pl, stream);
    if (a.nrm_weight != nullptr) {
        if (EPI == EPI_PLAIN) return (int)hipErrorInvalidValue;  // no entry point asks a plain projection for it
        constexpr int E = (EPI == EPI_PLAIN) ? EPI_SILU_MUL : EPI;
        if (a.K <= 4096) return perm ? launch_kernel<E, NW, DEPTH, true, 2, false>(a, pl, stream) : launch_kernel<E, NW, DEPTH, false, 2, false>(a, pl, stream);
        return perm ? launch_kernel<E, NW, DEPTH, true, 4, false>(a, pl, stream) : launch_kernel<E, NW, DEPTH, false, 4, false>(a, pl, stream);
    }
    return perm ? launch_kernel<EPI, NW, DEPTH, true, 0, false>(a, pl, stream) : launch_kernel<EPI, NW, DEPTH, false, 0, false>(a, pl, stream);
}

template <int EPI, int NW, int DEPTH, int NS>
int launch_tall(const StreamArgs &a, const StreamPlan &pl, hipStream_t stream) {
    static bool prepared = false;
    static std::mutex lock;
    {
        std::lock_guard<std::mutex> guard(lock);
        if (!prepared) {
            const void *fn = reinterpret_cast<const void *>(&gptq4_stream_tall_kernel<EPI, NW, DEPTH, NS>);
            const hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)STREAM_LDS_BUDGET);
            if (e != hipSuccess) return (int)e;
            prepared = true;
        }
    }
    hipLaunchKernelGGL((gptq4_stream_tall_kernel<EPI, NW, DEPTH, NS>), dim3((unsigned)pl.workgroups), dim3(64 * NW), pl.lds_bytes, stream,
                       STREAM_HOT_ARGS(a), a);
    return (int)hipGetLastError();
}

template <int EPI>
int launch_epi(const StreamArgs &a, const StreamPlan &pl, bool nomath, hipStream_t stream) {
    if (pl.tall) {
        if (nomath || a.perm != nullptr || a.nrm_weight != nullptr) return (int)hipErrorInvalidValue;
        switch ((pl.waves * 10 + pl.depth) * 10 + pl.strips) {
            case 811: return launch_tall<EPI, 8, 1, 1>(a, pl, stream);
            case 821: return launch_tall<EPI, 8, 2, 1>(a, pl, stream);
            case 1611: return launch_tall<EPI, 16, 1, 1>(a, pl, stream);
            case 1621: return launch_tall<EPI, 16, 2, 1>(a, pl, stream);
            case 812: return launch_tall<EPI, 8, 1, 2>(a, pl, stream);
            case 822: return launch_tall<EPI, 8, 2, 2>(a, pl, stream);
            case 1612: return launch_tall<EPI, 16, 1, 2>(a, pl, stream);
            case 1622: return launch_tall<EPI, 16, 2, 2>(a, pl, stream);
            default: return (int)hipErrorInvalidValue;
        }
    }
    switch (pl.waves * 10 + pl.depth) {
        case 81: return launch_shape<EPI, 8, 1>(a, pl, nomath, stream);
        case 82: return launch_shape<EPI, 8, 2>(a, pl, nomath, stream);
        case 83: return launch_shape<EPI, 8, 3>(a, pl, nomath, stream);
        case 161: return launch_shape<EPI, 16, 1>(a, pl, nomath, stream);
        case 162: return launch_shape<EPI, 16, 2>(a, pl, nomath, stream);
        default: return (int)hipErrorInvalidValue;
    }
}

uint32_t smagic(int d) { return d > 1 ? (uint32_t)(0x100000000ull / (unsigned)d + 1) : 0u; }

}  // namespace

StreamTuning g_stream_tuning = {0, 0};

static StreamPlan stream_plan_with(int epi, int M, int N, int K, bool norm, int strips);

StreamPlan stream_plan(int epi, int M, int N, int K, bool norm) {
    // 8 .. 16 rows: a unit is the 128 input rows of TWO adjacent tiles, so that the rows' chunks - twice the bytes of a
    // tile's weights at 16 rows - are fetched and turned once for both; only where a workgroup's range stays long (LLaMA-7B at
    // 16 rows: gate/up 16.8 against 17.7 us, down_proj 10.7 against 11.3 with 43 units to a workgroup; QKV 13.2 against
    // 11.4 and o_proj 7.3 against 5.9 with 24 and 16, where the ranges stop lining up with the tiles), where the tile
    // count is even and the partial sums of two tiles fit the LDS.  (depth + 10 in the tuning call: never; + 20: wherever
    // it can run.)
    const int tiles = (epi == EPI_ROPE) ? N / 32 : N / 16;
    const int mode = g_stream_tuning.depth / 10;
    if (M > STREAM_MAX_M && (tiles % 2) == 0 && mode != 1) {
        const StreamPlan two = stream_plan_with(epi, M, N, K, norm, 2);
        if (two.ok && (mode == 2 || (M >= 8 && two.q >= 40))) return two;
    }
    return stream_plan_with(epi, M, N, K, norm, 1);
}

static StreamPlan stream_plan_with(int epi, int M, int N, int K, bool norm, int strips) {
    StreamPlan pl = {};
    const int tuned_depth = g_stream_tuning.depth % 10;
    pl.depth = tuned_depth ? tuned_depth : 2;
    const int nv = (epi == EPI_PLAIN) ? 1 : 2;
    pl.strips = strips;
    pl.tiles = ((epi == EPI_ROPE) ? N / 32 : N / 16) / strips;
    pl.nb = K / 128;
    const long units = (long)pl.tiles * pl.nb;
    const int cus = device_shape().cus;
    pl.workgroups = (int)(units < cus ? units : cus);
    if (pl.workgroups < 1) return pl;
    pl.q = (int)(units / pl.workgroups);
    pl.r = (int)(units % pl.workgroups);
    // Launch shape, from sweeps at LLaMA-7B shapes with the weights coming from HBM (one row): two units in flight per
    // wave; eight waves per workgroup, sixteen for a plain projection with long ranges (down_proj: 8.1 against 8.6 us),
    // where a wave of eight would walk through a dozen units one after the other.
    pl.waves = g_stream_tuning.waves ? g_stream_tuning.waves : ((nv == 1 && pl.q >= 48) ? 16 : 8);
    if (!g_stream_tuning.waves && pl.nb < pl.waves) pl.waves = 8;
    if (pl.waves == 16 && pl.depth > 2) pl.depth = 2;
    pl.pieces = (pl.q + 1 + pl.nb - 1) / pl.nb + 1;
    if (M > STREAM_MAX_M) {
        // the A operand comes from memory with every unit, LDS holds the waves' partial sums (1 KiB per wave, matrix and
        // tile) and the rotary table rows of the tokens
        pl.tall = true;
        if (pl.depth > 2) pl.depth = 2;
        // eight waves for every shape here (LLaMA-7B down_proj at 16 rows: 11.2 us against 11.7 with sixteen)
        if (!g_stream_tuning.waves) pl.waves = 8;
        pl.xrow = 0;
        const int nv2 = nv * pl.strips;
        pl.red_off = pl.pieces * pl.waves * nv2 * 64;
        pl.nat_off = pl.red_off + 2 * 16 * 64 * (int)sizeof(float) / 16;  // behind the rotary table rows: a 16 x 17 chunk slot per wave
        size_t lds = ((size_t)pl.nat_off + (size_t)pl.waves * 16 * 17) * 16;
        if (lds < (size_t)81 * 1024) lds = (size_t)81 * 1024;
        pl.lds_bytes = lds;
        pl.ok = M <= STREAM_TALL_MAX_M && !norm && lds <= STREAM_LDS_BUDGET && (long)K * N < (1L << 32) && (long)M * K < (1L << 30) &&
                units < (1L << 24) && units * (pl.nb > pl.q + 1 ? pl.nb : pl.q + 1) < (1L << 32) &&
                (size_t)pl.workgroups * nv2 * 16 * M * sizeof(uint64_t) <= GPTQ4_WS_TAGGED_BYTES && pl.nb >= pl.waves &&
                pl.pieces * pl.strips * M < 1024 && (epi != EPI_ROPE || (N % 128) == 0);
        return pl;
    }
    pl.xrow = K / 8 + 1;
    pl.red_off = M * pl.xrow;
    const size_t red_chunks = (size_t)pl.pieces * pl.waves * nv * 16;  // one 16-byte chunk (four rows) per column
    pl.nat_off = pl.red_off + (int)red_chunks;
    size_t lds = ((size_t)pl.nat_off + (norm ? (size_t)M * (K / 8) : 0)) * 16;
    // one workgroup per CU: ask for more than half of a CU's 160 KiB
    if (lds < (size_t)81 * 1024) lds = (size_t)81 * 1024;
    pl.lds_bytes = lds;
    pl.ok = M >= 1 && M <= STREAM_MAX_M && lds <= STREAM_LDS_BUDGET && (long)K * N < (1L << 32) && (long)M * K < (1L << 30) &&
            units < (1L << 24) && units * (pl.nb > pl.q + 1 ? pl.nb : pl.q + 1) < (1L << 32) &&
            (size_t)pl.workgroups * nv * 16 * M * sizeof(uint64_t) <= GPTQ4_WS_TAGGED_BYTES && pl.pieces * M * 16 <= 64 * pl.waves && pl.nb >= pl.waves && (epi != EPI_ROPE || (N % 128) == 0);
    return pl;
}

int launch_stream(int epi, StreamArgs &a, const StreamPlan &pl, bool nomath, hipStream_t stream) {
    a.nb = pl.nb;
    a.q = pl.q;
    a.r = pl.r;
    a.xrow = pl.xrow;
    a.red_off = pl.red_off;
    a.nat_off = pl.nat_off;
    a.nb_magic = smagic(pl.nb);
    a.q_magic = smagic(pl.q);
    a.q1_magic = smagic(pl.q + 1);
    a.m_magic = (65536 + a.M - 1) / a.M;
    switch (epi) {
        case EPI_PLAIN: return launch_epi<EPI_PLAIN>(a, pl, nomath, stream);
        case EPI_SILU_MUL: return launch_epi<EPI_SILU_MUL>(a, pl, nomath, stream);
        default: return launch_epi<EPI_ROPE>(a, pl, nomath, stream);
    }
}

int launch_stream_pack(const uint32_t *qweight, const uint32_t *qzeros, const half_t *scales, uint32_t *sw, uint32_t *meta, int K,
                       int N, int groupsize, hipStream_t stream) {
    const size_t words = (size_t)(K >> 3) * N;
    hipLaunchKernelGGL(gptq4_stream_pack_kernel, dim3((unsigned)((words + 255) / 256)), dim3(256), 0, stream, qweight, sw, K, N);
    if (meta != nullptr) {
        const int G = K / groupsize;
        const size_t metas = (size_t)G * N;
        hipLaunchKernelGGL(gptq4_stream_meta_kernel, dim3((unsigned)((metas + 255) / 256)), dim3(256), 0, stream, qzeros, scales, meta, G, N);
    }
    return (int)hipGetLastError();
}

int launch_stream_unpack(const uint32_t *sw, const uint32_t *meta, uint32_t *qweight, uint32_t *qzeros, half_t *scales, int K, int N,
                         int groupsize, hipStream_t stream) {
    const size_t words = (size_t)(K >> 3) * N;
    (void)words;
    hipLaunchKernelGGL(gptq4_stream_unpack_kernel, dim3((unsigned)(N / 64), (unsigned)(K / 128)), dim3(256), 0, stream, sw, qweight, K, N);
    if (meta != nullptr) {
        const int G = K / groupsize;
        const size_t zwords = (size_t)G * (N >> 3);
        hipLaunchKernelGGL(gptq4_stream_unmeta_kernel, dim3((unsigned)((zwords + 255) / 256)), dim3(256), 0, stream, meta, qzeros, scales, G, N);
    }
    return (int)hipGetLastError();
}

int launch_stream_dequant(const uint32_t *sw, const uint32_t *meta, half_t *out, int K, int N, int groupsize, hipStream_t stream) {
    const size_t words = (size_t)(K >> 3) * N;
    hipLaunchKernelGGL(gptq4_stream_dequant_kernel, dim3((unsigned)((words + 255) / 256)), dim3(256), 0, stream, sw, meta, out, K, N,
                       groupsize);
    return (int)hipGetLastError();
}
