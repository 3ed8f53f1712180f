// Chained decode launch for gfx950: several small-M (1..4 rows) quantised projections in ONE persistent
// launch, e.g. o_proj -> residual add + RMSNorm -> gate/up + SiLU*mul -> down_proj.
//
// Why: a decode GEMV streams 9..47 MB in 6..15 us, of which about 6 us are a serial chain per launch (launch
// floor, prologue, first-load latency, partial-sum exchange) during which HBM idles.  Weights do not depend on
// activations, so here ONE grid (one workgroup per CU, resident for the whole launch) streams the weights of
// all phases as one sequence: every wave keeps DEPTH units of loads in flight at all times, and the loads of
// the next phase's first units are already under way while the phase before it is being reduced, handed over
// and normalised.
//
// Work decomposition (per phase)
//   unit   = (tile, 128-k batch): 2 strips of 32 columns x 128 k = 4 KiB of packed weights.  The two strips
//            are adjacent columns (plain projection), the same columns of gate and up (SiLU*mul), or head
//            columns d and d + 64 (rotary).  Lane l loads row l/16 of each 4-row K step and 2 adjacent words:
//            a word is the complete B operand of one v_mfma_f32_16x16x32_f16.
//   The units of a phase are one flat range dealt to workgroups (q or q+1 each) and inside a workgroup to
//   waves (contiguous sub-ranges), so every CU streams the same number of bytes +-1 unit whatever the tile
//   count.  A wave's range lies in one tile or crosses into the next.
//   x      = the M rows the phase multiplies with, staged once per workgroup in LDS in the k order the
//            decoded weights come out in ("pair order"); the A operand of every wave is read from there.
//   hand-over: the waves of a workgroup add their accumulators per tile through LDS (wave order) and the
//            workgroup stores one partial tile per touched tile in its slot of the workspace (slot = its rank
//            among the workgroups sharing the tile), every value as an 8-byte element {fp32 bits, tag}, tag =
//            the phase's number in the life of the workspace.  Nothing waits on the producer side.  A consumer
//            reads the partial tiles it needs, polls until all of them carry the tag it expects (bounded), adds
//            them in rank order - every consumer the same order, so results are deterministic - and applies
//            what lies between the two projections itself: rounding to fp16, bias, residual add, RMSNorm,
//            SiLU*mul.  There is no grid-wide barrier: a consumer waits for exactly the tiles it reads.
//   Outputs that must exist in memory (y, q/k/v with rotary) are written by all workgroups, a slice each,
//   where the launch reads the previous phase anyway (or at its end).
//
// Visibility across workgroups: partial sums are written with agent-scope (sc1) 8-byte stores and read with
// agent-scope loads, which go around the per-XCD L2s; an aligned 8-byte store is never seen half-written, so a
// value next to the expected tag is the value that was stored with it.  Every poll is bounded: a thread that
// gives up records CHAIN_ERR_TIMEOUT in the state, its workgroup returns at the next barrier, and the
// workgroups that depend on it give up in turn; the error is sticky until the host clears the workspace.
#include "gptq4_chain.h"

#include "../../include/gptq4.h"
#include "../../include/gptq4_experimental.h"
#include "gptq4_norm.h"

#include <mutex>

// Development aid, compiled out of the product build: per-workgroup 100 MHz clock stamps at the stage boundaries
// of every phase, written behind the partial sums (the workspace is then 1 MiB larger).
#ifdef GPTQ4_CHAIN_TIMERS
#define CHAIN_STAMP(i)                                                                                                   \
    do {                                                                                                                 \
        if (ht == 0)                                                                                                     \
            reinterpret_cast<unsigned long long *>(reinterpret_cast<char *>(A->partials) + A->partial_bytes)[wg * 64 + (i)] = wall_clock64(); \
    } while (0)
#else
#define CHAIN_STAMP(i)
#endif

namespace {

typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

constexpr uint32_t OFF_RANGE = 0x80000000u;  // a lane offset beyond any buffer: the load returns zeros, untouched memory
constexpr int AUX_SC1 = 16;                  // cache policy of buffer loads / stores: agent scope

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *p, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ int div_magic(int n, int d, uint32_t magic) { return d == 1 ? n : (int)__umulhi((unsigned)n, magic); }

typedef const __attribute__((address_space(4))) ChainPhase *PhasePtr;

struct UnitRegs {
    u32x2_t w[2][4];    // packed weights: [strip][K step], 2 adjacent columns per lane
    uint32_t raw_s[2];  // the 2 fp16 scales of the lane's columns
    uint32_t raw_z[2];  // the zero-point word holding the lane's columns
};

// tile -> first column of strip 0; the second strip lies 64 columns further (plain, rotary) or is the same
// columns of the second matrix (gate/up pair)
__device__ __forceinline__ int tile_col0(int epi, int tile) { return epi == EPI_SILU_MUL ? tile * 64 : tile * 128; }

// first unit and unit count of a workgroup / of one of its waves
__device__ __forceinline__ void wg_range(PhasePtr P, int wg, int &u0, int &n) {
    u0 = wg * P->q + min(wg, P->r);
    n = P->q + (wg < P->r ? 1 : 0);
}
template <int NW>
__device__ __forceinline__ void wave_range(PhasePtr P, int wg, int wave, int &u0, int &n) {
    int U0, nw;
    wg_range(P, wg, U0, nw);
    const int wq = nw / NW, wr = nw % NW;
    u0 = U0 + wave * wq + min(wave, wr);
    n = wq + (wave < wr ? 1 : 0);
}
// the workgroup that owns unit u
__device__ __forceinline__ int wg_of_unit(PhasePtr P, int u) {
    const int big = P->r * (P->q + 1);
    return u < big ? div_magic(u, P->q + 1, P->q1_magic) : P->r + div_magic(u - big, P->q, P->q_magic);
}

__device__ __forceinline__ float f_of(uint32_t u) { return __builtin_bit_cast(float, u); }

// Partial sums travel as 8-byte elements {fp32 bits, tag}: an aligned 8-byte store becomes visible as a whole,
// so a consumer that reads the tag it expects next to a value knows the value is this launch's, this phase's -
// no separate flag, no wait for store acknowledgements on the producer side, no grid-wide barrier.  The tag of
// phase p is the workgroup's launch-to-launch epoch + p + 1; the workspace starts zeroed and tags only grow.
//
// Sum over the contributing workgroups (rank order) of 8 adjacent columns; `base` = element offset of (tile,
// rank 0, row m, column) in the partial region, `stride` = elements between ranks.  Returns false if any element
// does not carry `tag` yet (the caller polls).
__device__ __forceinline__ bool sum_partials8(const __amdgpu_buffer_rsrc_t &rs, uint32_t base, uint32_t stride, int nc, uint32_t tag,
                                              float out[8]) {
#pragma unroll
    for (int i = 0; i < 8; ++i) out[i] = 0.f;
    bool valid = true;
    for (int r0 = 0; r0 < nc; r0 += 2) {
        u32x4_t a[2][4];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const uint32_t off = (base + (uint32_t)min(r0 + j, nc - 1) * stride) * 8u;
#pragma unroll
            for (int q = 0; q < 4; ++q) a[j][q] = __builtin_amdgcn_raw_buffer_load_b128(rs, off + 16u * q, 0, AUX_SC1);
        }
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            if (r0 + j < nc) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    valid = valid && a[j][q].y == tag && a[j][q].w == tag;
                    out[2 * q] += f_of(a[j][q].x);
                    out[2 * q + 1] += f_of(a[j][q].z);
                }
            }
        }
    }
    return valid;
}

__device__ __forceinline__ uint4 pack_h8(const half_t h[8]) {
    uint4 r;
    r.x = as_u32((h2_t){h[0], h[1]});
    r.y = as_u32((h2_t){h[2], h[3]});
    r.z = as_u32((h2_t){h[4], h[5]});
    r.w = as_u32((h2_t){h[6], h[7]});
    return r;
}

// What a bounded poll needs: the limit, where to report giving up.
struct PollCtx {
    uint32_t limit;
    int32_t *error;       // global error word
    uint32_t *abort_lds;  // workgroup flag: somebody gave up
};
__device__ __forceinline__ bool aborted(const PollCtx &ctx) {
    return __hip_atomic_load(ctx.abort_lds, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) != 0;
}
__device__ __forceinline__ void give_up(const PollCtx &ctx) {
    __hip_atomic_store(ctx.error, (int32_t)CHAIN_ERR_TIMEOUT, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(ctx.abort_lds, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}

// 8 adjacent output values of phase P (row m, columns n0 .. n0+7, n0 % 8 == 0) from its partial tiles, as the
// next consumer sees them: fp16(sum) (+ bias) of a plain phase, fp16(silu(gate) * up) of a pair.  Polls until the
// partial tiles carry `tag` (bounded: gives up after ctx.limit polls, reports it and returns what it has).
__device__ __forceinline__ uint4 phase_output8(PhasePtr P, const __amdgpu_buffer_rsrc_t &rs, int M, int m, int n0, uint32_t tag,
                                               const PollCtx &ctx) {
    const bool pair = P->epi == EPI_SILU_MUL;
    const int tile = pair ? (n0 >> 6) : (n0 >> 7);
    const int col = pair ? (n0 & 63) : (n0 & 127);
    const int first = wg_of_unit(P, tile * P->nb);
    const int nc = wg_of_unit(P, tile * P->nb + P->nb - 1) - first + 1;
    const uint32_t stride = (uint32_t)M * 128u;
    const uint32_t base = P->partial_off + ((uint32_t)tile * P->max_contrib * M + m) * 128u + col;
    float s[8], u[8];
    for (uint32_t spin = 0;; ++spin) {
        bool ok = sum_partials8(rs, base, stride, nc, tag, s);
        if (pair) ok = sum_partials8(rs, base + 64u, stride, nc, tag, u) && ok;
        if (ok) break;
        if (spin >= ctx.limit || ((spin & 15u) == 15u && aborted(ctx))) {
            give_up(ctx);
            break;
        }
        __builtin_amdgcn_s_sleep(1);
    }
    half_t h[8];
    if (!pair) {
#pragma unroll
        for (int i = 0; i < 8; ++i) h[i] = (half_t)s[i];
        if (P->bias != nullptr) {
            const uint4 bv = *reinterpret_cast<const uint4 *>(P->bias + n0);
            const h2_t b2[4] = {as_h2(bv.x), as_h2(bv.y), as_h2(bv.z), as_h2(bv.w)};
#pragma unroll
            for (int i = 0; i < 4; ++i) h[2 * i] = h[2 * i] + b2[i].x, h[2 * i + 1] = h[2 * i + 1] + b2[i].y;
        }
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) h[i] = (half_t)(silu_f32(s[i]) * u[i]);
    }
    return pack_h8(h);
}

// The finished values of a phase - fp16(sum) (+ bias), or fp16(silu(gate) * up) - exist once more in the workspace
// as 8-byte elements {2 fp16 values, tag}: every workgroup finishes a slice of the columns from the partial tiles
// (phase_output8) and all consumers read these, 4 bytes per value, instead of adding up to 8 partial tiles of 8
// bytes per value each themselves (256 KiB per workgroup for a 4096-wide projection whose K is split 8 ways).
// 8 adjacent values of phase P, row m, columns n0 ..; polls until they carry `tag` (bounded).
__device__ __forceinline__ uint4 final8(PhasePtr P, const __amdgpu_buffer_rsrc_t &rs, int m, int n0, uint32_t tag, const PollCtx &ctx) {
    const uint32_t off = (P->final_off + ((uint32_t)m * P->N + n0) / 2u) * 8u;
    u32x4_t a, b;
    for (uint32_t spin = 0;; ++spin) {
        a = __builtin_amdgcn_raw_buffer_load_b128(rs, off, 0, AUX_SC1);
        b = __builtin_amdgcn_raw_buffer_load_b128(rs, off + 16u, 0, AUX_SC1);
        if (a.y == tag && a.w == tag && b.y == tag && b.w == tag) break;
        if (spin >= ctx.limit || ((spin & 15u) == 15u && aborted(ctx))) {
            give_up(ctx);
            break;
        }
        __builtin_amdgcn_s_sleep(1);
    }
    return make_uint4(a.x, a.z, b.x, b.z);
}

// LDS-direct loads (global memory -> LDS without passing registers) issued as inline assembly: lane l's 16 (4)
// bytes land at lds_base + 16 l (4 l).  Written as assembly on purpose - the compiler does not know these loads
// exist, so it does not make every later LDS read of the wave wait for them (it cannot tell which LDS bytes they
// fill and would wait for all of them: no load could be in flight under the arithmetic).  The wave waits itself,
// with s_waitcnt vmcnt, before it reads a slot.
__device__ __forceinline__ u32x4_t rsrc_words(const void *p, uint32_t bytes) {
    const uint64_t a = reinterpret_cast<uint64_t>(p);
    return (u32x4_t){(uint32_t)a, (uint32_t)(a >> 32) & 0xffffu, bytes, 0x00020000u};
}
__device__ __forceinline__ void dma16(uint32_t lds_base, u32x4_t rsrc, uint32_t voff, uint32_t soff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds" ::"s"(lds_base), "v"(voff), "s"(rsrc), "s"(soff) : "memory");
}
__device__ __forceinline__ void dma4(uint32_t lds_base, u32x4_t rsrc, uint32_t voff, uint32_t soff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dword %1, %2, %3 offen lds" ::"s"(lds_base), "v"(voff), "s"(rsrc), "s"(soff) : "memory");
}
__device__ __forceinline__ uint32_t lds_address(const void *p) {
    return (uint32_t)reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) const char *)p);
}

// Waves of a workgroup have two roles, and after one barrier at the start they never meet at a workgroup barrier
// again: they signal each other through counters in LDS.
//   CHAIN_NS streaming waves own the weight stream and the matrix-core work.  A wave's units of all phases are
//   ONE sequence; it loads them straight into a ring of slots in LDS (buffer_load ... lds: no registers held, the
//   slot index is a run-time value) with ONE unit in flight at a time - one unit per wave is what keeps a CU's
//   share of HBM bandwidth busy; more only lengthens the queue every other load of the CU waits in - and it
//   keeps loading, one unit after the other, while it waits for the rows of its next phase: by the time a phase
//   has been handed over, up to `ring` units of it are in LDS already.
//   CHAIN_NH helper waves do what is latency-critical and small - polling and adding partial tiles, residual add
//   / RMSNorm / SiLU*mul into LDS, the workgroup's partial stores, the outputs.
constexpr int CHAIN_NS = 4;
constexpr int CHAIN_NH = 4;
constexpr int UNIT_WORD_BYTES = 8192;  // 2 strips x 4 K steps x 64 lanes x 16 bytes
constexpr int UNIT_LDS_BYTES = UNIT_WORD_BYTES + 4 * 256;  // + scales of both strips, zero words of both strips (a 64-lane dword load each)

__global__ __launch_bounds__(64 * (CHAIN_NS + CHAIN_NH)) void gptq4_chain_kernel(const ChainArgs args_by_value) {
    // The arguments are read where the launch put them, in the kernel-argument segment (constant memory, scalar
    // loads with a dynamic phase index); touching the by-value copy would make the compiler spill the whole
    // table to scratch memory to index it.
    const __attribute__((address_space(4))) ChainArgs *const A =
        (const __attribute__((address_space(4))) ChainArgs *)__builtin_amdgcn_kernarg_segment_ptr();
    constexpr int NS = CHAIN_NS, NH = CHAIN_NH;
    constexpr int TH = 64 * NH;  // helper threads
    static_assert(TH == 256, "the RMSNorm statistics follow the stand-alone kernel's 256-thread order");
    extern __shared__ uint4 smem[];
    __shared__ int s_ft[NS], s_lt[NS];
    __shared__ float s_part[CHAIN_MAX_M * 4];
    __shared__ uint32_t s_ctl[4];   // epoch, error word at the start, "somebody gave up"
    __shared__ uint32_t s_sync[4];  // phases whose rows are staged; streaming waves that finished a phase (running total); helper barrier arrivals

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const bool helper = wave >= NS;
    const int ht = tid - 64 * NS;  // index among the helper threads (negative in streaming waves)
    const int hw = wave - NS;
    const int lrow = lane >> 4;
    const int lcol = lane & 15;
    const int wg = blockIdx.x;
    const int G = gridDim.x;
    const int M = A->M;
    const int P = A->nphases;
    const int R = A->ring_slots;

    uint4 *const xs = smem;
    float *const red = reinterpret_cast<float *>(smem + A->red_off);
    uint4 *const keep = smem + A->keep_off;  // the last residual sums, for a later phase of this launch
    char *const ring = reinterpret_cast<char *>(smem + A->ring_off);
    const int xs_stride = A->xs_stride;

    ChainState *const st = A->state;
    PollCtx poll;
    poll.limit = A->spin_limit;
    poll.error = &st->error;
    poll.abort_lds = &s_ctl[2];
    auto lds_load = [](uint32_t *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP); };

    if (!helper) {
        // =============================================================== streaming waves
        u32x4_t rs_w0, rs_w1, rs_s0, rs_s1, rs_z0, rs_z1;
        int l_epi = 0, l_N = 0, l_nb = 1, l_strip1 = 0, l_u0 = 0, l_n = 0, l_bpg = 1;
        uint32_t l_nb_magic = 0, l_group_magic = 0;
        int lp = -1, li = 0;
        auto next_stream_phase = [&]() {
            for (;;) {
                ++lp;
                li = 0;
                if (lp >= P) return;
                const PhasePtr Q = A->ph + lp;
                wave_range<NS>(Q, wg, wave, l_u0, l_n);
                if (l_n == 0) continue;
                l_epi = Q->epi, l_N = Q->N, l_nb = Q->nb, l_nb_magic = Q->nb_magic, l_bpg = Q->bpg, l_group_magic = Q->group_magic;
                l_strip1 = (Q->epi == EPI_SILU_MUL) ? 0 : 64;
                const int m1 = (Q->epi == EPI_SILU_MUL) ? 1 : 0;
                const uint32_t wbytes = (uint32_t)(Q->K >> 3) * Q->N * 4u;
                rs_w0 = rsrc_words(Q->w[0].qweight, wbytes);
                rs_w1 = rsrc_words(Q->w[m1].qweight, wbytes);
                rs_s0 = rsrc_words(Q->w[0].scales, (uint32_t)Q->groups * Q->N * 2u);
                rs_s1 = rsrc_words(Q->w[m1].scales, (uint32_t)Q->groups * Q->N * 2u);
                rs_z0 = rsrc_words(Q->w[0].qzeros, (uint32_t)Q->groups * (Q->N >> 3) * 4u);
                rs_z1 = rsrc_words(Q->w[m1].qzeros, (uint32_t)Q->groups * (Q->N >> 3) * 4u);
                return;
            }
        };
        {
            const PhasePtr Q = A->ph;
            rs_w0 = rs_w1 = rsrc_words(Q->w[0].qweight, 16u);
            rs_s0 = rs_s1 = rsrc_words(Q->w[0].scales, 16u);
            rs_z0 = rs_z1 = rsrc_words(Q->w[0].qzeros, 16u);
        }
        next_stream_phase();
        int issued = 0, computed = 0;  // units of this wave, over all phases
        int issue_slot = 0, comp_slot = 0;
        char *const my_ring = ring + (size_t)wave * R * UNIT_LDS_BYTES;
        const uint32_t my_ring_lds = lds_address(my_ring);
        // the next unit of this wave's sequence -> its ring slot: 8 loads of 16 bytes per lane (lane l of K step k
        // and strip v lands at slot + (4 v + k) KiB + 16 l: its own B operands of four MFMAs), the scales and the
        // zero words of both strips as a dword per lane
        auto issue_next = [&]() {
            const int u = l_u0 + li;
            const int tile = div_magic(u, l_nb, l_nb_magic);
            const int b = u - tile * l_nb;
            const int col0 = tile_col0(l_epi, tile);
            const uint32_t N = (uint32_t)l_N;
            const uint32_t s1 = (uint32_t)l_strip1;
            const uint32_t dst = my_ring_lds + (uint32_t)issue_slot * UNIT_LDS_BYTES;
            const uint32_t vw = ((uint32_t)lrow * N + 4u * lcol) * 4u;
            const uint32_t sw = ((uint32_t)(b * 16) * N + col0) * 4u;
            const uint32_t kstep = 16u * N;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                dma16(dst + k * 1024, rs_w0, vw, sw + k * kstep);
                dma16(dst + (4 + k) * 1024, rs_w1, vw + s1 * 4u, sw + k * kstep);
            }
            const int g = div_magic(b, l_bpg, l_group_magic);
            const uint32_t vs = lane < 32 ? (uint32_t)lane * 4u : OFF_RANGE;  // 2 fp16 scales per lane: 64 columns
            const uint32_t vz = lane < 8 ? (uint32_t)lane * 4u : OFF_RANGE;   // 8 zero points per lane
            const uint32_t ss = ((uint32_t)g * N + col0) * 2u;
            const uint32_t sz = ((uint32_t)g * (N >> 3) + (col0 >> 3)) * 4u;
            dma4(dst + UNIT_WORD_BYTES, rs_s0, vs, ss);
            dma4(dst + UNIT_WORD_BYTES + 256, rs_s1, vs, ss + s1 * 2u);
            dma4(dst + UNIT_WORD_BYTES + 512, rs_z0, vz, sz);
            dma4(dst + UNIT_WORD_BYTES + 768, rs_z1, vz, sz + (s1 >> 3) * 4u);
            asm volatile("" ::: "memory");
            ++issued;
            issue_slot = (issue_slot + 1 == R) ? 0 : issue_slot + 1;
            if (++li >= l_n) next_stream_phase();
        };
        if (lp < P) issue_next();
        if (tid == 0) s_sync[0] = 0u, s_sync[1] = 0u, s_sync[2] = 0u, s_ctl[2] = 0u;
        __syncthreads();  // the only workgroup barrier: the counters are zero, the helper has read the epoch and the error word
        if (s_ctl[1] != 0) return;  // an earlier launch on this workspace gave up: its state is not trustworthy

        for (int p = 0; p < P; ++p) {
            const PhasePtr C = A->ph + p;
            int U0, nwg, u0, n;
            wg_range(C, wg, U0, nwg);
            wave_range<NS>(C, wg, wave, u0, n);
            const int nb = C->nb;
            const int st_b0 = C->stage_full ? 0 : U0 - div_magic(U0, nb, C->nb_magic) * nb;
            const int T0 = div_magic(U0, nb, C->nb_magic);  // first tile of the workgroup
            // ---- until the rows of this phase are staged: keep the ring filling, one unit in flight
            for (uint32_t spin = 0; lds_load(&s_sync[0]) < (uint32_t)(p + 1); ++spin) {
                if ((spin & 7u) == 7u && aborted(poll)) return;
                if (lp < P && issued - computed < R) {
                    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                    issue_next();
                } else {
                    __builtin_amdgcn_s_sleep(2);
                }
            }
            asm volatile("" ::: "memory");
            f4_t acc[2][4];
#pragma unroll
            for (int v = 0; v < 2; ++v)
#pragma unroll
                for (int t = 0; t < 4; ++t) acc[v][t] = (f4_t){0.f, 0.f, 0.f, 0.f};
            int cur_tile = div_magic(u0, nb, C->nb_magic);
            if (lane == 0) {
                s_ft[wave] = n > 0 ? cur_tile : 0x7fffffff;
                s_lt[wave] = n > 0 ? div_magic(u0 + n - 1, nb, C->nb_magic) : -1;
            }
            // accumulators of one tile -> this wave's slot of the reduction area (rows 0..3 live in lanes 0..15)
            auto flush_tile = [&](int tile) {
                float *dst = red + ((size_t)((tile - T0) * NS + wave) * M) * 128;
                if (lane < 16) {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (e < M) {
#pragma unroll
                            for (int v = 0; v < 2; ++v)
                                *reinterpret_cast<float4 *>(dst + e * 128 + v * 64 + 4 * lcol) =
                                    make_float4(acc[v][0][e], acc[v][1][e], acc[v][2][e], acc[v][3][e]);
                        }
                }
            };
            const uint4 *xa = xs + min(lcol, M - 1) * xs_stride + lrow;
            for (int i = 0; i < n; ++i) {
                // everything issued so far has landed after this wait - unit `computed` among it; then the next
                // unit goes out, to be in flight while this one is multiplied
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                if (lp < P && issued - computed < R) issue_next();
                const int u = u0 + i;
                const int tile = div_magic(u, nb, C->nb_magic);
                if (tile != cur_tile) {
                    flush_tile(cur_tile);
#pragma unroll
                    for (int v = 0; v < 2; ++v)
#pragma unroll
                        for (int t = 0; t < 4; ++t) acc[v][t] = (f4_t){0.f, 0.f, 0.f, 0.f};
                    cur_tile = tile;
                }
                int slot = u - tile * nb - st_b0;
                if (slot < 0) slot += nb;
                const uint4 *ap = xa + slot * 16;
                const char *sb = my_ring + comp_slot * UNIT_LDS_BYTES;
                h8_t a[4];
#pragma unroll
                for (int k = 0; k < 4; ++k) a[k] = __builtin_bit_cast(h8_t, ap[4 * k]);
                ColDecode cd[2][4];
#pragma unroll
                for (int v = 0; v < 2; ++v) {
                    const uint2 sc = *reinterpret_cast<const uint2 *>(sb + UNIT_WORD_BYTES + v * 256 + lcol * 8);
                    const uint32_t zw = *reinterpret_cast<const uint32_t *>(sb + UNIT_WORD_BYTES + 512 + v * 256 + (lcol >> 1) * 4);
                    const uint32_t zs = zw >> ((lcol & 1) * 16);
#pragma unroll
                    for (int t = 0; t < 4; ++t) cd[v][t] = make_col_decode((zs >> (4 * t)) & 0xFu, ((t >> 1) ? sc.y : sc.x) >> (16 * (t & 1)));
                }
#pragma unroll
                for (int k = 0; k < 4; ++k)
#pragma unroll
                    for (int v = 0; v < 2; ++v) {
                        const uint4 w = *reinterpret_cast<const uint4 *>(sb + (4 * v + k) * 1024 + lane * 16);
                        acc[v][0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[k], decode_word_h8(w.x, cd[v][0]), acc[v][0], 0, 0, 0);
                        acc[v][1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[k], decode_word_h8(w.y, cd[v][1]), acc[v][1], 0, 0, 0);
                        acc[v][2] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[k], decode_word_h8(w.z, cd[v][2]), acc[v][2], 0, 0, 0);
                        acc[v][3] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[k], decode_word_h8(w.w, cd[v][3]), acc[v][3], 0, 0, 0);
                    }
                ++computed;
                comp_slot = (comp_slot + 1 == R) ? 0 : comp_slot + 1;
            }
            if (n > 0) flush_tile(cur_tile);
            // this wave is through with the phase: its sums are in LDS (an LDS queue is in order per wave)
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            if (lane == 0) __hip_atomic_fetch_add(&s_sync[1], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        }
        return;
    }

    // =================================================================== helper waves
    if (ht == 0) {
        // the workgroup's own epoch: every launch on this workspace moves every workgroup's on by its phase count
        s_ctl[0] = __hip_atomic_load(&st->wg_epoch[wg], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        s_ctl[1] = (uint32_t)__hip_atomic_load(&st->error, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    CHAIN_STAMP(0);
    __syncthreads();
    if (s_ctl[1] != 0) return;
    const uint32_t epoch = s_ctl[0];
    CHAIN_STAMP(1);
    const __amdgpu_buffer_rsrc_t rs_part = make_rsrc(A->partials, A->partial_bytes);

    // barrier among the helper waves (a running count of arrivals); false: somebody gave up
    uint32_t hbars = 0;
    auto helper_barrier = [&]() -> bool {
        ++hbars;
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (lane == 0) __hip_atomic_fetch_add(&s_sync[2], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        for (uint32_t spin = 0; lds_load(&s_sync[2]) < hbars * NH; ++spin)
            if ((spin & 63u) == 63u && aborted(poll)) return false;
        asm volatile("" ::: "memory");
        return true;
    };
    // all streaming waves are through with `phases` phases
    auto wait_streamers = [&](int phases) -> bool {
        for (uint32_t spin = 0; lds_load(&s_sync[1]) < (uint32_t)(phases * NS); ++spin) {
            if ((spin & 63u) == 63u && aborted(poll)) return false;
            __builtin_amdgcn_s_sleep(1);
        }
        asm volatile("" ::: "memory");
        return true;
    };

    // ------------------------------------------------------------------ outputs that must exist in memory
    // What a phase leaves behind, written by all workgroups, a slice each, right after their own partial tiles: the
    // finished values for the next phase (and y), or q, k, v with the rotary embedding applied.
    auto finish_slice = [&](int p) {
        const PhasePtr C = A->ph + p;
        const uint32_t tag = epoch + (uint32_t)p + 1u;
        if (C->out_kind != CHAIN_OUT_ROPE) {
            const int row_chunks = C->N >> 3;
            const int total = M * row_chunks;
            for (int i = wg + G * ht; i < total; i += G * TH) {  // neighbouring items go to different workgroups
                const int m = i / row_chunks, c = i - m * row_chunks;
                const uint4 v = phase_output8(C, rs_part, M, m, 8 * c, tag, poll);
                if (C->out_kind == CHAIN_OUT_ROWS) *reinterpret_cast<uint4 *>(C->y + (size_t)m * C->N + 8 * c) = v;
                if (C->feeds_next) {
                    const uint32_t off = (C->final_off + ((uint32_t)m * C->N + 8u * c) / 2u) * 8u;
                    __builtin_amdgcn_raw_buffer_store_b128((u32x4_t){v.x, tag, v.y, tag}, rs_part, off, 0, AUX_SC1);
                    __builtin_amdgcn_raw_buffer_store_b128((u32x4_t){v.z, tag, v.w, tag}, rs_part, off + 16u, 0, AUX_SC1);
                }
            }
        } else if (C->out_kind == CHAIN_OUT_ROPE) {
            // item = (row, head of q, k or v, 8 head dimensions d and their partners d + 64)
            const __attribute__((address_space(4))) RopeArgs *r = &C->rope;
            const int total = M * C->tiles * 8;
            for (int i = wg + G * ht; i < total; i += G * TH) {  // neighbouring items go to different workgroups
                const int cc = i & 7;
                const int rest = i >> 3;
                const int m = rest / C->tiles, tile = rest - m * C->tiles;
                const int first = wg_of_unit(C, tile * C->nb);
                const int nc = wg_of_unit(C, tile * C->nb + C->nb - 1) - first + 1;
                const uint32_t stride = (uint32_t)M * 128u;
                const uint32_t base = C->partial_off + ((uint32_t)tile * C->max_contrib * M + m) * 128u + 8 * cc;
                float x1[8], x2[8];
                for (uint32_t spin = 0;; ++spin) {
                    bool ok = sum_partials8(rs_part, base, stride, nc, tag, x1);
                    ok = sum_partials8(rs_part, base + 64u, stride, nc, tag, x2) && ok;
                    if (ok) break;
                    if (spin >= poll.limit || ((spin & 15u) == 15u && aborted(poll))) {
                        give_up(poll);
                        break;
                    }
                    __builtin_amdgcn_s_sleep(1);
                }
                const int d = 8 * cc;
                const int which = tile / r->H;
                const int head = tile - which * r->H;
                const int pid = r->position_ids[m];
                half_t o1[8], o2[8];
                if (which < 2) {
                    const int pos = min(max(pid, 0), r->max_pos - 1);
                    const float *ct = r->cos_table + (size_t)pos * 64 + d;
                    const float *sn = r->sin_table + (size_t)pos * 64 + d;
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        const float cs = ct[j], sv = sn[j];
                        o1[j] = (half_t)(x1[j] * cs - x2[j] * sv);
                        o2[j] = (half_t)(x2[j] * cs + x1[j] * sv);
                    }
                } else {
#pragma unroll
                    for (int j = 0; j < 8; ++j) o1[j] = (half_t)x1[j], o2[j] = (half_t)x2[j];
                }
                half_t *dst;
                size_t off;
                if (which == 0) {
                    dst = r->q;
                    off = ((size_t)m * r->H + head) * 128;  // one token per sequence: [B, H, 1, D]
                } else {
                    dst = (which == 1) ? r->k : r->v;
                    const int crow = r->kv_offset >= 0 ? r->kv_offset : min(max(pid, 0), r->kv_capacity - 1);
                    off = (((size_t)m * r->H + head) * r->kv_capacity + crow) * 128;
                }
                *reinterpret_cast<uint4 *>(dst + off + d) = pack_h8(o1);
                *reinterpret_cast<uint4 *>(dst + off + 64 + d) = pack_h8(o2);
            }
        }
    };
    // ------------------------------------------------------------------ the phases
    for (int p = 0; p < P; ++p) {
        const PhasePtr C = A->ph + p;
        CHAIN_STAMP(2 + 7 * p);
        int U0, nwg;
        wg_range(C, wg, U0, nwg);
        const int nb = C->nb;
        const uint32_t prev_tag = epoch + (uint32_t)p;  // the tag of phase p - 1

        // ---- the rows this phase multiplies with -> LDS, pair order
        // staged batches: all of them (slot = batch) or the workgroup's own, starting at batch st_b0
        const int st_b0 = C->stage_full ? 0 : U0 - div_magic(U0, nb, C->nb_magic) * nb;
        const int st_n = C->stage_full ? nb : min(nwg, nb);
        const PhasePtr Pv = A->ph + (p > 0 ? p - 1 : 0);
        if (C->in_kind == CHAIN_IN_ROWS || C->in_kind == CHAIN_IN_PREV) {
            for (int m = 0; m < M; ++m) {
                for (int i = ht; i < st_n * 16; i += TH) {
                    int b = st_b0 + (i >> 4);
                    if (b >= nb) b -= nb;
                    const int k0 = b * 128 + (i & 15) * 8;
                    uint4 v;
                    if (C->in_kind == CHAIN_IN_ROWS)
                        v = *reinterpret_cast<const uint4 *>(C->x + (size_t)m * C->K + k0);
                    else
                        v = final8(Pv, rs_part, m, k0, prev_tag, poll);
                    xs[m * xs_stride + i] = pair_order_u4(v);
                }
            }
        } else {
            // residual add + RMSNorm of whole rows.  The sum of squares is taken by the 256 helper threads over the
            // chunks t, t + 256, ... and combined as the stand-alone kernel combines it: same bits.
            const int chunks = C->K >> 3;
            const bool writer = (wg == p % G) && C->sum_out != nullptr;
            for (int m = 0; m < M; ++m) {
                for (int c = ht; c < chunks; c += TH) {
                    // the residual rows: from memory, or the sums an earlier phase of this launch left in LDS
                    uint4 v = C->x_in_launch ? keep[m * chunks + c] : *reinterpret_cast<const uint4 *>(C->x + (size_t)m * C->K + 8 * c);
                    bool added = false;
                    uint4 d = v;
                    if (C->in_kind == CHAIN_IN_NORM_PREV) {
                        d = final8(Pv, rs_part, m, 8 * c, prev_tag, poll);
                        added = true;
                    } else if (C->delta != nullptr) {
                        d = *reinterpret_cast<const uint4 *>(C->delta + (size_t)m * C->K + 8 * c);
                        added = true;
                    }
                    if (added) {
                        float unused = 0.f;
                        v = norm_take<true>(v, d, unused);
                        if (writer) *reinterpret_cast<uint4 *>(C->sum_out + (size_t)m * C->K + 8 * c) = v;
                    }
                    if (C->keep_sums) keep[m * chunks + c] = v;
                    xs[m * xs_stride + c] = v;
                }
            }
            if (!helper_barrier()) return;
            for (int m = 0; m < M; ++m) {
                float ss = 0.f;
                for (int c = ht; c < chunks; c += TH) {
                    const uint4 v = xs[m * xs_stride + c];
                    norm_take<false>(v, v, ss);
                }
                ss = norm_wave_sum(ss);
                if (lane == 0) s_part[4 * m + hw] = ss;
            }
            if (!helper_barrier()) return;
            for (int m = 0; m < M; ++m) {
                const float inv = rsqrtf((s_part[4 * m] + s_part[4 * m + 1] + s_part[4 * m + 2] + s_part[4 * m + 3]) / (float)C->K + C->eps);
                for (int c = ht; c < chunks; c += TH) {
                    const uint4 g = *reinterpret_cast<const uint4 *>(C->norm_w + 8 * c);
                    xs[m * xs_stride + c] = pair_order_u4(norm_put(xs[m * xs_stride + c], g, inv));
                }
            }
        }
        if (!helper_barrier()) return;
        if (aborted(poll)) return;
        if (ht == 0) __hip_atomic_store(&s_sync[0], (uint32_t)(p + 1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        CHAIN_STAMP(5 + 7 * p);

        // ---- when the streaming waves are through: the workgroup's partial tiles -> its slots in the workspace, each
        //      value with the phase's tag (nothing waits for these stores)
        if (!wait_streamers(p + 1)) return;
        CHAIN_STAMP(7 + 7 * p);
        if (nwg > 0 && wg != A->skip_flag_wg) {
            const uint32_t tag = epoch + (uint32_t)p + 1u;
            const int T0 = div_magic(U0, nb, C->nb_magic);
            const int T1 = div_magic(U0 + nwg - 1, nb, C->nb_magic);
            const int per_tile = M * 128;
            const int total = (T1 - T0 + 1) * per_tile;
            for (int e = ht; e < total; e += TH) {
                const int tl = e / per_tile;
                const int rem = e - tl * per_tile;
                const int tile = T0 + tl;
                float s = 0.f;
#pragma unroll
                for (int w = 0; w < NS; ++w)
                    if (s_ft[w] <= tile && tile <= s_lt[w]) s += red[(size_t)(tl * NS + w) * per_tile + rem];
                const int rank = wg - wg_of_unit(C, tile * nb);
                const uint32_t off = C->partial_off + ((uint32_t)tile * C->max_contrib + rank) * per_tile + rem;
                const u32x2_t val = {__builtin_bit_cast(uint32_t, s), tag};
                __builtin_amdgcn_raw_buffer_store_b64(val, rs_part, off * 8u, 0, AUX_SC1);
            }
        }
        CHAIN_STAMP(8 + 7 * p);
        // ---- this workgroup's slice of the finished values / outputs (waits for the other workgroups' partial tiles)
        finish_slice(p);
        CHAIN_STAMP(3 + 7 * p);
        // the reduction area, s_ft / s_lt and the staged rows are free again once every helper wave is here
        if (!helper_barrier()) return;
    }
    // the end of the launch: the workgroup's epoch moves on
    if (ht == 0 && !aborted(poll)) __hip_atomic_store(&st->wg_epoch[wg], epoch + (uint32_t)P, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (wg == 0 && ht == 0) __hip_atomic_fetch_add(&st->launches, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ---------------------------------------------------------------------------------------------- host side
struct ChainTuning {
    int ring_slots;  // units of LDS per streaming wave: 2..4 (0 = as many as fit, at most 4)
    uint32_t spin_limit;
    int skip_flag_wg;
};
ChainTuning g_chain_tuning = {0, 0, -1};

uint32_t magic_of(int d) { return d > 1 ? (uint32_t)(0x100000000ull / (unsigned)d + 1) : 0u; }

struct DeviceInfo {
    int cus;
    size_t lds_per_wg;
    bool known;
};
// number of CUs and the LDS a workgroup may use, asked once per device
int device_info(DeviceInfo *out) {
    enum { MAX_DEVICES = 64 };
    static DeviceInfo info[MAX_DEVICES];
    static std::mutex lock;
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= MAX_DEVICES) return (int)hipErrorInvalidDevice;
    std::lock_guard<std::mutex> guard(lock);
    if (!info[dev].known) {
        hipDeviceProp_t prop;
        e = hipGetDeviceProperties(&prop, dev);
        if (e != hipSuccess) return (int)e;
        info[dev].cus = prop.multiProcessorCount;
        info[dev].lds_per_wg = prop.sharedMemPerBlock;
        info[dev].known = true;
    }
    *out = info[dev];
    return 0;
}

constexpr size_t CHAIN_LDS_BUDGET = 160 * 1024 - 1024;  // dynamic LDS a workgroup may ask for (the rest: the kernel's static words)

int launch_chain(const ChainArgs &a, int grid, size_t lds, hipStream_t stream) {
    static bool prepared = false;
    static std::mutex lock;
    {
        std::lock_guard<std::mutex> guard(lock);
        if (!prepared) {
            const void *fn = reinterpret_cast<const void *>(&gptq4_chain_kernel);
            hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)CHAIN_LDS_BUDGET);
            if (e != hipSuccess) return (int)e;
            prepared = true;
        }
    }
    // the grid must be resident as a whole (workgroups wait for each other's sums): one workgroup per CU
    int per_cu = 0;
    hipError_t e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, gptq4_chain_kernel, 64 * (CHAIN_NS + CHAIN_NH), lds);
    if (e != hipSuccess) return (int)e;
    if (per_cu < 1) return (int)hipErrorLaunchOutOfResources;
    hipLaunchKernelGGL(gptq4_chain_kernel, dim3((unsigned)grid), dim3(64 * (CHAIN_NS + CHAIN_NH)), lds, stream, a);
    return (int)hipGetLastError();
}

struct ChainPlan {
    ChainArgs a;
    int grid;
    size_t lds_bytes;
    size_t partial_bytes;
    int rc;  // 0 or a negative GPTQ4_E_* code
};

int epi_of(const gptq4_phase_t &ph) {
    if (ph.up_qweight != nullptr) return EPI_SILU_MUL;
    return ph.output == GPTQ4_OUT_ROPE ? EPI_ROPE : EPI_PLAIN;
}

// Validates the phase list and lays the launch out.  `grid` = number of CUs (0: do not ask the device, plan for 256).
ChainPlan plan_chain(const gptq4_phase_t *phases, int nphases, int M, int grid) {
    ChainPlan pl = {};
    pl.rc = -GPTQ4_E_SHAPE;
    if (phases == nullptr) {
        pl.rc = -GPTQ4_E_NULL;
        return pl;
    }
    if (nphases < 1 || nphases > CHAIN_MAX_PHASES || M < 1 || M > CHAIN_MAX_M) return pl;
    if (grid <= 0) grid = 256;
    if (grid > CHAIN_MAX_GRID) grid = CHAIN_MAX_GRID;
    pl.grid = grid;
    ChainArgs &a = pl.a;
    a.nphases = nphases;
    a.M = M;
    // a poll is one round trip to memory (1 - 2 us) and a hop between phases takes a few of them: 16384 polls give up
    // within tens of milliseconds on a grid that is not fully resident (another stream holding CUs), not seconds
    a.spin_limit = g_chain_tuning.spin_limit ? g_chain_tuning.spin_limit : (1u << 14);
    a.skip_flag_wg = g_chain_tuning.skip_flag_wg;
    size_t partial_elems = 0;
    int stage_chunks = 16, red_tiles = 1, keep_chunks = 0;
    for (int p = 0; p < nphases; ++p) {
        const gptq4_phase_t &ph = phases[p];
        ChainPhase &c = a.ph[p];
        if (!ph.qweight || !ph.qzeros || !ph.scales) {
            pl.rc = -GPTQ4_E_NULL;
            return pl;
        }
        const bool pair = ph.up_qweight != nullptr;
        if (pair && (!ph.up_qzeros || !ph.up_scales)) {
            pl.rc = -GPTQ4_E_NULL;
            return pl;
        }
        int g = ph.groupsize;
        const int K = ph.K, N = ph.N;
        if (K <= 0 || N <= 0 || (K % 128) != 0 || (N % 256) != 0) return pl;
        if (g == -1) g = K;
        if (g <= 0 || (g % 128) != 0 || (K % g) != 0) {
            pl.rc = -GPTQ4_E_GROUPSIZE;
            return pl;
        }
        if ((uint64_t)K * N / 2 >= (1ull << 31) || (uint64_t)M * K * 2 >= (1ull << 31)) return pl;
        if (ph.perm != nullptr) return pl;  // act-order inputs are not taken by the chained launch
        c.epi = epi_of(ph);
        if (pair && ph.output == GPTQ4_OUT_ROPE) return pl;
        c.w[0] = QMat{reinterpret_cast<const uint32_t *>(ph.qweight), reinterpret_cast<const uint32_t *>(ph.qzeros),
                      reinterpret_cast<const half_t *>(ph.scales)};
        c.w[1] = pair ? QMat{reinterpret_cast<const uint32_t *>(ph.up_qweight), reinterpret_cast<const uint32_t *>(ph.up_qzeros),
                             reinterpret_cast<const half_t *>(ph.up_scales)}
                      : c.w[0];
        c.K = K, c.N = N, c.nb = K / 128;
        c.tiles = pair ? N / 64 : N / 128;
        c.bpg = g / 128, c.groups = K / g;
        c.group_magic = magic_of(c.bpg), c.nb_magic = magic_of(c.nb);
        const long units = (long)c.tiles * c.nb;
        if (units >= (1L << 24)) return pl;
        c.q = (int)(units / grid), c.r = (int)(units % grid);
        c.q_magic = magic_of(c.q), c.q1_magic = magic_of(c.q + 1);
        c.max_contrib = c.q > 0 ? (c.nb + c.q - 1) / c.q + 1 : c.nb;
        if (c.max_contrib > c.nb) c.max_contrib = c.nb;
        if (c.max_contrib > grid) c.max_contrib = grid;
        // ---- input
        c.in_kind = ph.input;
        c.eps = ph.eps;
        c.x = reinterpret_cast<const half_t *>(ph.x);
        c.delta = reinterpret_cast<const half_t *>(ph.delta);
        c.norm_w = reinterpret_cast<const half_t *>(ph.norm_weight);
        c.sum_out = reinterpret_cast<half_t *>(ph.sum_out);
        c.bias = reinterpret_cast<const half_t *>(ph.bias);
        const bool norm = ph.input == GPTQ4_IN_NORM_ROWS || ph.input == GPTQ4_IN_NORM_PREV;
        const bool from_prev = ph.input == GPTQ4_IN_PREV || ph.input == GPTQ4_IN_NORM_PREV;
        if (ph.input < GPTQ4_IN_ROWS || ph.input > GPTQ4_IN_NORM_PREV) return pl;
        if (from_prev) {
            if (p == 0) return pl;
            const gptq4_phase_t &pv = phases[p - 1];
            if (pv.N != K || pv.output == GPTQ4_OUT_ROPE) return pl;             // the previous output is this phase's input row
            if (ph.input == GPTQ4_IN_NORM_PREV && pv.up_qweight != nullptr) return pl;  // a residual add takes a plain projection
        }
        if (ph.input != GPTQ4_IN_PREV && !ph.x) {
            pl.rc = -GPTQ4_E_NULL;
            return pl;
        }
        if (norm) {
            if (!ph.norm_weight) {
                pl.rc = -GPTQ4_E_NULL;
                return pl;
            }
            if (K > 8192 || !(ph.eps >= 0.f)) return pl;
            if (ph.sum_out != nullptr && (ph.sum_out == ph.x || ph.sum_out == ph.delta)) return pl;  // other workgroups still read them
            // the residual rows may be the sums an earlier phase of this launch wrote: only the latest such sums are
            // at hand (every workgroup keeps them in LDS; the copy in memory is not complete before the launch ends)
            int last_norm = -1;
            for (int e = 0; e < p; ++e) {
                const bool e_norm = phases[e].input == GPTQ4_IN_NORM_ROWS || phases[e].input == GPTQ4_IN_NORM_PREV;
                if (e_norm) last_norm = e;
            }
            for (int e = 0; e < p; ++e) {
                if (phases[e].sum_out == nullptr || phases[e].sum_out != ph.x) continue;
                if (e != last_norm || phases[e].K != K) return pl;
                c.x_in_launch = 1;
                a.ph[e].keep_sums = 1;
                if (K / 8 > keep_chunks) keep_chunks = K / 8;
            }
        }
        c.stage_full = norm ? 1 : 0;
        const int per_wg = c.q + (c.r ? 1 : 0);
        const int staged = (norm || per_wg >= c.nb) ? c.nb : per_wg;
        if (staged * 16 > stage_chunks) stage_chunks = staged * 16;
        const int touched = (per_wg + c.nb - 1) / c.nb + 1;
        if (touched > red_tiles) red_tiles = touched;
        // ---- output
        c.out_kind = ph.output;
        if (ph.output < GPTQ4_OUT_NONE || ph.output > GPTQ4_OUT_ROPE) return pl;
        if (ph.output == GPTQ4_OUT_ROWS) {
            if (!ph.y) {
                pl.rc = -GPTQ4_E_NULL;
                return pl;
            }
            c.y = reinterpret_cast<half_t *>(ph.y);
        } else if (ph.output == GPTQ4_OUT_ROPE) {
            if (!ph.position_ids || !ph.cos_table || !ph.sin_table || !ph.q || !ph.k || !ph.v) {
                pl.rc = -GPTQ4_E_NULL;
                return pl;
            }
            if (ph.H < 1 || N != 3 * ph.H * 128 || ph.max_pos < 1 || ph.kv_capacity < 1 || ph.kv_offset < GPTQ4_KV_AT_POSITION ||
                (ph.kv_offset >= 0 && ph.kv_capacity < ph.kv_offset + 1))
                return pl;
            c.rope.position_ids = ph.position_ids;
            c.rope.cos_table = ph.cos_table, c.rope.sin_table = ph.sin_table;
            c.rope.q = reinterpret_cast<half_t *>(ph.q), c.rope.k = reinterpret_cast<half_t *>(ph.k), c.rope.v = reinterpret_cast<half_t *>(ph.v);
            c.rope.S = 1, c.rope.H = ph.H, c.rope.kv_capacity = ph.kv_capacity, c.rope.kv_offset = ph.kv_offset, c.rope.max_pos = ph.max_pos;
        } else if (p + 1 == nphases || (phases[p + 1].input != GPTQ4_IN_PREV && phases[p + 1].input != GPTQ4_IN_NORM_PREV)) {
            return pl;  // a phase nobody reads and that leaves nothing in memory
        }
        if (ph.bias != nullptr && pair) return pl;
        c.partial_off = (uint32_t)partial_elems;
        partial_elems += (size_t)c.tiles * c.max_contrib * M * 128;
        c.feeds_next = (p + 1 < nphases && (phases[p + 1].input == GPTQ4_IN_PREV || phases[p + 1].input == GPTQ4_IN_NORM_PREV)) ? 1 : 0;
        c.final_off = (uint32_t)partial_elems;
        if (c.feeds_next) partial_elems += (size_t)M * N / 2;
        if (partial_elems * 8 >= (1ull << 31)) return pl;
    }
    pl.partial_bytes = partial_elems * 8;  // {fp32 bits, tag} per value
    a.partial_bytes = (uint32_t)pl.partial_bytes;
    // LDS: [M rows of staged activations][kept residual sums][reduction area]; rows 64 bytes apart modulo 128 so that two rows'
    // A-operand reads fall into different banks
    int stride = stage_chunks;
    if ((stride & 7) != 4) stride += (4 - (stride & 7) + 8) & 7;
    a.xs_stride = stride;
    a.keep_off = M * stride;
    a.red_off = a.keep_off + M * keep_chunks;
    a.red_tiles = red_tiles;
    const size_t red_bytes = (size_t)red_tiles * CHAIN_NS * M * 128 * sizeof(float);
    a.ring_off = a.red_off + (int)(red_bytes / 16);
    const size_t fixed = (size_t)a.ring_off * 16;
    // the ring takes what is left: 2 slots per streaming wave at least (one in flight, one being multiplied), up to 4
    int slots = 4;
    if (g_chain_tuning.ring_slots >= 2 && g_chain_tuning.ring_slots <= 4) slots = g_chain_tuning.ring_slots;
    while (slots > 2 && fixed + (size_t)slots * CHAIN_NS * UNIT_LDS_BYTES > CHAIN_LDS_BUDGET) --slots;
    a.ring_slots = slots;
    pl.lds_bytes = fixed + (size_t)slots * CHAIN_NS * UNIT_LDS_BYTES;
    if (pl.lds_bytes > CHAIN_LDS_BUDGET) return pl;
    // more than half of a CU's 160 KiB: no CU can take two workgroups, so the grid spreads over all CUs
    if (pl.lds_bytes < 84 * 1024) pl.lds_bytes = 84 * 1024;
    pl.rc = 0;
    return pl;
}

}  // namespace

extern "C" {

void gptq4_set_chain_tuning(int ring_slots, int reserved, unsigned spin_limit, int skip_flag_wg) {
    (void)reserved;
    g_chain_tuning.ring_slots = (ring_slots >= 2 && ring_slots <= 4) ? ring_slots : 0;
    g_chain_tuning.spin_limit = spin_limit;
    g_chain_tuning.skip_flag_wg = skip_flag_wg;
}

size_t gptq4_chain_workspace_bytes(const gptq4_phase_t *phases, int nphases, int M) {
    DeviceInfo di = {};
    const int grid = device_info(&di) == 0 ? di.cus : 0;
    const ChainPlan pl = plan_chain(phases, nphases, M, grid);
    if (pl.rc != 0) return 0;
#ifdef GPTQ4_CHAIN_TIMERS
    return (size_t)CHAIN_STATE_BYTES + pl.partial_bytes + (1u << 20);
#else
    return (size_t)CHAIN_STATE_BYTES + pl.partial_bytes;
#endif
}

int gptq4_decode_chain(const gptq4_phase_t *phases, int nphases, int M, void *workspace, size_t workspace_bytes, void *stream) {
    // argument errors first: they need no device
    ChainPlan pl = plan_chain(phases, nphases, M, 0);
    if (pl.rc != 0) return pl.rc;
    DeviceInfo di = {};
    int rc = device_info(&di);
    if (rc) return rc;
    pl = plan_chain(phases, nphases, M, di.cus);
    if (pl.rc != 0) return pl.rc;
    if (workspace == nullptr || workspace_bytes < (size_t)CHAIN_STATE_BYTES + pl.partial_bytes) return -GPTQ4_E_WORKSPACE;
    if ((reinterpret_cast<uintptr_t>(workspace) & 255u) != 0) return -GPTQ4_E_ALIGN;
    for (int p = 0; p < nphases; ++p) {
        const gptq4_phase_t &ph = phases[p];
        const void *ptrs[] = {ph.qweight, ph.scales, ph.up_qweight, ph.up_scales, ph.x, ph.delta, ph.norm_weight, ph.sum_out,
                              ph.y, ph.bias, ph.q, ph.k, ph.v, ph.cos_table, ph.sin_table};
        for (const void *q : ptrs)
            if (q != nullptr && (reinterpret_cast<uintptr_t>(q) & 15u) != 0) return -GPTQ4_E_ALIGN;
    }
    pl.a.state = reinterpret_cast<ChainState *>(workspace);
    pl.a.partials = reinterpret_cast<float *>(reinterpret_cast<char *>(workspace) + CHAIN_STATE_BYTES);
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    return launch_chain(pl.a, pl.grid, pl.lds_bytes, s);
}

}  // extern "C"
