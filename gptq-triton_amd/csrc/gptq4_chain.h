// Host/device contract of the chained decode launch (gptq4_chain.hip): a list of small-M quantised
// projections ("phases") that one persistent launch runs back to back, each phase reading either rows
// that were in memory before the launch or what the phase before it produced.
#pragma once

#include "gptq4_internal.h"

enum { CHAIN_MAX_PHASES = 8, CHAIN_MAX_M = 4, CHAIN_MAX_GRID = 1024, CHAIN_STATE_BYTES = 8192 };

// what a phase multiplies with
enum {
    CHAIN_IN_ROWS = 0,       // x: fp16 rows in memory before the launch
    CHAIN_IN_NORM_ROWS = 1,  // norm_weight * rmsnorm(x (+ delta)); x, delta in memory before the launch
    CHAIN_IN_PREV = 2,       // the output of the phase before: fp16(sums) of a plain phase, fp16(silu(gate) * up) of a pair
    CHAIN_IN_NORM_PREV = 3,  // norm_weight * rmsnorm(x + fp16(sums of the plain phase before))
};
// what a phase leaves in memory (on top of feeding the next phase)
enum { CHAIN_OUT_NONE = 0, CHAIN_OUT_ROWS = 1, CHAIN_OUT_ROPE = 2 };

struct ChainPhase {
    QMat w[2];  // w[1]: the up matrix of a gate/up pair (EPI_SILU_MUL)
    const half_t *x;         // IN_ROWS / IN_NORM_ROWS: [M, K]; IN_NORM_PREV: the residual rows [M, K] (may be an earlier phase's sum_out)
    const half_t *delta;     // IN_NORM_ROWS, nullable
    const half_t *norm_w;    // IN_NORM_*: [K]
    half_t *sum_out;         // IN_NORM_* with something added: x + delta / x + previous output, [M, K]; nullable
    half_t *y;               // OUT_ROWS: [M, N] (plain: sums (+ bias); pair: silu(gate) * up)
    const half_t *bias;      // plain OUT_ROWS / IN_PREV of the next phase, nullable
    RopeArgs rope;           // OUT_ROPE
    float eps;
    int epi;                 // EPI_PLAIN, EPI_SILU_MUL, EPI_ROPE: which strips make a tile
    int in_kind, out_kind;
    int x_in_launch;         // IN_NORM_PREV: x is the sum_out of the last norm phase before this one: taken from the copy in LDS
    int keep_sums;           // IN_NORM_*: a later phase reads this phase's sums as its x: keep them in LDS
    int K, N;                // N: columns of one matrix
    int nb;                  // K / 128
    int tiles;               // plain: N / 128; pair: N / 64 (64 columns of gate + the same 64 of up); rotary: N / 128 (one head: d and d + 64)
    int bpg, groups;         // batches per group, groups
    uint32_t group_magic, nb_magic;
    // units (tile, batch) dealt to workgroups: q each, the first r one more
    int q, r;
    uint32_t q_magic, q1_magic;
    int max_contrib;         // workgroups that can share one tile
    int stage_full;          // 1: the whole row is staged in LDS (slot = batch), 0: only the workgroup's batches
    uint32_t partial_off;    // this phase's partial sums: element offset ({fp32 bits, tag} pairs) into the partial region
    uint32_t final_off;      // its finished values for the next phase: element offset ({2 fp16, tag}), M * N / 2 elements
    int feeds_next;          // the next phase reads this one's output
};

// Persistent state in the chain workspace (zero before the first launch; launches maintain it).
struct ChainState {
    uint32_t launches;  // launches completed on this workspace (informational)
    int32_t error;      // 0, or CHAIN_ERR_* of the first launch that gave up (sticky: later launches return at once)
    uint32_t pad[30];
    uint32_t wg_epoch[CHAIN_MAX_GRID];  // per workgroup: phases of all earlier launches; phase p of a launch tags its sums epoch + p + 1
};
enum { CHAIN_ERR_TIMEOUT = 1 };

struct ChainArgs {
    ChainPhase ph[CHAIN_MAX_PHASES];
    ChainState *state;
    float *partials;
    uint32_t partial_bytes;
    int nphases;
    int M;
    int xs_stride;     // 16-byte chunks per staged row (LDS)
    int keep_off;      // LDS offset (chunks) of the residual sums kept for a later phase
    int red_off;       // LDS offset (chunks) of the reduction area
    int ring_off;      // LDS offset (chunks) of the streaming waves' unit ring
    int ring_slots;    // units per streaming wave in that ring (>= 2)
    int red_tiles;     // tiles a workgroup can touch in one phase
    uint32_t spin_limit;  // polls of a partial tile before a thread gives up
    int skip_flag_wg;     // test hook: this workgroup never stores its partial sums (-1: none)
};

static_assert(sizeof(ChainState) <= CHAIN_STATE_BYTES, "state region");
static_assert(sizeof(ChainArgs) <= 4096, "kernel arguments are passed by value");
