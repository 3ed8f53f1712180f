// C ABI of the library (declared in include/gptq4.h): argument validation on the
// host, then one kernel launch on the caller's stream.  No allocation, no
// synchronisation, no exceptions.
#include "../../include/gptq4.h"
#include "../../include/gptq4_experimental.h"

#include "gptq4_internal.h"
#include "gptq4_norm.h"

#include <mutex>

// Scratch memory of gptq4_matmul_static: arrival counters, then split-K partial sums, laid out like a
// caller's workspace.  Zero when the module is loaded; every launch leaves the counters zero again.
// In host code this name is only a handle for hipGetSymbolAddress: the kernels get the device address.
static __device__ __align__(256) unsigned char scratch[GPTQ4_STATIC_SCRATCH_BYTES];

namespace {

inline bool misaligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) != 0; }

// groupsize: -1 -> K.  Accepts what the reference accepts (quant_linear.py:244-257).
int check_dims(int K, int N, int *groupsize) {
    if (K <= 0 || N <= 0 || (K % 128) != 0 || (N % 256) != 0) return -GPTQ4_E_SHAPE;
    int g = *groupsize;
    if (g == -1) g = K;
    if (g <= 0 || (g % 128) != 0 || (K % g) != 0) return -GPTQ4_E_GROUPSIZE;
    *groupsize = g;
    return 0;
}

size_t partial_bytes(int splitk, int M, int ncols_total) {
    return (size_t)splitk * (size_t)M * (size_t)ncols_total * sizeof(float);
}

// Fill the split-K fields of `a` from the launch plan; `nmat` = matrices summed per
// tile (2 for the gate/up pair).
int setup_skinny(MatmulArgs &a, const SkinnyPlan &pl, int nmat, void *workspace, size_t workspace_bytes) {
    a.tiles = pl.tiles;
    a.splitk = pl.splitk;
    const int nbatches = a.K / 128, slots = pl.splitk * pl.waves;
    a.slot_q = nbatches / slots;
    a.slot_rem = nbatches % slots;
    a.batches_per_group = a.groupsize / 128;
    if (a.tiles > SKINNY_MAX_TILES) return -GPTQ4_E_SHAPE;
    if (workspace == nullptr || workspace_bytes < GPTQ4_WS_HEAD_BYTES) return -GPTQ4_E_WORKSPACE;
    if (a.splitk > 1 && workspace_bytes < GPTQ4_WS_HEAD_BYTES + partial_bytes(a.splitk, a.M, nmat * a.N))
        return -GPTQ4_E_WORKSPACE;
    a.counters = reinterpret_cast<int *>(workspace);
    a.partials = reinterpret_cast<float *>(reinterpret_cast<char *>(workspace) + GPTQ4_WS_HEAD_BYTES);
    // The exchange through marked 8-byte values where it is the faster one - up to 4 rows, and few enough splits
    // for the finishing workgroup to poll them all in one round (16 loads per thread: 8, 4 or 2 splits by the
    // values a thread holds) - and the values fit their region of the head; else arrival counters and plain
    // partial sums.  Measured at LLaMA-7B / 30B shapes: QKV 11.5 -> 10.9 / 24.4 -> 21.8 us at one row, o_proj and
    // down_proj 0.1 - 0.2 us ahead, but behind the counters from 8 rows on (gate/up 18.5 -> 19.4 us) and with 15
    // splits to poll (30B down_proj 18.9 -> 19.8 us).
    a.tagged = nullptr;
    const int per_thread = pl.words * nmat * (nmat == 1 && a.rope.q != nullptr ? 2 : 1);  // values a finishing thread holds per row block
    const int round = per_thread >= 8 ? 2 : (per_thread >= 4 ? 4 : 8);
    const bool marked = g_skinny_tuning.exchange == 2 || (g_skinny_tuning.exchange == 0 && a.M <= 4 && a.splitk - 1 <= round);
    if (a.splitk > 1 && marked && 2 * partial_bytes(a.splitk, a.M, nmat * a.N) <= GPTQ4_WS_TAGGED_BYTES)
        a.tagged = reinterpret_cast<uint64_t *>(reinterpret_cast<char *>(workspace) + GPTQ4_WS_COUNTER_BYTES);
    a.spin_limit = g_gemv_tuning.spin_limit ? g_gemv_tuning.spin_limit : (1u << 22);
    return 0;
}

// Act-order: gather the M rows of x into the workspace behind the partial sums (one small launch) and hand
// the kernel plain activations.  A kernel's own gather reads single 2-byte values, each a cache line to the
// texture path, and repeats that for every column tile: 3.5 us at one row, twice the time of the whole call
// at eight rows, +43 % for a 2048-row down_proj.
int stage_act_order(MatmulArgs &a, size_t partial_bytes_used, void *workspace, size_t workspace_bytes, hipStream_t s) {
    const size_t off = GPTQ4_WS_HEAD_BYTES + partial_bytes_used;
    const size_t bytes = (size_t)a.M * a.K * sizeof(half_t);
    if (workspace == nullptr || workspace_bytes < off + bytes) return -GPTQ4_E_WORKSPACE;
    // rows longer than 32768 values are gathered with the row index in grid.y, which ends at 65535
    if (a.M > 65535 && a.K > 32768) return -GPTQ4_E_SHAPE;
    half_t *xg = reinterpret_cast<half_t *>(reinterpret_cast<char *>(workspace) + off);
    const int rc = launch_gather_cols(a.x, a.perm, xg, a.M, a.K, s);
    a.x = xg;
    a.perm = nullptr;
    return rc;
}

// M <= 16: the balanced GEMV where its plan says so (by default the one-row gate/up pair),
// the split-K kernel otherwise.
int run_small(int epi, MatmulArgs &a, int nmat, void *workspace, size_t workspace_bytes, hipStream_t s) {
    if (a.nrm_weight != nullptr) {
        // the variants that normalise their own input exist for the automatic launch shapes only
        if (a.M <= GEMV_MAX_M) {
            const GemvPlan gp = gemv_plan(epi, a.M, a.N, a.K, true);
            if (gp.ok) {
                if (workspace == nullptr || workspace_bytes < GPTQ4_WS_HEAD_BYTES) return -GPTQ4_E_WORKSPACE;
                a.counters = reinterpret_cast<int *>(workspace);
                a.tagged = reinterpret_cast<uint64_t *>(reinterpret_cast<char *>(workspace) + GPTQ4_WS_COUNTER_BYTES);
                return launch_gemv(epi, a, gp, s);
            }
        }
        const SkinnyPlan pl = skinny_plan(epi, a.M, a.N, a.K, true);
        int rc = setup_skinny(a, pl, nmat, workspace, workspace_bytes);
        if (rc) return rc;
        return launch_skinny(epi, a, pl, s);
    }
    if (a.M <= GEMV_MAX_M) {
        const GemvPlan pl = gemv_plan(epi, a.M, a.N, a.K);
        if (pl.ok) {
            if (workspace == nullptr || workspace_bytes < GPTQ4_WS_HEAD_BYTES) return -GPTQ4_E_WORKSPACE;
            a.counters = reinterpret_cast<int *>(workspace);
            a.tagged = reinterpret_cast<uint64_t *>(reinterpret_cast<char *>(workspace) + GPTQ4_WS_COUNTER_BYTES);
            return launch_gemv(epi, a, pl, s);
        }
    }
    const SkinnyPlan pl = skinny_plan(epi, a.M, a.N, a.K);
    int rc = setup_skinny(a, pl, nmat, workspace, workspace_bytes);
    if (rc) return rc;
    if (a.perm != nullptr) {
        rc = stage_act_order(a, a.splitk > 1 ? partial_bytes(a.splitk, a.M, nmat * a.N) : 0, workspace, workspace_bytes, s);
        if (rc) return rc;
    }
    return launch_skinny(epi, a, pl, s);
}

// Fill the split-K fields of `a` for the tiled kernel.
int setup_gemm(int epi, MatmulArgs &a, const GemmPlan &pl, void *workspace, size_t workspace_bytes) {
    a.tiles = pl.tiles;
    a.splitk = pl.splitk;
    const int nk = a.K / 64;
    a.slot_q = nk / pl.splitk;
    a.slot_rem = nk % pl.splitk;
    a.tail_first = pl.tail_first;
    a.tail_split = pl.tail_split;
#ifdef GPTQ4_PHASE_TIMERS
    // (development build: the phase stamps go 32 MiB into the workspace, also of launches that exchange nothing)
    if (workspace != nullptr && workspace_bytes >= (size_t)(33 << 20)) a.counters = reinterpret_cast<int *>(workspace);
#endif
    // the tiles cut along K are the last column panels: the whole tiles cover the columns before them
    if (pl.tail_split > 1) a.n_count = (pl.tail_first / ((a.M + 127) / 128)) * ((epi == EPI_SILU_MUL) ? 128 : 256);
    if (pl.splitk > 1 || pl.streamed || pl.tail_split > 1) {
        if (workspace == nullptr || workspace_bytes < GPTQ4_WS_HEAD_BYTES + gemm_partial_bytes(pl))
            return -GPTQ4_E_WORKSPACE;
        a.counters = reinterpret_cast<int *>(workspace);
        a.partials = reinterpret_cast<float *>(reinterpret_cast<char *>(workspace) + GPTQ4_WS_HEAD_BYTES);
    }
    return 0;
}

// Fused residual add + RMSNorm of the input: decode-sized calls only (the workgroups of the small-M
// kernel each normalise all M rows into their LDS), and a sum_out that no workgroup still reads from.
int setup_norm(MatmulArgs &a, const void *delta, const void *norm_weight, void *sum_out, float eps) {
    if (!norm_weight || (delta && !sum_out)) return -GPTQ4_E_NULL;
    if (a.M > NORM_MAX_M || a.K > NORM_MAX_H || !(eps >= 0.f)) return -GPTQ4_E_SHAPE;
    if (delta && (sum_out == static_cast<const void *>(a.x) || sum_out == delta)) return -GPTQ4_E_SHAPE;
    if (misaligned16(norm_weight) || (delta && (misaligned16(delta) || misaligned16(sum_out)))) return -GPTQ4_E_ALIGN;
    a.nrm_delta = reinterpret_cast<const half_t *>(delta);
    a.nrm_weight = reinterpret_cast<const half_t *>(norm_weight);
    a.nrm_sum_out = delta ? reinterpret_cast<half_t *>(sum_out) : nullptr;
    a.nrm_eps = eps;
    return 0;
}

// M > 16: the mid-M kernel where it is the faster one, else the tiled kernel.  Measured at LLaMA-7B /
// 13B / 30B shapes, 256..768 rows: the tiled kernel takes over once it has enough wide tiles (72 for a plain
// projection, 160 for the gate/up pair, more than 192 with the rotary epilogue: LLaMA-7B QKV at 512 rows, 192 tiles, 75 -> 68 us).
// (Tile counts just over one per CU used to stay with the mid-M kernel for the rotary epilogue; since the tiled kernel
// cuts the panels past a whole round along K it is ahead there too: 7B QKV at 768 rows 93.5 against 101.6 us, 13B at
// 640 rows 110.4 against 123.4.)
bool prefer_kslice(const KslicePlan &kp, int epi, int M, int N, int K) {
    if (!kp.ok || g_kslice_tuning.mode == 0) return false;
    if (g_kslice_tuning.mode == 2) return true;
    if (M > 768) return false;
    const int wide_bn = (epi == EPI_SILU_MUL) ? 128 : 256;
    const long wide = (long)((M + 127) / 128) * (N / wide_bn);
    const long cus = device_shape().cus;  // the crossovers were measured on 256 CUs: 72, 160 and 192 wide tiles
    if (epi == EPI_PLAIN) return wide < 9 * cus / 32;
    // (gate/up at 129 .. 192 rows: the tiled kernel's second row tile is at most half full - a quarter or more of its
    // work is padding - while the mid-M kernel's 64-row tiles fit: 17920 x 6656 at 192 rows 148 against 114 us, 280 wide
    // tiles; 11008 x 4096 57.2 against 54.4; 13824 x 5120 level; 22016 x 8192 172 against 158; 28672 x 8192 214 against 205)
    if (epi == EPI_SILU_MUL && M > 128 && M <= 192) return true;
    if (epi == EPI_SILU_MUL) return wide < 5 * cus / 8;
    return wide <= 3 * cus / 4;
}

// Which kernel computes columns [.., .. + n) of an M > 16 call, with what plan, and the partial sums it exchanges.
struct TiledChoice {
    bool kslice;
    KslicePlan kp;
    GemmPlan gp;
    size_t partial;
};

TiledChoice choose_tiled(int epi, int M, int n, int K, bool kernel_gathers, bool allow_streamed = true) {
    TiledChoice c = {};
    c.kp = kslice_plan(epi, M, n, K, kernel_gathers);
    c.kslice = prefer_kslice(c.kp, epi, M, n, K);
    c.gp = gemm_plan(epi, M, n, K, kernel_gathers, allow_streamed);
    c.partial = c.kslice ? kslice_partial_bytes(epi, c.kp) : gemm_partial_bytes(c.gp);
    return c;
}

// An M > 16 call as one launch or as two launches over adjacent column ranges.  Whole wide tiles are dealt one per
// CU and round; a count just above a multiple of the CU count leaves most CUs idle for a whole round (344 tiles of
// the LLaMA-7B gate/up pair at 512 rows: 88 CUs work through two tiles, 168 through one; 516 at 768 rows: four CUs
// take a third).  Then the columns of the full rounds go to one launch of wide tiles and the remaining columns to a
// second launch that is planned by itself - narrower tiles, a K split or the mid-M kernel spread the remainder over
// the chip.  Nothing is exchanged between the two: they write different columns.
struct ColumnParts {
    int count;
    int begin[2], cols[2];
    bool first_is_wide;  // part 0 runs wide unsplit tiles whatever its own plan would say
};

ColumnParts tiled_parts(int epi, int M, int N, int K, bool kernel_gathers) {
    ColumnParts parts = {1, {0, 0}, {N, 0}, false};
    if (g_gemm_tuning.parts == 1 || g_gemm_tuning.mt != 0 || g_gemm_tuning.splitk != 0 || g_gemm_tuning.streamed == 2 || g_kslice_tuning.mode == 2)
        return parts;
    const TiledChoice whole = choose_tiled(epi, M, N, K, kernel_gathers);
    if (whole.kslice || whole.gp.mt != 4 || whole.gp.splitk != 1 || whole.gp.streamed || whole.gp.tail_split > 1) return parts;
    const long cus = device_shape().cus;
    const int bnw = (epi == EPI_SILU_MUL) ? 128 : 256;  // output columns of a wide tile
    const long tiles_m = (M + 127) / 128, tiles_n = N / bnw, tiles = tiles_m * tiles_n;
    const long rest = tiles % cus;
    // From one full round on, and only for a small remainder (up to an eighth of a round).  A second launch costs
    // 30 - 50 us at K = 4096 however little it computes, a round of wide tiles 55 - 75 us: LLaMA-7B gate/up at 384
    // rows (258 tiles) 108 -> 89 us, at 768 rows (516) 167 -> 143, at 1536 rows (1032) 283 -> 269; with 88 tiles left
    // over (512 rows) the two launches take what the one took, with 128 (QKV at 1024 rows) 7 % more.
    if (tiles <= cus || tiles > 8 * cus || rest == 0 || 8 * rest > cus || K < 2048) return parts;
    const long cols_a = (tiles - rest) / tiles_m;  // column tiles of the full rounds
    if (cols_a < 1 || cols_a >= tiles_n) return parts;
    parts.count = 2;
    parts.first_is_wide = true;
    parts.begin[0] = 0;
    parts.cols[0] = (int)(cols_a * bnw);
    parts.begin[1] = parts.cols[0];
    parts.cols[1] = N - parts.cols[0];
    return parts;
}

TiledChoice choose_part(int epi, int M, int K, const ColumnParts &parts, int i, bool kernel_gathers, bool allow_streamed = true) {
    if (i == 0 && parts.first_is_wide) {
        TiledChoice c = {};
        c.kslice = false;
        c.gp.mt = 4;
        c.gp.splitk = 1;
        c.gp.score = 1.0;
        c.gp.streamed = 0;
        c.gp.tail_first = 0;
        c.gp.tail_split = 1;
        c.gp.tiles = ((M + 127) / 128) * (parts.cols[0] / ((epi == EPI_SILU_MUL) ? 128 : 256));
        c.partial = 0;
        return c;
    }
    return choose_tiled(epi, M, parts.cols[i], K, kernel_gathers, allow_streamed);
}

int run_tiled(int epi, MatmulArgs &a, void *workspace, size_t workspace_bytes, hipStream_t s) {
    // act-order: staged activations wherever they fit the staging limit and the workspace (then the mid-M
    // kernel can run too); else the tiled kernel gathers by itself
    const size_t rows_bytes = (size_t)a.M * a.K * sizeof(half_t);
    bool stage = a.perm != nullptr && !g_gemm_tuning.own_gather && rows_bytes <= ACT_ORDER_STAGE_MAX;
    ColumnParts parts;
    TiledChoice choice[2];
    size_t partial = 0;
    bool allow_streamed = true;
    auto plan_all = [&]() {
        const bool kernel_gathers = a.perm != nullptr && !stage;
        parts = tiled_parts(epi, a.M, a.N, a.K, kernel_gathers);
        partial = 0;
        for (int i = 0; i < parts.count; ++i) {
            choice[i] = choose_part(epi, a.M, a.K, parts, i, kernel_gathers, allow_streamed);
            if (choice[i].partial > partial) partial = choice[i].partial;
        }
    };
    plan_all();
    // the streamed schedule keeps 128 MiB of partial sums: without the room for them, the unstreamed plan
    if (parts.count == 1 && !choice[0].kslice && choice[0].gp.streamed &&
        (workspace == nullptr || workspace_bytes < GPTQ4_WS_HEAD_BYTES + partial + (stage ? rows_bytes : 0))) {
        allow_streamed = false;
        plan_all();
    }
    if (stage && (workspace == nullptr || workspace_bytes < GPTQ4_WS_HEAD_BYTES + partial + rows_bytes)) {
        stage = false;
        plan_all();
    }
    if (partial > 0 && (workspace == nullptr || workspace_bytes < GPTQ4_WS_HEAD_BYTES + partial)) return -GPTQ4_E_WORKSPACE;
    if (stage) {
        // once, behind the largest partial-sum region any part uses
        const int rc = stage_act_order(a, partial, workspace, workspace_bytes, s);
        if (rc) return rc;
    }
    for (int i = 0; i < parts.count; ++i) {
        a.n_begin = parts.begin[i];
        a.n_count = parts.cols[i];
        const TiledChoice &c = choice[i];
        int rc;
        if (c.kslice) {
            a.tiles = c.kp.tiles;
            a.splitk = c.kp.splitk;
            const int nk = a.K / 64;
            a.slot_q = nk / c.kp.splitk;
            a.slot_rem = nk % c.kp.splitk;
            a.tail_first = c.kp.tail_first;
            a.tail_split = c.kp.tail_split;
            if (c.kp.splitk > 1 || c.kp.tail_split > 1) {
                a.counters = reinterpret_cast<int *>(workspace);
                a.partials = reinterpret_cast<float *>(reinterpret_cast<char *>(workspace) + GPTQ4_WS_HEAD_BYTES);
            }
#ifdef GPTQ4_PHASE_TIMERS
            if (workspace != nullptr && workspace_bytes >= (size_t)(33 << 20)) a.counters = reinterpret_cast<int *>(workspace);
#endif
            rc = launch_kslice(epi, a, c.kp, s);
        } else {
            rc = setup_gemm(epi, a, c.gp, workspace, workspace_bytes);
            if (rc) return rc;
            rc = launch_gemm(epi, a, c.gp, s);
        }
        if (rc) return rc;
    }
    return 0;
}

}  // namespace

extern "C" {

int gptq4_abi_version(void) { return GPTQ4_ABI_VERSION; }

const char *gptq4_strerror(int code) {
    if (code == 0) return "success";
    if (code > 0) return hipGetErrorString((hipError_t)code);
    switch (-code) {
        case GPTQ4_E_NULL:
            return "a required pointer is NULL";
        case GPTQ4_E_SHAPE:
            return "unsupported shape (need K % 128 == 0, N % 256 == 0, M >= 1, head_dim == 128)";
        case GPTQ4_E_GROUPSIZE:
            return "groupsize must be -1, K, or a multiple of 128 dividing K";
        case GPTQ4_E_WORKSPACE:
            return "workspace is NULL or too small (see gptq4_workspace_bytes)";
        case GPTQ4_E_EXCHANGE:
            return "a kernel's bounded wait for another workgroup's partial sums ran out: results of that call are invalid";
        case GPTQ4_E_ALIGN:
            return "a pointer is not 16-byte aligned";
        case GPTQ4_E_STATIC_LIMIT:
            return "the call needs more scratch memory than gptq4_matmul_static holds (GPTQ4_STATIC_SCRATCH_BYTES): use gptq4_matmul with a workspace";
        default:
            return "unknown gptq4 error";
    }
}

void gptq4_set_gemm_tuning(int mt, int splitk) {
    // 100: never the streamed schedule, 200: the streamed schedule wherever it can run (both with automatic tile and split);
    // 300: never two launches over column ranges (automatic otherwise)
    g_gemm_tuning.streamed = (mt == 100) ? 1 : (mt == 200) ? 2 : 0;
    g_gemm_tuning.parts = (mt == 300 || mt == 500) ? 1 : 0;
    // 400: never cut the tiles past a whole number of rounds along K; 500: neither that nor the two launches
    g_gemm_tuning.tail = (mt == 400 || mt == 500) ? 1 : 0;
    if (mt >= 100) mt = 0;
    // 10 + mt: act-order calls use the tiled kernel's own gather (no staging of the activations)
    g_gemm_tuning.own_gather = (mt >= 10) ? 1 : 0;
    if (mt >= 10) mt -= 10;
    g_gemm_tuning.mt = (mt == 2 || mt == 4) ? mt : 0;
    g_gemm_tuning.splitk = splitk > 0 ? splitk : 0;
}

void gptq4_set_midm_tuning(int mode, int mt, int splitk) {
    g_kslice_tuning.mode = (mode >= 0 && mode <= 2) ? mode : 1;
    // 1000 + mt: the rotary epilogue on tiles of 32 + 32 paired columns wherever the mid-M kernel runs, 2000 + mt: never
    g_kslice_tuning.paired = (mt >= 2000) ? 2 : (mt >= 1000) ? 1 : 0;
    mt %= 1000;
    // 100 + mt: four waves per workgroup, 200 + mt: eight where they fit (automatic: eight for plain projections)
    g_kslice_tuning.waves = (mt >= 200) ? 8 : (mt >= 100) ? 4 : 0;
    mt %= 100;
    // 10 + mt: 128-column strips for plain projections; a plain 1 or 2 also pins the 64-column strips
    g_kslice_tuning.wide = (mt >= 10) ? 1 : ((mt == 1 || mt == 2) ? -1 : 0);
    if (mt >= 10) mt -= 10;
    g_kslice_tuning.mt = (mt == 1 || mt == 2) ? mt : 0;
    g_kslice_tuning.splitk = splitk > 0 ? splitk : 0;
}

void gptq4_set_gemv_tuning(int mode, int depth, int waves, int waves_per_cu) {
    g_gemv_tuning.mode = (mode >= 0 && mode <= 2) ? mode : 1;
    g_gemv_tuning.depth = (depth >= 1 && depth <= 3) ? depth : 0;
    g_gemv_tuning.waves = (waves == 4 || waves == 8 || waves == 16) ? waves : 0;
    g_gemv_tuning.waves_per_cu = (waves_per_cu >= 4 && waves_per_cu <= 32) ? waves_per_cu : 0;
}
void gptq4_set_exchange_spin_limit(unsigned polls) { g_gemv_tuning.spin_limit = polls; }

static_assert(GPTQ4_WS_COUNTER_BYTES == SKINNY_MAX_TILES * COUNTER_STRIDE * 4, "one counter line per tile");

void gptq4_set_tuning(int words, int depth, int splitk) {
    // 10 + words: exchange the split-K partial sums through arrival counters; 20 + words: through marked values wherever they fit
    g_skinny_tuning.exchange = (words >= 20) ? 2 : (words >= 10) ? 1 : 0;
    words %= 10;
    g_skinny_tuning.waves = 0;
    g_skinny_tuning.words = (words == 1 || words == 2 || words == 4) ? words : 0;
    g_skinny_tuning.depth = (depth >= 1 && depth <= 4) ? depth : 0;
    g_skinny_tuning.splitk = splitk > 0 ? splitk : 0;
}

// allow_streamed = false: the need of the same call planned without the tiled kernel's streamed schedule (a
// measurement mode whose partial sums alone are 128 MiB)
static size_t workspace_need(int op, int M, int K, int N, bool allow_streamed) {
    size_t bytes = GPTQ4_WS_HEAD_BYTES;
    const bool with_perm = (op & GPTQ4_OP_WITH_PERM) != 0;
    op &= ~GPTQ4_OP_WITH_PERM;
    if (op == GPTQ4_OP_DECODE_ATTENTION) return (M < 1 || K < 1) ? bytes : bytes + attn_decode_partial_bytes(M, K);
    if (M < 1 || N <= 0 || K <= 0) return bytes;
    if (M <= SKINNY_MAX_M) {
        const int cols = (op == GPTQ4_OP_MLP_GATEUP) ? 2 * N : N;
        size_t need = partial_bytes(SKINNY_MAX_SPLITK, M, cols);
        bytes += need + (with_perm ? (size_t)M * K * 2 : 0);  // + the rows gathered for an act-order call
    } else if ((K % 64) == 0) {
        const int epi = (op == GPTQ4_OP_MLP_GATEUP) ? EPI_SILU_MUL : (op == GPTQ4_OP_QKV_ROTARY ? EPI_ROPE : EPI_PLAIN);
        // whichever kernel the current (automatic or forced) plans pick, with or without act-order, for the whole
        // matrix and for each of the column ranges a call may be cut into
        size_t need = gemm_partial_bytes(gemm_plan(epi, M, N, K, false, allow_streamed));
        const KslicePlan kp = kslice_plan(epi, M, N, K, false);
        if (kp.ok && kslice_partial_bytes(epi, kp) > need) need = kslice_partial_bytes(epi, kp);
        const ColumnParts parts = tiled_parts(epi, M, N, K, false);
        for (int i = 0; i < parts.count; ++i) {
            const TiledChoice c = choose_part(epi, M, K, parts, i, false, allow_streamed);
            if (c.partial > need) need = c.partial;
            const KslicePlan pk = kslice_plan(epi, M, parts.cols[i], K, false);
            if (pk.ok && kslice_partial_bytes(epi, pk) > need) need = kslice_partial_bytes(epi, pk);
        }
        bytes += need;
        // + the rows gathered for an act-order call
        if (with_perm && (size_t)M * K * 2 <= ACT_ORDER_STAGE_MAX) bytes += (size_t)M * K * 2;
    }
    return bytes;
}

size_t gptq4_workspace_bytes(int op, int M, int K, int N) { return workspace_need(op, M, K, N, true); }

int gptq4_column_parts(int op, int M, int K, int N, int *begin, int *cols) {
    op &= ~GPTQ4_OP_WITH_PERM;
    if (M <= SKINNY_MAX_M || N <= 0 || K <= 0 || (K % 64) != 0 || (N % 256) != 0 || op < GPTQ4_OP_MATMUL || op > GPTQ4_OP_QKV_ROTARY) {
        if (begin) begin[0] = 0;
        if (cols) cols[0] = N > 0 ? N : 0;
        return 1;
    }
    const int epi = (op == GPTQ4_OP_MLP_GATEUP) ? EPI_SILU_MUL : (op == GPTQ4_OP_QKV_ROTARY ? EPI_ROPE : EPI_PLAIN);
    const ColumnParts parts = tiled_parts(epi, M, N, K, false);
    for (int i = 0; i < parts.count; ++i) {
        if (begin) begin[i] = parts.begin[i];
        if (cols) cols[i] = parts.cols[i];
    }
    return parts.count;
}

int gptq4_dequant(const int32_t *qweight, const int32_t *qzeros, const void *scales, const int32_t *g_idx,
                  void *W_out, int K, int N, int groupsize, void *stream) {
    if (!qweight || !qzeros || !scales || !W_out) return -GPTQ4_E_NULL;
    if (K <= 0 || N <= 0 || (K % 8) != 0 || (N % 8) != 0) return -GPTQ4_E_SHAPE;
    if (groupsize == -1) groupsize = K;
    if (groupsize <= 0 || (groupsize % 8) != 0) return -GPTQ4_E_GROUPSIZE;
    return launch_dequant(reinterpret_cast<const uint32_t *>(qweight), reinterpret_cast<const uint32_t *>(qzeros),
                          reinterpret_cast<const half_t *>(scales), g_idx, reinterpret_cast<half_t *>(W_out), K,
                          N, groupsize, reinterpret_cast<hipStream_t>(stream));
}

int gptq4_actorder_sort_rows(const int32_t *qweight, const int32_t *perm, int32_t *qweight_out, int K, int N,
                             void *stream) {
    if (!qweight || !perm || !qweight_out) return -GPTQ4_E_NULL;
    if (K <= 0 || N <= 0 || (K % 8) != 0) return -GPTQ4_E_SHAPE;
    return launch_sort_rows(reinterpret_cast<const uint32_t *>(qweight), perm,
                            reinterpret_cast<uint32_t *>(qweight_out), K, N, reinterpret_cast<hipStream_t>(stream));
}

int gptq4_matmul(const void *x, const int32_t *qweight, const int32_t *qzeros, const void *scales,
                 const int32_t *perm, const void *bias, void *y, int M, int K, int N, int groupsize,
                 void *workspace, size_t workspace_bytes, void *stream) {
    if (!x || !qweight || !qzeros || !scales || !y) return -GPTQ4_E_NULL;
    if (M < 1) return -GPTQ4_E_SHAPE;
    int rc = check_dims(K, N, &groupsize);
    if (rc) return rc;
    if (misaligned16(x) || misaligned16(qweight) || misaligned16(scales) || misaligned16(y) ||
        (perm && misaligned16(perm)) || (bias && misaligned16(bias)))
        return -GPTQ4_E_ALIGN;
    MatmulArgs a = {};
    a.x = reinterpret_cast<const half_t *>(x);
    a.w[0] = QMat{reinterpret_cast<const uint32_t *>(qweight), reinterpret_cast<const uint32_t *>(qzeros),
                  reinterpret_cast<const half_t *>(scales)};
    a.perm = perm;
    a.bias = reinterpret_cast<const half_t *>(bias);
    a.y = reinterpret_cast<half_t *>(y);
    a.M = M;
    a.K = K;
    a.N = N;
    a.n_begin = 0;
    a.n_count = N;
    a.groupsize = groupsize;
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    if (M <= SKINNY_MAX_M) {
        return run_small(EPI_PLAIN, a, 1, workspace, workspace_bytes, s);
    }
    return run_tiled(EPI_PLAIN, a, workspace, workspace_bytes, s);
}

// The device address of `scratch` on the current device; looked up once per device.
static int static_scratch(void **out) {
    enum { MAX_DEVICES = 64 };
    static void *ptrs[MAX_DEVICES];
    static std::mutex lock;
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= MAX_DEVICES) return (int)hipErrorInvalidDevice;
    std::lock_guard<std::mutex> guard(lock);
    if (ptrs[dev] == nullptr) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (p == nullptr) return (int)hipErrorInvalidSymbol;
        ptrs[dev] = p;
    }
    *out = ptrs[dev];
    return 0;
}

int gptq4_matmul_static(const void *x, const int32_t *qweight, const int32_t *qzeros, const void *scales,
                        const void *bias, void *y, int M, int K, int N, int groupsize, void *stream) {
    if (!x || !qweight || !qzeros || !scales || !y) return -GPTQ4_E_NULL;
    if (M < 1) return -GPTQ4_E_SHAPE;
    int g = groupsize;
    int rc = check_dims(K, N, &g);
    if (rc) return rc;
    // what the same call would ask of a caller's workspace - planned without the streamed schedule of the tiled
    // kernel, whose partial sums alone are 128 MiB - has to fit the static array
    const size_t need = workspace_need(GPTQ4_OP_MATMUL, M, K, N, false);
    if (need > (size_t)GPTQ4_STATIC_SCRATCH_BYTES) return -GPTQ4_E_STATIC_LIMIT;
    void *ws = nullptr;
    rc = static_scratch(&ws);
    if (rc) return rc;
    return gptq4_matmul(x, qweight, qzeros, scales, nullptr, bias, y, M, K, N, groupsize, ws, GPTQ4_STATIC_SCRATCH_BYTES, stream);
}

int gptq4_static_status(void *stream) {
    void *ws = nullptr;
    int rc = static_scratch(&ws);
    if (rc) return rc;
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    int word = 0;
    hipError_t e = hipMemcpyAsync(&word, reinterpret_cast<const int *>(ws) + GPTQ4_WS_ERROR_WORD, sizeof(int), hipMemcpyDeviceToHost, s);
    if (e != hipSuccess) return (int)e;
    e = hipStreamSynchronize(s);
    if (e != hipSuccess) return (int)e;
    return word != 0 ? -GPTQ4_E_EXCHANGE : 0;
}

int gptq4_static_reset(void *stream) {
    void *ws = nullptr;
    int rc = static_scratch(&ws);
    if (rc) return rc;
    return (int)hipMemsetAsync(ws, 0, GPTQ4_WS_HEAD_BYTES, reinterpret_cast<hipStream_t>(stream));
}

static int mlp_gateup_impl(const void *x, const void *delta, const void *norm_weight, void *sum_out, float eps,
                           const int32_t *gate_qweight, const int32_t *gate_qzeros, const void *gate_scales,
                           const int32_t *up_qweight, const int32_t *up_qzeros, const void *up_scales,
                           const int32_t *perm, void *h, int M, int K, int I, int groupsize, void *workspace,
                           size_t workspace_bytes, void *stream, bool norm) {
    if (!x || !gate_qweight || !gate_qzeros || !gate_scales || !up_qweight || !up_qzeros || !up_scales || !h)
        return -GPTQ4_E_NULL;
    if (M < 1) return -GPTQ4_E_SHAPE;
    int rc = check_dims(K, I, &groupsize);
    if (rc) return rc;
    if (misaligned16(x) || misaligned16(gate_qweight) || misaligned16(up_qweight) || misaligned16(gate_scales) ||
        misaligned16(up_scales) || misaligned16(h) || (perm && misaligned16(perm)))
        return -GPTQ4_E_ALIGN;
    MatmulArgs a = {};
    a.x = reinterpret_cast<const half_t *>(x);
    a.w[0] = QMat{reinterpret_cast<const uint32_t *>(gate_qweight), reinterpret_cast<const uint32_t *>(gate_qzeros),
                  reinterpret_cast<const half_t *>(gate_scales)};
    a.w[1] = QMat{reinterpret_cast<const uint32_t *>(up_qweight), reinterpret_cast<const uint32_t *>(up_qzeros),
                  reinterpret_cast<const half_t *>(up_scales)};
    a.perm = perm;
    a.y = reinterpret_cast<half_t *>(h);
    a.M = M;
    a.K = K;
    a.N = I;
    a.n_begin = 0;
    a.n_count = I;
    a.groupsize = groupsize;
    if (norm) {
        rc = setup_norm(a, delta, norm_weight, sum_out, eps);
        if (rc) return rc;
    }
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    if (M <= SKINNY_MAX_M) {
        return run_small(EPI_SILU_MUL, a, 2, workspace, workspace_bytes, s);
    }
    return run_tiled(EPI_SILU_MUL, a, workspace, workspace_bytes, s);
}

int gptq4_mlp_gateup(const void *x, const int32_t *gate_qweight, const int32_t *gate_qzeros,
                     const void *gate_scales, const int32_t *up_qweight, const int32_t *up_qzeros,
                     const void *up_scales, const int32_t *perm, void *h, int M, int K, int I, int groupsize,
                     void *workspace, size_t workspace_bytes, void *stream) {
    return mlp_gateup_impl(x, nullptr, nullptr, nullptr, 0.f, gate_qweight, gate_qzeros, gate_scales, up_qweight, up_qzeros,
                           up_scales, perm, h, M, K, I, groupsize, workspace, workspace_bytes, stream, false);
}

int gptq4_norm_mlp_gateup(const void *x, const void *delta, const void *norm_weight, float eps, void *sum_out,
                          const int32_t *gate_qweight, const int32_t *gate_qzeros, const void *gate_scales,
                          const int32_t *up_qweight, const int32_t *up_qzeros, const void *up_scales,
                          const int32_t *perm, void *h, int M, int K, int I, int groupsize, void *workspace,
                          size_t workspace_bytes, void *stream) {
    return mlp_gateup_impl(x, delta, norm_weight, sum_out, eps, gate_qweight, gate_qzeros, gate_scales, up_qweight,
                           up_qzeros, up_scales, perm, h, M, K, I, groupsize, workspace, workspace_bytes, stream, true);
}

int gptq4_rope_table(float *cos_out, float *sin_out, int max_pos, int D, float base, void *stream) {
    if (!cos_out || !sin_out) return -GPTQ4_E_NULL;
    if (max_pos < 1 || D < 2 || (D % 2) != 0 || !(base > 0.f)) return -GPTQ4_E_SHAPE;
    return launch_rope_table(cos_out, sin_out, max_pos, D, base, reinterpret_cast<hipStream_t>(stream));
}

// round-up reciprocal of S for row -> (sequence, token): exact for every row < M when (M - 1) * (magic * S - 2^32) < 2^32; 0: divide
static uint32_t rope_s_magic(int S, int M) {
    if (S <= 1) return 0;
    const uint64_t magic = (1ull << 32) / (uint64_t)S + 1;
    const uint64_t err = magic * (uint64_t)S - (1ull << 32);
    return (magic < (1ull << 32) && (uint64_t)(M - 1) * err < (1ull << 32)) ? (uint32_t)magic : 0u;
}

static int qkv_rotary_impl(const void *x, const void *delta, const void *norm_weight, void *sum_out, float eps,
                           const int32_t *qweight, const int32_t *qzeros, const void *scales, const int32_t *perm,
                           const int32_t *position_ids, const float *cos_table, const float *sin_table, int max_pos,
                           void *q, void *k, void *v, int B, int S, int H, int D, int K, int groupsize, int kv_capacity,
                           int kv_offset, void *workspace, size_t workspace_bytes, void *stream, bool norm) {
    if (!x || !qweight || !qzeros || !scales || !position_ids || !cos_table || !sin_table || !q || !k || !v)
        return -GPTQ4_E_NULL;
    if (B < 1 || S < 1 || H < 1 || D != 128 || max_pos < 1) return -GPTQ4_E_SHAPE;
    if (kv_offset < GPTQ4_KV_AT_POSITION || kv_capacity < 1 || (kv_offset >= 0 && kv_capacity < kv_offset + S))
        return -GPTQ4_E_SHAPE;
    if ((long)B * S > 0x7fffffffL) return -GPTQ4_E_SHAPE;
    const int N = 3 * H * D;
    int rc = check_dims(K, N, &groupsize);
    if (rc) return rc;
    if (misaligned16(x) || misaligned16(qweight) || misaligned16(scales) || misaligned16(q) || misaligned16(k) ||
        misaligned16(v) || misaligned16(cos_table) || misaligned16(sin_table) || (perm && misaligned16(perm)))
        return -GPTQ4_E_ALIGN;
    MatmulArgs a = {};
    a.x = reinterpret_cast<const half_t *>(x);
    a.w[0] = QMat{reinterpret_cast<const uint32_t *>(qweight), reinterpret_cast<const uint32_t *>(qzeros),
                  reinterpret_cast<const half_t *>(scales)};
    a.perm = perm;
    a.M = B * S;
    a.K = K;
    a.N = N;
    a.n_begin = 0;
    a.n_count = N;
    a.groupsize = groupsize;
    a.rope.position_ids = position_ids;
    a.rope.cos_table = cos_table;
    a.rope.sin_table = sin_table;
    a.rope.q = reinterpret_cast<half_t *>(q);
    a.rope.k = reinterpret_cast<half_t *>(k);
    a.rope.v = reinterpret_cast<half_t *>(v);
    a.rope.S = S;
    a.rope.H = H;
    a.rope.kv_capacity = kv_capacity;
    a.rope.kv_offset = kv_offset;
    a.rope.max_pos = max_pos;
    a.rope.s_magic = rope_s_magic(S, a.M);
    if (norm) {
        rc = setup_norm(a, delta, norm_weight, sum_out, eps);
        if (rc) return rc;
    }
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    if (a.M <= SKINNY_MAX_M) {
        return run_small(EPI_ROPE, a, 1, workspace, workspace_bytes, s);
    }
    return run_tiled(EPI_ROPE, a, workspace, workspace_bytes, s);
}

int gptq4_qkv_rotary(const void *x, const int32_t *qweight, const int32_t *qzeros, const void *scales,
                     const int32_t *perm, const int32_t *position_ids, const float *cos_table,
                     const float *sin_table, int max_pos, void *q, void *k, void *v, int B, int S, int H, int D,
                     int K, int groupsize, int kv_capacity, int kv_offset, void *workspace,
                     size_t workspace_bytes, void *stream) {
    return qkv_rotary_impl(x, nullptr, nullptr, nullptr, 0.f, qweight, qzeros, scales, perm, position_ids, cos_table,
                           sin_table, max_pos, q, k, v, B, S, H, D, K, groupsize, kv_capacity, kv_offset, workspace,
                           workspace_bytes, stream, false);
}

int gptq4_norm_qkv_rotary(const void *x, const void *delta, const void *norm_weight, float eps, void *sum_out,
                          const int32_t *qweight, const int32_t *qzeros, const void *scales, const int32_t *perm,
                          const int32_t *position_ids, const float *cos_table, const float *sin_table, int max_pos,
                          void *q, void *k, void *v, int B, int S, int H, int D, int K, int groupsize, int kv_capacity,
                          int kv_offset, void *workspace, size_t workspace_bytes, void *stream) {
    return qkv_rotary_impl(x, delta, norm_weight, sum_out, eps, qweight, qzeros, scales, perm, position_ids, cos_table,
                           sin_table, max_pos, q, k, v, B, S, H, D, K, groupsize, kv_capacity, kv_offset, workspace,
                           workspace_bytes, stream, true);
}

int gptq4_rmsnorm(const void *x, const void *weight, void *y, const int32_t *y_index, int M, int H, float eps, void *stream) {
    if (!x || !weight || !y) return -GPTQ4_E_NULL;
    if (M < 1 || H < 8 || (H % 8) != 0 || !(eps >= 0.f)) return -GPTQ4_E_SHAPE;
    if (y_index && y == x) return -GPTQ4_E_SHAPE;  // the moved values would overwrite input still to be read
    if (misaligned16(x) || misaligned16(weight) || misaligned16(y) || (y_index && misaligned16(y_index))) return -GPTQ4_E_ALIGN;
    return launch_rmsnorm(reinterpret_cast<const half_t *>(x), nullptr, reinterpret_cast<const half_t *>(weight), nullptr,
                          reinterpret_cast<half_t *>(y), y_index, M, H, eps, reinterpret_cast<hipStream_t>(stream));
}

int gptq4_add_rmsnorm(const void *x, const void *delta, const void *weight, void *sum_out, void *y, const int32_t *y_index,
                      int M, int H, float eps, void *stream) {
    if (!x || !delta || !weight || !sum_out || !y) return -GPTQ4_E_NULL;
    if (M < 1 || H < 8 || (H % 8) != 0 || !(eps >= 0.f)) return -GPTQ4_E_SHAPE;
    if (y_index && (y == x || y == delta || y == sum_out)) return -GPTQ4_E_SHAPE;
    if (misaligned16(x) || misaligned16(delta) || misaligned16(weight) || misaligned16(sum_out) || misaligned16(y) ||
        (y_index && misaligned16(y_index)))
        return -GPTQ4_E_ALIGN;
    return launch_rmsnorm(reinterpret_cast<const half_t *>(x), reinterpret_cast<const half_t *>(delta),
                          reinterpret_cast<const half_t *>(weight), reinterpret_cast<half_t *>(sum_out),
                          reinterpret_cast<half_t *>(y), y_index, M, H, eps, reinterpret_cast<hipStream_t>(stream));
}

int gptq4_decode_attention(const void *q, const void *k_cache, const void *v_cache, const int32_t *positions, void *out,
                           const int32_t *out_index, int B, int H, int D, int kv_capacity, float scale, void *workspace, size_t workspace_bytes,
                           void *stream) {
    if (!q || !k_cache || !v_cache || !positions || !out) return -GPTQ4_E_NULL;
    if (B < 1 || H < 1 || D != 128 || kv_capacity < 1 || (long)B * H > SKINNY_MAX_TILES) return -GPTQ4_E_SHAPE;
    if (misaligned16(q) || misaligned16(k_cache) || misaligned16(v_cache) || misaligned16(out)) return -GPTQ4_E_ALIGN;
    if (workspace == nullptr || workspace_bytes < GPTQ4_WS_HEAD_BYTES + attn_decode_partial_bytes(B * H, kv_capacity))
        return -GPTQ4_E_WORKSPACE;
    float *partials = reinterpret_cast<float *>(reinterpret_cast<char *>(workspace) + GPTQ4_WS_HEAD_BYTES);
    return launch_attn_decode(reinterpret_cast<const half_t *>(q), reinterpret_cast<const half_t *>(k_cache),
                              reinterpret_cast<const half_t *>(v_cache), positions, reinterpret_cast<half_t *>(out), out_index, B, H,
                              kv_capacity, scale, reinterpret_cast<int *>(workspace), partials,
                              reinterpret_cast<hipStream_t>(stream));
}

int gptq4_lm_head_argmax(const void *x, const void *weight, int64_t *out, int B, int K, int V, void *workspace, size_t workspace_bytes,
                         void *stream) {
    if (!x || !weight || !out) return -GPTQ4_E_NULL;
    if (misaligned16(x) || misaligned16(weight) || (reinterpret_cast<uintptr_t>(out) & 7)) return -GPTQ4_E_ALIGN;
    if (workspace == nullptr || workspace_bytes < GPTQ4_WS_HEAD_BYTES + head_argmax_partial_bytes()) return -GPTQ4_E_WORKSPACE;
    float *part = reinterpret_cast<float *>(reinterpret_cast<char *>(workspace) + GPTQ4_WS_HEAD_BYTES);
    return launch_head_argmax(reinterpret_cast<const half_t *>(x), reinterpret_cast<const half_t *>(weight), reinterpret_cast<long long *>(out),
                              part, reinterpret_cast<int *>(workspace), B, K, V, reinterpret_cast<hipStream_t>(stream));
}

int gptq4_prefill_attention(const void *q, const void *k_cache, const void *v_cache, void *out, int B, int H, int S, int D,
                            int kv_capacity, int past, float scale, void *stream) {
    if (!q || !k_cache || !v_cache || !out) return -GPTQ4_E_NULL;
    if (B < 1 || H < 1 || S < 1 || D != 128 || past < 0 || kv_capacity < 1 || kv_capacity > (1 << 23) || (long)past + S > kv_capacity || (long)B * H * ((S + 127) / 128) >= (1L << 31) ||
        (long)B * H * kv_capacity * 128 >= (1L << 40))
        return -GPTQ4_E_SHAPE;
    if (misaligned16(q) || misaligned16(k_cache) || misaligned16(v_cache) || misaligned16(out)) return -GPTQ4_E_ALIGN;
    return launch_attn_prefill(reinterpret_cast<const half_t *>(q), reinterpret_cast<const half_t *>(k_cache),
                               reinterpret_cast<const half_t *>(v_cache), reinterpret_cast<half_t *>(out), B, H, S, kv_capacity, past, scale,
                               reinterpret_cast<hipStream_t>(stream));
}

// ---- streaming-order layout ---------------------------------------------------------------------------------------

static int stream_fill(StreamArgs &a, int epi, int groupsize, void *workspace, size_t workspace_bytes, StreamPlan &pl, bool norm,
                       void *stream) {
    pl = stream_plan(epi, a.M, a.N, a.K, norm);
    if (!pl.ok) return -GPTQ4_E_SHAPE;
    if (workspace == nullptr || workspace_bytes < GPTQ4_WS_HEAD_BYTES) return -GPTQ4_E_WORKSPACE;
    if (pl.tall && a.perm != nullptr) {
        // the kernel for more than STREAM_MAX_M rows does not gather: one small launch does, into the workspace behind the head
        const size_t bytes = (size_t)a.M * a.K * sizeof(half_t);
        if (workspace_bytes < GPTQ4_WS_HEAD_BYTES + bytes) return -GPTQ4_E_WORKSPACE;
        half_t *xg = reinterpret_cast<half_t *>(reinterpret_cast<char *>(workspace) + GPTQ4_WS_HEAD_BYTES);
        const int rc = launch_gather_cols(a.x, a.perm, xg, a.M, a.K, reinterpret_cast<hipStream_t>(stream));
        if (rc) return rc;
        a.x = xg;
        a.perm = nullptr;
    }
    a.counters = reinterpret_cast<int *>(workspace);
    a.tagged = reinterpret_cast<uint64_t *>(reinterpret_cast<char *>(workspace) + GPTQ4_WS_COUNTER_BYTES);
    a.spin_limit = g_gemv_tuning.spin_limit ? g_gemv_tuning.spin_limit : (1u << 22);
    a.groups = a.K / groupsize;
    a.batches_per_group = groupsize / 128;
    a.group_magic = a.batches_per_group > 1 ? (uint32_t)(0x100000000ull / (unsigned)a.batches_per_group + 1) : 0u;
    return 0;
}

// More rows than the streaming-order kernels take: the tiled kernel reads the same words (its SB variant).
static int stream_tiled(int epi, MatmulArgs &t, int M, int K, int N, int groupsize, void *workspace, size_t workspace_bytes, void *stream) {
    t.M = M;
    t.K = K;
    t.N = N;
    t.n_begin = 0;
    t.n_count = N;
    t.groupsize = groupsize;
    t.stream_b = 1;
    return run_tiled(epi, t, workspace, workspace_bytes, reinterpret_cast<hipStream_t>(stream));
}

static int stream_norm(StreamArgs &a, const void *delta, const void *norm_weight, void *sum_out, float eps) {
    if (delta && !sum_out) return -GPTQ4_E_NULL;
    if (a.M > NORM_MAX_M || a.K > NORM_MAX_H || !(eps >= 0.f)) return -GPTQ4_E_SHAPE;
    if (delta && (sum_out == static_cast<const void *>(a.x) || sum_out == delta)) return -GPTQ4_E_SHAPE;
    if (misaligned16(norm_weight) || (delta && (misaligned16(delta) || misaligned16(sum_out)))) return -GPTQ4_E_ALIGN;
    a.nrm_delta = reinterpret_cast<const half_t *>(delta);
    a.nrm_weight = reinterpret_cast<const half_t *>(norm_weight);
    a.nrm_sum_out = delta ? reinterpret_cast<half_t *>(sum_out) : nullptr;
    a.nrm_eps = eps;
    return 0;
}

int gptq4_stream_rows(int op, int K, int N, int groupsize) {
    op &= ~GPTQ4_OP_WITH_PERM;
    if (op < GPTQ4_OP_MATMUL || op > GPTQ4_OP_QKV_ROTARY) return 0;
    int g = groupsize;
    if (check_dims(K, N, &g)) return 0;
    const int epi = (op == GPTQ4_OP_MLP_GATEUP) ? EPI_SILU_MUL : (op == GPTQ4_OP_QKV_ROTARY ? EPI_ROPE : EPI_PLAIN);
    int rows = 0;
    for (int m = 1; m <= STREAM_TALL_MAX_M; ++m)
        if (stream_plan(epi, m, N, K, false).ok) rows = m;
    return rows;
}

int gptq4_stream_pack(const int32_t *qweight, const int32_t *qzeros, const void *scales, int32_t *sweight, int32_t *smeta, int K,
                      int N, int groupsize, void *stream) {
    if (!qweight || !sweight || (smeta && (!qzeros || !scales))) return -GPTQ4_E_NULL;
    int rc = check_dims(K, N, &groupsize);
    if (rc) return rc;
    if (static_cast<const void *>(qweight) == static_cast<const void *>(sweight)) return -GPTQ4_E_SHAPE;
    return launch_stream_pack(reinterpret_cast<const uint32_t *>(qweight), reinterpret_cast<const uint32_t *>(qzeros),
                              reinterpret_cast<const half_t *>(scales), reinterpret_cast<uint32_t *>(sweight),
                              reinterpret_cast<uint32_t *>(smeta), K, N, groupsize, reinterpret_cast<hipStream_t>(stream));
}

int gptq4_stream_unpack(const int32_t *sweight, const int32_t *smeta, int32_t *qweight, int32_t *qzeros, void *scales, int K, int N,
                        int groupsize, void *stream) {
    if (!sweight || !qweight || (smeta && (!qzeros || !scales))) return -GPTQ4_E_NULL;
    int rc = check_dims(K, N, &groupsize);
    if (rc) return rc;
    if (static_cast<const void *>(qweight) == static_cast<const void *>(sweight)) return -GPTQ4_E_SHAPE;
    return launch_stream_unpack(reinterpret_cast<const uint32_t *>(sweight), reinterpret_cast<const uint32_t *>(smeta),
                                reinterpret_cast<uint32_t *>(qweight), reinterpret_cast<uint32_t *>(qzeros),
                                reinterpret_cast<half_t *>(scales), K, N, groupsize, reinterpret_cast<hipStream_t>(stream));
}

int gptq4_stream_dequant(const int32_t *sweight, const int32_t *smeta, void *W_out, int K, int N, int groupsize, void *stream) {
    if (!sweight || !smeta || !W_out) return -GPTQ4_E_NULL;
    int rc = check_dims(K, N, &groupsize);
    if (rc) return rc;
    return launch_stream_dequant(reinterpret_cast<const uint32_t *>(sweight), reinterpret_cast<const uint32_t *>(smeta),
                                 reinterpret_cast<half_t *>(W_out), K, N, groupsize, reinterpret_cast<hipStream_t>(stream));
}

static int stream_matmul_impl(const void *x, const int32_t *sweight, const int32_t *smeta, const int32_t *perm, const void *bias,
                              void *y, int M, int K, int N, int groupsize, void *workspace, size_t workspace_bytes, void *stream,
                              bool nomath) {
    if (!x || !sweight || !smeta || !y) return -GPTQ4_E_NULL;
    if (M < 1) return -GPTQ4_E_SHAPE;
    int rc = check_dims(K, N, &groupsize);
    if (rc) return rc;
    if (misaligned16(x) || misaligned16(sweight) || misaligned16(smeta) || misaligned16(y) || (perm && misaligned16(perm)) ||
        (bias && misaligned16(bias)))
        return -GPTQ4_E_ALIGN;
    StreamArgs a = {};
    a.x = reinterpret_cast<const half_t *>(x);
    a.m[0] = SMat{reinterpret_cast<const uint32_t *>(sweight), reinterpret_cast<const uint32_t *>(smeta)};
    a.m[1] = a.m[0];
    a.perm = perm;
    a.bias = reinterpret_cast<const half_t *>(bias);
    a.y = reinterpret_cast<half_t *>(y);
    a.M = M;
    a.K = K;
    a.N = N;
    if (M > STREAM_TALL_MAX_M) {
        if (nomath) return -GPTQ4_E_SHAPE;
        MatmulArgs t = {};
        t.x = a.x;
        t.w[0] = QMat{a.m[0].w, a.m[0].meta, nullptr};
        t.perm = perm;
        t.bias = a.bias;
        t.y = a.y;
        return stream_tiled(EPI_PLAIN, t, M, K, N, groupsize, workspace, workspace_bytes, stream);
    }
    StreamPlan pl;
    rc = stream_fill(a, EPI_PLAIN, groupsize, workspace, workspace_bytes, pl, false, stream);
    if (rc) return rc;
    return launch_stream(EPI_PLAIN, a, pl, nomath, reinterpret_cast<hipStream_t>(stream));
}

int gptq4_stream_matmul(const void *x, const int32_t *sweight, const int32_t *smeta, const int32_t *perm, const void *bias, void *y,
                        int M, int K, int N, int groupsize, void *workspace, size_t workspace_bytes, void *stream) {
    return stream_matmul_impl(x, sweight, smeta, perm, bias, y, M, K, N, groupsize, workspace, workspace_bytes, stream, false);
}

static int stream_gateup_impl(const void *x, const void *delta, const void *norm_weight, float eps, void *sum_out,
                              const int32_t *gate_sweight, const int32_t *gate_smeta, const int32_t *up_sweight,
                              const int32_t *up_smeta, const int32_t *perm, void *h, int M, int K, int I, int groupsize,
                              void *workspace, size_t workspace_bytes, void *stream, bool nomath) {
    if (!x || !gate_sweight || !gate_smeta || !up_sweight || !up_smeta || !h) return -GPTQ4_E_NULL;
    if (M < 1) return -GPTQ4_E_SHAPE;
    int rc = check_dims(K, I, &groupsize);
    if (rc) return rc;
    if (misaligned16(x) || misaligned16(gate_sweight) || misaligned16(up_sweight) || misaligned16(gate_smeta) ||
        misaligned16(up_smeta) || misaligned16(h) || (perm && misaligned16(perm)))
        return -GPTQ4_E_ALIGN;
    StreamArgs a = {};
    a.x = reinterpret_cast<const half_t *>(x);
    a.m[0] = SMat{reinterpret_cast<const uint32_t *>(gate_sweight), reinterpret_cast<const uint32_t *>(gate_smeta)};
    a.m[1] = SMat{reinterpret_cast<const uint32_t *>(up_sweight), reinterpret_cast<const uint32_t *>(up_smeta)};
    a.perm = perm;
    a.y = reinterpret_cast<half_t *>(h);
    a.M = M;
    a.K = K;
    a.N = I;
    if (M > STREAM_TALL_MAX_M) {
        if (nomath || norm_weight) return -GPTQ4_E_SHAPE;
        MatmulArgs t = {};
        t.x = a.x;
        t.w[0] = QMat{a.m[0].w, a.m[0].meta, nullptr};
        t.w[1] = QMat{a.m[1].w, a.m[1].meta, nullptr};
        t.perm = perm;
        t.y = a.y;
        return stream_tiled(EPI_SILU_MUL, t, M, K, I, groupsize, workspace, workspace_bytes, stream);
    }
    if (norm_weight) {
        rc = stream_norm(a, delta, norm_weight, sum_out, eps);
        if (rc) return rc;
    }
    StreamPlan pl;
    rc = stream_fill(a, EPI_SILU_MUL, groupsize, workspace, workspace_bytes, pl, norm_weight != nullptr, stream);
    if (rc) return rc;
    return launch_stream(EPI_SILU_MUL, a, pl, nomath, reinterpret_cast<hipStream_t>(stream));
}

int gptq4_stream_mlp_gateup(const void *x, const void *delta, const void *norm_weight, float eps, void *sum_out,
                            const int32_t *gate_sweight, const int32_t *gate_smeta, const int32_t *up_sweight,
                            const int32_t *up_smeta, const int32_t *perm, void *h, int M, int K, int I, int groupsize,
                            void *workspace, size_t workspace_bytes, void *stream) {
    return stream_gateup_impl(x, delta, norm_weight, eps, sum_out, gate_sweight, gate_smeta, up_sweight, up_smeta, perm, h, M, K, I,
                              groupsize, workspace, workspace_bytes, stream, false);
}

int gptq4_stream_qkv_rotary(const void *x, const void *delta, const void *norm_weight, float eps, void *sum_out,
                            const int32_t *sweight, const int32_t *smeta, const int32_t *perm, const int32_t *position_ids,
                            const float *cos_table, const float *sin_table, int max_pos, void *q, void *k, void *v, int B, int S,
                            int H, int D, int K, int groupsize, int kv_capacity, int kv_offset, void *workspace,
                            size_t workspace_bytes, void *stream) {
    if (!x || !sweight || !smeta || !position_ids || !cos_table || !sin_table || !q || !k || !v) return -GPTQ4_E_NULL;
    if (B < 1 || S < 1 || H < 1 || D != 128 || max_pos < 1) return -GPTQ4_E_SHAPE;
    if (kv_offset < GPTQ4_KV_AT_POSITION || kv_capacity < 1 || (kv_offset >= 0 && kv_capacity < kv_offset + S)) return -GPTQ4_E_SHAPE;
    if ((long)B * S > 0x7fffffffL) return -GPTQ4_E_SHAPE;
    const int N = 3 * H * D;
    int rc = check_dims(K, N, &groupsize);
    if (rc) return rc;
    if (misaligned16(x) || misaligned16(sweight) || misaligned16(smeta) || misaligned16(q) || misaligned16(k) || misaligned16(v) ||
        misaligned16(cos_table) || misaligned16(sin_table) || (perm && misaligned16(perm)))
        return -GPTQ4_E_ALIGN;
    if ((long)B * S > STREAM_TALL_MAX_M) {
        if (norm_weight) return -GPTQ4_E_SHAPE;
        MatmulArgs t = {};
        t.x = reinterpret_cast<const half_t *>(x);
        t.w[0] = QMat{reinterpret_cast<const uint32_t *>(sweight), reinterpret_cast<const uint32_t *>(smeta), nullptr};
        t.perm = perm;
        t.rope.position_ids = position_ids;
        t.rope.cos_table = cos_table;
        t.rope.sin_table = sin_table;
        t.rope.q = reinterpret_cast<half_t *>(q);
        t.rope.k = reinterpret_cast<half_t *>(k);
        t.rope.v = reinterpret_cast<half_t *>(v);
        t.rope.S = S;
        t.rope.H = H;
        t.rope.kv_capacity = kv_capacity;
        t.rope.kv_offset = kv_offset;
        t.rope.max_pos = max_pos;
        t.rope.s_magic = rope_s_magic(S, B * S);
        return stream_tiled(EPI_ROPE, t, B * S, K, N, groupsize, workspace, workspace_bytes, stream);
    }
    StreamArgs a = {};
    a.x = reinterpret_cast<const half_t *>(x);
    a.m[0] = SMat{reinterpret_cast<const uint32_t *>(sweight), reinterpret_cast<const uint32_t *>(smeta)};
    a.m[1] = a.m[0];
    a.perm = perm;
    a.M = B * S;
    a.K = K;
    a.N = N;
    a.rope.position_ids = position_ids;
    a.rope.cos_table = cos_table;
    a.rope.sin_table = sin_table;
    a.rope.q = reinterpret_cast<half_t *>(q);
    a.rope.k = reinterpret_cast<half_t *>(k);
    a.rope.v = reinterpret_cast<half_t *>(v);
    a.rope.S = S;
    a.rope.H = H;
    a.rope.kv_capacity = kv_capacity;
    a.rope.kv_offset = kv_offset;
    a.rope.max_pos = max_pos;
    a.rope.s_magic = 0;  // a handful of rows: a plain division
    if (norm_weight) {
        rc = stream_norm(a, delta, norm_weight, sum_out, eps);
        if (rc) return rc;
    }
    StreamPlan pl;
    rc = stream_fill(a, EPI_ROPE, groupsize, workspace, workspace_bytes, pl, norm_weight != nullptr, stream);
    if (rc) return rc;
    return launch_stream(EPI_ROPE, a, pl, false, reinterpret_cast<hipStream_t>(stream));
}

void gptq4_set_stream_tuning(int waves, int depth) {
    g_stream_tuning.waves = (waves == 8 || waves == 16) ? waves : 0;
    // 10 + depth: one tile per unit in the kernel for 5 .. 16 rows, 20 + depth: two wherever they can run (automatic otherwise)
    const int single = depth >= 20 ? 20 : depth >= 10 ? 10 : 0;
    depth -= single;
    g_stream_tuning.depth = ((depth >= 1 && depth <= 3) ? depth : 0) + single;
}

int gptq4_stream_probe(int op, const void *x, const int32_t *sweight, const int32_t *smeta, const int32_t *up_sweight,
                       const int32_t *up_smeta, void *y, int M, int K, int N, int groupsize, void *workspace, size_t workspace_bytes,
                       void *stream) {
    if (op == GPTQ4_OP_MLP_GATEUP)
        return stream_gateup_impl(x, nullptr, nullptr, 0.f, nullptr, sweight, smeta, up_sweight, up_smeta, nullptr, y, M, K, N, groupsize,
                                  workspace, workspace_bytes, stream, true);
    return stream_matmul_impl(x, sweight, smeta, nullptr, nullptr, y, M, K, N, groupsize, workspace, workspace_bytes, stream, true);
}

}  // extern "C"
