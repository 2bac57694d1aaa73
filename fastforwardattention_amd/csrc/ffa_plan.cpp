// Launch planner for the gfx950 decode kernels.  Pure host code, no HIP calls.
//
// Stands where the reference has get_launch_params (kernel_launch_utils.h:135-180), which
// searches threads-per-block x threads-per-key x threads-per-value with a fitted time
// model.  On a 256-CU wave64 part with the reference's K layout the per-key work is best
// kept in one lane (threads_per_key = 1: every load instruction is 1 KiB contiguous), so
// the quantities that matter are how many wavefronts share a (batch, head) and how the
// sequence is split across workgroups.
#include <math.h>
#include <stdlib.h>

#include <vector>

#include "ffa_host.h"

namespace ffa {

static int pow2_floor(int v) {
    int p = 1;
    while (p * 2 <= v) p *= 2;
    return p;
}

static int ceil_div(int a, int b) { return (a + b - 1) / b; }

static void fill(ffa_launch_plan* plan, int kind, int waves, int n_splits, int tiles_per_split) {
    plan->kind = kind;
    plan->waves_per_wg = waves;
    plan->threads_per_key = 1;
    plan->keys_per_wave = kTileKeys;
    plan->n_splits = n_splits;
    plan->tiles_per_split = tiles_per_split;
    plan->combine = FFA_COMBINE_FUSED;
    plan->whole_heads = 0;
}

// Largest power-of-two wave count (<= 16) whose score buffer + merge buffer fit in LDS and
// that still leaves every wave at least one tile.
static int wg_waves_for(int ntiles, int want) {
    int w = pow2_floor(want < 1 ? 1 : want);
    if (w > 16) w = 16;
    while (w > 1 && w > ntiles) w /= 2;
    return w;
}

// ---------------------------------------------------------------------------------------
// Measured overrides (ffa_plan_table.inc, written by `python bench.py --sweep-plans` on the
// device): where a sweep over launch kinds, wave counts, lanes per key and split factors
// found something more than 3 % faster than the rules below, the table's row wins.  The table
// holds the BASELINE shapes themselves and matches them exactly; the grid further down covers
// everything else by nearest neighbour.
struct PlanRow {
    int override_rules, precision, head_dim, pairs, t_lo, t_hi, pruned;
    int kind, waves, tpk, n_splits, whole_heads;
    float chosen_us, best_us, rule_us;
};
static const PlanRow kPlanTable[] = {
#define FFA_PLAN_ROW(ov, prec, dh, pairs, tlo, thi, pruned, kind, waves, tpk, ns, whole, chosen, best, rule) \
    {ov, prec, dh, pairs, tlo, thi, pruned, kind, waves, tpk, ns, whole, chosen, best, rule},
#include "ffa_plan_table.inc"
#undef FFA_PLAN_ROW
    {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0.f, 0.f, 0.f}  // sentinel
};
constexpr int kTableCus = 256;  // the table was measured on a 256-CU device

// Applies a table row to the actual t: the split factor is kept, the pieces are re-cut.
// Returns kNoRow when no row covers the problem, kRowKeepsRules when one does and records that the
// rules' plan was within 3 % of the best (the grid is not consulted then either), kRowOverrides
// when *plan now holds the row's plan.
enum { kNoRow = 0, kRowKeepsRules = 1, kRowOverrides = 2 };
static int plan_from_table(int precision, int bh, int Dh, int t, float p, int cus, ffa_launch_plan* plan) {
    if (cus != kTableCus) return kNoRow;
    const int pruned = p > 0.f ? 1 : 0;
    const int ntiles = num_tiles(t);
    // Rows of different sweeps may overlap in t: the one whose centre is nearest decides.
    const PlanRow* r = nullptr;
    for (const PlanRow* c = kPlanTable; c->precision != 0; ++c) {
        if (c->precision != precision || c->head_dim != Dh || c->pairs != bh || c->pruned != pruned) continue;
        if (t < c->t_lo || t > c->t_hi) continue;
        if (r == nullptr || abs(2 * t - c->t_lo - c->t_hi) < abs(2 * t - r->t_lo - r->t_hi)) r = c;
    }
    if (r != nullptr) {
        if (!r->override_rules) return kRowKeepsRules;
        int n_splits = r->n_splits < 1 ? 1 : r->n_splits;
        if (n_splits > ntiles) n_splits = ntiles;
        const int tps = ceil_div(ntiles, n_splits);
        n_splits = ceil_div(ntiles, tps);
        fill(plan, r->kind, r->waves, n_splits, tps);
        plan->threads_per_key = r->tpk;
        plan->keys_per_wave = kTileKeys / r->tpk;
        plan->whole_heads = r->kind == FFA_LAUNCH_SPLIT ? (n_splits == 1 ? bh : r->whole_heads) : 0;
        return validate_plan(*plan, precision, Dh, bh, t, p) == FFA_OK ? kRowOverrides : kRowKeepsRules;
    }
    return kNoRow;
}

// ---------------------------------------------------------------------------------------
// The grid (ffa_plan_grid.inc, written by `python bench.py --sweep-plans grid`): the same sweep
// over a grid of pairs x head dimension x length x pruned-or-not, for problems away from the
// table's shapes.  A problem takes the nearest row of its (precision, head dimension, pruned)
// class, if one lies within a factor of sqrt 2 in both the number of pairs and the length; where
// that row overrides the rules, its launch kind, wave count and lanes per key are kept and its
// workgroup count is re-cut for the problem at hand.
struct GridRow {
    int override_rules, precision, head_dim, pairs, t, pruned;
    int kind, waves, tpk, n_splits, whole_heads;
    float chosen_us, best_us, rule_us;
};
static const GridRow kPlanGrid[] = {
#define FFA_GRID_ROW(ov, prec, dh, pairs, t, pruned, kind, waves, tpk, ns, whole, chosen, best, rule) \
    {ov, prec, dh, pairs, t, pruned, kind, waves, tpk, ns, whole, chosen, best, rule},
#include "ffa_plan_grid.inc"
#undef FFA_GRID_ROW
    {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0.f, 0.f, 0.f}  // sentinel
};

// The rows of one (precision, head dimension, pruned) class, gathered once: a lookup walks its
// own class (a tenth of the grid), not the whole table.
struct GridClass {
    int precision, head_dim, pruned;
    std::vector<const GridRow*> rows;
};
static const std::vector<GridClass>& grid_classes() {
    static const std::vector<GridClass> classes = [] {
        std::vector<GridClass> out;
        for (const GridRow* r = kPlanGrid; r->precision != 0; ++r) {
            GridClass* c = nullptr;
            for (GridClass& k : out)
                if (k.precision == r->precision && k.head_dim == r->head_dim && k.pruned == r->pruned) c = &k;
            if (c == nullptr) {
                out.push_back(GridClass{r->precision, r->head_dim, r->pruned, {}});
                c = &out.back();
            }
            c->rows.push_back(r);
        }
        return out;
    }();
    return classes;
}

static const GridRow* nearest_grid_row(int precision, int bh, int Dh, int t, int pruned) {
    const GridRow* best = nullptr;
    double best_d = 1e30;
    const GridClass* cls = nullptr;
    for (const GridClass& k : grid_classes())
        if (k.precision == precision && k.head_dim == Dh && k.pruned == pruned) cls = &k;
    if (cls == nullptr) return nullptr;
    for (const GridRow* r : cls->rows) {
        // Within a factor of sqrt(2) both ways, in integers (no integer ratio equals sqrt(2)): the
        // logarithms are taken for the handful of rows that pass, not for the whole class.
        const auto within = [](long long a, long long b) { return a >= b ? a * a <= 2 * b * b : b * b <= 2 * a * a; };
        if (!within(bh, r->pairs) || !within((long long)t + 1, (long long)r->t + 1)) continue;
        const double dp = fabs(log2((double)bh / r->pairs)), dt = fabs(log2((t + 1.0) / (r->t + 1.0)));
        if (dp + dt < best_d) {
            best_d = dp + dt;
            best = r;
        }
    }
    return best;
}

static bool plan_from_grid(int precision, int bh, int Dh, int t, float p, int cus, ffa_launch_plan* plan) {
    if (cus != kTableCus) return false;
    const GridRow* r = nearest_grid_row(precision, bh, Dh, t, p > 0.f ? 1 : 0);
    if (r == nullptr || !r->override_rules) return false;
    const int ntiles = num_tiles(t);
    int whole = 0;
    double n = 1.0;
    if (r->kind == FFA_LAUNCH_TWO_PASS) {
        n = (double)r->n_splits * r->pairs / bh;
    } else if (r->kind == FFA_LAUNCH_SPLIT) {
        if (r->n_splits <= 1 || r->whole_heads >= r->pairs) {
            whole = bh;  // one workgroup per pair
        } else if (r->whole_heads > 0) {
            // Hybrid: whole pairs in multiples of the CU count, the row's piece count for the rest.
            whole = (bh / cus) * cus;
            const int rest = bh - whole;
            if (rest == 0) whole = bh;
            else n = (double)r->n_splits * (r->pairs - r->whole_heads) / rest;
        } else {
            n = (double)r->n_splits * r->pairs / bh;
        }
    }
    int n_splits = (int)(n + 0.5);
    const int cap = max_splits_for(bh - (whole < bh ? whole : 0), t + 1);
    if (n_splits > cap) n_splits = cap;
    if (n_splits > ntiles) n_splits = ntiles;
    if (n_splits < 1) n_splits = 1;
    const int tps = ceil_div(ntiles, n_splits);
    n_splits = ceil_div(ntiles, tps);
    fill(plan, r->kind, r->waves, n_splits, tps);
    plan->threads_per_key = r->tpk;
    plan->keys_per_wave = kTileKeys / r->tpk;
    if (r->kind == FFA_LAUNCH_SPLIT) plan->whole_heads = n_splits == 1 ? bh : whole;
    return validate_plan(*plan, precision, Dh, bh, t, p) == FFA_OK;
}

static int plan_by_rules(int precision, int B, int H, int Dh, int t, float p, int use_default, int cus,
                         ffa_launch_plan* plan);

int plan_source(int precision, int B, int H, int Dh, int t, float p, int cus) {
    ffa_launch_plan tmp;
    if (cus <= 0) cus = 256;
    const int row = plan_from_table(precision, B * H, Dh, t, p, cus, &tmp);
    if (row == kRowOverrides) return 1;
    if (row == kNoRow && plan_from_grid(precision, B * H, Dh, t, p, cus, &tmp)) return 2;
    return 0;
}

int plan_launch(int precision, int B, int H, int Dh, int t, float p, int use_default, int cus,
                ffa_launch_plan* plan) {
    return plan_launch_ex(precision, B, H, Dh, t, p, use_default, cus, /*use_table=*/1, plan);
}

int plan_launch_ex(int precision, int B, int H, int Dh, int t, float p, int use_default, int cus,
                   int use_table, ffa_launch_plan* plan) {
    const int st = plan_by_rules(precision, B, H, Dh, t, p, use_default, cus, plan);
    if (st != FFA_OK || use_default || !use_table) return st;
    ffa_launch_plan from_table;
    const int row = plan_from_table(precision, B * H, Dh, t, p, cus <= 0 ? 256 : cus, &from_table);
    if (row == kRowOverrides) *plan = from_table;
    else if (row == kNoRow && plan_from_grid(precision, B * H, Dh, t, p, cus <= 0 ? 256 : cus, &from_table)) *plan = from_table;
    return FFA_OK;
}

static int plan_by_rules(int precision, int B, int H, int Dh, int t, float p, int use_default, int cus,
                         ffa_launch_plan* plan) {
    if (plan == nullptr) return FFA_ERR_NULL_POINTER;
    if (precision != FFA_PRECISION_F16 && precision != FFA_PRECISION_F32) return FFA_ERR_DTYPE;
    if (Dh != 64 && Dh != 80 && Dh != 128 && Dh != 256) return FFA_ERR_HEAD_DIM;
    if (B <= 0 || H <= 0) return FFA_ERR_SHAPE;
    if (t < 0) return FFA_ERR_TIMESTEP;
    if (!(p >= 0.f)) return FFA_ERR_PROB_THRESH;
    if (cus <= 0) cus = 256;

    const int ntiles = num_tiles(t);
    const int bh = B * H;
    const bool fits_wg = wg_dynamic_lds_bytes(t, 16, precision / 8) <= (size_t)kMaxDynamicLdsBytes;

    if (use_default) {
        // One workgroup per (batch, head); workgroup size by sequence length like the
        // FasterTransformer table (kernel_launch_utils.h:147-154: 64 / 128 / 256 threads).
        // Sequences whose scores outgrow LDS keep them in the workspace instead.
        const int waves = t < 32 ? 1 : (t < 2048 ? 2 : 4);
        fill(plan, fits_wg ? FFA_LAUNCH_WORKGROUP : FFA_LAUNCH_TWO_PASS, wg_waves_for(ntiles, waves), 1,
             ntiles);
        return FFA_OK;
    }

    if (p > 0.f) {
        // Pruning needs the global max and sum before it may touch V: either one workgroup per
        // (b,h) with the scores in LDS, or the two-pass pair of kernels cut along the sequence.
        // The second launch and the merge of the pieces cost about a dozen tile-times of narrow
        // rows, and a cut in two or three gains little, so cutting a pair into n pieces pays from
        // ntiles width (1 - 1.7/n) >= 12 on, and never with a pair or more per CU (grid sweep: 16
        // and 32 pairs go two-pass from 1024 keys, 64 pairs from 2048, 128 pairs from 8192; at 256
        // pairs and more the one-workgroup kernel wins at every length).
        // Both kernels of the pair carry only half of a tile's loads each, so from 4096 keys on
        // they want twice the workgroups of the exact path -- about two 8-wave workgroups per CU;
        // below that one workgroup per CU (grid sweep: 32 pairs x 1024 keys 8.4 vs 9.1 us).
        int n_splits = (ntiles >= 64 ? 2 : 1) * cus / bh;
        if (n_splits > ntiles) n_splits = ntiles;
        const int cap = max_splits_for(bh, t + 1);
        if (n_splits > cap) n_splits = cap;
        if (n_splits < 1) n_splits = 1;
        // Wide rows are cut earlier (a tile of 32 chunks per key weighs two of 8 in this balance:
        // 64 pairs x 768 keys of Dh 256 16-20 % ahead in 7 pieces), nothing below ten tiles.
        const int nch = Dh * (precision / 8) / 16;
        const double width = nch >= 32 ? 2.0 : nch >= 16 ? 1.3 : 1.0;
        const bool cut_pays = bh < cus && n_splits > 1 && ntiles >= 10 &&
                              ntiles * width * (n_splits - 1.7) >= 12.0 * n_splits;
        if (fits_wg && !cut_pays) {
            // Waves: one tile or two per wave up to 8 waves; 16 waves only for very long sequences
            // with a whole number of pairs per CU (512 pairs x 8192 keys); 4 waves when some CUs get
            // a second workgroup (320 pairs: 5-9 % at every length).
            int want = ntiles <= 5 ? 4 : 8;
            if (bh % cus == 0 && ntiles >= 128) want = 16;
            if (bh > cus && bh % cus != 0) want = 4;
            int w = wg_waves_for(ntiles, want);
            // Six or seven tiles take 8 waves, not 4 (one round instead of two: 10-12 % at 384
            // keys), and 16 where the rows are widest and the pairs few (Dh 256: 12.5 vs 17.6 us).
            if (ntiles > 5 && want >= 8 && w < 8 && bh <= 2 * cus) w = 8;
            if (ntiles > 5 && ntiles < 10 && nch >= 32 && 4 * bh <= cus) w = 16;
            fill(plan, FFA_LAUNCH_WORKGROUP, w, 1, ntiles);
            return FFA_OK;
        }
        const int tps = ceil_div(ntiles, n_splits);
        n_splits = ceil_div(ntiles, tps);
        fill(plan, FFA_LAUNCH_TWO_PASS, tps <= 4 ? 4 : 8, n_splits, tps);
        return FFA_OK;
    }

    // Exact path.  Measured on MI355X: the launch runs best with about one 4-wave workgroup
    // per CU, each walking a long run of tiles, and with as few cross-workgroup merges as
    // possible at the END of the kernel (a merge is a chain of three memory round trips).
    //  - At least one (batch, head) pair per CU: whole pairs go to single workgroups in
    //    multiples of the CU count (every CU gets the same number, LDS-only merge); only the
    //    remainder is split, into ceil(CUs/rest) pieces per pair, so that the pieces also
    //    cover all CUs and are done, merges included, long before the whole pairs are.
    //  - Fewer pairs than CUs: floor(CUs/pairs) pieces per pair (one workgroup per CU), but
    //    never so many that a wave is left without a tile -- and only where the split saves more
    //    than its merge costs.  The merge chain is worth the time of about ten 16 KiB tiles, so a
    //    cut into n pieces pays from ntiles (tile bytes / 16 KiB) (1 - 1/n) >= 10 on (grid sweep:
    //    at Dh = 64 fp16 128 pairs stay whole up to 1024 keys, 16 pairs up to 256); below that
    //    every pair is one workgroup of up to 8 waves.
    //  - Long sequences with a whole number of pairs per CU: the one-workgroup kernel with 16
    //    waves (separate K and V phases; 512 pairs x 8192 keys: all exact launches within 1 %).
    //    With a remainder the hybrid launch is 15-20 % ahead (320 pairs from 4096 keys on).
    //  - Wide rows (16 or more 16-byte chunks per key: Dh 128 / 256 in fp16, Dh 64 / 128 in fp32):
    //    four lanes per key, so that a tile's loads are all in flight at once (grid sweep: 5-25 %
    //    at every length below two pairs per CU), with 8 waves per workgroup below one pair per CU.
    int whole = (bh / cus) * cus;
    const int rest = bh - whole;
    if (rest == 0 && ntiles >= 64 && fits_wg) {
        fill(plan, FFA_LAUNCH_WORKGROUP, 16, 1, ntiles);
        return FFA_OK;
    }
    const int waves = wg_waves_for(ntiles, 4);
    int n_splits = 1;
    if (whole > 0) {
        if (rest > 0 && ntiles >= 8) n_splits = ceil_div(cus, rest);
    } else {
        n_splits = cus / bh;
    }
    const int nch = Dh * (precision / 8) / 16;  // 16-byte chunks per key: a 64-key tile is nch x 2 KiB
    const int tpk = (nch >= 16 && bh < 2 * cus && tpk_supported(precision, Dh, 4)) ? 4 : 1;
    // Never so many pieces that a wave is left without work: with four lanes per key a 64-key
    // tile is four units of work (16 x 256 at 384 keys: 7.5 us in 7 pieces, 8.6 in 4, 9.8 whole).
    const int most = ceil_div(ntiles * tpk, waves);
    if (n_splits > most) n_splits = most;
    const int cap = max_splits_for(rest > 0 ? rest : bh, t + 1);
    if (n_splits > cap) n_splits = cap;
    if (n_splits > ntiles) n_splits = ntiles;
    if (n_splits < 1) n_splits = 1;
    // A cut pays once it saves more than the merge costs: about ten 16 KiB tile-times where the
    // whole pairs already keep half the CUs busy (2 or 3 pieces), about seven where they leave
    // three quarters or more of them idle (32 pairs x 760 keys: 5.9 us whole, 4.6 us in 8 pieces).
    // Wide rows with four lanes per key: from five tiles on, and about a dozen tile-times.
    const long long cut_cost = tpk > 1 ? 100 : n_splits >= 4 ? 56 : 80;
    if (whole == 0 && n_splits > 1 &&
        ((long long)ntiles * nch * (n_splits - 1) < cut_cost * n_splits || (tpk > 1 && ntiles < 5)))
        n_splits = 1;
    const int tps = ceil_div(ntiles, n_splits);
    n_splits = ceil_div(ntiles, tps);
    if (n_splits == 1) {
        // Nothing is cut: one workgroup per pair.  Below one pair per CU the idle CUs are made up
        // for with 8 waves per workgroup (160 pairs, 1000 keys: 9.3 vs 9.8 us).
        const int w = bh < cus ? wg_waves_for(ntiles * tpk, 8) : waves;
        fill(plan, FFA_LAUNCH_SPLIT, tpk > 1 && w < 4 ? 4 : w, 1, ntiles);
        plan->whole_heads = bh;
    } else {
        const int w = tpk > 1 ? (bh < cus ? 8 : 4) : waves;
        fill(plan, FFA_LAUNCH_SPLIT, w, n_splits, tps);
        plan->whole_heads = whole;
    }
    plan->threads_per_key = tpk;
    plan->keys_per_wave = kTileKeys / tpk;
    return FFA_OK;
}

// Whether the exact split kernel exists with `tpk` lanes per key for this element size and
// head dimension: the chunks of a key must divide evenly and a tile's K loads and V loads
// must each fit one group of at most 8.
bool tpk_supported(int precision, int head_dim, int tpk) {
    if (tpk == 1) return true;
    if ((tpk != 2 && tpk != 4) || head_dim == 80) return false;
    const int nch = head_dim * (precision / 8) / 16;
    const int lpr = nch <= 8 ? 8 : nch <= 16 ? 16 : nch <= 32 ? 32 : 64;
    const int rpi = kTileKeys / lpr, kpt = kTileKeys / tpk;
    return nch % tpk == 0 && nch / tpk <= 8 && kpt % rpi == 0 && kpt / rpi <= 8;
}

int validate_plan(const ffa_launch_plan& plan, int precision, int head_dim, int bh, int t, float p) {
    const int w = plan.waves_per_wg;
    // Powers of two up to 16; the exact split kernel (one lane per key) also takes 3, 5, 6, 7.
    const bool pow2 = w == 1 || w == 2 || w == 4 || w == 8 || w == 16;
    if (!pow2 && !(plan.kind == FFA_LAUNCH_SPLIT && plan.threads_per_key == 1 && w >= 1 && w <= 8)) return FFA_ERR_PLAN;
    const int tpk = plan.threads_per_key;
    if ((tpk != 1 && tpk != 2 && tpk != 4) || plan.keys_per_wave != kTileKeys / tpk) return FFA_ERR_PLAN;
    // More than one lane per key exists in the exact split kernel only, with 4 or 8 waves.
    if (tpk > 1 && (plan.kind != FFA_LAUNCH_SPLIT || (w != 4 && w != 8) || !tpk_supported(precision, head_dim, tpk)))
        return FFA_ERR_PLAN;
    if (plan.n_splits < 1 || plan.n_splits > kMaxSplits || plan.tiles_per_split < 1) return FFA_ERR_PLAN;
    if (plan.combine != FFA_COMBINE_FUSED && plan.combine != FFA_COMBINE_KERNEL) return FFA_ERR_PLAN;
    const int ntiles = num_tiles(t);
    switch (plan.kind) {
        case FFA_LAUNCH_WORKGROUP:
            if (plan.n_splits != 1 || plan.whole_heads != 0) return FFA_ERR_PLAN;
            if (wg_dynamic_lds_bytes(t, w, precision / 8) > (size_t)kMaxDynamicLdsBytes)
                return FFA_ERR_TOO_LONG;
            return FFA_OK;
        case FFA_LAUNCH_SPLIT:
            if (p > 0.f) return FFA_ERR_PLAN;  // the split kernel is the exact path only
            if (w > 8) return FFA_ERR_PLAN;
            if (plan.whole_heads < 0 || plan.whole_heads > bh) return FFA_ERR_PLAN;
            if (plan.whole_heads < bh && (long long)plan.n_splits * plan.tiles_per_split < ntiles)
                return FFA_ERR_PLAN;
            // Unsplit pairs are one workgroup each however many there are; the cap is on splitting.
            if (plan.n_splits > 1 && (long long)(bh - plan.whole_heads) * plan.n_splits > 4 * kMaxSplitWorkgroups)
                return FFA_ERR_PLAN;
            return FFA_OK;
        case FFA_LAUNCH_TWO_PASS:
            if (w > 8 || plan.whole_heads != 0 || plan.combine != FFA_COMBINE_FUSED) return FFA_ERR_PLAN;
            if ((long long)plan.n_splits * plan.tiles_per_split < ntiles) return FFA_ERR_PLAN;
            if (plan.n_splits > 1 && (long long)bh * plan.n_splits > 4 * kMaxSplitWorkgroups) return FFA_ERR_PLAN;
            return FFA_OK;
        default:
            return FFA_ERR_PLAN;
    }
}

}  // namespace ffa
