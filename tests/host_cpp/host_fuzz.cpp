// Host-logic fuzz of the C ABI (argument validation, planning, workspace carving), built by
// tests/test_host_cpp.py from ffa_api.cpp + ffa_plan.cpp with AddressSanitizer and
// UndefinedBehaviorSanitizer and run on the CPU.  The launchers that ffa_kernels.hip provides are
// replaced by stubs that launch nothing and check what the host code hands them: a plan that
// passed validation, a grid within the documented bounds, workspace regions that lie inside the
// caller's buffer and do not overlap.  Pointers are made-up addresses; nothing dereferences them.
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#include <random>

#include "ffa_c_api.h"
#include "ffa_host.h"

#define CHECK(cond)                                                                   \
    do {                                                                              \
        if (!(cond)) {                                                                \
            fprintf(stderr, "%s:%d: check failed: %s\n", __FILE__, __LINE__, #cond); \
            abort();                                                                  \
        }                                                                             \
    } while (0)

namespace {
struct Expect {
    uintptr_t ws_lo = 0, ws_hi = 0;  // the caller's workspace, as integers (made-up addresses)
    long launches = 0, fills = 0;
} g;
char g_scratch_stand_in[1];  // address only
}  // namespace

namespace ffa {

int query_compute_units() { return 256; }
int current_device() { return 0; }
int static_scratch_address(void** ptr) {
    *ptr = reinterpret_cast<void*>(uintptr_t{0x7000000000});
    return FFA_OK;
}
int launch_fill_u32(unsigned int* p, size_t n, unsigned int, void*) {
    CHECK(p != nullptr || n == 0);
    ++g.fills;
    return FFA_OK;
}
int launch_init_cache(int precision, void* k_dst, void* v_dst, const void* k_src, const void* v_src, int B, int H,
                      int L, int Lmax, int Dh, void*) {
    CHECK(elem_bytes(precision) != 0 || precision == 16 || precision == 32);
    CHECK(k_dst && v_dst && k_src && v_src && B > 0 && H > 0 && L > 0 && L <= Lmax);
    CHECK(Dh == 64 || Dh == 80 || Dh == 128 || Dh == 256);
    return FFA_OK;
}

static void inside(const void* p, size_t bytes) {
    const uintptr_t c = reinterpret_cast<uintptr_t>(p);
    CHECK(c >= g.ws_lo && bytes <= g.ws_hi - g.ws_lo && c - g.ws_lo <= g.ws_hi - g.ws_lo - bytes);
}

int launch_decode(const DecodeArgs& a, const ffa_launch_plan& plan, const WorkspaceView& ws) {
    ++g.launches;
    const int bh = a.B * a.H;
    CHECK(validate_plan(plan, planner_precision(a.precision), a.Dh, bh, a.t, a.p) == FFA_OK);
    CHECK(a.t >= 0 && a.t < a.Lmax && a.p >= 0.f);
    CHECK(a.q && a.k && a.v && a.k_cache && a.v_cache && a.out);
    if (plan.kind == FFA_LAUNCH_SPLIT) {
        CHECK(a.p == 0.f && a.kept_count == nullptr && a.skip_mask == nullptr);
        const int split_heads = bh - plan.whole_heads;
        CHECK(split_heads >= 0);
        if (plan.n_splits > 1 && split_heads > 0) {
            const size_t slots = (size_t)split_heads * plan.n_splits;
            inside(ws.cnt, (size_t)bh * kCounterStride * 4);
            inside(ws.acc, slots * (a.Dh + kSlotTailFloats) * 4);
            CHECK(reinterpret_cast<const char*>(ws.acc) >= reinterpret_cast<const char*>(ws.cnt) + (size_t)bh * kCounterStride * 4);
            CHECK((long long)plan.n_splits * plan.tiles_per_split >= num_tiles(a.t));
        }
    } else if (plan.kind == FFA_LAUNCH_TWO_PASS) {
        const size_t slots = (size_t)bh * plan.n_splits;
        inside(ws.cnt, (size_t)bh * kCounterStride * 4);
        inside(ws.ml, slots * 2 * 4);
        inside(ws.acc, slots * a.Dh * 4);
        CHECK(ws.score_stride >= a.t + 1 && ws.score_stride % 64 == 0);
        inside(ws.scores, (size_t)bh * ws.score_stride * 4);
        CHECK(reinterpret_cast<const char*>(ws.acc) >= reinterpret_cast<const char*>(ws.ml) + slots * 8);
        CHECK(reinterpret_cast<const char*>(ws.scores) >= reinterpret_cast<const char*>(ws.acc) + slots * a.Dh * 4);
    } else {
        CHECK(plan.kind == FFA_LAUNCH_WORKGROUP);
        CHECK(wg_dynamic_lds_bytes(a.t, plan.waves_per_wg, elem_bytes(a.precision)) <= (size_t)kMaxDynamicLdsBytes);
    }
    if (a.cache_indir) CHECK(a.beam_width >= 1 && a.B % a.beam_width == 0);
    return FFA_OK;
}

}  // namespace ffa

int main(int argc, char** argv) {
    const long iters = argc > 1 ? atol(argv[1]) : 200000;
    std::mt19937_64 rng(argc > 2 ? atoll(argv[2]) : 12345);
    auto pick = [&](std::initializer_list<long long> v) { return *(v.begin() + rng() % v.size()); };
    auto uni = [&](long long lo, long long hi) { return lo + (long long)(rng() % (unsigned long long)(hi - lo + 1)); };
    long ok = 0, rejected = 0;
    for (long it = 0; it < iters; ++it) {
        // Half of the calls are tame (every argument from its valid range, so that most reach a
        // launch), the other half draw one argument in eight from a list of bad values.
        const bool wild = rng() % 2;
        auto pick2 = [&](std::initializer_list<long long> good, std::initializer_list<long long> bad) {
            return (wild && rng() % 8 == 0) ? pick(bad) : pick(good);
        };
        const int precision = (int)pick2({16, 16, 32, 32, FFA_PRECISION_BF16}, {8, 0, -1});
        const int B = (int)pick2({1, 1, 2, 5, 8, 10, 16, 64}, {0, -3, 5000, 70000});
        const int H = (int)pick2({1, 16, 32, 32, 40}, {0, 4096});
        const int Dh = (int)pick2({64, 64, 80, 128, 256}, {32, 96, 0});
        const int Lmax = (int)pick2({8, 64, 65, 1128, 1256, 2256, 8256, 16384, 70000}, {1, 0, -1});
        const int t = (int)pick2({0, 1, Lmax / 2, Lmax - 1, Lmax - 2, 63 % (Lmax > 0 ? Lmax : 1), 1000 % (Lmax > 0 ? Lmax : 1)},
                                 {-1, Lmax, Lmax + 5});
        const float p = wild && rng() % 8 == 0 ? (float[]){-1.f, NAN, INFINITY}[rng() % 3]
                                               : (float[]){0.f, 0.f, 0.f, 1e-4f, 1e-2f, 1.f}[rng() % 6];
        // Made-up device addresses.
        auto addr = [&](bool maybe_bad) -> void* {
            const int r = wild ? (int)(rng() % 32) : 31;
            if (maybe_bad && r == 0) return nullptr;
            if (maybe_bad && r == 1) return reinterpret_cast<void*>(uintptr_t{0x10000008});
            return reinterpret_cast<void*>(uintptr_t{0x10000000} + 0x1000 * (rng() % 1000));
        };
        ffa_launch_plan plan;
        const ffa_launch_plan* plan_p = nullptr;
        const int plan_mode = (int)(rng() % 4);
        if (plan_mode == 1) {  // the library's own plan, explicitly
            if (ffa_plan_launch(precision, B, H, Dh, t, p, (int)(rng() % 2), 256, &plan) == FFA_OK) plan_p = &plan;
        } else if (plan_mode == 2) {  // anything
            plan.kind = (int)pick({0, 1, 2, 3, -1});
            plan.waves_per_wg = (int)pick({1, 2, 3, 4, 5, 8, 16, 0, 32});
            plan.threads_per_key = (int)pick({1, 1, 2, 4, 3, 0});
            plan.keys_per_wave = rng() % 8 ? 64 / (plan.threads_per_key > 0 ? plan.threads_per_key : 1) : 7;
            plan.n_splits = (int)pick({1, 2, 4, 8, 16, 128, 129, 0, -2});
            plan.tiles_per_split = (int)pick({1, 2, 4, 16, 64, 1000, 0});
            plan.combine = (int)pick({0, 0, 1, 2});
            plan.whole_heads = (int)pick({0, 0, 256, 1, B > 0 && H > 0 ? B * H : 0, -1, 1 << 30});
            plan_p = &plan;
        }
        // Workspace: full size, the plan's own size, too small, or none.
        size_t full = ffa_workspace_bytes(B, H, Dh, Lmax);
        if (full > (size_t)1 << 40) full = (size_t)1 << 40;
        size_t ws_bytes = full;
        const int ws_mode = wild ? (int)(rng() % 5) : (int)(rng() % 2);
        if (ws_mode == 1 && plan_p && B > 0 && H > 0 && (long long)B * H < (1 << 24))
            ws_bytes = ffa::plan_workspace_bytes(*plan_p, B * H, Dh > 0 ? Dh : 64, Lmax > 0 ? Lmax : 1);
        if (ws_mode == 2) ws_bytes = full / 2;
        if (ws_mode == 3) ws_bytes = (size_t)uni(0, 4096);
        void* ws = ws_mode == 4 ? nullptr : reinterpret_cast<void*>(uintptr_t{0x20000000});
        if (ws_bytes > (size_t)1 << 40) ws_bytes = (size_t)1 << 40;
        g.ws_lo = reinterpret_cast<uintptr_t>(ws);
        g.ws_hi = g.ws_lo + (ws ? ws_bytes : 0);

        ffa_token_transform tr = {addr(true), nullptr, addr(true), (int)pick2({0, 64, 32}, {33, -2, 512}), 10000.f};
        ffa_beam_indirection bm = {static_cast<const int*>(addr(true)), (int)pick2({1, 1, 2, 5}, {0, 3})};
        const int entry = (int)(rng() % 5);
        int rc;
        void *q = addr(true), *k = addr(true), *v = addr(true), *kc = addr(true), *vc = addr(true), *out = addr(true);
        const int* sl = rng() % 2 ? static_cast<const int*>(addr(false)) : nullptr;
        const int ronp = (int)(rng() % 2);
        if (entry == 0 && (precision == 16 || precision == 32)) {
            rc = precision == 16
                     ? ffa_attention_f16(B, H, Dh, Lmax, 0.125f, t, (uint16_t*)q, (uint16_t*)k, (uint16_t*)v, (uint16_t*)kc,
                                         (uint16_t*)vc, (uint16_t*)out, sl, p, plan_p, ronp, ws, ws_bytes, nullptr)
                     : ffa_attention_f32(B, H, Dh, Lmax, 0.125f, t, (float*)q, (float*)k, (float*)v, (float*)kc, (float*)vc,
                                         (float*)out, sl, p, plan_p, ronp, ws, ws_bytes, nullptr);
        } else if (entry == 1) {
            rc = ffa_attention_diag(precision, B, H, Dh, Lmax, 0.125f, t, q, k, v, kc, vc, out, sl, p, plan_p, ronp, ws,
                                    ws_bytes, (uint32_t*)addr(true), (uint8_t*)addr(true), nullptr);
        } else if (entry == 2) {
            rc = ffa_attention_ex(precision, B, H, Dh, Lmax, 0.125f, t, q, k, v, kc, vc, out, sl, p, plan_p, ronp,
                                  rng() % 2 ? &tr : nullptr, rng() % 2 ? &bm : nullptr, ws, ws_bytes, nullptr);
        } else if (entry == 3) {
            // The library's own array stands where the workspace would: bounds are its size.
            g.ws_lo = uintptr_t{0x7000000000};
            g.ws_hi = g.ws_lo + FFA_STATIC_SCRATCH_BYTES;
            rc = ffa_attention_static_scratch(precision, B, H, Dh, Lmax, 0.125f, t, q, k, v, kc, vc, out, sl, p, plan_p,
                                              ronp, rng() % 2 ? &tr : nullptr, rng() % 2 ? &bm : nullptr, nullptr);
        } else {
            rc = ffa_init_cache_f16((uint16_t*)kc, (uint16_t*)vc, (const uint16_t*)k, (const uint16_t*)v, B,
                                    (int)pick({0, 1, 1000, Lmax, Lmax + 1, -1}), Lmax, Dh, H, nullptr);
        }
        CHECK(rc >= FFA_OK && rc <= FFA_ERR_BEAM);
        CHECK(ffa_status_string(rc) != nullptr);
        (rc == FFA_OK ? ok : rejected)++;

        // Whatever the planner returns validates, fits the workspace the library asks for, and
        // never splits finer than the documented bounds.
        if (B > 0 && H > 0 && (long long)B * H <= (1 << 24) && (Dh == 64 || Dh == 80 || Dh == 128 || Dh == 256) &&
            t >= 0 && Lmax > t && (precision == 16 || precision == 32) && p >= 0.f && !isinf(p)) {
            for (int use_default = 0; use_default < 2; ++use_default) {
                ffa_launch_plan pl;
                const int cus = (int)pick({256, 256, 304, 64, 1, 0});
                if (ffa_plan_launch(precision, B, H, Dh, t, p, use_default, cus, &pl) != FFA_OK) continue;
                const int vr = ffa::validate_plan(pl, precision, Dh, B * H, t, p);
                if (!(vr == FFA_OK || (vr == FFA_ERR_TOO_LONG && use_default)))
                    fprintf(stderr, "planner: prec %d B %d H %d Dh %d t %d p %g default %d cus %d -> kind %d waves %d tpk %d "
                            "splits %d tps %d whole %d: %s\n", precision, B, H, Dh, t, p, use_default, cus, pl.kind,
                            pl.waves_per_wg, pl.threads_per_key, pl.n_splits, pl.tiles_per_split, pl.whole_heads,
                            ffa_status_string(vr));
                CHECK(vr == FFA_OK || (vr == FFA_ERR_TOO_LONG && use_default));
                CHECK(ffa::plan_workspace_bytes(pl, B * H, Dh, Lmax) <= ffa_workspace_bytes(B, H, Dh, Lmax));
                CHECK(pl.n_splits >= 1 && pl.n_splits <= ffa::kMaxSplits);
            }
        }
    }
    printf("host fuzz: %ld calls, %ld accepted (%ld launches, %ld fills), %ld rejected\n", iters, ok, g.launches, g.fills,
           rejected);
    CHECK(ok > iters / 10 && g.launches > iters / 20 && rejected > iters / 10);
    return 0;
}
