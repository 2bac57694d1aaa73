"""CPU tests of the host side of the C ABI: the library loads, exports every symbol that
include/ffa_c_api.h declares, validates arguments before touching the GPU, and the launch
planner produces consistent plans.  No kernel is launched here."""
import ctypes as C
import os
import re

import pytest

from fastforwardattention_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "ffa_c_api.h")


@pytest.fixture(scope="module")
def lib():
    return capi.load()


def _declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ffa_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound(lib):
    names = _declared_functions()
    assert len(names) >= 11
    for n in names:
        assert hasattr(lib, n), f"{n} declared in ffa_c_api.h but not exported"
    assert sorted(capi.SIGNATURES) == names, "capi.SIGNATURES out of sync with the header"


def test_version_and_status_strings(lib):
    assert lib.ffa_api_version() == 1
    seen = set()
    for code in range(0, 15):
        s = capi.status_string(code)
        assert s and s != "unknown status"
        seen.add(s)
    assert len(seen) == 15
    assert capi.status_string(99) == "unknown status"


def test_struct_layout_matches_header():
    assert C.sizeof(capi.LaunchPlan) == 32


# dummy 16-byte aligned non-null "device pointers": validation must reject the call
# before any of them is dereferenced or a kernel is launched
P = C.c_void_p(0x1000)


def _attn(lib, precision=16, B=2, H=4, Dh=64, Lmax=128, scale=0.125, t=10, q=P, k=P, v=P, kc=P,
          vc=P, out=P, sl=None, p=0.0, plan=None, rnp=1, ws=None, ws_bytes=0):
    return lib.ffa_attention_diag(precision, B, H, Dh, Lmax, scale, t, q, k, v, kc, vc, out, sl, p,
                                  C.byref(plan) if plan is not None else None, rnp, ws, ws_bytes,
                                  None, None, None)


def test_attention_argument_validation(lib):
    wg = capi.make_plan(capi.FFA_LAUNCH_WORKGROUP, 4, 1, 1)
    assert _attn(lib, precision=8, plan=wg) == 2          # dtype
    assert _attn(lib, Dh=96, plan=wg) == 3                # head dim: 64, 80, 128, 256 like the reference
    assert _attn(lib, B=0, plan=wg) == 4
    assert _attn(lib, H=-1, plan=wg) == 4
    assert _attn(lib, t=-1, plan=wg) == 5
    assert _attn(lib, t=128, Lmax=128, plan=wg) == 5      # the reference writes out of bounds here
    assert _attn(lib, p=-0.5, plan=wg) == 10
    assert _attn(lib, p=float("nan"), plan=wg) == 10
    assert _attn(lib, q=None, plan=wg) == 1
    assert _attn(lib, out=None, plan=wg) == 1
    assert _attn(lib, kc=C.c_void_p(0x1008), plan=wg) == 6
    # malformed plans
    assert _attn(lib, plan=capi.make_plan(capi.FFA_LAUNCH_WORKGROUP, 3, 1, 1)) == 8
    assert _attn(lib, plan=capi.make_plan(capi.FFA_LAUNCH_WORKGROUP, 4, 2, 1)) == 8
    assert _attn(lib, plan=capi.make_plan(7, 4, 1, 1)) == 8
    assert _attn(lib, plan=capi.make_plan(capi.FFA_LAUNCH_SPLIT, 4, 1, 1, combine=5)) == 8
    assert _attn(lib, plan=capi.make_plan(capi.FFA_LAUNCH_SPLIT, 4, 1, 1, whole_heads=9)) == 8   # B*H = 8
    assert _attn(lib, plan=capi.make_plan(capi.FFA_LAUNCH_SPLIT, 4, 1, 1, whole_heads=-1)) == 8
    assert _attn(lib, plan=capi.make_plan(capi.FFA_LAUNCH_WORKGROUP, 4, 1, 1, whole_heads=2)) == 8
    assert _attn(lib, t=100, plan=capi.make_plan(capi.FFA_LAUNCH_SPLIT, 4, 1, 1)) == 8   # 1 tile < 2 needed
    assert _attn(lib, p=0.1, plan=capi.make_plan(capi.FFA_LAUNCH_SPLIT, 4, 2, 1)) == 8   # split is exact only
    assert _attn(lib, plan=capi.make_plan(capi.FFA_LAUNCH_SPLIT, 16, 2, 1)) == 8
    # lanes per key: 1, 2 or 4; more than one only in split plans with 4 or 8 waves and only for
    # head dimensions whose tile then fits one group of loads
    ok = lambda **kw: _attn(lib, t=100, ws=P, ws_bytes=1 << 20, **kw)
    assert ok(plan=capi.make_plan(capi.FFA_LAUNCH_SPLIT, 4, 2, 1, threads_per_key=3)) == 8
    bad = capi.make_plan(capi.FFA_LAUNCH_SPLIT, 4, 2, 1, threads_per_key=2)
    bad.keys_per_wave = 64
    assert ok(plan=bad) == 8
    assert ok(plan=capi.make_plan(capi.FFA_LAUNCH_WORKGROUP, 4, 1, 2, threads_per_key=2)) == 8
    assert ok(plan=capi.make_plan(capi.FFA_LAUNCH_TWO_PASS, 4, 2, 1, threads_per_key=2)) == 8
    assert ok(plan=capi.make_plan(capi.FFA_LAUNCH_SPLIT, 2, 2, 1, threads_per_key=2)) == 8
    assert ok(Dh=80, plan=capi.make_plan(capi.FFA_LAUNCH_SPLIT, 4, 2, 1, threads_per_key=2)) == 8
    assert ok(Dh=256, plan=capi.make_plan(capi.FFA_LAUNCH_SPLIT, 4, 2, 1, threads_per_key=2)) == 8      # 16 loads per tile
    assert ok(Dh=256, precision=32, plan=capi.make_plan(capi.FFA_LAUNCH_SPLIT, 4, 2, 1, threads_per_key=4)) == 8
    # split plan without / with too small a workspace
    sp = capi.make_plan(capi.FFA_LAUNCH_SPLIT, 4, 2, 1)
    assert _attn(lib, t=100, plan=sp) == 7
    assert _attn(lib, t=100, plan=sp, ws=P, ws_bytes=64) == 7
    # two-pass plans: coverage, wave count, whole_heads, workspace
    tp = capi.make_plan(capi.FFA_LAUNCH_TWO_PASS, 4, 2, 1)
    assert _attn(lib, t=100, plan=tp) == 7
    assert _attn(lib, t=100, plan=tp, ws=P, ws_bytes=4096) == 7                      # scores do not fit
    assert _attn(lib, t=200, Lmax=256, plan=tp, ws=P, ws_bytes=1 << 20) == 8         # 2 tiles < 4 needed
    assert _attn(lib, t=100, plan=capi.make_plan(capi.FFA_LAUNCH_TWO_PASS, 16, 2, 1), ws=P, ws_bytes=1 << 20) == 8
    assert _attn(lib, t=100, plan=capi.make_plan(capi.FFA_LAUNCH_TWO_PASS, 4, 2, 1, whole_heads=1), ws=P,
                 ws_bytes=1 << 20) == 8
    assert _attn(lib, t=100, plan=capi.make_plan(capi.FFA_LAUNCH_TWO_PASS, 4, 2, 1, combine=1), ws=P,
                 ws_bytes=1 << 20) == 8
    # one-workgroup launch whose scores cannot fit in LDS
    assert _attn(lib, t=60000, Lmax=65536, plan=wg) == 9


def test_static_scratch_entry_validates_before_any_launch(lib):
    """ffa_attention_static_scratch: bad arguments, malformed plans and plans whose workspace
    need exceeds the library's static array are refused on the host, before the GPU is touched."""
    def call(precision=16, B=2, H=4, Dh=64, Lmax=128, t=10, q=P, p=0.0, plan=None):
        return lib.ffa_attention_static_scratch(precision, B, H, Dh, Lmax, 0.125, t, q, P, P, P, P, P, None, p,
                                                C.byref(plan) if plan is not None else None, 1, None, None, None)
    wg = capi.make_plan(capi.FFA_LAUNCH_WORKGROUP, 4, 1, 1)
    assert call(precision=8, plan=wg) == capi.FFA_ERR_DTYPE
    assert call(Dh=96, plan=wg) == capi.FFA_ERR_HEAD_DIM
    assert call(t=128, plan=wg) == capi.FFA_ERR_TIMESTEP
    assert call(q=None, plan=wg) == capi.FFA_ERR_NULL_POINTER
    assert call(p=-1.0, plan=wg) == capi.FFA_ERR_PROB_THRESH
    assert call(plan=capi.make_plan(capi.FFA_LAUNCH_WORKGROUP, 3, 1, 1)) == capi.FFA_ERR_PLAN
    # 64 pairs x 20032 scores x 4 B = 5.1 MB of two-pass scores > 4 MiB
    nt = 20000 // 64 + 1
    big = capi.make_plan(capi.FFA_LAUNCH_TWO_PASS, 4, 4, -(-nt // 4))
    assert call(B=2, H=32, Lmax=20001, t=20000, p=0.01, plan=big) == capi.FFA_ERR_SCRATCH_LIMIT
    # split partials: 8192 pieces x (8 + 4*256) B = 8.4 MB
    many = capi.make_plan(capi.FFA_LAUNCH_SPLIT, 1, 64, 1)
    assert call(B=4, H=32, Dh=256, Lmax=4097, t=4095, plan=many) == capi.FFA_ERR_SCRATCH_LIMIT
    assert "scratch" in capi.status_string(capi.FFA_ERR_SCRATCH_LIMIT)


def test_attention_ex_validates_before_any_launch(lib):
    """ffa_attention_ex: element types, the token transform's fields and the beam table are checked
    on the host.  (The transform itself runs inside the decode kernels and needs no workspace.)"""
    def call(precision=16, Dh=64, t=10, rotary=0, q_bias=None, ws=None, ws_bytes=0, plan=None, transform=True,
             beams=None):
        tt = capi.TokenTransform(q_bias=q_bias, rotary_embedding_dim=rotary) if transform else None
        return lib.ffa_attention_ex(precision, 2, 4, Dh, 128, 0.125, t, P, P, P, P, P, P, None, 0.0,
                                    C.byref(plan) if plan is not None else None, 1,
                                    C.byref(tt) if tt is not None else None,
                                    C.byref(beams) if beams is not None else None, ws, ws_bytes, None)
    wg = capi.make_plan(capi.FFA_LAUNCH_WORKGROUP, 4, 1, 1)
    assert call(precision=8, plan=wg) == capi.FFA_ERR_DTYPE
    assert call(precision=17, plan=wg) == capi.FFA_ERR_DTYPE
    for rd in (-1, 7, 66):
        assert call(rotary=rd, plan=wg) == capi.FFA_ERR_TRANSFORM
    assert call(rotary=32, q_bias=C.c_void_p(0x1008), plan=wg) == capi.FFA_ERR_TRANSFORM
    # with a transform a sequence-split plan still needs exactly its own workspace, no more
    cut = capi.make_plan(capi.FFA_LAUNCH_SPLIT, 1, 2, 1)
    need = 256 + 256 + 8 * 2 * 64 * 4            # counters, (max, sum) of 16 pieces, 16 partials of 64 floats
    for prec in (16, 32, capi.FFA_PRECISION_BF16):
        assert call(precision=prec, t=100, rotary=32, plan=cut) == capi.FFA_ERR_WORKSPACE
        assert call(precision=prec, t=100, rotary=32, plan=cut, ws=P, ws_bytes=need - 1) == capi.FFA_ERR_WORKSPACE
    assert "rotary" in capi.status_string(capi.FFA_ERR_TRANSFORM)
    # beam indirection: batch 2 here
    BI = capi.BeamIndirection
    assert call(transform=False, plan=wg, beams=BI(None, 2)) == capi.FFA_ERR_BEAM
    assert call(transform=False, plan=wg, beams=BI(0x1002, 2)) == capi.FFA_ERR_BEAM      # not 4-byte aligned
    for bw in (0, -1, 3, 4):
        assert call(transform=False, plan=wg, beams=BI(0x1000, bw)) == capi.FFA_ERR_BEAM
    assert "beam" in capi.status_string(capi.FFA_ERR_BEAM)


def test_init_cache_argument_validation(lib):
    f = lib.ffa_init_cache_f16
    assert f(P, P, P, P, 1, 8, 4, 64, 2, None) == 4       # L > Lmax
    assert f(P, P, P, P, 1, 8, 16, 96, 2, None) == 3
    assert f(None, P, P, P, 1, 8, 16, 64, 2, None) == 1
    assert f(P, P, None, P, 1, 8, 16, 64, 2, None) == 1
    assert f(P, P, C.c_void_p(0x1004), P, 1, 8, 16, 64, 2, None) == 6
    assert f(P, P, None, None, 1, 0, 16, 64, 2, None) == 0  # empty prompt: nothing to do
    assert lib.ffa_workspace_init(None, 16, None) == 1


def test_workspace_bytes_covers_every_plan(lib):
    for (B, H, Dh, Lmax) in [(10, 32, 64, 1256), (1, 32, 64, 16384), (8, 16, 256, 2256), (16, 32, 64, 8256),
                             (1, 1, 64, 1), (3, 5, 128, 700)]:
        total = lib.ffa_workspace_bytes(B, H, Dh, Lmax)
        assert total > 0
        for prec in (16, 32):
            for t in sorted(t for t in {0, 1, 63, 64, Lmax // 2, Lmax - 1} if t < Lmax):
                for cus in (64, 256, 304):
                    plan = capi.plan_launch(prec, B, H, Dh, t, 0.0, False, cus)
                    bh = B * H
                    sh = bh - plan.whole_heads
                    need = -(-bh * 4 // 256) * 256
                    if plan.n_splits > 1 and sh > 0:
                        need += -(-sh * plan.n_splits * 8 // 256) * 256 + sh * plan.n_splits * Dh * 4
                    assert need <= total, (B, H, Dh, Lmax, t, plan)
                    for p_, dflt in ((1e-3, False), (0.0, True)):
                        plan = capi.plan_launch(prec, B, H, Dh, t, p_, dflt, cus)
                        if plan.kind != capi.FFA_LAUNCH_TWO_PASS:
                            continue
                        up = lambda v: -(-v // 256) * 256
                        need = (up(bh * 4) + up(bh * plan.n_splits * 8) + up(bh * plan.n_splits * Dh * 4) +
                                up(bh * (Lmax // 64 + 1) * 64 * 4))
                        assert need <= total, (B, H, Dh, Lmax, t, plan)
    assert lib.ffa_workspace_bytes(0, 1, 64, 8) == 0


@pytest.mark.parametrize("prec", [16, 32])
@pytest.mark.parametrize("Dh", [64, 80, 128, 256])
def test_planner_consistency(prec, Dh):
    for B, H in [(1, 1), (1, 32), (2, 32), (10, 32), (16, 32), (64, 64)]:
        for t in [0, 1, 31, 63, 64, 127, 999, 1000, 1255, 2047, 2048, 8191, 16383, 30000]:
            ntiles = t // 64 + 1
            for use_default in (False, True):
                for p in (0.0, 1e-3):
                    plan = capi.plan_launch(prec, B, H, Dh, t, p, use_default, 256, rules_only=True)
                    assert plan.keys_per_wave == 64 // plan.threads_per_key
                    assert plan.waves_per_wg in (1, 2, 4, 8, 16)
                    assert plan.n_splits * plan.tiles_per_split >= ntiles      # every key covered
                    fits_lds = ntiles * 64 * 4 <= 140 * 1024
                    wide = Dh * (prec // 8) // 16 >= 16                        # 16-byte chunks per key
                    if use_default:
                        assert plan.n_splits == 1 and plan.threads_per_key == 1
                        assert plan.kind == (capi.FFA_LAUNCH_WORKGROUP if fits_lds else capi.FFA_LAUNCH_TWO_PASS)
                    elif p > 0:
                        assert plan.threads_per_key == 1
                        if plan.kind == capi.FFA_LAUNCH_WORKGROUP:
                            assert plan.n_splits == 1 and fits_lds
                        else:
                            assert plan.kind == capi.FFA_LAUNCH_TWO_PASS
                            assert plan.n_splits > 1 or not fits_lds
                            if fits_lds:   # a cut must save about a dozen tile-times
                                assert B * H < 256 and ntiles * (plan.n_splits - 1) >= 10 * plan.n_splits, (B, H, t, plan)
                            assert (plan.n_splits - 1) * plan.tiles_per_split < ntiles  # no empty piece
                            assert B * H * plan.n_splits <= max(512, B * H)              # about two per CU
                            assert plan.waves_per_wg <= 8 and plan.whole_heads == 0
                    elif B * H % 256 == 0 and ntiles >= 64 and fits_lds:
                        # a whole number of pairs per CU, long sequence: the 16-wave one-workgroup kernel
                        assert plan.kind == capi.FFA_LAUNCH_WORKGROUP and plan.waves_per_wg == 16
                    else:
                        assert plan.kind == capi.FFA_LAUNCH_SPLIT
                        assert (plan.n_splits - 1) * plan.tiles_per_split < ntiles  # no empty split
                        assert 0 <= plan.whole_heads <= B * H
                        assert plan.whole_heads % 256 == 0 or plan.whole_heads == B * H
                        assert (B * H - plan.whole_heads) * plan.n_splits <= 16384
                        assert plan.waves_per_wg <= 8
                        if plan.n_splits == 1:
                            assert plan.whole_heads == B * H
                        elif plan.whole_heads == 0:
                            # fewer pairs than CUs: a cut must save about ten tile-times
                            assert ntiles * (Dh * (prec // 8) // 16) * (plan.n_splits - 1) >= 80 * plan.n_splits, (B, H, t, plan)
                        # wide rows: four lanes per key (unless there are very many pairs)
                        nch = Dh * (prec // 8) // 16
                        lpr = 8 if nch <= 8 else 16 if nch <= 16 else 32 if nch <= 32 else 64
                        four_ok = Dh != 80 and nch % 4 == 0 and nch // 4 <= 8 and 16 % (64 // lpr) == 0
                        want_tpk = 4 if (wide and B * H < 512 and four_ok) else 1
                        assert plan.threads_per_key == want_tpk, (prec, B, H, Dh, t, plan)
                        if want_tpk == 4:
                            assert plan.waves_per_wg in (4, 8)


def _plan_table_rows():
    path = os.path.join(ROOT, "fastforwardattention_amd", "csrc", "ffa_plan_table.inc")
    rows = []
    for m in re.finditer(r"^FFA_PLAN_ROW\(([^)]*)\)", open(path).read(), flags=re.M):
        f = [x.strip().rstrip("f") for x in m.group(1).split(",")]
        rows.append(dict(zip(["override", "precision", "Dh", "pairs", "t_lo", "t_hi", "pruned", "kind", "waves", "tpk",
                              "n_splits", "whole"], map(int, f[:12])), chosen_us=float(f[12]), best_us=float(f[13]),
                         rule_us=float(f[14])))
    return rows


def test_planner_follows_the_measured_table():
    """Every point of the device sweep (ffa_plan_table.inc, written by `bench.py --sweep-plans`):
    the plan the shipped planner returns there is the one the sweep chose, and that plan was
    measured within 3 % of the fastest candidate at the point.  Rows that override the rules
    must differ from them by more than 3 %, the others must leave the rules' plan in place."""
    rows = _plan_table_rows()
    assert len(rows) >= 30, "the table is generated by `python bench.py --sweep-plans` on the device"
    for r in rows:
        assert r["chosen_us"] <= r["best_us"] / 0.97 + 0.011, r    # the sweep's margin; times are written with two decimals
        B, H = (r["pairs"] // 32, 32) if r["pairs"] % 32 == 0 else (r["pairs"], 1)
        p = 1e-3 if r["pruned"] else 0.0
        for t in {r["t_lo"], (r["t_lo"] + r["t_hi"]) // 2, r["t_hi"]}:
            # rows of different sweeps may overlap in t: the one whose centre is nearest decides
            rivals = [o for o in rows if (o["precision"], o["Dh"], o["pairs"], o["pruned"]) ==
                      (r["precision"], r["Dh"], r["pairs"], r["pruned"]) and o["t_lo"] <= t <= o["t_hi"]]
            if min(rivals, key=lambda o: abs(2 * t - o["t_lo"] - o["t_hi"])) is not r:
                continue
            got = capi.plan_launch(r["precision"], B, H, r["Dh"], t, p, False, 256)
            rules = capi.plan_launch(r["precision"], B, H, r["Dh"], t, p, False, 256, rules_only=True)
            if r["override"]:
                assert r["chosen_us"] < 0.97 * r["rule_us"], r
                assert (got.kind, got.waves_per_wg, got.threads_per_key) == (r["kind"], r["waves"], r["tpk"]), (r, got)
                assert got.keys_per_wave == 64 // r["tpk"]
                ntiles = t // 64 + 1
                want_ns = -(-ntiles // -(-ntiles // min(r["n_splits"], ntiles)))
                assert got.n_splits == want_ns and got.n_splits * got.tiles_per_split >= ntiles, (r, got)
                assert got.whole_heads == (r["pairs"] if got.n_splits == 1 and got.kind == 1 else r["whole"])
            else:
                assert got.as_tuple() == rules.as_tuple(), (r, got, rules)
            # a table measured on 256 CUs says nothing about another device
            other = capi.plan_launch(r["precision"], B, H, r["Dh"], t, p, False, 304)
            assert other.as_tuple() == capi.plan_launch(r["precision"], B, H, r["Dh"], t, p, False, 304,
                                                        rules_only=True).as_tuple()
    assert any(r["override"] for r in rows)


def _plan_grid_rows():
    path = os.path.join(ROOT, "fastforwardattention_amd", "csrc", "ffa_plan_grid.inc")
    rows = []
    for m in re.finditer(r"^FFA_GRID_ROW\(([^)]*)\)", open(path).read(), flags=re.M):
        f = [x.strip().rstrip("f") for x in m.group(1).split(",")]
        rows.append(dict(zip(["override", "precision", "Dh", "pairs", "t", "pruned", "kind", "waves", "tpk", "n_splits",
                              "whole"], map(int, f[:11])), chosen_us=float(f[11]), best_us=float(f[12]),
                         rule_us=float(f[13])))
    return rows


def _grid_nearest(rows, prec, Dh, pairs, t, pruned):
    """The lookup rule restated: nearest row of the class within a factor of sqrt 2 both ways."""
    import math
    best, best_d = None, 1e30
    for r in rows:
        if (r["precision"], r["Dh"], r["pruned"]) != (prec, Dh, pruned):
            continue
        dp, dt = abs(math.log2(pairs / r["pairs"])), abs(math.log2((t + 1) / (r["t"] + 1)))
        if dp <= 0.5 and dt <= 0.5 and dp + dt < best_d:
            best, best_d = r, dp + dt
    return best


def test_planner_generalises_through_the_measured_grid():
    """ffa_plan_grid.inc (`bench.py --sweep-plans grid`): problems away from the BASELINE shapes take
    the nearest measured row.  At every grid point the shipped planner returns what the sweep
    chose; off the grid (other batch sizes, head counts, lengths) the nearest row decides the launch
    kind, the waves and the lanes per key, and the plan is valid for the problem at hand."""
    rows, exact = _plan_grid_rows(), _plan_table_rows()
    assert len(rows) >= 500, "the grid is generated by `python bench.py --sweep-plans grid` on the device"
    lib = capi.load()
    overrides = [r for r in rows if r["override"]]
    assert overrides, "a grid without a single override would make this test vacuous"
    for r in rows:
        assert r["chosen_us"] <= r["best_us"] / 0.97 + 0.011, r    # the sweep's margin; times are written with two decimals
        if r["override"]:
            assert r["chosen_us"] < 0.97 * r["rule_us"], r
        B, H = (r["pairs"] // 32, 32) if r["pairs"] % 32 == 0 else (1, r["pairs"])
        p = 1e-2 if r["pruned"] else 0.0
        src = lib.ffa_plan_source(r["precision"], B, H, r["Dh"], r["t"], p, 256)
        got = capi.plan_launch(r["precision"], B, H, r["Dh"], r["t"], p, False, 256)
        rules = capi.plan_launch(r["precision"], B, H, r["Dh"], r["t"], p, False, 256, rules_only=True)
        if src == 1 or any((e["precision"], e["Dh"], e["pairs"], e["pruned"]) == (r["precision"], r["Dh"], r["pairs"], r["pruned"])
                           and e["t_lo"] <= r["t"] <= e["t_hi"] for e in exact):
            continue            # a BASELINE shape: the exact table speaks first, also where it keeps the rules
        if r["override"]:
            assert src == 2, r
            assert (got.kind, got.waves_per_wg, got.threads_per_key, got.n_splits) == \
                (r["kind"], r["waves"], r["tpk"], r["n_splits"]), (r, got)
        else:
            assert src == 0 and got.as_tuple() == rules.as_tuple(), (r, got, rules)
        assert lib.ffa_plan_source(r["precision"], B, H, r["Dh"], r["t"], p, 304) == 0   # measured on 256 CUs only
    # Off the grid: odd batch sizes, head counts and lengths.
    checked = 0
    for prec, B, H, Dh, t, p in [(16, 4, 16, 256, 2200, 0.0), (16, 3, 12, 64, 700, 0.0), (16, 6, 40, 128, 3000, 0.0),
                                 (16, 24, 32, 64, 5000, 0.0), (16, 2, 20, 128, 12000, 0.0), (32, 3, 32, 64, 1500, 0.0),
                                 (16, 3, 16, 64, 6000, 1e-3), (16, 12, 32, 128, 9000, 1e-2), (16, 1, 24, 256, 900, 0.0),
                                 (0xBF16, 4, 16, 256, 2200, 0.0)]:
        pp = capi.FFA_PRECISION_F16 if prec == 0xBF16 else prec
        near = _grid_nearest(rows, pp, Dh, B * H, t, 1 if p > 0 else 0)
        assert near is not None, (prec, B, H, Dh, t, p)
        src = lib.ffa_plan_source(prec, B, H, Dh, t, p, 256)
        got = capi.plan_launch(prec, B, H, Dh, t, p, False, 256)
        rules = capi.plan_launch(prec, B, H, Dh, t, p, False, 256, rules_only=True)
        assert got.n_splits * got.tiles_per_split >= t // 64 + 1
        if src == 2:
            assert near["override"]
            assert (got.kind, got.waves_per_wg, got.threads_per_key) == (near["kind"], near["waves"], near["tpk"]), (near, got)
            checked += 1
        else:
            assert src == 0 and got.as_tuple() == rules.as_tuple()
    # Every overriding row also decides for its neighbourhood.
    for r in overrides:
        B, H = (r["pairs"] // 32, 34) if r["pairs"] % 32 == 0 else (1, r["pairs"] + 1)
        t = int(r["t"] * 1.15)
        p = 1e-2 if r["pruned"] else 0.0
        near = _grid_nearest(rows, r["precision"], r["Dh"], B * H, t, r["pruned"])
        if near is not r or lib.ffa_plan_source(r["precision"], B, H, r["Dh"], t, p, 256) != 2:
            continue        # a nearer row, the exact table, or a plan that does not fit the neighbour
        got = capi.plan_launch(r["precision"], B, H, r["Dh"], t, p, False, 256)
        assert (got.kind, got.waves_per_wg, got.threads_per_key) == (r["kind"], r["waves"], r["tpk"]), (r, got)
        checked += 1
    assert checked >= 1


def test_planner_default_follows_length_table():
    # kernel_launch_utils.h:147-154: 64 / 128 / 256 threads by prompt length
    assert capi.plan_launch(16, 10, 32, 64, 10, 0.0, True).waves_per_wg == 1
    assert capi.plan_launch(16, 10, 32, 64, 1000, 0.0, True).waves_per_wg == 2
    assert capi.plan_launch(16, 10, 32, 64, 4096, 0.0, True).waves_per_wg == 4


def test_planner_rejects_bad_input(lib):
    plan = capi.LaunchPlan()
    f = lib.ffa_plan_launch
    assert f(8, 1, 1, 64, 10, 0.0, 0, 256, C.byref(plan)) == 2
    assert f(16, 1, 1, 96, 10, 0.0, 0, 256, C.byref(plan)) == 3
    assert f(16, 1, 1, 80, 10, 0.0, 0, 256, C.byref(plan)) == 0
    assert f(16, 0, 1, 64, 10, 0.0, 0, 256, C.byref(plan)) == 4
    assert f(16, 1, 1, 64, -1, 0.0, 0, 256, C.byref(plan)) == 5
    assert f(16, 1, 1, 64, 10, -1.0, 0, 256, C.byref(plan)) == 10
    assert f(16, 1, 1, 64, 10, 0.0, 0, 256, None) == 1


def test_planner_long_sequences_leave_lds():
    # 50001 scores do not fit LDS: pruned and default launches keep them in the workspace
    for p, default in ((0.5, False), (0.0, True), (0.5, True)):
        plan = capi.plan_launch(16, 1, 1, 64, 50000, p, default, 256)
        assert plan.kind == capi.FFA_LAUNCH_TWO_PASS
        assert plan.n_splits * plan.tiles_per_split >= 50000 // 64 + 1
    assert capi.plan_launch(16, 1, 1, 64, 50000, 0.0, True, 256).n_splits == 1
    assert capi.plan_launch(16, 1, 1, 64, 50000, 0.5, False, 256).n_splits > 64
    # few pairs, pruning on: cut along the sequence
    plan = capi.plan_launch(16, 1, 32, 64, 8191, 1e-3, False, 256, rules_only=True)
    assert plan.kind == capi.FFA_LAUNCH_TWO_PASS and plan.n_splits == 16 and plan.waves_per_wg == 8
    # many pairs, scores fit: one workgroup per pair
    assert capi.plan_launch(16, 16, 32, 64, 8191, 1e-3, False, 256).kind == capi.FFA_LAUNCH_WORKGROUP


def test_extension_imports_and_refuses_cpu_tensors():
    import torch
    from fastforwardattention_amd import FastForwardAttn
    with pytest.raises(RuntimeError, match="GPU tensors"):
        FastForwardAttn(torch.zeros(1, 1, 4, 64), torch.zeros(1, 1, 4, 64), 8, False)
    import ff_attention  # the reference's module name resolves to the same extension
    assert ff_attention.FastForwardAttn is FastForwardAttn
