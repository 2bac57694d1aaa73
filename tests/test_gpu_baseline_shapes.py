"""GPU parity at the BASELINE shapes themselves, through the C ABI, against the CPU oracle:
the long-sequence sweep (B=1, 32x64, up to 16384 keys) with both launches, the pruned sweep
(B=16, 32x64, 8192 keys, peaked keys, four thresholds), the OPT-1.3b shape at B=1 and B=5,
the GPT-J shape (B=8, 16x256, 2000 to 2255 keys),
and the one-workgroup kernel in the range where its scores need more than 48 KiB of LDS.
Tolerances: 1e-3 max-abs for fp16 inputs, 1e-6 for fp32 inputs, against the float64 closed
form; caches bit for bit; skip sets equal to the rule's except within one quantum of the
threshold."""
import ctypes as C

import numpy as np
import pytest
import torch

from fastforwardattention_amd import capi
from oracle import ffa_oracle as O
from tests.ffa_testlib import CApiSession, ptr, rand_inputs, rand_token
from tests.test_gpu_parity import TOL, _near_threshold, _peaked, _tol

pytestmark = pytest.mark.gpu


def _say(*a):
    print(*a, flush=True)


# ------------------------------------------------------------------ configs[2]: long sequences, B = 1
@pytest.mark.parametrize("x", [1024, 2048, 4096, 8192, 16384])
@pytest.mark.parametrize("use_default", [False, True])
def test_long_sequence_sweep_consecutive_steps(x, use_default):
    """BASELINE configs[2]: batch 1, 32 heads x 64, fp16, prompt x-128 of N(0,1), then decode
    steps up to length x; here the first two and the last three of the 128 steps, each against
    the oracle, with the launch the library plans (sequence split) and the default launch (one
    workgroup per head)."""
    B, H, Dh, prec, steps = 1, 32, 64, 16, 128
    L = x - steps
    rng, K, V = rand_inputs(300 + x, B, H, x, Dh, prec)      # prompt + the tokens the skipped steps append
    sess = CApiSession(K[:, :, :L], V[:, :, :L], x)
    kc, vc = O.pack_k_cache(K[:, :, :L], x), O.pack_v_cache(V[:, :, :L], x)
    worst = 0.0
    for i in range(steps):
        t = L + i
        if 2 <= i < steps - 3:
            # steps not compared: append through the oracle and the device copy alike
            O.append_kv(kc, vc, K[:, :, t], V[:, :, t], t)
            continue
        if i == steps - 3:
            sess.k_cache.copy_(torch.from_numpy(kc).cuda())
            sess.v_cache.copy_(torch.from_numpy(vc).cuda())
        q, k, v = rand_token(rng, B, H, Dh, prec)
        plan = capi.plan_launch(prec, B, H, Dh, t, 0.0, use_default)
        _say("long", x, use_default, t, plan)
        got = sess.step(q, k, v, 0.125, t, plan=plan)
        want = O.decode_step(q, k, v, kc, vc, 0.125, t, acc=np.float64)
        worst = max(worst, float(np.abs(got - want).max()))
    assert worst <= TOL[prec], worst
    gk, gv = sess.caches()
    np.testing.assert_array_equal(gk.view(np.uint8), kc.view(np.uint8))
    np.testing.assert_array_equal(gv.view(np.uint8), vc.view(np.uint8))


# ------------------------------------------------------------------ configs[1] at B = 1 and B = 5
@pytest.mark.parametrize("B", [1, 5])
def test_opt13b_shape_small_batches(B):
    """BASELINE configs[1] at the batch sizes whose launch plans differ from B=2 and B=10
    (B=1: every pair split 8 ways; B=5: 160 pairs, one 8-wave workgroup each)."""
    H, Dh, prec, L, steps = 32, 64, 16, 1000, 6
    rng, K, V = rand_inputs(400 + B, B, H, L, Dh, prec, kv_scale=0.5)
    for use_default in (False, True):
        sess = CApiSession(K, V, L + steps)
        kc, vc = O.pack_k_cache(K, L + steps), O.pack_v_cache(V, L + steps)
        worst = 0.0
        for i in range(steps):
            t = L + i
            q, k, v = rand_token(rng, B, H, Dh, prec)
            plan = capi.plan_launch(prec, B, H, Dh, t, 0.0, use_default)
            _say("opt1.3b", B, use_default, t, plan)
            got = sess.step(q, k, v, 0.125, t, plan=plan)
            want = O.decode_step(q, k, v, kc, vc, 0.125, t, acc=np.float64)
            worst = max(worst, float(np.abs(got - want).max()))
        assert worst <= TOL[prec], worst
        gk, gv = sess.caches()
        np.testing.assert_array_equal(gk.view(np.uint8), kc.view(np.uint8))
        np.testing.assert_array_equal(gv.view(np.uint8), vc.view(np.uint8))


def test_opt13b_b10_whole_decode_at_the_reference_max_len():
    """BASELINE configs[1] as the reference's script sizes it (example.py:29-35: prompt 1000,
    max_len = 1000 + 128, so the chunk rows of K are 1128 x 16 bytes apart): B = 10, 32 heads x
    64, fp16, all 128 decode steps in one session through the C ABI with the library's own
    plans.  Every step is checked against the CPU oracle on two samples (64 of the 320 pairs);
    their caches bit for bit at the end."""
    B, H, Dh, prec, L, steps = 10, 32, 64, 16, 1000, 128
    Lmax = L + steps
    rng, K, V = rand_inputs(440, B, H, L, Dh, prec, kv_scale=0.5)
    sess = CApiSession(K, V, Lmax)
    sub = [0, 9]
    kc, vc = O.pack_k_cache(K[sub], Lmax), O.pack_v_cache(V[sub], Lmax)
    worst, kinds = 0.0, set()
    for i in range(steps):
        t = L + i
        q, k, v = rand_token(rng, B, H, Dh, prec)
        plan = capi.plan_launch(prec, B, H, Dh, t, 0.0, False)
        kinds.add((plan.kind, plan.n_splits, plan.whole_heads))
        if i % 32 == 0:
            _say("opt1.3b b10 Lmax 1128", t, plan)
        got = sess.step(q, k, v, 0.125, t)   # plan = NULL: what a caller of the reference's API gets
        want = O.decode_step(q[sub], k[sub], v[sub], kc, vc, 0.125, t, acc=np.float64)
        worst = max(worst, float(np.abs(got[sub] - want).max()))
    assert worst <= TOL[prec], worst
    assert all(kind == capi.FFA_LAUNCH_SPLIT and whole == 256 for kind, _, whole in kinds), kinds
    gk, gv = sess.caches()
    np.testing.assert_array_equal(gk[sub].view(np.uint16), kc.view(np.uint16))
    np.testing.assert_array_equal(gv[sub].view(np.uint16), vc.view(np.uint16))


def test_opt13b_shape_b2_last_step():
    """BASELINE configs[1] at B = 2 (64 pairs, every pair cut into four pieces), last steps of the
    256-step decode (t = 1253 .. 1255, max_len 1256), both launches."""
    B, H, Dh, prec, L, Lmax = 2, 32, 64, 16, 1253, 1256
    rng, K, V = rand_inputs(450, B, H, L, Dh, prec, kv_scale=0.5)
    for use_default in (False, True):
        sess = CApiSession(K, V, Lmax)
        kc, vc = O.pack_k_cache(K, Lmax), O.pack_v_cache(V, Lmax)
        for t in range(L, Lmax):
            q, k, v = rand_token(rng, B, H, Dh, prec)
            plan = capi.plan_launch(prec, B, H, Dh, t, 0.0, use_default)
            _say("opt1.3b b2", use_default, t, plan)
            got = sess.step(q, k, v, 0.125, t, plan=plan)
            want = O.decode_step(q, k, v, kc, vc, 0.125, t, acc=np.float64)
            assert float(np.abs(got - want).max()) <= TOL[prec]
        gk, gv = sess.caches()
        np.testing.assert_array_equal(gk.view(np.uint16), kc.view(np.uint16))
        np.testing.assert_array_equal(gv.view(np.uint16), vc.view(np.uint16))


# ------------------------------------------------------------------ configs[3]: GPT-J shape
@pytest.mark.parametrize("t0", [2000, 2060, 2250])
def test_gptj_shape_steps(t0):
    """BASELINE configs[3]: B=8, 16 heads x 256, fp16, prompt 2000, max_len 2256.  Steps around
    t0 with the launch the library plans (four lanes per key: wide rows), the same split with one
    lane per key, and the default launch, against the oracle; caches bit for bit."""
    B, H, Dh, prec, Lmax, steps = 8, 16, 256, 16, 2256, 6
    rng, K, V = rand_inputs(500 + t0, B, H, t0, Dh, prec, kv_scale=0.5)
    scale = 1.0 / 16.0
    kinds = set()
    for launch in ("library", "one lane per key", "default"):
        sess = CApiSession(K, V, Lmax)
        kc, vc = O.pack_k_cache(K, Lmax), O.pack_v_cache(V, Lmax)
        worst = 0.0
        for i in range(steps):
            t = t0 + i
            q, k, v = rand_token(rng, B, H, Dh, prec)
            plan = capi.plan_launch(prec, B, H, Dh, t, 0.0, launch == "default")
            if launch == "one lane per key":
                plan = capi.make_plan(capi.FFA_LAUNCH_SPLIT, 4, plan.n_splits, plan.tiles_per_split, 0, plan.whole_heads)
            kinds.add((plan.kind, plan.threads_per_key))
            _say("gptj", launch, t, plan)
            got = sess.step(q, k, v, scale, t, plan=plan)
            want = O.decode_step(q, k, v, kc, vc, scale, t, acc=np.float64)
            worst = max(worst, float(np.abs(got - want).max()))
        assert worst <= TOL[prec], worst
        gk, gv = sess.caches()
        n = t0 + steps                       # slots beyond are untouched (and unspecified) on both sides
        np.testing.assert_array_equal(gk[:, :, :, :n].view(np.uint16), kc[:, :, :, :n].view(np.uint16))
        np.testing.assert_array_equal(gv[:, :, :n].view(np.uint16), vc[:, :, :n].view(np.uint16))
    assert kinds == {(capi.FFA_LAUNCH_SPLIT, 4), (capi.FFA_LAUNCH_SPLIT, 1), (capi.FFA_LAUNCH_WORKGROUP, 1)}, kinds


# ------------------------------------------------------------------ configs[4]: pruned sweep, B = 16
class _DeviceProblem:
    """Caches built on the GPU from torch tensors (the full-size inputs are too large to draw
    with numpy in a test); drives the C ABI like CApiSession."""

    def __init__(self, K, V, Lmax):
        self.lib = capi.load()
        B, H, L, Dh = K.shape
        self.B, self.H, self.L, self.Dh, self.Lmax = B, H, L, Dh, Lmax
        self.k_cache = torch.empty(B, H, Dh // 8, Lmax, 8, dtype=torch.float16, device="cuda:0")
        self.v_cache = torch.empty(B, H, Lmax, Dh, dtype=torch.float16, device="cuda:0")
        capi.check(self.lib.ffa_init_cache_f16(ptr(self.k_cache), ptr(self.v_cache), ptr(K), ptr(V), B, L, Lmax, Dh, H,
                                               None), "ffa_init_cache_f16")
        n = self.lib.ffa_workspace_bytes(B, H, Dh, Lmax)
        self.ws = torch.empty(n, dtype=torch.uint8, device="cuda:0")
        capi.check(self.lib.ffa_workspace_init(ptr(self.ws), n, None), "ffa_workspace_init")
        torch.cuda.synchronize()

    def step(self, q, k, v, scale, t, p, plan=None, diag=True):
        out = torch.full((self.B, self.H, self.Dh), float("nan"), dtype=torch.float16, device="cuda:0")
        kept = torch.zeros(self.B, self.H, dtype=torch.int32, device="cuda:0") if diag else None
        mask = torch.zeros(self.B, self.H, self.Lmax, dtype=torch.uint8, device="cuda:0") if diag else None
        rc = self.lib.ffa_attention_diag(16, self.B, self.H, self.Dh, self.Lmax, scale, t, ptr(q), ptr(k), ptr(v),
                                         ptr(self.k_cache), ptr(self.v_cache), ptr(out), None, p,
                                         C.byref(plan) if plan is not None else None, 1, ptr(self.ws),
                                         self.ws.numel(), ptr(kept), ptr(mask), None)
        assert rc == capi.FFA_OK, capi.STATUS_NAMES.get(rc, rc)
        torch.cuda.synchronize()
        return out, kept, mask


def test_pruned_sweep_full_size():
    """BASELINE configs[4]: batch 16, 32 heads x 64, fp16, 8192 cached keys; per head 32 random
    key positions hold 4*q_dir + N(0, 0.1), the rest N(0,1); values N(0,1);
    p in {0, 1e-4, 1e-3, 1e-2}.  On every pair: kept_count equals the mask's count and p = 0
    reproduces the exact split kernel.  On a fixed subset of pairs (the numpy oracle over all
    512 would take minutes): skip set and output against the CPU transcription of the rule."""
    B, H, Dh, L, Lmax, scale = 16, 32, 64, 8192, 8192 + 64, 0.125
    dev = "cuda:0"
    g = torch.Generator(device=dev).manual_seed(0)
    q = torch.randn(B, H, Dh, device=dev, generator=g)
    qdir = q / q.norm(dim=-1, keepdim=True)
    K = torch.randn(B, H, L, Dh, device=dev, generator=g)
    pos = torch.rand(B, H, L, device=dev, generator=g).argsort(dim=-1)[:, :, :32]
    K.scatter_(2, pos[..., None].expand(-1, -1, -1, Dh),
               4 * qdir[:, :, None, :] + 0.1 * torch.randn(B, H, 32, Dh, device=dev, generator=g))
    K = K.half()
    V = torch.randn(B, H, L, Dh, device=dev, generator=g).half()
    q = q.half()
    k = torch.randn(B, H, Dh, device=dev, generator=g).half()
    v = torch.randn(B, H, Dh, device=dev, generator=g).half()
    prob = _DeviceProblem(K, V, Lmax)
    pairs = [(0, 0), (3, 17), (7, 31), (15, 5), (15, 31), (9, 12)]
    bi, hi = [b for b, _ in pairs], [h for _, h in pairs]
    Ks, Vs = K[bi, hi].cpu().numpy()[None], V[bi, hi].cpu().numpy()[None]          # [1, n, L, Dh]
    qs, ks, vs = (x[bi, hi].cpu().numpy()[None] for x in (q, k, v))
    kcs, vcs = O.pack_k_cache(Ks, Lmax), O.pack_v_cache(Vs, Lmax)
    Vall = np.concatenate([Vs, vs[:, :, None]], axis=2).astype(np.float32)

    ntiles = L // 64 + 1
    split = capi.make_plan(capi.FFA_LAUNCH_SPLIT, 4, 1, ntiles, 0, B * H)            # the exact kernel, whole pairs
    exact, _, _ = prob.step(q, k, v, scale, L, 0.0, plan=split, diag=False)
    want0 = O.decode_step(qs, ks, vs, kcs.copy(), vcs.copy(), scale, L, acc=np.float64)
    assert float(np.abs(exact[bi, hi].float().cpu().numpy()[None] - want0).max()) <= 1e-3
    last_skip = -1.0
    for p in (0.0, 1e-4, 1e-3, 1e-2):
        for name, plan in (("library", None), ("two_pass", capi.make_plan(capi.FFA_LAUNCH_TWO_PASS, 8, 1, ntiles))):
            if name == "two_pass" and p not in (0.0, 1e-2):
                continue
            _say("pruned full size", p, name)
            out, kept, mask = prob.step(q, k, v, scale, L, p, plan=plan)
            assert torch.equal(kept.long(), L - mask[:, :, :L].long().sum(-1)), "kept_count != mask count"
            assert not bool(mask[:, :, L:].any())
            if p == 0.0:
                assert int(mask.sum()) == 0
                assert float((out.float() - exact.float()).abs().max()) <= 1e-3
            want, skip, P, thr = O.pruned_decode_step(qs, ks, vs, kcs.copy(), vcs.copy(), scale, L, p)
            gmask = mask[bi, hi].cpu().numpy().astype(bool)[None]
            diff = gmask != skip
            assert not (diff & ~_near_threshold(16, P, thr)).any(), "skip decision differs away from the threshold"
            assert diff.mean() < 1e-3
            w = np.where(gmask[:, :, :L + 1], 0, P[:, :, :L + 1])
            want_g = np.einsum("bhn,bhnd->bhd", w, Vall)
            got = out[bi, hi].float().cpu().numpy()[None]
            assert float(np.abs(got - want_g).max()) <= 1e-3, (p, name)
            frac = float(mask[:, :, :L].float().mean())
            _say("   skipped fraction", frac, "max-abs vs exact", float((out.float() - exact.float()).abs().max()))
            if name == "library":
                assert frac >= last_skip          # the skip set grows with p
                last_skip = frac
    assert last_skip > 0.05                       # p = 1e-2 drops a visible share of the keys
    gk, gv = prob.k_cache.cpu(), prob.v_cache.cpu()
    assert torch.equal(gk[:, :, :, L, :].reshape(B, H, Dh), k.cpu()) and torch.equal(gv[:, :, L], v.cpu())
    assert torch.equal(gv[:, :, :L], V.cpu())


# ------------------------------------------------------------------ one-workgroup kernel, scores beyond 48 KiB of LDS
@pytest.mark.parametrize("prec", [16, 32])
@pytest.mark.parametrize("L", [20000, 35839])
def test_workgroup_kernel_with_large_lds(prec, L):
    """12.3k to 35.8k keys: the one-workgroup kernel needs 48 to 140 KiB of dynamic LDS, above
    the default ceiling (raised per function and device on first use).  35839 is the longest
    sequence a one-workgroup plan accepts.  4 and 16 waves and the default plan, exact and
    pruned, against the oracle; caches bit for bit."""
    B, H, Dh = 1, 2, 64
    K, V, q, k, v = _peaked(prec, 17 + L, B, H, L, Dh)
    Lmax, scale = L + 1, 0.125
    kc0, vc0 = O.pack_k_cache(K, Lmax), O.pack_v_cache(V, Lmax)
    want = O.decode_step(q, k, v, kc0, vc0, scale, L, acc=np.float64)
    ntiles = L // 64 + 1
    default = capi.plan_launch(prec, B, H, Dh, L, 0.0, True)
    assert default.kind == capi.FFA_LAUNCH_WORKGROUP
    plans = [("wg4", capi.make_plan(capi.FFA_LAUNCH_WORKGROUP, 4, 1, ntiles)),
             ("wg16", capi.make_plan(capi.FFA_LAUNCH_WORKGROUP, 16, 1, ntiles)), ("default", default)]
    for name, plan in plans:
        _say("large lds exact", prec, L, name)
        sess = CApiSession(K, V, Lmax)
        got = sess.step(q, k, v, scale, L, plan=plan)
        assert float(np.abs(got - want).max()) <= _tol(prec, V, v), name
        gk, gv = sess.caches()
        np.testing.assert_array_equal(gk.view(np.uint8), kc0.view(np.uint8))
        np.testing.assert_array_equal(gv.view(np.uint8), vc0.view(np.uint8))
    p = 0.05
    _, skip, P, thr = O.pruned_decode_step(q, k, v, kc0.copy(), vc0.copy(), scale, L, p)
    Vall = np.concatenate([V, v[:, :, None]], axis=2).astype(np.float32)
    for name, plan in plans:
        _say("large lds pruned", prec, L, name)
        got, kept, gmask = CApiSession(K, V, Lmax).step(q, k, v, scale, L, p=p, plan=plan, diag=True)
        diff = gmask != skip
        assert not (diff & ~_near_threshold(prec, P, thr)).any()
        np.testing.assert_array_equal(kept, (L - gmask[:, :, :L].sum(axis=-1)))
        w = np.where(gmask[:, :, :L + 1], 0, P[:, :, :L + 1])
        assert float(np.abs(got - np.einsum("bhn,bhnd->bhd", w, Vall)).max()) <= (1e-3 if prec == 16 else 1e-5)
    assert skip[:, :, :L].mean() > 0.5
    # one key more and the scores no longer fit: the plan is refused, nothing is launched
    too_long = capi.make_plan(capi.FFA_LAUNCH_WORKGROUP, 16, 1, 35840 // 64 + 1)
    CApiSession(K[:, :, :8], V[:, :, :8], 35841).step(q, k, v, scale, 35840, plan=too_long, expect=capi.FFA_ERR_TOO_LONG)


def test_first_large_lds_launch_inside_a_captured_graph():
    """The first launch of a one-workgroup instantiation that needs more than 48 KiB of LDS raises
    the function's LDS ceiling; that must also work while a stream is being captured (or come
    back as a status, never as an abort).  The instantiation used here (fp32, head dim 80,
    2 waves) is used at this length by no other test."""
    prec, B, H, Dh, L = 32, 1, 2, 80, 14000
    rng, K, V = rand_inputs(91, B, H, L, Dh, prec)
    q, k, v = rand_token(rng, B, H, Dh, prec)
    Lmax = L + 1
    sess = CApiSession(K, V, Lmax)
    want = O.decode_step(q, k, v, O.pack_k_cache(K, Lmax), O.pack_v_cache(V, Lmax), 0.125, L, acc=np.float64)
    plan = capi.make_plan(capi.FFA_LAUNCH_WORKGROUP, 2, 1, L // 64 + 1)
    dev = "cuda:0"
    qd, kd, vd = (torch.from_numpy(x).to(dev) for x in (q, k, v))
    out = torch.zeros(B, H, Dh, dtype=torch.float32, device=dev)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    rc = None
    try:
        with torch.cuda.graph(graph, stream=side):
            rc = sess.lib.ffa_attention_f32(B, H, Dh, Lmax, 0.125, L, ptr(qd), ptr(kd), ptr(vd), ptr(sess.k_cache),
                                            ptr(sess.v_cache), ptr(out), None, 0.0, C.byref(plan), 1, None, 0,
                                            torch.cuda.current_stream().cuda_stream)
    except RuntimeError as e:                     # capture invalidated by a refused call: a status, not an abort
        assert rc is not None and rc != capi.FFA_OK, e
        return
    if rc != capi.FFA_OK:                         # refused with a status: nothing was recorded
        assert rc == capi.FFA_ERR_LAUNCH, capi.STATUS_NAMES.get(rc, rc)
        pytest.skip("the runtime refuses to raise the LDS ceiling during capture; the call returned FFA_ERR_LAUNCH")
    for _ in range(3):
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert float(np.abs(out.cpu().numpy() - want).max()) <= _tol(prec, V, v)
