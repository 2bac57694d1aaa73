"""GPU parity tests: the HIP path, called through the C ABI, against the CPU oracle on the
same seeded inputs.  Tolerances, max-abs against the closed form: 1e-3 for fp16 inputs,
1e-6 for fp32 inputs.  The fp32 figure is an absolute bound for outputs of magnitude <= 1
(the BASELINE configurations: N(0,1) values averaged over >= 1000 keys, tested at exactly
1e-6 in test_baseline_config1_fp32); where a test lets single value rows of magnitude up
to ~4.5 through (one or two keys), 1e-6 would be less than four fp32 ulps of the result,
so those tests scale the bound by max(1, max|V|) and compare with the float64 closed form.
Cache contents are compared bit-exactly."""
import numpy as np
import pytest
import torch

from fastforwardattention_amd import capi
from oracle import ffa_oracle as O
from tests.ffa_testlib import CApiSession, rand_inputs, rand_token

pytestmark = pytest.mark.gpu

TOL = {16: 1e-3, 32: 1e-6}


def _tol(prec, V, v):
    vmax = max(1.0, float(np.abs(V).max()) if V.size else 0.0, float(np.abs(v).max()))
    return TOL[prec] * (vmax if prec == 32 else 1.0)


def _say(*a):
    print(*a, flush=True)


def _plans(prec, B, H, Dh, t):
    ntiles = t // 64 + 1
    plans = [("tuned", None),
             ("default", capi.plan_launch(prec, B, H, Dh, t, 0.0, True)),
             ("wg16", capi.make_plan(capi.FFA_LAUNCH_WORKGROUP, 16, 1, ntiles)),
             ("wg1", capi.make_plan(capi.FFA_LAUNCH_WORKGROUP, 1, 1, ntiles))]
    for waves, tps in [(1, 1), (2, 3), (4, 2), (8, 8), (4, ntiles)]:
        ns = -(-ntiles // tps)
        if ns <= 128:
            plans.append((f"split_w{waves}_tps{tps}", capi.make_plan(capi.FFA_LAUNCH_SPLIT, waves, ns, tps)))
            plans.append((f"split_w{waves}_tps{tps}_mergekernel",
                          capi.make_plan(capi.FFA_LAUNCH_SPLIT, waves, ns, tps, capi.FFA_COMBINE_KERNEL)))
    for waves, tps in [(3, 2), (5, 3), (6, 1), (7, ntiles)]:       # workgroups of 3, 5, 6, 7 waves
        ns = -(-ntiles // tps)
        if ns <= 128:
            plans.append((f"split_w{waves}_tps{tps}", capi.make_plan(capi.FFA_LAUNCH_SPLIT, waves, ns, tps)))
    # 2 and 4 lanes per key (tiles of 32 and 16 keys), where the kernel exists for this shape
    nch = Dh * (prec // 8) // 16
    for tpk in (2, 4):
        if Dh != 80 and nch % tpk == 0 and nch // tpk <= 8 and (tpk == 4 or nch <= 16):
            for waves, tps in [(4, 1), (8, 2), (4, ntiles)]:
                ns = -(-ntiles // tps)
                if ns <= 128:
                    plans.append((f"split_tpk{tpk}_w{waves}_tps{tps}",
                                  capi.make_plan(capi.FFA_LAUNCH_SPLIT, waves, ns, tps, threads_per_key=tpk)))
            plans.append((f"hybrid_tpk{tpk}_whole{B * H // 2}",
                          capi.make_plan(capi.FFA_LAUNCH_SPLIT, 8, -(-ntiles // 2), 2, capi.FFA_COMBINE_FUSED, B * H // 2,
                                         threads_per_key=tpk)))
    # two-pass launches (scores kernel, then weights x V): same answer at p == 0
    for waves, tps in [(1, 1), (4, 3), (8, 2), (2, ntiles)]:
        ns = -(-ntiles // tps)
        if ns <= 128:
            plans.append((f"twopass_w{waves}_tps{tps}", capi.make_plan(capi.FFA_LAUNCH_TWO_PASS, waves, ns, tps)))
    # hybrid launches: some (batch, head) pairs whole, the rest split
    bh = B * H
    for whole in sorted({1, bh // 2, bh - 1, bh}):
        if 0 < whole <= bh:
            tps = max(1, ntiles // 3)
            ns = -(-ntiles // tps)
            plans.append((f"hybrid_whole{whole}_w8_tps{tps}",
                          capi.make_plan(capi.FFA_LAUNCH_SPLIT, 8, ns, tps, capi.FFA_COMBINE_FUSED, whole)))
            plans.append((f"hybrid_whole{whole}_w2_tps{tps}_mergekernel",
                          capi.make_plan(capi.FFA_LAUNCH_SPLIT, 2, ns, tps, capi.FFA_COMBINE_KERNEL, whole)))
    return plans


# ------------------------------------------------------------------ cache construction
@pytest.mark.parametrize("prec", [16, 32])
@pytest.mark.parametrize("Dh", [64, 80, 128, 256])
@pytest.mark.parametrize("L,Lmax", [(1, 1), (63, 64), (64, 80), (130, 131), (257, 400)])
def test_init_cache_bit_exact(prec, Dh, L, Lmax):
    _say("init_cache", prec, Dh, L, Lmax)
    B, H = 2, 3
    _, K, V = rand_inputs(100 + L, B, H, L, Dh, prec)
    sentinel = 7.0
    sess = CApiSession(K, V, Lmax, sentinel=sentinel)
    kc, vc = sess.caches()
    dt = K.dtype
    np.testing.assert_array_equal(kc.view(np.uint8), O.pack_k_cache(K, Lmax, fill=dt.type(sentinel)).view(np.uint8))
    np.testing.assert_array_equal(vc.view(np.uint8), O.pack_v_cache(V, Lmax, fill=dt.type(sentinel)).view(np.uint8))


# ------------------------------------------------------------------ exact decode, one step
@pytest.mark.parametrize("prec", [16, 32])
@pytest.mark.parametrize("Dh", [64, 80, 128, 256])
@pytest.mark.parametrize("t", [0, 1, 63, 64, 65, 200, 777])
def test_exact_step_all_plans(prec, Dh, t):
    B, H = 2, 3
    Lmax = t + 3
    rng, K, V = rand_inputs(1000 * Dh + t, B, H, t, Dh, prec)
    q, k, v = rand_token(rng, B, H, Dh, prec)
    scale = 1.0 / np.sqrt(Dh)
    kc0, vc0 = O.pack_k_cache(K, Lmax, fill=9), O.pack_v_cache(V, Lmax, fill=9)
    want = O.decode_step(q, k, v, kc0, vc0, scale, t, acc=np.float64)
    for name, plan in _plans(prec, B, H, Dh, t):
        _say("exact_step", prec, Dh, t, name)
        sess = CApiSession(K, V, Lmax, sentinel=9.0)
        got = sess.step(q, k, v, scale, t, plan=plan)
        err = float(np.abs(got - want).max())
        assert err <= _tol(prec, V, v), (name, err)
        kc, vc = sess.caches()
        np.testing.assert_array_equal(kc.view(np.uint8), kc0.view(np.uint8), err_msg=name)
        np.testing.assert_array_equal(vc.view(np.uint8), vc0.view(np.uint8), err_msg=name)


def test_known_answers():
    """t = 0 -> the new value row; q = 0 -> mean of the values; a dominant key -> its row."""
    B, H, Dh, prec = 1, 2, 64, 32
    rng, K, V = rand_inputs(5, B, H, 300, Dh, prec)
    q, k, v = rand_token(rng, B, H, Dh, prec)
    for name, plan in _plans(prec, B, H, Dh, 0):
        _say("known t=0", name)
        got = CApiSession(K[:, :, :0], V[:, :, :0], 4).step(q, k, v, 0.125, 0, plan=plan)
        np.testing.assert_allclose(got, v, rtol=0, atol=1e-6)
    for name, plan in _plans(prec, B, H, Dh, 300):
        _say("known t=300", name)
        got = CApiSession(K, V, 301).step(0 * q, k, v, 0.125, 300, plan=plan)
        mean = np.concatenate([V, v[:, :, None]], axis=2).astype(np.float64).mean(axis=2)
        np.testing.assert_allclose(got, mean, atol=1e-6)
        K2 = K.copy()
        K2[:, :, 123] = 40 * q
        got = CApiSession(K2, V, 301).step(q, k, v, 1.0, 300, plan=plan)
        np.testing.assert_allclose(got, V[:, :, 123], atol=1e-6)


# ------------------------------------------------------------------ iterative decode
@pytest.mark.parametrize("prec,Dh,B,H,L,steps", [(16, 64, 2, 32, 1000, 24), (32, 64, 1, 8, 120, 20),
                                                 (16, 256, 2, 4, 500, 12), (16, 128, 1, 5, 61, 10),
                                                 (16, 80, 2, 32, 300, 12), (32, 80, 1, 3, 130, 8)])
@pytest.mark.parametrize("use_default", [False, True])
def test_iterative_decode_every_step(prec, Dh, B, H, L, steps, use_default):
    """BASELINE config 2 in miniature: prompt cache, then `steps` appended tokens, parity at
    every step and bit-exact caches at the end."""
    Lmax = L + steps
    rng, K, V = rand_inputs(42, B, H, L, Dh, prec, kv_scale=0.5)
    sess = CApiSession(K, V, Lmax)
    kc, vc = O.pack_k_cache(K, Lmax), O.pack_v_cache(V, Lmax)
    scale = 1.0 / np.sqrt(Dh)
    worst = 0.0
    for i in range(steps):
        t = L + i
        q, k, v = rand_token(rng, B, H, Dh, prec)
        plan = capi.plan_launch(prec, B, H, Dh, t, 0.0, use_default)
        _say("iter", prec, Dh, t, plan)
        got = sess.step(q, k, v, scale, t, plan=plan)
        want = O.decode_step(q, k, v, kc, vc, scale, t, acc=np.float64)
        worst = max(worst, float(np.abs(got - want).max()))
    assert worst <= TOL[prec], worst
    gk, gv = sess.caches()
    np.testing.assert_array_equal(gk.view(np.uint8), kc.view(np.uint8))
    np.testing.assert_array_equal(gv.view(np.uint8), vc.view(np.uint8))


def test_baseline_config1_fp32():
    """BASELINE config 1: B=1, 32 heads x 64, fp32, t=1000, scale 1/8, seed 0; 1e-6."""
    torch.manual_seed(0)
    q = torch.randn(32, 1, 64)
    Kc, Vc = torch.randn(32, 1000, 64), torch.randn(32, 1000, 64)
    k, v = torch.randn(32, 1, 64), torch.randn(32, 1, 64)
    K, V = Kc.numpy()[None], Vc.numpy()[None]
    kc, vc = O.pack_k_cache(K, 1001), O.pack_v_cache(V, 1001)
    want = O.decode_step(q.numpy().reshape(1, 32, 64), k.numpy().reshape(1, 32, 64),
                         v.numpy().reshape(1, 32, 64), kc, vc, 0.125, 1000, acc=np.float64)
    for name, plan in _plans(32, 1, 32, 64, 1000):
        _say("config1", name)
        got = CApiSession(K, V, 1001).step(q.numpy(), k.numpy(), v.numpy(), 0.125, 1000, plan=plan)
        assert float(np.abs(got - want).max()) <= 1e-6, name


# ------------------------------------------------------------------ padding variants
@pytest.mark.parametrize("prec", [16, 32])
def test_left_padding_first_key(prec):
    """seq_lengths with right_or_no_padding = 0: keys before first_key[b] are masked
    (attention.cu:814-817, :1054, :1112-1113)."""
    B, H, Dh, t = 4, 3, 64, 300
    rng, K, V = rand_inputs(7, B, H, t, Dh, prec)
    q, k, v = rand_token(rng, B, H, Dh, prec)
    first = np.array([0, 1, 130, 300], dtype=np.int32)
    want = O.decode_step(q, k, v, O.pack_k_cache(K, t + 1), O.pack_v_cache(V, t + 1), 0.125, t,
                         seq_lengths=first, right_or_no_padding=False, acc=np.float64)
    for name, plan in _plans(prec, B, H, Dh, t):
        _say("left_pad", prec, name)
        got = CApiSession(K, V, t + 1).step(q, k, v, 0.125, t, plan=plan, seq_lengths=first,
                                            right_or_no_padding=False)
        assert float(np.abs(got - want).max()) <= _tol(prec, V, v), name   # sample 3 sees one key
    # every key masked (first_key > t): sum = 0 and the reference's output is 0
    got = CApiSession(K, V, t + 1).step(q, k, v, 0.125, t, seq_lengths=np.full(B, t + 5, np.int32),
                                        right_or_no_padding=False)
    np.testing.assert_array_equal(got, np.zeros_like(got))


@pytest.mark.parametrize("prec", [16, 32])
def test_right_padding_per_sample_length(prec):
    """seq_lengths with right_or_no_padding = 1: per-sample slot replaces t
    (attention.cu:809-811)."""
    B, H, Dh, t = 3, 2, 64, 260
    rng, K, V = rand_inputs(8, B, H, t, Dh, prec)
    q, k, v = rand_token(rng, B, H, Dh, prec)
    lens = np.array([260, 64, 5], dtype=np.int32)
    kc0, vc0 = O.pack_k_cache(K, t + 1), O.pack_v_cache(V, t + 1)
    want = O.decode_step(q, k, v, kc0, vc0, 0.125, t, seq_lengths=lens, right_or_no_padding=True,
                         acc=np.float64)
    for name, plan in _plans(prec, B, H, Dh, t):
        _say("right_pad", prec, name)
        sess = CApiSession(K, V, t + 1)
        got = sess.step(q, k, v, 0.125, t, plan=plan, seq_lengths=lens, right_or_no_padding=True)
        assert float(np.abs(got - want).max()) <= _tol(prec, V, v), name
        gk, gv = sess.caches()
        for b in range(B):   # slot lens[b] now holds the new token; the prompt rows beyond are untouched
            n = lens[b] + 1
            np.testing.assert_array_equal(gk[b, :, :, :n], kc0[b, :, :, :n])
            np.testing.assert_array_equal(gv[b, :, :n], vc0[b, :, :n])


# ------------------------------------------------------------------ pruning (p > 0)
def _peaked(prec, seed, B, H, L, Dh, npeaks=16):
    rng, K, V = rand_inputs(seed, B, H, L, Dh, prec)
    q, k, v = rand_token(rng, B, H, Dh, prec)
    qd = q.astype(np.float32) / np.linalg.norm(q.astype(np.float32), axis=-1, keepdims=True)
    for b in range(B):
        for h in range(H):
            pos = rng.choice(L, npeaks, replace=False)
            K[b, h, pos] = (4 * qd[b, h] + 0.1 * rng.standard_normal((npeaks, Dh))).astype(K.dtype)
    return K, V, q, k, v


def _near_threshold(prec, P, thr):
    """Keys whose skip decision may legitimately differ between two correct evaluations of
    the rule: fp32 -- probability within 1e-5 relative of the threshold; fp16 -- moving the
    rounded probability or the rounded threshold by one fp16 ulp changes the decision."""
    if prec == 32:
        return np.abs(P - thr[:, :, None]) <= 1e-5 * np.abs(thr[:, :, None]) + 1e-30
    a = P.astype(np.float16).view(np.uint16).astype(np.int64)
    tb = np.broadcast_to(thr.astype(np.float16).view(np.uint16).astype(np.int64)[:, :, None], a.shape)
    base = O.leq_f16_bits(a, tb)
    near = np.zeros(a.shape, bool)
    for da in (-1, 0, 1):
        for db in (-1, 0, 1):
            near |= O.leq_f16_bits(np.clip(a + da, 0, 0x7BFF), np.clip(tb + db, 0, 0x7BFF)) != base
    return near


@pytest.mark.parametrize("prec", [16, 32])
@pytest.mark.parametrize("Dh,L", [(64, 900), (80, 500), (256, 300)])
@pytest.mark.parametrize("p", [1e-4, 1e-3, 1e-2, 0.3])
def test_pruned_step_matches_rule(prec, Dh, L, p):
    """Skip set and output against the CPU transcription of attention.cu's pruning rule.
    exp/sum are evaluated in a different order on the GPU, so a key whose probability sits
    within one quantum of the threshold may flip; every other key must agree, and the
    output must equal the rule's output for the GPU's own skip set."""
    B, H = 2, 3
    K, V, q, k, v = _peaked(prec, 11, B, H, L, Dh)
    Lmax = L + 1
    scale = 1.0 / np.sqrt(Dh)   # peaked keys score 4*|q|*scale ~ 4 against N(0,1) for the rest
    want, skip, P, thr = O.pruned_decode_step(q, k, v, O.pack_k_cache(K, Lmax), O.pack_v_cache(V, Lmax),
                                              scale, L, p)
    ntiles = L // 64 + 1
    plans = [capi.make_plan(capi.FFA_LAUNCH_WORKGROUP, waves, 1, ntiles) for waves in (1, 4, 16)]
    plans += [capi.make_plan(capi.FFA_LAUNCH_TWO_PASS, waves, -(-ntiles // tps), tps)
              for waves, tps in ((1, 1), (4, 2), (8, 5), (4, ntiles))]
    plans.append(None)   # planned by the library: few pairs -> two-pass
    for plan in plans:
        _say("pruned", prec, Dh, L, p, plan)
        got, kept, gmask = CApiSession(K, V, Lmax).step(q, k, v, scale, L, p=p, plan=plan, diag=True)
        near = _near_threshold(prec, P, thr)
        diff = gmask != skip
        assert not (diff & ~near).any(), "skip decision differs away from the threshold"
        assert diff.mean() < 1e-3
        np.testing.assert_array_equal(kept, (L - gmask[:, :, :L].sum(axis=-1)))
        assert not gmask[:, :, L:].any()
        Vall = np.concatenate([V, v[:, :, None]], axis=2).astype(np.float32)
        w = np.where(gmask[:, :, :L + 1], 0, P[:, :, :L + 1])
        want_g = np.einsum("bhn,bhnd->bhd", w, Vall)
        assert float(np.abs(got - want_g).max()) <= (1e-3 if prec == 16 else 1e-5)
    frac = skip[:, :, :L].mean()
    _say("  skipped fraction", frac)
    if p >= 1e-2:
        assert frac > 0.05


@pytest.mark.parametrize("prec", [16, 32])
def test_pruned_tiny_threshold_equals_exact(prec):
    B, H, Dh, L = 2, 2, 64, 500
    K, V, q, k, v = _peaked(prec, 12, B, H, L, Dh)
    plan = capi.make_plan(capi.FFA_LAUNCH_WORKGROUP, 4, 1, L // 64 + 1)
    exact = CApiSession(K, V, L + 1).step(q, k, v, 0.125, L, p=0.0, plan=plan)
    tiny = CApiSession(K, V, L + 1).step(q, k, v, 0.125, L, p=1e-30, plan=plan)
    assert np.abs(exact - tiny).max() <= (2e-3 if prec == 16 else 2e-6)


@pytest.mark.parametrize("prec", [16, 32])
def test_sequences_beyond_lds(prec):
    """45001 keys: the scores no longer fit LDS, so pruned and default launches go through the
    two-pass kernels; exact against the closed form, pruned against the rule."""
    B, H, Dh, L = 1, 2, 64, 45000
    K, V, q, k, v = _peaked(prec, 13, B, H, L, Dh)
    Lmax, scale = L + 8, 0.125
    kc0, vc0 = O.pack_k_cache(K, Lmax), O.pack_v_cache(V, Lmax)
    want = O.decode_step(q, k, v, kc0, vc0, scale, L, acc=np.float64)
    wg = capi.make_plan(capi.FFA_LAUNCH_WORKGROUP, 16, 1, L // 64 + 1)
    CApiSession(K[:, :, :8], V[:, :, :8], Lmax).step(q, k, v, scale, L, plan=wg, expect=capi.FFA_ERR_TOO_LONG)
    for name, plan in (("default", capi.plan_launch(prec, B, H, Dh, L, 0.0, True)), ("tuned", None)):
        _say("beyond_lds exact", prec, name)
        sess = CApiSession(K, V, Lmax)
        got = sess.step(q, k, v, scale, L, plan=plan)
        assert float(np.abs(got - want).max()) <= _tol(prec, V, v), name
        gk, gv = sess.caches()
        np.testing.assert_array_equal(gk[..., :L + 1, :], kc0[..., :L + 1, :])
        np.testing.assert_array_equal(gv[:, :, :L + 1], vc0[:, :, :L + 1])
    p = 0.05     # the rule compares exp(s_i - max) with p: peaks sit ~4.5 above the N(0,1) bulk
    want_p, skip, P, thr = O.pruned_decode_step(q, k, v, kc0, vc0, scale, L, p)
    for name, plan in (("default", capi.plan_launch(prec, B, H, Dh, L, p, True)), ("tuned", None)):
        _say("beyond_lds pruned", prec, name)
        got, kept, gmask = CApiSession(K, V, Lmax).step(q, k, v, scale, L, p=p, plan=plan, diag=True)
        diff = gmask != skip
        assert not (diff & ~_near_threshold(prec, P, thr)).any()
        np.testing.assert_array_equal(kept, (L - gmask[:, :, :L].sum(axis=-1)))
        Vall = np.concatenate([V, v[:, :, None]], axis=2).astype(np.float32)
        w = np.where(gmask[:, :, :L + 1], 0, P[:, :, :L + 1])
        assert float(np.abs(got - np.einsum("bhn,bhnd->bhd", w, Vall)).max()) <= (1e-3 if prec == 16 else 1e-5)
    assert skip[:, :, :L].mean() > 0.5


# ------------------------------------------------------------------ full-size properties
def test_full_size_config2_properties():
    """BASELINE config 2 at full size (B=10, 32x64, fp16, t=1255): the two independent
    kernels agree, both agree with an fp32 torch evaluation on the GPU, V = 1 gives 1, and
    repeating the step leaves the result unchanged (idempotent append)."""
    B, H, Dh, L, Lmax = 10, 32, 64, 1255, 1256
    g = torch.Generator().manual_seed(0)
    K = (0.5 * torch.randn(B, H, L, Dh, generator=g)).half()
    V = (0.5 * torch.randn(B, H, L, Dh, generator=g)).half()
    q, k, v = (torch.randn(B, H, Dh, generator=g).half() for _ in range(3))
    sess = CApiSession(K.numpy(), V.numpy(), Lmax)
    _say("full split")
    a = sess.step(q.numpy(), k.numpy(), v.numpy(), 0.125, L)
    _say("full split again")
    a2 = sess.step(q.numpy(), k.numpy(), v.numpy(), 0.125, L)
    _say("full default")
    b = sess.step(q.numpy(), k.numpy(), v.numpy(), 0.125, L, plan=capi.plan_launch(16, B, H, Dh, L, 0.0, True))
    np.testing.assert_array_equal(a, a2)
    Kc = torch.cat([K, k[:, :, None]], 2).cuda().float().reshape(B * H, L + 1, Dh)
    Vc = torch.cat([V, v[:, :, None]], 2).cuda().float().reshape(B * H, L + 1, Dh)
    w = torch.softmax(torch.bmm(q.cuda().float().reshape(B * H, 1, Dh), Kc.transpose(1, 2)) * 0.125, -1)
    ref = torch.bmm(w, Vc).reshape(B, H, Dh).cpu().numpy()
    assert np.abs(a - ref).max() <= 1e-3 and np.abs(b - ref).max() <= 1e-3
    assert np.abs(a - b).max() <= 1e-3
    ones = np.ones((B, H, L, Dh), np.float16)
    sess1 = CApiSession(K.numpy(), ones, Lmax)
    c = sess1.step(q.numpy(), k.numpy(), np.ones((B, H, Dh), np.float16), 0.125, L)
    np.testing.assert_allclose(c, 1.0, atol=1e-3)


# ------------------------------------------------------------------ randomized sweep
def _random_plan(rng, prec, B, H, Dh, t, p):
    ntiles = t // 64 + 1
    kinds = ["library", "default", "workgroup", "two_pass"] + (["split"] * 2 if p == 0 else [])
    kind = kinds[rng.integers(len(kinds))]
    if kind == "library":
        return kind, None
    if kind == "default":
        return kind, capi.plan_launch(prec, B, H, Dh, t, p, True)
    if kind == "workgroup":
        return kind, capi.make_plan(capi.FFA_LAUNCH_WORKGROUP, int(rng.choice([1, 2, 4, 8, 16])), 1, ntiles)
    waves = int(rng.choice([1, 2, 4, 8]))
    tps = int(rng.integers(1, ntiles + 1))
    ns = -(-ntiles // tps)
    if ns > 128:
        tps, ns = ntiles, 1
    if kind == "two_pass":
        return kind, capi.make_plan(capi.FFA_LAUNCH_TWO_PASS, waves, ns, tps)
    whole = int(rng.integers(0, B * H + 1))
    combine = int(rng.integers(2))
    return kind, capi.make_plan(capi.FFA_LAUNCH_SPLIT, waves, ns, tps, combine, whole)


@pytest.mark.parametrize("seed", range(12))
def test_random_shapes_plans_and_padding(seed):
    """Random head dims, lengths, paddings, thresholds and launch plans (every kind, every wave
    count, ragged pieces), ten cases per seed, each against the oracle."""
    rng = np.random.default_rng(1000 + seed)
    for case in range(10):
        prec = int(rng.choice([16, 32]))
        Dh = int(rng.choice([64, 80, 128, 256]))
        B, H = int(rng.integers(1, 4)), int(rng.integers(1, 6))
        t = int(rng.choice([0, 1, 63, 64, 65, 127, 128, int(rng.integers(2, 700))]))
        Lmax = t + int(rng.integers(1, 70))
        p = float(rng.choice([0.0, 0.0, 1e-3, 0.05]))
        pad = str(rng.choice(["none", "left", "right"]))
        K, V, q, k, v = _peaked(prec, int(rng.integers(1 << 30)), B, H, t, Dh, npeaks=min(8, t))
        scale = 1.0 / np.sqrt(Dh)
        sl, rnp = None, True
        if pad == "left":
            sl, rnp = rng.integers(0, t + 2, B).astype(np.int32), False      # t+1: every key masked
        elif pad == "right":
            sl = rng.integers(0, t + 1, B).astype(np.int32)
        kind, plan = _random_plan(rng, prec, B, H, Dh, t, p)
        _say("random", seed, case, dict(prec=prec, Dh=Dh, B=B, H=H, t=t, Lmax=Lmax, p=p, pad=pad,
                                        sl=None if sl is None else sl.tolist(), kind=kind, plan=plan))
        kc0, vc0 = O.pack_k_cache(K, Lmax), O.pack_v_cache(V, Lmax)
        sess = CApiSession(K, V, Lmax)
        if p == 0.0:
            want = O.decode_step(q, k, v, kc0, vc0, scale, t, seq_lengths=sl, right_or_no_padding=rnp,
                                 acc=np.float64)
            got = sess.step(q, k, v, scale, t, plan=plan, seq_lengths=sl, right_or_no_padding=rnp)
            assert float(np.abs(got - want).max()) <= _tol(prec, V, v)
        else:
            want, skip, P, thr = O.pruned_decode_step(q, k, v, kc0, vc0, scale, t, p, seq_lengths=sl,
                                                      right_or_no_padding=rnp)
            got, kept, gmask = sess.step(q, k, v, scale, t, p=p, plan=plan, seq_lengths=sl,
                                         right_or_no_padding=rnp, diag=True)
            diff = gmask != skip
            assert not (diff & ~_near_threshold(prec, P, thr)).any()
            tl = np.full(B, t) if (sl is None or not rnp) else sl
            for b in range(B):
                n = int(tl[b])
                np.testing.assert_array_equal(kept[b], n - gmask[b, :, :n].sum(axis=-1))
                Vb = np.concatenate([V[b, :, :n], v[b, :, None]], axis=1).astype(np.float32)
                w = np.where(gmask[b, :, :n + 1], 0, P[b, :, :n + 1])
                want_g = np.einsum("hn,hnd->hd", w, Vb)
                assert float(np.abs(got[b] - want_g).max()) <= (1e-3 if prec == 16 else 1e-5) * max(1.0, float(np.abs(Vb).max()))
        gk, gv = sess.caches()
        tl = np.full(B, t) if (sl is None or not rnp) else sl
        for b in range(B):        # caches: prompt + the appended token, bit for bit
            n = int(tl[b]) + 1
            np.testing.assert_array_equal(gk[b, :, :, :n], kc0[b, :, :, :n])
            np.testing.assert_array_equal(gv[b, :, :n], vc0[b, :, :n])


@pytest.mark.parametrize("prec,iters", [(16, 300), (32, 1200)])
def test_cross_workgroup_merge_stress(prec, iters):
    """Many launches of the hybrid whole/split plan (the pieces publish their partials while
    the whole pairs still stream at full bandwidth) and of a merge-heavy plan, against the
    one-workgroup kernel on the same inputs: a partial that is read before it has arrived
    shows up as a large error in some pair of some launch."""
    B, H, Dh, t = 10, 32, 64, 1100
    rng, K, V = rand_inputs(21, B, H, t, Dh, prec)
    Lmax = t + 4
    sess = CApiSession(K, V, Lmax)
    ntiles = t // 64 + 1
    wg = capi.make_plan(capi.FFA_LAUNCH_WORKGROUP, 8, 1, ntiles)
    hybrid = capi.make_plan(capi.FFA_LAUNCH_SPLIT, 4, -(-ntiles // 5), 5, 0, 256)
    fine = capi.make_plan(capi.FFA_LAUNCH_SPLIT, 4, -(-ntiles // 2), 2, 0, 0)
    two_pass = capi.make_plan(capi.FFA_LAUNCH_TWO_PASS, 4, -(-ntiles // 2), 2)
    tol = 1e-3 if prec == 16 else 2e-6
    dev, tdt = "cuda:0", torch.float16 if prec == 16 else torch.float32
    out = torch.empty(B, H, Dh, dtype=tdt, device=dev)
    ref = torch.empty(B, H, Dh, dtype=tdt, device=dev)
    fn = sess.lib.ffa_attention_f16 if prec == 16 else sess.lib.ffa_attention_f32
    from tests.ffa_testlib import ptr
    import ctypes as C

    def launch(plan, q, k, v, dst):
        rc = fn(B, H, Dh, Lmax, 0.125, t, ptr(q), ptr(k), ptr(v), ptr(sess.k_cache), ptr(sess.v_cache), ptr(dst),
                None, 0.0, C.byref(plan), 1, ptr(sess.ws), sess.ws.numel(), None)
        assert rc == 0

    g = torch.Generator(device=dev).manual_seed(3)
    worst = 0.0
    for it in range(iters):
        q, k, v = (torch.randn(B, H, Dh, device=dev, generator=g).to(tdt) for _ in range(3))
        launch(wg, q, k, v, ref)
        for plan in (hybrid, fine, two_pass) if it % 4 == 0 else (hybrid,):
            launch(plan, q, k, v, out)
            err = float((out.float() - ref.float()).abs().max())
            worst = max(worst, err)
            assert err <= tol, (it, plan, err)
    _say("merge stress", prec, iters, "launches, worst difference", worst)
