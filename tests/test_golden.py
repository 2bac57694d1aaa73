"""Golden fixtures (tests/golden/decode_cases.npz, written by tests/golden/make_golden.py):
the CPU oracle must still reproduce them, and the HIP path must match them through the C ABI
-- exact steps to 1e-3 (fp16) / 1e-6 scaled (fp32), pruned steps to the skip set and output
of the rule, cache contents bit for bit."""
import os

import numpy as np
import pytest

from oracle import ffa_oracle as O

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "decode_cases.npz")
# name: (B, H, Dh, t, first_key per sample or None)
CASES = {"t0": (1, 2, 64, 0, None), "t37": (2, 3, 64, 37, None), "dh256_t130": (1, 2, 256, 130, None),
         "leftpad_t300": (2, 2, 64, 300, [0, 77])}
THRESHOLDS = (1e-3, 1e-2, 0.2)
DTYPE = {16: np.float16, 32: np.float32}


@pytest.fixture(scope="module")
def golden():
    with np.load(GOLDEN, allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


def _inputs(golden, name, prec):
    return tuple(golden[f"{name}/{key}"].astype(DTYPE[prec]) for key in ("K", "V", "q", "k", "v"))


def _skip(golden, name, prec, p, Lmax):
    return np.unpackbits(golden[f"{name}/f{prec}/skip_p{p:g}"], axis=-1)[..., :Lmax].astype(bool)


@pytest.mark.parametrize("prec", [16, 32])
@pytest.mark.parametrize("name", list(CASES))
def test_oracle_reproduces_golden(golden, name, prec):
    B, H, Dh, t, first = CASES[name]
    K, V, q, k, v = _inputs(golden, name, prec)
    assert K.shape == (B, H, t, Dh)
    Lmax, scale = t + 2, 1.0 / np.sqrt(Dh)
    sl = None if first is None else np.asarray(first, np.int32)
    kc, vc = O.pack_k_cache(K, Lmax), O.pack_v_cache(V, Lmax)
    out = O.decode_step(q, k, v, kc, vc, scale, t, seq_lengths=sl, right_or_no_padding=sl is None,
                        acc=np.float64)
    assert float(np.abs(out - golden[f"{name}/f{prec}/out_exact"]).max()) <= 1e-6
    if f"{name}/f{prec}/k_cache" in golden:
        np.testing.assert_array_equal(kc, golden[f"{name}/f{prec}/k_cache"])
        np.testing.assert_array_equal(vc, golden[f"{name}/f{prec}/v_cache"])
    for p in THRESHOLDS:
        kc, vc = O.pack_k_cache(K, Lmax), O.pack_v_cache(V, Lmax)
        out, skip, P, thr = O.pruned_decode_step(q, k, v, kc, vc, scale, t, p, seq_lengths=sl,
                                                 right_or_no_padding=sl is None)
        np.testing.assert_array_equal(skip, _skip(golden, name, prec, p, Lmax))
        assert float(np.abs(out - golden[f"{name}/f{prec}/out_p{p:g}"]).max()) <= 1e-6


def test_golden_skip_sets_are_not_trivial(golden):
    """The fixture must exercise the rule: the thresholds prune something, never everything."""
    for prec in (16, 32):
        fr = [_skip(golden, "leftpad_t300", prec, p, 302)[1, :, 77:300].mean() for p in THRESHOLDS]
        assert 0.0 < fr[0] < fr[1] < fr[2] < 1.0
        assert _skip(golden, "leftpad_t300", prec, 1e-3, 302)[1, :, :77].all()      # left padding is dropped
        assert not _skip(golden, "t0", prec, 0.2, 2).any()                          # the new token never is


@pytest.mark.gpu
@pytest.mark.parametrize("prec", [16, 32])
@pytest.mark.parametrize("name", list(CASES))
def test_hip_matches_golden(golden, name, prec):
    from fastforwardattention_amd import capi
    from tests.ffa_testlib import CApiSession
    from tests.test_gpu_parity import _near_threshold, _tol

    B, H, Dh, t, first = CASES[name]
    K, V, q, k, v = _inputs(golden, name, prec)
    Lmax, scale = t + 2, 1.0 / np.sqrt(Dh)
    sl = None if first is None else np.asarray(first, np.int32)
    ntiles = t // 64 + 1
    plans = [None, capi.plan_launch(prec, B, H, Dh, t, 0.0, True),
             capi.make_plan(capi.FFA_LAUNCH_SPLIT, 2, ntiles, 1),
             capi.make_plan(capi.FFA_LAUNCH_TWO_PASS, 2, ntiles, 1)]
    for plan in plans:
        print("golden exact", name, prec, plan, flush=True)
        sess = CApiSession(K, V, Lmax, sentinel=0.0)
        got = sess.step(q, k, v, scale, t, plan=plan, seq_lengths=sl, right_or_no_padding=sl is None)
        assert float(np.abs(got - golden[f"{name}/f{prec}/out_exact"]).max()) <= _tol(prec, V, v)
        if f"{name}/f{prec}/k_cache" in golden:
            kc, vc = sess.caches()
            np.testing.assert_array_equal(kc, golden[f"{name}/f{prec}/k_cache"])
            np.testing.assert_array_equal(vc, golden[f"{name}/f{prec}/v_cache"])
    Vall = np.concatenate([V, v[:, :, None]], axis=2).astype(np.float32)
    for p in THRESHOLDS:
        skip = _skip(golden, name, prec, p, Lmax)
        P, thr = golden[f"{name}/f{prec}/prob_p{p:g}"], golden[f"{name}/f{prec}/thr_p{p:g}"]
        for plan in (None, capi.make_plan(capi.FFA_LAUNCH_WORKGROUP, 2, 1, ntiles),
                     capi.make_plan(capi.FFA_LAUNCH_TWO_PASS, 1, ntiles, 1)):
            print("golden pruned", name, prec, p, plan, flush=True)
            got, kept, gmask = CApiSession(K, V, Lmax).step(q, k, v, scale, t, p=p, plan=plan, seq_lengths=sl,
                                                            right_or_no_padding=sl is None, diag=True)
            diff = gmask != skip
            assert not (diff & ~_near_threshold(prec, P, thr)).any()
            w = np.where(gmask[:, :, :t + 1], 0, P[:, :, :t + 1])
            want = np.einsum("bhn,bhnd->bhd", w, Vall)
            assert float(np.abs(got - want).max()) <= (1e-3 if prec == 16 else 1e-5)
            if not diff.any():
                assert float(np.abs(got - golden[f"{name}/f{prec}/out_p{p:g}"]).max()) <= (1e-3 if prec == 16 else 1e-5)
