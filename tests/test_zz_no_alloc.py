"""GPU test of ffa_attention_static_scratch, the entry point that takes no workspace and
allocates nothing: through the C ABI, against ffa_attention_diag (caller-owned workspace) on
the same inputs and the same launch plan.  Same kernels, same plan, same merge order: the
outputs and the caches must agree bit for bit.  Each case makes two calls in a row on the
GPU's one scratch array, the second on a smaller problem, so whatever the first call left in
the array (counters, partials, scores) is there when the second one runs."""
import ctypes as C

import numpy as np
import pytest
import torch

from fastforwardattention_amd import capi
from tests.ffa_testlib import CApiSession, ptr, rand_inputs, rand_token

pytestmark = pytest.mark.gpu


def _both(sess, q, k, v, scale, t, p, plan):
    """(output via the static scratch, output via the workspace, caches after each)."""
    dev, tdt = "cuda:0", sess.k_cache.dtype
    qd, kd, vd = (torch.from_numpy(np.ascontiguousarray(x)).to(dev) for x in (q, k, v))
    plan_p = C.byref(plan) if plan is not None else None
    outs, caches = [], []
    kc0, vc0 = sess.k_cache.clone(), sess.v_cache.clone()
    for static in (True, False):
        sess.k_cache.copy_(kc0)
        sess.v_cache.copy_(vc0)
        out = torch.full((sess.B, sess.H, sess.Dh), float("nan"), dtype=tdt, device=dev)
        if static:
            rc = sess.lib.ffa_attention_static_scratch(
                sess.precision, sess.B, sess.H, sess.Dh, sess.Lmax, float(scale), int(t), ptr(qd), ptr(kd), ptr(vd),
                ptr(sess.k_cache), ptr(sess.v_cache), ptr(out), None, float(p), plan_p, 1, None, None, None)
        else:
            rc = sess.lib.ffa_attention_diag(
                sess.precision, sess.B, sess.H, sess.Dh, sess.Lmax, float(scale), int(t), ptr(qd), ptr(kd), ptr(vd),
                ptr(sess.k_cache), ptr(sess.v_cache), ptr(out), None, float(p), plan_p, 1, ptr(sess.ws),
                sess.ws.numel(), None, None, None)
        assert rc == capi.FFA_OK, capi.STATUS_NAMES.get(rc, rc)
        torch.cuda.synchronize()
        outs.append(out.cpu().numpy())
        caches.append((sess.k_cache.cpu().numpy(), sess.v_cache.cpu().numpy()))
    return outs, caches


def _check(tag, prec, B, H, Dh, t, p, plan):
    print("static scratch", tag, dict(prec=prec, B=B, H=H, Dh=Dh, t=t, p=p, plan=plan), flush=True)
    rng, K, V = rand_inputs(77 + t, B, H, t, Dh, prec, kv_scale=0.5)
    q, k, v = rand_token(rng, B, H, Dh, prec)
    sess = CApiSession(K, V, t + 2)
    (a, b), ((ka, va), (kb, vb)) = _both(sess, q, k, v, 0.125, t, p, plan)
    assert np.isfinite(a).all()
    np.testing.assert_array_equal(a.view(np.uint8), b.view(np.uint8), err_msg=tag)
    np.testing.assert_array_equal(ka.view(np.uint8), kb.view(np.uint8), err_msg=tag)
    np.testing.assert_array_equal(va.view(np.uint8), vb.view(np.uint8), err_msg=tag)


@pytest.mark.parametrize("prec", [16, 32])
def test_static_scratch_matches_workspace_entry(prec):
    # exact, library plan: hybrid whole/split launch (partials + counters in the scratch), then
    # a smaller problem whose pairs are all split
    _check("exact big", prec, 10, 32, 64, 1100, 0.0, None)
    _check("exact small", prec, 1, 32, 64, 500, 0.0, None)
    # pruned, few pairs: the two-pass kernels keep scores, (max, sum) and partials in the scratch
    _check("pruned big", prec, 1, 8, 128, 3000, 1e-2, None)
    _check("pruned small", prec, 1, 3, 64, 700, 1e-2, None)
    # explicit plans: fine split with the merge kernel, then a one-workgroup plan (no scratch)
    nt = 900 // 64 + 1
    _check("split merge-kernel", prec, 2, 5, 256, 900, 0.0,
           capi.make_plan(capi.FFA_LAUNCH_SPLIT, 2, -(-nt // 2), 2, capi.FFA_COMBINE_KERNEL, 3))
    _check("workgroup", prec, 2, 5, 80, 333, 0.0, capi.make_plan(capi.FFA_LAUNCH_WORKGROUP, 4, 1, 333 // 64 + 1))


def test_static_scratch_rejects_oversized_plan():
    """A plan whose workspace need exceeds the array is refused before anything is launched:
    two-pass scores of 64 pairs x 20000 keys are 5 MB."""
    B, H, Dh, t = 2, 32, 64, 20000
    sess = CApiSession(np.zeros((B, H, 8, Dh), np.float16), np.zeros((B, H, 8, Dh), np.float16), t + 1)
    x = torch.zeros(B, H, Dh, dtype=torch.float16, device="cuda:0")
    out = torch.full((B, H, Dh), 7.0, dtype=torch.float16, device="cuda:0")
    nt = t // 64 + 1
    plan = capi.make_plan(capi.FFA_LAUNCH_TWO_PASS, 4, 4, -(-nt // 4))
    rc = sess.lib.ffa_attention_static_scratch(16, B, H, Dh, t + 1, 0.125, t, ptr(x), ptr(x), ptr(x), ptr(sess.k_cache),
                                                ptr(sess.v_cache), ptr(out), None, 0.01, C.byref(plan), 1, None, None, None)
    assert rc == capi.FFA_ERR_SCRATCH_LIMIT
    assert b"scratch" in sess.lib.ffa_status_string(rc)
    torch.cuda.synchronize()
    assert float(out.min()) == 7.0 and float(out.max()) == 7.0      # nothing ran


def test_static_scratch_in_a_captured_graph():
    """The call allocates nothing and records no memset node, so it can be captured; every replay
    (with eager work and synchronisation in between) reproduces the eager result."""
    prec, B, H, Dh, t = 16, 1, 32, 64, 2000
    rng, K, V = rand_inputs(5, B, H, t, Dh, prec, kv_scale=0.5)
    q, k, v = rand_token(rng, B, H, Dh, prec)
    sess = CApiSession(K, V, t + 2)
    dev = "cuda:0"
    qd, kd, vd = (torch.from_numpy(x).to(dev) for x in (q, k, v))
    out = torch.zeros(B, H, Dh, dtype=torch.float16, device=dev)

    def call(stream_ptr):
        rc = sess.lib.ffa_attention_static_scratch(16, B, H, Dh, t + 2, 0.125, t, ptr(qd), ptr(kd), ptr(vd),
                                                    ptr(sess.k_cache), ptr(sess.v_cache), ptr(out), None, 0.0, None, 1,
                                                    None, None, stream_ptr)
        assert rc == capi.FFA_OK
    call(None)
    torch.cuda.synchronize()
    eager = out.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        call(torch.cuda.current_stream().cuda_stream)
    for _ in range(4):
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager)
        call(None)                       # eager work between the replays
        torch.cuda.synchronize()
        assert torch.equal(out, eager)


def _ex_pair(prec, B, H, Dh, t, bw, seed):
    """One step with a rotary embedding, a q and k bias and a random beam table: through the static
    scratch and through ffa_attention_ex with a workspace.  Bit-equal outputs and caches."""
    print("static scratch with transform and beams", dict(prec=prec, B=B, H=H, Dh=Dh, t=t, bw=bw), flush=True)
    rng, K, V = rand_inputs(seed, B, H, t, Dh, prec, kv_scale=0.5)
    q, k, v = rand_token(rng, B, H, Dh, prec)
    sess = CApiSession(K, V, t + 2)
    dev, tdt = "cuda:0", sess.k_cache.dtype
    qd, kd, vd = (torch.from_numpy(np.ascontiguousarray(x)).to(dev) for x in (q, k, v))
    bias = [torch.from_numpy((0.25 * rng.standard_normal((H, Dh))).astype(np.float32)).to(dev).to(tdt) for _ in range(2)]
    tt = capi.TokenTransform(bias[0].data_ptr(), bias[1].data_ptr(), None, Dh // 2, 0.0)
    table = torch.from_numpy(rng.integers(0, bw, size=(B, t + 2)).astype(np.int32)).to(dev)
    bi = capi.BeamIndirection(table.data_ptr(), bw)
    kc0, vc0 = sess.k_cache.clone(), sess.v_cache.clone()
    got = []
    for static in (True, False):
        sess.k_cache.copy_(kc0)
        sess.v_cache.copy_(vc0)
        out = torch.full((B, H, Dh), float("nan"), dtype=tdt, device=dev)
        head = (sess.precision, B, H, Dh, sess.Lmax, 0.125, t, ptr(qd), ptr(kd), ptr(vd), ptr(sess.k_cache),
                ptr(sess.v_cache), ptr(out), None, 0.0, None, 1, C.byref(tt), C.byref(bi))
        if static:
            rc = sess.lib.ffa_attention_static_scratch(*head, None)
        else:
            rc = sess.lib.ffa_attention_ex(*head, ptr(sess.ws), sess.ws.numel(), None)
        assert rc == capi.FFA_OK, capi.STATUS_NAMES.get(rc, rc)
        torch.cuda.synchronize()
        got.append((out.cpu().numpy(), sess.k_cache.cpu().numpy(), sess.v_cache.cpu().numpy()))
    assert np.isfinite(got[0][0].astype(np.float32)).all()
    for a, b in zip(*got):
        np.testing.assert_array_equal(a.view(np.uint8), b.view(np.uint8))
    # the transform did happen: the appended key differs from the raw k
    assert not np.array_equal(got[0][1], kc0.cpu().numpy())


@pytest.mark.parametrize("prec", [16, 32])
def test_static_scratch_takes_transform_and_beams(prec):
    """Two calls in a row on the GPU's one scratch array, the second on a smaller problem."""
    _ex_pair(prec, 4, 16, 64, 1500, 2, 11)     # split pairs: partials and counters in the scratch
    _ex_pair(prec, 2, 4, 128, 300, 2, 12)
