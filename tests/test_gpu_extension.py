"""GPU tests of the Python surface: class FastForwardAttn of the compiled extension
`ff_attention`, used exactly like the reference's example (example.py:28-46)."""
import math

import numpy as np
import pytest
import torch

from oracle.torch_attn import torch_attn_func

pytestmark = pytest.mark.gpu


def _say(*a):
    print(*a, flush=True)


@pytest.mark.parametrize("dtype,tol", [(torch.float16, 1e-3), (torch.float32, 1e-6)])
@pytest.mark.parametrize("default_launch", [False, True])
def test_example_loop(dtype, tol, default_launch):
    """The reference demo, shrunk: B=10, H=32, Dh=64, prompt 1024 -> here prompt 200, 20 steps;
    randn instead of rand inputs; absolute instead of relative tolerance."""
    from ff_attention import FastForwardAttn as FFA  # the reference's import line
    _say("example_loop", dtype, default_launch)
    B, H, Dh, L, steps = 3, 8, 64, 200, 20
    g = torch.Generator().manual_seed(1)
    K = torch.randn(B, H, L, Dh, generator=g).to(dtype)
    V = torch.randn(B, H, L, Dh, generator=g).to(dtype)
    ffa = FFA(K.cuda(), V.cuda(), L + steps, default_launch)
    scale = 1 / math.sqrt(Dh)
    Kf, Vf = K.float(), V.float()
    for i in range(steps):
        q, k, v = (torch.randn(B, H, 1, Dh, generator=g).to(dtype) for _ in range(3))
        t = L + i
        out = ffa.attention(q.cuda(), k.cuda(), v.cuda(), scale, t, 0)
        assert out.shape == (B, H, Dh) and out.dtype == dtype and out.is_cuda
        Kf = torch.cat([Kf, k.float()], dim=-2)
        Vf = torch.cat([Vf, v.float()], dim=-2)
        want = torch_attn_func(q.float().view(B * H, 1, Dh), Kf.view(B * H, t + 1, Dh),
                               Vf.view(B * H, t + 1, Dh), scale).view(B, H, Dh)
        assert float((out.float().cpu() - want).abs().max()) <= tol


def test_cache_shapes_aliasing_and_overloads():
    from fastforwardattention_amd import FastForwardAttn as FFA
    B, H, Dh, L, Lmax = 2, 4, 128, 70, 80
    g = torch.Generator().manual_seed(2)
    K = torch.randn(B, H, L, Dh, generator=g).half().cuda()
    V = torch.randn(B, H, L, Dh, generator=g).half().cuda()
    ffa = FFA(K, V, Lmax, False)
    kc, vc = ffa.get_cache()
    assert tuple(kc.shape) == (B, H, Dh // 8, Lmax, 8) and tuple(vc.shape) == (B, H, Lmax, Dh)
    assert torch.equal(kc[:, :, :, :L, :], K.view(B, H, L, Dh // 8, 8).permute(0, 1, 3, 2, 4))
    assert torch.equal(vc[:, :, :L], V)
    q, k, v = (torch.randn(B, 1, H * Dh, generator=g).half().cuda() for _ in range(3))  # OPT's shape
    o1 = ffa.attention(q, k, v, 0.1, L, 0)
    # the caches are aliases: the append is visible through get_cache()
    assert torch.equal(kc[:, :, :, L, :].reshape(B, H, Dh), k.view(B, H, Dh))
    assert torch.equal(vc[:, :, L, :], v.view(B, H, Dh))
    # 8-argument overload on the same caches: same result (slot L is rewritten with the same row)
    o2 = ffa.attention(q, k, v, kc, vc, 0.1, L, 0)
    assert torch.equal(o1, o2)
    # 9-argument overload with first_key = 0 everywhere: same again
    o3 = ffa.attention(q, k, v, kc, vc, 0.1, L, torch.zeros(B, dtype=torch.int32, device="cuda"), 0)
    assert torch.equal(o1, o3)
    # left padding really masks
    sl = torch.tensor([0, 40], dtype=torch.int32, device="cuda")
    o4 = ffa.attention(q, k, v, kc, vc, 0.1, L, sl, 0)
    assert torch.equal(o4[0], o1[0]) and not torch.equal(o4[1], o1[1])
    Kf = torch.cat([K, k.view(B, H, 1, Dh)], 2).float()[1, :, 40:]
    Vf = torch.cat([V, v.view(B, H, 1, Dh)], 2).float()[1, :, 40:]
    want = torch_attn_func(q.view(B, H, 1, Dh)[1].float(), Kf, Vf, 0.1)[:, 0]
    assert float((o4[1].float() - want).abs().max()) <= 1e-3


def test_errors_raise():
    from fastforwardattention_amd import FastForwardAttn as FFA
    K = torch.randn(1, 2, 10, 64).half().cuda()
    ffa = FFA(K, K.clone(), 12, False)
    q = torch.randn(1, 2, 64).half().cuda()
    with pytest.raises(RuntimeError, match="timestep"):
        ffa.attention(q, q, q, 0.1, 12, 0)           # the reference writes past the cache here
    with pytest.raises(RuntimeError, match="elements"):
        ffa.attention(q[:, :1], q, q, 0.1, 10, 0)
    with pytest.raises(RuntimeError, match="dtype"):
        ffa.attention(q.float(), q, q, 0.1, 10, 0)
    with pytest.raises(RuntimeError, match="prob_thresh"):
        ffa.attention(q, q, q, 0.1, 10, -1.0)
    with pytest.raises(RuntimeError, match="head dim"):
        FFA(torch.randn(1, 2, 10, 96).half().cuda(), torch.randn(1, 2, 10, 96).half().cuda(), 12, False)
    with pytest.raises(RuntimeError):
        FFA(torch.randn(1, 2, 10, 64).double().cuda(), torch.randn(1, 2, 10, 64).double().cuda(), 12, False)
    with pytest.raises(TypeError):
        ffa.attention(q, q, q, 0.1, 10)               # p is positional and mandatory, as in the reference


def test_pruned_diag_and_stream():
    from fastforwardattention_amd import FastForwardAttn as FFA
    B, H, Dh, L = 2, 4, 64, 600
    g = torch.Generator().manual_seed(3)
    K = torch.randn(B, H, L, Dh, generator=g).half().cuda()
    V = torch.randn(B, H, L, Dh, generator=g).half().cuda()
    q, k, v = (torch.randn(B, H, Dh, generator=g).half().cuda() for _ in range(3))
    ffa = FFA(K, V, L + 1, False)
    exact = ffa.attention(q, k, v, 0.5, L, 0)
    out, kept, mask = ffa.attention_diag(q, k, v, 0.5, L, 5e-2)
    assert kept.shape == (B, H) and mask.shape == (B, H, L + 1)
    assert torch.equal(kept.long(), L - mask[:, :, :L].sum(-1).long())
    assert 0 < mask.float().mean() < 1
    assert float((out.float() - exact.float()).abs().max()) < 0.2
    plain = ffa.attention(q, k, v, 0.5, L, 5e-2)     # another launch plan: the same rule, another order of summation
    assert float((plain.float() - out.float()).abs().max()) <= 1e-3
    # a side stream: the extension launches on torch's current stream
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        o2 = ffa.attention(q, k, v, 0.5, L, 0)
    s.synchronize()
    assert torch.equal(o2, exact)
    assert len(ffa.launch_plan(L, 0.0)) == 8


@pytest.mark.parametrize("name,dtype,tol,B,H,Dh,L,gen,scale", [
    ("opt1.3b_b10", torch.float16, 1e-3, 10, 32, 64, 1000, 256, 0.125),
    ("gptj_b8", torch.float16, 1e-3, 8, 16, 256, 2000, 256, 0.0625),
    ("opt2.7b_b2", torch.float16, 1e-3, 2, 32, 80, 1000, 64, 80 ** -0.5),
    # fp32 at the headline shape: twice the bytes per key, the hybrid whole/split launch; the
    # shape on which a missing wait before the cross-workgroup merge once showed up
    ("opt1.3b_b10_f32", torch.float32, 1e-6, 10, 32, 64, 1024, 128, 0.125)])
@pytest.mark.parametrize("use_default", [False, True])
def test_full_size_iterative_decode_every_step(name, dtype, tol, B, H, Dh, L, gen, scale, use_default):
    """The BASELINE decode loops at full size through the Python class: kernel output against
    an fp32 torch evaluation (softmax(q K^T scale) V on the upcast inputs, on the GPU) at EVERY
    step, max-abs <= 1e-3 (fp16) / 1e-6 (fp32); afterwards the caches hold prompt + generated
    tokens bit for bit in the reference's layouts."""
    from ff_attention import FastForwardAttn as FFA
    print("full-size decode", name, "default launch" if use_default else "tuned", flush=True)
    g = torch.Generator().manual_seed(0)
    K = (0.5 * torch.randn(B, H, L, Dh, generator=g)).to(dtype).cuda()
    V = (0.5 * torch.randn(B, H, L, Dh, generator=g)).to(dtype).cuda()
    Lmax = L + gen
    ffa = FFA(K, V, Lmax, use_default)
    Kf = torch.zeros(B * H, Lmax, Dh, device="cuda", dtype=torch.float32)
    Vf = torch.zeros(B * H, Lmax, Dh, device="cuda", dtype=torch.float32)
    Kf[:, :L] = K.float().reshape(B * H, L, Dh)
    Vf[:, :L] = V.float().reshape(B * H, L, Dh)
    worst = 0.0
    for i in range(gen):
        t = L + i
        q, k, v = (torch.randn(B, H, 1, Dh, generator=g).to(dtype).cuda() for _ in range(3))
        out = ffa.attention(q, k, v, scale, t, 0)
        Kf[:, t] = k.float().reshape(B * H, Dh)
        Vf[:, t] = v.float().reshape(B * H, Dh)
        w = torch.softmax(torch.bmm(q.float().reshape(B * H, 1, Dh), Kf[:, :t + 1].transpose(1, 2)) * scale, -1)
        ref = torch.bmm(w, Vf[:, :t + 1]).reshape(B, H, Dh)
        err = float((out.float() - ref).abs().max())
        worst = max(worst, err)
        assert err <= tol, (i, err)
    print("  worst max-abs over", gen, "steps:", worst, flush=True)
    kc, vc = ffa.get_cache()
    assert torch.equal(vc.float().reshape(B * H, Lmax, Dh), Vf)
    assert torch.equal(kc.permute(0, 1, 3, 2, 4).reshape(B * H, Lmax, Dh).float(), Kf)


@pytest.mark.parametrize("default_launch", [False, True])
def test_decode_steps_replay_from_a_captured_graph(default_launch):
    """Four consecutive decode steps captured into one HIP graph (static q/k/v buffers) and
    replayed with fresh inputs, eager work and synchronisations in between: every replay must
    reproduce what eager calls give for the same inputs (the library records kernels only: no
    memsets, no allocations of its own in the step)."""
    from ff_attention import FastForwardAttn as FFA
    B, H, Dh, L, steps = 4, 32, 64, 700, 4         # 128 pairs: the split kernel with cross-workgroup merges
    g = torch.Generator().manual_seed(5)
    K = torch.randn(B, H, L, Dh, generator=g).half().cuda()
    V = torch.randn(B, H, L, Dh, generator=g).half().cuda()
    ffa_graph = FFA(K, V, L + steps, default_launch)
    ffa_eager = FFA(K, V, L + steps, default_launch)
    qs, ks, vs = (torch.zeros(steps, B, H, 1, Dh, dtype=torch.float16, device="cuda") for _ in range(3))
    outs = torch.zeros(steps, B, H, Dh, dtype=torch.float16, device="cuda")

    def run_steps(ffa, dst):
        for i in range(steps):
            dst[i].copy_(ffa.attention(qs[i], ks[i], vs[i], 0.125, L + i, 0))

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run_steps(ffa_graph, outs)                  # warm-up on the capture stream
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        run_steps(ffa_graph, outs)
    for replay in range(3):
        for buf in (qs, ks, vs):
            buf.copy_(torch.randn(buf.shape, generator=g).half())
        graph.replay()
        torch.cuda.synchronize()
        got = outs.clone()
        want = torch.zeros_like(outs)
        run_steps(ffa_eager, want)                  # eager work between the replays
        torch.cuda.synchronize()
        assert float((got.float() - want.float()).abs().max()) <= 1e-3, replay
        for a, b in zip(ffa_graph.get_cache(), ffa_eager.get_cache()):
            assert torch.equal(a, b)
