"""CPU tests that pin the oracle (oracle/ffa_oracle.py) against independent evidence:
brute force, library routines, closed-form special cases and the reference's index
formulas.  None of these retypes the oracle's own formula."""
import math

import numpy as np
import pytest
import torch

from oracle import ffa_oracle as O
from oracle.torch_attn import CpuDecodeBaseline, torch_attn_func


def _rand(seed, *shape, dtype=np.float32):
    return np.random.default_rng(seed).standard_normal(shape).astype(dtype)


# ------------------------------------------------------------------ closed form
@pytest.mark.parametrize("T,Dh,first", [(1, 8, 0), (5, 8, 0), (9, 16, 3), (17, 8, 16)])
def test_closed_form_vs_bruteforce(T, Dh, first):
    q, K, V = _rand(1, Dh), _rand(2, T, Dh), _rand(3, T, Dh)
    want = O.attn_bruteforce(q, K, V, 0.37, first_key=first)
    got = O.attn_closed_form(q[None], K[None], V[None], 0.37, first_key=np.array([first]),
                             acc=np.float64)[0]
    np.testing.assert_allclose(got, want, rtol=1e-12, atol=1e-12)


def test_closed_form_vs_torch_library():
    N, T, Dh = 6, 301, 64
    q, K, V = _rand(4, N, Dh), _rand(5, N, T, Dh), _rand(6, N, T, Dh)
    want = torch_attn_func(torch.from_numpy(q)[:, None, :].double(), torch.from_numpy(K).double(),
                           torch.from_numpy(V).double(), 0.125)[:, 0].numpy()
    got64 = O.attn_closed_form(q, K, V, 0.125, acc=np.float64)
    got32 = O.attn_closed_form(q, K, V, 0.125, acc=np.float32)
    np.testing.assert_allclose(got64, want, rtol=1e-12, atol=1e-13)
    assert np.abs(got32 - want).max() < 2e-6  # fp32 oracle's own error bound


def test_special_cases():
    N, T, Dh = 3, 40, 16
    q, K, V = _rand(7, N, Dh), _rand(8, N, T, Dh), _rand(9, N, T, Dh)
    # one key only -> that value row, exactly
    np.testing.assert_array_equal(O.attn_closed_form(q, K[:, :1], V[:, :1], 0.3), V[:, 0])
    # q = 0 -> arithmetic mean of the values
    np.testing.assert_allclose(O.attn_closed_form(0 * q, K, V, 0.3, acc=np.float64),
                               V.astype(np.float64).mean(axis=1), rtol=1e-12)
    # one dominant key -> its value row
    K2 = K.copy()
    K2[:, 11] = 50.0 * q
    np.testing.assert_allclose(O.attn_closed_form(q, K2, V, 1.0, acc=np.float64), V[:, 11], atol=1e-9)
    # permutation of the cache positions leaves the result unchanged
    perm = np.random.default_rng(0).permutation(T)
    np.testing.assert_allclose(O.attn_closed_form(q, K[:, perm], V[:, perm], 0.3, acc=np.float64),
                               O.attn_closed_form(q, K, V, 0.3, acc=np.float64), rtol=1e-12)
    # (c*q, scale/c) invariance
    np.testing.assert_allclose(O.attn_closed_form(4 * q, K, V, 0.3 / 4, acc=np.float64),
                               O.attn_closed_form(q, K, V, 0.3, acc=np.float64), rtol=1e-12)
    # convexity
    out = O.attn_closed_form(q, K, V, 0.3, acc=np.float64)
    assert (out <= V.max(axis=1) + 1e-12).all() and (out >= V.min(axis=1) - 1e-12).all()
    # left padding == attention over the surviving suffix
    fk = np.array([0, 7, 39])
    got = O.attn_closed_form(q, K, V, 0.3, first_key=fk, acc=np.float64)
    for n in range(N):
        want = O.attn_closed_form(q[n:n + 1], K[n:n + 1, fk[n]:], V[n:n + 1, fk[n]:], 0.3, acc=np.float64)
        np.testing.assert_allclose(got[n], want[0], rtol=1e-12)


# ------------------------------------------------------------------ layouts
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_pack_matches_reference_index_formula(dtype):
    """Flat-index restatement of transpose_4d_batch_major_{k,v}_cache
    (attention.cu:1564-1582, :1593-1608), element by element."""
    B, H, L, Lmax, Dh = 2, 3, 5, 7, 16
    x = 16 // np.dtype(dtype).itemsize
    K = np.arange(B * H * L * Dh).reshape(B, H, L, Dh).astype(dtype)
    kc = O.pack_k_cache(K, Lmax, fill=-1).reshape(-1)
    vc = O.pack_v_cache(K, Lmax, fill=-1).reshape(-1)
    src = K.reshape(-1)
    nchunk = Dh // x
    for b in range(B):
        for h in range(H):
            src0 = b * H * Dh * L + h * Dh * L
            dst0 = b * H * Dh * Lmax + h * Dh * Lmax
            for out_idx in range(nchunk * Lmax):          # one uint4 per out_idx
                l = out_idx % Lmax
                c = (out_idx - l) // Lmax % nchunk
                for j in range(x):
                    got = kc[dst0 + out_idx * x + j]
                    if l < L:
                        assert got == src[src0 + (l * nchunk + c) * x + j]
                    else:
                        assert got == -1
            for idx in range(nchunk * L):
                for j in range(x):
                    assert vc[dst0 + idx * x + j] == src[src0 + idx * x + j]
    np.testing.assert_array_equal(O.unpack_k_cache(O.pack_k_cache(K, Lmax), L), K)


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_append_matches_reference_offsets(dtype):
    """K append offset bhi*Lmax*Dh + co*Lmax*x + t*x + ci (attention.cu:901-913);
    V append offset bhi*Lmax*Dh + t*Dh + vi (attention.cu:1142, :1246)."""
    B, H, Lmax, Dh, t = 2, 2, 6, 16, 4
    x = 16 // np.dtype(dtype).itemsize
    kc = np.zeros((B, H, Dh // x, Lmax, x), dtype)
    vc = np.zeros((B, H, Lmax, Dh), dtype)
    k = (1 + np.arange(B * H * Dh)).reshape(B, H, Dh).astype(dtype)
    v = (1000 + np.arange(B * H * Dh)).reshape(B, H, Dh).astype(dtype)
    O.append_kv(kc, vc, k, v, t)
    kflat, vflat = kc.reshape(-1), vc.reshape(-1)
    want_k, want_v = np.zeros_like(kflat), np.zeros_like(vflat)
    for bhi in range(B * H):
        for d in range(Dh):
            co, ci = d // x, d % x
            want_k[bhi * Lmax * Dh + co * Lmax * x + t * x + ci] = k.reshape(-1)[bhi * Dh + d]
            want_v[bhi * Lmax * Dh + t * Dh + d] = v.reshape(-1)[bhi * Dh + d]
    np.testing.assert_array_equal(kflat, want_k)
    np.testing.assert_array_equal(vflat, want_v)


def test_decode_step_equals_closed_form_on_concatenation():
    """example.py:40-42: append, then attend over the t+1 keys."""
    B, H, L, Dh, Lmax = 2, 3, 37, 64, 40
    K, V = _rand(10, B, H, L, Dh, dtype=np.float16), _rand(11, B, H, L, Dh, dtype=np.float16)
    q, k, v = (_rand(s, B, H, Dh, dtype=np.float16) for s in (12, 13, 14))
    kc, vc = O.pack_k_cache(K, Lmax), O.pack_v_cache(V, Lmax)
    out = O.decode_step(q, k, v, kc, vc, 0.125, L)
    Kcat = np.concatenate([K, k[:, :, None]], axis=2).reshape(B * H, L + 1, Dh)
    Vcat = np.concatenate([V, v[:, :, None]], axis=2).reshape(B * H, L + 1, Dh)
    want = torch_attn_func(torch.from_numpy(q.reshape(B * H, 1, Dh)).float(),
                           torch.from_numpy(Kcat).float(), torch.from_numpy(Vcat).float(), 0.125)
    np.testing.assert_allclose(out.reshape(B * H, Dh), want[:, 0].numpy(), atol=2e-6)
    # t = 0 with an empty cache: the output is the new value row
    kc0, vc0 = O.pack_k_cache(K[:, :, :0], 4), O.pack_v_cache(V[:, :, :0], 4)
    np.testing.assert_array_equal(O.decode_step(q, k, v, kc0, vc0, 0.125, 0), v.astype(np.float32))


def test_cpu_baseline_matches_oracle():
    B, H, L, Dh, Lmax = 1, 4, 50, 64, 53
    K, V = _rand(20, B, H, L, Dh), _rand(21, B, H, L, Dh)
    base = CpuDecodeBaseline(torch.from_numpy(K), torch.from_numpy(V), Lmax)
    kc, vc = O.pack_k_cache(K, Lmax), O.pack_v_cache(V, Lmax)
    for i in range(3):
        q, k, v = (_rand(30 + 3 * i + j, B, H, Dh) for j in range(3))
        got = base.attention(torch.from_numpy(q), torch.from_numpy(k), torch.from_numpy(v), 0.125, L + i)
        want = O.decode_step(q, k, v, kc, vc, 0.125, L + i)
        np.testing.assert_allclose(got.numpy(), want, atol=2e-6)


# ------------------------------------------------------------------ fp16 compare
def test_half_from_ushort_known_answers():
    f = O.half_from_ushort_rn
    assert f(np.array([0, 1, 2047, 2048]))[:].tolist() == [0, 1, 2047, 2048]
    # 11 significant bits, ties to even
    assert f(np.array([2049]))[0] == 2048      # tie -> even mantissa
    assert f(np.array([2051]))[0] == 2052      # tie -> even mantissa (2052 = 513*4, 2050 = 1025*2 is odd)
    assert f(np.array([2050]))[0] == 2050
    assert f(np.array([4099]))[0] == 4100
    assert f(np.array([4098]))[0] == 4096      # tie between 4096 and 4100 -> 4096 (even)
    assert f(np.array([65504]))[0] == 65504
    assert f(np.array([65519]))[0] == 65504
    assert np.isinf(f(np.array([65520]))[0]) and np.isinf(f(np.array([65535]))[0])


def test_half_from_ushort_exhaustive_vs_numpy_cast():
    u = np.arange(65536, dtype=np.uint16)
    with np.errstate(over="ignore"):
        want = u.astype(np.float16).astype(np.float64)  # numpy: IEEE RN-even integer -> half
    np.testing.assert_array_equal(O.half_from_ushort_rn(u), want)


def test_leq_f16_bits_semantics():
    # below 2048 the compare is an exact integer compare of the bit patterns
    assert O.leq_f16_bits(np.array([5]), np.array([5]))[0]
    assert not O.leq_f16_bits(np.array([6]), np.array([5]))[0]
    # above, patterns that round to the same 11-bit value compare equal
    assert O.leq_f16_bits(np.array([2049]), np.array([2048]))[0]
    assert not O.leq_f16_bits(np.array([2051]), np.array([2049]))[0]
    # monotone in the bit pattern for all positive finite halves
    u = np.arange(0x3C01, dtype=np.uint16)  # probabilities are <= 1.0 = 0x3C00
    r = O.half_from_ushort_rn(u)
    assert (np.diff(r) >= 0).all()


# ------------------------------------------------------------------ pruning rule
def _pruned_setup(dtype, seed=0, B=2, H=3, L=200, Dh=64, peaked=True):
    rng = np.random.default_rng(seed)
    K = rng.standard_normal((B, H, L, Dh)).astype(dtype)
    V = rng.standard_normal((B, H, L, Dh)).astype(dtype)
    q, k, v = (rng.standard_normal((B, H, Dh)).astype(dtype) for _ in range(3))
    if peaked:
        qd = q.astype(np.float32) / np.linalg.norm(q.astype(np.float32), axis=-1, keepdims=True)
        for b in range(B):
            for h in range(H):
                pos = rng.choice(L, 8, replace=False)
                K[b, h, pos] = (4 * qd[b, h] + 0.1 * rng.standard_normal((8, Dh))).astype(dtype)
    return K, V, q, k, v


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_pruned_invariants(dtype):
    K, V, q, k, v = _pruned_setup(dtype)
    B, H, L, Dh = K.shape
    Lmax = L + 2

    def run(p):
        kc, vc = O.pack_k_cache(K, Lmax), O.pack_v_cache(V, Lmax)
        return O.pruned_decode_step(q, k, v, kc, vc, 1.0, L, p)

    out0, skip0, P0, _ = run(0.0)
    exact = O.decode_step(q, k, v, O.pack_k_cache(K, Lmax), O.pack_v_cache(V, Lmax), 1.0, L)
    # p = 0 drops only probabilities that rounded to exactly zero: result == unpruned
    assert (P0[skip0] == 0).all()
    tol = 2e-3 if dtype == np.float16 else 1e-5  # P_i rounded to T in the rule
    assert np.abs(out0 - exact).max() < tol
    # a threshold below the resolution of T behaves like p = 0
    tiny = 1e-12 if dtype == np.float16 else 1e-44
    out_t, skip_t, _, _ = run(tiny)
    np.testing.assert_array_equal(skip_t, skip0)
    np.testing.assert_array_equal(out_t, out0)
    # monotone in p; the new token (slot L) is never dropped; nothing beyond it is marked
    prev = skip0
    for p in (1e-4, 1e-3, 1e-2, 1e-1, 1.0):
        out, skip, P, thr = run(p)
        assert (skip | ~prev).all(), "skip set must grow with p"
        assert not skip[:, :, L].any() and not skip[:, :, L + 1:].any()
        prev = skip
        # no renormalisation: out == sum over kept of P_i V_i, P_i independent of p
        np.testing.assert_array_equal(P, P0)
        Vall = np.concatenate([V, v[:, :, None]], axis=2).astype(np.float32)
        want = np.einsum("bhn,bhnd->bhd", np.where(skip[:, :, :L + 1], 0, P[:, :, :L + 1]), Vall)
        np.testing.assert_allclose(out, want, atol=1e-5)
    # p = 1: every cached key has P_i <= thr = inv -> only the new token survives
    assert skip[:, :, :L].all()
    np.testing.assert_allclose(out, P[:, :, L:L + 1] * v.astype(np.float32), atol=1e-6)


def test_pruned_fp32_rule_is_e_leq_p():
    """In fp32 the rule reduces to e_i <= p up to rounding of the two products."""
    K, V, q, k, v = _pruned_setup(np.float32, seed=3)
    B, H, L, Dh = K.shape
    kc, vc = O.pack_k_cache(K, L + 1), O.pack_v_cache(V, L + 1)
    p = 3e-2
    _, skip, P, thr = O.pruned_decode_step(q, k, v, kc, vc, 1.0, L, p)
    Kall = np.concatenate([K, k[:, :, None]], axis=2).astype(np.float64)
    s = np.einsum("bhd,bhnd->bhn", q.astype(np.float64), Kall)
    e = np.exp(s - s.max(axis=-1, keepdims=True))
    clear = np.abs(e[:, :, :L] - p) > 1e-5 * p          # away from the boundary
    np.testing.assert_array_equal(skip[:, :, :L][clear], (e[:, :, :L] <= p)[clear])
    assert 0.05 < skip[:, :, :L].mean() < 0.999


def test_pruned_fp16_threshold_in_subnormal_range_is_integer_compare():
    """With a flat score distribution over many keys the fp16 probabilities are below 2^-13,
    i.e. integer multiples n_i of 2^-24, and so is the threshold (m * 2^-24).  The bit
    pattern of a half below 2^-13 IS that integer, all below 2048, so the reference's
    compare must reduce to n_i <= m computed in value space (float64, no bit tricks)."""
    B, H, L, Dh = 1, 1, 20000, 64
    rng = np.random.default_rng(5)
    K = (0.05 * rng.standard_normal((B, H, L, Dh))).astype(np.float16)
    V = rng.standard_normal((B, H, L, Dh)).astype(np.float16)
    q, k, v = (rng.standard_normal((B, H, Dh)).astype(np.float16) for _ in range(3))
    kc, vc = O.pack_k_cache(K, L + 1), O.pack_v_cache(V, L + 1)
    p = 0.8
    _, skip, P, thr = O.pruned_decode_step(q, k, v, kc, vc, 0.125, L, p)
    Kall = np.concatenate([K, k[:, :, None]], axis=2).astype(np.float64)[0, 0]
    s = Kall @ q[0, 0].astype(np.float64) * 0.125
    e = np.exp(s - s.max())
    inv = 1.0 / (e.sum() + 1e-6)
    n_exact = e[:L] * inv * 2.0 ** 24
    m_exact = p * inv * 2.0 ** 24
    assert m_exact < 2047 and n_exact.max() < 2047          # all below 2^-13
    # keep away from rounding ties and from fp32-vs-fp64 noise in e_i
    frac = np.abs(n_exact - np.floor(n_exact) - 0.5)
    clear = (frac > 1e-3) & (abs(m_exact - math.floor(m_exact) - 0.5) > 1e-3)
    want = np.rint(n_exact) <= np.rint(m_exact)
    np.testing.assert_array_equal(skip[0, 0, :L][clear], want[clear])
    assert clear.mean() > 0.99
    assert 0.02 * L < skip.sum() < 0.98 * L


# --------------------------------------------------------------------------- bf16, bias, rotary embedding
def test_bf16_conversion_matches_torch_cast():
    """f32_to_bf16_bits against torch's own float32 -> bfloat16 cast (an independent
    implementation): random values over the whole exponent range, exact ties (round to even),
    denormals, infinities; NaN stays NaN.  bf16 -> f32 is exact."""
    rng = np.random.default_rng(0)
    x = np.concatenate([
        rng.standard_normal(200000).astype(np.float32),
        (rng.standard_normal(50000) * 10.0 ** rng.uniform(-40, 38, 50000)).astype(np.float32),
        np.array([0.0, -0.0, 1.0, np.inf, -np.inf, 3.4e38, 1e-45, 1.17549435e-38], np.float32),
        # ties: mantissa bits 0x8000 below an even / odd kept part
        np.array([0x3F808000, 0x3F818000, 0x3F80FFFF, 0x3F810001, 0x7F7F8000, 0x00008000, 0x00018000],
                 np.uint32).view(np.float32),
    ])
    got = O.f32_to_bf16_bits(x)
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    np.testing.assert_array_equal(got, want)
    assert got[np.flatnonzero(x.view(np.uint32) == 0x3F808000)[0]] == 0x3F80      # tie -> even (down)
    assert got[np.flatnonzero(x.view(np.uint32) == 0x3F818000)[0]] == 0x3F82      # tie -> even (up)
    assert np.isnan(O.bf16_bits_to_f32(O.f32_to_bf16_bits(np.array([np.nan], np.float32))))[0]
    np.testing.assert_array_equal(O.bf16_bits_to_f32(got).view(np.uint32), got.astype(np.uint32) << 16)
    np.testing.assert_array_equal(O.round_to(x[:1000], "f16"), x[:1000].astype(np.float16).astype(np.float32))


def test_rotary_matches_transformers_gptj():
    """token_transform's rotary embedding against the installed transformers' GPT-J functions on
    fp32 tensors: same element pairs (2i, 2i+1), same signs, same angles pos / 10000^(2i/d),
    elements beyond rotary_dim untouched."""
    gptj = pytest.importorskip("transformers.models.gptj.modeling_gptj")
    rng = np.random.default_rng(1)
    for Dh, rd in [(64, 32), (256, 64), (64, 64), (128, 2)]:
        B, H = 3, 2
        q, k, v = (rng.standard_normal((B, H, Dh)).astype(np.float32) for _ in range(3))
        emb = gptj.create_sinusoidal_positions(2048, rd)
        # The reference divides pos by base^(2i/d), transformers multiplies by the reciprocal: the
        # fp32 angles differ by an ulp or two, i.e. by up to 1.2e-4 rad at position 1500 and by
        # 4e-6 rad below position 40; the rotated values differ by that times |x| (<= 4.5 here).
        for pos, tol in ((np.array([0, 7, 39]), 2e-5), (np.array([0, 640, 1500]), 6e-4)):
            sin, cos = torch.split(emb[torch.from_numpy(pos)][:, None, :], rd // 2, dim=-1)
            def ref(x):
                x = torch.from_numpy(x)[:, None]                               # [B, 1, H, Dh]
                return torch.cat([gptj.apply_rotary_pos_emb(x[..., :rd], sin, cos), x[..., rd:]], -1)[:, 0].numpy()
            gq, gk, gv = O.token_transform(q, k, v, "f32", rotary_dim=rd, pos=pos)
            assert np.abs(gq - ref(q)).max() <= tol and np.abs(gk - ref(k)).max() <= tol
        np.testing.assert_array_equal(gv, v)
        np.testing.assert_array_equal(gq[..., rd:], q[..., rd:])
        np.testing.assert_array_equal(gq[0], q[0])                          # position 0: identity


def test_token_transform_invariants():
    """Rotations keep the norm of every pair, compose additively in the position, and the bias is a
    plain addition made before the rotation; results are values of the element type."""
    rng = np.random.default_rng(2)
    B, H, Dh, rd = 2, 3, 64, 48
    q, k, v = (rng.standard_normal((B, H, Dh)).astype(np.float32) for _ in range(3))
    qb, kb, vb = (rng.standard_normal((H, Dh)).astype(np.float32) for _ in range(3))
    pos = np.array([3, 41])
    gq, gk, gv = O.token_transform(q, k, v, "f32", qb, kb, vb, rd, pos)
    np.testing.assert_allclose(gv, v + vb[None], rtol=0, atol=1e-7)
    pn = lambda a: a[..., 0:rd:2] ** 2 + a[..., 1:rd:2] ** 2
    np.testing.assert_allclose(pn(gq), pn(q + qb[None]), rtol=2e-6)
    np.testing.assert_allclose(pn(gk), pn(k + kb[None]), rtol=2e-6)
    np.testing.assert_array_equal(gk[..., rd:], (k + kb[None])[..., rd:])
    # rotating by pos1 then pos2 (no bias) = rotating by pos1 + pos2, up to the fp32 angle rounding
    a1, _, _ = O.token_transform(q, k, v, "f32", rotary_dim=rd, pos=np.array([3, 5]))
    a2, _, _ = O.token_transform(a1, k, v, "f32", rotary_dim=rd, pos=np.array([4, 6]))
    a3, _, _ = O.token_transform(q, k, v, "f32", rotary_dim=rd, pos=np.array([7, 11]))
    np.testing.assert_allclose(a2, a3, atol=5e-6)
    # known answer: pair (1, 0) at pair index 0 (angle = pos) becomes (cos pos, sin pos)
    e = np.zeros((1, 1, 8), np.float32)
    e[0, 0, 0] = 1
    r, _, _ = O.token_transform(e, e, e, "f32", rotary_dim=8, pos=np.array([2]))
    np.testing.assert_allclose(r[0, 0, :2], [np.cos(2.0), np.sin(2.0)], atol=1e-7)
    for elem in ("f16", "bf16"):
        h, _, _ = O.token_transform(q, k, v, elem, qb, kb, vb, rd, pos)
        np.testing.assert_array_equal(h, O.round_to(h, elem))
        assert np.abs(h - gq).max() <= (2 ** -10 if elem == "f16" else 2 ** -7) * np.abs(gq).max()
    np.testing.assert_array_equal(O.rotary_positions(3, 50), [50, 50, 50])
    np.testing.assert_array_equal(O.rotary_positions(3, 50, [10, 50, 0], True), [10, 50, 0])
    np.testing.assert_array_equal(O.rotary_positions(3, 50, [10, 50, 60], False), [40, 0, 0])


# ------------------------------------------------------------------ beam-search indirection
def _beam_problem(seed, groups, bw, H, Dh, L, Lmax, dtype=np.float32):
    rng = np.random.default_rng(seed)
    B = groups * bw
    K = rng.standard_normal((B, H, L, Dh)).astype(dtype)
    V = rng.standard_normal((B, H, L, Dh)).astype(dtype)
    return rng, B, O.pack_k_cache(K, Lmax), O.pack_v_cache(V, Lmax)


def test_beam_identity_table_is_the_plain_step():
    groups, bw, H, Dh, L, Lmax = 2, 3, 2, 16, 21, 24
    rng, B, kc, vc = _beam_problem(70, groups, bw, H, Dh, L, Lmax)
    q, k, v = (rng.standard_normal((B, H, Dh)).astype(np.float32) for _ in range(3))
    own = np.repeat((np.arange(B) % bw)[:, None], Lmax, 1).astype(np.int32)
    kc1, vc1, kc2, vc2 = kc.copy(), vc.copy(), kc.copy(), vc.copy()
    plain = O.decode_step(q, k, v, kc1, vc1, 0.25, L)
    beam = O.decode_step(q, k, v, kc2, vc2, 0.25, L, cache_indir=own, beam_width=bw)
    assert np.array_equal(plain, beam) and np.array_equal(kc1, kc2) and np.array_equal(vc1, vc2)
    a = O.pruned_decode_step(q, k, v, kc.copy(), vc.copy(), 0.25, L, 1e-2)
    b = O.pruned_decode_step(q, k, v, kc.copy(), vc.copy(), 0.25, L, 1e-2, cache_indir=own, beam_width=bw)
    assert all(np.array_equal(x, y) for x, y in zip(a, b))


def test_beam_table_reads_follow_the_reference_offsets():
    """Element by element with the reference's flat offsets (attention.cu:1003, :1027-1031 for
    K, :1143, :1197-1201 for V): base = group's first beam, plus beam_src whole samples."""
    groups, bw, H, Dh, L, Lmax = 2, 2, 2, 8, 5, 7
    rng, B, kc, vc = _beam_problem(71, groups, bw, H, Dh, L, Lmax)
    x = O.elems_per_16b(np.float32)
    indir = rng.integers(0, bw, (B, Lmax)).astype(np.int32)
    kflat, vflat = kc.reshape(-1), vc.reshape(-1)
    for b in range(B):
        beami, bbi = b % bw, b // bw
        Kb, Vb = O.beam_keys_values(kc, vc, b, L + 1, indir, bw)
        for h in range(H):
            bbhi = bbi * bw * H + h
            for ti in range(L):                       # cached keys only: slot L is the new token
                beam_src = indir.reshape(-1)[(bbi * bw + beami) * Lmax + ti]
                beam_offset = beam_src * H * Lmax * Dh
                for d in range(Dh):
                    ko = bbhi * Lmax * Dh + beam_offset + (d // x) * Lmax * x + ti * x + d % x
                    vo = bbhi * Lmax * Dh + beam_offset + ti * Dh + d
                    assert Kb[h, ti, d] == kflat[ko] and Vb[h, ti, d] == vflat[vo]
            # the new token's slot is the sample's own
            assert np.array_equal(Kb[h, L], O.unpack_k_cache(kc[b:b + 1], L + 1)[0, h, L])
            assert np.array_equal(Vb[h, L], vc[b, h, L])


@pytest.mark.parametrize("p", [0.0, 2e-2])
def test_beam_search_by_table_equals_beam_search_by_cache_copy(p):
    """A toy beam search, two ways.  By copy: after every step the caches of each group are
    re-gathered by the chosen parents, as the reference's models do
    (_reorder_cache = index_select on the batch axis, modeling_opt.py:1072-1075), and the step
    reads a sample's own caches.  By table: caches stay where they were written; the table row
    of a beam becomes its parent's row, and the token a beam has just written is its own.
    Outputs must agree bit for bit at every step."""
    groups, bw, H, Dh, L, steps = 2, 3, 2, 16, 9, 7
    Lmax = L + steps
    rng, B, kc, vc = _beam_problem(72, groups, bw, H, Dh, L, Lmax)
    kc_copy, vc_copy = kc.copy(), vc.copy()
    table = np.repeat((np.arange(B) % bw)[:, None], Lmax, 1).astype(np.int32)
    for s in range(steps):
        t = L + s
        q, k, v = (rng.standard_normal((B, H, Dh)).astype(np.float32) for _ in range(3))
        if p == 0.0:
            by_copy = O.decode_step(q, k, v, kc_copy, vc_copy, 0.25, t)
            by_table = O.decode_step(q, k, v, kc, vc, 0.25, t, cache_indir=table, beam_width=bw)
        else:
            by_copy = O.pruned_decode_step(q, k, v, kc_copy, vc_copy, 0.25, t, p)[0]
            by_table = O.pruned_decode_step(q, k, v, kc, vc, 0.25, t, p, cache_indir=table, beam_width=bw)[0]
        assert np.array_equal(by_copy, by_table), s
        # every beam picks a parent inside its group
        parent = (np.arange(B) // bw) * bw + rng.integers(0, bw, B)
        kc_copy, vc_copy = kc_copy[parent].copy(), vc_copy[parent].copy()
        new_table = table[parent].copy()
        new_table[:, t] = parent % bw                 # slot t was written by the parent itself
        table = new_table
    assert len(np.unique(table[:, :Lmax - 1], axis=0)) > groups   # the search did mix beams
