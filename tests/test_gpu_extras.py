"""GPU parity of ffa_attention_ex: the bf16 element type, the new-token transform (q/k/v bias,
rotary embedding) and the beam-search cache indirection, through the C ABI, against the CPU oracle.

Tolerances.  fp16 / fp32 outputs: 1e-3 / 1e-6 max-abs against the float64 closed form, as in the
other parity tests.  bf16 outputs: one bf16 ulp of the closed form (|err| <= 2^-7 |want| + 1e-5;
the kernel accumulates in fp32 and rounds once, so the error is a single rounding, at most half
an ulp, plus the rare value that sits on a rounding boundary).  The transformed k and v that land
in the caches: the oracle's values (both sides evaluate the rotation in fp64), at most one ulp
apart on fewer than 1 % of the elements; bit for bit when only a bias is added."""
import ctypes as C

import numpy as np
import pytest
import torch

from fastforwardattention_amd import capi
from oracle import ffa_oracle as O
from tests.ffa_testlib import ptr
from tests.test_gpu_parity import _plans

pytestmark = pytest.mark.gpu

ELEMS = {"f16": (capi.FFA_PRECISION_F16, torch.float16), "bf16": (capi.FFA_PRECISION_BF16, torch.bfloat16),
         "f32": (capi.FFA_PRECISION_F32, torch.float32)}


def _say(*a):
    print(*a, flush=True)


def _to_dev(x, elem):
    """fp32 numpy values (already representable in `elem`) -> device tensor of that type."""
    return torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).to("cuda:0").to(ELEMS[elem][1])


def _bits(t):
    """Device tensor -> numpy array of its raw element bits."""
    if t.dtype == torch.float32:
        return t.cpu().numpy().view(np.uint32)
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


class ExSession:
    """Caches + workspace for one problem in any of the three element types, driven through
    ffa_init_cache_* and ffa_attention_ex.  K, V: fp32 numpy arrays of representable values."""

    def __init__(self, K, V, max_len, elem):
        self.lib = capi.load()
        self.elem, (self.precision, tdt) = elem, ELEMS[elem]
        B, H, L, Dh = K.shape
        self.B, self.H, self.L, self.Dh, self.Lmax = B, H, L, Dh, max_len
        x = 4 if elem == "f32" else 8
        self.k_cache = torch.zeros(B, H, Dh // x, max_len, x, dtype=tdt, device="cuda:0")
        self.v_cache = torch.zeros(B, H, max_len, Dh, dtype=tdt, device="cuda:0")
        Kd, Vd = _to_dev(K, elem), _to_dev(V, elem)
        init = self.lib.ffa_init_cache_f32 if elem == "f32" else self.lib.ffa_init_cache_f16   # 16-byte moves
        capi.check(init(ptr(self.k_cache), ptr(self.v_cache), ptr(Kd), ptr(Vd), B, L, max_len, Dh, H, None),
                   "ffa_init_cache")
        n = self.lib.ffa_workspace_bytes(B, H, Dh, max_len)
        self.ws = torch.empty(n, dtype=torch.uint8, device="cuda:0")
        capi.check(self.lib.ffa_workspace_init(ptr(self.ws), n, None), "ffa_workspace_init")
        torch.cuda.synchronize()

    def step(self, q, k, v, scale, t, p=0.0, plan=None, seq_lengths=None, rnp=True, transform=None,
             beams=None, expect=capi.FFA_OK):
        qd, kd, vd = (_to_dev(a, self.elem) for a in (q, k, v))
        out = torch.full((self.B, self.H, self.Dh), float("nan"), dtype=ELEMS[self.elem][1], device="cuda:0")
        sl = None if seq_lengths is None else torch.from_numpy(np.asarray(seq_lengths, np.int32)).to("cuda:0")
        tt, keep = None, []
        if transform is not None:
            tt = capi.TokenTransform()
            for name in ("q_bias", "k_bias", "v_bias"):
                b = transform.get(name)
                if b is not None:
                    keep.append(_to_dev(b, self.elem))
                    setattr(tt, name, keep[-1].data_ptr())
            tt.rotary_embedding_dim = transform.get("rotary_dim", 0)
            tt.rotary_base = transform.get("base", 0.0)
        bi = None
        if beams is not None:                      # (table [B, Lmax] or None, beam_width)
            table, bw = beams
            if table is not None:
                keep.append(torch.from_numpy(np.ascontiguousarray(table, np.int32)).to("cuda:0"))
            bi = capi.BeamIndirection(keep[-1].data_ptr() if table is not None else None, bw)
        rc = self.lib.ffa_attention_ex(self.precision, self.B, self.H, self.Dh, self.Lmax, float(scale), int(t),
                                       ptr(qd), ptr(kd), ptr(vd), ptr(self.k_cache), ptr(self.v_cache), ptr(out),
                                       ptr(sl), float(p), C.byref(plan) if plan is not None else None, int(rnp),
                                       C.byref(tt) if tt is not None else None,
                                       C.byref(bi) if bi is not None else None, ptr(self.ws), self.ws.numel(), None)
        assert rc == expect, capi.STATUS_NAMES.get(rc, rc)
        torch.cuda.synchronize()
        return None if rc != capi.FFA_OK else out.float().cpu().numpy()


def _inputs(seed, B, H, L, Dh, elem, kv_scale=1.0):
    rng = np.random.default_rng(seed)
    r = lambda *s: O.round_to(rng.standard_normal(s) * kv_scale, elem)
    return rng, r(B, H, L, Dh), r(B, H, L, Dh), r(B, H, Dh), r(B, H, Dh), r(B, H, Dh)


def _pack(K, V, Lmax, elem):
    """(k_cache, v_cache) as fp32 value arrays in the 8- or 4-element chunk layout of `elem`."""
    dt = np.float32 if elem == "f32" else np.float16          # only the chunk width matters here
    x = 16 // np.dtype(dt).itemsize
    B, H, L, Dh = K.shape
    kc = np.zeros((B, H, Dh // x, Lmax, x), np.float32)
    kc[:, :, :, :L, :] = K.reshape(B, H, L, Dh // x, x).transpose(0, 1, 3, 2, 4)
    vc = np.zeros((B, H, Lmax, Dh), np.float32)
    vc[:, :, :L] = V
    return kc, vc


def _ulp(x, elem):
    """One ulp of `elem` at |x| (fp32 arrays)."""
    bits = {"f16": 10, "bf16": 7, "f32": 23}[elem]
    tiny = {"f16": 2.0 ** -14, "bf16": 2.0 ** -126, "f32": 2.0 ** -126}[elem]
    return 2.0 ** (np.floor(np.log2(np.maximum(np.abs(x), tiny))) - bits)


def _out_tol(want, elem):
    return {"f16": 1e-3, "f32": 1e-6}.get(elem, None) or (2.0 ** -7 * np.abs(want) + 1e-5)


# ------------------------------------------------------------------ bf16, exact
@pytest.mark.parametrize("Dh", [64, 80, 128, 256])
@pytest.mark.parametrize("t", [0, 65, 777])
def test_bf16_exact_step_all_plans(Dh, t):
    B, H, elem = 2, 3, "bf16"
    Lmax = t + 3
    _, K, V, q, k, v = _inputs(5000 + Dh + t, B, H, t, Dh, elem)
    scale = 1.0 / np.sqrt(Dh)
    kc0, vc0 = _pack(K, V, Lmax, elem)
    want = O.decode_step(q, k, v, kc0, vc0, scale, t, acc=np.float64)
    for name, plan in _plans(16, B, H, Dh, t):
        _say("bf16 exact", Dh, t, name)
        sess = ExSession(K, V, Lmax, elem)
        got = sess.step(q, k, v, scale, t, plan=plan)
        assert (np.abs(got - want) <= _out_tol(want, elem)).all(), (name, float(np.abs(got - want).max()))
        np.testing.assert_array_equal(_bits(sess.k_cache), O.f32_to_bf16_bits(kc0), err_msg=name)
        np.testing.assert_array_equal(_bits(sess.v_cache), O.f32_to_bf16_bits(vc0), err_msg=name)


def test_bf16_iterative_decode_and_padding():
    """OPT-1.3b shape in miniature with bf16 caches: 12 appended tokens with the library's own plan,
    then a left-padded and a right-padded step."""
    B, H, Dh, L, steps, elem = 2, 32, 64, 1000, 12, "bf16"
    rng, K, V, *_ = _inputs(77, B, H, L, Dh, elem, kv_scale=0.5)
    sess = ExSession(K, V, L + steps, elem)
    kc, vc = _pack(K, V, L + steps, elem)
    for i in range(steps):
        q, k, v = (O.round_to(rng.standard_normal((B, H, Dh)), elem) for _ in range(3))
        got = sess.step(q, k, v, 0.125, L + i)
        want = O.decode_step(q, k, v, kc, vc, 0.125, L + i, acc=np.float64)
        assert (np.abs(got - want) <= _out_tol(want, elem)).all(), i
    np.testing.assert_array_equal(_bits(sess.k_cache), O.f32_to_bf16_bits(kc))
    np.testing.assert_array_equal(_bits(sess.v_cache), O.f32_to_bf16_bits(vc))
    t = L + steps - 1
    for sl, rnp in (([0, 400], False), ([t, 500], True)):
        q, k, v = (O.round_to(rng.standard_normal((B, H, Dh)), elem) for _ in range(3))
        got = sess.step(q, k, v, 0.125, t, seq_lengths=sl, rnp=rnp)
        want = O.decode_step(q, k, v, kc, vc, 0.125, t, seq_lengths=np.array(sl), right_or_no_padding=rnp,
                             acc=np.float64)
        assert (np.abs(got - want) <= _out_tol(want, elem)).all(), (sl, rnp)


@pytest.mark.parametrize("p", [1e-3, 1e-2])
def test_bf16_pruned_step_matches_rule(p):
    """Pruning with bf16 probabilities: the fp32 rule with T = bf16 rounding (the reference has no
    bf16 behaviour of its own).  Skip decisions may differ only where the probability is within
    one bf16 ulp of the threshold; the output equals the rule's for the GPU's own skip set."""
    B, H, Dh, L, elem = 2, 3, 64, 900, "bf16"
    rng, K, V, q, k, v = _inputs(31, B, H, L, Dh, elem)
    qd = q / np.linalg.norm(q, axis=-1, keepdims=True)
    for b in range(B):
        for h in range(H):
            pos = rng.choice(L, 16, replace=False)
            K[b, h, pos] = O.round_to(4 * qd[b, h] + 0.1 * rng.standard_normal((16, Dh)), elem)
    Lmax, scale = L + 1, 0.125
    kc0, vc0 = _pack(K, V, Lmax, elem)
    want, skip, P, thr = O.pruned_decode_step(q, k, v, kc0.copy(), vc0.copy(), scale, L, p, elem="bf16")
    ntiles = L // 64 + 1
    Vall = np.concatenate([V, v[:, :, None]], axis=2)
    for plan in (capi.make_plan(capi.FFA_LAUNCH_WORKGROUP, 4, 1, ntiles), capi.make_plan(capi.FFA_LAUNCH_WORKGROUP, 16, 1, ntiles),
                 capi.make_plan(capi.FFA_LAUNCH_TWO_PASS, 4, -(-ntiles // 2), 2), None):
        _say("bf16 pruned", p, plan)
        sess = ExSession(K, V, Lmax, elem)
        kept = torch.zeros(B, H, dtype=torch.int32, device="cuda:0")
        mask = torch.zeros(B, H, Lmax, dtype=torch.uint8, device="cuda:0")
        out = torch.zeros(B, H, Dh, dtype=torch.bfloat16, device="cuda:0")
        qd_, kd_, vd_ = (_to_dev(a, elem) for a in (q, k, v))
        rc = sess.lib.ffa_attention_diag(sess.precision, B, H, Dh, Lmax, scale, L, ptr(qd_), ptr(kd_), ptr(vd_),
                                         ptr(sess.k_cache), ptr(sess.v_cache), ptr(out), None, p,
                                         C.byref(plan) if plan is not None else None, 1, ptr(sess.ws), sess.ws.numel(),
                                         ptr(kept), ptr(mask), None)
        assert rc == capi.FFA_OK, capi.STATUS_NAMES.get(rc, rc)
        torch.cuda.synchronize()
        gmask = mask.cpu().numpy().astype(bool)
        near = np.abs(P - thr[:, :, None]) <= 2.0 ** -6 * np.abs(thr[:, :, None])
        assert not ((gmask != skip) & ~near).any()
        np.testing.assert_array_equal(kept.cpu().numpy(), L - gmask[:, :, :L].sum(-1))
        w = np.where(gmask[:, :, :L + 1], 0, P[:, :, :L + 1])
        want_g = np.einsum("bhn,bhnd->bhd", w, Vall)
        got = out.float().cpu().numpy()
        assert (np.abs(got - want_g) <= 2.0 ** -6 * np.abs(want_g) + 2e-3).all()
    assert skip[:, :, :L].mean() > 0.01 if p >= 1e-2 else True


# ------------------------------------------------------------------ bias and rotary embedding
def _check_transform(elem, B, H, Dh, L, rd, bias, padding, seed, plan=None):
    rng, K, V, q, k, v = _inputs(seed, B, H, L, Dh, elem)
    biases = {n: O.round_to(rng.standard_normal((H, Dh)), elem) for n in ("q_bias", "k_bias", "v_bias")} if bias else {}
    sl, rnp = None, True
    if padding == "left":
        sl, rnp = rng.integers(0, L // 2, B), False
    elif padding == "right":
        sl, rnp = rng.integers(L // 2, L + 1, B), True
    Lmax, scale = L + 2, 1.0 / np.sqrt(Dh)
    pos = O.rotary_positions(B, L, sl, rnp)
    q2, k2, v2 = O.token_transform(q, k, v, elem, biases.get("q_bias"), biases.get("k_bias"), biases.get("v_bias"), rd, pos)
    kc, vc = _pack(K, V, Lmax, elem)
    want = O.decode_step(q2, k2, v2, kc, vc, scale, L, seq_lengths=sl, right_or_no_padding=rnp, acc=np.float64)
    sess = ExSession(K, V, Lmax, elem)
    got = sess.step(q, k, v, scale, L, plan=plan, seq_lengths=sl, rnp=rnp, transform=dict(biases, rotary_dim=rd))
    # a q' or k' element on a rounding boundary may come out one ulp apart: a little slack for the scores
    slack = {"f16": 3e-4, "bf16": 0.0, "f32": 1e-6}[elem] if rd else 0.0
    tol = _out_tol(want, elem) * (2 if elem == "bf16" and rd else 1) + slack
    assert (np.abs(got - want) <= tol).all(), float(np.abs(got - want).max())
    # the caches received the transformed k, v at the slot of each sample
    gk = sess.k_cache.float().cpu().numpy()
    gv = sess.v_cache.float().cpu().numpy()
    slot = np.full(B, L) if (sl is None or not rnp) else np.asarray(sl)
    for b in range(B):
        gkb = gk[b, :, :, slot[b], :].reshape(H, Dh)
        if rd:
            # both sides evaluate in fp64: equal except where the value sits on a rounding boundary
            assert (np.abs(gkb - k2[b]) <= _ulp(k2[b], elem) * 1.01).all()
            assert (gkb != k2[b]).mean() < 0.01
            assert (gkb[:, rd:] == k2[b][:, rd:]).all()
        else:
            np.testing.assert_array_equal(gkb, k2[b])
        np.testing.assert_array_equal(gv[b, :, slot[b]], v2[b])
        np.testing.assert_array_equal(gk[b, :, :, :slot[b]], kc[b, :, :, :slot[b]])     # history untouched
    return got


@pytest.mark.parametrize("elem", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("Dh,rd", [(64, 32), (256, 64), (128, 128), (80, 16)])
@pytest.mark.parametrize("padding", ["none", "left", "right"])
def test_rotary_and_bias(elem, Dh, rd, padding):
    _say("rotary+bias", elem, Dh, rd, padding)
    _check_transform(elem, 3, 4, Dh, 300, rd, True, padding, 900 + Dh + rd)
    _check_transform(elem, 2, 2, Dh, 130, rd, False, padding, 901 + Dh + rd)


@pytest.mark.parametrize("padding", ["none", "left"])
def test_rotary_at_the_gptj_baseline_shape(padding):
    """BASELINE configs[3] (B = 8, 16 heads x 256, fp16) at 2000 cached keys with GPT-J's rotary
    embedding over 64 dims, the library's own plan (four lanes per key, every pair cut in two)."""
    _say("rotary at the gpt-j shape", padding)
    plan = capi.plan_launch(16, 8, 16, 256, 2000)
    assert plan.kind == capi.FFA_LAUNCH_SPLIT and plan.threads_per_key == 4 and plan.n_splits > 1
    _check_transform("f16", 8, 16, 256, 2000, 64, False, padding, 2024)


@pytest.mark.parametrize("elem", ["f16", "bf16", "f32"])
def test_rotary_and_bias_at_the_headline_shape(elem):
    """BASELINE configs[1] at B = 10 (320 pairs of 64) at 1100 cached keys: the hybrid launch, 256 whole
    pairs and 64 split ones, every workgroup with a wave that publishes the angles."""
    _say("rotary+bias at the headline shape", elem)
    plan = capi.plan_launch(32 if elem == "f32" else 16, 10, 32, 64, 1100)
    assert plan.kind == capi.FFA_LAUNCH_SPLIT and plan.whole_heads == 256 and plan.n_splits > 1
    _check_transform(elem, 10, 32, 64, 1100, 32, True, "right", 2025)


@pytest.mark.parametrize("elem", ["f16", "f32"])
def test_transform_in_the_one_workgroup_kernel_at_its_lds_ceiling(elem):
    """35839 keys through a 16-wave one-workgroup plan: 140 KiB of dynamic LDS for the scores beside
    the kernel's static LDS, in which the angles of the transform share their place with the
    survivor queues.  Widest head, so that the static part is at its largest."""
    L, Dh = 35839, 256
    plan = capi.make_plan(capi.FFA_LAUNCH_WORKGROUP, 16, 1, L // 64 + 1)
    _say("transform at the lds ceiling", elem)
    _check_transform(elem, 1, 2, Dh, L, 64, True, "none", 77, plan=plan)


@pytest.mark.parametrize("elem", ["f16", "f32"])
def test_bias_only_is_exact_and_every_plan_takes_the_transform(elem):
    B, H, Dh, L = 2, 3, 64, 333
    prec = 16 if elem == "f16" else 32
    for name, plan in _plans(prec, B, H, Dh, L)[:12]:
        _say("bias only", elem, name)
        _check_transform(elem, B, H, Dh, L, 0, True, "none", 5, plan=plan)
        _check_transform(elem, B, H, Dh, L, 32, True, "left", 6, plan=plan)


def test_rotary_matches_transformers_gptj_end_to_end():
    """One GPT-J-shaped step (16 heads x 256, rotary_dim 64) in fp32: q, k rotated by the installed
    transformers' own apply_rotary_pos_emb, attention in fp64 torch -- against the fused call."""
    gptj = pytest.importorskip("transformers.models.gptj.modeling_gptj")
    B, H, Dh, L, rd = 2, 16, 256, 200, 64
    _, K, V, q, k, v = _inputs(11, B, H, L, Dh, "f32")
    emb = gptj.create_sinusoidal_positions(512, rd)
    sin, cos = torch.split(emb[torch.full((B,), L)][:, None, :], rd // 2, dim=-1)
    rot = lambda x: torch.cat([gptj.apply_rotary_pos_emb(torch.from_numpy(x)[:, None][..., :rd], sin, cos),
                               torch.from_numpy(x)[:, None][..., rd:]], -1)[:, 0]
    q2, k2 = rot(q).double(), rot(k).double()
    Kall = torch.cat([torch.from_numpy(K).double(), k2[:, :, None]], 2)
    Vall = torch.cat([torch.from_numpy(V).double(), torch.from_numpy(v).double()[:, :, None]], 2)
    w = torch.softmax(torch.einsum("bhd,bhnd->bhn", q2, Kall) / 16.0, -1)
    want = torch.einsum("bhn,bhnd->bhd", w, Vall).numpy()
    got = ExSession(K, V, L + 1, "f32").step(q, k, v, 1 / 16.0, L, transform=dict(rotary_dim=rd))
    assert np.abs(got - want).max() <= 1e-4      # transformers' fp32 angle at position 200 is good to 2e-5 rad


def test_transform_argument_validation():
    B, H, Dh, L = 1, 2, 64, 20
    _, K, V, q, k, v = _inputs(3, B, H, L, Dh, "f16")
    sess = ExSession(K, V, L + 1, "f16")
    for rd in (-2, 3, 66):
        sess.step(q, k, v, 0.125, L, transform=dict(rotary_dim=rd), expect=capi.FFA_ERR_TRANSFORM)
    x = _to_dev(q, "f16")
    rc = sess.lib.ffa_attention_ex(12, B, H, Dh, L + 1, 0.125, L, ptr(x), ptr(x), ptr(x), ptr(sess.k_cache),
                                   ptr(sess.v_cache), ptr(x), None, 0.0, None, 1, None, None, ptr(sess.ws), sess.ws.numel(),
                                   None)
    assert rc == capi.FFA_ERR_DTYPE


# ------------------------------------------------------------------ beam-search cache indirection
def _cache_values(sess):
    """The session's caches as fp32 value arrays (k in chunk layout, v)."""
    return sess.k_cache.float().cpu().numpy(), sess.v_cache.float().cpu().numpy()


@pytest.mark.parametrize("elem,Dh", [("f16", 64), ("f16", 80), ("f16", 256), ("f32", 64), ("f32", 128), ("bf16", 128)])
@pytest.mark.parametrize("t", [0, 63, 500])
def test_beam_indirection_exact_step_all_plans(elem, Dh, t):
    """A random table (every key of every beam from a random sibling), every plan kind.  The
    output follows the table; the new token lands in the sample's own caches, nothing else
    in the caches changes."""
    groups, bw, H = 2, 3, 2
    B, Lmax = groups * bw, t + 3
    rng, K, V, q, k, v = _inputs(9000 + Dh + t, B, H, t, Dh, elem)
    scale = 1.0 / np.sqrt(Dh)
    table = rng.integers(0, bw, (B, Lmax)).astype(np.int32)
    kc0, vc0 = _pack(K, V, Lmax, elem)
    want = O.decode_step(q, k, v, kc0, vc0, scale, t, acc=np.float64, cache_indir=table, beam_width=bw)
    if t > 0:
        plain = O.decode_step(q, k, v, *_pack(K, V, Lmax, elem), scale, t, acc=np.float64)
        assert np.abs(want - plain).max() > 1e-2          # the table matters
    prec = 16 if elem != "f32" else 32
    for name, plan in _plans(prec, B, H, Dh, t) + [("library", None)]:
        _say("beams", elem, Dh, t, name)
        sess = ExSession(K, V, Lmax, elem)
        got = sess.step(q, k, v, scale, t, plan=plan, beams=(table, bw))
        assert (np.abs(got - want) <= _out_tol(want, elem)).all(), (name, float(np.abs(got - want).max()))
        kc, vc = _cache_values(sess)
        np.testing.assert_array_equal(kc, kc0, err_msg=name)
        np.testing.assert_array_equal(vc, vc0, err_msg=name)


@pytest.mark.parametrize("padding", ["left", "right"])
def test_beam_indirection_with_padding(padding):
    groups, bw, H, Dh, L, elem = 3, 2, 4, 64, 300, "f16"
    B, Lmax = groups * bw, L + 2
    rng, K, V, q, k, v = _inputs(9100, B, H, L, Dh, elem)
    table = rng.integers(0, bw, (B, Lmax)).astype(np.int32)
    if padding == "left":
        sl, rnp = rng.integers(0, L // 2, B), False
    else:
        sl, rnp = np.repeat(rng.integers(L // 2, L + 1, groups), bw), True   # one length per group
    kc0, vc0 = _pack(K, V, Lmax, elem)
    want = O.decode_step(q, k, v, kc0, vc0, 0.125, L, seq_lengths=sl, right_or_no_padding=rnp, acc=np.float64,
                         cache_indir=table, beam_width=bw)
    for name, plan in _plans(16, B, H, Dh, L) + [("library", None)]:
        _say("beams padding", padding, name)
        sess = ExSession(K, V, Lmax, elem)
        got = sess.step(q, k, v, 0.125, L, plan=plan, seq_lengths=sl, rnp=rnp, beams=(table, bw))
        assert np.abs(got - want).max() <= 1e-3, name
        kc, vc = _cache_values(sess)
        np.testing.assert_array_equal(kc, kc0, err_msg=name)
        np.testing.assert_array_equal(vc, vc0, err_msg=name)


@pytest.mark.parametrize("elem", ["f16", "f32"])
def test_beam_indirection_pruned_step(elem):
    """p > 0 through the table: one-workgroup and two-pass kernels.  The skip set is not returned
    by ffa_attention_ex, so keys whose probability sits within a rounding of the threshold may
    fall either way: their weight is the slack of the comparison."""
    groups, bw, H, Dh, L, p = 2, 2, 3, 64, 900, 1e-2
    B, Lmax = groups * bw, L + 1
    rng, K, V, q, k, v = _inputs(9200, B, H, L, Dh, elem)
    qd = q / np.linalg.norm(q, axis=-1, keepdims=True)
    table = rng.integers(0, bw, (B, Lmax)).astype(np.int32)
    for b in range(B):                                   # peaked keys, placed where sample b reads them
        for h in range(H):
            for pos in rng.choice(L, 16, replace=False):
                src = (b // bw) * bw + table[b, pos]
                K[src, h, pos] = O.round_to(4 * qd[b, h] + 0.1 * rng.standard_normal(Dh), elem)
    kc0, vc0 = _pack(K, V, Lmax, elem)
    dt = np.float16 if elem == "f16" else np.float32
    want, skip, P, thr = O.pruned_decode_step(q, k, v, kc0.astype(dt), vc0.astype(dt), 0.125, L, p,
                                              cache_indir=table, beam_width=bw)
    assert 0.1 < skip[:, :, :L].mean() < 0.999
    near = np.abs(P - thr[:, :, None]) <= 2.0 ** -9 * thr[:, :, None]
    Vread = np.stack([O.beam_keys_values(kc0, vc0, b, L, table, bw)[1] for b in range(B)])   # [B,H,L,Dh]
    slack = np.einsum("bhn,bhnd->bhd", np.where(near[:, :, :L], P[:, :, :L], 0), np.abs(Vread))
    ntiles = L // 64 + 1
    for plan in (capi.make_plan(capi.FFA_LAUNCH_WORKGROUP, 2, 1, ntiles), capi.make_plan(capi.FFA_LAUNCH_WORKGROUP, 16, 1, ntiles),
                 capi.make_plan(capi.FFA_LAUNCH_TWO_PASS, 4, -(-ntiles // 3), 3), None):
        _say("beams pruned", elem, plan)
        sess = ExSession(K, V, Lmax, elem)
        got = sess.step(q, k, v, 0.125, L, p=p, plan=plan, beams=(table, bw))
        assert (np.abs(got - want) <= (1e-3 if elem == "f16" else 1e-5) + slack).all(), plan


def test_beam_search_by_table_on_the_gpu_equals_search_by_cache_copy():
    """The toy beam search of the oracle's own pinning test, table side on the GPU: caches are
    never copied, rows of the table are; against the oracle searching by cache copy."""
    groups, bw, H, Dh, L, steps, elem = 2, 4, 8, 64, 130, 70, "f16"
    B, Lmax = groups * bw, L + steps
    rng, K, V, *_ = _inputs(9300, B, H, L, Dh, elem)
    sess = ExSession(K, V, Lmax, elem)
    kc, vc = _pack(K, V, Lmax, elem)
    table = np.repeat((np.arange(B) % bw)[:, None], Lmax, 1).astype(np.int32)
    for s in range(steps):
        t = L + s
        q, k, v = (O.round_to(rng.standard_normal((B, H, Dh)), elem) for _ in range(3))
        got = sess.step(q, k, v, 0.125, t, beams=(table, bw))
        want = O.decode_step(q, k, v, kc, vc, 0.125, t, acc=np.float64)
        assert np.abs(got - want).max() <= 1e-3, s
        parent = (np.arange(B) // bw) * bw + rng.integers(0, bw, B)
        kc, vc = kc[parent].copy(), vc[parent].copy()
        table = table[parent].copy()
        table[:, t] = parent % bw


def test_beam_argument_validation():
    B, H, Dh, L = 4, 2, 64, 20
    rng, K, V, q, k, v = _inputs(9400, B, H, L, Dh, "f16")
    sess = ExSession(K, V, L + 1, "f16")
    table = np.zeros((B, L + 1), np.int32)
    sess.step(q, k, v, 0.125, L, beams=(None, 2), expect=capi.FFA_ERR_BEAM)      # no table
    sess.step(q, k, v, 0.125, L, beams=(table, 0), expect=capi.FFA_ERR_BEAM)
    sess.step(q, k, v, 0.125, L, beams=(table, 3), expect=capi.FFA_ERR_BEAM)     # 4 % 3 != 0
    # entries outside [0, beam_width) are clamped, never followed out of the group
    wild = np.where(rng.random((B, L + 1)) < 0.5, -7, 1000).astype(np.int32)
    got = sess.step(q, k, v, 0.125, L, beams=(wild, 2))
    kc0, vc0 = _pack(K, V, L + 1, "f16")
    want = O.decode_step(q, k, v, kc0, vc0, 0.125, L, acc=np.float64, cache_indir=np.clip(wild, 0, 1), beam_width=2)
    assert np.abs(got - want).max() <= 1e-3


def test_beam_indirection_through_the_extension():
    """attention_ex(..., cache_indir=, beam_width=) of the PyTorch extension."""
    from fastforwardattention_amd import FastForwardAttn
    groups, bw, H, Dh, L = 2, 2, 16, 128, 2100       # 64 pairs x 2100 keys of Dh = 128
    B = groups * bw
    rng, K, V, q, k, v = _inputs(9500, B, H, L, Dh, "f16")
    table = rng.integers(0, bw, (B, L + 1)).astype(np.int32)
    dev = lambda a: torch.from_numpy(a).to("cuda:0").half()
    ffa = FastForwardAttn(dev(K), dev(V), L + 1, False)
    k_cache, v_cache = ffa.get_cache()
    out = ffa.attention_ex(dev(q), dev(k), dev(v), k_cache, v_cache, 0.1, L, None, 0.0, 0, None, None, None,
                           cache_indir=torch.from_numpy(table).to("cuda:0"), beam_width=bw)
    kc0, vc0 = _pack(K, V, L + 1, "f16")
    want = O.decode_step(q, k, v, kc0, vc0, 0.1, L, acc=np.float64, cache_indir=table, beam_width=bw)
    assert np.abs(out.float().cpu().numpy() - want).max() <= 1e-3


# ------------------------------------------------------------------ one workspace, changing plans
def _transform_step_check(sess, rng, kc, vc, t, elem, rd, biases, scale, p=0.0, plan=None, tag=""):
    """One ffa_attention_ex step with a transform on a long-lived session, against the oracle
    (which appends to kc, vc).  Returns the worst output error."""
    B, H, Dh = sess.B, sess.H, sess.Dh
    q, k, v = (O.round_to(rng.standard_normal((B, H, Dh)), elem) for _ in range(3))
    pos = O.rotary_positions(B, t)
    q2, k2, v2 = O.token_transform(q, k, v, elem, biases.get("q_bias"), biases.get("k_bias"), biases.get("v_bias"), rd, pos)
    want = O.decode_step(q2, k2, v2, kc, vc, scale, t, acc=np.float64)
    got = sess.step(q, k, v, scale, t, p=p, plan=plan, transform=dict(biases, rotary_dim=rd))
    assert np.isfinite(got).all(), (tag, t, "output was never written")
    err = float(np.abs(got - want).max())
    assert err <= {"f16": 1e-3 + 3e-4, "f32": 2e-6}[elem], (tag, t, err)
    return err


def _check_caches_after_transforms(sess, kc, vc, n, elem):
    gk, gv = _cache_values(sess)
    dk = np.abs(gk[:, :, :, :n] - kc[:, :, :, :n])
    assert (dk <= _ulp(kc[:, :, :, :n], elem) * 1.01).all() and (dk != 0).mean() < 0.01
    np.testing.assert_array_equal(gv[:, :, :n], vc[:, :, :n])


def test_rotary_decode_on_one_workspace_across_plan_changes():
    """GPT-J-shaped iterative decode at B = 1 (16 heads x 256, rotary_dim 64, fp16), t = 100 -> 300,
    ONE session and ONE workspace, the library's own plan at every step.  The planner moves between
    launches that use no workspace and sequence-split launches on the way (the test asserts that
    it does), so whatever a step leaves in the workspace meets the arrival counters of a later
    step.  Reference: the token transform of attention.cu:856-882 keeps no state between calls."""
    B, H, Dh, L, rd, elem, end = 1, 16, 256, 100, 64, "f16", 300
    rng, K, V, *_ = _inputs(4100, B, H, L, Dh, elem)
    sess = ExSession(K, V, end + 1, elem)
    kc, vc = _pack(K, V, end + 1, elem)
    kinds = set()
    for t in range(L, end):
        plan = capi.plan_launch(16, B, H, Dh, t, 0.0, False, sess.lib.ffa_device_compute_units())
        kinds.add((plan.kind, plan.n_splits > 1))
        _transform_step_check(sess, rng, kc, vc, t, elem, rd, {}, 1.0 / 16, tag=repr(plan))
    assert any(s for _, s in kinds) and any(not s for _, s in kinds), kinds   # both sides of the switch were run
    _check_caches_after_transforms(sess, kc, vc, end, elem)


@pytest.mark.parametrize("elem", ["f16", "f32"])
def test_transform_steps_of_every_launch_kind_share_one_workspace(elem):
    """Bias + rotary steps on one workspace in the order that used to break: a one-workgroup launch
    (needs no workspace of its own), a sequence-split launch with a fused merge, a pruned two-pass
    launch, a split launch merged by a second kernel, and round again."""
    B, H, Dh, L, rd = 2, 3, 64, 700, 32
    rng, K, V, *_ = _inputs(4200, B, H, L, Dh, elem)
    steps = 10
    sess = ExSession(K, V, L + steps, elem)
    kc, vc = _pack(K, V, L + steps, elem)
    biases = {n: O.round_to(rng.standard_normal((H, Dh)), elem) for n in ("q_bias", "k_bias", "v_bias")}
    for i in range(steps):
        t = L + i
        ntiles = t // 64 + 1
        plan, p = [
            (capi.make_plan(capi.FFA_LAUNCH_WORKGROUP, 4, 1, ntiles), 0.0),
            (capi.make_plan(capi.FFA_LAUNCH_SPLIT, 4, -(-ntiles // 3), 3), 0.0),
            (capi.make_plan(capi.FFA_LAUNCH_TWO_PASS, 4, -(-ntiles // 2), 2), 1e-7),   # below every probability
            (capi.make_plan(capi.FFA_LAUNCH_SPLIT, 2, -(-ntiles // 4), 4, capi.FFA_COMBINE_KERNEL), 0.0),
            (capi.make_plan(capi.FFA_LAUNCH_SPLIT, 4, 1, ntiles, whole_heads=B * H), 0.0),
        ][i % 5]
        _say("shared workspace", elem, i, plan)
        _transform_step_check(sess, rng, kc, vc, t, elem, rd, biases, 0.125, p=p, plan=plan, tag=repr(plan))
    _check_caches_after_transforms(sess, kc, vc, L + steps, elem)


def test_alternating_pruned_and_exact_calls_on_one_object():
    """attention_ex of the Python class with the rotary embedding, p > 0 and p = 0 in turn: at this
    shape a pruned step is a one-workgroup launch and an exact step a sequence-split one, on the
    object's one workspace."""
    from fastforwardattention_amd import FastForwardAttn
    B, H, Dh, L, rd, steps = 2, 32, 64, 995, 32, 12
    rng, K, V, *_ = _inputs(4300, B, H, L, Dh, "f16")
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a, np.float32)).to("cuda:0").half()
    ffa = FastForwardAttn(dev(K), dev(V), L + steps, False)
    k_cache, v_cache = ffa.get_cache()
    kc, vc = _pack(K, V, L + steps, "f16")
    plans = set()
    for i in range(steps):
        t, p = L + i, (1e-7 if i % 2 == 0 else 0.0)
        plans.add(tuple(ffa.launch_plan(t, p))[:1] + (tuple(ffa.launch_plan(t, p))[4] > 1,))
        q, k, v = (O.round_to(rng.standard_normal((B, H, Dh)), "f16") for _ in range(3))
        q2, k2, v2 = O.token_transform(q, k, v, "f16", rotary_dim=rd, pos=O.rotary_positions(B, t))
        want = O.decode_step(q2, k2, v2, kc, vc, 0.125, t, acc=np.float64)
        out = ffa.attention_ex(dev(q), dev(k), dev(v), k_cache, v_cache, 0.125, t, None, p, rd, None, None, None)
        got = out.float().cpu().numpy()
        assert np.isfinite(got).all(), i
        assert np.abs(got - want).max() <= 1e-3 + 3e-4, (i, p)
    assert (capi.FFA_LAUNCH_WORKGROUP, False) in plans and (capi.FFA_LAUNCH_SPLIT, True) in plans, plans


def test_load_floor_probe_runs_every_split_plan_and_touches_nothing():
    """ffa_load_floor (the measurement aid behind bench.py's `load_floor_us`): every split plan with
    one lane per key and 2 / 4 / 8 waves launches, the caches and the sink stay as they were (the
    probe only loads), other plans are refused before anything is launched."""
    lib = capi.load()
    for prec, Dh in ((16, 64), (16, 80), (16, 256), (32, 64), (32, 128)):
        B, H, L, Lmax = 2, 5, 700, 768
        tdt = torch.float16 if prec == 16 else torch.float32
        x = 16 // (prec // 8)
        g = torch.Generator(device="cuda:0").manual_seed(prec + Dh)
        kc = torch.randn(B, H, Dh // x, Lmax, x, device="cuda:0", generator=g).to(tdt)
        vc = torch.randn(B, H, Lmax, Dh, device="cuda:0", generator=g).to(tdt)
        kc0, vc0 = kc.clone(), vc.clone()
        sink = torch.full((4,), 7, dtype=torch.int32, device="cuda:0")
        ntiles = L // 64 + 1
        for waves in (2, 4, 8):
            for n_splits, whole in ((1, B * H), (3, 0), (4, 0), (11, 0)):
                tps = -(-ntiles // n_splits)
                plan = capi.make_plan(capi.FFA_LAUNCH_SPLIT, waves, -(-ntiles // tps), tps, 0, whole)
                _say("load floor", prec, Dh, plan)
                rc = lib.ffa_load_floor(prec, B, H, Dh, Lmax, L, ptr(kc), ptr(vc), None, 1, C.byref(plan), ptr(sink), None)
                assert rc == capi.FFA_OK, capi.STATUS_NAMES.get(rc, rc)
        torch.cuda.synchronize()
        assert torch.equal(kc, kc0) and torch.equal(vc, vc0) and bool((sink == 7).all())
        for bad in (capi.make_plan(capi.FFA_LAUNCH_WORKGROUP, 4, 1, ntiles),
                    capi.make_plan(capi.FFA_LAUNCH_SPLIT, 3, 1, ntiles, 0, B * H),
                    capi.make_plan(capi.FFA_LAUNCH_TWO_PASS, 4, 2, -(-ntiles // 2))):
            rc = lib.ffa_load_floor(prec, B, H, Dh, Lmax, L, ptr(kc), ptr(vc), None, 1, C.byref(bad), ptr(sink), None)
            assert rc == capi.FFA_ERR_PLAN, capi.STATUS_NAMES.get(rc, rc)
        assert lib.ffa_load_floor(prec, B, H, Dh, Lmax, L, ptr(kc), ptr(vc), None, 1, None, ptr(sink), None) == capi.FFA_ERR_NULL_POINTER
