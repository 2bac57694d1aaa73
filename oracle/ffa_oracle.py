"""CPU oracle for the FastForwardAttention decode step.  TEST INFRASTRUCTURE ONLY.

This module is the checker, never the product: only tests/, __graft_entry__.smoke()
and bench.py's cpu_baseline leg may import it.  The shipped path
(fastforwardattention_amd) must never import it and has no CPU fallback.

It restates, in numpy, what the reference computes for one decode step.  All
citations are file:line under the reference checkout.

  attn_closed_form      example.py:6-7, README.md:29-34   softmax(q.K^T*scale).V
  pack_k_cache          attention.cu:1564-1582            [B,H,L,Dh] -> [B,H,Dh/x,Lmax,x]
  pack_v_cache          attention.cu:1593-1608            [B,H,L,Dh] -> [B,H,Lmax,Dh]
  append_kv             attention.cu:901-914, :1246       write slot t of both caches
  decode_step           attention.cu:805-817, :1054, :1072, :1111-1116 (masking)
  beam_keys_values      attention.cu:779-793, :1003, :1024-1033, :1143, :1195-1202 (cache_indir)
  half_from_ushort_rn   cuda_fp16.h __half(unsigned short) == __ushort2half_rn
  leq_f16_bits          attention.cu:466-469              __hle on converted bit patterns
  pruned_decode_step    attention.cu:1108-1126, :1184-1191, :1227-1256
  token_transform       attention.cu:856-882, :1157-1158, :1242 (bias);
                        decoder_masked_multihead_attention_utils.h:1137-1160 (rotary)
  f32_to_bf16_bits / bf16_bits_to_f32   utils.h:44-125 (the bf16 build the reference never
                        enables): round-to-nearest-even truncation of an fp32 to 16 bits

Pinning status (what independent evidence fixes each function):
  attn_closed_form   pinned: brute-force Python loops, torch.softmax/bmm, fp64, and the
                     special cases t=0, q=0, one dominant key, permutation invariance.
  pack_*/append_kv   pinned: pure index permutations checked element by element against
                     the index formula of the reference kernels on tiny shapes.
  half_from_ushort_rn / leq_f16_bits
                     pinned: known answers of IEEE round-to-nearest-even at 11 significant
                     bits (2049->2048, 2051->2052, 65520->inf) and exhaustive comparison
                     with numpy's own uint16->float16 cast over all 65536 patterns.
  beam_keys_values   pinned: the identity table reproduces the plain step bit for bit; a
                     simulated beam search that re-parents beams by permuting table rows
                     gives, step by step, bit-identical outputs to one that copies whole
                     caches the way the reference's models do (_reorder_cache,
                     modeling_opt.py:1072-1075); an element-by-element Python loop over the
                     reference's flat offsets on a tiny case.
  token_transform    pinned: the installed transformers' GPT-J apply_rotary_pos_emb /
                     create_sinusoidal_positions on fp32 tensors (same pairs, signs and
                     angles), a rotation's invariants (norm of every pair, position 0 is
                     the identity, angles add), and the bias as plain addition.
  bf16 conversions   pinned: torch's own float32 -> bfloat16 cast over random, tie, tiny,
                     huge and special values; bf16 -> fp32 is a 16-bit shift.
  pruned_decode_step parity unpinned against the reference binary: no reference script
                     ever runs p>0 and the CUDA source cannot be built here.  It is pinned
                     only by invariants (p=0 and sub-resolution p reproduce the unpruned
                     result, the new token is never dropped, no renormalisation, the
                     skip set is monotone in p) and by reading the source.
"""
from __future__ import annotations

import numpy as np

EPS_SUM = np.float32(1.0e-6)  # attention.cu:1122  inv_sum = 1 / (sum + 1e-6)


def elems_per_16b(dtype) -> int:
    """x of the K-cache layout: 8 for fp16, 4 for fp32 (attention.cu:1562)."""
    return 16 // np.dtype(dtype).itemsize


# --------------------------------------------------------------------------- layouts
def pack_k_cache(K: np.ndarray, max_len: int, fill=0) -> np.ndarray:
    """k_dst[b,h,c,l,:] = K[b,h,l,c*x:(c+1)*x] for l < L (attention.cu:1575-1582).

    Slots l >= L are unspecified in the reference (torch::empty); `fill` marks them."""
    B, H, L, Dh = K.shape
    x = elems_per_16b(K.dtype)
    assert Dh % x == 0 and L <= max_len
    out = np.full((B, H, Dh // x, max_len, x), fill, dtype=K.dtype)
    out[:, :, :, :L, :] = K.reshape(B, H, L, Dh // x, x).transpose(0, 1, 3, 2, 4)
    return out


def unpack_k_cache(k_cache: np.ndarray, length: int) -> np.ndarray:
    """Inverse of pack_k_cache for the first `length` slots -> [B,H,length,Dh]."""
    B, H, C, Lmax, x = k_cache.shape
    return np.ascontiguousarray(
        k_cache[:, :, :, :length, :].transpose(0, 1, 3, 2, 4)).reshape(B, H, length, C * x)


def pack_v_cache(V: np.ndarray, max_len: int, fill=0) -> np.ndarray:
    """v_dst[b,h,l,:] = V[b,h,l,:] for l < L (attention.cu:1593-1608)."""
    B, H, L, Dh = V.shape
    out = np.full((B, H, max_len, Dh), fill, dtype=V.dtype)
    out[:, :, :L, :] = V
    return out


def append_kv(k_cache, v_cache, k_new, v_new, t):
    """In-place append at slot t.  K: offset (d/x)*Lmax*x + t*x + d%x (attention.cu:901-913);
    V: offset t*Dh + d (attention.cu:1246).  `t` is an int or a per-batch int array."""
    B, H, C, Lmax, x = k_cache.shape
    k_new = np.asarray(k_new).reshape(B, H, C, x)
    v_new = np.asarray(v_new).reshape(B, H, C * x)
    tt = np.broadcast_to(np.asarray(t, dtype=np.int64), (B,))
    for b in range(B):
        k_cache[b, :, :, tt[b], :] = k_new[b]
        v_cache[b, :, tt[b], :] = v_new[b]


# --------------------------------------------------------------------------- closed form
def attn_closed_form(q, K, V, scale, first_key=None, acc=np.float32):
    """out[n,:] = sum_i softmax_i(scale * q[n].K[n,i]) V[n,i]  (example.py:6-7).

    q [N,Dh]; K,V [N,T,Dh]; first_key: optional [N] ints, keys i < first_key[n] are
    excluded (left padding: attention.cu:1054, :1072, :1112-1113).  Arithmetic in `acc`."""
    q = np.asarray(q, dtype=acc)
    K = np.asarray(K, dtype=acc)
    V = np.asarray(V, dtype=acc)
    s = np.einsum("nd,ntd->nt", q, K).astype(acc) * acc(scale)
    if first_key is not None:
        idx = np.arange(K.shape[1])[None, :]
        s = np.where(idx < np.asarray(first_key)[:, None], -np.inf, s).astype(acc)
    m = s.max(axis=1, keepdims=True)
    e = np.exp(s - m).astype(acc)
    w = e / e.sum(axis=1, keepdims=True, dtype=acc)
    return np.einsum("nt,ntd->nd", w.astype(acc), V).astype(acc)


def _bounds(B, t, seq_lengths, right_or_no_padding):
    """(tlength[b], first_key[b]) exactly as attention.cu:805-817."""
    if seq_lengths is None:
        return np.full(B, t, np.int64), np.zeros(B, np.int64)
    sl = np.asarray(seq_lengths, dtype=np.int64).reshape(B)
    if right_or_no_padding:
        return sl.copy(), np.zeros(B, np.int64)
    return np.full(B, t, np.int64), sl.copy()


def beam_keys_values(k_cache, v_cache, b, n, cache_indir=None, beam_width=1):
    """Keys and values 0..n-1 that sample b attends over, as (K [H,n,Dh], V [H,n,Dh]); slot
    n-1 holds the token just appended.

    Without a table: the sample's own caches.  With one (beam search): sample b is beam
    b % beam_width of group bbi = b // beam_width (attention.cu:785-787); key ti < n-1 is read
    from sample bbi*beam_width + cache_indir[b*Lmax + ti] (attention.cu:1003, :1024-1033 for K,
    :1143, :1195-1202 for V -- the base pointer is the group's first beam, the table entry an
    offset of whole samples from it); the new token (ti = n-1) never goes through the table:
    it is taken from the registers that also write it to the sample's own slot
    (attention.cu:901-914, :1227-1256)."""
    B, H, C, Lmax, x = k_cache.shape
    if cache_indir is None:
        return unpack_k_cache(k_cache[b:b + 1], n)[0], v_cache[b, :, :n, :]
    indir = np.asarray(cache_indir).reshape(B, Lmax)
    bbi = b // beam_width
    src = np.full(n, b, np.int64)
    src[:n - 1] = bbi * beam_width + indir[b, :n - 1]
    K = np.empty((H, n, C * x), k_cache.dtype)
    V = np.empty((H, n, C * x), v_cache.dtype)
    for ti in range(n):
        K[:, ti, :] = k_cache[src[ti], :, :, ti, :].reshape(H, C * x)
        V[:, ti, :] = v_cache[src[ti], :, ti, :]
    return K, V


def decode_step(q, k, v, k_cache, v_cache, scale, t, seq_lengths=None,
                right_or_no_padding=True, acc=np.float32, cache_indir=None, beam_width=1):
    """One exact (p = 0) decode step: append k,v at slot tlength[b], attend over keys
    first_key[b] .. tlength[b] (read through `cache_indir` when given, see beam_keys_values).
    Mutates the caches.  Returns out [B,H,Dh] in `acc`."""
    B, H, C, Lmax, x = k_cache.shape
    Dh = C * x
    tlen, first = _bounds(B, t, seq_lengths, right_or_no_padding)
    append_kv(k_cache, v_cache, k, v, tlen)
    q = np.asarray(q).reshape(B, H, Dh)
    out = np.zeros((B, H, Dh), dtype=acc)
    for b in range(B):
        n = int(tlen[b]) + 1
        Kb, Vb = beam_keys_values(k_cache, v_cache, b, n, cache_indir, beam_width)
        if first[b] > tlen[b]:
            continue  # every key masked: sum = 0, all logits 0 -> out = 0 (attention.cu:1113)
        out[b] = attn_closed_form(q[b], Kb, Vb, scale,
                                  first_key=np.full(H, first[b]), acc=acc)
    return out


# --------------------------------------------------------------------------- fp16 compare
def half_from_ushort_rn(u) -> np.ndarray:
    """__ushort2half_rn: the NUMERIC value of an unsigned 16-bit integer rounded to
    fp16 with round-to-nearest-even (values >= 65520 become +inf).  Implemented on the
    integer itself (11 significant bits), not with numpy's cast, so that the cast can
    serve as an independent check in the tests."""
    u = np.asarray(u, dtype=np.int64)
    out = np.zeros(u.shape, dtype=np.float64)
    nz = u > 0
    nbits = np.zeros(u.shape, dtype=np.int64)
    nbits[nz] = np.floor(np.log2(u[nz])).astype(np.int64) + 1
    shift = np.maximum(nbits - 11, 0)
    low = u & ((1 << shift) - 1)
    half = np.where(shift > 0, 1 << np.maximum(shift - 1, 0), 0)
    base = u >> shift
    round_up = (shift > 0) & ((low > half) | ((low == half) & ((base & 1) == 1)))
    r = (base + round_up.astype(np.int64)) << shift
    out = r.astype(np.float64)
    out[r >= 65520] = np.inf
    return out


def leq_f16_bits(a_bits, b_bits) -> np.ndarray:
    """leq(uint16_t a, uint16_t b) = __hle(__half(a), __half(b)) (attention.cu:466-469),
    where __half(unsigned short) converts the integer VALUE (build flag
    -U__CUDA_NO_HALF_CONVERSIONS__, setup.py:11)."""
    return half_from_ushort_rn(a_bits) <= half_from_ushort_rn(b_bits)


# --------------------------------------------------------------------------- bf16, rounding to T
def f32_to_bf16_bits(x) -> np.ndarray:
    """fp32 -> bf16 bit pattern, round-to-nearest-even on the 16 dropped bits; NaN stays NaN."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    return np.where(nan, ((u >> 16) | 0x40).astype(np.uint16), r)


def bf16_bits_to_f32(b) -> np.ndarray:
    return (np.asarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def round_to(x, elem: str) -> np.ndarray:
    """x rounded to the element type T ("f16", "bf16" or "f32"), returned as fp32 values."""
    x = np.asarray(x, dtype=np.float32)
    if elem == "f16":
        return x.astype(np.float16).astype(np.float32)
    if elem == "bf16":
        return bf16_bits_to_f32(f32_to_bf16_bits(x))
    assert elem == "f32"
    return x


# --------------------------------------------------------------------------- bias and rotary embedding
def rotary_angles(pos, rotary_dim, base=10000.0) -> np.ndarray:
    """angle[b, i] = pos[b] / base^(2i / rotary_dim), i < rotary_dim/2
    (rotary_embedding_coefficient, utils.h:1137-1141), in float64."""
    zid = np.arange(0, rotary_dim, 2, dtype=np.float64)
    denom = np.power(np.float64(np.float32(base)), zid / np.float64(rotary_dim))
    return np.asarray(pos, dtype=np.float64).reshape(-1, 1) / denom[None, :]


def token_transform(q, k, v, elem, q_bias=None, k_bias=None, v_bias=None, rotary_dim=0, pos=None,
                    base=10000.0):
    """What the reference's kernel does to the new token before attending (disabled by its
    host code, attention.cu:1472-1483): q += q_bias, k += k_bias (attention.cu:856-873),
    v += v_bias (:1242); then for every pair (2i, 2i+1) with 2i < rotary_dim, q and k are
    rotated: (x, y) -> (c x - s y, c y + s x), c, s = cos, sin of rotary_angles (:874-882;
    utils.h:1143-1156).  The reference evaluates this in fp32 after adding the bias in T; here
    (and in the kernel this checks) it is evaluated in float64 on the T-valued inputs and
    rounded to fp32, then once to T: an fp32 angle of hundreds of radians is uncertain by 1e-5,
    more than an ulp of the result, and could not be checked across two math libraries.
    q, k, v: [B,H,Dh]; biases [H,Dh]; pos [B] = position of the new token of each sample.
    Returns fp32 arrays holding T-representable values."""
    q, k, v = (np.asarray(a, dtype=np.float32).astype(np.float64) for a in (q, k, v))
    if q_bias is not None:
        q = q + np.asarray(q_bias, dtype=np.float32).astype(np.float64)[None]
    if k_bias is not None:
        k = k + np.asarray(k_bias, dtype=np.float32).astype(np.float64)[None]
    if v_bias is not None:
        v = v + np.asarray(v_bias, dtype=np.float32).astype(np.float64)[None]
    if rotary_dim > 0:
        ang = rotary_angles(pos, rotary_dim, base)                     # [B, rotary_dim/2]
        c, s = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
        for a in (q, k):
            x, y = a[..., 0:rotary_dim:2].copy(), a[..., 1:rotary_dim:2].copy()
            a[..., 0:rotary_dim:2] = c * x - s * y
            a[..., 1:rotary_dim:2] = c * y + s * x
    return tuple(round_to(a.astype(np.float32), elem) for a in (q, k, v))


def rotary_positions(B, t, seq_lengths=None, right_or_no_padding=True) -> np.ndarray:
    """Position of the new token among the sample's real tokens: the slot it is written to
    minus the first unmasked key (t; seq_lengths[b] with right padding; t - seq_lengths[b]
    with left padding).  The reference rotates by t alone (attention.cu:879)."""
    tlen, first = _bounds(B, t, seq_lengths, right_or_no_padding)
    return np.maximum(tlen - first, 0)


# --------------------------------------------------------------------------- pruning rule
def pruned_decode_step(q, k, v, k_cache, v_cache, scale, t, p, seq_lengths=None,
                       right_or_no_padding=True, elem=None, cache_indir=None, beam_width=1):
    """One decode step with threshold-p pruning, transcribed from attention.cu.

    Per (b,h), with e_i = exp(s_i - max over unmasked s) (0 if masked, :1111-1116),
    S = sum_i e_i, inv = 1/(S + 1e-6) (:1122):
        P_i = T(e_i * inv)          (:1124-1126, T = dtype of the caches, RN for fp16)
        thr = T(p * inv)            (:1184-1185)
        for i < tlength: skip iff leq(P_i, thr)   (:1188-1191)
        slot tlength (the new token) is always kept (:1227-1256)
        out = sum_kept P_i * V_i    (no renormalisation)
    Scores s_i, the P.V products and their sum are carried in fp32 here (the reference
    carries them in T; this build's contract is fp32 accumulation), the result is
    returned in fp32 before the final rounding to T.

    Keys are read through `cache_indir` when given (beam_keys_values).

    elem = "bf16" (caches passed as fp32 arrays of bf16 values): T-rounding to bf16 and a
    numeric P_i <= thr; the reference has no bf16 behaviour to follow (ENABLE_BF16 is never
    defined), this is the fp32 rule with bf16 rounding.

    Returns (out [B,H,Dh] float32, skipped [B,H,Lmax] bool, P [B,H,Lmax] float32,
    thr [B,H] float32).  Mutates the caches (append)."""
    B, H, C, Lmax, x = k_cache.shape
    Dh = C * x
    is_half = k_cache.dtype == np.float16
    f32 = np.float32
    tlen, first = _bounds(B, t, seq_lengths, right_or_no_padding)
    append_kv(k_cache, v_cache, k, v, tlen)
    q = np.asarray(q).reshape(B, H, Dh).astype(f32)
    out = np.zeros((B, H, Dh), f32)
    skipped = np.zeros((B, H, Lmax), bool)
    Pall = np.zeros((B, H, Lmax), f32)
    thr_all = np.zeros((B, H), f32)
    for b in range(B):
        n = int(tlen[b]) + 1
        Kb, Vb = beam_keys_values(k_cache, v_cache, b, n, cache_indir, beam_width)   # [H,n,Dh]
        Kb, Vb = Kb.astype(f32), Vb.astype(f32)
        s = (np.einsum("hd,hnd->hn", q[b], Kb).astype(f32) * f32(scale)).astype(f32)
        masked = np.arange(n)[None, :] < first[b]
        masked = np.broadcast_to(masked, s.shape)
        smax = np.where(masked, -np.inf, s).max(axis=1, keepdims=True)
        smax = np.where(np.isfinite(smax), smax, f32(0)).astype(f32)
        e = np.where(masked, f32(0), np.exp((s - smax).astype(f32))).astype(f32)
        S = e.sum(axis=1, keepdims=True, dtype=f32)
        inv = (f32(1) / (S + EPS_SUM)).astype(f32)
        Pf = (e * inv).astype(f32)
        thrf = (f32(p) * inv).astype(f32)
        if elem == "bf16":
            Pv, thrv = round_to(Pf, "bf16"), round_to(thrf, "bf16")
            skip = Pv <= thrv
        elif is_half:
            Ph = Pf.astype(np.float16)
            thrh = thrf.astype(np.float16)
            skip = leq_f16_bits(Ph.view(np.uint16), thrh.view(np.uint16))
            Pv = Ph.astype(f32)
            thrv = thrh.astype(f32)
        else:
            skip = Pf <= thrf
            Pv, thrv = Pf, thrf
        skip = skip.copy()
        skip[:, n - 1] = False                       # current token never pruned
        w = np.where(skip, f32(0), Pv).astype(f32)
        out[b] = np.einsum("hn,hnd->hd", w, Vb).astype(f32)
        skipped[b, :, :n] = skip
        Pall[b, :, :n] = Pv
        thr_all[b] = thrv[:, 0]
    return out, skipped, Pall, thr_all


# --------------------------------------------------------------------------- brute force
def attn_bruteforce(q, K, V, scale, first_key=0):
    """Pure-Python-loop softmax attention for ONE head in float64; tiny inputs only."""
    import math
    T = len(K)
    Dh = len(q)
    s = []
    for i in range(T):
        if i < first_key:
            s.append(None)
            continue
        acc = 0.0
        for d in range(Dh):
            acc += float(q[d]) * float(K[i][d])
        s.append(acc * float(scale))
    live = [z for z in s if z is not None]
    m = max(live)
    e = [0.0 if z is None else math.exp(z - m) for z in s]
    tot = sum(e)
    out = [0.0] * Dh
    for i in range(T):
        for d in range(Dh):
            out[d] += e[i] / tot * float(V[i][d])
    return out
