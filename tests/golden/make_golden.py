"""Writes tests/golden/decode_cases.npz: small seeded decode-step cases with the results of
the CPU oracle (oracle/ffa_oracle.py).  The reference holds no golden vectors for this path
(its only check is example.py:46, max|out - torch_attn_func| printed on a CUDA GPU), so these
fixtures are produced by this repository's own oracle, which is pinned separately by closed
forms, brute force and known answers (tests/test_oracle.py).  They freeze the oracle's
outputs: a later change to the oracle or to the kernels that moves a result is caught even
where both would still agree with each other.

    python tests/golden/make_golden.py          # rewrites the fixture in place

Inputs are stored once, as fp16; the fp32 cases use the same values upcast, so both
precisions see the same numbers."""
from __future__ import annotations

import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import ffa_oracle as O  # noqa: E402

# name: (B, H, Dh, t, first_key per sample or None, npeaks)
CASES = {
    "t0": (1, 2, 64, 0, None, 0),
    "t37": (2, 3, 64, 37, None, 4),
    "dh256_t130": (1, 2, 256, 130, None, 8),
    "leftpad_t300": (2, 2, 64, 300, [0, 77], 8),
}
THRESHOLDS = (0.0, 1e-3, 1e-2, 0.2)


def build_inputs(name):
    B, H, Dh, t, first, npeaks = CASES[name]
    rng = np.random.default_rng(sum(map(ord, name)))   # a fixed seed per case
    K = rng.standard_normal((B, H, t, Dh)).astype(np.float16)
    V = rng.standard_normal((B, H, t, Dh)).astype(np.float16)
    q, k, v = (rng.standard_normal((B, H, Dh)).astype(np.float16) for _ in range(3))
    if npeaks and t:
        qd = q.astype(np.float32) / np.linalg.norm(q.astype(np.float32), axis=-1, keepdims=True)
        for b in range(B):
            for h in range(H):
                pos = rng.choice(t, min(npeaks, t), replace=False)
                K[b, h, pos] = (4 * qd[b, h] + 0.1 * rng.standard_normal((len(pos), Dh))).astype(np.float16)
    return K, V, q, k, v


def expected(name, K, V, q, k, v, dtype):
    """dict of arrays for one case in one precision."""
    B, H, Dh, t, first, _ = CASES[name]
    Lmax = t + 2
    scale = 1.0 / np.sqrt(Dh)
    K, V, q, k, v = (a.astype(dtype) for a in (K, V, q, k, v))
    sl = None if first is None else np.asarray(first, np.int32)
    res = {}
    kc, vc = O.pack_k_cache(K, Lmax), O.pack_v_cache(V, Lmax)
    res["out_exact"] = O.decode_step(q, k, v, kc, vc, scale, t, seq_lengths=sl,
                                     right_or_no_padding=sl is None, acc=np.float64).astype(np.float32)
    if K.size <= 20000:                              # the caches after the append (small cases)
        res["k_cache"], res["v_cache"] = kc, vc
    for p in THRESHOLDS[1:]:
        kc, vc = O.pack_k_cache(K, Lmax), O.pack_v_cache(V, Lmax)
        out, skip, P, thr = O.pruned_decode_step(q, k, v, kc, vc, scale, t, p, seq_lengths=sl,
                                                 right_or_no_padding=sl is None)
        res[f"out_p{p:g}"] = out.astype(np.float32)
        res[f"skip_p{p:g}"] = np.packbits(skip, axis=-1)
        res[f"prob_p{p:g}"] = P.astype(np.float32)
        res[f"thr_p{p:g}"] = thr.astype(np.float32)
    return res


def main():
    blob = {}
    for name in CASES:
        K, V, q, k, v = build_inputs(name)
        for key, arr in (("K", K), ("V", V), ("q", q), ("k", k), ("v", v)):
            blob[f"{name}/{key}"] = arr
        for prec, dtype in ((16, np.float16), (32, np.float32)):
            for key, arr in expected(name, K, V, q, k, v, dtype).items():
                blob[f"{name}/f{prec}/{key}"] = arr
    path = os.path.join(HERE, "decode_cases.npz")
    np.savez_compressed(path, **blob)
    print(path, os.path.getsize(path), "bytes,", len(blob), "arrays")


if __name__ == "__main__":
    main()
