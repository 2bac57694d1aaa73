"""Helpers shared by the GPU parity tests: a thin driver of the C ABI over torch device
memory, and seeded input builders.  Test infrastructure only."""
from __future__ import annotations

import ctypes as C

import numpy as np
import torch

from fastforwardattention_amd import capi

NP_DTYPE = {16: np.float16, 32: np.float32}
TORCH_DTYPE = {16: torch.float16, 32: torch.float32}


def ptr(t):
    return C.c_void_p(t.data_ptr()) if t is not None else None


class CApiSession:
    """Owns device caches + workspace for one (B,H,Dh,Lmax,precision) problem and drives
    ffa_init_cache_* / ffa_attention_* exactly as a foreign host would."""

    def __init__(self, K: np.ndarray, V: np.ndarray, max_len: int, sentinel=None):
        self.lib = capi.load()
        B, H, L, Dh = K.shape
        self.B, self.H, self.L, self.Dh, self.Lmax = B, H, L, Dh, max_len
        self.precision = 16 if K.dtype == np.float16 else 32
        tdt = TORCH_DTYPE[self.precision]
        x = 16 // K.dtype.itemsize
        dev = "cuda:0"
        self.k_cache = torch.empty(B, H, Dh // x, max_len, x, dtype=tdt, device=dev)
        self.v_cache = torch.empty(B, H, max_len, Dh, dtype=tdt, device=dev)
        if sentinel is not None:
            self.k_cache.fill_(sentinel)
            self.v_cache.fill_(sentinel)
        self.Kd = torch.from_numpy(K).to(dev).contiguous()
        self.Vd = torch.from_numpy(V).to(dev).contiguous()
        fn = self.lib.ffa_init_cache_f16 if self.precision == 16 else self.lib.ffa_init_cache_f32
        capi.check(fn(ptr(self.k_cache), ptr(self.v_cache), ptr(self.Kd), ptr(self.Vd),
                      B, L, max_len, Dh, H, None), "ffa_init_cache")
        nbytes = self.lib.ffa_workspace_bytes(B, H, Dh, max_len)
        self.ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        capi.check(self.lib.ffa_workspace_init(ptr(self.ws), nbytes, None), "ffa_workspace_init")
        torch.cuda.synchronize()

    def step(self, q, k, v, scale, t, p=0.0, plan=None, seq_lengths=None,
             right_or_no_padding=True, diag=False, expect=capi.FFA_OK):
        dev = "cuda:0"
        tdt = TORCH_DTYPE[self.precision]
        qd = torch.from_numpy(np.ascontiguousarray(q)).to(dev)
        kd = torch.from_numpy(np.ascontiguousarray(k)).to(dev)
        vd = torch.from_numpy(np.ascontiguousarray(v)).to(dev)
        out = torch.full((self.B, self.H, self.Dh), float("nan"), dtype=tdt, device=dev)
        sl = None
        if seq_lengths is not None:
            sl = torch.from_numpy(np.asarray(seq_lengths, dtype=np.int32)).to(dev)
        kept = mask = None
        if diag:
            kept = torch.zeros(self.B, self.H, dtype=torch.int32, device=dev)
            mask = torch.zeros(self.B, self.H, self.Lmax, dtype=torch.uint8, device=dev)
        plan_p = C.byref(plan) if plan is not None else None
        rc = self.lib.ffa_attention_diag(
            self.precision, self.B, self.H, self.Dh, self.Lmax, float(scale), int(t),
            ptr(qd), ptr(kd), ptr(vd), ptr(self.k_cache), ptr(self.v_cache), ptr(out), ptr(sl),
            float(p), plan_p, int(bool(right_or_no_padding)), ptr(self.ws), self.ws.numel(),
            ptr(kept), ptr(mask), None)
        assert rc == expect, f"status {capi.STATUS_NAMES.get(rc, rc)}, expected {capi.STATUS_NAMES.get(expect)}"
        torch.cuda.synchronize()
        if rc != capi.FFA_OK:
            return None
        res = out.float().cpu().numpy()
        if diag:
            return res, kept.cpu().numpy(), mask.cpu().numpy().astype(bool)
        return res

    def caches(self):
        return self.k_cache.cpu().numpy(), self.v_cache.cpu().numpy()


def rand_inputs(seed, B, H, L, Dh, precision, kv_scale=1.0):
    rng = np.random.default_rng(seed)
    dt = NP_DTYPE[precision]
    K = (rng.standard_normal((B, H, L, Dh)) * kv_scale).astype(dt)
    V = (rng.standard_normal((B, H, L, Dh)) * kv_scale).astype(dt)
    return rng, K, V


def rand_token(rng, B, H, Dh, precision):
    dt = NP_DTYPE[precision]
    return tuple(rng.standard_normal((B, H, Dh)).astype(dt) for _ in range(3))
