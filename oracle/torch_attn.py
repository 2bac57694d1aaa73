"""CPU restatement of the reference's torch path.  TEST / BASELINE INFRASTRUCTURE ONLY.

`torch_attn_func` restates example.py:6-7 (README.md:29-30): two bmm calls around a
softmax, in fp32, on CPU tensors.  It is (a) the p = 0 parity reference at full sizes
and (b) the thing bench.py times on the GPU box's host cores as `cpu_baseline`
(kind "port").  The shipped package never imports this file.

`CpuDecodeBaseline` keeps K and V in pre-allocated [B*H, Lmax, Dh] fp32 buffers and
writes row t in place, instead of the reference demo's per-step torch.cat
(example.py:40-41), so that the timed work is the attention itself and not a copy of
the whole cache.
"""
from __future__ import annotations

import torch


def torch_attn_func(Q, K, V, softmax_temp):
    # example.py:6-7
    w = torch.nn.functional.softmax(torch.bmm(Q, K.transpose(1, 2)) * softmax_temp, dim=-1)
    return torch.bmm(w, V)


class CpuDecodeBaseline:
    """fp32 CPU decode attention over a pre-allocated cache (see module docstring)."""

    def __init__(self, K: torch.Tensor, V: torch.Tensor, max_len: int):
        B, H, L, Dh = K.shape
        self.B, self.H, self.Dh, self.Lmax = B, H, Dh, max_len
        self.K = torch.zeros(B * H, max_len, Dh, dtype=torch.float32)
        self.V = torch.zeros(B * H, max_len, Dh, dtype=torch.float32)
        self.K[:, :L] = K.reshape(B * H, L, Dh).float()
        self.V[:, :L] = V.reshape(B * H, L, Dh).float()

    def attention(self, q, k, v, scale: float, t: int) -> torch.Tensor:
        BH, Dh = self.B * self.H, self.Dh
        self.K[:, t] = k.reshape(BH, Dh).float()
        self.V[:, t] = v.reshape(BH, Dh).float()
        out = torch_attn_func(q.reshape(BH, 1, Dh).float(), self.K[:, :t + 1],
                              self.V[:, :t + 1], scale)
        return out.reshape(self.B, self.H, Dh)
