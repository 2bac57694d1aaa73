"""Usage demo of the decode-attention engine on an MI355X: the counterpart of the reference's
example.py (example.py:1-46), which it follows in shapes and call pattern (prompt of 1024
keys, 128 generated tokens, B=10, 32 heads x 64).  Differences: inputs are N(0,1) instead of
U(0,1) (so the softmax is not flat), the check is an absolute tolerance against an fp32
evaluation of softmax(Q K^T scale) V (README.md:29-34), and the per-step time is printed.

    python -m fastforwardattention_amd.example [--dtype float32] [--default-launch] [--p 0.01]
"""
from __future__ import annotations

import argparse
from math import sqrt

import torch


def torch_attn_func(Q, K, V, softmax_temp):
    """The reference's ground truth (example.py:6-7)."""
    return torch.bmm(torch.nn.functional.softmax(torch.bmm(Q, K.transpose(1, 2)) * softmax_temp, dim=-1), V)


def main():
    ap = argparse.ArgumentParser(description=__doc__.splitlines()[0])
    ap.add_argument("--dtype", default="float16", choices=["float16", "float32"])
    ap.add_argument("--default-launch", action="store_true",
                    help="one workgroup per (batch, head), like FasterTransformer's launch")
    ap.add_argument("--p", type=float, default=0.0, help="pruning threshold (0 = exact attention)")
    args = ap.parse_args()

    # Same class object as the reference's "from ff_attention import FastForwardAttn" once the
    # package directory is on sys.path; raises ImportError if the extension is not built.
    from fastforwardattention_amd import FastForwardAttn as FFA

    batch_size, head_num, head_dim, prompt_len, output_len = 10, 32, 64, 1024, 128
    softmax_temp = 1 / sqrt(head_dim)
    dtype = getattr(torch, args.dtype)
    tol = 1e-3 if dtype == torch.float16 else 1e-6
    torch.manual_seed(0)
    K = torch.randn(batch_size, head_num, prompt_len, head_dim, dtype=dtype).cuda()
    V = torch.randn(batch_size, head_num, prompt_len, head_dim, dtype=dtype).cuda()

    total_sequence_length = prompt_len + output_len
    ffa = FFA(K, V, total_sequence_length, args.default_launch)

    BH = batch_size * head_num
    Kf = torch.zeros(BH, total_sequence_length, head_dim, device="cuda")
    Vf = torch.zeros(BH, total_sequence_length, head_dim, device="cuda")
    Kf[:, :prompt_len], Vf[:, :prompt_len] = K.float().view(BH, prompt_len, -1), V.float().view(BH, prompt_len, -1)
    worst, ms = 0.0, 0.0
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for i in range(output_len):
        new_token_k = torch.randn(batch_size, head_num, 1, head_dim, dtype=dtype).cuda()
        new_token_v = torch.randn(batch_size, head_num, 1, head_dim, dtype=dtype).cuda()
        new_token_q = torch.randn(batch_size, head_num, 1, head_dim, dtype=dtype).cuda()
        curr_timestep = prompt_len + i

        start.record()
        ffa_attn = ffa.attention(new_token_q, new_token_k, new_token_v, softmax_temp, curr_timestep, args.p)
        stop.record()

        Kf[:, curr_timestep], Vf[:, curr_timestep] = new_token_k.float().view(BH, -1), new_token_v.float().view(BH, -1)
        torch_attn = torch_attn_func(new_token_q.float().view(BH, 1, head_dim), Kf[:, :curr_timestep + 1],
                                     Vf[:, :curr_timestep + 1], softmax_temp)
        torch.cuda.synchronize()
        ms += start.elapsed_time(stop)
        worst = max(worst, float((torch_attn.view(batch_size, head_num, head_dim) - ffa_attn.float()).abs().max()))
    print(f"{output_len} steps, {args.dtype}, p={args.p}: worst max-abs difference {worst:.3g} "
          f"(tolerance {tol:g} for p=0), {ms * 1e3 / output_len:.1f} us per call incl. launch")
    if args.p == 0.0:
        assert worst <= tol, "decode attention differs from the fp32 evaluation"


if __name__ == "__main__":
    main()
