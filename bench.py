#!/usr/bin/env python3
"""Benchmark of the decode-attention hot path on ONE MI355X.

Headline workload (BASELINE.json configs[1], B = 10): OPT-1.3b-shaped iterative decode,
32 heads x 64, fp16, KV cache prefilled with a 1000-token prompt (N(0,1) * 0.5), then
t = 1000 -> 1255, fresh N(0,1) q/k/v, scale 1/8, p = 0.

A "step" is ONE decode-attention call: one layer's cache, one new token for the whole
batch.  OPT-1.3b has 24 layers, so the bench keeps 24 independent caches (2.5 GB) and step i
works on cache i % 24: consecutive steps never touch the same cache, as in a real decoder,
and the 103 MB of one cache cannot be served out of the 256 MB last-level cache.  Whatever
--steps K is, the K steps sample the WHOLE decode: t_i = prompt + (i * gen) // K, so K = 20
covers t = 1000 .. 1243 and the default K = 6144 is every (layer, token) of the 256-token
decode.  The sequence of K steps is repeated back to back until the timed region is at least
50 ms long; `ms_per_step` is the region divided by the launches in it.

Three timed legs over the same launches, each bracketed by torch.cuda.synchronize() and HIP
events recorded on the launch stream:
  graph   the launches captured once into a HIP graph and replayed (device-side rate, no
          host gaps); median of 5 replays -> `value`, `ms_per_step`, `roofline`
  capi    eager calls of ffa_attention_f16 through ctypes          -> `eager_capi_*`
  ext     eager calls of FastForwardAttn.attention (Python API)    -> `eager_ext_*`
plus `cpu_baseline`: the fp32 torch restatement of the reference's torch_attn_func on the
host cores, on a bounded sample of the same workload (and BASELINE configs[0] beside it),
and `suite`: short rows of the same measurement for the other BASELINE configurations
(other batch sizes, the long-sequence sweep with both launches, the GPT-J shape, the pruned
sweep); --no-suite leaves them out.

Prints ONE JSON line.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published

WORKLOADS = {
    # name: B, H, Dh, prompt, gen, scale, layers (independent caches), dtype
    "opt1.3b_b10": dict(B=10, H=32, Dh=64, prompt=1000, gen=256, scale=0.125, layers=24),
    "opt1.3b_b5": dict(B=5, H=32, Dh=64, prompt=1000, gen=256, scale=0.125, layers=24),
    "opt1.3b_b2": dict(B=2, H=32, Dh=64, prompt=1000, gen=256, scale=0.125, layers=24),
    "opt1.3b_b1": dict(B=1, H=32, Dh=64, prompt=1000, gen=256, scale=0.125, layers=24),
    "opt1.3b_b10_f32": dict(B=10, H=32, Dh=64, prompt=1000, gen=256, scale=0.125, layers=24, dtype="f32"),
    "opt2.7b_b10": dict(B=10, H=32, Dh=80, prompt=1000, gen=256, scale=80 ** -0.5, layers=32),
    "gptj_b8": dict(B=8, H=16, Dh=256, prompt=2000, gen=256, scale=0.0625, layers=8),
    "long_b1_16k": dict(B=1, H=32, Dh=64, prompt=16384 - 128, gen=128, scale=0.125, layers=24),
    "long_b1_8k": dict(B=1, H=32, Dh=64, prompt=8192 - 128, gen=128, scale=0.125, layers=24),
    "long_b1_4k": dict(B=1, H=32, Dh=64, prompt=4096 - 128, gen=128, scale=0.125, layers=24),
    "long_b1_2k": dict(B=1, H=32, Dh=64, prompt=2048 - 128, gen=128, scale=0.125, layers=24),
    "long_b1_1k": dict(B=1, H=32, Dh=64, prompt=1024 - 128, gen=128, scale=0.125, layers=24),
    # BASELINE configs[0] on the GPU: one fp32 step at t = 1000 (gen = 1: every launch is that step)
    "config1_f32_b1": dict(B=1, H=32, Dh=64, prompt=1000, gen=1, scale=0.125, layers=24, dtype="f32"),
}


def algorithmic_bytes(B, H, Dh, t, elem=2):
    """K and V cache reads of the t cached keys: 2*B*H*Dh*sizeof(T)*t."""
    return 2 * B * H * Dh * elem * t


class Workload:
    def __init__(self, name, use_default=False, plan_override=None, layers=None, steps=None):
        import torch
        from fastforwardattention_amd import capi
        self.torch, self.capi = torch, capi
        self.lib = capi.load()
        self.name = name
        w = WORKLOADS[name]
        self.B, self.H, self.Dh = w["B"], w["H"], w["Dh"]
        self.prompt, self.gen, self.scale, self.layers = w["prompt"], w["gen"], w["scale"], layers or w["layers"]
        self.Lmax = self.prompt + self.gen
        self.steps = steps or self.layers * self.gen     # launches per pass over the decode
        self.use_default = use_default
        self.plan_override = plan_override
        self.dtype = w.get("dtype", "f16")
        self.elem = 2 if self.dtype == "f16" else 4
        self.precision = 8 * self.elem
        self.tdtype = torch.float16 if self.dtype == "f16" else torch.float32
        self.fn_init = self.lib.ffa_init_cache_f16 if self.dtype == "f16" else self.lib.ffa_init_cache_f32
        self.fn_attn = self.lib.ffa_attention_f16 if self.dtype == "f16" else self.lib.ffa_attention_f32
        x, tdt = 16 // self.elem, self.tdtype
        dev = "cuda:0"
        # Every slot of the caches holds prompt-like data: a sampled schedule jumps over slots
        # that a step-by-step decode would have appended, and they must not hold garbage.
        B, H, Dh, L, Lmax = self.B, self.H, self.Dh, self.Lmax, self.Lmax
        g = torch.Generator(device=dev).manual_seed(0)
        self.kc, self.vc = [], []
        for _ in range(self.layers):
            K = (torch.randn(B, H, L, Dh, device=dev, generator=g) * 0.5).to(tdt)
            V = (torch.randn(B, H, L, Dh, device=dev, generator=g) * 0.5).to(tdt)
            kc = torch.empty(B, H, Dh // x, Lmax, x, dtype=tdt, device=dev)
            vc = torch.empty(B, H, Lmax, Dh, dtype=tdt, device=dev)
            capi.check(self.fn_init(kc.data_ptr(), vc.data_ptr(), K.data_ptr(), V.data_ptr(),
                                    B, L, Lmax, Dh, H, None), "ffa_init_cache")
            torch.cuda.synchronize()
            self.kc.append(kc)
            self.vc.append(vc)
            del K, V
        # a ring of fresh q/k/v tokens (N(0,1)), resident in HBM before the timed region
        self.ring = 64
        self.q = torch.randn(self.ring, B, H, Dh, device=dev, generator=g).to(tdt)
        self.k = torch.randn(self.ring, B, H, Dh, device=dev, generator=g).to(tdt)
        self.v = torch.randn(self.ring, B, H, Dh, device=dev, generator=g).to(tdt)
        self.out = torch.empty(self.ring, B, H, Dh, dtype=tdt, device=dev)
        nbytes = self.lib.ffa_workspace_bytes(B, H, Dh, Lmax)
        self.ws = torch.zeros(nbytes, dtype=torch.uint8, device=dev)
        self.ws_bytes = nbytes
        self._plans = {}
        self.transform = None     # a capi.TokenTransform: the step then goes through ffa_attention_ex
        torch.cuda.synchronize()

    @staticmethod
    def describe(name):
        """Shape of a workload without its device buffers (for the CPU baseline)."""
        from types import SimpleNamespace
        w = WORKLOADS[name]
        return SimpleNamespace(name=name, B=w["B"], H=w["H"], Dh=w["Dh"], prompt=w["prompt"], gen=w["gen"],
                               scale=w["scale"], Lmax=w["prompt"] + w["gen"])

    def t_of(self, i):
        """Cached keys at launch i: the `steps` launches of a pass sample the whole decode."""
        return self.prompt + ((i % self.steps) * self.gen) // self.steps

    def plan_for(self, t):
        p = self._plans.get(t)
        if p is None:
            if self.plan_override is not None:
                kind, waves, tps = self.plan_override[:3]
                combine = self.plan_override[3] if len(self.plan_override) > 3 else 0
                whole = self.plan_override[4] if len(self.plan_override) > 4 else 0
                ntiles = t // 64 + 1
                ns = 1 if kind == self.capi.FFA_LAUNCH_WORKGROUP else -(-ntiles // tps)
                p = self.capi.make_plan(kind, waves, ns, ntiles if ns == 1 and kind == 0 else tps, combine,
                                        whole)
            else:
                p = self.capi.plan_launch(self.precision, self.B, self.H, self.Dh, t, 0.0, self.use_default,
                                          self.lib.ffa_device_compute_units())
            self._plans[t] = p
        return p

    def launch(self, i, stream_ptr):
        """One step through the C ABI (no allocation, no sync)."""
        t = self.t_of(i)
        r, l = i % self.ring, i % self.layers
        if self.transform is not None:
            rc = self.lib.ffa_attention_ex(
                self.precision, self.B, self.H, self.Dh, self.Lmax, self.scale, t,
                self.q[r].data_ptr(), self.k[r].data_ptr(), self.v[r].data_ptr(),
                self.kc[l].data_ptr(), self.vc[l].data_ptr(), self.out[r].data_ptr(), None, 0.0,
                C.byref(self.plan_for(t)), 1, C.byref(self.transform), None, self.ws.data_ptr(), self.ws_bytes,
                stream_ptr)
            if rc != 0:
                raise RuntimeError(f"ffa_attention_ex failed: {self.capi.status_string(rc)}")
            return
        rc = self.fn_attn(
            self.B, self.H, self.Dh, self.Lmax, self.scale, t,
            self.q[r].data_ptr(), self.k[r].data_ptr(), self.v[r].data_ptr(),
            self.kc[l].data_ptr(), self.vc[l].data_ptr(), self.out[r].data_ptr(), None, 0.0,
            C.byref(self.plan_for(t)), 1, self.ws.data_ptr(), self.ws_bytes, stream_ptr)
        if rc != 0:
            raise RuntimeError(f"ffa_attention failed: {self.capi.status_string(rc)}")

    def floor_plan(self, t):
        """The step's plan as the load-floor probe takes it (split launch, one lane per key, 2 / 4 / 8
        waves: the same grid and bytes), or None when the step is not a split launch."""
        p = self.plan_for(t)
        if p.kind != self.capi.FFA_LAUNCH_SPLIT:
            return None
        waves = min((2, 4, 8), key=lambda w: abs(w - p.waves_per_wg))
        return self.capi.make_plan(p.kind, waves, p.n_splits, p.tiles_per_split, 0, p.whole_heads)

    def launch_floor(self, i, stream_ptr):
        """The load floor of step i: same grid, same loads, nothing else (ffa_load_floor)."""
        t = self.t_of(i)
        l = i % self.layers
        rc = self.lib.ffa_load_floor(self.precision, self.B, self.H, self.Dh, self.Lmax, t, self.kc[l].data_ptr(),
                                     self.vc[l].data_ptr(), None, 1, C.byref(self.floor_plan(t)),
                                     self.out.data_ptr(), stream_ptr)
        if rc != 0:
            raise RuntimeError(f"ffa_load_floor failed: {self.capi.status_string(rc)}")

    def mean_bytes(self, launches=None):
        n = launches or self.steps
        return sum(algorithmic_bytes(self.B, self.H, self.Dh, self.t_of(i), self.elem) for i in range(n)) / n

    def t_range(self):
        ts = [self.t_of(i) for i in range(self.steps)]
        return min(ts), max(ts)


def time_region(torch, fn):
    """fn() enqueues work on the current stream; returns elapsed ms between HIP events."""
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1)


MIN_REGION_MS = 50.0


def launches_for(wl, steps, warmup):
    """Launches in one timed region: whole passes over the `steps`-launch schedule, enough of
    them for MIN_REGION_MS at the rate the warm-up launches ran at."""
    torch = wl.torch
    sp = torch.cuda.current_stream().cuda_stream
    n = max(warmup, 8)
    for i in range(n):
        wl.launch(i, sp)
    torch.cuda.synchronize()
    ms = time_region(torch, lambda: [wl.launch(i, sp) for i in range(n)])
    passes = max(1, int(-(-MIN_REGION_MS * 1.2 // (ms / n * steps))))
    return steps * passes


def run_graph(wl, launches, replays=5, floor=False):
    """Returns the per-replay times (ms) of a graph holding `launches` launches (floor: of the
    load-floor probe of each step instead of the step itself)."""
    torch = wl.torch
    if floor:
        import types
        wl = types.SimpleNamespace(torch=torch, layers=wl.layers, launch=wl.launch_floor)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):          # warm-up on the capture stream, eager
        for i in range(min(launches, 2 * wl.layers)):
            wl.launch(i, side.cuda_stream)
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        sp = torch.cuda.current_stream().cuda_stream
        for i in range(launches):
            wl.launch(i, sp)
    graph.replay()                          # one untimed replay
    torch.cuda.synchronize()
    return [time_region(torch, graph.replay) for _ in range(replays)]


def median(xs):
    xs = sorted(xs)
    n = len(xs)
    return xs[n // 2] if n % 2 else 0.5 * (xs[n // 2 - 1] + xs[n // 2])


def run_capi(wl, launches):
    torch = wl.torch
    sp = torch.cuda.current_stream().cuda_stream
    for i in range(min(launches, 2 * wl.layers)):
        wl.launch(i, sp)

    def body():
        for i in range(launches):
            wl.launch(i, sp)
    return time_region(torch, body)


def run_ext(wl, launches):
    """The Python API on one object per layer, built over the same caches."""
    torch = wl.torch
    from fastforwardattention_amd import FastForwardAttn
    B, H, Dh = wl.B, wl.H, wl.Dh
    dummy = torch.zeros(B, H, 1, Dh, dtype=wl.tdtype, device="cuda:0")
    obj = FastForwardAttn(dummy, dummy, wl.Lmax, wl.use_default)  # its own caches are unused
    def step(i):
        r, l = i % wl.ring, i % wl.layers
        return obj.attention(wl.q[r], wl.k[r], wl.v[r], wl.kc[l], wl.vc[l], wl.scale, wl.t_of(i), 0.0)
    for i in range(min(launches, 2 * wl.layers)):
        step(i)

    def body():
        for i in range(launches):
            step(i)
    return time_region(torch, body)


def parity_check(wl):
    """The workload's whole decode loop on one layer cache, untimed: kernel output through the
    C ABI (the library's own launch plan at every step) against fp32 torch on the GPU
    (softmax(q K^T scale) V over the upcast inputs).  Returns the worst max-abs error; the
    tolerance is 1e-3 for fp16 inputs and 1e-6 for fp32 inputs."""
    torch, capi, lib = wl.torch, wl.capi, wl.lib
    B, H, Dh, L, Lmax, gen = wl.B, wl.H, wl.Dh, wl.prompt, wl.Lmax, wl.gen
    dev, tdt, x = "cuda:0", wl.tdtype, 16 // wl.elem
    tol = 1e-3 if wl.dtype == "f16" else 1e-6
    g = torch.Generator(device=dev).manual_seed(1)
    K = (torch.randn(B, H, L, Dh, device=dev, generator=g) * 0.5).to(tdt)
    V = (torch.randn(B, H, L, Dh, device=dev, generator=g) * 0.5).to(tdt)
    kc = torch.empty(B, H, Dh // x, Lmax, x, dtype=tdt, device=dev)
    vc = torch.empty(B, H, Lmax, Dh, dtype=tdt, device=dev)
    capi.check(wl.fn_init(kc.data_ptr(), vc.data_ptr(), K.data_ptr(), V.data_ptr(), B, L, Lmax, Dh, H, None),
               "ffa_init_cache")
    Kf = torch.zeros(B * H, Lmax, Dh, device=dev)
    Vf = torch.zeros(B * H, Lmax, Dh, device=dev)
    Kf[:, :L], Vf[:, :L] = K.float().reshape(B * H, L, Dh), V.float().reshape(B * H, L, Dh)
    out = torch.empty(B, H, Dh, dtype=tdt, device=dev)
    worst = 0.0
    for i in range(gen):
        t = L + i
        q, k, v = (torch.randn(B, H, Dh, device=dev, generator=g).to(tdt) for _ in range(3))
        plan = wl.plan_for(t)
        capi.check(wl.fn_attn(B, H, Dh, Lmax, wl.scale, t, q.data_ptr(), k.data_ptr(), v.data_ptr(),
                              kc.data_ptr(), vc.data_ptr(), out.data_ptr(), None, 0.0, C.byref(plan), 1,
                              wl.ws.data_ptr(), wl.ws_bytes, None), "ffa_attention")
        Kf[:, t], Vf[:, t] = k.float().reshape(B * H, Dh), v.float().reshape(B * H, Dh)
        w = torch.softmax(torch.bmm(q.float().reshape(B * H, 1, Dh), Kf[:, :t + 1].transpose(1, 2)) * wl.scale, -1)
        ref = torch.bmm(w, Vf[:, :t + 1]).reshape(B, H, Dh)
        worst = max(worst, float((out.float() - ref).abs().max()))
    return {"max_abs_err": worst, "tolerance": tol, "steps": gen, "ok": worst <= tol,
            "reference": "fp32 torch bmm/softmax/bmm on the GPU over the upcast inputs, every step"}


def cpu_baseline(wl, budget_s=12.0, max_steps=40000):
    """The reference's CPU path restated (oracle/torch_attn.py) on the host cores, on the same
    workload (one layer's cache): passes over the decode loop t = prompt .. prompt+gen-1 are
    repeated until about `budget_s` seconds of CPU work have been timed."""
    import torch
    from oracle.torch_attn import CpuDecodeBaseline
    B, H, Dh, L = wl.B, wl.H, wl.Dh, wl.prompt
    g = torch.Generator().manual_seed(0)
    nlayers = 4      # independent caches used round-robin, like the layers of the GPU legs
    bases = []
    for _ in range(nlayers):
        K = torch.randn(B, H, L, Dh, generator=g) * 0.5
        V = torch.randn(B, H, L, Dh, generator=g) * 0.5
        bases.append(CpuDecodeBaseline(K, V, wl.Lmax))
    del K, V
    base = bases[0]
    toks = [tuple(torch.randn(B, H, Dh, generator=g) for _ in range(3)) for _ in range(8)]
    span = max(1, wl.gen - 4)
    for i in range(3):
        q, k, v = toks[i % 8]
        base.attention(q, k, v, wl.scale, L + i)
    times, t0 = [], time.perf_counter()
    i = 0
    while i < max_steps and (time.perf_counter() - t0) < budget_s:
        q, k, v = toks[i % 8]
        s = time.perf_counter()
        bases[i % nlayers].attention(q, k, v, wl.scale, L + 3 + (i // nlayers) % span)
        times.append(time.perf_counter() - s)
        i += 1
    mean_s = sum(times) / len(times)
    per_layer = -(-len(times) // nlayers)
    t_mid = L + 3 + (min(per_layer, span) - 1) // 2
    gbs = algorithmic_bytes(B, H, Dh, t_mid, elem=4) / mean_s / 1e9
    # the same steps on one thread (a few of them: bounded at ~3 s)
    nthreads = torch.get_num_threads()
    torch.set_num_threads(1)
    one, t0 = [], time.perf_counter()
    while len(one) < 8 and (time.perf_counter() - t0) < 3.0:
        q, k, v = toks[len(one) % 8]
        s = time.perf_counter()
        base.attention(q, k, v, wl.scale, L + 3 + len(one))
        one.append(time.perf_counter() - s)
    torch.set_num_threads(nthreads)
    one_s = sum(one) / len(one)
    return {
        "value": round(gbs, 3), "unit": "GB/s", "cores": torch.get_num_threads(),
        "host_cpus": os.cpu_count(), "kind": "port",
        "us_per_step": round(mean_s * 1e6, 1),
        "one_thread": {"value": round(algorithmic_bytes(B, H, Dh, t_mid, elem=4) / one_s / 1e9, 3), "unit": "GB/s",
                       "us_per_step": round(one_s * 1e6, 1), "steps": len(one)},
        "sample": (f"{len(times)} decode steps of {wl.name} ({nlayers} layer caches round-robin, "
                   f"t={L + 3}..{L + 2 + min(-(-len(times) // nlayers), span)}"
                   f"{', repeated' if len(times) > span * nlayers else ''}; {sum(times):.1f} s of CPU work), "
                   "fp32 torch bmm/softmax/bmm over a pre-allocated cache; bytes counted at 4 B/element"),
        "config1": cpu_baseline_config1(),
        "small_batches": cpu_baseline_small_batches(wl),
    }


def cpu_baseline_small_batches(wl, budget_s=1.5):
    """The same CPU decode loop at the workload's shape with B = 1, 2, 5 (the other batch sizes of
    BASELINE configs[1]): at least 16 steps each, about `budget_s` seconds of CPU work per batch."""
    import torch
    from oracle.torch_attn import CpuDecodeBaseline
    H, Dh, L = wl.H, wl.Dh, wl.prompt
    out = []
    for B in (1, 2, 5):
        g = torch.Generator().manual_seed(B)
        base = CpuDecodeBaseline(torch.randn(B, H, L, Dh, generator=g) * 0.5, torch.randn(B, H, L, Dh, generator=g) * 0.5,
                                 wl.Lmax)
        toks = [tuple(torch.randn(B, H, Dh, generator=g) for _ in range(3)) for _ in range(4)]
        span = max(1, wl.gen - 4)
        for i in range(3):
            base.attention(*toks[i % 4], wl.scale, L + i)
        times, t0 = [], time.perf_counter()
        while len(times) < 16 or (time.perf_counter() - t0 < budget_s and len(times) < 20000):
            s = time.perf_counter()
            base.attention(*toks[len(times) % 4], wl.scale, L + 3 + len(times) % span)
            times.append(time.perf_counter() - s)
        mean_s = sum(times) / len(times)
        t_mid = L + 3 + (min(len(times), span) - 1) // 2
        out.append({"B": B, "us_per_step": round(mean_s * 1e6, 1), "steps": len(times),
                    "GBps": round(algorithmic_bytes(B, H, Dh, t_mid, elem=4) / mean_s / 1e9, 2),
                    "threads": torch.get_num_threads()})
    return out


def cpu_baseline_config1(budget_s=2.0):
    """BASELINE configs[0] on the host cores: one decode-attention step, B=1, 32 heads x 64,
    fp32, t=1000, seeded N(0,1), scale 1/8, p=0, through the restated torch_attn_func."""
    import torch
    from oracle.torch_attn import torch_attn_func
    torch.manual_seed(0)
    q = torch.randn(32, 1, 64)
    K, V = torch.randn(32, 1001, 64), torch.randn(32, 1001, 64)     # cache + the new token
    for _ in range(5):
        torch_attn_func(q, K, V, 0.125)
    times, t0 = [], time.perf_counter()
    while time.perf_counter() - t0 < budget_s:
        s = time.perf_counter()
        torch_attn_func(q, K, V, 0.125)
        times.append(time.perf_counter() - s)
    us = 1e6 * sum(times) / len(times)
    return {"workload": "configs[0]: B=1 H=32 Dh=64 fp32 t=1000 scale=0.125 p=0, torch_attn_func on CPU",
            "us_per_step": round(us, 1), "GBps": round(algorithmic_bytes(1, 32, 64, 1000, 4) / us / 1e3, 2),
            "threads": torch.get_num_threads(), "calls": len(times)}


class PrunedWorkload:
    """BASELINE.json configs[4]: B=16, 32x64, fp16, 8192 cached keys, 64 decode steps,
    peaked keys: per head 32 random positions hold 4*q_dir + N(0, 0.1), the rest N(0,1);
    V is N(0,1).  The query is held fixed per head over the 64 steps (the peaks are built
    for it once); k and v of the new token are fresh N(0,1) draws."""

    def __init__(self, B=16, H=32, Dh=64, L=8192, gen=64, kind="library"):
        import torch
        self.kind = kind
        from fastforwardattention_amd import capi
        self.torch, self.capi, self.lib = torch, capi, capi.load()
        self.B, self.H, self.Dh, self.L, self.gen, self.Lmax = B, H, Dh, L, gen, L + gen
        self.scale = 0.125
        dev = "cuda:0"
        g = torch.Generator(device=dev).manual_seed(0)
        q = torch.randn(B, H, Dh, device=dev, generator=g)
        qdir = q / q.norm(dim=-1, keepdim=True)
        K = torch.randn(B, H, L, Dh, device=dev, generator=g)
        pos = torch.rand(B, H, L, device=dev, generator=g).argsort(dim=-1)[:, :, :32]      # 32 distinct positions
        peaks = 4 * qdir[:, :, None, :] + 0.1 * torch.randn(B, H, 32, Dh, device=dev, generator=g)
        K.scatter_(2, pos[..., None].expand(-1, -1, -1, Dh), peaks)
        K = K.half()
        V = torch.randn(B, H, L, Dh, device=dev, generator=g).half()
        self.kc = torch.empty(B, H, Dh // 8, self.Lmax, 8, dtype=torch.float16, device=dev)
        self.vc = torch.empty(B, H, self.Lmax, Dh, dtype=torch.float16, device=dev)
        capi.check(self.lib.ffa_init_cache_f16(self.kc.data_ptr(), self.vc.data_ptr(), K.data_ptr(), V.data_ptr(),
                                               B, L, self.Lmax, Dh, H, None), "ffa_init_cache_f16")
        torch.cuda.synchronize()
        del K, V
        self.q = q.half()
        self.k = torch.randn(gen, B, H, Dh, device=dev, generator=g).half()
        self.v = torch.randn(gen, B, H, Dh, device=dev, generator=g).half()
        self.out = torch.empty(gen, B, H, Dh, dtype=torch.float16, device=dev)
        nbytes = self.lib.ffa_workspace_bytes(B, H, Dh, self.Lmax)
        self.ws = torch.zeros(nbytes, dtype=torch.uint8, device=dev)
        self.kept = torch.zeros(B, H, dtype=torch.int32, device=dev)
        torch.cuda.synchronize()

    def plan_for(self, t, p):
        capi = self.capi
        cus = self.lib.ffa_device_compute_units()
        if self.kind == "library":
            return capi.plan_launch(16, self.B, self.H, self.Dh, t, p, False, cus)
        ntiles = t // 64 + 1
        if self.kind == "workgroup":
            return capi.make_plan(capi.FFA_LAUNCH_WORKGROUP, 16, 1, ntiles)
        n = max(1, min(cus // (self.B * self.H), ntiles // 4))      # "two_pass"
        tps = -(-ntiles // n)
        return capi.make_plan(capi.FFA_LAUNCH_TWO_PASS, 4, -(-ntiles // tps), tps)

    def launch(self, i, p, stream_ptr, diag=False):
        t = self.L + i % self.gen
        plan = self.plan_for(t, p)
        rc = self.lib.ffa_attention_diag(
            16, self.B, self.H, self.Dh, self.Lmax, self.scale, t, self.q.data_ptr(),
            self.k[i % self.gen].data_ptr(), self.v[i % self.gen].data_ptr(), self.kc.data_ptr(),
            self.vc.data_ptr(), self.out[i % self.gen].data_ptr(), None, p,
            None if (diag and plan.kind == self.capi.FFA_LAUNCH_SPLIT) else C.byref(plan), 1,
            self.ws.data_ptr(), self.ws.numel(),
            self.kept.data_ptr() if diag else None, None, stream_ptr)
        if rc != 0:
            raise RuntimeError(f"ffa_attention_diag failed: {self.capi.status_string(rc)}")
        return plan

    def run(self, p, steps=320, warmup=8):
        # Timed as replays of a HIP graph holding the `steps` launches, like the headline: at
        # B = 1 a pruned step is two short kernels and eager launches from Python cannot keep up.
        torch = self.torch
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for i in range(warmup):
                plan = self.launch(i, p, side.cuda_stream)
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            sp = torch.cuda.current_stream().cuda_stream
            for i in range(steps):
                self.launch(i, p, sp)
        graph.replay()
        torch.cuda.synchronize()
        ms = median([time_region(torch, graph.replay) for _ in range(3)])
        sp = torch.cuda.current_stream().cuda_stream
        out_p = self.out.clone()
        # skip fraction at the last step (diagnostic launch, untimed)
        self.launch(steps - 1, p, sp, diag=True)
        torch.cuda.synchronize()
        t_last = self.L + (steps - 1) % self.gen
        skip_frac = 1.0 - float(self.kept.sum().item()) / (self.B * self.H * t_last)
        return ms * 1e3 / steps, skip_frac, out_p, plan


def run_pruned_sweep(B=16, kind="library"):
    """kind: "library" = the planner's choice; "workgroup" / "two_pass" force that launch kind
    (p = 0 included, so the two pruning-capable paths can be compared like for like)."""
    wl = PrunedWorkload(B=B, kind=kind)
    res = []
    ref = None
    bytes_full = sum(algorithmic_bytes(wl.B, wl.H, wl.Dh, wl.L + i) for i in range(wl.gen)) / wl.gen
    for p in (0.0, 1e-4, 1e-3, 1e-2, 5e-2, 0.2):     # the last two skip 87 % and 99 % of the rows: where pruning breaks even
        us, skip, out, plan = wl.run(p)
        if ref is None:
            ref = out
        err = float((out.float() - ref.float()).abs().max().item())
        actual = bytes_full * (1.0 - 0.5 * skip)
        res.append({"p": p, "us_per_step": round(us, 2), "skip_fraction": round(skip, 5),
                    "max_abs_vs_p0": err, "effective_GBps": round(bytes_full / us / 1e3, 1),
                    "actual_GBps": round(actual / us / 1e3, 1), "plan": repr(plan)})
    return {"workload": f"pruned sweep: B={B} H=32 Dh=64 fp16, 8192 cached keys, 64 steps, 32 peaked keys/head, "
                        "query fixed per head", "launch": kind, "algorithmic_bytes_per_step": round(bytes_full),
            "results": res}


def run_pruned_sweeps():
    for B, kind in ((16, "library"), (16, "workgroup"), (16, "two_pass"), (4, "library"), (1, "library"), (1, "workgroup")):
        print(json.dumps(run_pruned_sweep(B, kind)), flush=True)
        import torch
        torch.cuda.empty_cache()


def run_init_cache_bench():
    """Cache construction (ffa_init_cache_f16) at the BASELINE shapes: reads K, V [B,H,L,Dh] and
    writes both cache layouts, 4*B*H*L*Dh*sizeof(T) bytes per call.  Source and destination sets
    rotate so that no call finds its data in the 256 MB last-level cache."""
    import torch
    from fastforwardattention_amd import capi
    lib = capi.load()
    res = []
    for name, (B, H, Dh, L, gen) in {"opt1.3b_b10": (10, 32, 64, 1000, 256), "gptj_b8": (8, 16, 256, 2000, 256),
                                     "pruned_b16_8k": (16, 32, 64, 8192, 64)}.items():
        Lmax = L + gen
        per_call = 4 * B * H * L * Dh * 2
        nsets = max(2, int(1.5e9 // per_call) + 1)
        src = [(torch.randn(B, H, L, Dh, device="cuda:0", dtype=torch.float16),
                torch.randn(B, H, L, Dh, device="cuda:0", dtype=torch.float16)) for _ in range(nsets)]
        dst = [(torch.empty(B, H, Dh // 8, Lmax, 8, device="cuda:0", dtype=torch.float16),
                torch.empty(B, H, Lmax, Dh, device="cuda:0", dtype=torch.float16)) for _ in range(nsets)]
        sp = torch.cuda.current_stream().cuda_stream

        def body(n):
            for i in range(n):
                (ks, vs), (kd, vd) = src[i % nsets], dst[i % nsets]
                capi.check(lib.ffa_init_cache_f16(kd.data_ptr(), vd.data_ptr(), ks.data_ptr(), vs.data_ptr(),
                                                  B, L, Lmax, Dh, H, sp), "ffa_init_cache_f16")
        body(nsets)
        reps = 4 * nsets
        us = time_region(torch, lambda: body(reps)) * 1e3 / reps
        res.append({"workload": name, "shape": [B, H, L, Dh], "max_len": Lmax, "bytes_per_call": per_call,
                    "us_per_call": round(us, 2), "GBps": round(per_call / us / 1e3, 1),
                    "hbm_frac": round(per_call / us / 1e3 / HBM_PEAK_GBS, 4)})
        del src, dst
        torch.cuda.empty_cache()
    return {"kernel": "ffa_init_cache_kernel (cache construction, fp16)", "results": res}


def run_hf_end_to_end(family="opt", B=None, prompt=None, new_tokens=128):
    """The reference's end-to-end setting in miniature (summarize.py: a left-padded batch, greedy
    decoding): an OPT-1.3b-shaped or GPT-J-6B-shaped model with random weights (nothing is
    downloaded), `new_tokens` decode steps; wall time per generated token with transformers' own
    cache and attention against the FFACache hook (for GPT-J with the rotary embedding of the new
    token inside the engine's call and, as the reference does it, in torch).  Reported beside the
    kernel figures; the projections and MLPs of the model dominate a decode step, the attention
    call is what changes."""
    import torch
    import transformers
    from fastforwardattention_amd import hf
    beams = 1
    if family == "opt-beams":            # beam search: 2 prompts x 5 beams = the 10 rows of the headline batch
        family, beams, B = "opt", 5, B or 2
    if family == "opt":
        B, prompt = B or 10, prompt or 1000
        cfg = transformers.OPTConfig(vocab_size=50272, hidden_size=2048, num_hidden_layers=24, ffn_dim=8192,
                                     num_attention_heads=32, max_position_embeddings=2048, word_embed_proj_dim=2048,
                                     dropout=0.0, attention_dropout=0.0)
        build, label = transformers.OPTForCausalLM, "OPT-1.3b-shaped"
    else:
        B, prompt = B or 8, prompt or 2000
        cfg = transformers.GPTJConfig(vocab_size=50400, n_positions=4096, n_embd=4096, n_layer=28, n_head=16,
                                      rotary_dim=64, resid_pdrop=0.0, embd_pdrop=0.0, attn_pdrop=0.0)
        build, label = transformers.GPTJForCausalLM, "GPT-J-6B-shaped"
    torch.manual_seed(0)
    with torch.device("cuda:0"):
        model = build(cfg).half().eval()
    g = torch.Generator(device="cuda:0").manual_seed(0)
    ids = torch.randint(4, 50000, (B, prompt), device="cuda:0", generator=g)
    mask = torch.ones_like(ids)
    mask[1::2, :37] = 0                      # every other sample is left-padded by 37 tokens
    kw = dict(attention_mask=mask, max_new_tokens=new_tokens, min_new_tokens=new_tokens, do_sample=False,
              pad_token_id=1, eos_token_id=None)
    if beams > 1:
        kw.update(num_beams=beams, length_penalty=0.0)

    def per_token(run):
        """ms per generated token, the prompt pass excluded: (n tokens) - (1 token)."""
        with torch.no_grad():
            run(4)
            torch.cuda.synchronize()
            t0 = time.perf_counter(); run(1); torch.cuda.synchronize()
            t1 = time.perf_counter(); out = run(new_tokens); torch.cuda.synchronize()
            t2 = time.perf_counter()
        return out, ((t2 - t1) - (t1 - t0)) * 1e3 / (new_tokens - 1)

    res, ref_out = {}, None
    for impl in (("sdpa", "eager") if family == "opt" else ("eager",)):
        model.config._attn_implementation = impl
        ref_out, ms = per_token(lambda n: model.generate(ids, **{**kw, "max_new_tokens": n, "min_new_tokens": n}))
        res[f"transformers_{impl}_ms_per_token"] = round(ms, 3)
    outs = {}
    variants = [("ffa_tuned", False, True), ("ffa_default_launch", True, True)]
    if family != "opt":
        variants.append(("ffa_tuned_rotary_in_torch", False, False))
    for name, default, fused in variants:
        hf.enable(model, fused_rotary=fused)
        # a cache object serves one generate() call: build a new one per call
        outs[name], ms = per_token(lambda n: model.generate(
            ids, **{**kw, "max_new_tokens": n, "min_new_tokens": n},
            past_key_values=hf.FFACache(max_new_tokens=n, use_default_kernel_launch=default, num_beams=beams)))
        res[f"{name}_ms_per_token"] = round(ms, 3)
        hf.disable(model)
    res["same_tokens_as_transformers_eager"] = bool(torch.equal(outs["ffa_tuned"], ref_out))
    res["matching_token_fraction"] = round(float((outs["ffa_tuned"] == ref_out).double().mean().item()), 6)
    how = "greedy" if beams == 1 else f"beam-search (num_beams={beams}, {B * beams} cache rows)"
    return {"workload": f"{label} random model, fp16, B={B}, prompt {prompt} (odd samples left-padded by 37), "
                        f"{new_tokens} {how} tokens; per-token time excludes the prompt pass", **res}


def measure_row(name, use_default=False, steps=32, eager=True, rotary_dim=0):
    """One short row of the headline measurement for another workload: `steps` launches that
    sample its whole decode, repeated to a region of at least MIN_REGION_MS; graph replay
    (median of 5) and, beside it, the eager C-ABI leg.  With `rotary_dim` the step carries the
    rotary embedding of the new token (ffa_attention_ex); the plain step is timed beside it, the
    two alternating, and the row reports both."""
    import torch
    wl = Workload(name, use_default=use_default, steps=steps)
    n = launches_for(wl, steps, 16)
    if rotary_dim:
        from fastforwardattention_amd import capi
        tt, both = capi.TokenTransform(None, None, None, rotary_dim, 0.0), {False: [], True: []}
        for _ in range(3):
            for on in (False, True):
                wl.transform = tt if on else None
                both[on].append(median(run_graph(wl, n, replays=3)) * 1e3 / n)
        plain_us, us = median(both[False]), median(both[True])
        mb = wl.mean_bytes()
        row = {"workload": name, "token_transform": f"rotary embedding over {rotary_dim} of {wl.Dh} dims", "B": wl.B,
               "H": wl.H, "Dh": wl.Dh, "dtype": wl.dtype, "t_range": list(wl.t_range()), "timed_launches": n,
               "us_per_step": round(us, 2), "plain_us_per_step": round(plain_us, 2),
               "transform_costs_us": round(us - plain_us, 2), "GBps": round(mb / us / 1e3, 1)}
        del wl
        torch.cuda.empty_cache()
        return row
    us = median(run_graph(wl, n)) * 1e3 / n
    mb = wl.mean_bytes()
    row = {"workload": name, "use_default_kernel_launch": use_default, "B": wl.B, "H": wl.H, "Dh": wl.Dh,
           "dtype": wl.dtype, "t_range": list(wl.t_range()), "timed_launches": n, "us_per_step": round(us, 2),
           "GBps": round(mb / us / 1e3, 1), "hbm_frac": round(mb / us / 1e3 / HBM_PEAK_GBS, 4),
           "plan": repr(wl.plan_for(wl.t_of(0)))}
    if eager:
        row["eager_capi_us_per_step"] = round(run_capi(wl, n) * 1e3 / n, 2)
    if not use_default and all(wl.floor_plan(wl.t_of(i)) is not None for i in range(steps)):
        # The same launches with every load and nothing else: what this launch shape could reach
        # with free arithmetic and free merges.
        fl = median(run_graph(wl, n, floor=True)) * 1e3 / n
        row["load_floor_us_per_step"] = round(fl, 2)
        row["of_load_floor"] = round(fl / us, 3)
    del wl
    torch.cuda.empty_cache()
    return row


SUITE_ROWS = [  # (workload, also with the default launch)
    ("opt1.3b_b5", True), ("opt1.3b_b2", True), ("opt1.3b_b1", True),
    ("long_b1_1k", True), ("long_b1_2k", True), ("long_b1_4k", True), ("long_b1_8k", True), ("long_b1_16k", True),
    ("gptj_b8", True), ("config1_f32_b1", False), ("opt1.3b_b10_f32", False), ("opt2.7b_b10", False),
]


TRANSFORM_ROWS = [("gptj_b8", 64), ("opt1.3b_b10", 32), ("opt1.3b_b1", 32), ("long_b1_4k", 32)]  # workload, rotary dims


def run_transform_rows():
    """The step with the new token's rotary embedding inside the launch, beside the plain step."""
    return [measure_row(name, rotary_dim=rd) for name, rd in TRANSFORM_ROWS]


def run_suite_rows(full=False):
    """The other BASELINE configurations, same method as the headline line, short rows."""
    rows = []
    for name, with_default in SUITE_ROWS:
        rows.append(measure_row(name))
        if with_default:
            rows.append(measure_row(name, use_default=True, eager=False))
    rows.extend(run_transform_rows())
    sweep = run_pruned_sweep(16, "library")
    rows.append(sweep)
    rows.append(run_pruned_sweep(1, "library"))
    if full:
        for B, kind in ((16, "workgroup"), (16, "two_pass"), (1, "workgroup")):
            rows.append(run_pruned_sweep(B, kind))
        rows.append(run_init_cache_bench())
    return rows


def run_suite(args):
    """Every BASELINE configuration that fits one GPU, one JSON object per line."""
    for row in run_suite_rows(full=True):
        print(json.dumps(row), flush=True)


# ---------------------------------------------------------------------------------------------
# Launch-plan sweep: measures candidate launches at the BASELINE shapes and writes the table of
# overrides that the planner compiles in (fastforwardattention_amd/csrc/ffa_plan_table.inc).
SWEEP_SHAPES = [
    # precision, B, H, Dh, p, max_len (the BASELINE configuration's own), cached-key counts t that are timed
    (16, 10, 32, 64, 0.0, 1256, [1000, 1064, 1128, 1192, 1255]),
    (16, 5, 32, 64, 0.0, 1256, [1000, 1128, 1255]),
    (16, 2, 32, 64, 0.0, 1256, [1000, 1128, 1255]),
    (16, 1, 32, 64, 0.0, 1256, [1000, 1128, 1255]),
    (16, 1, 32, 64, 0.0, 1024, [896, 960]),
    (16, 1, 32, 64, 0.0, 2048, [1920, 1984, 2047]),
    (16, 1, 32, 64, 0.0, 4096, [3968, 4032, 4095]),
    (16, 1, 32, 64, 0.0, 8192, [8064, 8128, 8191]),
    (16, 1, 32, 64, 0.0, 16384, [16256, 16320, 16383]),
    (16, 8, 16, 256, 0.0, 2256, [2000, 2128, 2255]),
    (16, 16, 32, 64, 0.0, 8256, [8192, 8255]),
    (16, 10, 32, 80, 0.0, 1256, [1000, 1128, 1255]),
    (32, 10, 32, 64, 0.0, 1256, [1000, 1128, 1255]),
    (32, 1, 32, 64, 0.0, 1001, [1000]),
    (16, 16, 32, 64, 1e-3, 8256, [8192, 8255]),
    (16, 1, 32, 64, 1e-3, 8256, [8192, 8255]),
]
SWEEP_MARGIN = 0.97   # a candidate replaces the rules' plan only when it is more than 3 % faster


class SweepShape:
    """Device buffers for one (precision, B, H, Dh): enough independent caches (>= 1.5 GB in all)
    that no launch finds its data in the last-level cache.  For p > 0 the keys are peaked as in
    BASELINE configs[4] (32 positions per head hold 4*q_dir + N(0, 0.1)) and q is fixed."""

    def __init__(self, prec, B, H, Dh, p, max_len):
        import torch
        from fastforwardattention_amd import capi
        self.torch, self.capi, self.lib = torch, capi, capi.load()
        self.prec, self.B, self.H, self.Dh, self.p = prec, B, H, Dh, p
        self.Lmax = max_len
        elem = prec // 8
        tdt = torch.float16 if prec == 16 else torch.float32
        x, dev = 16 // elem, "cuda:0"
        per_layer = 2 * B * H * self.Lmax * Dh * elem
        self.layers = max(2, min(24, int(1.5e9 // per_layer) + 1))
        g = torch.Generator(device=dev).manual_seed(0)
        init = self.lib.ffa_init_cache_f16 if prec == 16 else self.lib.ffa_init_cache_f32
        self.fn = self.lib.ffa_attention_f16 if prec == 16 else self.lib.ffa_attention_f32
        self.q = torch.randn(B, H, Dh, device=dev, generator=g)
        qdir = self.q / self.q.norm(dim=-1, keepdim=True)
        self.kc, self.vc = [], []
        for _ in range(self.layers):
            K = torch.randn(B, H, self.Lmax, Dh, device=dev, generator=g)
            if p > 0:
                pos = torch.rand(B, H, self.Lmax, device=dev, generator=g).argsort(dim=-1)[:, :, :32]
                K.scatter_(2, pos[..., None].expand(-1, -1, -1, Dh),
                           4 * qdir[:, :, None, :] + 0.1 * torch.randn(B, H, 32, Dh, device=dev, generator=g))
            else:
                K *= 0.5
            K = K.to(tdt)
            V = (torch.randn(B, H, self.Lmax, Dh, device=dev, generator=g) * (1.0 if p > 0 else 0.5)).to(tdt)
            kc = torch.empty(B, H, Dh // x, self.Lmax, x, dtype=tdt, device=dev)
            vc = torch.empty(B, H, self.Lmax, Dh, dtype=tdt, device=dev)
            capi.check(init(kc.data_ptr(), vc.data_ptr(), K.data_ptr(), V.data_ptr(), B, self.Lmax, self.Lmax, Dh, H,
                            None), "ffa_init_cache")
            torch.cuda.synchronize()
            self.kc.append(kc)
            self.vc.append(vc)
            del K, V
        self.q = self.q.to(tdt)
        self.k = torch.randn(B, H, Dh, device=dev, generator=g).to(tdt)
        self.v = torch.randn(B, H, Dh, device=dev, generator=g).to(tdt)
        self.out = torch.empty(B, H, Dh, dtype=tdt, device=dev)
        n = self.lib.ffa_workspace_bytes(B, H, Dh, self.Lmax)
        self.ws = torch.zeros(n, dtype=torch.uint8, device=dev)
        torch.cuda.synchronize()

    def time_plan(self, plan, t, region_ms=4.0, repeats=3):
        """us per launch of `plan` at t cached keys: launches on rotating caches recorded into a HIP
        graph of about `region_ms` and replayed, best of `repeats` replays (eager launches from
        Python cannot keep up with the short steps).  None if the library refuses the plan."""
        torch = self.torch
        scale = self.Dh ** -0.5

        def go(n, sp):
            for i in range(n):
                l = i % self.layers
                rc = self.fn(self.B, self.H, self.Dh, self.Lmax, scale, t, self.q.data_ptr(), self.k.data_ptr(),
                             self.v.data_ptr(), self.kc[l].data_ptr(), self.vc[l].data_ptr(), self.out.data_ptr(),
                             None, self.p, C.byref(plan), 1, self.ws.data_ptr(), self.ws.numel(), sp)
                if rc != 0:
                    return rc
            return 0
        if not hasattr(self, "side"):
            self.side = torch.cuda.Stream()
        side = self.side
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            rc = go(self.layers, side.cuda_stream)
            side.synchronize()
            if rc != 0:
                return None
            ms = time_region(torch, lambda: go(2 * self.layers, side.cuda_stream))   # upper bound: eager
        n = max(2 * self.layers, min(4000, int(region_ms / (ms / (2 * self.layers)))))
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            go(n, torch.cuda.current_stream().cuda_stream)
        graph.replay()
        torch.cuda.synchronize()
        best = min(time_region(torch, graph.replay) for _ in range(repeats)) * 1e3 / n
        del graph
        return best


def candidate_plans(capi, prec, B, H, Dh, t, p, cus):
    """The rules' own plan first, then the alternatives worth timing: launch kinds, wave counts,
    lanes per key and split factors around one workgroup per CU."""
    ntiles, bh = t // 64 + 1, B * H
    fits_lds = ntiles * 64 * 4 <= 140 * 1024
    nch = Dh * (prec // 8) // 16
    tpk_ok = lambda k: Dh != 80 and nch % k == 0 and nch // k <= 8 and (k == 4 or nch <= 16)
    out = [("rules", capi.plan_launch(prec, B, H, Dh, t, p, False, cus, rules_only=True))]

    def cut(ns):
        ns = max(1, min(ns, ntiles, 128))
        tps = -(-ntiles // ns)
        return -(-ntiles // tps), tps

    if p > 0:
        if fits_lds:
            out += [(f"workgroup w{w}", capi.make_plan(capi.FFA_LAUNCH_WORKGROUP, w, 1, ntiles)) for w in (4, 8, 16)]
        for w in (4, 8):
            for f in (1, 2, 4):
                ns, tps = cut(f * cus // bh)
                out.append((f"two_pass w{w} x{ns}", capi.make_plan(capi.FFA_LAUNCH_TWO_PASS, w, ns, tps)))
    else:
        geos = []
        if bh >= cus:
            whole = bh // cus * cus
            rest = bh - whole
            if rest:
                base = -(-cus // rest)
                geos += [(whole, base), (whole, 2 * base), (whole, max(1, base // 2))]
            geos.append((bh, 1))
        else:
            geos += [(0, cus // bh), (0, max(1, cus // (2 * bh))), (0, max(1, cus // (4 * bh))), (0, 2 * cus // bh), (bh, 1)]
        lanes = [1] + [k for k in ((4,) if nch >= 16 else (2, 4)) if tpk_ok(k)]
        for w in (4, 8):
            for whole, ns in geos:
                ns, tps = cut(ns)
                for k in lanes:
                    out.append((f"split w{w}{f' lanes/key {k}' if k > 1 else ''} whole{bh if ns == 1 else whole} x{ns}",
                                capi.make_plan(capi.FFA_LAUNCH_SPLIT, w, ns, tps, 0, bh if ns == 1 else whole,
                                               threads_per_key=k)))
        if bh < cus and ntiles <= 16:      # short sequences: also workgroups of two waves
            for whole, ns in geos:
                ns, tps = cut(ns)
                out.append((f"split w2 whole{bh if ns == 1 else whole} x{ns}",
                            capi.make_plan(capi.FFA_LAUNCH_SPLIT, 2, ns, tps, 0, bh if ns == 1 else whole)))
        if fits_lds:
            out += [(f"workgroup w{w}", capi.make_plan(capi.FFA_LAUNCH_WORKGROUP, w, 1, ntiles)) for w in (4, 8, 16)]
    seen, uniq = set(), []
    for label, plan in out:
        if plan.as_tuple() not in seen:
            seen.add(plan.as_tuple())
            uniq.append((label, plan))
    return uniq


GRID_T = (128, 192, 256, 384, 512, 768, 1024, 1536, 2048, 3072, 4096, 6144, 8192, 12288, 16384)
GRID_BH = ((1, 16), (1, 32), (2, 32), (4, 32), (8, 32), (10, 32), (16, 32), (32, 32))


def grid_shapes():
    """The grid behind csrc/ffa_plan_grid.inc: pairs x head dim x length x pruned or not, away
    from the BASELINE shapes, so that any problem finds a measured neighbour."""
    out = []
    for prec, dhs in ((16, (64, 128, 256)), (32, (64, 128))):
        for Dh in dhs:
            for B, H in GRID_BH:
                for p in (0.0, 1e-2):
                    out.append((prec, B, H, Dh, p, GRID_T[-1] + 64, list(GRID_T)))
    return out


def run_plan_sweep(out_path, grid=False, part=(0, 1)):
    """Times every candidate at every sweep point, prints one JSON line per point and writes the
    table.  A point keeps the rules' plan unless a candidate beats it by more than 3 % in a
    second, longer timing of the two.  grid: the shapes of grid_shapes() (shape i belongs to part
    i % parts) and rows keyed by their own (pairs, t), which the planner matches by nearest
    neighbour; otherwise the BASELINE shapes and rows keyed by a range of t."""
    import torch
    from fastforwardattention_amd import capi
    lib = capi.load()
    cus = lib.ffa_device_compute_units()
    rows = []
    shapes = [sh for i, sh in enumerate(grid_shapes()) if i % part[1] == part[0]] if grid else SWEEP_SHAPES
    for prec, B, H, Dh, p, max_len, ts in shapes:
        shape = SweepShape(prec, B, H, Dh, p, max_len)
        for i, t in enumerate(ts):
            timed = []
            for label, plan in candidate_plans(capi, prec, B, H, Dh, t, p, cus):
                us = shape.time_plan(plan, t)
                if us is not None:
                    timed.append((us, label, plan))
            rule_us, _, rule_plan = timed[0]
            best_us, best_label, best_plan = min(timed, key=lambda x: x[0])
            chosen_us, chosen_label, chosen = rule_us, "rules", rule_plan
            if best_plan.as_tuple() != rule_plan.as_tuple() and best_us < SWEEP_MARGIN * rule_us:
                rule_us = shape.time_plan(rule_plan, t, region_ms=12.0)        # the two again, longer
                best_us = shape.time_plan(best_plan, t, region_ms=12.0)
                if best_us < SWEEP_MARGIN * rule_us:
                    chosen_us, chosen_label, chosen = best_us, best_label, best_plan
                else:
                    chosen_us = rule_us
            best_us = min(best_us, chosen_us)
            # the point stands for the t halfway to its neighbours (an eighth beyond the ends)
            lo = (ts[i - 1] + t) // 2 + 1 if i > 0 else (t - (ts[1] - t) // 2 if len(ts) > 1 else t * 7 // 8)
            hi = (t + ts[i + 1]) // 2 if i + 1 < len(ts) else (t + (t - ts[i - 1]) // 2 if len(ts) > 1 else t * 9 // 8)
            if grid:
                lo = hi = t
            rows.append((prec, Dh, B * H, max(lo, 0), hi, 1 if p > 0 else 0, chosen, chosen_us, best_us, rule_us,
                         0 if chosen_label == "rules" else 1))
            print(json.dumps({"sweep_point": {"precision": prec, "B": B, "H": H, "Dh": Dh, "max_len": max_len, "t": t, "p": p},
                              "t_range": [max(lo, 0), hi], "chosen": chosen_label, "chosen_us": round(chosen_us, 2),
                              "rules_us": round(rule_us, 2), "best": best_label, "best_us": round(best_us, 2),
                              "candidates": {label: round(us, 2) for us, label, _ in timed}}), flush=True)
        del shape
        torch.cuda.empty_cache()
    dev = torch.cuda.get_device_name(0)
    if grid:
        lines = [
            "// Launch-plan grid: what a sweep on the device found fastest on a grid of problem sizes.  The",
            "// planner looks up the nearest row (same precision, head dimension and pruned / exact; pairs and",
            "// length each within a factor of sqrt 2) and, where the row overrides the rules, launches its",
            "// kind, waves and lanes per key with the row's workgroup count re-cut for the actual problem.",
            "// GENERATED -- do not edit by hand.",
            "//   command : python bench.py --sweep-plans grid      (then rebuild the library)",
            f"//   device  : {dev}, {cus} compute units",
            "// Row: FFA_GRID_ROW(override, precision, head_dim, pairs, t, pruned, kind, waves, threads_per_key,",
            "//                   n_splits, whole_heads, chosen_us, best_us, rule_us)",
            "//   override = 0: the rules' own plan stayed within 3 % of the fastest candidate and is kept.",
        ] if part[0] == 0 else []
        for prec, Dh, pairs, lo, hi, pruned, plan, chosen_us, best_us, rule_us, override in rows:
            lines.append(f"FFA_GRID_ROW({override}, {prec}, {Dh}, {pairs}, {lo}, {pruned}, {plan.kind}, "
                         f"{plan.waves_per_wg}, {plan.threads_per_key}, {plan.n_splits}, {plan.whole_heads}, "
                         f"{chosen_us:.2f}f, {best_us:.2f}f, {rule_us:.2f}f)")
    else:
        lines = [
            "// Launch-plan table: measured choices that override the planner's rules at the points where a",
            "// sweep on the device found a faster launch.  GENERATED -- do not edit by hand.",
            "//   command : python bench.py --sweep-plans      (then rebuild the library)",
            f"//   device  : {dev}, {cus} compute units",
            "// Row: FFA_PLAN_ROW(override, precision, head_dim, pairs, t_lo, t_hi, pruned, kind, waves,",
            "//                   threads_per_key, n_splits, whole_heads, chosen_us, best_us, rule_us)",
            "//   override = 1: the planner launches this row's plan for t_lo <= t <= t_hi on a 256-CU device;",
            "//   override = 0: the rules' own plan stayed within 3 % of the fastest candidate and is kept (the",
            "//   row records the measurement).  pairs = batch * heads; pruned = 1 for prob_thresh > 0;",
            "//   chosen_us is the time of the row's plan, best_us the fastest candidate of the sweep, rule_us",
            "//   the time of what the rules alone launch.",
        ]
        for prec, Dh, pairs, lo, hi, pruned, plan, chosen_us, best_us, rule_us, override in rows:
            lines.append(f"FFA_PLAN_ROW({override}, {prec}, {Dh}, {pairs}, {lo}, {hi}, {pruned}, {plan.kind}, "
                         f"{plan.waves_per_wg}, {plan.threads_per_key}, {plan.n_splits}, {plan.whole_heads}, "
                         f"{chosen_us:.2f}f, {best_us:.2f}f, {rule_us:.2f}f)")
    with open(out_path, "w") as f:
        f.write("\n".join(lines) + "\n")
    print(json.dumps({"plan_table": out_path, "rows": len(rows),
                      "overridden": sum(r[10] for r in rows)}))


DEFAULT_SWEEP_OUT = os.path.join(ROOT, "fastforwardattention_amd", "csrc", "ffa_plan_table.inc")
DEFAULT_GRID_OUT = os.path.join(ROOT, "fastforwardattention_amd", "csrc", "ffa_plan_grid.inc")


def run_copy_calibration(mib=128, reps=40):
    """A plain device-to-device copy kernel of known size, for scaling rocprofv3's
    FETCH_SIZE / WRITE_SIZE readings: every launch reads `mib` MiB and writes `mib` MiB.
    Rotates over enough buffers that the source is never cache-resident."""
    import torch
    n = mib * (1 << 20) // 4
    nbuf = 6
    src = [torch.full((n,), float(i + 1), dtype=torch.float32, device="cuda:0") for i in range(nbuf)]
    dst = [torch.empty(n, dtype=torch.float32, device="cuda:0") for _ in range(nbuf)]
    torch.cuda.synchronize()
    for i in range(reps):
        dst[i % nbuf].copy_(src[i % nbuf])
    torch.cuda.synchronize()
    print(json.dumps({"calibration": "torch elementwise copy kernel", "bytes_read_per_launch": mib << 20,
                      "bytes_written_per_launch": mib << 20, "launches": reps}))


def load_traffic(name, algorithmic_bytes):
    """HBM bytes per launch: the ratio (FETCH_SIZE + WRITE_SIZE, each scaled by a plain copy
    kernel of known size) / algorithmic bytes measured with rocprofv3 --pmc and recorded in
    profiles/traffic.json, applied to this run's algorithmic mean.  None when the workload
    has no counter run on record."""
    path = os.path.join(ROOT, "profiles", "traffic.json")
    try:
        with open(path) as f:
            rec = json.load(f).get(name)
        return round(rec["hbm_bytes_over_algorithmic_bytes"] * algorithmic_bytes) if rec else None
    except (OSError, ValueError, KeyError):
        return None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=6144)
    ap.add_argument("--warmup", type=int, default=240)
    ap.add_argument("--workload", default="opt1.3b_b10", choices=sorted(WORKLOADS))
    ap.add_argument("--default-launch", action="store_true", help="use_default_kernel_launch=True")
    ap.add_argument("--layers", type=int, default=None,
                    help="independent layer caches used round-robin (default: the model's layer count; 1 = a single "
                         "cache, which at the headline shape stays resident in the 256 MB last-level cache)")
    ap.add_argument("--plan", default=None, help="kind,waves,tiles_per_split[,combine[,whole_heads]] (kind: 0 workgroup, 1 split; combine: 0 fused, 1 kernel)")
    ap.add_argument("--legs", default="graph,capi,ext", help="comma list of graph,capi,ext")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--hf-end-to-end", nargs="?", const="opt", default=None, choices=["opt", "gptj", "opt-beams"],
                    help="only: decode an OPT-1.3b-shaped (default; opt-beams: with beam search) or GPT-J-6B-shaped "
                         "random model with and without the FFACache hook")
    ap.add_argument("--no-parity", action="store_true", help="skip the untimed every-step parity check")
    ap.add_argument("--no-suite", action="store_true",
                    help="leave out the short rows for the other BASELINE configurations")
    ap.add_argument("--suite", action="store_true",
                    help="run every BASELINE configuration (tuned and default launch) and the pruned sweep; "
                         "one JSON line each instead of the single headline line")
    ap.add_argument("--sweep-plans", nargs="?", const="baseline", default=None, metavar="baseline|grid[:i/n]",
                    help="time candidate launch plans and write a table the planner compiles in (then rebuild the "
                         "library): 'baseline' (default) = the BASELINE shapes -> csrc/ffa_plan_table.inc; 'grid' = a "
                         "grid of problem sizes -> csrc/ffa_plan_grid.inc ('grid:i/n' = every n-th shape from the "
                         "i-th, rows to be concatenated in order of i)")
    ap.add_argument("--sweep-out", default=None, help="where --sweep-plans writes the table")
    ap.add_argument("--init-cache", action="store_true", help="only the cache-construction kernel at the BASELINE shapes")
    ap.add_argument("--pruned-sweep", action="store_true", help="only the pruned sweep (BASELINE configs[4])")
    ap.add_argument("--transform-rows", action="store_true",
                    help="only the rows that time the step with a rotary embedding against the plain step")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="run a plain 128 MiB copy kernel 40 times (reference for rocprofv3 --pmc FETCH_SIZE / "
                         "WRITE_SIZE scaling) and exit")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (one process, one MI355X); "
              f"--gpus {args.gpus} is not supported.", file=sys.stderr)
        sys.exit(2)

    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the hot path has no CPU fallback.", file=sys.stderr)
        sys.exit(3)

    from fastforwardattention_amd import _build
    _build.ensure_built()
    if args.calibrate_copy:
        run_copy_calibration()
        return
    if args.suite:
        run_suite(args)
        return
    if args.sweep_plans:
        if args.sweep_plans.startswith("grid"):
            part = tuple(int(x) for x in args.sweep_plans.split(":")[1].split("/")) if ":" in args.sweep_plans else (0, 1)
            run_plan_sweep(args.sweep_out or DEFAULT_GRID_OUT, grid=True, part=part)
        else:
            run_plan_sweep(args.sweep_out or DEFAULT_SWEEP_OUT)
        return
    if args.pruned_sweep:
        run_pruned_sweeps()
        return
    if args.transform_rows:
        for row in run_transform_rows():
            print(json.dumps(row), flush=True)
        return
    if args.init_cache:
        print(json.dumps(run_init_cache_bench()))
        return
    if args.hf_end_to_end:
        print(json.dumps(run_hf_end_to_end(args.hf_end_to_end)))
        return

    plan_override = tuple(int(x) for x in args.plan.split(",")) if args.plan else None
    steps, warmup = args.steps, args.warmup
    wl = Workload(args.workload, use_default=args.default_launch, plan_override=plan_override, layers=args.layers,
                  steps=steps)
    legs = [x for x in args.legs.split(",") if x]
    mean_b = wl.mean_bytes()
    launches = launches_for(wl, steps, warmup)

    res, replays_us = {}, None
    floor_us = None
    if "graph" in legs:
        reps = run_graph(wl, launches)
        replays_us = [round(ms * 1e3 / launches, 3) for ms in reps]
        res["graph"] = median(reps)
        if all(wl.floor_plan(wl.t_of(i)) is not None for i in range(steps)):
            floor_us = median(run_graph(wl, launches, floor=True)) * 1e3 / launches
    if "capi" in legs:
        res["capi"] = run_capi(wl, launches)
    if "ext" in legs:
        res["ext"] = run_ext(wl, launches)
    primary = "graph" if "graph" in res else legs[0]
    us_step = res[primary] * 1e3 / launches
    gbs = mean_b / (us_step * 1e-6) / 1e9

    plan0 = wl.plan_for(wl.t_of(0))
    t_lo, t_hi = wl.t_range()
    shape = f"B={wl.B} H={wl.H} Dh={wl.Dh} {wl.dtype}"
    out = {
        "metric": f"KV-cache HBM GB/s (decode attention, {args.workload}: {shape}, t={t_lo}->{t_hi + 1})",
        "value": round(gbs, 1), "unit": "GB/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": round(us_step / 1e3, 6), "us_per_step": round(us_step, 3),
        "tokens_per_s": round(wl.B / (us_step * 1e-6), 1),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": wl.dtype, "accumulate_dtype": "f32", "data": "synthetic",
        "config": {"workload": f"{args.workload}: {shape} prompt={wl.prompt} t={t_lo}->{t_hi + 1} p=0 "
                               f"scale={wl.scale}; step = one attention call on one of {wl.layers} independent "
                               f"layer caches; the {steps} steps sample the decode at t_i = {wl.prompt} + "
                               f"(i*{wl.gen})//{steps}",
                   "timing_leg": primary, "timed_launches": launches,
                   "timed_region_ms": round(res[primary], 3),
                   "launch_plan_at_first_step": repr(plan0)},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4),
                     "traffic": load_traffic(args.workload, mean_b),
                     "algorithmic_bytes_per_launch": round(mean_b),
                     "kernel": {0: "ffa_decode_wg_kernel", 1: "ffa_decode_split_kernel"}.get(plan0.kind, "two-pass pair"),
                     "launch_us": round(us_step, 3)},
    }
    if floor_us is not None:
        # the same launches with every load and nothing else (ffa_load_floor): what this launch
        # shape could reach with free arithmetic and free merges
        out["roofline"]["load_floor_us"] = round(floor_us, 3)
        out["roofline"]["of_load_floor"] = round(floor_us / us_step, 4)
    if replays_us is not None:
        out["graph_replays_us_per_step"] = replays_us
    for leg in ("capi", "ext"):
        if leg in res and leg != primary:
            u = res[leg] * 1e3 / launches
            out[f"eager_{leg}_us_per_step"] = round(u, 3)
            out[f"eager_{leg}_GBps"] = round(mean_b / (u * 1e-6) / 1e9, 1)
    if not args.no_parity:
        out["parity"] = parity_check(wl)
    del wl
    torch.cuda.empty_cache()
    if not args.no_suite:
        out["suite"] = run_suite_rows()
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(Workload.describe(args.workload))
    print(json.dumps(out))
    if not args.no_parity and not out["parity"]["ok"]:
        print("bench.py: parity check FAILED; the throughput above is not a valid result", file=sys.stderr)
        sys.exit(4)


if __name__ == "__main__":
    main()
