"""ctypes binding of the C ABI in include/ffa_c_api.h (libffa_hip.so).

For callers that hold raw device pointers (tests, the benchmark, non-torch hosts).  The
library is loaded on first use and a missing library is an error, never a fallback.
"""
from __future__ import annotations

import ctypes as C
import os

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG_DIR, "libffa_hip.so")

FFA_OK = 0
FFA_PRECISION_F16 = 16
FFA_PRECISION_F32 = 32
FFA_PRECISION_BF16 = 0xBF16
FFA_LAUNCH_WORKGROUP = 0
FFA_LAUNCH_SPLIT = 1
FFA_LAUNCH_TWO_PASS = 2
FFA_COMBINE_FUSED = 0
FFA_COMBINE_KERNEL = 1

STATUS_NAMES = {
    0: "FFA_OK", 1: "FFA_ERR_NULL_POINTER", 2: "FFA_ERR_DTYPE", 3: "FFA_ERR_HEAD_DIM",
    4: "FFA_ERR_SHAPE", 5: "FFA_ERR_TIMESTEP", 6: "FFA_ERR_ALIGNMENT", 7: "FFA_ERR_WORKSPACE",
    8: "FFA_ERR_PLAN", 9: "FFA_ERR_TOO_LONG", 10: "FFA_ERR_PROB_THRESH", 11: "FFA_ERR_LAUNCH",
    12: "FFA_ERR_NO_DEVICE", 13: "FFA_ERR_SCRATCH_LIMIT", 14: "FFA_ERR_TRANSFORM", 15: "FFA_ERR_BEAM",
}
globals().update({name: code for code, name in STATUS_NAMES.items()})   # FFA_OK, FFA_ERR_* as ints


class LaunchPlan(C.Structure):
    """struct ffa_launch_plan."""
    _fields_ = [("kind", C.c_int32), ("waves_per_wg", C.c_int32), ("threads_per_key", C.c_int32),
                ("keys_per_wave", C.c_int32), ("n_splits", C.c_int32),
                ("tiles_per_split", C.c_int32), ("combine", C.c_int32), ("whole_heads", C.c_int32)]

    def as_tuple(self):
        return (self.kind, self.waves_per_wg, self.threads_per_key, self.keys_per_wave,
                self.n_splits, self.tiles_per_split, self.combine, self.whole_heads)

    def __repr__(self):
        kind = {0: "workgroup", 1: "split", 2: "two_pass"}.get(self.kind, str(self.kind))
        return (f"LaunchPlan(kind={kind}, waves_per_wg={self.waves_per_wg}, "
                f"threads_per_key={self.threads_per_key}, n_splits={self.n_splits}, "
                f"tiles_per_split={self.tiles_per_split}, combine={self.combine}, "
                f"whole_heads={self.whole_heads})")


class TokenTransform(C.Structure):
    """struct ffa_token_transform."""
    _fields_ = [("q_bias", C.c_void_p), ("k_bias", C.c_void_p), ("v_bias", C.c_void_p),
                ("rotary_embedding_dim", C.c_int32), ("rotary_base", C.c_float)]


class BeamIndirection(C.Structure):
    """struct ffa_beam_indirection."""
    _fields_ = [("cache_indir", C.c_void_p), ("beam_width", C.c_int32)]


_vp, _i, _f, _sz = C.c_void_p, C.c_int, C.c_float, C.c_size_t
_PLAN_P = C.POINTER(LaunchPlan)
_TT_P = C.POINTER(TokenTransform)
_BI_P = C.POINTER(BeamIndirection)

# name -> (restype, argtypes); one entry per declaration in include/ffa_c_api.h
SIGNATURES = {
    "ffa_api_version": (_i, []),
    "ffa_status_string": (C.c_char_p, [_i]),
    "ffa_device_compute_units": (_i, []),
    "ffa_plan_launch": (_i, [_i, _i, _i, _i, _i, _f, _i, _i, _PLAN_P]),
    "ffa_plan_launch_rules": (_i, [_i, _i, _i, _i, _i, _f, _i, _i, _PLAN_P]),
    "ffa_plan_source": (_i, [_i, _i, _i, _i, _i, _f, _i]),
    "ffa_workspace_bytes": (_sz, [_i, _i, _i, _i]),
    "ffa_workspace_init": (_i, [_vp, _sz, _vp]),
    "ffa_init_cache_f16": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "ffa_init_cache_f32": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "ffa_attention_f16": (_i, [_i, _i, _i, _i, _f, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _f,
                               _PLAN_P, _i, _vp, _sz, _vp]),
    "ffa_attention_f32": (_i, [_i, _i, _i, _i, _f, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _f,
                               _PLAN_P, _i, _vp, _sz, _vp]),
    "ffa_attention_diag": (_i, [_i, _i, _i, _i, _i, _f, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _f,
                                _PLAN_P, _i, _vp, _sz, _vp, _vp, _vp]),
    "ffa_attention_ex": (_i, [_i, _i, _i, _i, _i, _f, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _f, _PLAN_P, _i, _TT_P,
                              _BI_P, _vp, _sz, _vp]),
    "ffa_attention_static_scratch": (_i, [_i, _i, _i, _i, _i, _f, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _f,
                                          _PLAN_P, _i, _TT_P, _BI_P, _vp]),
    "ffa_load_floor": (_i, [_i, _i, _i, _i, _i, _i, _vp, _vp, _vp, _i, _PLAN_P, _vp, _vp]),
}

_lib = None


def load() -> C.CDLL:
    """Load libffa_hip.so and attach the prototypes.  Raises OSError if it is not built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise OSError(f"{LIB_PATH} is not built; run `python -m fastforwardattention_amd._build --lib`")
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def status_string(status: int) -> str:
    return load().ffa_status_string(status).decode()


def check(status: int, what: str = "ffa call") -> None:
    if status != FFA_OK:
        raise RuntimeError(f"{what} failed: {STATUS_NAMES.get(status, status)}: {status_string(status)}")


def plan_launch(precision, B, H, Dh, t, p=0.0, use_default=False, compute_units=256, rules_only=False) -> LaunchPlan:
    plan = LaunchPlan()
    fn = load().ffa_plan_launch_rules if rules_only else load().ffa_plan_launch
    check(fn(precision, B, H, Dh, t, p, int(use_default), compute_units, C.byref(plan)), "ffa_plan_launch")
    return plan


def make_plan(kind, waves_per_wg, n_splits, tiles_per_split, combine=0, whole_heads=0, threads_per_key=1) -> LaunchPlan:
    plan = LaunchPlan()
    plan.kind, plan.waves_per_wg = kind, waves_per_wg
    plan.threads_per_key, plan.keys_per_wave = threads_per_key, 64 // threads_per_key
    plan.n_splits, plan.tiles_per_split, plan.combine = n_splits, tiles_per_split, combine
    plan.whole_heads = whole_heads
    return plan
