"""Hugging Face decoder hook: routes the one-token decode steps of OPT- and GPT-J-style
attention layers through `FastForwardAttn`.

Stands where the reference patches transformers' model files in place (modeling_opt.py:196-226,
modeling_gptj.py:252-281): the prompt pass runs ordinary attention and builds one
`FastForwardAttn` per layer from the prompt's keys and values; every later call with a single
query token goes to `attention(q, k, v, k_cache, v_cache, scale, t, seq_lens, p)` with
`seq_lens` = index of the first real key of each left-padded sample (modeling_opt.py:222,
modeling_gptj.py:274) and `t` = number of keys cached so far, carried per layer.

Written against the installed transformers (5.x) instead of a patched copy of its files:

* `FFACache` is a `transformers.Cache` whose layers own the engines.  Its `update` hands the
  new token's key/value through (tagged with the layer that owns them) instead of returning
  the concatenated history.
* models that dispatch through transformers' attention-function registry (OPT) select the
  registered function `"ffa"`; GPT-J, which calls its own `_attn`, gets that method wrapped.
* GPT-J's rotary embedding of the new token's q and k, which the reference leaves to torch
  ahead of the call (modeling_gptj.py:231-247), is taken over by the engine on decode steps
  (`attention_ex(..., rotary_dim, ...)`: the FasterTransformer feature of attention.cu:874-882):
  the layer's forward is wrapped and skips the torch-side sin/cos gather, split, rotate and
  concatenate.  `enable(model, fused_rotary=False)` keeps the reference's arrangement.
* beam search (`generate(num_beams=n, past_key_values=FFACache(..., num_beams=n))`): where the
  reference's models copy every layer's caches along the batch axis after each step
  (`_reorder_cache`, modeling_opt.py:1072-1075, modeling_gptj.py:911-918), the cache keeps one
  small table per layer -- for every sample and slot, the beam of the group whose caches hold
  that slot -- permutes its rows when beams are re-parented, and hands it to the engine
  (`attention_ex(..., cache_indir, beam_width)`: the FasterTransformer feature of
  attention.cu:1024-1033 that the reference switches off).  Keys and values never move.

    from fastforwardattention_amd import hf
    hf.enable(model)
    out = model.generate(ids, attention_mask=mask, max_new_tokens=n,
                         past_key_values=hf.FFACache(max_new_tokens=n))

The reference's environment switches are honoured by `FFACache.from_env()`:
`max_tokens`, `use_ffa_default_kl`, `prob_thresh` (summarize.py:77-96)."""
from __future__ import annotations

import functools
import os
import types

import torch
from transformers.cache_utils import Cache, CacheLayerMixin
from transformers.masking_utils import AttentionMaskInterface, eager_mask
from transformers.modeling_utils import AttentionInterface

ATTN_NAME = "ffa"
_TAG = "_ffa_layer"


def _default_engine():
    from . import FastForwardAttn  # raises ImportError when the HIP extension is not built
    return FastForwardAttn


class FFALayer(CacheLayerMixin):
    """One decoder layer's cache: a `FastForwardAttn` built at the prompt pass, the number of
    keys it holds, and the left-padding offsets of the batch."""

    is_sliding = False
    is_compileable = False

    def __init__(self, max_new_tokens: int, prob_thresh: float = 0.0,
                 use_default_kernel_launch: bool = False, engine=None, num_beams: int = 1):
        super().__init__()
        if max_new_tokens < 1:
            raise ValueError("max_new_tokens must be >= 1")
        if num_beams < 1:
            raise ValueError("num_beams must be >= 1")
        self.num_beams = int(num_beams)
        self.beam_table = None      # int32 [B, max_len]: beam of the group whose caches hold the slot
        self.max_new_tokens = int(max_new_tokens)
        self.prob_thresh = float(prob_thresh)
        self.use_default_kernel_launch = bool(use_default_kernel_launch)
        self._engine_cls = engine
        self.engine = None
        self.t = 0                  # keys cached so far = slot of the next token
        self.max_len = 0
        self.first_key = None       # int32 [B]: first real key of each left-padded sample
        self._hooked = False        # the attention hook has seen this layer's prompt pass
        self._pending = False       # a decode token was handed out and not yet attended

    # -- transformers.Cache protocol -----------------------------------------------------
    def lazy_initialization(self, key_states, value_states):
        self.dtype, self.device = key_states.dtype, key_states.device
        self.is_initialized = True

    def update(self, key_states, value_states, *args, **kwargs):
        if key_states.shape[-2] != 1 or self.engine is None:
            return self._prompt_pass(key_states, value_states)
        if not self._hooked:
            raise RuntimeError("FFACache: the model's attention does not go through the 'ffa' hook; "
                               "call fastforwardattention_amd.hf.enable(model) first")
        if self._pending:
            raise RuntimeError("FFACache: the previous decode token of this layer was never attended")
        if self.t >= self.max_len:
            raise RuntimeError(f"FFACache: cache full ({self.max_len} slots = prompt + max_new_tokens)")
        self._pending = True
        setattr(key_states, _TAG, self)
        return key_states, value_states

    def get_seq_length(self) -> int:
        return self.t

    def get_mask_sizes(self, query_length: int):
        return self.t + query_length, 0

    def get_max_length(self) -> int:
        return -1

    def reset(self):
        self.engine, self.t, self.max_len, self.first_key, self.beam_table = None, 0, 0, None, None
        self._hooked = self._pending = False

    def reorder_cache(self, beam_idx):
        """Beam search re-parents the samples: sample b continues sample beam_idx[b] of its own
        group.  Its history becomes the parent's -- a row copy in the table -- and the slot
        the parent wrote last (t - 1) is found in the parent's own caches."""
        if self.engine is None:
            return
        if self.num_beams == 1:
            raise NotImplementedError("FFACache: beam search needs FFACache(..., num_beams=n) with generate's "
                                      "num_beams (the caches are not copied between samples)")
        beam_idx = beam_idx.to(self.beam_table.device)
        B = self.beam_table.shape[0]
        own = torch.arange(B, device=beam_idx.device)
        if beam_idx.numel() != B or bool(((beam_idx // self.num_beams) != (own // self.num_beams)).any()):
            raise ValueError("FFACache: a beam can only continue a beam of its own group")
        table = self.beam_table.index_select(0, beam_idx)
        table[:, self.t - 1] = (beam_idx % self.num_beams).to(torch.int32)
        self.beam_table = table

    def _unsupported(self, *a, **k):
        raise NotImplementedError("FFACache holds the reference's fixed-layout caches: no cropping or batch "
                                  "reshaping")

    crop = batch_repeat_interleave = batch_select_indices = offload = prefetch = _unsupported

    # -- the two passes -------------------------------------------------------------------
    def _prompt_pass(self, key_states, value_states):
        if self.engine is not None:
            raise NotImplementedError("FFACache: a second multi-token pass (chunked prefill, assisted decoding) "
                                      "is not supported; the reference builds its caches from one prompt pass")
        if not self.is_initialized:
            self.lazy_initialization(key_states, value_states)
        cls = self._engine_cls or _default_engine()
        prompt_len = key_states.shape[-2]
        self.max_len = prompt_len + self.max_new_tokens
        self.engine = cls(key_states.contiguous(), value_states.to(key_states.dtype).contiguous(),
                          self.max_len, self.use_default_kernel_launch)
        self.t = prompt_len
        if self.num_beams > 1:
            B = key_states.shape[0]
            if B % self.num_beams:
                raise ValueError(f"FFACache: batch {B} is not a multiple of num_beams = {self.num_beams}")
            if not hasattr(self.engine, "attention_ex"):
                raise NotImplementedError("FFACache: this engine has no attention_ex, which beam search needs")
            own = (torch.arange(B, device=key_states.device) % self.num_beams).to(torch.int32)
            self.beam_table = own[:, None].expand(B, self.max_len).contiguous()   # every slot in the sample's own caches
        setattr(key_states, _TAG, self)
        return key_states, value_states

    def note_prompt_mask(self, attention_mask):
        """Left-padding offsets from the prompt pass's mask, as the reference takes them:
        index of the first maximum of the last query row (modeling_opt.py:222)."""
        self._hooked = True
        if attention_mask is None:
            self.first_key = None
            return
        row = attention_mask[:, :, -1, :]
        if row.dtype == torch.bool:
            row = row.to(torch.int8)
        self.first_key = torch.max(row, dim=-1).indices.reshape(-1).to(torch.int32).contiguous()

    def attend(self, query, key, value, scale: float):
        """One decode step: [B,H,1,Dh] q/k/v -> [B,H,Dh]; appends k, v at slot t."""
        if not self._pending:
            raise RuntimeError("FFACache: attend() without a pending decode token")
        dt = self.dtype
        q, k, v = query.to(dt), key.to(dt), value.to(dt)
        k_cache, v_cache = self.engine.get_cache()
        if self.beam_table is not None:
            out = self.engine.attention_ex(q, k, v, k_cache, v_cache, float(scale), self.t, self.first_key,
                                           self.prob_thresh, 0, None, None, None,
                                           cache_indir=self.beam_table, beam_width=self.num_beams)
        elif self.first_key is None:
            out = self.engine.attention(q, k, v, k_cache, v_cache, float(scale), self.t, self.prob_thresh)
        else:
            out = self.engine.attention(q, k, v, k_cache, v_cache, float(scale), self.t, self.first_key,
                                        self.prob_thresh)
        self.t += 1
        self._pending = False
        return out

    def attend_rotary(self, query, key, value, scale: float, rotary_dim: int):
        """One decode step on un-rotated q, k: [B,H,Dh] each -> [B,H,Dh].  The engine rotates q
        and k at position t - first_key[b] (the sample's real tokens so far, which is what
        transformers passes as position_ids for a left-padded batch) and appends."""
        if not self._hooked:
            raise RuntimeError("FFACache: the prompt pass did not go through the 'ffa' hook")
        if self.t >= self.max_len:
            raise RuntimeError(f"FFACache: cache full ({self.max_len} slots = prompt + max_new_tokens)")
        dt = self.dtype
        k_cache, v_cache = self.engine.get_cache()
        beams = {} if self.beam_table is None else dict(cache_indir=self.beam_table, beam_width=self.num_beams)
        out = self.engine.attention_ex(query.to(dt), key.to(dt), value.to(dt), k_cache, v_cache, float(scale), self.t,
                                       self.first_key, self.prob_thresh, int(rotary_dim), None, None, None, **beams)
        self.t += 1
        return out


class FFACache(Cache):
    """`past_key_values` object that keeps every layer's keys and values inside a
    `FastForwardAttn` (cache layouts [B,H,Dh/x,Lmax,x] / [B,H,Lmax,Dh], Lmax = prompt +
    max_new_tokens).  `engine` replaces the `FastForwardAttn` class (same constructor and
    methods); tests use it to run the bookkeeping without a GPU.  num_beams: generate's num_beams
    when beam search is used (samples are grouped num_beams at a time, as generate lays them out)."""

    def __init__(self, max_new_tokens: int, prob_thresh: float = 0.0,
                 use_default_kernel_launch: bool = False, engine=None, num_beams: int = 1):
        super().__init__(layer_class_to_replicate=functools.partial(
            FFALayer, max_new_tokens, prob_thresh, use_default_kernel_launch, engine, num_beams))

    @classmethod
    def from_env(cls, engine=None):
        """The reference's switches (summarize.py:77-96; modeling_opt.py:196-199)."""
        return cls(int(os.environ["max_tokens"]), float(os.environ.get("prob_thresh", "0")),
                   int(os.environ.get("use_ffa_default_kl", "0")) == 1, engine)


def enabled_by_env() -> bool:
    """`use_ffa=1` in the environment, the reference's master switch (modeling_opt.py:196)."""
    return int(os.environ.get("use_ffa", "0")) == 1


# -- attention hooks --------------------------------------------------------------------------
def _plain_attention(query, key, value, attention_mask, scaling):
    """Ordinary masked softmax attention for the prompt pass; [B,H,Lq,Dh] in and out."""
    w = torch.matmul(query, key.transpose(-1, -2)) * scaling
    if attention_mask is not None:
        w = w + attention_mask if attention_mask.dtype != torch.bool else w.masked_fill(~attention_mask, float("-inf"))
    w = torch.softmax(w, dim=-1, dtype=torch.float32).to(value.dtype)
    return torch.matmul(w, value)


def ffa_attention_forward(module, query, key, value, attention_mask, scaling=None, dropout=0.0, **kwargs):
    """Attention function for transformers' registry (`attn_implementation="ffa"`).
    Returns ([B, Lq, H, Dh], None) like the built-in ones."""
    if scaling is None:
        scaling = query.shape[-1] ** -0.5
    layer = getattr(key, _TAG, None)
    if layer is not None and layer._pending:
        return layer.attend(query, key, value, scaling).unsqueeze(1), None
    if layer is not None:
        layer.note_prompt_mask(attention_mask)
    out = _plain_attention(query, key, value, attention_mask, scaling)
    return out.transpose(1, 2).contiguous(), None


def _gptj_attn(self, query, key, value, attention_mask=None, *rest):
    """Replacement for GPTJAttention._attn (modeling_gptj.py:252-281): ([B,H,Lq,Dh], weights)."""
    layer = getattr(key, _TAG, None)
    if layer is not None and layer._pending:
        return layer.attend(query, key, value, 1.0 / self.scale_attn).unsqueeze(2), None
    if layer is not None:
        layer.note_prompt_mask(attention_mask)
    return self._ffa_original_attn(query, key, value, attention_mask, *rest)


def _gptj_forward(self, hidden_states, layer_past=None, attention_mask=None, position_ids=None, use_cache=False,
                  output_attentions=False, **kwargs):
    """Replacement for GPTJAttention.forward on one-token steps with an FFACache: projections,
    then the engine (rotary embedding, append, attention), then the output projection.  Every
    other call goes to the layer's own forward."""
    layer = None
    if isinstance(layer_past, FFACache) and self.layer_idx is not None and len(layer_past.layers) > self.layer_idx:
        layer = layer_past.layers[self.layer_idx]
    if (layer is None or layer.engine is None or hidden_states.shape[1] != 1 or output_attentions
            or not hasattr(layer.engine, "attention_ex")):
        return self._ffa_original_forward(hidden_states, layer_past, attention_mask, position_ids, use_cache,
                                          output_attentions, **kwargs)
    B, H, Dh = hidden_states.shape[0], self.num_attention_heads, self.head_dim
    q = self.q_proj(hidden_states).view(B, H, Dh)
    k = self.k_proj(hidden_states).view(B, H, Dh)
    v = self.v_proj(hidden_states).view(B, H, Dh)
    out = layer.attend_rotary(q, k, v, 1.0 / float(self.scale_attn), self.rotary_dim if self.rotary_dim is not None else Dh)
    out = self.out_proj(out.reshape(B, 1, H * Dh).to(hidden_states.dtype))
    return self.resid_dropout(out), None


def register():
    """Make `"ffa"` known to transformers' attention and mask registries (idempotent)."""
    AttentionInterface.register(ATTN_NAME, ffa_attention_forward)
    AttentionMaskInterface.register(ATTN_NAME, eager_mask)


def enable(model, fused_rotary=True):
    """Route `model`'s decode steps through FastForwardAttn.  Pass an `FFACache` as
    `past_key_values` afterwards; with any other cache the model behaves as before.
    fused_rotary: GPT-J's rotary embedding of the new token runs inside the engine's call
    instead of in torch (no effect on models without one)."""
    register()
    wrapped = 0
    for mod in model.modules():
        if type(mod).__name__.startswith("GPTJ") and hasattr(mod, "_attn") and hasattr(mod, "scale_attn"):
            if not hasattr(mod, "_ffa_original_attn"):
                mod._ffa_original_attn = mod._attn
                mod._attn = types.MethodType(_gptj_attn, mod)
            if fused_rotary and not hasattr(mod, "_ffa_original_forward") and hasattr(mod, "rotary_dim"):
                mod._ffa_original_forward = mod.forward
                mod.forward = types.MethodType(_gptj_forward, mod)
            wrapped += 1
    if wrapped == 0:
        model._ffa_previous_attn = model.config._attn_implementation
        model.config._attn_implementation = ATTN_NAME
    return model


def disable(model):
    """Undo `enable`."""
    for mod in model.modules():
        if hasattr(mod, "_ffa_original_attn"):
            del mod.__dict__["_attn"]          # the class's own method shows through again
            del mod._ffa_original_attn
        if hasattr(mod, "_ffa_original_forward"):
            del mod.__dict__["forward"]
            del mod._ffa_original_forward
    prev = getattr(model, "_ffa_previous_attn", None)
    if prev is not None:
        model.config._attn_implementation = prev
        del model._ffa_previous_attn
    return model
