"""Hugging Face hook (fastforwardattention_amd/hf.py): tiny random-weight OPT and GPT-J models
built from local configs (nothing is downloaded), a left-padded batch, teacher-forced decoding.
Logits with the FFACache must match the same model run with transformers' own cache.

On the CPU the engine behind the cache is a stand-in with FastForwardAttn's interface built on
the numpy oracle (test infrastructure: it checks the hook's bookkeeping -- time steps, padding
offsets, scales, shapes); the GPU tests run the real extension."""
import numpy as np
import pytest
import torch

from oracle import ffa_oracle as O

transformers = pytest.importorskip("transformers")
from fastforwardattention_amd import hf  # noqa: E402


class OracleEngine:
    """FastForwardAttn's constructor / get_cache / attention on top of the CPU oracle."""

    def __init__(self, K, V, max_len, use_default_kernel_launch):
        assert K.is_contiguous() and V.is_contiguous() and K.shape == V.shape
        self.B, self.H, self.L, self.Dh = K.shape
        self.kc = torch.from_numpy(O.pack_k_cache(K.detach().numpy(), max_len))
        self.vc = torch.from_numpy(O.pack_v_cache(V.detach().numpy(), max_len))
        self.calls = []

    def get_cache(self):
        return self.kc, self.vc

    def attention(self, q, k, v, k_cache, v_cache, scale, t, *rest, cache_indir=None, beam_width=1):
        seq_lens, p = (rest[0], rest[1]) if len(rest) == 2 else (None, rest[0])
        assert k_cache is self.kc and v_cache is self.vc and p == 0.0
        shape = (self.B, self.H, self.Dh)
        self.calls.append((t, None if seq_lens is None else seq_lens.tolist(), scale))
        out = O.decode_step(q.detach().numpy().reshape(shape), k.detach().numpy().reshape(shape),
                            v.detach().numpy().reshape(shape), self.kc.numpy(), self.vc.numpy(), scale, t,
                            seq_lengths=None if seq_lens is None else seq_lens.numpy(), right_or_no_padding=False,
                            cache_indir=None if cache_indir is None else cache_indir.numpy(), beam_width=beam_width)
        return torch.from_numpy(out.astype(np.float32))

    def attention_ex(self, q, k, v, k_cache, v_cache, scale, t, seq_lens, p, rotary_dim, q_bias, k_bias, v_bias,
                     cache_indir=None, beam_width=1):
        """The fused call: the oracle's token transform (rotary embedding at the position
        t - first_key[b]), then the step."""
        assert q_bias is None and k_bias is None and v_bias is None
        shape = (self.B, self.H, self.Dh)
        sl = None if seq_lens is None else seq_lens.numpy()
        pos = O.rotary_positions(self.B, t, sl, False)
        q2, k2, v2 = O.token_transform(q.detach().numpy().reshape(shape), k.detach().numpy().reshape(shape),
                                       v.detach().numpy().reshape(shape), "f32", rotary_dim=rotary_dim, pos=pos)
        self.rotary_calls = getattr(self, "rotary_calls", []) + [(t, rotary_dim, pos.tolist())]
        rest = (p,) if seq_lens is None else (seq_lens, p)
        return self.attention(torch.from_numpy(q2), torch.from_numpy(k2), torch.from_numpy(v2), k_cache, v_cache,
                              scale, t, *rest, cache_indir=cache_indir, beam_width=beam_width)


def tiny_opt(dtype=torch.float32):
    cfg = transformers.OPTConfig(vocab_size=96, hidden_size=128, num_hidden_layers=2, ffn_dim=256,
                                 num_attention_heads=2, max_position_embeddings=64, word_embed_proj_dim=128,
                                 dropout=0.0, attention_dropout=0.0, pad_token_id=1, bos_token_id=2, eos_token_id=2)
    torch.manual_seed(0)
    return transformers.OPTForCausalLM(cfg).to(dtype).eval()


def tiny_gptj(dtype=torch.float32):
    cfg = transformers.GPTJConfig(vocab_size=96, n_positions=64, n_embd=256, n_layer=2, n_head=2, rotary_dim=32,
                                  n_inner=256, resid_pdrop=0.0, embd_pdrop=0.0, attn_pdrop=0.0,
                                  bos_token_id=2, eos_token_id=2)
    torch.manual_seed(0)
    return transformers.GPTJForCausalLM(cfg).to(dtype).eval()


def padded_batch(device="cpu"):
    """Two prompts of 9 and 5 tokens, left-padded to 9."""
    ids = torch.tensor([[5, 6, 7, 8, 9, 10, 11, 12, 13], [1, 1, 1, 1, 20, 21, 22, 23, 24]], device=device)
    mask = torch.tensor([[1] * 9, [0] * 4 + [1] * 5], device=device)
    return ids, mask


def teacher_forced_logits(model, ids, mask, steps, cache):
    """Prompt pass, then `steps` single-token passes fed with fixed tokens; logits of each."""
    logits = []
    with torch.no_grad():
        out = model(input_ids=ids, attention_mask=mask, past_key_values=cache, use_cache=True)
        logits.append(out.logits[:, -1].float())
        cache = out.past_key_values
        for i in range(steps):
            tok = torch.full((ids.shape[0], 1), 30 + i % 60, device=ids.device, dtype=ids.dtype)   # stays inside the 96-token vocabulary
            mask = torch.cat([mask, torch.ones_like(mask[:, :1])], dim=1)
            pos = (mask.long().cumsum(-1) - 1)[:, -1:]
            kw = {"position_ids": pos} if "GPTJ" in type(model).__name__ else {}
            out = model(input_ids=tok, attention_mask=mask, past_key_values=cache, use_cache=True, **kw)
            logits.append(out.logits[:, -1].float())
            cache = out.past_key_values
    return torch.stack(logits), cache


@pytest.mark.parametrize("family", ["opt", "gptj", "gptj_torch_rotary"])
def test_hook_bookkeeping_against_plain_cache(family):
    fused = family != "gptj_torch_rotary"
    family = family.split("_")[0]
    model = tiny_opt() if family == "opt" else tiny_gptj()
    ids, mask = padded_batch()
    steps = 6
    want, _ = teacher_forced_logits(model, ids, mask, steps, None)
    hf.enable(model, fused_rotary=fused)
    cache = hf.FFACache(max_new_tokens=steps, engine=OracleEngine)
    got, cache = teacher_forced_logits(model, ids, mask, steps, cache)
    assert float((got - want).abs().max()) < 2e-4
    assert isinstance(cache, hf.FFACache) and len(cache.layers) == 2
    Dh = 64 if family == "opt" else 128
    for layer in cache.layers:
        assert layer.t == 9 + steps and layer.max_len == 9 + steps
        assert [c[0] for c in layer.engine.calls] == list(range(9, 9 + steps))      # t carried per layer
        assert all(c[1] == [0, 4] for c in layer.engine.calls)                       # first real key per sample
        # OPT scales q before the call (scale 1); GPT-J passes 1/sqrt(Dh) (modeling_gptj.py:265)
        assert all(abs(c[2] - (1.0 if family == "opt" else Dh ** -0.5)) < 1e-7 for c in layer.engine.calls)
        if family == "gptj" and fused:
            # the engine rotated q and k itself: rotary_dim of the config, position = real tokens so far
            assert layer.engine.rotary_calls == [(9 + i, 32, [9 + i, 5 + i]) for i in range(steps)]
        else:
            assert not hasattr(layer.engine, "rotary_calls")
    assert cache.get_seq_length() == 9 + steps
    # the cache is full now: one more token must be refused, not written out of bounds
    full = torch.cat([mask, torch.ones(2, steps + 1, dtype=mask.dtype)], 1)
    kw = {"position_ids": (full.long().cumsum(-1) - 1)[:, -1:]} if family == "gptj" else {}
    with pytest.raises(RuntimeError, match="cache full"), torch.no_grad():
        model(input_ids=torch.full((2, 1), 40), attention_mask=full, past_key_values=cache, use_cache=True, **kw)
    hf.disable(model)
    again, _ = teacher_forced_logits(model, ids, mask, steps, None)
    assert torch.equal(again, want)


def test_cache_refuses_unhooked_model_and_unsupported_operations():
    model = tiny_opt()
    ids, mask = padded_batch()
    cache = hf.FFACache(max_new_tokens=2, engine=OracleEngine)
    with pytest.raises(RuntimeError, match="enable"):
        teacher_forced_logits(model, ids, mask, 1, cache)        # attention never went through the hook
    layer = hf.FFALayer(2, engine=OracleEngine)
    with pytest.raises(NotImplementedError):
        layer.crop(1)
    with pytest.raises(ValueError):
        hf.FFALayer(0)
    with pytest.raises(ValueError):
        hf.FFALayer(2, num_beams=0)
    # beam search with a cache that was not told about the beams: refused, not silently wrong
    hf.enable(model)
    kw = dict(attention_mask=mask, max_new_tokens=3, do_sample=False, num_beams=2, pad_token_id=1, eos_token_id=None)
    with pytest.raises(NotImplementedError, match="num_beams"):
        model.generate(ids, past_key_values=hf.FFACache(max_new_tokens=3, engine=OracleEngine), **kw)
    hf.disable(model)


def test_env_switches(monkeypatch):
    monkeypatch.setenv("max_tokens", "7")
    monkeypatch.setenv("use_ffa_default_kl", "1")
    monkeypatch.setenv("use_ffa", "1")
    cache = hf.FFACache.from_env(engine=OracleEngine)
    layer = cache.layer_class_to_replicate()
    assert layer.max_new_tokens == 7 and layer.use_default_kernel_launch and layer.prob_thresh == 0.0
    assert hf.enabled_by_env()
    monkeypatch.setenv("use_ffa", "0")
    assert not hf.enabled_by_env()


def test_generate_with_ffa_cache_matches_plain_generate():
    model = tiny_opt()
    ids, mask = padded_batch()
    kw = dict(attention_mask=mask, max_new_tokens=5, do_sample=False, pad_token_id=1, eos_token_id=None)
    want = model.generate(ids, **kw)
    hf.enable(model)
    got = model.generate(ids, past_key_values=hf.FFACache(max_new_tokens=5, engine=OracleEngine), **kw)
    hf.disable(model)
    assert torch.equal(got, want)


@pytest.mark.parametrize("family", ["opt", "gptj", "gptj_torch_rotary"])
def test_beam_search_with_ffa_cache_matches_plain_beam_search(family):
    """generate(num_beams=3): transformers re-parents beams after every step.  Its own cache copies
    keys and values along the batch axis; the FFACache permutes rows of its table.  Same tokens,
    and the caches hold exactly what each sample wrote (nothing was moved)."""
    fused = family != "gptj_torch_rotary"
    model = tiny_opt() if family == "opt" else tiny_gptj()
    ids, mask = padded_batch()
    n, nb = 7, 3
    kw = dict(attention_mask=mask, max_new_tokens=n, do_sample=False, num_beams=nb, num_return_sequences=nb,
              pad_token_id=1, eos_token_id=None, length_penalty=0.0)
    want = model.generate(ids, **kw)
    hf.enable(model, fused_rotary=fused)
    cache = hf.FFACache(max_new_tokens=n, engine=OracleEngine, num_beams=nb)
    got = model.generate(ids, past_key_values=cache, **kw)
    hf.disable(model)
    assert torch.equal(got, want)
    layer = cache.layers[0]
    table = layer.beam_table.numpy()
    assert table.shape == (2 * nb, 9 + n) and table.min() >= 0 and table.max() < nb
    # the search did re-parent: some sample reads a sibling's slots
    assert (table != (np.arange(2 * nb) % nb)[:, None]).any()


@pytest.mark.gpu
@pytest.mark.parametrize("family,dtype", [("opt", torch.float32), ("gptj", torch.float32), ("gptj_torch_rotary", torch.float32),
                                          ("opt", torch.float16), ("gptj", torch.float16)])
def test_beam_search_with_hip_engine(family, dtype):
    """Beam search on the GPU through the real extension.  fp32: the same tokens as transformers'
    own cache.  fp16: sequence scores within 2e-2 (near-ties may order beams differently)."""
    print("hf beams", family, dtype, flush=True)
    fused = family != "gptj_torch_rotary"
    family = family.split("_")[0]
    model = (tiny_opt(dtype) if family == "opt" else tiny_gptj(dtype)).to("cuda:0")
    ids, mask = padded_batch("cuda:0")
    n, nb = 12, 4
    kw = dict(attention_mask=mask, max_new_tokens=n, do_sample=False, num_beams=nb, num_return_sequences=1,
              pad_token_id=1, eos_token_id=None, length_penalty=0.0, return_dict_in_generate=True, output_scores=True)
    want = model.generate(ids, **kw)
    hf.enable(model, fused_rotary=fused)
    for use_default in (False, True):
        cache = hf.FFACache(max_new_tokens=n, num_beams=nb, use_default_kernel_launch=use_default)
        got = model.generate(ids, past_key_values=cache, **kw)
        if dtype == torch.float32:
            assert torch.equal(got.sequences, want.sequences)
        assert float((got.sequences_scores - want.sequences_scores).abs().max()) < (1e-4 if dtype == torch.float32 else 2e-2)
        table = cache.layers[0].beam_table.cpu().numpy()
        assert (table != (np.arange(2 * nb) % nb)[:, None]).any()
    hf.disable(model)


@pytest.mark.gpu
@pytest.mark.parametrize("family,dtype,tol", [("opt", torch.float16, 3e-2), ("opt", torch.float32, 2e-4),
                                               ("gptj", torch.float16, 3e-2), ("gptj", torch.float32, 2e-4),
                                               ("gptj_torch_rotary", torch.float16, 3e-2),
                                               ("gptj_torch_rotary", torch.float32, 2e-4),
                                               ("opt", torch.bfloat16, 0.25), ("gptj", torch.bfloat16, 0.25)])
def test_hook_with_hip_engine(family, dtype, tol):
    """The real extension behind the cache, on the GPU, left-padded batch included.  GPT-J runs
    with the rotary embedding inside the engine's call and, as in the reference, in torch.
    bfloat16 (8 significant bits) is held to a quarter of a logit unit."""
    print("hf hook", family, dtype, flush=True)
    fused = family != "gptj_torch_rotary"
    family = family.split("_")[0]
    model = (tiny_opt(dtype) if family == "opt" else tiny_gptj(dtype)).to("cuda:0")
    ids, mask = padded_batch("cuda:0")
    steps = 8
    want, _ = teacher_forced_logits(model, ids, mask, steps, None)
    hf.enable(model, fused_rotary=fused)
    for use_default in (False, True):
        got, cache = teacher_forced_logits(model, ids, mask, steps,
                                           hf.FFACache(max_new_tokens=steps, use_default_kernel_launch=use_default))
        assert float((got - want).abs().max()) < tol
        import ff_attention
        assert all(isinstance(layer.engine, ff_attention.FastForwardAttn) for layer in cache.layers)
    # a threshold far below every probability: the pruning kernels must reproduce the exact logits
    got, _ = teacher_forced_logits(model, ids, mask, steps, hf.FFACache(max_new_tokens=steps, prob_thresh=1e-7))
    assert float((got - want).abs().max()) < tol
    hf.disable(model)


def small_gptj(dtype=torch.float32):
    """Four heads of 64, room for 1024 positions: long enough for the launch plan of a decode to
    move from one workgroup per head to sequence-split launches."""
    cfg = transformers.GPTJConfig(vocab_size=96, n_positions=1024, n_embd=256, n_layer=2, n_head=4, rotary_dim=32,
                                  n_inner=256, resid_pdrop=0.0, embd_pdrop=0.0, attn_pdrop=0.0,
                                  bos_token_id=2, eos_token_id=2)
    torch.manual_seed(0)
    return transformers.GPTJForCausalLM(cfg).to(dtype).eval()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-4), (torch.float16, 3e-2)])
def test_long_decode_with_fused_rotary_crosses_launch_plans(dtype, tol):
    """170 decode steps from a long prompt (one sample left-padded by 37) through the hook with
    the rotary embedding inside the engine's call, one engine (one workspace) per layer for the
    whole decode; the logits of every step against transformers' own cache.  The engine's plan
    changes from one workgroup per head to sequence-split launches on the way."""
    print("hf long decode", dtype, flush=True)
    model = small_gptj(dtype).to("cuda:0")
    g = torch.Generator().manual_seed(5)
    prompt, pad = (740 if dtype == torch.float16 else 430), 37    # the plans switch at 832 / 512 cached keys
    ids = torch.randint(3, 96, (2, prompt), generator=g).to("cuda:0")
    mask = torch.ones_like(ids)
    ids[1, :pad] = 1
    mask[1, :pad] = 0
    steps = 170
    want, _ = teacher_forced_logits(model, ids, mask, steps, None)
    hf.enable(model, fused_rotary=True)
    got, cache = teacher_forced_logits(model, ids, mask, steps, hf.FFACache(max_new_tokens=steps))
    hf.disable(model)
    assert torch.isfinite(got).all()
    err = (got - want).abs().amax(dim=(1, 2))
    assert float(err.max()) < tol, (int(err.argmax()), float(err.max()))
    engine = cache.layers[0].engine
    split = {engine.launch_plan(t, 0.0)[4] > 1 for t in range(prompt, prompt + steps)}
    assert split == {False, True}, "the decode never crossed from unsplit to sequence-split launches"
