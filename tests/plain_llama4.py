"""A plain, slow Llama 4 text decoder for tests: whole sequences, no cache, one
function per part, float32 (or float64) throughout.

It is written from the reference's formulas - each function cites the lines of
``llama4/llama4_jax/model.py`` (``model.py`` below) it follows -
and shares no code with the engine.  Where the task's configuration differs
from what the reference hard-codes, the function says so:

* which layers are NoPE comes from ``no_rope_layers`` (reference: every 4th, ``model.py:203, 913``);
* the chunk mask is applied on RoPE layers and NoPE layers are global
  (reference: the other way round, ``model.py:944``);
* llama3 frequency scaling constants come from ``rope_scaling`` and are skipped
  if it is null (reference: constants, always applied, ``model.py:159-163, 709``);
* NoPE layers scale queries by the attention temperature (absent in the reference).

It reads a model folder with the ``safetensors`` package and its own parsing of
``config.json``.
"""
from __future__ import annotations

import json
import math
import os

import torch


# ----------------------------------------------------------------------------- config
def read_config(model_dir: str) -> dict:
    """``model.py:229-231`` reads ``text_config``; a text-only config has the keys at top level."""
    with open(os.path.join(model_dir, "config.json")) as f:
        top = json.load(f)
    c = dict(top.get("text_config", top))
    L = c["num_hidden_layers"]
    if c.get("head_dim") is None:
        c["head_dim"] = c["hidden_size"] // c["num_attention_heads"]
    if not c.get("no_rope_layers"):
        c["no_rope_layers"] = [0 if (i + 1) % 4 == 0 else 1 for i in range(L)]  # model.py:203, 913
    if c.get("moe_layers") is None:
        step = c["interleave_moe_layer_step"]
        c["moe_layers"] = [i for i in range(L) if (i + 1) % step == 0]  # model.py:558
    c.setdefault("intermediate_size_mlp", c["intermediate_size"])
    c.setdefault("use_qk_norm", True)
    c.setdefault("attn_temperature_tuning", False)
    c.setdefault("floor_scale", 8192)
    c.setdefault("attn_scale", 0.1)
    c.setdefault("rope_scaling", None)
    c.setdefault("attention_chunk_size", None)
    return c


def read_weights(model_dir: str, dtype=torch.float32) -> dict:
    from safetensors.torch import load_file

    raw = load_file(os.path.join(model_dir, "model.safetensors"))
    out = {}
    for k, v in raw.items():
        if k.startswith("language_model."):
            k = k[len("language_model."):]
        out[k] = v.to(dtype)
    return out


# ----------------------------------------------------------------------------- parts
def rms_norm(x, gamma, eps):
    """``model.py:885-888``: ``rms = sqrt(mean(x^2) + eps)``; ``gamma * x / rms``; gamma None = 1."""
    rms = torch.sqrt(torch.mean(x * x, dim=-1, keepdim=True) + eps)
    return (gamma if gamma is not None else 1.0) * x / rms


def llama3_frequency_correction(freq, factor, low_freq_factor, high_freq_factor, old_context_len):
    """``model.py:654-672``.  With ``high == low`` there is no medium band
    (the reference's division by ``high - low`` would not be defined)."""
    low_freq_wavelen = old_context_len / low_freq_factor
    high_freq_wavelen = old_context_len / high_freq_factor
    wavelen = 2 * math.pi / freq
    out = torch.where(wavelen > low_freq_wavelen, freq / factor, freq)  # :666
    if high_freq_factor == low_freq_factor:
        return out
    smooth = (old_context_len / wavelen - low_freq_factor) / (high_freq_factor - low_freq_factor)  # :668
    smoothed = (1 - smooth) * out / factor + smooth * out  # :669
    is_medium = ~(wavelen < high_freq_wavelen) & ~(wavelen > low_freq_wavelen)  # :670
    return torch.where(is_medium, smoothed, out)  # :671


def rope_frequencies(head_dim, theta, scaling, dtype=torch.float32):
    """``model.py:706-709``: ``fraction = arange(0, dh, 2) / dh``; ``1 / theta**fraction``; then the correction.
    Always formed on the CPU in float32, wherever the model runs: another device's power function may round
    the last bit differently, and a last bit of a frequency is a thousandth of a radian at position 16,000."""
    fraction = torch.arange(0, head_dim, 2, dtype=torch.float32, device="cpu") / head_dim
    freq = 1.0 / (torch.tensor(float(theta), dtype=torch.float32, device="cpu") ** fraction)
    if scaling:
        freq = llama3_frequency_correction(
            freq, scaling["factor"], scaling["low_freq_factor"], scaling["high_freq_factor"],
            scaling["original_max_position_embeddings"])
    return freq.to(dtype)


ANGLES_IN_FLOAT32 = False


def rope_sin_cos(positions, freq):
    """``model.py:712-719``: ``angle[t, j] = pos[t] * freq[j]`` in float32, then sin and cos.  When the model
    runs in float64 as the yardstick of a float32 engine, ``ANGLES_IN_FLOAT32`` keeps this one product rounded
    to float32 as the reference computes it (at position 8,000 that rounding is 2e-4 of a radian: it belongs
    to what is computed, not to an implementation's error); sine and cosine in the model's dtype."""
    if ANGLES_IN_FLOAT32:
        ang = (positions.to(torch.float32)[:, None] * freq.to(torch.float32)[None, :]).to(freq.dtype)
    else:
        ang = positions.to(freq.dtype)[:, None] * freq[None, :]
    return torch.sin(ang), torch.cos(ang)


def apply_rope(x, sin, cos):
    """``model.py:722-728``: adjacent pairs ``(x[2j], x[2j+1])``;
    ``(x1*cos - x2*sin, x2*cos + x1*sin)``.  ``x``: ``[T, H, dh]``; sin, cos ``[T, dh/2]``."""
    x_ = x.reshape(*x.shape[:-1], -1, 2)
    x1, x2 = x_[..., 0], x_[..., 1]
    sin, cos = sin[:, None, :], cos[:, None, :]
    return torch.stack([x1 * cos - x2 * sin, x2 * cos + x1 * sin], dim=-1).reshape(x.shape)


def attention_mask(q_pos, k_pos, chunk):
    """``model.py:731-742``: causal ``q_pos >= k_pos`` and, with a chunk size, the same
    ``pos // chunk`` for query and key."""
    m = q_pos[:, None] >= k_pos[None, :]
    if chunk is not None:
        m = m & ((q_pos[:, None] // chunk) == (k_pos[None, :] // chunk))
    return m


def temperature_scale(positions, floor_scale, attn_scale, dtype=torch.float32):
    """Not in the reference.  ``1 + attn_scale * ln(1 + floor((pos + 1) / floor_scale))``."""
    return 1.0 + attn_scale * torch.log1p(torch.floor((positions.to(dtype) + 1.0) / floor_scale))


SCORE_ELEMENTS_AT_ONCE = 1 << 30  # beyond this attention() goes head by head
TOKENS_ONE_BY_ONE = 1024  # beyond this moe_block() takes the tokens of an expert together


def attention(q, k, v, mask, scale):
    """``model.py:774-794``: query head ``h`` uses kv head ``h // G``; scores times ``scale``;
    masked with -1e30; softmax over keys; times values.  ``q``: ``[T, Hq, dh]``, ``k, v``: ``[S, Hkv, dh]``."""
    T, hq, dh = q.shape
    hk = k.shape[1]
    g = hq // hk
    q_ = q.reshape(T, hk, g, dh)
    if hq * T * k.shape[0] > SCORE_ELEMENTS_AT_ONCE:
        # the same, one kv head after the other (heads do not meet): the scores of all heads of a long
        # sequence would not fit into memory together
        out = torch.empty(T, hk, g, dh, dtype=q.dtype, device=q.device)
        for h in range(hk):
            qk = torch.einsum("tgd,sd->gts", q_[:, h], k[:, h]) * scale
            qk = torch.where(mask[None], qk, torch.full_like(qk, -1e30))
            out[:, h] = torch.einsum("gts,sd->tgd", torch.softmax(qk, dim=-1), v[:, h])
        return out.reshape(T, hq * dh)
    qk = torch.einsum("thgd,shd->hgts", q_, k) * scale
    qk = torch.where(mask[None, None], qk, torch.full_like(qk, -1e30))
    attn = torch.softmax(qk, dim=-1)
    out = torch.einsum("hgts,shd->thgd", attn, v)
    return out.reshape(T, hq * dh)


def attention_block(x, w, prefix, cfg, layer_idx, positions):
    """``model.py:891-955``: q, k, v projections (``:907-909``); on RoPE layers rotation
    of q and k (``:915``) and then, if ``use_qk_norm``, weightless rms norm of both
    (``:916-917``); attention; output projection (``:952-954``)."""
    hq, hk, dh = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    T = x.shape[0]
    q = (x @ w[prefix + "self_attn.q_proj.weight"].T).reshape(T, hq, dh)
    k = (x @ w[prefix + "self_attn.k_proj.weight"].T).reshape(T, hk, dh)
    v = (x @ w[prefix + "self_attn.v_proj.weight"].T).reshape(T, hk, dh)
    uses_rope = bool(cfg["no_rope_layers"][layer_idx])
    chunk = None
    if uses_rope:
        freq = rope_frequencies(dh, cfg["rope_theta"], cfg["rope_scaling"], x.dtype).to(x.device)
        sin, cos = rope_sin_cos(positions.to(x.device), freq)
        q, k = apply_rope(q, sin, cos), apply_rope(k, sin, cos)
        if cfg["use_qk_norm"]:
            q, k = rms_norm(q, None, cfg["rms_norm_eps"]), rms_norm(k, None, cfg["rms_norm_eps"])
        chunk = cfg["attention_chunk_size"]
    elif cfg["attn_temperature_tuning"]:
        q = q * temperature_scale(positions, cfg["floor_scale"], cfg["attn_scale"], x.dtype)[:, None, None]
    mask = attention_mask(positions, positions, chunk)
    o = attention(q, k, v, mask, dh ** -0.5)  # scale: model.py:774
    return o @ w[prefix + "self_attn.o_proj.weight"].T


def mlp_block(x, w_gate, w_up, w_down):
    """``model.py:1142-1153``: ``(silu(x Wg) * (x Wu)) Wd``; weights ``[out, in]`` as stored."""
    return (torch.nn.functional.silu(x @ w_gate.T) * (x @ w_up.T)) @ w_down.T


def route(x, w_router, top_k):
    """``model.py:958-972``: scores ``x @ w_router`` in float32, ``top_k`` largest, sigmoid of
    the chosen scores.  Among equal scores the lowest index comes first."""
    scores = x @ w_router.T
    idx = torch.sort(scores, dim=-1, descending=True, stable=True).indices[:, :top_k]
    vals = torch.gather(scores, 1, idx)
    return torch.sigmoid(vals), idx, scores


def moe_block(x, w, prefix, cfg, forced=None):
    """``model.py:999-1139``: each chosen expert gets the token's input times its gate
    (``:1066-1071``); expert = SwiGLU with ``gate_up_proj[e]`` ``[D, 2F]`` (gate is the
    first half of the last axis, ``chkpt_utils.py:198-205``) and ``down_proj[e]`` ``[F, D]``
    (``:1076-1085``); outputs summed over the chosen experts (``:1111``); plus the shared
    expert on the unscaled input (``:1137-1139``).  Returns (output, ids, scores)."""
    F = cfg["intermediate_size"]
    gates, idx, scores = route(x, w[prefix + "router.weight"], cfg["num_experts_per_tok"])
    if forced is not None:
        idx = forced.to(idx.device).long()
        gates = torch.sigmoid(torch.gather(scores, 1, idx))
    gate_up, down = w[prefix + "experts.gate_up_proj"], w[prefix + "experts.down_proj"]
    out = torch.zeros_like(x)
    if x.shape[0] > TOKENS_ONE_BY_ONE:
        # the same sums with the tokens of an expert taken together (the reference's own oracle for its grouped
        # product is such a loop over experts, decode_ragged_dot.py:227-236): a long sequence token by token
        # would read every expert matrix thousands of times
        for j in range(idx.shape[1]):
            for e in torch.unique(idx[:, j]).tolist():
                rows = (idx[:, j] == e).nonzero().squeeze(-1)
                gu = (x[rows] * gates[rows, j:j + 1]) @ gate_up[e]
                out[rows] += (torch.nn.functional.silu(gu[:, :F]) * gu[:, F:]) @ down[e]
    else:
        for t in range(x.shape[0]):
            for j in range(idx.shape[1]):
                e = int(idx[t, j])
                xe = x[t] * gates[t, j]
                gu = xe @ gate_up[e]
                out[t] += (torch.nn.functional.silu(gu[:F]) * gu[F:]) @ down[e]
    shared = mlp_block(x, w[prefix + "shared_expert.gate_proj.weight"], w[prefix + "shared_expert.up_proj.weight"],
                       w[prefix + "shared_expert.down_proj.weight"])
    return out + shared, idx, scores


def forward_layer(x, w, cfg, i, positions, forced=None, info=None):
    """``model.py:1156-1183``: ``x + attn(norm(x))`` then ``+ ffn(norm(.))``."""
    p = f"model.layers.{i}."
    eps = cfg["rms_norm_eps"]
    x = x + attention_block(rms_norm(x, w[p + "input_layernorm.weight"], eps), w, p, cfg, i, positions)
    h = rms_norm(x, w[p + "post_attention_layernorm.weight"], eps)
    if i in cfg["moe_layers"]:
        ff, idx, scores = moe_block(h, w, p + "feed_forward.", cfg, None if forced is None else forced.get(i))
        if info is not None:
            info[i] = (idx, scores)
    else:
        ff = mlp_block(h, w[p + "feed_forward.gate_proj.weight"], w[p + "feed_forward.up_proj.weight"],
                       w[p + "feed_forward.down_proj.weight"])
    return x + ff


def forward(tokens, w, cfg, forced=None, info=None):
    """``model.py:1186-1210``: embedding, layers, final norm, lm head.  ``tokens``: ``[T]`` of one
    request from position 0; returns logits ``[T, V]``."""
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    x = w["model.embed_tokens.weight"][tokens]
    positions = torch.arange(tokens.shape[0])
    for i in range(cfg["num_hidden_layers"]):
        x = forward_layer(x, w, cfg, i, positions, forced, info)
    x = rms_norm(x, w["model.norm.weight"], cfg["rms_norm_eps"])
    return x @ w["lm_head.weight"].T


class PlainModel:
    def __init__(self, model_dir: str, dtype=torch.float32) -> None:
        self.cfg = read_config(model_dir)
        self.w = read_weights(model_dir, dtype)
        self.dtype = dtype

    @torch.no_grad()
    def logits(self, tokens, forced=None, info=None):
        return forward(tokens, self.w, self.cfg, forced, info)
