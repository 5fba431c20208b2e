"""A plain, slow Llama: whole sequences, no cache, one function per part, written from the
reference's formulas and sharing no code with the engine. It reads config.json and the
safetensors file itself, by the checkpoint's tensor names. Everything runs in the dtype of the
tensors it is given (float64 for the oracle, float32 to mirror the reference's CPU tests).

`round_to` mimics bfloat16 storage between operations where a test wants to see what rounding
does; the default keeps full precision.
"""

from __future__ import annotations

import json
import math
import os

import torch
from safetensors import safe_open


# ---- parts ------------------------------------------------------------------------------------

def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """tinyserve_llm/model/llama.py:52-58: x * rsqrt(mean(x^2) + eps) * weight."""
    var = x.pow(2).mean(dim=-1, keepdim=True)
    return x * torch.rsqrt(var + eps) * weight


def add_rms_norm(x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, eps: float
                 ) -> tuple[torch.Tensor, torch.Tensor]:
    """tinyserve_llm/model/llama.py:60-67: the sum is the new residual and what is normalised."""
    s = x + residual
    return rms_norm(s, weight, eps), s


def rope_inv_freq(head_dim: int, theta: float, scaling: dict | None, max_position: int) -> torch.Tensor:
    """tinyserve_llm/model/llama.py:148 and :107-128 (llama3 scaling), computed in float32 as
    the reference does; callers cast afterwards."""
    inv_freq = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float) / head_dim))
    if scaling is None:
        return inv_freq
    factor = scaling["factor"]
    low, high = scaling["low_freq_factor"], scaling["high_freq_factor"]
    old = scaling.get("original_max_position_embeddings", max_position)
    out = []
    for f in inv_freq.tolist():
        f32 = torch.tensor(f, dtype=torch.float)
        wavelen = 2 * math.pi / f32
        if wavelen > old / low:
            base = f32 / factor
        else:
            base = f32
        if not (wavelen < old / high) and not (wavelen > old / low):
            smooth = (old / wavelen - low) / (high - low)
            base = (1 - smooth) * base / factor + smooth * base
        out.append(base)
    return torch.stack(out)


def rope_tables(head_dim: int, theta: float, scaling: dict | None, max_position: int, num_positions: int,
                dtype: torch.dtype) -> tuple[torch.Tensor, torch.Tensor]:
    """tinyserve_llm/model/llama.py:158-160: angles = float32(position) * inv_freq, in float32;
    cos and sin of them. Returned in `dtype`."""
    inv_freq = rope_inv_freq(head_dim, theta, scaling, max_position)
    t = torch.arange(num_positions, dtype=torch.float)
    freqs = torch.outer(t, inv_freq)
    return freqs.cos().to(dtype), freqs.sin().to(dtype)


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """tinyserve_llm/model/llama.py:131-136: dimension i pairs with i + head_dim/2.
    x [tokens, heads, head_dim]; cos, sin [tokens, head_dim/2]."""
    half = x.shape[-1] // 2
    x1, x2 = x[..., :half], x[..., half:]
    c, s = cos[:, None, :], sin[:, None, :]
    return torch.cat((x1 * c - x2 * s, x2 * c + x1 * s), dim=-1)


def causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float | None = None,
                     window: int = 0) -> torch.Tensor:
    """tinyserve_llm/model/attention.py:40-57: per head softmax(q k^T * scale + causal mask) v,
    key/value head g serving query heads g*group .. (g+1)*group-1. q [n, heads, d], k, v [n, kv, d]."""
    n, heads, d = q.shape
    group = heads // k.shape[1]
    scale = d ** -0.5 if scale is None else scale
    out = torch.empty_like(q)
    for h in range(heads):
        kh, vh = k[:, h // group], v[:, h // group]
        scores = (q[:, h] @ kh.T) * scale
        i = torch.arange(n)
        hidden = i[None, :] > i[:, None]
        if window:
            hidden = hidden | (i[None, :] <= i[:, None] - window)
        scores = scores.masked_fill(hidden, float("-inf"))
        out[:, h] = torch.softmax(scores, dim=-1) @ vh
    return out


def silu_mul(gate_up: torch.Tensor) -> torch.Tensor:
    """tinyserve_llm/model/llama.py:80-83: silu(first half) * second half."""
    inter = gate_up.shape[-1] // 2
    g, u = gate_up[..., :inter], gate_up[..., inter:]
    return g * torch.sigmoid(g) * u


# ---- the model ----------------------------------------------------------------------------------

class PlainLlama:
    """Whole-sequence forward of a checkpoint folder; `logits(ids)` gives [len, vocab]."""

    def __init__(self, folder: str, dtype: torch.dtype = torch.float64, weights_as: torch.dtype | None = None) -> None:
        with open(os.path.join(folder, "config.json")) as f:
            c = json.load(f)
        self.c = c
        self.dtype = dtype
        self.hidden = c["hidden_size"]
        self.heads = c["num_attention_heads"]
        self.kv_heads = c.get("num_key_value_heads") or self.heads
        self.head_dim = c.get("head_dim") or self.hidden // self.heads
        self.layers = c["num_hidden_layers"]
        self.eps = c["rms_norm_eps"]
        self.max_position = c["max_position_embeddings"]
        params = c.get("rope_parameters")
        if params:
            self.theta, scaling = params.get("rope_theta", c.get("rope_theta", 10000.0)), params
        else:
            self.theta, scaling = c.get("rope_theta", 10000.0), c.get("rope_scaling")
        if scaling is not None and scaling.get("rope_type", scaling.get("type", "default")) == "default":
            scaling = None
        self.scaling = scaling
        self.tied = bool(c.get("tie_word_embeddings", False))
        self.w: dict[str, torch.Tensor] = {}
        for name in sorted(os.listdir(folder)):
            if name.startswith("model") and name.endswith(".safetensors"):
                with safe_open(os.path.join(folder, name), "pt", "cpu") as f:
                    for key in f.keys():
                        t = f.get_tensor(key)
                        if weights_as is not None:
                            t = t.to(weights_as)     # what the engine stores
                        self.w[key] = t.to(dtype)

    def hidden_states(self, ids: list[int]) -> torch.Tensor:
        """tinyserve_llm/model/llama.py:270-276 with the deferred residual written out plainly:
        h += attention(norm(h)); h += mlp(norm(h)); final norm."""
        w, n = self.w, len(ids)
        cos, sin = rope_tables(self.head_dim, self.theta, self.scaling, self.max_position, n, self.dtype)
        h = w["model.embed_tokens.weight"][torch.tensor(ids)]
        qs, ks = self.heads * self.head_dim, self.kv_heads * self.head_dim
        for i in range(self.layers):
            p = f"model.layers.{i}."
            x = rms_norm(h, w[p + "input_layernorm.weight"], self.eps)
            q = (x @ w[p + "self_attn.q_proj.weight"].T).view(n, self.heads, self.head_dim)
            k = (x @ w[p + "self_attn.k_proj.weight"].T).view(n, self.kv_heads, self.head_dim)
            v = (x @ w[p + "self_attn.v_proj.weight"].T).view(n, self.kv_heads, self.head_dim)
            q, k = apply_rope(q, cos, sin), apply_rope(k, cos, sin)
            o = causal_attention(q, k, v).reshape(n, qs)
            h = h + o @ w[p + "self_attn.o_proj.weight"].T
            x = rms_norm(h, w[p + "post_attention_layernorm.weight"], self.eps)
            gate_up = torch.cat((x @ w[p + "mlp.gate_proj.weight"].T, x @ w[p + "mlp.up_proj.weight"].T), dim=-1)
            h = h + silu_mul(gate_up) @ w[p + "mlp.down_proj.weight"].T
        assert ks == w["model.layers.0.self_attn.k_proj.weight"].shape[0]
        return rms_norm(h, w["model.norm.weight"], self.eps)

    def logits(self, ids: list[int]) -> torch.Tensor:
        """tinyserve_llm/model/llama.py:293-304: the head is the embedding when tied."""
        head = self.w["model.embed_tokens.weight"] if self.tied else self.w["lm_head.weight"]
        return self.hidden_states(ids) @ head.T

    def greedy(self, prompt: list[int], steps: int) -> list[int]:
        ids, out = list(prompt), []
        for _ in range(steps):
            tok = int(self.logits(ids)[-1].argmax())
            out.append(tok)
            ids.append(tok)
        return out
