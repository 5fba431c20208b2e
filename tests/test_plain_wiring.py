"""Pins of the plain model's wiring that do not rest on reading the reference's forward pass the
same way twice: a case small enough to be worked out with pencil and paper, whose logits stand
here as literals with their closed forms, and special weights under which the whole model must
collapse to a library routine applied to the embedding. A norm after the branch instead of before
it, a branch that replaces the stream instead of adding to it, heads read interleaved instead of
head-major, keys taken from the value projection, a rotation of the wrong sign or pairing, a
missing score scale, gate and up exchanged, and a projection used transposed each fail at least
one of them (tests/test_llama.py:148-152 of the reference pins the same things against an
installed library's model, which is no source here).
"""

from __future__ import annotations

import json
import os

import pytest
import torch
import torch.nn.functional as F
from safetensors.torch import save_file

from tests.helpers import TINY_A, TINY_B, prompt
from tests.plain import llama as P
from tinyserve_llm_amd.weights.random_init import write_random_model

D = torch.float64


def write_folder(folder, config: dict, tensors: dict[str, torch.Tensor]) -> str:
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(config, f)
    save_file({k: v.to(torch.float32).contiguous() for k, v in tensors.items()}, os.path.join(folder, "model.safetensors"))
    return str(folder)


def rows(*r):
    return torch.tensor(r, dtype=torch.float32)


def test_three_tokens_worked_out_by_hand(tmp_path):
    """One layer, width 4, one head of 4 dimensions, eps 0, every norm weight 1, rope base 10000 (so
    the pair (0, 2) turns by 1 radian a position and the pair (1, 3) by 0.01), identity q, k and v
    projections. The three embeddings have mean square 1, so the first norm changes nothing:

        e0 = (2, 0, 0, 0)   e1 = (0, 0, 2, 0)   e2 = (r, r, 0, 0),  r = sqrt 2.

    Written as complex numbers z = x0 + i x2, w = x1 + i x3, position m turns z by exp(i m) and w by
    exp(0.01 i m). Keys: k0: z = 2; k1: z = 2i exp(i); k2: z = r exp(2i), w = r exp(0.02i). The score
    of query a against key b is Re(z_a conj z_b + w_a conj w_b) / sqrt 4:

        token 1:  s10 = Re(2i exp(i) 2) / 2 = -2 sin 1,        s11 = 2
        token 2:  s20 = r cos 2,   s21 = Re(r exp(2i) conj(2i exp(i))) / 2 = r sin 1,   s22 = 2

    (the opposite sense of rotation gives +2 sin 1 and -r sin 1). With p = softmax of a row of
    scores the attention outputs are sums of the unrotated values:

        a0 = e0,   a1 = (2 p10, 0, 2 p11, 0),   a2 = (2 p20 + r p22, r p22, 2 p21, 0).

    o_proj has W[r][r + 1 mod 4] = 1, so it gives y_r = a_(r + 1) (used transposed it would give
    a_(r - 1)), and h = e + y. The feed-forward reads x = h / rms(h): gate = (x0, x1), up = (x3, x2),
    down puts silu(gate) * up into places 0 and 2 of the stream. The head's three rows read
    n0, n2 and n1 + n3 of n = h / rms(h) after the last sum. Evaluated with a pocket calculator:"""
    r = 2.0 ** 0.5
    folder = write_folder(tmp_path / "hand", dict(
        architectures=["LlamaForCausalLM"], model_type="llama", hidden_size=4, num_attention_heads=1,
        num_key_value_heads=1, head_dim=4, num_hidden_layers=1, intermediate_size=2, vocab_size=3, rms_norm_eps=0.0,
        rope_theta=10000.0, max_position_embeddings=8, tie_word_embeddings=False), {
        "model.embed_tokens.weight": rows((2, 0, 0, 0), (0, 0, 2, 0), (r, r, 0, 0)),
        "model.layers.0.input_layernorm.weight": torch.ones(4),
        "model.layers.0.post_attention_layernorm.weight": torch.ones(4),
        "model.norm.weight": torch.ones(4),
        "model.layers.0.self_attn.q_proj.weight": torch.eye(4),
        "model.layers.0.self_attn.k_proj.weight": torch.eye(4),
        "model.layers.0.self_attn.v_proj.weight": torch.eye(4),
        "model.layers.0.self_attn.o_proj.weight": rows((0, 1, 0, 0), (0, 0, 1, 0), (0, 0, 0, 1), (1, 0, 0, 0)),
        "model.layers.0.mlp.gate_proj.weight": rows((1, 0, 0, 0), (0, 1, 0, 0)),
        "model.layers.0.mlp.up_proj.weight": rows((0, 0, 0, 1), (0, 0, 1, 0)),
        "model.layers.0.mlp.down_proj.weight": rows((1, 0), (0, 0), (0, 1), (0, 0)),
        "lm_head.weight": rows((1, 0, 0, 0), (0, 0, 1, 0), (0, 1, 0, 1)),
    })
    got = P.PlainLlama(folder, D).logits([0, 1, 2])
    want = torch.tensor([[1.749326434227, 0.0, 0.969462235734],
                         [0.0, 1.758511470679, 0.976350694356],
                         [1.616056647929, 0.0, 1.586907660696]], dtype=D)
    # (sqrt 2 is stored as a 32-bit number: 2e-8 off)
    torch.testing.assert_close(got, want, rtol=0, atol=2e-7)
    # the last token alone sits at position 0 and sees only itself: a2 = e2, so
    # h = (r + r, r, 0, r), which no mask, rotation or softmax enters
    alone = P.PlainLlama(folder, D).logits([2])[0]
    h = torch.tensor([2 * r, r, 0.0, r], dtype=D)
    x = h / h.pow(2).mean().sqrt()
    h = h + torch.stack((F.silu(x[0]) * x[3], torch.zeros((), dtype=D), F.silu(x[1]) * x[2], torch.zeros((), dtype=D)))
    n = h / h.pow(2).mean().sqrt()
    torch.testing.assert_close(alone, torch.stack((n[0], n[2], n[1] + n[3])), rtol=0, atol=2e-7)


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    a, b = tmp_path_factory.mktemp("wa"), tmp_path_factory.mktemp("wb")
    write_random_model(str(a), TINY_A, 0, torch.float32)
    write_random_model(str(b), TINY_B, 1, torch.float32)
    return str(a), str(b)


def head_of_the_normalised(m: P.PlainLlama, stream: torch.Tensor) -> torch.Tensor:
    """Final norm and head by the library's routines."""
    head = m.w["model.embed_tokens.weight"] if m.tied else m.w["lm_head.weight"]
    return F.linear(F.rms_norm(stream, (m.hidden,), m.w["model.norm.weight"], m.eps), head)


@pytest.mark.parametrize("which", [0, 1])
def test_branches_that_give_nothing_leave_the_embedding(folders, which):
    """With o_proj and down_proj zero both branches of every layer add nothing, and the logits are
    the head of the normalised embedding. A norm applied to the stream after a branch, or a branch
    whose result replaces the stream, changes them."""
    cfg = (TINY_A, TINY_B)[which]
    m = P.PlainLlama(folders[which], D)
    for name in m.w:
        if name.endswith(("o_proj.weight", "down_proj.weight")):
            m.w[name] = torch.zeros_like(m.w[name])
    ids = prompt(11, 9, cfg.vocab_size)
    want = head_of_the_normalised(m, m.w["model.embed_tokens.weight"][torch.tensor(ids)])
    torch.testing.assert_close(m.logits(ids), want, rtol=1e-12, atol=1e-12)
    assert float(want.abs().max()) > 1e-3


def only_attention_of_layer_0(m: P.PlainLlama) -> None:
    """Every branch but the first layer's attention gives nothing."""
    for name in m.w:
        if name.endswith("down_proj.weight") or (name.endswith("o_proj.weight") and ".layers.0." not in name):
            m.w[name] = torch.zeros_like(m.w[name])


def test_heads_are_read_head_major_and_a_group_shares_its_key_value_head(folders):
    """Configuration A: 4 heads of 16 in 2 groups. Only query head 2's slice of o_proj is kept, so
    the logits may depend on value head 1 (rows 16..31 of v_proj) and on nothing of value head 0.
    Heads read interleaved (row r belonging to head r mod 4) spread every head over all rows."""
    m = P.PlainLlama(folders[0], D)
    only_attention_of_layer_0(m)
    d, ids = TINY_A.head_dim, prompt(12, 10, TINY_A.vocab_size)
    o = m.w["model.layers.0.self_attn.o_proj.weight"]
    kept = torch.zeros_like(o)
    kept[:, 2 * d:3 * d] = o[:, 2 * d:3 * d]
    m.w["model.layers.0.self_attn.o_proj.weight"] = kept
    base = m.logits(ids)
    nothing = head_of_the_normalised(m, m.w["model.embed_tokens.weight"][torch.tensor(ids)])
    assert float((base - nothing).abs().max()) > 1e-6, "head 2 contributes"
    v = m.w["model.layers.0.self_attn.v_proj.weight"].clone()
    for name, lo in (("v_proj", 0), ("k_proj", 0), ("q_proj", 0), ("q_proj", d), ("q_proj", 3 * d)):
        saved = m.w[f"model.layers.0.self_attn.{name}.weight"].clone()
        m.w[f"model.layers.0.self_attn.{name}.weight"][lo:lo + d] = 0          # another head's rows
        torch.testing.assert_close(m.logits(ids), base, rtol=0, atol=0)
        m.w[f"model.layers.0.self_attn.{name}.weight"] = saved
    m.w["model.layers.0.self_attn.v_proj.weight"] = v.clone()
    m.w["model.layers.0.self_attn.v_proj.weight"][d:2 * d] = 0                  # its own value head
    torch.testing.assert_close(m.logits(ids), nothing, rtol=1e-12, atol=1e-12)
    m.w["model.layers.0.self_attn.v_proj.weight"] = v
    for name, lo in (("k_proj", d), ("q_proj", 2 * d)):                          # its own key head and its own queries
        saved = m.w[f"model.layers.0.self_attn.{name}.weight"].clone()
        m.w[f"model.layers.0.self_attn.{name}.weight"][lo:lo + d] *= 3.0
        assert float((m.logits(ids) - base).abs().max()) > 1e-7, name
        m.w[f"model.layers.0.self_attn.{name}.weight"] = saved


def test_without_keys_attention_is_the_running_mean_of_the_values(folders):
    """k_proj zero: every score is 0, the softmax is uniform over the keys a token may see, and the
    attention output is the mean of the value rows up to it, whatever the rotation. Keys taken from
    v_proj and values from k_proj would give zero values instead."""
    m = P.PlainLlama(folders[1], D)
    only_attention_of_layer_0(m)
    m.w["model.layers.0.self_attn.k_proj.weight"] = torch.zeros_like(m.w["model.layers.0.self_attn.k_proj.weight"])
    ids = prompt(13, 8, TINY_B.vocab_size)
    e = m.w["model.embed_tokens.weight"][torch.tensor(ids)]
    x = F.rms_norm(e, (m.hidden,), m.w["model.layers.0.input_layernorm.weight"], m.eps)
    v = F.linear(x, m.w["model.layers.0.self_attn.v_proj.weight"])                         # [n, kv * d]
    mean = v.cumsum(0) / torch.arange(1, len(ids) + 1, dtype=D)[:, None]
    per_head = mean.view(len(ids), m.kv_heads, m.head_dim).repeat_interleave(m.heads // m.kv_heads, dim=1)
    stream = e + F.linear(per_head.reshape(len(ids), -1), m.w["model.layers.0.self_attn.o_proj.weight"])
    torch.testing.assert_close(m.logits(ids), head_of_the_normalised(m, stream), rtol=1e-11, atol=1e-11)


def test_one_token_sees_its_own_value_and_the_feed_forward_reads_the_new_stream(folders):
    """A single token at position 0: no rotation, one key, so attention returns its value row and
    the layer is a chain of library routines. The feed-forward's norm must read the stream after the
    attention's sum, and gate and up must not be exchanged."""
    for folder, cfg in zip(folders, (TINY_A, TINY_B)):
        m = P.PlainLlama(folder, D)
        tok = 7
        h = m.w["model.embed_tokens.weight"][tok][None]
        group = m.heads // m.kv_heads
        for i in range(m.layers):
            p = f"model.layers.{i}."
            x = F.rms_norm(h, (m.hidden,), m.w[p + "input_layernorm.weight"], m.eps)
            v = F.linear(x, m.w[p + "self_attn.v_proj.weight"]).view(1, m.kv_heads, m.head_dim)
            h = h + F.linear(v.repeat_interleave(group, dim=1).reshape(1, -1), m.w[p + "self_attn.o_proj.weight"])
            x = F.rms_norm(h, (m.hidden,), m.w[p + "post_attention_layernorm.weight"], m.eps)
            h = h + F.linear(F.silu(F.linear(x, m.w[p + "mlp.gate_proj.weight"])) * F.linear(x, m.w[p + "mlp.up_proj.weight"]),
                             m.w[p + "mlp.down_proj.weight"])
        torch.testing.assert_close(m.logits([tok]), head_of_the_normalised(m, h), rtol=1e-11, atol=1e-11)
