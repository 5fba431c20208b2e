"""Weights by tensor name: what loads, and the one error that lists everything wrong (CPU)."""

import os

import pytest
import torch
from safetensors import safe_open
from safetensors.torch import load_file, save_file

from tests.helpers import TINY_A, TINY_B
from tinyserve_llm_amd import models
from tinyserve_llm_amd.models.decoder import DecoderModel
from tinyserve_llm_amd.weights.loader import WeightsError, load_params
from tinyserve_llm_amd.weights.random_init import write_random_model


def model_of(config):
    return DecoderModel(models.ARCHITECTURES["LlamaForCausalLM"].build_spec(config))


def test_random_folder_has_the_checkpoint_names_and_loads(tmp_path):
    write_random_model(str(tmp_path), TINY_B, 1, torch.bfloat16)
    assert sorted(os.listdir(tmp_path)) == ["config.json", "model.safetensors"]
    stored = load_file(str(tmp_path / "model.safetensors"))
    assert "lm_head.weight" in stored and stored["model.layers.2.self_attn.k_proj.weight"].shape == (32, 96)
    assert all(t.dtype == torch.bfloat16 for t in stored.values())
    m = model_of(TINY_B)
    p16 = load_params(m, str(tmp_path), torch.bfloat16, "cpu")
    p32 = load_params(m, str(tmp_path), torch.float32, "cpu")
    assert all(t.dtype == torch.bfloat16 for t in p16.values()) and all(t.dtype == torch.float32 for t in p32.values())
    q, kv = TINY_B.q_size, TINY_B.kv_size
    fused = p32["layers.1.mixer.qkv"]
    assert torch.equal(fused[:q], stored["model.layers.1.self_attn.q_proj.weight"].float())
    assert torch.equal(fused[q:q + kv], stored["model.layers.1.self_attn.k_proj.weight"].float())
    assert torch.equal(fused[q + kv:], stored["model.layers.1.self_attn.v_proj.weight"].float())
    gu = p32["layers.0.ff.gate_up"]
    assert torch.equal(gu[:160], stored["model.layers.0.mlp.gate_proj.weight"].float())
    assert torch.equal(gu[160:], stored["model.layers.0.mlp.up_proj.weight"].float())
    assert not torch.equal(p32["head.weight"], p32["embed.weight"])


def test_same_seed_same_weights_other_seed_other_weights(tmp_path):
    a, b, c = tmp_path / "a", tmp_path / "b", tmp_path / "c"
    write_random_model(str(a), TINY_A, 0, torch.float32)
    write_random_model(str(b), TINY_A, 0, torch.float32)
    write_random_model(str(c), TINY_A, 5, torch.float32)
    sa, sb, sc = (load_file(str(x / "model.safetensors")) for x in (a, b, c))
    assert all(torch.equal(sa[k], sb[k]) for k in sa) and not torch.equal(sa["model.norm.weight"], sc["model.norm.weight"])
    assert "lm_head.weight" not in sa, "tied: the head is the embedding"
    norm, lin = sa["model.layers.0.input_layernorm.weight"], sa["model.embed_tokens.weight"]
    assert abs(float(norm.mean()) - 1.0) < 0.1 and 0.05 < float(norm.std()) < 0.15
    assert abs(float(lin.mean())) < 0.002 and 0.018 < float(lin.std()) < 0.022


def test_two_shards_and_a_tied_copy_of_the_head(tmp_path):
    write_random_model(str(tmp_path), TINY_A, 0, torch.float32)
    stored = load_file(str(tmp_path / "model.safetensors"))
    os.remove(tmp_path / "model.safetensors")
    names = sorted(stored)
    half = len(names) // 2
    first = {k: stored[k] for k in names[:half]}
    first["lm_head.weight"] = stored["model.embed_tokens.weight"].clone()     # allowed when tied
    first["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.ones(8)       # old checkpoints carry these
    save_file(first, str(tmp_path / "model-00001-of-00002.safetensors"))
    save_file({k: stored[k] for k in names[half:]}, str(tmp_path / "model-00002-of-00002.safetensors"))
    params = load_params(model_of(TINY_A), str(tmp_path), torch.float32, "cpu")
    assert torch.equal(params["embed.weight"], stored["model.embed_tokens.weight"]) and "head.weight" not in params


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    write_random_model(str(tmp_path), TINY_B, 1, torch.float32)
    stored = load_file(str(tmp_path / "model.safetensors"))
    del stored["model.layers.1.mlp.up_proj.weight"]
    del stored["lm_head.weight"]
    stored["model.layers.0.self_attn.o_proj.weight"] = torch.zeros(96, 95)
    stored["model.layers.9.mlp.down_proj.weight"] = torch.zeros(2, 2)
    save_file(stored, str(tmp_path / "model.safetensors"))
    with pytest.raises(WeightsError, match="did not fill") as e:
        load_params(model_of(TINY_B), str(tmp_path), torch.float32, "cpu")
    assert e.value.missing == ["lm_head.weight", "model.layers.1.mlp.up_proj.weight"]
    assert e.value.unexpected == ["model.layers.9.mlp.down_proj.weight"]
    assert len(e.value.wrong_shape) == 1 and "o_proj" in e.value.wrong_shape[0] and "[96, 95]" in e.value.wrong_shape[0]
    text = str(e.value)
    assert "unexpected tensors" in text and "wrong shapes" in text and isinstance(e.value, ValueError)


def test_missing_shard_is_reported_not_half_loaded(tmp_path):
    """tests/test_llama.py:189-194 of the reference: an incomplete checkpoint raises 'did not fill'."""
    write_random_model(str(tmp_path), TINY_B, 1, torch.float32)
    stored = load_file(str(tmp_path / "model.safetensors"))
    os.remove(tmp_path / "model.safetensors")
    names = sorted(stored)
    save_file({k: stored[k] for k in names[:len(names) // 2]}, str(tmp_path / "model-00001-of-00002.safetensors"))
    with pytest.raises(ValueError, match="did not fill"):
        load_params(model_of(TINY_B), str(tmp_path), torch.float32, "cpu")


def test_no_files(tmp_path):
    TINY_A.save(str(tmp_path))
    with pytest.raises(FileNotFoundError, match="safetensors"):
        load_params(model_of(TINY_A), str(tmp_path), torch.float32, "cpu")
    with pytest.raises(FileNotFoundError, match="config.json"):
        models.read_config(str(tmp_path / "nothing"))


def test_stored_types_are_kept_in_the_file(tmp_path):
    write_random_model(str(tmp_path), TINY_A, 0, torch.float32)
    with safe_open(str(tmp_path / "model.safetensors"), "pt", "cpu") as f:
        assert f.get_tensor("model.norm.weight").dtype == torch.float32


def test_destinations_slice_columns_transpose_and_fill_stacks(tmp_path):
    """What a checkpoint table can say beyond rows: a tensor may land in a column range, in one
    matrix of a stacked parameter, or transposed; wrong shapes are reported in the checkpoint's own
    orientation, and the random-weights mode writes the same tensors back out."""
    import torch
    from safetensors.torch import save_file
    from tinyserve_llm_amd.models.decoder import DecoderModel
    from tinyserve_llm_amd.models.spec import Destination, LayerRun, LayerSpec, ModelSpec
    from tinyserve_llm_amd.parts.base import FeedForward, ParamSpec, PartSpec, register
    from tinyserve_llm_amd.weights.loader import WeightsError, load_params
    from tinyserve_llm_amd.weights.random_init import checkpoint_tensors, random_params

    @register("feed_forward", "toy_stacked")
    class Stacked(FeedForward):
        def __init__(self, hidden_size, experts):
            self.hidden_size, self.experts = hidden_size, experts

        def param_specs(self):
            return {"w": ParamSpec((self.experts, self.hidden_size, self.hidden_size)),
                    "wide": ParamSpec((self.hidden_size, 3 * self.hidden_size))}

    h = 8
    norm = PartSpec("rmsnorm", dict(hidden_size=h, eps=1e-5))
    layer = LayerSpec.pre_norm(PartSpec("attention", dict(hidden_size=h, num_heads=1, num_kv_heads=1, head_dim=16)),
                               PartSpec("toy_stacked", dict(hidden_size=h, experts=2)), norm, norm)
    table = {"emb": Destination("embed.weight"), "n0": Destination("layers.0.mixer_norm.weight"),
             "n1": Destination("layers.0.ff_norm.weight"), "nf": Destination("final_norm.weight"),
             "qkv": Destination("layers.0.mixer.qkv"), "o_t": Destination("layers.0.mixer.o", transpose=True),
             "e0": Destination("layers.0.ff.w", index=(0,)), "e1_t": Destination("layers.0.ff.w", index=(1,), transpose=True),
             "left": Destination("layers.0.ff.wide", col=0, cols=h), "right": Destination("layers.0.ff.wide", col=h, cols=2 * h)}
    spec = ModelSpec("ToyW", 20, h, 32, [layer], [LayerRun(0)], norm, tie_word_embeddings=True, checkpoint=table,
                     position_encodings={"rope": PartSpec("rope", dict(head_dim=16, max_position=32, theta=10000.0))})
    model = DecoderModel(spec)
    params = random_params(model, 1, torch.float32)
    tensors = checkpoint_tensors(model, params)
    assert tensors["o_t"].shape == (16, h) and tensors["e1_t"].shape == (h, h) and tensors["right"].shape == (h, 2 * h)
    assert torch.equal(tensors["o_t"], params["layers.0.mixer.o"].t()) and torch.equal(tensors["e0"], params["layers.0.ff.w"][0])
    save_file(tensors, str(tmp_path / "model.safetensors"))
    loaded = load_params(model, str(tmp_path), torch.float32, "cpu")
    assert all(torch.equal(loaded[k], params[k]) for k in params)
    tensors["o_t"] = tensors["o_t"].t().contiguous()          # stored the model's way round: not what the table says
    del tensors["left"]
    save_file(tensors, str(tmp_path / "model.safetensors"))
    with pytest.raises(WeightsError) as e:
        load_params(model, str(tmp_path), torch.float32, "cpu")
    assert e.value.missing == ["left"] and e.value.wrong_shape == [f"o_t: checkpoint [{h}, 16], model [16, {h}]"]
