"""Each part of a layer alone on the GPU against its plain counterpart, built from explicit sizes
that no model of the tests uses; then parts the framework does not have (a mixer with state of its
own, a routed feed-forward, another position encoding) registered from here and stepped through
the unchanged engine; then the run order as data (a layer named twice, a layer reading another
layer's cache)."""

from __future__ import annotations

import pytest
import torch

from tests.helpers import prompt
from tests.plain import llama as P

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]
DEV = "cuda:0"


def tol(dtype):
    return dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=3e-2, atol=3e-2)


def context(lengths, starts, page, tables, encodings=None):
    """A StepContext by hand: requests with `lengths[i]` tokens starting at `starts[i]`."""
    from tinyserve_llm_amd.parts.base import StepContext
    pos, seq_of, slots, cu = [], [], [], [0]
    for s, (n, st) in enumerate(zip(lengths, starts)):
        pos += list(range(st, st + n))
        seq_of += [s] * n
        slots += [tables[s][p // page] * page + p % page for p in range(st, st + n)]
        cu.append(cu[-1] + n)
    width = max(len(t) for t in tables)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
    return StepContext(
        num_tokens=len(pos), num_seqs=len(lengths), token_ids=i32([0] * len(pos)), positions=i32(pos),
        seq_of_token=i32(seq_of), cu_seqlens=i32(cu), context_lens=i32([a + b for a, b in zip(lengths, starts)]),
        state_slots=i32(list(range(len(lengths)))), slot_mapping=[torch.tensor(slots, dtype=torch.int32, device=DEV)],
        block_tables=[i32([t + [0] * (width - len(t)) for t in tables])], host_cu_seqlens=cu, host_starts=list(starts),
        host_context_lens=[a + b for a, b in zip(lengths, starts)], host_state_slots=list(range(len(lengths))),
        position_encodings=encodings or {})


def bound(part, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    params = {}
    for name, ps in part.param_specs().items():
        mean, std = ps.init
        params[name] = (torch.randn(ps.shape, generator=g) * max(std, 0.05) + mean).to(dtype)
    part.bind({k: v.to(DEV) for k, v in params.items()})
    return {k: v.double() for k, v in params.items()}


@pytest.mark.parametrize("dtype", DTYPES)
def test_rmsnorm_part(dtype):
    from tinyserve_llm_amd.parts.norm import RMSNorm
    part = RMSNorm(hidden_size=176, eps=3e-6)
    w = bound(part, dtype, 0)["weight"]
    x, r = torch.randn(5, 176).to(dtype), torch.randn(5, 176).to(dtype)
    out, res = part(x.to(DEV), r.to(DEV))
    want, s = P.add_rms_norm(x.double(), r.double(), w, 3e-6)
    torch.testing.assert_close(out.double().cpu(), want, **tol(dtype))
    torch.testing.assert_close(res.double().cpu(), s, **tol(dtype))


def test_rope_part_table_is_the_reference_table():
    from tinyserve_llm_amd.parts.rope import Rope
    scaling = dict(factor=4.0, low_freq_factor=1.0, high_freq_factor=4.0, original_max_position_embeddings=32)
    part = Rope(head_dim=48, max_position=200, theta=12345.0, scaling=scaling)
    part.prepare(torch.device(DEV))
    cos, sin = P.rope_tables(48, 12345.0, scaling, 200, 200, torch.float32)
    assert torch.equal(part.rotary_table().cpu(), torch.cat((cos, sin), -1)), "bit-equal: same float32 operations"
    assert torch.equal(Rope(48, 200, 12345.0).inv_freq, P.rope_inv_freq(48, 12345.0, None, 200))


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_part_over_two_steps(dtype):
    """A prompt portion then the rest beside a second request: projections, rotation, cache
    write, attention over the pages and output projection against the plain parts."""
    from tinyserve_llm_amd.parts.attention import Attention
    from tinyserve_llm_amd.parts.base import LayerMemory
    from tinyserve_llm_amd.parts.rope import Rope
    hidden, heads, kv, hd, page = 80, 6, 2, 48, 8
    part = Attention(hidden_size=hidden, num_heads=heads, num_kv_heads=kv, head_dim=hd, position="rope")
    w = bound(part, dtype, 1)
    rope = Rope(hd, 64, 10000.0)
    rope.prepare(torch.device(DEV))
    mem = LayerMemory(k_cache=torch.zeros(6, page, kv, hd, dtype=dtype, device=DEV),
                      v_cache=torch.zeros(6, page, kv, hd, dtype=dtype, device=DEV))
    xa, xb = torch.randn(19, hidden).to(dtype), torch.randn(5, hidden).to(dtype)
    ta, tb = [4, 0, 2], [5]
    part.forward(xa[:11].to(DEV), context([11], [0], page, [ta], {"rope": rope}), mem)
    out = part.forward(torch.cat([xa[11:], xb]).to(DEV), context([8, 5], [11, 0], page, [ta, tb], {"rope": rope}), mem)

    def plain(x):
        n = x.shape[0]
        qkv = x.double() @ w["qkv"].T
        q, k, v = qkv[:, :heads * hd], qkv[:, heads * hd:(heads + kv) * hd], qkv[:, (heads + kv) * hd:]
        cos, sin = P.rope_tables(hd, 10000.0, None, 64, n, torch.float64)
        q, k = P.apply_rope(q.view(n, heads, hd), cos, sin), P.apply_rope(k.view(n, kv, hd), cos, sin)
        return P.causal_attention(q, k, v.view(n, kv, hd)).reshape(n, heads * hd) @ w["o"].T

    want = torch.cat([plain(xa)[11:], plain(xb)])
    torch.testing.assert_close(out.double().cpu(), want, **tol(dtype))
    assert part.kv_spec().num_kv_heads == kv and part.kv_spec().head_dim == hd and part.state_spec() is None


@pytest.mark.parametrize("dtype", DTYPES)
def test_gated_mlp_part(dtype):
    from tinyserve_llm_amd.parts.mlp import GatedMLP
    part = GatedMLP(hidden_size=72, intermediate_size=200)
    w = bound(part, dtype, 2)
    x = torch.randn(9, 72).to(dtype)
    out = part.forward(x.to(DEV), None)
    want = P.silu_mul(x.double() @ w["gate_up"].T) @ w["down"].T
    torch.testing.assert_close(out.double().cpu(), want, **tol(dtype))
    with pytest.raises(ValueError, match="silu"):
        GatedMLP(8, 8, activation="gelu")


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_part_with_a_rotation_of_part_of_the_head(dtype):
    """The attention part with a position encoding that turns 32 of a head's 64 dimensions: a step
    of a few tokens, which would take the one-kernel projection if heads turned whole, and a longer
    one, both against the plain formulas with the rotation applied to the leading part."""
    from tinyserve_llm_amd.parts.attention import Attention
    from tinyserve_llm_amd.parts.rope import Rope
    hidden, nh, nkv, hd, rot, page = 256, 4, 2, 64, 32, 16
    part = Attention(hidden_size=hidden, num_heads=nh, num_kv_heads=nkv, head_dim=hd, position="rope")
    w = bound(part, dtype, 3)
    rope = Rope(head_dim=hd, max_position=128, theta=10000.0, rotary_dim=rot)
    rope.prepare(torch.device(DEV))
    assert rope.rotary_table().shape == (128, rot)
    from tinyserve_llm_amd.parts.base import LayerMemory
    for n in (5, 70):
        x = (torch.randn(n, hidden, generator=torch.Generator().manual_seed(n)) * 0.5).to(dtype)
        pages = -(-n // page)
        kc = torch.zeros(pages, nkv, page, hd, dtype=dtype, device=DEV).permute(0, 2, 1, 3)
        vc = torch.zeros(pages, nkv, hd, page, dtype=dtype, device=DEV).permute(0, 3, 1, 2)
        ctx = context([n], [0], page, [list(range(pages))], {"rope": rope})
        out = part.forward(x.to(DEV), ctx, LayerMemory(k_cache=kc, v_cache=vc))
        cos, sin = P.rope_tables(rot, 10000.0, None, 128, n, torch.float64)
        qkv = x.double() @ w["qkv"].T
        q, k, v = qkv[:, :nh * hd].view(n, nh, hd), qkv[:, nh * hd:(nh + nkv) * hd].view(n, nkv, hd), qkv[:, (nh + nkv) * hd:].view(n, nkv, hd)
        turn = lambda t: torch.cat((P.apply_rope(t[..., :rot], cos, sin), t[..., rot:]), -1)
        want = P.causal_attention(turn(q), turn(k), v).reshape(n, nh * hd) @ w["o"].T
        torch.testing.assert_close(out.double().cpu(), want, **tol(dtype))


# ---- parts from outside the framework --------------------------------------------------------------

def register_toy_parts():
    from tinyserve_llm_amd.parts.base import (FeedForward, Mixer, ParamSpec, PositionEncoding, StateSpec, register)

    @register("mixer", "toy_running_mean")
    class RunningMean(Mixer):
        """y_t = W · mean(x_0..x_t): no keys, only a per-request state (sum, count)."""

        def __init__(self, hidden_size):
            self.hidden_size = hidden_size

        def param_specs(self):
            return {"w": ParamSpec((self.hidden_size, self.hidden_size), init=(0.0, 0.1))}

        def state_spec(self):
            return StateSpec((self.hidden_size + 1,), torch.float32)

        def forward(self, x, ctx, mem):
            out = torch.empty_like(x)
            for s in range(ctx.num_seqs):
                a, b = ctx.host_cu_seqlens[s], ctx.host_cu_seqlens[s + 1]
                state = mem.state[ctx.host_state_slots[s]]
                if ctx.host_starts[s] == 0:
                    state.zero_()
                sums = state[:-1] + torch.cumsum(x[a:b].float(), 0)
                counts = state[-1] + torch.arange(1, b - a + 1, device=x.device)
                out[a:b] = ((sums / counts[:, None]).to(x.dtype) @ self.w.T)
                state[:-1] = sums[-1]
                state[-1] = counts[-1]
            return out

    @register("mixer", "toy_running_mean_on_device")
    class RunningMeanOnDevice(RunningMean):
        """The same mixer from the step's device tensors alone (no host lists, no branches on
        them), so that decode steps with it can be recorded into graphs and replayed."""

        graph_safe = True

        def forward(self, x, ctx, mem):
            seq, slots, cu = ctx.seq_of_token.long(), ctx.state_slots.long(), ctx.cu_seqlens.long()
            carried = mem.state[slots] * (ctx.positions.long()[cu[:-1]] != 0).unsqueeze(1)   # a request's first token starts it
            run = torch.cumsum(x.float(), 0)
            before = torch.cat([run.new_zeros(1, run.shape[1]), run])[cu[:-1]]                # the sum up to each request's rows
            sums = carried[seq, :-1] + (run - before[seq])
            counts = (ctx.positions + 1).float()
            last = cu[1:] - 1
            mem.state[slots] = torch.cat([sums[last], counts[last, None]], 1)
            return (sums / counts[:, None]).to(x.dtype) @ self.w.T

    @register("feed_forward", "toy_routed")
    class Routed(FeedForward):
        """Top-1 of E small experts, chosen by a 32-bit router."""

        graph_safe = True

        def __init__(self, hidden_size, experts):
            self.hidden_size, self.experts = hidden_size, experts

        def param_specs(self):
            return {"router": ParamSpec((self.experts, self.hidden_size), storage="float32", init=(0.0, 0.5)),
                    "w": ParamSpec((self.experts * self.hidden_size, self.hidden_size), init=(0.0, 0.1))}

        def forward(self, x, ctx):
            choice = (x.float() @ self.router.T).argmax(-1)
            w = self.w.view(self.experts, self.hidden_size, self.hidden_size)[choice]
            return torch.einsum("toh,th->to", w.float(), x.float()).to(x.dtype)

    @register("position_encoding", "toy_learned")
    class Learned(PositionEncoding):
        """A learned vector per position, added to the embedded tokens."""

        graph_safe = True

        def __init__(self, hidden_size, max_position):
            self.hidden_size, self.max_position = hidden_size, max_position

        def param_specs(self):
            return {"table": ParamSpec((self.max_position, self.hidden_size), init=(0.0, 0.3))}

        def on_embedding(self, hidden, ctx):
            return hidden + self.table[ctx.positions.long()]


def toy_spec(hidden=48, vocab=97, mean_mixer="toy_running_mean"):
    from tinyserve_llm_amd.models.spec import LayerRun, LayerSpec, ModelSpec
    from tinyserve_llm_amd.parts.base import PartSpec
    norm = PartSpec("rmsnorm", dict(hidden_size=hidden, eps=1e-5))
    mlp = PartSpec("gated_mlp", dict(hidden_size=hidden, intermediate_size=64))
    attn = PartSpec("attention", dict(hidden_size=hidden, num_heads=3, num_kv_heads=1, head_dim=16, position=None))
    layers = [LayerSpec.pre_norm(PartSpec(mean_mixer, dict(hidden_size=hidden)), mlp, norm, norm),
              LayerSpec.pre_norm(attn, PartSpec("toy_routed", dict(hidden_size=hidden, experts=3)), norm, norm)]
    return ModelSpec(architecture="Toy", vocab_size=vocab, hidden_size=hidden, max_position=128, layers=layers,
                     order=[LayerRun(0), LayerRun(1), LayerRun(0)], final_norm=norm,
                     position_encodings={"learned": PartSpec("toy_learned", dict(hidden_size=hidden, max_position=128))},
                     tie_word_embeddings=True)


def toy_engine(dtype, seed=0, pages=24, page=8):
    from tinyserve_llm_amd.cache.manager import KVCacheManager
    from tinyserve_llm_amd.cache.storage import KVStorage
    from tinyserve_llm_amd.engine.runner import ModelRunner
    from tinyserve_llm_amd.models.decoder import DecoderModel
    from tinyserve_llm_amd.weights.random_init import random_params
    register_toy_parts()
    model = DecoderModel(toy_spec())
    params = random_params(model, seed, dtype, "cpu")
    model.bind({k: v.to(DEV) for k, v in params.items()}, dtype, torch.device(DEV))
    storage = KVStorage(model.cache_plan(), model.state_plan(), pages, page, dtype, DEV, num_state_slots=4)
    manager = KVCacheManager(storage)
    assert not manager.caching, "a model with state slots reuses no prefix"
    return model, {k: v.double() for k, v in params.items()}, storage, manager, ModelRunner(model, storage, manager)


def toy_plain(p, ids):
    """The toy model whole, in float64, from its definition."""
    n = len(ids)
    h = p["embed.weight"][torch.tensor(ids)] + p["positions.learned.table"][:n]

    def mean_mixer(x, w):
        return (torch.cumsum(x, 0) / torch.arange(1, n + 1)[:, None].double()) @ w.T

    def layer0(h):
        x = P.rms_norm(h, p["layers.0.mixer_norm.weight"], 1e-5)
        h = h + mean_mixer(x, p["layers.0.mixer.w"])
        x = P.rms_norm(h, p["layers.0.ff_norm.weight"], 1e-5)
        return h + P.silu_mul(x @ p["layers.0.ff.gate_up"].T) @ p["layers.0.ff.down"].T

    h = layer0(h)
    x = P.rms_norm(h, p["layers.1.mixer_norm.weight"], 1e-5)
    qkv = x @ p["layers.1.mixer.qkv"].T
    o = P.causal_attention(qkv[:, :48].reshape(n, 3, 16), qkv[:, 48:64].reshape(n, 1, 16), qkv[:, 64:].reshape(n, 1, 16))
    h = h + o.reshape(n, 48) @ p["layers.1.mixer.o"].T
    x = P.rms_norm(h, p["layers.1.ff_norm.weight"], 1e-5)
    choice = (x @ p["layers.1.ff.router"].T).argmax(-1)
    w = p["layers.1.ff.w"].view(3, 48, 48)[choice]
    h = h + torch.einsum("toh,th->to", w, x)
    h = layer0(h)                                     # the same layer, named twice in the order
    return P.rms_norm(h, p["final_norm.weight"], 1e-5) @ p["embed.weight"].T


def test_toy_parts_register_build_and_step_without_touching_the_framework():
    """A mixer with state of its own, a routed feed-forward and a learned position encoding,
    defined above, run through the framework's model, cache manager, storage and step function
    in portions and beside another request; layer 0 is named twice in the run order and has a
    state slot per run."""
    from tinyserve_llm_amd.engine.runner import StepEntry
    model, p, storage, manager, runner = toy_engine(torch.float32)
    assert [e.run for e in model.state_plan()] == [0, 2] and [e.owner for e in model.cache_plan()] == [1]
    assert storage.state(0).shape == (4, 49) and storage.state(1) is None
    a, b = [3, 50, 7, 7, 96, 1, 0, 22, 41, 5, 88, 13, 2], [9, 8, 7, 6, 5]
    want_a, want_b = toy_plain(p, a), toy_plain(p, b)
    got = {}
    manager.allocate(0, a[:4])
    out = runner.step([StepEntry(0, a[:4], 0, [0, 3])])
    got[("a", 0)], got[("a", 3)] = out[0], out[1]
    manager.commit(0, 4)
    manager.allocate(1, b)
    manager.append_slots(0, a[4:6])
    out = runner.step([StepEntry(1, b, 0, [4]), StepEntry(0, a[4:6], 4, [1])])
    got[("b", 4)], got[("a", 5)] = out[0], out[1]
    manager.commit(0, 2)
    manager.commit(1, 5)
    manager.release(1)
    for pos in range(6, len(a)):
        manager.append_slots(0, [a[pos]])
        got[("a", pos)] = runner.step([StepEntry(0, [a[pos]], pos, [0])])[0]
        manager.commit(0, 1)
    for (name, pos), row in got.items():
        want = (want_a if name == "a" else want_b)[pos]
        torch.testing.assert_close(row.double().cpu(), want, rtol=1e-4, atol=1e-5, msg=lambda m: f"{name}{pos}: {m}")
    manager.release(0)
    assert manager.num_available_blocks() == manager.num_blocks and len(manager.free_state_slots) == 4


def test_a_model_with_state_generates_through_the_entry_point_with_every_default():
    """The toy model whose mixer keeps state, through `LLM.generate` as any model goes: prefix reuse
    asked for (the default), prompts that share prefixes and repeat, portions, a pool so small that
    requests give up their pages and come back, decode steps replayed from graphs. A reused prefix
    or a step counted twice would leave tokens out of, or twice in, the running mean."""
    from tinyserve_llm_amd.engine.llm import LLM, CacheConfig
    from tinyserve_llm_amd.engine.scheduler import SchedulerConfig
    from tinyserve_llm_amd.engine.sequence import SamplingParams
    from tinyserve_llm_amd.models.decoder import DecoderModel
    from tinyserve_llm_amd.weights.random_init import random_params
    register_toy_parts()
    model = DecoderModel(toy_spec(mean_mixer="toy_running_mean_on_device"))
    params = random_params(model, 5, torch.float32, "cpu")
    model.bind({k: v.to(DEV) for k, v in params.items()}, torch.float32, torch.device(DEV))
    p = {k: v.double() for k, v in params.items()}

    def plain_greedy(ids, n):
        ids, out = list(ids), []
        for _ in range(n):
            out.append(int(toy_plain(p, ids)[-1].argmax()))
            ids.append(out[-1])
        return out

    shared = [3, 50, 7, 7, 96, 1, 0, 22, 41]
    prompts = [shared + [5], shared + [88, 13], shared[:6], [9, 8, 7, 6, 5], shared + [5], shared[:8] + [60]]
    want = [plain_greedy(q, 10) for q in prompts]
    sc = SchedulerConfig(max_model_len=64, max_num_seqs=4, max_num_batched_tokens=24, max_prefill_chunk=7)
    llm = LLM(None, sc, CacheConfig(block_size=4), model=model, num_blocks=16)
    assert llm.runner.graphs is not None, "every toy part is recordable"
    assert not llm.manager.caching, "the manager has seen the state slots"
    sp = SamplingParams(max_tokens=10, temperature=0.0, ignore_eos=True)
    for _ in range(2):           # the second round finds the first round's pages free, and must not reuse them
        got = llm.generate(prompts, sp)
        assert [r.token_ids[0] for r in got] == want
    st = llm.scheduler.stats()
    assert st.preemptions > 0 and st.cached_tokens == 0
    assert len(llm.runner.graphs.graphs) > 0, "decode steps were replayed from graphs"
    assert llm.manager.stats().blocks_in_use == 0 and len(llm.manager.free_state_slots) == 4


def test_a_layer_can_read_another_layers_cache():
    """order = [layer 0 (owns a cache), layer 1 reading layer 0's cache without writing]:
    layer 1's queries attend over layer 0's keys and values."""
    from tinyserve_llm_amd.cache.manager import KVCacheManager
    from tinyserve_llm_amd.cache.storage import KVStorage
    from tinyserve_llm_amd.engine.runner import ModelRunner, StepEntry
    from tinyserve_llm_amd.models.decoder import DecoderModel
    from tinyserve_llm_amd.models.spec import LayerRun, LayerSpec, ModelSpec
    from tinyserve_llm_amd.parts.base import PartSpec
    from tinyserve_llm_amd.weights.random_init import random_params
    hidden = 32
    norm = PartSpec("rmsnorm", dict(hidden_size=hidden, eps=1e-5))
    layer = LayerSpec.pre_norm(PartSpec("attention", dict(hidden_size=hidden, num_heads=2, num_kv_heads=2, head_dim=16, position=None)),
                      PartSpec("gated_mlp", dict(hidden_size=hidden, intermediate_size=48)), norm, norm)
    spec = ModelSpec("Toy2", 50, hidden, 64, [layer, layer], [LayerRun(0), LayerRun(1, cache=0, store=False)], norm,
                     tie_word_embeddings=True)
    model = DecoderModel(spec)
    assert len(model.cache_plan()) == 1
    params = random_params(model, 3, torch.float32, "cpu")
    model.bind({k: v.to(DEV) for k, v in params.items()}, torch.float32, torch.device(DEV))
    p = {k: v.double() for k, v in params.items()}
    storage = KVStorage(model.cache_plan(), model.state_plan(), 8, 4, torch.float32, DEV, 2)
    manager = KVCacheManager(storage, caching=False)
    runner = ModelRunner(model, storage, manager)
    ids = [4, 9, 33, 2, 17, 8, 40]
    n = len(ids)
    h = p["embed.weight"][torch.tensor(ids)]
    x = P.rms_norm(h, p["layers.0.mixer_norm.weight"], 1e-5)
    qkv0 = x @ p["layers.0.mixer.qkv"].T
    k0, v0 = qkv0[:, 32:64].reshape(n, 2, 16), qkv0[:, 64:].reshape(n, 2, 16)
    h = h + P.causal_attention(qkv0[:, :32].reshape(n, 2, 16), k0, v0).reshape(n, 32) @ p["layers.0.mixer.o"].T
    x = P.rms_norm(h, p["layers.0.ff_norm.weight"], 1e-5)
    h = h + P.silu_mul(x @ p["layers.0.ff.gate_up"].T) @ p["layers.0.ff.down"].T
    x = P.rms_norm(h, p["layers.1.mixer_norm.weight"], 1e-5)
    q1 = (x @ p["layers.1.mixer.qkv"].T)[:, :32].reshape(n, 2, 16)
    h = h + P.causal_attention(q1, k0, v0).reshape(n, 32) @ p["layers.1.mixer.o"].T
    x = P.rms_norm(h, p["layers.1.ff_norm.weight"], 1e-5)
    h = h + P.silu_mul(x @ p["layers.1.ff.gate_up"].T) @ p["layers.1.ff.down"].T
    want = P.rms_norm(h, p["final_norm.weight"], 1e-5) @ p["embed.weight"].T
    manager.allocate(0, ids[:5])
    first = runner.step([StepEntry(0, ids[:5], 0, list(range(5)))])
    manager.commit(0, 5)
    manager.append_slots(0, ids[5:])
    rest = runner.step([StepEntry(0, ids[5:], 5, [0, 1])])
    torch.testing.assert_close(torch.cat([first, rest]).double().cpu(), want, rtol=1e-4, atol=1e-5)


def test_bad_orders_are_refused_when_the_model_is_built():
    from tinyserve_llm_amd.models.decoder import DecoderModel
    from tinyserve_llm_amd.models.spec import LayerRun
    register_toy_parts()
    spec = toy_spec()
    spec.order = [LayerRun(0), LayerRun(1, cache=2)]
    with pytest.raises(ValueError, match="does not run before"):
        DecoderModel(spec)
    spec.order = [LayerRun(5)]
    with pytest.raises(ValueError, match="names layer 5"):
        DecoderModel(spec)
    spec.order = [LayerRun(1, store=False)]
    with pytest.raises(ValueError, match="neither owns"):
        DecoderModel(spec)
    from dataclasses import replace
    from tinyserve_llm_amd.parts.base import PartSpec
    spec.order = [LayerRun(0), LayerRun(1)]
    good = spec.layers[1]
    spec.layers[1] = replace(good, mixer=PartSpec("no_such_mixer", {}))
    with pytest.raises(KeyError, match="no mixer named"):
        DecoderModel(spec)
    spec.layers[1] = replace(good, norms={"mixer_norm": good.norms["mixer_norm"]})
    with pytest.raises(KeyError, match=r"asks for the norms \['ff_norm'\]"):
        DecoderModel(spec)
    spec.layers[1] = replace(good, block="no_such_block")
    with pytest.raises(KeyError, match="no block arrangement"):
        DecoderModel(spec)


def test_another_block_arrangement_another_embedding_and_another_head():
    """Parts of the kinds the built-in model has one of each, defined here: a block that runs mixer and
    feed-forward side by side from one norm and normalises each branch again on the way out (three
    norms under names of its own), an embedding that scales its rows, and a head that caps its
    logits. They are registered, named in a model description, built, bound to random weights and
    stepped in portions through the unchanged framework, against the same model written out plainly."""
    from tinyserve_llm_amd.engine.interface import build_cache
    from tinyserve_llm_amd.engine.runner import ModelRunner, StepEntry
    from tinyserve_llm_amd.models.decoder import DecoderModel
    from tinyserve_llm_amd.models.spec import LayerRun, LayerSpec, ModelSpec
    from tinyserve_llm_amd.parts.base import Embedding, Head, ParamSpec, PartSpec, register
    from tinyserve_llm_amd.parts.block import uses_norms
    from tinyserve_llm_amd.weights.random_init import random_params

    @register("block", "toy_side_by_side")
    @uses_norms("in_norm", "mixer_out_norm", "ff_out_norm")
    def side_by_side(layer, hidden, residual, ctx, mem):
        x, stream = layer.norms["in_norm"](hidden, residual)               # (norm(h), h) with h = hidden + residual
        a, _ = layer.norms["mixer_out_norm"](layer.mixer.forward(x, ctx, mem))
        b, _ = layer.norms["ff_out_norm"](layer.feed_forward.forward(x, ctx))
        return a + b, stream

    @register("embedding", "toy_scaled")
    class Scaled(Embedding):
        def __init__(self, vocab_size, hidden_size, scale):
            self.vocab_size, self.hidden_size, self.scale = vocab_size, hidden_size, scale

        def param_specs(self):
            return {"rows": ParamSpec((self.vocab_size, self.hidden_size), init=(0.0, 0.3))}

        def forward(self, ctx):
            return self.rows[ctx.token_ids.long()] * self.scale

    @register("head", "toy_capped")
    class Capped(Head):
        def __init__(self, vocab_size, hidden_size, cap):
            self.vocab_size, self.hidden_size, self.cap = vocab_size, hidden_size, cap

        def param_specs(self):
            return {"w": ParamSpec((self.vocab_size, self.hidden_size), init=(0.0, 0.5))}

        def forward(self, rows):
            return self.cap * torch.tanh((rows.float() @ self.w.float().T) / self.cap)

    hidden, vocab = 32, 61
    norm = PartSpec("rmsnorm", dict(hidden_size=hidden, eps=1e-6))
    layer = LayerSpec(PartSpec("attention", dict(hidden_size=hidden, num_heads=2, num_kv_heads=1, head_dim=16, position=None)),
                      PartSpec("gated_mlp", dict(hidden_size=hidden, intermediate_size=48)),
                      {"in_norm": norm, "mixer_out_norm": norm, "ff_out_norm": norm}, block="toy_side_by_side")
    spec = ModelSpec("Toy3", vocab, hidden, 64, [layer, layer], [LayerRun(0), LayerRun(1)], norm,
                     embedding=PartSpec("toy_scaled", dict(vocab_size=vocab, hidden_size=hidden, scale=2.5)),
                     head=PartSpec("toy_capped", dict(vocab_size=vocab, hidden_size=hidden, cap=3.0)))
    model = DecoderModel(spec)
    assert sorted(n for n in model.param_specs() if n.startswith("layers.0.") and "norm" in n) == [
        "layers.0.ff_out_norm.weight", "layers.0.in_norm.weight", "layers.0.mixer_out_norm.weight"]
    assert "embed.rows" in model.param_specs() and "head.w" in model.param_specs() and not model.graph_safe()
    params = random_params(model, 8, torch.float32, "cpu")
    model.bind({k: v.to(DEV) for k, v in params.items()}, torch.float32, torch.device(DEV))
    p = {k: v.double() for k, v in params.items()}
    ids = [4, 9, 33, 2, 17, 8, 40, 60, 0]
    n = len(ids)
    h = p["embed.rows"][torch.tensor(ids)] * 2.5
    for i in range(2):
        w = lambda name: p[f"layers.{i}.{name}"]
        x = P.rms_norm(h, w("in_norm.weight"), 1e-6)
        qkv = x @ w("mixer.qkv").T
        attn = P.causal_attention(qkv[:, :32].reshape(n, 2, 16), qkv[:, 32:48].reshape(n, 1, 16), qkv[:, 48:].reshape(n, 1, 16))
        a = P.rms_norm(attn.reshape(n, 32) @ w("mixer.o").T, w("mixer_out_norm.weight"), 1e-6)
        b = P.rms_norm(P.silu_mul(x @ w("ff.gate_up").T) @ w("ff.down").T, w("ff_out_norm.weight"), 1e-6)
        h = h + a + b
    want = 3.0 * torch.tanh((P.rms_norm(h, p["final_norm.weight"], 1e-6) @ p["head.w"].T) / 3.0)
    storage, manager = build_cache(model, 8, 4, torch.float32, DEV, num_state_slots=2)
    runner = ModelRunner(model, storage, manager)
    manager.allocate(0, ids[:6])
    first = runner.step([StepEntry(0, ids[:6], 0, list(range(6)))])
    manager.commit(0, 6)
    manager.append_slots(0, ids[6:])
    rest = runner.step([StepEntry(0, ids[6:], 6, [0, 1, 2])])
    torch.testing.assert_close(torch.cat([first, rest]).double().cpu(), want, rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_layer_that_reads_a_window_gives_its_pages_back_while_the_engine_steps(dtype):
    """Two layers, one that keeps every key and one that only ever reads the last 10 positions (no
    multiple of the page of 4): the windowed layer has a page space of its own, whose pages go back
    as the window passes them and are taken again by the other request. Portions, single tokens and
    a second request on the same few pages, against attention with the same window written plainly."""
    from tinyserve_llm_amd.engine.interface import build_cache
    from tinyserve_llm_amd.engine.runner import ModelRunner, StepEntry
    from tinyserve_llm_amd.models.decoder import DecoderModel
    from tinyserve_llm_amd.models.spec import LayerRun, LayerSpec, ModelSpec
    from tinyserve_llm_amd.parts.base import PartSpec
    from tinyserve_llm_amd.weights.random_init import random_params
    hidden, window, page = 32, 10, 4
    norm = PartSpec("rmsnorm", dict(hidden_size=hidden, eps=1e-5))
    mlp = PartSpec("gated_mlp", dict(hidden_size=hidden, intermediate_size=48))
    def attn(w):
        return PartSpec("attention", dict(hidden_size=hidden, num_heads=2, num_kv_heads=1, head_dim=16, position="rope", window=w))
    rope = PartSpec("rope", dict(head_dim=16, max_position=96, theta=10000.0))
    spec = ModelSpec("ToyWindow", 50, hidden, 96, [LayerSpec.pre_norm(attn(0), mlp, norm, norm), LayerSpec.pre_norm(attn(window), mlp, norm, norm)],
                     [LayerRun(0), LayerRun(1)], norm, position_encodings={"rope": rope}, tie_word_embeddings=True)
    model = DecoderModel(spec)
    params = random_params(model, 6, dtype, "cpu")
    model.bind({k: v.to(DEV) for k, v in params.items()}, dtype, torch.device(DEV))
    p = {k: v.double() for k, v in params.items()}
    storage, manager = build_cache(model, [24, 8], page, dtype, DEV, num_state_slots=2)    # 8 pages for the window: two requests cannot keep all theirs
    assert [s.window for s in storage.spaces] == [0, window] and not manager.caching
    runner = ModelRunner(model, storage, manager)

    def plain(ids):
        n = len(ids)
        cos, sin = P.rope_tables(16, 10000.0, None, 96, n, torch.float64)
        h = p["embed.weight"][torch.tensor(ids)]
        for i, w in enumerate((0, window)):
            x = P.rms_norm(h, p[f"layers.{i}.mixer_norm.weight"], 1e-5)
            qkv = x @ p[f"layers.{i}.mixer.qkv"].T
            q, k = P.apply_rope(qkv[:, :32].reshape(n, 2, 16), cos, sin), P.apply_rope(qkv[:, 32:48].reshape(n, 1, 16), cos, sin)
            o = P.causal_attention(q, k, qkv[:, 48:].reshape(n, 1, 16), window=w)
            h = h + o.reshape(n, 32) @ p[f"layers.{i}.mixer.o"].T
            x = P.rms_norm(h, p[f"layers.{i}.ff_norm.weight"], 1e-5)
            h = h + P.silu_mul(x @ p[f"layers.{i}.ff.gate_up"].T) @ p[f"layers.{i}.ff.down"].T
        return P.rms_norm(h, p["final_norm.weight"], 1e-5) @ p["embed.weight"].T

    a, b = prompt(1, 41, 50), prompt(2, 23, 50)
    want = {0: plain(a), 1: plain(b)}
    got, fed = {}, {0: 0, 1: 0}

    def step(entries):
        batch = []
        for r, n in entries:
            ids = (a, b)[r][fed[r]:fed[r] + n]
            (manager.allocate(r, ids) if fed[r] == 0 else manager.append_slots(r, ids))
            batch.append(StepEntry(r, ids, fed[r], [0, n - 1] if n > 1 else [0]))
        logits = runner.step(batch)
        row = 0
        for (r, n), e in zip(entries, batch):
            for wpos in e.want:
                got[(r, fed[r] + wpos)] = logits[row]
                row += 1
            manager.commit(r, n)
            fed[r] += n

    step([(0, 13)])
    step([(0, 2), (1, 9)])
    for _ in range(6):
        step([(0, 1), (1, 1)])
    step([(0, 5), (1, 3)])
    step([(0, 6), (1, 5)])
    assert manager.stats().window_frees > 0 and fed[1] == len(b)
    while fed[0] < len(a):
        step([(0, 1)])
    assert manager.block_table(0, 1)[0] < 0 and manager.block_table(0, 0)[0] >= 0, "only the windowed space lets go of old pages"
    tol = dict(rtol=1e-4, atol=1e-5) if dtype == torch.float32 else dict(rtol=3e-2, atol=3e-2)
    for (r, pos), row in got.items():
        torch.testing.assert_close(row.double().cpu(), want[r][pos], msg=lambda m: f"request {r} position {pos}: {m}", **tol)
    assert len(got) >= 30
    manager.release(0)
    manager.release(1)
    assert manager.num_available_blocks(1) == 8 and manager.num_available_blocks(0) == 24


def test_a_whole_architecture_is_a_config_with_from_dict_a_spec_and_one_registration(tmp_path, capsys):
    """A new architecture brings a configuration class with nothing but `from_dict`, a function from
    it to a ModelSpec, and one registration. The random-weights mode (on the device and as a
    folder), the loader, the entry point and the command line then run it as they are: they find
    the architecture by the configuration's type and write its config.json from its fields."""
    import json
    import os
    from dataclasses import dataclass

    from safetensors import safe_open

    from tinyserve_llm_amd import generate
    from tinyserve_llm_amd.engine.llm import LLM, CacheConfig
    from tinyserve_llm_amd.engine.loading import load_model, random_model
    from tinyserve_llm_amd.engine.scheduler import SchedulerConfig
    from tinyserve_llm_amd.engine.sequence import SamplingParams
    from tinyserve_llm_amd.models.decoder import DecoderModel
    from tinyserve_llm_amd.models.registry import Architecture, read_config, register_architecture
    from tinyserve_llm_amd.models.spec import Destination
    from tinyserve_llm_amd.weights.random_init import write_random_model
    register_toy_parts()

    @dataclass(frozen=True)
    class ToyConfig:
        vocab: int
        width: int
        mean_mixer: str

        @classmethod
        def from_dict(cls, raw):
            return cls(int(raw["vocab"]), int(raw["width"]), str(raw["mean_mixer"]))

    def spec_of(c: ToyConfig):
        spec = toy_spec(hidden=c.width, vocab=c.vocab, mean_mixer=c.mean_mixer)
        spec.checkpoint = {f"toy.{name}": Destination(name) for name in DecoderModel(spec).param_specs()
                           if not name.startswith("head.")}
        return spec

    register_architecture(Architecture("ToyForCausalLM", ("toy",), ToyConfig.from_dict, spec_of))
    cfg = ToyConfig(vocab=97, width=48, mean_mixer="toy_running_mean_on_device")
    folder = write_random_model(str(tmp_path / "toy"), cfg, 3, torch.float32)
    with open(os.path.join(folder, "config.json")) as f:
        raw = json.load(f)
    assert raw == dict(vocab=97, width=48, mean_mixer="toy_running_mean_on_device", architectures=["ToyForCausalLM"],
                       model_type="toy")
    assert read_config(folder)[1] == cfg
    model, config = load_model(folder, torch.float32, DEV)
    assert config == cfg and model.spec.architecture == "Toy"
    with safe_open(os.path.join(folder, "model.safetensors"), "pt", "cpu") as f:
        p = {k[len("toy."):]: f.get_tensor(k).double() for k in f.keys()}

    def plain_greedy(ids, n):
        ids, out = list(ids), []
        for _ in range(n):
            out.append(int(toy_plain(p, ids)[-1].argmax()))
            ids.append(out[-1])
        return out

    prompts = [[3, 50, 7, 7, 96, 1], [9, 8, 7]]
    sc = SchedulerConfig(max_model_len=64, max_num_seqs=4, max_num_batched_tokens=24, max_prefill_chunk=5)
    sp = SamplingParams(max_tokens=6, temperature=0.0, ignore_eos=True)
    got = LLM(folder, sc, CacheConfig(block_size=4), dtype=torch.float32, num_blocks=24).generate(prompts, sp)
    assert [r.token_ids[0] for r in got] == [plain_greedy(q, 6) for q in prompts]
    drawn = random_model(cfg, 3, torch.float32, DEV)
    again = LLM(None, sc, CacheConfig(block_size=4), model=drawn, num_blocks=24).generate(prompts, sp)
    assert all(len(r.token_ids[0]) == 6 for r in again)
    out = str(tmp_path / "record.json")
    rc = generate.main(["--random-config", os.path.join(folder, "config.json"), "--random-seed", "3", "--dtype", "float32",
                        "--prompt-ids", "3,50,7,7,96,1", "--max-tokens", "6", "--temperature", "0", "--ignore-eos",
                        "--block-size", "4", "--num-blocks", "24", "--max-model-len", "64", "--max-num-seqs", "4",
                        "--max-num-batched-tokens", "24", "--out", out])
    assert rc == 0
    with open(out) as f:
        record = json.load(f)
    assert record["completions"][0]["token_ids"] == [again[0].token_ids[0]], "the same seed on the device draws the same weights"
