"""Grouped-query attention over the paged cache (tinyserve_llm/model/llama.py:189-212,
tinyserve_llm/engine/model_runner.py:100-108, tinyserve_llm/attention/torch_paged.py:15-46).

One fused projection gives q | k | v; q and k are rotated by the named position encoding; k and v
of the step's tokens are written to their cache slots; then every token attends, causally, over
the cache pages of its request (its own key included), and the output projection follows.
For steps of few tokens (`hip.qkv_rope_max_rows` says how many for the layer's width) projection,
rotation and cache write are one kernel (`hip.qkv_rope_store`), which also takes a deferred norm
where it reaches; larger steps run them one after the other.
"""

from __future__ import annotations

import torch

from tinyserve_llm_amd.ops import hip
from tinyserve_llm_amd.parts.base import KVSpec, LayerMemory, Mixer, ParamSpec, StepContext, register
from tinyserve_llm_amd.parts.linear import DeferredNorm, linear, streaming_copy


@register("mixer", "attention")
class Attention(Mixer):
    graph_safe = True
    takes_deferred_norm = True
    finishes_into_norm = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 position: str | None = "rope", scale: float | None = None, window: int = 0) -> None:
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} heads do not divide into {num_kv_heads} key/value heads")
        if head_dim % 16 or head_dim > 256:
            raise ValueError(f"head_dim {head_dim}: the attention kernels take multiples of 16 up to 256")
        self.hidden_size = hidden_size
        self.num_heads = num_heads
        self.num_kv_heads = num_kv_heads
        self.head_dim = head_dim
        self.position = position
        self.scale = scale if scale is not None else head_dim ** -0.5
        self.window = window
        self.qkv: torch.Tensor | None = None
        self.o: torch.Tensor | None = None
        self.qkv_packed: hip.StreamingCopies | None = None
        self.qkv_rope_packed: torch.Tensor | None = None     # for the one-kernel path: `hip.pack_weight_rope`
        self.o_packed: hip.StreamingCopies | None = None

    @property
    def q_size(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_kv_heads * self.head_dim

    def keep_streaming_copies(self) -> int:
        self.qkv_packed, self.o_packed = streaming_copy(self.qkv), streaming_copy(self.o)
        if self.qkv_packed is not None and self.qkv_packed.by16 is not None and self.head_dim % 32 == 0:
            self.qkv_rope_packed = hip.pack_weight_rope(self.qkv, self.head_dim)
            if hip.qkv_rope_max_rows(self.hidden_size) >= hip.STREAMING_MAX_ROWS:
                self.qkv_packed = None           # every step that would stream the plain copy takes the one-kernel path
        copies = sum(c.nbytes() for c in (self.qkv_packed, self.o_packed) if c is not None)
        return copies + (0 if self.qkv_rope_packed is None else self.qkv_rope_packed.numel() * 2)

    def _project_fused(self, x, table, positions, slots, k_store, v_store) -> torch.Tensor | None:
        """Projection, rotation and cache write in one kernel where a step is small enough for the
        weight-streaming kernel (in two, with the reduction in slices, for a few dozen rows over a
        reduction that kernel does not take); None where neither serves."""
        d = x if isinstance(x, DeferredNorm) else None
        by16 = self.qkv_rope_packed
        if d is not None and d.prepared is not None:     # the norm's first half is done: its operand, then a scale per row
            rows = d.prepared.operand
            if not hip.qkv_rope_fuses(rows, self.qkv, self.head_dim, k_store, table=table):
                slices = 0 if by16 is None else hip.qkv_rope_sliced_slices(rows, self.qkv, self.head_dim, k_store, table)
                if not slices:
                    return None
                return hip.qkv_rope_store_sliced(rows, by16, slices, table, positions, slots, k_store, v_store, self.num_heads,
                                                 self.num_kv_heads, self.head_dim, eps=d.eps, squares=d.prepared.squares)
            return hip.qkv_rope_store(rows, self.qkv, table, positions, slots, k_store, v_store, self.num_heads,
                                      self.num_kv_heads, self.head_dim, eps=d.eps, packed=by16, squares=d.prepared.squares)[0]
        rows = d.x if d is not None else x
        if not (rows.is_cuda and hip.qkv_rope_fuses(rows, self.qkv, self.head_dim, k_store, table=table)):
            slices = 0 if by16 is None or not rows.is_cuda else hip.qkv_rope_sliced_slices(rows, self.qkv, self.head_dim, k_store, table)
            if not slices:
                return None
            if d is not None:
                rows = d.materialize()           # the norm by its own kernel
            return hip.qkv_rope_store_sliced(rows, by16, slices, table, positions, slots, k_store, v_store, self.num_heads,
                                             self.num_kv_heads, self.head_dim)
        if d is not None and not (hip.qkv_rope_fuses(rows, self.qkv, self.head_dim, k_store, norm=True)
                                  and d.weight.dtype == torch.bfloat16
                                  and (d.residual is None or d.residual.is_contiguous())):
            rows, d = d.materialize(), None      # the norm by its own kernel, the rest in one
        if d is None:
            return hip.qkv_rope_store(rows, self.qkv, table, positions, slots, k_store, v_store, self.num_heads,
                                      self.num_kv_heads, self.head_dim, packed=by16)[0]
        q, d.residual_out = hip.qkv_rope_store(rows, self.qkv, table, positions, slots, k_store, v_store, self.num_heads,
                                               self.num_kv_heads, self.head_dim, residual=d.residual,
                                               norm_weight=d.weight, eps=d.eps, packed=by16)
        return q

    def param_specs(self) -> dict[str, ParamSpec]:
        return {"qkv": ParamSpec((self.q_size + 2 * self.kv_size, self.hidden_size)),
                "o": ParamSpec((self.hidden_size, self.q_size))}

    def kv_spec(self) -> KVSpec:
        return KVSpec(self.num_kv_heads, self.head_dim, self.window)

    def forward(self, x: torch.Tensor, ctx: StepContext, mem: LayerMemory, then=None) -> torch.Tensor:
        table = ctx.position_encodings[self.position].rotary_table() if self.position else None
        slots = ctx.slot_mapping[mem.space] if mem.store else None
        k_store, v_store = (mem.k_cache, mem.v_cache) if mem.store else (None, None)
        q = self._project_fused(x, table, ctx.positions, slots, k_store, v_store)
        if q is None:
            qkv = linear(x, self.qkv, packed=self.qkv_packed)
            q = hip.rope_store(qkv, table, ctx.positions, slots, k_store, v_store, self.num_heads, self.num_kv_heads,
                               self.head_dim)
        # (a single token: the o projection adds the chunks of a split walk up itself, on its way in)
        o = hip.paged_attention(q, mem.k_cache, mem.v_cache, ctx, mem.space, self.scale, self.window,
                                leave_split=hip.split_attention_fuses(ctx.num_tokens, self.o))
        if not isinstance(o, hip.SplitAttention):
            o = o.view(ctx.num_tokens, self.q_size)
        return linear(o, self.o, packed=self.o_packed, then=then)
