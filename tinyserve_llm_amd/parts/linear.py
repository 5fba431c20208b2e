"""y = x · Wᵀ for bias-free projections stored [out, in] (tinyserve_llm/model/llama.py:179,201,221,293).

float32 runs the engine's own exact kernel (32-bit multiply-adds, ascending k, independent of the
batch). bfloat16 uses the weight-streaming kernel for few rows and the vendor matrix library for
many, as the reference uses a vendor library for every projection (or, if
`hip.many_rows_products("tiled")` says so, the engine's own tiled kernel, which is slower).

With few rows a step's time goes to launching kernels and to waiting for memory, so what
precedes or follows a projection can ride along with it: a norm may hand its input over as a
`DeferredNorm` and the projection applies residual add and normalisation while it reads x; a
gated feed-forward may ask for silu(gate) * up straight out of the gate|up projection; and a
projection whose result goes into a residual sum and a norm may be asked to finish into them
(`then=`, a `NormRequest`): it then leaves the sum, the next projection's operand and the rows'
sums of squares, and what comes back is again a `DeferredNorm`, half done already. Where the
fused kernel does not serve the shape, the same calls run the separate kernels.
"""

from __future__ import annotations

import torch

from tinyserve_llm_amd.ops import hip


class DeferredNorm:
    """norm(x + residual) * weight, not yet computed: the first projection that takes it either
    fuses it or materialises it. Either way `residual_out` then holds x + residual. With `prepared`
    (what the projection that made x has left: `hip.PreparedNorm`) the sum is there already and
    `x`, `residual` are not given."""

    def __init__(self, x: torch.Tensor | None, residual: torch.Tensor | None, weight: torch.Tensor, eps: float,
                 prepared: hip.PreparedNorm | None = None) -> None:
        self.x, self.residual, self.weight, self.eps, self.prepared = x, residual, weight, eps, prepared
        self.residual_out: torch.Tensor | None = None if prepared is None else prepared.summed

    @property
    def rows(self) -> int:
        return (self.x if self.prepared is None else self.prepared.operand).shape[0]

    def materialize(self) -> torch.Tensor:
        if self.prepared is not None:
            return hip.rmsnorm(self.prepared.summed, self.weight, self.eps, want_residual=False)[0]
        out, self.residual_out = hip.rmsnorm(self.x, self.weight, self.eps, self.residual)
        return out


class NormRequest:
    """Asks a projection to finish into the residual sum and the norm that follow it: `weight` and
    `eps` are that norm's, `residual` the stream its input is added to: a tensor, None, or a
    `DeferredNorm` whose `residual_out` is the stream once its projection has run (the norm before
    the part that holds this projection, fused into that part's first projection)."""

    def __init__(self, weight: torch.Tensor, eps: float, residual: "torch.Tensor | DeferredNorm | None") -> None:
        self.weight, self.eps, self._residual = weight, eps, residual

    def residual(self) -> torch.Tensor | None:
        r = self._residual
        return r.residual_out if isinstance(r, DeferredNorm) else r


def _streams(x: torch.Tensor, weight: torch.Tensor, dense_rows: bool = False) -> bool:
    """Whether the weight-streaming kernels take these operands; `dense_rows`: x need not be
    contiguous as long as its rows are (a prepared norm's operand, whose rows may lie further apart)."""
    rows_ok = (x.stride(1) == 1 and x.stride(0) % 8 == 0 and x.stride(0) >= x.shape[1]) if dense_rows and x.dim() == 2 else x.is_contiguous()
    return (x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and x.is_cuda and rows_ok
            and weight.is_contiguous() and x.data_ptr() % 16 == 0 and weight.data_ptr() % 16 == 0)


def streaming_copy(weight: torch.Tensor) -> hip.StreamingCopies | None:
    """The weight once more in the orders the weight-streaming kernels read it, for a part to keep
    beside the weight and hand to `linear` (decode steps read the copies, steps with many rows read
    the weight itself through the library); None where those kernels would never take the weight."""
    if not (weight.is_cuda and weight.dtype == torch.bfloat16 and weight.dim() == 2 and weight.is_contiguous()):
        return None
    n, k = weight.shape
    by16 = hip.pack_weight(weight) if (hip.skinny_takes(1, k) and k <= 4096) or hip.rows64_slices(hip.ROWS64_MAX_ROWS, n, k) else None
    by8 = hip.pack_weight8(weight) if hip.skinny8_takes(1, n, k) and n % 8 == 0 else None     # (one row: the widest reach of that form)
    return hip.StreamingCopies(by16, by8) if by16 is not None or by8 is not None else None


PACKED_ROWS_MIN = 2      # rows from which a gated product is handed on in the 8-row form's order (one row is read whole anyway)


def linear(x: "torch.Tensor | DeferredNorm | hip.PackedRows8 | hip.SplitAttention", weight: torch.Tensor, out_dtype: torch.dtype | None = None,
           glu: bool = False, packed: hip.StreamingCopies | None = None,
           then: NormRequest | None = None, feeds: torch.Tensor | None = None) -> "torch.Tensor | DeferredNorm | hip.PackedRows8":
    """x · Wᵀ; with `glu`, W holds gate rows then up rows and silu(gate) * up comes back.
    `packed` is `streaming_copy(weight)` if the part keeps one. With `then` the result is the
    `DeferredNorm` of that request: norm(x · Wᵀ + residual) * weight, prepared by this projection's
    kernel where it can be, left to the next projection otherwise. `feeds` (with `glu`): the weight of
    the projection that alone reads this product; where that projection's kernel reads its operand
    faster in an order of its own, the product comes back in that order (a `hip.PackedRows8`), to be
    handed to `linear` with that weight and to nothing else. x may be a `hip.SplitAttention` (an attention output
    still in its chunks' parts): the 8-row form adds the parts up on its way in where it can, the combining
    kernel does otherwise."""
    if isinstance(x, hip.SplitAttention):
        residual = then.residual() if then is not None else None
        if (not glu and out_dtype in (None, torch.bfloat16) and hip.split_attention_fuses(x.shape[0], weight)
                and (then is None or (then.weight.dtype == torch.bfloat16
                                      and (residual is None or (residual.is_contiguous() and residual.dtype == torch.bfloat16))))):
            by8 = None if packed is None else packed.by8
            if then is None:
                return hip.gemm_skinny8(x, weight, torch.bfloat16, by8)
            prepared = hip.gemm_skinny8(x, weight, torch.bfloat16, by8, next_norm=(residual, then.weight))
            return DeferredNorm(None, None, then.weight, then.eps, prepared)
        x = x.combined()
    if isinstance(x, hip.PackedRows8) and (glu or hip.rows8_reader_steps(x.shape[0], weight) != x.steps):
        x = x.rows()
    if isinstance(x, hip.PackedRows8) and then is None:
        return hip.linear_bf16(x, weight, out_dtype or torch.bfloat16, packed)
    if then is not None:
        if glu:
            raise ValueError("a gated projection does not finish into a norm")
        residual = then.residual()
        if isinstance(x, DeferredNorm):
            x = x.materialize()
        if (out_dtype in (None, torch.bfloat16) and then.weight.dtype == torch.bfloat16 and hip.next_norm_fuses(x, weight, packed)
                and (residual is None or (residual.is_contiguous() and residual.dtype == torch.bfloat16))):
            prepared = hip.linear_bf16(x, weight, torch.bfloat16, packed, next_norm=(residual, then.weight))
            return DeferredNorm(None, None, then.weight, then.eps, prepared)
        return DeferredNorm(linear(x, weight, out_dtype, packed=packed), residual, then.weight, then.eps)
    by16 = None if packed is None else packed.by16
    rows = x.rows if isinstance(x, DeferredNorm) else x.shape[0]
    pack8 = hip.rows8_reader_steps(rows, feeds) if glu and feeds is not None and PACKED_ROWS_MIN <= rows <= 8 else 0
    if pack8 and (weight.shape[0] // 2) % (64 * pack8):
        pack8 = 0
    if isinstance(x, DeferredNorm) and x.prepared is not None:
        d, op = x, x.prepared.operand
        if out_dtype in (None, torch.bfloat16) and _streams(op, weight, dense_rows=True) and not (glu and weight.shape[0] % 32):
            rows, (n, k) = op.shape[0], weight.shape
            wide = by16 is not None and hip.rows64_takes(rows, n, k, glu) and n % (128 if glu else 64) == 0
            if wide:
                return hip.gemm_rows64(op, by16, glu=glu, squares=d.prepared.squares, eps=d.eps)
            if (hip.skinny_fuses(rows, k, False, True) if glu else hip._skinny_serves(rows, n, k)):
                return hip.gemm_skinny(op, weight, glu=glu, packed=by16, squares=d.prepared.squares, eps=d.eps,
                                       pack8_steps=pack8 if glu else 0)[0]
        x = d.materialize()
    if isinstance(x, DeferredNorm):
        d = x
        if (out_dtype in (None, torch.bfloat16) and _streams(d.x, weight) and d.weight.dtype == torch.bfloat16
                and (d.residual is None or d.residual.is_contiguous())
                and hip.skinny_fuses(d.x.shape[0], weight.shape[1], True, glu) and (not glu or weight.shape[0] % 32 == 0)):
            y, d.residual_out = hip.gemm_skinny(d.x, weight, residual=d.residual, norm_weight=d.weight, eps=d.eps, glu=glu,
                                                packed=by16, pack8_steps=pack8 if glu else 0)
            return y
        x = d.materialize()
    if glu:
        if (out_dtype in (None, torch.bfloat16) and by16 is not None and _streams(x, weight)
                and hip.rows64_takes(x.shape[0], weight.shape[0], weight.shape[1], True) and weight.shape[0] % 128 == 0):
            return hip.gemm_rows64(x, by16, glu=True)
        if (out_dtype in (None, torch.bfloat16) and _streams(x, weight) and weight.shape[0] % 32 == 0
                and hip.skinny_fuses(x.shape[0], weight.shape[1], False, True)):
            return hip.gemm_skinny(x, weight, glu=True, packed=by16, pack8_steps=pack8)[0]
        if (out_dtype in (None, torch.bfloat16) and hip.many_rows_products() == "tiled" and x.is_cuda
                and hip.tiled_takes(x, weight, glu=True)):
            return hip.gemm_tiled(x, weight, glu=True)
        return hip.silu_mul(linear(x, weight, out_dtype, packed=packed))
    if x.dtype == torch.float32:
        return hip.gemm_exact(x, weight, out_dtype)
    if x.dtype != torch.bfloat16:
        raise hip.KernelError(f"linear: no path for {x.dtype}")
    if not x.is_cuda:
        raise hip.KernelError("linear: GPU tensors only; there is no CPU path")
    return hip.linear_bf16(x, weight, out_dtype or torch.bfloat16, packed)
