"""Token sampling: greedy at temperature 0, otherwise a draw from softmax(logits / temperature)
by the exponential race (tinyserve_llm/engine/sampler.py:8-23), in one HIP kernel.

The reference draws its noise from one generator over the whole [rows, vocab] batch, so a draw
depends on the row's place in the batch. Here the noise of a row is a function of
(seed, request, sample index, output position): the same request gives the same tokens however
it was batched, cut or preempted.
"""

from __future__ import annotations

import torch

from tinyserve_llm_amd.ops import hip

_MASK = (1 << 63) - 1


def row_key(request_id: int, sample_index: int, position: int) -> int:
    """Names one draw; a non-negative 63-bit integer."""
    x = (request_id * 0x9E3779B97F4A7C15 + sample_index * 0xC2B2AE3D27D4EB4F + position * 0x165667B19E3779F9 + 1)
    return x & _MASK


def sample(logits: torch.Tensor, temperatures: list[float], keys: list[int], seed: int,
           rows: list[int] | None = None) -> torch.Tensor:
    """One token id per draw from float32 logits [rows, vocab] -> int32 [draws] on the device. Draw i
    reads row i, or row rows[i] if `rows` is given (several draws may read one row)."""
    n = len(keys)
    if rows is not None and (len(rows) != n or min(rows, default=0) < 0 or max(rows, default=0) >= logits.shape[0]):
        raise ValueError(f"{n} draws name rows outside the {logits.shape[0]} rows of logits")
    # keys, temperatures and rows travel to the device in one copy
    words = [torch.tensor(keys, dtype=torch.int64).view(torch.int32), torch.tensor(temperatures, dtype=torch.float32).view(torch.int32)]
    if rows is not None:
        words.append(torch.tensor(rows, dtype=torch.int32))
    packed = torch.cat(words).to(logits.device, non_blocking=True)
    return hip.sample(logits, packed[2 * n:3 * n].view(torch.float32), packed[:2 * n].view(torch.int64), seed,
                      packed[3 * n:] if rows is not None else None, num_logit_rows_checked=True)
