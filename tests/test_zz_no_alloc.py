"""The entry point that allocates nothing (`ts_sample_static`, csrc/sample_static.h), called through
ctypes as a caller outside this package would: its tokens must be those of `ts_sample`, on two
calls in a row of which the second is smaller (it finds the first call's partial results in the
shared array and must not read them), and sizes beyond its fixed array are refused before any
launch. The reference has no counterpart; parity is with this repository's own `ts_sample`."""

from __future__ import annotations

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _static(lib, logits, temps, keys, seed):
    out = torch.full((logits.shape[0],), -7, dtype=torch.int32, device=logits.device)
    stream = torch.cuda.current_stream().cuda_stream
    rc = lib.ts_sample_static(ctypes.c_void_p(out.data_ptr()), ctypes.c_void_p(logits.data_ptr()),
                              ctypes.c_void_p(temps.data_ptr()), ctypes.c_void_p(keys.data_ptr()),
                              ctypes.c_uint64(seed), logits.shape[0], logits.shape[1], logits.stride(0),
                              ctypes.c_void_p(stream))
    return rc, out


def _case(rows, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    logits = (torch.randn(rows, vocab, generator=g) * 3).cuda()
    temps = torch.tensor([0.0 if r % 3 == 0 else 0.5 + 0.25 * (r % 4) for r in range(rows)]).cuda()
    keys = torch.randint(0, 2 ** 62, (rows,), generator=g).cuda()
    return logits, temps, keys


def test_static_sampler_matches_the_allocating_one_twice_in_a_row():
    from tinyserve_llm_amd.ops import hip
    lib = hip.library()
    with torch.cuda.device(0):
        for rows, vocab in ((37, 1003), (5, 130)):          # the second call is the smaller one
            logits, temps, keys = _case(rows, vocab, seed=rows)
            want = hip.sample(logits, temps, keys, seed=11)
            rc, got = _static(lib, logits, temps, keys, seed=11)
            assert rc == 0
            torch.cuda.synchronize()
            assert got.tolist() == want.tolist()
            greedy = [r for r in range(rows) if r % 3 == 0]
            assert [got[r].item() for r in greedy] == logits[greedy].argmax(dim=1).tolist()


def test_static_sampler_refuses_more_rows_than_its_array_holds():
    from tinyserve_llm_amd.ops import hip
    lib = hip.library()
    logits, temps, keys = _case(1025, 8, seed=3)
    rc, out = _static(lib, logits, temps, keys, seed=1)
    torch.cuda.synchronize()
    assert rc == 4
    assert out.tolist() == [-7] * 1025          # nothing was launched
    rc, _ = _static(lib, logits[:1024], temps[:1024], keys[:1024], seed=1)
    torch.cuda.synchronize()
    assert rc == 0
