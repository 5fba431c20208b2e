"""Each HIP kernel alone against a plain float64/float32 formula, at sizes other than the engine's
tiny models use: widths and vocabularies that are no power of two, head sizes from 16 to 256, odd
head groupings, several page sizes, strided cache views, out-of-order block tables."""

from __future__ import annotations

import math

import pytest
import torch

from tests.plain import llama as P

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


def dev():
    return torch.device("cuda:0")


def hip():
    from tinyserve_llm_amd.ops import hip as h
    return h


def tol(dtype):
    return dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)


def gen(seed):
    return torch.Generator().manual_seed(seed)


def test_missing_gpu_tensor_is_refused_not_run_on_the_cpu():
    with pytest.raises(hip().KernelError, match="GPU"):
        hip().silu_mul(torch.zeros(2, 4))
    with pytest.raises(hip().KernelError, match="float32 and bfloat16"):
        hip().silu_mul(torch.zeros(2, 4, dtype=torch.float16, device=dev()))


@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding(dtype):
    table = torch.randn(1000, 72, generator=gen(0)).to(dtype)
    ids = torch.tensor([999, 0, 17, 17, 500], dtype=torch.int32)
    out = hip().embedding(table.to(dev()), ids.to(dev()))
    assert torch.equal(out.cpu(), table[ids.long()])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden", [200, 72, 2048, 3000])
def test_rmsnorm_forms(dtype, hidden):
    g = gen(hidden)
    x, r = torch.randn(7, hidden, generator=g).to(dtype), torch.randn(7, hidden, generator=g).to(dtype)
    w = (1 + 0.1 * torch.randn(hidden, generator=g)).to(dtype)
    eps = 1e-5
    out, res = hip().rmsnorm(x.to(dev()), w.to(dev()), eps)
    want = P.rms_norm(x.double(), w.double(), eps)
    torch.testing.assert_close(out.double().cpu(), want, **tol(dtype))
    assert res.data_ptr() != 0 and torch.equal(res.cpu(), x), "without a residual the input is the residual"
    out, res = hip().rmsnorm(x.to(dev()), w.to(dev()), eps, r.to(dev()))
    want, s = P.add_rms_norm(x.double(), r.double(), w.double(), eps)
    torch.testing.assert_close(out.double().cpu(), want, **tol(dtype))
    assert torch.equal(res.cpu(), (x.float() + r.float()).to(dtype)), "the residual is the sum, rounded once"
    rows = torch.tensor([6, 0, 3], dtype=torch.int32)
    out, res = hip().rmsnorm(x.to(dev()), w.to(dev()), eps, r.to(dev()), rows.to(dev()))
    assert res is None
    torch.testing.assert_close(out.double().cpu(), want[rows.long()], **tol(dtype))


def test_rmsnorm_bfloat16_rounds_before_the_weight():
    """tinyserve_llm/model/llama.py:58,67: the normalised value is cast to the storage type and
    then multiplied by the weight in that type."""
    x = torch.randn(3, 96, generator=gen(1)).bfloat16()
    w = (1 + 0.1 * torch.randn(96, generator=gen(2))).bfloat16()
    out, _ = hip().rmsnorm(x.to(dev()), w.to(dev()), 1e-6)
    xf = x.float()
    y = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-6)).bfloat16() * w
    assert (out.cpu().float() - y.float()).abs().max() <= 2 ** -7 * y.float().abs().max()
    assert (out.cpu() == y).float().mean() > 0.98, "same two roundings nearly everywhere"


def test_rmsnorm_row_does_not_depend_on_the_batch():
    x = torch.randn(9, 1000, generator=gen(3)).to(dev())
    w = torch.randn(1000, generator=gen(4)).to(dev())
    a, _ = hip().rmsnorm(x, w, 1e-5)
    b, _ = hip().rmsnorm(x[4:5].contiguous(), w, 1e-5)
    assert torch.equal(a[4:5], b)


@pytest.mark.parametrize("dtype", DTYPES)
def test_rope_and_cache_write_on_a_strided_layer_view(dtype):
    """Slots [12,13,14,15,4,5,6] on pages of 4, a skipped row (-1), other layers untouched: the
    vectors of the reference's store tests (tests/test_attention.py:21-101), with rotation."""
    nh, nkv, hd, T, page = 5, 1, 48, 8, 4
    g = gen(5)
    qkv = torch.randn(T, (nh + 2 * nkv) * hd, generator=g).to(dtype)
    positions = torch.tensor([30, 31, 32, 33, 0, 1, 2, 7], dtype=torch.int32)
    slots = torch.tensor([12, 13, 14, 15, 4, 5, 6, -1], dtype=torch.int32)
    cos, sin = P.rope_tables(hd, 10000.0, None, 64, 64, torch.float64)
    table = torch.cat((cos, sin), -1).float()
    k_pool = torch.zeros(6, 3, page, nkv, hd, dtype=dtype, device=dev())
    v_pool = torch.zeros_like(k_pool)
    q = hip().rope_store(qkv.to(dev()), table.to(dev()), positions.to(dev()), slots.to(dev()), k_pool[:, 1],
                         v_pool[:, 1], nh, nkv, hd)
    x = qkv.double()
    qs, ks, vs = x[:, :nh * hd].view(T, nh, hd), x[:, nh * hd:(nh + nkv) * hd].view(T, nkv, hd), x[:, (nh + nkv) * hd:].view(T, nkv, hd)
    pos = positions.long()
    torch.testing.assert_close(q.double().cpu(), P.apply_rope(qs, cos[pos], sin[pos]), **tol(dtype))
    kr = P.apply_rope(ks, cos[pos], sin[pos])
    for t in range(T - 1):
        b, o = int(slots[t]) // page, int(slots[t]) % page
        torch.testing.assert_close(k_pool[b, 1, o].double().cpu(), kr[t], **tol(dtype))
        assert torch.equal(v_pool[b, 1, o].cpu(), qkv[t, (nh + nkv) * hd:].view(nkv, hd))
    assert k_pool[:, 0].eq(0).all() and k_pool[:, 2].eq(0).all() and v_pool[:, 0].eq(0).all(), "other layers untouched"
    assert int(k_pool.ne(0).any(dim=(-1, -2)).sum()) == 7, "exactly seven slots written; the -1 row skipped"
    # no table: q passes through, k is stored as it is
    q2 = hip().rope_store(qkv.to(dev()), None, positions.to(dev()), slots.to(dev()), k_pool[:, 2], v_pool[:, 2], nh, nkv, hd)
    assert torch.equal(q2.cpu(), qkv[:, :nh * hd].view(T, nh, hd))
    assert torch.equal(k_pool[3, 2, 0].cpu(), qkv[0, nh * hd:(nh + nkv) * hd].view(nkv, hd))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hd,rot,T", [(48, 16, 8), (64, 32, 40), (40, 6, 3), (128, 64, 17)])
def test_rotation_of_the_leading_part_of_a_head(dtype, hd, rot, T):
    """A table narrower than the head turns the first `rot` dimensions (j with j + rot / 2) and lets
    the rest pass, in q and in the keys that are written; the sixteen-byte path and the one element
    at a time (widths of 6 and 34 have no whole pieces)."""
    nh, nkv, page = 3, 1, 8
    g = gen(hd + rot)
    qkv = torch.randn(T, (nh + 2 * nkv) * hd, generator=g).to(dtype)
    positions = torch.randint(0, 64, (T,), generator=g, dtype=torch.int32)
    slots = torch.randperm(48, generator=g)[:T].to(torch.int32)
    cos, sin = P.rope_tables(rot, 10000.0, None, 64, 64, torch.float64)
    table = torch.cat((cos, sin), -1).float()
    k_pool = torch.zeros(6, page, nkv, hd, dtype=dtype, device=dev())
    v_pool = torch.zeros_like(k_pool)
    q = hip().rope_store(qkv.to(dev()), table.to(dev()), positions.to(dev()), slots.to(dev()), k_pool, v_pool, nh, nkv, hd)
    x = qkv.double()
    qs, ks = x[:, :nh * hd].view(T, nh, hd), x[:, nh * hd:(nh + nkv) * hd].view(T, nkv, hd)
    pos = positions.long()

    def turned(t):
        return torch.cat((P.apply_rope(t[..., :rot], cos[pos], sin[pos]), t[..., rot:]), -1)

    torch.testing.assert_close(q.double().cpu(), turned(qs), **tol(dtype))
    assert torch.equal(q[..., rot:].cpu(), qkv[:, :nh * hd].view(T, nh, hd)[..., rot:]), "what does not turn passes bit for bit"
    kr = turned(ks)
    for t in range(T):
        b, o = int(slots[t]) // page, int(slots[t]) % page
        torch.testing.assert_close(k_pool[b, o].double().cpu(), kr[t], **tol(dtype))
        assert torch.equal(v_pool[b, o].cpu(), qkv[t, (nh + nkv) * hd:].view(nkv, hd))
    with pytest.raises(hip().KernelError, match="rotation table"):
        hip().rope_store(qkv.to(dev()), torch.zeros(64, hd + 2, device=dev()), positions.to(dev()), None, None, None, nh, nkv, hd)
    w = torch.zeros((nh + 2 * nkv) * hd, 256, dtype=torch.bfloat16, device=dev())
    xs = torch.zeros(4, 256, dtype=torch.bfloat16, device=dev())
    if hd % 32 == 0:
        assert hip().qkv_rope_fuses(xs, w, hd, None) and not hip().qkv_rope_fuses(xs, w, hd, None, table=table.to(dev())), \
            "the one-kernel path turns whole heads only: a part leaves this table to the separate kernels"


def scattered(k, v, table, page, pages, dtype, layers=2, layer=1):
    """A pool full of junk with k/v of positions 0.. written to the pages `table` names."""
    g = gen(9)
    kp = torch.randn(pages, layers, page, k.shape[1], k.shape[2], generator=g).to(dtype)
    vp = torch.randn(pages, layers, page, k.shape[1], k.shape[2], generator=g).to(dtype)
    for p in range(k.shape[0]):
        kp[table[p // page], layer, p % page] = k[p]
        vp[table[p // page], layer, p % page] = v[p]
    return kp.to(dev())[:, layer], vp.to(dev())[:, layer]


def run_attention(q, kc, vc, tables, seq_of, positions, scale, window=0):
    return hip().paged_attention_wave(
        q.to(dev()), kc, vc, torch.tensor(tables, dtype=torch.int32, device=dev()),
        torch.tensor(seq_of, dtype=torch.int32, device=dev()), torch.tensor(positions, dtype=torch.int32, device=dev()),
        scale, window)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv,hd,page", [(4, 2, 16, 4), (3, 1, 32, 16), (6, 2, 48, 8), (8, 8, 64, 256),
                                              (5, 5, 128, 32), (2, 1, 256, 16)])
def test_paged_attention_prefill_prefix_and_decode_in_one_batch(dtype, heads, kv, hd, page):
    """A whole prompt, its last 4 tokens over a cached prefix and its last token as a decode, in
    one batch, through an out-of-order block table padded with zeros
    (tests/test_engine.py:69-82 of the reference)."""
    n = 11 if page <= 8 else 75
    g = gen(hd)
    q = torch.randn(n, heads, hd, generator=g).to(dtype)
    k, v = torch.randn(n, kv, hd, generator=g).to(dtype), torch.randn(n, kv, hd, generator=g).to(dtype)
    need = -(-n // page)
    table = [6, 1, 4, 9, 2, 7, 3, 8, 5, 0][:need]
    kc, vc = scattered(k, v, table, page, 10, dtype)
    dense = P.causal_attention(q.double(), k.double(), v.double())
    queries = torch.cat([q, q[n - 4:], q[n - 1:]])
    seq_of = [0] * n + [1] * 4 + [2]
    positions = list(range(n)) + list(range(n - 4, n)) + [n - 1]
    out = run_attention(queries, kc, vc, [table + [0], table + [0], table + [0]], seq_of, positions, hd ** -0.5)
    out = out.double().cpu()
    torch.testing.assert_close(out[:n], dense, **tol(dtype))
    torch.testing.assert_close(out[n:n + 4], dense[n - 4:], **tol(dtype))
    torch.testing.assert_close(out[n + 4:], dense[n - 1:], **tol(dtype))
    if dtype == torch.float32:
        assert torch.equal(out[n:n + 4], out[n - 4:n]) and torch.equal(out[n + 4:], out[n - 1:n]), \
            "a row's sums do not depend on the portion it came in"


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_finds_a_far_key_among_hundreds(dtype):
    """Random keys hide a lost page or a wrong offset: here one key, far back, is made to win
    every score, so the output must be that key's value."""
    n, heads, kv, hd, page = 700, 4, 2, 64, 64
    g = gen(11)
    q = torch.randn(n, heads, hd, generator=g) * 0.1
    k, v = torch.randn(n, kv, hd, generator=g) * 0.1, torch.randn(n, kv, hd, generator=g)
    for target in (0, 63, 64, 389, 640):
        kk = k.clone()
        kk[target] = 0
        kk[target, :, 5] = 40.0
        qq = q.clone()
        qq[:, :, 5] = 40.0
        table = list(range(10, -1, -1))
        kc, vc = scattered(kk.to(dtype), v.to(dtype), table, page, 11, dtype)
        rows = [target, target + 1 if target + 1 < n else target, n - 1]
        out = run_attention(qq[rows].to(dtype), kc, vc, [table], [0, 0, 0], rows, hd ** -0.5).float().cpu()
        for i, r in enumerate(rows):
            for h in range(heads):
                torch.testing.assert_close(out[i, h], v[target, h // 2].to(dtype).float(), rtol=1e-3, atol=1e-3)


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_window_edge(dtype):
    n, heads, kv, hd, page, window = 200, 2, 1, 32, 16, 37
    g = gen(12)
    q, k, v = torch.randn(n, heads, hd, generator=g), torch.randn(n, kv, hd, generator=g), torch.randn(n, kv, hd, generator=g)
    table = list(range(12, -1, -1))
    kc, vc = scattered(k.to(dtype), v.to(dtype), table, page, 13, dtype)
    want = P.causal_attention(q.to(dtype).double(), k.to(dtype).double(), v.to(dtype).double(), window=window)
    out = run_attention(q.to(dtype), kc, vc, [table], [0] * n, list(range(n)), hd ** -0.5, window).double().cpu()
    torch.testing.assert_close(out, want, **tol(dtype))
    # the key just inside the window wins, the key just outside must not be seen at all
    pos = 150
    for off, seen in ((window - 1, True), (window, False)):
        kk = k.clone()
        kk[pos - off] = 0
        kk[pos - off, 0, 3] = 50.0
        qq = q[pos:pos + 1].clone()
        qq[0, :, 3] = 50.0
        kc, vc = scattered(kk.to(dtype), v.to(dtype), table, page, 13, dtype)
        out = run_attention(qq.to(dtype), kc, vc, [table], [0], [pos], hd ** -0.5, window).float().cpu()
        is_it = torch.allclose(out[0, 0], v[pos - off, 0].to(dtype).float(), rtol=1e-2, atol=1e-2)
        assert is_it == seen


def engine_layout(k, v, table, page, pages, dtype):
    """The engine's own pools: keys [pages, kv_heads, page_size, head_dim], values transposed
    [pages, kv_heads, head_dim, page_size], both seen as [pages, page_size, kv_heads, head_dim]."""
    g = gen(19)
    kp = torch.randn(pages, k.shape[1], page, k.shape[2], generator=g).to(dtype)
    vp = torch.randn(pages, k.shape[1], k.shape[2], page, generator=g).to(dtype)
    for p in range(k.shape[0]):
        kp[table[p // page], :, p % page] = k[p]
        vp[table[p // page], :, :, p % page] = v[p]
    return kp.to(dev()).permute(0, 2, 1, 3), vp.to(dev()).permute(0, 3, 1, 2)


@pytest.mark.parametrize("heads,kv,hd,page", [(3, 1, 32, 16), (6, 2, 96, 8), (32, 8, 64, 256), (5, 5, 128, 32),
                                              (16, 1, 128, 64), (24, 8, 128, 64), (14, 2, 64, 24)])
@pytest.mark.parametrize("chunk,waves", [(128, 4), (256, 4), (256, 8), (640, 5), (1024, 8), (1024, 16)])
def test_split_key_decode_attention(heads, kv, hd, page, chunk, waves):
    """One query per request at different context lengths (1, a chunk's edge, mid-chunk, long)
    against the dense formula and against the wave kernel on the same pages."""
    dtype = torch.bfloat16
    n = 600
    g = gen(hd + chunk)
    q = torch.randn(n, heads, hd, generator=g).to(dtype)
    k, v = torch.randn(n, kv, hd, generator=g).to(dtype), torch.randn(n, kv, hd, generator=g).to(dtype)
    pages = -(-n // page)
    table = list(range(pages - 1, -1, -1))
    dense = P.causal_attention(q.double(), k.double(), v.double())
    rows = [min(x, n - 1) for x in (0, 1, 31, 32, chunk - 1, chunk, chunk + 1, 255, 256, 257, 400, 599)]
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev())
    kc, vc = engine_layout(k, v, table, page, pages, dtype)
    assert hip().decode_kernel_takes(q[rows].to(dev()), kc, vc)
    if waves > hip().decode_waves(hd, chunk == 32 * waves) or 4 * (32 * waves + waves * (heads // kv) * hd) > 65536:
        with pytest.raises(hip().KernelError, match="waves"):
            hip().paged_attention_decode(q[rows].to(dev()), kc, vc, i32([table, table]), i32([0, 1] * 6), i32(rows),
                                         hd ** -0.5, chunk=chunk, waves=waves)
        return
    out = hip().paged_attention_decode(q[rows].to(dev()), kc, vc, i32([table, table]), i32([0, 1] * 6), i32(rows),
                                       hd ** -0.5, chunk=chunk, waves=waves)
    torch.testing.assert_close(out.double().cpu(), dense[rows], **tol(dtype))
    wave = run_attention(q[rows], kc, vc, [table], [0] * len(rows), rows, hd ** -0.5)
    torch.testing.assert_close(out.float(), wave.float(), **tol(dtype))


@pytest.mark.parametrize("heads,kv,hd,page", [(3, 1, 32, 16), (6, 2, 96, 8), (32, 8, 64, 256), (5, 5, 128, 32),
                                              (16, 1, 128, 64), (14, 2, 64, 24), (12, 6, 32, 16), (32, 16, 64, 64),
                                              (8, 4, 96, 32), (24, 12, 32, 8)])
@pytest.mark.parametrize("row_tiles,waves", [(1, 4), (2, 4), (4, 4), (1, 8), (2, 8)])
def test_matrix_core_prefill_attention(heads, kv, hd, page, row_tiles, waves):
    """A packed step of three requests on shared pools: a whole prompt, a portion over a cached
    prefix, and single decoded tokens; tiles never cross a request. Once for each number of row
    tiles that a wave of the kernel may hold, in workgroups of four and of eight waves."""
    dtype = torch.bfloat16
    if waves == 8 and hd not in (64, 128):
        q0 = torch.zeros(4, heads, hd, dtype=dtype, device=dev())
        kc0 = torch.zeros(1, kv, page, hd, dtype=dtype, device=dev()).permute(0, 2, 1, 3)
        vc0 = torch.zeros(1, kv, hd, page, dtype=dtype, device=dev()).permute(0, 3, 1, 2)
        z = torch.zeros(4, dtype=torch.int32, device=dev())
        with pytest.raises(hip().KernelError, match="waves"):
            hip().paged_attention_prefill(q0, kc0, vc0, z[:1].view(1, 1), z, z, torch.tensor([[0, 4]], dtype=torch.int32, device=dev()),
                                          1.0, waves=8)
        return
    g = gen(hd * 3 + page)
    lens = [150, 77, 300]                       # keys each request has after the step
    fed = [150, 9, 1]                           # tokens of each in the step
    q_all, k_all, v_all = [], [], []
    pages_each = [-(-n // page) for n in lens]
    total_pages = sum(pages_each) + 1
    kp = torch.randn(total_pages, kv, page, hd, generator=g).to(dtype)
    vp = torch.randn(total_pages, kv, hd, page, generator=g).to(dtype)
    tables, nxt = [], 1
    for n, pe in zip(lens, pages_each):
        table = list(range(nxt + pe - 1, nxt - 1, -1))
        nxt += pe
        tables.append(table)
        k, v = torch.randn(n, kv, hd, generator=g).to(dtype), torch.randn(n, kv, hd, generator=g).to(dtype)
        for p_ in range(n):
            kp[table[p_ // page], :, p_ % page] = k[p_]
            vp[table[p_ // page], :, :, p_ % page] = v[p_]
        q_all.append(torch.randn(n, heads, hd, generator=g).to(dtype))
        k_all.append(k)
        v_all.append(v)
    width = max(pages_each)
    padded = [t + [0] * (width - len(t)) for t in tables]
    q_step = torch.cat([q_all[i][lens[i] - fed[i]:] for i in range(3)])
    seq_of = sum(([i] * fed[i] for i in range(3)), [])
    positions = sum((list(range(lens[i] - fed[i], lens[i])) for i in range(3)), [])
    cu = [0, fed[0], fed[0] + fed[1], sum(fed)]
    per_tile = row_tiles * waves * (16 // (heads // kv))
    flat = hip().attention_tiles(cu, [lens[i] - fed[i] for i in range(3)], per_tile)
    assert all(flat[2 * i + 1] <= per_tile for i in range(len(flat) // 2))
    assert sum(flat[1::2]) == sum(fed) and len(flat) // 2 == sum(-(-f // per_tile) for f in fed)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev())
    kc, vc = kp.to(dev()).permute(0, 2, 1, 3), vp.to(dev()).permute(0, 3, 1, 2)
    out = hip().paged_attention_prefill(q_step.to(dev()), kc, vc, i32(padded), i32(seq_of), i32(positions),
                                        i32(flat).view(-1, 2), hd ** -0.5, tile_tokens=per_tile, waves=waves)
    want = torch.cat([P.causal_attention(q_all[i].double(), k_all[i].double(), v_all[i].double())[lens[i] - fed[i]:]
                      for i in range(3)])
    torch.testing.assert_close(out.double().cpu(), want, **tol(dtype))
    wave = run_attention(q_step, kc, vc, padded, seq_of, positions, hd ** -0.5)
    torch.testing.assert_close(out.float(), wave.float(), **tol(dtype))
    win = hip().paged_attention_prefill(q_step.to(dev()), kc, vc, i32(padded), i32(seq_of), i32(positions),
                                        i32(flat).view(-1, 2), hd ** -0.5, window=40, tile_tokens=per_tile, waves=waves)
    want = torch.cat([P.causal_attention(q_all[i].double(), k_all[i].double(), v_all[i].double(), window=40)[lens[i] - fed[i]:]
                      for i in range(3)])
    torch.testing.assert_close(win.double().cpu(), want, **tol(dtype))


def test_decode_kernel_leaves_other_shapes_to_the_wave_kernel():
    q = torch.zeros(2, 4, 48, dtype=torch.bfloat16, device=dev())
    kc = torch.zeros(3, 2, 16, 48, dtype=torch.bfloat16, device=dev()).permute(0, 2, 1, 3)
    vc = torch.zeros(3, 2, 48, 16, dtype=torch.bfloat16, device=dev()).permute(0, 3, 1, 2)
    assert not hip().decode_kernel_takes(q, kc, vc), "head_dim 48"
    q64 = torch.zeros(2, 4, 64, dtype=torch.bfloat16, device=dev())
    plain = torch.zeros(3, 16, 2, 64, dtype=torch.bfloat16, device=dev())
    assert not hip().decode_kernel_takes(q64, plain, plain), "values not in transposed pages"
    assert not hip().decode_kernel_takes(q64.float(), plain.float(), plain.float()), "float32"
    with pytest.raises(hip().KernelError, match="decode kernel takes"):
        hip().paged_attention_decode(q, kc, vc, torch.zeros(1, 3, dtype=torch.int32, device=dev()),
                                     torch.zeros(2, dtype=torch.int32, device=dev()), torch.zeros(2, dtype=torch.int32, device=dev()), 1.0)


def test_split_key_decode_window_and_far_key():
    dtype = torch.bfloat16
    n, heads, kv, hd, page, window = 700, 4, 2, 64, 64, 300
    g = gen(21)
    q = torch.randn(n, heads, hd, generator=g) * 0.1
    k, v = torch.randn(n, kv, hd, generator=g) * 0.1, torch.randn(n, kv, hd, generator=g)
    table = list(range(10, -1, -1))
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev())
    kc, vc = engine_layout(k.to(dtype), v.to(dtype), table, page, 11, dtype)
    rows = [5, 299, 300, 301, 699]
    want = P.causal_attention(q.to(dtype).double(), k.to(dtype).double(), v.to(dtype).double(), window=window)[rows]
    out = hip().paged_attention_decode(q[rows].to(dtype).to(dev()), kc, vc, i32([table]), i32([0] * 5), i32(rows),
                                       hd ** -0.5, window=window, chunk=128)
    torch.testing.assert_close(out.double().cpu(), want, **tol(dtype))
    for target in (0, 63, 64, 389, 640):
        kk = k.clone()
        kk[target] = 0
        kk[target, :, 5] = 40.0
        qq = q[[699]].clone()
        qq[:, :, 5] = 40.0
        kc, vc = engine_layout(kk.to(dtype), v.to(dtype), table, page, 11, dtype)
        out = hip().paged_attention_decode(qq.to(dtype).to(dev()), kc, vc, i32([table]), i32([0]), i32([699]), hd ** -0.5)
        for h in range(heads):
            torch.testing.assert_close(out[0, h].float().cpu(), v[target, h // 2].to(dtype).float(), rtol=1e-3, atol=1e-3)
        seen = target > 699 - window
        out = hip().paged_attention_decode(qq.to(dtype).to(dev()), kc, vc, i32([table]), i32([0]), i32([699]), hd ** -0.5,
                                           window=window)
        assert torch.allclose(out[0, 0].float().cpu(), v[target, 0].to(dtype).float(), rtol=1e-2, atol=1e-2) == seen


@pytest.mark.parametrize("page,pool_page", [(256, 32), (64, 32), (128, 64), (48, 8)])
def test_block_tables_may_count_in_longer_pages_than_the_pools_are_cut_into(page, pool_page):
    """An entry of a block table may stand for several consecutive pages of the pools (the engine's
    bfloat16 pools are cut into pages of 32 slots whatever page size the manager counts in): the
    three attention kernels read the same keys either way, and give the same result bit for bit."""
    dtype = torch.bfloat16
    n, heads, kv, hd = 600, 8, 2, 64
    per = page // pool_page
    if per & (per - 1):
        with pytest.raises(hip().KernelError, match="power of two"):
            hip().paged_attention_wave(torch.zeros(1, heads, hd, dtype=dtype, device=dev()),
                                       torch.zeros(6, pool_page, kv, hd, dtype=dtype, device=dev()),
                                       torch.zeros(6, pool_page, kv, hd, dtype=dtype, device=dev()),
                                       torch.zeros(1, 1, dtype=torch.int32, device=dev()), torch.zeros(1, dtype=torch.int32, device=dev()),
                                       torch.zeros(1, dtype=torch.int32, device=dev()), 1.0, pages_per_entry=per)
        return
    g = gen(page + pool_page)
    q = torch.randn(n, heads, hd, generator=g).to(dtype)
    k, v = torch.randn(n, kv, hd, generator=g).to(dtype), torch.randn(n, kv, hd, generator=g).to(dtype)
    pages = -(-n // page) + 2
    table = torch.randperm(pages, generator=g)[:-(-n // page)].tolist()
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev())
    kc, vc = engine_layout(k, v, table, page, pages, dtype)                       # pools in pages of `page`
    # the same slots in pools of `pool_page`: page p of the table is the pool's pages p * per + j
    fine = [table[e] * per + j for e in range(len(table)) for j in range(per)]
    kf, vf = engine_layout(k, v, fine, pool_page, pages * per, dtype)
    rows = [0, 31, 32, pool_page, page - 1, page, 333, 599]
    qd, tables, seqs, positions = q[rows].to(dev()), i32([table]), i32([0] * len(rows)), i32(rows)
    want = P.causal_attention(q.double(), k.double(), v.double())[rows]
    for run in (lambda kc, vc, **kw: hip().paged_attention_wave(qd, kc, vc, tables, seqs, positions, hd ** -0.5, **kw),
                lambda kc, vc, **kw: hip().paged_attention_decode(qd, kc, vc, tables, seqs, positions, hd ** -0.5, chunk=256, waves=8, **kw),
                lambda kc, vc, **kw: hip().paged_attention_decode(qd, kc, vc, tables, seqs, positions, hd ** -0.5, window=100, **kw)):
        coarse, sub = run(kc, vc), run(kf, vf, pages_per_entry=per)
        assert torch.equal(coarse, sub)
    torch.testing.assert_close(hip().paged_attention_decode(qd, kf, vf, tables, seqs, positions, hd ** -0.5, pages_per_entry=per).double().cpu(),
                               want, **tol(dtype))
    # a whole prompt through the tile kernel
    tile_tokens = 4 * (16 // (heads // kv))
    tiles = i32(hip().attention_tiles([0, n], [0], tile_tokens)).view(-1, 2)
    every = i32(list(range(n)))
    whole = lambda kc, vc, **kw: hip().paged_attention_prefill(q.to(dev()), kc, vc, tables, i32([0] * n), every, tiles, hd ** -0.5,
                                                               tile_tokens=tile_tokens, **kw)
    coarse, sub = whole(kc, vc), whole(kf, vf, pages_per_entry=per)
    assert torch.equal(coarse, sub)
    torch.testing.assert_close(sub.double().cpu(), P.causal_attention(q.double(), k.double(), v.double()), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
def test_wave_kernel_reads_the_engine_layout(dtype):
    n, heads, kv, hd, page = 100, 6, 3, 48, 16
    g = gen(23)
    q, k, v = (torch.randn(n, h, hd, generator=g).to(dtype) for h in (heads, kv, kv))
    table = list(range(6, -1, -1))
    kc, vc = engine_layout(k, v, table, page, 7, dtype)
    out = run_attention(q, kc, vc, [table], [0] * n, list(range(n)), hd ** -0.5)
    torch.testing.assert_close(out.double().cpu(), P.causal_attention(q.double(), k.double(), v.double()), **tol(dtype))


def test_attention_refuses_sizes_it_cannot_take():
    kc = torch.zeros(2, 4, 1, 24, device=dev())
    with pytest.raises(hip().KernelError, match="multiple of 16"):
        hip().paged_attention_wave(torch.zeros(1, 1, 24, device=dev()), kc, kc, torch.zeros(1, 1, dtype=torch.int32, device=dev()),
                                   torch.zeros(1, dtype=torch.int32, device=dev()), torch.zeros(1, dtype=torch.int32, device=dev()), 1.0)
    kc = torch.zeros(2, 4, 2, 16, device=dev())
    with pytest.raises(hip().KernelError, match="divide"):
        hip().paged_attention_wave(torch.zeros(1, 3, 16, device=dev()), kc, kc, torch.zeros(1, 1, dtype=torch.int32, device=dev()),
                                   torch.zeros(1, dtype=torch.int32, device=dev()), torch.zeros(1, dtype=torch.int32, device=dev()), 1.0)


@pytest.mark.parametrize("m,n,k", [(70, 130, 50), (1, 384, 96), (3, 5, 7), (129, 64, 160), (33, 1000, 2048)])
def test_gemm_exact(m, n, k):
    g = gen(m * n)
    a, w = torch.randn(m, k, generator=g), torch.randn(n, k, generator=g)
    out = hip().gemm_exact(a.to(dev()), w.to(dev()))
    torch.testing.assert_close(out.double().cpu(), a.double() @ w.double().T, rtol=1e-5, atol=1e-5 * math.sqrt(k))
    one = hip().gemm_exact(a[m // 2:m // 2 + 1].contiguous().to(dev()), w.to(dev()))
    assert torch.equal(one, out[m // 2:m // 2 + 1]), "a row's result does not depend on the other rows"
    a16, w16 = a.bfloat16(), w.bfloat16()
    out = hip().gemm_exact(a16.to(dev()), w16.to(dev()), torch.float32)
    torch.testing.assert_close(out.double().cpu(), a16.double() @ w16.double().T, rtol=1e-5, atol=1e-5 * math.sqrt(k))
    out = hip().gemm_exact(a16.to(dev()), w16.to(dev()))
    assert out.dtype == torch.bfloat16
    torch.testing.assert_close(out.double().cpu(), a16.double() @ w16.double().T, rtol=1e-2, atol=1e-2 * math.sqrt(k))


@pytest.mark.parametrize("m,n,k", [(1, 384, 96), (8, 3072, 2048), (64, 2048, 8192), (200, 1000, 160), (2048, 512, 2048)])
def test_linear_bfloat16(m, n, k):
    from tinyserve_llm_amd.parts.linear import linear
    g = gen(m + n)
    a, w = torch.randn(m, k, generator=g).bfloat16(), (torch.randn(n, k, generator=g) * 0.05).bfloat16()
    out = linear(a.to(dev()), w.to(dev()))
    want = a.double() @ w.double().T
    assert out.dtype == torch.bfloat16 and out.shape == (m, n)
    torch.testing.assert_close(out.double().cpu(), want, rtol=2e-2, atol=2e-2 * float(want.abs().max()))
    f = linear(a.to(dev()), w.to(dev()), out_dtype=torch.float32)
    assert f.dtype == torch.float32


@pytest.mark.parametrize("m,n,k", [(33, 384, 96), (2056, 16384, 2048), (100, 1000, 160), (257, 130, 3072), (64, 128256, 512),
                                   (777, 2048, 8192), (2063, 4096, 1024)])
def test_library_product_called_directly(m, n, k):
    """x · W^T through the vendor's library with the algorithm kept per shape: against 64-bit, twice
    (the second call takes the kept plan), and with rows of x that lie apart in memory."""
    g = gen(m + n + k)
    a, w = torch.randn(m, 2 * k, generator=g).bfloat16(), (torch.randn(n, k, generator=g) * 0.05).bfloat16()
    want = a[:, :k].double() @ w.double().T
    tolerance = dict(rtol=2e-2, atol=2e-2 * float(want.abs().max()))
    ad, wd = a.to(dev()), w.to(dev())
    dense = ad[:, :k].contiguous()
    for _ in range(2):
        out = hip().gemm_library(dense, wd)
        assert out.dtype == torch.bfloat16 and out.shape == (m, n)
        torch.testing.assert_close(out.double().cpu(), want, **tolerance)
    # rows that lie apart are a shape of their own, which may keep another algorithm (another order of sums)
    torch.testing.assert_close(hip().gemm_library(ad[:, :k], wd).double().cpu(), want, **tolerance)
    with pytest.raises(hip().KernelError):
        hip().gemm_library(ad.t()[:k].t()[:, ::2], wd[:, ::2])      # elements of a row must be adjacent


@pytest.mark.parametrize("n,k", [(128256, 2048), (1000, 160), (32000, 4096)])
def test_float32_logits_are_the_32_bit_sums_whatever_the_number_of_rows(n, k):
    """The head's product for one row, for 16 (the weight-streaming kernel), and for 17, 40 and 300
    (the library, which is asked for its 32-bit sums instead of a bfloat16 result widened afterwards):
    a row's logits agree to 32-bit rounding whichever kernel its step takes, so the choice between two
    close tokens does not depend on how many requests share the step. A result that had passed through
    bfloat16 would be off by up to 2^-9 of its size."""
    from tinyserve_llm_amd.parts.linear import linear
    g = gen(n + k)
    a, w = torch.randn(300, k, generator=g).bfloat16(), (torch.randn(n, k, generator=g) * 0.05).bfloat16()
    want = (a[:1].double() @ w.double().T)[0]
    ad, wd = a.to(dev()), w.to(dev())
    scale = float(want.abs().max())
    for rows in (1, 16, 17, 40, 300):
        out = linear(ad[:rows].contiguous(), wd, out_dtype=torch.float32)
        assert out.dtype == torch.float32 and out.shape == (rows, n)
        err = float((out[0].double().cpu() - want).abs().max())
        assert err <= 2e-5 * scale, f"{rows} rows: error {err:.3e} of {scale:.3f}"
    if hip().tiled_takes(ad, wd):
        out = hip().gemm_tiled(ad[:40].contiguous(), wd, out_dtype=torch.float32)     # the engine's own product for many rows
        assert out.dtype == torch.float32 and float((out[0].double().cpu() - want).abs().max()) <= 2e-5 * scale


@pytest.mark.parametrize("m,n,k", [(300, 384, 64), (2056, 16384, 2048), (100, 1000, 192), (257, 132, 3072), (515, 128256, 128),
                                   (2048, 2048, 8192), (33, 8, 320), (1, 4, 64)])
def test_tiled_product(m, n, k):
    """The engine's own product for many rows against 64-bit: tiles that hang over the last rows
    and columns, one, two, three and many k-steps (odd and even counts end differently), rows of x
    that lie apart, and the gated form against the separate steps with their roundings."""
    g = gen(m + n + k)
    a, w = torch.randn(m, 2 * k, generator=g).bfloat16(), (torch.randn(n, k, generator=g) * 0.05).bfloat16()
    want = a[:, :k].double() @ w.double().T
    tolerance = dict(rtol=2e-2, atol=2e-2 * float(want.abs().max()))
    ad, wd = a.to(dev()), w.to(dev())
    out = hip().gemm_tiled(ad[:, :k].contiguous(), wd)
    assert out.dtype == torch.bfloat16 and out.shape == (m, n)
    torch.testing.assert_close(out.double().cpu(), want, **tolerance)
    assert torch.equal(hip().gemm_tiled(ad[:, :k], wd), out), "the order of the sums does not depend on the strides"
    if n % 8 == 0:
        gated = hip().gemm_tiled(ad[:, :k], wd, glu=True)
        y = want.bfloat16().double()
        ref = (torch.nn.functional.silu(y[:, :n // 2]) * y[:, n // 2:])
        assert gated.shape == (m, n // 2)
        torch.testing.assert_close(gated.double().cpu(), ref, rtol=3e-2, atol=3e-2 * float(ref.abs().max()))
    with pytest.raises(hip().KernelError, match="tiled kernel takes"):
        hip().gemm_tiled(ad[:, :k - 8], wd[:, :k - 8])
    with pytest.raises(hip().KernelError, match="tiled kernel takes"):
        hip().gemm_tiled(ad[:, :k], wd[:n - 1])


@pytest.mark.parametrize("m", [1, 3, 8, 16, 17, 32])
@pytest.mark.parametrize("n,k", [(3072, 2048), (2048, 2048), (16384, 2048), (2048, 8192), (992, 512), (130, 3072), (64, 4096),
                                 (8192, 3072), (8256, 4096)])
def test_weight_streaming_gemm_and_its_fused_inputs(m, n, k):
    """The skinny kernel plain, with residual + RMSNorm on the way in, and with the SiLU gate on
    the way in, against the same operations done one after the other in float64 with the storage
    type's roundings in between."""
    g = gen(m * 7 + n + k)
    w = (torch.randn(n, k, generator=g) * 0.05).bfloat16()
    x = torch.randn(m, k, generator=g).bfloat16()
    assert hip().skinny_takes(m, k)
    out, none = hip().gemm_skinny(x.to(dev()), w.to(dev()))
    want = x.double() @ w.double().T
    assert none is None and out.dtype == torch.bfloat16
    torch.testing.assert_close(out.double().cpu(), want, rtol=2e-2, atol=2e-2 * float(want.abs().max()))
    f32, _ = hip().gemm_skinny(x.to(dev()), w.to(dev()), torch.float32)
    torch.testing.assert_close(f32.double().cpu(), want, rtol=1e-4, atol=1e-4 * float(want.abs().max()))
    one, _ = hip().gemm_skinny(x[m // 2:m // 2 + 1].contiguous().to(dev()), w.to(dev()), torch.float32)
    assert torch.equal(one, f32[m // 2:m // 2 + 1]), "a row's result does not depend on the other rows"
    if hip().skinny_fuses(m, k, True, False):
        res = torch.randn(m, k, generator=g).bfloat16()
        nw = (1 + 0.1 * torch.randn(k, generator=g)).bfloat16()
        for r in (res, None):
            for glu in (False, True):
                if glu and not (n % 32 == 0 and hip().skinny_fuses(m, k, True, True)):
                    continue
                out, res_out = hip().gemm_skinny(x.to(dev()), w.to(dev()), residual=None if r is None else r.to(dev()),
                                                 norm_weight=nw.to(dev()), eps=1e-5, glu=glu)
                s = x.float() + (r.float() if r is not None else 0)
                assert torch.equal(res_out.cpu(), s.bfloat16()), "the new residual is the sum, rounded once"
                y = (s * torch.rsqrt(s.pow(2).mean(-1, keepdim=True) + 1e-5)).bfloat16() * nw      # llama.py:63-67
                want = y.double() @ w.double().T
                if glu:
                    want = P.silu_mul(want)
                torch.testing.assert_close(out.double().cpu(), want, rtol=2e-2, atol=2e-2 * float(want.abs().max()))
    if n % 32 == 0 and hip().skinny_fuses(m, k, False, True):
        out, _ = hip().gemm_skinny(x.to(dev()), w.to(dev()), glu=True)
        want = P.silu_mul(x.double() @ w.double().T)
        assert out.shape == (m, n // 2)
        torch.testing.assert_close(out.double().cpu(), want, rtol=2e-2, atol=2e-2 * float(want.abs().max()))


@pytest.mark.parametrize("m", [17, 32, 33, 48, 64])
@pytest.mark.parametrize("n,k", [(16384, 2048), (2048, 2048), (320, 768), (6144, 1024)])
def test_gate_on_the_way_out_for_up_to_64_rows(m, n, k):
    """silu(gate) * up straight from the gate|up product for two and four blocks of 16 rows of x,
    against the product in 64-bit followed by the gate; a row among many equals the row alone."""
    g = gen(m + n + k)
    w = (torch.randn(n, k, generator=g) * 0.05).bfloat16().to(dev())
    x = torch.randn(m, k, generator=g).bfloat16().to(dev())
    assert hip().skinny_fuses(m, k, False, True) and not hip().skinny_fuses(m, k, True, True)
    out, _ = hip().gemm_skinny(x, w, glu=True)
    want = P.silu_mul(x.double().cpu() @ w.double().cpu().T)
    assert out.shape == (m, n // 2) and out.dtype == torch.bfloat16
    torch.testing.assert_close(out.double().cpu(), want, rtol=2e-2, atol=2e-2 * float(want.abs().max()))
    alone, _ = hip().gemm_skinny(x[m - 1:].contiguous(), w, glu=True)
    assert torch.equal(alone[0], out[m - 1])
    from tinyserve_llm_amd.parts.linear import linear
    assert torch.equal(linear(x, w, glu=True), out), "the part's projection takes this path"
    with pytest.raises(hip().KernelError):
        hip().gemm_skinny(x.repeat(4, 1)[:65].contiguous(), w, glu=True)


def test_weight_streaming_gemm_refuses_what_it_cannot_take():
    x = torch.zeros(33, 2304, dtype=torch.bfloat16, device=dev())
    w = torch.zeros(64, 2304, dtype=torch.bfloat16, device=dev())
    assert hip().skinny_takes(33, 2048) and hip().skinny_takes(64, 256), "33 to 64 rows over reductions of up to 2048"
    assert not hip().skinny_takes(33, 2304) and not hip().skinny_takes(65, 2048)
    assert not hip().skinny_takes(8, 96) and not hip().skinny_takes(8, 14336)
    with pytest.raises(hip().KernelError, match="rows"):
        hip().gemm_skinny(x, w)
    from tinyserve_llm_amd.parts.linear import linear
    assert linear(x, w).shape == (33, 64), "the vendor library takes what the skinny kernel does not"


@pytest.mark.parametrize("m", [33, 48, 64])
@pytest.mark.parametrize("n,k", [(2048, 2048), (3072, 1024), (130, 768), (8200, 256)])
def test_weight_streaming_gemm_for_33_to_64_rows(m, n, k):
    """Three and four blocks of 16 rows of x against one tile of W a workgroup, x asked for before W."""
    g = gen(m + n + k)
    w = (torch.randn(n, k, generator=g) * 0.05).bfloat16().to(dev())
    x = torch.randn(m, k, generator=g).bfloat16().to(dev())
    want = x.double().cpu() @ w.double().cpu().T
    for packed in (None, hip().pack_weight(w)):
        out, _ = hip().gemm_skinny(x, w, packed=packed)
        assert out.shape == (m, n) and out.dtype == torch.bfloat16
        torch.testing.assert_close(out.double().cpu(), want, rtol=2e-2, atol=2e-2 * float(want.abs().max()))
    alone, _ = hip().gemm_skinny(x[m - 1:].contiguous(), w)
    assert torch.equal(alone[0], out[m - 1]), "a row's result does not depend on the other rows"


def bf(t):
    """Rounded to bfloat16 and back to 64-bit."""
    return t.float().bfloat16().double()


@pytest.mark.parametrize("m,n,k", [(1, 2048, 2048), (8, 2048, 8192), (5, 264, 512), (3, 44, 256), (8, 3072, 1024),     # the 8-row form
                                   (16, 2048, 2048), (9, 130, 768), (23, 992, 512), (32, 2048, 4096), (12, 8224, 256),  # 16-row tiles
                                   (48, 2048, 2048), (64, 3072, 1024), (33, 72, 512)])                                  # four blocks of x
@pytest.mark.parametrize("with_residual", [True, False])
def test_projection_that_finishes_into_a_residual_sum_and_a_norm(m, n, k, with_residual):
    """`next_norm=`: the projection leaves T(T(y) + res), T((T(y) + res) * nw) and the rows' sums of
    squares in parts, against the same steps in 64-bit with the storage type's roundings; then the
    projections that take the prepared operand (plain, gated, into the rotation and the cache, and
    the shared-x kernel) against their own definition on exactly these operands, and the whole chain
    against norm(y + res) * nw followed by the product without any rounding."""
    g = gen(m * 3 + n + k)
    x = torch.randn(m, k, generator=g).bfloat16()
    w = (torch.randn(n, k, generator=g) * k ** -0.5).bfloat16()
    res = torch.randn(m, n, generator=g).bfloat16() if with_residual else None
    nw = (1 + 0.1 * torch.randn(n, generator=g)).bfloat16()
    eps = 1e-5
    xd, wd, nwd = x.to(dev()), w.to(dev()), nw.to(dev())
    def finish(rows, residual):
        # (`linear_bf16` leaves 33 to 64 rows to the library; the kernel takes them when asked directly)
        request = (None if residual is None else residual.to(dev()), nwd)
        if hip().next_norm_fuses(rows, wd):
            return hip().linear_bf16(rows, wd, next_norm=request)
        return hip().gemm_skinny(rows, wd, next_norm=request)[0]

    assert hip().next_norm_fuses(xd, wd) == (m <= 32)
    prepared = finish(xd, res)
    assert isinstance(prepared, hip().PreparedNorm)
    y = x.double() @ w.double().T
    t = bf(y) + (res.double() if with_residual else 0)
    # (a product that lies next to a rounding boundary may round the other way than 64-bit does)
    torch.testing.assert_close(prepared.summed.double().cpu(), bf(t), rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(prepared.operand.double().cpu(), bf(t * nw.double()), rtol=2e-2, atol=2e-2)
    assert prepared.squares.dtype == torch.float32 and prepared.squares.shape[0] == m
    torch.testing.assert_close(prepared.squares.sum(1).double().cpu(), t.pow(2).sum(1), rtol=1e-2, atol=1e-3)
    # every part is the sum of squares of its own columns: 8 a part in the 8-row form, else 16
    width = 8 if hip().skinny8_takes(m, n, k) else 16
    assert prepared.squares.shape[1] >= -(-n // width)
    own = prepared.summed.float()      # (within a rounding of t)
    parts = torch.stack([own[:, i:i + width].pow(2).sum(1) for i in range(0, n, width)], 1)
    torch.testing.assert_close(prepared.squares[:, :parts.shape[1]].cpu(), parts.cpu(), rtol=3e-2, atol=1e-3)
    assert float(prepared.squares[:, parts.shape[1]:].abs().sum()) == 0.0, "tiles past the last column count nothing"
    alone = finish(xd[m - 1:].contiguous(), None if res is None else res[m - 1:])
    if hip().skinny8_takes(m, n, k) == hip().skinny8_takes(1, n, k):
        assert torch.equal(alone.summed[0], prepared.summed[m - 1]) and torch.equal(alone.operand[0], prepared.operand[m - 1])
    # ---- what takes the prepared operand: K of the next projection is this one's N
    scale = torch.rsqrt(prepared.squares.double().cpu().sum(1, keepdim=True) / n + eps)
    operand = prepared.operand.double().cpu()
    truth_in = t * torch.rsqrt(t.pow(2).mean(1, keepdim=True) + eps) * nw.double()          # no rounding
    if n % 256 == 0 and n <= 4096:
        for n2, glu in ((2 * 320, True), (264, False), (16384 if n <= 2048 else 512, True)):
            if not (hip().skinny_fuses(m, n, False, True) if glu else hip().skinny_takes(m, n)):
                continue
            w2 = (torch.randn(n2, n, generator=g) * n ** -0.5).bfloat16()
            out, _ = hip().gemm_skinny(prepared.operand, w2.to(dev()), glu=glu, squares=prepared.squares, eps=eps)
            want = (operand @ w2.double().T) * scale
            truth = truth_in @ w2.double().T
            if glu:
                want, truth = P.silu_mul(want), P.silu_mul(truth)
            torch.testing.assert_close(out.double().cpu(), want, rtol=2e-2, atol=2e-2 * float(want.abs().max()))
            torch.testing.assert_close(out.double().cpu(), truth, rtol=4e-2, atol=4e-2 * float(truth.abs().max()))
    if n % 1024 == 0 and m > 32:
        for glu in (False, True):
            w2 = (torch.randn(8192, n, generator=g) * n ** -0.5).bfloat16().to(dev())
            out = hip().gemm_rows64(prepared.operand, hip().pack_weight(w2), glu=glu, squares=prepared.squares, eps=eps)
            want = (operand @ w2.double().cpu().T) * scale
            want = P.silu_mul(want) if glu else want
            torch.testing.assert_close(out.double().cpu(), want, rtol=2e-2, atol=2e-2 * float(want.abs().max()))
    if hip().qkv_rope_fuses(prepared.operand, torch.empty(1, n, dtype=torch.bfloat16, device=dev()), 64, None):
        nh, nkv, hd = 3, 1, 64
        w2 = (torch.randn((nh + 2 * nkv) * hd, n, generator=g) * n ** -0.5).bfloat16().to(dev())
        table = torch.randn(32, hd, generator=g).to(dev())
        positions = torch.randint(0, 32, (m,), generator=g, dtype=torch.int32).to(dev())
        slots = torch.randperm(128, generator=g)[:m].to(torch.int32).to(dev())
        kp = [torch.zeros(4, nkv, 32, hd, dtype=torch.bfloat16, device=dev()) for _ in range(2)]
        vp = [torch.zeros(4, nkv, hd, 32, dtype=torch.bfloat16, device=dev()) for _ in range(2)]
        q, _ = hip().qkv_rope_store(prepared.operand, w2, table, positions, slots, kp[0].permute(0, 2, 1, 3),
                                    vp[0].permute(0, 3, 1, 2), nh, nkv, hd, eps=eps, squares=prepared.squares)
        # the same through the separate kernels: the norm applied to the operand first
        normed = (operand * scale).bfloat16().to(dev())
        q_want = hip().rope_store(hip().linear_bf16(normed, w2), table, positions, slots, kp[1].permute(0, 2, 1, 3),
                                  vp[1].permute(0, 3, 1, 2), nh, nkv, hd)
        torch.testing.assert_close(q.double(), q_want.double(), rtol=3e-2, atol=3e-2 * float(q_want.abs().max()))
        torch.testing.assert_close(kp[0].double(), kp[1].double(), rtol=3e-2, atol=3e-2 * float(kp[1].abs().max()))
        torch.testing.assert_close(vp[0].double(), vp[1].double(), rtol=3e-2, atol=3e-2 * float(vp[1].abs().max()))
        assert torch.equal(kp[0] == 0, kp[1] == 0), "the same slots are written"


def test_a_prepared_norm_is_refused_where_no_kernel_leaves_one():
    x = torch.zeros(70, 512, dtype=torch.bfloat16, device=dev())
    w = torch.zeros(64, 512, dtype=torch.bfloat16, device=dev())
    nw = torch.ones(64, dtype=torch.bfloat16, device=dev())
    assert not hip().next_norm_fuses(x, w), "70 rows go to the vendor's library"
    with pytest.raises(hip().KernelError, match="prepared norm"):
        hip().linear_bf16(x, w, next_norm=(None, nw))
    with pytest.raises(hip().KernelError, match="next norm's weight"):
        hip().linear_bf16(x[:8].contiguous(), w, next_norm=(None, nw[:32].contiguous()))
    with pytest.raises(hip().KernelError, match="residual"):
        hip().linear_bf16(x[:8].contiguous(), w, next_norm=(x[:8, :32], nw))
    with pytest.raises(hip().KernelError, match="sums of squares"):
        hip().gemm_skinny(x[:8].contiguous(), w, squares=torch.zeros(7, 4, device=dev()), eps=1e-5)
    from tinyserve_llm_amd.parts.linear import DeferredNorm, NormRequest, linear
    d = linear(x, w, then=NormRequest(nw, 1e-5, None))
    assert isinstance(d, DeferredNorm) and d.prepared is None and d.x.shape == (70, 64), "left to the next projection"
    d8 = linear(x[:8].contiguous(), w, then=NormRequest(nw, 1e-5, None))
    assert d8.prepared is not None and d8.residual_out is d8.prepared.summed
    assert d8.materialize().shape == (8, 64)


@pytest.mark.parametrize("dtype", DTYPES)
def test_silu_mul(dtype):
    gu = torch.randn(9, 2 * 150, generator=gen(13)).to(dtype)
    out = hip().silu_mul(gu.to(dev()))
    torch.testing.assert_close(out.double().cpu(), P.silu_mul(gu.double()), **tol(dtype))
    gu[:, :150] = 0
    assert float(hip().silu_mul(gu.to(dev())).abs().max()) == 0.0


@pytest.mark.parametrize("dtype", DTYPES)
def test_copy_slots_copies_the_leading_slots_of_every_layer(dtype):
    pool = torch.randn(5, 3, 2, 8, 16, generator=gen(14)).to(dtype).to(dev())   # [pages, x, heads, slots, dim]
    before = pool.clone()
    hip().copy_slots(pool, 3, 1, 5, slot_dim=3)
    assert torch.equal(pool[1, :, :, :5], before[3, :, :, :5]) and torch.equal(pool[1, :, :, 5:], before[1, :, :, 5:])
    keep = [0, 2, 3, 4]
    assert torch.equal(pool[keep], before[keep])
    vpool = torch.randn(5, 3, 2, 16, 8, generator=gen(15)).to(dtype).to(dev())  # [pages, layers, heads, dim, slots]
    vbefore = vpool.clone()
    hip().copy_slots(vpool, 3, 1, 5, slot_dim=4)
    assert torch.equal(vpool[1, ..., :5], vbefore[3, ..., :5]) and torch.equal(vpool[1, ..., 5:], vbefore[1, ..., 5:])
    assert torch.equal(vpool[keep], vbefore[keep])
    with pytest.raises(hip().KernelError):
        hip().copy_slots(pool, 3, 3, 2, slot_dim=3)
    with pytest.raises(hip().KernelError):
        hip().copy_slots(pool, 0, 5, 2, slot_dim=3)


def exp_noise(seed, key, n):
    """The kernel's counter hash, written out with Python integers."""
    M = (1 << 64) - 1

    def mix(x):
        x ^= x >> 30
        x = (x * 0xBF58476D1CE4E5B9) & M
        x ^= x >> 27
        x = (x * 0x94D049BB133111EB) & M
        return x ^ (x >> 31)

    out = []
    for i in range(n):
        x = mix((mix(seed ^ ((key * 0x9E3779B97F4A7C15) & M)) + i * 0xD1342543DE82EF95) & M)
        u = ((x >> 40) + 1) / 16777216.0
        out.append(max(-math.log(u), 1e-10))
    return torch.tensor(out, dtype=torch.float64)


def test_sampler_greedy_vector_frequencies_and_seeds():
    """The cases of the reference's sampler test (tests/test_engine.py:121-129)."""
    from tinyserve_llm_amd.sampling.sampler import row_key, sample
    logits = torch.tensor([[0.0, 5.0, 1.0], [3.0, 0.0, 0.0]], device=dev())
    assert sample(logits, [0.0, 0.0], [1, 2], seed=0).tolist() == [1, 0]
    assert sample(torch.tensor([[2.0, 7.0, 7.0, 1.0]], device=dev()), [0.0], [1], 0).tolist() == [1], "ties: lowest index"
    rows = 20000
    keys = [row_key(3, 0, i) for i in range(rows)]
    draws = sample(logits[:1].expand(rows, 3).contiguous(), [1.0] * rows, keys, seed=0)
    freq = torch.bincount(draws.long().cpu(), minlength=3).double() / rows
    torch.testing.assert_close(freq, torch.softmax(logits[0].double().cpu(), -1), atol=0.01, rtol=0)
    cold = sample(logits[:1].expand(rows, 3).contiguous(), [0.25] * rows, keys, seed=0)
    freq = torch.bincount(cold.long().cpu(), minlength=3).double() / rows
    torch.testing.assert_close(freq, torch.softmax(logits[0].double().cpu() / 0.25, -1), atol=0.01, rtol=0)
    again = sample(logits[:1].expand(rows, 3).contiguous(), [1.0] * rows, keys, seed=0)
    other = sample(logits[:1].expand(rows, 3).contiguous(), [1.0] * rows, keys, seed=1)
    assert torch.equal(draws, again) and not torch.equal(draws, other)


def test_sampler_draw_is_the_exponential_race_and_ignores_the_row_order():
    """argmax(softmax(logits / t) / E) with the kernel's own noise, computed here in float64
    (tinyserve_llm/engine/sampler.py:18-23); and a row's draw depends on its key, not its place."""
    from tinyserve_llm_amd.sampling.sampler import sample
    vocab, rows = 1500, 12
    logits = torch.randn(rows, vocab, generator=gen(15)) * 3
    temps = [0.7, 1.0, 0.0, 1.3] * 3
    keys = [1000 + 17 * r for r in range(rows)]
    got = sample(logits.to(dev()), temps, keys, seed=42).tolist()
    for r in range(rows):
        if temps[r] == 0:
            assert got[r] == int(logits[r].argmax())
            continue
        p = torch.softmax(logits[r].double() / temps[r], -1)
        assert got[r] == int((p / exp_noise(42, keys[r], vocab)).argmax())
    perm = torch.randperm(rows, generator=gen(16)).tolist()
    shuffled = sample(logits[perm].contiguous().to(dev()), [temps[i] for i in perm], [keys[i] for i in perm], seed=42).tolist()
    assert shuffled == [got[i] for i in perm]


def test_several_draws_may_read_one_row_of_logits():
    """The n samples of a prompt are drawn from the one row its last position gave: the draws name
    their rows, and the result is what separate copies of the rows would give."""
    from tinyserve_llm_amd.sampling.sampler import sample
    logits = (torch.randn(4, 700, generator=gen(31)) * 0.5).to(dev())        # flat enough for two draws of a row to differ
    rows, temps, keys = [2, 2, 2, 0, 3, 3], [0.8, 0.8, 0.0, 1.1, 0.6, 0.6], [11, 12, 13, 14, 15, 15]
    got = sample(logits, temps, keys, seed=5, rows=rows).tolist()
    want = sample(logits[torch.tensor(rows)].contiguous(), temps, keys, seed=5).tolist()
    assert got == want and got[2] == int(logits[2].argmax()) and got[4] == got[5] and got[0] != got[1]
    with pytest.raises(ValueError, match="rows"):
        sample(logits, temps, keys, seed=5, rows=[0, 1, 2, 3, 4, 0])


@pytest.mark.parametrize("nh,nkv,hd,K,M,page", [(32, 8, 64, 2048, 8, 64), (6, 2, 96, 768, 5, 16), (4, 4, 128, 256, 16, 8),
                                                 (3, 1, 32, 1280, 1, 32), (24, 8, 128, 3072, 8, 64), (8, 2, 128, 4096, 3, 32),
                                                 (32, 8, 64, 2048, 24, 64), (32, 8, 64, 2048, 64, 64), (6, 2, 96, 768, 40, 16),
                                                 (3, 1, 32, 1280, 33, 32)])
@pytest.mark.parametrize("norm", [False, True])
@pytest.mark.parametrize("rotate", [True, False])
def test_fused_projection_rotation_and_cache_write(nh, nkv, hd, K, M, page, norm, rotate):
    """The one-kernel path against projection, then rope_store: q, every written slot of k and v, and
    slots it must not touch (slot -1, and pages of other requests)."""
    g = gen(nh * 7 + K)
    dtype = torch.bfloat16
    x = (torch.randn(M, K, generator=g) * 0.5).to(dtype).to(dev())
    w = (torch.randn((nh + 2 * nkv) * hd, K, generator=g) * K ** -0.5).to(dtype).to(dev())
    res = (torch.randn(M, K, generator=g) * 0.5).to(dtype).to(dev())
    nw = (1 + 0.1 * torch.randn(K, generator=g)).to(dtype).to(dev())
    table = torch.randn(64, hd, generator=g).to(dev()) if rotate else None
    positions = torch.randint(0, 64, (M,), generator=g, dtype=torch.int32).to(dev())
    pages = 6
    perm = torch.randperm(pages * page, generator=g)[:M].to(torch.int32)
    if M > 2:
        perm[1] = -1
    slots = perm.to(dev())
    def pools():
        kp = torch.full((pages, nkv, page, hd), 7.0, dtype=dtype, device=dev())
        vp = torch.full((pages, nkv, hd, page), 7.0, dtype=dtype, device=dev())
        return kp, vp
    kp1, vp1 = pools()
    kp2, vp2 = pools()
    if norm:
        xn, res_want = hip().rmsnorm(x, nw, 1e-5, res)
    else:
        xn, res_want = x, None
    from tinyserve_llm_amd.parts.linear import linear
    qkv = linear(xn, w)
    q_want = hip().rope_store(qkv, table, positions, slots, kp1.permute(0, 2, 1, 3), vp1.permute(0, 3, 1, 2), nh, nkv, hd)
    assert hip().qkv_rope_fuses(x, w, hd, kp2.permute(0, 2, 1, 3))
    if norm and (K > 2048 or M > 16):   # the norm rides along only up to 2048 and 16 rows; a part runs it by itself beyond
        assert not hip().qkv_rope_fuses(x, w, hd, kp2.permute(0, 2, 1, 3), norm=True)
        with pytest.raises(hip().KernelError, match="qkv_rope_store takes"):
            hip().qkv_rope_store(x, w, table, positions, slots, kp2.permute(0, 2, 1, 3), vp2.permute(0, 3, 1, 2),
                                 nh, nkv, hd, residual=res, norm_weight=nw, eps=1e-5)
        return
    q, res_out = hip().qkv_rope_store(x, w, table, positions, slots, kp2.permute(0, 2, 1, 3), vp2.permute(0, 3, 1, 2),
                                      nh, nkv, hd, **(dict(residual=res, norm_weight=nw, eps=1e-5) if norm else {}))
    # Both paths round to the storage type on the way (the one kernel applies the norm's row scale
    # to the finished sums, the separate norm kernel to the operands), so neither is the measure of
    # the other: the measure is the same chain in float64 without any rounding, and the one kernel
    # must be as close to it as the kernels one after the other are.
    s64 = x.double().cpu() + (res.double().cpu() if norm else 0)
    y64 = s64 * torch.rsqrt(s64.pow(2).mean(-1, keepdim=True) + 1e-5) * nw.double().cpu() if norm else s64
    t64 = (y64 @ w.double().cpu().T).view(M, nh + 2 * nkv, hd)
    if rotate:
        cs = table.double().cpu()[positions.cpu().long()]
        c, sn = cs[:, None, :hd // 2], cs[:, None, hd // 2:]
        a, b = t64[:, :nh + nkv, :hd // 2].clone(), t64[:, :nh + nkv, hd // 2:].clone()
        t64[:, :nh + nkv, :hd // 2], t64[:, :nh + nkv, hd // 2:] = a * c - b * sn, b * c + a * sn
    live = (slots >= 0).cpu()
    pg, off = (slots.cpu().long() // page)[live], (slots.cpu().long() % page)[live]
    def written(kp, vp):
        return kp.double().cpu()[pg, :, off, :], vp.double().cpu()[pg, :, :, off]
    (k_one, v_one), (k_seq, v_seq) = written(kp2, vp2), written(kp1, vp1)
    for name, one, seq, truth in (("q", q.double().cpu(), q_want.double().cpu(), t64[:, :nh]),
                                  ("k", k_one, k_seq, t64[live][:, nh:nh + nkv]), ("v", v_one, v_seq, t64[live][:, nh + nkv:])):
        e_one, e_seq = (one - truth).abs(), (seq - truth).abs()
        assert float(e_seq.max()) <= 3e-2 * max(1.0, float(truth.abs().max())), f"{name}: the separate kernels are off"
        assert float(e_one.max()) <= 1.25 * float(e_seq.max()) + 1e-3, f"{name}: worst error {float(e_one.max())} vs {float(e_seq.max())}"
        assert float(e_one.pow(2).mean().sqrt()) <= 1.1 * float(e_seq.pow(2).mean().sqrt()) + 1e-4, f"{name}: mean error"
    assert int((kp2 != 7.0).any(dim=(1, 3)).sum()) == int((slots >= 0).sum()), "only the named slots are written"
    assert torch.equal(kp2 == 7.0, kp1 == 7.0) and torch.equal(vp2 == 7.0, vp1 == 7.0), "the same places are written"
    if norm:
        assert torch.equal(res_out, res_want)
    # without a cache of its own a layer only gets q
    q_only, _ = hip().qkv_rope_store(x, w, table, positions, None, None, None, nh, nkv, hd,
                                     **(dict(residual=res, norm_weight=nw, eps=1e-5) if norm else {}))
    assert torch.equal(q_only, q)


@pytest.mark.parametrize("nh,nkv,hd,K,M,page,slices,prepared", [
    (32, 8, 64, 2048, 64, 256, 4, True), (32, 8, 64, 2048, 33, 16, 4, False), (24, 8, 128, 3072, 20, 32, 3, True),
    (24, 8, 128, 3072, 40, 32, 3, True), (4, 2, 128, 4096, 64, 16, 2, False), (32, 8, 64, 2048, 128, 32, 4, True),
    (24, 8, 128, 3072, 90, 16, 3, False),
    (6, 2, 32, 512, 48, 8, 1, True), (5, 3, 96, 1024, 17, 24, 2, False)])
def test_projection_in_slices_with_rotation_and_cache_write(nh, nkv, hd, K, M, page, slices, prepared):
    """The qkv projection with its reduction in slices and the kernel that adds the parts, rotates and
    writes the cache, against projection then rope_store and against the chain in 64-bit: q, every written
    slot of k and v, and the slots it must not touch. With `prepared`, x is a prepared norm's operand and
    the rows' scales multiply the finished sums."""
    g = gen(nh * 11 + K + M)
    N = (nh + 2 * nkv) * hd
    if N % 64:
        with pytest.raises(hip().KernelError):
            hip().qkv_rope_store_sliced(torch.zeros(M, K, dtype=torch.bfloat16, device=dev()),
                                        torch.zeros(-(-N // 16), K // 32, 64, 8, dtype=torch.bfloat16, device=dev()), slices, None,
                                        torch.zeros(M, dtype=torch.int32, device=dev()), None, None, None, nh, nkv, hd)
        return
    x = (torch.randn(M, K, generator=g) * 0.5).bfloat16().to(dev())
    w = (torch.randn(N, K, generator=g) * K ** -0.5).bfloat16().to(dev())
    squares = (torch.rand(M, 3, generator=g) * K / 3 + 1).to(dev()) if prepared else None
    table = torch.randn(64, hd, generator=g).to(dev())
    positions = torch.randint(0, 64, (M,), generator=g, dtype=torch.int32).to(dev())
    pages = -(-2 * M // page) + 1
    perm = torch.randperm(pages * page, generator=g)[:M].to(torch.int32)
    perm[1] = -1
    slots = perm.to(dev())
    def pools():
        return (torch.full((pages, nkv, page, hd), 7.0, dtype=torch.bfloat16, device=dev()),
                torch.full((pages, nkv, hd, page), 7.0, dtype=torch.bfloat16, device=dev()))
    (kp1, vp1), (kp2, vp2) = pools(), pools()
    scale = torch.rsqrt(squares.double().cpu().sum(1, keepdim=True) / K + 1e-5) if prepared else 1.0
    y64 = (x.double().cpu() @ w.double().cpu().T) * scale
    q_want = hip().rope_store(y64.float().bfloat16().to(dev()), table, positions, slots, kp1.permute(0, 2, 1, 3), vp1.permute(0, 3, 1, 2),
                              nh, nkv, hd)
    takes = hip().qkv_rope_sliced_slices(x, w, hd, kp2.permute(0, 2, 1, 3), table)
    assert (takes > 0) == (M >= 33 and not hip().qkv_rope_fuses(x, w, hd, kp2.permute(0, 2, 1, 3))), "where the parts choose this path"
    q = hip().qkv_rope_store_sliced(x, hip().pack_weight_rope(w, hd), slices, table, positions, slots, kp2.permute(0, 2, 1, 3),
                                    vp2.permute(0, 3, 1, 2), nh, nkv, hd, eps=1e-5, squares=squares)
    t64 = y64.view(M, nh + 2 * nkv, hd).clone()
    cs = table.double().cpu()[positions.cpu().long()]
    c, sn = cs[:, None, :hd // 2], cs[:, None, hd // 2:]
    a, b = t64[:, :nh + nkv, :hd // 2].clone(), t64[:, :nh + nkv, hd // 2:].clone()
    t64[:, :nh + nkv, :hd // 2], t64[:, :nh + nkv, hd // 2:] = a * c - b * sn, b * c + a * sn
    live = (slots >= 0).cpu()
    pg, off = (slots.cpu().long() // page)[live], (slots.cpu().long() % page)[live]
    def written(kp, vp):
        return kp.double().cpu()[pg, :, off, :], vp.double().cpu()[pg, :, :, off]
    (k_one, v_one), (k_seq, v_seq) = written(kp2, vp2), written(kp1, vp1)
    for name, one, seq, truth in (("q", q.double().cpu(), q_want.double().cpu(), t64[:, :nh]),
                                  ("k", k_one, k_seq, t64[live][:, nh:nh + nkv]), ("v", v_one, v_seq, t64[live][:, nh + nkv:])):
        e_one, e_seq = (one - truth).abs(), (seq - truth).abs()
        assert float(e_seq.max()) <= 3e-2 * max(1.0, float(truth.abs().max())), f"{name}: the separate kernels are off"
        assert float(e_one.max()) <= 1.25 * float(e_seq.max()) + 1e-3, f"{name}: worst error {float(e_one.max())} vs {float(e_seq.max())}"
        assert float(e_one.pow(2).mean().sqrt()) <= 1.1 * float(e_seq.pow(2).mean().sqrt()) + 1e-4, f"{name}: mean error"
    assert torch.equal(kp2 == 7.0, kp1 == 7.0) and torch.equal(vp2 == 7.0, vp1 == 7.0), "the same places are written"
    q_only = hip().qkv_rope_store_sliced(x, hip().pack_weight_rope(w, hd), slices, table, positions, None, None, None, nh, nkv, hd,
                                         eps=1e-5, squares=squares)
    assert torch.equal(q_only, q)
    alone = hip().qkv_rope_store_sliced(x[M - 1:].contiguous(), hip().pack_weight_rope(w, hd), slices, table, positions[M - 1:].contiguous(),
                                        None, None, None, nh, nkv, hd, eps=1e-5, squares=None if squares is None else squares[M - 1:].contiguous())
    assert torch.equal(alone[0], q[M - 1]), "a row's result does not depend on the rows beside it"


def test_fused_projection_refuses_what_it_cannot_serve():
    x = torch.zeros(65, 256, dtype=torch.bfloat16, device=dev())
    w = torch.zeros(3 * 64, 256, dtype=torch.bfloat16, device=dev())
    assert hip().qkv_rope_fuses(x[:64], w, 64, None) and not hip().qkv_rope_fuses(x, w, 64, None), "65 rows"
    assert not hip().qkv_rope_fuses(x[:17], w, 64, None, norm=True), "17 rows with the norm"
    assert not hip().qkv_rope_fuses(torch.zeros(17, 2304, dtype=torch.bfloat16, device=dev()), w, 64, None), "17 rows over more than 2048"
    assert not hip().qkv_rope_fuses(x[:4], w, 48, None), "head_dim 48"
    assert not hip().qkv_rope_fuses(torch.zeros(4, 4352, dtype=torch.bfloat16, device=dev()), w, 64, None), "K beyond 4096"
    assert not hip().qkv_rope_fuses(torch.zeros(4, 2304, dtype=torch.bfloat16, device=dev()), w, 64, None, norm=True), \
        "K beyond 2048 with the norm"
    with pytest.raises(hip().KernelError, match="qkv_rope_store takes"):
        hip().qkv_rope_store(x, w, None, torch.zeros(65, dtype=torch.int32, device=dev()), None, None, None, 1, 1, 64)


@pytest.mark.parametrize("heads,kv,hd,page", [(32, 8, 64, 256), (8, 2, 128, 64), (3, 1, 32, 24)])
def test_split_key_decode_attention_over_a_long_context(heads, kv, hd, page):
    """Several thousand keys: many chunks per token, several 32-key steps per wave, the plans
    that `decode_plan` picks for long contexts, and one key far back made to dominate."""
    dtype = torch.bfloat16
    n = 5000
    g = gen(hd + page)
    q = (torch.randn(4, heads, hd, generator=g) * 0.5).to(dtype)
    k, v = (torch.randn(n, kv, hd, generator=g) * 0.5).to(dtype), torch.randn(n, kv, hd, generator=g).to(dtype)
    k[37] = 0
    k[37, :, 3] = 30.0
    q[3] = 0
    q[3, :, 3] = 30.0                                # its score with key 37 stands out by far
    pages = -(-n // page)
    table = torch.randperm(pages, generator=g).tolist()
    kc, vc = engine_layout(k, v, table, page, pages, dtype)
    rows = [4999, 2047, 1024, 4100]                  # positions of the four queries
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev())
    want = torch.stack([P.causal_attention(torch.cat([torch.zeros(p, heads, hd, dtype=torch.float64), q[i:i + 1].double()]),
                                           k[:p + 1].double(), v[:p + 1].double())[-1] for i, p in enumerate(rows)])
    waves = hip().decode_waves(hd)
    plans = [(32 * waves, waves), (128 * waves, waves), (1024, 4), hip().decode_plan(4, kv, heads // kv, hd, pages * page)]
    for chunk, w in plans:
        out = hip().paged_attention_decode(q.to(dev()), kc, vc, i32([table]), i32([0] * 4), i32(rows), hd ** -0.5,
                                           chunk=chunk, waves=w)
        torch.testing.assert_close(out.double().cpu(), want, **tol(dtype), msg=lambda m: f"chunk {chunk}, {w} waves: {m}")
    for h in range(heads):
        torch.testing.assert_close(out[3, h].float().cpu(), v[37, h // (heads // kv)].float(), rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("heads,kv,hd,page,row_tiles", [(8, 2, 64, 64, 4), (4, 1, 128, 256, 2), (6, 6, 32, 16, 1)])
def test_matrix_core_prefill_attention_over_a_long_prompt(heads, kv, hd, page, row_tiles):
    """A portion of 1,200 tokens over a cached prefix of 333: dozens of 32-key steps per tile, most
    of them inside every row's range (the loop without masks), the steps before a window's start and
    around the rows' own positions in the masked loops, long tiles first."""
    dtype = torch.bfloat16
    g = gen(hd + 11 * row_tiles)
    n, fed = 1533, 1200
    q = (torch.randn(n, heads, hd, generator=g) * 0.5).to(dtype)
    k, v = (torch.randn(n, kv, hd, generator=g) * 0.5).to(dtype), torch.randn(n, kv, hd, generator=g).to(dtype)
    pages = -(-n // page)
    table = torch.randperm(pages, generator=g).tolist()
    kc, vc = engine_layout(k, v, table, page, pages, dtype)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev())
    per_tile = row_tiles * hip().PREFILL_WAVES * (16 // (heads // kv))
    flat = hip().attention_tiles([0, fed], [n - fed], per_tile)
    positions = list(range(n - fed, n))
    for window in (0, 200):
        out = hip().paged_attention_prefill(q[n - fed:].to(dev()), kc, vc, i32([table]), i32([0] * fed), i32(positions),
                                            i32(flat).view(-1, 2), hd ** -0.5, window=window, tile_tokens=per_tile)
        want = P.causal_attention(q.double(), k.double(), v.double(), window=window)[n - fed:]
        torch.testing.assert_close(out.double().cpu(), want, **tol(dtype), msg=lambda m: f"window {window}: {m}")


@pytest.mark.parametrize("heads,kv,hd,page,row_tiles", [(8, 2, 64, 64, 1), (4, 1, 128, 256, 2), (6, 6, 32, 16, 4),
                                                       (14, 2, 96, 24, 1)])
@pytest.mark.parametrize("splits,chunk", [(2, 1024), (5, 288), (7, 224), (3, 96), (64, 32)])
def test_matrix_core_prefill_attention_with_the_keys_cut_into_chunks(heads, kv, hd, page, row_tiles, splits, chunk):
    """Two one-token requests that are left alone, then a portion of 90 tokens over a cached prefix
    of 1,357 and one of 41 tokens over 610, their keys walked in chunks: chunks that end inside the
    cached prefix, inside the portion (where the causal masks are), chunks that lie wholly before a
    window's start, chunks that a request does not reach, and chunks that together fall short of the
    context (the last one takes the rest). One key far back carries most of one row's weight, so a
    chunk that is dropped or weighted wrongly shows."""
    dtype = torch.bfloat16
    g = gen(hd + 7 * splits)
    lens, fed = [50, 20, 1447, 651], [1, 1, 90, 41]
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev())
    pages_each = [-(-n // page) for n in lens]
    order = torch.randperm(sum(pages_each), generator=g).tolist()
    kp = torch.randn(len(order), kv, page, hd, generator=g).to(dtype)
    vp = torch.randn(len(order), kv, hd, page, generator=g).to(dtype)
    qs, ks, vs, tables = [], [], [], []
    for n, pe in zip(lens, pages_each):
        table, order = order[:pe], order[pe:]
        q = (torch.randn(n, heads, hd, generator=g) * 0.5).to(dtype)
        k, v = (torch.randn(n, kv, hd, generator=g) * 0.5).to(dtype), torch.randn(n, kv, hd, generator=g).to(dtype)
        if n > 1000:
            k[3], q[n - 5] = k[3] * 6, q[n - 5].abs() * k[3].sign().repeat_interleave(heads // kv, 0)  # row n - 5 looks at key 3
        for p_ in range(n):
            kp[table[p_ // page], :, p_ % page] = k[p_]
            vp[table[p_ // page], :, :, p_ % page] = v[p_]
        qs.append(q), ks.append(k), vs.append(v), tables.append(table + [0] * (max(pages_each) - pe))
    kc, vc = kp.to(dev()).permute(0, 2, 1, 3), vp.to(dev()).permute(0, 3, 1, 2)
    q_step = torch.cat([qs[i][lens[i] - fed[i]:] for i in range(4)]).to(dev())
    seq_of = sum(([i] * fed[i] for i in range(4)), [])
    positions = sum((list(range(lens[i] - fed[i], lens[i])) for i in range(4)), [])
    cu = [0, 1, 2, 92, 133]
    per_tile = row_tiles * hip().PREFILL_WAVES * (16 // (heads // kv))
    flat = hip().attention_tiles(cu, [lens[i] - fed[i] for i in range(4)], per_tile, 2)
    for window in (0, 333):
        out = torch.full_like(q_step, 7.0)
        hip().paged_attention_prefill(q_step, kc, vc, i32(tables), i32(seq_of), i32(positions), i32(flat).view(-1, 2),
                                      hd ** -0.5, window=window, tile_tokens=per_tile, out=out, num_splits=splits,
                                      chunk=chunk, first_token=2)
        assert out[:2].eq(7.0).all(), "the tokens before first_token belong to another kernel"
        want = torch.cat([P.causal_attention(qs[i].double(), ks[i].double(), vs[i].double(), window=window)[lens[i] - fed[i]:]
                          for i in (2, 3)])
        torch.testing.assert_close(out[2:].double().cpu(), want, **tol(dtype), msg=lambda m: f"window {window}: {m}")
    with pytest.raises(hip().KernelError, match="multiple of 32"):
        hip().paged_attention_prefill(q_step, kc, vc, i32(tables), i32(seq_of), i32(positions), i32(flat).view(-1, 2),
                                      hd ** -0.5, tile_tokens=per_tile, num_splits=2, chunk=100, first_token=2)


@pytest.mark.parametrize("m", [1, 8, 16, 23])
@pytest.mark.parametrize("n,k", [(3072, 2048), (16384, 2048), (992, 512), (130, 3072), (64, 4096), (2048, 8192)])
def test_weight_streaming_gemm_reads_the_packed_copy_to_the_same_result(m, n, k):
    """`pack_weight` lays the matrix out in the kernel's reading order; every form of the kernel must
    give bit for bit what it gives from the matrix itself (a width that is no multiple of 16 ends in
    a tile padded with zeros)."""
    g = gen(m + n + k)
    w = (torch.randn(n, k, generator=g) * 0.05).bfloat16().to(dev())
    x = torch.randn(m, k, generator=g).bfloat16().to(dev())
    p = hip().pack_weight(w)
    assert p.shape == (-(-n // 16), k // 32, 64, 8)
    assert torch.equal(p[1, 2, 5 + 16 * 3], w[16 + 5, 64 + 24:64 + 32]), "lane r + 16 g: row 16 tile + r, k = 32 step + 8 g .."
    assert torch.equal(hip().gemm_skinny(x, w, packed=p)[0], hip().gemm_skinny(x, w)[0])
    assert torch.equal(hip().gemm_skinny(x, w, torch.float32, packed=p)[0], hip().gemm_skinny(x, w, torch.float32)[0])
    res = torch.randn(m, k, generator=g).bfloat16().to(dev())
    nw = (1 + 0.1 * torch.randn(k, generator=g)).bfloat16().to(dev())
    for norm in (False, True):
        for glu in (False, True):
            if not (norm or glu) or (glu and n % 32) or not hip().skinny_fuses(m, k, norm, glu):
                continue
            kw = dict(residual=res, norm_weight=nw, eps=1e-5) if norm else {}
            a, b = hip().gemm_skinny(x, w, glu=glu, packed=p, **kw), hip().gemm_skinny(x, w, glu=glu, **kw)
            assert torch.equal(a[0], b[0]) and (not norm or torch.equal(a[1], b[1]))
    with pytest.raises(hip().KernelError, match="packed copy"):
        hip().gemm_skinny(x, w, packed=p[1:])


@pytest.mark.parametrize("m,n,k", [(1, 2048, 2048), (8, 2048, 8192), (5, 3072, 3072), (8, 4096, 14336), (3, 44, 256),
                                   (8, 2048, 1024), (7, 8, 512), (2, 1000, 4096), (8, 24, 16384)])
def test_eight_row_form_of_the_weight_streaming_gemm(m, n, k):
    """The form for at most 8 rows of x (a matrix instruction multiplies 8 rows of W by 8 of x over two
    halves of 64 k; only the diagonal blocks of its result count): against 64-bit, in both output
    types, from the matrix and from its packed copy bit for bit, a single row as the same row among
    eight, and a width that is no multiple of 8. The matrix has one large entry per row in the upper
    half of a wave's k, which a block taken from off the diagonal would miss or count twice."""
    g = gen(m * 3 + n + k)
    w = (torch.randn(n, k, generator=g) * 0.05)
    steps = hip().skinny8_steps(k)
    assert steps and hip().skinny8_takes(min(m, 4), n, k) and hip().skinny8_takes(m, min(n, 2048), k)
    for row in range(n):
        w[row, (row * 37) % (32 * steps) + 32 * steps] = 3.0 + row % 5           # in the second half of wave 0's k
    w = w.bfloat16().to(dev())
    x = torch.randn(8, k, generator=g).bfloat16().to(dev())
    want = x[:m].double().cpu() @ w.double().cpu().T
    out = hip().gemm_skinny8(x[:m].contiguous(), w)
    assert out.dtype == torch.bfloat16 and out.shape == (m, n)
    torch.testing.assert_close(out.double().cpu(), want, rtol=1e-2, atol=1e-2 * float(want.abs().max()))
    f32 = hip().gemm_skinny8(x[:m].contiguous(), w, torch.float32)
    torch.testing.assert_close(f32.double().cpu(), want, rtol=1e-4, atol=1e-4 * float(want.abs().max()))
    alone = hip().gemm_skinny8(x[m - 1:m].contiguous(), w, torch.float32)
    assert torch.equal(alone[0], f32[m - 1]), "a row's sums do not depend on the rows beside it"
    if n % 8 == 0:
        p = hip().pack_weight8(w)
        assert p.shape == (n // 8, k // (64 * steps), steps, 64, 8)
        assert torch.equal(p[0, 0, 1, 3 + 8 + 16 * 2], w[3, 32 * steps + 32 + 16:32 * steps + 32 + 24]), \
            "lane r + 16 g: row r % 8, k = 32 steps (r // 8) + 32 step + 8 g .."
        assert torch.equal(hip().gemm_skinny8(x[:m].contiguous(), w, packed8=p), out)
        assert torch.equal(hip().gemm_skinny8(x[:m].contiguous(), w, torch.float32, packed8=p), f32)
        with pytest.raises(hip().KernelError, match="packed copy"):
            hip().gemm_skinny8(x[:m].contiguous(), w, packed8=p[..., :4])
    from tinyserve_llm_amd.parts.linear import linear, streaming_copy
    if hip().skinny8_takes(m, n, k):
        assert torch.equal(linear(x[:m].contiguous(), w, packed=streaming_copy(w)), out), "the parts' projections take this path"
    with pytest.raises(hip().KernelError):
        hip().gemm_skinny8(torch.cat([x, x])[:9].contiguous(), w)


@pytest.mark.parametrize("m", [1, 3, 8])
@pytest.mark.parametrize("k", [1024, 2048, 4096, 8192])
def test_rows_in_the_order_the_eight_row_form_reads_them(m, k):
    """Up to 8 rows packed lane by lane for the 8-row form: the packing and its inverse, the place of one
    piece spelled out, and the product from packed rows bit for bit the product from the matrix, stored or
    finished into the next norm. The lanes of the rows that are not there are filled with NaN: no row
    that is there may see them."""
    H = hip()
    g = gen(7 * m + k)
    steps = H.skinny8_steps(k)
    x = torch.randn(m, k, generator=g).bfloat16().to(dev())
    px = H.pack_rows8(x, steps)
    assert px.shape == (m, k) and px.data.shape == (k // (64 * steps), steps, 64, 8)
    assert torch.equal(px.rows(), x)
    row, wave, half, step, part = m - 1, k // (64 * steps) - 1, 1, steps - 2, 3
    at = 64 * steps * wave + 32 * steps * half + 32 * step + 8 * part
    assert torch.equal(px.data[wave, step, row + 8 * half + 16 * part], x[row, at:at + 8])
    lanes = px.data.view(-1, steps, 4, 2, 8, 8)
    lanes[:, :, :, :, m:] = float("nan")
    n = 2048
    w = (torch.randn(n, k, generator=g) * 0.05).bfloat16().to(dev())
    assert H.rows8_reader_steps(m, w) == steps
    for packed8 in (None, H.pack_weight8(w)):
        assert torch.equal(H.gemm_skinny8(px, w, packed8=packed8), H.gemm_skinny8(x, w, packed8=packed8))
        assert torch.equal(H.gemm_skinny8(px, w, torch.float32, packed8=packed8), H.gemm_skinny8(x, w, torch.float32, packed8=packed8))
    res = torch.randn(m, n, generator=g).bfloat16().to(dev())
    nw = (1 + 0.1 * torch.randn(n, generator=g)).bfloat16().to(dev())
    a, b = H.gemm_skinny8(px, w, next_norm=(res, nw)), H.gemm_skinny8(x, w, next_norm=(res, nw))
    assert torch.equal(a.summed, b.summed) and torch.equal(a.operand, b.operand) and torch.equal(a.squares, b.squares)
    assert torch.equal(H.linear_bf16(px, w), H.gemm_skinny8(x, w))
    with pytest.raises(H.KernelError, match="steps"):
        H.gemm_skinny8(H.PackedRows8(px.data, m, k, 4 if steps != 4 else 8), w)
    wide = (torch.randn(4096, k, generator=g) * 0.05).bfloat16().to(dev())
    assert H.rows8_reader_steps(m, wide) == steps and H.rows8_reader_steps(9, wide) == 0
    assert torch.equal(H.linear_bf16(px, wide), H.gemm_skinny8(x, wide)), "packed rows go to the 8-row form at any width"


@pytest.mark.parametrize("m", [2, 5, 8])
@pytest.mark.parametrize("inter,k", [(8192, 2048), (1024, 512), (4096, 1024)])
def test_gated_product_handed_on_in_the_eight_row_forms_order(m, inter, k):
    """The gate|up projection of a few rows leaves silu(gate) * up in the order the down projection's kernel
    reads it: the same numbers as the matrix it otherwise leaves, with the norm on the way in, prepared by the
    kernel before, or absent; and through `linear` the two projections give what they give without it."""
    H = hip()
    from tinyserve_llm_amd.parts.linear import DeferredNorm, NormRequest, linear, streaming_copy
    g = gen(m + inter + k)
    gate_up = (torch.randn(2 * inter, k, generator=g) * k ** -0.5).bfloat16().to(dev())
    down = (torch.randn(k, inter, generator=g) * inter ** -0.5).bfloat16().to(dev())
    x = torch.randn(m, k, generator=g).bfloat16().to(dev())
    steps = H.rows8_reader_steps(m, down)
    assert steps == H.skinny8_steps(inter) > 0
    plain = H.gemm_skinny(x, gate_up, glu=True)[0]
    packed = H.gemm_skinny(x, gate_up, glu=True, pack8_steps=steps)[0]
    assert isinstance(packed, H.PackedRows8) and packed.shape == (m, inter) and packed.steps == steps
    assert torch.equal(packed.rows(), plain)
    sq = (x.float() ** 2).sum(1, keepdim=True)
    assert torch.equal(H.gemm_skinny(x, gate_up, glu=True, squares=sq, eps=1e-5, pack8_steps=steps)[0].rows(),
                       H.gemm_skinny(x, gate_up, glu=True, squares=sq, eps=1e-5)[0])
    if H.skinny_fuses(m, k, True, True):
        nw = (1 + 0.1 * torch.randn(k, generator=g)).bfloat16().to(dev())
        assert torch.equal(H.gemm_skinny(x, gate_up, norm_weight=nw, eps=1e-5, glu=True, pack8_steps=steps)[0].rows(),
                           H.gemm_skinny(x, gate_up, norm_weight=nw, eps=1e-5, glu=True)[0])
    with pytest.raises(H.KernelError, match="packed rows"):
        H.gemm_skinny(x, gate_up, pack8_steps=steps)
    # through the parts' projections: handed on packed, and not
    res = torch.randn(m, k, generator=g).bfloat16().to(dev())
    nw2 = (1 + 0.1 * torch.randn(k, generator=g)).bfloat16().to(dev())
    copies = streaming_copy(gate_up), streaming_copy(down)
    handed = linear(x, gate_up, glu=True, packed=copies[0], feeds=down)
    assert isinstance(handed, H.PackedRows8)
    kept = linear(x, gate_up, glu=True, packed=copies[0])
    assert torch.equal(linear(handed, down, packed=copies[1]), linear(kept, down, packed=copies[1]))
    a = linear(handed, down, packed=copies[1], then=NormRequest(nw2, 1e-5, res))
    b = linear(kept, down, packed=copies[1], then=NormRequest(nw2, 1e-5, res))
    assert isinstance(a, DeferredNorm) and a.prepared is not None
    assert torch.equal(a.prepared.summed, b.prepared.summed) and torch.equal(a.prepared.operand, b.prepared.operand)
    # a reader it was not made for gets the matrix
    other = torch.zeros(64, inter, dtype=torch.bfloat16, device=dev())
    assert linear(handed, other).shape == (m, 64)
    assert not isinstance(linear(x[:1], gate_up, glu=True, packed=copies[0], feeds=down), H.PackedRows8), "one row is handed on as it is"


@pytest.mark.parametrize("m", [17, 33, 50, 64, 65, 100, 128])
@pytest.mark.parametrize("n,k", [(8192, 1024), (16384, 2048), (9152, 3072)])
def test_wide_product_for_a_few_dozen_rows(m, n, k):
    """The kernel that shares x among 64 rows of W through LDS, against 64-bit products: plain (bfloat16
    and 32-bit sums) and with the gate; each row's result does not depend on the rows beside it. Up to 64
    rows lie in four blocks of 16 in LDS, up to 128 in eight."""
    g = gen(m + n + k)
    x = torch.randn(m, k, generator=g).bfloat16().to(dev())
    w = (torch.randn(n, k, generator=g) * k ** -0.5).bfloat16().to(dev())
    packed = hip().pack_weight(w)
    want = x.double().cpu() @ w.double().cpu().T
    y32 = hip().gemm_rows64(x, packed, torch.float32)
    torch.testing.assert_close(y32.double().cpu(), want, rtol=1e-4, atol=1e-4 * float(want.abs().max()))
    assert torch.equal(hip().gemm_rows64(x, packed), y32.bfloat16())
    if n % 128 == 0:
        gate = P.silu_mul(want)
        yg = hip().gemm_rows64(x, packed, glu=True)
        assert yg.shape == (m, n // 2)
        torch.testing.assert_close(yg.double().cpu(), gate, rtol=2e-2, atol=2e-2 * float(gate.abs().max()))
    alone = hip().gemm_rows64(x[m - 1:].contiguous(), packed, torch.float32)
    assert torch.equal(alone[0], y32[m - 1])
    assert hip().rows64_takes(max(m, 33), n, k, glu=True) and not hip().rows64_takes(40, n, k + 512)
    assert hip().rows64_takes(64, n, k) and not hip().rows64_takes(65, n, k), "a plain product of more than 64 rows is the library's"
    assert hip().rows64_takes(128, n, k, glu=True) and not hip().rows64_takes(129, n, k, glu=True)
    with pytest.raises(hip().KernelError):
        hip().gemm_rows64(x[:1].expand(129, k).contiguous(), packed)


@pytest.mark.parametrize("m", [5, 17, 40, 64, 77, 128])
@pytest.mark.parametrize("n,k,slices", [(2048, 2048, 4), (2048, 8192, 8), (3072, 3072, 6), (192, 1536, 3), (4096, 14336, 4),
                                        (2048, 512, 1)])
def test_narrow_product_in_slices_of_its_reduction(m, n, k, slices):
    """The shared-x kernel with the reduction cut into slices and the kernel that adds the parts, against
    64-bit products: the plain product, and the product finished into the residual sum, the next
    operand and the rows' sums of squares. A row's result does not depend on the rows beside it."""
    g = gen(m + n + k)
    x = torch.randn(m, k, generator=g).bfloat16().to(dev())
    w = (torch.randn(n, k, generator=g) * k ** -0.5).bfloat16().to(dev())
    packed = hip().pack_weight(w)
    want = x.double().cpu() @ w.double().cpu().T
    y = hip().gemm_rows64_sliced(x, packed, slices)
    assert y.dtype == torch.bfloat16 and y.shape == (m, n)
    torch.testing.assert_close(y.double().cpu(), want, rtol=1e-2, atol=1e-2 * float(want.abs().max()))
    assert torch.equal(hip().gemm_rows64_sliced(x[m - 1:].contiguous(), packed, slices)[0], y[m - 1])
    res = torch.randn(m, n, generator=g).bfloat16().to(dev())
    nw = (1 + 0.1 * torch.randn(n, generator=g)).bfloat16().to(dev())
    for residual in (res, None):
        prepared = hip().gemm_rows64_sliced(x, packed, slices, next_norm=(residual, nw))
        t = y.double().cpu() + (0 if residual is None else residual.double().cpu())        # T(y) + res
        assert torch.equal(prepared.summed.cpu(), t.float().bfloat16())
        assert torch.equal(prepared.operand.cpu(), (t.float() * nw.float().cpu()).bfloat16())
        assert prepared.squares.shape == (m, 1), "a row's sum of squares comes whole"
        assert prepared.operand.stride() == (n + hip().OPERAND_ROW_SKEW, 1), "the operand's rows lie a little further apart than they are long"
        torch.testing.assert_close(prepared.squares.double().cpu(), t.pow(2).sum(1, keepdim=True), rtol=1e-5, atol=1e-6)
    with pytest.raises(hip().KernelError):
        hip().gemm_rows64_sliced(x, packed, slices * 2 if k % (1024 * slices) else 5 if (k // 512) % 5 else 7)
    with pytest.raises(hip().KernelError):
        hip().gemm_rows64_sliced(x[:1].expand(129, k).contiguous(), packed, slices)


def test_which_narrow_products_are_cut_into_slices():
    from tinyserve_llm_amd.parts.linear import linear, streaming_copy, NormRequest, DeferredNorm
    assert hip().rows64_slices(64, 2048, 2048) == 4 and hip().rows64_slices(33, 2048, 8192) == 8
    assert hip().rows64_slices(48, 3072, 3072) == 6 and hip().rows64_slices(64, 4096, 14336) == 4
    assert hip().rows64_slices(4, 2048, 8192) == 0 and hip().rows64_slices(129, 2048, 8192) == 0 and hip().rows64_slices(9, 2048, 8192) == 8 and hip().rows64_slices(128, 2048, 8192) == 8
    assert hip().rows64_slices(64, 16384, 2048) == 0, "a wide weight gives every compute unit a workgroup as it is"
    assert hip().rows64_slices(64, 2048, 2304) == 0 and hip().rows64_slices(64, 2000, 2048) == 0
    g = gen(5)
    for m, n, k in ((64, 2048, 8192), (40, 2048, 2048), (24, 2048, 8192), (9, 2048, 8192), (8, 3072, 8192)):
        x = torch.randn(m, k, generator=g).bfloat16().to(dev())
        w = (torch.randn(n, k, generator=g) * k ** -0.5).bfloat16().to(dev())
        copies = streaming_copy(w)
        assert copies is not None and copies.by16 is not None
        y = linear(x, w, packed=copies)
        assert torch.equal(y, hip().gemm_rows64_sliced(x, copies.by16, hip().rows64_slices(m, n, k))), "the parts' projections take this path"
        nw = torch.ones(n, dtype=torch.bfloat16, device=dev())
        d = linear(x, w, packed=copies, then=NormRequest(nw, 1e-5, None))
        assert isinstance(d, DeferredNorm) and d.prepared is not None and torch.equal(d.prepared.summed, y)
        d = linear(x, w, then=NormRequest(nw, 1e-5, None))
        assert d.prepared is None, "without the packed copy the library multiplies and the norm is a kernel of its own"


def test_fused_projection_reads_the_packed_copy_to_the_same_result():
    g = gen(77)
    nh, nkv, hd, K, M, page = 6, 2, 64, 1024, 7, 16
    x = torch.randn(M, K, generator=g).bfloat16().to(dev())
    w = (torch.randn((nh + 2 * nkv) * hd, K, generator=g) * K ** -0.5).bfloat16().to(dev())
    table = torch.randn(64, hd, generator=g).to(dev())
    positions = torch.randint(0, 64, (M,), generator=g, dtype=torch.int32).to(dev())
    slots = torch.randperm(4 * page, generator=g)[:M].to(torch.int32).to(dev())
    outs = []
    for packed in (None, hip().pack_weight_rope(w, hd)):
        kp = torch.zeros(4, nkv, page, hd, dtype=torch.bfloat16, device=dev())
        vp = torch.zeros(4, nkv, hd, page, dtype=torch.bfloat16, device=dev())
        q, _ = hip().qkv_rope_store(x, w, table, positions, slots, kp.permute(0, 2, 1, 3), vp.permute(0, 3, 1, 2),
                                    nh, nkv, hd, packed=packed)
        outs.append((q, kp, vp))
    assert all(torch.equal(a, b) for a, b in zip(*outs))


@pytest.mark.parametrize("heads,kv,hd,chunk,waves,window", [(32, 8, 64, 256, 8, 0), (32, 8, 64, 128, 4, 0), (16, 8, 128, 256, 4, 0),
                                                             (8, 2, 32, 128, 4, 300), (16, 4, 96, 512, 4, 0), (24, 8, 64, 128, 4, 700)])
def test_o_projection_adds_up_the_chunks_of_a_split_walk_itself(heads, kv, hd, chunk, waves, window):
    """The decode kernel told to leave its chunks' parts uncombined, and the 8-row form that makes its x
    from them on the way in (one token): bit for bit what the combining kernel and the 8-row form give one
    after the other, with and without finishing into the next norm, and what the combining kernel gives
    from the parts is what the decode kernel gives when it combines itself. Contexts that end inside
    the first chunk, at a chunk's edge and in the last chunk; a window that hides the first chunks."""
    dtype = torch.bfloat16
    n, page = 2000, 32
    g = gen(heads + hd + chunk)
    k, v = torch.randn(n, kv, hd, generator=g).to(dtype), torch.randn(n, kv, hd, generator=g).to(dtype)
    pages = -(-n // page)
    table = list(range(pages - 1, -1, -1))
    kc, vc = engine_layout(k, v, table, page, pages, dtype)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev())
    K = heads * hd
    w = (torch.randn(520, K, generator=g) * 0.05).to(dtype).to(dev())
    nw = (1 + 0.1 * torch.randn(520, generator=g)).to(dtype).to(dev())
    for pos in (5, chunk - 1, chunk, chunk + 1, 1000, 1999):
        q = torch.randn(1, heads, hd, generator=g).to(dtype).to(dev())
        res = torch.randn(1, 520, generator=g).to(dtype).to(dev())
        args = (q, kc, vc, i32([table]), i32([0]), i32([pos]), hd ** -0.5, window)
        whole = hip().paged_attention_decode(*args, chunk=chunk, waves=waves)
        split = hip().paged_attention_decode(*args, chunk=chunk, waves=waves, leave_split=True)
        if -(-n // chunk) > hip().SPLIT_ATTENTION_MAX_CHUNKS:
            assert isinstance(split, torch.Tensor) and torch.equal(split, whole), "too many chunks: combined as ever"
            continue
        assert isinstance(split, hip().SplitAttention) and split.shape == (1, K)
        x = split.combined()
        assert torch.equal(x.view(1, heads, hd), whole)
        assert hip().split_attention_fuses(1, w) == (K <= 2048)
        if K > 2048:
            with pytest.raises(hip().KernelError, match="parts"):
                hip().gemm_skinny8(split, w)
            continue
        assert torch.equal(hip().gemm_skinny8(split, w), hip().gemm_skinny8(x, w))
        assert torch.equal(hip().gemm_skinny8(split, w, packed8=hip().pack_weight8(w)), hip().gemm_skinny8(x, w))
        for residual in (res, None):
            a, b = hip().gemm_skinny8(split, w, next_norm=(residual, nw)), hip().gemm_skinny8(x, w, next_norm=(residual, nw))
            assert torch.equal(a.summed, b.summed) and torch.equal(a.operand, b.operand) and torch.equal(a.squares, b.squares)
    assert not hip().split_attention_fuses(2, w)
