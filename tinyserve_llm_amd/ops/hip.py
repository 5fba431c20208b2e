"""Python side of the HIP kernels: loads the library, checks every operand on the host, launches.

Every function takes torch tensors that live on the GPU and launches on torch's current stream.
There is no CPU path: a call with a CPU tensor, or without the library, raises. Operand shapes,
strides and storage types are checked here, before a launch, because a kernel that reads out of
bounds takes the GPU down with it.
"""

from __future__ import annotations

import contextlib
import ctypes
import threading

import torch

from tinyserve_llm_amd.csrc import build as _build

_lib = None
_lock = threading.Lock()

_DTYPE_CODE = {torch.float32: 0, torch.bfloat16: 1}
_ERRORS = {1: "unsupported storage type", 2: "unsupported shape or stride", 3: "the kernel launch failed",
           4: "more than the entry point's fixed workspace holds"}


class KernelError(RuntimeError):
    pass


def library() -> ctypes.CDLL:
    """The kernel library; built on first use if no current build exists. Never a fallback."""
    global _lib
    if _lib is None:
        with _lock:
            if _lib is None:
                path = _build.find_current() or _build.build(force=True)
                lib = ctypes.CDLL(path)
                _declare(lib)
                _lib = lib
    return _lib


def _declare(lib: ctypes.CDLL) -> None:
    p, i, i64, f, u64 = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_float, ctypes.c_uint64
    sig = {
        "ts_embedding": [p, p, p, i, i, i, p],
        "ts_rmsnorm": [p, p, p, p, p, p, i, i, f, i, i, p],
        "ts_rope_store": [p, p, p, p, p, p, p, i, i, i, i, i, i, i, i64, i64, i64, i64, i64, i64, i64, i, p],
        "ts_silu_mul": [p, p, i, i, i, p],
        "ts_copy_slots": [p, i64, i64, i64, i, i, p],
        "ts_paged_attention_wave": [p, p, p, p, p, p, p, i, i, i, i, i, i64, i64, i64, i64, i64, i64, i64, i, f, i, i, i, p],
        "ts_paged_attention_decode": [p, p, p, p, p, p, p, p, p, i, i, i, i, i, i64, i64, i64, i64, i64, i64, i, i, i, i, f,
                                      i, i, i, p],
        "ts_attention_combine": [p, p, p, p, i, i, i, i, i, i, p],
        "ts_gemm_exact": [p, p, p, i, i, i, i64, i64, i64, i, i, p],
        "ts_sample": [p, p, p, p, p, p, u64, i, i, i64, p],
        "ts_sample_static": [p, p, p, p, u64, i, i, i64, p],
        "ts_sample_rows": [p, p, p, p, p, p, p, u64, i, i, i64, p],
        "ts_feed_tokens": [p, p, p, i, i, p],
        "ts_gemm_library_bf16": [p, p, p, i, i, i, i64, i64, i64, i, i, p, ctypes.c_size_t, p],
        "ts_gemm_tiled_bf16": [p, p, p, i, i, i, i64, i64, i64, i, i, p],
        "ts_gemm_library_init": [],
        "ts_gemm_library_timing": [i],
        "ts_gemm_library_choices": [p, i],
        "ts_paged_attention_prefill": [p, p, p, p, p, p, p, p, i, i, i, i, i, i, i, i64, i64, i64, i64, i64, i64, i, f, i, i, i, i, i, p, p, i, p],
        "ts_gemm_skinny_bf16": [p, p, p, p, p, p, i, i, i, i64, i64, i64, f, i, i, i, i, p, i, p, p, p, p, p, i, p],
        "ts_gemm_skinny8_bf16": [p, p, p, i, i, i, i64, i64, i64, i, i, p, p, p, p, p, i, p, p, p, i, i, i, i, p],
        "ts_gemm_rows64_bf16": [p, p, p, i, i, i, i64, i64, i, i, p, i, f, p],
        "ts_gemm_rows64_sliced_bf16": [p, p, p, p, i, i, i, i64, i, p, p, p, p, p, i64, p],
        "ts_gemm_rows64_sliced_rope_bf16": [p, p, p, p, i, i, i64, i, p, i, f, p, p, p, p, p, i, i, i, i, i, i64, i64, i64, i64, i64,
                                            i64, i64, p],
        "ts_skinny_tiles": [i, i, i],
        "ts_peak_read": [p, ctypes.c_size_t, p, i, p],
        "ts_peak_mfma": [p, i, i, p],
        "ts_gemm_skinny_rope_bf16": [p, p, p, p, p, p, i, i, i64, i64, f, i, i, p, p, p, p, p, i, i, i, i, i, i64, i64, i64,
                                     i64, i64, i64, i64, p, i, p],
    }
    for name, args in sig.items():
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = ctypes.c_int


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    """The current stream's handle (the short way where torch has it: a launch asks for it every time)."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _ptr(t: torch.Tensor | None) -> int | None:
    return None if t is None else t.data_ptr()


def _code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise KernelError(f"kernels exist for float32 and bfloat16, not {dtype}") from None


def _need(cond: bool, msg) -> None:
    """Raises `KernelError(msg)` unless `cond`. A message that formats anything comes as a function
    that makes it: the checks run at every call of every kernel, and a step of a short prompt is
    bound by what the host does between launches."""
    if not cond:
        raise KernelError(msg() if callable(msg) else msg)


def _gpu(*tensors: torch.Tensor | None) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise KernelError("the HIP kernels take GPU tensors only; there is no CPU path")


def _run(name: str, rc: int) -> None:
    if rc:
        raise KernelError(f"{name}: {_ERRORS.get(rc, rc)}")


# ---------------------------------------------------------------------------------------------

def embedding(table: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
    """out[t] = table[ids[t]]; ids int32 and already checked against the vocabulary on the host."""
    _gpu(table, ids)
    _need(table.dim() == 2 and table.is_contiguous(), "embedding table must be contiguous [vocab, hidden]")
    _need(ids.dtype == torch.int32 and ids.dim() == 1 and ids.is_contiguous(), "ids must be int32 [tokens]")
    out = torch.empty((ids.shape[0], table.shape[1]), dtype=table.dtype, device=table.device)
    _run("embedding", library().ts_embedding(_ptr(out), _ptr(table), _ptr(ids), ids.shape[0], table.shape[1],
                                             _code(table.dtype), _stream()))
    return out


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, residual: torch.Tensor | None = None,
            rows: torch.Tensor | None = None, want_residual: bool = True
            ) -> tuple[torch.Tensor, torch.Tensor | None]:
    """(norm(x + residual) * weight, x + residual). With `rows` (int32) only those rows are
    normalised, in that order, and no residual is returned."""
    _gpu(x, weight, residual, rows)
    _need(x.dim() == 2 and x.is_contiguous(), "rmsnorm input must be contiguous [rows, hidden]")
    hidden = x.shape[1]
    _need(weight.shape == (hidden,) and weight.is_contiguous(), "rmsnorm weight must be [hidden]")
    if residual is not None:
        _need(residual.shape == x.shape and residual.dtype == x.dtype and residual.is_contiguous(),
              "residual must match the input")
    n = x.shape[0]
    if rows is not None:
        _need(rows.dtype == torch.int32 and rows.dim() == 1 and rows.is_contiguous(), "rows must be int32")
        n = rows.shape[0]
    out = torch.empty((n, hidden), dtype=x.dtype, device=x.device)
    res_out = None
    if rows is None and want_residual:
        res_out = x if residual is None else torch.empty_like(x)
    write_res = res_out if (residual is not None and res_out is not None) else None
    _run("rmsnorm", library().ts_rmsnorm(_ptr(out), _ptr(write_res), _ptr(x), _ptr(residual), _ptr(weight),
                                         _ptr(rows), n, hidden, float(eps), _code(x.dtype), _code(weight.dtype),
                                         _stream()))
    return out, res_out


def rope_store(qkv: torch.Tensor, cos_sin: torch.Tensor | None, positions: torch.Tensor,
               slots: torch.Tensor | None, k_cache: torch.Tensor | None, v_cache: torch.Tensor | None,
               num_heads: int, num_kv_heads: int, head_dim: int) -> torch.Tensor:
    """Rotates q and k of `qkv` [tokens, (nh + 2 nkv) hd] by the table rows of `positions`, returns q
    [tokens, nh, hd] and writes rotated k and v to the cache slots. `k_cache`/`v_cache` are one
    layer's view [pages, page_size, nkv, hd] (may be strided over pages and slots); None = no write.
    `cos_sin` None = no rotation; a table narrower than head_dim ([positions, rot], rot even) turns
    the first rot dimensions of every head (j with j + rot / 2) and lets the others pass."""
    _gpu(qkv, cos_sin, positions, slots, k_cache, v_cache)
    T = qkv.shape[0]
    row = (num_heads + 2 * num_kv_heads) * head_dim
    _need(qkv.dim() == 2 and qkv.shape[1] == row and qkv.is_contiguous(), lambda: f"qkv must be contiguous [tokens, {row}]")
    _need(positions.dtype == torch.int32 and positions.shape == (T,) and positions.is_contiguous(),
          "positions must be int32 [tokens]")
    rot = head_dim
    if cos_sin is not None:
        _need(cos_sin.dtype == torch.float32 and cos_sin.dim() == 2 and cos_sin.is_contiguous()
              and 2 <= cos_sin.shape[1] <= head_dim and cos_sin.shape[1] % 2 == 0,
              lambda: f"the rotation table must be float32 [positions, an even width up to head_dim {head_dim}]")
        rot = cos_sin.shape[1]
    page_size, kst, vst = 1, (0, 0, 0), (0, 0, 0, 0)
    if k_cache is not None:
        _need(v_cache is not None and slots is not None, "a cache write needs k, v and the slots")
        _need(slots.dtype == torch.int32 and slots.shape == (T,) and slots.is_contiguous(), "slots must be int32 [tokens]")
        _check_cache(k_cache, v_cache, qkv.dtype, num_kv_heads, head_dim)
        page_size, kst, vst = k_cache.shape[1], k_cache.stride()[:3], v_cache.stride()
    q = torch.empty((T, num_heads, head_dim), dtype=qkv.dtype, device=qkv.device)
    _run("rope_store", library().ts_rope_store(
        _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(qkv), _ptr(cos_sin), _ptr(positions), _ptr(slots), T, num_heads,
        num_kv_heads, head_dim, rot, int(cos_sin is not None), page_size, *kst, *vst, _code(qkv.dtype), _stream()))
    return q


def _check_cache(k_cache: torch.Tensor, v_cache: torch.Tensor, dtype: torch.dtype, nkv: int, hd: int) -> None:
    """A layer's caches are addressed as [pages, page_size, kv_heads, head_dim]. Keys: head_dim
    dense, the other three strided in any order. Values: all four strided in any order (the
    engine's pools keep a head's slots of one dimension together, i.e. pages transposed)."""
    for name, c in (("key", k_cache), ("value", v_cache)):
        _need(c.dim() == 4 and c.shape[2] == nkv and c.shape[3] == hd,
              lambda: f"{name} cache view must be [pages, page_size, {nkv}, {hd}], got {tuple(c.shape)}")
        _need(c.dtype == dtype, "cache and activations differ in storage type")
        # no two elements may overlap: sort the strides and check each spans the dimensions below it
        span = 1
        for stride, size in sorted(zip(c.stride(), c.shape)):
            if size > 1:
                _need(stride >= span, lambda: f"{name} cache elements overlap")
                span = stride * size
    _need(k_cache.shape == v_cache.shape, "key and value caches differ in shape")
    _need(k_cache.stride(3) == 1, "head_dim must be contiguous in the key cache")
    itemsize = k_cache.element_size()
    _need(all((k_cache.stride(i) * itemsize) % 16 == 0 for i in range(3)) and k_cache.data_ptr() % 16 == 0,
          "key rows must be 16-byte aligned")


def _page_run(pages_per_entry: int) -> int:
    """log2 of the pool pages that one entry of a block table names (a power of two)."""
    _need(pages_per_entry >= 1 and pages_per_entry & (pages_per_entry - 1) == 0 and pages_per_entry <= 65536,
          lambda: f"an entry of a block table names a power of two of pages, not {pages_per_entry}")
    return pages_per_entry.bit_length() - 1


def paged_attention_wave(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                         block_tables: torch.Tensor, seq_of_token: torch.Tensor, positions: torch.Tensor,
                         scale: float, window: int = 0, pages_per_entry: int = 1) -> torch.Tensor:
    """Attention of each token (at its position, causal, optionally windowed) over the cache
    pages that its request's row of `block_tables` names. `pages_per_entry` (a power of two): an
    entry e of a block table stands for that many consecutive pages of the cache, e * n + j (the
    pools may be cut into shorter pages than the tables count in)."""
    _gpu(q, k_cache, v_cache, block_tables, seq_of_token, positions)
    _need(q.dim() == 3 and q.is_contiguous(), "q must be contiguous [tokens, heads, head_dim]")
    T, nh, hd = q.shape
    nkv = k_cache.shape[2]
    _check_cache(k_cache, v_cache, q.dtype, nkv, hd)
    _need(hd % 16 == 0 and hd <= 256, lambda: f"head_dim {hd} is not a multiple of 16 up to 256")
    _need(nh % nkv == 0, lambda: f"{nh} heads do not divide into {nkv} key/value heads")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous(),
          "block_tables must be contiguous int32 [requests, pages]")
    for name, t in (("seq_of_token", seq_of_token), ("positions", positions)):
        _need(t.dtype == torch.int32 and t.shape == (T,) and t.is_contiguous(), lambda: f"{name} must be int32 [tokens]")
    out = torch.empty_like(q)
    _run("paged_attention_wave", library().ts_paged_attention_wave(
        _ptr(out), _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(block_tables), _ptr(seq_of_token), _ptr(positions),
        T, nh, nkv, hd, k_cache.shape[1], *k_cache.stride()[:3], *v_cache.stride(),
        block_tables.shape[1], float(scale), int(window), _code(q.dtype), _page_run(pages_per_entry), _stream()))
    return out


MAX_DECODE_SPLITS = 1024     # chunks per token that the combining kernel takes
MAX_DECODE_TOKENS = 65535    # tokens are a grid dimension of the decode kernel
DECODE_HEAD_DIMS = (32, 64, 96, 128)


MAX_DECODE_WAVES = 8


def decode_waves(hd: int, one_step: bool = False) -> int:
    """Most waves of a workgroup of the decode kernel: heads wider than 64 leave the loop over
    several steps registers for 4; the instance with one step per wave has room for 8."""
    return 4 if hd > 64 and not one_step else MAX_DECODE_WAVES


DECODE_ONE_STEP_SPLITS = 18      # up to this many chunks per token a wave takes one 32-key step (the leanest instance)
DECODE_TARGET_WORKGROUPS = 256   # beyond: as many chunks as give every compute unit a workgroup,
DECODE_MAX_CHUNK = 4096          # of at most this many keys
DECODE_FILL = 0.9                # a last round of workgroups should fill this share of the compute units
DECODE_ENOUGH_ROWS = 190         # (token, key/value head) pairs from which a workgroup each, over the whole context, is considered


def decode_plan(num_tokens: int, nkv: int, group: int, hd: int, capacity: int) -> tuple[int, int]:
    """(keys per workgroup, waves per workgroup) of the split-key kernel for a step of `num_tokens`
    one-query tokens over block tables that reach `capacity` positions. Measured over batches of 1
    to 64 and contexts of 2K to 32K at head sizes 64 and 128: where the step has a workgroup per
    (token, key/value head) for every compute unit anyway, a workgroup takes the whole context and
    nothing is combined (chunks of 4,096 keys beyond 16K); short contexts are cut so that a wave
    has a single 32-key step (the instance without a second buffer); longer ones into as many
    chunks as give the chip about one workgroup per compute unit, since the time of the combining
    kernel grows with the number of chunks (head size 128, 8 tokens over 16K keys: 151 µs in
    128-key chunks, 109 µs in 4,096-key chunks). Workgroups should come in full rounds of one per
    compute unit: 48 tokens of 8 heads over 8,192 keys take 332 µs as 384 workgroups that each walk
    the whole context and 289 µs as 768 that walk half of it; so where a workgroup per (token,
    key/value head) would leave the last round under nine tenths full, short contexts take the
    one-step form and longer ones the fewest chunks of equal length that fill their rounds. A sweep
    over batches of 4 to 96 and contexts of 2,304 to 16,384 has the plan within 10 % of the best
    chunk everywhere (it was up to 14 % off at 24 and 48 tokens before)."""
    def fitting(waves: int) -> int:          # the waves' partial results meet in 64 KB of LDS
        while waves > 1 and 4 * (32 * waves + waves * group * hd) > 65536:
            waves //= 2
        return waves
    most, wide = fitting(decode_waves(hd)), fitting(decode_waves(hd, one_step=True))
    one = 32 * wide
    if capacity <= one:
        waves = -(-capacity // 32)
        return 32 * waves, waves
    rows = num_tokens * nkv
    step = 32 * most
    whole = -(-capacity // step) * step if capacity <= 16384 else DECODE_MAX_CHUNK

    def fills(workgroups: int) -> bool:
        """Whether so many workgroups come in rounds of about one per compute unit: 256, 512 or 768
        of them keep the chip busy to the end, 192 or 384 leave a quarter of it idle."""
        rounds = -(-workgroups // DECODE_TARGET_WORKGROUPS)
        return workgroups >= DECODE_FILL * rounds * DECODE_TARGET_WORKGROUPS

    def even(n: int) -> int:                  # the context in n chunks of one length
        return -(-capacity // (n * step)) * step

    def filling(fallback: int) -> int:
        """The longest of those chunks, of at most DECODE_MAX_CHUNK keys, whose workgroups fill their rounds."""
        for n in range(max(2, -(-capacity // DECODE_MAX_CHUNK)), MAX_DECODE_SPLITS + 1):
            if even(n) <= DECODE_MAX_CHUNK and fills(rows * -(-capacity // even(n))):
                return even(n)
        return fallback

    one_step = -(-capacity // one) <= DECODE_ONE_STEP_SPLITS
    if rows >= DECODE_ENOUGH_ROWS:
        if rows < DECODE_TARGET_WORKGROUPS or fills(rows * -(-capacity // whole)) or rows >= 4 * DECODE_TARGET_WORKGROUPS:
            chunk = whole
        elif one_step:
            return one, wide
        else:
            chunk = filling(whole)
    elif one_step:
        return one, wide
    else:
        splits = max(1, DECODE_TARGET_WORKGROUPS // rows)
        chunk = filling(min(max(-(-capacity // (splits * step)) * step, step), DECODE_MAX_CHUNK))
    while -(-capacity // chunk) > MAX_DECODE_SPLITS:
        chunk *= 2
    return chunk, most


def decode_kernel_takes(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor) -> bool:
    """Whether the matrix-core decode kernel serves these operands (else the wave kernel does)."""
    nh, hd = q.shape[1], q.shape[2]
    nkv, page = k_cache.shape[2], k_cache.shape[1]
    return (q.dtype == torch.bfloat16 and hd in DECODE_HEAD_DIMS and nh // nkv <= 16 and (nh // nkv) * hd <= 2048
            and page % 8 == 0 and v_cache.stride(1) == 1
            and all(st % 8 == 0 for st in (*k_cache.stride()[:3], v_cache.stride(0), v_cache.stride(2), v_cache.stride(3)))
            and v_cache.data_ptr() % 16 == 0)


def paged_attention_decode(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_tables: torch.Tensor,
                           seq_of_token: torch.Tensor, positions: torch.Tensor, scale: float, window: int = 0,
                           chunk: int | None = None, waves: int | None = None,
                           out: torch.Tensor | None = None, pages_per_entry: int = 1,
                           leave_split: bool = False) -> "torch.Tensor | SplitAttention":
    """Split-key attention on the matrix cores for tokens that each bring one query (bfloat16,
    values in transposed pages). Every position in `positions` must lie inside the pages its row
    of `block_tables` has (checked by the caller on the host). `out`, if given, receives the result.
    `pages_per_entry`: as for `paged_attention_wave`. `leave_split`: where the keys are walked in
    2 to `SPLIT_ATTENTION_MAX_CHUNKS` chunks, the chunks' parts come back uncombined (a
    `SplitAttention`), for the projection that reads them."""
    _gpu(q, k_cache, v_cache, block_tables, seq_of_token, positions)
    _need(q.dim() == 3 and q.is_contiguous(), "q must be contiguous [tokens, heads, head_dim]")
    T, nh, hd = q.shape
    nkv = k_cache.shape[2]
    _check_cache(k_cache, v_cache, q.dtype, nkv, hd)
    _need(nh % nkv == 0, lambda: f"{nh} heads do not divide into {nkv} key/value heads")
    _need(decode_kernel_takes(q, k_cache, v_cache),
          "the decode kernel takes bfloat16, head_dim 32/64/96/128, groups of up to 16 heads, values in transposed pages")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous(),
          "block_tables must be contiguous int32 [requests, pages]")
    for name, t in (("seq_of_token", seq_of_token), ("positions", positions)):
        _need(t.dtype == torch.int32 and t.shape == (T,) and t.is_contiguous(), lambda: f"{name} must be int32 [tokens]")
    _need(T <= MAX_DECODE_TOKENS, lambda: f"the decode kernel takes up to {MAX_DECODE_TOKENS} tokens a launch")
    capacity = block_tables.shape[1] * pages_per_entry * k_cache.shape[1]
    if chunk is None:
        chunk, waves = decode_plan(T, nkv, nh // nkv, hd, capacity)
    waves = waves or 4
    splits = -(-capacity // chunk)
    _need(1 <= waves <= decode_waves(hd, chunk == 32 * waves) and chunk % (32 * waves) == 0 and splits <= MAX_DECODE_SPLITS,
          lambda: f"chunk {chunk} in {waves} waves over {capacity} positions")
    _need(4 * (32 * waves + waves * (nh // nkv) * hd) <= 65536, lambda: f"{waves} waves of {nh // nkv} heads exceed the LDS of a workgroup")
    part_o = part_ml = None
    if splits > 1:
        part_o = torch.empty((T, nh, splits, hd), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((T, nh, splits, 2), dtype=torch.float32, device=q.device)
    leave_split = leave_split and out is None and 1 < splits <= SPLIT_ATTENTION_MAX_CHUNKS
    out = None if leave_split else _out_like(q, out)
    _run("paged_attention_decode", library().ts_paged_attention_decode(
        _ptr(out), _ptr(part_o), _ptr(part_ml), _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(block_tables),
        _ptr(seq_of_token), _ptr(positions), T, nh, nkv, hd, k_cache.shape[1], *k_cache.stride()[:3],
        v_cache.stride(0), v_cache.stride(2), v_cache.stride(3), block_tables.shape[1], splits, chunk, waves,
        float(scale), int(window), _page_run(pages_per_entry), int(not leave_split), _stream()))
    return SplitAttention(part_o, part_ml, positions, chunk, int(window)) if leave_split else out


SPLIT_ATTENTION_MAX_CHUNKS = 16    # chunks that the 8-row form adds up on its way in
SPLIT_ATTENTION_MAX_K = 2048       # widest attention output it makes that way (a wave's 256 k through its kilobyte of LDS, 8 waves)


class SplitAttention:
    """What the split-key attention kernel leaves when it is told not to combine: `parts` [tokens, heads,
    chunks, head_dim] float32, a chunk's weighted values, and `sums` [tokens, heads, chunks, 2] float32, its
    running maximum (in units of log2) and its sum; `positions` [tokens], `chunk` keys a chunk and `window`
    say which chunks hold keys a token sees. The attention output is sum_s parts_s 2^(m_s - M) / sum_s l_s
    2^(m_s - M): `combined()` makes it with the combining kernel, `gemm_skinny8` makes it on its way in for a
    single token, bit for bit the same. `linear` decides which; nothing else takes it."""

    def __init__(self, parts: torch.Tensor, sums: torch.Tensor, positions: torch.Tensor, chunk: int, window: int) -> None:
        self.parts, self.sums, self.positions, self.chunk, self.window = parts, sums, positions, chunk, window

    @property
    def shape(self) -> tuple[int, int]:
        tokens, heads, _, hd = self.parts.shape
        return (tokens, heads * hd)

    def combined(self) -> torch.Tensor:
        """The attention output [tokens, heads * head_dim] in bfloat16."""
        tokens, heads, chunks, hd = self.parts.shape
        out = torch.empty((tokens, heads * hd), dtype=torch.bfloat16, device=self.parts.device)
        _run("attention_combine", library().ts_attention_combine(
            _ptr(out), _ptr(self.parts), _ptr(self.sums), _ptr(self.positions), tokens, heads, hd, chunks, self.chunk,
            self.window, _stream()))
        return out


def split_attention_fuses(rows: int, weight: torch.Tensor) -> bool:
    """Whether the 8-row form multiplies `weight` by the attention output of `rows` tokens that it adds up from the
    chunks' parts itself: one token (every workgroup of the projection adds up all of it), over a reduction of up
    to 2,048."""
    return (rows == 1 and weight.is_cuda and weight.dtype == torch.bfloat16 and weight.dim() == 2
            and weight.is_contiguous() and weight.data_ptr() % 16 == 0
            and weight.shape[1] % 256 == 0 and weight.shape[1] <= SPLIT_ATTENTION_MAX_K)


def gemm_exact(a: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype | None = None) -> torch.Tensor:
    """a [M, K] · w [N, K]^T with 32-bit multiply-adds in ascending k."""
    _gpu(a, w)
    _need(a.dim() == 2 and w.dim() == 2 and a.shape[1] == w.shape[1], lambda: f"shapes {tuple(a.shape)} x {tuple(w.shape)}^T")
    _need(a.dtype == w.dtype, "activations and weights differ in storage type")
    _need(a.stride(1) == 1 and w.stride(1) == 1, "rows must be contiguous")
    out_dtype = out_dtype or a.dtype
    out = torch.empty((a.shape[0], w.shape[0]), dtype=out_dtype, device=a.device)
    _run("gemm_exact", library().ts_gemm_exact(_ptr(out), _ptr(a), _ptr(w), a.shape[0], w.shape[0], a.shape[1],
                                               a.stride(0), w.stride(0), out.stride(0), _code(a.dtype),
                                               _code(out_dtype), _stream()))
    return out


def silu_mul(gate_up: torch.Tensor) -> torch.Tensor:
    """silu(gate) * up for rows laid out [gate | up]."""
    _gpu(gate_up)
    _need(gate_up.dim() == 2 and gate_up.shape[1] % 2 == 0 and gate_up.is_contiguous(),
          "gate_up must be contiguous [tokens, 2 * intermediate]")
    inter = gate_up.shape[1] // 2
    out = torch.empty((gate_up.shape[0], inter), dtype=gate_up.dtype, device=gate_up.device)
    _run("silu_mul", library().ts_silu_mul(_ptr(out), _ptr(gate_up), gate_up.shape[0], inter, _code(gate_up.dtype),
                                           _stream()))
    return out


def copy_slots(pool: torch.Tensor, src: int, dst: int, num_slots: int, slot_dim: int) -> None:
    """Copies the first `num_slots` slots of page `src` to page `dst` in a contiguous pool whose
    first dimension is the page and whose dimension `slot_dim` is the slot, e.g. keys
    [pages, heads, page_size, head_dim] (slot_dim 2) or transposed values
    [pages, heads, head_dim, page_size] (slot_dim 3)."""
    _gpu(pool)
    _need(pool.is_contiguous() and 1 <= slot_dim < pool.dim(), "pool must be contiguous, pages first")
    _need(pool.element_size() % 2 == 0, "pool elements must be 2 or 4 bytes")
    pages, page_size = pool.shape[0], pool.shape[slot_dim]
    _need(0 <= src < pages and 0 <= dst < pages and src != dst, lambda: f"pages {src}->{dst} outside 0..{pages - 1}")
    _need(0 <= num_slots <= page_size, lambda: f"{num_slots} slots do not fit a page of {page_size}")
    runs = 1
    for n in pool.shape[1:slot_dim]:
        runs *= n
    inner = pool.element_size()
    for n in pool.shape[slot_dim + 1:]:
        inner *= n
    _run("copy_slots", library().ts_copy_slots(_ptr(pool), runs, page_size * inner, num_slots * inner, src, dst,
                                               _stream()))


def feed_tokens(ids: torch.Tensor, prev: torch.Tensor, src: torch.Tensor) -> None:
    """ids[i] = prev[src[i]] where src[i] >= 0 (all int32, on the device): what one step drew becomes
    the next step's input without a trip to the host."""
    _gpu(ids, prev, src)
    _need(all(t.dtype == torch.int32 and t.dim() == 1 and t.is_contiguous() for t in (ids, prev, src))
          and src.shape[0] == ids.shape[0] and prev.shape[0] > 0, "feed_tokens takes int32 vectors, one source per id")
    _run("feed_tokens", library().ts_feed_tokens(_ptr(ids), _ptr(prev), _ptr(src), ids.shape[0], prev.shape[0], _stream()))


def sample(logits: torch.Tensor, temperatures: torch.Tensor, keys: torch.Tensor, seed: int,
           row_of: torch.Tensor | None = None, num_logit_rows_checked: bool = False) -> torch.Tensor:
    """One token per draw from float32 `logits`: argmax where the temperature is 0, else a draw whose
    noise is a function of (seed, keys[draw], vocabulary index) alone. Draw r reads row r, or with
    `row_of` (int32, values the caller has checked to lie inside `logits`) row row_of[r]: the n
    samples of one prompt all read the row of its last position."""
    _gpu(logits, temperatures, keys, row_of)
    _need(logits.dtype == torch.float32 and logits.dim() == 2 and logits.stride(1) == 1, "logits must be float32 [rows, vocab]")
    R = logits.shape[0]
    if row_of is not None:
        _need(num_logit_rows_checked, "the caller checks the rows that the draws read on the host")
        _need(row_of.dtype == torch.int32 and row_of.dim() == 1 and row_of.is_contiguous() and R > 0, "row_of must be int32 [draws]")
        R = row_of.shape[0]
    _need(temperatures.dtype == torch.float32 and temperatures.shape == (R,) and temperatures.is_contiguous(),
          "temperatures must be float32 [draws]")
    _need(keys.dtype == torch.int64 and keys.shape == (R,) and keys.is_contiguous(), "keys must be int64 [draws]")
    out = torch.empty((R,), dtype=torch.int32, device=logits.device)
    work_v = torch.empty((R, 64), dtype=torch.float32, device=logits.device)
    work_i = torch.empty((R, 64), dtype=torch.int32, device=logits.device)
    if row_of is None:
        rc = library().ts_sample(_ptr(out), _ptr(work_v), _ptr(work_i), _ptr(logits), _ptr(temperatures), _ptr(keys),
                                 seed & 0xFFFFFFFFFFFFFFFF, R, logits.shape[1], logits.stride(0), _stream())
    else:
        rc = library().ts_sample_rows(_ptr(out), _ptr(work_v), _ptr(work_i), _ptr(logits), _ptr(row_of), _ptr(temperatures),
                                      _ptr(keys), seed & 0xFFFFFFFFFFFFFFFF, R, logits.shape[1], logits.stride(0), _stream())
    _run("sample", rc)
    return out


# ---- dispatchers ---------------------------------------------------------------------------------

def _out_like(q: torch.Tensor, out: torch.Tensor | None) -> torch.Tensor:
    if out is None:
        return torch.empty_like(q)
    _gpu(out)
    _need(out.shape == q.shape and out.dtype == q.dtype and out.is_contiguous(), "out must match q")
    return out


PREFILL_WAVES = 4            # waves of a workgroup of the prefill kernel; each holds 1, 2 or 4 row tiles
PREFILL_TWO_TILES_WORKGROUPS = 384      # two row tiles per wave while this many workgroups remain (1.5 per compute unit)
PREFILL_FOUR_TILES_WORKGROUPS = 512     # four while this many remain,
PREFILL_FOUR_TILES_HEAD_DIM = 64        # only up to this head size (beyond it the accumulators crowd the registers)
PREFILL_FOUR_TILES_MEAN_KEYS = 4096     # and only where a row walks this many keys on average


def prefill_tile_tokens(num_tokens: int, nkv: int, group: int, head_dim: int, mean_keys: float = 0.0) -> int:
    """Tokens per tile of the prefill kernel. A wave that holds two or four row tiles works on them
    side by side and reads each key once for all of them, which is faster as long as the step still
    makes enough workgroups to fill the chip; four pay only for small heads over long contexts
    (`mean_keys`: the keys a row of the step walks on average). Thresholds from a sweep over steps of
    128 to 8,192 tokens, 0 to 6,144 cached tokens before them, head sizes 64 and 128 and groups of
    3, 4 and 8 heads: e.g. 2,048 tokens over 6,144 cached ones at head size 128 take 484 / 272 / 333 µs
    with 1 / 2 / 4 row tiles per wave, 512 tokens 161 / 181 / 267 µs; 4,096 tokens over 2,048 at
    head size 64 take 246 / 220 / 190 µs."""
    per_wave = PREFILL_WAVES * (16 // group)

    def workgroups(rt: int) -> int:
        return -(-num_tokens // (rt * per_wave)) * nkv

    if (head_dim <= PREFILL_FOUR_TILES_HEAD_DIM and workgroups(4) >= PREFILL_FOUR_TILES_WORKGROUPS
            and mean_keys >= PREFILL_FOUR_TILES_MEAN_KEYS):
        return 4 * per_wave
    if workgroups(2) >= PREFILL_TWO_TILES_WORKGROUPS:
        return 2 * per_wave
    return per_wave


PREFILL_EIGHT_WAVES_MEAN_KEYS = 1536    # a shorter walk than this on average takes workgroups of eight waves,
PREFILL_EIGHT_WAVES_HEAD_DIMS = (64, 128)   # for the head sizes whose registers of a step go round eight waves


def prefill_waves(tile_tokens: int, group: int, head_dim: int, mean_keys: float) -> int:
    """Waves of a workgroup of the prefill kernel for tiles of `tile_tokens` tokens: 4, or 8 where a
    wave of four would hold two row tiles and the walk is short. The longest tiles of a prompt run
    alone at the end, a step after a step; with eight waves a wave holds one row tile and a step takes
    it less time (2,048 tokens from position 0 at head size 64: 48.5 µs against 50.1, head size 128:
    60.6 against 64.6), but every wave reads the step's keys and values out of LDS, which costs more
    than that over long walks (8,192 tokens: 467 µs against 373)."""
    two_a_wave = tile_tokens == 2 * PREFILL_WAVES * (16 // group)
    if two_a_wave and head_dim in PREFILL_EIGHT_WAVES_HEAD_DIMS and 0.0 < mean_keys < PREFILL_EIGHT_WAVES_MEAN_KEYS:
        return 2 * PREFILL_WAVES
    return PREFILL_WAVES


PREFILL_SPLIT_BELOW_WORKGROUPS = 384    # a step whose tiles make fewer workgroups than this may cut its keys into chunks
PREFILL_SPLIT_TARGET_WORKGROUPS = 512   # so that about this many workgroups walk them,
PREFILL_SPLIT_MIN_CHUNK = 512           # each at least this many keys
PREFILL_SPLIT_MIN_CONTEXT = 2048        # if the longest context reaches this


def prefill_splits(workgroups: int, longest: int) -> tuple[int, int]:
    """(number of chunks, keys per chunk) for the prefill kernel's key walk; (1, 0) where it is not
    cut. Few tokens over a long context (a short new turn behind a cached conversation, a small
    portion of a long prompt) make too few tiles to fill the chip and each walks thousands of keys:
    128 tokens over 6,144 cached ones take 153 µs uncut and 42 µs in 8 chunks (heads of 128), 256
    tokens of a single key/value head over 8,000 take 193 µs and 36 µs in 16. `workgroups` is
    tiles times key/value heads, `longest` the longest context of the step's portions (the last chunk
    takes whatever lies beyond the others, so an estimate that is too low costs balance only)."""
    if workgroups >= PREFILL_SPLIT_BELOW_WORKGROUPS or longest < PREFILL_SPLIT_MIN_CONTEXT:
        return 1, 0
    splits = min(-(-PREFILL_SPLIT_TARGET_WORKGROUPS // max(1, workgroups)), longest // PREFILL_SPLIT_MIN_CHUNK, MAX_DECODE_SPLITS)
    if splits < 2:
        return 1, 0
    chunk = -(-longest // (splits * 32)) * 32
    return -(-longest // chunk), chunk


def attention_tiles(cu_seqlens: list[int], starts: list[int], tokens_per_tile: int, first_seq: int = 0) -> list[int]:
    """Tiles of a packed step for the matrix-core prefill kernel: (first token, token count) pairs,
    flattened, for the requests from `first_seq` on. A tile never crosses a request; `starts[s]` is
    the position of request s's first token in the step, and the tiles come in ascending order of
    their last position, which is the number of keys the kernel walks for them."""
    found: list[tuple[int, int, int]] = []
    for s in range(first_seq, len(cu_seqlens) - 1):
        a, b = cu_seqlens[s], cu_seqlens[s + 1]
        for t in range(a, b, tokens_per_tile):
            n = min(tokens_per_tile, b - t)
            found.append((starts[s] + t - a + n, t, n))
    found.sort()
    flat: list[int] = []
    for _, t, n in found:
        flat += (t, n)
    return flat


def paged_attention_prefill(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_tables: torch.Tensor,
                            seq_of_token: torch.Tensor, positions: torch.Tensor, tiles: torch.Tensor, scale: float,
                            window: int = 0, tile_tokens: int | None = None, out: torch.Tensor | None = None,
                            num_splits: int = 1, chunk: int = 0, first_token: int = 0, waves: int = PREFILL_WAVES,
                            pages_per_entry: int = 1) -> torch.Tensor:
    """Attention of a packed step on the matrix cores (bfloat16, values in transposed pages).
    `tiles` int32 [num_tiles, 2] lists (first token, token count <= tile_tokens) per workgroup,
    every tile inside one request and inside the step (the caller built the list from the step's
    own lengths and has checked positions against the block tables), long tiles last; `tile_tokens`
    is 4, 8 or 16 times 16 // group (default 4 times). Tokens that no tile lists keep what `out` held.
    With `num_splits` > 1 every tile's keys are walked in that many chunks of `chunk` keys (a
    multiple of 32; the last takes every key from its start on) by workgroups of their own, and the
    chunks are combined afterwards: for steps of few tokens over long contexts, which have too few
    tiles to fill the chip. The tiles must then list every token from `first_token` on.
    `pages_per_entry`: as for `paged_attention_wave`."""
    _gpu(q, k_cache, v_cache, block_tables, seq_of_token, positions, tiles)
    _need(q.dim() == 3 and q.is_contiguous(), "q must be contiguous [tokens, heads, head_dim]")
    T, nh, hd = q.shape
    nkv = k_cache.shape[2]
    _check_cache(k_cache, v_cache, q.dtype, nkv, hd)
    _need(nh % nkv == 0, lambda: f"{nh} heads do not divide into {nkv} key/value heads")
    _need(decode_kernel_takes(q, k_cache, v_cache),
          "the prefill kernel takes bfloat16, head_dim 32/64/96/128, groups of up to 16 heads, values in transposed pages")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous(),
          "block_tables must be contiguous int32 [requests, pages]")
    for name, t in (("seq_of_token", seq_of_token), ("positions", positions)):
        _need(t.dtype == torch.int32 and t.shape == (T,) and t.is_contiguous(), lambda: f"{name} must be int32 [tokens]")
    _need(tiles.dtype == torch.int32 and tiles.dim() == 2 and tiles.shape[1] == 2 and tiles.is_contiguous(),
          "tiles must be contiguous int32 [tiles, 2]")
    _need(waves == PREFILL_WAVES or (waves == 2 * PREFILL_WAVES and hd in (64, 128)),
          lambda: f"workgroups of {PREFILL_WAVES} waves, or of {2 * PREFILL_WAVES} for heads of 64 or 128 dimensions")
    per_wave = waves * (16 // (nh // nkv))
    tile_tokens = tile_tokens or per_wave
    _need(tile_tokens in (per_wave, 2 * per_wave) or (tile_tokens == 4 * per_wave and waves == PREFILL_WAVES),
          lambda: f"tiles of {tile_tokens} tokens; {per_wave}, twice or (4 waves) four times that")
    out = _out_like(q, out)
    part_o = part_ml = None
    if num_splits > 1:
        _need(chunk > 0 and chunk % 32 == 0 and 0 <= first_token < T, "chunks of a multiple of 32 keys, from a token of the step on")
        _need(num_splits <= MAX_DECODE_SPLITS, lambda: f"at most {MAX_DECODE_SPLITS} chunks")
        part_o = torch.empty((T, nh, num_splits, hd), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((T, nh, num_splits, 2), dtype=torch.float32, device=q.device)
    _run("paged_attention_prefill", library().ts_paged_attention_prefill(
        _ptr(out), _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(block_tables), _ptr(seq_of_token), _ptr(positions),
        _ptr(tiles), tiles.shape[0], tile_tokens, waves, nh, nkv, hd, k_cache.shape[1], *k_cache.stride()[:3], v_cache.stride(0),
        v_cache.stride(2), v_cache.stride(3), block_tables.shape[1], float(scale), int(window), first_token, T,
        num_splits, chunk, _ptr(part_o), _ptr(part_ml), _page_run(pages_per_entry), _stream()))
    return out


def paged_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, ctx, space: int,
                    scale: float, window: int = 0, leave_split: bool = False) -> "torch.Tensor | SplitAttention":
    """Attention of a packed step over the cache; picks the kernel for the storage type and shape.
    float32 always takes the one-wave-per-row kernel, whose sums do not depend on the batch;
    bfloat16 takes the matrix-core kernels where they serve the shape. `leave_split`: a step of single
    tokens whose keys are walked in chunks may come back as a `SplitAttention` (see `paged_attention_decode`)."""
    tables = ctx.block_tables[space]
    # (the tables count in pages of ctx.page_size tokens; the pools may be cut into shorter ones)
    table_page = getattr(ctx, "page_size", 0) or k_cache.shape[1]
    _need(table_page % k_cache.shape[1] == 0, lambda: f"block tables in pages of {table_page} over a cache in pages of {k_cache.shape[1]}")
    per_entry = table_page // k_cache.shape[1]
    if decode_kernel_takes(q, k_cache, v_cache):
        capacity = tables.shape[1] * table_page
        decode_ok = -(-capacity // 1024) <= MAX_DECODE_SPLITS and q.shape[0] <= MAX_DECODE_TOKENS
        if ctx.max_query_len == 1 and decode_ok:
            return paged_attention_decode(q, k_cache, v_cache, tables, ctx.seq_of_token, ctx.positions, scale, window,
                                          pages_per_entry=per_entry, leave_split=leave_split)
        # the one-token requests that lead the step go to the split-key kernel, the rest to the tiles
        cu = ctx.host_cu_seqlens
        lead = 0
        while decode_ok and lead + 1 < len(cu) and cu[lead + 1] - cu[lead] == 1:
            lead += 1
        nkv = k_cache.shape[2]
        walked = sum((cu[i + 1] - cu[i]) * (ctx.host_starts[i] + (cu[i + 1] - cu[i] + 1) / 2) for i in range(lead, len(cu) - 1))
        mean_keys = walked / max(1, q.shape[0] - lead)
        tile_tokens = prefill_tile_tokens(q.shape[0] - lead, nkv, q.shape[1] // nkv, q.shape[2], mean_keys)
        waves = prefill_waves(tile_tokens, q.shape[1] // nkv, q.shape[2], mean_keys)
        tiles = ctx.scratch.get(("attention_tiles", tile_tokens, lead))
        if tiles is None:
            flat = attention_tiles(cu, ctx.host_starts, tile_tokens, lead)
            tiles = torch.tensor(flat, dtype=torch.int32).view(-1, 2).to(q.device, non_blocking=True)
            ctx.scratch[("attention_tiles", tile_tokens, lead)] = tiles
        out = torch.empty_like(q)
        if lead:
            paged_attention_decode(q[:lead], k_cache, v_cache, tables, ctx.seq_of_token[:lead], ctx.positions[:lead],
                                   scale, window, out=out[:lead], pages_per_entry=per_entry)
        splits, chunk = prefill_splits(tiles.shape[0] * nkv, max(ctx.host_context_lens[lead:], default=0))
        return paged_attention_prefill(q, k_cache, v_cache, tables, ctx.seq_of_token, ctx.positions, tiles, scale,
                                       window, tile_tokens=tile_tokens, out=out, num_splits=splits, chunk=chunk,
                                       first_token=cu[lead], waves=waves, pages_per_entry=per_entry)
    return paged_attention_wave(q, k_cache, v_cache, tables, ctx.seq_of_token, ctx.positions, scale, window,
                                pages_per_entry=per_entry)


SKINNY_MAX_ROWS = 32
SKINNY_FUSED_ROWS = 16       # the fused norm serves one 16-row block of x,
SKINNY_EPILOGUE_ROWS = 64    # the gate and the rotation on the way out up to four,
SKINNY_EPILOGUE_WIDE_K = 2048    # for reductions up to this
SKINNY_NORM_MAX_K = 2048     # longest reduction with the norm on the way in,
SKINNY_EPILOGUE_MAX_K = 4096     # and with the gate or the rotation on the way out
SKINNY_WIDE_ELEMENTS = 8 << 20   # largest matrix that `linear_bf16` gives the kernel with 17 to 32 rows


def skinny_takes(rows: int, k: int) -> bool:
    """Whether the weight-streaming kernel serves `rows` rows of x over a reduction of `k` (33 to 64
    rows: reductions of up to 2048 in steps of 256, which fit a workgroup of 8 waves)."""
    if rows > SKINNY_MAX_ROWS:
        return rows <= SKINNY_EPILOGUE_ROWS and k % 256 == 0 and k <= SKINNY_EPILOGUE_WIDE_K
    return (k % 256 == 0 and k // 256 <= 16) or (k % 512 == 0 and k // 512 <= 16)


class PreparedNorm:
    """A residual sum and the first half of the norm that follows it, as the projection before them
    leaves them (`next_norm=` of the weight-streaming kernels): `summed` = T(T(y) + residual), the new
    residual [M, N]; `operand` = T((T(y) + residual) * weight), what the next projection multiplies;
    `squares` [M, parts] float32, whose row sums are the rows' sums of squares of T(y) + residual. The
    projection that takes `operand` multiplies its finished sums by rsqrt(sum(squares) / N + eps)
    (`squares=`, `eps=` of the same kernels): together that is norm(y + residual) * weight."""

    __slots__ = ("summed", "operand", "squares")

    def __init__(self, summed: torch.Tensor, operand: torch.Tensor, squares: torch.Tensor) -> None:
        self.summed, self.operand, self.squares = summed, operand, squares


OPERAND_ROW_SKEW = 8      # elements between the rows of an operand made for kernels that read 16 rows of x side by side
GATED_SKEW_MIN_ROWS = 5   # rows from which a gated product's result, the down projection's operand, gets the skew too


def _gated_output(rows: int, width: int, device) -> torch.Tensor:
    """Where silu(gate) * up goes: bfloat16 [rows, width], with the rows of more than a few lying
    `OPERAND_ROW_SKEW` elements further apart than they are long (the down projection over 8,192 of
    8 rows 10.2 -> 9.8 µs, of 64 rows 15.4 -> 15.0; up to 4 rows the dense form is as fast)."""
    skew = OPERAND_ROW_SKEW if rows >= GATED_SKEW_MIN_ROWS else 0
    return torch.empty((rows, width + skew), dtype=torch.bfloat16, device=device)[:, :width]


def _next_norm_outputs(x: torch.Tensor, n: int, parts: int, next_norm, skew: int = 0,
                       rows: int | None = None) -> tuple[PreparedNorm, torch.Tensor | None, torch.Tensor]:
    """Checks `next_norm` = (residual or None, weight) for a product [M, n] and makes its outputs.
    `skew`: the operand's rows lie n + skew elements apart. (The kernels that take it read the same
    64 bytes of 16 rows with one instruction; rows a power of two apart are slow to fetch that way:
    64 rows over 2,048 against the q|k|v weight 12.0 µs, 10.2 with rows 16 bytes further apart, against
    the gate|up weight 20.4 and 18.9.) `rows`: the product's rows where x is not [M, K] itself."""
    residual, weight = next_norm
    _gpu(residual, weight)
    M = x.shape[0] if rows is None else rows
    _need(weight.dtype == torch.bfloat16 and weight.shape == (n,) and weight.is_contiguous(), lambda: f"the next norm's weight must be bfloat16 [{n}]")
    if residual is not None:
        _need(residual.dtype == torch.bfloat16 and residual.shape == (M, n) and residual.is_contiguous(),
              lambda: f"the residual must be bfloat16 [{M}, {n}]")
    out = PreparedNorm(torch.empty((M, n), dtype=torch.bfloat16, device=x.device),
                       torch.empty((M, n + skew), dtype=torch.bfloat16, device=x.device)[:, :n],
                       torch.empty((M, parts), dtype=torch.float32, device=x.device))
    return out, residual, weight


def _check_squares(squares: torch.Tensor | None, rows: int) -> None:
    if squares is not None:
        _gpu(squares)
        _need(squares.dtype == torch.float32 and squares.dim() == 2 and squares.shape[0] == rows and squares.shape[1] >= 1
              and squares.is_contiguous(), lambda: f"the sums of squares must be contiguous float32 [{rows}, parts]")


def pack_weight(weight: torch.Tensor) -> torch.Tensor:
    """A copy of bfloat16 `weight` [N, K] (K a multiple of 32) in the order the weight-streaming
    kernel reads it: [N / 16 tiles, K / 32 steps, 64 lanes, 8], lane r + 16 g holding row 16 tile + r,
    k = 32 step + 8 g .. + 7; rows past N are zeros. Every load of a wave is then one contiguous
    kilobyte, which streams about a sixth faster than sixteen 64-byte pieces of sixteen rows."""
    _gpu(weight)
    _need(weight.dtype == torch.bfloat16 and weight.dim() == 2 and weight.shape[1] % 32 == 0,
          "pack_weight takes bfloat16 [N, K] with K a multiple of 32")
    n, k = weight.shape
    tiles = -(-n // 16)
    padded = weight if n == 16 * tiles else torch.cat([weight, weight.new_zeros(16 * tiles - n, k)])
    return padded.view(tiles, 16, k // 32, 4, 8).permute(0, 2, 3, 1, 4).contiguous().view(tiles, k // 32, 64, 8)


def pack_weight_rope(weight: torch.Tensor, head_dim: int) -> torch.Tensor:
    """A copy of a fused q|k|v weight [heads * head_dim, K] in the order `qkv_rope_store` reads it:
    `pack_weight` of the matrix with its rows regrouped so that a 16-row tile holds 8 rows of the first
    half of a head and, below them, the 8 rows that rotate with them (head_dim / 2 further on)."""
    _gpu(weight)
    _need(weight.dim() == 2 and head_dim % 16 == 0 and weight.shape[0] % head_dim == 0,
          "pack_weight_rope takes [heads * head_dim, K] with head_dim a multiple of 16")
    heads, half = weight.shape[0] // head_dim, head_dim // 2
    # [head, half (0: first, 1: second), block of 8, row] -> [head, block, half, row]
    regrouped = weight.view(heads, 2, half // 8, 8, weight.shape[1]).permute(0, 2, 1, 3, 4).reshape(weight.shape)
    return pack_weight(regrouped)


def _check_packed(packed: torch.Tensor | None, weight: torch.Tensor) -> None:
    if packed is not None:
        n, k = weight.shape
        _gpu(packed)
        _need(packed.dtype == torch.bfloat16 and packed.shape == (-(-n // 16), k // 32, 64, 8) and packed.is_contiguous()
              and packed.data_ptr() % 16 == 0, lambda: f"the packed copy does not belong to a weight of {n} x {k}")


SKINNY8_MAX_ROWS = 8          # rows of x that the 8-row form of the weight-streaming kernel takes
SKINNY8_FEW_ROWS = 4          # up to this many rows it is chosen for a matrix of any width,
SKINNY8_FULL_WIDTH = 2048     # with more rows only up to this width (a workgroup per compute unit)


def skinny8_steps(k: int) -> int:
    """32-wide k steps per wave of the 8-row form for a reduction of `k` (a wave covers 64 of them per
    step): the fewest steps that fit 8 waves, else 16 steps in up to 16 waves; 0 if it does not serve k."""
    for steps in (4, 8, 16):
        if k % (64 * steps) == 0 and k // (64 * steps) <= 8:
            return steps
    return 16 if k % 1024 == 0 and k // 1024 <= 16 else 0


def skinny8_takes(rows: int, n: int, k: int) -> bool:
    """Whether `linear_bf16` gives the product to the 8-row form. Every workgroup reads all rows of x
    for its 8 rows of W, twice as much of x per byte of W as the 16-row form: with 8 rows of x and a
    matrix of 3,072 or 4,096 rows the compute units' reads of x out of the second-level cache weigh
    as much as W itself, and the 16-row form or the library is faster (decode steps at the 3B and 8B
    layer sizes, batch 8: 2.59 against 2.67 ms and 4.39 against 4.55; at batch 1 the 8-row form wins
    at every width). So: few rows of x at any width, more rows only where the 8-row tiles are what
    gives every compute unit a workgroup."""
    return (rows <= SKINNY8_MAX_ROWS and skinny8_steps(k) > 0
            and (rows <= SKINNY8_FEW_ROWS or n <= SKINNY8_FULL_WIDTH))


class PackedRows8:
    """Up to 8 rows of a bfloat16 matrix [rows, k] in the order the lanes of the 8-row form read their
    x, for a reader of `steps` steps a wave: `data` [k / (64 steps), steps, 64, 8], lane r + 16 g of
    (wave, step) holding row r % 8 at k = 64 steps wave + 32 steps (r // 8) + 32 step + 8 g .. + 7.
    The kernel then loads contiguous kilobytes instead of 64 bytes of each row in two places (the
    down projection of 8 rows over 8,192: 10.8 -> 9.2 µs). Lanes of rows past `rows` hold anything.
    What makes it (`gemm_skinny` with `pack8_steps`) and what reads it (`gemm_skinny8`) are chosen
    together by `linear`; nothing else takes it but `rows()`."""

    def __init__(self, data: torch.Tensor, rows: int, k: int, steps: int) -> None:
        self.data, self.num_rows, self.k, self.steps = data, rows, k, steps

    @property
    def shape(self) -> tuple[int, int]:
        return (self.num_rows, self.k)

    def rows(self) -> torch.Tensor:
        """The matrix [rows, k] itself (a copy), for tests and for readers that take no packed operand."""
        waves = self.k // (64 * self.steps)
        # [wave, step, g, half, row, 8] -> [row, wave, half, step, g, 8]
        return (self.data.view(waves, self.steps, 4, 2, 8, 8).permute(4, 0, 3, 1, 2, 5).reshape(8, self.k)[:self.num_rows]
                .contiguous())


def rows8_reader_steps(rows: int, weight: torch.Tensor) -> int:
    """The steps of the `PackedRows8` that `linear_bf16` takes as the operand of a product of `rows`
    rows by `weight`; 0: that product does not go to the 8-row form, its operand stays a matrix.
    From packed rows the 8-row form is the fastest at every width (8 rows against the down weight of
    3,072 x 8,192: 14.1 µs, 16.2 from a matrix by the 16-row form; 4,096 x 14,336: 26.0 against 26.6),
    also where `skinny8_takes` leaves a matrix of so many rows to other kernels."""
    if not (weight.is_cuda and weight.dtype == torch.bfloat16 and weight.dim() == 2 and weight.is_contiguous()
            and weight.data_ptr() % 16 == 0):
        return 0
    return skinny8_steps(weight.shape[1]) if rows <= SKINNY8_MAX_ROWS else 0


def pack_rows8(x: torch.Tensor, steps: int) -> PackedRows8:
    """`x` [rows <= 8, k] as a `PackedRows8` for a reader of `steps` steps (rows past the last are zeros)."""
    _need(x.dim() == 2 and x.dtype == torch.bfloat16 and x.shape[0] <= 8 and steps in (4, 8, 16) and x.shape[1] % (64 * steps) == 0,
          "pack_rows8 takes bfloat16 [rows <= 8, k], k in whole waves of 64 steps")
    rows, k = x.shape
    full = x if rows == 8 else torch.cat([x, x.new_zeros(8 - rows, k)])
    data = full.view(8, k // (64 * steps), 2, steps, 4, 8).permute(1, 3, 4, 2, 0, 5).contiguous().view(k // (64 * steps), steps, 64, 8)
    return PackedRows8(data, rows, k, steps)


def pack_weight8(weight: torch.Tensor) -> torch.Tensor:
    """A copy of bfloat16 `weight` [N, K] in the order the 8-row form reads it:
    [N / 8 tiles, waves, steps, 64 lanes, 8], lane r + 16 g holding row 8 tile + r % 8 at
    k = 64 steps wave + 32 steps (r // 8) + 32 step + 8 g .. + 7; rows past N are zeros."""
    _gpu(weight)
    _need(weight.dtype == torch.bfloat16 and weight.dim() == 2, "pack_weight8 takes bfloat16 [N, K]")
    n, k = weight.shape
    steps = skinny8_steps(k)
    _need(steps > 0, lambda: f"the 8-row form does not take a reduction of {k}")
    waves, tiles = k // (64 * steps), -(-n // 8)
    padded = weight if n == 8 * tiles else torch.cat([weight, weight.new_zeros(8 * tiles - n, k)])
    # [tile, row, wave, half, step, g, 8] -> [tile, wave, step, g, half, row, 8]
    return (padded.view(tiles, 8, waves, 2, steps, 4, 8).permute(0, 2, 4, 5, 3, 1, 6).contiguous()
            .view(tiles, waves, steps, 64, 8))


def gemm_skinny8(x: "torch.Tensor | PackedRows8 | SplitAttention", weight: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16,
                 packed8: torch.Tensor | None = None, next_norm=None) -> "torch.Tensor | PreparedNorm":
    """bfloat16 x [M <= 8, K] · weight [N, K]^T by the weight-streaming kernel's 8-row form (a matrix
    instruction multiplies 8 rows of W by 8 rows of x over 64 k; a workgroup owns 8 rows of W).
    x may come as a `PackedRows8` made for this K. With `packed8` (= pack_weight8(weight)) the kernel
    reads that copy. With `next_norm` = (residual or None, weight of the norm that follows) the product
    is not stored: a `PreparedNorm` comes back. x may also be a `SplitAttention` that `split_attention_fuses`
    allows: the kernel then adds up the chunks' parts on its way in (bfloat16 out)."""
    x_packed = isinstance(x, PackedRows8)
    split = x if isinstance(x, SplitAttention) else None
    xt = x.data if x_packed else x.parts if split is not None else x
    _gpu(xt, weight, packed8)
    if split is not None:
        _gpu(split.sums, split.positions)
        tokens, heads, chunks, hd = split.parts.shape
        _need(split_attention_fuses(tokens, weight) and chunks <= SPLIT_ATTENTION_MAX_CHUNKS and hd % 32 == 0
              and out_dtype == torch.bfloat16
              and split.parts.dtype == torch.float32 and split.parts.is_contiguous() and split.sums.is_contiguous()
              and split.sums.shape == (tokens, heads, chunks, 2) and split.sums.dtype == torch.float32
              and split.positions.dtype == torch.int32 and split.positions.shape == (tokens,) and split.positions.is_contiguous()
              and split.parts.data_ptr() % 16 == 0 and split.sums.data_ptr() % 16 == 0,
              lambda: f"gemm_skinny8 does not take these parts: {tuple(split.parts.shape)} against {tuple(weight.shape)}")
    _need((split is not None or xt.dtype == torch.bfloat16) and weight.dtype == torch.bfloat16, "gemm_skinny8 takes bfloat16")
    _need(len(x.shape) == 2 and weight.dim() == 2 and x.shape[1] == weight.shape[1],
          lambda: f"shapes {tuple(x.shape)} x {tuple(weight.shape)}^T")
    M, K = x.shape
    N = weight.shape[0]
    steps = skinny8_steps(K)
    _need(M <= SKINNY8_MAX_ROWS and steps > 0, lambda: f"gemm_skinny8 takes up to {SKINNY8_MAX_ROWS} rows and K in steps of 256 up to "
          "8192 or of 1024 up to 16384")
    if x_packed:
        _need(x.steps == steps and xt.is_contiguous() and xt.numel() == 8 * K, lambda: f"the packed rows were made for a reader of {x.steps} steps, not {steps}")
    _need((x_packed or split is not None or _dense_rows(xt)) and weight.is_contiguous() and xt.data_ptr() % 16 == 0 and weight.data_ptr() % 16 == 0,
          "rows must be dense and 16-byte aligned")
    ldx = K if x_packed or split is not None else xt.stride(0)
    comb = ((_ptr(split.parts), _ptr(split.sums), _ptr(split.positions), split.parts.shape[2], split.chunk, split.window,
             split.parts.shape[3]) if split is not None else (None, None, None, 0, 0, 0, 0))
    x_arg = None if split is not None else _ptr(xt)
    _need(out_dtype in (torch.bfloat16, torch.float32), "the result is bfloat16 or float32")
    if packed8 is not None:
        _need(packed8.dtype == torch.bfloat16 and packed8.shape == (-(-N // 8), K // (64 * steps), steps, 64, 8)
              and packed8.is_contiguous() and packed8.data_ptr() % 16 == 0 and N % 8 == 0,
              lambda: f"the packed copy does not belong to a weight of {N} x {K}")
    if next_norm is not None:
        _need(out_dtype == torch.bfloat16, "a prepared norm comes with bfloat16")
        prepared, residual, nw = _next_norm_outputs(xt, N, -(-N // 8), next_norm, rows=M)
        _run("gemm_skinny8", library().ts_gemm_skinny8_bf16(
            None, x_arg, _ptr(weight if packed8 is None else packed8), M, N, K, ldx, weight.stride(0), N, 1,
            int(packed8 is not None), _ptr(residual), _ptr(nw), _ptr(prepared.summed), _ptr(prepared.operand),
            _ptr(prepared.squares), int(x_packed), *comb, _stream()))
        return prepared
    out = torch.empty((M, N), dtype=out_dtype, device=xt.device)
    _run("gemm_skinny8", library().ts_gemm_skinny8_bf16(
        _ptr(out), x_arg, _ptr(weight if packed8 is None else packed8), M, N, K, ldx, weight.stride(0),
        out.stride(0), _code(out_dtype), int(packed8 is not None), None, None, None, None, None, int(x_packed), *comb, _stream()))
    return out


def skinny_fuses(rows: int, k: int, norm: bool, glu: bool) -> bool:
    """Whether the kernel can apply the norm on the way in and/or the gate on the way out (a norm
    that the kernel before has prepared counts as none: it is a scale on the way out)."""
    if not (norm or glu):
        return skinny_takes(rows, k)
    if k % 256:
        return False
    if norm or rows <= SKINNY_FUSED_ROWS:
        return rows <= SKINNY_FUSED_ROWS and k <= (SKINNY_NORM_MAX_K if norm else SKINNY_EPILOGUE_MAX_K)
    return rows <= SKINNY_EPILOGUE_ROWS and k <= SKINNY_EPILOGUE_WIDE_K


def gemm_skinny(x: torch.Tensor, weight: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16, *,
                residual: torch.Tensor | None = None, norm_weight: torch.Tensor | None = None, eps: float = 0.0,
                glu: bool = False, packed: torch.Tensor | None = None, squares: torch.Tensor | None = None,
                next_norm=None, pack8_steps: int = 0) -> "tuple[torch.Tensor | PreparedNorm | PackedRows8, torch.Tensor | None]":
    """bfloat16 e(f(x) [M <= 32, K] · weight [N, K]^T) by the weight-streaming MFMA kernel (up to 64
    rows over reductions of up to 2048). With `norm_weight`: f = RMSNorm(x + residual) * norm_weight,
    and x + residual comes back as the second result. With `squares` (and `eps`): x is the operand of
    a `PreparedNorm` and `squares` its sums of squares; the rows' scales multiply the finished sums.
    With `glu`: weight holds gate rows then up rows and the result is silu(gate) * up, [M, N / 2].
    With `packed` (= pack_weight(weight)) the kernel reads that copy. With `next_norm` = (residual or
    None, weight of the norm that follows) the first result is a `PreparedNorm` instead of the product.
    With `pack8_steps` (and `glu`, up to 8 rows) the gated product comes back as a `PackedRows8` for a
    reader of that many steps."""
    _gpu(x, weight, residual, norm_weight)
    _need(x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16, "gemm_skinny takes bfloat16")
    _need(x.dim() == 2 and weight.dim() == 2 and x.shape[1] == weight.shape[1],
          lambda: f"shapes {tuple(x.shape)} x {tuple(weight.shape)}^T")
    M, K = x.shape
    N = weight.shape[0]
    norm = norm_weight is not None
    _need(skinny_fuses(M, K, norm, glu),
          lambda: f"gemm_skinny takes up to {SKINNY_MAX_ROWS} rows ({SKINNY_FUSED_ROWS} with the norm, {SKINNY_EPILOGUE_ROWS} with the gate alone "
          "over up to 2048) and K in steps of 256 up to 4096 (2048 with the norm) or of 512 up to 8192")
    _need((x.is_contiguous() if norm else _dense_rows(x)) and weight.is_contiguous() and x.data_ptr() % 16 == 0
          and weight.data_ptr() % 16 == 0, "rows must be dense and 16-byte aligned (contiguous with the norm on the way in)")
    _need(not glu or (N % 32 == 0), "gate and up rows come in whole 16-row tiles")
    _check_packed(packed, weight)
    _check_squares(squares, M)
    _need(squares is None or not norm, "a norm is either prepared by the kernel before or made here")
    mode = 1 if norm else 2 if squares is not None else 0
    if next_norm is not None:
        _need(not glu and not norm and out_dtype == torch.bfloat16, "a prepared norm follows a plain bfloat16 product")
        prepared, nres, nw = _next_norm_outputs(x, N, library().ts_skinny_tiles(M, N, K), next_norm)
        _run("gemm_skinny", library().ts_gemm_skinny_bf16(
            None, _ptr(x), _ptr(weight if packed is None else packed), None, None, None, M, N, K, x.stride(0),
            weight.stride(0), N, float(eps), mode, 0, 1, int(packed is not None), _ptr(squares),
            0 if squares is None else squares.shape[1], _ptr(nres), _ptr(nw), _ptr(prepared.summed), _ptr(prepared.operand),
            _ptr(prepared.squares), 0, _stream()))
        return prepared, None
    res_out = None
    if norm:
        _need(norm_weight.dtype == torch.bfloat16 and norm_weight.shape == (K,) and norm_weight.is_contiguous(),
              "the norm weight must be bfloat16 [K]")
        if residual is not None:
            _need(residual.shape == x.shape and residual.dtype == x.dtype and residual.is_contiguous(),
                  "residual must match the input")
            res_out = torch.empty_like(x)
        else:
            res_out = x
    else:
        _need(residual is None, "a residual comes with a norm weight")
    _need(out_dtype == torch.bfloat16 or not (norm or glu), "float32 output comes with the plain product only")
    if pack8_steps:
        _need(glu and M <= 8 and pack8_steps in (4, 8, 16) and (N // 2) % (64 * pack8_steps) == 0,
              "packed rows come from a gated product of up to 8 rows whose width is whole waves of the reader")
        out = torch.empty(((N // 2) // (64 * pack8_steps), pack8_steps, 64, 8), dtype=torch.bfloat16, device=x.device)
        ldy = N // 2
    else:
        out = _gated_output(M, N // 2, x.device) if glu else torch.empty((M, N), dtype=out_dtype, device=x.device)
        ldy = out.stride(0)
    _run("gemm_skinny", library().ts_gemm_skinny_bf16(
        _ptr(out), _ptr(x), _ptr(weight if packed is None else packed), _ptr(residual), _ptr(norm_weight),
        _ptr(res_out) if residual is not None else None, M, N, K, x.stride(0), weight.stride(0), ldy,
        float(eps), mode, int(glu), _code(out_dtype), int(packed is not None), _ptr(squares),
        0 if squares is None else squares.shape[1], None, None, None, None, None, int(pack8_steps), _stream()))
    return (PackedRows8(out, M, N // 2, pack8_steps) if pack8_steps else out), res_out


ROWS64_MIN_ROWS = 33         # fewer rows are the weight-streaming kernel's (gemm_skinny: 32 rows 16.6 µs against 17.7 here,
                             # 48 rows 23.7 against 19.3, 64 rows 26.9 against 20.7 for a gate|up weight of 16,384 x 2,048),
ROWS64_MAX_ROWS = 128        # rows of x the kernel takes (eight blocks of 16 in LDS): more are the matrix library's
ROWS64_PLAIN_MAX_ROWS = 64   # a plain wide product (the head) of more rows is the library's too: 128 rows against the
                             # vocabulary matrix take 147 µs here and 125 there. What rides on the kernel pays for 65 to
                             # 128 rows: the gate (24.0 µs against 24.2 for the library and the gate kernel), and for the
                             # narrow products in slices the finishing kernel (o 12.7 against 14.2 for the library and
                             # the norm kernel, down 18.6 against 23.9, q|k|v with the rotation 18.1 against 20.4): a
                             # decode step at batch 128 takes 2.99 ms instead of 3.20, at batch 96 2.47 instead of 2.76
ROWS64_MIN_WIDTH = 8192      # rows of W from which 64 of them a workgroup still give every compute unit one


def rows64_takes(rows: int, n: int, k: int, glu: bool = False) -> bool:
    """Whether `gemm_rows64` is the kernel for `rows` rows of x against a weight [n, k] (`glu`: with the gate)."""
    return (ROWS64_MIN_ROWS <= rows <= (ROWS64_MAX_ROWS if glu else ROWS64_PLAIN_MAX_ROWS) and n >= ROWS64_MIN_WIDTH
            and n % 64 == 0 and k % 1024 == 0)


def gemm_rows64(x: torch.Tensor, packed: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16, *,
                glu: bool = False, squares: torch.Tensor | None = None, eps: float = 0.0) -> torch.Tensor:
    """bfloat16 e(x [M <= 128, K] · W [N, K]^T) for a wide W given as `packed` = pack_weight(W), by the
    kernel that shares x among 64 rows of W through LDS (gemm_rows64.hip). With `glu`, W holds gate
    rows then up rows and the result is silu(gate) * up, [M, N / 2]. With `squares` (and `eps`) x is
    the operand of a `PreparedNorm` and the rows' scales multiply the finished sums."""
    _gpu(x, packed)
    _need(x.dtype == torch.bfloat16 and packed.dtype == torch.bfloat16 and x.dim() == 2 and packed.dim() == 4
          and packed.shape[2:] == (64, 8) and packed.is_contiguous(), "gemm_rows64 takes bfloat16 x [M, K] and pack_weight(W)")
    M, K = x.shape
    N = packed.shape[0] * 16
    _need(packed.shape[1] * 32 == K, lambda: f"the packed copy is of a weight over {packed.shape[1] * 32}, x is over {K}")
    _need(1 <= M <= ROWS64_MAX_ROWS and N % (128 if glu else 64) == 0 and K % 1024 == 0,
          lambda: f"gemm_rows64 takes up to {ROWS64_MAX_ROWS} rows, N in steps of 64 (128 with the gate) and K in steps of 1024, "
          f"not {M} x {K} against {N}")
    _need(x.stride(1) == 1 and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0, "rows of x must be dense and 16-byte aligned")
    _need(out_dtype == torch.bfloat16 or (out_dtype == torch.float32 and not glu), "32-bit output comes without the gate")
    _check_squares(squares, M)
    out = _gated_output(M, N // 2, x.device) if glu else torch.empty((M, N), dtype=out_dtype, device=x.device)
    _run("gemm_rows64", library().ts_gemm_rows64_bf16(
        _ptr(out), _ptr(x), _ptr(packed), M, N, K, x.stride(0), out.stride(0), int(glu), int(out_dtype == torch.float32),
        _ptr(squares), 0 if squares is None else squares.shape[1], float(eps), _stream()))
    return out


ROWS64_SLICE_K = 512           # a slice of the reduction is a multiple of this (one turn of a compute wave's ring of W)
ROWS64_SLICED_MIN_ROWS = 5     # (fewer rows are the 8-row form's at any width; where the weight-streaming kernels serve a shape, they come first)
ROWS64_WORKGROUPS = 192        # workgroups from which the chip's 256 compute units count as filled


def rows64_slices(rows: int, n: int, k: int) -> int:
    """Slices of the reduction that `gemm_rows64_sliced` cuts a product of `rows` rows of x against a
    narrow weight [n, k] into: the fewest that give every compute unit a workgroup of 64 rows of W
    (else the most the reduction allows); 0 where the kernel does not serve the shape or the weight
    is wide enough for `gemm_rows64` itself. Measured with the finishing kernel, against the library
    followed by the norm kernel, for a down projection over 8,192 (14,336 at the widest): 9 rows 12.9
    against 15.5 µs at a width of 2,048, 15.8 against 18.5 at 3,072, 27.0 against 31.1 at 4,096; 32 rows
    14.1 against 18.9, 17.3 against 21.6, 27.5 against 38.3; 64 rows 15.5 against 22.0 + 7 at 2,048."""
    if not (ROWS64_SLICED_MIN_ROWS <= rows <= ROWS64_MAX_ROWS) or n % 64 or n >= ROWS64_MIN_WIDTH or k % ROWS64_SLICE_K:
        return 0
    fits = [s for s in range(1, 17) if (k // ROWS64_SLICE_K) % s == 0]
    enough = [s for s in fits if (n // 64) * s >= ROWS64_WORKGROUPS]
    return enough[0] if enough else fits[-1]


def gemm_rows64_sliced(x: torch.Tensor, packed: torch.Tensor, slices: int, next_norm=None) -> "torch.Tensor | PreparedNorm":
    """bfloat16 x [M <= 64, K] · W [N, K]^T for a narrow W given as `packed` = pack_weight(W): the
    shared-x kernel with the reduction in `slices` slices (K / slices a multiple of 512), whose 32-bit
    parts a second kernel adds in ascending order. With `next_norm` = (residual or None, weight of the
    norm that follows) the product is not stored: a `PreparedNorm` comes back."""
    _gpu(x, packed)
    _need(x.dtype == torch.bfloat16 and packed.dtype == torch.bfloat16 and x.dim() == 2 and packed.dim() == 4
          and packed.shape[2:] == (64, 8) and packed.is_contiguous(), "gemm_rows64_sliced takes bfloat16 x [M, K] and pack_weight(W)")
    M, K = x.shape
    N = packed.shape[0] * 16
    _need(packed.shape[1] * 32 == K, lambda: f"the packed copy is of a weight over {packed.shape[1] * 32}, x is over {K}")
    _need(1 <= M <= ROWS64_MAX_ROWS and N % 64 == 0 and 1 <= slices <= 64 and K % (ROWS64_SLICE_K * slices) == 0,
          lambda: f"gemm_rows64_sliced takes up to {ROWS64_MAX_ROWS} rows, N in steps of 64 and slices of K that are multiples of "
          f"{ROWS64_SLICE_K}, not {M} x {K} against {N} in {slices}")
    _need(x.stride(1) == 1 and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0, "rows of x must be dense and 16-byte aligned")
    parts = torch.empty((slices, M, N), dtype=torch.float32, device=x.device)
    if next_norm is not None:
        prepared, residual, nw = _next_norm_outputs(x, N, 1, next_norm, skew=OPERAND_ROW_SKEW)
        _run("gemm_rows64_sliced", library().ts_gemm_rows64_sliced_bf16(
            None, _ptr(parts), _ptr(x), _ptr(packed), M, N, K, x.stride(0), slices, _ptr(residual), _ptr(nw),
            _ptr(prepared.summed), _ptr(prepared.operand), _ptr(prepared.squares), prepared.operand.stride(0), _stream()))
        return prepared
    out = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    _run("gemm_rows64_sliced", library().ts_gemm_rows64_sliced_bf16(
        _ptr(out), _ptr(parts), _ptr(x), _ptr(packed), M, N, K, x.stride(0), slices, None, None, None, None, None, 0, _stream()))
    return out


def _dense_rows(x: torch.Tensor) -> bool:
    """Whether the rows of a matrix are dense and begin at multiples of 16 bytes (they may lie further
    apart than they are long)."""
    return x.dim() == 2 and x.stride(1) == 1 and x.stride(0) % 8 == 0 and x.stride(0) >= x.shape[1]


def qkv_rope_max_rows(k: int, norm: bool = False) -> int:
    """Most rows of x that `qkv_rope_store` takes over a reduction of `k`, with or without the norm
    on the way in; 0 if it does not take the reduction at all."""
    if k % 256 or k > (SKINNY_NORM_MAX_K if norm else SKINNY_EPILOGUE_MAX_K):
        return 0
    return SKINNY_EPILOGUE_ROWS if not norm and k <= SKINNY_EPILOGUE_WIDE_K else SKINNY_FUSED_ROWS


STREAMING_MAX_ROWS = 64      # most rows of x for which `linear_bf16` reads a weight's streaming copy


def qkv_rope_fuses(x: torch.Tensor, weight: torch.Tensor, head_dim: int, k_cache: torch.Tensor | None,
                   norm: bool = False, table: torch.Tensor | None = None) -> bool:
    """Whether `qkv_rope_store` serves these operands: few bfloat16 rows, a reduction of up to 4096 in
    steps of 256 (2048 with the norm on the way in), heads of a multiple of 32 dimensions that turn
    whole (`table`, if given, as wide as a head), keys whose strides allow 8-byte stores."""
    rows_ok = x.dim() == 2 and x.shape[0] <= qkv_rope_max_rows(x.shape[1], norm) and (table is None or table.shape[1] == head_dim)
    return (x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and rows_ok and head_dim % 32 == 0
            and (x.is_contiguous() if norm else _dense_rows(x)) and weight.is_contiguous() and x.data_ptr() % 16 == 0
            and weight.data_ptr() % 16 == 0
            and (k_cache is None or (all(st % 4 == 0 for st in k_cache.stride()[:3]) and k_cache.data_ptr() % 8 == 0)))


def qkv_rope_store(x: torch.Tensor, weight: torch.Tensor, cos_sin: torch.Tensor | None, positions: torch.Tensor,
                   slots: torch.Tensor | None, k_cache: torch.Tensor | None, v_cache: torch.Tensor | None,
                   num_heads: int, num_kv_heads: int, head_dim: int, *, residual: torch.Tensor | None = None,
                   norm_weight: torch.Tensor | None = None, eps: float = 0.0, packed: torch.Tensor | None = None,
                   squares: torch.Tensor | None = None) -> tuple[torch.Tensor, torch.Tensor | None]:
    """`rope_store(f(x) · weight^T, ...)` in one kernel for few rows of x: the projection is never
    stored, q [tokens, nh, hd] comes back rotated, rotated k and v go to their cache slots. With
    `norm_weight`, f = RMSNorm(x + residual) * norm_weight and x + residual is the second result.
    With `squares` (and `eps`) x is the operand of a `PreparedNorm` instead, and the rows' scales
    multiply the finished sums. With `packed` (= pack_weight_rope(weight, head_dim)) the kernel reads
    that copy."""
    _gpu(x, weight, cos_sin, positions, slots, k_cache, v_cache, residual, norm_weight)
    _check_squares(squares, x.shape[0])
    _need(squares is None or norm_weight is None, "a norm is either prepared by the kernel before or made here")
    _need(qkv_rope_fuses(x, weight, head_dim, k_cache, norm_weight is not None),
          "qkv_rope_store takes up to 16 bfloat16 rows (64 over up to 2048 without the norm), K in steps of 256 up to 4096 "
          "(2048 with the norm), head_dim in steps of 32")
    M, K = x.shape
    _need(weight.shape == ((num_heads + 2 * num_kv_heads) * head_dim, K), lambda: f"weight {tuple(weight.shape)} for "
          f"{num_heads}+2x{num_kv_heads} heads of {head_dim} over {K}")
    _check_packed(packed, weight)
    _need(positions.dtype == torch.int32 and positions.shape == (M,) and positions.is_contiguous(),
          "positions must be int32 [tokens]")
    if cos_sin is not None:
        _need(cos_sin.dtype == torch.float32 and cos_sin.dim() == 2 and cos_sin.shape[1] == head_dim
              and cos_sin.is_contiguous(), "the rotation table must be float32 [positions, head_dim]")
    page_size, kst, vst = 1, (0, 0, 0), (0, 0, 0, 0)
    if k_cache is not None:
        _need(v_cache is not None and slots is not None, "a cache write needs k, v and the slots")
        _need(slots.dtype == torch.int32 and slots.shape == (M,) and slots.is_contiguous(), "slots must be int32 [tokens]")
        _check_cache(k_cache, v_cache, x.dtype, num_kv_heads, head_dim)
        page_size, kst, vst = k_cache.shape[1], k_cache.stride()[:3], v_cache.stride()
    norm = norm_weight is not None
    res_out = None
    if norm:
        _need(norm_weight.dtype == torch.bfloat16 and norm_weight.shape == (K,) and norm_weight.is_contiguous(),
              "the norm weight must be bfloat16 [K]")
        if residual is not None:
            _need(residual.shape == x.shape and residual.dtype == x.dtype and residual.is_contiguous(),
                  "residual must match the input")
            res_out = torch.empty_like(x)
        else:
            res_out = x
    else:
        _need(residual is None, "a residual comes with a norm weight")
    q = torch.empty((M, num_heads, head_dim), dtype=x.dtype, device=x.device)
    _run("qkv_rope_store", library().ts_gemm_skinny_rope_bf16(
        _ptr(q), _ptr(x), _ptr(weight if packed is None else packed), _ptr(residual), _ptr(norm_weight),
        _ptr(res_out) if residual is not None else None, M, K, x.stride(0), weight.stride(0), float(eps),
        1 if norm else 2 if squares is not None else 0,
        int(packed is not None), _ptr(cos_sin), _ptr(positions), _ptr(slots), _ptr(k_cache), _ptr(v_cache), num_heads, num_kv_heads, head_dim,
        int(cos_sin is not None), page_size, *kst, *vst, _ptr(squares), 0 if squares is None else squares.shape[1], _stream()))
    return q, res_out


QKV_SLICED_MIN_ROWS = 33       # fewer rows: the library and the rotation kernel are as fast


def qkv_rope_sliced_slices(x: torch.Tensor, weight: torch.Tensor, head_dim: int, k_cache: torch.Tensor | None,
                           table: torch.Tensor | None = None) -> int:
    """Slices in which `qkv_rope_store_sliced` should serve these operands; 0 if it should not: 33 to
    64 bfloat16 rows over a reduction that `qkv_rope_store` does not take with so many rows (where it
    does, it is the faster one: 64 rows over 2,048 against 3,072 columns 12.2 µs, 12.7 in slices), heads
    of a multiple of 32 dimensions that turn whole, a width in steps of 64, a reduction in steps of
    512. Measured against the library followed by the rotation kernel at 64 rows: 16.3 against 20.8 µs
    over 3,072 against 5,120 columns, 22.0 against 21.4 over 4,096 against 6,144."""
    if not (x.dim() == 2 and x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and head_dim % 32 == 0
            and x.stride(1) == 1 and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0
            and (table is None or table.shape[1] == head_dim)
            and (k_cache is None or (all(st % 4 == 0 for st in k_cache.stride()[:3]) and k_cache.data_ptr() % 8 == 0))):
        return 0
    rows, (n, k) = x.shape[0], weight.shape
    if not (QKV_SLICED_MIN_ROWS <= rows <= ROWS64_MAX_ROWS) or rows <= qkv_rope_max_rows(k) or n % 64 or k % ROWS64_SLICE_K:
        return 0
    fits = [s for s in range(1, 17) if (k // ROWS64_SLICE_K) % s == 0]
    enough = [s for s in fits if (n // 64) * s >= ROWS64_WORKGROUPS]
    return enough[0] if enough else fits[-1]


def qkv_rope_store_sliced(x: torch.Tensor, packed_rope: torch.Tensor, slices: int, cos_sin: torch.Tensor | None,
                          positions: torch.Tensor, slots: torch.Tensor | None, k_cache: torch.Tensor | None,
                          v_cache: torch.Tensor | None, num_heads: int, num_kv_heads: int, head_dim: int, *,
                          eps: float = 0.0, squares: torch.Tensor | None = None) -> torch.Tensor:
    """`qkv_rope_store` for 17 to 64 rows by the shared-x kernel with the reduction in `slices` and a
    second kernel that adds the parts, rotates and writes the cache: q [tokens, nh, hd] comes back.
    `packed_rope` = pack_weight_rope(weight, head_dim). With `squares` (and `eps`) x is the operand of
    a `PreparedNorm` and the rows' scales multiply the finished sums."""
    _gpu(x, packed_rope, cos_sin, positions, slots, k_cache, v_cache)
    _check_squares(squares, x.shape[0])
    M, K = x.shape
    N = (num_heads + 2 * num_kv_heads) * head_dim
    _need(x.dtype == torch.bfloat16 and packed_rope.dtype == torch.bfloat16 and packed_rope.dim() == 4
          and packed_rope.shape == (N // 16, K // 32, 64, 8) and packed_rope.is_contiguous() and packed_rope.data_ptr() % 16 == 0,
          lambda: f"qkv_rope_store_sliced takes bfloat16 x [M, K] and pack_weight_rope of a weight [{N}, {K}]")
    _need(1 <= M <= ROWS64_MAX_ROWS and N % 64 == 0 and head_dim % 32 == 0 and 1 <= slices <= 64 and K % (ROWS64_SLICE_K * slices) == 0,
          lambda: f"qkv_rope_store_sliced takes up to {ROWS64_MAX_ROWS} rows, a width in steps of 64, heads in steps of 32 and slices of K that "
          f"are multiples of {ROWS64_SLICE_K}, not {M} x {K} against {N} in {slices}")
    _need(x.stride(1) == 1 and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0, "rows of x must be dense and 16-byte aligned")
    _need(positions.dtype == torch.int32 and positions.shape == (M,) and positions.is_contiguous(), "positions must be int32 [tokens]")
    if cos_sin is not None:
        _need(cos_sin.dtype == torch.float32 and cos_sin.dim() == 2 and cos_sin.shape[1] == head_dim
              and cos_sin.is_contiguous(), "the rotation table must be float32 [positions, head_dim]")
    page_size, kst, vst = 1, (0, 0, 0), (0, 0, 0, 0)
    if k_cache is not None:
        _need(v_cache is not None and slots is not None, "a cache write needs k, v and the slots")
        _need(slots.dtype == torch.int32 and slots.shape == (M,) and slots.is_contiguous(), "slots must be int32 [tokens]")
        _check_cache(k_cache, v_cache, x.dtype, num_kv_heads, head_dim)
        _need(all(st % 4 == 0 for st in k_cache.stride()[:3]) and k_cache.data_ptr() % 8 == 0, "key strides must allow 8-byte stores")
        page_size, kst, vst = k_cache.shape[1], k_cache.stride()[:3], v_cache.stride()
    parts = torch.empty((slices, M, N), dtype=torch.float32, device=x.device)
    q = torch.empty((M, num_heads, head_dim), dtype=x.dtype, device=x.device)
    _run("qkv_rope_store_sliced", library().ts_gemm_rows64_sliced_rope_bf16(
        _ptr(q), _ptr(parts), _ptr(x), _ptr(packed_rope), M, K, x.stride(0), slices, _ptr(squares),
        0 if squares is None else squares.shape[1], float(eps), _ptr(cos_sin), _ptr(positions), _ptr(slots), _ptr(k_cache),
        _ptr(v_cache), num_heads, num_kv_heads, head_dim, int(cos_sin is not None), page_size, *kst, *vst, _stream()))
    return q


MANY_ROWS_PRODUCTS = ("library", "tiled")
_many_rows = "library"


def many_rows_products(which: str | None = None) -> str:
    """Which kernel serves bfloat16 products of many rows: "library" (the vendor's, the faster one
    and the default) or "tiled" (this repository's LDS-tiled matrix-core kernel, for the shapes it
    takes). Sets it if `which` is given; returns the setting. It holds for the process."""
    global _many_rows
    if which is not None:
        _need(which in MANY_ROWS_PRODUCTS, lambda: f"products of many rows are one of {MANY_ROWS_PRODUCTS}, not {which!r}")
        _many_rows = which
    return _many_rows


def tiled_takes(x: torch.Tensor, weight: torch.Tensor, glu: bool = False) -> bool:
    """Whether the tiled kernel serves these operands (see gemm_tiled.hip for the conditions)."""
    n, k = weight.shape
    return (x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and k % 64 == 0 and n % (8 if glu else 4) == 0
            and x.stride(1) == 1 and weight.stride(1) == 1 and x.stride(0) % 8 == 0 and weight.stride(0) % 8 == 0
            and x.data_ptr() % 16 == 0 and weight.data_ptr() % 16 == 0)


def gemm_tiled(x: torch.Tensor, weight: torch.Tensor, glu: bool = False,
               out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """bfloat16 x [M, K] · weight [N, K]^T by the LDS-tiled matrix-core kernel; with `glu` the weight
    holds N / 2 gate rows, then N / 2 up rows, and silu(gate) · up [M, N / 2] comes back. The result
    is bfloat16, or (without `glu`) the 32-bit sums themselves with `out_dtype` float32."""
    _gpu(x, weight)
    _need(x.dim() == 2 and weight.dim() == 2 and x.shape[1] == weight.shape[1],
          lambda: f"shapes {tuple(x.shape)} x {tuple(weight.shape)}^T")
    _need(tiled_takes(x, weight, glu), "the tiled kernel takes bfloat16 operands with dense, 16-byte aligned rows, a "
          "reduction that is a multiple of 64 and a width that is a multiple of 4 (8 with the gate)")
    _need(out_dtype == torch.bfloat16 or (out_dtype == torch.float32 and not glu),
          "the tiled product comes out as bfloat16, or without the gate as float32")
    M, K = x.shape
    N = weight.shape[0]
    y = torch.empty((M, N // 2 if glu else N), dtype=out_dtype, device=x.device)
    if M and N:
        _run("gemm_tiled", library().ts_gemm_tiled_bf16(_ptr(y), _ptr(x), _ptr(weight), M, N, K, x.stride(0),
                                                        weight.stride(0), y.stride(0), int(glu),
                                                        int(out_dtype == torch.float32), _stream()))
    return y


class StreamingCopies:
    """A weight once more in the orders the weight-streaming kernels read it: `by16` for the form
    with 16-row tiles (`pack_weight`), `by8` for the 8-row form (`pack_weight8`); either may be None."""

    def __init__(self, by16: torch.Tensor | None = None, by8: torch.Tensor | None = None) -> None:
        self.by16, self.by8 = by16, by8

    def nbytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in (self.by16, self.by8) if t is not None)


def next_norm_fuses(x: "torch.Tensor | PackedRows8", weight: torch.Tensor, packed: "StreamingCopies | None" = None) -> bool:
    """Whether `linear_bf16(x, weight, next_norm=...)` has a kernel that leaves a `PreparedNorm`."""
    if isinstance(x, PackedRows8):          # (made for the 8-row form, which does)
        return True
    if not (x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and x.is_cuda and x.dim() == 2 and weight.dim() == 2
            and _dense_rows(x) and weight.is_contiguous() and x.data_ptr() % 16 == 0 and weight.data_ptr() % 16 == 0):
        return False
    rows, (n, k) = x.shape[0], weight.shape
    return skinny8_takes(rows, n, k) or _skinny_serves(rows, n, k) or _sliced_serves(rows, n, k, packed) > 0


ROWS64_PLAIN_MAX_WIDTH = 4096  # widest product that takes the sliced kernel when nothing rides on its finishing kernel


def _sliced_serves(rows: int, n: int, k: int, packed: "StreamingCopies | None", finishing: bool = True) -> int:
    """The slices in which `linear_bf16` gives a product to `gemm_rows64_sliced` (0: it does not).
    `finishing`: the second kernel also makes the residual sum and the next norm's first half, and
    so saves a kernel; without that the parts' trip through memory only pays for narrow products (32
    rows against a weight of 5,120 x 3,072: 14.5 µs, the library 11)."""
    if packed is None or packed.by16 is None or skinny8_takes(rows, n, k) or _skinny_serves(rows, n, k):
        return 0
    if not finishing and n > ROWS64_PLAIN_MAX_WIDTH:
        return 0
    return rows64_slices(rows, n, k)


def _skinny_serves(rows: int, n: int, k: int) -> bool:
    """Whether `linear_bf16` gives a plain product to the 16-row weight-streaming kernel. Measured:
    reductions longer than 4096 leave it too few workgroups, and with more than 16 rows it only wins
    on small matrices (8M elements: a layer's qkv and o, not its gate_up or the head); the library
    streams the rest faster."""
    return (rows <= SKINNY_MAX_ROWS and skinny_takes(rows, k) and k <= 4096
            and (rows <= SKINNY_FUSED_ROWS or n * k <= SKINNY_WIDE_ELEMENTS))


def linear_bf16(x: torch.Tensor, weight: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16,
                packed: StreamingCopies | None = None, next_norm=None) -> "torch.Tensor | PreparedNorm":
    """bfloat16 x [M, K] · weight [N, K]^T: few rows go to the weight-streaming kernels (which read
    the weight's copy in their own order from `packed`, if there is one), many to the vendor matrix
    library. With `next_norm` (where `next_norm_fuses` says so) a `PreparedNorm` comes back."""
    if isinstance(x, PackedRows8):
        _need(rows8_reader_steps(x.shape[0], weight) == x.steps, "packed rows go to the projection they were made for")
        return gemm_skinny8(x, weight, out_dtype, None if packed is None else packed.by8, next_norm=next_norm)
    _gpu(x, weight)
    _need(x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16, "linear_bf16 takes bfloat16")
    _need(x.dim() == 2 and weight.dim() == 2 and x.shape[1] == weight.shape[1],
          lambda: f"shapes {tuple(x.shape)} x {tuple(weight.shape)}^T")
    streams = _dense_rows(x) and weight.is_contiguous() and x.data_ptr() % 16 == 0 and weight.data_ptr() % 16 == 0
    if streams and skinny8_takes(x.shape[0], weight.shape[0], x.shape[1]):
        return gemm_skinny8(x, weight, out_dtype, None if packed is None else packed.by8, next_norm=next_norm)
    if streams and _skinny_serves(x.shape[0], weight.shape[0], x.shape[1]):
        return gemm_skinny(x, weight, out_dtype, packed=None if packed is None else packed.by16, next_norm=next_norm)[0]
    slices = (_sliced_serves(x.shape[0], weight.shape[0], x.shape[1], packed, next_norm is not None)
              if streams and out_dtype == torch.bfloat16 else 0)
    if slices:
        return gemm_rows64_sliced(x, packed.by16, slices, next_norm=next_norm)
    _need(next_norm is None, "no kernel leaves a prepared norm for this product (ask next_norm_fuses first)")
    # (float32: the 32-bit sums themselves, as the weight-streaming kernel gives them for few rows, so
    # that a row's logits are rounded the same way whatever the number of rows beside it)
    _need(out_dtype in (torch.bfloat16, torch.float32), lambda: f"bfloat16 products come out as bfloat16 or float32, not {out_dtype}")
    if (streams and packed is not None and packed.by16 is not None
            and rows64_takes(x.shape[0], weight.shape[0], x.shape[1])):
        return gemm_rows64(x, packed.by16, out_dtype)
    if _many_rows == "tiled" and tiled_takes(x, weight):
        return gemm_tiled(x, weight, out_dtype=out_dtype)
    return gemm_library(x, weight, out_dtype)


def gemm_library_init() -> None:
    """Makes the matrix library's handle and workspace on the current device. Steps that are recorded
    into graphs need it done beforehand (the runner does it when it is made)."""
    _run("gemm_library_init", library().ts_gemm_library_init())


def library_timing(on: bool | None = None) -> bool:
    """Whether the matrix library's candidates may be timed and the fastest kept (`library_tuning`, and
    the choice among three for row counts beyond 256 that are no multiple of 256). With it off every
    shape keeps the library's first candidate, so two processes round every product alike: candidates
    sum in different orders, and which of them is fastest may differ from run to run. Sets it for the
    process if `on` is given (shapes already chosen keep their choice); returns what it was."""
    lib = library()
    was = lib.ts_gemm_library_timing(1)
    lib.ts_gemm_library_timing(int(was if on is None else on))
    return bool(was)


def library_choices() -> list[dict[str, int | str]]:
    """The algorithm kept for every shape the matrix library has served on the current device:
    rows, columns, reduction, whether the output is 32-bit, how it was chosen ("first": the library's
    first candidate; "timed": the fastest of those timed; "open": still to be timed) and the
    library's index of the solution. A record of them tells two runs' roundings apart."""
    lib = library()
    n = lib.ts_gemm_library_choices(None, 0)
    buf = (ctypes.c_int64 * (6 * max(n, 1)))()
    n = min(n, lib.ts_gemm_library_choices(buf, n))
    how = ("first", "timed", "open")
    return [dict(rows=buf[6 * r], columns=buf[6 * r + 1], reduction=buf[6 * r + 2], out_float32=bool(buf[6 * r + 3]),
                 chosen=how[buf[6 * r + 4]], solution=buf[6 * r + 5]) for r in range(n)]


LIBRARY_WORKSPACE_BYTES = 128 << 20       # what gemm_library.hip allocates once per device for the library
LIBRARY_TUNING_SWEEP_BYTES = 320 << 20    # overwritten between timed runs: more than the caches hold (256 MB)
_library_tuning: torch.Tensor | None = None


@contextlib.contextmanager
def library_tuning():
    """While this is open, library products of 9 to 256 rows whose shape has not been tuned yet
    are tuned at their call: the library's candidates are timed on the call's operands with the
    caches swept in between, and the fastest serves the shape from then on (in this process, for
    every caller). Open it around the eager run that precedes the recording of a decode step."""
    global _library_tuning
    _library_tuning = torch.empty(LIBRARY_TUNING_SWEEP_BYTES, dtype=torch.uint8, device="cuda")
    try:
        yield
    finally:
        _library_tuning = None


def gemm_library(x: torch.Tensor, weight: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """bfloat16 x [M, K] · weight [N, K]^T by the vendor's matrix library, called directly with the
    algorithm kept for the shape (see gemm_library.hip). Rows may be strided. The result is bfloat16,
    or the 32-bit sums themselves with `out_dtype` float32."""
    _need(x.stride(1) == 1 and weight.stride(1) == 1, "rows of x and of the weight must be dense")
    _need(out_dtype in (torch.bfloat16, torch.float32), "the library product comes out as bfloat16 or float32")
    M, K = x.shape
    N = weight.shape[0]
    y = torch.empty((M, N), dtype=out_dtype, device=x.device)
    if M and N:
        sweep = _library_tuning
        _run("gemm_library", library().ts_gemm_library_bf16(
            _ptr(y), _ptr(x), _ptr(weight), M, N, K, x.stride(0), weight.stride(0), N, int(out_dtype == torch.float32),
            int(sweep is not None),
            _ptr(sweep), 0 if sweep is None else sweep.numel(), _stream()))
    return y


def measure_peaks(read_bytes: int = 2 << 30, repeats: int = 5) -> dict[str, float]:
    """What this GPU reaches in a kernel that only reads `read_bytes` of memory once (GB/s) and in a
    loop of bfloat16 matrix instructions on registers (TFLOP/s): the best of `repeats` timed runs
    each (peaks.hip)."""
    data = torch.empty(read_bytes // 4, dtype=torch.int32, device="cuda").fill_(1)
    sink = torch.zeros(1 << 16, dtype=torch.float32, device="cuda")
    cus = torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count
    begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

    def best(launch) -> float:
        times = []
        for _ in range(repeats + 1):
            begin.record()
            launch()
            end.record()
            end.synchronize()
            times.append(begin.elapsed_time(end))
        return min(times[1:]) * 1e-3

    groups, iters = 16 * cus, 1 << 14
    read_s = best(lambda: _run("peak_read", library().ts_peak_read(_ptr(data), data.numel() * 4, _ptr(sink), 8 * cus, _stream())))
    mfma_s = best(lambda: _run("peak_mfma", library().ts_peak_mfma(_ptr(sink), iters, groups, _stream())))
    return {"read_GBps": data.numel() * 4 / read_s / 1e9,
            "mfma_bf16_TFLOPs": groups * 4 * iters * 4 * 2 * 16 * 16 * 32 / mfma_s / 1e12}

