"""Host-side planning of the attention kernels: pure Python, no GPU."""

import random

from tinyserve_llm_amd.ops import hip


def test_attention_tiles_cover_each_token_once_and_never_cross_a_request():
    rng = random.Random(3)
    for _ in range(50):
        lens = [rng.randrange(1, 200) for _ in range(rng.randrange(1, 6))]
        starts = [rng.randrange(0, 500) for _ in lens]
        cu = [0]
        for n in lens:
            cu.append(cu[-1] + n)
        per = rng.choice([4, 12, 16, 64])
        first = rng.randrange(0, len(lens))
        flat = hip.attention_tiles(cu, starts, per, first)
        tiles = list(zip(flat[::2], flat[1::2]))
        seen = []
        for t0, n in tiles:
            assert 1 <= n <= per
            seq = max(s for s in range(len(lens)) if cu[s] <= t0)
            assert t0 + n <= cu[seq + 1], "a tile stays inside its request"
            seen.extend(range(t0, t0 + n))
        assert sorted(seen) == list(range(cu[first], cu[-1]))
        # ascending in the last position of the tile: the longest walks come last
        ends = []
        for t0, n in tiles:
            seq = max(s for s in range(len(lens)) if cu[s] <= t0)
            ends.append(starts[seq] + t0 - cu[seq] + n)
        assert ends == sorted(ends)


def test_prefill_tile_tokens_keeps_the_chip_busy():
    assert hip.prefill_tile_tokens(512, 8, 4, 64) == 16           # one row tile per wave: 256 workgroups
    assert hip.prefill_tile_tokens(2048, 8, 4, 64) == 32          # two: 64 tiles for each of 8 heads
    assert hip.prefill_tile_tokens(2048, 8, 3, 128) == 40         # groups of three: 52 tiles of 40 tokens
    assert hip.prefill_tile_tokens(4096, 8, 4, 64, mean_keys=2048) == 32
    assert hip.prefill_tile_tokens(4096, 8, 4, 64, mean_keys=4096) == 64      # four: small heads, a long walk
    assert hip.prefill_tile_tokens(16384, 8, 4, 128, mean_keys=8192) == 32    # large heads stop at two
    assert hip.prefill_tile_tokens(10, 1, 16, 32) == 4
    # eight waves a workgroup where four would hold two row tiles each and the walk is short
    assert hip.prefill_waves(32, 4, 64, mean_keys=1024.5) == 8 and hip.prefill_waves(32, 4, 128, mean_keys=1024.5) == 8
    assert hip.prefill_waves(32, 4, 64, mean_keys=4096.0) == 4, "a long walk: the doubled reads of LDS cost more"
    assert hip.prefill_waves(16, 4, 64, mean_keys=256.0) == 4 and hip.prefill_waves(64, 4, 64, mean_keys=100.0) == 4
    assert hip.prefill_waves(40, 3, 96, mean_keys=500.0) == 4, "twelve registers a step do not go round eight waves"
    for tokens, nkv, group in ((100, 2, 3), (5000, 4, 8), (100000, 8, 1)):
        per_wave = hip.PREFILL_WAVES * (16 // group)
        assert hip.prefill_tile_tokens(tokens, nkv, group, 64, 5000.0) in (per_wave, 2 * per_wave, 4 * per_wave)


def test_prefill_splits_cut_long_walks_of_few_tiles():
    assert hip.prefill_splits(64, 6272) == (8, 800)            # 8 tiles for each of 8 heads over 6K keys
    assert hip.prefill_splits(512, 6272) == (1, 0)             # enough tiles: uncut
    assert hip.prefill_splits(64, 1500) == (1, 0)              # a short context: uncut
    assert hip.prefill_splits(8, 2304) == (4, 576)             # chunks of at least 512 keys
    for workgroups, longest in ((1, 100000), (300, 2048), (17, 5000), (2, 1 << 20), (1, 2049)):
        splits, chunk = hip.prefill_splits(workgroups, longest)
        assert splits == 1 or (chunk % 32 == 0 and splits * chunk >= longest and (splits - 1) * chunk < longest
                               and splits <= hip.MAX_DECODE_SPLITS)


def test_decode_plan_divides_the_context_into_32_key_steps_per_wave():
    for tokens in (1, 8, 64, 512):
        for nkv, group, hd in ((8, 4, 64), (1, 16, 128), (2, 3, 96), (5, 1, 32)):
            for capacity in (8, 64, 256, 300, 2304, 4096, 8192, 131072, 1 << 21):
                chunk, waves = hip.decode_plan(tokens, nkv, group, hd, capacity)
                assert 1 <= waves <= hip.decode_waves(hd, chunk == 32 * waves) and chunk % (32 * waves) == 0
                assert -(-capacity // chunk) <= hip.MAX_DECODE_SPLITS
                assert 4 * (32 * waves + waves * group * hd) <= 65536
    assert hip.decode_plan(8, 8, 4, 64, 2304) == (256, 8)          # one step per wave
    assert hip.decode_plan(8, 8, 4, 128, 2304) == (256, 8)         # wide heads too, where a wave has one step;
    assert hip.decode_plan(64, 8, 4, 64, 2304) == (2304, 8)        # a workgroup per compute unit: nothing to combine
    assert hip.decode_plan(64, 8, 4, 64, 32768) == (4096, 8)       # ... but not over a very long context
    assert hip.decode_plan(1, 8, 4, 64, 192) == (192, 6)           # short context: one workgroup
    assert hip.decode_plan(1, 8, 4, 64, 32768) == (1024, 8)        # long: 32 chunks of a token's 8 heads fill the chip
    assert hip.decode_plan(8, 8, 4, 128, 8192) == (2048, 4)        # four waves in the loop over several steps: 4 chunks for 64 (token, head) pairs
    assert hip.decode_plan(8, 8, 4, 128, 32768) == (4096, 4)       # chunks stay within 4,096 keys
    assert hip.decode_plan(4, 8, 4, 64, 8192) == (1024, 8)
    # workgroups in full rounds of one per compute unit: 384 that take everything leave a quarter of the chip idle
    assert hip.decode_plan(48, 8, 4, 128, 8192) == (4096, 4)       # 768 workgroups instead of 384
    assert hip.decode_plan(48, 8, 4, 128, 4096) == (256, 8)        # a short context: the one-step form instead
    assert hip.decode_plan(20, 8, 4, 128, 16384) == (2816, 4)      # 6 chunks of equal length: 960 workgroups, four rounds
    assert hip.decode_plan(12, 8, 4, 128, 8192) == (1664, 4)       # 5 chunks of equal length: 480 workgroups
    assert hip.decode_plan(31, 8, 4, 128, 8192) == (8192, 4)       # 248 workgroups are as good as 256
    assert hip.decode_plan(24, 8, 4, 64, 2304) == (2304, 8)        # and so are 192
    assert hip.decode_plan(80, 8, 4, 64, 2304) == (256, 8)         # 640 of 768 are not


def test_which_kernel_takes_a_projection_of_few_rows():
    """The row counts and shapes at which the 8-row form, the shared-x kernel and their fused
    epilogues are chosen (the thresholds are measured; this pins what the parts rely on)."""
    # 8-row form: up to 4 rows at any width, up to 8 rows for matrices of up to 2,048 rows; K in waves of 64 steps
    assert hip.skinny8_takes(1, 128256, 2048) and hip.skinny8_takes(4, 16384, 2048) and hip.skinny8_takes(8, 2048, 8192)
    assert not hip.skinny8_takes(8, 16384, 2048) and not hip.skinny8_takes(9, 2048, 2048) and not hip.skinny8_takes(1, 2048, 2000)
    for k in (256, 2048, 8192, 14336, 16384):
        steps = hip.skinny8_steps(k)
        assert steps in (4, 8, 16) and k % (64 * steps) == 0 and k // (64 * steps) <= 16
    assert hip.skinny8_steps(100) == 0
    # shared-x kernel: 33 to 64 rows (128 with the gate) against at least 8,192 rows of W in steps of 64, K in steps of 1,024
    assert hip.rows64_takes(33, 16384, 2048) and hip.rows64_takes(64, 128256, 2048) and hip.rows64_takes(40, 8192, 3072)
    assert hip.rows64_takes(65, 16384, 2048, glu=True) and hip.rows64_takes(128, 16384, 2048, glu=True)
    for rows, n, k in ((32, 16384, 2048), (65, 16384, 2048), (40, 4096, 2048), (40, 8200, 2048), (40, 16384, 2560)):
        assert not hip.rows64_takes(rows, n, k)
    assert not hip.rows64_takes(129, 16384, 2048, glu=True) and not hip.rows64_takes(32, 16384, 2048, glu=True)
    # the fused norm serves one block of 16 rows; the gate alone up to 64 rows over reductions of up to 2,048
    assert hip.skinny_fuses(16, 2048, True, True) and not hip.skinny_fuses(17, 2048, True, True)
    assert hip.skinny_fuses(64, 2048, False, True) and not hip.skinny_fuses(65, 2048, False, True)
    assert not hip.skinny_fuses(40, 4096, False, True)


def test_which_narrow_products_have_their_reduction_cut_into_slices():
    """The shared-x kernel with the reduction in slices: for weights too narrow to give every compute
    unit a workgroup of 64 rows; the fewest slices (multiples of 512 of k) that reach 192 workgroups."""
    assert hip.rows64_slices(64, 2048, 2048) == 4 and hip.rows64_slices(33, 2048, 8192) == 8 and hip.rows64_slices(9, 2048, 8192) == 8
    assert hip.rows64_slices(48, 3072, 3072) == 6 and hip.rows64_slices(8, 3072, 8192) == 4 and hip.rows64_slices(64, 4096, 14336) == 4
    for rows, n, k in ((4, 2048, 8192), (129, 2048, 8192), (64, 16384, 2048), (64, 2048, 2304), (64, 2000, 2048)):
        assert hip.rows64_slices(rows, n, k) == 0
    for n, k in ((64, 512), (2048, 8192), (3072, 3072), (4096, 14336), (4096, 4096)):
        s = hip.rows64_slices(40, n, k)
        assert 1 <= s <= 16 and k % (512 * s) == 0
        fewer = [t for t in range(1, s) if (k // 512) % t == 0]
        assert all((n // 64) * t < 192 for t in fewer), "a smaller number of slices would have filled the chip"
    # where the weight-streaming kernels serve a shape they come first: the o projection of up to 32 rows
    copies = hip.StreamingCopies(by16=object())
    assert hip._sliced_serves(32, 2048, 2048, copies) == 0 and hip._sliced_serves(33, 2048, 2048, copies) == 4
    assert hip._sliced_serves(8, 2048, 8192, copies) == 0 and hip._sliced_serves(9, 2048, 8192, copies) == 8
    assert hip._sliced_serves(40, 2048, 8192, None) == 0, "no packed copy: the library"
    assert hip._sliced_serves(24, 5120, 3072, copies) == 3 and hip._sliced_serves(24, 5120, 3072, copies, finishing=False) == 0
    assert hip._sliced_serves(24, 4096, 14336, copies, finishing=False) == 4
