"""Host only: the work the tile kernels' launches hand out, from the library's own planning
and mapping code (sonar_debug_tile_schedule / sonar_debug_moe_tile_schedule), checked against
what a GEMM needs: every output tile covered once, and its K steps covered once, by ranges the
wide kernel takes (whole passes of four steps)."""
import ctypes

import numpy as np
import pytest

from sonar_amd import _lib


def _rows(fn, *args):
    lib = _lib.load()
    n = getattr(lib, fn)(*args, None, 0)
    assert n >= 0, (fn, args, n)
    out = np.zeros((max(n, 1), 6), dtype=np.int32)
    got = getattr(lib, fn)(*args, out.ctypes.data_as(ctypes.c_void_p), n)
    assert got == n
    return out[:n]


def _check_cover(rows, tiles_by_rows, tiles_n, k_steps):
    """`tiles_by_rows`: {rows of a tile: set of row tiles that size must cover}.  Every (row tile,
    column tile) of every size gets [0, k_steps) exactly once; nothing else is worked on."""
    seen = {}
    for launch, tile_rows, tm, tn, k0, k1 in rows.tolist():
        assert tile_rows in tiles_by_rows and tm in tiles_by_rows[tile_rows], (tile_rows, tm)
        assert 0 <= tn < tiles_n and 0 <= k0 < k1 <= k_steps
        seen.setdefault((tile_rows, tm, tn), []).append((k0, k1))
    want = {(r, tm, tn) for r, tms in tiles_by_rows.items() for tm in tms for tn in range(tiles_n)}
    assert set(seen) == want
    for key, ranges in seen.items():
        ranges.sort()
        assert ranges[0][0] == 0 and ranges[-1][1] == k_steps, (key, ranges)
        for (a0, a1), (b0, b1) in zip(ranges, ranges[1:]):
            assert a1 == b0, (key, ranges)
        if len(ranges) > 1 and k_steps % 4 == 0:   # the wide kernel runs whole passes of four steps
            assert all((b - a) % 4 == 0 for a, b in ranges), (key, ranges)


LLAMA = {"qkv": (4096, 6144), "o": (4096, 4096), "gate_up": (4096, 28672), "down": (14336, 4096)}


def _check_dense(m, n, k, groups):
    """Returns what the call got: "none", "one launch" or "two launches"."""
    rows = _rows("sonar_debug_tile_schedule", m, n, k, groups)
    if len(rows) == 0:      # the call is not planned for the tile kernels (few rows on few strips)
        assert m <= 512
        return "none"
    tiles_n = (n + 255) // 256
    launches = sorted(set(rows[:, 0].tolist()))
    sizes = sorted(set(rows[:, 1].tolist()))
    if launches == [0]:
        assert len(sizes) == 1
        r = sizes[0]
        _check_cover(rows, {r: set(range((m + r - 1) // r))}, tiles_n, k // 64)
        return "one launch"
    # two launches: whole rounds of 256-row tiles, then the rest as 128-row tiles; every row of C is
    # covered by exactly one of the two sizes, per column tile
    assert launches == [0, 1] and sizes == [128, 256]
    assert np.all(rows[rows[:, 0] == 0][:, 1] == 256) and np.all(rows[rows[:, 0] == 1][:, 1] == 128)
    assert np.all(rows[:, 4] == 0) and np.all(rows[:, 5] == k // 64)     # nothing cut along K
    assert len(rows[rows[:, 0] == 0]) % 256 == 0                          # whole rounds of workgroups
    cover = np.zeros(((m + 127) // 128, tiles_n), dtype=np.int32)
    for _, r, tm, tn, _, _ in rows.tolist():
        if r == 256:
            cover[2 * tm:2 * tm + 2, tn] += 1
        else:
            cover[tm, tn] += 1
    assert np.all(cover == 1)
    return "two launches"


@pytest.mark.parametrize("m", [65, 100, 128, 200, 256, 300, 512, 1000, 1024, 2048, 3900, 4096, 5000, 8192])
@pytest.mark.parametrize("name", list(LLAMA))
def test_dense_launches_cover_every_tile_and_k_step_once(name, m):
    k, n = LLAMA[name]
    _check_dense(m, n, k, k // 128)


def test_dense_launches_of_random_shapes_cover_every_tile_and_k_step_once():
    """Seeded draws over rows, columns (multiples of 64), K (multiples of 64) and group sizes, small and
    large: one launch of either tile size, with and without ranges of K, and the two-launch form."""
    rng = np.random.default_rng(11)
    kinds = {}
    for i in range(600):
        if i % 2:
            m, n = int(rng.integers(65, 9000)), 64 * int(rng.integers(1, 513))
        else:
            m, n = int(rng.integers(65, 1200)), 64 * int(rng.integers(1, 100))
        k = 64 * int(rng.integers(1, 257))
        choices = [1] + [k // g for g in (32, 64, 128, 256) if k % g == 0 and k // g > 1]
        kind = _check_dense(m, n, k, int(rng.choice(choices)))
        kinds[kind] = kinds.get(kind, 0) + 1
    assert kinds.get("one launch", 0) > 100 and kinds.get("two launches", 0) > 10, kinds


def test_grouped_launches_of_random_shapes_cover_the_live_tiles_once():
    rng = np.random.default_rng(12)
    cut = 0
    for _ in range(600):
        max_row_tiles = int(rng.integers(1, 200))
        row_tiles = int(rng.integers(0, max_row_tiles + 1))
        n, k = 64 * int(rng.integers(1, 460)), 64 * int(rng.integers(1, 257))
        tile_rows, with_partial = int(rng.choice([256, 128])), int(rng.integers(0, 2))
        rows = _rows("sonar_debug_moe_tile_schedule", row_tiles, max_row_tiles, n, k, tile_rows, with_partial)
        if row_tiles == 0:
            assert len(rows) == 0
            continue
        _check_cover(rows, {tile_rows: set(range(row_tiles))}, (n + 255) // 256, k // 64)
        cut += bool(np.any(rows[:, 5] - rows[:, 4] != k // 64))
    assert cut > 5      # some of the draws are launches with tiles cut along K


def test_qkv_at_4096_rows_is_the_two_launch_case():
    rows = _rows("sonar_debug_tile_schedule", 4096, 6144, 4096, 32)
    assert sorted(set(rows[:, 0].tolist())) == [0, 1]
    assert (rows[:, 0] == 0).sum() == 256 and (rows[:, 0] == 1).sum() == 256


@pytest.mark.parametrize("tile_rows", [256, 128])
@pytest.mark.parametrize("with_partial", [0, 1])
@pytest.mark.parametrize("k,n", [(4096, 28672), (14336, 4096), (1024, 320), (2048, 256), (2880, 5760), (512, 4096)])
def test_grouped_launches_cover_the_live_tiles_once(k, n, with_partial, tile_rows):
    """Whatever number of row tiles the routing makes, up to the number the launch is sized for."""
    tiles_n = (n + 255) // 256
    max_row_tiles = 40
    split_seen = False
    for row_tiles in list(range(0, 41)):
        rows = _rows("sonar_debug_moe_tile_schedule", row_tiles, max_row_tiles, n, k, tile_rows, with_partial)
        if row_tiles == 0:
            assert len(rows) == 0
            continue
        _check_cover(rows, {tile_rows: set(range(row_tiles))}, tiles_n, k // 64)
        cut = np.any(rows[:, 5] - rows[:, 4] != k // 64)
        split_seen |= bool(cut)
        if not with_partial or k % 256 != 0 or k // 64 < 16:
            assert not cut                      # no room for partial tiles, or K does not allow whole passes
        if cut:   # few tiles, or a short last round of them on a long K: at most 256 workgroups on cut tiles
            tiles = row_tiles * tiles_n
            assert tiles < 256 or (tiles % 256 <= 128 and k // 64 >= 48)
            assert int((rows[:, 5] - rows[:, 4] != k // 64).sum()) <= 256
    if with_partial and k % 256 == 0 and k // 64 >= 16 and tiles_n * 40 >= 2:
        assert split_seen


def test_mixtral_down_at_4096_tokens_splits_its_last_round():
    # 36 row tiles x 16 column tiles = 576 = 2 rounds + 64 tiles, cut along K into 4 ranges of 56 steps
    rows = _rows("sonar_debug_moe_tile_schedule", 36, 136, 4096, 14336, 256, 1)
    whole = rows[rows[:, 5] - rows[:, 4] == 224]
    cut = rows[rows[:, 5] - rows[:, 4] != 224]
    assert len(whole) == 512 and len(cut) == 256
    assert set((cut[:, 5] - cut[:, 4]).tolist()) == {56}
    # without room for partial tiles: one workgroup per tile
    rows = _rows("sonar_debug_moe_tile_schedule", 36, 136, 4096, 14336, 256, 0)
    assert len(rows) == 576 and np.all(rows[:, 5] - rows[:, 4] == 224)


def test_schedule_rejects_arguments_out_of_range():
    lib = _lib.load()
    assert lib.sonar_debug_tile_schedule(0, 256, 256, 1, None, 0) == -1
    assert lib.sonar_debug_tile_schedule(256, 256, 100, 1, None, 0) == -1
    assert lib.sonar_debug_moe_tile_schedule(5, 4, 256, 256, 256, 0, None, 0) == -1
    assert lib.sonar_debug_moe_tile_schedule(1, 4, 256, 256, 64, 0, None, 0) == -1
