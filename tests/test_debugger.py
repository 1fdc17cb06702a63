"""Host-side replay of the kernels' index arithmetic (kernl_amd/debugger): runs on the CPU, over the address functions
the kernels themselves are compiled from (csrc/index_math.h through libkernl_index.so)."""
import numpy as np
import pytest

from kernl_amd.debugger import Lds, index_lib
from kernl_amd.debugger.attention_replay import check_mask_tile, check_tile, replay_tile
from kernl_amd.debugger.linear_replay import check_weight_placement, lane_columns
from kernl_amd.debugger.wave_ops import mfma32, transposing_read_b64


def test_lds_model_counts_bank_conflicts():
    lds = Lds(64 * 1024)
    data = [bytes(16)] * 64
    lds.wave_write([16 * lane for lane in range(64)], data, 16, "contiguous")
    assert lds.writes.passes == 4 and lds.writes.conflict_free          # 1 KB, 16 lanes per pass
    assert lds.once_written(0, 1024) and not lds.once_written(0, 1040)
    lds.wave_read([16 * lane for lane in range(64)], 16, "contiguous")
    assert lds.reads.conflict_free
    rows = Lds(64 * 1024)
    rows.wave_write([256 * lane for lane in range(64)], data, 16, "same banks")  # 256-byte stride: one bank group for all
    assert rows.writes.passes == 4 and rows.writes.cycles == 4 * 16 and rows.writes.worst == 16
    same = Lds(1024)
    same.wave_write([0] * 64, [bytes(4)] * 64, 4, "x")
    same.wave_read([0] * 64, 4, "broadcast")                            # one dword for everybody is no conflict
    assert same.reads.conflict_free
    with pytest.raises(ValueError, match="nothing has written"):
        same.wave_read([512] * 64, 4, "unwritten")
    with pytest.raises(IndexError):
        same.wave_read([1024] * 64, 4, "outside")
    with pytest.raises(ValueError, match="aligned"):
        same.wave_read([2] * 64, 4, "misaligned")


def test_mfma_and_transposing_read_models():
    rng = np.random.default_rng(1)
    a, b = rng.standard_normal((32, 16)), rng.standard_normal((32, 16))   # A rows x k, B columns x k
    to_frags = lambda m: np.stack([m[lane % 32, 8 * (lane // 32):8 * (lane // 32) + 8] for lane in range(64)])
    d = mfma32(to_frags(a), to_frags(b), np.zeros((64, 16)))
    want = a @ b.T
    for lane in range(64):
        for v in range(16):
            assert d[lane, v] == pytest.approx(want[8 * (v // 4) + 4 * (lane // 32) + v % 4, lane % 32])
    # transposing read: a 16-lane group addresses 4 keys x 16 features (lane i: key i / 4, features 4 (i % 4) ..) and
    # lane i gets feature i of the 4 keys
    lds = Lds(4 * 16 * 2 * 4)
    block = np.arange(4 * 4 * 16, dtype=np.uint16).reshape(4, 4, 16)      # [group, key, feature]
    lds.wave_write([8 * lane for lane in range(64)],
                   [block[lane // 16, (lane % 16) // 4, 4 * (lane % 4):4 * (lane % 4) + 4].tobytes() for lane in range(64)], 8, "fill")
    got = transposing_read_b64(lds, [8 * lane for lane in range(64)])
    for lane in range(64):
        assert got[lane].tolist() == block[lane // 16, :, lane % 16].tolist()


@pytest.mark.parametrize("head_size", [64, 128])
def test_attention_tile_replay(head_size):
    """Every score and output register of the four waves holds what the mathematics wants, the tiles are staged exactly
    once, and neither the K fragment reads nor the transposing V reads have bank conflicts."""
    rng = np.random.default_rng(head_size)
    q, k, v = (rng.standard_normal((n, head_size)).astype(np.float16) for n in (128, 64, 64))
    r = check_tile(q, k, v)
    assert r.writes.conflict_free and r.reads.conflict_free
    per_wave = (64 // 32) * (head_size // 16)
    assert r.reads.by_tag["K fragment"][0] == 4 * per_wave * 4            # 4 waves, 4 passes per 16-byte read
    assert r.reads.by_tag["V fragment"][0] == 4 * (64 // 16) * (head_size // 32) * 2 * 2


def test_attention_replay_catches_a_wrong_layout(monkeypatch):
    """The check is not vacuous: the same replay over a staging rule with the swizzle left out fails."""
    from kernl_amd.debugger import attention_replay, index_lib as get

    real = get()

    class Broken:
        def __getattr__(self, name):
            return getattr(real, name)

        def attention(self, head_size, what, a, b=0, c=0):
            if what == "k_stage_chunk":
                return a % (head_size // 8)                               # row-major, unswizzled
            return real.attention(head_size, what, a, b, c)

    monkeypatch.setattr(attention_replay, "index_lib", lambda: Broken())
    rng = np.random.default_rng(3)
    q, k, v = (rng.standard_normal((n, 64)).astype(np.float16) for n in (128, 64, 64))
    with pytest.raises(AssertionError, match="score register"):
        check_tile(q, k, v)


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_matrix_mask_staging_replay(dtype):
    rng = np.random.default_rng(5)
    lds = check_mask_tile(rng.standard_normal((32, 64)).astype(dtype))
    assert lds.writes.conflict_free
    if dtype == np.float32:
        assert lds.reads.conflict_free
    else:
        # 8-byte reads of 128-byte rows: the two 8-byte halves of a chunk belong to the two lane halves, and a pass
        # serves one lane half — 32 lanes share the 16 half-chunks a pass can reach: two cycles per pass, no more
        assert lds.reads.cycles == 2 * lds.reads.passes and lds.reads.worst == 2


@pytest.mark.parametrize("layout", ["256", "192", "gated"])
def test_wide_linear_weight_placement(layout):
    check_weight_placement(layout)
    cols = lane_columns(layout, 192 if layout == "192" else 256)
    if layout == "256":
        # lane l16: columns 8 l16 .. 8 l16 + 7 of each wave's 128 — 16 lanes cover the 256 contiguous bytes of a row
        assert cols[0] == [list(range(8)), list(range(128, 136))] and cols[15][1] == list(range(248, 256))
    if layout == "192":
        assert cols[0] == [list(range(6)), list(range(96, 102))] and cols[3][0] == list(range(18, 24))
    if layout == "gated":
        # lane 9: output columns 36 .. 39 of the wave's 64 = second 32-column group: gate rows 64 + 4 .., value rows 96 + 4 ..
        assert cols[9][0] == [68, 69, 70, 71, 100, 101, 102, 103]


def test_index_functions_known_values():
    ix = index_lib()
    assert [ix.rowperm16(i) for i in range(8)] == [0, 1, 2, 3, 16, 17, 18, 19]
    assert sorted(ix.rowperm16(i) for i in range(32)) == list(range(32))
    # 128-byte rows: chunk XOR (row / 2) % 8
    assert ix.swz_offset(128, 0, 3) == 48 and ix.swz_offset(128, 2, 3) == 2 * 128 + (3 ^ 1) * 16
    with pytest.raises(ValueError):
        ix.swz_offset(96, 0, 0)
    with pytest.raises(ValueError):
        ix.attention(80, "stage_row", 0)


@pytest.mark.parametrize("row_blocks, units_per_stage", [(1, 4), (2, 2), (4, 2), (8, 2)])
def test_few_row_stage_of_x_is_written_once_and_read_without_conflicts(row_blocks, units_per_stage):
    """The stream-K few-row linear kernel's x stage, replayed from the kernel's own index functions: the 512 threads'
    16-byte stores cover a stage exactly once, every lane's fragment reads return k = 16 g + 8 s .. + 7 of row
    16 mb + r of the unit (what `v_mfma_f32_16x16x32` expects on its B side), and no store or read conflicts on banks."""
    from kernl_amd.debugger.fewrow_replay import replay_stage

    writes, reads = replay_stage(row_blocks, units_per_stage)
    assert writes.conflict_free, (writes.passes, writes.cycles)
    assert reads.conflict_free, (reads.passes, reads.cycles)
    assert reads.instructions == units_per_stage * row_blocks * 2


@pytest.mark.parametrize("rows", [16, 32, 64])
def test_small_problem_tile_is_loaded_once_and_read_without_conflicts(rows):
    """An operand tile of the small-problem linear kernels, replayed from the kernels' own index functions: the direct-to-LDS
    loads bring every (row, chunk) of the tile exactly once, every lane's fragment reads return k = 32 s + 8 g .. + 7 of
    row 16 b + r (what `v_mfma_f32_16x16x32` expects of either operand), and no read conflicts on banks."""
    from kernl_amd.debugger.small_replay import replay_tile

    reads = replay_tile(rows)
    assert reads.conflict_free, (reads.passes, reads.cycles)
    assert reads.instructions == rows // 16 * 2


@pytest.mark.parametrize("n", [1, 7, 8, 9, 50, 192, 255, 256])
def test_small_problem_tiles_of_an_xcd_are_one_contiguous_run(n):
    """Workgroup b runs on XCD b % 8.  The small-problem kernels' workgroup -> tile map is a bijection, and the tiles of
    the workgroups of one XCD, taken in launch order, are consecutive indices — so the tiles that share a weight tile
    (consecutive indices) meet in one L2."""
    from kernl_amd.debugger.index_lib import index_lib

    ix = index_lib()
    tiles = [ix.xcd_contiguous(b, n) for b in range(n)]
    assert sorted(tiles) == list(range(n))
    runs = [[tiles[b] for b in range(x, n, 8)] for x in range(8)]
    assert all(run == list(range(run[0], run[0] + len(run))) for run in runs if run)
    starts = [run[0] for run in runs if run]
    assert starts == sorted(starts)

