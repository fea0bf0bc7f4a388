"""How products of few rows are dealt to the compute units (``ops.wide_plan``, ``ops.wide_waves``, ``ops.rows_plan``):
plain arithmetic on sizes, so it runs without a GPU when the number of compute units is given."""
import pytest

from nanospec_amd.kernels import ops

UNITS = 256  # an MI355X


def busiest(tiles: int, per_group: int, ksplit: int, units: int = UNITS) -> int:
    """Row tiles times ranges' share that the busiest unit streams when groups of tiles go round the units in turn."""
    groups = -(-tiles // per_group) * ksplit
    return -(-groups // units) * per_group


@pytest.mark.parametrize("n,k", [(6144, 4096), (4096, 4096), (4096, 14336), (3072, 2048), (2048, 2048), (2048, 8192), (10240, 8192), (200, 264)])
def test_one_matrix_takes_the_form_that_leaves_the_busiest_unit_least(n, k):
    ksplit, nt = ops.wide_plan(n, k, 64, units=UNITS)
    waves, halves = ops.wide_waves(n, k, 64, ksplit, nt, units=UNITS)
    assert not halves and waves in (3, 4) and 1 <= ksplit <= 16 and ksplit <= max(1, -(-k // 128) // 4)
    if nt == 1:
        k_tiles = -(-k // 128)
        cost = lambda w: busiest(-(-n // 16), w, ksplit) * -(-k_tiles // ksplit)
        assert cost(waves) == min(cost(3), cost(4))
        assert waves == 4 or cost(3) < cost(4)  # three waves only where they gain


def test_the_shapes_of_the_benchmark():
    assert ops.wide_plan(6144, 4096, 64, units=UNITS) == (2, 1) and ops.wide_waves(6144, 4096, 64, 2, 1, units=UNITS) == (3, False)
    assert ops.wide_plan(4096, 14336, 64, units=UNITS) == (4, 1) and ops.wide_waves(4096, 14336, 64, 4, 1, units=UNITS) == (4, False)
    # gate and up: 1,792 half tiles are 7 for each of 256 units; 1,024 are 4 for each; 448 workgroups of whole tiles fill the GPU
    assert ops.wide_waves(14336, 4096, 64, 1, 1, gated=True, units=UNITS) == (7, True)
    assert ops.wide_waves(8192, 2048, 64, 1, 1, gated=True, units=UNITS) == (4, True)
    assert ops.wide_waves(28672, 8192, 64, 1, 1, gated=True, units=UNITS) == (4, False)


def test_what_each_form_is_kept_for():
    assert ops.wide_waves(14336, 4096, 100, 1, 1, units=UNITS) == (4, False)             # more than 64 rows of one matrix
    assert ops.wide_waves(14336, 4096, 100, 1, 1, gated=True, units=UNITS) == (7, True)  # ... of gate and up: half tiles only
    assert ops.wide_waves(14336, 4096, 64, 2, 1, gated=True, units=UNITS) == (4, False)  # gate and up over ranges: whole tiles
    assert ops.wide_waves(128256, 4096, 64, 1, 2, units=UNITS) == (4, False)             # two tiles a wave
    # another GPU: 304 units are dealt 1,792 half tiles as 6 each in workgroups of ... the forms at hand, whichever is least
    waves, halves = ops.wide_waves(14336, 4096, 64, 1, 1, gated=True, units=304)
    assert (waves, halves) in ((4, False), (7, True), (4, True))


def test_many_rows_in_blocks():
    ksplit, nt = ops.rows_plan(8192, 8192, 2048, units=UNITS)
    assert nt == 4 and ksplit == 1  # 32 groups of row tiles times 16 blocks of rows fill the GPU without cutting K
    ksplit, nt = ops.rows_plan(4096, 14336, 130, gated=False, units=UNITS)
    assert nt == 4 and ksplit >= 2
