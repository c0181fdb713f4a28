"""What the host decides before a kernel is launched (no GPU): how a narrow product is cut
along K for the many-row tiled kernel, and how a decode step's keys are shared out among workgroups."""
import pytest

from xinfer_amd import kernels

SHAPES = [(6144, 4096), (4096, 4096), (4096, 12288), (7168, 5120), (5120, 5120), (5120, 17408), (10240, 5120),
          (5120, 8192), (5120, 25600), (4096, 1024), (1024, 2048), (1024, 3072), (24576, 4096), (1000, 2056), (48, 96)]


@pytest.mark.parametrize("N,K", SHAPES)
def test_tile_split_plan(N, K):
    """The slices are a power of two that divides K into multiples of 64, tiles x slices stay
    within the compute units, a slice keeps at least 512 of K, nothing is cut up to 128 or beyond
    1,024 rows, and beyond 256 rows only products with K >= 2 N."""
    for M in list(range(1, 1300, 7)) + [128, 129, 256, 257, 512, 513, 1024, 1025]:
        s, shape = kernels.tile_split_plan(M, N, K)
        assert s >= 1 and s & (s - 1) == 0 and shape in (0, 1)
        if s == 1:
            continue
        assert 128 < M <= 1024
        assert K % (s * 64) == 0 and N % 4 == 0
        assert K // s >= 512
        bm, bn = (256, 128) if shape == 1 else (128, 256)
        assert -(-M // bm) * -(-N // bn) * s <= 256
        assert M <= 256 or K >= 2 * N


def test_tile_split_plan_at_the_sizes_that_were_measured():
    table = {(256, 6144, 4096): (4, 1), (256, 4096, 4096): (8, 1), (256, 4096, 12288): (8, 1), (512, 4096, 12288): (4, 0),
             (768, 4096, 12288): (2, 0), (1024, 4096, 12288): (2, 0), (512, 4096, 4096): (1, 0), (512, 6144, 4096): (1, 0),
             (256, 7168, 5120): (4, 1), (256, 5120, 5120): (4, 1), (256, 5120, 17408): (4, 1), (256, 1024, 2048): (4, 1),
             (256, 1024, 3072): (4, 1), (192, 4096, 12288): (8, 1), (129, 4096, 4096): (8, 1), (200, 1000, 2056): (1, 0)}
    for (M, N, K), want in table.items():
        assert kernels.tile_split_plan(M, N, K) == want, (M, N, K)


@pytest.mark.parametrize("similar", [False, True])
def test_decode_keys_per_workgroup_is_a_multiple_of_128_and_covers_the_span(similar):
    for pairs in (1, 8, 64, 96, 256, 512, 2048):
        for span in (1, 100, 1024, 4096, 8704, 32768, 131072):
            kpw = kernels.decode_keys_per_workgroup(pairs, span, similar)
            assert kpw >= 128 and kpw % 128 == 0
            assert span // kpw + 1 <= 1025
