"""What the host decides before a kernel is launched (no GPU): how a narrow product is cut
along K for the many-row tiled kernel, and how a decode step's keys are shared out among workgroups."""
import pytest

from xinfer_amd import kernels

SHAPES = [(6144, 4096), (4096, 4096), (4096, 12288), (7168, 5120), (5120, 5120), (5120, 17408), (10240, 5120),
          (5120, 8192), (5120, 25600), (4096, 1024), (1024, 2048), (1024, 3072), (24576, 4096), (1000, 2056), (48, 96)]


@pytest.mark.parametrize("N,K", SHAPES)
def test_tile_split_plan(N, K):
    """Up to 16 slices of whole tiles of 64 k, the longest slice at least 512 of K, nothing is cut
    up to 128 or beyond 1,024 rows, beyond 256 rows only products with K >= 2 N, and never a weight
    of 8 MB or less."""
    for M in list(range(1, 1300, 7)) + [128, 129, 256, 257, 512, 513, 1024, 1025]:
        s, shape = kernels.tile_split_plan(M, N, K)
        assert 1 <= s <= 16 and shape in (0, 1, 2)
        if s == 1:
            continue
        assert 128 < M <= 1024
        assert K % 64 == 0 and N % 4 == 0
        assert -(-(K // 64) // s) * 64 >= 512 and N * K * 2 > 8 << 20
        assert M <= 256 or K >= 2 * N


def test_tile_split_plan_at_the_sizes_that_were_measured():
    table = {(256, 6144, 4096): (5, 1), (256, 4096, 4096): (6, 1), (256, 4096, 12288): (8, 1), (512, 4096, 12288): (8, 2), (768, 4096, 12288): (5, 2), (1024, 4096, 12288): (4, 2), (512, 4096, 4096): (1, 0), (512, 6144, 4096): (1, 0), (256, 7168, 5120): (4, 1), (256, 5120, 5120): (5, 1), (256, 5120, 17408): (6, 1), (256, 1024, 2048): (1, 0), (256, 1024, 3072): (1, 0), (192, 4096, 12288): (8, 1), (129, 4096, 4096): (8, 1), (200, 1000, 2056): (1, 0), (256, 5120, 25600): (6, 1), (512, 5120, 17408): (6, 2), (256, 10240, 5120): (3, 1)}
    for (M, N, K), want in table.items():
        assert kernels.tile_split_plan(M, N, K) == want, (M, N, K)


@pytest.mark.parametrize("similar", [False, True])
def test_decode_keys_per_workgroup_is_a_multiple_of_128_and_covers_the_span(similar):
    for pairs in (1, 8, 64, 96, 256, 512, 2048):
        for span in (1, 100, 1024, 4096, 8704, 32768, 131072):
            kpw = kernels.decode_keys_per_workgroup(pairs, span, similar)
            assert kpw >= 128 and kpw % 128 == 0
            assert span // kpw + 1 <= 1025


def test_decode_mixed_lengths_take_whole_sequences_where_there_are_many():
    assert kernels.decode_keys_per_workgroup(255, 4096, False) == 512
    assert kernels.decode_keys_per_workgroup(256, 4096, False) == 1024             # a pair a compute unit
    assert kernels.decode_keys_per_workgroup(256, 1024, False) == 512
    assert kernels.decode_keys_per_workgroup(383, 1024, False) == 512
    assert kernels.decode_keys_per_workgroup(384, 1024, False) == 1152             # one split: no second kernel
    assert kernels.decode_keys_per_workgroup(1536, 2048, False) == 2176
    assert kernels.decode_keys_per_workgroup(2048, 3072, False) == 2048
    assert kernels.decode_keys_per_workgroup(2048, 16384, False) == 2048
