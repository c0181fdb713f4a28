"""What the host decides before a kernel is launched (no GPU): how a narrow product is cut
along K for the library, and how a decode step's keys are shared out among workgroups."""
import pytest

from xinfer_amd import kernels

SHAPES = [(6144, 4096), (4096, 4096), (4096, 12288), (7168, 5120), (5120, 5120), (5120, 17408), (10240, 5120),
          (5120, 8192), (5120, 25600), (4096, 1024), (1024, 2048), (1024, 3072), (24576, 4096), (1000, 2056), (48, 96)]


@pytest.mark.parametrize("N,K", SHAPES)
def test_library_split_slices(N, K):
    """The slices are a power of two that divides K into multiples of 64, tiles x slices stay
    within the compute units, a slice keeps at least 1,024 of K (2,048 beyond 512 rows), nothing
    is cut up to 128 or beyond 1,024 rows, and beyond 256 rows only products with K >= 2 N."""
    for M in list(range(1, 1300, 7)) + [128, 129, 256, 257, 512, 513, 1024, 1025]:
        s = kernels.library_split_slices(M, N, K)
        assert s >= 1 and s & (s - 1) == 0
        if s == 1:
            continue
        assert 128 < M <= 1024
        assert K % (s * 64) == 0
        assert K // s >= (1024 if M <= 512 else 2048)
        assert -(-M // 256) * -(-N // 256) * s <= 256
        assert M <= 256 or K >= 2 * N


def test_library_split_slices_at_the_sizes_that_were_measured():
    table = {(256, 6144, 4096): 4, (256, 4096, 4096): 4, (256, 4096, 12288): 8, (512, 4096, 12288): 8,
             (768, 4096, 12288): 4, (1024, 4096, 12288): 4, (512, 4096, 4096): 1, (512, 6144, 4096): 1,
             (256, 7168, 5120): 4, (256, 5120, 5120): 4, (256, 5120, 17408): 8, (256, 1024, 2048): 2,
             (256, 1024, 3072): 2, (256, 4096, 1024): 1, (192, 4096, 12288): 8, (129, 4096, 4096): 4}
    for (M, N, K), want in table.items():
        assert kernels.library_split_slices(M, N, K) == want, (M, N, K)


@pytest.mark.parametrize("similar", [False, True])
def test_decode_keys_per_workgroup_is_a_multiple_of_128_and_covers_the_span(similar):
    for pairs in (1, 8, 64, 96, 256, 512, 2048):
        for span in (1, 100, 1024, 4096, 8704, 32768, 131072):
            kpw = kernels.decode_keys_per_workgroup(pairs, span, similar)
            assert kpw >= 128 and kpw % 128 == 0
            assert span // kpw + 1 <= 1025
