"""Rules of the layouts that need no GPU to evaluate: how many column slices the kernel that holds x in LDS cuts a
matrix into (pure arithmetic in the library, callable without a device).  The reference has no counterpart; its
one kernel reads x from global memory (src/kernel/dcu/level2/mv/csrmv/dcu_gemv_vector.h:14-57)."""
import pytest

from alsparse_amd import capi

LDS = 163840  # bytes of x a compute unit's LDS holds


def _need(vs, n):
    fill = LDS // vs
    return (n + fill - 1) // fill


@pytest.mark.parametrize("dtype,vs", [(0, 4), (1, 8), (2, 8), (3, 16)], ids=["f32", "f64", "c64", "c128"])
def test_x_fits_one_fill_up_to_the_whole_lds(dtype, vs):
    lib = capi.load()
    assert lib.asamd_spmv_xlds_fits(dtype, LDS // vs) == 1
    assert lib.asamd_spmv_xlds_fits(dtype, LDS // vs + 1) == 0
    assert lib.asamd_spmv_xlds_fits(dtype, 0) == 0
    assert lib.asamd_xlds_slices(dtype, LDS // vs) == 1
    assert lib.asamd_xlds_slices(dtype, LDS // vs + 1) == 2


def test_slice_counts_hold_x_and_prefer_even_shares_of_the_compute_units():
    lib = capi.load()
    for vs, dtype in ((4, 0), (8, 1)):
        for n in (1, 1000, 40960, 40961, 70000, 100000, 131072, 262144, 300000, 524288, 1048576, 1200000, 5000000,
                  20000000, 41943040):
            s = lib.asamd_xlds_slices(dtype, n)
            need = _need(vs, n)
            assert need <= s <= max(need, (need * 5) // 4), (vs, n, s, need)  # at most a quarter more than needed
            assert s * (LDS // vs) >= n, "the slices do not hold x"
            if s != need:
                assert 256 % s == 0 and all(256 % t for t in range(need, s)), (vs, n, s, need)
    # the figures the measurements were taken with
    assert lib.asamd_xlds_slices(0, 262144) == 8      # 7 needed
    assert lib.asamd_xlds_slices(0, 1048576) == 32    # 26 needed
    assert lib.asamd_xlds_slices(0, 131072) == 4
    assert lib.asamd_xlds_slices(1, 100000) == 5      # nothing within a quarter divides 256
    assert lib.asamd_xlds_slices(0, 0) == 0 and lib.asamd_xlds_slices(9, 100) == 0
