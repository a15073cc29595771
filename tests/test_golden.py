"""The oracle against the committed outputs of the reference's own CPU code
(tests/golden/reference_kernels.npz, produced by tests/golden/make_golden.py from the
reference sources compiled with gcc -O2 -ffp-contract=off).  Bit-exact: the oracle
restates the same loops in the same order.  Runs wherever the repository is, with or
without the reference tree."""
import os

import numpy as np
import pytest

from alsparse_amd import workloads as wl
from oracle import oracle as orc
from golden_cases import golden_complex_matrices, golden_matrices
from helpers_shapes import complex_vector

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "reference_kernels.npz"), allow_pickle=False)
CASES = golden_matrices()
CX_CASES = golden_complex_matrices()


@pytest.mark.parametrize("key", sorted(CASES))
def test_oracle_reproduces_reference_outputs_bit_for_bit(key):
    a = CASES[key]
    x, y0 = wl.uniform(a.cols, a.dtype, 3), wl.uniform(a.rows, a.dtype, 4)
    assert np.array_equal(orc.csrmv_plain(a, 2.0, x, 3.0, y0), GOLD[key + ".mv_plain"])
    assert np.array_equal(orc.csrmv_plain(a, 1.0, x, 0.0, y0), GOLD[key + ".mv_plain_beta0"])
    assert np.array_equal(orc.csrmv_omp(a, 2.0, x, 3.0, y0, threads=4, fast=False), GOLD[key + ".mv_omp4"])
    n = 4
    B = wl.uniform(a.cols * n, a.dtype, 5).reshape(a.cols, n)
    C0 = wl.uniform(a.rows * n, a.dtype, 4).reshape(a.rows, n)
    assert np.array_equal(orc.csrmm_plain(a, 1.5, B, 0.5, C0), GOLD[key + ".mm_row_plain"])
    col = orc.csrmm_plain(a, 1.5, np.asfortranarray(B), 0.5, np.asfortranarray(C0), layout="col")
    assert np.array_equal(np.ascontiguousarray(col), GOLD[key + ".mm_col_plain"])
    assert np.array_equal(orc.csr2coo(a), GOLD[key + ".coo_rows"])
    assert np.array_equal(orc.coomv_plain(a, orc.csr2coo(a), 2.0, x, 3.0, y0), GOLD[key + ".coomv_plain"])
    xt, yt = wl.uniform(a.rows, a.dtype, 3), wl.uniform(a.cols, a.dtype, 4)
    assert np.array_equal(orc.csrmv_trans_plain(a, 2.0, xt, 3.0, yt), GOLD[key + ".mv_trans_plain"])
    assert orc.csr2ell_width(a) == int(GOLD[key + ".ell_ld"][0])
    ev, ec = orc.csr2ell(a)
    assert np.array_equal(ev, GOLD[key + ".ell_val"]) and np.array_equal(ec, GOLD[key + ".ell_col"])


@pytest.mark.parametrize("key", sorted(CX_CASES))
def test_complex_oracle_reproduces_reference_outputs_bit_for_bit(key):
    """The reference's plain kernels compiled with -DCOMPLEX [-DDOUBLE]: A, A^T, A^H, SpMM, COO."""
    a = CX_CASES[key]
    al, be = 1.25 - 0.5j, 0.5 + 0.75j
    x, y0 = complex_vector(a.cols, a.dtype, 3), complex_vector(a.rows, a.dtype, 4)
    xt, yt = complex_vector(a.rows, a.dtype, 5), complex_vector(a.cols, a.dtype, 6)
    assert np.array_equal(orc.csrmv_plain(a, al, x, be, y0), GOLD[key + ".mv_plain"])
    assert np.array_equal(orc.csrmv_trans_plain(a, al, xt, be, yt), GOLD[key + ".mv_trans_plain"])
    assert np.array_equal(orc.csrmv_trans_plain(a, al, xt, be, yt, conj=True), GOLD[key + ".mv_conj_plain"])
    n = 3
    B = complex_vector(a.cols * n, a.dtype, 7).reshape(a.cols, n)
    C0 = complex_vector(a.rows * n, a.dtype, 8).reshape(a.rows, n)
    assert np.array_equal(orc.csrmm_plain(a, al, B, be, C0), GOLD[key + ".mm_row_plain"])
    col = orc.csrmm_plain(a, al, np.asfortranarray(B), be, np.asfortranarray(C0), layout="col")
    assert np.array_equal(np.ascontiguousarray(col), GOLD[key + ".mm_col_plain"])
    assert np.array_equal(orc.coomv_plain(a, orc.csr2coo(a) - a.base, al, x, be, y0), GOLD[key + ".coomv_plain"])
    # the transposed and the conjugate-transposed outputs differ: the fixture can tell them apart
    assert not np.array_equal(GOLD[key + ".mv_trans_plain"], GOLD[key + ".mv_conj_plain"])


def test_padding_convention_of_the_reference_converter():
    """convert_ell_?_coo pads with value 0 and index 0 and lays slots out column-major."""
    a = CASES["s.empty_rows"]
    ld = int(GOLD["s.empty_rows.ell_ld"][0])
    ev, ec = GOLD["s.empty_rows.ell_val"], GOLD["s.empty_rows.ell_col"]
    assert ld == 7 and ev.shape == (ld * a.rows,)
    lens = np.diff(a.row_ptr)
    for r in range(a.rows):
        for s in range(ld):
            if s >= lens[r]:
                assert ev[s * a.rows + r] == 0 and ec[s * a.rows + r] == 0
            else:
                assert ec[s * a.rows + r] == a.col_ind[a.row_ptr[r] + s]
