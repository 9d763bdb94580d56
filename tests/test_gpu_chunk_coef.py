"""The in-kernel generator of the chunkwise rule's gate coefficients (csrc/chunk_coef.h: block
scans of 2x2 triangular maps, no table in HBM) against the defining recurrences of
chunkwise_mm.hip evaluated in float64 on the host: c, bb, r from both tile orders and every
vector, for full and short chunks, random, constant and saturated gates."""
import numpy as np
import pytest
import torch

from nl_hecate_amd.ffi import lib
from tests.gpu_util import dev, host, zeros

pytestmark = pytest.mark.gpu


def host_coefficients(al, th, et, L):
    keep, eta = 1.0 - al.astype(np.float64), et.astype(np.float64)
    c, bb, r = np.zeros((64, 64)), np.zeros((64, 64)), np.zeros((64, 64))
    for j in range(L):
        b = cc = rr = 1.0
        for t in range(j, L):
            if t > j:
                b *= eta[t]
                rr *= keep[t]
                cc = keep[t] * cc + b
            c[t, j], bb[t, j], r[t, j] = cc, b, rr
    a, beta, h = np.zeros(64), np.zeros(64), np.zeros(64)
    av, hv, bv = 1.0, 1.0, 0.0
    for t in range(L):
        av *= keep[t]
        hv *= eta[t]
        bv = keep[t] * bv + hv
        a[t], beta[t], h[t] = av, bv, hv
    return c, bb, r, a, beta, h


CASES = [("random", 64), ("random", 37), ("random", 1), ("random", 16), ("random", 17), ("const", 64),
         ("saturated", 64), ("saturated", 50), ("delta", 64)]


@pytest.mark.parametrize("kind,L", CASES)
def test_generated_coefficients_match_the_recurrences(kind, L):
    rs = np.random.default_rng(L * 7 + len(kind))
    sig = lambda x: 1 / (1 + np.exp(-x))
    al, th, et = (sig(rs.standard_normal(64)).astype(np.float32) for _ in range(3))
    if kind == "const":
        al[:], th[:], et[:] = 0.05, 0.01, 0.9
    if kind == "saturated":   # exact zeros and ones at block edges, inside blocks and in runs
        for t in (0, 15, 16, 31, 40, 41, 42, 63):
            al[t] = 1.0
        for t in (3, 16, 47, 48, 49):
            et[t] = 0.0
        al[20:24] = 0.0
        et[5:9] = 1.0
        th[10] = 0.0
    if kind == "delta":
        et[:] = 0.0
    tj, jt, vecs = zeros(3, 64, 64), zeros(3, 64, 64), zeros(10, 64)
    assert lib.nlh_selftest_chunk_coef(dev(al).data_ptr(), dev(th).data_ptr(), dev(et).data_ptr(), L,
                                       tj.data_ptr(), jt.data_ptr(), vecs.data_ptr()) == 0
    torch.cuda.synchronize()
    tj, jt, vecs = host(tj), host(jt), host(vecs)
    c, bb, r, a, beta, h = host_coefficients(al, th, et, L)
    tol = dict(rtol=2e-5, atol=1e-30)
    for name, want, i in (("c", c, 0), ("bb", bb, 1), ("r", r, 2)):
        np.testing.assert_allclose(tj[i], want, err_msg=f"{name} token-major", **tol)
        np.testing.assert_allclose(jt[i], want, err_msg=f"{name} source-major", **tol)
    pad = lambda x: np.concatenate([x[:L], np.full(64 - L, x[L - 1])])
    np.testing.assert_allclose(vecs[0], pad(a), err_msg="a", **tol)
    np.testing.assert_allclose(vecs[1], pad(beta), err_msg="beta", **tol)
    np.testing.assert_allclose(vecs[2], pad(h), err_msg="h", **tol)
    z = lambda x: np.concatenate([x[:L], np.zeros(64 - L)])
    np.testing.assert_allclose(vecs[3][:L], c[L - 1, :L], err_msg="cl", **tol)
    np.testing.assert_allclose(vecs[4][:L], bb[L - 1, :L], err_msg="bl", **tol)
    np.testing.assert_allclose(vecs[5][:L], r[L - 1, :L], err_msg="rl", **tol)
    np.testing.assert_allclose(vecs[8], z(th), err_msg="theta", **tol)
    np.testing.assert_allclose(vecs[9][:3], [a[L - 1], beta[L - 1], h[L - 1]], err_msg="a_L beta_L h_L", **tol)


@pytest.mark.parametrize("kind,L", CASES)
def test_prepass_helpers_match_the_recurrences(kind, L):
    """coef_vectors and coef_table_columns (what cw_coef_kernel / cw_coef_bwd_kernel are made of) on one chunk."""
    rs = np.random.default_rng(L * 11 + len(kind))
    sig = lambda x: 1 / (1 + np.exp(-x))
    al, th, et = (sig(rs.standard_normal(64)).astype(np.float32) for _ in range(3))
    if kind == "const":
        al[:], th[:], et[:] = 0.05, 0.01, 0.9
    if kind == "saturated":
        for t in (0, 15, 16, 31, 40, 41, 42, 63):
            al[t] = 1.0
        for t in (3, 16, 47, 48, 49):
            et[t] = 0.0
        al[20:24] = 0.0
        et[5:9] = 1.0
        th[10] = 0.0
    if kind == "delta":
        et[:] = 0.0
    table, scaled, vecs = zeros(64, 64), zeros(64, 64), zeros(5, 64)
    assert lib.nlh_selftest_chunk_coef_prepass(dev(al).data_ptr(), dev(th).data_ptr(), dev(et).data_ptr(), L,
                                               table.data_ptr(), scaled.data_ptr(), vecs.data_ptr()) == 0
    torch.cuda.synchronize()
    table, scaled, vecs = host(table), host(scaled), host(vecs)
    c, bb, r, a, beta, h = host_coefficients(al, th, et, L)
    tol = dict(rtol=2e-5, atol=1e-30)
    np.testing.assert_allclose(table, c, err_msg="c", **tol)
    np.testing.assert_allclose(scaled, -th.astype(np.float64)[None, :] * c, err_msg="-theta c", **tol)
    pad = lambda x: np.concatenate([x[:L], np.full(64 - L, x[L - 1])])
    np.testing.assert_allclose(vecs[0], pad(a), err_msg="a", **tol)
    np.testing.assert_allclose(vecs[1], pad(beta), err_msg="beta", **tol)
    np.testing.assert_allclose(vecs[2], pad(h), err_msg="h", **tol)
    np.testing.assert_allclose(vecs[3][:L], c[L - 1, :L], err_msg="cl", **tol)
    np.testing.assert_allclose(vecs[4][:L], bb[L - 1, :L], err_msg="bl", **tol)
