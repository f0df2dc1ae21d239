"""Pins the numpy PowerSGD oracle (CPU only) through library routines and
invariants.  The reference holds no CPU PowerSGD and no test for it (its body
is ATen calls with swapped copy_ arguments): parity with the reference itself
is unpinned; the oracle is the comments' linear algebra in float64."""
import numpy as np
import pytest

from oracle import powersgd as ps


@pytest.mark.parametrize("n,m,r", [(64, 48, 4), (128, 256, 1), (100, 37, 3), (257, 129, 8)])
def test_orthogonalize_equals_qr_up_to_column_sign(n, m, r):
    rng = np.random.default_rng(n + m)
    P = rng.normal(0, 1, (n, r))
    Po = ps.orthogonalize(P)
    assert np.linalg.norm(Po.T @ Po - np.eye(r)) < 1e-12
    Qh, Rh = np.linalg.qr(P)                      # Householder (LAPACK geqrf/orgqr), as the reference calls it
    sign = np.sign(np.diag(Rh))
    np.testing.assert_allclose(Po, Qh * sign, atol=1e-12)
    # same column space: projector equality is sign-free
    np.testing.assert_allclose(Po @ Po.T, Qh @ Qh.T, atol=1e-12)


def test_orthogonalize_rank_deficient_column_stays_zero():
    P = np.zeros((16, 3)); P[:, 0] = 1.0; P[:, 2] = np.arange(16)
    Po = ps.orthogonalize(P)
    assert np.all(Po[:, 1] == 0)
    assert abs(Po[:, 0] @ Po[:, 2]) < 1e-14


@pytest.mark.parametrize("n,m,r,pad", [(64, 48, 4, 0), (33, 20, 2, 7), (128, 64, 4, 64)])
def test_phases_and_invariants(n, m, r, pad):
    rng = np.random.default_rng(n)
    numel = n * m - pad
    grad = rng.normal(0, 1e-2, numel).astype(np.float32)
    res = rng.normal(0, 1e-3, numel).astype(np.float32)
    Q = rng.normal(0, 1, (m, r)).astype(np.float32)
    M0 = rng.normal(0, 1, (n, m)).astype(np.float32)
    M, P = ps.encode1(grad, res, Q, M0)
    assert np.array_equal(M.reshape(-1)[:numel], grad + res)          # fp32 add, flat prefix
    assert np.array_equal(M.reshape(-1)[numel:], M0.reshape(-1)[numel:])  # padding untouched
    np.testing.assert_allclose(P, np.einsum("ik,kj->ij", M.astype(np.float64), Q.astype(np.float64)), rtol=1e-12, atol=1e-14)
    Po, Qn = ps.encode2(P, M)
    assert np.linalg.norm(Po.T @ Po - np.eye(r)) < 1e-10
    np.testing.assert_allclose(Qn, M.astype(np.float64).T @ Po, rtol=1e-12)
    Mn, Rn, Gn = ps.decode(Po, Qn, grad)
    # P P^T M is the orthogonal projection of M onto span(P)
    np.testing.assert_allclose(Mn, Po @ (Po.T @ M.astype(np.float64)), atol=1e-12)
    np.testing.assert_allclose(Gn + Rn, grad.astype(np.float64), atol=1e-15)   # grad_new + residual_new == grad_old
    assert ps.rel_fro(Mn, M) <= 1.0 + 1e-12                                      # a projection never grows the norm


def test_rank_r_matrix_is_reproduced_exactly():
    # if M has rank r and Q spans its row space, one power iteration returns M itself
    rng = np.random.default_rng(2)
    n, m, r = 96, 80, 4
    U, V = rng.normal(0, 1, (n, r)), rng.normal(0, 1, (m, r))
    Mtrue = (U @ V.T).astype(np.float32)
    grad = Mtrue.reshape(-1).copy(); res = np.zeros_like(grad)
    Q = rng.normal(0, 1, (m, r)).astype(np.float32)
    M, P = ps.encode1(grad, res, Q, np.zeros((n, m), np.float32))
    Po, Qn = ps.encode2(P, M)
    Mn, Rn, Gn = ps.decode(Po, Qn, grad)
    assert ps.rel_fro(Mn, Mtrue) < 1e-6
    assert np.linalg.norm(Rn) < 1e-5 * np.linalg.norm(grad)
