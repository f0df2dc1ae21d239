"""PowerSGD oracle: the three phases as the reference's comments state them
(powersgd_body.h:20-29, :41-50, :64-76), in numpy.

TEST INFRASTRUCTURE.  The reference has no CPU PowerSGD: its body is ATen calls
(torch::mm, geqrf, orgqr from PyTorch 1.3) whose literal `copy_` calls have
source and destination swapped, so nothing in the reference pins results for
this path: PARITY UNPINNED by the reference; the statement below is textbook
linear algebra evaluated in float64, and tests pin it through library routines
(numpy matmul, numpy.linalg.qr) and invariants.

Semantics (M is n x m, Q is m x r, P is n x r, N = grad.size <= n*m):
  encode1: M.flat[:N] = grad + residual  (fp32 add);  P = M @ Q
  encode2: P = orthonormal basis of P's columns (Gram-Schmidt order, i.e. the QR
           Q-factor with R's diagonal positive);  Q = M.T @ P
  decode:  M = P @ Q.T;  residual = grad - M.flat[:N];  grad = M.flat[:N]
"""
import numpy as np


def encode1(grad, residual, Q, M):
    """Returns (M_new float32 n x m, P float64 n x r)."""
    n_el = grad.size
    M_new = np.array(M, dtype=np.float32, copy=True)
    flat = M_new.reshape(-1)
    flat[:n_el] = (grad.reshape(-1).astype(np.float32) + residual.reshape(-1).astype(np.float32)).astype(np.float32)
    P = M_new.astype(np.float64) @ Q.astype(np.float64)
    return M_new, P


def orthogonalize(P):
    """Modified Gram-Schmidt in float64; a zero column stays zero."""
    P = np.array(P, dtype=np.float64, copy=True)
    for c in range(P.shape[1]):
        nrm = np.sqrt(np.sum(P[:, c] ** 2))
        if nrm > 0:
            P[:, c] /= nrm
        else:
            P[:, c] = 0
        for c2 in range(c + 1, P.shape[1]):
            P[:, c2] -= np.dot(P[:, c], P[:, c2]) * P[:, c]
    return P


def encode2(P, M):
    """Returns (P_orth float64, Q float64 m x r)."""
    Po = orthogonalize(P)
    return Po, M.astype(np.float64).T @ Po


def decode(P, Q, grad):
    """Returns (M float64 n x m, residual float64, grad_new float64) with grad's shape."""
    n_el = grad.size
    M = P.astype(np.float64) @ Q.astype(np.float64).T
    approx = M.reshape(-1)[:n_el].reshape(grad.shape)
    return M, grad.astype(np.float64) - approx, approx.copy()


def rel_fro(a, b):
    """||a-b||_F / ||b||_F."""
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    den = np.linalg.norm(b)
    return np.linalg.norm(a - b) / (den if den > 0 else 1.0)
