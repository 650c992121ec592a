"""SO(3) helpers for the steerable kernel basis: ZYZ Euler rotations, real
spherical harmonics, real Wigner-D matrices and the intertwiner Q_J
(reference: ss_conv/utils/SO3.py).

The reference takes its spherical harmonics and Wigner-D matrices from the
third-party package lie_learn (utils/SO3.py:71,90).  This module computes them
itself, in float64:

* real spherical harmonics Y_l^m, m = -l..l, orthonormal on the sphere
  ("quantum" normalisation), sin(|m| phi) for m < 0 and cos(m phi) for m > 0,
  all leading coefficients positive, so that Y_1 is proportional to (y, z, x)
  and Y_2 to (xy, yz, 3z^2 - r^2, xz, x^2 - y^2) -- the bases the reference's
  own change-of-basis matrices assume (utils/SO3.py:282-292, 304-335);
* D^l(R) defined by Y_l(R x) = D^l(R) Y_l(x)  (utils/SO3.py:360-383), obtained
  exactly from that identity on a fixed set of sample directions.

Sign conventions of lie_learn beyond these two anchors, and the sign of each
Q_J (a singular vector), cannot be reproduced without that package; a flipped
sign of a basis element is absorbed by the learned weight that multiplies it.
"""
import functools
import math

import numpy as np
import torch

from .cache_file import cached_npy


# ---- rotations (ZYZ Euler angles) -----------------------------------------------------
def _as_float(x):
    return float(x.item()) if torch.is_tensor(x) else float(x)


def rot_z(gamma):
    g = _as_float(gamma)
    c, s = math.cos(g), math.sin(g)
    return torch.tensor([[c, -s, 0.], [s, c, 0.], [0., 0., 1.]], dtype=torch.get_default_dtype())


def rot_y(beta):
    b = _as_float(beta)
    c, s = math.cos(b), math.sin(b)
    return torch.tensor([[c, 0., s], [0., 1., 0.], [-s, 0., c]], dtype=torch.get_default_dtype())


def rot(alpha, beta, gamma):
    """R = Rz(alpha) Ry(beta) Rz(gamma)."""
    return rot_z(alpha) @ rot_y(beta) @ rot_z(gamma)


def _rot_np(alpha, beta, gamma):
    def rz(t):
        c, s = math.cos(t), math.sin(t)
        return np.array([[c, -s, 0.], [s, c, 0.], [0., 0., 1.]])

    def ry(t):
        c, s = math.cos(t), math.sin(t)
        return np.array([[c, 0., s], [0., 1., 0.], [-s, 0., c]])

    return rz(alpha) @ ry(beta) @ rz(gamma)


def x_to_alpha_beta(x):
    """Point on the sphere -> (alpha, beta) with rot(alpha, beta, 0) e_z proportional to x."""
    if not torch.is_tensor(x):
        x = torch.tensor(x, dtype=torch.get_default_dtype())
    x = x / torch.norm(x, 2, -1, keepdim=True)
    beta = torch.acos(x[..., 2])
    alpha = torch.atan2(x[..., 1], x[..., 0])
    return alpha, beta


def compose(a1, b1, c1, a2, b2, c2):
    """Euler angles of rot(a1, b1, c1) @ rot(a2, b2, c2)."""
    comp = rot(a1, b1, c1) @ rot(a2, b2, c2)
    xyz = comp @ torch.tensor([0, 0, 1.], dtype=comp.dtype)
    a, b = x_to_alpha_beta(xyz)
    rotz = rot(0, -b, -a) @ comp
    c = torch.atan2(rotz[1, 0], rotz[0, 0])
    return a, b, c


def kron(x, y):
    assert x.ndimension() == 2 and y.ndimension() == 2
    return torch.einsum("ij,kl->ikjl", (x, y)).contiguous().view(x.size(0) * y.size(0),
                                                                  x.size(1) * y.size(1))


# ---- real spherical harmonics ---------------------------------------------------------
def _legendre_all(lmax, ct, st):
    """Associated Legendre functions P_l^m(cos t) without the Condon-Shortley
    phase, for 0 <= m <= l <= lmax.  ct, st: arrays of cos and sin.  Returns
    a dict {(l, m): array}."""
    P = {(0, 0): np.ones_like(ct)}
    for m in range(1, lmax + 1):
        P[(m, m)] = P[(m - 1, m - 1)] * (2 * m - 1) * st
    for m in range(0, lmax):
        P[(m + 1, m)] = ct * (2 * m + 1) * P[(m, m)]
    for m in range(0, lmax + 1):
        for l in range(m + 2, lmax + 1):
            P[(l, m)] = ((2 * l - 1) * ct * P[(l - 1, m)] - (l + m - 1) * P[(l - 2, m)]) / (l - m)
    return P


def real_sh_np(l, xyz):
    """Real spherical harmonics of order l at the directions xyz [..., 3]
    (need not be normalised; the zero vector gives Y_0 = 1/sqrt(4 pi), Y_{l>0} = 0).
    Returns [2l+1, ...] float64, m = -l..l."""
    xyz = np.asarray(xyz, dtype=np.float64)
    r = np.linalg.norm(xyz, axis=-1)
    zero = r == 0
    safe = np.where(zero, 1.0, r)
    x, y, z = xyz[..., 0] / safe, xyz[..., 1] / safe, xyz[..., 2] / safe
    ct = np.clip(z, -1.0, 1.0)
    st = np.sqrt(np.maximum(0.0, 1.0 - ct * ct))
    phi = np.arctan2(y, x)
    P = _legendre_all(l, ct, st)
    out = np.zeros((2 * l + 1,) + xyz.shape[:-1], dtype=np.float64)
    for m in range(0, l + 1):
        norm = math.sqrt((2 * l + 1) / (4 * math.pi) * math.factorial(l - m) / math.factorial(l + m))
        if m == 0:
            out[l] = norm * P[(l, 0)]
        else:
            out[l + m] = math.sqrt(2.0) * norm * P[(l, m)] * np.cos(m * phi)
            out[l - m] = math.sqrt(2.0) * norm * P[(l, m)] * np.sin(m * phi)
    if zero.any():
        out[:, zero] = 0.0
        if l == 0:
            out[0, zero] = 1.0 / math.sqrt(4 * math.pi)
    return out


def spherical_harmonics_xyz(order, xyz):
    """Real spherical harmonics at points xyz [..., 3] (reference: utils/SO3.py:109-128).
    order: int or list of ints.  Returns a float64 tensor [sum(2l+1), ...]."""
    if not isinstance(order, list):
        order = [order]
    pts = xyz.detach().cpu().numpy() if torch.is_tensor(xyz) else np.asarray(xyz)
    out = np.concatenate([real_sh_np(l, pts) for l in order], axis=0)
    return torch.tensor(out, dtype=torch.float64)


def spherical_harmonics(order, alpha, beta, dtype=None):
    """Real spherical harmonics at the direction rot(alpha, beta, 0) e_z
    (reference: utils/SO3.py:79-106).  Returns [m, ...]."""
    if not isinstance(order, list):
        order = [order]
    a = np.asarray(alpha.detach().cpu().numpy() if torch.is_tensor(alpha) else alpha, np.float64)
    b = np.asarray(beta.detach().cpu().numpy() if torch.is_tensor(beta) else beta, np.float64)
    xyz = np.stack([np.sin(b) * np.cos(a), np.sin(b) * np.sin(a), np.cos(b)], axis=-1)
    out = np.concatenate([real_sh_np(l, xyz) for l in order], axis=0)
    return torch.tensor(out, dtype=torch.get_default_dtype() if dtype is None else dtype)


# ---- Wigner-D in the real basis ------------------------------------------------------
@functools.lru_cache(maxsize=None)
def _sample_dirs(l):
    """Fixed, well-spread directions and the pseudo-inverse of Y_l on them."""
    n = 4 * (2 * l + 1) + 8
    k = np.arange(n) + 0.5
    z = 1.0 - 2.0 * k / n                      # Fibonacci sphere
    phi = k * math.pi * (3.0 - math.sqrt(5.0))
    s = np.sqrt(1.0 - z * z)
    X = np.stack([s * np.cos(phi), s * np.sin(phi), z], axis=-1)  # [n, 3]
    Y = real_sh_np(l, X)                       # [2l+1, n]
    return X, np.linalg.pinv(Y)


def wigner_D_np(l, alpha, beta, gamma):
    """D^l(R), R = rot(alpha, beta, gamma), with Y_l(R x) = D^l(R) Y_l(x)."""
    X, Ypinv = _sample_dirs(l)
    R = _rot_np(float(alpha), float(beta), float(gamma))
    return real_sh_np(l, X @ R.T) @ Ypinv


def irr_repr(order, alpha, beta, gamma, dtype=None):
    """Irreducible representation of SO(3) of the given order in the real basis
    (reference: utils/SO3.py:62-76)."""
    D = wigner_D_np(order, _as_float(alpha), _as_float(beta), _as_float(gamma))
    return torch.tensor(D, dtype=torch.get_default_dtype() if dtype is None else dtype)


# ---- intertwiner ----------------------------------------------------------------------
_SYLVESTER_ANGLES = (
    (4.41301023, 5.56684102, 4.59384642),
    (4.93325116, 6.12697327, 4.14574096),
    (0.53878964, 4.09050444, 5.36539036),
    (2.16017393, 3.48835314, 5.55174441),
    (2.52385107, 0.2908958, 3.90040975),
)


def get_matrix_kernel(A, eps=1e-10):
    """Orthonormal basis (rows) of the null space of A (reference: utils/SO3.py:211-225)."""
    A = A.detach().cpu().numpy() if torch.is_tensor(A) else np.asarray(A)
    _u, s, vt = np.linalg.svd(A, full_matrices=True)
    rank = int((s >= eps).sum())
    return torch.tensor(vt[rank:], dtype=torch.float64)


def get_matrices_kernel(As, eps=1e-10):
    return get_matrix_kernel(torch.cat([torch.as_tensor(a, dtype=torch.float64) for a in As], 0),
                             eps)


@cached_npy("trans_Q")
def _Q_J_np(J, order_in, order_out):
    do, di, dj = 2 * order_out + 1, 2 * order_in + 1, 2 * J + 1
    n = do * di * dj
    # Normal equations of the stacked Sylvester system  (R_out (x) R_in) Q = Q D_J
    # over the fixed rotations of utils/SO3.py:257-263.
    M = np.zeros((n, n))
    eye_j, eye_t = np.eye(dj), np.eye(do * di)
    for a, b, c in _SYLVESTER_ANGLES:
        Rt = np.kron(wigner_D_np(order_out, a, b, c), wigner_D_np(order_in, a, b, c))
        S = np.kron(Rt, eye_j) - np.kron(eye_t, wigner_D_np(J, a, b, c).T)
        M += S.T @ S
    w, v = np.linalg.eigh(M)
    # one-dimensional solution space (utils/SO3.py:265)
    assert w[0] < 1e-10, "the Sylvester system has no solution: %r" % (w[:3],)
    assert n == 1 or w[1] > 1e-8, "null space of the Sylvester system is not one-dimensional: %r" % (w[:3],)
    q = v[:, 0]
    q = q / np.linalg.norm(q)
    # The sign of a null vector is arbitrary; fix it so results do not depend on
    # the LAPACK build: the entry of largest magnitude (first one on ties) is positive.
    k = int(np.argmax(np.abs(q) > np.abs(q).max() * (1 - 1e-9)))
    if q[k] < 0:
        q = -q
    Q = q.reshape(do * di, dj)
    for a, b, c in ((0.3, 1.1, 2.0), (2.9, 0.4, 5.1), (4.4, 2.5, 0.7), (1.0, 2.0, 3.0)):
        Rt = np.kron(wigner_D_np(order_out, a, b, c), wigner_D_np(order_in, a, b, c))
        assert np.allclose(Rt @ Q, Q @ wigner_D_np(J, a, b, c), atol=1e-9)
    return Q


def basis_transformation_Q_J(J, order_in, order_out, version=3):  # pylint: disable=W0613
    """Q_J [(2 l_out + 1)(2 l_in + 1), 2J + 1], float64: the unit-norm solution of
    (D_out (x) D_in)(R) Q = Q D_J(R) (reference: utils/SO3.py:239-274)."""
    return torch.tensor(_Q_J_np(int(J), int(order_in), int(order_out)), dtype=torch.float64)


# ---- changes of basis the reference documents (used as convention anchors) -------------
def xyz_vector_basis_to_spherical_basis():
    """A with irr_repr(1, a, b, c) @ A == A @ rot(a, b, c) (reference: utils/SO3.py:282-292)."""
    return torch.tensor([[0, 1, 0], [0, 0, 1], [1, 0, 0]], dtype=torch.get_default_dtype())


def tensor3x3_repr(a, b, c):
    r = rot(a, b, c)
    return kron(r, r)


def tensor3x3_repr_basis_to_spherical_basis():
    """Rows that carry a 3x3 tensor (T -> R T R^t) into its l = 0, 1, 2 parts
    (reference: utils/SO3.py:304-335)."""
    dt = torch.get_default_dtype()
    to1 = torch.tensor([[1, 0, 0, 0, 1, 0, 0, 0, 1]], dtype=dt)
    to3 = torch.tensor([[0, 0, -1, 0, 0, 0, 1, 0, 0],
                        [0, 1, 0, -1, 0, 0, 0, 0, 0],
                        [0, 0, 0, 0, 0, 1, 0, -1, 0]], dtype=dt)
    s3 = 3 ** .5 / 3
    to5 = torch.tensor([[0, 1, 0, 1, 0, 0, 0, 0, 0],
                        [0, 0, 0, 0, 0, 1, 0, 1, 0],
                        [-s3, 0, 0, 0, -s3, 0, 0, 0, 12 ** .5 / 3],
                        [0, 0, 1, 0, 0, 0, 1, 0, 0],
                        [1, 0, 0, 0, -1, 0, 0, 0, 0]], dtype=dt)
    return to1, to3, to5
