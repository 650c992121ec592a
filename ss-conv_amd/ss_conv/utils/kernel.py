"""Steerable kernel basis and its contraction with the learned weights
(reference: ss_conv/utils/kernel.py).

The basis (real spherical harmonics sampled on the k^3 grid, mixed by Q_J and
windowed by Gaussian radial shells) is a one-off float64 host computation,
cached per process.  The contraction with the weights -- the part that runs in
every training forward -- is one HIP kernel that writes the dense kernel in the
[K, Cin, Cout] layout the sparse convolution consumes.
"""
import math

import numpy as np
import torch

from ss_conv import _ext
from .SO3 import irr_repr, real_sh_np, basis_transformation_Q_J
from .cache_file import cached_npy


@cached_npy("sh_cube")
def _sample_sh_cube_np(size, J):
    """Y_J on the integer grid centred on the kernel, float64 [2J+1, x, y, z]
    (reference: kernel.py:12-28; the centre voxel follows utils/SO3.py:125-127)."""
    rng = np.linspace(-((size - 1) / 2), (size - 1) / 2, size)
    grid = np.stack(np.meshgrid(rng, rng, rng, indexing="ij"), axis=-1)  # [x, y, z, 3]
    return real_sh_np(J, grid)


def _sample_sh_cube(size, J, version=3):  # pylint: disable=W0613
    return torch.tensor(_sample_sh_cube_np(int(size), int(J)), dtype=torch.float64)


def _check_y_quarter_turn(K, order_in, order_out, spatial_first):
    """rho_out(u) K(u^-1 x) rho_in(u^-1) == K(x) for u = +pi/2 about the y axis,
    the construction-time check of the reference (kernel.py:51-61, 80-90)."""
    moved = K.transpose(spatial_first, spatial_first + 2).flip(spatial_first + 2)
    d_out = irr_repr(order_out, 0, math.pi / 2, 0, dtype=K.dtype)
    d_in = irr_repr(order_in, 0, -math.pi / 2, 0, dtype=K.dtype)
    if spatial_first == 2:
        back = torch.einsum("ij,jkxyz,kl->ilxyz", d_out, moved, d_in)
    else:
        back = torch.einsum("ij,bjkxyz,kl->bilxyz", d_out, moved, d_in)
    assert torch.allclose(back, K, atol=1e-9), "basis is not equivariant under the y quarter turn"


def _sample_cube(size, order_in, order_out):
    """Angular solutions K_J = Q_J Y_J for J = |l_in - l_out| .. l_in + l_out
    (reference: kernel.py:30-64).  Returns (list of [d_out, d_in, x, y, z], r_field, orders)."""
    rng = torch.linspace(-((size - 1) / 2), (size - 1) / 2, steps=size, dtype=torch.float64)
    order_irreps = list(range(abs(order_in - order_out), order_in + order_out + 1))
    solutions = []
    for J in order_irreps:
        Y_J = _sample_sh_cube(size, J)
        Q_J = basis_transformation_Q_J(J, order_in, order_out)
        K_J = torch.einsum("mn,nxyz->mxyz", Q_J, Y_J)
        K_J = K_J.view(2 * order_out + 1, 2 * order_in + 1, size, size, size)
        _check_y_quarter_turn(K_J, order_in, order_out, spatial_first=2)
        solutions.append(K_J)
    r_field = (rng.view(-1, 1, 1).pow(2) + rng.view(1, -1, 1).pow(2)
               + rng.view(1, 1, -1).pow(2)).sqrt()
    return solutions, r_field, order_irreps


def cube_basis_kernels(size, order_in, order_out, radial_window):
    """Windowed basis [n_beta, d_out, d_in, x, y, z] or None (reference: kernel.py:67-92)."""
    basis = radial_window(*_sample_cube(size, order_in, order_out))
    if basis is None:
        return None
    _check_y_quarter_turn(basis, order_in, order_out, spatial_first=3)
    return basis


# ---- radial windows (reference: kernel.py:99-171) ---------------------------------------
def sigmoid_window(solutions, r_field, order_irreps, sharpness=5):
    size = r_field.size(0)
    n_radial = size // 2 + 1
    radii = torch.linspace(0.5, size // 2 + 0.5, steps=n_radial, dtype=torch.float64)
    basis = []
    for i, r in enumerate(radii):
        window = torch.sigmoid(sharpness * (r - r_field))
        J_max = 2 * i + 1 if i > 0 else 0
        basis += [sol * window for sol, J in zip(solutions, order_irreps) if J <= J_max]
    return torch.stack(basis, dim=0) if len(basis) > 0 else None


def gaussian_window(solutions, r_field, order_irreps, radii, J_max_list, sigma=.6):
    """Shell-major, J ascending inside a shell; shell r keeps the orders J <= J_max."""
    assert len(radii) == len(J_max_list)
    basis = []
    for r, J_max in zip(radii, J_max_list):
        window = torch.exp(-.5 * ((r_field - r) / sigma) ** 2) / (math.sqrt(2 * math.pi) * sigma)
        basis += [sol * window for sol, J in zip(solutions, order_irreps) if J <= J_max]
    return torch.stack(basis, dim=0) if len(basis) > 0 else None


def gaussian_window_wrapper(solutions, r_field, order_irreps, mode='compromise', border_dist=0.,
                            sigma=.6):
    assert mode in ['conservative', 'compromise', 'sfcnn']
    size = r_field.size(0)
    n_radial = size // 2 + 1
    radii = torch.linspace(0, size // 2 - border_dist, steps=n_radial, dtype=torch.float64)
    first = {'conservative': 2, 'compromise': 3, 'sfcnn': 4}[mode]
    J_max_list = ([0] + [first + 2 * i for i in range(7)])[:n_radial]
    return gaussian_window(solutions, r_field, order_irreps, radii, J_max_list, sigma)


def orthogonal_(tensor, gain=1):
    """Orthogonal initialisation used by dyn_iso (reference: kernel.py:178-199)."""
    if tensor.ndimension() < 2:
        raise ValueError("Only tensors with 2 or more dimensions are supported")
    rows = tensor.size(0)
    cols = tensor[0].numel()
    flattened = tensor.new_empty(rows, cols).normal_(0, 1)
    for i in range(0, rows, cols):
        q, r = torch.linalg.qr(flattened[i:i + cols].t())
        q = q * torch.diag(r, 0).sign()
        with torch.no_grad():
            tensor[i:i + cols].view_as(q.t()).copy_(q.t())
    with torch.no_grad():
        tensor.mul_(gain)
    return tensor


# ---- kernel module ----------------------------------------------------------------------
class _Combine(torch.autograd.Function):
    """dense[k, (j,v,b), (i,u,a)] = sum_n weight_ij[u,v,n] * basis_ij[n,a,b,k] in one native
    launch; the gradient with respect to the weights is the same contraction against the
    fixed basis, block by block (the blocks are small: torch einsum)."""

    @staticmethod
    def forward(ctx, weight, module, pack):
        basis, chan_out, chan_in, blocks, _ = module._tables
        ctx.module = module
        out = _ext.kernel_combine(weight.detach().float().contiguous(), basis, chan_out, chan_in,
                                  blocks, len(module.multiplicities_in), module.size ** 3,
                                  module.n_in, module.n_out, packed=bool(pack),
                                  defer=pack == "defer")
        if pack:
            out, module.packed = out
        return out

    @staticmethod
    def backward(ctx, grad):  # grad: [K, Cin, Cout]
        m = ctx.module
        K = m.size ** 3
        grads = []
        o_off = 0
        for i, (mi, di) in enumerate(zip(m.multiplicities_out, m.dims_out)):
            i_off = 0
            for j, (mj, dj) in enumerate(zip(m.multiplicities_in, m.dims_in)):
                kij = getattr(m, "kernel_{}_{}".format(i, j))
                if kij is not None:
                    nb = kij.size(0)
                    g = grad[:, i_off:i_off + mj * dj, o_off:o_off + mi * di]
                    g = g.reshape(K, mj, dj, mi, di)
                    basis = kij.to(grad.dtype).reshape(nb, di, dj, K)
                    grads.append(torch.einsum("kvbua,nabk->uvn", g, basis).reshape(-1))
                i_off += mj * dj
            o_off += mi * di
        return torch.cat(grads), None, None


class SE3Kernel(torch.nn.Module):
    """Dense steerable kernel [Cout, Cin, k, k, k] = sum_beta weight * basis.

    Parameters and buffers carry the reference's names (kernel.py:251-255):
    ``weight`` (flat; blocks in (i over Rs_out, j over Rs_in) order, each
    [m_out, m_in, n_beta]) and ``kernel_{i}_{j}`` ([n_beta, d_out, d_in, k, k, k]).
    """

    def __init__(self, Rs_in, Rs_out, size, radial_window=gaussian_window_wrapper, dyn_iso=False,
                 verbose=False):
        super().__init__()
        self.size = size
        self.Rs_out = [(m, l) for m, l in Rs_out if m >= 1]
        self.Rs_in = [(m, l) for m, l in Rs_in if m >= 1]
        self.multiplicities_out = [m for m, _ in self.Rs_out]
        self.multiplicities_in = [m for m, _ in self.Rs_in]
        self.dims_out = [2 * l + 1 for _, l in self.Rs_out]
        self.dims_in = [2 * l + 1 for _, l in self.Rs_in]
        self.n_out = sum(m * d for m, d in zip(self.multiplicities_out, self.dims_out))
        self.n_in = sum(m * d for m, d in zip(self.multiplicities_in, self.dims_in))

        weights = []
        for i, (m_out, l_out) in enumerate(self.Rs_out):
            for j, (m_in, l_in) in enumerate(self.Rs_in):
                basis = cube_basis_kernels(size, l_in, l_out, radial_window)
                if basis is None:
                    self.register_buffer("kernel_{}_{}".format(i, j), None)
                    continue
                basis = basis.clone()
                assert basis.size()[1:] == (2 * l_out + 1, 2 * l_in + 1, size, size, size)
                if verbose:
                    print("{} -> {} : {} basis elements".format(l_in, l_out, len(basis)))
                if dyn_iso:
                    w = torch.zeros(m_out, m_in, basis.size(0))
                    if abs(l_out - l_in) == min(abs(l_out - l_) for _m, l_ in self.Rs_in):
                        orthogonal_(w[:, :, 0])
                    weights.append(w.flatten())
                    basis /= basis.flatten(2).norm(dim=2).mean(1).view(-1, 1, 1, 1, 1, 1)
                else:
                    weights.append(torch.randn(m_out * m_in * basis.size(0)))
                    # unit L2 norm per element, then the variance-preserving scale
                    basis /= basis.flatten(1).norm(dim=1).view(-1, 1, 1, 1, 1, 1)
                    basis *= ((2 * l_out + 1) / (len(basis) * sum(self.multiplicities_in))) ** 0.5
                self.register_buffer("kernel_{}_{}".format(i, j),
                                     basis.type(torch.get_default_dtype()))
        self.weight = torch.nn.Parameter(torch.cat(weights))
        self._tables = None  # device tables for the native contraction, built on first use
        self.packed = None   # packed filters left by the last combination(pack=True)

    def __repr__(self):
        return "{name} ({Rs_in} -> {Rs_out}, size={size})".format(
            name=self.__class__.__name__, Rs_in=self.Rs_in, Rs_out=self.Rs_out, size=self.size)

    # -- native contraction -------------------------------------------------------------
    def _load_from_state_dict(self, *args, **kwargs):
        self._tables = None
        return super()._load_from_state_dict(*args, **kwargs)

    def _apply(self, fn, *args, **kwargs):
        self._tables = None
        return super()._apply(fn, *args, **kwargs)

    def _build_tables(self, device):
        K = self.size ** 3
        chan_out = [(i, u, a) for i, (m, d) in enumerate(zip(self.multiplicities_out, self.dims_out))
                    for u in range(m) for a in range(d)]
        chan_in = [(j, v, b) for j, (m, d) in enumerate(zip(self.multiplicities_in, self.dims_in))
                   for v in range(m) for b in range(d)]
        blocks, pieces = [], []
        w_off = b_off = 0
        for i, mi in enumerate(self.multiplicities_out):
            for j, mj in enumerate(self.multiplicities_in):
                kij = getattr(self, "kernel_{}_{}".format(i, j))
                if kij is None:
                    blocks.append((0, 0, 0, mj, self.dims_out[i], self.dims_in[j]))
                    continue
                nb = kij.size(0)
                blocks.append((w_off, b_off, nb, mj, self.dims_out[i], self.dims_in[j]))
                pieces.append(kij.reshape(-1).to(device=device, dtype=torch.float32))
                w_off += mi * mj * nb
                b_off += nb * self.dims_out[i] * self.dims_in[j] * K
        assert w_off == self.weight.numel()
        as_i32 = lambda rows: torch.tensor(rows, dtype=torch.int32, device=device).contiguous()
        self._tables = (torch.cat(pieces).contiguous(), as_i32(chan_out), as_i32(chan_in),
                        as_i32(blocks), device)

    def combination(self, weight, pack=False):
        """[Cout, Cin, k, k, k] view of the natively contracted [K, Cin, Cout] kernel
        (reference: kernel.py:267-299).  Differentiable with respect to `weight`.
        With `pack` the same launch leaves the filters in the convolution kernel's packed
        order in `self.packed` (for _ext.attach_packed); with pack="defer" that launch is
        left to the rulebook the caller queues next (_ext.kernel_combine), and the caller
        ends with _ext.flush_combine()."""
        if not weight.is_cuda:
            raise RuntimeError("SE3Kernel runs on the GPU only: move the module to a cuda device")
        if self._tables is None or self._tables[4] != weight.device:
            self._build_tables(weight.device)
        self.packed = None
        dense = _Combine.apply(weight, self, pack if pack == "defer" else bool(pack))
        k = self.size
        return dense.permute(2, 1, 0).reshape(self.n_out, self.n_in, k, k, k)

    def forward(self, pack=False):  # pylint: disable=W
        return self.combination(self.weight, pack)
