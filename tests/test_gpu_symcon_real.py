"""Symmetric contraction with the real l_max = 3 coupling tensors: the op module (packed tables as the reference
builds them) against the dense fp64 oracle evaluated with independently derived U tensors, forward and backward.
Exercises the kernel that is unrolled over the built-in monomial structure as well as the table-driven one."""
import numpy as np
import pytest
import torch

from oracle import ops as O
from oracle.u_tensors import u_tensors
from tests.util import close

pytestmark = pytest.mark.gpu


def _module(ne, C, seed):
    from cuda_mace.models.upstream_like import _SymmetricContraction
    from cuda_mace.ops.symmetric_contraction import SymmetricContraction

    up = _SymmetricContraction(C, ne, torch.Generator().manual_seed(seed))
    return up, SymmetricContraction(up, device="cuda")


@pytest.mark.parametrize("N,C,ne,seed", [(1, 32, 1, 0), (100, 128, 10, 1), (77, 96, 4, 2), (40, 192, 10, 3), (300, 64, 3, 4)])
def test_symmetric_contraction_module(cabi, N, C, ne, seed):
    print("symcon module", N, C, ne, seed, flush=True)
    up, mod = _module(ne, C, seed)
    con = up.contractions[0]
    U1, U2, U3 = (torch.from_numpy(u) for u in u_tensors())
    g = torch.Generator().manual_seed(seed)
    X = torch.randn(N, 16, C, generator=g, dtype=torch.float64)
    types = torch.randint(0, ne, (N,), generator=g).int()
    gout = torch.randn(N, C, generator=g, dtype=torch.float64)
    Xa = X.clone().requires_grad_(True)
    # the module holds fp32 copies of weights and tables; give the oracle the same rounded weights
    W3, W2, W1 = (w.detach().float().double() for w in (con.weights_max, con.weights[0], con.weights[1]))
    ref = O.symmetric_contraction(Xa, types, U3, U2, W3, W2, W1)
    (ref * gout).sum().backward()

    Xg = X.float().cuda().requires_grad_(True)
    out = mod(Xg, types.cuda())
    assert out.shape == (N, 1, C)
    (out.squeeze(1) * gout.float().cuda()).sum().backward()
    close(out.squeeze(1).detach(), ref.detach(), 3e-5, 3e-6)
    close(Xg.grad, Xa.grad, 3e-5, 3e-6)

    # built-in (unrolled) and table-driven kernels agree
    from cuda_mace.ops import _autograd as A

    (m3, o3, p3, v3), (m2, o2, p2, v2) = A.monomials_from_packed(mod.U3_num_nonsparse, mod.U3_indices, mod.U3_values,
                                                                 mod.U2_num_nonsparse, mod.U2_indices, mod.U2_values)
    b3, b2 = cabi.symcon_builtin_structure()
    assert np.array_equal(m3, b3) and np.array_equal(m2, b2)
    t = lambda a: torch.from_numpy(a).cuda()
    T3, T2, T1 = cabi.symcon_tables(t(o3), t(p3), t(v3), t(o2), t(p2), t(v2), mod.weights_3[0], mod.weights_2[0], mod.weights_1[0])
    perm, off = cabi.stable_key_sort(types.cuda(), ne)
    xa = X.float().cuda()
    out_b, grad_b = cabi.symcon_forward(xa, perm, off, t(m3), t(m2), T3, T2, T1, builtin=True)
    out_t, grad_t = cabi.symcon_forward(xa, perm, off, t(m3), t(m2), T3, T2, T1, builtin=False)
    close(out_b, out_t.double().cpu(), 1e-5, 1e-6)
    close(grad_b, grad_t.double().cpu(), 1e-5, 1e-6)
    out_ng, none = cabi.symcon_forward(xa, perm, off, t(m3), t(m2), T3, T2, T1, want_grad=False, builtin=True)
    assert none is None and torch.equal(out_ng, out_b)
