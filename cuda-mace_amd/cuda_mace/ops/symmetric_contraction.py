import numpy as np
import torch

from . import classes
from .u_matrix import U_matrix_real


U_ZERO = 1e-10  # coupling coefficients below this are rounding residue of a change of basis, not couplings


def coupling_tensors_of(symm_contract, correlation: int = 3):
    """{nu: fp64 tensor [16]*nu + [paths]} for nu = 1..correlation.

    The weights of a trained model multiply the coupling paths in the order and with the signs of the basis they were
    trained in.  The reference takes that basis from upstream's `U_matrix_real` (ops/symmetric_contraction.py:29-34);
    upstream's contraction modules keep the very same tensors as buffers `U_matrix_1`, `U_matrix_2`, `U_matrix_3`
    next to the weights, so they are read from there when the module has them (a leading axis of length 1, as a
    single scalar output can carry, is dropped).  Only a module without such buffers gets the tensors of
    `ops/u_matrix.py`, whose path order and signs are this package's own."""
    con = symm_contract.contractions[0]
    found = {nu: getattr(con, "U_matrix_%d" % nu, None) for nu in range(1, correlation + 1)}
    have = [nu for nu, U in found.items() if U is not None]
    if have and len(have) != correlation:
        raise ValueError("the contraction module has coupling buffers for orders %s only; need 1..%d" % (have, correlation))
    out = {}
    for nu in range(1, correlation + 1):
        if have:
            U = found[nu].detach().to("cpu", torch.float64)
            while U.dim() > nu + 1 and U.shape[0] == 1:
                U = U[0]
            U = torch.where(U.abs() < U_ZERO, torch.zeros_like(U), U)
        else:
            U = U_matrix_real(irreps_in=symm_contract.irreps_in, irreps_out="0e", correlation=nu, dtype=torch.float64)[-1]
        out[nu] = U
    return out


def check_coupling_tensor(U: torch.Tensor, nu: int, num_weight_paths: int) -> None:
    """What the packed tables and the kernels assume of a coupling tensor, whatever its source: shape [16]*nu +
    [paths] with as many paths as the weights have, at most one path per index tuple (the packed word has room for
    one), and unit Frobenius norm per path (the normalisation under which upstream's weights are trained; a tensor
    that fails it is most likely not a coupling tensor of this model)."""
    if tuple(U.shape[:-1]) != (16,) * nu:
        raise ValueError("coupling tensor of order %d has shape %s, expected %s + [paths]" % (nu, tuple(U.shape), [16] * nu))
    if U.shape[-1] != num_weight_paths:
        raise ValueError("coupling tensor of order %d has %d paths, the weights have %d" % (nu, U.shape[-1], num_weight_paths))
    if int((U != 0).sum(-1).max()) > 1:
        raise ValueError("coupling tensor of order %d couples one index tuple through several paths" % nu)
    if nu == 1 and not (float(U[0, 0]) == 1.0 and int((U != 0).sum()) == 1):
        # the kernels apply the order-1 weights to component 0 with coefficient 1, as the reference's do
        # (cuda/src/symmetric_contraction_impl.cu:113-117)
        raise ValueError("coupling tensor of order 1 must be the unit vector of component 0")
    norms = (U.double() ** 2).sum(dim=tuple(range(nu))).sqrt()
    if not torch.allclose(norms, torch.ones_like(norms), atol=1e-5):
        raise ValueError("coupling tensor of order %d: paths must have unit Frobenius norm, found %s" % (nu, norms.tolist()))


class SymmetricContraction(torch.nn.Module):
    """Correlation-3 symmetric contraction to a scalar per channel:  x [nnodes, 16, C], atom_types int32
    [nnodes] -> [nnodes, 1, C].

    Built from an upstream-like SymmetricContraction module as in the reference
    (ops/symmetric_contraction.py:6-64): reads `irreps_in`, `irreps_out` and, for every output irrep j,
    `contractions[j].weights_max` (order 3), `.weights[0]` (order 2), `.weights[1]` (order 1).  Buffer names
    and the packed sparse format of the coupling tables are the reference's (:91-232):

      U3_num_nonsparse int16 [16,16]    number of non-zero k for each (i, j)
      U3_indices       int32 [3,16,16]  bits 0-7 weight path of (i,j,k), 8-15 k, 16-23 path of (j,k,i),
                                        24-31 path of (j,i,k)
      U3_values        fp32  [3,16,16]
      U2_num_nonsparse int16 [16,16], U2_indices int16 [16,16], U2_values fp32 [16,16]
      U1_num_values, U1_index int16 [16]
      weights_3 [1, ne, 23, C], weights_2 [1, ne, 4, C], weights_1 [1, ne, 1, C]
    """

    def __init__(self, symm_contract, device="cuda", dtype=torch.float32):
        super().__init__()
        self.cuda_obj = classes.symm_contract.SymmetricContraction()
        self.device = device
        self.dtype = dtype
        self.irreps_in = symm_contract.irreps_in
        self.irreps_out = symm_contract.irreps_out
        self.correlation = 3
        self.nlout = (self.irreps_out.lmax + 1) ** 2
        assert self.nlout == 1, "only a scalar (0e) output is supported"

        self.U_matrices = {nu: {0: U} for nu, U in coupling_tensors_of(symm_contract, self.correlation).items()}
        self.W_tensors = {}
        for j in range(len(symm_contract.contractions)):
            con = symm_contract.contractions[j]
            self.W_tensors[str(j)] = {
                3: con.weights_max.detach().clone().type(torch.float32),
                2: con.weights[0].detach().clone().type(torch.float32),
                1: con.weights[1].detach().clone().type(torch.float32),
            }
        for nu in (1, 2, 3):
            check_coupling_tensor(self.U_matrices[nu][0], nu, int(self.W_tensors["0"][nu].shape[-2]))
        self.setup_sparse_matrices()
        self.setup_weights()

    def forward(self, x, atom_types):
        assert x.shape[-1] % 32 == 0, "channel dimension of x ([-1]) must be a multiple of 32."
        assert x.shape[1] == 16, "l dimension of x ([1]) must be 16."
        return self.cuda_obj.forward(
            x, atom_types, self.u3_max_nonsparse, self.U3_num_nonsparse, self.U3_indices, self.U3_values,
            self.U2_num_nonsparse, self.U2_indices, self.U2_values, self.U1_num_values, self.U1_index,
            self.weights_3, self.weights_2, self.weights_1, self.W3_L0_size, self.W2_L0_size, self.W1_L0_size,
        )

    def setup_sparse_matrices(self):
        U3 = self.U_matrices[3][0].numpy()
        U2 = self.U_matrices[2][0].numpy()
        U1 = self.U_matrices[1][0].numpy()
        nz3 = U3 != 0.0
        # exactly one weight path per non-zero (i, j, k): the packed word has room for one
        assert int(nz3.sum(-1).max()) <= 1
        num3 = nz3.any(-1).sum(-1).astype(np.int16)  # [16,16]
        kmax = int(num3.max())
        idx3 = np.zeros((kmax, 16, 16), dtype=np.int32)
        val3 = np.zeros((kmax, 16, 16), dtype=np.float32)
        path_of = lambda a, b, c: int(np.flatnonzero(U3[a, b, c])[0])  # noqa: E731
        for i in range(16):
            for j in range(16):
                for t, k in enumerate(np.flatnonzero(nz3[i, j].any(-1))):
                    k = int(k)
                    p1 = path_of(i, j, k)
                    p2 = path_of(j, i, k)  # same monomial, indices permuted: the weights of these paths
                    p3 = path_of(j, k, i)  # enter the derivative with respect to x_i
                    idx3[t, i, j] = (p2 << 24) | (p3 << 16) | (k << 8) | p1
                    val3[t, i, j] = U3[i, j, k, p1]
        nz2 = U2 != 0.0
        num2 = nz2.sum(-1).astype(np.int16)
        assert int(num2.max()) <= 1
        idx2 = nz2.argmax(-1).astype(np.int16)
        val2 = U2.sum(-1).astype(np.float32)
        num1 = (U1 != 0.0).any(-1).astype(np.int16)
        idx1 = (U1 != 0.0).argmax(-1).astype(np.int16)

        self.u3_max_nonsparse = kmax
        dev = self.device
        self.register_buffer("U3_num_nonsparse", torch.from_numpy(num3).to(dev))
        self.register_buffer("U3_indices", torch.from_numpy(idx3).to(dev))
        self.register_buffer("U3_values", torch.from_numpy(val3).to(dev))
        self.register_buffer("U2_num_nonsparse", torch.from_numpy(num2).to(dev))
        self.register_buffer("U2_indices", torch.from_numpy(idx2).to(dev))
        self.register_buffer("U2_values", torch.from_numpy(val2).to(dev))
        self.register_buffer("U1_num_values", torch.from_numpy(num1).to(dev))
        self.register_buffer("U1_index", torch.from_numpy(idx1).to(dev))

    def setup_weights(self):
        W = self.W_tensors["0"]
        stacked = {}
        for nu in (1, 2, 3):
            w = W[nu]  # [ne, npaths, C]
            stacked[nu] = w.reshape(1, *w.shape).to(device=self.device, dtype=self.dtype).contiguous()
        self.register_buffer("weights_3", stacked[3])
        self.register_buffer("weights_2", stacked[2])
        self.register_buffer("weights_1", stacked[1])
        dev = self.device
        self.register_buffer("nweights_3", torch.tensor([W[3].shape[-2]], dtype=torch.int32, device=dev))
        self.register_buffer("nweights_2", torch.tensor([W[2].shape[-2]], dtype=torch.int32, device=dev))
        self.register_buffer("nweights_1", torch.tensor([W[1].shape[-2]], dtype=torch.int32, device=dev))
        self.W3_L0_size = int(W[3].shape[-2])
        self.W2_L0_size = int(W[2].shape[-2])
        self.W1_L0_size = int(W[1].shape[-2])
