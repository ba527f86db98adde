import numpy as np
import torch

from . import classes
from .u_matrix import U_matrix_real


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

        self.U_matrices = {
            nu: {0: U_matrix_real(irreps_in=self.irreps_in, irreps_out="0e", correlation=nu, dtype=torch.float64)[-1]}
            for nu in range(1, self.correlation + 1)
        }
        self.W_tensors = {}
        for j in range(len(symm_contract.contractions)):
            con = symm_contract.contractions[j]
            self.W_tensors[str(j)] = {
                3: con.weights_max.detach().clone().type(torch.float32),
                2: con.weights[0].detach().clone().type(torch.float32),
                1: con.weights[1].detach().clone().type(torch.float32),
            }
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
