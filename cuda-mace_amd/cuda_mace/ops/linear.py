from math import prod

import torch

from . import classes


def _stack_blocks(instructions, flat_weights, lead_shape=()):
    """Cuts the flat e3nn-ordered weight vector into one [.., K, N'] block per instruction."""
    blocks = []
    at = 0
    for ins in instructions:
        n = prod(ins.path_shape)
        blocks.append(flat_weights.narrow(-1, at, n).reshape(list(lead_shape) + list(ins.path_shape)))
        at += n
    return blocks


class Linear(torch.nn.Module):
    """Per-l channel mixing  out[n, lm, :] = x[n, lm, :] @ W[l(lm)] / sqrt(K)  for x [nnodes, 16, K].

    Built from an e3nn-Linear-like object exactly as the reference does (ops/linear.py:7-54): attributes
    irreps_in, irreps_out, instructions (i_in, i_out, path_shape, path_weight) and the flat `weight`.
    Buffers `weights` [4, K, N'] and `weights_transposed` [4, N', K] as in the reference.
    """

    def __init__(self, linear):
        super().__init__()
        self.cuda_obj = classes.linear_wmma.Linear()
        self.irreps_out = linear.irreps_out
        self.irreps_in = linear.irreps_in.simplify()
        self.e3nn_instructions = linear.instructions
        self.e3nn_weights = linear.weight.clone().detach()
        self.out_lmax = int(self.irreps_out.lmax)
        self.out_dim = int(self.irreps_out.dim / (self.out_lmax + 1) ** 2)
        blocks = _stack_blocks(self.e3nn_instructions, self.e3nn_weights)
        weights = torch.stack(blocks).contiguous().float()
        self.register_buffer("weights", weights)
        self.register_buffer("weights_transposed", weights.transpose(-1, -2).contiguous())

    def forward(self, x: torch.Tensor):
        return self.cuda_obj.forward(x, self.weights, self.weights_transposed)


class ElementalLinear(torch.nn.Module):
    """Channel mixing with a weight block per chemical element and per l; y is the one-hot species
    matrix [nnodes, nelements].  Same constructor as the reference (ops/linear.py:57-108): the flat
    weights carry a leading element dimension; buffers `weights` [ne, 4, K, N'] and
    `weights_transposed` [ne, 4, N', K]."""

    def __init__(self, irreps_in, irreps_out, e3nn_instructions, e3nn_weights, num_elements):
        super().__init__()
        self.cuda_obj = classes.linear_wmma.ElementalLinear()
        self.num_elements = num_elements
        self.irreps_in = irreps_in
        self.irreps_out = irreps_out
        self.e3nn_instructions = e3nn_instructions
        self.e3nn_weights = e3nn_weights
        self.out_lmax = int(irreps_out.lmax)
        self.out_dim = int(irreps_out.dim / (self.out_lmax + 1) ** 2)
        blocks = _stack_blocks(e3nn_instructions, e3nn_weights.detach(), lead_shape=(-1,))
        weights = torch.stack(blocks, dim=1).contiguous().float()  # [ne, 4, K, N']
        self.register_buffer("weights", weights)
        self.register_buffer("weights_transposed", weights.transpose(-1, -2).contiguous())

    def forward(self, x, y):
        return self.cuda_obj.forward(x, self.weights, self.weights_transposed, y)


class ScalarElementalLinear(torch.nn.Module):
    """Per-element channel mixing of scalar features: out[n, :] = x[n, :] @ W[element(n)] / sqrt(K) for x [nnodes, K],
    y the one-hot species matrix.  Same kernels as ElementalLinear with a single component per node.  The reference
    leaves this case (the residual skip connection of the second layer) to the upstream e3nn tensor product
    (models/InvariantMACE.py:133, 149)."""

    def __init__(self, weights: torch.Tensor):
        super().__init__()
        self.cuda_obj = classes.linear_wmma.ElementalLinear()
        w = weights.detach().float().contiguous()  # [ne, K, N']
        self.register_buffer("weights", w)
        self.register_buffer("weights_transposed", w.transpose(-1, -2).contiguous())

    def forward(self, x, y):
        return self.cuda_obj.forward(x, self.weights, self.weights_transposed, y)
