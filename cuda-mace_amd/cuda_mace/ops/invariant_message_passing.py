import torch

from . import classes


class InvariantMessagePassingTP(torch.nn.Module):
    """out[n, m, c] = sum over edges received by n of node_feats[sender, c] * edge_attrs[m, e] * tp_weights[e, l(m), c].

    Same module name and call signature as the reference (ops/invariant_message_passing.py:3-22).
    Shapes as the kernels take them: node_feats [nnodes, C], edge_attrs [16, nedges] (the reference's
    comment says [nedges, 16]; its kernels index [16, nedges]), tp_weights [nedges, 4, C], both edge
    lists int32 with receiver_list non-decreasing; returns [nnodes, 16, C].
    """

    def __init__(self):
        super().__init__()
        self.cuda_obj = classes.inv_message_passing.InvariantMessagePassingTP()

    def forward(self, node_feats, edge_attrs, tp_weights, sender_list, receiver_list, nnodes):
        return self.cuda_obj.forward(node_feats, edge_attrs, tp_weights, sender_list, receiver_list, int(nnodes))

    def forward_spline(self, node_feats, edge_attrs, edge_lengths, spline, sender_list, receiver_list, nnodes):
        """Same result as forward(node_feats, edge_attrs, spline(edge_lengths).view(E, 4, C), ...) with the radial
        weights evaluated inside the kernels from `spline` (a cuda_mace.ops.CubicSpline): the [nedges, 4, C] weights
        and their gradient are never materialised.  Not part of the reference's interface."""
        from ._autograd import InvariantMessagePassingSplineTPAutograd

        return InvariantMessagePassingSplineTPAutograd.apply(
            node_feats, edge_attrs, edge_lengths, spline.r_knots, spline.coefficients, spline._h, spline._rmax,
            sender_list, receiver_list, int(nnodes))

    def forward_edges(self, node_feats, edge_vectors, spline, sender_list, receiver_list, nnodes):
        """Same result as forward_spline with edge_attrs = spherical harmonics of edge_vectors and edge_lengths =
        their norms, all evaluated inside the kernels: neither the harmonics nor the radial weights are ever stored.
        Not part of the reference's interface."""
        from ._autograd import InvariantMessagePassingEdgeTPAutograd

        return InvariantMessagePassingEdgeTPAutograd.apply(
            node_feats, edge_vectors, spline.r_knots, spline.coefficients, spline._h, spline._rmax, sender_list,
            receiver_list, int(nnodes))
