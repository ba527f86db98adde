import torch

from . import classes


class SphericalHarmonics(torch.nn.Module):
    """xyz [nedges, 3] -> [16, nedges] real spherical harmonics l <= 3 ("component" normalisation,
    normalised input).  The reference model instantiates the custom class directly
    (models/InvariantMACE.py:187, 306); this thin module does the same."""

    def __init__(self):
        super().__init__()
        self.cuda_obj = classes.spherical_harmonics.SphericalHarmonics()

    def forward(self, xyz: torch.Tensor):
        return self.cuda_obj.forward(xyz)
