"""The model behind the interface a LAMMPS pair style drives: energies of the atoms a rank owns, forces on all atoms it
sees.

A domain-decomposed MD code hands every rank its own ("local") atoms plus copies of the neighbouring ranks' atoms
within the interaction range ("ghosts").  The rank's energy is the sum of the node energies of its local atoms; the
forces it reports are minus the gradient of THAT sum with respect to every position it holds, ghosts included (the MD
code adds the ghosts' shares back to their owners).  This is the wrapper upstream MACE ships for that purpose
(mace/calculators/lammps_mace.py, class LAMMPS_MACE: same constructor, call signature and result keys); the reference
itself stops at the model (tools/model_surgery.py:217-229) and has no counterpart.

With this package's model the mask travels as data["node_weights"], which the library's one-call step takes as the
seed of every node energy, so the wrapper costs what the plain model costs.  Any other model with the same forward
signature (upstream's own) is driven as upstream's wrapper drives it: node energies out, autograd from here.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch


class LAMMPS_MACE(torch.nn.Module):
    def __init__(self, model: torch.nn.Module, head: Optional[int] = None):
        super().__init__()
        self.model = model
        self.register_buffer("atomic_numbers", model.atomic_numbers)
        self.register_buffer("r_max", torch.as_tensor(float(model.r_max), dtype=torch.float64))
        self.register_buffer("num_interactions", torch.as_tensor(int(model.num_interactions), dtype=torch.int64))
        self.head = head
        for param in self.model.parameters():
            param.requires_grad = False

    def forward(self, data: Dict[str, torch.Tensor], local_or_ghost: torch.Tensor,
                compute_virials: bool = False) -> Dict[str, Optional[torch.Tensor]]:
        """local_or_ghost [N]: 1 for the rank's own atoms, 0 for ghosts.  Returns total_energy_local [num_graphs],
        node_energy [N] (all atoms), forces [N, 3] = -d total_energy_local / d positions, virials [num_graphs, 3, 3]
        (minus the derivative with respect to the symmetric strain) or None."""
        data = dict(data)
        num_graphs = data["ptr"].numel() - 1
        if self.head is not None:
            data["head"] = torch.full((num_graphs,), int(self.head), dtype=torch.int64, device=data["positions"].device)
        if getattr(self.model, "supports_node_weights", False):
            data["node_weights"] = local_or_ghost.to(torch.float64)
            out = self.model(data, training=False, compute_force=True, compute_virials=compute_virials, compute_stress=False)
            return {"total_energy_local": out["energy"].detach(), "node_energy": out["node_energy"].detach(),
                    "forces": out["forces"].detach(), "virials": out["virials"].detach() if compute_virials else None}
        positions = data["positions"]
        if not positions.requires_grad:
            positions = positions.detach().requires_grad_(True)
            data["positions"] = positions
        out = self.model(data, training=False, compute_force=False, compute_virials=False, compute_stress=False,
                         compute_displacement=compute_virials)
        node_energy = out["node_energy"]
        if node_energy is None:
            return {"total_energy_local": None, "node_energy": None, "forces": None, "virials": None}
        weights = local_or_ghost.to(node_energy.dtype)
        total_energy_local = torch.zeros(num_graphs, dtype=node_energy.dtype, device=node_energy.device)
        total_energy_local = total_energy_local.index_add(0, data["batch"], node_energy * weights)
        seed = [torch.ones_like(total_energy_local)]
        virials = None
        if compute_virials:
            g_pos, g_strain = torch.autograd.grad([total_energy_local], [positions, out["displacement"]], grad_outputs=seed,
                                                  allow_unused=True)
            virials = torch.zeros_like(out["displacement"]) if g_strain is None else -g_strain
        else:
            (g_pos,) = torch.autograd.grad([total_energy_local], [positions], grad_outputs=seed, allow_unused=True)
        forces = torch.zeros_like(positions) if g_pos is None else -g_pos
        return {"total_energy_local": total_energy_local.detach(), "node_energy": node_energy.detach(), "forces": forces,
                "virials": virials}
