"""CPU oracle for the invariant-MACE hot path.  TEST INFRASTRUCTURE ONLY.

Nothing in the shipped package imports this directory.  It is a plain fp64
PyTorch/numpy restatement of what the reference's kernels compute (citations
in each function), used by tests/, by the smoke check and by the CPU-baseline
leg of the benchmark as the thing results are compared against.

Pin status of each function (what fixes it besides its own formula):

  first_occurences        numpy.searchsorted brute force
  stable_key_sort         numpy.argsort(kind="stable") / torch.sort(stable=True)
  mp_forward/backward     dense index_add_ definition + torch.autograd +
                          brute-force python loops on tiny graphs
  spherical_harmonics     scipy.special.sph_harm_y closed form, sum rule
                          sum_m Y_lm^2 = 2l+1, finite differences
  spline_*                scipy.interpolate.CubicSpline(bc_type="natural")
  linear/elemental_linear torch.einsum library routine
  symmetric_contraction   dense einsum over the un-packed U tensors +
                          python-loop brute force + torch.autograd
  u_matrices              two independent derivations (sympy Wigner-3j in the
                          real basis vs. numerical projection onto rotation
                          invariants); sign/order relative to upstream mace's
                          U_matrix_real is PARITY UNPINNED (upstream package
                          is not available offline; only matters for trained
                          checkpoints, not for random-init weights)
  readout_energies        scalar python loops over nodes, channels and hidden
                          units; special cases (dead hidden layer, one hidden
                          unit without layer-1 features, saturated gate); the
                          shift added after the scale; and, in the model, the
                          two-atom chain carried by hand through both layers
                          to the node energies (fan-in folds, gate constant,
                          scale, shift, E0)
  neighbour_list          scipy cKDTree (periodic, box > 2 cutoff), explicit
                          replication of the cell into a non-periodic cluster
                          searched by a non-periodic cKDTree (small cells,
                          several images of a pair), (i,j,S) <-> (j,i,-S)
  reference model         message passing, linears and readouts are the op
                          definitions above; Bessel basis by orthonormality
                          under r^2 dr (quadrature); envelope by its boundary
                          conditions f(0)=1, f(1)=f'(1)=f''(1)=0; activation
                          constant by the seeded Monte-Carlo recipe and
                          Gauss-Hermite quadrature; 1/sqrt(fan_in) by unit
                          second moments; nested contraction vs the dense
                          brute-force-pinned form; one- and two-atom closed
                          forms; rotation / translation / permutation
                          invariance, F = -dE/dx by central differences;
                          equality with upstream mace on a real checkpoint
                          (U path order/sign, e3nn flat weight order) is
                          PARITY UNPINNED: upstream is not available offline
"""
