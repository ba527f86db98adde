// Internal entry of node_glue.hip for the one-call step.
#pragma once

#include "common.hpp"

namespace cm {

// cm_node_glue_backward whose launch also sums the node energies per graph in extra workgroups (energies[g] = sum over
// graph g's nodes of node_weights[n] * node_es[n]; fixed order; total_energies[g] = energies[g] + graph_e0[g] when asked
// for, a missing graph_e0 counting as zero).  node_es must have been written by an earlier launch on the same stream.
// Operands as checked by the caller.
int node_glue_backward_with_energy_sums(const float *gX2, const float *d_h2, const float *up_W, const float *skip_W, const float *prod_W,
                                        const double *w1, double scale, const double *node_weights, const int32_t *node_perm,
                                        const int32_t *group_offsets, int64_t nnodes, int ngroups, int channels, float skip_scale,
                                        float *gB1, const double *node_es, const int32_t *graph_ptr, int ngraphs, double *energies,
                                        const double *graph_e0, double *total_energies, hipStream_t st);

}  // namespace cm
