// Internal entry of readout.hip for the one-call step.
#pragma once

#include "common.hpp"

namespace cm {

// cm_readout_forward that also writes, when node_total is given, the node's total energy node_energies[n] + node_e0[n]
// (node_e0 NULL: zero) to row rows[n] of node_total (rows NULL: row n), like the rows of node_feats64.
int readout_forward_with_totals(const float *h1, const float *h2, const double *w1, const double *W2a, const double *w2b,
                                double act_cst, double scale, double shift, int64_t nnodes, int channels, int hidden,
                                double *node_energies, float *d_h2, double *node_feats64, const int32_t *rows,
                                const double *node_e0, double *node_total, hipStream_t st);

}  // namespace cm
