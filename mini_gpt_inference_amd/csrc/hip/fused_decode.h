// Argument blocks of the fused kernels of a decode step with few rows (fused_decode.hip).
//
// Between these kernels the residual stream is not one array but a sum that nobody has added up
// yet:  x[row] = base[row] + sum_p partials[p][row]  (or, before the first layer, the token's and
// the position's table rows).  The kernel that produces an addition to the residual (attention with
// its output projection, the feed-forward) is split over workgroups along its inner size, and each
// workgroup leaves its share as one of the partials; the kernel that reads the residual next adds
// them up while its weights are on their way, and one of its workgroups per row stores the sum, so
// that the chain of sums never grows.  A kernel boundary then stands only where every workgroup
// needs all of a row: two per layer instead of five.
#pragma once
#include "linear_skinny.h"

struct FusedResidual {
  const float* base;        // [*, width] rows as they stand; null: table rows (below)
  const float* partials;    // [n_parts][part_rows][width] sums still to be added; null: none
  int n_parts;
  long part_stride;         // floats from one part to the next (part_rows * width)
  const bf16_t* tok_table;  // with base == null: x[row] = tok_table[ids[row]] + pos_table[positions[row]]
  const bf16_t* pos_table;  // may be null
  const int* ids;
  const int* positions;
  float* settled;           // the rows' sums are stored here; another array than base (rows are read
                            // by many workgroups while one writes); null: not stored
};

#define FUSED_MAX_WIDTH 512    // wider rows bring more parts than a reader can add up on its way in
#define RESIDUAL_MAX_WIDTH 4096  // the widest row that the kernels which only add a pending residual up (LayerNorm,
                                 // settle) take: a workgroup's threads hold four values each
#define FUSED_GROUP_PARTS 4    // parts of a row that one thread of a workgroup adds up
#define FUSED_THREADS 1024
#define FUSED_WAVES 16
#define FUSED_ATTN_ONE_TOKEN_WGS 256  // (token, head) pairs up to which the attention kernel gives each a workgroup of its own
#define FUSED_MLP_SLICE 64     // hidden units of the feed-forward that one workgroup owns
