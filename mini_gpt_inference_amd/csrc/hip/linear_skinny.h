// What the two kernels for products with few rows share: the argument block and epilogue codes.
#pragma once
#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(short)))) short bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;

#define SK_EPI_NONE 0
#define SK_EPI_GELU 1
#define SK_EPI_RESIDUAL 2
#define SK_EPI_QKV 3

#define SK_ROWS_SHARE_W 2
#define SK_ROWS_GROUPS 3

#define SK_WAVES 4        // waves of a workgroup without a prologue
#define SK_LN_WAVES 16    // waves of a workgroup with the LayerNorm prologue: one row each

struct SkinnyArgs {
  const bf16_t* act;  // [n_rows, k_dim] bfloat16, row stride lda (no prologue)
  long lda;
  const float* x;     // residual stream, float32, row stride k_dim (folded LayerNorm)
  const int* rows;    // optional gather of residual rows
  const float* colsum;  // S[o] of the folded matrix
  float eps;
  const bf16_t* w;    // [n_out, k_dim] (the folded matrix when x is given)
  const bf16_t* w_packed;  // the same matrix in fold_norm.hip's packed layout, or null
  const float* bias;  // [n_out] or null (the folded bias when x is given)
  void* out;          // [n_rows, n_out], row stride ldo
  long ldo;
  int n_rows, n_out, k_dim;
  int ksplit;         // waves of a workgroup that share a column tile: 1, 2 or 4
  // k split over workgroups (linear_decode_rows.hip): each writes its raw sums to
  // partials[part][row][column] and a second kernel adds them and applies the epilogue
  float* partials;
  int k_parts;
  int bias_in_part0;  // with the split: the first part carries the bias (nobody adds it afterwards)
  // more than 16 rows in linear_decode.hip: 0 = the launcher chooses, SK_ROWS_SHARE_W = one workgroup
  // per column tile takes all rows, SK_ROWS_GROUPS = one workgroup per column tile and 16 rows
  int rows_mode;
  int rows_per_group;  // linear_decode.hip, one tile a workgroup: rows of a group, 16, 8, 4, 2 or 1 (set by its launcher)
  // key/value scatter (SK_EPI_QKV)
  bf16_t* kpool;
  bf16_t* vpool;
  const int* slot_mapping;
  int q_width, kv_width, head_dim, n_kv_head, page_size;
  // linear_decode.hip, one tile a workgroup, float32 output without an epilogue: per row and column
  // tile the largest value among the tile's columns below best_limit and its column (the lowest
  // among equals), to best_val / best_idx [n_rows][n_out / 16]; null: off
  float* best_val;
  int* best_idx;
  int best_limit;
};

// linear_decode.hip: at most 64 rows, k_dim a multiple of 32.  Returns
// MGPT_ERR_BAD_SHAPE for what it does not take (the general kernel then runs).
int mgpt_launch_linear_decode(const SkinnyArgs& a, int epilogue, int out_dtype, hipStream_t stream);
// floats of partial sums the split over workgroups needs for this shape; 0: no split
long mgpt_linear_decode_partials(int n_rows, int n_out, int k_dim, bool ln, int epilogue, int rows_mode);
// whether 17 to 64 rows of this shape go to one workgroup per column tile and 16 rows
bool mgpt_linear_decode_row_groups(int n_rows, int n_out, int k_dim, int rows_mode);

// mgpt_linear_skinny for callers that cannot allocate device memory and bring no scratch of their
// own (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has
// no counterpart in the reference.  Where mgpt_linear_skinny would split a long inner size over
// workgroups (17 to 64 rows under a matrix too large for groups of rows, and 16 rows or fewer under
// an inner size of 3072 or more with few column tiles: whenever mgpt_linear_skinny_partials is not
// zero) the partial sums go to an array that
// the library itself holds in device memory, MGPT_STATIC_SCRATCH_FLOATS floats (1 MiB) on every GPU
// the library runs on, until the process ends; a shape that needs more is refused with
// MGPT_ERR_SCRATCH and nothing is launched.  The call allocates and frees nothing.  Every call on
// a GPU uses that GPU's one array, so calls that overlap on one GPU (on different streams, or from
// different threads) race; calls on one stream follow each other and are safe.  Nothing in the
// array has to start at zero: the first kernel writes every partial sum that the second reads.
// The array's address on a GPU is asked of the runtime once per GPU (hipGetSymbolAddress), at
// mgpt_linear_skinny_static_scratch_init() or else inside the first call on that GPU: a caller that
// captures a stream into a graph calls the init function (with that GPU current) before the capture
// begins, so that no call inside the capture is the first.
#define MGPT_STATIC_SCRATCH_FLOATS (4L * 64 * 1024)
#define MGPT_ERR_SCRATCH (-5)
extern "C" int mgpt_linear_skinny_static_scratch(
    const void* act, long lda, const float* x, const int* rows, const float* colsum, float eps, const void* w,
    const void* w_packed, const float* bias, void* out, int out_dtype, long ldo, int n_rows, int n_out, int k_dim,
    int epilogue, void* kpool, void* vpool, const int* slot_mapping, int q_width, int kv_width, int head_dim,
    int n_kv_head, int page_size, int mode, hipStream_t stream);
// the array's size in floats
extern "C" long mgpt_linear_skinny_static_scratch_floats();
// resolves the array's address on the current GPU (MGPT_OK, or the runtime's error code); launches nothing
extern "C" int mgpt_linear_skinny_static_scratch_init();
