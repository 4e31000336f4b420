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
  // more than 16 rows in linear_decode.hip: 0 = the launcher chooses, SK_ROWS_SHARE_W = one workgroup
  // per column tile takes all rows, SK_ROWS_GROUPS = one workgroup per column tile and 16 rows
  int rows_mode;
  int rows_per_group;  // linear_decode.hip, one tile a workgroup: rows of a group, 16, 8, 4, 2 or 1 (set by its launcher)
  // key/value scatter (SK_EPI_QKV)
  bf16_t* kpool;
  bf16_t* vpool;
  const int* slot_mapping;
  int q_width, kv_width, head_dim, n_kv_head, page_size;
};

// linear_decode.hip: at most 64 rows, k_dim a multiple of 32.  Returns
// MGPT_ERR_BAD_SHAPE for what it does not take (the general kernel then runs).
int mgpt_launch_linear_decode(const SkinnyArgs& a, int epilogue, int out_dtype, hipStream_t stream);
// floats of partial sums the split over workgroups needs for this shape; 0: no split
long mgpt_linear_decode_partials(int n_rows, int n_out, int k_dim, bool ln, int epilogue, int rows_mode);
// whether 17 to 64 rows of this shape go to one workgroup per column tile and 16 rows
bool mgpt_linear_decode_row_groups(int n_rows, int n_out, int k_dim, int rows_mode);
