// Arguments of attention without a softmax over the paged cache: the weight of a visible key
// is sigmoid((q . k) scale + bias of the head), weights are not normalised over keys; the
// heads' weights may be mixed by a [Hq, Hq] matrix (w'_a = sum_b mix[a, b] w_b) before head a
// applies them to the values of its own kv head. Visible: key position j <= the row's position
// i and, with chunk > 0, floor(i / chunk) == floor(j / chunk).
#pragma once
#include "common.h"

namespace ninfer {

struct SigAttnArgs {
  const void* qkv;          // [T, q_stride] rows: Hq x dim of q (then, when keys and values are
                            // written, Hkv x dim of k and Hkv x vdim of v)
  void* kpool;              // [pages, Hkv, page_size, dim]
  void* vpool;              // [pages, Hkv, page_size, vdim]
  void* out;                // [T, Hq * vdim]
  const int* block_table;   // [S, bt_stride]
  const int* positions;     // [T]
  const int* row_seq;       // [T]
  const int* seq_row_start; // [S + 1]
  const float* head_bias;   // [Hq] added to the scaled score, or null
  const float* mix;         // [Hq, Hq] row a: the weights of head a's mixture, or null
  float* workspace;         // partial outputs of key ranges cut into parts, or null
  int64_t workspace_floats;
  int q_stride;
  int bt_stride;
  int T;
  int S;
  int Hq;
  int Hkv;
  int dim;
  int vdim;
  int page_size;
  int dtype;
  int max_qlen;             // host-side bounds that size launches
  int max_kv_len;
  int chunk;                // 0: every earlier position is visible
  int force_plain;
  int single_rows;          // the first single_rows requests bring one row each: rows 0 .. single_rows - 1
  float scale;
};

int sigmoid_attention_plain(const SigAttnArgs& a, hipStream_t stream);
// the matrix-core kernel: row tiles of all heads, the visible keys cut into n_splits parts
// whose partial outputs (`part`: n_splits x T x Hq x vdim 32-bit numbers, null with one
// part) a second kernel adds up
bool sigmoid_attention_tiles_takes(const SigAttnArgs& a);
int sigmoid_attention_tiles_splits(const SigAttnArgs& a);
int sigmoid_attention_tiles(const SigAttnArgs& a, float* part, int n_splits, hipStream_t stream);

}  // namespace ninfer
