// Arguments of differential attention over the paged cache: every query head runs two
// softmax attentions (two "maps": two queries and two keys of `dim` numbers each, laid out
// [map 1 | map 2] head by head) over the same values of `vdim` numbers, and gives
//   o = a1 - lambda a2,  then  o <- o rsqrt(mean(o^2) + eps) out_scale   (eps < 0: no norm)
// Scores: (q . k) scale temp(p), temp(p) = 1 + t_coef ln(floor((p + 1) / t_every) + 1) at the
// row's position p (t_coef 0: none), then cap tanh(score / cap) (cap 0: none); causal.
#pragma once
#include "common.h"

namespace ninfer {

struct DiffAttnArgs {
  const void* qkv;          // [T, q_stride] rows: Hq x 2 dim of q, then Hkv x 2 dim of k, then Hkv x vdim of v
  void* kpool;              // [pages, Hkv, page_size, 2 dim]
  void* vpool;              // [pages, Hkv, page_size, vdim]
  void* out;                // [T, Hq * vdim]
  const int* block_table;   // [S, bt_stride]
  const int* positions;     // [T]
  const int* row_seq;       // [T]
  const int* seq_row_start; // [S + 1]
  float* workspace;         // partial results of contexts cut into chunks, or null
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
  int force_plain;
  int single_rows;          // the first single_rows requests bring one row each: rows 0 .. single_rows - 1
                            // (0 when the caller does not sort them)
  float scale;
  float cap;
  float t_coef;
  int t_every;
  float lambda;
  float eps;
  float out_scale;
};

int diff_attention_plain(const DiffAttnArgs& a, int chunk, int n_chunks, hipStream_t stream);
bool diff_attention_tiles_takes(const DiffAttnArgs& a);
// (the requests before `first_seq` are left out: their single rows run as decode rows do)
int diff_attention_tiles(const DiffAttnArgs& a, int first_seq, hipStream_t stream);
// single rows with the heads of a kv head as the tile's rows: chunks, then the merge
bool diff_attention_heads_takes(const DiffAttnArgs& a);
void diff_attention_heads_plan(const DiffAttnArgs& a, int* chunk, int* n_chunks);
int diff_attention_heads(const DiffAttnArgs& a, int chunk, int n_chunks, hipStream_t stream);
// the records {m1, l1, m2, l2, acc1[vdim], acc2[vdim]} of every row and head put together
int diff_attention_merge(const DiffAttnArgs& a, int n_records, hipStream_t stream);

}  // namespace ninfer
