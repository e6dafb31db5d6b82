// stack_meta.h — the description of one ragged engine step that every kernel of the layered models takes: which sequence slot and position each of the
// step's T tokens (the concatenated entries of the batch) belongs to, and the slots' page tables.
#pragma once

namespace tgx {

struct StepMeta {          // device arrays of one step (T tokens, S entries)
  const int* tok_id;       // [T] token id
  const int* tok_pos;      // [T] position inside its sequence
  const int* tok_ent;      // [T] entry of the token
  const int* tok_row;      // [T] its sequence slot, its index inside the entry, the entry's length and state buffer: copies of the per-entry values, so
  const int* tok_idx;      //     that a one-workgroup-per-token kernel reads everything it needs in one round trip instead of two dependent ones
  const int* tok_cnt;
  const int* tok_par;
  const int* ent_row;      // [S] sequence slot
  const int* ent_start;    // [S] first token of the entry
  const int* ent_count;    // [S]
  const int* ent_par;      // [S] which of the slot's two convolution-state buffers holds the state BEFORE this step
  const int* tbl;          // [slots][tbl_stride] pages of the latent pool
  int tbl_stride, page_shift, T, S;
};

// attention masks of the layered designs: the first key the query at position `pos` sees (its last is `pos`)
enum { MASK_CAUSAL = 0, MASK_WINDOW = 1, MASK_CHUNK = 2 };      // == tgx_mask (include/tgx.h)
__device__ __forceinline__ int first_key(int pos, int kind, int size) {
  return kind == MASK_WINDOW ? max(0, pos - size + 1) : kind == MASK_CHUNK ? pos - pos % size : 0;
}
// the distance bias of head h of `heads`: scores lose slope * (i - j)
__device__ __forceinline__ float distance_slope(int h, int heads) { return exp2f(-8.0f * (float)(h + 1) / (float)heads); }

}  // namespace tgx
