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

}  // namespace tgx
