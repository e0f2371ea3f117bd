// Lookup table of ahead-of-time specialised row kernels.  The generated sources
// rowprog_spec_gen<N>.hip each define one table; rowprog.hip searches them by the
// hash of the program it is asked to launch.
#pragma once
#include <stdint.h>
#include "nbk.h"

struct rp_spec_entry {
  uint64_t hash;
  // [0]: generic form (any row length).  [1..4]: register-resident forms for
  // reduction programs whose lanes own exactly 1 / 2 / 4 / 8 chunks of a row;
  // nullptr where that form was not generated.  All have the signature of
  // rp_block_kernel / rp_flat_kernel.
  const void* kernel[5];
  // [1..4]: the same register-resident forms compiled for rows of exactly
  // 1 / 2 / 4 / 8 chunks per lane (no masked lanes or elements); [0] unused.
  const void* kernel_full[5];
  // [1..4]: kernel_full with non-temporal loads and stores, for launches that move
  // more bytes than the last-level cache holds.
  const void* kernel_stream[5];
  // programs without reductions: the generic form compiled for launches of a single row (a flat
  // array: no row arithmetic per chunk); nullptr for reduction programs.
  const void* kernel_flat;
  // reduction programs over rows too long for a register-resident form, with a 16-bit input that
  // several phases read: the generic form with that row copied into LDS once, as it is stored
  // (2 bytes per element: a 32 000-element row and two workgroups fit a CU), and every phase
  // reading it from there; nullptr where not generated.
  const void* kernel_stage16;
  int block_mode;
};

// A hand-scheduled kernel for one program (rowprog_hand.hip), attached by hash to that program's
// entry above.  Signature of rp_block_kernel; launched with `block` lanes per row when
// `fits(program)` holds, `kernel_stream` (non-temporal loads and stores) for launches that move
// more than the last-level cache holds.
struct rp_hand_entry {
  uint64_t hash;
  const void* kernel;
  const void* kernel_stream;
  int block;
  bool (*fits)(const nbk_rowprog*);
};
extern const rp_hand_entry rp_hand_table[];
extern const int rp_hand_count;

#define NBK_RP_SPEC_FILES 4
extern const rp_spec_entry rp_spec_table_0[];
extern const rp_spec_entry rp_spec_table_1[];
extern const rp_spec_entry rp_spec_table_2[];
extern const rp_spec_entry rp_spec_table_3[];
extern const int rp_spec_count_0, rp_spec_count_1, rp_spec_count_2, rp_spec_count_3;
