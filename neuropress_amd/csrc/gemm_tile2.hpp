// Tile-decode GEMM, 128-column blocks: y = x @ W^T (+ bias), wave64 + MFMA 32x32x16, f32 accumulate, for VQ
// weights with 16-bit indices into a codebook too large for LDS (more than 4096 rows) and for int4 /
// int8 group-affine codes.
//
// Why a second block shape.  A block's x tile (BM rows x 64 k) passes the compute unit's vector
// memory path once per 64-k step whatever the block's width, and every 128-byte line of it is a
// request to the L2, like every codebook lookup: with 64 columns the x tile costs as many L2 requests
// per weight as two lookups in three.  128 columns halve the x requests per MFMA.
//
// Block = 8 waves, two per SIMD.  Waves w and w + 4 own rows [32 MW (w % 4), 32 MW (w % 4 + 1)) of the
// block tile and 64 of the 128 columns each: 2 MW accumulator tiles of 32 x 32 per wave.  There are no
// producer waves; every job of a step is dealt over all eight, and whenever the address unit makes
// one wave wait at a load, the other wave of its SIMD has MFMAs to issue.  Everything the kernel
// loads lands in LDS by itself (global_load_lds_dwordx4 / _dword: no register, no LDS store
// instruction): the x tile (rows of 128 bytes, piece p of row r in slot p ^ ((r >> 1) & 7)), the
// staged indices or packed bytes, and for VQ the weights themselves -- a lookup is a transfer from
// codebook + 16 index straight into the W slot the MFMAs read (the codebook the caller passes is
// already in the activation dtype).
//
// Roles of wave w in every 64-k step t:
//   MFMA:    4 k groups x 2 column tiles x MW row tiles; the operands of k group j + 1 are read
//            from LDS before the MFMAs of k group j.
//   x tile:  pieces (8 rows x 128 bytes) 2 i + w / 4 of its row group, of step t + 1, into the
//            buffer that is not being read, one piece behind each of the first 2 MW MFMA slots.
//   W tile:  column tile w % 4, operand pair J = w / 4.  VQ: lane (c = l % 32, h = l / 32) reads its
//            two indices of step t + 2 from the staged indices and issues two lookups; lookup j
//            lands in position l of KiB (w % 4, j) of W slot (t + 2) % 3, which is where lane l looks
//            for B operand j of column tile w % 4: MFMA j of a step contracts k = 64 t + 32 h + 8 j
//            .. + 7, x and W alike.  int4 / int8: the producers' arithmetic between the MFMAs.
// All loads of a wave complete in order and the waits are written by hand (s_waitcnt vmcnt(n) with
// the number of younger loads that may stay in flight): everything a wave requests in step t is due
// at the end of step t + 1 at the latest, in front of the step's only barrier.  The last two steps
// are instantiated apart: nothing is looked up or fetched for steps past the end.
//
// K is split in two (blockIdx.z) when the column blocks alone leave compute units idle:
// 14336 columns are 112 blocks of 128, so 224 workgroups each contract half of K, the first halves
// on four of the GPU's dies and the second halves on the other four (a die's L2 then holds half of
// x).  The halves meet without a second kernel and without spinning: whichever workgroup of a
// pair finishes first stores its f32 tile to the workspace and swaps the call's number into the
// tile's word; the other adds that tile to its registers, adds the bias and stores y.  Two addends
// commute, so the result does not depend on which half was first.  More than two splits (layers
// of few columns) store partial tiles for splitk_reduce_kernel as the 64-column kernel does.
#pragma once

#include "gemm_tile.hpp"

namespace npamd {

constexpr int kT2Cols = 128;
constexpr int kT2WSlotBytes = kT2Cols * kStepK * 2;  // 16 KiB: [column tile 4][operand j 4][lane 64][16 B]

struct T2Args {
  const uint8_t* packed;  // 16-bit indices, [N][K / 8]
  const void* cb;         // [nc][8] in the activation dtype
  uint32_t nc_minus_1;
  int chunks;             // K / 64
};

// int4 / int8 group-affine codes (group size a multiple of 32): what the providers of the 64-column kernel take.
struct T2QArgs {
  const uint8_t* w_pack;
  const uint16_t* scale;  // 4-byte aligned
  int chunks, groups_per_row, gs_shift_chunks;
  const uint16_t* zp;     // null: symmetric
};

// K in two halves: one word per block tile and the f32 tile of whichever half finished first,
// [2][tiles][BM * 128] in register order.
struct T2Pair {
  unsigned long long* words;  // one per tile: holds `call` while one half of the tile has arrived in this call
  float* tiles;
  unsigned long long call;    // this call's number, drawn at random: never what memory happens to hold
};

// Splits of K for the 128-column kernel: 1 while the block tiles cover most compute units, else as
// many as fill them, each at least 8 steps long.
int plan_tile2_splits(int M, int N, int chunks, int mw);
// 0: never take the 128-column kernel, 1: where it is the faster one (default), 2: wherever it applies.
int tile2_mode();

// Row tiles per wave for the group-affine producers, whose decode is cheap enough to repeat per row block: past
// 384 tokens two (256-row blocks: int4 14336 x 4096 at 512 / 1024 tokens 77 / 155 us against 97 / 173 with three,
// measured on the four-wave form of the kernel).
inline int plan_tile2_q_mw(int M) {
  const int mw = plan_tile_mw(M);
  return M > 384 && mw == 3 ? 2 : mw;
}

inline int64_t tile2_workspace_bytes(int M, int N, int chunks, int mw) {
  const int splits = plan_tile2_splits(M, N, chunks, mw);
  if (splits <= 1) return 0;
  if (splits > 2) return (int64_t)splits * M * N * 4;
  const int64_t tiles = (int64_t)((N + kT2Cols - 1) / kT2Cols) * ((M + 128 * mw - 1) / (128 * mw));
  return ((tiles * 8 + 255) & ~(int64_t)255) + 2 * tiles * (128 * mw) * kT2Cols * 4;
}

// Take the call when the workspace allows the planned split; return 1 when they did not take it.
// act: NPAMD_F16 or NPAMD_BF16 (activations, codebook and output).
int launch_tile2(int act, const GemmShape& s, const T2Args& a, hipStream_t st, const char* what, void* workspace,
                 int64_t workspace_bytes);
int launch_tile2_q(int act, int nbits, const GemmShape& s, const T2QArgs& q, hipStream_t st, const char* what,
                   void* workspace, int64_t workspace_bytes);

}  // namespace npamd
