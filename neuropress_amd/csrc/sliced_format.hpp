// Slice-list layout of a VQ index matrix, shared by the host builder and the
// sliced GEMV kernel.
//
// The codebook is cut into slices of `slice_rows` rows (a slice fits in one
// compute unit's LDS).  Every (row n, group g) index is filed under the slice
// its codebook row belongs to, so that a workgroup holding one slice in LDS
// sees only the lookups that hit it.
//
// A task is (slice, group range, output row): the entries of that row whose
// group lies in the range and whose codebook row lies in the slice.  A task is
// run by one lane, which keeps the row's partial sum in a register, so nothing
// is ever scattered; the partial sums of a row's tasks (one per slice and group
// range = one per "partial" vector) are added by a second kernel.
//
// A workgroup covers one (slice, group range) and up to 1024 rows.  Its tasks
// are sorted by length and cut into strips of 64 (one strip per wave, at most
// 16).  Strip w has the same length, header.wave_quads[w] quads, in every
// workgroup (the longest strip w of the layer; shorter ones are padded with
// entries that select an all-zero codebook row), so the address of a wave's
// entries follows from the workgroup and wave numbers alone and a wave can
// request them before anything it read has come back.  The row each lane works
// for is stored per lane.
//
// Entry (22 of 24 bits): a 13-bit codebook row inside the slice (kSlicedPadRow = the
// zero row) and a 9-bit group inside the workgroup's range.  Entries are stored
// four to a lane: quad q of a strip is 64 lanes x 12 bytes, lane-major, so one
// 12-byte load per lane fetches steps 4q .. 4q + 3.  The quads of a strip are
// consecutive, the strips of a workgroup follow each other in wave order and
// workgroup w starts at quad w * (sum of wave_quads).  Inside the 12 bytes the
// four rows come first (uint16 each: the row in bits 0-12, bit 8 of the group in bit
// 15), then the low eight bits of the four groups (uint8 each).
#pragma once

#include <stdint.h>

#include "../../include/npamd.h"

namespace npamd {

constexpr uint32_t kSlicedMagic = 0x4C53504Eu;  // "NPSL"
constexpr uint32_t kSlicedVersion = 3;
constexpr int kSlicedWaves = 16;             // waves (= strips) per workgroup
constexpr int kSlicedTasks = kSlicedWaves * 64;
constexpr int kSlicedMaxSliceRows = 4096;    // rows of a slice (64 KiB of LDS)
constexpr int kSlicedPadRow = 4096;          // row field of a padding entry: the zero row behind the slice
constexpr int kSlicedMaxGroups = 512;        // groups per range (9-bit field; 8 KiB of activations per token in LDS)
constexpr int kSlicedLdsBytes = 160 * 1024;
constexpr int kSlicedQuadBytes = 64 * 12;
constexpr uint32_t kSlicedNoRow = 0xFFFFFFFFu;

// header.flags
constexpr uint32_t kSlicedRoundRobin = 1u;  // workgroup w works on slice w % n_slices

struct SlicedWorkgroup {  // 32 bytes
  uint32_t slice;         // codebook rows [slice * slice_rows, ...)
  uint32_t partial;       // which partial-sum vector receives the results
  uint32_t g_begin;       // group range [g_begin, g_begin + g_count)
  uint32_t g_count;
  uint32_t row_begin;     // output rows [row_begin, row_begin + row_count), row_count <= kSlicedTasks
  uint32_t row_count;
  uint32_t reserved[2];
};

static_assert(sizeof(npamd_sliced_header) == 128, "header is 128 bytes");
static_assert(sizeof(SlicedWorkgroup) == 32, "packed layout");

}  // namespace npamd
