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
// 16); a strip is padded to its longest task with entries that select an
// all-zero codebook row.  The row each lane works for is stored per lane.
//
// Entry (24 bits): a 16-bit codebook row inside the slice (kSlicedPadRow = the
// zero row) and an 8-bit group inside the workgroup's range.  Entries are stored
// four to a lane: quad q of a strip is 64 lanes x 12 bytes, lane-major, so one
// 12-byte load per lane fetches steps 4q .. 4q + 3.  Inside the 12 bytes the
// four rows come first (uint16 each), then the four groups (uint8 each): every
// field sits on a 16- or 8-bit boundary and becomes an LDS address in one
// shift.
#pragma once

#include <stdint.h>

#include "../../include/npamd.h"

namespace npamd {

constexpr uint32_t kSlicedMagic = 0x4C53504Eu;  // "NPSL"
constexpr uint32_t kSlicedVersion = 2;
constexpr int kSlicedWaves = 16;             // waves (= strips) per workgroup
constexpr int kSlicedTasks = kSlicedWaves * 64;
constexpr int kSlicedMaxSliceRows = 8192;    // rows of a slice (128 KiB of LDS)
constexpr int kSlicedPadRow = 8192;          // row field of a padding entry: the zero row behind the slice
constexpr int kSlicedMaxGroups = 256;        // groups per range (8-bit field; 4 KiB of activations in LDS)
constexpr int kSlicedLdsBytes = 160 * 1024;
constexpr int kSlicedQuadBytes = 64 * 12;
constexpr uint32_t kSlicedNoRow = 0xFFFFFFFFu;

struct SlicedWave {
  uint32_t quad_begin;  // first 768-byte quad of the wave's strip
  uint32_t steps;       // entries per lane (0: the wave has no strip)
};

struct SlicedWorkgroup {  // 160 bytes
  uint32_t slice;         // codebook rows [slice * slice_rows, ...)
  uint32_t partial;       // which partial-sum vector receives the results
  uint32_t g_begin;       // group range [g_begin, g_begin + g_count)
  uint32_t g_count;
  uint32_t reserved[4];
  SlicedWave wave[kSlicedWaves];
};

static_assert(sizeof(npamd_sliced_header) == 128, "header is 128 bytes");
static_assert(sizeof(SlicedWorkgroup) == 160, "packed layout");

}  // namespace npamd
