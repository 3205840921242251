// Tile-decode GEMM: y = x @ W^T (+ bias) with W decoded inside the kernel,
// wave64 + MFMA 32x32x16, f32 accumulate.  The dense weight is never written.
//
// Block = 8 waves: four CONSUMER waves run the MFMAs, four PRODUCER waves
// decode the weight.  Output tile = BM x 64 with BM = 128*MW: consumer w owns
// rows [32*MW*w, 32*MW*(w+1)) of the tile and all 64 columns, so a weight
// element is decoded once per block and, for M <= 384, once per launch.  That
// matters because the decode (one 16-byte codebook gather per 8 weights,
// served by L2 for large codebooks) is the scarce resource, not the MFMA pipe:
// the producers exist to keep thousands of gathers in flight per CU, which the
// register-hungry consumers cannot do.
//
// One macro-step contracts 64 k = one packed "chunk" per weight row
// (providers.hpp).  Operand roles: A = x (rows m), B = W^T (columns n); for
// MFMA 32x32x16 lane l = (c = l % 32, h = l / 32) supplies 8 consecutive k of
// row c for k-half h, and MFMA j of a macro-step contracts
// k = 64*s + 32*h + 8*j .. +7.
//
// Both operands are staged in LDS so that 16-byte reads of 32 consecutive rows
// are bank-conflict free:
//   x tile  [BM][64 k], two or three buffers.  Every consumer fetches only the
//           rows it owns, one or more steps ahead, so the x tile needs no
//           synchronisation between waves.  The bytes go from memory straight
//           into LDS (swizzled 128-byte rows); see XStage.
//   W tile  [64][64 k], rows padded to 144 bytes, a ring of three.  Every
//           producer decodes a quarter of every step's tile (16 columns x 8 operands; lane = column x
//           operand pair), keeps kDepth steps in flight in registers -- packed
//           bytes and looked-up rows exactly as they arrived, all arithmetic on
//           them deferred to the iteration that needs its result -- and
//           writes a finished pair to LDS two iterations before its step.
// One block barrier per macro-step, executed by all eight waves.  Because the
// W tile of step t+1 is complete at the barrier that ends iteration t-1, a
// consumer fetches the first operands of step t+1 during the last MFMAs of
// step t: the matrix pipe does not drain across the barrier.
//
// Layers with few output columns (N = 4096: 64 column blocks) would leave most
// compute units idle, and the decode rate per compute unit is the limit; for
// them K is split over blockIdx.z, every split writes an f32 partial tile and
// a second kernel adds the splits (two or more addends in a fixed order), the
// bias, and rounds.
#pragma once

#include <atomic>

#include "gemv.hpp"
#include "providers.hpp"

namespace npamd {

constexpr int kStepK = 64;                      // k per macro-step (= one chunk)
constexpr int kRowBytes = kStepK * 2 + 16;      // padded LDS row stride
constexpr int kTileCols = 64;                   // output columns per block
constexpr int kWBufBytes = kTileCols * kRowBytes;
constexpr int kWRing = 3;                       // W tiles in LDS: read, complete, being written

struct GemmShape {
  const void* x;
  int64_t ldx;
  const float* bias;
  void* y;
  int64_t ldy;
  int M, N, K;
  int chunks;  // K / 64 = number of macro-steps
  int steps;   // == chunks
  // Split-K: blockIdx.z = split; split z contracts chunks [z * split_chunks, ...) and, when
  // splits > 1, stores its f32 tile to partials[z][M][N] (no bias) for splitk_reduce_kernel.
  int splits;
  int split_chunks;
  float* partials;
};

constexpr int kDepth = 8;  // steps in flight per producer wave (2 operands each)

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also drains
// every outstanding global load (vmcnt(0)), which would serialise the
// producers' in-flight gathers with each macro-step; here only LDS operations
// (lgkmcnt) are waited for.  Global loads are still waited for where their
// registers are consumed.
__device__ __forceinline__ void block_sync_lds() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}
// The same, except that the wave's KEEP youngest LDS operations may still be in flight: LDS
// operations of a wave complete in order, so everything issued before them (the producer's
// stores into the W tile) is done, while the codebook lookups it issued after the stores, whose
// results it needs many steps later, do not hold up the barrier.
template <int KEEP>
__device__ __forceinline__ void block_sync_lds_keep() {
  asm volatile("s_waitcnt lgkmcnt(%0)\n\ts_barrier" ::"n"(KEEP) : "memory");
}

// How the x tile reaches LDS: `global_load_lds_dwordx4` writes the loaded bytes straight into
// LDS, 64 lanes x 16 bytes = 1 KiB contiguous per instruction, with no register, no LDS store
// instruction and nothing for the issuing wave to wait for until the tile is read.  Rows are
// 128 bytes, unpadded (the transfer fills a contiguous KiB), and the 16-byte piece p of row r
// lies in slot p ^ ((r >> 1) & 7) of its row: a 16-byte read of 32 consecutive rows then touches
// every 16-byte bank group twice, as with padded rows.  A lane may fetch any source address, so
// the swizzle costs nothing at the load.  kBufs tiles are in LDS.  (Every provider takes x as
// it lies in memory; one that reordered k inside an operand would have to go through registers.)
// CB_LDS (codebooks of up to 64 KiB): the block copies the table into LDS behind the tiles and
// the producers look operands up there; to make room, two x tiles instead of three at 129..256
// tokens.  Larger tables and 257..384 tokens (LDS is full) gather from memory.
template <int MW, bool CB_LDS = false>
struct XStage {
  static constexpr int kBufs = (MW == 3 || (MW == 2 && CB_LDS)) ? 2 : 3;
  static constexpr int kXRowBytes = kStepK * 2;
  static constexpr int kBufBytes = 128 * MW * kXRowBytes;
  static constexpr int kLdsBytes = kBufs * kBufBytes + kWRing * kWBufBytes;  // the codebook copy follows
};
constexpr int kTileLdsCodebookMax = 64 * 1024;
constexpr int kTileLdsResidualMax = 16 * 1024;
constexpr int kLdsPerBlockMax = 160 * 1024;

// Output of one wave's MFMA 32x32 tiles: 32 MW rows x 32 NT columns of f32 sums (+ bias) -> 16-bit y.
// A lane holds one column of a tile, so storing from the registers is one 2-byte store per value
// (the vector memory path takes such an instruction lane by lane: 4 waves x 96..192 of them were
// 8 us of a 90 us launch).  Instead neighbouring lanes swap every second value, so that each
// holds two adjacent columns of one row, the pairs are parked in an LDS area of the wave's own
// (row-major, 16-byte pieces swizzled by row against bank conflicts), and the wave stores whole
// 16-byte pieces, 4 (NT = 4) or 8 (NT = 2) complete rows per instruction.
// `ep`: 32 MW x 64 NT bytes of LDS nobody else touches; y needs 16-byte aligned rows (else, and
// for the columns of a ragged last piece, element stores).
template <int NT>
__device__ __forceinline__ int ep_swizzle(int row, int piece) {
  const int g = NT == 4 ? ((row & 1) | (((row >> 2) & 1) << 1)) : ((row >> 2) & 1);
  return piece ^ (g << 2);
}
template <int ACT, int MW, int NT>
__device__ __forceinline__ void store_wave_tile(const f32x16 (&acc)[MW][NT], uint8_t* ep, int lane, void* y, int64_t ldy,
                                                int row0, int col0, int M, int N, const float* bias) {
  static_assert(NT == 2 || NT == 4, "two or four column tiles per wave");
  constexpr int kRowBytes = 64 * NT;
  const int c = lane & 31, h = lane >> 5;
  const bool odd = c & 1;
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int n = col0 + t * 32 + c;
    const float bv = (bias && n < N) ? bias[n] : 0.f;
#pragma unroll
    for (int mt = 0; mt < MW; ++mt) {
#pragma unroll
      for (int i = 0; i < 16; i += 2) {
        const float v0 = acc[mt][t][i] + bv, v1 = acc[mt][t][i + 1] + bv;
        // even lane keeps row i and gets the neighbour's (column c + 1); odd lane keeps row i + 1
        // neighbour in the lane pair, as a DPP move (quad_perm [1, 0, 3, 2]): one VALU instruction
        const float got = __builtin_bit_cast(
            float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, odd ? v0 : v1), 0xB1, 0xF, 0xF, true));
        const float lo = odd ? got : v0, hi = odd ? v1 : got;
        uint32_t packed;
        if constexpr (ACT == NPAMD_BF16) packed = f32_to_bf16_bits(lo) | (f32_to_bf16_bits(hi) << 16);
        else packed = f32_to_f16_bits(lo) | (f32_to_f16_bits(hi) << 16);
        const int row = mt * 32 + 8 * (i / 4) + 4 * h + (i % 4) + (odd ? 1 : 0);
        const int dw = t * 16 + (c >> 1);  // dword of the row: columns 2 dw, 2 dw + 1
        *reinterpret_cast<uint32_t*>(ep + row * kRowBytes + ep_swizzle<NT>(row, dw >> 2) * 16 + (dw & 3) * 4) = packed;
      }
    }
  }
  // The wave reads back what its own lanes wrote: LDS operations of a wave complete in order.
  constexpr int kPiecesPerRow = 4 * NT;            // 16-byte pieces
  constexpr int kRowsPerInst = 64 / kPiecesPerRow;  // 4 or 8
  const bool vec_ok = (ldy % 8 == 0) && ((reinterpret_cast<uintptr_t>(y) & 15) == 0);
  const int piece = lane % kPiecesPerRow;
  uint16_t* const yo = reinterpret_cast<uint16_t*>(y);
#pragma unroll
  for (int it = 0; it < 32 * MW / kRowsPerInst; ++it) {
    const int row = it * kRowsPerInst + lane / kPiecesPerRow;
    const int m = row0 + row, n = col0 + piece * 8;
    if (m >= M || n >= N) continue;
    const u32x4 v = *reinterpret_cast<const u32x4*>(ep + row * kRowBytes + ep_swizzle<NT>(row, piece) * 16);
    if (vec_ok && n + 8 <= N) {
      *reinterpret_cast<u32x4*>(yo + (int64_t)m * ldy + n) = v;
    } else {
      const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int e = 0; e < 8; ++e)
        if (n + e < N) yo[(int64_t)m * ldy + n + e] = (uint16_t)(w[e >> 1] >> (16 * (e & 1)));
    }
  }
}

template <int ACT, class Provider, int MW, bool CB_LDS = false>
__global__ void __launch_bounds__(512)
tile_gemm_kernel(const GemmShape s, const typename Provider::Args pargs) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  using XS = XStage<MW, CB_LDS && !Provider::kLdsResidual>;  // a residual table is small: no x tile given up
  constexpr int BM = 128 * MW;
  constexpr int kXBufBytes = XS::kBufBytes;
  uint8_t* const xs = lds;                             // [XS::kBufs][BM][XS::kXRowBytes]
  uint8_t* const ws = lds + XS::kBufs * kXBufBytes;    // [kWRing][64][kRowBytes]
  Provider prov(pargs);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: role branch is scalar
  const int m0 = blockIdx.y * BM;
  const int n0 = blockIdx.x * kTileCols;
  const int chunk0 = blockIdx.z * s.split_chunks;                 // first chunk of this split
  const int steps = min(s.split_chunks, s.chunks - chunk0);       // its number of macro-steps

  // Column blocks walk k in rotated order (iteration t contracts chunk
  // (t + rot) mod steps): at any instant different blocks read different parts
  // of the index rows and of x, which spreads the traffic over the L2 channels
  // instead of all blocks hitting the same few address bits in lock step.
  const int rot = (int)((blockIdx.x * 7u) % (unsigned)steps);
  auto chunk_of = [&](int step) {
    const int kc = step + rot;
    return chunk0 + (kc >= steps ? kc - steps : kc);
  };

  // Both software pipelines are unrolled by their depth with no branches inside
  // (a branch would make the compiler drain every outstanding load at the join),
  // so all waves run `total` iterations: steps rounded up to a multiple of kDepth.
  // The padding iterations decode clamped addresses into buffers nobody reads (lookups for steps past
  // the end all go to codebook row 0).
  const int total = (steps + kDepth - 1) / kDepth * kDepth;

  // Producer lane: column 16q + l % 16 of the tile, operand pair jp = l / 16 (see below).  Its
  // first packed bytes are requested here, in front of the codebook copy, so that the two
  // memory round trips at the start of a block overlap instead of following each other.
  const int pcol = 16 * (wave & 3) + (lane & 15);
  const int jp = lane >> 4;
  const int ncol = min(n0 + pcol, s.N - 1);  // columns past N read a clamped (valid) row
  typename Provider::PairRaw raws[kDepth];
  if (wave >= 4) {
    prov.prepare_row(ncol);
#pragma unroll
    for (int p = 0; p < kDepth; ++p) prov.load_pair(raws[p], ncol, chunk_of(min(p, steps - 1)), jp);
  }
  if constexpr (CB_LDS) {
    u32x4* cb_lds = reinterpret_cast<u32x4*>(lds + XS::kLdsBytes);
    const u32x4* src = prov.global_codebook();
    for (int i = threadIdx.x; i < prov.codebook_vec16(); i += 512) cb_lds[i] = src[i];
    prov.use_codebook(cb_lds);
    __syncthreads();
  }

  if (wave >= 4) {
    // ====================== producer wave q ================================
    // Every producer works every iteration on a quarter of the W tile: lane
    // (col = 16q + l % 16, jp = l / 16) owns operands 2jp and 2jp+1 of its
    // column, so the decode work (gathers, or int4 dequant VALU) is spread over
    // all four producers instead of falling on one wave per step.
    //
    // Software pipeline, kDepth steps deep, all in registers.  In iteration t
    // the wave
    //   1. writes the operands of step t+1 (issued kDepth iterations ago) to LDS,
    //   2. issues the gathers of step t+1+kDepth from packed bytes loaded kDepth
    //      iterations ago,
    //   3. loads the packed bytes of step t+1+2*kDepth.
    // Loads are consumed in the order they were issued, so waiting for the
    // oldest never drains the younger ones.  That only holds while nothing
    // touches a loaded value before its turn: the providers keep packed bytes
    // and looked-up rows as they arrived (load_pair, gather_pair) and do all
    // arithmetic on them in the iteration that needs the result (gather_pair on
    // the packed bytes, finish_pair on the rows) -- an index extraction or an
    // fp16 -> bf16 conversion placed next to its load makes the compiler wait
    // for that load, the youngest, and with it for every load in flight.
    // Branch-free decode: columns past N and steps past the last one read
    // clamped (valid) addresses; their results land where nobody looks.
    const int col = pcol;
    typename Provider::PairOps ops[kDepth];
    // LDS lookups that may stay in flight across the step's barrier (codebook in LDS only).
    constexpr int kKeep = CB_LDS ? Provider::kLdsOpsPerGather : 0;
    auto load_raw = [&](typename Provider::PairRaw& raw, int step) {
      prov.load_pair(raw, ncol, chunk_of(min(step, steps - 1)), jp);
    };
    auto store_w = [&](const typename Provider::PairOps& o, int slot) {
      u32x4 b0, b1;
      prov.finish_pair(o, b0, b1);
      uint8_t* dst = ws + slot * kWBufBytes + col * kRowBytes + jp * 32;
      *reinterpret_cast<u32x4*>(dst) = b0;
      *reinterpret_cast<u32x4*>(dst + 16) = b1;
    };
    // Iteration t: the operands of step t+2 (gathered kDepth iterations ago) go to ring slot
    // (t+2) % 3, their registers are refilled with the gathers of step t+2+kDepth, and the
    // packed bytes of step t+2+2*kDepth are requested.  The stores come first and the lookups
    // after them, in that order in the instruction stream: block_sync_lds_keep counts on it.
    auto advance = [&](typename Provider::PairOps& o, typename Provider::PairRaw& raw, int t, int slot) {
      store_w(o, slot);
      asm volatile("" ::: "memory");
      prov.gather_pair(raw, jp, o, t + 2 + kDepth < steps);
      load_raw(raw, t + 2 + 2 * kDepth);
    };

    // Prologue: steps 0..kDepth-1 in flight, packed bytes of kDepth..2*kDepth-1 loaded; then
    // "iterations -2 and -1": store steps 0 and 1 and refill their registers.
#pragma unroll
    for (int p = 0; p < kDepth; ++p) prov.gather_pair(raws[p], jp, ops[p], p < steps);  // packed bytes requested above
#pragma unroll
    for (int p = 0; p < kDepth; ++p) load_raw(raws[p], p + kDepth);
    advance(ops[0], raws[0], -2, 0);
    advance(ops[1], raws[1], -1, 1);
    block_sync_lds();

    // Iteration t handles step t+2, which lives in register set (t+2) % kDepth.
    int slot = 2;
    for (int t0 = 0; t0 < total; t0 += kDepth) {
#pragma unroll
      for (int d = 0; d < kDepth; ++d) {
        advance(ops[(d + 2) % kDepth], raws[(d + 2) % kDepth], t0 + d, slot);
        slot = slot == kWRing - 1 ? 0 : slot + 1;
        block_sync_lds_keep<kKeep>();
        // Operands that come from memory: nothing moves from one step into another.  Left
        // alone, the scheduler gathers the arithmetic of all kDepth steps of the unrolled body
        // at its top, and with it their waits, the last of which is for the gathers issued one
        // step earlier.  (With the codebook in LDS the free schedule already waits for the
        // oldest load only, and is the faster one at 128 tokens.)
        if constexpr (!CB_LDS || Provider::kLdsResidual) __builtin_amdgcn_sched_barrier(0);
      }
    }
    return;
  }

  // ========================= consumer wave ==================================
  const int c = lane & 31;
  const int h = lane >> 5;
  const int wrow0 = wave * (32 * MW);              // first tile row of this wave
  const bool wave_active = (m0 + wrow0) < s.M;     // false: every row of this wave lies past M
  const uint16_t* xg = reinterpret_cast<const uint16_t*>(s.x);

  if (!wave_active) {
    // All of this wave's rows lie past M (17..96 tokens leave one to three of the four consumers
    // without rows): it only keeps the others' barriers company, instead of reading the W tile and
    // running MFMAs on clamped rows -- at few tokens the LDS traffic per step sets the pace.
    block_sync_lds();
    for (int t = 0; t < total; ++t) block_sync_lds();
    return;
  }

  f32x16 acc[MW][2];
#pragma unroll
  for (int mt = 0; mt < MW; ++mt)
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mt][t][i] = 0.f;

  // ---- x tile by LDS-direct loads --------------------------------------------------------
  // Instruction i of a tile covers the wave's rows 8i .. 8i+7: lane l fills slot l & 7 of row
  // 8i + (l >> 3), i.e. fetches piece (l & 7) ^ ((row >> 1) & 7) of that row.  The address is
  // a scalar base (the wave's first row, this step's chunk) plus a 32-bit lane offset.
  constexpr int kPiecesW = 4 * MW;
  constexpr int kBufs = XS::kBufs;
  const int base_row = m0 + wrow0;                         // < M: waves without rows have left
  const uint8_t* const xbase = reinterpret_cast<const uint8_t*>(xg + (int64_t)base_row * s.ldx);
  uint32_t voff[kPiecesW];
#pragma unroll
  for (int i = 0; i < kPiecesW; ++i) {
    const int r = 8 * i + (lane >> 3);
    const int piece = (lane & 7) ^ ((r >> 1) & 7);
    voff[i] = (uint32_t)(((int64_t)min(r, s.M - 1 - base_row) * s.ldx + piece * 8) * 2);
  }
  const uint32_t xs_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)xs;
  const uint32_t wave_lds = xs_lds + (uint32_t)(wrow0 * XS::kXRowBytes);
  // The statement writes m0, which the compiler does not let an asm statement declare as
  // clobbered (a reserved register); it is sound as long as the compiler keeps nothing of its own
  // in m0 in this kernel, which tests/test_tile_gemm_codegen.py checks on the generated code.
  auto fetch_piece = [&](int i, int buf, const uint8_t* src) {
    const uint32_t dst = __builtin_amdgcn_readfirstlane(wave_lds + (uint32_t)(buf * kXBufBytes + i * 1024));
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :: "s"(dst), "v"(voff[i]), "s"(src) : "memory");
  };
  auto tile_src = [&](int step) { return xbase + (int64_t)chunk_of(min(step, steps - 1)) * (kStepK * 2); };
  // Operand sets in registers: the reads of k group j + kAhead are issued in front of the
  // MFMAs of group j.  One group ahead: reading three ahead (four sets, a fourth x tile) at up
  // to 128 tokens, where a group is only two MFMAs, changed nothing measurable.
  constexpr int kSets = 2;
  constexpr int kAhead = kSets - 1;
  constexpr int kPieceOfGroup[4] = {0, (kPiecesW + 2) / 3, (2 * kPiecesW + 2) / 3, kPiecesW};
  constexpr bool kIssueAtEnd = kBufs == 2;
  // The consumers issue no other vector memory instruction in the loop, so the in-order
  // counter counts tiles.  The first read of tile step + 1 comes in front of group 4 - kAhead
  // of step `step`; by then tiles up to step + kBufs - 2 are requested in full and of tile
  // step + kBufs - 1 the pieces issued behind the groups before that one, so tile step + 1
  // has landed once no more than those loads are outstanding.
  constexpr int kOutstandingOk = kIssueAtEnd ? 0 : (kBufs - 3) * kPiecesW + kPieceOfGroup[4 - kAhead];

  // With three or four tiles in LDS, tile step + kBufs - 1 is requested behind the MFMAs of k
  // groups 0..2 of step `step` (its buffer held tile step - 1).  With two, there is no such slack: tile
  // step + 2 goes into the buffer of tile `step` itself, as soon as that tile's last operands
  // have been read (behind the MFMAs of group 3), which leaves it almost two steps to arrive.
  constexpr int kPrologueTiles = kIssueAtEnd ? kBufs : kBufs - 1;
#pragma unroll
  for (int p = 0; p < kPrologueTiles; ++p) {
    const uint8_t* src = tile_src(p);
#pragma unroll
    for (int i = 0; i < kPiecesW; ++i) fetch_piece(i, p, src);
  }
  asm volatile("s_waitcnt vmcnt(%0)" :: "n"((kPrologueTiles - 1) * kPiecesW) : "memory");
  block_sync_lds();

  u32x4 a[kSets][MW], b[kSets][2];
  const uint32_t row_off = (uint32_t)((wrow0 + c) * XS::kXRowBytes);
  uint32_t slot_off[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) slot_off[j] = (uint32_t)((((h << 2) | j) ^ ((c >> 1) & 7)) << 4);
  auto read_ops = [&](int set, int buf, int wslot, int j) {
    const uint8_t* xa = xs + buf * kXBufBytes + row_off + slot_off[j];
    const uint8_t* wb = ws + wslot * kWBufBytes + c * kRowBytes + h * 64 + j * 16;
    b[set][0] = *reinterpret_cast<const u32x4*>(wb);
    b[set][1] = *reinterpret_cast<const u32x4*>(wb + 32 * kRowBytes);
#pragma unroll
    for (int mt = 0; mt < MW; ++mt)
      a[set][mt] = *reinterpret_cast<const u32x4*>(xa + mt * 32 * XS::kXRowBytes);
  };
  // buf = step % kBufs (compile-time through the unrolled loops below).
  auto one_step = [&](int buf, int step, int wslot) {
    const int wnext = wslot == kWRing - 1 ? 0 : wslot + 1;
    const int nbuf = buf == kBufs - 1 ? 0 : buf + 1;
    const int fbuf = kIssueAtEnd ? buf : (buf == 0 ? kBufs - 1 : buf - 1);  // where the requested tile goes
    const uint8_t* src = tile_src(kIssueAtEnd ? step + kBufs : step + kBufs - 1);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      constexpr int kFirstOfNext = 4 - kAhead;  // the group in front of which the next step's tiles are first read
      if (j < kFirstOfNext) {
        read_ops((j + kAhead) % kSets, buf, wslot, j + kAhead);
      } else {
        if (j == kFirstOfNext) asm volatile("s_waitcnt vmcnt(%0)" :: "n"(kOutstandingOk) : "memory");
        read_ops((j + kAhead) % kSets, nbuf, wnext, j + kAhead - 4);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int mt = 0; mt < MW; ++mt) {
        acc[mt][0] = mfma32<ACT>(a[j % kSets][mt], b[j % kSets][0], acc[mt][0]);
        acc[mt][1] = mfma32<ACT>(a[j % kSets][mt], b[j % kSets][1], acc[mt][1]);
      }
      if (!kIssueAtEnd && j < 3) {
#pragma unroll
        for (int i = kPieceOfGroup[j]; i < kPieceOfGroup[j + 1]; ++i) fetch_piece(i, fbuf, src);
      }
      if (kIssueAtEnd && j == 3) {
#pragma unroll
        for (int i = 0; i < kPiecesW; ++i) fetch_piece(i, fbuf, src);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };

#pragma unroll
  for (int g = 0; g < kAhead; ++g) read_ops(g, 0, 0, g);
  int wslot = 0;
  const int whole = steps / kBufs * kBufs;
  for (int t0 = 0; t0 < whole; t0 += kBufs) {
#pragma unroll
    for (int d = 0; d < kBufs; ++d) {
      one_step(d, t0 + d, wslot);
      wslot = wslot == kWRing - 1 ? 0 : wslot + 1;
      block_sync_lds();
    }
  }
#pragma unroll
  for (int d = 0; d < kBufs; ++d) {
    if (whole + d < steps) {
      one_step(d, whole + d, wslot);
      wslot = wslot == kWRing - 1 ? 0 : wslot + 1;
      block_sync_lds();
    }
  }
  for (int t = steps; t < total; ++t) block_sync_lds();
  // Nothing may still be on its way into LDS when the wave ends (the block's LDS is handed on).
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

  // ---- epilogue: D[m = 8*(i/4) + 4h + i%4][n = c] --------------------------
  if (s.splits <= 1) {
    // The rows this wave staged its x tile in (first buffer) are its own: 32 MW x 128 bytes.
    store_wave_tile<ACT, MW, 2>(acc, xs + wrow0 * XS::kXRowBytes, lane, s.y, s.ldy, m0 + wrow0, n0, s.M, s.N, s.bias);
    return;
  }
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const int n = n0 + t * 32 + c;
    if (n >= s.N) continue;
    float* part = s.partials + (size_t)blockIdx.z * s.M * s.N;
#pragma unroll
    for (int mt = 0; mt < MW; ++mt) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int m = m0 + wrow0 + mt * 32 + 8 * (i / 4) + 4 * h + (i % 4);
        if (m >= s.M) continue;
        part[(size_t)m * s.N + n] = acc[mt][t][i];
      }
    }
  }
}

// y[m][n] = round(sum over the splits of partials[z][m][n] + bias[n]); four columns per thread.
template <int ACT>
__global__ void __launch_bounds__(256)
splitk_reduce_kernel(const float* __restrict__ partials, int splits, int M, int N,
                     const float* __restrict__ bias, void* __restrict__ y, int64_t ldy) {
  const int64_t quads_per_row = (N + 3) / 4;
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= quads_per_row * M) return;
  const int m = (int)(i / quads_per_row);
  const int n = (int)(i - (int64_t)m * quads_per_row) * 4;
  float sum[4] = {0.f, 0.f, 0.f, 0.f};
  for (int z = 0; z < splits; ++z) {
    const float* p = partials + ((size_t)z * M + m) * N + n;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (n + j < N) sum[j] += p[j];
  }
#pragma unroll
  for (int j = 0; j < 4; ++j)
    if (n + j < N) store_from_f32<ACT>(y, (int64_t)m * ldy + n + j, sum[j] + (bias ? bias[n + j] : 0.f));
}

// Number of K splits for a tile GEMM of this shape: 1 while the (column block, row block) grid
// covers most compute units, else as many as fill them, each at least 8 macro-steps long.
int plan_tile_splits(int M, int N, int chunks, int mw);

// Rows per block: 128*MW with MW = ceil(M / 128) capped at 3, so that M <= 384
// is one row block and every weight element is decoded exactly once.
// NPAMD_TILE_MW overrides the choice (tuning aid).
int plan_tile_mw(int M);

bool tile_lds_codebook_enabled();  // NPAMD_TILE_LDS_CB=0 switches the LDS copy off (tuning aid)

template <int ACT, class Provider, int MW, bool CB_LDS>
int launch_tile_gemm_mw_cb(const GemmShape& s, const typename Provider::Args& pargs, int cb_bytes, hipStream_t st,
                           const char* what) {
  constexpr int BM = 128 * MW;
  const dim3 grid((s.N + kTileCols - 1) / kTileCols, (s.M + BM - 1) / BM, s.splits);
  const int lds = XStage<MW, CB_LDS && !Provider::kLdsResidual>::kLdsBytes + (CB_LDS ? cb_bytes : 0);
  static LdsLatch latch;  // per instantiation
  const hipError_t e =
      enable_dynamic_lds(latch, reinterpret_cast<const void*>(&tile_gemm_kernel<ACT, Provider, MW, CB_LDS>), lds);
  if (e != hipSuccess)
    return fail(NPAMD_ERR_LAUNCH, "%s: cannot reserve %d bytes of LDS: %s", what, lds, hipGetErrorString(e));
  tile_gemm_kernel<ACT, Provider, MW, CB_LDS><<<grid, 512, lds, st>>>(s, pargs);
  if (s.splits > 1) {
    const int64_t quads = (int64_t)s.M * ((s.N + 3) / 4);
    splitk_reduce_kernel<ACT><<<(unsigned)((quads + 255) / 256), 256, 0, st>>>(s.partials, s.splits, s.M, s.N,
                                                                             s.bias, s.y, s.ldy);
  }
  return check_launch(what);
}

// cb_bytes: size of the (single) codebook for providers that can look it up in LDS, else 0.
template <int ACT, class Provider, int MW>
int launch_tile_gemm_mw(const GemmShape& s, const typename Provider::Args& pargs, int cb_bytes, hipStream_t st,
                        const char* what) {
  if constexpr (Provider::kLdsResidual) {
    // Residual VQ: cb_bytes is the residual codebook; behind the tiles it takes half of the
    // producers' lookups off the vector memory path at every token count.
    if (cb_bytes > 0 && cb_bytes <= kTileLdsResidualMax && cb_bytes % 16 == 0 &&
        XStage<MW, false>::kLdsBytes + cb_bytes <= kLdsPerBlockMax && tile_lds_codebook_enabled())
      return launch_tile_gemm_mw_cb<ACT, Provider, MW, true>(s, pargs, cb_bytes, st, what);
  }
  if constexpr (Provider::kLdsCodebook && MW < 3) {
    // At 129..256 tokens the copy costs the third x tile: worth it only for tables the vector L1
    // does not hold anyway (14336 x 4096 at 256 tokens: 4096 rows 64 -> 57 us, 256 rows 49 -> 53 us).
    const bool pays = MW == 1 || cb_bytes > 16 * 1024;
    if (pays && cb_bytes > 0 && cb_bytes <= kTileLdsCodebookMax && cb_bytes % 16 == 0 &&
        XStage<MW, true>::kLdsBytes + cb_bytes <= kLdsPerBlockMax && tile_lds_codebook_enabled())
      return launch_tile_gemm_mw_cb<ACT, Provider, MW, true>(s, pargs, cb_bytes, st, what);
  }
  return launch_tile_gemm_mw_cb<ACT, Provider, MW, false>(s, pargs, 0, st, what);
}

// `workspace` (f32, may be null) decides whether K may be split: it must hold splits * M * N floats.
template <int ACT, class Provider>
int launch_tile_gemm(GemmShape s, const typename Provider::Args& pargs, hipStream_t st,
                     const char* what, void* workspace = nullptr, int64_t workspace_bytes = 0, int cb_bytes = 0) {
  s.steps = s.chunks;
  const int mw = plan_tile_mw(s.M);
  int splits = workspace ? plan_tile_splits(s.M, s.N, s.chunks, mw) : 1;
  while (splits > 1 && (int64_t)splits * s.M * s.N * 4 > workspace_bytes) --splits;
  s.splits = splits;
  s.split_chunks = (s.chunks + splits - 1) / splits;
  s.splits = (s.chunks + s.split_chunks - 1) / s.split_chunks;  // no empty split
  s.partials = (float*)workspace;
  switch (mw) {
    case 1: return launch_tile_gemm_mw<ACT, Provider, 1>(s, pargs, cb_bytes, st, what);
    case 2: return launch_tile_gemm_mw<ACT, Provider, 2>(s, pargs, cb_bytes, st, what);
    default: return launch_tile_gemm_mw<ACT, Provider, 3>(s, pargs, cb_bytes, st, what);
  }
}

// ---------------------------------------------------------------------------
// Fallback for shapes the MFMA kernel does not take: the element-wise GEMV kernel
// over blocks of 16 tokens (the weight is decoded once per block).  Slow; exists so
// every valid input has a HIP path.  The modules send such layers to decode + GEMM.
// ---------------------------------------------------------------------------
template <int ACT, class Elem>
int launch_generic_gemm(const void* x, int64_t ldx, const float* bias, void* y, int64_t ldy,
                        int M, int N, int K, const Elem& elem, hipStream_t st, const char* what) {
  return launch_generic_gemv<ACT, Elem>(x, ldx, bias, y, ldy, M, N, K, elem, st, what);
}

}  // namespace npamd
