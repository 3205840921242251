// The 128-column tile-decode GEMM (see gemm_tile2.hpp): kernel, weight-tile producers and launchers.
#include "gemm_tile2.hpp"

#include <stdlib.h>

#include <atomic>
#include <chrono>
#include <random>

#include <type_traits>

namespace npamd {

// A number for one call of the kernel whose two K halves meet through the workspace: the tile words
// there need no clearing, because a word only counts while it holds the number of the call that
// reads it, and 64 pseudo-random bits are never what memory happens to hold (the finishing
// workgroup stores zero over it, so a graph that replays one call, number included, starts clean).
static unsigned long long next_call_number() {
  static std::atomic<unsigned long long> counter{[] {
    std::random_device rd;
    return ((unsigned long long)rd() << 32) ^ (unsigned long long)rd() ^
           (unsigned long long)std::chrono::steady_clock::now().time_since_epoch().count();
  }()};
  unsigned long long z = counter.fetch_add(0x9E3779B97F4A7C15ull) + 0x9E3779B97F4A7C15ull;  // splitmix64
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  z ^= z >> 31;
  return z ? z : 1ull;  // zero is what a finished tile holds
}

// Four 16-byte stores of agent scope (sc1: coherent between the L2 caches of the GPU's dies without a
// cache write-back), 1 KiB apart: one 32 x 32 result tile of a wave.  `p`: the lane's address.
__device__ __forceinline__ void store4_sc1(float* p, const f32x4& v0, const f32x4& v1, const f32x4& v2, const f32x4& v3) {
  asm volatile(
      "global_store_dwordx4 %0, %1, off sc1\n\tglobal_store_dwordx4 %0, %2, off offset:1024 sc1\n\t"
      "global_store_dwordx4 %0, %3, off offset:2048 sc1\n\tglobal_store_dwordx4 %0, %4, off offset:3072 sc1"
      ::"v"(p), "v"(v0), "v"(v1), "v"(v2), "v"(v3)
      : "memory");
}

// Cache policy bits of a raw buffer load: bit 4 is sc1 (agent scope).
constexpr int kAuxSc1 = 16;

// A pointer that is the same in every lane, said so to the compiler (an "s" operand has to live in scalar registers).
__device__ __forceinline__ const uint8_t* uniform_ptr(const uint8_t* p) {
  const uint64_t v = reinterpret_cast<uint64_t>(p);
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  return reinterpret_cast<const uint8_t*>(((uint64_t)hi << 32) | lo);
}
// Loads that write LDS directly: lane l's 16 (4) bytes land at dst + 16 l (4 l); dst is uniform
// over the wave.  The statements write m0, which the compiler does not let an asm statement declare
// as clobbered; that is sound as long as the compiler keeps nothing of its own in m0 in these kernels.
__device__ __forceinline__ void lds_load16(uint32_t dst, uint32_t voff, const void* base) {
  dst = __builtin_amdgcn_readfirstlane(dst);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(voff), "s"(base) : "memory");
}
__device__ __forceinline__ void lds_load4(uint32_t dst, uint32_t voff, const void* base) {
  dst = __builtin_amdgcn_readfirstlane(dst);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" ::"s"(dst), "v"(voff), "s"(base) : "memory");
}

// The block's walk over K: step t contracts chunk (t + rot) mod steps of the block's range (column
// blocks start at different chunks, which spreads the traffic over the L2 channels); steps past the
// end repeat the last one (their loads land where nobody looks).
struct KWalk {
  int chunk0, steps, rot;
  __device__ __forceinline__ int chunk_of(int step) const {
    const int kc = min(step, steps - 1) + rot;
    return chunk0 + (kc >= steps ? kc - steps : kc);
  }
};

// ---------------------------------------------------------------------------------------------
// Producer: VQ, 16-bit indices, vector length 8, codebook in the activation dtype, looked up in
// memory.  A weight operand is one codebook row: the lookup is a load that writes the W slot directly.
//
// Wave w serves column tile w % 4 and the operand pair J = w / 4.  Lane (c, h) reads its two indices
// (k = 32 h + 16 J .. + 15 of the step) as one dword from the staged indices and issues two lookups,
// which land in KiB (w % 4, 2 J) and (w % 4, 2 J + 1) of the W slot; in step t it looks up the rows of
// step t + 2 (W ring of three).  Indices are staged four steps at a time: a column's 64 bytes of a
// quad of steps are half a cache line, and one load instruction fetches them for sixteen columns (16
// lines; a load of one step's 16 bytes for 32 columns touches 32, and the address unit's time goes
// with the lines).  Per column tile two quads of 32 columns x 64 bytes, wave w fetching columns
// 16 J .. 16 J + 15; piece p of column r sits in slot p ^ ((r >> 2) & 3) of its row, which spreads the
// reads of 32 columns over the banks.  What one wave loads another reads, which is safe because
// everything a step issues is waited for by the issuer at the end of the next step at the latest,
// in front of a barrier, and read after it.
// ---------------------------------------------------------------------------------------------
template <int ACT>
struct T2ProdVq16 {
  using Args = T2Args;
  static constexpr int kWRing = 3;
  static constexpr int kLoads = 2;
  static constexpr int kQuadLoads = 1;
  static constexpr int kHandoffBatch = 3;  // row tiles of the other half's tile loaded per round trip (registers)
  static constexpr int kQuadBytes = 32 * 64;
  static constexpr int kStageBytes = 4 * 2 * kQuadBytes;
  const Args& a;
  const KWalk& kw;
  int tcol, J, c, h;
  uint8_t* stage;
  uint32_t stage_lds, ws_lds;
  uint32_t row_off;
  int piece;
  __device__ T2ProdVq16(const Args& args, const KWalk& walk, int wave, int lane, int n0, int N, uint8_t* /*ws*/,
                         uint32_t ws_lds_, uint8_t* stage_, uint32_t stage_lds_)
      : a(args), kw(walk), tcol(wave & 3), J(wave >> 2), c(lane & 31), h(lane >> 5), stage(stage_), stage_lds(stage_lds_),
        ws_lds(ws_lds_) {
    const int r = 16 * J + (lane >> 2);
    const int n = min(n0 + 32 * tcol + r, N - 1);  // columns past N fetch a valid row nobody stores
    row_off = (uint32_t)n * (uint32_t)args.chunks * 16u;
    piece = (lane & 3) ^ ((lane >> 4) & 3);  // slot ^ ((r >> 2) & 3)
  }
  __device__ __forceinline__ void load_quad(int quad) const {
    const uint32_t chunk = (uint32_t)kw.chunk_of(4 * quad + piece) * 16u;
    lds_load16(stage_lds + (uint32_t)((tcol * 2 + (quad & 1)) * kQuadBytes + J * 1024), row_off + chunk, a.packed);
  }
  __device__ __forceinline__ void gathers(int step, int slot) const {
    const int q = step >> 2, p = step & 3;
    const uint32_t v = *reinterpret_cast<const uint32_t*>(stage + (tcol * 2 + (q & 1)) * kQuadBytes + c * 64 +
                                                          ((p ^ ((c >> 2) & 3)) << 4) + h * 8 + J * 4);
    const uint32_t off0 = min(v & 0xFFFFu, a.nc_minus_1) << 4, off1 = min(v >> 16, a.nc_minus_1) << 4;
    const uint32_t dst = ws_lds + (uint32_t)(slot * kT2WSlotBytes + (tcol * 4 + 2 * J) * 1024);
    lds_load16(dst, off0, a.cb);
    lds_load16(dst + 1024u, off1, a.cb);
  }
  __device__ __forceinline__ bool loads_quad(int step) const { return (step & 3) == 2; }
  // Index quads 0 and 1; then, once they are there and the waves have met, the W tiles of steps 0 and 1.
  __device__ __forceinline__ void prologue_issue() const {
    load_quad(0);
    load_quad(1);
  }
  __device__ __forceinline__ void prologue_finish() const {
    gathers(0, 0);
    gathers(1, 1);
  }
  // Work behind the MFMAs of k group J_, column tile T of `step` (W slot wslot = step % 3); `rem`: steps
  // after this one, 2 standing for two or more.  In step t the wave looks up its rows of step t + 2.
  template <int J_, int T>
  __device__ __forceinline__ void work(int step, int wslot, int rem) const {
    if (rem < 2) return;
    if (J_ == 3 && T == 0) gathers(step + 2, wslot == 0 ? 2 : wslot - 1);
    if (J_ == 3 && T == 1 && loads_quad(step)) load_quad((step >> 2) + 2);
  }
  __device__ __forceinline__ void work_all(int step, int wslot, int rem) const {
    work<3, 0>(step, wslot, rem);
    work<3, 1>(step, wslot, rem);
  }
  // Everything but the loads this step issued last (its lookups, and the index quad behind them in
  // the steps that fetch one) has to be there when the next step starts.
  __device__ __forceinline__ void wait_step_end(int step, int rem) const {
    if (rem < 2) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    else if (loads_quad(step)) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kLoads + kQuadLoads) : "memory");
    else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kLoads) : "memory");
  }
};

// ---------------------------------------------------------------------------------------------
// Producers: int4 / int8 group-affine codes.  Packed bytes and the dword that holds the group's scale
// (and zero point) go to an LDS staging ring of three steps per column tile (directly, like
// everything else the kernel loads, so that one in-order counter tracks all of a wave's loads).  Wave
// w decodes the operand pair J = w / 4 of column tile w % 4; the two waves of a column tile share its
// ring and request the bytes of alternate steps.  In step t the bytes of step t + 3 are requested,
// the operands of step t + 1 decoded from registers into the other W slot (ring of two) between
// the MFMAs, and the bytes of step t + 2 read out of the ring, a barrier ahead of their decoding so
// that it never waits for LDS.  The arithmetic is the providers' (providers.hpp): bit for bit the
// one-pass decode.
// ---------------------------------------------------------------------------------------------
template <int ACT, int NBITS, bool ASYM>
struct T2ProdQ {
  using P = typename std::conditional<NBITS == 4, Q4Provider<ACT, ASYM>, Q8Provider<ACT, ASYM>>::type;
  using Args = typename P::Args;
  static constexpr int kWRing = 2;
  static constexpr int kCodeLoads = NBITS == 4 ? 1 : 2;
  static constexpr int kSlot = kCodeLoads * 1024 + 256 + (ASYM ? 256 : 0);
  static constexpr int kHandoffBatch = 2;
  static constexpr int kStageTile = 3 * kSlot;
  static constexpr int kStageBytes = 4 * kStageTile;
  const Args& a;
  const KWalk& kw;
  const P prov;
  int tcol, J, lane, h;
  uint8_t* ws;
  uint8_t* stage;      // this column tile's ring
  uint32_t stage_lds;
  uint32_t code_off;   // byte offset of the lane's share of chunk 0 of its row
  uint32_t scale_row;  // index of the row's first scale
  int cur = 0;         // step % 3: the ring slot the bytes of step + 3 go to
  u32x2 raw0, raw1;    // the operand pair being decoded
  uint32_t s2, z;
  __device__ T2ProdQ(const Args& args, const KWalk& walk, int wave, int lane_, int n0, int N, uint8_t* ws_, uint32_t /*ws_lds*/,
                      uint8_t* stage_, uint32_t stage_lds_)
      : a(args), kw(walk), prov(args), tcol(wave & 3), J(wave >> 2), lane(lane_), h(lane_ >> 5), ws(ws_),
        stage(stage_ + (wave & 3) * kStageTile), stage_lds(stage_lds_ + (uint32_t)((wave & 3) * kStageTile)) {
    const int ncol = min(n0 + 32 * tcol + (lane_ & 31), N - 1);  // columns past N decode a valid row nobody stores
    code_off = (uint32_t)ncol * (uint32_t)args.chunks * (NBITS == 4 ? 32u : 64u) + (uint32_t)h * (NBITS == 4 ? 16u : 32u);
    scale_row = (uint32_t)ncol * (uint32_t)args.groups_per_row;
  }
  __device__ __forceinline__ uint32_t scale_index(int step) const {
    return scale_row + (uint32_t)((2 * kw.chunk_of(step) + h) >> a.gs_shift_chunks);
  }
  // The packed bytes and scales of `step` into ring slot `slot` (by the wave whose J is the step's parity).
  __device__ __forceinline__ void request(int step, int slot) const {
    if ((step & 1) != J) return;
    const uint32_t dst = stage_lds + (uint32_t)(slot * kSlot);
    const uint32_t off = code_off + (uint32_t)kw.chunk_of(step) * (NBITS == 4 ? 32u : 64u);
    lds_load16(dst, off, a.w_pack);
    if (NBITS == 8) lds_load16(dst + 1024, off + 16u, a.w_pack);
    const uint32_t sb = (scale_index(step) * 2u) & ~3u;
    lds_load4(dst + kCodeLoads * 1024, sb, a.scale);
    if (ASYM) lds_load4(dst + kCodeLoads * 1024 + 256, sb, a.zp);
  }
  // Reads the wave's half of the staged bytes of `step` out of ring slot `slot`.
  __device__ __forceinline__ void fetch(int step, int slot) {
    const uint8_t* src = stage + slot * kSlot;
    if (NBITS == 4) {
      raw0 = *reinterpret_cast<const u32x2*>(src + lane * 16 + J * 8);
    } else {  // operand O of a lane: dwords 2 (O & 1), 2 (O & 1) + 1 of its 16 bytes in KiB O / 2
      const u32x4 r = *reinterpret_cast<const u32x4*>(src + J * 1024 + lane * 16);
      raw0 = u32x2{r.x, r.y};
      raw1 = u32x2{r.z, r.w};
    }
    const uint32_t sh = (scale_index(step) & 1u) * 16u;
    const uint32_t sd = *reinterpret_cast<const uint32_t*>(src + kCodeLoads * 1024 + lane * 4);
    s2 = ((sd >> sh) & 0xFFFFu) * 0x10001u;
    z = 0;
    if (ASYM) z = (*reinterpret_cast<const uint32_t*>(src + kCodeLoads * 1024 + 256 + lane * 4) >> sh) & 0xFFFFu;
  }
  template <int I>
  __device__ __forceinline__ void decode(int wslot) const {
    u32x4 op;
    if constexpr (NBITS == 4) op = prov.dequant8(I == 0 ? raw0.x : raw0.y, s2, z);
    else op = I == 0 ? prov.dequant8(raw0.x, raw0.y, s2, z) : prov.dequant8(raw1.x, raw1.y, s2, z);
    *reinterpret_cast<u32x4*>(ws + wslot * kT2WSlotBytes + (tcol * 4 + 2 * J + I) * 1024 + lane * 16) = op;
  }
  __device__ __forceinline__ void prologue_issue() const {
    request(0, 0);
    request(1, 1);
    request(2, 2);
  }
  // Everything requested has arrived: the W tile of step 0, and the bytes of step 1 in registers.
  __device__ __forceinline__ void prologue_finish() {
    fetch(0, 0);
    decode<0>(0);
    decode<1>(0);
    fetch(1, 1);
  }
  // In step t: the bytes of step t + 3 requested (they are waited for with the x pieces at the end of
  // the step), the operands of step t + 1 decoded from the registers into the other W slot, and the
  // bytes of step t + 2 read out of the ring a barrier ahead of their decoding.
  template <int J_, int T>
  __device__ __forceinline__ void work(int step, int wslot, int rem) {
    if (J_ == 0 && T == 0 && rem >= 2) request(step + 3, cur);
    if (J_ == 1 && T == 0 && rem >= 1) decode<0>(wslot ^ 1);
    if (J_ == 2 && T == 0 && rem >= 1) decode<1>(wslot ^ 1);
    if (J_ == 3 && T == 1) {
      if (rem >= 2) fetch(step + 2, cur == 0 ? 2 : cur - 1);
      cur = cur == 2 ? 0 : cur + 1;
    }
  }
  __device__ __forceinline__ void work_all(int step, int wslot, int rem) {
    work<0, 0>(step, wslot, rem);
    work<1, 0>(step, wslot, rem);
    work<2, 0>(step, wslot, rem);
    work<3, 1>(step, wslot, rem);
  }
  __device__ __forceinline__ void wait_step_end(int, int) const { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
};

template <int ACT, int MW, class Prod>
__global__ void __launch_bounds__(512)
tile2_gemm_kernel(const GemmShape s, const typename Prod::Args pargs, const T2Pair pair) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  constexpr int BM = 128 * MW;
  constexpr int kXBufBytes = 128 * MW * kStepK * 2;
  constexpr int kPieces = 2 * MW;  // x-tile load instructions per wave and step (8 rows each): half of the pair's
  constexpr int kWRing = Prod::kWRing;
  static_assert(2 * kXBufBytes + kWRing * kT2WSlotBytes + Prod::kStageBytes <= kLdsPerBlockMax, "the block's tiles do not fit LDS");
  uint8_t* const xs = lds;                              // [2][BM][128]
  uint8_t* const ws = lds + 2 * kXBufBytes;             // [kWRing][16 KiB]
  uint8_t* const stage = ws + kWRing * kT2WSlotBytes;   // the producer's staging area

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int rg = wave & 3;   // row group: rows [32 MW rg, 32 MW (rg + 1)) of the block tile
  const int ch = wave >> 2;  // column half: columns [64 ch, 64 ch + 64)
  const int c = lane & 31;
  const int h = lane >> 5;
  // Workgroups go to the GPU's eight dies in turn (linear workgroup index mod 8).  When the grid has 2, 4 or
  // 8 (row block, part of K) pairs per column block, each pair gets dies of its own, so that a die's L2 holds the
  // x tile of one row block and one part of K next to the codebook instead of all of x (which, from 512 tokens
  // at K = 4096, is more than an L2 holds).
  int bx = blockIdx.x, by = blockIdx.y, bz = blockIdx.z;
  {
    const int groups = gridDim.y * gridDim.z;
    // Measured: 14336 x 4096 int4 at 512 / 1024 tokens 82.5 / 150 us against 88 / 164; with K in more than two
    // parts (layers of few columns) the parts are better left spread over all dies (4096 x 4096 int4 at 256
    // tokens: 30.6 us spread, 34.4 with a die per part).
    if (gridDim.z <= 2 && (groups == 2 || groups == 4 || groups == 8)) {
      const int dies = 8 / groups;  // per group
      if (gridDim.x % dies == 0) {
        const int id = (blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x;
        const int die = id & 7, group = die / dies;
        bx = (id >> 3) * dies + die % dies;
        by = group % (int)gridDim.y;
        bz = group / (int)gridDim.y;
      }
    }
  }
  const int m0 = by * BM;
  const int n0 = bx * kT2Cols;
  KWalk kw;
  kw.chunk0 = bz * s.split_chunks;
  kw.steps = min(s.split_chunks, s.chunks - kw.chunk0);
  kw.rot = (int)((bx * 7u) % (unsigned)kw.steps);
  const int steps = kw.steps;

  const uint32_t xs_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)xs;
  Prod prod(pargs, kw, wave, lane, n0, s.N, ws, (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)ws, stage,
            (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)stage);

  // ---- x tile: pieces 2 i + ch of the pair's rows ---------------------------------------------------
  const int wrow0 = rg * (32 * MW);
  const bool wave_active = (m0 + wrow0) < s.M;
  const int base_row = min(m0 + wrow0, s.M - 1);
  const uint8_t* const xbase = reinterpret_cast<const uint8_t*>(s.x) + (int64_t)base_row * s.ldx * 2;
  uint32_t voff[kPieces];
#pragma unroll
  for (int i = 0; i < kPieces; ++i) {
    const int r = 8 * (2 * i + ch) + (lane >> 3);
    const int piece = (lane & 7) ^ ((r >> 1) & 7);
    voff[i] = (uint32_t)(((int64_t)min(r, s.M - 1 - base_row) * s.ldx + piece * 8) * 2);
  }
  const uint32_t wave_x_lds = xs_lds + (uint32_t)(wrow0 * 128 + ch * 1024);
  auto fetch_piece = [&](int i, int buf, const uint8_t* src) {
    lds_load16(wave_x_lds + (uint32_t)(buf * kXBufBytes + i * 2048), voff[i], src);
  };
  auto tile_src = [&](int step) { return uniform_ptr(xbase + (int64_t)kw.chunk_of(step) * (kStepK * 2)); };

  // ---- prologue: index quads 0 and 1 and the x tile of step 0, then the W tiles of steps 0 and 1 ----
  prod.prologue_issue();
  if (wave_active) {
    const uint8_t* src = tile_src(0);
#pragma unroll
    for (int i = 0; i < kPieces; ++i) fetch_piece(i, steps & 1, src);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  block_sync_lds();
  prod.prologue_finish();
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  block_sync_lds();

  // The word through which the two halves of K meet is looked at a step before the loop ends, so that
  // the look costs no round trip after it: a stale "not there yet" only means that this half
  // writes its tile, and the swap that follows decides.
  unsigned long long* const word = pair.words + (by * gridDim.x + bx);
  unsigned long long early = 0;
  auto early_look = [&] {
    if (s.splits == 2 && tid == 0) early = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  };

  f32x16 acc[MW][2];
#pragma unroll
  for (int mt = 0; mt < MW; ++mt)
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mt][t][i] = 0.f;

  if (wave_active) {
    u32x4 ao[2][MW] = {}, bo[2][2] = {};
    const uint32_t row_off = (uint32_t)((wrow0 + c) * 128);
    uint32_t slot_off[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) slot_off[j] = (uint32_t)((((h << 2) | j) ^ ((c >> 1) & 7)) << 4);
    auto read_ops = [&](int set, int buf, int wslot, int j) {
      const uint8_t* wb = ws + wslot * kT2WSlotBytes + ch * 8192 + j * 1024 + lane * 16;
#pragma unroll
      for (int t = 0; t < 2; ++t) bo[set][t] = *reinterpret_cast<const u32x4*>(wb + t * 4096);
      const uint8_t* xa = xs + buf * kXBufBytes + row_off + slot_off[j];
#pragma unroll
      for (int mt = 0; mt < MW; ++mt) ao[set][mt] = *reinterpret_cast<const u32x4*>(xa + mt * 32 * 128);
    };
    // One step: eight (k group, column tile) slots of MW MFMAs; behind them, one instruction per
    // slot, the wave's x pieces of step + 1 (other buffer), and the producer's work.  `rem`: steps after
    // this one, 2 standing for two or more; the last step has no x tile to fetch and the producers
    // leave out what would serve steps past the end.
    auto one_step = [&](int buf, int step, int wslot, int rem) {
      read_ops(0, buf, wslot, 0);
      const uint8_t* src = tile_src(step + 1);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (j < 3) read_ops((j + 1) & 1, buf, wslot, j + 1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < 2; ++t) {
#pragma unroll
          for (int mt = 0; mt < MW; ++mt) acc[mt][t] = mfma32<ACT>(ao[j & 1][mt], bo[j & 1][t], acc[mt][t]);
          if (rem >= 1 && j * 2 + t < kPieces) fetch_piece(j * 2 + t, buf ^ 1, src);
          if (j == 0 && t == 0) prod.template work<0, 0>(step, wslot, rem);
          if (j == 0 && t == 1) prod.template work<0, 1>(step, wslot, rem);
          if (j == 1 && t == 0) prod.template work<1, 0>(step, wslot, rem);
          if (j == 1 && t == 1) prod.template work<1, 1>(step, wslot, rem);
          if (j == 2 && t == 0) prod.template work<2, 0>(step, wslot, rem);
          if (j == 2 && t == 1) prod.template work<2, 1>(step, wslot, rem);
          if (j == 3 && t == 0) prod.template work<3, 0>(step, wslot, rem);
          if (j == 3 && t == 1) prod.template work<3, 1>(step, wslot, rem);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      prod.wait_step_end(step, rem);
      if (rem >= 1) block_sync_lds();
    };
    // Step t reads x buffer (t + steps) % 2, so that the last two steps, which are instantiated
    // apart, and the pairs of the loop in front of them always see buffers 0 and 1 in this order;
    // an odd number of steps starts with a step of its own on buffer 1.
    int wslot = 0;
    auto next_slot = [&] { wslot = wslot == kWRing - 1 ? 0 : wslot + 1; };
    const int odd = steps & 1;
    if (odd) {
      one_step(1, 0, wslot, 2);
      next_slot();
    }
    for (int t0 = odd; t0 < steps - 2; t0 += 2) {
#pragma unroll
      for (int d = 0; d < 2; ++d) {
        one_step(d, t0 + d, wslot, 2);
        next_slot();
      }
    }
    one_step(0, steps - 2, wslot, 1);
    next_slot();
    early_look();
    one_step(1, steps - 1, wslot, 0);
  } else {
    // No rows of this pair of waves lie inside M: they still decode their share of the weights.
    int wslot = 0;
    for (int t = 0; t < steps - 1; ++t) {
      const int rem = min(steps - 1 - t, 2);
      prod.work_all(t, wslot, rem);
      prod.wait_step_end(t, rem);
      block_sync_lds();
      wslot = wslot == kWRing - 1 ? 0 : wslot + 1;
    }
  }
  // Nothing may still be on its way into LDS when the wave ends.
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

  // ---- epilogue: D[m = 8 (i / 4) + 4 h + i % 4][n = c] of each 32 x 32 tile ---------------------
  bool finish = true;
  if (s.splits == 2) {
    const int tile_id = by * gridDim.x + bx;
    const int tiles = gridDim.x * gridDim.y;
    constexpr int kTileFloats = BM * kT2Cols;
    // [tile][wave][row tile mt][column tile t][quarter q][lane] float4: 1 KiB per instruction
    float* const mine = pair.tiles + ((size_t)bz * tiles + tile_id) * kTileFloats + wave * (MW * 2 * 1024) + lane * 4;
    const float* const theirs_wave =
        pair.tiles + ((size_t)(bz ^ 1) * tiles + tile_id) * kTileFloats + wave * (MW * 2 * 1024);
    unsigned long long* const flag = reinterpret_cast<unsigned long long*>(stage);  // read for the last time two steps ago
    if (tid == 0) flag[0] = early;
    __syncthreads();  // every wave is past its last LDS read
    bool arrived = flag[0] == pair.call;  // the other half is there already: nothing to write
    if (!arrived) {
      if (wave_active) {
#pragma unroll
        for (int mt = 0; mt < MW; ++mt)
#pragma unroll
          for (int t = 0; t < 2; ++t) {
            const f32x16& r = acc[mt][t];
            store4_sc1(mine + (mt * 2 + t) * 1024, f32x4{r[0], r[1], r[2], r[3]}, f32x4{r[4], r[5], r[6], r[7]},
                       f32x4{r[8], r[9], r[10], r[11]}, f32x4{r[12], r[13], r[14], r[15]});
          }
      }
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the tile is where the other workgroup will read it
      __syncthreads();
      if (tid == 0) flag[1] = __hip_atomic_exchange(word, pair.call, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __syncthreads();
      arrived = flag[1] == pair.call;  // it came while this half was being written
    }
    finish = arrived;
    if (finish) {
      if (tid == 0) __hip_atomic_store(word, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // for a replay of this call
      if (wave_active) {
        // The other half's tile in one round trip: buffer loads of agent scope (cache policy sc1),
        // which the compiler, unlike atomic loads, leaves in flight together.
        const __amdgpu_buffer_rsrc_t rsrc =
            __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(theirs_wave), 0, MW * 2 * 4096, 0x00020000);
        constexpr int kBatch = Prod::kHandoffBatch < MW ? Prod::kHandoffBatch : MW;  // row tiles per round trip
#pragma unroll
        for (int m0t = 0; m0t < MW; m0t += kBatch) {
          f32x4 v[kBatch][8];
#pragma unroll
          for (int b = 0; b < kBatch; ++b)
#pragma unroll
            for (int i = 0; i < 8; ++i)
              if (m0t + b < MW)
                v[b][i] = __builtin_bit_cast(
                    f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, ((m0t + b) * 8 + i) * 1024 + lane * 16, 0, kAuxSc1));
#pragma unroll
          for (int b = 0; b < kBatch; ++b)
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
              for (int i = 0; i < 16; ++i)
                if (m0t + b < MW) acc[m0t + b][t][i] += v[b][t * 4 + i / 4][i % 4];
        }
      }
    }
  }
  if (s.splits <= 2) {
    // y through LDS (see store_wave_tile): every wave takes 32 MW x 128 bytes of the x buffers.
    if (s.splits != 2) __syncthreads();  // every wave is past its last LDS read (the pair path has met already)
    if (finish && wave_active)
      store_wave_tile<ACT, MW, 2>(acc, lds + wave * (32 * MW * 128), lane, s.y, s.ldy, m0 + wrow0, n0 + 64 * ch, s.M, s.N,
                                  s.bias);
    return;
  }
  if (!wave_active) return;
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const int n = n0 + 64 * ch + t * 32 + c;
    if (n >= s.N) continue;
    float* part = s.partials + (size_t)bz * s.M * s.N;
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

template <int ACT, int MW, class Prod>
int launch_tile2_mw(const GemmShape& s, const typename Prod::Args& a, const T2Pair& pair, hipStream_t st, const char* what) {
  constexpr int BM = 128 * MW;
  const dim3 grid((s.N + kT2Cols - 1) / kT2Cols, (s.M + BM - 1) / BM, s.splits);
  constexpr int lds = 2 * 128 * MW * kStepK * 2 + Prod::kWRing * kT2WSlotBytes + Prod::kStageBytes;
  static LdsLatch latch;
  const hipError_t e = enable_dynamic_lds(latch, reinterpret_cast<const void*>(&tile2_gemm_kernel<ACT, MW, Prod>), lds);
  if (e != hipSuccess)
    return fail(NPAMD_ERR_LAUNCH, "%s: cannot reserve %d bytes of LDS: %s", what, lds, hipGetErrorString(e));
  tile2_gemm_kernel<ACT, MW, Prod><<<grid, 512, lds, st>>>(s, a, pair);
  if (s.splits > 2) {
    const int64_t quads = (int64_t)s.M * ((s.N + 3) / 4);
    splitk_reduce_kernel<ACT><<<(unsigned)((quads + 255) / 256), 256, 0, st>>>(s.partials, s.splits, s.M, s.N,
                                                                             s.bias, s.y, s.ldy);
  }
  return check_launch(what);
}

template <int ACT, class Prod>
int launch_tile2_prod(GemmShape s, const typename Prod::Args& a, hipStream_t st, const char* what, void* workspace,
                      int64_t workspace_bytes, int mw) {
  const int splits = plan_tile2_splits(s.M, s.N, s.chunks, mw);
  if (splits > 1 && (!workspace || tile2_workspace_bytes(s.M, s.N, s.chunks, mw) > workspace_bytes)) return 1;
  s.steps = s.chunks;
  s.split_chunks = (s.chunks + splits - 1) / splits;
  s.splits = (s.chunks + s.split_chunks - 1) / s.split_chunks;
  // The kernel's loop ends in two steps of their own behind an even number of others.
  if (s.split_chunks < 3 || s.chunks - (s.splits - 1) * s.split_chunks < 3) return 1;
  s.partials = (float*)workspace;
  T2Pair pair{nullptr, nullptr, 0ull};
  if (s.splits == 2) {
    const int64_t tiles = (int64_t)((s.N + kT2Cols - 1) / kT2Cols) * ((s.M + 128 * mw - 1) / (128 * mw));
    pair.words = (unsigned long long*)workspace;
    pair.tiles = (float*)((uint8_t*)workspace + ((tiles * 8 + 255) & ~(int64_t)255));
    pair.call = next_call_number();
  }
  switch (mw) {
    case 1: return launch_tile2_mw<ACT, 1, Prod>(s, a, pair, st, what);
    case 2: return launch_tile2_mw<ACT, 2, Prod>(s, a, pair, st, what);
    default: return launch_tile2_mw<ACT, 3, Prod>(s, a, pair, st, what);
  }
}

int launch_tile2(int act, const GemmShape& s, const T2Args& a, hipStream_t st, const char* what, void* workspace,
                 int64_t workspace_bytes) {
  const int mw = plan_tile_mw(s.M);
  return act == NPAMD_BF16 ? launch_tile2_prod<NPAMD_BF16, T2ProdVq16<NPAMD_BF16>>(s, a, st, what, workspace, workspace_bytes, mw)
                           : launch_tile2_prod<NPAMD_F16, T2ProdVq16<NPAMD_F16>>(s, a, st, what, workspace, workspace_bytes, mw);
}

template <int ACT, int NBITS>
static int launch_tile2_q_bits(bool asym, const GemmShape& s, const T2QArgs& q, hipStream_t st, const char* what,
                               void* workspace, int64_t workspace_bytes) {
  if (asym) {
    using Prod = T2ProdQ<ACT, NBITS, true>;
    const typename Prod::Args a{q.w_pack, q.scale, q.chunks, q.groups_per_row, q.gs_shift_chunks, q.zp};
    return launch_tile2_prod<ACT, Prod>(s, a, st, what, workspace, workspace_bytes, plan_tile2_q_mw(s.M));
  }
  using Prod = T2ProdQ<ACT, NBITS, false>;
  const typename Prod::Args a{q.w_pack, q.scale, q.chunks, q.groups_per_row, q.gs_shift_chunks, q.zp};
  return launch_tile2_prod<ACT, Prod>(s, a, st, what, workspace, workspace_bytes, plan_tile2_q_mw(s.M));
}

int launch_tile2_q(int act, int nbits, const GemmShape& s, const T2QArgs& q, hipStream_t st, const char* what,
                   void* workspace, int64_t workspace_bytes) {
  const bool asym = q.zp != nullptr;
  if (act == NPAMD_BF16)
    return nbits == 4 ? launch_tile2_q_bits<NPAMD_BF16, 4>(asym, s, q, st, what, workspace, workspace_bytes)
                      : launch_tile2_q_bits<NPAMD_BF16, 8>(asym, s, q, st, what, workspace, workspace_bytes);
  return nbits == 4 ? launch_tile2_q_bits<NPAMD_F16, 4>(asym, s, q, st, what, workspace, workspace_bytes)
                    : launch_tile2_q_bits<NPAMD_F16, 8>(asym, s, q, st, what, workspace, workspace_bytes);
}

}  // namespace npamd
