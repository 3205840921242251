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

// Sixteen 16-byte loads / four 16-byte stores of agent scope (sc1: coherent between the L2 caches of
// the GPU's dies without a cache invalidate or write-back), issued together and waited for once.
// The compiler waits for every atomic load on its own; a tile handed over in 192 round trips
// costs 45 us.  `p`: the lane's address; consecutive vectors are 1 KiB apart.
__device__ __forceinline__ void load16_sc1(const float* p, f32x4 (&v)[16]) {
  asm volatile(
      "global_load_dwordx4 %0, %16, off sc1\n\tglobal_load_dwordx4 %1, %16, off offset:1024 sc1\n\t"
      "global_load_dwordx4 %2, %16, off offset:2048 sc1\n\tglobal_load_dwordx4 %3, %16, off offset:3072 sc1\n\t"
      "global_load_dwordx4 %4, %17, off sc1\n\tglobal_load_dwordx4 %5, %17, off offset:1024 sc1\n\t"
      "global_load_dwordx4 %6, %17, off offset:2048 sc1\n\tglobal_load_dwordx4 %7, %17, off offset:3072 sc1\n\t"
      "global_load_dwordx4 %8, %18, off sc1\n\tglobal_load_dwordx4 %9, %18, off offset:1024 sc1\n\t"
      "global_load_dwordx4 %10, %18, off offset:2048 sc1\n\tglobal_load_dwordx4 %11, %18, off offset:3072 sc1\n\t"
      "global_load_dwordx4 %12, %19, off sc1\n\tglobal_load_dwordx4 %13, %19, off offset:1024 sc1\n\t"
      "global_load_dwordx4 %14, %19, off offset:2048 sc1\n\tglobal_load_dwordx4 %15, %19, off offset:3072 sc1\n\t"
      "s_waitcnt vmcnt(0)"
      : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]), "=&v"(v[3]), "=&v"(v[4]), "=&v"(v[5]), "=&v"(v[6]), "=&v"(v[7]),
        "=&v"(v[8]), "=&v"(v[9]), "=&v"(v[10]), "=&v"(v[11]), "=&v"(v[12]), "=&v"(v[13]), "=&v"(v[14]), "=&v"(v[15])
      : "v"(p), "v"(p + 1024), "v"(p + 2048), "v"(p + 3072)
      : "memory");
}
__device__ __forceinline__ void store4_sc1(float* p, const f32x4& v0, const f32x4& v1, const f32x4& v2, const f32x4& v3) {
  asm volatile(
      "global_store_dwordx4 %0, %1, off sc1\n\tglobal_store_dwordx4 %0, %2, off offset:1024 sc1\n\t"
      "global_store_dwordx4 %0, %3, off offset:2048 sc1\n\tglobal_store_dwordx4 %0, %4, off offset:3072 sc1"
      ::"v"(p), "v"(v0), "v"(v1), "v"(v2), "v"(v3)
      : "memory");
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

// What a producer needs to know about its wave: it decodes columns [32 wave, 32 wave + 32) of the
// block's W tile, lane (c = lane % 32, h = lane / 32) the operands 4h .. 4h + 3 (k = 32 h .. 32 h + 31
// of the step) of column c, and operand j of a step goes to byte (wave * 4 + j) * 1024 + 16 * lane
// of the step's W slot.
struct WaveCtx {
  int wave, lane, c, h;
  int ncol;            // the lane's weight row, clamped to N - 1
  int n_first, n_last; // the wave's first weight row (may lie past N - 1), and N - 1
  uint8_t* ws;         // W slots, kWRing x 16 KiB
  uint32_t ws_lds;     // the same as an LDS address
  uint8_t* stage;      // the block's staging area
  uint32_t stage_lds;
};

// ---------------------------------------------------------------------------------------------
// Producer: VQ, 16-bit indices, vector length 8, codebook in the activation dtype, looked up in
// memory.  A weight operand is one codebook row: the gather writes the W slot directly.  In step t
// the wave gathers for step t + 2 (W ring of three) from the indices it staged in step t - 2.
// ---------------------------------------------------------------------------------------------
template <int ACT>
struct T2ProdVq16 {
  using Args = T2Args;
  static constexpr int kWRing = 3;
  static constexpr int kLoads = 4;                 // per step: four gathers ...
  static constexpr int kQuadLoads = 2;             // ... and, every fourth step, two index loads behind them
  static constexpr bool kLoadsLast = true;         // issued behind the step's x pieces, in k group 3
  // Indices are staged four steps at a time: a column's 64 bytes of a quad of steps are half a cache
  // line, and one load instruction fetches them for sixteen columns (16 lines; a load of one
  // step's 16 bytes for 32 columns touches 32 lines, and the address unit's time goes with the
  // lines).  Per wave two quads of 32 columns x 64 bytes; piece p of column r sits in slot
  // p ^ ((r >> 2) & 3) of its row, which spreads the 8-byte reads of 32 columns over the banks.
  static constexpr int kQuadBytes = 32 * 64;
  static constexpr int kStageBytes = 4 * 2 * kQuadBytes;
  const Args& a;
  const KWalk& kw;
  const WaveCtx& w;
  uint32_t row_off[2];  // byte offset of the index rows this lane fetches (columns lane / 4 and 16 + lane / 4 of the wave)
  int piece;            // which of a quad's four steps the lane fetches for those columns
  __device__ T2ProdVq16(const Args& args, const KWalk& walk, const WaveCtx& ctx) : a(args), kw(walk), w(ctx) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int r = 16 * i + (ctx.lane >> 2);
      const int n = min(ctx.n_first + r, ctx.n_last);  // columns past N fetch a valid row nobody stores
      row_off[i] = (uint32_t)n * (uint32_t)args.chunks * 16u;
    }
    piece = (ctx.lane & 3) ^ ((ctx.lane >> 4) & 3);  // slot ^ ((r >> 2) & 3), r = 16 i + lane / 4
  }
  // Steps 4 quad .. 4 quad + 3 of the wave's 32 columns into staging slot quad % 2.
  __device__ __forceinline__ void load_quad(int quad) const {
    const uint32_t chunk = (uint32_t)kw.chunk_of(4 * quad + piece) * 16u;
    const uint32_t dst = w.stage_lds + (uint32_t)((w.wave * 2 + (quad & 1)) * kQuadBytes);
    lds_load16(dst, row_off[0] + chunk, a.packed);
    lds_load16(dst + 1024u, row_off[1] + chunk, a.packed);
  }
  // The lookups of step `step` into W slot `slot`, from the staged indices.
  __device__ __forceinline__ void gathers(int step, int slot) const {
    const int q = step >> 2, p = step & 3;
    const u32x2 v = *reinterpret_cast<const u32x2*>(w.stage + (w.wave * 2 + (q & 1)) * kQuadBytes + w.c * 64 +
                                                    ((p ^ ((w.c >> 2) & 3)) << 4) + w.h * 8);
    const uint32_t off[4] = {(uint32_t)(min(v.x & 0xFFFFu, a.nc_minus_1) << 4), (uint32_t)(min(v.x >> 16, a.nc_minus_1) << 4),
                             (uint32_t)(min(v.y & 0xFFFFu, a.nc_minus_1) << 4), (uint32_t)(min(v.y >> 16, a.nc_minus_1) << 4)};
#pragma unroll
    for (int j = 0; j < 4; ++j)
      lds_load16(w.ws_lds + (uint32_t)(slot * kT2WSlotBytes + (w.wave * 4 + j) * 1024), off[j], a.cb);
  }
  // Before the loop: the indices of steps 0 .. 7 staged, the W tiles of steps 0 and 1 requested.
  __device__ __forceinline__ void prologue_issue() const {
    load_quad(0);
    load_quad(1);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    gathers(0, 0);
    gathers(1, 1);
  }
  __device__ __forceinline__ void prologue_finish() const {}
  // In step t the wave looks up the rows of step t + 2 (W ring of three); after the lookups of
  // t = 4 q + 2, which read quad q + 1, quad q's slot is free (its last reader was step 4 q + 1) and
  // takes quad q + 2, first read in step 4 q + 6.
  __device__ __forceinline__ bool loads_quad(int step) const { return (step & 3) == 2; }
  // Work behind the MFMAs of k group J, column tile T of step `step` (W slot wslot = step % 3).
  template <int J, int T>
  __device__ __forceinline__ void work(int step, int wslot) const {
    if (J == 0 && T == 0) gathers(step + 2, wslot == 0 ? 2 : wslot - 1);
    if (J == 0 && T == 1 && loads_quad(step)) load_quad((step >> 2) + 2);
  }
  __device__ __forceinline__ void work_all(int step, int wslot) const {
    work<0, 0>(step, wslot);
    work<0, 1>(step, wslot);
  }
  // Wait until everything but the loads this step issued last (its lookups, and the index quads
  // behind them in the steps that fetch one) has landed.
  __device__ __forceinline__ void wait_all_but_own(int step) const {
    if (loads_quad(step)) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kLoads + kQuadLoads) : "memory");
    else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kLoads) : "memory");
  }
};

// ---------------------------------------------------------------------------------------------
// Producers: int4 / int8 group-affine codes.  Packed bytes and scales go to an LDS staging ring
// (directly, like everything else the kernel loads, so that one in-order counter tracks all of a
// wave's loads); in step t the wave requests the bytes of step t + 3, and turns the bytes of step
// t + 1, which arrived during step t - 1, into four operands that it writes to the other W slot
// (ring of two): 16 (int4, f16) to 40 VALU instructions per operand, issued between the MFMAs.
// The arithmetic is the providers' (providers.hpp): bit for bit the one-pass decode.
// ---------------------------------------------------------------------------------------------
template <int ACT, int NBITS, bool ASYM>
struct T2ProdQ {
  using P = typename std::conditional<NBITS == 4, Q4Provider<ACT, ASYM>, Q8Provider<ACT, ASYM>>::type;
  using Args = typename P::Args;
  static constexpr int kWRing = 2;
  static constexpr int kCodeLoads = NBITS == 4 ? 1 : 2;         // 16 bytes of nibbles, 32 of bytes per lane and step
  static constexpr int kLoads = kCodeLoads + 1 + (ASYM ? 1 : 0);  // + the dword that holds the scale (+ zero point)
  static constexpr bool kLoadsLast = false;        // requested in k group 0, in front of the step's x pieces
  static constexpr int kSlot = kCodeLoads * 1024 + 256 + (ASYM ? 256 : 0);
  static constexpr int kStageWave = 3 * kSlot;
  static constexpr int kStageBytes = 4 * kStageWave;
  const Args& a;
  const KWalk& kw;
  const WaveCtx& w;
  const P prov;
  uint32_t code_off;   // byte offset of the lane's share of chunk 0 of its row
  uint32_t scale_row;  // index of the row's first scale
  int req_slot = 0;    // staging slot of the next request (the bytes of step s live in slot s % 3)
  int fetch_slot = 0;  // staging slot of the next step to decode
  u32x4 raw0, raw1;    // the step being decoded
  uint32_t s2, z;
  __device__ T2ProdQ(const Args& args, const KWalk& walk, const WaveCtx& ctx)
      : a(args), kw(walk), w(ctx), prov(args),
        code_off((uint32_t)ctx.ncol * (uint32_t)args.chunks * (NBITS == 4 ? 32u : 64u) + (uint32_t)ctx.h * (NBITS == 4 ? 16u : 32u)),
        scale_row((uint32_t)ctx.ncol * (uint32_t)args.groups_per_row) {}
  __device__ __forceinline__ uint32_t scale_index(int step) const {
    return scale_row + (uint32_t)((2 * kw.chunk_of(step) + w.h) >> a.gs_shift_chunks);
  }
  __device__ __forceinline__ void request(int step) {
    const uint32_t dst = w.stage_lds + (uint32_t)(w.wave * kStageWave + req_slot * kSlot);
    const uint32_t off = code_off + (uint32_t)kw.chunk_of(step) * (NBITS == 4 ? 32u : 64u);
    lds_load16(dst, off, a.w_pack);
    if (NBITS == 8) lds_load16(dst + 1024, off + 16u, a.w_pack);
    const uint32_t sb = (scale_index(step) * 2u) & ~3u;
    lds_load4(dst + kCodeLoads * 1024, sb, a.scale);
    if (ASYM) lds_load4(dst + kCodeLoads * 1024 + 256, sb, a.zp);
    req_slot = req_slot == 2 ? 0 : req_slot + 1;
  }
  // Reads the staged bytes of `step`; steps are requested and fetched in order.
  __device__ __forceinline__ void fetch(int step) {
    const uint8_t* src = w.stage + w.wave * kStageWave + fetch_slot * kSlot;
    fetch_slot = fetch_slot == 2 ? 0 : fetch_slot + 1;
    raw0 = *reinterpret_cast<const u32x4*>(src + w.lane * 16);
    if (NBITS == 8) raw1 = *reinterpret_cast<const u32x4*>(src + 1024 + w.lane * 16);
    const uint32_t sh = (scale_index(step) & 1u) * 16u;
    const uint32_t sd = *reinterpret_cast<const uint32_t*>(src + kCodeLoads * 1024 + w.lane * 4);
    s2 = ((sd >> sh) & 0xFFFFu) * 0x10001u;
    z = 0;
    if (ASYM) z = (*reinterpret_cast<const uint32_t*>(src + kCodeLoads * 1024 + 256 + w.lane * 4) >> sh) & 0xFFFFu;
  }
  template <int O>
  __device__ __forceinline__ void decode(int wslot) const {
    u32x4 op;
    if constexpr (NBITS == 4) {
      op = prov.dequant8(O == 0 ? raw0.x : O == 1 ? raw0.y : O == 2 ? raw0.z : raw0.w, s2, z);
    } else {
      const u32x4& r = O < 2 ? raw0 : raw1;
      op = prov.dequant8((O & 1) ? r.z : r.x, (O & 1) ? r.w : r.y, s2, z);
    }
    *reinterpret_cast<u32x4*>(w.ws + wslot * kT2WSlotBytes + (w.wave * 4 + O) * 1024 + w.lane * 16) = op;
  }
  __device__ __forceinline__ void prologue_issue() {
    request(0);
    request(1);
    request(2);
  }
  // Everything requested has arrived: the W tile of step 0.
  __device__ __forceinline__ void prologue_finish() {
    fetch(0);
    decode<0>(0);
    decode<1>(0);
    decode<2>(0);
    decode<3>(0);
    fetch(1);
  }
  template <int J, int T>
  __device__ __forceinline__ void work(int step, int wslot) {
    if (J == 0 && T == 0) request(step + 3);
    if (J == 0 && T == 2) decode<0>(wslot ^ 1);
    if (J == 0 && T == 3) decode<1>(wslot ^ 1);
    if (J == 1 && T == 0) decode<2>(wslot ^ 1);
    if (J == 1 && T == 1) decode<3>(wslot ^ 1);
    // The bytes the next step decodes are read out of the staging ring a k group and a barrier ahead
    // of their first use, so that the decoding never waits for LDS.
    if (J == 3 && T == 3) fetch(step + 2);
  }
  __device__ __forceinline__ void work_all(int step, int wslot) {
    request(step + 3);
    decode<0>(wslot ^ 1);
    decode<1>(wslot ^ 1);
    decode<2>(wslot ^ 1);
    decode<3>(wslot ^ 1);
    fetch(step + 2);
  }
};

template <int MW, class Prod>
struct T2Lds {
  static constexpr int kXBufBytes = 128 * MW * kStepK * 2;
  static constexpr int kBytes = 2 * kXBufBytes + Prod::kWRing * kT2WSlotBytes + Prod::kStageBytes;
  static_assert(kBytes <= kLdsPerBlockMax, "the block's tiles do not fit LDS");
};

// ABL (builds with -DNPAMD_TILE2_ABLATIONS only; 0 in the library): parts of the step compiled out, to time the
// others -- 1 no weight tile (the producer's work), 2 no x loads, 4 no MFMAs, 8 no operand reads, 32 element-wise epilogue.
#ifdef NPAMD_TILE2_ABLATIONS
__device__ unsigned long long* g_t2_debug = nullptr;
#endif
template <int ACT, int MW, class Prod, int ABL = 0>
__global__ void __launch_bounds__(256)
tile2_gemm_kernel(const GemmShape s, const typename Prod::Args pargs, const T2Pair pair) {
#ifdef NPAMD_TILE2_ABLATIONS
  const unsigned long long t_start = __builtin_amdgcn_s_memrealtime();
#endif
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  constexpr int BM = 128 * MW;
  constexpr int kXBufBytes = T2Lds<MW, Prod>::kXBufBytes;
  constexpr int kPieces = 4 * MW;  // x-tile load instructions per wave and step (8 rows each)
  constexpr int kWRing = Prod::kWRing;
  uint8_t* const xs = lds;                              // [2][BM][128]
  uint8_t* const ws = lds + 2 * kXBufBytes;             // [kWRing][16 KiB]
  uint8_t* const stage = ws + kWRing * kT2WSlotBytes;   // the producer's staging area

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = lane & 31;
  const int h = lane >> 5;
  const int m0 = blockIdx.y * BM;
  const int n0 = blockIdx.x * kT2Cols;
  KWalk kw;
  kw.chunk0 = blockIdx.z * s.split_chunks;
  kw.steps = min(s.split_chunks, s.chunks - kw.chunk0);
  kw.rot = (int)((blockIdx.x * 7u) % (unsigned)kw.steps);
  const int steps = kw.steps;

  const uint32_t xs_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)xs;
  WaveCtx wc;
  wc.wave = wave;
  wc.lane = lane;
  wc.c = c;
  wc.h = h;
  wc.ncol = min(n0 + 32 * wave + c, s.N - 1);  // columns past N decode a valid row nobody stores
  wc.n_first = n0 + 32 * wave;
  wc.n_last = s.N - 1;
  wc.ws = ws;
  wc.ws_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)ws;
  wc.stage = stage;
  wc.stage_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)stage;
  Prod prod(pargs, kw, wc);

  // ---- x tile ----------------------------------------------------------------------------------
  const int wrow0 = wave * (32 * MW);
  const bool wave_active = (m0 + wrow0) < s.M;
  const int base_row = min(m0 + wrow0, s.M - 1);
  const uint8_t* const xbase = reinterpret_cast<const uint8_t*>(s.x) + (int64_t)base_row * s.ldx * 2;
  uint32_t voff[kPieces];
#pragma unroll
  for (int i = 0; i < kPieces; ++i) {
    const int r = 8 * i + (lane >> 3);
    const int piece = (lane & 7) ^ ((r >> 1) & 7);
    voff[i] = (uint32_t)(((int64_t)min(r, s.M - 1 - base_row) * s.ldx + piece * 8) * 2);
  }
  const uint32_t wave_x_lds = xs_lds + (uint32_t)(wrow0 * 128);
  auto fetch_piece = [&](int i, int buf, const uint8_t* src) {
    if (ABL & 2) return;
    lds_load16(wave_x_lds + (uint32_t)(buf * kXBufBytes + i * 1024), voff[i], src);
  };
  auto tile_src = [&](int step) { return xbase + (int64_t)kw.chunk_of(step) * (kStepK * 2); };

  // ---- prologue ----------------------------------------------------------------------------------
  if (!(ABL & 1)) prod.prologue_issue();
  if (wave_active) {
    const uint8_t* src = tile_src(0);
#pragma unroll
    for (int i = 0; i < kPieces; ++i) fetch_piece(i, 0, src);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  if (!(ABL & 1)) prod.prologue_finish();
  block_sync_lds();

  f32x16 acc[MW][4];
#pragma unroll
  for (int mt = 0; mt < MW; ++mt)
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mt][t][i] = 0.f;

  if (wave_active) {
    u32x4 ao[2][MW] = {}, bo[2][4] = {};
    const uint32_t row_off = (uint32_t)((wrow0 + c) * 128);
    uint32_t slot_off[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) slot_off[j] = (uint32_t)((((h << 2) | j) ^ ((c >> 1) & 7)) << 4);
    auto read_ops = [&](int set, int buf, int wslot, int j) {
      if (ABL & 8) return;
      const uint8_t* wb = ws + wslot * kT2WSlotBytes + j * 1024 + lane * 16;
#pragma unroll
      for (int t = 0; t < 4; ++t) bo[set][t] = *reinterpret_cast<const u32x4*>(wb + t * 4096);
      const uint8_t* xa = xs + buf * kXBufBytes + row_off + slot_off[j];
#pragma unroll
      for (int mt = 0; mt < MW; ++mt) ao[set][mt] = *reinterpret_cast<const u32x4*>(xa + mt * 32 * 128);
    };
    // One step; buf = step % 2 is a compile-time constant through the unrolled loops below.
    // The step's loads are issued behind MFMAs, one at a time, so that the address unit is fed all
    // through the step instead of in two bursts: the x tile of step + 1 piece by piece in k groups
    // 0 to 2 (it goes into the other buffer, which this wave read for the last time a step ago),
    // a producer's lookups behind them in k group 3 (they fill the W slot of step + 2 and may stay
    // in flight over the barrier), a producer's streamed bytes in k groups 0 and 1.
    auto one_step = [&](int buf, int step, int wslot) {
      read_ops(0, buf, wslot, 0);
      const uint8_t* src = tile_src(step + 1);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (j < 3) read_ops((j + 1) & 1, buf, wslot, j + 1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
#pragma unroll
          for (int mt = 0; mt < MW; ++mt)
            if (!(ABL & 4)) acc[mt][t] = mfma32<ACT>(ao[j & 1][mt], bo[j & 1][t], acc[mt][t]);
          if (!(ABL & 1)) {
            if constexpr (Prod::kLoadsLast) {
              if (j == 3 && t == 0) prod.template work<0, 0>(step, wslot);
              if (j == 3 && t == 1) prod.template work<0, 1>(step, wslot);
            } else {
              if (j == 0 && t == 0) prod.template work<0, 0>(step, wslot);
              if (j == 0 && t == 1) prod.template work<0, 1>(step, wslot);
              if (j == 0 && t == 2) prod.template work<0, 2>(step, wslot);
              if (j == 0 && t == 3) prod.template work<0, 3>(step, wslot);
              if (j == 1 && t == 0) prod.template work<1, 0>(step, wslot);
              if (j == 1 && t == 1) prod.template work<1, 1>(step, wslot);
              if (j == 3 && t == 3) prod.template work<3, 3>(step, wslot);
            }
          }
          if (j * 4 + t < kPieces) fetch_piece(j * 4 + t, buf ^ 1, src);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      // Everything but a producer's lookups of this step has to be there when the next step starts.
      if constexpr (Prod::kLoadsLast && !(ABL & 1)) prod.wait_all_but_own(step);
      else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      block_sync_lds();
    };
    int wslot = 0;
    const int whole = steps / 2 * 2;
    for (int t0 = 0; t0 < whole; t0 += 2) {
#pragma unroll
      for (int d = 0; d < 2; ++d) {
        one_step(d, t0 + d, wslot);
        wslot = wslot == kWRing - 1 ? 0 : wslot + 1;
      }
    }
    if (whole < steps) one_step(0, whole, wslot);
  } else {
    // No rows of this wave lie inside M: it still decodes its 32 columns for the others.
    int wslot = 0;
    for (int t = 0; t < steps; ++t) {
      if (!(ABL & 1)) prod.work_all(t, wslot);
      if constexpr (Prod::kLoadsLast && !(ABL & 1)) prod.wait_all_but_own(t);
      else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // as the waves with rows do
      block_sync_lds();
      wslot = wslot == kWRing - 1 ? 0 : wslot + 1;
    }
  }
  // Nothing may still be on its way into LDS when the wave ends.
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

#ifdef NPAMD_TILE2_ABLATIONS
  if (g_t2_debug && (threadIdx.x & 63) == 0) {
    unsigned long long* d = g_t2_debug + ((size_t)(blockIdx.z * gridDim.x + blockIdx.x) * 4 + (threadIdx.x >> 6)) * 4;
    d[0] = t_start;
    d[1] = __builtin_amdgcn_s_memrealtime();
    d[2] = 0;
    d[3] = 0;
  }
#endif
  // ---- epilogue: D[m = 8 (i / 4) + 4 h + i % 4][n = c] of each 32 x 32 tile ---------------------
  bool finish = true;
  if (s.splits == 2) {
    // Whichever workgroup of the pair arrives first stores its f32 tile and counts itself in; the
    // other adds that tile to its registers.  Stores and loads of the tile and the counter are of
    // agent scope (sc1): they bypass the caches that are not shared by the whole GPU (every die has
    // an L2 of its own), so no cache is written back or invalidated to hand the tile over (an
    // agent-scope fence does both for a whole L2, under the workgroups still running their loops).
    // Measured and dropped: ordinary stores and loads when both halves run on the same die (each
    // said so at its start): the tiles then sit dirty in that die's L2, 2.7 of its 4 MiB at 384
    // tokens, and the last workgroups finish 6 us later than with the trip through memory.
    const int tile_id = blockIdx.y * gridDim.x + blockIdx.x;
    const int tiles = gridDim.x * gridDim.y;
    constexpr int kTileFloats = BM * kT2Cols;
    // [tile][wave][row tile mt][column tile t][quarter q][lane] float4: 1 KiB per instruction
    float* const mine = pair.tiles + ((size_t)blockIdx.z * tiles + tile_id) * kTileFloats + wave * (MW * 64 * 64) + lane * 4;
    const float* const theirs =
        pair.tiles + ((size_t)(blockIdx.z ^ 1) * tiles + tile_id) * kTileFloats + wave * (MW * 64 * 64) + lane * 4;
    unsigned long long* const flag = reinterpret_cast<unsigned long long*>(ws);  // outside the waves' output areas
    unsigned long long* const word = pair.words + tile_id;
    __syncthreads();  // every wave is past its last LDS read
    if (tid == 0) flag[0] = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    bool arrived = flag[0] == pair.call;  // the other half is there already: nothing to write
    if (!arrived) {
      if (wave_active) {
#pragma unroll
        for (int mt = 0; mt < MW; ++mt)
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            const f32x16& r = acc[mt][t];
            store4_sc1(mine + (mt * 4 + t) * 1024, f32x4{r[0], r[1], r[2], r[3]}, f32x4{r[4], r[5], r[6], r[7]},
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
#pragma unroll
          for (int mt = 0; mt < MW; ++mt) {
            f32x4 v[16];
            load16_sc1(theirs + mt * 4096, v);
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
              for (int i = 0; i < 16; ++i) acc[mt][t][i] += v[t * 4 + i / 4][i % 4];
          }
      }
    }
  }
#ifdef NPAMD_TILE2_ABLATIONS
  if (g_t2_debug && (threadIdx.x & 63) == 0)
    g_t2_debug[((size_t)(blockIdx.z * gridDim.x + blockIdx.x) * 4 + (threadIdx.x >> 6)) * 4 + 2] = __builtin_amdgcn_s_memrealtime();
#endif
  if (s.splits <= 2 && !(ABL & 32)) {
    // y through LDS (see store_wave_tile): every wave takes 32 MW x 256 bytes of the x buffers.
    if (s.splits != 2) __syncthreads();  // every wave is past its last LDS read (the pair path has met already)
    if (finish && wave_active)
      store_wave_tile<ACT, MW, 4>(acc, lds + wave * (32 * MW * 256), lane, s.y, s.ldy, m0 + wrow0, n0, s.M, s.N, s.bias);
#ifdef NPAMD_TILE2_ABLATIONS
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (g_t2_debug && (threadIdx.x & 63) == 0)
      g_t2_debug[((size_t)(blockIdx.z * gridDim.x + blockIdx.x) * 4 + (threadIdx.x >> 6)) * 4 + 3] = __builtin_amdgcn_s_memrealtime();
#endif
    return;
  }
  if (!wave_active || !finish) return;
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const int n = n0 + t * 32 + c;
    if (n >= s.N) continue;
    const float bv = s.bias ? s.bias[n] : 0.f;
    float* part = s.partials + (size_t)blockIdx.z * s.M * s.N;
#pragma unroll
    for (int mt = 0; mt < MW; ++mt) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int m = m0 + wrow0 + mt * 32 + 8 * (i / 4) + 4 * h + (i % 4);
        if (m >= s.M) continue;
        if (s.splits > 2) part[(size_t)m * s.N + n] = acc[mt][t][i];
        else store_from_f32<ACT>(s.y, (int64_t)m * s.ldy + n, acc[mt][t][i] + bv);
      }
    }
  }
}

template <int ACT, int MW, class Prod, int ABL = 0>
int launch_tile2_mw(const GemmShape& s, const typename Prod::Args& a, const T2Pair& pair, hipStream_t st, const char* what) {
  constexpr int BM = 128 * MW;
  const dim3 grid((s.N + kT2Cols - 1) / kT2Cols, (s.M + BM - 1) / BM, s.splits);
  constexpr int lds = T2Lds<MW, Prod>::kBytes;
  static LdsLatch latch;
  const hipError_t e = enable_dynamic_lds(latch, reinterpret_cast<const void*>(&tile2_gemm_kernel<ACT, MW, Prod, ABL>), lds);
  if (e != hipSuccess)
    return fail(NPAMD_ERR_LAUNCH, "%s: cannot reserve %d bytes of LDS: %s", what, lds, hipGetErrorString(e));
  tile2_gemm_kernel<ACT, MW, Prod, ABL><<<grid, 256, lds, st>>>(s, a, pair);
  if (s.splits > 2) {
    const int64_t quads = (int64_t)s.M * ((s.N + 3) / 4);
    splitk_reduce_kernel<ACT><<<(unsigned)((quads + 255) / 256), 256, 0, st>>>(s.partials, s.splits, s.M, s.N,
                                                                             s.bias, s.y, s.ldy);
  }
  return check_launch(what);
}

// Plans the split, carves the workspace and picks the row-tile count; returns 1 when the
// workspace does not allow the planned split (the caller then takes the 64-column kernel).
template <int ACT, class Prod>
int launch_tile2_prod(GemmShape s, const typename Prod::Args& a, hipStream_t st, const char* what, void* workspace,
                      int64_t workspace_bytes, int mw) {
  const int splits = plan_tile2_splits(s.M, s.N, s.chunks, mw);
  if (splits > 1 && (!workspace || tile2_workspace_bytes(s.M, s.N, s.chunks, mw) > workspace_bytes)) return 1;
  s.steps = s.chunks;
  s.split_chunks = (s.chunks + splits - 1) / splits;
  s.splits = (s.chunks + s.split_chunks - 1) / s.split_chunks;
  s.partials = (float*)workspace;
  T2Pair pair{nullptr, nullptr, 0ull};
  if (s.splits == 2) {
    const int64_t tiles = (int64_t)((s.N + kT2Cols - 1) / kT2Cols) * ((s.M + 128 * mw - 1) / (128 * mw));
    pair.words = (unsigned long long*)workspace;
    pair.tiles = (float*)((uint8_t*)workspace + ((tiles * 8 + 255) & ~(int64_t)255));
    pair.call = next_call_number();
  }
#ifdef NPAMD_TILE2_ABLATIONS
  if (const char* e = getenv("NPAMD_T2_DEBUG_PTR")) {
    unsigned long long* p = (unsigned long long*)strtoull(e, nullptr, 10);
    (void)hipMemcpyToSymbol(HIP_SYMBOL(g_t2_debug), &p, sizeof(p));
  }
  if constexpr (ACT == NPAMD_BF16 || std::is_same<Prod, T2ProdQ<NPAMD_F16, 4, false>>::value) {
    const char* e = getenv("NPAMD_T2_ABL");
    const int abl = e ? atoi(e) : 0;
    if (abl && mw == 3) {
      switch (abl) {
        case 1: return launch_tile2_mw<ACT, 3, Prod, 1>(s, a, pair, st, what);
        case 2: return launch_tile2_mw<ACT, 3, Prod, 2>(s, a, pair, st, what);
        case 4: return launch_tile2_mw<ACT, 3, Prod, 4>(s, a, pair, st, what);
        case 3: return launch_tile2_mw<ACT, 3, Prod, 3>(s, a, pair, st, what);
        case 6: return launch_tile2_mw<ACT, 3, Prod, 6>(s, a, pair, st, what);
        case 11: return launch_tile2_mw<ACT, 3, Prod, 11>(s, a, pair, st, what);
        case 15: return launch_tile2_mw<ACT, 3, Prod, 15>(s, a, pair, st, what);
      }
    }
    if (abl && mw == 2) {
      switch (abl) {
        case 1: return launch_tile2_mw<ACT, 2, Prod, 1>(s, a, pair, st, what);
        case 2: return launch_tile2_mw<ACT, 2, Prod, 2>(s, a, pair, st, what);
        case 4: return launch_tile2_mw<ACT, 2, Prod, 4>(s, a, pair, st, what);
        case 3: return launch_tile2_mw<ACT, 2, Prod, 3>(s, a, pair, st, what);
        case 6: return launch_tile2_mw<ACT, 2, Prod, 6>(s, a, pair, st, what);
        case 11: return launch_tile2_mw<ACT, 2, Prod, 11>(s, a, pair, st, what);
        case 15: return launch_tile2_mw<ACT, 2, Prod, 15>(s, a, pair, st, what);
      }
    }
  }
#endif
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
