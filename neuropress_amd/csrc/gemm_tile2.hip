// The 128-column tile-decode GEMM (see gemm_tile2.hpp): kernel and launcher.
#include "gemm_tile2.hpp"
#include <stdlib.h>

namespace npamd {

__global__ void __launch_bounds__(256) tile2_zero_counters_kernel(uint32_t* counters, int n) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) counters[i] = 0u;
}

// ABL (builds with -DNPAMD_TILE2_ABLATIONS only; 0 in the library): parts of the step compiled out, to time the
// others -- 1 no gathers, 2 no x loads, 4 no MFMAs, 8 no operand reads, 16 no index loads, 32 element-wise epilogue.
// Sixteen 16-byte loads / stores of agent scope (sc1: coherent between the L2 caches of the GPU's
// dies without a cache invalidate or write-back), issued together and waited for once.  The
// compiler waits for every atomic load on its own; a tile handed over in 192 round trips costs
// 45 us.  `p`: the lane's address; consecutive vectors are 1 KiB apart.
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

#ifdef NPAMD_TILE2_ABLATIONS
__device__ unsigned long long* g_t2_debug = nullptr;
#endif
template <int ACT, int MW, int ABL = 0>
__global__ void __launch_bounds__(256)
tile2_gemm_kernel(const GemmShape s, const T2Args a) {
#ifdef NPAMD_TILE2_ABLATIONS
  const unsigned long long t_start = __builtin_amdgcn_s_memrealtime();
#endif
  constexpr int kNG = (ABL & 1) ? 0 : 4, kNI = (ABL & 16) ? 0 : 1;
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  constexpr int BM = 128 * MW;
  constexpr int kXBufBytes = T2Lds<MW>::kXBufBytes;
  constexpr int kPieces = 4 * MW;  // x-tile load instructions per wave and step (8 rows each)
  uint8_t* const xs = lds;                                   // [2][BM][128]
  uint8_t* const ws = lds + 2 * kXBufBytes;                  // [3][16 KiB]
  uint8_t* const is = ws + kT2WRing * kT2WSlotBytes;         // [4 waves][2][1 KiB]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = lane & 31;
  const int h = lane >> 5;
  const int m0 = blockIdx.y * BM;
  const int n0 = blockIdx.x * kT2Cols;
  const int chunk0 = blockIdx.z * s.split_chunks;
  const int steps = min(s.split_chunks, s.chunks - chunk0);
  const int rot = (int)((blockIdx.x * 7u) % (unsigned)steps);
  auto chunk_of = [&](int step) {
    const int kc = min(step, steps - 1) + rot;
    return chunk0 + (kc >= steps ? kc - steps : kc);
  };

  const uint32_t xs_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)xs;
  const uint32_t ws_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)ws;
  const uint32_t is_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)is;

  // ---- W tile: indices and gathers -----------------------------------------------------------
  const int ncol = min(n0 + 32 * wave + c, s.N - 1);  // columns past N decode a valid row nobody stores
  const uint32_t idx_row_off = (uint32_t)ncol * (uint32_t)s.chunks * 16u;  // byte offset of the column's first chunk
  auto load_idx = [&](int step, int par) {
    if (ABL & 16) return;
    const uint32_t dst = __builtin_amdgcn_readfirstlane(is_lds + (uint32_t)((wave * 2 + par) * 1024));
    const uint32_t off = idx_row_off + (uint32_t)chunk_of(step) * 16u;
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(off), "s"(a.packed)
                 : "memory");
  };
  auto row_off16 = [&](uint32_t i) { return (uint32_t)(min(i, a.nc_minus_1) << 4); };
  auto gather_rows = [&](const u32x2 v, int slot) {
    if (ABL & 1) return;
    const uint32_t off[4] = {row_off16(v.x & 0xFFFFu), row_off16(v.x >> 16), row_off16(v.y & 0xFFFFu), row_off16(v.y >> 16)};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t dst =
          __builtin_amdgcn_readfirstlane(ws_lds + (uint32_t)(slot * kT2WSlotBytes + (wave * 4 + j) * 1024));
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(off[j]), "s"(a.cb)
                   : "memory");
    }
  };
  auto gathers = [&](int par, int slot) {
    gather_rows(*reinterpret_cast<const u32x2*>(is + (wave * 2 + par) * 1024 + lane * 16 + h * 8), slot);
  };

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
    const uint32_t dst = __builtin_amdgcn_readfirstlane(wave_x_lds + (uint32_t)(buf * kXBufBytes + i * 1024));
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(voff[i]), "s"(src)
                 : "memory");
  };
  auto tile_src = [&](int step) { return xbase + (int64_t)chunk_of(step) * (kStepK * 2); };

  // ---- prologue: indices of steps 0..3, W tiles and x tiles of steps 0 and 1 -------------------
  load_idx(0, 0);
  load_idx(1, 1);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  gathers(0, 0);
  gathers(1, 1);
  load_idx(2, 0);
  load_idx(3, 1);
  if (wave_active) {
#pragma unroll
    for (int p = 0; p < 2; ++p) {
      const uint8_t* src = tile_src(p);
#pragma unroll
      for (int i = 0; i < kPieces; ++i) fetch_piece(i, p, src);
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
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
    // The step's loads are issued behind MFMAs: the gathers of step + 2 and the next indices in k
    // group 0, the x tile of step + 2 in k group 3, whose operands are the last this step reads
    // from the buffer the tile goes into (the wait in front of the first piece makes sure they
    // have arrived, wherever the scheduler puts that piece among the group's MFMAs).
    auto one_step = [&](int buf, int step, int wslot) {
      const int gslot = wslot == 0 ? 2 : wslot - 1;  // (step + 2) % 3
      read_ops(0, buf, wslot, 0);
      const u32x2 iv = *reinterpret_cast<const u32x2*>(is + (wave * 2 + buf) * 1024 + lane * 16 + h * 8);
      const uint8_t* src = tile_src(step + 2);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (j < 3) read_ops((j + 1) & 1, buf, wslot, j + 1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
#pragma unroll
          for (int mt = 0; mt < MW; ++mt)
            if (!(ABL & 4)) acc[mt][t] = mfma32<ACT>(ao[j & 1][mt], bo[j & 1][t], acc[mt][t]);
          if (j == 0 && t == 0) gather_rows(iv, gslot);
          if (j == 0 && t == 1) load_idx(step + 4, buf);
          if (j == 3 && t < 3) {
            if (t == 0) asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
            for (int i = t * kPieces / 3; i < (t + 1) * kPieces / 3; ++i) fetch_piece(i, buf, src);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kNG + kNI + ((ABL & 2) ? 0 : kPieces)) : "memory");
      block_sync_lds();
    };
    int wslot = 0;
    const int whole = steps / 2 * 2;
    for (int t0 = 0; t0 < whole; t0 += 2) {
#pragma unroll
      for (int d = 0; d < 2; ++d) {
        one_step(d, t0 + d, wslot);
        wslot = wslot == kT2WRing - 1 ? 0 : wslot + 1;
      }
    }
    if (whole < steps) one_step(0, whole, wslot);
  } else {
    // No rows of this wave lie inside M: it still decodes its 32 columns for the others.
    int wslot = 0;
    for (int t = 0; t < steps; ++t) {
      const int gslot = wslot == 0 ? 2 : wslot - 1;
      gathers(t & 1, gslot);
      load_idx(t + 4, t & 1);
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kNG + kNI) : "memory");
      block_sync_lds();
      wslot = wslot == kT2WRing - 1 ? 0 : wslot + 1;
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
    // Registers as they are, 256 bytes per store instruction: [tile][wave][register 0 .. 64 MW)[lane] floats.
    // Stores and loads of the tile and the counter are relaxed atomics of agent scope, i.e. they
    // bypass the caches that are not shared by the whole GPU: no cache is written back or
    // invalidated to hand the tile over (an agent-scope fence does both for a whole L2, under
    // the other workgroups still running their loops).
    const int tile_id = blockIdx.y * gridDim.x + blockIdx.x;
    const int tiles = gridDim.x * gridDim.y;
    constexpr int kTileFloats = BM * kT2Cols;
    // [tile][wave][row tile mt][column tile t][quarter q][lane] float4: 1 KiB per instruction
    float* const mine = a.pair_tiles + ((size_t)blockIdx.z * tiles + tile_id) * kTileFloats + wave * (MW * 64 * 64) + lane * 4;
    const float* const theirs =
        a.pair_tiles + ((size_t)(blockIdx.z ^ 1) * tiles + tile_id) * kTileFloats + wave * (MW * 64 * 64) + lane * 4;
    uint32_t* const flag = reinterpret_cast<uint32_t*>(is);  // outside the waves' output areas
    uint32_t* const cnt = a.counters + tile_id;
    __syncthreads();  // every wave is past its last LDS read
    if (tid == 0) flag[0] = __hip_atomic_load(cnt, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    uint32_t arrived = flag[0];
    if (arrived == 0) {
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
      if (tid == 0) flag[1] = __hip_atomic_fetch_add(cnt, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __syncthreads();
      arrived = flag[1];
    }
    finish = arrived != 0;
    if (finish) {
      if (tid == 0) __hip_atomic_store(cnt, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // for the next call
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

template <int ACT, int MW, int ABL = 0>
int launch_tile2_mw(GemmShape s, T2Args a, hipStream_t st, const char* what) {
  constexpr int BM = 128 * MW;
  const dim3 grid((s.N + kT2Cols - 1) / kT2Cols, (s.M + BM - 1) / BM, s.splits);
  constexpr int lds = T2Lds<MW>::kBytes;
  static LdsLatch latch;
  const hipError_t e = enable_dynamic_lds(latch, reinterpret_cast<const void*>(&tile2_gemm_kernel<ACT, MW, ABL>), lds);
  if (e != hipSuccess)
    return fail(NPAMD_ERR_LAUNCH, "%s: cannot reserve %d bytes of LDS: %s", what, lds, hipGetErrorString(e));
  if (s.splits == 2) {
    const int tiles = (int)(grid.x * grid.y);
    tile2_zero_counters_kernel<<<(tiles + 255) / 256, 256, 0, st>>>(a.counters, tiles);
  }
  tile2_gemm_kernel<ACT, MW, ABL><<<grid, 256, lds, st>>>(s, a);
  if (s.splits > 2) {
    const int64_t quads = (int64_t)s.M * ((s.N + 3) / 4);
    splitk_reduce_kernel<ACT><<<(unsigned)((quads + 255) / 256), 256, 0, st>>>(s.partials, s.splits, s.M, s.N,
                                                                             s.bias, s.y, s.ldy);
  }
  return check_launch(what);
}

template <int ACT>
int launch_tile2_act(GemmShape s, T2Args a, hipStream_t st, const char* what, void* workspace, int64_t workspace_bytes) {
  const int mw = plan_tile_mw(s.M);
  int splits = plan_tile2_splits(s.M, s.N, s.chunks, mw);
  if (splits > 1 && (!workspace || tile2_workspace_bytes(s.M, s.N, s.chunks, mw) > workspace_bytes)) return 1;
  s.steps = s.chunks;
  s.split_chunks = (s.chunks + splits - 1) / splits;
  s.splits = (s.chunks + s.split_chunks - 1) / s.split_chunks;
  s.partials = (float*)workspace;
  if (s.splits == 2) {
    const int64_t tiles = (int64_t)((s.N + kT2Cols - 1) / kT2Cols) * ((s.M + 128 * mw - 1) / (128 * mw));
    a.counters = (uint32_t*)workspace;
    a.pair_tiles = (float*)((uint8_t*)workspace + ((tiles * 4 + 255) & ~(int64_t)255));
  }
#ifdef NPAMD_TILE2_ABLATIONS
  if constexpr (ACT == NPAMD_BF16) {
    const char* e = getenv("NPAMD_T2_ABL");
    const int abl = e ? atoi(e) : 0;
    if (abl && mw == 3) {
      switch (abl) {
        case 32: return launch_tile2_mw<ACT, 3, 32>(s, a, st, what);
        case 27: return launch_tile2_mw<ACT, 3, 27>(s, a, st, what);
        case 23: return launch_tile2_mw<ACT, 3, 23>(s, a, st, what);
        case 51: return launch_tile2_mw<ACT, 3, 51>(s, a, st, what);
        case 1: return launch_tile2_mw<ACT, 3, 1>(s, a, st, what);
        case 2: return launch_tile2_mw<ACT, 3, 2>(s, a, st, what);
        case 4: return launch_tile2_mw<ACT, 3, 4>(s, a, st, what);
        case 8: return launch_tile2_mw<ACT, 3, 8>(s, a, st, what);
        case 16: return launch_tile2_mw<ACT, 3, 16>(s, a, st, what);
        case 17: return launch_tile2_mw<ACT, 3, 17>(s, a, st, what);
        case 14: return launch_tile2_mw<ACT, 3, 14>(s, a, st, what);
        case 12: return launch_tile2_mw<ACT, 3, 12>(s, a, st, what);
        case 19: return launch_tile2_mw<ACT, 3, 19>(s, a, st, what);
        case 31: return launch_tile2_mw<ACT, 3, 31>(s, a, st, what);
        case 3: return launch_tile2_mw<ACT, 3, 3>(s, a, st, what);
      }
    }
    if (abl && mw == 1) {
      switch (abl) {
        case 1: return launch_tile2_mw<ACT, 1, 1>(s, a, st, what);
        case 2: return launch_tile2_mw<ACT, 1, 2>(s, a, st, what);
        case 16: return launch_tile2_mw<ACT, 1, 16>(s, a, st, what);
        case 14: return launch_tile2_mw<ACT, 1, 14>(s, a, st, what);
        case 30: return launch_tile2_mw<ACT, 1, 30>(s, a, st, what);
        case 31: return launch_tile2_mw<ACT, 1, 31>(s, a, st, what);
      }
    }
  }
#endif
  switch (mw) {
    case 1: return launch_tile2_mw<ACT, 1>(s, a, st, what);
    case 2: return launch_tile2_mw<ACT, 2>(s, a, st, what);
    default: return launch_tile2_mw<ACT, 3>(s, a, st, what);
  }
}


int launch_tile2(int act, GemmShape s, T2Args a, hipStream_t st, const char* what, void* workspace, int64_t workspace_bytes) {
#ifdef NPAMD_TILE2_ABLATIONS
  if (const char* e = getenv("NPAMD_T2_DEBUG_PTR")) {
    unsigned long long* p = (unsigned long long*)strtoull(e, nullptr, 10);
    (void)hipMemcpyToSymbol(HIP_SYMBOL(g_t2_debug), &p, sizeof(p));
  }
#endif
  return act == NPAMD_BF16 ? launch_tile2_act<NPAMD_BF16>(s, a, st, what, workspace, workspace_bytes)
                           : launch_tile2_act<NPAMD_F16>(s, a, st, what, workspace, workspace_bytes);
}

}  // namespace npamd
