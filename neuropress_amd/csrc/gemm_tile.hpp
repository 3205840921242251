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
// Both operands are staged in LDS, rows padded to 144 bytes so 16-byte reads of
// 32 consecutive rows are bank-conflict free:
//   x tile  [BM][64 k], double buffered, loaded coalesced by the consumers one
//           step ahead through registers;
//   W tile  [64][64 k], double buffered.  Producer q decodes the steps
//           p == q (mod 4), lane = column.  It keeps kDepth decodes in flight
//           in registers (issued 4*kDepth iterations before they are consumed)
//           and writes a finished one to LDS one iteration before its step.
// One block barrier per macro-step, executed by all eight waves.
#pragma once

#include "providers.hpp"

namespace npamd {

constexpr int kStepK = 64;                      // k per macro-step (= one chunk)
constexpr int kRowBytes = kStepK * 2 + 16;      // padded LDS row stride
constexpr int kTileCols = 64;                   // output columns per block
constexpr int kWBufBytes = kTileCols * kRowBytes;

struct GemmShape {
  const void* x;
  int64_t ldx;
  const float* bias;
  void* y;
  int64_t ldy;
  int M, N, K;
  int chunks;  // K / 64 = number of macro-steps
  int steps;   // == chunks
};

constexpr int kDepth = 4;  // decodes in flight per producer wave

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also drains
// every outstanding global load (vmcnt(0)), which would serialise the
// producers' in-flight gathers with each macro-step; here only LDS operations
// (lgkmcnt) are waited for.  Global loads are still waited for where their
// registers are consumed.
__device__ __forceinline__ void block_sync_lds() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

template <int ACT, class Provider, int MW>
__global__ void __launch_bounds__(512)
tile_gemm_kernel(const GemmShape s, const typename Provider::Args pargs) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  constexpr int BM = 128 * MW;
  constexpr int kXBufBytes = BM * kRowBytes;
  constexpr int kPieces = BM * (kStepK / 8) / 256;  // 16-byte pieces of the x tile per consumer thread
  uint8_t* const xs = lds;                     // [2][BM][kRowBytes]
  uint8_t* const ws = lds + 2 * kXBufBytes;    // [2][64][kRowBytes]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: role branch is scalar
  const int m0 = blockIdx.y * BM;
  const int n0 = blockIdx.x * kTileCols;

  // Every wave executes the same number of barriers: one after the prologue and
  // one per iteration t = 0 .. total-1, where the last three iterations are
  // padding that lets the producers' four-iteration rounds end cleanly.
  const int total = s.steps + 3;
  // Column blocks walk k in rotated order (iteration t contracts chunk
  // (t + rot) mod steps): at any instant different blocks read different parts
  // of the index rows and of x, which spreads the traffic over the L2 channels
  // instead of all blocks hitting the same few address bits in lock step.
  const int rot = (int)((blockIdx.x * 7u) % (unsigned)s.steps);
  auto chunk_of = [&](int step) {
    const int kc = step + rot;
    return kc >= s.steps ? kc - s.steps : kc;
  };

  if (wave >= 4) {
    // ====================== producer wave q: steps p == q (mod 4) ==========
    // Production k of this wave is step q + 4k.  Its "slot" is iteration
    // q + 4k - 1, the one before the step is consumed.  In slot k the wave
    //   1. writes production k (gathered kDepth slots ago) to the W buffer,
    //   2. issues the gathers of production k + kDepth from the packed chunk it
    //      loaded kDepth slots ago,
    //   3. loads the packed chunk of production k + 2*kDepth.
    // Loads are consumed in the order they were issued, so the in-order VMEM
    // counter never has to drain younger gathers to release an older one.
    const Provider prov(pargs);
    const int q = wave - 4;
    // Branch-free decode: columns past N and productions past the last step
    // read clamped (valid) addresses; their results land in columns / buffers
    // nobody consumes.
    const int ncol = min(n0 + lane, s.N - 1);
    typename Provider::Raw raws[kDepth];
    u32x4 ops[kDepth][8];
    auto load_raw = [&](typename Provider::Raw& raw, int k) {
      prov.load(raw, ncol, chunk_of(min(q + 4 * k, s.steps - 1)));
    };
    auto produce = [&](u32x4 (&b)[8], const typename Provider::Raw& raw) {
      b[0] = prov.template operand<0>(raw);
      b[1] = prov.template operand<1>(raw);
      b[2] = prov.template operand<2>(raw);
      b[3] = prov.template operand<3>(raw);
      b[4] = prov.template operand<4>(raw);
      b[5] = prov.template operand<5>(raw);
      b[6] = prov.template operand<6>(raw);
      b[7] = prov.template operand<7>(raw);
    };
    auto store_w = [&](const u32x4 (&b)[8], int k) {
      uint8_t* dst = ws + ((q + 4 * k) & 1) * kWBufBytes + lane * kRowBytes;
#pragma unroll
      for (int j = 0; j < 8; ++j) *reinterpret_cast<u32x4*>(dst + j * 16) = b[j];
    };
    int t = 0;  // next iteration whose barrier this wave has not passed yet
    auto slot = [&](u32x4 (&b)[8], typename Provider::Raw& raw, int k) {
      store_w(b, k);
      produce(b, raw);
      load_raw(raw, k + 2 * kDepth);
    };
    auto round = [&](u32x4 (&b)[8], typename Provider::Raw& raw, int k) {  // slot + 3 idle iterations
      slot(b, raw, k);
      block_sync_lds();
      block_sync_lds();
      block_sync_lds();
      block_sync_lds();
      t += 4;
    };

    // Prologue: productions 0..kDepth-1 in flight, chunks kDepth..2*kDepth-1 loaded.
#pragma unroll
    for (int k = 0; k < kDepth; ++k) load_raw(raws[k], k);
#pragma unroll
    for (int k = 0; k < kDepth; ++k) produce(ops[k], raws[k]);
#pragma unroll
    for (int k = 0; k < kDepth; ++k) load_raw(raws[k], k + kDepth);
    // Step 0 is consumed in iteration 0: producer 0 runs its slot 0 now.
    if (q == 0) slot(ops[0], raws[0], 0);
    block_sync_lds();

    // Idle until the first slot after the prologue: iteration q - 1 (q >= 1),
    // or iteration 3 (q == 0, production 1).
    const int first = (q == 0) ? 3 : q - 1;
    while (t < first) {
      block_sync_lds();
      ++t;
    }
    // Rounds of four iterations, unrolled by kDepth so the register sets rotate
    // statically.  Producer 0 starts at production 1, the others at production 0.
    if (q == 0) {
      for (int k = 1; t + 4 <= total; k += 4) {
        round(ops[1], raws[1], k);
        if (t + 4 > total) break;
        round(ops[2], raws[2], k + 1);
        if (t + 4 > total) break;
        round(ops[3], raws[3], k + 2);
        if (t + 4 > total) break;
        round(ops[0], raws[0], k + 3);
      }
    } else {
      for (int k = 0; t + 4 <= total; k += 4) {
        round(ops[0], raws[0], k);
        if (t + 4 > total) break;
        round(ops[1], raws[1], k + 1);
        if (t + 4 > total) break;
        round(ops[2], raws[2], k + 2);
        if (t + 4 > total) break;
        round(ops[3], raws[3], k + 3);
      }
    }
    while (t < total) {
      block_sync_lds();
      ++t;
    }
    return;
  }

  // ========================= consumer wave ==================================
  const int c = lane & 31;
  const int h = lane >> 5;
  const int wrow0 = wave * (32 * MW);              // first tile row of this wave
  const bool wave_active = (m0 + wrow0) < s.M;     // waves past M still load x and keep the barriers
  const uint16_t* xg = reinterpret_cast<const uint16_t*>(s.x);

  f32x16 acc[MW][2];
#pragma unroll
  for (int mt = 0; mt < MW; ++mt)
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mt][t][i] = 0.f;

  auto load_x = [&](u32x4 (&xr)[kPieces], int step) {
#pragma unroll
    for (int i = 0; i < kPieces; ++i) {
      const int p = tid + i * 256;
      const int row = p >> 3, col8 = p & 7;
      const int m = min(m0 + row, s.M - 1);  // rows past M: clamped, never stored
      xr[i] = *reinterpret_cast<const u32x4*>(xg + (int64_t)m * s.ldx + chunk_of(step) * kStepK + col8 * 8);
      if constexpr (Provider::kPermuteA) xr[i] = permute_a_0415(xr[i]);
    }
  };
  auto store_x = [&](const u32x4 (&xr)[kPieces], int buf) {
#pragma unroll
    for (int i = 0; i < kPieces; ++i) {
      const int p = tid + i * 256;
      const int row = p >> 3, col8 = p & 7;
      *reinterpret_cast<u32x4*>(xs + buf * kXBufBytes + row * kRowBytes + col8 * 16) = xr[i];
    }
  };
  auto mma = [&](int step) {
    const uint8_t* xa = xs + (step & 1) * kXBufBytes + (wrow0 + c) * kRowBytes + h * 64;
    const uint8_t* wb = ws + (step & 1) * kWBufBytes + c * kRowBytes + h * 64;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const u32x4 b0 = *reinterpret_cast<const u32x4*>(wb + j * 16);
      const u32x4 b1 = *reinterpret_cast<const u32x4*>(wb + 32 * kRowBytes + j * 16);
#pragma unroll
      for (int mt = 0; mt < MW; ++mt) {
        const u32x4 a = *reinterpret_cast<const u32x4*>(xa + mt * 32 * kRowBytes + j * 16);
        acc[mt][0] = mfma32<ACT>(a, b0, acc[mt][0]);
        acc[mt][1] = mfma32<ACT>(a, b1, acc[mt][1]);
      }
    }
  };

  // x tile pipeline: the registers loaded during iteration s-1 hold tile s+1;
  // they are written to LDS at the top of iteration s and immediately reloaded
  // with tile s+2, so every global load has a full iteration to land.
  u32x4 xr[kPieces];
  load_x(xr, 0);
  store_x(xr, 0);
  if (s.steps > 1) load_x(xr, 1);
  block_sync_lds();

  for (int step = 0; step < total; ++step) {
    if (step + 1 < s.steps) store_x(xr, (step + 1) & 1);
    if (step + 2 < s.steps) load_x(xr, step + 2);
    if (wave_active && step < s.steps) mma(step);
    block_sync_lds();
  }

  // ---- epilogue: D[m = 8*(i/4) + 4h + i%4][n = c] --------------------------
  if (!wave_active) return;
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const int n = n0 + t * 32 + c;
    if (n >= s.N) continue;
    const float bv = s.bias ? s.bias[n] : 0.f;
#pragma unroll
    for (int mt = 0; mt < MW; ++mt) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int m = m0 + wrow0 + mt * 32 + 8 * (i / 4) + 4 * h + (i % 4);
        if (m < s.M) store_from_f32<ACT>(s.y, (int64_t)m * s.ldy + n, acc[mt][t][i] + bv);
      }
    }
  }
}

// Rows per block: 128*MW with MW = ceil(M / 128) capped at 3, so that M <= 384
// is one row block and every weight element is decoded exactly once.
// NPAMD_TILE_MW overrides the choice (tuning aid).
int plan_tile_mw(int M);

template <int ACT, class Provider, int MW>
int launch_tile_gemm_mw(const GemmShape& s, const typename Provider::Args& pargs, hipStream_t st,
                        const char* what) {
  constexpr int BM = 128 * MW;
  const dim3 grid((s.N + kTileCols - 1) / kTileCols, (s.M + BM - 1) / BM);
  const int lds = 2 * BM * kRowBytes + 2 * kWBufBytes;
  static bool attr_set = false;  // per instantiation: allow more than 64 KiB of dynamic LDS
  if (!attr_set) {
    const hipError_t e = hipFuncSetAttribute(
        reinterpret_cast<const void*>(&tile_gemm_kernel<ACT, Provider, MW>),
        hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (e != hipSuccess) return fail(NPAMD_ERR_LAUNCH, "%s: cannot reserve %d bytes of LDS: %s", what, lds,
                                     hipGetErrorString(e));
    attr_set = true;
  }
  tile_gemm_kernel<ACT, Provider, MW><<<grid, 512, lds, st>>>(s, pargs);
  return check_launch(what);
}

template <int ACT, class Provider>
int launch_tile_gemm(GemmShape s, const typename Provider::Args& pargs, hipStream_t st,
                     const char* what) {
  s.steps = s.chunks;
  switch (plan_tile_mw(s.M)) {
    case 1: return launch_tile_gemm_mw<ACT, Provider, 1>(s, pargs, st, what);
    case 2: return launch_tile_gemm_mw<ACT, Provider, 2>(s, pargs, st, what);
    default: return launch_tile_gemm_mw<ACT, Provider, 3>(s, pargs, st, what);
  }
}

// ---------------------------------------------------------------------------
// Fallback for shapes the MFMA kernel does not take: one thread per output
// element.  Slow by design; exists so every valid input has a HIP path.
// ---------------------------------------------------------------------------
template <int ACT, class Elem>
__global__ void __launch_bounds__(256)
generic_gemm_kernel(const void* __restrict__ x, int64_t ldx, const float* __restrict__ bias,
                    void* __restrict__ y, int64_t ldy, int M, int N, int K, const Elem elem) {
  const int n = blockIdx.x * 64 + (threadIdx.x & 63);
  const int m = blockIdx.y * 4 + (threadIdx.x >> 6);
  if (n >= N || m >= M) return;
  float acc = 0.f;
  for (int k = 0; k < K; ++k)
    acc = __builtin_fmaf(load_as_f32<ACT>(x, (int64_t)m * ldx + k), elem.get(n, k), acc);
  if (bias) acc += bias[n];
  store_from_f32<ACT>(y, (int64_t)m * ldy + n, acc);
}

template <int ACT, class Elem>
int launch_generic_gemm(const void* x, int64_t ldx, const float* bias, void* y, int64_t ldy,
                        int M, int N, int K, const Elem& elem, hipStream_t st, const char* what) {
  const dim3 grid((N + 63) / 64, (M + 3) / 4);
  generic_gemm_kernel<ACT, Elem><<<grid, 256, 0, st>>>(x, ldx, bias, y, ldy, M, N, K, elem);
  return check_launch(what);
}

}  // namespace npamd
