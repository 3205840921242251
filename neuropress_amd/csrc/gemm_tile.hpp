// Tile-decode GEMM: y = x @ W^T (+ bias) with W decoded inside the kernel,
// wave64 + MFMA 32x32x16, f32 accumulate.
//
// Operand roles: A = x tile (rows m), B = W^T (columns n).  For MFMA 32x32x16
// lane l = (c = l % 32, h = l / 32) supplies 8 consecutive k of row c for
// k-half h.  A weight "chunk" (64 k of one row = 8 B-operands, see
// providers.hpp) is decoded straight into registers in B layout -- the weight
// never passes through LDS.  Only the x tile is staged in LDS (double
// buffered), shared by the four waves of a block, which own 64 output columns
// each and all BM = 32*MT rows of the block.
//
// k order inside one MFMA is free as long as A and B agree: MFMA j of a
// macro-step (128 k) contracts k = {64h + 8j .. +7 : h = 0, 1}, which lets each
// lane fetch its 8 operands of a macro-step with a single packed-chunk load.
//
// Pipeline per macro-step s: packed chunk of s+2 and x tile of s+1 are loaded
// from global memory, the gathers/dequant for s+1 are issued, then the MFMAs
// of s run; one barrier per step.
#pragma once

#include "providers.hpp"

namespace npamd {

constexpr int kTileK = 128;                       // k per macro-step
constexpr int kTileRowBytes = kTileK * 2 + 16;    // padded LDS row stride (bank-conflict free b128 reads)
constexpr int kTileCols = 256;                    // output columns per block (4 waves x 64)

struct GemmShape {
  const void* x;
  int64_t ldx;
  const float* bias;
  void* y;
  int64_t ldy;
  int M, N, K;
  int chunks;  // K / 64
  int steps;   // ceil(K / 128)
};

template <int ACT, class Provider, int MT>
__global__ void __launch_bounds__(256)
tile_gemm_kernel(const GemmShape s, const typename Provider::Args pargs) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];  // [2][32*MT][kTileRowBytes]
  constexpr int BM = 32 * MT;
  constexpr int kBufBytes = BM * kTileRowBytes;
  constexpr int kPieces = BM * (kTileK / 8) / 256;  // 16-byte pieces of the x tile per thread

  const Provider prov(pargs);
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int c = lane & 31;
  const int h = lane >> 5;
  const int m0 = blockIdx.y * BM;
  const int n0 = blockIdx.x * kTileCols + wave * 64;
  const int nrow[2] = {n0 + c, n0 + 32 + c};
  const bool nvalid[2] = {nrow[0] < s.N, nrow[1] < s.N};
  const uint16_t* xg = reinterpret_cast<const uint16_t*>(s.x);

  f32x16 acc[MT][2];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mt][t][i] = 0.f;

  // ---- helpers ----------------------------------------------------------
  auto load_x = [&](u32x4 (&xr)[kPieces], int step) {
#pragma unroll
    for (int i = 0; i < kPieces; ++i) {
      const int p = tid + i * 256;
      const int row = p >> 4, col8 = p & 15;
      const int m = m0 + row, k = step * kTileK + col8 * 8;
      xr[i] = u32x4{0, 0, 0, 0};
      if (m < s.M && k < s.K) {
        xr[i] = *reinterpret_cast<const u32x4*>(xg + (int64_t)m * s.ldx + k);
        if constexpr (Provider::kPermuteA) xr[i] = permute_a_0415(xr[i]);
      }
    }
  };
  auto store_x = [&](const u32x4 (&xr)[kPieces], int buf) {
#pragma unroll
    for (int i = 0; i < kPieces; ++i) {
      const int p = tid + i * 256;
      const int row = p >> 4, col8 = p & 15;
      *reinterpret_cast<u32x4*>(lds + buf * kBufBytes + row * kTileRowBytes + col8 * 16) = xr[i];
    }
  };
  auto load_raw = [&](typename Provider::Raw (&raw)[2], int step) {
    const int kc = step * 2 + h;
    const bool kv = kc < s.chunks;
#pragma unroll
    for (int t = 0; t < 2; ++t) prov.load(raw[t], nrow[t], kc, kv && nvalid[t]);
  };
  auto make_b = [&](u32x4 (&b)[2][8], const typename Provider::Raw (&raw)[2], int step) {
    const bool kv = (step * 2 + h) < s.chunks;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const bool v = kv && nvalid[t];
      b[t][0] = prov.template operand<0>(raw[t], v);
      b[t][1] = prov.template operand<1>(raw[t], v);
      b[t][2] = prov.template operand<2>(raw[t], v);
      b[t][3] = prov.template operand<3>(raw[t], v);
      b[t][4] = prov.template operand<4>(raw[t], v);
      b[t][5] = prov.template operand<5>(raw[t], v);
      b[t][6] = prov.template operand<6>(raw[t], v);
      b[t][7] = prov.template operand<7>(raw[t], v);
    }
  };
  auto mma = [&](const u32x4 (&b)[2][8], int buf) {
    const uint8_t* base = lds + buf * kBufBytes + c * kTileRowBytes + h * 128;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const u32x4 a = *reinterpret_cast<const u32x4*>(base + mt * 32 * kTileRowBytes + j * 16);
        acc[mt][0] = mfma32<ACT>(a, b[0][j], acc[mt][0]);
        acc[mt][1] = mfma32<ACT>(a, b[1][j], acc[mt][1]);
      }
    }
  };

  // ---- prologue ---------------------------------------------------------
  u32x4 xr[kPieces];
  typename Provider::Raw raw[2];
  u32x4 b0[2][8], b1[2][8];

  load_x(xr, 0);
  load_raw(raw, 0);
  make_b(b0, raw, 0);
  load_raw(raw, 1);  // invalid past the end -> zeros
  store_x(xr, 0);
  __syncthreads();

  // ---- main loop, unrolled by two so the operand buffers ping-pong ------
  for (int step = 0; step < s.steps; step += 2) {
    {  // even step: use b0 / buf 0, fill b1 / buf 1
      const bool more = step + 1 < s.steps;
      if (more) load_x(xr, step + 1);
      make_b(b1, raw, step + 1);
      load_raw(raw, step + 2);
      mma(b0, 0);
      if (more) store_x(xr, 1);
      __syncthreads();
    }
    if (step + 1 < s.steps) {  // odd step: use b1 / buf 1, fill b0 / buf 0
      const bool more = step + 2 < s.steps;
      if (more) load_x(xr, step + 2);
      make_b(b0, raw, step + 2);
      load_raw(raw, step + 3);
      mma(b1, 1);
      if (more) store_x(xr, 0);
      __syncthreads();
    }
  }

  // ---- epilogue: D[m = 8*(i/4) + 4h + i%4][n = c] ------------------------
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    if (!nvalid[t]) continue;
    const int n = nrow[t];
    const float bv = s.bias ? s.bias[n] : 0.f;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int m = m0 + mt * 32 + 8 * (i / 4) + 4 * h + (i % 4);
        if (m < s.M) store_from_f32<ACT>(s.y, (int64_t)m * s.ldy + n, acc[mt][t][i] + bv);
      }
    }
  }
}

// Rows-per-block choice: fewest passes of the grid over the CUs, weighted by
// the per-block cost (MT tiles of MFMA work + one tile-equivalent of decode).
int plan_tile_mt(int M, int N);

template <int ACT, class Provider, int MT>
int launch_tile_gemm_mt(const GemmShape& s, const typename Provider::Args& pargs, hipStream_t st,
                        const char* what) {
  const dim3 grid((s.N + kTileCols - 1) / kTileCols, (s.M + 32 * MT - 1) / (32 * MT));
  const size_t lds = 2 * 32 * MT * kTileRowBytes;
  tile_gemm_kernel<ACT, Provider, MT><<<grid, 256, lds, st>>>(s, pargs);
  return check_launch(what);
}

template <int ACT, class Provider>
int launch_tile_gemm(GemmShape s, const typename Provider::Args& pargs, hipStream_t st,
                     const char* what) {
  s.steps = (s.K + kTileK - 1) / kTileK;
  switch (plan_tile_mt(s.M, s.N)) {
    case 1: return launch_tile_gemm_mt<ACT, Provider, 1>(s, pargs, st, what);
    case 2: return launch_tile_gemm_mt<ACT, Provider, 2>(s, pargs, st, what);
    case 3: return launch_tile_gemm_mt<ACT, Provider, 3>(s, pargs, st, what);
    default: return launch_tile_gemm_mt<ACT, Provider, 4>(s, pargs, st, what);
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
