// Group-affine n-bit weights (Q4_0 / GPTQ style): decode, fused GEMV, fused GEMM.
//
//   q = (w_pack[n, k/vpb] >> ((k%vpb)*nbits)) & mask ;  w = (float(q) - zp) * float(scale)
//
// Fast kernels cover the Q4_0 / Q8_0 / GPTQ layouts (4 or 8 bits, symmetric or with per-group
// fp16 zero points, group size a power-of-two multiple of 32, K % 64 == 0); every other valid
// combination (1/2 bits, odd group sizes, odd K) runs the element-wise fallback.
#include <stdlib.h>

#include "gemm_tile2.hpp"
#include "gemv.hpp"

namespace npamd {

// Decode, element-wise: any nbits / group size / zero point.
template <int OUT>
__global__ void __launch_bounds__(256)
q_dequant_generic_kernel(const uint8_t* __restrict__ w_pack, const uint16_t* __restrict__ scale,
                         const uint16_t* __restrict__ zero_point, int64_t total, int K, int nbits,
                         int group_size, void* __restrict__ out) {
#pragma clang fp contract(off)
  const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (e >= total) return;
  const int64_t n = e / K;
  const int k = (int)(e - n * K);
  const int vpb = 8 / nbits;
  const int q = (w_pack[n * (K / vpb) + k / vpb] >> ((k % vpb) * nbits)) & ((1 << nbits) - 1);
  const int64_t sidx = n * (K / group_size) + k / group_size;
  const float zp = zero_point ? f16_bits_to_f32(zero_point[sidx]) : (float)(1 << (nbits - 1));
  const float d = (float)q - zp;
  store_from_f32<OUT>(out, e, d * f16_bits_to_f32(scale[sidx]));
}

// Decode, 4-bit (symmetric, or ASYM with per-group zero points): one thread per dword of
// nibbles = 8 weights, one 16-byte (32-byte for f32) store.  group_size % 8 == 0 so the 8
// share a scale.
template <int OUT, bool ASYM>
__global__ void __launch_bounds__(256)
q4_dequant_kernel(const uint32_t* __restrict__ w_pack, const uint16_t* __restrict__ scale,
                  const uint16_t* __restrict__ zero_point, int64_t n_words, int words_per_row,
                  int groups_per_row, int words_per_group, void* __restrict__ out) {
#pragma clang fp contract(off)
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n_words) return;
  const int64_t n = i / words_per_row;
  const int wr = (int)(i - n * words_per_row);
  const int64_t sidx = n * groups_per_row + wr / words_per_group;
  const float sc = f16_bits_to_f32(scale[sidx]);
  const float zp = ASYM ? f16_bits_to_f32(zero_point[sidx]) : 8.0f;
  const uint32_t w = w_pack[i];
  float v[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) v[j] = ((float)((w >> (4 * j)) & 0xFu) - zp) * sc;
  if constexpr (OUT == NPAMD_F32) {
    reinterpret_cast<f32x4*>(out)[2 * i] = f32x4{v[0], v[1], v[2], v[3]};
    reinterpret_cast<f32x4*>(out)[2 * i + 1] = f32x4{v[4], v[5], v[6], v[7]};
  } else {
    u32x4 o;
    if constexpr (OUT == NPAMD_F16) {
      o.x = f32_to_f16_bits(v[0]) | (f32_to_f16_bits(v[1]) << 16);
      o.y = f32_to_f16_bits(v[2]) | (f32_to_f16_bits(v[3]) << 16);
      o.z = f32_to_f16_bits(v[4]) | (f32_to_f16_bits(v[5]) << 16);
      o.w = f32_to_f16_bits(v[6]) | (f32_to_f16_bits(v[7]) << 16);
    } else {
      o.x = f32_to_bf16_bits(v[0]) | (f32_to_bf16_bits(v[1]) << 16);
      o.y = f32_to_bf16_bits(v[2]) | (f32_to_bf16_bits(v[3]) << 16);
      o.z = f32_to_bf16_bits(v[4]) | (f32_to_bf16_bits(v[5]) << 16);
      o.w = f32_to_bf16_bits(v[6]) | (f32_to_bf16_bits(v[7]) << 16);
    }
    reinterpret_cast<u32x4*>(out)[i] = o;
  }
}

// Decode, 1 / 2 / 8 bits: one thread per eight weights (NBITS bytes of codes), same arithmetic
// as the element-wise kernel, one 16-byte (32-byte for f32) store.
template <int NBITS, int OUT>
__global__ void __launch_bounds__(256)
qn_dequant_kernel(const uint8_t* __restrict__ w_pack, const uint16_t* __restrict__ scale,
                  const uint16_t* __restrict__ zero_point, int64_t n_octets, int octets_per_row,
                  int groups_per_row, int octets_per_group, void* __restrict__ out) {
#pragma clang fp contract(off)
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n_octets) return;
  const int64_t n = i / octets_per_row;
  const int o = (int)(i - n * octets_per_row);
  const int64_t sidx = n * groups_per_row + o / octets_per_group;
  const float sc = f16_bits_to_f32(scale[sidx]);
  const float zp = zero_point ? f16_bits_to_f32(zero_point[sidx]) : (float)(1 << (NBITS - 1));
  uint64_t bits;
  if constexpr (NBITS == 8) {
    const u32x2 t = *reinterpret_cast<const u32x2*>(w_pack + i * 8);
    bits = (uint64_t)t.x | ((uint64_t)t.y << 32);
  } else if constexpr (NBITS == 2) {
    bits = *reinterpret_cast<const uint16_t*>(w_pack + i * 2);
  } else {
    bits = w_pack[i];
  }
  float v[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) v[j] = ((float)(uint32_t)((bits >> (NBITS * j)) & ((1u << NBITS) - 1u)) - zp) * sc;
  if constexpr (OUT == NPAMD_F32) {
    reinterpret_cast<f32x4*>(out)[2 * i] = f32x4{v[0], v[1], v[2], v[3]};
    reinterpret_cast<f32x4*>(out)[2 * i + 1] = f32x4{v[4], v[5], v[6], v[7]};
  } else {
    uint32_t h[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) h[j] = OUT == NPAMD_F16 ? f32_to_f16_bits(v[j]) : f32_to_bf16_bits(v[j]);
    reinterpret_cast<u32x4*>(out)[i] = u32x4{h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16), h[6] | (h[7] << 16)};
  }
}

// ---------------------------------------------------------------------------
// Row-wise GEMV for 4-bit weights, one token (written out for the symmetric case, zero point 8).
//
// A lane takes 16 bytes of one weight row = 32 nibbles = one 32-k group, so the
// weight stream is read with plain coalesced 16-byte loads and the kernel is
// meant to run at HBM speed.  Nibbles become fp16 without a subtraction or a
// multiplication: a nibble in mantissa bits 0..3 of 0x6400 reads as 1024 + q, one
// in bits 4..7 of 0x5400 as 64 + q, so with b[k] = 1024 for even k and 64 for odd k
//     sum_k x[k] * (q[k] - 8) * s = s * (sum_k x[k] * (b[k] + q[k]) - sum_k (b[k] + 8) * x[k])
// with the first sum taken by packed dot products (products exact in f32) and the
// second, which depends on x only, precomputed per 32-k group.  One shift and four
// and-or instructions turn eight nibbles into four fp16 pairs (k, k+4); x is staged
// in LDS once per block in the same pair order and in a lane-major layout, so its
// reads are conflict-free.  f32 accumulation; a group's sum is up to ~500 times
// larger than its useful part, i.e. nine of the 24 bits: the result still carries
// more bits than the fp16 output keeps (measured: error = output rounding).
// bf16 activations: 7 mantissa bits leave room for 128 + q only, three shifts.
// ---------------------------------------------------------------------------
struct Q4RowArgs {
  const uint16_t* x; int64_t ldx;
  const uint8_t* w_pack;   // [N, K/2]
  const uint16_t* scale;   // [N, K/gs]
  const uint16_t* zp;      // [N, K/gs] or null (zero point 8)
  const float* bias; uint16_t* y; int64_t ldy;
  int N, K;
  int groups32;            // K / 32
  int passes;              // ceil(groups32 / 64)
  int scales_per_row;      // K / gs
  int gs_shift;            // log2(gs / 32)
};

// Operands by value (a bit cast applied directly to a vector element reads element 0).
template <int ACT>
__device__ __forceinline__ float fdot2_act(uint32_t a, uint32_t b, float c) {
  if constexpr (ACT == NPAMD_BF16)
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a), __builtin_bit_cast(bf16x2, b), c, false);
  else
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, a), __builtin_bit_cast(f16x2, b), c, false);
}

// (v & mask) | magic in one instruction; the compiler emits two when both constants are literals.
__device__ __forceinline__ uint32_t and_or(uint32_t v, uint32_t mask, uint32_t magic) {
  uint32_t r;
  asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(v), "s"(mask), "v"(magic));
  return r;
}

// The row-wise kernel's blocks have W = 4 or 8 waves; a wave owns R consecutive rows.

template <int R>
struct Q4RowItem {   // one pass (64 groups of 32 k) of R rows
  u32x4 w[R];
  uint16_t sc[R];
  uint16_t zp[R];    // ASYM only
};

template <int R, bool ASYM>
__device__ __forceinline__ void q4_row_load(Q4RowItem<R>& it, const Q4RowArgs& a, int r0, int p, int lane) {
  const int g = min(p * 64 + lane, a.groups32 - 1);
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int n = min(r0 + i, a.N - 1);
    it.w[i] = *reinterpret_cast<const u32x4*>(a.w_pack + (int64_t)n * (a.K / 2) + (int64_t)g * 16);
    it.sc[i] = a.scale[(int64_t)n * a.scales_per_row + (g >> a.gs_shift)];
    if constexpr (ASYM) it.zp[i] = a.zp[(int64_t)n * a.scales_per_row + (g >> a.gs_shift)];
  }
}

// With a zero point z instead of 8 the part that depends on x only becomes
// sum_k (b[k] + z) * x[k] = off + (z - 8) * sum_k x[k]: a second table (the plain sum of the
// group's activations) and one more multiply-add per row and group.
template <int ACT, int M, int R, bool ASYM>
__device__ __forceinline__ void q4_row_compute(const Q4RowItem<R>& it, const Q4RowArgs& a, const u32x4* xs,
                                               const float* off, const float* sumx, int p, int lane,
                                               float (&acc)[R][M]) {
  const bool live = p * 64 + lane < a.groups32;
  // fp16: 1024 + q (nibble in mantissa bits 0..3) and 64 + q (bits 4..7).
  // bf16 has 7 mantissa bits: only 128 + q (bits 0..3 of 0x4300), so three shifts.
  const uint32_t magic_lo = ACT == NPAMD_BF16 ? 0x43004300u : 0x64006400u, magic_hi = 0x54005400u;
  u32x4 xv[M][4];
  float of[M], sx[M];
#pragma unroll
  for (int m = 0; m < M; ++m) {
#pragma unroll
    for (int j = 0; j < 4; ++j) xv[m][j] = xs[((size_t)m * a.passes * 4 + (size_t)p * 4 + j) * 64 + lane];
    of[m] = off[(m * a.passes + p) * 64 + lane];
    if constexpr (ASYM) sx[m] = sumx[(m * a.passes + p) * 64 + lane];
  }
#pragma unroll
  for (int i = 0; i < R; ++i) {
    float g_acc[M];
#pragma unroll
    for (int m = 0; m < M; ++m) {
      g_acc[m] = -of[m];
      if constexpr (ASYM) g_acc[m] = __builtin_fmaf(8.0f - f16_bits_to_f32(it.zp[i]), sx[m], g_acc[m]);
    }
    const uint32_t wd[4] = {it.w[i].x, it.w[i].y, it.w[i].z, it.w[i].w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t u = wd[j], u8 = u >> 8;
      uint32_t p0, p1, p2, p3;
      p0 = and_or(u, 0x000F000Fu, magic_lo);   // (b + q0, b + q4)
      p2 = and_or(u8, 0x000F000Fu, magic_lo);  // (b + q2, b + q6)
      if constexpr (ACT == NPAMD_BF16) {
        p1 = and_or(u >> 4, 0x000F000Fu, magic_lo);   // (128 + q1, 128 + q5)
        p3 = and_or(u >> 12, 0x000F000Fu, magic_lo);  // (128 + q3, 128 + q7)
      } else {
        p1 = and_or(u, 0x00F000F0u, magic_hi);   // (64 + q1, 64 + q5)
        p3 = and_or(u8, 0x00F000F0u, magic_hi);  // (64 + q3, 64 + q7)
      }
#pragma unroll
      for (int m = 0; m < M; ++m) {
        const u32x4 xx = xv[m][j];
        float t = g_acc[m];
        t = fdot2_act<ACT>(p0, xx.x, t);
        t = fdot2_act<ACT>(p1, xx.y, t);
        t = fdot2_act<ACT>(p2, xx.z, t);
        t = fdot2_act<ACT>(p3, xx.w, t);
        g_acc[m] = t;
      }
    }
    const float s_eff = live ? f16_bits_to_f32(it.sc[i]) : 0.f;
#pragma unroll
    for (int m = 0; m < M; ++m) acc[i][m] = __builtin_fmaf(s_eff, g_acc[m], acc[i][m]);
  }
}

template <int ACT, int M, int R, bool ASYM, int W>
__global__ void __launch_bounds__(W * 64) q4_rowwise_gemv_kernel(Q4RowArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  // xs[m][pass][piece 0..3][lane] (16-byte vectors), then off[m][pass][lane] (floats), then
  // (ASYM) sumx[m][pass][lane].
  u32x4* xs = reinterpret_cast<u32x4*>(smem);
  float* off = reinterpret_cast<float*>(smem + (size_t)M * a.passes * 4 * 64 * 16);
  float* sumx = off + (size_t)M * a.passes * 64;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r0 = (blockIdx.x * W + wave) * R;

  // The first pass of weights is requested before x is staged (requesting two here is
  // slower: 11.5 vs 9.2 us on 14336 x 4096).
  Q4RowItem<R> cur, nxt;
  q4_row_load<R, ASYM>(cur, a, r0, 0, lane);

  // Stage x: one thread per (token, 32-k group): its four vectors go to the lane-major
  // layout in (k, k+4) pair order, sum (b[k] + 8) * x[k] to the offset table.
  for (int i = tid; i < M * a.passes * 64; i += W * 64) {
    const int m = i / (a.passes * 64), g = i % (a.passes * 64);
    const u32x4* xg = reinterpret_cast<const u32x4*>(a.x + (int64_t)m * a.ldx) + (size_t)g * 4;
    float sum_even = 0.f, sum_odd = 0.f;  // over even / odd k of the group
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      u32x4 v = {0u, 0u, 0u, 0u};
      if (g < a.groups32) v = permute_a_0415(xg[j]);
      const uint32_t d[4] = {v.x, v.y, v.z, v.w};  // (k0,k4) (k1,k5) (k2,k6) (k3,k7)
      sum_even += act_bits_to_f32<ACT>(d[0] & 0xFFFFu) + act_bits_to_f32<ACT>(d[0] >> 16) +
                  act_bits_to_f32<ACT>(d[2] & 0xFFFFu) + act_bits_to_f32<ACT>(d[2] >> 16);
      sum_odd += act_bits_to_f32<ACT>(d[1] & 0xFFFFu) + act_bits_to_f32<ACT>(d[1] >> 16) +
                 act_bits_to_f32<ACT>(d[3] & 0xFFFFu) + act_bits_to_f32<ACT>(d[3] >> 16);
      xs[((size_t)m * a.passes * 4 + (size_t)(g >> 6) * 4 + j) * 64 + (g & 63)] = v;
    }
    off[i] = ACT == NPAMD_BF16 ? 136.f * (sum_even + sum_odd) : 1032.f * sum_even + 72.f * sum_odd;
    if constexpr (ASYM) sumx[i] = sum_even + sum_odd;
  }
  __syncthreads();
  if (r0 >= a.N) return;

  float acc[R][M];
#pragma unroll
  for (int i = 0; i < R; ++i)
#pragma unroll
    for (int m = 0; m < M; ++m) acc[i][m] = 0.f;
  // Two passes in flight: the next one is requested before the current one is used.
  int p = 0;
  for (; p + 2 <= a.passes; p += 2) {
    q4_row_load<R, ASYM>(nxt, a, r0, p + 1, lane);
    q4_row_compute<ACT, M, R, ASYM>(cur, a, xs, off, sumx, p, lane, acc);
    q4_row_load<R, ASYM>(cur, a, r0, min(p + 2, a.passes - 1), lane);
    q4_row_compute<ACT, M, R, ASYM>(nxt, a, xs, off, sumx, p + 1, lane, acc);
  }
  if (p < a.passes) q4_row_compute<ACT, M, R, ASYM>(cur, a, xs, off, sumx, p, lane, acc);

#pragma unroll
  for (int i = 0; i < R; ++i)
#pragma unroll
    for (int m = 0; m < M; ++m) {
      const float total = wave_reduce_sum(acc[i][m]);
      const int n = r0 + i;
      if (lane == 0 && n < a.N)
        store_from_f32<ACT>(a.y, (int64_t)m * a.ldy + n, total + (a.bias ? a.bias[n] : 0.f));
    }
}

// ---------------------------------------------------------------------------
// One token, whole layer streamed by one resident grid: at most one block per compute unit, no
// LDS on the way in.  A lane owns two adjacent 32-k groups (32 bytes of a row, 64 values of x),
// a wave 4096 columns ("pass" p of the row), a block's waves are arranged as (row lane j, pass
// p).  In iteration `it` the grid contracts rows [it * row_stride, (it + 1) * row_stride), so
// at any time it reads one contiguous window of the weights.  Every wave keeps its x values (in
// the (k, k+4) pair order of the decoded nibbles) and their offsets in registers for its whole
// life; x is requested first, then up to four rows' weights and scales, and each row is
// contracted as it arrives.  A row's sum is reduced inside the wave with DPP adds and lane
// reads; with more than one pass the parts meet in LDS and are added in pass order.
// Same arithmetic as the kernel above (base + q nibbles, group offsets folded out, f32).
// ---------------------------------------------------------------------------
constexpr int kQ4StreamMaxWaves = 16;

struct Q4StreamGeom {
  int passes;           // ceil(K / 4096)
  int waves;            // per block: row_lanes * passes
  int row_lanes;        // L: rows a block works on at a time
  int blocks;
  int row_stride;       // blocks * L: rows the grid works on at a time
  int iterations;       // ceil(N / row_stride)
  int pairs;            // K / 64
};

struct Q4StreamItem {
  u32x4 w[2];
  uint32_t sc, zp;      // two fp16 values each: the lane's two groups
};

// A lane's two groups are 64 groups apart: each of the two weight loads of a wave covers one
// contiguous KiB.
template <bool ASYM>
__device__ __forceinline__ void q4_stream_load(Q4StreamItem& it, const Q4RowArgs& a, int row, int g0, int g1) {
  const uint8_t* w = a.w_pack + (int64_t)row * (a.K / 2);
  it.w[0] = *reinterpret_cast<const u32x4*>(w + (int64_t)g0 * 16);
  it.w[1] = *reinterpret_cast<const u32x4*>(w + (int64_t)g1 * 16);
  const int64_t at = (int64_t)row * a.scales_per_row;
  it.sc = a.scale[at + (g0 >> a.gs_shift)] | ((uint32_t)a.scale[at + (g1 >> a.gs_shift)] << 16);
  if constexpr (ASYM) it.zp = a.zp[at + (g0 >> a.gs_shift)] | ((uint32_t)a.zp[at + (g1 >> a.gs_shift)] << 16);
}

template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
  const int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false);
  return v + __builtin_bit_cast(float, moved);
}

// Sum over the 64 lanes, the same value in every lane: four rotations inside each row of 16
// lanes, then the four row totals are read out and added in lane order.
__device__ __forceinline__ float wave_total(float v) {
  v = dpp_add<0x128>(v);  // row_ror:8
  v = dpp_add<0x124>(v);  // row_ror:4
  v = dpp_add<0x122>(v);  // row_ror:2
  v = dpp_add<0x121>(v);  // row_ror:1
  const int b = __builtin_bit_cast(int, v);
  const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0));
  const float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16));
  const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32));
  const float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48));
  return (r0 + r1) + (r2 + r3);
}

struct Q4StreamX {
  u32x4 v[2][4];        // per group: four vectors of (k, k+4) pairs
  float off[2], sum[2]; // per group: what base + 8 adds to the dot product; plain sum (zero points)
};

template <int ACT>
__device__ __forceinline__ float q4_group_dot(const u32x4& w, const u32x4 (&xv)[4], float t) {
  const uint32_t magic_lo = ACT == NPAMD_BF16 ? 0x43004300u : 0x64006400u, magic_hi = 0x54005400u;
  const uint32_t wd[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const uint32_t u = wd[q], u8 = u >> 8;
    uint32_t p0, p1, p2, p3;
    p0 = and_or(u, 0x000F000Fu, magic_lo);
    p2 = and_or(u8, 0x000F000Fu, magic_lo);
    if constexpr (ACT == NPAMD_BF16) {
      p1 = and_or(u >> 4, 0x000F000Fu, magic_lo);
      p3 = and_or(u >> 12, 0x000F000Fu, magic_lo);
    } else {
      p1 = and_or(u, 0x00F000F0u, magic_hi);
      p3 = and_or(u8, 0x00F000F0u, magic_hi);
    }
    t = fdot2_act<ACT>(p0, xv[q].x, t);
    t = fdot2_act<ACT>(p1, xv[q].y, t);
    t = fdot2_act<ACT>(p2, xv[q].z, t);
    t = fdot2_act<ACT>(p3, xv[q].w, t);
  }
  return t;
}

constexpr int kQ4StreamXStride = 80;   // bytes between the x values of two groups in LDS: 64 + 16, so
                                       // that 16 lanes reading their own piece hit 16 different bank groups

template <int ACT, bool ASYM>
__device__ __forceinline__ void q4_stream_row(const Q4StreamItem& item, const Q4StreamX& x, bool live0, bool live1,
                                              float* slot, int lane) {
  float v = 0.f;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    float t = -x.off[h];
    if constexpr (ASYM) t = __builtin_fmaf(8.0f - f16_bits_to_f32((item.zp >> (16 * h)) & 0xFFFFu), x.sum[h], t);
    t = q4_group_dot<ACT>(item.w[h], x.v[h], t);
    v = __builtin_fmaf((h ? live1 : live0) ? f16_bits_to_f32((item.sc >> (16 * h)) & 0xFFFFu) : 0.f, t, v);
  }
  const float total = wave_total(v);
  // Parked in LDS: the bias load of a store issued here would have to wait for every weight
  // request of the wave that is still under way (loads return in order).
  if (lane == 0 && slot) *slot = total;
}

// The code is kept small on purpose (one row loop, two rows in flight per wave): a kernel that
// lasts a few microseconds executes every instruction for the first time, and straight-line
// code for many rows is paced by instruction-cache misses.
template <int ACT, bool ASYM>
__global__ void __launch_bounds__(kQ4StreamMaxWaves * 64) q4_stream_gemv_kernel(Q4RowArgs a, Q4StreamGeom geo) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  uint8_t* xs = smem;  // x: 80 bytes per 32-k group
  float* part = reinterpret_cast<float*>(smem + geo.passes * 128 * kQ4StreamXStride);  // [iteration][row lane][pass]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int p = wave % geo.passes, j = wave / geo.passes;
  const bool live0 = p * 128 + lane < a.groups32, live1 = p * 128 + 64 + lane < a.groups32;
  const int g0 = min(p * 128 + lane, a.groups32 - 1), g1 = min(p * 128 + 64 + lane, a.groups32 - 1);
  const int row_first = blockIdx.x * geo.row_lanes + j;
  const int threads = geo.waves * 64, pieces = a.groups32 * 4;

  // x is requested ahead of the weights (loads return in order: behind them it would hold the
  // first row back) and goes through LDS once per block.
  u32x4 piece[2];
#pragma unroll
  for (int r = 0; r < 2; ++r)
    if (tid + r * threads < pieces) piece[r] = reinterpret_cast<const u32x4*>(a.x)[tid + r * threads];
  Q4StreamItem cur, nxt;
  q4_stream_load<ASYM>(cur, a, min(row_first, a.N - 1), g0, g1);
  q4_stream_load<ASYM>(nxt, a, min(row_first + geo.row_stride, a.N - 1), g0, g1);
#pragma unroll
  for (int r = 0; r < 2; ++r) {
    const int q = tid + r * threads;
    if (q < pieces) *reinterpret_cast<u32x4*>(xs + (q >> 2) * kQ4StreamXStride + (q & 3) * 16) = piece[r];
  }
  for (int q = tid + 2 * threads; q < pieces; q += threads)  // rows too few to fill the block with waves
    *reinterpret_cast<u32x4*>(xs + (q >> 2) * kQ4StreamXStride + (q & 3) * 16) = reinterpret_cast<const u32x4*>(a.x)[q];
  block_sync_lds();
  Q4StreamX x;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    float sum_even = 0.f, sum_odd = 0.f;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      x.v[h][q] = permute_a_0415(*reinterpret_cast<const u32x4*>(xs + (h ? g1 : g0) * kQ4StreamXStride + q * 16));
      const uint32_t d[4] = {x.v[h][q].x, x.v[h][q].y, x.v[h][q].z, x.v[h][q].w};
      sum_even += act_bits_to_f32<ACT>(d[0] & 0xFFFFu) + act_bits_to_f32<ACT>(d[0] >> 16) +
                  act_bits_to_f32<ACT>(d[2] & 0xFFFFu) + act_bits_to_f32<ACT>(d[2] >> 16);
      sum_odd += act_bits_to_f32<ACT>(d[1] & 0xFFFFu) + act_bits_to_f32<ACT>(d[1] >> 16) +
                 act_bits_to_f32<ACT>(d[3] & 0xFFFFu) + act_bits_to_f32<ACT>(d[3] >> 16);
    }
    x.off[h] = ACT == NPAMD_BF16 ? 136.f * (sum_even + sum_odd) : 1032.f * sum_even + 72.f * sum_odd;
    x.sum[h] = sum_even + sum_odd;
  }

  // Rows beyond the last iteration are clamped to the last row (cache hits) and not recorded.
  for (int it = 0; it < geo.iterations; it += 2) {
    q4_stream_row<ACT, ASYM>(cur, x, live0, live1, part + (it * geo.row_lanes + j) * geo.passes + p, lane);
    q4_stream_load<ASYM>(cur, a, min(row_first + (it + 2) * geo.row_stride, a.N - 1), g0, g1);
    q4_stream_row<ACT, ASYM>(nxt, x, live0, live1,
                             it + 1 < geo.iterations ? part + ((it + 1) * geo.row_lanes + j) * geo.passes + p : nullptr, lane);
    q4_stream_load<ASYM>(nxt, a, min(row_first + (it + 3) * geo.row_stride, a.N - 1), g0, g1);
  }
  __syncthreads();
  for (int r = tid; r < geo.iterations * geo.row_lanes; r += geo.waves * 64) {
    const int n = (r / geo.row_lanes) * geo.row_stride + blockIdx.x * geo.row_lanes + r % geo.row_lanes;
    if (n >= a.N) continue;
    float total = 0.f;
    for (int q = 0; q < geo.passes; ++q) total += part[r * geo.passes + q];
    store_from_f32<ACT>(a.y, n, total + (a.bias ? a.bias[n] : 0.f));
  }
}

struct QCall {
  const void* x; int64_t ldx;
  const uint8_t* w_pack; const void* scale; const void* zp;
  const float* bias; void* y; int64_t ldy;
  int M, N, K, nbits, gs, act;
  hipStream_t st;
  const char* what;
  void* ws = nullptr;      // tile GEMM only: f32 scratch for split-K partial tiles (may stay null)
  int64_t ws_bytes = 0;
};

static int log2i(int v) { int s = 0; while ((1 << s) < v) ++s; return s; }
static bool is_pow2(int v) { return v > 0 && (v & (v - 1)) == 0; }
static bool ptr_aligned(const void* p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

static int validate_q(const char* what, int N, int K, int nbits, int gs) {
  NPAMD_REQUIRE(nbits == 1 || nbits == 2 || nbits == 4 || nbits == 8,
                "%s: nbits must be one of {1, 2, 4, 8}, got %d", what, nbits);
  NPAMD_REQUIRE(N >= 0 && K >= 0, "%s: negative dimension", what);
  NPAMD_REQUIRE(gs > 0 && K % gs == 0, "%s: K=%d not divisible by group_size=%d", what, K, gs);
  NPAMD_REQUIRE(K % (8 / nbits) == 0, "%s: K=%d not a whole number of packed bytes", what, K);
  return NPAMD_OK;
}

static bool q_fast_ok(const QCall& c) {
  return (c.nbits == 4 || c.nbits == 8) && c.gs % 32 == 0 && is_pow2(c.gs / 32) && c.K % 64 == 0 &&
         c.K > 0 && c.ldx % 8 == 0 && ptr_aligned(c.x, 16) && ptr_aligned(c.w_pack, 16);
}



static int device_cus_q4() {
  static std::atomic<int> cached{0};
  int cus = cached.load(std::memory_order_relaxed);
  if (cus == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    cus = (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess &&
           prop.multiProcessorCount > 0) ? prop.multiProcessorCount : 256;
    cached.store(cus, std::memory_order_relaxed);
  }
  return cus;
}

template <int ACT, int M, int R, int W>
static int launch_q4_rowwise_rw(const Q4RowArgs& a, hipStream_t st, const char* what) {
  const int rows_per_block = R * W;
  const int blocks = (a.N + rows_per_block - 1) / rows_per_block;
  const int lds = M * a.passes * (4 * 64 * 16 + 64 * 4 * 2);
  if (a.zp) q4_rowwise_gemv_kernel<ACT, M, R, true, W><<<blocks, W * 64, lds, st>>>(a);
  else q4_rowwise_gemv_kernel<ACT, M, R, false, W><<<blocks, W * 64, lds, st>>>(a);
  return check_launch(what);
}

template <int ACT, int M, int R>
static int launch_q4_rowwise_r(const Q4RowArgs& a, int waves, hipStream_t st, const char* what) {
  return waves >= 8 ? launch_q4_rowwise_rw<ACT, M, R, 8>(a, st, what) : launch_q4_rowwise_rw<ACT, M, R, 4>(a, st, what);
}

template <int ACT, int M>
static int launch_q4_rowwise(const QCall& c) {
  Q4RowArgs a;
  a.x = (const uint16_t*)c.x; a.ldx = c.ldx;
  a.w_pack = c.w_pack; a.scale = (const uint16_t*)c.scale; a.zp = (const uint16_t*)c.zp;
  a.bias = c.bias; a.y = (uint16_t*)c.y; a.ldy = c.ldy;
  a.N = c.N; a.K = c.K;
  a.groups32 = c.K / 32;
  a.passes = (a.groups32 + 63) / 64;
  a.scales_per_row = c.K / c.gs;
  a.gs_shift = log2i(c.gs / 32);
  // Rows per wave: 2 when that still leaves sixteen waves per compute unit, else 1; waves per
  // block (x is staged once per block): 8 from four passes up, else 4.  Measured (us, 4 / 8 / 16
  // waves): 14336 x 4096 one row 11.6 / 10.9 / 11.2, two rows 9.7 / 10.7 / 10.6, four 10.2 / 10.3 / 10.1;
  // 4096 x 4096 one row 5.07 / 5.0 / 5.05, two 5.3 / 5.3 / 5.9; 4096 x 14336 one row 10.5 / 9.3 / 9.2,
  // two 10.0 / 9.6 / 11.3.
  const int cus = device_cus_q4();
  const int r_env = tuning().q4_rows;
  const int r = r_env ? r_env : (c.N >= 32 * cus ? 2 : 1);
  const int waves = a.passes >= 4 ? 8 : 4;
  if (r >= 4) return launch_q4_rowwise_r<ACT, M, 4>(a, waves, c.st, c.what);
  if (r >= 2) return launch_q4_rowwise_r<ACT, M, 2>(a, waves, c.st, c.what);
  return launch_q4_rowwise_r<ACT, M, 1>(a, waves, c.st, c.what);
}

// The resident-grid kernel takes one token of a layer with at most 16 passes (K <= 65536) whose
// per-block tables fit 64 KiB of LDS, from 64 Mi weights (32 MiB packed) up: it then streams at
// the rate of a plain read, while the kernel above restages x in every block, and its longer
// start (x through LDS before the first row can be contracted, two rows in flight per wave)
// loses on less.  Measured, us per call, row-wise / resident: 11008 x 4096 8.6 / 9.3,
// 16384 x 2048 8.4 / 8.7, 14336 x 4096 9.75 / 9.8, 8192 x 8192 10.8 / 10.7, 16384 x 4096
// 11.9 / 10.2, 32768 x 2048 13.3 / 12.8, 24576 x 4096 15.6 / 12.7, 28672 x 4096 17.7 / 14.6.
// NPAMD_Q4_STREAM=2 takes it wherever it fits, 0 never.  Blocks are as many as give every block
// the same number of rows.
static bool q4_stream_geometry(const QCall& c, Q4StreamGeom& geo) {
  geo.pairs = c.K / 64;
  geo.passes = (geo.pairs + 63) / 64;
  if (c.M != 1 || geo.passes < 1 || geo.passes > kQ4StreamMaxWaves || tuning().q4_stream == 0) return false;
  geo.row_lanes = kQ4StreamMaxWaves / geo.passes;
  if (geo.row_lanes > c.N) geo.row_lanes = c.N;
  const int row_groups = (c.N + geo.row_lanes - 1) / geo.row_lanes;
  const int cus = device_cus_q4();
  geo.iterations = (row_groups + cus - 1) / cus;
  geo.blocks = (row_groups + geo.iterations - 1) / geo.iterations;
  geo.row_stride = geo.blocks * geo.row_lanes;
  geo.waves = geo.row_lanes * geo.passes;
  if ((int64_t)c.N * c.K < ((int64_t)64 << 20) && tuning().q4_stream < 2) return false;
  return (int64_t)geo.iterations * geo.row_lanes * geo.passes * 4 + geo.passes * 128 * kQ4StreamXStride <= 64 * 1024;
}

template <int ACT>
static int launch_q4_stream(const QCall& c, const Q4StreamGeom& geo) {
  Q4RowArgs a;
  a.x = (const uint16_t*)c.x; a.ldx = c.ldx;
  a.w_pack = c.w_pack; a.scale = (const uint16_t*)c.scale; a.zp = (const uint16_t*)c.zp;
  a.bias = c.bias; a.y = (uint16_t*)c.y; a.ldy = c.ldy;
  a.N = c.N; a.K = c.K;
  a.groups32 = c.K / 32;
  a.passes = geo.passes;
  a.scales_per_row = c.K / c.gs;
  a.gs_shift = log2i(c.gs / 32);
  const int lds = geo.passes * 128 * kQ4StreamXStride + geo.iterations * geo.row_lanes * geo.passes * 4;
  const dim3 grid(geo.blocks), block(geo.waves * 64);
  if (a.zp) q4_stream_gemv_kernel<ACT, true><<<grid, block, lds, c.st>>>(a, geo);
  else q4_stream_gemv_kernel<ACT, false><<<grid, block, lds, c.st>>>(a, geo);
  return check_launch(c.what);
}

// bf16: the row-wise kernel keeps the unrounded weight (q - 8) * s, while the dequant-then-matmul
// path it is checked against rounds every weight to bf16 (8 bits); at K = 14336 the two differ by
// up to 4.5e-2, more than the 1e-2 parity bound, so bf16 stays on the MFMA GEMV (which rounds the
// same way) unless NPAMD_Q4_ROWWISE_BF16=1 asks for the faster, more exact kernel.
// The row-wise kernel serves one token (at two tokens the MFMA GEMV is as fast:
// 13.5 vs 13.8 us on 14336 x 4096), x staged in at most 64 KiB of LDS.
static bool q4_rowwise_ok(const QCall& c) {
  const int passes = (c.K / 32 + 63) / 64;
  return (c.act == NPAMD_F16 || tuning().q4_rowwise_bf16 != 0) && c.M == 1 && c.M * passes * (4 * 64 * 16 + 64 * 4 * 2) <= 64 * 1024 &&
         ptr_aligned(c.scale, 2) && tuning().q4_rowwise != 0;
}

template <int ACT, bool ASYM>
static int q4_fused(const QCall& c, bool gemv) {
  using P = Q4Provider<ACT, ASYM>;
  typename P::Args a{c.w_pack, (const uint16_t*)c.scale, c.K / 64, c.K / c.gs, log2i(c.gs / 32), (const uint16_t*)c.zp};
  if (gemv) {
    GemvShape s{c.x, c.ldx, c.bias, c.y, c.ldy, c.M, c.N, c.K / 64, 0, 0};
    return launch_fused_gemv<ACT, P>(s, a, c.st, c.what);
  }
  GemmShape s{c.x, c.ldx, c.bias, c.y, c.ldy, c.M, c.N, c.K, c.K / 64, 0};
  return launch_tile_gemm<ACT, P>(s, a, c.st, c.what, c.ws, c.ws_bytes);
}

int npamd::q_gemv_plan_stages(int M, int N, int K) {
  int staged = 0;
  GemvShape s{nullptr, K, nullptr, nullptr, N, M, N, K / 64, 0, 0};
  s.plan_only = &staged;
  using P = Q4Provider<NPAMD_F16, false>;  // int4 / int8, with or without zero points: one plan
  typename P::Args a{};
  launch_fused_gemv<NPAMD_F16, P>(s, a, nullptr, "plan");
  return staged;
}

template <int ACT, bool ASYM>
static int q8_fused(const QCall& c, bool gemv) {
  using P = Q8Provider<ACT, ASYM>;
  typename P::Args a{c.w_pack, (const uint16_t*)c.scale, c.K / 64, c.K / c.gs, log2i(c.gs / 32), (const uint16_t*)c.zp};
  if (gemv) {
    GemvShape s{c.x, c.ldx, c.bias, c.y, c.ldy, c.M, c.N, c.K / 64, 0, 0};
    return launch_fused_gemv<ACT, P>(s, a, c.st, c.what);
  }
  GemmShape s{c.x, c.ldx, c.bias, c.y, c.ldy, c.M, c.N, c.K, c.K / 64, 0};
  return launch_tile_gemm<ACT, P>(s, a, c.st, c.what, c.ws, c.ws_bytes);
}

// The 128-column tile GEMM (gemm_tile2.hpp) for int4 / int8: 0 when it took the call.
static int q_tile_wide(const QCall& c) {
  const int mode = tile2_mode();
  // Measured against the 64-column kernel, int4, us at 17 / 128 / 256 / 384 / 512 tokens: 14336 x 4096 26.7 / 32.7 /
  // 46.9 / 62.4 / 80.1 against 27.5 / 35.0 / 50.1 / 77.4 / 116; 6144 x 4096 17.9 / 26.2 / 33.9 / 49.0 / 45.4 against 20.3 /
  // 26.4 / 35.9 / 50.9 / 66.0; 4096 x 14336 30.8 / 40.3 / 54.0 / 69.5 / 83.9 against 29.8 / 38.9 / 59.9 / 82.0 / 121 (ahead
  // from 192 tokens: 47.4 against 51.0); 4096 x 4096 16.5 / 25.2 / 29.7 / 39.8 / 39.2 against 16.7 / 22.7 / 29.0 / 38.8 /
  // 50.6; 8192 x 2048 14.4 / 24.2 / 31.3 / 42.8 / 31.1 against 15.7 / 22.8 / 30.9 / 40.0 / 38.6.
  const int64_t weights = (int64_t)c.N * c.K;
  const bool wins = (c.N >= 6144 && c.K >= 4096) || (weights >= ((int64_t)1 << 25) && c.M > 128) || c.M > 384;
  if (!(mode >= 2 || (mode == 1 && wins))) return 1;
  if (!ptr_aligned(c.scale, 4) || (c.zp && !ptr_aligned(c.zp, 4)) || (int64_t)c.N * c.K >= ((int64_t)1 << 32)) return 1;
  const GemmShape s{c.x, c.ldx, c.bias, c.y, c.ldy, c.M, c.N, c.K, c.K / 64, 0};
  const T2QArgs q{c.w_pack, (const uint16_t*)c.scale, c.K / 64, c.K / c.gs, log2i(c.gs / 32), (const uint16_t*)c.zp};
  return launch_tile2_q(c.act, c.nbits, s, q, c.st, c.what, c.ws, c.ws_bytes);
}

template <int ACT>
static int q_dispatch(const QCall& c, bool gemv) {
  if (q_fast_ok(c)) {
    if (!gemv) {
      const int rc = q_tile_wide(c);
      if (rc != 1) return rc;
    }
    if (c.nbits == 8) return c.zp ? q8_fused<ACT, true>(c, gemv) : q8_fused<ACT, false>(c, gemv);
    if (gemv && q4_rowwise_ok(c)) {
      Q4StreamGeom geo;
      if (q4_stream_geometry(c, geo)) return launch_q4_stream<ACT>(c, geo);
      return launch_q4_rowwise<ACT, 1>(c);
    }
    return c.zp ? q4_fused<ACT, true>(c, gemv) : q4_fused<ACT, false>(c, gemv);
  }
  const QElem e{c.w_pack, (const uint16_t*)c.scale, (const uint16_t*)c.zp, c.K, c.nbits, c.gs, c.act};
  if (gemv) return launch_generic_gemv<ACT>(c.x, c.ldx, c.bias, c.y, c.ldy, c.M, c.N, c.K, e, c.st, c.what);
  return launch_generic_gemm<ACT>(c.x, c.ldx, c.bias, c.y, c.ldy, c.M, c.N, c.K, e, c.st, c.what);
}

static int q_run(const QCall& c, bool gemv) {
  const int rc = validate_q(c.what, c.N, c.K, c.nbits, c.gs);
  if (rc) return rc;
  NPAMD_REQUIRE(c.act == NPAMD_F16 || c.act == NPAMD_BF16,
                "%s: activations must be f16 or bf16 (got dtype code %d)", c.what, c.act);
  NPAMD_REQUIRE(c.M >= 0, "%s: negative M", c.what);
  NPAMD_REQUIRE(!gemv || c.M <= NPAMD_GEMV_MAX_M, "%s: M=%d exceeds the fused limit %d", c.what, c.M,
                NPAMD_GEMV_MAX_M);
  NPAMD_REQUIRE(c.ldx >= c.K && c.ldy >= c.N, "%s: row stride smaller than the row", c.what);
  if (c.M == 0 || c.N == 0) return NPAMD_OK;
  NPAMD_REQUIRE(c.x && c.y && (c.K == 0 || (c.w_pack && c.scale)), "%s: null pointer", c.what);
  return c.act == NPAMD_BF16 ? q_dispatch<NPAMD_BF16>(c, gemv) : q_dispatch<NPAMD_F16>(c, gemv);
}

}  // namespace npamd

using namespace npamd;

extern "C" int npamd_q_dequant(const uint8_t* w_pack, const void* scale_f16, const void* zero_point_f16,
                               int N, int K, int nbits, int group_size, void* out, int out_dtype,
                               void* stream) {
  const int rc = validate_q("npamd_q_dequant", N, K, nbits, group_size);
  if (rc) return rc;
  NPAMD_REQUIRE(out_dtype == NPAMD_F16 || out_dtype == NPAMD_BF16 || out_dtype == NPAMD_F32,
                "npamd_q_dequant: out_dtype must be f16, bf16 or f32");
  const int64_t total = (int64_t)N * K;
  if (total == 0) return NPAMD_OK;
  NPAMD_REQUIRE(w_pack && scale_f16 && out, "npamd_q_dequant: null pointer");
  hipStream_t st = (hipStream_t)stream;
  const bool fast = nbits == 4 && K % 8 == 0 && group_size % 8 == 0 &&
                    ptr_aligned(w_pack, 4) && ptr_aligned(out, 16);
  if (fast) {
    const int64_t n_words = total / 8;
    const unsigned blocks = (unsigned)((n_words + 255) / 256);
#define NPAMD_Q4_LAUNCH(OUT)                                                                              \
  do {                                                                                                    \
    if (zero_point_f16)                                                                                   \
      q4_dequant_kernel<OUT, true><<<blocks, 256, 0, st>>>(                                               \
          (const uint32_t*)w_pack, (const uint16_t*)scale_f16, (const uint16_t*)zero_point_f16, n_words,  \
          K / 8, K / group_size, group_size / 8, out);                                                    \
    else                                                                                                  \
      q4_dequant_kernel<OUT, false><<<blocks, 256, 0, st>>>(                                              \
          (const uint32_t*)w_pack, (const uint16_t*)scale_f16, nullptr, n_words, K / 8, K / group_size,   \
          group_size / 8, out);                                                                           \
  } while (0)
    if (out_dtype == NPAMD_F16) NPAMD_Q4_LAUNCH(NPAMD_F16);
    else if (out_dtype == NPAMD_BF16) NPAMD_Q4_LAUNCH(NPAMD_BF16);
    else NPAMD_Q4_LAUNCH(NPAMD_F32);
#undef NPAMD_Q4_LAUNCH
  } else if ((nbits == 8 || nbits == 2 || nbits == 1) && K % 8 == 0 && group_size % 8 == 0 &&
             ptr_aligned(w_pack, nbits) && ptr_aligned(out, 16)) {
    const int64_t n_octets = total / 8;
    const unsigned blocks = (unsigned)((n_octets + 255) / 256);
#define NPAMD_QN_LAUNCH(NB, OUT)                                                                       \
  qn_dequant_kernel<NB, OUT><<<blocks, 256, 0, st>>>(w_pack, (const uint16_t*)scale_f16,               \
                                                     (const uint16_t*)zero_point_f16, n_octets, K / 8, \
                                                     K / group_size, group_size / 8, out)
#define NPAMD_QN_OUT(NB)                                         \
  do {                                                           \
    if (out_dtype == NPAMD_F16) NPAMD_QN_LAUNCH(NB, NPAMD_F16);  \
    else if (out_dtype == NPAMD_BF16) NPAMD_QN_LAUNCH(NB, NPAMD_BF16); \
    else NPAMD_QN_LAUNCH(NB, NPAMD_F32);                         \
  } while (0)
    if (nbits == 8) NPAMD_QN_OUT(8);
    else if (nbits == 2) NPAMD_QN_OUT(2);
    else NPAMD_QN_OUT(1);
#undef NPAMD_QN_OUT
#undef NPAMD_QN_LAUNCH
  } else {
    const unsigned blocks = (unsigned)((total + 255) / 256);
#define NPAMD_QG_LAUNCH(OUT)                                                                   \
  q_dequant_generic_kernel<OUT><<<blocks, 256, 0, st>>>(w_pack, (const uint16_t*)scale_f16,    \
                                                        (const uint16_t*)zero_point_f16, total, \
                                                        K, nbits, group_size, out)
    if (out_dtype == NPAMD_F16) NPAMD_QG_LAUNCH(NPAMD_F16);
    else if (out_dtype == NPAMD_BF16) NPAMD_QG_LAUNCH(NPAMD_BF16);
    else NPAMD_QG_LAUNCH(NPAMD_F32);
#undef NPAMD_QG_LAUNCH
  }
  return check_launch("npamd_q_dequant");
}

extern "C" int npamd_q_fused_supported(int K, int nbits, int group_size) {
  return (nbits == 4 || nbits == 8) && group_size > 0 && group_size % 32 == 0 && is_pow2(group_size / 32) && K > 0 && K % 64 == 0 &&
                 K % group_size == 0
             ? 1
             : 0;
}

extern "C" int npamd_q_gemv(const void* x, int64_t ldx, const uint8_t* w_pack, const void* scale_f16,
                            const void* zero_point_f16, const float* bias, void* y, int64_t ldy,
                            int M, int N, int K, int nbits, int group_size, int act_dtype,
                            void* stream) {
  const QCall c{x, ldx, w_pack, scale_f16, zero_point_f16, bias, y, ldy, M, N, K, nbits, group_size,
                act_dtype, (hipStream_t)stream, "npamd_q_gemv"};
  return q_run(c, true);
}

extern "C" int npamd_q_gemm_tile(const void* x, int64_t ldx, const uint8_t* w_pack,
                                 const void* scale_f16, const void* zero_point_f16, const float* bias,
                                 void* y, int64_t ldy, int M, int N, int K, int nbits, int group_size,
                                 int act_dtype, void* workspace, int64_t workspace_bytes, void* stream) {
  QCall c{x, ldx, w_pack, scale_f16, zero_point_f16, bias, y, ldy, M, N, K, nbits, group_size,
          act_dtype, (hipStream_t)stream, "npamd_q_gemm_tile"};
  NPAMD_REQUIRE(workspace == nullptr || ptr_aligned(workspace, 16), "npamd_q_gemm_tile: workspace must be 16-byte aligned");
  c.ws = workspace;
  c.ws_bytes = workspace_bytes;
  return q_run(c, false);
}
