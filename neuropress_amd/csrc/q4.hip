// Group-affine n-bit weights (Q4_0 / GPTQ style): decode, fused GEMV, fused GEMM.
//
//   q = (w_pack[n, k/vpb] >> ((k%vpb)*nbits)) & mask ;  w = (float(q) - zp) * float(scale)
//
// Fast kernels cover the layout the BASELINE config uses (4 bits, symmetric,
// group size a power-of-two multiple of 32, K % 64 == 0); every other valid
// combination (1/2/8 bits, zero points, odd K) runs the element-wise fallback.
#include "gemm_tile.hpp"
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

// Decode, 4-bit symmetric: one thread per dword of nibbles = 8 weights, one
// 16-byte (32-byte for f32) store.  group_size % 8 == 0 so the 8 share a scale.
template <int OUT>
__global__ void __launch_bounds__(256)
q4_dequant_kernel(const uint32_t* __restrict__ w_pack, const uint16_t* __restrict__ scale,
                  int64_t n_words, int words_per_row, int groups_per_row, int words_per_group,
                  void* __restrict__ out) {
#pragma clang fp contract(off)
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n_words) return;
  const int64_t n = i / words_per_row;
  const int wr = (int)(i - n * words_per_row);
  const float sc = f16_bits_to_f32(scale[n * groups_per_row + wr / words_per_group]);
  const uint32_t w = w_pack[i];
  float v[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) v[j] = ((float)((w >> (4 * j)) & 0xFu) - 8.0f) * sc;
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

struct QCall {
  const void* x; int64_t ldx;
  const uint8_t* w_pack; const void* scale; const void* zp;
  const float* bias; void* y; int64_t ldy;
  int M, N, K, nbits, gs, act;
  hipStream_t st;
  const char* what;
};

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
  return c.nbits == 4 && c.zp == nullptr && c.gs % 32 == 0 && is_pow2(c.gs / 32) && c.K % 64 == 0 &&
         c.K > 0 && c.ldx % 8 == 0 && ptr_aligned(c.x, 16) && ptr_aligned(c.w_pack, 16);
}

static int log2i(int v) { int s = 0; while ((1 << s) < v) ++s; return s; }

template <int ACT>
static int q_dispatch(const QCall& c, bool gemv) {
  if (q_fast_ok(c)) {
    using P = Q4Provider<ACT>;
    typename P::Args a{c.w_pack, (const uint16_t*)c.scale, c.K / 64, c.K / c.gs, log2i(c.gs / 32)};
    if (gemv) {
      GemvShape s{c.x, c.ldx, c.bias, c.y, c.ldy, c.M, c.N, c.K / 64, 0, 0};
      return launch_fused_gemv<ACT, P>(s, a, c.st, c.what);
    }
    GemmShape s{c.x, c.ldx, c.bias, c.y, c.ldy, c.M, c.N, c.K, c.K / 64, 0};
    return launch_tile_gemm<ACT, P>(s, a, c.st, c.what);
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
  const bool fast = nbits == 4 && !zero_point_f16 && K % 8 == 0 && group_size % 8 == 0 &&
                    ptr_aligned(w_pack, 4) && ptr_aligned(out, 16);
  if (fast) {
    const int64_t n_words = total / 8;
    const unsigned blocks = (unsigned)((n_words + 255) / 256);
#define NPAMD_Q4_LAUNCH(OUT)                                                                 \
  q4_dequant_kernel<OUT><<<blocks, 256, 0, st>>>((const uint32_t*)w_pack,                    \
                                                 (const uint16_t*)scale_f16, n_words, K / 8, \
                                                 K / group_size, group_size / 8, out)
    if (out_dtype == NPAMD_F16) NPAMD_Q4_LAUNCH(NPAMD_F16);
    else if (out_dtype == NPAMD_BF16) NPAMD_Q4_LAUNCH(NPAMD_BF16);
    else NPAMD_Q4_LAUNCH(NPAMD_F32);
#undef NPAMD_Q4_LAUNCH
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
                                 int act_dtype, void* stream) {
  const QCall c{x, ldx, w_pack, scale_f16, zero_point_f16, bias, y, ldy, M, N, K, nbits, group_size,
                act_dtype, (hipStream_t)stream, "npamd_q_gemm_tile"};
  return q_run(c, false);
}
