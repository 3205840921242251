// One-pass VQ decode kernels: packed index stream + fp16 codebook -> dense weight.
//
//   out.flat[v*VL + j] = cast(codebook[idx(v), j])
//
// HBM-bound byte work: one thread per vector, coalesced index reads (2 B/lane
// at 16 bits), one 16-byte codebook gather (L2-resident table), one vector
// store.  Traffic = index stream + output; the codebook is read from cache.
#include "common.hpp"

namespace npamd {

#pragma clang fp contract(off)

// Index of vector v.  BITS is 8 or 16 for the byte-aligned widths, 0 for the
// bounds-checked window reader.
template <int BITS>
__device__ __forceinline__ uint32_t vec_index(const uint8_t* __restrict__ packed, int64_t n_bytes,
                                              int64_t v, int bits) {
  if constexpr (BITS == 16) return reinterpret_cast<const uint16_t*>(packed)[v];
  else if constexpr (BITS == 8) return packed[v];
  else return read_index(packed, n_bytes, v, bits);
}

template <int OUT>
__device__ __forceinline__ void store8(void* out, int64_t v, u32x4 c) {
  if constexpr (OUT == NPAMD_F16) {
    reinterpret_cast<u32x4*>(out)[v] = c;
  } else if constexpr (OUT == NPAMD_BF16) {
    reinterpret_cast<u32x4*>(out)[v] = cb_to_act<NPAMD_BF16>(c);
  } else {
    f32x4 lo, hi;
    lo.x = f16_bits_to_f32(c.x & 0xFFFFu); lo.y = f16_bits_to_f32(c.x >> 16);
    lo.z = f16_bits_to_f32(c.y & 0xFFFFu); lo.w = f16_bits_to_f32(c.y >> 16);
    hi.x = f16_bits_to_f32(c.z & 0xFFFFu); hi.y = f16_bits_to_f32(c.z >> 16);
    hi.z = f16_bits_to_f32(c.w & 0xFFFFu); hi.w = f16_bits_to_f32(c.w >> 16);
    reinterpret_cast<f32x4*>(out)[2 * v] = lo;
    reinterpret_cast<f32x4*>(out)[2 * v + 1] = hi;
  }
}

// VL = 8: one 16-byte gather and one vector store per thread.
template <int BITS, int OUT>
__global__ void __launch_bounds__(256)
vq_dequant_vl8_kernel(const uint8_t* __restrict__ packed, int64_t n_bytes, int bits,
                      const u32x4* __restrict__ codebook, uint32_t nc, void* __restrict__ out,
                      int64_t n_vectors) {
  const int64_t v = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (v >= n_vectors) return;
  // An index past the codebook is clamped to the last row so a corrupt stream
  // cannot read outside the table.
  const uint32_t idx = min(vec_index<BITS>(packed, n_bytes, v, bits), nc - 1u);
  store8<OUT>(out, v, codebook[idx]);
}

// VL = 4: two vectors per thread -- two 8-byte gathers, one 16-byte (f32: 32-byte) store.
template <int OUT>
__device__ __forceinline__ void store4x2(void* out, int64_t v0, u32x2 c0, u32x2 c1, bool both) {
  if (both) {
    store8<OUT>(out, v0 >> 1, u32x4{c0.x, c0.y, c1.x, c1.y});  // v0 is even: 8 values = one store8 unit
  } else if constexpr (OUT == NPAMD_F16) {
    reinterpret_cast<u32x2*>(out)[v0] = c0;
  } else if constexpr (OUT == NPAMD_BF16) {
    reinterpret_cast<u32x2*>(out)[v0] = u32x2{f16x2_to_bf16x2(c0.x), f16x2_to_bf16x2(c0.y)};
  } else {
    reinterpret_cast<f32x4*>(out)[v0] = f32x4{f16_bits_to_f32(c0.x & 0xFFFFu), f16_bits_to_f32(c0.x >> 16),
                                              f16_bits_to_f32(c0.y & 0xFFFFu), f16_bits_to_f32(c0.y >> 16)};
  }
}

template <int BITS, int OUT>
__global__ void __launch_bounds__(256)
vq_dequant_vl4_kernel(const uint8_t* __restrict__ packed, int64_t n_bytes, int bits,
                      const u32x2* __restrict__ codebook, uint32_t nc, void* __restrict__ out,
                      int64_t n_vectors) {
  const int64_t v0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 2;
  if (v0 >= n_vectors) return;
  const bool both = v0 + 1 < n_vectors;
  const u32x2 c0 = codebook[min(vec_index<BITS>(packed, n_bytes, v0, bits), nc - 1u)];
  const u32x2 c1 = codebook[min(vec_index<BITS>(packed, n_bytes, both ? v0 + 1 : v0, bits), nc - 1u)];
  store4x2<OUT>(out, v0, c0, c1, both);
}

// VL = 8 or 4, a table of 16 to 64 KiB copied into LDS first.  Such a table overflows or fills
// the 32 KiB vector L1, so gathers from memory run at the L1-miss rate (36 us for a
// 14336 x 4096 layer with 4096 rows of 16 bytes, the same as a 65536-row table); from LDS the
// kernel is bound by the store stream.  Two blocks of 1024 threads per compute unit, each
// decoding a contiguous run of vectors.
template <int BITS, int OUT, int VL>
__global__ void __launch_bounds__(1024)
vq_dequant_lds_kernel(const uint8_t* __restrict__ packed, int64_t n_bytes, int bits,
                      const u32x4* __restrict__ codebook, uint32_t nc, void* __restrict__ out,
                      int64_t n_vectors, int64_t vectors_per_block) {
  extern __shared__ __attribute__((aligned(16))) u32x4 cb_lds[];
  const uint32_t vec16 = VL == 8 ? nc : (nc + 1) / 2;  // the allocation behind an odd VL = 4 table is not read past:
  for (uint32_t i = threadIdx.x; i < vec16; i += 1024) {  // its last half-filled unit is fetched as 8 bytes
    if (VL == 4 && (nc & 1) && i == vec16 - 1) {
      const u32x2 t = reinterpret_cast<const u32x2*>(codebook)[nc - 1];
      cb_lds[i] = u32x4{t.x, t.y, 0u, 0u};
    } else {
      cb_lds[i] = codebook[i];
    }
  }
  __syncthreads();
  const int64_t begin = (int64_t)blockIdx.x * vectors_per_block;
  const int64_t end = min(begin + vectors_per_block, n_vectors);
  if constexpr (VL == 8) {
    for (int64_t v = begin + threadIdx.x; v < end; v += 1024) {
      const uint32_t idx = min(vec_index<BITS>(packed, n_bytes, v, bits), nc - 1u);
      store8<OUT>(out, v, cb_lds[idx]);
    }
  } else {
    // two vectors per thread (a run starts at an even vector: vectors_per_block is a multiple of 1024)
    const u32x2* cb2 = reinterpret_cast<const u32x2*>(cb_lds);
    for (int64_t v0 = begin + 2 * threadIdx.x; v0 < end; v0 += 2048) {
      const bool both = v0 + 1 < end;
      const u32x2 c0 = cb2[min(vec_index<BITS>(packed, n_bytes, v0, bits), nc - 1u)];
      const u32x2 c1 = cb2[min(vec_index<BITS>(packed, n_bytes, both ? v0 + 1 : v0, bits), nc - 1u)];
      store4x2<OUT>(out, v0, c0, c1, both);
    }
  }
}

// Any VL: scalar copy of the codebook row.
template <int OUT>
__global__ void __launch_bounds__(256)
vq_dequant_generic_kernel(const uint8_t* __restrict__ packed, int64_t n_bytes, int bits,
                          const uint16_t* __restrict__ codebook, uint32_t nc,
                          void* __restrict__ out, int64_t n_vectors, int vl) {
  const int64_t v = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (v >= n_vectors) return;
  const uint32_t idx = min(read_index(packed, n_bytes, v, bits), nc - 1u);
  const uint16_t* c = codebook + (int64_t)idx * vl;
  for (int j = 0; j < vl; ++j) store_from_f16_bits<OUT>(out, v * vl + j, c[j]);
}

__global__ void __launch_bounds__(256)
vq_widen_u16_kernel(const uint8_t* __restrict__ packed, int64_t n_bytes, int bits,
                    int64_t n_indices, uint16_t* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n_indices) return;
  out[i] = (uint16_t)read_index(packed, n_bytes, i, bits);
}

// Residual VQ: three separately rounded fp16 operations per element.
__device__ __forceinline__ uint32_t rvq_elem(uint32_t cm, uint32_t cr, bool has_s, _Float16 s,
                                             bool has_b, _Float16 b) {
  _Float16 h = __builtin_bit_cast(_Float16, (uint16_t)cm) + __builtin_bit_cast(_Float16, (uint16_t)cr);
  if (has_s) h = h * s;
  if (has_b) h = h + b;
  return (uint32_t)__builtin_bit_cast(uint16_t, h);
}

template <int OUT>
__global__ void __launch_bounds__(256)
rvq_dequant_kernel(const uint8_t* __restrict__ pm, int64_t nbm, int bits_m,
                   const uint8_t* __restrict__ pr, int64_t nbr, int bits_r,
                   const uint16_t* __restrict__ cbm, uint32_t ncm,
                   const uint16_t* __restrict__ cbr, uint32_t ncr,
                   const uint16_t* __restrict__ row_scale, const uint16_t* __restrict__ row_bias,
                   int vl, int64_t groups, int64_t n_vectors, void* __restrict__ out) {
  const int64_t v = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (v >= n_vectors) return;
  const uint32_t im = min(read_index(pm, nbm, v, bits_m), ncm - 1u);
  const uint32_t ir = min(read_index(pr, nbr, v, bits_r), ncr - 1u);
  const int64_t n = v / groups;
  const bool has_s = row_scale != nullptr, has_b = row_bias != nullptr;
  const _Float16 s = has_s ? __builtin_bit_cast(_Float16, row_scale[n]) : (_Float16)1.0f;
  const _Float16 b = has_b ? __builtin_bit_cast(_Float16, row_bias[n]) : (_Float16)0.0f;
  const uint16_t* cm = cbm + (int64_t)im * vl;
  const uint16_t* cr = cbr + (int64_t)ir * vl;
  for (int j = 0; j < vl; ++j)
    store_from_f16_bits<OUT>(out, v * vl + j, rvq_elem(cm[j], cr[j], has_s, s, has_b, b));
}

// VL = 8: two 16-byte gathers, packed fp16 arithmetic (each operation rounds per element, like
// the scalar form), one vector store.  Grid = (row, 256 groups of the row): no division.
template <int BITS_M, int BITS_R, int OUT>
__global__ void __launch_bounds__(256)
rvq_dequant_vl8_kernel(const uint8_t* __restrict__ pm, int64_t nbm, int bits_m,
                       const uint8_t* __restrict__ pr, int64_t nbr, int bits_r,
                       const u32x4* __restrict__ cbm, uint32_t ncm, const u32x4* __restrict__ cbr, uint32_t ncr,
                       const uint16_t* __restrict__ row_scale, const uint16_t* __restrict__ row_bias,
                       int groups, void* __restrict__ out) {
  const int n = blockIdx.x;
  const int g = blockIdx.y * 256 + threadIdx.x;
  if (g >= groups) return;
  const int64_t v = (int64_t)n * groups + g;
  const uint32_t im = min(vec_index<BITS_M>(pm, nbm, v, bits_m), ncm - 1u);
  const uint32_t ir = min(vec_index<BITS_R>(pr, nbr, v, bits_r), ncr - 1u);
  const u32x4 a = cbm[im], r = cbr[ir];
  const bool has_s = row_scale != nullptr, has_b = row_bias != nullptr;
  const uint32_t s2 = has_s ? (uint32_t)row_scale[n] * 0x10001u : 0u;
  const uint32_t b2 = has_b ? (uint32_t)row_bias[n] * 0x10001u : 0u;
  const uint32_t am[4] = {a.x, a.y, a.z, a.w}, rr[4] = {r.x, r.y, r.z, r.w};
  uint32_t o[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f16x2 h = __builtin_bit_cast(f16x2, am[i]) + __builtin_bit_cast(f16x2, rr[i]);
    if (has_s) h = h * __builtin_bit_cast(f16x2, s2);
    if (has_b) h = h + __builtin_bit_cast(f16x2, b2);
    o[i] = __builtin_bit_cast(uint32_t, h);
  }
  store8<OUT>(out, v, u32x4{o[0], o[1], o[2], o[3]});
}

template <int OUT>
static int launch_vq_dequant(const uint8_t* packed, int64_t n_bytes, int bits, const void* cb,
                             uint32_t nc, int vl, int64_t n_vectors, void* out, hipStream_t st) {
  const unsigned blocks = (unsigned)((n_vectors + 255) / 256);
  const bool cb_aligned = (reinterpret_cast<uintptr_t>(cb) % 16) == 0;
  const bool out_aligned = (reinterpret_cast<uintptr_t>(out) % 16) == 0;
  // Tables of 16 to 64 KiB on layers large enough to pay for one copy per block.
  const int64_t table_bytes = (int64_t)nc * vl * 2;
  if ((vl == 8 || vl == 4) && cb_aligned && out_aligned && table_bytes > 16 * 1024 && table_bytes <= 64 * 1024 &&
      n_vectors >= (1 << 20)) {
    const u32x4* c = reinterpret_cast<const u32x4*>(cb);
    const int lds = (int)((table_bytes + 15) / 16 * 16);
    const int64_t per_block = ((n_vectors + 511) / 512 + 1023) / 1024 * 1024;
    const unsigned grid = (unsigned)((n_vectors + per_block - 1) / per_block);
    const bool b16 = bits == 16 && (reinterpret_cast<uintptr_t>(packed) % 2) == 0;
#define NPAMD_VQ_LDS(B, V) \
  vq_dequant_lds_kernel<B, OUT, V><<<grid, 1024, lds, st>>>(packed, n_bytes, bits, c, nc, out, n_vectors, per_block)
    if (vl == 8) {
      if (b16) NPAMD_VQ_LDS(16, 8);
      else NPAMD_VQ_LDS(0, 8);
    } else {
      if (b16) NPAMD_VQ_LDS(16, 4);
      else NPAMD_VQ_LDS(0, 4);
    }
#undef NPAMD_VQ_LDS
    return check_launch("npamd_vq_dequant");
  }
  if (vl == 8 && cb_aligned && out_aligned) {
    const u32x4* c = reinterpret_cast<const u32x4*>(cb);
    if (bits == 16 && (reinterpret_cast<uintptr_t>(packed) % 2) == 0)
      vq_dequant_vl8_kernel<16, OUT><<<blocks, 256, 0, st>>>(packed, n_bytes, bits, c, nc, out, n_vectors);
    else if (bits == 8)
      vq_dequant_vl8_kernel<8, OUT><<<blocks, 256, 0, st>>>(packed, n_bytes, bits, c, nc, out, n_vectors);
    else
      vq_dequant_vl8_kernel<0, OUT><<<blocks, 256, 0, st>>>(packed, n_bytes, bits, c, nc, out, n_vectors);
  } else if (vl == 4 && (reinterpret_cast<uintptr_t>(cb) % 8) == 0 && out_aligned) {
    const u32x2* c = reinterpret_cast<const u32x2*>(cb);
    const unsigned blocks = (unsigned)(((n_vectors + 1) / 2 + 255) / 256);  // two vectors per thread
    if (bits == 16 && (reinterpret_cast<uintptr_t>(packed) % 2) == 0)
      vq_dequant_vl4_kernel<16, OUT><<<blocks, 256, 0, st>>>(packed, n_bytes, bits, c, nc, out, n_vectors);
    else if (bits == 8)
      vq_dequant_vl4_kernel<8, OUT><<<blocks, 256, 0, st>>>(packed, n_bytes, bits, c, nc, out, n_vectors);
    else
      vq_dequant_vl4_kernel<0, OUT><<<blocks, 256, 0, st>>>(packed, n_bytes, bits, c, nc, out, n_vectors);
  } else {
    vq_dequant_generic_kernel<OUT><<<blocks, 256, 0, st>>>(
        packed, n_bytes, bits, reinterpret_cast<const uint16_t*>(cb), nc, out, n_vectors, vl);
  }
  return check_launch("npamd_vq_dequant");
}

// LUT gather: y[m, j] = sum over groups g of lut[m, g, idx(j, g)], float32.
// One wave per output row j: lane l takes groups l, l + 64, ... (consecutive indices of the
// stream), the 64 partial sums are added pairwise across the wave in a fixed order.
// blockIdx.y = token.
__global__ void __launch_bounds__(256) vq_lut_gather_kernel(const float* __restrict__ lut,
                                                             const uint8_t* __restrict__ packed, int64_t n_bytes,
                                                             int bits, float* __restrict__ y, int N, int groups,
                                                             int nc) {
  const int lane = threadIdx.x & 63;
  const int j = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (j >= N) return;
  const float* lut_m = lut + (int64_t)blockIdx.y * groups * nc;
  float acc = 0.f;
  for (int g = lane; g < groups; g += 64) {
    uint32_t c = read_index(packed, n_bytes, (int64_t)j * groups + g, bits);
    if (c > (uint32_t)nc - 1u) c = (uint32_t)nc - 1u;  // same clamp as the decode kernels
    acc += lut_m[(int64_t)g * nc + c];
  }
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) acc += __shfl_xor(acc, o, 64);
  if (lane == 0) y[(int64_t)blockIdx.y * N + j] = acc;
}

}  // namespace npamd

using namespace npamd;

extern "C" int npamd_vq_dequant(const uint8_t* packed, int64_t n_bytes, int bits,
                                const void* codebook_f16, int nc, int vl, int64_t n_vectors,
                                void* out, int out_dtype, void* stream) {
  NPAMD_REQUIRE(bits >= 4 && bits <= 20, "npamd_vq_dequant: bits must be in [4, 20], got %d", bits);
  NPAMD_REQUIRE(vl >= 1 && nc >= 1, "npamd_vq_dequant: bad codebook shape [%d, %d]", nc, vl);
  NPAMD_REQUIRE(n_vectors >= 0, "npamd_vq_dequant: negative n_vectors");
  NPAMD_REQUIRE((n_vectors * bits + 7) / 8 <= n_bytes,
                "npamd_vq_dequant: packed buffer too short for %lld indices of %d bits",
                (long long)n_vectors, bits);
  if (n_vectors == 0) return NPAMD_OK;
  NPAMD_REQUIRE(packed && codebook_f16 && out, "npamd_vq_dequant: null pointer");
  NPAMD_REQUIRE(n_vectors <= (int64_t)0x7FFFFFFF * 256, "npamd_vq_dequant: too many vectors");
  hipStream_t st = (hipStream_t)stream;
  switch (out_dtype) {
    case NPAMD_F16: return launch_vq_dequant<NPAMD_F16>(packed, n_bytes, bits, codebook_f16, (uint32_t)nc, vl, n_vectors, out, st);
    case NPAMD_BF16: return launch_vq_dequant<NPAMD_BF16>(packed, n_bytes, bits, codebook_f16, (uint32_t)nc, vl, n_vectors, out, st);
    case NPAMD_F32: return launch_vq_dequant<NPAMD_F32>(packed, n_bytes, bits, codebook_f16, (uint32_t)nc, vl, n_vectors, out, st);
  }
  return fail(NPAMD_ERR_INVALID, "npamd_vq_dequant: out_dtype must be f16, bf16 or f32");
}

extern "C" int npamd_vq_widen_u16(const uint8_t* packed, int64_t n_bytes, int bits,
                                  int64_t n_indices, uint16_t* out, void* stream) {
  NPAMD_REQUIRE(bits >= 4 && bits <= 16, "npamd_vq_widen_u16: bits must be in [4, 16], got %d", bits);
  NPAMD_REQUIRE(n_indices >= 0 && (n_indices * bits + 7) / 8 <= n_bytes,
                "npamd_vq_widen_u16: packed buffer too short");
  if (n_indices == 0) return NPAMD_OK;
  NPAMD_REQUIRE(packed && out, "npamd_vq_widen_u16: null pointer");
  const unsigned blocks = (unsigned)((n_indices + 255) / 256);
  vq_widen_u16_kernel<<<blocks, 256, 0, (hipStream_t)stream>>>(packed, n_bytes, bits, n_indices, out);
  return check_launch("npamd_vq_widen_u16");
}

extern "C" int npamd_vq_lut_gather(const float* lut, const uint8_t* packed, int64_t n_bytes, int bits,
                                   float* y, int M, int N, int groups, int nc, void* stream) {
  const char* what = "npamd_vq_lut_gather";
  NPAMD_REQUIRE(bits >= 4 && bits <= 20, "%s: bits must be in [4, 20], got %d", what, bits);
  NPAMD_REQUIRE(M >= 0 && N >= 0 && groups >= 1 && nc >= 1, "%s: bad shape M=%d N=%d groups=%d NC=%d", what, M, N,
                groups, nc);
  NPAMD_REQUIRE(((int64_t)N * groups * bits + 7) / 8 <= n_bytes, "%s: packed buffer too short", what);
  NPAMD_REQUIRE(M <= 65535, "%s: at most 65535 tokens per call (got %d)", what, M);
  if (M == 0 || N == 0) return NPAMD_OK;
  NPAMD_REQUIRE(lut && packed && y, "%s: null pointer", what);
  const dim3 grid((unsigned)((N + 3) / 4), (unsigned)M);
  vq_lut_gather_kernel<<<grid, 256, 0, (hipStream_t)stream>>>(lut, packed, n_bytes, bits, y, N, groups, nc);
  return check_launch(what);
}

extern "C" int npamd_rvq_dequant(const uint8_t* packed_main, int64_t n_bytes_main, int bits_main,
                                 const uint8_t* packed_res, int64_t n_bytes_res, int bits_res,
                                 const void* cb_main_f16, int nc_main, const void* cb_res_f16,
                                 int nc_res, const void* row_scale_f16, const void* row_bias_f16,
                                 int vl, int N, int K, void* out, int out_dtype, void* stream) {
  NPAMD_REQUIRE(bits_main >= 4 && bits_main <= 20 && bits_res >= 4 && bits_res <= 20,
                "npamd_rvq_dequant: bits must be in [4, 20]");
  NPAMD_REQUIRE(vl >= 1 && nc_main >= 1 && nc_res >= 1, "npamd_rvq_dequant: bad codebook shape");
  NPAMD_REQUIRE(N >= 0 && K >= 0 && K % vl == 0, "npamd_rvq_dequant: K=%d not divisible by VL=%d", K, vl);
  const int64_t groups = K / vl, n_vectors = (int64_t)N * groups;
  NPAMD_REQUIRE((n_vectors * bits_main + 7) / 8 <= n_bytes_main &&
                    (n_vectors * bits_res + 7) / 8 <= n_bytes_res,
                "npamd_rvq_dequant: packed buffer too short");
  if (n_vectors == 0) return NPAMD_OK;
  NPAMD_REQUIRE(packed_main && packed_res && cb_main_f16 && cb_res_f16 && out,
                "npamd_rvq_dequant: null pointer");
  const unsigned blocks = (unsigned)((n_vectors + 255) / 256);
  hipStream_t st = (hipStream_t)stream;
  const bool aligned16 = ((reinterpret_cast<uintptr_t>(cb_main_f16) | reinterpret_cast<uintptr_t>(cb_res_f16) |
                           reinterpret_cast<uintptr_t>(out)) % 16) == 0;
  if (vl == 8 && aligned16 && (groups + 255) / 256 <= 65535) {
    const dim3 grid((unsigned)N, (unsigned)((groups + 255) / 256));
    const bool m16 = bits_main == 16 && (reinterpret_cast<uintptr_t>(packed_main) % 2) == 0;
    const bool r8 = bits_res == 8;
#define NPAMD_RVQ8_LAUNCH(BM, BR, OUT)                                                               \
  rvq_dequant_vl8_kernel<BM, BR, OUT><<<grid, 256, 0, st>>>(                                         \
      packed_main, n_bytes_main, bits_main, packed_res, n_bytes_res, bits_res, (const u32x4*)cb_main_f16, \
      (uint32_t)nc_main, (const u32x4*)cb_res_f16, (uint32_t)nc_res, (const uint16_t*)row_scale_f16,  \
      (const uint16_t*)row_bias_f16, (int)groups, out)
#define NPAMD_RVQ8_BITS(OUT)                                \
  do {                                                      \
    if (m16 && r8) NPAMD_RVQ8_LAUNCH(16, 8, OUT);           \
    else if (m16) NPAMD_RVQ8_LAUNCH(16, 0, OUT);            \
    else NPAMD_RVQ8_LAUNCH(0, 0, OUT);                      \
  } while (0)
    switch (out_dtype) {
      case NPAMD_F16: NPAMD_RVQ8_BITS(NPAMD_F16); break;
      case NPAMD_BF16: NPAMD_RVQ8_BITS(NPAMD_BF16); break;
      case NPAMD_F32: NPAMD_RVQ8_BITS(NPAMD_F32); break;
      default: return fail(NPAMD_ERR_INVALID, "npamd_rvq_dequant: out_dtype must be f16, bf16 or f32");
    }
#undef NPAMD_RVQ8_BITS
#undef NPAMD_RVQ8_LAUNCH
    return check_launch("npamd_rvq_dequant");
  }
#define NPAMD_RVQ_LAUNCH(OUT)                                                                   \
  rvq_dequant_kernel<OUT><<<blocks, 256, 0, st>>>(                                              \
      packed_main, n_bytes_main, bits_main, packed_res, n_bytes_res, bits_res,                  \
      (const uint16_t*)cb_main_f16, (uint32_t)nc_main, (const uint16_t*)cb_res_f16,             \
      (uint32_t)nc_res, (const uint16_t*)row_scale_f16, \
      (const uint16_t*)row_bias_f16, vl, groups, n_vectors, out)
  switch (out_dtype) {
    case NPAMD_F16: NPAMD_RVQ_LAUNCH(NPAMD_F16); break;
    case NPAMD_BF16: NPAMD_RVQ_LAUNCH(NPAMD_BF16); break;
    case NPAMD_F32: NPAMD_RVQ_LAUNCH(NPAMD_F32); break;
    default: return fail(NPAMD_ERR_INVALID, "npamd_rvq_dequant: out_dtype must be f16, bf16 or f32");
  }
#undef NPAMD_RVQ_LAUNCH
  return check_launch("npamd_rvq_dequant");
}
