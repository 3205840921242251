// Neighbours of the quantized linear on the decode step: fused RMSNorm and the
// embedding lookups of VQ- and int-quantized tables.  All three are bound by
// HBM traffic (or, at one token, by the launch); none of them has matrix work.
#include "common.hpp"

using namespace npamd;

namespace {

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

template <int DT>
__device__ __forceinline__ void unpack8(const u32x4& v, float (&f)[8]) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f[2 * i] = act_bits_to_f32<DT>(v[i] & 0xFFFFu);
    f[2 * i + 1] = act_bits_to_f32<DT>(v[i] >> 16);
  }
}

template <int DT>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  if constexpr (DT == NPAMD_BF16) return f32_to_bf16_bits(lo) | (f32_to_bf16_bits(hi) << 16);
  else return f32_to_f16_bits(lo) | (f32_to_f16_bits(hi) << 16);
}

// ---------------------------------------------------------------------------
// RMSNorm: out[m, i] = round(x[m, i] * rsqrt(mean_i(x[m, i]^2) + eps) * w[i]),
// all arithmetic in f32, one rounding at the store.
//
// One wave per row; the row stays in registers between the sum of squares and
// the scaling (NV 16-byte vectors per lane), so x is read from memory once and
// the only cross-lane traffic is the wave reduction.  Four rows per block.
// ---------------------------------------------------------------------------
template <int DT, int NV>
__global__ void __launch_bounds__(256)
rms_norm_wave_kernel(const uint16_t* __restrict__ x, int64_t ldx, const uint16_t* __restrict__ w,
                     uint16_t* __restrict__ out, int64_t ldo, int M, int H, float eps) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= M) return;
  const int n_vec = H >> 3;
  const uint16_t* xr = x + (int64_t)row * ldx;
  u32x4 v[NV], wv[NV];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int p = lane + 64 * i;
    v[i] = p < n_vec ? *reinterpret_cast<const u32x4*>(xr + 8 * p) : u32x4{0, 0, 0, 0};
  }
  // the weight does not depend on the reduction: requested now, it arrives while the sum is formed
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int p = lane + 64 * i;
    wv[i] = p < n_vec ? *reinterpret_cast<const u32x4*>(w + 8 * p) : u32x4{0, 0, 0, 0};
  }
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    float f[8];
    unpack8<DT>(v[i], f);
#pragma unroll
    for (int e = 0; e < 8; ++e) ss = __builtin_fmaf(f[e], f[e], ss);
  }
  ss = wave_reduce_sum(ss);
  const float scale = 1.0f / __builtin_sqrtf(ss / (float)H + eps);
  uint16_t* orow = out + (int64_t)row * ldo;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int p = lane + 64 * i;
    if (p >= n_vec) continue;
    float f[8], g[8];
    unpack8<DT>(v[i], f);
    unpack8<DT>(wv[i], g);
    u32x4 o;
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = pack2<DT>(f[2 * e] * scale * g[2 * e], f[2 * e + 1] * scale * g[2 * e + 1]);
    *reinterpret_cast<u32x4*>(orow + 8 * p) = o;
  }
}

// Any H, any alignment: one block per row, x read twice.
template <int DT>
__global__ void __launch_bounds__(256)
rms_norm_block_kernel(const void* __restrict__ x, int64_t ldx, const void* __restrict__ w,
                      void* __restrict__ out, int64_t ldo, int H, float eps) {
  __shared__ float part[4];
  const int64_t row = blockIdx.x;
  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += 256) {
    const float f = load_as_f32<DT>(x, row * ldx + i);
    ss = __builtin_fmaf(f, f, ss);
  }
  ss = wave_reduce_sum(ss);
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = ss;
  __syncthreads();
  const float scale = 1.0f / __builtin_sqrtf((part[0] + part[1] + part[2] + part[3]) / (float)H + eps);
  for (int i = threadIdx.x; i < H; i += 256)
    store_from_f32<DT>(out, row * ldo + i, load_as_f32<DT>(x, row * ldx + i) * scale * load_as_f32<DT>(w, i));
}

template <int DT>
int launch_rms_norm(const void* x, int64_t ldx, const void* w, void* out, int64_t ldo, int M, int H, float eps,
                    hipStream_t st) {
  const bool vec = DT != NPAMD_F32 && H % 8 == 0 && ldx % 8 == 0 && ldo % 8 == 0 && aligned16(x) && aligned16(w) &&
                   aligned16(out) && H <= 8 * 64 * 16;
  if constexpr (DT != NPAMD_F32) {
    if (vec) {
      const int nv = (H / 8 + 63) / 64;
      const dim3 grid((M + 3) / 4);
      auto xs = (const uint16_t*)x;
      auto ws = (const uint16_t*)w;
      auto os = (uint16_t*)out;
      if (nv <= 1) rms_norm_wave_kernel<DT, 1><<<grid, 256, 0, st>>>(xs, ldx, ws, os, ldo, M, H, eps);
      else if (nv <= 2) rms_norm_wave_kernel<DT, 2><<<grid, 256, 0, st>>>(xs, ldx, ws, os, ldo, M, H, eps);
      else if (nv <= 4) rms_norm_wave_kernel<DT, 4><<<grid, 256, 0, st>>>(xs, ldx, ws, os, ldo, M, H, eps);
      else if (nv <= 8) rms_norm_wave_kernel<DT, 8><<<grid, 256, 0, st>>>(xs, ldx, ws, os, ldo, M, H, eps);
      else rms_norm_wave_kernel<DT, 16><<<grid, 256, 0, st>>>(xs, ldx, ws, os, ldo, M, H, eps);
      return check_launch("npamd_rms_norm");
    }
  }
  rms_norm_block_kernel<DT><<<M, 256, 0, st>>>(x, ldx, w, out, ldo, H, eps);
  return check_launch("npamd_rms_norm");
}

// ---------------------------------------------------------------------------
// VQ embedding lookup:
//   row[t, g*VL + v] = C[idx[ids[t], g], v]                       (fp16)
//   out[t, j] = cast(f16(row[t, inv_perm[j]] * scale))            (scale applied when != 1)
// idx is the pre-unpacked [vocab, groups] table of 16-bit indices.
// ---------------------------------------------------------------------------
template <int OUT>
__device__ __forceinline__ void store_embedding8(void* out, int64_t at, const uint32_t (&h)[8], float scale,
                                                  bool scaled) {
  uint32_t r[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) r[e] = scaled ? f32_to_f16_bits(f16_bits_to_f32(h[e]) * scale) : h[e];
  if constexpr (OUT == NPAMD_F16) {
    *reinterpret_cast<u32x4*>((uint16_t*)out + at) =
        u32x4{r[0] | (r[1] << 16), r[2] | (r[3] << 16), r[4] | (r[5] << 16), r[6] | (r[7] << 16)};
  } else if constexpr (OUT == NPAMD_BF16) {
    uint32_t b[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) b[e] = f32_to_bf16_bits(f16_bits_to_f32(r[e]));
    *reinterpret_cast<u32x4*>((uint16_t*)out + at) =
        u32x4{b[0] | (b[1] << 16), b[2] | (b[3] << 16), b[4] | (b[5] << 16), b[6] | (b[7] << 16)};
  } else {
    float* o = (float*)out + at;
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = f16_bits_to_f32(r[e]);
  }
}

// VL = 8, D % 8 == 0: one thread per eight output elements.
template <int OUT, bool PERM>
__global__ void __launch_bounds__(256)
vq_embedding_vl8_kernel(const int64_t* __restrict__ ids, int64_t n_ids, const uint16_t* __restrict__ idx,
                        int64_t vocab, int groups, const uint16_t* __restrict__ cb, uint32_t nc_minus_1,
                        const int32_t* __restrict__ inv_perm, float scale, bool scaled, void* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n_ids * groups) return;
  const int64_t t = i / groups;
  const int g8 = (int)(i - t * groups);
  int64_t tok = ids[t];
  tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);  // ids are clamped, never followed out of the table
  const uint16_t* trow = idx + tok * groups;
  uint32_t h[8];
  if constexpr (PERM) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int src = inv_perm[g8 * 8 + e];
      const uint32_t c = min((uint32_t)trow[src >> 3], nc_minus_1);
      h[e] = cb[(int64_t)c * 8 + (src & 7)];
    }
  } else {
    const uint32_t c = min((uint32_t)trow[g8], nc_minus_1);
    const u32x4 v = *reinterpret_cast<const u32x4*>(cb + (int64_t)c * 8);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      h[2 * e] = v[e] & 0xFFFFu;
      h[2 * e + 1] = v[e] >> 16;
    }
  }
  store_embedding8<OUT>(out, i * 8, h, scale, scaled);
}

// Any vector length: one thread per output element.
template <int OUT>
__global__ void __launch_bounds__(256)
vq_embedding_generic_kernel(const int64_t* __restrict__ ids, int64_t n_ids, const uint16_t* __restrict__ idx,
                            int64_t vocab, int groups, int vl, const uint16_t* __restrict__ cb, uint32_t nc_minus_1,
                            const int32_t* __restrict__ inv_perm, float scale, bool scaled, void* __restrict__ out) {
  const int dim = groups * vl;
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n_ids * dim) return;
  const int64_t t = i / dim;
  const int j = (int)(i - t * dim);
  int64_t tok = ids[t];
  tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
  const int src = inv_perm ? inv_perm[j] : j;
  const uint32_t c = min((uint32_t)idx[tok * groups + src / vl], nc_minus_1);
  uint32_t h = cb[(int64_t)c * vl + src % vl];
  if (scaled) h = f32_to_f16_bits(f16_bits_to_f32(h) * scale);
  store_from_f16_bits<OUT>(out, i, h);
}

template <int OUT>
int launch_vq_embedding(const int64_t* ids, int64_t n_ids, const uint16_t* idx, int64_t vocab, int groups,
                        const uint16_t* cb, int nc, int vl, const int32_t* inv_perm, float scale, void* out,
                        hipStream_t st) {
  const bool scaled = scale != 1.0f;
  if (vl == 8 && aligned16(cb) && aligned16(out)) {
    const int64_t n = n_ids * groups;
    const unsigned blocks = (unsigned)((n + 255) / 256);
    if (inv_perm)
      vq_embedding_vl8_kernel<OUT, true><<<blocks, 256, 0, st>>>(ids, n_ids, idx, vocab, groups, cb, (uint32_t)nc - 1u,
                                                                 inv_perm, scale, scaled, out);
    else
      vq_embedding_vl8_kernel<OUT, false><<<blocks, 256, 0, st>>>(ids, n_ids, idx, vocab, groups, cb,
                                                                  (uint32_t)nc - 1u, nullptr, scale, scaled, out);
  } else {
    const int64_t n = n_ids * groups * vl;
    vq_embedding_generic_kernel<OUT><<<(unsigned)((n + 255) / 256), 256, 0, st>>>(
        ids, n_ids, idx, vocab, groups, vl, cb, (uint32_t)nc - 1u, inv_perm, scale, scaled, out);
  }
  return check_launch("npamd_vq_embedding");
}

// ---------------------------------------------------------------------------
// Group-affine n-bit embedding lookup (n in {1, 2, 4, 8}):
//   v16 = f16((q - zp) * s)          f32 arithmetic, zp = 2^(n-1) without a zero-point tensor
//   v16 = 0 on the padding row
//   out = round_out(cast_out(v16) * embed_scale)   (the multiply only when embed_scale != 1)
// ---------------------------------------------------------------------------
template <int OUT>
__device__ __forceinline__ void store_q_embedding(void* out, int64_t at, float v, float embed_scale, bool scaled) {
  const uint32_t h = f32_to_f16_bits(v);
  if (!scaled) {
    store_from_f16_bits<OUT>(out, at, h);
    return;
  }
  if constexpr (OUT == NPAMD_F16) store_from_f32<OUT>(out, at, f16_bits_to_f32(h) * embed_scale);
  else if constexpr (OUT == NPAMD_BF16)
    store_from_f32<OUT>(out, at, bf16_bits_to_f32(f32_to_bf16_bits(f16_bits_to_f32(h))) * embed_scale);
  else store_from_f32<OUT>(out, at, f16_bits_to_f32(h) * embed_scale);
}

// 4-bit codes, group size a multiple of 8: one thread per eight elements (one 32-bit load of codes).
template <int OUT>
__global__ void __launch_bounds__(256)
q4_embedding_kernel(const int64_t* __restrict__ ids, int64_t n_ids, const uint8_t* __restrict__ w_pack,
                    const uint16_t* __restrict__ scale, const uint16_t* __restrict__ zp, int group_size,
                    int64_t vocab, int dim, int64_t padding_idx, float embed_scale, bool scaled,
                    void* __restrict__ out) {
  const int per_row = dim >> 3;
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n_ids * per_row) return;
  const int64_t t = i / per_row;
  const int j8 = (int)(i - t * per_row);
  const int64_t raw = ids[t];
  const int64_t tok = raw < 0 ? 0 : (raw >= vocab ? vocab - 1 : raw);
  const uint32_t codes = *reinterpret_cast<const uint32_t*>(w_pack + tok * (dim >> 1) + j8 * 4);
  const int64_t grp = tok * (dim / group_size) + (j8 * 8) / group_size;
  const float s = f16_bits_to_f32(scale[grp]);
  const float z = zp ? f16_bits_to_f32(zp[grp]) : 8.0f;
  const bool pad = raw == padding_idx;
  if constexpr (OUT == NPAMD_F32) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float q = (float)((codes >> (4 * e)) & 0xFu);
      store_q_embedding<OUT>(out, i * 8 + e, pad ? 0.f : (q - z) * s, embed_scale, scaled);
    }
  } else {
    // eight 16-bit results leave as one 16-byte store; same roundings as store_q_embedding
    uint32_t r[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float q = (float)((codes >> (4 * e)) & 0xFu);
      const uint32_t h = f32_to_f16_bits(pad ? 0.f : (q - z) * s);
      if constexpr (OUT == NPAMD_F16) {
        r[e] = scaled ? f32_to_f16_bits(f16_bits_to_f32(h) * embed_scale) : h;
      } else {
        const uint32_t b = f32_to_bf16_bits(f16_bits_to_f32(h));
        r[e] = scaled ? f32_to_bf16_bits(bf16_bits_to_f32(b) * embed_scale) : b;
      }
    }
    *reinterpret_cast<u32x4*>((uint16_t*)out + i * 8) =
        u32x4{r[0] | (r[1] << 16), r[2] | (r[3] << 16), r[4] | (r[5] << 16), r[6] | (r[7] << 16)};
  }
}

template <int OUT>
__global__ void __launch_bounds__(256)
q_embedding_generic_kernel(const int64_t* __restrict__ ids, int64_t n_ids, const uint8_t* __restrict__ w_pack,
                           const uint16_t* __restrict__ scale, const uint16_t* __restrict__ zp, int nbits,
                           int group_size, int64_t vocab, int dim, int64_t padding_idx, float embed_scale,
                           bool scaled, void* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n_ids * dim) return;
  const int64_t t = i / dim;
  const int j = (int)(i - t * dim);
  const int64_t raw = ids[t];
  const int64_t tok = raw < 0 ? 0 : (raw >= vocab ? vocab - 1 : raw);
  const int vpb = 8 / nbits;
  const uint32_t byte = w_pack[tok * (dim / vpb) + j / vpb];
  const float q = (float)((byte >> ((j % vpb) * nbits)) & ((1u << nbits) - 1u));
  const int64_t grp = tok * (dim / group_size) + j / group_size;
  const float z = zp ? f16_bits_to_f32(zp[grp]) : (float)(1 << (nbits - 1));
  const float v = raw == padding_idx ? 0.f : (q - z) * f16_bits_to_f32(scale[grp]);
  store_q_embedding<OUT>(out, i, v, embed_scale, scaled);
}

template <int OUT>
int launch_q_embedding(const int64_t* ids, int64_t n_ids, const uint8_t* w_pack, const uint16_t* scale,
                       const uint16_t* zp, int nbits, int group_size, int64_t vocab, int dim, int64_t padding_idx,
                       float embed_scale, void* out, hipStream_t st) {
  const bool scaled = embed_scale != 1.0f;
  if (nbits == 4 && group_size % 8 == 0 && dim % 8 == 0 && (reinterpret_cast<uintptr_t>(w_pack) & 3) == 0 &&
      aligned16(out)) {
    const int64_t n = n_ids * (dim / 8);
    q4_embedding_kernel<OUT><<<(unsigned)((n + 255) / 256), 256, 0, st>>>(ids, n_ids, w_pack, scale, zp, group_size,
                                                                          vocab, dim, padding_idx, embed_scale, scaled,
                                                                          out);
  } else {
    const int64_t n = n_ids * dim;
    q_embedding_generic_kernel<OUT><<<(unsigned)((n + 255) / 256), 256, 0, st>>>(
        ids, n_ids, w_pack, scale, zp, nbits, group_size, vocab, dim, padding_idx, embed_scale, scaled, out);
  }
  return check_launch("npamd_q_embedding");
}

}  // namespace

extern "C" int npamd_rms_norm(const void* x, int64_t ldx, const void* weight, void* out, int64_t ldo, int M, int H,
                              float eps, int dtype, void* stream) {
  NPAMD_REQUIRE(dtype == NPAMD_F16 || dtype == NPAMD_BF16 || dtype == NPAMD_F32, "npamd_rms_norm: bad dtype code %d",
                dtype);
  NPAMD_REQUIRE(M >= 0 && H >= 1, "npamd_rms_norm: bad shape [%d, %d]", M, H);
  NPAMD_REQUIRE(ldx >= H && ldo >= H, "npamd_rms_norm: row stride smaller than the row");
  if (M == 0) return NPAMD_OK;
  NPAMD_REQUIRE(x && weight && out, "npamd_rms_norm: null pointer");
  hipStream_t st = (hipStream_t)stream;
  if (dtype == NPAMD_F16) return launch_rms_norm<NPAMD_F16>(x, ldx, weight, out, ldo, M, H, eps, st);
  if (dtype == NPAMD_BF16) return launch_rms_norm<NPAMD_BF16>(x, ldx, weight, out, ldo, M, H, eps, st);
  return launch_rms_norm<NPAMD_F32>(x, ldx, weight, out, ldo, M, H, eps, st);
}

extern "C" int npamd_vq_embedding(const int64_t* ids, int64_t n_ids, const int16_t* indices, int64_t vocab, int groups,
                                  const void* codebook_f16, int nc, int vl, const int32_t* inv_perm, float scale,
                                  void* out, int out_dtype, void* stream) {
  NPAMD_REQUIRE(out_dtype == NPAMD_F16 || out_dtype == NPAMD_BF16 || out_dtype == NPAMD_F32,
                "npamd_vq_embedding: bad dtype code %d", out_dtype);
  NPAMD_REQUIRE(n_ids >= 0 && vocab >= 1 && groups >= 1 && nc >= 1 && vl >= 1, "npamd_vq_embedding: bad shape");
  NPAMD_REQUIRE(nc <= 65536, "npamd_vq_embedding: the index table holds 16-bit indices, codebook has %d rows", nc);
  if (n_ids == 0) return NPAMD_OK;
  NPAMD_REQUIRE(ids && indices && codebook_f16 && out, "npamd_vq_embedding: null pointer");
  hipStream_t st = (hipStream_t)stream;
  auto idx = (const uint16_t*)indices;
  auto cb = (const uint16_t*)codebook_f16;
  if (out_dtype == NPAMD_F16)
    return launch_vq_embedding<NPAMD_F16>(ids, n_ids, idx, vocab, groups, cb, nc, vl, inv_perm, scale, out, st);
  if (out_dtype == NPAMD_BF16)
    return launch_vq_embedding<NPAMD_BF16>(ids, n_ids, idx, vocab, groups, cb, nc, vl, inv_perm, scale, out, st);
  return launch_vq_embedding<NPAMD_F32>(ids, n_ids, idx, vocab, groups, cb, nc, vl, inv_perm, scale, out, st);
}

extern "C" int npamd_q_embedding(const int64_t* ids, int64_t n_ids, const uint8_t* w_pack, const void* scale_f16,
                                 const void* zero_point_f16, int nbits, int group_size, int64_t vocab, int dim,
                                 int64_t padding_idx, float embed_scale, void* out, int out_dtype, void* stream) {
  NPAMD_REQUIRE(out_dtype == NPAMD_F16 || out_dtype == NPAMD_BF16 || out_dtype == NPAMD_F32,
                "npamd_q_embedding: bad dtype code %d", out_dtype);
  NPAMD_REQUIRE(nbits == 1 || nbits == 2 || nbits == 4 || nbits == 8, "npamd_q_embedding: nbits must be 1, 2, 4 or 8");
  NPAMD_REQUIRE(n_ids >= 0 && vocab >= 1 && dim >= 1 && group_size >= 1 && dim % group_size == 0 &&
                    dim % (8 / nbits) == 0,
                "npamd_q_embedding: bad shape (dim %d, group size %d)", dim, group_size);
  if (n_ids == 0) return NPAMD_OK;
  NPAMD_REQUIRE(ids && w_pack && scale_f16 && out, "npamd_q_embedding: null pointer");
  hipStream_t st = (hipStream_t)stream;
  auto sc = (const uint16_t*)scale_f16;
  auto zp = (const uint16_t*)zero_point_f16;
  if (out_dtype == NPAMD_F16)
    return launch_q_embedding<NPAMD_F16>(ids, n_ids, w_pack, sc, zp, nbits, group_size, vocab, dim, padding_idx,
                                         embed_scale, out, st);
  if (out_dtype == NPAMD_BF16)
    return launch_q_embedding<NPAMD_BF16>(ids, n_ids, w_pack, sc, zp, nbits, group_size, vocab, dim, padding_idx,
                                          embed_scale, out, st);
  return launch_q_embedding<NPAMD_F32>(ids, n_ids, w_pack, sc, zp, nbits, group_size, vocab, dim, padding_idx,
                                       embed_scale, out, st);
}
