// Decode GEMV over the prefix-coded index streams (two-tier, n-tier, zero-escape), read as
// they are stored: fewer bytes per index than the fixed-width stream on skewed index
// distributions.  One wave per output row; per 64-index segment of the row every lane finds
// the class (tier) of its index from the class bits, a wave ballot and a population count
// below the lane give the index's place in its class's payload stream, the payload becomes
// the codebook row, and the lane adds that row's dot product with its activation vector.
//
// Two class encodings cover the three formats:
//   cascade  D <= 4 one-bit streams; stream k holds one bit per index that tiers < k did not
//            claim, 0 = "tier k" (two-tier: D = 2, stream 0 bit 1 = cold).  The bit of index i
//            in stream k sits at position i - (number of indices before i in tiers < k).
//   flat     two class bits per index (zero-escape: 0 -> index 0, no payload).
// Per class: payload stream, payload width, base added to the payload, and the cumulative
// count of the class over the rows before each row ([N + 1] int32, built on the host when the
// layer is created), which is what lets rows be decoded independently.
#include "common.hpp"

namespace npamd {

constexpr int kCodedMaxClasses = 4;

struct CodedArgs {
  const uint16_t* x; int64_t ldx;
  const uint8_t* cls[kCodedMaxClasses - 1];  // cascade: D - 1 streams; flat: cls[0]
  int64_t cls_bytes[kCodedMaxClasses - 1];
  const uint8_t* payload[kCodedMaxClasses];
  int64_t payload_bytes[kCodedMaxClasses];
  int bits[kCodedMaxClasses];
  uint32_t base[kCodedMaxClasses];
  const int32_t* row_off[kCodedMaxClasses];
  int n_classes;
  int flat;  // 1: two class bits per index in cls[0]
  const uint16_t* codebook; uint32_t nc_minus_1; int vl;
  const float* bias; uint16_t* y; int64_t ldy;
  int M, N, G;  // G = K / VL groups per row
};

__device__ __forceinline__ uint32_t read_bit_field(const uint8_t* s, int64_t n_bytes, int64_t bit, int width) {
  const int64_t b0 = bit >> 3;
  uint32_t w = 0;
  if (b0 < n_bytes) w = s[b0];
  if (width > 1 && b0 + 1 < n_bytes) w |= (uint32_t)s[b0 + 1] << 8;
  return (w >> (bit & 7)) & ((1u << width) - 1u);
}

__device__ __forceinline__ uint32_t lanes_below(uint64_t mask) {
  return __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
}

// Codebook row index of group g of row n for every lane with `valid`; `run` carries the
// per-class counts of the row's earlier segments (wave-uniform).
__device__ __forceinline__ uint32_t coded_index(const CodedArgs& a, int n, int g, bool valid,
                                                uint32_t (&run)[kCodedMaxClasses]) {
  const int64_t i = (int64_t)n * a.G + g;
  int my_class = -1;
  uint32_t my_rank = 0;
  if (a.flat) {
    const uint32_t c = valid ? read_bit_field(a.cls[0], a.cls_bytes[0], 2 * i, 2) : 0xFFu;
#pragma unroll
    for (int k = 0; k < kCodedMaxClasses; ++k) {
      const bool is_k = c == (uint32_t)k;
      const uint64_t mask = __builtin_amdgcn_ballot_w64(is_k);
      if (is_k) {
        my_class = k;
        my_rank = run[k] + lanes_below(mask);
      }
      run[k] += (uint32_t)__builtin_popcountll(mask);
    }
  } else {
    bool undecided = valid;
    int64_t pos = i;  // position of this index's bit in the current level's stream
#pragma unroll
    for (int k = 0; k < kCodedMaxClasses; ++k) {
      if (k >= a.n_classes) break;
      bool is_k = undecided;
      if (k < a.n_classes - 1) is_k = undecided && read_bit_field(a.cls[k], a.cls_bytes[k], pos, 1) == 0u;
      const uint64_t mask = __builtin_amdgcn_ballot_w64(is_k);
      const uint32_t before = run[k] + lanes_below(mask);  // tier-k indices of this row before mine
      if (is_k) {
        my_class = k;
        my_rank = before;
        undecided = false;
      }
      pos -= (int64_t)a.row_off[k][n] + before;  // tier-k indices before index i, all rows
      run[k] += (uint32_t)__builtin_popcountll(mask);
    }
  }
  uint32_t idx = 0;
  if (my_class >= 0) {
    idx = a.base[my_class];
    if (a.bits[my_class] > 0)
      idx += read_index(a.payload[my_class], a.payload_bytes[my_class],
                        (int64_t)a.row_off[my_class][n] + my_rank, a.bits[my_class]);
  }
  return min(idx, a.nc_minus_1);
}

template <int ACT, int MT>
__global__ void __launch_bounds__(256) coded_gemv_kernel(const CodedArgs a) {
  const int lane = threadIdx.x & 63;
  const int n = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int m0 = blockIdx.y * MT;
  const int mt = min(MT, a.M - m0);
  if (n >= a.N) return;  // whole waves leave together: the ballots below see full waves
  uint32_t run[kCodedMaxClasses] = {0u, 0u, 0u, 0u};
  float acc[MT];
#pragma unroll
  for (int j = 0; j < MT; ++j) acc[j] = 0.f;
  for (int g0 = 0; g0 < a.G; g0 += 64) {
    const int g = g0 + lane;
    const bool valid = g < a.G;
    const uint32_t idx = coded_index(a, n, min(g, a.G - 1), valid, run);
    if (!valid) continue;
    if (a.vl == 8) {
      const u32x4 c = reinterpret_cast<const u32x4*>(a.codebook)[idx];
      const uint32_t cw[4] = {c.x, c.y, c.z, c.w};
#pragma unroll
      for (int j = 0; j < MT; ++j) {
        if (j >= mt) break;
        const u32x4 xv = *reinterpret_cast<const u32x4*>(a.x + (int64_t)(m0 + j) * a.ldx + (int64_t)g * 8);
        const uint32_t xw[4] = {xv.x, xv.y, xv.z, xv.w};
        float s = acc[j];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          s = __builtin_fmaf(act_bits_to_f32<ACT>(xw[e] & 0xFFFFu), act_bits_to_f32<ACT>(cw[e] & 0xFFFFu), s);
          s = __builtin_fmaf(act_bits_to_f32<ACT>(xw[e] >> 16), act_bits_to_f32<ACT>(cw[e] >> 16), s);
        }
        acc[j] = s;
      }
    } else {
      const uint16_t* c = a.codebook + (int64_t)idx * a.vl;
      for (int e = 0; e < a.vl; ++e) {
        const float w = act_bits_to_f32<ACT>(c[e]);
#pragma unroll
        for (int j = 0; j < MT; ++j)
          if (j < mt)
            acc[j] = __builtin_fmaf(act_bits_to_f32<ACT>(a.x[(int64_t)(m0 + j) * a.ldx + (int64_t)g * a.vl + e]), w, acc[j]);
      }
    }
  }
#pragma unroll
  for (int j = 0; j < MT; ++j) {
    if (j >= mt) break;
    float total = wave_reduce_sum(acc[j]);
    if (lane == 0) {
      if (a.bias) total += a.bias[n];
      store_from_f32<ACT>(a.y, (int64_t)(m0 + j) * a.ldy + n, total);
    }
  }
}

template <int ACT>
static int launch_coded(const CodedArgs& a, hipStream_t st, const char* what) {
  const unsigned rows = (unsigned)((a.N + 3) / 4);
  if (a.M == 1) coded_gemv_kernel<ACT, 1><<<dim3(rows, 1), 256, 0, st>>>(a);
  else if (a.M <= 4) coded_gemv_kernel<ACT, 4><<<dim3(rows, 1), 256, 0, st>>>(a);
  else coded_gemv_kernel<ACT, 8><<<dim3(rows, (unsigned)((a.M + 7) / 8)), 256, 0, st>>>(a);
  return check_launch(what);
}

}  // namespace npamd

using namespace npamd;

extern "C" int npamd_vq_gemv_coded(const void* x, int64_t ldx, int flat, int n_classes,
                                   const uint8_t* const* class_streams, const int64_t* class_bytes,
                                   const uint8_t* const* payload_streams, const int64_t* payload_bytes,
                                   const int* payload_bits, const uint32_t* payload_base,
                                   const int32_t* const* row_offsets, const void* codebook, int codebook_dtype,
                                   int nc, int vl, const float* bias, void* y, int64_t ldy, int M, int N, int K,
                                   int act_dtype, void* stream) {
  const char* what = "npamd_vq_gemv_coded";
  NPAMD_REQUIRE(act_dtype == NPAMD_F16 || act_dtype == NPAMD_BF16,
                "%s: activations must be f16 or bf16 (got dtype code %d)", what, act_dtype);
  NPAMD_REQUIRE(codebook_dtype == act_dtype, "%s: the codebook must be in the activation dtype", what);
  NPAMD_REQUIRE(flat == 0 || flat == 1, "%s: flat must be 0 (cascaded one-bit streams) or 1 (two class bits)", what);
  NPAMD_REQUIRE(flat ? n_classes == 4 : (n_classes >= 2 && n_classes <= kCodedMaxClasses),
                "%s: %d classes (cascade: 2..4, flat: 4)", what, n_classes);
  NPAMD_REQUIRE(vl >= 1 && nc >= 1 && N >= 0 && K >= 0 && K % vl == 0, "%s: bad shape N=%d K=%d NC=%d VL=%d", what, N, K, nc, vl);
  NPAMD_REQUIRE(M >= 0 && M <= NPAMD_GEMV_MAX_M, "%s: M=%d exceeds the fused limit %d", what, M, NPAMD_GEMV_MAX_M);
  NPAMD_REQUIRE(ldx >= K && ldy >= N, "%s: row stride smaller than the row", what);
  if (M == 0 || N == 0) return NPAMD_OK;
  NPAMD_REQUIRE(x && y && codebook && class_streams && class_bytes && payload_streams && payload_bytes && payload_bits &&
                    payload_base && row_offsets, "%s: null pointer", what);
  NPAMD_REQUIRE((int64_t)N * (K / vl) < ((int64_t)1 << 31), "%s: more than 2^31 indices", what);
  NPAMD_REQUIRE(vl != 8 || ((reinterpret_cast<uintptr_t>(x) % 16) == 0 && ldx % 8 == 0 &&
                            (reinterpret_cast<uintptr_t>(codebook) % 16) == 0),
                "%s: x and the codebook must be 16-byte aligned (ldx a multiple of 8)", what);
  CodedArgs a;
  a.x = (const uint16_t*)x; a.ldx = ldx;
  a.n_classes = n_classes; a.flat = flat;
  const int n_cls_streams = flat ? 1 : n_classes - 1;
  for (int k = 0; k < kCodedMaxClasses - 1; ++k) {
    a.cls[k] = k < n_cls_streams ? class_streams[k] : nullptr;
    a.cls_bytes[k] = k < n_cls_streams ? class_bytes[k] : 0;
    NPAMD_REQUIRE(k >= n_cls_streams || (a.cls[k] && a.cls_bytes[k] >= 0), "%s: class stream %d is null", what, k);
  }
  for (int k = 0; k < kCodedMaxClasses; ++k) {
    const bool used = k < n_classes;
    a.payload[k] = used ? payload_streams[k] : nullptr;
    a.payload_bytes[k] = used ? payload_bytes[k] : 0;
    a.bits[k] = used ? payload_bits[k] : 0;
    a.base[k] = used ? payload_base[k] : 0u;
    a.row_off[k] = used ? row_offsets[k] : nullptr;
    if (used) {
      NPAMD_REQUIRE(a.bits[k] >= 0 && a.bits[k] <= 20, "%s: payload width %d of class %d outside [0, 20]", what, a.bits[k], k);
      NPAMD_REQUIRE(a.row_off[k] && (a.bits[k] == 0 || a.payload[k] || a.payload_bytes[k] == 0),
                    "%s: class %d: null row offsets or payload stream", what, k);
    }
  }
  a.codebook = (const uint16_t*)codebook; a.nc_minus_1 = (uint32_t)nc - 1u; a.vl = vl;
  a.bias = bias; a.y = (uint16_t*)y; a.ldy = ldy;
  a.M = M; a.N = N; a.G = K / vl;
  return act_dtype == NPAMD_BF16 ? launch_coded<NPAMD_BF16>(a, (hipStream_t)stream, what)
                                 : launch_coded<NPAMD_F16>(a, (hipStream_t)stream, what);
}
