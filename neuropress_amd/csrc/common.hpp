// Shared device helpers for the gfx950 quantized-linear kernels.
//
// Wave size is 64 throughout; MFMA operands are handled as four 32-bit
// registers (u32x4 = eight 16-bit values) and bit-cast at the call site.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>
#include <mutex>

#include "../../include/npamd.h"

namespace npamd {

typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int kWave = 64;

// ---------------------------------------------------------------------------
// Error plumbing (host side)
// ---------------------------------------------------------------------------
void set_error(const char* fmt, ...);
int fail(int code, const char* fmt, ...);
int check_launch(const char* what);

// Values of the NPAMD_* tuning environment variables, read once per process.
struct Tuning {
  int gemv_lds_cb, tile_lds_cb, gemv_lds_x, gemv_r, gemv_spw, gemv_parts, gemv_xstage, tile_splits, tile_mw, tile_wide;
  int q4_rows, q4_rowwise, q4_rowwise_bf16, q4_stream;
};
const Tuning& tuning();

// Dynamic LDS beyond 64 KiB has to be enabled per kernel and per device (hipFuncSetAttribute).
// One latch per kernel instantiation (a function-local static of its launcher) holds the largest
// size enabled so far on each device; the attribute only ever grows, and two threads enabling
// sizes at once both leave it large enough.  Devices past the table are enabled on every launch.
constexpr int kLdsLatchDevices = 64;
struct LdsLatch {
  std::atomic<int> reserved[kLdsLatchDevices];
};
inline hipError_t enable_dynamic_lds(LdsLatch& latch, const void* kernel, int bytes) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess) dev = -1;
  std::atomic<int>* slot = (dev >= 0 && dev < kLdsLatchDevices) ? &latch.reserved[dev] : nullptr;
  if (slot && bytes <= slot->load(std::memory_order_acquire)) return hipSuccess;
  // Raising the limit is serialised: two first callers with different sizes must not leave the
  // kernel with the smaller one while the latch records the larger.
  static std::mutex raise;
  std::lock_guard<std::mutex> lock(raise);
  if (slot && bytes <= slot->load(std::memory_order_acquire)) return hipSuccess;
  const hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e == hipSuccess && slot) slot->store(bytes, std::memory_order_release);
  return e;
}

#define NPAMD_REQUIRE(cond, ...)                                  \
  do {                                                            \
    if (!(cond)) return ::npamd::fail(NPAMD_ERR_INVALID, __VA_ARGS__); \
  } while (0)

// ---------------------------------------------------------------------------
// 16-bit float conversions
// ---------------------------------------------------------------------------

__device__ __forceinline__ float f16_bits_to_f32(uint32_t h) {
  return (float)__builtin_bit_cast(_Float16, (uint16_t)h);
}
__device__ __forceinline__ uint32_t f32_to_f16_bits(float f) {
  return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)f);  // RNE
}
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) {
  return __builtin_bit_cast(float, b << 16);
}
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  return (uint32_t)__builtin_bit_cast(uint16_t, (__bf16)f);  // RNE (v_cvt_pk_bf16_f32)
}

template <int ACT>
__device__ __forceinline__ float act_bits_to_f32(uint32_t v) {
  if constexpr (ACT == NPAMD_BF16) return bf16_bits_to_f32(v);
  else return f16_bits_to_f32(v);
}

// Two packed fp16 values -> two packed bf16 values (RNE of the exact f32 value).
__device__ __forceinline__ uint32_t f16x2_to_bf16x2(uint32_t h2) {
  const f16x2 v = __builtin_bit_cast(f16x2, h2);
  bf16x2 r;
  r.x = (__bf16)(float)v.x;
  r.y = (__bf16)(float)v.y;
  return __builtin_bit_cast(uint32_t, r);
}

// Eight packed fp16 codebook values -> the activation dtype's packed form.
template <int ACT>
__device__ __forceinline__ u32x4 cb_to_act(u32x4 c) {
  if constexpr (ACT == NPAMD_BF16) {
    u32x4 r;
    r.x = f16x2_to_bf16x2(c.x);
    r.y = f16x2_to_bf16x2(c.y);
    r.z = f16x2_to_bf16x2(c.z);
    r.w = f16x2_to_bf16x2(c.w);
    return r;
  } else {
    return c;
  }
}

template <int DT>
__device__ __forceinline__ float load_as_f32(const void* p, int64_t i) {
  if constexpr (DT == NPAMD_F16) return f16_bits_to_f32(((const uint16_t*)p)[i]);
  else if constexpr (DT == NPAMD_BF16) return bf16_bits_to_f32(((const uint16_t*)p)[i]);
  else return ((const float*)p)[i];
}

template <int DT>
__device__ __forceinline__ void store_from_f32(void* p, int64_t i, float v) {
  if constexpr (DT == NPAMD_F16) ((uint16_t*)p)[i] = (uint16_t)f32_to_f16_bits(v);
  else if constexpr (DT == NPAMD_BF16) ((uint16_t*)p)[i] = (uint16_t)f32_to_bf16_bits(v);
  else ((float*)p)[i] = v;
}

// fp16 bit pattern -> output dtype bit pattern / value, exactly as a dtype cast
// of the fp16 value (copy, RNE to bf16, or exact widening).
template <int DT>
__device__ __forceinline__ void store_from_f16_bits(void* p, int64_t i, uint32_t h) {
  if constexpr (DT == NPAMD_F16) ((uint16_t*)p)[i] = (uint16_t)h;
  else if constexpr (DT == NPAMD_BF16) ((uint16_t*)p)[i] = (uint16_t)f32_to_bf16_bits(f16_bits_to_f32(h));
  else ((float*)p)[i] = f16_bits_to_f32(h);
}

// ---------------------------------------------------------------------------
// Index bit-stream: index i occupies stream bits [i*bits, (i+1)*bits), LSB
// first.  Generic reader: a byte window that never reads at or past n_bytes.
// bits <= 20 and bit_off <= 7 need at most 27 bits = 4 bytes.
// ---------------------------------------------------------------------------
__device__ __forceinline__ uint32_t read_index(const uint8_t* __restrict__ packed,
                                               int64_t n_bytes, int64_t i, int bits) {
  const int64_t bit = i * (int64_t)bits;
  const int64_t b0 = bit >> 3;
  const int off = (int)(bit & 7);
  uint32_t w = 0;
  if (b0 < n_bytes) w = packed[b0];
  if (b0 + 1 < n_bytes) w |= (uint32_t)packed[b0 + 1] << 8;
  if (b0 + 2 < n_bytes) w |= (uint32_t)packed[b0 + 2] << 16;
  if (bits > 16 && b0 + 3 < n_bytes) w |= (uint32_t)packed[b0 + 3] << 24;
  return (w >> off) & ((1u << bits) - 1u);
}

// Eight consecutive indices starting at index i0 (i0 % 8 == 0), returned as
// eight 16-bit values packed in four dwords, for the widths whose 8-index
// group is a whole number of dwords.  The caller guarantees the group lies
// inside the stream and the stream base is 16-byte aligned.
// The two halves of that: the memory reads alone (BITS / 4 dwords, the rest of the vector
// zero), and the arithmetic that spreads them into eight 16-bit fields.  A software pipeline
// that requests packed bytes many iterations before it needs the indices keeps the raw
// dwords and extracts at the point of use -- arithmetic on a loaded value placed next to the
// load makes the compiler wait for the load there.
template <int BITS>
__device__ __forceinline__ u32x4 load_raw8(const uint8_t* __restrict__ packed, int64_t i0) {
  static_assert(BITS == 4 || BITS == 8 || BITS == 12 || BITS == 16, "fast widths only");
  u32x4 r{0u, 0u, 0u, 0u};
  if constexpr (BITS == 16) {
    r = *reinterpret_cast<const u32x4*>(packed + i0 * 2);
  } else if constexpr (BITS == 8) {
    const u32x2 w = *reinterpret_cast<const u32x2*>(packed + i0);
    r.x = w.x;
    r.y = w.y;
  } else if constexpr (BITS == 4) {
    r.x = *reinterpret_cast<const uint32_t*>(packed + (i0 >> 1));
  } else {  // 12 bits: 8 indices in 3 dwords
    const uint32_t* p = reinterpret_cast<const uint32_t*>(packed + (i0 >> 3) * 12);
    r.x = p[0];
    r.y = p[1];
    r.z = p[2];
  }
  return r;
}

template <int BITS>
__device__ __forceinline__ u32x4 extract_idx8(const u32x4& raw) {
  u32x4 r;
  if constexpr (BITS == 16) {
    r = raw;
  } else if constexpr (BITS == 8) {
    r.x = (raw.x & 0xFFu) | ((raw.x & 0xFF00u) << 8);
    r.y = ((raw.x >> 16) & 0xFFu) | ((raw.x >> 8) & 0xFF0000u);
    r.z = (raw.y & 0xFFu) | ((raw.y & 0xFF00u) << 8);
    r.w = ((raw.y >> 16) & 0xFFu) | ((raw.y >> 8) & 0xFF0000u);
  } else if constexpr (BITS == 4) {
    const uint32_t w = raw.x;
    r.x = (w & 0xFu) | ((w & 0xF0u) << 12);
    r.y = ((w >> 8) & 0xFu) | ((w & 0xF000u) << 4);
    r.z = ((w >> 16) & 0xFu) | ((w >> 4) & 0xF0000u);
    r.w = ((w >> 24) & 0xFu) | ((w >> 12) & 0xF0000u);
  } else {
    const uint32_t a = raw.x, b = raw.y, c = raw.z;
    r.x = (a & 0xFFFu) | ((a << 4) & 0x0FFF0000u);
    r.y = ((a >> 24) | ((b & 0xFu) << 8)) | ((b << 12) & 0x0FFF0000u);
    r.z = ((b >> 16) & 0xFFFu) | (((b >> 28) | ((c & 0xFFu) << 4)) << 16);
    r.w = ((c >> 8) & 0xFFFu) | ((c >> 4) & 0x0FFF0000u);
  }
  return r;
}

template <int BITS>
__device__ __forceinline__ u32x4 load_idx8(const uint8_t* __restrict__ packed, int64_t i0) {
  return extract_idx8<BITS>(load_raw8<BITS>(packed, i0));
}

__device__ __forceinline__ uint32_t idx8_get(const u32x4& v, int j) {
  const uint32_t w = (j < 2) ? v.x : (j < 4) ? v.y : (j < 6) ? v.z : v.w;
  return (j & 1) ? (w >> 16) : (w & 0xFFFFu);
}

// ---------------------------------------------------------------------------
// MFMA wrappers on raw registers
// ---------------------------------------------------------------------------
template <int ACT>
__device__ __forceinline__ f32x4 mfma16(u32x4 a, u32x4 b, f32x4 c) {
  if constexpr (ACT == NPAMD_BF16)
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

template <int ACT>
__device__ __forceinline__ f32x16 mfma32(u32x4 a, u32x4 b, f32x16 c) {
  if constexpr (ACT == NPAMD_BF16)
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

__device__ __forceinline__ float wave_reduce_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

}  // namespace npamd
