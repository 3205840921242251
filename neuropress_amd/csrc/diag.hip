// Diagnostic kernels: the memory-system ceilings the decode kernels are judged
// against, measured with the same access pattern and nothing else.
//   stream read  -- read a buffer once, 16 bytes per lane (HBM streaming rate
//                   for a buffer of that size in a single launch)
//   gather       -- stream 16-bit indices (8 per lane) and fetch one 16-byte
//                   table row per index from global memory or from an LDS copy
//                   of the table; results are xor-folded and never stored
#include "common.hpp"
#include "../../include/npamd_diag.h"

namespace npamd {

__global__ void __launch_bounds__(256)
diag_stream_read_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ sink, int64_t n16) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n16) return;
  const u32x4 v = src[i];
  if (v.x == 0x12345678u && v.y == 0x9abcdef0u && v.z == 0x0fedcba9u) sink[0] = v;  // never true in practice
}

__device__ __forceinline__ void split8(const u32x4& v, uint32_t (&id)[8]) {
  id[0] = v.x & 0xffffu; id[1] = v.x >> 16; id[2] = v.y & 0xffffu; id[3] = v.y >> 16;
  id[4] = v.z & 0xffffu; id[5] = v.z >> 16; id[6] = v.w & 0xffffu; id[7] = v.w >> 16;
}

__global__ void __launch_bounds__(256)
diag_gather_global_kernel(const u32x4* __restrict__ idx, const u32x4* __restrict__ table,
                          uint32_t mask, u32x4* __restrict__ sink, int64_t n8) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n8) return;
  uint32_t id[8];
  split8(idx[i], id);
  u32x4 acc{0, 0, 0, 0};
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const u32x4 c = table[id[j] & mask];
    acc.x ^= c.x; acc.y ^= c.y; acc.z ^= c.z; acc.w ^= c.w;
  }
  if (acc.x == 0x12345678u && acc.y == 0x9abcdef0u) sink[0] = acc;
}

__global__ void __launch_bounds__(1024)
diag_gather_lds_kernel(const u32x4* __restrict__ idx, const u32x4* __restrict__ table, int entries,
                       u32x4* __restrict__ sink, int64_t n8, int64_t per_block) {
  extern __shared__ u32x4 tab[];
  for (int i = threadIdx.x; i < entries; i += blockDim.x) tab[i] = table[i];
  __syncthreads();
  const int64_t base = (int64_t)blockIdx.x * per_block;
  const int64_t end = base + per_block < n8 ? base + per_block : n8;
  u32x4 acc{0, 0, 0, 0};
  for (int64_t i = base + threadIdx.x; i < end; i += blockDim.x) {
    uint32_t id[8];
    split8(idx[i], id);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const u32x4 c = tab[id[j] & (uint32_t)(entries - 1)];
      acc.x ^= c.x; acc.y ^= c.y; acc.z ^= c.z; acc.w ^= c.w;
    }
  }
  if (acc.x == 0x12345678u && acc.y == 0x9abcdef0u) sink[0] = acc;
}

// The matrix pipes alone: twelve independent accumulator tiles per wave, one wave per SIMD.
template <int ACT>
__global__ void __launch_bounds__(256)
diag_mfma_kernel(const u32x4* __restrict__ operands, float* __restrict__ sink, int rounds) {
  u32x4 a[3], b[4];
#pragma unroll
  for (int i = 0; i < 3; ++i) a[i] = operands[(threadIdx.x & 63) + 64 * i];
#pragma unroll
  for (int i = 0; i < 4; ++i) b[i] = operands[(threadIdx.x & 63) + 64 * (3 + i)];
  f32x16 acc[12];
#pragma unroll
  for (int i = 0; i < 12; ++i)
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[i][j] = 0.f;
  for (int r = 0; r < rounds; ++r) {
#pragma unroll
    for (int i = 0; i < 12; ++i) acc[i] = mfma32<ACT>(a[i % 3], b[i / 3], acc[i]);
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 12; ++i)
#pragma unroll
    for (int j = 0; j < 16; ++j) s += acc[i][j];
  if (s == 12345.678f) sink[0] = s;  // never true in practice
}

}  // namespace npamd

using namespace npamd;

extern "C" int npamd_diag_mfma(const void* operands, int blocks, int mfmas_per_wave, int act_dtype, void* sink16,
                               void* stream) {
  NPAMD_REQUIRE(operands && sink16 && blocks >= 1 && mfmas_per_wave >= 1, "npamd_diag_mfma: bad arguments");
  NPAMD_REQUIRE(act_dtype == NPAMD_F16 || act_dtype == NPAMD_BF16, "npamd_diag_mfma: f16 or bf16");
  const int rounds = (mfmas_per_wave + 11) / 12;
  if (act_dtype == NPAMD_BF16)
    diag_mfma_kernel<NPAMD_BF16><<<blocks, 256, 0, (hipStream_t)stream>>>((const u32x4*)operands, (float*)sink16, rounds);
  else
    diag_mfma_kernel<NPAMD_F16><<<blocks, 256, 0, (hipStream_t)stream>>>((const u32x4*)operands, (float*)sink16, rounds);
  return check_launch("npamd_diag_mfma");
}

extern "C" int npamd_diag_stream_read(const void* src, int64_t n_bytes, void* sink16, void* stream) {
  NPAMD_REQUIRE(src && sink16 && n_bytes >= 16 && n_bytes % 16 == 0,
                "npamd_diag_stream_read: need a non-null buffer of a multiple of 16 bytes");
  const int64_t n16 = n_bytes / 16;
  diag_stream_read_kernel<<<(unsigned)((n16 + 255) / 256), 256, 0, (hipStream_t)stream>>>(
      (const u32x4*)src, (u32x4*)sink16, n16);
  return check_launch("npamd_diag_stream_read");
}

extern "C" int npamd_diag_gather(const void* idx_u16, int64_t n_indices, const void* table16,
                                 int table_entries, int from_lds, void* sink16, void* stream) {
  NPAMD_REQUIRE(idx_u16 && table16 && sink16, "npamd_diag_gather: null pointer");
  NPAMD_REQUIRE(n_indices >= 8 && n_indices % 8 == 0, "npamd_diag_gather: n_indices must be a multiple of 8");
  NPAMD_REQUIRE(table_entries >= 1 && (table_entries & (table_entries - 1)) == 0,
                "npamd_diag_gather: table_entries must be a power of two");
  const int64_t n8 = n_indices / 8;
  hipStream_t st = (hipStream_t)stream;
  if (!from_lds) {
    diag_gather_global_kernel<<<(unsigned)((n8 + 255) / 256), 256, 0, st>>>(
        (const u32x4*)idx_u16, (const u32x4*)table16, (uint32_t)table_entries - 1u, (u32x4*)sink16, n8);
    return check_launch("npamd_diag_gather");
  }
  NPAMD_REQUIRE(table_entries <= 8192, "npamd_diag_gather: an LDS table holds at most 8192 rows");
  const int lds = table_entries * 16;
  if (lds > 64 * 1024) {
    static LdsLatch latch;
    const hipError_t e = enable_dynamic_lds(latch, reinterpret_cast<const void*>(&diag_gather_lds_kernel), lds);
    if (e != hipSuccess) return fail(NPAMD_ERR_LAUNCH, "npamd_diag_gather: %s", hipGetErrorString(e));
  }
  const int blocks = 512;
  const int64_t per_block = (n8 + blocks - 1) / blocks;
  diag_gather_lds_kernel<<<blocks, 1024, lds, st>>>((const u32x4*)idx_u16, (const u32x4*)table16,
                                                    table_entries, (u32x4*)sink16, n8, per_block);
  return check_launch("npamd_diag_gather");
}
