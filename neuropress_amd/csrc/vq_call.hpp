// Argument bundle, validation and fast-path test shared by the VQ GEMV and
// tile-GEMM entry points.
#pragma once

#include "gemv.hpp"

namespace npamd {

struct VqCall {
  const void* x; int64_t ldx;
  const uint8_t* packed; int64_t n_bytes; int bits;
  const void* cb; int cb_dtype; int nc; int vl;
  const uint8_t* packed_r; int64_t n_bytes_r; int bits_r;
  const void* cb_r; int nc_r;
  const void* row_scale; const void* row_bias;
  const float* bias; void* y; int64_t ldy;
  int M, N, K, act;
  hipStream_t st;
  const char* what;
  void* ws = nullptr;      // tile GEMM only: f32 scratch for split-K partial tiles (may stay null)
  int64_t ws_bytes = 0;
  const int32_t* perm = nullptr;  // fused GEMV only: contract x[m, perm[k]] with W[n, k]
};

inline bool aligned(const void* p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

inline int validate(const VqCall& c, int max_m) {
  NPAMD_REQUIRE(c.act == NPAMD_F16 || c.act == NPAMD_BF16,
                "%s: activations must be f16 or bf16 (got dtype code %d)", c.what, c.act);
  NPAMD_REQUIRE(c.cb_dtype == NPAMD_F16 || c.cb_dtype == c.act,
                "%s: codebook must be f16 or the activation dtype", c.what);
  NPAMD_REQUIRE(c.bits >= 4 && c.bits <= 20, "%s: bits must be in [4, 20], got %d", c.what, c.bits);
  NPAMD_REQUIRE(c.vl >= 1 && c.nc >= 1, "%s: bad codebook shape [%d, %d]", c.what, c.nc, c.vl);
  NPAMD_REQUIRE(c.M >= 0 && c.N >= 0 && c.K >= 0, "%s: negative dimension", c.what);
  NPAMD_REQUIRE(max_m <= 0 || c.M <= max_m, "%s: M=%d exceeds the fused limit %d", c.what, c.M, max_m);
  NPAMD_REQUIRE(c.K % c.vl == 0, "%s: K=%d not divisible by VL=%d", c.what, c.K, c.vl);
  NPAMD_REQUIRE(c.ldx >= c.K && c.ldy >= c.N, "%s: row stride smaller than the row", c.what);
  const int64_t n_idx = (int64_t)c.N * (c.K / c.vl);
  NPAMD_REQUIRE((n_idx * c.bits + 7) / 8 <= c.n_bytes, "%s: packed buffer too short", c.what);
  if (c.packed_r) {
    NPAMD_REQUIRE(c.cb_dtype == NPAMD_F16, "%s: residual codebooks must be f16", c.what);
    NPAMD_REQUIRE(c.bits_r >= 4 && c.bits_r <= 20 && c.nc_r >= 1 && c.cb_r,
                  "%s: bad residual codebook / bits", c.what);
    NPAMD_REQUIRE((n_idx * c.bits_r + 7) / 8 <= c.n_bytes_r, "%s: residual packed buffer too short", c.what);
  }
  if (c.M == 0 || c.N == 0) return 1;  // nothing to do
  NPAMD_REQUIRE(c.x && c.y && (c.K == 0 || (c.packed && c.cb)), "%s: null pointer", c.what);
  return NPAMD_OK;
}

inline VqElem make_elem(const VqCall& c) {
  VqElem e{};
  e.packed = c.packed; e.n_bytes = c.n_bytes; e.bits = c.bits;
  e.cb = (const uint16_t*)c.cb; e.nc_minus_1 = (uint32_t)c.nc - 1u;
  e.vl = c.vl; e.groups = c.K / c.vl; e.act = c.act; e.cb_dtype = c.cb_dtype;
  e.packed_r = c.packed_r; e.n_bytes_r = c.n_bytes_r; e.bits_r = c.bits_r;
  e.cb_r = (const uint16_t*)c.cb_r; e.ncr_minus_1 = (uint32_t)(c.nc_r > 0 ? c.nc_r : 1) - 1u;
  e.row_scale = (const uint16_t*)c.row_scale; e.row_bias = (const uint16_t*)c.row_bias;
  return e;
}

inline bool fast_ok(const VqCall& c) {
  const bool bits_ok = c.bits == 4 || c.bits == 8 || c.bits == 12 || c.bits == 16;
  return (c.vl == 8 || (c.vl == 4 && !c.packed_r)) && bits_ok && c.K % 64 == 0 && c.K > 0 && c.ldx % 8 == 0 && aligned(c.x, 16) &&
         aligned(c.packed, 16) && aligned(c.cb, 16);
}

}  // namespace npamd
