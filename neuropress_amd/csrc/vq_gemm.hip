// C-ABI entry points of the tile-decode MFMA GEMM (plain and residual VQ).
#include "gemm_tile2.hpp"
#include "vq_call.hpp"

using namespace npamd;

namespace {

template <int ACT, int BITS, int VL>
int run_vq(const VqCall& c, const GemmShape& s) {
  if constexpr (ACT == NPAMD_BF16) {
    if (c.cb_dtype == NPAMD_F16) {
      using P = VqProvider<ACT, BITS, true, VL>;
      typename P::Args a{c.packed, (const u32x4*)c.cb, (uint32_t)c.nc - 1u, s.chunks};
      return launch_tile_gemm<ACT, P>(s, a, c.st, c.what, c.ws, c.ws_bytes, (VL == 8 ? c.nc * 16 : (c.nc % 2 == 0 ? c.nc * 8 : 0)));
    }
  }
  if constexpr (BITS == 16 && VL == 8) {
    // Codebooks LDS does not hold, in the activation dtype: the 128-column kernel, whose gathers write LDS directly.
    const int mode = tile2_mode();
    const bool big = (int64_t)c.nc * 16 > kTileLdsCodebookMax;
    // Measured against the 64-column kernel on 65536-row codebooks, 17 / 384 tokens (us): 14336 x 4096 40.8 / 66.6
    // against 48.9 / 86.0, 4096 x 14336 42.8 / 75.8 against 49.5 / 92.0, 8192 x 8192 44.8 / 88.5 against 53.2 / 108,
    // 28672 x 4096 72.3 / 112 against 84.4 / 157, 6144 x 4096 23.6 / 54.9 against 29.1 / 57.7, 4096 x 4096 20.4 / 41.6
    // against 24.6 / 43.7, 2048 x 8192 23.8 / 43.4 against 26.4 / 44.8, 8192 x 2048 18.4 / 45.4 against 23.6 / 46.1:
    // ahead on every layer whose codebook stays in memory.
    const bool wins = big;
    if (c.cb_dtype == c.act && c.n_bytes < ((int64_t)1 << 32) && (mode >= 2 || (mode == 1 && wins))) {
      const T2Args t2{c.packed, c.cb, (uint32_t)c.nc - 1u, s.chunks};
      const int rc = launch_tile2(ACT, s, t2, c.st, c.what, c.ws, c.ws_bytes);
      if (rc != 1) return rc;
    }
  }
  using P = VqProvider<ACT, BITS, false, VL>;
  typename P::Args a{c.packed, (const u32x4*)c.cb, (uint32_t)c.nc - 1u, s.chunks};
  return launch_tile_gemm<ACT, P>(s, a, c.st, c.what, c.ws, c.ws_bytes, (VL == 8 ? c.nc * 16 : (c.nc % 2 == 0 ? c.nc * 8 : 0)));
}

template <int ACT, int VL>
int run_vq_bits_vl(const VqCall& c, const GemmShape& s) {
  switch (c.bits) {
    case 4: return run_vq<ACT, 4, VL>(c, s);
    case 8: return run_vq<ACT, 8, VL>(c, s);
    case 12: return run_vq<ACT, 12, VL>(c, s);
    default: return run_vq<ACT, 16, VL>(c, s);
  }
}

template <int ACT>
int run_vq_bits(const VqCall& c, const GemmShape& s) {
  return c.vl == 4 ? run_vq_bits_vl<ACT, 4>(c, s) : run_vq_bits_vl<ACT, 8>(c, s);
}

template <int ACT, int BM_, int BR_>
int run_rvq(const VqCall& c, const GemmShape& s) {
  using P = RvqProvider<ACT, BM_, BR_>;
  typename P::Args a{c.packed, c.packed_r, (const u32x4*)c.cb, (const u32x4*)c.cb_r,
                     (const uint16_t*)c.row_scale, (const uint16_t*)c.row_bias,
                     (uint32_t)c.nc - 1u, (uint32_t)c.nc_r - 1u, s.chunks};
  return launch_tile_gemm<ACT, P>(s, a, c.st, c.what, c.ws, c.ws_bytes, c.nc_r * 16);
}

template <int ACT>
int dispatch(const VqCall& c) {
  GemmShape s{c.x, c.ldx, c.bias, c.y, c.ldy, c.M, c.N, c.K, c.K / 64, 0};
  if (fast_ok(c)) {
    if (!c.packed_r) return run_vq_bits<ACT>(c, s);
    const bool res_ok = aligned(c.packed_r, 16) && aligned(c.cb_r, 16);
    if (res_ok && c.bits == 16 && c.bits_r == 8) return run_rvq<ACT, 16, 8>(c, s);
    if (res_ok && c.bits == 16 && c.bits_r == 16) return run_rvq<ACT, 16, 16>(c, s);
    if (res_ok && c.bits == 12 && c.bits_r == 8) return run_rvq<ACT, 12, 8>(c, s);
    if (res_ok && c.bits == 8 && c.bits_r == 8) return run_rvq<ACT, 8, 8>(c, s);
  }
  return launch_generic_gemm<ACT>(c.x, c.ldx, c.bias, c.y, c.ldy, c.M, c.N, c.K, make_elem(c), c.st, c.what);
}

int run(const VqCall& c) {
  const int rc = validate(c, 0);
  if (rc < 0) return rc;
  if (rc == 1) return NPAMD_OK;
  NPAMD_REQUIRE(c.ws == nullptr || (aligned(c.ws, 16) && c.ws_bytes >= 0), "%s: workspace must be 16-byte aligned", c.what);
  return c.act == NPAMD_BF16 ? dispatch<NPAMD_BF16>(c) : dispatch<NPAMD_F16>(c);
}

}  // namespace

extern "C" int npamd_vq_gemm_tile(const void* x, int64_t ldx, const uint8_t* packed, int64_t n_bytes,
                             int bits, const void* codebook, int codebook_dtype, int nc, int vl,
                             const float* bias, void* y, int64_t ldy, int M, int N, int K,
                             int act_dtype, void* workspace, int64_t workspace_bytes, void* stream) {
  VqCall c{x, ldx, packed, n_bytes, bits, codebook, codebook_dtype, nc, vl,
               nullptr, 0, 0, nullptr, 0, nullptr, nullptr,
               bias, y, ldy, M, N, K, act_dtype, (hipStream_t)stream, "npamd_vq_gemm_tile"};
  c.ws = workspace;
  c.ws_bytes = workspace_bytes;
  return run(c);
}

extern "C" int npamd_rvq_gemm_tile(const void* x, int64_t ldx,
                              const uint8_t* packed_main, int64_t n_bytes_main, int bits_main,
                              const uint8_t* packed_res, int64_t n_bytes_res, int bits_res,
                              const void* cb_main_f16, int nc_main, const void* cb_res_f16, int nc_res,
                              const void* row_scale_f16, const void* row_bias_f16, int vl,
                              const float* bias, void* y, int64_t ldy, int M, int N, int K,
                              int act_dtype, void* workspace, int64_t workspace_bytes, void* stream) {
  if (!packed_res) return fail(NPAMD_ERR_INVALID, "npamd_rvq_gemm_tile: residual stream is null");
  VqCall c{x, ldx, packed_main, n_bytes_main, bits_main, cb_main_f16, NPAMD_F16, nc_main, vl,
               packed_res, n_bytes_res, bits_res, cb_res_f16, nc_res, row_scale_f16, row_bias_f16,
               bias, y, ldy, M, N, K, act_dtype, (hipStream_t)stream, "npamd_rvq_gemm_tile"};
  c.ws = workspace;
  c.ws_bytes = workspace_bytes;
  return run(c);
}
