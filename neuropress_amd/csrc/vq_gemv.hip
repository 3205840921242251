// C-ABI entry points of the fused decode GEMV (plain and residual VQ).
#include "vq_call.hpp"

using namespace npamd;

namespace {

template <int ACT, int BITS, int VL>
int run_vq(const VqCall& c, const GemvShape& s) {
  if constexpr (ACT == NPAMD_BF16) {
    if (c.cb_dtype == NPAMD_F16) {
      using P = VqProvider<ACT, BITS, true, VL>;
      typename P::Args a{c.packed, (const u32x4*)c.cb, (uint32_t)c.nc - 1u, s.chunks};
      return launch_fused_gemv<ACT, P>(s, a, c.st, c.what, (VL == 8 ? c.nc * 16 : (c.nc % 2 == 0 ? c.nc * 8 : 0)));
    }
  }
  using P = VqProvider<ACT, BITS, false, VL>;
  typename P::Args a{c.packed, (const u32x4*)c.cb, (uint32_t)c.nc - 1u, s.chunks};
  return launch_fused_gemv<ACT, P>(s, a, c.st, c.what, (VL == 8 ? c.nc * 16 : (c.nc % 2 == 0 ? c.nc * 8 : 0)));
}

}  // namespace

int npamd::vq_gemv_plan_stages(int M, int N, int K, int nc) {
  int staged = 0;
  GemvShape s{nullptr, K, nullptr, nullptr, N, M, N, K / 64, 0, 0};
  s.plan_only = &staged;
  using P = VqProvider<NPAMD_F16, 16, false, 8>;  // the choice depends on the table's size, not on the index width
  typename P::Args a{};
  launch_fused_gemv<NPAMD_F16, P>(s, a, nullptr, "plan", nc * 16);
  return staged;
}

namespace {

template <int ACT, int VL>
int run_vq_bits_vl(const VqCall& c, const GemvShape& s) {
  switch (c.bits) {
    case 4: return run_vq<ACT, 4, VL>(c, s);
    case 8: return run_vq<ACT, 8, VL>(c, s);
    case 12: return run_vq<ACT, 12, VL>(c, s);
    default: return run_vq<ACT, 16, VL>(c, s);
  }
}

template <int ACT>
int run_vq_bits(const VqCall& c, const GemvShape& s) {
  return c.vl == 4 ? run_vq_bits_vl<ACT, 4>(c, s) : run_vq_bits_vl<ACT, 8>(c, s);
}

template <int ACT, int BM_, int BR_>
int run_rvq(const VqCall& c, const GemvShape& s) {
  using P = RvqProvider<ACT, BM_, BR_>;
  typename P::Args a{c.packed, c.packed_r, (const u32x4*)c.cb, (const u32x4*)c.cb_r,
                     (const uint16_t*)c.row_scale, (const uint16_t*)c.row_bias,
                     (uint32_t)c.nc - 1u, (uint32_t)c.nc_r - 1u, s.chunks};
  return launch_fused_gemv<ACT, P>(s, a, c.st, c.what, c.nc_r * 16);
}

template <int ACT>
int dispatch(const VqCall& c) {
  GemvShape s{c.x, c.ldx, c.bias, c.y, c.ldy, c.M, c.N, c.K / 64, 0, 0};
  if (c.perm) {
    // The gather is done while x is copied to LDS, which only the MFMA kernel for plain VQ does.
    if (!(fast_ok(c) && !c.packed_r && c.M <= 16 && (int64_t)c.M * c.K <= kGemvLdsActivationsMax && aligned(c.perm, 16)))
      return fail(NPAMD_ERR_UNSUPPORTED,
                  "%s: column_perm needs VL = 8 or 4, 4/8/12/16-bit indices, K %% 64 == 0, 16-byte aligned "
                  "buffers, M <= 16 and M * K <= %d (got M=%d K=%d)", c.what, kGemvLdsActivationsMax, c.M, c.K);
    s.perm = c.perm;
  }
  if (fast_ok(c)) {
    if (!c.packed_r) return run_vq_bits<ACT>(c, s);
    const bool res_ok = aligned(c.packed_r, 16) && aligned(c.cb_r, 16);
    if (res_ok && c.bits == 16 && c.bits_r == 8) return run_rvq<ACT, 16, 8>(c, s);
    if (res_ok && c.bits == 16 && c.bits_r == 16) return run_rvq<ACT, 16, 16>(c, s);
    if (res_ok && c.bits == 12 && c.bits_r == 8) return run_rvq<ACT, 12, 8>(c, s);
    if (res_ok && c.bits == 8 && c.bits_r == 8) return run_rvq<ACT, 8, 8>(c, s);
  }
  return launch_generic_gemv<ACT>(c.x, c.ldx, c.bias, c.y, c.ldy, c.M, c.N, c.K, make_elem(c), c.st, c.what);
}

int run(const VqCall& c) {
  const int rc = validate(c, NPAMD_GEMV_MAX_M);
  if (rc < 0) return rc;
  if (rc == 1) return NPAMD_OK;
  return c.act == NPAMD_BF16 ? dispatch<NPAMD_BF16>(c) : dispatch<NPAMD_F16>(c);
}

}  // namespace

extern "C" int npamd_vq_gemv(const void* x, int64_t ldx, const uint8_t* packed, int64_t n_bytes,
                             int bits, const void* codebook, int codebook_dtype, int nc, int vl,
                             const float* bias, void* y, int64_t ldy, int M, int N, int K,
                             int act_dtype, void* stream) {
  VqCall c{x, ldx, packed, n_bytes, bits, codebook, codebook_dtype, nc, vl,
               nullptr, 0, 0, nullptr, 0, nullptr, nullptr,
               bias, y, ldy, M, N, K, act_dtype, (hipStream_t)stream, "npamd_vq_gemv"};
  return run(c);
}

extern "C" int npamd_vq_gemv_perm(const void* x, int64_t ldx, const int32_t* column_perm,
                                  const uint8_t* packed, int64_t n_bytes, int bits,
                                  const void* codebook, int codebook_dtype, int nc, int vl,
                                  const float* bias, void* y, int64_t ldy, int M, int N, int K,
                                  int act_dtype, void* stream) {
  VqCall c{x, ldx, packed, n_bytes, bits, codebook, codebook_dtype, nc, vl,
               nullptr, 0, 0, nullptr, 0, nullptr, nullptr,
               bias, y, ldy, M, N, K, act_dtype, (hipStream_t)stream, "npamd_vq_gemv_perm"};
  c.perm = column_perm;
  return run(c);
}

extern "C" int npamd_vq_fused_supported(int K, int vl, int bits) {
  const bool bits_ok = bits == 4 || bits == 8 || bits == 12 || bits == 16;
  return (vl == 8 || vl == 4) && bits_ok && K > 0 && K % 64 == 0 ? 1 : 0;
}

extern "C" int npamd_vq_gemv_perm_supported(int M, int N, int K, int nc, int vl, int bits) {
  const bool bits_ok = bits == 4 || bits == 8 || bits == 12 || bits == 16;
  if (!((vl == 8 || vl == 4) && bits_ok && K > 0 && K % 64 == 0 && M >= 1 && M <= 16 && N >= 1 && nc >= 1)) return 0;
  if ((int64_t)M * K > kGemvLdsActivationsMax) return 0;
  return gemv_perm_keeps_occupancy(M, N, K / 64, vl == 8 ? nc * 16 : (nc % 2 == 0 ? nc * 8 : 0)) ? 1 : 0;
}

extern "C" int npamd_rvq_gemv(const void* x, int64_t ldx,
                              const uint8_t* packed_main, int64_t n_bytes_main, int bits_main,
                              const uint8_t* packed_res, int64_t n_bytes_res, int bits_res,
                              const void* cb_main_f16, int nc_main, const void* cb_res_f16, int nc_res,
                              const void* row_scale_f16, const void* row_bias_f16, int vl,
                              const float* bias, void* y, int64_t ldy, int M, int N, int K,
                              int act_dtype, void* stream) {
  if (!packed_res) return fail(NPAMD_ERR_INVALID, "npamd_rvq_gemv: residual stream is null");
  VqCall c{x, ldx, packed_main, n_bytes_main, bits_main, cb_main_f16, NPAMD_F16, nc_main, vl,
               packed_res, n_bytes_res, bits_res, cb_res_f16, nc_res, row_scale_f16, row_bias_f16,
               bias, y, ldy, M, N, K, act_dtype, (hipStream_t)stream, "npamd_rvq_gemv"};
  return run(c);
}
