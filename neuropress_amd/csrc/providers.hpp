// Weight-operand providers for the fused kernels.
//
// The fused GEMV and the tile GEMM never see a dense weight.  Each lane owns a
// "chunk": 64 consecutive k of one weight row n, i.e. eight MFMA B-operands of
// eight 16-bit values.  A provider turns the packed bytes of that chunk into
// those operands:
//
//   load(raw, n, kc)   -- global loads of the packed chunk kc of row n
//   operand<j>(raw)    -- B-operand j (k = 64*kc + 8*j .. +7) in the activation dtype
//
// Both are branch-free: the caller passes in-range (clamped) coordinates and
// discards or zeroes what it does not need.  A predicated load would put every
// gather behind its own branch and its own wait, serialising them.
//
// The tile GEMM splits a chunk four ways: lane-group jp (0..3) of a producer
// wave owns operands 2*jp and 2*jp+1 of its column:
//
//   load_pair(raw, n, kc, jp)     -- packed bytes for that operand pair
//   gather_pair(raw, jp, ops)     -- issues the lookups (or dequantizes) for the two operands
//   finish_pair(ops, b0, b1)      -- the two operands, once the producer is about to write them
//   prepare_row(n)                -- once per producer lane: what its row needs besides packed bytes
//
// A B-operand of a VQ weight with VL = 8 is exactly one codebook row, so the
// 16-byte gather lands in MFMA layout with no shuffling (VL = 4: two rows, two 8-byte gathers).  For int4 the eight
// nibbles of one dword are one operand, for int8 eight bytes.
#pragma once

#include "common.hpp"

namespace npamd {

// Dword jp (lane-varying, 0..3) of a four-dword vector.
__device__ __forceinline__ uint32_t select_dword(const u32x4& v, int jp) {
  const uint32_t lo = (jp & 1) ? v.y : v.x;
  const uint32_t hi = (jp & 1) ? v.w : v.z;
  return (jp & 2) ? hi : lo;
}

// ---------------------------------------------------------------------------
// Single-codebook VQ, fast index widths, VL = 8 or 4.
//   CONV : codebook is fp16 but activations are bf16 -> convert per gather.
// VL = 8: a codebook row is one operand (one 16-byte gather).  VL = 4 (the reference's default
// vector length): an operand is two rows, two 8-byte gathers; a 64-k chunk holds 16 indices.
// ---------------------------------------------------------------------------
template <int ACT, int BITS, bool CONV, int VL = 8>
struct VqProvider {
  static_assert(VL == 8 || VL == 4, "vector length 8 or 4");
  static constexpr int kIdxPerChunk = 64 / VL;
  struct Args {
    const uint8_t* packed;
    const u32x4* cb;   // VL = 4: rows of 8 bytes behind this pointer
    uint32_t nc_minus_1;
    int chunks;  // K / 64
  };
  struct Raw {
    u32x4 idx;     // indices 0..7 of the chunk, 16 bits each
    u32x4 idx_hi;  // indices 8..15 (VL = 4 only)
  };
  static constexpr bool kLdsCodebook = true;  // the codebook may be staged in LDS (use_codebook)
  static constexpr bool kLdsResidual = false;
  static constexpr bool kGathers = true;  // operands are codebook lookups, not arithmetic on the packed bytes
  const Args& a;
  const u32x4* cb;  // where operands are gathered from: global memory, or an LDS copy
  __device__ explicit VqProvider(const Args& args) : a(args), cb(args.cb) {}
  __device__ __forceinline__ void use_codebook(const u32x4* p) { cb = p; }
  __device__ __forceinline__ const u32x4* global_codebook() const { return a.cb; }
  // Size of the table in 16-byte units (VL = 4: callers stage it in LDS only when it has an even number of rows).
  __device__ __forceinline__ int codebook_vec16() const {
    return VL == 8 ? (int)a.nc_minus_1 + 1 : ((int)a.nc_minus_1 + 1) / 2;
  }

  __device__ __forceinline__ u32x4 row_pair(uint32_t i0, uint32_t i1) const {  // VL = 4: two rows = one operand
    const u32x2* c2 = reinterpret_cast<const u32x2*>(cb);
    const u32x2 lo = c2[min(i0, a.nc_minus_1)], hi = c2[min(i1, a.nc_minus_1)];
    return u32x4{lo.x, lo.y, hi.x, hi.y};
  }

  __device__ __forceinline__ void load(Raw& r, int n, int kc) const {
    const int64_t i0 = ((int64_t)n * a.chunks + kc) * kIdxPerChunk;
    r.idx = load_idx8<BITS>(a.packed, i0);
    if constexpr (VL == 4) r.idx_hi = load_idx8<BITS>(a.packed, i0 + 8);
  }
  template <int J>
  __device__ __forceinline__ u32x4 operand(const Raw& r) const {
    u32x4 c;
    if constexpr (VL == 8) {
      c = cb[min(idx8_get(r.idx, J), a.nc_minus_1)];
    } else {
      const u32x4& v = (J < 4) ? r.idx : r.idx_hi;
      c = row_pair(idx8_get(v, (2 * J) % 8), idx8_get(v, (2 * J + 1) % 8));
    }
    if constexpr (CONV) c = cb_to_act<ACT>(c);
    return c;
  }

  // The tile GEMM's producers request packed bytes sixteen steps ahead: PairRaw holds what the
  // load returned, untouched, and gather_pair extracts the indices when it looks them up.
  __device__ __forceinline__ void prepare_row(int) {}  // nothing per row outside the packed bytes
  struct PairRaw {
    u32x4 w;  // the 8-index group that holds this lane's operands, as loaded
  };
  __device__ __forceinline__ void load_pair(PairRaw& r, int n, int kc, int jp) const {
    const int64_t i0 = ((int64_t)n * a.chunks + kc) * kIdxPerChunk;
    // VL = 8: the four lane-groups of a column read the same 8-index group: one request.
    // VL = 4: operands 2jp, 2jp+1 = indices 4jp .. 4jp+3, half of index group jp >> 1.
    r.w = load_raw8<BITS>(a.packed, VL == 8 ? i0 : i0 + 8 * (jp >> 1));
  }
  // gather_pair only issues the lookups; what they return stays untouched in PairOps until the
  // producer writes the pair, many steps later, and finish_pair converts it then.  Arithmetic
  // on the looked-up rows next to the lookup would make the wave wait for it on the spot.
  struct PairOps {
    u32x4 b0, b1;
  };
  static constexpr int kLdsOpsPerGather = VL == 8 ? 2 : 4;  // LDS reads of one gather_pair from an LDS codebook
  // `live` false (a step past the end, issued to keep the pipeline free of branches): every lane looks up
  // row 0, one cache line per instruction instead of up to 64.
  __device__ __forceinline__ void gather_pair(const PairRaw& r, int jp, PairOps& o, bool live = true) const {
    const u32x4 v = extract_idx8<BITS>(r.w);
    if constexpr (VL == 8) {
      const uint32_t lim = live ? a.nc_minus_1 : 0u;
      const uint32_t pair = select_dword(v, jp);  // indices of operands 2*jp (low half) and 2*jp+1
      o.b0 = cb[min(pair & 0xFFFFu, lim)];
      o.b1 = cb[min(pair >> 16, lim)];
    } else {
      const uint32_t pair = (jp & 1) ? v.z : v.x;   // the two rows of operand 2*jp
      const uint32_t pair1 = (jp & 1) ? v.w : v.y;  // those of operand 2*jp+1
      o.b0 = row_pair(pair & 0xFFFFu, pair >> 16);
      o.b1 = row_pair(pair1 & 0xFFFFu, pair1 >> 16);
    }
  }
  __device__ __forceinline__ void finish_pair(const PairOps& o, u32x4& b0, u32x4& b1) const {
    b0 = CONV ? cb_to_act<ACT>(o.b0) : o.b0;
    b1 = CONV ? cb_to_act<ACT>(o.b1) : o.b1;
  }
};

// ---------------------------------------------------------------------------
// Residual VQ: main + residual codebook (fp16), per-row fp16 scale and bias.
//   w = f16(f16(f16(cm + cr) * s) + b), each op rounded separately.
// ---------------------------------------------------------------------------
template <int ACT, int BITS_M, int BITS_R>
struct RvqProvider {
  struct Args {
    const uint8_t* packed_m;
    const uint8_t* packed_r;
    const u32x4* cb_m;
    const u32x4* cb_r;
    const uint16_t* row_scale;  // may be null
    const uint16_t* row_bias;   // may be null
    uint32_t ncm_minus_1, ncr_minus_1;
    int chunks;
  };
  struct Raw {
    u32x4 im, ir;
    uint32_t s2, b2;  // scale / bias replicated in both halves
  };
  static constexpr bool kLdsCodebook = false;
  // The GEMV can keep the residual codebook (4 KiB at 256 rows) in LDS: lookups through the
  // vector memory path cost one cache-tag cycle per lane whether they hit or not, and the
  // residual's are half of them.  The main codebook stays in memory.
  static constexpr bool kLdsResidual = true;
  static constexpr bool kGathers = true;  // operands are codebook lookups, not arithmetic on the packed bytes
  const Args& a;
  const u32x4* cbr;  // where residual rows are looked up: global memory, or an LDS copy
  __device__ explicit RvqProvider(const Args& args) : a(args), cbr(args.cb_r) {}
  __device__ __forceinline__ void use_codebook(const u32x4* p) { cbr = p; }
  __device__ __forceinline__ const u32x4* global_codebook() const { return a.cb_r; }
  __device__ __forceinline__ int codebook_vec16() const { return (int)a.ncr_minus_1 + 1; }

  __device__ __forceinline__ void load(Raw& r, int n, int kc) const {
    const int64_t i0 = ((int64_t)n * a.chunks + kc) * 8;
    r.im = load_idx8<BITS_M>(a.packed_m, i0);
    r.ir = load_idx8<BITS_R>(a.packed_r, i0);
    r.s2 = 0x3C003C00u;  // 1.0, 1.0
    r.b2 = 0u;
    if (a.row_scale) r.s2 = (uint32_t)a.row_scale[n] * 0x10001u;  // uniform branches
    if (a.row_bias) r.b2 = (uint32_t)a.row_bias[n] * 0x10001u;
  }
  template <int J>
  __device__ __forceinline__ u32x4 operand(const Raw& r) const {
    return combine(idx8_get(r.im, J), idx8_get(r.ir, J), r.s2, r.b2);
  }

  // As loaded (see VqProvider::PairRaw); the row's scale and bias do not change from step to
  // step, so the producer reads them once (prepare_row) instead of with every pair.
  struct PairRaw {
    u32x4 wm, wr;
  };
  uint32_t s2 = 0x3C003C00u, b2 = 0u;  // scale (1.0) and bias of the producer lane's row, replicated pairs
  __device__ __forceinline__ void prepare_row(int n) {
    if (a.row_scale) s2 = (uint32_t)a.row_scale[n] * 0x10001u;
    if (a.row_bias) b2 = (uint32_t)a.row_bias[n] * 0x10001u;
  }
  __device__ __forceinline__ void load_pair(PairRaw& r, int n, int kc, int jp) const {
    const int64_t i0 = ((int64_t)n * a.chunks + kc) * 8;
    r.wm = load_raw8<BITS_M>(a.packed_m, i0);
    r.wr = load_raw8<BITS_R>(a.packed_r, i0);
  }
  struct PairOps {
    u32x4 cm0, cr0, cm1, cr1;  // main and residual rows of the two operands, as gathered
  };
  static constexpr int kLdsOpsPerGather = 2;  // with the residual codebook in LDS: its two lookups
  __device__ __forceinline__ void gather_pair(const PairRaw& r, int jp, PairOps& o, bool live = true) const {
    const uint32_t pm = select_dword(extract_idx8<BITS_M>(r.wm), jp);
    const uint32_t pr = select_dword(extract_idx8<BITS_R>(r.wr), jp);
    const uint32_t lim_m = live ? a.ncm_minus_1 : 0u, lim_r = live ? a.ncr_minus_1 : 0u;  // see VqProvider::gather_pair
    o.cm0 = a.cb_m[min(pm & 0xFFFFu, lim_m)];
    o.cm1 = a.cb_m[min(pm >> 16, lim_m)];
    o.cr0 = cbr[min(pr & 0xFFFFu, lim_r)];
    o.cr1 = cbr[min(pr >> 16, lim_r)];
  }
  __device__ __forceinline__ void finish_pair(const PairOps& o, u32x4& b0, u32x4& b1) const {
    b0 = combine_rows(o.cm0, o.cr0, s2, b2);
    b1 = combine_rows(o.cm1, o.cr1, s2, b2);
  }

  __device__ __forceinline__ u32x4 combine(uint32_t im, uint32_t ir, uint32_t s2, uint32_t b2) const {
    return combine_rows(a.cb_m[min(im, a.ncm_minus_1)], cbr[min(ir, a.ncr_minus_1)], s2, b2);
  }
  __device__ __forceinline__ u32x4 combine_rows(const u32x4& cm, const u32x4& cr, uint32_t s2, uint32_t b2) const {
#pragma clang fp contract(off)
    const f16x2 s = __builtin_bit_cast(f16x2, s2);
    const f16x2 b = __builtin_bit_cast(f16x2, b2);
    const bool has_s = a.row_scale != nullptr, has_b = a.row_bias != nullptr;
    uint32_t o[4];
    const uint32_t m4[4] = {cm.x, cm.y, cm.z, cm.w};
    const uint32_t r4[4] = {cr.x, cr.y, cr.z, cr.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f16x2 h = __builtin_bit_cast(f16x2, m4[i]) + __builtin_bit_cast(f16x2, r4[i]);
      if (has_s) h = h * s;
      if (has_b) h = h + b;
      o[i] = __builtin_bit_cast(uint32_t, h);
    }
    return cb_to_act<ACT>(u32x4{o[0], o[1], o[2], o[3]});
  }
};

// ---------------------------------------------------------------------------
// int4, group size a multiple of 32; symmetric (zero point 8) or, with ASYM, a
// per-group fp16 zero point.
// One dword of nibbles = one operand, in natural k order: byte i of the dword (nibbles 2i and
// 2i+1) is copied under both halves of a pair (v_perm_b32); masked with 0x00F0000F and or-ed
// with 0x54006400, the low half reads as fp16 1024 + q[2i] (nibble in mantissa bits 0..3 of
// 0x6400) and the high half as 64 + q[2i+1] (bits 4..7 of 0x5400), both exact.
// Symmetric f16: minus (1032, 72) -> q - 8 exactly, times the scale -- exact product, one
// rounding: the oracle's weight.
// Otherwise w = round((f32(q) - f32(zp)) * f32(s)), the difference exact, the product
// rounded to f32 and then to the activation type, operation for operation as the
// element-wise decode does it.
// ---------------------------------------------------------------------------
template <int ACT, bool ASYM = false>
struct Q4Provider {
  struct Args {
    const uint8_t* w_pack;   // [N, K/2]
    const uint16_t* scale;   // [N, K/gs]
    int chunks;              // K / 64
    int groups_per_row;      // K / gs
    int gs_shift_chunks;     // log2(gs/32): scale index = (2*kc + half) >> gs_shift_chunks
    const uint16_t* zp;      // [N, K/gs] (ASYM only)
  };
  struct Raw {
    u32x4 w0, w1;
    uint32_t s_lo, s_hi;  // scale (replicated pair) for operands 0-3 and 4-7
    uint32_t z_lo, z_hi;  // zero points (fp16 bits) of the same two groups (ASYM only)
  };
  static constexpr bool kLdsCodebook = false;
  static constexpr bool kLdsResidual = false;
  static constexpr bool kGathers = false;  // operands are codebook lookups, not arithmetic on the packed bytes
  const Args& a;
  __device__ explicit Q4Provider(const Args& args) : a(args) {}

  __device__ __forceinline__ void load(Raw& r, int n, int kc) const {
    const u32x4* p = reinterpret_cast<const u32x4*>(a.w_pack + ((int64_t)n * a.chunks + kc) * 32);
    r.w0 = p[0];
    r.w1 = p[1];
    const int64_t row = (int64_t)n * a.groups_per_row;
    const int g_lo = (2 * kc) >> a.gs_shift_chunks, g_hi = (2 * kc + 1) >> a.gs_shift_chunks;
    r.s_lo = (uint32_t)a.scale[row + g_lo] * 0x10001u;
    r.s_hi = (uint32_t)a.scale[row + g_hi] * 0x10001u;
    if constexpr (ASYM) {
      r.z_lo = a.zp[row + g_lo];
      r.z_hi = a.zp[row + g_hi];
    }
  }
  template <int J>
  __device__ __forceinline__ u32x4 operand(const Raw& r) const {
    const u32x4& ww = (J < 4) ? r.w0 : r.w1;
    const uint32_t w = (J % 4 == 0) ? ww.x : (J % 4 == 1) ? ww.y : (J % 4 == 2) ? ww.z : ww.w;
    return dequant8(w, (J < 4) ? r.s_lo : r.s_hi, (J < 4) ? r.z_lo : r.z_hi);
  }

  __device__ __forceinline__ void prepare_row(int) {}  // nothing per row outside the packed bytes
  struct PairRaw {
    u32x2 w;      // 16 nibbles = operands 2*jp, 2*jp+1
    uint32_t s2;  // their scale (one 32-k group), replicated
    uint32_t z;   // their zero point, fp16 bits (ASYM only)
  };
  __device__ __forceinline__ void load_pair(PairRaw& r, int n, int kc, int jp) const {
    r.w = *reinterpret_cast<const u32x2*>(a.w_pack + ((int64_t)n * a.chunks + kc) * 32 + jp * 8);
    const int64_t g = (int64_t)n * a.groups_per_row + ((2 * kc + (jp >> 1)) >> a.gs_shift_chunks);
    r.s2 = (uint32_t)a.scale[g] * 0x10001u;
    if constexpr (ASYM) r.z = a.zp[g];
  }
  struct PairOps {
    u32x4 b0, b1;  // finished operands: the dequantization waits for nothing but the packed bytes
  };
  static constexpr int kLdsOpsPerGather = 0;
  __device__ __forceinline__ void gather_pair(const PairRaw& r, int, PairOps& o, bool = true) const {
    o.b0 = dequant8(r.w.x, r.s2, r.z);
    o.b1 = dequant8(r.w.y, r.s2, r.z);
  }
  __device__ __forceinline__ void finish_pair(const PairOps& o, u32x4& b0, u32x4& b1) const {
    b0 = o.b0;
    b1 = o.b1;
  }

  // Eight nibbles of one dword -> one operand, natural k order.
  __device__ __forceinline__ u32x4 dequant8(uint32_t w, uint32_t s2, uint32_t z) const {
#pragma clang fp contract(off)
    uint32_t o[4];
    const float sf = f16_bits_to_f32(s2 & 0xFFFFu);
    const float zf = ASYM ? f16_bits_to_f32(z & 0xFFFFu) : 0.f;
    // byte i of w into bytes 0 and 2 (bytes 1 and 3: zero)
    const uint32_t spread[4] = {__builtin_amdgcn_perm(0u, w, 0x0c000c00u), __builtin_amdgcn_perm(0u, w, 0x0c010c01u),
                                __builtin_amdgcn_perm(0u, w, 0x0c020c02u), __builtin_amdgcn_perm(0u, w, 0x0c030c03u)};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t pair = (spread[i] & 0x00F0000Fu) | 0x54006400u;  // (1024 + q[2i], 64 + q[2i+1])
      if constexpr (ACT == NPAMD_F16 && !ASYM) {
        // minus (1032, 72) -> q - 8 exactly; times the scale: one rounding.
        const f16x2 q = __builtin_bit_cast(f16x2, pair) - __builtin_bit_cast(f16x2, 0x54806408u);
        o[i] = __builtin_bit_cast(uint32_t, q * __builtin_bit_cast(f16x2, s2));
      } else {
        // q (ASYM) or q - 8 exactly, in fp16; the rest in f32.
        const f16x2 q = __builtin_bit_cast(f16x2, pair) - __builtin_bit_cast(f16x2, ASYM ? 0x54006400u : 0x54806408u);
        float lo = (float)q.x, hi = (float)q.y;
        if constexpr (ASYM) {
          lo -= zf;
          hi -= zf;
        }
        lo *= sf;
        hi *= sf;
        if constexpr (ACT == NPAMD_F16) {
          f16x2 h;
          h.x = (_Float16)lo;
          h.y = (_Float16)hi;
          o[i] = __builtin_bit_cast(uint32_t, h);
        } else {
          bf16x2 b;
          b.x = (__bf16)lo;
          b.y = (__bf16)hi;
          o[i] = __builtin_bit_cast(uint32_t, b);
        }
      }
    }
    return u32x4{o[0], o[1], o[2], o[3]};
  }
};

// ---------------------------------------------------------------------------
// int8, group size a multiple of 32; symmetric (zero point 128) or, with ASYM, a per-group
// fp16 zero point.  Eight bytes = one operand, in natural k order (no A permutation).
// A byte b placed under the exponent byte 0x64 reads as fp16 1024 + b exactly (v_perm_b32,
// two weights per instruction).  Symmetric f16: minus 1152 -> q - 128 exactly, times the
// scale: one rounding of an exact product, the oracle's weight.  Otherwise as Q4Provider:
// difference and product in f32, then rounded to the activation type.
// ---------------------------------------------------------------------------
template <int ACT, bool ASYM = false>
struct Q8Provider {
  struct Args {
    const uint8_t* w_pack;   // [N, K]
    const uint16_t* scale;   // [N, K/gs]
    int chunks;              // K / 64
    int groups_per_row;      // K / gs
    int gs_shift_chunks;     // log2(gs/32)
    const uint16_t* zp;      // [N, K/gs] (ASYM only)
  };
  struct Raw {
    u32x4 w[4];           // 64 bytes = operands 0..7
    uint32_t s_lo, s_hi;  // scale (replicated pair) for operands 0-3 and 4-7
    uint32_t z_lo, z_hi;  // zero points (fp16 bits), ASYM only
  };
  static constexpr bool kLdsCodebook = false;
  static constexpr bool kLdsResidual = false;
  static constexpr bool kGathers = false;  // operands are arithmetic on the packed bytes
  const Args& a;
  __device__ explicit Q8Provider(const Args& args) : a(args) {}

  __device__ __forceinline__ void load(Raw& r, int n, int kc) const {
    const u32x4* p = reinterpret_cast<const u32x4*>(a.w_pack + ((int64_t)n * a.chunks + kc) * 64);
#pragma unroll
    for (int i = 0; i < 4; ++i) r.w[i] = p[i];
    const int64_t row = (int64_t)n * a.groups_per_row;
    const int g_lo = (2 * kc) >> a.gs_shift_chunks, g_hi = (2 * kc + 1) >> a.gs_shift_chunks;
    r.s_lo = (uint32_t)a.scale[row + g_lo] * 0x10001u;
    r.s_hi = (uint32_t)a.scale[row + g_hi] * 0x10001u;
    if constexpr (ASYM) {
      r.z_lo = a.zp[row + g_lo];
      r.z_hi = a.zp[row + g_hi];
    }
  }
  template <int J>
  __device__ __forceinline__ u32x4 operand(const Raw& r) const {
    const u32x4& ww = r.w[J / 2];
    return dequant8((J & 1) ? ww.z : ww.x, (J & 1) ? ww.w : ww.y, (J < 4) ? r.s_lo : r.s_hi, (J < 4) ? r.z_lo : r.z_hi);
  }

  __device__ __forceinline__ void prepare_row(int) {}  // nothing per row outside the packed bytes
  struct PairRaw {
    u32x4 w;      // 16 bytes = operands 2*jp, 2*jp+1
    uint32_t s2;  // their scale (one 32-k group), replicated
    uint32_t z;   // their zero point, fp16 bits (ASYM only)
  };
  __device__ __forceinline__ void load_pair(PairRaw& r, int n, int kc, int jp) const {
    r.w = *reinterpret_cast<const u32x4*>(a.w_pack + ((int64_t)n * a.chunks + kc) * 64 + jp * 16);
    const int64_t g = (int64_t)n * a.groups_per_row + ((2 * kc + (jp >> 1)) >> a.gs_shift_chunks);
    r.s2 = (uint32_t)a.scale[g] * 0x10001u;
    if constexpr (ASYM) r.z = a.zp[g];
  }
  struct PairOps {
    u32x4 b0, b1;  // finished operands
  };
  static constexpr int kLdsOpsPerGather = 0;
  __device__ __forceinline__ void gather_pair(const PairRaw& r, int, PairOps& o, bool = true) const {
    o.b0 = dequant8(r.w.x, r.w.y, r.s2, r.z);
    o.b1 = dequant8(r.w.z, r.w.w, r.s2, r.z);
  }
  __device__ __forceinline__ void finish_pair(const PairOps& o, u32x4& b0, u32x4& b1) const {
    b0 = o.b0;
    b1 = o.b1;
  }

  // Eight bytes (two dwords) -> one operand.
  __device__ __forceinline__ u32x4 dequant8(uint32_t d0, uint32_t d1, uint32_t s2, uint32_t z) const {
#pragma clang fp contract(off)
    const float sf = f16_bits_to_f32(s2 & 0xFFFFu);
    const float zf = ASYM ? f16_bits_to_f32(z & 0xFFFFu) : 0.f;
    const uint32_t pairs[4] = {__builtin_amdgcn_perm(0x64646464u, d0, 0x04010400u),   // (1024 + b0, 1024 + b1)
                               __builtin_amdgcn_perm(0x64646464u, d0, 0x04030402u),   // (1024 + b2, 1024 + b3)
                               __builtin_amdgcn_perm(0x64646464u, d1, 0x04010400u),
                               __builtin_amdgcn_perm(0x64646464u, d1, 0x04030402u)};
    uint32_t o[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if constexpr (ACT == NPAMD_F16 && !ASYM) {
        const f16x2 q = __builtin_bit_cast(f16x2, pairs[i]) - __builtin_bit_cast(f16x2, 0x64806480u);  // 1152
        o[i] = __builtin_bit_cast(uint32_t, q * __builtin_bit_cast(f16x2, s2));
      } else {
        const f16x2 q = __builtin_bit_cast(f16x2, pairs[i]) - __builtin_bit_cast(f16x2, ASYM ? 0x64006400u : 0x64806480u);
        float lo = (float)q.x, hi = (float)q.y;
        if constexpr (ASYM) {
          lo -= zf;
          hi -= zf;
        }
        lo *= sf;
        hi *= sf;
        if constexpr (ACT == NPAMD_F16) {
          f16x2 h;
          h.x = (_Float16)lo;
          h.y = (_Float16)hi;
          o[i] = __builtin_bit_cast(uint32_t, h);
        } else {
          bf16x2 b;
          b.x = (__bf16)lo;
          b.y = (__bf16)hi;
          o[i] = __builtin_bit_cast(uint32_t, b);
        }
      }
    }
    return u32x4{o[0], o[1], o[2], o[3]};
  }
};

// Eight 16-bit values reordered (0,4,1,5,2,6,3,7): the (k, k+4) pair order in which the row-wise
// int4 GEMV stages its activations.
__device__ __forceinline__ u32x4 permute_a_0415(u32x4 x) {
  u32x4 r;
  r.x = (x.x & 0xFFFFu) | (x.z << 16);
  r.y = (x.x >> 16) | (x.z & 0xFFFF0000u);
  r.z = (x.y & 0xFFFFu) | (x.w << 16);
  r.w = (x.y >> 16) | (x.w & 0xFFFF0000u);
  return r;
}

}  // namespace npamd
