// Fused decode GEMV for small token counts (M <= 32), wave64 + MFMA 16x16x32.
//
// The contraction y[m, n] = sum_k x[m, k] * W[n, k] is issued as
// D[16 x 16] += A[16 x 32] * B[32 x 16] with A = x (rows m, zero beyond M) and
// B = W^T (columns n).  Lane l = (c = l % 16, q = l / 16) supplies
//   A: x[m = c][8 consecutive k of k-slot q]      (16 bytes, zero if c >= M)
//   B: W[n = n0 + c][the same 8 k]                (16 bytes = one VQ codebook row)
// so a gathered codebook row is already a B-operand: no LDS, no VALU work on
// the weights, and M = 1 ... 16 all cost the same (17 ... 32 tokens: two token
// tiles, each weight operand feeds two MFMAs).  The kernel is bound by the
// packed-weight stream from HBM plus, for codebooks larger than L1, the
// 16-byte gathers out of L2.
//
// Work split: a "chunk" is 64 k of one row (8 operands); one "step" is the 4
// k-slots of a wave = 256 k.  A block owns 16*R rows and all of K; its S waves
// split the steps and their partial tiles are summed through LDS.  (Layers of
// few rows: 16 / H rows per block and H parts of k per k-slot, see the kernel.)
#pragma once

#include <atomic>

#include "providers.hpp"

namespace npamd {

struct GemvShape {
  const void* x;
  int64_t ldx;
  const float* bias;
  void* y;
  int64_t ldy;
  int M, N;
  int chunks;          // K / 64 (K % 64 == 0 is a precondition of this kernel)
  int steps;           // ceil(chunks / 4)
  int steps_per_wave;  // steps each wave of the block covers
  // Optional gather of the activation columns: the kernel contracts x[m, perm[k]] with W[n, k].
  // Only with the X_LDS variant (every block first copies the permuted rows of x into LDS).
  const int32_t* perm = nullptr;
  int stage_offset = 0;  // XS kernels: byte offset of the waves' activation staging areas in LDS
  // Planning only: when set, the launcher writes here whether the kernel it chose stages its
  // activations (1 / 0) and launches nothing.
  int* plan_only = nullptr;
};

// Largest M * K (elements) whose activations the GEMV stages in LDS (32 KiB; the unpermuted
// copy shares its place with the codebook of up to 64 KiB).
constexpr int kGemvLdsActivationsMax = 16 * 1024;

// R = 4 keeps 32 gathered operands (128 registers) live per lane, so it is
// limited to 8 waves per block; R <= 2 fits the 128-register budget of 16 waves.
// MT = 2 (17..32 tokens: two MFMA row tiles of tokens share every weight operand) holds a
// second set of eight x operands and accumulators: 8 waves at up to 256 registers.
template <int R, int MT = 1>
constexpr int kGemvMaxWaves = (R >= 4 || MT >= 2) ? 8 : 16;

// CB_LDS: the block first copies the whole codebook into LDS and gathers from
// there (ds_read_b128) instead of from L1/L2.  Pays off when the table is too
// big for L1 (> 32 KiB) yet fits LDS, or is so small that the copy is free.
// X_LDS: the block also copies x (all M rows, all of K) into LDS, applying the
// column permutation s.perm on the way when there is one, and reads its A
// operands from there: the gather x[m, perm[k]] costs K element loads per block
// instead of a kernel of its own in front of this one.
// H > 1 (layers of few rows, at most 16 / H tokens): the 16 columns of the MFMA tile are 16 / H
// weight rows x H parts of k, and A carries the matching part of x in the row of the same
// number, so D[m'][n'] is a wanted partial sum where m' and n' name the same part and is
// ignored elsewhere.  A block then owns 16 / H rows: H times the blocks, each with 1 / H of the
// lookups, for layers that would leave most compute units without a block.
// XS (one row tile per block, from three tokens): a step's activations -- the tile's tokens x
// 256 * H k -- are loaded 1 KiB of contiguous row bytes per instruction, parked in an LDS area of
// the wave's own (GemvStage) and read back in operand layout.  Straight from memory every x load
// instruction touches 64 cache lines at 16 tokens (a lane's 16 bytes lie in a line only the
// lanes of its token and k-slot share), eight times per step, and with one row tile nothing
// shares that cost.
// Staging layout of one wave: [token][chunk of the step][128 bytes], H parts: 4 * H chunks per
// token.  Chunk and row strides are padded so that the 16 lanes of a read pass (one k-slot: 16 / H
// tokens x H parts) fall into 16 different 16-byte bank groups: in units of 16 bytes the strides
// are (chunk, row) = (8, 33) for whole tiles, (8, 65) for two parts, (9, 148) for four.
template <int H>
struct GemvStage {
  static constexpr int kChunk = H == 4 ? 144 : 128;
  static constexpr int kRow = 4 * H * kChunk + (H == 4 ? 64 : 16);
  static constexpr int kRowData = 512 * H;      // bytes of one token's activations in a step
  static constexpr int kBytes = (16 / H) * kRow;  // per token tile
};
template <int ACT, class Provider, int R, bool CB_LDS, bool X_LDS, int MT = 1, int H = 1, bool XS = false>
__global__ void __launch_bounds__((kGemvMaxWaves<R, MT> * 64))
fused_gemv_kernel(const GemvShape s, const typename Provider::Args pargs) {
  static_assert(H == 1 || ((H == 2 || H == 4) && R == 1 && MT == 1), "k parts only with one row tile and one token tile");
  static_assert(!XS || (R == 1 && !X_LDS), "staged activations: one row tile, x not already in LDS");
  constexpr int RT = 16 / H;  // weight rows (and tokens) per MFMA tile
  extern __shared__ __attribute__((aligned(16))) float red[];  // [waves][M][16*R] (+ codebook copy)
  Provider prov(pargs);
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int n_waves = blockDim.x >> 6;
  // LDS after the reduction buffer (16-byte aligned): the codebook copy, then the copy of x.
  // While x is being permuted its unpermuted copy lies where the codebook goes afterwards, so
  // the region in front of x is max(codebook, x) bytes.
  const int red_floats = (n_waves * s.M * 16 * R + 3) & ~3;
  // Without a copy of x the reduction buffer, needed only after the loop, lies over the codebook.
  constexpr bool kRedOverCodebook = CB_LDS && !X_LDS;
  uint8_t* const lds0 = reinterpret_cast<uint8_t*>(red) + (kRedOverCodebook ? 0 : red_floats * (int)sizeof(float));
  int cb_lds_bytes = 0;
  if constexpr (CB_LDS) cb_lds_bytes = prov.codebook_vec16() * 16;
  const uint16_t* x_lds = nullptr;
  if constexpr (X_LDS) {
    // Rows of x: a coalesced copy into LDS, then (with a permutation) a second LDS buffer filled
    // by 2-byte LDS reads at the permuted columns -- element gathers are an order of magnitude
    // cheaper from LDS than through the vector memory path, and every block needs all of them.
    const int K = s.chunks * 64;
    const int k8s = s.chunks * 8;  // 8-element pieces per row
    const int items = s.M * k8s;
    const int x_bytes = s.M * K * 2;
    uint16_t* const xs = reinterpret_cast<uint16_t*>(lds0 + (s.perm ? max(cb_lds_bytes, x_bytes) : cb_lds_bytes));
    uint16_t* const xraw = s.perm ? reinterpret_cast<uint16_t*>(lds0) : xs;
    const uint16_t* xg = reinterpret_cast<const uint16_t*>(s.x);
    for (int i = threadIdx.x; i < items; i += blockDim.x) {
      const int m = i / k8s;
      const int k8 = i - m * k8s;
      *reinterpret_cast<u32x4*>(xraw + (int64_t)i * 8) =
          *reinterpret_cast<const u32x4*>(xg + (int64_t)m * s.ldx + k8 * 8);
    }
    if (s.perm) {
      __syncthreads();
      for (int i = threadIdx.x; i < items; i += blockDim.x) {
        const int m = i / k8s;
        const int k8 = i - m * k8s;
        const uint16_t* xr = xraw + (int64_t)m * K;
        const u32x4 p0 = *reinterpret_cast<const u32x4*>(s.perm + k8 * 8);
        const u32x4 p1 = *reinterpret_cast<const u32x4*>(s.perm + k8 * 8 + 4);
        u32x4 v;
        v.x = (uint32_t)xr[p0.x] | ((uint32_t)xr[p0.y] << 16);
        v.y = (uint32_t)xr[p0.z] | ((uint32_t)xr[p0.w] << 16);
        v.z = (uint32_t)xr[p1.x] | ((uint32_t)xr[p1.y] << 16);
        v.w = (uint32_t)xr[p1.z] | ((uint32_t)xr[p1.w] << 16);
        *reinterpret_cast<u32x4*>(xs + (int64_t)i * 8) = v;
      }
      if constexpr (CB_LDS) __syncthreads();  // the codebook overwrites the unpermuted copy
    }
    x_lds = xs;
  }
  if constexpr (CB_LDS) {
    // Four requests per thread in flight: a block of few waves (short K) would otherwise copy
    // the table one round trip per 16 bytes and thread.
    u32x4* cb_lds = reinterpret_cast<u32x4*>(lds0);
    const u32x4* src = prov.global_codebook();
    const int n16 = prov.codebook_vec16();
    constexpr int kBatch = 4;
    if ((n16 & 63) == 0) {
      // Whole KiB at a time, straight into LDS (M0 = destination, lane l writes at + 16 l): no
      // register, no LDS store instruction.  8192 x 2048 with a 4096-row table 5.13 -> 4.87 us at one
      // token, 14336 x 4096 8.1 -> 7.8, 2048 x 2048 at 16 tokens 5.9 -> 5.65; never slower.  The
      // statement writes m0, which an asm statement cannot declare as clobbered: sound while the
      // compiler keeps nothing of its own in m0 in this kernel (checked on the generated code).
      const uint32_t dst0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) u32x4*)cb_lds;
      for (int chunk = wave; chunk * 64 < n16; chunk += n_waves) {
        const uint32_t dst = __builtin_amdgcn_readfirstlane(dst0 + (uint32_t)chunk * 1024u);
        const uint32_t voff = (uint32_t)(chunk * 64 + lane) * 16u;
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(voff), "s"(src) : "memory");
      }
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    } else
    for (int base = threadIdx.x; base < n16; base += (int)blockDim.x * kBatch) {
      u32x4 t[kBatch];
#pragma unroll
      for (int j = 0; j < kBatch; ++j)
        if (base + j * (int)blockDim.x < n16) t[j] = src[base + j * (int)blockDim.x];
#pragma unroll
      for (int j = 0; j < kBatch; ++j)
        if (base + j * (int)blockDim.x < n16) cb_lds[base + j * (int)blockDim.x] = t[j];
    }
    prov.use_codebook(cb_lds);
  }
  if constexpr (CB_LDS || X_LDS) __syncthreads();
  const int c = lane & 15;
  const int q = lane >> 4;
  const int cr = c & (RT - 1), part = c / RT;  // H = 1: cr = c, part = 0
  const int row0 = blockIdx.x * (RT * R);

  f32x4 acc[R][MT];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[r][t] = f32x4{0.f, 0.f, 0.f, 0.f};

  const int step_begin = wave * s.steps_per_wave;
  const int step_end = min(step_begin + s.steps_per_wave, s.steps);
  // Loads are branch-free: out-of-range lanes read a clamped (valid) address and
  // their operand is zeroed afterwards, so all gathers of a step are in flight
  // together instead of each sitting behind its own branch and wait.
  const uint16_t* xrow[MT];
  bool x_lane[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int x_row = min(16 * t + cr, s.M - 1);
    xrow[t] = X_LDS ? x_lds + (int64_t)x_row * (s.chunks * 64)
                    : reinterpret_cast<const uint16_t*>(s.x) + (int64_t)x_row * s.ldx;
    x_lane[t] = 16 * t + cr < s.M;
  }
  const u32x4 zero4{0, 0, 0, 0};

  for (int step = step_begin; step < step_end; ++step) {
    const int kc_raw = (step * 4 + q) * H + part;
    const bool kvalid = kc_raw < s.chunks;
    const int kc = min(kc_raw, s.chunks - 1);

    typename Provider::Raw raw[R];
#pragma unroll
    for (int r = 0; r < R; ++r) prov.load(raw[r], min(row0 + 16 * r + cr, s.N - 1), kc);

    u32x4 xa[MT][8];
    if constexpr (XS) {
      // LDS operations of a wave complete in order, so the reads below see the stores above
      // them without a barrier; rows past M repeat row M - 1 and are zeroed after the read.
      using SL = GemvStage<H>;
      uint8_t* const mine = reinterpret_cast<uint8_t*>(red) + s.stage_offset + wave * (MT * SL::kBytes);
      u32x4 tmp[8 * MT];
#pragma unroll
      for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int i = 0; i < 8; ++i) {  // 1 KiB per instruction of the tile's RT x kRowData bytes
          const int flat = i * 1024 + lane * 16;
          const int row = min(RT * t + flat / SL::kRowData, s.M - 1);
          const int off = flat % SL::kRowData;
          const int kcp = min(step * 4 * H + off / 128, s.chunks - 1);
          tmp[t * 8 + i] = *reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(s.x) + (int64_t)row * s.ldx +
                                                           (int64_t)kcp * 64 + (off % 128) / 2);
        }
#pragma unroll
      for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int flat = i * 1024 + lane * 16;
          const int off = flat % SL::kRowData;
          *reinterpret_cast<u32x4*>(mine + (RT * t + flat / SL::kRowData) * SL::kRow + (off / 128) * SL::kChunk + off % 128) =
              tmp[t * 8 + i];
        }
#pragma unroll
      for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          xa[t][j] = *reinterpret_cast<const u32x4*>(mine + (RT * t + cr) * SL::kRow + (q * H + part) * SL::kChunk + j * 16);
          xa[t][j] = (x_lane[t] && kvalid) ? xa[t][j] : zero4;
        }
    } else {
#pragma unroll
      for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          xa[t][j] = *reinterpret_cast<const u32x4*>(xrow[t] + (int64_t)kc * 64 + j * 8);
          xa[t][j] = (x_lane[t] && kvalid) ? xa[t][j] : zero4;
        }
    }

    // Rows past N are computed on a clamped row and never stored; a k-slot past
    // K must contribute exactly zero, so its operands are zeroed (x is zero
    // there too, but 0 * inf would not be).
    u32x4 b[R][8];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      b[r][0] = prov.template operand<0>(raw[r]);
      b[r][1] = prov.template operand<1>(raw[r]);
      b[r][2] = prov.template operand<2>(raw[r]);
      b[r][3] = prov.template operand<3>(raw[r]);
      b[r][4] = prov.template operand<4>(raw[r]);
      b[r][5] = prov.template operand<5>(raw[r]);
      b[r][6] = prov.template operand<6>(raw[r]);
      b[r][7] = prov.template operand<7>(raw[r]);
    }
    if (s.chunks % (4 * H)) {  // uniform: only shapes with a ragged last step pay for the select
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int j = 0; j < 8; ++j) b[r][j] = kvalid ? b[r][j] : zero4;
    }
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int t = 0; t < MT; ++t) acc[r][t] = mfma16<ACT>(xa[t][j], b[r][j], acc[r][t]);
  }

  if constexpr (kRedOverCodebook) __syncthreads();  // every wave is done with the codebook
  // D layout: lane (c, q) holds D[m = 16t + 4q + i][n = c], i = 0..3, for token tile t.
  // With k parts: D row m' = 4q + i is token m' % RT of part m' / RT, wanted where that is the
  // lane's own part; every (wave, part) files its sums as one more partial tile.
  const int cols = RT * R;
#pragma unroll
  for (int r = 0; r < R; ++r) {
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int mp = 4 * q + i;
        const int m = 16 * t + (mp & (RT - 1));
        if (m < s.M && mp / RT == part)
          red[((int64_t)(wave * H + part) * s.M + m) * cols + r * 16 + cr] = acc[r][t][i];
      }
  }
  __syncthreads();
  for (int o = threadIdx.x; o < s.M * cols; o += blockDim.x) {
    const int m = o / cols;
    const int col = o - m * cols;
    const int n = row0 + col;
    if (n >= s.N) continue;
    float v = 0.f;
    for (int w = 0; w < n_waves * H; ++w) v += red[((int64_t)w * s.M + m) * cols + col];
    if (s.bias) v += s.bias[n];
    store_from_f32<ACT>(s.y, (int64_t)m * s.ldy + n, v);
  }
}

// Launch geometry: enough waves to put the whole packed stream in flight at
// once (the kernel lasts a few microseconds, about one HBM round trip), capped
// at 16 waves per block.
struct GemvPlan {
  int R;               // row tiles (of 16) per block
  int waves;           // waves per block
  int steps_per_wave;
};

// max_r: most row tiles per block the caller wants (4, or 2 for lookups served by L2);
// max_waves_cap: most waves per block its kernel variant is built for.
GemvPlan plan_gemv(int N, int chunks, int max_r = 4, int max_waves_cap = 16);
// k parts per MFMA tile (1, 2 or 4) for M tokens on an N-row layer: more than one only where
// whole 16-row tiles would leave most compute units without a block.  NPAMD_GEMV_PARTS overrides.
// lds_rows: rows of the table every block copies into LDS first (0: none).
int plan_gemv_parts(int M, int N, int chunks, int lds_rows);
// One row tile of `rows` rows per block, `steps` steps to split over its waves.
GemvPlan plan_gemv_rows(int N, int rows, int steps);

// Codebooks up to this many bytes are staged in LDS by the GEMV (64 KiB = 4096 x 8 fp16).
constexpr int kGemvLdsCodebookMax = 64 * 1024;
constexpr int kGemvLdsResidualMax = 16 * 1024;   // residual codebooks of up to 1024 rows
constexpr int kGemvLdsPerBlockMax = 160 * 1024;
// Whether a one-row-tile launch of M tokens stages its activations (XS kernels): from three tokens
// (NPAMD_GEMV_XSTAGE: 0 never, 2 at every token count).
bool gemv_stage_activations(int M);
// Whether this thread's last fused GEMV launch was of a kernel that stages its activations (-1:
// none yet).  Tests compare it with what npamd_gemv_stages_activations answers for the same shape.
int& last_gemv_staged();
// The launcher's own answer, without a launch, for a plain VQ layer with a codebook of `nc` rows of
// eight (vq_gemv.hip) and for a group-quantized layer (q4.hip).
int vq_gemv_plan_stages(int M, int N, int K, int nc);
int q_gemv_plan_stages(int M, int N, int K);
bool gemv_lds_codebook_enabled();  // NPAMD_GEMV_LDS_CB=0 switches the LDS copy off (tuning aid)
bool gemv_lds_activations_forced();  // NPAMD_GEMV_LDS_X=1: stage x in LDS also without a permutation (tuning aid)

template <int ACT, class Provider, int R, bool CB_LDS, bool X_LDS = false, int MT = 1, int H = 1, bool XS = false>
int launch_fused_gemv_r(GemvShape s, const typename Provider::Args& pargs, const GemvPlan& plan,
                        int cb_bytes, hipStream_t st, const char* what) {
  s.steps_per_wave = plan.steps_per_wave;
  const int blocks = (s.N + 16 / H * R - 1) / (16 / H * R);
  const int red_bytes = ((plan.waves * s.M * 16 * R + 3) & ~3) * (int)sizeof(float);
  const int x_bytes = X_LDS ? s.M * s.chunks * 64 * 2 : 0;
  const int cb_lds_bytes = CB_LDS ? cb_bytes : 0;
  int lds = (CB_LDS && !X_LDS)
                      ? (red_bytes > cb_lds_bytes ? red_bytes : cb_lds_bytes)
                      : red_bytes + x_bytes +
                            ((X_LDS && s.perm) ? (cb_lds_bytes > x_bytes ? cb_lds_bytes : x_bytes) : cb_lds_bytes);
  if constexpr (XS) {
    s.stage_offset = (lds + 15) & ~15;
    lds = s.stage_offset + plan.waves * MT * GemvStage<H>::kBytes;
    if (lds > kGemvLdsPerBlockMax)  // no room for the staging areas: the same kernel without them
      return launch_fused_gemv_r<ACT, Provider, R, CB_LDS, X_LDS, MT, H, false>(s, pargs, plan, cb_bytes, st, what);
  }
  if (s.plan_only) {
    *s.plan_only = XS ? 1 : 0;
    return 0;
  }
  if (lds > 64 * 1024) {
    static LdsLatch latch;  // per instantiation
    const hipError_t e = enable_dynamic_lds(
        latch, reinterpret_cast<const void*>(&fused_gemv_kernel<ACT, Provider, R, CB_LDS, X_LDS, MT, H, XS>), lds);
    if (e != hipSuccess)
      return fail(NPAMD_ERR_LAUNCH, "%s: cannot reserve %d bytes of LDS: %s", what, lds, hipGetErrorString(e));
  }
  last_gemv_staged() = XS ? 1 : 0;
  fused_gemv_kernel<ACT, Provider, R, CB_LDS, X_LDS, MT, H, XS><<<blocks, plan.waves * 64, lds, st>>>(s, pargs);
  return check_launch(what);
}

// Whether the LDS copies of x leave the kernel's occupancy alone: two blocks per compute unit
// (80 KiB each) while the grid has more blocks than compute units, else one (160 KiB).  Measured
// on a 8192 x 2048 layer with a 64 KiB codebook: 4.8 us up to 76.5 KiB per block, 6.9 us at 80.5.
bool gemv_perm_keeps_occupancy(int M, int N, int chunks, int cb_bytes);

// cb_bytes: size of the (single) codebook for providers that can stage it in LDS, else 0.
template <int ACT, class Provider>
int launch_fused_gemv(GemvShape s, const typename Provider::Args& pargs, hipStream_t st,
                      const char* what, int cb_bytes = 0) {
  s.steps = (s.chunks + 3) / 4;
  // Layers of few rows, few tokens: 16 / H rows x H parts of k per tile (see the kernel).
  bool lds_table = false;
  if constexpr (Provider::kLdsResidual)
    lds_table = cb_bytes > 0 && cb_bytes <= kGemvLdsResidualMax && gemv_lds_codebook_enabled();
  if constexpr (Provider::kLdsCodebook)
    lds_table = cb_bytes > 0 && cb_bytes <= kGemvLdsCodebookMax && gemv_lds_codebook_enabled();
  int h = plan_gemv_parts(s.M, s.N, s.chunks, lds_table ? cb_bytes / 16 : 0);
  bool whole_codebook_in_lds = lds_table && Provider::kLdsCodebook;
  if (whole_codebook_in_lds && s.M <= 16 && !s.perm && !gemv_lds_activations_forced()) {
    // A block that has few lookups to make does them in memory rather than copy the table first:
    // with as many parts as the layer admits when nothing is copied, up to 2048 lookups per
    // block.  One token, 4096-row table, copy / memory at the parts each admits (us): 512 x 2048
    // 4.15 / 3.0, 2048 x 2048 4.2 / 3.85, 1024 x 1024 4.2 / 3.05, 1024 x 4096 4.4 / 3.95; above the
    // limit 2048 x 4096 4.5 / 5.3, 2048 x 8192 5.5 / 8.6, 512 x 8192 4.5 / 4.8; 1024-row table
    // 1024 x 2048 3.5 / 3.0; 256-row table 1024 x 4096 3.5 / 3.4, 512 x 512 2.95 / 2.7.
    const int h_mem = plan_gemv_parts(s.M, s.N, s.chunks, 0);
    if ((int64_t)16 * s.chunks * 8 / h_mem <= 2048) {
      h = h_mem;
      lds_table = whole_codebook_in_lds = false;
    }
  }
  if (h > 1 && !s.perm && !gemv_lds_activations_forced()) {
    s.steps = (s.chunks + 4 * h - 1) / (4 * h);
    const GemvPlan plan = plan_gemv_rows(s.N, 16 / h, s.steps);
    // Staged activations as for whole tiles, except next to a whole codebook in LDS.
    const bool staged = gemv_stage_activations(s.M) && !(lds_table && Provider::kLdsCodebook);
    if constexpr (Provider::kLdsResidual || Provider::kLdsCodebook) {
      if (lds_table) {
        if constexpr (Provider::kLdsResidual) {
          if (staged && h == 4) return launch_fused_gemv_r<ACT, Provider, 1, true, false, 1, 4, true>(s, pargs, plan, cb_bytes, st, what);
          if (staged) return launch_fused_gemv_r<ACT, Provider, 1, true, false, 1, 2, true>(s, pargs, plan, cb_bytes, st, what);
        }
        if (h == 4) return launch_fused_gemv_r<ACT, Provider, 1, true, false, 1, 4>(s, pargs, plan, cb_bytes, st, what);
        return launch_fused_gemv_r<ACT, Provider, 1, true, false, 1, 2>(s, pargs, plan, cb_bytes, st, what);
      }
    }
    if (staged && h == 4) return launch_fused_gemv_r<ACT, Provider, 1, false, false, 1, 4, true>(s, pargs, plan, 0, st, what);
    if (staged) return launch_fused_gemv_r<ACT, Provider, 1, false, false, 1, 2, true>(s, pargs, plan, 0, st, what);
    if (h == 4) return launch_fused_gemv_r<ACT, Provider, 1, false, false, 1, 4>(s, pargs, plan, 0, st, what);
    return launch_fused_gemv_r<ACT, Provider, 1, false, false, 1, 2>(s, pargs, plan, 0, st, what);
  }
  if constexpr (Provider::kLdsResidual) {
    // Residual VQ: cb_bytes is the residual codebook.  In LDS its lookups leave the vector memory
    // path to the main codebook's; row tiles per block stay at two, as for every provider that
    // looks up in memory.
    if (cb_bytes > 0 && cb_bytes <= kGemvLdsResidualMax && gemv_lds_codebook_enabled()) {
      if (s.M > 16) {
        const GemvPlan plan = plan_gemv(s.N, s.chunks, gemv_stage_activations(s.M) ? 1 : 2, 8);  // as for plain VQ below
        if (plan.R == 2) return launch_fused_gemv_r<ACT, Provider, 2, true, false, 2>(s, pargs, plan, cb_bytes, st, what);
        if (gemv_stage_activations(s.M))
          return launch_fused_gemv_r<ACT, Provider, 1, true, false, 2, 1, true>(s, pargs, plan, cb_bytes, st, what);
        return launch_fused_gemv_r<ACT, Provider, 1, true, false, 2>(s, pargs, plan, cb_bytes, st, what);
      }
      const GemvPlan plan = plan_gemv(s.N, s.chunks, 2);
      if (plan.R == 2) return launch_fused_gemv_r<ACT, Provider, 2, true>(s, pargs, plan, cb_bytes, st, what);
      if (gemv_stage_activations(s.M))
        return launch_fused_gemv_r<ACT, Provider, 1, true, false, 1, 1, true>(s, pargs, plan, cb_bytes, st, what);
      return launch_fused_gemv_r<ACT, Provider, 1, true>(s, pargs, plan, cb_bytes, st, what);
    }
  }
  const bool cb_in_lds = whole_codebook_in_lds;
  // Lookups that go to L2 want many waves in flight more than they want shared x operands
  // (14336 x 4096, 65536-row codebook, one token: 34.6 us with two row tiles, 37.2 with four).
  if (s.M > 16) {
    // 17..32 tokens: two token tiles per weight operand, eight waves.  Every block reads all of
    // x, twice as much as at 16 tokens, so four row tiles per block (half the blocks) pay more
    // than anywhere else: 14336 x 4096, 4096-row codebook, 17 tokens: 20.0 us at R = 2, 12.9 at 4.
    // Lookups in memory: one staged row tile per block instead of two plain ones (65536-row
    // codebook, 24 / 32 tokens, us: 6144 x 4096 22.45 / 24.3 -> 22.2 / 22.8, 11008 x 4096 41.5 /
    // 44.8 -> 34.9 / 35.75, 14336 x 4096 46.7 / 49.7 -> 44.8 / 45.8, 28672 x 4096 83.3 / 89.75 ->
    // 74.8 / 77.7, 8192 x 8192 47.0 / 50.3 -> 45.3 / 46.8); at 16 tokens and below it depends on
    // the layer (6144 x 4096 20.5 -> 21.45 at 16), so there the plan stands.
    const bool memory_lookups = Provider::kGathers && !cb_in_lds;
    const GemvPlan plan = plan_gemv(s.N, s.chunks, memory_lookups ? (gemv_stage_activations(s.M) ? 1 : 2) : 4, 8);
    if constexpr (Provider::kLdsCodebook) {
      if (cb_in_lds) {
        if (plan.R == 4) return launch_fused_gemv_r<ACT, Provider, 4, true, false, 2>(s, pargs, plan, cb_bytes, st, what);
        if (plan.R == 2) return launch_fused_gemv_r<ACT, Provider, 2, true, false, 2>(s, pargs, plan, cb_bytes, st, what);
        return launch_fused_gemv_r<ACT, Provider, 1, true, false, 2>(s, pargs, plan, cb_bytes, st, what);
      }
    }
    if constexpr (!Provider::kGathers)
      if (plan.R == 4) return launch_fused_gemv_r<ACT, Provider, 4, false, false, 2>(s, pargs, plan, 0, st, what);
    if (plan.R == 2) return launch_fused_gemv_r<ACT, Provider, 2, false, false, 2>(s, pargs, plan, 0, st, what);
    if (gemv_stage_activations(s.M))
      return launch_fused_gemv_r<ACT, Provider, 1, false, false, 2, 1, true>(s, pargs, plan, 0, st, what);
    return launch_fused_gemv_r<ACT, Provider, 1, false, false, 2>(s, pargs, plan, 0, st, what);
  }
  const GemvPlan plan = plan_gemv(s.N, s.chunks, (Provider::kGathers && !cb_in_lds) ? 2 : 4);
  if constexpr (Provider::kLdsCodebook) {
    const bool x_fits = (int64_t)s.M * s.chunks * 64 <= kGemvLdsActivationsMax;
    if (s.perm || (x_fits && gemv_lds_activations_forced())) {  // with a permutation the caller has checked the size
      if (cb_in_lds) {
        if (plan.R == 4) return launch_fused_gemv_r<ACT, Provider, 4, true, true>(s, pargs, plan, cb_bytes, st, what);
        if (plan.R == 2) return launch_fused_gemv_r<ACT, Provider, 2, true, true>(s, pargs, plan, cb_bytes, st, what);
        return launch_fused_gemv_r<ACT, Provider, 1, true, true>(s, pargs, plan, cb_bytes, st, what);
      }
      if (plan.R == 4) return launch_fused_gemv_r<ACT, Provider, 4, false, true>(s, pargs, plan, 0, st, what);
      if (plan.R == 2) return launch_fused_gemv_r<ACT, Provider, 2, false, true>(s, pargs, plan, 0, st, what);
      return launch_fused_gemv_r<ACT, Provider, 1, false, true>(s, pargs, plan, 0, st, what);
    }
    if (cb_in_lds) {
      if (plan.R == 4) return launch_fused_gemv_r<ACT, Provider, 4, true>(s, pargs, plan, cb_bytes, st, what);
      if (plan.R == 2) return launch_fused_gemv_r<ACT, Provider, 2, true>(s, pargs, plan, cb_bytes, st, what);
      return launch_fused_gemv_r<ACT, Provider, 1, true>(s, pargs, plan, cb_bytes, st, what);
    }
  }
  if (plan.R == 4) return launch_fused_gemv_r<ACT, Provider, 4, false>(s, pargs, plan, 0, st, what);
  if (plan.R == 2) return launch_fused_gemv_r<ACT, Provider, 2, false>(s, pargs, plan, 0, st, what);
  if (gemv_stage_activations(s.M))
    return launch_fused_gemv_r<ACT, Provider, 1, false, false, 1, 1, true>(s, pargs, plan, 0, st, what);
  return launch_fused_gemv_r<ACT, Provider, 1, false>(s, pargs, plan, 0, st, what);
}

// ---------------------------------------------------------------------------
// Fallback for shapes the MFMA kernel does not take (odd vector length or index
// width, K not a multiple of 64, unaligned buffers): one wave per output
// element, lanes stride over k, every weight element decoded on its own.
// Slow by design; exists so that every valid input has a HIP path.
//   Elem::get(n, k) -> float weight value in the activation dtype's rounding.
// ---------------------------------------------------------------------------
template <int ACT, class Elem, int MT>
__global__ void __launch_bounds__(256)
generic_rows_kernel(const void* __restrict__ x, int64_t ldx, const float* __restrict__ bias,
                    void* __restrict__ y, int64_t ldy, int M, int N, int K, const Elem elem) {
  // One wave per output row and block of up to MT tokens (blockIdx.y): a weight element is
  // decoded once per MT tokens, each lane summing its k = lane, lane + 64, ... in order.
  const int lane = threadIdx.x & 63;
  const int n = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int m0 = blockIdx.y * MT;
  const int mt = min(MT, M - m0);
  if (n >= N) return;
  float acc[MT];
#pragma unroll
  for (int j = 0; j < MT; ++j) acc[j] = 0.f;
  for (int k = lane; k < K; k += 64) {
    const float w = elem.get(n, k);
#pragma unroll
    for (int j = 0; j < MT; ++j)
      if (j < mt) acc[j] = __builtin_fmaf(load_as_f32<ACT>(x, (int64_t)(m0 + j) * ldx + k), w, acc[j]);
  }
#pragma unroll
  for (int j = 0; j < MT; ++j) {
    if (j >= mt) break;
    float total = wave_reduce_sum(acc[j]);
    if (lane == 0) {
      if (bias) total += bias[n];
      store_from_f32<ACT>(y, (int64_t)(m0 + j) * ldy + n, total);
    }
  }
}

template <int ACT, class Elem>
int launch_generic_gemv(const void* x, int64_t ldx, const float* bias, void* y, int64_t ldy,
                        int M, int N, int K, const Elem& elem, hipStream_t st, const char* what) {
  const unsigned rows = (unsigned)((N + 3) / 4);
  if (M == 1) generic_rows_kernel<ACT, Elem, 1><<<dim3(rows, 1), 256, 0, st>>>(x, ldx, bias, y, ldy, M, N, K, elem);
  else if (M <= 4) generic_rows_kernel<ACT, Elem, 4><<<dim3(rows, 1), 256, 0, st>>>(x, ldx, bias, y, ldy, M, N, K, elem);
  else generic_rows_kernel<ACT, Elem, 16><<<dim3(rows, (unsigned)((M + 15) / 16)), 256, 0, st>>>(x, ldx, bias, y, ldy, M, N, K, elem);
  return check_launch(what);
}

// Weight element of a (residual) VQ layer, any VL / index width.
struct VqElem {
  const uint8_t* packed;
  int64_t n_bytes;
  int bits;
  const uint16_t* cb;
  uint32_t nc_minus_1;
  int vl, groups;
  int act;       // activation dtype the weight is rounded to
  int cb_dtype;  // NPAMD_F16, or NPAMD_BF16 when the caller pre-cast the codebook
  // residual part (packed_r == nullptr -> plain VQ)
  const uint8_t* packed_r;
  int64_t n_bytes_r;
  int bits_r;
  const uint16_t* cb_r;
  uint32_t ncr_minus_1;
  const uint16_t* row_scale;
  const uint16_t* row_bias;

  __device__ __forceinline__ float get(int n, int k) const {
#pragma clang fp contract(off)
    const int g = k / vl, v = k - g * vl;
    const int64_t flat = (int64_t)n * groups + g;
    const uint32_t i = min(read_index(packed, n_bytes, flat, bits), nc_minus_1);
    if (cb_dtype == NPAMD_BF16) return bf16_bits_to_f32(cb[(int64_t)i * vl + v]);
    _Float16 h = __builtin_bit_cast(_Float16, cb[(int64_t)i * vl + v]);
    if (packed_r) {
      const uint32_t ir = min(read_index(packed_r, n_bytes_r, flat, bits_r), ncr_minus_1);
      h = h + __builtin_bit_cast(_Float16, cb_r[(int64_t)ir * vl + v]);
      if (row_scale) h = h * __builtin_bit_cast(_Float16, row_scale[n]);
      if (row_bias) h = h + __builtin_bit_cast(_Float16, row_bias[n]);
    }
    const float f = (float)h;
    return act == NPAMD_BF16 ? bf16_bits_to_f32(f32_to_bf16_bits(f)) : f;
  }
};

// Weight element of a group-affine n-bit layer, any nbits in {1,2,4,8}, sym or asym.
struct QElem {
  const uint8_t* w_pack;
  const uint16_t* scale;
  const uint16_t* zero_point;  // may be null
  int K, nbits, group_size;
  int act;

  __device__ __forceinline__ float get(int n, int k) const {
#pragma clang fp contract(off)
    const int vpb = 8 / nbits;
    const int q = (w_pack[(int64_t)n * (K / vpb) + k / vpb] >> ((k % vpb) * nbits)) & ((1 << nbits) - 1);
    const int64_t sidx = (int64_t)n * (K / group_size) + k / group_size;
    const float zp = zero_point ? f16_bits_to_f32(zero_point[sidx]) : (float)(1 << (nbits - 1));
    const float d = (float)q - zp;
    const float w = d * f16_bits_to_f32(scale[sidx]);
    return act == NPAMD_BF16 ? bf16_bits_to_f32(f32_to_bf16_bits(w))
                             : f16_bits_to_f32(f32_to_f16_bits(w));
  }
};

}  // namespace npamd
