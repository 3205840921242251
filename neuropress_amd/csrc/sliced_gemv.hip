// Decode GEMV over the slice-list form of the indices (see sliced_format.hpp).
//
// One workgroup of 16 waves holds the activations of its group range (up to 8 KiB
// per token, up to seven tokens per launch), one 4096-row codebook slice (64 KiB)
// and a zero row in LDS.  Every lane owns one output row and
// walks the entries filed under (slice, group range, row): two 16-byte LDS reads
// (codebook row, activation vector) and four packed dot products per entry, the
// sum kept in registers.
//
// Finish.  A row's result is spread over the workgroups that hold the slices its indices
// point into (n_partials of them).  With fewer than 256 per row -- every codebook of up to
// 2^16 rows -- each lane rounds its partial sum to a multiple of 2^-24 and adds it, with one
// 64-bit integer atomic, to the row's word of the workspace, which also counts the arrivals;
// the lane that completes the count converts the total, adds the bias, rounds once to the
// activation dtype, stores y and zeroes the word.  Integer addition commutes, so the result
// does not depend on the order of arrival; it differs from the exact sum by at most
// n_partials * 2^-25 plus the final roundings, whatever the magnitude of y.  Partial sums of
// magnitude 2^15 or more (and NaN / infinity) do not fit the word: they are added to a float
// accumulator with a float atomic instead, and only then -- two or more such partial sums in
// one row -- can the last bits depend on the order of arrival.  With 256 partial vectors or
// more every lane writes its partial sum out and a second kernel adds them in a fixed order.
#include <stdlib.h>

#include <mutex>

#include "common.hpp"
#include "sliced_format.hpp"

namespace npamd {

struct SlicedArgs {
  const uint16_t* x;  // first token of the launch; a token is K/8 vectors of eight 16-bit values
  int64_t ldx;        // elements between tokens
  int64_t token_stride;  // floats between the partial sums of consecutive tokens
  const int32_t* column_perm;  // optional [K]: the kernel reads x[perm[k]] where it would read x[k]
  const u32x4* codebook;
  const SlicedWorkgroup* wgs;
  const uint32_t* rowmap;
  const uint8_t* entries;
  float* partials;  // two-kernel finish: [n_partials][n] per token
  // Fused finish (n_partials < 256): one 64-bit word per (token, row), zero between calls.
  // Bits 16-63: sum of the partial sums in units of 2^-24 (two's complement); bits 8-15: how
  // many of them went to `spill` instead; bits 0-7: how many lanes have added so far.
  unsigned long long* sums;
  float* spill;       // [token][row], zero between calls: partial sums the fixed-point word cannot hold
  const float* bias;  // f32 [n] or null
  void* y;
  int64_t ldy;
  int n_partials, fused_finish;
  int n, nc, slice_rows;
  int wg_quads;       // entry quads per workgroup
  // Regular geometry (regular != 0): every slice has `parts` group ranges of `range_groups`
  // groups and workgroup w = (part * row_blocks + row block) * n_slices + slice, so a workgroup
  // knows its slice and group range without reading its record.
  int regular, n_slices, row_blocks, parts, range_groups, groups, rows_per_block;
  uint32_t magic_slices, magic_blocks;  // ceil(2^32 / n_slices), ceil(2^32 / row_blocks)
  uint32_t wave_info[kSlicedWaves];     // quads of the wave's strip | first quad inside the workgroup << 16
};

// n / d for n * d < 2^32 with magic = ceil(2^32 / d) (d = 1: magic does not fit, n is returned).
__device__ __forceinline__ uint32_t fast_div(uint32_t n, uint32_t d, uint32_t magic) {
  return d == 1u ? n : __umulhi(n, magic);
}

// Operands are taken by value: __builtin_bit_cast applied directly to a vector
// element expression (v.y) reads element 0 with this compiler.
template <int ACT>
__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
  if constexpr (ACT == NPAMD_BF16)
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a), __builtin_bit_cast(bf16x2, b), c, false);
  else
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, a), __builtin_bit_cast(f16x2, b), c, false);
}

template <int ACT>
__device__ __forceinline__ float dot8(u32x4 a, u32x4 b, float c) {
  c = dot2<ACT>(a.x, b.x, c);
  c = dot2<ACT>(a.y, b.y, c);
  c = dot2<ACT>(a.z, b.z, c);
  return dot2<ACT>(a.w, b.w, c);
}

struct Quad {
  uint32_t d0, d1, d2;
};

// Entry quads a lane keeps requested ahead of the one it works on.
constexpr int kDepth = 3;
// Straight-line code exists for strips of up to this many quads, at the token counts where it
// measured faster than the loops (config 3: 1 / 2 tokens, and 6 / 7 tokens 26.9 -> 25.1 / 29.9 -> 28.4 us;
// no difference at 3-5 tokens, which keep the smaller code).
constexpr int kMaxStraightQuads = 16;
constexpr bool straight_tokens(int m) { return m <= 2 || m >= 6; }
// LDS map: activations of the group range, then the slice, then the zero row that
// padding entries select.  Both bases fit the 16-bit offset field of an LDS read.
constexpr int kMaxTokens = 7;  // tokens per pass over the entries (an eighth token's activations would not fit in LDS)
constexpr int kLdsX = 0;       // [token][group] vectors: a token's 512 vectors are contiguous, so the
                               // lanes of a read spread over all sixteen 16-byte bank groups
// The map is sized by the launch's token count M (76 KiB at one token).  Two workgroups per compute
// unit -- 512 workgroups of 448 rows, 64 registers per lane -- were measured at one token and lose:
// 12.8 against 11.4 us (more slice copies, waves without a strip, and 10.9 us with 71 registers).
constexpr int lds_slice(int m) { return kSlicedMaxGroups * 16 * m; }
constexpr int lds_stage(int m) { return lds_slice(m) + (kSlicedMaxSliceRows + 1) * 16; }  // [token][row of the block] sums, fused finish
constexpr int lds_bytes(int m) { return lds_stage(m) + m * kSlicedTasks * 4; }
static_assert(lds_bytes(kMaxTokens) <= kSlicedLdsBytes && lds_slice(kMaxTokens) < 65536, "LDS map");
// The first eight waves copy the slice into LDS.
constexpr int kLoaderThreads = kSlicedTasks / 2;
constexpr int kSliceLoads = kSlicedMaxSliceRows / kLoaderThreads;

__device__ __forceinline__ void load_quad(Quad& q, const uint8_t* p) {
  __builtin_memcpy(&q, __builtin_assume_aligned(p, 4), 12);
}

template <uint32_t MASK>
__device__ __forceinline__ uint32_t low_field(uint32_t v) {
  uint32_t r;
  asm("v_and_b32 %0, %1, %2" : "=v"(r) : "s"(MASK), "v"(v));
  return r;
}

// The LDS byte addresses of the four entries of one quad: codebook row and activation vector.
// A lane's record is four 16-bit row fields followed by four group bytes.
struct QuadAddr {
  uint32_t row[4], grp[4];
};

__device__ __forceinline__ QuadAddr quad_addresses(const Quad& q) {
  QuadAddr ad;
  // Row fields: bits 0-12 the row, bit 15 the ninth bit of the group (256 groups = 4096 bytes).
  const uint32_t f[4] = {q.d0, q.d0 >> 16, q.d1, q.d1 >> 16};
  const uint32_t glow[4] = {low_field<0xFFu>(q.d2), (q.d2 >> 8) & 0xFFu, (q.d2 >> 16) & 0xFFu, q.d2 >> 24};
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    ad.row[j] = (f[j] & 0x1FFFu) << 4;
    ad.grp[j] = (glow[j] << 4) | ((f[j] & 0x8000u) >> 3);
  }
  return ad;
}

// Per entry: one codebook row and M activation vectors from LDS, 4 M dot products.
template <int ACT, int M>
__device__ __forceinline__ void run_quad(const QuadAddr& ad, const uint8_t* lds, float (&acc)[M][2]) {
  constexpr int kBatch = M > 2 ? 2 : 4;  // entries whose LDS reads are issued together
#pragma unroll
  for (int j0 = 0; j0 < 4; j0 += kBatch) {
    u32x4 c[kBatch], xv[kBatch][M];
#pragma unroll
    for (int j = 0; j < kBatch; ++j) {
      c[j] = *reinterpret_cast<const u32x4*>(lds + lds_slice(M) + ad.row[j0 + j]);
      const uint8_t* xg = lds + kLdsX + ad.grp[j0 + j];
#pragma unroll
      for (int m = 0; m < M; ++m) xv[j][m] = *reinterpret_cast<const u32x4*>(xg + m * (kSlicedMaxGroups * 16));
    }
#pragma unroll
    for (int j = 0; j < kBatch; ++j)
#pragma unroll
      for (int m = 0; m < M; ++m) acc[m][j & 1] = dot8<ACT>(c[j], xv[j][m], acc[m][j & 1]);
  }
}

// Fused finish: the lane adds its partial sum, as a 40.24 fixed-point number, to the row's word
// with one returning atomic; integer addition does not depend on the order of arrival, so the
// result is the same from run to run.  The lane whose addition completes the count converts the
// sum back, adds the bias, rounds once, stores y and clears the word for the next call.  A
// partial sum of magnitude 2^15 or more (or a NaN) goes to a float accumulator instead, which
// the finishing lane adds in (those sums are added in order of arrival).
constexpr float kFixedOne = 16777216.f;     // 2^24
constexpr float kFixedLimit = 32768.f;      // 2^15: 255 such sums stay inside 47 bits
template <int ACT>
__device__ __forceinline__ void finish_row(const SlicedArgs& a, int m, uint32_t row, float v, float bias) {
  const size_t cell = (size_t)m * a.n + row;
  const bool fits = fabsf(v) < kFixedLimit;  // false for NaN and infinities
  unsigned long long add = 1ull;
  if (fits) {
    add += (unsigned long long)(long long)__float2ll_rn(v * kFixedOne) << 16;
  } else {
    // The addition must have been performed before this lane's arrival is counted (the lane that
    // completes the count reads the accumulator): its result is asked for and waited for -- an
    // atomic without a use of its result is issued as fire-and-forget, and nothing orders it
    // against the atomic on the row's word, which may live in another L2 channel.
    const float before = __hip_atomic_fetch_add(a.spill + cell, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    asm volatile("" ::"v"(before) : "memory");
    add += 0x100ull;
  }
  const unsigned long long old = __hip_atomic_fetch_add(a.sums + cell, add, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if ((int)(old & 0xFFull) != a.n_partials - 1) return;
  const unsigned long long total = old + add;
  float sum = (float)((double)((long long)total >> 16) * (1.0 / 16777216.0));  // exact product, one rounding
  if ((total >> 8) & 0xFFull) sum += __hip_atomic_exchange(a.spill + cell, 0.f, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  sum += bias;  // requested before the atomic: a load issued here would add a memory round trip to the call's tail
  store_from_f32<ACT>((uint16_t*)a.y + (size_t)m * a.ldy, row, sum);
  __hip_atomic_store(a.sums + cell, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The NQ quads of a strip, of which the first min(kDepth, NQ) have been requested into q.
// Straight-line code: the compiler knows how many loads are in flight at each use of a quad.
template <int ACT, int M, int NQ>
__device__ __forceinline__ void walk_strip(Quad (&q)[kDepth], const uint8_t* strip_lane, const uint8_t* lds,
                                           float (&acc)[M][2]) {
  constexpr int D = kDepth;
#pragma unroll
  for (int i = 0; i < NQ; ++i) {
    // The addresses are taken out of the quad before its registers are asked for again.
    const QuadAddr ad = quad_addresses(q[i % D]);
    if (i + D < NQ) load_quad(q[i % D], strip_lane + (size_t)(i + D) * kSlicedQuadBytes);
    run_quad<ACT, M>(ad, lds, acc);
  }
}

template <int ACT, int M, bool PERM>
__global__ void __launch_bounds__(kSlicedTasks, 1) sliced_gemv_kernel(SlicedArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  constexpr int D = kDepth;
  u32x4* xl = reinterpret_cast<u32x4*>(lds + kLdsX);
  u32x4* cb = reinterpret_cast<u32x4*>(lds + lds_slice(M));
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t info = a.wave_info[wave];
  const int nq = (int)(info & 0xFFFFu);
  // A wave without a strip (nq = 0) reads the workgroup's first quad and ignores it.
  const uint8_t* const strip_lane = a.entries +
                                    ((size_t)blockIdx.x * (size_t)a.wg_quads + (size_t)(nq ? info >> 16 : 0u)) * kSlicedQuadBytes +
                                    (size_t)lane * 12;
  uint32_t slice, partial, g_begin, g_count, row_begin, row_count;
  if (a.regular) {
    const uint32_t w = blockIdx.x;
    const uint32_t j = fast_div(w, (uint32_t)a.n_slices, a.magic_slices);
    const uint32_t part = fast_div(j, (uint32_t)a.row_blocks, a.magic_blocks);
    slice = w - j * (uint32_t)a.n_slices;
    partial = slice * (uint32_t)a.parts + part;
    g_begin = part * (uint32_t)a.range_groups;
    g_count = min((uint32_t)a.range_groups, (uint32_t)a.groups - g_begin);
    row_begin = min((j - part * (uint32_t)a.row_blocks) * (uint32_t)a.rows_per_block, (uint32_t)a.n);
    row_count = min((uint32_t)a.rows_per_block, (uint32_t)a.n - row_begin);
  } else {
    const SlicedWorkgroup wg = a.wgs[blockIdx.x];
    slice = wg.slice; partial = wg.partial; g_begin = wg.g_begin; g_count = wg.g_count;
    row_begin = wg.row_begin; row_count = wg.row_count;
  }

  // The slice and the activations are requested first and stored to LDS; only then are the
  // first entry quads requested.  The 256 workgroups of a launch ask for 16 MiB of slices at
  // once, which keeps the L2 -> L1 path busy for the whole prologue: entry requests issued in
  // front of the wait for the slice only queue between the slice's (measured: 10.5 against
  // 10.3 us per call at one token, 13.35 against 13.0 us at two).  The first eight waves copy
  // the slice.
  Quad q[D];
  {
    const int slice_len = min(a.slice_rows, a.nc - (int)slice * a.slice_rows);
    const u32x4* src = a.codebook + (int64_t)slice * a.slice_rows;
    const bool loader = tid < kLoaderThreads;  // wave-uniform
    u32x4 t[kSliceLoads];
    if (loader) {
#pragma unroll
      for (int i = 0; i < kSliceLoads; ++i) t[i] = src[min(tid + i * kLoaderThreads, slice_len - 1)];
    }
    // Thread t stages group t % 512 of tokens t / 512, t / 512 + 2, ... (512 groups x 7 tokens at most).
    constexpr int kXLoads = (M + 1) / 2;
    const int xg = tid & (kSlicedMaxGroups - 1), xm = tid / kSlicedMaxGroups;
    const int xvec = (int)g_begin + min(xg, (int)g_count - 1);
    const uint16_t* xrow[kXLoads];
    u32x4 xt[kXLoads], perm_lo, perm_hi;
#pragma unroll
    for (int i = 0; i < kXLoads; ++i) xrow[i] = a.x + (int64_t)min(xm + 2 * i, M - 1) * a.ldx;
    if constexpr (PERM) {  // the eight source columns of this vector; the elements follow below
      perm_lo = reinterpret_cast<const u32x4*>(a.column_perm)[2 * xvec];
      perm_hi = reinterpret_cast<const u32x4*>(a.column_perm)[2 * xvec + 1];
    } else {
#pragma unroll
      for (int i = 0; i < kXLoads; ++i)
        if (xm + 2 * i < M) xt[i] = reinterpret_cast<const u32x4*>(xrow[i])[xvec];  // wave-uniform: xm = tid / 512
    }
    if constexpr (PERM) {
      const uint32_t pc[8] = {perm_lo.x, perm_lo.y, perm_lo.z, perm_lo.w, perm_hi.x, perm_hi.y, perm_hi.z, perm_hi.w};
#pragma unroll
      for (int i = 0; i < kXLoads; ++i) {
        uint32_t e[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) e[j] = xrow[i][pc[j]];
        xt[i] = u32x4{e[0] | (e[1] << 16), e[2] | (e[3] << 16), e[4] | (e[5] << 16), e[6] | (e[7] << 16)};
      }
    }
    if (loader) {
#pragma unroll
      for (int i = 0; i < kSliceLoads; ++i)
        if (tid + i * kLoaderThreads < slice_len) cb[tid + i * kLoaderThreads] = t[i];
    }
#pragma unroll
    for (int i = 0; i < kXLoads; ++i)
      if (xg < (int)g_count && xm + 2 * i < M) xl[(xm + 2 * i) * kSlicedMaxGroups + xg] = xt[i];
    if (tid == kSlicedTasks - 1) cb[kSlicedPadRow] = u32x4{0u, 0u, 0u, 0u};  // what padding entries select
    __builtin_amdgcn_sched_barrier(0);  // keep the entry requests behind the stores
    // The first quads (past the strip's end: its last quad again; no branch around a load).
#pragma unroll
    for (int i = 0; i < D; ++i) load_quad(q[i], strip_lane + (size_t)max(min(i, nq - 1), 0) * kSlicedQuadBytes);
    __builtin_amdgcn_sched_barrier(0);
  }
  const uint32_t row = a.rowmap[(size_t)blockIdx.x * kSlicedTasks + tid];
  __syncthreads();

  float acc[M][2];
#pragma unroll
  for (int m = 0; m < M; ++m) acc[m][0] = acc[m][1] = 0.f;
  if (straight_tokens(M) && nq <= kMaxStraightQuads) {
    // Strips of up to kMaxStraightQuads quads (all of them, unless a row's indices crowd into one
    // slice) are walked by straight-line code picked by the strip's length: no loop carries a
    // register that is being loaded (a loop drains the quads in flight at every back-edge to
    // rename them).
    switch (nq) {
#define NPAMD_STRIP_CASE(NQ) \
  case NQ: walk_strip<ACT, M, NQ>(q, strip_lane, lds, acc); break;
      NPAMD_STRIP_CASE(1) NPAMD_STRIP_CASE(2) NPAMD_STRIP_CASE(3) NPAMD_STRIP_CASE(4)
      NPAMD_STRIP_CASE(5) NPAMD_STRIP_CASE(6) NPAMD_STRIP_CASE(7) NPAMD_STRIP_CASE(8)
      NPAMD_STRIP_CASE(9) NPAMD_STRIP_CASE(10) NPAMD_STRIP_CASE(11) NPAMD_STRIP_CASE(12)
      NPAMD_STRIP_CASE(13) NPAMD_STRIP_CASE(14) NPAMD_STRIP_CASE(15) NPAMD_STRIP_CASE(16)
#undef NPAMD_STRIP_CASE
      default: break;
    }
  } else {
    // Longer strips and more tokens: three plain loops.
    int q0 = 0;
    for (; q0 + 2 * D <= nq; q0 += D) {
#pragma unroll
      for (int i = 0; i < D; ++i) {
        const QuadAddr ad = quad_addresses(q[i]);
        load_quad(q[i], strip_lane + (size_t)(q0 + i + D) * kSlicedQuadBytes);
        run_quad<ACT, M>(ad, lds, acc);
      }
    }
#pragma unroll
    for (int i = 0; i < D; ++i) {
      if (q0 + i >= nq) break;
      const QuadAddr ad = quad_addresses(q[i]);
      if (q0 + i + D < nq) load_quad(q[i], strip_lane + (size_t)(q0 + i + D) * kSlicedQuadBytes);
      run_quad<ACT, M>(ad, lds, acc);
    }
    q0 += D;
#pragma unroll
    for (int i = 0; i < D; ++i) {
      if (q0 + i >= nq) break;
      run_quad<ACT, M>(quad_addresses(q[i]), lds, acc);
    }
  }
  if (a.fused_finish) {
    // The lanes of a wave work for rows scattered over the workgroup's block (strips are sorted
    // by length); the sums change hands through LDS so that thread t finishes row row_begin + t
    // and a wave's atomics, bias reads and stores fall on consecutive addresses.
    float* stage = reinterpret_cast<float*>(lds + lds_stage(M));
    if (row != kSlicedNoRow) {
#pragma unroll
      for (int m = 0; m < M; ++m) stage[m * kSlicedTasks + (row - row_begin)] = acc[m][0] + acc[m][1];
    }
    __syncthreads();
    if ((uint32_t)tid < row_count) {
      const float bias = a.bias ? a.bias[row_begin + (uint32_t)tid] : 0.f;
#pragma unroll
      for (int m = 0; m < M; ++m) finish_row<ACT>(a, m, row_begin + (uint32_t)tid, stage[m * kSlicedTasks + tid], bias);
    }
  } else if (row != kSlicedNoRow) {
#pragma unroll
    for (int m = 0; m < M; ++m)
      a.partials[(size_t)m * a.token_stride + (size_t)partial * a.n + row] = acc[m][0] + acc[m][1];
  }
}

// Two-kernel finish (256 partial vectors or more per row):
// y[token][row] = round(sum over the partial vectors + bias).  16 rows per block
// (blockIdx.y = token); the partial vectors are dealt over 16 threads per row,
// whose sums are then added in a fixed order.
template <int ACT>
__global__ void __launch_bounds__(256) sliced_reduce_kernel(float* __restrict__ partials, int n_partials,
                                                             int n, const float* __restrict__ bias,
                                                             void* __restrict__ y, int64_t ldy) {
  __shared__ float red[16][17];
  const int r = threadIdx.x & 15, j = threadIdx.x >> 4;
  const int row = blockIdx.x * 16 + r;
  partials += (size_t)blockIdx.y * n_partials * n;
  y = (uint16_t*)y + (size_t)blockIdx.y * ldy;
  float sum = 0.f;
  if (row < n)
    for (int p = j; p < n_partials; p += 16) {
      sum += partials[(size_t)p * n + row];
      partials[(size_t)p * n + row] = 0.f;  // the workspace is handed back zero-filled
    }
  red[j][r] = sum;
  __syncthreads();
  if (j == 0 && row < n) {
    float total = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) total += red[i][r];
    if (bias) total += bias[row];
    store_from_f32<ACT>(y, row, total);
  }
}

template <int ACT, int M, bool PERM>
int launch_sliced_tokens_p(const SlicedArgs& a, int n_workgroups, hipStream_t st, const char* what) {
  static LdsLatch latch;  // per instantiation
  constexpr int kLdsBytes = lds_bytes(M);
  const hipError_t e = enable_dynamic_lds(latch, reinterpret_cast<const void*>(&sliced_gemv_kernel<ACT, M, PERM>), kLdsBytes);
  if (e != hipSuccess)
    return fail(NPAMD_ERR_LAUNCH, "%s: cannot reserve %d bytes of LDS: %s", what, kLdsBytes, hipGetErrorString(e));
  sliced_gemv_kernel<ACT, M, PERM><<<n_workgroups, kSlicedTasks, kLdsBytes, st>>>(a);
  return check_launch(what);
}

template <int ACT, int M>
int launch_sliced_tokens(const SlicedArgs& a, int n_workgroups, hipStream_t st, const char* what) {
  return a.column_perm ? launch_sliced_tokens_p<ACT, M, true>(a, n_workgroups, st, what)
                       : launch_sliced_tokens_p<ACT, M, false>(a, n_workgroups, st, what);
}

// The fused finish counts the partial sums of a row in eight bits.
inline bool sliced_fused_finish(const npamd_sliced_header& h) { return h.n_partials < 256; }

// ceil(2^32 / d) for fast_div; d = 1 never uses it.
inline uint32_t div_magic(uint32_t d) { return d <= 1u ? 0u : (uint32_t)(((1ull << 32) + d - 1) / d); }

template <int ACT>
int launch_sliced(const npamd_sliced_header& h, const uint8_t* blob, const void* x, int64_t ldx,
                  const void* codebook, const int32_t* column_perm, const float* bias, void* y, int64_t ldy,
                  int M, float* workspace, hipStream_t st, const char* what) {
  SlicedArgs a;
  a.column_perm = column_perm;
  a.codebook = (const u32x4*)codebook;
  a.wgs = (const SlicedWorkgroup*)(blob + h.off_workgroups);
  a.rowmap = (const uint32_t*)(blob + h.off_rowmap);
  a.entries = blob + h.off_entries;
  a.n = h.n; a.nc = h.nc; a.slice_rows = h.slice_rows;
  a.ldx = ldx;
  a.token_stride = (int64_t)h.n_partials * (int64_t)h.n;
  a.n_partials = h.n_partials;
  a.fused_finish = sliced_fused_finish(h);
  a.bias = bias;
  a.ldy = ldy;
  uint32_t begin = 0;
  for (int w = 0; w < kSlicedWaves; ++w) {
    a.wave_info[w] = (uint32_t)h.wave_quads[w] | (begin << 16);
    begin += h.wave_quads[w];
  }
  a.wg_quads = (int)(begin ? begin : 1u);
  // The regular geometry, when the header states it and the counts bear it out.
  a.groups = h.k / 8;
  a.n_slices = h.n_slices;
  a.parts = h.n_partials / h.n_slices;
  a.row_blocks = a.parts ? h.n_workgroups / (a.parts * h.n_slices) : 0;
  a.range_groups = a.parts ? (a.groups + a.parts - 1) / a.parts : 0;
  a.rows_per_block = a.row_blocks ? (h.n + a.row_blocks - 1) / a.row_blocks : 0;
  a.regular = (h.flags & kSlicedRoundRobin) && a.parts >= 1 && a.row_blocks >= 1 &&
              a.parts * h.n_slices == h.n_partials && a.row_blocks * h.n_partials == h.n_workgroups &&
              (int64_t)(a.parts - 1) * a.range_groups < a.groups && a.rows_per_block <= kSlicedTasks &&
              h.n_workgroups < 65536 && h.n_slices < 65536;
  a.magic_slices = div_magic((uint32_t)a.n_slices);
  a.magic_blocks = div_magic((uint32_t)a.row_blocks);
  for (int m0 = 0; m0 < M; m0 += kMaxTokens) {
    a.x = (const uint16_t*)x + (size_t)m0 * ldx;
    a.partials = workspace + (size_t)m0 * a.token_stride;
    a.sums = reinterpret_cast<unsigned long long*>(workspace) + (size_t)m0 * h.n;
    a.spill = workspace + 2 * (size_t)M * h.n + (size_t)m0 * h.n;
    a.y = (uint16_t*)y + (size_t)m0 * ldy;
    int rc;
    switch (M - m0 >= kMaxTokens ? kMaxTokens : M - m0) {
      case 1: rc = launch_sliced_tokens<ACT, 1>(a, h.n_workgroups, st, what); break;
      case 2: rc = launch_sliced_tokens<ACT, 2>(a, h.n_workgroups, st, what); break;
      case 3: rc = launch_sliced_tokens<ACT, 3>(a, h.n_workgroups, st, what); break;
      case 4: rc = launch_sliced_tokens<ACT, 4>(a, h.n_workgroups, st, what); break;
      case 5: rc = launch_sliced_tokens<ACT, 5>(a, h.n_workgroups, st, what); break;
      case 6: rc = launch_sliced_tokens<ACT, 6>(a, h.n_workgroups, st, what); break;
      default: rc = launch_sliced_tokens<ACT, 7>(a, h.n_workgroups, st, what); break;
    }
    if (rc != NPAMD_OK) return rc;
  }
  if (!a.fused_finish)
    sliced_reduce_kernel<ACT><<<dim3((h.n + 15) / 16, M), 256, 0, st>>>(workspace, h.n_partials, h.n, bias, y, ldy);
  return check_launch(what);
}

}  // namespace npamd

using namespace npamd;

// Argument checks shared by the two entry points.  `workspace` may be null on entry when the
// caller fetches it afterwards (the entry point that brings its own): then only the rest is checked.
static int check_sliced_call(const char* what, const void* x, int64_t ldx, const int32_t* column_perm,
                             const npamd_sliced_header* hp, const void* blob, const void* codebook,
                             int codebook_dtype, const void* y, int64_t ldy, int M, int act_dtype) {
  NPAMD_REQUIRE(hp != nullptr, "%s: header is null", what);
  const npamd_sliced_header h = *hp;
  NPAMD_REQUIRE(h.magic == kSlicedMagic && h.version == kSlicedVersion, "%s: not a slice-list header", what);
  NPAMD_REQUIRE(act_dtype == NPAMD_F16 || act_dtype == NPAMD_BF16,
                "%s: activations must be f16 or bf16 (got dtype code %d)", what, act_dtype);
  NPAMD_REQUIRE(codebook_dtype == act_dtype, "%s: the codebook must be in the activation dtype", what);
  NPAMD_REQUIRE(M >= 0 && M <= NPAMD_GEMV_MAX_M, "%s: M=%d exceeds the fused limit %d", what, M, NPAMD_GEMV_MAX_M);
  NPAMD_REQUIRE(h.n > 0 && h.k > 0 && h.vl == 8 && h.k % 8 == 0 && h.nc >= 1, "%s: bad layer shape in header", what);
  NPAMD_REQUIRE(h.slice_rows >= 1 && h.slice_rows <= kSlicedMaxSliceRows && h.groups_max >= 1 &&
                    h.groups_max <= kSlicedMaxGroups,
                "%s: slice geometry does not fit the kernel's LDS map", what);
  NPAMD_REQUIRE(h.n_workgroups >= 1 && h.n_partials >= 1, "%s: bad counts in header", what);
  NPAMD_REQUIRE(ldx >= h.k && ldy >= h.n, "%s: row stride smaller than the row", what);
  if (M == 0) return NPAMD_OK;
  NPAMD_REQUIRE(x && blob && codebook && y, "%s: null pointer", what);
  NPAMD_REQUIRE(ldx % 8 == 0 && (reinterpret_cast<uintptr_t>(x) % 16) == 0 &&
                    (reinterpret_cast<uintptr_t>(codebook) % 16) == 0 &&
                    (reinterpret_cast<uintptr_t>(blob) % 16) == 0 &&
                    (reinterpret_cast<uintptr_t>(column_perm) % 16) == 0,
                "%s: x, column_perm, codebook and blob must be 16-byte aligned (ldx a multiple of 8)", what);
  return NPAMD_OK;
}

static int run_sliced(const char* what, const void* x, int64_t ldx, const int32_t* column_perm,
                      const npamd_sliced_header& h, const void* blob, const void* codebook, const float* bias,
                      void* y, int64_t ldy, int M, int act_dtype, void* workspace, void* stream) {
  hipStream_t st = (hipStream_t)stream;
  if (act_dtype == NPAMD_BF16)
    return launch_sliced<NPAMD_BF16>(h, (const uint8_t*)blob, x, ldx, codebook, column_perm, bias, y, ldy, M, (float*)workspace, st, what);
  return launch_sliced<NPAMD_F16>(h, (const uint8_t*)blob, x, ldx, codebook, column_perm, bias, y, ldy, M, (float*)workspace, st, what);
}

extern "C" int npamd_vq_gemv_sliced(const void* x, int64_t ldx, const int32_t* column_perm,
                                    const npamd_sliced_header* hp, const void* blob, const void* codebook,
                                    int codebook_dtype, const float* bias, void* y, int64_t ldy, int M, int act_dtype,
                                    void* workspace, int64_t workspace_bytes, void* stream) {
  const char* what = "npamd_vq_gemv_sliced";
  const int rc = check_sliced_call(what, x, ldx, column_perm, hp, blob, codebook, codebook_dtype, y, ldy, M, act_dtype);
  if (rc != NPAMD_OK || M == 0) return rc;
  NPAMD_REQUIRE(workspace != nullptr && (reinterpret_cast<uintptr_t>(workspace) % 16) == 0,
                "%s: workspace must be a 16-byte aligned device pointer", what);
  NPAMD_REQUIRE(workspace_bytes >= npamd_vq_sliced_workspace_bytes(hp, M), "%s: workspace of %lld bytes, %lld needed",
                what, (long long)workspace_bytes, (long long)npamd_vq_sliced_workspace_bytes(hp, M));
  return run_sliced(what, x, ldx, column_perm, *hp, blob, codebook, bias, y, ldy, M, act_dtype, workspace, stream);
}

// ---- the same call for callers that cannot allocate ---------------------------------------
// The workspace lives in a device array of this library: every GPU the library runs on holds
// its own copy at its own address, which is looked up once per device, with that device
// current.  Static storage starts zero-filled, and every call hands the workspace back
// zero-filled, which is all the kernels ask of it.
static __device__ __align__(256) unsigned char scratch[NPAMD_SLICED_STATIC_WORKSPACE_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex scratch_mutex;
void* scratch_of_device[kMaxDevices];  // the device address of `scratch`, per device (null: not looked up yet)
bool scratch_suspect[kMaxDevices];     // a call on this device failed after it may have launched: zero before the next use

// The kernels count on a zero-filled workspace and hand it back zero-filled; a call that fails between
// two of its launches (more than seven tokens) cannot promise that.  A fill kernel, not a memset: the
// caller may be capturing a graph.
__global__ void __launch_bounds__(256) scratch_zero_kernel(u32x4* p, int n16) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < n16) p[i] = u32x4{0u, 0u, 0u, 0u};
}
}  // namespace

extern "C" int npamd_vq_gemv_sliced_static(const void* x, int64_t ldx, const int32_t* column_perm,
                                           const npamd_sliced_header* hp, const void* blob, const void* codebook,
                                           int codebook_dtype, const float* bias, void* y, int64_t ldy, int M,
                                           int act_dtype, void* stream) {
  const char* what = "npamd_vq_gemv_sliced_static";
  const int rc = check_sliced_call(what, x, ldx, column_perm, hp, blob, codebook, codebook_dtype, y, ldy, M, act_dtype);
  if (rc != NPAMD_OK || M == 0) return rc;
  const int64_t need = npamd_vq_sliced_workspace_bytes(hp, M);
  NPAMD_REQUIRE(need <= (int64_t)NPAMD_SLICED_STATIC_WORKSPACE_BYTES,
                "%s: this layer and token count need %lld bytes of workspace, the built-in one holds %lld "
                "(use npamd_vq_gemv_sliced with a workspace of your own)",
                what, (long long)need, (long long)NPAMD_SLICED_STATIC_WORKSPACE_BYTES);
  int device = -1;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return fail(NPAMD_ERR_LAUNCH, "%s: hipGetDevice: %s", what, hipGetErrorString(e));
  NPAMD_REQUIRE(device >= 0 && device < kMaxDevices, "%s: device %d outside the %d this library keeps track of", what,
                device, kMaxDevices);
  void* workspace = nullptr;
  {
    std::lock_guard<std::mutex> lock(scratch_mutex);
    if (scratch_of_device[device] == nullptr) {
      void* ptr = nullptr;
      e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
      if (e != hipSuccess || ptr == nullptr)
        return fail(NPAMD_ERR_LAUNCH, "%s: hipGetSymbolAddress: %s", what, hipGetErrorString(e));
      scratch_of_device[device] = ptr;
    }
    workspace = scratch_of_device[device];
    if (scratch_suspect[device]) {
      constexpr int n16 = NPAMD_SLICED_STATIC_WORKSPACE_BYTES / 16;
      scratch_zero_kernel<<<(n16 + 255) / 256, 256, 0, (hipStream_t)stream>>>((u32x4*)workspace, n16);
      const int zrc = check_launch(what);
      if (zrc != NPAMD_OK) return zrc;
      scratch_suspect[device] = false;
    }
  }
  const int run_rc = run_sliced(what, x, ldx, column_perm, *hp, blob, codebook, bias, y, ldy, M, act_dtype, workspace, stream);
  if (run_rc != NPAMD_OK) {
    std::lock_guard<std::mutex> lock(scratch_mutex);
    scratch_suspect[device] = true;
  }
  return run_rc;
}
