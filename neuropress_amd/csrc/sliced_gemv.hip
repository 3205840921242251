// Decode GEMV over the slice-list form of the indices (see sliced_format.hpp).
//
// One workgroup of 16 waves holds the activations of its group range (up to 4 KiB
// per token, up to seven tokens per launch), one 8192-row codebook slice (128 KiB)
// and a zero row in LDS.  Every lane owns one output row and
// walks the entries filed under (slice, group range, row): two 16-byte LDS reads
// (codebook row, activation vector) and four packed dot products per entry, the
// sum kept in registers.  Each lane then writes one float into the partial-sum
// vector of its (slice, group range); a second kernel adds the partial vectors
// of a row in a fixed order, adds the bias and rounds once.  No atomics: the
// result does not depend on timing.
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
  float* partials;  // [n_partials][n]
  int n, nc, slice_rows;
};

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

// Entry quads requested ahead per lane.  Measured on a 14336 x 4096 layer: 3 in flight 10.6 us,
// 8 in flight 12.1 us (the entries then arrive wave by wave instead of interleaved, and the
// last waves start working late).
constexpr int kQuadsInFlight = 3;
// LDS map: activations of the group range, then the slice, then the zero row that
// padding entries select.  Both bases fit the 16-bit offset field of an LDS read.
constexpr int kMaxTokens = 7;  // tokens per pass over the entries (an eighth token's activations would not fit in LDS)
constexpr int kLdsX = 0;       // [token][group] vectors: a token's 256 vectors are contiguous, so the
                               // lanes of a read spread over all sixteen 16-byte bank groups
constexpr int kLdsSlice = kSlicedMaxGroups * 16 * kMaxTokens;
constexpr int kLdsBytes = kLdsSlice + (kSlicedMaxSliceRows + 1) * 16;
static_assert(kLdsBytes <= kSlicedLdsBytes && kLdsSlice < 65536, "LDS map");

__device__ __forceinline__ void load_quad(Quad& q, const uint8_t* strip_lane, int qi) {
  __builtin_memcpy(&q, __builtin_assume_aligned(strip_lane + (size_t)qi * kSlicedQuadBytes, 4), 12);
}

template <uint32_t MASK>
__device__ __forceinline__ uint32_t low_field(uint32_t v) {
  uint32_t r;
  asm("v_and_b32 %0, %1, %2" : "=v"(r) : "s"(MASK), "v"(v));
  return r;
}

// The four entries of one quad.  A lane's record is four 16-bit rows followed by
// four 8-bit groups, so each LDS address is one field extracted and shifted: two
// instructions.  (Written as a plain mask, the low fields become shift + mask + add.)
// Per entry: one codebook row and M activation vectors from LDS, 4 M dot products.
template <int ACT, int M>
__device__ __forceinline__ void run_quad(const Quad& q, const uint8_t* lds, float (&acc)[M][2]) {
  const uint32_t row[4] = {low_field<0xFFFFu>(q.d0), q.d0 >> 16, low_field<0xFFFFu>(q.d1), q.d1 >> 16};
  const uint32_t grp[4] = {low_field<0xFFu>(q.d2), (q.d2 >> 8) & 0xFFu, (q.d2 >> 16) & 0xFFu, q.d2 >> 24};
  constexpr int kBatch = M > 2 ? 2 : 4;  // entries whose LDS reads are issued together
#pragma unroll
  for (int j0 = 0; j0 < 4; j0 += kBatch) {
    u32x4 c[kBatch], xv[kBatch][M];
#pragma unroll
    for (int j = 0; j < kBatch; ++j) {
      c[j] = *reinterpret_cast<const u32x4*>(lds + kLdsSlice + (row[j0 + j] << 4));
      const uint8_t* xg = lds + kLdsX + (grp[j0 + j] << 4);
#pragma unroll
      for (int m = 0; m < M; ++m) xv[j][m] = *reinterpret_cast<const u32x4*>(xg + m * (kSlicedMaxGroups * 16));
    }
#pragma unroll
    for (int j = 0; j < kBatch; ++j)
#pragma unroll
      for (int m = 0; m < M; ++m) acc[m][j & 1] = dot8<ACT>(c[j], xv[j][m], acc[m][j & 1]);
  }
}

template <int ACT, int M, bool PERM>
__global__ void __launch_bounds__(kSlicedTasks, 1) sliced_gemv_kernel(SlicedArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  u32x4* xl = reinterpret_cast<u32x4*>(lds + kLdsX);
  u32x4* cb = reinterpret_cast<u32x4*>(lds + kLdsSlice);
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const SlicedWorkgroup& wg = a.wgs[blockIdx.x];
  const int steps = (int)wg.wave[wave].steps;
  const int nq = (steps + 3) >> 2;  // a strip is padded to whole quads, so padded steps are run too
  const uint8_t* strip_lane = a.entries + (size_t)wg.wave[wave].quad_begin * kSlicedQuadBytes + (size_t)lane * 12;

  // Requests in the order they are needed: the slice and the activations (mostly
  // L2 hits) first, then the entries, which stream from HBM while the slice is
  // being stored and the first quads are worked on.
  Quad q[kQuadsInFlight];
  {
    const int slice_len = min(a.slice_rows, a.nc - (int)wg.slice * a.slice_rows);
    const u32x4* src = a.codebook + (int64_t)wg.slice * a.slice_rows;
    const int g_count = (int)wg.g_count;
    u32x4 t[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) t[i] = src[min(tid + i * kSlicedTasks, slice_len - 1)];
    // Thread t stages group t % 256 of tokens t / 256 and t / 256 + 4 (256 groups x 7 tokens at most).
    constexpr int kXLoads = M > 4 ? 2 : 1;
    const int xg = tid & (kSlicedMaxGroups - 1), xm = tid / kSlicedMaxGroups;
    const int xvec = (int)wg.g_begin + min(xg, g_count - 1);
    const uint16_t* xrow[kXLoads];
    u32x4 xt[kXLoads], perm_lo, perm_hi;
#pragma unroll
    for (int i = 0; i < kXLoads; ++i) xrow[i] = a.x + (int64_t)min(xm + 4 * i, M - 1) * a.ldx;
    if constexpr (PERM) {  // the eight source columns of this vector; the elements follow below
      perm_lo = reinterpret_cast<const u32x4*>(a.column_perm)[2 * xvec];
      perm_hi = reinterpret_cast<const u32x4*>(a.column_perm)[2 * xvec + 1];
    } else {
#pragma unroll
      for (int i = 0; i < kXLoads; ++i) xt[i] = reinterpret_cast<const u32x4*>(xrow[i])[xvec];
    }
    __builtin_amdgcn_sched_barrier(0);  // keep the entry requests behind the slice's
    // The first quads (past the strip's end: its last quad again, or quad 0
    // of the blob for a wave without a strip; no branch around a load).
#pragma unroll
    for (int i = 0; i < kQuadsInFlight; ++i) load_quad(q[i], strip_lane, max(min(i, nq - 1), 0));
    __builtin_amdgcn_sched_barrier(0);
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
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if (tid + i * kSlicedTasks < slice_len) cb[tid + i * kSlicedTasks] = t[i];
#pragma unroll
    for (int i = 0; i < kXLoads; ++i)
      if (xg < g_count && xm + 4 * i < M) xl[(xm + 4 * i) * kSlicedMaxGroups + xg] = xt[i];
    if (tid == kSlicedTasks - 1) cb[kSlicedPadRow] = u32x4{0u, 0u, 0u, 0u};  // what padding entries select
  }
  const uint32_t row = a.rowmap[(size_t)blockIdx.x * kSlicedTasks + tid];
  __syncthreads();

  // kQuadsInFlight quads stay in flight: each one is replaced by the quad that many
  // further on as soon as it has been read.
  float acc[M][2];
#pragma unroll
  for (int m = 0; m < M; ++m) acc[m][0] = acc[m][1] = 0.f;
  int q0 = 0;
  for (; q0 + 2 * kQuadsInFlight <= nq; q0 += kQuadsInFlight) {
#pragma unroll
    for (int i = 0; i < kQuadsInFlight; ++i) {
      const Quad cur = q[i];
      load_quad(q[i], strip_lane, q0 + i + kQuadsInFlight);
      run_quad<ACT, M>(cur, lds, acc);
    }
  }
#pragma unroll
  for (int i = 0; i < kQuadsInFlight; ++i) {
    if (q0 + i >= nq) break;
    const Quad cur = q[i];
    if (q0 + i + kQuadsInFlight < nq) load_quad(q[i], strip_lane, q0 + i + kQuadsInFlight);
    run_quad<ACT, M>(cur, lds, acc);
  }
  q0 += kQuadsInFlight;
#pragma unroll
  for (int i = 0; i < kQuadsInFlight; ++i) {
    if (q0 + i >= nq) break;
    run_quad<ACT, M>(q[i], lds, acc);
  }
  if (row != kSlicedNoRow) {
#pragma unroll
    for (int m = 0; m < M; ++m)
      a.partials[(size_t)m * a.token_stride + (size_t)wg.partial * a.n + row] = acc[m][0] + acc[m][1];
  }
}

// y[token][row] = round(sum over the partial vectors + bias).  16 rows per block
// (blockIdx.y = token); the partial vectors are dealt over 16 threads per row,
// whose sums are then added in a fixed order.
template <int ACT>
__global__ void __launch_bounds__(256) sliced_reduce_kernel(const float* __restrict__ partials, int n_partials,
                                                             int n, const float* __restrict__ bias,
                                                             void* __restrict__ y, int64_t ldy) {
  __shared__ float red[16][17];
  const int r = threadIdx.x & 15, j = threadIdx.x >> 4;
  const int row = blockIdx.x * 16 + r;
  partials += (size_t)blockIdx.y * n_partials * n;
  y = (uint16_t*)y + (size_t)blockIdx.y * ldy;
  float sum = 0.f;
  if (row < n)
    for (int p = j; p < n_partials; p += 16) sum += partials[(size_t)p * n + row];
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
  static int reserved = 0;
  if (reserved == 0) {
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&sliced_gemv_kernel<ACT, M, PERM>),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
    if (e != hipSuccess)
      return fail(NPAMD_ERR_LAUNCH, "%s: cannot reserve %d bytes of LDS: %s", what, kLdsBytes, hipGetErrorString(e));
    reserved = kLdsBytes;
  }
  sliced_gemv_kernel<ACT, M, PERM><<<n_workgroups, kSlicedTasks, kLdsBytes, st>>>(a);
  return NPAMD_OK;
}

template <int ACT, int M>
int launch_sliced_tokens(const SlicedArgs& a, int n_workgroups, hipStream_t st, const char* what) {
  return a.column_perm ? launch_sliced_tokens_p<ACT, M, true>(a, n_workgroups, st, what)
                       : launch_sliced_tokens_p<ACT, M, false>(a, n_workgroups, st, what);
}

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
  for (int m0 = 0; m0 < M; m0 += kMaxTokens) {
    a.x = (const uint16_t*)x + (size_t)m0 * ldx;
    a.partials = workspace + (size_t)m0 * a.token_stride;
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
  if (y)
    sliced_reduce_kernel<ACT><<<dim3((h.n + 15) / 16, M), 256, 0, st>>>(workspace, h.n_partials, h.n, bias, y, ldy);
  return check_launch(what);
}

}  // namespace npamd

using namespace npamd;

extern "C" int npamd_vq_gemv_sliced(const void* x, int64_t ldx, const int32_t* column_perm,
                                    const npamd_sliced_header* hp, const void* blob, const void* codebook,
                                    int codebook_dtype, const float* bias, void* y, int64_t ldy, int M, int act_dtype,
                                    void* workspace, int64_t workspace_bytes, void* stream) {
  const char* what = "npamd_vq_gemv_sliced";
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
  NPAMD_REQUIRE(x && blob && codebook && workspace, "%s: null pointer", what);
  NPAMD_REQUIRE(ldx % 8 == 0 && (reinterpret_cast<uintptr_t>(x) % 16) == 0 &&
                    (reinterpret_cast<uintptr_t>(codebook) % 16) == 0 &&
                    (reinterpret_cast<uintptr_t>(blob) % 16) == 0 &&
                    (reinterpret_cast<uintptr_t>(workspace) % 16) == 0 &&
                    (reinterpret_cast<uintptr_t>(column_perm) % 16) == 0,
                "%s: x, column_perm, codebook, blob and workspace must be 16-byte aligned (ldx a multiple of 8)", what);
  NPAMD_REQUIRE(workspace_bytes >= npamd_vq_sliced_workspace_bytes(&h, M), "%s: workspace of %lld bytes, %lld needed",
                what, (long long)workspace_bytes, (long long)npamd_vq_sliced_workspace_bytes(&h, M));
  hipStream_t st = (hipStream_t)stream;
  if (act_dtype == NPAMD_BF16)
    return launch_sliced<NPAMD_BF16>(h, (const uint8_t*)blob, x, ldx, codebook, column_perm, bias, y, ldy, M, (float*)workspace, st, what);
  return launch_sliced<NPAMD_F16>(h, (const uint8_t*)blob, x, ldx, codebook, column_perm, bias, y, ldy, M, (float*)workspace, st, what);
}
