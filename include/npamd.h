/*
 * npamd.h -- C ABI of libnpamd.so: the MI355X (gfx950) backend for
 * neuropress's quantized-linear forward path.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless the comment says otherwise;
 *   - the library never allocates, frees or keeps a pointer after return;
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream);
 *     launches are asynchronous, nothing here synchronises;
 *   - return value 0 = success, negative = NPAMD_ERR_*; npamd_last_error()
 *     then returns a thread-local human-readable message;
 *   - dtype codes: NPAMD_F16 / NPAMD_BF16 / NPAMD_F32;
 *   - x is [M, K] with row stride ldx (elements), y is [M, N] with row stride
 *     ldy; weights are never materialised by the gemv / gemm_tile entry points.
 *
 * Index bit-stream ("packed"): index i occupies bits [i*bits, (i+1)*bits) of a
 * byte stream, LSB first; flat index of (row n, group g) is n*(K/VL)+g.
 * Codebooks are fp16 [NC, VL] row-major (NPAMD_F16), or -- for the gemv /
 * gemm_tile entry points only -- already cast to the activation dtype.
 *
 * Paths are relative to the reference repository (DreamerMind/neuropress).
 */
#ifndef NPAMD_H
#define NPAMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NPAMD_F16 0
#define NPAMD_BF16 1
#define NPAMD_F32 2

#define NPAMD_OK 0
#define NPAMD_ERR_INVALID (-1)     /* bad argument (shape, dtype, null, alignment) */
#define NPAMD_ERR_UNSUPPORTED (-2) /* valid request this build has no kernel for */
#define NPAMD_ERR_LAUNCH (-3)      /* HIP reported an error at launch */

/* Largest token count the fused decode-GEMV entry points accept.  Up to 16 tokens are one MFMA
 * operand; 17..32 reuse every decoded weight operand for two (the slice-list, prefix-coded and
 * element-wise kernels take further passes over the weight instead). */
#define NPAMD_GEMV_MAX_M 32

/* Library ABI version (bumped on any signature change). */
int npamd_version(void);

/* Thread-local message for the last failing call on this thread ("" if none). */
const char* npamd_last_error(void);

/* ---------------------------------------------------------------- VQ ---- */

/*
 * One-pass decode: out.flat[v*VL + j] = cast(codebook[idx(v), j]).
 * Replaces vq_dequant (neuropress/kernels/vq_dequant.cu:105-146) and
 * dequantize_vq_weight (neuropress/kernels/vq_linear.cu:458-479).
 * bits in [4, 20]; out_dtype any of the three; out holds n_vectors*VL elements.
 */
int npamd_vq_dequant(const uint8_t* packed, int64_t n_bytes, int bits,
                     const void* codebook_f16, int nc, int vl,
                     int64_t n_vectors, void* out, int out_dtype, void* stream);

/*
 * Fused decode GEMV, M <= NPAMD_GEMV_MAX_M:
 *   y[m, n] = sum_k x[m, k] * codebook[idx(n, k/VL), k%VL] (+ bias[n]), f32 accumulate.
 * Replaces vq_linear (neuropress/kernels/vq_linear.cu:344-424) and the GEMV
 * branch of vq_linear_wmma (neuropress/kernels/vq_linear_wmma.cu:187-240, 468-540).
 * act_dtype: NPAMD_F16 or NPAMD_BF16 (x and y).  codebook_dtype: NPAMD_F16, or
 * the activation dtype when the caller pre-cast the codebook.  bias: f32 [N] or NULL.
 */
int npamd_vq_gemv(const void* x, int64_t ldx, const uint8_t* packed, int64_t n_bytes,
                  int bits, const void* codebook, int codebook_dtype, int nc, int vl,
                  const float* bias, void* y, int64_t ldy, int M, int N, int K,
                  int act_dtype, void* stream);

/*
 * The same GEMV with the reference's column permutation folded in:
 *   y[m, n] = sum_k x[m, column_perm[k]] * W[n, k] (+ bias[n]),
 * i.e. vq_linear applied to x[..., column_perm] (neuropress/nn/np_vq_linear.py:1027-1028)
 * without the separate gather kernel.  column_perm: K int32 column numbers, each < K,
 * 16-byte aligned.  Every workgroup copies the M rows of x into LDS and permutes them there,
 * so this entry point takes M <= 16 tokens, M * K <= 16384 elements, VL = 8 or 4,
 * 4/8/12/16-bit indices and K % 64 == 0 only;
 * other requests return NPAMD_ERR_UNSUPPORTED (gather x yourself and call npamd_vq_gemv).
 */
int npamd_vq_gemv_perm(const void* x, int64_t ldx, const int32_t* column_perm,
                       const uint8_t* packed, int64_t n_bytes, int bits,
                       const void* codebook, int codebook_dtype, int nc, int vl,
                       const float* bias, void* y, int64_t ldy, int M, int N, int K,
                       int act_dtype, void* stream);

/* 1 when npamd_vq_gemv_perm takes this shape AND its LDS copies of x do not cost the kernel
 * workgroups per compute unit (then it beats a separate gather by about 2.5 us per call);
 * 0 otherwise: gather x yourself and call npamd_vq_gemv.  Host-only arithmetic. */
int npamd_vq_gemv_perm_supported(int M, int N, int K, int nc, int vl, int bits);

/* 1 when the MFMA kernels behind npamd_vq_gemv / npamd_vq_gemm_tile (and the residual forms) take
 * a layer of this shape (VL = 8, K % 64 == 0, index width 4 / 8 / 12 / 16), pointer alignment
 * aside; 0 when they would run their element-wise fallback, which decodes the weight once per 16
 * tokens: beyond 16 tokens decode once (npamd_vq_dequant) and use a dense GEMM instead, as the
 * reference does for shapes its kernels do not take (neuropress/nn/np_vq_linear.py:1127-1148).
 * Host-only arithmetic. */
int npamd_vq_fused_supported(int K, int vl, int bits);

/* 1 when a fused GEMV call of M tokens on an N x K layer runs the kernel that stages every step's
 * activations through LDS: npamd_vq_gemv on a layer with a codebook of `nc` rows of eight (nc > 0),
 * or npamd_q_gemv (nc = 0).  Such a call stays ahead of the tile GEMM up to the GEMV's 32 tokens
 * whatever K is, which is what the callers' band thresholds ask (the reference fixes its own
 * thresholds per backend, neuropress/nn/np_vq_linear.py:73-98).  The answer is the launcher's own:
 * it is run up to the point of the launch.  Host-only arithmetic. */
int npamd_gemv_stages_activations(int M, int N, int K, int nc);

/*
 * Tile-decode MFMA GEMM, any M >= 1: same contraction, weight tiles decoded
 * inside the kernel, dense weight never written.
 * Replaces vq_gemm_triton (neuropress/kernels/vq_triton.py:119-179) and the
 * WMMA GEMM branch of vq_linear_wmma (neuropress/kernels/vq_linear_wmma.cu:261-394).
 * `workspace` (all three *_gemm_tile entry points): NULL, or 16-byte aligned device
 * memory of npamd_gemm_tile_workspace_bytes(M, N, K) bytes.  With it, layers
 * whose column blocks would not fill the GPU split K over more workgroups, which
 * hand their f32 partial tiles over through it: two parts meet inside the kernel
 * (whichever finishes second adds the other's tile), more are added by a second
 * kernel; without it, or when it is too small, K is not split.  Contents
 * irrelevant before and after (nobody clears it); two calls that may run at the
 * same time need a workspace each.
 */
int npamd_vq_gemm_tile(const void* x, int64_t ldx, const uint8_t* packed, int64_t n_bytes,
                       int bits, const void* codebook, int codebook_dtype, int nc, int vl,
                       const float* bias, void* y, int64_t ldy, int M, int N, int K,
                       int act_dtype, void* workspace, int64_t workspace_bytes, void* stream);

/* Bytes of workspace the *_gemm_tile entry points can use for this shape (0: K is not split). */
int64_t npamd_gemm_tile_workspace_bytes(int M, int N, int K);

/*
 * Widen a bit-stream to one uint16 per index (the layout the fast kernels
 * stream at bits=16).  Same stream semantics as unpack_indices
 * (neuropress/kernels/kmeans_assign.cu:405-451); bits in [4, 16].
 */
int npamd_vq_widen_u16(const uint8_t* packed, int64_t n_bytes, int bits,
                       int64_t n_indices, uint16_t* out, void* stream);

/*
 * Gather phase of the look-up-table formulation: y[m, j] = sum_g lut[m, g, idx(j, g)] in float32,
 * where the caller built lut[m, g, c] = x[m, g*VL:(g+1)*VL] . codebook[c] with one matrix product.
 * Replaces vq_lut_gather (neuropress/kernels/__init__.py:405-433, kernels/vq_linear_lut.cu:121-142).
 * lut: f32 [M, groups, NC]; y: f32 [M, N]; bits in [4, 20]; indices beyond NC - 1 are clamped.
 * The modules do not use this path (the table is M * K/VL * NC floats: 128 MiB per token for a
 * 4096-wide layer with 65536 codebook rows); it is kept for callers of the reference's wrapper.
 */
int npamd_vq_lut_gather(const float* lut, const uint8_t* packed, int64_t n_bytes, int bits,
                        float* y, int M, int N, int groups, int nc, void* stream);

/* ------------------------------------- slice-list form of the indices ---- */
/*
 * For codebooks too large for a compute unit's LDS (more than 4096 rows) the
 * decode GEMV is bound by random 16-byte codebook lookups in L2.  The slice-list
 * form files every index under the 4096-row codebook slice it points into, so a
 * workgroup that holds one slice in LDS only sees the lookups that hit it; every
 * lane sums the entries of one output row in a register.  It is
 * built once per layer from the packed stream (a construction-time re-layout,
 * as the reference pre-unpacks embedding indices to an int16 table,
 * neuropress/nn/np_vq_embedding.py:244-246) and used by npamd_vq_gemv_sliced.
 * The format itself has no counterpart in the reference.
 *
 * The blob starts with this header; the rest is described in
 * neuropress_amd/csrc/sliced_format.hpp.  All offsets are bytes from the start.
 */
typedef struct npamd_sliced_header {
  uint32_t magic;         /* "NPSL" */
  uint32_t version;
  int32_t n, k, vl, nc;   /* the layer the blob was built for */
  int32_t slice_rows;     /* codebook rows per slice */
  int32_t n_slices;
  int32_t n_workgroups;   /* grid size of the GEMV */
  int32_t n_partials;     /* partial-sum vectors per output row */
  int32_t groups_max;     /* largest group range of a workgroup */
  uint32_t flags;         /* bit 0: workgroup w works on codebook slice w % n_slices */
  int64_t n_quads;        /* 768-byte entry quads = n_workgroups * (sum of wave_quads) */
  int64_t n_entries;      /* real (non-padding) entries = N * K / VL */
  int64_t off_workgroups, off_rowmap, off_entries;
  int64_t total_bytes;
  uint16_t wave_quads[16]; /* entry quads of wave w's strip, the same in every workgroup */
} npamd_sliced_header;

/*
 * HOST function: build the slice-list blob from a packed index stream in host
 * memory.  `target_workgroups` = compute units to fill (0 = 256).  Writes the
 * size to *blob_bytes; if `blob` is NULL or `capacity` is too small nothing else
 * is written and NPAMD_ERR_INVALID is returned when blob != NULL.
 * Call once with blob = NULL for the size, then with a buffer.  VL must be 8.
 */
int npamd_vq_sliced_build(const uint8_t* packed_host, int64_t n_bytes, int bits,
                          int N, int K, int vl, int nc, int target_workgroups,
                          void* blob_host, int64_t capacity, int64_t* blob_bytes);

/*
 * HOST function: structural check of a blob in host memory (offsets inside
 * total_bytes, every row / group / slice field in range, every index filed
 * exactly once).  A blob that passes cannot make
 * npamd_vq_gemv_sliced read outside the blob, the codebook or its LDS arrays.
 */
int npamd_vq_sliced_check(const void* blob_host, int64_t blob_bytes);

/* Bytes of workspace npamd_vq_gemv_sliced needs for M tokens (zero-filled by the caller once). */
int64_t npamd_vq_sliced_workspace_bytes(const npamd_sliced_header* header_host, int M);

/*
 * Decode GEMV over the slice-list form, M <= NPAMD_GEMV_MAX_M (up to seven tokens
 * share one pass over the entries; more tokens take further passes):
 *   y[m, n] = sum_k x[m, k] * codebook[idx(n, k/VL), k%VL] (+ bias[n]).
 * `header_host` is a host copy of the blob's header, `blob` the whole blob in
 * device memory.  The codebook must be in the activation dtype.  `workspace`
 * is device memory of npamd_vq_sliced_workspace_bytes() bytes, 16-byte aligned,
 * ZERO-FILLED before its first use; every call hands it back zero-filled, so calls
 * that follow each other on one stream may share it (calls that overlap must not).
 * A row's result is spread over the workgroups that hold the codebook slices its
 * indices point into.  With fewer than 256 of them per row (any codebook of up to
 * 2^16 rows) every lane adds its partial sum, as a fixed-point number in units of
 * 2^-24, to a 64-bit word of the workspace with one atomic; the lane that completes
 * a row's count adds the bias, rounds once and stores y -- one kernel, and the sum
 * does not depend on the order of arrival.  The rounding of the partial sums adds an absolute
 * error of at most n_partials * 2^-25 (n_partials from the header: 4.8e-7 at 16) to the float32
 * sum, whatever the magnitude of y: outputs far below 1e-4 lose relative precision against a
 * float32 accumulation.  Partial sums of magnitude 2^15 or more, NaN and infinities go through a
 * float accumulator with a float atomic: a row with two or more of those may differ in its last
 * bits from run to run.  Otherwise the partial sums are written out and a
 * second kernel adds them in a fixed order.
 * `column_perm`: NULL, or K int32 column numbers (16-byte aligned, each < ldx):
 * the kernel then reads x[m, column_perm[k]] wherever it would read x[m, k],
 * i.e. the x[..., column_perm] the reference applies before every VQ matmul
 * (neuropress/nn/np_vq_linear.py:1027-1028) without a separate gather kernel.
 */
int npamd_vq_gemv_sliced(const void* x, int64_t ldx, const int32_t* column_perm,
                         const npamd_sliced_header* header_host,
                         const void* blob, const void* codebook, int codebook_dtype,
                         const float* bias, void* y, int64_t ldy, int M, int act_dtype,
                         void* workspace, int64_t workspace_bytes, void* stream);

/*
 * npamd_vq_gemv_sliced for callers that cannot allocate device memory or pass a workspace along:
 * code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no
 * counterpart in the reference.  The workspace is a device array inside this library,
 * NPAMD_SLICED_STATIC_WORKSPACE_BYTES long, which every GPU the library runs on holds until the
 * process ends; the call allocates and frees nothing (the array's address is looked up on the
 * first call on each device, so make that call before a capture begins).  Requests whose
 * npamd_vq_sliced_workspace_bytes() exceeds the array are rejected with NPAMD_ERR_INVALID.
 * All calls on one GPU share the array: it starts zero-filled and every call hands it back
 * zero-filled, so calls that follow each other (on one stream, or ordered by events) are
 * fine, and calls that overlap on one GPU race.  A call that returns an error after it may have
 * launched part of its work leaves the array suspect; the next call on that GPU zero-fills it
 * (a kernel on the caller's stream, not a memset) before it uses it.  Same arguments and results
 * as npamd_vq_gemv_sliced otherwise.
 */
#define NPAMD_SLICED_STATIC_WORKSPACE_BYTES (4 * 1024 * 1024)
int npamd_vq_gemv_sliced_static(const void* x, int64_t ldx, const int32_t* column_perm,
                                const npamd_sliced_header* header_host,
                                const void* blob, const void* codebook, int codebook_dtype,
                                const float* bias, void* y, int64_t ldy, int M, int act_dtype,
                                void* stream);

/*
 * Decode GEMV over a prefix-coded index stream, read as it is stored (M <= NPAMD_GEMV_MAX_M):
 *   y[m, n] = sum_k x[m, k] * codebook[idx(n, k/VL), k%VL] (+ bias[n]).
 * Replaces vq_linear_tiered / vq_linear_ntier / vq_linear_zero_escape
 * (neuropress/kernels/__init__.py:589-659, 711-762, 974-1049; kernels/vq_linear_tiered.cu,
 * vq_linear_ntier.cu, vq_linear_zero_escape.cu): one entry point for the three formats of
 * neuropress/transforms/vq_packing.py:298-1384, whose streams the caller passes separately, with
 * the per-row cumulative class counts ([N + 1] int32 each) of the packers' compute_row_offsets.
 *   flat = 0: n_classes - 1 cascaded one-bit class streams (stream k: one bit per index not
 *             claimed by classes < k, 0 = class k).  Two-tier: n_classes = 2, bases {0, 0};
 *             n-tier: bases {0, 2^bits[0], 2^bits[1], ...}.
 *   flat = 1: one stream of two class bits per index, n_classes = 4 (zero-escape: widths
 *             {0, 4, 8, cold_bits}, bases {0, 1, 17, 257}).
 * Index = payload_base[c] + the payload_bits[c]-bit field number (row_offsets[c][n] + rank of the
 * index among the row's class-c indices) of payload_streams[c]; a width of 0 means no payload.
 * The pointer arrays are host arrays of device pointers.  The codebook must be in the activation
 * dtype.  One wave per output row, wave64 ballot + population count for the ranks.
 */
int npamd_vq_gemv_coded(const void* x, int64_t ldx, int flat, int n_classes,
                        const uint8_t* const* class_streams, const int64_t* class_bytes,
                        const uint8_t* const* payload_streams, const int64_t* payload_bytes,
                        const int* payload_bits, const uint32_t* payload_base,
                        const int32_t* const* row_offsets, const void* codebook, int codebook_dtype,
                        int nc, int vl, const float* bias, void* y, int64_t ldy, int M, int N, int K,
                        int act_dtype, void* stream);

/* ------------------------------------------------- residual VQ (RVQ) ---- */
/*
 * Two codebooks + per-output-row fp16 scale and bias (no counterpart in the
 * reference; the benchmark's residual-VQ configuration):
 *   W[n, g*VL+j] = f16(f16(f16(Cm[im(n,g),j] + Cr[ir(n,g),j]) * s[n]) + b[n])
 * row_scale / row_bias: fp16 [N] or NULL.  Both codebooks fp16, same VL.
 */
int npamd_rvq_dequant(const uint8_t* packed_main, int64_t n_bytes_main, int bits_main,
                      const uint8_t* packed_res, int64_t n_bytes_res, int bits_res,
                      const void* cb_main_f16, int nc_main, const void* cb_res_f16, int nc_res,
                      const void* row_scale_f16, const void* row_bias_f16, int vl,
                      int N, int K, void* out, int out_dtype, void* stream);

int npamd_rvq_gemv(const void* x, int64_t ldx,
                   const uint8_t* packed_main, int64_t n_bytes_main, int bits_main,
                   const uint8_t* packed_res, int64_t n_bytes_res, int bits_res,
                   const void* cb_main_f16, int nc_main, const void* cb_res_f16, int nc_res,
                   const void* row_scale_f16, const void* row_bias_f16, int vl,
                   const float* bias, void* y, int64_t ldy, int M, int N, int K,
                   int act_dtype, void* stream);

int npamd_rvq_gemm_tile(const void* x, int64_t ldx,
                        const uint8_t* packed_main, int64_t n_bytes_main, int bits_main,
                        const uint8_t* packed_res, int64_t n_bytes_res, int bits_res,
                        const void* cb_main_f16, int nc_main, const void* cb_res_f16, int nc_res,
                        const void* row_scale_f16, const void* row_bias_f16, int vl,
                        const float* bias, void* y, int64_t ldy, int M, int N, int K,
                        int act_dtype, void* workspace, int64_t workspace_bytes, void* stream);

/* ------------------------------------------- group-affine n-bit (Q4) ---- */
/*
 * w_pack: uint8 [N, K/vpb], vpb = 8/nbits, value k of row n =
 *   (w_pack[n, k/vpb] >> ((k%vpb)*nbits)) & mask   (low nibble = even k);
 * scale: fp16 [N*(K/group_size)]; zero_point: fp16 same shape or NULL
 * (symmetric: zp = 2^(nbits-1));  w = (float(q) - zp) * float(scale), f32.
 */

/*
 * Decode to a dense [N, K] weight, one RNE rounding to out_dtype.
 * Restates the decode half of _q_dequant_linear (neuropress/nn/np_linear.py:333-353).
 */
int npamd_q_dequant(const uint8_t* w_pack, const void* scale_f16, const void* zero_point_f16,
                    int N, int K, int nbits, int group_size, void* out, int out_dtype,
                    void* stream);

/* 1 when the MFMA kernels behind npamd_q_gemv / npamd_q_gemm_tile take the layer (4 or 8 bits, with or
 * without zero points, group size 32 * 2^j, K % 64 == 0), pointer alignment aside; 0 when they would
 * run the element-wise fallback (1 / 2 bits, other group sizes), which decodes the weight once per
 * 16 tokens: beyond 16 tokens use npamd_q_dequant and a dense GEMM.  The reference runs its one GEMV
 * kernel at every token count (neuropress/kernels/q4_linear.cu:137-139).  Host-only arithmetic. */
int npamd_q_fused_supported(int K, int nbits, int group_size);

/*
 * Fused dequant GEMV, M <= NPAMD_GEMV_MAX_M.
 * Replaces q_linear (neuropress/kernels/q4_linear.cu:80-131, 179-253).
 */
int npamd_q_gemv(const void* x, int64_t ldx, const uint8_t* w_pack, const void* scale_f16,
                 const void* zero_point_f16, const float* bias, void* y, int64_t ldy,
                 int M, int N, int K, int nbits, int group_size, int act_dtype, void* stream);

/*
 * Fused dequant MFMA GEMM, any M.  The reference has no kernel of its own here
 * (it defers to the third-party gemlite: neuropress/nn/np_linear.py:763-776).
 */
int npamd_q_gemm_tile(const void* x, int64_t ldx, const uint8_t* w_pack, const void* scale_f16,
                      const void* zero_point_f16, const float* bias, void* y, int64_t ldy,
                      int M, int N, int K, int nbits, int group_size, int act_dtype,
                      void* workspace, int64_t workspace_bytes, void* stream);

/* ------------------------------------- neighbours of the linear on a decode step ---- */
/*
 * Fused RMSNorm over the last dimension, one pass over x:
 *   out[m, i] = round(x[m, i] * rsqrt(mean_i(x[m, i]^2) + eps) * weight[i]),  f32 arithmetic.
 * Replaces rms_norm (neuropress/kernels/rms_norm.cu:27-110).  x, weight, out share `dtype`
 * (NPAMD_F16 / NPAMD_BF16 / NPAMD_F32); ldx, ldo are row strides in elements.
 */
int npamd_rms_norm(const void* x, int64_t ldx, const void* weight, void* out, int64_t ldo,
                   int M, int H, float eps, int dtype, void* stream);

/*
 * Embedding lookup in a VQ-compressed table (NPVQEmbedding.forward,
 * neuropress/nn/np_vq_embedding.py:120-142):
 *   row[t, g*VL + v] = codebook[indices[ids[t], g], v]
 *   out[t, j] = cast(f16(row[t, inv_perm[j]] * scale))
 * `indices`: [vocab, groups] 16-bit indices (read as unsigned); `inv_perm`: NULL or `groups*VL`
 * int32 column numbers; the multiply is skipped (no rounding) when scale == 1.  ids outside
 * [0, vocab) are clamped.  out: [n_ids, groups*VL] of out_dtype.
 */
int npamd_vq_embedding(const int64_t* ids, int64_t n_ids, const int16_t* indices, int64_t vocab,
                       int groups, const void* codebook_f16, int nc, int vl,
                       const int32_t* inv_perm, float scale, void* out, int out_dtype, void* stream);

/*
 * Embedding lookup in a group-affine n-bit table, n in {1, 2, 4, 8} (_emb_dequant and
 * NPEmbedding.forward, neuropress/nn/np_embedding.py:120-183, 455-473):
 *   v = f16((q - zp) * scale) in f32 arithmetic (zp = 2^(n-1) when zero_point_f16 is NULL),
 *   v = 0 where ids[t] == padding_idx (pass -1 for none),
 *   out = round(cast(v) * embed_scale), the multiply skipped when embed_scale == 1.
 * w_pack: [vocab, dim * n / 8] codes, low bits first; scale / zero point: [vocab * dim / group_size] f16.
 */
int npamd_q_embedding(const int64_t* ids, int64_t n_ids, const uint8_t* w_pack,
                      const void* scale_f16, const void* zero_point_f16, int nbits, int group_size,
                      int64_t vocab, int dim, int64_t padding_idx, float embed_scale,
                      void* out, int out_dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* NPAMD_H */
