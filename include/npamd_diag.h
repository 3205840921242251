/*
 * Measurement aids of libnpamd.so -- NOT part of the drop-in contract of npamd.h.
 *
 * Nothing here has a counterpart in the reference.  The benchmark uses these entry points to
 * measure, in the same run as the kernels, what bounds them on this machine (a plain read of the
 * same bytes, one table lookup per index, the matrix pipe alone), and the tests use
 * npamd_diag_reload_tuning to force kernel variants.  A binding of the reference needs none of them.
 */
#ifndef NPAMD_DIAG_H
#define NPAMD_DIAG_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/*
 * Results are discarded; `sink16` is a 16-byte device buffer.  All return 0 or a negative NPAMD_ERR_* code.
 *
 * npamd_diag_stream_read: read `n_bytes` (multiple of 16) once.
 * npamd_diag_gather: stream `n_indices` uint16 indices (multiple of 8) and fetch
 *   one 16-byte row of `table16` per index (index masked to `table_entries`, a
 *   power of two), from global memory or, with from_lds != 0, from an LDS copy
 *   of the table (at most 8192 rows).
 * npamd_diag_mfma: `blocks` workgroups of four waves (one per SIMD) each issue `mfmas_per_wave`
 *   (rounded up to a multiple of 12) independent MFMA 32x32x16 (act_dtype NPAMD_F16 / NPAMD_BF16)
 *   on operands read from `operands` (7 KiB of device memory, any finite values) and nothing
 *   else: the time the matrix pipes alone need for that many flops.
 *
 * npamd_diag_last_gemv_staged: 1 / 0 when the calling thread's last fused GEMV launch (npamd_vq_gemv,
 *   npamd_q_gemv and their variants) was / was not of a kernel that stages activations in LDS, -1
 *   before the first; npamd_gemv_stages_activations (npamd.h) must predict it.
 *
 * npamd_diag_reload_tuning: the NPAMD_* tuning environment variables are read once, at the first
 *   launch; this reads them again.  For tests and tuning runs only: it must not run while
 *   another thread launches.
 */
void npamd_diag_reload_tuning(void);
int npamd_diag_last_gemv_staged(void);
int npamd_diag_stream_read(const void* src, int64_t n_bytes, void* sink16, void* stream);
int npamd_diag_gather(const void* idx_u16, int64_t n_indices, const void* table16,
                      int table_entries, int from_lds, void* sink16, void* stream);
int npamd_diag_mfma(const void* operands, int blocks, int mfmas_per_wave, int act_dtype, void* sink16, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* NPAMD_DIAG_H */
