// Library-level entry points: version, thread-local error text, launch check.
#include <stdarg.h>
#include <stdio.h>

#include <stdlib.h>

#include "../../include/npamd_diag.h"
#include "gemm_tile2.hpp"
#include "gemv.hpp"

namespace npamd {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int check_launch(const char* what) {
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(NPAMD_ERR_LAUNCH, "%s: launch failed: %s", what, hipGetErrorString(e));
  return NPAMD_OK;
}

const char* error_text() { return g_err; }

static int env_int(const char* name, int dflt) {
  const char* v = getenv(name);
  return (v && *v) ? atoi(v) : dflt;
}

// The NPAMD_* tuning variables, read once per process (initialisation of a function-local
// static is thread-safe); launches only read the table.  npamd_diag_reload_tuning() reads them
// again, for tests and tuning runs that change them between launches.
static Tuning read_tuning() {
  Tuning t;
  t.gemv_lds_cb = env_int("NPAMD_GEMV_LDS_CB", 1);
  t.tile_lds_cb = env_int("NPAMD_TILE_LDS_CB", 1);
  t.gemv_lds_x = env_int("NPAMD_GEMV_LDS_X", 0);
  t.gemv_r = env_int("NPAMD_GEMV_R", 0);
  t.gemv_spw = env_int("NPAMD_GEMV_SPW", 0);
  t.gemv_parts = env_int("NPAMD_GEMV_PARTS", 0);
  t.gemv_xstage = env_int("NPAMD_GEMV_XSTAGE", 1);
  t.tile_splits = env_int("NPAMD_TILE_SPLITS", 0);
  t.tile_mw = env_int("NPAMD_TILE_MW", 0);
  t.tile_wide = env_int("NPAMD_TILE_WIDE", 1);
  t.q4_rows = env_int("NPAMD_Q4_ROWS", 0);
  t.q4_rowwise = env_int("NPAMD_Q4_ROWWISE", 1);
  t.q4_rowwise_bf16 = env_int("NPAMD_Q4_ROWWISE_BF16", 0);
  t.q4_stream = env_int("NPAMD_Q4_STREAM", 1);
  return t;
}

static Tuning& tuning_table() {
  static Tuning table = read_tuning();
  return table;
}

const Tuning& tuning() { return tuning_table(); }

static int device_cu_count() {
  // Looked up at most a few times per process (racing first callers all store the same value).
  static std::atomic<int> cached{0};
  int cus = cached.load(std::memory_order_relaxed);
  if (cus == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess)
      cus = prop.multiProcessorCount;
    if (cus <= 0) cus = 256;
    cached.store(cus, std::memory_order_relaxed);
  }
  return cus;
}

// One "job" = one 16-row tile x one 256-k step.  The kernel lasts about one
// HBM round trip, so the plan aims at every job's packed bytes being requested
// as soon as the grid starts: jobs per wave is kept near jobs / (16 waves * CUs).
// NPAMD_GEMV_R / NPAMD_GEMV_SPW override the choice (tuning aid).
bool gemv_lds_codebook_enabled() { return tuning().gemv_lds_cb != 0; }
bool tile_lds_codebook_enabled() { return tuning().tile_lds_cb != 0; }
bool gemv_lds_activations_forced() { return tuning().gemv_lds_x != 0; }
// One row tile per block, us, straight from memory / staged: int4 4096 x 4096 6.6 / 6.6 at 2 tokens,
// 6.9 / 6.5 at 4, 7.9 / 6.6 at 8, 9.2 / 7.5 at 16, 13.2 / 9.0 at 32; 4096 x 14336 17.5 / 15.7 at 4,
// 20.5 / 16.2 at 8, 27.5 / 18.9 at 16, 38.7 / 25.4 at 32; 65536-row codebook 4096 x 14336 35.8 / 34.6
// at 4, 37.8 / 35.4 at 8, 42.4 / 37.6 at 16, 52 / 41 at 32.  With more row tiles per block
// (14336 x 4096) or the table in LDS it does not pay.
int& last_gemv_staged() {
  static thread_local int staged = -1;
  return staged;
}

bool gemv_stage_activations(int M) {
  const int mode = tuning().gemv_xstage;
  return mode >= 2 || (mode == 1 && M >= 3);
}

GemvPlan plan_gemv(int N, int chunks, int max_r, int max_waves_cap) {
  const int steps = (chunks + 3) / 4;
  const int tiles = (N + 15) / 16;
  const int64_t jobs = (int64_t)tiles * steps;
  const int cus = device_cu_count();
  const int64_t target_waves = (int64_t)cus * 16;
  int jpw = (int)((jobs + target_waves - 1) / target_waves);
  if (jpw < 1) jpw = 1;
  GemvPlan p;
  // Row tiles of one block share the x operands (every block reads all of x, from L2: with R
  // tiles per block that traffic, which passes the weight bytes at a few tokens, drops R-fold)
  // and one copy of the codebook in LDS.  The largest R that leaves blocks for at least 0.6 of
  // the compute units wins at every token count, measured on N = 2048 ... 28672.
  p.R = (tiles * 10 >= cus * 24) ? 4 : (tiles * 10 >= cus * 12) ? 2 : 1;
  if (p.R > max_r) p.R = max_r;
  int spw = (jpw + p.R - 1) / p.R;
  const int r_env = tuning().gemv_r;
  if (r_env == 1 || r_env == 2 || r_env == 4) p.R = r_env;
  const int spw_env = tuning().gemv_spw;
  if (spw_env > 0) spw = spw_env;
  int max_waves = p.R >= 4 ? 8 : 16;
  if (max_waves > max_waves_cap) max_waves = max_waves_cap;
  if ((steps + spw - 1) / spw > max_waves) spw = (steps + max_waves - 1) / max_waves;
  p.steps_per_wave = spw;
  p.waves = (steps + spw - 1) / spw;
  return p;
}

// Measured, one token, 16 rows per block against 8 / 4 (us): residual VQ 1024 x 4096 7.7 -> 4.4,
// 65536-row codebook 1024 x 4096 8.4 -> 4.8, 2048 x 4096 9.2 -> 7.1 and 1024 x 1024 3.8 -> 3.3,
// int4 1024 x 4096 at two tokens 5.8 -> 3.8, 2048 x 8192 with a 4096-row table in LDS 6.5 -> 5.5,
// 2048 x 4096 with it 5.0 -> 4.5; but 2048 x 2048 and 512 x 2048 with that table 4.2 -> 4.4 and
// 4.15 -> 4.9 (every block copies the 64 KiB first, and there are then two or four times as
// many), 4096 x 4096 (whole tiles cover the compute units) 5.3 -> 5.5.  Hence: K of at least 512
// per part, whole tiles leave a quarter of the compute units empty, and a block keeps at least
// one lookup per row of the table it copies.
int plan_gemv_parts(int M, int N, int chunks, int lds_rows) {
  const int env = tuning().gemv_parts;
  const int cus = device_cu_count();
  int h = 1;
  while (h < 4) {
    const int next = 2 * h;
    const int tiles = (N + 16 / h - 1) / (16 / h);
    const bool fits = M <= 16 / next && chunks >= 8 * next;
    const bool wanted = tiles * 4 < cus * 3;
    const bool pays = (int64_t)(16 / next) * chunks * 8 >= (int64_t)lds_rows;
    if (!(fits && wanted && pays)) break;
    h = next;
  }
  if (env == 1 || env == 2 || env == 4) h = (M <= 16 / env) ? env : 1;
  return h;
}

GemvPlan plan_gemv_rows(int N, int rows, int steps) {
  const int tiles = (N + rows - 1) / rows;
  const int64_t jobs = (int64_t)tiles * steps;
  const int64_t target_waves = (int64_t)device_cu_count() * 16;
  int spw = (int)((jobs + target_waves - 1) / target_waves);
  if (spw < 1) spw = 1;
  if ((steps + spw - 1) / spw > 16) spw = (steps + 15) / 16;
  GemvPlan p;
  p.R = 1;
  p.steps_per_wave = spw;
  p.waves = (steps + spw - 1) / spw;
  return p;
}

bool gemv_perm_keeps_occupancy(int M, int N, int chunks, int cb_bytes) {
  const int cbl = (cb_bytes > 0 && cb_bytes <= kGemvLdsCodebookMax && gemv_lds_codebook_enabled()) ? cb_bytes : 0;
  const GemvPlan plan = plan_gemv(N, chunks, cbl ? 4 : 2);
  const int red = ((plan.waves * M * 16 * plan.R + 3) & ~3) * (int)sizeof(float);
  const int xb = M * chunks * 64 * 2;
  const int lds = red + (cbl > xb ? cbl : xb) + xb;
  const int blocks = (N + 16 * plan.R - 1) / (16 * plan.R);
  return lds <= 80 * 1024 || (blocks <= device_cu_count() && lds <= 160 * 1024);
}

int plan_tile_splits(int M, int N, int chunks, int mw) {
  const int env = tuning().tile_splits;
  const int cus = device_cu_count();
  const int blocks = ((N + 63) / 64) * ((M + 128 * mw - 1) / (128 * mw));
  int splits = 1;
  if (env > 0) splits = env;
  else if (blocks * 10 < cus * 7) splits = cus / blocks;
  const int max_by_k = chunks / 8 > 1 ? chunks / 8 : 1;
  if (splits > max_by_k) splits = max_by_k;
  if (splits > 16) splits = 16;
  return splits < 1 ? 1 : splits;
}

int tile2_mode() { return tuning().tile_wide; }

int plan_tile2_splits(int M, int N, int chunks, int mw) {
  const int env = tuning().tile_splits;
  const int cus = device_cu_count();
  const int blocks = ((N + kT2Cols - 1) / kT2Cols) * ((M + 128 * mw - 1) / (128 * mw));
  int splits = 1;
  if (env > 0) splits = env;
  else if (blocks * 10 < cus * 7) splits = cus / blocks;
  const int max_by_k = chunks / 8 > 1 ? chunks / 8 : 1;
  if (splits > max_by_k) splits = max_by_k;
  if (splits > 16) splits = 16;
  return splits < 1 ? 1 : splits;
}

extern "C" int64_t npamd_gemm_tile_workspace_bytes(int M, int N, int K);

int plan_tile_mw(int M) {
  const int mw_env = tuning().tile_mw;
  if (mw_env >= 1 && mw_env <= 3) return mw_env;
  const int mw = (M + 127) / 128;
  return mw < 1 ? 1 : (mw > 3 ? 3 : mw);
}

}  // namespace npamd

extern "C" int npamd_version(void) { return 3; }

extern "C" int npamd_gemv_stages_activations(int M, int N, int K, int nc) {
  if (M < 1 || M > NPAMD_GEMV_MAX_M || N < 1 || K < 64 || K % 64 || nc < 0) return 0;
  return nc ? npamd::vq_gemv_plan_stages(M, N, K, nc) : npamd::q_gemv_plan_stages(M, N, K);
}

extern "C" int npamd_diag_last_gemv_staged(void) { return npamd::last_gemv_staged(); }

extern "C" void npamd_diag_reload_tuning(void) { npamd::tuning_table() = npamd::read_tuning(); }

extern "C" int64_t npamd_gemm_tile_workspace_bytes(int M, int N, int K) {
  if (M <= 0 || N <= 0 || K < 64) return 0;
  const int mw = npamd::plan_tile_mw(M);
  const int splits = npamd::plan_tile_splits(M, N, K / 64, mw);
  const int64_t narrow = splits > 1 ? (int64_t)splits * M * N * 4 : 0;
  int64_t wide = 0;
  if (npamd::tile2_mode()) {
    wide = npamd::tile2_workspace_bytes(M, N, K / 64, mw);
    const int64_t wide_q = npamd::tile2_workspace_bytes(M, N, K / 64, npamd::plan_tile2_q_mw(M));
    if (wide_q > wide) wide = wide_q;
  }
  return narrow > wide ? narrow : wide;
}

extern "C" const char* npamd_last_error(void) { return npamd::error_text(); }
