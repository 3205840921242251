// Host-side builder and checker of the slice-list form (see sliced_format.hpp).
// Nothing in this file touches the GPU.
#include <string.h>

#include <stdlib.h>

#include <algorithm>
#include <atomic>
#include <numeric>
#include <thread>
#include <vector>

#include "common.hpp"
#include "sliced_format.hpp"

using namespace npamd;

namespace {

inline int64_t align_up(int64_t v, int64_t a) { return (v + a - 1) / a * a; }

// Host threads for the builder: NPAMD_BUILD_THREADS, else the core count, at most 16.
int builder_threads() {
  const char* v = getenv("NPAMD_BUILD_THREADS");
  int t = (v && *v) ? atoi(v) : (int)std::thread::hardware_concurrency();
  return t < 1 ? 1 : (t > 16 ? 16 : t);
}

// fn(i) for i in [0, count), dealt dynamically to the builder's threads.
template <class Fn>
void parallel_for(int count, Fn fn) {
  const int threads = std::min(builder_threads(), count);
  if (threads <= 1) {
    for (int i = 0; i < count; ++i) fn(i);
    return;
  }
  std::atomic<int> next{0};
  std::vector<std::thread> pool;
  for (int t = 0; t < threads; ++t)
    pool.emplace_back([&] {
      for (int i = next.fetch_add(1); i < count; i = next.fetch_add(1)) fn(i);
    });
  for (auto& th : pool) th.join();
}

inline uint32_t host_read_index(const uint8_t* packed, int64_t n_bytes, int64_t i, int bits) {
  const int64_t bit = i * (int64_t)bits;
  const int64_t b0 = bit >> 3;
  const int off = (int)(bit & 7);
  uint64_t w = 0;
  for (int j = 0; j < 4; ++j)
    if (b0 + j < n_bytes) w |= (uint64_t)packed[b0 + j] << (8 * j);
  return (uint32_t)((w >> off) & ((1u << bits) - 1u));
}

// Entry j of a lane's 12-byte quad record: row = bytes 2j, 2j+1 (little endian), group = byte 8 + j.
// In memory an entry is handled as row | group << 16.
inline void put_entry(uint8_t* quad_lane, int j, uint32_t e) {
  quad_lane[2 * j + 0] = (uint8_t)(e & 0xFF);
  quad_lane[2 * j + 1] = (uint8_t)((e >> 8) & 0xFF);
  quad_lane[8 + j] = (uint8_t)((e >> 16) & 0xFF);
}

inline uint32_t get_entry(const uint8_t* quad_lane, int j) {
  return (uint32_t)quad_lane[2 * j] | ((uint32_t)quad_lane[2 * j + 1] << 8) | ((uint32_t)quad_lane[8 + j] << 16);
}

// Order the entries of the 64 tasks of a strip so that, step by step, the LDS reads of a
// wave collide as little as possible.  A 64-lane 16-byte LDS read is served in two halves of 32
// lanes; a half takes as many cycles as its fullest 16-byte bank group holds distinct addresses
// ((address / 16) % 16, two being free) -- measured: 2.2 ns conflict-free, 3.6 ns with four
// addresses per group, 13.4 ns with sixteen.  Random rows give about five per group.  A lane may
// sum its entries in any order, so for every step each lane takes, among its remaining
// entries, the one whose activation vector (group % 16; shared vectors count once) and codebook
// row (row % 16) fall into the emptiest groups of its half.
void spread_bank_groups(std::vector<uint32_t>* const* tasks, int lanes, int64_t steps) {
  constexpr int kXWeight = 2;  // the activation read is repeated per token
  for (int64_t t = 0; t < steps; ++t) {
    for (int half = 0; half < 2; ++half) {
      int g_count[16] = {0}, r_count[16] = {0};
      uint8_t g_seen[kSlicedMaxGroups] = {0};
      for (int lane = half * 32; lane < std::min(lanes, half * 32 + 32); ++lane) {
        std::vector<uint32_t>& e = *tasks[lane];
        if ((int64_t)e.size() <= t) continue;
        size_t best = (size_t)t;
        int best_cost = 1 << 30;
        for (size_t i = (size_t)t; i < e.size(); ++i) {
          const uint32_t row = e[i] & 0xFFFFu, g = e[i] >> 16;
          const int gc = g_seen[g] ? 0 : std::max(0, g_count[g & 15] - 1);
          const int rc = std::max(0, r_count[row & 15] - 1);
          const int cost = kXWeight * gc + rc;
          if (cost < best_cost) {
            best_cost = cost;
            best = i;
            if (cost == 0) break;
          }
        }
        std::swap(e[(size_t)t], e[best]);
        const uint32_t row = e[(size_t)t] & 0xFFFFu, g = e[(size_t)t] >> 16;
        if (!g_seen[g]) {
          g_seen[g] = 1;
          ++g_count[g & 15];
        }
        ++r_count[row & 15];
      }
    }
  }
}

// How the layer is cut: `row_blocks` row ranges of `rows_per_block` rows, and per
// slice `parts[s]` group ranges.  One workgroup per (slice, group range, row block).
struct Geometry {
  int row_blocks = 1, rows_per_block = 1;
  std::vector<int> parts;
  int64_t workgroups = 0;
};

constexpr double kSlicedStartupShare = 0.7;  // a workgroup's start-up time in units of a 1 / target share of the layer

Geometry plan_geometry(int N, int G, const std::vector<int64_t>& slice_count, int64_t n_idx, int target) {
  const int S = (int)slice_count.size();
  const int rb_min = (N + kSlicedTasks - 1) / kSlicedTasks;
  const int kp_min = (G + kSlicedMaxGroups - 1) / kSlicedMaxGroups;
  std::vector<double> share((size_t)S);
  std::vector<int> kp_max((size_t)S);
  for (int s = 0; s < S; ++s) {
    share[s] = (double)slice_count[s] / (double)n_idx;
    // Group ranges no finer than about 16 entries per row and range: a workgroup pays for
    // loading its slice.
    kp_max[s] = std::max(kp_min, (int)((double)G * share[s] / 16.0 + 0.5));
  }
  Geometry best;
  double best_cost = 0;
  // Cost of a geometry: rounds of workgroups over the compute units times (the heaviest
  // workgroup + the charge for starting one: launch, record and slice loads, barrier, about
  // 3.9 us, against 5.5 us of streaming for a 1 / target share of a 14336 x 4096 layer).
  auto consider = [&](Geometry& geo) {
    geo.workgroups = 0;
    double heaviest = 0;
    for (int s = 0; s < S; ++s) {
      geo.workgroups += (int64_t)geo.parts[s] * geo.row_blocks;
      heaviest = std::max(heaviest, share[s] / ((double)geo.parts[s] * geo.row_blocks));
    }
    const double rounds = (double)((geo.workgroups + target - 1) / target);
    const double cost = rounds * (heaviest + kSlicedStartupShare / (double)target);
    if (best.workgroups == 0 || cost < best_cost - 1e-12) {
      best = geo;
      best_cost = cost;
    }
  };
  for (int rb = rb_min; rb <= 2 * rb_min + 1; ++rb) {
    Geometry geo;
    geo.row_blocks = rb;
    geo.rows_per_block = (N + rb - 1) / rb;
    geo.parts.resize((size_t)S);
    // (1) Group ranges in proportion to the slice's load (may need more than one round).
    for (int s = 0; s < S; ++s) {
      const int kp = (int)((double)target * share[s] / rb + 0.5);
      geo.parts[s] = std::max(kp_min, std::min(kp, kp_max[s]));
    }
    consider(geo);
    // (2) The best that fits one round: start from the fewest ranges and keep splitting the
    // heaviest slice while the compute units are not all taken.
    if ((int64_t)S * kp_min * rb <= target) {
      for (int s = 0; s < S; ++s) geo.parts[s] = kp_min;
      int64_t used = (int64_t)S * kp_min * rb;
      while (used + rb <= target) {
        int pick = -1;
        double worst = 0;
        for (int s = 0; s < S; ++s) {
          const double load = share[s] / ((double)geo.parts[s] * rb);
          if (geo.parts[s] < kp_max[s] && load > worst) { worst = load; pick = s; }
        }
        if (pick < 0) break;
        geo.parts[pick]++;
        used += rb;
      }
      consider(geo);
    }
  }
  return best;
}

}  // namespace

extern "C" int npamd_vq_sliced_build(const uint8_t* packed, int64_t n_bytes, int bits, int N, int K,
                                     int vl, int nc, int target_workgroups, void* blob,
                                     int64_t capacity, int64_t* blob_bytes) {
  const char* what = "npamd_vq_sliced_build";
  NPAMD_REQUIRE(blob_bytes != nullptr, "%s: blob_bytes is null", what);
  NPAMD_REQUIRE(vl == 8, "%s: the slice-list form needs VL = 8 (got %d)", what, vl);
  NPAMD_REQUIRE(bits >= 4 && bits <= 20, "%s: bits must be in [4, 20], got %d", what, bits);
  NPAMD_REQUIRE(N > 0 && K > 0 && nc >= 1, "%s: bad shape N=%d K=%d NC=%d", what, N, K, nc);
  NPAMD_REQUIRE(K % vl == 0, "%s: K=%d not divisible by VL=%d", what, K, vl);
  const int G = K / vl;
  const int64_t n_idx = (int64_t)N * G;
  NPAMD_REQUIRE(packed != nullptr && (n_idx * bits + 7) / 8 <= n_bytes, "%s: packed buffer too short", what);
  if (target_workgroups <= 0) target_workgroups = 256;

  const int slice_rows = kSlicedMaxSliceRows;
  const int S = (nc + slice_rows - 1) / slice_rows;

  // Indices transposed to [G][N] so a (group, row range) scan is contiguous.
  std::vector<uint32_t> idx_t((size_t)n_idx);
  std::vector<int64_t> slice_count((size_t)S, 0);
  {
    const int chunk = 256;  // rows per work item
    const int chunks = (N + chunk - 1) / chunk;
    std::vector<std::vector<int64_t>> counts((size_t)chunks, std::vector<int64_t>((size_t)S, 0));
    parallel_for(chunks, [&](int c) {
      for (int n = c * chunk; n < std::min(N, (c + 1) * chunk); ++n)
        for (int g = 0; g < G; ++g) {
          uint32_t v = host_read_index(packed, n_bytes, (int64_t)n * G + g, bits);
          if (v > (uint32_t)nc - 1u) v = (uint32_t)nc - 1u;  // same clamp as the decode kernels
          idx_t[(size_t)g * N + n] = v;
          counts[(size_t)c][v / slice_rows]++;
        }
    });
    for (auto& c : counts)
      for (int s = 0; s < S; ++s) slice_count[(size_t)s] += c[(size_t)s];
  }

  const Geometry geo = plan_geometry(N, G, slice_count, n_idx, target_workgroups);
  std::vector<int> partial_base((size_t)S);
  int n_partials = 0;
  for (int s = 0; s < S; ++s) {
    partial_base[s] = n_partials;
    n_partials += geo.parts[s];
  }

  // Workgroups, dealt round-robin over the slices so that workgroup id mod 8
  // (the XCD it lands on) tends to see one slice only.
  struct Job { int slice, part, block; };
  std::vector<Job> jobs;
  {
    std::vector<std::vector<Job>> per_slice((size_t)S);
    for (int s = 0; s < S; ++s)
      for (int kp = 0; kp < geo.parts[s]; ++kp)
        for (int rb = 0; rb < geo.row_blocks; ++rb) per_slice[s].push_back(Job{s, kp, rb});
    size_t remaining = 0;
    for (auto& v : per_slice) remaining += v.size();
    for (size_t j = 0; remaining > 0; ++j)
      for (int s = 0; s < S; ++s)
        if (j < per_slice[s].size()) {
          jobs.push_back(per_slice[s][j]);
          --remaining;
        }
  }
  const int n_wg = (int)jobs.size();

  // Every workgroup is built on its own (quad numbers local to the workgroup), then the entry
  // sections are concatenated in workgroup order.
  std::vector<SlicedWorkgroup> wgs((size_t)n_wg);
  std::vector<uint32_t> rowmap((size_t)n_wg * kSlicedTasks, kSlicedNoRow);
  std::vector<std::vector<uint8_t>> wg_quads((size_t)n_wg);
  std::vector<int64_t> wg_entries((size_t)n_wg, 0);

  const char* spread_env = getenv("NPAMD_SLICED_SPREAD");
  const bool spread = !(spread_env && *spread_env == '0');
  parallel_for(n_wg, [&](int w) {
    std::vector<std::vector<uint32_t>> task((size_t)geo.rows_per_block);
    std::vector<int> order;
    std::vector<uint8_t>& quads = wg_quads[(size_t)w];
    int64_t real_entries = 0;
    const Job& job = jobs[w];
    SlicedWorkgroup& wg = wgs[w];
    memset(&wg, 0, sizeof(wg));
    const int g_begin = (int)((int64_t)G * job.part / geo.parts[job.slice]);
    const int g_end = (int)((int64_t)G * (job.part + 1) / geo.parts[job.slice]);
    const int row0 = job.block * geo.rows_per_block;
    const int rows = std::max(0, std::min(geo.rows_per_block, N - row0));
    wg.slice = (uint32_t)job.slice;
    wg.partial = (uint32_t)(partial_base[job.slice] + job.part);
    wg.g_begin = (uint32_t)g_begin;
    wg.g_count = (uint32_t)(g_end - g_begin);

    for (int r = 0; r < rows; ++r) task[(size_t)r].clear();
    for (int g = g_begin; g < g_end; ++g) {
      const uint32_t* col = &idx_t[(size_t)g * N + row0];
      for (int r = 0; r < rows; ++r) {
        const uint32_t v = col[r];
        if ((int)(v / slice_rows) == job.slice)
          task[(size_t)r].push_back((v % slice_rows) | ((uint32_t)(g - g_begin) << 16));
      }
    }
    // Longest tasks first; 64 neighbours in that order share a strip.
    order.resize((size_t)rows);
    std::iota(order.begin(), order.end(), 0);
    std::stable_sort(order.begin(), order.end(),
                     [&](int a, int b) { return task[(size_t)a].size() > task[(size_t)b].size(); });
    const uint32_t pad = (uint32_t)kSlicedPadRow;  // the zero row, group 0
    for (int s = 0; s * 64 < rows; ++s) {
      const int first = s * 64;
      const int lanes = std::min(64, rows - first);
      const int64_t steps = (int64_t)task[(size_t)order[(size_t)first]].size();
      const int64_t nq = (steps + 3) / 4;
      if (spread) {
        std::vector<uint32_t>* strip_tasks[64];
        for (int lane = 0; lane < lanes; ++lane) strip_tasks[lane] = &task[(size_t)order[(size_t)(first + lane)]];
        spread_bank_groups(strip_tasks, lanes, steps);
      }
      wg.wave[s].quad_begin = nq ? (uint32_t)(quads.size() / kSlicedQuadBytes) : 0u;
      wg.wave[s].steps = (uint32_t)steps;
      const size_t base = quads.size();
      quads.resize(base + (size_t)nq * kSlicedQuadBytes);
      for (int lane = 0; lane < 64; ++lane) {
        const std::vector<uint32_t>* t = nullptr;
        if (lane < lanes) {
          const int r = order[(size_t)(first + lane)];
          t = &task[(size_t)r];
          rowmap[(size_t)w * kSlicedTasks + (size_t)s * 64 + lane] = (uint32_t)(row0 + r);
          real_entries += (int64_t)t->size();
        }
        for (int64_t i = 0; i < nq * 4; ++i) {
          const uint32_t e = (t && i < (int64_t)t->size()) ? (*t)[(size_t)i] : pad;
          put_entry(&quads[base + (size_t)(i / 4) * kSlicedQuadBytes + (size_t)lane * 12], (int)(i % 4), e);
        }
      }
    }
    wg_entries[(size_t)w] = real_entries;
  });

  std::vector<uint8_t> quads;
  int64_t real_entries = 0;
  int groups_max = 1;
  {
    size_t total = 0;
    for (auto& q : wg_quads) total += q.size();
    quads.reserve(std::max<size_t>(total, kSlicedQuadBytes));
    for (int w = 0; w < n_wg; ++w) {
      const uint32_t base = (uint32_t)(quads.size() / kSlicedQuadBytes);
      for (int s = 0; s < kSlicedWaves; ++s)
        if (wgs[(size_t)w].wave[s].steps) wgs[(size_t)w].wave[s].quad_begin += base;
      quads.insert(quads.end(), wg_quads[(size_t)w].begin(), wg_quads[(size_t)w].end());
      std::vector<uint8_t>().swap(wg_quads[(size_t)w]);
      real_entries += wg_entries[(size_t)w];
      groups_max = std::max(groups_max, (int)wgs[(size_t)w].g_count);
    }
  }
  if (quads.empty()) quads.resize(kSlicedQuadBytes, 0);  // waves without a strip still load quad 0

  npamd_sliced_header h;
  memset(&h, 0, sizeof(h));
  h.magic = kSlicedMagic;
  h.version = kSlicedVersion;
  h.n = N; h.k = K; h.vl = vl; h.nc = nc;
  h.slice_rows = slice_rows;
  h.n_slices = S;
  h.n_workgroups = n_wg;
  h.n_partials = n_partials;
  h.groups_max = groups_max;
  h.n_quads = (int64_t)(quads.size() / kSlicedQuadBytes);
  h.n_entries = real_entries;
  h.off_workgroups = sizeof(h);
  h.off_rowmap = align_up(h.off_workgroups + (int64_t)n_wg * (int64_t)sizeof(SlicedWorkgroup), 256);
  h.off_entries = align_up(h.off_rowmap + (int64_t)rowmap.size() * 4, 256);
  h.total_bytes = align_up(h.off_entries + (int64_t)quads.size(), 256);
  *blob_bytes = h.total_bytes;
  if (blob == nullptr) return NPAMD_OK;
  NPAMD_REQUIRE(capacity >= h.total_bytes, "%s: buffer of %lld bytes, %lld needed", what,
                (long long)capacity, (long long)h.total_bytes);
  uint8_t* out = (uint8_t*)blob;
  memset(out, 0, (size_t)h.total_bytes);
  memcpy(out, &h, sizeof(h));
  memcpy(out + h.off_workgroups, wgs.data(), wgs.size() * sizeof(SlicedWorkgroup));
  memcpy(out + h.off_rowmap, rowmap.data(), rowmap.size() * 4);
  memcpy(out + h.off_entries, quads.data(), quads.size());
  return NPAMD_OK;
}

extern "C" int npamd_vq_sliced_check(const void* blob, int64_t blob_bytes) {
  const char* what = "npamd_vq_sliced_check";
  NPAMD_REQUIRE(blob != nullptr && blob_bytes >= (int64_t)sizeof(npamd_sliced_header), "%s: blob too short", what);
  npamd_sliced_header h;
  memcpy(&h, blob, sizeof(h));
  NPAMD_REQUIRE(h.magic == kSlicedMagic && h.version == kSlicedVersion, "%s: not a slice-list blob (magic/version)", what);
  NPAMD_REQUIRE(h.total_bytes <= blob_bytes, "%s: blob holds %lld bytes, header says %lld", what,
                (long long)blob_bytes, (long long)h.total_bytes);
  NPAMD_REQUIRE(h.n > 0 && h.k > 0 && h.vl == 8 && h.nc >= 1 && h.k % 8 == 0, "%s: bad layer shape", what);
  NPAMD_REQUIRE(h.slice_rows >= 1 && h.slice_rows <= kSlicedMaxSliceRows &&
                    h.n_slices == (h.nc + h.slice_rows - 1) / h.slice_rows,
                "%s: bad slice geometry", what);
  NPAMD_REQUIRE(h.groups_max >= 1 && h.groups_max <= kSlicedMaxGroups, "%s: group range %d too long", what, h.groups_max);
  NPAMD_REQUIRE(h.n_workgroups >= 1 && h.n_partials >= 1 && h.n_quads >= 1, "%s: bad counts", what);
  const int64_t end_wg = h.off_workgroups + (int64_t)h.n_workgroups * (int64_t)sizeof(SlicedWorkgroup);
  const int64_t end_rm = h.off_rowmap + (int64_t)h.n_workgroups * kSlicedTasks * 4;
  const int64_t end_en = h.off_entries + h.n_quads * kSlicedQuadBytes;
  NPAMD_REQUIRE(h.off_workgroups >= (int64_t)sizeof(h) && end_wg <= h.off_rowmap && end_rm <= h.off_entries &&
                    end_en <= h.total_bytes && h.off_entries % 16 == 0 && h.off_rowmap % 4 == 0 &&
                    h.off_workgroups % 4 == 0,
                "%s: section offsets out of order or outside the blob", what);
  const uint8_t* base = (const uint8_t*)blob;
  const SlicedWorkgroup* wgs = (const SlicedWorkgroup*)(base + h.off_workgroups);
  const uint32_t* rowmap = (const uint32_t*)(base + h.off_rowmap);
  const uint8_t* quads = base + h.off_entries;
  const int G = h.k / 8;
  std::vector<uint8_t> covered((size_t)h.n_partials * (size_t)h.n, 0);
  std::vector<uint8_t> filed((size_t)h.n * (size_t)G, 0);
  for (int w = 0; w < h.n_workgroups; ++w) {
    const SlicedWorkgroup& wg = wgs[w];
    NPAMD_REQUIRE(wg.slice < (uint32_t)h.n_slices && wg.partial < (uint32_t)h.n_partials,
                  "%s: workgroup %d: slice/partial out of range", what, w);
    NPAMD_REQUIRE(wg.g_count >= 1 && wg.g_count <= (uint32_t)h.groups_max && (int64_t)wg.g_begin + wg.g_count <= G,
                  "%s: workgroup %d: group range out of bounds", what, w);
    const uint32_t slice_len = (uint32_t)std::min(h.slice_rows, h.nc - (int)wg.slice * h.slice_rows);
    for (int s = 0; s < kSlicedWaves; ++s) {
      const SlicedWave& wave = wg.wave[s];
      const int64_t nq = ((int64_t)wave.steps + 3) / 4;
      NPAMD_REQUIRE((int64_t)wave.quad_begin + std::max<int64_t>(nq, 1) <= h.n_quads,
                    "%s: workgroup %d wave %d: entries out of bounds", what, w, s);
      for (int lane = 0; lane < 64; ++lane) {
        const uint32_t row = rowmap[(size_t)w * kSlicedTasks + (size_t)s * 64 + lane];
        NPAMD_REQUIRE(row == kSlicedNoRow || row < (uint32_t)h.n, "%s: workgroup %d: row out of range", what, w);
        if (row != kSlicedNoRow) {
          uint8_t& c = covered[(size_t)wg.partial * h.n + row];
          NPAMD_REQUIRE(c == 0, "%s: partial %u row %u written twice", what, wg.partial, row);
          c = 1;
        }
        for (int64_t i = 0; i < nq * 4; ++i) {
          const uint32_t e = get_entry(quads + ((size_t)wave.quad_begin + (size_t)(i / 4)) * kSlicedQuadBytes + (size_t)lane * 12, (int)(i % 4));
          const uint32_t local = e & 0xFFFFu, g_local = e >> 16;
          NPAMD_REQUIRE(g_local < wg.g_count && (local < slice_len || local == (uint32_t)kSlicedPadRow),
                        "%s: workgroup %d: entry field out of range", what, w);
          if (local != (uint32_t)kSlicedPadRow) {
            NPAMD_REQUIRE(row != kSlicedNoRow && i < (int64_t)wave.steps, "%s: workgroup %d: live entry in a lane without a row", what, w);
            uint8_t& f = filed[(size_t)row * G + wg.g_begin + g_local];
            NPAMD_REQUIRE(f == 0, "%s: index (%u, %u) filed twice", what, row, wg.g_begin + g_local);
            f = 1;
          }
        }
      }
    }
  }
  for (uint8_t c : covered) NPAMD_REQUIRE(c == 1, "%s: some (partial, row) pair is never written", what);
  for (uint8_t f : filed) NPAMD_REQUIRE(f == 1, "%s: some index is not filed", what);
  NPAMD_REQUIRE(h.n_entries == (int64_t)h.n * G, "%s: entry count in the header is wrong", what);
  return NPAMD_OK;
}

extern "C" int64_t npamd_vq_sliced_workspace_bytes(const npamd_sliced_header* h, int M) {
  if (h == nullptr || M < 1) return 0;
  return (int64_t)h->n_partials * (int64_t)h->n * 4 * (int64_t)M;
}
