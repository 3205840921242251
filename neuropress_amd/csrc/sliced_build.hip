// Host-side builder and checker of the slice-list form (see sliced_format.hpp).
// Nothing in this file touches the GPU.
#include <string.h>

#include <stdlib.h>

#include <algorithm>
#include <atomic>
#include <numeric>
#include <string>
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

// Entry j of a lane's 12-byte quad record: bytes 2j, 2j+1 (little endian) hold the row in bits 0-12
// and bit 8 of the group in bit 15, byte 8 + j the group's low eight bits.
// In memory an entry is handled as row | group << 16.
inline void put_entry(uint8_t* quad_lane, int j, uint32_t e) {
  const uint32_t row = e & 0x1FFFu, g = e >> 16;
  const uint32_t field = row | ((g >> 8) << 15);
  quad_lane[2 * j + 0] = (uint8_t)(field & 0xFF);
  quad_lane[2 * j + 1] = (uint8_t)(field >> 8);
  quad_lane[8 + j] = (uint8_t)(g & 0xFF);
}

inline uint32_t get_entry(const uint8_t* quad_lane, int j) {
  const uint32_t field = (uint32_t)quad_lane[2 * j] | ((uint32_t)quad_lane[2 * j + 1] << 8);
  const uint32_t g = (uint32_t)quad_lane[8 + j] | ((field >> 15) << 8);
  return (field & 0x1FFFu) | (g << 16);
}

// Order the entries of the 64 tasks of a strip so that, step by step, the LDS reads of a
// wave collide as little as possible.  A 64-lane 16-byte LDS read (ds_read_b128) is served
// in four passes of 16 lanes -- lanes {0-3, 12-15, 20-27}, {4-11, 16-19, 28-31} and the same
// two sets 32 lanes further on (found by timing reads in which exactly two lanes share a bank
// group) -- and a pass takes one cycle per distinct address of its fullest 16-byte bank
// group ((address / 16) % 16): 4.3 cycles per read when every pass has its 16 lanes in 16
// different groups, one more for every further address in a group.  Random rows put about three
// addresses into the fullest group of a pass.  A lane may sum its entries in any order, so
// for every step each lane takes, among its remaining entries, the one whose activation
// vector (group % 16; a vector already read in the pass costs nothing) and codebook row
// (row % 16) fall into the emptiest bank groups of its pass.
inline int lds_pass_of_lane(int lane) {
  const int l = lane & 31;
  const bool first = l < 4 || (l >= 12 && l < 16) || (l >= 20 && l < 28);
  return (lane >> 5) * 2 + (first ? 0 : 1);
}

// A task's entries: a run of the builder's flat entry array.
struct TaskSpan {
  uint32_t* e;
  uint32_t n;
  uint32_t size() const { return n; }
};

void spread_bank_groups(const TaskSpan* tasks, int lanes, int64_t steps) {
  constexpr int kXWeight = 1;
  int pass_lanes[4][16], pass_count[4] = {0, 0, 0, 0};
  for (int lane = 0; lane < lanes; ++lane) {
    const int p = lds_pass_of_lane(lane);
    pass_lanes[p][pass_count[p]++] = lane;
  }
  // Lanes with the fewest entries choose first: they have the least freedom.
  int order[4][16];
  for (int p = 0; p < 4; ++p) {
    for (int i = 0; i < pass_count[p]; ++i) order[p][i] = pass_lanes[p][i];
    std::stable_sort(order[p], order[p] + pass_count[p], [&](int a, int b) { return tasks[a].size() < tasks[b].size(); });
  }
  for (int64_t t = 0; t < steps; ++t) {
    for (int p = 0; p < 4; ++p) {
      int g_count[16] = {0}, r_count[16] = {0};
      uint8_t g_seen[kSlicedMaxGroups] = {0};
      for (int i = 0; i < pass_count[p]; ++i) {
        const TaskSpan& task = tasks[order[p][i]];
        uint32_t* const e = task.e;
        if ((int64_t)task.size() <= t) continue;
        size_t best = (size_t)t;
        int best_cost = 1 << 30;
        for (size_t j = (size_t)t; j < task.size(); ++j) {
          const uint32_t row = e[j] & 0xFFFFu, g = e[j] >> 16;
          const int gc = g_seen[g] ? 0 : g_count[g & 15];
          const int cost = kXWeight * gc + r_count[row & 15];
          if (cost < best_cost) {
            best_cost = cost;
            best = j;
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

  // Indices as 32-bit values, row-major, clamped as the decode kernels clamp them; per-slice counts.
  std::vector<uint32_t> idx((size_t)n_idx);
  std::vector<int64_t> slice_count((size_t)S, 0);
  const int chunk = 64;  // rows per work item
  const int chunks = (N + chunk - 1) / chunk;
  {
    std::vector<std::vector<int64_t>> counts((size_t)chunks, std::vector<int64_t>((size_t)S, 0));
    parallel_for(chunks, [&](int c) {
      int64_t* cnt = counts[(size_t)c].data();
      for (int n = c * chunk; n < std::min(N, (c + 1) * chunk); ++n) {
        uint32_t* row = &idx[(size_t)n * G];
        if (bits == 16) {
          const uint16_t* src = reinterpret_cast<const uint16_t*>(packed) + (size_t)n * G;  // little endian
          for (int g = 0; g < G; ++g) row[g] = src[g];
        } else {
          for (int g = 0; g < G; ++g) row[g] = host_read_index(packed, n_bytes, (int64_t)n * G + g, bits);
        }
        for (int g = 0; g < G; ++g) {
          if (row[g] > (uint32_t)nc - 1u) row[g] = (uint32_t)nc - 1u;  // same clamp as the decode kernels
          cnt[row[g] / (uint32_t)slice_rows]++;
        }
      }
    });
    for (auto& c : counts)
      for (int s = 0; s < S; ++s) slice_count[(size_t)s] += c[(size_t)s];
  }

  Geometry geo = plan_geometry(N, G, slice_count, n_idx, target_workgroups);
  // Group ranges have a fixed length per slice, ceil(G / parts); no range may come out empty.
  for (int& parts : geo.parts) parts = (G + (G + parts - 1) / parts - 1) / ((G + parts - 1) / parts);
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

  // Every index is filed under its workgroup (slice, group range, row block) and row in one sweep
  // over the rows: count, turn the counts into places in one flat entry array, fill.  A task's
  // entries come out in ascending group order.
  const int rpb = geo.rows_per_block;
  std::vector<int> range_groups((size_t)S), wg_base((size_t)S);  // groups per range; first workgroup slot of a slice
  std::vector<int> wg_of;                                        // (slice, part, row block) -> workgroup
  {
    int slots = 0;
    for (int s = 0; s < S; ++s) {
      range_groups[(size_t)s] = (G + geo.parts[(size_t)s] - 1) / geo.parts[(size_t)s];
      wg_base[(size_t)s] = slots;
      slots += geo.parts[(size_t)s] * geo.row_blocks;
    }
    wg_of.assign((size_t)slots, -1);
    for (int w = 0; w < n_wg; ++w)
      wg_of[(size_t)(wg_base[(size_t)jobs[w].slice] + jobs[w].part * geo.row_blocks + jobs[w].block)] = w;
  }
  std::vector<uint32_t> task_len((size_t)n_wg * rpb, 0u);   // entries of (workgroup, row of its block)
  parallel_for(chunks, [&](int c) {
    for (int n = c * chunk; n < std::min(N, (c + 1) * chunk); ++n) {
      const uint32_t* row = &idx[(size_t)n * G];
      const int rb = n / rpb, r = n - rb * rpb;
      for (int g = 0; g < G; ++g) {
        const int sl = (int)(row[g] / (uint32_t)slice_rows);
        const int w = wg_of[(size_t)(wg_base[(size_t)sl] + (g / range_groups[(size_t)sl]) * geo.row_blocks + rb)];
        ++task_len[(size_t)w * rpb + r];
      }
    }
  });
  std::vector<int64_t> task_begin((size_t)n_wg * rpb + 1);
  task_begin[0] = 0;
  for (size_t i = 0; i < (size_t)n_wg * rpb; ++i) task_begin[i + 1] = task_begin[i] + task_len[i];
  std::vector<uint32_t> entries((size_t)n_idx);
  parallel_for(chunks, [&](int c) {
    std::vector<uint32_t> filled;
    for (int n = c * chunk; n < std::min(N, (c + 1) * chunk); ++n) {
      const uint32_t* row = &idx[(size_t)n * G];
      const int rb = n / rpb, r = n - rb * rpb;
      // per workgroup of this row: how many entries are in place (a row belongs to one work item)
      filled.assign((size_t)n_wg, 0u);
      for (int g = 0; g < G; ++g) {
        const uint32_t v = row[g];
        const int sl = (int)(v / (uint32_t)slice_rows);
        const int part = g / range_groups[(size_t)sl];
        const int w = wg_of[(size_t)(wg_base[(size_t)sl] + part * geo.row_blocks + rb)];
        entries[(size_t)(task_begin[(size_t)w * rpb + r] + filled[(size_t)w]++)] =
            (v % (uint32_t)slice_rows) | ((uint32_t)(g - part * range_groups[(size_t)sl]) << 16);
      }
    }
  });
  idx.clear();
  idx.shrink_to_fit();

  // One workgroup at a time: strips, lane order and the order of the entries inside a task.
  struct Built {
    std::vector<uint16_t> order;  // task (row of the block) of every lane, strip by strip
    int steps[kSlicedWaves];      // longest task of each strip
    int64_t real_entries;
  };
  std::vector<SlicedWorkgroup> wgs((size_t)n_wg);
  std::vector<uint32_t> rowmap((size_t)n_wg * kSlicedTasks, kSlicedNoRow);
  std::vector<Built> built((size_t)n_wg);

  const char* spread_env = getenv("NPAMD_SLICED_SPREAD");
  const bool spread = !(spread_env && *spread_env == '0');
  parallel_for(n_wg, [&](int w) {
    Built& b = built[(size_t)w];
    const Job& job = jobs[w];
    SlicedWorkgroup& wg = wgs[w];
    const int g_begin = job.part * range_groups[(size_t)job.slice];
    const int g_end = std::min(G, g_begin + range_groups[(size_t)job.slice]);
    const int row0 = job.block * rpb;
    const int rows = std::max(0, std::min(rpb, N - row0));
    wg.slice = (uint32_t)job.slice;
    wg.partial = (uint32_t)(partial_base[job.slice] + job.part);
    wg.g_begin = (uint32_t)g_begin;
    wg.g_count = (uint32_t)(g_end - g_begin);
    wg.row_begin = (uint32_t)std::min(row0, N);
    wg.row_count = (uint32_t)rows;
    wg.reserved[0] = wg.reserved[1] = 0;

    const uint32_t* len = &task_len[(size_t)w * rpb];
    // Longest tasks first; 64 neighbours in that order share a strip.
    b.order.resize((size_t)rows);
    std::iota(b.order.begin(), b.order.end(), (uint16_t)0);
    std::stable_sort(b.order.begin(), b.order.end(), [&](uint16_t a, uint16_t c) { return len[a] > len[c]; });
    b.real_entries = 0;
    for (int s = 0; s < kSlicedWaves; ++s) {
      const int first = s * 64;
      const int lanes = std::max(0, std::min(64, rows - first));
      b.steps[s] = lanes ? (int)len[b.order[(size_t)first]] : 0;
      TaskSpan strip_tasks[64];
      for (int lane = 0; lane < lanes; ++lane) {
        const int r = b.order[(size_t)(first + lane)];
        strip_tasks[lane] = TaskSpan{&entries[(size_t)task_begin[(size_t)w * rpb + r]], len[r]};
        rowmap[(size_t)w * kSlicedTasks + (size_t)first + lane] = (uint32_t)(row0 + r);
        b.real_entries += len[r];
      }
      if (spread && lanes) spread_bank_groups(strip_tasks, lanes, b.steps[s]);
    }
  });

  // Strip w of every workgroup gets the length of the layer's longest strip w.
  uint16_t wave_quads[kSlicedWaves];
  int64_t wave_begin[kSlicedWaves + 1];
  int64_t real_entries = 0;
  int groups_max = 1;
  wave_begin[0] = 0;
  for (int s = 0; s < kSlicedWaves; ++s) {
    int longest = 0;
    for (int w = 0; w < n_wg; ++w) longest = std::max(longest, built[(size_t)w].steps[s]);
    NPAMD_REQUIRE((longest + 3) / 4 <= 65535, "%s: a row has %d indices in one slice and group range", what, longest);
    wave_quads[s] = (uint16_t)((longest + 3) / 4);
    wave_begin[s + 1] = wave_begin[s] + wave_quads[s];
  }
  const int64_t wg_quads = std::max<int64_t>(wave_begin[kSlicedWaves], 1);  // never an empty entry section
  for (int w = 0; w < n_wg; ++w) {
    real_entries += built[(size_t)w].real_entries;
    groups_max = std::max(groups_max, (int)wgs[(size_t)w].g_count);
  }
  bool round_robin = true;
  for (int s = 0; s < S; ++s) round_robin = round_robin && geo.parts[(size_t)s] == geo.parts[0];

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
  h.flags = round_robin ? kSlicedRoundRobin : 0u;
  h.n_quads = (int64_t)n_wg * wg_quads;
  h.n_entries = real_entries;
  memcpy(h.wave_quads, wave_quads, sizeof(wave_quads));
  h.off_workgroups = sizeof(h);
  h.off_rowmap = align_up(h.off_workgroups + (int64_t)n_wg * (int64_t)sizeof(SlicedWorkgroup), 256);
  h.off_entries = align_up(h.off_rowmap + (int64_t)rowmap.size() * 4, 256);
  h.total_bytes = align_up(h.off_entries + h.n_quads * kSlicedQuadBytes, 256);
  *blob_bytes = h.total_bytes;
  if (blob == nullptr) return NPAMD_OK;
  NPAMD_REQUIRE(capacity >= h.total_bytes, "%s: buffer of %lld bytes, %lld needed", what,
                (long long)capacity, (long long)h.total_bytes);
  uint8_t* out = (uint8_t*)blob;
  memset(out, 0, (size_t)h.off_entries);
  memcpy(out, &h, sizeof(h));
  memcpy(out + h.off_workgroups, wgs.data(), wgs.size() * sizeof(SlicedWorkgroup));
  memcpy(out + h.off_rowmap, rowmap.data(), rowmap.size() * 4);
  memset(out + h.off_entries + h.n_quads * kSlicedQuadBytes, 0,
         (size_t)(h.total_bytes - h.off_entries - h.n_quads * kSlicedQuadBytes));
  // Pass 2: every lane's entries, padded to the strip's length with the zero row (group 0).
  const uint32_t pad = (uint32_t)kSlicedPadRow;
  parallel_for(n_wg, [&](int w) {
    const Built& b = built[(size_t)w];
    uint8_t* wg_out = out + h.off_entries + (int64_t)w * wg_quads * kSlicedQuadBytes;
    if (wave_begin[kSlicedWaves] == 0) memset(wg_out, 0, kSlicedQuadBytes);  // the one quad of an entry-less layer
    for (int s = 0; s < kSlicedWaves; ++s) {
      uint8_t* strip = wg_out + wave_begin[s] * kSlicedQuadBytes;
      const int64_t slots = 4 * (int64_t)wave_quads[s];
      for (int lane = 0; lane < 64; ++lane) {
        const size_t pos = (size_t)s * 64 + lane;
        const bool real = pos < b.order.size();
        const size_t task = real ? (size_t)w * rpb + b.order[pos] : 0;
        const uint32_t* e = real ? &entries[(size_t)task_begin[task]] : nullptr;
        const int64_t len = real ? (int64_t)task_len[task] : 0;
        for (int64_t i = 0; i < slots; ++i)
          put_entry(strip + (size_t)(i / 4) * kSlicedQuadBytes + (size_t)lane * 12, (int)(i % 4), i < len ? e[i] : pad);
      }
    }
  });
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
  int64_t wave_begin[kSlicedWaves + 1];
  wave_begin[0] = 0;
  for (int s = 0; s < kSlicedWaves; ++s) wave_begin[s + 1] = wave_begin[s] + h.wave_quads[s];
  const int64_t wg_quads = std::max<int64_t>(wave_begin[kSlicedWaves], 1);
  NPAMD_REQUIRE(h.n_quads == (int64_t)h.n_workgroups * wg_quads, "%s: entry section does not match the strip lengths", what);
  NPAMD_REQUIRE((h.flags & ~kSlicedRoundRobin) == 0, "%s: unknown flags", what);
  const int64_t end_wg = h.off_workgroups + (int64_t)h.n_workgroups * (int64_t)sizeof(SlicedWorkgroup);
  const int64_t end_rm = h.off_rowmap + (int64_t)h.n_workgroups * kSlicedTasks * 4;
  const int64_t end_en = h.off_entries + h.n_quads * kSlicedQuadBytes;
  NPAMD_REQUIRE(h.off_workgroups >= (int64_t)sizeof(h) && end_wg <= h.off_rowmap && end_rm <= h.off_entries &&
                    end_en <= h.total_bytes && h.off_entries % 16 == 0 && h.off_rowmap % 4 == 0 &&
                    h.off_workgroups % 16 == 0,
                "%s: section offsets out of order or outside the blob", what);
  const uint8_t* base = (const uint8_t*)blob;
  const SlicedWorkgroup* wgs = (const SlicedWorkgroup*)(base + h.off_workgroups);
  const uint32_t* rowmap = (const uint32_t*)(base + h.off_rowmap);
  const uint8_t* quads = base + h.off_entries;
  const int G = h.k / 8;
  std::vector<uint8_t> covered((size_t)h.n_partials * (size_t)h.n, 0);
  std::vector<uint8_t> filed((size_t)h.n * (size_t)G, 0);
  // One workgroup per work item; the first violation found (lowest workgroup) is the one reported.
  std::vector<std::string> errors((size_t)h.n_workgroups);
#define WG_REQUIRE(cond, ...)                          \
  do {                                                 \
    if (!(cond)) {                                     \
      char msg[256];                                   \
      snprintf(msg, sizeof(msg), __VA_ARGS__);         \
      errors[(size_t)w] = msg;                         \
      return;                                          \
    }                                                  \
  } while (0)
  parallel_for(h.n_workgroups, [&](int w) {
    const SlicedWorkgroup& wg = wgs[w];
    WG_REQUIRE(wg.slice < (uint32_t)h.n_slices && wg.partial < (uint32_t)h.n_partials,
                  "%s: workgroup %d: slice/partial out of range", what, w);
    if (h.flags & kSlicedRoundRobin) {
      // What the kernel computes instead of reading the record.
      const int parts = h.n_partials / h.n_slices;
      const int row_blocks = parts ? h.n_workgroups / (parts * h.n_slices) : 0;
      WG_REQUIRE(parts >= 1 && row_blocks >= 1 && parts * h.n_slices == h.n_partials &&
                        row_blocks * h.n_partials == h.n_workgroups,
                    "%s: counts do not form the regular geometry the header states", what);
      const int range_groups = (G + parts - 1) / parts;
      const int rows_per_block = (h.n + row_blocks - 1) / row_blocks;
      const uint32_t part = (uint32_t)((w / h.n_slices) / row_blocks);
      const int block = (w / h.n_slices) % row_blocks;
      const int row_begin = std::min(block * rows_per_block, h.n);
      WG_REQUIRE(wg.slice == (uint32_t)(w % h.n_slices) && wg.partial == wg.slice * (uint32_t)parts + part &&
                        wg.g_begin == part * (uint32_t)range_groups &&
                        wg.g_count == (uint32_t)std::min(range_groups, G - (int)wg.g_begin) &&
                        wg.row_begin == (uint32_t)row_begin &&
                        wg.row_count == (uint32_t)std::max(0, std::min(rows_per_block, h.n - row_begin)),
                    "%s: workgroup %d does not follow the regular geometry the header states", what, w);
    }
    WG_REQUIRE(wg.g_count >= 1 && wg.g_count <= (uint32_t)h.groups_max && (int64_t)wg.g_begin + wg.g_count <= G,
                  "%s: workgroup %d: group range out of bounds", what, w);
    WG_REQUIRE(wg.row_count <= (uint32_t)kSlicedTasks && (int64_t)wg.row_begin + wg.row_count <= h.n,
                  "%s: workgroup %d: row block out of bounds", what, w);
    const uint32_t slice_len = (uint32_t)std::min(h.slice_rows, h.nc - (int)wg.slice * h.slice_rows);
    for (int s = 0; s < kSlicedWaves; ++s) {
      const int64_t nq = h.wave_quads[s];
      const int64_t quad_begin = (int64_t)w * wg_quads + wave_begin[s];
      for (int lane = 0; lane < 64; ++lane) {
        const uint32_t row = rowmap[(size_t)w * kSlicedTasks + (size_t)s * 64 + lane];
        WG_REQUIRE(row == kSlicedNoRow || (row >= wg.row_begin && row - wg.row_begin < wg.row_count),
                      "%s: workgroup %d: row outside the workgroup's row block", what, w);
        if (row != kSlicedNoRow) {
          const uint8_t seen = __atomic_fetch_add(&covered[(size_t)wg.partial * h.n + row], (uint8_t)1, __ATOMIC_RELAXED);
          WG_REQUIRE(seen == 0, "%s: partial %u row %u written twice", what, wg.partial, row);
        }
        for (int64_t i = 0; i < nq * 4; ++i) {
          const uint32_t e = get_entry(quads + ((size_t)quad_begin + (size_t)(i / 4)) * kSlicedQuadBytes + (size_t)lane * 12, (int)(i % 4));
          const uint32_t local = e & 0xFFFFu, g_local = e >> 16;
          WG_REQUIRE(g_local < wg.g_count && (local < slice_len || local == (uint32_t)kSlicedPadRow),
                        "%s: workgroup %d: entry field out of range", what, w);
          if (local != (uint32_t)kSlicedPadRow) {
            WG_REQUIRE(row != kSlicedNoRow, "%s: workgroup %d: live entry in a lane without a row", what, w);
            const uint8_t seen = __atomic_fetch_add(&filed[(size_t)row * G + wg.g_begin + g_local], (uint8_t)1, __ATOMIC_RELAXED);
            WG_REQUIRE(seen == 0, "%s: index (%u, %u) filed twice", what, row, wg.g_begin + g_local);
          }
        }
      }
    }
  });
#undef WG_REQUIRE
  for (const std::string& e : errors) NPAMD_REQUIRE(e.empty(), "%s", e.c_str());
  for (uint8_t c : covered) NPAMD_REQUIRE(c == 1, "%s: some (partial, row) pair is never written", what);
  for (uint8_t f : filed) NPAMD_REQUIRE(f == 1, "%s: some index is not filed", what);
  NPAMD_REQUIRE(h.n_entries == (int64_t)h.n * G, "%s: entry count in the header is wrong", what);
  return NPAMD_OK;
}

extern "C" int64_t npamd_vq_sliced_workspace_bytes(const npamd_sliced_header* h, int M) {
  if (h == nullptr || M < 1) return 0;
  // Fewer than 256 partial sums per row: a 64-bit word and a float per (token, row).
  if (h->n_partials < 256) return (int64_t)h->n * 12 * (int64_t)M;
  return (int64_t)h->n_partials * (int64_t)h->n * 4 * (int64_t)M;
}
