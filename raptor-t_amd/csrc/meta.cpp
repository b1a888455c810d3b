// Host metadata of the padding-free block-sparse layer: numpy-compatible RNG, BigBird
// random-block plans, to-block CSR and the LPT work plan.  No GPU code in this file.
//
// What each part replaces in the reference:
//   NpRng + plans      python/modeling_big_bird.py:573-597, :1039-1314 (numpy global RNG)
//   build_to_index     layers/multi_headed_attention.cpp:15-140
//   block costs, LPT   python/util.py:11-50
#include <algorithm>
#include <cstdint>
#include <cstring>
#include <map>
#include <memory>
#include <mutex>
#include <queue>
#include <tuple>
#include <vector>

#include "rt_common.h"

namespace rt {

static thread_local char g_err[512];
char* error_buffer() { return g_err; }
int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

static thread_local LaunchEvents g_launch_events = {nullptr, nullptr};
LaunchEvents take_launch_events() {
  const LaunchEvents ev = g_launch_events;
  g_launch_events = LaunchEvents{nullptr, nullptr};
  return ev;
}
static void set_launch_events(void* start, void* stop) { g_launch_events = LaunchEvents{start, stop}; }

// numpy's legacy generator: MT19937 seeded by init_genrand, 32-bit tempered draws,
// bounded integers by masked rejection, Fisher-Yates from the top (numpy
// RandomState.seed / .permutation).
class NpRng {
 public:
  explicit NpRng(uint32_t seed) { reseed(seed); }
  void reseed(uint32_t seed) {
    mt_[0] = seed;
    for (int i = 1; i < 624; ++i) mt_[i] = 1812433253u * (mt_[i - 1] ^ (mt_[i - 1] >> 30)) + uint32_t(i);
    pos_ = 624;
  }
  uint32_t next() {
    if (pos_ >= 624) refill();
    uint32_t y = mt_[pos_++];
    y ^= y >> 11;
    y ^= (y << 7) & 0x9d2c5680u;
    y ^= (y << 15) & 0xefc60000u;
    y ^= y >> 18;
    return y;
  }
  uint32_t below_or_equal(uint32_t max) {
    if (max == 0) return 0;
    uint32_t mask = max;
    mask |= mask >> 1; mask |= mask >> 2; mask |= mask >> 4; mask |= mask >> 8; mask |= mask >> 16;
    uint32_t v;
    do { v = next() & mask; } while (v > max);
    return v;
  }
  void permute(std::vector<int>& a) {
    for (size_t i = a.size(); i-- > 1;) std::swap(a[i], a[below_or_equal(uint32_t(i))]);
  }

 private:
  void refill() {
    for (int k = 0; k < 624; ++k) {
      uint32_t y = (mt_[k] & 0x80000000u) | (mt_[(k + 1) % 624] & 0x7fffffffu);
      mt_[k] = mt_[(k + 397) % 624] ^ (y >> 1) ^ ((y & 1u) ? 0x9908b0dfu : 0u);
    }
    pos_ = 0;
  }
  uint32_t mt_[624];
  int pos_;
};

static std::vector<int> iota_range(int lo, int hi) {
  std::vector<int> v;
  for (int x = lo; x < hi; ++x) v.push_back(x);
  return v;
}

// Truncated max-length plan of one head: rows for from-blocks 1..nb-2 of a `max_pos`
// token sequence; candidates stop before block last_idx/64 - 1.
// python/modeling_big_bird.py:1072-1125.
static void max_plan_one_head(NpRng& rng, int max_pos, int last_idx, int rows_wanted, int* out) {
  const int nb = max_pos / RT_BLOCK;
  int last = nb - 1;
  if (last_idx > 2 * RT_BLOCK) last = last_idx / RT_BLOCK - 1;
  // middle_seq[a:b] of arange(1, nb-1) is the value range [1+a, 1+min(b, nb-2))
  auto mid = [&](int a, int b) { return iota_range(1 + std::max(a, 0), 1 + std::min(b, nb - 2)); };
  for (int i = 1; i < nb - 1; ++i) {
    std::vector<int> cand;
    if (i == 1) cand = mid(2, last);
    else if (i == 2) cand = mid(3, last);
    else if (i == nb - 3 || i == nb - 2) cand = mid(0, last);
    else if (i - 2 > last) cand = mid(0, last);
    else if (i + 1 == last) cand = mid(0, i - 2);
    else {
      cand = mid(0, i - 2);
      std::vector<int> tail = mid(i + 1, last);
      cand.insert(cand.end(), tail.begin(), tail.end());
    }
    rng.permute(cand);                       // the RNG is consumed for every row of max_pos
    if (i - 1 < rows_wanted)
      for (int c = 0; c < RT_NUM_RAND; ++c) out[(i - 1) * RT_NUM_RAND + c] = cand[c];
  }
}

// First `want` legal blocks of a permutation of [to_start, to_end):
// python/modeling_big_bird.py:1261-1314.
static std::vector<int> single_row(NpRng& rng, int block_id, int to_start, int to_end, int want) {
  static thread_local std::vector<int> perm;           // called once per row and head: no allocation per call
  perm.clear();
  for (int x = to_start; x < to_end; ++x) perm.push_back(x);
  rng.permute(perm);
  auto illegal = [&](int b) {
    if (b >= block_id - 1 && b <= block_id + 1) return true;
    if (b == 0 || b == to_end - 1) return true;
    if (block_id == 1 && b == to_end - 2) return true;
    if (block_id == to_end - 2 && b == 1) return true;
    return false;
  };
  std::vector<int> got;
  for (int b : perm) {
    if (!illegal(b)) got.push_back(b);
    if (int(got.size()) == want) break;
  }
  return got;
}

// Per-head planned variant: python/modeling_big_bird.py:1039-1069 (plan) and :1127-1258.
// rand[h] is a [nb][width] table; rows 1..nb-2 are copied out.
static int with_head_plan(NpRng& rng, int length, int heads, int* out) {
  const int nb = length / RT_BLOCK, r = RT_NUM_RAND;
  std::vector<int> plan_len, plan_cnt;
  if (2 * r + 5 < nb) { plan_len = {(2 * r + 5), nb}; plan_cnt = {r, 0}; }
  else if (r + 5 < nb) { plan_len = {(r + 5), nb}; plan_cnt = {r / 2, r - r / 2}; }
  else { plan_len = {nb}; plan_cnt = {r}; }
  const int np_ = int(plan_len.size());
  auto prefix = [&](int upto) { int s = 0; for (int i = 0; i < upto; ++i) s += plan_cnt[i]; return s; };
  const int width = prefix(np_);
  std::vector<std::vector<int>> rand(heads, std::vector<int>(size_t(nb) * width, 0));
  bool short_row = false;
  auto fill = [&](int row, int c0, int c1, int to_start, int to_end, int count) {
    for (int h = 0; h < heads; ++h) {
      std::vector<int> got = single_row(rng, row, to_start, to_end, count);
      if (int(got.size()) != c1 - c0) { short_row = true; continue; }
      for (int c = c0; c < c1; ++c) rand[h][size_t(row) * width + c] = got[c - c0];
    }
  };
  for (int p = 0; p < np_; ++p) {
    int c0 = 0;
    if (p > 0) {
      if (plan_cnt[p] > 0) {
        c0 = prefix(p);
        for (int row = 1; row < plan_len[p - 1]; ++row)
          fill(row, c0, prefix(p + 1), plan_len[p - 1], plan_len[p], plan_cnt[p]);
      }
      for (int q = 0; q < p; ++q) {
        if (plan_cnt[q] == 0) continue;
        for (int row = plan_len[p - 1]; row < plan_len[p]; ++row) {
          c0 = q > 0 ? prefix(q) : 0;
          fill(row, c0, prefix(q + 1), q > 0 ? plan_len[q - 1] : 0, plan_len[q], plan_cnt[q]);
        }
      }
    }
    if (plan_cnt[p] == 0) continue;
    int from_start = 1, to_start = 0;
    if (p > 0) { c0 = prefix(p); from_start = plan_len[p - 1]; to_start = plan_len[p - 1]; }
    for (int row = from_start; row < plan_len[p]; ++row)
      fill(row, c0, prefix(p + 1), to_start, plan_len[p], plan_cnt[p]);
  }
  if (short_row || width != r) return fail(RT_EINVAL, "plan for %d tokens has a row with fewer than %d legal blocks", length, r);
  for (int h = 0; h < heads; ++h)
    for (int row = 1; row < nb - 1; ++row)
      for (int c = 0; c < r; ++c)
        out[(size_t(h) * (nb - 2) + (row - 1)) * r + c] = rand[h][size_t(row) * width + c];
  return RT_OK;
}

static bool uses_max_plan(int length, int policy) {
  if (policy == RT_POLICY_HF_UPSTREAM) return length == 1024 || length == 3072 || length == 4096;
  return length % 256 == 0 && length >= 1024;      // python/modeling_big_bird.py:574, from 1024 up
}

static int rand_attn_compute(int length, uint32_t seed, int heads, int max_pos, int policy, int* out);

// Memo table of the plans: a plan is a pure function of (length, seed, heads, max_pos, policy), and drawing one
// costs as many generator steps as the oracle's numpy code (0.1-0.2 ms for a 4096-token sequence of 12 heads), which
// a server would otherwise repeat for every batch and layer.  Bounded by bytes; when full, nothing more is kept.
namespace {
typedef std::tuple<int, uint32_t, int, int, int> PlanKey;
struct PlanCache {
  std::mutex m;
  std::map<PlanKey, std::shared_ptr<const std::vector<int>>> plans;
  int64_t bytes = 0, limit = int64_t(64) << 20, hits = 0, misses = 0;
};
PlanCache& plan_cache() { static PlanCache c; return c; }
}  // namespace

static int rand_attn_impl(int length, uint32_t seed, int heads, int max_pos, int policy, int* out) {
  PlanCache& c = plan_cache();
  const PlanKey key(length, seed, heads, max_pos, policy);
  const size_t cnt = size_t(heads) * size_t(length / RT_BLOCK - 2) * RT_NUM_RAND;
  {
    std::lock_guard<std::mutex> lk(c.m);
    if (c.limit > 0) {
      auto it = c.plans.find(key);
      if (it != c.plans.end()) {
        ++c.hits;
        std::shared_ptr<const std::vector<int>> plan = it->second;
        std::copy(plan->begin(), plan->end(), out);
        return RT_OK;
      }
      ++c.misses;
    }
  }
  const int rc = rand_attn_compute(length, seed, heads, max_pos, policy, out);
  if (rc != RT_OK) return rc;
  std::lock_guard<std::mutex> lk(c.m);
  const int64_t add = int64_t(cnt) * int64_t(sizeof(int)) + 64;
  if (c.limit > 0 && c.bytes + add <= c.limit && !c.plans.count(key)) {
    c.plans[key] = std::make_shared<const std::vector<int>>(out, out + cnt);
    c.bytes += add;
  }
  return RT_OK;
}

static int rand_attn_compute(int length, uint32_t seed, int heads, int max_pos, int policy, int* out) {
  const int nb = length / RT_BLOCK;
  NpRng rng(seed);
  if (uses_max_plan(length, policy)) {
    RT_REQUIRE(max_pos >= length && max_pos % RT_BLOCK == 0, RT_EINVAL,
               "max_pos %d must be a multiple of 64 and at least the sequence length %d", max_pos, length);
    for (int h = 0; h < heads; ++h)
      max_plan_one_head(rng, max_pos, 1024, nb - 2, out + size_t(h) * (nb - 2) * RT_NUM_RAND);
    return RT_OK;
  }
  return with_head_plan(rng, length, heads, out);
}

// Reference generator (head shared): three distinct blocks from the slice each branch of
// layers/multi_headed_attention.cpp:52-123 shuffles.
static void reference_row(NpRng& rng, int i, int n, int* out3) {
  std::vector<int> cand;
  if (i == 1) cand = iota_range(3, n - 1);
  else if (i == 2) cand = iota_range(4, n - 1);
  else if (i == n - 3) cand = iota_range(1, n - 4);
  else if (i == n - 2) cand = iota_range(1, n - 3);
  else
    for (int b = 1; b < n - 1; ++b)
      if (b < i - 1 || b > i + 1) cand.push_back(b);
  rng.permute(cand);
  for (int c = 0; c < RT_NUM_RAND; ++c) out3[c] = cand[c];
}

static int row_len(int i, int n) {
  if (n < RT_MIN_SPARSE_BLOCKS || i == 0 || i == n - 1) return n;
  return (i == 1 || i == n - 2) ? 7 : 8;
}

static int check_seq_blocks(const int* sb, int batch) {
  RT_REQUIRE(sb != nullptr && batch >= 1, RT_EINVAL, "seq_blocks is NULL or the batch is empty (batch=%d)", batch);
  RT_REQUIRE(sb[0] == 0, RT_EINVAL, "seq_blocks[0] must be 0, got %d", sb[0]);
  for (int s = 0; s < batch; ++s)
    RT_REQUIRE(sb[s + 1] > sb[s], RT_EINVAL, "sequence %d has %d blocks", s, sb[s + 1] - sb[s]);
  return RT_OK;
}

}  // namespace rt

using namespace rt;

extern "C" {

const char* rt_last_error_string(void) { return error_buffer(); }
int rt_time_next_launch(void* start_event, void* stop_event) {
  const rt::LaunchEvents pending = rt::take_launch_events();
  rt::set_launch_events(start_event, stop_event);
  return (pending.start || pending.stop) ? 1 : 0;
}
int rt_abi_version(void) { return 1; }

int rt_meta_np_permutations(uint32_t seed, const int* n, int count, int* out) {
  RT_REQUIRE(n && out && count >= 0, RT_EINVAL, "NULL argument");
  NpRng rng(seed);
  for (int c = 0; c < count; ++c) {
    RT_REQUIRE(n[c] >= 0, RT_EINVAL, "negative length %d", n[c]);
    std::vector<int> v = iota_range(0, n[c]);
    rng.permute(v);
    std::copy(v.begin(), v.end(), out);
    out += n[c];
  }
  return RT_OK;
}

int rt_meta_seq_prefix_blocks(const int* seq_lens, int batch, int* out) {
  RT_REQUIRE(seq_lens && out && batch >= 1, RT_EINVAL, "NULL argument or empty batch (batch=%d)", batch);
  out[0] = 0;
  for (int s = 0; s < batch; ++s) {
    RT_REQUIRE(seq_lens[s] > 0 && seq_lens[s] % RT_BLOCK == 0, RT_EINVAL,
               "sequence %d has %d tokens: must be a positive multiple of %d", s, seq_lens[s], RT_BLOCK);
    out[s + 1] = out[s] + seq_lens[s] / RT_BLOCK;
  }
  return RT_OK;
}

int rt_meta_rand_attn(int length, uint32_t seed, int heads, int max_pos, int policy, int* out) {
  RT_REQUIRE(out && heads >= 1, RT_EINVAL, "NULL output or heads=%d", heads);
  RT_REQUIRE(length % RT_BLOCK == 0 && length / RT_BLOCK >= RT_MIN_SPARSE_BLOCKS, RT_EINVAL,
             "length %d: block-sparse plans exist from %d tokens, multiples of %d", length,
             RT_MIN_SPARSE_BLOCKS * RT_BLOCK, RT_BLOCK);
  return rand_attn_impl(length, seed, heads, max_pos, policy, out);
}

int rt_meta_set_plan_cache(int64_t max_bytes, int64_t* hits, int64_t* misses) {
  PlanCache& c = plan_cache();
  std::lock_guard<std::mutex> lk(c.m);
  if (hits) *hits = c.hits;
  if (misses) *misses = c.misses;
  if (max_bytes >= 0) {
    c.limit = max_bytes;
    if (c.bytes > c.limit) { c.plans.clear(); c.bytes = 0; }
  }
  return RT_OK;
}

int rt_meta_to_index_size(const int* sb, int batch, int plan_heads, int64_t* idx_len, int64_t* pos_len) {
  int rc = check_seq_blocks(sb, batch);
  if (rc) return rc;
  RT_REQUIRE(plan_heads >= 1 && idx_len && pos_len, RT_EINVAL, "bad plan_heads=%d or NULL output", plan_heads);
  int64_t e = 0;
  for (int s = 0; s < batch; ++s) {
    int64_t n = sb[s + 1] - sb[s];
    e += n < RT_MIN_SPARSE_BLOCKS ? n * n : 10 * n - 18;
  }
  *idx_len = e * plan_heads;
  *pos_len = int64_t(sb[batch]) * plan_heads + 1;
  return RT_OK;
}

int rt_meta_build_to_index(const int* sb, int batch, int plan_heads, int mode, uint32_t seed, int max_pos,
                           int policy, const int* rand_attn, int* out_idx, int64_t idx_cap, int* out_pos,
                           int64_t pos_cap) {
  int64_t need_idx = 0, need_pos = 0;
  int rc = rt_meta_to_index_size(sb, batch, plan_heads, &need_idx, &need_pos);
  if (rc) return rc;
  RT_REQUIRE(out_idx && out_pos, RT_EINVAL, "NULL output");
  RT_REQUIRE(idx_cap >= need_idx && pos_cap >= need_pos, RT_ENOMEM,
             "CSR needs %lld indices and %lld positions, capacity is %lld / %lld", (long long)need_idx,
             (long long)need_pos, (long long)idx_cap, (long long)pos_cap);
  RT_REQUIRE(mode == RT_PLAN_HF || mode == RT_PLAN_REFERENCE || mode == RT_PLAN_EXPLICIT, RT_EINVAL, "unknown plan mode %d", mode);
  RT_REQUIRE(mode != RT_PLAN_REFERENCE || plan_heads == 1, RT_EINVAL, "the reference plan is shared by all heads (plan_heads must be 1)");
  RT_REQUIRE(mode != RT_PLAN_EXPLICIT || rand_attn, RT_EINVAL, "explicit plan mode needs rand_attn");

  // rand[s] = [plan_heads][n-2][3] for every sparse sequence
  std::vector<std::vector<int>> rand(batch);
  const int* cursor = rand_attn;
  NpRng ref_rng(seed);
  for (int s = 0; s < batch; ++s) {
    const int n = sb[s + 1] - sb[s];
    if (n < RT_MIN_SPARSE_BLOCKS) continue;
    const size_t cnt = size_t(plan_heads) * (n - 2) * RT_NUM_RAND;
    rand[s].resize(cnt);
    if (mode == RT_PLAN_EXPLICIT) {
      for (size_t e = 0; e < cnt; ++e) {
        RT_REQUIRE(cursor[e] >= 0 && cursor[e] < n, RT_EINVAL, "rand_attn names block %d of a %d-block sequence", cursor[e], n);
        rand[s][e] = cursor[e];
      }
      cursor += cnt;
    } else if (mode == RT_PLAN_HF) {
      rc = rand_attn_impl(n * RT_BLOCK, seed, plan_heads, max_pos, policy, rand[s].data());
      if (rc) return rc;
      for (size_t e = 0; e < cnt; ++e)
        RT_REQUIRE(rand[s][e] >= 0 && rand[s][e] < n, RT_EINVAL, "plan names block %d of a %d-block sequence", rand[s][e], n);
    } else {
      for (int i = 1; i < n - 1; ++i) reference_row(ref_rng, i, n, &rand[s][size_t(i - 1) * RT_NUM_RAND]);
    }
  }

  const int nb_total = sb[batch];
  int64_t w = 0;
  out_pos[0] = 0;
  for (int hp = 0; hp < plan_heads; ++hp) {
    for (int s = 0; s < batch; ++s) {
      const int n = sb[s + 1] - sb[s];
      for (int i = 0; i < n; ++i) {
        int* row = out_idx + w;
        if (row_len(i, n) == n) {
          for (int b = 0; b < n; ++b) row[b] = b;
        } else {
          const int* r3 = &rand[s][(size_t(hp) * (n - 2) + (i - 1)) * RT_NUM_RAND];
          int c = 0;
          if (i == 1) { row[c++] = 0; row[c++] = 1; row[c++] = 2; row[c++] = n - 1; }
          else if (i == 2) { row[c++] = 1; row[c++] = 2; row[c++] = 3; row[c++] = n - 1; row[c++] = 0; }
          else if (i == n - 2) { row[c++] = i - 1; row[c++] = i; row[c++] = i + 1; row[c++] = 0; }
          else { row[c++] = i - 1; row[c++] = i; row[c++] = i + 1; row[c++] = 0; row[c++] = n - 1; }
          for (int k = 0; k < RT_NUM_RAND; ++k) row[c++] = r3[k];
        }
        w += row_len(i, n);
        out_pos[size_t(hp) * nb_total + sb[s] + i + 1] = int(w);
      }
    }
  }
  return RT_OK;
}

int rt_meta_block_costs(const int* sb, int batch, int* out_costs, int64_t* total) {
  int rc = check_seq_blocks(sb, batch);
  if (rc) return rc;
  int64_t t = 0;
  for (int s = 0; s < batch; ++s) {
    const int n = sb[s + 1] - sb[s];
    for (int i = 0; i < n; ++i) {
      if (out_costs) out_costs[sb[s] + i] = row_len(i, n);
      t += row_len(i, n);
    }
  }
  if (total) *total = t;
  return RT_OK;
}

int rt_meta_partition_lpt(const int* sb, int batch, int heads, int n_wg, int* out_pos, int* out_ids) {
  int rc = check_seq_blocks(sb, batch);
  if (rc) return rc;
  RT_REQUIRE(heads >= 1 && n_wg >= 1 && out_pos && out_ids, RT_EINVAL, "bad heads=%d / n_wg=%d or NULL output", heads, n_wg);
  const int nb = sb[batch];
  std::vector<int> cost(nb), seq_of(nb);
  for (int s = 0; s < batch; ++s)
    for (int i = sb[s]; i < sb[s + 1]; ++i) { cost[i] = row_len(i - sb[s], sb[s + 1] - sb[s]); seq_of[i] = s; }
  std::vector<int> order(nb);
  for (int i = 0; i < nb; ++i) order[i] = i;
  std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return cost[a] > cost[b]; });
  // min-heap on (load, workgroup id): python/util.py:15,19,27-28
  typedef std::pair<int64_t, int> slot;
  std::priority_queue<slot, std::vector<slot>, std::greater<slot>> heap;
  for (int c = 0; c < n_wg; ++c) heap.push(slot(0, c));
  std::vector<std::vector<int>> parts(n_wg);
  for (int b : order) {
    const int s = seq_of[b], n = sb[s + 1] - sb[s];
    for (int h = 0; h < heads; ++h) {
      slot top = heap.top();
      heap.pop();
      parts[top.second].push_back(b - sb[s] + h * n + sb[s] * heads);
      heap.push(slot(top.first + cost[b], top.second));
    }
  }
  int w = 0;
  out_pos[0] = 0;
  for (int c = 0; c < n_wg; ++c) {
    for (int u : parts[c]) out_ids[w++] = u;
    out_pos[c + 1] = w;
  }
  return RT_OK;
}

int rt_meta_check_partition(const int* from_pos, const int* from_idx, int n_wg, int total_blocks, int heads) {
  RT_REQUIRE(from_pos && from_idx, RT_EINVAL, "NULL pointer");
  RT_REQUIRE(n_wg >= 1 && total_blocks >= 1 && heads >= 1, RT_EINVAL, "bad n_wg=%d / total_blocks=%d / heads=%d", n_wg,
             total_blocks, heads);
  const int64_t units = int64_t(total_blocks) * heads;
  RT_REQUIRE(units < (int64_t(1) << 31), RT_EINVAL, "too many units: %d blocks x %d heads", total_blocks, heads);
  RT_REQUIRE(from_pos[0] == 0 && from_pos[n_wg] == units, RT_EINVAL,
             "partition: from_pos must run from 0 to %lld, got %d .. %d", (long long)units, from_pos[0], from_pos[n_wg]);
  for (int c = 0; c < n_wg; ++c)
    RT_REQUIRE(from_pos[c] <= from_pos[c + 1], RT_EINVAL, "partition: from_pos decreases at workgroup %d", c);
  std::vector<uint8_t> seen(size_t(units), 0);
  for (int64_t i = 0; i < units; ++i) {
    const int u = from_idx[i];
    RT_REQUIRE(u >= 0 && u < units, RT_EINVAL, "partition: unit id %d at position %lld is outside [0, %lld)", u,
               (long long)i, (long long)units);
    RT_REQUIRE(!seen[u], RT_EINVAL, "partition: unit id %d is listed twice", u);
    seen[u] = 1;
  }
  return RT_OK;
}

int rt_meta_check_to_index(const int* to_idx, const int* to_pos, int64_t idx_len, const int* seq_blocks, int batch,
                           int plan_heads) {
  RT_REQUIRE(to_idx && to_pos && seq_blocks, RT_EINVAL, "NULL pointer");
  RT_REQUIRE(batch >= 1 && plan_heads >= 1 && idx_len >= 0, RT_EINVAL, "bad batch=%d / plan_heads=%d / idx_len=%lld", batch,
             plan_heads, (long long)idx_len);
  RT_REQUIRE(seq_blocks[0] == 0, RT_EINVAL, "block index: seq_blocks must start at 0, got %d", seq_blocks[0]);
  for (int s = 0; s < batch; ++s)
    RT_REQUIRE(seq_blocks[s + 1] > seq_blocks[s], RT_EINVAL, "block index: sequence %d has no blocks", s);
  const int nb = seq_blocks[batch];
  const int64_t rows = int64_t(plan_heads) * nb;
  RT_REQUIRE(to_pos[0] == 0, RT_EINVAL, "block index: to_pos must start at 0, got %d", to_pos[0]);
  RT_REQUIRE(to_pos[rows] <= idx_len, RT_EINVAL, "block index: to_pos ends at %d, to_idx holds %lld entries", to_pos[rows],
             (long long)idx_len);
  for (int hp = 0; hp < plan_heads; ++hp)
    for (int s = 0; s < batch; ++s) {
      const int n = seq_blocks[s + 1] - seq_blocks[s];
      for (int i = 0; i < n; ++i) {
        const int64_t row = int64_t(hp) * nb + seq_blocks[s] + i;
        const int p0 = to_pos[row], p1 = to_pos[row + 1];
        RT_REQUIRE(p1 > p0, RT_EINVAL, "block index: row %lld (plan head %d, sequence %d, block %d) is empty or to_pos decreases",
                   (long long)row, hp, s, i);
        for (int p = p0; p < p1; ++p)
          RT_REQUIRE(to_idx[p] >= 0 && to_idx[p] < n, RT_EINVAL,
                     "block index: entry %d of row %lld names block %d, the sequence has %d", p - p0, (long long)row, to_idx[p], n);
      }
    }
  return RT_OK;
}

}  // extern "C"
