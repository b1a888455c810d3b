// Host-only driver of the metadata entry points, meant to be built with AddressSanitizer and
// UndefinedBehaviorSanitizer: random batch geometries (including sequences below 12 blocks, which
// run full attention, and the shortest sparse ones), exact-capacity output buffers allocated on the
// heap so that one element too many is caught, capacities one short (must be refused without a
// write), and malformed arguments (must be refused, never dereferenced).
#include <cstdio>
#include <cstdlib>
#include <memory>
#include <vector>

#include "../../include/raptor_t_hip.h"

#define CHECK(x)                                                                      \
  do {                                                                                \
    int rc_ = (x);                                                                    \
    if (rc_ != RT_OK) { std::printf("FAILED %s -> %d: %s\n", #x, rc_, rt_last_error_string()); return 1; } \
  } while (0)
#define REFUSED(x)                                                                    \
  do {                                                                                \
    int rc_ = (x);                                                                    \
    if (rc_ == RT_OK) { std::printf("FAILED: %s was accepted\n", #x); return 1; }     \
  } while (0)

int main() {
  unsigned rng = 2024;
  auto next = [&]() { rng = rng * 1664525u + 1013904223u; return rng >> 8; };
  for (int round = 0; round < 300; ++round) {
    const int batch = 1 + int(next() % 5);
    const int heads = 1 + int(next() % 4);
    std::vector<int> lens(batch);
    for (int& l : lens) {
      const unsigned kind = next() % 4;
      const int blocks = kind == 0 ? 1 + int(next() % 11) : (kind == 1 ? 12 + int(next() % 3) : 12 + int(next() % 53));
      l = 64 * blocks;
    }
    std::unique_ptr<int[]> sb(new int[batch + 1]);
    CHECK(rt_meta_seq_prefix_blocks(lens.data(), batch, sb.get()));
    const int nb = sb[batch];
    for (int mode : {RT_PLAN_HF, RT_PLAN_REFERENCE}) {
      const int ph = mode == RT_PLAN_HF ? heads : 1;
      int64_t n_idx = 0, n_pos = 0;
      CHECK(rt_meta_to_index_size(sb.get(), batch, ph, &n_idx, &n_pos));
      std::unique_ptr<int[]> idx(new int[n_idx]), pos(new int[n_pos]);
      const int policy = (round & 1) ? RT_POLICY_HF_UPSTREAM : RT_POLICY_REFERENCE_PATCHED;
      CHECK(rt_meta_build_to_index(sb.get(), batch, ph, mode, unsigned(round), 4096, policy, nullptr, idx.get(), n_idx,
                                   pos.get(), n_pos));
      if (pos[n_pos - 1] != n_idx) { std::printf("FAILED: last position %d != %lld\n", pos[n_pos - 1], (long long)n_idx); return 1; }
      for (int64_t r = 0; r + 1 < n_pos; ++r) {
        if (pos[r] > pos[r + 1]) { std::printf("FAILED: positions decrease at row %lld\n", (long long)r); return 1; }
      }
      // every listed block must lie inside the row's own sequence
      for (int hp = 0; hp < ph; ++hp)
        for (int s = 0; s < batch; ++s)
          for (int g = sb[s]; g < sb[s + 1]; ++g)
            for (int e = pos[int64_t(hp) * nb + g]; e < pos[int64_t(hp) * nb + g + 1]; ++e)
              if (idx[e] < 0 || idx[e] >= sb[s + 1] - sb[s]) { std::printf("FAILED: block %d outside its sequence\n", idx[e]); return 1; }
      if (n_idx > 0)
        REFUSED(rt_meta_build_to_index(sb.get(), batch, ph, mode, 0u, 4096, policy, nullptr, idx.get(), n_idx - 1, pos.get(), n_pos));
      REFUSED(rt_meta_build_to_index(sb.get(), batch, ph, mode, 0u, 4096, policy, nullptr, idx.get(), n_idx, pos.get(), n_pos - 1));
    }
    // per-head plans of single sequences, exact-size heap buffers
    for (int s = 0; s < batch; ++s) {
      const int n = lens[s] / 64;
      if (n < RT_MIN_SPARSE_BLOCKS) continue;
      std::unique_ptr<int[]> plan(new int[size_t(heads) * (n - 2) * RT_NUM_RAND]);
      CHECK(rt_meta_rand_attn(lens[s], unsigned(round), heads, 4096, RT_POLICY_REFERENCE_PATCHED, plan.get()));
      for (int i = 0; i < heads * (n - 2) * RT_NUM_RAND; ++i)
        if (plan[i] < 0 || plan[i] >= n) { std::printf("FAILED: plan entry %d outside [0, %d)\n", plan[i], n); return 1; }
    }
    // LPT plan
    const int n_wg = 1 + int(next() % 200);
    std::unique_ptr<int[]> fpos(new int[n_wg + 1]), fids(new int[size_t(heads) * nb]);
    CHECK(rt_meta_partition_lpt(sb.get(), batch, heads, n_wg, fpos.get(), fids.get()));
    if (fpos[0] != 0 || fpos[n_wg] != heads * nb) { std::printf("FAILED: plan does not cover the units\n"); return 1; }
    std::vector<char> seen(size_t(heads) * nb, 0);
    for (int i = 0; i < heads * nb; ++i) {
      if (fids[i] < 0 || fids[i] >= heads * nb || seen[fids[i]]) { std::printf("FAILED: unit %d missing or twice\n", fids[i]); return 1; }
      seen[fids[i]] = 1;
    }
    std::unique_ptr<int[]> costs(new int[nb]);
    int64_t total = 0;
    CHECK(rt_meta_block_costs(sb.get(), batch, costs.get(), &total));
    int64_t sum = 0;
    for (int g = 0; g < nb; ++g) sum += costs[g];
    if (sum != total) { std::printf("FAILED: costs do not add up\n"); return 1; }
    // numpy permutations into an exact-size buffer
    int sizes[3] = {1 + int(next() % 50), 1 + int(next() % 50), 1 + int(next() % 50)};
    std::unique_ptr<int[]> perm(new int[sizes[0] + sizes[1] + sizes[2]]);
    CHECK(rt_meta_np_permutations(unsigned(round), sizes, 3, perm.get()));
  }
  // malformed arguments
  int one[2] = {0, 1}, out[8], bad_len[1] = {100}, neg[2] = {0, -3}, len64[1] = {64};
  int64_t a = 0, b = 0;
  REFUSED(rt_meta_seq_prefix_blocks(bad_len, 1, out));
  REFUSED(rt_meta_seq_prefix_blocks(nullptr, 1, out));
  REFUSED(rt_meta_seq_prefix_blocks(len64, 0, out));
  REFUSED(rt_meta_to_index_size(neg, 1, 1, &a, &b));
  REFUSED(rt_meta_to_index_size(one, 1, 0, &a, &b));
  REFUSED(rt_meta_to_index_size(one, 1, 1, nullptr, &b));
  REFUSED(rt_meta_rand_attn(64 * 11, 0u, 1, 4096, RT_POLICY_REFERENCE_PATCHED, out));
  REFUSED(rt_meta_rand_attn(8192, 0u, 1, 4096, RT_POLICY_REFERENCE_PATCHED, out));
  REFUSED(rt_meta_partition_lpt(one, 1, 1, 0, out, out));
  REFUSED(rt_meta_build_to_index(one, 1, 1, 99, 0u, 4096, 0, nullptr, out, 8, out, 8));
  REFUSED(rt_meta_build_to_index(one, 1, 1, RT_PLAN_EXPLICIT, 0u, 4096, 0, nullptr, out, 0, out, 0));
  std::printf("meta_fuzz OK\n");
  return 0;
}
