// Host-only stress of the metadata pipeline (device = -1: no GPU call is made), meant to be
// built with ThreadSanitizer: publish / acquire / release in the orders the layer API can
// produce, back-to-back publishes, and destruction right after a publish.
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "../../include/raptor_t_hip.h"

#define CHECK(x)                                                                      \
  do {                                                                                \
    int rc_ = (x);                                                                    \
    if (rc_ != RT_OK) { std::printf("FAILED %s -> %d: %s\n", #x, rc_, rt_last_error_string()); return 1; } \
  } while (0)

int main() {
  const int layers = 8, heads = 4;
  unsigned rng = 12345;
  auto next = [&]() { rng = rng * 1664525u + 1013904223u; return rng >> 8; };
  for (int round = 0; round < 6; ++round) {
    rt_pipeline* p = nullptr;
    CHECK(rt_pipeline_create(&p, layers, heads, RT_PLAN_HF, 4096, RT_POLICY_REFERENCE_PATCHED, round % 3 != 2, -1));
    for (int batch = 0; batch < 40; ++batch) {
      const int b = 1 + int(next() % 6);
      std::vector<int> sb(b + 1, 0);
      for (int s = 0; s < b; ++s) sb[s + 1] = sb[s] + 1 + int(next() % 40);
      CHECK(rt_pipeline_publish(p, sb.data(), b));
      if (next() % 4 == 0) CHECK(rt_pipeline_publish(p, sb.data(), b));      // two signals, one batch
      int64_t n_idx = 0, n_pos = 0;
      CHECK(rt_meta_to_index_size(sb.data(), b, heads, &n_idx, &n_pos));
      std::vector<int> want_idx(n_idx), want_pos(n_pos);
      for (int l = 0; l < layers; ++l) {
        const int layer = (round & 1) ? layers - 1 - l : l;
        const int *idx = nullptr, *pos = nullptr;
        int ph = 0;
        double wait = 0;
        CHECK(rt_pipeline_acquire(p, layer, nullptr, &idx, &pos, &ph, &wait));
        CHECK(rt_meta_build_to_index(sb.data(), b, heads, RT_PLAN_HF, unsigned(layer), 4096, RT_POLICY_REFERENCE_PATCHED,
                                     nullptr, want_idx.data(), n_idx, want_pos.data(), n_pos));
        for (int64_t i = 0; i < n_idx; ++i)
          if (idx[i] != want_idx[i]) { std::printf("FAILED: layer %d index %lld differs\n", layer, (long long)i); return 1; }
        for (int64_t i = 0; i < n_pos; ++i)
          if (pos[i] != want_pos[i]) { std::printf("FAILED: layer %d position %lld differs\n", layer, (long long)i); return 1; }
        CHECK(rt_pipeline_release(p, layer, nullptr));
      }
    }
    if (round % 2 == 0) {                       // destroy while the workers are busy with a fresh batch
      std::vector<int> sb = {0, 64, 128, 192};
      CHECK(rt_pipeline_publish(p, sb.data(), 3));
    }
    CHECK(rt_pipeline_destroy(p));
  }
  std::printf("pipeline_stress OK\n");
  return 0;
}
