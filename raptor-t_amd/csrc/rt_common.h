// Shared helpers of the C-ABI library: per-thread error text and argument checks.
#pragma once
#include <cstdarg>
#include <cstdio>

#include "../../include/raptor_t_hip.h"

namespace rt {

char* error_buffer();                       // per-thread, 512 bytes
int fail(int code, const char* fmt, ...);   // formats into the buffer, returns code

// The pair of events rt_time_next_launch left for this thread's next kernel launch (both null: none); taking
// them clears them.
struct LaunchEvents { void* start; void* stop; };
LaunchEvents take_launch_events();

// Block-sparse attention with every tensor in fp32 (bs_attention_f32.hip); arguments as the fp16 / bf16 launch,
// already checked by it.
int launch_attention_f32(const void* q, const void* q_rows, const void* q_bias, float q_scale, const void* k,
                         const void* vt, void* out, const int* seq_blocks_dev, const int* seq_tokens_dev, int batch,
                         int total_blocks, int heads, const int* to_idx, const int* to_pos, int plan_heads,
                         const int* from_idx, const int* from_pos, int n_wg, void* stream);

}  // namespace rt

#define RT_REQUIRE(cond, code, ...) \
  do {                              \
    if (!(cond)) return rt::fail((code), __VA_ARGS__); \
  } while (0)
