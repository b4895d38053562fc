/* wave.c -- lane-level models of the wave coalescer and of the wave-aggregated
 * fetch-and-add.  Test infrastructure only (see oracle.h).
 *
 * orc_coalesce restates WfCoalOn::coalesce, library/src/wf_coal_policy.cpp:57-172:
 * lane l is absorbed iff l != 0, lane l-1 is active, sizes (compared as 32-bit
 * values, :87) and PEs match, and lane l's source and destination start where
 * lane l-1's end; a lane that is not absorbed sends, and its size grows by one
 * `size` for each lane of the unbroken absorbed run directly above it.
 * Pinned by: the three-message example in the reference's own comment
 * (wf_coal_policy.cpp:39-53) and exhaustive agreement with a brute-force
 * "longest run" formulation on 8-lane miniatures.
 *
 * orc_fetch_incr restates Block::fetch_incr,
 * library/src/containers/share_strategy.hpp:70-83 with its helpers in
 * share_strategy.cpp:32-212: the lowest active lane adds the number of active
 * lanes to the counter, every active lane returns the old counter plus the
 * number of active lanes below it.
 * Pinned by: clients/unit_tests/bitwise_gtest.cpp:1384-1526 (mask 0xA -> counter 2,
 * all ones -> 64, upper half -> 32, 0xF0F0... -> 32, 1024 x 1024 threads ->
 * 1048576, logical lane 1 receives a value congruent to 1 modulo the number
 * of active lanes).
 */
#include "oracle.h"

void orc_coalesce(uint64_t lane_mask, const int32_t *pe, const uint64_t *src, const uint64_t *dst,
                  const uint64_t *size, uint8_t *must_send, uint64_t *out_size) {
  int absorbed[64];
  for (int l = 0; l < 64; ++l) {
    absorbed[l] = 0;
    if (!((lane_mask >> l) & 1)) continue;
    if (l == 0 || !((lane_mask >> (l - 1)) & 1)) continue;
    absorbed[l] = (uint32_t)size[l - 1] == (uint32_t)size[l] && src[l - 1] + size[l] == src[l] &&
                  dst[l - 1] + size[l] == dst[l] && pe[l - 1] == pe[l];
  }
  for (int l = 0; l < 64; ++l) {
    if (!((lane_mask >> l) & 1)) continue;
    must_send[l] = (uint8_t)!absorbed[l];
    out_size[l] = size[l];
    if (!absorbed[l]) {
      int run = 0;
      for (int u = l + 1; u < 64 && absorbed[u]; ++u) ++run;
      out_size[l] = size[l] * (uint64_t)(1 + run);
    }
  }
}

void orc_fetch_incr(uint64_t lane_mask, uint64_t *counter, uint64_t out[64]) {
  uint64_t base = *counter;
  uint64_t below = 0;
  for (int l = 0; l < 64; ++l) {
    if ((lane_mask >> l) & 1) {
      out[l] = base + below;
      ++below;
    } else {
      out[l] = ~0ull;
    }
  }
  *counter = base + below;
}
