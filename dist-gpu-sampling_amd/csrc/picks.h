// Which neighbour positions a seed row keeps: the "dgs-philox-1" contract shared by the
// per-hop sampler (sample.hip), the fused sampler (pipeline.hip) and the CPU oracle.
#ifndef DGS_CSRC_PICKS_H_
#define DGS_CSRC_PICKS_H_

#include "common.h"

namespace dgs {

__host__ __device__ inline int64_t pick_count(int64_t deg, int64_t k, bool replace) {
  if (replace) return deg == 0 ? 0 : k;
  return deg < k ? deg : k;
}

// Position inside the row for output slot l (0 <= l < G, k <= G) of a row of degree deg.
// All G lanes of the group call this together (G consecutive lanes of one wave, the first
// being lane group_lane0 of the wave); returns false when the slot holds no pick.
//   replacement:        slot l holds draw l reduced to [0, deg)
//   deg <= k:           the whole row, slot l = position l
//   deg >  k (Floyd):   slot s draws t in [0, deg-k+s] and keeps it unless a lower slot
//                       already kept t, in which case it keeps deg-k+s (which no lower slot
//                       can hold); the slots are resolved in order with __shfl / __ballot.
// `words` is the Philox block of draw l of the row (philox_draw_words), which the caller may have
// computed before the degree was known.
template <int G>
__device__ __forceinline__ bool pick_position(uint32_t deg, int k, bool replace, int l, int group_lane0,
                                              const PhiloxWords& words, uint32_t* pos) {
  if (replace) {
    if (deg == 0 || l >= k) return false;
    *pos = philox_reduce(words, deg);
    return true;
  }
  if (deg <= uint32_t(k)) {
    *pos = uint32_t(l);
    return uint32_t(l) < deg;
  }
  constexpr uint64_t group_mask = G == 64 ? ~uint64_t(0) : ((uint64_t(1) << (G & 63)) - 1);
  const uint32_t top = deg - uint32_t(k) + uint32_t(l);
  uint32_t cand = 0xffffffffu;
  if (l < k) cand = philox_reduce(words, top + 1u);
  uint32_t kept = cand;
  for (int s = 1; s < k; ++s) {
    const uint32_t c = __shfl(cand, s, G);
    const uint64_t hit = (__ballot(kept == c && l < s) >> group_lane0) & group_mask;
    if (l == s && hit) kept = top;
  }
  *pos = kept;
  return l < k;
}

template <int G>
__device__ __forceinline__ bool pick_position(uint32_t deg, int k, bool replace, int l, int group_lane0,
                                              uint64_t rng_seed, uint32_t rng_stream, int64_t row,
                                              uint32_t* pos) {
  return pick_position<G>(deg, k, replace, l, group_lane0, philox_draw_words(rng_seed, rng_stream, row, uint32_t(l)),
                          pos);
}

}  // namespace dgs
#endif
