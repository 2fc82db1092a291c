// The two weighted pick rules as device procedures over one seed row, shared by the per-hop
// weighted operator (weighted.hip) and the fused multi-hop sampler (pipeline.hip).
//   without replacement: every position races with the key E / w (E a unit exponential variate
//     from the row's Philox stream); a group of G lanes keeps the num_picks smallest
//     (key, position) pairs in order, lane l holding the l-th;
//   with replacement: weights become integer shares floor(w * 2^(32-E)), 2^E the power of two
//     above the row's largest weight; their sums are exact in any order, and draws in [0, sum)
//     are located against the running inclusive sum.
// Both are evaluated from exactly rounded operations only (weights.h), so the picks equal the CPU
// oracle's bit for bit whatever the launch shape.  Loops that contain cross-lane operations run a
// wave-uniform number of times: a group that has run out of work keeps executing with empty
// candidates.  Rows above long_row<G>() positions are meant for the *_long_row procedures, which
// spread a row over the 16 waves of a 1024-thread block.
#ifndef DGS_CSRC_RACE_H_
#define DGS_CSRC_RACE_H_

#include "common.h"
#include "weights.h"

namespace dgs {

constexpr int kLongBlock = 1024;
constexpr int kLongWaves = kLongBlock / kWave;
constexpr int kMaxWeightedPicks = 64;      // without replacement: one lane per kept pair
constexpr uint64_t kNoKey = ~uint64_t(0);  // above every key, +inf included
constexpr uint32_t kNoPos = 0xffffffffu;

// Rows above this many neighbours leave the G-lane groups for the block-per-row kernels.
template <int G>
constexpr uint32_t long_row() { return 32u * G; }

// The lanes of one G-lane group: l = lane in the group, lane0 = the group's first lane in the wave.
template <int G>
struct Group {
  int l;
  int lane0;
  __device__ __forceinline__ Group() : l(int(threadIdx.x) & (G - 1)), lane0((int(threadIdx.x) & (kWave - 1)) & ~(G - 1)) {}
  __device__ __forceinline__ uint64_t ballot(bool pred) const {
    constexpr uint64_t mask = G == 64 ? ~uint64_t(0) : ((uint64_t(1) << (G & 63)) - 1);
    return (__ballot(pred) >> lane0) & mask;
  }
};

__device__ __forceinline__ bool race_less(uint64_t ka, uint32_t pa, uint64_t kb, uint32_t pb) {
  return ka < kb || (ka == kb && pa < pb);
}

// Cross-lane moves on the data-parallel-primitive path of the VALU where the pattern allows it
// (no LDS round trip), through ds_bpermute otherwise.
__device__ __forceinline__ uint32_t lane_xor(uint32_t v, int stride) {
  switch (stride) {
    case 1: return uint32_t(__builtin_amdgcn_update_dpp(int(v), int(v), 0xB1, 0xf, 0xf, false));  // quad_perm 1,0,3,2
    case 2: return uint32_t(__builtin_amdgcn_update_dpp(int(v), int(v), 0x4E, 0xf, 0xf, false));  // quad_perm 2,3,0,1
    case 4: {  // lanes with bit 2 clear read four lanes up (row_shl:4), the others four lanes down (row_shr:4)
      const int t = __builtin_amdgcn_update_dpp(int(v), int(v), 0x104, 0xf, 0x5, false);
      return uint32_t(__builtin_amdgcn_update_dpp(t, int(v), 0x114, 0xf, 0xa, false));
    }
    case 8: return uint32_t(__builtin_amdgcn_update_dpp(int(v), int(v), 0x128, 0xf, 0xf, false));  // row_ror:8
    default: return __shfl_xor(v, stride, kWave);
  }
}
__device__ __forceinline__ uint64_t lane_xor(uint64_t v, int stride) {
  return uint64_t(lane_xor(uint32_t(v), stride)) | (uint64_t(lane_xor(uint32_t(v >> 32), stride)) << 32);
}
// value of the lane below; lane 0 of the wave keeps its own (callers ignore a group's lane 0)
__device__ __forceinline__ uint32_t lane_below(uint32_t v) {
  return uint32_t(__builtin_amdgcn_update_dpp(int(v), int(v), 0x138, 0xf, 0xf, false));  // wave_shr:1
}
__device__ __forceinline__ uint64_t lane_below(uint64_t v) {
  return uint64_t(lane_below(uint32_t(v))) | (uint64_t(lane_below(uint32_t(v >> 32))) << 32);
}
// value of lane `src` (the same for the whole wave) as a scalar
__device__ __forceinline__ uint32_t lane_read(uint32_t v, int src) {
  return uint32_t(__builtin_amdgcn_readlane(int(v), src));
}
__device__ __forceinline__ uint64_t lane_read(uint64_t v, int src) {
  return uint64_t(lane_read(uint32_t(v), src)) | (uint64_t(lane_read(uint32_t(v >> 32), src)) << 32);
}

// A value known to be the same in every lane of the wave, moved to scalar registers: it stops
// occupying a vector register per lane, and loads addressed by it become scalar loads.
__device__ __forceinline__ uint32_t wave_uniform(uint32_t v) {
  return uint32_t(__builtin_amdgcn_readfirstlane(int(v)));
}
__device__ __forceinline__ int64_t wave_uniform(int64_t v) {
  const uint64_t u = uint64_t(v);
  return int64_t(uint64_t(wave_uniform(uint32_t(u))) | (uint64_t(wave_uniform(uint32_t(u >> 32))) << 32));
}

// A group's num_picks best so far, ascending over lanes 0 .. k-1; other lanes hold (kNoKey, kNoPos).
struct Race {
  uint64_t key;
  uint32_t pos;
  uint64_t last_key;  // entry of lane k-1: what a candidate has to beat
  uint32_t last_pos;
};

__device__ __forceinline__ void race_reset(Race& r) {
  r.key = r.last_key = kNoKey;
  r.pos = r.last_pos = kNoPos;
}

template <int G>
__device__ __forceinline__ void race_refresh_last(Race& r, int k) {
  if constexpr (G == kWave) {
    r.last_key = lane_read(r.key, k - 1);
    r.last_pos = lane_read(r.pos, k - 1);
  } else {
    r.last_key = __shfl(r.key, k - 1, G);
    r.last_pos = __shfl(r.pos, k - 1, G);
  }
}

// Bitonic sort of one (key, position) pair per lane over every G-lane group, ascending.  With
// kByKeyOnly the positions ride along uncompared, which is right whenever the keys are distinct.
template <int G, bool kByKeyOnly, typename KeyT>
__device__ __forceinline__ void group_sort(KeyT& key, uint32_t& pos, int l) {
#pragma unroll
  for (int size = 2; size <= G; size <<= 1) {
#pragma unroll
    for (int stride = size >> 1; stride > 0; stride >>= 1) {
      const KeyT ok = lane_xor(key, stride);
      const uint32_t op = lane_xor(pos, stride);
      const bool take_min = ((l & stride) == 0) == ((l & size) == 0);
      // distinct pairs: "the other one is smaller" decides both the lower and the upper lane
      const bool other_less = kByKeyOnly ? ok < key : race_less(ok, op, key, pos);
      const bool same = kByKeyOnly ? ok == key : (ok == key && op == pos);
      if (other_less == take_min && !same) {
        key = ok;
        pos = op;
      }
    }
  }
}

// First G candidates (kNoKey = none): sorted over the group, then cut to k.  Keys are distinct
// unless two finite keys coincide bit for bit (keys of unusable weights carry their position):
// the sort compares keys alone and is redone on full pairs when equal neighbours show up.
template <int G>
__device__ __forceinline__ void race_seed(Race& r, const Group<G>& g, uint64_t ck, uint32_t cp, int k) {
  uint64_t key = ck;
  uint32_t pos = ck == kNoKey ? kNoPos : cp;
  group_sort<G, true>(key, pos, g.l);
  if (__ballot(g.l > 0 && key != kNoKey && key == lane_below(key))) {
    key = ck;
    pos = ck == kNoKey ? kNoPos : cp;
    group_sort<G, false>(key, pos, g.l);
  }
  if (g.l >= k) {
    key = kNoKey;
    pos = kNoPos;
  }
  r.key = key;
  r.pos = pos;
  race_refresh_last<G>(r, k);
}

// G more candidates: those that beat the group's last entry are inserted one by one, each by
// shifting the entries above it up a lane.  With one group per wave the newcomer and the bar are
// scalars and the loop is a scalar branch.
template <int G>
__device__ __forceinline__ void race_offer(Race& r, const Group<G>& g, uint64_t ck, uint32_t cp, int k) {
  uint64_t hits = g.ballot(ck != kNoKey && race_less(ck, cp, r.last_key, r.last_pos));
  if constexpr (G == kWave) {
    while (hits) {
      const int b = __builtin_ctzll(hits);
      hits &= hits - 1;
      const uint64_t nk = lane_read(ck, b);
      const uint32_t np = lane_read(cp, b);
      if (!race_less(nk, np, r.last_key, r.last_pos)) continue;  // the bar moved since the ballot
      const uint64_t pk = lane_below(r.key);
      const uint32_t pp = lane_below(r.pos);
      if (race_less(nk, np, r.key, r.pos)) {  // an entry above the newcomer moves up or makes room
        const bool shift = g.l > 0 && race_less(nk, np, pk, pp);
        r.key = shift ? pk : nk;
        r.pos = shift ? pp : np;
      }
      if (g.l >= k) {
        r.key = kNoKey;
        r.pos = kNoPos;
      }
      race_refresh_last<G>(r, k);
    }
  } else {
    while (__ballot(hits != 0)) {
      const bool has = hits != 0;
      const int b = has ? __builtin_ctzll(hits) : 0;
      hits &= hits - 1;
      const uint64_t nk = __shfl(ck, b, G);
      const uint32_t np = __shfl(cp, b, G);
      const uint64_t pk = lane_below(r.key);
      const uint32_t pp = lane_below(r.pos);
      if (has && race_less(nk, np, r.last_key, r.last_pos) && race_less(nk, np, r.key, r.pos)) {
        const bool shift = g.l > 0 && race_less(nk, np, pk, pp);
        r.key = shift ? pk : nk;
        r.pos = shift ? pp : np;
      }
      if (g.l >= k) {
        r.key = kNoKey;
        r.pos = kNoPos;
      }
      race_refresh_last<G>(r, k);
    }
  }
}

// The waves of a block that share one row publish the key of their last entry once they hold
// num_picks entries (kNoKey before); the smallest of these bounds the row's final last key from
// above, so a candidate beyond it can be dropped unseen.  Stale reads only make the bound looser.
__device__ __forceinline__ uint64_t lowest_bar(uint64_t* bars, int lane) {
  uint64_t v = __atomic_load_n(&bars[lane & (kLongWaves - 1)], __ATOMIC_RELAXED);
#pragma unroll
  for (int stride = 1; stride < kLongWaves; stride <<= 1) {
    const uint64_t o = lane_xor(v, stride);
    if (o < v) v = o;
  }
  return v;
}

__device__ __forceinline__ uint64_t lowest_bar_after_sync(uint64_t* bars, int lane) {
  __syncthreads();  // every wave of the block has published its final bar
  return lowest_bar(bars, lane);
}

// Race keys of the four G-position steps of the stretch that begins at position sb (a multiple of
// 4 G) of the group's row, kNoKey from `end` on: one Philox block per lane covers the stretch
// (four words each), the word of position sb + G c + l sits in lane (G / 4) c + l / 4 of the
// group.  The four steps are independent: their loads are issued together and their key
// arithmetic (long dependent float64 chains) interleaves.
template <int G>
__device__ __forceinline__ void stretch_keys(const Group<G>& g, const TierView<float>& probs, int64_t start,
                                             uint64_t sb, uint64_t end, uint64_t rng_seed, uint32_t rng_stream,
                                             int64_t row, uint64_t ck[4]) {
  float wt[4];
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const uint64_t p = sb + uint64_t(G) * c + uint32_t(g.l);
    wt[c] = p < end ? probs.at(start + int64_t(p)) : 0.0f;
  }
  PhiloxWords w{{0, 0, 0, 0}};
  if (sb + 4u * uint32_t(g.l) < end)
    w = philox4x32_10(0x80000000u | (uint32_t(sb >> 2) + uint32_t(g.l)), rng_stream, uint32_t(uint64_t(row)),
                      uint32_t(uint64_t(row) >> 32), uint32_t(rng_seed), uint32_t(rng_seed >> 32));
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const int src = (G / 4) * c + (g.l >> 2);
    const uint32_t a0 = __shfl(w.w[0], src, G), a1 = __shfl(w.w[1], src, G);
    const uint32_t a2 = __shfl(w.w[2], src, G), a3 = __shfl(w.w[3], src, G);
    const uint32_t x = (g.l & 2) ? ((g.l & 1) ? a3 : a2) : ((g.l & 1) ? a1 : a0);
    const uint64_t p = sb + uint64_t(G) * c + uint32_t(g.l);
    ck[c] = p < end ? race_key(x, wt[c], uint32_t(p)) : kNoKey;
  }
}

// Runs positions [begin, end) of the group's row, in steps of `stride` (begin and stride multiples
// of 4 G), through its race.  `bars` (block-per-row kernel only) is the block's table of published
// last keys.
template <int G>
__device__ __forceinline__ void race_scan(Race& r, const Group<G>& g, const TierView<float>& probs, int64_t start,
                                          uint64_t begin, uint64_t end, uint64_t stride, int k, uint64_t rng_seed,
                                          uint32_t rng_stream, int64_t row, uint64_t* bars = nullptr) {
  bool first = true;
  uint64_t published = kNoKey;
  for (uint64_t sb = begin; __ballot(sb < end); sb += stride) {
    uint64_t ck[4];
    stretch_keys<G>(g, probs, start, sb, end, rng_seed, rng_stream, row, ck);
    const uint64_t bar = bars != nullptr ? lowest_bar(bars, g.l) : kNoKey;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const uint64_t cb = sb + uint64_t(G) * c;
      if (!__ballot(cb < end)) break;
      const uint32_t p = uint32_t(cb) + uint32_t(g.l);
      if (first) {
        race_seed<G>(r, g, ck[c], p, k);
        first = false;
      } else {
        race_offer<G>(r, g, ck[c] > bar ? kNoKey : ck[c], p, k);
      }
    }
    if (bars != nullptr && r.last_key < published) {
      published = r.last_key;
      if (g.l == 0) __atomic_store_n(&bars[threadIdx.x / kWave], published, __ATOMIC_RELAXED);
    }
  }
}

// ---- the same race on the upper halves of the keys ----
//
// The upper 32 bits of a key (sign, exponent, 20 bits of the fraction) decide nearly every
// comparison.  A group first races on them alone, at a fraction of the instructions of 64-bit
// compare-and-move sequences, and keeps track of whether that was enough: it was unless two of the
// kept halves are equal, or a candidate that was dropped (refused at the bar, cut after the first
// sort, or pushed out) had the half that ends up as the bar.  Then, and only then, the row is
// raced again on full (key, position) pairs.  Halves of unusable weights (0x7ff00000) tie with
// each other, which only matters when they reach the kept entries.

constexpr uint32_t kNoHalf = 0xffffffffu;  // upper half of kNoKey

// Lane l < k holds the l-th smallest half and its position; lanes from k on hold leftovers that
// nothing reads.
struct HalfRace {
  uint32_t key;
  uint32_t pos;
  uint32_t last;  // entry of lane k-1 (the bar)
  uint32_t tie;   // the latest bar value that a dropped candidate shared (kNoHalf: none)
};

__device__ __forceinline__ void half_race_reset(HalfRace& r) {
  r.key = r.last = r.tie = kNoHalf;
  r.pos = kNoPos;
}

template <int G>
__device__ __forceinline__ uint32_t group_read(uint32_t v, int src) {
  if constexpr (G == kWave) return lane_read(v, src);
  else return __shfl(v, src, G);
}

template <int G>
__device__ __forceinline__ void half_race_seed(HalfRace& r, const Group<G>& g, uint32_t h, uint32_t p, int k) {
  r.key = h;
  r.pos = p;
  group_sort<G, true>(r.key, r.pos, g.l);
  r.last = group_read<G>(r.key, k - 1);
  const uint32_t cut = group_read<G>(r.key, k < G ? k : G - 1);  // first entry that is dropped
  r.tie = (k < G && cut == r.last) ? cut : kNoHalf;
}

// G more candidates: halves h, positions p.
template <int G>
__device__ __forceinline__ void half_race_offer(HalfRace& r, const Group<G>& g, uint32_t h, uint32_t p, int k) {
  uint64_t hits = g.ballot(h < r.last);
  if (g.ballot(h == r.last)) r.tie = r.last;
  if constexpr (G == kWave) {
    while (hits) {
      const int b = __builtin_ctzll(hits);
      hits &= hits - 1;
      const uint32_t v = lane_read(h, b);
      if (v >= r.last) {  // the bar moved since the ballot
        if (v == r.last) r.tie = v;
        continue;
      }
      const uint32_t pk = lane_below(r.key);
      const uint32_t pp = lane_below(r.pos);
      if (v < r.key) {  // an entry above the newcomer moves up or makes room
        const bool shift = g.l > 0 && v < pk;
        r.key = shift ? pk : v;
        r.pos = shift ? pp : lane_read(p, b);
      }
      const uint32_t pushed_out = r.last;
      r.last = lane_read(r.key, k - 1);
      if (r.last == pushed_out) r.tie = pushed_out;
    }
  } else {
    while (__ballot(hits != 0)) {
      const bool has = hits != 0;
      const int b = has ? __builtin_ctzll(hits) : 0;
      hits &= hits - 1;
      const uint32_t v = __shfl(h, b, G);
      const uint32_t vp = __shfl(p, b, G);
      const uint32_t pk = lane_below(r.key);
      const uint32_t pp = lane_below(r.pos);
      const bool in = has && v < r.last;
      if (has && v == r.last) r.tie = v;
      if (in && v < r.key) {
        const bool shift = g.l > 0 && v < pk;
        r.key = shift ? pk : v;
        r.pos = shift ? pp : vp;
      }
      const uint32_t pushed_out = r.last;
      r.last = __shfl(r.key, k - 1, G);
      if (in && r.last == pushed_out) r.tie = pushed_out;
    }
  }
}

// Positions [0, end) of the group's row through the race on halves.
template <int G>
__device__ __forceinline__ void half_race_scan(HalfRace& r, const Group<G>& g, const TierView<float>& probs,
                                               int64_t start, uint64_t end, int k, uint64_t rng_seed,
                                               uint32_t rng_stream, int64_t row) {
  bool first = true;
  for (uint64_t sb = 0; __ballot(sb < end); sb += 4u * G) {
    uint64_t ck[4];
    stretch_keys<G>(g, probs, start, sb, end, rng_seed, rng_stream, row, ck);
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const uint64_t cb = sb + uint64_t(G) * c;
      if (!__ballot(cb < end)) break;
      const uint32_t h = uint32_t(ck[c] >> 32);
      const uint32_t p = uint32_t(cb) + uint32_t(g.l);
      if (first) {
        half_race_seed<G>(r, g, h, p, k);
        first = false;
      } else {
        half_race_offer<G>(r, g, h, p, k);
      }
    }
  }
}

// Whether the halves left the group's winners or their order open.
template <int G>
__device__ __forceinline__ bool half_race_open(const HalfRace& r, const Group<G>& g, int k) {
  const uint32_t below = lane_below(r.key);
  return r.tie == r.last || g.ballot(g.l > 0 && g.l < k && r.key == below) != 0;
}

// ---- with replacement ----

template <int G>
__device__ __forceinline__ float group_max(float v) {
#pragma unroll
  for (int d = G / 2; d > 0; d >>= 1) {
    const float o = __shfl_xor(v, d, G);
    if (o > v) v = o;
  }
  return v;
}

template <int G>
__device__ __forceinline__ uint64_t group_sum(uint64_t v) {
#pragma unroll
  for (int d = G / 2; d > 0; d >>= 1) v += __shfl_xor(v, d, G);
  return v;
}

template <int G>
__device__ __forceinline__ uint64_t group_inclusive_sum(uint64_t v, int l) {
#pragma unroll
  for (int d = 1; d < G; d <<= 1) {
    const uint64_t t = __shfl_up(v, d, G);
    if (l >= d) v += t;
  }
  return v;
}

// Largest weight of positions [lo, hi) of the group's row (0 when none is positive).
template <int G>
__device__ __forceinline__ float range_max(const Group<G>& g, const TierView<float>& probs, int64_t start,
                                           int64_t lo, int64_t hi) {
  float m = 0.0f;
  for (int64_t p = lo + g.l; p < hi; p += G) {
    const float w = probs.at(start + p);
    if (w > m) m = w;
  }
  return group_max<G>(m);
}

template <int G>
__device__ __forceinline__ uint64_t range_sum(const Group<G>& g, const TierView<float>& probs, int64_t start,
                                              int64_t lo, int64_t hi, const QuantumScale& qs) {
  uint64_t s = 0;
  for (int64_t p = lo + g.l; p < hi; p += G) s += weight_quantum(probs.at(start + p), qs);
  return group_sum<G>(s);
}

// Among the group's draws (r, one per lane where `wanted`), finds the position of each one that
// falls into the quanta of positions [lo, hi), which begin at the running sum `before`; a draw
// belongs to the first position whose inclusive sum exceeds it.  Returns the lanes it settled.
template <int G>
__device__ __forceinline__ uint64_t locate_draws(const Group<G>& g, const TierView<float>& probs, int64_t start,
                                                 int64_t lo, int64_t hi, const QuantumScale& qs, uint64_t before,
                                                 uint64_t r,
                                                 bool wanted, int64_t* pick) {
  uint64_t settled = 0;
  uint64_t pending = g.ballot(wanted && r >= before);
  for (int64_t cb = lo; __ballot(cb < hi && pending != 0); cb += G) {
    const int64_t p = cb + g.l;
    const uint64_t q = p < hi ? weight_quantum(probs.at(start + p), qs) : 0;
    const uint64_t incl = before + group_inclusive_sum<G>(q, g.l);
    const uint64_t after = __shfl(incl, G - 1, G);
    uint64_t here = pending & g.ballot(r < after);
    pending &= ~here;
    settled |= here;
    while (__ballot(here != 0)) {
      const bool has = here != 0;
      const int b = has ? __builtin_ctzll(here) : 0;
      here &= here - 1;
      const uint64_t rb = __shfl(r, b, G);
      const uint64_t above = g.ballot(incl > rb);
      if (has && g.l == b) *pick = cb + __builtin_ctzll(above);
    }
    before = after;
  }
  return settled;
}

// LDS of a block that works on long rows.
struct LongRowScratch {
  uint64_t key[kLongBlock];
  uint32_t half[kLongBlock];
  uint32_t pos[kLongBlock];
  uint64_t bars[kLongWaves];
  uint64_t sum[kLongWaves];
  float max[kLongWaves];
  uint32_t half_bars[kLongWaves];
  uint32_t ties[kLongWaves];
  uint32_t listed;  // entries of half[] / pos[]
  uint32_t open;    // the halves did not settle the row
};

// Without replacement, a row of up to long_row<G>() positions raced by one G-lane group (end = 0:
// nothing races): returns, in lane l < k of the group, the position of the l-th winner (kNoPos in
// a group without a row).  Groups whose halves left something open race again on full keys; the
// wave's other groups idle through that with empty candidates.
template <int G>
__device__ __forceinline__ uint32_t race_row(const Group<G>& g, const TierView<float>& probs, int64_t start,
                                             uint32_t end, int k, uint64_t rng_seed, uint32_t rng_stream,
                                             int64_t row) {
  HalfRace hr;
  half_race_reset(hr);
  half_race_scan<G>(hr, g, probs, start, end, k, rng_seed, rng_stream, row);
  const bool again = end > 0 && half_race_open<G>(hr, g, k);
  uint32_t pos = end > 0 ? hr.pos : kNoPos;
  if (__ballot(again)) {
    Race r;
    race_reset(r);
    race_scan<G>(r, g, probs, start, 0, again ? end : 0u, 4 * G, k, rng_seed, rng_stream, row);
    if (again) pos = r.pos;
  }
  return pos;
}

// Without replacement, a long row raced by a whole 1024-thread block on full keys: each wave
// races an interleaved share of the row, then the waves' winners are merged pairwise (wave w takes
// over the entries of wave w + step: 16 lists become one in four rounds; entries beyond the lowest
// published bar cannot be among the row's best).  On return lane l < k of wave 0 holds the l-th
// winner in r.pos.  Every thread of the block must call it.
__device__ __forceinline__ void race_long_row_full(Race& r, LongRowScratch& lds, const TierView<float>& probs,
                                                   int64_t start, uint32_t deg, int k, uint64_t rng_seed,
                                                   uint32_t rng_stream, int64_t row) {
  const Group<kWave> g;
  const int wave = threadIdx.x / kWave;
  if (threadIdx.x < kLongWaves) lds.bars[threadIdx.x] = kNoKey;
  __syncthreads();
  race_reset(r);
  race_scan<kWave>(r, g, probs, start, 256u * wave, deg, 256u * kLongWaves, k, rng_seed, rng_stream, row, lds.bars);
  const uint64_t bar = lowest_bar_after_sync(lds.bars, g.l);
  for (int step = 1; step < kLongWaves; step <<= 1) {
    lds.key[threadIdx.x] = r.key;
    lds.pos[threadIdx.x] = r.pos;
    __syncthreads();
    if ((wave & (2 * step - 1)) == 0) {
      const uint64_t ck = lds.key[(wave + step) * kWave + g.l];
      race_offer<kWave>(r, g, ck > bar ? kNoKey : ck, lds.pos[(wave + step) * kWave + g.l], k);
    }
    __syncthreads();  // the arrays are rewritten by the next round and by the block's next row
  }
}

__device__ __forceinline__ uint32_t lowest_half_bar(uint32_t* bars, int lane) {
  uint32_t v = __atomic_load_n(&bars[lane & (kLongWaves - 1)], __ATOMIC_RELAXED);
#pragma unroll
  for (int stride = 1; stride < kLongWaves; stride <<= 1) {
    const uint32_t o = lane_xor(v, stride);
    if (o < v) v = o;
  }
  return v;
}

// Without replacement, a long row raced by a whole 1024-thread block (every thread must call it):
// returns, in lane l < k of wave 0, the position of the l-th winner.  The race runs on key halves
// first.  Each wave races an interleaved share of the row and publishes its bar, which lets all
// of them drop candidates beyond the lowest bar unseen; the entries that survive the final lowest
// bar (between k and 16 k, usually close to k) are listed in LDS and raced by wave 0.  Whether the
// halves settled the row is judged as in a group's race, with every wave's record of ties at its
// bar taken into account: a dropped candidate can only share the final bar if it shared its own
// wave's bar when it was dropped.  An unsettled row is raced again on full keys.
__device__ __forceinline__ uint32_t race_long_row(LongRowScratch& lds, const TierView<float>& probs, int64_t start,
                                                  uint32_t deg, int k, uint64_t rng_seed, uint32_t rng_stream,
                                                  int64_t row) {
  const Group<kWave> g;
  const int wave = threadIdx.x / kWave;
  if (threadIdx.x < kLongWaves) lds.half_bars[threadIdx.x] = kNoHalf;
  if (threadIdx.x == 0) lds.listed = 0;
  __syncthreads();
  HalfRace r;
  half_race_reset(r);
  bool first = true;
  uint32_t published = kNoHalf;
  for (uint64_t sb = 256u * wave; __ballot(sb < deg); sb += 256u * kLongWaves) {
    uint64_t ck[4];
    stretch_keys<kWave>(g, probs, start, sb, deg, rng_seed, rng_stream, row, ck);
    const uint32_t bar = lowest_half_bar(lds.half_bars, g.l);
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const uint64_t cb = sb + uint64_t(kWave) * c;
      if (!__ballot(cb < deg)) break;
      const uint32_t h = uint32_t(ck[c] >> 32);
      const uint32_t p = uint32_t(cb) + uint32_t(g.l);
      if (first) {
        half_race_seed<kWave>(r, g, h, p, k);
        first = false;
      } else {
        half_race_offer<kWave>(r, g, h > bar ? kNoHalf : h, p, k);
      }
    }
    if (r.last < published) {
      published = r.last;
      if (g.l == 0) __atomic_store_n(&lds.half_bars[wave], published, __ATOMIC_RELAXED);
    }
  }
  if (g.l == 0) lds.ties[wave] = r.tie;
  __syncthreads();  // every wave has published its final bar
  const uint32_t bar = lowest_half_bar(lds.half_bars, g.l);
  {
    const bool keep = g.l < k && r.key <= bar;  // a wave that raced nothing holds kNoHalf only
    const uint64_t kept = __ballot(keep);
    uint32_t base = 0;
    if (g.l == 0 && kept) base = atomicAdd(&lds.listed, uint32_t(__builtin_popcountll(kept)));
    base = wave_uniform(base);
    if (keep) {
      const uint32_t at = base + uint32_t(__builtin_popcountll(kept & ((uint64_t(1) << g.l) - 1)));
      lds.half[at] = r.key;
      lds.pos[at] = r.pos;
    }
  }
  __syncthreads();
  if (wave == 0) {
    const uint32_t listed = lds.listed;
    half_race_reset(r);
    for (uint32_t cb = 0; cb < listed; cb += kWave) {
      const uint32_t at = cb + uint32_t(g.l);
      const uint32_t h = at < listed ? lds.half[at] : kNoHalf;
      const uint32_t p = at < listed ? lds.pos[at] : kNoPos;
      if (cb == 0) half_race_seed<kWave>(r, g, h, p, k);
      else half_race_offer<kWave>(r, g, h, p, k);
    }
    const bool dropped_at_bar = __ballot(g.l < kLongWaves && lds.ties[g.l & (kLongWaves - 1)] == r.last) != 0;
    const bool open = half_race_open<kWave>(r, g, k) || dropped_at_bar;
    if (g.l == 0) lds.open = open ? 1u : 0u;
  }
  __syncthreads();
  const bool again = lds.open != 0;
  __syncthreads();  // lds.open and the lists are rewritten by the block's next row
  uint32_t pos = wave == 0 ? r.pos : kNoPos;
  if (again) {
    Race full;
    race_long_row_full(full, lds, probs, start, deg, k, rng_seed, rng_stream, row);
    pos = wave == 0 ? full.pos : kNoPos;
  }
  return pos;
}

// With replacement, a row of up to long_row<G>() positions (deg = 0: nothing to draw) handled by
// one G-lane group: three passes (largest weight, sum of shares, locate), G draws at a time;
// emit(j, position) is called by the lane that owns draw j.  A row without a positive finite
// share keeps its last neighbour.
template <int G, typename Emit>
__device__ __forceinline__ void draw_row(const Group<G>& g, const TierView<float>& probs, int64_t start, int64_t deg,
                                         int64_t k, uint64_t rng_seed, uint32_t rng_stream, int64_t row, Emit emit) {
  const QuantumScale qs = quantum_scale(range_max<G>(g, probs, start, 0, deg));
  const uint64_t total = range_sum<G>(g, probs, start, 0, deg, qs);
  for (int64_t first = 0; __ballot(first < k); first += G) {
    const int64_t j = first + g.l;
    const bool active = deg > 0 && j < k;
    int64_t pick = deg - 1;
    uint64_t r = 0;
    if (active && total > 0) r = philox_bounded64(rng_seed, rng_stream, row, uint32_t(j), total);
    locate_draws<G>(g, probs, start, 0, deg, qs, 0, r, active && total > 0, &pick);
    if (active && pick < deg) emit(j, pick);
  }
}

// With replacement, a long row handled by a whole 1024-thread block: each wave owns a contiguous
// sixteenth of the row (a multiple of 64 positions); block-wide maximum, per-wave sums and their
// prefix go through LDS; every wave then settles the draws that fall into its own part and calls
// emit(j, position) for them.  Every thread of the block must call it.
template <typename Emit>
__device__ __forceinline__ void draw_long_row(LongRowScratch& lds, const TierView<float>& probs, int64_t start,
                                              int64_t deg, int64_t k, uint64_t rng_seed, uint32_t rng_stream,
                                              int64_t row, Emit emit) {
  const Group<kWave> g;
  const int wave = threadIdx.x / kWave;
  const int64_t part = ((deg + kLongWaves - 1) / kLongWaves + kWave - 1) / kWave * kWave;
  const int64_t lo = part * wave < deg ? part * wave : deg;
  const int64_t hi = lo + part < deg ? lo + part : deg;
  const float m = range_max<kWave>(g, probs, start, lo, hi);
  if (g.l == 0) lds.max[wave] = m;
  __syncthreads();
  float wmax = 0.0f;
  for (int w = 0; w < kLongWaves; ++w) wmax = lds.max[w] > wmax ? lds.max[w] : wmax;
  const QuantumScale qs = quantum_scale(wmax);
  const uint64_t mine = range_sum<kWave>(g, probs, start, lo, hi, qs);
  if (g.l == 0) lds.sum[wave] = mine;
  __syncthreads();
  uint64_t before = 0, total = 0;
  for (int w = 0; w < kLongWaves; ++w) {
    if (w < wave) before += lds.sum[w];
    total += lds.sum[w];
  }
  for (int64_t first = 0; first < k; first += kWave) {
    const int64_t j = first + g.l;
    const bool active = j < k;
    if (total > 0) {
      uint64_t r = 0;
      int64_t pick = 0;
      if (active) r = philox_bounded64(rng_seed, rng_stream, row, uint32_t(j), total);
      const uint64_t settled = locate_draws<kWave>(g, probs, start, lo, hi, qs, before, r,
                                                   active && r < before + mine, &pick);
      if (((settled >> g.l) & 1) && pick < deg) emit(j, pick);
    } else if (wave == 0 && active) {
      emit(j, deg - 1);
    }
  }
  __syncthreads();  // the arrays are reused by the block's next row
}

}  // namespace dgs
#endif
