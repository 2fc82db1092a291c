// Row-wise weighted neighbour sampling: a float32 weight per edge, stored like `indices`.
//
// The count pass is the uniform sampler's (same pick counts).  The fill hands every seed row to a
// group of G lanes (G = 16, 32 or 64, so a wave64 serves up to four rows; chosen on the host from
// num_picks); rows of more than 32 G neighbours are queued and then split over the 16 waves of a
// 1024-thread block.
//   without replacement: every position races with the key E / w (E a unit exponential variate
//     from the row's Philox stream); a group keeps the num_picks smallest (key, position) pairs
//     in order, lane l holding the l-th;
//   with replacement: weights become integer shares floor(w * 2^(32-E)), 2^E the power of two
//     above the row's largest weight; their sums are exact in any order, and draws in [0, sum)
//     are located against the running inclusive sum.
// Both rules are evaluated from exactly rounded operations only (see weights.h), so the picks
// equal the CPU oracle's bit for bit whatever the launch shape.  Loops that contain cross-lane
// operations run a wave-uniform number of times: a group that has run out of work keeps
// executing with empty candidates.
#include <cstdlib>

#include "common.h"
#include "sample_workspace.h"
#include "weights.h"

namespace dgs {
namespace {

constexpr int kLongBlock = 1024;
constexpr int kLongWaves = kLongBlock / kWave;
constexpr int kMaxLongGrid = 512;  // two 1024-thread blocks fit a CU: one round over 256 CUs
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
template <int G, bool kByKeyOnly>
__device__ __forceinline__ void group_sort(uint64_t& key, uint32_t& pos, int l) {
#pragma unroll
  for (int size = 2; size <= G; size <<= 1) {
#pragma unroll
    for (int stride = size >> 1; stride > 0; stride >>= 1) {
      const uint64_t ok = lane_xor(key, stride);
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

// Runs positions [begin, end) of the group's row, in steps of `stride`, through its race.  begin
// and stride are multiples of 4 G: one Philox block per lane covers 4 G positions (four words
// each), and the word of position sb + G c + l sits in lane (G / 4) c + l / 4 of the group.
// `bars` (block-per-row kernel only) is the block's table of published last keys.
template <int G>
__device__ __forceinline__ void race_scan(Race& r, const Group<G>& g, const TierView<float>& probs, int64_t start,
                                          uint64_t begin, uint64_t end, uint64_t stride, int k, uint64_t rng_seed,
                                          uint32_t rng_stream, int64_t row, uint64_t* bars = nullptr) {
  bool first = true;
  uint64_t published = kNoKey;
  for (uint64_t sb = begin; __ballot(sb < end); sb += stride) {
    // the four steps of this stretch are independent until they meet the race: their loads are
    // issued together and their key arithmetic (long dependent float64 chains) interleaves
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
    uint64_t ck[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int src = (G / 4) * c + (g.l >> 2);
      const uint32_t a0 = __shfl(w.w[0], src, G), a1 = __shfl(w.w[1], src, G);
      const uint32_t a2 = __shfl(w.w[2], src, G), a3 = __shfl(w.w[3], src, G);
      const uint32_t x = (g.l & 2) ? ((g.l & 1) ? a3 : a2) : ((g.l & 1) ? a1 : a0);
      const uint64_t p = sb + uint64_t(G) * c + uint32_t(g.l);
      ck[c] = p < end ? race_key(x, wt[c], uint32_t(p)) : kNoKey;
    }
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

struct RowArgs {
  const int64_t* row_start;
  const uint32_t* row_deg;
  const int64_t* row_off;
  const int64_t* tile_off;
  int64_t* long_rows;
  int64_t* long_count;
};

__device__ __forceinline__ void queue_long_row(const RowArgs& a, int64_t i) {
  a.long_rows[atomicAdd(reinterpret_cast<unsigned long long*>(a.long_count), 1ull)] = i;
}

__global__ void clear_long_count_kernel(int64_t* long_count) { *long_count = 0; }

// Without replacement, one G-lane group per row; rows above long_row<G>() are queued.
template <typename IdT, int G>
__global__ __launch_bounds__(kTile) void fill_weighted_kernel(const IdT* __restrict__ seeds, int64_t n_seeds,
                                                              RowArgs a, TierView<IdT> indices,
                                                              TierView<float> probs, int k, uint64_t rng_seed,
                                                              uint32_t rng_stream, IdT* __restrict__ out_rows,
                                                              IdT* __restrict__ out_cols) {
  const Group<G> g;
  const int64_t i = (int64_t(blockIdx.x) * kTile + threadIdx.x) / G;
  int64_t start = 0, off = 0, row = 0;
  uint32_t end = 0;  // positions that race: 0 for rows that are copied, queued or absent
  if (i < n_seeds) {
    const uint32_t deg = a.row_deg[i];
    if (deg > long_row<G>()) {
      if (g.l == 0) queue_long_row(a, i);
    } else {
      start = a.row_start[i];
      off = a.tile_off[i / kTile] + a.row_off[i];
      row = int64_t(seeds[i]);
      if (deg <= uint32_t(k)) {
        if (uint32_t(g.l) < deg) {
          out_rows[off + g.l] = IdT(row);
          out_cols[off + g.l] = indices.at(start + g.l);
        }
      } else {
        end = deg;
      }
    }
  }
  Race r;
  race_reset(r);
  race_scan<G>(r, g, probs, start, 0, end, 4 * G, k, rng_seed, rng_stream, row);
  if (end > 0 && g.l < k && r.pos < end) {  // a row that races has more than k positions: every entry is filled
    out_rows[off + g.l] = IdT(row);
    out_cols[off + g.l] = indices.at(start + r.pos);
  }
}

// Without replacement, queued long rows: each wave races an interleaved share of the row, then
// the waves' winners are merged pairwise.
template <typename IdT>
__global__ __launch_bounds__(kLongBlock) void fill_weighted_long_kernel(const IdT* __restrict__ seeds, RowArgs a,
                                                                        TierView<IdT> indices,
                                                                        TierView<float> probs, int k,
                                                                        uint64_t rng_seed, uint32_t rng_stream,
                                                                        IdT* __restrict__ out_rows,
                                                                        IdT* __restrict__ out_cols) {
  __shared__ uint64_t lds_key[kLongBlock];
  __shared__ uint32_t lds_pos[kLongBlock];
  __shared__ uint64_t bars[kLongWaves];
  const Group<kWave> g;
  const int wave = threadIdx.x / kWave;
  const int64_t n_long = *a.long_count;
  for (int64_t t = blockIdx.x; t < n_long; t += gridDim.x) {
    const int64_t i = a.long_rows[t];
    const int64_t start = a.row_start[i];
    const int64_t off = a.tile_off[i / kTile] + a.row_off[i];
    const int64_t row = int64_t(seeds[i]);
    const uint32_t deg = a.row_deg[i];
    if (threadIdx.x < kLongWaves) bars[threadIdx.x] = kNoKey;
    __syncthreads();
    Race r;
    race_reset(r);
    race_scan<kWave>(r, g, probs, start, 256u * wave, deg, 256u * kLongWaves, k, rng_seed, rng_stream, row, bars);
    // pairwise rounds: wave w takes over the entries of wave w + step, 16 lists become one in four
    // rounds; entries beyond the lowest published bar cannot be among the row's best
    const uint64_t bar = lowest_bar_after_sync(bars, g.l);
    for (int step = 1; step < kLongWaves; step <<= 1) {
      lds_key[threadIdx.x] = r.key;
      lds_pos[threadIdx.x] = r.pos;
      __syncthreads();
      if ((wave & (2 * step - 1)) == 0) {
        const uint64_t ck = lds_key[(wave + step) * kWave + g.l];
        race_offer<kWave>(r, g, ck > bar ? kNoKey : ck, lds_pos[(wave + step) * kWave + g.l], k);
      }
      __syncthreads();  // the arrays are rewritten by the next round and by the block's next row
    }
    if (wave == 0 && g.l < k && r.pos < deg) {  // deg > k: every entry is filled
      out_rows[off + g.l] = IdT(row);
      out_cols[off + g.l] = indices.at(start + r.pos);
    }
  }
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

template <typename IdT, int G>
__global__ __launch_bounds__(kTile) void fill_weighted_replace_kernel(const IdT* __restrict__ seeds,
                                                                      int64_t n_seeds, RowArgs a,
                                                                      TierView<IdT> indices, TierView<float> probs,
                                                                      int64_t k, uint64_t rng_seed,
                                                                      uint32_t rng_stream,
                                                                      IdT* __restrict__ out_rows,
                                                                      IdT* __restrict__ out_cols) {
  const Group<G> g;
  const int64_t i = (int64_t(blockIdx.x) * kTile + threadIdx.x) / G;
  int64_t start = 0, off = 0, row = 0, deg = 0;  // deg stays 0 for rows that are empty, queued or absent
  if (i < n_seeds) {
    const uint32_t d = a.row_deg[i];
    if (d > long_row<G>()) {
      if (g.l == 0) queue_long_row(a, i);
    } else if (d > 0) {
      start = a.row_start[i];
      off = a.tile_off[i / kTile] + a.row_off[i];
      row = int64_t(seeds[i]);
      deg = d;
    }
  }
  const QuantumScale qs = quantum_scale(range_max<G>(g, probs, start, 0, deg));
  const uint64_t total = range_sum<G>(g, probs, start, 0, deg, qs);
  for (int64_t first = 0; first < k; first += G) {
    const int64_t j = first + g.l;
    const bool active = deg > 0 && j < k;
    int64_t pick = deg - 1;  // a row without a positive finite share keeps its last neighbour
    uint64_t r = 0;
    if (active && total > 0) r = philox_bounded64(rng_seed, rng_stream, row, uint32_t(j), total);
    locate_draws<G>(g, probs, start, 0, deg, qs, 0, r, active && total > 0, &pick);
    if (active && pick < deg) {
      out_rows[off + j] = IdT(row);
      out_cols[off + j] = indices.at(start + pick);
    }
  }
}

// Queued long rows: each wave owns a contiguous sixteenth of the row (a multiple of 64 positions);
// block-wide maximum, per-wave sums and their prefix go through LDS; every wave then settles the
// draws that fall into its own part.
template <typename IdT>
__global__ __launch_bounds__(kLongBlock) void fill_weighted_replace_long_kernel(
    const IdT* __restrict__ seeds, RowArgs a, TierView<IdT> indices, TierView<float> probs, int64_t k,
    uint64_t rng_seed, uint32_t rng_stream, IdT* __restrict__ out_rows, IdT* __restrict__ out_cols) {
  __shared__ float lds_max[kLongWaves];
  __shared__ uint64_t lds_sum[kLongWaves];
  const Group<kWave> g;
  const int wave = threadIdx.x / kWave;
  const int64_t n_long = *a.long_count;
  for (int64_t t = blockIdx.x; t < n_long; t += gridDim.x) {
    const int64_t i = a.long_rows[t];
    const int64_t start = a.row_start[i];
    const int64_t off = a.tile_off[i / kTile] + a.row_off[i];
    const int64_t row = int64_t(seeds[i]);
    const int64_t deg = int64_t(a.row_deg[i]);
    const int64_t part = ((deg + kLongWaves - 1) / kLongWaves + kWave - 1) / kWave * kWave;
    const int64_t lo = part * wave < deg ? part * wave : deg;
    const int64_t hi = lo + part < deg ? lo + part : deg;
    const float m = range_max<kWave>(g, probs, start, lo, hi);
    if (g.l == 0) lds_max[wave] = m;
    __syncthreads();
    float wmax = 0.0f;
    for (int w = 0; w < kLongWaves; ++w) wmax = lds_max[w] > wmax ? lds_max[w] : wmax;
    const QuantumScale qs = quantum_scale(wmax);
    const uint64_t mine = range_sum<kWave>(g, probs, start, lo, hi, qs);
    if (g.l == 0) lds_sum[wave] = mine;
    __syncthreads();
    uint64_t before = 0, total = 0;
    for (int w = 0; w < kLongWaves; ++w) {
      if (w < wave) before += lds_sum[w];
      total += lds_sum[w];
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
        if (((settled >> g.l) & 1) && pick < deg) {
          out_rows[off + j] = IdT(row);
          out_cols[off + j] = indices.at(start + pick);
        }
      } else if (wave == 0 && active) {
        out_rows[off + j] = IdT(row);
        out_cols[off + j] = indices.at(start + deg - 1);
      }
    }
    __syncthreads();  // the arrays are reused by the block's next row
  }
}

template <typename IdT, int G>
void launch_groups(const IdT* seeds, int64_t n_seeds, const RowArgs& a, const TierView<IdT>& indices,
                   const TierView<float>& probs, int64_t k, bool replace, uint64_t rng_seed, uint32_t rng_stream,
                   IdT* out_rows, IdT* out_cols, hipStream_t st) {
  const uint32_t blocks = uint32_t((n_seeds * G + kTile - 1) / kTile);
  if (replace)
    hipLaunchKernelGGL((fill_weighted_replace_kernel<IdT, G>), dim3(blocks), dim3(kTile), 0, st, seeds, n_seeds, a,
                       indices, probs, k, rng_seed, rng_stream, out_rows, out_cols);
  else
    hipLaunchKernelGGL((fill_weighted_kernel<IdT, G>), dim3(blocks), dim3(kTile), 0, st, seeds, n_seeds, a, indices,
                       probs, int(k), rng_seed, rng_stream, out_rows, out_cols);
}

template <typename IdT>
dgs_status run_fill_weighted(const void* seeds_v, int64_t n_seeds, const dgs_view& indices_v, const dgs_view& probs_v,
                             int64_t k, bool replace, uint64_t rng_seed, uint32_t rng_stream,
                             const SampleWorkspace& w, void* out_rows_v, void* out_cols_v, hipStream_t st) {
  if (n_seeds == 0 || k <= 0) return DGS_OK;
  const IdT* seeds = static_cast<const IdT*>(seeds_v);
  IdT* out_rows = static_cast<IdT*>(out_rows_v);
  IdT* out_cols = static_cast<IdT*>(out_cols_v);
  const TierView<IdT> indices(indices_v);
  const TierView<float> probs(probs_v);
  const RowArgs a{w.row_start, w.row_deg, w.row_off, w.tile_off, w.long_rows, w.long_count};
  const uint32_t long_blocks = uint32_t(n_seeds < kMaxLongGrid ? n_seeds : kMaxLongGrid);
  hipLaunchKernelGGL(clear_long_count_kernel, dim3(1), dim3(1), 0, st, w.long_count);
  DGS_LAUNCH_CHECK();
  // Without replacement a wider group seeds its race from more candidates at once, which pays
  // as soon as more than a handful of entries are kept.
  int group = replace ? (k <= 16 ? 16 : (k <= 32 ? 32 : 64)) : (k <= 4 ? 16 : 64);
  if (const char* forced = std::getenv("DGS_WEIGHTED_GROUP")) {  // test hook: 16, 32 or 64
    const int f = std::atoi(forced);
    if ((f == 16 || f == 32 || f == 64) && (replace || k <= f)) group = f;
  }
  if (group == 16)
    launch_groups<IdT, 16>(seeds, n_seeds, a, indices, probs, k, replace, rng_seed, rng_stream, out_rows, out_cols, st);
  else if (group == 32)
    launch_groups<IdT, 32>(seeds, n_seeds, a, indices, probs, k, replace, rng_seed, rng_stream, out_rows, out_cols, st);
  else
    launch_groups<IdT, 64>(seeds, n_seeds, a, indices, probs, k, replace, rng_seed, rng_stream, out_rows, out_cols, st);
  DGS_LAUNCH_CHECK();
  if (replace)
    hipLaunchKernelGGL((fill_weighted_replace_long_kernel<IdT>), dim3(long_blocks), dim3(kLongBlock), 0, st, seeds, a,
                       indices, probs, k, rng_seed, rng_stream, out_rows, out_cols);
  else
    hipLaunchKernelGGL((fill_weighted_long_kernel<IdT>), dim3(long_blocks), dim3(kLongBlock), 0, st, seeds, a,
                       indices, probs, int(k), rng_seed, rng_stream, out_rows, out_cols);
  DGS_LAUNCH_CHECK();
  return DGS_OK;
}

}  // namespace
}  // namespace dgs

DGS_API dgs_status dgs_sample_fill_weighted(const void* seeds, int32_t id_bytes, int64_t n_seeds,
                                            dgs_view indices, dgs_view probs, int64_t num_picks, int32_t replace,
                                            uint64_t rng_seed, uint32_t rng_stream, void* out_rows,
                                            void* out_cols, void* workspace, size_t workspace_bytes,
                                            void* stream) {
  using namespace dgs;
  dgs_status s = check_sample_args("sample_fill_weighted", seeds, id_bytes, n_seeds, num_picks, workspace,
                                   workspace_bytes);
  if (s != DGS_OK) return s;
  DGS_REQUIRE(indices.elem_bytes == id_bytes, DGS_ERR_INVALID,
              "sample_fill_weighted: indices width %d differs from the seed width %d", indices.elem_bytes, id_bytes);
  DGS_REQUIRE(probs.elem_bytes == 4, DGS_ERR_INVALID, "sample_fill_weighted: weights must be float32 (width %d)",
              probs.elem_bytes);
  DGS_REQUIRE(probs.total == indices.total, DGS_ERR_INVALID,
              "sample_fill_weighted: %lld weights for %lld edges", (long long)probs.total, (long long)indices.total);
  DGS_REQUIRE(replace != 0 || num_picks <= kMaxWeightedPicks, DGS_ERR_UNSUPPORTED,
              "sample_fill_weighted: num_picks %lld above %d without replacement", (long long)num_picks,
              kMaxWeightedPicks);
  DGS_REQUIRE(num_picks < (int64_t(1) << 30), DGS_ERR_UNSUPPORTED, "sample_fill_weighted: num_picks %lld too large",
              (long long)num_picks);
  DGS_REQUIRE(n_seeds == 0 || num_picks == 0 || (out_rows != nullptr && out_cols != nullptr), DGS_ERR_INVALID,
              "sample_fill_weighted: null output");
  hipStream_t st = static_cast<hipStream_t>(stream);
  SampleWorkspace w;
  sample_workspace_layout(n_seeds, workspace, &w);
  const bool rep = replace != 0;
  return id_bytes == 8 ? run_fill_weighted<int64_t>(seeds, n_seeds, indices, probs, num_picks, rep, rng_seed,
                                                    rng_stream, w, out_rows, out_cols, st)
                       : run_fill_weighted<int32_t>(seeds, n_seeds, indices, probs, num_picks, rep, rng_seed,
                                                    rng_stream, w, out_rows, out_cols, st);
}

DGS_API dgs_status dgs_sample_neighbors_weighted(const void* seeds, int32_t id_bytes, int64_t n_seeds,
                                                 dgs_view indptr, dgs_view indices, dgs_view probs,
                                                 int64_t num_picks, int32_t replace, uint64_t rng_seed,
                                                 uint32_t rng_stream, void* out_rows, void* out_cols,
                                                 int64_t* nnz_dev, void* workspace, size_t workspace_bytes,
                                                 void* stream) {
  DGS_REQUIRE(replace != 0 || num_picks <= dgs::kMaxWeightedPicks, DGS_ERR_UNSUPPORTED,
              "sample_neighbors_weighted: num_picks %lld above %d without replacement", (long long)num_picks,
              dgs::kMaxWeightedPicks);
  dgs_status s = dgs_sample_count(seeds, id_bytes, n_seeds, indptr, num_picks, replace, nnz_dev, workspace,
                                  workspace_bytes, stream);
  if (s != DGS_OK) return s;
  return dgs_sample_fill_weighted(seeds, id_bytes, n_seeds, indices, probs, num_picks, replace, rng_seed,
                                  rng_stream, out_rows, out_cols, workspace, workspace_bytes, stream);
}
