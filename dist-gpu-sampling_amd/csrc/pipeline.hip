// Multi-hop sampling + relabel as one stream of kernels with no host round trip and no
// synchronisation between blocks inside a kernel.
//
// The per-hop operators (sample.hip, unique.hip) each read a length back to the host so
// that they can return exactly-sized arrays.  Here every buffer has its worst-case size
// (hop h has at most S_h = S_{h-1} (1 + k_{h-1}) seeds), lengths stay in device memory,
// grids are sized for the worst case and surplus blocks retire at once.
//
// What makes the chain short and cheap:
//   * ranks depend on the ORDER of mapping positions only, so every pick gets the padded
//     position P_h + i*k + l (hop h, row i, pick l; P_h is a host-side constant): no
//     count/scan has to run before the picks are inserted, and positions are unique over
//     the whole call;
//   * a hop's frontier is the next hop's seed list, so ONE table serves all hops, holding
//     for every id the smallest position at which it was seen; seeds are never
//     re-inserted and the frontier is a single array that grows hop by hop;
//   * the table is touched once per pick: the atomicMin that inserts a position also
//     tells whether it is (so far) the smallest of its id and which position it displaced;
//     the displaced one is marked lost.  "First occurrence" is then decided from two
//     streamed arrays, without a second random read of the table.  Random 8-byte
//     accesses are what bounds these kernels (on MI355X: loads 71 G/s, atomics 26.7 G/s, every
//     device-scope atomic being executed at the memory side), and a hop costs two of them
//     per pick: the indices read and the table atomic.
//
// A large last hop of uniform picks does without the table altogether (see Buckets below): its
// fill records the picked ids, two launches group them by id and take the smallest position of
// every id in LDS, and flag / compact / relabel read the same slot words as on the table path.
//
// Critical path per hop (3 launches): fill -> flag -> compact.
//   fill     G lanes per seed row (G = 8..64): indptr pair, picks by the dgs-philox-1
//            contract, one insert_min per pick.
//   flag     finalises the first-occurrence bit (hop 0, whose seed list may repeat ids and
//            whose lost marks nobody cleared, asks the table instead) and counts per
//            1024-position tile.
//   compact  every block sums the tile counts before its own (the list is short), ranks
//            its first occurrences, appends them to the frontier and records the rank
//            at the position.
// Off the critical path, as surplus blocks of later launches: per-row pick counts are
// scanned per 256-row tile, and the packed edge list (src_local, dst_local) is written
// (rank of a pick = rank recorded at its id's smallest position).
//
// These kernels are chains of dependent memory accesses, so what a thread will need is requested
// as early as its address is known: a hop's length lives in device memory, but every buffer has
// its worst-case size, so a thread asks for its own elements (inside the buffer whatever the
// length turns out to be) together with the length and only then decides whether they count.
#include <type_traits>

#include "common.h"
#include "picks.h"
#include "race.h"
#include "table.h"

namespace dgs {
namespace {

constexpr int kBlock = 256;
constexpr int kRowTile = 256;                  // seed rows per offsets tile
constexpr int kPosItems = 4;
constexpr int kPosTile = kBlock * kPosItems;   // padded positions per flag/compact block
constexpr uint32_t kFirstBit = 0x80000000u;
constexpr uint32_t kInvalidSlot = 0xffffffffu; // padded position that holds no pick
// row_cnt markers of rows that make the call fail (bit (kBadRow - marker) of the hop's flag word)
constexpr uint32_t kBadRow = 0xffffffffu;      // degree >= 2^32, or offsets outside the edge array
constexpr uint32_t kBadSeed = 0xfffffffeu;     // the seed id is not a row of the graph
constexpr uint32_t kBadPick = 0xfffffffdu;     // a picked neighbour id is outside what the table holds
__device__ __forceinline__ bool is_bad_row(uint32_t row_cnt) { return row_cnt >= kBadPick; }
constexpr int kMaxPicks = 64;
constexpr int64_t kMaxPositions = int64_t(1) << 30;
constexpr int64_t kInlineTiles = 2048;         // above this a separate scan launch is used
// Launches are sized for the worst case, which can exceed the real work many times over (a hub
// graph deduplicates heavily).  Grids are capped and blocks stride over the virtual block index,
// so a mostly empty worst case costs a few loop trips instead of 10^5 empty blocks.
constexpr int64_t kGridCap = 16384;
// A launch that loops anyway is given fewer blocks than the cap: its worst case is far beyond the
// work, and blocks that find none still take a slot each from whatever else shares the GPU
// (measured with batches in flight, 1024 / 2048 / 4096 / 16384 blocks: 111 M-node graph 0.169-0.180 /
// 0.167-0.178 / 0.165-0.169 / 0.183-0.187 ms per step, R-MAT [50,50] 0.342-0.352 / 0.345-0.356 /
// 0.343-0.353 / 0.357-0.361; a batch alone is level or 2 % faster).
constexpr int64_t kLoopGrid = 4096;
inline int64_t grid_cap() {
  const int64_t forced = debug_option(DGS_DEBUG_SAMPLER_GRID_CAP);
  return forced > 0 ? forced : kGridCap;
}
inline uint32_t capped_grid(int64_t virtual_blocks) {
  const int64_t cap = grid_cap();
  if (virtual_blocks <= cap) return uint32_t(virtual_blocks < 1 ? 1 : virtual_blocks);
  return uint32_t(cap < kLoopGrid ? cap : kLoopGrid);  // (a forced cap below kLoopGrid is the grid itself)
}
inline bool is_capped(int64_t virtual_blocks) { return virtual_blocks > grid_cap(); }
// Kernels come in two flavours: STRIDE = false runs exactly one virtual block per block (the
// common, uncapped launch, with no loop in the instruction stream), STRIDE = true strides.
#define DGS_FOR_VIRTUAL_BLOCKS(vb, total)                                                       \
  for (int64_t vb = blockIdx.x; vb < (total); vb += STRIDE ? int64_t(gridDim.x) : (total))

struct Hop {
  const void* seeds;        // seed ids: caller's seeds (hop 0) or the frontier array
  // The three device scalars below are read without a test in front of them, so that the reads
  // leave together with a thread's first own reads: the pointers name readable words in every
  // hop, also where the value is not used (hop 0 takes its count from n_seeds_host and has no
  // previous hop).
  const int64_t* n_seeds;   // device scalar: seeds of this hop (used when n_seeds_host < 0)
  int64_t n_seeds_host;     // hop 0: the caller's count; later hops: -1
  int64_t* n_seeds_out;     // hop 0: where to publish n_seeds on the device
  const int64_t* prev_nnz;      // device scalar: edges of the previous hop
  const int64_t* prev_n_seeds;  // device scalar: seeds of the previous hop
  int64_t* n_unique;        // device scalar: frontier size after this hop
  int64_t* nnz;             // device scalar: edges of this hop
  int64_t* flags;           // device scalar: bit 0 degree, bit 1 seed id, bit 2 picked id of a bad row
  int64_t* host_sizes;      // optional pinned mirror of the whole sizes array (NULL: none)
  int32_t n_hops;           // layout of the mirror: [0..H] seeds, then H edge counts, then H flags
  int32_t pad0_;
  uint32_t* row_cnt;        // [s_max] picks of every row (kBadRow on error)
  uint32_t* row_off;        // [s_max] exclusive offset of the row inside its 256-row tile
  int* tile_sum;            // [row tiles]
  int* tile_flag;           // [row tiles]
  int64_t* tile_off;        // [row tiles] only when row tiles > kInlineTiles
  uint32_t* slot;           // [all positions] table slot of a position, bit 31 = first occurrence
  uint32_t* rank_at;        // [all positions] rank of the id first seen at that position
  uint8_t* lost;            // [all positions] non-zero: a smaller position of the same id exists
  int64_t* long_rows;       // weighted only: [s_max] rows handed to the block-per-row launch
  int64_t* long_count;      // weighted only: entries of long_rows
  int* pos_cnt;             // [position tiles of this hop] first occurrences per tile
  int64_t* pos_off;         // [position tiles] only when position tiles > kInlineTiles
  void* frontier;           // growing array of distinct ids
  void* src_local;          // out [nnz]
  void* dst_local;          // out [nnz]
  int64_t s_max;
  int64_t pos_base;         // first position of this hop (P_h)
  int64_t len_max;          // positions of this hop in the worst case: (hop 0: s_max) + s_max * k
  int32_t k;
  int32_t index;            // hop number
  uint32_t rng_stream;
  int32_t bucketed;         // non-zero: first occurrences come from the bucketed pass (see Buckets) ...
  int32_t pad1_;
  int64_t bucket_pos_cap;   // ... as long as the hop's padded positions (seeds * k) are no more than this: decided on the device
  int* bucket_overflow;     // set by the pass when a bucket held more ids than its LDS table takes (the call fails)
};

// (written without a conditional so that the read is not moved behind a test)
__device__ __forceinline__ int64_t seeds_of(const Hop& h) {
  const int64_t on_device = *h.n_seeds;
  const int64_t use_device = h.n_seeds_host >> 63;  // all ones when the count lives on the device
  return (on_device & use_device) | (h.n_seeds_host & ~use_device);
}
// Whether this hop finds its first occurrences by the bucketed pass.  Its worst case may be far
// beyond what the pass has room for (it grows with the product of the fanouts, the hop does not),
// so the host only says whether the hop is eligible and every kernel decides from the hop's real
// length, the same way.  (A bucketed hop is never hop 0: its positions are seeds * k.)
__device__ __forceinline__ bool bucketed_now(const Hop& h, int64_t s) {
  return h.bucketed != 0 && s * h.k <= h.bucket_pos_cap;
}
// the first seed_part positions of hop 0 are the caller's seeds themselves
__device__ __forceinline__ int64_t seed_part(const Hop& h, int64_t s) { return h.index == 0 ? s : 0; }
// rank of the first id this hop can add: later hops append behind their seeds
__device__ __forceinline__ int64_t first_rank(const Hop& h, int64_t s) { return h.index == 0 ? 0 : s; }
// the wave-local search for repeated draws of a row (fill_rows): entries per wave, and the longest
// row, in multiples of the fanout, that is searched (k draws from 4 k positions repeat one in nine)
constexpr int kFoldSlotBits = 7;
constexpr int kFoldSlots = 1 << kFoldSlotBits;
constexpr int kFoldMaxRowPerPick = 4;
constexpr int kRelabelItems = 4;  // padded picks per thread in relabel_tile
__host__ __device__ __forceinline__ int relabel_groups(int k) { return (k + kRelabelItems - 1) / kRelabelItems; }

// ---- a large last hop without memory-side atomics -------------------------------------------
// The atomicMin per pick is what a large hop costs most (every device-scope atomic executes at
// the memory side: 26.7 G/s, 31 us for the 832 k picks of a 1024 x [5,10,15] batch, and as much
// again while other batches share the GPU).  The last hop needs no table entry afterwards, so its
// first occurrences can be found without the table.  The hop's units -- the ids the frontier
// already holds (order value = rank) and the padded positions (order value = position, above
// every rank) -- are cut into tiles of 4096; a block puts its tile's units in bucket order
// (bucket = low bits of the id) and notes where every bucket's piece begins; then one block per
// bucket walks that bucket's pieces in all tiles and takes the smallest order value of every id in
// an LDS array indexed by the id's high bits.  A pick's slot word then says everything the later
// stages need: first occurrence (id | kFirstBit, as the fill left it), a repeat of an id the
// frontier held before this hop (its rank | kRankBit: final, no further lookup), or a repeat of
// a pick of this hop (that pick's position, whose rank the compaction records).  Same result as
// the table gives.
constexpr int kBucketTile = 4096;                    // units per tile
constexpr int kBucketTileItems = kBucketTile / kBlock;
constexpr int kMinBuckets = 512;
constexpr int kMaxBuckets = 2048;
constexpr int kBucketRange = 8192;                   // ids per bucket at most: 32 KB of LDS
constexpr int kMaxBucketTiles = 2048;                // tiles a bucket's block can walk (its LDS index of them)
constexpr int64_t kBucketedMaxNodes = int64_t(kMaxBuckets) * kBucketRange;
constexpr int64_t kBucketedMinPicks = int64_t(1) << 18;  // worst-case picks of the hop below which the table is cheaper
constexpr uint32_t kRankBit = 0x40000000u;
// Graphs with more nodes than kBucketedMaxNodes: buckets by a hash of the id, and a bucket's ids
// are told apart in an open-addressing table in LDS (ids + smallest order values, 128 KB of the
// CU's 160 KB) instead of an array indexed by the id's high bits.  A bucket may hold up to half as
// many units as the table has slots on average, which bounds the hop the pass accepts.
constexpr int kHashBlock = 1024;
constexpr int kHashSlots = 16384;
constexpr uint32_t kHashEmpty = 0xffffffffu;         // no id: ids are below 2^31
constexpr int kErrBucketOverflow = 8;                // hop flag bit: a bucket's ids did not fit its LDS table

struct Buckets {
  uint2* items;      // [tiles_max][kBucketTile] (id, order value), every tile's units in bucket order
  uint16_t* piece;   // [tiles_max][buckets + 1] where every bucket's piece begins inside its tile; [buckets] = the tile's units
  int32_t tiles_max; // tiles of units: front_tiles over the frontier array, the rest over the hop's padded positions
  int32_t front_tiles;
  int32_t log_buckets;
  uint32_t n_nodes;
  int32_t hashed;    // buckets by a hash of the id, ids told apart in an LDS hash table (any node count)
  int32_t hash_slots;  // slots of that table the kernels use: kHashSlots (a test hook makes it small, so that small inputs fill it)
};
// Buckets of the hop.  The direct form's count follows from the node count (host); the hashed
// form's follows from the hop's real size, on the device: as few buckets as keep a bucket's units
// within its table's slots on average (a bucket that is fuller than that goes over its units in
// parts), because every bucket costs its block a fixed chain of waits: a hop that fits 256 buckets
// is one block per CU, all at once.
constexpr int kMinHashLogBuckets = 8;
__device__ __forceinline__ int log_buckets_of(const Buckets& b, const Hop& h, int64_t s) {
  if (!b.hashed) return b.log_buckets;
  const int64_t units = s + s * h.k;  // at most: short rows leave padded positions empty, ids repeat
  int lb = kMinHashLogBuckets;
  while (lb < b.log_buckets && (int64_t(b.hash_slots) << lb) < units) ++lb;
  return lb;
}
__device__ __forceinline__ uint32_t bucket_of(const Buckets& b, int log_buckets, uint32_t id) {
  return (b.hashed ? hash_id(id) : id) & uint32_t((1 << log_buckets) - 1);
}

// rank of the id at position p, given p's slot word
template <typename TableT>
__device__ __forceinline__ uint32_t rank_of(const Hop& h, const TableT& table, int64_t p, uint32_t slot_word) {
  if (slot_word & kFirstBit) return h.rank_at[p];
  return h.rank_at[table.value(slot_word)];  // smallest position of the id: a first occurrence
}

template <int NT, typename T>
__device__ __forceinline__ T block_sum(T v, T* lds /* NT/64 */) {
#pragma unroll
  for (int d = kWave / 2; d > 0; d >>= 1) v += __shfl_xor(v, d, kWave);
  if ((threadIdx.x & (kWave - 1)) == 0) lds[threadIdx.x / kWave] = v;
  __syncthreads();
  T s = 0;
#pragma unroll
  for (int w = 0; w < NT / kWave; ++w) s += lds[w];
  __syncthreads();
  return s;
}

template <int NT>
__device__ __forceinline__ int block_or(int v, int* lds /* NT/64 */) {
#pragma unroll
  for (int d = kWave / 2; d > 0; d >>= 1) v |= __shfl_xor(v, d, kWave);
  if ((threadIdx.x & (kWave - 1)) == 0) lds[threadIdx.x / kWave] = v;
  __syncthreads();
  int s = 0;
#pragma unroll
  for (int w = 0; w < NT / kWave; ++w) s |= lds[w];
  __syncthreads();
  return s;
}

// ---- packed edge list of one hop (off the critical path) -----------------------------

// One block per 256-row tile: scan of the rows' pick counts.
__device__ __forceinline__ void offsets_tile(const Hop& h, int tile) {
  __shared__ int lds[kBlock / kWave];
  __shared__ int bad;
  if (threadIdx.x == 0) bad = 0;
  __syncthreads();
  const int64_t s = seeds_of(h);
  const int64_t i = int64_t(tile) * kRowTile + threadIdx.x;
  const uint32_t rc = i < h.s_max ? h.row_cnt[i] : 0u;  // requested together with s
  int c = 0;
  if (i < s) {
    if (is_bad_row(rc)) atomicOr(&bad, 1 << (kBadRow - rc)); else c = int(rc);
  }
  int total;
  const int ex = block_exclusive_scan<kBlock, int>(c, &total, lds);
  if (i < s) h.row_off[i] = uint32_t(ex);
  if (threadIdx.x == 0) {
    h.tile_sum[tile] = total;
    h.tile_flag[tile] = bad;
  }
}

// One block per (256-row tile, 4 x 256 padded picks): writes the rows' edges at their packed
// offsets; a thread handles four picks, 256 apart, so that a wave has four times the loads in
// flight and the launch a quarter of the waves.  src_local = rank of the picked id; dst_local = rank of the row's seed, which is
// the row number itself except in hop 0, whose seeds may repeat.
//
// EARLY (here and in the other tile functions): the launch is about as large as the hop really
// is, so a thread requests its own elements together with the hop's length and tests afterwards.
// Without it the launch was sized for a worst case that may exceed the hop many times over
// (and loops over its virtual blocks): the length is waited for first and blocks beyond it
// leave without having read anything.
template <typename IdT, typename TableT, bool EARLY>
__device__ __forceinline__ void relabel_tile(const Hop& h, const TableT& table, int64_t b) {
  __shared__ int64_t lds[kBlock / kWave];
  const int k = h.k;
  if (k == 0) return;
  const int groups = relabel_groups(k);
  const int64_t tile = b / groups;
  const int group = int(b - tile * groups);
  // the hop's length and this thread's own rows and picks, requested together
  const int64_t s = seeds_of(h);
  if (!EARLY && tile * kRowTile >= s) return;
  // (hop 0's seed part is the caller's count, a kernel argument: positions hang on no load)
  const int64_t p0 = h.pos_base + (h.index == 0 ? h.n_seeds_host : 0);
  int64_t i[kRelabelItems], p[kRelabelItems];
  int l[kRelabelItems];
  bool mine[kRelabelItems];
  uint32_t rc[kRelabelItems], off[kRelabelItems], word[kRelabelItems], seed_word[kRelabelItems];
#pragma unroll
  for (int j = 0; j < kRelabelItems; ++j) {
    const int chunk = group * kRelabelItems + j;
    const int t = chunk * kBlock + threadIdx.x;  // padded pick inside the tile
    const int r = t / k;
    l[j] = t - r * k;
    i[j] = tile * kRowTile + r;
    p[j] = p0 + i[j] * k + l[j];
    mine[j] = chunk < k && i[j] < h.s_max;
    rc[j] = off[j] = word[j] = seed_word[j] = 0;
    if (mine[j]) {
      rc[j] = h.row_cnt[i[j]];
      off[j] = h.row_off[i[j]];
      word[j] = h.slot[p[j]];
      if (h.index == 0) seed_word[j] = h.slot[h.pos_base + i[j]];
    }
  }
  int64_t part = 0;
  if (h.tile_off) {
    if (threadIdx.x == 0) part = h.tile_off[tile];
  } else {
    for (int64_t j = threadIdx.x; j < tile; j += kBlock) part += h.tile_sum[j];
  }
  if (tile * kRowTile >= s) return;  // whole blocks leave together
  // Rank of a pick = rank recorded at the smallest position of its id: its own position when it
  // is a first occurrence, else the position the table holds.  Two rounds of loads, each issued
  // for all of the thread's picks before any is used, and both before the block adds up its
  // prefix (whose barrier nothing here has to wait behind).
  const bool bucketed = bucketed_now(h, s);
  bool live[kRelabelItems];
  bool known[kRelabelItems];  // bucketed hop: the word of a repeat may be the rank itself
  uint32_t at[kRelabelItems];
#pragma unroll
  for (int j = 0; j < kRelabelItems; ++j) {
    live[j] = mine[j] && i[j] < s && !is_bad_row(rc[j]) && uint32_t(l[j]) < rc[j];
    at[j] = uint32_t(p[j]);
    known[j] = false;
    if (live[j] && !(word[j] & kFirstBit)) {
      if (bucketed) {
        known[j] = (word[j] & kRankBit) != 0;
        at[j] = word[j] & (kRankBit - 1);
      } else {
        at[j] = table.value(word[j]);
      }
    }
  }
  uint32_t rank[kRelabelItems];
#pragma unroll
  for (int j = 0; j < kRelabelItems; ++j) rank[j] = !live[j] ? 0u : known[j] ? at[j] : h.rank_at[at[j]];
  const int64_t prefix = block_sum<kBlock, int64_t>(part, lds);
#pragma unroll
  for (int j = 0; j < kRelabelItems; ++j) {
    if (!live[j]) continue;
    const int64_t o = prefix + off[j] + l[j];
    static_cast<IdT*>(h.src_local)[o] = IdT(rank[j]);
    static_cast<IdT*>(h.dst_local)[o] =
        h.index == 0 ? IdT(rank_of(h, table, h.pos_base + i[j], seed_word[j])) : IdT(i[j]);
  }
}

inline int64_t relabel_blocks(int64_t s_max, int k) {
  return ((s_max + kRowTile - 1) / kRowTile) * relabel_groups(k);
}

// ---- critical path ------------------------------------------------------------------------

// Marks `displaced` (a position of this call) as no longer the smallest of its id.
__device__ __forceinline__ void mark_lost(const Hop& h, uint32_t displaced) {
  if (displaced != kNoPosition) h.lost[displaced] = 1;
}

// The slot word of padded position p, which holds a pick of neighbour id `col`: the id goes into
// the table (or, in a bucketed hop, into the word itself).  Returns false, and the word of an empty
// position, when the id is one the table cannot hold (the caller marks the row bad): the id is
// checked before it addresses anything.
template <typename IdT, typename TableT>
__device__ __forceinline__ bool place_pick(const Hop& h, const TableT& table, IdT col, int64_t p, bool look_first,
                                           bool bucketed, uint32_t* word) {
  *word = kInvalidSlot;
  if (!table.holds(col)) return false;
  if (bucketed) {
    *word = uint32_t(col) | kFirstBit;  // a first occurrence until the bucketed pass says otherwise; the table is left alone
    return true;
  }
  bool first;
  uint32_t displaced;
  uint32_t w = table.insert_min(col, uint32_t(p), &first, &displaced, look_first);
  if (h.index != 0) {
    if (first) w |= kFirstBit;  // provisional: cleared by flag() if the position gets lost
    mark_lost(h, displaced);
  }
  *word = w;
  return true;
}

// What becomes of padded position p: with a pick (edge `edge` of the graph) the picked id is placed
// and p's slot word recorded; without one the position is marked empty.
template <typename IdT, typename TableT>
__device__ __forceinline__ bool emit_pick(const Hop& h, const TableT& table, const TierView<IdT>& indices, int64_t p,
                                          bool have, int64_t edge, bool look_first, bool bucketed) {
  uint32_t word = kInvalidSlot;
  bool ok = true;
  if (have) ok = place_pick<IdT>(h, table, indices.at(edge), p, look_first, bucketed, &word);
  h.slot[p] = word;
  return ok;
}

// Ids that repeat a lot (hub sources) are cheaper to insert with a look at the entry first;
// the previous hop tells: if more than a fifth of its picks were not new ids, look first.
// (hop 0 has no history: look first only when it is big enough for contention to matter)
__device__ __forceinline__ bool look_before_insert(const Hop& h, int64_t s) {
  const int64_t picked = *h.prev_nnz;
  const int64_t fresh = s - *h.prev_n_seeds;  // ids the previous hop added to the frontier
  const bool first_hop = h.index == 0;
  const bool big = s * h.k >= (int64_t(1) << 17);
  const bool repeats = fresh * 5 < picked * 4;
  return bool((int(first_hop) & int(big)) | (int(!first_hop) & int(repeats)));
}

// One virtual block of the fill launch: 256 / G seed rows.
template <typename IdT, typename PtrT, typename TableT, int G, bool EARLY>
__device__ __forceinline__ void fill_rows(const Hop& h, int64_t vb, const TableT& table,
                                          const TierView<PtrT>& indptr, const TierView<IdT>& indices,
                                          bool replace, uint64_t rng_seed) {
  const int64_t gid = vb * kBlock + threadIdx.x;
  const int64_t i = gid / G;
  const int l = int(gid % G);
  // a launch sized far beyond the hop: blocks past its end wait for nothing but the length
  if (!EARLY && vb != 0 && vb * (kBlock / G) >= seeds_of(h)) return;
  // the wave's table for the search for repeated draws (below) is emptied here, where every lane
  // of the wave is still present
  __shared__ unsigned long long fold_lds[kBlock / kWave][kFoldSlots];
  if (replace) {
    unsigned long long* offers = fold_lds[threadIdx.x / kWave];
#pragma unroll
    for (int q = 0; q < kFoldSlots / kWave; ++q) offers[q * kWave + (threadIdx.x & (kWave - 1))] = ~0ull;
  }
  // the hop's length, what the previous hop found, and this group's seed id, requested together
  // (the seed list has room for s_max ids whatever the length turns out to be)
  const IdT seed = i < h.s_max ? static_cast<const IdT*>(h.seeds)[i] : IdT(0);
  const int64_t s = seeds_of(h);
  const bool look_first = look_before_insert(h, s);
  const bool bucketed = bucketed_now(h, s);
  const bool fold = replace && !bucketed;
  if (h.n_seeds_out && vb == 0 && threadIdx.x == 0) *h.n_seeds_out = s;
  if (i >= s) return;  // whole groups leave together
  const int group_lane0 = (threadIdx.x & (kWave - 1)) - l;
  const int64_t row = int64_t(seed);
  // this lane's random block hangs on the ids only: computed while the offsets are on their way
  const PhiloxWords words = philox_draw_words(rng_seed, h.rng_stream, row, uint32_t(l));
  // nothing is addressed by an id or an offset before it has been checked
  const bool seed_ok = row_in_range(indptr, row) && table.holds(seed);
  int64_t b = 0, deg64 = 0;
  if (seed_ok) {
    b = int64_t(indptr.at(row));
    deg64 = int64_t(indptr.at(row + 1)) - b;
  }
  const bool bad = deg64 < 0 || deg64 > 0xffffffffLL || b < 0 || b + deg64 > indices.n;
  const uint32_t deg = bad ? 0u : uint32_t(deg64);
  const int k = h.k;
  if (l == 0 && h.index == 0) {  // the caller's seeds open the mapping list; flag() decides their first bits
    bool first;
    uint32_t displaced;
    h.slot[h.pos_base + i] =
        seed_ok ? table.insert_min(seed, uint32_t(h.pos_base + i), &first, &displaced) : kInvalidSlot;
  }
  uint32_t pos;
  const bool have = pick_position<G>(deg, k, replace, l, group_lane0, words, &pos);
  const bool live = l < k && have;
  const int64_t p = h.pos_base + seed_part(h, s) + i * k + l;
  // Draws with replacement repeat positions: on a row shorter than k most slots do.  Only the
  // lowest slot of each position reads the edge array and goes to the table; a repeat can never be
  // its id's smallest position, so it takes its leader's id and slot word (without the first bit)
  // and touches nothing.  Repeats are found through a small table of the wave's own in LDS: every
  // slot of the row offers (position, lane) to the entry its position hashes to, the smallest
  // offer stays, and a slot that then reads its own position with a lower lane of its row has found
  // its leader.  Two positions that meet in one entry cost a missed repeat, never a wrong one.
  // Long rows (whose draws rarely repeat) skip the search.
  int leader = l;
  if (fold) {
    unsigned long long* offers = fold_lds[threadIdx.x / kWave];
    const int lane = threadIdx.x & (kWave - 1);
    const bool search = live && deg <= uint32_t(kFoldMaxRowPerPick * k);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const uint32_t entry = ((pos + uint32_t(group_lane0) * 0x9E3779B1u) * 0x85EBCA6Bu) >> (32 - kFoldSlotBits);
    if (search) atomicMin(&offers[entry], (static_cast<unsigned long long>(pos) << 8) | uint32_t(lane));
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    if (search) {
      const unsigned long long best = offers[entry];
      const int best_lane = int(best & 255u);
      if (uint32_t(best >> 8) == pos && best_lane < lane && best_lane >= group_lane0) leader = best_lane - group_lane0;
    }
  }
  uint32_t word = kInvalidSlot;
  bool pick_ok = true;
  if (live && leader == l) pick_ok = place_pick<IdT>(h, table, indices.at(b + pos), p, look_first, bucketed, &word);
  if (fold) {
    const uint32_t leader_word = __shfl(word, leader, G);
    const int leader_ok = __shfl(int(pick_ok), leader, G);
    if (live && leader != l) {
      word = leader_word == kInvalidSlot ? kInvalidSlot : (leader_word & ~kFirstBit);
      pick_ok = leader_ok != 0;
    }
  }
  if (l < k) h.slot[p] = word;
  constexpr uint64_t group_mask = G == 64 ? ~uint64_t(0) : ((uint64_t(1) << (G & 63)) - 1);
  const bool picks_ok = ((__ballot(!pick_ok) >> group_lane0) & group_mask) == 0;
  if (l == 0)
    h.row_cnt[i] = !seed_ok ? kBadSeed : bad ? kBadRow : !picks_ok ? kBadPick
                 : (replace ? (deg == 0 ? 0u : uint32_t(k)) : (deg < uint32_t(k) ? deg : uint32_t(k)));
}

// Virtual blocks [0, fill_blocks): seed rows of this hop; then relabel_count blocks writing the
// previous hop's edge list (off the critical path); then, in hop 0's launch, blocks clearing the
// lost marks of the later hops.
template <typename IdT, typename PtrT, typename TableT, int G, bool STRIDE>
__global__ __launch_bounds__(kBlock) void hop_fill_kernel(Hop h, Hop prev, int64_t fill_blocks,
                                                          int64_t relabel_count, uint4* clear_begin,
                                                          int64_t clear_n16, TableT table, TierView<PtrT> indptr,
                                                          TierView<IdT> indices, bool replace, uint64_t rng_seed) {
  const int64_t clear_blocks = (clear_n16 + kBlock - 1) / kBlock;
  const int64_t total = fill_blocks + relabel_count + clear_blocks;
  DGS_FOR_VIRTUAL_BLOCKS(vb, total) {
    if (vb < fill_blocks) {
      fill_rows<IdT, PtrT, TableT, G, !STRIDE>(h, vb, table, indptr, indices, replace, rng_seed);
    } else if (!STRIDE && vb < fill_blocks + relabel_count) {  // (a striding launch is given no such blocks)
      relabel_tile<IdT, TableT, !STRIDE>(prev, table, vb - fill_blocks);
    } else {
      const int64_t i = (vb - fill_blocks - relabel_count) * kBlock + threadIdx.x;
      if (i < clear_n16) clear_begin[i] = make_uint4(0u, 0u, 0u, 0u);
    }
  }
}

// ---- weighted picks (race.h): one wave per seed row, a block per row for long rows ----

constexpr int64_t kMaxLongGrid = 512;

// Lanes that one row's picks occupy when a wave writes them out: the wave races its rows one
// after the other (64 lanes on a row), parks every row's picks in that row's lanes and then
// inserts and records the picks of all its rows in one go, so that the instructions of that step
// are not spent on a mostly idle wave.
__host__ __device__ __forceinline__ int weighted_row_lanes(int64_t k) { return k <= 16 ? 16 : (k <= 32 ? 32 : kWave); }
inline int64_t weighted_rows_per_block(int64_t k) { return (kBlock / kWave) * (kWave / weighted_row_lanes(k)); }

// One virtual block of the weighted fill launch: four waves with 64 / weighted_row_lanes(k) seed
// rows each.  Rows above long_row<64>() positions are queued for hop_fill_weighted_long_kernel,
// which fills their positions; everything else about a row is what fill_rows does.
template <typename IdT, typename PtrT, typename TableT, bool REPLACE>
__device__ __forceinline__ void fill_rows_weighted(const Hop& h, int64_t vb, const TableT& table,
                                                   const TierView<PtrT>& indptr, const TierView<IdT>& indices,
                                                   const TierView<float>& probs, uint64_t rng_seed) {
  const Group<kWave> g;
  const int64_t s = seeds_of(h);
  const bool look_first = look_before_insert(h, s);
  if (h.n_seeds_out && vb == 0 && threadIdx.x == 0) *h.n_seeds_out = s;
  const int k = h.k;
  const int lanes = weighted_row_lanes(k);
  const int rows = kWave / lanes;
  const int64_t first = (vb * (kBlock / kWave) + int64_t(wave_uniform(uint32_t(threadIdx.x / kWave)))) * rows;
  if (first >= s) return;  // whole waves leave together
  // every lane looks up the row whose picks it will write out
  const int mine = g.l / lanes;  // that row among the wave's
  const int l = g.l - mine * lanes;
  const int64_t i = first + mine;
  int64_t b = 0;
  uint32_t deg = 0;
  bool bad = false;
  IdT seed = 0;
  bool seed_ok = true;
  if (i < s) {
    seed = static_cast<const IdT*>(h.seeds)[i];
    // nothing is addressed by an id or an offset before it has been checked
    seed_ok = row_in_range(indptr, int64_t(seed)) && table.holds(seed);
    int64_t deg64 = 0;
    if (seed_ok) {
      b = int64_t(indptr.at(int64_t(seed)));
      deg64 = int64_t(indptr.at(int64_t(seed) + 1)) - b;
    }
    bad = deg64 < 0 || deg64 > 0xffffffffLL || b < 0 || b + deg64 > indices.n;
    deg = bad ? 0u : uint32_t(deg64);
  }
  if (i < s && l == 0 && h.index == 0) {
    bool first_seen;
    uint32_t displaced;
    h.slot[h.pos_base + i] =
        seed_ok ? table.insert_min(seed, uint32_t(h.pos_base + i), &first_seen, &displaced) : kInvalidSlot;
  }
  // rows that are copied need no work; long rows are queued and written by the other launch
  const bool is_long = deg > long_row<kWave>() && (REPLACE || deg > uint32_t(k));
  if (is_long && l == 0) h.long_rows[atomicAdd(reinterpret_cast<unsigned long long*>(h.long_count), 1ull)] = i;
  uint32_t pick = uint32_t(l);  // what a copied row keeps: its positions in order
  for (int r = 0; r < rows; ++r) {
    // row r of the wave, in scalar registers
    const int src = r * lanes;
    const uint32_t rdeg = lane_read(deg, src);
    const bool rlong = rdeg > long_row<kWave>() && (REPLACE || rdeg > uint32_t(k));
    if (rdeg == 0 || rlong || (!REPLACE && rdeg <= uint32_t(k))) continue;
    const int64_t rrow = int64_t(lane_read(uint64_t(int64_t(seed)), src));
    const int64_t rb = int64_t(lane_read(uint64_t(b), src));
    uint32_t won = kNoPos;  // lane j: pick j of this row
    if (REPLACE) {  // at most 64 draws: draw j is found by lane j
      draw_row<kWave>(g, probs, rb, int64_t(rdeg), int64_t(k), rng_seed, h.rng_stream, rrow,
                      [&](int64_t, int64_t at) { won = uint32_t(at); });
    } else {
      won = race_row<kWave>(g, probs, rb, rdeg, k, rng_seed, h.rng_stream, rrow);
    }
    const uint32_t parked = __shfl(won, l, kWave);
    if (mine == r) pick = parked;
  }
  bool pick_ok = true;
  if (i < s && l < k && !is_long)
    pick_ok = emit_pick<IdT>(h, table, indices, h.pos_base + seed_part(h, s) + i * k + l, pick < deg, b + pick, look_first,
                             bucketed_now(h, s));
  const uint64_t row_mask = lanes == kWave ? ~uint64_t(0) : ((uint64_t(1) << lanes) - 1);
  const bool picks_ok = ((__ballot(!pick_ok) >> (mine * lanes)) & row_mask) == 0;
  if (i < s && l == 0)
    h.row_cnt[i] = !seed_ok ? kBadSeed : bad ? kBadRow : !picks_ok ? kBadPick
                 : (REPLACE ? (deg == 0 ? 0u : uint32_t(k)) : (deg < uint32_t(k) ? deg : uint32_t(k)));
}

// Same layout of virtual blocks as hop_fill_kernel (fill, previous hop's edge list, clearing).
template <typename IdT, typename PtrT, typename TableT, bool REPLACE>
__global__ __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu(5, 8))) void hop_fill_weighted_kernel(Hop h, Hop prev, int64_t fill_blocks,
                                                                   int64_t relabel_count, uint4* clear_begin,
                                                                   int64_t clear_n16, TableT table,
                                                                   TierView<PtrT> indptr, TierView<IdT> indices,
                                                                   TierView<float> probs, uint64_t rng_seed) {
  const int64_t clear_blocks = (clear_n16 + kBlock - 1) / kBlock;
  const int64_t total = fill_blocks + relabel_count + clear_blocks;
  for (int64_t vb = blockIdx.x; vb < total; vb += gridDim.x) {
    if (vb < fill_blocks) {
      fill_rows_weighted<IdT, PtrT, TableT, REPLACE>(h, vb, table, indptr, indices, probs, rng_seed);
    } else if (vb < fill_blocks + relabel_count) {
      relabel_tile<IdT, TableT, false>(prev, table, vb - fill_blocks);  // always a striding launch
    } else {
      const int64_t i = (vb - fill_blocks - relabel_count) * kBlock + threadIdx.x;
      if (i < clear_n16) clear_begin[i] = make_uint4(0u, 0u, 0u, 0u);
    }
  }
}

// The queued long rows of a hop, a 1024-thread block per row.
template <typename IdT, typename PtrT, typename TableT, bool REPLACE>
__global__ __launch_bounds__(kLongBlock) void hop_fill_weighted_long_kernel(Hop h, TableT table,
                                                                            TierView<PtrT> indptr,
                                                                            TierView<IdT> indices,
                                                                            TierView<float> probs, uint64_t rng_seed) {
  __shared__ LongRowScratch lds;
  const int64_t n_long = *h.long_count;
  const int64_t s = seeds_of(h);
  const bool look_first = look_before_insert(h, s);
  const bool bucketed = bucketed_now(h, s);
  const int k = h.k;
  for (int64_t t = blockIdx.x; t < n_long; t += gridDim.x) {
    const int64_t i = h.long_rows[t];
    const int64_t row = int64_t(static_cast<const IdT*>(h.seeds)[i]);
    const int64_t b = int64_t(indptr.at(row));
    const uint32_t deg = uint32_t(int64_t(indptr.at(row + 1)) - b);  // queued rows have a valid degree
    const int64_t p0 = h.pos_base + seed_part(h, s) + i * k;
    if (REPLACE) {
      draw_long_row(lds, probs, b, int64_t(deg), int64_t(k), rng_seed, h.rng_stream, row,
                    [&](int64_t j, int64_t pick) {
                      if (!emit_pick<IdT>(h, table, indices, p0 + j, true, b + pick, look_first, bucketed))
                        h.row_cnt[i] = kBadPick;
                    });
    } else {
      const uint32_t pos = race_long_row(lds, probs, b, deg, k, rng_seed, h.rng_stream, row);
      const int l = threadIdx.x;  // wave 0 holds the winners
      if (l < k && !emit_pick<IdT>(h, table, indices, p0 + l, pos < deg, b + pos, look_first, bucketed))
        h.row_cnt[i] = kBadPick;
    }
  }
}

// ---- the bucketed pass (see Buckets) --------------------------------------------------------

// Tiles are laid out so that no address depends on the hop's length: front_tiles tiles over the
// frontier array as large as it can get, then the tiles of the padded positions.  A block can
// therefore ask for its units at once and decide afterwards which of them count.
struct TileOfUnits {
  bool front;      // a tile of frontier ids
  int64_t first;   // its first rank, or its first position relative to the hop's pos_base
};
__device__ __forceinline__ TileOfUnits bucket_tile(const Buckets& b, int64_t tile) {
  TileOfUnits t;
  t.front = tile < b.front_tiles;
  t.first = (t.front ? tile : tile - b.front_tiles) * kBucketTile;
  return t;
}
// whether the tile holds anything at the hop's real length
__device__ __forceinline__ bool bucket_tile_live(const Hop& h, const TileOfUnits& t, int64_t s) {
  return t.first < (t.front ? s : s * h.k);
}
// A thread's units of a tile, requested without knowing the hop's length (every address lies inside
// its array whatever the length turns out to be); `valid` then says which of them count.
template <typename IdT>
struct UnitsOfThread {
  uint32_t id[kBucketTileItems];
  uint32_t order[kBucketTileItems];
  bool inside[kBucketTileItems];  // the address was inside the array, so id[] was loaded
  __device__ __forceinline__ void load(const Hop& h, const TileOfUnits& t) {
#pragma unroll
    for (int j = 0; j < kBucketTileItems; ++j) {
      const int64_t at = t.first + j * kBlock + threadIdx.x;
      if (t.front) {
        inside[j] = at < h.s_max;
        id[j] = inside[j] ? uint32_t(static_cast<const IdT*>(h.frontier)[at]) : 0u;
        order[j] = uint32_t(at);
      } else {
        inside[j] = at < h.len_max;
        const uint32_t word = inside[j] ? h.slot[h.pos_base + at] : kInvalidSlot;  // id | kFirstBit as the fill left it
        inside[j] = inside[j] && word != kInvalidSlot;
        id[j] = word & ~kFirstBit;
        order[j] = uint32_t(h.pos_base + at);
      }
    }
  }
  __device__ __forceinline__ bool valid(const Hop& h, const TileOfUnits& t, int64_t s, int j) const {
    const int64_t at = t.first + j * kBlock + threadIdx.x;
    return inside[j] && at < (t.front ? s : s * h.k);
  }
};

// One block per tile: the tile's units in bucket order (counted, placed and staged in LDS, then
// written as one contiguous run), and where every bucket's piece begins.
template <typename IdT>
__global__ __launch_bounds__(kBlock) void bucket_sort_kernel(Hop h, Buckets b) {
  __shared__ int cnt[kMaxBuckets];     // units per bucket, then the next free place of every bucket in the stage
  __shared__ uint2 stage[kBucketTile];
  __shared__ int lds[kBlock / kWave];
  if (blockIdx.x == 0 && threadIdx.x == 0) *h.bucket_overflow = 0;  // (the per-bucket launch comes behind this one)
  for (int64_t tile = blockIdx.x; tile < b.tiles_max; tile += gridDim.x) {
    const TileOfUnits t = bucket_tile(b, tile);
    UnitsOfThread<IdT> units;
    units.load(h, t);
    const int64_t s = seeds_of(h);
    if (!bucketed_now(h, s)) return;           // the hop outgrew the pass: it runs on the table
    if (!bucket_tile_live(h, t, s)) continue;  // whole blocks skip a tile together
    const int log_buckets = log_buckets_of(b, h, s);
    const int buckets = 1 << log_buckets;
    const int mine = buckets / kBlock;  // 1..8 consecutive buckets per thread
    for (int j = threadIdx.x; j < buckets; j += kBlock) cnt[j] = 0;
    __syncthreads();
#pragma unroll
    for (int j = 0; j < kBucketTileItems; ++j)
      if (units.valid(h, t, s, j)) atomicAdd(&cnt[bucket_of(b, log_buckets, units.id[j])], 1);
    __syncthreads();
    int own[kMaxBuckets / kBlock];
    int sum = 0;
#pragma unroll
    for (int j = 0; j < kMaxBuckets / kBlock; ++j) {
      own[j] = j < mine ? cnt[threadIdx.x * mine + j] : 0;
      sum += own[j];
    }
    int all;
    int at = block_exclusive_scan<kBlock, int>(sum, &all, lds);
    uint16_t* piece = b.piece + tile * (buckets + 1);
#pragma unroll
    for (int j = 0; j < kMaxBuckets / kBlock; ++j) {
      if (j < mine) {
        cnt[threadIdx.x * mine + j] = at;  // (the scan's barriers lie between the reads above and this)
        piece[threadIdx.x * mine + j] = uint16_t(at);
        at += own[j];
      }
    }
    if (threadIdx.x == 0) piece[buckets] = uint16_t(all);  // <= 4096
    __syncthreads();
#pragma unroll
    for (int j = 0; j < kBucketTileItems; ++j) {
      if (units.valid(h, t, s, j)) {
        const int to = atomicAdd(&cnt[bucket_of(b, log_buckets, units.id[j])], 1);
        if (to >= 0 && to < kBucketTile) stage[to] = make_uint2(units.id[j], units.order[j]);
      }
    }
    __syncthreads();
    const int staged = all < kBucketTile ? all : kBucketTile;
    for (int e = threadIdx.x; e < staged; e += kBlock) b.items[tile * kBucketTile + e] = stage[e];
    __syncthreads();
  }
}

// One block per bucket.  It lists the bucket's pieces in the live tiles (LDS: where each begins in
// items[] and how many units came before it), so that its threads can share the bucket's units
// evenly whatever their spread over the tiles; then the smallest order value of every id (LDS,
// indexed by id / buckets), then the slot word of every pick that is not its id's first occurrence.
__global__ __launch_bounds__(kBlock) void bucket_first_kernel(Hop h, Buckets b) {
  __shared__ uint32_t best[kBucketRange];
  __shared__ int piece_at[kMaxBucketTiles];      // first unit of the tile's piece, as an index into items[]
  __shared__ int piece_before[kMaxBucketTiles];  // units of the bucket in the tiles before
  __shared__ int lds[kBlock / kWave];
  const int buckets = 1 << b.log_buckets;
  const uint32_t range = (b.n_nodes + uint32_t(buckets) - 1) >> b.log_buckets;  // <= kBucketRange by the plan
  const uint32_t pos_begin = uint32_t(h.pos_base), pos_end = uint32_t(h.pos_base + h.len_max);
  const int64_t s = seeds_of(h);
  if (!bucketed_now(h, s)) return;
  const int tiles = b.tiles_max < kMaxBucketTiles ? b.tiles_max : kMaxBucketTiles;
  const int64_t item_count = int64_t(b.tiles_max) * kBucketTile;
  for (int bucket = blockIdx.x; bucket < buckets; bucket += gridDim.x) {
    for (uint32_t j = threadIdx.x; j < range && j < uint32_t(kBucketRange); j += kBlock) best[j] = 0xffffffffu;
    // the bucket's pieces: every thread asks for those of its tiles (tile = round * kBlock + thread)
    // at once, then the rounds are scanned one after the other, a running total carried along
    constexpr int kRounds = kMaxBucketTiles / kBlock;
    int from[kRounds], upto[kRounds];
#pragma unroll
    for (int q = 0; q < kRounds; ++q) {
      const int tile = q * kBlock + threadIdx.x;
      from[q] = upto[q] = 0;
      if (tile < tiles && bucket_tile_live(h, bucket_tile(b, tile), s)) {
        const uint16_t* piece = b.piece + int64_t(tile) * (buckets + 1);
        from[q] = piece[bucket];
        upto[q] = piece[bucket + 1];
      }
    }
    int total = 0;
#pragma unroll
    for (int q = 0; q < kRounds; ++q) {
      if (q * kBlock >= tiles) break;  // the same for every thread
      const int tile = q * kBlock + threadIdx.x;
      const int count = from[q] <= upto[q] && upto[q] <= kBucketTile ? upto[q] - from[q] : 0;
      int sum;
      const int before = block_exclusive_scan<kBlock, int>(count, &sum, lds);
      if (tile < tiles) {
        piece_at[tile] = tile * kBucketTile + from[q];
        piece_before[tile] = total + before;
      }
      total += sum;
    }
    __syncthreads();
    // unit j of the bucket lives in the last tile whose piece_before is <= j
    const auto unit = [&](int j) {
      int lo = 0, hi = tiles - 1;
      while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (piece_before[mid] <= j) lo = mid; else hi = mid - 1;
      }
      const int64_t at = int64_t(piece_at[lo]) + (j - piece_before[lo]);
      return at >= 0 && at < item_count ? b.items[at] : make_uint2(0u, 0u);
    };
    // a thread's first kKept units stay in registers for the second pass
    constexpr int kKept = 8;
    uint2 kept[kKept];
#pragma unroll
    for (int r = 0; r < kKept; ++r) {
      const int j = threadIdx.x + r * kBlock;
      kept[r] = j < total ? unit(j) : make_uint2(0u, 0u);
    }
    for (int j = threadIdx.x, r = 0; j < total; j += kBlock, ++r) {
      uint2 it = make_uint2(0u, 0u);
      if (r < kKept) {
#pragma unroll
        for (int q = 0; q < kKept; ++q) if (q == r) it = kept[q];
      } else {
        it = unit(j);
      }
      const uint32_t at = it.x >> b.log_buckets;
      if (at < range && at < uint32_t(kBucketRange)) atomicMin(&best[at], it.y);
    }
    __syncthreads();
    for (int j = threadIdx.x, r = 0; j < total; j += kBlock, ++r) {
      uint2 it = make_uint2(0u, 0u);
      if (r < kKept) {
#pragma unroll
        for (int q = 0; q < kKept; ++q) if (q == r) it = kept[q];
      } else {
        it = unit(j);
      }
      const uint32_t at = it.x >> b.log_buckets;
      if (it.y < pos_begin || it.y >= pos_end || at >= range || at >= uint32_t(kBucketRange)) continue;  // a frontier id
      const uint32_t least = best[at];  // first occurrences keep the word the fill gave them
      if (least != it.y) h.slot[it.y] = least < pos_begin ? (least | kRankBit) : least;
    }
    __syncthreads();
  }
}

// The per-bucket kernel for graphs of any node count: as bucket_first_kernel, but a bucket's ids
// are told apart in an open-addressing table in LDS (the id claims a slot with a compare-and-swap,
// the slot's second word takes the smallest order value), since an array indexed by the id itself
// would not fit.  Buckets are chosen by low bits of a hash of the id, slots by the next bits.
// A bucket with more units than three quarters of the table's slots (its ids might not fit) is
// gone over in parts, by yet other bits of the hash, one table's worth at a time.  Ids that crowd
// one part all the same (more than kHashSlots distinct ones: not by chance) set the hop's overflow
// word, which fails the call.
__global__ __launch_bounds__(kHashBlock) void bucket_first_hashed_kernel(Hop h, Buckets b) {
  __shared__ uint32_t owner[kHashSlots];
  __shared__ uint32_t best[kHashSlots];
  __shared__ int piece_at[kMaxBucketTiles];      // first unit of the tile's piece, as an index into items[]
  __shared__ int piece_before[kMaxBucketTiles];  // units of the bucket in the tiles before
  __shared__ int lds[kHashBlock / kWave];
  __shared__ int overflow;
  const uint32_t pos_begin = uint32_t(h.pos_base), pos_end = uint32_t(h.pos_base + h.len_max);
  const int64_t s = seeds_of(h);
  if (!bucketed_now(h, s)) return;
  const int log_buckets = log_buckets_of(b, h, s);
  const int buckets = 1 << log_buckets;
  const int tiles = b.tiles_max < kMaxBucketTiles ? b.tiles_max : kMaxBucketTiles;
  const int64_t item_count = int64_t(b.tiles_max) * kBucketTile;
  for (int bucket = blockIdx.x; bucket < buckets; bucket += gridDim.x) {
    if (threadIdx.x == 0) overflow = 0;
    constexpr int kRounds = kMaxBucketTiles / kHashBlock;
    int from[kRounds], upto[kRounds];
#pragma unroll
    for (int q = 0; q < kRounds; ++q) {
      const int tile = q * kHashBlock + threadIdx.x;
      from[q] = upto[q] = 0;
      if (tile < tiles && bucket_tile_live(h, bucket_tile(b, tile), s)) {
        const uint16_t* piece = b.piece + int64_t(tile) * (buckets + 1);
        from[q] = piece[bucket];
        upto[q] = piece[bucket + 1];
      }
    }
    int total = 0;
#pragma unroll
    for (int q = 0; q < kRounds; ++q) {
      if (q * kHashBlock >= tiles) break;  // the same for every thread
      const int tile = q * kHashBlock + threadIdx.x;
      const int count = from[q] <= upto[q] && upto[q] <= kBucketTile ? upto[q] - from[q] : 0;
      int sum;
      const int before = block_exclusive_scan<kHashBlock, int>(count, &sum, lds);
      if (tile < tiles) {
        piece_at[tile] = tile * kBucketTile + from[q];
        piece_before[tile] = total + before;
      }
      total += sum;
    }
    // The table is as large as the bucket needs: at least twice its units (all of them may be
    // distinct ids), all of the array when that is not enough; beyond three quarters of the array
    // the bucket is split into parts.
    const int capacity = b.hash_slots;
    const int parts = total <= capacity * 3 / 4 ? 1 : (total + capacity / 2 - 1) / (capacity / 2);
    int slots = capacity < 1024 ? capacity : 1024;
    while (slots < 2 * (total / parts + 1) && slots < capacity) slots <<= 1;
    const uint32_t slot_mask = uint32_t(slots - 1);
    __syncthreads();  // piece_at / piece_before are complete
    const auto unit = [&](int j) {
      int lo = 0, hi = tiles - 1;
      while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (piece_before[mid] <= j) lo = mid; else hi = mid - 1;
      }
      const int64_t at = int64_t(piece_at[lo]) + (j - piece_before[lo]);
      return at >= 0 && at < item_count ? b.items[at] : make_uint2(kHashEmpty, 0u);
    };
    // where an id's slot search starts, and which part it belongs to: bits of its hash that the
    // choice of the bucket did not use
    const auto home = [&](uint32_t hash) { return (hash >> log_buckets) & slot_mask; };
    const auto part_of = [&](uint32_t hash) { return int((hash >> 23) % uint32_t(parts)); };
    constexpr int kKept = 8;  // a thread's first units stay in registers across the passes
    uint2 kept[kKept];
#pragma unroll
    for (int r = 0; r < kKept; ++r) {
      const int j = threadIdx.x + r * kHashBlock;
      kept[r] = j < total ? unit(j) : make_uint2(kHashEmpty, 0u);
    }
    for (int part = 0; part < parts; ++part) {
      for (int j = threadIdx.x; j < slots; j += kHashBlock) {
        owner[j] = kHashEmpty;
        best[j] = 0xffffffffu;
      }
      __syncthreads();
      // every unit of the part claims its id's slot (or finds it claimed by the same id) and offers its order value
      uint32_t kept_slot[kKept];
#pragma unroll
      for (int r = 0; r < kKept; ++r) kept_slot[r] = kHashEmpty;
      for (int j = threadIdx.x, r = 0; j < total; j += kHashBlock, ++r) {
        uint2 it = make_uint2(kHashEmpty, 0u);
        if (r < kKept) {
#pragma unroll
          for (int q = 0; q < kKept; ++q) if (q == r) it = kept[q];
        } else {
          it = unit(j);
        }
        if (it.x == kHashEmpty) continue;
        const uint32_t hash = hash_id(it.x);
        if (parts > 1 && part_of(hash) != part) continue;
        uint32_t slot = home(hash);
        bool placed = false;
        for (int probes = 0; probes < slots; ++probes) {
          uint32_t seen = owner[slot];
          if (seen == kHashEmpty) seen = atomicCAS(&owner[slot], kHashEmpty, it.x);
          if (seen == kHashEmpty || seen == it.x) {
            placed = true;
            break;
          }
          slot = (slot + 1) & slot_mask;
        }
        if (placed) atomicMin(&best[slot], it.y); else overflow = 1;
        if (r < kKept) {
#pragma unroll
          for (int q = 0; q < kKept; ++q) if (q == r) kept_slot[q] = placed ? slot : kHashEmpty;
        }
      }
      __syncthreads();
      if (overflow == 0) {  // (an overflowing part's answers are void: the call fails, nothing is rewritten)
        for (int j = threadIdx.x, r = 0; j < total; j += kHashBlock, ++r) {
          uint2 it = make_uint2(kHashEmpty, 0u);
          uint32_t slot = kHashEmpty;
          if (r < kKept) {
#pragma unroll
            for (int q = 0; q < kKept; ++q) if (q == r) { it = kept[q]; slot = kept_slot[q]; }
          } else {
            it = unit(j);
          }
          if (it.x == kHashEmpty || it.y < pos_begin || it.y >= pos_end) continue;  // not a pick of this hop
          const uint32_t hash = hash_id(it.x);
          if (parts > 1 && part_of(hash) != part) continue;
          if (slot == kHashEmpty) {  // beyond what the registers kept: find the id's slot again
            slot = home(hash);
            for (int probes = 0; probes < slots && owner[slot] != it.x; ++probes) slot = (slot + 1) & slot_mask;
          }
          const uint32_t least = best[slot];  // first occurrences keep the word the fill gave them
          if (least != it.y) h.slot[it.y] = least < pos_begin ? (least | kRankBit) : least;
        }
      }
      __syncthreads();
    }
    if (threadIdx.x == 0 && overflow != 0) *h.bucket_overflow = 1;
    __syncthreads();
  }
}

// One virtual block of the flag launch: 1024 padded positions.
template <typename IdT, typename TableT, bool EARLY>
__device__ __forceinline__ void flag_tile(const Hop& h, int64_t tile, const TableT& table) {
  __shared__ int lds[kBlock / kWave];
  const int64_t s = seeds_of(h);
  const int64_t len = seed_part(h, s) + s * h.k;
  if (!EARLY && tile * kPosTile >= len) {
    if (threadIdx.x == 0) h.pos_cnt[tile] = 0;
    return;
  }
  const int64_t base = tile * kPosTile + threadIdx.x * kPosItems;
  // this thread's slot words and lost marks (EARLY: requested together with the hop's length)
  const int64_t readable = EARLY ? h.len_max : len;
  uint32_t w[kPosItems];
  uint8_t gone[kPosItems];
#pragma unroll
  for (int j = 0; j < kPosItems; ++j) {
    const bool inside = base + j < readable;
    w[j] = inside ? h.slot[h.pos_base + base + j] : kInvalidSlot;
    gone[j] = inside && h.index != 0 ? h.lost[h.pos_base + base + j] : uint8_t(0);
  }
  int c = 0;
  if (tile * kPosTile < len) {
#pragma unroll
    for (int j = 0; j < kPosItems; ++j) {
      const int64_t rel = base + j;
      if (rel < len && w[j] != kInvalidSlot) {
        const int64_t p = h.pos_base + rel;
        if (h.index == 0) {
          if (table.value(w[j]) == uint32_t(p)) {
            h.slot[p] = w[j] | kFirstBit;
            ++c;
          }
        } else if (w[j] & kFirstBit) {
          if (gone[j]) h.slot[p] = w[j] & ~kFirstBit; else ++c;
        }
      }
    }
    c = block_sum<kBlock, int>(c, lds);
  }
  if (threadIdx.x == 0) h.pos_cnt[tile] = c;
}

// Virtual blocks [0, flag_blocks): position tiles; then row_tiles blocks scanning the rows' pick
// counts per 256-row tile (for the packed edge list, off the critical path).
template <typename IdT, typename TableT, bool STRIDE>
__global__ __launch_bounds__(kBlock) void hop_flag_kernel(Hop h, int64_t flag_blocks, int64_t row_tiles,
                                                          TableT table) {
  DGS_FOR_VIRTUAL_BLOCKS(vb, flag_blocks + row_tiles) {
    if (vb < flag_blocks) flag_tile<IdT, TableT, !STRIDE>(h, vb, table);
    else offsets_tile(h, int(vb - flag_blocks));
  }
}

// Separate scans for very long tile lists (one block), over the tiles the hop really has.
__device__ __forceinline__ int64_t real_pos_tiles(const Hop& h, int64_t s) {
  return (seed_part(h, s) + s * h.k + kPosTile - 1) / kPosTile;
}
__global__ __launch_bounds__(1024) void pos_scan_kernel(Hop h) {
  int64_t sum;
  single_block_scan<1024, int, int64_t>(h.pos_cnt, h.pos_off, real_pos_tiles(h, seeds_of(h)), &sum);
}
__global__ __launch_bounds__(1024) void tile_scan_kernel(Hop h) {
  int64_t sum;
  single_block_scan<1024, int, int64_t>(h.tile_sum, h.tile_off, (seeds_of(h) + kRowTile - 1) / kRowTile, &sum);
}

// One virtual block of the compact launch: the first occurrences of one 1024-position tile.
// `pos_tiles` / `row_tiles` are the worst-case tile counts the flag launch covered: the counts of
// tiles beyond the hop's real length are zero there, so sums may run over all of them.
template <typename IdT, typename TableT, bool EARLY>
__device__ __forceinline__ void compact_tile(const Hop& h, int64_t tile, int64_t pos_tiles, int64_t row_tiles,
                                             const TableT& table) {
  __shared__ int64_t lds64[kBlock / kWave];
  __shared__ int lds[kBlock / kWave];
  // the hop's length, this thread's slot words and its share of the tile counts (EARLY: requested together)
  const int64_t s = seeds_of(h);
  const int64_t len = seed_part(h, s) + s * h.k;
  if (!EARLY && tile != 0 && tile * kPosTile >= len) return;
  const int64_t base = tile * kPosTile + threadIdx.x * kPosItems;
  const int64_t readable = EARLY ? h.len_max : len;
  uint32_t w[kPosItems];
#pragma unroll
  for (int j = 0; j < kPosItems; ++j) w[j] = base + j < readable ? h.slot[h.pos_base + base + j] : kInvalidSlot;
  // first occurrences in the tiles before this one (block 0 needs the grand total instead)
  int64_t part = 0;
  if (h.pos_off) {  // scanned by pos_scan_kernel over the hop's real tiles
    const int64_t last = real_pos_tiles(h, s) - 1;
    if (threadIdx.x == 0) part = tile != 0 ? h.pos_off[tile] : last >= 0 ? h.pos_off[last] + h.pos_cnt[last] : 0;
  } else {
    const int64_t upto = tile == 0 ? pos_tiles : tile;
    for (int64_t j = threadIdx.x; j < upto; j += kBlock) part += h.pos_cnt[j];
  }
  int64_t edges = 0;
  int bad = 0;
  if (tile == 0) {
    for (int64_t j = threadIdx.x; j < row_tiles; j += kBlock) {
      edges += h.tile_sum[j];
      bad |= h.tile_flag[j];
    }
  }
  const int64_t rank0 = first_rank(h, s);
  if (tile != 0 && tile * kPosTile >= len) return;  // whole blocks leave together
  part = block_sum<kBlock, int64_t>(part, lds64);
  if (tile == 0) {
    // this hop's lengths, written even when there is nothing to do: frontier size, edge count
    // (row tiles were scanned by the surplus blocks of the flag launch) and error bits
    edges = block_sum<kBlock, int64_t>(edges, lds64);
    bad = block_or<kBlock>(bad, lds);
    if (h.bucketed != 0 && *h.bucket_overflow != 0) bad |= kErrBucketOverflow;
    if (threadIdx.x == 0) {
      *h.n_unique = rank0 + part;
      *h.nnz = edges;
      *h.flags = bad;
      if (h.host_sizes) {
        if (h.index == 0) mirror_to_host(h.host_sizes, s);
        mirror_to_host(h.host_sizes + h.index + 1, rank0 + part);
        mirror_to_host(h.host_sizes + h.n_hops + 1 + h.index, edges);
        mirror_to_host(h.host_sizes + 2 * h.n_hops + 1 + h.index, bad);
      }
    }
    if (len <= 0) return;
  }
  const int64_t before = tile == 0 ? 0 : part;
  int c = 0;
#pragma unroll
  for (int j = 0; j < kPosItems; ++j) {
    if (base + j >= len || w[j] == kInvalidSlot) w[j] = 0;  // bit 31 clear: not a first occurrence
    c += (w[j] & kFirstBit) != 0;
  }
  int total;
  int64_t rank = rank0 + before + block_exclusive_scan<kBlock, int>(c, &total, lds);
#pragma unroll
  for (int j = 0; j < kPosItems; ++j) {
    if (w[j] & kFirstBit) {
      static_cast<IdT*>(h.frontier)[rank] = table.key(w[j] & ~kFirstBit);
      h.rank_at[h.pos_base + base + j] = uint32_t(rank);
      ++rank;
    }
  }
}

template <typename IdT, typename TableT, bool STRIDE>
__global__ __launch_bounds__(kBlock) void hop_compact_kernel(Hop h, int64_t blocks, int64_t pos_tiles,
                                                             int64_t row_tiles, TableT table) {
  DGS_FOR_VIRTUAL_BLOCKS(vb, blocks) compact_tile<IdT, TableT, !STRIDE>(h, vb, pos_tiles, row_tiles, table);
}

template <typename IdT, typename TableT, bool STRIDE>
__global__ __launch_bounds__(kBlock) void hop_relabel_kernel(Hop h, int64_t blocks, TableT table) {
  DGS_FOR_VIRTUAL_BLOCKS(vb, blocks) relabel_tile<IdT, TableT, !STRIDE>(h, table, vb);
}

__global__ void zero_sizes_kernel(int64_t* __restrict__ sizes, int n) {
  for (int i = threadIdx.x; i < n; i += blockDim.x) sizes[i] = 0;
}

__global__ __launch_bounds__(kBlock) void clear_kernel(uint4* __restrict__ p, int64_t n16) {
  for (int64_t i = int64_t(blockIdx.x) * kBlock + threadIdx.x; i < n16; i += int64_t(gridDim.x) * kBlock)
    p[i] = make_uint4(~0u, ~0u, ~0u, ~0u);
}

// ---- host side -------------------------------------------------------------------------------

enum class TableKind { kDirect, kPacked, kSplit };

struct Plan {
  int n_hops = 0;
  TableKind kind = TableKind::kSplit;
  int64_t s_max[DGS_MAX_HOPS + 1];
  int64_t nnz_max[DGS_MAX_HOPS];
  uint32_t capacity = 0;     // hash table slots (one table for all hops)
  size_t table_bytes = 0;    // 0 for the direct table
  bool weighted = false;     // picks by edge weight: per-hop queues for long rows
  bool bucketed = false;     // the last hop may find its first occurrences by the bucketed pass (if it turns out to fit)
  bool bucket_hashed = false; // ... with ids told apart by an LDS hash table (graphs beyond kBucketedMaxNodes)
  bool bucket_space = false; // the workspace has room for that pass
  int32_t bucket_front_tiles = 0;  // tiles over the frontier array as large as it can be before the last hop
  int32_t bucket_pos_tiles = 0;    // tiles over the last hop's padded positions: all of them, or as many as there is room for
  int32_t log_buckets = 0;
  int32_t hash_slots = kHashSlots;
  uint32_t n_nodes = 0;
};

// Tiles of the bucketed pass: the frontier before the last hop at its worst case, and as many of the
// hop's padded positions as the per-bucket kernels can index (a hop beyond that runs on the table).
inline void plan_bucket_tiles(Plan* p) {
  const int64_t front = (p->s_max[p->n_hops - 1] + kBucketTile - 1) / kBucketTile;
  const int64_t pos = (p->nnz_max[p->n_hops - 1] + kBucketTile - 1) / kBucketTile;
  const int64_t room = int64_t(kMaxBucketTiles) - 2 - front;
  p->bucket_space = p->n_hops >= 2 && room >= 1;
  p->bucket_front_tiles = int32_t(front);
  p->bucket_pos_tiles = int32_t(pos < room ? pos : (room > 0 ? room : 0));
}

dgs_status make_plan(int64_t n_seeds, const int64_t* fanouts, int32_t n_hops, int32_t id_bytes,
                     int64_t n_nodes, bool have_node_table, Plan* p) {
  DGS_REQUIRE(n_hops >= 1 && n_hops <= DGS_MAX_HOPS, DGS_ERR_INVALID, "sample_blocks: %d hops (1..%d)", n_hops,
              DGS_MAX_HOPS);
  DGS_REQUIRE(fanouts != nullptr && n_seeds >= 0, DGS_ERR_INVALID, "sample_blocks: bad argument");
  DGS_REQUIRE(width_ok(id_bytes), DGS_ERR_INVALID, "sample_blocks: id width %d is not 4 or 8", id_bytes);
  p->n_hops = n_hops;
  p->s_max[0] = n_seeds;
  for (int h = 0; h < n_hops; ++h) {
    DGS_REQUIRE(fanouts[h] >= 0 && fanouts[h] <= kMaxPicks, DGS_ERR_UNSUPPORTED,
                "sample_blocks: fanout %lld outside 0..%d (use the per-hop operators)", (long long)fanouts[h],
                kMaxPicks);
    p->nnz_max[h] = p->s_max[h] * fanouts[h];
    p->s_max[h + 1] = p->s_max[h] + p->nnz_max[h];
    DGS_REQUIRE(p->s_max[h + 1] <= kMaxPositions, DGS_ERR_UNSUPPORTED,
                "sample_blocks: worst-case frontier of hop %d exceeds 2^30 ids", h);
  }
  // room for the bucketed pass (whether a hop takes it is decided below and, from its real size, on the device)
  plan_bucket_tiles(p);
  if (have_node_table) {
    DGS_REQUIRE(n_nodes >= 0 && n_nodes < 0x7fffffffLL, DGS_ERR_UNSUPPORTED,
                "sample_blocks: a node table needs fewer than 2^31 nodes (have %lld)", (long long)n_nodes);
    p->kind = TableKind::kDirect;
    // the bucketed pass: slot words are ids (the direct table's), and the hop is large enough for
    // its two extra launches to cost less than the atomics they replace.  Ids that fit the LDS
    // array of a bucket (kBucketRange ids in each of at most kMaxBuckets buckets) index it directly;
    // larger graphs take the hashed form.
    // (test hook: 1 never, 2 whatever the size, 3 whatever the size and hashed whatever the graph,
    // 4 like 3 with on-chip tables of 256 slots, so that small inputs fill them and go over their
    // buckets in parts)
    const int64_t mode = debug_option(DGS_DEBUG_SAMPLER_BUCKETED);
    const bool large = p->nnz_max[n_hops - 1] >= kBucketedMinPicks;
    p->bucket_hashed = n_nodes > kBucketedMaxNodes || mode == 3 || mode == 4;
    // By size only the direct form runs.  The hashed form gives the same results on any graph and
    // takes the atomics out of the hop just the same, but it does not pay: 111 M nodes, 944 k picks
    // of mostly new ids: fill 64 -> 35 us and relabel 14 -> 12, against 19 + 22 us for its two
    // launches (0.187-0.200 ms per step in flight against 0.191); R-MAT with two thirds repeats: every
    // repeat costs a scattered 4-byte store where the table's look before the atomic gets cheaper
    // (0.382 against 0.373 ms).  It runs when the test hook asks for it.
    p->bucketed = p->bucket_space && n_nodes >= 1 && fanouts[n_hops - 1] >= 1 && mode != 1 &&
                  (p->bucket_hashed ? mode >= 2 : (large || mode >= 2));
    p->hash_slots = mode == 4 ? 256 : kHashSlots;
    int log_b = 0;
    if (p->bucket_hashed) {
      // a bucket's LDS table takes kHashSlots ids: at most half as many units per bucket on average
      const int64_t units = int64_t(p->bucket_front_tiles + p->bucket_pos_tiles) * kBucketTile;
      while ((1 << log_b) < kMinBuckets || ((int64_t(kHashSlots) << log_b) < units && (1 << log_b) < kMaxBuckets)) ++log_b;
    } else {
      while ((1 << log_b) < kMinBuckets || (int64_t(kBucketRange) << log_b) < n_nodes) ++log_b;
    }
    p->log_buckets = log_b;
    p->n_nodes = uint32_t(n_nodes);
  } else {
    // ids fit the packed slot when every node id is below 2^32 - 1
    p->kind = id_bytes == 4 || (n_nodes >= 0 && n_nodes < 0xffffffffLL) ? TableKind::kPacked : TableKind::kSplit;
    // test hook: exercise the split (id array + value array) table on small graphs
    if (id_bytes == 8 && debug_option(DGS_DEBUG_FORCE_SPLIT_TABLE) != 0) p->kind = TableKind::kSplit;
    p->capacity = table_capacity(p->s_max[n_hops]);
    p->table_bytes = size_t(p->capacity) * (p->kind == TableKind::kPacked ? 8 : size_t(id_bytes) + 4);
  }
  return DGS_OK;
}

// Lays the workspace out; with base == nullptr only the size is computed.
size_t layout(const Plan& p, const int64_t* fanouts, void* base, Hop* hops, void** table,
              Buckets* buckets = nullptr) {
  Carver c(base);
  char* t = c.take<char>(p.table_bytes);
  if (table) *table = t;
  const size_t positions = size_t(p.s_max[p.n_hops]);  // sum over hops of (seed part + s_max * k)
  uint32_t* slot = c.take<uint32_t>(positions);
  uint32_t* rank_at = c.take<uint32_t>(positions);
  uint8_t* lost = c.take<uint8_t>(positions + 16);
  int64_t* long_counts = p.weighted ? c.take<int64_t>(DGS_MAX_HOPS) : nullptr;
  int64_t pos_base = 0;
  for (int h = 0; h < p.n_hops; ++h) {
    const size_t s = size_t(p.s_max[h]);
    const size_t len = (h == 0 ? s : 0) + size_t(p.nnz_max[h]);
    const size_t row_tiles = (s + kRowTile - 1) / kRowTile;
    const size_t pos_tiles = (len + kPosTile - 1) / kPosTile;
    Hop v{};
    v.row_cnt = c.take<uint32_t>(s);
    v.row_off = c.take<uint32_t>(s);
    v.tile_sum = c.take<int>(row_tiles);
    v.tile_flag = c.take<int>(row_tiles);
    v.tile_off = row_tiles > size_t(kInlineTiles) ? c.take<int64_t>(row_tiles) : nullptr;
    v.slot = slot;
    v.rank_at = rank_at;
    v.lost = lost;
    v.long_rows = p.weighted ? c.take<int64_t>(s) : nullptr;
    v.long_count = p.weighted ? long_counts + h : nullptr;
    v.pos_cnt = c.take<int>(pos_tiles + 1);
    v.pos_off = pos_tiles > size_t(kInlineTiles) ? c.take<int64_t>(pos_tiles) : nullptr;
    v.s_max = p.s_max[h];
    v.pos_base = pos_base;
    v.len_max = int64_t(len);
    v.k = int32_t(fanouts[h]);
    v.index = h;
    v.bucketed = p.bucketed && h == p.n_hops - 1;
    v.bucket_pos_cap = int64_t(p.bucket_pos_tiles) * kBucketTile;
    if (hops) hops[h] = v;
    pos_base += int64_t(len);
  }
  if (p.bucket_space) {
    Buckets b{};
    b.front_tiles = p.bucket_front_tiles;
    b.tiles_max = p.bucket_front_tiles + p.bucket_pos_tiles;
    b.items = c.take<uint2>(size_t(b.tiles_max) * kBucketTile);
    b.piece = c.take<uint16_t>(size_t(b.tiles_max) * (kMaxBuckets + 1));
    int* overflow = c.take<int>(4);
    b.log_buckets = p.log_buckets;
    b.n_nodes = p.n_nodes;
    b.hashed = p.bucket_hashed ? 1 : 0;
    b.hash_slots = p.hash_slots;
    if (buckets) *buckets = b;
    if (hops)
      for (int h = 0; h < p.n_hops; ++h) hops[h].bucket_overflow = overflow;
  }
  return c.used + 256;
}

// The packed edge list of one hop as a launch of its own.
template <typename IdT, typename TableT>
void launch_relabel(const Hop& hop, const TableT& table, hipStream_t st) {
  const int64_t blocks = relabel_blocks(hop.s_max, hop.k);
  if (blocks <= 0) return;
  if (is_capped(blocks))
    hipLaunchKernelGGL((hop_relabel_kernel<IdT, TableT, true>), dim3(capped_grid(blocks)), dim3(kBlock), 0, st, hop,
                       blocks, table);
  else
    hipLaunchKernelGGL((hop_relabel_kernel<IdT, TableT, false>), dim3(capped_grid(blocks)), dim3(kBlock), 0, st, hop,
                       blocks, table);
}

template <typename IdT, typename PtrT, typename TableT, int G>
void launch_fill(const Hop& cur, const Hop& prev, int64_t relabel_count, uint4* clear_begin, int64_t clear_n16,
                 const TableT& table, const dgs_view& indptr, const dgs_view& indices, bool replace,
                 uint64_t rng_seed, hipStream_t st) {
  const int64_t fill_blocks = (cur.s_max * G + kBlock - 1) / kBlock;
  const int64_t clear_blocks = (clear_n16 + kBlock - 1) / kBlock;
  int64_t total = fill_blocks + relabel_count + clear_blocks;
  if (is_capped(total)) {
    // A launch that loops over its virtual blocks keeps the previous hop's edge list out of the
    // loop: with it the kernel needs 85-90 vector registers and five waves fit a SIMD instead of
    // seven (measured on a 136 k-row hop: 46 us against 39).  That list becomes a launch of its own,
    // behind this one (the previous hop's table entries do not change any more: positions only grow).
    total -= relabel_count;
    hipLaunchKernelGGL((hop_fill_kernel<IdT, PtrT, TableT, G, true>), dim3(capped_grid(total)), dim3(kBlock), 0, st,
                       cur, prev, fill_blocks, int64_t(0), clear_begin, clear_n16, table,
                       TierView<PtrT>(indptr), TierView<IdT>(indices), replace, rng_seed);
    if (relabel_count > 0) launch_relabel<IdT>(prev, table, st);
  } else
    hipLaunchKernelGGL((hop_fill_kernel<IdT, PtrT, TableT, G, false>), dim3(capped_grid(total)), dim3(kBlock), 0, st,
                       cur, prev, fill_blocks, relabel_count, clear_begin, clear_n16, table,
                       TierView<PtrT>(indptr), TierView<IdT>(indices), replace, rng_seed);
}

// The weighted fill of one hop: the main launch (a wave per row) and the block-per-row launch for
// the rows it queued.  Only the direct table is supported (the entry point insists on one).
template <typename IdT, typename PtrT, typename TableT, bool REPLACE>
dgs_status launch_fill_weighted(const Hop& cur, const Hop& prev, int64_t relabel_count, uint4* clear_begin,
                                int64_t clear_n16, const TableT& table, const dgs_view& indptr,
                                const dgs_view& indices, const dgs_view& probs, uint64_t rng_seed, hipStream_t st) {
  const int64_t rows_per_block = weighted_rows_per_block(cur.k);
  const int64_t fill_blocks = (cur.s_max + rows_per_block - 1) / rows_per_block;
  const int64_t clear_blocks = (clear_n16 + kBlock - 1) / kBlock;
  const int64_t total = fill_blocks + relabel_count + clear_blocks;
  hipLaunchKernelGGL((hop_fill_weighted_kernel<IdT, PtrT, TableT, REPLACE>), dim3(capped_grid(total)), dim3(kBlock),
                     0, st, cur, prev, fill_blocks, relabel_count, clear_begin, clear_n16, table,
                     TierView<PtrT>(indptr), TierView<IdT>(indices), TierView<float>(probs), rng_seed);
  DGS_LAUNCH_CHECK();
  // two 1024-thread blocks fit a CU: at most one round over the 256 CUs
  const uint32_t long_blocks = uint32_t(cur.s_max < kMaxLongGrid ? (cur.s_max < 1 ? 1 : cur.s_max) : kMaxLongGrid);
  hipLaunchKernelGGL((hop_fill_weighted_long_kernel<IdT, PtrT, TableT, REPLACE>), dim3(long_blocks),
                     dim3(kLongBlock), 0, st, cur, table, TierView<PtrT>(indptr), TierView<IdT>(indices),
                     TierView<float>(probs), rng_seed);
  DGS_LAUNCH_CHECK();
  return DGS_OK;
}

template <typename IdT, typename PtrT, typename TableT>
dgs_status run_blocks(const Plan& p, Hop* hops, const Buckets& buckets, const TableT& table, const dgs_view& indptr,
                      const dgs_view& indices, const dgs_view* probs, bool replace, uint64_t rng_seed,
                      void** sizes_ticket, hipStream_t st) {
  if (p.weighted) {  // the long-row queues of all hops start empty (their counters are one array, hop 0's first)
    hipLaunchKernelGGL(zero_sizes_kernel, dim3(1), dim3(64), 0, st, hops[0].long_count, p.n_hops);
    DGS_LAUNCH_CHECK();
  }
  for (int h = 0; h < p.n_hops; ++h) {
    const Hop& cur = hops[h];
    const Hop prev = h > 0 ? hops[h - 1] : Hop{};
    const int64_t surplus = h > 0 ? relabel_blocks(prev.s_max, prev.k) : 0;
    // the launch of hop 0 also clears the lost marks of all later hops (16-byte granules; the
    // first one may reach back into hop 0's own range, whose marks are never read or written)
    uint4* clear_begin = nullptr;
    int64_t clear_n16 = 0;
    if (h == 0 && p.n_hops > 1) {
      const int64_t first = hops[1].pos_base / 16 * 16;
      const int64_t last = (p.s_max[p.n_hops] + 15) / 16 * 16;  // the array has 16 spare bytes
      clear_begin = reinterpret_cast<uint4*>(cur.lost + first);
      clear_n16 = last > first ? (last - first) / 16 : 0;
    }
    if (p.weighted) {
      const dgs_status ws = replace ? launch_fill_weighted<IdT, PtrT, TableT, true>(cur, prev, surplus, clear_begin, clear_n16, table, indptr, indices, *probs, rng_seed, st)
                                    : launch_fill_weighted<IdT, PtrT, TableT, false>(cur, prev, surplus, clear_begin, clear_n16, table, indptr, indices, *probs, rng_seed, st);
      if (ws != DGS_OK) return ws;
    } else if (cur.k <= 8) launch_fill<IdT, PtrT, TableT, 8>(cur, prev, surplus, clear_begin, clear_n16, table, indptr, indices, replace, rng_seed, st);
    else if (cur.k <= 16) launch_fill<IdT, PtrT, TableT, 16>(cur, prev, surplus, clear_begin, clear_n16, table, indptr, indices, replace, rng_seed, st);
    else if (cur.k <= 32) launch_fill<IdT, PtrT, TableT, 32>(cur, prev, surplus, clear_begin, clear_n16, table, indptr, indices, replace, rng_seed, st);
    else launch_fill<IdT, PtrT, TableT, 64>(cur, prev, surplus, clear_begin, clear_n16, table, indptr, indices, replace, rng_seed, st);
    DGS_LAUNCH_CHECK();

    if (cur.bucketed) {  // the picks' slot words hold ids so far: group them and find the first occurrences
      const int n_buckets = 1 << buckets.log_buckets;
      hipLaunchKernelGGL(bucket_sort_kernel<IdT>, dim3(capped_grid(buckets.tiles_max)), dim3(kBlock), 0, st, cur,
                         buckets);
      DGS_LAUNCH_CHECK();
      if (buckets.hashed)
        hipLaunchKernelGGL(bucket_first_hashed_kernel, dim3(capped_grid(n_buckets)), dim3(kHashBlock), 0, st, cur,
                           buckets);
      else
        hipLaunchKernelGGL(bucket_first_kernel, dim3(capped_grid(n_buckets)), dim3(kBlock), 0, st, cur, buckets);
      DGS_LAUNCH_CHECK();
    }

    const int64_t len_max = (h == 0 ? cur.s_max : 0) + cur.s_max * cur.k;
    const int64_t pos_tiles = (len_max + kPosTile - 1) / kPosTile;
    const int64_t row_tiles = (cur.s_max + kRowTile - 1) / kRowTile;
    if (is_capped(pos_tiles + row_tiles))
      hipLaunchKernelGGL((hop_flag_kernel<IdT, TableT, true>), dim3(capped_grid(pos_tiles + row_tiles)),
                         dim3(kBlock), 0, st, cur, pos_tiles, row_tiles, table);
    else
      hipLaunchKernelGGL((hop_flag_kernel<IdT, TableT, false>), dim3(capped_grid(pos_tiles + row_tiles)),
                         dim3(kBlock), 0, st, cur, pos_tiles, row_tiles, table);
    DGS_LAUNCH_CHECK();
    if (cur.pos_off) {
      hipLaunchKernelGGL(pos_scan_kernel, dim3(1), dim3(1024), 0, st, cur);
      DGS_LAUNCH_CHECK();
    }
    if (cur.tile_off) {
      hipLaunchKernelGGL(tile_scan_kernel, dim3(1), dim3(1024), 0, st, cur);
      DGS_LAUNCH_CHECK();
    }
    const int64_t compact_blocks = pos_tiles > 0 ? pos_tiles : 1;  // block 0 always writes the lengths
    if (is_capped(compact_blocks))
      hipLaunchKernelGGL((hop_compact_kernel<IdT, TableT, true>), dim3(capped_grid(compact_blocks)), dim3(kBlock),
                         0, st, cur, compact_blocks, pos_tiles, row_tiles, table);
    else
      hipLaunchKernelGGL((hop_compact_kernel<IdT, TableT, false>), dim3(capped_grid(compact_blocks)), dim3(kBlock),
                         0, st, cur, compact_blocks, pos_tiles, row_tiles, table);
    DGS_LAUNCH_CHECK();
  }
  // every length is final here: mark the point the caller may wait for
  if (sizes_ticket) {
    const dgs_status ts = dgs_ticket_record(st, sizes_ticket);
    if (ts != DGS_OK) return ts;
  }
  launch_relabel<IdT>(hops[p.n_hops - 1], table, st);
  DGS_LAUNCH_CHECK();
  return DGS_OK;
}

template <typename IdT, typename PtrT>
dgs_status run_blocks_table(const Plan& p, Hop* hops, const Buckets& buckets, void* hash_table, void* node_table,
                            uint32_t epoch, const dgs_view& indptr, const dgs_view& indices, const dgs_view* probs,
                            bool replace, uint64_t rng_seed, void** sizes_ticket, hipStream_t st) {
  if (p.kind == TableKind::kDirect)
    return run_blocks<IdT, PtrT, DirectTable<IdT>>(p, hops, buckets, DirectTable<IdT>(node_table, epoch, uint32_t(indptr.total - 1)),
                                                   indptr, indices, probs, replace, rng_seed, sizes_ticket, st);
  const int64_t n16 = int64_t(p.table_bytes / 16);
  hipLaunchKernelGGL(clear_kernel, dim3(capped_grid((n16 + kBlock - 1) / kBlock)), dim3(kBlock), 0, st,
                     static_cast<uint4*>(hash_table), n16);
  DGS_LAUNCH_CHECK();
  if (p.kind == TableKind::kPacked)
    return run_blocks<IdT, PtrT, Table<IdT, true>>(p, hops, buckets, Table<IdT, true>(hash_table, p.capacity), indptr,
                                                   indices, probs, replace, rng_seed, sizes_ticket, st);
  return run_blocks<IdT, PtrT, Table<IdT, false>>(p, hops, buckets, Table<IdT, false>(hash_table, p.capacity), indptr,
                                                  indices, probs, replace, rng_seed, sizes_ticket, st);
}

}  // namespace
}  // namespace dgs

DGS_API dgs_status dgs_sample_blocks_plan(int64_t n_seeds, const int64_t* fanouts, int32_t n_hops,
                                          int64_t* seeds_max, int64_t* edges_max) {
  dgs::Plan p;
  dgs_status s = dgs::make_plan(n_seeds, fanouts, n_hops, 8, -1, false, &p);
  if (s != DGS_OK) return s;
  DGS_REQUIRE(seeds_max && edges_max, DGS_ERR_INVALID, "sample_blocks_plan: null output");
  for (int h = 0; h <= n_hops; ++h) seeds_max[h] = p.s_max[h];
  for (int h = 0; h < n_hops; ++h) edges_max[h] = p.nnz_max[h];
  return DGS_OK;
}

DGS_API size_t dgs_sample_blocks_workspace_bytes(int64_t n_seeds, const int64_t* fanouts, int32_t n_hops,
                                                 int32_t id_bytes) {
  dgs::Plan p;
  // sized for the split hash table, the largest of the layouts
  if (dgs::make_plan(n_seeds, fanouts, n_hops, id_bytes, -1, false, &p) != DGS_OK) return 0;
  p.kind = dgs::TableKind::kSplit;
  p.table_bytes = size_t(p.capacity) * (size_t(id_bytes) + 4);
  return dgs::layout(p, fanouts, nullptr, nullptr, nullptr);
}

DGS_API size_t dgs_node_table_bytes(int64_t n_nodes) {
  return n_nodes > 0 && n_nodes < 0x7fffffffLL ? size_t(n_nodes) * 8 : 0;
}

DGS_API size_t dgs_sample_blocks_weighted_workspace_bytes(int64_t n_seeds, const int64_t* fanouts, int32_t n_hops,
                                                          int32_t id_bytes) {
  dgs::Plan p;
  // sized for the split hash table, the largest of the layouts (used when there is no node table)
  if (dgs::make_plan(n_seeds, fanouts, n_hops, id_bytes, -1, false, &p) != DGS_OK) return 0;
  p.kind = dgs::TableKind::kSplit;
  p.table_bytes = size_t(p.capacity) * (size_t(id_bytes) + 4);
  p.weighted = true;
  return dgs::layout(p, fanouts, nullptr, nullptr, nullptr);
}

namespace {
dgs_status sample_blocks_entry(const void* seeds, int32_t id_bytes, int64_t n_seeds, dgs_view indptr,
                               dgs_view indices, const dgs_view* probs, const int64_t* fanouts, int32_t n_hops,
                               int32_t replace, uint64_t rng_seed, uint32_t first_stream, void* node_table,
                               uint32_t node_table_epoch, void* frontier, const dgs_block_out* outs,
                               int64_t* sizes_dev, int64_t* sizes_host, void** sizes_ticket, void* workspace,
                               size_t workspace_bytes, void* stream) {
  using namespace dgs;
  Plan p;
  // node count = indptr entries - 1
  dgs_status s = make_plan(n_seeds, fanouts, n_hops, id_bytes, indptr.total - 1, node_table != nullptr, &p);
  if (s != DGS_OK) return s;
  if (probs != nullptr) {
    DGS_REQUIRE(probs->elem_bytes == 4 && probs->total == indices.total, DGS_ERR_INVALID,
                "sample_blocks_weighted: %lld weights of %d bytes for %lld edges (float32, one per edge)",
                (long long)probs->total, probs->elem_bytes, (long long)indices.total);
    p.weighted = true;
    // weighted picks: the fill is bound by the races, not by its atomics, and the bucketed pass
    // changes the step by a per cent either way (measured with three and four batches in flight)
    if (debug_option(DGS_DEBUG_SAMPLER_BUCKETED) < 2) p.bucketed = false;
  }
  const size_t need = probs != nullptr ? dgs_sample_blocks_weighted_workspace_bytes(n_seeds, fanouts, n_hops, id_bytes)
                                       : dgs_sample_blocks_workspace_bytes(n_seeds, fanouts, n_hops, id_bytes);
  DGS_REQUIRE(width_ok(indptr.elem_bytes), DGS_ERR_INVALID, "sample_blocks: indptr width %d", indptr.elem_bytes);
  DGS_REQUIRE(indices.elem_bytes == id_bytes, DGS_ERR_INVALID,
              "sample_blocks: indices width %d differs from the seed width %d", indices.elem_bytes, id_bytes);
  DGS_REQUIRE(outs != nullptr && sizes_dev != nullptr, DGS_ERR_INVALID, "sample_blocks: null output");
  DGS_REQUIRE(node_table == nullptr || (node_table_epoch >= 1 && node_table_epoch < 0xfffffff0u), DGS_ERR_INVALID,
              "sample_blocks: node table epoch %u outside 1..2^32-17 (refill the table with 0xFF and restart at 1)",
              node_table_epoch);
  DGS_REQUIRE(sizes_ticket == nullptr || sizes_host != nullptr, DGS_ERR_INVALID,
              "sample_blocks: a sizes_ticket needs sizes_host");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (n_seeds == 0) {  // nothing to launch: every size is zero
    // a fill kernel, not a memset node: the call may be recorded into a graph
    hipLaunchKernelGGL(zero_sizes_kernel, dim3(1), dim3(64), 0, st, sizes_dev, 3 * n_hops + 1);
    DGS_LAUNCH_CHECK();
    if (sizes_host)
      for (int i = 0; i < 3 * n_hops + 1; ++i) sizes_host[i] = 0;
    return sizes_ticket ? dgs_ticket_record(st, sizes_ticket) : DGS_OK;
  }
  DGS_REQUIRE(seeds != nullptr && frontier != nullptr, DGS_ERR_INVALID, "sample_blocks: null seeds or frontier");
  DGS_REQUIRE(workspace != nullptr && workspace_bytes >= need, DGS_ERR_WORKSPACE,
              "sample_blocks: workspace of %zu B, need %zu", workspace_bytes, need);
  DGS_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255) == 0, DGS_ERR_WORKSPACE,
              "sample_blocks: workspace must be 256-byte aligned");
  Hop hops[DGS_MAX_HOPS];
  void* hash_table = nullptr;
  Buckets buckets{};
  layout(p, fanouts, workspace, hops, &hash_table, &buckets);
  for (int h = 0; h < n_hops; ++h) {
    Hop& t = hops[h];
    DGS_REQUIRE(p.nnz_max[h] == 0 || (outs[h].src_local && outs[h].dst_local), DGS_ERR_INVALID,
                "sample_blocks: null edge buffers for hop %d", h);
    t.seeds = h == 0 ? seeds : frontier;
    t.n_seeds = sizes_dev + h;
    t.n_seeds_host = h == 0 ? n_seeds : -1;
    t.n_seeds_out = h == 0 ? sizes_dev : nullptr;
    t.prev_nnz = sizes_dev + n_hops + (h == 0 ? 1 : h);  // edges of hop h - 1 (hop 0: any readable word)
    t.prev_n_seeds = sizes_dev + (h == 0 ? 0 : h - 1);
    t.n_unique = sizes_dev + h + 1;
    t.nnz = sizes_dev + n_hops + 1 + h;
    t.flags = sizes_dev + 2 * n_hops + 1 + h;
    t.host_sizes = sizes_host;
    t.n_hops = n_hops;
    t.frontier = frontier;
    t.src_local = outs[h].src_local;
    t.dst_local = outs[h].dst_local;
    t.rng_stream = first_stream + uint32_t(h);
  }
  const bool rep = replace != 0;
  if (id_bytes == 8)
    return indptr.elem_bytes == 8
               ? run_blocks_table<int64_t, int64_t>(p, hops, buckets, hash_table, node_table, node_table_epoch, indptr, indices, probs, rep, rng_seed, sizes_ticket, st)
               : run_blocks_table<int64_t, int32_t>(p, hops, buckets, hash_table, node_table, node_table_epoch, indptr, indices, probs, rep, rng_seed, sizes_ticket, st);
  return indptr.elem_bytes == 8
             ? run_blocks_table<int32_t, int64_t>(p, hops, buckets, hash_table, node_table, node_table_epoch, indptr, indices, probs, rep, rng_seed, sizes_ticket, st)
             : run_blocks_table<int32_t, int32_t>(p, hops, buckets, hash_table, node_table, node_table_epoch, indptr, indices, probs, rep, rng_seed, sizes_ticket, st);
}
}  // namespace

DGS_API dgs_status dgs_sample_blocks(const void* seeds, int32_t id_bytes, int64_t n_seeds, dgs_view indptr,
                                     dgs_view indices, const int64_t* fanouts, int32_t n_hops, int32_t replace,
                                     uint64_t rng_seed, uint32_t first_stream, void* node_table,
                                     uint32_t node_table_epoch, void* frontier, const dgs_block_out* outs,
                                     int64_t* sizes_dev, int64_t* sizes_host, void** sizes_ticket,
                                     void* workspace, size_t workspace_bytes, void* stream) {
  return sample_blocks_entry(seeds, id_bytes, n_seeds, indptr, indices, nullptr, fanouts, n_hops, replace, rng_seed,
                             first_stream, node_table, node_table_epoch, frontier, outs, sizes_dev, sizes_host,
                             sizes_ticket, workspace, workspace_bytes, stream);
}

DGS_API dgs_status dgs_sample_blocks_weighted(const void* seeds, int32_t id_bytes, int64_t n_seeds, dgs_view indptr,
                                              dgs_view indices, dgs_view probs, const int64_t* fanouts,
                                              int32_t n_hops, int32_t replace, uint64_t rng_seed,
                                              uint32_t first_stream, void* node_table, uint32_t node_table_epoch,
                                              void* frontier, const dgs_block_out* outs, int64_t* sizes_dev,
                                              int64_t* sizes_host, void** sizes_ticket, void* workspace,
                                              size_t workspace_bytes, void* stream) {
  return sample_blocks_entry(seeds, id_bytes, n_seeds, indptr, indices, &probs, fanouts, n_hops, replace, rng_seed,
                             first_stream, node_table, node_table_epoch, frontier, outs, sizes_dev, sizes_host,
                             sizes_ticket, workspace, workspace_bytes, stream);
}
