// Row gather from a two-tier store, and the tier partition of an index list.
//
// The gather is a pure byte mover: rows are cut into chunks of VEC bytes
// (16 when sizes and addresses allow) and the (row, chunk) space is flattened,
// so a wavefront always issues 64 full-width loads and 64 contiguous stores no
// matter how the row length relates to 64 lanes (a 400-byte row is 25 chunks,
// so one wave covers 2.56 rows).  VEC divides both the row size and the byte
// offset of the device/host boundary, hence no chunk ever straddles the tiers
// and a straddling ROW is still resolved exactly, chunk by chunk.
//
// Index values are checked before they address anything: a row outside the rows the
// requested tier holds is not read, its output row is filled with zero bytes and the
// caller's flag word (if any) is set.
#include "common.h"

namespace dgs {
namespace {

constexpr int kGatherThreads = 256;
constexpr int kGatherUnroll = 3;  // chunks in flight per thread: 2 to 4 measure within 2 % of each other
constexpr int kChunksPerBlock = kGatherThreads * kGatherUnroll;
// largest chunks-per-row for which the multiply-high division below is exact
constexpr uint32_t kMaxFlatChunksPerRow = 32768;
// A launch sized for a worst-case row count (dgs_gather_rows_dyn) is capped at this many blocks;
// blocks stride over the tiles, so a mostly unused worst case does not cost 10^5 empty blocks.
constexpr int64_t kMaxDynGrid = 32768;
constexpr int kGatherBlocksPerCu = 8;  // what fits by registers and wave slots when nothing is reserved

// LDS of one CU on the current device (160 KB on gfx950); asked once per process.
inline int64_t lds_per_cu() {
  static const int64_t bytes = [] {
    int dev = 0, per_cu = 0, per_block = 0;
    if (hipGetDevice(&dev) != hipSuccess) return int64_t(65536);
    if (hipDeviceGetAttribute(&per_cu, hipDeviceAttributeMaxSharedMemoryPerMultiprocessor, dev) != hipSuccess) per_cu = 0;
    if (hipDeviceGetAttribute(&per_block, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) != hipSuccess) per_block = 0;
    const int64_t most = per_cu > per_block ? per_cu : per_block;
    return most > 0 ? most : int64_t(65536);
  }();
  return bytes;
}

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
template <int VEC> struct Chunk;
template <> struct Chunk<16> { using type = u32x4; };
template <> struct Chunk<8> { using type = u32x2; };
template <> struct Chunk<4> { using type = uint32_t; };
template <> struct Chunk<2> { using type = uint16_t; };
template <> struct Chunk<1> { using type = uint8_t; };

template <int TIER>
__device__ __forceinline__ const char* resolve(const char* dev, const char* host, int64_t thr_bytes,
                                               int64_t g) {
  if (TIER == DGS_TIER_DEVICE) return dev + g;
  if (TIER == DGS_TIER_HOST) return host + (g - thr_bytes);
  return g < thr_bytes ? dev + g : host + (g - thr_bytes);
}

// One block moves kChunksPerBlock consecutive output chunks.
// chunk c -> row c / cpr, column c % cpr; the division runs on a block-local
// 32-bit offset with a precomputed reciprocal (exact while
// (cpr + kChunksPerBlock) * cpr < 2^32, guaranteed by kMaxFlatChunksPerRow).
// Rows [row_lo, row_hi) are the ones the launch may read; the range is not empty.
//
// The kChunksPerBlock output chunks from chunk c0 on; returns whether an index outside
// [row_lo, row_hi) was met.
// Three passes, each over all of the thread's chunks, so that nothing but the row ids, then
// nothing but the chunks themselves, is alive across the waits: the row ids (all requested
// before any is used), the loads, the stores.
// `readable_chunks` bounds the ids that may be read (the index array holds that many rows' ids
// whatever the count turns out to be); the number of chunks that count is `total_chunks`, or, when
// `n_rows_dev` is given, is read from the device here, together with the ids: a block of a launch
// that is about as large as the work does not wait for the count before it asks for its ids.
template <int VEC, int TIER, typename IndexT>
__device__ __forceinline__ bool gather_tile(const char* __restrict__ dev, const char* __restrict__ host,
                                            int64_t thr_bytes, int64_t row_bytes, uint32_t cpr, uint32_t magic,
                                            const IndexT* __restrict__ index, int64_t readable_chunks,
                                            int64_t total_chunks, const int64_t* __restrict__ n_rows_dev,
                                            int64_t row_lo, int64_t row_hi, char* __restrict__ out, int64_t c0,
                                            int64_t* counted_chunks) {
  using C = typename Chunk<VEC>::type;
  bool bad = false;
  const int64_t row0 = c0 / cpr;
  const uint32_t rem0 = uint32_t(c0 - row0 * cpr);
  const IndexT* __restrict__ index0 = index + row0;
  int64_t src[kGatherUnroll];
  uint32_t off[kGatherUnroll];  // byte offset of the chunk inside its row
#pragma unroll
  for (int u = 0; u < kGatherUnroll; ++u) {
    const uint32_t t = u * kGatherThreads + threadIdx.x;
    const uint32_t lc = rem0 + t;
    const uint32_t q = cpr == 1 ? lc : __umulhi(lc, magic);
    off[u] = (lc - q * cpr) * uint32_t(VEC);
    src[u] = c0 + t < readable_chunks ? int64_t(index0[q]) : row_lo;  // past the end: some row, never stored
  }
  if (n_rows_dev) {  // row count decided on the device; one that exceeds the output's rows gathers nothing
    const int64_t rows = *n_rows_dev;
    total_chunks = rows >= 0 && rows * cpr <= readable_chunks ? rows * cpr : 0;
  }
  *counted_chunks = total_chunks;
  if (c0 >= total_chunks) return false;  // whole blocks leave together
  // An id outside [row_lo, row_hi) is replaced by row_lo before it addresses anything (the
  // launcher guarantees that row_lo is a row the tier holds), and what was read for it is
  // dropped: no branch around the loads, so all of them are in flight together.  The same goes
  // for the ids behind the last chunk that counts (whatever the index array holds there).
  C val[kGatherUnroll];
  bool in_range[kGatherUnroll];
#pragma unroll
  for (int u = 0; u < kGatherUnroll; ++u) {
    const bool counts = c0 + u * kGatherThreads + threadIdx.x < total_chunks;
    in_range[u] = src[u] >= row_lo && src[u] < row_hi;
    if (!in_range[u] || !counts) {
      src[u] = row_lo;
      bad |= counts;
    }
    const int64_t g = src[u] * row_bytes + int64_t(off[u]);
    val[u] = *reinterpret_cast<const C*>(resolve<TIER>(dev, host, thr_bytes, g));
  }
#pragma unroll
  for (int u = 0; u < kGatherUnroll; ++u)
    if (!in_range[u]) val[u] = C(0);
  char* __restrict__ o = out + (c0 + threadIdx.x) * VEC;
#pragma unroll
  for (int u = 0; u < kGatherUnroll; ++u) {
    if (c0 + u * kGatherThreads + threadIdx.x < total_chunks)
      __builtin_nontemporal_store(val[u], reinterpret_cast<C*>(o + int64_t(u) * kGatherThreads * VEC));
  }
  return bad;
}

// STRIDE: the grid is smaller than the tile count (a launch sized for fewer rows than the output
// holds) and blocks stride over the tiles; otherwise a block has exactly one tile and no loop in
// its instruction stream.  `total_chunks` is the launch's worst case: what the index array and the
// output hold.
template <int VEC, int TIER, typename IndexT, bool STRIDE>
__global__ __launch_bounds__(kGatherThreads) void gather_flat_kernel(
    const char* __restrict__ dev, const char* __restrict__ host, int64_t thr_bytes,
    int64_t row_bytes, uint32_t cpr, uint32_t magic, const IndexT* __restrict__ index,
    int64_t total_chunks, const int64_t* __restrict__ n_rows_dev, int64_t row_lo, int64_t row_hi,
    int64_t* __restrict__ bad_index, char* __restrict__ out) {
  const int64_t first = int64_t(blockIdx.x) * kChunksPerBlock;
  if (first >= total_chunks) return;
  int64_t counted;
  bool bad = gather_tile<VEC, TIER, IndexT>(dev, host, thr_bytes, row_bytes, cpr, magic, index, total_chunks,
                                            total_chunks, n_rows_dev, row_lo, row_hi, out, first, &counted);
  if (STRIDE) {  // the count is known from here on
    for (int64_t c0 = first + int64_t(gridDim.x) * kChunksPerBlock; c0 < counted;
         c0 += int64_t(gridDim.x) * kChunksPerBlock) {
      int64_t unused;
      bad |= gather_tile<VEC, TIER, IndexT>(dev, host, thr_bytes, row_bytes, cpr, magic, index, counted, counted,
                                            nullptr, row_lo, row_hi, out, c0, &unused);
    }
  }
  if (bad && bad_index) *bad_index = 1;
}

// Rows wider than kMaxFlatChunksPerRow chunks, and any launch whose tier holds no whole row
// (every id is refused): a block owns one segment of kChunksPerBlock chunks of one row.
template <int VEC, int TIER, typename IndexT>
__global__ __launch_bounds__(kGatherThreads) void gather_wide_kernel(
    const char* __restrict__ dev, const char* __restrict__ host, int64_t thr_bytes,
    int64_t row_bytes, int64_t cpr, int64_t blocks_per_row, const IndexT* __restrict__ index,
    int64_t n_max, const int64_t* __restrict__ n_rows_dev, int64_t row_lo, int64_t row_hi,
    int64_t* __restrict__ bad_index, char* __restrict__ out) {
  using C = typename Chunk<VEC>::type;
  const int64_t row = int64_t(blockIdx.x) / blocks_per_row;
  if (n_rows_dev && (row >= *n_rows_dev || *n_rows_dev > n_max)) return;
  const int64_t seg = int64_t(blockIdx.x) - row * blocks_per_row;
  const int64_t src_row = int64_t(index[row]);
  const bool in_range = src_row >= row_lo && src_row < row_hi;
  if (!in_range && bad_index && threadIdx.x == 0) *bad_index = 1;
#pragma unroll
  for (int u = 0; u < kGatherUnroll; ++u) {
    const int64_t col = seg * kChunksPerBlock + u * kGatherThreads + threadIdx.x;
    if (col < cpr) {
      C v = C(0);
      if (in_range) {
        const int64_t g = src_row * row_bytes + col * VEC;
        v = *reinterpret_cast<const C*>(resolve<TIER>(dev, host, thr_bytes, g));
      }
      *reinterpret_cast<C*>(out + row * row_bytes + col * VEC) = v;
    }
  }
}

template <int VEC, int TIER, typename IndexT>
dgs_status launch_gather(const dgs_view& v, int64_t row_bytes, const void* index, int64_t n,
                         const int64_t* n_dev, int64_t n_expected, int32_t blocks_per_cu, int64_t* bad_index, void* out, hipStream_t st) {
  const int64_t cpr = row_bytes / VEC;
  const int64_t thr_bytes = v.threshold * v.elem_bytes;
  // rows the tier holds whole: the device tier the rows that end at or before the boundary, the
  // host tier the rows that begin at or after it (a straddling row is served by the "any" kernel)
  const int64_t n_rows = v.total * v.elem_bytes / row_bytes;
  const int64_t row_lo = TIER == DGS_TIER_HOST ? (thr_bytes + row_bytes - 1) / row_bytes : 0;
  const int64_t row_hi = TIER == DGS_TIER_DEVICE ? thr_bytes / row_bytes : n_rows;
  const char* dev = static_cast<const char*>(v.dev);
  const char* host = static_cast<const char*>(v.host);
  if (cpr <= kMaxFlatChunksPerRow && row_lo < row_hi) {
    const int64_t total_chunks = n * cpr;
    const int64_t tiles = (total_chunks + kChunksPerBlock - 1) / kChunksPerBlock;
    int64_t blocks = tiles;
    if (n_dev != nullptr) {
      // a count read on the device: the launch is sized for the rows the caller expects (all of
      // them when it says nothing), and blocks stride should there be more
      if (n_expected > 0 && n_expected < n) blocks = (n_expected * cpr + kChunksPerBlock - 1) / kChunksPerBlock;
      if (blocks > kMaxDynGrid) blocks = kMaxDynGrid;
      if (blocks > tiles) blocks = tiles;
    }
    if (blocks > 0x7fffffff) blocks = 0x7fffffff;
    const uint32_t magic = cpr > 1 ? uint32_t((uint64_t(1) << 32) / uint64_t(cpr)) + 1u : 0u;
    // LDS that the kernel does not use, reserved so that fewer of its blocks fit a CU: a caller's
    // limit (dgs_gather_rows_dyn_shared), or the measurement hook's byte count
    int64_t lds = debug_option(DGS_DEBUG_GATHER_LDS_BYTES);
    if (lds <= 0 && blocks_per_cu > 0 && blocks_per_cu < kGatherBlocksPerCu) lds = lds_per_cu() / blocks_per_cu / 256 * 256;
    lds = lds < 0 ? 0 : (lds > 65536 ? 65536 : lds);
    if (blocks < tiles)
      hipLaunchKernelGGL((gather_flat_kernel<VEC, TIER, IndexT, true>), dim3(uint32_t(blocks)),
                         dim3(kGatherThreads), uint32_t(lds), st, dev, host, thr_bytes, row_bytes, uint32_t(cpr),
                         magic, static_cast<const IndexT*>(index), total_chunks, n_dev, row_lo, row_hi,
                         bad_index, static_cast<char*>(out));
    else
      hipLaunchKernelGGL((gather_flat_kernel<VEC, TIER, IndexT, false>), dim3(uint32_t(blocks)),
                         dim3(kGatherThreads), uint32_t(lds), st, dev, host, thr_bytes, row_bytes, uint32_t(cpr),
                         magic, static_cast<const IndexT*>(index), total_chunks, n_dev, row_lo, row_hi,
                         bad_index, static_cast<char*>(out));
  } else {
    const int64_t bpr = (cpr + kChunksPerBlock - 1) / kChunksPerBlock;
    DGS_REQUIRE(n * bpr <= 0x7fffffff, DGS_ERR_UNSUPPORTED, "gather: %lld rows of %lld B exceed one launch",
                (long long)n, (long long)row_bytes);
    hipLaunchKernelGGL((gather_wide_kernel<VEC, TIER, IndexT>), dim3(uint32_t(n * bpr)),
                       dim3(kGatherThreads), 0, st, dev, host, thr_bytes, row_bytes, cpr, bpr,
                       static_cast<const IndexT*>(index), n, n_dev, row_lo, row_hi, bad_index,
                       static_cast<char*>(out));
  }
  DGS_LAUNCH_CHECK();
  return DGS_OK;
}

template <int VEC, int TIER>
dgs_status dispatch_index(const dgs_view& v, int64_t row_bytes, const void* index,
                          int32_t index_bytes, int64_t n, const int64_t* n_dev, int64_t n_expected, int32_t blocks_per_cu, int64_t* bad,
                          void* out, hipStream_t st) {
  return index_bytes == 8 ? launch_gather<VEC, TIER, int64_t>(v, row_bytes, index, n, n_dev, n_expected, blocks_per_cu, bad, out, st)
                          : launch_gather<VEC, TIER, int32_t>(v, row_bytes, index, n, n_dev, n_expected, blocks_per_cu, bad, out, st);
}

template <int TIER>
dgs_status dispatch_vec(int vec, const dgs_view& v, int64_t row_bytes, const void* index,
                        int32_t index_bytes, int64_t n, const int64_t* n_dev, int64_t n_expected, int32_t blocks_per_cu, int64_t* bad,
                        void* out, hipStream_t st) {
  switch (vec) {
    case 16: return dispatch_index<16, TIER>(v, row_bytes, index, index_bytes, n, n_dev, n_expected, blocks_per_cu, bad, out, st);
    case 8: return dispatch_index<8, TIER>(v, row_bytes, index, index_bytes, n, n_dev, n_expected, blocks_per_cu, bad, out, st);
    case 4: return dispatch_index<4, TIER>(v, row_bytes, index, index_bytes, n, n_dev, n_expected, blocks_per_cu, bad, out, st);
    case 2: return dispatch_index<2, TIER>(v, row_bytes, index, index_bytes, n, n_dev, n_expected, blocks_per_cu, bad, out, st);
    default: return dispatch_index<1, TIER>(v, row_bytes, index, index_bytes, n, n_dev, n_expected, blocks_per_cu, bad, out, st);
  }
}

// Largest power of two <= 16 dividing every quantity that decides chunk alignment.
int pick_vec(const dgs_view& v, int64_t row_bytes, const void* out, int tier) {
  uint64_t bits = uint64_t(row_bytes) | uint64_t(reinterpret_cast<uintptr_t>(out));
  const bool dev_used = tier != DGS_TIER_HOST && v.threshold > 0;
  const bool host_used = tier != DGS_TIER_DEVICE && v.threshold < v.total;
  if (dev_used) bits |= uint64_t(reinterpret_cast<uintptr_t>(v.dev));
  if (host_used) {
    bits |= uint64_t(reinterpret_cast<uintptr_t>(v.host));
    bits |= uint64_t(v.threshold) * uint64_t(v.elem_bytes);  // offset of the boundary
  }
  int vec = 16;
  while (vec > 1 && (bits & uint64_t(vec - 1))) vec >>= 1;
  return vec;
}

// ---- split_index ----------------------------------------------------------------
constexpr int kSplitThreads = 256;
constexpr int kSplitItems = 4;  // ids per thread
constexpr int kSplitTile = kSplitThreads * kSplitItems;

// Pass 1: per-tile count of host-resident ids.
template <typename IndexT>
__global__ __launch_bounds__(kSplitThreads) void split_count_kernel(
    const IndexT* __restrict__ index, int64_t n, int64_t first_host_row, int* __restrict__ tile_host) {
  __shared__ int lds[kSplitThreads / kWave + 1];
  const int64_t base = int64_t(blockIdx.x) * kSplitTile + threadIdx.x * kSplitItems;
  int c = 0;
#pragma unroll
  for (int j = 0; j < kSplitItems; ++j)
    if (base + j < n && int64_t(index[base + j]) >= first_host_row) ++c;
  int total;
  block_exclusive_scan<kSplitThreads>(c, &total, lds);
  if (threadIdx.x == 0) tile_host[blockIdx.x] = total;
}

// Pass 2 (one block): exclusive scan of the tile counts, totals to counts_dev.
__global__ __launch_bounds__(1024) void split_scan_kernel(const int* __restrict__ tile_host,
                                                          int64_t* __restrict__ tile_host_off,
                                                          int64_t tiles, int64_t n,
                                                          int64_t* __restrict__ counts_dev) {
  __shared__ int lds[1024 / kWave + 1];
  __shared__ int64_t carry;
  if (threadIdx.x == 0) carry = 0;
  __syncthreads();
  for (int64_t t0 = 0; t0 < tiles; t0 += 1024) {
    const int64_t t = t0 + threadIdx.x;
    const int v = t < tiles ? tile_host[t] : 0;
    int total;
    const int ex = block_exclusive_scan<1024>(v, &total, lds);
    if (t < tiles) tile_host_off[t] = carry + ex;
    __syncthreads();
    if (threadIdx.x == 0) carry += total;
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    counts_dev[0] = n - carry;
    counts_dev[1] = carry;
  }
}

// Pass 3: stable scatter.  An id at position p with h host ids before it goes to
// out_host[h] or out_local[p - h].
template <typename IndexT>
__global__ __launch_bounds__(kSplitThreads) void split_scatter_kernel(
    const IndexT* __restrict__ index, int64_t n, int64_t first_host_row,
    const int64_t* __restrict__ tile_host_off, IndexT* __restrict__ out_local,
    IndexT* __restrict__ out_host) {
  __shared__ int lds[kSplitThreads / kWave + 1];
  const int64_t base = int64_t(blockIdx.x) * kSplitTile + threadIdx.x * kSplitItems;
  IndexT id[kSplitItems];
  bool is_host[kSplitItems];
  int c = 0;
#pragma unroll
  for (int j = 0; j < kSplitItems; ++j) {
    is_host[j] = false;
    if (base + j < n) {
      id[j] = index[base + j];
      is_host[j] = int64_t(id[j]) >= first_host_row;
      c += is_host[j];
    }
  }
  int total;
  int64_t h = tile_host_off[blockIdx.x] + block_exclusive_scan<kSplitThreads>(c, &total, lds);
#pragma unroll
  for (int j = 0; j < kSplitItems; ++j) {
    if (base + j < n) {
      if (is_host[j]) out_host[h++] = id[j];
      else out_local[base + j - h] = id[j];
    }
  }
}

}  // namespace
}  // namespace dgs

namespace {
dgs_status gather_entry(dgs_view v, int64_t row_elems, const void* index, int32_t index_bytes, int64_t n,
                        const int64_t* n_dev, int64_t n_expected, int32_t blocks_per_cu, void* out, int32_t tier, int64_t* bad,
                        void* stream) {
  using namespace dgs;
  DGS_REQUIRE(width_ok(index_bytes), DGS_ERR_INVALID, "gather: index width %d is not 4 or 8", index_bytes);
  DGS_REQUIRE(n >= 0 && row_elems > 0, DGS_ERR_INVALID, "gather: n=%lld row_elems=%lld", (long long)n,
              (long long)row_elems);
  DGS_REQUIRE(v.elem_bytes == 1 || v.elem_bytes == 2 || v.elem_bytes == 4 || v.elem_bytes == 8,
              DGS_ERR_INVALID, "gather: element width %d", v.elem_bytes);
  DGS_REQUIRE(tier >= DGS_TIER_ANY && tier <= DGS_TIER_HOST, DGS_ERR_INVALID, "gather: tier %d", tier);
  DGS_REQUIRE(v.threshold >= 0 && v.threshold <= v.total, DGS_ERR_INVALID, "gather: bad view");
  if (n == 0) return DGS_OK;
  DGS_REQUIRE(index != nullptr && out != nullptr, DGS_ERR_INVALID, "gather: null pointer");
  // an "any" gather over a single-tier store needs no per-chunk test
  if (tier == DGS_TIER_ANY && v.threshold == v.total) tier = DGS_TIER_DEVICE;
  if (tier == DGS_TIER_ANY && v.threshold == 0) tier = DGS_TIER_HOST;
  // A row that straddles the boundary is listed as a host row by dgs_split_index; it begins in
  // the device slice, so the host-only address arithmetic would reach in front of the host slice
  // (as upstream's HostAt does, src/chunk_tensor.h:56-58).  Such a store is served chunk by chunk.
  if (tier == DGS_TIER_HOST && v.threshold > 0 && v.threshold % row_elems != 0) tier = DGS_TIER_ANY;
  DGS_REQUIRE(tier == DGS_TIER_HOST || v.dev != nullptr, DGS_ERR_INVALID, "gather: store has no device slice");
  DGS_REQUIRE(tier == DGS_TIER_DEVICE || v.host != nullptr, DGS_ERR_INVALID, "gather: store has no host slice");
  const int64_t row_bytes = row_elems * v.elem_bytes;
  const int vec = pick_vec(v, row_bytes, out, tier);
  hipStream_t st = static_cast<hipStream_t>(stream);
  switch (tier) {
    case DGS_TIER_DEVICE: return dispatch_vec<DGS_TIER_DEVICE>(vec, v, row_bytes, index, index_bytes, n, n_dev, n_expected, blocks_per_cu, bad, out, st);
    case DGS_TIER_HOST: return dispatch_vec<DGS_TIER_HOST>(vec, v, row_bytes, index, index_bytes, n, n_dev, n_expected, blocks_per_cu, bad, out, st);
    default: return dispatch_vec<DGS_TIER_ANY>(vec, v, row_bytes, index, index_bytes, n, n_dev, n_expected, blocks_per_cu, bad, out, st);
  }
}
}  // namespace

DGS_API dgs_status dgs_gather_rows(dgs_view v, int64_t row_elems, const void* index,
                                   int32_t index_bytes, int64_t n, void* out, int32_t tier,
                                   int64_t* bad_index, void* stream) {
  return gather_entry(v, row_elems, index, index_bytes, n, nullptr, 0, 0, out, tier, bad_index, stream);
}

DGS_API dgs_status dgs_gather_rows_dyn(dgs_view v, int64_t row_elems, const void* index,
                                       int32_t index_bytes, int64_t n_max, const int64_t* n_rows_dev,
                                       int64_t n_expected, void* out, int32_t tier, int64_t* bad_index,
                                       void* stream) {
  DGS_REQUIRE(n_rows_dev != nullptr, DGS_ERR_INVALID, "gather_dyn: null n_rows_dev");
  return gather_entry(v, row_elems, index, index_bytes, n_max, n_rows_dev, n_expected, 0, out, tier, bad_index, stream);
}

DGS_API dgs_status dgs_gather_rows_dyn_shared(dgs_view v, int64_t row_elems, const void* index,
                                              int32_t index_bytes, int64_t n_max, const int64_t* n_rows_dev,
                                              int64_t n_expected, void* out, int32_t tier, int32_t blocks_per_cu,
                                              int64_t* bad_index, void* stream) {
  DGS_REQUIRE(n_rows_dev != nullptr, DGS_ERR_INVALID, "gather_dyn_shared: null n_rows_dev");
  DGS_REQUIRE(blocks_per_cu >= 0, DGS_ERR_INVALID, "gather_dyn_shared: blocks_per_cu %d", blocks_per_cu);
  return gather_entry(v, row_elems, index, index_bytes, n_max, n_rows_dev, n_expected, blocks_per_cu, out, tier, bad_index,
                      stream);
}

DGS_API size_t dgs_split_index_workspace_bytes(int64_t n) {
  if (n < 0) n = 0;
  const size_t tiles = size_t((n + dgs::kSplitTile - 1) / dgs::kSplitTile);
  size_t used = dgs::carve_size(0, tiles * sizeof(int));
  return dgs::carve_size(used, tiles * sizeof(int64_t)) + 256;
}

DGS_API dgs_status dgs_split_index(dgs_view v, int64_t row_elems, const void* index,
                                   int32_t index_bytes, int64_t n, void* out_local, void* out_host,
                                   int64_t* counts_dev, void* workspace, size_t workspace_bytes,
                                   void* stream) {
  using namespace dgs;
  DGS_REQUIRE(width_ok(index_bytes), DGS_ERR_INVALID, "split_index: index width %d", index_bytes);
  DGS_REQUIRE(n >= 0 && row_elems > 0 && counts_dev != nullptr, DGS_ERR_INVALID, "split_index: bad argument");
  DGS_REQUIRE(workspace_bytes >= dgs_split_index_workspace_bytes(n) && workspace != nullptr,
              DGS_ERR_WORKSPACE, "split_index: workspace of %zu B, need %zu", workspace_bytes,
              dgs_split_index_workspace_bytes(n));
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int64_t tiles = (n + kSplitTile - 1) / kSplitTile;
  DGS_REQUIRE(tiles <= 0x7fffffff, DGS_ERR_UNSUPPORTED, "split_index: too many ids");
  const int64_t first_host_row = v.threshold / row_elems;
  Carver ws(workspace);
  int* tile_host = ws.take<int>(size_t(tiles));
  int64_t* tile_off = ws.take<int64_t>(size_t(tiles));
  if (tiles > 0) {
    DGS_REQUIRE(index && out_local && out_host, DGS_ERR_INVALID, "split_index: null pointer");
    if (index_bytes == 8)
      hipLaunchKernelGGL(split_count_kernel<int64_t>, dim3(uint32_t(tiles)), dim3(kSplitThreads), 0, st,
                         static_cast<const int64_t*>(index), n, first_host_row, tile_host);
    else
      hipLaunchKernelGGL(split_count_kernel<int32_t>, dim3(uint32_t(tiles)), dim3(kSplitThreads), 0, st,
                         static_cast<const int32_t*>(index), n, first_host_row, tile_host);
    DGS_LAUNCH_CHECK();
  }
  hipLaunchKernelGGL(split_scan_kernel, dim3(1), dim3(1024), 0, st, tile_host, tile_off, tiles, n, counts_dev);
  DGS_LAUNCH_CHECK();
  if (tiles > 0) {
    if (index_bytes == 8)
      hipLaunchKernelGGL(split_scatter_kernel<int64_t>, dim3(uint32_t(tiles)), dim3(kSplitThreads), 0, st,
                         static_cast<const int64_t*>(index), n, first_host_row, tile_off,
                         static_cast<int64_t*>(out_local), static_cast<int64_t*>(out_host));
    else
      hipLaunchKernelGGL(split_scatter_kernel<int32_t>, dim3(uint32_t(tiles)), dim3(kSplitThreads), 0, st,
                         static_cast<const int32_t*>(index), n, first_host_row, tile_off,
                         static_cast<int32_t*>(out_local), static_cast<int32_t*>(out_host));
    DGS_LAUNCH_CHECK();
  }
  return DGS_OK;
}
