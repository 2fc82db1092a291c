// First-occurrence unique + relabel of node ids.
//
// A linear-probing table in HBM (table.h: packed 64-bit slots, or id array + value array for
// 8-byte ids that may not fit 32 bits) maps each id to the smallest position at which it occurs.
// The atomic that inserts a position tells whether it is, so far, its id's smallest and which
// position it displaced (marked lost): a position is a "first occurrence" when it was smallest
// at insertion and never lost.  Flags are scanned tile by tile, first occurrences are compacted
// in input order (which is what makes the result independent of the table layout) and the
// table value becomes the id's rank.  Every mapping id remembers its slot, so a tensor that
// is both mapped and relabelled (the picked neighbours of the upstream sampler
// loop) is not probed a second time.
#include "common.h"
#include "table.h"

namespace dgs {
namespace {

constexpr int kThreads = 256;
constexpr int kItems = 4;
constexpr int kTileIds = kThreads * kItems;   // ids per block in flag / compact
constexpr uint32_t kFirstBit = 0x80000000u;   // marks a first occurrence in slot[]
constexpr int64_t kMaxMappingIds = int64_t(1) << 30;
// slot[] word of a mapping id the table could not take (the call's results are void then: the
// overflow word is set).  It lies beyond the mask of every table but the largest possible one
// (2^31 slots), where it names a real slot; lookup_kernel checks a word against the mask, and what
// the slot holds against the number of positions, before either is used as an index.
constexpr uint32_t kNoSlot = 0x7fffffffu;

// Element i of the logical concatenation, or of a single array when count == 1.
template <typename IdT>
__device__ __forceinline__ IdT seg_load(const dgs_segments& s, int64_t i) {
  const IdT* p = static_cast<const IdT*>(s.ptr[0]);
  int64_t j = i;
#pragma unroll
  for (int k = 1; k < DGS_MAX_SEGMENTS; ++k) {
    if (k < s.count && i >= s.len[k - 1]) {
      i -= s.len[k - 1];
      p = static_cast<const IdT*>(s.ptr[k]);
      j = i;
    } else {
      i = -1;  // stays negative: no later segment can match
    }
  }
  return p[j];
}

// Table bytes become 0xFF (empty slots), the lost marks and the overflow word 0.
__global__ __launch_bounds__(kThreads) void clear_kernel(uint4* __restrict__ table, int64_t table16,
                                                         uint4* __restrict__ zeros, int64_t zeros16) {
  const int64_t i = int64_t(blockIdx.x) * kThreads + threadIdx.x;
  if (i < table16) table[i] = make_uint4(~0u, ~0u, ~0u, ~0u);
  else if (i - table16 < zeros16) zeros[i - table16] = make_uint4(0u, 0u, 0u, 0u);
}

// Every mapping id goes into the table with its position; the atomic that does it also tells
// whether the position is (so far) the smallest of its id and which one it displaced, so "first
// occurrence" is later decided from the two streamed arrays slot[] and lost[] without a second
// random read of the table.  An id the table cannot hold sets the overflow word.
template <typename IdT, typename TableT>
__global__ __launch_bounds__(kThreads) void insert_kernel(dgs_segments mapping, int64_t n, TableT table,
                                                          uint32_t* __restrict__ slot, uint8_t* __restrict__ lost,
                                                          int* __restrict__ overflow) {
  const int64_t i = int64_t(blockIdx.x) * kThreads + threadIdx.x;
  if (i >= n) return;
  const IdT key = seg_load<IdT>(mapping, i);
  if (!table.holds(key)) {
    *overflow = 1;
    slot[i] = kNoSlot;  // no slot, no first bit: the call's results are void, and a lookup through this word gives -1
    return;
  }
  bool first;
  uint32_t displaced;
  const uint32_t w = table.insert_min(key, uint32_t(i), &first, &displaced);
  slot[i] = first ? (w | kFirstBit) : w;
  if (displaced != kNoPosition) lost[displaced] = 1;
}

__global__ __launch_bounds__(kThreads) void flag_kernel(int64_t n, uint32_t* __restrict__ slot,
                                                        const uint8_t* __restrict__ lost, int* __restrict__ tile_cnt) {
  __shared__ int lds[kThreads / kWave];
  const int64_t base = int64_t(blockIdx.x) * kTileIds + threadIdx.x * kItems;
  int c = 0;
#pragma unroll
  for (int j = 0; j < kItems; ++j) {
    const int64_t i = base + j;
    if (i < n) {
      const uint32_t s = slot[i];
      if (s & kFirstBit) {
        if (lost[i]) slot[i] = s & ~kFirstBit; else ++c;
      }
    }
  }
  int total;
  block_exclusive_scan<kThreads, int>(c, &total, lds);
  if (threadIdx.x == 0) tile_cnt[blockIdx.x] = total;
}

// counts_dev[0] = number of distinct ids, [1] = 1 if an id did not fit the table (then everything
// else the call wrote is void); mirrored into pinned host memory when the caller gave some.
__global__ __launch_bounds__(1024) void unique_scan_kernel(const int* __restrict__ tile_cnt,
                                                           int* __restrict__ tile_off, int64_t tiles,
                                                           const int* __restrict__ overflow,
                                                           int64_t* __restrict__ counts_dev,
                                                           int64_t* __restrict__ counts_host) {
  int sum;
  single_block_scan_1024<int>(tile_cnt, tile_off, tiles, &sum);
  if (threadIdx.x == 0) {
    const int64_t bad = *overflow != 0;
    counts_dev[0] = sum;
    counts_dev[1] = bad;
    if (counts_host) {
      mirror_to_host(counts_host, sum);
      mirror_to_host(counts_host + 1, bad);
    }
  }
}

template <typename IdT, typename TableT>
__global__ __launch_bounds__(kThreads) void compact_kernel(dgs_segments mapping, int64_t n,
                                                           uint32_t* __restrict__ slot,
                                                           const int* __restrict__ tile_off,
                                                           IdT* __restrict__ unique_out) {
  __shared__ int lds[kThreads / kWave];
  const int64_t base = int64_t(blockIdx.x) * kTileIds + threadIdx.x * kItems;
  uint32_t s[kItems];
  int c = 0;
#pragma unroll
  for (int j = 0; j < kItems; ++j) {
    s[j] = base + j < n ? slot[base + j] : 0u;
    c += (s[j] & kFirstBit) != 0;
  }
  int total;
  int rank = tile_off[blockIdx.x] + block_exclusive_scan<kThreads, int>(c, &total, lds);
#pragma unroll
  for (int j = 0; j < kItems; ++j) {
    if (s[j] & kFirstBit) {
      unique_out[rank] = seg_load<IdT>(mapping, base + j);
      slot[base + j] = uint32_t(rank) | kFirstBit;  // a first occurrence's word now holds its rank
      ++rank;
    }
  }
}

// Where element i of a segment list lives: its segment and its offset inside it.
__device__ __forceinline__ void seg_locate(const dgs_segments& s, int64_t i, int* seg, int64_t* off) {
  int k = 0;
  while (k + 1 < s.count && i >= s.len[k]) {
    i -= s.len[k];
    ++k;
  }
  *seg = k;
  *off = i;
}

// Mapping positions of the requiring segments that are mapping segments themselves (-1: not one).
struct SegmentAlias {
  int64_t mapping_begin[DGS_MAX_SEGMENTS];
};

// out[j] = rank of requiring[j], -1 when the id is not in the table.  Ranks live in the slot
// words of the first occurrences (a streamed array), the table keeps every id's smallest
// position: an element that is itself a first occurrence of the mapping list needs no random
// read at all, any other one reads the table entry and then that position's word.
// Nothing read from the table or from slot[] is used as an index before it has been checked: a
// slot word must name a slot of the table, and the position a table entry holds must be one of
// the n mapping positions (an entry that was never filled holds 0xffffffff).
template <typename IdT, typename TableT>
__global__ __launch_bounds__(kThreads) void lookup_kernel(dgs_segments requiring, int64_t m, TableT table,
                                                          const uint32_t* __restrict__ slot, int64_t n,
                                                          SegmentAlias alias, dgs_segments out) {
  const int64_t j = int64_t(blockIdx.x) * kThreads + threadIdx.x;
  if (j >= m) return;
  int seg;
  int64_t off;
  seg_locate(requiring, j, &seg, &off);
  uint32_t s;
  bool holds_rank = false;  // s is the word of a first occurrence of the mapping list
  if (alias.mapping_begin[seg] >= 0) {
    s = slot[alias.mapping_begin[seg] + off];
    holds_rank = (s & kFirstBit) != 0;
    s &= ~kFirstBit;
  } else {
    const IdT key = static_cast<const IdT*>(requiring.ptr[seg])[off];
    s = table.holds(key) ? table.find(key) : table.mask + 1;  // an id the table cannot hold is not in it
  }
  IdT rank = IdT(-1);
  if (holds_rank) {
    rank = IdT(s);
  } else if (s <= table.mask) {
    const uint32_t first_at = table.value(s);  // smallest mapping position of the id
    if (int64_t(first_at) < n) rank = IdT(slot[first_at] & ~kFirstBit);
  }
  static_cast<IdT*>(const_cast<void*>(out.ptr[seg]))[off] = rank;
}

// ---- small inputs: one block, the table in LDS -----------------------------------------------
//
// Up to kSmallIds mapping ids are handled by a single 1024-thread block whose hash table lives in
// LDS: one launch instead of six, LDS atomics instead of memory-side ones.  One block is one CU,
// though: its probe chains run at one CU's pace, and beyond a few thousand ids the six launches
// over the whole GPU are faster (measured on 8-byte ids: 1024 ids 11 us against 20 us of kernels,
// 6144 ids 43 us against 25, 10240 ids 84 us against 35), hence the low limit.
// Slots are packed words (id in the high half, position / rank in the low half), so an id
// of 2^32 - 1 or more sets the overflow word like the packed table in HBM does.
constexpr int kSmallThreads = 1024;
constexpr int kSmallSlots = 8192;                        // 64 KB of the CU's 160 KB
constexpr int64_t kSmallIds = 2048;                      // load factor <= 0.25: short probe chains
constexpr int kSmallPerThread = int(kSmallIds / kSmallThreads);
constexpr int64_t kSmallRequiring = int64_t(1) << 17;    // ids relabelled by the one block

template <typename IdT>
__global__ __launch_bounds__(kSmallThreads) void small_relabel_kernel(dgs_segments mapping, int64_t n,
                                                                      dgs_segments requiring, int64_t m,
                                                                      IdT* __restrict__ unique_out,
                                                                      int64_t* __restrict__ counts_dev,
                                                                      int64_t* __restrict__ counts_host,
                                                                      dgs_segments out) {
  __shared__ unsigned long long table[kSmallSlots];
  __shared__ int lds[kSmallThreads / kWave];
  __shared__ int overflow;
  constexpr unsigned long long kEmpty = ~0ull;
  constexpr uint32_t kMask = kSmallSlots - 1;
  for (int i = threadIdx.x; i < kSmallSlots; i += kSmallThreads) table[i] = kEmpty;
  if (threadIdx.x == 0) overflow = 0;
  __syncthreads();
  // insert: position i of the mapping list belongs to thread i % 1024, round i / 1024
  // (one block has one CU's worth of memory parallelism: a thread asks for all its ids at once)
  IdT key[kSmallPerThread];
  uint32_t slot[kSmallPerThread];
#pragma unroll
  for (int r = 0; r < kSmallPerThread; ++r) {
    const int64_t i = int64_t(r) * kSmallThreads + threadIdx.x;
    key[r] = i < n ? seg_load<IdT>(mapping, i) : IdT(0);
  }
#pragma unroll
  for (int r = 0; r < kSmallPerThread; ++r) {
    const int64_t i = int64_t(r) * kSmallThreads + threadIdx.x;
    slot[r] = kSmallSlots;  // none
    if (i >= n) continue;
    if (uint64_t(int64_t(key[r])) >= 0xffffffffull) {
      overflow = 1;
      continue;
    }
    const unsigned long long packed = (static_cast<unsigned long long>(uint32_t(key[r])) << 32) | uint32_t(i);
    uint32_t pos = hash_id(uint32_t(key[r])) & kMask;
    for (;;) {
      unsigned long long cur = table[pos];
      if (cur == kEmpty) {
        cur = atomicCAS(&table[pos], kEmpty, packed);
        if (cur == kEmpty) break;
      }
      if (uint32_t(cur >> 32) == uint32_t(key[r])) {
        atomicMin(&table[pos], packed);
        break;
      }
      pos = (pos + 1) & kMask;
    }
    slot[r] = pos;
  }
  __syncthreads();
  // first occurrences: the positions the table kept.  All of them are read before any slot is
  // rewritten with a rank.
  bool first[kSmallPerThread];
#pragma unroll
  for (int r = 0; r < kSmallPerThread; ++r)
    first[r] = slot[r] < kSmallSlots && uint32_t(table[slot[r]]) == uint32_t(r * kSmallThreads + threadIdx.x);
  __syncthreads();
  int base = 0;
#pragma unroll
  for (int r = 0; r < kSmallPerThread; ++r) {  // round by round: ranks follow the order of positions
    int total;
    const int ex = block_exclusive_scan<kSmallThreads, int>(first[r] ? 1 : 0, &total, lds);
    if (first[r]) {
      const uint32_t rank = uint32_t(base + ex);
      unique_out[rank] = key[r];
      table[slot[r]] = (static_cast<unsigned long long>(uint32_t(key[r])) << 32) | rank;
    }
    base += total;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    counts_dev[0] = base;
    counts_dev[1] = overflow;
    if (counts_host) {
      mirror_to_host(counts_host, base);
      mirror_to_host(counts_host + 1, overflow);
    }
  }
  // relabel: rank of every requiring id, -1 when it is not in the table; eight ids a thread at a time
  constexpr int kBatch = 8;
  for (int64_t j0 = 0; j0 < m; j0 += int64_t(kSmallThreads) * kBatch) {
    IdT id[kBatch];
    IdT* dst[kBatch];
#pragma unroll
    for (int b = 0; b < kBatch; ++b) {
      const int64_t j = j0 + int64_t(b) * kSmallThreads + threadIdx.x;
      dst[b] = nullptr;
      id[b] = IdT(-1);
      if (j < m) {
        int seg;
        int64_t off;
        seg_locate(requiring, j, &seg, &off);
        id[b] = static_cast<const IdT*>(requiring.ptr[seg])[off];
        dst[b] = static_cast<IdT*>(const_cast<void*>(out.ptr[seg])) + off;
      }
    }
#pragma unroll
    for (int b = 0; b < kBatch; ++b) {
      if (dst[b] == nullptr) continue;
      IdT rank = IdT(-1);
      if (uint64_t(int64_t(id[b])) < 0xffffffffull) {
        uint32_t pos = hash_id(uint32_t(id[b])) & kMask;
        for (;;) {
          const unsigned long long cur = table[pos];
          if (cur == kEmpty) break;
          if (uint32_t(cur >> 32) == uint32_t(id[b])) {
            rank = IdT(uint32_t(cur));
            break;
          }
          pos = (pos + 1) & kMask;
        }
      }
      *dst[b] = rank;
    }
  }
}

struct UniqueWorkspace {
  void* table;       // capacity slots of the table layout in use
  uint8_t* lost;     // [n + 16] then the overflow word: one region to zero
  int* overflow;
  uint32_t* slot;    // [n]
  int* tile_cnt;
  int* tile_off;
  uint32_t capacity;
  size_t table_bytes;  // multiple of 16 (sized for the larger layout)
  size_t zero_bytes;   // multiple of 16
};

// packed 64-bit slots, or id array + value array (the larger: what the workspace is sized for)
size_t slot_bytes(int32_t id_bytes, bool packed) { return packed ? 8 : size_t(id_bytes) + 4; }

size_t unique_workspace_layout(int64_t n, int32_t id_bytes, void* base, UniqueWorkspace* w) {
  if (n < 0) n = 0;
  if (n > kMaxMappingIds) n = kMaxMappingIds;
  const size_t tiles = size_t((n + kTileIds - 1) / kTileIds);
  Carver c(base);
  UniqueWorkspace t;
  t.capacity = table_capacity(n);
  t.table_bytes = size_t(t.capacity) * slot_bytes(id_bytes, id_bytes == 4);
  t.table = c.take<char>(t.table_bytes);
  t.zero_bytes = (size_t(n) + 16 + sizeof(int) + 15) / 16 * 16;
  t.lost = c.take<uint8_t>(t.zero_bytes);
  t.overflow = reinterpret_cast<int*>(t.lost + (size_t(n) + 16) / 16 * 16);
  t.slot = c.take<uint32_t>(size_t(n));
  t.tile_cnt = c.take<int>(tiles);
  t.tile_off = c.take<int>(tiles);
  if (w) *w = t;
  return c.used + 256;
}

int64_t seg_total(const dgs_segments& s) {
  int64_t t = 0;
  for (int k = 0; k < s.count; ++k) t += s.len[k];
  return t;
}

template <typename IdT, typename TableT>
dgs_status run_unique_relabel(const dgs_segments& mapping, int64_t n, const dgs_segments& requiring,
                              int64_t m, void* unique_out, int64_t* counts_dev, int64_t* counts_host,
                              void** ticket, const dgs_segments& out, const UniqueWorkspace& w, size_t table_bytes,
                              hipStream_t st) {
  const TableT table(w.table, w.capacity);
  const int64_t table16 = int64_t(table_bytes / 16), zeros16 = int64_t(w.zero_bytes / 16);
  hipLaunchKernelGGL(clear_kernel, dim3(uint32_t((table16 + zeros16 + kThreads - 1) / kThreads)), dim3(kThreads), 0,
                     st, static_cast<uint4*>(w.table), table16, reinterpret_cast<uint4*>(w.lost), zeros16);
  DGS_LAUNCH_CHECK();
  const int64_t tiles = (n + kTileIds - 1) / kTileIds;
  if (n > 0) {
    hipLaunchKernelGGL((insert_kernel<IdT, TableT>), dim3(uint32_t((n + kThreads - 1) / kThreads)), dim3(kThreads),
                       0, st, mapping, n, table, w.slot, w.lost, w.overflow);
    DGS_LAUNCH_CHECK();
    hipLaunchKernelGGL(flag_kernel, dim3(uint32_t(tiles)), dim3(kThreads), 0, st, n, w.slot, w.lost, w.tile_cnt);
    DGS_LAUNCH_CHECK();
  }
  hipLaunchKernelGGL(unique_scan_kernel, dim3(1), dim3(1024), 0, st, w.tile_cnt, w.tile_off, tiles, w.overflow,
                     counts_dev, counts_host);
  DGS_LAUNCH_CHECK();
  // the counts are final here: mark the point the caller may wait for
  if (ticket) {
    const dgs_status ts = dgs_ticket_record(st, ticket);
    if (ts != DGS_OK) return ts;
  }
  if (n > 0) {
    hipLaunchKernelGGL((compact_kernel<IdT, TableT>), dim3(uint32_t(tiles)), dim3(kThreads), 0, st, mapping, n,
                       w.slot, w.tile_off, static_cast<IdT*>(unique_out));
    DGS_LAUNCH_CHECK();
  }
  if (m > 0) {
    SegmentAlias alias;
    for (int r = 0; r < DGS_MAX_SEGMENTS; ++r) {
      alias.mapping_begin[r] = -1;
      int64_t begin = 0;
      for (int k = 0; k < mapping.count && r < requiring.count; ++k) {
        if (requiring.len[r] > 0 && mapping.ptr[k] == requiring.ptr[r] && mapping.len[k] == requiring.len[r])
          alias.mapping_begin[r] = begin;
        begin += mapping.len[k];
      }
    }
    hipLaunchKernelGGL((lookup_kernel<IdT, TableT>), dim3(uint32_t((m + kThreads - 1) / kThreads)), dim3(kThreads),
                       0, st, requiring, m, table, w.slot, n, alias, out);
    DGS_LAUNCH_CHECK();
  }
  return DGS_OK;
}

// Whether the current device lets one block have the LDS the small kernel declares (checked once
// per process; a device that does not takes the general path).
bool small_path_fits() {
  static const bool fits = [] {
    int dev = 0, lds_per_block = 0;
    if (hipGetDevice(&dev) != hipSuccess) return false;
    if (hipDeviceGetAttribute(&lds_per_block, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) != hipSuccess) {
      (void)hipGetLastError();
      return false;
    }
    return size_t(lds_per_block) >= sizeof(unsigned long long) * kSmallSlots + 1024;
  }();
  return fits;
}

}  // namespace
}  // namespace dgs

DGS_API size_t dgs_unique_relabel_workspace_bytes(int64_t n_mapping, int32_t id_bytes) {
  if (!dgs::width_ok(id_bytes)) id_bytes = 8;
  return dgs::unique_workspace_layout(n_mapping, id_bytes, nullptr, nullptr);
}

DGS_API dgs_status dgs_unique_relabel(dgs_segments mapping, dgs_segments requiring, int32_t id_bytes,
                                      int32_t packed_table, void* unique_out, int64_t* counts_dev,
                                      int64_t* counts_host, void** counts_ticket, dgs_segments out, void* workspace,
                                      size_t workspace_bytes, void* stream) {
  using namespace dgs;
  DGS_REQUIRE(width_ok(id_bytes), DGS_ERR_INVALID, "relabel: id width %d is not 4 or 8", id_bytes);
  DGS_REQUIRE(mapping.count >= 0 && mapping.count <= DGS_MAX_SEGMENTS && requiring.count >= 0 &&
                  requiring.count <= DGS_MAX_SEGMENTS,
              DGS_ERR_INVALID, "relabel: segment count out of range");
  DGS_REQUIRE(out.count == requiring.count, DGS_ERR_INVALID, "relabel: %d outputs for %d inputs", out.count,
              requiring.count);
  for (int k = 0; k < mapping.count; ++k)
    DGS_REQUIRE(mapping.len[k] >= 0 && (mapping.len[k] == 0 || mapping.ptr[k]), DGS_ERR_INVALID,
                "relabel: bad mapping segment %d", k);
  for (int k = 0; k < requiring.count; ++k)
    DGS_REQUIRE(requiring.len[k] >= 0 && out.len[k] == requiring.len[k] &&
                    (requiring.len[k] == 0 || (requiring.ptr[k] && out.ptr[k])),
                DGS_ERR_INVALID, "relabel: bad requiring/output segment %d", k);
  DGS_REQUIRE(counts_dev != nullptr, DGS_ERR_INVALID, "relabel: null counts_dev");
  DGS_REQUIRE(counts_ticket == nullptr || counts_host != nullptr, DGS_ERR_INVALID,
              "relabel: a counts_ticket needs counts_host");
  const int64_t n = seg_total(mapping);
  const int64_t m = seg_total(requiring);
  DGS_REQUIRE(n <= kMaxMappingIds, DGS_ERR_UNSUPPORTED, "relabel: %lld mapping ids exceed 2^30", (long long)n);
  DGS_REQUIRE(m <= int64_t(0x7fffffff) * kThreads, DGS_ERR_UNSUPPORTED, "relabel: too many ids to relabel");
  DGS_REQUIRE(n == 0 || unique_out != nullptr, DGS_ERR_INVALID, "relabel: null unique_out");
  DGS_REQUIRE(workspace != nullptr && workspace_bytes >= dgs_unique_relabel_workspace_bytes(n, id_bytes),
              DGS_ERR_WORKSPACE, "relabel: workspace of %zu B, need %zu", workspace_bytes,
              dgs_unique_relabel_workspace_bytes(n, id_bytes));
  DGS_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255) == 0, DGS_ERR_WORKSPACE,
              "relabel: workspace must be 256-byte aligned");
  UniqueWorkspace w;
  unique_workspace_layout(n, id_bytes, workspace, &w);
  hipStream_t st = static_cast<hipStream_t>(stream);
  // small inputs with packable ids: the one-block kernel with its table in LDS
  if (n <= kSmallIds && m <= kSmallRequiring && (id_bytes == 4 || packed_table != 0) && small_path_fits()) {
    if (id_bytes == 4)
      hipLaunchKernelGGL(small_relabel_kernel<int32_t>, dim3(1), dim3(kSmallThreads), 0, st, mapping, n, requiring, m,
                         static_cast<int32_t*>(unique_out), counts_dev, counts_host, out);
    else
      hipLaunchKernelGGL(small_relabel_kernel<int64_t>, dim3(1), dim3(kSmallThreads), 0, st, mapping, n, requiring, m,
                         static_cast<int64_t*>(unique_out), counts_dev, counts_host, out);
    DGS_LAUNCH_CHECK();
    return counts_ticket ? dgs_ticket_record(st, counts_ticket) : DGS_OK;
  }
  if (id_bytes == 4)
    return run_unique_relabel<int32_t, Table<int32_t, true>>(mapping, n, requiring, m, unique_out, counts_dev,
                                                             counts_host, counts_ticket, out, w, w.table_bytes, st);
  if (packed_table != 0)  // 8-byte ids in 8-byte slots: ids of 2^32 - 1 or more set the overflow word
    return run_unique_relabel<int64_t, Table<int64_t, true>>(mapping, n, requiring, m, unique_out, counts_dev,
                                                             counts_host, counts_ticket, out, w,
                                                             size_t(w.capacity) * 8, st);
  return run_unique_relabel<int64_t, Table<int64_t, false>>(mapping, n, requiring, m, unique_out, counts_dev,
                                                            counts_host, counts_ticket, out, w, w.table_bytes, st);
}
