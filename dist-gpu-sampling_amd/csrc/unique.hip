// First-occurrence unique + relabel of node ids.
//
// A linear-probing table in HBM (table.h: packed 64-bit slots for 4-byte ids, id array +
// value array for 8-byte ids) maps each id to the smallest position at which it occurs; a position is
// a "first occurrence" when the table holds exactly that position.  Flags are
// scanned tile by tile, first occurrences are compacted in input order (which is
// what makes the result independent of the table layout) and the table value
// becomes the id's rank.  Every mapping id remembers its slot, so a tensor that
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

__global__ __launch_bounds__(kThreads) void fill_ones_kernel(uint4* __restrict__ p, int64_t n16) {
  const int64_t i = int64_t(blockIdx.x) * kThreads + threadIdx.x;
  if (i < n16) p[i] = make_uint4(~0u, ~0u, ~0u, ~0u);
}

template <typename IdT, typename TableT>
__global__ __launch_bounds__(kThreads) void insert_kernel(dgs_segments mapping, int64_t n, TableT table,
                                                          uint32_t* __restrict__ slot) {
  const int64_t i = int64_t(blockIdx.x) * kThreads + threadIdx.x;
  if (i >= n) return;
  slot[i] = table.insert(seg_load<IdT>(mapping, i), uint32_t(i));
}

template <typename TableT>
__global__ __launch_bounds__(kThreads) void flag_kernel(int64_t n, TableT table, uint32_t* __restrict__ slot,
                                                        int* __restrict__ tile_cnt) {
  __shared__ int lds[kThreads / kWave];
  const int64_t base = int64_t(blockIdx.x) * kTileIds + threadIdx.x * kItems;
  int c = 0;
#pragma unroll
  for (int j = 0; j < kItems; ++j) {
    const int64_t i = base + j;
    if (i < n) {
      const uint32_t s = slot[i];
      if (table.value(s) == uint32_t(i)) {
        slot[i] = s | kFirstBit;
        ++c;
      }
    }
  }
  int total;
  block_exclusive_scan<kThreads, int>(c, &total, lds);
  if (threadIdx.x == 0) tile_cnt[blockIdx.x] = total;
}

__global__ __launch_bounds__(1024) void unique_scan_kernel(const int* __restrict__ tile_cnt,
                                                           int* __restrict__ tile_off, int64_t tiles,
                                                           int64_t* __restrict__ num_unique_dev) {
  int sum;
  single_block_scan_1024<int>(tile_cnt, tile_off, tiles, &sum);
  if (threadIdx.x == 0) *num_unique_dev = sum;
}

template <typename IdT, typename TableT>
__global__ __launch_bounds__(kThreads) void compact_kernel(dgs_segments mapping, int64_t n,
                                                           const uint32_t* __restrict__ slot,
                                                           const int* __restrict__ tile_off, TableT table,
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
      table.set_value(s[j] & ~kFirstBit, uint32_t(rank));
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

// out[j] = rank of requiring[j], -1 when the id is not in the table.
template <typename IdT, typename TableT>
__global__ __launch_bounds__(kThreads) void lookup_kernel(dgs_segments requiring, int64_t m, TableT table,
                                                          const uint32_t* __restrict__ slot, SegmentAlias alias,
                                                          dgs_segments out) {
  const int64_t j = int64_t(blockIdx.x) * kThreads + threadIdx.x;
  if (j >= m) return;
  int seg;
  int64_t off;
  seg_locate(requiring, j, &seg, &off);
  uint32_t s;
  if (alias.mapping_begin[seg] >= 0) s = slot[alias.mapping_begin[seg] + off] & ~kFirstBit;
  else s = table.find(static_cast<const IdT*>(requiring.ptr[seg])[off]);
  static_cast<IdT*>(const_cast<void*>(out.ptr[seg]))[off] = s > table.mask ? IdT(-1) : IdT(table.value(s));
}

struct UniqueWorkspace {
  void* table;       // capacity slots of the table layout in use
  uint32_t* slot;    // [n]
  int* tile_cnt;
  int* tile_off;
  uint32_t capacity;
  size_t table_bytes;  // multiple of 16
};

// 4-byte ids always fit the packed 64-bit slot; 8-byte ids get the id array + value array.
size_t slot_bytes(int32_t id_bytes) { return id_bytes == 4 ? 8 : size_t(id_bytes) + 4; }

size_t unique_workspace_layout(int64_t n, int32_t id_bytes, void* base, UniqueWorkspace* w) {
  if (n < 0) n = 0;
  if (n > kMaxMappingIds) n = kMaxMappingIds;
  const size_t tiles = size_t((n + kTileIds - 1) / kTileIds);
  Carver c(base);
  UniqueWorkspace t;
  t.capacity = table_capacity(n);
  t.table_bytes = size_t(t.capacity) * slot_bytes(id_bytes);
  t.table = c.take<char>(t.table_bytes);
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
                              int64_t m, void* unique_out, int64_t* num_unique_dev,
                              const dgs_segments& out, const UniqueWorkspace& w, hipStream_t st) {
  const TableT table(w.table, w.capacity);
  const int64_t n16 = int64_t(w.table_bytes / 16);
  hipLaunchKernelGGL(fill_ones_kernel, dim3(uint32_t((n16 + kThreads - 1) / kThreads)), dim3(kThreads), 0, st,
                     static_cast<uint4*>(w.table), n16);
  DGS_LAUNCH_CHECK();
  const int64_t tiles = (n + kTileIds - 1) / kTileIds;
  if (n > 0) {
    hipLaunchKernelGGL((insert_kernel<IdT, TableT>), dim3(uint32_t((n + kThreads - 1) / kThreads)), dim3(kThreads),
                       0, st, mapping, n, table, w.slot);
    DGS_LAUNCH_CHECK();
    hipLaunchKernelGGL(flag_kernel<TableT>, dim3(uint32_t(tiles)), dim3(kThreads), 0, st, n, table, w.slot,
                       w.tile_cnt);
    DGS_LAUNCH_CHECK();
  }
  hipLaunchKernelGGL(unique_scan_kernel, dim3(1), dim3(1024), 0, st, w.tile_cnt, w.tile_off, tiles, num_unique_dev);
  DGS_LAUNCH_CHECK();
  if (n > 0) {
    hipLaunchKernelGGL((compact_kernel<IdT, TableT>), dim3(uint32_t(tiles)), dim3(kThreads), 0, st, mapping, n,
                       w.slot, w.tile_off, table, static_cast<IdT*>(unique_out));
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
                       0, st, requiring, m, table, w.slot, alias, out);
    DGS_LAUNCH_CHECK();
  }
  return DGS_OK;
}

}  // namespace
}  // namespace dgs

DGS_API size_t dgs_unique_relabel_workspace_bytes(int64_t n_mapping, int32_t id_bytes) {
  if (!dgs::width_ok(id_bytes)) id_bytes = 8;
  return dgs::unique_workspace_layout(n_mapping, id_bytes, nullptr, nullptr);
}

DGS_API dgs_status dgs_unique_relabel(dgs_segments mapping, dgs_segments requiring, int32_t id_bytes,
                                      void* unique_out, int64_t* num_unique_dev, dgs_segments out,
                                      void* workspace, size_t workspace_bytes, void* stream) {
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
  DGS_REQUIRE(num_unique_dev != nullptr, DGS_ERR_INVALID, "relabel: null num_unique_dev");
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
  return id_bytes == 8 ? run_unique_relabel<int64_t, Table<int64_t, false>>(mapping, n, requiring, m, unique_out,
                                                                           num_unique_dev, out, w, st)
                       : run_unique_relabel<int32_t, Table<int32_t, true>>(mapping, n, requiring, m, unique_out,
                                                                          num_unique_dev, out, w, st);
}
