// Row-wise uniform neighbour sampling over CSC held in two-tier views: the per-hop operator
// (exact-size outputs, any fanout).
//
// Three launches per hop, no host round trip in between:
//   count : one thread per seed reads its indptr pair, keeps (start, degree), scans the pick
//           counts of a 256-seed tile (offset inside the tile + tile total);
//   scan  : one block turns the tile totals into tile offsets and the edge count;
//   fill  : num_picks <= 64: a group of G lanes per seed row over the whole grid (G = 8..64,
//           the smallest power of two holding num_picks), so a wave64 serves 64/G rows;
//           larger num_picks: one wave per row, Floyd's kept set in LDS (num_picks <= 2048) or
//           in the row's own output slots (any num_picks).
// Random picks follow the "dgs-philox-1" contract: every (seed, stream, row, draw) names one
// Philox block, so results do not depend on the launch shape.
#include <mutex>
#include <type_traits>

#include "common.h"
#include "picks.h"
#include "sample_workspace.h"

namespace dgs {
namespace {

// Scratch of the entry point that allocates nothing: one copy per GPU, held until the process
// ends.  In host code the array's name is only a stand-in; the device address of each GPU's copy
// comes from hipGetSymbolAddress (static_scratch_of) and is what kernels and checks receive.
constexpr int64_t kStaticMaxSeeds = DGS_STATIC_MAX_SEEDS;
constexpr size_t kStaticScratchBytes = size_t(2) << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
constexpr int kMaxDevices = 64;
std::mutex g_static_mutex;
void* g_static_scratch[kMaxDevices] = {};

// The current device's copy of `scratch`, looked up once per device.
dgs_status static_scratch_of(void** out) {
  int dev = -1;
  DGS_HIP_TRY(hipGetDevice(&dev));
  DGS_REQUIRE(dev >= 0 && dev < kMaxDevices, DGS_ERR_UNSUPPORTED, "sample_neighbors_static: device %d", dev);
  std::lock_guard<std::mutex> lock(g_static_mutex);
  if (g_static_scratch[dev] == nullptr) {
    void* p = nullptr;
    DGS_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    DGS_REQUIRE(p != nullptr && (reinterpret_cast<uintptr_t>(p) & 255) == 0, DGS_ERR_HIP,
                "sample_neighbors_static: scratch symbol resolved to %p", p);
    g_static_scratch[dev] = p;
  }
  *out = g_static_scratch[dev];
  return DGS_OK;
}

constexpr int kMaxGroupPicks = 64;   // fill_group_kernel handles num_picks <= 64
constexpr int kMaxLdsPicks = 2048;   // fill_wave_kernel keeps Floyd's set in LDS
constexpr int kFlagDegree = 1;       // some row has degree >= 2^32, or offsets outside the edge array
constexpr int kFlagSeed = 2;         // some seed id is not a row of the graph

template <typename IdT, typename PtrT>
__global__ __launch_bounds__(kTile) void sample_count_kernel(
    const IdT* __restrict__ seeds, int64_t n_seeds, TierView<PtrT> indptr, int64_t n_edges, int64_t k,
    bool replace, int64_t* __restrict__ row_start, uint32_t* __restrict__ row_deg, int64_t* __restrict__ row_off,
    int64_t* __restrict__ tile_sum, int* __restrict__ tile_flag) {
  __shared__ int64_t lds[kTile / kWave];
  __shared__ int flag;
  if (threadIdx.x == 0) flag = 0;
  __syncthreads();
  const int64_t i = int64_t(blockIdx.x) * kTile + threadIdx.x;
  int64_t c = 0;
  if (i < n_seeds) {
    const int64_t row = int64_t(seeds[i]);
    int64_t b = 0, deg = 0;
    int bad = 0;
    if (row_in_range(indptr, row)) {  // checked before the offsets are read
      b = int64_t(indptr.at(row));
      deg = int64_t(indptr.at(row + 1)) - b;
      // offsets that leave the edge array are refused here, before the fill reads through them
      if (deg < 0 || deg > 0xffffffffLL || b < 0 || b + deg > n_edges) { bad |= kFlagDegree; b = 0; deg = 0; }
    } else {
      bad |= kFlagSeed;
    }
    if (bad) atomicOr(&flag, bad);
    row_start[i] = b;
    row_deg[i] = uint32_t(deg);
    c = pick_count(deg, k, replace);
  }
  int64_t total;
  const int64_t ex = block_exclusive_scan<kTile, int64_t>(c, &total, lds);
  if (i < n_seeds) row_off[i] = ex;
  if (threadIdx.x == 0) {
    tile_sum[blockIdx.x] = total;
    tile_flag[blockIdx.x] = flag;
  }
}

__global__ __launch_bounds__(1024) void sample_scan_kernel(const int64_t* __restrict__ tile_sum,
                                                           int64_t* __restrict__ tile_off,
                                                           const int* __restrict__ tile_flag,
                                                           int64_t tiles, int64_t* __restrict__ nnz_dev,
                                                           int64_t* __restrict__ nnz_host) {
  __shared__ int any_flag;
  if (threadIdx.x == 0) any_flag = 0;
  __syncthreads();
  int f = 0;
  for (int64_t t = threadIdx.x; t < tiles; t += 1024) f |= tile_flag[t];
  if (f) atomicOr(&any_flag, f);
  int64_t sum;
  single_block_scan_1024<int64_t>(tile_sum, tile_off, tiles, &sum);
  __syncthreads();
  if (threadIdx.x == 0) {
    nnz_dev[0] = sum;
    nnz_dev[1] = any_flag;
    if (nnz_host) {  // pinned host memory: the caller reads the length without a copy
      mirror_to_host(nnz_host, sum);
      mirror_to_host(nnz_host + 1, any_flag);
    }
  }
}

// num_picks <= 64: G lanes per row over the whole grid, lane l owns output slot l.
template <typename IdT, int G>
__global__ __launch_bounds__(kTile) void fill_group_kernel(
    const IdT* __restrict__ seeds, int64_t n_seeds, const int64_t* __restrict__ row_start,
    const uint32_t* __restrict__ row_deg, const int64_t* __restrict__ row_off,
    const int64_t* __restrict__ tile_off, TierView<IdT> indices, int k, bool replace, uint64_t rng_seed,
    uint32_t rng_stream, IdT* __restrict__ out_rows, IdT* __restrict__ out_cols) {
  const int64_t gid = int64_t(blockIdx.x) * kTile + threadIdx.x;
  const int64_t i = gid / G;
  const int l = int(gid % G);
  if (i >= n_seeds) return;  // whole groups leave together
  const int group_lane0 = (threadIdx.x & (kWave - 1)) - l;
  const int64_t row = int64_t(seeds[i]);
  uint32_t pos;
  if (!pick_position<G>(row_deg[i], k, replace, l, group_lane0, rng_seed, rng_stream, row, &pos)) return;
  const int64_t o = tile_off[i / kTile] + row_off[i] + l;
  out_rows[o] = IdT(row);
  out_cols[o] = indices.at(row_start[i] + pos);
}

// Any num_picks: one wave per row, lanes stride over the slots; Floyd's kept set lives in LDS
// (num_picks <= kMaxLdsPicks; the launcher sends larger requests to fill_wave_global_kernel).
template <typename IdT>
__global__ __launch_bounds__(kTile) void fill_wave_kernel(
    const IdT* __restrict__ seeds, int64_t n_seeds, const int64_t* __restrict__ row_start,
    const uint32_t* __restrict__ row_deg, const int64_t* __restrict__ row_off,
    const int64_t* __restrict__ tile_off, TierView<IdT> indices, int64_t k, bool replace, uint64_t rng_seed,
    uint32_t rng_stream, IdT* __restrict__ out_rows, IdT* __restrict__ out_cols) {
  extern __shared__ uint32_t kept_lds[];  // (kTile / kWave) * min(k, kMaxLdsPicks) entries
  const int wave = threadIdx.x / kWave;
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t i = int64_t(blockIdx.x) * (kTile / kWave) + wave;
  if (i >= n_seeds) return;  // whole waves leave together
  const int64_t kk = k < kMaxLdsPicks ? k : kMaxLdsPicks;
  uint32_t* kept = kept_lds + int64_t(wave) * kk;
  const int64_t start = row_start[i];
  const int64_t off = tile_off[i / kTile] + row_off[i];
  const int64_t row = int64_t(seeds[i]);
  const uint32_t deg = row_deg[i];
  if (replace) {
    if (deg > 0) {
      for (int64_t s = lane; s < k; s += kWave) {
        const uint32_t p = philox_bounded(rng_seed, rng_stream, row, uint32_t(s), deg);
        out_rows[off + s] = IdT(row);
        out_cols[off + s] = indices.at(start + p);
      }
    }
  } else if (int64_t(deg) <= k) {
    for (uint32_t s = lane; s < deg; s += kWave) {
      out_rows[off + s] = IdT(row);
      out_cols[off + s] = indices.at(start + s);
    }
  } else {
    // Floyd, 64 candidates at a time; each is checked against everything kept so far
    const uint32_t base_top = deg - uint32_t(k);
    for (int s0 = 0; s0 < int(k); s0 += kWave) {
      const int s = s0 + lane;
      uint32_t cand = 0xffffffffu;
      if (s < k) cand = philox_bounded(rng_seed, rng_stream, row, uint32_t(s), base_top + s + 1u);
      const int batch = int(k) - s0 < kWave ? int(k) - s0 : kWave;
      for (int b = 0; b < batch; ++b) {
        const uint32_t c = __shfl(cand, b, kWave);
        const int slot = s0 + b;
        bool hit = false;
        for (int q = lane; q < slot; q += kWave) hit |= kept[q] == c;
        const bool any = __ballot(hit) != 0;
        if (lane == 0) kept[slot] = any ? base_top + uint32_t(slot) : c;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      }
    }
    for (int64_t s = lane; s < k; s += kWave) {
      out_rows[off + s] = IdT(row);
      out_cols[off + s] = indices.at(start + kept[s]);
    }
  }
}

// num_picks above kMaxLdsPicks: one wave per row, Floyd's kept set lives in the row's own slots
// of out_cols (a position fits an id slot) and is turned into neighbour ids at the end.  Slots are
// resolved 64 at a time: every lane first compares its candidate with all positions kept by
// earlier batches (read 64 at a time, handed round with __shfl), then the batch settles its own
// order lane by lane as pick_position does.
template <typename IdT>
__global__ __launch_bounds__(kTile) void fill_wave_global_kernel(
    const IdT* __restrict__ seeds, int64_t n_seeds, const int64_t* __restrict__ row_start,
    const uint32_t* __restrict__ row_deg, const int64_t* __restrict__ row_off,
    const int64_t* __restrict__ tile_off, TierView<IdT> indices, int64_t k, bool replace, uint64_t rng_seed,
    uint32_t rng_stream, IdT* __restrict__ out_rows, IdT* __restrict__ out_cols) {
  using U = typename std::make_unsigned<IdT>::type;
  const int wave = threadIdx.x / kWave;
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t i = int64_t(blockIdx.x) * (kTile / kWave) + wave;
  if (i >= n_seeds) return;  // whole waves leave together
  const int64_t start = row_start[i];
  const int64_t off = tile_off[i / kTile] + row_off[i];
  const int64_t row = int64_t(seeds[i]);
  const uint32_t deg = row_deg[i];
  if (replace) {
    if (deg > 0) {
      for (int64_t s = lane; s < k; s += kWave) {
        const uint32_t p = philox_bounded(rng_seed, rng_stream, row, uint32_t(s), deg);
        out_rows[off + s] = IdT(row);
        out_cols[off + s] = indices.at(start + p);
      }
    }
    return;
  }
  if (int64_t(deg) <= k) {
    for (uint32_t s = lane; s < deg; s += kWave) {
      out_rows[off + s] = IdT(row);
      out_cols[off + s] = indices.at(start + s);
    }
    return;
  }
  U* kept = reinterpret_cast<U*>(out_cols + off);  // [k] positions, zero-extended
  const uint32_t base_top = deg - uint32_t(k);
  for (int64_t s0 = 0; s0 < k; s0 += kWave) {
    const int64_t s = s0 + lane;
    const bool live = s < k;
    const uint32_t top = base_top + uint32_t(s);
    uint32_t cand = 0xffffffffu;  // no kept position has this value: deg <= 2^32 - 1
    if (live) cand = philox_bounded(rng_seed, rng_stream, row, uint32_t(s), top + 1u);
    // against the batches before this one (their stores were fenced below)
    bool hit = false;
    for (int64_t q0 = 0; q0 < s0; q0 += kWave) {
      const uint32_t mine = uint32_t(kept[q0 + lane]);  // s0 is a multiple of 64: always in range
#pragma unroll 8
      for (int j = 0; j < kWave; ++j) hit |= __shfl(mine, j, kWave) == cand;
    }
    uint32_t keep = hit ? top : cand;
    // inside the batch: slot t sees what the slots before it finally kept
    const int batch = int(k - s0 < kWave ? k - s0 : kWave);
    for (int t = 1; t < batch; ++t) {
      const uint32_t c = __shfl(cand, t, kWave);
      const bool clash = __ballot(keep == c && lane < t) != 0;
      if (lane == t && clash && !hit) keep = top;
    }
    if (live) kept[s] = U(keep);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  }
  for (int64_t s = lane; s < k; s += kWave) {
    out_rows[off + s] = IdT(row);
    out_cols[off + s] = indices.at(start + int64_t(uint32_t(kept[s])));
  }
}

template <typename IdT, typename PtrT>
dgs_status run_count(const void* seeds, int64_t n_seeds, const dgs_view& indptr, int64_t n_edges, int64_t k,
                     bool replace, const SampleWorkspace& w, int64_t* nnz_dev, int64_t* nnz_host, hipStream_t st) {
  const int64_t tiles = (n_seeds + kTile - 1) / kTile;
  if (tiles > 0) {
    hipLaunchKernelGGL((sample_count_kernel<IdT, PtrT>), dim3(uint32_t(tiles)), dim3(kTile), 0, st,
                       static_cast<const IdT*>(seeds), n_seeds, TierView<PtrT>(indptr), n_edges, k, replace,
                       w.row_start, w.row_deg, w.row_off, w.tile_sum, w.tile_flag);
    DGS_LAUNCH_CHECK();
  }
  hipLaunchKernelGGL(sample_scan_kernel, dim3(1), dim3(1024), 0, st, w.tile_sum, w.tile_off, w.tile_flag,
                     tiles, nnz_dev, nnz_host);
  DGS_LAUNCH_CHECK();
  return DGS_OK;
}

template <typename IdT, int G>
void launch_group(const void* seeds, int64_t n_seeds, const SampleWorkspace& w,
                  const dgs_view& indices, int k, bool replace, uint64_t rng_seed, uint32_t rng_stream,
                  void* out_rows, void* out_cols, hipStream_t st) {
  const int64_t blocks = (n_seeds * G + kTile - 1) / kTile;
  hipLaunchKernelGGL((fill_group_kernel<IdT, G>), dim3(uint32_t(blocks)), dim3(kTile), 0, st,
                     static_cast<const IdT*>(seeds), n_seeds, w.row_start, w.row_deg, w.row_off, w.tile_off,
                     TierView<IdT>(indices), k, replace, rng_seed, rng_stream, static_cast<IdT*>(out_rows),
                     static_cast<IdT*>(out_cols));
}

template <typename IdT>
dgs_status run_fill(const void* seeds, int64_t n_seeds, const dgs_view& indices, int64_t k, bool replace,
                    uint64_t rng_seed, uint32_t rng_stream, const SampleWorkspace& w, void* out_rows,
                    void* out_cols, hipStream_t st) {
  const int64_t tiles = (n_seeds + kTile - 1) / kTile;
  if (tiles == 0 || k <= 0) return DGS_OK;
  if (k <= kMaxGroupPicks) {
    const int kk = int(k);
    if (kk <= 8) launch_group<IdT, 8>(seeds, n_seeds, w, indices, kk, replace, rng_seed, rng_stream, out_rows, out_cols, st);
    else if (kk <= 16) launch_group<IdT, 16>(seeds, n_seeds, w, indices, kk, replace, rng_seed, rng_stream, out_rows, out_cols, st);
    else if (kk <= 32) launch_group<IdT, 32>(seeds, n_seeds, w, indices, kk, replace, rng_seed, rng_stream, out_rows, out_cols, st);
    else launch_group<IdT, 64>(seeds, n_seeds, w, indices, kk, replace, rng_seed, rng_stream, out_rows, out_cols, st);
  } else if (k > kMaxLdsPicks) {
    const int64_t blocks = (n_seeds + kTile / kWave - 1) / (kTile / kWave);
    hipLaunchKernelGGL((fill_wave_global_kernel<IdT>), dim3(uint32_t(blocks)), dim3(kTile), 0, st,
                       static_cast<const IdT*>(seeds), n_seeds, w.row_start, w.row_deg, w.row_off, w.tile_off,
                       TierView<IdT>(indices), k, replace, rng_seed, rng_stream, static_cast<IdT*>(out_rows),
                       static_cast<IdT*>(out_cols));
  } else {
    const int64_t kk = k;
    const size_t lds = replace ? 0 : size_t(kTile / kWave) * size_t(kk) * sizeof(uint32_t);
    const int64_t blocks = (n_seeds + kTile / kWave - 1) / (kTile / kWave);
    hipLaunchKernelGGL((fill_wave_kernel<IdT>), dim3(uint32_t(blocks)), dim3(kTile), lds, st,
                       static_cast<const IdT*>(seeds), n_seeds, w.row_start, w.row_deg, w.row_off, w.tile_off,
                       TierView<IdT>(indices), k, replace, rng_seed, rng_stream, static_cast<IdT*>(out_rows),
                       static_cast<IdT*>(out_cols));
  }
  DGS_LAUNCH_CHECK();
  return DGS_OK;
}

}  // namespace
}  // namespace dgs

DGS_API size_t dgs_sample_workspace_bytes(int64_t n_seeds) {
  return dgs::sample_workspace_layout(n_seeds, nullptr, nullptr);
}

DGS_API dgs_status dgs_sample_count(const void* seeds, int32_t id_bytes, int64_t n_seeds, dgs_view indptr,
                                    int64_t n_edges, int64_t num_picks, int32_t replace, int64_t* nnz_dev, int64_t* nnz_host,
                                    void* workspace, size_t workspace_bytes, void* stream) {
  using namespace dgs;
  dgs_status s = check_sample_args("sample_count", seeds, id_bytes, n_seeds, num_picks, workspace, workspace_bytes);
  if (s != DGS_OK) return s;
  DGS_REQUIRE(width_ok(indptr.elem_bytes), DGS_ERR_INVALID, "sample_count: indptr width %d is not 4 or 8",
              indptr.elem_bytes);
  DGS_REQUIRE(nnz_dev != nullptr, DGS_ERR_INVALID, "sample_count: null nnz_dev");
  DGS_REQUIRE(n_edges >= 0, DGS_ERR_INVALID, "sample_count: n_edges=%lld", (long long)n_edges);
  hipStream_t st = static_cast<hipStream_t>(stream);
  SampleWorkspace w;
  sample_workspace_layout(n_seeds, workspace, &w);
  const bool rep = replace != 0;
  if (id_bytes == 8)
    return indptr.elem_bytes == 8 ? run_count<int64_t, int64_t>(seeds, n_seeds, indptr, n_edges, num_picks, rep, w, nnz_dev, nnz_host, st)
                                  : run_count<int64_t, int32_t>(seeds, n_seeds, indptr, n_edges, num_picks, rep, w, nnz_dev, nnz_host, st);
  return indptr.elem_bytes == 8 ? run_count<int32_t, int64_t>(seeds, n_seeds, indptr, n_edges, num_picks, rep, w, nnz_dev, nnz_host, st)
                                : run_count<int32_t, int32_t>(seeds, n_seeds, indptr, n_edges, num_picks, rep, w, nnz_dev, nnz_host, st);
}

DGS_API dgs_status dgs_sample_fill(const void* seeds, int32_t id_bytes, int64_t n_seeds, dgs_view indices,
                                   int64_t num_picks, int32_t replace, uint64_t rng_seed, uint32_t rng_stream,
                                   void* out_rows, void* out_cols, void* workspace, size_t workspace_bytes,
                                   void* stream) {
  using namespace dgs;
  dgs_status s = check_sample_args("sample_fill", seeds, id_bytes, n_seeds, num_picks, workspace, workspace_bytes);
  if (s != DGS_OK) return s;
  DGS_REQUIRE(indices.elem_bytes == id_bytes, DGS_ERR_INVALID,
              "sample_fill: indices width %d differs from the seed width %d", indices.elem_bytes, id_bytes);
  DGS_REQUIRE(n_seeds == 0 || num_picks == 0 || (out_rows != nullptr && out_cols != nullptr), DGS_ERR_INVALID,
              "sample_fill: null output");
  hipStream_t st = static_cast<hipStream_t>(stream);
  SampleWorkspace w;
  sample_workspace_layout(n_seeds, workspace, &w);
  const bool rep = replace != 0;
  return id_bytes == 8
             ? run_fill<int64_t>(seeds, n_seeds, indices, num_picks, rep, rng_seed, rng_stream, w, out_rows, out_cols, st)
             : run_fill<int32_t>(seeds, n_seeds, indices, num_picks, rep, rng_seed, rng_stream, w, out_rows, out_cols, st);
}

DGS_API dgs_status dgs_sample_neighbors(const void* seeds, int32_t id_bytes, int64_t n_seeds,
                                        dgs_view indptr, dgs_view indices, int64_t num_picks,
                                        int32_t replace, uint64_t rng_seed, uint32_t rng_stream,
                                        void* out_rows, void* out_cols, int64_t* nnz_dev, void* workspace,
                                        size_t workspace_bytes, void* stream) {
  dgs_status s = dgs_sample_count(seeds, id_bytes, n_seeds, indptr, indices.total, num_picks, replace, nnz_dev, nullptr, workspace,
                                  workspace_bytes, stream);
  if (s != DGS_OK) return s;
  return dgs_sample_fill(seeds, id_bytes, n_seeds, indices, num_picks, replace, rng_seed, rng_stream, out_rows,
                         out_cols, workspace, workspace_bytes, stream);
}

DGS_API dgs_status dgs_sample_neighbors_static(const void* seeds, int32_t id_bytes, int64_t n_seeds,
                                               dgs_view indptr, dgs_view indices, int64_t num_picks,
                                               int32_t replace, uint64_t rng_seed, uint32_t rng_stream,
                                               void* out_rows, void* out_cols, int64_t* nnz_dev, void* stream) {
  using namespace dgs;
  DGS_REQUIRE(n_seeds >= 0 && n_seeds <= kStaticMaxSeeds, DGS_ERR_UNSUPPORTED,
              "sample_neighbors_static: %lld seeds, at most %lld fit the static scratch (use dgs_sample_neighbors "
              "with a workspace)", (long long)n_seeds, (long long)kStaticMaxSeeds);
  DGS_REQUIRE(sample_workspace_layout(n_seeds, nullptr, nullptr) <= kStaticScratchBytes, DGS_ERR_UNSUPPORTED,
              "sample_neighbors_static: scratch of %zu B is too small for %lld seeds", kStaticScratchBytes,
              (long long)n_seeds);
  void* ws = nullptr;
  const dgs_status s = static_scratch_of(&ws);
  if (s != DGS_OK) return s;
  // every word of the layout that the fill reads is written by the count pass of the same call,
  // so nothing of the previous call's contents has to be cleared
  return dgs_sample_neighbors(seeds, id_bytes, n_seeds, indptr, indices, num_picks, replace, rng_seed, rng_stream,
                              out_rows, out_cols, nnz_dev, ws, kStaticScratchBytes, stream);
}
