// Row-wise weighted neighbour sampling, the per-hop operator: a float32 weight per edge, stored
// like `indices`.  The pick rules live in race.h.
//
// The count pass is the uniform sampler's (same pick counts).  The fill hands every seed row to a
// group of G lanes (G = 16, 32 or 64, so a wave64 serves up to four rows; chosen on the host from
// num_picks); rows of more than 32 G neighbours are queued (one atomic per such row) and then
// handled by a second launch that spends a 1024-thread block on a row.

#include "common.h"
#include "race.h"
#include "sample_workspace.h"

namespace dgs {
namespace {

constexpr int kMaxLongGrid = 512;  // two 1024-thread blocks fit a CU: one round over 256 CUs

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
  const uint32_t pos = race_row<G>(g, probs, start, end, k, rng_seed, rng_stream, row);
  if (end > 0 && g.l < k && pos < end) {  // a row that races has more than k positions: every entry is filled
    out_rows[off + g.l] = IdT(row);
    out_cols[off + g.l] = indices.at(start + pos);
  }
}

// Without replacement, queued long rows: a block per row.
template <typename IdT>
__global__ __launch_bounds__(kLongBlock) void fill_weighted_long_kernel(const IdT* __restrict__ seeds, RowArgs a,
                                                                        TierView<IdT> indices,
                                                                        TierView<float> probs, int k,
                                                                        uint64_t rng_seed, uint32_t rng_stream,
                                                                        IdT* __restrict__ out_rows,
                                                                        IdT* __restrict__ out_cols) {
  __shared__ LongRowScratch lds;
  const int64_t n_long = *a.long_count;
  for (int64_t t = blockIdx.x; t < n_long; t += gridDim.x) {
    const int64_t i = a.long_rows[t];
    const int64_t start = a.row_start[i];
    const int64_t off = a.tile_off[i / kTile] + a.row_off[i];
    const int64_t row = int64_t(seeds[i]);
    const uint32_t deg = a.row_deg[i];
    const uint32_t pos = race_long_row(lds, probs, start, deg, k, rng_seed, rng_stream, row);
    const int l = threadIdx.x;
    if (l < k && pos < deg) {  // wave 0 holds the winners; deg > k: every entry is filled
      out_rows[off + l] = IdT(row);
      out_cols[off + l] = indices.at(start + pos);
    }
  }
}

// With replacement, one G-lane group per row; rows above long_row<G>() are queued.
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
  draw_row<G>(g, probs, start, deg, k, rng_seed, rng_stream, row, [&](int64_t j, int64_t pick) {
    out_rows[off + j] = IdT(row);
    out_cols[off + j] = indices.at(start + pick);
  });
}

// With replacement, queued long rows: a block per row.
template <typename IdT>
__global__ __launch_bounds__(kLongBlock) void fill_weighted_replace_long_kernel(
    const IdT* __restrict__ seeds, RowArgs a, TierView<IdT> indices, TierView<float> probs, int64_t k,
    uint64_t rng_seed, uint32_t rng_stream, IdT* __restrict__ out_rows, IdT* __restrict__ out_cols) {
  __shared__ LongRowScratch lds;
  const int64_t n_long = *a.long_count;
  for (int64_t t = blockIdx.x; t < n_long; t += gridDim.x) {
    const int64_t i = a.long_rows[t];
    const int64_t start = a.row_start[i];
    const int64_t off = a.tile_off[i / kTile] + a.row_off[i];
    const int64_t row = int64_t(seeds[i]);
    const int64_t deg = int64_t(a.row_deg[i]);
    draw_long_row(lds, probs, start, deg, k, rng_seed, rng_stream, row, [&](int64_t j, int64_t pick) {
      out_rows[off + j] = IdT(row);
      out_cols[off + j] = indices.at(start + pick);
    });
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
  if (const int64_t f = debug_option(DGS_DEBUG_WEIGHTED_GROUP)) {  // test hook: 16, 32 or 64
    if ((f == 16 || f == 32 || f == 64) && (replace || k <= f)) group = int(f);
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
  dgs_status s = dgs_sample_count(seeds, id_bytes, n_seeds, indptr, indices.total, num_picks, replace, nnz_dev, nullptr, workspace,
                                  workspace_bytes, stream);
  if (s != DGS_OK) return s;
  return dgs_sample_fill_weighted(seeds, id_bytes, n_seeds, indices, probs, num_picks, replace, rng_seed,
                                  rng_stream, out_rows, out_cols, workspace, workspace_bytes, stream);
}
