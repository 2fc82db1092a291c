// Renumbering of a CSC graph so that row ids follow a given order (hottest rows first): what puts
// the most-used rows of every positional store into its HBM slice.
//
// Given order[new] = old and its inverse rank[old] = new, and the new row offsets (the scan of the
// permuted degrees), one launch writes new_indices: edge e of the new graph lies in the new row r
// with new_indptr[r] <= e < new_indptr[r+1]; it is edge old_indptr[order[r]] + (e - new_indptr[r])
// of the old graph, and its endpoint is renamed through rank.  The order of a row's edges is kept.
// The launch is flat over edges (a hub row costs what its edges cost): a block owns 1024
// consecutive edges, two threads locate the block's first and last row by binary search, every
// thread then searches only inside that range.
#include "common.h"

namespace dgs {
namespace {

constexpr int kBlock = 256;
constexpr int kEdgesPerThread = 4;
constexpr int kEdgesPerBlock = kBlock * kEdgesPerThread;
constexpr int64_t kMaxGrid = 1 << 20;

// largest r in [lo, hi] with ptr[r] <= e (ptr is non-decreasing, ptr[lo] <= e)
template <typename PtrT>
__device__ __forceinline__ int64_t row_of(const PtrT* __restrict__ ptr, int64_t lo, int64_t hi, int64_t e) {
  while (lo < hi) {
    const int64_t mid = lo + (hi - lo + 1) / 2;
    if (int64_t(ptr[mid]) <= e) lo = mid;
    else hi = mid - 1;
  }
  return lo;
}

template <typename IdT, typename PtrT>
__global__ __launch_bounds__(kBlock) void renumber_kernel(const PtrT* __restrict__ old_indptr,
                                                          const IdT* __restrict__ old_indices,
                                                          const int64_t* __restrict__ order,
                                                          const IdT* __restrict__ rank,
                                                          const PtrT* __restrict__ new_indptr, int64_t n_rows,
                                                          int64_t n_edges, IdT* __restrict__ new_indices) {
  __shared__ int64_t range[2];
  for (int64_t tile = blockIdx.x; tile * kEdgesPerBlock < n_edges; tile += gridDim.x) {
    const int64_t first = tile * kEdgesPerBlock;
    const int64_t last = first + kEdgesPerBlock - 1 < n_edges - 1 ? first + kEdgesPerBlock - 1 : n_edges - 1;
    if (threadIdx.x < 2) range[threadIdx.x] = row_of(new_indptr, 0, n_rows - 1, threadIdx.x == 0 ? first : last);
    __syncthreads();
    const int64_t row_lo = range[0], row_hi = range[1];
#pragma unroll
    for (int j = 0; j < kEdgesPerThread; ++j) {
      const int64_t e = first + int64_t(j) * kBlock + threadIdx.x;
      if (e < n_edges) {
        const int64_t r = row_of(new_indptr, row_lo, row_hi, e);
        const int64_t src = int64_t(old_indptr[order[r]]) + (e - int64_t(new_indptr[r]));
        new_indices[e] = rank[old_indices[src]];
      }
    }
    __syncthreads();  // range is rewritten by the block's next tile
  }
}

template <typename IdT, typename PtrT>
dgs_status run(const void* old_indptr, const void* old_indices, const int64_t* order, const void* rank,
               const void* new_indptr, int64_t n_rows, int64_t n_edges, void* new_indices, hipStream_t st) {
  const int64_t tiles = (n_edges + kEdgesPerBlock - 1) / kEdgesPerBlock;
  const uint32_t grid = uint32_t(tiles < kMaxGrid ? tiles : kMaxGrid);
  hipLaunchKernelGGL((renumber_kernel<IdT, PtrT>), dim3(grid), dim3(kBlock), 0, st,
                     static_cast<const PtrT*>(old_indptr), static_cast<const IdT*>(old_indices), order,
                     static_cast<const IdT*>(rank), static_cast<const PtrT*>(new_indptr), n_rows, n_edges,
                     static_cast<IdT*>(new_indices));
  DGS_LAUNCH_CHECK();
  return DGS_OK;
}

}  // namespace
}  // namespace dgs

DGS_API dgs_status dgs_renumber_csc(const void* old_indptr, int32_t ptr_bytes, const void* old_indices,
                                    int32_t id_bytes, const int64_t* order, const void* rank,
                                    const void* new_indptr, int64_t n_rows, int64_t n_edges, void* new_indices,
                                    void* stream) {
  using namespace dgs;
  DGS_REQUIRE(width_ok(ptr_bytes) && width_ok(id_bytes), DGS_ERR_INVALID,
              "renumber_csc: widths %d / %d are not 4 or 8", ptr_bytes, id_bytes);
  DGS_REQUIRE(n_rows >= 0 && n_edges >= 0, DGS_ERR_INVALID, "renumber_csc: n_rows=%lld n_edges=%lld",
              (long long)n_rows, (long long)n_edges);
  if (n_edges == 0) return DGS_OK;
  DGS_REQUIRE(n_rows > 0, DGS_ERR_INVALID, "renumber_csc: %lld edges in a graph without rows", (long long)n_edges);
  DGS_REQUIRE(old_indptr && old_indices && order && rank && new_indptr && new_indices, DGS_ERR_INVALID,
              "renumber_csc: null pointer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (id_bytes == 8)
    return ptr_bytes == 8
               ? run<int64_t, int64_t>(old_indptr, old_indices, order, rank, new_indptr, n_rows, n_edges, new_indices, st)
               : run<int64_t, int32_t>(old_indptr, old_indices, order, rank, new_indptr, n_rows, n_edges, new_indices, st);
  return ptr_bytes == 8
             ? run<int32_t, int64_t>(old_indptr, old_indices, order, rank, new_indptr, n_rows, n_edges, new_indices, st)
             : run<int32_t, int32_t>(old_indptr, old_indices, order, rank, new_indptr, n_rows, n_edges, new_indices, st);
}
