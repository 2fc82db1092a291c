// Scratch layout shared by the count pass and the fills (uniform and weighted) of one hop.
#ifndef DGS_CSRC_SAMPLE_WORKSPACE_H_
#define DGS_CSRC_SAMPLE_WORKSPACE_H_

#include "common.h"

namespace dgs {

constexpr int kTile = 256;  // seeds per block in the count pass, threads per block in the fills

struct SampleWorkspace {
  int64_t* row_start;   // per seed: first edge of its row
  uint32_t* row_deg;    // per seed: degree (0 for rows the count pass flagged)
  int64_t* row_off;     // per seed: first output slot, relative to its 256-seed tile
  int64_t* tile_sum;
  int64_t* tile_off;    // per tile: first output slot
  int* tile_flag;
  int64_t* long_rows;   // weighted fills: seeds whose rows are handed to the block-per-row kernel
  int64_t* long_count;  // [0] = entries of long_rows
};

inline size_t sample_workspace_layout(int64_t n_seeds, void* base, SampleWorkspace* w) {
  const size_t n = size_t(n_seeds < 0 ? 0 : n_seeds);
  const size_t tiles = (n + kTile - 1) / kTile;
  Carver c(base);
  SampleWorkspace tmp;
  tmp.row_start = c.take<int64_t>(n);
  tmp.row_deg = c.take<uint32_t>(n);
  tmp.row_off = c.take<int64_t>(n);
  tmp.tile_sum = c.take<int64_t>(tiles);
  tmp.tile_off = c.take<int64_t>(tiles);
  tmp.tile_flag = c.take<int>(tiles);
  tmp.long_rows = c.take<int64_t>(n);
  tmp.long_count = c.take<int64_t>(1);
  if (w) *w = tmp;
  return c.used + 256;
}

// Argument checks common to the sampling entry points.
inline dgs_status check_sample_args(const char* who, const void* seeds, int32_t id_bytes, int64_t n_seeds,
                                    int64_t num_picks, const void* workspace, size_t workspace_bytes) {
  DGS_REQUIRE(width_ok(id_bytes), DGS_ERR_INVALID, "%s: id width %d is not 4 or 8", who, id_bytes);
  DGS_REQUIRE(n_seeds >= 0 && num_picks >= 0, DGS_ERR_INVALID, "%s: n_seeds=%lld num_picks=%lld", who,
              (long long)n_seeds, (long long)num_picks);
  // the widest fill launch spends one wave on a row: kTile / kWave rows a block, 31-bit grids
  DGS_REQUIRE(n_seeds <= int64_t(0x7fffffff) * (kTile / kWave), DGS_ERR_UNSUPPORTED, "%s: too many seeds", who);
  const size_t need = sample_workspace_layout(n_seeds, nullptr, nullptr);
  DGS_REQUIRE(workspace != nullptr && workspace_bytes >= need, DGS_ERR_WORKSPACE, "%s: workspace of %zu B, need %zu",
              who, workspace_bytes, need);
  DGS_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255) == 0, DGS_ERR_WORKSPACE,
              "%s: workspace must be 256-byte aligned", who);
  DGS_REQUIRE(n_seeds == 0 || seeds != nullptr, DGS_ERR_INVALID, "%s: null seeds", who);
  return DGS_OK;
}

}  // namespace dgs
#endif
