// libdgs.so: the torch-facing layer.  It registers the operator surface of the
// upstream library (src/pybind.cc:11-38) -- torch.classes.dgs_classes.ChunkTensor
// and the torch.ops.dgs_ops free functions on the sampling / relabel / gather
// path -- and does nothing but validate arguments, allocate outputs and
// workspaces with torch, and call the C ABI of libdgs_hip.so on torch's current
// HIP stream.  There is no CPU implementation behind these operators: without
// the HIP library the shared object does not load.
//
// Deliberate differences from upstream, all on the safe side:
//   - argument violations raise (TORCH_CHECK) where upstream aborts the process
//     (CHECK / LOG(FATAL) / exit in src/chunk_tensor.cc:39-40,174-181,
//     src/dgs_headers.h:33-45);
//   - world size is 1: _CAPI_get_unique_id / _CAPI_set_nccl are inert shims and
//     _CAPI_remote_index returns an empty [0, D] tensor;
//   - seeds/indices share one id width but indptr may have the other one;
//   - the store accepts every dtype of 1, 2, 4 or 8 bytes (upstream: i32, i64,
//     f32 only, src/dgs_headers.h:60-74);
//   - random picks come from a counter-based generator whose (seed, stream) is
//     settable; upstream re-seeds the constant 7777 on every call
//     (src/cuda/rowwise_sampling_with_chunk_tensor.cu:162);
//   - seed ids and gather indices outside the graph / the store are refused instead of
//     dereferenced (upstream does not check, src/cuda/index_with_chunk_tensor.cu:16-23):
//     sampling raises; a gather zero-fills the row and the store raises at its next call.
#include <c10/hip/HIPFunctions.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <c10/core/StreamGuard.h>
#include <c10/hip/HIPStream.h>
#include <torch/custom_class.h>
#include <torch/script.h>

#include <atomic>
#include <condition_variable>
#include <deque>
#include <string>
#include <thread>
#include <map>
#include <memory>
#include <mutex>
#include <tuple>
#include <vector>

#include "dgs_hip.h"

namespace dgs {
namespace {

void check(dgs_status s) {
  TORCH_CHECK(s == DGS_OK, "dgs: ", dgs_status_name(s), ": ", dgs_last_error());
}

void* current_stream() { return c10::hip::getCurrentHIPStream().stream(); }

// A ticket (an event recorded on a stream) that several parties look at: the host thread that
// waits for a batch's lengths, the next batch's gather waiting its turn, the owner of a node table.
// Every event between two kernels costs the GPU about 6 us of idling, so a batch records ONE, behind
// its last launch, and shares it; it goes back to the library's pool when the last holder lets go.
struct SharedTicket {
  void* handle = nullptr;
  SharedTicket() = default;
  SharedTicket(const SharedTicket&) = delete;
  SharedTicket& operator=(const SharedTicket&) = delete;
  ~SharedTicket() {
    if (handle != nullptr) dgs_ticket_release(handle);
  }
};
using TicketRef = std::shared_ptr<SharedTicket>;
TicketRef record_ticket(void* stream) {
  auto t = std::make_shared<SharedTicket>();
  check(dgs_ticket_record(stream, &t->handle));
  return t;
}

#define DGS_CHECK_GPU(x) TORCH_CHECK((x).device().is_cuda(), #x " must be a GPU tensor")

int32_t id_width(const torch::Tensor& t, const char* what) {
  TORCH_CHECK(t.scalar_type() == torch::kInt32 || t.scalar_type() == torch::kInt64, what,
              " must be int32 or int64, got ", t.scalar_type());
  return t.scalar_type() == torch::kInt64 ? 8 : 4;
}

torch::Tensor device_bytes(size_t n, const torch::Device& dev) {
  // torch's caching allocator hands out 512-byte aligned blocks
  return torch::empty({static_cast<int64_t>(n)}, torch::TensorOptions().dtype(torch::kUInt8).device(dev));
}

// Blocking read of a few int64 values from the device through a pinned buffer.
std::vector<int64_t> read_back(const torch::Tensor& dev, int64_t count) {
  thread_local torch::Tensor pinned =
      torch::empty({32}, torch::TensorOptions().dtype(torch::kInt64).pinned_memory(true));
  TORCH_CHECK(count <= 32);
  check(dgs_read_back(pinned.data_ptr(), dev.data_ptr(), sizeof(int64_t) * count, current_stream()));
  const int64_t* p = pinned.data_ptr<int64_t>();
  return std::vector<int64_t>(p, p + count);
}

// ---- generator state for the sampling ops ------------------------------------
std::mutex g_rng_mutex;
uint64_t g_rng_seed = 7777;  // upstream's constant, used until the caller sets one
uint32_t g_rng_stream = 0;   // advanced by one per sampling call

// Reserves `calls` consecutive streams and returns (seed, first stream).
std::pair<uint64_t, uint32_t> next_rng(uint32_t calls = 1) {
  std::lock_guard<std::mutex> lock(g_rng_mutex);
  const uint32_t first = g_rng_stream;
  g_rng_stream += calls;
  return {g_rng_seed, first};
}

// Above this many bytes a worst-case feature buffer is not allocated: the fused operator waits
// for the frontier's size and allocates exactly (see PendingBlocks::Begin).
std::atomic<int64_t> g_gather_buffer_cap{int64_t(2) << 30};

// Node tables (8 bytes per node and stream, persistent) for the fused operators: graphs up to this
// many nodes get them, larger ones build a hash table per call in the call's workspace.
// -1: every graph that dgs_node_table_bytes accepts (below 8 GiB per table).
std::atomic<int64_t> g_node_table_max_nodes{-1};

// What the error bits of a sampling call mean (include/dgs_hip.h, sizes_dev / nnz_dev flags).
void check_sampling_flags(int64_t flags, const char* who, int hop) {
  if (flags == 0) return;
  const std::string where = hop >= 0 ? std::string(who) + ": hop " + std::to_string(hop) : std::string(who);
  TORCH_CHECK((flags & 2) == 0, where, ": a seed id is not a row of the graph (outside 0 .. nodes - 1)");
  TORCH_CHECK((flags & 4) == 0, where, ": a neighbour id stored in the graph is not a node (outside 0 .. nodes - 1)");
  TORCH_CHECK((flags & 1) == 0, where, ": a seed row has a degree of 2^32 or more, or offsets outside the edge array");
  TORCH_CHECK((flags & 8) == 0, where, ": the ids of this hop crowd one bucket of the on-chip pass that finds first "
              "occurrences (more distinct ids in a bucket than its table holds); sample on the node table instead "
              "(dgs_debug_set(DGS_DEBUG_SAMPLER_BUCKETED, 1))");
  TORCH_CHECK(false, where, ": error bits ", flags);
}

}  // namespace

// ---------------------------------------------------------------------------------
// ChunkTensor (upstream src/chunk_tensor.h:61-106)
// ---------------------------------------------------------------------------------
class ChunkTensor : public torch::CustomClassHolder {
 public:
  ChunkTensor(std::vector<int64_t> shapes, torch::ScalarType dtype, int64_t capacity_per_gpu)
      : shapes_(std::move(shapes)), dtype_(dtype) {
    TORCH_CHECK(shapes_.size() == 1 || shapes_.size() == 2, "ChunkTensor: shapes must have 1 or 2 entries, got ",
                shapes_.size());
    TORCH_CHECK(capacity_per_gpu >= 0, "ChunkTensor: capacity_per_gpu must be >= 0, got ", capacity_per_gpu);
    strides_.resize(shapes_.size());
    int64_t stride = 1;
    for (int i = static_cast<int>(shapes_.size()) - 1; i >= 0; --i) {
      TORCH_CHECK(shapes_[i] >= 0, "ChunkTensor: negative extent");
      strides_[i] = stride;
      stride *= shapes_[i];
    }
    elem_stride_ = strides_[0];
    total_ = stride;
    const size_t eb = c10::elementSize(dtype_);
    TORCH_CHECK(eb == 1 || eb == 2 || eb == 4 || eb == 8, "ChunkTensor: unsupported dtype ", dtype_);
    check(dgs_store_create(total_, static_cast<int32_t>(eb), capacity_per_gpu, &store_));
    check(dgs_store_view(store_, &view_));
    // torch on ROCm names its GPU device type CUDA; only the index comes from the HIP stream
    device_ = c10::Device(c10::DeviceType::CUDA, c10::hip::getCurrentHIPStream().device_index());
    // the word a gather sets when it meets an index outside the store (pinned: the host reads it
    // without a copy, the kernels write it through its device mapping)
    bad_index_ = torch::zeros({1}, torch::TensorOptions().dtype(torch::kInt64).pinned_memory(true));
  }
  ~ChunkTensor() override { dgs_store_destroy(store_); }

  // Raises if a gather that has run since the last check met an index outside the rows it may
  // read (those output rows were zero-filled).  Gathers are asynchronous, so the error surfaces
  // at the store's next operator call, or here after a synchronisation.
  void CheckErrors() {
    int64_t* w = bad_index_.data_ptr<int64_t>();
    if (__atomic_load_n(w, __ATOMIC_RELAXED) != 0) {
      __atomic_store_n(w, int64_t(0), __ATOMIC_RELAXED);
      TORCH_CHECK(false, "ChunkTensor: an earlier gather was given row ids outside the store (or outside the "
                         "tier of _CAPI_local_index / _CAPI_host_index); those output rows were filled with zeros");
    }
  }
  void SynchronizeAndCheck() {
    void* ticket = nullptr;
    check(dgs_ticket_record(current_stream(), &ticket));
    check(dgs_ticket_wait(ticket));
    CheckErrors();
  }
  int64_t* bad_index_word() const { return bad_index_.data_ptr<int64_t>(); }

  // upstream GetHostTensor (src/chunk_tensor.cc:151-160): flat, non-owning
  torch::Tensor GetHostTensor() {
    void* p = nullptr;
    int64_t n = 0;
    check(dgs_store_slices(store_, nullptr, nullptr, &p, &n));
    auto opt = torch::TensorOptions().device(torch::kCPU).dtype(dtype_);
    return n > 0 ? torch::from_blob(p, {n}, opt) : torch::empty({0}, opt);
  }

  // upstream GetSubDeviceTensor (src/chunk_tensor.cc:162-171): flat, non-owning
  torch::Tensor GetSubDeviceTensor() {
    void* p = nullptr;
    int64_t n = 0;
    check(dgs_store_slices(store_, &p, &n, nullptr, nullptr));
    auto opt = torch::TensorOptions().device(device_).dtype(dtype_);
    return n > 0 ? torch::from_blob(p, {n}, opt) : torch::empty({0}, opt);
  }

  // upstream LoadFromTensor (src/chunk_tensor.cc:173-200)
  void LoadFromTensor(torch::Tensor data) {
    TORCH_CHECK(static_cast<size_t>(data.dim()) == shapes_.size(), "load_from_tensor: expected ", shapes_.size(),
                " dimensions, got ", data.dim());
    TORCH_CHECK(data.scalar_type() == dtype_, "load_from_tensor: expected dtype ", dtype_, ", got ",
                data.scalar_type());
    TORCH_CHECK(data.device().is_cpu(), "load_from_tensor: data must be a CPU tensor");
    for (size_t i = 0; i < shapes_.size(); ++i) {
      TORCH_CHECK(data.size(i) == shapes_[i], "load_from_tensor: extent ", i, " is ", data.size(i), ", expected ",
                  shapes_[i]);
      TORCH_CHECK(data.size(i) <= 1 || data.stride(i) == strides_[i], "load_from_tensor: data must be contiguous");
    }
    check(dgs_store_load(store_, data.data_ptr(), total_));
  }

  torch::Tensor Gather(const torch::Tensor& index_in, int32_t tier) {
    CheckErrors();
    DGS_CHECK_GPU(index_in);
    const int32_t w = id_width(index_in, "index");
    torch::Tensor index = index_in.contiguous();
    const int64_t n = index.numel();
    torch::Tensor out = torch::empty({n, elem_stride_}, torch::TensorOptions().dtype(dtype_).device(index.device()));
    check(dgs_gather_rows(view_, elem_stride_, index.data_ptr(), w, n, out.data_ptr(), tier, bad_index_word(),
                          current_stream()));
    return out;
  }
  // upstream Index / LocalIndex / RemoteIndex / HostIndex (src/chunk_tensor.cc:207-221)
  torch::Tensor Index(torch::Tensor index) { return Gather(index, DGS_TIER_ANY); }
  torch::Tensor LocalIndex(torch::Tensor index) { return Gather(index, DGS_TIER_DEVICE); }
  torch::Tensor HostIndex(torch::Tensor index) { return Gather(index, DGS_TIER_HOST); }
  torch::Tensor RemoteIndex(torch::Tensor index) {
    DGS_CHECK_GPU(index);
    TORCH_CHECK(index.numel() == 0, "_CAPI_remote_index: there is no peer tier at world size 1, but ", index.numel(),
                " rows were requested");
    return torch::empty({0, elem_stride_}, torch::TensorOptions().dtype(dtype_).device(index.device()));
  }

  // upstream SplitIndex (src/chunk_tensor.cc:202-205)
  std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> SplitIndex(torch::Tensor index_in) {
    CheckErrors();
    DGS_CHECK_GPU(index_in);
    const int32_t w = id_width(index_in, "index");
    torch::Tensor index = index_in.contiguous().view({-1});
    const int64_t n = index.numel();
    torch::Tensor local = torch::empty_like(index);
    torch::Tensor host = torch::empty_like(index);
    torch::Tensor counts = torch::empty({2}, index.options().dtype(torch::kInt64));
    const size_t ws_bytes = dgs_split_index_workspace_bytes(n);
    torch::Tensor ws = device_bytes(ws_bytes, index.device());
    check(dgs_split_index(view_, elem_stride_, index.data_ptr(), w, n, local.data_ptr(), host.data_ptr(),
                          counts.data_ptr<int64_t>(), ws.data_ptr(), ws_bytes, current_stream()));
    const std::vector<int64_t> c = read_back(counts, 2);
    return std::make_tuple(local.narrow(0, 0, c[0]), torch::empty({0}, index.options()), host.narrow(0, 0, c[1]));
  }

  // Persistent direct-address table for sample_blocks when this store is a graph's indptr
  // (one entry per node).  Created on first use; returns (pointer, epoch for this call).
  // Calls in flight on different streams must not share a table, so there is one per stream
  // (up to kMaxNodeTables; further streams get none and the call uses a hash table instead).
  // Two calls on the same stream share their table one after the other, which is only right if
  // all launches of the first precede all launches of the second: the caller holds
  // enqueue_lock() from before this call until node_table_used() behind its last launch that
  // reads the table.
  std::unique_lock<std::mutex> enqueue_lock() { return std::unique_lock<std::mutex>(node_table_mutex_); }
  // When every table belongs to another stream, the caller takes over the one used longest ago
  // among those whose last call has finished (a stream that is no longer used, such as one made
  // per epoch).  "Finished" is asked of a ticket recorded behind that call (node_table_used),
  // never of the other stream's handle, which may have been destroyed since.  If all tables are
  // busy the caller gets none and its call builds a hash table in its workspace.
  std::pair<void*, uint32_t> node_table(void* stream) {
    const int64_t n_nodes = total_ - 1;
    const size_t bytes = dgs_node_table_bytes(n_nodes);
    if (bytes == 0 || bytes > (size_t(8) << 30)) return {nullptr, 0u};
    const int64_t max_nodes = g_node_table_max_nodes.load();
    if (max_nodes >= 0 && n_nodes > max_nodes) return {nullptr, 0u};
    auto it = node_tables_.find(stream);
    if (it == node_tables_.end()) {
      if (node_tables_.size() >= kMaxNodeTables) {
        auto pick = node_tables_.end();
        for (auto jt = node_tables_.begin(); jt != node_tables_.end(); ++jt) {
          int32_t finished = 1;  // a table that was handed out and never used has nothing pending
          if (jt->second.done) check(dgs_ticket_query(jt->second.done->handle, &finished));
          if (finished && (pick == node_tables_.end() || jt->second.last_use < pick->second.last_use)) pick = jt;
        }
        if (pick == node_tables_.end()) return {nullptr, 0u};
        NodeTable taken = std::move(pick->second);
        node_tables_.erase(pick);
        // the memory came from another stream's pool: it must not be handed out again while
        // this stream still uses it
        // (torch on ROCm files its allocations under the device type CUDA, hence the stream type)
        if (taken.entries.defined())
          taken.entries.record_stream(c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().unwrap());
        it = node_tables_.emplace(stream, std::move(taken)).first;
      } else {
        it = node_tables_.emplace(stream, NodeTable{}).first;
      }
    }
    NodeTable& t = it->second;
    if (!t.entries.defined() || t.epoch >= 0xffffff00u) {
      t.entries = torch::full({static_cast<int64_t>(bytes / 8)}, int64_t(-1),
                              torch::TensorOptions().dtype(torch::kInt64).device(device_));
      t.epoch = 0;
    }
    t.last_use = ++uses_;
    return {t.entries.data_ptr(), ++t.epoch};
  }
  // Says when the call that just used `stream`'s table will have finished with it: at `done`, a
  // ticket recorded on the stream behind the call's last launch that reads the table (or later).
  // (Called with enqueue_lock() held.)
  void node_table_used(void* stream, TicketRef done) {
    auto it = node_tables_.find(stream);
    if (it != node_tables_.end()) it->second.done = std::move(done);
  }
  // Gives up the node table of a stream (0: the current stream), e.g. before the stream is
  // destroyed; returns whether there was one.  Kernels of earlier calls that still use the table
  // keep their memory: torch's allocator hands a block out again in stream order only.
  bool ReleaseNodeTable(int64_t stream_handle) {
    const std::unique_lock<std::mutex> lock = enqueue_lock();
    void* key = stream_handle != 0 ? reinterpret_cast<void*>(static_cast<intptr_t>(stream_handle)) : current_stream();
    auto it = node_tables_.find(key);
    if (it == node_tables_.end()) return false;
    node_tables_.erase(it);
    return true;
  }
  int64_t NodeTableCount() {
    const std::unique_lock<std::mutex> lock = enqueue_lock();
    return static_cast<int64_t>(node_tables_.size());
  }

  // Final frontier size of the last fused batch that finished on this graph (0: none yet): what
  // the next batch's feature gather is sized for.  Batches of very different sizes on one graph
  // make it a poor guess, never a wrong result.
  int64_t frontier_hint() const { return frontier_hint_.load(std::memory_order_relaxed); }
  void set_frontier_hint(int64_t rows) { frontier_hint_.store(rows, std::memory_order_relaxed); }

  const dgs_view& view() const { return view_; }
  c10::Device device() const { return device_; }
  torch::ScalarType dtype() const { return dtype_; }
  int64_t elem_stride() const { return elem_stride_; }

 private:
  std::vector<int64_t> shapes_;
  std::vector<int64_t> strides_;
  torch::ScalarType dtype_;
  int64_t elem_stride_ = 1;
  int64_t total_ = 0;
  dgs_store* store_ = nullptr;
  dgs_view view_{};
  c10::Device device_{c10::DeviceType::CUDA, 0};
  torch::Tensor bad_index_;
  struct NodeTable {
    torch::Tensor entries;
    uint32_t epoch = 0;
    uint64_t last_use = 0;
    TicketRef done;  // ticket behind the last call that used the table (none: never used)
  };
  uint64_t uses_ = 0;
  std::atomic<int64_t> frontier_hint_{0};
  static constexpr size_t kMaxNodeTables = 4;
  std::map<void*, NodeTable> node_tables_;
  std::mutex node_table_mutex_;
};

namespace {

dgs_view tensor_view(const torch::Tensor& t) {
  dgs_view v{};
  v.dev = t.data_ptr();
  v.host = nullptr;
  v.threshold = t.numel();
  v.total = t.numel();
  v.elem_bytes = static_cast<int32_t>(t.element_size());
  return v;
}

// Shared body of the sampling operators; `probs` is null for the uniform ones.
std::tuple<torch::Tensor, torch::Tensor> sample_impl(const torch::Tensor& seeds_in, const dgs_view& indptr,
                                                     const dgs_view& indices, torch::ScalarType indices_dtype,
                                                     int64_t num_picks, bool replace,
                                                     const dgs_view* probs = nullptr) {
  DGS_CHECK_GPU(seeds_in);
  const int32_t w = id_width(seeds_in, "seeds");
  TORCH_CHECK(seeds_in.scalar_type() == indices_dtype, "seeds (", seeds_in.scalar_type(), ") and indices (",
              indices_dtype, ") must have the same dtype");
  TORCH_CHECK(indptr.elem_bytes == 4 || indptr.elem_bytes == 8, "indptr must be int32 or int64");
  TORCH_CHECK(num_picks >= 0, "num_picks must be >= 0, got ", num_picks);
  if (probs != nullptr) {
    TORCH_CHECK(probs->total == indices.total, "probs holds ", probs->total, " weights for ", indices.total,
                " edges");
    TORCH_CHECK(replace || num_picks <= 64,
                "weighted sampling without replacement supports num_picks <= 64, got ", num_picks);
  }
  torch::Tensor seeds = seeds_in.contiguous().view({-1});
  const int64_t n = seeds.numel();
  const auto rng = next_rng();
  void* st = current_stream();

  const size_t ws_bytes = dgs_sample_workspace_bytes(n);
  torch::Tensor ws = device_bytes(ws_bytes, seeds.device());
  torch::Tensor nnz_dev = torch::empty({2}, seeds.options().dtype(torch::kInt64));

  // Worst case n * num_picks ids per output: when that is modest (two buffers of at most 256 MB,
  // of which the results are prefixes) the whole hop is enqueued before the one blocking length
  // read; otherwise count first and allocate exactly.
  const bool one_shot = num_picks <= (int64_t(1) << 20) && n * num_picks <= (int64_t(1) << 25);
  torch::Tensor rows, cols;
  std::vector<int64_t> len;
  if (one_shot) {
    rows = torch::empty({n * num_picks}, seeds.options());
    cols = torch::empty({n * num_picks}, seeds.options());
    // count (which mirrors the length into pinned memory), then the fill: the host waits for the
    // mirrored words only, and the fill is still running when the operator returns
    thread_local torch::Tensor pinned =
        torch::empty({2}, torch::TensorOptions().dtype(torch::kInt64).pinned_memory(true));
    int64_t* words = pinned.data_ptr<int64_t>();
    words[0] = words[1] = -1;  // the kernel's words are never negative: the wait below polls them
    check(dgs_sample_count(seeds.data_ptr(), w, n, indptr, indices.total, num_picks, replace, nnz_dev.data_ptr<int64_t>(), words,
                           ws.data_ptr(), ws_bytes, st));
    const dgs_status fill_status =
        probs != nullptr
            ? dgs_sample_fill_weighted(seeds.data_ptr(), w, n, indices, *probs, num_picks, replace, rng.first,
                                       rng.second, rows.data_ptr(), cols.data_ptr(), ws.data_ptr(), ws_bytes, st)
            : dgs_sample_fill(seeds.data_ptr(), w, n, indices, num_picks, replace, rng.first, rng.second,
                              rows.data_ptr(), cols.data_ptr(), ws.data_ptr(), ws_bytes, st);
    check(dgs_stream_wait_words(st, words, 2));
    check(fill_status);
    TORCH_CHECK(words[0] >= 0 && words[1] >= 0, "sample_neighbors: the count kernel left no lengths");
    len.assign(words, words + 2);
  } else {
    check(dgs_sample_count(seeds.data_ptr(), w, n, indptr, indices.total, num_picks, replace, nnz_dev.data_ptr<int64_t>(), nullptr,
                           ws.data_ptr(), ws_bytes, st));
    len = read_back(nnz_dev, 2);
    rows = torch::empty({len[0]}, seeds.options());
    cols = torch::empty({len[0]}, seeds.options());
    if (probs != nullptr)
      check(dgs_sample_fill_weighted(seeds.data_ptr(), w, n, indices, *probs, num_picks, replace, rng.first,
                                     rng.second, rows.data_ptr(), cols.data_ptr(), ws.data_ptr(), ws_bytes, st));
    else
      check(dgs_sample_fill(seeds.data_ptr(), w, n, indices, num_picks, replace, rng.first, rng.second,
                            rows.data_ptr(), cols.data_ptr(), ws.data_ptr(), ws_bytes, st));
  }
  check_sampling_flags(len[1], "sample_neighbors", -1);
  return std::make_tuple(rows.narrow(0, 0, len[0]), cols.narrow(0, 0, len[0]));
}

// upstream RowWiseSamplingUniformCUDA (src/cuda/rowwise_sampling.cu:176-187)
std::tuple<torch::Tensor, torch::Tensor> SampleNeighbors(torch::Tensor seeds, torch::Tensor indptr,
                                                         torch::Tensor indices, int64_t num_picks, bool replace) {
  DGS_CHECK_GPU(indptr);
  DGS_CHECK_GPU(indices);
  id_width(indptr, "indptr");
  id_width(indices, "indices");
  torch::Tensor ip = indptr.contiguous();
  torch::Tensor ix = indices.contiguous();
  return sample_impl(seeds, tensor_view(ip), tensor_view(ix), ix.scalar_type(), num_picks, replace);
}

// upstream RowWiseSamplingUniformWithChunkTensorCUDA
// (src/cuda/rowwise_sampling_with_chunk_tensor.cu:185-194)
std::tuple<torch::Tensor, torch::Tensor> SampleNeighborsWithChunkTensor(torch::Tensor seeds,
                                                                        c10::intrusive_ptr<ChunkTensor> indptr,
                                                                        c10::intrusive_ptr<ChunkTensor> indices,
                                                                        int64_t num_picks, bool replace) {
  TORCH_CHECK(indptr->dtype() == torch::kInt32 || indptr->dtype() == torch::kInt64,
              "indptr store must be int32 or int64");
  return sample_impl(seeds, indptr->view(), indices->view(), indices->dtype(), num_picks, replace);
}

// upstream RowWiseSamplingProbCUDA (src/cuda/rowwise_sampling_probs.cu:265-279)
std::tuple<torch::Tensor, torch::Tensor> SampleNeighborsWithProbs(torch::Tensor seeds, torch::Tensor indptr,
                                                                  torch::Tensor indices, torch::Tensor probs,
                                                                  int64_t num_picks, bool replace) {
  DGS_CHECK_GPU(indptr);
  DGS_CHECK_GPU(indices);
  DGS_CHECK_GPU(probs);
  id_width(indptr, "indptr");
  id_width(indices, "indices");
  TORCH_CHECK(probs.scalar_type() == torch::kFloat32, "probs must be float32, got ", probs.scalar_type());
  torch::Tensor ip = indptr.contiguous();
  torch::Tensor ix = indices.contiguous();
  torch::Tensor pr = probs.contiguous().view({-1});
  const dgs_view pv = tensor_view(pr);
  return sample_impl(seeds, tensor_view(ip), tensor_view(ix), ix.scalar_type(), num_picks, replace, &pv);
}

// upstream RowWiseSamplingProbWithChunkTensorCUDA
// (src/cuda/rowwise_sampling_probs_with_chunk_tensor.cu:281-293)
std::tuple<torch::Tensor, torch::Tensor> SampleNeighborsWithProbsWithChunkTensor(
    torch::Tensor seeds, c10::intrusive_ptr<ChunkTensor> indptr, c10::intrusive_ptr<ChunkTensor> indices,
    c10::intrusive_ptr<ChunkTensor> probs, int64_t num_picks, bool replace) {
  TORCH_CHECK(indptr->dtype() == torch::kInt32 || indptr->dtype() == torch::kInt64,
              "indptr store must be int32 or int64");
  TORCH_CHECK(probs->dtype() == torch::kFloat32, "probs store must be float32, got ", probs->dtype());
  const dgs_view pv = probs->view();
  return sample_impl(seeds, indptr->view(), indices->view(), indices->dtype(), num_picks, replace, &pv);
}

// Not in upstream: the graph renumbered so that new id r is old id order[r] (stable, e.g. by
// decreasing degree).  Returns (new_indptr, new_indices, rank) with rank[old] = new.
std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> RenumberCSC(torch::Tensor indptr, torch::Tensor indices,
                                                                    torch::Tensor order) {
  DGS_CHECK_GPU(indptr);
  DGS_CHECK_GPU(indices);
  DGS_CHECK_GPU(order);
  const int32_t pw = id_width(indptr, "indptr");
  const int32_t iw = id_width(indices, "indices");
  TORCH_CHECK(order.scalar_type() == torch::kInt64, "order must be int64, got ", order.scalar_type());
  TORCH_CHECK(indptr.dim() == 1 && indptr.numel() >= 1, "indptr must be 1-D with n + 1 entries");
  const int64_t n = indptr.numel() - 1;
  TORCH_CHECK(order.dim() == 1 && order.numel() == n, "order holds ", order.numel(), " ids for ", n, " rows");
  torch::Tensor ip = indptr.contiguous();
  torch::Tensor ix = indices.contiguous().view({-1});
  torch::Tensor ord = order.contiguous();
  // rank = inverse permutation; it doubles as the check that order is one
  torch::Tensor rank = torch::full({n}, -1, ix.options());
  rank.index_put_({ord}, torch::arange(n, ix.options()));
  TORCH_CHECK(n == 0 || rank.min().item<int64_t>() >= 0, "order is not a permutation of the row ids");
  torch::Tensor deg = ip.slice(0, 1) - ip.slice(0, 0, n);
  torch::Tensor new_ip = torch::zeros({n + 1}, ip.options());
  if (n > 0) new_ip.slice(0, 1).copy_(deg.index_select(0, ord).cumsum(0));
  torch::Tensor new_ix = torch::empty_like(ix);
  check(dgs_renumber_csc(ip.data_ptr(), pw, ix.data_ptr(), iw, ord.data_ptr<int64_t>(), rank.data_ptr(),
                         new_ip.data_ptr(), n, ix.numel(), new_ix.data_ptr(), current_stream()));
  return std::make_tuple(new_ip, new_ix, rank);
}

// Packs up to DGS_MAX_SEGMENTS tensors; more are concatenated first.
dgs_segments pack_segments(std::vector<torch::Tensor>& tensors, std::vector<torch::Tensor>& keep_alive) {
  dgs_segments s{};
  if (tensors.size() > DGS_MAX_SEGMENTS) {
    torch::Tensor all = torch::cat(tensors, 0);
    keep_alive.push_back(all);
    s.count = 1;
    s.ptr[0] = all.data_ptr();
    s.len[0] = all.numel();
    return s;
  }
  s.count = static_cast<int32_t>(tensors.size());
  for (size_t i = 0; i < tensors.size(); ++i) {
    tensors[i] = tensors[i].contiguous().view({-1});
    keep_alive.push_back(tensors[i]);
    s.ptr[i] = tensors[i].data_ptr();
    s.len[i] = tensors[i].numel();
  }
  return s;
}

// upstream TensorRelabelCUDA (src/cuda/tensor_reindex.cu:182-205)
std::tuple<torch::Tensor, std::vector<torch::Tensor>> TensorRelabel(std::vector<torch::Tensor> mapping_tensors,
                                                                    std::vector<torch::Tensor> requiring_relabel_tensors) {
  TORCH_CHECK(!mapping_tensors.empty(), "tensor_relabel: mapping_tensors is empty");
  const torch::ScalarType dt = mapping_tensors[0].scalar_type();
  const int32_t w = id_width(mapping_tensors[0], "mapping tensors");
  const torch::Device dev = mapping_tensors[0].device();
  for (const auto& t : mapping_tensors) {
    DGS_CHECK_GPU(t);
    TORCH_CHECK(t.scalar_type() == dt, "tensor_relabel: all tensors must share one dtype");
  }
  for (const auto& t : requiring_relabel_tensors) {
    DGS_CHECK_GPU(t);
    TORCH_CHECK(t.scalar_type() == dt, "tensor_relabel: all tensors must share one dtype");
  }
  std::vector<torch::Tensor> keep;
  dgs_segments map_seg = pack_segments(mapping_tensors, keep);
  int64_t n = 0;
  for (int i = 0; i < map_seg.count; ++i) n += map_seg.len[i];

  // outputs: one flat buffer split like the inputs (upstream split_with_sizes, :201-202)
  std::vector<int64_t> sizes;
  int64_t m = 0;
  for (const auto& t : requiring_relabel_tensors) {
    sizes.push_back(t.numel());
    m += t.numel();
  }
  auto opt = torch::TensorOptions().dtype(dt).device(dev);
  torch::Tensor relabelled = torch::empty({m}, opt);
  dgs_segments req_seg = pack_segments(requiring_relabel_tensors, keep);
  dgs_segments out_seg{};
  out_seg.count = req_seg.count;
  {
    char* p = static_cast<char*>(relabelled.data_ptr());
    for (int i = 0; i < req_seg.count; ++i) {
      out_seg.ptr[i] = p;
      out_seg.len[i] = req_seg.len[i];
      p += req_seg.len[i] * w;
    }
  }
  torch::Tensor unique = torch::empty({n}, opt);
  torch::Tensor counts = torch::empty({2}, opt.dtype(torch::kInt64));
  const size_t ws_bytes = dgs_unique_relabel_workspace_bytes(n, w);
  torch::Tensor ws = device_bytes(ws_bytes, dev);
  // The kernels mirror the counts into pinned memory as soon as they are final, and the host
  // waits for that point only: the kernels that write `unique` and the relabelled ids are still
  // running when the operator returns (its results are ordered on the stream as always).
  thread_local torch::Tensor pinned =
      torch::empty({2}, torch::TensorOptions().dtype(torch::kInt64).pinned_memory(true));
  int64_t* counts_host = pinned.data_ptr<int64_t>();
  // 8-byte ids first go into one-word slots (one atomic per id); an id of 2^32 - 1 or more voids
  // that attempt and the call is repeated with the two-array table
  int64_t u = 0;
  for (const int32_t packed : {1, 0}) {
    counts_host[0] = counts_host[1] = -1;  // the kernels' words are never negative: the wait polls them
    check(dgs_unique_relabel(map_seg, req_seg, w, packed, unique.data_ptr(), counts.data_ptr<int64_t>(), counts_host,
                             nullptr, out_seg, ws.data_ptr(), ws_bytes, current_stream()));
    check(dgs_stream_wait_words(current_stream(), counts_host, 2));
    TORCH_CHECK(counts_host[0] >= 0 && counts_host[1] >= 0, "tensor_relabel: the kernels left no counts");
    u = counts_host[0];
    if (counts_host[1] == 0) break;
    TORCH_CHECK(packed != 0, "tensor_relabel: the table rejected an id");
  }
  return std::make_tuple(unique.narrow(0, 0, u), relabelled.split_with_sizes(sizes, 0));
}

using BlocksResult = std::tuple<std::vector<torch::Tensor>, std::vector<torch::Tensor>, std::vector<torch::Tensor>,
                                torch::Tensor, torch::Tensor>;

}  // namespace

// A sample_blocks call whose kernels are enqueued but whose lengths have not been read yet.
// Finish() waits for the lengths (not for the relabel of the last hop or the gather, which stay
// queued on the call's stream) and cuts the worst-case buffers to size.  Holding several of these
// on different streams keeps one batch's gather and the next batch's sampling on the GPU together.
class PendingBlocks : public torch::CustomClassHolder {
 public:
  PendingBlocks() = default;
  ~PendingBlocks() override {
    // a batch nobody finished: its kernels still write the pinned words, which must outlive them
    if (!finished_ && end_) dgs_ticket_sync(end_->handle);
  }

  BlocksResult Finish() {
    TORCH_CHECK(!finished_, "PendingBlocks: already finished");
    finished_ = true;
    // the lengths are mirrored into the pinned words when the last hop's compaction has run, well
    // before the batch's end: the words are polled, and the batch's ticket only bounds the wait
    dgs_status ws_status = DGS_OK;
    if (end_) ws_status = dgs_ticket_sync_words(end_->handle, pinned_.data_ptr<int64_t>(), 3 * hops_ + 1);
    check(gather_status_);
    check(ws_status);
    const int64_t* sizes_host = pinned_.data_ptr<int64_t>();
    const int n_sizes = 3 * hops_ + 1;
    for (int i = 0; i < n_sizes; ++i) TORCH_CHECK(sizes_host[i] >= 0, "sample_blocks: the kernels left no lengths");
    const std::vector<int64_t> sz(sizes_host, sizes_host + n_sizes);
    std::vector<torch::Tensor> frontier(hops_);
    for (int h = 0; h < hops_; ++h) {
      check_sampling_flags(sz[2 * hops_ + 1 + h], "sample_blocks", h);
      frontier[h] = all_.narrow(0, 0, sz[h + 1]);
      src_[h] = src_[h].narrow(0, 0, sz[hops_ + 1 + h]);
      dst_[h] = dst_[h].narrow(0, 0, sz[hops_ + 1 + h]);
    }
    if (indptr_) indptr_->set_frontier_hint(sz[hops_]);
    if (features_) {
      const int64_t rows = sz[hops_];
      if (rows <= x_rows_) {
        x_ = x_.narrow(0, 0, rows);
      } else {
        // the frontier did not fit the capped buffer and the gather enqueued behind the last hop
        // wrote nothing: gather now into exactly `rows` rows, on the stream the batch was begun on
        // (the lengths are final, so the frontier is complete)
        const c10::StreamGuard on_begin_stream(stream_);
        x_ = torch::empty({rows, features_->elem_stride()}, x_.options());
        check(dgs_gather_rows(features_->view(), features_->elem_stride(), all_.data_ptr(), width_, rows,
                              x_.data_ptr(), DGS_TIER_ANY, features_->bad_index_word(), current_stream()));
        gathered_late_ = true;
      }
    }
    return std::make_tuple(frontier, src_, dst_, features_ ? x_ : torch::empty({0}, seeds_.options()), seeds_);
  }

  static c10::intrusive_ptr<PendingBlocks> Begin(const torch::Tensor& seeds_in,
                                                 const c10::intrusive_ptr<ChunkTensor>& indptr,
                                                 const c10::intrusive_ptr<ChunkTensor>& indices,
                                                 const std::vector<int64_t>& fanouts, bool replace,
                                                 const c10::intrusive_ptr<ChunkTensor>& features,
                                                 const c10::intrusive_ptr<ChunkTensor>& probs =
                                                     c10::intrusive_ptr<ChunkTensor>(),
                                                 const std::pair<uint64_t, uint32_t>* own_rng = nullptr,
                                                 void* gather_after = nullptr) {
    const int32_t w = id_width(seeds_in, "seeds");
    if (features) features->CheckErrors();
    if (probs) TORCH_CHECK(probs->dtype() == torch::kFloat32, "probs store must be float32, got ", probs->dtype());
    TORCH_CHECK(seeds_in.scalar_type() == indices->dtype(), "seeds (", seeds_in.scalar_type(), ") and indices (",
                indices->dtype(), ") must have the same dtype");
    TORCH_CHECK(indptr->dtype() == torch::kInt32 || indptr->dtype() == torch::kInt64,
                "indptr store must be int32 or int64");
    const int32_t hops = static_cast<int32_t>(fanouts.size());
    TORCH_CHECK(hops >= 1 && hops <= DGS_MAX_HOPS, "sample_blocks: between 1 and ", DGS_MAX_HOPS, " fanouts");
    const int64_t n = seeds_in.numel();
    std::vector<int64_t> seeds_max(hops + 1), edges_max(hops);
    check(dgs_sample_blocks_plan(n, fanouts.data(), hops, seeds_max.data(), edges_max.data()));
    const int n_sizes = 3 * hops + 1;
    TORCH_CHECK(n_sizes <= 32);

    const c10::Device dev = indptr->device();
    TORCH_CHECK(seeds_in.device().is_cpu() || seeds_in.device() == dev, "seeds must be on the host or on ", dev);
    void* st = current_stream();

    auto p = c10::make_intrusive<PendingBlocks>();
    p->hops_ = hops;
    p->indptr_ = indptr;
    p->stream_ = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().unwrap();
    // the kernels mirror the lengths into this call's own pinned words
    p->pinned_ = torch::empty({32}, torch::TensorOptions().dtype(torch::kInt64).pinned_memory(true));
    for (int i = 0; i < 32; ++i) p->pinned_.data_ptr<int64_t>()[i] = -1;  // Finish polls them: lengths are never negative
    if (seeds_in.device().is_cpu() && !seeds_in.is_pinned() && n > 0) {
      // pageable host seeds (what upstream's DataLoader passes): staged through pinned memory of
      // this batch, so that the upload is a plain asynchronous copy the host does not wait for
      p->staged_seeds_ = torch::empty({n}, seeds_in.options().pinned_memory(true));
      p->staged_seeds_.copy_(seeds_in.contiguous().view({-1}));
      p->seeds_ = p->staged_seeds_.to(dev, /*non_blocking=*/true);
    } else {
      p->seeds_ = seeds_in.to(dev, /*non_blocking=*/true).contiguous().view({-1});
    }
    const auto opt = p->seeds_.options();
    p->src_.resize(hops);
    p->dst_.resize(hops);
    std::vector<dgs_block_out> outs(hops);
    // The id outputs of the batch (the frontier array, of which every hop's frontier is a prefix,
    // and the edge lists) and its device-side lengths are pieces of ONE allocation: a dozen
    // tensors cost a dozen trips to the allocator here, and as many stream records and events
    // again when the batch is handed to another stream and dropped there.
    int64_t carved = 0;
    const auto piece = [&carved](int64_t bytes) {
      const int64_t at = carved;
      carved += (bytes + 255) / 256 * 256;
      return at;
    };
    const int64_t all_at = piece(seeds_max[hops] * w);
    std::vector<int64_t> src_at(hops), dst_at(hops);
    for (int h = 0; h < hops; ++h) {
      src_at[h] = piece(edges_max[h] * w);
      dst_at[h] = piece(edges_max[h] * w);
    }
    const int64_t sizes_at = piece(n_sizes * 8);
    // (up to kOneBlockBytes: beyond that the pieces are hundreds of megabytes each, the calls to the
    // allocator no longer matter and separate blocks are reused more freely: C4, whose worst case
    // is 511 MB of ids per batch, ran 4 % slower out of one block)
    constexpr int64_t kOneBlockBytes = int64_t(128) << 20;
    torch::Tensor sizes_dev;
    if (carved <= kOneBlockBytes) {
      torch::Tensor block = device_bytes(static_cast<size_t>(carved), dev);
      const auto ids_of = [&](int64_t at, int64_t count) {
        return block.narrow(0, at, count * w).view(p->seeds_.scalar_type());
      };
      p->all_ = ids_of(all_at, seeds_max[hops]);
      for (int h = 0; h < hops; ++h) {
        p->src_[h] = ids_of(src_at[h], edges_max[h]);
        p->dst_[h] = ids_of(dst_at[h], edges_max[h]);
      }
      sizes_dev = block.narrow(0, sizes_at, n_sizes * 8).view(torch::kInt64);
      p->owned_.push_back(block);
    } else {
      p->all_ = torch::empty({seeds_max[hops]}, opt);
      p->owned_.push_back(p->all_);
      for (int h = 0; h < hops; ++h) {
        p->src_[h] = torch::empty({edges_max[h]}, opt);
        p->dst_[h] = torch::empty({edges_max[h]}, opt);
        p->owned_.push_back(p->src_[h]);
        p->owned_.push_back(p->dst_[h]);
      }
      sizes_dev = torch::empty({n_sizes}, opt.dtype(torch::kInt64));
      p->owned_.push_back(sizes_dev);  // (kept with the batch: the kernels write it after this call returns)
    }
    for (int h = 0; h < hops; ++h) outs[h] = dgs_block_out{p->src_[h].data_ptr(), p->dst_[h].data_ptr()};
    const size_t ws_bytes = probs ? dgs_sample_blocks_weighted_workspace_bytes(n, fanouts.data(), hops, w)
                                  : dgs_sample_blocks_workspace_bytes(n, fanouts.data(), hops, w);
    torch::Tensor ws = device_bytes(ws_bytes, dev);  // freed on return: the allocator reuses it in stream order
    // host threads that sample from the same graph enqueue their calls one at a time
    const std::unique_lock<std::mutex> one_call_at_a_time = indptr->enqueue_lock();
    const auto table = indptr->node_table(st);
    // the caller's own (seed, first stream) when given, else the next `hops` streams of the
    // process-wide generator
    const auto rng = own_rng != nullptr ? *own_rng : next_rng(static_cast<uint32_t>(hops));
    if (probs)
      check(dgs_sample_blocks_weighted(p->seeds_.data_ptr(), w, n, indptr->view(), indices->view(), probs->view(),
                                       fanouts.data(), hops, replace, rng.first, rng.second, table.first,
                                       table.second, p->all_.data_ptr(), outs.data(), sizes_dev.data_ptr<int64_t>(),
                                       p->pinned_.data_ptr<int64_t>(), nullptr, ws.data_ptr(), ws_bytes, st));
    else
      check(dgs_sample_blocks(p->seeds_.data_ptr(), w, n, indptr->view(), indices->view(), fanouts.data(), hops,
                              replace, rng.first, rng.second, table.first, table.second, p->all_.data_ptr(),
                              outs.data(), sizes_dev.data_ptr<int64_t>(), p->pinned_.data_ptr<int64_t>(),
                              nullptr, ws.data_ptr(), ws_bytes, st));
    if (features) {
      const auto xopt = torch::TensorOptions().dtype(features->dtype()).device(dev);
      const int64_t row_bytes = features->elem_stride() * static_cast<int64_t>(c10::elementSize(features->dtype()));
      // The lengths are final at the ticket; the gather is enqueued before anybody waits for them,
      // into a buffer of which the result is a prefix: one for the worst case, or, where that would
      // exceed the cap (the worst case grows with the product of the fanouts, the frontier does
      // not), the largest the cap allows.  A frontier that does not fit such a buffer is left
      // alone by the kernel and gathered in Finish, into exactly its size.
      int64_t buffer_rows = seeds_max[hops];
      if (buffer_rows * row_bytes > g_gather_buffer_cap.load()) buffer_rows = g_gather_buffer_cap.load() / row_bytes;
      p->features_ = features;
      p->width_ = w;
      p->x_rows_ = buffer_rows > 0 ? buffer_rows : -1;
      p->x_ = torch::empty({buffer_rows, features->elem_stride()}, xopt);
      // the caller may hold the gather back until an event of another stream (the previous
      // batch's gather, say), while the sampler kernels above run as soon as they can
      if (gather_after != nullptr) check(dgs_ticket_stream_wait(st, gather_after));
      if (buffer_rows > 0)
      {
        // the launch is sized for what the graph's last finished batch gathered (a hint: a larger
        // frontier is gathered all the same, by blocks that loop; measured on 1.2 M rows of 256
        // bytes, a launch of exactly the right size 113 us, of half the size 114, with a quarter
        // more blocks than needed 116, at the 32768-block cap 118)
        const int64_t last = indptr->frontier_hint();
        // Weighted fills are bound by vector arithmetic and need wave slots beside other batches'
        // gathers, which by themselves take every slot of a CU: such a batch's gather keeps half of
        // them (measured with four weighted batches in flight, 8 / 5 / 4 / 3 blocks per CU: 0.2165 /
        // 0.197 / 0.193 / 0.205 ms per step; the uniform sampler's kernels wait for memory, and its
        // steps are 9 % slower at 5 and 4)
        const int32_t gather_blocks_per_cu = probs ? 4 : 0;
        p->gather_status_ = dgs_gather_rows_dyn_shared(features->view(), features->elem_stride(), p->all_.data_ptr(), w,
                                                       buffer_rows, sizes_dev.data_ptr<int64_t>() + hops, last,
                                                       p->x_.data_ptr(), DGS_TIER_ANY, gather_blocks_per_cu,
                                                       features->bad_index_word(), st);
      }
    }
    // the batch's one ticket, behind its last launch: it bounds the wait for the lengths, tells the
    // next batch's gather when this one's is through, and the graph when its node table is free again
    p->end_ = record_ticket(st);
    if (table.first != nullptr) indptr->node_table_used(st, p->end_);
    return p;
  }

  // The stream the batch was begun on, and a way to mark the batch's buffers as used on another
  // stream (so that the allocator does not hand them out again while that stream still reads them).
  c10::Stream stream() const { return stream_; }
  // The ticket behind everything the batch has enqueued: the one recorded by Begin, unless Finish
  // had to enqueue a gather of its own afterwards (a fresh one then).
  TicketRef last_ticket() {
    if (gathered_late_) {
      end_ = record_ticket(c10::hip::HIPStreamMasqueradingAsCUDA(stream_).stream());
      gathered_late_ = false;
    }
    return end_;
  }
  void RecordStream(const c10::Stream& consumer) {
    // (the frontier and the edge lists are, or are views of, the tensors in owned_)
    for (const torch::Tensor* t : {&seeds_, &x_})
      if (t->defined() && t->is_cuda()) t->record_stream(consumer);
    for (const torch::Tensor& t : owned_) t.record_stream(consumer);
  }

 private:
  int hops_ = 0;
  bool finished_ = false;
  TicketRef end_;               // recorded behind the last launch of Begin
  bool gathered_late_ = false;  // Finish enqueued a gather behind end_
  dgs_status gather_status_ = DGS_OK;
  torch::Tensor pinned_, seeds_, all_, x_;
  std::vector<torch::Tensor> owned_;  // the allocations behind all_, src_, dst_ and the device-side lengths
  torch::Tensor staged_seeds_;  // pinned copy of host seeds, alive until the batch is finished
  std::vector<torch::Tensor> src_, dst_;
  // the feature gather: rows of the buffer it was enqueued into (-1: none), and what a second,
  // exact gather in Finish needs
  c10::intrusive_ptr<ChunkTensor> features_;
  c10::intrusive_ptr<ChunkTensor> indptr_;  // the graph: it remembers the last frontier size (launch sizing)
  int64_t x_rows_ = -1;
  int32_t width_ = 0;
  c10::Stream stream_ = c10::Stream(c10::Stream::DEFAULT, c10::Device(c10::DeviceType::CPU, -1));
};

// Batches in flight without a Python step per enqueue: a worker thread begins batches
// (PendingBlocks::Begin: some hundred microseconds of host work each, most of it kernel launches)
// on the loop's streams in turn while the caller's thread takes delivery of finished ones.
// Push hands seeds to the worker, Pop returns the oldest batch not yet returned, in order.
// At most `streams.size()` batches are begun and not yet popped.
class BatchLoop : public torch::CustomClassHolder {
 public:
  BatchLoop(c10::intrusive_ptr<ChunkTensor> indptr, c10::intrusive_ptr<ChunkTensor> indices,
            c10::optional<c10::intrusive_ptr<ChunkTensor>> probs, std::vector<int64_t> fanouts, bool replace,
            c10::optional<c10::intrusive_ptr<ChunkTensor>> features, std::vector<int64_t> streams, bool hand_over,
            bool gathers_in_turn, std::vector<int64_t> rng)
      : indptr_(std::move(indptr)), indices_(std::move(indices)),
        probs_(probs.has_value() ? *probs : c10::intrusive_ptr<ChunkTensor>()), fanouts_(std::move(fanouts)),
        replace_(replace), features_(features.has_value() ? *features : c10::intrusive_ptr<ChunkTensor>()),
        hand_over_(hand_over), turn_(gathers_in_turn), rng_(std::move(rng)) {
    TORCH_CHECK(!streams.empty() && streams.size() % 3 == 0,
                "BatchLoop: streams are (stream_id, device_index, device_type) triples");
    TORCH_CHECK(rng_.size() <= 1, "BatchLoop: rng is [] (the process-wide generator) or [seed] (the caller's own)");
    for (size_t i = 0; i < streams.size(); i += 3)
      streams_.push_back(c10::Stream::unpack3(streams[i], static_cast<c10::DeviceIndex>(streams[i + 1]),
                                               static_cast<c10::DeviceType>(streams[i + 2])));
    done_.assign(streams_.size() + 1, TicketRef());
    worker_ = std::thread([this] { Work(); });
  }
  ~BatchLoop() override { Close(); }

  // Seeds on the device are ordered behind what the calling thread's current stream holds at this
  // moment (they may have been made there just now); host seeds need nothing, unless the caller
  // asks for the same order (behind_caller: the first batches of an iteration, say, behind the
  // set-up that precedes it).
  // `first_stream`: with a generator of the caller's own (rng = [seed]), the stream of the batch's
  // first hop, which the caller counts (a sampler numbers its batches in submission order);
  // ignored otherwise.
  void Push(torch::Tensor seeds, bool behind_caller, int64_t first_stream) {
    Item item;
    item.seeds = std::move(seeds);
    item.first_stream = first_stream;
    TORCH_CHECK(rng_.empty() || (first_stream >= 0 && first_stream <= 0xffffffffLL),
                "BatchLoop: a generator of the caller's own needs the batch's first stream, 0..2^32-1");
    if (item.seeds.is_cuda() || behind_caller) {
      void* st = current_stream();
      int32_t idle = 0;
      check(dgs_stream_query(st, &idle));
      if (!idle) check(dgs_ticket_record(st, &item.seeds_ready));
    }
    bool closed;
    {
      const std::lock_guard<std::mutex> lock(mutex_);
      closed = stop_;
      if (!closed) {
        input_.push_back(std::move(item));
        ++pushed_;
      }
    }
    if (closed) {  // the ticket taken above goes back before the call fails
      if (item.seeds_ready) dgs_ticket_release(item.seeds_ready);
      TORCH_CHECK(false, "BatchLoop: closed");
    }
    wake_worker_.notify_one();
  }

  BlocksResult Pop() {
    Item item;
    {
      std::unique_lock<std::mutex> lock(mutex_);
      TORCH_CHECK(!stop_, "BatchLoop: closed");
      TORCH_CHECK(popped_ < pushed_, "BatchLoop: nothing to pop");
      // (a loop that is closed while this thread waits gives its pending batches up: the wait ends)
      wake_caller_.wait(lock, [this] { return stop_ || !output_.empty(); });
      TORCH_CHECK(!output_.empty(), "BatchLoop: closed");
      item = std::move(output_.front());
      output_.pop_front();
      ++popped_;
    }
    wake_worker_.notify_one();  // a slot is free
    TORCH_CHECK(item.error.empty(), item.error);
    BlocksResult result = item.batch->Finish();
    if (hand_over_) {
      // the calling thread's stream waits for everything the batch has enqueued (Finish may just have
      // added a gather), and the batch's buffers are marked as used there
      check(dgs_ticket_stream_wait(current_stream(), item.batch->last_ticket()->handle));
      item.batch->RecordStream(c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().unwrap());
    }
    return result;
  }

  int64_t Pending() {
    const std::lock_guard<std::mutex> lock(mutex_);
    return pushed_ - popped_;
  }

  void Close() {
    {
      const std::lock_guard<std::mutex> lock(mutex_);
      if (stop_) return;
      stop_ = true;
    }
    wake_worker_.notify_all();
    if (worker_.joinable()) worker_.join();
    std::deque<Item> unbegun, unclaimed;
    {
      // batches that were pushed and never popped are given up: nothing is pending afterwards, and a
      // thread that waits in Pop is woken (it finds the loop closed)
      const std::lock_guard<std::mutex> lock(mutex_);
      unbegun.swap(input_);
      unclaimed.swap(output_);
      popped_ = pushed_;
    }
    wake_caller_.notify_all();
    for (Item& item : unbegun)
      if (item.seeds_ready) dgs_ticket_release(item.seeds_ready);
    unbegun.clear();
    unclaimed.clear();  // batches nobody asked for: their destructors wait for their kernels' lengths
    for (TicketRef& t : done_) t.reset();
  }

 private:
  struct Item {
    torch::Tensor seeds;
    void* seeds_ready = nullptr;  // ticket on the pushing thread's stream, or null
    int64_t first_stream = -1;
    c10::intrusive_ptr<PendingBlocks> batch;
    std::string error;
  };

  static void* stream_handle(const c10::Stream& s) {
    return c10::hip::HIPStreamMasqueradingAsCUDA(s).stream();
  }

  void Work() {
    int64_t index = 0;
    const int64_t n = static_cast<int64_t>(streams_.size());
    for (;;) {
      Item item;
      {
        std::unique_lock<std::mutex> lock(mutex_);
        wake_worker_.wait(lock, [&] { return stop_ || (!input_.empty() && begun_ - popped_ < n); });
        if (stop_) return;
        item = std::move(input_.front());
        input_.pop_front();
        ++begun_;
      }
      try {
        const c10::Stream st = streams_[index % n];
        const c10::StreamGuard on_stream(st);  // allocations and launches of this batch go to its stream
        void* raw = current_stream();
        if (item.seeds_ready) {
          const dgs_status ws = dgs_ticket_stream_wait(raw, item.seeds_ready);
          dgs_ticket_release(item.seeds_ready);
          item.seeds_ready = nullptr;
          check(ws);
        }
        const bool turn = turn_ && features_ && n > 1;
        const TicketRef before = turn && index > 0 ? done_[(index - 1) % (n + 1)] : TicketRef();
        void* gather_after = before ? before->handle : nullptr;
        std::pair<uint64_t, uint32_t> own{0, 0};
        if (!rng_.empty()) own = {static_cast<uint64_t>(rng_[0]), static_cast<uint32_t>(item.first_stream)};
        item.batch = PendingBlocks::Begin(item.seeds, indptr_, indices_, fanouts_, replace_, features_, probs_,
                                          rng_.empty() ? nullptr : &own, gather_after);
        // (the slot's old ticket belongs to a batch that was popped long ago: at most n are in flight)
        if (turn) done_[index % (n + 1)] = item.batch->last_ticket();
      } catch (const std::exception& err) {
        item.error = err.what();
      }
      item.seeds = torch::Tensor();
      ++index;
      {
        const std::lock_guard<std::mutex> lock(mutex_);
        output_.push_back(std::move(item));
      }
      wake_caller_.notify_one();
    }
  }

  c10::intrusive_ptr<ChunkTensor> indptr_, indices_, probs_;
  std::vector<int64_t> fanouts_;
  bool replace_;
  c10::intrusive_ptr<ChunkTensor> features_;
  std::vector<c10::Stream> streams_;
  bool hand_over_, turn_;
  std::vector<int64_t> rng_;
  std::vector<TicketRef> done_;  // ring of the last batches' tickets (worker thread only)
  std::mutex mutex_;
  std::condition_variable wake_worker_, wake_caller_;
  std::deque<Item> input_, output_;
  int64_t pushed_ = 0, begun_ = 0, popped_ = 0;
  bool stop_ = false;
  std::thread worker_;
};

namespace {

BlocksResult sample_blocks_impl(const torch::Tensor& seeds_in, const c10::intrusive_ptr<ChunkTensor>& indptr,
                                const c10::intrusive_ptr<ChunkTensor>& indices, const std::vector<int64_t>& fanouts,
                                bool replace, const c10::intrusive_ptr<ChunkTensor>& features) {
  return PendingBlocks::Begin(seeds_in, indptr, indices, fanouts, replace, features)->Finish();
}

// Both operators also return the seeds as a device tensor (the upload they did anyway).
std::tuple<std::vector<torch::Tensor>, std::vector<torch::Tensor>, std::vector<torch::Tensor>, torch::Tensor>
SampleBlocks(torch::Tensor seeds, c10::intrusive_ptr<ChunkTensor> indptr, c10::intrusive_ptr<ChunkTensor> indices,
             std::vector<int64_t> fanouts, bool replace) {
  auto r = sample_blocks_impl(seeds, indptr, indices, fanouts, replace, c10::intrusive_ptr<ChunkTensor>());
  return std::make_tuple(std::get<0>(r), std::get<1>(r), std::get<2>(r), std::get<4>(r));
}

std::tuple<std::vector<torch::Tensor>, std::vector<torch::Tensor>, std::vector<torch::Tensor>, torch::Tensor,
           torch::Tensor>
SampleBlocksAndIndex(torch::Tensor seeds, c10::intrusive_ptr<ChunkTensor> indptr,
                     c10::intrusive_ptr<ChunkTensor> indices, std::vector<int64_t> fanouts, bool replace,
                     c10::intrusive_ptr<ChunkTensor> features) {
  TORCH_CHECK(features, "sample_blocks_and_index: features store is null");
  return sample_blocks_impl(seeds, indptr, indices, fanouts, replace, features);
}

// The same two operators in two halves: *_begin enqueues everything on the current stream and
// returns at once, PendingBlocks._CAPI_finish waits for the lengths and returns the results.
c10::intrusive_ptr<PendingBlocks> SampleBlocksBegin(torch::Tensor seeds, c10::intrusive_ptr<ChunkTensor> indptr,
                                                    c10::intrusive_ptr<ChunkTensor> indices,
                                                    std::vector<int64_t> fanouts, bool replace) {
  return PendingBlocks::Begin(seeds, indptr, indices, fanouts, replace, c10::intrusive_ptr<ChunkTensor>());
}
c10::intrusive_ptr<PendingBlocks> SampleBlocksAndIndexBegin(torch::Tensor seeds,
                                                            c10::intrusive_ptr<ChunkTensor> indptr,
                                                            c10::intrusive_ptr<ChunkTensor> indices,
                                                            std::vector<int64_t> fanouts, bool replace,
                                                            c10::intrusive_ptr<ChunkTensor> features) {
  TORCH_CHECK(features, "sample_blocks_and_index: features store is null");
  return PendingBlocks::Begin(seeds, indptr, indices, fanouts, replace, features);
}

// Weighted picks (chunktensor_sampler.py:97-100) through the fused driver; `features` may be None.
c10::intrusive_ptr<PendingBlocks> SampleBlocksWeightedBegin(torch::Tensor seeds,
                                                            c10::intrusive_ptr<ChunkTensor> indptr,
                                                            c10::intrusive_ptr<ChunkTensor> indices,
                                                            c10::intrusive_ptr<ChunkTensor> probs,
                                                            std::vector<int64_t> fanouts, bool replace,
                                                            c10::optional<c10::intrusive_ptr<ChunkTensor>> features) {
  TORCH_CHECK(probs, "sample_blocks_weighted: probs store is null");
  return PendingBlocks::Begin(seeds, indptr, indices, fanouts, replace,
                              features.has_value() ? *features : c10::intrusive_ptr<ChunkTensor>(), probs);
}

// Any of the *_begin operators with the generator state passed in: the hops draw from streams
// rng_stream, rng_stream + 1, ... of seed rng_seed and the process-wide generator is left alone,
// so a caller that keeps its own counter gets the same picks whatever other threads do.
// The general form of the *_begin operators: `probs` and `features` are optional, `rng` is empty
// (the process-wide generator) or [seed, first stream]; `gather_after` is 0 or the handle of an
// event (torch.cuda.Event.cuda_event) that the feature gather, and only it, waits for.
c10::intrusive_ptr<PendingBlocks> SampleBlocksSubmit(torch::Tensor seeds, c10::intrusive_ptr<ChunkTensor> indptr,
                                                     c10::intrusive_ptr<ChunkTensor> indices,
                                                     c10::optional<c10::intrusive_ptr<ChunkTensor>> probs,
                                                     std::vector<int64_t> fanouts, bool replace,
                                                     c10::optional<c10::intrusive_ptr<ChunkTensor>> features,
                                                     std::vector<int64_t> rng, int64_t gather_after) {
  TORCH_CHECK(rng.empty() || rng.size() == 2, "sample_blocks_submit: rng is [] or [seed, stream]");
  std::pair<uint64_t, uint32_t> own{0, 0};
  if (!rng.empty()) own = {static_cast<uint64_t>(rng[0]), static_cast<uint32_t>(rng[1])};
  return PendingBlocks::Begin(seeds, indptr, indices, fanouts, replace,
                              features.has_value() ? *features : c10::intrusive_ptr<ChunkTensor>(),
                              probs.has_value() ? *probs : c10::intrusive_ptr<ChunkTensor>(),
                              rng.empty() ? nullptr : &own,
                              reinterpret_cast<void*>(static_cast<intptr_t>(gather_after)));
}

// Largest worst-case feature buffer (bytes) the fused operators allocate ahead of the sizes.
void SetGatherBufferCap(int64_t bytes) {
  TORCH_CHECK(bytes >= 0, "gather buffer cap must be >= 0");
  g_gather_buffer_cap.store(bytes);
}
int64_t GetGatherBufferCap() { return g_gather_buffer_cap.load(); }

// Largest graph (nodes) whose fused calls use persistent node tables; -1: no limit of its own.
void SetNodeTableMaxNodes(int64_t nodes) { g_node_table_max_nodes.store(nodes < 0 ? -1 : nodes); }
int64_t GetNodeTableMaxNodes() { return g_node_table_max_nodes.load(); }

int64_t GetCurrentAllocated() { return dgs_current_allocated(); }

// upstream nccl::GetUniqueId / nccl::SetNCCL (src/nccl_context.cc:17-34): there is no
// communicator at world size 1; the shims keep unmodified harness code running.
std::vector<int64_t> GetUniqueId() { return std::vector<int64_t>(16, 0); }
void SetNCCL(int64_t nranks, std::vector<int64_t> /*unique_id*/, int64_t rank) {
  TORCH_CHECK(nranks == 1 && rank == 0, "_CAPI_set_nccl: this build runs at world size 1 (got nranks=", nranks,
              ", rank=", rank, ")");
}

void SetRngState(int64_t seed, int64_t stream) {
  std::lock_guard<std::mutex> lock(g_rng_mutex);
  g_rng_seed = static_cast<uint64_t>(seed);
  g_rng_stream = static_cast<uint32_t>(stream);
}
std::vector<int64_t> GetRngState() {
  std::lock_guard<std::mutex> lock(g_rng_mutex);
  return {static_cast<int64_t>(g_rng_seed), static_cast<int64_t>(g_rng_stream)};
}

}  // namespace
}  // namespace dgs

using dgs::ChunkTensor;
using dgs::PendingBlocks;

TORCH_LIBRARY(dgs_classes, m) {
  m.class_<ChunkTensor>("ChunkTensor")
      .def(torch::init<std::vector<int64_t>, torch::ScalarType, int64_t>())
      .def("_CAPI_get_host_tensor", &ChunkTensor::GetHostTensor)
      .def("_CAPI_get_sub_device_tensor", &ChunkTensor::GetSubDeviceTensor)
      .def("_CAPI_index", &ChunkTensor::Index)
      .def("_CAPI_split_index", &ChunkTensor::SplitIndex)
      .def("_CAPI_local_index", &ChunkTensor::LocalIndex)
      .def("_CAPI_remote_index", &ChunkTensor::RemoteIndex)
      .def("_CAPI_host_index", &ChunkTensor::HostIndex)
      .def("_CAPI_load_from_tensor", &ChunkTensor::LoadFromTensor)
      // not in upstream: waits for the current stream, then raises if a gather met a bad row id
      .def("_CAPI_synchronize_and_check", &ChunkTensor::SynchronizeAndCheck)
      // not in upstream: the fused sampler's per-stream node tables of a graph's indptr store
      .def("_CAPI_release_node_table", &ChunkTensor::ReleaseNodeTable)
      .def("_CAPI_node_table_count", &ChunkTensor::NodeTableCount);
  // not in upstream: a sample_blocks call in flight
  m.class_<PendingBlocks>("PendingBlocks").def("_CAPI_finish", &PendingBlocks::Finish);
  // not in upstream: batches in flight, begun by a worker thread of the extension
  m.class_<dgs::BatchLoop>("BatchLoop")
      .def(torch::init<c10::intrusive_ptr<ChunkTensor>, c10::intrusive_ptr<ChunkTensor>,
                       c10::optional<c10::intrusive_ptr<ChunkTensor>>, std::vector<int64_t>, bool,
                       c10::optional<c10::intrusive_ptr<ChunkTensor>>, std::vector<int64_t>, bool, bool,
                       std::vector<int64_t>>())
      .def("_CAPI_push", &dgs::BatchLoop::Push)
      .def("_CAPI_pop", &dgs::BatchLoop::Pop)
      .def("_CAPI_pending", &dgs::BatchLoop::Pending)
      .def("_CAPI_close", &dgs::BatchLoop::Close);
}

TORCH_LIBRARY(dgs_ops, m) {
  // an operator layer and a kernel library built from different headers would pass each other
  // arguments in the wrong places: refuse to register on top of such a pair
  TORCH_CHECK(dgs_abi_version() == DGS_ABI_VERSION, "libdgs_hip.so reports C ABI version ", dgs_abi_version(),
              ", this operator layer was built against ", DGS_ABI_VERSION, ": rebuild both (build.py)");
  m.def("_CAPI_tensor_relabel", &dgs::TensorRelabel)
      .def("_CAPI_sample_neighbors", &dgs::SampleNeighbors)
      .def("_CAPI_sample_neighbors_with_chunk_tensor", &dgs::SampleNeighborsWithChunkTensor)
      .def("_CAPI_sample_neighbors_with_probs", &dgs::SampleNeighborsWithProbs)
      .def("_CAPI_sample_neighbors_with_probs_with_chunk_tensor", &dgs::SampleNeighborsWithProbsWithChunkTensor)
      .def("_CAPI_get_unique_id", &dgs::GetUniqueId)
      .def("_CAPI_set_nccl", &dgs::SetNCCL)
      .def("_CAPI_get_current_allocated", &dgs::GetCurrentAllocated)
      // not in upstream: the whole sampler loop (and optionally the feature gather) in one call
      .def("_CAPI_sample_blocks", &dgs::SampleBlocks)
      .def("_CAPI_sample_blocks_and_index", &dgs::SampleBlocksAndIndex)
      .def("_CAPI_sample_blocks_begin", &dgs::SampleBlocksBegin)
      .def("_CAPI_sample_blocks_and_index_begin", &dgs::SampleBlocksAndIndexBegin)
      .def("_CAPI_sample_blocks_weighted_begin", &dgs::SampleBlocksWeightedBegin)
      .def("_CAPI_sample_blocks_submit", &dgs::SampleBlocksSubmit)
      .def("_CAPI_set_gather_buffer_cap", &dgs::SetGatherBufferCap)
      .def("_CAPI_get_gather_buffer_cap", &dgs::GetGatherBufferCap)
      .def("_CAPI_set_node_table_max_nodes", &dgs::SetNodeTableMaxNodes)
      .def("_CAPI_get_node_table_max_nodes", &dgs::GetNodeTableMaxNodes)
      // not in upstream: node renumbering (hottest rows first) for the positional stores
      .def("_CAPI_renumber_csc", &dgs::RenumberCSC)
      // not in upstream: the sampling generator's (seed, stream)
      .def("_CAPI_set_rng_state", &dgs::SetRngState)
      .def("_CAPI_get_rng_state", &dgs::GetRngState);
}
