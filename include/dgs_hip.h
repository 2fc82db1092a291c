/*
 * dgs_hip.h -- C ABI of libdgs_hip.so: the gfx950 kernels behind the
 * torch.classes.dgs_classes.ChunkTensor / torch.ops.dgs_ops operator surface.
 *
 * Conventions
 *   - every entry point returns a dgs_status (0 = ok); nothing aborts or throws;
 *     dgs_last_error() gives a thread-local message for the last failure;
 *   - all pointers named dev_* / *_dev / out_* are device-accessible addresses
 *     (HBM, or pinned host memory mapped into the device address space);
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream); every
 *     kernel is enqueued there and nothing synchronises unless the name says so;
 *   - entry points that need temporary device memory take a caller-owned
 *     workspace whose size the matching *_workspace_bytes() call reports; the
 *     kernels themselves never allocate;
 *   - ids are int32 or int64 (`id_bytes` 4 or 8), selected at run time.
 *
 * Each declaration cites the reference interface (file:line under the upstream
 * source tree) whose behaviour it reproduces.
 */
#ifndef DGS_HIP_H_
#define DGS_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef int dgs_status;
enum {
  DGS_OK = 0,
  DGS_ERR_INVALID = 1,      /* bad argument (null pointer, negative size, width not 4/8 ...) */
  DGS_ERR_HIP = 2,          /* a HIP runtime call failed */
  DGS_ERR_WORKSPACE = 3,    /* workspace too small or misaligned */
  DGS_ERR_UNSUPPORTED = 4,  /* valid request outside what the kernels cover */
  DGS_ERR_RANGE = 5         /* data-dependent failure reported by a kernel (see each call) */
};

/* Message of the last failing call on this thread ("" if none). */
const char* dgs_last_error(void);
/* Static name of a status code. */
const char* dgs_status_name(dgs_status s);
/* ABI version of this header (bumped on incompatible change): a binding compares what the library
 * it loaded reports with the DGS_ABI_VERSION it was written against, before any other call. */
#define DGS_ABI_VERSION 3
int dgs_abi_version(void);
/*
 * Test hooks, process-wide: force code paths that small test inputs would not reach by
 * themselves.  Results never depend on them.  Not for production use.
 *   DGS_DEBUG_FORCE_SPLIT_TABLE  non-zero: dgs_sample_blocks without a node table uses the
 *                                id-array + value-array hash table also where ids would fit
 *                                the packed one
 *   DGS_DEBUG_WEIGHTED_GROUP     16, 32 or 64: lanes per row of the weighted per-hop fill
 *                                (0: chosen from num_picks)
 *   DGS_DEBUG_GATHER_LDS_BYTES   bytes of (unused) LDS that every block of the row gather
 *                                reserves, 0..65536: bounds how many of its blocks share a CU
 *   DGS_DEBUG_SAMPLER_GRID_CAP   > 0: most blocks a launch of dgs_sample_blocks may have
 *                                (larger launches loop over their blocks)
 *   DGS_DEBUG_SAMPLER_BUCKETED   how the last hop of dgs_sample_blocks[_weighted] with a node
 *                                table finds its first occurrences: 0 by size (the bucketed LDS
 *                                pass for a large hop of uniform picks, the table's atomics
 *                                otherwise), 1 always the table, 2 the bucketed pass whatever
 *                                the size and the kind of picks, 3 like 2 and in the form for
 *                                graphs of any node count (buckets by a hash of the id, an LDS
 *                                hash table per bucket) whatever the graph's size, 4 like 3 with
 *                                those tables cut to 256 slots (small inputs then fill them and
 *                                are gone over in parts)
 */
enum {
  DGS_DEBUG_FORCE_SPLIT_TABLE = 0,
  DGS_DEBUG_WEIGHTED_GROUP = 1,
  DGS_DEBUG_GATHER_LDS_BYTES = 2,
  DGS_DEBUG_SAMPLER_GRID_CAP = 3,
  DGS_DEBUG_SAMPLER_BUCKETED = 4
};
dgs_status dgs_debug_set(int32_t option, int64_t value);

/*
 * Measurement aid, no counterpart in the reference: `n_ops` threads each touch one 8-byte
 * slot of `table` (`slots` of them, device memory), slot = a hash of (thread index, salt)
 * reduced modulo `slots`, with
 *   DGS_PROBE_LOAD        a load,
 *   DGS_PROBE_STORE       a store of the thread's index,
 *   DGS_PROBE_ATOMIC_MIN  an atomicMin with the old value returned (what the fused sampler does
 *                         once per pick on its node table),
 *   DGS_PROBE_ATOMIC_MIN_NO_RETURN  the same without using the old value.
 * What the loads and atomics returned is folded into *sink (8 bytes of device memory) so that
 * nothing is optimised away.  Timed by the caller (events on `stream`), it gives the rate at
 * which this GPU serves random 8-byte accesses of each kind: the bound of the table kernels.
 */
enum { DGS_PROBE_LOAD = 0, DGS_PROBE_STORE = 1, DGS_PROBE_ATOMIC_MIN = 2, DGS_PROBE_ATOMIC_MIN_NO_RETURN = 3 };
dgs_status dgs_debug_probe_table(int32_t op, void* table, int64_t slots, int64_t n_ops, uint64_t salt,
                                 void* sink, void* stream);

/* ------------------------------------------------------------------------ */
/* Two-tier positional store (ChunkTensor)                                   */
/* ------------------------------------------------------------------------ */

/*
 * Device-side view of a store, passed to kernels BY VALUE.
 * Element i lives at dev[i] when i < threshold, else at host[i - threshold].
 * Replaces the device-resident accessor struct chunk_tensor_wrapper<T>
 * (src/chunk_tensor.h:10-59) at world size 1.  A plain device array is the
 * view {dev = ptr, host = NULL, threshold = total = n}.
 */
typedef struct dgs_view {
  const void* dev;    /* HBM slice: elements [0, threshold)                  */
  const void* host;   /* device-visible address of the pinned host slice     */
  int64_t threshold;  /* elements held in HBM                                */
  int64_t total;      /* elements in the whole store                         */
  int32_t elem_bytes; /* 1, 2, 4 or 8                                        */
  int32_t reserved_;
} dgs_view;

typedef struct dgs_store dgs_store; /* opaque, owns both slices */

/*
 * Split arithmetic of ChunkTensor::ChunkTensor (src/chunk_tensor.cc:37-73) at
 * world size 1: device elements = capacity_bytes / elem_bytes clamped to
 * total_elems; host elements = the rest.  Pure host arithmetic, no GPU needed.
 */
dgs_status dgs_store_split(int64_t total_elems, int32_t elem_bytes,
                           int64_t capacity_bytes, int64_t* device_elems,
                           int64_t* host_elems);

/*
 * Allocates the HBM slice (filled with 0xFF bytes, src/chunk_tensor.cc:100-109)
 * and the pinned, device-mapped host slice (hipHostMalloc; replaces SysV shm +
 * cudaHostRegister, src/chunk_tensor.cc:76-96) on the current device.
 */
dgs_status dgs_store_create(int64_t total_elems, int32_t elem_bytes,
                            int64_t capacity_bytes, dgs_store** out);
/* ChunkTensor::_Free (src/chunk_tensor.cc:235-263). NULL is accepted. */
dgs_status dgs_store_destroy(dgs_store* s);
/*
 * ChunkTensor::LoadFromTensor (src/chunk_tensor.cc:173-200): copies
 * total_elems elements from pageable or pinned HOST memory `src` into the two
 * slices.  Blocking.
 */
dgs_status dgs_store_load(dgs_store* s, const void* src, int64_t n_elems);
/* Fills *v with the by-value kernel view of the store. */
dgs_status dgs_store_view(const dgs_store* s, dgs_view* v);
/*
 * Raw slices for GetSubDeviceTensor / GetHostTensor (src/chunk_tensor.cc:151-171).
 * host_cpu_ptr is the CPU address of the pinned slice.
 */
dgs_status dgs_store_slices(const dgs_store* s, void** dev_ptr,
                            int64_t* device_elems, void** host_cpu_ptr,
                            int64_t* host_elems);
/*
 * Bytes of HBM currently held by stores: CUDAContext::GetCurrAllocated
 * (src/cuda_context.h:13-15, src/cuda_context.cc:5-6).
 */
int64_t dgs_current_allocated(void);

/* ------------------------------------------------------------------------ */
/* Row gather                                                                */
/* ------------------------------------------------------------------------ */

enum {
  DGS_TIER_ANY = 0,   /* _CAPI_index:       per-element device/host resolution */
  DGS_TIER_DEVICE = 1,/* _CAPI_local_index: every row read from the HBM slice  */
  DGS_TIER_HOST = 2   /* _CAPI_host_index:  every row read from the host slice */
};

/*
 * out[i, 0:row_elems] = X[index[i], 0:row_elems] for i in [0, n), X the
 * row-major [total/row_elems, row_elems] matrix behind `v`.
 * Replaces IndexFromChunkTensorCUDA / LocalIndex... / HostIndex...
 * (src/cuda/index_with_chunk_tensor.cu:9-53, :110-128/:170-194, :150-168/:223-247).
 * A row that straddles the device/host boundary is resolved per element, like
 * chunk_tensor_wrapper::At (src/chunk_tensor.h:33-42), also for DGS_TIER_HOST
 * (the reference's HostAt, src/chunk_tensor.h:56-58, reaches in front of the host
 * slice for such a row).  `out` holds n * row_elems elements.
 * Index values are checked before they address anything (the reference does not
 * check, src/cuda/index_with_chunk_tensor.cu:16-23): a row outside the store, or
 * with DGS_TIER_DEVICE / DGS_TIER_HOST a row the tier does not hold whole, is not
 * read; its output row is zero bytes and *bad_index (device-visible int64, may be
 * NULL, never cleared by the library) is set to 1 when the kernel runs.
 */
dgs_status dgs_gather_rows(dgs_view v, int64_t row_elems, const void* index,
                           int32_t index_bytes, int64_t n, void* out,
                           int32_t tier, int64_t* bad_index, void* stream);

/*
 * Same gather with the row count read from device memory when the kernel runs:
 * `n_rows_dev` points to an int64; `index` must hold n_max readable ids (whatever the count turns
 * out to be, the kernel may read all of them) and `out` n_max rows.  A count above n_max (or
 * below 0) gathers nothing at all, so a caller may offer a buffer smaller than the worst case and
 * gather again, exactly, when the count turns out not to fit.  Lets a caller enqueue the gather
 * of a frontier whose length a previous kernel on the same stream is still computing.
 * `n_expected` sizes the launch: the number of rows the caller expects (the previous batch's
 * count plus a margin, say); 0 or less, or more than n_max: n_max.  It is a hint only: any count
 * up to n_max is gathered in full, by blocks that loop when there are more rows than expected.
 * No counterpart in the reference (which reads every length back to the host first).
 */
dgs_status dgs_gather_rows_dyn(dgs_view v, int64_t row_elems, const void* index,
                               int32_t index_bytes, int64_t n_max,
                               const int64_t* n_rows_dev, int64_t n_expected, void* out,
                               int32_t tier, int64_t* bad_index, void* stream);

/*
 * dgs_gather_rows_dyn for a gather that shares the GPU with other streams' kernels which need
 * wave slots more than memory bandwidth (the weighted sampler's fills are bound by vector
 * arithmetic): at most `blocks_per_cu` of the gather's 256-thread blocks are resident on a CU at
 * a time (3..7; 0, or 8 and more: all that fit, as dgs_gather_rows_dyn).  The kernel reserves
 * on-chip memory it does not use, nothing else changes; results are those of dgs_gather_rows_dyn.
 * By itself the gather loses about 1.5 % at 4 blocks per CU and 4 % at 3; a step of weighted
 * batches in flight gains 11 % at 4.  No counterpart in the reference.
 */
dgs_status dgs_gather_rows_dyn_shared(dgs_view v, int64_t row_elems, const void* index,
                                      int32_t index_bytes, int64_t n_max,
                                      const int64_t* n_rows_dev, int64_t n_expected, void* out,
                                      int32_t tier, int32_t blocks_per_cu, int64_t* bad_index,
                                      void* stream);

/*
 * Stable partition of an index list into (device-resident rows, host-resident
 * rows): row r is "host" iff r >= threshold / row_elems
 * (src/cuda/index_with_chunk_tensor.cu:55-108; the "remote" class is empty at
 * world size 1).  out_local / out_host each hold up to n ids; counts_dev[0..1]
 * (int64, device) receive the two lengths.
 */
size_t dgs_split_index_workspace_bytes(int64_t n);
dgs_status dgs_split_index(dgs_view v, int64_t row_elems, const void* index,
                           int32_t index_bytes, int64_t n, void* out_local,
                           void* out_host, int64_t* counts_dev, void* workspace,
                           size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------ */
/* Row-wise uniform neighbour sampling over CSC                              */
/* ------------------------------------------------------------------------ */

/*
 * Random-number contract ("dgs-philox-1"), shared bit for bit with the CPU
 * oracle: draw number j of row r is the Philox4x32-10 block with
 *   key     = (rng_seed & 0xffffffff, rng_seed >> 32)
 *   counter = (j, rng_stream, r & 0xffffffff, r >> 32)
 * reduced to [0, n) by Lemire's multiply-shift with rejection over the block's
 * four words in order (the fourth word is accepted unconditionally).
 *   - without replacement, deg > k: Floyd's subset algorithm; step i (0-based)
 *     draws t in [0, deg-k+i] and keeps t unless an earlier step kept it, in
 *     which case it keeps deg-k+i; output slot i holds that position;
 *   - without replacement, deg <= k: the whole row in CSC order;
 *   - with replacement, deg > 0: slot i holds draw i reduced to [0, deg).
 */

/*
 * One hop.  For every seed row (in order) emits its picks contiguously:
 *   out_rows[e] = seed id, out_cols[e] = picked neighbour id.
 * Replaces RowWiseSamplingUniformWithChunkTensorCUDA and
 * RowWiseSamplingUniformCUDA (src/cuda/rowwise_sampling_with_chunk_tensor.cu:113-194,
 * src/cuda/rowwise_sampling.cu:13-187).
 *   seeds    : device, n_seeds ids of width id_bytes (also the width of
 *              out_rows / out_cols and of `indices`)
 *   indptr   : view of N+1 offsets, elem_bytes 4 or 8
 *   indices  : view of E ids, elem_bytes == id_bytes
 *   n_edges  : (dgs_sample_count) entries of the edge array the offsets point into
 *              (indices.total); a row whose offsets leave [0, n_edges] is flagged
 *   nnz_dev  : device int64[2]; [0] receives the number of emitted edges,
 *              [1] flags: bit 0 = some row has degree >= 2^32 or offsets outside
 *              the edge array, bit 1 = some seed id is not a row of the graph (the
 *              reference checks neither; here an id is tested before it addresses
 *              indptr, and offsets before the fill uses them).  Flagged
 *              rows emit nothing; the caller reports DGS_ERR_RANGE.
 *              Every num_picks is served, as by the reference's reservoir
 *              kernel (src/cuda/rowwise_sampling.cu:42-99).
 *   workspace: dgs_sample_workspace_bytes(n_seeds) bytes, 256-byte aligned,
 *              shared by the count and the fill of the same hop
 *
 * dgs_sample_count is the degree/count/scan half (the reference's sub_indptr,
 * rowwise_sampling_with_chunk_tensor.cu:127-156): it leaves the per-row
 * offsets in the workspace and the edge count in nnz_dev, and mirrors nnz_dev
 * into nnz_host when that is given (int64[2] of pinned host memory that the
 * device can write; NULL: no mirror): a caller that records a ticket behind
 * this call, enqueues the fill and then waits for the ticket reads the length
 * while the fill still runs.
 * dgs_sample_fill is the COO fill (:15-111, :158-180); out_rows / out_cols
 * must hold nnz ids.  dgs_sample_neighbors runs both; its outputs must hold
 * n_seeds * num_picks ids (the worst case), so no length is read back between
 * the two halves.  Nothing synchronises: copy nnz_dev when the length is needed.
 */
size_t dgs_sample_workspace_bytes(int64_t n_seeds);
dgs_status dgs_sample_count(const void* seeds, int32_t id_bytes, int64_t n_seeds,
                            dgs_view indptr, int64_t n_edges, int64_t num_picks, int32_t replace,
                            int64_t* nnz_dev, int64_t* nnz_host, void* workspace,
                            size_t workspace_bytes, void* stream);
dgs_status dgs_sample_fill(const void* seeds, int32_t id_bytes, int64_t n_seeds,
                           dgs_view indices, int64_t num_picks, int32_t replace,
                           uint64_t rng_seed, uint32_t rng_stream, void* out_rows,
                           void* out_cols, void* workspace, size_t workspace_bytes,
                           void* stream);
dgs_status dgs_sample_neighbors(const void* seeds, int32_t id_bytes,
                                int64_t n_seeds, dgs_view indptr,
                                dgs_view indices, int64_t num_picks,
                                int32_t replace, uint64_t rng_seed,
                                uint32_t rng_stream, void* out_rows,
                                void* out_cols, int64_t* nnz_dev,
                                void* workspace, size_t workspace_bytes,
                                void* stream);

/*
 * dgs_sample_neighbors without a workspace argument and without any allocation.  No
 * counterpart in the reference; it is for callers that cannot allocate device memory at the
 * point of the call: code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc.  The per-seed temporaries live in a fixed array inside the library (2 MiB per GPU,
 * held until the process ends), which bounds the call to DGS_STATIC_MAX_SEEDS seeds
 * (DGS_ERR_UNSUPPORTED above that).  Arguments, outputs (out_rows / out_cols hold
 * n_seeds * num_picks ids), flags and results are those of dgs_sample_neighbors.  Calls on one
 * GPU share that GPU's array: two calls that overlap in time on the same GPU (different
 * streams or host threads) race; calls on one stream do not.  The first call on a device
 * looks the array's address up and should be made outside graph capture.
 */
#define DGS_STATIC_MAX_SEEDS 65536
dgs_status dgs_sample_neighbors_static(const void* seeds, int32_t id_bytes,
                                       int64_t n_seeds, dgs_view indptr,
                                       dgs_view indices, int64_t num_picks,
                                       int32_t replace, uint64_t rng_seed,
                                       uint32_t rng_stream, void* out_rows,
                                       void* out_cols, int64_t* nnz_dev,
                                       void* stream);

/*
 * One weighted hop: like dgs_sample_neighbors with a float32 weight per edge
 * (`probs`, a view of E floats laid out like `indices`).  Replaces
 * RowWiseSamplingProbCUDA and RowWiseSamplingProbWithChunkTensorCUDA
 * (src/cuda/rowwise_sampling_probs.cu:218-279,
 * src/cuda/rowwise_sampling_probs_with_chunk_tensor.cu:181-293).  Pick counts are
 * those of the uniform sampler, so dgs_sample_count is the shared first half.
 *   - without replacement, deg <= num_picks: the whole row in CSC order;
 *   - without replacement, deg > num_picks (num_picks <= 64; the reference
 *     asserts <= 32): every position p races with the key E_p / w_p, E_p =
 *     -ln((x + 0.5) / 2^32) for x = word p & 3 of the Philox block with counter
 *     (0x80000000 | p >> 2, rng_stream, row), computed in float64 from exactly
 *     rounded operations; weights that are not > 0 get the key +inf.  The
 *     num_picks smallest (key, position) pairs win and are emitted in that order.
 *     This is the reference's A-Res rule (largest u^(1/w)) in logarithms;
 *   - with replacement, deg > 0: slot j picks position i with probability
 *     q_i / sum(q), q_i = floor(w_i * 2^(32-E)) with 2^(E-1) <= max(w) < 2^E
 *     (an exact power-of-two scaling; 0 for weights not > 0):
 *     the Philox block with counter (0x40000000 | j, rng_stream, row) is reduced to
 *     [0, sum(q)) by Lemire's rule on its first 64 bits (second 64 bits accepted
 *     unconditionally) and located by an upper bound on the inclusive sums of q;
 *     a row with sum(q) == 0 picks its last position, like the reference's
 *     clamped search (rowwise_sampling_probs.cu:203-204).
 * Both rules are shared bit for bit with the CPU oracle.
 */
dgs_status dgs_sample_fill_weighted(const void* seeds, int32_t id_bytes,
                                    int64_t n_seeds, dgs_view indices,
                                    dgs_view probs, int64_t num_picks,
                                    int32_t replace, uint64_t rng_seed,
                                    uint32_t rng_stream, void* out_rows,
                                    void* out_cols, void* workspace,
                                    size_t workspace_bytes, void* stream);
dgs_status dgs_sample_neighbors_weighted(const void* seeds, int32_t id_bytes,
                                         int64_t n_seeds, dgs_view indptr,
                                         dgs_view indices, dgs_view probs,
                                         int64_t num_picks, int32_t replace,
                                         uint64_t rng_seed, uint32_t rng_stream,
                                         void* out_rows, void* out_cols,
                                         int64_t* nnz_dev, void* workspace,
                                         size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------ */
/* Unique + relabel                                                          */
/* ------------------------------------------------------------------------ */

#define DGS_MAX_SEGMENTS 8
/* A logical concatenation of up to DGS_MAX_SEGMENTS device arrays of ids. */
typedef struct dgs_segments {
  const void* ptr[DGS_MAX_SEGMENTS];
  int64_t len[DGS_MAX_SEGMENTS];
  int32_t count;
  int32_t reserved_;
} dgs_segments;

/*
 * unique  = distinct ids of cat(mapping) in first-occurrence order;
 * out[t][i] = position of requiring[t][i] in unique, or -1 when absent.
 * Replaces TensorRelabelCUDA / Unique / Relabel / RelabelHashmap
 * (src/cuda/tensor_reindex.cu:11-205).
 *   packed_table   : 8-byte ids only.  Non-zero: the table keeps id and position in one 64-bit
 *                    slot (one atomic per id instead of two), which holds ids below 2^32 - 1; an
 *                    id beyond that sets counts_dev[1] and voids the call's results (call again
 *                    with 0).  Zero: id array + value array, any id >= 0.
 *   unique_out     : device, capacity sum(mapping.len) ids
 *   counts_dev     : device int64[2]: [0] number of distinct ids, [1] non-zero if an id did not
 *                    fit the packed table
 *   counts_host / counts_ticket : optional (a ticket only with counts_host; counts_host alone
 *                    is for callers that poll it, dgs_stream_wait_words).  counts_host is pinned host memory
 *                    that the device can write; the kernels mirror counts_dev into it, and
 *                    *counts_ticket marks the point on `stream` after which it is complete:
 *                    before `unique_out` and `out` are written, so that a caller can wait for the
 *                    count (dgs_ticket_wait) while those kernels still run.  Saves the reference's
 *                    blocking read at the end (src/cuda/tensor_reindex.cu:129).
 *   out            : device arrays, out.len must equal requiring.len
 * Mapping ids must be >= 0 (-1 is the empty-slot marker, as in the reference); a requiring id that
 * is negative or not in the mapping list gives -1.
 * sum(mapping.len) must be <= 2^30.
 */
size_t dgs_unique_relabel_workspace_bytes(int64_t n_mapping, int32_t id_bytes);
dgs_status dgs_unique_relabel(dgs_segments mapping, dgs_segments requiring,
                              int32_t id_bytes, int32_t packed_table, void* unique_out,
                              int64_t* counts_dev, int64_t* counts_host,
                              void** counts_ticket, dgs_segments out,
                              void* workspace, size_t workspace_bytes,
                              void* stream);

/* ------------------------------------------------------------------------ */
/* Multi-hop driver                                                          */
/* ------------------------------------------------------------------------ */

#define DGS_MAX_HOPS 8
/* Caller-allocated edge outputs of one hop, each sized for the worst case reported by
 * dgs_sample_blocks_plan (edges_max[h] ids). */
typedef struct dgs_block_out {
  void* src_local; /* rank of every picked neighbour in the hop's frontier */
  void* dst_local; /* rank of every edge's seed in the hop's frontier      */
} dgs_block_out;

/*
 * All hops of ChunkTensorSampler.sample_blocks
 * (oppo_bench/single_node/utils/chunktensor_sampler.py:93-118) as one sequence of
 * kernels with no host synchronisation: for hop h (fanouts[h], ALREADY in hop order,
 * i.e. the reversed model fanouts) sample the current seeds, relabel
 * ([seeds, picked], [seed of edge, picked]) and continue with the frontier as seeds.
 * Results are identical to calling dgs_sample_neighbors (rng_stream = first_stream + h)
 * and dgs_unique_relabel per hop.
 *
 * Because a hop's frontier starts with its seeds, the frontiers of successive hops are
 * prefixes of one array: `frontier` (capacity seeds_max[n_hops] ids) receives it, and
 * hop h's frontier is frontier[0 .. sizes[h+1]).
 *
 *   dgs_sample_blocks_plan : worst-case sizes; seeds_max has n_hops + 1 entries
 *                            (seeds_max[0] = n_seeds), edges_max has n_hops
 *   sizes_dev              : device int64[3 * n_hops + 1]:
 *                            [0 .. n_hops]                 seeds of hop h (h = n_hops: final frontier size)
 *                            [n_hops + 1 .. 2 n_hops]      edges of hop h
 *                            [2 n_hops + 1 .. 3 n_hops]    error bits of hop h: 1 a row had degree >= 2^32 or
 *                                                          offsets outside the edge array, 2 a seed id is
 *                                                          not a row of the graph, 4 a picked neighbour id
 *                                                          is not a node (each checked before it addresses
 *                                                          anything; such rows emit nothing), 8 the last hop's
 *                                                          bucketed pass met a bucket with more distinct ids
 *                                                          than its on-chip table holds (the hop's results are
 *                                                          void; ids that crowd one bucket of the library's
 *                                                          hash: run the call again with
 *                                                          DGS_DEBUG_SAMPLER_BUCKETED = 1)
 *   sizes_host / ticket    : optional (a ticket only with sizes_host).  sizes_host is pinned host
 *                            memory that the device can write (hipHostMalloc); the kernels mirror
 *                            sizes_dev into it, and *sizes_ticket marks the point on `stream`
 *                            after which it is complete -- before the last hop's edge lists are
 *                            written, so a caller can enqueue more work (a feature gather) and
 *                            only then call dgs_ticket_wait.  Saves the device-to-host copy.
 *                            A caller that polls the words (dgs_stream_wait_words, or
 *                            dgs_ticket_sync_words on a ticket of its own recorded later) passes
 *                            sizes_host alone: every ticket is an event on the stream, and an
 *                            event between two kernels costs the GPU some 6 us of idling.
 *   node_table / epoch     : optional persistent direct-address table of
 *                            dgs_node_table_bytes(n_nodes) bytes (n_nodes = indptr entries - 1,
 *                            < 2^31), filled with 0xFF bytes before its first use and then never
 *                            cleared: pass a strictly increasing epoch (1, 2, 3, ...) with every
 *                            call that uses it, and do not share it between calls that may run
 *                            concurrently.  With NULL the call builds a hash table inside the
 *                            workspace instead (one extra clearing launch, slower inserts).
 * Limits of this entry point (each is DGS_ERR_UNSUPPORTED, none is silent): fanouts above 64 (use
 * the per-hop entry points, which take any fanout); a worst-case frontier S * prod(1 + k_h) above
 * 2^30 ids (positions are 32-bit words with two flag bits); a node table for 2^31 nodes or more
 * (dgs_node_table_bytes returns 0).  The operator layer above adds two of its own: it makes node
 * tables only below 8 GiB each (larger graphs sample on the per-call hash table) and keeps at
 * most four per graph, one per stream that samples from it.
 */
dgs_status dgs_sample_blocks_plan(int64_t n_seeds, const int64_t* fanouts,
                                  int32_t n_hops, int64_t* seeds_max,
                                  int64_t* edges_max);
size_t dgs_sample_blocks_workspace_bytes(int64_t n_seeds, const int64_t* fanouts,
                                         int32_t n_hops, int32_t id_bytes);
size_t dgs_node_table_bytes(int64_t n_nodes);
dgs_status dgs_sample_blocks(const void* seeds, int32_t id_bytes, int64_t n_seeds,
                             dgs_view indptr, dgs_view indices,
                             const int64_t* fanouts, int32_t n_hops, int32_t replace,
                             uint64_t rng_seed, uint32_t first_stream,
                             void* node_table, uint32_t node_table_epoch,
                             void* frontier, const dgs_block_out* outs,
                             int64_t* sizes_dev, int64_t* sizes_host,
                             void** sizes_ticket, void* workspace,
                             size_t workspace_bytes, void* stream);

/*
 * The same multi-hop driver with weighted picks: every hop chooses neighbours by the
 * edge weights `probs` (float32, one per edge, laid out like `indices`), by the rules
 * stated at dgs_sample_fill_weighted.  Results are identical to calling
 * dgs_sample_neighbors_weighted (rng_stream = first_stream + h) and dgs_unique_relabel
 * per hop: the loop of ChunkTensorSampler.sample_blocks with chunk_probs
 * (oppo_bench/single_node/utils/chunktensor_sampler.py:93-118).  All other arguments are
 * those of dgs_sample_blocks (`node_table` optional, as there); the workspace is sized by
 * the _weighted_ query.
 */
size_t dgs_sample_blocks_weighted_workspace_bytes(int64_t n_seeds, const int64_t* fanouts,
                                                  int32_t n_hops, int32_t id_bytes);
dgs_status dgs_sample_blocks_weighted(const void* seeds, int32_t id_bytes, int64_t n_seeds,
                                      dgs_view indptr, dgs_view indices, dgs_view probs,
                                      const int64_t* fanouts, int32_t n_hops,
                                      int32_t replace, uint64_t rng_seed,
                                      uint32_t first_stream, void* node_table,
                                      uint32_t node_table_epoch, void* frontier,
                                      const dgs_block_out* outs, int64_t* sizes_dev,
                                      int64_t* sizes_host, void** sizes_ticket,
                                      void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------ */
/* Placement                                                                 */
/* ------------------------------------------------------------------------ */

/*
 * Rewrites the edge array of a CSC graph for a renumbering of its nodes, so that the
 * rows a positional store keeps in HBM (the first ones) are the hottest.  No counterpart
 * in the reference's native code: its stores are positional too (src/chunk_tensor.h:33-42)
 * and the harness caches "the first rows" (chunktensor_sampler.py:32-60), which only
 * pays when the caller has ordered the nodes beforehand.
 *   order      : device int64[n_rows], order[new] = old
 *   rank       : device ids (id_bytes wide)[n_rows], rank[old] = new
 *   new_indptr : device offsets (ptr_bytes wide)[n_rows + 1], the exclusive scan of the
 *                old degrees taken in the new order
 *   new_indices: device ids[n_edges]; new row r receives the edges of old row order[r]
 *                in their old order, endpoints renamed through rank
 * All arrays are plain device memory (a renumbering is done before the stores are filled).
 */
dgs_status dgs_renumber_csc(const void* old_indptr, int32_t ptr_bytes,
                            const void* old_indices, int32_t id_bytes,
                            const int64_t* order, const void* rank,
                            const void* new_indptr, int64_t n_rows, int64_t n_edges,
                            void* new_indices, void* stream);

/* ------------------------------------------------------------------------ */
/* Small utilities                                                           */
/* ------------------------------------------------------------------------ */

/*
 * Copies n_bytes from device memory to `host_dst` on `stream` and waits for the
 * stream: the blocking length read the reference does after each scan
 * (src/cuda/rowwise_sampling_with_chunk_tensor.cu:154-156, src/cuda/tensor_reindex.cu:129).
 */
dgs_status dgs_read_back(void* host_dst, const void* dev_src, size_t n_bytes,
                         void* stream);
/*
 * The same read in two halves: _begin enqueues the copy on `stream` and marks that point,
 * _wait blocks until the copy (not later work on the stream) has finished.  Work enqueued
 * between the two keeps the GPU busy while the host waits for the lengths.  `host_dst`
 * should be pinned memory and must stay untouched until _wait returns.  Every ticket must
 * be waited on exactly once.
 */
dgs_status dgs_read_back_begin(void* host_dst, const void* dev_src, size_t n_bytes,
                               void* stream, void** ticket);
dgs_status dgs_read_back_wait(void* ticket);
/*
 * Tickets on their own: _record marks the current end of `stream`; _wait blocks the host
 * until that point is reached (and retires the ticket: exactly one _wait per ticket);
 * _stream_wait makes `stream` wait for it without blocking the host (call before _wait
 * or _release); _release retires a ticket nobody on the host needs to wait for.
 * dgs_read_back_wait is dgs_ticket_wait.
 */
dgs_status dgs_ticket_record(void* stream, void** ticket);
dgs_status dgs_ticket_stream_wait(void* stream, void* ticket);
dgs_status dgs_ticket_wait(void* ticket);
/*
 * dgs_ticket_wait for a ticket that stands for length words mirrored into pinned host memory
 * (nnz_host of dgs_sample_count, counts_host of dgs_unique_relabel, sizes_host of
 * dgs_sample_blocks[_weighted]).  The kernels store every mirrored word at system scope, each
 * final the moment it is written and never negative, so a caller that sets the words to -1
 * before the call may take them as soon as all have turned non-negative: this call polls the
 * `n_words` words and returns then, some microseconds before the ticket's event would have been
 * seen (6 against 12 us after a short kernel on an MI355X), or when the ticket's point is
 * reached, whichever comes first.  It retires the ticket like dgs_ticket_wait.  Words that are
 * still negative on return were not written by the call.  No counterpart in the reference,
 * which copies its lengths back with a blocking cudaMemcpy.
 */
dgs_status dgs_ticket_wait_words(void* ticket, const int64_t* words, int32_t n_words);
/*
 * dgs_ticket_wait and dgs_ticket_wait_words for a ticket that more than one party looks at (the
 * host thread that wants a batch's lengths, a later batch whose gather waits its turn, the owner
 * of a node table): they block in the same way but leave the ticket valid; whoever lets go of it
 * last calls dgs_ticket_release.
 */
dgs_status dgs_ticket_sync(void* ticket);
dgs_status dgs_ticket_sync_words(void* ticket, const int64_t* words, int32_t n_words);
/*
 * The same wait without a ticket (recording one costs the caller 1-4 us per call): polls the
 * words and gives up once `stream`, the stream the call was enqueued on, has drained.  For
 * callers that wait right after the call, on the thread that made it.
 */
dgs_status dgs_stream_wait_words(void* stream, const int64_t* words, int32_t n_words);
dgs_status dgs_ticket_release(void* ticket);
/*
 * *idle = 1 when everything enqueued on `stream` so far has finished, else 0.  Never blocks.
 * A handle that no longer names a live stream counts as drained (the runtime's "invalid handle"
 * answer, and only that one, is taken as idle); any other failure of the query is DGS_ERR_HIP and
 * stays visible to the caller's next HIP call.  Meant for streams the caller knows to be alive;
 * to learn whether earlier work has finished without holding on to a stream, record a ticket
 * behind it and ask dgs_ticket_query.
 */
dgs_status dgs_stream_query(void* stream, int32_t* idle);
/*
 * *reached = 1 when the point a ticket marks has been reached, else 0.  Never blocks and does not
 * retire the ticket.  A ticket belongs to the library, not to the stream it was recorded on, so
 * the answer is well defined whatever has become of that stream since.
 */
dgs_status dgs_ticket_query(void* ticket, int32_t* reached);

#ifdef __cplusplus
}
#endif
#endif /* DGS_HIP_H_ */
