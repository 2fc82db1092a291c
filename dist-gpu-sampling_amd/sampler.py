"""Host-side counterpart of the upstream sampler glue
(oppo_bench/single_node/utils/chunktensor_sampler.py) at world size 1, without
DGL: a block is a plain record instead of a DGLBlock.
"""
import threading
from collections import deque, namedtuple

import torch

class _FastOps:
    """torch.ops.dgs_ops.<name> by their C++ entries (`OpOverloadPacket._op`): the same callables
    with the same arguments, results and errors, minus the packet's Python-side walk over the
    arguments for FakeScriptObjects (export / compile tracing, which operators that block on
    data-dependent sizes do not support anyway; 4 us a call).  Nothing of torch is modified."""

    def __getattr__(self, name):
        packet = getattr(torch.ops.dgs_ops, name)
        entry = getattr(packet, "_op", None)
        entry = entry if callable(entry) else packet
        setattr(self, name, entry)
        return entry


fast_ops = _FastOps()


# One message-flow block: edges (src_local[e] -> dst_local[e]); src_ids / dst_ids map
# local to global node ids (upstream: block.srcdata[dgl.NID] / block.dstdata[dgl.NID]).
Block = namedtuple("Block", ["src_local", "dst_local", "num_src", "num_dst", "src_ids", "dst_ids"])


def set_rng_state(seed, stream=0):
    """Seeds the process-wide sampling generator; its stream advances by one per sampled hop.
    Samplers made with `seed=` keep their own state and do not touch this one."""
    torch.ops.dgs_ops._CAPI_set_rng_state(int(seed), int(stream))


def set_gather_buffer_cap(nbytes):
    """Largest worst-case feature buffer the fused operators allocate before a batch's sizes are
    known (default 2 GiB).  Above it a batch waits for its frontier size and gathers into exactly
    that many rows: memory stays bounded, the host blocks a little earlier."""
    torch.ops.dgs_ops._CAPI_set_gather_buffer_cap(int(nbytes))


# guards the process-wide generator while a sampler with its own state borrows it for a per-hop call
_rng_lock = threading.Lock()


def create_dgs_communicator(group_size=1, local_group=None):
    """chunktensor_sampler.py:7-19.  World size is 1: the id exchange is a no-op."""
    unique_ids = torch.ops.dgs_ops._CAPI_get_unique_id()
    torch.ops.dgs_ops._CAPI_set_nccl(group_size, unique_ids, 0)


def get_available_memory(device, reserved_mem, local_group=None):
    """chunktensor_sampler.py:22-29 without the all_reduce(MIN) over ranks."""
    available = (torch.cuda.mem_get_info(device)[1] - reserved_mem
                 - torch.ops.dgs_ops._CAPI_get_current_allocated()
                 - 0.3 * torch.cuda.max_memory_reserved())
    return int(max(available, 0))


def cached_bytes_per_gpu(total_bytes, num_gpus, available_mem, cache_rate=1.0):
    """chunktensor_sampler.py:40-42: int(min(total_bytes * cache_rate // num_gpus, available_mem))."""
    return int(min(total_bytes * cache_rate // num_gpus, available_mem))


def create_chunktensor(tensor, num_gpus, available_mem, cache_rate=1.0, root_rank=0, local_group=None):
    """chunktensor_sampler.py:32-60: a store of the tensor's shape and dtype whose capacity per GPU
    is cached_bytes_per_gpu(...), filled from the tensor."""
    if num_gpus != 1:
        raise ValueError("this build runs at world size 1")
    total_size = tensor.numel() * tensor.element_size()
    cached_size_per_gpu = cached_bytes_per_gpu(total_size, num_gpus, available_mem, cache_rate)
    chunk_tensor = torch.classes.dgs_classes.ChunkTensor(list(tensor.shape), tensor.dtype, cached_size_per_gpu)
    chunk_tensor._CAPI_load_from_tensor(tensor)
    return chunk_tensor


class PendingBatch:
    """A batch whose kernels are enqueued (ChunkTensorSampler.submit).  result() waits until the
    batch's sizes are known and returns what sample_blocks / sample_blocks_and_index return; the
    last kernels of the batch may still be running on the stream it was submitted on, so a consumer
    on another stream orders itself after that stream (`consumer.wait_stream(batch.stream)`)."""

    def __init__(self, handle, seed_nodes, with_features, stream):
        self._handle = handle
        self._seed_nodes = seed_nodes
        self._with_features = with_features
        self.stream = stream

    def result(self):
        frontiers, srcs, dsts, x, seeds = self._handle._CAPI_finish()
        blocks = ChunkTensorSampler._blocks(seeds, frontiers, srcs, dsts)
        if self._with_features:
            return frontiers[-1], self._seed_nodes, blocks, x
        return frontiers[-1], self._seed_nodes, blocks


class ChunkTensorSampler:
    """chunktensor_sampler.py:62-118, same positional arguments (the DGL prefetch options of
    BlockSampler have no counterpart here).

    sample_blocks runs the upstream loop -- per hop one sampling call and one relabel call,
    over reversed(fanouts) -- through the single fused operator when every fanout is at most
    64 (`fused=False` forces the per-hop operators; both give identical results).  With
    `chunk_probs` (a float32 ChunkTensor of edge weights) every hop picks by weight, as
    upstream does (:97-100).

    With `seed` the sampler owns its random state: batch number b (counted per sampler, or given
    as `batch=` to submit / sample_blocks) draws hop h from stream `b * len(fanouts) + h` of that
    seed, whatever other samplers or host threads do.  Without it the process-wide generator of
    set_rng_state is used, as upstream's single global state.
    """

    FUSED_MAX_FANOUT = 64

    def __init__(self, fanouts, chunk_indptr, chunk_indices, chunk_probs=None, replace=False, fused=True,
                 seed=None):
        self.chunk_indptr = chunk_indptr
        self.chunk_indices = chunk_indices
        self.chunk_probs = chunk_probs
        self.fanouts = list(fanouts)
        self.replace = replace
        self.fused = fused and all(0 <= f <= self.FUSED_MAX_FANOUT for f in self.fanouts)
        self.seed = None if seed is None else int(seed)
        self._batches = 0
        self._count_lock = threading.Lock()
        self._loops = {}  # BatchPipeline's native loops (each with a worker thread), kept for reuse
        # where the operators are looked up: their C++ entries, or torch.ops.dgs_ops itself (what
        # an unmodified upstream harness calls through) when a caller sets that
        self.ops = fast_ops

    def _first_stream(self, batch):
        """Stream of the first hop of a batch drawn from the sampler's own state."""
        if batch is None:
            with self._count_lock:
                batch = self._batches
                self._batches += 1
        return int(batch) * len(self.fanouts)

    @staticmethod
    def _blocks(seeds, frontiers, srcs, dsts):
        blocks = []
        for frontier, src, dst in zip(frontiers, srcs, dsts):
            blocks.insert(0, Block(src, dst, frontier.numel(), seeds.numel(), frontier, seeds))
            seeds = frontier
        return blocks

    def sample_blocks(self, g, seed_nodes, exclude_eids=None, batch=None):
        """Returns (input_nodes, seed_nodes, blocks); `g` is unused, as upstream.  Host-side
        seed_nodes (what upstream's DataLoader passes) are uploaded by the operator itself."""
        if self.fused and (self.chunk_probs is not None or self.seed is not None):
            return self.submit(g, seed_nodes, batch=batch).result()
        if self.seed is not None:  # per-hop operators draw from the process-wide state: lend it ours
            with _rng_lock:
                saved = torch.ops.dgs_ops._CAPI_get_rng_state()
                torch.ops.dgs_ops._CAPI_set_rng_state(self.seed, self._first_stream(batch))
                try:
                    return self._sample_blocks_per_hop(seed_nodes)
                finally:
                    torch.ops.dgs_ops._CAPI_set_rng_state(*saved)
        if self.fused:
            frontiers, srcs, dsts, seeds = self.ops._CAPI_sample_blocks(
                seed_nodes, self.chunk_indptr, self.chunk_indices, list(reversed(self.fanouts)), self.replace)
            return frontiers[-1], seed_nodes, self._blocks(seeds, frontiers, srcs, dsts)
        return self._sample_blocks_per_hop(seed_nodes)

    def _sample_blocks_per_hop(self, seed_nodes):
        """The upstream loop itself (chunktensor_sampler.py:93-118), one operator call per step."""
        seeds = seed_nodes.cuda()
        blocks = []
        frontier = seeds
        for fan_out in reversed(self.fanouts):
            if self.chunk_probs is not None:
                coo_row, coo_col = self.ops._CAPI_sample_neighbors_with_probs_with_chunk_tensor(
                    seeds, self.chunk_indptr, self.chunk_indices, self.chunk_probs, fan_out, self.replace)
            else:
                coo_row, coo_col = self.ops._CAPI_sample_neighbors_with_chunk_tensor(
                    seeds, self.chunk_indptr, self.chunk_indices, fan_out, self.replace)
            frontier, (coo_row, coo_col) = self.ops._CAPI_tensor_relabel(
                [seeds, coo_col], [coo_row, coo_col])
            blocks.insert(0, Block(coo_col, coo_row, frontier.numel(), seeds.numel(), frontier, seeds))
            seeds = frontier
        return frontier, seed_nodes, blocks

    def submit(self, g, seed_nodes, chunk_features=None, batch=None, gather_after=None):
        """Enqueues a batch on the current stream and returns at once (fused path only).  Batches
        submitted on different streams overlap on the GPU: the short kernels of one batch's first
        hops fill the gaps between the large kernels of another.  Results come from
        PendingBatch.result(), in any order."""
        if not self.fused:
            raise RuntimeError("submit() needs the fused path: every fanout <= 64")
        hop_fanouts = list(reversed(self.fanouts))
        rng = [] if self.seed is None else [self.seed, self._first_stream(batch)]
        handle = self.ops._CAPI_sample_blocks_submit(
            seed_nodes, self.chunk_indptr, self.chunk_indices, self.chunk_probs, hop_fanouts, self.replace,
            chunk_features, rng, 0 if gather_after is None else gather_after.cuda_event)
        return PendingBatch(handle, seed_nodes, chunk_features is not None, torch.cuda.current_stream())

    def sample_blocks_and_index(self, g, seed_nodes, chunk_features):
        """sample_blocks followed by chunk_features._CAPI_index(input_nodes)
        (oppo_bench/single_node/chunktensor.py:142-151), with the gather enqueued behind
        the last hop before any length is read back.  Returns (input_nodes, seed_nodes,
        blocks, features_of_input_nodes)."""
        if not self.fused:
            frontier, _, blocks = self.sample_blocks(g, seed_nodes)
            return frontier, seed_nodes, blocks, chunk_features._CAPI_index(frontier)
        if self.chunk_probs is not None or self.seed is not None:
            return self.submit(g, seed_nodes, chunk_features).result()
        frontiers, srcs, dsts, x, seeds = self.ops._CAPI_sample_blocks_and_index(
            seed_nodes, self.chunk_indptr, self.chunk_indices, list(reversed(self.fanouts)), self.replace,
            chunk_features)
        return frontiers[-1], seed_nodes, self._blocks(seeds, frontiers, srcs, dsts), x


_pipeline_streams = []
_event_sets = {}  # streams of a pipeline -> spare (seeds ready, batch done) event lists


OVERLAP_PROBE_BYTES = 1 << 30  # what the probe's long fill writes at most (a fill of some 300 us)


def _overlap_scratch():
    """The buffer streams_overlap fills: OVERLAP_PROBE_BYTES, or an eighth of the free device memory
    if that is less; None when even 16 MiB cannot be had (the probe is skipped then)."""
    try:
        free = torch.cuda.mem_get_info()[0]
        nbytes = min(OVERLAP_PROBE_BYTES, free // 8)
        if nbytes < (16 << 20):
            return None
        return torch.empty(nbytes // 4, dtype=torch.float32, device="cuda")
    except torch.cuda.OutOfMemoryError:
        return None


def streams_overlap(a, b, scratch=None):
    """Whether work on stream `b` can run while stream `a` is busy.  HIP spreads a process's streams
    over a few hardware queues (four by default), and two streams that land on the same queue run
    their kernels in submission order however independent they are.  Measured, not looked up: a
    long fill is enqueued on `a`, a tiny one on `b`, and the host watches which finishes when.
    Without memory for the long fill nothing can be measured and the answer is True."""
    import time
    if scratch is None:
        scratch = _overlap_scratch()
        if scratch is None:
            return True
    tiny = torch.empty(64, dtype=torch.float32, device="cuda")
    done_a, done_b = torch.cuda.Event(), torch.cuda.Event()
    votes = 0
    for _ in range(3):
        torch.cuda.synchronize()
        with torch.cuda.stream(a):
            scratch.fill_(1.0)
            done_a.record()
        with torch.cuda.stream(b):
            tiny.fill_(1.0)
            done_b.record()
        t0 = time.perf_counter()
        done_b.synchronize()
        t1 = time.perf_counter()
        done_a.synchronize()
        t2 = time.perf_counter()
        votes += (t1 - t0) < 0.5 * (t2 - t0)
    return votes >= 2


def pipeline_streams(n):
    """The first n of the streams that BatchPipeline objects run on by default.  They are shared by
    all pipelines of the process: a graph keeps one node table per stream that ever sampled from
    it (at most four), so pipelines that come and go should not each bring new streams.
    A new stream joins only if it overlaps with every stream already chosen (streams_overlap):
    in a process that has made other streams before, freshly made ones may share a hardware queue.
    After a few candidates without luck, or when there is no memory to measure with, the next one
    is taken as it is."""
    if len(_pipeline_streams) < n:
        scratch = _overlap_scratch() if _pipeline_streams or n > 1 else None
        rejected = []  # kept alive until the choice is made, so that new candidates are new streams
        while len(_pipeline_streams) < n:
            candidate = torch.cuda.Stream()
            if (scratch is not None and len(rejected) < 6
                    and not all(streams_overlap(s, candidate, scratch) for s in _pipeline_streams)):
                rejected.append(candidate)
                continue
            _pipeline_streams.append(candidate)
        del scratch
    return _pipeline_streams[:n]


class BatchPipeline:
    """Runs seed batches through a ChunkTensorSampler with `inflight` batches on the GPU at any
    time, each on a stream of its own (what upstream leaves to the DataLoader's prefetching):

        for input_nodes, seeds, blocks, x in BatchPipeline(sampler, feats_ct)(seed_batches):
            ...                                   # on the caller's current stream

    Results come back in submission order, as ChunkTensorSampler.sample_blocks[_and_index] returns
    them.  Before a batch is handed out the caller's stream is made to wait for the batch's last
    kernels, and the batch's tensors are recorded on that stream, so they can be used there (and
    dropped) without further care.  With hand_over=False neither happens: the batch's last kernels
    may still be running on the stream it was submitted on, and whoever uses it elsewhere orders
    that stream behind it; a consumer that works on the batch's own stream needs nothing, and the
    allocator can reuse the batch's buffers as soon as they are dropped (measured on a 288 MB
    feature block per batch: 5 % more batches per second).
    By default all pipelines share pipeline_streams(inflight).
    Streams of one pipeline should sit on different hardware queues to overlap; the first
    four streams a process makes do.
    """

    def __init__(self, sampler, chunk_features=None, inflight=3, streams=None, hand_over=True,
                 gathers_in_turn=True, native_loop=True):
        self.hand_over = hand_over
        self.gathers_in_turn = gathers_in_turn
        self.native_loop = native_loop
        if inflight < 1:
            raise ValueError("inflight must be at least 1")
        self.sampler = sampler
        self.chunk_features = chunk_features
        self.streams = list(streams) if streams is not None else pipeline_streams(inflight)
        if not self.streams:
            raise ValueError("no streams to run on")

    def _hand_out(self, pending, done, consumer):
        out = pending.result()
        if not self.hand_over:
            return out
        # behind everything the batch has enqueued on its stream, including a gather that result()
        # may just have launched for a frontier that did not fit its capped buffer
        done.record(pending.stream)
        consumer.wait_event(done)
        tensors = [out[0]]
        for b in out[2]:
            tensors += [b.src_local, b.dst_local]
        if out[2]:
            tensors.append(out[2][-1].dst_ids)  # the seeds on the device (an upload, if they came from the host)
        if len(out) > 3:
            tensors.append(out[3])
        for t in tensors:  # frontiers and seeds are views of these or of the caller's own tensor
            if t.is_cuda:
                t.record_stream(consumer)
        return out

    def _native(self):
        """The extension's own loop for this pipeline: a worker thread of the extension begins the
        batches, so that Python pays one call to hand seeds in and one to take a batch out.
        Loops are kept with the sampler (starting a thread costs as much as half a batch) and
        shared by its pipelines over the same features, streams and settings; returns None
        while another iteration is using the one this pipeline would take."""
        smp = self.sampler
        key = (id(self.chunk_features), tuple(st.stream_id for st in self.streams), self.hand_over,
               self.gathers_in_turn, tuple(smp.fanouts), smp.replace, id(smp.chunk_probs), smp.seed)
        entry = smp._loops.get(key)
        if entry is None:
            triples = []
            for st in self.streams:
                triples += [st.stream_id, st.device_index, st.device_type]
            loop = torch.classes.dgs_classes.BatchLoop(
                smp.chunk_indptr, smp.chunk_indices, smp.chunk_probs, list(reversed(smp.fanouts)), smp.replace,
                self.chunk_features, triples, self.hand_over, self.gathers_in_turn,
                [] if smp.seed is None else [smp.seed])
            # (the features are kept with the entry so that their id stays theirs)
            entry = smp._loops[key] = {"loop": loop, "busy": False, "features": self.chunk_features}
        if entry["busy"]:
            return None
        return entry

    def _iterate_native(self, entry, seed_batches):
        loop = entry["loop"]
        n = len(self.streams)
        with_x = self.chunk_features is not None
        waiting = deque()
        pushed = 0
        seeded = self.sampler.seed

        def take():
            frontiers, srcs, dsts, x, seeds_dev = loop._CAPI_pop()
            blocks = ChunkTensorSampler._blocks(seeds_dev, frontiers, srcs, dsts)
            seed_nodes = waiting.popleft()
            return (frontiers[-1], seed_nodes, blocks, x) if with_x else (frontiers[-1], seed_nodes, blocks)

        entry["busy"] = True
        try:
            for seeds in seed_batches:
                # the first batch on each stream goes behind what the caller's stream holds now,
                # later ones only if their seeds are on the device (see the Python loop below)
                # (a sampler with its own generator numbers its batches here, in submission order)
                loop._CAPI_push(seeds, pushed < n, -1 if seeded is None else self.sampler._first_stream(None))
                pushed += 1
                waiting.append(seeds)
                if len(waiting) >= n:
                    yield take()
            while waiting:
                yield take()
        finally:
            while loop._CAPI_pending() > 0:  # an iteration that was left early: nothing stays behind in the loop
                try:
                    loop._CAPI_pop()
                except RuntimeError:
                    pass
            entry["busy"] = False

    def __call__(self, seed_batches):
        # (a second iteration that starts while one is under way cannot share the first one's
        # queue: it keeps the Python loop)
        if self.native_loop and self.sampler.fused:
            entry = self._native()
            if entry is not None:
                yield from self._iterate_native(entry, seed_batches)
                return
        consumer = torch.cuda.current_stream()
        n = len(self.streams)
        # Events are made once per process and reused (making one costs more than the stream wait
        # it serves, and a fresh set per iteration showed in short iterations).  A wait refers to
        # the record that precedes it, so reuse by later batches is safe; an iteration takes a
        # set of its own, so iterations that overlap do not mix.
        spare = _event_sets.setdefault(n, [])
        events = spare.pop() if spare else (
            [torch.cuda.Event() for _ in range(n)], [torch.cuda.Event() for _ in range(n)])
        seeds_ready, batch_done = events
        queue = deque()
        try:
            for i, seeds in enumerate(seed_batches):
                st = self.streams[i % n]
                # Seeds on the device may have been made just now on the caller's stream (a generator
                # that builds them lazily, or uploads them without blocking): the batch's stream waits
                # for that stream as it stands.  This also orders the batch behind everything else the
                # caller has enqueued there, so seeds that should overlap with the caller's work are
                # better passed as host tensors (the operator uploads them on the batch's own stream).
                # (nothing to wait for when the caller's stream has drained: a query costs a tenth
                # of what the event pair costs)
                if (i < n or (torch.is_tensor(seeds) and seeds.is_cuda)) and not consumer.query():
                    seeds_ready[i % n].record(consumer)
                    st.wait_event(seeds_ready[i % n])
                turn = self.gathers_in_turn and self.chunk_features is not None and n > 1
                with torch.cuda.stream(st):
                    pending = self.sampler.submit(None, seeds, self.chunk_features,
                                                  gather_after=batch_done[(i - 1) % n] if turn and i > 0 else None)
                    if self.hand_over or turn:
                        batch_done[i % n].record(st)
                queue.append((pending, batch_done[i % n]))
                if len(queue) >= n:
                    yield self._hand_out(*queue.popleft(), consumer)
            while queue:
                yield self._hand_out(*queue.popleft(), consumer)
        finally:
            spare.append(events)


class SeedLoader:
    """Stands where upstream's training loop has `dgl.dataloading.DataLoader(graph, train_idx, sampler,
    device='cuda', batch_size=..., shuffle=True, drop_last=False, num_workers=0, use_ddp=True,
    use_uva=True)` (oppo_bench/single_node/chunktensor.py:123-139), with the same leading arguments:

        for input_nodes, output_nodes, blocks in SeedLoader(graph, train_idx, sampler, batch_size=1024,
                                                            shuffle=True):

    cuts `indices` into batches of `batch_size` seed ids (a fresh random order per iteration with
    `shuffle`, the short last batch left out with `drop_last`) and yields what
    `graph_sampler.sample_blocks(graph, batch)` returns for each.  With `chunk_features` it yields a
    fourth element, `chunk_features._CAPI_index(input_nodes)`: the loop's next line upstream (:151).
    Upstream runs one batch at a time (`num_workers=0`); here a fused sampler's batches go through a
    BatchPipeline with `inflight` of them on the GPU (1: one at a time), and a sampler that cannot
    run fused (a fanout above 64) is called batch by batch.  `graph` is unused, as in the sampler.
    `device` moves the seed ids there first (upstream passes 'cuda': batches of device ids are
    ordered behind the caller's stream; host ids are uploaded by the operator on the batch's own
    stream).  `generator` is the torch.Generator of the shuffle (CPU).  The DataLoader options that
    only matter with several ranks or worker processes are accepted and change nothing here.
    """

    _INERT_OPTIONS = ("use_ddp", "ddp_seed", "use_uva", "use_prefetch_thread", "use_alternate_streams",
                      "pin_prefetcher", "persistent_workers")

    def __init__(self, graph, indices, graph_sampler, device=None, batch_size=1, shuffle=False, drop_last=False,
                 num_workers=0, chunk_features=None, inflight=3, generator=None, **options):
        unknown = sorted(set(options) - set(self._INERT_OPTIONS))
        if unknown:
            raise TypeError(f"SeedLoader: unknown option(s) {unknown}")
        if num_workers != 0:
            raise ValueError("SeedLoader: num_workers must be 0 (batches overlap on the GPU, not in worker processes)")
        if batch_size < 1 or inflight < 1:
            raise ValueError("SeedLoader: batch_size and inflight must be at least 1")
        indices = torch.as_tensor(indices)
        if indices.dim() != 1 or indices.dtype not in (torch.int32, torch.int64):
            raise ValueError("SeedLoader: indices must be a 1-D int32 or int64 tensor")
        self.indices = indices if device is None else indices.to(device)
        self.graph_sampler = graph_sampler
        self.chunk_features = chunk_features
        self.batch_size = int(batch_size)
        self.shuffle = bool(shuffle)
        self.drop_last = bool(drop_last)
        self.inflight = int(inflight)
        self.generator = generator

    def __len__(self):
        n = self.indices.numel()
        return n // self.batch_size if self.drop_last else -(-n // self.batch_size)

    def _batches(self):
        ids = self.indices
        if self.shuffle:
            ids = ids[torch.randperm(ids.numel(), generator=self.generator).to(ids.device)]
        return list(ids.split(self.batch_size))[:len(self)]

    def __iter__(self):
        smp, feats = self.graph_sampler, self.chunk_features
        batches = self._batches()
        if getattr(smp, "fused", False) and self.inflight > 1:
            yield from BatchPipeline(smp, feats, self.inflight)(batches)
            return
        for seeds in batches:
            if feats is None:
                yield smp.sample_blocks(None, seeds)
            else:
                yield smp.sample_blocks_and_index(None, seeds, feats)
