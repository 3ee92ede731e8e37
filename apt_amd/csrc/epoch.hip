// Epoch driver: the host side of a trainer's data loader, in C.
//
// The reference's trainer iterates a dgl DataLoader whose sampler is
// MixedPSNeighborSampler and then calls load_subtensor (examples/train.py:84-94,
// 139; python/npc/utils/utils.py:425): per batch that is a Python loop over the
// hops, two operator calls per hop, each with a stream synchronisation, and a
// third for the features.  Here a batch is enqueued by a worker thread of this
// library -- fused sampling + relabel, the gather (or, for a partitioned feature
// store, the bucketing of the requests and the gather of the rows present here),
// the blocks' COO / CSC / CSR where asked for, the copy of the batch's sizes to pinned host memory and the event that marks
// it complete -- on one of a few "slots" (a set of device buffers and a HIP
// stream each), so that several batches are in flight and the consumer's thread
// does nothing per batch but wait for the next one and say when it is done with
// it.  No device memory is allocated here: the slots' buffers come from the
// caller.
#include "common.hpp"

#include <chrono>
#include <condition_variable>
#include <cstring>
#include <deque>
#include <mutex>
#include <new>
#include <thread>

namespace apt {

void set_thread_launch_caps(int sample_blocks, int gather_blocks);  // lib.hip

// With four or more streams the batches' two large kernels are launched at half width each: a sampling kernel
// takes at most 512 workgroups of 512 threads and a gather at most 1024 of 256, half of the CUs' wave slots
// either way, so that one batch's gather (bound by bandwidth) and another's last-hop sampler (bound by random
// transactions) are resident together instead of taking turns at full width.  Measured on the 111 M-node graph
// with four streams: 0.151-0.157 against 0.160-0.163 ms per batch of 4096 seeds, 0.064 against 0.067 ms per batch
// of 1024; with two or three streams, or a batch alone (0.208-0.223 against 0.202 ms), full width is faster.
constexpr int kCoResidentStreams = 4;
constexpr int kCoResidentSampleBlocks = 512;
constexpr int kCoResidentGatherBlocks = 1024;

// int64 words of pinned memory per slot: the sizes, the request bucket sizes, the blocks' edge counts
constexpr int kPinnedReq = APT_MAX_HOPS + 2;
constexpr int kPinnedEdges = kPinnedReq + APT_MAX_BUCKETS;
constexpr int kPinnedPerSlot = kPinnedEdges + APT_MAX_HOPS;

// The batch's sizes (and request bucket sizes) go to pinned host memory by a one-wavefront kernel rather than a
// hipMemcpyAsync of 40 bytes: the stores stay on the stream's compute queue, with no hand-over to a copy engine
// and back between a batch and the next one on the stream.
__global__ void publish_sizes_kernel(const int64_t* __restrict__ sizes, int n, const int64_t* __restrict__ req,
                                     int r, const int64_t* __restrict__ edges, int e,
                                     int64_t* __restrict__ host_words) {
  const int t = threadIdx.x;
  if (t < n) host_words[t] = sizes[t];
  if (t < r) host_words[kPinnedReq + t] = req[t];
  if (t < e) host_words[kPinnedEdges + t] = edges[t];
}

struct EpochWork {
  int64_t batch;
  int slot;
  hipEvent_t after;  // the slot's stream waits for it first (may be NULL)
};

}  // namespace apt

struct apt_epoch {
  apt_epoch_desc d;
  int device = 0;
  std::thread worker;
  std::mutex mu;
  std::condition_variable cv_work, cv_done;
  std::deque<apt::EpochWork> queue;
  bool stop = false;
  bool busy = false;  // the worker is enqueueing a batch
  // the current epoch
  bool active = false;
  const int64_t* seeds = nullptr;
  int64_t num_batches = 0;
  uint64_t rng0 = 0;
  int64_t handed_out = 0;  // batches returned by apt_epoch_next so far
  int64_t enqueued = 0;    // batches [0, enqueued) are on their streams
  bool last_released = true;
  int error = 0;
  char error_text[512] = {0};
  hipEvent_t done[APT_MAX_SLOTS] = {};
  hipEvent_t released[APT_MAX_SLOTS] = {};
  int64_t* pinned = nullptr;      // host address of the pinned size words
  int64_t* pinned_dev = nullptr;  // the same memory as the GPU addresses it
  apt_pending_lookup pending[APT_MAX_SLOTS];
  // what the worker thread spent enqueueing (host time), since the handle was created
  double enqueue_seconds = 0.0;
  int64_t enqueued_total = 0;
  // what apt_epoch_next spent waiting: for the worker to have enqueued the batch, then for the GPU
  double wait_enqueue_seconds = 0.0, wait_gpu_seconds = 0.0, release_seconds = 0.0;
};

namespace apt {

static int enqueue_batch(apt_epoch* ep, const EpochWork& w) {
  const apt_epoch_desc& d = ep->d;
  const apt_batch_slot& s = d.slots[w.slot];
  hipStream_t st = static_cast<hipStream_t>(s.stream);
  const int H = d.num_hops;
  if (w.after != nullptr) APT_HIP(hipStreamWaitEvent(st, w.after, 0));
  const int64_t* seeds = ep->seeds + w.batch * d.batch;
  const uint64_t rng = ep->rng0 + static_cast<uint64_t>(w.batch);
  int64_t* const* counts = s.counts[0] != nullptr ? s.counts : nullptr;
  int rc;
  if (s.features != nullptr && d.has_requests == 0) {
    // the relabel's last pass rides in the gather's launch
    rc = apt_minibatch_sample_deferred(&d.graph, seeds, d.batch, d.hop_fanouts, H, d.replace, rng, nullptr,
                                       s.rank_table, d.rank_table_len, s.nodes, s.neighbors, s.relabeled, counts,
                                       s.sizes, s.workspace, s.workspace_bytes, st, &ep->pending[w.slot]);
    if (rc != APT_OK) return rc;
    const int64_t cap = apt_minibatch_capacity(d.batch, d.hop_fanouts, H, H);
    rc = apt_gather_rows_with_lookup(&d.store, s.nodes, cap, s.sizes + H, s.features, s.miss_count,
                                     &ep->pending[w.slot], st);
    if (rc != APT_OK) return rc;
  } else {
    rc = apt_minibatch_sample(&d.graph, seeds, d.batch, d.hop_fanouts, H, d.replace, rng, nullptr, s.rank_table,
                              d.rank_table_len, s.nodes, s.neighbors, s.relabeled, counts, s.sizes, s.workspace,
                              s.workspace_bytes, st);
    if (rc != APT_OK) return rc;
    if (d.has_requests != 0) {
      const int64_t cap = apt_minibatch_capacity(d.batch, d.hop_fanouts, H, H);
      rc = apt_cluster_reqs(s.nodes, cap, s.sizes + H, d.request_pos_map, d.request_num_total_nodes,
                            d.remote_worker_map, d.min_vids, d.world_size, d.num_remote_workers, s.request_sizes,
                            s.request_offsets, s.request_ids, s.request_perm, s.request_workspace,
                            s.request_workspace_bytes, st);
      if (rc != APT_OK) return rc;
      if (s.features != nullptr) {
        // rows that are here: features[k] belongs to request_ids[k], k < request_sizes[0]
        rc = apt_gather_rows(&d.store, s.request_ids, cap, s.request_sizes, s.features, s.miss_count, st);
        if (rc != APT_OK) return rc;
      }
    }
  }
  if (d.formats != 0) {
    // the blocks in the formats a layer consumes, after the relabel's last pass (which may have ridden in the gather)
    for (int h = 0; h < H; ++h) {
      const apt_block_buffers& b = s.blocks[h];
      rc = apt_block_formats(s.relabeled[h], apt_minibatch_capacity(d.batch, d.hop_fanouts, H, h), s.sizes + h,
                             d.hop_fanouts[h], apt_minibatch_capacity(d.batch, d.hop_fanouts, H, h + 1), b.coo_row,
                             b.coo_col, b.csc_indptr, s.block_edges + h, b.csr_indptr, b.csr_indices, b.csr_eids,
                             b.workspace, b.workspace_bytes, st);
      if (rc != APT_OK) return rc;
    }
  }
  static_assert(APT_MAX_HOPS + 2 <= 64 && APT_MAX_BUCKETS <= 64, "publish_sizes_kernel runs one wavefront");
  hipLaunchKernelGGL(publish_sizes_kernel, dim3(1), dim3(64), 0, st, s.sizes, H + 2,
                     d.has_requests != 0 ? s.request_sizes : nullptr, d.has_requests != 0 ? d.num_remote_workers : 0,
                     d.formats != 0 ? s.block_edges : nullptr, d.formats != 0 ? H : 0,
                     ep->pinned_dev + static_cast<size_t>(w.slot) * kPinnedPerSlot);
  APT_LAUNCH_CHECK("publish_sizes_kernel");
  APT_HIP(hipEventRecord(ep->done[w.slot], st));
  return APT_OK;
}

static void worker_main(apt_epoch* ep) {
  (void)hipSetDevice(ep->device);
  int streams = 0;
  for (int k = 0; k < ep->d.num_slots; ++k) {
    bool seen = false;
    for (int j = 0; j < k; ++j) seen |= ep->d.slots[j].stream == ep->d.slots[k].stream;
    streams += seen ? 0 : 1;
  }
  if (streams >= kCoResidentStreams) set_thread_launch_caps(kCoResidentSampleBlocks, kCoResidentGatherBlocks);
  for (;;) {
    EpochWork w;
    bool failed;  // an earlier batch (or a release) has failed: nothing more is enqueued
    {
      std::unique_lock<std::mutex> lk(ep->mu);
      ep->cv_work.wait(lk, [ep] { return ep->stop || !ep->queue.empty(); });
      if (ep->queue.empty()) return;  // stop
      w = ep->queue.front();
      ep->queue.pop_front();
      ep->busy = true;
      failed = ep->error != 0;
    }
    const auto t0 = std::chrono::steady_clock::now();
    const int rc = failed ? APT_OK : enqueue_batch(ep, w);
    const double dt = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
    {
      std::lock_guard<std::mutex> lk(ep->mu);
      ep->enqueue_seconds += dt;
      ep->enqueued_total += 1;
      if (rc != APT_OK && ep->error == 0) {
        ep->error = rc;
        std::strncpy(ep->error_text, apt_last_error(), sizeof(ep->error_text) - 1);
      }
      ep->enqueued = w.batch + 1;
      ep->busy = false;
    }
    ep->cv_done.notify_all();
  }
}

static int check_desc(const apt_epoch_desc* d) {
  APT_REQUIRE(d != nullptr, APT_EINVAL, "apt_epoch_create: desc is NULL");
  APT_REQUIRE(d->batch > 0, APT_EINVAL, "apt_epoch_create: batch %lld must be > 0", (long long)d->batch);
  APT_REQUIRE(d->num_hops >= 1 && d->num_hops <= APT_MAX_HOPS, APT_ELIMIT, "apt_epoch_create: num_hops %d outside [1, %d]",
              d->num_hops, APT_MAX_HOPS);
  APT_REQUIRE(d->num_slots >= 1 && d->num_slots <= APT_MAX_SLOTS, APT_ELIMIT,
              "apt_epoch_create: num_slots %d outside [1, %d]", d->num_slots, APT_MAX_SLOTS);
  APT_REQUIRE(apt_minibatch_capacity(d->batch, d->hop_fanouts, d->num_hops, d->num_hops) > 0, APT_ELIMIT,
              "apt_epoch_create: unsupported batch / fanouts");
  const size_t need = apt_minibatch_workspace_bytes(d->batch, d->hop_fanouts, d->num_hops);
  if (d->has_requests != 0) {
    APT_REQUIRE(d->request_pos_map != nullptr && d->remote_worker_map != nullptr && d->min_vids != nullptr &&
                    d->world_size >= 1 && d->num_remote_workers >= 1 && d->num_remote_workers <= APT_MAX_BUCKETS,
                APT_EINVAL, "apt_epoch_create: incomplete request description");
  }
  for (int k = 0; k < d->num_slots; ++k) {
    const apt_batch_slot& s = d->slots[k];
    APT_REQUIRE(s.nodes != nullptr && s.sizes != nullptr && s.rank_table != nullptr && s.workspace != nullptr,
                APT_EINVAL, "apt_epoch_create: slot %d: nodes / sizes / rank_table / workspace is NULL", k);
    APT_REQUIRE(s.workspace_bytes >= need, APT_EWORKSPACE, "apt_epoch_create: slot %d: workspace of %zu bytes, %zu needed",
                k, s.workspace_bytes, need);
    for (int h = 0; h < d->num_hops; ++h)
      APT_REQUIRE(s.neighbors[h] != nullptr && s.relabeled[h] != nullptr, APT_EINVAL,
                  "apt_epoch_create: slot %d: neighbors[%d] / relabeled[%d] is NULL", k, h, h);
    if (d->has_requests != 0)
      APT_REQUIRE(s.request_sizes != nullptr && s.request_ids != nullptr && s.request_perm != nullptr &&
                      s.request_workspace != nullptr,
                  APT_EINVAL, "apt_epoch_create: slot %d: request buffers missing", k);
    if (d->formats != 0) {
      APT_REQUIRE(s.block_edges != nullptr, APT_EINVAL, "apt_epoch_create: slot %d: block_edges is NULL", k);
      for (int h = 0; h < d->num_hops; ++h) {
        const apt_block_buffers& b = s.blocks[h];
        APT_REQUIRE(b.coo_row != nullptr && b.coo_col != nullptr && b.csc_indptr != nullptr && b.workspace != nullptr,
                    APT_EINVAL, "apt_epoch_create: slot %d: block buffers of hop %d missing", k, h);
        APT_REQUIRE((b.csr_indptr == nullptr) == (b.csr_indices == nullptr) && (b.csr_indptr == nullptr) == (b.csr_eids == nullptr),
                    APT_EINVAL, "apt_epoch_create: slot %d: hop %d: all three CSR buffers or none", k, h);
        const size_t want = apt_block_workspace_bytes(apt_minibatch_capacity(d->batch, d->hop_fanouts, d->num_hops, h),
                                                      d->hop_fanouts[h],
                                                      apt_minibatch_capacity(d->batch, d->hop_fanouts, d->num_hops, h + 1),
                                                      b.csr_indptr != nullptr);
        APT_REQUIRE(b.workspace_bytes >= want, APT_EWORKSPACE,
                    "apt_epoch_create: slot %d: hop %d: block workspace of %zu bytes, %zu needed", k, h, b.workspace_bytes,
                    want);
      }
    }
  }
  return APT_OK;
}

}  // namespace apt

extern "C" int apt_epoch_create(const apt_epoch_desc* desc, apt_epoch** out) {
  using namespace apt;
  APT_REQUIRE(out != nullptr, APT_EINVAL, "apt_epoch_create: out is NULL");
  *out = nullptr;
  if (const int rc = check_desc(desc)) return rc;
  apt_epoch* ep = new (std::nothrow) apt_epoch();
  APT_REQUIRE(ep != nullptr, APT_EINVAL, "apt_epoch_create: out of host memory");
  ep->d = *desc;
  auto fail_create = [ep](int code) {
    for (int k = 0; k < APT_MAX_SLOTS; ++k) {
      if (ep->done[k] != nullptr) (void)hipEventDestroy(ep->done[k]);
      if (ep->released[k] != nullptr) (void)hipEventDestroy(ep->released[k]);
    }
    if (ep->pinned != nullptr) (void)hipHostFree(ep->pinned);
    delete ep;
    return code;
  };
  if (hipGetDevice(&ep->device) != hipSuccess) return fail_create(fail(APT_EHIP, "apt_epoch_create: hipGetDevice failed"));
  for (int k = 0; k < ep->d.num_slots; ++k) {
    // done[k] makes a kernel's stores to host memory visible to the host that waits for it
    if (hipEventCreateWithFlags(&ep->done[k], hipEventDisableTiming | hipEventReleaseToSystem) != hipSuccess ||
        hipEventCreateWithFlags(&ep->released[k], hipEventDisableTiming) != hipSuccess)
      return fail_create(fail(APT_EHIP, "apt_epoch_create: hipEventCreate failed"));
  }
  if (hipHostMalloc(reinterpret_cast<void**>(&ep->pinned),
                    sizeof(int64_t) * kPinnedPerSlot * static_cast<size_t>(ep->d.num_slots),
                    hipHostMallocMapped | hipHostMallocCoherent) != hipSuccess ||
      hipHostGetDevicePointer(reinterpret_cast<void**>(&ep->pinned_dev), ep->pinned, 0) != hipSuccess)
    return fail_create(fail(APT_EHIP, "apt_epoch_create: pinned, device-visible host memory for the sizes is not available"));
  std::memset(ep->pinned, 0, sizeof(int64_t) * kPinnedPerSlot * static_cast<size_t>(ep->d.num_slots));
  ep->worker = std::thread(worker_main, ep);
  *out = ep;
  return APT_OK;
}

// Ends the current epoch (if any): batches not yet on a stream are dropped, the
// one being enqueued is waited for, and the slots' streams are synchronised, so
// that the caller may reuse or free every buffer afterwards.
extern "C" int apt_epoch_end(apt_epoch* ep) {
  using namespace apt;
  APT_REQUIRE(ep != nullptr, APT_EINVAL, "apt_epoch_end: epoch is NULL");
  {
    std::unique_lock<std::mutex> lk(ep->mu);
    ep->queue.clear();
    ep->cv_done.wait(lk, [ep] { return !ep->busy; });
    ep->active = false;
  }
  for (int k = 0; k < ep->d.num_slots; ++k)
    APT_HIP(hipStreamSynchronize(static_cast<hipStream_t>(ep->d.slots[k].stream)));
  return APT_OK;
}

extern "C" int apt_epoch_destroy(apt_epoch* ep) {
  if (ep == nullptr) return APT_OK;
  const int rc = apt_epoch_end(ep);
  {
    std::lock_guard<std::mutex> lk(ep->mu);
    ep->stop = true;
  }
  ep->cv_work.notify_all();
  if (ep->worker.joinable()) ep->worker.join();
  for (int k = 0; k < ep->d.num_slots; ++k) {
    (void)hipEventDestroy(ep->done[k]);
    (void)hipEventDestroy(ep->released[k]);
  }
  (void)hipHostFree(ep->pinned);
  delete ep;
  return rc;
}

extern "C" int apt_epoch_begin(apt_epoch* ep, const int64_t* seeds, int64_t num_batches, uint64_t rng_seed0,
                               void* ready_event) {
  using namespace apt;
  APT_REQUIRE(ep != nullptr, APT_EINVAL, "apt_epoch_begin: epoch is NULL");
  APT_REQUIRE(num_batches >= 0 && (seeds != nullptr || num_batches == 0), APT_EINVAL,
              "apt_epoch_begin: seeds is NULL or num_batches < 0");
  if (ep->active)
    if (const int rc = apt_epoch_end(ep)) return rc;
  std::lock_guard<std::mutex> lk(ep->mu);
  ep->seeds = seeds;
  ep->num_batches = num_batches;
  ep->rng0 = rng_seed0;
  ep->handed_out = 0;
  ep->enqueued = 0;
  ep->last_released = true;
  ep->error = 0;
  ep->error_text[0] = 0;
  ep->active = true;
  const int64_t first = std::min<int64_t>(num_batches, ep->d.num_slots);
  for (int64_t i = 0; i < first; ++i)
    ep->queue.push_back(EpochWork{i, static_cast<int>(i), static_cast<hipEvent_t>(ready_event)});
  ep->cv_work.notify_all();
  return APT_OK;
}

extern "C" int apt_epoch_next(apt_epoch* ep, int* slot, int64_t* sizes_host, int64_t* request_sizes_host) {
  using namespace apt;
  APT_REQUIRE(ep != nullptr && slot != nullptr && sizes_host != nullptr, APT_EINVAL,
              "apt_epoch_next: epoch / slot / sizes_host is NULL");
  int64_t i;
  {
    std::unique_lock<std::mutex> lk(ep->mu);
    APT_REQUIRE(ep->active, APT_EINVAL, "apt_epoch_next: no epoch has been begun");
    APT_REQUIRE(ep->handed_out < ep->num_batches, APT_EINVAL, "apt_epoch_next: the epoch has no batch left");
    APT_REQUIRE(ep->last_released, APT_EINVAL, "apt_epoch_next: the previous batch has not been released");
    i = ep->handed_out;
    const auto t0 = std::chrono::steady_clock::now();
    ep->cv_done.wait(lk, [ep, i] { return ep->enqueued > i || ep->error != 0; });
    ep->wait_enqueue_seconds += std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
    if (ep->error != 0) return fail(ep->error, "apt_epoch_next: batch could not be enqueued: %s", ep->error_text);
  }
  const int k = static_cast<int>(i % ep->d.num_slots);
  const auto t1 = std::chrono::steady_clock::now();
  APT_HIP(hipEventSynchronize(ep->done[k]));
  const double gpu_wait = std::chrono::duration<double>(std::chrono::steady_clock::now() - t1).count();
  const int64_t* pin = ep->pinned + static_cast<size_t>(k) * kPinnedPerSlot;
  for (int j = 0; j < ep->d.num_hops + 2; ++j) sizes_host[j] = pin[j];
  if (ep->d.formats != 0)
    for (int j = 0; j < ep->d.num_hops; ++j) sizes_host[ep->d.num_hops + 2 + j] = pin[kPinnedEdges + j];
  if (request_sizes_host != nullptr && ep->d.has_requests != 0)
    for (int j = 0; j < ep->d.num_remote_workers; ++j) request_sizes_host[j] = pin[kPinnedReq + j];
  {
    std::lock_guard<std::mutex> lk(ep->mu);
    ep->handed_out = i + 1;
    ep->last_released = false;
    ep->wait_gpu_seconds += gpu_wait;
  }
  *slot = k;
  return APT_OK;
}

extern "C" int apt_epoch_release(apt_epoch* ep, void* consumer_stream) {
  using namespace apt;
  APT_REQUIRE(ep != nullptr, APT_EINVAL, "apt_epoch_release: epoch is NULL");
  std::unique_lock<std::mutex> lk(ep->mu);
  APT_REQUIRE(ep->active && !ep->last_released, APT_EINVAL, "apt_epoch_release: no batch is held");
  ep->last_released = true;
  const int64_t i = ep->handed_out - 1;
  const int64_t next = i + ep->d.num_slots;
  if (next >= ep->num_batches) return APT_OK;
  const int k = static_cast<int>(i % ep->d.num_slots);
  lk.unlock();
  // Whatever the consumer enqueued on its stream for batch i runs before the slot's buffers are reused.  When
  // that stream has nothing pending there is nothing to wait for, and no event is recorded: a marker in the
  // consumer's stream may share a hardware queue with one of the slots' streams (there are few hardware queues)
  // and would then complete only after that stream's queued batches, stalling the slot for no reason.
  hipEvent_t after = nullptr;
  const auto t0 = std::chrono::steady_clock::now();
  hipError_t err = hipStreamQuery(static_cast<hipStream_t>(consumer_stream));
  if (err == hipErrorNotReady) {
    err = hipEventRecord(ep->released[k], static_cast<hipStream_t>(consumer_stream));
    after = ep->released[k];
  }
  lk.lock();
  ep->release_seconds += std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
  if (err != hipSuccess) {
    // the slot cannot be handed back: the epoch ends here, and apt_epoch_next says why instead of waiting
    const int rc = fail(APT_EHIP, "apt_epoch_release: the consumer's stream: %s", hipGetErrorString(err));
    if (ep->error == 0) {
      ep->error = rc;
      std::strncpy(ep->error_text, apt_last_error(), sizeof(ep->error_text) - 1);
    }
    ep->cv_done.notify_all();
    return rc;
  }
  if (ep->active) {
    ep->queue.push_back(EpochWork{next, k, after});
    ep->cv_work.notify_all();
  }
  return APT_OK;
}

extern "C" int apt_epoch_host_cost(apt_epoch* ep, apt_epoch_cost* cost) {
  using namespace apt;
  APT_REQUIRE(ep != nullptr && cost != nullptr, APT_EINVAL, "apt_epoch_host_cost: a pointer is NULL");
  std::lock_guard<std::mutex> lk(ep->mu);
  cost->batches = ep->enqueued_total;
  cost->enqueue_seconds = ep->enqueue_seconds;
  cost->wait_enqueue_seconds = ep->wait_enqueue_seconds;
  cost->wait_gpu_seconds = ep->wait_gpu_seconds;
  cost->release_seconds = ep->release_seconds;
  return APT_OK;
}
