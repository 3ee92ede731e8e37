/* A trainer's data loop in plain C over libapt_hip.so: no Python, no torch.
 *
 * What the reference does in examples/train.py:84-94,139 with a dgl DataLoader,
 * MixedPSNeighborSampler and load_subtensor is done here through the epoch driver
 * of include/apt_amd.h: the program builds a small graph and feature table whose
 * contents are arithmetic in the node id, hands four slots on two streams to
 * apt_epoch_create, takes the batches of two epochs in order and checks each one
 * on the host (seeds first among the input nodes, every relabeled entry names the
 * sampled neighbour, every feature row is the row of its node, edge count = the
 * valid slots, and the last hop's block in COO, CSC and CSR says the same as its
 * fixed-stride form).  It prints one line a test can compare with what the Python
 * pipeline gets for the same seeds and keys:
 *     ok batches=<n> edges=<sampled edges> nodes=<input nodes> checksum=<sum of all input node ids>
 *
 * Built by apt_amd/build.py (gcc, C11); run by tests/test_gpu_c_abi.py.
 */
#include <hip/hip_runtime_api.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "apt_amd.h"

#define N 20000
#define DIM 16
#define BATCH 192
#define HOPS 2
#define SLOTS 4
#define STREAMS 2
#define BATCHES 9

#define HIP(call)                                                                         \
  do {                                                                                    \
    hipError_t e_ = (call);                                                               \
    if (e_ != hipSuccess) {                                                               \
      fprintf(stderr, "%s:%d: %s: %s\n", __FILE__, __LINE__, #call, hipGetErrorString(e_)); \
      exit(2);                                                                            \
    }                                                                                     \
  } while (0)
#define APT(call)                                                                  \
  do {                                                                             \
    int rc_ = (call);                                                              \
    if (rc_ != APT_OK) {                                                           \
      fprintf(stderr, "%s:%d: %s: [%d] %s\n", __FILE__, __LINE__, #call, rc_, apt_last_error()); \
      exit(3);                                                                     \
    }                                                                              \
  } while (0)
#define REQUIRE(cond, ...)            \
  do {                                \
    if (!(cond)) {                    \
      fprintf(stderr, "check failed: %s: ", #cond); \
      fprintf(stderr, __VA_ARGS__);   \
      fprintf(stderr, "\n");          \
      exit(4);                        \
    }                                 \
  } while (0)

static int64_t degree_of(int64_t v) { return 3 + v % 9; }
static int64_t neighbour_of(int64_t v, int64_t k) { return (v * 7 + k * 1301 + 1) % N; }

static void* dev_alloc(size_t bytes) {
  void* p = NULL;
  HIP(hipMalloc(&p, bytes ? bytes : 256));
  return p;
}

int main(void) {
  if (apt_abi_version() != APT_ABI_VERSION) {
    fprintf(stderr, "libapt_hip.so has ABI version %d, this program was built against %d\n", apt_abi_version(),
            APT_ABI_VERSION);
    return 1;
  }
  const int fanouts[HOPS] = {4, 3};

  /* the graph and the features, on the host, then in device memory */
  int64_t* indptr = malloc(sizeof(int64_t) * (N + 1));
  indptr[0] = 0;
  for (int64_t v = 0; v < N; ++v) indptr[v + 1] = indptr[v] + degree_of(v);
  const int64_t num_edges = indptr[N];
  int64_t* indices = malloc(sizeof(int64_t) * num_edges);
  for (int64_t v = 0; v < N; ++v)
    for (int64_t k = 0; k < degree_of(v); ++k) indices[indptr[v] + k] = neighbour_of(v, k);
  float* feats = malloc(sizeof(float) * N * DIM);
  for (int64_t i = 0; i < (int64_t)N * DIM; ++i) feats[i] = (float)i;   /* row v = v * DIM + 0 .. DIM - 1 */
  int64_t* d_indptr = dev_alloc(sizeof(int64_t) * (N + 1));
  int64_t* d_indices = dev_alloc(sizeof(int64_t) * num_edges);
  float* d_feats = dev_alloc(sizeof(float) * N * DIM);
  HIP(hipMemcpy(d_indptr, indptr, sizeof(int64_t) * (N + 1), hipMemcpyHostToDevice));
  HIP(hipMemcpy(d_indices, indices, sizeof(int64_t) * num_edges, hipMemcpyHostToDevice));
  HIP(hipMemcpy(d_feats, feats, sizeof(float) * N * DIM, hipMemcpyHostToDevice));

  apt_epoch_desc d;
  memset(&d, 0, sizeof d);
  d.graph.indptr = d_indptr;
  d.graph.indices = d_indices;
  d.graph.row_begin = 0;
  d.graph.num_rows = N;
  d.graph.num_total_nodes = N;
  d.store.local_table = d_feats;
  d.store.num_local_rows = N;
  d.store.local_dim = DIM;
  d.store.num_total_nodes = N;
  d.store.out_dim = DIM;
  d.store.elem_size = 4;
  d.batch = BATCH;
  d.num_hops = HOPS;
  for (int h = 0; h < HOPS; ++h) d.hop_fanouts[h] = fanouts[h];
  d.rank_table_len = N;
  d.num_slots = SLOTS;

  hipStream_t streams[STREAMS], consumer;
  for (int s = 0; s < STREAMS; ++s) HIP(hipStreamCreateWithFlags(&streams[s], hipStreamNonBlocking));
  HIP(hipStreamCreateWithFlags(&consumer, hipStreamNonBlocking));
  const size_t table_bytes = apt_rank_table_bytes(N);
  const size_t ws_bytes = apt_minibatch_workspace_bytes(BATCH, fanouts, HOPS);
  REQUIRE(table_bytes > 0 && ws_bytes > 0, "sizes out of range");
  void* tables[STREAMS];
  for (int s = 0; s < STREAMS; ++s) {   /* the slots of one stream share its table */
    tables[s] = dev_alloc(table_bytes);
    APT(apt_rank_table_init(tables[s], table_bytes, streams[s]));
  }
  int64_t cap[HOPS + 1];
  for (int h = 0; h <= HOPS; ++h) cap[h] = apt_minibatch_capacity(BATCH, fanouts, HOPS, h);
  for (int k = 0; k < SLOTS; ++k) {
    apt_batch_slot* s = &d.slots[k];
    s->stream = streams[k % STREAMS];
    s->rank_table = tables[k % STREAMS];
    s->nodes = dev_alloc(sizeof(int64_t) * cap[HOPS]);
    s->sizes = dev_alloc(sizeof(int64_t) * (HOPS + 2));
    for (int h = 0; h < HOPS; ++h) {
      s->neighbors[h] = dev_alloc(sizeof(int64_t) * cap[h] * fanouts[h]);
      s->relabeled[h] = dev_alloc(sizeof(int64_t) * cap[h] * fanouts[h]);
      s->counts[h] = dev_alloc(sizeof(int64_t) * cap[h]);
    }
    s->workspace = dev_alloc(ws_bytes);
    s->workspace_bytes = ws_bytes;
    APT(apt_minibatch_workspace_init(s->workspace, ws_bytes, streams[k % STREAMS]));
    s->features = dev_alloc(sizeof(float) * cap[HOPS] * DIM);
    s->miss_count = dev_alloc(sizeof(int64_t));
    HIP(hipMemset(s->miss_count, 0, sizeof(int64_t)));
    /* every hop's block also in COO + CSC + CSR */
    s->block_edges = dev_alloc(sizeof(int64_t) * HOPS);
    for (int h = 0; h < HOPS; ++h) {
      apt_block_buffers* b = &s->blocks[h];
      const int64_t slots = cap[h] * fanouts[h];
      b->coo_row = dev_alloc(sizeof(int64_t) * slots);
      b->coo_col = dev_alloc(sizeof(int64_t) * slots);
      b->csc_indptr = dev_alloc(sizeof(int64_t) * (cap[h] + 1));
      b->csr_indptr = dev_alloc(sizeof(int64_t) * (cap[h + 1] + 1));
      b->csr_indices = dev_alloc(sizeof(int64_t) * slots);
      b->csr_eids = dev_alloc(sizeof(int64_t) * slots);
      b->workspace_bytes = apt_block_workspace_bytes(cap[h], fanouts[h], cap[h + 1], 1);
      REQUIRE(b->workspace_bytes > 0, "block sizes out of range");
      b->workspace = dev_alloc(b->workspace_bytes);
    }
  }
  d.formats = 1;
  HIP(hipDeviceSynchronize());

  apt_epoch* ep = NULL;
  APT(apt_epoch_create(&d, &ep));

  int64_t* seeds = malloc(sizeof(int64_t) * BATCHES * BATCH);
  int64_t* d_seeds = dev_alloc(sizeof(int64_t) * BATCHES * BATCH);
  int64_t* h_nodes = malloc(sizeof(int64_t) * cap[HOPS]);
  int64_t* h_nbr = malloc(sizeof(int64_t) * cap[HOPS - 1] * fanouts[HOPS - 1]);
  int64_t* h_rel = malloc(sizeof(int64_t) * cap[HOPS - 1] * fanouts[HOPS - 1]);
  float* h_feat = malloc(sizeof(float) * cap[HOPS] * DIM);
  const int64_t last_slots = cap[HOPS - 1] * fanouts[HOPS - 1];
  int64_t* h_row = malloc(sizeof(int64_t) * last_slots);
  int64_t* h_col = malloc(sizeof(int64_t) * last_slots);
  int64_t* h_csc = malloc(sizeof(int64_t) * (cap[HOPS - 1] + 1));
  int64_t* h_csr = malloc(sizeof(int64_t) * (cap[HOPS] + 1));
  int64_t* h_csr_idx = malloc(sizeof(int64_t) * last_slots);
  int64_t* h_csr_eid = malloc(sizeof(int64_t) * last_slots);
  long long total_edges = 0, total_nodes = 0, checksum = 0;
  int batches_seen = 0;
  for (int epoch = 0; epoch < 2; ++epoch) {
    for (int64_t i = 0; i < (int64_t)BATCHES * BATCH; ++i) seeds[i] = (i * 97 + epoch * 31) % N;   /* distinct within a batch */
    HIP(hipMemcpy(d_seeds, seeds, sizeof(int64_t) * BATCHES * BATCH, hipMemcpyHostToDevice));
    APT(apt_epoch_begin(ep, d_seeds, BATCHES, 1000u * (uint64_t)(epoch + 1), NULL));
    for (int i = 0; i < BATCHES; ++i) {
      int slot = -1;
      int64_t sizes[2 * APT_MAX_HOPS + 2];
      APT(apt_epoch_next(ep, &slot, sizes, NULL));
      REQUIRE(slot == i % SLOTS, "batch %d came in slot %d", i, slot);
      const apt_batch_slot* s = &d.slots[slot];
      const int64_t n_in = sizes[HOPS], n_mid = sizes[HOPS - 1];
      REQUIRE(sizes[0] == BATCH && n_mid >= BATCH && n_in >= n_mid && n_in <= cap[HOPS], "sizes %lld %lld %lld",
              (long long)sizes[0], (long long)n_mid, (long long)n_in);
      /* the consumer reads the batch on its own stream, then hands the slot back */
      HIP(hipMemcpyAsync(h_nodes, s->nodes, sizeof(int64_t) * n_in, hipMemcpyDeviceToHost, consumer));
      HIP(hipMemcpyAsync(h_feat, s->features, sizeof(float) * n_in * DIM, hipMemcpyDeviceToHost, consumer));
      HIP(hipMemcpyAsync(h_nbr, s->neighbors[HOPS - 1], sizeof(int64_t) * n_mid * fanouts[HOPS - 1], hipMemcpyDeviceToHost, consumer));
      HIP(hipMemcpyAsync(h_rel, s->relabeled[HOPS - 1], sizeof(int64_t) * n_mid * fanouts[HOPS - 1], hipMemcpyDeviceToHost, consumer));
      const apt_block_buffers* b = &s->blocks[HOPS - 1];
      const int64_t block_edges = sizes[HOPS + 2 + HOPS - 1];   /* the blocks' edge counts follow the sizes */
      REQUIRE(block_edges >= 0 && block_edges <= n_mid * fanouts[HOPS - 1], "edge count %lld", (long long)block_edges);
      HIP(hipMemcpyAsync(h_row, b->coo_row, sizeof(int64_t) * block_edges, hipMemcpyDeviceToHost, consumer));
      HIP(hipMemcpyAsync(h_col, b->coo_col, sizeof(int64_t) * block_edges, hipMemcpyDeviceToHost, consumer));
      HIP(hipMemcpyAsync(h_csc, b->csc_indptr, sizeof(int64_t) * (n_mid + 1), hipMemcpyDeviceToHost, consumer));
      HIP(hipMemcpyAsync(h_csr, b->csr_indptr, sizeof(int64_t) * (n_in + 1), hipMemcpyDeviceToHost, consumer));
      HIP(hipMemcpyAsync(h_csr_idx, b->csr_indices, sizeof(int64_t) * block_edges, hipMemcpyDeviceToHost, consumer));
      HIP(hipMemcpyAsync(h_csr_eid, b->csr_eids, sizeof(int64_t) * block_edges, hipMemcpyDeviceToHost, consumer));
      APT(apt_epoch_release(ep, consumer));
      HIP(hipStreamSynchronize(consumer));
      for (int64_t k = 0; k < BATCH; ++k)
        REQUIRE(h_nodes[k] == seeds[(int64_t)i * BATCH + k], "input node %lld is not the seed", (long long)k);
      long long valid = 0;
      for (int64_t j = 0; j < n_mid * fanouts[HOPS - 1]; ++j) {
        if (h_nbr[j] < 0) {
          REQUIRE(h_rel[j] < 0, "padding relabeled to %lld", (long long)h_rel[j]);
          continue;
        }
        ++valid;
        REQUIRE(h_rel[j] >= 0 && h_rel[j] < n_in && h_nodes[h_rel[j]] == h_nbr[j], "slot %lld: relabeled %lld",
                (long long)j, (long long)h_rel[j]);
        /* a sampled neighbour is a neighbour */
        const int64_t v = h_nodes[j / fanouts[HOPS - 1]];
        int found = 0;
        for (int64_t k = 0; k < degree_of(v); ++k) found |= neighbour_of(v, k) == h_nbr[j];
        REQUIRE(found, "node %lld has no neighbour %lld", (long long)v, (long long)h_nbr[j]);
      }
      REQUIRE(valid <= sizes[HOPS + 1], "edge total %lld below the last hop's %lld", (long long)sizes[HOPS + 1], valid);
      /* COO = the valid slots in order; CSC offsets count them per destination */
      REQUIRE(valid == block_edges, "the block has %lld edges, its COO %lld", valid, (long long)block_edges);
      int64_t e = 0;
      for (int64_t j = 0; j < n_mid * fanouts[HOPS - 1]; ++j) {
        if (j % fanouts[HOPS - 1] == 0) REQUIRE(h_csc[j / fanouts[HOPS - 1]] == e, "csc_indptr[%lld]", (long long)(j / fanouts[HOPS - 1]));
        if (h_nbr[j] < 0) continue;
        REQUIRE(h_row[e] == h_rel[j] && h_col[e] == j / fanouts[HOPS - 1], "COO edge %lld", (long long)e);
        ++e;
      }
      REQUIRE(h_csc[n_mid] == block_edges, "csc_indptr ends at %lld", (long long)h_csc[n_mid]);
      /* CSR: the same edges grouped by source, a source's edges by increasing edge id */
      REQUIRE(h_csr[0] == 0 && h_csr[n_in] == block_edges, "csr_indptr spans %lld..%lld", (long long)h_csr[0], (long long)h_csr[n_in]);
      for (int64_t src = 0; src < n_in; ++src) {
        REQUIRE(h_csr[src] <= h_csr[src + 1], "csr_indptr decreases at %lld", (long long)src);
        for (int64_t q = h_csr[src]; q < h_csr[src + 1]; ++q) {
          const int64_t id = h_csr_eid[q];
          REQUIRE(id >= 0 && id < block_edges && h_row[id] == src && h_col[id] == h_csr_idx[q], "CSR entry %lld", (long long)q);
          REQUIRE(q == h_csr[src] || h_csr_eid[q - 1] < id, "CSR entry %lld out of order", (long long)q);
        }
      }
      for (int64_t k = 0; k < n_in; ++k) {
        checksum += h_nodes[k];
        for (int c = 0; c < DIM; ++c)
          REQUIRE(h_feat[k * DIM + c] == (float)(h_nodes[k] * DIM + c), "feature row %lld is not node %lld's",
                  (long long)k, (long long)h_nodes[k]);
      }
      total_edges += sizes[HOPS + 1];
      total_nodes += n_in;
      ++batches_seen;
    }
    APT(apt_epoch_end(ep));
  }
  int64_t misses = 0;
  for (int k = 0; k < SLOTS; ++k) {
    int64_t m = 0;
    HIP(hipMemcpy(&m, d.slots[k].miss_count, sizeof m, hipMemcpyDeviceToHost));
    misses += m;
  }
  REQUIRE(misses == 0, "%lld feature rows were reported missing", (long long)misses);
  APT(apt_epoch_destroy(ep));
  printf("ok batches=%d edges=%lld nodes=%lld checksum=%lld\n", batches_seen, total_edges, total_nodes, checksum);
  return 0;
}
