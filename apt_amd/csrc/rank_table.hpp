// The per-slot step of the rank-table relabel, shared by the sampling kernel
// (marking fused into sampling) and the stand-alone marking pass.
#pragma once

#include "common.hpp"

namespace apt {

// States of a relabeled[] slot before its compact id is known.  They are the
// 2^32 + 2 most negative values, and the bidding turns a (corrupt) neighbour id
// in that range into plain padding, so that no id a graph can hold is mistaken
// for a state; every other negative id is padding that passes through
// unchanged, as in the hash-table relabel.
constexpr int64_t kSlotLoser = INT64_MIN;      // another slot holds a smaller bid for the same node
constexpr int64_t kSlotOwner = INT64_MIN + 1;  // bid placed and, so far, the smallest for its node
// kSlotLoserSaw + s: like kSlotLoser, and slot s of the hop was seen holding a
// smaller bid for the node.  Slot s got kSlotOwner when it bid, so after the
// owners are placed it holds the node's id, unless a still smaller bid displaced
// it later (then it holds kSlotOwner until the lookup pass reaches it).
constexpr int64_t kSlotLoserSaw = INT64_MIN + 2;
constexpr int64_t kSlotStatesEnd = kSlotLoserSaw + (int64_t{1} << 32);

struct RankTable {
  uint32_t* entries;        // one per node: (epoch << payload bits) | id or bid
  int64_t len;
  const uint32_t* state;    // [0] epoch, [1] payload bits
  uint8_t* displaced;       // per slot of the current hop: set when a smaller bid took the node over
};

// What the sampling kernel needs to do the rank-table step for every id it has just loaded (the marking fused
// into sampling).
struct SampleMark {
  RankTable table;
  int64_t* relabeled;          // [rows * fanout]: receives the slot states / ids of rank_table_bid
  int first_hop;               // the frontier rows bid for their nodes too (with their row index)
  int64_t* outside = nullptr;  // optional, first hop: counts the frontier ids the table cannot hold
};

// Smallest entry value of the current batch.
__device__ __forceinline__ uint32_t table_base(const uint32_t* state) { return state[0] << state[1]; }

// The epoch state of a batch, read once per kernel: it does not change while a
// batch's kernels run, but the compiler cannot know that and would fetch it from
// memory again after every atomic (a dependent load on the path of every bid).
struct RankEpoch {
  uint32_t epoch, bits, base;   // base = epoch << bits, the smallest entry value of the batch
};
__device__ __forceinline__ RankEpoch rank_epoch(const uint32_t* state) {
  RankEpoch e;
  e.epoch = state[0];
  e.bits = state[1];
  e.base = e.epoch << e.bits;
  return e;
}

// Slot j (of ns * fanout) of a hop with ns frontier rows sampled node v.
//   v already in the batch (id < ns in the table)  -> its id, no atomic;
//   otherwise bid ns + j: the smallest bid owns the node.  A returning
//   atomicMin tells the bidder whether it is the smallest so far, and which
//   earlier bid it displaced; that slot is flagged, so after the kernel a slot
//   owns its node iff it is kSlotOwner and not flagged: no second look at the
//   table is needed.  (The value only ever decreases, and every decrease is an
//   atomicMin that returns the bid it replaces, so exactly the final minimum is
//   never flagged.)
// first_hop: the table holds seed indices, not ids, so hits cannot be resolved
// yet and ownership is decided by re-reading the table; no flags are kept.
// probe: read the entry before bidding (a plain read is cheaper than an atomic, and a third of a large hop's
// slots need no atomic after it).  A launch too small to be bound by the number of its atomics skips the read:
// there it is one more dependent round trip in a chain of them, and the returning atomic tells the same.
__device__ __forceinline__ int64_t rank_table_bid(const RankTable& t, const RankEpoch& ep, bool first_hop,
                                                  int64_t v, int64_t ns, int64_t j, bool probe = true) {
  const uint32_t tb = ep.base;
  if (v < 0) return v < kSlotStatesEnd ? -1 : v;  // padding; never one of the states above
  if (v >= t.len) return -1;  // an id the table cannot hold: treated as padding
  const uint32_t first_bid = tb + static_cast<uint32_t>(ns);
  const uint32_t bid = first_bid + static_cast<uint32_t>(j);
  // A stale read can only show a larger value than the table holds now, which
  // at worst causes a redundant atomic.
  const uint32_t cur = probe ? t.entries[v] : 0xFFFFFFFFu;
  if (first_hop) {
    if (cur > bid) atomicMin(&t.entries[v], bid);
    return kSlotOwner;
  }
  if (cur < first_bid) return static_cast<int64_t>(cur - tb);
  if (cur < bid) return kSlotLoserSaw + static_cast<int64_t>(cur - first_bid);
  const uint32_t old = atomicMin(&t.entries[v], bid);
  if (old < bid)
    return old < first_bid ? static_cast<int64_t>(old - tb) : kSlotLoserSaw + static_cast<int64_t>(old - first_bid);
  // old > bid: this slot is the smallest so far.  If old belongs to this batch it
  // is a bid of this hop (ids are below first_bid): that slot has been displaced.
  if ((old >> ep.bits) == ep.epoch) t.displaced[old - first_bid] = 1;
  return kSlotOwner;
}

// The pass that gives the slots that lost their race the winner's id, for all
// hops of a batch at once.  It depends on the placing of the last hop's owners
// and on nothing after it, and nothing but the caller's reading of relabeled[]
// depends on it, so it can run as a kernel of its own (mb_lookup_kernel) or
// ride along in the launch of the feature gather that follows the sampling
// (gather.hip): the gather is bound by bandwidth, this pass by a few dependent
// random reads.
constexpr int kLookupBlock = 256;
struct LookupParams {
  int num_hops;
  int64_t block_begin[APT_MAX_HOPS + 1];  // workgroup ranges per hop
  const int64_t* neighbors[APT_MAX_HOPS];
  int64_t* relabeled[APT_MAX_HOPS];
  const int64_t* ns_dev[APT_MAX_HOPS];
  int64_t ns_cap[APT_MAX_HOPS];
  int64_t fanout[APT_MAX_HOPS];
  const uint32_t* table;
  const uint32_t* state;
  int last_is_bid;  // the last hop's table entries are still bids (its ids are not written back)
};

// Work of workgroup `block` (of block_begin[num_hops]) of the pass; kLookupBlock threads.
__device__ __forceinline__ void lookup_block(const LookupParams& p, int64_t block) {
  int h = 0;
  while (h + 1 < p.num_hops && block >= p.block_begin[h + 1]) ++h;
  const int64_t ns = actual_count(p.ns_cap[h], p.ns_dev[h]);
  const int64_t nn = ns * p.fanout[h];
  const int64_t blocks = p.block_begin[h + 1] - p.block_begin[h];
  const uint32_t tb = table_base(p.state);
  const bool via_owner = p.last_is_bid && h == p.num_hops - 1;
  for (int64_t j = (block - p.block_begin[h]) * kLookupBlock + threadIdx.x; j < nn; j += blocks * kLookupBlock) {
    const int64_t r = p.relabeled[h][j];
    if (r >= kSlotStatesEnd) continue;  // an id, or padding (any other negative value)
    if (via_owner && r >= kSlotLoserSaw) {
      // the slot that was seen with a smaller bid holds the node's id by now, unless it was displaced itself
      const int64_t id = p.relabeled[h][r - kSlotLoserSaw];
      if (id >= 0) {
        p.relabeled[h][j] = id;
        continue;
      }
    }
    const int64_t e = p.table[p.neighbors[h][j]] - tb;
    // via_owner: e is the winning bid ns + slot; the winner's slot holds the id
    // (it is an owner, so its slot is final and never pending).
    p.relabeled[h][j] = via_owner ? p.relabeled[h][e - ns] : e;
  }
}

// What apt_pending_lookup holds.
struct PendingLookup {
  uint32_t magic;   // kPendingMagic when blocks and lp are valid
  uint32_t blocks;  // workgroups of the pass; 0: nothing to do
  LookupParams lp;
};
constexpr uint32_t kPendingMagic = 0x4C4B5550u;
static_assert(sizeof(PendingLookup) <= sizeof(apt_pending_lookup), "apt_pending_lookup is too small");

}  // namespace apt
