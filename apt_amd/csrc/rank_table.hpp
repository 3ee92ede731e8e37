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
__device__ __forceinline__ int64_t rank_table_bid(const RankTable& t, const RankEpoch& ep, bool first_hop,
                                                  int64_t v, int64_t ns, int64_t j) {
  const uint32_t tb = ep.base;
  if (v < 0) return v < kSlotStatesEnd ? -1 : v;  // padding; never one of the states above
  if (v >= t.len) return -1;  // an id the table cannot hold: treated as padding
  const uint32_t first_bid = tb + static_cast<uint32_t>(ns);
  const uint32_t bid = first_bid + static_cast<uint32_t>(j);
  // A stale read can only show a larger value than the table holds now, which
  // at worst causes a redundant atomic.
  const uint32_t cur = t.entries[v];
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

}  // namespace apt
