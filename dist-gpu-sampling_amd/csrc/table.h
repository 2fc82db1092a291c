// Device-side open-addressing tables for unique/relabel (linear probing, capacity 2^m).
//
// A table maps a node id to the smallest position at which it occurs in the mapping
// list.  unique.hip later overwrites that field with the id's rank (set_value); the
// multi-hop pipeline keeps positions and learns from insert_min() whether a position
// is, so far, the smallest of its id and which position it displaced.
//   packed   one 64-bit word per slot: id in the high half, position/rank in the low
//            half (ids must be < 2^32 - 1); insertion is a single 64-bit atomic;
//   split    id array + uint32 value array (any 64-bit id >= 0).
// Slots only ever change from empty to a key, and positions only decrease, so a plain
// (possibly stale) load is a safe first look before the atomic.
#ifndef DGS_CSRC_TABLE_H_
#define DGS_CSRC_TABLE_H_

#include "common.h"

namespace dgs {

__device__ __forceinline__ uint32_t hash_id(uint64_t k) {
  uint32_t h = uint32_t(k) ^ (uint32_t(k >> 32) * 0x9E3779B1u);
  h ^= h >> 16; h *= 0x85EBCA6Bu;
  h ^= h >> 13; h *= 0xC2B2AE35u;
  h ^= h >> 16;
  return h;
}

template <typename IdT> struct AtomicWord;
template <> struct AtomicWord<int64_t> { using type = unsigned long long; };
template <> struct AtomicWord<int32_t> { using type = unsigned int; };

constexpr uint32_t kNoPosition = 0xffffffffu;

template <typename IdT, bool PACKED> struct Table;

template <typename IdT>
struct Table<IdT, true> {
  unsigned long long* slots;
  uint32_t mask;
  static constexpr unsigned long long kEmpty = ~0ull;
  static constexpr size_t kSlotBytes = 8;

  __host__ __device__ Table(void* base, uint32_t capacity)
      : slots(static_cast<unsigned long long*>(base)), mask(capacity - 1) {}

  // ids the table can hold: 0 .. 2^32 - 2 (the all-ones word marks an empty slot)
  __device__ __forceinline__ bool holds(IdT key) const { return uint64_t(int64_t(key)) < 0xffffffffull; }

  __device__ __forceinline__ uint32_t insert(IdT key, uint32_t idx) const {
    const unsigned long long packed = (static_cast<unsigned long long>(uint32_t(key)) << 32) | idx;
    uint32_t pos = hash_id(uint32_t(key)) & mask;
    for (;;) {
      unsigned long long cur = slots[pos];
      if (cur == kEmpty) {
        cur = atomicCAS(slots + pos, kEmpty, packed);
        if (cur == kEmpty) return pos;
      }
      if (uint32_t(cur >> 32) == uint32_t(key)) {
        if (uint32_t(cur) > idx) atomicMin(slots + pos, packed);
        return pos;
      }
      pos = (pos + 1) & mask;
    }
  }
  // Same, reporting whether idx became the smallest position of its key (*first) and, if it
  // replaced a larger one, which (*displaced, else kNoPosition).
  __device__ __forceinline__ uint32_t insert_min(IdT key, uint32_t idx, bool* first, uint32_t* displaced,
                                                 bool /*look_first*/ = true) const {
    const unsigned long long packed = (static_cast<unsigned long long>(uint32_t(key)) << 32) | idx;
    uint32_t pos = hash_id(uint32_t(key)) & mask;
    *displaced = kNoPosition;
    for (;;) {
      unsigned long long cur = slots[pos];
      if (cur == kEmpty) {
        cur = atomicCAS(slots + pos, kEmpty, packed);
        if (cur == kEmpty) { *first = true; return pos; }
      }
      if (uint32_t(cur >> 32) == uint32_t(key)) {
        const unsigned long long old = atomicMin(slots + pos, packed);
        *first = old > packed;
        if (*first) *displaced = uint32_t(old);
        return pos;
      }
      pos = (pos + 1) & mask;
    }
  }
  __device__ __forceinline__ uint32_t value(uint32_t slot) const { return uint32_t(slots[slot]); }
  __device__ __forceinline__ IdT key(uint32_t slot) const { return IdT(uint32_t(slots[slot] >> 32)); }
  __device__ __forceinline__ void set_value(uint32_t slot, uint32_t v) const {
    reinterpret_cast<uint32_t*>(slots)[2 * size_t(slot)] = v;  // low half (little endian)
  }
  // slot of `key`, or mask + 1 when absent
  __device__ __forceinline__ uint32_t find(IdT key) const {
    uint32_t pos = hash_id(uint32_t(key)) & mask;
    for (;;) {
      const unsigned long long cur = slots[pos];
      if (cur == kEmpty) return mask + 1;
      if (uint32_t(cur >> 32) == uint32_t(key)) return pos;
      pos = (pos + 1) & mask;
    }
  }
};

template <typename IdT>
struct Table<IdT, false> {
  IdT* keys;
  uint32_t* vals;
  uint32_t mask;
  static constexpr size_t kSlotBytes = sizeof(IdT) + 4;

  // keys first, values right behind them (one contiguous region to clear)
  __host__ __device__ Table(void* base, uint32_t capacity)
      : keys(static_cast<IdT*>(base)),
        vals(reinterpret_cast<uint32_t*>(static_cast<char*>(base) + size_t(capacity) * sizeof(IdT))),
        mask(capacity - 1) {}

  // ids the table can hold: every id >= 0 (-1 marks an empty slot)
  __device__ __forceinline__ bool holds(IdT key) const { return key >= 0; }

  __device__ __forceinline__ uint32_t insert(IdT key, uint32_t idx) const {
    using W = typename AtomicWord<IdT>::type;
    uint32_t pos = hash_id(uint64_t(int64_t(key))) & mask;
    for (;;) {
      IdT cur = keys[pos];
      if (cur == IdT(-1)) cur = IdT(atomicCAS(reinterpret_cast<W*>(keys + pos), W(IdT(-1)), W(key)));
      if (cur == IdT(-1) || cur == key) break;
      pos = (pos + 1) & mask;
    }
    atomicMin(vals + pos, idx);
    return pos;
  }
  __device__ __forceinline__ uint32_t insert_min(IdT key, uint32_t idx, bool* first, uint32_t* displaced,
                                                 bool /*look_first*/ = true) const {
    using W = typename AtomicWord<IdT>::type;
    uint32_t pos = hash_id(uint64_t(int64_t(key))) & mask;
    for (;;) {
      IdT cur = keys[pos];
      if (cur == IdT(-1)) cur = IdT(atomicCAS(reinterpret_cast<W*>(keys + pos), W(IdT(-1)), W(key)));
      if (cur == IdT(-1) || cur == key) break;
      pos = (pos + 1) & mask;
    }
    const uint32_t old = atomicMin(vals + pos, idx);
    *first = old > idx;
    *displaced = (*first && old != 0xffffffffu) ? old : kNoPosition;
    return pos;
  }
  __device__ __forceinline__ uint32_t value(uint32_t slot) const { return vals[slot]; }
  __device__ __forceinline__ IdT key(uint32_t slot) const { return keys[slot]; }
  __device__ __forceinline__ void set_value(uint32_t slot, uint32_t v) const { vals[slot] = v; }
  __device__ __forceinline__ uint32_t find(IdT key) const {
    uint32_t pos = hash_id(uint64_t(int64_t(key))) & mask;
    for (;;) {
      const IdT cur = keys[pos];
      if (cur == key) return pos;
      if (cur == IdT(-1)) return mask + 1;
      pos = (pos + 1) & mask;
    }
  }
};

// Direct-address table over all node ids (ids < 2^32 - 1): one 64-bit entry per node,
// high half = a tag that DEcreases from one use of the table to the next, low half =
// position/rank.  Entries of earlier uses carry a larger tag, so atomicMin treats them as
// empty and the array never needs clearing between uses (fill it with 0xFF bytes once).
// The "slot" of an id is the id itself.
template <typename IdT>
struct DirectTable {
  unsigned long long* entries;
  uint32_t tag;  // ~epoch
  uint32_t n;    // entries: one per node
  static constexpr uint32_t kNoSlot = 0xffffffffu;

  __host__ __device__ DirectTable(void* base, uint32_t epoch, uint32_t n_nodes)
      : entries(static_cast<unsigned long long*>(base)), tag(~epoch), n(n_nodes) {}

  // ids the table has an entry for; everything else must be kept away from insert_min
  __device__ __forceinline__ bool holds(IdT key) const { return uint64_t(int64_t(key)) < uint64_t(n); }

  // `look_first`: read the entry before the atomic.  A value already below v (a stale read can
  // only be larger than the truth) settles the matter without an atomic, which is what keeps
  // popular ids from serialising thousands of atomics on one address; on ids that are mostly
  // new the extra read is pure cost.  The result is the same either way.
  __device__ __forceinline__ uint32_t insert_min(IdT key, uint32_t idx, bool* first, uint32_t* displaced,
                                                 bool look_first = true) const {
    const unsigned long long v = (static_cast<unsigned long long>(tag) << 32) | idx;
    unsigned long long* e = entries + uint32_t(key);
    if (look_first && *e < v) { *first = false; *displaced = kNoPosition; return uint32_t(key); }
    const unsigned long long old = atomicMin(e, v);
    *first = old > v;
    // an entry of this use that was larger: that position is no longer its id's smallest
    *displaced = (*first && uint32_t(old >> 32) == tag) ? uint32_t(old) : kNoPosition;
    return uint32_t(key);
  }
  __device__ __forceinline__ uint32_t value(uint32_t slot) const { return uint32_t(entries[slot]); }
  __device__ __forceinline__ IdT key(uint32_t slot) const { return IdT(slot); }
};

// capacity for n keys: power of two >= 1.4 n (load factor <= 0.72, ~0.5 typical), >= 1024
inline uint32_t table_capacity(int64_t n) {
  uint64_t need = uint64_t(n) + uint64_t(n) * 2 / 5 + 1;
  uint64_t c = 1024;
  while (c < need) c <<= 1;
  return uint32_t(c);
}

}  // namespace dgs
#endif
