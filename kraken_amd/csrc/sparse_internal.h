// Device-side layout of a sparse table and the probe routines shared by its kernels.
//
// HBM layout (one table):
//   slots   [slot_cap + 1] x 16 B   open-addressing index, linear probing, load <= 1/2:
//                                   {u64 key, u32 row, u32 pad}. All-ones key = empty; the extra
//                                   last slot belongs to the one id whose value is all-ones.
//   recs    [row_cap] x stride      one record per row, rows numbered in insertion order:
//                                   [ weight D | state columns D each, in creation order | steps ]
//                                   so a push touches one contiguous record instead of one line
//                                   per state array.
//   row_key [row_cap] x 8 B         id of each row (export and re-indexing walk rows, not slots)
//   counters[4] x 4 B               {rows used, error bits, -, -}
#pragma once

#include "krk_internal.h"

namespace krk {

struct Slot {
  unsigned long long key;
  uint32_t row;
  uint32_t pad;
};
static_assert(sizeof(Slot) == 16, "slot is one 16-byte load");

constexpr uint32_t kErrMissingId = 1u;   // a push named an id that is not in the table
constexpr uint32_t kErrOverflow = 2u;    // a probe or the row counter ran past capacity

struct TableView {
  Slot* slots;
  uint64_t mask;        // slot_cap - 1
  float* recs;
  int64_t stride;       // floats per record
  unsigned long long* row_key;
  uint32_t* counters;   // [0] rows used, [1] error bits
  uint32_t row_cap;
};

__device__ __forceinline__ void load_slot(const Slot* s, unsigned long long& key, uint32_t& row) {
  const uint4 raw = *reinterpret_cast<const uint4*>(s);
  key = (unsigned long long)raw.x | ((unsigned long long)raw.y << 32);
  row = raw.z;
}

// id -> row, or kEmptyRow.
__device__ inline uint32_t probe_find(const TableView& tv, uint64_t id) {
  unsigned long long key;
  uint32_t row;
  if (id == kEmptyKey) {
    load_slot(&tv.slots[tv.mask + 1], key, row);
    return key != kEmptyKey ? row : kEmptyRow;
  }
  uint64_t idx = mix64(id) & tv.mask;
  for (uint64_t n = 0; n <= tv.mask; ++n) {
    load_slot(&tv.slots[idx], key, row);
    if (key == id) return row;
    if (key == kEmptyKey) return kEmptyRow;
    idx = (idx + 1) & tv.mask;
  }
  return kEmptyRow;
}

// id -> row, claiming a slot and the next free row when absent. *owner is set for the one
// caller that created the row. A caller that finds a slot another thread of the same launch
// is still filling gets kEmptyRow back and must treat the row as freshly initialised.
__device__ inline uint32_t probe_insert(const TableView& tv, uint64_t id, bool* owner) {
  *owner = false;
  Slot* slot = nullptr;
  if (id == kEmptyKey) {
    slot = &tv.slots[tv.mask + 1];
    unsigned long long old = atomicCAS(&slot->key, kEmptyKey, 0ull);
    if (old != kEmptyKey) return __atomic_load_n(&slot->row, __ATOMIC_RELAXED);
  } else {
    uint64_t idx = mix64(id) & tv.mask;
    uint64_t n = 0;
    for (; n <= tv.mask; ++n) {
      unsigned long long key;
      uint32_t row;
      load_slot(&tv.slots[idx], key, row);
      if (key == kEmptyKey) {
        unsigned long long old = atomicCAS(&tv.slots[idx].key, kEmptyKey, (unsigned long long)id);
        if (old == kEmptyKey) {
          slot = &tv.slots[idx];
          break;
        }
        key = old;
        row = kEmptyRow;  // whoever holds it may not have published the row yet
        if (key == id) return __atomic_load_n(&tv.slots[idx].row, __ATOMIC_RELAXED);
      } else if (key == id) {
        return row;
      }
      idx = (idx + 1) & tv.mask;
    }
    if (!slot) {
      atomicOr(&tv.counters[1], kErrOverflow);
      return kEmptyRow;
    }
  }
  uint32_t row = atomicAdd(&tv.counters[0], 1u);
  if (row >= tv.row_cap) {
    atomicOr(&tv.counters[1], kErrOverflow);
    return kEmptyRow;
  }
  __atomic_store_n(&slot->row, row, __ATOMIC_RELAXED);
  tv.row_key[row] = id;
  *owner = true;
  return row;
}

}  // namespace krk

// The handle behind krk_sparse*.
struct krk_sparse : krk::ObjBase {
  int64_t dim = 0;
  int vec = 1;            // floats per lane access: 4 when dim % 4 == 0, else 1
  int elems = 0;          // dim / vec
  int group = 1;          // lanes cooperating on one row (power of two, <= 64)
  krk_init init{};
  krk::InitK initk{};

  krk::Slot* slots = nullptr;
  uint64_t slot_cap = 0;
  float* recs = nullptr;
  int64_t stride = 0;
  int64_t row_cap = 0;
  unsigned long long* row_key = nullptr;
  uint32_t* counters = nullptr;       // device
  uint32_t* host_counters = nullptr;  // pinned
  int64_t size_ub = 0;                // upper bound of rows used, exact after a blocking call
  bool async_inflight = false;        // an async call was enqueued since the last blocking one

  int32_t col_off[KRK_ST_COUNT];      // float offset of each state column in a record, -1 = absent
  int32_t meta_off = -1;              // float offset of the step counter (two u32), -1 = absent
  int32_t meta_floats = 0;

  krk::DeviceBuffer scratch[6];       // push_raw / dedup work space

  krk::TableView view() const {
    krk::TableView tv;
    tv.slots = slots;
    tv.mask = slot_cap - 1;
    tv.recs = recs;
    tv.stride = stride;
    tv.row_key = row_key;
    tv.counters = counters;
    tv.row_cap = (uint32_t)row_cap;
    return tv;
  }
};

namespace krk {
// Host-side pieces shared between the table's translation units.
int32_t sparse_ensure_room(krk_sparse* t, int64_t extra_rows);
int32_t sparse_ensure_columns(krk_sparse* t, uint32_t state_mask);
int32_t sparse_finish(krk_sparse* t, uint32_t flags);
// Column offsets an optimizer's three state slots map to (-1 = unused).
void sparse_optim_columns(const krk_sparse* t, const krk_optim& o, int32_t cols[3]);
}  // namespace krk
