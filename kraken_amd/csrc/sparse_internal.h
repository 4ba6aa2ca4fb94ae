// Device-side layout of a sparse table and the probe routines shared by its kernels.
//
// HBM layout (one table):
//   slots   [slot_cap + 1] x 16 B   open-addressing index, linear probing, load <= 1/2:
//                                   {u64 key, u32 row, u32 epoch}. All-ones key = empty; the
//                                   extra last slot belongs to the one id whose value is all-ones.
//                                   epoch = number of the launch that created the row.
//   recs    [row_cap] x stride      one record per row, rows numbered in insertion order:
//                                   [ weight D | state columns D each, in creation order | steps ]
//                                   so a push touches one contiguous record instead of one line
//                                   per state array.
//   row_key [row_cap] x 8 B         id of each row (export and re-indexing walk rows, not slots)
//   counters[4] x 4 B               {rows used, error bits, -, workgroups finished}
//   host_pub   8 B, pinned host     {rows used, launch number} of the last finished launch that
//                                   could insert, written by the device so that the host can
//                                   bound the row count without waiting for the stream
#pragma once

#include <vector>

#include "krk_internal.h"

namespace krk {

struct Slot {
  unsigned long long key;
  unsigned long long row_epoch;   // low 32 bits: row, high 32 bits: epoch (one atomic word)
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
  uint32_t epoch;       // number of this launch, for launches that may insert
  unsigned long long* host_pub;   // pinned host memory, see publish_rows
};

__device__ __forceinline__ void load_slot(const Slot* s, unsigned long long& key,
                                          unsigned long long& row_epoch) {
  const uint4 raw = *reinterpret_cast<const uint4*>(s);
  key = (unsigned long long)raw.x | ((unsigned long long)raw.y << 32);
  row_epoch = (unsigned long long)raw.z | ((unsigned long long)raw.w << 32);
}

// id -> row, or kEmptyRow.
__device__ inline uint32_t probe_find(const TableView& tv, uint64_t id) {
  unsigned long long key, re;
  if (id == kEmptyKey) {
    load_slot(&tv.slots[tv.mask + 1], key, re);
    return key != kEmptyKey ? (uint32_t)re : kEmptyRow;
  }
  uint64_t idx = mix64(id) & tv.mask;
  for (uint64_t n = 0; n <= tv.mask; ++n) {
    load_slot(&tv.slots[idx], key, re);
    if (key == id) return (uint32_t)re;
    if (key == kEmptyKey) return kEmptyRow;
    idx = (idx + 1) & tv.mask;
  }
  return kEmptyRow;
}

// id -> row, claiming a slot and the next free row when absent. *owner is set for the one
// caller that created the row; *fresh for every caller whose row was created by this launch
// (its record may not be written yet, so its value must be recomputed, not read). A caller that
// meets a slot whose creator has not published the row number yet gets kEmptyRow and fresh.
__device__ inline uint32_t probe_insert(const TableView& tv, uint64_t id, bool* owner, bool* fresh) {
  *owner = false;
  *fresh = false;
  Slot* slot = nullptr;
  if (id == kEmptyKey) {
    slot = &tv.slots[tv.mask + 1];
    const unsigned long long old = atomicCAS(&slot->key, kEmptyKey, 0ull);
    if (old != kEmptyKey) {
      const unsigned long long re = __atomic_load_n(&slot->row_epoch, __ATOMIC_RELAXED);
      *fresh = (uint32_t)re == kEmptyRow || (uint32_t)(re >> 32) == tv.epoch;
      return (uint32_t)re;
    }
  } else {
    uint64_t idx = mix64(id) & tv.mask;
    for (uint64_t n = 0; n <= tv.mask; ++n) {
      unsigned long long key, re;
      load_slot(&tv.slots[idx], key, re);
      bool raced = false;
      if (key == kEmptyKey) {
        const unsigned long long old = atomicCAS(&tv.slots[idx].key, kEmptyKey, (unsigned long long)id);
        if (old == kEmptyKey) {
          slot = &tv.slots[idx];
          break;
        }
        key = old;
        raced = true;
      }
      if (key == id) {
        // the 16-byte load above may have straddled the creator's update: read the word again
        if (raced || (uint32_t)re == kEmptyRow)
          re = __atomic_load_n(&tv.slots[idx].row_epoch, __ATOMIC_RELAXED);
        *fresh = (uint32_t)re == kEmptyRow || (uint32_t)(re >> 32) == tv.epoch;
        return (uint32_t)re;
      }
      idx = (idx + 1) & tv.mask;
    }
    if (!slot) {
      atomicOr(&tv.counters[1], kErrOverflow);
      return kEmptyRow;
    }
  }
  const uint32_t row = atomicAdd(&tv.counters[0], 1u);
  if (row >= tv.row_cap) {
    atomicOr(&tv.counters[1], kErrOverflow);
    return kEmptyRow;
  }
  __atomic_store_n(&slot->row_epoch, (unsigned long long)row | ((unsigned long long)tv.epoch << 32),
                   __ATOMIC_RELAXED);
  tv.row_key[row] = id;
  *owner = true;
  *fresh = true;
  return row;
}

// Called by every thread of every workgroup of a launch that may insert, after its inserts.
// The workgroup that finishes last publishes {rows used, launch number} to pinned host memory:
// the host then knows the exact row count as of that launch without synchronising, and bounds
// the current count by adding the sizes of the requests enqueued since.
__device__ __forceinline__ void publish_rows(const TableView& tv, uint32_t workgroups) {
  // Every insert of this workgroup took its row number from a returning atomic on counters[0],
  // so those atomics have been performed once the barrier is passed; the counter of finished
  // workgroups is bumped with another atomic at the same place. No fence is needed, and none is
  // wanted: a release fence would write back the whole L2 once per workgroup.
  __syncthreads();
  if (threadIdx.x == 0) {
    const uint32_t done = atomicAdd(&tv.counters[3], 1u) + 1u;
    if (done == workgroups) {
      atomicExch(&tv.counters[3], 0u);
      const uint32_t rows = atomicAdd(&tv.counters[0], 0u);
      __hip_atomic_store(tv.host_pub, (unsigned long long)rows | ((unsigned long long)tv.epoch << 32),
                         __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    }
  }
}

}  // namespace krk

struct krk_group;

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
  unsigned long long* host_pub = nullptr;   // pinned, written by the device (publish_rows)
  uint64_t enq_total = 0;             // ids handed to inserting launches so far
  uint64_t enq_at[256] = {};          // enq_total right after the launch with number e (mod 256)
  uint32_t epoch = 0;                 // number of the last launch that could insert
  uint64_t layout_version = 0;        // bumped whenever slots, records or columns move

  int32_t col_off[KRK_ST_COUNT];      // float offset of each state column in a record, -1 = absent
  int32_t meta_off = -1;              // float offset of the step counter (two u32), -1 = absent
  int32_t meta_floats = 0;

  hipStream_t own_stream = nullptr;   // the stream created with the table (a group lends its own)
  krk_group* member_of = nullptr;

  krk::DeviceBuffer scratch[6];       // push_raw work space

  krk::TableView view() const {
    krk::TableView tv;
    tv.slots = slots;
    tv.mask = slot_cap - 1;
    tv.recs = recs;
    tv.stride = stride;
    tv.row_key = row_key;
    tv.counters = counters;
    tv.row_cap = (uint32_t)row_cap;
    tv.epoch = epoch;
    tv.host_pub = host_pub;
    return tv;
  }
};

namespace krk {
// Host-side pieces shared between the table's translation units.
int32_t sparse_ensure_room(krk_sparse* t, int64_t extra_rows);
int32_t sparse_ensure_columns(krk_sparse* t, uint32_t state_mask);
int32_t sparse_finish(krk_sparse* t, uint32_t flags);
// A new launch number for a launch that may insert up to n rows into t; call right before it.
int32_t sparse_next_epoch(krk_sparse* t, int64_t n);
// Column offsets an optimizer's three state slots map to (-1 = unused).
void sparse_optim_columns(const krk_sparse* t, const krk_optim& o, int32_t cols[3]);
// The three state types an optimizer's slots s0/s1/s2 hold (-1 = unused).
void optim_state_slots(const krk_optim& o, int32_t st[3]);
}  // namespace krk
