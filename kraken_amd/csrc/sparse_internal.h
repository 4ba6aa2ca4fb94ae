// Device-side layout of a sparse table and the probe routines shared by its kernels.
//
// HBM layout (one table):
//   slots   [slot_cap + 1] x 16 B   open-addressing index, buckets of 4 slots (one 64 B sector),
//                                   linear probing over buckets, load <= 1/2:
//                                   {u64 key, u32 row, u32 epoch}. All-ones key = empty; the
//                                   extra last slot belongs to the one id whose value is all-ones.
//                                   epoch = number of the launch that created the row.
//   recs    [row_cap] x stride      one record per row, rows numbered in insertion order:
//                                   [ weight D | state columns D each, in creation order | word ]
//                                   (word: 64 bits of counter and flag, see kHasMomentumBit;
//                                   a 64-byte sector of its own where dim is a multiple of 16)
//                                   so a push touches one contiguous record instead of one line
//                                   per state array.
//   row_key [row_cap] x 8 B         id of each row (export and re-indexing walk rows, not slots)
//   counters                        {rows used, error bits, 2 unused}, then the counters of the
//                                   lists a large pull queues its missing ids in
//   host_pub   8 B, pinned host     {rows used, launch number}: written by a one-wave kernel that
//                                   the host enqueues behind an inserting launch when the table
//                                   is close to full, so that it can bound the row count later
//                                   without waiting for the stream
//   + 4 B behind it                 set by a pull that found ids to insert; the host looks at it
//                                   when it enqueues the next pull and picks the launches for a
//                                   request that inserts if so
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
  uint32_t* inserted;   // pinned host word: a pull that makes rows sets it (see pull_enqueue)
};

constexpr int kBucket = 4;   // slots per bucket: one aligned 64-byte sector

// The 64-bit word a record keeps when an optimizer needs it: the low 63 bits count Adam's
// updates of the row (ps/optim/adam.cc:60, StateType::kSteps), the top bit says that the row has a
// momentum buffer, which is how SGD with momentum tells its first update of a row from the later
// ones (ps/optim/sgd.cc:46-52 looks for the state in the row's map).
constexpr unsigned long long kHasMomentumBit = 1ull << 63;

// Room of that word in a record, in floats. A row whose arrays are whole 64-byte sectors
// (dim a multiple of 16) gives the word a sector of its own, pads the record to a whole 128-byte
// line, and the push kernels write everything behind the arrays whole: a line written in part
// costs the memory a read as well, and a packed word (records of 208 or 400 bytes) shifts every
// array off its sectors. Measured per million rows at dim 32: Adam push 299 -> 266 us, pull
// 102 -> 84 us. Narrow rows keep the word packed behind the arrays.
__host__ __device__ inline int row_word_floats(int dim, int vec) {
  return (dim & 15) == 0 ? 16 : (vec == 4 ? 4 : 2);
}

// Writes the word of a record from inside a kernel whose lane groups have at least four lanes
// (gl = lane within the group; every lane of the group calls this). room = floats from the
// word to the end of the record: 16, or 32 when the padding sector follows.
template <int VEC>
__device__ __forceinline__ void store_row_word(float* word, unsigned long long value, int gl, int dim,
                                               int room) {
  if (VEC == 4 && (dim & 15) == 0) {
    if (gl < 4) {
      uint4 v = {0u, 0u, 0u, 0u};
      const uint4 zero = {0u, 0u, 0u, 0u};
      if (gl == 0) {
        v.x = (uint32_t)value;
        v.y = (uint32_t)(value >> 32);
      }
      reinterpret_cast<uint4*>(word)[gl] = v;   // four lanes: the sector is written whole
      if (room >= 32) reinterpret_cast<uint4*>(word)[gl + 4] = zero;   // and the rest of its line
    }
  } else if (gl == 0) {
    uint32_t* meta = reinterpret_cast<uint32_t*>(word);
    meta[0] = (uint32_t)value;
    meta[1] = (uint32_t)(value >> 32);
  }
}

__device__ __forceinline__ void unpack_slot(const uint4& raw, unsigned long long& key,
                                            unsigned long long& row_epoch) {
  key = (unsigned long long)raw.x | ((unsigned long long)raw.y << 32);
  row_epoch = (unsigned long long)raw.z | ((unsigned long long)raw.w << 32);
}

// Probing is done by the lane group that owns the id (at least four lanes, all holding the same
// id). The index is read a bucket at a time: the group's first four lanes load one slot each,
// which the hardware serves as a single 64-byte request, and two wave ballots tell every lane
// of the group whether the id or an empty slot was seen. Buckets are tried in linear order
// from the id's home bucket; a bucket fills from slot 0 upwards and slots are never released,
// so the first empty slot ends a search. What bounds a launch is the longest chain among its
// ids; chains are counted in buckets here, a quarter of what slot-by-slot probing walks.
//
// Every lane of the wavefront must call these functions together (they use wave-wide ballots
// and shuffles); lanes without work pass active = false.

struct ProbeResult {
  uint32_t row;   // kEmptyRow when absent (find) or when the creator has not published it yet
  bool owner;     // this group created the row
  bool fresh;     // the row was created by this launch: recompute its value, do not read it
};

__device__ __forceinline__ int wave_lane() { return (int)(threadIdx.x & (kWave - 1)); }

// Called by one lane of a wavefront that found ids to insert. A relaxed store to host memory:
// nothing waits for it, and the host only reads it as a hint.
__device__ __forceinline__ void note_inserting(const TableView& tv) {
  if (tv.inserted) __hip_atomic_store(tv.inserted, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// What a search that never writes reports: whether the id has a slot, and the slot's second
// word (row number in the low half, number of the launch that created the row in the high half).
struct FindResult {
  bool found;
  unsigned long long row_epoch;
};

__device__ inline FindResult probe_find_slot(const TableView& tv, uint64_t id, bool active, int gl,
                                             int group) {
  const int lane = wave_lane();
  const int base = lane & ~(group - 1);
  const uint64_t nb_mask = tv.mask >> 2;
  FindResult res;
  res.found = false;
  res.row_epoch = ~0ull;
  bool done = !active;
  if (active && id == kEmptyKey) {   // the id that equals the empty marker has a slot of its own
    unsigned long long key, re;
    unpack_slot(*reinterpret_cast<const uint4*>(&tv.slots[tv.mask + 1]), key, re);
    res.found = key != kEmptyKey;
    if (res.found) res.row_epoch = re;
    done = true;
  }
  uint64_t b = mix64(id) & nb_mask;
  uint64_t tried = 0;
  for (;;) {
    const bool part = !done && gl < kBucket;
    unsigned long long key = 0, re = 0;
    if (part) unpack_slot(*reinterpret_cast<const uint4*>(&tv.slots[b * kBucket + gl]), key, re);
    const unsigned long long m_match = __ballot(part && key == id);
    const unsigned long long m_empty = __ballot(part && key == kEmptyKey);
    int src = lane;
    int action = 0;   // 1 hit, 2 miss, 3 next bucket
    if (!done) {
      const uint32_t mm = (uint32_t)(m_match >> base) & 0xFu;
      const uint32_t me = (uint32_t)(m_empty >> base) & 0xFu;
      if (mm) {
        action = 1;
        src = base + __ffs(mm) - 1;
      } else {
        action = me ? 2 : 3;
      }
    }
    const unsigned long long r = __shfl(re, src);
    if (action == 1) {
      res.found = true;
      res.row_epoch = r;
      done = true;
    } else if (action == 2) {
      done = true;
    } else if (action == 3) {
      b = (b + 1) & nb_mask;
      if (++tried > nb_mask) done = true;
    }
    if (__ballot(!done) == 0ull) break;
  }
  return res;
}

// id -> row for every lane of the group, kEmptyRow when absent.
__device__ inline uint32_t probe_find(const TableView& tv, uint64_t id, bool active, int gl, int group) {
  const FindResult f = probe_find_slot(tv, id, active, gl, group);
  return f.found ? (uint32_t)f.row_epoch : kEmptyRow;
}

// id -> row, claiming a slot and the next free row when absent.
// DEFER: the slot is claimed here and the row is numbered by the caller (number_claimed_rows),
// for a whole workgroup with one addition to the row counter. The lane that claimed a slot
// reports it in won / slot; every lane of its group gets owner = true, row = kEmptyRow and in src
// the wavefront lane that holds the claim. Until the caller stores the row number the slot reads
// as a row whose creator has not published it yet.
template <bool DEFER>
__device__ inline ProbeResult probe_insert_impl(const TableView& tv, uint64_t id, bool active, int gl,
                                                int group, bool& won_out, Slot*& slot_out, int& src_out) {
  const int lane = wave_lane();
  const int base = lane & ~(group - 1);
  const uint64_t nb_mask = tv.mask >> 2;
  ProbeResult res;
  res.row = kEmptyRow;
  res.owner = false;
  res.fresh = false;
  bool done = !active;
  const bool special = active && id == kEmptyKey;
  if (special) {
    // handled by the group's first lane alone, shared with the others after the loop
    if (gl == 0) {
      Slot* slot = &tv.slots[tv.mask + 1];
      const unsigned long long old = atomicCAS(&slot->key, kEmptyKey, 0ull);
      if (old != kEmptyKey) {
        const unsigned long long re = __atomic_load_n(&slot->row_epoch, __ATOMIC_RELAXED);
        res.row = (uint32_t)re;
        res.fresh = res.row == kEmptyRow || (uint32_t)(re >> 32) == tv.epoch;
      } else if constexpr (DEFER) {
        won_out = true;
        slot_out = slot;
        res.owner = true;
        res.fresh = true;
      } else {
        const uint32_t row = atomicAdd(&tv.counters[0], 1u);
        if (row < tv.row_cap) {
          __atomic_store_n(&slot->row_epoch, (unsigned long long)row | ((unsigned long long)tv.epoch << 32),
                           __ATOMIC_RELAXED);
          tv.row_key[row] = id;
          res.row = row;
          res.owner = true;
        } else {
          atomicOr(&tv.counters[1], kErrOverflow);
        }
        res.fresh = true;
      }
    }
    done = true;
  }
  uint64_t b = mix64(id) & nb_mask;
  uint64_t tried = 0;
  for (;;) {
    const bool part = !done && gl < kBucket;
    unsigned long long key = 0, re = 0;
    Slot* mine = &tv.slots[b * kBucket + (gl < kBucket ? gl : 0)];
    if (part) unpack_slot(*reinterpret_cast<const uint4*>(mine), key, re);
    const unsigned long long m_match = __ballot(part && key == id);
    const unsigned long long m_empty = __ballot(part && key == kEmptyKey);
    int src = lane;
    int action = 0;   // 1 hit, 2 try to claim the first empty slot, 3 next bucket
    if (!done) {
      const uint32_t mm = (uint32_t)(m_match >> base) & 0xFu;
      const uint32_t me = (uint32_t)(m_empty >> base) & 0xFu;
      if (mm) {
        action = 1;
        src = base + __ffs(mm) - 1;
      } else if (me) {
        action = 2;
        src = base + __ffs(me) - 1;
      } else {
        action = 3;
      }
    }
    unsigned long long cas_old = 0;
    uint32_t new_row = kEmptyRow;
    bool won = false;
    if (action == 2 && lane == src) {
      cas_old = atomicCAS(&mine->key, kEmptyKey, (unsigned long long)id);
      won = cas_old == kEmptyKey;
      if (!won && cas_old == id) re = __atomic_load_n(&mine->row_epoch, __ATOMIC_RELAXED);
    } else if (action == 1 && lane == src && (uint32_t)re == kEmptyRow) {
      // the 16-byte load may have caught the creator between its two stores: read the word again
      re = __atomic_load_n(&mine->row_epoch, __ATOMIC_RELAXED);
    }
    // The slots claimed in this step get consecutive rows from one addition to the row counter per
    // wavefront: one addition per new id serialises on the counter's address (40 ns each, which
    // made 52k new ids in a request of a million cost 0.76 ms).
    if constexpr (DEFER) {
      if (won) {
        won_out = true;
        slot_out = mine;
      }
    }
    const unsigned long long winners = DEFER ? 0ull : __ballot(won);
    if (winners) {
      const int first_winner = __ffsll(winners) - 1;
      uint32_t first_row = 0;
      if (lane == first_winner) first_row = atomicAdd(&tv.counters[0], (uint32_t)__popcll(winners));
      first_row = __shfl(first_row, first_winner);
      if (won) {
        const uint32_t row = first_row + (uint32_t)__popcll(winners & ((1ull << lane) - 1ull));
        if (row < tv.row_cap) {
          __atomic_store_n(&mine->row_epoch, (unsigned long long)row | ((unsigned long long)tv.epoch << 32),
                           __ATOMIC_RELAXED);
          tv.row_key[row] = id;
          new_row = row;
        } else {
          atomicOr(&tv.counters[1], kErrOverflow);
        }
      }
    }
    const unsigned long long re_b = __shfl(re, src);
    const unsigned long long old_b = __shfl(cas_old, src);
    const uint32_t new_b = __shfl(new_row, src);
    if (action == 1 || (action == 2 && old_b == id)) {
      res.row = (uint32_t)re_b;
      res.fresh = res.row == kEmptyRow || (uint32_t)(re_b >> 32) == tv.epoch;
      done = true;
    } else if (action == 2 && old_b == kEmptyKey) {
      res.row = new_b;
      res.owner = DEFER || new_b != kEmptyRow;
      res.fresh = true;
      if (DEFER) src_out = src;
      done = true;
    } else if (action == 3) {
      b = (b + 1) & nb_mask;
      if (++tried > nb_mask) {
        atomicOr(&tv.counters[1], kErrOverflow);
        res.fresh = true;
        done = true;
      }
    }
    // action 2 with another id in the slot: somebody else took it, look at the same bucket again
    if (__ballot(!done) == 0ull) break;
  }
  if (group > 1) {
    // the special id was resolved by the first lane only
    const uint32_t row0 = __shfl(res.row, base);
    const int own0 = __shfl((int)res.owner, base);
    const int fresh0 = __shfl((int)res.fresh, base);
    if (special) {
      res.row = row0;
      res.owner = own0 != 0;
      res.fresh = fresh0 != 0;
      if (DEFER) src_out = base;
    }
  }
  return res;
}

__device__ inline ProbeResult probe_insert(const TableView& tv, uint64_t id, bool active, int gl,
                                           int group) {
  bool won = false;
  Slot* slot = nullptr;
  int src = 0;
  return probe_insert_impl<false>(tv, id, active, gl, group, won, slot, src);
}

// One lane looking an id up by itself (no votes): the rare second look of pooled_sum_kernel.
__device__ inline uint32_t probe_find_alone(const TableView& tv, uint64_t id) {
  if (id == kEmptyKey) {
    const Slot* s = &tv.slots[tv.mask + 1];
    return __atomic_load_n(&s->key, __ATOMIC_RELAXED) != kEmptyKey
               ? (uint32_t)__atomic_load_n(&s->row_epoch, __ATOMIC_RELAXED) : kEmptyRow;
  }
  const uint64_t nb_mask = tv.mask >> 2;
  uint64_t b = mix64(id) & nb_mask;
  for (uint64_t tried = 0; tried <= nb_mask; ++tried) {
    for (int i = 0; i < kBucket; ++i) {
      const Slot* s = &tv.slots[b * kBucket + i];
      const unsigned long long key = __atomic_load_n(&s->key, __ATOMIC_RELAXED);
      if (key == id) return (uint32_t)__atomic_load_n(&s->row_epoch, __ATOMIC_RELAXED);
      if (key == kEmptyKey) return kEmptyRow;
    }
    b = (b + 1) & nb_mask;
  }
  return kEmptyRow;
}

}  // namespace krk

struct krk_group;

namespace krk {
// Requests of at most this many ids a table keep row notes (KRK_NOTE_ROWS): the pulls that run
// as one launch.
constexpr int64_t kNotedMax = (1 << 18) - 1;
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
  unsigned long long* host_pub = nullptr;   // pinned, written by the device (publish_kernel)
  uint32_t* host_inserted = nullptr;        // pinned, behind host_pub: set by pulls that insert
  int64_t last_request = 0;           // size of the last inserting request
  uint64_t enq_total = 0;             // ids handed to inserting launches so far
  uint64_t enq_at[256] = {};          // enq_total right after the launch with number e (mod 256)
  uint32_t epoch = 0;                 // number of the last launch that could insert
  uint64_t layout_version = 0;        // bumped whenever slots, records or columns move
  int pull_parity = 0;                // which set of list counters the next two-launch pull queues into

  int32_t col_off[KRK_ST_COUNT];      // float offset of each state column in a record, -1 = absent
  int32_t meta_off = -1;              // float offset of the step counter (two u32), -1 = absent
  int32_t meta_floats = 0;

  hipStream_t own_stream = nullptr;   // the stream created with the table (a group lends its own)
  krk_group* member_of = nullptr;

  krk::DeviceBuffer scratch[6];       // push_raw work space

  // Row notes (KRK_NOTE_ROWS): the row of every position of one pull, kept for a push_raw of the
  // same ids. Valid while noted_ids is not null and noted_version == layout_version.
  krk::DeviceBuffer notes;
  const uint64_t* noted_ids = nullptr;
  int64_t noted_n = 0;
  uint64_t noted_version = 0;

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
    tv.inserted = host_inserted;
    return tv;
  }
};

namespace krk {
constexpr int kMaxGroupTables = 32;

// What a kernel of a combined request needs to know about one member table.
struct TableDesc {
  TableView tv;
  InitK init;
  int32_t col_off[KRK_ST_COUNT];
  int32_t meta_off;
};

// One combined request: the launch number of each member, and where each member's ids start,
// in workgroups of the one-launch kernels (block_start) and in positions (row_start).
struct GroupCall {
  int32_t n_tables;
  // > 0: every member owns exactly this many workgroups (block_start[t] = t * even_blocks), so a
  // workgroup finds its member by one division instead of walking block_start. The host lays a
  // request out like this whenever that costs at most a quarter more workgroups.
  uint32_t even_blocks;
  uint32_t epoch[kMaxGroupTables];
  uint32_t block_start[kMaxGroupTables + 1];
  int64_t row_start[kMaxGroupTables + 1];
};

// What a combined pull carries besides when it queues its missing ids (the members' tables are
// being filled): every member has its own 64 lists, counted by its own table's list counters.
struct GroupFill {
  uint32_t todo_start[kMaxGroupTables];   // first word of member t's lists in the work space
  uint32_t parity_bits;                   // bit t: the set of member t's list counters in use
};
}  // namespace krk

// Tables of one combined request (CombinePull/PushSparseTable): they share one stream, and a
// device-resident array of their layouts that is refreshed only when a table has moved.
struct krk_group : krk::ObjBase {
  std::vector<krk_sparse*> tables;
  std::vector<uint64_t> versions;
  krk::TableDesc* d_descs = nullptr;
  krk::TableDesc* h_descs = nullptr;   // pinned
  int64_t dim = 0;
  int vec = 1, elems = 0, group = 1;
  hipStream_t own_stream = nullptr;    // the stream created with the group
  krk::DeviceBuffer scratch[5];        // push_raw work space
  // Row notes of one combined pull (see krk_sparse::notes): valid while noted_ids is not null
  // and every member's layout_version is what it was.
  krk::DeviceBuffer notes;
  krk::DeviceBuffer todo;              // the lists of a combined pull that queues its missing ids
  const uint64_t* noted_ids = nullptr;
  std::vector<int64_t> noted_offsets;
  std::vector<uint64_t> noted_versions;
};

namespace krk {
// KRK_IDS_AS_PULLED: the row notes of the pull of these very ids, or null when they do not apply
// (another buffer or count, nothing noted, rows moved since). The caller holds the lock(s).
inline const uint32_t* noted_rows(const krk_sparse* t, const uint64_t* ids, int64_t n, uint32_t flags) {
  const bool ok = (flags & KRK_IDS_AS_PULLED) && t->noted_ids && t->noted_ids == ids && t->noted_n == n &&
                  t->noted_version == t->layout_version;
  return ok ? t->notes.as<uint32_t>() : nullptr;
}
inline const uint32_t* noted_rows(const krk_group* g, const uint64_t* ids, const int64_t* offsets, uint32_t flags) {
  const size_t n = g->tables.size();
  bool ok = (flags & KRK_IDS_AS_PULLED) && g->noted_ids && g->noted_ids == ids && g->noted_offsets.size() == n + 1 &&
            g->noted_versions.size() == n;
  for (size_t m = 0; ok && m < n; ++m)
    ok = g->noted_offsets[m] == offsets[m] && g->noted_offsets[m + 1] == offsets[m + 1] &&
         g->noted_versions[m] == g->tables[m]->layout_version;
  return ok ? g->notes.as<uint32_t>() : nullptr;
}

// Takes the group's lock and then every member's, in member order.
struct GroupLock {
  krk_group* g;
  explicit GroupLock(krk_group* gg) : g(gg) {
    g->mu.lock();
    for (krk_sparse* t : g->tables) t->mu.lock();
  }
  ~GroupLock() {
    for (auto it = g->tables.rbegin(); it != g->tables.rend(); ++it) (*it)->mu.unlock();
    g->mu.unlock();
  }
  GroupLock(const GroupLock&) = delete;
  GroupLock& operator=(const GroupLock&) = delete;
};
// Checks the offsets of a combined request and lays its members out over the grid.
// per_block: positions a workgroup of the launch takes (0: kBlock / the group's lanes per row)
int32_t group_plan(krk_group* g, const int64_t* offsets, GroupCall* call, int64_t* total, int per_block = 0);
// Uploads the layouts of members that moved since the last call.
int32_t group_refresh(krk_group* g);
// Blocking calls: waits for the group's stream and reports the first member's error.
int32_t group_finish(krk_group* g, uint32_t flags);

// Host-side pieces shared between the table's translation units.
int32_t sparse_ensure_room(krk_sparse* t, int64_t extra_rows);
int32_t sparse_ensure_columns(krk_sparse* t, uint32_t state_mask);
int32_t sparse_finish(krk_sparse* t, uint32_t flags);
// A new launch number for a launch that may insert up to n rows into t; call right before it.
int32_t sparse_next_epoch(krk_sparse* t, int64_t n);
// True when only a few more requests like the last one fit under the current row bound.
bool sparse_near_full(const krk_sparse* t);
// Enqueues the kernel that publishes {rows used, launch number} of each table to the host.
int32_t sparse_publish(krk_sparse* const* tables, int n, hipStream_t stream);
// Host ids -> each row's stored 64-bit word (counter and momentum flag), blocking.
int32_t sparse_fetch_words(krk_sparse* t, const uint64_t* ids, int64_t n, int64_t* words);
// Column offsets an optimizer's three state slots map to (-1 = unused).
void sparse_optim_columns(const krk_sparse* t, const krk_optim& o, int32_t cols[3]);
// The three state types an optimizer's slots s0/s1/s2 hold (-1 = unused).
void optim_state_slots(const krk_optim& o, int32_t st[3]);
}  // namespace krk
