// Sparse table: id -> row lookup in an HBM-resident open-addressing index, pull (gather with
// insert-on-miss) and push (one fused read-modify-write of weight + optimizer state per row).
//
// Replaces SparseTable::Pull / ::Push (ps/sparse_table.cc:33-108), the per-row Optim::Update
// chains (ps/optim/*.cc), the row initialisers (ps/initializer/*.cc, t/math.cc:333-517) and, for
// a group of tables, the loops of Ps::CombinePullSparseTable / CombinePushSparseTable
// (ps/ps_op.cc:370-387, 456-469), which become one launch over all tables of the request.
//
// Work mapping: `group` adjacent lanes (at least four) of a 64-wide wavefront own one id. Four
// of them read an index bucket together (one 64-byte request per probe step) and wave ballots
// give every lane of the group the row number; then every lane moves `vec` floats of the
// record per step, so a dim-16 row is four float4 lanes and sixteen rows share one wavefront
// instruction.
#include <algorithm>
#include <cmath>
#include <new>

#include "sparse_internal.h"

namespace krk {

constexpr int kBlock = 256;
constexpr int64_t kTwoLaunchPull = 1 << 18;   // ids from which a pull runs as two launches
constexpr int64_t kTwoLaunchWhileFilling = 1 << 13;   // the same while the pulls before it inserted rows
// A wavefront tells the host that the table is being filled when that many of its sixteen (or
// fewer) ids are new. From one new id in 250 on, the fused kernel's additions to the row counter
// cost a request of 98 600 ids more than a second launch does (7 us more). Three new ids in one
// wavefront: once in five such requests at that share, in every request from one new id in a
// hundred on, and once in three hundred requests at one in a thousand (two in one wavefront
// would send every other of those through the two launches for nothing).
constexpr int kFillingIds = 3;
// A combined request spreads its additions over its members' counters, and its two launches cost
// 15 us more than its fused kernel where nothing is new: over 26 tables they pay from one new id
// in five on (98.6k ids, one in ten new: 21 us fused, 27 us in two launches; all new: 64 and 34).
constexpr int kFillingIdsCombined = 8;
constexpr int kMissingGrid = 512;             // workgroups (of 1024 lanes) of the launch that inserts missing ids
// The positions whose id is missing are queued in kQueues lists, each with a counter on a line
// of its own: workgroup b of the first launch appends to list b mod kQueues. One counter for the
// whole request serialises on its address: 36k additions of a 5 %-new request of a million ids
// made the first launch take 428 us instead of 131.
constexpr int kQueues = 64;
constexpr int kQueueCounterStride = 32;       // 32-bit words between two lists' counters: 128 bytes
constexpr int kQueueCounterWords = 2 * kQueues * kQueueCounterStride;   // two sets, used in turn
constexpr int kCounterWords = 4 + kQueueCounterWords;                    // what t->counters holds

// Entries list q of a request of n positions can hold: every workgroup appends at most
// ids_per_block entries to its list.
__host__ __device__ inline int64_t queue_capacity(int64_t n, int ids_per_block) {
  const int64_t blocks = (n + ids_per_block - 1) / ids_per_block;
  return ((blocks + kQueues - 1) / kQueues) * ids_per_block;
}
__device__ __forceinline__ uint32_t* queue_counter(const TableView& tv, int parity, int q) {
  return tv.counters + 4 + (parity * kQueues + q) * kQueueCounterStride;
}

// VEC initial values of a new row (first is a multiple of VEC), evaluated one after the other:
// the loop stays rolled so that the double-precision Box-Muller of the rare branch is live once,
// not VEC times, and the kernels that carry it keep their occupancy (the pulls are bound by the
// reads in flight).
// (UNROLLED: the kernels that only handle new ids evaluate the values side by side instead, and
// normal draws a pair at a time: an evaluation is a long chain of dependent double-precision
// operations, and those kernels have few wavefronts to hide it behind.)
template <int VEC, bool UNROLLED = false>
__device__ __forceinline__ void init_vec(const InitK& init, uint64_t id, int64_t first, float (&v)[VEC]) {
  if constexpr (UNROLLED) {
    if constexpr (VEC == 4) {
      if (init.kind == 2) {
        const uint64_t key = splitmix64(id ^ init.seed_mix);
        init_normal_pair(init, key, first >> 1, v[0], v[1]);
        init_normal_pair(init, key, (first >> 1) + 1, v[2], v[3]);
        return;
      }
    }
#pragma unroll
    for (int c = 0; c < VEC; ++c) v[c] = init_element(init, id, first + c);
  } else {
#pragma unroll
    for (int c = 0; c < VEC; ++c) v[c] = 0.0f;
#pragma unroll 1
    for (int c = 0; c < VEC; ++c) {
      const float x = init_element(init, id, first + c);
#pragma unroll
      for (int k = 0; k < VEC; ++k) v[k] = k == c ? x : v[k];
    }
  }
}

template <int VEC>
__device__ __forceinline__ void vload(const float* p, float (&v)[VEC]) {
  if constexpr (VEC == 4) {
    const float4 x = *reinterpret_cast<const float4*>(p);
    v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
  } else {
    v[0] = *p;
  }
}
// Streams that pass once (gradient rows in, pulled rows out): non-temporal, so they leave the
// caches to the index and the records.
typedef float vfloat4_t __attribute__((ext_vector_type(4)));
template <int VEC>
__device__ __forceinline__ void vload_once(const float* p, float (&v)[VEC]) {
  if constexpr (VEC == 4) {
    const vfloat4_t x = __builtin_nontemporal_load(reinterpret_cast<const vfloat4_t*>(p));
    v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
  } else {
    v[0] = __builtin_nontemporal_load(p);
  }
}
template <int VEC>
__device__ __forceinline__ void vstore_once(float* p, const float (&v)[VEC]) {
  if constexpr (VEC == 4) {
    const vfloat4_t x = {v[0], v[1], v[2], v[3]};
    __builtin_nontemporal_store(x, reinterpret_cast<vfloat4_t*>(p));
  } else {
    __builtin_nontemporal_store(v[0], p);
  }
}
template <int VEC>
__device__ __forceinline__ void vstore(float* p, const float (&v)[VEC]) {
  if constexpr (VEC == 4) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  } else {
    *p = v[0];
  }
}

// ---------------------------------------------------------------------------
// pull: gather rows, inserting and initialising the ones that are missing.
// `i` is this lane group's position in ids/out, gl the lane's index in the group.
// ---------------------------------------------------------------------------
template <int VEC, bool MOSTLY_NEW = false>
__device__ __forceinline__ void pull_body(const TableView& tv, const InitK& init,
                                          const uint64_t* __restrict__ ids, int64_t i, bool active,
                                          int gl, float* __restrict__ out, int dim, int elems,
                                          int group, uint32_t* __restrict__ notes = nullptr,
                                          int filling_ids = kFillingIds) {
  const uint64_t id = active ? ids[i] : 0;
  // Most ids are resident: a search that never writes settles them, and only a wavefront that
  // holds a missing id goes through the claiming search as well.
  const FindResult f = probe_find_slot(tv, id, active, gl, group);
  ProbeResult pr;
  pr.row = (uint32_t)f.row_epoch;
  pr.owner = false;
  pr.fresh = pr.row == kEmptyRow || (uint32_t)(f.row_epoch >> 32) == tv.epoch;
  const bool miss = active && !f.found;
  if (__any(miss)) {
    const ProbeResult q = probe_insert(tv, id, miss, gl, group);
    if (miss) pr = q;
    // (a wavefront of a table whose lane groups are 64 lanes wide carries one id: any new id counts)
    const int enough = filling_ids < kWave / group ? filling_ids : kWave / group;
    if (__popcll(__ballot(miss && gl == 0)) >= enough && wave_lane() == 0) note_inserting(tv);
  }
  if (!active) return;
  const uint32_t row = pr.row;
  const bool owner = pr.owner;
  const bool fresh = pr.fresh;
  // where the id lives, for a push of the same ids that follows (kEmptyRow: the table is full)
  if (notes && gl == 0) notes[i] = row;
  float* rec = row == kEmptyRow ? nullptr : tv.recs + (int64_t)row * tv.stride;
  float* dst = out + i * (int64_t)dim;
  for (int e = gl; e < elems; e += group) {
    float v[VEC];
    if (fresh) {
      // the value of a new row is a pure function of (seed, id, element): every group that
      // meets it computes the same numbers, only the creator stores them
      init_vec<VEC, MOSTLY_NEW>(init, id, (int64_t)e * VEC, v);
      if (owner) vstore<VEC>(rec + e * VEC, v);
    } else {
      vload<VEC>(rec + e * VEC, v);
    }
    vstore_once<VEC>(dst + e * VEC, v);
  }
}

// ---------------------------------------------------------------------------
// push: per unique id, one fused update of the record
// ---------------------------------------------------------------------------
struct PushCols {
  int c0, c1, c2, meta;
};

// The row of ids[i] for a push: looked up, or taken from the notes of the pull of the same ids
// (KRK_IDS_AS_PULLED). A note of kEmptyRow was taken before the row's creator had published the
// number (or the table was full): those are looked up after all. Wave-wide like probe_find.
__device__ __forceinline__ uint32_t row_for_push(const TableView& tv, const uint64_t* __restrict__ ids,
                                                 int64_t i, bool active, int gl, int group,
                                                 const uint32_t* __restrict__ notes) {
  if (!notes) return probe_find(tv, active ? ids[i] : 0, active, gl, group);
  uint32_t row = active ? notes[i] : kEmptyRow;
  const bool again = active && row == kEmptyRow;
  if (__any(again)) {
    const uint32_t r = probe_find(tv, again ? ids[i] : 0, again, gl, group);
    if (again) row = r;
  }
  return row;
}

template <int OPT, int VEC>
__device__ __forceinline__ void push_body(const TableView& tv, const uint64_t* __restrict__ ids,
                                          int64_t i, bool active, int gl,
                                          const float* __restrict__ grads, int dim, int elems,
                                          int group, float lr, const OptimK& k, const PushCols& pc,
                                          const uint32_t* __restrict__ notes = nullptr) {
  // The gradient row does not depend on the index: its first slice is requested before the
  // probe so that it travels while the probe waits for its bucket.
  const float* g = grads + i * (int64_t)dim;
  float g_first[VEC];
#pragma unroll
  for (int c = 0; c < VEC; ++c) g_first[c] = 0.0f;
  if (active && gl < elems) vload_once<VEC>(g + gl * VEC, g_first);
  const uint32_t row = row_for_push(tv, ids, i, active, gl, group, notes);
  if (!active) return;
  if (row == kEmptyRow) {
    if (gl == 0) atomicOr(&tv.counters[1], kErrMissingId);
    return;
  }
  float* rec = tv.recs + (int64_t)row * tv.stride;

  // The lane's first slice of the record is requested before the 64-bit word is looked at: the
  // bias corrections (two powf) then overlap with the loads instead of preceding them.
  float w[VEC], s0[VEC], s1[VEC], s2[VEC];
  if (gl < elems) {
    vload<VEC>(rec + gl * VEC, w);
    if (pc.c0 >= 0) vload<VEC>(rec + pc.c0 + gl * VEC, s0);
    if (pc.c1 >= 0) vload<VEC>(rec + pc.c1 + gl * VEC, s1);
    if (pc.c2 >= 0) vload<VEC>(rec + pc.c2 + gl * VEC, s2);
  }
  bool first = false;
  float bc1 = 1.0f, bc2 = 1.0f;
  uint64_t steps = 0;
  if (pc.meta >= 0) {
    const uint32_t* meta = reinterpret_cast<const uint32_t*>(rec + pc.meta);
    steps = (uint64_t)meta[0] | ((uint64_t)meta[1] << 32);
    if (OPT == KRK_ADAM) {
      steps += 1;                           // the flag bit rides along untouched
    } else {
      first = (steps & kHasMomentumBit) == 0;
      steps |= kHasMomentumBit;
    }
    if (OPT == KRK_ADAM) {
      // ps/optim/adam.cc:61-64 : per-row step counter, float pow, double subtraction
      const float count = (float)(steps & ~kHasMomentumBit);
      bc1 = (float)(1.0 - (double)powf(k.beta1, count));
      bc2 = (float)(1.0 - (double)powf(k.beta2, count));
    }
  }
  for (int e = gl; e < elems; e += group) {
    float gv[VEC];
    if (e == gl) {
#pragma unroll
      for (int c = 0; c < VEC; ++c) gv[c] = g_first[c];
    } else {
      vload_once<VEC>(g + e * VEC, gv);
      vload<VEC>(rec + e * VEC, w);
      if (pc.c0 >= 0) vload<VEC>(rec + pc.c0 + e * VEC, s0);
      if (pc.c1 >= 0) vload<VEC>(rec + pc.c1 + e * VEC, s1);
      if (pc.c2 >= 0) vload<VEC>(rec + pc.c2 + e * VEC, s2);
    }
#pragma unroll
    for (int c = 0; c < VEC; ++c) {
      if (pc.c0 < 0) s0[c] = 0.0f;
      if (pc.c1 < 0) s1[c] = 0.0f;
      if (pc.c2 < 0) s2[c] = 0.0f;
      optim_element<OPT>(k, lr, gv[c], w[c], s0[c], s1[c], s2[c], first, bc1, bc2);
    }
    // written once per launch and not read again by it: past the caches, so that the end of the
    // kernel has no dirty lines left to write back
    vstore_once<VEC>(rec + e * VEC, w);
    if (pc.c0 >= 0) vstore_once<VEC>(rec + pc.c0 + e * VEC, s0);
    if (pc.c1 >= 0) vstore_once<VEC>(rec + pc.c1 + e * VEC, s1);
    if (pc.c2 >= 0) vstore_once<VEC>(rec + pc.c2 + e * VEC, s2);
  }
  if (pc.meta >= 0) store_row_word<VEC>(rec + pc.meta, steps, gl, dim, (int)tv.stride - pc.meta);
}

// ---- single-table launches ---------------------------------------------------
template <int VEC>
__global__ __launch_bounds__(kBlock) void pull_kernel(TableView tv, InitK init,
                                                      const uint64_t* __restrict__ ids, int64_t n,
                                                      float* __restrict__ out, int dim, int elems,
                                                      int group, uint32_t* __restrict__ notes) {
  const int per_block = kBlock / group;
  const int64_t i = (int64_t)blockIdx.x * per_block + threadIdx.x / group;
  pull_body<VEC>(tv, init, ids, i, i < n, threadIdx.x & (group - 1), out, dim, elems, group, notes);
}

// ---- large pulls in two launches ------------------------------------------------
// A large pull is bound by the random reads in flight, and in the fused kernels a wavefront that
// inserts holds up the other ids it carries and adds to the row counter on its own. So a large
// request first runs a kernel that only searches and copies and queues the positions whose id is
// missing; a second, small launch walks those lists (pull_missing_kernel). In steady state the
// lists are empty and the second launch ends at once.
// Two sets of list counters are used in turn; the second launch clears the other set for the
// request after it (same stream, so that request's first kernel has not started).
// bx: the workgroup's number among those of this table's request
template <int VEC>
__device__ __forceinline__ void pull_resident_body(const TableView& tv, const uint64_t* __restrict__ ids,
                                                   int64_t n, float* __restrict__ out,
                                                   uint32_t* __restrict__ todo, int parity, int dim,
                                                   int elems, int group, uint32_t bx,
                                                   uint32_t* __restrict__ notes) {
  const int per_block = kBlock / group;
  const int64_t i = (int64_t)bx * per_block + threadIdx.x / group;
  const int gl = threadIdx.x & (group - 1);
  const bool active = i < n;
  const uint32_t row = probe_find(tv, active ? ids[i] : 0, active, gl, group);
  // one atomic per wavefront reserves entries of the workgroup's list for all of its missing ids
  const bool queue = active && row == kEmptyRow && gl == 0;
  const unsigned long long votes = __ballot(queue);
  if (votes) {
    const int lane = wave_lane();
    const int first = __ffsll(votes) - 1;
    const int q = bx & (kQueues - 1);
    uint32_t base = 0;
    if (lane == first) base = atomicAdd(queue_counter(tv, parity, q), (uint32_t)__popcll(votes));
    base = __shfl(base, first);
    if (queue)
      todo[q * queue_capacity(n, per_block) + base + (uint32_t)__popcll(votes & ((1ull << lane) - 1ull))] =
          (uint32_t)i;
  }
  // the note of a missing id is written by the launch that inserts it
  if (notes && active && gl == 0 && row != kEmptyRow) notes[i] = row;
  if (!active || row == kEmptyRow) return;
  const float* rec = tv.recs + (int64_t)row * tv.stride;
  float* dst = out + i * (int64_t)dim;
  for (int e = gl; e < elems; e += group) {
    float v[VEC];
    vload<VEC>(rec + e * VEC, v);
    vstore_once<VEC>(dst + e * VEC, v);
  }
}

template <int VEC>
__global__ __launch_bounds__(kBlock) void pull_resident_kernel(TableView tv, const uint64_t* __restrict__ ids,
                                                               int64_t n, float* __restrict__ out,
                                                               uint32_t* __restrict__ todo, int parity, int dim,
                                                               int elems, int group, uint32_t* __restrict__ notes) {
  pull_resident_body<VEC>(tv, ids, n, out, todo, parity, dim, elems, group, blockIdx.x, notes);
}

// The second launch: workgroups of 1024 lanes walk the lists, 256 entries at a time.
//   1. Four lanes per entry claim a slot for its id (or find that another entry did).
//   2. The rows of everything the workgroup claimed are numbered with one addition to the row
//      counter. Additions to one address are served one after the other, some 15 ns each, and one
//      per wavefront made a million new ids take 0.87 ms and 98 600 take 131 us, twelve times a
//      pull of resident ids, at every row width.
//   3. The lanes regroup, one lane group per entry as in pull_body, and initialise, store and
//      copy the rows; an entry's id, position, row and state pass through LDS.
// The trip count is the same for every lane of a workgroup (barriers inside).
// ROWS_ONLY (the pooled pull while a table is being filled): nothing is copied; the creator
// initialises the record and every entry's row number goes to rows_out[position] (kEmptyRow where
// the creator, another entry, has not published it yet: pooled_sum_kernel looks those up).
constexpr int kMissBlock = 1024;
constexpr int kMissEntries = kMissBlock / kBucket;
constexpr int kMissWaves = kMissBlock / kWave;

// Entries k_first, k_first + stride, ... of `count` queued positions, kMissEntries at a time (the
// workgroups that share them are `stride` apart); position_of(k) names the k-th.
// MODE: what is done with an entry once its row is known.
constexpr int kInsertAndCopy = 0;   // a pull: new rows are initialised, every entry's row goes to out
constexpr int kInsertOnly = 1;      // ROWS_ONLY
constexpr int kInsertGiven = 2;     // an import: the creator copies the row out[position] into the record
template <int VEC, int MODE, typename PositionOf>
__device__ __forceinline__ void insert_queued(const TableView& tv, const InitK& init,
                                              const uint64_t* __restrict__ ids, float* __restrict__ out,
                                              PositionOf position_of, uint32_t count,
                                              uint32_t k_first, uint32_t stride, int dim, int elems, int group,
                                              uint32_t* __restrict__ rows_out) {
  __shared__ unsigned long long s_id[kMissEntries];
  __shared__ uint32_t s_pos[kMissEntries], s_row[kMissEntries], s_state[kMissEntries];
  __shared__ uint32_t s_wave[kMissWaves];
  const int lane = wave_lane();
  const int wave = threadIdx.x / kWave;
  const int gl4 = threadIdx.x & (kBucket - 1);
  const int entry = threadIdx.x / kBucket;
  const int gl = threadIdx.x & (group - 1);
  for (uint32_t k0 = k_first; k0 < count; k0 += stride) {
    const uint32_t k = k0 + (uint32_t)entry;
    const bool active = k < count;
    const uint32_t pos = active ? position_of(k) : 0u;
    const uint64_t id = active ? ids[pos] : 0;
    bool won = false;
    Slot* slot = nullptr;
    int src = lane;
    ProbeResult pr = probe_insert_impl<true>(tv, id, active, gl4, kBucket, won, slot, src);
    // one addition for the workgroup: the wavefronts' counts meet in LDS
    const unsigned long long winners = __ballot(won);
    if (lane == 0) s_wave[wave] = (uint32_t)__popcll(winners);
    __syncthreads();
    if (wave == 0) {
      const uint32_t mine = lane < kMissWaves ? s_wave[lane] : 0u;
      uint32_t incl = mine;
#pragma unroll
      for (int d = 1; d < kMissWaves; d <<= 1) {
        const uint32_t y = __shfl_up(incl, d);
        if (lane >= d) incl += y;
      }
      const uint32_t total = __shfl(incl, kMissWaves - 1);
      uint32_t first_row = 0;
      if (lane == 0 && total) first_row = atomicAdd(&tv.counters[0], total);
      first_row = __shfl(first_row, 0);
      if (lane < kMissWaves) s_wave[lane] = first_row + incl - mine;
    }
    __syncthreads();
    uint32_t new_row = kEmptyRow;
    if (won) {
      const uint32_t row = s_wave[wave] + (uint32_t)__popcll(winners & ((1ull << lane) - 1ull));
      if (row < tv.row_cap) {
        __atomic_store_n(&slot->row_epoch, (unsigned long long)row | ((unsigned long long)tv.epoch << 32),
                         __ATOMIC_RELAXED);
        tv.row_key[row] = id;
        new_row = row;
      } else {
        atomicOr(&tv.counters[1], kErrOverflow);
      }
    }
    const uint32_t numbered = __shfl(new_row, src);
    if (pr.owner) {
      pr.row = numbered;
      pr.owner = numbered != kEmptyRow;
    }
    if (gl4 == 0) {
      s_id[entry] = id;
      s_pos[entry] = pos;
      s_row[entry] = pr.row;
      s_state[entry] = (active ? 1u : 0u) | (pr.owner ? 2u : 0u) | (pr.fresh ? 4u : 0u);
      if (rows_out && active) rows_out[pos] = pr.row;
    }
    __syncthreads();
    for (int j = threadIdx.x / group; j < kMissEntries; j += kMissBlock / group) {
      const uint32_t state = s_state[j];
      if (!(state & 1u)) break;                      // the entries past the list's end come last
      const uint32_t row = s_row[j];
      const uint64_t its_id = s_id[j];
      float* rec = row == kEmptyRow ? nullptr : tv.recs + (int64_t)row * tv.stride;
      if constexpr (MODE != kInsertAndCopy) {
        if ((state & 6u) == 6u) {                    // created here: the record's first values
          const float* given = out + (int64_t)s_pos[j] * dim;
          for (int e = gl; e < elems; e += group) {
            float v[VEC];
            if constexpr (MODE == kInsertGiven) {
              vload<VEC>(given + e * VEC, v);
            } else {
              init_vec<VEC, true>(init, its_id, (int64_t)e * VEC, v);
            }
            vstore<VEC>(rec + e * VEC, v);
          }
        }
        continue;
      }
      float* dst = out + (int64_t)s_pos[j] * dim;
      for (int e = gl; e < elems; e += group) {
        float v[VEC];
        if (state & 4u) {
          // the value of a new row is a pure function of (seed, id, element): every entry that
          // meets it computes the same numbers, only the creator stores them
          init_vec<VEC, true>(init, its_id, (int64_t)e * VEC, v);
          if (state & 2u) vstore<VEC>(rec + e * VEC, v);
        } else {
          vload<VEC>(rec + e * VEC, v);
        }
        vstore_once<VEC>(dst + e * VEC, v);
      }
    }
    __syncthreads();                                   // the next trip writes the same LDS
  }
}

template <int VEC, bool ROWS_ONLY = false>
__global__ __launch_bounds__(kMissBlock) void pull_missing_kernel(TableView tv, InitK init,
                                                                  const uint64_t* __restrict__ ids,
                                                                  float* __restrict__ out,
                                                                  const uint32_t* __restrict__ todo, int parity,
                                                                  int64_t list_capacity, int dim, int elems,
                                                                  int group, uint32_t* __restrict__ rows_out = nullptr) {
  // workgroup b walks list b mod kQueues, together with the other gridDim.x / kQueues of that list
  const int q = blockIdx.x & (kQueues - 1);
  const uint32_t count = __atomic_load_n(queue_counter(tv, parity, q), __ATOMIC_RELAXED);
  if (blockIdx.x < kQueues && threadIdx.x == 0) {
    *queue_counter(tv, parity ^ 1, q) = 0u;
    // still being filled: this list's share of the request's missing ids is 0.4 % of it or more
    if ((uint64_t)count * 256u >= (uint64_t)list_capacity) note_inserting(tv);
  }
  const uint32_t* list = todo + q * list_capacity;
  insert_queued<VEC, ROWS_ONLY ? kInsertOnly : kInsertAndCopy>(tv, init, ids, out, [list](uint32_t k) { return list[k]; }, count,
                                (blockIdx.x / kQueues) * kMissEntries, (gridDim.x / kQueues) * kMissEntries, dim,
                                elems, group, rows_out);
}

// ---------------------------------------------------------------------------
// pooled pull: Pull fused with the worker's jagged sum / mean (pytorch/py/jagged_ops.cc:14-56,
// 206-236, called from pytorch/jagged_embedding.py:32-52), in two launches.
//   1. every position is probed on its own (four lanes per id, all positions in flight at once);
//      ids that are not in the table are inserted and their creator initialises the record, as
//      in pull_body; the row number of each position goes to a scratch array (a position that
//      meets a row while its creator is still numbering it leaves the entry open).
//   2. one lane group per bag adds the bag's records in position order: the first row is copied,
//      the others are added to it, exactly the reference's order, so the pooled row is
//      bit-identical to pooling the pulled rows on the host. The loads of a bag do not depend
//      on each other and are issued four at a time.
// The n pulled rows themselves are never written anywhere.
// ---------------------------------------------------------------------------
// The first launch while the table is being filled: positions are only looked up, the ones whose
// id is missing are queued as in pull_resident_kernel and inserted by pull_missing_kernel.
__global__ __launch_bounds__(kBlock) void pooled_find_kernel(TableView tv, const uint64_t* __restrict__ ids,
                                                             int64_t n, uint32_t* __restrict__ rows,
                                                             uint32_t* __restrict__ todo, int parity) {
  constexpr int per_block = kBlock / kBucket;
  const int64_t p = (int64_t)blockIdx.x * per_block + threadIdx.x / kBucket;
  const int gl = threadIdx.x & (kBucket - 1);
  const bool active = p < n;
  const uint32_t row = probe_find(tv, active ? ids[p] : 0, active, gl, kBucket);
  const bool queue = active && row == kEmptyRow && gl == 0;
  const unsigned long long votes = __ballot(queue);
  if (votes) {
    const int lane = wave_lane();
    const int first = __ffsll(votes) - 1;
    const int q = blockIdx.x & (kQueues - 1);
    uint32_t base = 0;
    if (lane == first) base = atomicAdd(queue_counter(tv, parity, q), (uint32_t)__popcll(votes));
    base = __shfl(base, first);
    if (queue)
      todo[q * queue_capacity(n, per_block) + base + (uint32_t)__popcll(votes & ((1ull << lane) - 1ull))] =
          (uint32_t)p;
  }
  if (active && gl == 0) rows[p] = row;
}

template <int VEC>
__global__ __launch_bounds__(kBlock) void pooled_probe_kernel(TableView tv, InitK init,
                                                              const uint64_t* __restrict__ ids, int64_t n,
                                                              uint32_t* __restrict__ rows, int elems) {
  const int64_t p = (int64_t)blockIdx.x * (kBlock / kBucket) + threadIdx.x / kBucket;
  const int gl = threadIdx.x & (kBucket - 1);
  const bool active = p < n;
  const uint64_t id = active ? ids[p] : 0;
  const ProbeResult pr = probe_insert(tv, id, active, gl, kBucket);
  if (__popcll(__ballot(active && pr.owner && gl == 0)) >= kFillingIds && wave_lane() == 0) note_inserting(tv);
  if (!active) return;
  if (pr.fresh && pr.owner && pr.row != kEmptyRow) {
    float* rec = tv.recs + (int64_t)pr.row * tv.stride;
    for (int e = gl; e < elems; e += kBucket) {
      float v[VEC];
      init_vec<VEC>(init, id, (int64_t)e * VEC, v);
      vstore<VEC>(rec + e * VEC, v);
    }
  }
  if (gl == 0) rows[p] = pr.row;
}

constexpr int kPoolAhead = 4;   // records of one bag requested together

template <int VEC>
__global__ __launch_bounds__(kBlock) void pooled_sum_kernel(TableView tv, const uint32_t* __restrict__ rows,
                                                            const uint64_t* __restrict__ ids,
                                                            int64_t n, const long long* __restrict__ offsets,
                                                            int64_t bags, const float* __restrict__ weights,
                                                            int mean, float patch, float* __restrict__ out,
                                                            int dim, int elems, int group) {
  const int per_block = kBlock / group;
  const int64_t bag = (int64_t)blockIdx.x * per_block + threadIdx.x / group;
  const int gl = threadIdx.x & (group - 1);
  if (bag >= bags || gl >= elems) return;      // the host only launches this with elems <= group
  long long lo = offsets[bag], hi = offsets[bag + 1];
  if (lo < 0) lo = 0;
  if (hi > n) hi = n;
  float acc[VEC];
#pragma unroll
  for (int c = 0; c < VEC; ++c) acc[c] = patch;
  for (long long j0 = lo; j0 < hi; j0 += kPoolAhead) {
    float v[kPoolAhead][VEC];
    float w[kPoolAhead];
#pragma unroll
    for (int u = 0; u < kPoolAhead; ++u) {
      const long long j = j0 + u;
      uint32_t row = j < hi ? rows[j] : kEmptyRow;
      // A position that met its id while another position's group was still creating the row
      // could not learn the row number in the first launch; by now it is in the index.
      if (j < hi && row == kEmptyRow) row = probe_find_alone(tv, ids[j]);
      w[u] = (weights && j < hi) ? weights[j] : 1.0f;
      if (row != kEmptyRow) {
        vload<VEC>(tv.recs + (int64_t)row * tv.stride + gl * VEC, v[u]);
      } else {
#pragma unroll
        for (int c = 0; c < VEC; ++c) v[u][c] = 0.0f;
      }
    }
#pragma unroll
    for (int u = 0; u < kPoolAhead; ++u) {
      const long long j = j0 + u;
      if (j >= hi) break;
#pragma unroll
      for (int c = 0; c < VEC; ++c) {
        // pytorch/jagged_embedding.py:41-45 scales the rows before pooling
        const float x = weights ? v[u][c] * w[u] : v[u][c];
        acc[c] = j == lo ? x : acc[c] + x;
      }
    }
  }
  if (mean && hi > lo) {
    const float ratio = (float)(1.0 / (double)(float)(hi - lo));   // jagged_ops.cc:219
#pragma unroll
    for (int c = 0; c < VEC; ++c) acc[c] = acc[c] * ratio;
  }
  vstore_once<VEC>(out + bag * (int64_t)dim + gl * VEC, acc);
}

template <int OPT, int VEC>
__global__ __launch_bounds__(kBlock) void push_kernel(TableView tv, const uint64_t* __restrict__ ids,
                                                      int64_t n, const float* __restrict__ grads,
                                                      int dim, int elems, int group, float lr,
                                                      OptimK k, PushCols pc,
                                                      const uint32_t* __restrict__ notes) {
  const int per_block = kBlock / group;
  const int64_t i = (int64_t)blockIdx.x * per_block + threadIdx.x / group;
  push_body<OPT, VEC>(tv, ids, i, i < n, threadIdx.x & (group - 1), grads, dim, elems, group, lr, k, pc, notes);
}

// ---- pulls of rows 32 to 128 floats wide -------------------------------------------------------
// With one lane group of dim / 4 lanes per id from the search on, a wavefront of a wide table
// looks up only two to eight ids at a time, and a pull is then bound by how few index buckets
// are on their way. Here the search and the copy use different lane mappings: a wavefront takes
// sixteen ids, four lanes search for each (all sixteen buckets requested at once), and then its
// lane groups of dim / 4 lanes copy the sixteen rows, several at a time, taking each row's number
// from the lanes that found it. INSERT: missing ids are inserted and initialised as in pull_body;
// otherwise they are queued for pull_missing_kernel as in pull_resident_kernel.
constexpr int kWideIds = kWave / kBucket;        // ids a wavefront takes: 16

// STEPS: the copy's trips, 2, 4 or 8 for lane groups of 8, 16 or 32 lanes (a template argument so
// that a lane holds STEPS slices and not eight: the fused kernel for rows of 32 and 64 floats then
// keeps all wavefronts of a 98k-id request on the chip at once instead of five sixths of them).
template <int VEC, bool INSERT, int STEPS>
__device__ __forceinline__ void pull_wide(const TableView& tv, const InitK& init,
                                          const uint64_t* __restrict__ ids, int64_t first, int64_t end,
                                          float* __restrict__ out, int dim, int elems,
                                          uint32_t* __restrict__ todo, int parity,
                                          uint32_t* __restrict__ notes = nullptr,
                                          int filling_ids = kFillingIds) {
  const int lane = wave_lane();
  const int gl4 = lane & (kBucket - 1);
  const int64_t i = first + (lane >> 2);
  const bool active = i < end;
  const uint64_t id = active ? ids[i] : 0;
  const FindResult f = probe_find_slot(tv, id, active, gl4, kBucket);
  ProbeResult pr;
  pr.row = (uint32_t)f.row_epoch;
  pr.owner = false;
  pr.fresh = pr.row == kEmptyRow || (uint32_t)(f.row_epoch >> 32) == tv.epoch;
  const bool miss = active && !f.found;
  bool copy = active;
  if constexpr (INSERT) {
    if (__any(miss)) {
      const ProbeResult q = probe_insert(tv, id, miss, gl4, kBucket);
      if (miss) pr = q;
      if (__popcll(__ballot(miss && gl4 == 0)) >= filling_ids && lane == 0) note_inserting(tv);
    }
    // where the id lives, for a push of the same ids that follows (kEmptyRow: the table is full)
    if (notes && active && gl4 == 0) notes[i] = pr.row;
  } else {
    // one atomic per wavefront reserves entries of the workgroup's list for all of its missing ids
    // (here `end` is the request's length: the lists' capacity follows from it)
    const bool queue = miss && gl4 == 0;
    const unsigned long long votes = __ballot(queue);
    if (votes) {
      const int leader = __ffsll(votes) - 1;
      const int q = blockIdx.x & (kQueues - 1);
      uint32_t base = 0;
      if (lane == leader) base = atomicAdd(queue_counter(tv, parity, q), (uint32_t)__popcll(votes));
      base = __shfl(base, leader);
      if (queue)
        todo[q * queue_capacity(end, (int)(blockDim.x / kWave) * kWideIds) + base +
             (uint32_t)__popcll(votes & ((1ull << lane) - 1ull))] = (uint32_t)i;
    }
    copy = active && f.found;
    pr.fresh = false;                              // nothing is created here: what was found is read
    if (notes && copy && gl4 == 0) notes[i] = pr.row;   // a missing id's note: by the launch that inserts it
  }
  // the copy: lane group `sub` of the wavefront takes ids sub, sub + rows_per_step, ...
  constexpr int rows_per_step = kWideIds / STEPS;   // 8, 4 or 2
  constexpr int group = kWave / rows_per_step;      // 8, 16 or 32
  const int sub = lane / group;
  const int gl = lane & (group - 1);
  const uint32_t id_lo = (uint32_t)id, id_hi = (uint32_t)(id >> 32);
  float v[STEPS][VEC];
  uint32_t live = 0;                             // bit s: this lane has a slice of step s to store
#pragma unroll
  for (int s = 0; s < STEPS; ++s) {
    {
      const int src = kBucket * (s * rows_per_step + sub);
      const uint32_t row = __shfl(pr.row, src);
      const int fresh = __shfl((int)pr.fresh, src);
      const int owner = __shfl((int)pr.owner, src);
      const int on = __shfl((int)copy, src);
      const uint64_t its_id = (uint64_t)__shfl(id_lo, src) | ((uint64_t)__shfl(id_hi, src) << 32);
      if (on && gl < elems) {
        float* rec = row == kEmptyRow ? nullptr : tv.recs + (int64_t)row * tv.stride;
        if (fresh) {
          // the value of a new row is a pure function of (seed, id, element): every group that
          // meets it computes the same numbers, only the creator stores them
          init_vec<VEC>(init, its_id, (int64_t)gl * VEC, v[s]);
          if (owner) vstore<VEC>(rec + gl * VEC, v[s]);
        } else {
          vload<VEC>(rec + gl * VEC, v[s]);
        }
        live |= 1u << s;
      }
    }
  }
#pragma unroll
  for (int s = 0; s < STEPS; ++s) {
    if (live & (1u << s)) {
      const int64_t p = first + s * rows_per_step + sub;
      vstore_once<VEC>(out + p * (int64_t)dim + gl * VEC, v[s]);
    }
  }
}

// whether a table's rows take the wide pull: lane groups of 8 to 32 lanes that hold a whole row
__host__ __device__ inline bool pull_is_wide(int group, int elems) {
  return group >= 8 && group <= 32 && elems <= group;
}

// ---- pushes of rows 20 to 64 floats wide --------------------------------------------------------
// The same split for the push: sixteen ids searched per wavefront with four lanes each, then lane
// groups of 4 * STEPS lanes (8 or 16: a whole row each) update the sixteen records,
// 16 / STEPS rows per step. The sixteen gradient rows are one contiguous block that does not
// depend on the index and is requested before the search; every line of a step's records is
// requested before the first optimizer operation on them. One step's records at a time: with
// two or four steps' loads issued together the wavefronts of a launch (six per SIMD for 98k ids,
// all resident at once) read in one burst and write in the next, and a 64-float Adagrad push of
// 98k rows takes 29.1 or 31.8 us instead of 28.8.
template <int OPT, int STEPS>
__device__ __forceinline__ void push_wide(const TableView& tv, const uint64_t* __restrict__ ids,
                                          int64_t first, int64_t end, const float* __restrict__ grads,
                                          int dim, int elems, float lr, const OptimK& k,
                                          const PushCols& pc, const uint32_t* __restrict__ notes = nullptr) {
  constexpr int VEC = 4;
  constexpr int rows_per_step = kWideIds / STEPS;   // 8, 4 or 2
  constexpr int group = kWave / rows_per_step;      // 8, 16 or 32
  constexpr bool more_states = OPT == KRK_ADAM || OPT == KRK_RMSPROP;
  const int lane = wave_lane();
  const int sub = lane / group;
  const int gl = lane & (group - 1);
  const bool part = gl < elems;
  float gv[STEPS][VEC];
#pragma unroll
  for (int s = 0; s < STEPS; ++s) {
    const int64_t p = first + s * rows_per_step + sub;
#pragma unroll
    for (int c = 0; c < VEC; ++c) gv[s][c] = 0.0f;
    if (part && p < end) vload_once<VEC>(grads + p * (int64_t)dim + gl * VEC, gv[s]);
  }
  const int64_t i = first + (lane >> 2);
  const bool active = i < end;
  const uint32_t my_row = row_for_push(tv, ids, i, active, lane & (kBucket - 1), kBucket, notes);
  if (active && my_row == kEmptyRow && (lane & (kBucket - 1)) == 0) atomicOr(&tv.counters[1], kErrMissingId);
#pragma unroll
  for (int s = 0; s < STEPS; ++s) {
    const uint32_t row = __shfl(my_row, kBucket * (s * rows_per_step + sub));
    if (row == kEmptyRow) continue;                 // a position past the end, or an id the table lacks
    float* rec = tv.recs + (int64_t)row * tv.stride;
    float w[VEC], s0[VEC], s1[VEC], s2[VEC];        // s1, s2 stay zero and unused for SGD and Adagrad
#pragma unroll
    for (int c = 0; c < VEC; ++c) w[c] = s0[c] = s1[c] = s2[c] = 0.0f;
    if (part) {
      vload<VEC>(rec + gl * VEC, w);
      if (pc.c0 >= 0) vload<VEC>(rec + pc.c0 + gl * VEC, s0);
      if constexpr (more_states) {
        if (pc.c1 >= 0) vload<VEC>(rec + pc.c1 + gl * VEC, s1);
        if (pc.c2 >= 0) vload<VEC>(rec + pc.c2 + gl * VEC, s2);
      }
    }
    bool first_update = false;
    float bc1 = 1.0f, bc2 = 1.0f;
    uint64_t steps = 0;
    if (pc.meta >= 0) {
      const uint32_t* meta = reinterpret_cast<const uint32_t*>(rec + pc.meta);
      steps = (uint64_t)meta[0] | ((uint64_t)meta[1] << 32);
      if (OPT == KRK_ADAM) {
        // ps/optim/adam.cc:61-64 : per-row step counter, float pow, double subtraction
        steps += 1;                                 // the flag bit rides along untouched
        const float count = (float)(steps & ~kHasMomentumBit);
        bc1 = (float)(1.0 - (double)powf(k.beta1, count));
        bc2 = (float)(1.0 - (double)powf(k.beta2, count));
      } else {
        first_update = (steps & kHasMomentumBit) == 0;
        steps |= kHasMomentumBit;
      }
    }
    if (part) {
#pragma unroll
      for (int c = 0; c < VEC; ++c)
        optim_element<OPT>(k, lr, gv[s][c], w[c], s0[c], s1[c], s2[c], first_update, bc1, bc2);
      // written once per launch and not read again by it: past the caches
      vstore_once<VEC>(rec + gl * VEC, w);
      if (pc.c0 >= 0) vstore_once<VEC>(rec + pc.c0 + gl * VEC, s0);
      if constexpr (more_states) {
        if (pc.c1 >= 0) vstore_once<VEC>(rec + pc.c1 + gl * VEC, s1);
        if (pc.c2 >= 0) vstore_once<VEC>(rec + pc.c2 + gl * VEC, s2);
      }
    }
    if (pc.meta >= 0) store_row_word<VEC>(rec + pc.meta, steps, gl, dim, (int)tv.stride - pc.meta);
  }
}

// whether a table's rows take the wide push: whole rows of up to 64 floats in 16-byte lane
// accesses. (Rows of 65 to 128 floats gain nothing from it: a million of them are pushed in
// 547 us against 535 us with one lane group per id from the search on.)
__host__ __device__ inline bool push_is_wide(int vec, int group, int elems) {
  return vec == 4 && pull_is_wide(group, elems) && group <= 16;
}

template <int OPT, int STEPS>
__global__ __launch_bounds__(kBlock) void push_wide_kernel(TableView tv, const uint64_t* __restrict__ ids,
                                                           int64_t n, const float* __restrict__ grads,
                                                           int dim, int elems, float lr, OptimK k,
                                                           PushCols pc, const uint32_t* __restrict__ notes) {
  const int64_t first = ((int64_t)blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave) * kWideIds;
  if (first >= n) return;                        // the whole wavefront
  push_wide<OPT, STEPS>(tv, ids, first, n, grads, dim, elems, lr, k, pc, notes);
}

template <int VEC, int STEPS>
__global__ __launch_bounds__(kBlock) void pull_wide_kernel(TableView tv, InitK init,
                                                           const uint64_t* __restrict__ ids, int64_t n,
                                                           float* __restrict__ out, int dim, int elems,
                                                           uint32_t* __restrict__ notes) {
  const int64_t first = ((int64_t)blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave) * kWideIds;
  if (first >= n) return;                        // the whole wavefront
  pull_wide<VEC, true, STEPS>(tv, init, ids, first, n, out, dim, elems, nullptr, 0, notes);
}

template <int VEC, int STEPS>
__global__ __launch_bounds__(kBlock) void pull_resident_wide_kernel(TableView tv,
                                                                    const uint64_t* __restrict__ ids,
                                                                    int64_t n, float* __restrict__ out,
                                                                    uint32_t* __restrict__ todo, int parity,
                                                                    int dim, int elems,
                                                                    uint32_t* __restrict__ notes) {
  const int64_t first = ((int64_t)blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave) * kWideIds;
  if (first >= n) return;
  InitK none{};
  pull_wide<VEC, false, STEPS>(tv, none, ids, first, n, out, dim, elems, todo, parity, notes);
}

// ---- one launch over several tables of equal row width ------------------------
// Table t owns workgroups [block_start[t], block_start[t+1]) and the positions
// [row_start[t], row_start[t+1]) of the concatenated ids / rows.
__device__ __forceinline__ int find_table(const GroupCall& c, uint32_t bx) {
  if (c.even_blocks) return (int)(bx / c.even_blocks);
  int t = 0;
  while (t + 1 < c.n_tables && bx >= c.block_start[t + 1]) ++t;
  return t;
}
__device__ __forceinline__ int find_table(const GroupCall& c) { return find_table(c, blockIdx.x); }

template <int VEC>
__global__ __launch_bounds__(kBlock) void group_pull_kernel(const TableDesc* __restrict__ descs,
                                                            GroupCall call,
                                                            const uint64_t* __restrict__ ids,
                                                            float* __restrict__ out, int dim, int elems,
                                                            int group, uint32_t* __restrict__ notes) {
  const int t = find_table(call);
  TableView tv = descs[t].tv;
  tv.epoch = call.epoch[t];
  const InitK init = descs[t].init;
  const int per_block = kBlock / group;
  const int64_t local = (int64_t)(blockIdx.x - call.block_start[t]) * per_block + threadIdx.x / group;
  const int64_t i = call.row_start[t] + local;
  pull_body<VEC>(tv, init, ids, i, i < call.row_start[t + 1], threadIdx.x & (group - 1), out, dim,
                 elems, group, notes, kFillingIdsCombined);
}

// the same for rows 32 to 128 floats wide: a workgroup takes 64 positions of its table
template <int VEC, int STEPS>
__global__ __launch_bounds__(kBlock) void group_pull_wide_kernel(const TableDesc* __restrict__ descs,
                                                                 GroupCall call,
                                                                 const uint64_t* __restrict__ ids,
                                                                 float* __restrict__ out, int dim,
                                                                 int elems, uint32_t* __restrict__ notes) {
  const int t = find_table(call);
  TableView tv = descs[t].tv;
  tv.epoch = call.epoch[t];
  const InitK init = descs[t].init;
  const int64_t local = ((int64_t)(blockIdx.x - call.block_start[t]) * (blockDim.x / kWave) + threadIdx.x / kWave) *
                        kWideIds;
  const int64_t first = call.row_start[t] + local;
  if (first >= call.row_start[t + 1]) return;    // the whole wavefront
  pull_wide<VEC, true, STEPS>(tv, init, ids, first, call.row_start[t + 1], out, dim, elems, nullptr, 0, notes,
                              kFillingIdsCombined);
}

// ---- combined pulls while the members' tables are being filled ---------------------------------
// The two launches of a large pull, member by member: the first looks up and copies and queues
// the positions whose id is missing in the member's own lists (positions count from the member's
// first), the second gives every member kGroupMissPerTable workgroups of 1024 lanes that walk
// four lists each. The fused kernels add to a member's row counter once per wavefront that
// inserts: 98.6k new ids over 26 tables took 67 us that way against 9 us resident.
constexpr int kGroupMissPerTable = 16;
static_assert(kQueues % kGroupMissPerTable == 0, "every workgroup walks the same number of lists");

template <int VEC>
__global__ __launch_bounds__(kBlock) void group_pull_resident_kernel(const TableDesc* __restrict__ descs,
                                                                     GroupCall call, GroupFill fill,
                                                                     const uint64_t* __restrict__ ids,
                                                                     float* __restrict__ out,
                                                                     uint32_t* __restrict__ todo, int dim,
                                                                     int elems, int group,
                                                                     uint32_t* __restrict__ notes) {
  const uint32_t bx = blockIdx.x;
  const int t = find_table(call, bx);
  const int64_t a = call.row_start[t];
  pull_resident_body<VEC>(descs[t].tv, ids + a, call.row_start[t + 1] - a, out + a * dim,
                          todo + fill.todo_start[t], (int)((fill.parity_bits >> t) & 1u), dim, elems, group,
                          bx - call.block_start[t], notes ? notes + a : nullptr);
}

template <int VEC, int STEPS>
__global__ __launch_bounds__(kBlock) void group_pull_resident_wide_kernel(const TableDesc* __restrict__ descs,
                                                                          GroupCall call, GroupFill fill,
                                                                          const uint64_t* __restrict__ ids,
                                                                          float* __restrict__ out,
                                                                          uint32_t* __restrict__ todo, int dim,
                                                                          int elems, uint32_t* __restrict__ notes) {
  const uint32_t bx = blockIdx.x;
  const int t = find_table(call, bx);
  const int64_t a = call.row_start[t];
  const int64_t n = call.row_start[t + 1] - a;
  const int64_t first = ((int64_t)(bx - call.block_start[t]) * (blockDim.x / kWave) + threadIdx.x / kWave) * kWideIds;
  if (first >= n) return;                        // the whole wavefront
  InitK none{};
  pull_wide<VEC, false, STEPS>(descs[t].tv, none, ids + a, first, n, out + a * dim, dim, elems,
                               todo + fill.todo_start[t], (int)((fill.parity_bits >> t) & 1u),
                               notes ? notes + a : nullptr);
}

template <int VEC>
__global__ __launch_bounds__(kMissBlock) void group_pull_missing_kernel(const TableDesc* __restrict__ descs,
                                                                        GroupCall call, GroupFill fill,
                                                                        const uint64_t* __restrict__ ids,
                                                                        float* __restrict__ out,
                                                                        const uint32_t* __restrict__ todo,
                                                                        int per_block, int dim, int elems,
                                                                        int group, uint32_t* __restrict__ notes) {
  const int t = blockIdx.x / kGroupMissPerTable;
  const int w = blockIdx.x % kGroupMissPerTable;
  const int64_t a = call.row_start[t];
  const int64_t n = call.row_start[t + 1] - a;
  if (n <= 0) return;                              // a member without ids: its lists were not used
  TableView tv = descs[t].tv;
  tv.epoch = call.epoch[t];
  const InitK init = descs[t].init;
  const int parity = (int)((fill.parity_bits >> t) & 1u);
  const int64_t capacity = queue_capacity(n, per_block);
  const uint32_t* lists = todo + fill.todo_start[t];
  // the workgroup's lists w, w + 16, ... as one: a member's lists are short (a sixty-fourth of
  // its missing ids each), and a trip costs the same whether its 256 entries are all there or not
  constexpr int kMine = kQueues / kGroupMissPerTable;
  uint32_t upto[kMine];                              // entries in the workgroup's first j + 1 lists
  uint32_t total = 0;
#pragma unroll
  for (int j = 0; j < kMine; ++j) {
    const int q = w + j * kGroupMissPerTable;
    total += __atomic_load_n(queue_counter(tv, parity, q), __ATOMIC_RELAXED);
    upto[j] = total;
    if (threadIdx.x == 0) *queue_counter(tv, parity ^ 1, q) = 0u;
  }
  // still being filled: the workgroup holds a sixteenth of the member's missing ids; a fifth of the
  // member's ids or more are missing
  if (threadIdx.x == 0 && (uint64_t)total * (5u * kGroupMissPerTable) >= (uint64_t)n) note_inserting(tv);
  auto position_of = [&](uint32_t k) {
    int j = 0;
#pragma unroll
    for (int i = 0; i + 1 < kMine; ++i) j += k >= upto[i] ? 1 : 0;
    return lists[(int64_t)(w + j * kGroupMissPerTable) * capacity + (k - (j ? upto[j - 1] : 0u))];
  };
  insert_queued<VEC, kInsertAndCopy>(tv, init, ids + a, out + a * dim, position_of, total, 0u, kMissEntries, dim,
                                     elems, group, notes ? notes + a : nullptr);
}

template <int OPT, int VEC>
__global__ __launch_bounds__(kBlock) void group_push_kernel(const TableDesc* __restrict__ descs,
                                                            GroupCall call,
                                                            const uint64_t* __restrict__ ids,
                                                            const float* __restrict__ grads, int dim,
                                                            int elems, int group, float lr, OptimK k,
                                                            int st0, int st1, int st2, int use_meta,
                                                            const uint32_t* __restrict__ notes) {
  const uint32_t bx = blockIdx.x;
  const int t = find_table(call, bx);
  const TableView tv = descs[t].tv;
  PushCols pc;
  pc.c0 = st0 >= 0 ? descs[t].col_off[st0] : -1;
  pc.c1 = st1 >= 0 ? descs[t].col_off[st1] : -1;
  pc.c2 = st2 >= 0 ? descs[t].col_off[st2] : -1;
  pc.meta = use_meta ? descs[t].meta_off : -1;
  const int per_block = kBlock / group;
  const int64_t local = (int64_t)(bx - call.block_start[t]) * per_block + threadIdx.x / group;
  const int64_t i = call.row_start[t] + local;
  push_body<OPT, VEC>(tv, ids, i, i < call.row_start[t + 1], threadIdx.x & (group - 1), grads, dim,
                      elems, group, lr, k, pc, notes);
}

// the same for rows 32 to 128 floats wide: a workgroup takes 64 positions of its table
template <int OPT, int STEPS>
__global__ __launch_bounds__(kBlock) void group_push_wide_kernel(const TableDesc* __restrict__ descs,
                                                                 GroupCall call,
                                                                 const uint64_t* __restrict__ ids,
                                                                 const float* __restrict__ grads, int dim,
                                                                 int elems, float lr, OptimK k, int st0,
                                                                 int st1, int st2, int use_meta,
                                                                 const uint32_t* __restrict__ notes) {
  const uint32_t bx = blockIdx.x;
  const int t = find_table(call, bx);
  const TableView tv = descs[t].tv;
  PushCols pc;
  pc.c0 = st0 >= 0 ? descs[t].col_off[st0] : -1;
  pc.c1 = st1 >= 0 ? descs[t].col_off[st1] : -1;
  pc.c2 = st2 >= 0 ? descs[t].col_off[st2] : -1;
  pc.meta = use_meta ? descs[t].meta_off : -1;
  const int64_t local = ((int64_t)(bx - call.block_start[t]) * (blockDim.x / kWave) + threadIdx.x / kWave) *
                        kWideIds;
  const int64_t first = call.row_start[t] + local;
  if (first >= call.row_start[t + 1]) return;    // the whole wavefront
  push_wide<OPT, STEPS>(tv, ids, first, call.row_start[t + 1], grads, dim, elems, lr, k, pc, notes);
}

__global__ __launch_bounds__(kBlock) void lookup_kernel(TableView tv, const uint64_t* __restrict__ ids,
                                                        int64_t n, int32_t* __restrict__ rows) {
  const int64_t i = (int64_t)blockIdx.x * (kBlock / kBucket) + threadIdx.x / kBucket;
  const int gl = threadIdx.x & (kBucket - 1);
  const bool active = i < n;
  const uint32_t r = probe_find(tv, active ? ids[i] : 0, active, gl, kBucket);
  if (active && gl == 0) rows[i] = r == kEmptyRow ? -1 : (int32_t)r;
}

// import: like pull, but a new row takes its values from the caller. Workgroups of 1024 lanes
// take 256 ids each and number the rows they make with one addition to the row counter (a
// checkpoint of 1e8 rows 32 floats wide is 12.5 million wavefronts of the table kernels' size).
template <int VEC>
__global__ __launch_bounds__(kMissBlock) void import_kernel(TableView tv, const uint64_t* __restrict__ ids,
                                                            int64_t n, const float* __restrict__ vals,
                                                            int dim, int elems, int group) {
  InitK none{};
  insert_queued<VEC, kInsertGiven>(tv, none, ids, const_cast<float*>(vals), [](uint32_t k) { return k; },
                                   (uint32_t)n, blockIdx.x * kMissEntries, gridDim.x * kMissEntries, dim, elems,
                                   group, nullptr);
}

// {rows used, launch number} of up to 32 tables -> pinned host memory. Runs behind the launch
// whose number it carries, so the count is exact as of that launch. The store is a relaxed
// system-scope atomic: only the value itself has to arrive, nothing is ordered behind it.
struct PublishArgs {
  int32_t n;
  uint32_t epoch[kMaxGroupTables];
  const uint32_t* counters[kMaxGroupTables];
  unsigned long long* host_pub[kMaxGroupTables];
};
__global__ void publish_kernel(PublishArgs a) {
  const int i = threadIdx.x;
  if (i >= a.n) return;
  const uint32_t rows = a.counters[i][0];
  __hip_atomic_store(a.host_pub[i], (unsigned long long)rows | ((unsigned long long)a.epoch[i] << 32),
                     __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// export: rows in insertion order
__global__ __launch_bounds__(kBlock) void export_kernel(TableView tv, int64_t rows, int dim,
                                                        unsigned long long* __restrict__ ids,
                                                        float* __restrict__ vals, int state_off,
                                                        float* __restrict__ state, int meta_off,
                                                        long long* __restrict__ steps) {
  const int64_t total = rows * dim;
  const int64_t step = (int64_t)gridDim.x * kBlock;   // grid-stride: see restride_kernel
  for (int64_t t = (int64_t)blockIdx.x * kBlock + threadIdx.x; t < total; t += step) {
    const int64_t r = t / dim;
    const int j = (int)(t - r * dim);
    const float* rec = tv.recs + r * tv.stride;
    if (vals) vals[t] = rec[j];
    if (state) state[t] = state_off >= 0 ? rec[state_off + j] : 0.0f;
    if (j == 0) {
      if (ids) ids[r] = tv.row_key[r];
      if (steps) {
        long long s = 0;
        if (meta_off >= 0) {
          const uint32_t* meta = reinterpret_cast<const uint32_t*>(rec + meta_off);
          s = (long long)(((uint64_t)meta[0] | ((uint64_t)meta[1] << 32)) & ~kHasMomentumBit);
        }
        steps[r] = s;
      }
    }
  }
}

// fetch: the rows of the ids that exist, nothing inserted (ps/ps.cc:914-935)
template <int VEC>
__global__ __launch_bounds__(kBlock) void fetch_kernel(TableView tv, const uint64_t* __restrict__ ids,
                                                       int64_t n, unsigned char* __restrict__ found,
                                                       float* __restrict__ vals, int state_off,
                                                       float* __restrict__ state, int meta_off,
                                                       long long* __restrict__ steps, bool raw_word,
                                                       int dim, int elems, int group) {
  const int per_block = kBlock / group;
  const int64_t i = (int64_t)blockIdx.x * per_block + threadIdx.x / group;
  const int gl = threadIdx.x & (group - 1);
  const bool active = i < n;
  const uint32_t row = probe_find(tv, active ? ids[i] : 0, active, gl, group);
  if (!active) return;
  const bool hit = row != kEmptyRow;
  const float* rec = hit ? tv.recs + (int64_t)row * tv.stride : nullptr;
  if (gl == 0) {
    if (found) found[i] = hit ? 1 : 0;
    if (steps) {
      long long s = 0;
      if (hit && meta_off >= 0) {
        const uint32_t* meta = reinterpret_cast<const uint32_t*>(rec + meta_off);
        const uint64_t word = (uint64_t)meta[0] | ((uint64_t)meta[1] << 32);
        s = (long long)(raw_word ? word : word & ~kHasMomentumBit);
      }
      steps[i] = s;
    }
  }
  for (int e = gl; e < elems; e += group) {
    float v[VEC];
#pragma unroll
    for (int c = 0; c < VEC; ++c) v[c] = 0.0f;
    if (vals) {
      if (hit) vload<VEC>(rec + e * VEC, v);
      vstore<VEC>(vals + i * (int64_t)dim + e * VEC, v);
    }
    if (state) {
#pragma unroll
      for (int c = 0; c < VEC; ++c) v[c] = 0.0f;
      if (hit && state_off >= 0) vload<VEC>(rec + state_off + e * VEC, v);
      vstore<VEC>(state + i * (int64_t)dim + e * VEC, v);
    }
  }
}

// import_state: optimizer state and step counters of rows that exist (checkpoint load,
// transfer-in: checkpoint/checkpoint.cc:620-645 inserts whole Values)
template <int VEC>
__global__ __launch_bounds__(kBlock) void import_state_kernel(TableView tv, const uint64_t* __restrict__ ids,
                                                              int64_t n, int state_off,
                                                              const float* __restrict__ state, int meta_off,
                                                              const long long* __restrict__ steps,
                                                              bool mark_momentum, int dim, int elems,
                                                              int group) {
  const int per_block = kBlock / group;
  const int64_t i = (int64_t)blockIdx.x * per_block + threadIdx.x / group;
  const int gl = threadIdx.x & (group - 1);
  const bool active = i < n;
  const uint32_t row = probe_find(tv, active ? ids[i] : 0, active, gl, group);
  if (!active) return;
  if (row == kEmptyRow) {
    if (gl == 0) atomicOr(&tv.counters[1], kErrMissingId);
    return;
  }
  float* rec = tv.recs + (int64_t)row * tv.stride;
  if (state) {
    for (int e = gl; e < elems; e += group) {
      float v[VEC];
      vload<VEC>(state + i * (int64_t)dim + e * VEC, v);
      vstore<VEC>(rec + state_off + e * VEC, v);
    }
  }
  if ((steps || mark_momentum) && gl == 0) {
    // a count replaces the count, a momentum buffer sets the flag: neither disturbs the other
    uint32_t* meta = reinterpret_cast<uint32_t*>(rec + meta_off);
    unsigned long long s = (unsigned long long)meta[0] | ((unsigned long long)meta[1] << 32);
    if (steps) s = (s & kHasMomentumBit) | ((unsigned long long)steps[i] & ~kHasMomentumBit);
    if (mark_momentum) s |= kHasMomentumBit;
    meta[0] = (uint32_t)s;
    meta[1] = (uint32_t)(s >> 32);
  }
}

// ---- which rows a node of the cluster owns ------------------------------------------------------
// common/utils.h:30-44: the mixer behind utils::Hash, which routes rows to servers.
__host__ __device__ inline unsigned long long route_hash64(unsigned long long v) {
  v = v * 3935559000370003845ull + 2691343689449507681ull;
  v ^= v >> 21;
  v ^= v << 37;
  v ^= v >> 4;
  v *= 4768777513237032717ull;
  v ^= v << 20;
  v ^= v >> 41;
  v ^= v << 5;
  return v;
}

// Rings of up to this many virtual nodes are searched in LDS (the same 512 or so entries are looked
// at by every id: nine dependent reads that should not go to memory each time).
constexpr int kRingLds = 2048;

// First virtual node at or above `hv`, or the ring's first when hv lies above them all.
__device__ __forceinline__ int ring_position(const unsigned long long* ring, int m, unsigned long long hv) {
  int lo = 0, hi = m;
  while (lo < hi) {
    const int mid = lo + ((hi - lo) >> 1);
    if (ring[mid] < hv) lo = mid + 1; else hi = mid;
  }
  return lo == m ? 0 : lo;
}

// the ring's hashes into LDS when they fit (-> true); every thread of the workgroup calls this.
// The callers search `lds` or `ring_hash` by name, each in its own branch: through one pointer
// that may be either, every read of the search would be a flat access instead of an LDS read.
__device__ __forceinline__ bool stage_ring(unsigned long long* lds, const unsigned long long* __restrict__ ring_hash,
                                           int m) {
  if (m > kRingLds) return false;
  for (int i = threadIdx.x; i < m; i += kBlock) lds[i] = ring_hash[i];
  __syncthreads();
  return true;
}

// flag[r] = 1 where Router::Hit(utils::Hash(table_id, id of row r)) (common/router.cc:262-277,
// common/utils.h:46-48) is node_id (want_owned) or another node (!want_owned). The ring is the
// virtual nodes in ascending hash order: a hash belongs to the first one at or above it, or to
// the first of the ring when it lies above them all; an empty ring owns nothing.
__global__ __launch_bounds__(kBlock) void route_flag_kernel(const unsigned long long* __restrict__ row_key,
                                                            int64_t rows, unsigned long long table_hash,
                                                            const unsigned long long* __restrict__ ring_hash,
                                                            const unsigned long long* __restrict__ ring_node,
                                                            int m, unsigned long long node_id, bool want_owned,
                                                            int32_t* __restrict__ flag) {
  __shared__ unsigned long long sring[kRingLds];
  const bool in_lds = stage_ring(sring, ring_hash, m);
  // a workgroup walks several stretches of rows, so the ring is staged once for many rows
  const int64_t step = (int64_t)gridDim.x * kBlock;
  for (int64_t r = (int64_t)blockIdx.x * kBlock + threadIdx.x; r < rows; r += step) {
    const unsigned long long hv = table_hash ^ route_hash64(__builtin_nontemporal_load(row_key + r));
    unsigned long long owner = ~0ull;
    if (m > 0) owner = ring_node[in_lds ? ring_position(sring, m, hv) : ring_position(ring_hash, m, hv)];
    flag[r] = ((owner == node_id) == want_owned) ? 1 : 0;
  }
}

__global__ __launch_bounds__(kBlock) void route_emit_kernel(const unsigned long long* __restrict__ row_key,
                                                            int64_t rows, const int32_t* __restrict__ flag,
                                                            const int32_t* __restrict__ rank,
                                                            unsigned long long* __restrict__ ids) {
  const int64_t r = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (r < rows && flag[r]) ids[rank[r]] = row_key[r];
}

// ---- a request's ids by owning node (worker/emitter.cc:139-149) ---------------------------------
// rank8[p] = index (in ascending node-id order) of the node that owns ids[p]; owner[p] = that
// node's id; block_counts[k * blocks + block] = ids of this workgroup owned by node k.
constexpr int kRouteMaxNodes = 256;

__global__ __launch_bounds__(kBlock) void route_rank_kernel(const uint64_t* __restrict__ ids, int64_t n,
                                                            unsigned long long table_hash,
                                                            const unsigned long long* __restrict__ ring_hash,
                                                            const uint32_t* __restrict__ ring_rank, int m,
                                                            const unsigned long long* __restrict__ node_of_rank,
                                                            int nodes, unsigned long long* __restrict__ owner,
                                                            uint8_t* __restrict__ rank8,
                                                            int32_t* __restrict__ block_counts) {
  __shared__ int32_t hist[kRouteMaxNodes];
  __shared__ unsigned long long sring[kRingLds];
  if ((int)threadIdx.x < nodes) hist[threadIdx.x] = 0;
  const bool in_lds = stage_ring(sring, ring_hash, m);
  __syncthreads();
  const int64_t p = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (p < n) {
    const unsigned long long hv = table_hash ^ route_hash64(ids[p]);
    const uint32_t k = ring_rank[in_lds ? ring_position(sring, m, hv) : ring_position(ring_hash, m, hv)];
    rank8[p] = (uint8_t)k;
    if (owner) owner[p] = node_of_rank[k];
    atomicAdd(&hist[k], 1);
  }
  __syncthreads();
  if ((int)threadIdx.x < nodes) block_counts[(int64_t)threadIdx.x * gridDim.x + blockIdx.x] = hist[threadIdx.x];
}

// node_count[k] = ids of node k, read off the scanned per-workgroup counts: where node k + 1's
// ids begin minus where node k's do (thousands of workgroups adding to the same few counters
// in memory cost more than the rest of the routing together).
__global__ __launch_bounds__(kRouteMaxNodes) void route_counts_kernel(const int32_t* __restrict__ block_base,
                                                                      int64_t blocks, int nodes, int32_t n,
                                                                      int32_t* __restrict__ node_count) {
  const int k = threadIdx.x;
  if (k >= nodes) return;
  const int32_t end = k + 1 < nodes ? block_base[(int64_t)(k + 1) * blocks] : n;
  node_count[k] = end - block_base[(int64_t)k * blocks];
}

// perm[where node k's ids begin + ids of node k in earlier workgroups + earlier in this one] = p:
// a stable partition of the positions by owner.
__global__ __launch_bounds__(kBlock) void route_scatter_kernel(const uint8_t* __restrict__ rank8, int64_t n,
                                                               const int32_t* __restrict__ block_base,
                                                               long long* __restrict__ perm) {
  __shared__ int32_t wave_count[kBlock / kWave][kRouteMaxNodes];
  for (int i = threadIdx.x; i < (kBlock / kWave) * kRouteMaxNodes; i += kBlock) (&wave_count[0][0])[i] = 0;
  __syncthreads();
  const int64_t p = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  const bool on = p < n;
  const uint32_t k = on ? rank8[p] : 0u;
  const int lane = wave_lane();
  const int wave = threadIdx.x / kWave;
  unsigned long long same = __ballot(on);
#pragma unroll
  for (int b = 0; b < 8; ++b) {
    const bool bit = (k >> b) & 1u;
    const unsigned long long votes = __ballot(bit);
    same &= bit ? votes : ~votes;
  }
  const int before = __popcll(same & ((1ull << lane) - 1ull));
  if (on && before == 0) wave_count[wave][k] = __popcll(same);
  __syncthreads();
  if (!on) return;
  int offset = before;
  for (int w = 0; w < wave; ++w) offset += wave_count[w][k];
  perm[block_base[(int64_t)k * gridDim.x + blockIdx.x] + offset] = p;
}

// ---- erase -------------------------------------------------------------------
// Rows are kept dense: the rows that go leave holes, and the live rows at the tail move into
// the holes below the new row count. Sources lie at or above that count, destinations below
// it, so all moves can run at once. The index is rebuilt from the row keys afterwards.
__global__ __launch_bounds__(kBlock) void erase_mark_kernel(TableView tv, const uint64_t* __restrict__ ids,
                                                            int64_t n, int32_t* __restrict__ dead) {
  const int64_t i = (int64_t)blockIdx.x * (kBlock / kBucket) + threadIdx.x / kBucket;
  const int gl = threadIdx.x & (kBucket - 1);
  const bool active = i < n;
  const uint32_t r = probe_find(tv, active ? ids[i] : 0, active, gl, kBucket);
  if (active && gl == 0 && r != kEmptyRow) dead[r] = 1;   // an id listed twice writes the same 1
}

// dead_before[r] = dead rows among [0, r). keep = rows that stay.
__global__ __launch_bounds__(kBlock) void erase_plan_kernel(const int32_t* __restrict__ dead,
                                                            const int32_t* __restrict__ dead_before,
                                                            int64_t rows, int64_t keep,
                                                            uint32_t* __restrict__ holes,
                                                            uint32_t* __restrict__ movers) {
  const int64_t r = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (r >= rows) return;
  if (r < keep) {
    if (dead[r]) holes[dead_before[r]] = (uint32_t)r;
  } else if (!dead[r]) {
    // live rows among [keep, r): all rows there minus the dead ones there
    const int64_t dead_below_keep = dead_before[keep];
    movers[(r - keep) - (dead_before[r] - dead_below_keep)] = (uint32_t)r;
  }
}

__global__ __launch_bounds__(kBlock) void erase_move_kernel(TableView tv, const uint32_t* __restrict__ holes,
                                                            const uint32_t* __restrict__ movers,
                                                            int64_t count) {
  const int64_t total = count * tv.stride;
  const int64_t step = (int64_t)gridDim.x * kBlock;
  for (int64_t t = (int64_t)blockIdx.x * kBlock + threadIdx.x; t < total; t += step) {
    const int64_t k = t / tv.stride;
    const int64_t j = t - k * tv.stride;
    const int64_t src = movers[k], dst = holes[k];
    tv.recs[dst * tv.stride + j] = tv.recs[src * tv.stride + j];
    if (j == 0) tv.row_key[dst] = tv.row_key[src];
  }
}

__global__ void set_row_count_kernel(uint32_t* counters, uint32_t rows) {
  if (threadIdx.x == 0 && blockIdx.x == 0) counters[0] = rows;
}

// re-index every existing row into a fresh (larger) slot array; launch number 0 = "old row"
__global__ __launch_bounds__(kBlock) void reindex_kernel(Slot* slots, uint64_t mask,
                                                         const unsigned long long* __restrict__ row_key,
                                                         int64_t rows) {
  const int64_t r = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (r >= rows) return;
  const unsigned long long id = row_key[r];
  if (id == kEmptyKey) {
    slots[mask + 1].key = 0ull;
    slots[mask + 1].row_epoch = (unsigned long long)r;
    return;
  }
  const uint64_t nb_mask = mask >> 2;
  uint64_t b = mix64(id) & nb_mask;
  for (uint64_t n = 0; n <= nb_mask; ++n) {
    for (int s = 0; s < kBucket; ++s) {
      Slot* slot = &slots[b * kBucket + s];
      const unsigned long long old = atomicCAS(&slot->key, kEmptyKey, id);
      if (old == kEmptyKey) {
        slot->row_epoch = (unsigned long long)r;
        return;
      }
    }
    b = (b + 1) & nb_mask;
  }
}

// launch numbers wrapped around: forget them all (every row becomes an "old row")
__global__ __launch_bounds__(kBlock) void clear_epochs_kernel(Slot* slots, uint64_t count) {
  const uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= count) return;
  if (slots[i].key != kEmptyKey) slots[i].row_epoch &= 0xFFFFFFFFull;
}

// copy records into a slab with a wider stride (new state columns stay zero)
__global__ __launch_bounds__(kBlock) void restride_kernel(const float* __restrict__ src,
                                                          int64_t src_stride, float* __restrict__ dst,
                                                          int64_t dst_stride, int64_t rows,
                                                          int copy_floats) {
  // grid-stride: a launch cannot carry more than 2^32 work-items, a large table has more floats
  const int64_t total = rows * copy_floats;
  const int64_t step = (int64_t)gridDim.x * kBlock;
  for (int64_t t = (int64_t)blockIdx.x * kBlock + threadIdx.x; t < total; t += step) {
    const int64_t r = t / copy_floats;
    const int j = (int)(t - r * copy_floats);
    dst[r * dst_stride + j] = src[r * src_stride + j];
  }
}

// ---------------------------------------------------------------------------
// Rows in the reference's wire layout (std::vector<Tensor> as Serialize writes it,
// common/serialize.h:156-176, 214-228): u64 count, then per row 18 header bytes {u8 layout 0,
// u64 rank 1, i64 dim, u8 dtype 11} and dim floats. A row starts on an even offset that is not
// always a multiple of four, so both directions move 16-bit halves.
// ---------------------------------------------------------------------------
constexpr int kWireHeader = 18;

__device__ __forceinline__ uint32_t wire_header_byte(int b, int dim) {
  if (b == 1) return 1u;                                   // rank, low byte
  if (b >= 9 && b <= 16) return ((uint64_t)dim >> (8 * (b - 9))) & 0xFFu;
  if (b == 17) return 11u;                                 // DType::kFloat32
  return 0u;                                               // layout kStride, upper bytes
}

__global__ __launch_bounds__(kBlock) void rows_to_wire_kernel(const float* __restrict__ rows, int64_t n,
                                                              int dim, uint16_t* __restrict__ wire) {
  const int per_row = kWireHeader / 2 + 2 * dim;           // 16-bit halves per row
  const int64_t total = 4 + n * per_row;
  const int64_t step = (int64_t)gridDim.x * kBlock;
  for (int64_t h = (int64_t)blockIdx.x * kBlock + threadIdx.x; h < total; h += step) {
    uint32_t v;
    if (h < 4) {
      v = (uint32_t)(((uint64_t)n >> (16 * h)) & 0xFFFFu);
    } else {
      const int64_t r = (h - 4) / per_row;
      const int k = (int)((h - 4) - r * per_row);
      if (k < kWireHeader / 2) {
        v = wire_header_byte(2 * k, dim) | (wire_header_byte(2 * k + 1, dim) << 8);
      } else {
        const uint32_t bits = __float_as_uint(rows[r * dim + (k - kWireHeader / 2) / 2]);
        v = ((k - kWireHeader / 2) & 1) ? bits >> 16 : bits & 0xFFFFu;
      }
    }
    wire[h] = (uint16_t)v;
  }
}

__global__ __launch_bounds__(kBlock) void wire_to_rows_kernel(const uint16_t* __restrict__ wire, int64_t n,
                                                              int dim, float* __restrict__ rows) {
  const int per_row = kWireHeader / 2 + 2 * dim;
  const int64_t total = n * dim;
  const int64_t step = (int64_t)gridDim.x * kBlock;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < total; i += step) {
    const int64_t r = i / dim;
    const int f = (int)(i - r * dim);
    const uint16_t* p = wire + 4 + r * per_row + kWireHeader / 2 + 2 * f;
    rows[i] = __uint_as_float((uint32_t)p[0] | ((uint32_t)p[1] << 16));
  }
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
static inline unsigned grid_for(int64_t items, int per_block) {
  return (unsigned)((items + per_block - 1) / per_block);
}

// Workgroups for a grid-stride kernel over `items`: enough to fill the chip many times over,
// never so many that workgroups x 256 passes the 2^32 work-items one launch can carry.
static inline unsigned strided_grid(int64_t items) {
  int64_t blocks = (items + kBlock - 1) / kBlock;
  const int64_t cap = 1 << 20;
  if (blocks > cap) blocks = cap;
  if (blocks < 1) blocks = 1;
  return (unsigned)blocks;
}

// Ids one launch of a `group`-lanes-per-id kernel may take so that ids x group stays below 2^31.
static inline int64_t max_ids_per_launch(int group) { return ((int64_t)1 << 31) / group - kBlock; }

static int32_t alloc_slots(uint64_t cap, Slot** out, hipStream_t s) {
  Slot* p = nullptr;
  KRK_HIP(hipMalloc((void**)&p, (cap + 1) * sizeof(Slot)));
  hipError_t e = hipMemsetAsync(p, 0xFF, (cap + 1) * sizeof(Slot), s);
  if (e != hipSuccess) {
    (void)hipFree(p);
    return hip_fail(e, "hipMemsetAsync(slots)", __FILE__, __LINE__);
  }
  *out = p;
  return KRK_SUCCESS;
}

static int32_t refresh_rows(krk_sparse* t) {
  KRK_HIP(hipMemcpyAsync(t->host_counters, t->counters, 16, hipMemcpyDeviceToHost, t->stream));
  KRK_HIP(hipStreamSynchronize(t->stream));
  t->size_ub = t->host_counters[0];
  return KRK_SUCCESS;
}

static int32_t grow_rows(krk_sparse* t, int64_t new_cap, int64_t new_stride) {
  KRK_TRY(refresh_rows(t));   // rows in use must be known exactly before records are moved
  const int64_t rows = t->size_ub;
  if (new_cap < rows) new_cap = rows;
  if (new_cap >= (int64_t)kEmptyRow) {
    set_error("sparse table cannot hold more than 2^32-2 rows");
    return KRK_E_CAPACITY;
  }
  DeviceGuard recs_guard, keys_guard;
  const size_t rec_bytes = (size_t)new_cap * (size_t)new_stride * sizeof(float);
  KRK_HIP(hipMalloc(&recs_guard.p, rec_bytes ? rec_bytes : 16));
  KRK_HIP(hipMalloc(&keys_guard.p, (size_t)(new_cap ? new_cap : 1) * sizeof(unsigned long long)));
  float* nrecs = reinterpret_cast<float*>(recs_guard.p);
  unsigned long long* nkeys = reinterpret_cast<unsigned long long*>(keys_guard.p);
  const size_t used = (size_t)rows * (size_t)t->stride * sizeof(float);
  if (used) KRK_HIP(hipMemcpyAsync(nrecs, t->recs, used, hipMemcpyDeviceToDevice, t->stream));
  if (rec_bytes > used)
    KRK_HIP(hipMemsetAsync(reinterpret_cast<char*>(nrecs) + used, 0, rec_bytes - used, t->stream));
  if (rows)
    KRK_HIP(hipMemcpyAsync(nkeys, t->row_key, (size_t)rows * sizeof(unsigned long long),
                           hipMemcpyDeviceToDevice, t->stream));
  KRK_HIP(hipStreamSynchronize(t->stream));
  if (t->recs) (void)hipFree(t->recs);
  if (t->row_key) (void)hipFree(t->row_key);
  t->recs = recs_guard.release<float>();
  t->row_key = keys_guard.release<unsigned long long>();
  t->row_cap = new_cap;
  t->layout_version++;
  return KRK_SUCCESS;
}

static int32_t grow_slots(krk_sparse* t, uint64_t new_cap) {
  Slot* ns = nullptr;
  KRK_TRY(alloc_slots(new_cap, &ns, t->stream));
  DeviceGuard guard;
  guard.p = ns;
  KRK_TRY(refresh_rows(t));
  const int64_t rows = t->size_ub;
  if (rows) {
    hipLaunchKernelGGL(reindex_kernel, dim3(grid_for(rows, kBlock)), dim3(kBlock), 0, t->stream, ns,
                       new_cap - 1, t->row_key, rows);
    KRK_HIP(hipGetLastError());
  }
  KRK_HIP(hipStreamSynchronize(t->stream));
  if (t->slots) (void)hipFree(t->slots);
  t->slots = guard.release<Slot>();
  t->slot_cap = new_cap;
  t->layout_version++;
  return KRK_SUCCESS;
}

static uint64_t pow2_at_least(uint64_t x) {
  uint64_t c = 1024;
  while (c < x) c <<= 1;
  return c;
}

// Lowers the row bound with the count the device published last: exact as of that launch,
// plus everything enqueued after it.
static void tighten_bound(krk_sparse* t) {
  const unsigned long long pub = __atomic_load_n(t->host_pub, __ATOMIC_ACQUIRE);
  const uint32_t ep = (uint32_t)(pub >> 32);
  if (ep == 0 || ep > t->epoch || t->epoch - ep >= 256) return;
  const int64_t cand = (int64_t)(uint32_t)pub + (int64_t)(t->enq_total - t->enq_at[ep & 255]);
  if (cand < t->size_ub) t->size_ub = cand;
}

// Room for `extra_rows` more rows: records, row keys, and an index at most half full.
int32_t sparse_ensure_room(krk_sparse* t, int64_t extra_rows) {
  int64_t need = t->size_ub + extra_rows;
  if (need > t->row_cap || (uint64_t)need * 2 > t->slot_cap) {
    tighten_bound(t);
    need = t->size_ub + extra_rows;
  }
  if (need > t->row_cap || (uint64_t)need * 2 > t->slot_cap) {
    // the bound may be stale (async pulls add their whole request to it): refresh it first
    KRK_TRY(refresh_rows(t));
    need = t->size_ub + extra_rows;
  }
  if (need > t->row_cap) {
    int64_t cap = t->row_cap * 2;
    if (cap < need) cap = need;
    if (cap >= (int64_t)kEmptyRow) cap = (int64_t)kEmptyRow - 1;
    if (cap < need) {
      set_error("sparse table cannot hold %lld rows", (long long)need);
      return KRK_E_CAPACITY;
    }
    KRK_TRY(grow_rows(t, cap, t->stride));
  }
  if ((uint64_t)need * 2 > t->slot_cap) KRK_TRY(grow_slots(t, pow2_at_least((uint64_t)need * 2)));
  return KRK_SUCCESS;
}

int32_t sparse_next_epoch(krk_sparse* t, int64_t n) {
  if (t->epoch >= 0xFFFFFFF0u) {
    hipLaunchKernelGGL(clear_epochs_kernel, dim3(grid_for((int64_t)t->slot_cap + 1, kBlock)),
                       dim3(kBlock), 0, t->stream, t->slots, t->slot_cap + 1);
    KRK_HIP(hipGetLastError());
    KRK_TRY(refresh_rows(t));   // drains the stream: no launch with an old number is in flight
    __atomic_store_n(t->host_pub, 0ull, __ATOMIC_RELEASE);
    t->epoch = 0;
  }
  t->epoch += 1;
  t->enq_total += (uint64_t)n;
  t->enq_at[t->epoch & 255] = t->enq_total;
  t->size_ub += n;
  t->last_request = n;
  return KRK_SUCCESS;
}

bool sparse_near_full(const krk_sparse* t) {
  const int64_t room = std::min<int64_t>(t->row_cap, (int64_t)(t->slot_cap / 2)) - t->size_ub;
  return room < 4 * t->last_request;
}

int32_t sparse_publish(krk_sparse* const* tables, int n, hipStream_t stream) {
  PublishArgs a;
  a.n = n;
  for (int i = 0; i < n; ++i) {
    a.epoch[i] = tables[i]->epoch;
    a.counters[i] = tables[i]->counters;
    a.host_pub[i] = tables[i]->host_pub;
  }
  hipLaunchKernelGGL(publish_kernel, dim3(1), dim3(64), 0, stream, a);
  KRK_HIP(hipGetLastError());
  return KRK_SUCCESS;
}

// Adds the state columns an optimizer needs; existing records are re-strided once.
int32_t sparse_ensure_columns(krk_sparse* t, uint32_t mask) {
  bool change = false;
  int32_t col_off[KRK_ST_COUNT];
  memcpy(col_off, t->col_off, sizeof(col_off));
  // the step counter, when present, stays the last column: it is re-placed after new columns
  int64_t body = t->meta_off >= 0 ? t->meta_off : t->stride;
  for (int st = 1; st < KRK_ST_COUNT; ++st) {
    if ((mask & (1u << st)) && col_off[st] < 0) {
      col_off[st] = (int32_t)body;
      body += t->dim;
      change = true;
    }
  }
  const bool want_meta = (mask & (1u << KRK_ST_STEPS)) || t->meta_off >= 0;
  if (want_meta && t->meta_off < 0) change = true;
  if (!change) return KRK_SUCCESS;
  const int32_t meta_off = want_meta ? (int32_t)body : -1;
  // A record that carries the word ends on a 128-byte line where its arrays are whole sectors:
  // the push kernels then write the word's sector and the padding behind it, so no line of the
  // record is written in part (see store_row_word).
  int64_t stride = body + (want_meta ? t->meta_floats : 0);
  if (want_meta && t->dim % 16 == 0) stride = (stride + 31) & ~(int64_t)31;

  const int64_t old_stride = t->stride;
  const int32_t old_meta = t->meta_off;
  const int64_t old_body = old_meta >= 0 ? old_meta : old_stride;
  KRK_TRY(refresh_rows(t));
  const int64_t rows = t->size_ub;
  DeviceGuard guard;
  const size_t rec_bytes = (size_t)t->row_cap * (size_t)stride * sizeof(float);
  KRK_HIP(hipMalloc(&guard.p, rec_bytes ? rec_bytes : 16));
  float* nrecs = reinterpret_cast<float*>(guard.p);
  KRK_HIP(hipMemsetAsync(nrecs, 0, rec_bytes, t->stream));
  if (rows) {
    hipLaunchKernelGGL(restride_kernel, dim3(strided_grid(rows * old_body)), dim3(kBlock), 0,
                       t->stream, t->recs, old_stride, nrecs, stride, rows, (int)old_body);
    if (old_meta >= 0) {
      hipLaunchKernelGGL(restride_kernel, dim3(strided_grid(rows * 2)), dim3(kBlock), 0, t->stream,
                         t->recs + old_meta, old_stride, nrecs + meta_off, stride, rows, 2);
    }
    KRK_HIP(hipGetLastError());
  }
  KRK_HIP(hipStreamSynchronize(t->stream));
  if (t->recs) (void)hipFree(t->recs);
  t->recs = guard.release<float>();
  t->stride = stride;
  t->meta_off = meta_off;
  memcpy(t->col_off, col_off, sizeof(col_off));
  t->layout_version++;
  return KRK_SUCCESS;
}

void optim_state_slots(const krk_optim& o, int32_t st[3]) {
  st[0] = st[1] = st[2] = -1;
  switch (o.type) {
    case KRK_SGD:
      if (o.has_momentum) st[0] = KRK_ST_MOMENTUM_BUFFER;
      break;
    case KRK_ADAGRAD:
      st[0] = KRK_ST_STATE_SUM;
      break;
    case KRK_ADAM:
      st[0] = KRK_ST_FIRST_MOMENT;
      st[1] = KRK_ST_SECOND_MOMENT;
      if (o.amsgrad) st[2] = KRK_ST_SECOND_MOMENT_MAX;
      break;
    case KRK_RMSPROP:
      st[0] = KRK_ST_SQUARE_AVERAGE;
      if (o.centered) st[1] = KRK_ST_G_AVE;
      if (o.has_momentum) st[2] = KRK_ST_MOMENTUM_BUFFER;
      break;
    default:
      break;
  }
}

void sparse_optim_columns(const krk_sparse* t, const krk_optim& o, int32_t cols[3]) {
  int32_t st[3];
  optim_state_slots(o, st);
  for (int i = 0; i < 3; ++i) cols[i] = st[i] >= 0 ? t->col_off[st[i]] : -1;
}

// After the stream has drained and counters were copied to host_counters: take the exact row
// count and turn device-side error bits into a return code.
int32_t collect_counters(krk_sparse* t) {
  t->size_ub = t->host_counters[0];
  const uint32_t err = t->host_counters[1];
  if (err) {
    KRK_HIP(hipMemsetAsync(t->counters + 1, 0, sizeof(uint32_t), t->stream));
    KRK_HIP(hipStreamSynchronize(t->stream));
    if (err & kErrOverflow) {
      set_error("sparse table index or row storage overflowed on the device");
      return KRK_E_CAPACITY;
    }
    set_error("push named an id that is not in the table");
    return KRK_SPARSE_ID_NOT_EXIST;
  }
  return KRK_SUCCESS;
}

// End of an API call: blocking calls wait, refresh the row count and surface device-side errors.
int32_t sparse_finish(krk_sparse* t, uint32_t flags) {
  if (flags & KRK_ASYNC) return KRK_SUCCESS;
  KRK_HIP(hipMemcpyAsync(t->host_counters, t->counters, 16, hipMemcpyDeviceToHost, t->stream));
  KRK_HIP(hipStreamSynchronize(t->stream));
  return collect_counters(t);
}

static InitK make_init_k(const krk_init& in, int64_t dim) {
  InitK k;
  k.seed_mix = splitmix64(in.seed);
  k.kind = 0;
  k.p0 = 0.0f;
  k.p1 = 0.0f;
  // t/math.cc:24-50 : for a 1-D [dim] tensor fan_out = dim and fan_in = 1;
  // t/math.cc:476-484, 507-517 : std = gain * sqrt(2.0 / float(fan_in + fan_out)), a = sqrt(3.0) * std
  const float xstd = (float)((double)in.a * std::sqrt(2.0 / (double)(float)(1 + dim)));
  switch (in.type) {
    case KRK_INIT_CONSTANT: k.kind = 0; k.p0 = in.a; break;
    case KRK_INIT_UNIFORM: k.kind = 1; k.p0 = in.a; k.p1 = in.b; break;
    case KRK_INIT_NORMAL: k.kind = 2; k.p0 = in.a; k.p1 = in.b; break;
    case KRK_INIT_XAVIER_UNIFORM: {
      const float a = (float)(std::sqrt(3.0) * (double)xstd);
      k.kind = 1; k.p0 = -a; k.p1 = a;
      break;
    }
    case KRK_INIT_XAVIER_NORMAL: k.kind = 2; k.p0 = 0.0f; k.p1 = xstd; break;
    default: break;
  }
  return k;
}

// Enqueues push_kernel or, for whole rows of 32 to 128 floats, push_wide_kernel.
template <int OPT, int VEC>
static void launch_push_opt(krk_sparse* t, const uint64_t* ids, int64_t n, const float* grads, float lr,
                            const OptimK& k, const PushCols& pc, const uint32_t* notes) {
  const TableView tv = t->view();
  const int dim = (int)t->dim;
  const dim3 block(kBlock);
  if constexpr (VEC == 4) {
    if (push_is_wide(t->vec, t->group, t->elems)) {
      const dim3 grid(grid_for(n, (kBlock / kWave) * kWideIds));
      if (t->group == 8) {
        hipLaunchKernelGGL((push_wide_kernel<OPT, 2>), grid, block, 0, t->stream, tv, ids, n, grads, dim,
                           t->elems, lr, k, pc, notes);
      } else {
        hipLaunchKernelGGL((push_wide_kernel<OPT, 4>), grid, block, 0, t->stream, tv, ids, n, grads, dim,
                           t->elems, lr, k, pc, notes);
      }
      return;
    }
  }
  const dim3 grid(grid_for(n, kBlock / t->group));
  hipLaunchKernelGGL((push_kernel<OPT, VEC>), grid, block, 0, t->stream, tv, ids, n, grads, dim, t->elems,
                     t->group, lr, k, pc, notes);
}

template <int VEC>
static void launch_push(krk_sparse* t, const krk_optim& o, const uint64_t* ids, int64_t n,
                        const float* grads, float lr, const uint32_t* notes = nullptr) {
  const OptimK k = make_optim_k(o);
  int32_t cols[3];
  sparse_optim_columns(t, o, cols);
  const bool needs_meta = (optim_state_mask(o) >> KRK_ST_STEPS) & 1u;
  const PushCols pc{cols[0], cols[1], cols[2], needs_meta ? t->meta_off : -1};
  switch (o.type) {
    case KRK_SGD: launch_push_opt<KRK_SGD, VEC>(t, ids, n, grads, lr, k, pc, notes); break;
    case KRK_ADAGRAD: launch_push_opt<KRK_ADAGRAD, VEC>(t, ids, n, grads, lr, k, pc, notes); break;
    case KRK_ADAM: launch_push_opt<KRK_ADAM, VEC>(t, ids, n, grads, lr, k, pc, notes); break;
    default: launch_push_opt<KRK_RMSPROP, VEC>(t, ids, n, grads, lr, k, pc, notes); break;
  }
}

}  // namespace krk

using namespace krk;

static int32_t check_table(krk_sparse* t) {
  if (!t) {
    set_error("null sparse table handle");
    return KRK_E_ARGUMENT;
  }
  return ensure_runtime();
}

static bool valid_optim(const krk_optim* o) {
  return o && o->type >= KRK_ADAGRAD && o->type <= KRK_SGD;
}

static bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

extern "C" {

int32_t krk_sparse_create(int64_t dim, const krk_init* init, int64_t capacity_hint,
                          krk_sparse** out) {
  if (!out || !init || dim <= 0 || dim > (1 << 20) || capacity_hint < 0) {
    set_error("krk_sparse_create: bad argument (dim=%lld)", (long long)dim);
    return KRK_E_ARGUMENT;
  }
  if (init->type < KRK_INIT_CONSTANT || init->type > KRK_INIT_XAVIER_NORMAL) {
    set_error("initializer type %d is not supported", init->type);
    return KRK_UNSUPPORTED_INITIALIZER;   // ps/ps.cc:684-688
  }
  KRK_TRY(ensure_runtime());
  krk_sparse* t = new (std::nothrow) krk_sparse();
  if (!t) return KRK_E_DEVICE;
  t->dim = dim;
  t->vec = (dim % 4 == 0) ? 4 : 1;
  t->elems = (int)(dim / t->vec);
  int g = kBucket;   // at least the four lanes that read an index bucket together
  while (g < t->elems && g < kWave) g <<= 1;
  t->group = g;
  t->init = *init;
  t->initk = make_init_k(*init, dim);
  t->stride = dim;
  t->meta_floats = row_word_floats((int)dim, t->vec);
  for (auto& c : t->col_off) c = -1;
  int32_t rc = t->open_stream();
  t->own_stream = t->stream;
  if (rc == KRK_SUCCESS) {
    hipError_t e = hipMalloc((void**)&t->counters, kCounterWords * sizeof(uint32_t));
    if (e == hipSuccess) e = hipMemsetAsync(t->counters, 0, kCounterWords * sizeof(uint32_t), t->stream);
    if (e == hipSuccess) e = hipHostMalloc((void**)&t->host_counters, 16, hipHostMallocDefault);
    if (e == hipSuccess) e = hipHostMalloc((void**)&t->host_pub, 16, hipHostMallocCoherent);
    if (e == hipSuccess) {
      *t->host_pub = 0ull;
      t->host_inserted = reinterpret_cast<uint32_t*>(t->host_pub + 1);
      *t->host_inserted = 1u;   // an empty table is about to be filled
    }
    if (e != hipSuccess) rc = hip_fail(e, "krk_sparse_create allocations", __FILE__, __LINE__);
  }
  if (rc == KRK_SUCCESS) {
    int64_t rows = capacity_hint > 0 ? capacity_hint : 4096;
    rc = sparse_ensure_room(t, rows);
  }
  if (rc != KRK_SUCCESS) {
    krk_sparse_destroy(t);
    return rc;
  }
  *out = t;
  return KRK_SUCCESS;
}

int32_t krk_sparse_destroy(krk_sparse* t) {
  if (!t) return KRK_SUCCESS;
  if (t->member_of) {
    set_error("destroy the group before its tables");
    return KRK_E_ARGUMENT;
  }
  (void)hipStreamSynchronize(t->stream);   // also when the table runs on the null stream
  if (t->slots) (void)hipFree(t->slots);
  if (t->recs) (void)hipFree(t->recs);
  if (t->row_key) (void)hipFree(t->row_key);
  if (t->counters) (void)hipFree(t->counters);
  if (t->host_counters) (void)hipHostFree(t->host_counters);
  if (t->host_pub) (void)hipHostFree(t->host_pub);
  for (auto& b : t->scratch) b.release();
  t->notes.release();
  t->stream = t->own_stream;
  t->close_stream();
  delete t;
  return KRK_SUCCESS;
}

int32_t krk_sparse_set_stream(krk_sparse* t, void* stream) {
  KRK_TRY(check_table(t));
  std::lock_guard<std::mutex> lk(t->mu);
  if (t->member_of) {
    set_error("a group member runs on its group's stream");
    return KRK_E_ARGUMENT;
  }
  hipStream_t next = stream == KRK_OWN_STREAM ? t->own_stream : reinterpret_cast<hipStream_t>(stream);
  if (next == t->stream) return KRK_SUCCESS;
  // what is enqueued on the old stream must be complete before work on the new one may follow
  KRK_TRY(sparse_finish(t, 0));
  t->stream = next;
  return KRK_SUCCESS;
}

int32_t krk_sparse_dim(krk_sparse* t, int64_t* dim) {
  if (!t || !dim) return KRK_E_ARGUMENT;
  *dim = t->dim;
  return KRK_SUCCESS;
}

int32_t krk_sparse_size(krk_sparse* t, int64_t* rows) {
  KRK_TRY(check_table(t));
  if (!rows) return KRK_E_ARGUMENT;
  std::lock_guard<std::mutex> lk(t->mu);
  KRK_TRY(refresh_rows(t));
  *rows = t->size_ub;
  return KRK_SUCCESS;
}

int32_t krk_sparse_reserve(krk_sparse* t, int64_t rows) {
  KRK_TRY(check_table(t));
  if (rows < 0) return KRK_E_ARGUMENT;
  std::lock_guard<std::mutex> lk(t->mu);
  const int64_t extra = rows - t->size_ub;
  return extra > 0 ? sparse_ensure_room(t, extra) : KRK_SUCCESS;
}

int32_t krk_sparse_sync(krk_sparse* t) {
  KRK_TRY(check_table(t));
  std::lock_guard<std::mutex> lk(t->mu);
  return sparse_finish(t, 0);
}

// The launches of one pull of n > 0 ids into d_out [n, dim]; the caller holds the table's lock
// and has made room for n more rows.
static int32_t pull_enqueue(krk_sparse* t, const uint64_t* d_ids, int64_t n, float* d_out,
                            uint32_t* notes = nullptr) {
  KRK_TRY(sparse_next_epoch(t, n));
  const bool wide = t->vec == 4 && pull_is_wide(t->group, t->elems);
  const int per_block = wide ? (kBlock / kWave) * kWideIds : kBlock / t->group;
  const dim3 grid(grid_for(n, per_block)), block(kBlock);
  // Two launches pay for many repeats of resident ids (8.9 million ids over a table of ten
  // million rows: 590 us in two launches, 730 us fused) and for requests of new ids alike (a
  // million ids that are all new, 16 floats a row: 195 us, 870 us fused). A smaller request takes
  // them while the table is being filled: the fused kernel adds to the row counter once per
  // wavefront that inserts, and those additions are served one after the other (98 600 new ids:
  // 137 us fused). Whether the table is being filled is what the pull before this one left
  // behind in host memory; it may lag by the requests that are still queued, and either choice
  // gives the same rows.
  const bool filling = t->host_inserted && __atomic_exchange_n(t->host_inserted, 0u, __ATOMIC_RELAXED) != 0u;
  if (n >= kTwoLaunchPull || (filling && n >= kTwoLaunchWhileFilling)) {
    KRK_TRY(t->scratch[5].reserve((size_t)kQueues * queue_capacity(n, per_block) * sizeof(uint32_t)));
    uint32_t* todo = t->scratch[5].as<uint32_t>();
    const int parity = t->pull_parity;
    t->pull_parity ^= 1;
    const dim3 small(kMissingGrid), missing_block(kMissBlock);
    const int64_t list_capacity = queue_capacity(n, per_block);
    if (t->vec == 4) {
      if (wide && t->group == 8) {
        hipLaunchKernelGGL((pull_resident_wide_kernel<4, 2>), grid, block, 0, t->stream, t->view(), d_ids, n, d_out,
                           todo, parity, (int)t->dim, t->elems, notes);
      } else if (wide && t->group == 16) {
        hipLaunchKernelGGL((pull_resident_wide_kernel<4, 4>), grid, block, 0, t->stream, t->view(), d_ids, n, d_out,
                           todo, parity, (int)t->dim, t->elems, notes);
      } else if (wide) {
        hipLaunchKernelGGL((pull_resident_wide_kernel<4, 8>), grid, block, 0, t->stream, t->view(), d_ids, n, d_out,
                           todo, parity, (int)t->dim, t->elems, notes);
      } else {
        hipLaunchKernelGGL((pull_resident_kernel<4>), grid, block, 0, t->stream, t->view(), d_ids, n, d_out, todo,
                           parity, (int)t->dim, t->elems, t->group, notes);
      }
      hipLaunchKernelGGL((pull_missing_kernel<4>), small, missing_block, 0, t->stream, t->view(), t->initk, d_ids,
                         d_out, todo, parity, list_capacity, (int)t->dim, t->elems, t->group, notes);
    } else {
      hipLaunchKernelGGL((pull_resident_kernel<1>), grid, block, 0, t->stream, t->view(), d_ids, n, d_out, todo,
                         parity, (int)t->dim, t->elems, t->group, notes);
      hipLaunchKernelGGL((pull_missing_kernel<1>), small, missing_block, 0, t->stream, t->view(), t->initk, d_ids,
                         d_out, todo, parity, list_capacity, (int)t->dim, t->elems, t->group, notes);
    }
  } else if (t->vec == 4 && wide && t->group == 8) {
    hipLaunchKernelGGL((pull_wide_kernel<4, 2>), grid, block, 0, t->stream, t->view(), t->initk, d_ids, n, d_out,
                       (int)t->dim, t->elems, notes);
  } else if (t->vec == 4 && wide && t->group == 16) {
    hipLaunchKernelGGL((pull_wide_kernel<4, 4>), grid, block, 0, t->stream, t->view(), t->initk, d_ids, n, d_out,
                       (int)t->dim, t->elems, notes);
  } else if (t->vec == 4 && wide) {
    hipLaunchKernelGGL((pull_wide_kernel<4, 8>), grid, block, 0, t->stream, t->view(), t->initk, d_ids, n, d_out,
                       (int)t->dim, t->elems, notes);
  } else if (t->vec == 4) {
    hipLaunchKernelGGL((pull_kernel<4>), grid, block, 0, t->stream, t->view(), t->initk, d_ids, n, d_out,
                       (int)t->dim, t->elems, t->group, notes);
  } else {
    hipLaunchKernelGGL((pull_kernel<1>), grid, block, 0, t->stream, t->view(), t->initk, d_ids, n, d_out,
                       (int)t->dim, t->elems, t->group, notes);
  }
  KRK_HIP(hipGetLastError());
  return KRK_SUCCESS;
}

int32_t krk_sparse_pull(krk_sparse* t, const uint64_t* ids, int64_t n, float* out, uint32_t flags) {
  KRK_TRY(check_table(t));
  KRK_TRY(check_flags(flags));
  if (n < 0 || (n > 0 && (!ids || !out))) return KRK_E_ARGUMENT;
  if ((flags & KRK_DEVICE_PTRS) && t->vec == 4 && !aligned16(out)) {
    set_error("device output must be 16-byte aligned");
    return KRK_E_ARGUMENT;
  }
  if (n > max_ids_per_launch(t->group)) {
    set_error("at most %lld ids per call for this row width; split the request",
              (long long)max_ids_per_launch(t->group));
    return KRK_E_CAPACITY;
  }
  std::lock_guard<std::mutex> lk(t->mu);
  if (n == 0) return sparse_finish(t, flags);
  KRK_TRY(sparse_ensure_room(t, n));
  const uint64_t* d_ids;
  float* d_out;
  KRK_TRY(t->input(ids, (size_t)n, flags, 0, &d_ids));
  KRK_TRY(t->output(out, (size_t)n * t->dim, flags, 1, &d_out));
  // KRK_NOTE_ROWS: requests served by one launch leave the row of every position behind
  uint32_t* notes = nullptr;
  if (flags & KRK_NOTE_ROWS) {
    t->noted_ids = nullptr;
    if ((flags & KRK_DEVICE_PTRS) && n <= kNotedMax) {
      KRK_TRY(t->notes.reserve((size_t)n * sizeof(uint32_t)));
      notes = t->notes.as<uint32_t>();
    }
  }
  KRK_TRY(pull_enqueue(t, d_ids, n, d_out, notes));
  if (notes) {
    t->noted_ids = ids;
    t->noted_n = n;
    t->noted_version = t->layout_version;
  }
  if ((flags & KRK_ASYNC) && sparse_near_full(t)) KRK_TRY(sparse_publish(&t, 1, t->stream));
  KRK_TRY(t->output_back(out, (size_t)n * t->dim, flags, 1));
  return sparse_finish(t, flags);
}

int32_t krk_sparse_pull_pooled(krk_sparse* t, const uint64_t* ids, int64_t n, const int64_t* offsets,
                               int64_t bags, const float* weights, int32_t mode, float patch_value,
                               float* out, uint32_t flags) {
  KRK_TRY(check_table(t));
  KRK_TRY(check_flags(flags));
  if (n < 0 || bags < 0 || (mode != KRK_POOL_SUM && mode != KRK_POOL_MEAN) || !offsets ||
      (n > 0 && !ids) || (bags > 0 && !out))
    return KRK_E_ARGUMENT;
  if (t->elems > t->group) {
    set_error("pooled pull supports rows of at most %d floats for this layout", 64 * t->vec);
    return KRK_INTERFACE_UNIMPLEMENTED;
  }
  if ((flags & KRK_DEVICE_PTRS) && t->vec == 4 && !aligned16(out)) {
    set_error("device output must be 16-byte aligned");
    return KRK_E_ARGUMENT;
  }
  if (bags > max_ids_per_launch(t->group) || n > max_ids_per_launch(kBucket)) {
    set_error("at most %lld bags per call for this row width; split the request",
              (long long)max_ids_per_launch(t->group));
    return KRK_E_CAPACITY;
  }
  if (!(flags & KRK_DEVICE_PTRS) && (offsets[0] != 0 || offsets[bags] != n)) {
    set_error("offsets must start at 0 and end at the number of ids");
    return KRK_E_ARGUMENT;
  }
  std::lock_guard<std::mutex> lk(t->mu);
  if (bags == 0) return sparse_finish(t, flags);
  KRK_TRY(sparse_ensure_room(t, n));
  const uint64_t* d_ids = nullptr;
  const long long* d_off;
  const float* d_w = nullptr;
  float* d_out;
  if (n > 0) KRK_TRY(t->input(ids, (size_t)n, flags, 0, &d_ids));
  KRK_TRY(t->input(reinterpret_cast<const long long*>(offsets), (size_t)bags + 1, flags, 1, &d_off));
  if (weights && n > 0) KRK_TRY(t->input(weights, (size_t)n, flags, 2, &d_w));
  KRK_TRY(t->output(out, (size_t)bags * t->dim, flags, 3, &d_out));
  KRK_TRY(sparse_next_epoch(t, n));
  // While the table is being filled (see pull_enqueue) the positions are looked up by a launch
  // that inserts nothing and the missing ones go through pull_missing_kernel: the probing
  // kernel that inserts adds to the row counter once per wavefront, 8.9 million positions of
  // which one in ten is new cost it half a million additions, served one after the other.
  const bool filling = t->host_inserted && __atomic_exchange_n(t->host_inserted, 0u, __ATOMIC_RELAXED) != 0u;
  const bool queued = filling && n >= kTwoLaunchWhileFilling;
  const int64_t list_capacity = queued ? queue_capacity(n, kBlock / kBucket) : 0;
  const size_t rows_words = ((size_t)(n > 0 ? n : 1) + 63) & ~(size_t)63;
  KRK_TRY(t->scratch[5].reserve((rows_words + (size_t)kQueues * (size_t)list_capacity) * sizeof(uint32_t)));
  uint32_t* rows = t->scratch[5].as<uint32_t>();
  uint32_t* todo = rows + rows_words;
  const int per_block = kBlock / t->group;
  const dim3 probe_grid(grid_for(n, kBlock / kBucket)), grid(grid_for(bags, per_block)), block(kBlock);
  const dim3 small(kMissingGrid), missing_block(kMissBlock);
  const int mean = mode == KRK_POOL_MEAN;
  int parity = 0;
  if (queued) {
    parity = t->pull_parity;
    t->pull_parity ^= 1;
    hipLaunchKernelGGL(pooled_find_kernel, probe_grid, block, 0, t->stream, t->view(), d_ids, n, rows, todo, parity);
  }
  if (t->vec == 4) {
    if (queued)
      hipLaunchKernelGGL((pull_missing_kernel<4, true>), small, missing_block, 0, t->stream, t->view(), t->initk,
                         d_ids, nullptr, todo, parity, list_capacity, (int)t->dim, t->elems, t->group, rows);
    else if (n > 0)
      hipLaunchKernelGGL((pooled_probe_kernel<4>), probe_grid, block, 0, t->stream, t->view(), t->initk, d_ids,
                         n, rows, t->elems);
    hipLaunchKernelGGL((pooled_sum_kernel<4>), grid, block, 0, t->stream, t->view(), rows, d_ids, n, d_off, bags, d_w,
                       mean, patch_value, d_out, (int)t->dim, t->elems, t->group);
  } else {
    if (queued)
      hipLaunchKernelGGL((pull_missing_kernel<1, true>), small, missing_block, 0, t->stream, t->view(), t->initk,
                         d_ids, nullptr, todo, parity, list_capacity, (int)t->dim, t->elems, t->group, rows);
    else if (n > 0)
      hipLaunchKernelGGL((pooled_probe_kernel<1>), probe_grid, block, 0, t->stream, t->view(), t->initk, d_ids,
                         n, rows, t->elems);
    hipLaunchKernelGGL((pooled_sum_kernel<1>), grid, block, 0, t->stream, t->view(), rows, d_ids, n, d_off, bags, d_w,
                       mean, patch_value, d_out, (int)t->dim, t->elems, t->group);
  }
  KRK_HIP(hipGetLastError());
  if ((flags & KRK_ASYNC) && sparse_near_full(t)) KRK_TRY(sparse_publish(&t, 1, t->stream));
  KRK_TRY(t->output_back(out, (size_t)bags * t->dim, flags, 3));
  return sparse_finish(t, flags);
}

int32_t krk_sparse_push(krk_sparse* t, const krk_optim* o, const uint64_t* ids, int64_t n,
                        const float* grads, int64_t grad_dim, float lr, uint32_t flags) {
  KRK_TRY(check_table(t));
  KRK_TRY(check_flags(flags));
  if (!valid_optim(o)) {
    set_error("optimizer type is not supported");
    return KRK_UNSUPPORTED_OPTIM;
  }
  if (n < 0 || (n > 0 && (!ids || !grads))) return KRK_E_ARGUMENT;
  if ((flags & KRK_DEVICE_PTRS) && t->vec == 4 && !aligned16(grads)) {
    set_error("device gradients must be 16-byte aligned");
    return KRK_E_ARGUMENT;
  }
  if (n > max_ids_per_launch(t->group)) {
    set_error("at most %lld ids per call for this row width; split the request",
              (long long)max_ids_per_launch(t->group));
    return KRK_E_CAPACITY;
  }
  std::lock_guard<std::mutex> lk(t->mu);
  if (n == 0) return sparse_finish(t, flags);
  if (grad_dim != t->dim) {   // ps/optim/adagrad.cc:29-32
    set_error("gradient width %lld does not match table dimension %lld", (long long)grad_dim,
              (long long)t->dim);
    return KRK_GRADIENT_UNCOMPATIBLE;
  }
  KRK_TRY(sparse_ensure_columns(t, optim_state_mask(*o)));
  const uint64_t* d_ids;
  const float* d_g;
  KRK_TRY(t->input(ids, (size_t)n, flags, 0, &d_ids));
  KRK_TRY(t->input(grads, (size_t)n * t->dim, flags, 1, &d_g));
  const uint32_t* notes = noted_rows(t, ids, n, flags);   // KRK_IDS_AS_PULLED: no second look-up
  if (t->vec == 4) {
    launch_push<4>(t, *o, d_ids, n, d_g, lr, notes);
  } else {
    launch_push<1>(t, *o, d_ids, n, d_g, lr, notes);
  }
  KRK_HIP(hipGetLastError());
  return sparse_finish(t, flags);
}

int64_t krk_wire_rows_bytes(int64_t n, int64_t dim) {
  if (n < 0 || dim <= 0) return -1;
  return 8 + n * (kWireHeader + 4 * dim);
}

int32_t krk_sparse_pull_wire(krk_sparse* t, const uint64_t* ids, int64_t n, void* reply) {
  KRK_TRY(check_table(t));
  if (n < 0 || !reply || (n > 0 && !ids) || ((uintptr_t)reply & 7)) {
    set_error("krk_sparse_pull_wire: reply must be an 8-byte aligned host buffer");
    return KRK_E_ARGUMENT;
  }
  if (n > max_ids_per_launch(t->group)) {
    set_error("at most %lld ids per call for this row width; split the request",
              (long long)max_ids_per_launch(t->group));
    return KRK_E_CAPACITY;
  }
  std::lock_guard<std::mutex> lk(t->mu);
  const size_t bytes = (size_t)krk_wire_rows_bytes(n, t->dim);
  uint8_t* d_reply;
  KRK_TRY(t->output(reinterpret_cast<uint8_t*>(reply), bytes, 0, 1, &d_reply));
  float* d_rows = nullptr;
  if (n > 0) {
    KRK_TRY(sparse_ensure_room(t, n));
    const uint64_t* d_ids;
    KRK_TRY(t->input(ids, (size_t)n, 0, 0, &d_ids));
    KRK_TRY(t->stage[2].reserve((size_t)n * t->dim * sizeof(float) + 16));
    d_rows = t->stage[2].as<float>();
    KRK_TRY(pull_enqueue(t, d_ids, n, d_rows));
  }
  hipLaunchKernelGGL(rows_to_wire_kernel, dim3(strided_grid((int64_t)(bytes / 2))), dim3(kBlock), 0, t->stream,
                     d_rows, n, (int)t->dim, reinterpret_cast<uint16_t*>(d_reply));
  KRK_HIP(hipGetLastError());
  KRK_TRY(t->output_back(reinterpret_cast<uint8_t*>(reply), bytes, 0, 1));
  return sparse_finish(t, 0);
}

int32_t krk_sparse_push_wire(krk_sparse* t, const krk_optim* o, const uint64_t* ids, int64_t n,
                             const void* grads_wire, int64_t wire_bytes, float lr) {
  KRK_TRY(check_table(t));
  if (!valid_optim(o)) {
    set_error("optimizer type is not supported");
    return KRK_UNSUPPORTED_OPTIM;
  }
  if (n < 0 || !grads_wire || (n > 0 && !ids) || ((uintptr_t)grads_wire & 7)) {
    set_error("krk_sparse_push_wire: grads_wire must be an 8-byte aligned host buffer");
    return KRK_E_ARGUMENT;
  }
  if (n > max_ids_per_launch(t->group)) {
    set_error("at most %lld ids per call for this row width; split the request",
              (long long)max_ids_per_launch(t->group));
    return KRK_E_CAPACITY;
  }
  // The request is checked before anything is applied: as many gradients as ids, each a dense
  // fp32 vector of the table's width (ps/optim/adagrad.cc:29-32 and its siblings return 11).
  const uint8_t* w = reinterpret_cast<const uint8_t*>(grads_wire);
  uint64_t count = 0;
  if (wire_bytes >= 8) memcpy(&count, w, 8);
  uint8_t want[kWireHeader] = {0};
  want[1] = 1;
  const uint64_t d64 = (uint64_t)t->dim;
  memcpy(want + 9, &d64, 8);
  want[17] = 11;
  const int64_t row_bytes = kWireHeader + 4 * t->dim;
  bool ok = wire_bytes >= 8 && count == (uint64_t)n && wire_bytes >= 8 + n * row_bytes;
  for (int64_t r = 0; ok && r < n; ++r) ok = memcmp(w + 8 + r * row_bytes, want, kWireHeader) == 0;
  if (!ok) {
    set_error("gradients do not match the ids or the table dimension %lld", (long long)t->dim);
    return KRK_GRADIENT_UNCOMPATIBLE;
  }
  std::lock_guard<std::mutex> lk(t->mu);
  if (n == 0) return sparse_finish(t, 0);
  KRK_TRY(sparse_ensure_columns(t, optim_state_mask(*o)));
  const uint64_t* d_ids;
  const uint8_t* d_wire;
  KRK_TRY(t->input(ids, (size_t)n, 0, 0, &d_ids));
  KRK_TRY(t->input(w, (size_t)(8 + n * row_bytes), 0, 1, &d_wire));
  KRK_TRY(t->stage[2].reserve((size_t)n * t->dim * sizeof(float) + 16));
  float* d_rows = t->stage[2].as<float>();
  hipLaunchKernelGGL(wire_to_rows_kernel, dim3(strided_grid(n * t->dim)), dim3(kBlock), 0, t->stream,
                     reinterpret_cast<const uint16_t*>(d_wire), n, (int)t->dim, d_rows);
  if (t->vec == 4) {
    launch_push<4>(t, *o, d_ids, n, d_rows, lr);
  } else {
    launch_push<1>(t, *o, d_ids, n, d_rows, lr);
  }
  KRK_HIP(hipGetLastError());
  return sparse_finish(t, 0);
}

int32_t krk_sparse_lookup(krk_sparse* t, const uint64_t* ids, int64_t n, int32_t* rows,
                          uint32_t flags) {
  KRK_TRY(check_table(t));
  KRK_TRY(check_flags(flags));
  if (n < 0 || (n > 0 && (!ids || !rows))) return KRK_E_ARGUMENT;
  if (n > max_ids_per_launch(kBucket)) {
    set_error("at most %lld ids per call for this row width; split the request",
              (long long)max_ids_per_launch(kBucket));
    return KRK_E_CAPACITY;
  }
  std::lock_guard<std::mutex> lk(t->mu);
  if (n == 0) return sparse_finish(t, flags);
  const uint64_t* d_ids;
  int32_t* d_rows;
  KRK_TRY(t->input(ids, (size_t)n, flags, 0, &d_ids));
  KRK_TRY(t->output(rows, (size_t)n, flags, 1, &d_rows));
  hipLaunchKernelGGL(lookup_kernel, dim3(grid_for(n, kBlock / kBucket)), dim3(kBlock), 0, t->stream,
                     t->view(), d_ids, n, d_rows);
  KRK_HIP(hipGetLastError());
  KRK_TRY(t->output_back(rows, (size_t)n, flags, 1));
  return sparse_finish(t, flags);
}

int32_t krk_sparse_import(krk_sparse* t, const uint64_t* ids, int64_t n, const float* vals,
                          uint32_t flags) {
  KRK_TRY(check_table(t));
  KRK_TRY(check_flags(flags));
  if (n < 0 || (n > 0 && (!ids || !vals))) return KRK_E_ARGUMENT;
  if ((flags & KRK_DEVICE_PTRS) && t->vec == 4 && !aligned16(vals)) return KRK_E_ARGUMENT;
  if (n > max_ids_per_launch(t->group)) {
    set_error("at most %lld ids per call for this row width; split the request",
              (long long)max_ids_per_launch(t->group));
    return KRK_E_CAPACITY;
  }
  std::lock_guard<std::mutex> lk(t->mu);
  if (n == 0) return sparse_finish(t, flags);
  KRK_TRY(sparse_ensure_room(t, n));
  const uint64_t* d_ids;
  const float* d_vals;
  KRK_TRY(t->input(ids, (size_t)n, flags, 0, &d_ids));
  KRK_TRY(t->input(vals, (size_t)n * t->dim, flags, 1, &d_vals));
  KRK_TRY(sparse_next_epoch(t, n));
  const dim3 grid(grid_for(n, kMissEntries)), block(kMissBlock);
  if (t->vec == 4) {
    hipLaunchKernelGGL((import_kernel<4>), grid, block, 0, t->stream, t->view(), d_ids, n, d_vals,
                       (int)t->dim, t->elems, t->group);
  } else {
    hipLaunchKernelGGL((import_kernel<1>), grid, block, 0, t->stream, t->view(), d_ids, n, d_vals,
                       (int)t->dim, t->elems, t->group);
  }
  KRK_HIP(hipGetLastError());
  if ((flags & KRK_ASYNC) && sparse_near_full(t)) KRK_TRY(sparse_publish(&t, 1, t->stream));
  return sparse_finish(t, flags);
}

int32_t krk_sparse_export(krk_sparse* t, uint64_t* ids, float* vals, int32_t state_type, float* state,
                          int64_t* steps, int64_t capacity, int64_t* rows_out, uint32_t flags) {
  KRK_TRY(check_table(t));
  KRK_TRY(check_flags(flags));
  if (flags & KRK_ASYNC) return KRK_E_ARGUMENT;
  if (state && (state_type < 1 || state_type >= KRK_ST_COUNT)) return KRK_E_ARGUMENT;
  std::lock_guard<std::mutex> lk(t->mu);
  KRK_TRY(sparse_finish(t, 0));
  const int64_t rows = t->size_ub;
  if (rows_out) *rows_out = rows;
  if (rows > capacity) {
    set_error("export needs room for %lld rows, caller offered %lld", (long long)rows,
              (long long)capacity);
    return KRK_E_CAPACITY;
  }
  if (rows == 0) return KRK_SUCCESS;
  unsigned long long* d_ids = nullptr;
  float* d_vals = nullptr;
  float* d_state = nullptr;
  long long* d_steps = nullptr;
  const size_t cells = (size_t)rows * t->dim;
  if (ids) KRK_TRY(t->output(reinterpret_cast<unsigned long long*>(ids), (size_t)rows, flags, 0, &d_ids));
  if (vals) KRK_TRY(t->output(vals, cells, flags, 1, &d_vals));
  if (state) KRK_TRY(t->output(state, cells, flags, 2, &d_state));
  if (steps) KRK_TRY(t->output(reinterpret_cast<long long*>(steps), (size_t)rows, flags, 3, &d_steps));
  const int state_off = state ? t->col_off[state_type] : -1;
  hipLaunchKernelGGL(export_kernel, dim3(strided_grid((int64_t)cells)), dim3(kBlock), 0, t->stream,
                     t->view(), rows, (int)t->dim, d_ids, d_vals, state_off, d_state, t->meta_off,
                     d_steps);
  KRK_HIP(hipGetLastError());
  if (ids) KRK_TRY(t->output_back(reinterpret_cast<unsigned long long*>(ids), (size_t)rows, flags, 0));
  if (vals) KRK_TRY(t->output_back(vals, cells, flags, 1));
  if (state) KRK_TRY(t->output_back(state, cells, flags, 2));
  if (steps) KRK_TRY(t->output_back(reinterpret_cast<long long*>(steps), (size_t)rows, flags, 3));
  return sparse_finish(t, 0);
}

int32_t krk_sparse_states(krk_sparse* t, uint32_t* mask) {
  KRK_TRY(check_table(t));
  if (!mask) return KRK_E_ARGUMENT;
  std::lock_guard<std::mutex> lk(t->mu);
  uint32_t m = t->meta_off >= 0 ? 1u : 0u;
  for (int st = 1; st < KRK_ST_COUNT; ++st) {
    if (t->col_off[st] >= 0) m |= 1u << st;
  }
  *mask = m;
  return KRK_SUCCESS;
}

static int32_t fetch_impl(krk_sparse* t, const uint64_t* ids, int64_t n, uint8_t* found, float* vals,
                          int32_t state_type, float* state, int64_t* steps, uint32_t flags, bool raw_word);

int32_t krk_sparse_fetch(krk_sparse* t, const uint64_t* ids, int64_t n, uint8_t* found, float* vals,
                         int32_t state_type, float* state, int64_t* steps, uint32_t flags) {
  return fetch_impl(t, ids, n, found, vals, state_type, state, steps, flags, false);
}

static int32_t fetch_impl(krk_sparse* t, const uint64_t* ids, int64_t n, uint8_t* found, float* vals,
                          int32_t state_type, float* state, int64_t* steps, uint32_t flags, bool raw_word) {
  KRK_TRY(check_table(t));
  KRK_TRY(check_flags(flags));
  if (flags & KRK_ASYNC) return KRK_E_ARGUMENT;
  if (n < 0 || (n > 0 && !ids)) return KRK_E_ARGUMENT;
  if (state && (state_type < 1 || state_type >= KRK_ST_COUNT)) return KRK_E_ARGUMENT;
  if (n > max_ids_per_launch(t->group)) {
    set_error("at most %lld ids per call for this row width; split the request",
              (long long)max_ids_per_launch(t->group));
    return KRK_E_CAPACITY;
  }
  std::lock_guard<std::mutex> lk(t->mu);
  if (n == 0) return sparse_finish(t, 0);
  const bool host = !(flags & KRK_DEVICE_PTRS);
  const size_t cells = (size_t)n * t->dim;
  // the four staging buffers of a table carry ids, values, state; flags and counters of a
  // host call travel through the work space instead
  const uint64_t* d_ids;
  float* d_vals = nullptr;
  float* d_state = nullptr;
  unsigned char* d_found = found;
  long long* d_steps = reinterpret_cast<long long*>(steps);
  KRK_TRY(t->input(ids, (size_t)n, flags, 0, &d_ids));
  if (vals) KRK_TRY(t->output(vals, cells, flags, 1, &d_vals));
  if (state) KRK_TRY(t->output(state, cells, flags, 2, &d_state));
  if (host && (found || steps)) {
    const size_t steps_bytes = (size_t)n * sizeof(long long);
    KRK_TRY(t->scratch[5].reserve(steps_bytes + (size_t)n + 16));
    d_steps = steps ? t->scratch[5].as<long long>() : nullptr;
    d_found = found ? reinterpret_cast<unsigned char*>(t->scratch[5].as<char>() + steps_bytes) : nullptr;
  }
  const int per_block = kBlock / t->group;
  const dim3 grid(grid_for(n, per_block)), block(kBlock);
  const int state_off = state ? t->col_off[state_type] : -1;
  if (t->vec == 4) {
    hipLaunchKernelGGL((fetch_kernel<4>), grid, block, 0, t->stream, t->view(), d_ids, n, d_found, d_vals,
                       state_off, d_state, t->meta_off, d_steps, raw_word, (int)t->dim, t->elems, t->group);
  } else {
    hipLaunchKernelGGL((fetch_kernel<1>), grid, block, 0, t->stream, t->view(), d_ids, n, d_found, d_vals,
                       state_off, d_state, t->meta_off, d_steps, raw_word, (int)t->dim, t->elems, t->group);
  }
  KRK_HIP(hipGetLastError());
  if (vals) KRK_TRY(t->output_back(vals, cells, flags, 1));
  if (state) KRK_TRY(t->output_back(state, cells, flags, 2));
  if (host && steps)
    KRK_HIP(hipMemcpyAsync(steps, d_steps, (size_t)n * sizeof(long long), hipMemcpyDeviceToHost, t->stream));
  if (host && found) KRK_HIP(hipMemcpyAsync(found, d_found, (size_t)n, hipMemcpyDeviceToHost, t->stream));
  return sparse_finish(t, 0);
}

int32_t krk_sparse_import_state(krk_sparse* t, const uint64_t* ids, int64_t n, int32_t state_type,
                                const float* state, const int64_t* steps, uint32_t flags) {
  KRK_TRY(check_table(t));
  KRK_TRY(check_flags(flags));
  if (n < 0 || (n > 0 && !ids)) return KRK_E_ARGUMENT;
  if (state && (state_type < 1 || state_type >= KRK_ST_COUNT)) return KRK_E_ARGUMENT;
  if (n > max_ids_per_launch(t->group)) {
    set_error("at most %lld ids per call for this row width; split the request",
              (long long)max_ids_per_launch(t->group));
    return KRK_E_CAPACITY;
  }
  std::lock_guard<std::mutex> lk(t->mu);
  if (n == 0 || (!state && !steps)) return sparse_finish(t, flags);
  uint32_t mask = 0;
  if (state) mask |= 1u << state_type;
  // a row that is given a momentum buffer is marked as having one (the flag lives with the counter)
  const bool mark_momentum = state && state_type == KRK_ST_MOMENTUM_BUFFER;
  if (steps || mark_momentum) mask |= 1u << KRK_ST_STEPS;
  KRK_TRY(sparse_ensure_columns(t, mask));
  const uint64_t* d_ids;
  const float* d_state = nullptr;
  const long long* d_steps = nullptr;
  KRK_TRY(t->input(ids, (size_t)n, flags, 0, &d_ids));
  if (state) KRK_TRY(t->input(state, (size_t)n * t->dim, flags, 1, &d_state));
  if (steps) KRK_TRY(t->input(reinterpret_cast<const long long*>(steps), (size_t)n, flags, 2, &d_steps));
  const int per_block = kBlock / t->group;
  const dim3 grid(grid_for(n, per_block)), block(kBlock);
  const int state_off = state ? t->col_off[state_type] : -1;
  if (t->vec == 4) {
    hipLaunchKernelGGL((import_state_kernel<4>), grid, block, 0, t->stream, t->view(), d_ids, n, state_off,
                       d_state, t->meta_off, d_steps, mark_momentum, (int)t->dim, t->elems, t->group);
  } else {
    hipLaunchKernelGGL((import_state_kernel<1>), grid, block, 0, t->stream, t->view(), d_ids, n, state_off,
                       d_state, t->meta_off, d_steps, mark_momentum, (int)t->dim, t->elems, t->group);
  }
  KRK_HIP(hipGetLastError());
  return sparse_finish(t, flags);
}

int32_t krk_sparse_erase(krk_sparse* t, const uint64_t* ids, int64_t n, int64_t* erased, uint32_t flags) {
  KRK_TRY(check_table(t));
  KRK_TRY(check_flags(flags));
  if (flags & KRK_ASYNC) return KRK_E_ARGUMENT;   // the count comes back by value
  if (n < 0 || (n > 0 && !ids)) return KRK_E_ARGUMENT;
  if (n > max_ids_per_launch(kBucket)) {
    set_error("at most %lld ids per call; split the request", (long long)max_ids_per_launch(kBucket));
    return KRK_E_CAPACITY;
  }
  if (erased) *erased = 0;
  std::lock_guard<std::mutex> lk(t->mu);
  KRK_TRY(sparse_finish(t, 0));        // drains the stream and reports what earlier calls left
  KRK_TRY(refresh_rows(t));
  const int64_t rows = t->size_ub;
  if (n == 0 || rows == 0) return KRK_SUCCESS;
  const uint64_t* d_ids;
  KRK_TRY(t->input(ids, (size_t)n, flags, 0, &d_ids));
  // work space: dead[rows] | dead_before[rows] | holes[rows] | movers[rows] | scan scratch | total
  const size_t r4 = ((size_t)rows * 4 + 255) & ~(size_t)255;
  const size_t scan_b = (scan_scratch_bytes(rows) + 255) & ~(size_t)255;
  KRK_TRY(t->scratch[5].reserve(4 * r4 + scan_b + 256));
  char* base = t->scratch[5].as<char>();
  int32_t* dead = reinterpret_cast<int32_t*>(base);
  int32_t* dead_before = reinterpret_cast<int32_t*>(base + r4);
  uint32_t* holes = reinterpret_cast<uint32_t*>(base + 2 * r4);
  uint32_t* movers = reinterpret_cast<uint32_t*>(base + 3 * r4);
  void* scan_tmp = base + 4 * r4;
  int32_t* d_total = reinterpret_cast<int32_t*>(base + 4 * r4 + scan_b);
  KRK_HIP(hipMemsetAsync(dead, 0, (size_t)rows * 4, t->stream));
  const TableView tv = t->view();
  hipLaunchKernelGGL(erase_mark_kernel, dim3(grid_for(n, kBlock / kBucket)), dim3(kBlock), 0, t->stream, tv,
                     d_ids, n, dead);
  KRK_HIP(hipGetLastError());
  KRK_TRY(exclusive_scan_i32(dead, dead_before, rows, d_total, scan_tmp, t->stream));
  int32_t gone = 0;
  KRK_HIP(hipMemcpyAsync(&gone, d_total, sizeof(gone), hipMemcpyDeviceToHost, t->stream));
  KRK_HIP(hipStreamSynchronize(t->stream));
  if (erased) *erased = gone;
  if (gone == 0) return KRK_SUCCESS;
  const int64_t keep = rows - gone;
  if (keep > 0) {
    hipLaunchKernelGGL(erase_plan_kernel, dim3(grid_for(rows, kBlock)), dim3(kBlock), 0, t->stream, dead,
                       dead_before, rows, keep, holes, movers);
    // as many live rows sit at or above `keep` as dead ones below it; that count is
    // dead_before[keep], known only on the device, and at most min(gone, keep)
    int32_t to_move = 0;
    KRK_HIP(hipMemcpyAsync(&to_move, dead_before + keep, sizeof(to_move), hipMemcpyDeviceToHost, t->stream));
    KRK_HIP(hipStreamSynchronize(t->stream));
    if (to_move > 0) {
      hipLaunchKernelGGL(erase_move_kernel, dim3(strided_grid((int64_t)to_move * t->stride)), dim3(kBlock), 0,
                         t->stream, tv, holes, movers, (int64_t)to_move);
    }
    KRK_HIP(hipGetLastError());
  }
  // rows at and above `keep` are free again: a row that is created later must find zeroed
  // optimizer state and a zero step counter there, as in a slab that was never used
  KRK_HIP(hipMemsetAsync(t->recs + keep * t->stride, 0, (size_t)gone * (size_t)t->stride * sizeof(float),
                         t->stream));
  // the index is rebuilt from the keys of the rows that remain
  KRK_HIP(hipMemsetAsync(t->slots, 0xFF, (t->slot_cap + 1) * sizeof(Slot), t->stream));
  if (keep > 0) {
    hipLaunchKernelGGL(reindex_kernel, dim3(grid_for(keep, kBlock)), dim3(kBlock), 0, t->stream, t->slots,
                       t->slot_cap - 1, t->row_key, keep);
  }
  hipLaunchKernelGGL(set_row_count_kernel, dim3(1), dim3(64), 0, t->stream, t->counters, (uint32_t)keep);
  KRK_HIP(hipGetLastError());
  KRK_HIP(hipStreamSynchronize(t->stream));
  t->size_ub = keep;
  t->layout_version++;
  return KRK_SUCCESS;
}

int32_t krk_sparse_select_routed(krk_sparse* t, uint64_t table_id, const uint64_t* ring_hash,
                                 const uint64_t* ring_node, int64_t ring_n, uint64_t node_id, int32_t owned,
                                 uint64_t* ids, int64_t capacity, int64_t* count, uint32_t flags) {
  KRK_TRY(check_table(t));
  KRK_TRY(check_flags(flags));
  if (flags & KRK_ASYNC) return KRK_E_ARGUMENT;   // the count comes back by value
  if (!count || ring_n < 0 || ring_n > (1 << 24) || (ring_n > 0 && (!ring_hash || !ring_node)) || capacity < 0 ||
      (capacity > 0 && !ids))
    return KRK_E_ARGUMENT;
  for (int64_t i = 1; i < ring_n; ++i) {
    if (ring_hash[i - 1] > ring_hash[i]) {
      set_error("krk_sparse_select_routed: the ring must be in ascending hash order");
      return KRK_E_ARGUMENT;
    }
  }
  *count = 0;
  std::lock_guard<std::mutex> lk(t->mu);
  KRK_TRY(sparse_finish(t, 0));
  KRK_TRY(refresh_rows(t));
  const int64_t rows = t->size_ub;
  if (rows == 0) return KRK_SUCCESS;
  // work space: flag[rows] | rank[rows] | scan scratch | total | ring hashes | ring nodes
  const size_t r4 = ((size_t)rows * 4 + 255) & ~(size_t)255;
  const size_t scan_b = (scan_scratch_bytes(rows) + 255) & ~(size_t)255;
  const size_t ring_b = ((size_t)ring_n * 8 + 255) & ~(size_t)255;
  KRK_TRY(t->scratch[5].reserve(2 * r4 + scan_b + 256 + 2 * ring_b + 16));
  char* base = t->scratch[5].as<char>();
  int32_t* flag = reinterpret_cast<int32_t*>(base);
  int32_t* rank = reinterpret_cast<int32_t*>(base + r4);
  void* scan_tmp = base + 2 * r4;
  int32_t* d_total = reinterpret_cast<int32_t*>(base + 2 * r4 + scan_b);
  unsigned long long* d_ring_hash = reinterpret_cast<unsigned long long*>(base + 2 * r4 + scan_b + 256);
  unsigned long long* d_ring_node = reinterpret_cast<unsigned long long*>(base + 2 * r4 + scan_b + 256 + ring_b);
  if (ring_n) {
    // pageable sources: these copies return once the bytes are staged
    KRK_HIP(hipMemcpyAsync(d_ring_hash, ring_hash, (size_t)ring_n * 8, hipMemcpyHostToDevice, t->stream));
    KRK_HIP(hipMemcpyAsync(d_ring_node, ring_node, (size_t)ring_n * 8, hipMemcpyHostToDevice, t->stream));
  }
  // a few thousand workgroups that stride over the rows: each stages the ring once
  const unsigned flag_grid = (unsigned)std::min<int64_t>(grid_for(rows, kBlock), 256 * 16);
  hipLaunchKernelGGL(route_flag_kernel, dim3(flag_grid), dim3(kBlock), 0, t->stream, t->row_key, rows,
                     route_hash64(table_id), d_ring_hash, d_ring_node, (int)ring_n, (unsigned long long)node_id,
                     owned != 0, flag);
  KRK_HIP(hipGetLastError());
  KRK_TRY(exclusive_scan_i32(flag, rank, rows, d_total, scan_tmp, t->stream));
  int32_t total = 0;
  KRK_HIP(hipMemcpyAsync(&total, d_total, sizeof(total), hipMemcpyDeviceToHost, t->stream));
  KRK_HIP(hipStreamSynchronize(t->stream));
  *count = total;
  if (total > capacity) {
    set_error("krk_sparse_select_routed: %lld ids selected, room for %lld", (long long)total, (long long)capacity);
    return KRK_E_CAPACITY;
  }
  if (total == 0) return KRK_SUCCESS;
  unsigned long long* d_ids;
  KRK_TRY(t->output(reinterpret_cast<unsigned long long*>(ids), (size_t)total, flags, 0, &d_ids));
  hipLaunchKernelGGL(route_emit_kernel, dim3(grid_for(rows, kBlock)), dim3(kBlock), 0, t->stream, t->row_key, rows,
                     flag, rank, d_ids);
  KRK_HIP(hipGetLastError());
  KRK_TRY(t->output_back(reinterpret_cast<unsigned long long*>(ids), (size_t)total, flags, 0));
  KRK_HIP(hipStreamSynchronize(t->stream));
  return KRK_SUCCESS;
}

// The routing call owns no table: its work space is kept between calls under one lock, and it
// runs on the null stream.
static std::mutex g_route_mu;
static DeviceBuffer g_route_pool;
static char* g_route_pinned = nullptr;      // page-locked staging for the ring and the counts
static size_t g_route_pinned_bytes = 0;
static std::vector<char> g_route_last;        // the ring block the device holds ...
static const void* g_route_on_device = nullptr;   // ... and where (null: nothing usable there)

int32_t krk_route_ids(uint64_t table_id, const uint64_t* ring_hash, const uint64_t* ring_node, int64_t ring_n,
                      const uint64_t* ids, int64_t n, uint64_t* owner, int64_t* perm, uint64_t* node_ids,
                      int64_t* counts, int64_t node_capacity, int64_t* n_nodes, uint32_t flags) {
  KRK_TRY(check_flags(flags));
  if (flags & KRK_ASYNC) return KRK_E_ARGUMENT;   // the counts come back by value
  if (!n_nodes || ring_n < 0 || ring_n > (1 << 24) || (ring_n > 0 && (!ring_hash || !ring_node)) || n < 0 ||
      (n > 0 && (!ids || !perm)) || node_capacity < 0 || (node_capacity > 0 && (!node_ids || !counts)))
    return KRK_E_ARGUMENT;
  if (n > ((int64_t)1 << 30)) {
    set_error("krk_route_ids handles at most 2^30 ids per call");
    return KRK_E_CAPACITY;
  }
  for (int64_t i = 1; i < ring_n; ++i) {
    if (ring_hash[i - 1] > ring_hash[i]) {
      set_error("krk_route_ids: the ring must be in ascending hash order");
      return KRK_E_ARGUMENT;
    }
  }
  KRK_TRY(ensure_runtime());
  // the nodes of the ring in ascending id order, and each virtual node's index among them
  std::vector<unsigned long long> nodes(ring_node, ring_node + ring_n);
  std::sort(nodes.begin(), nodes.end());
  nodes.erase(std::unique(nodes.begin(), nodes.end()), nodes.end());
  const int64_t m = (int64_t)nodes.size();
  *n_nodes = m;
  if (m > node_capacity) {
    set_error("krk_route_ids: the ring has %lld nodes, room for %lld", (long long)m, (long long)node_capacity);
    return KRK_E_CAPACITY;
  }
  if (m > kRouteMaxNodes) {
    set_error("krk_route_ids handles rings of at most %d nodes", kRouteMaxNodes);
    return KRK_E_CAPACITY;
  }
  for (int64_t k = 0; k < m; ++k) {
    node_ids[k] = nodes[(size_t)k];
    counts[k] = 0;
  }
  if (n == 0) return KRK_SUCCESS;
  if (m == 0) {
    set_error("krk_route_ids: an empty ring owns nothing");   // Router::Hit on an empty ring has no answer
    return KRK_E_ARGUMENT;
  }
  std::vector<uint32_t> ring_rank((size_t)ring_n);
  for (int64_t i = 0; i < ring_n; ++i)
    ring_rank[(size_t)i] = (uint32_t)(std::lower_bound(nodes.begin(), nodes.end(), ring_node[i]) - nodes.begin());

  const bool host = !(flags & KRK_DEVICE_PTRS);
  const int64_t blocks = (n + kBlock - 1) / kBlock;
  const auto r256 = [](size_t b) { return (b + 255) & ~(size_t)255; };
  const size_t ring_hash_b = r256((size_t)ring_n * 8), ring_rank_b = r256((size_t)ring_n * 4);
  const size_t nodes_b = r256((size_t)m * 8), count_b = r256((size_t)m * 4);
  const size_t rank8_b = r256((size_t)n), bc_b = r256((size_t)m * (size_t)blocks * 4);
  const size_t scan_b = r256(scan_scratch_bytes(m * blocks));
  const size_t n8 = r256((size_t)n * 8);
  std::lock_guard<std::mutex> pool_lock(g_route_mu);
  const size_t pool_before = g_route_pool.bytes;
  const int32_t pool_rc = g_route_pool.reserve(ring_hash_b + ring_rank_b + nodes_b + count_b + rank8_b + bc_b +
                                               scan_b + 256 + (host ? 3 * n8 : 0));
  if (g_route_pool.bytes != pool_before || pool_rc != KRK_SUCCESS) g_route_on_device = nullptr;   // a new allocation
  KRK_TRY(pool_rc);
  char* cur = g_route_pool.as<char>();
  unsigned long long* d_ring_hash = reinterpret_cast<unsigned long long*>(cur); cur += ring_hash_b;
  uint32_t* d_ring_rank = reinterpret_cast<uint32_t*>(cur); cur += ring_rank_b;
  unsigned long long* d_nodes = reinterpret_cast<unsigned long long*>(cur); cur += nodes_b;
  cur += count_b;
  uint8_t* d_rank8 = reinterpret_cast<uint8_t*>(cur); cur += rank8_b;
  int32_t* d_bc = reinterpret_cast<int32_t*>(cur); cur += bc_b;
  void* d_scan = cur; cur += scan_b;
  int32_t* d_total = reinterpret_cast<int32_t*>(cur); cur += 256;
  const uint64_t* d_ids = ids;
  unsigned long long* d_owner = reinterpret_cast<unsigned long long*>(owner);
  long long* d_perm = reinterpret_cast<long long*>(perm);
  hipStream_t st = nullptr;
  if (host) {
    uint64_t* s_ids = reinterpret_cast<uint64_t*>(cur);
    d_owner = owner ? reinterpret_cast<unsigned long long*>(cur + n8) : nullptr;
    d_perm = reinterpret_cast<long long*>(cur + 2 * n8);
    KRK_HIP(hipMemcpy(s_ids, ids, (size_t)n * 8, hipMemcpyHostToDevice));
    d_ids = s_ids;
  }
  // The ring, its ranks and the node list travel in one copy out of page-locked memory, and only
  // when they differ from what the last call left on the device (rings change with the
  // cluster's membership, not between requests). The counts are written by the device straight
  // into page-locked memory: the call waits for the stream once and copies nothing back.
  const size_t up_b = ring_hash_b + ring_rank_b + nodes_b;
  if (g_route_pinned_bytes < up_b + count_b) {
    if (g_route_pinned) (void)hipHostFree(g_route_pinned);
    g_route_pinned = nullptr;
    g_route_pinned_bytes = 0;
    g_route_on_device = nullptr;
    KRK_HIP(hipHostMalloc((void**)&g_route_pinned, 2 * (up_b + count_b), hipHostMallocDefault));
    g_route_pinned_bytes = 2 * (up_b + count_b);
  }
  const bool same_ring = g_route_on_device == (const void*)d_ring_hash && g_route_last.size() == up_b &&
                         std::memcmp(g_route_last.data(), ring_hash, (size_t)ring_n * 8) == 0 &&
                         std::memcmp(g_route_last.data() + ring_hash_b, ring_rank.data(), (size_t)ring_n * 4) == 0 &&
                         std::memcmp(g_route_last.data() + ring_hash_b + ring_rank_b, nodes.data(), (size_t)m * 8) == 0;
  int32_t* h_count = reinterpret_cast<int32_t*>(g_route_pinned + up_b);
  int32_t* d_count = nullptr;
  KRK_HIP(hipHostGetDevicePointer((void**)&d_count, h_count, 0));
  if (!same_ring) {
    g_route_on_device = nullptr;
    g_route_last.assign(up_b, 0);
    std::memcpy(g_route_last.data(), ring_hash, (size_t)ring_n * 8);
    std::memcpy(g_route_last.data() + ring_hash_b, ring_rank.data(), (size_t)ring_n * 4);
    std::memcpy(g_route_last.data() + ring_hash_b + ring_rank_b, nodes.data(), (size_t)m * 8);
    std::memcpy(g_route_pinned, g_route_last.data(), up_b);
    KRK_HIP(hipMemcpyAsync(d_ring_hash, g_route_pinned, up_b, hipMemcpyHostToDevice, st));
  }
  hipLaunchKernelGGL(route_rank_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, st, d_ids, n,
                     (unsigned long long)route_hash64(table_id), d_ring_hash, d_ring_rank, (int)ring_n, d_nodes,
                     (int)m, d_owner, d_rank8, d_bc);
  KRK_HIP(hipGetLastError());
  KRK_TRY(exclusive_scan_i32(d_bc, d_bc, m * blocks, d_total, d_scan, st));
  hipLaunchKernelGGL(route_counts_kernel, dim3(1), dim3(kRouteMaxNodes), 0, st, d_bc, blocks, (int)m, (int32_t)n,
                     d_count);
  hipLaunchKernelGGL(route_scatter_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, st, d_rank8, n, d_bc, d_perm);
  KRK_HIP(hipGetLastError());
  if (host) {
    if (owner) KRK_HIP(hipMemcpy(owner, d_owner, (size_t)n * 8, hipMemcpyDeviceToHost));
    KRK_HIP(hipMemcpy(perm, d_perm, (size_t)n * 8, hipMemcpyDeviceToHost));
  }
  KRK_HIP(hipStreamSynchronize(st));
  g_route_on_device = d_ring_hash;   // only now: a call that failed above leaves the ring to be sent again
  for (int64_t k = 0; k < m; ++k) counts[k] = h_count[k];
  return KRK_SUCCESS;
}

// ---------------------------------------------------------------------------
// groups of tables: one launch per combined request
// ---------------------------------------------------------------------------
int32_t krk_group_create(krk_sparse** tables, int32_t n, krk_group** out) {
  if (!tables || !out || n <= 0 || n > kMaxGroupTables) {
    set_error("a group holds 1..%d tables", kMaxGroupTables);
    return KRK_E_ARGUMENT;
  }
  KRK_TRY(ensure_runtime());
  for (int i = 0; i < n; ++i) {
    if (!tables[i] || tables[i]->member_of || tables[i]->dim != tables[0]->dim) {
      set_error("group members must be distinct tables of equal dimension that are in no other group");
      return KRK_E_ARGUMENT;
    }
    for (int j = 0; j < i; ++j)
      if (tables[j] == tables[i]) return KRK_E_ARGUMENT;
  }
  krk_group* g = new (std::nothrow) krk_group();
  if (!g) return KRK_E_DEVICE;
  int32_t rc = g->open_stream();
  if (rc == KRK_SUCCESS) {
    hipError_t e = hipMalloc((void**)&g->d_descs, sizeof(TableDesc) * kMaxGroupTables);
    if (e == hipSuccess)
      e = hipHostMalloc((void**)&g->h_descs, sizeof(TableDesc) * kMaxGroupTables, hipHostMallocDefault);
    if (e != hipSuccess) rc = hip_fail(e, "krk_group_create", __FILE__, __LINE__);
  }
  if (rc != KRK_SUCCESS) {
    if (g->d_descs) (void)hipFree(g->d_descs);
    g->close_stream();
    delete g;
    return rc;
  }
  g->own_stream = g->stream;
  g->dim = tables[0]->dim;
  g->vec = tables[0]->vec;
  g->elems = tables[0]->elems;
  g->group = tables[0]->group;
  for (int i = 0; i < n; ++i) {
    krk_sparse* t = tables[i];
    std::lock_guard<std::mutex> lk(t->mu);
    (void)hipStreamSynchronize(t->stream);
    t->stream = g->stream;   // from now on the table's own calls are ordered with the group's
    t->member_of = g;
    g->tables.push_back(t);
    g->versions.push_back(~0ull);
  }
  *out = g;
  return KRK_SUCCESS;
}

int32_t krk_group_destroy(krk_group* g) {
  if (!g) return KRK_SUCCESS;
  (void)hipStreamSynchronize(g->stream);   // also when the group runs on the null stream
  for (krk_sparse* t : g->tables) {
    std::lock_guard<std::mutex> lk(t->mu);
    t->stream = t->own_stream;
    t->member_of = nullptr;
  }
  if (g->d_descs) (void)hipFree(g->d_descs);
  if (g->h_descs) (void)hipHostFree(g->h_descs);
  for (auto& b : g->scratch) b.release();
  g->notes.release();
  g->stream = g->own_stream;
  g->close_stream();
  delete g;
  return KRK_SUCCESS;
}

int32_t krk_group_set_stream(krk_group* g, void* stream) {
  if (!g) return KRK_E_ARGUMENT;
  KRK_TRY(ensure_runtime());
  GroupLock lk(g);
  hipStream_t next = stream == KRK_OWN_STREAM ? g->own_stream : reinterpret_cast<hipStream_t>(stream);
  if (next == g->stream) return KRK_SUCCESS;
  // what is enqueued on the old stream must be complete before work on the new one may follow
  KRK_TRY(group_finish(g, 0));
  g->stream = next;
  for (krk_sparse* t : g->tables) t->stream = next;
  return KRK_SUCCESS;
}

}  // extern "C"

// The 64-bit word of each row as it is stored (counter and "has a momentum buffer" flag), zero
// for ids that are absent: what the table-file writer needs besides krk_sparse_fetch.
int32_t krk::sparse_fetch_words(krk_sparse* t, const uint64_t* ids, int64_t n, int64_t* words) {
  return fetch_impl(t, ids, n, nullptr, nullptr, 1, nullptr, words, 0, true);
}

// Uploads the layouts of tables that moved since the last call.
int32_t krk::group_refresh(krk_group* g) {
  bool dirty = false;
  for (size_t i = 0; i < g->tables.size(); ++i) {
    krk_sparse* t = g->tables[i];
    if (g->versions[i] == t->layout_version) continue;
    TableDesc& d = g->h_descs[i];
    d.tv = t->view();
    d.init = t->initk;
    memcpy(d.col_off, t->col_off, sizeof(d.col_off));
    d.meta_off = t->meta_off;
    g->versions[i] = t->layout_version;
    dirty = true;
  }
  if (dirty) {
    // in-flight launches read the old array: wait for them before it is overwritten
    KRK_HIP(hipStreamSynchronize(g->stream));
    KRK_HIP(hipMemcpyAsync(g->d_descs, g->h_descs, sizeof(TableDesc) * g->tables.size(),
                           hipMemcpyHostToDevice, g->stream));
  }
  return KRK_SUCCESS;
}

int32_t krk::group_plan(krk_group* g, const int64_t* offsets, GroupCall* call, int64_t* total, int per_block) {
  const int n = (int)g->tables.size();
  if (per_block <= 0) per_block = kBlock / g->group;
  call->n_tables = n;
  call->even_blocks = 0;
  uint64_t blocks = 0, widest = 0;
  if (offsets[0] != 0) return KRK_E_ARGUMENT;
  for (int i = 0; i < n; ++i) {
    const int64_t cnt = offsets[i + 1] - offsets[i];
    if (cnt < 0) {
      set_error("offsets must not decrease");
      return KRK_E_ARGUMENT;
    }
    call->block_start[i] = (uint32_t)blocks;
    call->row_start[i] = offsets[i];
    const uint64_t mine = (uint64_t)((cnt + per_block - 1) / per_block);
    blocks += mine;
    if (mine > widest) widest = mine;
  }
  // Members of similar size (the usual combined request): give each the same number of
  // workgroups. The surplus workgroups find no position of theirs and leave at once.
  if (widest > 0 && widest * (uint64_t)n <= blocks + blocks / 4 + (uint64_t)n) {
    call->even_blocks = (uint32_t)widest;
    for (int i = 0; i < n; ++i) call->block_start[i] = (uint32_t)(widest * (uint64_t)i);
    blocks = widest * (uint64_t)n;
  }
  if (blocks * (uint64_t)kBlock >= 0x7FFFFFFFull) {
    set_error("combined request too large for one launch; split it");
    return KRK_E_CAPACITY;
  }
  call->block_start[n] = (uint32_t)blocks;
  call->row_start[n] = offsets[n];
  *total = offsets[n];
  return KRK_SUCCESS;
}

int32_t krk::group_finish(krk_group* g, uint32_t flags) {
  if (flags & KRK_ASYNC) return KRK_SUCCESS;
  // one wait for all members: they share the group's stream
  for (krk_sparse* t : g->tables)
    KRK_HIP(hipMemcpyAsync(t->host_counters, t->counters, 16, hipMemcpyDeviceToHost, g->stream));
  KRK_HIP(hipStreamSynchronize(g->stream));
  int32_t first = KRK_SUCCESS;
  for (krk_sparse* t : g->tables) {
    const int32_t rc = krk::collect_counters(t);
    if (rc != KRK_SUCCESS && first == KRK_SUCCESS) first = rc;
  }
  return first;
}

extern "C" {

int32_t krk_group_sync(krk_group* g) {
  if (!g) return KRK_E_ARGUMENT;
  KRK_TRY(ensure_runtime());
  GroupLock lk(g);
  return group_finish(g, 0);
}

// Lanes of a workgroup of the combined kernels for wide rows. Rows of 64 floats take 128: their
// launches are bound by what a compute unit moves, and the 6162 wavefronts of the benchmark's
// request come to 6.02 workgroups of 256 lanes a unit, i.e. seven on some and six on the others
// (a step at dim 64: 42.7 us with 256 lanes, 41.7 us with 128; rows of 16 and 32 floats lose with 128).
static int group_wide_block(int group) { return group == 16 ? 128 : kBlock; }

int32_t krk_group_pull(krk_group* g, const uint64_t* ids, const int64_t* offsets, float* out,
                       uint32_t flags) {
  if (!g || !offsets) return KRK_E_ARGUMENT;
  KRK_TRY(ensure_runtime());
  KRK_TRY(check_flags(flags));
  GroupLock lk(g);
  GroupCall call;
  int64_t total = 0;
  const bool wide = g->vec == 4 && pull_is_wide(g->group, g->elems);
  KRK_TRY(group_plan(g, offsets, &call, &total, wide ? (group_wide_block(g->group) / kWave) * kWideIds : 0));
  if (total == 0) return group_finish(g, flags);
  if (!ids || !out) return KRK_E_ARGUMENT;
  if ((flags & KRK_DEVICE_PTRS) && g->vec == 4 && !aligned16(out)) return KRK_E_ARGUMENT;
  for (size_t i = 0; i < g->tables.size(); ++i) {
    krk_sparse* t = g->tables[i];
    const int64_t cnt = offsets[i + 1] - offsets[i];
    if (cnt == 0) {
      call.epoch[i] = t->epoch;
      continue;
    }
    KRK_TRY(sparse_ensure_room(t, cnt));
    KRK_TRY(sparse_next_epoch(t, cnt));
    call.epoch[i] = t->epoch;
  }
  KRK_TRY(group_refresh(g));
  const uint64_t* d_ids;
  float* d_out;
  KRK_TRY(g->input(ids, (size_t)total, flags, 0, &d_ids));
  KRK_TRY(g->output(out, (size_t)total * g->dim, flags, 1, &d_out));
  const dim3 grid(call.block_start[call.n_tables]), block(wide ? group_wide_block(g->group) : kBlock);
  // KRK_NOTE_ROWS: the row of every position stays behind
  uint32_t* notes = nullptr;
  if (flags & KRK_NOTE_ROWS) {
    g->noted_ids = nullptr;
    if (flags & KRK_DEVICE_PTRS) {
      KRK_TRY(g->notes.reserve((size_t)total * sizeof(uint32_t)));
      notes = g->notes.as<uint32_t>();
    }
  }
  // While the members' tables are being filled (see pull_enqueue) the request takes the two
  // launches of a large pull, member by member.
  bool filling = false;
  for (krk_sparse* t : g->tables)
    if (t->host_inserted && __atomic_exchange_n(t->host_inserted, 0u, __ATOMIC_RELAXED) != 0u) filling = true;
  if (filling && total >= kTwoLaunchWhileFilling) {
    GroupFill fill{};
    const int per_block = wide ? (group_wide_block(g->group) / kWave) * kWideIds : kBlock / g->group;
    uint64_t words = 0;
    for (size_t i = 0; i < g->tables.size(); ++i) {
      const int64_t cnt = offsets[i + 1] - offsets[i];
      fill.todo_start[i] = (uint32_t)words;
      if (cnt <= 0) continue;
      krk_sparse* t = g->tables[i];
      words += (uint64_t)kQueues * (uint64_t)queue_capacity(cnt, per_block);
      if (t->pull_parity) fill.parity_bits |= 1u << i;
      t->pull_parity ^= 1;
    }
    KRK_TRY(g->todo.reserve((size_t)words * sizeof(uint32_t)));
    uint32_t* todo = g->todo.as<uint32_t>();
    const dim3 missing_grid((unsigned)call.n_tables * kGroupMissPerTable), missing_block(kMissBlock);
    if (wide && g->group == 8) {
      hipLaunchKernelGGL((group_pull_resident_wide_kernel<4, 2>), grid, block, 0, g->stream, g->d_descs, call, fill,
                         d_ids, d_out, todo, (int)g->dim, g->elems, notes);
    } else if (wide && g->group == 16) {
      hipLaunchKernelGGL((group_pull_resident_wide_kernel<4, 4>), grid, block, 0, g->stream, g->d_descs, call, fill,
                         d_ids, d_out, todo, (int)g->dim, g->elems, notes);
    } else if (wide) {
      hipLaunchKernelGGL((group_pull_resident_wide_kernel<4, 8>), grid, block, 0, g->stream, g->d_descs, call, fill,
                         d_ids, d_out, todo, (int)g->dim, g->elems, notes);
    } else if (g->vec == 4) {
      hipLaunchKernelGGL((group_pull_resident_kernel<4>), grid, block, 0, g->stream, g->d_descs, call, fill, d_ids,
                         d_out, todo, (int)g->dim, g->elems, g->group, notes);
    } else {
      hipLaunchKernelGGL((group_pull_resident_kernel<1>), grid, block, 0, g->stream, g->d_descs, call, fill, d_ids,
                         d_out, todo, (int)g->dim, g->elems, g->group, notes);
    }
    if (g->vec == 4) {
      hipLaunchKernelGGL((group_pull_missing_kernel<4>), missing_grid, missing_block, 0, g->stream, g->d_descs, call,
                         fill, d_ids, d_out, todo, per_block, (int)g->dim, g->elems, g->group, notes);
    } else {
      hipLaunchKernelGGL((group_pull_missing_kernel<1>), missing_grid, missing_block, 0, g->stream, g->d_descs, call,
                         fill, d_ids, d_out, todo, per_block, (int)g->dim, g->elems, g->group, notes);
    }
  } else if (wide && g->group == 8) {
    hipLaunchKernelGGL((group_pull_wide_kernel<4, 2>), grid, block, 0, g->stream, g->d_descs, call, d_ids, d_out,
                       (int)g->dim, g->elems, notes);
  } else if (wide && g->group == 16) {
    hipLaunchKernelGGL((group_pull_wide_kernel<4, 4>), grid, block, 0, g->stream, g->d_descs, call, d_ids, d_out,
                       (int)g->dim, g->elems, notes);
  } else if (wide) {
    hipLaunchKernelGGL((group_pull_wide_kernel<4, 8>), grid, block, 0, g->stream, g->d_descs, call, d_ids, d_out,
                       (int)g->dim, g->elems, notes);
  } else if (g->vec == 4) {
    hipLaunchKernelGGL((group_pull_kernel<4>), grid, block, 0, g->stream, g->d_descs, call, d_ids, d_out,
                       (int)g->dim, g->elems, g->group, notes);
  } else {
    hipLaunchKernelGGL((group_pull_kernel<1>), grid, block, 0, g->stream, g->d_descs, call, d_ids, d_out,
                       (int)g->dim, g->elems, g->group, notes);
  }
  KRK_HIP(hipGetLastError());
  if (notes) {
    g->noted_ids = ids;
    g->noted_offsets.assign(offsets, offsets + call.n_tables + 1);
    g->noted_versions.clear();
    for (krk_sparse* t : g->tables) g->noted_versions.push_back(t->layout_version);
  }
  if (flags & KRK_ASYNC) {
    bool any = false;
    for (krk_sparse* t : g->tables) any = any || sparse_near_full(t);
    if (any) KRK_TRY(sparse_publish(g->tables.data(), (int)g->tables.size(), g->stream));
  }
  KRK_TRY(g->output_back(out, (size_t)total * g->dim, flags, 1));
  return group_finish(g, flags);
}

}  // extern "C"

template <int OPT, int VEC>
static void launch_group_push_opt(krk_group* g, const GroupCall& call, const uint64_t* ids,
                                  const float* grads, float lr, const OptimK& k, const int32_t st[3],
                                  int use_meta, bool wide, const uint32_t* notes) {
  const dim3 grid(call.block_start[call.n_tables]), block(wide ? group_wide_block(g->group) : kBlock);
  const int dim = (int)g->dim;
  if constexpr (VEC == 4) {
    if (wide) {
      if (g->group == 8) {
        hipLaunchKernelGGL((group_push_wide_kernel<OPT, 2>), grid, block, 0, g->stream, g->d_descs, call,
                           ids, grads, dim, g->elems, lr, k, st[0], st[1], st[2], use_meta, notes);
      } else {
        hipLaunchKernelGGL((group_push_wide_kernel<OPT, 4>), grid, block, 0, g->stream, g->d_descs, call,
                           ids, grads, dim, g->elems, lr, k, st[0], st[1], st[2], use_meta, notes);
      }
      return;
    }
  }
  hipLaunchKernelGGL((group_push_kernel<OPT, VEC>), grid, block, 0, g->stream, g->d_descs, call, ids, grads,
                     dim, g->elems, g->group, lr, k, st[0], st[1], st[2], use_meta, notes);
}

// wide: the request was laid out for group_push_wide_kernel (group_wide_block lanes a workgroup)
template <int VEC>
static void launch_group_push(krk_group* g, const krk_optim& o, const GroupCall& call,
                              const uint64_t* ids, const float* grads, float lr, bool wide,
                              const uint32_t* notes) {
  const OptimK k = make_optim_k(o);
  int32_t st[3];
  optim_state_slots(o, st);
  const int use_meta = (optim_state_mask(o) >> KRK_ST_STEPS) & 1u;
  switch (o.type) {
    case KRK_SGD: launch_group_push_opt<KRK_SGD, VEC>(g, call, ids, grads, lr, k, st, use_meta, wide, notes); break;
    case KRK_ADAGRAD:
      launch_group_push_opt<KRK_ADAGRAD, VEC>(g, call, ids, grads, lr, k, st, use_meta, wide, notes);
      break;
    case KRK_ADAM: launch_group_push_opt<KRK_ADAM, VEC>(g, call, ids, grads, lr, k, st, use_meta, wide, notes); break;
    default: launch_group_push_opt<KRK_RMSPROP, VEC>(g, call, ids, grads, lr, k, st, use_meta, wide, notes); break;
  }
}

extern "C" {

int32_t krk_group_push(krk_group* g, const krk_optim* o, const uint64_t* ids, const int64_t* offsets,
                       const float* grads, int64_t grad_dim, float lr, uint32_t flags) {
  if (!g || !offsets) return KRK_E_ARGUMENT;
  KRK_TRY(ensure_runtime());
  KRK_TRY(check_flags(flags));
  if (!valid_optim(o)) {
    set_error("optimizer type is not supported");
    return KRK_UNSUPPORTED_OPTIM;
  }
  GroupLock lk(g);
  GroupCall call;
  int64_t total = 0;
  const bool wide = push_is_wide(g->vec, g->group, g->elems);
  KRK_TRY(group_plan(g, offsets, &call, &total, wide ? (group_wide_block(g->group) / kWave) * kWideIds : 0));
  if (total == 0) return group_finish(g, flags);
  if (!ids || !grads) return KRK_E_ARGUMENT;
  if ((flags & KRK_DEVICE_PTRS) && g->vec == 4 && !aligned16(grads)) return KRK_E_ARGUMENT;
  if (grad_dim != g->dim) {
    set_error("gradient width %lld does not match table dimension %lld", (long long)grad_dim,
              (long long)g->dim);
    return KRK_GRADIENT_UNCOMPATIBLE;
  }
  const uint32_t mask = optim_state_mask(*o);
  for (krk_sparse* t : g->tables) KRK_TRY(sparse_ensure_columns(t, mask));
  KRK_TRY(group_refresh(g));
  const uint64_t* d_ids;
  const float* d_g;
  KRK_TRY(g->input(ids, (size_t)total, flags, 0, &d_ids));
  KRK_TRY(g->input(grads, (size_t)total * g->dim, flags, 1, &d_g));
  for (int i = 0; i < call.n_tables; ++i) call.epoch[i] = 0;
  const uint32_t* notes = noted_rows(g, ids, offsets, flags);   // KRK_IDS_AS_PULLED: no second look-up
  if (g->vec == 4) {
    launch_group_push<4>(g, *o, call, d_ids, d_g, lr, wide, notes);
  } else {
    launch_group_push<1>(g, *o, call, d_ids, d_g, lr, false, notes);
  }
  KRK_HIP(hipGetLastError());
  return group_finish(g, flags);
}

}  // extern "C"
