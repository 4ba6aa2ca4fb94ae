// The worker-side half of a sparse push, moved onto the device and fused with the table update:
//   krk_dedup            Emitter::PullSparseTableImpl's dedup (worker/emitter.cc:131-149)
//   krk_sparse_push_raw  Emitter::PushSparseTable's dedup + duplicate-gradient sum
//                        (worker/emitter.cc:510-531) followed by SparseTable::Push
//
// push_raw never builds the unique list. Positions are sorted by the row their id maps to
// (stable, so equal rows keep position order), then a tiled segmented reduction walks the
// sorted sequence: every group of lanes owns a fixed-size tile, sums each run of equal rows in
// registers and, when a run lies wholly inside the tile, applies the optimizer to that row at
// once. Runs that touch a tile border meet the other tiles' pieces in the workgroup's LDS; only
// a run that crosses the workgroup's own border leaves a partial sum in a carry list, which is
// itself a sorted sequence of (row, partial) and is reduced by the same kernel again until one
// workgroup is left. Work per group is bounded by the tile size however skewed the ids are, and
// the order of additions is fixed, so results do not change from run to run.
#include <cstring>
#include <new>


#include "sparse_internal.h"

namespace krk {

constexpr int kBlock = 256;
constexpr uint32_t kNoRow = 0xFFFFFFFFu;

template <int VEC>
__device__ __forceinline__ void vload(const float* p, float (&v)[VEC]) {
  if constexpr (VEC == 4) {
    const float4 x = *reinterpret_cast<const float4*>(p);
    v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
  } else {
    v[0] = *p;
  }
}
// A row that is read exactly once (the gradient rows a reduction gathers): non-temporal, so the
// half gigabyte that passes through does not push the table's records out of the caches.
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
// The same accesses through pointers the compiler is told lie in global memory. A table's record
// pointer that a kernel reads out of a descriptor is a generic pointer to the compiler, which
// then uses flat instructions; those count as LDS operations too, so every wait for an LDS read
// (the sorted positions, the run starts) would also wait for the records requested before it.
#define KRK_GLOBAL __attribute__((address_space(1)))
template <int VEC>
__device__ __forceinline__ void gload(const float* p, float (&v)[VEC]) {
  if constexpr (VEC == 4) {
    const vfloat4_t x = *(const KRK_GLOBAL vfloat4_t*)p;
    v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
  } else {
    v[0] = *(const KRK_GLOBAL float*)p;
  }
}
template <int VEC>
__device__ __forceinline__ void gstore_once(float* p, const float (&v)[VEC]) {
  if constexpr (VEC == 4) {
    const vfloat4_t x = {v[0], v[1], v[2], v[3]};
    __builtin_nontemporal_store(x, (KRK_GLOBAL vfloat4_t*)p);
  } else {
    __builtin_nontemporal_store(v[0], (KRK_GLOBAL float*)p);
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

static inline unsigned grid_for(int64_t items, int per_block) {
  return (unsigned)((items + per_block - 1) / per_block);
}

// ---------------------------------------------------------------------------
// dedup in first-occurrence order with a request-local hash index
// ---------------------------------------------------------------------------
struct DSlot {
  unsigned long long key;
  uint32_t minpos;   // smallest position holding this id
  uint32_t uidx;     // its index in the unique list
};

// Equal ids are folded inside the workgroup first, through a small hash table in LDS: the lane
// that claims an LDS entry speaks for every position of that id in the workgroup's 1024
// consecutive positions (the entry collects their smallest position), and only it goes to the
// request-wide index. An id that fills a quarter of the request then costs one global probe
// and at most one atomic per workgroup instead of 256, and a workgroup of all-distinct ids pays
// one LDS atomic per lane rather than a vote per distinct id.
constexpr int kDedupBlock = 1024;
constexpr int kDedupLds = 2048;   // entries: at most half full

__global__ __launch_bounds__(kDedupBlock) void dedup_claim_kernel(DSlot* slots, uint64_t mask,
                                                                  const uint64_t* __restrict__ ids, int64_t n,
                                                                  uint32_t* __restrict__ slot_of,
                                                                  uint32_t first_block) {
  __shared__ unsigned long long lkey[kDedupLds + 1];   // the last entry belongs to the all-ones id
  __shared__ uint32_t lmin[kDedupLds + 1];
  __shared__ uint32_t lidx[kDedupLds + 1];
  for (int i = threadIdx.x; i <= kDedupLds; i += kDedupBlock) {
    lkey[i] = kEmptyKey;
    lmin[i] = 0xFFFFFFFFu;
  }
  __syncthreads();
  const int64_t p = (int64_t)(blockIdx.x + first_block) * kDedupBlock + threadIdx.x;
  const bool active = p < n;
  const unsigned long long id = active ? ids[p] : 0ull;
  int entry = kDedupLds;
  bool owner = false;
  if (active) {
    if (id == kEmptyKey) {
      owner = atomicCAS(&lkey[kDedupLds], kEmptyKey, 0ull) == kEmptyKey;
    } else {
      entry = (int)(mix64(id) >> 32) & (kDedupLds - 1);   // high bits: the index below uses the low ones
      for (;;) {
        const unsigned long long old = atomicCAS(&lkey[entry], kEmptyKey, id);
        if (old == kEmptyKey || old == id) {
          owner = old == kEmptyKey;
          break;
        }
        entry = (entry + 1) & (kDedupLds - 1);
      }
    }
    atomicMin(&lmin[entry], (uint32_t)p);
  }
  __syncthreads();
  if (owner) {
    uint64_t idx;
    if (id == kEmptyKey) {
      idx = mask + 1;   // the all-ones id owns the extra last slot
    } else {
      idx = mix64(id) & mask;
      for (uint64_t t = 0; t <= mask; ++t) {
        // A plain (cacheable) load: a key never changes once it is set, so a hit is final.
        // A stale "empty" only costs the CAS below.
        unsigned long long key = slots[idx].key;
        if (key == kEmptyKey) {
          const unsigned long long old = atomicCAS(&slots[idx].key, kEmptyKey, id);
          key = old == kEmptyKey ? id : old;
        }
        if (key == id) break;
        idx = (idx + 1) & mask;
      }
    }
    // minpos only ever decreases, so a stale (cached) read can at worst cause a redundant
    // atomic; later workgroups mostly find a smaller position already there and skip it.
    const uint32_t first = lmin[entry];
    if (slots[idx].minpos > first) atomicMin(&slots[idx].minpos, first);
    lidx[entry] = (uint32_t)idx;
  }
  __syncthreads();
  if (active) slot_of[p] = lidx[entry];
}

__global__ __launch_bounds__(kBlock) void dedup_flag_kernel(const DSlot* __restrict__ slots,
                                                            const uint32_t* __restrict__ slot_of,
                                                            int64_t n, int32_t* __restrict__ flag) {
  const int64_t p = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (p >= n) return;
  flag[p] = slots[slot_of[p]].minpos == (uint32_t)p ? 1 : 0;
}

// Every position learns its id's index in the unique list from the rank of the id's first
// position, and the first position also writes the id there and leaves the index in the slot
// (one launch: a second one that read the index out of the slot had to wait for this one).
__global__ __launch_bounds__(kBlock) void dedup_emit_kernel(DSlot* slots,
                                                            const uint32_t* __restrict__ slot_of,
                                                            const int32_t* __restrict__ rank,
                                                            const uint64_t* __restrict__ ids, int64_t n,
                                                            uint64_t* __restrict__ uids,
                                                            long long* __restrict__ inv,
                                                            const int32_t* __restrict__ total,
                                                            int32_t* __restrict__ host_total) {
  const int64_t p = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (p >= n) return;
  if (p == 0 && host_total) *host_total = *total;      // the count, where a blocking caller reads it
  DSlot* s = &slots[slot_of[p]];
  const uint32_t first = s->minpos;
  const int32_t r = rank[first];
  if (inv) inv[p] = (long long)r;
  if (first == (uint32_t)p) {
    uids[r] = ids[p];
    s->uidx = (uint32_t)r;
  }
}

// Requests of at most kDedupSmall ids: the whole dedup in one launch of one workgroup. The ids
// sit in LDS; an open-addressing table of positions (a slot holds the smallest position of the
// id that owns it, and the id itself is looked up through that position) replaces the index in
// global memory; a lane owns eight consecutive positions, so one scan over the workgroup gives
// every first occurrence its place in the unique list. The unique ids are compacted in LDS (over
// the ids, which nobody reads after the claims) and every position's slot is kept there too, so
// that both results leave in position order, a wavefront's stores side by side: a lane writing
// its own eight positions touched a 64-byte piece per store, 3.5 us more for 8192 ids.
constexpr int kDedupSmall = 8192;
constexpr int kDedupSmallSlots = 2 * kDedupSmall;
constexpr int kDedupSmallOwn = kDedupSmall / kDedupBlock;
constexpr uint32_t kNoPos = 0xFFFFFFFFu;
static_assert(kDedupSmallSlots <= 65536, "a position's slot is kept in 16 bits");
// Where id number p sits in LDS: one entry is left out after every eight, so that the lanes of a
// wavefront, which own eight consecutive ids each, do not all meet in the same two banks.
__device__ __forceinline__ int dedup_small_at(int p) { return p + (p >> 3); }

__global__ __launch_bounds__(kDedupBlock) void dedup_small_kernel(const uint64_t* __restrict__ ids, int n,
                                                                  uint64_t* __restrict__ uids,
                                                                  long long* __restrict__ inv,
                                                                  int32_t* __restrict__ total,
                                                                  int32_t* __restrict__ host_total) {
  __shared__ unsigned long long sid[kDedupSmall + kDedupSmall / 8];   // the ids by position, then the unique ids
  __shared__ uint32_t tab[kDedupSmallSlots];           // position of the id's first occurrence, then its unique index
  __shared__ uint16_t slot_of[kDedupSmall];
  __shared__ uint32_t wave_total[kDedupBlock / kWave];
  const int t = threadIdx.x;
  // table size by request size: a small request clears and probes a small table
  int bits = 5;
  while ((1 << bits) < 2 * n) ++bits;
  const uint32_t mask = (1u << bits) - 1u;
  for (int i = t; i <= (int)mask; i += kDedupBlock) tab[i] = kNoPos;
  for (int i = t; i < n; i += kDedupBlock) sid[dedup_small_at(i)] = ids[i];
  __syncthreads();
  uint32_t slot[kDedupSmallOwn];
  unsigned long long mine_id[kDedupSmallOwn];
#pragma unroll
  for (int i = 0; i < kDedupSmallOwn; ++i) {
    const int p = t * kDedupSmallOwn + i;
    slot[i] = 0;
    mine_id[i] = 0;
    if (p < n) {
      const unsigned long long id = sid[dedup_small_at(p)];
      uint32_t h = (uint32_t)(mix64(id) >> 32) & mask;
      for (;;) {
        uint32_t q = tab[h];
        if (q == kNoPos) {
          q = atomicCAS(&tab[h], kNoPos, (uint32_t)p);
          if (q == kNoPos) break;                      // the slot is this id's now
        }
        if (sid[dedup_small_at((int)q)] == id) {        // whoever holds it, it is the same id
          atomicMin(&tab[h], (uint32_t)p);
          break;
        }
        h = (h + 1) & mask;
      }
      slot[i] = h;
      mine_id[i] = id;
      slot_of[p] = (uint16_t)h;
    }
  }
  __syncthreads();                                     // the claims are over: nobody reads sid[] by position again
  uint32_t first = 0;                                  // bit i: my position i is its id's first
#pragma unroll
  for (int i = 0; i < kDedupSmallOwn; ++i) {
    const int p = t * kDedupSmallOwn + i;
    if (p < n && tab[slot[i]] == (uint32_t)p) first |= 1u << i;
  }
  // exclusive scan of the counts over the workgroup
  const int lane = t & (kWave - 1), wave = t / kWave;
  const uint32_t mine = (uint32_t)__popc(first);
  uint32_t incl = mine;
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const uint32_t y = __shfl_up(incl, d);
    if (lane >= d) incl += y;
  }
  if (lane == kWave - 1) wave_total[wave] = incl;
  __syncthreads();                                     // also: every first occurrence has been read from the table
  uint32_t rank = incl - mine, all = 0;
  for (int w = 0; w < kDedupBlock / kWave; ++w) {
    const uint32_t x = wave_total[w];
    if (w < wave) rank += x;
    all += x;
  }
#pragma unroll
  for (int i = 0; i < kDedupSmallOwn; ++i) {
    if (first & (1u << i)) {
      sid[dedup_small_at((int)rank)] = mine_id[i];
      tab[slot[i]] = rank;                             // the table now answers with the unique index
      ++rank;
    }
  }
  if (t == 0) {
    *total = (int32_t)all;
    if (host_total) *host_total = (int32_t)all;
  }
  __syncthreads();
  for (int r = t; r < (int)all; r += kDedupBlock) uids[r] = sid[dedup_small_at(r)];
  if (!inv) return;
  for (int p = t; p < n; p += kDedupBlock) inv[p] = (long long)tab[slot_of[p]];
}

// ---------------------------------------------------------------------------
// push_raw stage 1: position -> row number (the sort key), positions as payload
// ---------------------------------------------------------------------------
// bag_of (pooled pushes only): the bag each position belongs to, kNoBag outside every bag.
// Such positions get the skip key without raising the missing-id error. With payload_is_bag
// the sort carries the bag number instead of the position: the reduction then reads the
// bag's gradient row directly.
constexpr uint32_t kNoBag = 0xFFFFFFFFu;

__global__ __launch_bounds__(kBlock) void rows_of_ids_kernel(TableView tv, const uint64_t* __restrict__ ids,
                                                             int64_t n, uint32_t miss_key,
                                                             const uint32_t* __restrict__ bag_of,
                                                             bool payload_is_bag,
                                                             uint32_t* __restrict__ keys,
                                                             uint32_t* __restrict__ pos) {
  const int64_t p = (int64_t)blockIdx.x * (kBlock / kBucket) + threadIdx.x / kBucket;
  const int gl = threadIdx.x & (kBucket - 1);
  const uint32_t bag = (bag_of && p < n) ? bag_of[p] : 0u;
  const bool active = p < n && bag != kNoBag;
  uint32_t r = probe_find(tv, active ? ids[p] : 0, active, gl, kBucket);
  if (p >= n || gl != 0) return;
  if (!active) {
    r = miss_key;
  } else if (r == kEmptyRow) {
    atomicOr(&tv.counters[1], kErrMissingId);
    r = miss_key;
  }
  keys[p] = r;
  if (pos) pos[p] = payload_is_bag ? bag : (uint32_t)p;
}

// The same for a combined request: position p belongs to the member whose [row_start, row_start
// of the next) holds it; its key is (member << row_bits) | row. A missing id raises the error
// on its own member.
__global__ __launch_bounds__(kBlock) void group_rows_of_ids_kernel(const TableDesc* __restrict__ descs,
                                                                   GroupCall call,
                                                                   const uint64_t* __restrict__ ids, int64_t n,
                                                                   int row_bits, uint32_t miss_key,
                                                                   uint32_t* __restrict__ keys,
                                                                   uint32_t* __restrict__ pos) {
  // a workgroup serves one member (call.block_start counts workgroups of kBlock / kBucket
  // positions here), so the member's layout comes in through scalar loads
  int m = 0;
  if (call.even_blocks) {
    m = (int)(blockIdx.x / call.even_blocks);          // members of equal length: no walk
  } else {
    while (m + 1 < call.n_tables && blockIdx.x >= call.block_start[m + 1]) ++m;
  }
  const int64_t p = call.row_start[m] + (int64_t)(blockIdx.x - call.block_start[m]) * (kBlock / kBucket) +
                    threadIdx.x / kBucket;
  const int gl = threadIdx.x & (kBucket - 1);
  const bool active = p < call.row_start[m + 1];
  const TableView tv = descs[m].tv;
  uint32_t r = probe_find(tv, active ? ids[p] : 0, active, gl, kBucket);
  if (!active || gl != 0) return;
  if (r == kEmptyRow) {
    atomicOr(&tv.counters[1], kErrMissingId);
    r = miss_key;
  } else {
    r |= (uint32_t)m << row_bits;
  }
  keys[p] = r;
  if (pos) pos[p] = (uint32_t)p;
}

// ---- pooled pushes: from bag offsets to per-position bag numbers ----------------
__global__ __launch_bounds__(kBlock) void fill_u32_kernel(uint32_t* __restrict__ dst, int64_t n, uint32_t v) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i < n) dst[i] = v;
}

constexpr int kBagLanes = 8;   // lanes that share one bag's positions

__global__ __launch_bounds__(kBlock) void bag_expand_kernel(const long long* __restrict__ offsets, int64_t bags,
                                                            int64_t n, uint32_t* __restrict__ bag_of) {
  const int64_t b = (int64_t)blockIdx.x * (kBlock / kBagLanes) + threadIdx.x / kBagLanes;
  if (b >= bags) return;
  long long lo = offsets[b], hi = offsets[b + 1];
  if (lo < 0) lo = 0;
  if (hi > n) hi = n;
  for (long long p = lo + (threadIdx.x & (kBagLanes - 1)); p < hi; p += kBagLanes) bag_of[p] = (uint32_t)b;
}

// pytorch/py/jagged_ops.cc:303-334 : a mean bag hands every one of its rows grads * ratio,
// ratio = (float)(1.0 / float(len)); computed once per bag here as there.
__global__ __launch_bounds__(kBlock) void bag_scale_kernel(const float* __restrict__ grads,
                                                           const long long* __restrict__ offsets,
                                                           int64_t bags, int dim, float* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= bags * dim) return;
  const int64_t b = i / dim;
  const long long len = offsets[b + 1] - offsets[b];
  const float ratio = len > 0 ? (float)(1.0 / (double)(float)len) : 0.0f;
  out[i] = grads[i] * ratio;
}

// ---------------------------------------------------------------------------
// push_raw stage 3: tiled segmented reduction fused with the optimizer update
// ---------------------------------------------------------------------------
struct ApplyArgs {
  float lr;
  OptimK k;
  int c0, c1, c2, meta_off;
};

// What a closed run does with its sum: one of the four optimizers, or (stand-alone dedup + sum)
// just store it as row `row` of the output.
constexpr int kOptStore = 4;

// A lane's slice of a record: weight and the optimizer's state columns.
template <int VEC>
struct RowRegs {
  float w[VEC], s0[VEC], s1[VEC], s2[VEC];
};

// Requests the lane's slice of row `row`. Kept apart from the update so that a caller can have
// the record on its way while it is still adding up the row's gradient.
template <int OPT, int VEC>
__device__ __forceinline__ void load_row(const TableView& tv, uint32_t row, int e, bool lane_on, const ApplyArgs& a,
                                         RowRegs<VEC>& r) {
  if constexpr (OPT == kOptStore) return;
  const float* rec = tv.recs + (int64_t)row * tv.stride;
  if (lane_on) {
    gload<VEC>(rec + e * VEC, r.w);
    if (a.c0 >= 0) gload<VEC>(rec + a.c0 + e * VEC, r.s0);
    if (a.c1 >= 0) gload<VEC>(rec + a.c1 + e * VEC, r.s1);
    if (a.c2 >= 0) gload<VEC>(rec + a.c2 + e * VEC, r.s2);
  }
}

// The update of row `row` with the summed gradient, on the slice load_row requested.
template <int OPT, int VEC>
__device__ __forceinline__ void finish_row(const TableView& tv, uint32_t row, const float (&gsum)[VEC], int e,
                                           bool lane_on, int gl, bool last_chunk, int dim, const ApplyArgs& a,
                                           RowRegs<VEC>& r) {
  float* rec = tv.recs + (int64_t)row * tv.stride;
  if constexpr (OPT == kOptStore) {
    if (lane_on) vstore<VEC>(rec + e * VEC, gsum);
    return;
  }
  bool first = false;
  float bc1 = 1.0f, bc2 = 1.0f;
  uint64_t steps = 0;
  if (a.meta_off >= 0) {
    const KRK_GLOBAL uint32_t* meta = (const KRK_GLOBAL uint32_t*)(rec + a.meta_off);
    steps = (uint64_t)meta[0] | ((uint64_t)meta[1] << 32);
    if (OPT == KRK_ADAM) {
      steps += 1;                           // the flag bit rides along untouched
    } else {
      first = (steps & kHasMomentumBit) == 0;
      steps |= kHasMomentumBit;
    }
    if (OPT == KRK_ADAM) {
      const float count = (float)(steps & ~kHasMomentumBit);
      bc1 = (float)(1.0 - (double)powf(a.k.beta1, count));
      bc2 = (float)(1.0 - (double)powf(a.k.beta2, count));
    }
  }
  if (lane_on) {
#pragma unroll
    for (int c = 0; c < VEC; ++c) {
      if (a.c0 < 0) r.s0[c] = 0.0f;
      if (a.c1 < 0) r.s1[c] = 0.0f;
      if (a.c2 < 0) r.s2[c] = 0.0f;
      optim_element<OPT>(a.k, a.lr, gsum[c], r.w[c], r.s0[c], r.s1[c], r.s2[c], first, bc1, bc2);
    }
    // a record is written once per request: past the caches, so the kernel ends with no dirty
    // lines to write back
    gstore_once<VEC>(rec + e * VEC, r.w);
    if (a.c0 >= 0) gstore_once<VEC>(rec + a.c0 + e * VEC, r.s0);
    if (a.c1 >= 0) gstore_once<VEC>(rec + a.c1 + e * VEC, r.s1);
    if (a.c2 >= 0) gstore_once<VEC>(rec + a.c2 + e * VEC, r.s2);
  }
  // The counter is read by every chunk of the row before the last chunk advances it.
  if (a.meta_off >= 0 && last_chunk) store_row_word<VEC>(rec + a.meta_off, steps, gl, dim, (int)tv.stride - a.meta_off);
}

// The lane's slice of the record is requested before the 64-bit word is looked at: the bias
// corrections (two powf) then overlap with the loads instead of preceding them.
template <int OPT, int VEC>
__device__ __forceinline__ void apply_row(const TableView& tv, uint32_t row, const float (&gsum)[VEC],
                                          int e, bool lane_on, int gl, bool last_chunk, int dim,
                                          const ApplyArgs& a) {
  RowRegs<VEC> r;
  load_row<OPT, VEC>(tv, row, e, lane_on, a, r);
  finish_row<OPT, VEC>(tv, row, gsum, e, lane_on, gl, last_chunk, dim, a, r);
}

// keys[cnt] ascending (entries >= empty_from are holes). LEVEL0: the value of entry j is gradient
// row pos[j]; otherwise it is vals[j, :].
//
// A workgroup first stages the keys (and positions) of all its tiles in LDS with coalesced loads,
// including one neighbour on each side, so the walk itself only waits for value rows; those are
// requested four entries ahead of where the sums are. A lane group walks its tile and applies
// every run that lies wholly inside it. A run that touches a tile border leaves its partial sum
// in LDS instead: slot 2t for the run entering tile t from the left, 2t + 1 for the one leaving
// it to the right (a run that covers the whole tile fills both, the second with zeros). Equal
// keys are adjacent in that list, so after a barrier the lane group that owns the first partial
// of a run adds up the following ones (in order, from LDS) and applies the sum. Only the runs that
// cross the workgroup's own borders go on to the next level: carry slots 2w and 2w + 1 of
// workgroup w, which form a sorted sequence again. A level shrinks the sequence by the
// workgroup's span over two, so two or three launches serve any request.
//
// Running the last, short levels in one launch of a single workgroup (barrier between levels)
// was measured too: on one CU every level pays its dependent memory round trips one after the
// other, 36 us against four launches of about 8 us for the tail of an 8192-id request.
constexpr int kPrefetch = 4;
constexpr int kPrefetchCarry = 4;
constexpr int kCarryTile = 4;   // 16, 32 and 64 were measured: 254, 272 and 304 us for a million dim-128 ids against 244

// Weighted bags (level 0 only): the sorted payload is a position p, its gradient row is
// vals[bag_of[p]] times weight[p]. Both null otherwise: the payload itself names the row.
struct PooledSrc {
  const uint32_t* bag_of;
  const float* weight;
};

// Combined pushes (GROUPED): a key is (member number << row_bits) | row, and a closed run takes
// its member's record layout from descs. st0..st2 are the state types of the optimizer's three
// slots (-1 = unused); the column each lives in differs from member to member.
struct GroupSrc {
  const TableDesc* descs;
  int row_bits;
  int st0, st1, st2;
  int use_meta;
};

// LDS of one workgroup, in 32-bit words: partial sums [2 * per_block][group * VEC] first (vector
// accesses, 16-byte aligned), then partial keys [2 * per_block], the two carry keys, the staged
// keys [span + 2], payloads [span] and weights [span].
__host__ __device__ inline size_t segreduce_lds_words(int per_block, int group, int vec, int tile) {
  return (size_t)2 * per_block * group * vec + 2 * per_block + 2 + 3 * (size_t)per_block * tile + 2;
}

template <int OPT, int VEC, bool LEVEL0, bool GROUPED>
__global__ __launch_bounds__(kBlock) void segreduce_kernel(
    TableView tv, const uint32_t* __restrict__ keys, const uint32_t* __restrict__ pos,
    const float* __restrict__ vals, int64_t cnt, int tile, uint32_t empty_from,
    uint32_t* __restrict__ keys_out, float* __restrict__ vals_out, int dim, int elems, int group,
    ApplyArgs args, PooledSrc ps, GroupSrc gs) {
  extern __shared__ uint32_t lds[];
  const int per_block = kBlock / group;
  const int span = per_block * tile;                       // entries staged by this workgroup
  const int64_t first = (int64_t)blockIdx.x * span;        // global index of lds_keys[1]
  float* part_val = reinterpret_cast<float*>(lds);         // [2 * per_block][group * VEC]
  uint32_t* part_key = lds + 2 * per_block * group * VEC;  // [2 * per_block]
  uint32_t* out_key = part_key + 2 * per_block;            // [2]: what this workgroup carries on
  uint32_t* lds_keys = out_key + 2;                        // [span + 2], shifted by one
  uint32_t* lds_pos = lds_keys + span + 2;                 // [span]
  float* lds_w = reinterpret_cast<float*>(lds_pos + span); // [span], weighted bags only
  for (int i = threadIdx.x; i < span + 2; i += kBlock) {
    const int64_t j = first + i - 1;
    lds_keys[i] = (j >= 0 && j < cnt) ? keys[j] : kNoRow;
  }
  const bool weighted = LEVEL0 && ps.weight != nullptr;
  if (LEVEL0) {
    for (int i = threadIdx.x; i < span; i += kBlock) {
      const int64_t j = first + i;
      uint32_t p = j < cnt ? pos[j] : 0u;
      if (weighted) {
        // the payload is the position: it names the weight and, through bag_of, the row
        lds_w[i] = j < cnt ? ps.weight[p] : 0.0f;
        const uint32_t b = j < cnt ? ps.bag_of[p] : 0u;
        p = b == kNoBag ? 0u : b;
      }
      lds_pos[i] = p;
    }
  }
  if (threadIdx.x < 2) out_key[threadIdx.x] = kNoRow;
  __syncthreads();

  const int lt = threadIdx.x / group;                       // this lane group's tile in the workgroup
  const int gl = threadIdx.x & (group - 1);
  const int64_t a = ((int64_t)blockIdx.x * per_block + lt) * tile;
  const bool have = a < cnt;                                // the last workgroup may have idle groups
  const int64_t b = a + tile < cnt ? a + tile : cnt;
  const int la = (int)(a - first);                          // tile's first entry, LDS-relative
  const int lb = have ? (int)(b - first) : la;
  const uint32_t left_key = have ? lds_keys[la] : kNoRow;   // entry a - 1
  const uint32_t right_key = have ? lds_keys[lb + 1] : kNoRow;   // entry b
  const int64_t rem_tiles = (cnt - first + tile - 1) / tile;
  const int tiles_here = rem_tiles < per_block ? (int)rem_tiles : per_block;
  const bool leader = gl == 0;
  const int lane_floats = group * VEC;

  // whose record a key names: the table's, or in a combined push the member's
  auto resolve = [&](uint32_t key, TableView& member, ApplyArgs& aa) -> uint32_t {
    if constexpr (GROUPED) {
      const TableDesc& d = gs.descs[key >> gs.row_bits];
      member.recs = d.tv.recs;
      member.stride = d.tv.stride;
      aa.c0 = gs.st0 >= 0 ? d.col_off[gs.st0] : -1;
      aa.c1 = gs.st1 >= 0 ? d.col_off[gs.st1] : -1;
      aa.c2 = gs.st2 >= 0 ? d.col_off[gs.st2] : -1;
      aa.meta_off = gs.use_meta ? d.meta_off : -1;
      return key & ((1u << gs.row_bits) - 1u);
    } else {
      return key;
    }
  };

  // A finished sum goes to the optimizer (or is stored) once per run and chunk, in two steps: the
  // record is requested when the run closes, and updated when the lane group closes its next run
  // or has walked its tile. In between it goes on requesting and adding gradient rows, so the
  // record's round trip is not waited for on its own.
  RowRegs<VEC> pend_regs;
  float pend_sum[VEC];
  uint32_t pend_key = kNoRow;
  auto finish_pending = [&](int e, bool lane_on, bool last_chunk) {
    if (pend_key == kNoRow) return;
    TableView member = tv;
    ApplyArgs aa = args;
    const uint32_t row = resolve(pend_key, member, aa);
    finish_row<OPT, VEC>(member, row, pend_sum, e, lane_on, gl, last_chunk, dim, aa, pend_regs);
    pend_key = kNoRow;
  };
  auto apply = [&](uint32_t key, const float (&sum)[VEC], int e, bool lane_on, bool last_chunk) {
    finish_pending(e, lane_on, last_chunk);
    TableView member = tv;
    ApplyArgs aa = args;
    const uint32_t row = resolve(key, member, aa);
    load_row<OPT, VEC>(member, row, e, lane_on, aa, pend_regs);
    pend_key = key;
#pragma unroll
    for (int c = 0; c < VEC; ++c) pend_sum[c] = sum[c];
  };

  for (int e0 = 0; e0 < elems; e0 += group) {
    const int e = e0 + gl;
    const bool lane_on = e < elems;
    const bool last_chunk = e0 + group >= elems;
    uint32_t pk0 = kNoRow, pk1 = kNoRow;                    // keys of this tile's two partials
    if (have) {
      float acc[VEC];
#pragma unroll
      for (int c = 0; c < VEC; ++c) acc[c] = 0.0f;
      uint32_t run_key = lds_keys[la + 1];
      int run_start = la;

      // closes the run [run_start, end) of run_key
      auto close_run = [&](int end) {
        if (run_key >= empty_from) return;
        const bool open_left = run_start == la && left_key == run_key;
        const bool open_right = end == lb && right_key == run_key;
        if (!open_left && !open_right) {
          apply(run_key, acc, e, lane_on, last_chunk);
          return;
        }
        const int slot = open_left ? 2 * lt : 2 * lt + 1;
        vstore<VEC>(part_val + slot * lane_floats + gl * VEC, acc);
        if (open_left) pk0 = run_key; else pk1 = run_key;
        if (open_left && open_right) {
          // the run covers the whole tile: keep the list contiguous with a zero piece
          float z[VEC];
#pragma unroll
          for (int c = 0; c < VEC; ++c) z[c] = 0.0f;
          vstore<VEC>(part_val + (slot + 1) * lane_floats + gl * VEC, z);
          pk1 = run_key;
        }
      };

      constexpr int kAhead = LEVEL0 ? kPrefetch : kPrefetchCarry;
      for (int j0 = la; j0 < lb; j0 += kAhead) {
        float v[kAhead][VEC];
        uint32_t k[kAhead];
#pragma unroll
        for (int u = 0; u < kAhead; ++u) {
          const int j = j0 + u;
          k[u] = j < lb ? lds_keys[j + 1] : kNoRow;
          if (j < lb && k[u] < empty_from && lane_on) {
            const float* src = LEVEL0 ? vals + (int64_t)lds_pos[j] * dim : vals + (first + j) * dim;
            if constexpr (LEVEL0) vload_once<VEC>(src + e * VEC, v[u]); else vload<VEC>(src + e * VEC, v[u]);
            if (weighted) {
              const float w = lds_w[j];
#pragma unroll
              for (int c = 0; c < VEC; ++c) v[u][c] = v[u][c] * w;
            }
          } else {
#pragma unroll
            for (int c = 0; c < VEC; ++c) v[u][c] = 0.0f;
          }
        }
#pragma unroll
        for (int u = 0; u < kAhead; ++u) {
          const int j = j0 + u;
          if (j >= lb) break;
          if (k[u] != run_key) {
            close_run(j);
            run_key = k[u];
            run_start = j;
          }
          if (j == run_start) {
            // the first addend is copied, not added to zero (worker/emitter.cc:527 clones it)
#pragma unroll
            for (int c = 0; c < VEC; ++c) acc[c] = v[u][c];
          } else {
#pragma unroll
            for (int c = 0; c < VEC; ++c) acc[c] = acc[c] + v[u][c];
          }
        }
      }
      close_run(lb);
    }
    if (leader) {
      part_key[2 * lt] = pk0;
      part_key[2 * lt + 1] = pk1;
    }
    __syncthreads();

    // the partials of one run are adjacent: the group that owns the first adds the others to it
    if (have) {
      const int last = 2 * tiles_here - 1;
      for (int side = 0; side < 2; ++side) {
        const int en = 2 * lt + side;
        const uint32_t key = part_key[en];
        if (key == kNoRow || (en > 0 && part_key[en - 1] == key)) continue;
        float sum[VEC];
        vload<VEC>(part_val + en * lane_floats + gl * VEC, sum);
        int f = en;
        while (f < last && part_key[f + 1] == key) {
          ++f;
          float nx[VEC];
          vload<VEC>(part_val + f * lane_floats + gl * VEC, nx);
#pragma unroll
          for (int c = 0; c < VEC; ++c) sum[c] = sum[c] + nx[c];
        }
        // slot 0 exists only for a run that enters the workgroup from the left, the last slot
        // only for one that leaves it to the right
        const bool open_left = en == 0;
        const bool open_right = f == last;
        if (!open_left && !open_right) {
          apply(key, sum, e, lane_on, last_chunk);
          continue;
        }
        const int64_t slot = 2 * (int64_t)blockIdx.x + (open_left ? 0 : 1);
        if (lane_on) vstore<VEC>(vals_out + slot * dim + e * VEC, sum);
        if (leader) out_key[open_left ? 0 : 1] = key;
        if (open_left && open_right) {
          float z[VEC];
#pragma unroll
          for (int c = 0; c < VEC; ++c) z[c] = 0.0f;
          if (lane_on) vstore<VEC>(vals_out + (slot + 1) * dim + e * VEC, z);
          if (leader) out_key[1] = key;
        }
      }
    }
    finish_pending(e, lane_on, last_chunk);
    __syncthreads();                                        // the next chunk reuses the partials
  }
  if (threadIdx.x < 2 && keys_out) keys_out[2 * (int64_t)blockIdx.x + threadIdx.x] = out_key[threadIdx.x];
}

// Row width and lane mapping of a reduction: a table's, or those of a stand-alone call.
struct ReduceShape {
  int64_t dim;
  int vec, elems, group;
};

template <int OPT, int VEC>
static void launch_segreduce(bool level0, const TableView& tv, const uint32_t* keys, const uint32_t* pos,
                             const float* vals, int64_t cnt, int tile, uint32_t empty_from,
                             uint32_t* keys_out, float* vals_out, const ReduceShape* t,
                             const ApplyArgs& args, const PooledSrc& ps, const GroupSrc* gs,
                             hipStream_t stream) {
  const int per_block = kBlock / t->group;
  const int64_t tiles = (cnt + tile - 1) / tile;
  const dim3 grid(grid_for(tiles, per_block)), block(kBlock);
  const size_t lds_bytes = segreduce_lds_words(per_block, t->group, VEC, tile) * sizeof(uint32_t);
  const PooledSrc none{nullptr, nullptr};
  if constexpr (OPT != kOptStore) {
    if (gs) {
      if (level0) {
        hipLaunchKernelGGL((segreduce_kernel<OPT, VEC, true, true>), grid, block, lds_bytes, stream, tv, keys,
                           pos, vals, cnt, tile, empty_from, keys_out, vals_out, (int)t->dim, t->elems,
                           t->group, args, ps, *gs);
      } else {
        hipLaunchKernelGGL((segreduce_kernel<OPT, VEC, false, true>), grid, block, lds_bytes, stream, tv, keys,
                           pos, vals, cnt, tile, empty_from, keys_out, vals_out, (int)t->dim, t->elems,
                           t->group, args, none, *gs);
      }
      return;
    }
  }
  const GroupSrc plain{nullptr, 0, -1, -1, -1, 0};
  if (level0) {
    hipLaunchKernelGGL((segreduce_kernel<OPT, VEC, true, false>), grid, block, lds_bytes, stream, tv, keys, pos,
                       vals, cnt, tile, empty_from, keys_out, vals_out, (int)t->dim, t->elems, t->group,
                       args, ps, plain);
  } else {
    hipLaunchKernelGGL((segreduce_kernel<OPT, VEC, false, false>), grid, block, lds_bytes, stream, tv, keys, pos,
                       vals, cnt, tile, empty_from, keys_out, vals_out, (int)t->dim, t->elems, t->group,
                       args, none, plain);
  }
}

template <int VEC>
static void dispatch_segreduce(int opt, bool level0, const TableView& tv, const uint32_t* keys,
                               const uint32_t* pos, const float* vals, int64_t cnt, int tile,
                               uint32_t empty_from, uint32_t* keys_out, float* vals_out,
                               const ReduceShape* t, const ApplyArgs& args, const PooledSrc& ps,
                               const GroupSrc* gs, hipStream_t stream) {
  switch (opt) {
    case kOptStore:
      launch_segreduce<kOptStore, VEC>(level0, tv, keys, pos, vals, cnt, tile, empty_from, keys_out,
                                       vals_out, t, args, ps, gs, stream);
      break;
    case KRK_SGD:
      launch_segreduce<KRK_SGD, VEC>(level0, tv, keys, pos, vals, cnt, tile, empty_from, keys_out,
                                     vals_out, t, args, ps, gs, stream);
      break;
    case KRK_ADAGRAD:
      launch_segreduce<KRK_ADAGRAD, VEC>(level0, tv, keys, pos, vals, cnt, tile, empty_from, keys_out,
                                         vals_out, t, args, ps, gs, stream);
      break;
    case KRK_ADAM:
      launch_segreduce<KRK_ADAM, VEC>(level0, tv, keys, pos, vals, cnt, tile, empty_from, keys_out,
                                      vals_out, t, args, ps, gs, stream);
      break;
    default:
      launch_segreduce<KRK_RMSPROP, VEC>(level0, tv, keys, pos, vals, cnt, tile, empty_from, keys_out,
                                         vals_out, t, args, ps, gs, stream);
      break;
  }
}

static int pick_tile(int64_t cnt) {
  // The carry list has two entries per workgroup whatever the tile length, so tiles only trade
  // lane groups in flight against per-tile work: 8 entries up to half a million ids, 16 beyond
  // (measured 4 to 64). The carry lists themselves are short: tiles of 4 there.
  if (cnt >= (1 << 19)) return 16;
  return 8;
}

// ---------------------------------------------------------------------------
// Requests of at most 8192 ids per table: two launches, no carry levels, no global sort.
//   1. ids -> rows for every position, over the whole chip (rows_of_ids / group_rows_of_ids).
//   2. bucket_push_kernel, one workgroup of 1024 lanes for each of a table's 8 to 32 buckets
//      (bucket = row mod the number of buckets; as many as keep the request at about one
//      workgroup per compute unit), so that both one table and 26 tables use much of the chip:
//      a. the workgroup reads its table's row numbers and keeps the positions of its bucket, in
//         position order (one scan over the workgroup);
//      b. the (row, position) pairs are sorted by row in LDS with a stable radix sort, nine bits
//         a pass (two passes for tables of up to two million rows). Every wavefront ranks its own
//         elements with wave-wide votes (lanes holding the same digit find each other through
//         nine ballots), a per-wavefront histogram in LDS turns into offsets by one scan over
//         (digit, wavefront), and the pairs are scattered through LDS;
//      c. every run of equal rows is summed in position order (worker/emitter.cc:527-529) and
//         applied once. Who adds a run up depends on its length: a lane group (up to 16
//         positions, two runs in flight per group), a wavefront (up to 16 positions per lane
//         group of it: the groups add a stretch each and the stretches' sums are added in order
//         inside the wavefront), or the whole workgroup the same way (the very head of a skewed
//         distribution). The three lists are made in one pass over the run lengths.
//      Nothing but the row numbers passes through global memory between the stages.
// Measured on the way here, 8192 Zipf ids, dim 16: the whole push in one workgroup per table
// 88 us (one compute unit keeps too few random reads in flight for index, gradients and
// records); sorting a table's 8192 pairs in one workgroup 20-30 us whoever wrote the sort (a
// pass is a chain of LDS round trips and barriers, and a wavefront instruction holds its SIMD
// for four cycles), 19 us even for a bucket's 1024 pairs when the pairs arrive unordered and
// position has to be sorted as well (five passes); the whole request in one launch (buckets by a
// hash of the id, the look-up inside the bucket's workgroup, gradient rows staged through LDS a
// chunk at a time) 38 us, 57 us for 26 tables: the workgroup that draws the hottest id holds five
// times the entries of the others, and the sixteen wavefronts of a workgroup share four SIMDs,
// so every instruction of a wavefront costs sixteen cycles there. Smaller workgroups over more
// buckets for a single table (256 lanes x 128 buckets, 512 x 64) take 28 and 25 us against 26:
// the bucket that holds the hottest id has fewer lane groups to share its run out to.
// ---------------------------------------------------------------------------
constexpr int kSortBlock = 1024;
constexpr int kSortItems = 8;
constexpr int kSortMax = kSortBlock * kSortItems;      // ids per table
static_assert(kSortMax <= kNotedMax, "row notes are kept for the requests that take this path");
constexpr int kSortWaves = kSortBlock / kWave;
constexpr int kMaxBucketBits = 5;                      // up to 32 buckets a table
constexpr int kDigitBits = 9;
constexpr int kDigits = 1 << kDigitBits;
constexpr int kRunAhead = 8;                           // gradient rows requested ahead of the sums
constexpr int kShortRun = 16;                          // runs up to this length: one lane group each
constexpr int kWaveRunPerGroup = 16;                   // a wavefront takes runs of up to this many entries per lane group;
                                                       // longer runs are shared out over the whole workgroup
constexpr int kRunListMax = kSortMax / (kShortRun + 1) + 1;   // runs above kShortRun a bucket can hold
constexpr int kPartOffset = (kSortMax + 1 + 2 * kRunListMax + 3) & ~3;   // the partial sums start on 16 bytes
constexpr int kShortMaxDim = 64;
static_assert(kSortWaves * kDigits <= kSortMax + 1, "the histogram fits the work space");

struct SortCall {
  int32_t n_tables;
  int32_t bucket_bits;                                 // a table's rows are dealt to 2^bucket_bits workgroups
  int32_t row_bits;                                    // bits of a row number
  uint32_t row_mask;                                   // a key's row (member bits above it)
  uint32_t miss_key;                                   // keys at or above it stand for missing ids
  // Not null: `keys` are the row notes of the pull of these ids (a member's own row numbers).
  // A note of kEmptyRow was taken while the row's creator, another wavefront of that pull, had
  // not published the row number yet (further occurrences of an id that the pull inserted):
  // such a position is looked up here.
  const uint64_t* note_ids;
  int64_t row_start[kMaxGroupTables + 1];
};

// lanes of this wavefront (bit mask) whose `digit` equals this lane's
__device__ __forceinline__ unsigned long long match_digit(uint32_t digit) {
  unsigned long long same = ~0ull;
#pragma unroll
  for (int b = 0; b < kDigitBits; ++b) {
    const bool bit = (digit >> b) & 1u;
    const unsigned long long votes = __ballot(bit);
    same &= bit ? votes : ~votes;
  }
  return same;
}

// A barrier for phases that exchange data through LDS only: waits for the wavefront's LDS
// operations, not for its global loads and stores as __syncthreads() does. (Requesting the
// records' lines ahead of the sort, behind such barriers, was measured too: no gain.)
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// exclusive prefix sum of one value per lane over the workgroup (1024 lanes); total to all
__device__ __forceinline__ uint32_t sort_block_scan(uint32_t v, uint32_t* wave_total, uint32_t& total) {
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  uint32_t incl = v;
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const uint32_t y = __shfl_up(incl, d);
    if (lane >= d) incl += y;
  }
  lds_barrier();                                     // wave_total may still be read from a previous scan
  if (lane == kWave - 1) wave_total[wave] = incl;
  lds_barrier();
  uint32_t offset = incl - v;
  uint32_t sum = 0;
  for (int w = 0; w < kSortWaves; ++w) {
    const uint32_t x = wave_total[w];
    if (w < wave) offset += x;
    sum += x;
  }
  total = sum;
  return offset;
}

// grid: one workgroup per bucket (n_tables << bucket_bits)
template <int OPT, int VEC, bool GROUPED>
__global__ __launch_bounds__(kSortBlock) void bucket_push_kernel(const TableDesc* __restrict__ descs, TableView tv,
                                                                 SortCall call, const uint32_t* __restrict__ keys,
                                                                 const float* __restrict__ grads, int dim,
                                                                 int elems, int group, ApplyArgs args, GroupSrc gs) {
  __shared__ uint32_t skey[kSortMax];                  // row >> bucket_bits
  __shared__ uint16_t spos[kSortMax];
  // histogram [wave][digit] while sorting; partial sums and their keys while reducing
  // histogram [wave][digit] while sorting; then run starts, the list of long runs, and the
  // wavefronts' partial sums of a long run
  __shared__ __align__(16) uint32_t work[kPartOffset + kSortWaves * kWave * 4];
  __shared__ uint32_t wave_total[kSortWaves];
  const int mb = blockIdx.x;
  const int bucket_bits = call.bucket_bits;
  const uint32_t n_buckets = 1u << bucket_bits;
  const int m = mb >> bucket_bits;
  const uint32_t bucket = (uint32_t)mb & (n_buckets - 1);
  const int t = threadIdx.x;
  const int64_t a = call.row_start[m];
  const int all = (int)(call.row_start[m + 1] - a);    // positions of the table's request
  if (all <= 0) return;                                // uniform for the workgroup
  if constexpr (GROUPED) {
    const TableDesc& d = descs[m];
    tv = d.tv;
    args.c0 = gs.st0 >= 0 ? d.col_off[gs.st0] : -1;
    args.c1 = gs.st1 >= 0 ? d.col_off[gs.st1] : -1;
    args.c2 = gs.st2 >= 0 ? d.col_off[gs.st2] : -1;
    args.meta_off = gs.use_meta ? d.meta_off : -1;
  }
  const int lane = t & (kWave - 1);
  const int wave = t / kWave;

  // ---- a. the bucket's positions, in position order -------------------------------------------
  // a lane looks at four or eight consecutive positions, read straight from global memory with
  // 16-byte loads where the member's keys begin on 16 bytes (as eight 4-byte loads, each of
  // them fetched a 32-byte piece of a line for four bytes: 3-4 us of the kernel's 20)
  const int own = all > 4 * kSortBlock ? kSortItems : 4;
  uint32_t mine[kSortItems];
  if ((reinterpret_cast<uintptr_t>(keys + a) & 15) == 0 && (t + 1) * own <= all) {
    const uint4 x = *reinterpret_cast<const uint4*>(keys + a + t * own);
    mine[0] = x.x; mine[1] = x.y; mine[2] = x.z; mine[3] = x.w;
    if (own == kSortItems) {
      const uint4 y = *reinterpret_cast<const uint4*>(keys + a + t * own + 4);
      mine[4] = y.x; mine[5] = y.y; mine[6] = y.z; mine[7] = y.w;
    }
  } else {
#pragma unroll
    for (int i = 0; i < kSortItems; ++i) {
      const int j = t * own + i;
      if (i < own) mine[i] = keys[a + (j < all ? j : all - 1)];
    }
  }
  if (call.note_ids) {
#pragma unroll
    for (int i = 0; i < kSortItems; ++i) {
      const int j = t * own + i;
      if (i < own && j < all && mine[i] == kEmptyRow) mine[i] = probe_find_alone(tv, call.note_ids[a + j]);
    }
  }
  uint32_t take = 0;
#pragma unroll
  for (int i = 0; i < kSortItems; ++i) {
    const int j = t * own + i;
    if (i < own && j < all && mine[i] < call.miss_key && ((mine[i] & call.row_mask) & (n_buckets - 1)) == bucket)
      take |= 1u << i;
  }
  uint32_t total;
  uint32_t at = sort_block_scan((uint32_t)__popc(take), wave_total, total);
#pragma unroll
  for (int i = 0; i < kSortItems; ++i) {
    if (take & (1u << i)) {
      skey[at] = (mine[i] & call.row_mask) >> bucket_bits;
      spos[at] = (uint16_t)(t * own + i);
      ++at;
    }
  }
  const int len = (int)total;
  if (len == 0) return;                                // uniform
  const int per_lane = (len + kSortBlock - 1) / kSortBlock;   // 1..8
  const int padded = per_lane * kSortBlock;
  for (int j = len + t; j < padded; j += kSortBlock) {   // beyond what the lanes above wrote

    skey[j] = 0xFFFFFFFFu;                             // padding sorts behind everything
    spos[j] = 0;
  }
  lds_barrier();

  // ---- b. stable radix sort by row -----------------------------------------------------------
  // element i of lane l in wavefront w is pair w * 64 * per_lane + i * 64 + l: a wavefront's
  // elements are consecutive, and taking i in ascending order visits them in list order
  {
    uint32_t* hist = work;                             // [kSortWaves][kDigits]
    const int wbase = wave * kWave * per_lane + lane;
    const int bits = call.row_bits > bucket_bits ? call.row_bits - bucket_bits : 1;
    const int passes = (bits + kDigitBits - 1) / kDigitBits;
    const int width = (bits + passes - 1) / passes;    // bits per pass, at most kDigitBits
    const uint32_t digit_mask = (1u << width) - 1u;
    for (int pass = 0; pass < passes; ++pass) {
      const int shift = pass * width;
      uint32_t key[kSortItems], rank[kSortItems];
      uint16_t pos[kSortItems];
#pragma unroll
      for (int i = 0; i < kSortItems; ++i) {
        if (i < per_lane) {
          key[i] = skey[wbase + i * kWave];
          pos[i] = spos[wbase + i * kWave];
        }
      }
      for (int i = t; i < kSortWaves * kDigits; i += kSortBlock) hist[i] = 0u;
      lds_barrier();                                 // everyone holds its pairs; the histogram is clear
#pragma unroll
      for (int i = 0; i < kSortItems; ++i) {
        if (i < per_lane) {                            // uniform
          // the last pass also sees the padding's upper bits: they stay the largest digit
          const uint32_t digit = (key[i] >> shift) & digit_mask;
          const unsigned long long same = match_digit(digit);
          const uint32_t before = (uint32_t)__popcll(same & ((1ull << lane) - 1ull));
          uint32_t* cell = &hist[wave * kDigits + digit];
          const uint32_t old = *cell;                  // read by all lanes of the digit ...
          if (before == 0) *cell = old + (uint32_t)__popcll(same);   // ... then advanced by their first
          rank[i] = old + before;
        }
      }
      lds_barrier();
      // exclusive scan over (digit, wavefront): lane t owns digit t / 2, wavefronts 8 (t % 2) .. + 7
      {
        const int digit = t >> 1;
        const int w0 = (t & 1) * 8;
        uint32_t c[8], sum = 0, whole;
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          c[k] = hist[(w0 + k) * kDigits + digit];
          sum += c[k];
        }
        uint32_t offset = sort_block_scan(sum, wave_total, whole);
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          hist[(w0 + k) * kDigits + digit] = offset;
          offset += c[k];
        }
      }
      lds_barrier();
#pragma unroll
      for (int i = 0; i < kSortItems; ++i) {
        if (i < per_lane) {
          const uint32_t dest = hist[wave * kDigits + ((key[i] >> shift) & digit_mask)] + rank[i];
          skey[dest] = key[i];
          spos[dest] = pos[i];
        }
      }
      lds_barrier();
    }
  }

  // ---- c. runs of equal rows: sums in position order, one update per row -----------------------
  uint32_t* run_start = work;                          // [runs + 1]; the histogram is done with
  uint32_t* long_run = work + kSortMax + 1;            // [kRunListMax] runs for the whole workgroup
  uint32_t* wave_run = long_run + kRunListMax;         // [kRunListMax] runs for one wavefront each
  __shared__ uint32_t n_long, n_wave;
  uint32_t runs;
  {
    // lane t looks at entries [t * per_lane, (t + 1) * per_lane): where does a new row begin?
    const int j0 = t * per_lane;
    uint32_t heads = 0;
#pragma unroll
    for (int i = 0; i < kSortItems; ++i) {
      const int j = j0 + i;
      if (i < per_lane && j < len && (j == 0 || skey[j - 1] != skey[j])) heads |= 1u << i;
    }
    if (t == 0) n_long = n_wave = 0u;
    uint32_t r = sort_block_scan((uint32_t)__popc(heads), wave_total, runs);
#pragma unroll
    for (int i = 0; i < kSortItems; ++i)
      if (heads & (1u << i)) run_start[r++] = (uint32_t)(j0 + i);
    if (t == 0) run_start[runs] = (uint32_t)len;
    lds_barrier();
  }
  const int per_block = kSortBlock / group;
  const int lt = t / group;
  const int gl = t & (group - 1);
  const bool lane_on = gl < elems;
  const float* g_base = grads + a * (int64_t)dim;
  // Who adds a run up: a lane group (up to kShortRun entries, the reference's order exactly), a
  // wavefront (its lane groups take a stretch each and the stretches' sums are added in order),
  // or the whole workgroup. A lane group walking 64 entries on its own took eight trips to memory
  // while the others waited at the barrier: 10 of the kernel's 30 us for 26 tables of 8192 ids.
  const int groups_per_wave = kWave / group;
  const int wave_run_max = kWaveRunPerGroup * groups_per_wave;
  for (uint32_t q = (uint32_t)t; q < runs; q += kSortBlock) {
    const int count = (int)(run_start[q + 1] - run_start[q]);
    if (count > wave_run_max) {
      long_run[atomicAdd(&n_long, 1u)] = q;
    } else if (count > kShortRun) {
      wave_run[atomicAdd(&n_wave, 1u)] = q;
    }
  }
  lds_barrier();

  // adds entries [lo, hi) of the sorted list in list order; the first addend is copied, not added
  // to zero (worker/emitter.cc:527 clones it)
  auto sum_entries = [&](int lo, int hi, float (&acc)[VEC]) {
#pragma unroll
    for (int c = 0; c < VEC; ++c) acc[c] = 0.0f;
    for (int j0 = lo; j0 < hi; j0 += kRunAhead) {
      float v[kRunAhead][VEC];
#pragma unroll
      for (int u = 0; u < kRunAhead; ++u) {
        if (j0 + u < hi && lane_on) {
          gload<VEC>(g_base + (int64_t)spos[j0 + u] * dim + gl * VEC, v[u]);
        } else {
#pragma unroll
          for (int c = 0; c < VEC; ++c) v[u][c] = 0.0f;
        }
      }
#pragma unroll
      for (int u = 0; u < kRunAhead; ++u) {
        if (j0 + u >= hi) break;
        if (j0 + u == lo) {
#pragma unroll
          for (int c = 0; c < VEC; ++c) acc[c] = v[u][c];
        } else {
#pragma unroll
          for (int c = 0; c < VEC; ++c) acc[c] = acc[c] + v[u][c];
        }
      }
    }
  };

  // Runs of at most kShortRun entries: one lane group each, exactly the reference's order. A lane
  // group takes two runs at a time: both records and the first kPairAhead gradient rows of both
  // are requested before anything is added, so a round costs one trip to memory for two rows (a
  // bucket's workgroup has 256 lane groups for some 500 runs, and the trips were most of the
  // phase: 13 of 39 us for 26 tables of 8192 ids).
  constexpr int kPairAhead = 2;
  auto request_head = [&](int lo, int hi, float (&v)[kPairAhead][VEC]) {
#pragma unroll
    for (int u = 0; u < kPairAhead; ++u) {
      if (lo + u < hi && lane_on) {
        gload<VEC>(g_base + (int64_t)spos[lo + u] * dim + gl * VEC, v[u]);
      } else {
#pragma unroll
        for (int c = 0; c < VEC; ++c) v[u][c] = 0.0f;
      }
    }
  };
  // the head's rows first (already requested), then the rest of the run in chunks
  auto sum_from_head = [&](int lo, int hi, const float (&v)[kPairAhead][VEC], float (&acc)[VEC]) {
#pragma unroll
    for (int c = 0; c < VEC; ++c) acc[c] = v[0][c];      // the first addend is copied (emitter.cc:527)
#pragma unroll
    for (int u = 1; u < kPairAhead; ++u) {
      if (lo + u < hi) {
#pragma unroll
        for (int c = 0; c < VEC; ++c) acc[c] = acc[c] + v[u][c];
      }
    }
    for (int j0 = lo + kPairAhead; j0 < hi; j0 += kRunAhead) {
      float w[kRunAhead][VEC];
#pragma unroll
      for (int u = 0; u < kRunAhead; ++u) {
        if (j0 + u < hi && lane_on) {
          gload<VEC>(g_base + (int64_t)spos[j0 + u] * dim + gl * VEC, w[u]);
        } else {
#pragma unroll
          for (int c = 0; c < VEC; ++c) w[u][c] = 0.0f;
        }
      }
#pragma unroll
      for (int u = 0; u < kRunAhead; ++u) {
        if (j0 + u >= hi) break;
#pragma unroll
        for (int c = 0; c < VEC; ++c) acc[c] = acc[c] + w[u][c];
      }
    }
  };
  // runs for one wavefront each: lane group i of the wavefront adds the i-th stretch, then the
  // stretches' sums are added in order inside the wavefront (neighbours first, by doubling)
  {
    const int sub = lane / group;
    const uint32_t waves_runs = n_wave;
    for (uint32_t k = (uint32_t)wave; k < waves_runs; k += kSortWaves) {
      const uint32_t q = wave_run[k];                  // in any order: the runs are different rows
      const int first = (int)run_start[q], count = (int)run_start[q + 1] - first;
      const int stretch = (count + groups_per_wave - 1) / groups_per_wave;
      const int lo = first + sub * stretch < first + count ? first + sub * stretch : first + count;
      const int hi = lo + stretch < first + count ? lo + stretch : first + count;
      const uint32_t row = (skey[first] << bucket_bits) | bucket;
      RowRegs<VEC> rec;
      if (sub == 0) load_row<OPT, VEC>(tv, row, gl, lane_on, args, rec);
      float acc[VEC];
      sum_entries(lo, hi, acc);
      for (int d = group; d < kWave; d <<= 1) {
#pragma unroll
        for (int c = 0; c < VEC; ++c) {
          const float other = __shfl_down(acc[c], d);
          if ((sub & ((2 * d / group) - 1)) == 0) acc[c] = acc[c] + other;
        }
      }
      if (sub == 0) finish_row<OPT, VEC>(tv, row, acc, gl, lane_on, gl, true, dim, args, rec);
    }
  }
  for (uint32_t q0 = (uint32_t)lt; q0 < runs; q0 += 2u * (uint32_t)per_block) {
    int start[2], end[2];
    bool on[2];
    uint32_t row[2];
    RowRegs<VEC> rec[2];
    float head[2][kPairAhead][VEC];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const uint32_t q = q0 + (uint32_t)h * (uint32_t)per_block;
      on[h] = q < runs;
      start[h] = on[h] ? (int)run_start[q] : 0;
      end[h] = on[h] ? (int)run_start[q + 1] : 0;
      if (on[h] && end[h] - start[h] > kShortRun) on[h] = false;   // a wavefront's or the workgroup's
      row[h] = on[h] ? ((skey[start[h]] << bucket_bits) | bucket) : 0u;
      if (on[h]) {
        load_row<OPT, VEC>(tv, row[h], gl, lane_on, args, rec[h]);
        request_head(start[h], end[h], head[h]);
      }
    }
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      if (!on[h]) continue;
      float acc[VEC];
      sum_from_head(start[h], end[h], head[h], acc);
      finish_row<OPT, VEC>(tv, row[h], acc, gl, lane_on, gl, true, dim, args, rec[h]);
    }
  }
  __syncthreads();
  // hot ids: every lane group adds a stretch of the run; the stretches' sums are added in order,
  // first inside each wavefront (neighbouring lane groups, by doubling), then across wavefronts
  float* part = reinterpret_cast<float*>(work + kPartOffset);   // [2][kSortWaves][group * VEC]
  const uint32_t longs = n_long;
  const int lane_floats = group * VEC;
  for (uint32_t k = 0; k < longs; ++k) {
    const uint32_t q = long_run[k];                    // in any order: the runs are different rows
    const int start = (int)run_start[q], count = (int)run_start[q + 1] - start;
    const int stretch = (count + per_block - 1) / per_block;
    const int lo = start + lt * stretch < start + count ? start + lt * stretch : start + count;
    const int hi = lo + stretch < start + count ? lo + stretch : start + count;
    const uint32_t row = (skey[start] << bucket_bits) | bucket;
    RowRegs<VEC> rec;
    if (lt == 0) load_row<OPT, VEC>(tv, row, gl, lane_on, args, rec);   // on its way while the stretches are added
    float acc[VEC];
    sum_entries(lo, hi, acc);
    // inside the wavefront: lane group i takes in group i + 1, then i + 2, i + 4, ...
    for (int d = group; d < kWave; d <<= 1) {
#pragma unroll
      for (int c = 0; c < VEC; ++c) {
        const float other = __shfl_down(acc[c], d);
        if (((lane / group) & ((2 * d / group) - 1)) == 0) acc[c] = acc[c] + other;
      }
    }
    // two sets of partial sums in turn: one barrier a run, the next run's stretches are requested
    // while the first lane group still updates this run's row
    float* mine = part + (k & 1u) * kSortWaves * lane_floats;
    if (lane < group) vstore<VEC>(mine + wave * lane_floats + gl * VEC, acc);
    __syncthreads();
    if (lt == 0) {
      float w[kSortWaves][VEC];
#pragma unroll
      for (int f = 1; f < kSortWaves; ++f) vload<VEC>(mine + f * lane_floats + gl * VEC, w[f]);
#pragma unroll
      for (int f = 1; f < kSortWaves; ++f) {
#pragma unroll
        for (int c = 0; c < VEC; ++c) acc[c] = acc[c] + w[f][c];
      }
      finish_row<OPT, VEC>(tv, row, acc, gl, lane_on, gl, true, dim, args, rec);
    }
  }
}

template <int VEC, bool GROUPED>
static void launch_bucket_push(int opt, unsigned buckets, hipStream_t stream, const TableDesc* descs,
                               const TableView& tv, const SortCall& call, const uint32_t* keys, const float* grads,
                               int dim, int elems, int group, const ApplyArgs& args, const GroupSrc& gs) {
  const dim3 grid(buckets), block(kSortBlock);
  switch (opt) {
    case KRK_SGD:
      hipLaunchKernelGGL((bucket_push_kernel<KRK_SGD, VEC, GROUPED>), grid, block, 0, stream, descs, tv, call, keys,
                         grads, dim, elems, group, args, gs);
      break;
    case KRK_ADAGRAD:
      hipLaunchKernelGGL((bucket_push_kernel<KRK_ADAGRAD, VEC, GROUPED>), grid, block, 0, stream, descs, tv, call,
                         keys, grads, dim, elems, group, args, gs);
      break;
    case KRK_ADAM:
      hipLaunchKernelGGL((bucket_push_kernel<KRK_ADAM, VEC, GROUPED>), grid, block, 0, stream, descs, tv, call, keys,
                         grads, dim, elems, group, args, gs);
      break;
    default:
      hipLaunchKernelGGL((bucket_push_kernel<KRK_RMSPROP, VEC, GROUPED>), grid, block, 0, stream, descs, tv, call,
                         keys, grads, dim, elems, group, args, gs);
      break;
  }
}

// Workgroups per table: as many as keep the request within about one workgroup per compute unit
// (a workgroup's LDS leaves room for one per unit), between 8 and 32.
static int short_bucket_bits(int n_tables) {
  int bits = kMaxBucketBits;
  while (bits > 3 && (n_tables << bits) > 256) --bits;
  return bits;
}

// Whether a request whose longest table brings `longest` ids takes the two-launch path: a lane
// group must own a whole row, and a bucket's gradients pass through one compute unit.
static bool short_push_fits(int64_t longest, int64_t dim, int elems, int group) {
  return longest <= kSortMax && dim <= kShortMaxDim && elems <= group;
}

// Stable sort of (key, payload) by key, then the tiled segmented reduction: every run of equal
// keys is summed in payload order and handed to apply_row<opt> once. `fill(keys, payload)`
// enqueues the kernel that writes the n unsorted pairs; keys >= miss_key are skipped. d_vals
// holds one value row per payload. scratch[0..4] is the caller's work space.
template <typename Fill>
static int32_t sort_and_reduce(const ReduceShape& sh, hipStream_t stream, DeviceBuffer* scratch,
                               const TableView& tv, int opt, int64_t n, uint32_t miss_key, int bits,
                               const float* d_vals, const ApplyArgs& args, const PooledSrc& ps,
                               const GroupSrc* gs, Fill fill) {
  const int tile0 = pick_tile(n);
  const int per_block = kBlock / sh.group;
  const int64_t groups0 = ((n + tile0 - 1) / tile0 + per_block - 1) / per_block;   // workgroups of level 0
  const size_t n4 = (size_t)n * sizeof(uint32_t);
  const size_t sort_bytes = radix_sort_work_bytes(n);
  const size_t carry_entries = (size_t)(2 * groups0);
  KRK_TRY(scratch[0].reserve(4 * n4));                       // keys, payload, sorted keys, sorted payload
  KRK_TRY(scratch[1].reserve(sort_bytes));
  KRK_TRY(scratch[2].reserve(carry_entries * sizeof(uint32_t) * 2));              // carry keys A|B
  KRK_TRY(scratch[3].reserve(carry_entries * (size_t)sh.dim * sizeof(float)));    // carry vals A
  KRK_TRY(scratch[4].reserve((carry_entries / 2 + 16) * (size_t)sh.dim * sizeof(float)));  // B
  uint32_t* keys = scratch[0].as<uint32_t>();
  uint32_t* pos = keys + n;
  uint32_t* skeys = nullptr;
  uint32_t* spos = nullptr;

  fill(keys, pos);
  KRK_HIP(hipGetLastError());
  KRK_TRY(radix_sort_pairs(keys, pos, pos + n, pos + 2 * n, n, bits, scratch[1].ptr, stream, &skeys, &spos));

  // level 0 reads value rows through the sorted payloads; later levels read the carry list
  uint32_t* ckeys[2] = {scratch[2].as<uint32_t>(), scratch[2].as<uint32_t>() + carry_entries};
  float* cvals[2] = {scratch[3].as<float>(), scratch[4].as<float>()};
  const uint32_t* in_keys = skeys;
  const float* in_vals = d_vals;
  int64_t cnt = n;
  int tile = tile0;
  bool level0 = true;
  int which = 0;
  for (;;) {
    const int64_t groups = ((cnt + tile - 1) / tile + per_block - 1) / per_block;
    uint32_t* okeys = nullptr;
    float* ovals = nullptr;
    if (groups > 1) {
      okeys = ckeys[which];
      ovals = cvals[which];
    }
    if (sh.vec == 4) {
      dispatch_segreduce<4>(opt, level0, tv, in_keys, spos, in_vals, cnt, tile, miss_key, okeys, ovals, &sh,
                            args, ps, gs, stream);
    } else {
      dispatch_segreduce<1>(opt, level0, tv, in_keys, spos, in_vals, cnt, tile, miss_key, okeys, ovals, &sh,
                            args, ps, gs, stream);
    }
    KRK_HIP(hipGetLastError());
    if (groups <= 1) break;
    in_keys = okeys;
    in_vals = ovals;
    cnt = 2 * groups;
    level0 = false;
    which ^= 1;
    tile = kCarryTile;
  }
  return KRK_SUCCESS;
}

// Positions -> rows -> sort_and_reduce fused with the optimizer. d_g holds one gradient row per
// sort payload (per position, or per bag for pooled pushes). The caller holds the table's lock
// and has made the optimizer's columns exist.
static int32_t push_sorted(krk_sparse* t, const krk_optim* o, const uint64_t* d_ids, int64_t n,
                           const float* d_g, float lr, const uint32_t* bag_of, bool payload_is_bag,
                           const PooledSrc& ps) {
  // sort key width: rows are < row_cap; one value above them marks a missing id
  uint32_t miss_key = 1;
  int bits = 1;
  while ((int64_t)miss_key < t->row_cap) {
    miss_key <<= 1;
    ++bits;
  }
  ApplyArgs args;
  args.lr = lr;
  args.k = make_optim_k(*o);
  int32_t cols[3];
  sparse_optim_columns(t, *o, cols);
  args.c0 = cols[0];
  args.c1 = cols[1];
  args.c2 = cols[2];
  args.meta_off = ((optim_state_mask(*o) >> KRK_ST_STEPS) & 1u) ? t->meta_off : -1;
  const TableView tv = t->view();
  const ReduceShape sh{t->dim, t->vec, t->elems, t->group};
  return sort_and_reduce(sh, t->stream, t->scratch, tv, o->type, n, miss_key, bits, d_g, args, ps, nullptr,
                         [&](uint32_t* keys, uint32_t* pos) {
                           hipLaunchKernelGGL(rows_of_ids_kernel, dim3(grid_for(n, kBlock / kBucket)),
                                              dim3(kBlock), 0, t->stream, tv, d_ids, n, miss_key, bag_of,
                                              payload_is_bag, keys, pos);
                         });
}

// stand-alone dedup + sum: (unique index, position) pairs for the sort
__global__ __launch_bounds__(kBlock) void dedup_pairs_kernel(const DSlot* __restrict__ slots,
                                                             const uint32_t* __restrict__ slot_of, int64_t n,
                                                             uint32_t* __restrict__ keys,
                                                             uint32_t* __restrict__ pos) {
  const int64_t p = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (p >= n) return;
  keys[p] = slots[slot_of[p]].uidx;
  pos[p] = (uint32_t)p;
}

// worker/emitter.cc:162-182 : rows of the unique ids back to one row per position
template <int VEC>
__global__ __launch_bounds__(kBlock) void expand_rows_kernel(const float* __restrict__ rows,
                                                             const long long* __restrict__ inv, int64_t n,
                                                             int64_t n_rows, float* __restrict__ out, int dim,
                                                             int elems, uint32_t* __restrict__ err) {
  const int64_t total = n * elems;
  const int64_t step = (int64_t)gridDim.x * kBlock;
  for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < total; i += step) {
    const int64_t p = i / elems;
    const int e = (int)(i - p * elems);
    const long long u = inv[p];
    float v[VEC];
#pragma unroll
    for (int c = 0; c < VEC; ++c) v[c] = 0.0f;
    if (u >= 0 && u < n_rows) {
      vload<VEC>(rows + u * dim + e * VEC, v);
    } else if (e == 0) {
      atomicOr(err, 1u);
    }
    vstore<VEC>(out + p * dim + e * VEC, v);
  }
}

}  // namespace krk

using namespace krk;

extern "C" {

// The stand-alone dedup calls block and own no table: their work space is kept between calls
// under one lock, and they run on the null stream.
static std::mutex g_dedup_mu;
static DeviceBuffer g_dedup_pool;
static DeviceBuffer g_dedup_reduce[5];

struct DedupWork {
  DSlot* slots;
  uint64_t cap;
  uint32_t* slot_of;
  int32_t* flag;
  int32_t* rank;
  void* scan_tmp;
  int32_t* d_total;
  char* extra;   // `extra_bytes` more for the caller (staged host arguments)
};

static size_t round256(size_t b) { return (b + 255) & ~(size_t)255; }

static int32_t dedup_layout(int64_t n, size_t extra_bytes, DedupWork* w) {
  uint64_t cap = 1024;
  while (cap < (uint64_t)n * 2) cap <<= 1;
  const size_t slots_b = (cap + 1) * sizeof(DSlot);
  const size_t n4 = round256((size_t)n * 4);
  const size_t scan_b = round256(scan_scratch_bytes(n));
  KRK_TRY(g_dedup_pool.reserve(slots_b + 3 * n4 + scan_b + 256 + extra_bytes));
  char* cur = g_dedup_pool.as<char>();
  w->slots = reinterpret_cast<DSlot*>(cur); cur += slots_b;
  w->cap = cap;
  w->slot_of = reinterpret_cast<uint32_t*>(cur); cur += n4;
  w->flag = reinterpret_cast<int32_t*>(cur); cur += n4;
  w->rank = reinterpret_cast<int32_t*>(cur); cur += n4;
  w->scan_tmp = cur; cur += scan_b;
  w->d_total = reinterpret_cast<int32_t*>(cur); cur += 256;
  w->extra = cur;
  return KRK_SUCCESS;
}

// unique ids in first-occurrence order into d_uids, every position's slot into w.slot_of (the
// slot then holds the id's index in the unique list), every position's index in the unique list
// into d_inv (when not null); *u = number of unique ids. The count is read back last, so the
// call waits for the device once.
// The launches alone, nothing read back. The index is cleared by a fill kernel rather than a
// memset node so that a caller may record these launches into a graph.
// The claims of a request. Its first workgroups (32, or 8 for a request of under 128) go ahead of
// the others in a launch of their own: the ids that fill much of a skewed request are all among
// the first few thousand positions, so every later workgroup finds their slots claimed and
// holding a smaller position, with plain loads. Launched all at once, the few hundred workgroups
// that start together each see such a slot empty and each send it a compare-and-swap and a
// minimum, and the memory serves the atomics of one address one after the other (a million ids
// of a Zipf 1.3 draw: 98 us a blocking call that way, 74 us this way).
constexpr unsigned kDedupHead = 32, kDedupHeadSmall = 8;

static void launch_dedup_claims(const DedupWork& w, const uint64_t* d_ids, int64_t n, hipStream_t s) {
  const unsigned blocks = grid_for(n, kDedupBlock);
  unsigned head = 0;
  if (blocks >= 4 * kDedupHeadSmall) {
    head = blocks >= 4 * kDedupHead ? kDedupHead : kDedupHeadSmall;
    hipLaunchKernelGGL(dedup_claim_kernel, dim3(head), dim3(kDedupBlock), 0, s, w.slots, w.cap - 1, d_ids, n,
                       w.slot_of, 0u);
  }
  hipLaunchKernelGGL(dedup_claim_kernel, dim3(blocks - head), dim3(kDedupBlock), 0, s, w.slots, w.cap - 1, d_ids,
                     n, w.slot_of, head);
}

static int32_t dedup_enqueue(const DedupWork& w, const uint64_t* d_ids, int64_t n, uint64_t* d_uids,
                             long long* d_inv, hipStream_t s) {
  const int64_t words = (int64_t)(w.cap + 1) * (int64_t)(sizeof(DSlot) / 4);
  hipLaunchKernelGGL(fill_u32_kernel, dim3(grid_for(words, kBlock)), dim3(kBlock), 0, s,
                     reinterpret_cast<uint32_t*>(w.slots), words, 0xFFFFFFFFu);
  const dim3 grid(grid_for(n, kBlock)), block(kBlock);
  launch_dedup_claims(w, d_ids, n, s);
  hipLaunchKernelGGL(dedup_flag_kernel, grid, block, 0, s, w.slots, w.slot_of, n, w.flag);
  KRK_HIP(hipGetLastError());
  KRK_TRY(exclusive_scan_i32(w.flag, w.rank, n, w.d_total, w.scan_tmp, s));
  hipLaunchKernelGGL(dedup_emit_kernel, grid, block, 0, s, w.slots, w.slot_of, w.rank, d_ids, n, d_uids, d_inv,
                     w.d_total, (int32_t*)nullptr);
  KRK_HIP(hipGetLastError());
  return KRK_SUCCESS;
}

// Where a blocking dedup's count lands: page-locked host memory that the kernel which knows the
// total writes to, so the host waits for the stream once and reads it (no copy in the stream).
static int32_t* g_dedup_count = nullptr;

static int32_t dedup_count_buffer() {
  if (g_dedup_count) return KRK_SUCCESS;
  KRK_HIP(hipHostMalloc((void**)&g_dedup_count, 64, hipHostMallocDefault));
  return KRK_SUCCESS;
}

static int32_t dedup_read_count(hipStream_t s, int32_t* u) {
  KRK_HIP(hipStreamSynchronize(s));
  *u = *static_cast<volatile int32_t*>(g_dedup_count);
  return KRK_SUCCESS;
}

static int32_t dedup_core(const DedupWork& w, const uint64_t* d_ids, int64_t n, uint64_t* d_uids,
                          long long* d_inv, hipStream_t s, int32_t* u) {
  KRK_TRY(dedup_count_buffer());
  KRK_HIP(hipMemsetAsync(w.slots, 0xFF, (w.cap + 1) * sizeof(DSlot), s));
  const dim3 grid(grid_for(n, kBlock)), block(kBlock);
  launch_dedup_claims(w, d_ids, n, s);
  hipLaunchKernelGGL(dedup_flag_kernel, grid, block, 0, s, w.slots, w.slot_of, n, w.flag);
  KRK_HIP(hipGetLastError());
  KRK_TRY(exclusive_scan_i32(w.flag, w.rank, n, w.d_total, w.scan_tmp, s));
  hipLaunchKernelGGL(dedup_emit_kernel, grid, block, 0, s, w.slots, w.slot_of, w.rank, d_ids, n, d_uids, d_inv,
                     w.d_total, g_dedup_count);
  KRK_HIP(hipGetLastError());
  return dedup_read_count(s, u);
}

int32_t krk_dedup(const uint64_t* ids, int64_t n, uint64_t* uids, int64_t* inv, int64_t* n_unique,
                  uint32_t flags) {
  KRK_TRY(check_flags(flags));
  if (flags & KRK_ASYNC) return KRK_E_ARGUMENT;   // the count comes back by value
  if (n < 0 || !n_unique || (n > 0 && (!ids || !uids))) return KRK_E_ARGUMENT;
  if (n > ((int64_t)1 << 30)) {   // one thread per id, and slot numbers are 32 bits wide
    set_error("krk_dedup handles at most 2^30 ids per call");
    return KRK_E_CAPACITY;
  }
  KRK_TRY(ensure_runtime());
  *n_unique = 0;
  if (n == 0) return KRK_SUCCESS;
  const bool host = !(flags & KRK_DEVICE_PTRS);
  const size_t n8 = round256((size_t)n * 8);
  std::lock_guard<std::mutex> pool_lock(g_dedup_mu);
  DedupWork w;
  KRK_TRY(dedup_layout(n, host ? 3 * n8 : 0, &w));
  const uint64_t* d_ids = ids;
  uint64_t* d_uids = uids;
  long long* d_inv = reinterpret_cast<long long*>(inv);
  if (host) {
    uint64_t* s_ids = reinterpret_cast<uint64_t*>(w.extra);
    d_uids = reinterpret_cast<uint64_t*>(w.extra + n8);
    d_inv = reinterpret_cast<long long*>(w.extra + 2 * n8);
    KRK_HIP(hipMemcpy(s_ids, ids, (size_t)n * 8, hipMemcpyHostToDevice));
    d_ids = s_ids;
  }
  hipStream_t s = nullptr;
  int32_t u = 0;
  if (n <= kDedupSmall) {
    KRK_TRY(dedup_count_buffer());
    hipLaunchKernelGGL(dedup_small_kernel, dim3(1), dim3(kDedupBlock), 0, s, d_ids, (int)n, d_uids,
                       inv ? d_inv : nullptr, w.d_total, g_dedup_count);
    KRK_HIP(hipGetLastError());
    KRK_TRY(dedup_read_count(s, &u));
  } else {
    KRK_TRY(dedup_core(w, d_ids, n, d_uids, inv ? d_inv : nullptr, s, &u));
  }
  *n_unique = u;
  if (host) {
    KRK_HIP(hipMemcpy(uids, d_uids, (size_t)u * 8, hipMemcpyDeviceToHost));
    if (inv) KRK_HIP(hipMemcpy(inv, d_inv, (size_t)n * 8, hipMemcpyDeviceToHost));
  }
  KRK_HIP(hipStreamSynchronize(s));
  return KRK_SUCCESS;
}

// ---- krk_dedup for callers that cannot allocate ---------------------------------------------
// Same launches as krk_dedup, with the request-local index, the per-position arrays and the scan's
// partial sums in one fixed array of device memory that belongs to the library image instead of
// a pool that grows. The array is shared by every call on the device and keeps the last call's
// contents: the index is cleared by the first launch, everything else is written before it is
// read. Calls that overlap on one device race.
constexpr int64_t kNoAllocCap = (int64_t)KRK_DEDUP_NOALLOC_MAX * 2;   // index slots: at most half full
constexpr size_t kNoAllocSlotsBytes = (((size_t)kNoAllocCap + 1) * sizeof(DSlot) + 255) & ~(size_t)255;
constexpr size_t kNoAllocN4 = (size_t)KRK_DEDUP_NOALLOC_MAX * 4;
constexpr size_t kNoAllocScanBytes = 4096;   // one partial sum per 2048 positions: 512 bytes at the maximum
constexpr size_t kNoAllocBytes = kNoAllocSlotsBytes + 3 * kNoAllocN4 + kNoAllocScanBytes + 256;

static __device__ __align__(256) unsigned char scratch[kNoAllocBytes];

constexpr int kMaxDevices = 64;
static std::mutex g_noalloc_mu;
static unsigned char* g_noalloc_ptr[kMaxDevices] = {};   // the array's address on each device

namespace krk {
__global__ void widen_total_kernel(const int32_t* __restrict__ total, long long* __restrict__ out) {
  if (threadIdx.x == 0 && blockIdx.x == 0) *out = (long long)*total;
}
}  // namespace krk

// The address of `scratch` on the current device (each device holds its own copy of the array
// at its own address), resolved once per device.
static int32_t noalloc_scratch(unsigned char** out) {
  const int dev = current_device();
  if (dev < 0 || dev >= kMaxDevices) {
    set_error("device %d out of range for krk_dedup_noalloc", dev);
    return KRK_E_ARGUMENT;
  }
  std::lock_guard<std::mutex> lk(g_noalloc_mu);
  if (!g_noalloc_ptr[dev]) {
    void* p = nullptr;
    KRK_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p) {
      set_error("hipGetSymbolAddress returned no address for the dedup work space");
      return KRK_E_DEVICE;
    }
    g_noalloc_ptr[dev] = reinterpret_cast<unsigned char*>(p);
  }
  *out = g_noalloc_ptr[dev];
  return KRK_SUCCESS;
}

// Called when the library binds a device (krk_runtime_init, or the first call of anything): the
// array's address is resolved there, with whatever that costs the runtime the first time (loading
// the code object, backing the array), so that krk_dedup_noalloc itself finds it ready, also
// under stream capture.
}  // extern "C"
int32_t krk::noalloc_prepare() {
  unsigned char* base = nullptr;
  return noalloc_scratch(&base);
}
extern "C" {

int32_t krk_dedup_noalloc(const uint64_t* ids, int64_t n, uint64_t* uids, int64_t* inv,
                          int64_t* n_unique, void* stream) {
  if (n < 0 || !n_unique || (n > 0 && (!ids || !uids))) return KRK_E_ARGUMENT;
  if (n > (int64_t)KRK_DEDUP_NOALLOC_MAX) {
    set_error("krk_dedup_noalloc handles at most %d ids per call (%lld given); use krk_dedup",
              (int)KRK_DEDUP_NOALLOC_MAX, (long long)n);
    return KRK_E_CAPACITY;
  }
  KRK_TRY(ensure_runtime());
  unsigned char* base = nullptr;
  KRK_TRY(noalloc_scratch(&base));
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  DedupWork w;
  uint64_t cap = 1024;
  while (cap < (uint64_t)n * 2) cap <<= 1;
  unsigned char* cur = base;
  w.slots = reinterpret_cast<DSlot*>(cur); cur += kNoAllocSlotsBytes;
  w.cap = cap;
  w.slot_of = reinterpret_cast<uint32_t*>(cur); cur += kNoAllocN4;
  w.flag = reinterpret_cast<int32_t*>(cur); cur += kNoAllocN4;
  w.rank = reinterpret_cast<int32_t*>(cur); cur += kNoAllocN4;
  w.scan_tmp = cur; cur += kNoAllocScanBytes;
  w.d_total = reinterpret_cast<int32_t*>(cur);
  w.extra = nullptr;
  if (n == 0) {
    // the count still has to arrive in the caller's memory, in stream order
    hipLaunchKernelGGL(fill_u32_kernel, dim3(1), dim3(kBlock), 0, s, reinterpret_cast<uint32_t*>(n_unique),
                       (int64_t)2, 0u);
    KRK_HIP(hipGetLastError());
    return KRK_SUCCESS;
  }
  KRK_TRY(dedup_enqueue(w, ids, n, uids, reinterpret_cast<long long*>(inv), s));
  hipLaunchKernelGGL(widen_total_kernel, dim3(1), dim3(64), 0, s, w.d_total,
                     reinterpret_cast<long long*>(n_unique));
  KRK_HIP(hipGetLastError());
  return KRK_SUCCESS;
}

int32_t krk_dedup_sum(const uint64_t* ids, int64_t n, const float* grads, int64_t dim, uint64_t* uids,
                      int64_t* inv, float* sums, int64_t* n_unique, uint32_t flags) {
  KRK_TRY(check_flags(flags));
  if (flags & KRK_ASYNC) return KRK_E_ARGUMENT;   // the count comes back by value
  if (n < 0 || dim <= 0 || !n_unique || (n > 0 && (!ids || !grads || !uids || !sums))) return KRK_E_ARGUMENT;
  if (n > ((int64_t)1 << 28)) {
    set_error("krk_dedup_sum handles at most 2^28 ids per call; split the request");
    return KRK_E_CAPACITY;
  }
  KRK_TRY(ensure_runtime());
  *n_unique = 0;
  if (n == 0) return KRK_SUCCESS;
  ReduceShape sh;
  sh.dim = dim;
  sh.vec = dim % 4 == 0 ? 4 : 1;
  sh.elems = (int)(dim / sh.vec);
  sh.group = 4;
  while (sh.group < sh.elems && sh.group < 64) sh.group <<= 1;
  const bool host = !(flags & KRK_DEVICE_PTRS);
  if (!host && sh.vec == 4 && ((((uintptr_t)grads) | ((uintptr_t)sums)) & 15)) {
    set_error("device gradients and sums must be 16-byte aligned");
    return KRK_E_ARGUMENT;
  }
  const size_t n8 = round256((size_t)n * 8);
  const size_t rows_b = round256((size_t)n * (size_t)dim * sizeof(float));
  std::lock_guard<std::mutex> pool_lock(g_dedup_mu);
  DedupWork w;
  KRK_TRY(dedup_layout(n, host ? 3 * n8 + 2 * rows_b : 0, &w));
  const uint64_t* d_ids = ids;
  const float* d_g = grads;
  uint64_t* d_uids = uids;
  long long* d_inv = reinterpret_cast<long long*>(inv);
  float* d_sums = sums;
  if (host) {
    uint64_t* s_ids = reinterpret_cast<uint64_t*>(w.extra);
    d_uids = reinterpret_cast<uint64_t*>(w.extra + n8);
    d_inv = reinterpret_cast<long long*>(w.extra + 2 * n8);
    float* s_g = reinterpret_cast<float*>(w.extra + 3 * n8);
    d_sums = reinterpret_cast<float*>(w.extra + 3 * n8 + rows_b);
    KRK_HIP(hipMemcpy(s_ids, ids, (size_t)n * 8, hipMemcpyHostToDevice));
    KRK_HIP(hipMemcpy(s_g, grads, (size_t)n * (size_t)dim * sizeof(float), hipMemcpyHostToDevice));
    d_ids = s_ids;
    d_g = s_g;
  }
  hipStream_t s = nullptr;
  int32_t u = 0;
  KRK_TRY(dedup_core(w, d_ids, n, d_uids, inv ? d_inv : nullptr, s, &u));
  // positions sorted by unique index (stable: position order inside a run, as
  // worker/emitter.cc:527-529 adds them), every run summed and stored as row `index` of sums
  uint32_t miss_key = 1;
  int bits = 1;
  while ((int64_t)miss_key < (int64_t)u) {
    miss_key <<= 1;
    ++bits;
  }
  TableView tv{};
  tv.recs = d_sums;
  tv.stride = dim;
  ApplyArgs args{};
  args.c0 = args.c1 = args.c2 = args.meta_off = -1;
  const DSlot* slots = w.slots;
  const uint32_t* slot_of = w.slot_of;
  KRK_TRY(sort_and_reduce(sh, s, g_dedup_reduce, tv, kOptStore, n, miss_key, bits, d_g, args,
                          PooledSrc{nullptr, nullptr}, nullptr, [&](uint32_t* keys, uint32_t* pos) {
                            hipLaunchKernelGGL(dedup_pairs_kernel, dim3(grid_for(n, kBlock)), dim3(kBlock), 0, s,
                                               slots, slot_of, n, keys, pos);
                          }));
  *n_unique = u;
  if (host) {
    KRK_HIP(hipMemcpy(uids, d_uids, (size_t)u * 8, hipMemcpyDeviceToHost));
    if (inv) KRK_HIP(hipMemcpy(inv, d_inv, (size_t)n * 8, hipMemcpyDeviceToHost));
    KRK_HIP(hipMemcpy(sums, d_sums, (size_t)u * (size_t)dim * sizeof(float), hipMemcpyDeviceToHost));
  }
  KRK_HIP(hipStreamSynchronize(s));
  return KRK_SUCCESS;
}

int32_t krk_expand_rows(const float* rows, int64_t n_rows, const int64_t* inv, int64_t n, int64_t dim,
                        float* out, uint32_t flags) {
  KRK_TRY(check_flags(flags));
  if (n < 0 || n_rows < 0 || dim <= 0 || (n > 0 && (!rows || !inv || !out))) return KRK_E_ARGUMENT;
  KRK_TRY(ensure_runtime());
  if (n == 0) return KRK_SUCCESS;
  const int vec = dim % 4 == 0 ? 4 : 1;
  const int elems = (int)(dim / vec);
  const bool host = !(flags & KRK_DEVICE_PTRS);
  if (!host && vec == 4 && ((((uintptr_t)rows) | ((uintptr_t)out)) & 15)) {
    set_error("device rows and output must be 16-byte aligned");
    return KRK_E_ARGUMENT;
  }
  const size_t in_b = round256((size_t)n_rows * (size_t)dim * sizeof(float));
  const size_t inv_b = round256((size_t)n * 8);
  const size_t out_b = round256((size_t)n * (size_t)dim * sizeof(float));
  std::lock_guard<std::mutex> pool_lock(g_dedup_mu);
  KRK_TRY(g_dedup_pool.reserve(256 + (host ? in_b + inv_b + out_b : 0)));
  char* base = g_dedup_pool.as<char>();
  uint32_t* d_err = reinterpret_cast<uint32_t*>(base);
  const float* d_rows = rows;
  const long long* d_inv = reinterpret_cast<const long long*>(inv);
  float* d_out = out;
  hipStream_t s = nullptr;
  if (host) {
    float* s_rows = reinterpret_cast<float*>(base + 256);
    long long* s_inv = reinterpret_cast<long long*>(base + 256 + in_b);
    d_out = reinterpret_cast<float*>(base + 256 + in_b + inv_b);
    KRK_HIP(hipMemcpy(s_rows, rows, (size_t)n_rows * (size_t)dim * sizeof(float), hipMemcpyHostToDevice));
    KRK_HIP(hipMemcpy(s_inv, inv, (size_t)n * 8, hipMemcpyHostToDevice));
    d_rows = s_rows;
    d_inv = s_inv;
  }
  KRK_HIP(hipMemsetAsync(d_err, 0, 4, s));
  int64_t blocks = (n * elems + kBlock - 1) / kBlock;
  if (blocks > 256 * 64) blocks = 256 * 64;   // grid-stride beyond that
  if (vec == 4) {
    hipLaunchKernelGGL((expand_rows_kernel<4>), dim3((unsigned)blocks), dim3(kBlock), 0, s, d_rows, d_inv, n,
                       n_rows, d_out, (int)dim, elems, d_err);
  } else {
    hipLaunchKernelGGL((expand_rows_kernel<1>), dim3((unsigned)blocks), dim3(kBlock), 0, s, d_rows, d_inv, n,
                       n_rows, d_out, (int)dim, elems, d_err);
  }
  KRK_HIP(hipGetLastError());
  uint32_t err = 0;
  KRK_HIP(hipMemcpy(&err, d_err, 4, hipMemcpyDeviceToHost));
  if (host) KRK_HIP(hipMemcpy(out, d_out, (size_t)n * (size_t)dim * sizeof(float), hipMemcpyDeviceToHost));
  KRK_HIP(hipStreamSynchronize(s));
  if (err) {
    set_error("an index lies outside the %lld rows", (long long)n_rows);
    return KRK_E_ARGUMENT;
  }
  return KRK_SUCCESS;
}

int32_t krk_sparse_push_raw(krk_sparse* t, const krk_optim* o, const uint64_t* ids, int64_t n,
                            const float* grads, int64_t grad_dim, float lr, uint32_t flags) {
  if (!t) return KRK_E_ARGUMENT;
  KRK_TRY(ensure_runtime());
  KRK_TRY(check_flags(flags));
  if (!o || o->type < KRK_ADAGRAD || o->type > KRK_SGD) {
    set_error("optimizer type is not supported");
    return KRK_UNSUPPORTED_OPTIM;
  }
  if (n < 0 || (n > 0 && (!ids || !grads))) return KRK_E_ARGUMENT;
  if (n > ((int64_t)1 << 28)) {
    set_error("krk_sparse_push_raw handles at most 2^28 ids per call; split the request");
    return KRK_E_CAPACITY;
  }
  std::lock_guard<std::mutex> lk(t->mu);
  if (n == 0) return sparse_finish(t, flags);
  if (grad_dim != t->dim) {
    set_error("gradient width %lld does not match table dimension %lld", (long long)grad_dim,
              (long long)t->dim);
    return KRK_GRADIENT_UNCOMPATIBLE;
  }
  KRK_TRY(sparse_ensure_columns(t, optim_state_mask(*o)));
  const uint64_t* d_ids;
  const float* d_g;
  KRK_TRY(t->input(ids, (size_t)n, flags, 0, &d_ids));
  KRK_TRY(t->input(grads, (size_t)n * t->dim, flags, 1, &d_g));

  if (short_push_fits(n, t->dim, t->elems, t->group)) {
    // a short request: see bucket_push_kernel
    SortCall sc;
    sc.n_tables = 1;
    sc.bucket_bits = short_bucket_bits(1);
    sc.row_bits = 1;
    while (((int64_t)1 << sc.row_bits) < t->row_cap) ++sc.row_bits;
    sc.row_mask = 0xFFFFFFFFu;
    sc.miss_key = kNoRow;
    sc.note_ids = nullptr;
    sc.row_start[0] = 0;
    sc.row_start[1] = n;
    ApplyArgs args;
    args.lr = lr;
    args.k = make_optim_k(*o);
    int32_t cols[3];
    sparse_optim_columns(t, *o, cols);
    args.c0 = cols[0];
    args.c1 = cols[1];
    args.c2 = cols[2];
    args.meta_off = ((optim_state_mask(*o) >> KRK_ST_STEPS) & 1u) ? t->meta_off : -1;
    const TableView tv = t->view();
    // KRK_IDS_AS_PULLED: the rows of these very ids were noted by the pull before (and nothing
    // has moved since): the look-up launch is not needed
    const uint32_t* keys = noted_rows(t, ids, n, flags);
    const bool noted = keys != nullptr;
    if (!noted) {
      KRK_TRY(t->scratch[0].reserve((size_t)n * sizeof(uint32_t)));
      uint32_t* found = t->scratch[0].as<uint32_t>();
      hipLaunchKernelGGL(rows_of_ids_kernel, dim3(grid_for(n, kBlock / kBucket)), dim3(kBlock), 0, t->stream, tv,
                         d_ids, n, kNoRow, (const uint32_t*)nullptr, false, found, (uint32_t*)nullptr);
      keys = found;
    } else {
      sc.note_ids = d_ids;
    }
    const GroupSrc none{nullptr, 0, -1, -1, -1, 0};
    if (t->vec == 4) {
      launch_bucket_push<4, false>(o->type, 1u << sc.bucket_bits, t->stream, nullptr, tv, sc, keys, d_g, (int)t->dim, t->elems,
                                   t->group, args, none);
    } else {
      launch_bucket_push<1, false>(o->type, 1u << sc.bucket_bits, t->stream, nullptr, tv, sc, keys, d_g, (int)t->dim, t->elems,
                                   t->group, args, none);
    }
    KRK_HIP(hipGetLastError());
    return sparse_finish(t, flags);
  }
  KRK_TRY(push_sorted(t, o, d_ids, n, d_g, lr, nullptr, false, PooledSrc{nullptr, nullptr}));
  return sparse_finish(t, flags);
}

int32_t krk_group_push_raw(krk_group* g, const krk_optim* o, const uint64_t* ids, const int64_t* offsets,
                           const float* grads, int64_t grad_dim, float lr, uint32_t flags) {
  if (!g || !offsets) return KRK_E_ARGUMENT;
  KRK_TRY(ensure_runtime());
  KRK_TRY(check_flags(flags));
  if (!o || o->type < KRK_ADAGRAD || o->type > KRK_SGD) {
    set_error("optimizer type is not supported");
    return KRK_UNSUPPORTED_OPTIM;
  }
  GroupLock lk(g);
  GroupCall call;
  int64_t total = 0;
  KRK_TRY(group_plan(g, offsets, &call, &total));
  if (total == 0) return group_finish(g, flags);
  if (!ids || !grads) return KRK_E_ARGUMENT;
  if (total > ((int64_t)1 << 28)) {
    set_error("krk_group_push_raw handles at most 2^28 ids per call; split the request");
    return KRK_E_CAPACITY;
  }
  if (grad_dim != g->dim) {
    set_error("gradient width %lld does not match table dimension %lld", (long long)grad_dim,
              (long long)g->dim);
    return KRK_GRADIENT_UNCOMPATIBLE;
  }
  const uint32_t mask = optim_state_mask(*o);
  for (krk_sparse* t : g->tables) KRK_TRY(sparse_ensure_columns(t, mask));
  KRK_TRY(group_refresh(g));
  // sort key: member number above the row number; one value above every key marks a missing id
  int row_bits = 1;
  for (krk_sparse* t : g->tables)
    while (((int64_t)1 << row_bits) < t->row_cap) ++row_bits;
  const int n_tables = (int)g->tables.size();
  int member_bits = 1;
  while ((1 << member_bits) <= n_tables) ++member_bits;
  if (row_bits + member_bits > 32) {
    set_error("combined push with repeats: %d tables of up to 2^%d rows do not fit a 32-bit sort key",
              n_tables, row_bits);
    return KRK_E_CAPACITY;
  }
  const uint32_t miss_key = (uint32_t)n_tables << row_bits;
  // members of at most 8192 ids each are sorted one workgroup a member
  bool by_member = true;
  int64_t longest = 0;
  for (int m = 0; m < n_tables; ++m) {
    by_member = by_member && offsets[m + 1] - offsets[m] <= kSortMax;
    longest = std::max(longest, offsets[m + 1] - offsets[m]);
  }
  // the launch that turns ids into rows gives every member whole workgroups of its own
  GroupCall rows_call = call;
  uint32_t blocks = 0;
  bool even = true;
  for (int m = 0; m < n_tables; ++m) {
    rows_call.block_start[m] = blocks;
    const uint32_t mine = grid_for(offsets[m + 1] - offsets[m], kBlock / kBucket);
    even = even && mine == grid_for(offsets[1] - offsets[0], kBlock / kBucket);
    blocks += mine;
  }
  rows_call.block_start[n_tables] = blocks;
  rows_call.even_blocks = even && blocks > 0 ? blocks / (uint32_t)n_tables : 0u;
  const uint64_t* d_ids;
  const float* d_g;
  KRK_TRY(g->input(ids, (size_t)total, flags, 0, &d_ids));
  KRK_TRY(g->input(grads, (size_t)total * g->dim, flags, 1, &d_g));
  ApplyArgs args;
  args.lr = lr;
  args.k = make_optim_k(*o);
  args.c0 = args.c1 = args.c2 = args.meta_off = -1;     // taken per member from its layout
  int32_t st[3];
  optim_state_slots(*o, st);
  const GroupSrc gs{g->d_descs, row_bits, st[0], st[1], st[2], (int)((mask >> KRK_ST_STEPS) & 1u)};
  if (by_member && short_push_fits(longest, g->dim, g->elems, g->group)) {
    // short members: see bucket_push_kernel
    SortCall sc;
    sc.n_tables = n_tables;
    sc.bucket_bits = short_bucket_bits(n_tables);
    sc.row_bits = row_bits;
    sc.row_mask = row_bits >= 32 ? 0xFFFFFFFFu : ((1u << row_bits) - 1u);
    sc.miss_key = miss_key;
    sc.note_ids = nullptr;
    for (int m = 0; m <= n_tables; ++m) sc.row_start[m] = offsets[m];
    // KRK_IDS_AS_PULLED: the rows of these very ids were noted by the combined pull before (and
    // nothing has moved since): the look-up launch is not needed. A note is a member's own row
    // number, which is all the bucket kernel reads of a key.
    const uint32_t* keys = noted_rows(g, ids, offsets, flags);
    const bool noted = keys != nullptr;
    if (!noted) {
      KRK_TRY(g->scratch[0].reserve((size_t)total * sizeof(uint32_t)));
      uint32_t* found = g->scratch[0].as<uint32_t>();
      hipLaunchKernelGGL(group_rows_of_ids_kernel, dim3(rows_call.block_start[n_tables]), dim3(kBlock), 0,
                         g->stream, g->d_descs, rows_call, d_ids, total, row_bits, miss_key, found,
                         (uint32_t*)nullptr);
      keys = found;
    } else {
      sc.note_ids = d_ids;
    }
    if (g->vec == 4) {
      launch_bucket_push<4, true>(o->type, (unsigned)n_tables << sc.bucket_bits, g->stream, g->d_descs, TableView{}, sc,
                                  keys, d_g, (int)g->dim, g->elems, g->group, args, gs);
    } else {
      launch_bucket_push<1, true>(o->type, (unsigned)n_tables << sc.bucket_bits, g->stream, g->d_descs, TableView{}, sc,
                                  keys, d_g, (int)g->dim, g->elems, g->group, args, gs);
    }
    KRK_HIP(hipGetLastError());
    return group_finish(g, flags);
  }
  TableView none{};
  const ReduceShape sh{g->dim, g->vec, g->elems, g->group};
  KRK_TRY(sort_and_reduce(sh, g->stream, g->scratch, none, o->type, total, miss_key, row_bits + member_bits,
                          d_g, args, PooledSrc{nullptr, nullptr}, &gs, [&](uint32_t* keys, uint32_t* pos) {
                            hipLaunchKernelGGL(group_rows_of_ids_kernel, dim3(rows_call.block_start[n_tables]),
                                               dim3(kBlock), 0, g->stream, g->d_descs, rows_call, d_ids, total,
                                               row_bits, miss_key, keys, pos);
                          }));
  return group_finish(g, flags);
}

int32_t krk_sparse_push_pooled(krk_sparse* t, const krk_optim* o, const uint64_t* ids, int64_t n,
                               const int64_t* offsets, int64_t bags, const float* weights, int32_t mode,
                               const float* bag_grads, int64_t grad_dim, float lr, uint32_t flags) {
  if (!t) return KRK_E_ARGUMENT;
  KRK_TRY(ensure_runtime());
  KRK_TRY(check_flags(flags));
  if (!o || o->type < KRK_ADAGRAD || o->type > KRK_SGD) {
    set_error("optimizer type is not supported");
    return KRK_UNSUPPORTED_OPTIM;
  }
  if (n < 0 || bags < 0 || (mode != KRK_POOL_SUM && mode != KRK_POOL_MEAN) || !offsets ||
      (n > 0 && !ids) || (bags > 0 && !bag_grads))
    return KRK_E_ARGUMENT;
  if (n > ((int64_t)1 << 28) || bags > ((int64_t)1 << 28)) {
    set_error("krk_sparse_push_pooled handles at most 2^28 ids and bags per call; split the request");
    return KRK_E_CAPACITY;
  }
  if (bags * t->dim >= ((int64_t)1 << 31)) {   // one work-item per bag gradient element
    set_error("krk_sparse_push_pooled: bags x dim must stay below 2^31; split the request");
    return KRK_E_CAPACITY;
  }
  const bool host = !(flags & KRK_DEVICE_PTRS);
  if (host && (offsets[0] != 0 || offsets[bags] != n)) {
    set_error("offsets must start at 0 and end at the number of ids");
    return KRK_E_ARGUMENT;
  }
  std::lock_guard<std::mutex> lk(t->mu);
  if (n == 0 || bags == 0) return sparse_finish(t, flags);
  if (grad_dim != t->dim) {
    set_error("gradient width %lld does not match table dimension %lld", (long long)grad_dim,
              (long long)t->dim);
    return KRK_GRADIENT_UNCOMPATIBLE;
  }
  KRK_TRY(sparse_ensure_columns(t, optim_state_mask(*o)));
  const uint64_t* d_ids;
  const long long* d_off;
  const float* d_w = nullptr;
  const float* d_g;
  KRK_TRY(t->input(ids, (size_t)n, flags, 0, &d_ids));
  KRK_TRY(t->input(reinterpret_cast<const long long*>(offsets), (size_t)bags + 1, flags, 1, &d_off));
  if (weights) KRK_TRY(t->input(weights, (size_t)n, flags, 2, &d_w));
  KRK_TRY(t->input(bag_grads, (size_t)bags * t->dim, flags, 3, &d_g));

  const size_t bag_of_bytes = ((size_t)n * sizeof(uint32_t) + 255) & ~(size_t)255;
  const size_t scaled_bytes = mode == KRK_POOL_MEAN ? (size_t)bags * t->dim * sizeof(float) : 0;
  KRK_TRY(t->scratch[5].reserve(bag_of_bytes + scaled_bytes));
  uint32_t* bag_of = t->scratch[5].as<uint32_t>();
  hipLaunchKernelGGL(fill_u32_kernel, dim3(grid_for(n, kBlock)), dim3(kBlock), 0, t->stream, bag_of, n, kNoBag);
  hipLaunchKernelGGL(bag_expand_kernel, dim3(grid_for(bags, kBlock / kBagLanes)), dim3(kBlock), 0, t->stream,
                     d_off, bags, n, bag_of);
  if (mode == KRK_POOL_MEAN) {
    float* scaled = reinterpret_cast<float*>(t->scratch[5].as<char>() + bag_of_bytes);
    hipLaunchKernelGGL(bag_scale_kernel, dim3(grid_for(bags * t->dim, kBlock)), dim3(kBlock), 0, t->stream,
                       d_g, d_off, bags, (int)t->dim, scaled);
    d_g = scaled;
  }
  KRK_HIP(hipGetLastError());
  // Unweighted: the sort carries bag numbers and the reduction reads bag rows directly.
  // Weighted: it carries positions, which name the weight and (through bag_of) the bag.
  KRK_TRY(push_sorted(t, o, d_ids, n, d_g, lr, bag_of, d_w == nullptr, PooledSrc{d_w ? bag_of : nullptr, d_w}));
  return sparse_finish(t, flags);
}

}  // extern "C"
