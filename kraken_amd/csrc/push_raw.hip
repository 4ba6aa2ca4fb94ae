// The worker-side half of a sparse push, moved onto the device and fused with the table update:
//   krk_dedup            Emitter::PullSparseTableImpl's dedup (worker/emitter.cc:131-149)
//   krk_sparse_push_raw  Emitter::PushSparseTable's dedup + duplicate-gradient sum
//                        (worker/emitter.cc:510-531) followed by SparseTable::Push
//
// push_raw never builds the unique list. Positions are sorted by the row their id maps to
// (stable, so equal rows keep position order), then a tiled segmented reduction walks the
// sorted sequence: every group of lanes owns a fixed-size tile, sums each run of equal rows in
// registers and, when a run lies wholly inside the tile, applies the optimizer to that row at
// once. Runs that touch a tile border leave a partial sum in a carry list, which is itself a
// sorted sequence of (row, partial) and is reduced by the same kernel again until one tile is
// left. Work per group is bounded by the tile size however skewed the ids are, and the order
// of additions is fixed, so results do not change from run to run.
#include <cstring>
#include <new>

#include <rocprim/device/device_radix_sort.hpp>

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

__global__ __launch_bounds__(kBlock) void dedup_claim_kernel(DSlot* slots, uint64_t mask,
                                                             const uint64_t* __restrict__ ids, int64_t n,
                                                             uint32_t* __restrict__ slot_of) {
  const int64_t p = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  const bool active = p < n;
  const unsigned long long id = active ? ids[p] : 0ull;
  const int lane = (int)(threadIdx.x & (kWave - 1));
  // Equal ids inside one wavefront are folded first: positions grow with the lane number, so
  // the lowest lane holding an id also holds its smallest position in this wave. Only that lane
  // goes to the index; the others take the slot number from it. An id that fills a quarter of
  // the request then costs one atomic per wave instead of sixteen.
  int leader = lane;
  unsigned long long todo = __ballot(active);
  while (todo) {
    const int first = __ffsll((unsigned long long)todo) - 1;
    const unsigned int lo = __builtin_amdgcn_readlane((unsigned int)id, first);
    const unsigned int hi = __builtin_amdgcn_readlane((unsigned int)(id >> 32), first);
    const unsigned long long lid = (unsigned long long)lo | ((unsigned long long)hi << 32);
    const bool same = active && id == lid;
    if (same) leader = first;
    todo &= ~__ballot(same);
  }
  uint64_t idx = 0;
  if (active && leader == lane) {
    if (id == kEmptyKey) {
      idx = mask + 1;   // the all-ones id owns the extra last slot
    } else {
      idx = mix64(id) & mask;
      for (uint64_t t = 0; t <= mask; ++t) {
        unsigned long long key = __atomic_load_n(&slots[idx].key, __ATOMIC_RELAXED);
        if (key == kEmptyKey) {
          const unsigned long long old = atomicCAS(&slots[idx].key, kEmptyKey, id);
          key = old == kEmptyKey ? id : old;
        }
        if (key == id) break;
        idx = (idx + 1) & mask;
      }
    }
    // minpos only ever decreases, so a stale read can at worst cause a redundant atomic; later
    // waves mostly find a smaller position already there and skip it.
    if (__builtin_nontemporal_load(&slots[idx].minpos) > (uint32_t)p)
      atomicMin(&slots[idx].minpos, (uint32_t)p);
  }
  const uint32_t shared_idx = __shfl((uint32_t)idx, leader);
  if (active) slot_of[p] = shared_idx;
}

__global__ __launch_bounds__(kBlock) void dedup_flag_kernel(const DSlot* __restrict__ slots,
                                                            const uint32_t* __restrict__ slot_of,
                                                            int64_t n, int32_t* __restrict__ flag) {
  const int64_t p = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (p >= n) return;
  flag[p] = slots[slot_of[p]].minpos == (uint32_t)p ? 1 : 0;
}

__global__ __launch_bounds__(kBlock) void dedup_emit_kernel(DSlot* slots,
                                                            const uint32_t* __restrict__ slot_of,
                                                            const int32_t* __restrict__ rank,
                                                            const uint64_t* __restrict__ ids, int64_t n,
                                                            uint64_t* __restrict__ uids) {
  const int64_t p = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (p >= n) return;
  DSlot* s = &slots[slot_of[p]];
  if (s->minpos == (uint32_t)p) {
    uids[rank[p]] = ids[p];
    s->uidx = (uint32_t)rank[p];
  }
}

__global__ __launch_bounds__(kBlock) void dedup_inv_kernel(const DSlot* __restrict__ slots,
                                                           const uint32_t* __restrict__ slot_of,
                                                           int64_t n, long long* __restrict__ inv) {
  const int64_t p = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (p >= n) return;
  inv[p] = (long long)slots[slot_of[p]].uidx;
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
  pos[p] = payload_is_bag ? bag : (uint32_t)p;
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

template <int OPT, int VEC>
__device__ __forceinline__ void apply_row(const TableView& tv, uint32_t row, const float (&gsum)[VEC],
                                          int e, bool lane_on, bool leader, bool last_chunk,
                                          const ApplyArgs& a) {
  float* rec = tv.recs + (int64_t)row * tv.stride;
  bool first = false;
  float bc1 = 1.0f, bc2 = 1.0f;
  uint64_t steps = 0;
  if (a.meta_off >= 0) {
    const uint32_t* meta = reinterpret_cast<const uint32_t*>(rec + a.meta_off);
    steps = (uint64_t)meta[0] | ((uint64_t)meta[1] << 32);
    first = steps == 0;
    steps += 1;
    if (OPT == KRK_ADAM) {
      bc1 = (float)(1.0 - (double)powf(a.k.beta1, (float)steps));
      bc2 = (float)(1.0 - (double)powf(a.k.beta2, (float)steps));
    }
  }
  if (lane_on) {
    float w[VEC], s0[VEC], s1[VEC], s2[VEC];
    vload<VEC>(rec + e * VEC, w);
    if (a.c0 >= 0) vload<VEC>(rec + a.c0 + e * VEC, s0);
    if (a.c1 >= 0) vload<VEC>(rec + a.c1 + e * VEC, s1);
    if (a.c2 >= 0) vload<VEC>(rec + a.c2 + e * VEC, s2);
#pragma unroll
    for (int c = 0; c < VEC; ++c) {
      if (a.c0 < 0) s0[c] = 0.0f;
      if (a.c1 < 0) s1[c] = 0.0f;
      if (a.c2 < 0) s2[c] = 0.0f;
      optim_element<OPT>(a.k, a.lr, gsum[c], w[c], s0[c], s1[c], s2[c], first, bc1, bc2);
    }
    vstore<VEC>(rec + e * VEC, w);
    if (a.c0 >= 0) vstore<VEC>(rec + a.c0 + e * VEC, s0);
    if (a.c1 >= 0) vstore<VEC>(rec + a.c1 + e * VEC, s1);
    if (a.c2 >= 0) vstore<VEC>(rec + a.c2 + e * VEC, s2);
  }
  // The counter is read by every chunk of the row before the last chunk's leader advances it.
  if (a.meta_off >= 0 && leader && last_chunk) {
    uint32_t* meta = reinterpret_cast<uint32_t*>(rec + a.meta_off);
    meta[0] = (uint32_t)steps;
    meta[1] = (uint32_t)(steps >> 32);
  }
}

// keys[cnt] ascending (entries >= empty_from are holes). LEVEL0: the value of entry j is gradient
// row pos[j]; otherwise it is vals[j, :]. Each tile of `tile` entries writes carry slots 2t
// (run entering from the left) and 2t+1 (run leaving to the right).
//
// A workgroup first stages the keys (and positions) of all its tiles in LDS with coalesced loads,
// including one neighbour on each side, so the walk itself only waits for value rows; those are
// requested four entries ahead of where the sums are. Carry levels use short tiles: the lists
// are short, so short tiles keep many lane groups busy (tiles of 32 with eight entries in
// flight save one or two dependent launches but measured slower, 442 vs 432 us at 1M ids).
constexpr int kPrefetch = 4;
constexpr int kPrefetchCarry = 4;
constexpr int kCarryTile = 16;

// Weighted bags (level 0 only): the sorted payload is a position p, its gradient row is
// vals[bag_of[p]] times weight[p]. Both null otherwise: the payload itself names the row.
struct PooledSrc {
  const uint32_t* bag_of;
  const float* weight;
};

template <int OPT, int VEC, bool LEVEL0>
__global__ __launch_bounds__(kBlock) void segreduce_kernel(
    TableView tv, const uint32_t* __restrict__ keys, const uint32_t* __restrict__ pos,
    const float* __restrict__ vals, int64_t cnt, int tile, uint32_t empty_from,
    uint32_t* __restrict__ keys_out, float* __restrict__ vals_out, int dim, int elems, int group,
    ApplyArgs args, PooledSrc ps) {
  extern __shared__ uint32_t lds[];
  const int per_block = kBlock / group;
  const int span = per_block * tile;                       // entries staged by this workgroup
  const int64_t first = (int64_t)blockIdx.x * span;        // global index of lds_keys[1]
  uint32_t* lds_keys = lds;                                // [span + 2], shifted by one
  uint32_t* lds_pos = lds + span + 2;                      // [span]
  float* lds_w = reinterpret_cast<float*>(lds + 2 * span + 2);   // [span], weighted bags only
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
  __syncthreads();

  const int64_t t = (int64_t)blockIdx.x * per_block + threadIdx.x / group;
  const int gl = threadIdx.x & (group - 1);
  const int64_t a = t * tile;
  if (a >= cnt) return;
  const int64_t b = a + tile < cnt ? a + tile : cnt;
  const int la = (int)(a - first);                          // tile's first entry, LDS-relative
  const int lb = (int)(b - first);
  const uint32_t left_key = lds_keys[la];                   // entry a - 1
  const uint32_t right_key = lds_keys[lb + 1];              // entry b
  const bool leader = gl == 0;
  uint32_t carry_key0 = kNoRow, carry_key1 = kNoRow;        // what this tile leaves in the carry list

  for (int e0 = 0; e0 < elems; e0 += group) {
    const int e = e0 + gl;
    const bool lane_on = e < elems;
    const bool last_chunk = e0 + group >= elems;
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
        apply_row<OPT, VEC>(tv, run_key, acc, e, lane_on, leader, last_chunk, args);
        return;
      }
      const int64_t slot = open_left ? 2 * t : 2 * t + 1;
      if (lane_on) vstore<VEC>(vals_out + slot * dim + e * VEC, acc);
      if (open_left) carry_key0 = run_key; else carry_key1 = run_key;
      if (open_left && open_right) {
        // the run covers the whole tile: keep the carry list contiguous with a zero piece
        float z[VEC];
#pragma unroll
        for (int c = 0; c < VEC; ++c) z[c] = 0.0f;
        if (lane_on) vstore<VEC>(vals_out + (slot + 1) * dim + e * VEC, z);
        carry_key1 = run_key;
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
          vload<VEC>(src + e * VEC, v[u]);
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
  if (leader && keys_out) {
    keys_out[2 * t] = carry_key0;
    keys_out[2 * t + 1] = carry_key1;
  }
}

template <int OPT, int VEC>
static void launch_segreduce(bool level0, const TableView& tv, const uint32_t* keys, const uint32_t* pos,
                             const float* vals, int64_t cnt, int tile, uint32_t empty_from,
                             uint32_t* keys_out, float* vals_out, const krk_sparse* t,
                             const ApplyArgs& args, const PooledSrc& ps, hipStream_t stream) {
  const int per_block = kBlock / t->group;
  const int64_t tiles = (cnt + tile - 1) / tile;
  const dim3 grid(grid_for(tiles, per_block)), block(kBlock);
  const size_t lds_bytes = (size_t)(3 * per_block * tile + 2) * sizeof(uint32_t);
  if (level0) {
    hipLaunchKernelGGL((segreduce_kernel<OPT, VEC, true>), grid, block, lds_bytes, stream, tv, keys, pos,
                       vals, cnt, tile, empty_from, keys_out, vals_out, (int)t->dim, t->elems, t->group,
                       args, ps);
  } else {
    hipLaunchKernelGGL((segreduce_kernel<OPT, VEC, false>), grid, block, lds_bytes, stream, tv, keys, pos,
                       vals, cnt, tile, empty_from, keys_out, vals_out, (int)t->dim, t->elems, t->group,
                       args, PooledSrc{nullptr, nullptr});
  }
}

template <int VEC>
static void dispatch_segreduce(int opt, bool level0, const TableView& tv, const uint32_t* keys,
                               const uint32_t* pos, const float* vals, int64_t cnt, int tile,
                               uint32_t empty_from, uint32_t* keys_out, float* vals_out,
                               const krk_sparse* t, const ApplyArgs& args, const PooledSrc& ps,
                               hipStream_t stream) {
  switch (opt) {
    case KRK_SGD:
      launch_segreduce<KRK_SGD, VEC>(level0, tv, keys, pos, vals, cnt, tile, empty_from, keys_out,
                                     vals_out, t, args, ps, stream);
      break;
    case KRK_ADAGRAD:
      launch_segreduce<KRK_ADAGRAD, VEC>(level0, tv, keys, pos, vals, cnt, tile, empty_from, keys_out,
                                         vals_out, t, args, ps, stream);
      break;
    case KRK_ADAM:
      launch_segreduce<KRK_ADAM, VEC>(level0, tv, keys, pos, vals, cnt, tile, empty_from, keys_out,
                                      vals_out, t, args, ps, stream);
      break;
    default:
      launch_segreduce<KRK_RMSPROP, VEC>(level0, tv, keys, pos, vals, cnt, tile, empty_from, keys_out,
                                         vals_out, t, args, ps, stream);
      break;
  }
}

static int pick_tile(int64_t cnt) {
  // Large requests: long tiles keep the carry list small. Small ones: short tiles keep the
  // whole GPU busy; extra reduction levels cost only a few microseconds each.
  if (cnt >= (1 << 20)) return 32;
  if (cnt >= (1 << 16)) return 16;
  return 8;
}

// Positions -> rows -> stable sort by row -> tiled segmented reduction fused with the update.
// d_vals holds one gradient row per sort payload (per position, or per bag for pooled pushes).
// The caller holds the table's lock and has made the optimizer's columns exist.
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
  const int tile0 = pick_tile(n);
  const int64_t tiles0 = (n + tile0 - 1) / tile0;
  const size_t n4 = (size_t)n * sizeof(uint32_t);
  size_t sort_bytes = 0;
  KRK_HIP(rocprim::radix_sort_pairs(nullptr, sort_bytes, (uint32_t*)nullptr, (uint32_t*)nullptr,
                                    (uint32_t*)nullptr, (uint32_t*)nullptr, (size_t)n, 0, bits,
                                    t->stream));
  const size_t carry_entries = (size_t)(2 * tiles0);
  KRK_TRY(t->scratch[0].reserve(4 * n4));                       // keys, pos, sorted keys, sorted pos
  KRK_TRY(t->scratch[1].reserve(sort_bytes));
  KRK_TRY(t->scratch[2].reserve(carry_entries * sizeof(uint32_t) * 2));              // carry keys A|B
  KRK_TRY(t->scratch[3].reserve(carry_entries * (size_t)t->dim * sizeof(float)));    // carry vals A
  KRK_TRY(t->scratch[4].reserve((carry_entries / 2 + 16) * (size_t)t->dim * sizeof(float)));  // B
  uint32_t* keys = t->scratch[0].as<uint32_t>();
  uint32_t* pos = keys + n;
  uint32_t* skeys = pos + n;
  uint32_t* spos = skeys + n;

  const TableView tv = t->view();
  hipLaunchKernelGGL(rows_of_ids_kernel, dim3(grid_for(n, kBlock / kBucket)), dim3(kBlock), 0, t->stream,
                     tv, d_ids, n, miss_key, bag_of, payload_is_bag, keys, pos);
  KRK_HIP(hipGetLastError());
  KRK_HIP(rocprim::radix_sort_pairs(t->scratch[1].ptr, sort_bytes, keys, skeys, pos, spos, (size_t)n, 0,
                                    bits, t->stream));

  ApplyArgs args;
  args.lr = lr;
  args.k = make_optim_k(*o);
  int32_t cols[3];
  sparse_optim_columns(t, *o, cols);
  args.c0 = cols[0];
  args.c1 = cols[1];
  args.c2 = cols[2];
  args.meta_off = ((optim_state_mask(*o) >> KRK_ST_STEPS) & 1u) ? t->meta_off : -1;

  // level 0 reads gradients through the sorted positions; later levels read the carry list
  uint32_t* ckeys[2] = {t->scratch[2].as<uint32_t>(), t->scratch[2].as<uint32_t>() + carry_entries};
  float* cvals[2] = {t->scratch[3].as<float>(), t->scratch[4].as<float>()};
  const uint32_t* in_keys = skeys;
  const float* in_vals = d_g;
  int64_t cnt = n;
  int tile = tile0;
  bool level0 = true;
  int which = 0;
  uint32_t empty_from = miss_key;
  for (;;) {
    const int64_t tiles = (cnt + tile - 1) / tile;
    uint32_t* okeys = nullptr;
    float* ovals = nullptr;
    if (tiles > 1) {
      okeys = ckeys[which];
      ovals = cvals[which];
    }
    if (t->vec == 4) {
      dispatch_segreduce<4>(o->type, level0, tv, in_keys, spos, in_vals, cnt, tile, empty_from, okeys,
                            ovals, t, args, ps, t->stream);
    } else {
      dispatch_segreduce<1>(o->type, level0, tv, in_keys, spos, in_vals, cnt, tile, empty_from, okeys,
                            ovals, t, args, ps, t->stream);
    }
    KRK_HIP(hipGetLastError());
    if (tiles <= 1) break;
    in_keys = okeys;
    in_vals = ovals;
    cnt = 2 * tiles;
    level0 = false;
    which ^= 1;
    tile = kCarryTile;
  }
  return KRK_SUCCESS;
}

}  // namespace krk

using namespace krk;

extern "C" {

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

  uint64_t cap = 1024;
  while (cap < (uint64_t)n * 2) cap <<= 1;
  const size_t slots_b = (cap + 1) * sizeof(DSlot);
  const size_t n4 = ((size_t)n * 4 + 255) & ~(size_t)255;
  const size_t n8 = ((size_t)n * 8 + 255) & ~(size_t)255;
  const size_t scan_b = (scan_scratch_bytes(n) + 255) & ~(size_t)255;
  const bool host = !(flags & KRK_DEVICE_PTRS);
  // one allocation: slots | slot_of | flag | rank | scan scratch | total | (staged ids, uids, inv)
  size_t total = slots_b + 3 * n4 + scan_b + 256 + (host ? 3 * n8 : 0);
  // work space is kept between calls (the call blocks, so one buffer under a lock is enough)
  static std::mutex pool_mu;
  static DeviceBuffer pool;
  std::lock_guard<std::mutex> pool_lock(pool_mu);
  KRK_TRY(pool.reserve(total));
  char* base = pool.as<char>();
  char* cur = base;
  DSlot* slots = reinterpret_cast<DSlot*>(cur); cur += slots_b;
  uint32_t* slot_of = reinterpret_cast<uint32_t*>(cur); cur += n4;
  int32_t* flag = reinterpret_cast<int32_t*>(cur); cur += n4;
  int32_t* rank = reinterpret_cast<int32_t*>(cur); cur += n4;
  void* scan_tmp = cur; cur += scan_b;
  int32_t* d_total = reinterpret_cast<int32_t*>(cur); cur += 256;
  const uint64_t* d_ids = ids;
  uint64_t* d_uids = uids;
  long long* d_inv = reinterpret_cast<long long*>(inv);
  if (host) {
    uint64_t* s_ids = reinterpret_cast<uint64_t*>(cur); cur += n8;
    d_uids = reinterpret_cast<uint64_t*>(cur); cur += n8;
    d_inv = reinterpret_cast<long long*>(cur); cur += n8;
    KRK_HIP(hipMemcpy(s_ids, ids, (size_t)n * 8, hipMemcpyHostToDevice));
    d_ids = s_ids;
  }
  hipStream_t s = nullptr;   // the null stream: this call owns no table and blocks anyway
  KRK_HIP(hipMemsetAsync(slots, 0xFF, slots_b, s));
  const dim3 grid(grid_for(n, kBlock)), block(kBlock);
  hipLaunchKernelGGL(dedup_claim_kernel, grid, block, 0, s, slots, cap - 1, d_ids, n, slot_of);
  hipLaunchKernelGGL(dedup_flag_kernel, grid, block, 0, s, slots, slot_of, n, flag);
  KRK_HIP(hipGetLastError());
  KRK_TRY(exclusive_scan_i32(flag, rank, n, d_total, scan_tmp, s));
  hipLaunchKernelGGL(dedup_emit_kernel, grid, block, 0, s, slots, slot_of, rank, d_ids, n, d_uids);
  if (inv) hipLaunchKernelGGL(dedup_inv_kernel, grid, block, 0, s, slots, slot_of, n, d_inv);
  KRK_HIP(hipGetLastError());
  int32_t u = 0;
  KRK_HIP(hipMemcpy(&u, d_total, sizeof(u), hipMemcpyDeviceToHost));
  *n_unique = u;
  if (host) {
    KRK_HIP(hipMemcpy(uids, d_uids, (size_t)u * 8, hipMemcpyDeviceToHost));
    if (inv) KRK_HIP(hipMemcpy(inv, d_inv, (size_t)n * 8, hipMemcpyDeviceToHost));
  }
  KRK_HIP(hipStreamSynchronize(s));
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

  KRK_TRY(push_sorted(t, o, d_ids, n, d_g, lr, nullptr, false, PooledSrc{nullptr, nullptr}));
  return sparse_finish(t, flags);
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
