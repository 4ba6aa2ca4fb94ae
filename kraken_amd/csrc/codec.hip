// Threshold gradient codec ("DCT" = dynamic communication thresholding in the reference):
// DCTEmitter::DenseBag::MaybeToCoo (worker/dct_emitter.cc:16-43) and its decode,
// CooTensorImpl::ToDense (t/coo_tensor_impl.cc:250-260).
//
//   f = grad + e                                   error feedback
//   every life_span steps: tau = k-th largest |f|, k = (int64)(n * (1.0 - eta))
//   emit (idx, f[idx]) for |f| >= tau, idx ascending; e = |f| < tau ? f : 0
//
// tau comes from a three-pass radix select over the bit patterns of |f| (non-negative floats
// order like their bit patterns): 11 + 11 + 10 bits, each pass one LDS histogram per workgroup.
// The emit step is a count pass, a scan of the per-tile counts and a write pass that recomputes
// f, so the output order is the input order.
#include <new>

#include "krk_internal.h"

struct krk_dct : krk::ObjBase {
  int64_t n = 0;
  float* e = nullptr;            // residual
  float* e_next = nullptr;       // written by the emit pass, swapped in on success
  uint32_t* sel = nullptr;       // device: [0] prefix bits, [1] k remaining (lo), [2] tau bits, [3] nnz
  uint32_t* hist = nullptr;      // 2048 bins
  int32_t* tile_counts = nullptr;
  int32_t* tile_offsets = nullptr;
  void* scan_tmp = nullptr;
  uint32_t* host_sel = nullptr;  // pinned
  float tau = 0.0f;
  uint64_t step = 0;
  int64_t tiles = 0;
};

namespace krk {

constexpr int kCodecBlock = 256;
constexpr int kCodecItems = 8;
constexpr int kCodecTile = kCodecBlock * kCodecItems;
constexpr int kBins = 2048;

__device__ __forceinline__ uint32_t abs_bits(float f) { return __float_as_uint(f) & 0x7FFFFFFFu; }

struct Quad {
  float v[4];
};
typedef float vfloat4 __attribute__((ext_vector_type(4)));   // what the non-temporal builtins accept

// four consecutive elements from j on; elements at or behind n read as zero
__device__ __forceinline__ Quad load_quad(const float* __restrict__ p, int64_t j, int64_t n, bool vec) {
  Quad q;
  if (vec && j + 3 < n) {
    const vfloat4 x = __builtin_nontemporal_load(reinterpret_cast<const vfloat4*>(p + j));
    q.v[0] = x[0]; q.v[1] = x[1]; q.v[2] = x[2]; q.v[3] = x[3];
  } else {
#pragma unroll
    for (int c = 0; c < 4; ++c) q.v[c] = j + c < n ? p[j + c] : 0.0f;
  }
  return q;
}

// Histogram of `bits` bits of |g+e| at `shift`, over the elements whose higher bits equal the
// prefix chosen by the earlier passes. sel[0] = prefix (already shifted down to those bits).
__global__ __launch_bounds__(kCodecBlock) void select_hist_kernel(const float* __restrict__ g,
                                                                  const float* __restrict__ e, int64_t n,
                                                                  int shift, int bits, int prefix_shift,
                                                                  const uint32_t* __restrict__ sel,
                                                                  uint32_t* __restrict__ hist) {
  __shared__ uint32_t lh[kBins];
  for (int i = threadIdx.x; i < kBins; i += kCodecBlock) lh[i] = 0;
  __syncthreads();
  const uint32_t prefix = sel[0];
  const uint32_t mask = (1u << bits) - 1u;
  const int64_t stride = (int64_t)gridDim.x * kCodecBlock;
  const bool vec = ((uintptr_t)g & 15) == 0;
  // four consecutive elements a lane and trip, two trips in flight
  const int64_t quads = (n + 3) / 4;
  for (int64_t q = (int64_t)blockIdx.x * kCodecBlock + threadIdx.x; q < quads; q += 2 * stride) {
    Quad a[2], b[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int64_t j = (q + u * stride) * 4;
      a[u] = load_quad(g, j, n, vec);
      b[u] = load_quad(e, j, n, true);
    }
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int64_t j = (q + u * stride) * 4;
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        if (j + c >= n) continue;
        const uint32_t v = abs_bits(a[u].v[c] + b[u].v[c]);
        if (prefix_shift >= 32 || (v >> prefix_shift) == prefix) atomicAdd(&lh[(v >> shift) & mask], 1u);
      }
    }
  }
  __syncthreads();
  for (int i = threadIdx.x; i < kBins; i += kCodecBlock) {
    const uint32_t c = lh[i];
    if (c) atomicAdd(&hist[i], c);
  }
}

// Finds the bin that holds the k-th largest element, counting from the top bin down; extends the
// prefix by that bin and leaves the rank still to be found inside it. One workgroup; clears the
// histogram. Every thread owns kBins / kCodecBlock consecutive bins: the bins above a thread's
// own are summed with a scan over the threads' totals, and the one thread whose bins straddle k
// walks them. Bin 0 takes whatever no higher bin covers (k larger than the histogram's total).
__global__ __launch_bounds__(kCodecBlock) void select_pick_kernel(uint32_t* __restrict__ hist, int bits,
                                                                  uint32_t* __restrict__ sel, int last) {
  constexpr int kPer = kBins / kCodecBlock;
  __shared__ uint32_t lh[kBins];
  __shared__ uint32_t above[kCodecBlock];      // inclusive suffix sums of the threads' totals
  const int nb = 1 << bits;
  const uint32_t k = sel[1];                   // read by all before the barriers, written by one after
  for (int i = threadIdx.x; i < kBins; i += kCodecBlock) {
    lh[i] = i < nb ? hist[i] : 0;
    hist[i] = 0;
  }
  __syncthreads();
  const int t = threadIdx.x;
  uint32_t mine = 0;
#pragma unroll
  for (int j = 0; j < kPer; ++j) mine += lh[t * kPer + j];
  above[t] = mine;
  __syncthreads();
  for (int d = 1; d < kCodecBlock; d <<= 1) {
    const uint32_t add = t + d < kCodecBlock ? above[t + d] : 0u;
    __syncthreads();
    above[t] += add;
    __syncthreads();
  }
  const uint32_t higher = above[t] - mine;     // elements in the bins of the threads above this one
  const bool owner = t == 0 ? higher < k : (higher < k && k <= higher + mine);
  if (owner) {
    uint32_t rem = k - higher;                 // rank inside this thread's bins, from the top
    int b = t * kPer + kPer - 1;
    for (; b > t * kPer; --b) {
      const uint32_t c = lh[b];
      if (c >= rem) break;
      rem -= c;
    }
    // b stopped on the bin, or on the thread's lowest bin: for thread 0 that is bin 0, the
    // catch-all; for the others the rank is known to lie inside it
    const uint32_t prefix = (sel[0] << bits) | (uint32_t)b;
    sel[0] = prefix;
    sel[1] = rem;
    if (last) sel[2] = prefix;   // the full bit pattern of tau
  }
}

__global__ void select_begin_kernel(uint32_t* sel, uint32_t k) {
  sel[0] = 0;
  sel[1] = k;
}

// A tile is kCodecTile consecutive elements; inside it each wavefront owns 512 consecutive
// elements and reads them as two rows of 256, a lane four consecutive floats of each (one
// 16-byte access), so every load and store is fully coalesced and the output order is still the
// input order: within a row an element's rank is the number of kept elements in lower lanes (four
// ballots, one per component, and population counts) plus those of the lane's own lower
// components; rows and waves are offset by running totals. A workgroup walks several tiles: a
// few hundred workgroups with many wide accesses in flight stream faster on this memory system
// than one workgroup per tile (6.5-7 TB/s against 4.5 TB/s for plain reads).
constexpr int kCodecRows = kCodecItems / 4;      // rows of 256 elements per wavefront and tile
constexpr int kCodecGrid = 1024;                 // workgroups of the two emit passes

// Per tile: how many elements have |g+e| >= tau. vec: g is 16-byte aligned (e always is).
__global__ __launch_bounds__(kCodecBlock) void emit_count_kernel(const float* __restrict__ g,
                                                                 const float* __restrict__ e, int64_t n,
                                                                 int64_t tiles, bool vec,
                                                                 const uint32_t* __restrict__ sel,
                                                                 int32_t* __restrict__ tile_counts) {
  __shared__ int wave_sum[kCodecBlock / 64];
  const uint32_t tau_bits = sel[2];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  for (int64_t tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
    const int64_t base = tile * kCodecTile + (int64_t)wave * (64 * kCodecItems) + lane * 4;
    Quad a[kCodecRows], b[kCodecRows];
#pragma unroll
    for (int r = 0; r < kCodecRows; ++r) {
      a[r] = load_quad(g, base + r * 256, n, vec);
      b[r] = load_quad(e, base + r * 256, n, true);
    }
    int c = 0;
#pragma unroll
    for (int r = 0; r < kCodecRows; ++r) {
#pragma unroll
      for (int k = 0; k < 4; ++k)
        c += (base + r * 256 + k < n && abs_bits(a[r].v[k] + b[r].v[k]) >= tau_bits) ? 1 : 0;
    }
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) c += __shfl_down(c, d, 64);
    if (lane == 0) wave_sum[wave] = c;
    __syncthreads();
    if (threadIdx.x == 0) {
      int s = 0;
#pragma unroll
      for (int w = 0; w < kCodecBlock / 64; ++w) s += wave_sum[w];
      tile_counts[tile] = s;
    }
    __syncthreads();                               // the next tile reuses wave_sum
  }
}

// Writes the kept (index, value) pairs in input order and the new residual. A tile's pairs are
// first gathered in LDS in output order and then written out by consecutive lanes, so that the
// index and value arrays are written in whole lines (a lane writing its own few kept elements
// leaves partly written lines behind).
__global__ __launch_bounds__(kCodecBlock) void emit_write_kernel(
    const float* __restrict__ g, const float* __restrict__ e, int64_t n, int64_t tiles, bool vec,
    const uint32_t* __restrict__ sel, const int32_t* __restrict__ tile_offsets,
    const int32_t* __restrict__ tile_counts, long long* __restrict__ idx, float* __restrict__ val,
    float* __restrict__ e_next) {
  __shared__ int wave_sum[kCodecBlock / 64];
  __shared__ uint16_t kept_at[kCodecTile];         // element's place inside the tile
  __shared__ float kept_val[kCodecTile];
  const uint32_t tau_bits = sel[2];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const unsigned long long below = (1ull << lane) - 1ull;
  for (int64_t tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
    const int local = wave * (64 * kCodecItems) + lane * 4;
    const int64_t base = tile * kCodecTile + local;
    Quad f[kCodecRows];
    unsigned long long masks[kCodecRows][4];
    int wave_total = 0;
    {
      Quad a[kCodecRows], b[kCodecRows];
#pragma unroll
      for (int r = 0; r < kCodecRows; ++r) {
        a[r] = load_quad(g, base + r * 256, n, vec);
        b[r] = load_quad(e, base + r * 256, n, true);
      }
#pragma unroll
      for (int r = 0; r < kCodecRows; ++r) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          f[r].v[k] = a[r].v[k] + b[r].v[k];
          masks[r][k] = __ballot(base + r * 256 + k < n && abs_bits(f[r].v[k]) >= tau_bits);
          wave_total += __popcll(masks[r][k]);
        }
      }
    }
    if (lane == 0) wave_sum[wave] = wave_total;
    __syncthreads();
    int off = 0;                                   // inside the tile's stretch of the output
#pragma unroll
    for (int w = 0; w < kCodecBlock / 64; ++w)
      if (w < wave) off += wave_sum[w];
#pragma unroll
    for (int r = 0; r < kCodecRows; ++r) {
      const int64_t j = base + r * 256;
      // kept elements of lower lanes, all four components of each
      int at = off;
      int row_total = 0;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        at += __popcll(masks[r][k] & below);
        row_total += __popcll(masks[r][k]);
      }
      float rest[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const bool keep = (masks[r][k] >> lane) & 1ull;
        if (keep) {
          kept_at[at] = (uint16_t)(local + r * 256 + k);
          kept_val[at] = f[r].v[k];
          ++at;
        }
        rest[k] = keep ? 0.0f : f[r].v[k];         // t/math.cc:1098-1123 : |x| < th keeps x
      }
      if (j + 3 < n) {
        const vfloat4 out = {rest[0], rest[1], rest[2], rest[3]};
        __builtin_nontemporal_store(out, reinterpret_cast<vfloat4*>(e_next + j));
      } else {
#pragma unroll
        for (int k = 0; k < 4; ++k)
          if (j + k < n) e_next[j + k] = rest[k];
      }
      off += row_total;
    }
    __syncthreads();
    const int count = tile_counts[tile];
    const int64_t out0 = tile_offsets[tile];
    const int64_t tile_base = tile * kCodecTile;
    for (int i = threadIdx.x; i < count; i += kCodecBlock) {
      __builtin_nontemporal_store((long long)(tile_base + kept_at[i]), idx + out0 + i);
      __builtin_nontemporal_store(kept_val[i], val + out0 + i);
    }
    __syncthreads();                               // the next tile reuses the LDS arrays
  }
}


// ---- densify in one pass over the output ------------------------------------------------------
constexpr int kTileElems = 4096;                 // floats of one output tile: 16 KB of LDS
constexpr int64_t kTiledFrom = 1 << 22;          // smaller tensors: zero + scatter, two launches are quicker
constexpr uint32_t kNoStart = 0xFFFFFFFFu;

__global__ __launch_bounds__(kCodecBlock) void coo_tiles_init_kernel(uint32_t* __restrict__ starts, int64_t tiles,
                                                                     uint32_t* __restrict__ unordered) {
  const int64_t i = (int64_t)blockIdx.x * kCodecBlock + threadIdx.x;
  if (i < tiles) starts[i] = kNoStart;
  if (i == 0) *unordered = 0u;
}

// starts[T] / ends[T] = the entries whose index lies in tile T (ends is only read where starts is
// set); *unordered is raised when the indices do not ascend strictly or leave [0, n).
__global__ __launch_bounds__(kCodecBlock) void coo_tiles_bounds_kernel(const long long* __restrict__ idx,
                                                                       int64_t nnz, int64_t n,
                                                                       uint32_t* __restrict__ starts,
                                                                       uint32_t* __restrict__ ends,
                                                                       uint32_t* __restrict__ unordered) {
  const int64_t step = (int64_t)gridDim.x * kCodecBlock;
  for (int64_t j = (int64_t)blockIdx.x * kCodecBlock + threadIdx.x; j < nnz; j += step) {
    const long long cur = __builtin_nontemporal_load(idx + j);
    const long long prev = j ? idx[j - 1] : -1;
    if (cur <= prev || cur >= n) {
      atomicOr(unordered, 1u);
    } else {
      if (prev < 0 || cur / kTileElems != prev / kTileElems) {
        starts[cur / kTileElems] = (uint32_t)j;
        if (prev >= 0) ends[prev / kTileElems] = (uint32_t)j;
      }
      if (j == nnz - 1) ends[cur / kTileElems] = (uint32_t)nnz;
    }
  }
}

// One workgroup per output tile: the tile is put together in LDS (zeros, then the tile's entries,
// whose range is known, so their loads do not wait for one another) and leaves in whole lines,
// past the caches.
__global__ __launch_bounds__(kCodecBlock) void coo_tiles_write_kernel(const long long* __restrict__ idx,
                                                                      const float* __restrict__ val, int64_t nnz,
                                                                      float* __restrict__ dense, int64_t n,
                                                                      const uint32_t* __restrict__ starts,
                                                                      const uint32_t* __restrict__ ends,
                                                                      const uint32_t* __restrict__ unordered) {
  if (*unordered) return;                        // the scatter launches that follow do the work
  __shared__ __align__(16) float tile[kTileElems];
  const int64_t base = (int64_t)blockIdx.x * kTileElems;
  const uint32_t start = starts[blockIdx.x];
  const uint32_t end = start != kNoStart ? ends[blockIdx.x] : 0u;
  for (int i = threadIdx.x; i < kTileElems / 4; i += kCodecBlock)
    reinterpret_cast<float4*>(tile)[i] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
  __syncthreads();
  if (start != kNoStart) {
    for (int64_t j0 = (int64_t)start + threadIdx.x; j0 < (int64_t)end; j0 += 4 * kCodecBlock) {
      long long at[4];
      float v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int64_t j = j0 + u * kCodecBlock;
        if (j < (int64_t)end) {
          at[u] = __builtin_nontemporal_load(idx + j);
          v[u] = __builtin_nontemporal_load(val + j);
        }
      }
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (j0 + u * kCodecBlock < (int64_t)end) tile[at[u] - base] = v[u];
    }
  }
  __syncthreads();
  const int64_t left = n - base;
  const int cnt = left < kTileElems ? (int)left : kTileElems;
  if (cnt == kTileElems && (((uintptr_t)dense) & 15) == 0) {
    typedef float tile4 __attribute__((ext_vector_type(4)));
    for (int i = threadIdx.x; i < kTileElems / 4; i += kCodecBlock)
      __builtin_nontemporal_store(reinterpret_cast<const tile4*>(tile)[i], reinterpret_cast<tile4*>(dense + base) + i);
  } else {
    for (int i = threadIdx.x; i < cnt; i += kCodecBlock) dense[base + i] = tile[i];
  }
}

__global__ __launch_bounds__(kCodecBlock) void coo_zero_if_kernel(float* __restrict__ dense, int64_t n,
                                                                  const uint32_t* __restrict__ unordered) {
  if (!*unordered) return;
  const int64_t step = (int64_t)gridDim.x * kCodecBlock;
  for (int64_t i = (int64_t)blockIdx.x * kCodecBlock + threadIdx.x; i < n; i += step) dense[i] = 0.0f;
}

// dense[idx[j]] += val[j]; repeated indices add up (t/math.cc:1043). unordered null: always.
__global__ __launch_bounds__(kCodecBlock) void coo_add_kernel(const long long* __restrict__ idx,
                                                              const float* __restrict__ val, int64_t nnz,
                                                              float* __restrict__ dense, int64_t n,
                                                              const uint32_t* __restrict__ unordered,
                                                              uint32_t* __restrict__ err) {
  if (unordered && !*unordered) return;
  const int64_t step = (int64_t)gridDim.x * kCodecBlock;
  for (int64_t j = (int64_t)blockIdx.x * kCodecBlock + threadIdx.x; j < nnz; j += step) {
    const long long i = idx[j];
    if (i < 0 || i >= n) {
      if (err) atomicOr(err, 1u);
      continue;
    }
    unsafeAtomicAdd(&dense[i], val[j]);   // hardware fp32 add, no CAS loop
  }
}

static unsigned stream_grid(int64_t n) {
  int64_t blocks = (n + kCodecBlock - 1) / kCodecBlock;
  if (blocks > 256 * 8) blocks = 256 * 8;
  if (blocks < 1) blocks = 1;
  return (unsigned)blocks;
}

size_t coo_densify_work_bytes(int64_t n) {
  return (2 * (size_t)((n + kTileElems - 1) / kTileElems) + 4) * sizeof(uint32_t);
}

int32_t coo_densify(const long long* d_idx, const float* d_val, int64_t nnz, float* d_dense, int64_t n,
                    void* work, uint32_t* err, hipStream_t stream) {
  if (n <= 0) return KRK_SUCCESS;
  const dim3 block(kCodecBlock);
  const unsigned per_entry = (unsigned)((nnz + kCodecBlock - 1) / kCodecBlock);
  if (n < kTiledFrom || nnz >= ((int64_t)1 << 31) || !work) {
    KRK_HIP(hipMemsetAsync(d_dense, 0, (size_t)n * sizeof(float), stream));   // t/math.cc:1066 dense.Zero()
    if (nnz)
      hipLaunchKernelGGL(coo_add_kernel, dim3(per_entry), block, 0, stream, d_idx, d_val, nnz, d_dense, n,
                         (const uint32_t*)nullptr, err);
    KRK_HIP(hipGetLastError());
    return KRK_SUCCESS;
  }
  const int64_t tiles = (n + kTileElems - 1) / kTileElems;
  uint32_t* starts = reinterpret_cast<uint32_t*>(work);
  uint32_t* ends = starts + tiles;
  uint32_t* unordered = ends + tiles;
  hipLaunchKernelGGL(coo_tiles_init_kernel, dim3((unsigned)((tiles + kCodecBlock - 1) / kCodecBlock)), block, 0,
                     stream, starts, tiles, unordered);
  if (nnz)
    hipLaunchKernelGGL(coo_tiles_bounds_kernel, dim3(stream_grid(nnz)), block, 0, stream, d_idx, nnz, n, starts,
                       ends, unordered);
  hipLaunchKernelGGL(coo_tiles_write_kernel, dim3((unsigned)tiles), block, 0, stream, d_idx, d_val, nnz, d_dense,
                     n, starts, ends, unordered);
  if (nnz) {
    hipLaunchKernelGGL(coo_zero_if_kernel, dim3(stream_grid(n)), block, 0, stream, d_dense, n, unordered);
    // a few workgroups that stride over the entries: when the tiles did the work they only look at
    // the flag and leave
    hipLaunchKernelGGL(coo_add_kernel, dim3(stream_grid(nnz)), block, 0, stream, d_idx, d_val, nnz, d_dense, n,
                       (const uint32_t*)unordered, err);
  }
  KRK_HIP(hipGetLastError());
  return KRK_SUCCESS;
}

}  // namespace krk

using namespace krk;

static std::mutex g_densify_mu;          // krk_coo_to_dense owns no object: one shared work buffer
static DeviceBuffer g_densify_work;

extern "C" {

int32_t krk_dct_create(int64_t n, krk_dct** out) {
  if (!out || n < 0 || n >= (int64_t)0x7FFFFFFF) return KRK_E_ARGUMENT;
  KRK_TRY(ensure_runtime());
  krk_dct* s = new (std::nothrow) krk_dct();
  if (!s) return KRK_E_DEVICE;
  s->n = n;
  s->tiles = (n + kCodecTile - 1) / kCodecTile;
  if (s->tiles < 1) s->tiles = 1;
  int32_t rc = s->open_stream();
  if (rc == KRK_SUCCESS) {
    const size_t nb = (size_t)(n ? n : 1) * sizeof(float);
    hipError_t e = hipMalloc((void**)&s->e, nb);
    if (e == hipSuccess) e = hipMalloc((void**)&s->e_next, nb);
    if (e == hipSuccess) e = hipMalloc((void**)&s->sel, 64);
    if (e == hipSuccess) e = hipMalloc((void**)&s->hist, kBins * sizeof(uint32_t));
    if (e == hipSuccess) e = hipMalloc((void**)&s->tile_counts, (size_t)s->tiles * sizeof(int32_t));
    if (e == hipSuccess) e = hipMalloc((void**)&s->tile_offsets, (size_t)s->tiles * sizeof(int32_t));
    if (e == hipSuccess) e = hipMalloc(&s->scan_tmp, scan_scratch_bytes(s->tiles));
    if (e == hipSuccess) e = hipHostMalloc((void**)&s->host_sel, 64, hipHostMallocDefault);
    if (e == hipSuccess) e = hipMemsetAsync(s->e, 0, nb, s->stream);   // dct_emitter.cc:54 : val.Clone().Zero()
    if (e == hipSuccess) e = hipMemsetAsync(s->sel, 0, 64, s->stream);
    if (e == hipSuccess) e = hipMemsetAsync(s->hist, 0, kBins * sizeof(uint32_t), s->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(s->stream);
    if (e != hipSuccess) rc = hip_fail(e, "krk_dct_create", __FILE__, __LINE__);
  }
  if (rc != KRK_SUCCESS) {
    krk_dct_destroy(s);
    return rc;
  }
  *out = s;
  return KRK_SUCCESS;
}

int32_t krk_dct_destroy(krk_dct* s) {
  if (!s) return KRK_SUCCESS;
  if (s->stream) (void)hipStreamSynchronize(s->stream);
  if (s->e) (void)hipFree(s->e);
  if (s->e_next) (void)hipFree(s->e_next);
  if (s->sel) (void)hipFree(s->sel);
  if (s->hist) (void)hipFree(s->hist);
  if (s->tile_counts) (void)hipFree(s->tile_counts);
  if (s->tile_offsets) (void)hipFree(s->tile_offsets);
  if (s->scan_tmp) (void)hipFree(s->scan_tmp);
  if (s->host_sel) (void)hipHostFree(s->host_sel);
  s->close_stream();
  delete s;
  return KRK_SUCCESS;
}

int32_t krk_dct_compress(krk_dct* s, const float* grad, uint64_t life_span, float eta, int64_t* idx,
                         float* val, int64_t capacity, int64_t* nnz, uint32_t flags) {
  if (!s || !nnz) return KRK_E_ARGUMENT;
  KRK_TRY(ensure_runtime());
  KRK_TRY(check_flags(flags));
  if (flags & KRK_ASYNC) return KRK_E_ARGUMENT;   // the count comes back by value
  if (life_span == 0 || capacity < 0) return KRK_E_ARGUMENT;
  std::lock_guard<std::mutex> lk(s->mu);
  const int64_t n = s->n;
  if (n < 256) {   // worker/dct_emitter.cc:18-20
    *nnz = -1;
    return KRK_SUCCESS;
  }
  if (!grad || (capacity > 0 && (!idx || !val))) return KRK_E_ARGUMENT;
  const float* d_g;
  KRK_TRY(s->input(grad, (size_t)n, flags, 0, &d_g));
  const bool reselect = s->step % life_span == 0;   // :25
  if (reselect) {
    const int64_t k = (int64_t)((double)n * (1.0 - (double)eta));   // :27
    if (k < 1 || k > n) {
      set_error("eta %g keeps %lld of %lld elements; TopK needs 1..n", (double)eta, (long long)k,
                (long long)n);
      return KRK_E_ARGUMENT;   // t/math.cc:628-633 rejects k == 0
    }
    hipLaunchKernelGGL(select_begin_kernel, dim3(1), dim3(1), 0, s->stream, s->sel, (uint32_t)k);
    const int pass_bits[3] = {11, 11, 10};
    int shift = 32;
    for (int p = 0; p < 3; ++p) {
      const int prefix_shift = shift;        // bits above this pass are already fixed
      shift -= pass_bits[p];
      hipLaunchKernelGGL(select_hist_kernel, dim3(stream_grid(n)), dim3(kCodecBlock), 0, s->stream, d_g,
                         s->e, n, shift, pass_bits[p], prefix_shift, s->sel, s->hist);
      hipLaunchKernelGGL(select_pick_kernel, dim3(1), dim3(kCodecBlock), 0, s->stream, s->hist,
                         pass_bits[p], s->sel, p == 2 ? 1 : 0);
    }
    KRK_HIP(hipGetLastError());
  }
  const bool vec = ((uintptr_t)d_g & 15) == 0;
  const unsigned emit_grid = (unsigned)(s->tiles < kCodecGrid ? s->tiles : kCodecGrid);
  hipLaunchKernelGGL(emit_count_kernel, dim3(emit_grid), dim3(kCodecBlock), 0, s->stream, d_g, s->e, n,
                     s->tiles, vec, s->sel, s->tile_counts);
  KRK_HIP(hipGetLastError());
  KRK_TRY(exclusive_scan_i32(s->tile_counts, s->tile_offsets, s->tiles,
                             reinterpret_cast<int32_t*>(s->sel + 3), s->scan_tmp, s->stream));
  const unsigned emit_blocks = emit_grid;
  // Room for every element and device buffers: nothing can overflow and nothing is staged, so the
  // write pass follows at once and the count is read back once, at the end.
  const bool sure = (flags & KRK_DEVICE_PTRS) && capacity >= n;
  if (sure) {
    hipLaunchKernelGGL(emit_write_kernel, dim3(emit_blocks), dim3(kCodecBlock), 0, s->stream, d_g, s->e, n,
                       s->tiles, vec, s->sel, s->tile_offsets, s->tile_counts, reinterpret_cast<long long*>(idx),
                       val, s->e_next);
    KRK_HIP(hipGetLastError());
  }
  KRK_HIP(hipMemcpyAsync(s->host_sel, s->sel, 16, hipMemcpyDeviceToHost, s->stream));
  KRK_HIP(hipStreamSynchronize(s->stream));
  const int64_t count = (int64_t)s->host_sel[3];
  const float new_tau = __builtin_bit_cast(float, s->host_sel[2]);
  *nnz = count;
  if (!sure) {
    if (count > capacity) {
      // nothing was committed: restore the threshold the next call will see
      if (reselect) {
        const uint32_t old_bits = __builtin_bit_cast(uint32_t, s->tau);
        KRK_HIP(hipMemcpyAsync(s->sel + 2, &old_bits, 4, hipMemcpyHostToDevice, s->stream));
        KRK_HIP(hipStreamSynchronize(s->stream));
      }
      set_error("compress needs room for %lld entries, caller offered %lld", (long long)count,
                (long long)capacity);
      return KRK_E_CAPACITY;
    }
    long long* d_idx;
    float* d_val;
    KRK_TRY(s->output(reinterpret_cast<long long*>(idx), (size_t)count, flags, 1, &d_idx));
    KRK_TRY(s->output(val, (size_t)count, flags, 2, &d_val));
    hipLaunchKernelGGL(emit_write_kernel, dim3(emit_blocks), dim3(kCodecBlock), 0, s->stream, d_g, s->e, n,
                       s->tiles, vec, s->sel, s->tile_offsets, s->tile_counts, d_idx, d_val, s->e_next);
    KRK_HIP(hipGetLastError());
    KRK_TRY(s->output_back(reinterpret_cast<long long*>(idx), (size_t)count, flags, 1));
    KRK_TRY(s->output_back(val, (size_t)count, flags, 2));
    KRK_HIP(hipStreamSynchronize(s->stream));
  }
  float* tmp = s->e;
  s->e = s->e_next;
  s->e_next = tmp;
  s->tau = new_tau;
  s->step += 1;   // :40
  return KRK_SUCCESS;
}

int32_t krk_dct_tau(krk_dct* s, float* tau) {
  if (!s || !tau) return KRK_E_ARGUMENT;
  std::lock_guard<std::mutex> lk(s->mu);
  *tau = s->tau;
  return KRK_SUCCESS;
}

int32_t krk_dct_step(krk_dct* s, uint64_t* step) {
  if (!s || !step) return KRK_E_ARGUMENT;
  std::lock_guard<std::mutex> lk(s->mu);
  *step = s->step;
  return KRK_SUCCESS;
}

int32_t krk_dct_residual(krk_dct* s, float* out, uint32_t flags) {
  if (!s || (s->n > 0 && !out)) return KRK_E_ARGUMENT;
  KRK_TRY(ensure_runtime());
  KRK_TRY(check_flags(flags));
  std::lock_guard<std::mutex> lk(s->mu);
  if (s->n)
    KRK_HIP(hipMemcpyAsync(out, s->e, (size_t)s->n * sizeof(float),
                           (flags & KRK_DEVICE_PTRS) ? hipMemcpyDeviceToDevice : hipMemcpyDeviceToHost,
                           s->stream));
  if (!(flags & KRK_ASYNC)) KRK_HIP(hipStreamSynchronize(s->stream));
  return KRK_SUCCESS;
}

int32_t krk_coo_to_dense(const int64_t* idx, const float* val, int64_t nnz, float* dense, int64_t n,
                         uint32_t flags) {
  KRK_TRY(ensure_runtime());
  KRK_TRY(check_flags(flags));
  if (n < 0 || nnz < 0 || (n > 0 && !dense) || (nnz > 0 && (!idx || !val))) return KRK_E_ARGUMENT;
  if (n == 0) return KRK_SUCCESS;
  hipStream_t st = nullptr;   // owns no object: runs on the null stream
  const bool host = !(flags & KRK_DEVICE_PTRS);
  float* d_dense = dense;
  const long long* d_idx = reinterpret_cast<const long long*>(idx);
  const float* d_val = val;
  char* tmp = nullptr;
  if (host) {
    const size_t nb = ((size_t)n * 4 + 255) & ~(size_t)255;
    const size_t ib = ((size_t)nnz * 8 + 255) & ~(size_t)255;
    KRK_HIP(hipMalloc((void**)&tmp, nb + ib + (size_t)nnz * 4 + 256));
    d_dense = reinterpret_cast<float*>(tmp);
    long long* si = reinterpret_cast<long long*>(tmp + nb);
    float* sv = reinterpret_cast<float*>(tmp + nb + ib);
    if (nnz) {
      hipError_t e = hipMemcpy(si, idx, (size_t)nnz * 8, hipMemcpyHostToDevice);
      if (e == hipSuccess) e = hipMemcpy(sv, val, (size_t)nnz * 4, hipMemcpyHostToDevice);
      if (e != hipSuccess) {
        (void)hipFree(tmp);
        return hip_fail(e, "krk_coo_to_dense staging", __FILE__, __LINE__);
      }
    }
    d_idx = si;
    d_val = sv;
  }
  hipError_t e = hipSuccess;
  {
    std::lock_guard<std::mutex> lk(g_densify_mu);
    int32_t rc = g_densify_work.reserve(coo_densify_work_bytes(n));
    if (rc == KRK_SUCCESS) rc = coo_densify(d_idx, d_val, nnz, d_dense, n, g_densify_work.ptr, nullptr, st);
    // the shared work buffer is free for the next caller once this call's launches are done
    if (rc == KRK_SUCCESS && n >= kTiledFrom) e = hipStreamSynchronize(st);
    if (rc != KRK_SUCCESS) {
      if (tmp) (void)hipFree(tmp);
      return rc;
    }
  }
  if (e == hipSuccess && host) e = hipMemcpy(dense, d_dense, (size_t)n * sizeof(float), hipMemcpyDeviceToHost);
  if (e == hipSuccess && !(flags & KRK_ASYNC)) e = hipStreamSynchronize(st);
  if (tmp) (void)hipFree(tmp);
  if (e != hipSuccess) return hip_fail(e, "krk_coo_to_dense", __FILE__, __LINE__);
  return KRK_SUCCESS;
}

}  // extern "C"
