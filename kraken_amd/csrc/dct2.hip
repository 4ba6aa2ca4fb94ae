// Blockwise orthonormal DCT-II / DCT-III over blocks of 256 floats on the fp32 matrix cores.
//
// There is NO reference counterpart: the reference's "DCT" emitter is a threshold codec
// (worker/dct_emitter.cc:16-43) and contains no cosine transform. This file exists because the
// build's target names a blockwise DCT; it is pinned by the closed form
//     y[k] = s_k * sum_j x[j] * cos(pi * (2j + 1) * k / (2B)),  s_0 = sqrt(1/B), s_k = sqrt(2/B)
// and by the round trip inverse(forward(x)) == x. Keeping only the first `keep` coefficients of
// each block (keep = B * (1 - eta) = 64 for the emitter's default eta = 0.75) is the compression.
//
// Shape of the work: Y[M, N] = X[M, K] * Basis[K, N] with M = n / 256 blocks. Forward: K = 256,
// N = keep. Inverse: K = keep, N = 256. A workgroup keeps a 64- or 128-column basis tile resident
// in LDS and walks over row tiles of 256 blocks; each of its eight wavefronts owns 32 rows, holds
// their X values in registers and feeds v_mfma_f32_32x32x2_f32.
#include <cmath>
#include <mutex>

#include "krk_internal.h"

namespace krk {

constexpr int kDctB = 256;      // block length
constexpr int kThreads = 512;   // eight wavefronts, two per SIMD
constexpr int kTileM = 256;     // rows (blocks) per output tile: 32 per wavefront
constexpr int kSliceK = 32;     // reduction slice held in registers per step

typedef float v16f __attribute__((ext_vector_type(16)));

// fwd[j * B + k] = inv[k * B + j] = s_k cos(pi (2j+1) k / (2B)), evaluated in double.
__global__ void dct2_basis_kernel(float* __restrict__ fwd, float* __restrict__ inv) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= kDctB * kDctB) return;
  const int k = t / kDctB;
  const int j = t - k * kDctB;
  const double s = k == 0 ? sqrt(1.0 / kDctB) : sqrt(2.0 / kDctB);
  const double v = s * cos(3.14159265358979323846 * (2.0 * j + 1.0) * k / (2.0 * kDctB));
  fwd[j * kDctB + k] = (float)v;
  inv[k * kDctB + j] = (float)v;
}

// Y[M, N] = X[M, K] * Bm[K, N]; ldx / ldb / ldy are row strides in floats. K is a multiple of 64,
// N a multiple of 32 * NT. grid.x workgroups share the row tiles, grid.y = N / (32 * NT).
//
// The basis tile sits in LDS for the whole launch and is only read. It is laid out
// [K + kPadRows][32][NT]: the NT values a lane needs for one step (columns r, r + 32, ...) are one
// vector read, at an offset from the slice's first row that is known at compile time. X never
// passes through LDS: the matrix instruction takes, per lane (r = lane % 32, h = lane / 32),
// one value A[r][k_h] for its two reduction indices k_0, k_1, and the order in which the
// reduction indices are consumed is free as long as the basis rows follow it. So lane (r, h)
// loads the 16 consecutive floats X[row r][32 s + 16 h ...] of slice s as four float4 and
// step j multiplies them against basis rows 32 s + 16 h + j. Wavefronts never wait on each
// other inside the loop; the next slice's loads are in flight while this one multiplies.
//
// (This kernel serves the 64-column tiles, keep = 64 and 192.)
// A tile's results are not stored when the tile is done: the two wavefronts that share a SIMD
// run in step, so both would store while the matrix pipe idles (10 % of the kernel's time).
// They are kept in registers and leave between the multiplies of the next tile's first two
// slices, two (NT = 4) or one (NT = 2) store a step; the last tile's follow the loop.
constexpr int kPadRows = 17;   // the step after a tile's last one still reads "its" basis rows

template <int NT>
struct BasisVec;
template <>
struct BasisVec<4> {
  typedef float type __attribute__((ext_vector_type(4)));
};
template <>
struct BasisVec<2> {
  typedef float type __attribute__((ext_vector_type(2)));
};

template <int V>
struct IntTag {
  static constexpr int value = V;
};

template <int NT>
__global__ __launch_bounds__(kThreads) void dct2_gemm_kernel(const float* __restrict__ X, int64_t ldx,
                                                             const float* __restrict__ Bm, int ldb,
                                                             float* __restrict__ Y, int64_t ldy,
                                                             int64_t M, int K) {
  typedef typename BasisVec<NT>::type bvec;
  constexpr int kTileN = 32 * NT;
  extern __shared__ float Bs[];                     // [K + kPadRows][32][NT]
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int r = lane & 31;
  const int h = lane >> 5;
  const int n0 = blockIdx.y * kTileN;

  for (int i = tid; i < K * (kTileN / 4); i += kThreads) {
    const int br = i / (kTileN / 4);
    const int c4 = i - br * (kTileN / 4);
    const float4 v = *reinterpret_cast<const float4*>(Bm + (size_t)br * ldb + n0 + c4 * 4);
    const float e[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int c = c4 * 4 + u;                     // column c of the tile is (r, t) = (c % 32, c / 32)
      Bs[br * kTileN + (c & 31) * NT + (c >> 5)] = e[u];
    }
  }
  __syncthreads();

  const int64_t tiles = (M + kTileM - 1) / kTileM;
  const int slices = K / kSliceK;                   // at least two
  // Rows past the end are clamped, not masked: row r of X only reaches row r of Y, and those
  // rows are never stored, so the loads carry no branch.
  auto row_ptr = [&](int64_t tile) {
    int64_t row = tile * kTileM + wave * 32 + r;
    if (row >= M) row = M - 1;
    return X + row * ldx + 16 * h;
  };
  const float* bs = Bs + (size_t)(16 * h) * kTileN + r * NT;
  const float* xrow = row_ptr(blockIdx.x);
  // X runs two slices ahead of the multiplies.
  float4 cur[4], nx1[4], nx2[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    cur[q] = reinterpret_cast<const float4*>(xrow)[q];
    nx1[q] = reinterpret_cast<const float4*>(xrow + kSliceK)[q];
  }
  v16f acc[NT], prev[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) prev[t] = v16f{0};
  int64_t prev_base = M;                            // first row of the tile prev holds: none yet
  bvec bcur, bnxt;

  // accumulator element i of lane l is C[(i / 4) * 8 + (l / 32) * 4 + i % 4][l % 32]
  auto store_prev = [&](int i, int t) {
    const int64_t orow = prev_base + (i >> 2) * 8 + h * 4 + (i & 3);
    if (orow < M) Y[orow * ldy + n0 + r + 32 * t] = prev[t][i];
  };

  // One reduction slice: 16 steps of NT multiplies. STORE 0 / 1: the first / second half of the
  // previous tile's results leaves between the multiplies; -1: nothing to store.
  auto slice = [&](auto store_tag, int s, const float* xnext) {
    constexpr int STORE = decltype(store_tag)::value;
    // slice s + 2 of this tile, or one of the first two slices of the next tile
    const float* ahead = s + 2 < slices ? xrow + (s + 2) * kSliceK : xnext + (s + 2 - slices) * kSliceK;
#pragma unroll
    for (int q = 0; q < 4; ++q) nx2[q] = reinterpret_cast<const float4*>(ahead)[q];
    __builtin_amdgcn_sched_barrier(0);              // keep the requests ahead of the multiplies
    const float* brow = bs + (size_t)s * kSliceK * kTileN;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const float a4[4] = {cur[q].x, cur[q].y, cur[q].z, cur[q].w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int j = q * 4 + e;
        // basis values of the following step are requested before this step multiplies: row j + 1
        // of this slice, or row 0 of the next one (past the last slice: padding, never used)
        bnxt = *reinterpret_cast<const bvec*>(brow + (j < 15 ? (j + 1) * kTileN : kSliceK * kTileN));
        if constexpr (STORE >= 0) {
          constexpr int kPerStep = NT / 2;
#pragma unroll
          for (int u = 0; u < kPerStep; ++u) {
            const int idx = (STORE * 16 + j) * kPerStep + u;
            store_prev(idx / NT, idx % NT);
          }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < NT; ++t)
          acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(a4[e], bcur[t], acc[t], 0, 0, 0);
        bcur = bnxt;
      }
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      cur[q] = nx1[q];
      nx1[q] = nx2[q];
    }
  };

  for (int64_t tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
    // the tile after this one (or this one again at the end: its values are then unused)
    const float* xnext = row_ptr(tile + gridDim.x < tiles ? tile + gridDim.x : tile);
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[t] = v16f{0};
    bcur = *reinterpret_cast<const bvec*>(bs);
    slice(IntTag<0>{}, 0, xnext);
    slice(IntTag<1>{}, 1, xnext);
    for (int s = 2; s < slices; ++s) slice(IntTag<-1>{}, s, xnext);
#pragma unroll
    for (int t = 0; t < NT; ++t) prev[t] = acc[t];
    prev_base = tile * kTileM + wave * 32;
    xrow = xnext;
  }
#pragma unroll
  for (int i = 0; i < 16; ++i) {
#pragma unroll
    for (int t = 0; t < NT; ++t) store_prev(i, t);
  }
}

// The 128-column tiles run with sixteen wavefronts a workgroup (four per SIMD instead of two): a
// wavefront keeps 128 registers, so a tile's results are stored as soon as the tile is done
// (no copy of them survives into the next tile) and X runs one slice ahead, not two. What the
// wavefronts of a SIMD lose while one of them stores, the other three fill in. Against the
// eight-wavefront kernel above at the same tile width: keep 128 forward 160 -> 152 us, inverse
// 175 -> 160 us; keep 256 is the same 302 us either way (113 TFLOP/s: with four wavefronts a SIMD
// the matrix pipe is not waiting for anybody any more, and the rate still moves with the operand
// values, which is what a clock held down by power looks like).
constexpr int kThreads16 = 1024;
constexpr int kTileM16 = 512;

template <int NT>
__global__ __launch_bounds__(kThreads16) void dct2_gemm16_kernel(const float* __restrict__ X, int64_t ldx,
                                                                 const float* __restrict__ Bm, int ldb,
                                                                 float* __restrict__ Y, int64_t ldy,
                                                                 int64_t M, int K) {
  typedef typename BasisVec<NT>::type bvec;
  constexpr int kTileN = 32 * NT;
  extern __shared__ float Bs[];                     // [K + kPadRows][32][NT]
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int r = lane & 31;
  const int h = lane >> 5;
  const int n0 = blockIdx.y * kTileN;

  for (int i = tid; i < K * (kTileN / 4); i += kThreads16) {
    const int br = i / (kTileN / 4);
    const int c4 = i - br * (kTileN / 4);
    const float4 v = *reinterpret_cast<const float4*>(Bm + (size_t)br * ldb + n0 + c4 * 4);
    const float e[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int c = c4 * 4 + u;
      Bs[br * kTileN + (c & 31) * NT + (c >> 5)] = e[u];
    }
  }
  __syncthreads();

  const int64_t tiles = (M + kTileM16 - 1) / kTileM16;
  const int slices = K / kSliceK;
  auto row_ptr = [&](int64_t tile) {
    int64_t row = tile * kTileM16 + wave * 32 + r;
    if (row >= M) row = M - 1;
    return X + row * ldx + 16 * h;
  };
  const float* bs = Bs + (size_t)(16 * h) * kTileN + r * NT;
  const float* xrow = row_ptr(blockIdx.x);
  float4 cur[4], nxt[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) cur[q] = reinterpret_cast<const float4*>(xrow)[q];
  v16f acc[NT];
  bvec bcur, bnxt;

  for (int64_t tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
    const float* xnext = row_ptr(tile + gridDim.x < tiles ? tile + gridDim.x : tile);
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[t] = v16f{0};
    bcur = *reinterpret_cast<const bvec*>(bs);
    for (int s = 0; s < slices; ++s) {
      // the next slice of this tile, or the first slice of the next tile
      const float* ahead = s + 1 < slices ? xrow + (s + 1) * kSliceK : xnext;
#pragma unroll
      for (int q = 0; q < 4; ++q) nxt[q] = reinterpret_cast<const float4*>(ahead)[q];
      __builtin_amdgcn_sched_barrier(0);            // keep the requests ahead of the multiplies
      const float* brow = bs + (size_t)s * kSliceK * kTileN;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const float a4[4] = {cur[q].x, cur[q].y, cur[q].z, cur[q].w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int j = q * 4 + e;
          bnxt = *reinterpret_cast<const bvec*>(brow + (j < 15 ? (j + 1) * kTileN : kSliceK * kTileN));
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int t = 0; t < NT; ++t)
            acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(a4[e], bcur[t], acc[t], 0, 0, 0);
          bcur = bnxt;
        }
      }
#pragma unroll
      for (int q = 0; q < 4; ++q) cur[q] = nxt[q];
    }
    // accumulator element i of lane l is C[(i / 4) * 8 + (l / 32) * 4 + i % 4][l % 32]
    const int64_t base = tile * kTileM16 + wave * 32;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int64_t orow = base + (i >> 2) * 8 + h * 4 + (i & 3);
      if (orow < M) {
#pragma unroll
        for (int t = 0; t < NT; ++t) Y[orow * ldy + n0 + r + 32 * t] = acc[t][i];
      }
    }
    xrow = xnext;
  }
}

static std::mutex g_basis_mu;
static float* g_basis_fwd = nullptr;
static float* g_basis_inv = nullptr;

static int32_t ensure_basis(hipStream_t s) {
  std::lock_guard<std::mutex> lk(g_basis_mu);
  if (g_basis_fwd) return KRK_SUCCESS;
  DeviceGuard guard;
  KRK_HIP(hipMalloc(&guard.p, 2 * sizeof(float) * kDctB * kDctB));
  float* p = reinterpret_cast<float*>(guard.p);
  hipLaunchKernelGGL(dct2_basis_kernel, dim3(kDctB * kDctB / 256), dim3(256), 0, s, p, p + kDctB * kDctB);
  KRK_HIP(hipGetLastError());
  KRK_HIP(hipStreamSynchronize(s));
  g_basis_fwd = guard.release<float>();
  g_basis_inv = p + kDctB * kDctB;
  return KRK_SUCCESS;
}

static int32_t dct2_run(const float* in, float* out, int64_t n, int32_t keep, uint32_t flags, bool forward) {
  KRK_TRY(ensure_runtime());
  KRK_TRY(check_flags(flags));
  if (n < 0 || n % kDctB != 0 || keep <= 0 || keep > kDctB || keep % 64 != 0 || (n > 0 && (!in || !out))) {
    set_error("dct2: n must be a multiple of 256 and keep one of 64, 128, 192, 256");
    return KRK_E_ARGUMENT;
  }
  if (n == 0) return KRK_SUCCESS;
  hipStream_t s = nullptr;   // owns no object: runs on the null stream
  KRK_TRY(ensure_basis(s));
  const int64_t M = n / kDctB;
  const int64_t in_count = forward ? n : M * keep;
  const int64_t out_count = forward ? M * keep : n;
  const bool host = !(flags & KRK_DEVICE_PTRS);
  const float* d_in = in;
  float* d_out = out;
  float* tmp = nullptr;
  if (host) {
    KRK_HIP(hipMalloc((void**)&tmp, sizeof(float) * (size_t)(in_count + out_count)));
    hipError_t e = hipMemcpy(tmp, in, sizeof(float) * (size_t)in_count, hipMemcpyHostToDevice);
    if (e != hipSuccess) {
      (void)hipFree(tmp);
      return hip_fail(e, "dct2 staging", __FILE__, __LINE__);
    }
    d_in = tmp;
    d_out = tmp + in_count;
  } else if (((uintptr_t)in & 15) || ((uintptr_t)out & 15)) {
    set_error("dct2: device pointers must be 16-byte aligned");
    return KRK_E_ARGUMENT;
  }
  const int K = forward ? kDctB : keep;
  const int N = forward ? keep : kDctB;
  const float* basis = forward ? g_basis_fwd : g_basis_inv;
  const int nt = (N % 128 == 0) ? 4 : 2;          // 128-column tiles where the width allows
  const int tile_n = 32 * nt;
  const size_t lds_bytes = sizeof(float) * (size_t)(K + kPadRows) * tile_n;
  const int64_t tiles = (M + kTileM - 1) / kTileM;
  const int64_t per_cu = lds_bytes <= 80 * 1024 ? 2 : 1;   // workgroups that fit one CU's 160 KB of LDS
  int64_t gx = 256 * per_cu / (N / tile_n);
  if (gx > tiles) gx = tiles;
  if (gx < 1) gx = 1;
  hipError_t e;
  if (nt == 4) {
    const int64_t tiles16 = (M + kTileM16 - 1) / kTileM16;
    int64_t gx16 = 256 / (N / tile_n);
    if (gx16 > tiles16) gx16 = tiles16;
    if (gx16 < 1) gx16 = 1;
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(dct2_gemm16_kernel<4>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
    if (e == hipSuccess) {
      hipLaunchKernelGGL(dct2_gemm16_kernel<4>, dim3((unsigned)gx16, (unsigned)(N / tile_n)), dim3(kThreads16),
                         lds_bytes, s, d_in, (int64_t)K, basis, kDctB, d_out, (int64_t)N, M, K);
      e = hipGetLastError();
    }
  } else {
    auto kernel = dct2_gemm_kernel<2>;
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)lds_bytes);
    if (e == hipSuccess) {
      hipLaunchKernelGGL(kernel, dim3((unsigned)gx, (unsigned)(N / tile_n)), dim3(kThreads), lds_bytes, s,
                         d_in, (int64_t)K, basis, kDctB, d_out, (int64_t)N, M, K);
      e = hipGetLastError();
    }
  }
  if (e == hipSuccess && host)
    e = hipMemcpy(out, d_out, sizeof(float) * (size_t)out_count, hipMemcpyDeviceToHost);
  if (e == hipSuccess && !(flags & KRK_ASYNC)) e = hipStreamSynchronize(s);
  if (tmp) (void)hipFree(tmp);
  if (e != hipSuccess) return hip_fail(e, "dct2", __FILE__, __LINE__);
  return KRK_SUCCESS;
}

}  // namespace krk

extern "C" {

int32_t krk_dct2_forward(const float* x, float* coeff, int64_t n, int32_t keep, uint32_t flags) {
  return krk::dct2_run(x, coeff, n, keep, flags, true);
}

int32_t krk_dct2_inverse(const float* coeff, float* x, int64_t n, int32_t keep, uint32_t flags) {
  return krk::dct2_run(coeff, x, n, keep, flags, false);
}

}  // extern "C"
