// Blockwise orthonormal DCT-II / DCT-III over blocks of 256 floats on the fp32 matrix cores.
//
// There is NO reference counterpart: the reference's "DCT" emitter is a threshold codec
// (worker/dct_emitter.cc:16-43) and contains no cosine transform. This file exists because the
// build's target names a blockwise DCT; it is pinned by the closed form
//     y[k] = s_k * sum_j x[j] * cos(pi * (2j + 1) * k / (2B)),  s_0 = sqrt(1/B), s_k = sqrt(2/B)
// and by the round trip inverse(forward(x)) == x. Keeping only the first `keep` coefficients of
// each block (keep = B * (1 - eta) = 64 for the emitter's default eta = 0.75) is the compression.
//
// Shape of the work: Y[M, N] = X[M, K] * Basis[K, N] with M = n / 256 blocks (forward: K = 256,
// N = keep; inverse: K = keep, N = 256), folded in half by the basis' mirror symmetry (below) and
// fed to v_mfma_f32_32x32x2_f32: a workgroup keeps its basis tile resident in LDS and walks over
// row tiles of 512 blocks; each of its sixteen wavefronts owns 32 rows and holds their X values
// in registers.
#include <cmath>
#include <mutex>

#include "krk_internal.h"

namespace krk {

constexpr int kDctB = 256;      // block length
constexpr int kThreads = 1024;  // sixteen wavefronts, four per SIMD
constexpr int kTileM = 512;     // rows (blocks) per output tile: 32 per wavefront

typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v2f __attribute__((ext_vector_type(2)));

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

// The cosine basis is mirror symmetric: c[255 - j][k] = (-1)^k c[j][k]. So the even coefficients
// of a block are a 128-term sum over x[j] + x[255 - j] and the odd ones over x[j] - x[255 - j]
// (forward), and a block's values come back as x[j] = E[j] + O[j], x[255 - j] = E[j] - O[j] with
// E over the even and O over the odd coefficients (inverse): half the multiplies of the plain
// product, at one more fp32 rounding per input pair (forward) or output pair (inverse).
//
// Shape of the work per workgroup: 512 blocks (rows) by 32 * NT folded columns, each folded
// column carrying two results (forward: coefficients 2c and 2c + 1; inverse: positions j and
// 255 - j), so a wavefront owns 32 rows and 2 * NT accumulator tiles, the first NT fed with the
// first operand of a pair (sum, or even coefficient), the others with the second (difference,
// or odd coefficient).
//
// The basis tile sits in LDS for the whole launch and is only read. It is laid out
// [KF + kPadRows][32][2 NT]: the 2 NT values a lane needs for one step are one vector read, at an
// offset from the slice's first row that is known at compile time. X never passes through LDS:
// the matrix instruction takes, per lane (r = lane % 32, h = lane / 32), one value A[r][k_h] for
// its two reduction indices k_0, k_1, and the order in which the reduction indices are consumed
// is free as long as the basis rows follow it. So lane (r, h) holds the operands of 8 or 16
// consecutive folded indices per slice (two or four float4 from the row and as many from its
// mirror image) and step e multiplies operand e against the basis row of its index.
// Sixteen wavefronts a workgroup (four per SIMD, 128 registers each): wavefronts never wait on
// each other inside the loop, the next slice's loads are in flight while this one multiplies,
// and what the wavefronts of a SIMD lose while one of them stores its tile, the other three fill in.
//
// Measured on fp32 [4096, 16384] against the plain 256-term product this replaces (same tiling,
// every multiply done): keep 256 forward 302 -> 160-175 us, keep 128 152 -> 93 us, keep 64 93 ->
// 58 us; inverse 302 -> 166-175, 160 -> 100, 100 -> 61 us. Two wavefronts side by side on the
// same rows (all of keep 256's columns in one workgroup, X read from memory once) was slower,
// 200 us: the second read is already served by the L2 the two workgroups of a row tile share.
constexpr int kPadRows = 17;   // the step after a tile's last one still reads "its" basis rows
constexpr int kFoldB = kDctB / 2;

template <int NT2>
struct BasisVec;
template <>
struct BasisVec<4> {
  typedef float type __attribute__((ext_vector_type(4)));
};
template <>
struct BasisVec<2> {
  typedef float type __attribute__((ext_vector_type(2)));
};

template <int NT, bool FWD>
__global__ __launch_bounds__(kThreads) void dct2_fold_kernel(const float* __restrict__ X, int64_t ldx,
                                                             const float* __restrict__ Bm,
                                                             float* __restrict__ Y, int64_t ldy,
                                                             int64_t M, int KF) {
  constexpr int NT2 = 2 * NT;
  typedef typename BasisVec<NT2>::type bvec;
  constexpr int kRow = 32 * NT2;                    // floats per basis row in LDS
  extern __shared__ float Bs[];                     // [KF + kPadRows][32][NT2]
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int r = lane & 31;
  const int h = lane >> 5;
  const int c0 = blockIdx.y * 32 * NT;              // first folded column of this workgroup

  if (FWD) {
    // row j of the tile: fwd[j][2 c0 .. 2 c0 + 64 NT), consecutive in memory
    for (int i = tid; i < KF * kRow; i += kThreads) {
      const int j = i / kRow;
      const int kk = i - j * kRow;
      const int cl = kk >> 1, second = kk & 1;
      Bs[(j * 32 + cl / NT) * NT2 + second * NT + cl % NT] = Bm[(size_t)j * kDctB + 2 * c0 + kk];
    }
  } else {
    // reduction index c: inv[2 c][c0 ..] feeds E, inv[2 c + 1][c0 ..] feeds O
    for (int i = tid; i < KF * kRow; i += kThreads) {
      const int kk = i / (32 * NT);                 // coefficient 2 c + second
      const int cl = i - kk * (32 * NT);
      const int c = kk >> 1, second = kk & 1;
      Bs[(c * 32 + cl / NT) * NT2 + second * NT + cl % NT] = Bm[(size_t)kk * kDctB + c0 + cl];
    }
  }
  __syncthreads();

  // Folded reduction indices a lane holds per slice: 8, or 16 where the accumulators leave the
  // registers for it (a row's loads are then whole 64-byte pieces, which memory serves better;
  // the narrow tiles are the ones that wait for memory).
  constexpr int E = NT == 1 ? 16 : 8;
  constexpr int kSliceK = 2 * E;                    // both halves of the wavefront
  constexpr int V = E / 2;                          // float4 per lane and slice
  const int64_t tiles = (M + kTileM - 1) / kTileM;
  const int slices = KF / kSliceK;
  // A lane's loads are addressed as (uniform tile and slice base) + (32-bit lane offset): two
  // registers per lane instead of a 64-bit pointer per stream. Rows past the end are clamped,
  // not masked: row r of X only reaches row r of Y, and those rows are never stored, so the
  // loads carry no branch.
  auto lane_row = [&](int64_t tile) -> uint32_t {
    int64_t row = wave * 32 + r;
    const int64_t last = M - 1 - tile * kTileM;
    if (row > last) row = last;
    return (uint32_t)(row * ldx);                   // at most 512 rows of 256 floats
  };
  // Which folded indices lane half h holds in step e of slice s: first(s) + kHalf h + e. Forward,
  // the two halves are 16 apart whatever E is, so that the kernels of all widths add a
  // coefficient's products up in the same order and keep-64 output equals the first 64 columns
  // of keep-256 output bit for bit. Inverse: the halves follow each other (a lane pair then
  // reads 128 consecutive bytes).
  constexpr int kHalf = FWD ? 16 : E;
  auto first = [&](int s) { return FWD && E == 8 ? 32 * (s >> 1) + 8 * (s & 1) : kSliceK * s; };
  // Slice s of a row. Forward: x[j ..+E) from j = first(s) + 16 h and its mirror image
  // x[256 - E - j ..+E) (element e pairs with element E - 1 - e of the mirror). Inverse: the 2E
  // coefficients 2 j ..+2E, even and odd ones interleaved.
  auto load_slice = [&](int64_t tile, uint32_t lrow, int s, float4 (&v)[V]) {
    const float* tb = X + tile * kTileM * ldx;       // uniform
    if (FWD) {
      const float* a = tb + first(s);
      const float* b = tb + (kDctB - E - kHalf - first(s));
      const uint32_t ia = lrow + kHalf * h, ib = lrow + kHalf - kHalf * h;
#pragma unroll
      for (int q = 0; q < V / 2; ++q) {
        v[q] = *reinterpret_cast<const float4*>(a + ia + 4 * q);
        v[V / 2 + q] = *reinterpret_cast<const float4*>(b + ib + 4 * q);
      }
    } else {
      const float* a = tb + 2 * first(s);
      const uint32_t ia = lrow + 2 * kHalf * h;
#pragma unroll
      for (int q = 0; q < V; ++q) v[q] = *reinterpret_cast<const float4*>(a + ia + 4 * q);
    }
  };
  const float* bs = Bs + (size_t)(kHalf * h) * kRow + r * NT2;
  uint32_t lrow = lane_row(blockIdx.x);
  float4 cur[V], nxt[V];
  load_slice(blockIdx.x, lrow, 0, cur);
  v16f acc[NT2];
  bvec bcur, bnxt;

  for (int64_t tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
    // the tile after this one (or this one again at the end: its values are then unused)
    const int64_t tile_next = tile + gridDim.x < tiles ? tile + gridDim.x : tile;
#pragma unroll
    for (int t = 0; t < NT2; ++t) acc[t] = v16f{0};
    bcur = *reinterpret_cast<const bvec*>(bs);
#pragma unroll 1
    for (int s = 0; s < slices; ++s) {
      // the next slice of this tile, or the first slice of the next tile
      if (s + 1 < slices) {
        load_slice(tile, lrow, s + 1, nxt);
      } else {
        lrow = lane_row(tile_next);
        load_slice(tile_next, lrow, 0, nxt);
      }
      __builtin_amdgcn_sched_barrier(0);            // keep the requests ahead of the multiplies
      const float* brow = bs + first(s) * kRow;
      const float* brow_next = bs + first(s + 1) * kRow;
      // the slice as scalars: the values, then their mirror images (forward), or the
      // interleaved even and odd coefficients (inverse)
      float v[2 * E];
#pragma unroll
      for (int q = 0; q < V; ++q) {
        v[4 * q] = cur[q].x;
        v[4 * q + 1] = cur[q].y;
        v[4 * q + 2] = cur[q].z;
        v[4 * q + 3] = cur[q].w;
      }
#pragma unroll
      for (int e = 0; e < E; ++e) {
        // basis values of the following step are requested before this step multiplies: row e + 1
        // of this slice, or the first row of the next one (past the last slice: padding, never used)
        bnxt = *reinterpret_cast<const bvec*>(e < E - 1 ? brow + (e + 1) * kRow : brow_next);
        const float first = FWD ? v[e] + v[2 * E - 1 - e] : v[2 * e];
        const float second = FWD ? v[e] - v[2 * E - 1 - e] : v[2 * e + 1];
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < NT; ++t)
          acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(first, bcur[t], acc[t], 0, 0, 0);
#pragma unroll
        for (int t = NT; t < NT2; ++t)
          acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(second, bcur[t], acc[t], 0, 0, 0);
        bcur = bnxt;
      }
#pragma unroll
      for (int q = 0; q < V; ++q) cur[q] = nxt[q];
    }
    // accumulator element i of lane l is C[(i / 4) * 8 + (l / 32) * 4 + i % 4][l % 32]. The
    // row offsets are compile-time numbers times the (uniform) row stride, so that no address
    // is kept in registers across the multiplies.
    const int64_t row0 = tile * kTileM + wave * 32 + h * 4;
    const int64_t left = M - row0;
    // lane r holds the folded columns c0 + NT r + t, t < NT: neighbours, so that a row's results
    // leave as one vector per lane (forward: coefficients 2 c .. 2 c + 2 NT; inverse: positions
    // c .. c + NT and their mirror images 255 - c - NT + 1 .. 255 - c). The results are written
    // once and not read again here: the stores go past the caches, which took keep 64 from 68 to
    // 58 us forward and from 81 to 61 us back. (The same hint on the X loads costs a factor of
    // two: a row's 128-byte lines are asked for in two or four pieces.)
    const int cl = c0 + NT * r;
    float* yp = Y + row0 * ldy + (FWD ? 2 * cl : cl);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int off = (i >> 2) * 8 + (i & 3);
      if (off < left) {
        float* p = yp + off * ldy;
        if (FWD) {
          if constexpr (NT == 2) {
            __builtin_nontemporal_store(v4f{acc[0][i], acc[2][i], acc[1][i], acc[3][i]}, reinterpret_cast<v4f*>(p));
          } else {
            __builtin_nontemporal_store(v2f{acc[0][i], acc[1][i]}, reinterpret_cast<v2f*>(p));
          }
        } else {
          float* q = p + (kDctB - NT - 2 * cl);     // position 255 - (cl + NT - 1)
          if constexpr (NT == 2) {
            __builtin_nontemporal_store(v2f{acc[0][i] + acc[2][i], acc[1][i] + acc[3][i]}, reinterpret_cast<v2f*>(p));
            __builtin_nontemporal_store(v2f{acc[1][i] - acc[3][i], acc[0][i] - acc[2][i]}, reinterpret_cast<v2f*>(q));
          } else {
            p[0] = acc[0][i] + acc[1][i];
            q[0] = acc[0][i] - acc[1][i];
          }
        }
      }
    }
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
  // folded shapes: the reduction runs over 128 input pairs (forward) or keep / 2 coefficient
  // pairs (inverse), the columns over keep / 2 coefficient pairs (forward) or 128 position pairs
  const int KF = forward ? kFoldB : keep / 2;
  const int NF = forward ? keep / 2 : kFoldB;
  const int nt = (NF % 64 == 0) ? 2 : 1;          // 64 folded columns a wavefront where the width allows
  const int gy = NF / (32 * nt);
  const size_t lds_bytes = sizeof(float) * (size_t)(KF + kPadRows) * 64 * nt;
  const int64_t tiles = (M + kTileM - 1) / kTileM;
  int64_t gx = 256 / gy;                           // one workgroup a compute unit
  if (gx > tiles) gx = tiles;
  if (gx < 1) gx = 1;
  const float* basis = forward ? g_basis_fwd : g_basis_inv;
  const dim3 grid((unsigned)gx, (unsigned)gy), block(kThreads);
  const int64_t ldx = forward ? kDctB : keep, ldy = forward ? keep : kDctB;
  hipError_t e = hipSuccess;
  auto launch = [&](auto kernel) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)lds_bytes);
    if (e != hipSuccess) return;
    hipLaunchKernelGGL(kernel, grid, block, lds_bytes, s, d_in, ldx, basis, d_out, ldy, M, KF);
    e = hipGetLastError();
  };
  if (!forward) {
    launch(dct2_fold_kernel<2, false>);
  } else if (nt == 2) {
    launch(dct2_fold_kernel<2, true>);             // keep 128 and 256
  } else {
    launch(dct2_fold_kernel<1, true>);             // keep 64 and 192
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
