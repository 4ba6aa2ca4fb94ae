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
// N = keep. Inverse: K = keep, N = 256. A workgroup keeps its 64-column basis tile resident in
// LDS, walks over row tiles of 256 blocks, stages X through LDS in 32-wide slices and feeds
// v_mfma_f32_32x32x2_f32: eight wavefronts, each owning a 32 x 64 piece of the output tile.
#include <cmath>
#include <mutex>

#include "krk_internal.h"

namespace krk {

constexpr int kDctB = 256;      // block length
constexpr int kThreads = 512;   // eight wavefronts: two per SIMD, so one can wait while one multiplies
constexpr int kTileM = 256;     // rows (blocks) per output tile: 32 per wavefront
constexpr int kTileN = 64;      // basis columns per workgroup
constexpr int kSliceK = 32;     // reduction slice staged per step
constexpr int kXsLd = kSliceK + 1;   // padded: a column read by 32 lanes hits 32 banks
constexpr int kStageVec = (kTileM * kSliceK / 4) / kThreads;   // float4 loads per thread per slice

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

// Y[M, N] = X[M, K] * Bm[K, N]; ldx / ldb / ldy are row strides in floats. K is a multiple of 32,
// N a multiple of 64 (both <= 256). grid.x workgroups share the row tiles, grid.y = N / 64.
//
// Pipeline per 32-wide slice of the reduction: the next slice of X is requested from HBM into
// registers, the current slice (already in LDS) is multiplied, and only then are the registers
// written to the other LDS buffer, so the memory latency sits behind 32 matrix instructions.
__global__ __launch_bounds__(kThreads) void dct2_gemm_kernel(const float* __restrict__ X, int64_t ldx,
                                                             const float* __restrict__ Bm, int ldb,
                                                             float* __restrict__ Y, int64_t ldy,
                                                             int64_t M, int K) {
  extern __shared__ float lds[];
  float* Bs = lds;                                  // [K][kTileN], resident for the whole launch
  float* Xs = lds + (size_t)K * kTileN;             // 2 x [kTileM][kXsLd]
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int n0 = blockIdx.y * kTileN;

  for (int i = tid; i < K * (kTileN / 4); i += kThreads) {
    const int r = i / (kTileN / 4);
    const int c4 = i - r * (kTileN / 4);
    reinterpret_cast<float4*>(Bs)[i] = *reinterpret_cast<const float4*>(Bm + (size_t)r * ldb + n0 + c4 * 4);
  }

  const int64_t tiles = (M + kTileM - 1) / kTileM;
  const int slices = K / kSliceK;
  for (int64_t tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
    const int64_t m0 = tile * kTileM;
    v16f acc0 = {0}, acc1 = {0};
    float4 regs[kStageVec];
    auto fetch = [&](int slice) {
#pragma unroll
      for (int it = 0; it < kStageVec; ++it) {
        const int i = it * kThreads + tid;       // float4 index inside the slice
        const int r = i >> 3;                    // 8 float4 per 32-float row piece
        const int c4 = i & 7;
        regs[it] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (m0 + r < M)
          regs[it] = *reinterpret_cast<const float4*>(X + (m0 + r) * ldx + slice * kSliceK + c4 * 4);
      }
    };
    auto park = [&](int buf) {
      float* dst = Xs + buf * (kTileM * kXsLd);
#pragma unroll
      for (int it = 0; it < kStageVec; ++it) {
        const int i = it * kThreads + tid;
        float* d = dst + (i >> 3) * kXsLd + (i & 7) * 4;
        d[0] = regs[it].x; d[1] = regs[it].y; d[2] = regs[it].z; d[3] = regs[it].w;
      }
    };
    fetch(0);
    park(0);
    __syncthreads();
    for (int s = 0; s < slices; ++s) {
      const int buf = s & 1;
      if (s + 1 < slices) fetch(s + 1);
      const float* xs = Xs + buf * (kTileM * kXsLd) + (wave * 32 + (lane & 31)) * kXsLd + (lane >> 5);
      const float* bs = Bs + (size_t)(s * kSliceK + (lane >> 5)) * kTileN + (lane & 31);
#pragma unroll
      for (int kk = 0; kk < kSliceK; kk += 2) {
        const float a = xs[kk];
        const float b0 = bs[kk * kTileN];
        const float b1 = bs[kk * kTileN + 32];
        acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b0, acc0, 0, 0, 0);
        acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b1, acc1, 0, 0, 0);
      }
      if (s + 1 < slices) park(buf ^ 1);
      __syncthreads();
    }
    // accumulator element i of lane l is C[(i / 4) * 8 + (l / 32) * 4 + i % 4][l % 32]
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int r = wave * 32 + (i >> 2) * 8 + (lane >> 5) * 4 + (i & 3);
      if (m0 + r < M) {
        float* y = Y + (m0 + r) * ldy + n0 + (lane & 31);
        y[0] = acc0[i];
        y[32] = acc1[i];
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
  float* p = nullptr;
  KRK_HIP(hipMalloc((void**)&p, 2 * sizeof(float) * kDctB * kDctB));
  hipLaunchKernelGGL(dct2_basis_kernel, dim3(kDctB * kDctB / 256), dim3(256), 0, s, p, p + kDctB * kDctB);
  KRK_HIP(hipGetLastError());
  KRK_HIP(hipStreamSynchronize(s));
  g_basis_fwd = p;
  g_basis_inv = p + kDctB * kDctB;
  return KRK_SUCCESS;
}

static int32_t dct2_run(const float* in, float* out, int64_t n, int32_t keep, uint32_t flags, bool forward) {
  KRK_TRY(ensure_runtime());
  KRK_TRY(check_flags(flags));
  if (n < 0 || n % kDctB != 0 || keep <= 0 || keep > kDctB || keep % kTileN != 0 || (n > 0 && (!in || !out))) {
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
  const size_t lds_bytes = sizeof(float) * ((size_t)K * kTileN + 2 * kTileM * kXsLd);
  const int64_t tiles = (M + kTileM - 1) / kTileM;
  int64_t gx = tiles < 256 / (N / kTileN) ? tiles : 256 / (N / kTileN);   // one workgroup per CU
  if (gx < 1) gx = 1;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(dct2_gemm_kernel),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
  if (e == hipSuccess) {
    hipLaunchKernelGGL(dct2_gemm_kernel, dim3((unsigned)gx, (unsigned)(N / kTileN)), dim3(kThreads), lds_bytes, s,
                       d_in, (int64_t)K, basis, kDctB, d_out, (int64_t)N, M, K);
    e = hipGetLastError();
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
