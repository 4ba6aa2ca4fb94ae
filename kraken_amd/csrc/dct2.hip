// Blockwise orthonormal DCT-II / DCT-III over blocks of 256 floats on the matrix cores, at fp32
// accuracy.
//
// There is NO reference counterpart: the reference's "DCT" emitter is a threshold codec
// (worker/dct_emitter.cc:16-43) and contains no cosine transform. This file exists because the
// build's target names a blockwise DCT; it is pinned by the closed form
//     y[k] = s_k * sum_j x[j] * cos(pi * (2j + 1) * k / (2B)),  s_0 = sqrt(1/B), s_k = sqrt(2/B)
// and by the round trip inverse(forward(x)) == x. Keeping only the first `keep` coefficients of
// each block (keep = B * (1 - eta) = 64 for the emitter's default eta = 0.75) is the compression.
//
// Shape of the work: Y[M, N] = X[M, K] * Basis[K, N] with M = n / 256 blocks (forward: K = 256,
// N = keep; inverse: K = keep, N = 256), (1) folded in half by the basis' mirror symmetry and
// (2) multiplied as six bf16 products per fp32 product on v_mfma_f32_32x32x16_bf16, both below.
// A workgroup keeps its basis tile resident in LDS and walks over row tiles of 512 blocks; each
// of its sixteen wavefronts owns 32 rows and holds their X values in registers.
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

// (1) The cosine basis is mirror symmetric: c[255 - j][k] = (-1)^k c[j][k]. So the even
// coefficients of a block are a 128-term sum over x[j] + x[255 - j] and the odd ones over
// x[j] - x[255 - j] (forward), and a block's values come back as x[j] = E[j] + O[j],
// x[255 - j] = E[j] - O[j] with E over the even and O over the odd coefficients (inverse): half
// the multiplies of the plain product, at one more fp32 rounding per input pair (forward) or
// output pair (inverse).
//
// Shape of the work per workgroup: 512 blocks (rows) by 32 * NT folded columns, each folded
// column carrying two results (forward: coefficients 2c and 2c + 1; inverse: positions j and
// 255 - j), so a wavefront owns 32 rows and 2 * NT accumulator tiles, the first NT fed with the
// first operand of a pair (sum, or even coefficient), the others with the second (difference,
// or odd coefficient). X never passes through LDS: the matrix instruction takes, per lane
// (r = lane % 32, h = lane / 32), the values A[r][k] of eight reduction indices k, a set that
// depends on h only, and the order in which the reduction indices are consumed is free as long
// as the basis follows it. So lane (r, h) holds the operands of 8 or 16 consecutive folded
// indices per slice (two or four float4 from the row and as many from its mirror image).
// Sixteen wavefronts a workgroup (four per SIMD, 128 registers each): wavefronts never wait on
// each other inside the loop, the next slice's loads are in flight while this one multiplies,
// and what the wavefronts of a SIMD lose while one of them stores its tile, the other three fill in.
//
// Measured on fp32 [4096, 16384], forward / inverse, microseconds:
//                                                        keep 64      keep 128     keep 256
//   plain 256-term product, v_mfma_f32_32x32x2_f32       93 / 100     152 / 160    302 / 302
//   folded, same instruction, stores past the caches     58 / 61       93 / 100    165 / 170
//   folded, six bf16 products (this file)                56 / 55       88 / 72     117 / 128
// The last row moves 4.2 to 6.0 TB/s of the bytes the transform has to read and write: memory,
// not the matrix pipe, is what it waits for. Two wavefronts side by side on the same rows (all
// of keep 256's columns in one workgroup, X read from memory once) was slower (200 against
// 172 us with the fp32 instruction): the second read is already served by the L2 that the two
// workgroups of a row tile share. 64-column tiles for keep 128 and 256 (whole-line loads, more
// workgroups a row tile): 89 and 163 us.
constexpr int kFoldB = kDctB / 2;

// A wavefront's finished tile. Accumulator element i of lane l is
// C[(i / 4) * 8 + (l / 32) * 4 + i % 4][l % 32]. ybase points at the wavefront's first row
// (uniform), `rows` is how many rows exist from there on, and the lane's part of the address is
// a 32-bit offset: no 64-bit address is kept in registers across the multiplies. Lane r holds
// the folded columns cl = c0 + NT r + t, t < NT: neighbours, so that a row's results leave as
// one vector per lane (forward: coefficients 2 cl .. 2 cl + 2 NT; inverse: positions
// cl .. cl + NT and their mirror images 255 - cl - NT + 1 .. 255 - cl). The results are written
// once and not read again here: the stores go past the caches, which took keep 64 from 68 to
// 58 us forward and from 81 to 61 us back. (The same hint on the X loads costs a factor of two:
// a row's 128-byte lines are asked for in two or four pieces.)
template <int NT, bool FWD>
__device__ __forceinline__ void store_tile(const v16f (&acc)[2 * NT], float* __restrict__ ybase, int ldy,
                                           int64_t rows, int h, int cl) {
  // (the two offsets are a handful of operations: made here, once per tile, not kept in
  // registers for the whole launch)
  asm volatile("" : "+v"(h), "+v"(cl));
  const int left = (int)(rows < 32 ? rows : 32) - 4 * h;
  const uint32_t lane_off = (uint32_t)(4 * h * ldy + (FWD ? 2 * cl : cl));
  const uint32_t mirror_off = (uint32_t)(4 * h * ldy + kDctB - NT - cl);   // position 255 - (cl + NT - 1)
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int off = (i >> 2) * 8 + (i & 3);
    if (off < left) {
      float* row = ybase + off * ldy;               // uniform
      if (FWD) {
        if constexpr (NT == 2) {
          __builtin_nontemporal_store(v4f{acc[0][i], acc[2][i], acc[1][i], acc[3][i]},
                                      reinterpret_cast<v4f*>(row + lane_off));
        } else {
          __builtin_nontemporal_store(v2f{acc[0][i], acc[1][i]}, reinterpret_cast<v2f*>(row + lane_off));
        }
      } else {
        if constexpr (NT == 2) {
          __builtin_nontemporal_store(v2f{acc[0][i] + acc[2][i], acc[1][i] + acc[3][i]},
                                      reinterpret_cast<v2f*>(row + lane_off));
          __builtin_nontemporal_store(v2f{acc[1][i] - acc[3][i], acc[0][i] - acc[2][i]},
                                      reinterpret_cast<v2f*>(row + mirror_off));
        } else {
          row[lane_off] = acc[0][i] + acc[1][i];
          row[mirror_off] = acc[0][i] - acc[1][i];
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------
// (2) The folded product on the bf16 matrix instruction, at fp32 accuracy: every fp32 operand is
// split into three bf16 pieces, x = x0 + x1 + x2 with x0 = bf16(x), x1 = bf16(x - x0),
// x2 = bf16(x - x0 - x1) (round to nearest: |x1| <= 2^-9 |x|, |x2| <= 2^-18 |x|, and the three
// carry all 24 bits of x but for a last piece below 2^-27 |x|), and a product a b becomes the six
// pieces a0 b0 + a0 b1 + a1 b0 + a1 b1 + a0 b2 + a2 b0; the three left out are below 2^-26 |a b|,
// under the rounding of the fp32 sum they would be added to. A bf16 x bf16 product is exact in
// fp32 and v_mfma_f32_32x32x16_bf16 adds in fp32, sixteen reduction indices an instruction at
// sixteen times the fp32 instruction's rate: six of them cost 3/8 of the fp32 multiplies they
// replace. The basis is split once, from its double-precision values; X is split in registers,
// a slice at a time (about five VALU operations a value). Against scipy's float64 transform on
// N(0, 1) blocks the coefficients are off by 1.0e-8 of the block norm (rms; 1.5e-7 at worst),
// the fp32 instruction's by 1.3e-8 (1.7e-7), a plain fp32 matrix product's by 1.8e-8 (2.3e-7).
//
// LDS holds the basis pieces as [reduction group of 8][piece][tile][32 lanes][8 bf16]: the eight
// values a lane feeds to one instruction are one 16-byte read, and the global arrays are laid
// out so that the tile is filled with 16-byte copies.
// ---------------------------------------------------------------------------
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

struct Split3 {
  bf16x8 p0, p1, p2;
};

__device__ __forceinline__ Split3 split3(const float (&x)[8]) {
  Split3 o;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const v2f a = {x[2 * q], x[2 * q + 1]};
    const bf16x2 h0 = __builtin_convertvector(a, bf16x2);
    const v2f r1 = a - __builtin_convertvector(h0, v2f);
    const bf16x2 h1 = __builtin_convertvector(r1, bf16x2);
    const v2f r2 = r1 - __builtin_convertvector(h1, v2f);
    const bf16x2 h2 = __builtin_convertvector(r2, bf16x2);
    o.p0[2 * q] = h0[0];
    o.p0[2 * q + 1] = h0[1];
    o.p1[2 * q] = h1[0];
    o.p1[2 * q + 1] = h1[1];
    o.p2[2 * q] = h2[0];
    o.p2[2 * q + 1] = h2[1];
  }
  return o;
}

// The basis in pieces. fwd3[g][piece][k][i] = piece of c[8 g + i][k] (g < 16: the folded rows
// j < 128); inv3[second][g][piece][j][i] = piece of c[j][2 (8 g + i) + second] (j < 128).
__global__ void dct2_basis3_kernel(__bf16* __restrict__ fwd3, __bf16* __restrict__ inv3) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= kFoldB * kDctB) return;
  const int j = t / kDctB;                           // position, < 128
  const int k = t - j * kDctB;                       // coefficient
  const double s = k == 0 ? sqrt(1.0 / kDctB) : sqrt(2.0 / kDctB);
  const double v = s * cos(3.14159265358979323846 * (2.0 * j + 1.0) * k / (2.0 * kDctB));
  const __bf16 b0 = (__bf16)(float)v;
  const double r1 = v - (double)(float)b0;
  const __bf16 b1 = (__bf16)(float)r1;
  const double r2 = r1 - (double)(float)b1;
  const __bf16 b2 = (__bf16)(float)r2;
  const __bf16 piece[3] = {b0, b1, b2};
#pragma unroll
  for (int p = 0; p < 3; ++p) {
    fwd3[(((size_t)(j >> 3) * 3 + p) * kDctB + k) * 8 + (j & 7)] = piece[p];
    const int c = k >> 1, second = k & 1;
    inv3[((((size_t)second * 16 + (c >> 3)) * 3 + p) * kFoldB + j) * 8 + (c & 7)] = piece[p];
  }
}

template <int NT, bool FWD>
__global__ __launch_bounds__(kThreads) void dct2_split_kernel(const float* __restrict__ X, int64_t ldx,
                                                              const __bf16* __restrict__ B3,
                                                              float* __restrict__ Y, int64_t ldy,
                                                              int64_t M, int KF) {
  constexpr int NT2 = 2 * NT;
  // Folded indices a lane holds per slice: one group of 8, or two where the accumulators leave
  // the registers for it (a row's loads are then whole 64-byte pieces, which memory serves
  // better; the narrow tiles are the ones that wait for memory). Either way the groups are taken
  // in the same order, so the kernels of all widths add a coefficient's products up alike.
  constexpr int E = (FWD && NT == 1) ? 16 : 8;
  constexpr int V = E / 2;                          // float4 per lane and slice
  constexpr int kSliceK = 2 * E;
  extern __shared__ uint4 Bl[];                     // [KF / 8][3][NT2][32] x 8 bf16
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int r = lane & 31;
  const int h = lane >> 5;
  const int c0 = blockIdx.y * 32 * NT;              // first folded column of this workgroup
  const int groups = KF / 8;

  for (int i = tid; i < groups * 3 * NT2 * 32; i += kThreads) {
    const int rr = i & 31;
    const int t = (i >> 5) % NT2;
    const int gp = (i >> 5) / NT2;                  // group * 3 + piece
    const int cl = c0 + NT * rr + t % NT, second = t / NT;
    const uint4* src = reinterpret_cast<const uint4*>(B3);
    Bl[i] = FWD ? src[(size_t)gp * kDctB + 2 * cl + second]
                : src[((size_t)second * 16 * 3 + gp) * kFoldB + cl];
  }
  __syncthreads();

  const int64_t tiles = (M + kTileM - 1) / kTileM;
  const int slices = KF / kSliceK;
  auto lane_row = [&](int64_t tile) -> uint32_t {
    const int64_t left = M - 1 - tile * kTileM;      // uniform
    const int last = left < kTileM - 1 ? (int)left : kTileM - 1;
    int row = wave * 32 + r;
    if (row > last) row = last;
    return (uint32_t)row * (uint32_t)ldx;
  };
  constexpr int kHalf = FWD ? 16 : E;
  auto first = [&](int s) { return FWD && E == 8 ? 32 * (s >> 1) + 8 * (s & 1) : kSliceK * s; };
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
  uint32_t lrow = lane_row(blockIdx.x);
  float4 cur[V];
  load_slice(blockIdx.x, lrow, 0, cur);
  v16f acc[NT2];
  const uint4* bl = Bl + r;

  for (int64_t tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
    const int64_t tile_next = tile + gridDim.x < tiles ? tile + gridDim.x : tile;
#pragma unroll
    for (int t = 0; t < NT2; ++t) acc[t] = v16f{0};
#pragma unroll 1
    for (int s = 0; s < slices; ++s) {
      float v[2 * E];
#pragma unroll
      for (int q = 0; q < V; ++q) {
        v[4 * q] = cur[q].x;
        v[4 * q + 1] = cur[q].y;
        v[4 * q + 2] = cur[q].z;
        v[4 * q + 3] = cur[q].w;
      }
      // forward: the values, then their mirror images; inverse: even and odd coefficients interleaved
      float one[E], two[E];
#pragma unroll
      for (int e = 0; e < E; ++e) {
        one[e] = FWD ? v[e] + v[2 * E - 1 - e] : v[2 * e];
        two[e] = FWD ? v[e] - v[2 * E - 1 - e] : v[2 * e + 1];
      }
      Split3 piece[E / 8][2];
#pragma unroll
      for (int g = 0; g < E / 8; ++g) {
        float x8[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) x8[e] = one[8 * g + e];
        piece[g][0] = split3(x8);
#pragma unroll
        for (int e = 0; e < 8; ++e) x8[e] = two[8 * g + e];
        piece[g][1] = split3(x8);
      }
      // the slice's values are used up: the next slice's take their registers
      if (s + 1 < slices) {
        load_slice(tile, lrow, s + 1, cur);
      } else {
        lrow = lane_row(tile_next);
        load_slice(tile_next, lrow, 0, cur);
      }
#pragma unroll
      for (int g = 0; g < E / 8; ++g) {
        // group g of the slice: folded indices first(s) + 8 g + kHalf h ..+8
        const uint4* bg = bl + (size_t)((first(s) + 8 * g + kHalf * h) >> 3) * (3 * NT2 * 32);
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          const Split3& a = piece[g][half];
#pragma unroll
          for (int tt = 0; tt < NT; ++tt) {
            const int t = half * NT + tt;
            const uint4 u0 = bg[(0 * NT2 + t) * 32], u1 = bg[(1 * NT2 + t) * 32], u2 = bg[(2 * NT2 + t) * 32];
            const bf16x8 b0 = __builtin_bit_cast(bf16x8, u0), b1 = __builtin_bit_cast(bf16x8, u1),
                         b2 = __builtin_bit_cast(bf16x8, u2);
            // the small pieces first
            acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.p2, b0, acc[t], 0, 0, 0);
            acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.p0, b2, acc[t], 0, 0, 0);
            acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.p1, b1, acc[t], 0, 0, 0);
            acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.p1, b0, acc[t], 0, 0, 0);
            acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.p0, b1, acc[t], 0, 0, 0);
            acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.p0, b0, acc[t], 0, 0, 0);
          }
        }
      }
    }
    {
      const int64_t row0 = tile * kTileM + __builtin_amdgcn_readfirstlane(wave) * 32;
      store_tile<NT, FWD>(acc, Y + row0 * ldy, (int)ldy, M - row0, h, c0 + NT * r);
    }
  }
}

static std::mutex g_basis_mu;
static __bf16* g_basis3_fwd = nullptr;
static __bf16* g_basis3_inv = nullptr;
constexpr size_t kBasis3Count = (size_t)16 * 3 * kDctB * 8;   // per direction

static int32_t ensure_basis(hipStream_t s) {
  std::lock_guard<std::mutex> lk(g_basis_mu);
  if (g_basis3_fwd) return KRK_SUCCESS;
  DeviceGuard guard;
  KRK_HIP(hipMalloc(&guard.p, 2 * sizeof(__bf16) * kBasis3Count));
  __bf16* p3 = reinterpret_cast<__bf16*>(guard.p);
  hipLaunchKernelGGL(dct2_basis3_kernel, dim3(kFoldB * kDctB / 256), dim3(256), 0, s, p3, p3 + kBasis3Count);
  KRK_HIP(hipGetLastError());
  KRK_HIP(hipStreamSynchronize(s));
  g_basis3_fwd = guard.release<__bf16>();
  g_basis3_inv = p3 + kBasis3Count;
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
  const size_t lds_bytes = (size_t)(KF / 8) * 3 * 2 * nt * 32 * 16;   // [KF / 8][3][2 nt][32] x 16 bytes
  const int64_t tiles = (M + kTileM - 1) / kTileM;
  int64_t gx = 256 / gy;                           // one workgroup a compute unit
  if (gx > tiles) gx = tiles;
  if (gx < 1) gx = 1;
  const __bf16* basis = forward ? g_basis3_fwd : g_basis3_inv;
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
    launch(dct2_split_kernel<2, false>);
  } else if (nt == 2) {
    launch(dct2_split_kernel<2, true>);            // keep 128 and 256
  } else {
    launch(dct2_split_kernel<1, true>);            // keep 64 and 192
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
