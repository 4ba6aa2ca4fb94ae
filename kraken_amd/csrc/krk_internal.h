// Shared internals of the HIP table engine (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <mutex>

#include "kraken_hip.h"

namespace krk {

// ---- error plumbing -------------------------------------------------------
void set_error(const char* fmt, ...);
int32_t hip_fail(hipError_t e, const char* what, const char* file, int line);

#define KRK_HIP(expr)                                                     \
  do {                                                                    \
    hipError_t krk_e_ = (expr);                                           \
    if (krk_e_ != hipSuccess) return ::krk::hip_fail(krk_e_, #expr, __FILE__, __LINE__); \
  } while (0)

#define KRK_TRY(expr)                    \
  do {                                   \
    int32_t krk_rc_ = (expr);            \
    if (krk_rc_ != KRK_SUCCESS) return krk_rc_; \
  } while (0)

int32_t ensure_runtime();
int current_device();
// Resolves, for the current device, the address of the fixed work space krk_dedup_noalloc uses.
int32_t noalloc_prepare();

// A device buffer that only ever grows; used for staging and scratch.
struct DeviceBuffer {
  void* ptr = nullptr;
  size_t bytes = 0;
  int32_t reserve(size_t want);
  void release();
  template <typename T>
  T* as() const {
    return reinterpret_cast<T*>(ptr);
  }
};

// Owns a fresh device allocation until it is handed over: error paths between hipMalloc and the
// hand-over free it.
struct DeviceGuard {
  void* p = nullptr;
  DeviceGuard() = default;
  DeviceGuard(const DeviceGuard&) = delete;
  DeviceGuard& operator=(const DeviceGuard&) = delete;
  ~DeviceGuard() {
    if (p) (void)hipFree(p);
  }
  template <typename T>
  T* release() {
    T* q = reinterpret_cast<T*>(p);
    p = nullptr;
    return q;
  }
};

// A host pointer that HIP knows as page-locked (hipHostMalloc, krk_host_malloc, a framework's
// pinned tensors) can be handed to kernels as it is: they read and write it across PCIe, which
// saves the staging copy and its launch. Returns the address kernels use, or null when the
// memory is pageable or not aligned to `align` bytes.
void* direct_host_pointer(const void* p, size_t align);

// Every API object starts with this: its own stream, the host lock that serialises
// calls on it, and the staging buffers used when the caller hands over host pointers.
struct ObjBase {
  hipStream_t stream = nullptr;
  std::mutex mu;
  DeviceBuffer stage[4];
  bool direct[4] = {false, false, false, false};   // output slot is the caller's own page-locked buffer
  int32_t open_stream();
  void close_stream();
  // Copies a host array into staging buffer `slot` (or passes a device pointer through).
  template <typename T>
  int32_t input(const T* p, size_t count, uint32_t flags, int slot, const T** dev) {
    if (flags & KRK_DEVICE_PTRS) {
      *dev = p;
      return KRK_SUCCESS;
    }
    if (void* d = direct_host_pointer(p, 16)) {
      *dev = reinterpret_cast<const T*>(d);
      return KRK_SUCCESS;
    }
    KRK_TRY(stage[slot].reserve(count * sizeof(T) + 16));
    if (count) KRK_HIP(hipMemcpyAsync(stage[slot].ptr, p, count * sizeof(T), hipMemcpyHostToDevice, stream));
    *dev = stage[slot].as<T>();
    return KRK_SUCCESS;
  }
  // Device destination for an output: the caller's pointer, or staging buffer `slot`.
  template <typename T>
  int32_t output(T* p, size_t count, uint32_t flags, int slot, T** dev) {
    if (flags & KRK_DEVICE_PTRS) {
      *dev = p;
      return KRK_SUCCESS;
    }
    direct[slot] = false;
    if (void* d = direct_host_pointer(p, 16)) {
      direct[slot] = true;
      *dev = reinterpret_cast<T*>(d);
      return KRK_SUCCESS;
    }
    KRK_TRY(stage[slot].reserve(count * sizeof(T) + 16));
    *dev = stage[slot].as<T>();
    return KRK_SUCCESS;
  }
  template <typename T>
  int32_t output_back(T* p, size_t count, uint32_t flags, int slot) {
    if ((flags & KRK_DEVICE_PTRS) || !count || direct[slot]) return KRK_SUCCESS;
    KRK_HIP(hipMemcpyAsync(p, stage[slot].ptr, count * sizeof(T), hipMemcpyDeviceToHost, stream));
    return KRK_SUCCESS;
  }
};

inline int32_t check_flags(uint32_t flags) {
  if (flags & ~(KRK_DEVICE_PTRS | KRK_ASYNC | KRK_NOTE_ROWS | KRK_IDS_AS_PULLED)) {
    set_error("unknown flag bits 0x%x", flags);
    return KRK_E_ARGUMENT;
  }
  if ((flags & KRK_ASYNC) && !(flags & KRK_DEVICE_PTRS)) {
    set_error("KRK_ASYNC needs KRK_DEVICE_PTRS");
    return KRK_E_ARGUMENT;
  }
  return KRK_SUCCESS;
}

constexpr int kWave = 64;
constexpr uint64_t kEmptyKey = 0xFFFFFFFFFFFFFFFFull;
constexpr uint32_t kEmptyRow = 0xFFFFFFFFu;

// 64-bit finaliser used to place ids in the open-addressing table.
__host__ __device__ inline uint64_t mix64(uint64_t x) {
  x ^= x >> 33;
  x *= 0xFF51AFD7ED558CCDull;
  x ^= x >> 33;
  x *= 0xC4CEB9FE1A85EC53ull;
  x ^= x >> 33;
  return x;
}

__host__ __device__ inline uint64_t splitmix64(uint64_t x) {
  uint64_t z = x + 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

// ---- row initialiser, evaluated per element on the device ------------------
// kind 0: constant p0; kind 1: uniform [p0, p1); kind 2: normal(mean p0, std p1).
struct InitK {
  int32_t kind;
  float p0;
  float p1;
  uint64_t seed_mix;  // splitmix64(seed)
};

// Normal draws come in pairs: elements 2q and 2q + 1 of a row are the two values of one
// Box-Muller step on the bits drawn for q: k = upper 24 bits + 1 gives the radius
// sqrt(-2 log(k / 2^24)), j = the next 24 bits the angle 2 pi j / 2^24; the values are
// radius * cos(angle) and radius * sin(angle), independent standard normals.
//
// The logarithm and the sine / cosine are written out here, in double-precision +, -, *, /
// only (no library call, no fused multiply-add: the build contracts nothing), so that this file
// and the CPU oracle evaluate the same sequence of IEEE operations and agree to the bit, and so
// that the rare branch of a pull that creates rows stays small: the general-purpose library
// routines handle every argument there is and take several times the instructions and registers.
// Their arguments here are 24-bit fractions, which makes the argument reductions exact.

// log(k / 2^24) for k in [1, 2^24]: k = m 2^e with m in (1/sqrt 2, sqrt 2], log m by the atanh
// series in f = (m - 1) / (m + 1), |f| <= 0.1716 (eight terms: below 1e-14).
__device__ inline double log_u24(uint32_t k) {
  int e = 31 - __clz((int)k);
  double m = (double)k * (1.0 / (double)(1u << e));   // exact, in [1, 2)
  if (m > 1.4142135623730951) {
    m = m * 0.5;
    e = e + 1;
  }
  const double f = (m - 1.0) / (m + 1.0);
  const double z = f * f;
  double p = 0.066666666666666666;                    // 1/15
  p = p * z + 0.076923076923076927;                   // 1/13
  p = p * z + 0.090909090909090912;                   // 1/11
  p = p * z + 0.11111111111111111;                    // 1/9
  p = p * z + 0.14285714285714285;                    // 1/7
  p = p * z + 0.2;                                    // 1/5
  p = p * z + 0.33333333333333331;                    // 1/3
  p = p * z + 1.0;
  return 2.0 * f * p + (double)(e - 24) * 0.69314718055994529;
}

// sin and cos of 2 pi j / 2^24 for j in [0, 2^24): the nearest quarter turn is taken off in
// integers (exact), the rest, at most pi/4 either way, goes through the Taylor polynomials
// (degree 13 and 14: below 3e-14), and the quarter turns are put back by swapping and negating.
__device__ inline void sincos_u24(uint32_t j, double& sn, double& cs) {
  const int32_t quarter = (int32_t)((j + (1u << 21)) >> 22);
  const int32_t rest = (int32_t)j - (quarter << 22);          // in [-2^21, 2^21)
  const double t = (double)rest * 3.7450702829239286e-07;      // 2 pi / 2^24
  const double z = t * t;
  double s = 1.6059043836821613e-10;                  // 1/13!
  s = s * z - 2.505210838544172e-08;                  // 1/11!
  s = s * z + 2.7557319223985893e-06;                 // 1/9!
  s = s * z - 0.00019841269841269841;                 // 1/7!
  s = s * z + 0.0083333333333333332;                  // 1/5!
  s = s * z - 0.16666666666666666;                    // 1/3!
  s = s * z + 1.0;
  s = s * t;
  double c = -1.1470745597729725e-11;                 // 1/14!
  c = c * z + 2.08767569878681e-09;                   // 1/12!
  c = c * z - 2.7557319223985888e-07;                 // 1/10!
  c = c * z + 2.4801587301587302e-05;                 // 1/8!
  c = c * z - 0.0013888888888888889;                  // 1/6!
  c = c * z + 0.041666666666666664;                   // 1/4!
  c = c * z - 0.5;
  c = c * z + 1.0;
  switch (quarter & 3) {
    case 0: sn = s; cs = c; break;
    case 1: sn = c; cs = -s; break;
    case 2: sn = -s; cs = -c; break;
    default: sn = -c; cs = s; break;
  }
}

// both values of pair q of the row whose bits start at `key`
__device__ inline void init_normal_pair(const InitK& k, uint64_t key, int64_t q, float& even, float& odd) {
  const uint64_t r = splitmix64(key + (uint64_t)q * 0x9E3779B97F4A7C15ull);
  const double radius = sqrt(-2.0 * log_u24((uint32_t)(r >> 40) + 1u));
  double sn, cs;
  sincos_u24((uint32_t)(r >> 16) & 0xFFFFFFu, sn, cs);
  even = (float)((double)k.p0 + (double)k.p1 * (radius * cs));
  odd = (float)((double)k.p0 + (double)k.p1 * (radius * sn));
}

__device__ inline float init_element(const InitK& k, uint64_t id, int64_t j) {
  if (k.kind == 0) return k.p0;
  uint64_t key = splitmix64(id ^ k.seed_mix);
  if (k.kind == 1) {
    uint64_t r = splitmix64(key + (uint64_t)j * 0x9E3779B97F4A7C15ull);
    double u = (double)(r >> 40) * (1.0 / 16777216.0);
    return (float)((double)k.p0 + ((double)k.p1 - (double)k.p0) * u);
  }
  float even, odd;
  init_normal_pair(k, key, j >> 1, even, odd);
  return (j & 1) ? odd : even;
}

// ---- optimizer arithmetic, one element at a time ---------------------------
// Pre-narrowed scalars: the reference evaluates (1.0 - beta) in double and
// narrows to float at the Tensor operator (ps/optim/adam.cc:57-58 etc.).
struct OptimK {
  int32_t type;
  int32_t has_wd;
  int32_t has_momentum;
  int32_t nesterov;
  int32_t amsgrad;
  int32_t centered;
  float wd;
  float momentum;
  float one_minus_damp;
  float beta1;
  float beta2;
  float one_minus_b1;
  float one_minus_b2;
  float eps;
  float alpha;
  float one_minus_alpha;
  float acc0;
};

OptimK make_optim_k(const krk_optim& o);
// Which state columns (bit per KRK_ST_*) and whether a step counter this optimizer touches.
uint32_t optim_state_mask(const krk_optim& o);

// State slots s0/s1/s2 per optimizer:
//   SGD      s0 = momentum buffer
//   Adagrad  s0 = state sum
//   Adam     s0 = first moment, s1 = second moment, s2 = second moment max
//   RMSprop  s0 = square average, s1 = g ave, s2 = momentum buffer
// `first` = this row has never been updated (SGD momentum copies the gradient then,
// ps/optim/sgd.cc:46-47). c1/c2 are Adam's (float)(1.0 - powf(beta, t)).
template <int OPT>
__device__ __forceinline__ void optim_element(const OptimK& k, float lr, float g, float& w,
                                              float& s0, float& s1, float& s2, bool first,
                                              float c1, float c2) {
  if (k.has_wd) g = g + k.wd * w;
  if (OPT == KRK_SGD) {
    // ps/optim/sgd.cc:41-60
    if (k.has_momentum) {
      if (first) {
        s0 = g;
      } else {
        s0 = k.momentum * s0 + k.one_minus_damp * g;
      }
      if (k.nesterov) {
        g = g + k.momentum * s0;
      } else {
        g = s0;
      }
    }
    w = w - g * lr;
  } else if (OPT == KRK_ADAGRAD) {
    // ps/optim/adagrad.cc:42-45
    s0 = s0 + g * g;
    float den = sqrtf(s0 + k.acc0) + k.eps;
    w = w - lr * (g / den);
  } else if (OPT == KRK_ADAM) {
    // ps/optim/adam.cc:57-78
    s0 = k.beta1 * s0 + k.one_minus_b1 * g;
    s1 = k.beta2 * s1 + k.one_minus_b2 * (g * g);
    float mt = s0 / c1;
    float vt = s1 / c2;
    float den;
    if (k.amsgrad) {
      s2 = fmaxf(s2, vt);
      den = sqrtf(s2) + k.eps;
    } else {
      den = sqrtf(vt) + k.eps;
    }
    w = w - (lr * mt) / den;
  } else {
    // ps/optim/rmsprop.cc:39-75
    s0 = k.alpha * s0 + k.one_minus_alpha * (g * g);
    float d = s0;
    if (k.centered) {
      s1 = s1 * k.alpha + k.one_minus_alpha * g;
      d = s0 - s1 * s1;
    }
    float den = sqrtf(d) + k.eps;
    if (k.has_momentum) {
      s2 = s2 * k.momentum + g / den;
      w = w - lr * s2;
    } else {
      w = w - (lr * g) / den;
    }
  }
}

// ---- device-wide exclusive scan of int32 (three plain launches, no spinning) ----
// out[i] = sum(in[0..i)), total written to *total_out (device). in/out may alias.
// CooTensorImpl::ToDense (t/coo_tensor_impl.cc:250-260, t/math.cc:1006-1096) on the device:
// dense[0, n) = 0, then dense[idx[j]] += val[j]. Large tensors whose indices ascend strictly and
// lie in range (what ToCoo produces) are written tile by tile in one pass over the output; any
// other input is zeroed and scattered into, decided on the device inside the same launches.
// work holds coo_densify_work_bytes(n); err (may be null) gets bit 0 set when an index is out
// of range.
size_t coo_densify_work_bytes(int64_t n);
int32_t coo_densify(const long long* d_idx, const float* d_val, int64_t nnz, float* d_dense, int64_t n,
                    void* work, uint32_t* err, hipStream_t stream);

// Stable radix sort of n (key, payload) pairs by the low `bits` bits of the key (radix_sort.hip).
// keys / vals are overwritten; keys_alt / vals_alt hold n entries each; work holds
// radix_sort_work_bytes(n). *keys_sorted / *vals_sorted say which of the two pairs of arrays the
// result is in.
size_t radix_sort_work_bytes(int64_t n);
int32_t radix_sort_pairs(uint32_t* keys, uint32_t* vals, uint32_t* keys_alt, uint32_t* vals_alt, int64_t n,
                         int bits, void* work, hipStream_t stream, uint32_t** keys_sorted,
                         uint32_t** vals_sorted);

// scratch must hold scan_scratch_bytes(n).
size_t scan_scratch_bytes(int64_t n);
int32_t exclusive_scan_i32(const int32_t* in, int32_t* out, int64_t n, int32_t* total_out,
                           void* scratch, hipStream_t stream);

}  // namespace krk
