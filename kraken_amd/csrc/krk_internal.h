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
// Box-Muller step on the bits drawn for q (radius from the upper 24 bits, angle from the next
// 24: radius * cos(angle) and radius * cos(angle - pi/2), independent standard normals; the
// second is written as a cosine so that both take the same code). A kernel that makes whole
// rows pays the logarithm and the square root once per two elements (init_normal_pair); one
// that makes a single element evaluates only the half it needs.
constexpr double kHalfPi = 1.5707963267948966192313216916398;
__device__ inline void normal_polar(uint64_t key, int64_t q, double& radius, double& angle) {
  const uint64_t r = splitmix64(key + (uint64_t)q * 0x9E3779B97F4A7C15ull);
  const double u1 = (double)((r >> 40) + 1) * (1.0 / 16777216.0);
  const double u2 = (double)((r >> 16) & 0xFFFFFFull) * (1.0 / 16777216.0);
  radius = sqrt(-2.0 * log(u1));
  angle = 6.283185307179586476925286766559 * u2;
}

__device__ inline void init_normal_pair(const InitK& k, uint64_t key, int64_t q, float& even, float& odd) {
  double radius, angle;
  normal_polar(key, q, radius, angle);
  even = (float)((double)k.p0 + (double)k.p1 * (radius * cos(angle)));
  odd = (float)((double)k.p0 + (double)k.p1 * (radius * cos(angle - kHalfPi)));
}

__device__ inline float init_element(const InitK& k, uint64_t id, int64_t j) {
  if (k.kind == 0) return k.p0;
  uint64_t key = splitmix64(id ^ k.seed_mix);
  // uniform: bits drawn for element j; normal: for the pair j / 2
  uint64_t r = splitmix64(key + (uint64_t)(k.kind == 1 ? j : j >> 1) * 0x9E3779B97F4A7C15ull);
  if (k.kind == 1) {
    double u = (double)(r >> 40) * (1.0 / 16777216.0);
    return (float)((double)k.p0 + ((double)k.p1 - (double)k.p0) * u);
  }
  double u1 = (double)((r >> 40) + 1) * (1.0 / 16777216.0);
  double u2 = (double)((r >> 16) & 0xFFFFFFull) * (1.0 / 16777216.0);
  double z = sqrt(-2.0 * log(u1)) * cos(6.283185307179586476925286766559 * u2 - ((j & 1) ? kHalfPi : 0.0));
  return (float)((double)k.p0 + (double)k.p1 * z);
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
