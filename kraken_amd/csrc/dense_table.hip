// Dense table: one parameter vector in HBM with its optimizer state, updated by a single fused
// pass per push. Replaces DenseTable::Pull / ::Push (ps/dense_table.cc:31-43), the whole-tensor
// Optim::Update chains (ps/optim/*.cc) and COO densification (t/coo_tensor_impl.cc:250-260,
// t/math.cc:1006-1046).
#include <cmath>
#include <new>
#include <vector>

#include "krk_internal.h"

struct krk_dense_group;

struct krk_dense : krk::ObjBase {
  int64_t n = 0;
  float* w = nullptr;
  float* state[KRK_ST_COUNT] = {};   // created on first use, zero filled
  float* coo_grad = nullptr;         // densified COO gradient
  krk::DeviceBuffer coo_work;        // work space of the tiled densify
  int64_t steps = 0;                 // Adam's kSteps (one counter for the whole tensor)
  bool sgd_started = false;          // momentum buffer exists (first update copies the gradient)
  hipStream_t own_stream = nullptr;  // the stream created with the table (a group lends its own)
  krk_dense_group* member_of = nullptr;
};

// The dense tables of one combined request: they share one stream, and one launch serves all.
struct krk_dense_group : krk::ObjBase {
  std::vector<krk_dense*> tables;
  std::vector<int64_t> start;        // where each member begins in the concatenated arrays
  int64_t total = 0;
  hipStream_t own_stream = nullptr;
};

namespace krk {

constexpr int kDenseBlock = 256;

// The gradient passes once: it is read with a non-temporal load. Parameters and moments keep
// ordinary accesses, so a small table stays in L2 from step to step (for a large one the hint was
// measured to change nothing).
typedef float dfloat4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ dfloat4 dense_load(const float* p, int64_t i) {
  return reinterpret_cast<const dfloat4*>(p)[i];
}
__device__ __forceinline__ void dense_store(float* p, int64_t i, dfloat4 v) {
  reinterpret_cast<dfloat4*>(p)[i] = v;
}

template <int OPT>
__global__ __launch_bounds__(kDenseBlock) void dense_update_kernel(
    float* __restrict__ w, float* __restrict__ s0, float* __restrict__ s1, float* __restrict__ s2,
    const float* __restrict__ grad, int64_t n, float lr, OptimK k, bool first, float bc1, float bc2) {
  const int64_t n4 = n >> 2;
  const int64_t stride = (int64_t)gridDim.x * kDenseBlock;
  const dfloat4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
  for (int64_t i = (int64_t)blockIdx.x * kDenseBlock + threadIdx.x; i < n4; i += stride) {
    const dfloat4 g4 = __builtin_nontemporal_load(reinterpret_cast<const dfloat4*>(grad) + i);
    const dfloat4 w4 = dense_load(w, i);
    const dfloat4 a4 = s0 ? dense_load(s0, i) : zero;
    const dfloat4 b4 = s1 ? dense_load(s1, i) : zero;
    const dfloat4 c4 = s2 ? dense_load(s2, i) : zero;
    float ww[4], a[4], b[4], c[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      ww[j] = w4[j]; a[j] = a4[j]; b[j] = b4[j]; c[j] = c4[j];
      optim_element<OPT>(k, lr, g4[j], ww[j], a[j], b[j], c[j], first, bc1, bc2);
    }
    dense_store(w, i, (dfloat4){ww[0], ww[1], ww[2], ww[3]});
    if (s0) dense_store(s0, i, (dfloat4){a[0], a[1], a[2], a[3]});
    if (s1) dense_store(s1, i, (dfloat4){b[0], b[1], b[2], b[3]});
    if (s2) dense_store(s2, i, (dfloat4){c[0], c[1], c[2], c[3]});
  }
  // tail (n not a multiple of 4)
  for (int64_t i = (n4 << 2) + (int64_t)blockIdx.x * kDenseBlock + threadIdx.x; i < n; i += stride) {
    float g = grad[i], ww = w[i];
    float a = s0 ? s0[i] : 0.0f, b = s1 ? s1[i] : 0.0f, c = s2 ? s2[i] : 0.0f;
    optim_element<OPT>(k, lr, g, ww, a, b, c, first, bc1, bc2);
    w[i] = ww;
    if (s0) s0[i] = a;
    if (s1) s1[i] = b;
    if (s2) s2[i] = c;
  }
}

static unsigned dense_grid(int64_t n) {
  int64_t blocks = (n / 4 + kDenseBlock - 1) / kDenseBlock;
  if (blocks < 1) blocks = 1;
  // Two workgroups per compute unit, grid-stride beyond that: seven streams (four read, three
  // written) through 512 workgroups run at 5.4 TB/s, through 256 or 4096 at 4.7-4.9.
  if (blocks > 512) blocks = 512;
  return (unsigned)blocks;
}

static int32_t ensure_state(krk_dense* t, int st) {
  if (t->state[st]) return KRK_SUCCESS;
  DeviceGuard guard;
  KRK_HIP(hipMalloc(&guard.p, (size_t)(t->n ? t->n : 1) * sizeof(float)));
  KRK_HIP(hipMemsetAsync(guard.p, 0, (size_t)t->n * sizeof(float), t->stream));
  t->state[st] = guard.release<float>();   // only a zeroed column counts as present
  return KRK_SUCCESS;
}

// One Optim::Update on the whole tensor with a device-resident gradient.
static int32_t dense_apply(krk_dense* t, const krk_optim& o, const float* d_grad, float lr) {
  const uint32_t mask = optim_state_mask(o);
  for (int st = 1; st < KRK_ST_COUNT; ++st)
    if (mask & (1u << st)) KRK_TRY(ensure_state(t, st));
  const OptimK k = make_optim_k(o);
  const dim3 grid(dense_grid(t->n)), block(kDenseBlock);
  float *s0 = nullptr, *s1 = nullptr, *s2 = nullptr;
  bool first = false;
  float bc1 = 1.0f, bc2 = 1.0f;
  switch (o.type) {
    case KRK_SGD:
      if (o.has_momentum) {
        s0 = t->state[KRK_ST_MOMENTUM_BUFFER];
        first = !t->sgd_started;
        t->sgd_started = true;
      }
      hipLaunchKernelGGL((dense_update_kernel<KRK_SGD>), grid, block, 0, t->stream, t->w, s0, s1, s2,
                         d_grad, t->n, lr, k, first, bc1, bc2);
      break;
    case KRK_ADAGRAD:
      s0 = t->state[KRK_ST_STATE_SUM];
      hipLaunchKernelGGL((dense_update_kernel<KRK_ADAGRAD>), grid, block, 0, t->stream, t->w, s0, s1,
                         s2, d_grad, t->n, lr, k, first, bc1, bc2);
      break;
    case KRK_ADAM: {
      s0 = t->state[KRK_ST_FIRST_MOMENT];
      s1 = t->state[KRK_ST_SECOND_MOMENT];
      if (o.amsgrad) s2 = t->state[KRK_ST_SECOND_MOMENT_MAX];
      const int64_t steps = ++t->steps;   // ps/optim/adam.cc:61
      bc1 = (float)(1.0 - (double)std::pow(o.beta1, (float)steps));   // :63-64, float pow
      bc2 = (float)(1.0 - (double)std::pow(o.beta2, (float)steps));
      hipLaunchKernelGGL((dense_update_kernel<KRK_ADAM>), grid, block, 0, t->stream, t->w, s0, s1, s2,
                         d_grad, t->n, lr, k, first, bc1, bc2);
      break;
    }
    default:
      s0 = t->state[KRK_ST_SQUARE_AVERAGE];
      if (o.centered) s1 = t->state[KRK_ST_G_AVE];
      if (o.has_momentum) s2 = t->state[KRK_ST_MOMENTUM_BUFFER];
      hipLaunchKernelGGL((dense_update_kernel<KRK_RMSPROP>), grid, block, 0, t->stream, t->w, s0, s1,
                         s2, d_grad, t->n, lr, k, first, bc1, bc2);
      break;
  }
  KRK_HIP(hipGetLastError());
  return KRK_SUCCESS;
}

// ---- several dense tables in one launch ------------------------------------------------------
// Ps::CombinePullDenseTable (ps/ps_op.cc:177-252) pulls every dense parameter of the model in one
// request, and the worker does that after every step (pytorch/optimizer.py:151-173); one table per
// launch makes a model with dozens of small tensors pay a launch per tensor. Here the members'
// values (and, for the push, gradients) are one concatenated array in member order and a launch
// takes up to kDenseGroupChunk members: workgroups [block_start[m], block_start[m + 1]) belong to
// member m.
constexpr int kDenseGroupChunk = 32;

struct DenseMember {
  float* w;
  float* s0;
  float* s1;
  float* s2;
  int64_t n;
  int64_t start;     // first element in the concatenated arrays
  float bc1, bc2;    // Adam's bias corrections of this member's step
  int32_t first;     // SGD with momentum: the buffer does not exist yet
};

struct DenseGroupArgs {
  int32_t members;
  uint32_t block_start[kDenseGroupChunk + 1];
  DenseMember m[kDenseGroupChunk];
};

__device__ __forceinline__ int dense_member_of_block(const DenseGroupArgs& a) {
  int m = 0;
  while (m + 1 < a.members && blockIdx.x >= a.block_start[m + 1]) ++m;
  return m;
}

__global__ __launch_bounds__(kDenseBlock) void dense_group_pull_kernel(DenseGroupArgs a, float* __restrict__ out) {
  const int mi = dense_member_of_block(a);
  const DenseMember& m = a.m[mi];
  const int64_t lane = (int64_t)(blockIdx.x - a.block_start[mi]) * kDenseBlock + threadIdx.x;
  const int64_t stride = (int64_t)(a.block_start[mi + 1] - a.block_start[mi]) * kDenseBlock;
  float* dst = out + m.start;
  // 16-byte accesses where the member begins on a 16-byte boundary of the output
  const int64_t n4 = (m.start & 3) == 0 ? m.n >> 2 : 0;
  for (int64_t i = lane; i < n4; i += stride)
    __builtin_nontemporal_store(dense_load(m.w, i), reinterpret_cast<dfloat4*>(dst) + i);
  for (int64_t i = (n4 << 2) + lane; i < m.n; i += stride) dst[i] = m.w[i];
}

template <int OPT>
__global__ __launch_bounds__(kDenseBlock) void dense_group_update_kernel(DenseGroupArgs a,
                                                                         const float* __restrict__ grads,
                                                                         float lr, OptimK k) {
  const int mi = dense_member_of_block(a);
  const DenseMember& m = a.m[mi];
  const int64_t lane = (int64_t)(blockIdx.x - a.block_start[mi]) * kDenseBlock + threadIdx.x;
  const int64_t stride = (int64_t)(a.block_start[mi + 1] - a.block_start[mi]) * kDenseBlock;
  const float* grad = grads + m.start;
  float* w = m.w;
  float* s0 = m.s0;
  float* s1 = m.s1;
  float* s2 = m.s2;
  const bool first = m.first != 0;
  const dfloat4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
  const int64_t n4 = (m.start & 3) == 0 ? m.n >> 2 : 0;
  for (int64_t i = lane; i < n4; i += stride) {
    const dfloat4 g4 = __builtin_nontemporal_load(reinterpret_cast<const dfloat4*>(grad) + i);
    const dfloat4 w4 = dense_load(w, i);
    const dfloat4 a4 = s0 ? dense_load(s0, i) : zero;
    const dfloat4 b4 = s1 ? dense_load(s1, i) : zero;
    const dfloat4 c4 = s2 ? dense_load(s2, i) : zero;
    float ww[4], sa[4], sb[4], sc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      ww[j] = w4[j]; sa[j] = a4[j]; sb[j] = b4[j]; sc[j] = c4[j];
      optim_element<OPT>(k, lr, g4[j], ww[j], sa[j], sb[j], sc[j], first, m.bc1, m.bc2);
    }
    dense_store(w, i, (dfloat4){ww[0], ww[1], ww[2], ww[3]});
    if (s0) dense_store(s0, i, (dfloat4){sa[0], sa[1], sa[2], sa[3]});
    if (s1) dense_store(s1, i, (dfloat4){sb[0], sb[1], sb[2], sb[3]});
    if (s2) dense_store(s2, i, (dfloat4){sc[0], sc[1], sc[2], sc[3]});
  }
  for (int64_t i = (n4 << 2) + lane; i < m.n; i += stride) {
    float g = grad[i], ww = w[i];
    float sa = s0 ? s0[i] : 0.0f, sb = s1 ? s1[i] : 0.0f, sc = s2 ? s2[i] : 0.0f;
    optim_element<OPT>(k, lr, g, ww, sa, sb, sc, first, m.bc1, m.bc2);
    w[i] = ww;
    if (s0) s0[i] = sa;
    if (s1) s1[i] = sb;
    if (s2) s2[i] = sc;
  }
}

// What one Optim::Update of table t reads and writes, with the host-side bookkeeping of
// dense_apply (state columns created, Adam's counter advanced, SGD's first momentum step noted).
static int32_t dense_member(krk_dense* t, const krk_optim& o, DenseMember* m) {
  const uint32_t mask = optim_state_mask(o);
  for (int st = 1; st < KRK_ST_COUNT; ++st)
    if (mask & (1u << st)) KRK_TRY(ensure_state(t, st));
  m->w = t->w;
  m->s0 = m->s1 = m->s2 = nullptr;
  m->n = t->n;
  m->bc1 = m->bc2 = 1.0f;
  m->first = 0;
  switch (o.type) {
    case KRK_SGD:
      if (o.has_momentum) {
        m->s0 = t->state[KRK_ST_MOMENTUM_BUFFER];
        m->first = t->sgd_started ? 0 : 1;
        t->sgd_started = true;
      }
      break;
    case KRK_ADAGRAD:
      m->s0 = t->state[KRK_ST_STATE_SUM];
      break;
    case KRK_ADAM: {
      m->s0 = t->state[KRK_ST_FIRST_MOMENT];
      m->s1 = t->state[KRK_ST_SECOND_MOMENT];
      if (o.amsgrad) m->s2 = t->state[KRK_ST_SECOND_MOMENT_MAX];
      const int64_t steps = ++t->steps;   // ps/optim/adam.cc:61
      m->bc1 = (float)(1.0 - (double)std::pow(o.beta1, (float)steps));
      m->bc2 = (float)(1.0 - (double)std::pow(o.beta2, (float)steps));
      break;
    }
    default:
      m->s0 = t->state[KRK_ST_SQUARE_AVERAGE];
      if (o.centered) m->s1 = t->state[KRK_ST_G_AVE];
      if (o.has_momentum) m->s2 = t->state[KRK_ST_MOMENTUM_BUFFER];
      break;
  }
  return KRK_SUCCESS;
}

// Workgroups a member of n elements gets in a combined launch.
static unsigned dense_member_blocks(int64_t n) {
  int64_t blocks = (n / 4 + kDenseBlock - 1) / kDenseBlock;
  if (blocks < 1) blocks = 1;
  if (blocks > 512) blocks = 512;
  return (unsigned)blocks;
}

// Takes the group's lock and then every member's, in member order.
struct DenseGroupLock {
  krk_dense_group* g;
  explicit DenseGroupLock(krk_dense_group* gg) : g(gg) {
    g->mu.lock();
    for (krk_dense* t : g->tables) t->mu.lock();
  }
  ~DenseGroupLock() {
    for (auto it = g->tables.rbegin(); it != g->tables.rend(); ++it) (*it)->mu.unlock();
    g->mu.unlock();
  }
  DenseGroupLock(const DenseGroupLock&) = delete;
  DenseGroupLock& operator=(const DenseGroupLock&) = delete;
};

static int32_t dense_finish(krk_dense* t, uint32_t flags) {
  if (flags & KRK_ASYNC) return KRK_SUCCESS;
  KRK_HIP(hipStreamSynchronize(t->stream));
  return KRK_SUCCESS;
}

}  // namespace krk

using namespace krk;

static int32_t check_dense(krk_dense* t) {
  if (!t) {
    set_error("null dense table handle");
    return KRK_E_ARGUMENT;
  }
  return ensure_runtime();
}

extern "C" {

int32_t krk_dense_create(const float* val, int64_t n, uint32_t flags, krk_dense** out) {
  if (!out || n < 0 || (n > 0 && !val)) return KRK_E_ARGUMENT;
  KRK_TRY(check_flags(flags & ~KRK_ASYNC));
  KRK_TRY(ensure_runtime());
  krk_dense* t = new (std::nothrow) krk_dense();
  if (!t) return KRK_E_DEVICE;
  t->n = n;
  int32_t rc = t->open_stream();
  t->own_stream = t->stream;
  if (rc == KRK_SUCCESS) {
    hipError_t e = hipMalloc((void**)&t->w, (size_t)(n ? n : 1) * sizeof(float));
    if (e == hipSuccess && n)
      e = hipMemcpyAsync(t->w, val, (size_t)n * sizeof(float),
                         (flags & KRK_DEVICE_PTRS) ? hipMemcpyDeviceToDevice : hipMemcpyHostToDevice,
                         t->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(t->stream);
    if (e != hipSuccess) rc = hip_fail(e, "krk_dense_create", __FILE__, __LINE__);
  }
  if (rc != KRK_SUCCESS) {
    krk_dense_destroy(t);
    return rc;
  }
  *out = t;
  return KRK_SUCCESS;
}

int32_t krk_dense_destroy(krk_dense* t) {
  if (!t) return KRK_SUCCESS;
  if (t->member_of) {
    set_error("the dense table is still a member of a group: destroy the group first");
    return KRK_E_ARGUMENT;
  }
  if (t->stream) (void)hipStreamSynchronize(t->stream);
  if (t->w) (void)hipFree(t->w);
  if (t->coo_grad) (void)hipFree(t->coo_grad);
  t->coo_work.release();
  for (auto& s : t->state)
    if (s) (void)hipFree(s);
  t->close_stream();
  delete t;
  return KRK_SUCCESS;
}

int32_t krk_dense_sync(krk_dense* t) {
  KRK_TRY(check_dense(t));
  std::lock_guard<std::mutex> lk(t->mu);
  return dense_finish(t, 0);
}

int32_t krk_dense_pull(krk_dense* t, float* out, uint32_t flags) {
  KRK_TRY(check_dense(t));
  KRK_TRY(check_flags(flags));
  if (t->n > 0 && !out) return KRK_E_ARGUMENT;
  std::lock_guard<std::mutex> lk(t->mu);
  if (t->n)
    KRK_HIP(hipMemcpyAsync(out, t->w, (size_t)t->n * sizeof(float),
                           (flags & KRK_DEVICE_PTRS) ? hipMemcpyDeviceToDevice : hipMemcpyDeviceToHost,
                           t->stream));
  return dense_finish(t, flags);
}

int32_t krk_dense_push(krk_dense* t, const krk_optim* o, const float* grad, int64_t n, float lr,
                       uint32_t flags) {
  KRK_TRY(check_dense(t));
  KRK_TRY(check_flags(flags));
  if (!o || o->type < KRK_ADAGRAD || o->type > KRK_SGD) return KRK_UNSUPPORTED_OPTIM;
  if (n < 0 || (n > 0 && !grad)) return KRK_E_ARGUMENT;
  std::lock_guard<std::mutex> lk(t->mu);
  if (n != t->n) {   // ps/optim/sgd.cc:36-39: the reference's answer, whatever else is wrong with the request
    set_error("gradient has %lld elements, table has %lld", (long long)n, (long long)t->n);
    return KRK_GRADIENT_UNCOMPATIBLE;
  }
  if ((flags & KRK_DEVICE_PTRS) && ((uintptr_t)grad & 15)) {   // the update moves 16 bytes per lane
    set_error("device gradient must be 16-byte aligned");
    return KRK_E_ARGUMENT;
  }
  if (n == 0) return KRK_SUCCESS;
  const float* d_grad;
  KRK_TRY(t->input(grad, (size_t)n, flags, 0, &d_grad));
  KRK_TRY(dense_apply(t, *o, d_grad, lr));
  return dense_finish(t, flags);
}

int32_t krk_dense_push_coo(krk_dense* t, const krk_optim* o, const int64_t* idx, const float* val,
                           int64_t nnz, float lr, uint32_t flags) {
  KRK_TRY(check_dense(t));
  KRK_TRY(check_flags(flags));
  if (!o || o->type < KRK_ADAGRAD || o->type > KRK_SGD) return KRK_UNSUPPORTED_OPTIM;
  if (nnz < 0 || (nnz > 0 && (!idx || !val))) return KRK_E_ARGUMENT;
  std::lock_guard<std::mutex> lk(t->mu);
  if (nnz == 0) return KRK_SUCCESS;   // ps/optim/adam.cc:26-29 : nothing is touched, not even kSteps
  if (t->n == 0) return KRK_GRADIENT_UNCOMPATIBLE;
  if (!t->coo_grad) KRK_HIP(hipMalloc((void**)&t->coo_grad, (size_t)t->n * sizeof(float) + 16));
  const int64_t* d_idx;
  const float* d_val;
  KRK_TRY(t->input(idx, (size_t)nnz, flags, 0, &d_idx));
  KRK_TRY(t->input(val, (size_t)nnz, flags, 1, &d_val));
  // entries whose index lies outside [0, n) are skipped
  KRK_TRY(t->coo_work.reserve(coo_densify_work_bytes(t->n)));
  KRK_TRY(coo_densify(reinterpret_cast<const long long*>(d_idx), d_val, nnz, t->coo_grad, t->n, t->coo_work.ptr,
                      nullptr, t->stream));
  KRK_TRY(dense_apply(t, *o, t->coo_grad, lr));
  return dense_finish(t, flags);
}

int32_t krk_dense_state(krk_dense* t, int32_t state_type, float* out, uint32_t flags) {
  KRK_TRY(check_dense(t));
  KRK_TRY(check_flags(flags));
  if (state_type < 1 || state_type >= KRK_ST_COUNT || (t->n > 0 && !out)) return KRK_E_ARGUMENT;
  std::lock_guard<std::mutex> lk(t->mu);
  if (t->n == 0) return KRK_SUCCESS;
  const size_t bytes = (size_t)t->n * sizeof(float);
  if (t->state[state_type]) {
    KRK_HIP(hipMemcpyAsync(out, t->state[state_type], bytes,
                           (flags & KRK_DEVICE_PTRS) ? hipMemcpyDeviceToDevice : hipMemcpyDeviceToHost,
                           t->stream));
  } else if (flags & KRK_DEVICE_PTRS) {
    KRK_HIP(hipMemsetAsync(out, 0, bytes, t->stream));
  } else {
    memset(out, 0, bytes);
  }
  return dense_finish(t, flags);
}

int32_t krk_dense_size(krk_dense* t, int64_t* n) {
  if (!t || !n) return KRK_E_ARGUMENT;
  *n = t->n;
  return KRK_SUCCESS;
}

int32_t krk_dense_states(krk_dense* t, uint32_t* mask) {
  if (!t || !mask) return KRK_E_ARGUMENT;
  std::lock_guard<std::mutex> lk(t->mu);
  uint32_t m = t->steps > 0 ? 1u : 0u;
  for (int st = 1; st < KRK_ST_COUNT; ++st) {
    if (t->state[st]) m |= 1u << st;   // states are created by the first update that needs them
  }
  *mask = m;
  return KRK_SUCCESS;
}

int32_t krk_dense_import_state(krk_dense* t, int32_t state_type, const float* state, int64_t steps,
                               uint32_t flags) {
  KRK_TRY(check_dense(t));
  KRK_TRY(check_flags(flags));
  if (state && (state_type < 1 || state_type >= KRK_ST_COUNT)) return KRK_E_ARGUMENT;
  std::lock_guard<std::mutex> lk(t->mu);
  if (state && t->n > 0) {
    KRK_TRY(ensure_state(t, state_type));
    KRK_HIP(hipMemcpyAsync(t->state[state_type], state, (size_t)t->n * sizeof(float),
                           (flags & KRK_DEVICE_PTRS) ? hipMemcpyDeviceToDevice : hipMemcpyHostToDevice,
                           t->stream));
    if (state_type == KRK_ST_MOMENTUM_BUFFER) t->sgd_started = true;
  }
  if (steps >= 0) t->steps = steps;
  // a host source buffer may be reused by the caller as soon as this returns
  return dense_finish(t, (flags & KRK_DEVICE_PTRS) ? flags : (flags & ~KRK_ASYNC));
}

int32_t krk_dense_group_create(krk_dense** tables, int32_t n, krk_dense_group** out) {
  if (!tables || !out || n <= 0) return KRK_E_ARGUMENT;
  KRK_TRY(ensure_runtime());
  for (int i = 0; i < n; ++i) {
    if (!tables[i] || tables[i]->member_of) {
      set_error("group members must be dense tables that are in no other group");
      return KRK_E_ARGUMENT;
    }
    for (int j = 0; j < i; ++j)
      if (tables[j] == tables[i]) return KRK_E_ARGUMENT;
  }
  krk_dense_group* g = new (std::nothrow) krk_dense_group();
  if (!g) return KRK_E_DEVICE;
  const int32_t rc = g->open_stream();
  if (rc != KRK_SUCCESS) {
    delete g;
    return rc;
  }
  g->own_stream = g->stream;
  for (int i = 0; i < n; ++i) {
    krk_dense* t = tables[i];
    std::lock_guard<std::mutex> lk(t->mu);
    (void)hipStreamSynchronize(t->stream);
    t->stream = g->stream;   // from now on the table's own calls are ordered with the group's
    t->member_of = g;
    g->tables.push_back(t);
    g->start.push_back(g->total);
    g->total += t->n;
  }
  *out = g;
  return KRK_SUCCESS;
}

int32_t krk_dense_group_destroy(krk_dense_group* g) {
  if (!g) return KRK_SUCCESS;
  (void)hipStreamSynchronize(g->stream);
  for (krk_dense* t : g->tables) {
    std::lock_guard<std::mutex> lk(t->mu);
    t->stream = t->own_stream;
    t->member_of = nullptr;
  }
  g->stream = g->own_stream;
  g->close_stream();
  delete g;
  return KRK_SUCCESS;
}

int32_t krk_dense_group_sync(krk_dense_group* g) {
  if (!g) return KRK_E_ARGUMENT;
  KRK_TRY(ensure_runtime());
  DenseGroupLock lk(g);
  KRK_HIP(hipStreamSynchronize(g->stream));
  return KRK_SUCCESS;
}

int32_t krk_dense_group_size(krk_dense_group* g, int64_t* total) {
  if (!g || !total) return KRK_E_ARGUMENT;
  *total = g->total;
  return KRK_SUCCESS;
}

int32_t krk_dense_group_pull(krk_dense_group* g, float* out, uint32_t flags) {
  if (!g) return KRK_E_ARGUMENT;
  KRK_TRY(ensure_runtime());
  KRK_TRY(check_flags(flags));
  if (g->total > 0 && !out) return KRK_E_ARGUMENT;
  DenseGroupLock lk(g);
  if (g->total == 0) return KRK_SUCCESS;
  float* d_out;
  KRK_TRY(g->output(out, (size_t)g->total, flags, 0, &d_out));
  for (size_t i = 0; i < g->tables.size();) {
    DenseGroupArgs a;
    a.members = 0;
    uint32_t blocks = 0;
    for (; i < g->tables.size() && a.members < kDenseGroupChunk; ++i) {
      krk_dense* t = g->tables[i];
      DenseMember& m = a.m[a.members];
      m = DenseMember{t->w, nullptr, nullptr, nullptr, t->n, g->start[i], 1.0f, 1.0f, 0};
      a.block_start[a.members++] = blocks;
      blocks += dense_member_blocks(t->n);
    }
    a.block_start[a.members] = blocks;
    hipLaunchKernelGGL(dense_group_pull_kernel, dim3(blocks), dim3(kDenseBlock), 0, g->stream, a, d_out);
    KRK_HIP(hipGetLastError());
  }
  KRK_TRY(g->output_back(out, (size_t)g->total, flags, 0));
  if (!(flags & KRK_ASYNC)) KRK_HIP(hipStreamSynchronize(g->stream));
  return KRK_SUCCESS;
}

int32_t krk_dense_group_push(krk_dense_group* g, const krk_optim* o, const float* grads, int64_t n, float lr,
                             uint32_t flags) {
  if (!g) return KRK_E_ARGUMENT;
  KRK_TRY(ensure_runtime());
  KRK_TRY(check_flags(flags));
  if (!o || o->type < KRK_ADAGRAD || o->type > KRK_SGD) return KRK_UNSUPPORTED_OPTIM;
  if (n < 0 || (n > 0 && !grads)) return KRK_E_ARGUMENT;
  DenseGroupLock lk(g);
  if (n != g->total) {   // every member's ps/optim/sgd.cc:36-39 at once
    set_error("gradients hold %lld elements, the group's tables %lld", (long long)n, (long long)g->total);
    return KRK_GRADIENT_UNCOMPATIBLE;
  }
  if (n == 0) return KRK_SUCCESS;
  if ((flags & KRK_DEVICE_PTRS) && ((uintptr_t)grads & 15)) {
    set_error("device gradients must be 16-byte aligned");
    return KRK_E_ARGUMENT;
  }
  const float* d_grads;
  KRK_TRY(g->input(grads, (size_t)n, flags, 0, &d_grads));
  const OptimK k = make_optim_k(*o);
  for (size_t i = 0; i < g->tables.size();) {
    DenseGroupArgs a;
    a.members = 0;
    uint32_t blocks = 0;
    for (; i < g->tables.size() && a.members < kDenseGroupChunk; ++i) {
      krk_dense* t = g->tables[i];
      if (t->n == 0) continue;
      DenseMember& m = a.m[a.members];
      KRK_TRY(dense_member(t, *o, &m));
      m.start = g->start[i];
      a.block_start[a.members++] = blocks;
      blocks += dense_member_blocks(t->n);
    }
    if (a.members == 0) continue;
    a.block_start[a.members] = blocks;
    const dim3 grid(blocks), block(kDenseBlock);
    switch (o->type) {
      case KRK_SGD:
        hipLaunchKernelGGL((dense_group_update_kernel<KRK_SGD>), grid, block, 0, g->stream, a, d_grads, lr, k);
        break;
      case KRK_ADAGRAD:
        hipLaunchKernelGGL((dense_group_update_kernel<KRK_ADAGRAD>), grid, block, 0, g->stream, a, d_grads, lr, k);
        break;
      case KRK_ADAM:
        hipLaunchKernelGGL((dense_group_update_kernel<KRK_ADAM>), grid, block, 0, g->stream, a, d_grads, lr, k);
        break;
      default:
        hipLaunchKernelGGL((dense_group_update_kernel<KRK_RMSPROP>), grid, block, 0, g->stream, a, d_grads, lr, k);
        break;
    }
    KRK_HIP(hipGetLastError());
  }
  if (!(flags & KRK_ASYNC)) KRK_HIP(hipStreamSynchronize(g->stream));
  return KRK_SUCCESS;
}

int32_t krk_dense_steps(krk_dense* t, int64_t* steps) {
  if (!t || !steps) return KRK_E_ARGUMENT;
  std::lock_guard<std::mutex> lk(t->mu);
  *steps = t->steps;
  return KRK_SUCCESS;
}

}  // extern "C"
