/*
 * kraken_oracle.h -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A CPU restatement, in plain C, of the sparse/dense table hot path of
 * amazingyyc/Kraken. It exists only as the checker for the HIP path and as the
 * timed CPU baseline: nothing in the shipped library may call it. Only tests,
 * the smoke check and the benchmark's cpu_baseline leg load it.
 *
 * Every function names the reference file:line (relative to the reference
 * tree's kraken/ directory) whose behaviour it restates. The restatement keeps
 * the reference's cost structure on purpose: eight skip lists selected by
 * id % 8, one heap tensor per row and per optimizer state, and one heap
 * temporary per elementwise operation in the optimizer chains.
 *
 * Parity status of each group (what pins it is in the tests that load this):
 *   hash, skip list, routing ring, dedup, codec KATs, optimizers (closed
 *   forms + library optimizers), COO densify ............ pinned
 *   Normal/Uniform/Xavier row initialisers ............... parity unpinned:
 *     the reference seeds a fresh mt19937 from std::random_device on every
 *     call (t/math.cc:455-464, 486-495), so no reproducible output exists.
 *     The oracle defines a counter-based generator instead (kro_init_row) and
 *     only its distribution moments can be compared with the reference.
 *   Adam AMSGrad branch (bias-corrected max, unlike torch)  pinned by closed
 *     forms: an impulse gradient (the maximum keeps the first, exact value;
 *     weights follow sum 1/(2^t - 1)), doubling gradients (the maximum is
 *     always the newest value: plain Adam, which torch pins), a constant
 *     gradient and a single step (both reduce to torch's AMSGrad).
 */
#ifndef KRAKEN_ORACLE_H_
#define KRAKEN_ORACLE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* common/error_code.h:7-33 */
enum {
  KRO_SUCCESS = 0,
  KRO_UNSUPPORTED_OPTIM = 6,
  KRO_INTERFACE_UNIMPLEMENTED = 10,
  KRO_GRADIENT_UNCOMPATIBLE = 11,
  KRO_SPARSE_ID_NOT_EXIST = 12,
  KRO_UNSUPPORTED_INITIALIZER = 13
};

/* common/info.h:46-72 */
enum { KRO_ADAGRAD = 0, KRO_ADAM = 1, KRO_RMSPROP = 2, KRO_SGD = 3 };
enum {
  KRO_INIT_CONSTANT = 0,
  KRO_INIT_UNIFORM = 1,
  KRO_INIT_NORMAL = 2,
  KRO_INIT_XAVIER_UNIFORM = 3,
  KRO_INIT_XAVIER_NORMAL = 4
};
enum {
  KRO_ST_STEPS = 0,
  KRO_ST_MOMENTUM_BUFFER = 1,
  KRO_ST_STATE_SUM = 2,
  KRO_ST_FIRST_MOMENT = 3,
  KRO_ST_SECOND_MOMENT = 4,
  KRO_ST_SECOND_MOMENT_MAX = 5,
  KRO_ST_SQUARE_AVERAGE = 6,
  KRO_ST_G_AVE = 7,
  KRO_ST_COUNT = 8
};

/* Flattened result of Optim::Create (ps/optim/optim.cc:18-105). */
typedef struct kro_optim {
  int32_t type;
  int32_t has_weight_decay;
  float weight_decay;
  int32_t has_momentum;
  float momentum;
  int32_t has_dampening;
  float dampening;
  int32_t nesterov;
  float beta1;
  float beta2;
  float eps;
  int32_t amsgrad;
  float alpha;
  int32_t centered;
} kro_optim;

/* Flattened result of Initializer::Create (ps/initializer/initializer.cc:22-61).
 * a,b = value,- | lower,upper | mean,stddev | gain,- | gain,- */
typedef struct kro_init {
  int32_t type;
  float a;
  float b;
  uint64_t seed;
} kro_init;

/* ---- integer helpers ---------------------------------------------------- */
uint64_t kro_hash64(uint64_t v);                 /* common/utils.h:30-44 */
uint64_t kro_hash64_pair(uint64_t a, uint64_t b);/* common/utils.h:46-48 */
/* common/router.cc:262-277; ring_hash ascending, m virtual nodes */
uint64_t kro_ring_hit(const uint64_t* ring_hash, const uint64_t* ring_node, int64_t m, uint64_t hv);
/* ps/ps.cc:100, 306 : Router::Hit(utils::Hash(table_id, sparse_id)) */
uint64_t kro_route_owner(const uint64_t* ring_hash, const uint64_t* ring_node, int64_t m,
                         uint64_t table_id, uint64_t id);
uint64_t kro_hit_slot(uint64_t id);              /* common/parallel_skip_list.h:12-21,100-102 */
uint64_t kro_splitmix64(uint64_t x);             /* harness generator, no reference counterpart */

/* ---- optimizers ---------------------------------------------------------- */
void kro_optim_defaults(int32_t type, kro_optim* o); /* ps/optim/optim.cc:23-101 */

typedef struct kro_value kro_value;                  /* common/info.h:74-92 */
kro_value* kro_value_create(const float* val, int64_t n);
void kro_value_destroy(kro_value* v);
const float* kro_value_val(const kro_value* v);
/* NULL when the state has not been created yet (lazy creation). */
const float* kro_value_state(const kro_value* v, int32_t state_type);
int64_t kro_value_steps(const kro_value* v);
/* ps/optim/{sgd,adagrad,adam,rmsprop}.cc ::Update on a dense gradient. */
int32_t kro_optim_update(const kro_optim* o, const float* grad, int64_t n,
                         float lr, kro_value* v);

/* ---- row initialisers ---------------------------------------------------- */
/* Constant is exact (t/math.cc:333-362); the random ones follow this
 * repository's counter-based definition keyed by (seed, id, element). */
void kro_init_row(const kro_init* init, uint64_t id, int64_t dim, float* out);
float kro_xavier_std(float gain, int64_t dim);     /* t/math.cc:24-50,476-484 */
/* The two elementary functions inside the normal draw, written out as part of the definition. */
double kro_log_u24(uint32_t k);                                /* log(k / 2^24), k in [1, 2^24] */
void kro_sincos_u24(uint32_t j, double* sn, double* cs);       /* of 2 pi j / 2^24, j in [0, 2^24) */

/* ---- sparse table -------------------------------------------------------- */
typedef struct kro_sparse kro_sparse;
kro_sparse* kro_sparse_create(int64_t dim, const kro_init* init);
void kro_sparse_destroy(kro_sparse* t);
int64_t kro_sparse_size(const kro_sparse* t);
/* ps/sparse_table.cc:33-75 : insert-on-miss, copy rows out as [n, dim]. */
int32_t kro_sparse_pull(kro_sparse* t, const uint64_t* ids, int64_t n, float* out);
/* ps/sparse_table.cc:77-108 : stops at the first missing id (code 12), rows
 * visited before it stay updated. grad_dim != dim gives code 11. */
int32_t kro_sparse_push(kro_sparse* t, const kro_optim* o, const uint64_t* ids,
                        int64_t n, const float* grads, int64_t grad_dim, float lr);
/* Bulk load used by harnesses: rows given explicitly (skip list Insert). */
void kro_sparse_load(kro_sparse* t, const uint64_t* ids, int64_t n, const float* vals);
/* Export in slot-major, key-ascending order (checkpoint order,
 * checkpoint/checkpoint.cc:465-509). state may be NULL; missing states read 0. */
int64_t kro_sparse_export(const kro_sparse* t, uint64_t* ids, float* vals,
                          int32_t state_type, float* state, int64_t* steps);
/* 1 if id is present. */
int32_t kro_sparse_contains(const kro_sparse* t, uint64_t id);
/* ps/ps.cc:92-109 with common/skip_list.h:336-359 : remove the listed ids; returns how many
 * were present. */
int64_t kro_sparse_erase(kro_sparse* t, const uint64_t* ids, int64_t n);
/* ps/ps.cc:914-935 : values of the ids that exist, nothing inserted. Returns the hits. */
int64_t kro_sparse_fetch(const kro_sparse* t, const uint64_t* ids, int64_t n, uint8_t* found,
                         float* vals);
/* Thread-safe variants that take the per-slot lock like the reference does;
 * used by the multi-threaded CPU baseline. */
int32_t kro_sparse_pull_mt(kro_sparse* t, const uint64_t* ids, int64_t n, float* out);
int32_t kro_sparse_push_mt(kro_sparse* t, const kro_optim* o, const uint64_t* ids,
                           int64_t n, const float* grads, int64_t grad_dim, float lr);

/* ---- dense table --------------------------------------------------------- */
typedef struct kro_dense kro_dense;
kro_dense* kro_dense_create(const float* val, int64_t n);   /* ps/dense_table.cc:10-13 */
void kro_dense_destroy(kro_dense* t);
int32_t kro_dense_pull(kro_dense* t, float* out);           /* ps/dense_table.cc:31-37 */
int32_t kro_dense_push(kro_dense* t, const kro_optim* o, const float* grad,
                       int64_t n, float lr);                /* ps/dense_table.cc:39-43 */
/* COO gradient: empty => success without touching anything
 * (ps/optim/adam.cc:25-32), else densify then update. */
int32_t kro_dense_push_coo(kro_dense* t, const kro_optim* o, const int64_t* idx,
                           const float* val, int64_t nnz, float lr);
const kro_value* kro_dense_value(const kro_dense* t);

/* ---- worker-side dedup --------------------------------------------------- */
/* worker/emitter.cc:131-149 : unique ids in first-occurrence order and the
 * position -> unique-index map. Returns U. */
int64_t kro_dedup(const uint64_t* ids, int64_t n, uint64_t* uids, int64_t* inv);
/* worker/emitter.cc:510-531 : same order, duplicate gradient rows summed in
 * position order starting from a copy of the first. Returns U. */
int64_t kro_dedup_sum(const uint64_t* ids, int64_t n, const float* grads,
                      int64_t dim, uint64_t* uids, float* out);

/* ---- jagged (multi-hot) pooling ------------------------------------------- */
/* pytorch/py/jagged_ops.cc:14-56 : out[i] = v[offsets[i]] copied, then the bag's other
 * rows added in position order; an empty bag gets patch_value. v [rows, col], out [k, col]. */
void kro_jagged_sum_forward(const float* v, int64_t col, const int64_t* offsets, int64_t k,
                            float patch_value, float* out);
/* pytorch/py/jagged_ops.cc:206-236 : the sum, then times (float)(1.0 / float(len)). */
void kro_jagged_mean_forward(const float* v, int64_t col, const int64_t* offsets, int64_t k,
                             float patch_value, float* out);
/* Derivative of the sum: every row of bag i receives grads[i]. This is NOT what
 * pytorch/py/jagged_ops.cc:148-160 does: its destination pointer never advances, so only
 * the first row of a bag is written and the others stay uninitialised. The intended
 * semantics (the transpose of the forward) is what is stated here. */
void kro_jagged_sum_backward(const int64_t* offsets, int64_t k, const float* grads, int64_t col,
                             float* vgrads);
/* pytorch/py/jagged_ops.cc:303-334 : every row of bag i receives grads[i] * ratio. */
void kro_jagged_mean_backward(const int64_t* offsets, int64_t k, const float* grads, int64_t col,
                              float* vgrads);

/* ---- threshold ("DCT") codec --------------------------------------------- */
void kro_abs(const float* x, float* y, int64_t n);            /* t/math.cc:540-546 */
/* t/math.cc:564-626 with t_num workers: chunk stride n / t_num, elements past
 * t_num*stride are never examined. y receives k values, descending. */
void kro_topk_chunked(const float* x, int64_t n, float* y, int64_t k, int64_t t_num);
/* t_num as the reference derives it: min(n / k, hw_threads). */
void kro_topk(const float* x, int64_t n, float* y, int64_t k, int64_t hw_threads);
/* True k-th largest of |x| (what the GPU path defines as tau). */
float kro_kth_largest_abs(const float* x, int64_t n, int64_t k);
/* t/tensor_impl.cc:521-560, t/math.cc:804-852,719-746 : indices ascending. */
int64_t kro_to_coo(const float* x, int64_t n, float th, int64_t* idx, float* val);
void kro_lt_keep(const float* x, float th, float* y, int64_t n); /* t/math.cc:1098-1123 */
/* t/math.cc:1006-1046 via t/coo_tensor_impl.cc:250-260 (1-D case). */
void kro_coo_to_dense(const int64_t* idx, const float* val, int64_t nnz,
                      float* dense, int64_t n);
void kro_take(const float* x, const int64_t* idx, float* y, int64_t k); /* t/math.cc:719-746 */

typedef struct kro_dct kro_dct;                               /* worker/dct_emitter.cc:12-14 */
kro_dct* kro_dct_create(int64_t n);
void kro_dct_destroy(kro_dct* s);
/* worker/dct_emitter.cc:16-43. Returns nnz, or -1 when n < 256 (gradient is
 * passed through dense and no state changes). exact_select != 0 replaces the
 * chunked TopK by the true k-th largest. */
int64_t kro_dct_compress(kro_dct* s, const float* grad, uint64_t life_span,
                         float eta, int64_t hw_threads, int32_t exact_select,
                         int64_t* idx, float* val);
float kro_dct_tau(const kro_dct* s);
const float* kro_dct_residual(const kro_dct* s);
uint64_t kro_dct_step(const kro_dct* s);

#ifdef __cplusplus
}
#endif
#endif /* KRAKEN_ORACLE_H_ */
