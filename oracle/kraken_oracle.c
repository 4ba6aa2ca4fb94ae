/*
 * kraken_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE (see kraken_oracle.h).
 *
 * Plain-C restatement of Kraken's CPU table path. File:line citations are
 * relative to the reference tree's kraken/ directory.
 */
#include "kraken_oracle.h"

#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

/* ========================================================================== */
/* integer helpers                                                            */
/* ========================================================================== */

/* common/utils.h:30-44 -- 64-bit mixer used for routing. */
uint64_t kro_hash64(uint64_t v) {
  v = v * 3935559000370003845ULL + 2691343689449507681ULL;
  v ^= v >> 21;
  v ^= v << 37;
  v ^= v >> 4;
  v *= 4768777513237032717ULL;
  v ^= v << 20;
  v ^= v >> 41;
  v ^= v << 5;
  return v;
}

/* common/utils.h:46-48 */
uint64_t kro_hash64_pair(uint64_t a, uint64_t b) {
  return kro_hash64(a) ^ kro_hash64(b);
}

/* common/router.cc:262-277 (Router::Hit): the ring is the virtual nodes in ascending hash
 * order; a hash belongs to the first virtual node at or above it, or to the first of the ring
 * when it lies above them all. An empty ring owns nothing (uint64 -1). */
uint64_t kro_ring_hit(const uint64_t* ring_hash, const uint64_t* ring_node, int64_t m, uint64_t hv) {
  if (m <= 0) return UINT64_MAX;
  int64_t lo = 0, hi = m;                        /* std::lower_bound */
  while (lo < hi) {
    int64_t mid = lo + (hi - lo) / 2;
    if (ring_hash[mid] < hv) lo = mid + 1; else hi = mid;
  }
  return ring_node[lo == m ? 0 : lo];
}

/* ps/ps.cc:100, 306: who owns row `id` of table `table_id` */
uint64_t kro_route_owner(const uint64_t* ring_hash, const uint64_t* ring_node, int64_t m,
                         uint64_t table_id, uint64_t id) {
  return kro_ring_hit(ring_hash, ring_node, m, kro_hash64_pair(table_id, id));
}

/* common/parallel_skip_list.h:12-21 (identity hash, 8 slots), :100-102 */
#define KRO_SLOTS 8
uint64_t kro_hit_slot(uint64_t id) { return id % KRO_SLOTS; }

/* Steele/Lea/Flood splitmix64 output function applied to x + golden gamma.
 * Shared by the harness generators and the row initialisers; no reference
 * counterpart. */
uint64_t kro_splitmix64(uint64_t x) {
  uint64_t z = x + 0x9E3779B97F4A7C15ULL;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
  return z ^ (z >> 31);
}

/* ========================================================================== */
/* heap tensors and the unfused elementwise ops (t/tensor_impl.cc, t/math.cc) */
/* ========================================================================== */

typedef struct tens {
  float* p;
  int64_t n;
} tens;

/* t/tensor_impl.cc:28-34 + t/storage.cc:33-39: one allocation for the handle,
 * one for the storage. */
static tens* t_new(int64_t n) {
  tens* t = (tens*)malloc(sizeof(tens));
  t->n = n;
  t->p = (float*)malloc(sizeof(float) * (size_t)(n > 0 ? n : 1));
  return t;
}
static void t_free(tens* t) {
  if (t) {
    free(t->p);
    free(t);
  }
}
/* t/tensor_impl.cc:328-336 */
static tens* t_clone(const tens* x) {
  tens* y = t_new(x->n);
  memcpy(y->p, x->p, sizeof(float) * (size_t)x->n);
  return y;
}
static tens* t_from(const float* p, int64_t n) {
  tens* y = t_new(n);
  memcpy(y->p, p, sizeof(float) * (size_t)n);
  return y;
}
/* t/tensor_impl.cc:315-325 : Like().Zero() */
static tens* t_zeros(int64_t n) {
  tens* y = t_new(n);
  memset(y->p, 0, sizeof(float) * (size_t)n);
  return y;
}

/* t/math.cc:69-76 */
static void m_add(const float* x, const float* y, float* z, int64_t n) {
  for (int64_t i = 0; i < n; ++i) z[i] = x[i] + y[i];
}
/* t/math.cc:122-130 */
static void m_sub(const float* x, const float* y, float* z, int64_t n) {
  for (int64_t i = 0; i < n; ++i) z[i] = x[i] - y[i];
}
/* t/math.cc:198-206 */
static void m_mul(const float* x, const float* y, float* z, int64_t n) {
  for (int64_t i = 0; i < n; ++i) z[i] = x[i] * y[i];
}
/* t/math.cc:254-262 */
static void m_div(const float* x, const float* y, float* z, int64_t n) {
  for (int64_t i = 0; i < n; ++i) z[i] = x[i] / y[i];
}
/* t/math.cc:98-104 : v + x */
static void m_adds(float v, const float* x, float* y, int64_t n) {
  for (int64_t i = 0; i < n; ++i) y[i] = v + x[i];
}
/* t/math.cc:229-235 : v * x */
static void m_muls(float v, const float* x, float* y, int64_t n) {
  for (int64_t i = 0; i < n; ++i) y[i] = v * x[i];
}
/* t/math.cc:308-314 : x / v (true division) */
static void m_divs(const float* x, float v, float* y, int64_t n) {
  for (int64_t i = 0; i < n; ++i) y[i] = x[i] / v;
}
/* t/math.cc:364-370 */
static void m_sqrt(const float* x, float* y, int64_t n) {
  for (int64_t i = 0; i < n; ++i) y[i] = sqrtf(x[i]);
}
/* t/math.cc:388-395 */
static void m_max(const float* x, const float* y, float* z, int64_t n) {
  for (int64_t i = 0; i < n; ++i) z[i] = x[i] > y[i] ? x[i] : y[i];
}

/* Out-of-place Tensor operators: each allocates its result like
 * t/tensor_impl.cc:110-164, 214-248 do. */
static tens* o_add(const tens* a, const tens* b) { tens* r = t_new(a->n); m_add(a->p, b->p, r->p, a->n); return r; }
static tens* o_sub(const tens* a, const tens* b) { tens* r = t_new(a->n); m_sub(a->p, b->p, r->p, a->n); return r; }
static tens* o_div(const tens* a, const tens* b) { tens* r = t_new(a->n); m_div(a->p, b->p, r->p, a->n); return r; }
static tens* o_adds(const tens* a, float v) { tens* r = t_new(a->n); m_adds(v, a->p, r->p, a->n); return r; }
static tens* o_muls(const tens* a, float v) { tens* r = t_new(a->n); m_muls(v, a->p, r->p, a->n); return r; }
static tens* o_divs(const tens* a, float v) { tens* r = t_new(a->n); m_divs(a->p, v, r->p, a->n); return r; }
/* t/tensor_impl.cc:346-354 : Square(false) == Mul(*this) */
static tens* o_square(const tens* a) { tens* r = t_new(a->n); m_mul(a->p, a->p, r->p, a->n); return r; }
/* t/tensor_impl.cc:356-369 */
static tens* o_sqrt(const tens* a) { tens* r = t_new(a->n); m_sqrt(a->p, r->p, a->n); return r; }
static tens* o_max(const tens* a, const tens* b) { tens* r = t_new(a->n); m_max(a->p, b->p, r->p, a->n); return r; }
/* In-place forms, t/tensor_impl.cc:166-188 */
static void i_add(tens* a, const tens* b) { m_add(a->p, b->p, a->p, a->n); }
static void i_sub(tens* a, const tens* b) { m_sub(a->p, b->p, a->p, a->n); }

/* ========================================================================== */
/* Value and the optimizers                                                   */
/* ========================================================================== */

/* common/info.h:74-92 */
struct kro_value {
  tens* val;
  tens* states[KRO_ST_COUNT];
  int64_t steps;
};

kro_value* kro_value_create(const float* val, int64_t n) {
  kro_value* v = (kro_value*)calloc(1, sizeof(kro_value));
  v->val = val ? t_from(val, n) : t_zeros(n);
  return v;
}
void kro_value_destroy(kro_value* v) {
  if (!v) return;
  t_free(v->val);
  for (int i = 0; i < KRO_ST_COUNT; ++i) t_free(v->states[i]);
  free(v);
}
const float* kro_value_val(const kro_value* v) { return v->val->p; }
const float* kro_value_state(const kro_value* v, int32_t st) {
  if (st < 0 || st >= KRO_ST_COUNT || !v->states[st]) return NULL;
  return v->states[st]->p;
}
int64_t kro_value_steps(const kro_value* v) { return v->steps; }

/* ps/optim/optim.cc:23-101 : defaults before the conf map is applied. */
void kro_optim_defaults(int32_t type, kro_optim* o) {
  memset(o, 0, sizeof(*o));
  o->type = type;
  o->beta1 = 0.9f;
  o->beta2 = 0.999f;
  o->alpha = 0.99f;
  if (type == KRO_ADAGRAD) {
    o->eps = 1e-10f;
  } else {
    o->eps = 1e-8f;
  }
}

static void swap_state(kro_value* v, int st, tens* nt) {
  t_free(v->states[st]);
  v->states[st] = nt;
}

/* ps/optim/sgd.cc:25-63 */
static int32_t sgd_update(const kro_optim* o, tens* g, float lr, kro_value* v) {
  if (o->has_weight_decay) {          /* :41-43  g += wd * w */
    tens* t = o_muls(v->val, o->weight_decay);
    i_add(g, t);
    t_free(t);
  }
  tens* step = g;
  tens* owned = NULL;
  if (o->has_momentum) {
    if (!v->states[KRO_ST_MOMENTUM_BUFFER]) {   /* :46-47 first time: clone */
      v->states[KRO_ST_MOMENTUM_BUFFER] = t_clone(g);
    } else {                                    /* :49-50 */
      tens* a = o_muls(v->states[KRO_ST_MOMENTUM_BUFFER], o->momentum);
      tens* b = o_muls(g, (float)(1.0 - (double)o->dampening));
      tens* nb = o_add(a, b);
      t_free(a);
      t_free(b);
      swap_state(v, KRO_ST_MOMENTUM_BUFFER, nb);
    }
    if (o->nesterov) {                          /* :53-54 */
      tens* t = o_muls(v->states[KRO_ST_MOMENTUM_BUFFER], o->momentum);
      i_add(g, t);
      t_free(t);
    } else {                                    /* :56 */
      step = v->states[KRO_ST_MOMENTUM_BUFFER];
    }
  }
  owned = o_muls(step, lr);                     /* :60  w -= g * lr */
  i_sub(v->val, owned);
  t_free(owned);
  return KRO_SUCCESS;
}

/* ps/optim/adagrad.cc:18-48 */
static int32_t adagrad_update(const kro_optim* o, tens* g, float lr, kro_value* v) {
  if (!v->states[KRO_ST_STATE_SUM]) v->states[KRO_ST_STATE_SUM] = t_zeros(g->n); /* :34-36 */
  if (o->has_weight_decay) {                    /* :38-40 */
    tens* t = o_muls(v->val, o->weight_decay);
    i_add(g, t);
    t_free(t);
  }
  tens* sum = v->states[KRO_ST_STATE_SUM];
  tens* sq = o_square(g);                       /* :43 */
  i_add(sum, sq);
  t_free(sq);
  tens* rt = o_sqrt(sum);                       /* :45 */
  tens* den = o_adds(rt, o->eps);
  tens* q = o_div(g, den);
  tens* upd = o_muls(q, lr);
  i_sub(v->val, upd);
  t_free(rt);
  t_free(den);
  t_free(q);
  t_free(upd);
  return KRO_SUCCESS;
}

/* ps/optim/adam.cc:23-81 */
static int32_t adam_update(const kro_optim* o, tens* g, float lr, kro_value* v) {
  if (!v->states[KRO_ST_FIRST_MOMENT]) v->states[KRO_ST_FIRST_MOMENT] = t_zeros(g->n);   /* :41-43 */
  if (!v->states[KRO_ST_SECOND_MOMENT]) v->states[KRO_ST_SECOND_MOMENT] = t_zeros(g->n); /* :45-47 */
  if (o->has_weight_decay) {                    /* :50-52 */
    tens* t = o_muls(v->val, o->weight_decay);
    i_add(g, t);
    t_free(t);
  }
  {                                             /* :57 */
    tens* a = o_muls(v->states[KRO_ST_FIRST_MOMENT], o->beta1);
    tens* b = o_muls(g, (float)(1.0 - (double)o->beta1));
    swap_state(v, KRO_ST_FIRST_MOMENT, o_add(a, b));
    t_free(a);
    t_free(b);
  }
  {                                             /* :58 */
    tens* a = o_muls(v->states[KRO_ST_SECOND_MOMENT], o->beta2);
    tens* sq = o_square(g);
    tens* b = o_muls(sq, (float)(1.0 - (double)o->beta2));
    swap_state(v, KRO_ST_SECOND_MOMENT, o_add(a, b));
    t_free(a);
    t_free(sq);
    t_free(b);
  }
  int64_t steps = ++v->steps;                   /* :61 */
  /* :63-64 : std::pow(float, float) is the float overload; 1.0 - it is double,
   * narrowed to float by the Tensor/float operator. */
  float c1 = (float)(1.0 - (double)powf(o->beta1, (float)steps));
  float c2 = (float)(1.0 - (double)powf(o->beta2, (float)steps));
  tens* mt = o_divs(v->states[KRO_ST_FIRST_MOMENT], c1);
  tens* vt = o_divs(v->states[KRO_ST_SECOND_MOMENT], c2);
  tens* num = o_muls(mt, lr);                   /* lr * mt */
  tens* den;
  if (o->amsgrad) {                             /* :66-75 */
    if (!v->states[KRO_ST_SECOND_MOMENT_MAX]) v->states[KRO_ST_SECOND_MOMENT_MAX] = t_zeros(g->n);
    swap_state(v, KRO_ST_SECOND_MOMENT_MAX, o_max(v->states[KRO_ST_SECOND_MOMENT_MAX], vt));
    tens* rt = o_sqrt(v->states[KRO_ST_SECOND_MOMENT_MAX]);
    den = o_adds(rt, o->eps);
    t_free(rt);
  } else {                                      /* :77 : Sqrt(true) in place */
    m_sqrt(vt->p, vt->p, vt->n);
    den = o_adds(vt, o->eps);
  }
  tens* upd = o_div(num, den);
  i_sub(v->val, upd);
  t_free(mt);
  t_free(vt);
  t_free(num);
  t_free(den);
  t_free(upd);
  return KRO_SUCCESS;
}

/* ps/optim/rmsprop.cc:23-78 */
static int32_t rmsprop_update(const kro_optim* o, tens* g, float lr, kro_value* v) {
  if (o->has_weight_decay) {                    /* :39-41 */
    tens* t = o_muls(v->val, o->weight_decay);
    i_add(g, t);
    t_free(t);
  }
  if (!v->states[KRO_ST_SQUARE_AVERAGE]) v->states[KRO_ST_SQUARE_AVERAGE] = t_zeros(g->n); /* :43-45 */
  float om = (float)(1.0 - (double)o->alpha);
  {                                             /* :47-51 */
    tens* a = o_muls(v->states[KRO_ST_SQUARE_AVERAGE], o->alpha);
    tens* sq = o_square(g);
    tens* b = o_muls(sq, om);
    swap_state(v, KRO_ST_SQUARE_AVERAGE, o_add(a, b));
    t_free(a);
    t_free(sq);
    t_free(b);
  }
  tens* d = v->states[KRO_ST_SQUARE_AVERAGE];
  tens* d_owned = NULL;
  if (o->centered) {                            /* :53-62 */
    if (!v->states[KRO_ST_G_AVE]) v->states[KRO_ST_G_AVE] = t_zeros(g->n);
    tens* a = o_muls(v->states[KRO_ST_G_AVE], o->alpha);
    tens* b = o_muls(g, om);
    swap_state(v, KRO_ST_G_AVE, o_add(a, b));
    t_free(a);
    t_free(b);
    tens* gs = o_square(v->states[KRO_ST_G_AVE]);
    d_owned = o_sub(d, gs);
    t_free(gs);
    d = d_owned;
  }
  tens* rt = o_sqrt(d);
  tens* den = o_adds(rt, o->eps);
  if (o->has_momentum) {                        /* :64-72 */
    if (!v->states[KRO_ST_MOMENTUM_BUFFER]) v->states[KRO_ST_MOMENTUM_BUFFER] = t_zeros(g->n);
    tens* a = o_muls(v->states[KRO_ST_MOMENTUM_BUFFER], o->momentum);
    tens* q = o_div(g, den);
    swap_state(v, KRO_ST_MOMENTUM_BUFFER, o_add(a, q));
    t_free(a);
    t_free(q);
    tens* upd = o_muls(v->states[KRO_ST_MOMENTUM_BUFFER], lr);
    i_sub(v->val, upd);
    t_free(upd);
  } else {                                      /* :74 : (lr * g) / (sqrt(d) + eps) */
    tens* num = o_muls(g, lr);
    tens* upd = o_div(num, den);
    i_sub(v->val, upd);
    t_free(num);
    t_free(upd);
  }
  t_free(rt);
  t_free(den);
  t_free(d_owned);
  return KRO_SUCCESS;
}

/* Common prologue of every ::Update (size check, e.g. ps/optim/adagrad.cc:29-32).
 * The gradient is copied because weight decay mutates the aliased request
 * buffer in the reference (ps/optim/sgd.cc:27,42); callers here pass const. */
int32_t kro_optim_update(const kro_optim* o, const float* grad, int64_t n, float lr,
                         kro_value* v) {
  if (n != v->val->n) return KRO_GRADIENT_UNCOMPATIBLE;
  tens* g = t_from(grad, n);
  int32_t rc;
  switch (o->type) {
    case KRO_SGD: rc = sgd_update(o, g, lr, v); break;
    case KRO_ADAGRAD: rc = adagrad_update(o, g, lr, v); break;
    case KRO_ADAM: rc = adam_update(o, g, lr, v); break;
    case KRO_RMSPROP: rc = rmsprop_update(o, g, lr, v); break;
    default: rc = KRO_UNSUPPORTED_OPTIM; break;
  }
  t_free(g);
  return rc;
}

/* ========================================================================== */
/* row initialisers                                                           */
/* ========================================================================== */

/* t/math.cc:24-50 : a 1-D [dim] tensor has fan_out = dim, fan_in = 1;
 * t/math.cc:476-484 : std = gain * sqrt(2.0 / float(fan_in + fan_out)). */
float kro_xavier_std(float gain, int64_t dim) {
  return (float)((double)gain * sqrt(2.0 / (double)(float)(1 + dim)));
}

static uint64_t row_key(uint64_t seed, uint64_t id) {
  return kro_splitmix64(id ^ kro_splitmix64(seed));
}
static uint64_t elem_bits(uint64_t key, int64_t j) {
  return kro_splitmix64(key + (uint64_t)j * 0x9E3779B97F4A7C15ULL);
}
static float draw_uniform(uint64_t r, float lower, float upper) {
  double u = (double)(r >> 40) * (1.0 / 16777216.0);
  return (float)((double)lower + ((double)upper - (double)lower) * u);
}
/* Elements 2q and 2q + 1 of a row are the two values of one Box-Muller step on the bits drawn
 * for q: k = upper 24 bits + 1 gives the radius sqrt(-2 log(k / 2^24)), j = the next 24 bits the
 * angle 2 pi j / 2^24; the values are radius * cos(angle) and radius * sin(angle).
 *
 * The logarithm and the sine / cosine are part of the definition: they are written out below in
 * double-precision +, -, *, / (this file is compiled without contraction), so that every
 * implementation of the definition evaluates the same IEEE operations in the same order and
 * agrees to the bit. Both are exact in their argument reduction because their arguments are
 * 24-bit fractions, and accurate to a few 1e-14 (tests/test_oracle_pins.py holds them against
 * libm). */
double kro_log_u24(uint32_t k) {                      /* log(k / 2^24), k in [1, 2^24] */
  int e = 31 - __builtin_clz(k);
  double m = (double)k * (1.0 / (double)(1u << e));   /* exact, in [1, 2) */
  if (m > 1.4142135623730951) {
    m = m * 0.5;
    e = e + 1;
  }
  /* log m = 2 atanh f, f = (m - 1) / (m + 1), |f| <= 0.1716: eight terms of the series */
  const double f = (m - 1.0) / (m + 1.0);
  const double z = f * f;
  double p = 0.066666666666666666;                    /* 1/15 */
  p = p * z + 0.076923076923076927;                   /* 1/13 */
  p = p * z + 0.090909090909090912;                   /* 1/11 */
  p = p * z + 0.11111111111111111;                    /* 1/9 */
  p = p * z + 0.14285714285714285;                    /* 1/7 */
  p = p * z + 0.2;                                    /* 1/5 */
  p = p * z + 0.33333333333333331;                    /* 1/3 */
  p = p * z + 1.0;
  return 2.0 * f * p + (double)(e - 24) * 0.69314718055994529;
}

void kro_sincos_u24(uint32_t j, double* sn, double* cs) {   /* of 2 pi j / 2^24, j in [0, 2^24) */
  /* the nearest quarter turn comes off in integers; the rest is at most pi/4 either way */
  const int32_t quarter = (int32_t)((j + (1u << 21)) >> 22);
  const int32_t rest = (int32_t)j - (int32_t)((uint32_t)quarter << 22);
  const double t = (double)rest * 3.7450702829239286e-07;      /* 2 pi / 2^24 */
  const double z = t * t;
  double s = 1.6059043836821613e-10;                  /* Taylor: 1/13! */
  s = s * z - 2.505210838544172e-08;                  /* 1/11! */
  s = s * z + 2.7557319223985893e-06;                 /* 1/9! */
  s = s * z - 0.00019841269841269841;                 /* 1/7! */
  s = s * z + 0.0083333333333333332;                  /* 1/5! */
  s = s * z - 0.16666666666666666;                    /* 1/3! */
  s = s * z + 1.0;
  s = s * t;
  double c = -1.1470745597729725e-11;                 /* 1/14! */
  c = c * z + 2.08767569878681e-09;                   /* 1/12! */
  c = c * z - 2.7557319223985888e-07;                 /* 1/10! */
  c = c * z + 2.4801587301587302e-05;                 /* 1/8! */
  c = c * z - 0.0013888888888888889;                  /* 1/6! */
  c = c * z + 0.041666666666666664;                   /* 1/4! */
  c = c * z - 0.5;
  c = c * z + 1.0;
  switch (quarter & 3) {
    case 0: *sn = s; *cs = c; break;
    case 1: *sn = c; *cs = -s; break;
    case 2: *sn = -s; *cs = -c; break;
    default: *sn = -c; *cs = s; break;
  }
}

static float draw_normal(uint64_t key, int64_t j, float mean, float stddev) {
  uint64_t r = elem_bits(key, j >> 1);
  double radius = sqrt(-2.0 * kro_log_u24((uint32_t)(r >> 40) + 1u));
  double sn, cs;
  kro_sincos_u24((uint32_t)(r >> 16) & 0xFFFFFFu, &sn, &cs);
  double z = radius * ((j & 1) ? sn : cs);
  return (float)((double)mean + (double)stddev * z);
}

void kro_init_row(const kro_init* init, uint64_t id, int64_t dim, float* out) {
  uint64_t key = row_key(init->seed, id);
  switch (init->type) {
    case KRO_INIT_CONSTANT:                     /* t/math.cc:333-362 */
      for (int64_t j = 0; j < dim; ++j) out[j] = init->a;
      break;
    case KRO_INIT_UNIFORM:                      /* t/math.cc:486-505 (distribution only) */
      for (int64_t j = 0; j < dim; ++j) out[j] = draw_uniform(elem_bits(key, j), init->a, init->b);
      break;
    case KRO_INIT_NORMAL:                       /* t/math.cc:455-474 (distribution only) */
      for (int64_t j = 0; j < dim; ++j) out[j] = draw_normal(key, j, init->a, init->b);
      break;
    case KRO_INIT_XAVIER_UNIFORM: {             /* t/math.cc:507-517 */
      float std = kro_xavier_std(init->a, dim);
      float a = (float)(sqrt(3.0) * (double)std);
      for (int64_t j = 0; j < dim; ++j) out[j] = draw_uniform(elem_bits(key, j), -a, a);
      break;
    }
    case KRO_INIT_XAVIER_NORMAL: {              /* t/math.cc:476-484 */
      float std = kro_xavier_std(init->a, dim);
      for (int64_t j = 0; j < dim; ++j) out[j] = draw_normal(key, j, 0.0f, std);
      break;
    }
    default:
      for (int64_t j = 0; j < dim; ++j) out[j] = 0.0f;
  }
}

/* ========================================================================== */
/* skip list (common/skip_list.h) and the 8-slot table around it              */
/* ========================================================================== */

#define SL_MAX_HEIGHT 24 /* common/skip_list.h:14 */

typedef struct sl_node {
  uint64_t key;
  kro_value* value;
  struct sl_node* next[]; /* common/skip_list.h:18-22 : tower sized at allocation */
} sl_node;

typedef struct skiplist {
  sl_node* head;
  size_t max_height;
  uint64_t rng;
  size_t count;
} skiplist;

static sl_node* sl_new_node(size_t height) {
  sl_node* n = (sl_node*)malloc(sizeof(sl_node) + height * sizeof(sl_node*));
  n->key = 0;
  n->value = NULL;
  return n;
}
static void sl_init(skiplist* s, uint64_t seed) {
  s->head = sl_new_node(SL_MAX_HEIGHT);
  for (size_t i = 0; i < SL_MAX_HEIGHT; ++i) s->head->next[i] = NULL;
  s->max_height = 1;
  s->rng = kro_splitmix64(seed);
  s->count = 0;
}
/* common/skip_list.h:129-136 : grow while a draw from {0,1,2,3} is 0. */
static size_t sl_random_height(skiplist* s) {
  size_t h = 1;
  for (;;) {
    s->rng = s->rng * 6364136223846793005ULL + 1442695040888963407ULL;
    if (h < SL_MAX_HEIGHT && ((s->rng >> 33) & 3) == 0) {
      ++h;
    } else {
      break;
    }
  }
  return h;
}
/* common/skip_list.h:142-162 */
static sl_node* sl_find_ge(const skiplist* s, uint64_t key, sl_node** prev) {
  sl_node* x = s->head;
  size_t level = s->max_height - 1;
  for (;;) {
    sl_node* nx = x->next[level];
    if (nx != NULL && nx->key < key) {
      x = nx;
    } else {
      if (prev) prev[level] = x;
      if (level == 0) return nx;
      --level;
    }
  }
}
/* common/skip_list.h:315-324 */
static sl_node* sl_find(const skiplist* s, uint64_t key) {
  sl_node* prev[SL_MAX_HEIGHT]; /* the reference's Find fills an iterator's prev_ too */
  sl_node* x = sl_find_ge(s, key, prev);
  return (x != NULL && x->key == key) ? x : NULL;
}
/* common/skip_list.h:237-264 */
static int sl_insert(skiplist* s, uint64_t key, kro_value* value) {
  sl_node* prev[SL_MAX_HEIGHT];
  sl_node* x = sl_find_ge(s, key, prev);
  if (x != NULL && x->key == key) return 0;
  size_t h = sl_random_height(s);
  if (h > s->max_height) {
    for (size_t i = s->max_height; i < h; ++i) prev[i] = s->head;
    s->max_height = h;
  }
  x = sl_new_node(h);
  x->key = key;
  x->value = value;
  for (size_t i = 0; i < h; ++i) {
    x->next[i] = prev[i]->next[i];
    prev[i]->next[i] = x;
  }
  s->count++;
  return 1;
}
/* common/skip_list.h:336-359 : unlink the node on every level whose predecessor points at
 * it, then free it. */
static int sl_remove(skiplist* s, uint64_t key) {
  sl_node* prev[SL_MAX_HEIGHT];
  sl_node* x = sl_find_ge(s, key, prev);
  if (x == NULL || x->key != key) return 0;
  for (size_t i = 0; i < s->max_height; ++i) {
    if (prev[i]->next[i] == x) prev[i]->next[i] = x->next[i];
  }
  kro_value_destroy(x->value);
  free(x);
  s->count--;
  return 1;
}
static void sl_clear(skiplist* s) {
  sl_node* x = s->head->next[0];
  while (x) {
    sl_node* nx = x->next[0];
    kro_value_destroy(x->value);
    free(x);
    x = nx;
  }
  free(s->head);
}

/* ps/sparse_table.h:18-29 */
struct kro_sparse {
  int64_t dim;
  kro_init init;
  skiplist lists[KRO_SLOTS];
  pthread_rwlock_t locks[KRO_SLOTS];
};

kro_sparse* kro_sparse_create(int64_t dim, const kro_init* init) {
  kro_sparse* t = (kro_sparse*)calloc(1, sizeof(kro_sparse));
  t->dim = dim;
  t->init = *init;
  for (int s = 0; s < KRO_SLOTS; ++s) {
    sl_init(&t->lists[s], 0x5EEDULL + (uint64_t)s);
    pthread_rwlock_init(&t->locks[s], NULL);
  }
  return t;
}
void kro_sparse_destroy(kro_sparse* t) {
  if (!t) return;
  for (int s = 0; s < KRO_SLOTS; ++s) {
    sl_clear(&t->lists[s]);
    pthread_rwlock_destroy(&t->locks[s]);
  }
  free(t);
}
int64_t kro_sparse_size(const kro_sparse* t) {
  int64_t n = 0;
  for (int s = 0; s < KRO_SLOTS; ++s) n += (int64_t)t->lists[s].count;
  return n;
}
int32_t kro_sparse_contains(const kro_sparse* t, uint64_t id) {
  return sl_find(&t->lists[kro_hit_slot(id)], id) != NULL;
}

/* Per-slot position lists: the reference builds
 * unordered_map<slot, vector<position>> (ps/sparse_table.cc:39-44). */
typedef struct slot_buckets {
  int64_t* pos[KRO_SLOTS];
  int64_t cnt[KRO_SLOTS];
} slot_buckets;

static void bucket_ids(const uint64_t* ids, int64_t n, slot_buckets* b) {
  int64_t cap[KRO_SLOTS];
  for (int s = 0; s < KRO_SLOTS; ++s) {
    b->cnt[s] = 0;
    cap[s] = 16;
    b->pos[s] = (int64_t*)malloc(sizeof(int64_t) * (size_t)cap[s]);
  }
  for (int64_t i = 0; i < n; ++i) {
    int s = (int)kro_hit_slot(ids[i]);
    if (b->cnt[s] == cap[s]) {
      cap[s] *= 2;
      b->pos[s] = (int64_t*)realloc(b->pos[s], sizeof(int64_t) * (size_t)cap[s]);
    }
    b->pos[s][b->cnt[s]++] = i;
  }
}
static void bucket_free(slot_buckets* b) {
  for (int s = 0; s < KRO_SLOTS; ++s) free(b->pos[s]);
}

/* ps/sparse_table.cc:33-75 */
static int32_t sparse_pull_impl(kro_sparse* t, const uint64_t* ids, int64_t n, float* out,
                                int lock) {
  slot_buckets b;
  bucket_ids(ids, n, &b);
  for (int s = 0; s < KRO_SLOTS; ++s) {
    if (b.cnt[s] == 0) continue;
    if (lock) pthread_rwlock_wrlock(&t->locks[s]); /* :48 unique lock even for Pull */
    for (int64_t j = 0; j < b.cnt[s]; ++j) {
      int64_t i = b.pos[s][j];
      sl_node* node = sl_find(&t->lists[s], ids[i]);
      if (node) {                                   /* :55-57 hit: Clone */
        tens* c = t_clone(node->value->val);
        memcpy(out + i * t->dim, c->p, sizeof(float) * (size_t)t->dim);
        t_free(c);
      } else {                                      /* :59-69 miss: create, init, Clone, Insert */
        tens* row = t_new(t->dim);
        kro_init_row(&t->init, ids[i], t->dim, row->p);
        tens* c = t_clone(row);
        memcpy(out + i * t->dim, c->p, sizeof(float) * (size_t)t->dim);
        t_free(c);
        kro_value* v = (kro_value*)calloc(1, sizeof(kro_value));
        v->val = row;
        sl_insert(&t->lists[s], ids[i], v);
      }
    }
    if (lock) pthread_rwlock_unlock(&t->locks[s]);
  }
  bucket_free(&b);
  return KRO_SUCCESS;
}

/* ps/sparse_table.cc:77-108. Slots are visited in ascending order here; the
 * reference visits them in unordered_map order, which is unspecified, so which
 * rows are already updated when code 12 comes back is unspecified there too. */
static int32_t sparse_push_impl(kro_sparse* t, const kro_optim* o, const uint64_t* ids,
                                int64_t n, const float* grads, int64_t grad_dim, float lr,
                                int lock) {
  slot_buckets b;
  bucket_ids(ids, n, &b);
  int32_t rc = KRO_SUCCESS;
  for (int s = 0; s < KRO_SLOTS && rc == KRO_SUCCESS; ++s) {
    if (b.cnt[s] == 0) continue;
    if (lock) pthread_rwlock_wrlock(&t->locks[s]);
    for (int64_t j = 0; j < b.cnt[s]; ++j) {
      int64_t i = b.pos[s][j];
      sl_node* node = sl_find(&t->lists[s], ids[i]);
      if (!node) {                                  /* :96-98 */
        rc = KRO_SPARSE_ID_NOT_EXIST;
        break;
      }
      rc = kro_optim_update(o, grads + i * grad_dim, grad_dim, lr, node->value); /* :100 */
      if (rc != KRO_SUCCESS) break;
    }
    if (lock) pthread_rwlock_unlock(&t->locks[s]);
  }
  bucket_free(&b);
  return rc;
}

int32_t kro_sparse_pull(kro_sparse* t, const uint64_t* ids, int64_t n, float* out) {
  return sparse_pull_impl(t, ids, n, out, 0);
}
int32_t kro_sparse_push(kro_sparse* t, const kro_optim* o, const uint64_t* ids, int64_t n,
                        const float* grads, int64_t grad_dim, float lr) {
  return sparse_push_impl(t, o, ids, n, grads, grad_dim, lr, 0);
}
int32_t kro_sparse_pull_mt(kro_sparse* t, const uint64_t* ids, int64_t n, float* out) {
  return sparse_pull_impl(t, ids, n, out, 1);
}
int32_t kro_sparse_push_mt(kro_sparse* t, const kro_optim* o, const uint64_t* ids, int64_t n,
                           const float* grads, int64_t grad_dim, float lr) {
  return sparse_push_impl(t, o, ids, n, grads, grad_dim, lr, 1);
}

void kro_sparse_load(kro_sparse* t, const uint64_t* ids, int64_t n, const float* vals) {
  for (int64_t i = 0; i < n; ++i) {
    kro_value* v = kro_value_create(vals + i * t->dim, t->dim);
    if (!sl_insert(&t->lists[kro_hit_slot(ids[i])], ids[i], v)) kro_value_destroy(v);
  }
}

int64_t kro_sparse_export(const kro_sparse* t, uint64_t* ids, float* vals, int32_t state_type,
                          float* state, int64_t* steps) {
  int64_t k = 0;
  for (int s = 0; s < KRO_SLOTS; ++s) {
    for (sl_node* x = t->lists[s].head->next[0]; x; x = x->next[0], ++k) {
      if (ids) ids[k] = x->key;
      if (vals) memcpy(vals + k * t->dim, x->value->val->p, sizeof(float) * (size_t)t->dim);
      if (state) {
        const float* sp = kro_value_state(x->value, state_type);
        if (sp) {
          memcpy(state + k * t->dim, sp, sizeof(float) * (size_t)t->dim);
        } else {
          memset(state + k * t->dim, 0, sizeof(float) * (size_t)t->dim);
        }
      }
      if (steps) steps[k] = x->value->steps;
    }
  }
  return k;
}

/* ps/ps.cc:92-109 : the clean-up after a cluster change walks every slot under its unique
 * lock and removes the rows that are routed elsewhere. The routing decision is the caller's;
 * this removes the listed ids and returns how many were present. */
int64_t kro_sparse_erase(kro_sparse* t, const uint64_t* ids, int64_t n) {
  int64_t removed = 0;
  for (int64_t i = 0; i < n; ++i) removed += sl_remove(&t->lists[kro_hit_slot(ids[i])], ids[i]);
  return removed;
}

/* ps/ps.cc:914-935 (TryFetchSparseValues) : values of the ids that exist, nothing inserted.
 * found[i] = 1 and vals[i] filled where id i is present; other rows of vals are left alone. */
int64_t kro_sparse_fetch(const kro_sparse* t, const uint64_t* ids, int64_t n, uint8_t* found,
                         float* vals) {
  int64_t hits = 0;
  for (int64_t i = 0; i < n; ++i) {
    const sl_node* x = sl_find(&t->lists[kro_hit_slot(ids[i])], ids[i]);
    found[i] = x != NULL;
    if (x) {
      memcpy(vals + i * t->dim, x->value->val->p, sizeof(float) * (size_t)t->dim);
      ++hits;
    }
  }
  return hits;
}

/* ========================================================================== */
/* dense table (ps/dense_table.cc)                                            */
/* ========================================================================== */

struct kro_dense {
  kro_value* v;
  pthread_rwlock_t mu;
};

kro_dense* kro_dense_create(const float* val, int64_t n) {
  kro_dense* t = (kro_dense*)calloc(1, sizeof(kro_dense));
  t->v = kro_value_create(val, n);
  pthread_rwlock_init(&t->mu, NULL);
  return t;
}
void kro_dense_destroy(kro_dense* t) {
  if (!t) return;
  kro_value_destroy(t->v);
  pthread_rwlock_destroy(&t->mu);
  free(t);
}
const kro_value* kro_dense_value(const kro_dense* t) { return t->v; }

/* ps/dense_table.cc:31-37 */
int32_t kro_dense_pull(kro_dense* t, float* out) {
  pthread_rwlock_rdlock(&t->mu);
  tens* c = t_clone(t->v->val);
  memcpy(out, c->p, sizeof(float) * (size_t)c->n);
  t_free(c);
  pthread_rwlock_unlock(&t->mu);
  return KRO_SUCCESS;
}
/* ps/dense_table.cc:39-43 */
int32_t kro_dense_push(kro_dense* t, const kro_optim* o, const float* grad, int64_t n,
                       float lr) {
  pthread_rwlock_wrlock(&t->mu);
  int32_t rc = kro_optim_update(o, grad, n, lr, t->v);
  pthread_rwlock_unlock(&t->mu);
  return rc;
}
/* COO prologue shared by all optimizers, e.g. ps/optim/adam.cc:25-32. */
int32_t kro_dense_push_coo(kro_dense* t, const kro_optim* o, const int64_t* idx,
                           const float* val, int64_t nnz, float lr) {
  if (nnz == 0) return KRO_SUCCESS;
  int64_t n = t->v->val->n;
  tens* g = t_new(n);
  kro_coo_to_dense(idx, val, nnz, g->p, n);
  int32_t rc = kro_dense_push(t, o, g->p, n, lr);
  t_free(g);
  return rc;
}

/* ========================================================================== */
/* worker-side dedup (worker/emitter.cc)                                      */
/* ========================================================================== */

/* Stand-in for std::unordered_map<uint64_t, size_t>: open addressing. */
typedef struct idmap {
  uint64_t* keys;
  int64_t* vals;
  uint8_t* used;
  size_t cap;
} idmap;

static void idmap_init(idmap* m, int64_t n) {
  size_t cap = 16;
  while (cap < (size_t)n * 2 + 2) cap <<= 1;
  m->cap = cap;
  m->keys = (uint64_t*)malloc(sizeof(uint64_t) * cap);
  m->vals = (int64_t*)malloc(sizeof(int64_t) * cap);
  m->used = (uint8_t*)calloc(cap, 1);
}
static void idmap_free(idmap* m) {
  free(m->keys);
  free(m->vals);
  free(m->used);
}
/* Returns the stored value, or -1 after inserting (key -> val). */
static int64_t idmap_find_or_insert(idmap* m, uint64_t key, int64_t val) {
  size_t i = (size_t)kro_splitmix64(key) & (m->cap - 1);
  while (m->used[i]) {
    if (m->keys[i] == key) return m->vals[i];
    i = (i + 1) & (m->cap - 1);
  }
  m->used[i] = 1;
  m->keys[i] = key;
  m->vals[i] = val;
  return -1;
}

/* worker/emitter.cc:131-149 (ids), :162-182 (re-expansion uses the same map). */
int64_t kro_dedup(const uint64_t* ids, int64_t n, uint64_t* uids, int64_t* inv) {
  idmap m;
  idmap_init(&m, n);
  int64_t u = 0;
  for (int64_t i = 0; i < n; ++i) {
    int64_t at = idmap_find_or_insert(&m, ids[i], u);
    if (at < 0) {
      uids[u] = ids[i];
      at = u++;
    }
    if (inv) inv[i] = at;
  }
  idmap_free(&m);
  return u;
}

/* worker/emitter.cc:510-531 : first occurrence clones the row, later ones do
 * an in-place fp32 += in position order. */
int64_t kro_dedup_sum(const uint64_t* ids, int64_t n, const float* grads, int64_t dim,
                      uint64_t* uids, float* out) {
  idmap m;
  idmap_init(&m, n);
  int64_t u = 0;
  for (int64_t i = 0; i < n; ++i) {
    int64_t at = idmap_find_or_insert(&m, ids[i], u);
    if (at < 0) {
      uids[u] = ids[i];
      memcpy(out + u * dim, grads + i * dim, sizeof(float) * (size_t)dim);
      ++u;
    } else {
      m_add(out + at * dim, grads + i * dim, out + at * dim, dim);
    }
  }
  idmap_free(&m);
  return u;
}

/* ========================================================================== */
/* jagged pooling                                                             */
/* ========================================================================== */

/* pytorch/py/jagged_ops.cc:14-56 (the AVX2 variant :59-110 does the same fp32 adds) */
void kro_jagged_sum_forward(const float* v, int64_t col, const int64_t* offsets, int64_t k,
                            float patch_value, float* out) {
  for (int64_t i = 0; i < k; ++i) {
    float* o = out + i * col;
    if (offsets[i + 1] <= offsets[i]) {
      for (int64_t l = 0; l < col; ++l) o[l] = patch_value;
      continue;
    }
    memcpy(o, v + offsets[i] * col, sizeof(float) * (size_t)col);
    for (int64_t j = offsets[i] + 1; j < offsets[i + 1]; ++j) {
      const float* r = v + j * col;
      for (int64_t l = 0; l < col; ++l) o[l] += r[l];
    }
  }
}

/* pytorch/py/jagged_ops.cc:206-236 : `T ratio = 1.0 / T(len)` divides in double */
static float jagged_ratio(int64_t len) {
  return (float)(1.0 / (double)(float)len);
}

void kro_jagged_mean_forward(const float* v, int64_t col, const int64_t* offsets, int64_t k,
                             float patch_value, float* out) {
  kro_jagged_sum_forward(v, col, offsets, k, patch_value, out);
  for (int64_t i = 0; i < k; ++i) {
    if (offsets[i + 1] <= offsets[i]) continue;
    const float ratio = jagged_ratio(offsets[i + 1] - offsets[i]);
    float* o = out + i * col;
    for (int64_t l = 0; l < col; ++l) o[l] *= ratio;
  }
}

void kro_jagged_sum_backward(const int64_t* offsets, int64_t k, const float* grads, int64_t col,
                             float* vgrads) {
  for (int64_t i = 0; i < k; ++i)
    for (int64_t j = offsets[i]; j < offsets[i + 1]; ++j)
      memcpy(vgrads + j * col, grads + i * col, sizeof(float) * (size_t)col);
}

/* pytorch/py/jagged_ops.cc:303-334 */
void kro_jagged_mean_backward(const int64_t* offsets, int64_t k, const float* grads, int64_t col,
                              float* vgrads) {
  for (int64_t i = 0; i < k; ++i) {
    if (offsets[i + 1] <= offsets[i]) continue;
    const float ratio = jagged_ratio(offsets[i + 1] - offsets[i]);
    float* first = vgrads + offsets[i] * col;
    for (int64_t l = 0; l < col; ++l) first[l] = grads[i * col + l] * ratio;
    for (int64_t j = offsets[i] + 1; j < offsets[i + 1]; ++j)
      memcpy(vgrads + j * col, first, sizeof(float) * (size_t)col);
  }
}

/* ========================================================================== */
/* threshold codec                                                            */
/* ========================================================================== */

/* t/math.cc:540-546 */
void kro_abs(const float* x, float* y, int64_t n) {
  for (int64_t i = 0; i < n; ++i) y[i] = fabsf(x[i]);
}

/* std::priority_queue<T, vector<T>, greater<T>> : binary min-heap. */
typedef struct minheap {
  float* a;
  int64_t n;
} minheap;
static void heap_push(minheap* h, float v) {
  int64_t i = h->n++;
  h->a[i] = v;
  while (i > 0) {
    int64_t p = (i - 1) / 2;
    if (h->a[p] <= h->a[i]) break;
    float t = h->a[p];
    h->a[p] = h->a[i];
    h->a[i] = t;
    i = p;
  }
}
static void heap_pop(minheap* h) {
  h->a[0] = h->a[--h->n];
  int64_t i = 0;
  for (;;) {
    int64_t l = 2 * i + 1, r = l + 1, m = i;
    if (l < h->n && h->a[l] < h->a[m]) m = l;
    if (r < h->n && h->a[r] < h->a[m]) m = r;
    if (m == i) break;
    float t = h->a[m];
    h->a[m] = h->a[i];
    h->a[i] = t;
    i = m;
  }
}
/* The selection loop of t/math.cc:588-603 (and :606-621): keep the k largest,
 * then unload ascending into y from the back. */
static void select_k(const float* x, int64_t n, float* y, int64_t k, float* scratch) {
  minheap h = {scratch, 0};
  for (int64_t j = 0; j < n; ++j) {
    if (h.n < k) {
      heap_push(&h, x[j]);
    } else if (h.a[0] < x[j]) {
      heap_pop(&h);
      heap_push(&h, x[j]);
    }
  }
  int64_t l = k;
  while (h.n > 0) {
    y[--l] = h.a[0];
    heap_pop(&h);
  }
}

/* t/math.cc:564-626 */
void kro_topk_chunked(const float* x, int64_t n, float* y, int64_t k, int64_t t_num) {
  if (t_num < 1) t_num = 1;
  int64_t stride = n / t_num;                      /* :573 : tail n % t_num is dropped */
  float* tp = (float*)malloc(sizeof(float) * (size_t)(t_num * k));
#pragma omp parallel for
  for (int64_t i = 0; i < t_num; ++i) {
    int64_t start = i * stride;
    int64_t end = start + stride < n ? start + stride : n;
    float* scratch = (float*)malloc(sizeof(float) * (size_t)(k + 1));
    select_k(x + start, end - start, tp + i * k, k, scratch);
    free(scratch);
  }
  float* scratch = (float*)malloc(sizeof(float) * (size_t)(k + 1));
  select_k(tp, t_num * k, y, k, scratch);
  free(scratch);
  free(tp);
}

void kro_topk(const float* x, int64_t n, float* y, int64_t k, int64_t hw_threads) {
  int64_t t_num = n / k;                           /* :567-571 */
  if (hw_threads < t_num) t_num = hw_threads;
  kro_topk_chunked(x, n, y, k, t_num);
}

static int cmp_float_desc(const void* a, const void* b) {
  float x = *(const float*)a, y = *(const float*)b;
  return (x < y) - (x > y);
}
float kro_kth_largest_abs(const float* x, int64_t n, int64_t k) {
  float* a = (float*)malloc(sizeof(float) * (size_t)n);
  kro_abs(x, a, n);
  qsort(a, (size_t)n, sizeof(float), cmp_float_desc);
  float r = a[k - 1];
  free(a);
  return r;
}

/* t/math.cc:719-746 */
void kro_take(const float* x, const int64_t* idx, float* y, int64_t k) {
  for (int64_t j = 0; j < k; ++j) y[j] = x[idx[j]];
}

/* t/tensor_impl.cc:521-560 : FlatNonZero (t/math.cc:804-852, chunks are
 * concatenated in order so indices ascend) then Take. */
int64_t kro_to_coo(const float* x, int64_t n, float th, int64_t* idx, float* val) {
  int64_t nnz = 0;
  for (int64_t j = 0; j < n; ++j) {
    if (fabsf(x[j]) >= th) idx[nnz++] = j;
  }
  kro_take(x, idx, val, nnz);
  return nnz;
}

/* t/math.cc:1098-1123 */
void kro_lt_keep(const float* x, float th, float* y, int64_t n) {
  for (int64_t j = 0; j < n; ++j) y[j] = fabsf(x[j]) < th ? x[j] : 0.0f;
}

/* t/math.cc:1006-1046 for a 1-D dense shape: zero, then dense[idx] += val. */
void kro_coo_to_dense(const int64_t* idx, const float* val, int64_t nnz, float* dense,
                      int64_t n) {
  memset(dense, 0, sizeof(float) * (size_t)n);
  for (int64_t j = 0; j < nnz; ++j) dense[idx[j]] = val[j] + dense[idx[j]];
}

/* worker/dct_emitter.cc:12-14 */
struct kro_dct {
  int64_t n;
  float* e;
  float tau;
  uint64_t step;
};
kro_dct* kro_dct_create(int64_t n) {
  kro_dct* s = (kro_dct*)calloc(1, sizeof(kro_dct));
  s->n = n;
  s->e = (float*)calloc((size_t)(n > 0 ? n : 1), sizeof(float)); /* dct_emitter.cc:54 : val.Clone().Zero() */
  return s;
}
void kro_dct_destroy(kro_dct* s) {
  if (!s) return;
  free(s->e);
  free(s);
}
float kro_dct_tau(const kro_dct* s) { return s->tau; }
const float* kro_dct_residual(const kro_dct* s) { return s->e; }
uint64_t kro_dct_step(const kro_dct* s) { return s->step; }

/* worker/dct_emitter.cc:16-43 */
int64_t kro_dct_compress(kro_dct* s, const float* grad, uint64_t life_span, float eta,
                         int64_t hw_threads, int32_t exact_select, int64_t* idx, float* val) {
  int64_t n = s->n;
  if (n < 256) return -1;                           /* :18-20 */
  float* f = (float*)malloc(sizeof(float) * (size_t)n);
  m_add(grad, s->e, f, n);                          /* :23 */
  if (s->step % life_span == 0) {                   /* :25-31 */
    int64_t k = (int64_t)((double)n * (1.0 - (double)eta));
    if (exact_select) {
      s->tau = kro_kth_largest_abs(f, n, k);
    } else {
      float* a = (float*)malloc(sizeof(float) * (size_t)n);
      float* top = (float*)malloc(sizeof(float) * (size_t)k);
      kro_abs(f, a, n);
      kro_topk(a, n, top, k, hw_threads);
      s->tau = top[k - 1];
      free(a);
      free(top);
    }
  }
  int64_t nnz = kro_to_coo(f, n, s->tau, idx, val); /* :34 */
  kro_lt_keep(f, s->tau, s->e, n);                  /* :37 */
  s->step += 1;                                     /* :40 */
  free(f);
  return nnz;
}
