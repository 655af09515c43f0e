/*
 * pccl_oracle.c -- CPU restatement of the reduce-copy semantics.
 * TEST INFRASTRUCTURE ONLY (see pccl_oracle.h for the rules and for which
 * parts are pinned by what).  Build: make -C oracle  (gcc, -ffp-contract=off).
 */
#include "pccl_oracle.h"

#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------ */
/* bit casts                                                                 */
/* ------------------------------------------------------------------------ */
static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* ------------------------------------------------------------------------ */
/* bf16: top 16 bits of binary32 (the __nv_bfloat16 of                       */
/* include/plugins/cuda_executor/utils/vector_datatype.h:17-18,62,68,71)     */
/* ------------------------------------------------------------------------ */
float pccl_oracle_bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

uint16_t pccl_oracle_f32_to_bf16(float x) {
  uint32_t u = f2u(x);
  if ((u & 0x7fffffffu) > 0x7f800000u) /* NaN: keep sign and top payload, set quiet bit */
    return (uint16_t)((u >> 16) | 0x0040u);
  /* round to nearest, ties to even; a carry out of the mantissa walks into the
   * exponent, which is exactly overflow-to-infinity when it reaches 0xff */
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

/* ------------------------------------------------------------------------ */
/* f16: IEEE binary16 (the __half of vector_datatype.h:61,67,70)             */
/* ------------------------------------------------------------------------ */
float pccl_oracle_f16_to_f32(uint16_t h) {
  uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  if (exp == 0x1fu) return u2f(sign | 0x7f800000u | (man << 13)); /* inf / NaN */
  if (exp != 0) return u2f(sign | ((exp + 112u) << 23) | (man << 13));
  if (man == 0) return u2f(sign);
  /* subnormal: value = man * 2^-24, normalise */
  int e = 113;
  while (!(man & 0x400u)) { man <<= 1; --e; }
  return u2f(sign | ((uint32_t)e << 23) | ((man & 0x3ffu) << 13));
}

uint16_t pccl_oracle_f32_to_f16(float x) {
  uint32_t u = f2u(x);
  uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
  uint32_t a = u & 0x7fffffffu;
  if (a > 0x7f800000u) /* NaN: quiet, keep the top ten payload bits */
    return (uint16_t)(sign | 0x7e00u | ((a >> 13) & 0x3ffu));
  if (a >= 0x47800000u) return (uint16_t)(sign | 0x7c00u); /* >= 65536 or inf */
  if (a >= 0x38800000u) { /* normal binary16 range, 2^-14 and up */
    uint32_t v = a - 0x38000000u; /* rebias 127 -> 15 */
    v += 0xfffu + ((v >> 13) & 1u); /* RNE on the 13 dropped bits; 65520 carries to inf */
    return (uint16_t)(sign | (v >> 13));
  }
  /* result is subnormal (or zero): integer count of 2^-24 units, RNE */
  uint32_t e = a >> 23;
  if (e == 0) return sign; /* binary32 subnormals are far below 2^-25 */
  uint32_t man = (a & 0x7fffffu) | 0x800000u; /* value = man * 2^(e-150) */
  uint32_t shift = 126u - e;                  /* units of 2^-24: man >> shift */
  if (shift > 31u) return sign;
  uint32_t q = man >> shift;
  uint32_t rem = man & ((1u << shift) - 1u);
  uint32_t half = 1u << (shift - 1u);
  if (rem > half || (rem == half && (q & 1u))) ++q;
  return (uint16_t)(sign | q); /* q == 0x400 is the smallest normal: correct */
}

/* ------------------------------------------------------------------------ */
/* 8-bit floats.  One routine for both layouts: MAN mantissa bits, BIAS, and  */
/* whether the top exponent code is reserved for inf/NaN (e5m2) or only       */
/* S.1111.111 is NaN (e4m3).                                                  */
/* ------------------------------------------------------------------------ */
static float f8_to_f32(uint8_t h, int man_bits, int bias, int ieee_specials) {
  const int exp_bits = 7 - man_bits;
  const uint32_t sign = ((uint32_t)h & 0x80u) << 24;
  const uint32_t exp = ((uint32_t)h >> man_bits) & ((1u << exp_bits) - 1u);
  const uint32_t man = (uint32_t)h & ((1u << man_bits) - 1u);
  const uint32_t exp_max = (1u << exp_bits) - 1u;
  if (ieee_specials && exp == exp_max)
    return u2f(sign | 0x7f800000u | (man ? 0x00400000u | (man << (23 - man_bits)) : 0u));
  if (!ieee_specials && exp == exp_max && man == (1u << man_bits) - 1u) return u2f(sign | 0x7fc00000u);
  if (exp != 0) return u2f(sign | ((exp + 127u - (uint32_t)bias) << 23) | (man << (23 - man_bits)));
  /* subnormal: man * 2^(1 - bias - man_bits); small integers and powers of two are exact */
  float v = (float)man * u2f((uint32_t)(127 + 1 - bias - man_bits) << 23);
  return sign ? -v : v;
}

static uint8_t f32_to_f8(float x, int man_bits, int bias, int ieee_specials) {
  const int exp_bits = 7 - man_bits;
  const uint32_t u = f2u(x);
  const uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
  const uint32_t a = u & 0x7fffffffu;
  const uint8_t nan_code = 0x7fu; /* S.1111.111 and S.11111.11 */
  /* largest finite code: e4m3 S.1111.110, e5m2 S.11110.11 */
  const uint8_t max_code = ieee_specials ? (uint8_t)(((((1u << exp_bits) - 2u)) << man_bits) | ((1u << man_bits) - 1u))
                                         : (uint8_t)0x7eu;
  if (a > 0x7f800000u) return (uint8_t)(sign | nan_code);
  /* a true infinity stays infinite where the format has one and is NaN where it has none */
  if (a == 0x7f800000u) return (uint8_t)(sign | (ieee_specials ? 0x7cu : nan_code));
  const int e = (int)(a >> 23) - 127;         /* unbiased exponent of |x| (normal binary32) */
  const int min_normal = 1 - bias;            /* unbiased exponent of the smallest normal */
  uint32_t q;                                  /* result without the sign */
  if ((a >> 23) == 0) {
    q = 0;                                     /* binary32 subnormals are far below half the smallest step */
  } else if (e >= min_normal) {
    /* normal result: keep man_bits of mantissa, round to nearest even on the rest */
    const int drop = 23 - man_bits;
    uint32_t v = a - ((uint32_t)(127 - bias) << 23);   /* rebias the exponent field */
    v += ((1u << (drop - 1)) - 1u) + ((v >> drop) & 1u);
    q = v >> drop;                             /* a mantissa carry walks into the exponent */
  } else {
    /* subnormal result: integer count of steps of 2^(min_normal - man_bits) */
    const uint32_t man = (a & 0x7fffffu) | 0x800000u;  /* value = man * 2^(e - 23) */
    const int shift = (min_normal - man_bits) - (e - 23);
    if (shift > 31) {
      q = 0;
    } else {
      q = man >> shift;
      const uint32_t rem = man & ((1u << shift) - 1u), half = 1u << (shift - 1);
      if (rem > half || (rem == half && (q & 1u))) ++q;  /* q == 2^man_bits is the smallest normal */
    }
  }
  if (q > max_code) q = max_code;              /* saturate: finite overflow and rounding past the top */
  return (uint8_t)(sign | q);
}

uint8_t pccl_oracle_f32_to_e4m3(float x) { return f32_to_f8(x, 3, 7, 0); }
float pccl_oracle_e4m3_to_f32(uint8_t h) { return f8_to_f32(h, 3, 7, 0); }
uint8_t pccl_oracle_f32_to_e5m2(float x) { return f32_to_f8(x, 2, 15, 1); }
float pccl_oracle_e5m2_to_f32(uint8_t h) { return f8_to_f32(h, 2, 15, 1); }

void pccl_oracle_narrow_array8(int dtype, const float *src, uint8_t *dst, long n) {
  for (long i = 0; i < n; ++i)
    dst[i] = dtype == PCCL_ORACLE_F8E4M3 ? pccl_oracle_f32_to_e4m3(src[i]) : pccl_oracle_f32_to_e5m2(src[i]);
}

void pccl_oracle_widen_array8(int dtype, const uint8_t *src, float *dst, long n) {
  for (long i = 0; i < n; ++i)
    dst[i] = dtype == PCCL_ORACLE_F8E4M3 ? pccl_oracle_e4m3_to_f32(src[i]) : pccl_oracle_e5m2_to_f32(src[i]);
}

void pccl_oracle_narrow_array(int dtype, const float *src, uint16_t *dst, long n) {
  for (long i = 0; i < n; ++i)
    dst[i] = dtype == PCCL_ORACLE_BF16 ? pccl_oracle_f32_to_bf16(src[i])
                                       : pccl_oracle_f32_to_f16(src[i]);
}

void pccl_oracle_widen_array(int dtype, const uint16_t *src, float *dst, long n) {
  for (long i = 0; i < n; ++i)
    dst[i] = dtype == PCCL_ORACLE_BF16 ? pccl_oracle_bf16_to_f32(src[i])
                                       : pccl_oracle_f16_to_f32(src[i]);
}

/* ------------------------------------------------------------------------ */
/* reduce-copy                                                               */
/* ------------------------------------------------------------------------ */
static inline float op_sum_f(float a, float b) { return a + b; }
static inline float op_prod_f(float a, float b) { return a * b; }
static inline float op_min_f(float a, float b) { return b < a ? b : a; }
static inline float op_max_f(float a, float b) { return a < b ? b : a; }
/* i32 accumulates in uint32 so that sum/prod wrap instead of overflowing */
static inline uint32_t op_sum_i(uint32_t a, uint32_t b) { return a + b; }
static inline uint32_t op_prod_i(uint32_t a, uint32_t b) { return a * b; }
static inline uint32_t op_min_i(uint32_t a, uint32_t b) { return (int32_t)b < (int32_t)a ? b : a; }
static inline uint32_t op_max_i(uint32_t a, uint32_t b) { return (int32_t)a < (int32_t)b ? b : a; }

/* f64 accumulates in double; u32 differs from i32 only in the order min / max use */
static inline double op_sum_d(double a, double b) { return a + b; }
static inline double op_prod_d(double a, double b) { return a * b; }
static inline double op_min_d(double a, double b) { return b < a ? b : a; }
static inline double op_max_d(double a, double b) { return a < b ? b : a; }
static inline uint32_t op_sum_u(uint32_t a, uint32_t b) { return a + b; }
static inline uint32_t op_prod_u(uint32_t a, uint32_t b) { return a * b; }
static inline uint32_t op_min_u(uint32_t a, uint32_t b) { return b < a ? b : a; }
static inline uint32_t op_max_u(uint32_t a, uint32_t b) { return a < b ? b : a; }

static size_t dtype_size(int dtype) {
  switch (dtype) {
    case PCCL_ORACLE_F64: return 8;
    case PCCL_ORACLE_F32: case PCCL_ORACLE_I32: case PCCL_ORACLE_U32: return 4;
    case PCCL_ORACLE_BF16: case PCCL_ORACLE_F16: return 2;
    case PCCL_ORACLE_F8E4M3: case PCCL_ORACLE_F8E5M2: return 1;
    default: return 0;
  }
}

#define FOLD_LOOP(ELEM, ACC, UP, DOWN, OPFN)                                   \
  do {                                                                         \
    for (long i = lo; i < hi; ++i) {                                           \
      ACC acc = UP(((const ELEM *)ins[0])[i]);                                 \
      for (int k = 1; k < n_in; ++k) acc = OPFN(acc, UP(((const ELEM *)ins[k])[i])); \
      ELEM r = DOWN(acc);                                                      \
      for (int j = 0; j < n_out; ++j) ((ELEM *)outs[j])[i] = r;                \
    }                                                                          \
  } while (0)

#define BY_OP(ELEM, ACC, UP, DOWN, SFX)                                        \
  switch (op) {                                                                \
    case PCCL_ORACLE_SUM: FOLD_LOOP(ELEM, ACC, UP, DOWN, op_sum_##SFX); break;   \
    case PCCL_ORACLE_PROD: FOLD_LOOP(ELEM, ACC, UP, DOWN, op_prod_##SFX); break; \
    case PCCL_ORACLE_MIN: FOLD_LOOP(ELEM, ACC, UP, DOWN, op_min_##SFX); break;   \
    case PCCL_ORACLE_MAX: FOLD_LOOP(ELEM, ACC, UP, DOWN, op_max_##SFX); break;   \
    default: return -1;                                                        \
  }

#define IDENT(x) (x)

/* elements [lo, hi) of one reduce-copy */
static int reduce_range(int dtype, int op, const void *const *ins, int n_in,
                        void *const *outs, int n_out, long lo, long hi) {
  if (n_in == 1) { /* COPY: bytes move unchanged */
    size_t es = dtype_size(dtype);
    for (int j = 0; j < n_out; ++j)
      if ((const char *)outs[j] != (const char *)ins[0])
        memmove((char *)outs[j] + lo * es, (const char *)ins[0] + lo * es, (size_t)(hi - lo) * es);
    return 0;
  }
  switch (dtype) {
    case PCCL_ORACLE_F32: BY_OP(float, float, IDENT, IDENT, f); break;
    case PCCL_ORACLE_I32: BY_OP(uint32_t, uint32_t, IDENT, IDENT, i); break;
    case PCCL_ORACLE_U32: BY_OP(uint32_t, uint32_t, IDENT, IDENT, u); break;
    case PCCL_ORACLE_F64: BY_OP(double, double, IDENT, IDENT, d); break;
    case PCCL_ORACLE_BF16:
      BY_OP(uint16_t, float, pccl_oracle_bf16_to_f32, pccl_oracle_f32_to_bf16, f);
      break;
    case PCCL_ORACLE_F16:
      BY_OP(uint16_t, float, pccl_oracle_f16_to_f32, pccl_oracle_f32_to_f16, f);
      break;
    case PCCL_ORACLE_F8E4M3:
      BY_OP(uint8_t, float, pccl_oracle_e4m3_to_f32, pccl_oracle_f32_to_e4m3, f);
      break;
    case PCCL_ORACLE_F8E5M2:
      BY_OP(uint8_t, float, pccl_oracle_e5m2_to_f32, pccl_oracle_f32_to_e5m2, f);
      break;
    default: return -1;
  }
  return 0;
}

static int check_args(int dtype, int op, const void *const *ins, int n_in,
                      void *const *outs, int n_out, long count) {
  if (dtype_size(dtype) == 0) return -1;
  if (op < PCCL_ORACLE_SUM || op > PCCL_ORACLE_MAX) return -1;
  if (n_in < 1 || n_in > 8 || n_out < 1 || n_out > 8 || count < 0) return -1;
  if (!ins || !outs) return -1;
  for (int k = 0; k < n_in; ++k) if (!ins[k] && count) return -1;
  for (int j = 0; j < n_out; ++j) if (!outs[j] && count) return -1;
  return 0;
}

int pccl_oracle_reduce_copy(int dtype, int op, const void *const *ins, int n_in,
                            void *const *outs, int n_out, long count) {
  if (check_args(dtype, op, ins, n_in, outs, n_out, count)) return -1;
  return reduce_range(dtype, op, ins, n_in, outs, n_out, 0, count);
}

struct mt_job {
  int dtype, op, n_in, n_out, rc;
  const void *const *ins;
  void *const *outs;
  long lo, hi;
};

static void *mt_worker(void *p) {
  struct mt_job *j = (struct mt_job *)p;
  j->rc = reduce_range(j->dtype, j->op, j->ins, j->n_in, j->outs, j->n_out, j->lo, j->hi);
  return NULL;
}

int pccl_oracle_reduce_copy_mt(int dtype, int op, const void *const *ins, int n_in,
                               void *const *outs, int n_out, long count, int nthreads) {
  if (check_args(dtype, op, ins, n_in, outs, n_out, count)) return -1;
  if (nthreads < 1) nthreads = 1;
  if (nthreads > 256) nthreads = 256;
  if (nthreads == 1 || count < 4096)
    return reduce_range(dtype, op, ins, n_in, outs, n_out, 0, count);
  pthread_t tid[256];
  struct mt_job job[256];
  /* slices start on multiples of 64 elements so that threads never share a cache line */
  long per = ((count + nthreads - 1) / nthreads + 63) / 64 * 64;
  int started = 0, rc = 0;
  for (int t = 0; t < nthreads; ++t) {
    long lo = (long)t * per, hi = lo + per;
    if (lo >= count) break;
    if (hi > count) hi = count;
    job[t] = (struct mt_job){dtype, op, n_in, n_out, 0, ins, outs, lo, hi};
    if (pthread_create(&tid[t], NULL, mt_worker, &job[t]) != 0) {
      mt_worker(&job[t]); /* no thread available: do the slice here */
      tid[t] = 0;
    }
    ++started;
  }
  for (int t = 0; t < started; ++t) {
    if (tid[t]) pthread_join(tid[t], NULL);
    if (job[t].rc) rc = -1;
  }
  return rc;
}

int pccl_oracle_run_ops(const pccl_oracle_op *ops, int n_ops, const int *order) {
  for (int s = 0; s < n_ops; ++s) {
    int i = order ? order[s] : s;
    if (i < 0 || i >= n_ops) return -1;
    const pccl_oracle_op *o = &ops[i];
    if (pccl_oracle_reduce_copy(o->dtype, o->op, o->ins, o->n_in, (void *const *)o->outs,
                                o->n_out, o->count))
      return -1;
  }
  return 0;
}

/* ------------------------------------------------------------------------ */
/* DAG order: pccl/lang/utils/graph.py:94-112                                */
/* ------------------------------------------------------------------------ */
int pccl_oracle_topo_sort(int n_nodes, const int *edge_src, const int *edge_dst,
                          int n_edges, int *order_out) {
  if (n_nodes < 0 || n_edges < 0) return -1;
  if (n_nodes == 0) return 0;
  /* successor lists in edge-insertion order (graph.py:29-36 appends to out_edges) */
  int *deg = (int *)calloc((size_t)n_nodes + 1, sizeof(int));
  int *start = (int *)calloc((size_t)n_nodes + 1, sizeof(int));
  int *succ = (int *)malloc(sizeof(int) * (size_t)(n_edges > 0 ? n_edges : 1));
  int *state = (int *)calloc((size_t)n_nodes, sizeof(int)); /* 0 new, 1 on stack, 2 done */
  int *stack = (int *)malloc(sizeof(int) * (size_t)n_nodes);
  int *cursor = (int *)malloc(sizeof(int) * (size_t)n_nodes);
  int rc = 0, n_done = 0;
  if (!deg || !start || !succ || !state || !stack || !cursor) { rc = -1; goto out; }
  for (int e = 0; e < n_edges; ++e) {
    if (edge_src[e] < 0 || edge_src[e] >= n_nodes || edge_dst[e] < 0 || edge_dst[e] >= n_nodes) {
      rc = -1; /* graph.py:30-31 raises ValueError("Invalid node IDs") */
      goto out;
    }
    ++deg[edge_src[e]];
  }
  for (int v = 0; v < n_nodes; ++v) start[v + 1] = start[v] + deg[v];
  memset(deg, 0, sizeof(int) * (size_t)n_nodes);
  for (int e = 0; e < n_edges; ++e) succ[start[edge_src[e]] + deg[edge_src[e]]++] = edge_dst[e];
  /* iterative form of the recursive dfs(); post-order collected front to back,
   * then reversed (graph.py:112 result[::-1]) */
  for (int root = 0; root < n_nodes; ++root) {
    if (state[root]) continue;
    int sp = 0;
    stack[sp] = root; cursor[sp] = start[root]; state[root] = 1; ++sp;
    while (sp) {
      int v = stack[sp - 1];
      if (cursor[sp - 1] < start[v + 1]) {
        int w = succ[cursor[sp - 1]++];
        if (state[w] == 1) { rc = -1; goto out; } /* back edge: cycle */
        if (state[w] == 0) {
          stack[sp] = w; cursor[sp] = start[w]; state[w] = 1; ++sp;
        }
      } else {
        state[v] = 2;
        order_out[n_done++] = v;
        --sp;
      }
    }
  }
  for (int i = 0, j = n_nodes - 1; i < j; ++i, --j) {
    int t = order_out[i]; order_out[i] = order_out[j]; order_out[j] = t;
  }
out:
  free(deg); free(start); free(succ); free(state); free(stack); free(cursor);
  return rc;
}

/* ------------------------------------------------------------------------ */
/* seeded inputs                                                             */
/* ------------------------------------------------------------------------ */
static inline uint64_t mix64(uint64_t z) { /* splitmix64 finaliser */
  z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
  z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
  return z ^ (z >> 31);
}

uint64_t pccl_oracle_rng_u64(uint64_t seed, uint64_t stream, uint64_t index) {
  uint64_t key = mix64(seed * 0x9e3779b97f4a7c15ull + stream + 0x632be59bd9b4e019ull);
  return mix64(key + (index + 1) * 0x9e3779b97f4a7c15ull);
}

void pccl_oracle_fill_uniform_f32(float *dst, long n, uint64_t seed, uint64_t stream,
                                  float lo, float hi) {
  for (long i = 0; i < n; ++i) {
    float u = (float)(pccl_oracle_rng_u64(seed, stream, (uint64_t)i) >> 40) * (1.0f / 16777216.0f);
    dst[i] = lo + (hi - lo) * u; /* u in [0, 1) */
  }
}

void pccl_oracle_fill_normal_at(void *dst, int dtype, long first, long n, uint64_t seed, uint64_t stream,
                                double mean, double sigma) {
  const double two_pi = 6.283185307179586476925286766559;
  for (long i = 0; i < n; ++i) {
    const uint64_t at = (uint64_t)(first + i);
    uint64_t a = pccl_oracle_rng_u64(seed, stream, 2 * at);
    uint64_t b = pccl_oracle_rng_u64(seed, stream, 2 * at + 1);
    double u1 = ((double)(a >> 11) + 1.0) * (1.0 / 9007199254740992.0); /* (0, 1] */
    double u2 = (double)(b >> 11) * (1.0 / 9007199254740992.0);         /* [0, 1) */
    const double zd = mean + sigma * sqrt(-2.0 * log(u1)) * cos(two_pi * u2);
    float z = (float)zd;
    switch (dtype) {
      case PCCL_ORACLE_F64: ((double *)dst)[i] = zd; break;
      case PCCL_ORACLE_F32: ((float *)dst)[i] = z; break;
      case PCCL_ORACLE_BF16: ((uint16_t *)dst)[i] = pccl_oracle_f32_to_bf16(z); break;
      case PCCL_ORACLE_F16: ((uint16_t *)dst)[i] = pccl_oracle_f32_to_f16(z); break;
      case PCCL_ORACLE_F8E4M3: ((uint8_t *)dst)[i] = pccl_oracle_f32_to_e4m3(z); break;
      case PCCL_ORACLE_F8E5M2: ((uint8_t *)dst)[i] = pccl_oracle_f32_to_e5m2(z); break;
      default: return;
    }
  }
}

void pccl_oracle_fill_normal(void *dst, int dtype, long n, uint64_t seed, uint64_t stream,
                             double mean, double sigma) {
  pccl_oracle_fill_normal_at(dst, dtype, 0, n, seed, stream, mean, sigma);
}

void pccl_oracle_fill_int32(int32_t *dst, long n, uint64_t seed, uint64_t stream,
                            int32_t lo, int32_t hi) {
  uint64_t span = (uint64_t)((int64_t)hi - (int64_t)lo) + 1u;
  for (long i = 0; i < n; ++i)
    dst[i] = (int32_t)((int64_t)lo + (int64_t)(pccl_oracle_rng_u64(seed, stream, (uint64_t)i) % span));
}
