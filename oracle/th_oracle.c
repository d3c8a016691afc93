/*
 * th_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * CPU restatement of the semantics that torch7's TH FloatTensor path gives to
 * the operations behind cutorch's THCudaTensor_add/cadd/cmul/cdiv/addcmul/
 * sum/max/min/norm (+ the *all forms). cutorch's own tests compare every CUDA
 * op with that CPU path (test/test.lua:247-323); TH itself is not part of the
 * cutorch tree (it is the external rock "torch >= 7.0",
 * rocks/cutorch-scm-1.rockspec:16-18), so this file restates the published
 * algorithm of TH's TH_TENSOR_APPLY / dimension-reduction loops:
 *
 *   - operands are walked in logical row-major order, each through its own
 *     sizes/strides, and paired by logical linear index (the same pairing as
 *     lib/THC/THCTensorInfo.cuh:229-278 and THCApply.cuh:81-97);
 *   - pointwise results are one correctly rounded binary32 operation per
 *     arithmetic step, never fused (compile with -ffp-contract=off);
 *     functor formulas as in lib/THC/THCTensorMathPointwise.cuh:103-112,
 *     141-154,229-238,366-377,622-654 and THCTensorMathPairwise.cu:9-191,
 *     with true division for the scalar divide;
 *   - sum/prod/norm accumulate sequentially in double (TH's accreal for
 *     float) and round once; operation selection for norm (p == 0, 1, 2,
 *     other) as in lib/THC/generic/THCTensorMathReduce.cu:160-232;
 *   - max/min scan sequentially, keep the first occurrence, stop at the first
 *     NaN, and report 1-based int64 indices (TH_INDEX_BASE;
 *     lib/THC/THCTensorMathReduce.cuh:473,553);
 *   - output shape of a dim reduction: input sizes with size[dim] = 1
 *     (lib/THC/THCReduce.cuh:328-332).
 *
 * Pinned by tests/test_oracle.py against numpy's IEEE binary32 arithmetic on
 * independently built strided views, math.fsum, numpy.argmax/argmin,
 * exhaustive numpy.float16 conversion, and integer-valued known answers.
 * Parity unpinned (no TH build, no stored vectors in the reference): the
 * accumulator type/order inside TH's sum/norm and TH's NaN policy for max/min
 * are restated from TH's published source from memory; both are immaterial at
 * the stated tolerances / on NaN-free configs.
 *
 * Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may
 * load this library.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define TH_MAX_DIMS 25

typedef struct {
  void *data;          /* element 0 of the view (storage + offset) */
  int nd;              /* 0 = empty tensor */
  const long *size;
  const long *stride;  /* in elements */
} th_view;

enum {
  TH_OP_COPY = 0, TH_OP_ADDC, TH_OP_SUBC, TH_OP_MULC, TH_OP_DIVC,
  TH_OP_ADD, TH_OP_SUB, TH_OP_MUL, TH_OP_DIV, TH_OP_CADD,
  TH_OP_ADDCMUL, TH_OP_ADDCDIV, TH_OP_FILL, TH_OP_POW,
  TH_OP_LERP,                 /* a + v * (b - a) */
  TH_OP_MATH1 = 100,          /* TH_OP_MATH1 + fn: out = fn(a; v, w) */
  TH_OP_MATH2 = 200           /* TH_OP_MATH2 + fn: out = fn(a, b) */
};

/* Function codes of the unary / binary math family; formulas as in
 * lib/THC/THCNumerics.cuh:536-579 (float row) and
 * lib/THC/THCTensorMathPointwise.cuh (sigmoid, sign, clamp, pow special
 * cases 1, 2, 3, -1, -2, tpow, max/min, fmod/remainder, lerp). */
enum {
  TH_FN_SIGMOID = 0, TH_FN_LOG, TH_FN_LGAMMA, TH_FN_LOG1P, TH_FN_EXP, TH_FN_COS, TH_FN_ACOS,
  TH_FN_COSH, TH_FN_SIN, TH_FN_ASIN, TH_FN_SINH, TH_FN_TAN, TH_FN_ATAN, TH_FN_TANH, TH_FN_SQRT,
  TH_FN_RSQRT, TH_FN_CEIL, TH_FN_FLOOR, TH_FN_ROUND, TH_FN_TRUNC, TH_FN_FRAC, TH_FN_CINV,
  TH_FN_NEG, TH_FN_ABS, TH_FN_SIGN, TH_FN_CLAMP, TH_FN_SQDIFFVALUE, TH_FN_POWSCALAR, TH_FN_TPOW, TH_FN_MAXVALUE,
  TH_FN_MINVALUE, TH_FN_FMODVALUE, TH_FN_REMAINDERVALUE,
  TH_FN_CPOW, TH_FN_CMAX, TH_FN_CMIN, TH_FN_CFMOD, TH_FN_CREMAINDER, TH_FN_ATAN2, TH_FN_EQUAL,
  TH_FN_SQDIFF, TH_FN_LSHIFTVALUE, TH_FN_RSHIFTVALUE, TH_FN_BITANDVALUE, TH_FN_BITORVALUE,
  TH_FN_BITXORVALUE, TH_FN_CLSHIFT, TH_FN_CRSHIFT
};

static int g_threads = 1;
void th_set_num_threads(int n) { g_threads = n < 1 ? 1 : n; }
int th_get_num_threads(void) { return g_threads; }

static long th_numel(const th_view *v) {
  if (v->nd == 0) return 0;
  long n = 1;
  for (int d = 0; d < v->nd; ++d) n *= v->size[d];
  return n;
}

static int th_is_contiguous(const th_view *v) {
  long z = 1;
  for (int d = v->nd - 1; d >= 0; --d) {
    if (v->size[d] == 1) continue;
    if (v->stride[d] != z) return 0;
    z *= v->size[d];
  }
  return 1;
}

/* Odometer over the logical index space of one view. */
typedef struct {
  long idx[TH_MAX_DIMS];
  long off;
} th_odo;

static void odo_seek(th_odo *o, const th_view *v, long lin) {
  o->off = 0;
  for (int d = v->nd - 1; d >= 0; --d) {
    o->idx[d] = lin % v->size[d];
    lin /= v->size[d];
    o->off += o->idx[d] * v->stride[d];
  }
}

static inline void odo_next(th_odo *o, const th_view *v) {
  for (int d = v->nd - 1; d >= 0; --d) {
    o->off += v->stride[d];
    if (++o->idx[d] < v->size[d]) return;
    o->off -= o->idx[d] * v->stride[d];
    o->idx[d] = 0;
  }
}

/* ---------------------------------------------------------------- half -- */
/* binary16 <-> binary32, round-to-nearest-even, subnormals kept. */
float th_half2float(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16, e = (h >> 10) & 0x1f, m = h & 0x3ff, x;
  if (e == 0x1f) x = sign | 0x7f800000u | (m << 13);
  else if (e == 0) {
    if (m == 0) x = sign;
    else {
      e = 113;
      while (!(m & 0x400)) { m <<= 1; --e; }
      x = sign | (e << 23) | ((m & 0x3ff) << 13);
    }
  } else x = sign | ((e + 112) << 23) | (m << 13);
  float f;
  memcpy(&f, &x, 4);
  return f;
}

uint16_t th_float2half(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
  x &= 0x7fffffffu;
  if (x > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((x >> 13) & 0x3ffu)); /* NaN */
  if (x == 0x7f800000u) return (uint16_t)(sign | 0x7c00u);
  /* scale in double and let rint() do the RNE step on an exactly
   * representable quotient */
  double a = fabs((double)f);
  if (a >= 65520.0) return (uint16_t)(sign | 0x7c00u);
  int ex;
  (void)frexp(a, &ex);             /* a = m * 2^ex, m in [0.5, 1) */
  int e = ex - 1;                  /* unbiased exponent of a */
  if (a == 0.0) return sign;
  if (e < -14) e = -14;            /* subnormal range: fixed quantum 2^-24 */
  double q = ldexp(a, 10 - e);     /* units of the half ulp at that exponent */
  double r = rint(q);              /* current rounding mode: to nearest even */
  uint32_t bits;
  if (e == -14 && r < 1024.0) bits = (uint32_t)r;                 /* subnormal */
  else bits = (uint32_t)((e + 15) << 10) + ((uint32_t)r - 1024u); /* carry ok */
  return (uint16_t)(sign | bits);
}

void th_half2float_array(float *dst, const uint16_t *src, long n) {
  for (long i = 0; i < n; ++i) dst[i] = th_half2float(src[i]);
}
void th_float2half_array(uint16_t *dst, const float *src, long n) {
  for (long i = 0; i < n; ++i) dst[i] = th_float2half(src[i]);
}

/* ------------------------------------------------------------ pointwise -- */
static float math1(int fn, float x, float v, float w) {
  switch (fn) {
    case TH_FN_SIGMOID: return 1.0f / (1.0f + expf(-x));
    case TH_FN_LOG: return logf(x);
    case TH_FN_LGAMMA: return lgammaf(x);
    case TH_FN_LOG1P: return log1pf(x);
    case TH_FN_EXP: return expf(x);
    case TH_FN_COS: return cosf(x);
    case TH_FN_ACOS: return acosf(x);
    case TH_FN_COSH: return coshf(x);
    case TH_FN_SIN: return sinf(x);
    case TH_FN_ASIN: return asinf(x);
    case TH_FN_SINH: return sinhf(x);
    case TH_FN_TAN: return tanf(x);
    case TH_FN_ATAN: return atanf(x);
    case TH_FN_TANH: return tanhf(x);
    case TH_FN_SQRT: return sqrtf(x);
    case TH_FN_RSQRT: { float r = sqrtf(x); return 1.0f / r; }
    case TH_FN_CEIL: return ceilf(x);
    case TH_FN_FLOOR: return floorf(x);
    case TH_FN_ROUND: return roundf(x);
    case TH_FN_TRUNC: return truncf(x);
    case TH_FN_FRAC: return x - truncf(x);
    case TH_FN_CINV: return 1.0f / x;
    case TH_FN_NEG: return -x;
    case TH_FN_ABS: return fabsf(x);
    case TH_FN_SIGN: return (float)((x > 0.f) - (x < 0.f));
    case TH_FN_CLAMP: return x < v ? v : (x > w ? w : x);
    case TH_FN_SQDIFFVALUE: { float t = x - v; return t * t; }
    case TH_FN_POWSCALAR:
      if (v == 1.f) return x;
      if (v == 2.f) return x * x;
      if (v == 3.f) { float t = x * x; return t * x; }
      if (v == -1.f) return 1.0f / x;
      if (v == -2.f) { float t = x * x; return 1.0f / t; }
      return powf(x, v);
    case TH_FN_TPOW: return powf(v, x);
    case TH_FN_MAXVALUE: return x > v ? x : v;
    case TH_FN_MINVALUE: return x < v ? x : v;
    case TH_FN_FMODVALUE: return fmodf(x, v);
    case TH_FN_REMAINDERVALUE: { if (v == 0.f) return NAN; float q = x / v; q = floorf(q); q = v * q; return x - q; }
    /* shifts of floating types scale by a power of two (THCTensorMathPairwise.cu:436-462) */
    case TH_FN_LSHIFTVALUE: { float t = powf(2.f, v); return x * t; }
    case TH_FN_RSHIFTVALUE: { float t = powf(2.f, v); return x / t; }
  }
  return x;
}

static float math2(int fn, float a, float b) {
  switch (fn) {
    case TH_FN_CPOW: return powf(a, b);
    case TH_FN_CMAX: return a > b ? a : b;
    case TH_FN_CMIN: return a < b ? a : b;
    case TH_FN_CFMOD: return fmodf(a, b);
    case TH_FN_CREMAINDER: { if (b == 0.f) return NAN; float q = a / b; q = floorf(q); q = b * q; return a - q; }
    case TH_FN_ATAN2: return atan2f(a, b);
    case TH_FN_EQUAL: return a == b ? 1.f : 0.f;
    case TH_FN_SQDIFF: { float t = a - b; return t * t; }
    case TH_FN_CLSHIFT: { float t = powf(2.f, b); return a * t; }
    case TH_FN_CRSHIFT: { float t = powf(2.f, b); return a / t; }
  }
  return a;
}

static float g_w = 0.f; /* second scalar of clamp, set through th_set_second_scalar */
void th_set_second_scalar(float w) { g_w = w; }

static inline float point_op(int op, float v, float a, float b, float c) {
  if (op >= TH_OP_MATH2) return math2(op - TH_OP_MATH2, a, b);
  if (op >= TH_OP_MATH1) return math1(op - TH_OP_MATH1, a, v, g_w);
  switch (op) {
    case TH_OP_COPY: return a;
    case TH_OP_ADDC: return a + v;
    case TH_OP_SUBC: return a - v;
    case TH_OP_MULC: return a * v;
    case TH_OP_DIVC: return a / v;
    case TH_OP_ADD: return a + b;
    case TH_OP_SUB: return a - b;
    case TH_OP_MUL: return a * b;
    case TH_OP_DIV: return a / b;
    case TH_OP_CADD: { float t = v * b; return a + t; }
    case TH_OP_ADDCMUL: { float t = b * c; t = v * t; return a + t; }
    case TH_OP_ADDCDIV: { float t = b / c; t = v * t; return a + t; }
    case TH_OP_FILL: return v;
    case TH_OP_POW: return powf(a, v);
    case TH_OP_LERP: { float t = b - a; t = v * t; return a + t; }
  }
  return 0.f;
}

static int op_inputs(int op) {
  if (op >= TH_OP_MATH2) return 2;
  if (op >= TH_OP_MATH1) return 1;
  if (op == TH_OP_LERP) return 2;
  if (op == TH_OP_FILL) return 0;
  if (op <= TH_OP_DIVC || op == TH_OP_POW) return 1;
  if (op <= TH_OP_CADD) return 2;
  return 3;
}

/* out[i] = op(a[i], b[i], c[i]) for every logical linear index i.
 * Returns 0 on success, 1 if element counts differ. Unused inputs may be NULL.
 * An `out` that aliases an input is handled element by element (in place). */
int th_pointwise_float(int op, float v, const th_view *out, const th_view *a, const th_view *b,
                       const th_view *c) {
  const int nin = op_inputs(op);
  const th_view *in[3] = {a, b, c};
  const long n = th_numel(out);
  for (int k = 0; k < nin; ++k)
    if (th_numel(in[k]) != n) return 1;
  if (n == 0) return 0;
  int flat = th_is_contiguous(out);
  for (int k = 0; k < nin; ++k) flat = flat && th_is_contiguous(in[k]);
  float *o = (float *)out->data;
  const float *pa = nin > 0 ? (const float *)a->data : 0;
  const float *pb = nin > 1 ? (const float *)b->data : 0;
  const float *pc = nin > 2 ? (const float *)c->data : 0;
  if (flat) {
#pragma omp parallel for num_threads(g_threads) schedule(static) if (g_threads > 1)
    for (long i = 0; i < n; ++i)
      o[i] = point_op(op, v, pa ? pa[i] : 0.f, pb ? pb[i] : 0.f, pc ? pc[i] : 0.f);
    return 0;
  }
  const int T = g_threads;
#pragma omp parallel for num_threads(T) schedule(static) if (T > 1)
  for (int t = 0; t < T; ++t) {
    const long lo = n * t / T, hi = n * (t + 1) / T;
    th_odo oo, oi[3];
    odo_seek(&oo, out, lo);
    for (int k = 0; k < nin; ++k) odo_seek(&oi[k], in[k], lo);
    for (long i = lo; i < hi; ++i) {
      const float x = pa ? pa[oi[0].off] : 0.f;
      const float y = pb ? pb[oi[1].off] : 0.f;
      const float z = pc ? pc[oi[2].off] : 0.f;
      o[oo.off] = point_op(op, v, x, y, z);
      odo_next(&oo, out);
      for (int k = 0; k < nin; ++k) odo_next(&oi[k], in[k]);
    }
  }
  return 0;
}

/* fp16 tensors: compute in binary32 on the converted inputs, round once. */
int th_pointwise_half(int op, float v, const th_view *out, const th_view *a, const th_view *b,
                      const th_view *c) {
  const int nin = op_inputs(op);
  const th_view *in[3] = {a, b, c};
  const long n = th_numel(out);
  for (int k = 0; k < nin; ++k)
    if (th_numel(in[k]) != n) return 1;
  if (n == 0) return 0;
  th_odo oo, oi[3];
  odo_seek(&oo, out, 0);
  for (int k = 0; k < nin; ++k) odo_seek(&oi[k], in[k], 0);
  uint16_t *o = (uint16_t *)out->data;
  for (long i = 0; i < n; ++i) {
    float x[3] = {0.f, 0.f, 0.f};
    for (int k = 0; k < nin; ++k) x[k] = th_half2float(((const uint16_t *)in[k]->data)[oi[k].off]);
    o[oo.off] = th_float2half(point_op(op, v, x[0], x[1], x[2]));
    odo_next(&oo, out);
    for (int k = 0; k < nin; ++k) odo_next(&oi[k], in[k]);
  }
  return 0;
}

/* ----------------------------------------------------------- reductions -- */
/* VAR / STD (+ their unbiased forms) follow TH's one-sweep formula in double:
 * sum and sum of squares, then E[x^2] - E[x]^2 with the n/(n-1) correction. */
enum { TH_R_SUM = 0, TH_R_PROD, TH_R_MIN, TH_R_MAX, TH_R_NORM, TH_R_MEAN,
       TH_R_VAR_BIASED, TH_R_VAR, TH_R_STD_BIASED, TH_R_STD };

static inline float load_elem(const void *base, long off, int is_half) {
  return is_half ? th_half2float(((const uint16_t *)base)[off]) : ((const float *)base)[off];
}

/* One slice: n elements `stride` apart starting at base[off]. */
static double reduce_slice(int kind, double p, const void *base, long off, long n, long stride,
                           int is_half) {
  double acc;
  switch (kind) {
    case TH_R_SUM:
    case TH_R_MEAN:
      acc = 0;
      for (long i = 0; i < n; ++i) acc += load_elem(base, off + i * stride, is_half);
      return kind == TH_R_MEAN ? (double)((float)acc) : acc;
    case TH_R_PROD:
      acc = 1;
      for (long i = 0; i < n; ++i) acc *= load_elem(base, off + i * stride, is_half);
      return acc;
    case TH_R_VAR_BIASED: case TH_R_VAR: case TH_R_STD_BIASED: case TH_R_STD: {
      double sum = 0, sum2 = 0;
      for (long i = 0; i < n; ++i) {
        const double z = load_elem(base, off + i * stride, is_half);
        sum += z;
        sum2 += z * z;
      }
      const int biased = kind == TH_R_VAR_BIASED || kind == TH_R_STD_BIASED;
      sum /= (double)n;
      if (biased) {
        sum2 /= (double)n;
        sum2 -= sum * sum;
      } else {
        sum2 /= (double)(n - 1);
        sum2 -= ((double)n) / ((double)(n - 1)) * sum * sum;
      }
      if (sum2 < 0) sum2 = 0;
      return (kind == TH_R_STD_BIASED || kind == TH_R_STD) ? sqrt(sum2) : sum2;
    }
    case TH_R_NORM:
      acc = 0;
      if (p == 0) {
        for (long i = 0; i < n; ++i) acc += load_elem(base, off + i * stride, is_half) != 0.f;
        return acc;
      } else if (p == 1) {
        for (long i = 0; i < n; ++i) acc += fabs((double)load_elem(base, off + i * stride, is_half));
        return acc;
      } else if (p == 2) {
        for (long i = 0; i < n; ++i) {
          const double z = load_elem(base, off + i * stride, is_half);
          acc += z * z;
        }
        return sqrt(acc);
      }
      for (long i = 0; i < n; ++i)
        acc += pow(fabs((double)load_elem(base, off + i * stride, is_half)), p);
      return pow(acc, 1.0 / p);
  }
  return 0;
}

/* out = reduce(in, dim); out must be viewed with the shape of `in` except
 * size[dim] == 1 (its stride at dim is ignored). kind TH_R_MEAN divides the
 * float-rounded sum by the slice length in float (sum, then div).
 * Returns 0, or 1 on a shape mismatch. */
static int reduce_dim_impl(int kind, double p, const th_view *out, const th_view *in, int dim,
                           int is_half) {
  if (in->nd == 0) return 0;
  if (out->nd != in->nd || dim < 0 || dim >= in->nd) return 1;
  long osz[TH_MAX_DIMS];
  for (int d = 0; d < in->nd; ++d) {
    osz[d] = d == dim ? 1 : in->size[d];
    if (out->size[d] != osz[d]) return 1;
  }
  th_view islice = *in;
  islice.size = osz; /* walk the input with the reduced dim pinned to 0 */
  const long nout = th_numel(out);
  const long n = in->size[dim], st = in->stride[dim];
  const int T = g_threads;
#pragma omp parallel for num_threads(T) schedule(static) if (T > 1)
  for (int t = 0; t < T; ++t) {
    const long lo = nout * t / T, hi = nout * (t + 1) / T;
    th_odo oo, oi;
    odo_seek(&oo, out, lo);
    odo_seek(&oi, &islice, lo);
    for (long j = lo; j < hi; ++j) {
      double r = reduce_slice(kind, p, in->data, oi.off, n, st, is_half);
      float rf = (float)r;
      if (kind == TH_R_MEAN) rf = rf / (float)n;
      if (is_half) ((uint16_t *)out->data)[oo.off] = th_float2half(rf);
      else ((float *)out->data)[oo.off] = rf;
      odo_next(&oo, out);
      odo_next(&oi, &islice);
    }
  }
  return 0;
}

int th_reduce_dim_float(int kind, double p, const th_view *out, const th_view *in, int dim) {
  return reduce_dim_impl(kind, p, out, in, dim, 0);
}
int th_reduce_dim_half(int kind, double p, const th_view *out, const th_view *in, int dim) {
  return reduce_dim_impl(kind, p, out, in, dim, 1);
}

/* Inclusive prefix sum (product = 0) or product (product = 1) along dim with
 * a sequential double accumulator, rounded per output element (TH's cumsum /
 * cumprod loops; entry semantics lib/THC/generic/THCTensorMathScan.cu:76-126).
 * `out` has the shape of `in`. */
static int scan_dim_impl(int product, const th_view *out, const th_view *in, int dim, int is_half) {
  if (in->nd == 0) return 0;
  if (out->nd != in->nd || dim < 0 || dim >= in->nd) return 1;
  long osz[TH_MAX_DIMS];
  for (int d = 0; d < in->nd; ++d) {
    if (out->size[d] != in->size[d]) return 1;
    osz[d] = d == dim ? 1 : in->size[d];
  }
  th_view il = *in, ol = *out;
  il.size = osz;
  ol.size = osz;
  const long lines = th_numel(&il), n = in->size[dim];
  th_odo oi, oo;
  odo_seek(&oi, &il, 0);
  odo_seek(&oo, &ol, 0);
  for (long l = 0; l < lines; ++l) {
    double acc = product ? 1.0 : 0.0;
    for (long i = 0; i < n; ++i) {
      const double x = load_elem(in->data, oi.off + i * in->stride[dim], is_half);
      acc = product ? acc * x : acc + x;
      const long at = oo.off + i * out->stride[dim];
      if (is_half) ((uint16_t *)out->data)[at] = th_float2half((float)acc);
      else ((float *)out->data)[at] = (float)acc;
    }
    odo_next(&oi, &il);
    odo_next(&oo, &ol);
  }
  return 0;
}
int th_scan_dim_float(int product, const th_view *out, const th_view *in, int dim) {
  return scan_dim_impl(product, out, in, dim, 0);
}
int th_scan_dim_half(int product, const th_view *out, const th_view *in, int dim) {
  return scan_dim_impl(product, out, in, dim, 1);
}

/* (value, 1-based index) of the max / min along dim; first occurrence wins,
 * the first NaN wins over everything and ends the scan. */
static int minmax_dim_impl(int is_max, const th_view *val, const th_view *idx, const th_view *in,
                           int dim, int is_half) {
  if (in->nd == 0) return 0;
  if (val->nd != in->nd || idx->nd != in->nd || dim < 0 || dim >= in->nd) return 1;
  long osz[TH_MAX_DIMS];
  for (int d = 0; d < in->nd; ++d) {
    osz[d] = d == dim ? 1 : in->size[d];
    if (val->size[d] != osz[d] || idx->size[d] != osz[d]) return 1;
  }
  th_view islice = *in;
  islice.size = osz;
  const long nout = th_numel(val);
  const long n = in->size[dim], st = in->stride[dim];
  const int T = g_threads;
#pragma omp parallel for num_threads(T) schedule(static) if (T > 1)
  for (int t = 0; t < T; ++t) {
    const long lo = nout * t / T, hi = nout * (t + 1) / T;
    th_odo ov, ox, oi;
    odo_seek(&ov, val, lo);
    odo_seek(&ox, idx, lo);
    odo_seek(&oi, &islice, lo);
    for (long j = lo; j < hi; ++j) {
      float best = load_elem(in->data, oi.off, is_half);
      long where = 0;
      if (best == best) {
        for (long i = 1; i < n; ++i) {
          const float x = load_elem(in->data, oi.off + i * st, is_half);
          if (is_max ? !(x <= best) : !(x >= best)) {
            best = x;
            where = i;
            if (x != x) break;
          }
        }
      }
      if (is_half) ((uint16_t *)val->data)[ov.off] = th_float2half(best);
      else ((float *)val->data)[ov.off] = best;
      ((int64_t *)idx->data)[ox.off] = where + 1;
      odo_next(&ov, val);
      odo_next(&ox, idx);
      odo_next(&oi, &islice);
    }
  }
  return 0;
}

int th_max_dim_float(const th_view *val, const th_view *idx, const th_view *in, int dim) {
  return minmax_dim_impl(1, val, idx, in, dim, 0);
}
int th_min_dim_float(const th_view *val, const th_view *idx, const th_view *in, int dim) {
  return minmax_dim_impl(0, val, idx, in, dim, 0);
}
int th_max_dim_half(const th_view *val, const th_view *idx, const th_view *in, int dim) {
  return minmax_dim_impl(1, val, idx, in, dim, 1);
}
int th_min_dim_half(const th_view *val, const th_view *idx, const th_view *in, int dim) {
  return minmax_dim_impl(0, val, idx, in, dim, 1);
}

/* Whole-tensor reductions, sequential in logical order, double accumulator.
 * kind: TH_R_SUM / PROD / MIN / MAX / NORM(p) / MEAN. Returned as double; the
 * C API under test returns accreal = float, i.e. (float) of this value. */
static double reduce_all_impl(int kind, double p, const th_view *in, int is_half) {
  const long n = th_numel(in);
  if (n == 0) return kind == TH_R_PROD ? 1.0 : 0.0;
  if (kind == TH_R_MIN || kind == TH_R_MAX) {
    th_odo o;
    odo_seek(&o, in, 0);
    float best = load_elem(in->data, o.off, is_half);
    for (long i = 1; i < n && best == best; ++i) {
      odo_next(&o, in);
      const float x = load_elem(in->data, o.off, is_half);
      if (kind == TH_R_MAX ? !(x <= best) : !(x >= best)) best = x;
    }
    return best;
  }
  const int T = (kind == TH_R_PROD) ? 1 : g_threads; /* keep prod strictly sequential */
  double part[256];
  const int TT = T > 256 ? 256 : T;
#pragma omp parallel for num_threads(TT) schedule(static) if (TT > 1)
  for (int t = 0; t < TT; ++t) {
    const long lo = n * t / TT, hi = n * (t + 1) / TT;
    th_odo o;
    odo_seek(&o, in, lo);
    double acc = kind == TH_R_PROD ? 1.0 : 0.0;
    for (long i = lo; i < hi; ++i) {
      const double x = load_elem(in->data, o.off, is_half);
      switch (kind) {
        case TH_R_SUM: case TH_R_MEAN: acc += x; break;
        case TH_R_PROD: acc *= x; break;
        default:
          if (p == 0) acc += x != 0.0;
          else if (p == 1) acc += fabs(x);
          else if (p == 2) acc += x * x;
          else acc += pow(fabs(x), p);
      }
      odo_next(&o, in);
    }
    part[t] = acc;
  }
  double acc = part[0];
  for (int t = 1; t < TT; ++t) acc = kind == TH_R_PROD ? acc * part[t] : acc + part[t];
  if (kind == TH_R_MEAN) return acc / (double)n;
  if (kind == TH_R_NORM) {
    if (p == 0 || p == 1) return acc;
    if (p == 2) return sqrt(acc);
    return pow(acc, 1.0 / p);
  }
  return acc;
}

/* varall: mean first, then the sum of squared deviations (two sweeps, as
 * lib/THC/generic/THCTensorMathReduce.cu:122-144), divided by n or n-1. */
static double var_all_impl(const th_view *in, int biased, int is_half) {
  const long n = th_numel(in);
  const double mean = reduce_all_impl(TH_R_SUM, 0, in, is_half) / (double)n;
  th_odo o;
  odo_seek(&o, in, 0);
  double acc = 0;
  for (long i = 0; i < n; ++i) {
    const double d = load_elem(in->data, o.off, is_half) - mean;
    acc += d * d;
    odo_next(&o, in);
  }
  return acc / (double)(n - (biased ? 0 : 1));
}
double th_var_all_float(const th_view *in, int biased) { return var_all_impl(in, biased, 0); }
double th_var_all_half(const th_view *in, int biased) { return var_all_impl(in, biased, 1); }

double th_reduce_all_float(int kind, double p, const th_view *in) {
  return reduce_all_impl(kind, p, in, 0);
}
double th_reduce_all_half(int kind, double p, const th_view *in) {
  return reduce_all_impl(kind, p, in, 1);
}
