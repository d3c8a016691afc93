/*
 * th_oracle_types.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * CPU restatement of the pointwise, comparison and conversion semantics for
 * the element types beyond float/half: byte (unsigned char), char, short,
 * int, long and double. The reference instantiates one set of functors per
 * type (lib/THC/THCGenerateAllTypes.h:9-30); their arithmetic is C's on the
 * element type (lib/THC/THCNumerics.cuh:16-113):
 *   - byte/char/short operands are promoted to int, the result is converted
 *     back to the element type (wraps); int and long wrap in two's complement;
 *   - integer division truncates toward zero; fmod has the sign of the
 *     dividend, remainder the sign of the divisor
 *     (lib/THC/THCTensorMathPairwise.cu:244-258,329-340);
 *   - double uses libm in double precision;
 *   - comparisons give 0/1 (lib/THC/THCTensorMathCompare.cuh:10-74);
 *   - conversions are C casts, half goes through float
 *     (lib/THC/THCTensorCopy.cu:11-22 CopyOp, THCNumerics.cuh ScalarConvert).
 * Division by zero and shifts by out-of-range counts are undefined in the
 * reference; here x/0 = 0, x%0 = 0 and shift counts are taken modulo the
 * compute width (32 bits, 64 for long), the same choice as the engine, and the
 * tests keep away from them anyway.
 *
 * Pinned by tests/test_types.py against numpy's fixed-width integer
 * arithmetic (wrapping add/sub/mul, numpy.fix of the true quotient,
 * numpy.fmod, numpy.remainder, bit ops, astype casts) and float64 ufuncs.
 *
 * Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may
 * load this library.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#define TH_MAX_DIMS 25
typedef struct {
  void *data;
  int nd;
  const long *size;
  const long *stride;
} th_view;

uint16_t th_float2half(float f);
float th_half2float(uint16_t h);

/* same numbering as the engine's element type codes */
enum { T_F32 = 0, T_F16, T_I64, T_U8, T_I8, T_I16, T_I32, T_F64 };
enum { OP_ADDC = 1, OP_SUBC, OP_MULC, OP_DIVC, OP_ADD, OP_SUB, OP_MUL, OP_DIV, OP_CADD, OP_ADDCMUL,
       OP_ADDCDIV, OP_FILL, OP_POW, OP_LERP, OP_MATH1 = 100, OP_MATH2 = 200 };
/* function codes: first 41 as in th_oracle.c, then the shift / bit family */
enum { FN_SIGMOID = 0, FN_LOG, FN_LGAMMA, FN_LOG1P, FN_EXP, FN_COS, FN_ACOS, FN_COSH, FN_SIN, FN_ASIN,
       FN_SINH, FN_TAN, FN_ATAN, FN_TANH, FN_SQRT, FN_RSQRT, FN_CEIL, FN_FLOOR, FN_ROUND, FN_TRUNC,
       FN_FRAC, FN_CINV, FN_NEG, FN_ABS, FN_SIGN, FN_CLAMP, FN_SQDIFFVALUE, FN_POWSCALAR, FN_TPOW,
       FN_MAXVALUE, FN_MINVALUE, FN_FMODVALUE, FN_REMAINDERVALUE, FN_CPOW, FN_CMAX, FN_CMIN, FN_CFMOD,
       FN_CREMAINDER, FN_ATAN2, FN_EQUAL, FN_SQDIFF, FN_LSHIFTVALUE, FN_RSHIFTVALUE, FN_BITANDVALUE,
       FN_BITORVALUE, FN_BITXORVALUE, FN_CLSHIFT, FN_CRSHIFT, FN_CBITAND, FN_CBITOR, FN_CBITXOR };
enum { CMP_LT = 0, CMP_GT, CMP_LE, CMP_GE, CMP_EQ, CMP_NE };

static long numel(const th_view *v) {
  if (v->nd == 0) return 0;
  long n = 1;
  for (int d = 0; d < v->nd; ++d) n *= v->size[d];
  return n;
}
typedef struct { long idx[TH_MAX_DIMS]; long off; } odo;
static void odo_start(odo *o) { memset(o, 0, sizeof(*o)); }
static void odo_next(odo *o, const th_view *v) {
  for (int d = v->nd - 1; d >= 0; --d) {
    o->off += v->stride[d];
    if (++o->idx[d] < v->size[d]) return;
    o->off -= o->idx[d] * v->stride[d];
    o->idx[d] = 0;
  }
}

static int is_float_type(int t) { return t == T_F32 || t == T_F16 || t == T_F64; }

/* element <-> (int64 | double) */
static int64_t load_i(int t, const void *p, long off) {
  switch (t) {
    case T_U8: return ((const uint8_t *)p)[off];
    case T_I8: return ((const int8_t *)p)[off];
    case T_I16: return ((const int16_t *)p)[off];
    case T_I32: return ((const int32_t *)p)[off];
    default: return ((const int64_t *)p)[off];
  }
}
static double load_f(int t, const void *p, long off) {
  switch (t) {
    case T_F32: return ((const float *)p)[off];
    case T_F16: return th_half2float(((const uint16_t *)p)[off]);
    default: return ((const double *)p)[off];
  }
}
/* store with the element type's own conversion (wrap for integers) */
static void store_i(int t, void *p, long off, int64_t v) {
  switch (t) {
    case T_U8: ((uint8_t *)p)[off] = (uint8_t)v; break;
    case T_I8: ((int8_t *)p)[off] = (int8_t)v; break;
    case T_I16: ((int16_t *)p)[off] = (int16_t)v; break;
    case T_I32: ((int32_t *)p)[off] = (int32_t)v; break;
    default: ((int64_t *)p)[off] = v; break;
  }
}
static void store_f(int t, void *p, long off, double v) {
  switch (t) {
    case T_F32: ((float *)p)[off] = (float)v; break;
    case T_F16: ((uint16_t *)p)[off] = th_float2half((float)v); break;
    default: ((double *)p)[off] = v; break;
  }
}

/* ------------------------------------------------------ integer arithmetic */
/* int / long results wrap; the narrow types compute in int (C promotion) and
 * wrap on store, which is the same as computing in 64 bits and truncating for
 * add, sub, mul. Computing in the promoted width matters for /, %, shifts and
 * comparisons, where operands this small never overflow the promoted type. */
static int width_of(int t) { return t == T_I64 ? 64 : 32; }
static int64_t wrap_to(int t, int64_t v) { return t == T_I64 ? v : (int64_t)(int32_t)v; }
static int64_t iadd(int t, int64_t a, int64_t b) { return wrap_to(t, (int64_t)((uint64_t)a + (uint64_t)b)); }
static int64_t isub(int t, int64_t a, int64_t b) { return wrap_to(t, (int64_t)((uint64_t)a - (uint64_t)b)); }
static int64_t imul(int t, int64_t a, int64_t b) { return wrap_to(t, (int64_t)((uint64_t)a * (uint64_t)b)); }
static int64_t idiv(int t, int64_t a, int64_t b) {
  if (b == 0) return 0;
  if (b == -1) return isub(t, 0, a);
  return a / b;
}
static int64_t imod(int64_t a, int64_t b) { return (b == 0 || b == -1) ? 0 : a % b; }
static int64_t ipow(int t, int64_t a, int64_t e) {
  if (e < 0) return a == 1 ? 1 : (a == -1 ? ((e & 1) ? -1 : 1) : 0);
  int64_t r = 1;
  while (e) {
    if (e & 1) r = imul(t, r, a);
    a = imul(t, a, a);
    e >>= 1;
  }
  return r;
}
static int64_t iremainder(int t, int64_t a, int64_t b) {
  int64_t r = imod(a, b);
  if (r != 0 && ((r < 0) != (b < 0))) r = iadd(t, r, b);
  return r;
}
static int64_t ishl(int t, int64_t a, int64_t n) {
  n &= width_of(t) - 1;
  return wrap_to(t, (int64_t)((uint64_t)a << n));
}
static int64_t ishr(int t, int64_t a, int64_t n) {
  n &= width_of(t) - 1;
  return a >> n; /* arithmetic on the promoted (sign-extended) value */
}

static int64_t int_point(int t, int op, int fn, int64_t v, int64_t w, int64_t a, int64_t b, int64_t c) {
  switch (op) {
    case OP_FILL: return v;
    case OP_ADDC: return iadd(t, a, v);
    case OP_SUBC: return isub(t, a, v);
    case OP_MULC: return imul(t, a, v);
    case OP_DIVC: return idiv(t, a, v);
    case OP_ADD: return iadd(t, a, b);
    case OP_SUB: return isub(t, a, b);
    case OP_MUL: return imul(t, a, b);
    case OP_DIV: return idiv(t, a, b);
    case OP_CADD: return iadd(t, a, imul(t, v, b));
    case OP_ADDCMUL: return iadd(t, a, imul(t, v, imul(t, b, c)));
    case OP_ADDCDIV: return iadd(t, a, imul(t, v, idiv(t, b, c)));
    case OP_MATH1:
      switch (fn) {
        case FN_NEG: return isub(t, 0, a);
        case FN_ABS: return a < 0 ? isub(t, 0, a) : a;
        case FN_SIGN: return (a > 0) - (a < 0);
        case FN_CLAMP: return a < v ? v : (a > w ? w : a);
        case FN_POWSCALAR: return ipow(t, a, v);
        case FN_TPOW: return ipow(t, v, a);
        case FN_MAXVALUE: return a > v ? a : v;
        case FN_MINVALUE: return a < v ? a : v;
        case FN_FMODVALUE: return imod(a, v);
        case FN_REMAINDERVALUE: return iremainder(t, a, v);
        case FN_LSHIFTVALUE: return ishl(t, a, v);
        case FN_RSHIFTVALUE: return ishr(t, a, v);
        case FN_BITANDVALUE: return a & v;
        case FN_BITORVALUE: return a | v;
        case FN_BITXORVALUE: return a ^ v;
      }
      return a;
    case OP_MATH2:
      switch (fn) {
        case FN_CPOW: return ipow(t, a, b);
        case FN_CMAX: return a > b ? a : b;
        case FN_CMIN: return a < b ? a : b;
        case FN_CFMOD: return imod(a, b);
        case FN_CREMAINDER: return iremainder(t, a, b);
        case FN_EQUAL: return a == b;
        case FN_CLSHIFT: return ishl(t, a, b);
        case FN_CRSHIFT: return ishr(t, a, b);
        case FN_CBITAND: return a & b;
        case FN_CBITOR: return a | b;
        case FN_CBITXOR: return a ^ b;
      }
      return a;
  }
  return a;
}

/* ------------------------------------------------------- double arithmetic */
static double dbl_point(int op, int fn, double v, double w, double a, double b, double c) {
  switch (op) {
    case OP_FILL: return v;
    case OP_ADDC: return a + v;
    case OP_SUBC: return a - v;
    case OP_MULC: return a * v;
    case OP_DIVC: return a / v;
    case OP_ADD: return a + b;
    case OP_SUB: return a - b;
    case OP_MUL: return a * b;
    case OP_DIV: return a / b;
    case OP_CADD: { double t = v * b; return a + t; }
    case OP_LERP: { double t = b - a; t = v * t; return a + t; }
    case OP_ADDCMUL: { double t = b * c; t = v * t; return a + t; }
    case OP_ADDCDIV: { double t = b / c; t = v * t; return a + t; }
    case OP_MATH1:
      switch (fn) {
        case FN_SIGMOID: return 1.0 / (1.0 + exp(-a));
        case FN_LOG: return log(a);
        case FN_LGAMMA: return lgamma(a);
        case FN_LOG1P: return log1p(a);
        case FN_EXP: return exp(a);
        case FN_COS: return cos(a);
        case FN_ACOS: return acos(a);
        case FN_COSH: return cosh(a);
        case FN_SIN: return sin(a);
        case FN_ASIN: return asin(a);
        case FN_SINH: return sinh(a);
        case FN_TAN: return tan(a);
        case FN_ATAN: return atan(a);
        case FN_TANH: return tanh(a);
        case FN_SQRT: return sqrt(a);
        case FN_RSQRT: return 1.0 / sqrt(a);
        case FN_CEIL: return ceil(a);
        case FN_FLOOR: return floor(a);
        case FN_ROUND: return round(a);
        case FN_TRUNC: return trunc(a);
        case FN_FRAC: return a - trunc(a);
        case FN_CINV: return 1.0 / a;
        case FN_NEG: return -a;
        case FN_ABS: return fabs(a);
        case FN_SIGN: return (double)((a > 0) - (a < 0));
        case FN_CLAMP: return a < v ? v : (a > w ? w : a);
        case FN_POWSCALAR: return pow(a, v);
        case FN_TPOW: return pow(v, a);
        case FN_MAXVALUE: return a > v ? a : v;
        case FN_MINVALUE: return a < v ? a : v;
        case FN_FMODVALUE: return fmod(a, v);
        case FN_REMAINDERVALUE: return v == 0.0 ? NAN : a - v * floor(a / v);
        case FN_LSHIFTVALUE: return a * pow(2.0, v);
        case FN_RSHIFTVALUE: return a / pow(2.0, v);
      }
      return a;
    case OP_MATH2:
      switch (fn) {
        case FN_CPOW: return pow(a, b);
        case FN_CMAX: return a > b ? a : b;
        case FN_CMIN: return a < b ? a : b;
        case FN_CFMOD: return fmod(a, b);
        case FN_CREMAINDER: return b == 0.0 ? NAN : a - b * floor(a / b);
        case FN_ATAN2: return atan2(a, b);
        case FN_EQUAL: return a == b;
        case FN_CLSHIFT: return a * pow(2.0, b);
        case FN_CRSHIFT: return a / pow(2.0, b);
      }
      return a;
  }
  return a;
}

static int n_inputs(int op, int fn) {
  (void)fn;
  if (op == OP_FILL) return 0;
  if (op == OP_MATH2 || op == OP_LERP) return 2;
  if (op == OP_MATH1 || op <= OP_DIVC || op == OP_POW) return 1;
  if (op <= OP_CADD) return 2;
  return 3;
}

/* out[i] = op(a[i], b[i], c[i]) on byte/char/short/int/long/double views.
 * Integer scalars arrive in vi/wi (already of the element type's range),
 * double scalars in vf/wf. Returns 1 if element counts differ. */
int th_typed_pointwise(int t, int op, int fn, double vf, long vi, double wf, long wi,
                       const th_view *out, const th_view *a, const th_view *b, const th_view *c) {
  const int nin = n_inputs(op, fn);
  const th_view *in[3] = {a, b, c};
  const long n = numel(out);
  for (int k = 0; k < nin; ++k)
    if (numel(in[k]) != n) return 1;
  odo oo, oi[3];
  odo_start(&oo);
  for (int k = 0; k < 3; ++k) odo_start(&oi[k]);
  for (long i = 0; i < n; ++i) {
    if (t == T_F64) {
      double x[3] = {0, 0, 0};
      for (int k = 0; k < nin; ++k) x[k] = load_f(t, in[k]->data, oi[k].off);
      store_f(t, out->data, oo.off, dbl_point(op, fn, vf, wf, x[0], x[1], x[2]));
    } else {
      int64_t x[3] = {0, 0, 0};
      for (int k = 0; k < nin; ++k) x[k] = load_i(t, in[k]->data, oi[k].off);
      store_i(t, out->data, oo.off, int_point(t, op, fn, vi, wi, x[0], x[1], x[2]));
    }
    odo_next(&oo, out);
    for (int k = 0; k < nin; ++k) odo_next(&oi[k], in[k]);
  }
  return 0;
}

/* out[i] = a[i] (cmp) (b ? b[i] : value) as 0/1 stored with out's type
 * (T_U8 for the Byte forms, t for the ...T forms). Works for all 8 types. */
int th_typed_compare(int t, int outT, int cmp, double vf, long vi, const th_view *out,
                     const th_view *a, const th_view *b) {
  const long n = numel(out);
  if (numel(a) != n || (b && numel(b) != n)) return 1;
  odo oo, oa, ob;
  odo_start(&oo);
  odo_start(&oa);
  odo_start(&ob);
  for (long i = 0; i < n; ++i) {
    int r;
    if (is_float_type(t)) {
      /* half scalars are compared as the float they convert to */
      const double x = load_f(t, a->data, oa.off), y = b ? load_f(t, b->data, ob.off) : vf;
      r = cmp == CMP_LT ? x < y : cmp == CMP_GT ? x > y : cmp == CMP_LE ? x <= y
        : cmp == CMP_GE ? x >= y : cmp == CMP_EQ ? x == y : x != y;
    } else {
      const int64_t x = load_i(t, a->data, oa.off), y = b ? load_i(t, b->data, ob.off) : (int64_t)vi;
      r = cmp == CMP_LT ? x < y : cmp == CMP_GT ? x > y : cmp == CMP_LE ? x <= y
        : cmp == CMP_GE ? x >= y : cmp == CMP_EQ ? x == y : x != y;
    }
    if (is_float_type(outT)) store_f(outT, out->data, oo.off, r);
    else store_i(outT, out->data, oo.off, r);
    odo_next(&oo, out);
    odo_next(&oa, a);
    if (b) odo_next(&ob, b);
  }
  return 0;
}

/* dst[i] = (dst's type) src[i], paired by logical linear index. C casts; half
 * goes through float in both directions. */
int th_typed_convert(int dstT, const th_view *dst, int srcT, const th_view *src) {
  const long n = numel(dst);
  if (numel(src) != n) return 1;
  odo od, os;
  odo_start(&od);
  odo_start(&os);
  for (long i = 0; i < n; ++i) {
    if (is_float_type(srcT)) {
      const double x = load_f(srcT, src->data, os.off);
      if (is_float_type(dstT)) {
        if (dstT == T_F16 && srcT == T_F64) store_f(dstT, dst->data, od.off, (double)(float)x);
        else store_f(dstT, dst->data, od.off, x);
      } else if (srcT == T_F64) {
        /* C cast from double at the destination's own width */
        switch (dstT) {
          case T_U8: ((uint8_t *)dst->data)[od.off] = (uint8_t)x; break;
          case T_I8: ((int8_t *)dst->data)[od.off] = (int8_t)x; break;
          case T_I16: ((int16_t *)dst->data)[od.off] = (int16_t)x; break;
          case T_I32: ((int32_t *)dst->data)[od.off] = (int32_t)x; break;
          default: ((int64_t *)dst->data)[od.off] = (int64_t)x; break;
        }
      } else {
        const float xf = (float)x;
        switch (dstT) {
          case T_U8: ((uint8_t *)dst->data)[od.off] = (uint8_t)xf; break;
          case T_I8: ((int8_t *)dst->data)[od.off] = (int8_t)xf; break;
          case T_I16: ((int16_t *)dst->data)[od.off] = (int16_t)xf; break;
          case T_I32: ((int32_t *)dst->data)[od.off] = (int32_t)xf; break;
          default: ((int64_t *)dst->data)[od.off] = (int64_t)xf; break;
        }
      }
    } else {
      const int64_t x = load_i(srcT, src->data, os.off);
      if (dstT == T_F16) store_f(dstT, dst->data, od.off, (double)(float)x);
      else if (dstT == T_F32) ((float *)dst->data)[od.off] = (float)x;
      else if (dstT == T_F64) ((double *)dst->data)[od.off] = (double)x;
      else store_i(dstT, dst->data, od.off, x);
    }
    odo_next(&od, dst);
    odo_next(&os, src);
  }
  return 0;
}

/* ------------------------------------------------------------ reductions -- */
/* Integer types accumulate in long (accreal = long, lib/THC/THCGenerate*Type.h)
 * with two's complement wrap-around; the stored result wraps in the element
 * type. Double accumulates sequentially in long double and rounds once, which
 * pins a sum to within half an ulp of the exact value. mean = sum converted to
 * the element type, divided by the size converted to the element type
 * (lib/THC/generic/THCTensorMathReduce.cu:37-43). */
enum { RK_SUM = 0, RK_PROD, RK_MIN, RK_MAX, RK_MEAN };

static void reduce_slice_typed(int t, int kind, const void *base, long off, long n, long stride,
                               int64_t *ri, double *rf) {
  if (t == T_F64) {
    long double acc = kind == RK_PROD ? 1.0L : 0.0L;
    double best = 0;
    for (long i = 0; i < n; ++i) {
      const double x = ((const double *)base)[off + i * stride];
      if (kind == RK_SUM || kind == RK_MEAN) acc += x;
      else if (kind == RK_PROD) acc *= x;
      else if (i == 0) best = x;
      else if (best == best) { /* the first NaN stays */
        if (x != x) best = x;
        else if (kind == RK_MIN ? x < best : x > best) best = x;
      }
    }
    if (kind == RK_MIN || kind == RK_MAX) *rf = best;
    else if (kind == RK_MEAN) *rf = (double)acc / (double)n;
    else *rf = (double)acc;
    return;
  }
  uint64_t acc = kind == RK_PROD ? 1 : 0;
  int64_t best = 0;
  for (long i = 0; i < n; ++i) {
    const int64_t x = load_i(t, base, off + i * stride);
    if (kind == RK_SUM || kind == RK_MEAN) acc += (uint64_t)x;
    else if (kind == RK_PROD) acc *= (uint64_t)x;
    else if (i == 0) best = x;
    else if (kind == RK_MIN ? x < best : x > best) best = x;
  }
  *ri = (kind == RK_MIN || kind == RK_MAX) ? best : (int64_t)acc;
}

/* truncate v to the element type and widen again */
static int64_t as_type(int t, int64_t v) {
  switch (t) {
    case T_U8: return (uint8_t)v;
    case T_I8: return (int8_t)v;
    case T_I16: return (int16_t)v;
    case T_I32: return (int32_t)v;
    default: return v;
  }
}

int th_typed_reduce_dim(int t, int kind, const th_view *out, const th_view *in, int dim) {
  if (in->nd == 0) return 0;
  if (out->nd != in->nd || dim < 0 || dim >= in->nd) return 1;
  long osz[TH_MAX_DIMS];
  for (int d = 0; d < in->nd; ++d) {
    osz[d] = d == dim ? 1 : in->size[d];
    if (out->size[d] != osz[d]) return 1;
  }
  th_view il = *in;
  il.size = osz;
  const long lines = numel(out), n = in->size[dim];
  odo oi, oo;
  odo_start(&oi);
  odo_start(&oo);
  for (long l = 0; l < lines; ++l) {
    int64_t ri = 0;
    double rf = 0;
    reduce_slice_typed(t, kind, in->data, oi.off, n, in->stride[dim], &ri, &rf);
    if (t == T_F64) store_f(t, out->data, oo.off, rf);
    else if (kind == RK_MEAN) store_i(t, out->data, oo.off, as_type(t, ri) / as_type(t, n));
    else store_i(t, out->data, oo.off, ri);
    odo_next(&oi, &il);
    odo_next(&oo, out);
  }
  return 0;
}

/* (value, 1-based index of the first occurrence) of the max / min along dim */
int th_typed_minmax_dim(int t, int is_max, const th_view *val, const th_view *idx, const th_view *in,
                        int dim) {
  if (in->nd == 0) return 0;
  if (val->nd != in->nd || idx->nd != in->nd || dim < 0 || dim >= in->nd) return 1;
  long osz[TH_MAX_DIMS];
  for (int d = 0; d < in->nd; ++d) osz[d] = d == dim ? 1 : in->size[d];
  th_view il = *in;
  il.size = osz;
  const long lines = numel(val), n = in->size[dim], st = in->stride[dim];
  odo oi, ov, ox;
  odo_start(&oi);
  odo_start(&ov);
  odo_start(&ox);
  for (long l = 0; l < lines; ++l) {
    long at = 0;
    if (t == T_F64) {
      double best = ((const double *)in->data)[oi.off];
      for (long i = 1; i < n && best == best; ++i) {
        const double x = ((const double *)in->data)[oi.off + i * st];
        if (x != x || (is_max ? x > best : x < best)) { best = x; at = i; }
      }
      ((double *)val->data)[ov.off] = best;
    } else {
      int64_t best = load_i(t, in->data, oi.off);
      for (long i = 1; i < n; ++i) {
        const int64_t x = load_i(t, in->data, oi.off + i * st);
        if (is_max ? x > best : x < best) { best = x; at = i; }
      }
      store_i(t, val->data, ov.off, best);
    }
    ((int64_t *)idx->data)[ox.off] = at + 1;
    odo_next(&oi, &il);
    odo_next(&ov, val);
    odo_next(&ox, idx);
  }
  return 0;
}

/* Whole-tensor reduction in logical order; integer result in *ri (accreal =
 * long), double result returned. */
double th_typed_reduce_all(int t, int kind, const th_view *in, long *ri_out) {
  const long n = numel(in);
  odo o;
  odo_start(&o);
  long double acc = kind == RK_PROD ? 1.0L : 0.0L;
  uint64_t iacc = kind == RK_PROD ? 1 : 0;
  double bestf = 0;
  int64_t besti = 0;
  for (long i = 0; i < n; ++i) {
    if (t == T_F64) {
      const double x = ((const double *)in->data)[o.off];
      if (kind == RK_SUM || kind == RK_MEAN) acc += x;
      else if (kind == RK_PROD) acc *= x;
      else if (i == 0) bestf = x;
      else if (bestf == bestf) {
        if (x != x) bestf = x;
        else if (kind == RK_MIN ? x < bestf : x > bestf) bestf = x;
      }
    } else {
      const int64_t x = load_i(t, in->data, o.off);
      if (kind == RK_SUM || kind == RK_MEAN) iacc += (uint64_t)x;
      else if (kind == RK_PROD) iacc *= (uint64_t)x;
      else if (i == 0) besti = x;
      else if (kind == RK_MIN ? x < besti : x > besti) besti = x;
    }
    odo_next(&o, in);
  }
  if (t == T_F64) {
    if (kind == RK_MIN || kind == RK_MAX) return bestf;
    if (kind == RK_MEAN) return (double)acc / (double)n;
    return (double)acc;
  }
  int64_t r = (kind == RK_MIN || kind == RK_MAX) ? besti : (int64_t)iacc;
  if (kind == RK_MEAN) r = r / n;   /* accreal division (sumall / nElement) */
  *ri_out = r;
  return (double)r;
}

/* ------------------------------------------------------------------ scans -- */
/* Inclusive prefix sum / product along dim for the integer types (64-bit
 * wrapping accumulator, stored wrapped to the element type) and double
 * (sequential long double accumulator, rounded per element). Entry semantics
 * as lib/THC/generic/THCTensorMathScan.cu:76-126. */
int th_typed_scan_dim(int t, int product, const th_view *out, const th_view *in, int dim) {
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
  const long lines = numel(&il), n = in->size[dim];
  odo oi, oo;
  odo_start(&oi);
  odo_start(&oo);
  for (long l = 0; l < lines; ++l) {
    long double facc = product ? 1.0L : 0.0L;
    uint64_t iacc = product ? 1 : 0;
    for (long i = 0; i < n; ++i) {
      const long src = oi.off + i * in->stride[dim], dst = oo.off + i * out->stride[dim];
      if (t == T_F64) {
        const double x = ((const double *)in->data)[src];
        facc = product ? facc * x : facc + x;
        ((double *)out->data)[dst] = (double)facc;
      } else {
        const uint64_t x = (uint64_t)load_i(t, in->data, src);
        iacc = product ? iacc * x : iacc + x;
        store_i(t, out->data, dst, (int64_t)iacc);
      }
    }
    odo_next(&oi, &il);
    odo_next(&oo, &ol);
  }
  return 0;
}

/* ----------------------------------------------------------------- renorm -- */
/* out = in with every slice along `dim` whose p-norm exceeds maxnorm scaled by
 * maxnorm / (norm + 1e-7) (lib/THC/THCTensorMathReduce.cuh:132-178,
 * generic/THCTensorMathReduce.cu:46-74). float, half or double views; the norm
 * and the factor are computed in (long) double, each output rounded once. */
int th_renorm(int t, const th_view *out, const th_view *in, double p, int dim, double maxnorm) {
  if (in->nd < 2 || out->nd != in->nd || dim < 0 || dim >= in->nd) return 1;
  long ssz[TH_MAX_DIMS];
  for (int d = 0; d < in->nd; ++d) {
    if (out->size[d] != in->size[d]) return 1;
    ssz[d] = d == dim ? 1 : in->size[d];
  }
  for (long i = 0; i < in->size[dim]; ++i) {
    th_view is = *in, os = *out;
    is.size = ssz;
    os.size = ssz;
    const long ibase = i * in->stride[dim], obase = i * out->stride[dim];
    const long n = numel(&is);
    odo o1;
    odo_start(&o1);
    long double acc = 0;
    for (long k = 0; k < n; ++k) {
      acc += powl(fabsl((long double)load_f(t, in->data, ibase + o1.off)), (long double)p);
      odo_next(&o1, &is);
    }
    const double norm = (double)powl(acc, 1.0L / (long double)p);
    const double factor = norm > maxnorm ? maxnorm / (norm + 1e-7) : 1.0;
    odo oi, oo;
    odo_start(&oi);
    odo_start(&oo);
    for (long k = 0; k < n; ++k) {
      store_f(t, out->data, obase + oo.off, load_f(t, in->data, ibase + oi.off) * factor);
      odo_next(&oi, &is);
      odo_next(&oo, &os);
    }
  }
  return 0;
}
