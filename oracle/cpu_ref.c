/*
 * TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.
 *
 * CPU restatement of the reference's `cpu_ref` tensor path (TypeScript, single thread):
 * f32 storage, every intermediate in f64 (a JS `number`), loops in the reference's order.
 * Only tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py may load this
 * library; nothing under alpha2_amd/ does.
 *
 * Each function cites the reference lines it restates (paths relative to the reference root).
 *
 * Pinning status (see tests/test_oracle_*.py):
 *   - ops: pinned by the reference's own known answers (packages/tests/src/tensor.test.ts,
 *     autograd.test.ts, optimizer.test.ts, memory-leak.test.ts, gpu-perf.test.ts) and by
 *     PyTorch-CPU float64 library routines / closed forms.
 *   - orc_rng_*: integer stream pinned by an independent Python big-int restatement
 *     (bit-exact); the reference holds no golden stream -> "parity unpinned" against a
 *     reference run for the exact values of nextGauss (libm last-ulp).
 *   - orc_dropout_mask: restates the f64-multiply-then-|0 hash; pinned by an independent
 *     Python restatement (doubles + big ints, every index range incl. products past 2^53)
 *     and by the published MurmurHash3 fmix32 known answers for its mixing rounds.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_MAX_DIMS 8

/* ------------------------------------------------------------------------------------------
 * helpers: packages/core/src/types.ts:34-48 (shapeSize / shapeStrides)
 * ---------------------------------------------------------------------------------------- */
static int64_t shape_size(const int64_t *shape, int nd) {
  int64_t s = 1;
  for (int i = 0; i < nd; i++) s *= shape[i];
  return s;
}
static void shape_strides(const int64_t *shape, int nd, int64_t *strides) {
  int64_t st = 1;
  for (int i = nd - 1; i >= 0; i--) { strides[i] = st; st *= shape[i]; }
}

/* ------------------------------------------------------------------------------------------
 * SeededRng: packages/core/src/rng.ts:6-68.  State is two int32; all shifts are JS int32
 * shifts (<< wraps, >>> is logical); next() = ((s0+s1)>>>0) / 2^32.
 * ---------------------------------------------------------------------------------------- */
typedef struct { int32_t s0, s1; int has_spare; double spare; } orc_rng;

double orc_rng_next(orc_rng *r) {               /* rng.ts:38-50 */
  uint32_t s1 = (uint32_t)r->s0;
  const uint32_t s0 = (uint32_t)r->s1;
  r->s0 = (int32_t)s0;
  s1 ^= s1 << 23;
  s1 ^= s1 >> 17;
  s1 ^= s0;
  s1 ^= s0 >> 26;
  r->s1 = (int32_t)s1;
  /* JS: (this._s0 + this._s1) is an f64 sum of two int32, then >>>0 wraps modulo 2^32 */
  uint32_t sum = (uint32_t)((int64_t)r->s0 + (int64_t)r->s1);
  return (double)sum / 4294967296.0;
}
void orc_rng_seed(orc_rng *r, int32_t seed) {   /* rng.ts:13-28 */
  r->s0 = seed;
  r->s1 = seed ^ (int32_t)0xdeadbeef;
  r->has_spare = 0; r->spare = 0;
  for (int i = 0; i < 20; i++) orc_rng_next(r);
}
double orc_rng_next_gauss(orc_rng *r) {         /* rng.ts:53-67 (polar Box-Muller, cached spare) */
  if (r->has_spare) { r->has_spare = 0; return r->spare; }
  double u, v, s;
  do {
    u = orc_rng_next(r) * 2 - 1;
    v = orc_rng_next(r) * 2 - 1;
    s = u * u + v * v;
  } while (s >= 1 || s == 0);
  const double mul = sqrt(-2.0 * log(s) / s);
  r->spare = v * mul; r->has_spare = 1;
  return u * mul;
}
/* initWeight: packages/model/src/gpt.ts:53-59 -- data[i] = nextGauss()*std rounded to f32 */
void orc_rng_fill_gauss(orc_rng *r, float *out, int64_t n, double std) {
  for (int64_t i = 0; i < n; i++) out[i] = (float)(orc_rng_next_gauss(r) * std);
}
void orc_rng_fill_uniform(orc_rng *r, double *out, int64_t n) {
  for (int64_t i = 0; i < n; i++) out[i] = orc_rng_next(r);
}

/* ------------------------------------------------------------------------------------------
 * Broadcasting binary ops: packages/tensor/src/cpu_ref.ts:55-72,150-164 with
 * packages/core/src/broadcast.ts:13-65.  op: 0 add, 1 sub, 2 mul, 3 div.
 * `out` has the broadcast result shape (returned through out_shape / *out_nd by the caller's
 * own computation; this routine recomputes it to drive the index walk).
 * Returns the result size, or -1 when the shapes cannot be broadcast.
 * ---------------------------------------------------------------------------------------- */
int64_t orc_broadcast_shape(const int64_t *sa, int na, const int64_t *sb, int nb,
                            int64_t *res, int64_t *stra, int64_t *strb) {
  int nd = na > nb ? na : nb;
  int padA = nd - na, padB = nd - nb;
  for (int i = 0; i < nd; i++) {
    int64_t da = i < padA ? 1 : sa[i - padA];
    int64_t db = i < padB ? 1 : sb[i - padB];
    if (da != db && da != 1 && db != 1) return -1;
    res[i] = da > db ? da : db;
  }
  int64_t strA = 1, strB = 1;
  for (int i = nd - 1; i >= 0; i--) {
    int64_t da = i < padA ? 1 : sa[i - padA];
    int64_t db = i < padB ? 1 : sb[i - padB];
    stra[i] = (da == 1 && res[i] != 1) ? 0 : strA;
    strb[i] = (db == 1 && res[i] != 1) ? 0 : strB;
    strA *= da; strB *= db;
  }
  return shape_size(res, nd);
}

int64_t orc_binary(int op, const float *a, const int64_t *sa, int na,
                   const float *b, const int64_t *sb, int nb, float *out) {
  int64_t res[ORC_MAX_DIMS], stra[ORC_MAX_DIMS], strb[ORC_MAX_DIMS];
  int nd = na > nb ? na : nb;
  int64_t size = orc_broadcast_shape(sa, na, sb, nb, res, stra, strb);
  if (size < 0) return -1;
  for (int64_t i = 0; i < size; i++) {
    int64_t ia = 0, ib = 0, rem = i;
    for (int d = nd - 1; d >= 0; d--) {
      int64_t c = rem % res[d];
      rem = (rem - c) / res[d];
      ia += c * stra[d]; ib += c * strb[d];
    }
    double x = a[ia], y = b[ib], r;
    switch (op) { case 0: r = x + y; break; case 1: r = x - y; break;
                  case 2: r = x * y; break; default: r = x / y; }
    out[i] = (float)r;
  }
  return size;
}

/* ------------------------------------------------------------------------------------------
 * Unary ops: cpu_ref.ts:74-83, 334-360, 422-435.
 * op: 0 neg, 1 exp, 2 log, 3 sqrt, 4 pow(p0), 5 scale(p0), 6 clamp(p0,p1), 7 gelu, 8 relu, 9 silu
 * ---------------------------------------------------------------------------------------- */
void orc_unary(int op, const float *a, float *out, int64_t n, double p0, double p1) {
  const double SQRT_2_OVER_PI = sqrt(2.0 / M_PI);
  for (int64_t i = 0; i < n; i++) {
    double x = a[i], r;
    switch (op) {
      case 0: r = -x; break;
      case 1: r = exp(x); break;
      case 2: r = log(x); break;
      case 3: r = sqrt(x); break;
      case 4: r = pow(x, p0); break;
      case 5: r = x * p0; break;
      case 6: { double m = p1 < x ? p1 : x; r = p0 > m ? p0 : m; } break; /* max(lo,min(hi,x)) */
      case 7: r = 0.5 * x * (1 + tanh(SQRT_2_OVER_PI * (x + 0.044715 * x * x * x))); break;
      case 8: r = x > 0 ? x : 0; break;
      default: r = x / (1 + exp(-x)); break;
    }
    out[i] = (float)r;
  }
}

/* ------------------------------------------------------------------------------------------
 * matmul: cpu_ref.ts:166-258.  One call handles `batch` [M,K]x[K,N] products whose operand
 * offsets (already resolved from the broadcast batch dims by the caller exactly as
 * cpu_ref.ts:231-243 does) are a_off[b], b_off[b].  m-n-k loop, f64 accumulator.
 * ---------------------------------------------------------------------------------------- */
void orc_matmul(const float *a, const float *b, float *out, int64_t batch,
                const int64_t *a_off, const int64_t *b_off, int64_t M, int64_t K, int64_t N) {
  for (int64_t bt = 0; bt < batch; bt++) {
    const float *ad = a + a_off[bt], *bd = b + b_off[bt];
    float *od = out + bt * M * N;
    for (int64_t m = 0; m < M; m++)
      for (int64_t n = 0; n < N; n++) {
        double sum = 0;
        for (int64_t k = 0; k < K; k++) sum += (double)ad[m * K + k] * (double)bd[k * N + n];
        od[m * N + n] = (float)sum;
      }
  }
}

/* ------------------------------------------------------------------------------------------
 * sum / mean: cpu_ref.ts:260-330.  axis < 0 means "all elements" (axis === undefined).
 * ---------------------------------------------------------------------------------------- */
void orc_sum_all(const float *a, int64_t n, float *out, int mean) {
  double s = 0;
  for (int64_t i = 0; i < n; i++) s += a[i];
  out[0] = (float)(mean ? s / (double)n : s);
}
void orc_sum_axis(const float *a, const int64_t *shape, int nd, int ax, float *out, int mean) {
  int64_t strides[ORC_MAX_DIMS];
  shape_strides(shape, nd, strides);
  int64_t dim = shape[ax], axs = strides[ax];
  int64_t outer = 1;                          /* the other dimensions' product (cpu_ref.ts:272-280): an empty reduced axis gives */
  for (int d = 0; d < nd; d++)                /* one zero per output (mean: 0 / 0), and no division by its length here        */
    if (d != ax) outer *= shape[d];
  /* output flat index -> coords over the non-reduced dims (row-major), as flatToMulti does */
  for (int64_t i = 0; i < outer; i++) {
    int64_t rem = i, base = 0;
    for (int d = nd - 1; d >= 0; d--) {
      if (d == ax) continue;
      int64_t c = rem % shape[d];
      rem = (rem - c) / shape[d];
      base += c * strides[d];
    }
    double s = 0;
    for (int64_t j = 0; j < dim; j++) s += a[base + j * axs];
    float sf = (float)s;                      /* sum() stores f32 ... */
    if (mean) sf = (float)((double)sf / (double)dim);  /* ... mean() divides the stored f32 (cpu_ref.ts:324-328) */
    out[i] = sf;
  }
}

/* embedding: cpu_ref.ts:364-385 */
void orc_embedding(const float *w, int64_t dim, int64_t vocab, const int32_t *idx, int64_t n, float *out) {
  for (int64_t i = 0; i < n; i++) {
    int64_t src = (int64_t)idx[i] * dim, dst = i * dim;
    /* an element outside the weight array reads as undefined and is stored as NaN (typed-array semantics of the loop) */
    for (int64_t d = 0; d < dim; d++) out[dst + d] = (src + d >= 0 && src + d < vocab * dim) ? w[src + d] : NAN;
  }
}
/* embedding backward (scatter-add, sequential in index order): packages/autograd/src/ops.ts:495-505 */
void orc_embedding_bwd(const int32_t *idx, int64_t n, const float *g, int64_t dim,
                       int64_t vocab, float *grad /* [vocab,dim], zero-filled here */) {
  memset(grad, 0, sizeof(float) * (size_t)(vocab * dim));
  for (int64_t i = 0; i < n; i++) {
    int64_t r = idx[i];
    for (int64_t d = 0; d < dim; d++) {
      int64_t f = r * dim + d;
      if (f < 0 || f >= vocab * dim) continue;    /* a store past either end of a typed array is dropped */
      grad[f] = (float)((double)grad[f] + (double)g[i * dim + d]); /* Float32Array += */
    }
  }
}

/* layerNorm forward: cpu_ref.ts:387-420 */
void orc_layernorm(const float *x, const float *w, const float *b, double eps,
                   int64_t outer, int64_t dim, float *out) {
  for (int64_t i = 0; i < outer; i++) {
    int64_t off = i * dim;
    double mean = 0;
    for (int64_t j = 0; j < dim; j++) mean += x[off + j];
    mean /= (double)dim;
    double var = 0;
    for (int64_t j = 0; j < dim; j++) { double d = x[off + j] - mean; var += d * d; }
    var /= (double)dim;
    double inv = 1 / sqrt(var + eps);
    for (int64_t j = 0; j < dim; j++)
      out[off + j] = (float)((x[off + j] - mean) * inv * w[j] + b[j]);
  }
}
/* layerNorm backward: packages/autograd/src/ops.ts:523-569.  dw/db accumulate in Float32Array
 * (each += rounds to f32), dx per row. */
void orc_layernorm_bwd(const float *x, const float *w, const float *g, double eps,
                       int64_t n, int64_t dim, float *dx, float *dw, float *db) {
  memset(dw, 0, sizeof(float) * (size_t)dim);
  memset(db, 0, sizeof(float) * (size_t)dim);
  for (int64_t i = 0; i < n; i++) {
    int64_t off = i * dim;
    double mu = 0;
    for (int64_t j = 0; j < dim; j++) mu += x[off + j];
    mu /= (double)dim;
    double var = 0;
    for (int64_t j = 0; j < dim; j++) { double d = x[off + j] - mu; var += d * d; }
    var /= (double)dim;
    double inv = 1 / sqrt(var + eps);
    for (int64_t j = 0; j < dim; j++) {
      double xhat = (x[off + j] - mu) * inv;
      dw[j] = (float)((double)dw[j] + g[off + j] * xhat);
      db[j] = (float)((double)db[j] + (double)g[off + j]);
    }
    double sum1 = 0, sum2 = 0;
    for (int64_t j = 0; j < dim; j++) {
      double dy = (double)g[off + j] * (double)w[j];
      sum1 += dy;
      sum2 += dy * (x[off + j] - mu) * inv;
    }
    for (int64_t j = 0; j < dim; j++) {
      double xhat = (x[off + j] - mu) * inv;
      double dy = (double)g[off + j] * (double)w[j];
      dx[off + j] = (float)(inv * (dy - (sum1 + xhat * sum2) / (double)dim));
    }
  }
}

/* softmax over `ax`: cpu_ref.ts:437-491.  exp is STORED to the f32 output before the divide,
 * so the numerator is the f32-rounded exp while sumExp is the f64 sum of unrounded exps. */
void orc_softmax(const float *a, const int64_t *shape, int nd, int ax, float *out) {
  int64_t strides[ORC_MAX_DIMS];
  shape_strides(shape, nd, strides);
  int64_t dim = shape[ax], axs = strides[ax];
  int64_t outer = 1;                          /* the other dimensions' product (cpu_ref.ts:272-280): an empty reduced axis gives */
  for (int d = 0; d < nd; d++)                /* one zero per output (mean: 0 / 0), and no division by its length here        */
    if (d != ax) outer *= shape[d];
  for (int64_t o = 0; o < outer; o++) {
    int64_t rem = o, base = 0;
    for (int d = nd - 1; d >= 0; d--) {
      if (d == ax) continue;
      int64_t c = rem % shape[d];
      rem = (rem - c) / shape[d];
      base += c * strides[d];
    }
    double max = -INFINITY;
    for (int64_t j = 0; j < dim; j++) { double v = a[base + j * axs]; if (v > max) max = v; }
    double sum = 0;
    for (int64_t j = 0; j < dim; j++) {
      double e = exp(a[base + j * axs] - max);
      out[base + j * axs] = (float)e;
      sum += e;
    }
    for (int64_t j = 0; j < dim; j++)
      out[base + j * axs] = (float)((double)out[base + j * axs] / sum);
  }
}
/* logSoftmax: cpu_ref.ts:493-541 */
void orc_log_softmax(const float *a, const int64_t *shape, int nd, int ax, float *out) {
  int64_t strides[ORC_MAX_DIMS];
  shape_strides(shape, nd, strides);
  int64_t dim = shape[ax], axs = strides[ax];
  int64_t outer = 1;                          /* the other dimensions' product (cpu_ref.ts:272-280): an empty reduced axis gives */
  for (int d = 0; d < nd; d++)                /* one zero per output (mean: 0 / 0), and no division by its length here        */
    if (d != ax) outer *= shape[d];
  for (int64_t o = 0; o < outer; o++) {
    int64_t rem = o, base = 0;
    for (int d = nd - 1; d >= 0; d--) {
      if (d == ax) continue;
      int64_t c = rem % shape[d];
      rem = (rem - c) / shape[d];
      base += c * strides[d];
    }
    double max = -INFINITY;
    for (int64_t j = 0; j < dim; j++) { double v = a[base + j * axs]; if (v > max) max = v; }
    double sum = 0;
    for (int64_t j = 0; j < dim; j++) sum += exp(a[base + j * axs] - max);
    double lse = max + log(sum);
    for (int64_t j = 0; j < dim; j++) out[base + j * axs] = (float)(a[base + j * axs] - lse);
  }
}
/* crossEntropy: cpu_ref.ts:543-563 -- logSoftmax materialised in f32, then -mean of picks.
 * `scratch` is an [N,C] f32 buffer for the log-probabilities. */
float orc_cross_entropy(const float *logits, const int32_t *targets, int64_t N, int64_t C,
                        float *scratch) {
  int64_t shape[2] = {N, C};
  orc_log_softmax(logits, shape, 2, 1, scratch);
  double loss = 0;
  for (int64_t i = 0; i < N; i++) loss -= scratch[i * C + targets[i]];
  loss /= (double)N;
  return (float)loss;
}
/* crossEntropy backward, CPU fallback: packages/autograd/src/ops.ts:713-727:
 * probs = softmax (f32), diff = probs - onehot (f32), result = diff * (gScalar/N) (f32). */
void orc_cross_entropy_bwd(const float *logits, const int32_t *targets, double g_scalar,
                           int64_t N, int64_t C, float *out) {
  int64_t shape[2] = {N, C};
  orc_softmax(logits, shape, 2, 1, out);
  double s = g_scalar / (double)N;
  for (int64_t i = 0; i < N; i++)
    for (int64_t c = 0; c < C; c++) {
      float diff = (float)((double)out[i * C + c] - (c == targets[i] ? 1.0 : 0.0));
      out[i * C + c] = (float)((double)diff * s);
    }
}

/* transpose(dim0, dim1): cpu_ref.ts:578-607 */
void orc_transpose(const float *a, const int64_t *shape, int nd, int d0, int d1, float *out) {
  int64_t ns[ORC_MAX_DIMS], dst[ORC_MAX_DIMS], coords[ORC_MAX_DIMS];
  for (int i = 0; i < nd; i++) ns[i] = shape[i];
  ns[d0] = shape[d1]; ns[d1] = shape[d0];
  shape_strides(ns, nd, dst);
  int64_t total = shape_size(shape, nd);
  for (int64_t i = 0; i < total; i++) {
    int64_t rem = i;
    for (int d = nd - 1; d >= 0; d--) { coords[d] = rem % shape[d]; rem = (rem - coords[d]) / shape[d]; }
    int64_t t = coords[d0]; coords[d0] = coords[d1]; coords[d1] = t;
    int64_t di = 0;
    for (int d = 0; d < nd; d++) di += coords[d] * dst[d];
    out[di] = a[i];
  }
}
/* slice: cpu_ref.ts:609-634 */
void orc_slice(const float *a, const int64_t *shape, int nd, const int64_t *starts,
               const int64_t *ends, float *out) {
  int64_t os[ORC_MAX_DIMS], ss[ORC_MAX_DIMS];
  for (int d = 0; d < nd; d++) os[d] = ends[d] - starts[d];
  shape_strides(shape, nd, ss);
  int64_t n = shape_size(os, nd);
  for (int64_t i = 0; i < n; i++) {
    int64_t rem = i, src = 0;
    for (int d = nd - 1; d >= 0; d--) {
      int64_t c = rem % os[d];
      rem = (rem - c) / os[d];
      src += (c + starts[d]) * ss[d];
    }
    out[i] = a[src];
  }
}
/* scatterSlice: cpu_ref.ts:636-652 (zero-filled output of origShape) */
void orc_scatter_slice(const float *g, const int64_t *gshape, const int64_t *orig, int nd,
                       const int64_t *starts, float *out) {
  int64_t os[ORC_MAX_DIMS];
  shape_strides(orig, nd, os);
  memset(out, 0, sizeof(float) * (size_t)shape_size(orig, nd));
  int64_t n = shape_size(gshape, nd);
  for (int64_t i = 0; i < n; i++) {
    int64_t rem = i, dst = 0;
    for (int d = nd - 1; d >= 0; d--) {
      int64_t c = rem % gshape[d];
      rem = (rem - c) / gshape[d];
      dst += (c + starts[d]) * os[d];
    }
    out[dst] = g[i];
  }
}

/* argmax along `ax` (first index wins; strict > from -Infinity; NaN never selected):
 * cpu_ref.ts:698-756.  ax < 0: global argmax over n = shape_size. */
void orc_argmax(const float *a, const int64_t *shape, int nd, int ax, int32_t *out) {
  if (ax < 0) {
    int64_t n = shape_size(shape, nd), mi = 0;
    double mv = -INFINITY;
    for (int64_t i = 0; i < n; i++) if ((double)a[i] > mv) { mv = a[i]; mi = i; }
    out[0] = (int32_t)mi;
    return;
  }
  int64_t strides[ORC_MAX_DIMS];
  shape_strides(shape, nd, strides);
  int64_t dim = shape[ax], axs = strides[ax];
  int64_t outer = 1;                          /* the other dimensions' product (cpu_ref.ts:272-280): an empty reduced axis gives */
  for (int d = 0; d < nd; d++)                /* one zero per output (mean: 0 / 0), and no division by its length here        */
    if (d != ax) outer *= shape[d];
  for (int64_t o = 0; o < outer; o++) {
    int64_t rem = o, base = 0;
    for (int d = nd - 1; d >= 0; d--) {
      if (d == ax) continue;
      int64_t c = rem % shape[d];
      rem = (rem - c) / shape[d];
      base += c * strides[d];
    }
    double mv = -INFINITY; int64_t mi = 0;
    for (int64_t j = 0; j < dim; j++) { double v = a[base + j * axs]; if (v > mv) { mv = v; mi = j; } }
    out[o] = (int32_t)mi;
  }
}

/* causalMask: cpu_ref.ts:880-889 (0 on/below the diagonal, -Infinity above) */
void orc_causal_mask(int64_t size, float *out) {
  for (int64_t i = 0; i < size; i++)
    for (int64_t j = 0; j < size; j++) out[i * size + j] = j > i ? -INFINITY : 0.0f;
}
/* maskedFill: cpu_ref.ts:891-911 (mask != 0 -> value; mask tiled by i % maskSize) */
void orc_masked_fill(const float *a, int64_t n, const float *mask, int64_t mask_n, double value,
                     float *out) {
  for (int64_t i = 0; i < n; i++) out[i] = (mask[i % mask_n] != 0) ? (float)value : a[i];
}

/* gelu backward, CPU fallback: packages/autograd/src/ops.ts:405-417.  The derivative is stored
 * as an f32 array first, then multiplied by g through backend.mul (second f32 rounding).
 * fused != 0 restates the matmulTransposedGelu closure (ops.ts:449-463) that multiplies in f64
 * and rounds once. */
void orc_gelu_bwd(const float *x, const float *g, float *out, int64_t n, int fused) {
  const double S = sqrt(2.0 / M_PI);
  for (int64_t i = 0; i < n; i++) {
    double xv = x[i];
    double inner = S * (xv + 0.044715 * xv * xv * xv);
    double t = tanh(inner);
    double sech2 = 1 - t * t;
    double dInner = S * (1 + 3 * 0.044715 * xv * xv);
    double d = 0.5 * (1 + t) + 0.5 * xv * sech2 * dInner;
    if (fused) out[i] = (float)((double)g[i] * d);
    else { float df = (float)d; out[i] = (float)((double)g[i] * (double)df); }
  }
}
/* relu backward: ops.ts:284-289; silu backward: ops.ts:346-356; clamp backward: ops.ts:299-305 */
void orc_relu_bwd(const float *x, const float *g, float *out, int64_t n) {
  for (int64_t i = 0; i < n; i++) out[i] = (float)((double)g[i] * (x[i] > 0 ? 1.0 : 0.0));
}
void orc_silu_bwd(const float *x, const float *g, float *out, int64_t n) {
  for (int64_t i = 0; i < n; i++) {
    double xv = x[i], sig = 1 / (1 + exp(-xv));
    out[i] = (float)((double)g[i] * (sig * (1 + xv * (1 - sig))));
  }
}
void orc_clamp_bwd(const float *x, const float *g, float *out, int64_t n, double lo, double hi) {
  for (int64_t i = 0; i < n; i++) out[i] = ((double)x[i] > lo && (double)x[i] < hi) ? g[i] : 0.0f;
}

/* Sum of squares of one tensor in f64: packages/train/src/trainer.ts:488-496 */
double orc_sum_sq(const float *a, int64_t n) {
  double s = 0;
  for (int64_t i = 0; i < n; i++) { double v = a[i]; s += v * v; }
  return s;
}
/* checkFinite contract (packages/core/src/interfaces.ts:146; semantics fixed by
 * packages/tests/src/gpu-perf.test.ts:106-149): 0.0 if all finite else 1.0 */
float orc_check_finite(const float *a, int64_t n) {
  for (int64_t i = 0; i < n; i++) if (!isfinite(a[i])) return 1.0f;
  return 0.0f;
}

/* AdamW, one tensor: packages/train/src/optimizers.ts:76-92 (CPU loop of stepParamEntries).
 * p, m, v are Float32Array (each store rounds); scalars are f64. */
void orc_adamw(float *p, const float *grad, float *m, float *v, int64_t n, double lr,
               double beta1, double beta2, double eps, double wd, double bc1, double bc2,
               double grad_scale) {
  for (int64_t j = 0; j < n; j++) {
    double g = (double)grad[j] * grad_scale;
    if (wd > 0) p[j] = (float)((double)p[j] - lr * wd * (double)p[j]);
    m[j] = (float)(beta1 * (double)m[j] + (1 - beta1) * g);
    v[j] = (float)(beta2 * (double)v[j] + (1 - beta2) * g * g);
    double mHat = (double)m[j] / bc1;
    double vHat = (double)v[j] / bc2;
    p[j] = (float)((double)p[j] - lr * mHat / (sqrt(vHat) + eps));
  }
}

/* DropoutRng.nextMask: packages/autograd/src/ops.ts:41-51,74-81.  The first line of hash() is
 * evaluated in f64 and only then truncated with |0 (ToInt32 = modulo 2^32 of the EXACT f64
 * value, which has already lost low bits once the sum exceeds 2^53). */
static int32_t js_to_int32(double d) {
  if (!isfinite(d)) return 0;
  double t = trunc(d);
  double m = fmod(t, 4294967296.0);
  if (m < 0) m += 4294967296.0;
  return (int32_t)(uint32_t)m;
}
static uint32_t js_imul(uint32_t a, uint32_t b) { return a * b; }
/* mask[i - lo] for element indices lo <= i < hi */
void orc_dropout_mask(int32_t seed, int32_t counter, double p, float *mask, int64_t lo, int64_t hi) {
  double scale = 1 / (1 - p);
  mask -= lo;
  for (int64_t i = lo; i < hi; i++) {
    double sum = (double)seed + (double)counter * 2654435761.0 + (double)i * 2246822519.0;
    uint32_t h = (uint32_t)js_to_int32(sum);
    h = js_imul(h ^ (h >> 16), 0x85ebca6bu);
    h = js_imul(h ^ (h >> 13), 0xc2b2ae35u);
    h = h ^ (h >> 16);
    double x = (double)h / 4294967296.0;
    mask[i] = x > p ? (float)scale : 0.0f;
  }
}
