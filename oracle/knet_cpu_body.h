/*
 * TEST INFRASTRUCTURE -- typed body of the CPU oracle (see knet_cpu.c for the
 * contract).  Included twice: once with T=float/S=32/W=double and once with
 * T=double/S=64/W=long double.  W is the wide accumulator used where the
 * reference sums many terms (Julia's Base.sum association order cannot be
 * reproduced bit-for-bit, so the oracle returns the correctly rounded sum and
 * the parity tests allow 1e-5 relative).
 *
 * Every function restates a formula of the reference's CPU Array path; the
 * citation after each name is the file:line in the reference it follows.
 * All arithmetic is done in T with one rounding per operation (this file is
 * compiled with -ffp-contract=off) in the operation order the Julia source has.
 */

#define CAT_(a, b) a##_##b
#define CAT(a, b) CAT_(a, b)
#define F(name) CAT(name, S)

/* ---- forward activations: src/ops20/activation.jl:12,26,39,55 ------------ */

/* relu(x) = max(x,T(0))  -- src/ops20/activation.jl:26.  Julia's max returns
 * NaN for a NaN operand and +0 for max(-0,+0). */
static inline T F(s_relu)(T x) { return (x != x) ? x : (x > 0 ? x : (T)0); }
/* elu(x) = x>=0 ? x : exp(x)-1  -- src/ops20/activation.jl:12 */
static inline T F(s_elu)(T x) { return x >= 0 ? x : EXP(x) - (T)1; }
/* selu(x) = x>=0 ? T(l)*x : T(la)*(exp(x)-1)  -- src/ops20/activation.jl:39,43-45 */
static inline T F(s_selu)(T x) {
  return x >= 0 ? (T)KO_LAMBDA01 * x : (T)KO_LAMBDAALPHA01 * (EXP(x) - (T)1);
}
/* sigm(x) = x>=0 ? 1/(1+exp(-x)) : (z=exp(x); z/(1+z))  -- src/ops20/activation.jl:55 */
static inline T F(s_sigm)(T x) {
  if (x >= 0) return (T)1 / ((T)1 + EXP(-x));
  T z = EXP(x);
  return z / ((T)1 + z);
}
static inline T F(s_tanh)(T x) { return TANH(x); }

/* ---- two-input gradients (dy,y)->dx -------------------------------------- */
/* reluback(dy,y) = y>0 ? dy : 0  -- src/ops20/activation.jl:27 */
static inline T F(s_reluback)(T dy, T y) { return y > 0 ? dy : (T)0; }
/* sigmback(dy,y) = dy*y*(1-y), evaluated (dy*y)*(1-y)  -- src/ops20/activation.jl:56 */
static inline T F(s_sigmback)(T dy, T y) { T a = dy * y; T b = (T)1 - y; return a * b; }
/* tanhback(dy,y) = dy*(1-y*y)  -- src/ops20_gpu/activation.jl:11 */
static inline T F(s_tanhback)(T dy, T y) { T a = y * y; T b = (T)1 - a; return dy * b; }
/* eluback(dy,y) = y>=0 ? dy : dy*(1+y)  -- src/ops20/activation.jl:13 */
static inline T F(s_eluback)(T dy, T y) { if (y >= 0) return dy; T b = (T)1 + y; return dy * b; }
/* seluback(dy,y) = y>=0 ? dy*T(l) : dy*(y+T(la))  -- src/ops20/activation.jl:40 */
static inline T F(s_seluback)(T dy, T y) {
  if (y >= 0) return dy * (T)KO_LAMBDA01;
  T b = y + (T)KO_LAMBDAALPHA01;
  return dy * b;
}

/* ---- ops21 forwards and three-input gradients (x,y,dy)->dx --------------- */
/* gelu(x) = x*(1+erf(x/T(sqrt(2))))/2  -- src/ops21/activation.jl:37 */
static inline T F(s_gelu)(T x) { T a = x / (T)KO_SQRT2; T b = (T)1 + ERF(a); T c = x * b; return c / (T)2; }
/* geluback = dy*((1+erf(x/T(sqrt2)))/2 + x*exp(-x^2/2)/T(sqrt(2pi)))  -- src/ops21/activation.jl:38 */
static inline T F(s_geluback)(T x, T y, T dy) {
  (void)y;
  T a = x / (T)KO_SQRT2; T b = ((T)1 + ERF(a)) / (T)2;
  T x2 = x * x; T e = EXP(-x2 / (T)2); T c = (x * e) / (T)KO_SQRT2PI;
  T d = b + c;
  return dy * d;
}
/* hardsigmoid(x) = x<=-3 ? 0 : x>=3 ? 1 : (x+3)/6  -- src/ops21/activation.jl:61 */
static inline T F(s_hardsigmoid)(T x) { return x <= (T)-3 ? (T)0 : x >= (T)3 ? (T)1 : (x + (T)3) / (T)6; }
/* hardsigmoidback = dy*(x<=-3 ? 0 : x>=3 ? 0 : T(1/6))  -- src/ops21/activation.jl:62 */
static inline T F(s_hardsigmoidback)(T x, T y, T dy) {
  (void)y;
  T g = x <= (T)-3 ? (T)0 : x >= (T)3 ? (T)0 : (T)(1.0 / 6.0);
  return dy * g;
}
/* hardswish(x) = x<=-3 ? 0 : x>=3 ? x : x*(x+3)/6  -- src/ops21/activation.jl:81 */
static inline T F(s_hardswish)(T x) {
  if (x <= (T)-3) return (T)0;
  if (x >= (T)3) return x;
  T a = x + (T)3; T b = x * a; return b / (T)6;
}
/* hardswishback = dy*(x<=-3 ? 0 : x>=3 ? 1 : (2x+3)/6)  -- src/ops21/activation.jl:82 */
static inline T F(s_hardswishback)(T x, T y, T dy) {
  (void)y;
  T g;
  if (x <= (T)-3) g = (T)0; else if (x >= (T)3) g = (T)1;
  else { T a = (T)2 * x; T b = a + (T)3; g = b / (T)6; }
  return dy * g;
}
/* swish(x) = x*sigm(x)  -- src/ops21/activation.jl:170 */
static inline T F(s_swish)(T x) { return x * F(s_sigm)(x); }
/* swishback -- src/ops21/activation.jl:171 */
static inline T F(s_swishback)(T x, T y, T dy) {
  (void)y;
  T g;
  if (x >= 0) { T z = EXP(-x); T zx = z * x; T num = (zx + z) + (T)1; T d = z + (T)1; g = num / (d * d); }
  else { T z = EXP(x); T s = (x + z) + (T)1; T num = z * s; T d = z + (T)1; g = num / (d * d); }
  return dy * g;
}
/* ops21 eluback/seluback/sigmback/tanh_back(x,y,dy): same formulas as the two-input
 * forms with x unused -- src/ops21/activation.jl:17,130,152,187 */
static inline T F(s_eluback3)(T x, T y, T dy) { (void)x; return F(s_eluback)(dy, y); }
static inline T F(s_seluback3)(T x, T y, T dy) { (void)x; return F(s_seluback)(dy, y); }
static inline T F(s_sigmback3)(T x, T y, T dy) { (void)x; return F(s_sigmback)(dy, y); }
/* tanh_back = dy*(1-abs2(y))  -- src/ops21/activation.jl:187 */
static inline T F(s_tanh_back3)(T x, T y, T dy) { (void)x; return F(s_tanhback)(dy, y); }

/* relu(x;max_value,negative_slope,threshold)  -- src/ops21/activation.jl:101-106 */
static inline T F(s_relu_kw)(T x, T maxv, T slope, T thr) {
  if (x >= maxv) return maxv;
  if (x >= thr) return x;
  if (slope == 0) return (T)0;
  T a = x - thr;
  return slope * a;
}
/* reluback(x,y,dy;...) = dy*(x>=max ? 0 : x>=thr ? 1 : slope)  -- src/ops21/activation.jl:108-112 */
static inline T F(s_reluback_kw)(T x, T dy, T maxv, T slope, T thr) {
  T g = x >= maxv ? (T)0 : x >= thr ? (T)1 : slope;
  return dy * g;
}

#define KO_UNARY(name) \
  void F(ko_##name)(long n, const T *x, T *y) { for (long i = 0; i < n; i++) y[i] = F(s_##name)(x[i]); }
KO_UNARY(relu) KO_UNARY(elu) KO_UNARY(selu) KO_UNARY(sigm) KO_UNARY(tanh)
KO_UNARY(gelu) KO_UNARY(hardsigmoid) KO_UNARY(hardswish) KO_UNARY(swish)
#undef KO_UNARY

#define KO_BACK11(name) \
  void F(ko_##name)(long n, const T *dy, const T *y, T *dx) { for (long i = 0; i < n; i++) dx[i] = F(s_##name)(dy[i], y[i]); }
KO_BACK11(reluback) KO_BACK11(sigmback) KO_BACK11(tanhback) KO_BACK11(eluback) KO_BACK11(seluback)
#undef KO_BACK11

#define KO_BACK111(name, fn) \
  void F(ko_##name)(long n, const T *x, const T *y, const T *dy, T *dx) { for (long i = 0; i < n; i++) dx[i] = F(fn)(x[i], y[i], dy[i]); }
KO_BACK111(eluback_111, s_eluback3) KO_BACK111(seluback_111, s_seluback3) KO_BACK111(sigmback_111, s_sigmback3)
KO_BACK111(tanh_back_111, s_tanh_back3) KO_BACK111(geluback_111, s_geluback)
KO_BACK111(hardsigmoidback_111, s_hardsigmoidback) KO_BACK111(hardswishback_111, s_hardswishback)
KO_BACK111(swishback_111, s_swishback)
#undef KO_BACK111

void F(ko_relu_1)(long n, T maxv, T slope, T thr, const T *x, T *y) {
  for (long i = 0; i < n; i++) y[i] = F(s_relu_kw)(x[i], maxv, slope, thr);
}
void F(ko_reluback_1)(long n, T maxv, T slope, T thr, const T *x, const T *y, const T *dy, T *dx) {
  (void)y;
  for (long i = 0; i < n; i++) dx[i] = F(s_reluback_kw)(x[i], dy[i], maxv, slope, thr);
}

/* ---- reductions ----------------------------------------------------------
 * Reduce a column-major array x of shape dims[0..nd) over the dimensions whose
 * mask[k] != 0; y has the same shape with the reduced dims set to 1
 * (src/knetarrays/reduction.jl:35-73 keeps singleton dims).  op codes follow
 * the order of reduction_ops in src/libknet8/ops.jl:144-156.  sum-like ops
 * accumulate in W and round once; max/min-like ops are exact in T. */
void F(ko_reduce)(int op, int nd, const long *dims, const int *mask, const T *x, T *y) {
  long nx = 1, ny = 1;
  long ystr[16], xdim[16];
  for (int k = 0; k < nd; k++) { xdim[k] = dims[k]; nx *= dims[k]; }
  for (int k = 0; k < nd; k++) { ystr[k] = mask[k] ? 0 : ny; if (!mask[k]) ny *= dims[k]; }
  if (ny == 0 || nd > 16) return;
  W *acc = (W *)malloc(sizeof(W) * (size_t)ny);
  W init = 0;
  switch (op) {
    case 1: init = 1; break;                       /* prod */
    case 2: init = (W)-INFINITY; break;            /* maximum */
    case 3: case 7: init = (W)INFINITY; break;     /* minimum, minabs */
    default: init = 0;                             /* sum,sumabs,sumabs2,maxabs,countnz */
  }
  for (long j = 0; j < ny; j++) acc[j] = init;
  long idx[16] = {0};
  long yi = 0;
  for (long i = 0; i < nx; i++) {
    W xi = (W)x[i], ai = acc[yi];
    switch (op) {
      case 0: ai = ai + xi; break;
      case 1: ai = ai * xi; break;
      case 2: ai = (ai > xi ? ai : xi); break;
      case 3: ai = (ai < xi ? ai : xi); break;
      case 4: xi = (xi < 0 ? -xi : xi); ai = ai + xi; break;
      case 5: xi = xi * xi; ai = ai + xi; break;
      case 6: xi = (xi < 0 ? -xi : xi); ai = (ai > xi ? ai : xi); break;
      case 7: xi = (xi < 0 ? -xi : xi); ai = (ai < xi ? ai : xi); break;
      case 8: ai = ai + (xi != 0 ? 1 : 0); break;
    }
    acc[yi] = ai;
    /* advance the column-major odometer */
    for (int k = 0; k < nd; k++) {
      idx[k]++; yi += ystr[k];
      if (idx[k] < xdim[k]) break;
      yi -= ystr[k] * xdim[k]; idx[k] = 0;
    }
  }
  for (long j = 0; j < ny; j++) y[j] = (T)acc[j];
  free(acc);
}

/* The `_21` contract stated directly: x[i] goes into y[(i/sy)%ny] (src/libknet8/cuda21.jl:23), walked in memory
 * order with a wide accumulator per output.  Same result as ko_reduce on the (sy,ny,nx/(sy*ny)) view with dims 1
 * and 3 reduced; kept separate because it is the form the C ABI takes and the loop the CPU baseline times. */
void F(ko_sum_21)(long nx, const T *x, long sy, long ny, T *y) {
  W *acc = (W *)calloc((size_t)(ny > 0 ? ny : 1), sizeof(W));
  const long slab = sy * ny;
  for (long o = 0; o + slab <= nx; o += slab)
    for (long j = 0; j < ny; j++) {
      const T *run = x + o + j * sy;
      W a = acc[j];
      for (long s = 0; s < sy; s++) a += (W)run[s];
      acc[j] = a;
    }
  for (long j = 0; j < ny; j++) y[j] = (T)acc[j];
  free(acc);
}

/* ---- softmax family over the middle axis of an (inner, d, outer) view ------
 * dims=1 of an (m,n) matrix is inner=1,d=m,outer=n; dims=2 is inner=m,d=n,outer=1.
 * _logsoftmax: x = x .- maximum(x); x .- log.(sum(exp.(x)))  -- src/ops20/softmax.jl:42-47 */
void F(ko_logsoftmax)(long inner, long d, long outer, const T *x, T *y) {
  for (long o = 0; o < outer; o++) for (long a = 0; a < inner; a++) {
    const T *xp = x + o * d * inner + a; T *yp = y + o * d * inner + a;
    T mx = (T)-INFINITY;
    for (long k = 0; k < d; k++) { T v = xp[k * inner]; if (v > mx || v != v) mx = v; }
    W s = 0;
    for (long k = 0; k < d; k++) { T c = xp[k * inner] - mx; s += (W)EXP(c); }
    T ls = LOG((T)s);
    for (long k = 0; k < d; k++) { T c = xp[k * inner] - mx; yp[k * inner] = c - ls; }
  }
}
/* ∇logsoftmax: dx = dy - exp.(y).*sum(dy;dims)  -- src/ops20/softmax.jl:49-51 */
void F(ko_logsoftmaxback)(long inner, long d, long outer, const T *y, const T *dy, T *dx) {
  for (long o = 0; o < outer; o++) for (long a = 0; a < inner; a++) {
    long base = o * d * inner + a;
    W s = 0;
    for (long k = 0; k < d; k++) s += (W)dy[base + k * inner];
    T st = (T)s;
    for (long k = 0; k < d; k++) { T e = EXP(y[base + k * inner]); T p = e * st; dx[base + k * inner] = dy[base + k * inner] - p; }
  }
}
/* _softmax: x = exp.(x .- maximum(x)); x ./ sum(x)  -- src/ops20/softmax.jl:53-59 */
void F(ko_softmax)(long inner, long d, long outer, const T *x, T *y) {
  for (long o = 0; o < outer; o++) for (long a = 0; a < inner; a++) {
    long base = o * d * inner + a;
    T mx = (T)-INFINITY;
    for (long k = 0; k < d; k++) { T v = x[base + k * inner]; if (v > mx || v != v) mx = v; }
    W s = 0;
    for (long k = 0; k < d; k++) { T c = x[base + k * inner] - mx; s += (W)EXP(c); }
    T st = (T)s;
    for (long k = 0; k < d; k++) { T c = x[base + k * inner] - mx; y[base + k * inner] = EXP(c) / st; }
  }
}
/* ∇softmax: dx = y.*dy .- y.*sum(y.*dy;dims)  -- src/ops20/softmax.jl:61-63 */
void F(ko_softmaxback)(long inner, long d, long outer, const T *y, const T *dy, T *dx) {
  for (long o = 0; o < outer; o++) for (long a = 0; a < inner; a++) {
    long base = o * d * inner + a;
    W s = 0;
    for (long k = 0; k < d; k++) { T p = y[base + k * inner] * dy[base + k * inner]; s += (W)p; }
    T st = (T)s;
    for (long k = 0; k < d; k++) {
      T yy = y[base + k * inner]; T p = yy * dy[base + k * inner]; T q = yy * st;
      dx[base + k * inner] = p - q;
    }
  }
}
/* _logsumexp: xmax + log.(sum(exp.(x .- xmax)))  -- src/ops20/softmax.jl:65-70; y has d collapsed to 1 */
void F(ko_logsumexp)(long inner, long d, long outer, const T *x, T *y) {
  for (long o = 0; o < outer; o++) for (long a = 0; a < inner; a++) {
    long base = o * d * inner + a;
    T mx = (T)-INFINITY;
    for (long k = 0; k < d; k++) { T v = x[base + k * inner]; if (v > mx || v != v) mx = v; }
    W s = 0;
    for (long k = 0; k < d; k++) { T c = x[base + k * inner] - mx; s += (W)EXP(c); }
    y[o * inner + a] = mx + LOG((T)s);
  }
}
/* ∇logsumexp: dy .* exp.(x .- y)  -- src/ops20/softmax.jl:72-74 */
void F(ko_logsumexpback)(long inner, long d, long outer, const T *x, const T *y, const T *dy, T *dx) {
  for (long o = 0; o < outer; o++) for (long a = 0; a < inner; a++) {
    long base = o * d * inner + a; T yy = y[o * inner + a], g = dy[o * inner + a];
    for (long k = 0; k < d; k++) { T c = x[base + k * inner] - yy; dx[base + k * inner] = g * EXP(c); }
  }
}

/* ---- gather / scatter-add on 1-based linear indices ------------------------
 * getents: y[i] = x[ents[i]-1]  -- src/libknet8/cuda1.jl:342-348
 * addents: x[ents[i]-1] += y[i] -- src/libknet8/cuda1.jl:356-362 */
void F(ko_getents)(long n, const int *ents, const T *x, T *y) { for (long i = 0; i < n; i++) y[i] = x[ents[i] - 1]; }
void F(ko_addents)(long n, const int *ents, T *x, const T *y) { for (long i = 0; i < n; i++) x[ents[i] - 1] += y[i]; }

/* nll(scores,labels;dims,average=true) = -sum(lp)/length(lp), lp = logsoftmax(scores)[indices]
 * -- src/ops20/loss.jl:37-41.  scores is (y1,y2) column-major; returns the loss and stores
 * the number of counted instances. */
T F(ko_nll)(long y1, long y2, const T *scores, const int *labels, int dims, long *count) {
  long ninst = dims == 1 ? y2 : y1;
  long *ind = (long *)malloc(sizeof(long) * (size_t)(ninst > 0 ? ninst : 1));
  long c = ko_findindices(y1, y2, labels, ninst, dims, ind);
  T *lp = (T *)malloc(sizeof(T) * (size_t)(y1 * y2 > 0 ? y1 * y2 : 1));
  if (dims == 1) F(ko_logsoftmax)(1, y1, y2, scores, lp); else F(ko_logsoftmax)(y1, y2, 1, scores, lp);
  W s = 0;
  for (long j = 0; j < c; j++) s += (W)lp[ind[j] - 1];
  T total = (T)s;
  free(lp); free(ind);
  if (count) *count = c;
  return -total / (T)c;
}
/* gradient of nll wrt scores: AutoGrad chain of src/ops20/loss.jl:38-40 --
 * d(-sum(lp)/c)/dlp = -1/c at the gathered indices (ungetindex scatter-add into zeros,
 * src/autograd_gpu/getindex.jl:5-13), then ∇logsoftmax (src/ops20/softmax.jl:49-51). */
void F(ko_nll_back)(long y1, long y2, const T *scores, const int *labels, int dims, T *dx) {
  long ninst = dims == 1 ? y2 : y1, n = y1 * y2;
  long *ind = (long *)malloc(sizeof(long) * (size_t)(ninst > 0 ? ninst : 1));
  long c = ko_findindices(y1, y2, labels, ninst, dims, ind);
  T *lp = (T *)malloc(sizeof(T) * (size_t)(n > 0 ? n : 1));
  T *dlp = (T *)calloc((size_t)(n > 0 ? n : 1), sizeof(T));
  if (dims == 1) F(ko_logsoftmax)(1, y1, y2, scores, lp); else F(ko_logsoftmax)(y1, y2, 1, scores, lp);
  T g = -((T)1 / (T)c);
  for (long j = 0; j < c; j++) dlp[ind[j] - 1] += g;
  if (dims == 1) F(ko_logsoftmaxback)(1, y1, y2, lp, dlp, dx); else F(ko_logsoftmaxback)(y1, y2, 1, lp, dlp, dx);
  free(lp); free(dlp); free(ind);
}

/* ---- dropout ---------------------------------------------------------------
 * dropout!(p,x,y): y holds U[0,1) on entry; y = y>p ? x/q : 0, q=1-p  -- src/ops20/dropout.jl:45-58
 * dropback!(p,x,y,dy,dx): dx = y==0 ? 0 : dy/q                         -- src/ops20/dropout.jl:60-71 */
void F(ko_dropout)(long n, T p, const T *x, T *y) {
  T q = (T)1 - p;
  for (long i = 0; i < n; i++) y[i] = (y[i] > p) ? x[i] / q : (T)0;
}
void F(ko_dropback)(long n, T p, const T *x, const T *y, const T *dy, T *dx) {
  (void)x;
  T q = (T)1 - p;
  for (long i = 0; i < n; i++) dx[i] = (y[i] == 0) ? (T)0 : dy[i] / q;
}

/* ---- small helpers used by the MLP restatement ------------------------------
 * z = x .+ b with b a vector along one dim: b[(i/sb)%nb]  -- src/libknet8/cuda12.jl:18-27 */
void F(ko_add_12)(long n, const T *x, const T *b, long sb, long nb, T *z) {
  for (long i = 0; i < n; i++) z[i] = x[i] + b[(i / sb) % nb];
}
/* axpy!(a,x,y): y += a*x  -- src/knetarrays/linalg.jl:58-73 (addto!, src/autograd_gpu/addto.jl:7-10) */
void F(ko_axpy)(long n, T a, const T *x, T *y) { for (long i = 0; i < n; i++) { T p = a * x[i]; y[i] = y[i] + p; } }
/* column-major C = op(A)*op(B) with W accumulation (yardstick for the vendor GEMM) */
void F(ko_gemm)(int ta, int tb, long m, long n, long k, const T *A, long lda, const T *B, long ldb, T *C, long ldc) {
  for (long j = 0; j < n; j++) for (long i = 0; i < m; i++) {
    W s = 0;
    for (long l = 0; l < k; l++) {
      T a = ta ? A[l + i * lda] : A[i + l * lda];
      T b = tb ? B[j + l * ldb] : B[l + j * ldb];
      s += (W)a * (W)b;
    }
    C[i + j * ldc] = (T)s;
  }
}

/* bce(scores,labels): l = max.(0,s) .- y.*s .+ log.(1 .+ exp.(-abs.(s)))  -- src/ops20/loss.jl:107-111, labels already
 * converted to T (oftype(scores,labels)); per-element losses.  Its gradient wrt s (sub-gradient 0 at s == 0 for max and abs,
 * as AutoGrad's rules give): step(s) - y - sign(s)*e/(1+e), e = exp(-|s|), times the upstream scale. */
void F(ko_bce)(long n, const T *s, const T *y, T *l) {
  for (long i = 0; i < n; i++) {
    T a = s[i] > 0 ? s[i] : (T)0; T b = y[i] * s[i]; T c = a - b; T ab = s[i] < 0 ? -s[i] : s[i];
    T e = EXP(-ab); T f = (T)1 + e; l[i] = c + LOG(f);
  }
}
void F(ko_bceback)(long n, T scale, const T *s, const T *y, T *ds) {
  for (long i = 0; i < n; i++) {
    T ab = s[i] < 0 ? -s[i] : s[i]; T e = EXP(-ab); T q = e / ((T)1 + e);
    T step = s[i] > 0 ? (T)1 : (T)0; T sg = s[i] > 0 ? (T)1 : s[i] < 0 ? (T)-1 : (T)0;
    T g = (step - y[i]) - sg * q; ds[i] = scale * g;
  }
}

/* ---- optimizer updates, per element, in the order of the lmul!/axpy!/broadcast chains of
 * src/train20/update.jl:513-570 (lmul!(a,x): x = a*x; axpy!(a,x,y): y = y + a*x, product rounded first).
 * Scalars arrive already rounded to T, as the Julia code rounds them (alpha = T[alpha], T(p.eps), T(1 - beta^t)). */
void F(ko_momentum)(long n, T nlr, T gamma, const T *g, T *vel, T *w) {                       /* update.jl:517-522 */
  for (long i = 0; i < n; i++) { T v1 = gamma * vel[i]; T p = nlr * g[i]; T v2 = v1 + p; vel[i] = v2; w[i] = w[i] + v2; }
}
void F(ko_nesterov)(long n, T nlr, T gamma, T opg, const T *g, T *vel, T *w) {                /* update.jl:525-531 */
  for (long i = 0; i < n; i++) {
    T v1 = gamma * vel[i]; T m1 = (T)-1 * v1; T w1 = w[i] + m1; T p = nlr * g[i]; T v2 = v1 + p; T q = opg * v2;
    vel[i] = v2; w[i] = w1 + q;
  }
}
void F(ko_adagrad)(long n, T nlr, T eps, const T *g, T *G, T *w) {                            /* update.jl:533-538 */
  for (long i = 0; i < n; i++) { T gg = g[i] * g[i]; T G1 = G[i] + gg; T t = G1 + eps; T q = g[i] / SQRT(t); T p = nlr * q; G[i] = G1; w[i] = w[i] + p; }
}
void F(ko_rmsprop)(long n, T nlr, T rho, T omr, T eps, const T *g, T *G, T *w) {              /* update.jl:540-546 */
  for (long i = 0; i < n; i++) {
    T G1 = rho * G[i]; T gg = g[i] * g[i]; T a = omr * gg; T G2 = G1 + a; T t = G2 + eps; T q = g[i] / SQRT(t); T p = nlr * q;
    G[i] = G2; w[i] = w[i] + p;
  }
}
void F(ko_adadelta)(long n, T nlr, T rho, T omr, T eps, const T *g, T *G, T *delta, T *w) {   /* update.jl:548-557 */
  for (long i = 0; i < n; i++) {
    T G1 = rho * G[i]; T gg = g[i] * g[i]; T a = omr * gg; T G2 = G1 + a; T sd = SQRT(delta[i] + eps); T num = g[i] * sd;
    T dw = num / SQRT(G2 + eps); T d1 = rho * delta[i]; T dd = dw * dw; T b = omr * dd; T p = nlr * dw;
    G[i] = G2; delta[i] = d1 + b; w[i] = w[i] + p;
  }
}
void F(ko_adam)(long n, T nlr, T beta1, T omb1, T beta2, T omb2, T c1, T c2, T eps, const T *g, T *m, T *v, T *w) { /* update.jl:559-570 */
  for (long i = 0; i < n; i++) {
    T m1 = beta1 * m[i]; T a = omb1 * g[i]; T m2 = m1 + a; T s1 = beta2 * v[i]; T gg = g[i] * g[i]; T b = omb2 * gg; T s2 = s1 + b;
    T mc = m2 / c1; T sc = s2 / c2; T den = SQRT(sc) + eps; T q = mc / den; T p = nlr * q;
    m[i] = m2; v[i] = s2; w[i] = w[i] + p;
  }
}

#undef F
#undef CAT
#undef CAT_
