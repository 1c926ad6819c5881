/* TEST INFRASTRUCTURE — the parity checker, never the product.  See sdpa_oracle.h for scope and pinning status.
 *
 * Every arithmetic step below is done in the order and precision of the reference's fp32 CPU path; the file is
 * compiled with -ffp-contract=off so no multiply-add is fused (the reference's Release build targets baseline
 * x86-64, which has no FMA).
 */
#include "sdpa_oracle.h"

#include <float.h>
#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------------------------------------------------
 * 16-bit float conversions
 * ---------------------------------------------------------------------------------------------------------------- */

static inline uint32_t f32_bits(float x) {
  uint32_t u;
  memcpy(&u, &x, 4);
  return u;
}
static inline float bits_f32(uint32_t u) {
  float x;
  memcpy(&x, &u, 4);
  return x;
}

/* Round to nearest even on the upper 16 bits; every NaN becomes the canonical 0x7FC0
 * (reference src/Utils/BFloat16.h:72-85). */
uint16_t oracle_f32_to_bf16_bits(float x) {
  uint32_t u = f32_bits(x);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return 0x7FC0;
  uint32_t lsb = (u >> 16) & 1u;
  return (uint16_t)((u + 0x7FFFu + lsb) >> 16);
}

float oracle_bf16_bits_to_f32(uint16_t b) { return bits_f32((uint32_t)b << 16); }

/* IEEE binary16, round to nearest even, overflow to inf, gradual underflow, NaN -> 0x7E00 with the sign kept
 * (what the reference's bit-trick conversion yields, src/Utils/Half.h:226-257).  Written as explicit
 * exponent/mantissa handling rather than the reference's scaled-float trick, so agreement is a real check. */
uint16_t oracle_f32_to_f16_bits(float x) {
  uint32_t u = f32_bits(x);
  uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
  uint32_t a = u & 0x7FFFFFFFu;
  if (a > 0x7F800000u) return (uint16_t)(sign | 0x7E00u);
  if (a >= 0x47800000u) return (uint16_t)(sign | 0x7C00u); /* >= 65536: inf (65520..65536 handled by rounding) */
  int32_t e = (int32_t)(a >> 23) - 127;
  uint32_t m = a & 0x7FFFFFu;
  if (e < -25) return sign; /* below half of the smallest subnormal */
  uint32_t half;
  if (e < -14) {
    /* subnormal result: value = (1.m) * 2^e = M * 2^-24 with M = (1.m) * 2^(e+24) */
    uint32_t full = m | 0x800000u; /* 24 significant bits, binary point after bit 23 */
    int shift = -e - 1;            /* full * 2^(e+24-23) = full >> (-e-1), shift in [14, 24] */
    uint32_t q = full >> shift;
    uint32_t rem = full & ((1u << shift) - 1u);
    uint32_t halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (q & 1u))) q++;
    half = q; /* may carry into the smallest normal, which is the right encoding */
  } else {
    uint32_t q = ((uint32_t)(e + 15) << 10) | (m >> 13);
    uint32_t rem = m & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (q & 1u))) q++;
    half = q; /* mantissa carry bumps the exponent; 0x7C00 is inf */
  }
  return (uint16_t)(sign | half);
}

float oracle_f16_bits_to_f32(uint16_t b) {
  uint32_t sign = ((uint32_t)b & 0x8000u) << 16;
  uint32_t e = (b >> 10) & 0x1Fu;
  uint32_t m = b & 0x3FFu;
  if (e == 0x1F) return bits_f32(sign | 0x7F800000u | (m << 13));
  if (e == 0) {
    if (m == 0) return bits_f32(sign);
    float f = (float)m * 0x1.0p-24f; /* exact */
    return sign ? -f : f;
  }
  return bits_f32(sign | ((e + 112u) << 23) | (m << 13));
}

void oracle_round_array(const float* in, float* out_f32, uint16_t* out_bits, int64_t n, int dtype) {
  for (int64_t i = 0; i < n; i++) {
    if (dtype == ORACLE_BF16) {
      uint16_t b = oracle_f32_to_bf16_bits(in[i]);
      if (out_bits) out_bits[i] = b;
      if (out_f32) out_f32[i] = oracle_bf16_bits_to_f32(b);
    } else if (dtype == ORACLE_F16) {
      uint16_t b = oracle_f32_to_f16_bits(in[i]);
      if (out_bits) out_bits[i] = b;
      if (out_f32) out_f32[i] = oracle_f16_bits_to_f32(b);
    } else {
      if (out_f32) out_f32[i] = in[i];
    }
  }
}

void oracle_bits_to_f32_array(const uint16_t* in, float* out, int64_t n, int dtype) {
  for (int64_t i = 0; i < n; i++)
    out[i] = dtype == ORACLE_BF16 ? oracle_bf16_bits_to_f32(in[i]) : oracle_f16_bits_to_f32(in[i]);
}

/* ------------------------------------------------------------------------------------------------------------------
 * Work distribution: tasks 0..ntasks-1 pulled from an atomic counter by nthreads workers.
 * ---------------------------------------------------------------------------------------------------------------- */

typedef void (*task_fn)(void* ctx, int64_t task, void* scratch);

typedef struct {
  task_fn fn;
  void* ctx;
  int64_t ntasks;
  int64_t next;
  size_t scratch_bytes;
  int failed;
} pool_t;

static void* pool_worker(void* arg) {
  pool_t* p = (pool_t*)arg;
  void* scratch = NULL;
  if (p->scratch_bytes) {
    scratch = malloc(p->scratch_bytes);
    if (!scratch) {
      __atomic_store_n(&p->failed, 1, __ATOMIC_RELAXED);
      return NULL;
    }
  }
  for (;;) {
    int64_t t = __atomic_fetch_add(&p->next, 1, __ATOMIC_RELAXED);
    if (t >= p->ntasks) break;
    p->fn(p->ctx, t, scratch);
  }
  free(scratch);
  return NULL;
}

static int run_pool(task_fn fn, void* ctx, int64_t ntasks, size_t scratch_bytes, int nthreads) {
  pool_t p = {fn, ctx, ntasks, 0, scratch_bytes, 0};
  if (nthreads < 1) nthreads = 1;
  if ((int64_t)nthreads > ntasks) nthreads = (int)(ntasks > 0 ? ntasks : 1);
  if (nthreads == 1) {
    pool_worker(&p);
    return p.failed ? -1 : 0;
  }
  pthread_t* th = (pthread_t*)malloc(sizeof(pthread_t) * (size_t)nthreads);
  if (!th) return -1;
  int started = 0;
  for (int i = 0; i < nthreads; i++) {
    if (pthread_create(&th[i], NULL, pool_worker, &p) != 0) break;
    started++;
  }
  if (started == 0) pool_worker(&p);
  for (int i = 0; i < started; i++) pthread_join(th[i], NULL);
  free(th);
  return p.failed ? -1 : 0;
}

/* ------------------------------------------------------------------------------------------------------------------
 * PRNG: splitmix64 finaliser over a counter, Box-Muller in double.
 * ---------------------------------------------------------------------------------------------------------------- */

static inline uint64_t mix64(uint64_t z) {
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

typedef struct {
  uint64_t key;
  int64_t n;
  float mul;
  float* out;
} randn_ctx;

#define RANDN_CHUNK 65536

static void randn_task(void* vctx, int64_t task, void* scratch) {
  (void)scratch;
  randn_ctx* c = (randn_ctx*)vctx;
  int64_t lo = task * RANDN_CHUNK, hi = lo + RANDN_CHUNK;
  if (hi > c->n) hi = c->n;
  for (int64_t i = lo; i < hi; i++) {
    uint64_t a = mix64(c->key + 2ull * (uint64_t)i);
    uint64_t b = mix64(c->key + 2ull * (uint64_t)i + 1ull);
    double u1 = ((double)(a >> 11) + 1.0) * 0x1.0p-53; /* (0, 1] */
    double u2 = (double)(b >> 11) * 0x1.0p-53;         /* [0, 1) */
    double z = sqrt(-2.0 * log(u1)) * cos(6.283185307179586476925286766559 * u2);
    c->out[i] = (float)((double)c->mul * z);
  }
}

void oracle_randn(uint64_t seed, uint64_t stream, int64_t n, float mul, float* out, int nthreads) {
  randn_ctx c;
  c.key = mix64(seed ^ mix64(stream * 0xD1342543DE82EF95ull + 0x632BE59BD9B4E019ull));
  c.n = n;
  c.mul = mul;
  c.out = out;
  run_pool(randn_task, &c, (n + RANDN_CHUNK - 1) / RANDN_CHUNK, 0, nthreads);
}

/* ------------------------------------------------------------------------------------------------------------------
 * The attention path
 * ---------------------------------------------------------------------------------------------------------------- */

/* One row of softmax, in place (reference src/Operation/OpNNLayerCpu.h:27-54): running max starts at -FLT_MAX and is
 * replaced only on strict '>', e = expf(x - max), the sum is accumulated left to right in fp32, and the row is
 * multiplied by (float)(1.0 / (double)sum).  A row whose entries are all -inf therefore gives 0 * inf = NaN. */
static void softmax_row(float* x, int64_t n) {
  float mx = -FLT_MAX;
  for (int64_t j = 0; j < n; j++)
    if (x[j] > mx) mx = x[j];
  float sum = 0.f;
  for (int64_t j = 0; j < n; j++) {
    float e = expf(x[j] - mx);
    x[j] = e;
    sum += e;
  }
  float inv = (float)(1.0 / (double)sum);
  for (int64_t j = 0; j < n; j++) x[j] *= inv;
}

/* scores *= scale (reference FuncNNLayer.h:238, OpElemWiseCpu.h:154-159), then scores = scores + 1 * bias with the
 * bias the reference builds (FuncNNLayer.h:240-259): causal -> 0 / -inf by j <= i (OpTransformCpu.h:202-209);
 * Bool mask -> 0 / -inf; float mask -> 0 + 1 * mask. */
static void scale_and_bias_row(float* x, int64_t S, int64_t i, float scale, int causal, int mask_kind,
                               const void* mask) {
  for (int64_t j = 0; j < S; j++) x[j] = x[j] * scale;
  if (causal) {
    for (int64_t j = 0; j < S; j++) {
      float bias = (j <= i) ? 0.f : -INFINITY;
      x[j] = x[j] + 1.f * bias;
    }
  }
  if (mask_kind == ORACLE_MASK_BOOL) {
    const uint8_t* m = (const uint8_t*)mask + i * S;
    for (int64_t j = 0; j < S; j++) {
      float bias = m[j] ? 0.f : -INFINITY;
      x[j] = x[j] + 1.f * bias;
    }
  } else if (mask_kind == ORACLE_MASK_FLOAT) {
    const float* m = (const float*)mask + i * S;
    for (int64_t j = 0; j < S; j++) {
      float bias = 0.f + 1.f * m[j];
      x[j] = x[j] + 1.f * bias;
    }
  }
}

typedef struct {
  const float *q, *k, *v;
  float* out;
  int64_t B, Hq, Hkv, L, S, D;
  int causal;
  float scale;
  int mask_kind;
  const void* mask;
  int64_t row_block;
  /* row-subset form */
  const int64_t* rows;
  int64_t nrows;
} sdpa_ctx;

/* One (batch, head) slice.  scratch = kT [D,S] followed by scores [row_block,S].
 * gemm loops follow reference src/Operation/OpLinalgCpu.h:139-150: C zeroed, then for i, p, j: c[i,j] += a[i,p]*b[p,j]
 * (per output element: left-to-right fp32 sum over p, product rounded before the add).  K is transposed into a dense
 * [D,S] copy first, as op::transpose does (src/Operation/OpTransformCpu.h:54-87). */
static void slice_task(void* vctx, int64_t task, void* scratch) {
  sdpa_ctx* c = (sdpa_ctx*)vctx;
  int64_t b = task / c->Hq, h = task % c->Hq;
  int64_t G = c->Hq / c->Hkv, hk = h / G;
  int64_t L = c->L, S = c->S, D = c->D;
  const float* q = c->q + (b * c->Hq + h) * L * D;
  const float* k = c->k + (b * c->Hkv + hk) * S * D;
  const float* v = c->v + (b * c->Hkv + hk) * S * D;
  float* out = c->out + (b * c->Hq + h) * L * D;
  float* kT = (float*)scratch;
  float* sc = kT + D * S;
  for (int64_t j = 0; j < S; j++)
    for (int64_t p = 0; p < D; p++) kT[p * S + j] = k[j * D + p];
  for (int64_t i0 = 0; i0 < L; i0 += c->row_block) {
    int64_t i1 = i0 + c->row_block < L ? i0 + c->row_block : L;
    for (int64_t i = i0; i < i1; i++) {
      float* row = sc + (i - i0) * S;
      memset(row, 0, sizeof(float) * (size_t)S);
      for (int64_t p = 0; p < D; p++) {
        float a = q[i * D + p];
        const float* bp = kT + p * S;
        for (int64_t j = 0; j < S; j++) row[j] += a * bp[j];
      }
      scale_and_bias_row(row, S, i, c->scale, c->causal, c->mask_kind, c->mask);
      softmax_row(row, S);
    }
    for (int64_t i = i0; i < i1; i++) {
      const float* row = sc + (i - i0) * S;
      float* o = out + i * D;
      memset(o, 0, sizeof(float) * (size_t)D);
      for (int64_t p = 0; p < S; p++) {
        float a = row[p];
        const float* vp = v + p * D;
        for (int64_t d = 0; d < D; d++) o[d] += a * vp[d];
      }
    }
  }
}

static int bad_dims(int64_t B, int64_t Hq, int64_t Hkv, int64_t L, int64_t S, int64_t D) {
  return B < 0 || Hq < 1 || Hkv < 1 || L < 0 || S < 0 || D < 1 || Hq % Hkv != 0;
}

int oracle_sdpa_f32(const float* q, const float* k, const float* v, float* out, int64_t B, int64_t Hq, int64_t Hkv,
                    int64_t L, int64_t S, int64_t D, int causal, float scale, int mask_kind, const void* mask,
                    int nthreads) {
  if (bad_dims(B, Hq, Hkv, L, S, D)) return -1;
  if (mask_kind != ORACLE_MASK_NONE && !mask) return -1;
  if (B == 0 || L == 0) return 0;
  sdpa_ctx c;
  memset(&c, 0, sizeof(c));
  c.q = q, c.k = k, c.v = v, c.out = out;
  c.B = B, c.Hq = Hq, c.Hkv = Hkv, c.L = L, c.S = S, c.D = D;
  c.causal = causal, c.scale = scale, c.mask_kind = mask_kind, c.mask = mask;
  c.row_block = L < 64 ? L : 64;
  size_t scratch = sizeof(float) * (size_t)(D * S + c.row_block * S);
  if (scratch == 0) scratch = sizeof(float);
  return run_pool(slice_task, &c, B * Hq, scratch, nthreads);
}

/* One query row: the same per-element sums as slice_task (a left-to-right dot product over p is what the i,p,j loop
 * nest accumulates into each c[i,j]). */
static void row_task(void* vctx, int64_t task, void* scratch) {
  sdpa_ctx* c = (sdpa_ctx*)vctx;
  int64_t b = c->rows[3 * task], h = c->rows[3 * task + 1], i = c->rows[3 * task + 2];
  int64_t G = c->Hq / c->Hkv, hk = h / G;
  int64_t L = c->L, S = c->S, D = c->D;
  const float* q = c->q + ((b * c->Hq + h) * L + i) * D;
  const float* k = c->k + (b * c->Hkv + hk) * S * D;
  const float* v = c->v + (b * c->Hkv + hk) * S * D;
  float* o = c->out + task * D;
  float* row = (float*)scratch;
  for (int64_t j = 0; j < S; j++) {
    float acc = 0.f;
    const float* kj = k + j * D;
    for (int64_t p = 0; p < D; p++) acc += q[p] * kj[p];
    row[j] = acc;
  }
  scale_and_bias_row(row, S, i, c->scale, c->causal, ORACLE_MASK_NONE, NULL);
  softmax_row(row, S);
  memset(o, 0, sizeof(float) * (size_t)D);
  for (int64_t p = 0; p < S; p++) {
    float a = row[p];
    const float* vp = v + p * D;
    for (int64_t d = 0; d < D; d++) o[d] += a * vp[d];
  }
}

int oracle_sdpa_rows_f32(const float* q, const float* k, const float* v, float* out, int64_t B, int64_t Hq,
                         int64_t Hkv, int64_t L, int64_t S, int64_t D, int causal, float scale, const int64_t* rows,
                         int64_t nrows, int nthreads) {
  if (bad_dims(B, Hq, Hkv, L, S, D) || nrows < 0) return -1;
  for (int64_t t = 0; t < nrows; t++) {
    if (rows[3 * t] < 0 || rows[3 * t] >= B || rows[3 * t + 1] < 0 || rows[3 * t + 1] >= Hq || rows[3 * t + 2] < 0 ||
        rows[3 * t + 2] >= L)
      return -1;
  }
  if (nrows == 0) return 0;
  sdpa_ctx c;
  memset(&c, 0, sizeof(c));
  c.q = q, c.k = k, c.v = v, c.out = out;
  c.B = B, c.Hq = Hq, c.Hkv = Hkv, c.L = L, c.S = S, c.D = D;
  c.causal = causal, c.scale = scale;
  c.rows = rows, c.nrows = nrows;
  size_t scratch = sizeof(float) * (size_t)(S > 0 ? S : 1);
  return run_pool(row_task, &c, nrows, scratch, nthreads);
}

/* ------------------------------------------------------------------------------------------------------------------
 * Gradients of the attention path.  The reference has none (FuncSDPAttention::backward and FuncMatmul::backward are
 * NOT_IMPLEMENTED, reference src/Function/FuncNNLayer.h:267, src/Function/FuncLinalg.h:20): this is the chain rule
 * through the forward above, accumulated in double.  The softmax step is the reference's own
 * (src/Operation/OpNNLayerCpu.h:79-109: dx_j = y_j * (dy_j - sum_t y_t dy_t)); the matmul steps are dA = dC B^T,
 * dB = A^T dC.  One task per (batch, kv head): dK and dV sum over the query heads of the group in head order.
 * ---------------------------------------------------------------------------------------------------------------- */

typedef struct {
  const float *q, *k, *v, *dout;
  float *dq, *dk, *dv;
  int64_t B, Hq, Hkv, L, S, D;
  int causal;
  float scale;
  int mask_kind;
  const void* mask;
} sdpa_bwd_ctx;

/* scratch: p [S] double, dp [S] double, dk [S*D] double, dv [S*D] double */
static void bwd_task(void* vctx, int64_t task, void* scratch) {
  sdpa_bwd_ctx* c = (sdpa_bwd_ctx*)vctx;
  const int64_t b = task / c->Hkv, hk = task % c->Hkv;
  const int64_t G = c->Hq / c->Hkv, L = c->L, S = c->S, D = c->D;
  const float* k = c->k + (b * c->Hkv + hk) * S * D;
  const float* v = c->v + (b * c->Hkv + hk) * S * D;
  double* p = (double*)scratch;
  double* dp = p + S;
  double* dka = dp + S;
  double* dva = dka + S * D;
  for (int64_t i = 0; i < S * D; i++) dka[i] = 0.0, dva[i] = 0.0;
  for (int64_t g = 0; g < G; g++) {
    const int64_t h = hk * G + g;
    const float* q = c->q + (b * c->Hq + h) * L * D;
    const float* go = c->dout + (b * c->Hq + h) * L * D;
    float* dq = c->dq + (b * c->Hq + h) * L * D;
    for (int64_t i = 0; i < L; i++) {
      /* scores of row i with the forward's bias, softmax in double */
      double mx = -INFINITY;
      for (int64_t j = 0; j < S; j++) {
        double s = 0.0;
        for (int64_t d = 0; d < D; d++) s += (double)q[i * D + d] * (double)k[j * D + d];
        s *= (double)c->scale;
        if (c->causal && j > i) s = -INFINITY;
        if (c->mask_kind == ORACLE_MASK_BOOL && !((const uint8_t*)c->mask)[i * S + j]) s = -INFINITY;
        if (c->mask_kind == ORACLE_MASK_FLOAT) s += (double)((const float*)c->mask)[i * S + j];
        p[j] = s;
        if (s > mx) mx = s;
      }
      double sum = 0.0;
      for (int64_t j = 0; j < S; j++) {
        p[j] = exp(p[j] - mx);
        sum += p[j];
      }
      for (int64_t j = 0; j < S; j++) p[j] /= sum;
      /* out = P V:  dV += P^T dOut,  dP = dOut V^T */
      double dot = 0.0;
      for (int64_t j = 0; j < S; j++) {
        double t = 0.0;
        for (int64_t d = 0; d < D; d++) {
          t += (double)go[i * D + d] * (double)v[j * D + d];
          dva[j * D + d] += p[j] * (double)go[i * D + d];
        }
        dp[j] = t;
        dot += p[j] * t;
      }
      /* softmax: dS_j = P_j (dP_j - sum_t P_t dP_t); scores = scale * Q K^T: dQ = scale dS K, dK += scale dS^T Q */
      double acc[1024]; /* dQ row i; D <= 1024 is checked by the entry point */
      for (int64_t d = 0; d < D; d++) acc[d] = 0.0;
      for (int64_t j = 0; j < S; j++) {
        const double ds = p[j] * (dp[j] - dot) * (double)c->scale;
        if (ds == 0.0) continue;
        for (int64_t d = 0; d < D; d++) {
          acc[d] += ds * (double)k[j * D + d];
          dka[j * D + d] += ds * (double)q[i * D + d];
        }
      }
      for (int64_t d = 0; d < D; d++) dq[i * D + d] = (float)acc[d];
    }
  }
  float* dk = c->dk + (b * c->Hkv + hk) * S * D;
  float* dv = c->dv + (b * c->Hkv + hk) * S * D;
  for (int64_t i = 0; i < S * D; i++) dk[i] = (float)dka[i], dv[i] = (float)dva[i];
}

int oracle_sdpa_backward_f32(const float* q, const float* k, const float* v, const float* dout, float* dq, float* dk,
                             float* dv, int64_t B, int64_t Hq, int64_t Hkv, int64_t L, int64_t S, int64_t D,
                             int causal, float scale, int mask_kind, const void* mask, int nthreads) {
  if (bad_dims(B, Hq, Hkv, L, S, D) || D > 1024) return -1;
  if (mask_kind != ORACLE_MASK_NONE && !mask) return -1;
  if (B == 0) return 0;
  sdpa_bwd_ctx c;
  memset(&c, 0, sizeof(c));
  c.q = q, c.k = k, c.v = v, c.dout = dout, c.dq = dq, c.dk = dk, c.dv = dv;
  c.B = B, c.Hq = Hq, c.Hkv = Hkv, c.L = L, c.S = S, c.D = D;
  c.causal = causal, c.scale = scale, c.mask_kind = mask_kind, c.mask = mask;
  size_t scratch = sizeof(double) * (size_t)(2 * S + 2 * S * D + 1);
  return run_pool(bwd_task, &c, B * Hkv, scratch, nthreads);
}
