/* CPU oracle (test infrastructure only; see oracle.h). Build with -ffp-contract=off: Q5_K's d*q - m must not fuse. */
#include "oracle.h"

#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

#include "../macseek_amd/csrc/iq_codebooks.h"

/* ---------------------------------------------------------------- geometry (src/kernels/quant_types.hpp:13-34) */
int orc_block_elems(int t) {
  switch (t) {
    case ORC_F32: case ORC_F16: case ORC_BF16: return 1;
    case ORC_Q8_0: case ORC_IQ4_NL: return 32;
    case ORC_Q5_K: case ORC_Q6_K: case ORC_IQ2_XXS: case ORC_IQ1_S: return 256;
  }
  return 0;
}
size_t orc_block_bytes(int t) {
  switch (t) {
    case ORC_F32: return 4;
    case ORC_F16: case ORC_BF16: return 2;
    case ORC_Q8_0: return 34;
    case ORC_Q5_K: return 176;
    case ORC_Q6_K: return 210;
    case ORC_IQ2_XXS: return 66;
    case ORC_IQ1_S: return 50;
    case ORC_IQ4_NL: return 18;
  }
  return 0;
}
size_t orc_row_bytes(int t, int64_t cols) {
  const int be = orc_block_elems(t);
  return be ? (size_t)(cols / be) * orc_block_bytes(t) : 0;
}

/* ---------------------------------------------------------------- scalar conversions (tests/ref/dequant.cpp:17-19) */
float orc_fp16_to_f32(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1Fu, man = h & 0x3FFu, bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else { /* subnormal: normalise */
      int e = -1;
      do { man <<= 1; e++; } while (!(man & 0x400u));
      bits = sign | ((uint32_t)(112 - e) << 23) | ((man & 0x3FFu) << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7F800000u | (man << 13);
  } else {
    bits = sign | ((exp + 112) << 23) | (man << 13);
  }
  float f; memcpy(&f, &bits, 4); return f;
}
uint16_t orc_f32_to_fp16(float f) {
  uint32_t x; memcpy(&x, &f, 4);
  const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
  const uint32_t ax = x & 0x7FFFFFFFu;
  if (ax >= 0x7F800000u) return (uint16_t)(sign | 0x7C00u | (ax > 0x7F800000u ? 0x200u | ((ax >> 13) & 0x3FFu) : 0));
  if (ax >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u); /* >= 65520 rounds to inf */
  if (ax < 0x33000001u) return sign;                        /* <= 2^-25 rounds to zero */
  int e = (int)(ax >> 23) - 127;
  uint32_t man = (ax & 0x7FFFFFu) | 0x800000u;
  int shift; uint32_t hexp;
  if (e < -14) { shift = 13 + (-14 - e); hexp = 0; } else { shift = 13; hexp = (uint32_t)(e + 15); }
  uint32_t q = man >> shift, rem = man & ((1u << shift) - 1), half = 1u << (shift - 1);
  if (rem > half || (rem == half && (q & 1))) q++;
  /* q includes the implicit bit for normals: adding (hexp-1)<<10 lets a mantissa carry bump the exponent */
  uint32_t r = hexp ? ((hexp - 1) << 10) + q : q;
  return (uint16_t)(sign | r);
}
float orc_bf16_to_f32(uint16_t h) { uint32_t u = (uint32_t)h << 16; float f; memcpy(&f, &u, 4); return f; }
uint16_t orc_f32_to_bf16(float f) {
  uint32_t x; memcpy(&x, &f, 4);
  if ((x & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((x >> 16) | 0x40u);
  x += 0x7FFFu + ((x >> 16) & 1u);
  return (uint16_t)(x >> 16);
}

static inline uint16_t rd16(const uint8_t* p) { uint16_t v; memcpy(&v, p, 2); return v; }
static inline uint32_t rd32(const uint8_t* p) { uint32_t v; memcpy(&v, p, 4); return v; }

/* ---------------------------------------------------------------- codebooks */
static int8_t g_iq1s[MSQ_IQ1S_GRID_N][8];
static uint8_t g_iq2xxs[MSQ_IQ2XXS_GRID_N][8];
static pthread_once_t g_once = PTHREAD_ONCE_INIT;
static void init_tables(void) {
  static const uint8_t v2[3] = {8, 25, 43};
  for (int i = 0; i < MSQ_IQ1S_GRID_N; i++) {
    unsigned c = msq_iq1s_code[i];
    for (int j = 0; j < 8; j++, c /= 3) g_iq1s[i][j] = (int8_t)((int)(c % 3) - 1);
  }
  for (int i = 0; i < MSQ_IQ2XXS_GRID_N; i++) {
    unsigned c = msq_iq2xxs_code[i];
    for (int j = 0; j < 8; j++, c /= 3) g_iq2xxs[i][j] = v2[c % 3];
  }
}
static void tables(void) { pthread_once(&g_once, init_tables); }

void orc_iq1s_entry(int i, int8_t out[8]) { tables(); memcpy(out, g_iq1s[i & 2047], 8); }
void orc_iq2xxs_entry(int i, uint8_t out[8]) { tables(); memcpy(out, g_iq2xxs[i & 255], 8); }
/* ksigns_iq2xs[i] = i | parity(i) << 7 (tests/ref/dequant.cpp:13 uses the table; closed form per the format) */
uint8_t orc_ksign(int i) {
  i &= 127;
  return (uint8_t)(i | ((__builtin_popcount((unsigned)i) & 1) << 7));
}

static const int8_t kIQ4NL[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};

/* 6-bit scale/min of sub-block j from the 12 packed bytes (tests/ref/dequant.cpp:29-32) */
static void scale_min_k4(int j, const uint8_t* q, uint8_t* d, uint8_t* m) {
  if (j < 4) { *d = q[j] & 63; *m = q[j + 4] & 63; }
  else { *d = (uint8_t)((q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4)); *m = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4)); }
}

/* ---------------------------------------------------------------- dequant_row (tests/ref/dequant.cpp:34-120) */
int orc_dequant_row(int t, const void* srcv, float* y, int64_t n) {
  const uint8_t* s = (const uint8_t*)srcv;
  tables();
  switch (t) {
    case ORC_F32: memcpy(y, s, (size_t)n * 4); return 0;                                       /* :37 */
    case ORC_F16: for (int64_t i = 0; i < n; i++) y[i] = orc_fp16_to_f32(rd16(s + 2 * i)); return 0;  /* :38 */
    case ORC_BF16: for (int64_t i = 0; i < n; i++) y[i] = orc_bf16_to_f32(rd16(s + 2 * i)); return 0; /* :39 */
    case ORC_Q8_0:                                                                              /* :40-45 */
      for (int64_t b = 0; b < n / 32; b++, s += 34) {
        const float d = orc_fp16_to_f32(rd16(s));
        for (int j = 0; j < 32; j++) *y++ = (float)(int8_t)s[2 + j] * d;
      }
      return 0;
    case ORC_Q5_K:                                                                              /* :46-59 */
      for (int64_t b = 0; b < n / 256; b++, s += 176) {
        const float d = orc_fp16_to_f32(rd16(s)), mn = orc_fp16_to_f32(rd16(s + 2));
        const uint8_t *sc = s + 4, *qh = s + 16, *ql = s + 48;
        uint8_t u1 = 1, u2 = 2;
        for (int j = 0, is = 0; j < 256; j += 64, is += 2, ql += 32, u1 <<= 2, u2 <<= 2) {
          uint8_t a, m;
          scale_min_k4(is, sc, &a, &m);
          const float d1 = d * (float)a, m1 = mn * (float)m;
          scale_min_k4(is + 1, sc, &a, &m);
          const float d2 = d * (float)a, m2 = mn * (float)m;
          for (int l = 0; l < 32; l++) *y++ = d1 * (float)((ql[l] & 0xF) + (qh[l] & u1 ? 16 : 0)) - m1;
          for (int l = 0; l < 32; l++) *y++ = d2 * (float)((ql[l] >> 4) + (qh[l] & u2 ? 16 : 0)) - m2;
        }
      }
      return 0;
    case ORC_Q6_K:                                                                              /* :60-76 */
      for (int64_t b = 0; b < n / 256; b++, s += 210) {
        const float d = orc_fp16_to_f32(rd16(s + 208));
        const uint8_t *ql = s, *qh = s + 128;
        const int8_t* sc = (const int8_t*)(s + 192);
        for (int h = 0; h < 2; h++, y += 128, ql += 64, qh += 32, sc += 8)
          for (int l = 0; l < 32; l++) {
            const int is = l / 16;
            const int8_t q1 = (int8_t)((int8_t)((ql[l] & 0xF) | (((qh[l] >> 0) & 3) << 4)) - 32);
            const int8_t q2 = (int8_t)((int8_t)((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32);
            const int8_t q3 = (int8_t)((int8_t)((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32);
            const int8_t q4 = (int8_t)((int8_t)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32);
            y[l] = d * (float)sc[is] * (float)q1;
            y[l + 32] = d * (float)sc[is + 2] * (float)q2;
            y[l + 64] = d * (float)sc[is + 4] * (float)q3;
            y[l + 96] = d * (float)sc[is + 6] * (float)q4;
          }
      }
      return 0;
    case ORC_IQ1_S:                                                                             /* :77-91 */
      for (int64_t b = 0; b < n / 256; b++, s += 50) {
        const float d = orc_fp16_to_f32(rd16(s));
        const uint8_t* qs = s + 2;
        for (int ib = 0; ib < 8; ib++, qs += 4) {
          const uint16_t qh = rd16(s + 34 + 2 * ib);
          const float dl = d * (float)(2 * ((qh >> 12) & 7) + 1);
          const float delta = (qh & 0x8000) ? -0.125f : 0.125f;
          for (int l = 0; l < 4; l++, y += 8) {
            const int8_t* g = g_iq1s[qs[l] | (((qh >> 3 * l) & 7) << 8)];
            for (int j = 0; j < 8; j++) y[j] = dl * ((float)g[j] + delta);
          }
        }
      }
      return 0;
    case ORC_IQ2_XXS:                                                                           /* :92-106 */
      for (int64_t b = 0; b < n / 256; b++, s += 66) {
        const float d = orc_fp16_to_f32(rd16(s));
        for (int ib = 0; ib < 8; ib++) {
          const uint8_t* a8 = s + 2 + 8 * ib;
          const uint32_t a1 = rd32(a8 + 4);
          const float db = d * (0.5f + (float)(a1 >> 28)) * 0.25f;
          for (int l = 0; l < 4; l++, y += 8) {
            const uint8_t* g = g_iq2xxs[a8[l]];
            const uint8_t sg = orc_ksign((int)((a1 >> 7 * l) & 127));
            for (int j = 0; j < 8; j++) y[j] = db * (float)g[j] * ((sg & (1 << j)) ? -1.f : 1.f);
          }
        }
      }
      return 0;
    case ORC_IQ4_NL:                                                                            /* :107-112 */
      for (int64_t b = 0; b < n / 32; b++, s += 18, y += 32) {
        const float d = orc_fp16_to_f32(rd16(s));
        for (int j = 0; j < 16; j++) {
          y[j] = d * (float)kIQ4NL[s[2 + j] & 0xF];
          y[j + 16] = d * (float)kIQ4NL[s[2 + j] >> 4];
        }
      }
      return 0;
  }
  return -1;
}

/* ---------------------------------------------------------------- threads */
typedef void (*row_fn)(void* ctx, int r0, int r1);
typedef struct { row_fn fn; void* ctx; int r0, r1; } job_t;
static void* job_main(void* p) { job_t* j = (job_t*)p; j->fn(j->ctx, j->r0, j->r1); return NULL; }
static void par_rows(int rows, int nthreads, row_fn fn, void* ctx) {
  if (nthreads < 1) nthreads = 1;
  if (nthreads > rows) nthreads = rows > 0 ? rows : 1;
  if (nthreads == 1) { fn(ctx, 0, rows); return; }
  pthread_t* th = (pthread_t*)malloc(sizeof(pthread_t) * (size_t)nthreads);
  job_t* jb = (job_t*)malloc(sizeof(job_t) * (size_t)nthreads);
  for (int i = 0; i < nthreads; i++) {
    jb[i].fn = fn; jb[i].ctx = ctx;
    jb[i].r0 = (int)((int64_t)rows * i / nthreads); jb[i].r1 = (int)((int64_t)rows * (i + 1) / nthreads);
    pthread_create(&th[i], NULL, job_main, &jb[i]);
  }
  for (int i = 0; i < nthreads; i++) pthread_join(th[i], NULL);
  free(th); free(jb);
}

/* ---------------------------------------------------------------- matvec (tests/quant_test_util.hpp:29-42) */
typedef struct {
  int t, rows, cols, groups; const uint8_t* W; const float* x; double *y, *mag, *wn2;
} mv_ctx;
static void mv_rows(void* p, int r0, int r1) {
  mv_ctx* c = (mv_ctx*)p;
  float* w = (float*)malloc(sizeof(float) * (size_t)c->cols);
  const size_t rb = orc_row_bytes(c->t, c->cols);
  const int rpg = c->rows / c->groups;
  for (int r = r0; r < r1; r++) {
    orc_dequant_row(c->t, c->W + rb * (size_t)r, w, c->cols);
    const float* xg = c->x + (size_t)(r / rpg) * (size_t)c->cols;
    double s = 0, m = 0, n2 = 0;
    for (int k = 0; k < c->cols; k++) {
      const double pr = (double)w[k] * (double)xg[k];
      s += pr; m += fabs(pr); n2 += (double)w[k] * (double)w[k];
    }
    if (c->y) c->y[r] = s;
    if (c->mag) c->mag[r] = m;
    if (c->wn2) c->wn2[r] = n2;
  }
  free(w);
}
int orc_matvec(int t, const void* W, int rows, int cols, const float* x, int groups, double* y, double* mag,
               double* wn2, int nthreads) {
  const int be = orc_block_elems(t);
  if (!be || cols % be || groups < 1 || rows % groups) return -1;
  mv_ctx c = {t, rows, cols, groups, (const uint8_t*)W, x, y, mag, wn2};
  par_rows(rows, nthreads, mv_rows, &c);
  return 0;
}

/* ---------------------------------------------------------------- SwiGLU (tests/test_quant_moe.mm:14-18) */
double orc_swiglu(double g, double u, double w) {
  g = g < 10.0 ? g : 10.0;
  u = u < -10.0 ? -10.0 : (u > 10.0 ? 10.0 : u);
  return g / (1.0 + exp(-g)) * u * w;
}

/* ---------------------------------------------------------------- MoE decode (tests/test_quant_moe.mm:64-93) */
int orc_moe_decode(int t_gu, int t_down, int t_shared, int n_routed, int has_shared, int dim, int inter,
                   const void* const* gate, const void* const* up, const void* const* down, const float* wts,
                   const float* x, double* y, double* ymag, float* h_out, double* hscale, int nthreads) {
  const int n_exp = n_routed + (has_shared ? 1 : 0);
  double* g = (double*)malloc(sizeof(double) * (size_t)inter * 4);
  double *gm = g + inter, *u = gm + inter, *um = u + inter;
  float* h = (float*)malloc(sizeof(float) * (size_t)inter);
  double* yd = (double*)malloc(sizeof(double) * (size_t)dim * 2);
  double* ydm = yd + dim;
  if (ymag) for (int i = 0; i < dim; i++) ymag[i] = fabs(y[i]);
  int rc = 0;
  for (int e = 0; e < n_exp && !rc; e++) {
    const int sh = e == n_routed;
    const int tgu = sh ? t_shared : t_gu, td = sh ? t_shared : t_down;
    const double we = sh ? 1.0 : (double)wts[e];
    rc |= orc_matvec(tgu, gate[e], inter, dim, x, 1, g, gm, NULL, nthreads);
    rc |= orc_matvec(tgu, up[e], inter, dim, x, 1, u, um, NULL, nthreads);
    for (int r = 0; r < inter; r++) {
      h[r] = (float)orc_swiglu(g[r], u[r], we);
      if (h_out) h_out[(size_t)e * inter + r] = h[r];
      if (hscale) hscale[(size_t)e * inter + r] = fabs(we) * (gm[r] + um[r]);
    }
    rc |= orc_matvec(td, down[e], dim, inter, h, 1, yd, ydm, NULL, nthreads);
    for (int i = 0; i < dim; i++) { y[i] += yd[i]; if (ymag) ymag[i] += ydm[i]; }
  }
  free(g); free(h); free(yd);
  return rc;
}

/* ---------------------------------------------------------------- MoE prefill (tests/test_quant_moe_prefill.mm) */
static float round_act(float v, int mode) {
  if (mode == 1) return orc_fp16_to_f32(orc_f32_to_fp16(v));
  if (mode == 2) return orc_bf16_to_f32(orc_f32_to_bf16(v));
  return v;
}
/* out[q][r] = sum_c W[r][c] in[q][c], mag = sum |.| : rows split over threads like mm_ref (:25-47), double sums */
typedef struct {
  int t, rows, cols, nq; const uint8_t* W; const float* in; double *out, *mag;
} mm_ctx;
static void mm_rows(void* p, int r0, int r1) {
  mm_ctx* c = (mm_ctx*)p;
  float* w = (float*)malloc(sizeof(float) * (size_t)c->cols);
  const size_t rb = orc_row_bytes(c->t, c->cols);
  for (int r = r0; r < r1; r++) {
    orc_dequant_row(c->t, c->W + rb * (size_t)r, w, c->cols);
    for (int q = 0; q < c->nq; q++) {
      const float* x = c->in + (size_t)q * c->cols;
      double s = 0, a = 0;
      for (int k = 0; k < c->cols; k++) { const double pr = (double)w[k] * (double)x[k]; s += pr; a += fabs(pr); }
      c->out[(size_t)q * c->rows + r] = s;
      if (c->mag) c->mag[(size_t)q * c->rows + r] = a;
    }
  }
  free(w);
}
static void mm_ref(int t, const void* W, int rows, int cols, const float* in, int nq, double* out, double* mag, int nth) {
  mm_ctx c = {t, rows, cols, nq, (const uint8_t*)W, in, out, mag};
  par_rows(rows, nth, mm_rows, &c);
}

int orc_moe_prefill(int t_gu, int t_down, int t_shared, int n_tokens, int n_exp, int has_shared, int dim, int inter,
                    const void* const* gate, const void* const* up, const void* const* down, const int* offs,
                    const int* tok, const float* wt, const float* X, const int* chk, int n_chk, int x_round,
                    double* Y, double* Ymag, int nthreads) {
  int* ci = (int*)malloc(sizeof(int) * (size_t)n_tokens);
  for (int t = 0; t < n_tokens; t++) ci[t] = -1;
  for (int q = 0; q < n_chk; q++) ci[chk[q]] = q;
  const int ne_all = n_exp + (has_shared ? 1 : 0);
  int* toks = (int*)malloc(sizeof(int) * (size_t)(n_chk > 0 ? n_chk : 1));
  float* ws = (float*)malloc(sizeof(float) * (size_t)(n_chk > 0 ? n_chk : 1));
  for (int j = 0; j < ne_all; j++) {
    int nq = 0;
    if (j == n_exp) {
      for (int q = 0; q < n_chk; q++) { toks[nq] = chk[q]; ws[nq++] = 1.f; }
    } else {
      for (int i = offs[j]; i < offs[j + 1]; i++)
        if (ci[tok[i]] >= 0) { toks[nq] = tok[i]; ws[nq++] = wt[i]; }
    }
    if (!nq) continue;
    const int tgu = j == n_exp ? t_shared : t_gu, td = j == n_exp ? t_shared : t_down;
    float* xin = (float*)malloc(sizeof(float) * (size_t)nq * dim);
    for (int q = 0; q < nq; q++)
      for (int i = 0; i < dim; i++) xin[(size_t)q * dim + i] = round_act(X[(size_t)toks[q] * dim + i], x_round);
    double* g = (double*)malloc(sizeof(double) * (size_t)nq * inter * 2);
    double* u = g + (size_t)nq * inter;
    mm_ref(tgu, gate[j], inter, dim, xin, nq, g, NULL, nthreads);
    mm_ref(tgu, up[j], inter, dim, xin, nq, u, NULL, nthreads);
    float* h = (float*)malloc(sizeof(float) * (size_t)nq * inter);
    for (int q = 0; q < nq; q++)
      for (int r = 0; r < inter; r++)
        h[(size_t)q * inter + r] =
            round_act((float)orc_swiglu(g[(size_t)q * inter + r], u[(size_t)q * inter + r], (double)ws[q]), x_round);
    double* o = (double*)malloc(sizeof(double) * (size_t)nq * dim * 2);
    double* om = o + (size_t)nq * dim;
    mm_ref(td, down[j], dim, inter, h, nq, o, om, nthreads);
    for (int q = 0; q < nq; q++) {
      const int c = ci[toks[q]];
      for (int i = 0; i < dim; i++) {
        Y[(size_t)c * dim + i] += o[(size_t)q * dim + i];
        if (Ymag) Ymag[(size_t)c * dim + i] += om[(size_t)q * dim + i];
      }
    }
    free(xin); free(g); free(h); free(o);
  }
  free(ci); free(toks); free(ws);
  return 0;
}

/* ---------------------------------------------------------------- seeded inputs */
static inline uint64_t splitmix64(uint64_t* s) {
  uint64_t z = (*s += 0x9E3779B97F4A7C15ull);
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}
static inline double u01(uint64_t* s) { return ((double)(splitmix64(s) >> 11) + 0.5) * (1.0 / 9007199254740992.0); }
static inline double gauss(uint64_t* s) {
  const double a = u01(s), b = u01(s);
  return sqrt(-2.0 * log(a)) * cos(6.283185307179586476925 * b);
}
void orc_randn(float* out, int64_t n, uint64_t seed, float scale) {
  uint64_t s = seed * 0x9E3779B97F4A7C15ull + 0x1234567ull;
  for (int64_t i = 0; i < n; i++) out[i] = (float)(gauss(&s) * (double)scale);
}
int orc_random_blocks(int t, int64_t n, uint64_t seed, float scale, uint8_t* out) {
  const int be = orc_block_elems(t);
  const size_t bb = orc_block_bytes(t);
  if (!be || n % be) return -1;
  const int64_t nb = n / be;
  uint64_t s = seed * 0xD1342543DE82EF95ull + 0x9E3779B9ull;
  const size_t total = (size_t)nb * bb;
  size_t i = 0;
  for (; i + 8 <= total; i += 8) { uint64_t v = splitmix64(&s); memcpy(out + i, &v, 8); }
  if (i < total) { uint64_t v = splitmix64(&s); memcpy(out + i, &v, total - i); }
  for (int64_t b = 0; b < nb; b++) {
    uint8_t* p = out + (size_t)b * bb;
    const float sc = scale * (0.5f + 0.5f * (float)fabs(gauss(&s)));
    uint16_t h;
    switch (t) {
      case ORC_F32: { float f = (float)gauss(&s) * scale * 10; memcpy(p, &f, 4); } break;
      case ORC_F16: h = orc_f32_to_fp16((float)gauss(&s) * scale * 10); memcpy(p, &h, 2); break;
      case ORC_BF16: h = orc_f32_to_bf16((float)gauss(&s) * scale * 10); memcpy(p, &h, 2); break;
      case ORC_Q8_0: h = orc_f32_to_fp16(sc / 16); memcpy(p, &h, 2); break;
      case ORC_IQ4_NL: case ORC_IQ1_S: case ORC_IQ2_XXS: h = orc_f32_to_fp16(sc); memcpy(p, &h, 2); break;
      case ORC_Q5_K:
        h = orc_f32_to_fp16(sc / 8); memcpy(p, &h, 2);
        h = orc_f32_to_fp16(sc / 4); memcpy(p + 2, &h, 2);
        break;
      case ORC_Q6_K: h = orc_f32_to_fp16(sc / 32); memcpy(p + 208, &h, 2); break;
    }
  }
  return 0;
}

/* ---------------------------------------------------------------------------------------------- router, route lists */
void orc_router(const float* logits, const float* bias, int n_exp, int top_k, float route_scale, int* ids, float* w) {
  double* sc = (double*)malloc(sizeof(double) * (size_t)n_exp);
  double* key = (double*)malloc(sizeof(double) * (size_t)n_exp);
  for (int e = 0; e < n_exp; e++) {
    const double x = logits[e];
    const double sp = x > 20 ? x : log1p(exp(x));
    sc[e] = sqrt(sp);
    key[e] = (double)(float)((float)sc[e] + bias[e]);
  }
  double sum = 0;
  for (int k = 0; k < top_k; k++) { /* the first top_k of a stable descending sort: repeated first-maximum */
    int best = -1;
    for (int e = 0; e < n_exp; e++) {
      int taken = 0;
      for (int j = 0; j < k; j++) taken |= ids[j] == e;
      if (!taken && (best < 0 || key[e] > key[best])) best = e;
    }
    ids[k] = best;
    sum += sc[best];
  }
  for (int k = 0; k < top_k; k++) w[k] = (float)(sc[ids[k]] / (sum + 1e-20) * route_scale);
  free(sc);
  free(key);
}

void orc_route_lists(const int* ids, const float* w, int n_entries, int n_exp, int top_k, uint32_t* counts,
                     uint32_t* offsets, uint32_t* entry, uint32_t* tok, float* lw, uint32_t* slot_of) {
  memset(counts, 0, sizeof(uint32_t) * (size_t)n_exp);
  for (int i = 0; i < n_entries; i++) counts[ids[i]]++;
  offsets[0] = 0;
  for (int e = 0; e < n_exp; e++) offsets[e + 1] = offsets[e] + counts[e];
  uint32_t* fill = (uint32_t*)malloc(sizeof(uint32_t) * (size_t)n_exp);
  memcpy(fill, offsets, sizeof(uint32_t) * (size_t)n_exp);
  for (int i = 0; i < n_entries; i++) {
    const uint32_t p = fill[ids[i]]++;
    entry[p] = (uint32_t)i;
    tok[p] = (uint32_t)(i / top_k);
    lw[p] = w[i];
    slot_of[i] = p;
  }
  free(fill);
}

void orc_rmsnorm(const float* x, const float* w, float* y, int dim, double eps) {
  double ss = 0;
  for (int i = 0; i < dim; i++) ss += (double)x[i] * x[i];
  const double r = 1.0 / sqrt(ss / dim + eps);
  for (int i = 0; i < dim; i++) y[i] = (float)(x[i] * r * (w ? w[i] : 1.0f));
}
