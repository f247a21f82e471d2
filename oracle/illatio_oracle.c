/*
 * illatio_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A plain-C restatement of the CPU path of modus-lisp/illatio's quantized
 * matrix products, used only as the parity checker by tests/, by
 * __graft_entry__.smoke() and by bench.py's cpu_baseline leg.  Nothing in
 * the shipped library links, loads or calls this file.
 *
 * The reference is Common Lisp (SBCL); it cannot be built here, so every
 * function below follows the Lisp it cites, expression by expression, in
 * IEEE single precision with no fused multiply-add (build with
 * -ffp-contract=off, no -ffast-math).  Weights are read in GGUF byte order
 * (the reference's kmat reorders Q6_K in memory; the arithmetic is the same).
 *
 * Pinning (tests/test_oracle_*.py): fp16 conversions exhaustively against
 * IEEE binary16; block decoders against an independent numpy restatement of
 * the GGUF layouts and hand-built blocks; integer block sums by brute force;
 * the quantizers' special cases; row dots against a double-precision dot of
 * dequantized values (the reference's own criterion, inspect/iquant-test.lisp:
 * 45-53); d4-route against a stable sort (its hash-table branch against an
 * explicit evaluation and against the other branch on a row that is the
 * top choice); the IQ2_XXS tables against the
 * reference's three copies; swiglu!, f32-dot16, rope-table, rope-head!,
 * attend-head! against explicit evaluations in numpy (with the plausible
 * misreadings shown to give other bits), forward-1 as those pieces in order.
 *
 * No function here is unpinned.  Notes on three pins: orc_silu / orc_softplus /
 * orc_sigmoid use (float)f((double)x) as SBCL does for single-float arguments
 * (ds4f.lisp:248-254); they are checked against the correctly rounded value from
 * an independent extended-precision evaluation, which SBCL's libm call yields
 * except where the double result falls within ~2^-29 of a single-precision
 * rounding boundary (no test input does).  orc_rope_table's cos and sin are the
 * C library's double routines rounded to single, likewise; its theta sequence
 * and roundings are pinned against numpy with each rounding explicit.
 * orc_rmsnorm has no vector of the reference's: it is pinned by what its text
 * fixes, on inputs where each misreading gives other bits (see its comment).
 */
#include <float.h>
#include <math.h>
#include <pthread.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include "iq2xxs_tables.h"

#define QK_K 256

enum { ORC_Q8_0 = 8, ORC_Q2_K = 10, ORC_Q4_K = 12, ORC_Q6_K = 14, ORC_IQ2_XXS = 16 };

/* ---- src/half.lisp:20-36 ------------------------------------------------ */
static inline float bits_single(uint32_t b) { float f; memcpy(&f, &b, 4); return f; }
static inline uint32_t single_bits(float f) { uint32_t b; memcpy(&b, &f, 4); return b; }

float orc_half_to_single(uint16_t h) {
  uint32_t sign = (uint32_t)(h >> 15) << 31, exp = (h >> 10) & 31, man = h & 1023;
  if (exp == 31) return bits_single(sign | 0x7f800000u | (man << 13));
  if (exp != 0) return bits_single(sign | ((exp + 112) << 23) | (man << 13));
  if (man == 0) return bits_single(sign);
  uint32_t e = 113;
  while (!(man & 1024)) { man <<= 1; e--; }
  return bits_single(sign | (e << 23) | ((man & 1023) << 13));
}

/* ---- src/half.lisp:38-73: round to nearest even ----------------------------- */
uint16_t orc_single_to_half(float x) {
  uint32_t b = single_bits(x), sign = (b >> 31) << 15, exp = (b >> 23) & 255, man = b & 0x7fffff;
  if (exp == 255) return (uint16_t)(sign | 0x7c00 | (man ? 0x200 : 0));
  int e = (int)exp - 127;
  uint32_t sig = exp ? (man | 0x800000u) : man;
  if (e > 15) return (uint16_t)(sign | 0x7c00);
  int he = e + 15;
  int shift = he > 0 ? 13 : 13 + (1 - he);
  if (exp == 0 && shift < 14) shift = 14;
  if (shift > 24) return (uint16_t)sign;
  uint32_t q = sig >> shift, rem = sig & ((1u << shift) - 1), half = 1u << (shift - 1);
  if (rem > half || (rem == half && (q & 1))) q++;
  return (uint16_t)(sign | (he > 0 ? (((uint32_t)(he - 1) << 10) + q) : q));
}

static inline float f16_at(const uint8_t* p) { return orc_half_to_single((uint16_t)(p[0] | (p[1] << 8))); }
static inline uint32_t u32_le(const uint8_t* p) {
  return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
}

int64_t orc_block_bytes(int type) {
  switch (type) {
    case ORC_Q8_0: return 34; case ORC_Q2_K: return 84; case ORC_Q4_K: return 144;
    case ORC_Q6_K: return 210; case ORC_IQ2_XXS: return 66; default: return 0;
  }
}
int64_t orc_block_weights(int type) { return type == ORC_Q8_0 ? 32 : 256; }
int64_t orc_row_bytes(int type, int64_t cols) { return cols / orc_block_weights(type) * orc_block_bytes(type); }

/* ---- activations: src/tensor.lisp:245-262 (quantize-q8!) ------------------------ */
/* d = amax/127; the stored scale is d rounded through fp16 when f16_scale
   (*q8-f16-scale*), else d; q = round-half-even(x * (1/d)) with the unrounded d. */
void orc_quantize_q8(const float* x, int64_t n, int f16_scale, int8_t* q, float* s) {
  for (int64_t b = 0; b < n / 32; b++) {
    float amax = 0.0f;
    for (int j = 0; j < 32; j++) { float a = fabsf(x[b * 32 + j]); if (a > amax) amax = a; }
    float d = amax / 127.0f;
    float id = d == 0.0f ? 0.0f : 1.0f / d;
    s[b] = f16_scale ? orc_half_to_single(orc_single_to_half(d)) : d;
    for (int j = 0; j < 32; j++) q[b * 32 + j] = (int8_t)(int)rintf(x[b * 32 + j] * id);
  }
}

/* ---- activations: src/kquant.lisp:130-167 (quantize-q8k!) ----------------------- */
/* bsums: 16 per block (sums of 16 quants). */
void orc_quantize_q8k(const float* x, int64_t n, int8_t* q, float* d, int32_t* bsums) {
  for (int64_t b = 0; b < n / QK_K; b++) {
    const float* xb = x + b * QK_K;
    float mx = 0.0f, amax = 0.0f;
    for (int j = 0; j < QK_K; j++) { float v = xb[j], a = fabsf(v); if (a > amax) { amax = a; mx = v; } }
    if (amax == 0.0f) {
      d[b] = 0.0f;
      memset(q + b * QK_K, 0, QK_K);
      for (int g = 0; g < 16; g++) bsums[b * 16 + g] = 0;
      continue;
    }
    float iscale = -127.0f / mx;
    for (int g = 0; g < 16; g++) {
      int sum = 0;
      for (int k = 0; k < 16; k++) {
        int j = g * 16 + k;
        int v = (int)rintf(iscale * xb[j]);
        if (v > 127) v = 127;
        q[b * QK_K + j] = (int8_t)v;
        sum += v;
      }
      bsums[b * 16 + g] = sum;
    }
    d[b] = 1.0f / iscale;
  }
}

/* ---- Q8_0: src/tensor.lisp:321-336 (q8-row-dot-at) -------------------------------- */
/* wrow: GGUF Q8_0 blocks (f16 d, 32 int8).  acc_out (optional): the int32 block sums. */
float orc_q8_0_row_dot(const uint8_t* wrow, int64_t cols, const int8_t* xq, const float* xs, int32_t* acc_out) {
  float sum = 0.0f;
  for (int64_t b = 0; b < cols / 32; b++) {
    const uint8_t* blk = wrow + b * 34;
    const int8_t* wq = (const int8_t*)(blk + 2);
    int32_t acc = 0;
    for (int j = 0; j < 32; j++) acc += (int32_t)wq[j] * (int32_t)xq[b * 32 + j];
    if (acc_out) acc_out[b] = acc;
    float scale = f16_at(blk) * xs[b];
    sum = sum + (float)acc * scale;
  }
  return sum;
}

/* ---- src/kquant.lisp:64-72 (scale-min-k4) ------------------------------------------ */
void orc_scale_min_k4(int j, const uint8_t* q, int* sc, int* m) {
  if (j < 4) { *sc = q[j] & 63; *m = q[j + 4] & 63; }
  else { *sc = (q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4); *m = (q[j + 4] >> 4) | ((q[j] >> 6) << 4); }
}

/* ---- Q4_K: src/kquant.lisp:171-201 (q4k-row-dot) ------------------------------------- */
float orc_q4k_row_dot(const uint8_t* wrow, int64_t nb, const int8_t* yq, const float* yd, const int32_t* ybs,
                      int32_t* isum_out, int32_t* imin_out) {
  float sum = 0.0f;
  for (int64_t i = 0; i < nb; i++) {
    const uint8_t* blk = wrow + i * 144;
    float ydi = yd[i];
    float d = ydi * f16_at(blk), dmin = ydi * f16_at(blk + 2);
    int sc[8], mn[8];
    for (int g = 0; g < 8; g++) orc_scale_min_k4(g, blk + 4, &sc[g], &mn[g]);
    int32_t imin = 0, isum = 0;
    for (int g = 0; g < 8; g++) imin += mn[g] * (ybs[i * 16 + 2 * g] + ybs[i * 16 + 2 * g + 1]);
    sum = sum - dmin * (float)imin;
    for (int k = 0; k < 4; k++) {
      int32_t lo = 0, hi = 0;
      const uint8_t* qs = blk + 16 + k * 32;
      const int8_t* y = yq + i * QK_K + k * 64;
      for (int l = 0; l < 32; l++) { lo += (qs[l] & 0xF) * y[l]; hi += (qs[l] >> 4) * y[32 + l]; }
      isum += lo * sc[2 * k] + hi * sc[2 * k + 1];
    }
    if (isum_out) { isum_out[i] = isum; imin_out[i] = imin; }
    sum = sum + d * (float)isum;
  }
  return sum;
}

/* Q6_K weight idx (0..255) of a GGUF block as the 6-bit value 0..63 and its scale index. */
static inline int q6k_q(const uint8_t* blk, int idx, int* scale_idx) {
  int c = idx >> 7, r = idx & 127, part = r >> 5, l = r & 31;
  const uint8_t* ql = blk + 64 * c; const uint8_t* qh = blk + 128 + 32 * c;
  int lowbyte = ql[(part & 1) * 32 + l];
  int low = part < 2 ? (lowbyte & 0xF) : (lowbyte >> 4);
  int high = (qh[l] >> (2 * part)) & 3;
  *scale_idx = 8 * c + 2 * part + (l >> 4);
  return low | (high << 4);
}

/* ---- Q6_K: src/kquant.lisp:203-236 (q6k-row-dot) ----------------------------------------- */
float orc_q6k_row_dot(const uint8_t* wrow, int64_t nb, const int8_t* yq, const float* yd, const int32_t* ybs,
                      int32_t* isum_out, int32_t* imins_out) {
  float sum = 0.0f;
  for (int64_t i = 0; i < nb; i++) {
    const uint8_t* blk = wrow + i * 210;
    const int8_t* sc = (const int8_t*)(blk + 192);
    int32_t imins = 0, isum = 0;
    for (int g = 0; g < 16; g++) imins += ybs[i * 16 + g] * (int32_t)sc[g];
    for (int g = 0; g < 16; g++) {
      /* group g in scale order: c = g/8, part = (g%8)/2, half = g%2 -> weights 128c + 32part + 16half .. +16 */
      int base = 128 * (g >> 3) + 32 * ((g & 7) >> 1) + 16 * (g & 1);
      int32_t dot = 0; int si;
      for (int l = 0; l < 16; l++) dot += q6k_q(blk, base + l, &si) * (int32_t)yq[i * QK_K + base + l];
      isum += dot * (int32_t)sc[g];
    }
    if (isum_out) { isum_out[i] = isum; imins_out[i] = imins; }
    sum = sum + (f16_at(blk + 208) * yd[i]) * (float)(isum - 32 * imins);
  }
  return sum;
}

/* ---- IQ2_XXS: src/iquant.lisp:126-159 (iq2xxs-row-dot; ds4's NEON order) ------------------- */
static inline int32_t iq2xxs_sub_dot(const uint8_t* so, const int8_t* xb, uint32_t* aux_out) {
  uint32_t aux = u32_le(so + 4);
  int32_t isum = 0;
  for (int l = 0; l < 4; l++) {
    uint64_t g = orc_iq2xxs_grid[so[l]];
    uint8_t s = orc_ksigns_iq2xs[(aux >> (7 * l)) & 127];
    for (int j = 0; j < 8; j++) {
      int mag = (int)((g >> (8 * j)) & 0xFF);
      int sg = (s >> j) & 1 ? -1 : 1;
      isum += mag * sg * (int32_t)xb[l * 8 + j];
    }
  }
  *aux_out = aux;
  return isum;
}

float orc_iq2xxs_row_dot(const uint8_t* wrow, int64_t nb, const int8_t* yq, const float* yd, int32_t* isum_out) {
  float total = 0.0f;
  for (int64_t b = 0; b < nb; b++) {
    const uint8_t* bo = wrow + b * 66;
    float d = f16_at(bo) * yd[b];
    float suma = 0.0f, sumb = 0.0f;
    for (int ib = 0; ib < 8; ib++) {
      uint32_t aux;
      int32_t isum = iq2xxs_sub_dot(bo + 2 + ib * 8, yq + b * QK_K + ib * 32, &aux);
      if (isum_out) isum_out[b * 8 + ib] = isum;
      float term = (float)isum * (0.5f + (float)(aux >> 28));
      if ((ib & 1) == 0) suma = suma + term; else sumb = sumb + term;
    }
    total = total + d * (suma + sumb);
  }
  return 0.25f * total;
}

/* ---- IQ2_XXS, ggml's x86 order: src/avx2.lisp:77-110 (iq2xxs-dot-avx2) -------------------- */
float orc_iq2xxs_row_dot_avx2(const uint8_t* wrow, int64_t nb, const int8_t* yq, const float* yd) {
  float total = 0.0f;
  for (int64_t b = 0; b < nb; b++) {
    const uint8_t* bo = wrow + b * 66;
    int32_t sumi = 0;
    for (int ib = 0; ib < 8; ib++) {
      uint32_t aux;
      int32_t isum = iq2xxs_sub_dot(bo + 2 + ib * 8, yq + b * QK_K + ib * 32, &aux);
      sumi += isum * (int32_t)(2 * (aux >> 28) + 1);
    }
    total = total + (f16_at(bo) * yd[b]) * (float)sumi;
  }
  return 0.125f * total;
}

/* ---- Q2_K: src/iquant.lisp:179-215 (q2k-row-dot; ds4's NEON order) ------------------------- */
static void q2k_block_ints(const uint8_t* bo, const int8_t* xb, const int32_t* bs, int32_t* isum_o, int32_t* mins_o) {
  int32_t mins = 0, isum = 0;
  for (int j = 0; j < 16; j++) mins += (bo[j] >> 4) * bs[j];
  for (int h = 0; h < 2; h++)
    for (int k = 0; k < 4; k++)
      for (int half = 0; half < 2; half++) {
        int sc = bo[h * 8 + 2 * k + half] & 15;
        const uint8_t* qo = bo + 16 + h * 32 + half * 16;
        const int8_t* x2 = xb + h * 128 + k * 32 + half * 16;
        int32_t dot = 0;
        for (int l = 0; l < 16; l++) dot += ((qo[l] >> (2 * k)) & 3) * (int32_t)x2[l];
        isum += sc * dot;
      }
  *isum_o = isum; *mins_o = mins;
}

float orc_q2k_row_dot(const uint8_t* wrow, int64_t nb, const int8_t* yq, const float* yd, const int32_t* ybs,
                      int32_t* isum_out, int32_t* mins_out) {
  float sum = 0.0f;
  for (int64_t b = 0; b < nb; b++) {
    const uint8_t* bo = wrow + b * 84;
    float ydb = yd[b];
    float d = ydb * f16_at(bo + 80);
    float dmin = (-ydb) * f16_at(bo + 82);
    int32_t isum, mins;
    q2k_block_ints(bo, yq + b * QK_K, ybs + b * 16, &isum, &mins);
    if (isum_out) { isum_out[b] = isum; mins_out[b] = mins; }
    sum = sum + dmin * (float)mins;
    sum = sum + d * (float)isum;
  }
  return sum;
}

/* ---- Q2_K, ggml's x86 order: src/avx2.lisp:112-150 (q2k-dot-avx2) --------------------------- */
float orc_q2k_row_dot_avx2(const uint8_t* wrow, int64_t nb, const int8_t* yq, const float* yd, const int32_t* ybs) {
  float total = 0.0f;
  for (int64_t b = 0; b < nb; b++) {
    const uint8_t* bo = wrow + b * 84;
    float yb = yd[b];
    int32_t isum, mins;
    q2k_block_ints(bo, yq + b * QK_K, ybs + b * 16, &isum, &mins);
    float a = (yb * f16_at(bo + 80)) * (float)isum;
    float c = (yb * f16_at(bo + 82)) * (float)mins;
    total = total + (a - c);
  }
  return total;
}

/* ---- rows as floats: tensor.lisp:354-361, kquant.lisp:466-497, iquant.lisp:161-175, 217-230 ---- */
void orc_dequant_row(int type, const uint8_t* wrow, int64_t cols, float* out) {
  if (type == ORC_Q8_0) {
    for (int64_t b = 0; b < cols / 32; b++) {
      const uint8_t* blk = wrow + b * 34; float d = f16_at(blk);
      for (int j = 0; j < 32; j++) out[b * 32 + j] = d * (float)(int8_t)blk[2 + j];
    }
    return;
  }
  for (int64_t i = 0; i < cols / QK_K; i++) {
    float* y = out + i * QK_K;
    if (type == ORC_Q4_K) {
      const uint8_t* blk = wrow + i * 144;
      float d = f16_at(blk), mn = f16_at(blk + 2);
      for (int k = 0; k < 4; k++) {
        int s1, m1i, s2, m2i;
        orc_scale_min_k4(2 * k, blk + 4, &s1, &m1i); orc_scale_min_k4(2 * k + 1, blk + 4, &s2, &m2i);
        float d1 = d * (float)s1, m1 = mn * (float)m1i, d2 = d * (float)s2, m2 = mn * (float)m2i;
        for (int l = 0; l < 32; l++) {
          uint8_t byte = blk[16 + k * 32 + l];
          y[k * 64 + l] = d1 * (float)(byte & 0xF) - m1;
          y[k * 64 + 32 + l] = d2 * (float)(byte >> 4) - m2;
        }
      }
    } else if (type == ORC_Q6_K) {
      const uint8_t* blk = wrow + i * 210;
      const int8_t* sc = (const int8_t*)(blk + 192);
      float d = f16_at(blk + 208);
      for (int idx = 0; idx < 256; idx++) {
        int si; int q = q6k_q(blk, idx, &si);
        y[idx] = (d * (float)sc[si]) * (float)(q - 32);
      }
    } else if (type == ORC_Q2_K) {
      const uint8_t* bo = wrow + i * 84;
      float d = f16_at(bo + 80), dmin = f16_at(bo + 82);
      for (int h = 0; h < 2; h++) for (int k = 0; k < 4; k++) for (int half = 0; half < 2; half++) {
        uint8_t sb = bo[h * 8 + 2 * k + half];
        float dl = d * (float)(sb & 15), ml = dmin * (float)(sb >> 4);
        for (int l = 0; l < 16; l++)
          y[h * 128 + k * 32 + half * 16 + l] = dl * (float)((bo[16 + h * 32 + half * 16 + l] >> (2 * k)) & 3) - ml;
      }
    } else if (type == ORC_IQ2_XXS) {
      const uint8_t* bo = wrow + i * 66;
      float d = f16_at(bo);
      for (int ib = 0; ib < 8; ib++) {
        const uint8_t* so = bo + 2 + ib * 8;
        uint32_t aux = u32_le(so + 4);
        float db = (d * (0.5f + (float)(aux >> 28))) * 0.25f;
        for (int l = 0; l < 4; l++) {
          uint64_t g = orc_iq2xxs_grid[so[l]];
          uint8_t s = orc_ksigns_iq2xs[(aux >> (7 * l)) & 127];
          for (int j = 0; j < 8; j++)
            y[ib * 32 + l * 8 + j] = (db * (float)((g >> (8 * j)) & 0xFF)) * ((s >> j) & 1 ? -1.0f : 1.0f);
        }
      }
    }
  }
}

/* ---- the thread pool: src/pool.lisp:120-178.  Workers that stay: a worker spins on the pool's generation
        for a while after a job, then parks on a condition variable; pool-run publishes the job, wakes
        sleepers if there are any, runs share 0 itself and spins until the others are done.  One pool,
        remade when another size is asked for. ------------------------------------------------------------ */
typedef void (*orc_job_fn)(void* arg, int index, int count);
typedef struct {
  int size, stop;
  pthread_t* th;
  orc_job_fn fn; void* arg;
  unsigned generation; int pending, sleepers;
  pthread_mutex_t lock; pthread_cond_t wake;
} orc_pool;
typedef struct { orc_pool* p; int index; } orc_worker_arg;
static orc_pool* g_pool = NULL;
static pthread_mutex_t g_pool_lock = PTHREAD_MUTEX_INITIALIZER;
#define ORC_SPINS 200000

static void* orc_worker(void* va) {
  orc_worker_arg* wa = (orc_worker_arg*)va;
  orc_pool* p = wa->p; const int index = wa->index;
  free(wa);
  unsigned seen = 0;
  for (;;) {
    int spins = 0;
    while (__atomic_load_n(&p->generation, __ATOMIC_ACQUIRE) == seen && !__atomic_load_n(&p->stop, __ATOMIC_ACQUIRE)) {
      if (++spins < ORC_SPINS) { __builtin_ia32_pause(); continue; }
      pthread_mutex_lock(&p->lock);
      __atomic_fetch_add(&p->sleepers, 1, __ATOMIC_SEQ_CST);
      while (__atomic_load_n(&p->generation, __ATOMIC_ACQUIRE) == seen && !p->stop) pthread_cond_wait(&p->wake, &p->lock);
      __atomic_fetch_sub(&p->sleepers, 1, __ATOMIC_SEQ_CST);
      pthread_mutex_unlock(&p->lock);
    }
    if (__atomic_load_n(&p->stop, __ATOMIC_ACQUIRE)) return NULL;
    seen = __atomic_load_n(&p->generation, __ATOMIC_ACQUIRE);
    p->fn(p->arg, index, p->size);
    __atomic_fetch_sub(&p->pending, 1, __ATOMIC_RELEASE);
  }
}
static void orc_pool_free(orc_pool* p) {
  pthread_mutex_lock(&p->lock);
  __atomic_store_n(&p->stop, 1, __ATOMIC_RELEASE);
  pthread_cond_broadcast(&p->wake);
  pthread_mutex_unlock(&p->lock);
  for (int i = 1; i < p->size; i++) pthread_join(p->th[i], NULL);
  free(p->th); free(p);
}
static orc_pool* orc_pool_of(int size) {
  if (g_pool && g_pool->size == size) return g_pool;
  if (g_pool) { orc_pool_free(g_pool); g_pool = NULL; }
  orc_pool* p = (orc_pool*)calloc(1, sizeof(orc_pool));
  p->size = size; p->th = (pthread_t*)calloc(size, sizeof(pthread_t));
  pthread_mutex_init(&p->lock, NULL); pthread_cond_init(&p->wake, NULL);
  for (int i = 1; i < size; i++) {
    orc_worker_arg* wa = (orc_worker_arg*)malloc(sizeof(orc_worker_arg));
    wa->p = p; wa->index = i;
    pthread_create(&p->th[i], NULL, orc_worker, wa);
  }
  return g_pool = p;
}
static void orc_pool_run(int nthreads, orc_job_fn fn, void* arg) {
  if (nthreads <= 1) { fn(arg, 0, 1); return; }
  pthread_mutex_lock(&g_pool_lock);                   /* one caller at a time */
  orc_pool* p = orc_pool_of(nthreads);
  p->fn = fn; p->arg = arg;
  __atomic_store_n(&p->pending, p->size - 1, __ATOMIC_RELEASE);
  __atomic_fetch_add(&p->generation, 1, __ATOMIC_SEQ_CST);
  if (__atomic_load_n(&p->sleepers, __ATOMIC_SEQ_CST) > 0) {
    pthread_mutex_lock(&p->lock); pthread_cond_broadcast(&p->wake); pthread_mutex_unlock(&p->lock);
  }
  fn(arg, 0, p->size);
  while (__atomic_load_n(&p->pending, __ATOMIC_ACQUIRE) != 0) __builtin_ia32_pause();
  pthread_mutex_unlock(&g_pool_lock);
}
static inline void share(int64_t n, int index, int count, int64_t* s, int64_t* e) {
  *s = n * index / count; *e = n * (index + 1) / count;
}

/* ---- one quantized activation set (qact, kquant.lisp:504-530) ------------------------------------ */
typedef struct {
  int64_t n;            /* elements per token */
  int8_t* q8; float* s8;                    /* Q8_0 */
  int8_t* q8k; float* dk; int32_t* bsums;   /* Q8_K */
} orc_act;

/* ---- W.x for ntok tokens: matvec!/kmatvec!/matmul! (tensor.lisp:338-352, kquant.lisp:537-554,
        batch.lisp:128-153): out[t*rows + r] = row dot, each (row, token) on its own ------------------ */
typedef struct {
  int type; const uint8_t* w; int64_t rows, cols, ntok;
  const int8_t* xq; const float* xs; const int32_t* bsums; float* out;
} orc_mm_args;

static float orc_row_dot_any(int type, const uint8_t* wrow, int64_t cols, const int8_t* xq, const float* xs,
                             const int32_t* bs) {
  switch (type) {
    case ORC_Q8_0: return orc_q8_0_row_dot(wrow, cols, xq, xs, NULL);
    case ORC_Q4_K: return orc_q4k_row_dot(wrow, cols / QK_K, xq, xs, bs, NULL, NULL);
    case ORC_Q6_K: return orc_q6k_row_dot(wrow, cols / QK_K, xq, xs, bs, NULL, NULL);
    case ORC_Q2_K: return orc_q2k_row_dot(wrow, cols / QK_K, xq, xs, bs, NULL, NULL);
    case ORC_IQ2_XXS: return orc_iq2xxs_row_dot(wrow, cols / QK_K, xq, xs, NULL);
  }
  return NAN;
}

static void orc_mm_job(void* p, int index, int count) {
  orc_mm_args* a = (orc_mm_args*)p;
  int64_t rb = orc_row_bytes(a->type, a->cols), bw = orc_block_weights(a->type);
  if (a->type == ORC_Q8_0) {
    /* groups of four rows split across the pool (tensor.lisp:345-347) */
    int64_t s, e; share(a->rows / 4, index, count, &s, &e);
    for (int64_t g = s; g < e; g++)
      for (int64_t t = 0; t < a->ntok; t++)
        for (int k = 0; k < 4; k++) {
          int64_t r = 4 * g + k;
          a->out[t * a->rows + r] = orc_q8_0_row_dot(a->w + r * rb, a->cols, a->xq + t * a->cols,
                                                    a->xs + t * (a->cols / 32), NULL);
        }
    if (index == count - 1)
      for (int64_t r = a->rows / 4 * 4; r < a->rows; r++)
        for (int64_t t = 0; t < a->ntok; t++)
          a->out[t * a->rows + r] = orc_q8_0_row_dot(a->w + r * rb, a->cols, a->xq + t * a->cols,
                                                    a->xs + t * (a->cols / 32), NULL);
    return;
  }
  /* rows shared out, 64 KB tiles of rows, every token over a tile before the next
     (kquant.lisp:261-267, 315-326) */
  int64_t s, e; share(a->rows, index, count, &s, &e);
  int64_t tile = 65536 / rb; if (tile < 1) tile = 1;
  for (int64_t t0 = s; t0 < e; t0 += tile)
    for (int64_t t = 0; t < a->ntok; t++)
      for (int64_t r = t0; r < e && r < t0 + tile; r++)
        a->out[t * a->rows + r] = orc_row_dot_any(a->type, a->w + r * rb, a->cols, a->xq + t * a->cols,
                                                  a->xs + t * (a->cols / bw),
                                                  a->bsums ? a->bsums + t * (a->cols / 16) : NULL);
}

/* x: ntok rows of cols floats.  Quantizes as the format asks (Q8_0 -> Q8_0 activations with
   f16_scale; others -> Q8_K), then the product.  out[t*rows + r]. */
void orc_matmul(int type, const uint8_t* w, int64_t rows, int64_t cols, const float* x, int64_t ntok,
                int f16_scale, float* out, int nthreads) {
  int64_t n = ntok * cols;
  int8_t* xq = (int8_t*)malloc(n);
  float* xs; int32_t* bs = NULL;
  if (type == ORC_Q8_0) {
    xs = (float*)malloc(sizeof(float) * (n / 32));
    for (int64_t t = 0; t < ntok; t++) orc_quantize_q8(x + t * cols, cols, f16_scale, xq + t * cols, xs + t * (cols / 32));
  } else {
    xs = (float*)malloc(sizeof(float) * (n / QK_K));
    bs = (int32_t*)malloc(sizeof(int32_t) * (n / 16));
    for (int64_t t = 0; t < ntok; t++)
      orc_quantize_q8k(x + t * cols, cols, xq + t * cols, xs + t * (cols / QK_K), bs + t * (cols / 16));
  }
  orc_mm_args a = { type, w, rows, cols, ntok, xq, xs, bs, out };
  orc_pool_run(nthreads, orc_mm_job, &a);
  free(xq); free(xs); free(bs);
}

/* The product alone, activations already quantized (for timing the kernel loop by itself). */
void orc_matmul_q(int type, const uint8_t* w, int64_t rows, int64_t cols, const int8_t* xq, const float* xs,
                  const int32_t* bsums, int64_t ntok, float* out, int nthreads) {
  orc_mm_args a = { type, w, rows, cols, ntok, xq, xs, bsums, out };
  orc_pool_run(nthreads, orc_mm_job, &a);
}

/* ---- f32-dot16 (src/tensor.lisp:370-378): column i's product into partial sum i mod 16; the sixteen sums
        combined as c(j) = (s[j] + s[4+j]) + (s[8+j] + s[12+j]), (c(0) + c(1)) + (c(2) + c(3)) ------------------ */
float orc_f32_dot16(const float* a, const float* b, int64_t n) {
  float s[16];
  for (int l = 0; l < 16; l++) s[l] = 0.0f;
  for (int64_t i = 0; i < n; i++) { volatile float p = a[i] * b[i]; s[i & 15] = s[i & 15] + p; }
  float c[4];
  for (int j = 0; j < 4; j++) { volatile float u = s[j] + s[4 + j], v = s[8 + j] + s[12 + j]; c[j] = u + v; }
  volatile float u = c[0] + c[1], v = c[2] + c[3];
  return u + v;
}
/* f32mm! (src/ds4f.lisp:278-293) for a matrix held as halves (widening is exact): out[t*rows + r] */
void orc_f16mm(const uint16_t* w, int64_t rows, int64_t cols, const float* x, int64_t ntok, float* out) {
  float* wr = (float*)malloc(sizeof(float) * cols);
  for (int64_t r = 0; r < rows; r++) {
    for (int64_t c = 0; c < cols; c++) wr[c] = orc_half_to_single(w[r * cols + c]);
    for (int64_t t = 0; t < ntok; t++) out[t * rows + r] = orc_f32_dot16(wr, x + t * cols, cols);
  }
  free(wr);
}

/* ---- src/ds4f.lisp:248-254 ------------------------------------------------------------------------ */
static inline float sb_exp(float x) { return (float)exp((double)x); }
static inline float sb_log(float x) { return (float)log((double)x); }
/* rmsnorm! (model.lisp:205-216): the squares are single-float products, added one after
   another in double; scale = 1 / sqrt(float(sum/n + eps)); out = (x * scale) * w.
   The reference holds no vector for it; tests pin it against what the formula fixes (closed
   forms, the float-rounded squares, the order of the two products), on inputs where each
   misreading gives other bits. */
void orc_rmsnorm(const float* x, const float* w, float* out, float eps, int64_t n) {
  double sum = 0.0;
  for (int64_t i = 0; i < n; i++) { volatile float sq = x[i] * x[i]; sum += (double)sq; }
  const float scale = 1.0f / sqrtf((float)(sum / (double)n + (double)eps));
  for (int64_t i = 0; i < n; i++) { volatile float t = x[i] * scale; out[i] = t * w[i]; }
}

float orc_sigmoid(float x) {
  if (x >= 0.0f) return 1.0f / (1.0f + sb_exp(-x));
  float e = sb_exp(x); return e / (1.0f + e);
}
float orc_silu(float x) { return x * orc_sigmoid(x); }
float orc_softplus(float x) {
  if (x > 20.0f) return x;
  if (x < -20.0f) return sb_exp(x);
  return sb_log(1.0f + sb_exp(x));
}

/* ---- src/model.lisp:364-378 (swiglu!): silu(x) = x / (1 + e^-x), times b ------------------------------ */
float orc_swiglu(float x, float b) { return (x / (1.0f + sb_exp(-x))) * b; }

/* ---- src/ds4f.lisp:950-978 (d4-route), the top-N_USED branch --------------------------------------- */
/* sel: nu expert indices in descending-score order; w: their weights.  bias may be NULL. */
void orc_route(const float* logits, const float* bias, int ne, int nu, float scale, int32_t* sel, float* w) {
  float* probs = (float*)malloc(sizeof(float) * ne);
  float* s = (float*)malloc(sizeof(float) * ne);
  for (int i = 0; i < ne; i++) { probs[i] = sqrtf(orc_softplus(logits[i])); s[i] = probs[i]; }
  if (bias) for (int i = 0; i < ne; i++) s[i] = s[i] + bias[i];
  for (int j = 0; j < nu; j++) sel[j] = -1;
  for (int i = 0; i < ne; i++)
    for (int j = 0; j < nu; j++)
      if (sel[j] < 0 || s[i] > s[sel[j]]) {
        for (int k = nu - 1; k > j; k--) sel[k] = sel[k - 1];
        sel[j] = i;
        break;
      }
  float sum = 0.0f;
  for (int i = 0; i < nu; i++) { w[i] = probs[sel[i]]; sum = sum + w[i]; }
  if (sum < 6.103515625e-5f) sum = 6.103515625e-5f;
  for (int i = 0; i < nu; i++) w[i] = (w[i] / sum) * scale;
  free(probs); free(s);
}

/* ---- src/ds4f.lisp:961-963, 973-977 (d4-route), the hash-table branch ------------------------------- */
/* The first layers of the model take a token's experts from a table: sel[i] = tid2eid[token*nu + i],
   in the table's order (no sorting, duplicates and all); the weights are formed from the unbiased
   probabilities exactly as in the top-N_USED branch (the bias plays no part: it only enters the
   scores the other branch picks by). */
void orc_route_table(const float* logits, const int32_t* tid2eid, int token, int ne, int nu, float scale,
                     int32_t* sel, float* w) {
  for (int i = 0; i < nu; i++) sel[i] = tid2eid[(int64_t)token * nu + i];
  float sum = 0.0f;
  for (int i = 0; i < nu; i++) { w[i] = sqrtf(orc_softplus(logits[sel[i]])); sum = sum + w[i]; }
  if (sum < 6.103515625e-5f) sum = 6.103515625e-5f;
  for (int i = 0; i < nu; i++) w[i] = (w[i] / sum) * scale;
  (void)ne;
}

/* ---- the routed experts of one token: src/ds4f.lisp:994-1037 (d4-routed!) ------------------------ */
/* Expert e's gate rows at gate + e*ff*grb, up likewise, down at down + e*d*drb
   (ds4f.lisp:95-100, 1014).  mid_out (optional): nu*ff floats. */
typedef struct {
  const uint8_t *gate, *up, *down; int d, ff, nu; const int32_t* sel; const float* w; float clamp;
  const int8_t* xq; const float* xd; float* mid;
  const int8_t* mq; const float* md; const int32_t* mbs; float* moe; int avx2;
} orc_routed_args;

static void orc_routed_gu_job(void* p, int index, int count) {
  orc_routed_args* a = (orc_routed_args*)p;
  int64_t grb = (int64_t)a->d / QK_K * 66, nb = a->d / QK_K;
  int64_t s, e; share((int64_t)a->nu * a->ff, index, count, &s, &e);
  for (int64_t idx = s; idx < e; idx++) {
    int slot = (int)(idx / a->ff); int64_t r = idx % a->ff;
    int64_t ex = a->sel[slot];
    const uint8_t* grow = a->gate + (ex * a->ff + r) * grb;
    const uint8_t* urow = a->up + (ex * a->ff + r) * grb;
    float g = a->avx2 ? orc_iq2xxs_row_dot_avx2(grow, nb, a->xq, a->xd) : orc_iq2xxs_row_dot(grow, nb, a->xq, a->xd, NULL);
    float u = a->avx2 ? orc_iq2xxs_row_dot_avx2(urow, nb, a->xq, a->xd) : orc_iq2xxs_row_dot(urow, nb, a->xq, a->xd, NULL);
    if (a->clamp > 1e-6f) { g = g < a->clamp ? g : a->clamp; float t = u < a->clamp ? u : a->clamp; u = t > -a->clamp ? t : -a->clamp; }
    a->mid[idx] = (orc_silu(g) * u) * a->w[slot];
  }
}

static void orc_routed_down_job(void* p, int index, int count) {
  orc_routed_args* a = (orc_routed_args*)p;
  int64_t drb = (int64_t)a->ff / QK_K * 84, nb = a->ff / QK_K;
  int64_t s, e; share(a->d, index, count, &s, &e);
  for (int64_t r = s; r < e; r++) {
    float acc = 0.0f;
    for (int i = 0; i < a->nu; i++) {
      const uint8_t* row = a->down + ((int64_t)a->sel[i] * a->d + r) * drb;
      const int8_t* q = a->mq + (int64_t)i * a->ff; const float* dd = a->md + (int64_t)i * nb;
      const int32_t* bs = a->mbs + (int64_t)i * (a->ff / 16);
      acc = acc + (a->avx2 ? orc_q2k_row_dot_avx2(row, nb, q, dd, bs) : orc_q2k_row_dot(row, nb, q, dd, bs, NULL, NULL));
    }
    a->moe[r] = acc;
  }
}

void orc_moe_routed(const uint8_t* gate, const uint8_t* up, const uint8_t* down, int d, int ff, int nu,
                    const int32_t* sel, const float* w, float clamp, const float* norm,
                    float* moe, float* mid_out, int avx2, int nthreads) {
  int8_t* xq = (int8_t*)malloc(d); float* xd = (float*)malloc(sizeof(float) * (d / QK_K));
  int32_t* xbs = (int32_t*)malloc(sizeof(int32_t) * (d / 16));
  orc_quantize_q8k(norm, d, xq, xd, xbs);
  float* mid = (float*)malloc(sizeof(float) * nu * ff);
  int8_t* mq = (int8_t*)malloc((size_t)nu * ff); float* md = (float*)malloc(sizeof(float) * nu * (ff / QK_K));
  int32_t* mbs = (int32_t*)malloc(sizeof(int32_t) * nu * (ff / 16));
  orc_routed_args a = { gate, up, down, d, ff, nu, sel, w, clamp, xq, xd, mid, mq, md, mbs, moe, avx2 };
  orc_pool_run(nthreads, orc_routed_gu_job, &a);
  for (int i = 0; i < nu; i++)
    orc_quantize_q8k(mid + (int64_t)i * ff, ff, mq + (int64_t)i * ff, md + (int64_t)i * (ff / QK_K), mbs + (int64_t)i * (ff / 16));
  orc_pool_run(nthreads, orc_routed_down_job, &a);
  if (mid_out) memcpy(mid_out, mid, sizeof(float) * nu * ff);
  free(xq); free(xd); free(xbs); free(mid); free(mq); free(md); free(mbs);
}

/* ---- the shared expert: src/ds4f.lisp:1039-1048 (d4-shared!), q8mv! :293-296 with
        *q8-f16-scale* NIL (ds4f.lisp:1052-1053) ------------------------------------------------------ */
void orc_moe_shared(const uint8_t* sgate, const uint8_t* sup, const uint8_t* sdown, int d, int ff, float clamp,
                    const float* norm, float* out, int nthreads) {
  float* g = (float*)malloc(sizeof(float) * ff); float* u = (float*)malloc(sizeof(float) * ff);
  orc_matmul(ORC_Q8_0, sgate, ff, d, norm, 1, 0, g, nthreads);
  orc_matmul(ORC_Q8_0, sup, ff, d, norm, 1, 0, u, nthreads);
  for (int i = 0; i < ff; i++) {
    float gi = g[i], ui = u[i];
    if (clamp > 1e-6f) { gi = gi < clamp ? gi : clamp; float t = ui < clamp ? ui : clamp; ui = t > -clamp ? t : -clamp; }
    g[i] = orc_silu(gi) * ui;
  }
  orc_matmul(ORC_Q8_0, sdown, d, ff, g, 1, 0, out, nthreads);
  free(g); free(u);
}

/* ---- one token's FFN past the router: d4-ffn (ds4f.lisp:980-992) without HC ----------------------- */
void orc_moe_token(const uint8_t* gate, const uint8_t* up, const uint8_t* down,
                   const uint8_t* sgate, const uint8_t* sup, const uint8_t* sdown,
                   int d, int ff, int ne, int nu, float scale, float clamp,
                   const float* logits, const float* bias, const float* norm,
                   int32_t* sel_out, float* w_out, float* out, int avx2, int nthreads) {
  int32_t* sel = (int32_t*)malloc(sizeof(int32_t) * nu); float* w = (float*)malloc(sizeof(float) * nu);
  float* shared = (float*)malloc(sizeof(float) * d);
  orc_route(logits, bias, ne, nu, scale, sel, w);
  orc_moe_routed(gate, up, down, d, ff, nu, sel, w, clamp, norm, out, NULL, avx2, nthreads);
  orc_moe_shared(sgate, sup, sdown, d, ff, clamp, norm, shared, nthreads);
  for (int i = 0; i < d; i++) out[i] = out[i] + shared[i];
  if (sel_out) memcpy(sel_out, sel, sizeof(int32_t) * nu);
  if (w_out) memcpy(w_out, w, sizeof(float) * nu);
  free(sel); free(w); free(shared);
}

/* ---- a chunk, layer-major: src/ds4f.lisp:1169-1239.  Route every token, group (token, slot)
        rows by expert in token order, experts ascending, each expert's rows once for all its
        tokens, each (token, slot)'s down row kept apart, summed per token in slot order --------------- */
typedef struct {
  const uint8_t *gate, *up, *down; int d, ff, nu, n; float clamp;
  int nexp; const int32_t* experts; const int32_t* ubase; const int32_t* users; /* (tk*nu+slot) per user */
  const float* ws; const int8_t* xq; const float* xd;
  float* mid; const int8_t* mq; const float* md; const int32_t* mbs; float* downs;
} orc_chunk_args;

static void orc_chunk_gu_job(void* p, int index, int count) {
  orc_chunk_args* a = (orc_chunk_args*)p;
  int64_t grb = (int64_t)a->d / QK_K * 66, nb = a->d / QK_K;
  int64_t s, e; share((int64_t)a->nexp * a->ff, index, count, &s, &e);
  for (int64_t item = s; item < e; item++) {
    int k = (int)(item / a->ff); int64_t r = item % a->ff; int64_t ex = a->experts[k];
    const uint8_t* grow = a->gate + (ex * a->ff + r) * grb;
    const uint8_t* urow = a->up + (ex * a->ff + r) * grb;
    for (int32_t ui = a->ubase[k]; ui < a->ubase[k + 1]; ui++) {
      int64_t ts = a->users[ui], tk = ts / a->nu;
      float g = orc_iq2xxs_row_dot(grow, nb, a->xq + tk * a->d, a->xd + tk * nb, NULL);
      float u = orc_iq2xxs_row_dot(urow, nb, a->xq + tk * a->d, a->xd + tk * nb, NULL);
      if (a->clamp > 1e-6f) { g = g < a->clamp ? g : a->clamp; float t = u < a->clamp ? u : a->clamp; u = t > -a->clamp ? t : -a->clamp; }
      a->mid[ts * a->ff + r] = (orc_silu(g) * u) * a->ws[ts];
    }
  }
}

static void orc_chunk_down_job(void* p, int index, int count) {
  orc_chunk_args* a = (orc_chunk_args*)p;
  int64_t drb = (int64_t)a->ff / QK_K * 84, nb = a->ff / QK_K;
  int64_t s, e; share((int64_t)a->nexp * a->d, index, count, &s, &e);
  for (int64_t item = s; item < e; item++) {
    int k = (int)(item / a->d); int64_t r = item % a->d; int64_t ex = a->experts[k];
    const uint8_t* row = a->down + (ex * a->d + r) * drb;
    for (int32_t ui = a->ubase[k]; ui < a->ubase[k + 1]; ui++) {
      int64_t ts = a->users[ui];
      a->downs[ts * a->d + r] = orc_q2k_row_dot(row, nb, a->mq + ts * a->ff, a->md + ts * nb, a->mbs + ts * (a->ff / 16), NULL, NULL);
    }
  }
}

/* logits: n*ne; norms: n*d; shared (optional): n*d added after the slot-ordered sum.
   out: n*d.  sel_out/w_out (optional): n*nu.  counts_out (optional): ne rows per expert. */
void orc_moe_chunk(const uint8_t* gate, const uint8_t* up, const uint8_t* down, int d, int ff, int ne, int nu,
                   float scale, float clamp, int n, const float* logits, const float* bias, const float* norms,
                   const float* shared, float* out, int32_t* sel_out, float* w_out, int32_t* counts_out,
                   int nthreads) {
  int64_t rows = (int64_t)n * nu;
  int32_t* sels = (int32_t*)malloc(sizeof(int32_t) * rows); float* ws = (float*)malloc(sizeof(float) * rows);
  for (int t = 0; t < n; t++) orc_route(logits + (int64_t)t * ne, bias, ne, nu, scale, sels + (int64_t)t * nu, ws + (int64_t)t * nu);
  int32_t* counts = (int32_t*)calloc(ne + 1, sizeof(int32_t));
  for (int64_t i = 0; i < rows; i++) counts[sels[i]]++;
  int32_t* experts = (int32_t*)malloc(sizeof(int32_t) * ne); int32_t* ubase = (int32_t*)malloc(sizeof(int32_t) * (ne + 1));
  int32_t* ebase = (int32_t*)malloc(sizeof(int32_t) * ne);
  int nexp = 0; int32_t acc = 0;
  for (int e = 0; e < ne; e++) { ebase[e] = acc; if (counts[e]) { experts[nexp] = e; ubase[nexp] = acc; nexp++; } acc += counts[e]; }
  ubase[nexp] = acc;
  int32_t* users = (int32_t*)malloc(sizeof(int32_t) * rows); int32_t* fill = (int32_t*)calloc(ne, sizeof(int32_t));
  for (int64_t i = 0; i < rows; i++) { int e = sels[i]; users[ebase[e] + fill[e]++] = (int32_t)i; }
  int8_t* xq = (int8_t*)malloc((size_t)n * d); float* xd = (float*)malloc(sizeof(float) * n * (d / QK_K));
  int32_t* xbs = (int32_t*)malloc(sizeof(int32_t) * n * (d / 16));
  for (int t = 0; t < n; t++)
    orc_quantize_q8k(norms + (int64_t)t * d, d, xq + (int64_t)t * d, xd + (int64_t)t * (d / QK_K), xbs + (int64_t)t * (d / 16));
  float* mid = (float*)malloc(sizeof(float) * rows * ff);
  int8_t* mq = (int8_t*)malloc((size_t)rows * ff); float* md = (float*)malloc(sizeof(float) * rows * (ff / QK_K));
  int32_t* mbs = (int32_t*)malloc(sizeof(int32_t) * rows * (ff / 16));
  float* downs = (float*)malloc(sizeof(float) * rows * d);
  orc_chunk_args a = { gate, up, down, d, ff, nu, n, clamp, nexp, experts, ubase, users, ws, xq, xd, mid, mq, md, mbs, downs };
  orc_pool_run(nthreads, orc_chunk_gu_job, &a);
  for (int64_t i = 0; i < rows; i++)
    orc_quantize_q8k(mid + i * ff, ff, mq + i * ff, md + i * (ff / QK_K), mbs + i * (ff / 16));
  orc_pool_run(nthreads, orc_chunk_down_job, &a);
  for (int t = 0; t < n; t++)
    for (int r = 0; r < d; r++) {
      float s = 0.0f;
      for (int slot = 0; slot < nu; slot++) s = s + downs[((int64_t)t * nu + slot) * d + r];
      if (shared) s = s + shared[(int64_t)t * d + r];
      out[(int64_t)t * d + r] = s;
    }
  if (sel_out) memcpy(sel_out, sels, sizeof(int32_t) * rows);
  if (w_out) memcpy(w_out, ws, sizeof(float) * rows);
  if (counts_out) memcpy(counts_out, counts, sizeof(int32_t) * ne);
  free(sels); free(ws); free(counts); free(experts); free(ubase); free(ebase); free(users); free(fill);
  free(xq); free(xd); free(xbs); free(mid); free(mq); free(md); free(mbs); free(downs);
}

/* ---- the dense decoder, one token: src/model.lisp:205-462 (forward-1 and what it calls) ------------------ */
/* rope-table (model.lisp:218-231): theta advanced by repeated single-float multiplication from pos;
   theta-scale = expt(base, -2/hd), which SBCL evaluates through double pow and rounds to single; cos and sin of
   a single float likewise through double. */
void orc_rope_table(int head_dim, int pos, float base, float* cosv, float* sinv) {
  const int half = head_dim / 2;
  const float e = -2.0f / (float)head_dim;
  const float theta_scale = (float)pow((double)base, (double)e);
  float theta = (float)pos;
  for (int i = 0; i < half; i++) {
    cosv[i] = (float)cos((double)theta); sinv[i] = (float)sin((double)theta);
    theta = theta * theta_scale;
  }
}
/* rope-head! (model.lisp:233-244): pairs (i, i + half) when neox, else (2i, 2i + 1) */
void orc_rope_head(float* x, int head_dim, int neox, const float* cosv, const float* sinv) {
  const int half = head_dim / 2;
  for (int i = 0; i < half; i++) {
    const int a = neox ? i : 2 * i, b = neox ? i + half : 2 * i + 1;
    const float x0 = x[a], x1 = x[b], c = cosv[i], s = sinv[i];
    volatile float p0 = x0 * c, p1 = x1 * s, p2 = x0 * s, p3 = x1 * c;
    x[a] = p0 - p1; x[b] = p2 + p3;
  }
}
/* attend-head! (model.lisp:298-334): scores in f32-dot16's order times 1/sqrt(hd); softmax with exp in single
   (through double, as SBCL evaluates it), the sum in double, scaled by single(1/sum); then out += score * V row,
   position after position.  kc, vc: the layer's caches, kvd floats a position; ko: the KV head's offset. */
void orc_attend_head(const float* kc, const float* vc, const float* q, float* out, int n, int hd, int kvd, int ko, float* scores) {
  const float scale = 1.0f / sqrtf((float)hd);
  float mx = -FLT_MAX;
  for (int p = 0; p < n; p++) {
    const float s = orc_f32_dot16(kc + (int64_t)p * kvd + ko, q, hd) * scale;
    scores[p] = s;
    if (s > mx) mx = s;
  }
  double sum = 0.0;
  for (int p = 0; p < n; p++) { const float e = sb_exp(scores[p] - mx); scores[p] = e; sum += (double)e; }
  const float inv = (float)(1.0 / sum);
  for (int p = 0; p < n; p++) scores[p] = scores[p] * inv;
  for (int i = 0; i < hd; i++) out[i] = 0.0f;
  for (int p = 0; p < n; p++) {
    const float w = scores[p]; const float* v = vc + (int64_t)p * kvd + ko;
    for (int i = 0; i < hd; i++) { volatile float t = w * v[i]; out[i] = out[i] + t; }
  }
}

typedef struct {
  const uint8_t *wq, *wk, *wv, *wo, *wgate, *wup, *wdown;
  int tq, tk, tv, to, tg, tu, td;                       /* GGUF type codes */
  const float *attn_norm, *ffn_norm, *q_norm, *k_norm;  /* q_norm, k_norm: null for a model without head norms */
  const float *bq, *bk, *bv;                            /* or null */
} orc_layer;
typedef struct {
  int d, ffn, nh, nkv, hd, nl, vocab, neox;
  float eps, rope_base;
  const uint8_t *embd, *output; int embd_type, output_type;
  const float* output_norm;
  const orc_layer* layers;
} orc_model;

static void orc_qmv(int type, const uint8_t* w, int64_t rows, int64_t cols, const float* x, const float* bias, float* out, int nt) {
  orc_matmul(type, w, rows, cols, x, 1, 1, out, nt);   /* quantize-act! (Q8_0 scales through f16) + qmatvec! */
  if (bias) for (int64_t r = 0; r < rows; r++) out[r] = out[r] + bias[r];
}
typedef struct { const orc_model* m; const float *kc, *vc, *q; float* att; int n; float* scores; } orc_att_args;
static void orc_att_job(void* p, int index, int count) {
  orc_att_args* a = (orc_att_args*)p;
  const orc_model* m = a->m;
  int64_t s, e; share(m->nh, index, count, &s, &e);
  const int group = m->nh / m->nkv, kvd = m->nkv * m->hd;
  for (int64_t h = s; h < e; h++)
    orc_attend_head(a->kc, a->vc, a->q + h * m->hd, a->att + h * m->hd, a->n, m->hd, kvd, (int)(h / group) * m->hd, a->scores + h * a->n);
}
/* forward-1 (model.lisp:396-462) at position pos; kcache/vcache: nl x nctx x kvd floats.  logits may be null. */
void orc_forward(const orc_model* m, int token, int pos, float* kcache, float* vcache, int nctx, float* logits, float* x_out, int nthreads) {
  const int d = m->d, hd = m->hd, kvd = m->nkv * m->hd, qd = m->nh * m->hd;
  float* x = (float*)malloc(sizeof(float) * d); float* h = (float*)malloc(sizeof(float) * d);
  float* q = (float*)malloc(sizeof(float) * qd); float* k = (float*)malloc(sizeof(float) * kvd); float* v = (float*)malloc(sizeof(float) * kvd);
  float* att = (float*)malloc(sizeof(float) * qd);
  float* fa = (float*)malloc(sizeof(float) * m->ffn); float* fb = (float*)malloc(sizeof(float) * m->ffn);
  float* cosv = (float*)malloc(sizeof(float) * hd); float* sinv = cosv + hd / 2;
  float* scores = (float*)malloc(sizeof(float) * (size_t)m->nh * (pos + 1));
  const int64_t erb = m->d / (m->embd_type == ORC_Q8_0 ? 32 : QK_K) * orc_block_bytes(m->embd_type);
  orc_dequant_row(m->embd_type, m->embd + (int64_t)token * erb, d, x);
  orc_rope_table(hd, pos, m->rope_base, cosv, sinv);
  for (int li = 0; li < m->nl; li++) {
    const orc_layer* l = &m->layers[li];
    float* kc = kcache + (int64_t)li * nctx * kvd; float* vc = vcache + (int64_t)li * nctx * kvd;
    orc_rmsnorm(x, l->attn_norm, h, m->eps, d);
    orc_qmv(l->tq, l->wq, qd, d, h, l->bq, q, nthreads);
    orc_qmv(l->tk, l->wk, kvd, d, h, l->bk, k, nthreads);
    orc_qmv(l->tv, l->wv, kvd, d, h, l->bv, v, nthreads);
    for (int u = 0; u < m->nh; u++) { if (l->q_norm) orc_rmsnorm(q + u * hd, l->q_norm, q + u * hd, m->eps, hd); orc_rope_head(q + u * hd, hd, m->neox, cosv, sinv); }
    for (int u = 0; u < m->nkv; u++) { if (l->k_norm) orc_rmsnorm(k + u * hd, l->k_norm, k + u * hd, m->eps, hd); orc_rope_head(k + u * hd, hd, m->neox, cosv, sinv); }
    memcpy(kc + (int64_t)pos * kvd, k, sizeof(float) * kvd);
    memcpy(vc + (int64_t)pos * kvd, v, sizeof(float) * kvd);
    orc_att_args aa = { m, kc, vc, q, att, pos + 1, scores };
    orc_pool_run(nthreads, orc_att_job, &aa);
    orc_qmv(l->to, l->wo, d, qd, att, NULL, h, nthreads);
    for (int i = 0; i < d; i++) x[i] = x[i] + h[i];
    orc_rmsnorm(x, l->ffn_norm, h, m->eps, d);
    orc_qmv(l->tg, l->wgate, m->ffn, d, h, NULL, fa, nthreads);
    orc_qmv(l->tu, l->wup, m->ffn, d, h, NULL, fb, nthreads);
    for (int i = 0; i < m->ffn; i++) fa[i] = orc_swiglu(fa[i], fb[i]);
    orc_qmv(l->td, l->wdown, d, m->ffn, fa, NULL, h, nthreads);
    for (int i = 0; i < d; i++) x[i] = x[i] + h[i];
  }
  if (x_out) memcpy(x_out, x, sizeof(float) * d);
  if (logits) {
    orc_rmsnorm(x, m->output_norm, h, m->eps, d);
    orc_qmv(m->output_type, m->output, m->vocab, d, h, NULL, logits, nthreads);
  }
  free(x); free(h); free(q); free(k); free(v); free(att); free(fa); free(fb); free(cosv); free(scores);
}
