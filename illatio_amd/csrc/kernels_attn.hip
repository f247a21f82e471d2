// What a dense decoder layer needs between its quantized products, for the harness that runs
// the whole forward pass (the reference's cuda-forward-n, src/cuda-dense.lisp:380-432): the Q/K
// head norms, RoPE and the KV caches' update (qk_rope, src/cuda/dense.cu:318-362), attention, and
// swiglu! on rows.  The floats follow the reference's CPU path (src/model.lisp:205-334, 364-378)
// operation for operation and sum for sum, so a token's logits have the CPU path's bits; speed is
// not the point of these kernels (the reference's CUDA attention splits the keys and lets the
// partial sums meet in its own order, dense.cu:364-373).
#include "ilt_device.h"
#include <atomic>
#include <mutex>
#include "ilt_kernels.h"
#include <stdlib.h>

namespace {

// What one lane of a wave stored in LDS, for the other lanes of that wave: the hardware keeps a wave's LDS
// accesses in program order; this keeps the compiler from moving them across.
__device__ __forceinline__ void wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// The softmax's 1/sum as the CPU rounds it to a single, from a sum of n exps added in another order than the CPU's
// (within sum * (n + 8) * 2^-51 of the CPU's): one division, then whether every sum that near has the same single for
// its reciprocal -- the reciprocals of all of them lie within inv * (1 -+ d), d a little more than twice that slack
// plus the division's own rounding, and rounding to single keeps their order.  False: the caller adds the exps again
// in the CPU's order.
__device__ __forceinline__ bool recip_settled(double sum, int n, float* inv) {
  const double r = 1.0 / sum, d = (double)(n + 8) * 0x1p-50 + 0x1p-50;
  *inv = (float)r;
  return (float)(r - r * d) == (float)(r + r * d);
}

// One head by one wave: x (hd floats) into xs (LDS): rmsnorm! of the head when its weights are given
// (model.lisp:205-216: the squares, rounded to floats, added in double one after another), then rope-head!
// from the position's table cs (cos, then sin, rd/2 each).  Only this wave touches xs and sd.  The lanes add
// the squares in parallel; where the order of the adds could show in the single the mean is rounded to, one
// lane adds them again one after another, as the CPU does.
// In two steps, so that a kernel can ask for the head, its norm weights and the table's row before the loads it
// makes for other things, and wait for these alone: lane i's share of the three (NT floats of the head: hd <= 64 NT).
template <int NT> struct RopeIn { float x[NT], w[NT], c[(NT + 1) / 2], s[(NT + 1) / 2]; };
template <int NT>
__device__ __forceinline__ void rope_head_load(RopeIn<NT>& r, const float* __restrict__ x, const float* __restrict__ nw, const float* __restrict__ cs,
                                               int hd, int rd, int i) {
  const int half = rd >> 1;
#pragma unroll
  for (int t = 0; t < NT; t++) {
    const int j = min(i + 64 * t, hd - 1);
    r.x[t] = x[j];
    r.w[t] = nw ? nw[j] : 0.0f;
  }
#pragma unroll
  for (int t = 0; t < (NT + 1) / 2; t++) {
    const int p = min(i + 64 * t, max(half - 1, 0));
    r.c[t] = half > 0 ? cs[p] : 0.0f; r.s[t] = half > 0 ? cs[half + p] : 0.0f;
  }
}
template <int NT>
__device__ __forceinline__ void rope_head_turn(const RopeIn<NT>& r, bool norm, float* xs, double* sd, int hd, int rd, float eps, int neox, int i) {
  const int half = rd >> 1;
#pragma unroll
  for (int t = 0; t < NT; t++) if (i + 64 * t < hd) xs[i + 64 * t] = r.x[t];
  wave_lds_sync();
  if (norm) {
    double s = 0.0;
#pragma unroll
    for (int t = 0; t < NT; t++) if (i + 64 * t < hd) { const float sq = r.x[t] * r.x[t]; s += (double)sq; }
    s = wave_sum_double(s);
    const double slack = s * ((double)(hd + 8) * 0x1p-51);
    if ((float)((s - slack) / (double)hd + (double)eps) != (float)((s + slack) / (double)hd + (double)eps)) {      // the same in every lane
      if (i == 0) {
        double s2 = 0.0;
        for (int j = 0; j < hd; j++) { const float sq = xs[j] * xs[j]; s2 += (double)sq; }
        *sd = s2;
      }
      wave_lds_sync();
      s = *sd;
    }
    const float scale = 1.0f / sqrtf((float)(s / (double)hd + (double)eps));
#pragma unroll
    for (int t = 0; t < NT; t++) if (i + 64 * t < hd) xs[i + 64 * t] = (r.x[t] * scale) * r.w[t];
    wave_lds_sync();
  }
#pragma unroll
  for (int t = 0; t < (NT + 1) / 2; t++) {
    const int p = i + 64 * t;
    if (p < half) {
      const int a = neox ? p : 2 * p, b = neox ? p + half : 2 * p + 1;
      const float x0 = xs[a], x1 = xs[b], c = r.c[t], sn = r.s[t];
      xs[a] = x0 * c - x1 * sn;                    // (no contraction: each product rounds on its own)
      xs[b] = x0 * sn + x1 * c;
    }
  }
  wave_lds_sync();
}
__device__ __forceinline__ void rope_head_wave(const float* __restrict__ x, const float* __restrict__ nw, const float* __restrict__ cs,
                                               float* xs, double* sd, int hd, int rd, float eps, int neox, int i) {
  RopeIn<8> r;                                     // hd <= 512
  rope_head_load(r, x, nw, cs, hd, rd, i);
  rope_head_turn(r, nw != nullptr, xs, sd, hd, rd, eps, neox, i);
}

// qk_rope: a workgroup (one wave) a head of a token; K and V into the caches at pos0 + t.
__global__ __launch_bounds__(64) void qk_rope_kernel(float* __restrict__ q, float* __restrict__ k, const float* __restrict__ v,
                                                     const float* __restrict__ qn, const float* __restrict__ kn,
                                                     const float* __restrict__ rope, float* __restrict__ kc, float* __restrict__ vc,
                                                     int nh, int nkv, int hd, int rd, int pos0, float eps, int neox) {
  __shared__ float xs[512];
  __shared__ double sc;
  const int head = blockIdx.x, t = blockIdx.y, i = threadIdx.x;
  const int pos = pos0 + t;
  const int qd = nh * hd, kvd = nkv * hd;
  const bool isq = head < nh;
  float* x = isq ? q + (long long)t * qd + head * hd : k + (long long)t * kvd + (head - nh) * hd;
  rope_head_wave(x, isq ? qn : kn, rope + (long long)pos * rd, xs, &sc, hd, rd, eps, neox, i);
  for (int j = i; j < hd; j += 64) x[j] = xs[j];
  if (!isq) {
    const int kh = head - nh;
    const long long o = (long long)pos * kvd + kh * hd;
    for (int j = i; j < hd; j += 64) {
      kc[o + j] = xs[j];
      vc[o + j] = v[(long long)t * kvd + kh * hd + j];
    }
  }
}

// attend-head! (model.lisp:298-334) for query head blockIdx.x of token blockIdx.y, which sees positions
// 0 .. pos0 + t.  Scores: F32-DOT16 (tensor.lisp:370-378; 16 lanes a position, lane l the partial sum l)
// times 1/sqrt(hd).  Softmax: exp of a single through double; the sum of the exps in double -- added in
// parallel here and, where that order could change the single 1/sum is rounded to, once more one after
// another as the CPU adds them.  Then out += score * V row, position after position: the adds of a column are a
// chain, so a column is one thread's; the value rows come through LDS in tiles of 64 positions that all sixteen
// waves load (two tiles in flight), so the chain never waits for memory.
constexpr int kAttnThreads = 1024, kAttnTile = 64;
__global__ __launch_bounds__(kAttnThreads) void attn_rows_kernel(const float* __restrict__ q, const float* __restrict__ kc,
                                                                 const float* __restrict__ vc, float* __restrict__ out, int nh, int nkv, int hd,
                                                                 int pos0, float scale, int smax) {
  extern __shared__ __align__(16) float dyn[];
  float* scores = dyn;                             // smax floats (a multiple of 4)
  float* vt = dyn + smax;                          // two tiles of kAttnTile x hd floats
  __shared__ float redf[16];
  __shared__ double redd[16];
  const int h = blockIdx.x, t = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int npos = pos0 + t + 1;
  const int group = nh / nkv, kvd = nkv * hd, ko = (h / group) * hd;
  const float* qh = q + ((long long)t * nh + h) * hd;
  const int l = tid & 15, pg = tid >> 4;           // 64 positions at a time
  const int nj = hd >> 4;                          // terms a partial sum (hd <= 256: at most 16)
  float qv[16];
#pragma unroll
  for (int j = 0; j < 16; j++) qv[j] = j < nj ? qh[l + 16 * j] : 0.0f;
  float mx = -3.402823466e38f;
  for (int p0 = 0; p0 < npos; p0 += 128) {         // two passes' loads before either is used
    float kv[2][16];
#pragma unroll
    for (int u = 0; u < 2; u++) {
      const float* kr = kc + (long long)min(p0 + 64 * u + pg, npos - 1) * kvd + ko;
#pragma unroll
      for (int j = 0; j < 16; j++) kv[u][j] = j < nj ? kr[l + 16 * j] : 0.0f;
    }
#pragma unroll
    for (int u = 0; u < 2; u++) {
      const int p = p0 + 64 * u + pg;
      float s = 0.0f;
#pragma unroll
      for (int j = 0; j < 16; j++) if (j < nj) s = s + kv[u][j] * qv[j];
      s = s + ilt_dppf<ILT_DPP_SHL(4)>(s);
      s = s + ilt_dppf<ILT_DPP_SHL(8)>(s);
      s = s + ilt_dppf<ILT_DPP_SHL(1)>(s);
      s = s + ilt_dppf<ILT_DPP_SHL(2)>(s);
      if (l == 0 && p < npos) { const float sv = s * scale; scores[p] = sv; mx = fmaxf(mx, sv); }
    }
  }
  mx = wave_max_float(mx);
  if (lane == 0) redf[wave] = mx;
  __syncthreads();
  mx = redf[0];
#pragma unroll
  for (int w = 1; w < 16; w++) mx = fmaxf(mx, redf[w]);
  double part = 0.0;
  for (int p = tid; p < npos; p += kAttnThreads) { const float e = ilt_expf_via_double(scores[p] - mx); scores[p] = e; part += (double)e; }
  part = wave_sum_double(part);
  if (lane == 0) redd[wave] = part;
  __syncthreads();
  double sum = 0.0;
#pragma unroll
  for (int w = 0; w < 16; w++) sum += redd[w];
  float inv;
  if (!recip_settled(sum, npos, &inv)) {           // the same in every thread
    __syncthreads();
    if (tid == 0) { double s2 = 0.0; for (int p = 0; p < npos; p++) s2 += (double)scores[p]; redd[0] = s2; }
    __syncthreads();
    inv = (float)(1.0 / redd[0]);
  }
  __syncthreads();
  for (int p = tid; p < npos; p += kAttnThreads) scores[p] = scores[p] * inv;
  // the values: tile i of 64 positions into buffer i & 1, loaded a tile ahead of the adds
  const int ntile = (npos + kAttnTile - 1) / kAttnTile;
  const int per = kAttnTile * hd / 4;              // float4 pieces a tile
  auto load_tile = [&](int ti) {
    float* dst = vt + (ti & 1) * kAttnTile * hd;
    for (int i = tid; i < per; i += kAttnThreads) {
      const int pp = i / (hd / 4), c4 = i - pp * (hd / 4);
      const int p = min(ti * kAttnTile + pp, npos - 1);
      *(float4*)(dst + pp * hd + 4 * c4) = *(const float4*)(vc + (long long)p * kvd + ko + 4 * c4);
    }
  };
  load_tile(0);
  float o = 0.0f;
  for (int ti = 0; ti < ntile; ti++) {
    __syncthreads();                               // tile ti is in LDS (and the scores are scaled); buffer (ti + 1) & 1 is free
    if (ti + 1 < ntile) load_tile(ti + 1);
    if (tid < hd) {
      const float* col = vt + (ti & 1) * kAttnTile * hd + tid;
      const int np = min(kAttnTile, npos - ti * kAttnTile);
      const float* sc = scores + ti * kAttnTile;
      int pp = 0;
      for (; pp + 8 <= np; pp += 8) {
        float pr[8];
#pragma unroll
        for (int u = 0; u < 8; u++) pr[u] = sc[pp + u] * col[(pp + u) * hd];
#pragma unroll
        for (int u = 0; u < 8; u++) o = o + pr[u];
      }
      for (; pp < np; pp++) o = o + sc[pp] * col[pp * hd];
    }
  }
  if (tid < hd) out[((long long)t * nh + h) * hd + tid] = o;
}

// The same attention as two launches, for contexts whose scores and value slice fit LDS (2048 positions): the
// scores of all positions at once over many workgroups (nothing in them depends on anything else), then the
// softmax and the ordered sums, a workgroup taking a query head's 16-column slice of the values for a group of
// TG tokens: the whole slice is asked for at once (one trip to memory), and 16 threads a token then run the
// chains from LDS.  A group's tokens share the keys (registers) and the value slice (LDS), so a prompt's chunk
// reads them once for 16 tokens.  The numbers are attn_rows_kernel's: the same operations in the same order.
// raw[(t*nh + h)*spitch + p] = F32-DOT16(K[p], q) * scale
// NJ: hd / 16 as a constant (heads of 64 and of 128), or 0: any head up to 256, the count read at run time
template <int TG, int NJ = 0>
__global__ __launch_bounds__(1024) void attn_scores_kernel(const float* __restrict__ q, const float* __restrict__ kc, float* __restrict__ raw,
                                                           int nh, int nkv, int hd, int pos0, int ntok, float scale, int spitch) {
  constexpr int NJM = NJ ? NJ : 16;
  __shared__ float qs[TG > 1 ? TG * 256 : 1];
  const int h = blockIdx.x, t0 = blockIdx.z * TG, tid = threadIdx.x;
  const int tn = min(TG, ntok - t0), nposmax = pos0 + t0 + tn, pbase = blockIdx.y * 256;
  if (pbase >= nposmax) return;                    // the same in every thread
  const int group = nh / nkv, kvd = nkv * hd, ko = (h / group) * hd;
  const int l = tid & 15, pg = tid >> 4, nj = NJ ? NJ : hd >> 4;
  float kv[4][NJM];
#pragma unroll
  for (int u = 0; u < 4; u++) {
    const float* kr = kc + (long long)min(pbase + 64 * u + pg, nposmax - 1) * kvd + ko;
#pragma unroll
    for (int j = 0; j < NJM; j++) kv[u][j] = (NJ || j < nj) ? kr[l + 16 * j] : 0.0f;
  }
  if (TG > 1) {
    for (int i = tid; i < tn * hd; i += 1024) { const int tt = i / hd, c = i - tt * hd; qs[tt * 256 + c] = q[((long long)(t0 + tt) * nh + h) * hd + c]; }
    __syncthreads();
  }
  for (int tt = 0; tt < tn; tt++) {
    const int npos = pos0 + t0 + tt + 1;
    if (pbase >= npos) continue;
    const float* qh = q + ((long long)(t0 + tt) * nh + h) * hd;
    float qv[NJM];
#pragma unroll
    for (int j = 0; j < NJM; j++) qv[j] = (NJ || j < nj) ? (TG > 1 ? qs[tt * 256 + l + 16 * j] : qh[l + 16 * j]) : 0.0f;
#pragma unroll
    for (int u = 0; u < 4; u++) {
      const int p = pbase + 64 * u + pg;
      if (pbase + 64 * u >= npos) continue;        // none of the pass's 64 positions is the token's to see (the same in every thread)
      float sacc = 0.0f;
#pragma unroll
      for (int j = 0; j < NJM; j++) if (NJ || j < nj) sacc = sacc + kv[u][j] * qv[j];
      sacc = sacc + ilt_dppf<ILT_DPP_SHL(4)>(sacc);
      sacc = sacc + ilt_dppf<ILT_DPP_SHL(8)>(sacc);
      sacc = sacc + ilt_dppf<ILT_DPP_SHL(1)>(sacc);
      sacc = sacc + ilt_dppf<ILT_DPP_SHL(2)>(sacc);
      if (l == 0 && p < npos) raw[((long long)(t0 + tt) * nh + h) * spitch + p] = sacc * scale;
    }
  }
}

// A prompt chunk's scores, sixteen of them a thread: a workgroup of 256 threads takes 64 tokens x 64 positions of a
// query head, thread (tq, pq) the tokens tq + 16a and the positions pq + 16b.  F32-DOT16 keeps sixteen running sums,
// sum l over the columns l, l + 16, ..., and adds them as ((s_l + s_l+4) + (s_l+8 + s_l+12)) = X_l for l = 0..3, then
// (X_0 + X_1) + (X_2 + X_3).  The kernel above gives a score to sixteen lanes, a running sum each, and every lane
// then goes through the four adds of the tree and the scaling for the sake of lane 0; here one thread keeps a score's
// four sums l = e, e+4, e+8, e+12 for e = 0, 1, 2, 3 in turn, so that nothing is added that the score does not need, and
// a 16-byte read of a token's or a position's row serves four scores.  For that the rows lie in LDS with every sixteen
// columns transposed as 4 x 4 (place 4e + m holds column 4m + e): a thread that brings a row's sixteen columns in
// stores them as four pieces of 16 bytes.  Row pitch HD + 4 floats: sixteen lanes' 16-byte reads of sixteen
// consecutive rows fall on different banks.  The numbers are those of the kernel above.
template <int NJ>      // HD / 16
__global__ __launch_bounds__(256, 2) void attn_scores_quad_kernel(const float* __restrict__ q, const float* __restrict__ kc, float* __restrict__ raw,
                                                               int nh, int nkv, int pos0, int ntok, float scale, int spitch) {
  constexpr int HD = 16 * NJ, RP = HD + 4;
  extern __shared__ __align__(16) float dyn[];     // 2 * 64 * RP floats
  float* const qs = dyn;
  float* const ks = dyn + 64 * RP;
  const int h = blockIdx.x, p0 = blockIdx.y * 64, t0 = blockIdx.z * 64, tid = threadIdx.x;
  const int tn = min(64, ntok - t0), nposmax = pos0 + t0 + tn;
  if (p0 >= nposmax) return;                       // the same in every thread
  const int group = nh / nkv, kvd = nkv * HD, ko = (h / group) * HD;
  // rows 0..63: the tokens' q, 64..127: the positions' keys; 128 * NJ groups of sixteen columns, NJ / 2 a thread
#pragma unroll
  for (int u = 0; u < NJ / 2; u++) {
    const int g = tid + 256 * u, row = g / NJ, j = g - row * NJ;
    const float* src = row < 64 ? q + ((long long)(t0 + min(row, tn - 1)) * nh + h) * HD + 16 * j
                                : kc + (long long)min(p0 + row - 64, nposmax - 1) * kvd + ko + 16 * j;
    const float4 m0 = *(const float4*)src, m1 = *(const float4*)(src + 4), m2 = *(const float4*)(src + 8), m3 = *(const float4*)(src + 12);
    float* dst = (row < 64 ? qs + row * RP : ks + (row - 64) * RP) + 16 * j;
    *(float4*)dst = make_float4(m0.x, m1.x, m2.x, m3.x);
    *(float4*)(dst + 4) = make_float4(m0.y, m1.y, m2.y, m3.y);
    *(float4*)(dst + 8) = make_float4(m0.z, m1.z, m2.z, m3.z);
    *(float4*)(dst + 12) = make_float4(m0.w, m1.w, m2.w, m3.w);
  }
  __syncthreads();
  const int tq = tid >> 4, pq = tid & 15;
  // none of the thread's positions is any of its tokens' to see (its first position, its last token)
  if (p0 + pq >= pos0 + t0 + tq + 48 + 1) return;
  const float* Q = qs + tq * RP;
  const float* K = ks + pq * RP;
  float y[4][4], z[4][4];
  auto read_step = [&](float4 (&qr)[4], float4 (&kr)[4], const float* Qe, const float* Ke) {
#pragma unroll
    for (int a = 0; a < 4; a++) qr[a] = *(const float4*)(Qe + 16 * a * RP);
#pragma unroll
    for (int b = 0; b < 4; b++) kr[b] = *(const float4*)(Ke + 16 * b * RP);
  };
  // sums e, e+4, e+8, e+12 of the sixteen scores: two steps of sixteen columns a turn of the loop, each step's reads sent
  // off before the step before it is multiplied (left to itself the compiler reads every step's rows first and spills)
  auto sums = [&](auto Ec) {
    constexpr int e = decltype(Ec)::value;
    float4 acc[4][4], qa[4], ka[4], qb[4], kb[4];
#pragma unroll
    for (int a = 0; a < 4; a++)
#pragma unroll
      for (int b = 0; b < 4; b++) acc[a][b] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    auto mac = [&](const float4 (&qr)[4], const float4 (&kr)[4]) {
#pragma unroll
      for (int a = 0; a < 4; a++)
#pragma unroll
        for (int b = 0; b < 4; b++) {
          acc[a][b].x = acc[a][b].x + kr[b].x * qr[a].x;
          acc[a][b].y = acc[a][b].y + kr[b].y * qr[a].y;
          acc[a][b].z = acc[a][b].z + kr[b].z * qr[a].z;
          acc[a][b].w = acc[a][b].w + kr[b].w * qr[a].w;
        }
    };
    const float* Qe = Q + 4 * e;
    const float* Ke = K + 4 * e;
    read_step(qa, ka, Qe, Ke);
#pragma unroll 1
    for (int j = 0; j < NJ; j += 2) {
      read_step(qb, kb, Qe + 16 * (j + 1), Ke + 16 * (j + 1));
      mac(qa, ka);
      asm volatile("" ::: "memory");
      const int jn = min(j + 2, NJ - 2);           // (after the last step: rows read again, for nobody)
      read_step(qa, ka, Qe + 16 * jn, Ke + 16 * jn);
      mac(qb, kb);
      asm volatile("" ::: "memory");
    }
#pragma unroll
    for (int a = 0; a < 4; a++)
#pragma unroll
      for (int b = 0; b < 4; b++) {
        float x = (acc[a][b].x + acc[a][b].y) + (acc[a][b].z + acc[a][b].w);      // X_e
        asm volatile("" : "+v"(x));                // (added here, not where the score is stored: the four sums are not kept till then)
        if (e == 0) y[a][b] = x;
        if (e == 1) y[a][b] = y[a][b] + x;
        if (e == 2) z[a][b] = x;
        if (e == 3) z[a][b] = z[a][b] + x;
      }
    __builtin_amdgcn_sched_barrier(0);             // (one set of sums in registers at a time)
  };
  sums(std::integral_constant<int, 0>{});
  sums(std::integral_constant<int, 1>{});
  sums(std::integral_constant<int, 2>{});
  sums(std::integral_constant<int, 3>{});
#pragma unroll
  for (int a = 0; a < 4; a++) {
    const int tt = tq + 16 * a, npos = pos0 + t0 + tt + 1;
    if (tt < tn) {
      float* dst = raw + ((long long)(t0 + tt) * nh + h) * spitch;
#pragma unroll
      for (int b = 0; b < 4; b++) {
        const int p = p0 + pq + 16 * b;
        if (p < npos) dst[p] = (y[a][b] + z[a][b]) * scale;
      }
    }
  }
}

// One token's qk_rope and scores in one launch: every workgroup of a query head norms and turns that head
// itself (wave 0; a sixteenth of a microsecond of arithmetic against a launch), the workgroup whose 256
// positions hold the token's own does the same for its KV head's key (wave 1) and takes that key from LDS,
// and the group's first query head there writes the key and the value into the caches, for the launch with
// the values.  q and k are left as they came.
template <int NJ>      // hd / 16 as a constant, or 0: read at run time (heads up to 256)
__global__ __launch_bounds__(1024) void attn_step_scores_kernel(const float* __restrict__ q, const float* __restrict__ k, const float* __restrict__ v,
                                                                const float* __restrict__ qn, const float* __restrict__ kn,
                                                                const float* __restrict__ rope, float* __restrict__ kc, float* __restrict__ vc,
                                                                float* __restrict__ raw, int nh, int nkv, int hd, int rd, int pos, float eps,
                                                                int neox, float scale, int spitch) {
  __shared__ float qsh[256], ksh[256];
  __shared__ double scs[2];
  const int h = blockIdx.x, tid = threadIdx.x, npos = pos + 1, pbase = blockIdx.y * 256;
  if (pbase >= npos) return;
  const int group = nh / nkv, kvd = nkv * hd, kh = h / group, ko = kh * hd;
  constexpr int NJM = NJ ? NJ : 16;
  const int l = tid & 15, pg = tid >> 4, nj = NJ ? NJ : hd >> 4, wave = tid >> 6;
  const bool own = pos < pbase + 256;              // this workgroup's positions hold the token's own
  // the head's own loads first (waves 0 and 1), the keys' after: the norms and the turn wait for the first alone
  const float* cs = rope + (long long)pos * rd;
  RopeIn<4> rin;
  const bool turns = wave == 0 || (wave == 1 && own);
  if (turns) rope_head_load(rin, wave == 0 ? q + h * hd : k + ko, wave == 0 ? qn : kn, cs, hd, rd, tid & 63);
  float kv[4][NJM];
#pragma unroll
  for (int u = 0; u < 4; u++) {
    const float* kr = kc + (long long)min(pbase + 64 * u + pg, max(pos - 1, 0)) * kvd + ko;      // rows before the token's own
#pragma unroll
    for (int j = 0; j < NJM; j++) kv[u][j] = (NJ || j < nj) ? kr[l + 16 * j] : 0.0f;
  }
  if (turns) rope_head_turn(rin, (wave == 0 ? qn : kn) != nullptr, wave == 0 ? qsh : ksh, &scs[wave], hd, rd, eps, neox, tid & 63);
  __syncthreads();
  if (own && h == kh * group && tid < hd) {
    kc[(long long)pos * kvd + ko + tid] = ksh[tid];
    vc[(long long)pos * kvd + ko + tid] = v[ko + tid];
  }
  float qv[NJM];
#pragma unroll
  for (int j = 0; j < NJM; j++) qv[j] = (NJ || j < nj) ? qsh[l + 16 * j] : 0.0f;
#pragma unroll
  for (int u = 0; u < 4; u++) {
    const int p = pbase + 64 * u + pg;
    if (p == pos) {
#pragma unroll
      for (int j = 0; j < NJM; j++) kv[u][j] = (NJ || j < nj) ? ksh[l + 16 * j] : 0.0f;
    }
    float sacc = 0.0f;
#pragma unroll
    for (int j = 0; j < NJM; j++) if (NJ || j < nj) sacc = sacc + kv[u][j] * qv[j];
    sacc = sacc + ilt_dppf<ILT_DPP_SHL(4)>(sacc);
    sacc = sacc + ilt_dppf<ILT_DPP_SHL(8)>(sacc);
    sacc = sacc + ilt_dppf<ILT_DPP_SHL(1)>(sacc);
    sacc = sacc + ilt_dppf<ILT_DPP_SHL(2)>(sacc);
    if (l == 0 && p < npos) raw[(long long)h * spitch + p] = sacc * scale;
  }
}

// Eight 16-byte LDS reads (32 floats from P on) into A##0 .. A##7 that the compiler does not wait for, and the wait
// that hands those registers over once at most LEFT LDS reads asked for after them are still on their way (LDS
// answers in order).  Between a read and its wait the program may ask LDS for nothing else but more of these reads.
#define ILT_LDS_READ32_AHEAD(A, P)                                                                                                          \
  asm volatile("ds_read_b128 %0, %8\n\tds_read_b128 %1, %8 offset:16\n\tds_read_b128 %2, %8 offset:32\n\tds_read_b128 %3, %8 offset:48\n\t" \
               "ds_read_b128 %4, %8 offset:64\n\tds_read_b128 %5, %8 offset:80\n\tds_read_b128 %6, %8 offset:96\n\tds_read_b128 %7, %8 offset:112" \
               : "=&v"(A##0), "=&v"(A##1), "=&v"(A##2), "=&v"(A##3), "=&v"(A##4), "=&v"(A##5), "=&v"(A##6), "=&v"(A##7)                   \
               : "v"((u32)(uintptr_t)(ILT_LDS const void*)(P)) : "memory")
#define ILT_LDS_READ32_WAIT(A, LEFT)                                                                                                        \
  asm volatile("s_waitcnt lgkmcnt(" #LEFT ")" : "+v"(A##0), "+v"(A##1), "+v"(A##2), "+v"(A##3), "+v"(A##4), "+v"(A##5), "+v"(A##6), "+v"(A##7) :: "memory")
#define ILT_CHAIN_ADD32(O, A)                                                                                                               \
  do {                                                                                                                                      \
    O = O + (A##0).x; O = O + (A##0).y; O = O + (A##0).z; O = O + (A##0).w; O = O + (A##1).x; O = O + (A##1).y; O = O + (A##1).z; O = O + (A##1).w;          \
    O = O + (A##2).x; O = O + (A##2).y; O = O + (A##2).z; O = O + (A##2).w; O = O + (A##3).x; O = O + (A##3).y; O = O + (A##3).z; O = O + (A##3).w;          \
    O = O + (A##4).x; O = O + (A##4).y; O = O + (A##4).z; O = O + (A##4).w; O = O + (A##5).x; O = O + (A##5).y; O = O + (A##5).z; O = O + (A##5).w;          \
    O = O + (A##6).x; O = O + (A##6).y; O = O + (A##6).z; O = O + (A##6).w; O = O + (A##7).x; O = O + (A##7).y; O = O + (A##7).z; O = O + (A##7).w;          \
  } while (0)

// The same for a chain of products: 16 scores from PS into S##0 .. S##3 and 16 values from PV into V##0 .. V##3.
#define ILT_LDS_READ16X2_AHEAD(S, V, PS, PV)                                                                                                \
  asm volatile("ds_read_b128 %0, %8\n\tds_read_b128 %1, %8 offset:16\n\tds_read_b128 %2, %8 offset:32\n\tds_read_b128 %3, %8 offset:48\n\t" \
               "ds_read_b128 %4, %9\n\tds_read_b128 %5, %9 offset:16\n\tds_read_b128 %6, %9 offset:32\n\tds_read_b128 %7, %9 offset:48"   \
               : "=&v"(S##0), "=&v"(S##1), "=&v"(S##2), "=&v"(S##3), "=&v"(V##0), "=&v"(V##1), "=&v"(V##2), "=&v"(V##3)                   \
               : "v"((u32)(uintptr_t)(ILT_LDS const void*)(PS)), "v"((u32)(uintptr_t)(ILT_LDS const void*)(PV)) : "memory")
#define ILT_LDS_READ16X2_WAIT(S, V, LEFT)                                                                                                   \
  asm volatile("s_waitcnt lgkmcnt(" #LEFT ")" : "+v"(S##0), "+v"(S##1), "+v"(S##2), "+v"(S##3), "+v"(V##0), "+v"(V##1), "+v"(V##2), "+v"(V##3) :: "memory")
#define ILT_CHAIN_MULADD4(O, S, V)                                                                                                          \
  do {                                                                                                                                      \
    const float a0_ = (S).x * (V).x, a1_ = (S).y * (V).y, a2_ = (S).z * (V).z, a3_ = (S).w * (V).w;                                         \
    O = O + a0_; O = O + a1_; O = O + a2_; O = O + a3_;                                                                                     \
  } while (0)
#define ILT_CHAIN_MULADD16(O, S, V)                                                                                                         \
  do { ILT_CHAIN_MULADD4(O, S##0, V##0); ILT_CHAIN_MULADD4(O, S##1, V##1); ILT_CHAIN_MULADD4(O, S##2, V##2); ILT_CHAIN_MULADD4(O, S##3, V##3); } while (0)

// The chain of one column: o = ((0 + col[0]) + col[1]) + .. over npos floats of a row in LDS; last_read: the last
// float of the row from which 32 can be read (the row is padded past npos).  The reads of 32 positions are on their
// way while the 32 before them are added: left to itself the compiler moves every read down to its use, and a chain
// of adds then waits for LDS once every 32 positions.
__device__ __forceinline__ float chain_add_from(float o, const float* col, int npos, int last_read);
__device__ __forceinline__ float chain_add_row(const float* col, int npos, int last_read) { return chain_add_from(0.0f, col, npos, last_read); }
// (the same carried on from o: a column that comes in tiles)
__device__ __forceinline__ float chain_add_from(float o, const float* col, int npos, int last_read) {
  int p = 0;
  typedef float f4v __attribute__((ext_vector_type(4)));
  f4v v0, v1, v2, v3, v4, v5, v6, v7, w0, w1, w2, w3, w4, w5, w6, w7;
  ILT_LDS_READ32_AHEAD(v, col);
  for (; p + 64 <= npos; p += 64) {
    ILT_LDS_READ32_AHEAD(w, col + p + 32);
    ILT_LDS_READ32_WAIT(v, 8);
    ILT_CHAIN_ADD32(o, v);
    ILT_LDS_READ32_AHEAD(v, col + min(p + 64, last_read));
    ILT_LDS_READ32_WAIT(w, 8);
    ILT_CHAIN_ADD32(o, w);
  }
  ILT_LDS_READ32_WAIT(v, 0);
  if (p + 32 <= npos) {                            // v holds positions p .. p+31
    ILT_CHAIN_ADD32(o, v);
    p += 32;
  }
  for (; p < npos; p++) o = o + col[p];
  return o;
}

// The chain of one column with the products made on the way: o = ((0 + sc[0] col[0]) + sc[1] col[1]) + ..; the reads
// of 16 positions on their way while the 16 before them are multiplied and added.  last_read: the last float of col's
// row from which 16 can be read; sc's row may be read 16 floats past npos.
__device__ __forceinline__ float chain_muladd_from(float o, const float* sc, const float* col, int npos, int last_read);
__device__ __forceinline__ float chain_muladd_row(const float* sc, const float* col, int npos, int last_read) {
  return chain_muladd_from(0.0f, sc, col, npos, last_read);
}
// (carried on from o: scores and column that come in tiles.  sc's row too is read from min(.., last_read) here, so both
// rows need 16 floats of room past last_read and no more)
__device__ __forceinline__ float chain_muladd_from(float o, const float* sc, const float* col, int npos, int last_read) {
  typedef float f4v __attribute__((ext_vector_type(4)));
  int p = 0;
  f4v s0, s1, s2, s3, v0, v1, v2, v3, t0, t1, t2, t3, w0, w1, w2, w3;
  ILT_LDS_READ16X2_AHEAD(s, v, sc, col);
  for (; p + 32 <= npos; p += 32) {
    ILT_LDS_READ16X2_AHEAD(t, w, sc + p + 16, col + p + 16);
    ILT_LDS_READ16X2_WAIT(s, v, 8);
    ILT_CHAIN_MULADD16(o, s, v);
    ILT_LDS_READ16X2_AHEAD(s, v, sc + min(p + 32, last_read), col + min(p + 32, last_read));
    ILT_LDS_READ16X2_WAIT(t, w, 8);
    ILT_CHAIN_MULADD16(o, t, w);
  }
  ILT_LDS_READ16X2_WAIT(s, v, 0);
  if (p + 16 <= npos) {                            // s, v hold positions p .. p+15
    ILT_CHAIN_MULADD16(o, s, v);
    p += 16;
  }
  for (; p < npos; p++) o = o + sc[p] * col[p];
  return o;
}

// softmax of one token's raw scores into sc (LDS) by the NT threads that call it (me = 0..NT-1): NT = 64, one
// wave, or the whole workgroup of 256 with red/redd for the waves to meet.  PRE: the thread's raw scores
// (positions me, me + NT, ..) are in pre already, at most eight of them.
template <int NT, bool PRE>
__device__ __forceinline__ void attn_softmax(const float* __restrict__ rw, const float* pre, float* sc, int npos, int me, float* redf, double* redd) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float mx = -3.402823466e38f;
  if (PRE) {
#pragma unroll
    for (int u = 0; u < 8; u++) if (me + NT * u < npos) { sc[me + NT * u] = pre[u]; mx = fmaxf(mx, pre[u]); }
  } else {
    for (int p = me; p < npos; p += NT) { const float sv = rw[p]; sc[p] = sv; mx = fmaxf(mx, sv); }
  }
  mx = wave_max_float(mx);
  if (NT > 64) {
    if (lane == 0) redf[wave] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(redf[0], redf[1]), fmaxf(redf[2], redf[3]));
  }
  double part = 0.0;
  for (int p = me; p < npos; p += NT) { const float e = ilt_expf_via_double(sc[p] - mx); sc[p] = e; part += (double)e; }
  part = wave_sum_double(part);
  double sum = part;
  if (NT > 64) {
    if (lane == 0) redd[wave] = part;
    __syncthreads();
    sum = (redd[0] + redd[1]) + (redd[2] + redd[3]);
  }
  // the CPU adds the terms one after another: take its sum where the order could show in the rounded reciprocal
  float inv;
  if (!recip_settled(sum, npos, &inv)) {           // the same in all NT threads
    if (NT > 64) __syncthreads();
    if (me == 0) { double s2 = 0.0; for (int p = 0; p < npos; p++) s2 += (double)sc[p]; redd[NT > 64 ? 0 : 4 + wave] = s2; }
    if (NT > 64) __syncthreads();
    inv = (float)(1.0 / redd[NT > 64 ? 0 : 4 + wave]);
  }
  for (int p = me; p < npos; p += NT) sc[p] = sc[p] * inv;
}

// grid x = head * (hd/16) + column slice; grid y = token group.  LDS: TG rows of spitch scores, then the value
// slice with the positions along a row, vt[c * vpitch + p] (vpitch = 4 mod 64: sixteen threads' 16-byte reads
// of sixteen rows fall on different banks).  NB: the slice is at most NB * 2048 16-byte pieces (512 NB positions).
// With one token a workgroup the slice is stored times that token's scores, by all threads, and the chains add.
// A prompt chunk's softmax, once a (head, token) instead of once in each of the head's hd/16 workgroups of
// attn_values_kernel (the exps go through double: eight times over they were most of that kernel): the raw scores of
// row (t, h) become the scaled scores, in place.
__global__ __launch_bounds__(256) void attn_softmax_kernel(float* __restrict__ raw, int nh, int pos0, int spitch) {
  extern __shared__ __align__(16) float dyn[];
  __shared__ float redf[4];
  __shared__ double redd[8];
  const int h = blockIdx.x, t = blockIdx.y, npos = pos0 + t + 1;
  float* rw = raw + ((long long)t * nh + h) * spitch;
  attn_softmax<256, false>(rw, nullptr, dyn, npos, threadIdx.x, redf, redd);
  for (int p = threadIdx.x; p < npos; p += 256) rw[p] = dyn[p];       // (each thread the entries it scaled itself)
}

// PROB: raw holds the scaled scores already (attn_softmax_kernel ran).
template <int TG, int NB, bool PROB = false>
__global__ __launch_bounds__(256) void attn_values_kernel(const float* __restrict__ raw, const float* __restrict__ vc, float* __restrict__ out,
                                                          int nh, int nkv, int hd, int pos0, int ntok, int spitch, int vpitch) {
  extern __shared__ __align__(16) float dyn[];
  __shared__ float redf[4];
  __shared__ double redd[8];
  // (a head's hd/16 workgroups on one die, as in attn_step_fused_kernel: the head's score rows come into one L2)
  const int gx = gridDim.x, bx = (gx & 7) ? (int)blockIdx.x : (int)(blockIdx.x & 7) * (gx >> 3) + (int)(blockIdx.x >> 3);
  const int ns = hd >> 4, h = bx / ns, cs = bx - h * ns, t0 = blockIdx.y * TG, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int tn = min(TG, ntok - t0), nposmax = pos0 + t0 + tn;
  const int group = nh / nkv, kvd = nkv * hd, ko = (h / group) * hd + 16 * cs;
  float* scores = dyn;
  // a token's scores 4 floats further on in LDS than a multiple of 64: the 16-byte reads of a wave's four tokens fall on
  // different banks (at a multiple they all want the same four)
  const int lp = TG > 1 ? spitch + 4 : spitch;
  float* vt = dyn + TG * lp;
  // every load is asked for before anything waits, the scores first: no branch around a load, so that the
  // softmax waits for the scores alone and the value slice arrives meanwhile
  float pre[8];
  if (TG == 1) {
    const float* rw = raw + ((long long)t0 * nh + h) * spitch;
#pragma unroll
    for (int u = 0; u < 2 * NB; u++) pre[u] = rw[min(tid + 256 * u, nposmax - 1)];
  }
  float4 r[8 * NB];
  const int total = nposmax * 4;                   // 16-byte pieces
#pragma unroll
  for (int u = 0; u < 8 * NB; u++) {
    const int i = min(tid + 256 * u, total - 1);
    r[u] = *(const float4*)(vc + (long long)(i >> 2) * kvd + ko + 4 * (i & 3));
  }
  if (TG == 1) {
#pragma unroll
    for (int u = 2 * NB; u < 8; u++) pre[u] = 0.0f;
    attn_softmax<256, true>(nullptr, pre, scores, nposmax, tid, redf, redd);
    __syncthreads();                               // every thread's scaled scores, for the products below
  } else if (PROB) {
    // the group's rows of scaled scores, 16 bytes a thread, eight loads in flight before the first is stored (a load
    // and its store one pair after another would be a trip to memory each); what lies past a token's own positions in
    // its row is carried along and never read
    const int q4 = spitch >> 2, totalq = tn * q4;
    const float* rbase = raw + ((long long)t0 * nh + h) * spitch;
    for (int base = 0; base < totalq; base += 256 * 8) {
      float4 tmp[8];
#pragma unroll
      for (int u = 0; u < 8; u++) {
        const int i = min(base + tid + 256 * u, totalq - 1), tt = i / q4, j = i - tt * q4;
        tmp[u] = *(const float4*)(rbase + (long long)tt * nh * spitch + 4 * j);
      }
#pragma unroll
      for (int u = 0; u < 8; u++) {
        const int i = base + tid + 256 * u, tt = i / q4, j = i - tt * q4;
        if (i < totalq) *(float4*)(scores + tt * lp + 4 * j) = tmp[u];
      }
    }
  } else {
    for (int tt = wave; tt < tn; tt += 4)
      attn_softmax<64, false>(raw + ((long long)(t0 + tt) * nh + h) * spitch, nullptr, scores + tt * lp, pos0 + t0 + tt + 1, lane, redf, redd);
  }
#pragma unroll
  for (int u = 0; u < 8 * NB; u++) {
    const int i = tid + 256 * u;
    if (i < total) {
      float* dst = vt + (4 * (i & 3)) * vpitch + (i >> 2);
      if (TG == 1) {
        const float sp = scores[i >> 2];
        dst[0] = sp * r[u].x; dst[vpitch] = sp * r[u].y; dst[2 * vpitch] = sp * r[u].z; dst[3 * vpitch] = sp * r[u].w;
      } else {
        dst[0] = r[u].x; dst[vpitch] = r[u].y; dst[2 * vpitch] = r[u].z; dst[3 * vpitch] = r[u].w;
      }
    }
  }
  __syncthreads();                                 // the scores are scaled, the slice is in place
  if (tid < tn * 16) {
    const int tt = tid >> 4, c = tid & 15, npos = pos0 + t0 + tt + 1;
    const float* sc = scores + tt * lp;
    const float* col = vt + c * vpitch;
    out[((long long)(t0 + tt) * nh + h) * hd + 16 * cs + c] = TG == 1 ? chain_add_row(col, npos, vpitch - 36) : chain_muladd_row(sc, col, npos, vpitch - 16);
  }
}

// One token's whole attention in one launch, for contexts of up to 1,024 positions: a workgroup of 1,024 threads a
// (query head, CS columns of the values).  Each norms and turns its query head and its KV head's key itself
// (waves 0 and 1), takes the head's scores for every position (attn_step_scores_kernel's sums; the keys of a head
// come from L2 once for each of its hd/CS workgroups, which is what bounds the context), scales them, and adds its
// CS columns as attn_values_kernel<1> does.  The group's first query head's first workgroup writes the key and the
// value into the caches; the token's own key and value are taken from k and v, never from the caches.  NJ = hd/16.
// SHARE set: the head's scores are shared out over its hd / CS workgroups -- each takes the passes of 64 positions
// numbered its slice, its slice + hd / CS, .. (at most two) -- instead of each taking all of them (the keys of 640
// positions are 330 KB a workgroup, read by every one of the head's eight).  A score travels as eight bytes, its bits
// and a tag (the head's generation on the device, the host's count of launches, the writer's die), written with one
// plain store into attn_xrow, a buffer of the library's; the thread that wants position p reads that word until it
// carries this launch's tag.  A plain store is seen in its die's L2 and no further within a launch, so the tag's die
// must be the reader's own (HW_REG_XCC_ID): the launcher asks for SHARE where a head's workgroups run on one die, and
// where the hardware puts them elsewhere -- or a partner is not resident and nothing arrives within PATIENCE ticks of
// the 100 MHz clock -- the workgroup takes all the scores itself, as without SHARE.  The head's first workgroup
// advances the generation as it ends (every workgroup read it as it started, microseconds earlier), so a launch
// replayed from a graph finds new tags; the host's count tells apart launches that overlap on one GPU, which make each
// other give up (they share the buffer) but do not read each other's scores.  (24 bits of generation: a word left in
// the buffer could pass for a fresh one only if it was written exactly 2^24 - 1 launches of its head earlier.)
// A workgroup that gives up writes its own words over with a tag no launch uses (generation 0xFFFFFF is skipped),
// so that what it wrote under a generation its partners did not share -- it started after its head's first workgroup
// had ended and read the advanced generation -- cannot pass for fresh in a later launch that reaches that generation
// with the same count of launches (the same captured launch replayed), and it counts itself in attn_giveups.
// Launches overlap on a GPU only across streams, so each stream gets a buffer of its own (kAttnSlots of them; the
// streams past that share the last one): two decoders on one GPU do not make each other give up.
// What sharing out relies on, beyond its tests: consecutive workgroups go to the eight dies in turn, and a head's
// workgroups are resident together (256 workgroups of 1,024 threads: one a CU on an otherwise idle GPU).  Where either
// fails the cost is the wait (PATIENCE, 200 us a launch), not the result.
constexpr int kAttnSlots = 8;
constexpr unsigned kAttnNoGen = 0xFFFFFFu;
__device__ unsigned attn_gen[kAttnSlots][256];
__device__ unsigned long long attn_xrow[kAttnSlots][256 * 1024];
__device__ unsigned long long attn_giveups;
template <int NJ, int CS>
__global__ __launch_bounds__(1024) void attn_step_fused_kernel(const float* __restrict__ q, const float* __restrict__ k, const float* __restrict__ v,
                                                               const float* __restrict__ qn, const float* __restrict__ kn,
                                                               const float* __restrict__ rope, float* __restrict__ kc, float* __restrict__ vc,
                                                               float* __restrict__ out, int nh, int nkv, int rd, int pos, float eps, int neox,
                                                               float scale, int vpitch, int share, unsigned epoch, int patience,
                                                               unsigned* __restrict__ xgen, unsigned long long* __restrict__ xrow) {
  extern __shared__ __align__(16) float dyn[];
  __shared__ float qsh[16 * NJ], ksh[16 * NJ], redf[16];
  __shared__ double scs[2], redd[17];
  __shared__ int got_all;
  __shared__ unsigned tag_sh;
  constexpr int hd = 16 * NJ;
  // the hardware deals consecutive workgroups to the eight dies in turn: die x takes the workgroups of consecutive heads
  // (with 32 query heads on 8 KV heads, one KV head's), so a head's keys and values come from memory into one L2 only
  const int nwg = gridDim.x, wg = (nwg & 7) ? (int)blockIdx.x : (int)(blockIdx.x & 7) * (nwg >> 3) + (int)(blockIdx.x >> 3);
  const int ns = hd / CS, h = wg / ns, cs = wg - h * ns, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, npos = pos + 1;
  const int group = nh / nkv, kvd = nkv * hd, kh = h / group, ko = kh * hd, vo = ko + CS * cs;
  const int l = tid & 15, pg = tid >> 4, last = max(pos - 1, 0);
  float* sc = dyn;                                 // 1,024 scores
  float* vt = dyn + 1024;                          // the slice times the scores, a column a row of vpitch
  // the keys of positions 256 b .. 256 b + 255 for this thread's four passes (rows before the token's own)
  auto load_keys = [&](float (&kv)[4][NJ], int b) {
#pragma unroll
    for (int u = 0; u < 4; u++) {
      const float* kr = kc + (long long)min(256 * b + 64 * u + pg, last) * kvd + ko;
#pragma unroll
      for (int j = 0; j < NJ; j++) kv[u][j] = kr[l + 16 * j];
    }
  };
  // the head's own loads first (waves 0 and 1): the norms and the turn then wait for these alone
  const float* cst = rope + (long long)pos * rd;
  RopeIn<(NJ + 3) / 4> rin;
  if (wave < 2) rope_head_load(rin, wave == 0 ? q + h * hd : k + ko, wave == 0 ? qn : kn, cst, hd, rd, lane);
  float ka[4][NJ], kb[4][NJ];
  constexpr int NPASS = 16 / (hd / CS);            // passes of 64 positions a workgroup takes of a head's shared-out scores
  float kx[NPASS][NJ];
  const bool split = share != 0;
  // (the head's generation, read now and wanted after the heads are turned: the barrier there hands it round)
  if (split && tid == 0) {
    const unsigned gen = ((__hip_atomic_load(&xgen[h], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) & 0xFFFFFFu) + 1) % kAttnNoGen;
    tag_sh = gen << 8 | (epoch & 31u) << 3;
    got_all = 1;
  }
  if (split) {
#pragma unroll
    for (int i = 0; i < NPASS; i++) {
      const float* kr = kc + (long long)min(64 * (cs + ns * i) + pg, last) * kvd + ko;
#pragma unroll
      for (int j = 0; j < NJ; j++) kx[i][j] = kr[l + 16 * j];
    }
  } else load_keys(ka, 0);
  // (the rest of the loads after the heads are turned: sixteen waves' loads take as long to ask for as the turn takes,
  // and the workgroup would wait for the slowest wave's)
  if (wave < 2) rope_head_turn(rin, (wave == 0 ? qn : kn) != nullptr, wave == 0 ? qsh : ksh, &scs[wave], hd, rd, eps, neox, lane);
  __syncthreads();
  if (!split) load_keys(kb, 1);
  // the slice: 16-byte piece i = position i / PP, part i % PP; the token's own row from v
  constexpr int PP = CS / 4;
  float4 r[PP];
  const int total = npos * PP;
  auto load_slice = [&]() {
#pragma unroll
    for (int u = 0; u < PP; u++) {
      const int i = min(tid + 1024 * u, total - 1), p = i / PP;
      const float* src = p == pos ? v + vo : vc + (long long)p * kvd + vo;
      r[u] = *(const float4*)(src + 4 * (i % PP));
    }
  };
  if (!split) load_slice();          // (shared-out scores: asked for once the scores are written, whose stores would wait for these loads)
  if (h == kh * group && cs == 0 && tid < hd) {
    kc[(long long)pos * kvd + ko + tid] = ksh[tid];
    vc[(long long)pos * kvd + ko + tid] = v[ko + tid];
  }
  float qv[NJ];
#pragma unroll
  for (int j = 0; j < NJ; j++) qv[j] = qsh[l + 16 * j];
  auto take_scores = [&](float (&kv)[4][NJ], int b) {
#pragma unroll
    for (int u = 0; u < 4; u++) {
      const int p = 256 * b + 64 * u + pg;
      if (p == pos) {
#pragma unroll
        for (int j = 0; j < NJ; j++) kv[u][j] = ksh[l + 16 * j];
      }
      float sacc = 0.0f;
#pragma unroll
      for (int j = 0; j < NJ; j++) sacc = sacc + kv[u][j] * qv[j];
      sacc = sacc + ilt_dppf<ILT_DPP_SHL(4)>(sacc);
      sacc = sacc + ilt_dppf<ILT_DPP_SHL(8)>(sacc);
      sacc = sacc + ilt_dppf<ILT_DPP_SHL(1)>(sacc);
      sacc = sacc + ilt_dppf<ILT_DPP_SHL(2)>(sacc);
      if (l == 0 && p < npos) sc[p] = sacc * scale;
    }
  };
  const int nb = (npos + 255) >> 8;                // 1 .. 4
  bool shared = false;
  if (split) {
    const unsigned die = __builtin_amdgcn_s_getreg((4 - 1) << 11 | 20) & 7u, tag = tag_sh | die;
    unsigned long long* const row = xrow + (long long)h * 1024;
#pragma unroll
    for (int i = 0; i < NPASS; i++) {
      const int p = 64 * (cs + ns * i) + pg;
      if (p == pos) {
#pragma unroll
        for (int j = 0; j < NJ; j++) kx[i][j] = ksh[l + 16 * j];
      }
      float sacc = 0.0f;
#pragma unroll
      for (int j = 0; j < NJ; j++) sacc = sacc + kx[i][j] * qv[j];
      sacc = sacc + ilt_dppf<ILT_DPP_SHL(4)>(sacc);
      sacc = sacc + ilt_dppf<ILT_DPP_SHL(8)>(sacc);
      sacc = sacc + ilt_dppf<ILT_DPP_SHL(1)>(sacc);
      sacc = sacc + ilt_dppf<ILT_DPP_SHL(2)>(sacc);
      if (l == 0 && p < npos) row[p] = (unsigned long long)tag << 32 | __float_as_uint(sacc * scale);
    }
    // position tid's score: its word until it carries the tag (any die's: this launch's, and then its die decides)
    if (tid < npos) {
      const long long t0 = wall_clock64();
      bool ok = false;
      unsigned long long w = 0;
      for (;;) {
        w = __hip_atomic_load(row + tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const unsigned t = (unsigned)(w >> 32);
        if ((t ^ tag) >> 3 == 0) { ok = (t & 7u) == die; break; }
        if (wall_clock64() - t0 >= (long long)patience) break;
        __builtin_amdgcn_s_sleep(1);
      }
      if (ok) sc[tid] = __uint_as_float((unsigned)w);
      else got_all = 0;
    }
    // (the slice behind the row: loads come back in the order asked for, and the row is wanted first.  From here to
    // the products the barriers wait for LDS only -- __syncthreads waits for every load in flight, the slice's too)
    load_slice();
    ilt_barrier_lds();
    shared = got_all != 0;
    if (!shared) {
      // giving up: this workgroup's words made unmatchable (see above), and the give-up counted
#pragma unroll
      for (int i = 0; i < NPASS; i++) {
        const int p = 64 * (cs + ns * i) + pg;
        if (l == 0 && p < npos) row[p] = ~0ull;
      }
      if (tid == 0) atomicAdd(&attn_giveups, 1ull);
    }
  }
  if (!shared) {
    if (split) { load_keys(ka, 0); load_keys(kb, 1); }
    take_scores(ka, 0);
    if (nb > 2) load_keys(ka, 2);
    if (nb > 1) take_scores(kb, 1);
    if (nb > 3) load_keys(kb, 3);
    if (nb > 2) take_scores(ka, 2);
    if (nb > 3) take_scores(kb, 3);
  }
  ilt_barrier_lds();
  // softmax (attn_softmax's steps with a position a thread)
  const bool mine = tid < npos;
  float mx = mine ? sc[tid] : -3.402823466e38f;
  const float sv = mx;
  mx = wave_max_float(mx);
  if (lane == 0) redf[wave] = mx;
  ilt_barrier_lds();
  mx = redf[0];
#pragma unroll
  for (int w = 1; w < 16; w++) mx = fmaxf(mx, redf[w]);
  const float e = mine ? ilt_expf_via_double(sv - mx) : 0.0f;
  const double part = wave_sum_double((double)e);
  if (lane == 0) redd[wave] = part;
  if (mine) sc[tid] = e;
  ilt_barrier_lds();
  double sum = redd[0];
#pragma unroll
  for (int w = 1; w < 16; w++) sum += redd[w];
  // the CPU adds the terms one after another: take its sum where the order could show in the rounded reciprocal
  float inv;
  if (!recip_settled(sum, npos, &inv)) {           // the same in every thread
    if (tid == 0) { double s2 = 0.0; for (int p = 0; p < npos; p++) s2 += (double)sc[p]; redd[16] = s2; }
    ilt_barrier_lds();
    inv = (float)(1.0 / redd[16]);
  }
  // (a position's probability, e * inv, is made by the threads that multiply with it: sc keeps the e's, which every
  // thread may read since the barrier above, and the barrier that handing the products round would take is saved)
#pragma unroll
  for (int u = 0; u < PP; u++) {
    const int i = tid + 1024 * u;
    if (i < total) {
      float* dst = vt + (4 * (i % PP)) * vpitch + i / PP;
      const float sp = sc[i / PP] * inv;
      dst[0] = sp * r[u].x; dst[vpitch] = sp * r[u].y; dst[2 * vpitch] = sp * r[u].z; dst[3 * vpitch] = sp * r[u].w;
    }
  }
  ilt_barrier_lds();
  if (tid < CS) {
    const float* col = vt + tid * vpitch;
    out[h * hd + CS * cs + tid] = chain_add_row(col, npos, vpitch - 36);
  }
  // The head's first workgroup advances the generation as it ends: every workgroup of this launch read it as it
  // started, many microseconds ago (one that starts only now finds the new one, matches no flag and takes all the scores
  // itself).  A store: a counter of readers would be a read-modify-write whose answer a workgroup waits 2 us for.
  if (split && tid == 0 && cs == 0) __hip_atomic_store(&xgen[h], tag_sh >> 8, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The same for contexts whose value slice no longer fits LDS (2,049 to 8,192 positions): the slice comes through
// LDS in tiles of kValTile positions, and a chain carries its sum from tile to tile -- position after position all
// the same.  TG 1: the token's scores are taken and scaled here and stay in LDS.  TG 16 (a prompt's chunk): the
// scores come scaled from attn_softmax_kernel and go through LDS tile by tile like the values.
constexpr int kValTile = 1024, kValPitch = kValTile + 4;
template <int TG>
__global__ __launch_bounds__(256) void attn_values_tiled_kernel(const float* __restrict__ raw, const float* __restrict__ vc, float* __restrict__ out,
                                                                int nh, int nkv, int hd, int pos0, int ntok, int spitch) {
  extern __shared__ __align__(16) float dyn[];
  __shared__ float redf[4];
  __shared__ double redd[8];
  const int ns = hd >> 4, h = blockIdx.x / ns, cs = blockIdx.x - h * ns, t0 = blockIdx.y * TG, tid = threadIdx.x;
  const int tn = min(TG, ntok - t0), nposmax = pos0 + t0 + tn;
  const int group = nh / nkv, kvd = nkv * hd, ko = (h / group) * hd + 16 * cs;
  const int lp = TG > 1 ? kValPitch : spitch;        // TG > 1: a token's scores of the tile; TG 1: all of the token's
  float* scores = dyn;
  float* vt = dyn + TG * lp;
  const float* rbase = raw + ((long long)t0 * nh + h) * spitch;
  if (TG == 1) attn_softmax<256, false>(rbase, nullptr, scores, nposmax, tid, redf, redd);
  const int tt = tid >> 4, c = tid & 15, npos = pos0 + t0 + tt + 1;       // a chain's token and column (tid < tn * 16)
  const float* sc = scores + tt * lp;
  const float* col = vt + c * kValPitch;
  float o = 0.0f;
  for (int p0 = 0; p0 < nposmax; p0 += kValTile) {
    const int npt = min(kValTile, nposmax - p0), total = npt * 4;       // the tile's positions, its 16-byte pieces of values
    float4 r[16];
#pragma unroll
    for (int u = 0; u < 16; u++) {
      const int i = min(tid + 256 * u, total - 1);
      r[u] = *(const float4*)(vc + (long long)(p0 + (i >> 2)) * kvd + ko + 4 * (i & 3));
    }
    __syncthreads();                                 // the scores are there (TG 1, first tile); the chains are through with the tile before
    if (TG > 1) {
      // the group's scores of the tile's positions: 256 pieces a row at most (what lies past a token's own positions is
      // carried along and never read; past the row's end nothing is loaded)
      const int q4 = (npt + 3) >> 2, totalq = tn * q4;
      for (int base = 0; base < totalq; base += 256 * 8) {
        float4 tmp[8];
#pragma unroll
        for (int u = 0; u < 8; u++) {
          const int i = min(base + tid + 256 * u, totalq - 1), rt = i / q4, j = i - rt * q4;
          tmp[u] = *(const float4*)(rbase + (long long)rt * nh * spitch + p0 + 4 * j);
        }
#pragma unroll
        for (int u = 0; u < 8; u++) {
          const int i = base + tid + 256 * u, rt = i / q4, j = i - rt * q4;
          if (i < totalq) *(float4*)(scores + rt * lp + 4 * j) = tmp[u];
        }
      }
    }
#pragma unroll
    for (int u = 0; u < 16; u++) {
      const int i = tid + 256 * u;
      if (i < total) {
        float* dst = vt + (4 * (i & 3)) * kValPitch + (i >> 2);
        if (TG == 1) {
          const float sp = scores[p0 + (i >> 2)];
          dst[0] = sp * r[u].x; dst[kValPitch] = sp * r[u].y; dst[2 * kValPitch] = sp * r[u].z; dst[3 * kValPitch] = sp * r[u].w;
        } else {
          dst[0] = r[u].x; dst[kValPitch] = r[u].y; dst[2 * kValPitch] = r[u].z; dst[3 * kValPitch] = r[u].w;
        }
      }
    }
    __syncthreads();
    if (tid < tn * 16) {
      const int np = min(kValTile, npos - p0);       // of the tile's positions, the token's own (may be none)
      int p = 0;
      if (TG == 1) {
        for (; p + 32 <= np; p += 32) {
          float4 v4[8];
#pragma unroll
          for (int u = 0; u < 8; u++) v4[u] = *(const float4*)(col + p + 4 * u);
#pragma unroll
          for (int u = 0; u < 8; u++) { o = o + v4[u].x; o = o + v4[u].y; o = o + v4[u].z; o = o + v4[u].w; }
        }
        for (; p < np; p++) o = o + col[p];
      } else {
        for (; p + 16 <= np; p += 16) {
          float4 s4[4], v4[4];
#pragma unroll
          for (int u = 0; u < 4; u++) { s4[u] = *(const float4*)(sc + p + 4 * u); v4[u] = *(const float4*)(col + p + 4 * u); }
#pragma unroll
          for (int u = 0; u < 4; u++) {
            const float a0 = s4[u].x * v4[u].x, a1 = s4[u].y * v4[u].y, a2 = s4[u].z * v4[u].z, a3 = s4[u].w * v4[u].w;
            o = o + a0; o = o + a1; o = o + a2; o = o + a3;
          }
        }
        for (; p < np; p++) o = o + sc[p] * col[p];
      }
    }
  }
  if (tid < tn * 16) out[((long long)(t0 + tt) * nh + h) * hd + 16 * cs + c] = o;
}

// One token's values for contexts past the one-launch kernel's, with the slice's tiles arriving while the chains run:
// a workgroup of sixteen waves a (query head, 16 columns); wave 0's first sixteen lanes do nothing but add -- a column
// each, tile after tile -- and the other fifteen waves bring the tiles in: tile t+1 is multiplied by its positions'
// scores and stored into the buffer tile t-1 has left while tile t is being added, and tile t+2's loads are on their way
// from then on.  All sixteen waves take the softmax first (the scores come from attn_step_scores_kernel, raw).  The
// numbers are attn_values_tiled_kernel<1>'s: every product and every sum the same, in the same order.
constexpr int kStreamTile = 480, kStreamPitch = kStreamTile + 36;      // (a row: 32 floats of room past a tile for the reads ahead; 4 mod 64)
__global__ __launch_bounds__(1024) void attn_values_stream_kernel(const float* __restrict__ raw, const float* __restrict__ vc, float* __restrict__ out,
                                                                  int nh, int nkv, int hd, int pos, int spitch) {
  extern __shared__ __align__(16) float dyn[];
  __shared__ float redf[16];
  __shared__ double redd[17];
  const int gx = gridDim.x, bx = (gx & 7) ? (int)blockIdx.x : (int)(blockIdx.x & 7) * (gx >> 3) + (int)(blockIdx.x >> 3);
  const int ns = hd >> 4, h = bx / ns, cs = bx - h * ns, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int npos = pos + 1, group = nh / nkv, kvd = nkv * hd, ko = (h / group) * hd + 16 * cs;
  float* sc = dyn;                                 // the token's scores, all of them
  float* vt = dyn + spitch;                        // two tiles of the slice times the scores, a column a row of kStreamPitch
  const float* rw = raw + (long long)h * spitch;
  const int ntiles = (npos + kStreamTile - 1) / kStreamTile, li = tid - 64;      // li: a loading thread's number, 0 .. 959
  // tile's 16-byte pieces li and li + 960: position piece / 4, columns 4 * (piece % 4) ..
  auto load_tile = [&](int tile, float4 (&r)[2]) {
    const int p0 = tile * kStreamTile, total = min(kStreamTile, npos - p0) * 4;
#pragma unroll
    for (int u = 0; u < 2; u++) {
      const int i = min(li + 960 * u, total - 1);
      r[u] = *(const float4*)(vc + (long long)(p0 + (i >> 2)) * kvd + ko + 4 * (i & 3));
    }
  };
  auto store_tile = [&](int tile, const float4 (&r)[2]) {
    const int p0 = tile * kStreamTile, total = min(kStreamTile, npos - p0) * 4;
    float* b = vt + (tile & 1) * (16 * kStreamPitch);
#pragma unroll
    for (int u = 0; u < 2; u++) {
      const int i = li + 960 * u;
      if (i < total) {
        float* dst = b + (4 * (i & 3)) * kStreamPitch + (i >> 2);
        const float sp = sc[p0 + (i >> 2)];
        dst[0] = sp * r[u].x; dst[kStreamPitch] = sp * r[u].y; dst[2 * kStreamPitch] = sp * r[u].z; dst[3 * kStreamPitch] = sp * r[u].w;
      }
    }
  };
  float4 ra[2], rb[2];
  if (wave > 0) {
    load_tile(0, ra);
    if (ntiles > 1) load_tile(1, rb);
  }
  // softmax (attn_softmax's steps over sixteen waves)
  float mx = -3.402823466e38f;
  for (int p = tid; p < npos; p += 1024) { const float sv = rw[p]; sc[p] = sv; mx = fmaxf(mx, sv); }
  mx = wave_max_float(mx);
  if (lane == 0) redf[wave] = mx;
  __syncthreads();
  mx = redf[0];
#pragma unroll
  for (int w = 1; w < 16; w++) mx = fmaxf(mx, redf[w]);
  double part = 0.0;
  for (int p = tid; p < npos; p += 1024) { const float e = ilt_expf_via_double(sc[p] - mx); sc[p] = e; part += (double)e; }
  part = wave_sum_double(part);
  if (lane == 0) redd[wave] = part;
  __syncthreads();
  double sum = redd[0];
#pragma unroll
  for (int w = 1; w < 16; w++) sum += redd[w];
  float inv;
  if (!recip_settled(sum, npos, &inv)) {           // the same in every thread
    if (tid == 0) { double s2 = 0.0; for (int p = 0; p < npos; p++) s2 += (double)sc[p]; redd[16] = s2; }
    __syncthreads();
    inv = (float)(1.0 / redd[16]);
  }
  for (int p = tid; p < npos; p += 1024) sc[p] = sc[p] * inv;
  __syncthreads();                                 // every position's scaled score, for the products
  if (wave > 0) store_tile(0, ra);
  float o = 0.0f;
  const float* col = vt + lane * kStreamPitch;     // (lanes 0 .. 15 of wave 0)
  auto step = [&](int t, float4 (&next)[2], float4 (&after)[2]) {      // next holds tile t+1; after: free, takes tile t+2
    __syncthreads();                               // tile t is in place, and tile t-1's chains are through with the other buffer
    if (wave == 0) {
      if (lane < 16) o = chain_add_from(o, col + (t & 1) * (16 * kStreamPitch), min(kStreamTile, npos - t * kStreamTile), kStreamPitch - 36);
    } else {
      if (t + 1 < ntiles) store_tile(t + 1, next);
      if (t + 2 < ntiles) load_tile(t + 2, after);
    }
  };
  for (int t = 0; t < ntiles; t += 2) {
    step(t, rb, ra);
    if (t + 1 < ntiles) step(t + 1, ra, rb);
  }
  if (tid < 16) out[h * hd + 16 * cs + tid] = o;
}

// A prompt chunk's values, 32 tokens x 32 columns of a query head a workgroup of 1,024 threads, a chain each: the scaled
// scores (attn_softmax_kernel's) and the value slice come through LDS in tiles of 256 positions, each tile's loads on
// their way while the tile before it is multiplied and added.  A tile of scores serves 32 columns and a tile of values
// 32 tokens -- attn_values_kernel<16> and attn_values_tiled_kernel<16> bring a tile in for 16 of each, and what those
// kernels wait for is the tiles, not the chains.  The numbers are theirs: the same products and sums in the same order.
constexpr int kChunkTile = 256, kChunkPitch = kChunkTile + 4;      // (4 mod 64: sixteen rows' 16-byte reads on different banks)
__global__ __launch_bounds__(1024) void attn_values_chunk_kernel(const float* __restrict__ raw, const float* __restrict__ vc, float* __restrict__ out,
                                                                 int nh, int nkv, int hd, int pos0, int ntok, int spitch) {
  extern __shared__ __align__(16) float dyn[];
  float* const scs = dyn;                          // a row a token
  float* const vts = dyn + 32 * kChunkPitch;       // a row a column
  const int gx = gridDim.x, bx = (gx & 7) ? (int)blockIdx.x : (int)(blockIdx.x & 7) * (gx >> 3) + (int)(blockIdx.x >> 3);
  const int ns = hd >> 5, h = bx / ns, cs = bx - h * ns, t0 = blockIdx.y * 32, tid = threadIdx.x;
  const int tn = min(32, ntok - t0), nposmax = pos0 + t0 + tn;
  const int group = nh / nkv, kvd = nkv * hd, ko = (h / group) * hd + 32 * cs;
  const float* rbase = raw + ((long long)t0 * nh + h) * spitch;
  const int tt = tid >> 5, c = tid & 31, npos = tt < tn ? pos0 + t0 + tt + 1 : 0;      // this thread's chain: token t0 + tt, column 32 cs + c
  const int ntiles = (nposmax + kChunkTile - 1) / kChunkTile;
  float4 rs[2], rv[2];
  // a tile's 16-byte pieces: of the scores, q4 a token's row (what lies past a token's own positions is carried along and
  // never read; past the rows' end nothing is loaded); of the values, eight a position
  auto load_tile = [&](int tile) {
    const int p0 = tile * kChunkTile, q4 = min(kChunkTile, spitch - p0) >> 2, totalq = tn * q4;
    const int totalv = min(kChunkTile, nposmax - p0) * 8;
#pragma unroll
    for (int u = 0; u < 2; u++) {
      const int i = min(tid + 1024 * u, totalq - 1), rt = i / q4, j = i - rt * q4;
      rs[u] = *(const float4*)(rbase + (long long)rt * nh * spitch + p0 + 4 * j);
      const int k = min(tid + 1024 * u, totalv - 1);
      rv[u] = *(const float4*)(vc + (long long)(p0 + (k >> 3)) * kvd + ko + 4 * (k & 7));
    }
  };
  auto store_tile = [&](int tile) {
    const int p0 = tile * kChunkTile, q4 = min(kChunkTile, spitch - p0) >> 2, totalq = tn * q4;
    const int totalv = min(kChunkTile, nposmax - p0) * 8;
#pragma unroll
    for (int u = 0; u < 2; u++) {
      const int i = tid + 1024 * u, rt = i / q4, j = i - rt * q4;
      if (i < totalq) *(float4*)(scs + rt * kChunkPitch + 4 * j) = rs[u];
      const int k = tid + 1024 * u;
      if (k < totalv) {
        float* dst = vts + (4 * (k & 7)) * kChunkPitch + (k >> 3);
        dst[0] = rv[u].x; dst[kChunkPitch] = rv[u].y; dst[2 * kChunkPitch] = rv[u].z; dst[3 * kChunkPitch] = rv[u].w;
      }
    }
  };
  load_tile(0);
  float o = 0.0f;
  for (int t = 0; t < ntiles; t++) {
    if (t) __syncthreads();                        // the chains are through with the tile before
    store_tile(t);
    if (t + 1 < ntiles) load_tile(t + 1);          // on their way while this tile is added
    __syncthreads();
    const int np = min(kChunkTile, npos - t * kChunkTile);       // of the tile's positions, the token's own (may be none)
    if (np > 0) o = chain_muladd_from(o, scs + tt * kChunkPitch, vts + c * kChunkPitch, np, kChunkPitch - 16);
  }
  if (tt < tn) out[((long long)(t0 + tt) * nh + h) * hd + 32 * cs + c] = o;
}

// The same values with sixteen chains a thread, four tokens by four columns: a workgroup of 256 threads takes a query
// head's HD columns for 4096 / HD tokens (32 at HD = 128).  The kernel above reads LDS eight times (16 bytes each) per
// chain and 16 positions, which is what it waits for; here the four scores of a token (16 bytes along the positions)
// serve four columns and a position's four values (16 bytes along the columns, as the cache holds them: no transpose)
// four tokens -- half a read per chain and 4 positions -- and what is left is the multiplies and adds.  Tiles of 32
// positions, in two LDS buffers, loaded into registers a tile ahead of their store.  A tile that lies wholly below all
// of a wave's tokens goes without a test; the one or two at the tokens' own positions leave a chain alone from its
// token's last position on.  Every chain: the same products and sums in the
// same order as above.
template <int HD>
__global__ __launch_bounds__(256) void attn_values_quad_kernel(const float* __restrict__ raw, const float* __restrict__ vc, float* __restrict__ out,
                                                               int nh, int nkv, int pos0, int ntok, int spitch) {
  constexpr int CQ = HD / 4, TQ = 256 / CQ, NTOK = 4 * TQ, P = 32, SP = P + 4;
  constexpr int NV = P * CQ / 256;                 // 16-byte pieces of a tile a thread brings in: of the values,
  constexpr int NS = NTOK * (P / 4) / 256;         // of the scores
  static_assert((NV == 2 || NV == 4) && (NS == 1 || NS == 2) && 256 % CQ == 0, "HD 64 or 128");
  __shared__ __align__(16) float scs[2][NTOK * SP];      // a row a token
  __shared__ __align__(16) float vts[2][P * HD];         // a row a position
  const int gx = gridDim.x, h = (gx & 7) ? (int)blockIdx.x : (int)(blockIdx.x & 7) * (gx >> 3) + (int)(blockIdx.x >> 3);
  // (token tiles: the first half of the launch takes them from the last -- the longest -- downwards, the second half
  // from the first upwards: workgroups half a launch apart tend to share a CU, and so a long one meets a short one)
  const int ny = gridDim.y, yh = ny >> 1, by = blockIdx.y;
  const int t0 = (by < yh ? ny - 1 - by : by - yh) * NTOK, tid = threadIdx.x;
  const int tn = min(NTOK, ntok - t0), nposmax = pos0 + t0 + tn;
  const int group = nh / nkv, kvd = nkv * HD, ko = (h / group) * HD;
  const float* rbase = raw + ((long long)t0 * nh + h) * spitch;
  const int tq = tid / CQ, cq = tid - tq * CQ;     // tokens t0 + 4 tq .. + 3, columns 4 cq .. + 3
  const int wtq = (tid >> 6) * (64 / CQ);          // the wave's first tq
  const int ntiles = (nposmax + P - 1) / P;
  // (named registers: arrays indexed in these loops were left in private memory)
  float4 rs0 = {}, rs1 = {}, rv0 = {}, rv1 = {}, rv2 = {}, rv3 = {};
  // (past a token's own positions, past the rows' end and past the chunk's last token: a piece that exists, never used)
  auto load_s = [&](int p0, int u) {
    const int i = tid + 256 * u, rt = min(i >> 3, tn - 1), pc = min((p0 >> 2) + (i & 7), (spitch >> 2) - 1);
    return *(const float4*)(rbase + (long long)rt * nh * spitch + 4 * pc);
  };
  auto load_v = [&](int p0, int u) {
    const int k = tid + 256 * u, p = min(p0 + k / CQ, nposmax - 1);
    return *(const float4*)(vc + (long long)p * kvd + ko + 4 * (k % CQ));
  };
  auto load_tile = [&](int tile) {
    const int p0 = tile * P;
    rs0 = load_s(p0, 0);
    if (NS > 1) rs1 = load_s(p0, 1);
    rv0 = load_v(p0, 0);
    if (NV > 1) rv1 = load_v(p0, 1);
    if (NV > 2) { rv2 = load_v(p0, 2); rv3 = load_v(p0, 3); }
  };
  auto store_s = [&](int buf, int u, const float4& r) {
    const int i = tid + 256 * u;
    *(float4*)(scs[buf] + (i >> 3) * SP + 4 * (i & 7)) = r;
  };
  auto store_tile = [&](int buf) {
    store_s(buf, 0, rs0);
    if (NS > 1) store_s(buf, 1, rs1);
    *(float4*)(vts[buf] + 4 * tid) = rv0;
    if (NV > 1) *(float4*)(vts[buf] + 4 * (tid + 256)) = rv1;
    if (NV > 2) { *(float4*)(vts[buf] + 4 * (tid + 512)) = rv2; *(float4*)(vts[buf] + 4 * (tid + 768)) = rv3; }
  };
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int k = 0; k < 4; k++) acc[i][k] = 0.0f;
  load_tile(0);
  store_tile(0);
  if (ntiles > 1) load_tile(1);
  __syncthreads();
  for (int t = 0; t < ntiles; t++) {
    // tile t is in buffer t & 1; the registers hold tile t+1, and the other buffer's readers passed the last barrier
    if (t + 1 < ntiles) store_tile((t + 1) & 1);
    if (t + 2 < ntiles) load_tile(t + 2);
    const float* S = scs[t & 1] + 4 * tq * SP;
    const float* V = vts[t & 1] + 4 * cq;
    // of the tile's positions, token 4 tq + i has the first np + i (all of them from 32 on, none up to 0)
    const int np = pos0 + t0 + 4 * tq + 1 - t * P;
    const int npw = pos0 + t0 + 4 * wtq + 1 - t * P;       // the wave's first tokens': its least
    if (npw >= P) {
#pragma unroll
      for (int q = 0; q < P / 4; q++) {
        float4 s[4], v[4];
#pragma unroll
        for (int i = 0; i < 4; i++) s[i] = *(const float4*)(S + i * SP + 4 * q);
#pragma unroll
        for (int j = 0; j < 4; j++) v[j] = *(const float4*)(V + (4 * q + j) * HD);
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
          for (int i = 0; i < 4; i++) {
            const float sv = j == 0 ? s[i].x : j == 1 ? s[i].y : j == 2 ? s[i].z : s[i].w;
            acc[i][0] = acc[i][0] + sv * v[j].x;
            acc[i][1] = acc[i][1] + sv * v[j].y;
            acc[i][2] = acc[i][2] + sv * v[j].z;
            acc[i][3] = acc[i][3] + sv * v[j].w;
          }
      }
    } else if (npw + 4 * (64 / CQ) - 1 > 0) {              // some lane of the wave has positions here
#pragma unroll 1
      for (int q = 0; q < P / 4; q++) {
        if (4 * q >= np + 3) break;
        float4 s[4], v[4];
#pragma unroll
        for (int i = 0; i < 4; i++) s[i] = *(const float4*)(S + i * SP + 4 * q);
#pragma unroll
        for (int j = 0; j < 4; j++) v[j] = *(const float4*)(V + (4 * q + j) * HD);
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
          for (int i = 0; i < 4; i++) {
            const float sv = j == 0 ? s[i].x : j == 1 ? s[i].y : j == 2 ? s[i].z : s[i].w;
            const bool own = 4 * q + j < np + i;
            const float a0 = acc[i][0] + sv * v[j].x, a1 = acc[i][1] + sv * v[j].y;
            const float a2 = acc[i][2] + sv * v[j].z, a3 = acc[i][3] + sv * v[j].w;
            acc[i][0] = own ? a0 : acc[i][0];
            acc[i][1] = own ? a1 : acc[i][1];
            acc[i][2] = own ? a2 : acc[i][2];
            acc[i][3] = own ? a3 : acc[i][3];
          }
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int tk = t0 + 4 * tq + i;
    if (tk < ntok) *(float4*)(out + ((long long)tk * nh + h) * HD + 4 * cq) = make_float4(acc[i][0], acc[i][1], acc[i][2], acc[i][3]);
  }
}

// ARGMAX (model.lisp:464-468): best = 0; an element replaces the best when it is greater -- so the first of equal
// maxima, a NaN never (and if v[0] is a NaN nothing replaces it).  Two steps: each workgroup the best of its
// stretch (every thread's own elements first, eight 16-byte loads in flight, then the threads', a smaller index
// winning among equals) into part[blockIdx]; then one workgroup the best of those.  With no room for the parts
// (part null) one workgroup does it all.
struct ArgBest { float v; int i; };
__device__ __forceinline__ void arg_take(ArgBest& b, float x, int i) { if (x > b.v || (x == b.v && i < b.i)) { b.v = x; b.i = i; } }
__device__ __forceinline__ ArgBest arg_block(ArgBest b) {      // the workgroup's best, in thread 0
  __shared__ float bv[16];
  __shared__ int bi[16];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nw = blockDim.x >> 6;
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) arg_take(b, __shfl_xor(b.v, off), __shfl_xor(b.i, off));
  if (lane == 0) { bv[wave] = b.v; bi[wave] = b.i; }
  __syncthreads();
  if (tid == 0) for (int w = 1; w < nw; w++) arg_take(b, bv[w], bi[w]);
  return b;
}
__global__ __launch_bounds__(1024) void argmax_part_kernel(const float* __restrict__ v, int n, ArgBest* __restrict__ part, int* __restrict__ out) {
  const int tid = threadIdx.x, nt = blockDim.x, n4 = n >> 2;
  const int per = (n4 + gridDim.x - 1) / gridDim.x, lo = blockIdx.x * per, hi = min(n4, lo + per);      // this workgroup's 16-byte pieces
  ArgBest b = { -__builtin_inff(), 0x7FFFFFFF };
  for (int base = lo; base < hi; base += 8 * nt) {
    float4 x[8];
#pragma unroll
    for (int u = 0; u < 8; u++) x[u] = *(const float4*)(v + 4 * min(base + tid + nt * u, hi - 1));       // (past the end: the last piece again)
#pragma unroll
    for (int u = 0; u < 8; u++) {
      const int i = 4 * min(base + tid + nt * u, hi - 1);
      arg_take(b, x[u].x, i); arg_take(b, x[u].y, i + 1); arg_take(b, x[u].z, i + 2); arg_take(b, x[u].w, i + 3);
    }
  }
  if (blockIdx.x == gridDim.x - 1)
    for (int i = 4 * n4 + tid; i < n; i += nt) arg_take(b, v[i], i);
  b = arg_block(b);
  if (tid == 0) {
    if (part) part[blockIdx.x] = b;
    else { const float v0 = v[0]; out[0] = (v0 != v0 || b.i == 0x7FFFFFFF) ? 0 : b.i; }
  }
}
__global__ __launch_bounds__(256) void argmax_last_kernel(const float* __restrict__ v, const ArgBest* __restrict__ part, int nparts, int* __restrict__ out) {
  ArgBest b = { -__builtin_inff(), 0x7FFFFFFF };
  for (int i = threadIdx.x; i < nparts; i += 256) arg_take(b, part[i].v, part[i].i);
  b = arg_block(b);
  // a NaN in front (nothing is greater than a NaN) or nothing but NaNs: the scan never leaves index 0
  if (threadIdx.x == 0) { const float v0 = v[0]; out[0] = (v0 != v0 || b.i == 0x7FFFFFFF) ? 0 : b.i; }
}

// swiglu! (model.lisp:364-378) on n values: a = (a / (1 + e^-a)) * b, the exponential through double
__global__ __launch_bounds__(256) void swiglu_rows_kernel(float* __restrict__ a, const float* __restrict__ b, long long n) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i < n) { const float g = a[i]; a[i] = (g / (1.0f + ilt_expf_via_double(-g))) * b[i]; }
}

template <int TG>
void launch_scores(dim3 grid, hipStream_t st, const float* q, const float* kc, float* raw, int nh, int nkv, int hd, int pos0, int ntok, float scale,
                   int spitch) {
  if (hd == 128) hipLaunchKernelGGL((attn_scores_kernel<TG, 8>), grid, dim3(1024), 0, st, q, kc, raw, nh, nkv, hd, pos0, ntok, scale, spitch);
  else if (hd == 64) hipLaunchKernelGGL((attn_scores_kernel<TG, 4>), grid, dim3(1024), 0, st, q, kc, raw, nh, nkv, hd, pos0, ntok, scale, spitch);
  else hipLaunchKernelGGL((attn_scores_kernel<TG, 0>), grid, dim3(1024), 0, st, q, kc, raw, nh, nkv, hd, pos0, ntok, scale, spitch);
}

// one token's values past 2,048 positions (the scores: smax floats a head in scratch, raw)
hipError_t launch_values_stream(int dev, const float* scratch, const float* vc, float* out, int nh, int nkv, int hd, int pos, int smax,
                                hipStream_t st) {
  static bool set[64] = {};
  const size_t smem = sizeof(float) * ((size_t)smax + 2 * 16 * (size_t)kStreamPitch);
  if (smem > 152 * 1024 || dev < 0 || dev >= 64) return hipErrorInvalidValue;
  if (!set[dev]) {
    const hipError_t e = hipFuncSetAttribute((const void*)attn_values_stream_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 152 * 1024);
    if (e != hipSuccess) return e;
    set[dev] = true;
  }
  hipLaunchKernelGGL(attn_values_stream_kernel, dim3(nh * (hd / 16)), dim3(1024), smem, st, scratch, vc, out, nh, nkv, hd, pos, smax);
  return hipGetLastError();
}

}  // namespace

hipError_t ilt_k_qk_rope(float* q, float* k, const float* v, const float* qn, const float* kn, const float* rope, float* kc, float* vc,
                         int nh, int nkv, int hd, int rd, int pos0, float eps, int neox, int ntok, hipStream_t st) {
  if (ntok <= 0) return hipSuccess;
  if (hd > 512 || hd < 2 || rd > hd || (rd & 1) || nh < 1 || nkv < 1) return hipErrorInvalidValue;
  hipLaunchKernelGGL(qk_rope_kernel, dim3(nh + nkv, ntok), dim3(64), 0, st, q, k, v, qn, kn, rope, kc, vc, nh, nkv, hd, rd, pos0, eps, neox);
  return hipGetLastError();
}

// scratch: ntok * nh * ((pos0 + ntok + 3) & ~3) floats for the variants of two or three launches (contexts up to 8192
// positions), or null: one launch
hipError_t ilt_k_attn_rows(const float* q, const float* kc, const float* vc, float* out, int nh, int nkv, int hd, int pos0, int ntok,
                           float* scratch, hipStream_t st) {
  if (ntok <= 0) return hipSuccess;
  if (hd % 16 || hd > 256 || nh % nkv || pos0 < 0) return hipErrorInvalidValue;
  const int smax = (pos0 + ntok + 3) & ~3;
  const float scale = 1.0f / sqrtf((float)hd);
  static bool attr_set[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 0;
  // A chunk: scores, softmax, then 32 tokens x 32 columns a workgroup.  "ILT_ATTN_CHUNK=0": the kernels of 16 tokens x 16
  // columns below instead (tests).
  if (scratch && ntok > 1 && pos0 + ntok <= 8192 && hd % 32 == 0) {
    const char* off = getenv("ILT_ATTN_CHUNK");
    if (!(off && off[0] == '0')) {
      static bool set[64] = {};
      const size_t smem = sizeof(float) * 2 * 32 * (size_t)kChunkPitch;
      if (!set[dev]) {
        const hipError_t e = hipFuncSetAttribute((const void*)attn_values_chunk_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        if (e != hipSuccess) return e;
        set[dev] = true;
      }
      const int ctx = pos0 + ntok;
      // sixteen scores a thread for heads of 64 or 128 columns (16-byte loads of q and kc); "ILT_ATTN_QUAD=0" or "=v": the
      // kernel of sixteen lanes a score (tests)
      const char* quad = getenv("ILT_ATTN_QUAD");
      const bool qaligned = ((((uintptr_t)q) | ((uintptr_t)kc)) & 15) == 0;
      // (either kernel where it fills the GPU: 14 heads of 64 on 512 tokens are 112 workgroups of the values kernel,
      // and the kernel of a chain a thread, 448 workgroups, takes 59 us for the chunk's attention where this one took 78;
      // "ILT_ATTN_QUAD=1": whatever the shape)
      const bool forced = quad && quad[0] == '1';
      const long long swgs = (long long)nh * ((ctx + 63) / 64) * ((ntok + 63) / 64);
      const long long vwgs = (long long)nh * ((ntok + (hd == 128 ? 31 : 63)) / (hd == 128 ? 32 : 64));
      if ((hd == 128 || hd == 64) && qaligned && !(quad && (quad[0] == '0' || quad[0] == 'v')) && (forced || swgs >= 256)) {
        static bool qset[64] = {};
        const size_t qsmem = sizeof(float) * 2 * 64 * (size_t)(hd + 4);
        if (!qset[dev]) {
          hipError_t e = hipFuncSetAttribute((const void*)attn_scores_quad_kernel<8>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)(sizeof(float) * 2 * 64 * 132));
          if (e == hipSuccess)
            e = hipFuncSetAttribute((const void*)attn_scores_quad_kernel<4>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)(sizeof(float) * 2 * 64 * 68));
          if (e != hipSuccess) return e;
          qset[dev] = true;
        }
        const dim3 gq(nh, (ctx + 63) / 64, (ntok + 63) / 64);
        if (hd == 128) hipLaunchKernelGGL(attn_scores_quad_kernel<8>, gq, dim3(256), qsmem, st, q, kc, scratch, nh, nkv, pos0, ntok, scale, smax);
        else hipLaunchKernelGGL(attn_scores_quad_kernel<4>, gq, dim3(256), qsmem, st, q, kc, scratch, nh, nkv, pos0, ntok, scale, smax);
      } else {
        launch_scores<16>(dim3(nh, (ctx + 255) / 256, (ntok + 15) / 16), st, q, kc, scratch, nh, nkv, hd, pos0, ntok, scale, smax);
      }
      hipLaunchKernelGGL(attn_softmax_kernel, dim3(nh, ntok), dim3(256), sizeof(float) * smax, st, scratch, nh, pos0, smax);
      // sixteen chains a thread for heads of 64 or 128 columns (16-byte loads and stores: of scratch, vc and out);
      // "ILT_ATTN_QUAD=0": the kernel of one chain a thread (tests)
      const bool aligned = ((((uintptr_t)scratch) | ((uintptr_t)vc) | ((uintptr_t)out)) & 15) == 0;
      if ((hd == 128 || hd == 64) && aligned && !(quad && quad[0] == '0') && (forced || vwgs >= 192)) {
        if (hd == 128)
          hipLaunchKernelGGL(attn_values_quad_kernel<128>, dim3(nh, (ntok + 31) / 32), dim3(256), 0, st, scratch, vc, out, nh, nkv, pos0, ntok, smax);
        else
          hipLaunchKernelGGL(attn_values_quad_kernel<64>, dim3(nh, (ntok + 63) / 64), dim3(256), 0, st, scratch, vc, out, nh, nkv, pos0, ntok, smax);
        return hipGetLastError();
      }
      hipLaunchKernelGGL(attn_values_chunk_kernel, dim3(nh * (hd / 32), (ntok + 31) / 32), dim3(1024), smem, st, scratch, vc, out, nh, nkv, hd, pos0,
                         ntok, smax);
      return hipGetLastError();
    }
  }
  if (scratch && pos0 + ntok <= 2048) {
    const int ctx = pos0 + ntok, vpitch = ((ctx + 63) & ~63) + 4;
    // tokens a workgroup: as many as leave their scores and the value slice room in LDS (150 KB)
    auto bytes = [&](int tg) { return sizeof(float) * ((size_t)tg * (smax + (tg > 1 ? 4 : 0)) + 16 * (size_t)vpitch); };
    const int tg = ntok == 1 ? 1 : bytes(16) <= 150 * 1024 ? 16 : bytes(4) <= 150 * 1024 ? 4 : 1;
    // (a chunk whose sixteen tokens' scores and slice no longer fit LDS together -- past about 1,100 positions --
    // goes through the tiled kernels below, sixteen tokens a workgroup still: with four tokens a workgroup its values
    // took 1.6 ms a layer at 1,536 positions, with one 6.1 ms at 2,048)
    if (ntok == 1 || tg == 16) {
    const int nb = (ctx + 511) / 512;
    const dim3 gs(nh, (ctx + 255) / 256, (ntok + tg - 1) / tg), gv(nh * (hd / 16), (ntok + tg - 1) / tg);
    hipError_t e = hipErrorInvalidValue;
#define ILT_ATTN(TG, NB)                                                                                                                       \
  if (tg == TG && nb == NB) {                                                                                                                  \
    static bool set[64] = {};                                                                                                                  \
    e = set[dev] ? hipSuccess                                                                                                                  \
                 : hipFuncSetAttribute((const void*)attn_values_kernel<TG, NB, (TG > 1)>, hipFuncAttributeMaxDynamicSharedMemorySize,          \
                                       152 * 1024);                                                                                            \
    if (e == hipSuccess) {                                                                                                                     \
      set[dev] = true;                                                                                                                         \
      launch_scores<TG>(gs, st, q, kc, scratch, nh, nkv, hd, pos0, ntok, scale, smax);                                                         \
      if (TG > 1) hipLaunchKernelGGL(attn_softmax_kernel, dim3(nh, ntok), dim3(256), sizeof(float) * smax, st, scratch, nh, pos0, smax);        \
      hipLaunchKernelGGL((attn_values_kernel<TG, NB, (TG > 1)>), gv, dim3(256), bytes(TG), st, scratch, vc, out, nh, nkv, hd, pos0, ntok,      \
                         smax, vpitch);                                                                                                        \
      e = hipGetLastError();                                                                                                                   \
    }                                                                                                                                          \
  }
    ILT_ATTN(1, 1) ILT_ATTN(1, 2) ILT_ATTN(1, 3) ILT_ATTN(1, 4)
    ILT_ATTN(16, 1) ILT_ATTN(16, 2) ILT_ATTN(16, 3)
#undef ILT_ATTN
    return e;
    }
  }
  if (scratch && pos0 + ntok <= 8192) {              // the value slice through LDS in tiles
    const int ctx = pos0 + ntok, tg = ntok > 1 ? 16 : 1;
    const size_t smem = sizeof(float) * ((tg > 1 ? (size_t)tg * kValPitch : (size_t)smax) + 16 * (size_t)kValPitch);
    const dim3 gs(nh, (ctx + 255) / 256, (ntok + tg - 1) / tg), gv(nh * (hd / 16), (ntok + tg - 1) / tg);
    static bool set[64] = {};
    if (!set[dev]) {
      hipError_t e = hipFuncSetAttribute((const void*)attn_values_tiled_kernel<1>, hipFuncAttributeMaxDynamicSharedMemorySize, 152 * 1024);
      if (e == hipSuccess) e = hipFuncSetAttribute((const void*)attn_values_tiled_kernel<16>, hipFuncAttributeMaxDynamicSharedMemorySize, 152 * 1024);
      if (e != hipSuccess) return e;
      set[dev] = true;
    }
    if (tg == 16) {
      launch_scores<16>(gs, st, q, kc, scratch, nh, nkv, hd, pos0, ntok, scale, smax);
      hipLaunchKernelGGL(attn_softmax_kernel, dim3(nh, ntok), dim3(256), sizeof(float) * smax, st, scratch, nh, pos0, smax);
      hipLaunchKernelGGL(attn_values_tiled_kernel<16>, gv, dim3(256), smem, st, scratch, vc, out, nh, nkv, hd, pos0, ntok, smax);
    } else {
      launch_scores<1>(gs, st, q, kc, scratch, nh, nkv, hd, pos0, ntok, scale, smax);
      const hipError_t e = launch_values_stream(dev, scratch, vc, out, nh, nkv, hd, pos0, smax, st);
      if (e != hipSuccess) return e;
    }
    return hipGetLastError();
  }
  if (!attr_set[dev]) {
    const hipError_t e = hipFuncSetAttribute((const void*)attn_rows_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 152 * 1024);
    if (e != hipSuccess) return e;
    attr_set[dev] = true;
  }
  const size_t smem = sizeof(float) * ((size_t)smax + 2 * (size_t)kAttnTile * hd);
  if (smem > 150 * 1024) return hipErrorInvalidValue;      // a query's scores sit in LDS: about 20,000 positions at hd 128
  hipLaunchKernelGGL(attn_rows_kernel, dim3(nh, ntok), dim3(kAttnThreads), smem, st, q, kc, vc, out, nh, nkv, hd, pos0, scale, smax);
  return hipGetLastError();
}

// The exchange buffers of stream ST on device DEV: the device arrays' addresses (asked of the runtime once a device) and
// the stream's slot -- its own while fewer than kAttnSlots streams have asked on this device, else the last one, shared.
static hipError_t attn_exchange_of(int dev, hipStream_t st, unsigned** xgen, unsigned long long** xrow) {
  struct PerDev { unsigned* gen; unsigned long long* row; unsigned long long* giveups; hipStream_t streams[kAttnSlots]; int n; };
  static PerDev devs[64] = {};
  static std::mutex mu;
  std::lock_guard<std::mutex> lock(mu);
  PerDev& d = devs[dev];
  if (!d.gen) {
    void *g = nullptr, *r = nullptr, *c = nullptr;
    hipError_t e = hipGetSymbolAddress(&g, HIP_SYMBOL(attn_gen));
    if (e == hipSuccess) e = hipGetSymbolAddress(&r, HIP_SYMBOL(attn_xrow));
    if (e == hipSuccess) e = hipGetSymbolAddress(&c, HIP_SYMBOL(attn_giveups));
    if (e != hipSuccess) return e;
    d.gen = (unsigned*)g; d.row = (unsigned long long*)r; d.giveups = (unsigned long long*)c;
  }
  int slot = -1;
  for (int i = 0; i < d.n; i++) if (d.streams[i] == st) { slot = i; break; }
  if (slot < 0) {
    if (d.n < kAttnSlots) { slot = d.n; d.streams[d.n++] = st; }
    else slot = kAttnSlots - 1;
  }
  *xgen = d.gen + slot * 256;
  *xrow = d.row + (long long)slot * 256 * 1024;
  return hipSuccess;
}

// Workgroups of the one-launch attention that gave up waiting for their partners' scores, on the current device, since
// the library was loaded (waits for the device's work).
hipError_t ilt_k_attn_giveups(unsigned long long* out) {
  return hipMemcpyFromSymbol(out, HIP_SYMBOL(attn_giveups), sizeof(unsigned long long), 0, hipMemcpyDeviceToHost);
}

// One token at position pos: qk_rope and attention in two launches instead of three
hipError_t ilt_k_attn_step(const float* q, const float* k, const float* v, const float* qn, const float* kn, const float* rope, float* kc,
                           float* vc, float* out, int nh, int nkv, int hd, int rd, int pos, float eps, int neox, float* scratch, hipStream_t st) {
  if (hd % 16 || hd > 256 || rd > hd || (rd & 1) || nh % nkv || pos < 0 || pos >= 8192 || !scratch) return hipErrorInvalidValue;
  const int ctx = pos + 1, smax = (ctx + 3) & ~3, vpitch = ((ctx + 63) & ~63) + 4, nb = (ctx + 511) / 512;
  const float scale = 1.0f / sqrtf((float)hd);
  const size_t smem = sizeof(float) * ((size_t)smax + 16 * (size_t)vpitch);
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 0;
  // up to 1,024 positions, heads of 64 or 128: one launch ("ILT_ATTN_FUSED=0": the two launches below, for tests)
  static const bool fused_ok = []{ const char* f = getenv("ILT_ATTN_FUSED"); return !(f && f[0] == '0'); }();
  if (fused_ok && ctx <= 1024 && (hd == 64 || hd == 128)) {
    // 16 columns a workgroup: with 32, half as many workgroups read a head's keys, and the launch is no faster (each
    // workgroup takes as long over them: 9,000 cycles for 640 positions, its own loads and sums, not L2's bandwidth)
    static bool set[64] = {};
    if (!set[dev]) {
      hipError_t e = hipFuncSetAttribute((const void*)attn_step_fused_kernel<4, 16>, hipFuncAttributeMaxDynamicSharedMemorySize, 80 * 1024);
      if (e == hipSuccess) e = hipFuncSetAttribute((const void*)attn_step_fused_kernel<8, 16>, hipFuncAttributeMaxDynamicSharedMemorySize, 80 * 1024);
      if (e != hipSuccess) return e;
      set[dev] = true;
    }
    const size_t fsmem = sizeof(float) * (1024 + 16 * (size_t)vpitch);
    // A head's scores shared out over its workgroups where those run on one die: consecutive workgroups go to the
    // eight dies in turn and the kernel renumbers them so that a die takes nwg / 8 consecutive (head, slice) pairs.
    // "ILT_ATTN_SPLIT=0": never; "=2": every workgroup gives up waiting at once and takes all the scores (tests).
    const int ns = hd / 16, nwg = nh * ns;
    const char* sp = getenv("ILT_ATTN_SPLIT");
    const bool split = !(sp && sp[0] == '0') && (nwg & 7) == 0 && ((nwg >> 3) % ns) == 0 && nh <= 256 && ctx >= 64;
    const int patience = sp && sp[0] == '2' ? 0 : 20000;       // 200 us
    static std::atomic<unsigned> launches{0};
    const unsigned epoch = ++launches;
    unsigned* xgen = nullptr; unsigned long long* xrow = nullptr;
    if (split) {
      const hipError_t e = attn_exchange_of(dev, st, &xgen, &xrow);
      if (e != hipSuccess) return e;
    }
    if (hd == 64)
      hipLaunchKernelGGL((attn_step_fused_kernel<4, 16>), dim3(nwg), dim3(1024), fsmem, st, q, k, v, qn, kn, rope, kc, vc, out, nh, nkv, rd, pos, eps,
                         neox, scale, vpitch, split ? 1 : 0, epoch, patience, xgen, xrow);
    else
      hipLaunchKernelGGL((attn_step_fused_kernel<8, 16>), dim3(nwg), dim3(1024), fsmem, st, q, k, v, qn, kn, rope, kc, vc, out, nh, nkv, rd, pos, eps,
                         neox, scale, vpitch, split ? 1 : 0, epoch, patience, xgen, xrow);
    return hipGetLastError();
  }
  {
    const dim3 gs(nh, (ctx + 255) / 256);
    if (hd == 128)
      hipLaunchKernelGGL(attn_step_scores_kernel<8>, gs, dim3(1024), 0, st, q, k, v, qn, kn, rope, kc, vc, scratch, nh, nkv, hd, rd, pos, eps, neox, scale, smax);
    else if (hd == 64)
      hipLaunchKernelGGL(attn_step_scores_kernel<4>, gs, dim3(1024), 0, st, q, k, v, qn, kn, rope, kc, vc, scratch, nh, nkv, hd, rd, pos, eps, neox, scale, smax);
    else
      hipLaunchKernelGGL(attn_step_scores_kernel<0>, gs, dim3(1024), 0, st, q, k, v, qn, kn, rope, kc, vc, scratch, nh, nkv, hd, rd, pos, eps, neox, scale, smax);
  }
  // past the one-launch kernel's 1,024 positions the values come in tiles while the chains run (at 1,536 positions 523
  // tok/s at the Qwen3-4B shape against 493 with the whole slice brought into LDS first, at 1,990 500 against 464);
  // "ILT_ATTN_STREAM_FROM=2048": the whole slice first up to 2,048 positions (tests)
  static const int stream_from = []{ const char* f = getenv("ILT_ATTN_STREAM_FROM"); return f ? atoi(f) : 1024; }();
  if (ctx > stream_from || ctx > 2048) return launch_values_stream(dev, scratch, vc, out, nh, nkv, hd, pos, smax, st);
  hipError_t e = hipErrorInvalidValue;
#define ILT_ATTN1(NB)                                                                                                                         \
  if (nb == NB) {                                                                                                                             \
    static bool set[64] = {};                                                                                                                 \
    e = set[dev] ? hipSuccess                                                                                                                 \
                 : hipFuncSetAttribute((const void*)attn_values_kernel<1, NB>, hipFuncAttributeMaxDynamicSharedMemorySize, 152 * 1024);       \
    if (e == hipSuccess) {                                                                                                                    \
      set[dev] = true;                                                                                                                        \
      hipLaunchKernelGGL((attn_values_kernel<1, NB>), dim3(nh * (hd / 16), 1), dim3(256), smem, st, scratch, vc, out, nh, nkv, hd, pos, 1,    \
                         smax, vpitch);                                                                                                       \
      e = hipGetLastError();                                                                                                                  \
    }                                                                                                                                         \
  }
  ILT_ATTN1(1) ILT_ATTN1(2) ILT_ATTN1(3) ILT_ATTN1(4)
#undef ILT_ATTN1
  return e;
}

// scratch: 2048 bytes of the caller's for the workgroups' bests, or null (one workgroup then reads everything)
hipError_t ilt_k_argmax(const float* v, int n, int* out, void* scratch, hipStream_t st) {
  if (n <= 0) return hipErrorInvalidValue;
  const int nparts = scratch && n >= (1 << 15) ? 128 : 1;
  if (nparts == 1) {
    hipLaunchKernelGGL(argmax_part_kernel, dim3(1), dim3(1024), 0, st, v, n, (ArgBest*)nullptr, out);
  } else {
    hipLaunchKernelGGL(argmax_part_kernel, dim3(nparts), dim3(256), 0, st, v, n, (ArgBest*)scratch, out);
    hipLaunchKernelGGL(argmax_last_kernel, dim3(1), dim3(256), 0, st, v, (const ArgBest*)scratch, nparts, out);
  }
  return hipGetLastError();
}

hipError_t ilt_k_swiglu_rows(float* a, const float* b, long long n, hipStream_t st) {
  if (n <= 0) return hipSuccess;
  hipLaunchKernelGGL(swiglu_rows_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, a, b, n);
  return hipGetLastError();
}
