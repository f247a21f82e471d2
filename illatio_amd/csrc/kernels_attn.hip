// What a dense decoder layer needs between its quantized products, for the harness that runs
// the whole forward pass (the reference's cuda-forward-n, src/cuda-dense.lisp:380-432): the Q/K
// head norms, RoPE and the KV caches' update (qk_rope, src/cuda/dense.cu:318-362), attention, and
// swiglu! on rows.  The floats follow the reference's CPU path (src/model.lisp:205-334, 364-378)
// operation for operation and sum for sum, so a token's logits have the CPU path's bits; speed is
// not the point of these kernels (the reference's CUDA attention splits the keys and lets the
// partial sums meet in its own order, dense.cu:364-373).
#include "ilt_device.h"
#include "ilt_kernels.h"

namespace {

// qk_rope: a workgroup (one wave) a head of a token.  rmsnorm! of the head when its weights are given
// (model.lisp:205-216: the squares, rounded to floats, added in double one after another), rope-head!
// from the position's table (cos, then sin, rd/2 each), K and V into the caches at pos0 + t.
__global__ __launch_bounds__(64) void qk_rope_kernel(float* __restrict__ q, float* __restrict__ k, const float* __restrict__ v,
                                                     const float* __restrict__ qn, const float* __restrict__ kn,
                                                     const float* __restrict__ rope, float* __restrict__ kc, float* __restrict__ vc,
                                                     int nh, int nkv, int hd, int rd, int pos0, float eps, int neox) {
  __shared__ float xs[512];
  __shared__ float sc;
  const int head = blockIdx.x, t = blockIdx.y, i = threadIdx.x, half = rd >> 1;
  const int pos = pos0 + t;
  const int qd = nh * hd, kvd = nkv * hd;
  const bool isq = head < nh;
  float* x = isq ? q + (long long)t * qd + head * hd : k + (long long)t * kvd + (head - nh) * hd;
  const float* nw = isq ? qn : kn;
  for (int j = i; j < hd; j += 64) xs[j] = x[j];
  __syncthreads();
  if (nw) {
    if (i == 0) {
      double s = 0.0;
      for (int j = 0; j < hd; j++) { const float sq = xs[j] * xs[j]; s += (double)sq; }
      sc = 1.0f / sqrtf((float)(s / (double)hd + (double)eps));
    }
    __syncthreads();
    const float scale = sc;
    for (int j = i; j < hd; j += 64) xs[j] = (xs[j] * scale) * nw[j];
    __syncthreads();
  }
  const float* cs = rope + (long long)pos * rd;
  for (int p = i; p < half; p += 64) {
    const int a = neox ? p : 2 * p, b = neox ? p + half : 2 * p + 1;
    const float x0 = xs[a], x1 = xs[b], c = cs[p], s = cs[half + p];
    xs[a] = x0 * c - x1 * s;                       // (no contraction: each product rounds on its own)
    xs[b] = x0 * s + x1 * c;
  }
  __syncthreads();
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
// another as the CPU adds them; then out += score * V row, position after position, an output column a thread.
__global__ __launch_bounds__(256) void attn_rows_kernel(const float* __restrict__ q, const float* __restrict__ kc, const float* __restrict__ vc,
                                                        float* __restrict__ out, int nh, int nkv, int hd, int pos0, float scale) {
  extern __shared__ float scores[];                // npos floats
  __shared__ float redf[4];
  __shared__ double redd[4];
  const int h = blockIdx.x, t = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int npos = pos0 + t + 1;
  const int group = nh / nkv, kvd = nkv * hd, ko = (h / group) * hd;
  const float* qh = q + ((long long)t * nh + h) * hd;
  const int l = tid & 15, pg = tid >> 4;           // 16 positions at a time
  const int nj = hd >> 4;                          // terms a partial sum (hd <= 256: at most 16)
  float qv[16];
#pragma unroll
  for (int j = 0; j < 16; j++) qv[j] = j < nj ? qh[l + 16 * j] : 0.0f;
  float mx = -3.402823466e38f;
  for (int p0 = 0; p0 < npos; p0 += 16) {
    const int p = p0 + pg;
    const float* kr = kc + (long long)min(p, npos - 1) * kvd + ko;
    float s = 0.0f;
#pragma unroll
    for (int j = 0; j < 16; j++) if (j < nj) s = s + kr[l + 16 * j] * qv[j];
    s = s + ilt_dppf<ILT_DPP_SHL(4)>(s);
    s = s + ilt_dppf<ILT_DPP_SHL(8)>(s);
    s = s + ilt_dppf<ILT_DPP_SHL(1)>(s);
    s = s + ilt_dppf<ILT_DPP_SHL(2)>(s);
    if (l == 0 && p < npos) { const float sv = s * scale; scores[p] = sv; mx = fmaxf(mx, sv); }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
  if (lane == 0) redf[wave] = mx;
  __syncthreads();
  mx = fmaxf(fmaxf(redf[0], redf[1]), fmaxf(redf[2], redf[3]));
  double part = 0.0;
  for (int p = tid; p < npos; p += 256) { const float e = ilt_expf_via_double(scores[p] - mx); scores[p] = e; part += (double)e; }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) part += __shfl_xor(part, off);
  if (lane == 0) redd[wave] = part;
  __syncthreads();
  double sum = (redd[0] + redd[1]) + (redd[2] + redd[3]);
  const double slack = sum * ((double)(npos + 8) * 0x1p-51);
  if ((float)(1.0 / (sum - slack)) != (float)(1.0 / (sum + slack))) {      // the same in every thread
    __syncthreads();
    if (tid == 0) { double s2 = 0.0; for (int p = 0; p < npos; p++) s2 += (double)scores[p]; redd[0] = s2; }
    __syncthreads();
    sum = redd[0];
  }
  const float inv = (float)(1.0 / sum);
  __syncthreads();
  for (int p = tid; p < npos; p += 256) scores[p] = scores[p] * inv;
  __syncthreads();
  if (tid < hd) {
    const float* vr = vc + ko + tid;
    float o = 0.0f;
    int p = 0;
    for (; p + 8 <= npos; p += 8) {
      float vv[8];
#pragma unroll
      for (int u = 0; u < 8; u++) vv[u] = vr[(long long)(p + u) * kvd];
#pragma unroll
      for (int u = 0; u < 8; u++) o = o + scores[p + u] * vv[u];
    }
    for (; p < npos; p++) o = o + scores[p] * vr[(long long)p * kvd];
    out[((long long)t * nh + h) * hd + tid] = o;
  }
}

// swiglu! (model.lisp:364-378) on n values: a = (a / (1 + e^-a)) * b, the exponential through double
__global__ __launch_bounds__(256) void swiglu_rows_kernel(float* __restrict__ a, const float* __restrict__ b, long long n) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i < n) { const float g = a[i]; a[i] = (g / (1.0f + ilt_expf_via_double(-g))) * b[i]; }
}

}  // namespace

hipError_t ilt_k_qk_rope(float* q, float* k, const float* v, const float* qn, const float* kn, const float* rope, float* kc, float* vc,
                         int nh, int nkv, int hd, int rd, int pos0, float eps, int neox, int ntok, hipStream_t st) {
  if (ntok <= 0) return hipSuccess;
  if (hd > 512 || hd < 2 || rd > hd || (rd & 1) || nh < 1 || nkv < 1) return hipErrorInvalidValue;
  hipLaunchKernelGGL(qk_rope_kernel, dim3(nh + nkv, ntok), dim3(64), 0, st, q, k, v, qn, kn, rope, kc, vc, nh, nkv, hd, rd, pos0, eps, neox);
  return hipGetLastError();
}

hipError_t ilt_k_attn_rows(const float* q, const float* kc, const float* vc, float* out, int nh, int nkv, int hd, int pos0, int ntok,
                           hipStream_t st) {
  if (ntok <= 0) return hipSuccess;
  if (hd % 16 || hd > 256 || nh % nkv || pos0 < 0 || pos0 + ntok > 15000) return hipErrorInvalidValue;      // the scores of a query sit in LDS
  const float scale = 1.0f / sqrtf((float)hd);
  hipLaunchKernelGGL(attn_rows_kernel, dim3(nh, ntok), dim3(256), sizeof(float) * (size_t)(pos0 + ntok), st, q, kc, vc, out, nh, nkv, hd, pos0, scale);
  return hipGetLastError();
}

hipError_t ilt_k_swiglu_rows(float* a, const float* b, long long n, hipStream_t st) {
  if (n <= 0) return hipSuccess;
  hipLaunchKernelGGL(swiglu_rows_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, a, b, n);
  return hipGetLastError();
}
