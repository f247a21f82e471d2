// The MoE expert path's small kernels for gfx950: routing, grouping (token, slot) rows
// by expert, the gather, the gated activation and the slot-ordered sums.  Names,
// argument meaning and results follow the reference's kernels
// (src/cuda/ds4f_chunk.cu:393-508, src/cuda/ds4f.cu:645-655, 902-910); the floats follow
// its CPU path (src/ds4f.lisp:248-254, 950-978, 1013-1036).
#include "ilt_device.h"
#include "ilt_kernels.h"
#include "ilt_route.h"

namespace {

template <int K>
__global__ __launch_bounds__(64 * ROUTE_WAVES) void route_kernel(int ntok, int ne, int nu, int hash, float scale, int has_bias,
                                                                 const float* __restrict__ logits, const float* __restrict__ bias,
                                                                 const int* __restrict__ tid2eid, const u32* __restrict__ tokens,
                                                                 u32* __restrict__ sel, float* __restrict__ wout) {
  __shared__ u32 s_idx[ROUTE_WAVES][64];
  __shared__ float s_sc[ROUTE_WAVES][64];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int t = blockIdx.x * ROUTE_WAVES + wv;
  if (t >= ntok) return;                                      // whole waves leave; no barrier below
  route_token<K>(lane, ne, nu, scale, logits + (long long)t * ne, has_bias ? bias + (has_bias == 2 ? (long long)t * ne : 0) : nullptr,
                 hash == 1 ? tid2eid + (long long)tokens[t] * nu : nullptr, sel + (long long)t * nu, wout + (long long)t * nu, s_idx[wv], s_sc[wv]);
}

__global__ void group_zero_kernel(int ne, u32* counts) {
  const int e = blockIdx.x * blockDim.x + threadIdx.x;
  if (e < ne) counts[e] = 0u;
}

// rank[row] = the row's place among its expert's rows.  The order inside an expert is
// whatever the atomics give; every later step goes through rmap/smap, so results do not
// depend on it.
// A workgroup counts its rows per expert in LDS first, then reserves each expert's run of
// places with one global atomic: a popular expert costs one atomic a workgroup, not one a row.
__global__ __launch_bounds__(256) void group_count_kernel(int n, int ne, const u32* __restrict__ sel, u32* counts, u32* __restrict__ rank) {
  __shared__ u32 h[1024];
  const int gid = blockIdx.x * blockDim.x + threadIdx.x;
  for (int e = threadIdx.x; e < ne; e += blockDim.x) h[e] = 0;
  __syncthreads();
  u32 e = 0, mine = 0;
  if (gid < n) { e = sel[gid]; mine = atomicAdd(&h[e], 1u); }
  __syncthreads();
  for (int x = threadIdx.x; x < ne; x += blockDim.x) {
    const u32 c = h[x];
    if (c) h[x] = atomicAdd(counts + x, c);       // now the first place of this workgroup's rows of expert x
  }
  __syncthreads();
  if (gid < n) rank[gid] = h[e] + mine;
}

// bases[e] = rows before expert e's.  One workgroup of 1024; ne <= 1024.
__global__ __launch_bounds__(1024) void group_scan_kernel(int ne, const u32* __restrict__ counts, u32* __restrict__ bases) {
  __shared__ u32 sh[1024];
  const int e = threadIdx.x;
  sh[e] = e < ne ? counts[e] : 0u;
  __syncthreads();
  for (int off = 1; off < 1024; off <<= 1) {
    const u32 v = e >= off ? sh[e - off] : 0u;
    __syncthreads();
    sh[e] += v;
    __syncthreads();
  }
  if (e < ne) bases[e] = sh[e] - counts[e];
}

__global__ void group_scatter_kernel(int n, int nu, const u32* __restrict__ sel, const u32* __restrict__ rank,
                                     const u32* __restrict__ bases, const float* __restrict__ w,
                                     u32* __restrict__ rmap, u32* __restrict__ smap, float* __restrict__ wrow) {
  const int gid = blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= n) return;
  const u32 row = bases[sel[gid]] + rank[gid];
  rmap[row] = gid / nu; smap[gid] = row; wrow[row] = w[gid];
}

// rexp[row] = the expert of grouped row `row` (row smap[i] is (token, slot) i's)
__global__ void rows_expert_kernel(int n, const u32* __restrict__ sel, const u32* __restrict__ smap, u32* __restrict__ rexp) {
  const int gid = blockIdx.x * blockDim.x + threadIdx.x;
  if (gid < n) rexp[smap[gid]] = sel[gid];
}

__global__ void gather_rows_kernel(int d, int nrows, const float* __restrict__ src, const u32* __restrict__ map,
                                   float* __restrict__ x) {
  const long long gid = ((long long)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (gid >= (long long)nrows * d) return;
  const int r = (int)(gid / d), j = (int)(gid % d);
  *(float4*)(x + gid) = *(const float4*)(src + (long long)map[r] * d + j);
}

// mid[r][j] = (silu(g) * u) * w[r], g and u clamped first when clamp > 1e-6
// (d4-routed!, ds4f.lisp:1016-1019); quantized to Q8_0 with a float scale as well when xq
// is given (the shared expert's down projection takes Q8_0 activations).
__global__ __launch_bounds__(256) void swiglu_w_kernel(long long total, int ff, float clamp, const float* __restrict__ g,
                                                       const float* __restrict__ u, const float* __restrict__ w,
                                                       float* __restrict__ mid, i8* __restrict__ xq, float* __restrict__ xs) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  const bool live = i < total;
  float v = 0.0f;
  if (live) {
    float gv = g[i], uv = u[i];
    if (clamp > 1e-6f) { gv = fminf(gv, clamp); uv = fmaxf(-clamp, fminf(uv, clamp)); }
    v = (ilt_silu(gv) * uv) * w[i / ff];
    mid[i] = v;
  }
  if (xq) {
    float amax = ilt_max16(fabsf(v));
    amax = fmaxf(amax, __shfl_xor(amax, 16));
    const float d = amax / 127.0f;
    const float id = d == 0.0f ? 0.0f : 1.0f / d;
    if (live) {
      xq[i] = (i8)(int)rintf(v * id);
      if ((threadIdx.x & 31) == 0) xs[i >> 5] = d;
    }
  }
}

// The same gated activation rounded to bf16 (nearest even), for the bf16 grouped product: 8 values a thread.
__global__ __launch_bounds__(256) void swiglu_w_bf16_kernel(long long total8, int ff, float clamp, const float* __restrict__ g,
                                                            const float* __restrict__ u, const float* __restrict__ w,
                                                            u16* __restrict__ mid) {
  typedef float v2f __attribute__((ext_vector_type(2)));
  typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= total8) return;
  const float4 g0 = ((const float4*)g)[2 * i], g1 = ((const float4*)g)[2 * i + 1];
  const float4 u0 = ((const float4*)u)[2 * i], u1 = ((const float4*)u)[2 * i + 1];
  const float wv = w[(8 * i) / ff];            // ff is a multiple of 8: the eight values share a row
  float gv[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w}, uv[8] = {u0.x, u0.y, u0.z, u0.w, u1.x, u1.y, u1.z, u1.w};
  u32 pk[4];
#pragma unroll
  for (int k = 0; k < 4; k++) {
    float o[2];
#pragma unroll
    for (int h = 0; h < 2; h++) {
      float a = gv[2 * k + h], b = uv[2 * k + h];
      if (clamp > 1e-6f) { a = fminf(a, clamp); b = fmaxf(-clamp, fminf(b, clamp)); }
      o[h] = (ilt_silu(a) * b) * wv;
    }
    const v2f v = {o[0], o[1]};
    const v2bf r = __builtin_convertvector(v, v2bf);
    __builtin_memcpy(&pk[k], &r, 4);
  }
  ((int4*)mid)[i] = make_int4(pk[0], pk[1], pk[2], pk[3]);
}

__global__ void moe_sum_kernel(int d, int k, const float* __restrict__ down, const float* __restrict__ shared_,
                               float* __restrict__ moe, const u32* __restrict__ perm) {
  const int r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= d) return;
  float acc = 0.0f;
  for (int i = 0; i < k; i++) acc = acc + down[(long long)(perm ? perm[i] : i) * d + r];
  moe[r] = shared_ ? acc + shared_[r] : acc;
}

// Four columns a thread (16-byte loads); the slots are added in order, all loads sent first.
__global__ __launch_bounds__(256) void moe_sum_rows_kernel(int d, int nu, int ntok, const float* __restrict__ down, const u32* __restrict__ map,
                                                           const float* __restrict__ shared_, float* __restrict__ moe) {
  const long long gid = ((long long)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (gid >= (long long)ntok * d) return;
  const int t = (int)(gid / d), j = (int)(gid % d);
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int s0 = 0; s0 < nu; s0 += 8) {
    float4 v[8];
#pragma unroll
    for (int s = 0; s < 8; s++)
      if (s0 + s < nu) v[s] = *(const float4*)(down + (long long)map[(long long)t * nu + s0 + s] * d + j);
#pragma unroll
    for (int s = 0; s < 8; s++)
      if (s0 + s < nu) { acc.x = acc.x + v[s].x; acc.y = acc.y + v[s].y; acc.z = acc.z + v[s].z; acc.w = acc.w + v[s].w; }
  }
  if (shared_) {
    const float4 sh = *(const float4*)(shared_ + gid);
    acc.x = acc.x + sh.x; acc.y = acc.y + sh.y; acc.z = acc.z + sh.z; acc.w = acc.w + sh.w;
  }
  *(float4*)(moe + gid) = acc;
}

}  // namespace

hipError_t ilt_k_route(int ne, int nu, int hash, float scale, int has_bias, const float* logits, const float* bias,
                       const int* tid2eid, const uint32_t* tokens, uint32_t* sel, float* wout, int ntok, hipStream_t st) {
  if (ntok <= 0) return hipSuccess;
  if (ne < 1 || ne > 1024 || nu < 1 || nu > ne || nu > 64 || hash < 0 || hash > 1) return hipErrorInvalidValue;
  if (hash == 1 && (!tid2eid || !tokens)) return hipErrorInvalidValue;
  const dim3 grid((ntok + ROUTE_WAVES - 1) / ROUTE_WAVES), block(64 * ROUTE_WAVES);
#define ROUTE_LAUNCH(K) hipLaunchKernelGGL(route_kernel<K>, grid, block, 0, st, ntok, ne, nu, hash, scale, has_bias, logits, bias, \
                                           tid2eid, tokens, sel, wout)
  const int k = (ne + 63) / 64;
  if (k <= 1) ROUTE_LAUNCH(1); else if (k <= 2) ROUTE_LAUNCH(2); else if (k <= 4) ROUTE_LAUNCH(4);
  else if (k <= 8) ROUTE_LAUNCH(8); else ROUTE_LAUNCH(16);
#undef ROUTE_LAUNCH
  return hipGetLastError();
}

hipError_t ilt_k_group_zero(int ne, uint32_t* counts, hipStream_t st) {
  hipLaunchKernelGGL(group_zero_kernel, dim3((ne + 255) / 256), dim3(256), 0, st, ne, counts);
  return hipGetLastError();
}

hipError_t ilt_k_group_count(int n, int ne, int nu, const uint32_t* sel, uint32_t* counts, uint32_t* rank, hipStream_t st) {
  if (n <= 0) return hipSuccess;
  if (ne < 1 || ne > 1024) return hipErrorInvalidValue;
  hipLaunchKernelGGL(group_count_kernel, dim3((n + 255) / 256), dim3(256), 0, st, n, ne, sel, counts, rank);
  return hipGetLastError();
}

hipError_t ilt_k_group_scan(int n, int ne, int nu, const uint32_t* counts, uint32_t* bases, hipStream_t st) {
  if (ne > 1024) return hipErrorInvalidValue;
  hipLaunchKernelGGL(group_scan_kernel, dim3(1), dim3(1024), 0, st, ne, counts, bases);
  return hipGetLastError();
}

hipError_t ilt_k_group_scatter(int n, int ne, int nu, const uint32_t* sel, const uint32_t* rank, const uint32_t* bases,
                               const float* w, uint32_t* rmap, uint32_t* smap, float* wrow, hipStream_t st) {
  if (n <= 0) return hipSuccess;
  hipLaunchKernelGGL(group_scatter_kernel, dim3((n + 255) / 256), dim3(256), 0, st, n, nu, sel, rank, bases, w, rmap, smap, wrow);
  return hipGetLastError();
}

hipError_t ilt_k_rows_expert(int n, const uint32_t* sel, const uint32_t* smap, uint32_t* rexp, hipStream_t st) {
  if (n <= 0) return hipSuccess;
  hipLaunchKernelGGL(rows_expert_kernel, dim3((n + 255) / 256), dim3(256), 0, st, n, sel, smap, rexp);
  return hipGetLastError();
}

hipError_t ilt_k_gather_rows(int d, int nrows, const float* src, const uint32_t* map, float* x, hipStream_t st) {
  if (nrows <= 0) return hipSuccess;
  if (d % 4) return hipErrorInvalidValue;
  const long long n4 = (long long)nrows * d / 4;
  hipLaunchKernelGGL(gather_rows_kernel, dim3((unsigned)((n4 + 255) / 256)), dim3(256), 0, st, d, nrows, src, map, x);
  return hipGetLastError();
}

hipError_t ilt_k_swiglu_w(int n, int ff, float clamp, const float* g, const float* u, const float* w, float* mid,
                          int8_t* xq, float* xs, hipStream_t st) {
  const long long total = (long long)n * ff;
  if (total <= 0) return hipSuccess;
  if (xq && (total % 32)) return hipErrorInvalidValue;
  hipLaunchKernelGGL(swiglu_w_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, total, ff, clamp, g, u, w, mid, xq, xs);
  return hipGetLastError();
}

hipError_t ilt_k_swiglu_w_bf16(int n, int ff, float clamp, const float* g, const float* u, const float* w, uint16_t* mid, hipStream_t st) {
  const long long total = (long long)n * ff;
  if (total <= 0) return hipSuccess;
  if (ff % 8) return hipErrorInvalidValue;
  hipLaunchKernelGGL(swiglu_w_bf16_kernel, dim3((unsigned)((total / 8 + 255) / 256)), dim3(256), 0, st, total / 8, ff, clamp, g, u, w, mid);
  return hipGetLastError();
}

hipError_t ilt_k_moe_sum(int d, int k, const float* down, const float* shared_, float* moe, const uint32_t* perm, hipStream_t st) {
  hipLaunchKernelGGL(moe_sum_kernel, dim3((d + 255) / 256), dim3(256), 0, st, d, k, down, shared_, moe, perm);
  return hipGetLastError();
}

hipError_t ilt_k_moe_sum_rows(int d, int nu, int ntok, const float* down, const uint32_t* map, const float* shared_,
                              float* moe, hipStream_t st) {
  const long long n = (long long)ntok * d;
  if (n <= 0) return hipSuccess;
  if (d % 4) return hipErrorInvalidValue;
  hipLaunchKernelGGL(moe_sum_rows_kernel, dim3((unsigned)((n / 4 + 255) / 256)), dim3(256), 0, st, d, nu, ntok, down, map, shared_, moe);
  return hipGetLastError();
}
