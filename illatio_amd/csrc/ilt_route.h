// d4-route for one token by one wave (src/ds4f.lisp:950-978), shared by the routing kernel and by the launch that
// carries a token's routing along (the shared expert's gate/up product of a decode step).
#pragma once
#include "ilt_device.h"

namespace {

__device__ __forceinline__ float softplus(float x) {
  if (x > 20.0f) return x;
  if (x < -20.0f) return ilt_expf_via_double(x);
  return ilt_logf_via_double(1.0f + ilt_expf_via_double(x));
}

// d4-route (ds4f.lisp:950-978): p = sqrt(softplus(logit)); the top NU of p (+ bias), the
// earlier expert first of equal ones; weights p/sum(p)*scale with the sum taken in slot order
// and floored at 2^-14.  hash 1: the experts come from tid2eid[token].
//
// A wave a token, K experts a lane (expert k*64 + lane), everything in registers.  A round
// picks one expert: each lane's best remaining score as an order-preserving integer key
// (0 = nothing left), the wave's largest key, then the smallest expert index among the lanes
// that hold it; the winning lane strikes its expert off a bit mask.  Lane j keeps slot j.
// Scores that are NaN (an overflow upstream) compare false both ways in the CPU's insertion,
// whose result then depends on the order of the insertions: such a token takes the slow
// branch, one lane doing the CPU's insertion as it is written, so that sel always holds NU
// different experts below NE, which the kernels downstream index tables with.
#define ROUTE_WAVES 4

__device__ __forceinline__ u32 wave_max_u32(u32 v) {
  v = max(v, (u32)ilt_dpp<ILT_DPP_XOR1>((int)v));
  v = max(v, (u32)ilt_dpp<ILT_DPP_XOR2>((int)v));
  v = max(v, (u32)ilt_dpp<ILT_DPP_HALF_MIRROR>((int)v));
  v = max(v, (u32)ilt_dpp<ILT_DPP_ROW_MIRROR>((int)v));
  const u32 a = __builtin_amdgcn_readlane(v, 0), b = __builtin_amdgcn_readlane(v, 16);
  const u32 c = __builtin_amdgcn_readlane(v, 32), d = __builtin_amdgcn_readlane(v, 48);
  return max(max(a, b), max(c, d));
}

__device__ __forceinline__ float route_prob(float logit) { return sqrtf(softplus(logit)); }

// One token by one wave (all 64 lanes active): lg its ne logits, bs its bias or null, eids its nu experts when they
// come from a table (hash layers) or null; sel and wout its nu slots; s_idx and s_sc 64 entries of LDS of this wave's.
// PRE: the lane's K logits (expert k*64 + lane) and biases were read beforehand, into plg and pbs.
template <int K, bool PRE = false>
__device__ __forceinline__ void route_token(int lane, int ne, int nu, float scale, const float* __restrict__ lg, const float* __restrict__ bs,
                                            const int* __restrict__ eids, u32* __restrict__ sel, float* __restrict__ wout, u32* s_idx, float* s_sc,
                                            const float* plg = nullptr, const float* pbs = nullptr) {
  u32 my_sel = 0;
  float my_p = 0.0f;
  if (eids) {
    if (lane < nu) {
      // A table entry names an expert below ne in every model file; the reference's CPU path indexes probs with it
      // unchecked (an array-bounds error in Lisp, whatever lies behind the array in its CUDA kernel).  Here an entry
      // from outside is brought inside, so that neither this read nor a later launch's slot table is indexed out of
      // bounds; entries below ne pass unchanged.
      const u32 e = min((u32)eids[lane], (u32)(ne - 1));
      my_sel = e;
      my_p = route_prob(lg[e]);
    }
  } else {
    float p[K], sc[K];
    u32 left = 0;                                             // bit k: expert k*64 + lane can still be picked
    bool nan = false;
#pragma unroll
    for (int k = 0; k < K; k++) {
      const int e = k * 64 + lane;
      p[k] = 0.0f; sc[k] = 0.0f;
      if (e < ne) {
        p[k] = route_prob(PRE ? plg[k] : lg[e]);
        sc[k] = (bs ? p[k] + (PRE ? pbs[k] : bs[e]) : p[k]) + 0.0f;      // + 0: no minus zero, which the integer key would rank below zero
        left |= 1u << k;
        nan |= sc[k] != sc[k];
      }
    }
    if (__builtin_amdgcn_ballot_w64(nan) == 0) {
      for (int j = 0; j < nu; j++) {
        u32 key = 0; int bk = 0;
#pragma unroll
        for (int k = 0; k < K; k++) {
          const u32 b = __float_as_uint(sc[k]);
          const u32 ord = (b & 0x80000000u) ? ~b : (b | 0x80000000u);      // > 0 for every number, -inf included
          if (((left >> k) & 1u) && ord > key) { key = ord; bk = k; }      // strict: the lane's earliest expert of equal ones
        }
        const u32 top = wave_max_u32(key);
        const u32 cand = (key == top && key != 0) ? (u32)(bk * 64 + lane) : 0xFFFFFFFFu;
        const u32 e = ~wave_max_u32(~cand);                                // the smallest index holding the top score
        const int wl = (int)(e & 63u);
        float pe = 0.0f;
#pragma unroll
        for (int k = 0; k < K; k++) if ((int)(e >> 6) == k) pe = p[k];
        pe = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, pe), wl));
        if (lane == wl) left &= ~(1u << (e >> 6));
        if (lane == j) { my_sel = e; my_p = pe; }
      }
    } else {
      // the CPU's insertion, verbatim, by one lane (slots fill from the left, so "empty" is j >= cnt)
      if (lane == 0) {
        int cnt = 0;
        for (int i = 0; i < ne; i++) {
          const float pi = route_prob(lg[i]);
          const float si = bs ? pi + bs[i] : pi;
          for (int j = 0; j < nu; j++) {
            if (j >= cnt || si > s_sc[j]) {
              for (int k = min(cnt, nu - 1); k > j; k--) { s_sc[k] = s_sc[k - 1]; s_idx[k] = s_idx[k - 1]; }
              s_sc[j] = si; s_idx[j] = (u32)i;
              if (cnt < nu) cnt++;
              break;
            }
          }
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      if (lane < nu) { my_sel = s_idx[lane]; my_p = route_prob(lg[my_sel]); }
    }
  }
  float sum = 0.0f;
  for (int j = 0; j < nu; j++) sum = sum + __shfl(my_p, j);   // in slot order, as the CPU adds them
  if (sum < 6.103515625e-5f) sum = 6.103515625e-5f;
  if (lane < nu) {
    sel[lane] = my_sel;
    wout[lane] = (my_p / sum) * scale;
  }
}

}  // namespace
