// Decode GEMV kernels for gfx950: y = W.x for W in GGUF Q8_0 / Q4_K / Q6_K / Q2_K /
// IQ2_XXS blocks, x already quantized as the reference's CPU path quantizes it
// (Q8_0 blocks for Q8_0 weights, Q8_K blocks for the rest).
//
// Every kernel has the same two phases.
//   A. A workgroup owns RW consecutive rows, i.e. one contiguous run of RW*S blocks
//      (S blocks per row).  Groups of LPB lanes walk that run block by block, so a
//      wave's loads cover consecutive bytes.  Each group forms the block's exact
//      integer sums (v_dot4_i32_i8, DPP adds) and one lane turns them into the
//      block's float terms, exactly as the CPU kernels do
//      (tensor.lisp:329-336, kquant.lisp:180-236, iquant.lisp:138-215), into LDS.
//   B. One lane per row adds its row's terms in block order: the CPU's sequential
//      sum, so the result has the CPU path's bits.
// The activations live in LDS for the whole workgroup.
#include "ilt_device.h"
#include "ilt_iq2xxs_tables.h"
#include "ilt_kernels.h"

namespace {

constexpr int kThreads = 256;

__device__ const u64 ilt_iq2xxs_grid_dev[256] = { ILT_IQ2XXS_GRID_VALUES };

template <int FMT> struct Fmt;
template <> struct Fmt<ILT_Q8_0>    { static constexpr int LPB = 2, TERMS = 1, BW = 32; };
template <> struct Fmt<ILT_Q4_K>    { static constexpr int LPB = 8, TERMS = 2, BW = 256; };
template <> struct Fmt<ILT_Q6_K>    { static constexpr int LPB = 8, TERMS = 1, BW = 256; };
template <> struct Fmt<ILT_Q2_K>    { static constexpr int LPB = 8, TERMS = 2, BW = 256; };
template <> struct Fmt<ILT_IQ2_XXS> { static constexpr int LPB = 8, TERMS = 1, BW = 256; };

struct Lds {
  const i8* xq;        // cols int8
  const float* xs;     // one scale per block (32 or 256 activations)
  const int* bsums;    // sums of 16 quants (Q8_K only)
  const u64* grid;     // IQ2_XXS codebook
  float* terms;
};

// ggml's get_scale_min_k4 on the 12 scale bytes held in three words.
__device__ __forceinline__ void scale_min_k4(int g, u32 s0, u32 s1, u32 s2, int& sc, int& m) {
  const int sh = 8 * (g & 3);
  const u32 a = (s0 >> sh) & 0xFF, b = (s1 >> sh) & 0xFF, c = (s2 >> sh) & 0xFF;
  if (g < 4) { sc = a & 63; m = b & 63; }
  else { sc = (c & 0xF) | ((a >> 6) << 4); m = (c >> 4) | ((b >> 6) << 4); }
}

__device__ __forceinline__ int4 and4(const int4& v, int m) { return make_int4(v.x & m, v.y & m, v.z & m, v.w & m); }
__device__ __forceinline__ int4 shr4(const int4& v, int n) {
  return make_int4((u32)v.x >> n, (u32)v.y >> n, (u32)v.z >> n, (u32)v.w >> n);
}

// ---- phase A, one block per group of LPB lanes ---------------------------------------------
template <int FMT> __device__ __forceinline__ void block_terms(const u8* w, const u16* wd, long f, int s, int j, const Lds& L);

template <> __device__ __forceinline__ void block_terms<ILT_Q8_0>(const u8* w, const u16* wd, long f, int s, int j, const Lds& L) {
  const int4 q = *(const int4*)(w + f * 32 + 16 * j);
  const int4 x = *(const int4*)(L.xq + s * 32 + 16 * j);
  const int acc = ilt_sum2(ilt_dot16(q, x, 0));
  if (j == 0) L.terms[f] = (float)acc * (ilt_h2f(wd[f]) * L.xs[s]);
}

template <> __device__ __forceinline__ void block_terms<ILT_Q4_K>(const u8* w, const u16*, long f, int s, int j, const Lds& L) {
  const u8* blk = w + f * 144;
  const int4 hdr = *(const int4*)blk;
  const int4 q = *(const int4*)(blk + 16 + 16 * j);
  const int k = j >> 1;
  const i8* xb = L.xq + s * 256 + 64 * k + 16 * (j & 1);
  const int lo = ilt_dot16(and4(q, 0x0F0F0F0F), *(const int4*)xb, 0);
  const int hi = ilt_dot16(and4(shr4(q, 4), 0x0F0F0F0F), *(const int4*)(xb + 32), 0);
  int sc0, sc1, m0, m1, mj, scj;
  scale_min_k4(2 * k, hdr.y, hdr.z, hdr.w, sc0, m0);
  scale_min_k4(2 * k + 1, hdr.y, hdr.z, hdr.w, sc1, m1);
  scale_min_k4(j, hdr.y, hdr.z, hdr.w, scj, mj);
  const int2 bs = *(const int2*)(L.bsums + s * 16 + 2 * j);
  const int isum = ilt_sum8(lo * sc0 + hi * sc1);
  const int imin = ilt_sum8(mj * (bs.x + bs.y));
  if (j == 0) {
    const float ydi = L.xs[s];
    const float d = ydi * ilt_h2f((u16)(hdr.x & 0xFFFF)), dmin = ydi * ilt_h2f((u16)((u32)hdr.x >> 16));
    L.terms[2 * f] = dmin * (float)imin;
    L.terms[2 * f + 1] = d * (float)isum;
  }
}

template <> __device__ __forceinline__ void block_terms<ILT_Q6_K>(const u8* w, const u16*, long f, int s, int j, const Lds& L) {
  const u8* blk = w + f * 210;
  const int c = j >> 2, isb = (j >> 1) & 1, l16 = j & 1;
  const int4 ql = ilt_ld16(blk + 64 * c + 32 * isb + 16 * l16);
  const int4 qh = ilt_ld16(blk + 128 + 32 * c + 16 * l16);
  const i8* sc = (const i8*)(blk + 192);
  const int sclo = sc[8 * c + 2 * isb + l16], schi = sc[8 * c + 4 + 2 * isb + l16];
  const int scA = sc[2 * j], scB = sc[2 * j + 1];
  const int4 hl = shr4(qh, 2 * isb), hh = shr4(qh, 4 + 2 * isb);
  int4 lo = and4(ql, 0x0F0F0F0F), hi = and4(shr4(ql, 4), 0x0F0F0F0F);
  lo.x |= (hl.x & 0x03030303) << 4; lo.y |= (hl.y & 0x03030303) << 4; lo.z |= (hl.z & 0x03030303) << 4; lo.w |= (hl.w & 0x03030303) << 4;
  hi.x |= (hh.x & 0x03030303) << 4; hi.y |= (hh.y & 0x03030303) << 4; hi.z |= (hh.z & 0x03030303) << 4; hi.w |= (hh.w & 0x03030303) << 4;
  const i8* xb = L.xq + s * 256 + 128 * c + 32 * isb + 16 * l16;
  const int dlo = ilt_dot16(lo, *(const int4*)xb, 0), dhi = ilt_dot16(hi, *(const int4*)(xb + 64), 0);
  const int2 bs = *(const int2*)(L.bsums + s * 16 + 2 * j);
  const int isum = ilt_sum8(dlo * sclo + dhi * schi);
  const int imins = ilt_sum8(bs.x * scA + bs.y * scB);
  if (j == 0) L.terms[f] = (ilt_h2f(ilt_ld2(blk + 208)) * L.xs[s]) * (float)(isum - 32 * imins);
}

template <> __device__ __forceinline__ void block_terms<ILT_Q2_K>(const u8* w, const u16*, long f, int s, int j, const Lds& L) {
  const u8* blk = w + f * 84;
  const int h = j >> 2, half = (j >> 1) & 1, lh = j & 1;
  const int2 q = ilt_ld8(blk + 16 + 32 * h + 16 * half + 8 * lh);
  const int2 sb = ilt_ld8(blk + 8 * h);
  const i8* xb = L.xq + s * 256 + 128 * h + 16 * half + 8 * lh;
  int isum = 0;
#pragma unroll
  for (int k = 0; k < 4; k++) {
    const int2 x = *(const int2*)(xb + 32 * k);
    const int dot = ilt_dot4(((u32)q.y >> (2 * k)) & 0x03030303, x.y, ilt_dot4(((u32)q.x >> (2 * k)) & 0x03030303, x.x, 0));
    const u32 sw = ((u32)(k < 2 ? sb.x : sb.y) >> (16 * (k & 1) + 8 * half)) & 0xF;
    isum += (int)sw * dot;
  }
  const u32 mb = ilt_ld2(blk + 2 * j);
  const int2 bs = *(const int2*)(L.bsums + s * 16 + 2 * j);
  const int mins = ilt_sum8((int)((mb >> 4) & 0xF) * bs.x + (int)(mb >> 12) * bs.y);
  isum = ilt_sum8(isum);
  if (j == 0) {
    const float ydb = L.xs[s];
    const u32 dd = ilt_ld4(blk + 80);
    const float d = ydb * ilt_h2f((u16)(dd & 0xFFFF)), dmin = (-ydb) * ilt_h2f((u16)(dd >> 16));
    L.terms[2 * f] = dmin * (float)mins;
    L.terms[2 * f + 1] = d * (float)isum;
  }
}

// One IQ2_XXS sub-block (32 weights): its integer dot with 32 activations.  The sign of
// weight i of an 8-group is bit i of the 7-bit pattern, bit 7 their parity; with m the
// bytes to negate, sum(sign*mag*x) = sum(mag*x) - 2*sum((mag&m)*x).
__device__ __forceinline__ int iq2xxs_sub_dot(u32 g, u32 aux, const i8* xb, const u64* grid) {
  int pos = 0, neg = 0;
#pragma unroll
  for (int l = 0; l < 4; l++) {
    const uint2 mag = *(const uint2*)(grid + ((g >> (8 * l)) & 0xFF));
    u32 s = (aux >> (7 * l)) & 127;
    s |= (__popc(s) & 1) << 7;
    const u32 mlo = (((s & 0xF) * 0x00204081u) & 0x01010101u) * 0xFFu;
    const u32 mhi = (((s >> 4) * 0x00204081u) & 0x01010101u) * 0xFFu;
    const int2 x = *(const int2*)(xb + 8 * l);
    pos = ilt_dot4((int)mag.y, x.y, ilt_dot4((int)mag.x, x.x, pos));
    neg = ilt_dot4((int)(mag.y & mhi), x.y, ilt_dot4((int)(mag.x & mlo), x.x, neg));
  }
  return pos - 2 * neg;
}

template <> __device__ __forceinline__ void block_terms<ILT_IQ2_XXS>(const u8* w, const u16*, long f, int s, int j, const Lds& L) {
  const u8* blk = w + f * 66;
  const int2 sb = ilt_ld8(blk + 2 + 8 * j);
  const u32 aux = (u32)sb.y;
  const int isum = iq2xxs_sub_dot((u32)sb.x, aux, L.xq + s * 256 + 32 * j, L.grid);
  const float term = (float)isum * (0.5f + (float)(aux >> 28));
  // lane 0 gathers the even sub-blocks' terms in order, lane 1 the odd ones'
  float a = 0.0f + term;
  a = a + ilt_dppf<ILT_DPP_SHL(2)>(term);
  a = a + ilt_dppf<ILT_DPP_SHL(4)>(term);
  a = a + ilt_dppf<ILT_DPP_SHL(6)>(term);
  const float b = ilt_dppf<ILT_DPP_SHL(1)>(a);
  if (j == 0) L.terms[f] = (ilt_h2f(ilt_ld2(blk)) * L.xs[s]) * (a + b);
}

// ---- phase B: a row's terms in block order -------------------------------------------------
template <int FMT> __device__ __forceinline__ float row_sum(const float* t, int S) {
  float sum = 0.0f;
  if (FMT == ILT_Q4_K) { for (int s = 0; s < S; s++) { sum = sum - t[2 * s]; sum = sum + t[2 * s + 1]; } }
  else if (FMT == ILT_Q2_K) { for (int s = 0; s < S; s++) { sum = sum + t[2 * s]; sum = sum + t[2 * s + 1]; } }
  else { for (int s = 0; s < S; s++) sum = sum + t[s]; }
  if (FMT == ILT_IQ2_XXS) sum = 0.25f * sum;
  return sum;
}

template <int FMT>
__global__ __launch_bounds__(kThreads) void gemv_kernel(IltGemvParams p) {
  using F = Fmt<FMT>;
  extern __shared__ __align__(16) unsigned char smem[];
  const int S = p.cols / F::BW;
  const int z = blockIdx.z;
  // LDS: xq | bsums | xs | (grid) | terms
  i8* lxq = (i8*)smem;
  int* lbs = (int*)(smem + p.cols);
  const int nbs = (FMT == ILT_Q8_0 || FMT == ILT_IQ2_XXS) ? 0 : p.cols / 16;
  float* lxs = (float*)(lbs + nbs);
  u64* lgrid = (u64*)(((uintptr_t)(lxs + S) + 7) & ~(uintptr_t)7);
  float* terms = (float*)(lgrid + (FMT == ILT_IQ2_XXS ? 256 : 0));

  const long xoff = (long)z * p.x_stride + (p.group_rows > 0 ? (long)(blockIdx.x * p.rw / p.group_rows) * p.cols : 0);
  const i8* gxq = p.xq + xoff;
  for (int i = threadIdx.x * 16; i < p.cols; i += kThreads * 16) *(int4*)(lxq + i) = *(const int4*)(gxq + i);
  for (int i = threadIdx.x; i < S; i += kThreads) lxs[i] = p.xs[xoff / F::BW + i];
  for (int i = threadIdx.x; i < nbs; i += kThreads) lbs[i] = p.bsums[xoff / 16 + i];
  if (FMT == ILT_IQ2_XXS) lgrid[threadIdx.x] = ilt_iq2xxs_grid_dev[threadIdx.x];
  __syncthreads();

  const int r0 = blockIdx.x * p.rw;
  const int nrows = min(p.rw, p.rows - r0);
  const u8* wbase = p.ptrs ? (const u8*)(p.ptrs[z] + p.add) : p.w;
  const u8* w = wbase + (long)r0 * p.row_bytes;
  const u16* wd = p.wd ? p.wd + (long)r0 * S : nullptr;
  const Lds L = { lxq, lxs, lbs, lgrid, terms };

  const int j = threadIdx.x % F::LPB;
  const int nblk = nrows * S;
  // whole groups stay together: every lane of a group sees the same f
  for (int f = threadIdx.x / F::LPB; f < nblk; f += kThreads / F::LPB)
    block_terms<FMT>(w, wd, f, f % S, j, L);
  __syncthreads();

  for (int r = threadIdx.x; r < nrows; r += kThreads) {
    float v = row_sum<FMT>(terms + (long)r * S * F::TERMS, S);
    const long o = (long)z * p.y_stride + r0 + r;
    if (p.bias) v = v + p.bias[r0 + r];
    if (p.acc) v = p.y[o] + v;
    p.y[o] = v;
  }
}

template <int FMT>
size_t gemv_smem(const IltGemvParams& p) {
  using F = Fmt<FMT>;
  const int S = p.cols / F::BW;
  size_t b = p.cols + 4 * S + ((FMT == ILT_Q8_0 || FMT == ILT_IQ2_XXS) ? 0 : p.cols / 16 * 4) + 8;
  if (FMT == ILT_IQ2_XXS) b += 2048;
  return b + (size_t)p.rw * S * F::TERMS * 4;
}

template <int FMT>
hipError_t launch(const IltGemvParams& p, int nz, hipStream_t st) {
  dim3 grid((p.rows + p.rw - 1) / p.rw, 1, nz);
  const size_t smem = gemv_smem<FMT>(p);
  hipLaunchKernelGGL(gemv_kernel<FMT>, grid, dim3(kThreads), smem, st, p);
  return hipGetLastError();
}

}  // namespace

// Rows per workgroup: enough workgroups to cover the chip several times over, but no
// more rows than LDS terms allow and at least 4 so the activations' staging is shared.
int ilt_gemv_pick_rw(int fmt, int rows, int cols, int nz) {
  const int bw = fmt == ILT_Q8_0 ? 32 : 256;
  const int S = cols / bw, terms = (fmt == ILT_Q4_K || fmt == ILT_Q2_K) ? 2 : 1;
  int rw = 32;
  while (rw > 4 && (long)((rows + rw - 1) / rw) * nz < 2048) rw >>= 1;
  while (rw > 1 && (size_t)rw * S * terms * 4 > 48 * 1024) rw >>= 1;
  return rw;
}

hipError_t ilt_gemv_launch(int fmt, const IltGemvParams& p, int nz, hipStream_t st) {
  switch (fmt) {
    case ILT_Q8_0: return launch<ILT_Q8_0>(p, nz, st);
    case ILT_Q4_K: return launch<ILT_Q4_K>(p, nz, st);
    case ILT_Q6_K: return launch<ILT_Q6_K>(p, nz, st);
    case ILT_Q2_K: return launch<ILT_Q2_K>(p, nz, st);
    case ILT_IQ2_XXS: return launch<ILT_IQ2_XXS>(p, nz, st);
  }
  return hipErrorInvalidValue;
}
