// Prefill products on the int8 matrix cores of gfx950, exact: Y[t][r] = W[r].x_t for many
// tokens, W in GGUF Q8_0 / Q4_K / Q6_K / Q2_K / IQ2_XXS blocks, activations quantized as
// the reference's CPU path quantizes them.  Each result has the bits the decode kernel
// gives for the same row and token, as the reference's MATMUL! does on the CPU
// (src/batch.lisp:10-12): v_mfma_i32_16x16x32_i8 forms each 32- (or 16-) weight group's
// integer dot for a 16x16 patch of (row, token) pairs, and the patch's owner lanes scale
// and add them, block after block, in the CPU kernels' expression order
// (tensor.lisp:329-336, kquant.lisp:180-236, iquant.lisp:138-215).
//
// A workgroup (256 threads, 4 waves) computes 64 rows x 64 tokens; per step it unpacks one
// 256-column slab of its 64 rows into int8 in LDS next to the tokens' quants; wave w owns
// rows 32*(w/2).. and tokens 32*(w%2).. as 2x2 MFMA patches.  The same body serves the
// grouped expert product (D4_MM_ID, src/cuda/ds4f_mm.cu:228-257): grid x then walks the
// 64-token tiles of every expert's rows in turn.
#include "ilt_device.h"
#include "ilt_iq2xxs_tables.h"
#include "ilt_kernels.h"
#include <stdlib.h>

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int TM = 64, TN = 64, KS = 256;   // rows, tokens, columns per step
constexpr int LDW = KS + 16;                // LDS row pitch in bytes

__device__ const u64 mm_grid_dev[256] = { ILT_IQ2XXS_GRID_VALUES };

struct Smem {
  i8 wt[TM * LDW];
  i8 xt[TN * LDW];
  // per-row scale data for the slab, transposed so four consecutive rows read as one word
  float wf[16 * TM];    // Q8_0: dw[g][row] (8 used); IQ2_XXS: 0.5+LS [ib][row]; others unused
  float wd[2 * TM];     // d[row], dmin[row]
  u8 wsc[16 * TM];      // integer scales [g][row]
  u8 wmn[16 * TM];      // integer mins [g][row]
  float xf[8 * TN];     // Q8_0: dx[g][tok]
  float xd[TN];         // Q8_K: yd[tok]
  int xbs[16 * TN];     // Q8_K: bsums [g16][tok]
  u64 grid[256];        // IQ2_XXS codebook
  int tile_z, tile_t0, tile_n;
  u32 scan[256];
};

template <int FMT> struct MF;
template <> struct MF<ILT_Q8_0>    { static constexpr int G = 32; };
template <> struct MF<ILT_Q4_K>    { static constexpr int G = 32; };
template <> struct MF<ILT_Q6_K>    { static constexpr int G = 16; };
template <> struct MF<ILT_Q2_K>    { static constexpr int G = 16; };
template <> struct MF<ILT_IQ2_XXS> { static constexpr int G = 32; };

__device__ __forceinline__ void st16(i8* p, int a, int b, int c, int d) { *(int4*)p = make_int4(a, b, c, d); }

// ---- unpack one 256-column slab of rows [r0, r0+64) into S.wt and the scale tables --------------
template <int FMT>
__device__ __forceinline__ void stage_w(Smem& S, const u8* __restrict__ w, const u16* __restrict__ wdq, long row_bytes,
                                        int rows, int r0, int sb, int cols) {
  const int t = threadIdx.x;
  if (FMT == ILT_Q8_0) {
    const int nb = cols >> 5;
    for (int c = t; c < TM * 16; c += 256) {
      const int row = c >> 4, kc = c & 15;
      int4 v = make_int4(0, 0, 0, 0);
      if (r0 + row < rows && sb * KS + 16 * kc < cols) v = *(const int4*)(w + (long)(r0 + row) * cols + sb * KS + 16 * kc);
      *(int4*)(S.wt + row * LDW + 16 * kc) = v;
    }
    for (int c = t; c < TM * 8; c += 256) {
      const int row = c & 63, g = c >> 6;
      S.wf[g * TM + row] = (r0 + row < rows && sb * 8 + g < nb) ? ilt_h2f(wdq[(long)(r0 + row) * nb + sb * 8 + g]) : 0.0f;
    }
  } else if (FMT == ILT_Q4_K) {
    const int row = t >> 2, k4 = t & 3;
    const bool live = r0 + row < rows;
    const u8* blk = w + (long)(live ? r0 + row : r0) * row_bytes + (long)sb * 144;
    const int4 hdr = *(const int4*)blk;
    const int4 a = *(const int4*)(blk + 16 + 32 * k4), b = *(const int4*)(blk + 32 + 32 * k4);
    const int m = live ? 0x0F0F0F0F : 0;
    i8* o = S.wt + row * LDW + 64 * k4;
    st16(o, a.x & m, a.y & m, a.z & m, a.w & m);
    st16(o + 16, b.x & m, b.y & m, b.z & m, b.w & m);
    st16(o + 32, ((u32)a.x >> 4) & m, ((u32)a.y >> 4) & m, ((u32)a.z >> 4) & m, ((u32)a.w >> 4) & m);
    st16(o + 48, ((u32)b.x >> 4) & m, ((u32)b.y >> 4) & m, ((u32)b.z >> 4) & m, ((u32)b.w >> 4) & m);
#pragma unroll
    for (int e = 0; e < 2; e++) {
      const int g = 2 * k4 + e, sh = 8 * (g & 3);
      const u32 x0 = ((u32)hdr.y >> sh) & 0xFF, x1 = ((u32)hdr.z >> sh) & 0xFF, x2 = ((u32)hdr.w >> sh) & 0xFF;
      const u32 sc = g < 4 ? (x0 & 63) : ((x2 & 0xF) | ((x0 >> 6) << 4));
      const u32 mn = g < 4 ? (x1 & 63) : ((x2 >> 4) | ((x1 >> 6) << 4));
      S.wsc[g * TM + row] = live ? (u8)sc : 0;
      S.wmn[g * TM + row] = live ? (u8)mn : 0;
    }
    if (k4 == 0) {
      S.wd[row] = live ? ilt_h2f((u16)(hdr.x & 0xFFFF)) : 0.0f;
      S.wd[TM + row] = live ? ilt_h2f((u16)((u32)hdr.x >> 16)) : 0.0f;
    }
  } else if (FMT == ILT_Q6_K) {
    const int row = t >> 2, c = (t >> 1) & 1, pp = t & 1;
    const bool live = r0 + row < rows;
    const u8* blk = w + (long)(live ? r0 + row : r0) * row_bytes + (long)sb * ILT_Q6K_STRIDE;
    const int m = live ? -1 : 0;
#pragma unroll
    for (int h = 0; h < 2; h++) {
      const int4 ql = ilt_ld16(blk + 64 * c + 32 * pp + 16 * h), qh = ilt_ld16(blk + 128 + 32 * c + 16 * h);
      const int s0 = 2 * pp, s1 = 2 * pp + 4;
      i8* lo = S.wt + row * LDW + 128 * c + 32 * pp + 16 * h;
      st16(lo, ((ql.x & 0x0F0F0F0F) | ((((u32)qh.x >> s0) & 0x03030303) << 4)) & m,
               ((ql.y & 0x0F0F0F0F) | ((((u32)qh.y >> s0) & 0x03030303) << 4)) & m,
               ((ql.z & 0x0F0F0F0F) | ((((u32)qh.z >> s0) & 0x03030303) << 4)) & m,
               ((ql.w & 0x0F0F0F0F) | ((((u32)qh.w >> s0) & 0x03030303) << 4)) & m);
      st16(lo + 64, ((((u32)ql.x >> 4) & 0x0F0F0F0F) | ((((u32)qh.x >> s1) & 0x03030303) << 4)) & m,
                    ((((u32)ql.y >> 4) & 0x0F0F0F0F) | ((((u32)qh.y >> s1) & 0x03030303) << 4)) & m,
                    ((((u32)ql.z >> 4) & 0x0F0F0F0F) | ((((u32)qh.z >> s1) & 0x03030303) << 4)) & m,
                    ((((u32)ql.w >> 4) & 0x0F0F0F0F) | ((((u32)qh.w >> s1) & 0x03030303) << 4)) & m);
    }
    const int q4 = t & 3;
#pragma unroll
    for (int e = 0; e < 4; e++) S.wsc[(4 * q4 + e) * TM + row] = live ? blk[192 + 4 * q4 + e] : 0;
    if (q4 == 0) S.wd[row] = live ? ilt_h2f(ilt_ld2(blk + 208)) : 0.0f;
  } else if (FMT == ILT_Q2_K) {
    const int row = t >> 2, h = (t >> 1) & 1, half = t & 1;
    const bool live = r0 + row < rows;
    const u8* blk = w + (long)(live ? r0 + row : r0) * row_bytes + (long)sb * 84;
    const int2 qa = ilt_ld8(blk + 16 + 32 * h + 16 * half), qb = ilt_ld8(blk + 24 + 32 * h + 16 * half);
    const int m = live ? 0x03030303 : 0;
#pragma unroll
    for (int k = 0; k < 4; k++)
      st16(S.wt + row * LDW + 128 * h + 32 * k + 16 * half, ((u32)qa.x >> (2 * k)) & m, ((u32)qa.y >> (2 * k)) & m,
           ((u32)qb.x >> (2 * k)) & m, ((u32)qb.y >> (2 * k)) & m);
    const int q4 = t & 3;
    const u32 sbw = ilt_ld4(blk + 4 * q4);
#pragma unroll
    for (int e = 0; e < 4; e++) {
      const u32 s = (sbw >> (8 * e)) & 0xFF;
      S.wsc[(4 * q4 + e) * TM + row] = live ? (u8)(s & 15) : 0;
      S.wmn[(4 * q4 + e) * TM + row] = live ? (u8)(s >> 4) : 0;
    }
    if (q4 == 0) {
      const u32 dd = ilt_ld4(blk + 80);
      S.wd[row] = live ? ilt_h2f((u16)(dd & 0xFFFF)) : 0.0f;
      S.wd[TM + row] = live ? ilt_h2f((u16)(dd >> 16)) : 0.0f;
    }
  } else {  // IQ2_XXS
#pragma unroll
    for (int u = 0; u < 2; u++) {
      const int unit = t + 256 * u, row = unit >> 3, ib = unit & 7;
      const bool live = r0 + row < rows;
      const u8* blk = w + (long)(live ? r0 + row : r0) * row_bytes + (long)sb * 66;
      const int2 sbk = ilt_ld8(blk + 2 + 8 * ib);
      const u32 g = (u32)sbk.x, aux = (u32)sbk.y;
      int o[8];
#pragma unroll
      for (int l = 0; l < 4; l++) {
        const uint2 mag = *(const uint2*)(S.grid + ((g >> (8 * l)) & 0xFF));
        u32 s = (aux >> (7 * l)) & 127;
        s |= (__popc(s) & 1) << 7;
        const u32 mlo = (((s & 0xF) * 0x00204081u) & 0x01010101u) * 0xFFu;
        const u32 mhi = (((s >> 4) * 0x00204081u) & 0x01010101u) * 0xFFu;
        // bytes are 8, 25 or 43: negating one never carries into the next
        o[2 * l] = live ? (int)((mag.x ^ mlo) + (mlo & 0x01010101u)) : 0;
        o[2 * l + 1] = live ? (int)((mag.y ^ mhi) + (mhi & 0x01010101u)) : 0;
      }
      st16(S.wt + row * LDW + 32 * ib, o[0], o[1], o[2], o[3]);
      st16(S.wt + row * LDW + 32 * ib + 16, o[4], o[5], o[6], o[7]);
      S.wf[ib * TM + row] = 0.5f + (float)(aux >> 28);
      if (ib == 0) S.wd[row] = live ? ilt_h2f(ilt_ld2(blk)) : 0.0f;
    }
  }
}

// ---- the tokens' quants for the slab: rows t0.. of the activation arrays -------------------------
template <int FMT>
__device__ __forceinline__ void stage_x(Smem& S, const i8* __restrict__ xq, const float* __restrict__ xs,
                                        const int* __restrict__ bsums, long t0, int ntok, int sb, int cols) {
  const int t = threadIdx.x;
  for (int c = t; c < TN * 16; c += 256) {
    const int tok = c >> 4, kc = c & 15;
    int4 v = make_int4(0, 0, 0, 0);
    if (tok < ntok && sb * KS + 16 * kc < cols) v = *(const int4*)(xq + (t0 + tok) * cols + sb * KS + 16 * kc);
    *(int4*)(S.xt + tok * LDW + 16 * kc) = v;
  }
  if (FMT == ILT_Q8_0) {
    const int nb = cols >> 5;
    for (int c = t; c < TN * 8; c += 256) {
      const int tok = c & 63, g = c >> 6;
      S.xf[g * TN + tok] = (tok < ntok && sb * 8 + g < nb) ? xs[(t0 + tok) * nb + sb * 8 + g] : 0.0f;
    }
  } else {
    const int nb = cols >> 8;
    if (t < TN) S.xd[t] = t < ntok ? xs[(t0 + t) * nb + sb] : 0.0f;
    if (FMT != ILT_IQ2_XXS)
      for (int c = t; c < TN * 16; c += 256) {
        const int tok = c >> 4, g = c & 15;
        S.xbs[g * TN + tok] = tok < ntok ? bsums[(t0 + tok) * (cols >> 4) + sb * 16 + g] : 0;
      }
  }
}

struct GemmParams {
  const u8* w; const u16* wdq;            // dense
  const u64* ptrs; long long add;         // grouped: expert z's matrix at ptrs[z] + add
  const u32* counts; const u32* bases; int ne;
  int rows, cols; long row_bytes;
  const i8* xq; const float* xs; const int* bsums;
  float* y; const float* bias; int acc; int ntok;
  long ldy;                               // floats from one token's results to the next token's
};

template <int FMT>
__global__ __launch_bounds__(256) void gemm_i8_kernel(GemmParams p) {
  __shared__ Smem S;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  // ---- which tokens: a dense tile, or tile blockIdx.x of the experts' rows taken in turn ----
  long tok0; int ntok; const u8* w = p.w;
  if (p.ptrs) {
    // inclusive scan of the experts' tile counts (ne <= 256: a thread an expert)
    S.scan[t] = t < p.ne ? (p.counts[t] + TN - 1) / TN : 0;
    __syncthreads();
    for (int off = 1; off < 256; off <<= 1) {
      const u32 v = t >= off ? S.scan[t - off] : 0;
      __syncthreads();
      S.scan[t] += v;
      __syncthreads();
    }
    if (t == 0) S.tile_z = -1;
    __syncthreads();
    if (t < p.ne) {
      const u32 incl = S.scan[t], tiles = (p.counts[t] + TN - 1) / TN, excl = incl - tiles;
      if (blockIdx.x >= excl && blockIdx.x < incl) {
        S.tile_z = t;
        S.tile_t0 = (int)(p.bases[t] + (blockIdx.x - excl) * TN);
        S.tile_n = (int)min((u32)TN, p.counts[t] - (blockIdx.x - excl) * TN);
      }
    }
    __syncthreads();
    if (S.tile_z < 0) return;
    tok0 = S.tile_t0; ntok = S.tile_n;
    w = (const u8*)(p.ptrs[S.tile_z] + p.add);
  } else {
    tok0 = (long)blockIdx.x * TN;
    ntok = min(TN, p.ntok - (int)tok0);
  }
  const int r0 = blockIdx.y * TM;
  if (FMT == ILT_IQ2_XXS) S.grid[t] = mm_grid_dev[t];

  const int wr = 32 * (wave >> 1), wt0 = 32 * (wave & 1);   // this wave's rows and tokens in the tile
  const int li = lane & 15, lq = lane >> 4;
  float sum[2][2][4];
#pragma unroll
  for (int a = 0; a < 2; a++)
#pragma unroll
    for (int b = 0; b < 2; b++)
#pragma unroll
      for (int r = 0; r < 4; r++) sum[a][b][r] = 0.0f;

  const int nslab = (p.cols + KS - 1) / KS;
  for (int sb = 0; sb < nslab; sb++) {
    __syncthreads();
    stage_w<FMT>(S, w, p.wdq, p.row_bytes, p.rows, r0, sb, p.cols);
    stage_x<FMT>(S, p.xq, p.xs, p.bsums, tok0, ntok, sb, p.cols);
    __syncthreads();

    int isum[2][2][4];
    float fa[2][2][4], fb[2][2][4];
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
      for (int b = 0; b < 2; b++)
#pragma unroll
        for (int r = 0; r < 4; r++) { isum[a][b][r] = 0; fa[a][b][r] = 0.0f; fb[a][b][r] = 0.0f; }

    const int ngroups = FMT == ILT_Q8_0 ? min(8, (p.cols - sb * KS) >> 5) : 8;
    for (int g = 0; g < ngroups; g++) {
      long af[2], bf[2];
#pragma unroll
      for (int a = 0; a < 2; a++) af[a] = *(const long*)(S.wt + (wr + 16 * a + li) * LDW + 32 * g + 8 * lq);
#pragma unroll
      for (int b = 0; b < 2; b++) bf[b] = *(const long*)(S.xt + (wt0 + 16 * b + li) * LDW + 32 * g + 8 * lq);
#pragma unroll
      for (int a = 0; a < 2; a++) {
        const int rb = wr + 16 * a + 4 * lq;      // this lane's four rows of the patch
#pragma unroll
        for (int b = 0; b < 2; b++) {
          const int tk = wt0 + 16 * b + li;       // and its token
          const v4i z = {0, 0, 0, 0};
          if (MF<FMT>::G == 32) {
            const v4i d = __builtin_amdgcn_mfma_i32_16x16x32_i8(af[a], bf[b], z, 0, 0, 0);
            if (FMT == ILT_Q8_0) {
              const float4 dw = *(const float4*)(S.wf + g * TM + rb);
              const float dx = S.xf[g * TN + tk];
              sum[a][b][0] = sum[a][b][0] + (float)d[0] * (dw.x * dx);
              sum[a][b][1] = sum[a][b][1] + (float)d[1] * (dw.y * dx);
              sum[a][b][2] = sum[a][b][2] + (float)d[2] * (dw.z * dx);
              sum[a][b][3] = sum[a][b][3] + (float)d[3] * (dw.w * dx);
            } else if (FMT == ILT_Q4_K) {
              const u32 sc = *(const u32*)(S.wsc + g * TM + rb);
#pragma unroll
              for (int r = 0; r < 4; r++) isum[a][b][r] += (int)((sc >> (8 * r)) & 0xFF) * d[r];
            } else {  // IQ2_XXS: even sub-blocks to one sum, odd to the other, each in order
              const float4 ls = *(const float4*)(S.wf + g * TM + rb);
              const float lsv[4] = {ls.x, ls.y, ls.z, ls.w};
#pragma unroll
              for (int r = 0; r < 4; r++) {
                const float term = (float)d[r] * lsv[r];
                if ((g & 1) == 0) fa[a][b][r] = fa[a][b][r] + term; else fb[a][b][r] = fb[a][b][r] + term;
              }
            }
          } else {
            // scales per 16 weights: the two halves of the group apart, by zeroing the other
            // half of the tokens' bytes (lanes 0-31 carry columns 0-15 of the group)
            const long blo = lq < 2 ? bf[b] : 0, bhi = lq < 2 ? 0 : bf[b];
            const v4i d0 = __builtin_amdgcn_mfma_i32_16x16x32_i8(af[a], blo, z, 0, 0, 0);
            const v4i d1 = __builtin_amdgcn_mfma_i32_16x16x32_i8(af[a], bhi, z, 0, 0, 0);
            const u32 s0 = *(const u32*)(S.wsc + (2 * g) * TM + rb), s1 = *(const u32*)(S.wsc + (2 * g + 1) * TM + rb);
#pragma unroll
            for (int r = 0; r < 4; r++) {
              if (FMT == ILT_Q6_K)
                isum[a][b][r] += (int)(i8)((s0 >> (8 * r)) & 0xFF) * d0[r] + (int)(i8)((s1 >> (8 * r)) & 0xFF) * d1[r];
              else
                isum[a][b][r] += (int)((s0 >> (8 * r)) & 0xFF) * d0[r] + (int)((s1 >> (8 * r)) & 0xFF) * d1[r];
            }
          }
        }
      }
    }
    // ---- the slab's block, combined as the CPU kernels combine it ----
    if (FMT != ILT_Q8_0) {
#pragma unroll
      for (int a = 0; a < 2; a++) {
        const int rb = wr + 16 * a + 4 * lq;
        const float4 dv = *(const float4*)(S.wd + rb), mv = *(const float4*)(S.wd + TM + rb);
        const float dd[4] = {dv.x, dv.y, dv.z, dv.w}, dm[4] = {mv.x, mv.y, mv.z, mv.w};
#pragma unroll
        for (int b = 0; b < 2; b++) {
          const int tk = wt0 + 16 * b + li;
          const float yd = S.xd[tk];
          if (FMT == ILT_IQ2_XXS) {
#pragma unroll
            for (int r = 0; r < 4; r++) sum[a][b][r] = sum[a][b][r] + (dd[r] * yd) * (fa[a][b][r] + fb[a][b][r]);
          } else {
            int im[4] = {0, 0, 0, 0};
            if (FMT == ILT_Q4_K) {
#pragma unroll
              for (int g = 0; g < 8; g++) {
                const u32 mn = *(const u32*)(S.wmn + g * TM + rb);
                const int bs = S.xbs[(2 * g) * TN + tk] + S.xbs[(2 * g + 1) * TN + tk];
#pragma unroll
                for (int r = 0; r < 4; r++) im[r] += (int)((mn >> (8 * r)) & 0xFF) * bs;
              }
#pragma unroll
              for (int r = 0; r < 4; r++) {
                sum[a][b][r] = sum[a][b][r] - (yd * dm[r]) * (float)im[r];
                sum[a][b][r] = sum[a][b][r] + (yd * dd[r]) * (float)isum[a][b][r];
              }
            } else if (FMT == ILT_Q6_K) {
#pragma unroll
              for (int g = 0; g < 16; g++) {
                const u32 sc = *(const u32*)(S.wsc + g * TM + rb);
                const int bs = S.xbs[g * TN + tk];
#pragma unroll
                for (int r = 0; r < 4; r++) im[r] += (int)(i8)((sc >> (8 * r)) & 0xFF) * bs;
              }
#pragma unroll
              for (int r = 0; r < 4; r++)
                sum[a][b][r] = sum[a][b][r] + (dd[r] * yd) * (float)(isum[a][b][r] - 32 * im[r]);
            } else {  // Q2_K
#pragma unroll
              for (int g = 0; g < 16; g++) {
                const u32 mn = *(const u32*)(S.wmn + g * TM + rb);
                const int bs = S.xbs[g * TN + tk];
#pragma unroll
                for (int r = 0; r < 4; r++) im[r] += (int)((mn >> (8 * r)) & 0xFF) * bs;
              }
#pragma unroll
              for (int r = 0; r < 4; r++) {
                sum[a][b][r] = sum[a][b][r] + ((-yd) * dm[r]) * (float)im[r];
                sum[a][b][r] = sum[a][b][r] + (yd * dd[r]) * (float)isum[a][b][r];
              }
            }
          }
        }
      }
    }
  }

  // ---- store: y[token][row] ----
#pragma unroll
  for (int a = 0; a < 2; a++) {
    const int row = r0 + wr + 16 * a + 4 * lq;
#pragma unroll
    for (int b = 0; b < 2; b++) {
      const int tk = wt0 + 16 * b + li;
      if (tk >= ntok) continue;
      float* yo = p.y + (tok0 + tk) * p.ldy + row;
#pragma unroll
      for (int r = 0; r < 4; r++) {
        if (row + r >= p.rows) continue;
        float v = sum[a][b][r];
        if (FMT == ILT_IQ2_XXS) v = 0.25f * v;
        if (p.bias) v = v + p.bias[row + r];
        if (p.acc) v = yo[r] + v;
        yo[r] = v;
      }
    }
  }
}

template <int FMT>
hipError_t launch_gemm(const GemmParams& p, unsigned tiles_x, hipStream_t st) {
  dim3 grid(tiles_x, (p.rows + TM - 1) / TM);
  hipLaunchKernelGGL(gemm_i8_kernel<FMT>, grid, dim3(256), 0, st, p);
  return hipGetLastError();
}

hipError_t dispatch(int fmt, const GemmParams& p, unsigned tiles_x, hipStream_t st) {
  switch (fmt) {
    case ILT_Q8_0: return launch_gemm<ILT_Q8_0>(p, tiles_x, st);
    case ILT_Q4_K: return launch_gemm<ILT_Q4_K>(p, tiles_x, st);
    case ILT_Q6_K: return launch_gemm<ILT_Q6_K>(p, tiles_x, st);
    case ILT_Q2_K: return launch_gemm<ILT_Q2_K>(p, tiles_x, st);
    case ILT_IQ2_XXS: return launch_gemm<ILT_IQ2_XXS>(p, tiles_x, st);
  }
  return hipErrorInvalidValue;
}

}  // namespace

hipError_t ilt_k_gemm_i8(int fmt, const uint8_t* w, const uint16_t* wd, long long row_bytes, int rows, int cols,
                         const int8_t* xq, const float* xs, const int* bsums, int ntok, float* y, const float* bias,
                         int acc, hipStream_t st, long long ldy) {
  if (ntok <= 0 || rows <= 0) return hipSuccess;
  if (ldy == 0) ldy = rows;
  if (ldy < rows) return hipErrorInvalidValue;
  // Q6_K, Q4_K and Q2_K with enough tokens and rows to fill 128 x 128 tiles: the pipelined kernel with scale * quant
  // as int8 planes, the same bits.  ILT_I8_PLANES (tests): "0" never, "1" whenever the format allows.
  const char* force = getenv("ILT_I8_PLANES");
  const int forced = force ? atoi(force) : -1;
  const bool fits = rows < (1 << 21) && ldy < (1 << 21) && (long long)rows * row_bytes < 0x7FFFFFFFLL;      // the pipelined kernels' 32-bit offsets
  if (fits && (fmt == ILT_Q6_K || fmt == ILT_Q4_K || fmt == ILT_Q2_K) && cols % 256 == 0 && forced != 0 && (forced == 1 || (ntok >= 96 && rows >= 128)))
    return ilt_k_gemm_i8_planes(fmt, w, row_bytes, rows, cols, xq, xs, bsums, ntok, y, bias, acc, st, ldy);
  if (fits && fmt == ILT_Q8_0 && cols % 64 == 0 && forced != 0 && (forced == 1 || (ntok >= 96 && rows >= 128)))
    return ilt_k_gemm_i8_q8(w, wd, rows, cols, xq, xs, ntok, y, bias, acc, st, ldy);
  GemmParams p = {};
  p.w = w; p.wdq = wd; p.rows = rows; p.cols = cols; p.row_bytes = row_bytes;
  p.xq = xq; p.xs = xs; p.bsums = bsums; p.y = y; p.bias = bias; p.acc = acc; p.ntok = ntok; p.ldy = (long)ldy;
  return dispatch(fmt, p, (unsigned)((ntok + TN - 1) / TN), st);
}

hipError_t ilt_k_gemm_i8_id(int fmt, const uint64_t* ptrs, long long add, const uint32_t* counts, const uint32_t* bases,
                            int ne, long long row_bytes, int rows, int cols, const int8_t* xq, const float* xs,
                            const int* bsums, long long total_rows, float* y, hipStream_t st) {
  if (total_rows <= 0 || rows <= 0 || ne <= 0) return hipSuccess;
  if (ne > 256) return hipErrorInvalidValue;
  {
    // the experts' IQ2_XXS and Q2_K (and Q4_K / Q6_K) matrices on the planes kernel when the groups average at least a quarter of a tile of 128 rows
    const char* force = getenv("ILT_I8_PLANES");
    const int forced = force ? atoi(force) : -1;
    if (rows < (1 << 21) && (long long)rows * row_bytes < 0x7FFFFFFFLL &&
        (fmt == ILT_Q6_K || fmt == ILT_Q4_K || fmt == ILT_Q2_K || fmt == ILT_IQ2_XXS) && cols % 256 == 0 && forced != 0 &&
        (forced == 1 || (total_rows >= 32LL * ne && rows >= 128)))
      return ilt_k_gemm_i8_planes_id(fmt, ptrs, add, counts, bases, ne, row_bytes, rows, cols, xq, xs, bsums, total_rows, y, st);
  }
  GemmParams p = {};
  p.ptrs = ptrs; p.add = add; p.counts = counts; p.bases = bases; p.ne = ne;
  p.rows = rows; p.cols = cols; p.row_bytes = row_bytes;
  p.xq = xq; p.xs = xs; p.bsums = bsums; p.y = y; p.ntok = (int)total_rows; p.ldy = rows;
  // sum over experts of ceil(count/64) <= total/64 + ne
  return dispatch(fmt, p, (unsigned)(total_rows / TN + ne), st);
}
