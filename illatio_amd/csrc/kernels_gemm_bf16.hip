// Prefill products on the bf16 matrix cores of gfx950: Y[t][r] = W[r].x_t for many tokens,
// W dequantized from GGUF Q4_K / Q6_K / Q2_K / IQ2_XXS blocks to bf16 on the way into LDS,
// the activations taken as floats and rounded to bf16 likewise, fp32 accumulation in
// v_mfma_f32_32x32x16_bf16.  This is the fast path: its results differ from the CPU path's
// by the bf16 roundings (tolerance 2e-2 relative, against 1e-5 / bit-exact for the int8
// path in kernels_gemm.hip).  Each weight is dequantized exactly as the reference's
// *-row-floats! / kmat-row! do (kquant.lisp:466-497, iquant.lisp:161-230) before rounding.
//
// A workgroup (256 threads, 4 waves) computes 128 rows x 128 tokens in steps of 64
// columns.  Per step every thread dequantizes 32 weights of one row and converts 32
// activations of one token into LDS; the loads for the next step are issued before the
// step's MFMAs and held in registers.  Wave w owns rows 64*(w/2).. and tokens 64*(w%2)..
// as 2x2 patches of 32x32.  The MFMA's M side is the tokens and its N side the rows, so a
// lane's 16 results of a patch are one row for 16 tokens and a store instruction writes
// 32 consecutive rows of a token.  The grouped expert product (d4_mm_id_*) walks the
// 128-token tiles of every expert's rows in turn, as the int8 kernel does.
#include "ilt_device.h"
#include "ilt_iq2xxs_tables.h"
#include "ilt_kernels.h"

namespace {

typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v2f __attribute__((ext_vector_type(2)));

constexpr int TM = 128, TN = 128, KS = 64;   // rows, tokens, columns per step
constexpr int PITCH = KS + 8;                // LDS row pitch in bf16 elements (144 bytes)

__device__ const u64 bf_grid_dev[256] = { ILT_IQ2XXS_GRID_VALUES };

__device__ __forceinline__ u32 pack_bf16(float a, float b) {
  const v2f v = {a, b};
  const v2bf r = __builtin_convertvector(v, v2bf);
  u32 u; __builtin_memcpy(&u, &r, 4); return u;
}

struct Smem {
  __bf16 wt[TM * PITCH];
  __bf16 xt[TN * PITCH];
  u64 grid[256];
  u32 scan[256];
  int tile_z, tile_t0, tile_n;
};

// What a thread holds of the next step: the raw bytes of its 32 weights, its 32 activations.
template <int FMT> struct WRaw;
template <> struct WRaw<ILT_Q4_K> { int4 hdr, qa, qb; };
template <> struct WRaw<ILT_Q6_K> { int4 qla, qlb, qha, qhb; u32 sc, d; };
template <> struct WRaw<ILT_Q2_K> { int4 qa, qb; u32 sb, dd; };
template <> struct WRaw<ILT_IQ2_XXS> { int2 q; u32 d; };

constexpr u32 kOob = 0xFFFFFFF0u;   // an offset past any buffer: the load returns zeros

template <int FMT> __device__ __forceinline__ void load_w(WRaw<FMT>& r, __amdgpu_buffer_rsrc_t rw, u32 rowoff, int ks, int e, bool live);

template <> __device__ __forceinline__ void load_w<ILT_Q4_K>(WRaw<ILT_Q4_K>& r, __amdgpu_buffer_rsrc_t rw, u32 rowoff, int ks, int e, bool live) {
  const u32 b = live ? rowoff + (u32)(ks >> 2) * 144 : kOob;
  r.hdr = ilt_bld16(rw, b);
  r.qa = ilt_bld16(rw, b + 16 + 32 * (ks & 3));
  r.qb = ilt_bld16(rw, b + 32 + 32 * (ks & 3));
}
template <> __device__ __forceinline__ void load_w<ILT_Q6_K>(WRaw<ILT_Q6_K>& r, __amdgpu_buffer_rsrc_t rw, u32 rowoff, int ks, int e, bool live) {
  const u32 b = live ? rowoff + (u32)(ks >> 2) * ILT_Q6K_STRIDE : kOob;
  const int c = (ks >> 1) & 1, part = 2 * (ks & 1) + e;
  r.qla = ilt_bld16(rw, b + 64 * c + 32 * e);
  r.qlb = ilt_bld16(rw, b + 64 * c + 32 * e + 16);
  r.qha = ilt_bld16(rw, b + 128 + 32 * c);
  r.qhb = ilt_bld16(rw, b + 128 + 32 * c + 16);
  r.sc = ilt_bld2(rw, b + 192 + 8 * c + 2 * part);
  r.d = ilt_bld2(rw, b + 208);
}
template <> __device__ __forceinline__ void load_w<ILT_Q2_K>(WRaw<ILT_Q2_K>& r, __amdgpu_buffer_rsrc_t rw, u32 rowoff, int ks, int e, bool live) {
  const u32 b = live ? rowoff + (u32)(ks >> 2) * 84 : kOob;
  const int h = (ks >> 1) & 1, k = 2 * (ks & 1) + e;
  r.qa = ilt_bld16(rw, b + 16 + 32 * h);
  r.qb = ilt_bld16(rw, b + 32 + 32 * h);
  r.sb = ilt_bld2(rw, b + 8 * h + 2 * k);
  r.dd = ilt_bld4(rw, b + 80);
}
template <> __device__ __forceinline__ void load_w<ILT_IQ2_XXS>(WRaw<ILT_IQ2_XXS>& r, __amdgpu_buffer_rsrc_t rw, u32 rowoff, int ks, int e, bool live) {
  const u32 b = live ? rowoff + (u32)(ks >> 2) * 66 : kOob;
  r.q = ilt_bld8(rw, b + 2 + 8 * (2 * (ks & 3) + e));
  r.d = ilt_bld2(rw, b);
}

// 32 weights as floats, in column order, each computed as the CPU dequantizers compute it.
template <int FMT> __device__ __forceinline__ void dequant32(const WRaw<FMT>& r, int ks, int e, const u64* grid, float* o);

template <> __device__ __forceinline__ void dequant32<ILT_Q4_K>(const WRaw<ILT_Q4_K>& r, int ks, int e, const u64*, float* o) {
  const int g = 2 * (ks & 3) + e, sh = 8 * (g & 3);
  const u32 x0 = ((u32)r.hdr.y >> sh) & 0xFF, x1 = ((u32)r.hdr.z >> sh) & 0xFF, x2 = ((u32)r.hdr.w >> sh) & 0xFF;
  const u32 sc = g < 4 ? (x0 & 63) : ((x2 & 0xF) | ((x0 >> 6) << 4));
  const u32 mn = g < 4 ? (x1 & 63) : ((x2 >> 4) | ((x1 >> 6) << 4));
  const float d1 = ilt_h2f((u16)(r.hdr.x & 0xFFFF)) * (float)sc, m1 = ilt_h2f((u16)((u32)r.hdr.x >> 16)) * (float)mn;
  const u32 w[8] = {(u32)r.qa.x, (u32)r.qa.y, (u32)r.qa.z, (u32)r.qa.w, (u32)r.qb.x, (u32)r.qb.y, (u32)r.qb.z, (u32)r.qb.w};
#pragma unroll
  for (int i = 0; i < 8; i++) {
    const u32 v = (w[i] >> (4 * e)) & 0x0F0F0F0F;
#pragma unroll
    for (int k = 0; k < 4; k++) o[4 * i + k] = d1 * (float)((v >> (8 * k)) & 0xFF) - m1;
  }
}

template <> __device__ __forceinline__ void dequant32<ILT_Q6_K>(const WRaw<ILT_Q6_K>& r, int ks, int e, const u64*, float* o) {
  const int h = ks & 1, part = 2 * h + e;
  const float d = ilt_h2f((u16)r.d);
  const float s0 = d * (float)(i8)(r.sc & 0xFF), s1 = d * (float)(i8)((r.sc >> 8) & 0xFF);
  const u32 ql[8] = {(u32)r.qla.x, (u32)r.qla.y, (u32)r.qla.z, (u32)r.qla.w, (u32)r.qlb.x, (u32)r.qlb.y, (u32)r.qlb.z, (u32)r.qlb.w};
  const u32 qh[8] = {(u32)r.qha.x, (u32)r.qha.y, (u32)r.qha.z, (u32)r.qha.w, (u32)r.qhb.x, (u32)r.qhb.y, (u32)r.qhb.z, (u32)r.qhb.w};
#pragma unroll
  for (int i = 0; i < 8; i++) {
    const u32 v = ((ql[i] >> (4 * h)) & 0x0F0F0F0F) | (((qh[i] >> (2 * part)) & 0x03030303) << 4);
    const float s = i < 4 ? s0 : s1;
#pragma unroll
    for (int k = 0; k < 4; k++) o[4 * i + k] = s * (float)((int)((v >> (8 * k)) & 0xFF) - 32);
  }
}

template <> __device__ __forceinline__ void dequant32<ILT_Q2_K>(const WRaw<ILT_Q2_K>& r, int ks, int e, const u64*, float* o) {
  const int k2 = 2 * (2 * (ks & 1) + e);
  const float d = ilt_h2f((u16)(r.dd & 0xFFFF)), dmin = ilt_h2f((u16)(r.dd >> 16));
  const u32 sa = r.sb & 0xFF, sbb = (r.sb >> 8) & 0xFF;
  const float dl0 = d * (float)(sa & 15), ml0 = dmin * (float)(sa >> 4);
  const float dl1 = d * (float)(sbb & 15), ml1 = dmin * (float)(sbb >> 4);
  const u32 w[8] = {(u32)r.qa.x, (u32)r.qa.y, (u32)r.qa.z, (u32)r.qa.w, (u32)r.qb.x, (u32)r.qb.y, (u32)r.qb.z, (u32)r.qb.w};
#pragma unroll
  for (int i = 0; i < 8; i++) {
    const u32 v = (w[i] >> k2) & 0x03030303;
    const float dl = i < 4 ? dl0 : dl1, ml = i < 4 ? ml0 : ml1;
#pragma unroll
    for (int k = 0; k < 4; k++) o[4 * i + k] = dl * (float)((v >> (8 * k)) & 0xFF) - ml;
  }
}

template <> __device__ __forceinline__ void dequant32<ILT_IQ2_XXS>(const WRaw<ILT_IQ2_XXS>& r, int ks, int e, const u64* grid, float* o) {
  const u32 g = (u32)r.q.x, aux = (u32)r.q.y;
  const float db = (ilt_h2f((u16)r.d) * (0.5f + (float)(aux >> 28))) * 0.25f;
#pragma unroll
  for (int l = 0; l < 4; l++) {
    const int2 mag = ilt_lds_ld8(grid + ((g >> (8 * l)) & 0xFF));
    u32 s = (aux >> (7 * l)) & 127;
    s |= (__popc(s) & 1) << 7;
#pragma unroll
    for (int k = 0; k < 8; k++) {
      const u32 m = ((k < 4 ? (u32)mag.x : (u32)mag.y) >> (8 * (k & 3))) & 0xFF;
      o[8 * l + k] = (db * (float)m) * (((s >> k) & 1) ? -1.0f : 1.0f);
    }
  }
}

struct BfParams {
  const u8* w;                               // dense
  const u64* ptrs; long long add;            // grouped: expert z's matrix at ptrs[z] + add
  const u32* counts; const u32* bases; int ne;
  int rows, cols; long long row_bytes;
  const float* x;                            // activations, cols floats per token (gathered rows when grouped)
  float* y; const float* bias; int acc; int ntok;
};

template <int FMT>
__global__ __launch_bounds__(256) void gemm_bf16_kernel(BfParams p) {
  __shared__ __align__(16) Smem S;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  long tok0; int ntok; const u8* w = p.w;
  if (p.ptrs) {
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
  if (FMT == ILT_IQ2_XXS) S.grid[t] = bf_grid_dev[t];

  // this thread's share of a step: 32 weights of row wrow (half e), 32 activations of token xtok (half e)
  const int wrow = t >> 1, e = t & 1;
  const bool wlive = r0 + wrow < p.rows, xlive = wrow < ntok;
  const __amdgpu_buffer_rsrc_t rw = ilt_rsrc(ilt_uniform_ptr(w), (u32)min((long long)p.rows * p.row_bytes, 0xFFFFFFF0LL));
  const __amdgpu_buffer_rsrc_t rx = ilt_rsrc(ilt_uniform_ptr(p.x + tok0 * p.cols), (u32)min((long long)ntok * p.cols * 4, 0xFFFFFFF0LL));
  const u32 wrowoff = (u32)((long long)(r0 + wrow) * p.row_bytes);
  const u32 xrowoff = xlive ? (u32)(((long long)wrow * p.cols + 32 * e) * 4) : kOob;

  v16f acc[2][2];
#pragma unroll
  for (int a = 0; a < 2; a++)
#pragma unroll
    for (int b = 0; b < 2; b++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[a][b][r] = 0.0f;

  const int wt0 = 64 * (wave & 1), wr0 = 64 * (wave >> 1);   // this wave's tokens and rows in the tile
  const int l32 = lane & 31, lh = lane >> 5;

  WRaw<FMT> wraw;
  int4 xraw[8];
  load_w<FMT>(wraw, rw, wrowoff, 0, e, wlive);
#pragma unroll
  for (int i = 0; i < 8; i++) xraw[i] = ilt_bld16(rx, xrowoff + 16 * i);

  const int nk = p.cols / KS;
  for (int ks = 0; ks < nk; ks++) {
    __syncthreads();     // the previous step's MFMAs have read the tiles (and the codebook is in place)
    {
      float o[32];
      dequant32<FMT>(wraw, ks, e, S.grid, o);
      u32 pk[16];
#pragma unroll
      for (int i = 0; i < 16; i++) pk[i] = pack_bf16(o[2 * i], o[2 * i + 1]);
      int4* dst = (int4*)(S.wt + wrow * PITCH + 32 * e);
#pragma unroll
      for (int i = 0; i < 4; i++) dst[i] = make_int4(pk[4 * i], pk[4 * i + 1], pk[4 * i + 2], pk[4 * i + 3]);
      u32 px[16];
#pragma unroll
      for (int i = 0; i < 8; i++) {
        px[2 * i] = pack_bf16(__int_as_float(xraw[i].x), __int_as_float(xraw[i].y));
        px[2 * i + 1] = pack_bf16(__int_as_float(xraw[i].z), __int_as_float(xraw[i].w));
      }
      int4* dx = (int4*)(S.xt + wrow * PITCH + 32 * e);
#pragma unroll
      for (int i = 0; i < 4; i++) dx[i] = make_int4(px[4 * i], px[4 * i + 1], px[4 * i + 2], px[4 * i + 3]);
    }
    __syncthreads();
    if (ks + 1 < nk) {   // the next step's loads, in flight under this step's MFMAs
      load_w<FMT>(wraw, rw, wrowoff, ks + 1, e, wlive);
#pragma unroll
      for (int i = 0; i < 8; i++) xraw[i] = ilt_bld16(rx, xrowoff + (u32)(ks + 1) * (KS * 4) + 16 * i);
    }
#pragma unroll
    for (int kk = 0; kk < KS / 16; kk++) {
      v8bf af[2], bf[2];
#pragma unroll
      for (int a = 0; a < 2; a++) af[a] = *(const v8bf*)(S.xt + (wt0 + 32 * a + l32) * PITCH + 16 * kk + 8 * lh);
#pragma unroll
      for (int b = 0; b < 2; b++) bf[b] = *(const v8bf*)(S.wt + (wr0 + 32 * b + l32) * PITCH + 16 * kk + 8 * lh);
#pragma unroll
      for (int a = 0; a < 2; a++)
#pragma unroll
        for (int b = 0; b < 2; b++) acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[a], bf[b], acc[a][b], 0, 0, 0);
    }
  }

  // ---- store: patch (a, b): token = wt0 + 32a + 8*(r/4) + 4*lh + r%4, row = wr0 + 32b + l32 ----
#pragma unroll
  for (int b = 0; b < 2; b++) {
    const int row = r0 + wr0 + 32 * b + l32;
    if (row >= p.rows) continue;
    const float bv = p.bias ? p.bias[row] : 0.0f;
#pragma unroll
    for (int a = 0; a < 2; a++) {
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int tk = wt0 + 32 * a + 8 * (r >> 2) + 4 * lh + (r & 3);
        if (tk >= ntok) continue;
        float* yo = p.y + (tok0 + tk) * (long)p.rows + row;
        float v = acc[a][b][r];
        if (p.bias) v = v + bv;
        if (p.acc) v = *yo + v;
        *yo = v;
      }
    }
  }
}

template <int FMT>
hipError_t launch_bf16(const BfParams& p, unsigned tiles_x, hipStream_t st) {
  dim3 grid(tiles_x, (p.rows + TM - 1) / TM);
  hipLaunchKernelGGL(gemm_bf16_kernel<FMT>, grid, dim3(256), 0, st, p);
  return hipGetLastError();
}

hipError_t dispatch_bf16(int fmt, const BfParams& p, unsigned tiles_x, hipStream_t st) {
  switch (fmt) {
    case ILT_Q4_K: return launch_bf16<ILT_Q4_K>(p, tiles_x, st);
    case ILT_Q6_K: return launch_bf16<ILT_Q6_K>(p, tiles_x, st);
    case ILT_Q2_K: return launch_bf16<ILT_Q2_K>(p, tiles_x, st);
    case ILT_IQ2_XXS: return launch_bf16<ILT_IQ2_XXS>(p, tiles_x, st);
  }
  return hipErrorInvalidValue;
}

}  // namespace

hipError_t ilt_k_gemm_bf16(int fmt, const uint8_t* w, long long row_bytes, int rows, int cols, const float* x, int ntok,
                           float* y, const float* bias, int acc, hipStream_t st) {
  if (ntok <= 0 || rows <= 0) return hipSuccess;
  BfParams p = {};
  p.w = w; p.rows = rows; p.cols = cols; p.row_bytes = row_bytes; p.x = x; p.y = y; p.bias = bias; p.acc = acc; p.ntok = ntok;
  return dispatch_bf16(fmt, p, (unsigned)((ntok + TN - 1) / TN), st);
}

hipError_t ilt_k_gemm_bf16_id(int fmt, const uint64_t* ptrs, long long add, const uint32_t* counts, const uint32_t* bases,
                              int ne, long long row_bytes, int rows, int cols, const float* x, long long total_rows,
                              float* y, hipStream_t st) {
  if (total_rows <= 0 || rows <= 0 || ne <= 0) return hipSuccess;
  if (ne > 256) return hipErrorInvalidValue;
  BfParams p = {};
  p.ptrs = ptrs; p.add = add; p.counts = counts; p.bases = bases; p.ne = ne;
  p.rows = rows; p.cols = cols; p.row_bytes = row_bytes; p.x = x; p.y = y; p.ntok = (int)total_rows;
  return dispatch_bf16(fmt, p, (unsigned)(total_rows / TN + ne), st);
}
