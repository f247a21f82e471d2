// Prefill products on the bf16 matrix cores of gfx950: Y[t][r] = W[r].x_t for many tokens,
// W dequantized from GGUF Q4_K / Q6_K / Q2_K / IQ2_XXS blocks to bf16 on the way into LDS,
// the activations already rounded to bf16 (ilt_k_cvt_bf16), fp32 accumulation in
// v_mfma_f32_32x32x16_bf16.  This is the fast path: its results differ from the CPU path's
// by the bf16 roundings (tolerance 2e-2 relative, against bit-exact for the int8 path in
// kernels_gemm.hip).  Each weight is dequantized exactly as the reference's
// *-row-floats! / kmat-row! do (kquant.lisp:466-497, iquant.lisp:161-230) before rounding.
//
// A workgroup (256 threads, 4 waves) computes 128 rows x TN tokens (TN 256, or 128 for few
// tokens and for the expert groups) in steps of 32 columns:
//   - the activations' 32-column slab goes from global memory straight into LDS
//     (global_load_lds_dwordx4), two steps ahead, into a ring of three slabs;
//   - every thread holds the raw bytes of 16 weights of one row one step ahead in registers,
//     dequantizes them and writes them as bf16 into one of two weight slabs;
//   - one barrier per step; then wave w multiplies rows 64*(w/2).. by tokens (TN/2)*(w%2)..
//     as patches of 32x32.  The MFMA's M side is the tokens and its N side the rows, so a
//     lane's 16 results of a patch are one row for 16 tokens and a store instruction writes
//     32 consecutive rows of a token.
// Both kinds of slab hold 64 bytes per row as four 16-byte pieces, piece p of row r at
// 4*r + (p ^ ((r>>2)&3)): rows 0..15 of one piece index cover all 64 banks once, with no
// padding (the direct loads write 1 KB per wave instruction contiguously, so the swizzle
// is applied by choosing which global piece each lane fetches).
// Two workgroups share a CU, so one's dequantization overlaps the other's MFMAs.
// Tiles are numbered so that the workgroups resident on one XCD (every eighth workgroup id)
// form a block of 8 row tiles x 8 token tiles and share W and x slabs through that XCD's L2.
// The grouped expert product (d4_mm_id_*) walks the token tiles of every expert's rows in turn.
#include "ilt_device.h"
#include "ilt_iq2xxs_tables.h"
#include "ilt_kernels.h"

namespace {

typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v2f __attribute__((ext_vector_type(2)));

constexpr int TM = 128, KS = 32;       // rows per tile, columns per step
constexpr int GR = 8;                  // row tiles per block of tiles sharing an L2
constexpr int WSLAB = TM * KS * 2;     // bytes of a weight slab

__device__ const u64 bf_grid_dev[256] = { ILT_IQ2XXS_GRID_VALUES };

__device__ __forceinline__ u32 pack_bf16(float a, float b) {
  const v2f v = {a, b};
  const v2bf r = __builtin_convertvector(v, v2bf);
  u32 u; __builtin_memcpy(&u, &r, 4); return u;
}

// The raw bytes of a thread's 16 weights (row = t/2, columns 16*(t%2).. of the step's 32).
template <int FMT> struct WRaw;
template <> struct WRaw<ILT_Q4_K> { int4 hdr, q; };
template <> struct WRaw<ILT_Q6_K> { int4 ql, qh; u32 sc, d; };
template <> struct WRaw<ILT_Q2_K> { int4 q; u32 sc, dd; };
template <> struct WRaw<ILT_IQ2_XXS> { int2 q; u32 d; };

template <int FMT> __device__ __forceinline__ void load_w(WRaw<FMT>& r, __amdgpu_buffer_rsrc_t rw, u32 rowoff, int ks, int e);

template <> __device__ __forceinline__ void load_w<ILT_Q4_K>(WRaw<ILT_Q4_K>& r, __amdgpu_buffer_rsrc_t rw, u32 rowoff, int ks, int e) {
  const u32 b = rowoff + (u32)(ks >> 3) * 144;
  r.hdr = ilt_bld16(rw, b);
  r.q = ilt_bld16(rw, b + 16 + 32 * ((ks >> 1) & 3) + 16 * e);
}
template <> __device__ __forceinline__ void load_w<ILT_Q6_K>(WRaw<ILT_Q6_K>& r, __amdgpu_buffer_rsrc_t rw, u32 rowoff, int ks, int e) {
  const u32 b = rowoff + (u32)(ks >> 3) * ILT_Q6K_STRIDE;
  const int c = (ks >> 2) & 1, part = ks & 3;
  r.ql = ilt_bld16(rw, b + 64 * c + 32 * (part & 1) + 16 * e);
  r.qh = ilt_bld16(rw, b + 128 + 32 * c + 16 * e);
  r.sc = ilt_bld1(rw, b + 192 + 8 * c + 2 * part + e);
  r.d = ilt_bld2(rw, b + 208);
}
template <> __device__ __forceinline__ void load_w<ILT_Q2_K>(WRaw<ILT_Q2_K>& r, __amdgpu_buffer_rsrc_t rw, u32 rowoff, int ks, int e) {
  const u32 b = rowoff + (u32)(ks >> 3) * 84;
  const int h = (ks >> 2) & 1, j = ks & 3;
  r.q = ilt_bld16(rw, b + 16 + 32 * h + 16 * e);
  r.sc = ilt_bld1(rw, b + 8 * h + 2 * j + e);
  r.dd = ilt_bld4(rw, b + 80);
}
template <> __device__ __forceinline__ void load_w<ILT_IQ2_XXS>(WRaw<ILT_IQ2_XXS>& r, __amdgpu_buffer_rsrc_t rw, u32 rowoff, int ks, int e) {
  const u32 b = rowoff + (u32)(ks >> 3) * 66;
  r.q = ilt_bld8(rw, b + 2 + 8 * (ks & 7));
  r.d = ilt_bld2(rw, b);
}

// 16 weights as floats, in column order, each computed as the CPU dequantizers compute it.
template <int FMT> __device__ __forceinline__ void dequant16(const WRaw<FMT>& r, int ks, int e, const u64* grid, float* o);

template <> __device__ __forceinline__ void dequant16<ILT_Q4_K>(const WRaw<ILT_Q4_K>& r, int ks, int e, const u64*, float* o) {
  const int g = ks & 7, sh = 8 * (g & 3), hl = ks & 1;
  const u32 x0 = ((u32)r.hdr.y >> sh) & 0xFF, x1 = ((u32)r.hdr.z >> sh) & 0xFF, x2 = ((u32)r.hdr.w >> sh) & 0xFF;
  const u32 sc = g < 4 ? (x0 & 63) : ((x2 & 0xF) | ((x0 >> 6) << 4));
  const u32 mn = g < 4 ? (x1 & 63) : ((x2 >> 4) | ((x1 >> 6) << 4));
  const float d1 = ilt_h2f((u16)(r.hdr.x & 0xFFFF)) * (float)sc, m1 = ilt_h2f((u16)((u32)r.hdr.x >> 16)) * (float)mn;
  const u32 w[4] = {(u32)r.q.x, (u32)r.q.y, (u32)r.q.z, (u32)r.q.w};
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const u32 v = (w[i] >> (4 * hl)) & 0x0F0F0F0F;
#pragma unroll
    for (int k = 0; k < 4; k++) o[4 * i + k] = d1 * (float)((v >> (8 * k)) & 0xFF) - m1;
  }
}

template <> __device__ __forceinline__ void dequant16<ILT_Q6_K>(const WRaw<ILT_Q6_K>& r, int ks, int e, const u64*, float* o) {
  const int part = ks & 3, h = part >> 1;
  const float s = ilt_h2f((u16)r.d) * (float)(i8)(r.sc & 0xFF);
  const u32 ql[4] = {(u32)r.ql.x, (u32)r.ql.y, (u32)r.ql.z, (u32)r.ql.w};
  const u32 qh[4] = {(u32)r.qh.x, (u32)r.qh.y, (u32)r.qh.z, (u32)r.qh.w};
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const u32 v = ((ql[i] >> (4 * h)) & 0x0F0F0F0F) | (((qh[i] >> (2 * part)) & 0x03030303) << 4);
#pragma unroll
    for (int k = 0; k < 4; k++) o[4 * i + k] = s * (float)((int)((v >> (8 * k)) & 0xFF) - 32);
  }
}

template <> __device__ __forceinline__ void dequant16<ILT_Q2_K>(const WRaw<ILT_Q2_K>& r, int ks, int e, const u64*, float* o) {
  const int j = ks & 3;
  const float dl = ilt_h2f((u16)(r.dd & 0xFFFF)) * (float)(r.sc & 15), ml = ilt_h2f((u16)(r.dd >> 16)) * (float)((r.sc >> 4) & 15);
  const u32 w[4] = {(u32)r.q.x, (u32)r.q.y, (u32)r.q.z, (u32)r.q.w};
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const u32 v = (w[i] >> (2 * j)) & 0x03030303;
#pragma unroll
    for (int k = 0; k < 4; k++) o[4 * i + k] = dl * (float)((v >> (8 * k)) & 0xFF) - ml;
  }
}

template <> __device__ __forceinline__ void dequant16<ILT_IQ2_XXS>(const WRaw<ILT_IQ2_XXS>& r, int ks, int e, const u64* grid, float* o) {
  const u32 g = (u32)r.q.x >> (16 * e), aux = (u32)r.q.y;
  const float db = (ilt_h2f((u16)r.d) * (0.5f + (float)(aux >> 28))) * 0.25f;
#pragma unroll
  for (int l = 0; l < 2; l++) {
    const int2 mag = ilt_lds_ld8(grid + ((g >> (8 * l)) & 0xFF));
    u32 s = (aux >> (7 * (2 * e + l))) & 127;
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
  const u16* x;                              // bf16 activations, cols per token (the gathered rows when grouped)
  float* y; const float* bias; int acc; int ntok;
};

template <int TN> struct Smem {
  __align__(16) u8 xs[3][TN * KS * 2];
  __align__(16) u8 ws[2][WSLAB];
  u64 grid[256];
  u32 scan[256];
  int tile_z, tile_t0, tile_n;
};

// piece p (16 bytes) of row r of a slab
__device__ __forceinline__ u32 slab_off(int r, int p) { return (u32)(4 * r + (p ^ ((r >> 2) & 3))) * 16; }

template <int FMT, int TN>
__global__ __launch_bounds__(256, TN == 256 ? 2 : 3) void gemm_bf16_kernel(BfParams p) {
  __shared__ Smem<TN> S;
  constexpr int NA = TN / 64;        // 32-token patches per wave; also direct-load instructions per wave and step
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int NR = (p.rows + TM - 1) / TM;

  // ---- which tile ----
  long tok0; int ntok, rt; const u8* w = p.w;
  {
    int NT;
    if (p.ptrs) {
      S.scan[t] = t < p.ne ? (p.counts[t] + TN - 1) / TN : 0;
      __syncthreads();
      for (int off = 1; off < 256; off <<= 1) {
        const u32 v = t >= off ? S.scan[t - off] : 0;
        __syncthreads();
        S.scan[t] += v;
        __syncthreads();
      }
      NT = (int)S.scan[255];
    } else {
      NT = (p.ntok + TN - 1) / TN;
    }
    const int total = NT * NR, per = (total + 7) / 8;
    const int L = blockIdx.x, j = L >> 3;
    const int s = (L & 7) * per + j;
    if (j >= per || s >= total) return;
    const int rg = s / (GR * NT), rem = s - rg * GR * NT, nr = min(GR, NR - rg * GR);
    const int tt = rem / nr;
    rt = rg * GR + (rem - tt * nr);
    if (p.ptrs) {
      if (t < p.ne) {
        const u32 incl = S.scan[t], tiles = (p.counts[t] + TN - 1) / TN, excl = incl - tiles;
        if ((u32)tt >= excl && (u32)tt < incl) {
          S.tile_z = t;
          S.tile_t0 = (int)(p.bases[t] + ((u32)tt - excl) * TN);
          S.tile_n = (int)min((u32)TN, p.counts[t] - ((u32)tt - excl) * TN);
        }
      }
      __syncthreads();
      tok0 = S.tile_t0; ntok = S.tile_n;
      w = (const u8*)(p.ptrs[S.tile_z] + p.add);
    } else {
      tok0 = (long)tt * TN;
      ntok = min(TN, p.ntok - (int)tok0);
    }
  }
  const int r0 = rt * TM;
  if (FMT == ILT_IQ2_XXS) { S.grid[t] = bf_grid_dev[t]; __syncthreads(); }

  // ---- this thread's shares of a step ----
  const int wrow = t >> 1, e = t & 1;                      // 16 weights of row wrow
  const __amdgpu_buffer_rsrc_t rw = ilt_rsrc(ilt_uniform_ptr(w), (u32)min((long long)p.rows * p.row_bytes, 0xFFFFFFF0LL));
  const u32 wrowoff = (u32)((long long)min(r0 + wrow, p.rows - 1) * p.row_bytes);
  const u32 wdst = slab_off(wrow, 2 * e);                  // its two pieces: 2e and 2e+1 (the second at wdst ^ 16)
  const u8* xsrc[NA];                                      // the x pieces it sends to LDS
#pragma unroll
  for (int i = 0; i < NA; i++) {
    const int P = (wave * NA + i) * 64 + lane, tok = P >> 2, kp = (P & 3) ^ ((tok >> 2) & 3);
    xsrc[i] = (const u8*)(p.x + (tok0 + min(tok, ntok - 1)) * (long)p.cols) + 16 * kp;
  }

  v16f acc[NA][2];
#pragma unroll
  for (int a = 0; a < NA; a++)
#pragma unroll
    for (int b = 0; b < 2; b++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[a][b][r] = 0.0f;

  const int wt0 = (TN / 2) * (wave & 1), wr0 = 64 * (wave >> 1);   // this wave's tokens and rows in the tile
  const int l32 = lane & 31, lh = lane >> 5;
  u32 aoff[NA], boff[2];                                   // fragment offsets for the step's first 16 columns; the second 16 at ^ 32
#pragma unroll
  for (int a = 0; a < NA; a++) aoff[a] = slab_off(wt0 + 32 * a + l32, lh);
#pragma unroll
  for (int b = 0; b < 2; b++) boff[b] = slab_off(wr0 + 32 * b + l32, lh);

  const int nk = p.cols / KS;
  auto issue_x = [&](int stage, int ks) {
#pragma unroll
    for (int i = 0; i < NA; i++) ilt_g2lds16(xsrc[i] + (long)ks * (KS * 2), S.xs[stage] + (wave * NA + i) * 1024);
  };

  WRaw<FMT> wraw;
  load_w<FMT>(wraw, rw, wrowoff, 0, e);
  issue_x(0, 0);
  issue_x(1, min(1, nk - 1));
  int st0 = 0, st1 = 1, st2 = 2;                           // ring: the step's slab, the next step's, the one after

  for (int ks = 0; ks < nk; ks++) {
    {
      float o[16];
      dequant16<FMT>(wraw, ks, e, S.grid, o);
      u32 pk[8];
#pragma unroll
      for (int i = 0; i < 8; i++) pk[i] = pack_bf16(o[2 * i], o[2 * i + 1]);
      u8* ws = S.ws[ks & 1];
      *(int4*)(ws + wdst) = make_int4(pk[0], pk[1], pk[2], pk[3]);
      *(int4*)(ws + (wdst ^ 16)) = make_int4(pk[4], pk[5], pk[6], pk[7]);
    }
    // all but the newest NA loads have landed: this step's x slab has (it was sent two steps ago)
    if (NA == 4) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
    __syncthreads();
    load_w<FMT>(wraw, rw, wrowoff, min(ks + 1, nk - 1), e);
    issue_x(st2, min(ks + 2, nk - 1));
    const u8* xs = S.xs[st0];
    const u8* ws = S.ws[ks & 1];
#pragma unroll
    for (int kk = 0; kk < 2; kk++) {
      v8bf af[NA], bf[2];
#pragma unroll
      for (int a = 0; a < NA; a++) af[a] = *(const v8bf*)(xs + (aoff[a] ^ (32 * kk)));
#pragma unroll
      for (int b = 0; b < 2; b++) bf[b] = *(const v8bf*)(ws + (boff[b] ^ (32 * kk)));
#pragma unroll
      for (int a = 0; a < NA; a++)
#pragma unroll
        for (int b = 0; b < 2; b++) acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[a], bf[b], acc[a][b], 0, 0, 0);
    }
    const int s = st0; st0 = st1; st1 = st2; st2 = s;
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the tail's redundant loads: nothing may land in LDS after the workgroup ends

  // ---- store: patch (a, b): token = wt0 + 32a + 8*(r/4) + 4*lh + r%4, row = wr0 + 32b + l32 ----
#pragma unroll
  for (int b = 0; b < 2; b++) {
    const int row = r0 + wr0 + 32 * b + l32;
    if (row >= p.rows) continue;
    const float bv = p.bias ? p.bias[row] : 0.0f;
#pragma unroll
    for (int a = 0; a < NA; a++) {
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

__global__ __launch_bounds__(256) void cvt_bf16_kernel(const float* __restrict__ x, u16* __restrict__ xb, long long n8) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= n8) return;
  const float4 a = ((const float4*)x)[2 * i], b = ((const float4*)x)[2 * i + 1];
  ((int4*)xb)[i] = make_int4(pack_bf16(a.x, a.y), pack_bf16(a.z, a.w), pack_bf16(b.x, b.y), pack_bf16(b.z, b.w));
}

template <int FMT, int TN>
hipError_t launch_bf16(const BfParams& p, long long token_tiles, hipStream_t st) {
  const long long total = token_tiles * ((p.rows + TM - 1) / TM), per = (total + 7) / 8;
  if (per * 8 > 0x7FFFFFFFLL) return hipErrorInvalidValue;
  hipLaunchKernelGGL((gemm_bf16_kernel<FMT, TN>), dim3((unsigned)(per * 8)), dim3(256), 0, st, p);
  return hipGetLastError();
}

template <int TN>
hipError_t dispatch_bf16(int fmt, const BfParams& p, long long token_tiles, hipStream_t st) {
  switch (fmt) {
    case ILT_Q4_K: return launch_bf16<ILT_Q4_K, TN>(p, token_tiles, st);
    case ILT_Q6_K: return launch_bf16<ILT_Q6_K, TN>(p, token_tiles, st);
    case ILT_Q2_K: return launch_bf16<ILT_Q2_K, TN>(p, token_tiles, st);
    case ILT_IQ2_XXS: return launch_bf16<ILT_IQ2_XXS, TN>(p, token_tiles, st);
  }
  return hipErrorInvalidValue;
}

}  // namespace

hipError_t ilt_k_cvt_bf16(const float* x, uint16_t* xb, long long n, hipStream_t st) {
  if (n <= 0) return hipSuccess;
  const long long n8 = n / 8;
  hipLaunchKernelGGL(cvt_bf16_kernel, dim3((unsigned)((n8 + 255) / 256)), dim3(256), 0, st, x, xb, n8);
  return hipGetLastError();
}

hipError_t ilt_k_gemm_bf16(int fmt, const uint8_t* w, long long row_bytes, int rows, int cols, const uint16_t* xb, int ntok,
                           float* y, const float* bias, int acc, hipStream_t st) {
  if (ntok <= 0 || rows <= 0) return hipSuccess;
  BfParams p = {};
  p.w = w; p.rows = rows; p.cols = cols; p.row_bytes = row_bytes; p.x = xb; p.y = y; p.bias = bias; p.acc = acc; p.ntok = ntok;
  // 256-token tiles halve the dequantization per product, but need enough tiles to fill 512 workgroup slots
  const long long nr = (rows + TM - 1) / TM;
  if ((long long)((ntok + 255) / 256) * nr >= 1024) return dispatch_bf16<256>(fmt, p, (ntok + 255) / 256, st);
  return dispatch_bf16<128>(fmt, p, (ntok + 127) / 128, st);
}

hipError_t ilt_k_gemm_bf16_id(int fmt, const uint64_t* ptrs, long long add, const uint32_t* counts, const uint32_t* bases,
                              int ne, long long row_bytes, int rows, int cols, const uint16_t* xb, long long total_rows,
                              float* y, hipStream_t st) {
  if (total_rows <= 0 || rows <= 0 || ne <= 0) return hipSuccess;
  if (ne > 256) return hipErrorInvalidValue;
  BfParams p = {};
  p.ptrs = ptrs; p.add = add; p.counts = counts; p.bases = bases; p.ne = ne;
  p.rows = rows; p.cols = cols; p.row_bytes = row_bytes; p.x = xb; p.y = y; p.ntok = (int)total_rows;
  return dispatch_bf16<128>(fmt, p, total_rows / 128 + ne, st);
}
