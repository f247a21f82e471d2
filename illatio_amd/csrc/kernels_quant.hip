// Activation quantizers, the Q8_0 upload repack, and row dequantizers for gfx950.
// Every result is bit-for-bit what the reference's CPU path stores
// (tensor.lisp:245-262, kquant.lisp:130-167, 466-497, iquant.lisp:161-230).
#include "ilt_device.h"
#include "ilt_iq2xxs_tables.h"
#include "ilt_kernels.h"

namespace {

__device__ const u64 q_grid_dev[256] = { ILT_IQ2XXS_GRID_VALUES };

// Q8_0 activations (quantize-q8!): a block of 32 per half wave.  d = amax/127; the
// stored scale is d through fp16 when f16_scale; q = round-half-even(x * (1/d)) with the
// unrounded d.  xsum (optional) gets the block's integer sum.
__global__ __launch_bounds__(256) void quant_q8_kernel(const float* __restrict__ x, i8* __restrict__ xq,
                                                       float* __restrict__ xs, int* __restrict__ xsum,
                                                       long long nblocks, int f16_scale, long long bpr, long long x_stride) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  const long long b = i >> 5;
  const bool live = b < nblocks;
  // bpr > 0: rows of bpr blocks, x_stride floats from one row's start to the next's (the output stays packed)
  const float v = live ? x[bpr > 0 ? (b / bpr) * x_stride + (b % bpr) * 32 + (i & 31) : i] : 0.0f;
  float amax = ilt_max16(fabsf(v));
  amax = fmaxf(amax, __shfl_xor(amax, 16));
  const float d = amax / 127.0f;
  const float id = d == 0.0f ? 0.0f : 1.0f / d;
  const int q = (int)rintf(v * id);
  int sum = ilt_sum16(q);
  sum += __shfl_xor(sum, 16);
  if (!live) return;
  xq[i] = (i8)q;
  if ((threadIdx.x & 31) == 0) {
    xs[b] = f16_scale ? __half2float(__float2half_rn(d)) : d;
    if (xsum) xsum[b] = sum;
  }
}

// Q8_K activations (quantize-q8k!): a block of 256 per wave, four consecutive values a lane
// (a 16-byte load, a 4-byte store; no LDS, no barrier).  The largest-magnitude value, the
// first of equals, sets iscale = -127/max; q = min(127, round-half-even(iscale*x));
// d = 1/iscale; sums of each 16 quants.
// GLU: the values quantized are swiglu!'s (model.lisp:364-378) of x and up, (x / (1 + e^-x)) * up with the exponential
// through double -- a prompt chunk's gated activations go straight into the blocks the down product reads, and the
// floats are neither written nor read again.
template <bool GLU>
__global__ __launch_bounds__(256) void quant_q8k_kernel(const float* __restrict__ x, const float* __restrict__ up, i8* __restrict__ xq,
                                                        float* __restrict__ xd, int* __restrict__ bsums, long long nblocks,
                                                        long long bpr, long long x_stride) {
  const int lane = threadIdx.x & 63;
  const long long b = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (b >= nblocks) return;
  // bpr > 0: rows of bpr blocks, x_stride floats (a multiple of 4) from one row's start to the next's
  const float4 v4 = ((const float4*)(x + (bpr > 0 ? (b / bpr) * x_stride + (b % bpr) * 256 : b * 256)))[lane];
  float v[4] = {v4.x, v4.y, v4.z, v4.w};
  if (GLU) {
    const float4 u4 = ((const float4*)(up + b * 256))[lane];
    const float u[4] = {u4.x, u4.y, u4.z, u4.w};
#pragma unroll
    for (int k = 0; k < 4; k++) v[k] = (v[k] / (1.0f + ilt_expf_via_double(-v[k]))) * u[k];
  }
  // |v|'s bits order as |v| does; the low word prefers the earlier index
  u64 key = 0;
#pragma unroll
  for (int k = 0; k < 4; k++) {
    const u64 kk = ((u64)__float_as_uint(fabsf(v[k])) << 32) | (u32)(255 - (4 * lane + k));
    key = kk > key ? kk : key;
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const u32 hi = __shfl_xor((u32)(key >> 32), off), lo = __shfl_xor((u32)key, off);
    const u64 o = ((u64)hi << 32) | lo;
    key = o > key ? o : key;
  }
  const int idx = 255 - (int)(key & 0xFFFFFFFFu);             // the same in every lane
  const int ik = idx & 3;
  const float mine = ik == 0 ? v[0] : ik == 1 ? v[1] : ik == 2 ? v[2] : v[3];
  const float mx = __shfl(mine, idx >> 2);
  int q[4] = {0, 0, 0, 0};
  float iscale = 0.0f;
  const bool any = (key >> 32) != 0;
  if (any) {
    iscale = -127.0f / mx;
#pragma unroll
    for (int k = 0; k < 4; k++) q[k] = min(127, (int)rintf(iscale * v[k]));
  }
  ((u32*)(xq + b * 256))[lane] = (u32)(q[0] & 0xFF) | ((u32)(q[1] & 0xFF) << 8) | ((u32)(q[2] & 0xFF) << 16) | ((u32)(q[3] & 0xFF) << 24);
  int s = (q[0] + q[1]) + (q[2] + q[3]);
  s += __shfl_xor(s, 1);
  s += __shfl_xor(s, 2);
  if ((lane & 3) == 0) bsums[b * 16 + (lane >> 2)] = s;
  if (lane == 0) xd[b] = any ? 1.0f / iscale : 0.0f;
}

// GGUF Q8_0 blocks (f16 d, 32 int8) split into an int8 array and an f16 scale array.
__global__ __launch_bounds__(256) void repack_q8_kernel(const u8* __restrict__ raw, i8* __restrict__ qs,
                                                        u16* __restrict__ d, long long nblocks) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;   // one thread per 2 bytes of quants
  const long long b = i >> 4;
  if (b >= nblocks) return;
  const int k = (int)(i & 15);
  const u8* blk = raw + b * 34;
  *(u16*)(qs + b * 32 + 2 * k) = *(const u16*)(blk + 2 + 2 * k);
  if (k == 0) d[b] = *(const u16*)blk;
}

// GGUF Q6_K blocks (210 bytes) to the device block: the same bytes, then two of padding.
__global__ __launch_bounds__(256) void repack_q6k_kernel(const u8* __restrict__ raw, u8* __restrict__ out, long long nblocks) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;   // one thread per 2 bytes
  const long long b = i / (ILT_Q6K_STRIDE / 2);
  if (b >= nblocks) return;
  const int k = (int)(i % (ILT_Q6K_STRIDE / 2));
  *(u16*)(out + b * ILT_Q6K_STRIDE + 2 * k) = k < 105 ? *(const u16*)(raw + b * 210 + 2 * k) : (u16)0;
}

__global__ __launch_bounds__(256) void copy_bytes_kernel(const u8* __restrict__ src, u8* __restrict__ dst, long long bytes) {
  const long long i = ((long long)blockIdx.x * 256 + threadIdx.x) * 2;
  if (i + 1 < bytes) *(u16*)(dst + i) = *(const u16*)(src + i);
  else if (i < bytes) dst[i] = src[i];
}

// d4_read_through (ds4f.cu:742-760) as a launch in front of the product: the experts whose srcs entry is set have the
// BYTES at srcs[z] + add (host memory the device can read) copied to ptrs[z] + add, their slot.  Grid y = the expert;
// 16 bytes a lane where both addresses allow, else two.
__global__ __launch_bounds__(256) void read_through_kernel(const unsigned long long* __restrict__ srcs, const unsigned long long* __restrict__ ptrs,
                                                           long long add, long long bytes) {
  const unsigned long long s0 = srcs[blockIdx.y];
  if (!s0) return;
  const u8* src = (const u8*)(s0 + add);
  u8* dst = (u8*)(ptrs[blockIdx.y] + add);
  const long long step = (long long)gridDim.x * 256, t = (long long)blockIdx.x * 256 + threadIdx.x;
  if ((((unsigned long long)src | (unsigned long long)dst) & 15) == 0) {
    const long long n16 = bytes >> 4;
    for (long long i = t; i < n16; i += step) ((int4*)dst)[i] = ((const int4*)src)[i];
    for (long long i = (n16 << 4) + t; i < bytes; i += step) dst[i] = src[i];
  } else {
    for (long long i = 2 * t; i < bytes; i += 2 * step) {
      if (i + 1 < bytes) *(u16*)(dst + i) = *(const u16*)(src + i);
      else dst[i] = src[i];
    }
  }
}

// ---- rows as floats (embed_q8 / embed_k; q8mat-row!, kmat-row!, *-row-floats!) ------------------
__device__ __forceinline__ void scale_min_k4_bytes(int j, const u8* q, int& sc, int& m) {
  if (j < 4) { sc = q[j] & 63; m = q[j + 4] & 63; }
  else { sc = (q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4); m = (q[j + 4] >> 4) | ((q[j] >> 6) << 4); }
}

__device__ float dequant_one(int fmt, const u8* wrow, const u16* wdrow, int col) {
  if (fmt == ILT_Q8_0) {
    // split layout: wrow = int8 quants of the row, wdrow = its f16 scales
    return ilt_h2f(wdrow[col >> 5]) * (float)((const i8*)wrow)[col];
  }
  const int i = col >> 8, idx = col & 255;
  if (fmt == ILT_Q4_K) {
    const u8* blk = wrow + (long)i * 144;
    const int g = idx >> 5, l = idx & 31;
    int sc, m; scale_min_k4_bytes(g, blk + 4, sc, m);
    const u8 byte = blk[16 + (g >> 1) * 32 + l];
    const int q = (g & 1) ? (byte >> 4) : (byte & 0xF);
    const float d1 = ilt_h2f(ilt_ld2(blk)) * (float)sc, m1 = ilt_h2f(ilt_ld2(blk + 2)) * (float)m;
    return d1 * (float)q - m1;
  }
  if (fmt == ILT_Q6_K) {
    const u8* blk = wrow + (long)i * ILT_Q6K_STRIDE;
    const int c = idx >> 7, r = idx & 127, part = r >> 5, l = r & 31;
    const int lowbyte = blk[64 * c + (part & 1) * 32 + l];
    const int low = part < 2 ? (lowbyte & 0xF) : (lowbyte >> 4);
    const int q = low | (((blk[128 + 32 * c + l] >> (2 * part)) & 3) << 4);
    const int sc = ((const i8*)blk)[192 + 8 * c + 2 * part + (l >> 4)];
    return (ilt_h2f(ilt_ld2(blk + 208)) * (float)sc) * (float)(q - 32);
  }
  if (fmt == ILT_Q2_K) {
    const u8* blk = wrow + (long)i * 84;
    const int h = idx >> 7, k = (idx >> 5) & 3, half = (idx >> 4) & 1, l = idx & 15;
    const u8 sb = blk[8 * h + 2 * k + half];
    const float dl = ilt_h2f(ilt_ld2(blk + 80)) * (float)(sb & 15), ml = ilt_h2f(ilt_ld2(blk + 82)) * (float)(sb >> 4);
    return dl * (float)((blk[16 + 32 * h + 16 * half + l] >> (2 * k)) & 3) - ml;
  }
  // IQ2_XXS
  const u8* blk = wrow + (long)i * 66;
  const int ib = idx >> 5, l = (idx >> 3) & 3, jj = idx & 7;
  const u8* so = blk + 2 + 8 * ib;
  const u32 aux = (u32)so[4] | ((u32)so[5] << 8) | ((u32)so[6] << 16) | ((u32)so[7] << 24);
  const float db = (ilt_h2f(ilt_ld2(blk)) * (0.5f + (float)(aux >> 28))) * 0.25f;
  const u64 g = q_grid_dev[so[l]];
  u32 s = (aux >> (7 * l)) & 127;
  s |= (__popc(s) & 1) << 7;
  return (db * (float)((g >> (8 * jj)) & 0xFF)) * (((s >> jj) & 1) ? -1.0f : 1.0f);
}

// out[n][col] = W[rows_idx[n]][col] (rows_idx null: row n).
__global__ __launch_bounds__(256) void dequant_rows_kernel(int fmt, const u8* __restrict__ w, const u16* __restrict__ wd,
                                                           const int* __restrict__ rows_idx, int cols,
                                                           long long row_bytes, float* __restrict__ out) {
  const long long n = blockIdx.y;
  const long long r = rows_idx ? rows_idx[n] : n;
  const u8* wrow = w + r * row_bytes;
  const u16* wdrow = wd ? wd + r * (cols >> 5) : nullptr;
  for (int col = blockIdx.x * 256 + threadIdx.x; col < cols; col += gridDim.x * 256)
    out[n * cols + col] = dequant_one(fmt, wrow, wdrow, col);
}


// y[t*y_stride + r] = W[r] . x[t*x_stride ..] for an F16 matrix and float activations (the router's product,
// ds4f_mm.cu:253; CPU: f32mm!, ds4f.lisp:278-293).  Each dot is F32-DOT16's (tensor.lisp:370-378): column i's
// product, rounded to a float, is added to partial sum i mod 16; the sixteen sums meet as
// c(j) = (s[j] + s[4+j]) + (s[8+j] + s[12+j]), (c(0) + c(1)) + (c(2) + c(3)) -- the CPU's bits.
// 16 lanes a row (lane l = partial sum l), 16 rows a workgroup, 16 tokens a workgroup whose activations go
// through LDS 256 columns at a time; a thread keeps its 16 tokens' partial sums.
__global__ __launch_bounds__(256) void mm_f16_dot16_kernel(int ncols, int nrows, int ntok, long long row_halfs, int x_stride, int y_stride,
                                                           const u16* __restrict__ w, const float* __restrict__ x, float* __restrict__ y) {
  __shared__ float xs[16][256];
  const int l = threadIdx.x & 15, rl = threadIdx.x >> 4;
  const int r = blockIdx.y * 16 + rl, t0 = blockIdx.x * 16;
  const u16* wr = w + (long long)min(r, nrows - 1) * row_halfs;
  float acc[16];
#pragma unroll
  for (int tt = 0; tt < 16; tt++) acc[tt] = 0.0f;
  for (int c0 = 0; c0 < ncols; c0 += 256) {
    const int nc = min(256, ncols - c0);                   // a multiple of 16
    __syncthreads();
    for (int i = threadIdx.x; i < 16 * 256; i += 256) {
      const int tt = i >> 8, c = i & 255;
      xs[tt][c] = (t0 + tt < ntok && c < nc) ? x[(long long)(t0 + tt) * x_stride + c0 + c] : 0.0f;
    }
    __syncthreads();
    for (int jj = 0; jj < nc; jj += 16) {
      const float wv = ilt_h2f(wr[c0 + jj + l]);
#pragma unroll
      for (int tt = 0; tt < 16; tt++) acc[tt] = acc[tt] + wv * xs[tt][jj + l];
    }
  }
#pragma unroll
  for (int tt = 0; tt < 16; tt++) {
    float a = acc[tt];
    a = a + ilt_dppf<ILT_DPP_SHL(4)>(a);                   // lanes 0-3 and 8-11: s[l] + s[l+4]
    a = a + ilt_dppf<ILT_DPP_SHL(8)>(a);                   // lanes 0-3: c(l)
    a = a + ilt_dppf<ILT_DPP_SHL(1)>(a);                   // lanes 0, 2: c(0)+c(1), c(2)+c(3)
    a = a + ilt_dppf<ILT_DPP_SHL(2)>(a);                   // lane 0: the dot
    if (l == 0 && r < nrows && t0 + tt < ntok) y[(long long)(t0 + tt) * y_stride + r] = a;
  }
}

}  // namespace

hipError_t ilt_k_quant_q8(const float* x, int8_t* xq, float* xs, int* xsum, long long nblocks, int f16_scale, hipStream_t st) {
  if (nblocks <= 0) return hipSuccess;
  hipLaunchKernelGGL(quant_q8_kernel, dim3((unsigned)((nblocks * 32 + 255) / 256)), dim3(256), 0, st, x, xq, xs, xsum, nblocks, f16_scale,
                     0LL, 0LL);
  return hipGetLastError();
}

hipError_t ilt_k_quant_q8k(const float* x, int8_t* xq, float* xd, int* bsums, long long nblocks, hipStream_t st) {
  if (nblocks <= 0) return hipSuccess;
  hipLaunchKernelGGL(quant_q8k_kernel<false>, dim3((unsigned)((nblocks + 3) / 4)), dim3(256), 0, st, x, (const float*)nullptr, xq, xd, bsums, nblocks, 0LL, 0LL);
  return hipGetLastError();
}

hipError_t ilt_k_swiglu_quant_q8k(const float* gate, const float* up, int8_t* xq, float* xd, int* bsums, long long nblocks, hipStream_t st) {
  if (nblocks <= 0) return hipSuccess;
  hipLaunchKernelGGL(quant_q8k_kernel<true>, dim3((unsigned)((nblocks + 3) / 4)), dim3(256), 0, st, gate, up, xq, xd, bsums, nblocks, 0LL, 0LL);
  return hipGetLastError();
}

hipError_t ilt_k_quant_rows(int k, const float* x, int8_t* xq, float* xs, int* bsums, long long ntok, int cols, long long x_stride,
                            int f16_scale, hipStream_t st) {
  const int bw = k ? 256 : 32;
  if (ntok <= 0) return hipSuccess;
  if (cols <= 0 || cols % bw != 0 || x_stride < cols || (k && x_stride % 4 != 0)) return hipErrorInvalidValue;
  const long long bpr = cols / bw, nblocks = ntok * bpr;
  if (k) hipLaunchKernelGGL(quant_q8k_kernel<false>, dim3((unsigned)((nblocks + 3) / 4)), dim3(256), 0, st, x, (const float*)nullptr, xq, xs, bsums, nblocks, bpr, x_stride);
  else hipLaunchKernelGGL(quant_q8_kernel, dim3((unsigned)((nblocks * 32 + 255) / 256)), dim3(256), 0, st, x, xq, xs, (int*)nullptr, nblocks,
                          f16_scale, bpr, x_stride);
  return hipGetLastError();
}

hipError_t ilt_k_repack_q8(const uint8_t* raw, int8_t* qs, uint16_t* d, long long nblocks, hipStream_t st) {
  if (nblocks <= 0) return hipSuccess;
  hipLaunchKernelGGL(repack_q8_kernel, dim3((unsigned)((nblocks * 16 + 255) / 256)), dim3(256), 0, st, raw, qs, d, nblocks);
  return hipGetLastError();
}

hipError_t ilt_k_repack_q6k(const uint8_t* raw, uint8_t* out, long long nblocks, hipStream_t st) {
  if (nblocks <= 0) return hipSuccess;
  const long long n = nblocks * (ILT_Q6K_STRIDE / 2);
  hipLaunchKernelGGL(repack_q6k_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, raw, out, nblocks);
  return hipGetLastError();
}

hipError_t ilt_k_copy_bytes(const uint8_t* src, uint8_t* dst, long long bytes, hipStream_t st) {
  if (bytes <= 0) return hipSuccess;
  hipLaunchKernelGGL(copy_bytes_kernel, dim3((unsigned)((bytes / 2 + 256) / 256)), dim3(256), 0, st, src, dst, bytes);
  return hipGetLastError();
}

hipError_t ilt_k_read_through(const unsigned long long* srcs, const unsigned long long* ptrs, int nz, long long add, long long bytes,
                              hipStream_t st) {
  if (bytes <= 0 || nz <= 0) return hipSuccess;
  if (nz > 65535 || (add & 1)) return hipErrorInvalidValue;
  const long long wgs = (bytes / 16 + 255) / 256;
  hipLaunchKernelGGL(read_through_kernel, dim3((unsigned)(wgs < 1 ? 1 : wgs > 64 ? 64 : wgs), (unsigned)nz), dim3(256), 0, st, srcs, ptrs, add, bytes);
  return hipGetLastError();
}

hipError_t ilt_k_dequant_rows(int fmt, const uint8_t* w, const uint16_t* wd, const int* rows_idx, long long nrows,
                              int cols, long long row_bytes, float* out, hipStream_t st) {
  if (nrows <= 0) return hipSuccess;
  const unsigned gx = (unsigned)min((cols + 255) / 256, 64);
  for (long long n0 = 0; n0 < nrows; n0 += 65535) {
    const unsigned gy = (unsigned)min(nrows - n0, (long long)65535);
    hipLaunchKernelGGL(dequant_rows_kernel, dim3(gx, gy), dim3(256), 0, st, fmt, w, wd,
                       rows_idx ? rows_idx + n0 : nullptr, cols, row_bytes, out + n0 * cols);
    if (!rows_idx) w += 65535 * row_bytes, wd = wd ? wd + 65535LL * (cols >> 5) : nullptr;
  }
  return hipGetLastError();
}

hipError_t ilt_k_mm_f16(int ncols, int nrows, int ntok, long long row_halfs, int x_stride, int y_stride, const uint16_t* w, const float* x,
                        float* y, hipStream_t st) {
  if (nrows <= 0 || ntok <= 0) return hipSuccess;
  if (ncols <= 0 || ncols % 16) return hipErrorInvalidValue;
  hipLaunchKernelGGL(mm_f16_dot16_kernel, dim3((ntok + 15) / 16, (nrows + 15) / 16), dim3(256), 0, st, ncols, nrows, ntok, row_halfs, x_stride,
                     y_stride, w, x, y);
  return hipGetLastError();
}
