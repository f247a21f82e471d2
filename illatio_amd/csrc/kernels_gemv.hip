// Decode GEMV kernels for gfx950: y = W.x for W in GGUF Q8_0 / Q4_K / Q6_K / Q2_K /
// IQ2_XXS blocks, x quantized as the reference's CPU path quantizes it (Q8_0 blocks for
// Q8_0 weights, Q8_K blocks for the rest) -- either beforehand or here, by each workgroup
// as it stages x into LDS.
//
// A workgroup (4 waves) stages the activations once and then takes chunks of rows in turn
// (a persistent grid); inside a chunk each wave owns RWW consecutive rows, i.e. one
// contiguous run of RWW*S blocks.  Two phases per wave and chunk:
//   A. Groups of LPB lanes (4; 2 for Q8_0) walk the run block by block, so a wave's
//      128-bit loads cover consecutive bytes, two steps in flight.  Each group forms the
//      block's exact integer sums (v_dot4_i32_i8, DPP adds) and one lane turns them into
//      the block's float terms exactly as the CPU kernels do (tensor.lisp:329-336,
//      kquant.lisp:180-236, iquant.lisp:138-215), into the wave's own piece of LDS.
//   B. One lane per row adds its row's terms in block order: the CPU's sequential sum, so
//      the result has the CPU path's bits.
// One launch may cover several matrices that share x (Q, K, V; gate and up), and may end
// in silu(gate)*up (swiglu!, model.lisp:364-378).
// Two kernels share those phases: gemv_kernel walks its rows with loads two steps ahead (any
// size; the 300 MB output head), gemv_stream_kernel has every wave ask for all of its rows at
// once as direct loads into LDS (products of half a megabyte and more whose share fits a CU's LDS).  The
// host chooses (ilt_gemv_launch).
#include "ilt_device.h"
#include "ilt_iq2xxs_tables.h"
#include "ilt_kernels.h"
#include "ilt_route.h"
#include <type_traits>

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = 4;
constexpr int XP = 256 + 16;   // LDS pitch of one Q8_K activation block: spreads banks

__device__ const u64 ilt_iq2xxs_grid_dev[256] = { ILT_IQ2XXS_GRID_VALUES };

template <int FMT> struct Fmt;
// LPB lanes per block; TERMS floats per block
template <> struct Fmt<ILT_Q8_0>    { static constexpr int LPB = 2, TERMS = 1; };
template <> struct Fmt<ILT_Q4_K>    { static constexpr int LPB = 4, TERMS = 2; };
template <> struct Fmt<ILT_Q6_K>    { static constexpr int LPB = 4, TERMS = 1; };
template <> struct Fmt<ILT_Q2_K>    { static constexpr int LPB = 4, TERMS = 2; };
template <> struct Fmt<ILT_IQ2_XXS> { static constexpr int LPB = 4, TERMS = 1; };

struct Lds {
  const i8* xq;        // Q8_0: cols bytes; Q8_K: XP bytes per block of 256
  const float* xs;     // one scale per activation block
  const int* bsums;    // Q8_K: sums of 16 quants
  const u64* grid;     // IQ2_XXS codebook (256 entries), then its sign masks (128 entries, see iq2_sign_mask)
};

__device__ __forceinline__ int4 and4(const int4& v, int m) { return make_int4(v.x & m, v.y & m, v.z & m, v.w & m); }
__device__ __forceinline__ int4 shr4(const int4& v, int n) {
  return make_int4((u32)v.x >> n, (u32)v.y >> n, (u32)v.z >> n, (u32)v.w >> n);
}
// (two levels of selects, no chain of comparisons: that one becomes branches)
__device__ __forceinline__ int sel4(const int4& v, int i) {
  const int even = (i & 2) ? v.z : v.x, odd = (i & 2) ? v.w : v.y;
  return (i & 1) ? odd : even;
}
__device__ __forceinline__ int4 shl4(const int4& v, int n) {
  return make_int4((int)((u32)v.x << n), (int)((u32)v.y << n), (int)((u32)v.z << n), (int)((u32)v.w << n));
}
__device__ __forceinline__ int4 or_and4(const int4& a, const int4& b, int m) {           // a | (b & m)
  return make_int4(a.x | (b.x & m), a.y | (b.y & m), a.z | (b.z & m), a.w | (b.w & m));
}

// ---- the raw bytes a lane needs for one block (issued early, consumed a step later) ------------
template <int FMT> struct Raw;
template <> struct Raw<ILT_Q8_0> { int4 q; u16 d; };
template <> struct Raw<ILT_Q4_K> { int4 hdr, qa, qb; };
template <> struct Raw<ILT_Q6_K> { int4 ql0, ql1, qh0, qh1, sc; u16 d; };
template <> struct Raw<ILT_Q2_K> { int4 q, sb; u32 dd; };
template <> struct Raw<ILT_IQ2_XXS> { int4 q; u16 d; };

// rw: the wave's rows (for Q8_0 their int8 quants); rd: Q8_0's scales.  f: block within them.
template <int FMT> __device__ __forceinline__ void load_raw(Raw<FMT>& r, __amdgpu_buffer_rsrc_t rw, __amdgpu_buffer_rsrc_t rd, u32 f, int j);
template <> __device__ __forceinline__ void load_raw<ILT_Q8_0>(Raw<ILT_Q8_0>& r, __amdgpu_buffer_rsrc_t rw, __amdgpu_buffer_rsrc_t rd, u32 f, int j) {
  r.q = ilt_bld16(rw, f * 32 + 16 * j);
  r.d = ilt_bld2(rd, f * 2);
}
template <> __device__ __forceinline__ void load_raw<ILT_Q4_K>(Raw<ILT_Q4_K>& r, __amdgpu_buffer_rsrc_t rw, __amdgpu_buffer_rsrc_t, u32 f, int j) {
  const u32 b = f * 144;
  r.hdr = ilt_bld16(rw, b);
  r.qa = ilt_bld16(rw, b + 16 + 32 * j);
  r.qb = ilt_bld16(rw, b + 32 + 32 * j);
}
template <> __device__ __forceinline__ void load_raw<ILT_Q6_K>(Raw<ILT_Q6_K>& r, __amdgpu_buffer_rsrc_t rw, __amdgpu_buffer_rsrc_t, u32 f, int j) {
  const u32 b = f * ILT_Q6K_STRIDE;
  const int c = j >> 1, pp = j & 1;
  r.ql0 = ilt_bld16(rw, b + 64 * c + 32 * pp);
  r.ql1 = ilt_bld16(rw, b + 64 * c + 32 * pp + 16);
  r.qh0 = ilt_bld16(rw, b + 128 + 32 * c);
  r.qh1 = ilt_bld16(rw, b + 128 + 32 * c + 16);
  r.sc = ilt_bld16(rw, b + 192);
  r.d = ilt_bld2(rw, b + 208);
}
template <> __device__ __forceinline__ void load_raw<ILT_Q2_K>(Raw<ILT_Q2_K>& r, __amdgpu_buffer_rsrc_t rw, __amdgpu_buffer_rsrc_t, u32 f, int j) {
  const u32 b = f * 84;
  r.q = ilt_bld16(rw, b + 16 + 16 * j);       // h = j>>1, half = j&1: qs[32h + 16half ..]
  r.sb = ilt_bld16(rw, b);
  r.dd = ilt_bld4(rw, b + 80);
}
template <> __device__ __forceinline__ void load_raw<ILT_IQ2_XXS>(Raw<ILT_IQ2_XXS>& r, __amdgpu_buffer_rsrc_t rw, __amdgpu_buffer_rsrc_t, u32 f, int j) {
  const u32 b = f * 66;
  r.q = ilt_bld16(rw, b + 2 + 16 * j);        // sub-blocks 2j and 2j+1: (grid idx, aux) twice
  r.d = ilt_bld2(rw, b);
}

// One IQ2_XXS sub-block (32 weights): its integer dot with 32 activations.  The sign of
// weight i of an 8-group is bit i of the 7-bit pattern, bit 7 their parity; with m the
// bytes to negate, sum(sign*mag*x) = sum(mag*x) - 2*sum((mag&m)*x).
// The byte masks (0xFF where the weight is negative) of the 128 sign patterns come from a table
// in LDS behind the codebook: building them in registers takes four 32-bit multiplies a pattern,
// which run at a quarter of the rate of the rest.
__device__ __forceinline__ u64 iq2_sign_mask(u32 s7) {      // table entry s7 (0..127)
  const u32 s = s7 | ((__popc(s7) & 1) << 7);
  const u32 mlo = (((s & 0xF) * 0x00204081u) & 0x01010101u) * 0xFFu;
  const u32 mhi = (((s >> 4) * 0x00204081u) & 0x01010101u) * 0xFFu;
  return ((u64)mhi << 32) | mlo;
}
// XR: the 32 activations come from registers (xr) instead of LDS (xb).
template <bool XR = false>
__device__ __forceinline__ int iq2xxs_sub_dot(u32 g, u32 aux, const i8* xb, const u64* grid, const int2* xr = nullptr) {
  // the eight table reads first, then the dots: read one by one, each dot waits out an LDS round trip
  int2 mag[4], m[4];
#pragma unroll
  for (int l = 0; l < 4; l++) {
    mag[l] = ilt_lds_ld8(grid + ((g >> (8 * l)) & 0xFF));
    m[l] = ilt_lds_ld8(grid + 256 + ((aux >> (7 * l)) & 127));
  }
  int pos = 0, neg = 0;
#pragma unroll
  for (int l = 0; l < 4; l++) {
    int2 x;
    if constexpr (XR) x = xr[l]; else x = ilt_lds_ld8(xb + 8 * l);
    pos = ilt_dot4((int)mag[l].y, x.y, ilt_dot4((int)mag[l].x, x.x, pos));
    neg = ilt_dot4((int)(mag[l].y & m[l].y), x.y, ilt_dot4((int)(mag[l].x & m[l].x), x.x, neg));
  }
  return pos - 2 * neg;
}

// ---- phase A for one block: the group's lanes reduce, lane j == 0 writes the terms --------------
template <int FMT> __device__ __forceinline__ void block_terms(const Raw<FMT>& r, int s, int j, const Lds& L, float* t);

template <> __device__ __forceinline__ void block_terms<ILT_Q8_0>(const Raw<ILT_Q8_0>& r, int s, int j, const Lds& L, float* t) {
  const int4 x = ilt_lds_ld16(L.xq + s * 32 + 16 * j);
  const int acc = ilt_sum2(ilt_dot16(r.q, x, 0));
  if (j == 0) ilt_lds_stf(t, (float)acc * (ilt_h2f(r.d) * ilt_lds_ldf(L.xs + s)));
}

template <> __device__ __forceinline__ void block_terms<ILT_Q4_K>(const Raw<ILT_Q4_K>& r, int s, int j, const Lds& L, float* t) {
  const i8* xb = L.xq + ilt_mul24(s, XP) + 64 * j;
  int lo = ilt_dot16(and4(r.qa, 0x0F0F0F0F), ilt_lds_ld16(xb), 0);
  lo = ilt_dot16(and4(r.qb, 0x0F0F0F0F), ilt_lds_ld16(xb + 16), lo);
  int hi = ilt_dot16(and4(shr4(r.qa, 4), 0x0F0F0F0F), ilt_lds_ld16(xb + 32), 0);
  hi = ilt_dot16(and4(shr4(r.qb, 4), 0x0F0F0F0F), ilt_lds_ld16(xb + 48), hi);
  // get_scale_min_k4 for groups 2j and 2j+1 at once, on the two bytes of a 16-bit field of the 12 scale
  // bytes, without a branch: groups 0..3 take six bits of a byte, groups 4..7 a nibble and two top bits
  const int sh = 16 * (j & 1);
  const u32 a = (u32)r.hdr.y >> sh, b = (u32)r.hdr.z >> sh, c = (u32)r.hdr.w >> sh;
  // (both forms computed and one taken by a mask: a branch here would hide the values' ranges from the
  // multiplies below, which then would not be the 24-bit ones)
  const u32 upper = j < 2 ? 0u : 0xFFFFFFFFu;
  const u32 sc = ((a & 0x3F3F) & ~upper) | (((c & 0x0F0F) | ((a >> 2) & 0x3030)) & upper);
  const u32 mn = ((b & 0x3F3F) & ~upper) | ((((c >> 4) & 0x0F0F) | ((b >> 2) & 0x3030)) & upper);
  const int4 bs = ilt_lds_ld16(L.bsums + s * 16 + 4 * j);
  // 24-bit multiplies (full rate): a group's dot is at most 32 * 15 * 128, two sums of 16 at most 32 * 127
  const int isum = ilt_sum4(ilt_mad24(lo, (int)(sc & 0xFF), ilt_mul24(hi, (int)(sc >> 8))));
  const int imin = ilt_sum4(ilt_mad24((int)(mn & 0xFF), bs.x + bs.y, ilt_mul24((int)(mn >> 8), bs.z + bs.w)));
  if (j == 0) {
    const float ydi = ilt_lds_ldf(L.xs + s);
    const float d = ydi * ilt_h2f((u16)(r.hdr.x & 0xFFFF)), dmin = ydi * ilt_h2f((u16)((u32)r.hdr.x >> 16));
    ilt_lds_stf2(t, -(dmin * (float)imin), d * (float)isum);        // (-A, B): the row's sum subtracts A (row_sum)
  }
}

template <> __device__ __forceinline__ void block_terms<ILT_Q6_K>(const Raw<ILT_Q6_K>& r, int s, int j, const Lds& L, float* t) {
  const int c = j >> 1, pp = j & 1;
  const i8* xb = L.xq + ilt_mul24(s, XP) + 128 * c + 32 * pp;
  const int s0 = 2 * pp;                  // (and s1 = s0 + 4)
  // low nibbles: weights 128c + 32pp + l; high nibbles: the same + 64 (l = 0..31)
  // the two top bits of a quant are bits s0, s0 + 1 (low nibbles) and s1, s1 + 1 (high) of its qh byte: one shift
  // by 4 - s0 to the left, or by s1 - 4 = s0 to the right, brings them to bits 4 and 5 (what crosses into a
  // neighbouring byte lands outside the mask)
  const int4 lo0 = or_and4(and4(r.ql0, 0x0F0F0F0F), shl4(r.qh0, 4 - s0), 0x30303030);
  const int4 lo1 = or_and4(and4(r.ql1, 0x0F0F0F0F), shl4(r.qh1, 4 - s0), 0x30303030);
  const int4 hi0 = or_and4(and4(shr4(r.ql0, 4), 0x0F0F0F0F), shr4(r.qh0, s0), 0x30303030);
  const int4 hi1 = or_and4(and4(shr4(r.ql1, 4), 0x0F0F0F0F), shr4(r.qh1, s0), 0x30303030);
  const int dl0 = ilt_dot16(lo0, ilt_lds_ld16(xb), 0), dl1 = ilt_dot16(lo1, ilt_lds_ld16(xb + 16), 0);
  const int dh0 = ilt_dot16(hi0, ilt_lds_ld16(xb + 64), 0), dh1 = ilt_dot16(hi1, ilt_lds_ld16(xb + 80), 0);
  // int8 scales: groups 8c+2pp+{0,1} for the low nibbles, 8c+4+2pp+{0,1} for the high
  const u32 wl = (u32)(c ? r.sc.z : r.sc.x) >> (16 * pp), wh = (u32)(c ? r.sc.w : r.sc.y) >> (16 * pp);
  // (24-bit multiplies, full rate: a dot of 16 is at most 16 * 63 * 128, a sum of 16 at most 16 * 128)
  int isum = ilt_mad24(dl0, (int)(i8)(wl & 0xFF), ilt_mul24(dl1, (int)(i8)((wl >> 8) & 0xFF)));
  isum = ilt_mad24(dh0, (int)(i8)(wh & 0xFF), ilt_mad24(dh1, (int)(i8)((wh >> 8) & 0xFF), isum));
  const u32 wj = (u32)sel4(r.sc, j);
  const int4 bs = ilt_lds_ld16(L.bsums + s * 16 + 4 * j);
  int imins = ilt_mad24(bs.x, (int)(i8)(wj & 0xFF), ilt_mul24(bs.y, (int)(i8)((wj >> 8) & 0xFF)));
  imins = ilt_mad24(bs.z, (int)(i8)((wj >> 16) & 0xFF), ilt_mad24(bs.w, (int)(i8)(wj >> 24), imins));
  isum = ilt_sum4(isum);
  imins = ilt_sum4(imins);
  if (j == 0) ilt_lds_stf(t, (ilt_h2f(r.d) * ilt_lds_ldf(L.xs + s)) * (float)(isum - 32 * imins));
}

// A lane's share of one block's activations (and lane 0's: the block's scale), kept in registers
// over a run of blocks that all sit at the same place in their rows (wave_rows_lds).
template <int FMT> struct XRegs {};
template <> struct XRegs<ILT_IQ2_XXS> { int2 x[8]; float xs; };
template <> struct XRegs<ILT_Q2_K> { int4 x[4]; int4 bs; float xs; };
template <int FMT> __device__ __forceinline__ void load_xregs(XRegs<FMT>& X, int s, int j, const Lds& L);
template <> __device__ __forceinline__ void load_xregs<ILT_IQ2_XXS>(XRegs<ILT_IQ2_XXS>& X, int s, int j, const Lds& L) {
  const i8* xb = L.xq + ilt_mul24(s, XP) + 64 * j;
#pragma unroll
  for (int l = 0; l < 8; l++) X.x[l] = ilt_lds_ld8(xb + 8 * l);
  X.xs = ilt_lds_ldf(L.xs + s);
}
template <> __device__ __forceinline__ void load_xregs<ILT_Q2_K>(XRegs<ILT_Q2_K>& X, int s, int j, const Lds& L) {
  const i8* xb = L.xq + ilt_mul24(s, XP) + 128 * (j >> 1) + 16 * (j & 1);
#pragma unroll
  for (int k = 0; k < 4; k++) X.x[k] = ilt_lds_ld16(xb + 32 * k);
  X.bs = ilt_lds_ld16(L.bsums + s * 16 + 4 * j);
  X.xs = ilt_lds_ldf(L.xs + s);
}

template <bool XR>
__device__ __forceinline__ void block_terms_q2k(const Raw<ILT_Q2_K>& r, int s, int j, const Lds& L, float* t, const XRegs<ILT_Q2_K>* X) {
  const int h = j >> 1, half = j & 1;
  const i8* xb = XR ? nullptr : L.xq + ilt_mul24(s, XP) + 128 * h + 16 * half;
  const u32 wa = (u32)(h ? r.sb.z : r.sb.x) >> (8 * half), wb = (u32)(h ? r.sb.w : r.sb.y) >> (8 * half);
  int isum = 0;
#pragma unroll
  for (int k = 0; k < 4; k++) {
    int4 xk;
    if constexpr (XR) xk = X->x[k]; else xk = ilt_lds_ld16(xb + 32 * k);
    const int dot = ilt_dot16(and4(shr4(r.q, 2 * k), 0x03030303), xk, 0);
    const u32 sw = ((k < 2 ? wa : wb) >> (16 * (k & 1))) & 0xF;
    isum = ilt_mad24((int)sw, dot, isum);
  }
  const u32 wj = (u32)sel4(r.sb, j);
  int4 bs;
  if constexpr (XR) bs = X->bs; else bs = ilt_lds_ld16(L.bsums + s * 16 + 4 * j);
  int mins = ilt_mad24((int)((wj >> 4) & 0xF), bs.x, ilt_mul24((int)((wj >> 12) & 0xF), bs.y));
  mins = ilt_mad24((int)((wj >> 20) & 0xF), bs.z, ilt_mad24((int)(wj >> 28), bs.w, mins));
  isum = ilt_sum4(isum);
  mins = ilt_sum4(mins);
  if (j == 0) {
    float ydb;
    if constexpr (XR) ydb = X->xs; else ydb = ilt_lds_ldf(L.xs + s);
    const float d = ydb * ilt_h2f((u16)(r.dd & 0xFFFF)), dmin = (-ydb) * ilt_h2f((u16)(r.dd >> 16));
    ilt_lds_stf2(t, dmin * (float)mins, d * (float)isum);
  }
}
template <> __device__ __forceinline__ void block_terms<ILT_Q2_K>(const Raw<ILT_Q2_K>& r, int s, int j, const Lds& L, float* t) {
  block_terms_q2k<false>(r, s, j, L, t, nullptr);
}

template <bool XR>
__device__ __forceinline__ void block_terms_iq2xxs(const Raw<ILT_IQ2_XXS>& r, int s, int j, const Lds& L, float* t, const XRegs<ILT_IQ2_XXS>* X) {
  const i8* xb = XR ? nullptr : L.xq + ilt_mul24(s, XP) + 64 * j;
  const u32 aux0 = (u32)r.q.y, aux1 = (u32)r.q.w;
  const float te = (float)iq2xxs_sub_dot<XR>((u32)r.q.x, aux0, xb, L.grid, XR ? X->x : nullptr) * (0.5f + (float)(aux0 >> 28));
  const float to = (float)iq2xxs_sub_dot<XR>((u32)r.q.z, aux1, xb + 32, L.grid, XR ? X->x + 4 : nullptr) * (0.5f + (float)(aux1 >> 28));
  // lane 0 adds the even sub-blocks' terms in order, then the odd ones' (ds4's order)
  float a = 0.0f + te, b = 0.0f + to;
  a = a + ilt_dppf<ILT_DPP_SHL(1)>(te); b = b + ilt_dppf<ILT_DPP_SHL(1)>(to);
  a = a + ilt_dppf<ILT_DPP_SHL(2)>(te); b = b + ilt_dppf<ILT_DPP_SHL(2)>(to);
  a = a + ilt_dppf<ILT_DPP_SHL(3)>(te); b = b + ilt_dppf<ILT_DPP_SHL(3)>(to);
  if (j == 0) ilt_lds_stf(t, (ilt_h2f(r.d) * (XR ? X->xs : ilt_lds_ldf(L.xs + s))) * (a + b));
}
template <> __device__ __forceinline__ void block_terms<ILT_IQ2_XXS>(const Raw<ILT_IQ2_XXS>& r, int s, int j, const Lds& L, float* t) {
  block_terms_iq2xxs<false>(r, s, j, L, t, nullptr);
}

// ---- phase B: a row's terms in block order -------------------------------------------------
// The adds are a chain (a dependent add issues every 8 cycles or so); the LDS reads are not, so 16 terms are on their
// way while the 16 before them are added.  Left to itself the compiler moves every read down to its use and the
// chain waits for LDS once a batch: the reads are inline asm with their own waits.  ds_read2_b32: the terms of a
// row are 4-byte aligned, no more.  A read past the row's end starts again at its last 16 terms instead.
typedef float ilt_f2v __attribute__((ext_vector_type(2)));
#define ILT_TERMS16_AHEAD(A, P)                                                                                                            \
  asm volatile("ds_read2_b32 %0, %8 offset1:1\n\tds_read2_b32 %1, %8 offset0:2 offset1:3\n\tds_read2_b32 %2, %8 offset0:4 offset1:5\n\t"   \
               "ds_read2_b32 %3, %8 offset0:6 offset1:7\n\tds_read2_b32 %4, %8 offset0:8 offset1:9\n\tds_read2_b32 %5, %8 offset0:10 offset1:11\n\t" \
               "ds_read2_b32 %6, %8 offset0:12 offset1:13\n\tds_read2_b32 %7, %8 offset0:14 offset1:15"                                    \
               : "=&v"(A##0), "=&v"(A##1), "=&v"(A##2), "=&v"(A##3), "=&v"(A##4), "=&v"(A##5), "=&v"(A##6), "=&v"(A##7)                  \
               : "v"((u32)(uintptr_t)(ILT_LDS const void*)(P)) : "memory")
#define ILT_TERMS16_WAIT(A, LEFT)                                                                                                          \
  asm volatile("s_waitcnt lgkmcnt(" #LEFT ")" : "+v"(A##0), "+v"(A##1), "+v"(A##2), "+v"(A##3), "+v"(A##4), "+v"(A##5), "+v"(A##6), "+v"(A##7) :: "memory")
#define ILT_TERMS16_ADD(O, A)                                                                                                              \
  do {                                                                                                                                     \
    O = O + (A##0).x; O = O + (A##0).y; O = O + (A##1).x; O = O + (A##1).y; O = O + (A##2).x; O = O + (A##2).y; O = O + (A##3).x; O = O + (A##3).y;        \
    O = O + (A##4).x; O = O + (A##4).y; O = O + (A##5).x; O = O + (A##5).y; O = O + (A##6).x; O = O + (A##6).y; O = O + (A##7).x; O = O + (A##7).y;        \
  } while (0)
__device__ __forceinline__ float chain_terms(const float* t, int n) {       // ((0 + t[0]) + t[1]) + ... + t[n-1]
  float o = 0.0f;
  int q = 0;
  if (n >= 64) {                                // a long row (Q8_0: a term every 32 columns)
    ilt_f2v a0, a1, a2, a3, a4, a5, a6, a7, b0, b1, b2, b3, b4, b5, b6, b7;
    ILT_TERMS16_AHEAD(a, t);
    for (; q + 32 <= n; q += 32) {
      ILT_TERMS16_AHEAD(b, t + q + 16);
      ILT_TERMS16_WAIT(a, 8);
      ILT_TERMS16_ADD(o, a);
      ILT_TERMS16_AHEAD(a, t + min(q + 32, n - 16));
      ILT_TERMS16_WAIT(b, 8);
      ILT_TERMS16_ADD(o, b);
    }
    ILT_TERMS16_WAIT(a, 0);
    if (q + 16 <= n) {                          // a holds terms q .. q+15
      ILT_TERMS16_ADD(o, a);
      q += 16;
    }
  }
  // a short row, or a long one's last terms: eight reads together, then their adds
  for (; q + 8 <= n; q += 8) {
    float v[8];
#pragma unroll
    for (int k = 0; k < 8; k++) v[k] = ilt_lds_ldf(t + q + k);
#pragma unroll
    for (int k = 0; k < 8; k++) o = o + v[k];
  }
  for (; q < n; q++) o = o + ilt_lds_ldf(t + q);
  return o;
}
// Q4_K's two terms a block are stored as -A and B: sum - A + B is sum + (-A) + B to the bit.
template <int FMT> __device__ __forceinline__ float row_sum(const float* t, int S) {
  float sum = chain_terms(t, S * Fmt<FMT>::TERMS);
  if (FMT == ILT_IQ2_XXS) sum = 0.25f * sum;
  return sum;
}


// A wave's rows [row0, row0+nrows) of one matrix: terms into t (nrows*S*TERMS floats, the wave's own).
// No branch inside the run of full steps: the next step's loads (index clamped into the
// run, so always in bounds) are issued before the current step is computed, two register
// sets taking turns; the ragged last step's lanes find their block already loaded.
// The first step's loads of a run, on their own: a wave issues them for its first batch
// before the activations are staged, so the two latencies overlap.
template <int FMT>
__device__ __forceinline__ void first_load(Raw<FMT>& r, const u8* w, const u16* wd, long row0, int nrows, int S,
                                           long row_bytes, int lane) {
  using F = Fmt<FMT>;
  const int j = lane % F::LPB, gl = lane / F::LPB;
  const int nblk = nrows * S;
  const __amdgpu_buffer_rsrc_t wr = ilt_rsrc(ilt_uniform_ptr(w + row0 * row_bytes), __builtin_amdgcn_readfirstlane((u32)(nrows * row_bytes)));
  const __amdgpu_buffer_rsrc_t wdr = ilt_rsrc(ilt_uniform_ptr(wd ? wd + row0 * S : nullptr), wd ? __builtin_amdgcn_readfirstlane((u32)nblk * 2) : 0);
  load_raw<FMT>(r, wr, wdr, min(gl, nblk - 1), j);
}

template <int FMT>
__device__ __forceinline__ void wave_rows(const u8* w, const u16* wd, long row0, int nrows, int S, u32 s_magic,
                                          long row_bytes, const Lds& L, float* t, int lane, const Raw<FMT>& pre, bool use_pre) {
  using F = Fmt<FMT>;
  constexpr int GPW = ILT_WAVE / F::LPB;           // blocks per wave step
  const int j = lane % F::LPB, gl = lane / F::LPB;
  const int nblk = nrows * S, last = nblk - 1;
  const __amdgpu_buffer_rsrc_t wr = ilt_rsrc(ilt_uniform_ptr(w + row0 * row_bytes), __builtin_amdgcn_readfirstlane((u32)(nrows * row_bytes)));
  const __amdgpu_buffer_rsrc_t wdr = ilt_rsrc(ilt_uniform_ptr(wd ? wd + row0 * S : nullptr), wd ? __builtin_amdgcn_readfirstlane((u32)nblk * 2) : 0);
  const int nfull = nblk / GPW;
#define ILT_COMPUTE(reg, ff)                                                           \
  {                                                                                    \
    const int f_ = (ff);                                                               \
    const int s_ = S > 1 ? f_ - (int)__umulhi((u32)f_, s_magic) * S : 0;               \
    block_terms<FMT>(reg, s_, j, L, t + (long)f_ * F::TERMS);                          \
  }
  int f = gl;
  Raw<FMT> ra, rb;
  // (no pointer to the preloaded set anywhere: a set whose address is taken lives in scratch memory)
  if (use_pre) ra = pre; else load_raw<FMT>(ra, wr, wdr, min(f, last), j);
  int k = 0;
  for (; k + 2 <= nfull; k += 2) {
    load_raw<FMT>(rb, wr, wdr, min(f + GPW, last), j);
    ILT_COMPUTE(ra, f)
    load_raw<FMT>(ra, wr, wdr, min(f + 2 * GPW, last), j);
    ILT_COMPUTE(rb, f + GPW)
    f += 2 * GPW;
  }
  if (k < nfull) {
    load_raw<FMT>(rb, wr, wdr, min(f + GPW, last), j);
    ILT_COMPUTE(ra, f)
    f += GPW;
    if (f < nblk) ILT_COMPUTE(rb, f)
  } else if (f < nblk) {
    ILT_COMPUTE(ra, f)
  }
#undef ILT_COMPUTE
}

// silu(g)*u as swiglu! computes it (model.lisp:374): x / (1 + exp(-x)), exp through double
__device__ __forceinline__ float dense_glu(float g, float u) { return (g / (1.0f + ilt_expf_via_double(-g))) * u; }

// ---- activation staging: copy quantized x, or quantize fp32 x here --------------------------------
// Q8_K (quantize-q8k!, kquant.lisp:130-167): 16 lanes a block of 256, so a wave quantizes four
// blocks at once and every reduction stays inside a 16-lane DPP row.  Lane l of a row holds
// the values 4*(l+16i)+c (i, c = 0..3).  The largest-magnitude value, the first of equals,
// sets iscale = -127/max.
__device__ __forceinline__ int ilt_min16(int v) {
  v = min(v, ilt_dpp<ILT_DPP_XOR1>(v)); v = min(v, ilt_dpp<ILT_DPP_XOR2>(v));
  v = min(v, ilt_dpp<ILT_DPP_HALF_MIRROR>(v)); return min(v, ilt_dpp<ILT_DPP_ROW_MIRROR>(v));
}
__device__ __forceinline__ int ilt_or16(int v) {
  v |= ilt_dpp<ILT_DPP_XOR1>(v); v |= ilt_dpp<ILT_DPP_XOR2>(v);
  v |= ilt_dpp<ILT_DPP_HALF_MIRROR>(v); return v | ilt_dpp<ILT_DPP_ROW_MIRROR>(v);
}

// This lane's 16 values of the block its 16-lane row takes in pass PASS (zeros past the end).
template <int NW = kWaves>
__device__ __forceinline__ void load_q8k_pass(const float* __restrict__ x, int nblk, int pass, float4* t) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, g = lane >> 4, l = lane & 15;
  const int b = 4 * wave + 4 * NW * pass + g;
#pragma unroll
  for (int i = 0; i < 4; i++) t[i] = b < nblk ? *(const float4*)(x + b * 256 + 4 * (l + 16 * i)) : make_float4(0.f, 0.f, 0.f, 0.f);
}

// The same without the branch: a lane whose block does not exist reads the last block's values
// instead (the quantizer stores nothing for such a lane).  A conditional load makes the compiler
// wait for it at the join, before whatever the caller wanted to issue next.
template <int NW = kWaves>
__device__ __forceinline__ void load_q8k_pass_clamped(const float* __restrict__ x, int nblk, int pass, float4* t) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, g = lane >> 4, l = lane & 15;
  const int b = min(4 * wave + 4 * NW * pass + g, nblk - 1);
#pragma unroll
  for (int i = 0; i < 4; i++) t[i] = *(const float4*)(x + b * 256 + 4 * (l + 16 * i));
}

// FIRST: the first pass's values, loaded by the caller ahead of time (load_q8k_pass(.., 0, ..)).
// NW: x is weighted first as rmsnorm! weights it, (x * nscale) * nw (model.lisp:215-216), NFIRST
// being nw's first pass; H: those floats are stored as well.  PITCH: bytes from one block's
// quants to the next's at LXQ.
// One pass: this wave's four blocks 4*wave + 4*NW*pass + (0..3).  PRE: the pass's values, loaded by
// the caller ahead of time (load_q8k_pass), or null to load them here; NPRE likewise for nw.
template <int PITCH, int NW, bool SEARCH>
__device__ __forceinline__ bool q8k_pass_impl(const float* __restrict__ x, int nblk, int pass, const float4* pre, i8* lxq, float* lxs, int* lbs,
                                              const float* __restrict__ nw, const float4* npre, float nscale, float* __restrict__ h) {
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), g = lane >> 4, l = lane & 15;
  if (4 * wave + 4 * NW * pass >= nblk) return false;  // none of this wave's four blocks exists
  const int b = 4 * wave + 4 * NW * pass + g;
  const bool live = b < nblk;
  float4 t4[4];
  if (pre) { t4[0] = pre[0]; t4[1] = pre[1]; t4[2] = pre[2]; t4[3] = pre[3]; }
  else load_q8k_pass<NW>(x, nblk, pass, t4);
  if (nw) {
    float4 n4[4];
    if (npre) { n4[0] = npre[0]; n4[1] = npre[1]; n4[2] = npre[2]; n4[3] = npre[3]; }
    else load_q8k_pass<NW>(nw, nblk, pass, n4);
#pragma unroll
    for (int i = 0; i < 4; i++) {
      t4[i] = make_float4((t4[i].x * nscale) * n4[i].x, (t4[i].y * nscale) * n4[i].y, (t4[i].z * nscale) * n4[i].z, (t4[i].w * nscale) * n4[i].w);
      if (h && live) *(float4*)(h + b * 256 + 4 * (l + 16 * i)) = t4[i];
    }
  }
  float v[16];
#pragma unroll
  for (int i = 0; i < 4; i++) { v[4 * i] = t4[i].x; v[4 * i + 1] = t4[i].y; v[4 * i + 2] = t4[i].z; v[4 * i + 3] = t4[i].w; }
  // The block's scale comes from its first value of the largest magnitude, sign and all (quantize-q8k!).  The largest
  // and the smallest value tell which it is unless they are equal in magnitude; the pass is then made again with
  // SEARCH set, which looks for the first position (three instructions a value: a quarter of the pass, for one
  // block in very many).  Without SEARCH there is no branch in here, so that a wave's passes interleave.
  float amax, mx;
  bool tie = false;
  if constexpr (SEARCH) {
    float sa, sm;
    {
      float a8[8];
#pragma unroll
      for (int k = 0; k < 8; k++) a8[k] = fmaxf(fabsf(v[2 * k]), fabsf(v[2 * k + 1]));
      const float am = fmaxf(fmaxf(fmaxf(a8[0], a8[1]), fmaxf(a8[2], a8[3])), fmaxf(fmaxf(a8[4], a8[5]), fmaxf(a8[6], a8[7])));
      const float amax_s = ilt_max16(am);
      // this lane's first position holding the maximum (its values are in rising position order), and the value there
      int idx = 1 << 20;
      float val = 0.0f;
#pragma unroll
      for (int k = 15; k >= 0; k--) {
        const bool hit = fabsf(v[k]) == amax_s;
        idx = hit ? 4 * (l + 16 * (k >> 2)) + (k & 3) : idx;
        val = hit ? v[k] : val;
      }
      const int firstpos = ilt_min16(idx);
      const float mx_s = __int_as_float(ilt_or16(idx == firstpos ? __float_as_int(val) : 0));
      sa = amax_s; sm = mx_s;
    }
    amax = sa; mx = sm;
  } else {
    float hi = fmaxf(fmaxf(fmaxf(v[0], v[1]), fmaxf(v[2], v[3])), fmaxf(fmaxf(v[4], v[5]), fmaxf(v[6], v[7])));
    hi = fmaxf(hi, fmaxf(fmaxf(fmaxf(v[8], v[9]), fmaxf(v[10], v[11])), fmaxf(fmaxf(v[12], v[13]), fmaxf(v[14], v[15]))));
    float lo = fminf(fminf(fminf(v[0], v[1]), fminf(v[2], v[3])), fminf(fminf(v[4], v[5]), fminf(v[6], v[7])));
    lo = fminf(lo, fminf(fminf(fminf(v[8], v[9]), fminf(v[10], v[11])), fminf(fminf(v[12], v[13]), fminf(v[14], v[15]))));
    hi = ilt_max16(hi);
    lo = -ilt_max16(-lo);
    amax = fmaxf(hi, -lo);
    mx = hi >= -lo ? hi : lo;
    if (amax != amax) mx = 0.0f;        // nothing but NaNs: no value is the largest (the CPU's comparisons all fail), the scale is 1 / (-127 / 0)
    tie = hi == -lo && amax != 0.0f;
  }
  const bool nz = amax != 0.0f;
  const float iscale = nz ? -127.0f / mx : 0.0f;
  const float d = nz ? 1.0f / iscale : 0.0f;
  int q[16];
  // (quantize-q8k!'s (min 127 ..) never takes effect: |iscale * v| <= 127 (1 + 2^-23), which rounds to 127)
#pragma unroll
  for (int k = 0; k < 16; k++) q[k] = nz ? (int)rintf(iscale * v[k]) : 0;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int s = ilt_sum4(q[4 * i] + q[4 * i + 1] + q[4 * i + 2] + q[4 * i + 3]);
    if (live) {
      *(int*)(lxq + b * PITCH + 4 * (l + 16 * i)) =
          (q[4 * i] & 0xFF) | ((q[4 * i + 1] & 0xFF) << 8) | ((q[4 * i + 2] & 0xFF) << 16) | ((q[4 * i + 3] & 0xFF) << 24);
      if (lbs && (l & 3) == 0) lbs[b * 16 + (l >> 2) + 4 * i] = s;     // IQ2_XXS takes no 16-sums: none staged
    }
  }
  if (live && l == 0) lxs[b] = d;
  return tie;
}
// A pass, and where a block's largest magnitude comes with both signs (the lanes of that block only) once more.
template <int PITCH, int NW>
__device__ __forceinline__ void q8k_pass(const float* __restrict__ x, int nblk, int pass, const float4* pre, i8* lxq, float* lxs, int* lbs,
                                         const float* __restrict__ nw, const float4* npre, float nscale, float* __restrict__ h) {
  if (q8k_pass_impl<PITCH, NW, false>(x, nblk, pass, pre, lxq, lxs, lbs, nw, npre, nscale, h))
    q8k_pass_impl<PITCH, NW, true>(x, nblk, pass, pre, lxq, lxs, lbs, nw, npre, nscale, h);
}

// All passes; FIRST / NFIRST: the first pass's values (x's, the norm weights'), loaded by the caller.
template <int PITCH, int NW = kWaves>
__device__ __forceinline__ void stage_q8k_from_f32(const float* __restrict__ x, int nblk, i8* lxq, float* lxs, int* lbs, const float4* first,
                                                   const float* __restrict__ nw = nullptr, const float4* nfirst = nullptr,
                                                   float nscale = 1.0f, float* __restrict__ h = nullptr) {
  const int npass = (nblk + 4 * NW - 1) / (4 * NW);
  q8k_pass<PITCH, NW>(x, nblk, 0, first, lxq, lxs, lbs, nw, nfirst, nscale, h);
  for (int pass = 1; pass < npass; pass++) q8k_pass<PITCH, NW>(x, nblk, pass, nullptr, lxq, lxs, lbs, nw, nullptr, nscale, h);
}

// Q8_0 (quantize-q8!, tensor.lisp:245-262): 8 lanes a block of 32.  XSUM: each block's sum of
// quants as well.  NW, NSCALE, H as for the Q8_K staging.
// NP passes of the workgroup's first 256 threads over the blocks' float4s from c0 on: every pass's loads are asked for
// before the first is quantized (a pass a trip to memory otherwise), without a branch around any of them (past the
// end: the last float4 again; nothing is stored for it).
template <int NP>
__device__ __forceinline__ void stage_q8_passes(const float* __restrict__ x, int n8, int c0, int f16_scale, i8* lxq, float* lxs, int* xsum,
                                                const float* __restrict__ nw, float nscale, float* __restrict__ h, int tid, int nthreads) {
  float4 v[NP], n[NP];
  const float* const nwp = nw ? nw : x;
#pragma unroll
  for (int i = 0; i < NP; i++) {
    const int cc = min(c0 + i * nthreads + tid, n8 - 1);
    v[i] = *(const float4*)(x + 4 * cc);
    n[i] = *(const float4*)(nwp + 4 * cc);
  }
#pragma unroll
  for (int i = 0; i < NP; i++) {
    const int c = c0 + i * nthreads + tid;
    float4 w = v[i];
    if (nw) {
      w = make_float4((w.x * nscale) * n[i].x, (w.y * nscale) * n[i].y, (w.z * nscale) * n[i].z, (w.w * nscale) * n[i].w);
      if (h && c < n8) *(float4*)(h + 4 * c) = w;
    }
    float amax = fmaxf(fmaxf(fabsf(w.x), fabsf(w.y)), fmaxf(fabsf(w.z), fabsf(w.w)));
    amax = fmaxf(amax, ilt_dppf<ILT_DPP_XOR1>(amax));
    amax = fmaxf(amax, ilt_dppf<ILT_DPP_XOR2>(amax));
    amax = fmaxf(amax, ilt_dppf<ILT_DPP_HALF_MIRROR>(amax));
    const float d = amax / 127.0f;
    const float id = d == 0.0f ? 0.0f : 1.0f / d;
    const int q0 = (int)rintf(w.x * id), q1 = (int)rintf(w.y * id), q2 = (int)rintf(w.z * id), q3 = (int)rintf(w.w * id);
    const int qs = xsum ? ilt_sum8(q0 + q1 + q2 + q3) : 0;
    if (c < n8) {
      *(int*)(lxq + 4 * c) = (q0 & 0xFF) | ((q1 & 0xFF) << 8) | ((q2 & 0xFF) << 16) | ((q3 & 0xFF) << 24);
      if ((c & 7) == 0) {
        lxs[c >> 3] = f16_scale ? __half2float(__float2half_rn(d)) : d;
        if (xsum) xsum[c >> 3] = qs;
      }
    }
  }
}
// TID, NTHREADS: the threads that stage (a multiple of 8, eight lanes a block), numbered from 0: the workgroup's first
// 256 unless said otherwise.
__device__ __forceinline__ void stage_q8_from_f32(const float* __restrict__ x, int nblk, int f16_scale, i8* lxq, float* lxs,
                                                  int* xsum = nullptr, const float* __restrict__ nw = nullptr, float nscale = 1.0f,
                                                  float* __restrict__ h = nullptr, int tid = -1, int nthreads = kThreads) {
  if (tid < 0) tid = (int)threadIdx.x;
  const int n8 = nblk * 8;
  int c0 = 0;
  for (; c0 + 3 * nthreads < n8; c0 += 4 * nthreads) stage_q8_passes<4>(x, n8, c0, f16_scale, lxq, lxs, xsum, nw, nscale, h, tid, nthreads);
  if (c0 + 2 * nthreads < n8) stage_q8_passes<3>(x, n8, c0, f16_scale, lxq, lxs, xsum, nw, nscale, h, tid, nthreads);
  else if (c0 + nthreads < n8) stage_q8_passes<2>(x, n8, c0, f16_scale, lxq, lxs, xsum, nw, nscale, h, tid, nthreads);
  else if (c0 < n8) stage_q8_passes<1>(x, n8, c0, f16_scale, lxq, lxs, xsum, nw, nscale, h, tid, nthreads);
}

// ---- rmsnorm!'s scale (model.lisp:205-214) ----------------------------------------------------
// The CPU adds the squares (each rounded to a float first) one after another in double and
// scales by 1 / sqrt(float(sum / n + eps)).  Here the workgroup adds them in parallel: another
// order, so the double may differ in its last bits, by less than n * 2^-52 of its value.  Where
// every double that close rounds to the same float, the float is the CPU's; otherwise (about
// one row in ten thousand), or when SEQ asks for it, one thread adds them again in the CPU's order.
__device__ __forceinline__ double sq4(const float4& v) {
  return (((double)(v.x * v.x) + (double)(v.y * v.y)) + (double)(v.z * v.z)) + (double)(v.w * v.w);
}

// The squares of this thread's share of x[0..n) (n a multiple of 4), any share of the whole.
__device__ __forceinline__ double norm_partial(const float* __restrict__ x, int n) {
  double s = 0.0;
  for (int c = threadIdx.x; c < n / 4; c += kThreads) s += sq4(*(const float4*)(x + 4 * c));
  return s;
}

// PART: this thread's part of the sum; all threads of the workgroup call this.
__device__ __forceinline__ float norm_scale(double part, const float* __restrict__ x, int n, float eps, int seq) {
  __shared__ double red[kWaves];
  part = wave_sum_double(part);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = part;
  __syncthreads();
  double sum = red[0];
#pragma unroll
  for (int w = 1; w < kWaves; w++) sum += red[w];
  double v = sum / (double)n + (double)eps;
  const double slack = v * ((double)(n + 8) * 0x1p-51);
  if (seq || (float)(v - slack) != (float)(v + slack)) {       // the same for every thread
    __syncthreads();
    if (threadIdx.x == 0) {
      double s = 0.0;
      for (int i = 0; i < n; i++) { const float xi = x[i]; s += (double)(xi * xi); }
      red[0] = s;
    }
    __syncthreads();
    v = red[0] / (double)n + (double)eps;
  }
  return 1.0f / sqrtf((float)v);
}

template <int FMT>
__device__ __forceinline__ void run_rows(const IltGemvMat& m, const IltGemvParams& p, long row0, int nrows, int S,
                                         const Lds& L, float* t, int lane, int z, const Raw<FMT>& pre, bool use_pre) {
  const u8* w = p.ptrs ? (const u8*)(p.ptrs[p.sel ? p.sel[z] : z] + m.add) : m.w;
  wave_rows<FMT>(w, m.wd, row0, nrows, S, p.s_magic, m.row_bytes, L, t, lane, pre, use_pre);
}

// FSET: one format (its GGUF number), or 0 = the launch's matrices mix Q4_K and Q6_K
// The preloaded first step: one register set for the launch's format (two when they mix)
template <int FSET> struct Pre {
  Raw<(FSET ? FSET : ILT_Q4_K)> a;
  Raw<(FSET ? FSET : ILT_Q6_K)> b;      // used only when FSET == 0, for a Q6_K matrix
};

template <int FSET>
__device__ __forceinline__ void run_any(const IltGemvMat& m, const IltGemvParams& p, long row0, int nrows, int S,
                                        const Lds& L, float* t, int lane, int z, const Pre<FSET>& pre, bool use_pre) {
  if constexpr (FSET != 0) run_rows<FSET>(m, p, row0, nrows, S, L, t, lane, z, pre.a, use_pre);
  else if (m.fmt == ILT_Q4_K) run_rows<ILT_Q4_K>(m, p, row0, nrows, S, L, t, lane, z, pre.a, use_pre);
  else run_rows<ILT_Q6_K>(m, p, row0, nrows, S, L, t, lane, z, pre.b, use_pre);
}

__device__ __forceinline__ float sum_any(int fmt, const float* t, int S) {
  switch (fmt) {
    case ILT_Q8_0: return row_sum<ILT_Q8_0>(t, S);
    case ILT_Q4_K: return row_sum<ILT_Q4_K>(t, S);
    case ILT_Q6_K: return row_sum<ILT_Q6_K>(t, S);
    case ILT_Q2_K: return row_sum<ILT_Q2_K>(t, S);
    default: return row_sum<ILT_IQ2_XXS>(t, S);
  }
}

// FSET: the format of every matrix of the launch, or 0 when they mix Q4_K and Q6_K.  The
// expert formats (IQ2_XXS, Q2_K) take grid y = expert.
// (z: grid y, which chooses the expert; xy: the row of activations and of the output it works on)
template <int FSET>
__device__ __forceinline__ void gemv_body(const IltGemvParams& p, const int z, const long xy, unsigned char* smem) {
  constexpr bool q8 = FSET == ILT_Q8_0;
  const int S = q8 ? p.cols / 32 : p.cols / 256;
  // LDS: xq | bsums | xs | (grid) | terms (per wave)
  i8* lxq = (i8*)smem;
  const int xq_bytes = q8 ? p.cols : S * XP;
  int* lbs = (int*)(smem + xq_bytes);
  const int nbs = (q8 || FSET == ILT_IQ2_XXS) ? 0 : p.cols / 16;
  float* lxs = (float*)(lbs + nbs);
  u64* lgrid = (u64*)(((uintptr_t)(lxs + S) + 7) & ~(uintptr_t)7);
  float* terms = (float*)(lgrid + (FSET == ILT_IQ2_XXS ? 384 : 0));

  // grouped rows (d4_mvq8): wgs_per_group workgroups share one group's rows and activations
  const int group = p.group_rows > 0 ? blockIdx.x / p.wgs_per_group : 0;
  const int wg_in = p.group_rows > 0 ? blockIdx.x % p.wgs_per_group : blockIdx.x;
  const int nwg = p.group_rows > 0 ? p.wgs_per_group : gridDim.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int RB = p.batch;                             // rows per batch

  // Batches of RB rows (never across two matrices) are dealt out to the grid's waves in turn,
  // so at any time the waves' reads lie close together in memory.
  const int nw = nwg * kWaves, wid = wg_in * kWaves + wave;
  const long grow0 = (long)group * p.group_rows;      // first row of this group (0 when ungrouped)
  auto locate = [&](int b, int& mi, long& row0, int& nrows) {
    mi = 0;
    if (!p.glu) while (mi + 1 < p.nmat && b >= p.mat[mi + 1].batch0) mi++;
    // the rows dealt out evenly over the matrix's batches: rq each, one more for the first rr
    const int bl = b - p.mat[mi].batch0, rq = p.mat[mi].rq, rr = p.mat[mi].rr;
    row0 = (long)bl * rq + min(bl, rr) + grow0;
    nrows = rq + (bl < rr ? 1 : 0);
  };

  // Float activations to quantize here: their first loads go out before any weight load, since
  // loads return in order and these (hot in L2) are needed first.
  const long xoff = xy * p.x_stride + (long)group * p.cols;
  float4 xfirst[4], nfirst[4];
  if (!q8 && p.xf) load_q8k_pass(p.xf + xoff, S, 0, xfirst);
  // ... and when they are normalized first: the norm's weights likewise, and now the squares
  // of what xfirst does not hold
  double sq = 0.0;
  if (p.norm_w) {
    if (q8) sq = norm_partial(p.xf + xoff, p.cols);
    else {
      load_q8k_pass(p.norm_w, S, 0, nfirst);
      for (int pass = 1; pass * 4 * kWaves < S; pass++) {
        float4 t[4];
        load_q8k_pass(p.xf + xoff, S, pass, t);
        sq += (sq4(t[0]) + sq4(t[1])) + (sq4(t[2]) + sq4(t[3]));
      }
    }
  }
  // the first batch's first loads go out now, so they are on their way while x is staged
  Pre<FSET> pre;
  int warm[4] = {0, 0, 0, 0};
  if (wid < p.nbatches) {
    int mi; long row0; int nrows;
    locate(wid, mi, row0, nrows);
    const IltGemvMat& m = p.mat[mi];
    const u8* w0 = p.ptrs ? (const u8*)(p.ptrs[p.sel ? p.sel[z] : z] + m.add) : m.w;
    if (FSET != 0 || m.fmt == ILT_Q4_K) first_load<(FSET ? FSET : ILT_Q4_K)>(pre.a, w0, m.wd, row0, nrows, S, m.row_bytes, lane);
    else first_load<(FSET ? FSET : ILT_Q6_K)>(pre.b, w0, m.wd, row0, nrows, S, m.row_bytes, lane);
    // and a touch of every 64-byte line of the batch's first 16 KB, so the later steps hit in L2 -- where the touched
    // lines of all the grid's waves together fit the dies' L2s (32 MB): in a launch of thousands of waves (the output
    // head: 64 MB touched at once) most are evicted again before their wave reads them, and the matrix is then
    // fetched 1.12 times over
    const u8* wb = w0 + row0 * m.row_bytes;
    const long bytes = (long)nrows * m.row_bytes;
    // (the values are looked at only when the kernel ends: nothing waits for these loads here)
    if ((long)nw * 16384 <= (24L << 20)) {
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const long o = 64L * lane + 4096L * i;
        if (o < bytes) warm[i] = *(const int*)(wb + (o & ~3L));
      }
    }
  }

  // ---- stage the activations ----
  if (p.xf) {
    float nscale = 1.0f;
    if (p.norm_w) {
      if (!q8) sq += (sq4(xfirst[0]) + sq4(xfirst[1])) + (sq4(xfirst[2]) + sq4(xfirst[3]));
      nscale = norm_scale(sq, p.xf + xoff, p.cols, p.eps, p.norm_seq);
    }
    if (q8) stage_q8_from_f32(p.xf + xoff, S, p.f16_scale, lxq, lxs, nullptr, p.norm_w, nscale);
    else stage_q8k_from_f32<XP>(p.xf + xoff, S, lxq, lxs, nbs ? lbs : nullptr, xfirst, p.norm_w, nfirst, nscale);
  } else {
    const i8* gxq = p.xq + xoff;
    if (q8) {
      for (int i = threadIdx.x * 16; i < p.cols; i += kThreads * 16) *(int4*)(lxq + i) = *(const int4*)(gxq + i);
      for (int i = threadIdx.x; i < S; i += kThreads) lxs[i] = p.xs[xoff / 32 + i];
    } else {
      for (int i = threadIdx.x; i < S * 16; i += kThreads)
        *(int4*)(lxq + (i >> 4) * XP + 16 * (i & 15)) = *(const int4*)(gxq + 16 * i);
      for (int i = threadIdx.x; i < S; i += kThreads) lxs[i] = p.xs[xoff / 256 + i];
      for (int i = threadIdx.x; i < nbs; i += kThreads) lbs[i] = p.bsums[xoff / 16 + i];
    }
  }
  if (FSET == ILT_IQ2_XXS) {
    lgrid[threadIdx.x] = ilt_iq2xxs_grid_dev[threadIdx.x];
    if (threadIdx.x < 128) lgrid[256 + threadIdx.x] = iq2_sign_mask(threadIdx.x);
  }
  __syncthreads();

  const Lds L = { lxq, lxs, lbs, lgrid };
  const int tpr = q8 ? S : S * 2;                     // floats of terms per row (the larger TERMS)
  float* tw = terms + (long)wave * RB * tpr * (p.glu ? 2 : 1);

  for (int b = wid; b < p.nbatches; b += nw) {
    int mi; long row0; int nrows;
    locate(b, mi, row0, nrows);
    const IltGemvMat& m = p.mat[mi];
    const int fmt = FSET != 0 ? FSET : m.fmt;
    run_any<FSET>(m, p, row0, nrows, S, L, tw, lane, z, pre, b == wid);
    if (p.glu) run_any<FSET>(p.mat[1], p, row0, nrows, S, L, tw + (long)RB * tpr, lane, z, pre, false);   // the same rows of up
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    if (lane < nrows) {
      const int tper = (fmt == ILT_Q4_K || fmt == ILT_Q2_K) ? 2 : 1;
      float v = FSET != 0 ? row_sum<(FSET ? FSET : ILT_Q4_K)>(tw + (long)lane * S * tper, S) : sum_any(fmt, tw + (long)lane * S * tper, S);
      const long r = row0 + lane;
      if (p.glu) {
        const int ufmt = FSET != 0 ? FSET : p.mat[1].fmt;
        const float uv = sum_any(ufmt, tw + (long)RB * tpr + (long)lane * S * ((ufmt == ILT_Q4_K || ufmt == ILT_Q2_K) ? 2 : 1), S);
        float* y = m.y + xy * p.y_stride;
        if (p.glu == 1) {
          y[r] = dense_glu(v, uv);
        } else {        // the experts' gated activation, as d4_swiglu_w computes it
          float gv = v, uu = uv;
          if (p.clamp > 1e-6f) { gv = fminf(gv, p.clamp); uu = fmaxf(-p.clamp, fminf(uu, p.clamp)); }
          float o = ilt_silu(gv) * uu;
          if (p.wts) o = o * p.wts[xy];
          y[r] = o;
        }
      } else {
        float* y = m.y + xy * p.y_stride;
        if (m.bias) v = v + m.bias[r];
        if (p.acc) v = y[r] + v;
        y[r] = v;
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
  }
  asm volatile("" :: "v"(warm[0]), "v"(warm[1]), "v"(warm[2]), "v"(warm[3]));
}

template <int FSET>
__global__ __launch_bounds__(kThreads) void gemv_kernel(IltGemvParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  gemv_body<FSET>(p, blockIdx.y, blockIdx.y, smem);
}

// Grid y's expert on its counts[y] rows of activations, one after another: the rows after the first find the matrix
// in the cache (ds4f.cu:762-772).  An expert with no rows ends at once.
template <int FSET>
__global__ __launch_bounds__(kThreads) void gemv_rows_kernel(IltGemvParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int z = blockIdx.y, n = (int)p.counts[z];
  const long t0 = p.bases[z];
  for (int tk = 0; tk < n; tk++) {
    if (tk) __syncthreads();                           // the row before is through with the staged activations
    gemv_body<FSET>(p, z, t0 + tk, smem);
  }
}

// ---- the streamed variant: matrices of up to ~100 KB per CU, every format ---------------------------
// A mid-size product (6-28 MB) is over before its loop's load -> use -> load chain has made a few
// round trips to memory: its time is latency, not bytes.  Here every row wave asks for its whole
// share of the rows at once, as direct loads from global memory into its own piece of LDS; the
// matrix streams in at the memory's rate while other waves quantize the activations, and the
// blocks' terms are then formed from LDS.  One workgroup a CU, one batch of rows a wave.
// A block in LDS: LB bytes as PPB pieces of 16 bytes, every piece 16-byte aligned there whatever the
// block's size in memory (BB); goff(pc) = where piece pc comes from within the block.  No piece
// reaches past its block's end (the last block of a matrix may be the last bytes of an allocation).
template <int FMT> struct LdsBlk;
template <> struct LdsBlk<ILT_Q4_K> {
  static constexpr int LB = 144, PPB = 9, BB = 144;
  static __device__ __forceinline__ u32 goff(u32 pc) { return 16 * pc; }
};
// Q6_K: 212 bytes spread to 224; the last piece is bytes 196..211, so the scale d lands at 220.
template <> struct LdsBlk<ILT_Q6_K> {
  static constexpr int LB = 224, PPB = 14, BB = ILT_Q6K_STRIDE;
  static __device__ __forceinline__ u32 goff(u32 pc) { return pc == 13 ? 196u : 16 * pc; }
};
// IQ2_XXS: 66 bytes (d, then 8 sub-blocks of 8 bytes) as the four 16-byte pairs of sub-blocks, then
// the block's first 16 bytes, whose first two are d: d lands at 64.
template <> struct LdsBlk<ILT_IQ2_XXS> {
  static constexpr int LB = 80, PPB = 5, BB = 66;
  static __device__ __forceinline__ u32 goff(u32 pc) { return pc == 4 ? 0u : 2 + 16 * pc; }
};
// Q2_K: 84 bytes (16 scale bytes, 64 of quants, d and dmin) as those five pieces and bytes 68..83,
// whose last four are d and dmin: they land at 92.
template <> struct LdsBlk<ILT_Q2_K> {
  static constexpr int LB = 96, PPB = 6, BB = 84;
  static __device__ __forceinline__ u32 goff(u32 pc) { return pc == 5 ? 68u : 16 * pc; }
};

// Q8_0 (split at upload): the quants as they are, two pieces a block; the f16 scales are a second
// run, copied four bytes a lane (stream_scales) behind the quants' room.
template <> struct LdsBlk<ILT_Q8_0> {
  static constexpr int LB = 32, PPB = 2, BB = 32;
  static __device__ __forceinline__ u32 goff(u32 pc) { return 16 * pc; }
};

// NBYTES (a multiple of 4) from src to LDS, four bytes a lane.  Returns the number of instructions.
__device__ __forceinline__ int stream_scales(const u8* src_, int nbytes, u8* lds, int lane) {
  const u8* src = (const u8*)ilt_uniform_ptr(src_);
  const int n4 = __builtin_amdgcn_readfirstlane(nbytes >> 2), nfull = n4 >> 6, tail = n4 & 63;
  for (int i = 0; i < nfull; i++)
    __builtin_amdgcn_global_load_lds((const ILT_GLOBAL void*)(src + (i * 64 + lane) * 4), (ILT_LDS void*)(lds + i * 256), 4, 0, 0);
  if (tail && lane < tail)
    __builtin_amdgcn_global_load_lds((const ILT_GLOBAL void*)(src + (nfull * 64 + lane) * 4), (ILT_LDS void*)(lds + nfull * 256), 4, 0, 0);
  return nfull + (tail ? 1 : 0);
}

// Returns the number of load instructions issued (the same in every lane).
template <int FMT>
__device__ __forceinline__ int stream_run(const u8* w, long row0, int nrows, int S, long row_bytes, u8* lds_run, int lane) {
  using B = LdsBlk<FMT>;
  const u8* src = (const u8*)ilt_uniform_ptr(w + row0 * row_bytes);
  const int npieces = __builtin_amdgcn_readfirstlane(nrows * S * B::PPB);
  const int nfull = npieces >> 6, tail = npieces & 63;
  // this lane's piece of the first instruction; each further instruction is 64 pieces on
  u32 blk = (u32)lane / B::PPB, pc = (u32)lane % B::PPB;
  for (int i = 0; i < nfull; i++) {
    ilt_g2lds16(src + blk * B::BB + B::goff(pc), lds_run + i * 1024);
    blk += 64 / B::PPB; pc += 64 % B::PPB;
    if (pc >= B::PPB) { pc -= B::PPB; blk += 1; }
  }
  if (tail && lane < tail) ilt_g2lds16(src + blk * B::BB + B::goff(pc), lds_run + nfull * 1024);   // the lanes past the end load nothing
  return nfull + (tail ? 1 : 0);
}

// run2: Q8_0's scales (unused by the rest)
template <int FMT> __device__ __forceinline__ void load_raw_lds(Raw<FMT>& r, const u8* run, const u8* run2, u32 f, int j);
template <> __device__ __forceinline__ void load_raw_lds<ILT_Q8_0>(Raw<ILT_Q8_0>& r, const u8* run, const u8* run2, u32 f, int j) {
  r.q = ilt_lds_ld16(run + f * LdsBlk<ILT_Q8_0>::LB + 16 * j);
  r.d = *ILT_LDS_PTR(const u16, run2 + 2 * f);
}
template <> __device__ __forceinline__ void load_raw_lds<ILT_Q4_K>(Raw<ILT_Q4_K>& r, const u8* run, const u8*, u32 f, int j) {
  const u8* b = run + f * LdsBlk<ILT_Q4_K>::LB;
  r.hdr = ilt_lds_ld16(b);
  r.qa = ilt_lds_ld16(b + 16 + 32 * j);
  r.qb = ilt_lds_ld16(b + 32 + 32 * j);
}
template <> __device__ __forceinline__ void load_raw_lds<ILT_Q6_K>(Raw<ILT_Q6_K>& r, const u8* run, const u8*, u32 f, int j) {
  const u8* b = run + f * LdsBlk<ILT_Q6_K>::LB;
  const int c = j >> 1, pp = j & 1;
  r.ql0 = ilt_lds_ld16(b + 64 * c + 32 * pp);
  r.ql1 = ilt_lds_ld16(b + 64 * c + 32 * pp + 16);
  r.qh0 = ilt_lds_ld16(b + 128 + 32 * c);
  r.qh1 = ilt_lds_ld16(b + 128 + 32 * c + 16);
  r.sc = ilt_lds_ld16(b + 192);
  r.d = *ILT_LDS_PTR(const u16, b + 220);
}
template <> __device__ __forceinline__ void load_raw_lds<ILT_IQ2_XXS>(Raw<ILT_IQ2_XXS>& r, const u8* run, const u8*, u32 f, int j) {
  const u8* b = run + f * LdsBlk<ILT_IQ2_XXS>::LB;
  r.q = ilt_lds_ld16(b + 16 * j);
  r.d = *ILT_LDS_PTR(const u16, b + 64);
}
template <> __device__ __forceinline__ void load_raw_lds<ILT_Q2_K>(Raw<ILT_Q2_K>& r, const u8* run, const u8*, u32 f, int j) {
  const u8* b = run + f * LdsBlk<ILT_Q2_K>::LB;
  r.q = ilt_lds_ld16(b + 16 + 16 * j);
  r.sb = ilt_lds_ld16(b);
  r.dd = *ILT_LDS_PTR(const u32, b + 92);
}

// A wave's run of nrows*S blocks, in LDS: terms into t.
template <int FMT>
__device__ __forceinline__ void wave_rows_lds(const u8* run, const u8* run2, int nrows, int S, u32 s_magic, const Lds& L, float* t, int lane) {
  using F = Fmt<FMT>;
  constexpr int GPW = ILT_WAVE / F::LPB;
  const int j = lane % F::LPB, gl = lane / F::LPB;
  const int nblk = nrows * S;
  // the block's place in its row, f mod S, kept by addition (a division by multiplication takes two
  // quarter-rate instructions a step)
  const int step = S > 1 ? GPW - (int)__umulhi((u32)GPW, s_magic) * S : 0;      // GPW mod S
  int s_ = S > 1 ? gl - (int)__umulhi((u32)gl, s_magic) * S : 0;
  if constexpr (FMT == ILT_IQ2_XXS || FMT == ILT_Q2_K) {
    // the experts' widths (4096, 2048 columns: S = 16, 8) divide the 16 blocks of a step: a lane's blocks all sit
    // at one place in their rows, so its share of the activations is read from LDS once, not once a row
    if (step == 0 && nblk > GPW) {
      XRegs<FMT> X;
      load_xregs<FMT>(X, s_, j, L);
      for (int f = gl; f < nblk; f += GPW) {
        Raw<FMT> r;
        load_raw_lds<FMT>(r, run, run2, f, j);
        if constexpr (FMT == ILT_IQ2_XXS) block_terms_iq2xxs<true>(r, s_, j, L, t + (long)f * F::TERMS, &X);
        else block_terms_q2k<true>(r, s_, j, L, t + (long)f * F::TERMS, &X);
      }
      return;
    }
  }
  for (int f = gl; f < nblk; f += GPW) {
    Raw<FMT> r;
    load_raw_lds<FMT>(r, run, run2, f, j);
    block_terms<FMT>(r, s_, j, L, t + (long)f * F::TERMS);
    s_ += step;
    if (s_ >= S) s_ -= S;
  }
}

// 16 waves a workgroup (four a SIMD), in two roles.  Waves 0-3 load and quantize the activations
// and have no rows; waves 4-15 send off the loads of their rows at once and wait.  So the
// quantizer's chain of dependent instructions runs while the matrix streams in, and no wave
// has activation loads queued ahead of matrix loads (loads return in the order issued: waiting
// for the first would mean counting the second, whose number is not known at compile time).
constexpr int kStreamWaves = 16, kStreamThreads = 64 * kStreamWaves, kStagers = 4, kRowWaves = kStreamWaves - kStagers;

// rmsnorm!'s scale (see norm_scale) in the streamed kernel: the first kStagers waves hold the
// squares; the other waves have no part in it.
// The four activation waves meet three times on the way (partial sums written; read by all before one of them is
// written again; the sum added again where that was needed).  They meet through counters in LDS, cleared at the
// kernel's start: s_barrier would have to be reached by the row waves too, and those are held up while they send off
// their loads (the memory pipeline takes a wave's loads at the rate the rows arrive: the last row wave of a 28 MB
// launch reaches a barrier 4 us into the launch).  meet: this wave's LDS writes are done, it counts itself, and waits
// until all four have; nothing that is waited for waits for anything itself, the polls are bounded all the same.
__device__ __forceinline__ void stagers_meet(u32* slot) {
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  if ((threadIdx.x & 63) == 0) __hip_atomic_fetch_add(slot, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  for (int polls = 0; polls < (1 << 22); polls++) {
    if (__hip_atomic_load(slot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) >= (u32)kStagers) break;
    __builtin_amdgcn_s_sleep(1);
  }
  asm volatile("" ::: "memory");
}
__device__ __forceinline__ float norm_scale_stagers(double part, const float* __restrict__ x, int n, float eps, int seq, u32* meet) {
  __shared__ double red[kStagers];
  part = wave_sum_double(part);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = part;
  stagers_meet(meet);
  double sum = red[0];
#pragma unroll
  for (int w = 1; w < kStagers; w++) sum += red[w];
  double v = sum / (double)n + (double)eps;
  const double slack = v * ((double)(n + 8) * 0x1p-51);
  const bool again = seq || (float)(v - slack) != (float)(v + slack);       // the same for every thread
  stagers_meet(meet + 1);
  if (again && threadIdx.x == 0) {
    double s = 0.0;
    for (int i = 0; i < n; i++) { const float xi = x[i]; s += (double)(xi * xi); }
    red[0] = s;
  }
  stagers_meet(meet + 2);
  if (again) v = red[0] / (double)n + (double)eps;
  return 1.0f / sqrtf((float)v);
}

// Calls f(integral_constant<int, FMT>) for the format FMT of a matrix.
template <int FSET, typename F>
__device__ __forceinline__ void with_format(int fmt, F&& f) {
  if constexpr (FSET != 0) f(std::integral_constant<int, FSET>{});
  else if (fmt == ILT_Q4_K) f(std::integral_constant<int, ILT_Q4_K>{});
  else f(std::integral_constant<int, ILT_Q6_K>{});
}
__device__ __forceinline__ int lds_block_bytes(int fmt) {
  return fmt == ILT_Q4_K ? 144 : fmt == ILT_Q6_K ? 224 : fmt == ILT_Q2_K ? 96 : fmt == ILT_Q8_0 ? 32 : 80;
}

// What the activation waves (256 threads a workgroup) read ahead for the next launch; the values go nowhere, the
// lines stay in this die's L2.  The loads queue behind the row waves' (all asked for at the kernel's start), so they
// take memory's time when the rows have arrived.
__device__ __forceinline__ void cache_ahead(const IltCacheAhead& h, float* sink) {
  const int die = blockIdx.x & 7, w4 = h.width[die] >> 2;
  const int me = (int)(blockIdx.x >> 3) * (64 * kStagers) + (int)threadIdx.x, all = (int)((gridDim.x + 7) >> 3) * (64 * kStagers);
  float keep = 0.0f;
  if (w4 > 0) {
    // four pieces of each array a thread at a time, all asked for before any is looked at (a piece a trip to memory
    // otherwise); past the end the last piece again
    const int total = h.nrows * w4;
    for (int i0 = me; i0 < total; i0 += 4 * all) {
      float4 x[4], y[4];
#pragma unroll
      for (int u = 0; u < 4; u++) {
        const int i = min(i0 + u * all, total - 1), row = i / w4, c = i - row * w4;
        const long long o = (long long)row * h.stride + h.off[die] + 4 * c;
        x[u] = *(const float4*)(h.a + o); y[u] = *(const float4*)(h.b + o);
      }
#pragma unroll
      for (int u = 0; u < 4; u++) keep += (x[u].x + x[u].y + x[u].z + x[u].w) + (y[u].x + y[u].y + y[u].z + y[u].w);
    }
  }
  if ((blockIdx.x >> 3) == 0) {
#pragma unroll
    for (int r = 0; r < 3; r++)
      if (h.small[r]) for (int i = threadIdx.x; i < h.nsmall[r]; i += 64 * kStagers) keep += h.small[r][i];
  }
  if (keep == 1.2345678e38f) *sink = keep;               // (never: the loads must not be dropped)
}

// The next product's rows for this die, a 128-byte line a lane (one dword of a line brings the line into L2).  Batch b of
// the next launch goes to its workgroup b % 256, die b % 8: this die's batches of matrix i are bl = r0, r0 + 8, ...
__device__ __forceinline__ void rows_ahead(const IltRowsAhead& h, float* sink) {
  const int die = blockIdx.x & 7;
  const int me = (int)(blockIdx.x >> 3) * (64 * kStagers) + (int)threadIdx.x, all = (int)((gridDim.x + 7) >> 3) * (64 * kStagers);
  u32 keep = 0;
  for (int i = 0; i < h.nm; i++) {
    const IltRowsAhead::M& m = h.m[i];
    const int r0 = (((die - m.batch0) % 8) + 8) % 8;
    if (r0 >= m.nbat) continue;
    const int K = (m.nbat - r0 + 7) >> 3;
    const int maxl = (int)(((long long)(m.rq + 1) * m.row_bytes + 127) >> 7) + 1;      // lines a batch, at most
    const int total = K * maxl;
    for (int i0 = me; i0 < total; i0 += 4 * all) {
      u32 v[4];
#pragma unroll
      for (int u = 0; u < 4; u++) {
        const int j = min(i0 + u * all, total - 1), k = j / maxl, ll = j - k * maxl, bl = r0 + 8 * k;
        const long long row0 = (long long)bl * m.rq + min(bl, m.rr), nrows = m.rq + (bl < m.rr ? 1 : 0);
        const u64 start = (u64)(uintptr_t)m.w + (u64)(row0 * m.row_bytes), end = start + (u64)(nrows * m.row_bytes);
        const u64 a = min((start & ~127ULL) + 128ULL * (u64)ll, (end - 1) & ~127ULL);     // past the batch's end: its last line again
        v[u] = *(const u32*)(uintptr_t)max(a, start & ~3ULL);                            // (never before the batch's first dword)
      }
      keep ^= (v[0] ^ v[1]) ^ (v[2] ^ v[3]);
    }
  }
  if (keep == 0x9E3779B9u && h.nm < 0) *sink = 0.0f;       // (never: the loads must not be dropped)
}

// FSET: ILT_Q4_K, ILT_Q6_K, 0 (those two mixed), or the expert formats ILT_IQ2_XXS, ILT_Q2_K (then
// p.ptrs gives the experts' slots and p.nz how many take part: a batch is rows of one expert,
// batches per expert = p.mat[0].nbat).  p.batch = the most rows a wave takes; p.region = bytes
// of LDS per wave for its rows (both matrices' when glu).
// EARLY 1: the launch adds to y or has a bias (never a gate/up pair): those values are asked for behind the rows.
// EARLY 2: the launch adds its rows to an ordered sum of up to eight vectors (IltSumAlong), asked for likewise.
template <int FSET, int EARLY = 0>
__global__ __launch_bounds__(kStreamThreads) void gemv_stream_kernel(IltGemvParams p) {
  static_assert(offsetof(IltGemvParams, route) <= 456 && sizeof(IltGemvParams) >= 448, "ilt_kernarg_warm7 covers the arguments' first 448 bytes");
  ilt_kernarg_warm7();
  __shared__ u32 s_meet[4];            // the norm's three meetings of the activation waves (stagers_meet)
  asm volatile("" ::"s"(p.norm_w), "s"(p.cols), "s"(p.x_stride), "s"(p.nz));      // (read together with what every wave reads first anyway)
  if (p.norm_w) {                      // (the workgroup's waves start within a few cycles of one another: this barrier is cheap)
    if (threadIdx.x < 4) s_meet[threadIdx.x] = 0;
    ilt_barrier_lds();
  }
  extern __shared__ __align__(16) unsigned char smem[];
  constexpr bool iq2 = FSET == ILT_IQ2_XXS, q8 = FSET == ILT_Q8_0;
  const int S = q8 ? p.cols / 32 : p.cols / 256;
  const int nx = p.x_stride ? p.nz : 1;                  // activation vectors staged (one per expert, or one for all)
  const int SX = S * nx;
  i8* lxq = (i8*)smem;
  int* lbs = (int*)(smem + (q8 ? p.cols : SX * XP));
  float* lxs = (float*)(lbs + ((iq2 || q8) ? 0 : SX * 16));
  u64* lgrid = (u64*)(((uintptr_t)(lxs + SX) + 15) & ~(uintptr_t)15);
  float* terms = (float*)(lgrid + (iq2 ? 384 : 0));
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);     // the same in every lane, said so
  const int tpr = q8 ? S : S * 2, nglu = p.glu ? 2 : 1;

  // 1. the activations into LDS, by the first four waves
  if (wave < kStagers && q8) {
    // A token's routing carried along (IltRouteAlong): the first workgroup's first wave does not stage -- its other
    // three activation waves take its share -- but reads its logits at once, ahead of the row waves' loads (behind
    // them they would come in when the whole matrix has), and routes when the barrier is behind it.
    bool routing = false;
    float r_lg[4] = {0.f, 0.f, 0.f, 0.f}, r_bs[4] = {0.f, 0.f, 0.f, 0.f};
    if constexpr (!EARLY) routing = p.route.logits && blockIdx.x == 0;
    if (routing && wave == 0) {
#pragma unroll
      for (int k = 0; k < 4; k++) {
        const int e = k * 64 + lane;
        if (e < p.route.ne) { r_lg[k] = p.route.logits[e]; if (p.route.bias) r_bs[k] = p.route.bias[e]; }
      }
    } else if (p.xf) {
      if (routing) stage_q8_from_f32(p.xf, S, p.f16_scale, lxq, lxs, nullptr, nullptr, 1.0f, nullptr, (int)threadIdx.x - 64, 64 * (kStagers - 1));
      else stage_q8_from_f32(p.xf, S, p.f16_scale, lxq, lxs);
    } else {
      const int tid = routing ? (int)threadIdx.x - 64 : (int)threadIdx.x, nt = routing ? 64 * (kStagers - 1) : 64 * kStagers;
      for (int i = tid * 16; i < p.cols; i += nt * 16) *(int4*)(lxq + i) = *(const int4*)(p.xq + i);
      for (int i = tid; i < S; i += nt) lxs[i] = p.xs[i];
    }
    ilt_barrier_lds();
    if (p.ahead.a) cache_ahead(p.ahead, p.mat[0].y);
    if (p.rows_ahead.nm) rows_ahead(p.rows_ahead, p.mat[0].y);
    if constexpr (!EARLY) {
      if (routing && wave == 0) {
        __shared__ u32 r_idx[64];
        __shared__ float r_sc[64];
        route_token<4, true>(lane, p.route.ne, p.route.nu, p.route.scale, p.route.logits, p.route.bias, nullptr, p.route.sel, p.route.wout, r_idx,
                             r_sc, r_lg, r_bs);
      }
    }
    return;
  }
  if (wave < kStagers) {
    if (iq2) {
      lgrid[threadIdx.x] = ilt_iq2xxs_grid_dev[threadIdx.x];
      if (threadIdx.x < 128) lgrid[256 + threadIdx.x] = iq2_sign_mask(threadIdx.x);
    }
    int* sbs = iq2 ? nullptr : lbs;
    if (p.xf && p.norm_w) {
      float4 xall[4], nall[4];
      load_q8k_pass<kStagers>(p.xf, S, 0, xall);           // zeros where there is no block: they are squared
      load_q8k_pass_clamped<kStagers>(p.norm_w, S, 0, nall);
      double sq = 0.0;
      for (int pass = 1; pass * 4 * kStagers < S; pass++) {
        float4 t[4];
        load_q8k_pass<kStagers>(p.xf, S, pass, t);
        sq += (sq4(t[0]) + sq4(t[1])) + (sq4(t[2]) + sq4(t[3]));
      }
      sq += (sq4(xall[0]) + sq4(xall[1])) + (sq4(xall[2]) + sq4(xall[3]));
      const float nscale = norm_scale_stagers(sq, p.xf, p.cols, p.eps, p.norm_seq, s_meet);
      stage_q8k_from_f32<XP, kStagers>(p.xf, S, lxq, lxs, sbs, xall, p.norm_w, nall, nscale);
    } else if (p.xf && SX > 4 * kStagers) {
      // up to three passes (12288 activations): all their loads first, then the three passes' chains
      // of dependent instructions, which are independent of one another and interleave
      float4 x0[4], x1[4], x2[4];
      load_q8k_pass_clamped<kStagers>(p.xf, SX, 0, x0);
      load_q8k_pass_clamped<kStagers>(p.xf, SX, 1, x1);
      load_q8k_pass_clamped<kStagers>(p.xf, SX, 2, x2);
      const bool t0 = q8k_pass_impl<XP, kStagers, false>(p.xf, SX, 0, x0, lxq, lxs, sbs, nullptr, nullptr, 1.0f, nullptr);
      const bool t1 = q8k_pass_impl<XP, kStagers, false>(p.xf, SX, 1, x1, lxq, lxs, sbs, nullptr, nullptr, 1.0f, nullptr);
      const bool t2 = q8k_pass_impl<XP, kStagers, false>(p.xf, SX, 2, x2, lxq, lxs, sbs, nullptr, nullptr, 1.0f, nullptr);
      if (t0) q8k_pass_impl<XP, kStagers, true>(p.xf, SX, 0, x0, lxq, lxs, sbs, nullptr, nullptr, 1.0f, nullptr);
      if (t1) q8k_pass_impl<XP, kStagers, true>(p.xf, SX, 1, x1, lxq, lxs, sbs, nullptr, nullptr, 1.0f, nullptr);
      if (t2) q8k_pass_impl<XP, kStagers, true>(p.xf, SX, 2, x2, lxq, lxs, sbs, nullptr, nullptr, 1.0f, nullptr);
      for (int pass = 3; pass * 4 * kStagers < SX; pass++)
        q8k_pass<XP, kStagers>(p.xf, SX, pass, nullptr, lxq, lxs, sbs, nullptr, nullptr, 1.0f, nullptr);
    } else if (p.xf) {
      float4 xall[4];
      load_q8k_pass_clamped<kStagers>(p.xf, SX, 0, xall);
      stage_q8k_from_f32<XP, kStagers>(p.xf, SX, lxq, lxs, sbs, xall);
    } else {
      for (int i = threadIdx.x; i < SX * 16; i += 64 * kStagers)
        *(int4*)(lxq + (i >> 4) * XP + 16 * (i & 15)) = *(const int4*)(p.xq + 16 * i);
      for (int i = threadIdx.x; i < SX; i += 64 * kStagers) lxs[i] = p.xs[i];
      if (!iq2) for (int i = threadIdx.x; i < SX * 16; i += 64 * kStagers) lbs[i] = p.bsums[i];
    }
    ilt_barrier_lds();
    if (p.ahead.a) cache_ahead(p.ahead, p.mat[0].y);
    if (p.rows_ahead.nm) rows_ahead(p.rows_ahead, p.mat[0].y);
    return;
  }
  const int rw = wave - kStagers;
  const int wid = rw * gridDim.x + blockIdx.x;          // consecutive batches on different CUs
  // What a row wave must know before its first loads, read from the arguments in two goes -- the launch's numbers and
  // the matrices' first batches; then this wave's matrix, whole.  (Argument loads left where the values are used
  // come one after another, each behind a branch on the one before: a dozen round trips to the scalar cache.)
  const int a_nbatches = p.nbatches, a_nmat = p.nmat, a_glu = p.glu, a_batch = p.batch, a_region = p.region, a_cols = p.cols;
  const int b1 = p.mat[1].batch0, b2 = p.mat[2].batch0, b3 = p.mat[3].batch0;
  const uint64_t* const a_ptrs = p.ptrs;
  const uint32_t* const a_sel = p.sel;
  const u8* const u_w = p.mat[1].w;
  const u16* const u_wd = p.mat[1].wd;
  const long long u_row_bytes = p.mat[1].row_bytes, u_add = p.mat[1].add;
  const int u_fmt = p.mat[1].fmt;
  IltGemvMat m = p.mat[0];          // (the first matrix with them: the only one of most launches, no second go for those)
  asm volatile("" ::"s"(a_nbatches), "s"(a_nmat), "s"(a_glu), "s"(a_batch), "s"(a_region), "s"(a_cols), "s"(b1), "s"(b2), "s"(b3), "s"(a_ptrs),
               "s"(a_sel), "s"(u_w), "s"(u_wd), "s"(u_row_bytes), "s"(u_add), "s"(u_fmt), "s"(m.w), "s"(m.wd), "s"(m.y), "s"(m.bias),
               "s"(m.row_bytes), "s"(m.add), "s"(m.rows), "s"(m.fmt), "s"(m.batch0), "s"(m.nbat), "s"(m.rq), "s"(m.rr));
  float* tw = terms + (long)rw * a_batch * tpr * nglu;
  u8* region = (u8*)(terms + (long)kRowWaves * a_batch * tpr * nglu) + (long)rw * a_region;

  // 2. this wave's rows, all of them
  int mi = 0, nrows = 0, z = 0; long row0 = 0;
  const bool live = wid < a_nbatches;
  // (the matrices' first batches rise: the matrix of batch wid is the last one that starts at or before it)
  if (!a_ptrs && !a_glu) mi = (a_nmat > 1 && wid >= b1 ? 1 : 0) + (a_nmat > 2 && wid >= b2 ? 1 : 0) + (a_nmat > 3 && wid >= b3 ? 1 : 0);
  if (mi != 0) {
    m = p.mat[mi];
    asm volatile("" ::"s"(m.w), "s"(m.wd), "s"(m.y), "s"(m.bias), "s"(m.row_bytes), "s"(m.add), "s"(m.rows), "s"(m.fmt), "s"(m.batch0),
                 "s"(m.nbat), "s"(m.rq), "s"(m.rr));
  }
  int bl = wid;
  if (live) {
    if (a_ptrs) { z = wid / m.nbat; bl = wid - z * m.nbat; }
    else if (!a_glu) bl = wid - m.batch0;
    row0 = (long)bl * m.rq + min(bl, m.rr);
    nrows = m.rq + (bl < m.rr ? 1 : 0);
  }
  const int fmt = FSET != 0 ? FSET : m.fmt;
  const int ufmt = FSET != 0 ? FSET : u_fmt;
  const u8* slot = (live && a_ptrs) ? (const u8*)a_ptrs[a_sel ? a_sel[z] : z] : nullptr;
  const u8* wg = a_ptrs ? slot + m.add : m.w;
  const u8* wu = a_ptrs ? slot + u_add : u_w;
  u8* region_up = region + a_region / 2;
  // Q8_0: the scales' room behind the quants'
  const u8* scales = region + (long)a_batch * a_cols;
  const u8* scales_up = region_up + (long)a_batch * a_cols;
  // What the sum is added to (acc) and the bias are asked for ahead of the rows: they are there when the sums are,
  // instead of a trip to memory after them (asked for behind the rows they come in last and gain nothing).
  float* const ydst = m.y + (long)z * p.y_stride;
  const long rmine = row0 + min(lane, max(nrows - 1, 0));
  const float* const bsrc = m.bias ? m.bias : ydst;
  float yold = 0.0f, bval = 0.0f;
  float srow[8];
  if constexpr (EARLY == 1) { yold = ydst[rmine]; bval = bsrc[rmine]; }
  if constexpr (EARLY == 2) {
#pragma unroll
    for (int i = 0; i < 8; i++) srow[i] = p.sum.rows[(long)min(i, p.sum.k - 1) * p.sum.stride + rmine];
  }
  int nup = 0;              // load instructions of the up matrix's rows: the last ones issued
  if (live) {
    with_format<FSET>(fmt, [&](auto F) { stream_run<decltype(F)::value>(wg, row0, nrows, S, m.row_bytes, region, lane); });
    if (q8) stream_scales((const u8*)(m.wd + row0 * S), nrows * S * 2, (u8*)scales, lane);
    if (a_glu) {
      with_format<FSET>(ufmt, [&](auto F) { nup = stream_run<decltype(F)::value>(wu, row0, nrows, S, u_row_bytes, region_up, lane); });
      if (q8) nup += stream_scales((const u8*)(u_wd + row0 * S), nrows * S * 2, (u8*)scales_up, lane);
    }
  }
  // (no branch around the loads, which the compiler would wait out at the join: a launch that has neither runs the
  // kernel built without them; one that has only one of them reads y twice)
  // The barrier is for the activations only, so it comes before this wave waits for its rows (no
  // fence: the loads stay in flight): a wave whose rows land early starts on them while the
  // other waves' rows are still streaming in.
  ilt_barrier_lds();
  if (!live) return;
  // The gate's rows (or the only matrix's) have landed when at most the up matrix's loads are
  // still on their way: they return in the order they were issued.
  // (the count in the instruction is a constant: the largest of 12, 8, 4, 0 that is not above nup)
  if (nup >= 12) asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
  else if (nup >= 8) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
  else if (nup >= 4) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
  else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

  const int zx = p.x_stride ? z : 0;
  const Lds L = { q8 ? lxq : lxq + (long)zx * S * XP, lxs + zx * S, lbs + zx * S * 16, lgrid };
  with_format<FSET>(fmt, [&](auto F) { wave_rows_lds<decltype(F)::value>(region, scales, nrows, S, p.s_magic, L, tw, lane); });
  if (p.glu) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    with_format<FSET>(ufmt, [&](auto F) { wave_rows_lds<decltype(F)::value>(region_up, scales_up, nrows, S, p.s_magic, L, tw + (long)p.batch * tpr, lane); });
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  // A row's sum is one lane's chain of adds.  Of a gate/up pair the gate rows are summed by lanes 0.., the up rows by
  // lanes 32.. at the same time (a wave has at most 16 rows), and a lane of the first half fetches its partner's sum.
  const int tper = (fmt == ILT_Q4_K || fmt == ILT_Q2_K) ? 2 : 1, uper = (ufmt == ILT_Q4_K || ufmt == ILT_Q2_K) ? 2 : 1;      // floats a block
  const int rl = lane & 31;
  const bool up_lane = lane >= 32;
  float v = 0.0f;
  if (rl < nrows && (!up_lane || a_glu)) {        // (one call for both halves: two would run one after the other)
    const int per = up_lane ? uper : tper;
    v = chain_terms(up_lane ? tw + (long)a_batch * tpr + (long)rl * S * uper : tw + (long)rl * S * tper, S * per);
    if ((up_lane ? ufmt : fmt) == ILT_IQ2_XXS) v = 0.25f * v;
  }
  const float uv = __int_as_float(__builtin_amdgcn_ds_bpermute(4 * (lane ^ 32), __float_as_int(v)));
  if (lane < nrows) {
    const long r = row0 + lane;
    float* y = m.y + (long)z * p.y_stride;
    if (p.glu) {
      if (p.glu == 1) {
        y[r] = dense_glu(v, uv);
      } else {        // the experts' gated activation, as d4_swiglu_w computes it
        float gv = v, uu = uv;
        if (p.clamp > 1e-6f) { gv = fminf(gv, p.clamp); uu = fmaxf(-p.clamp, fminf(uu, p.clamp)); }
        float o = ilt_silu(gv) * uu;
        if (p.wts) o = o * p.wts[z];
        y[r] = o;
      }
    } else {
      if constexpr (EARLY == 2) {
        float a = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; i++) a = i < p.sum.k ? a + srow[i] : a;
        v = a + v;
      } else {
        if (m.bias) v = v + (EARLY ? bval : m.bias[r]);
        if (p.acc) v = (EARLY ? yold : y[r]) + v;
      }
      y[r] = v;
    }
  }
}

// rmsnorm! and the quantizer in one launch, a workgroup a row of DIM floats (the reference's
// rmsnorm_q8, cuda/dense.cu:144-160): H (unless null) gets the floats, XQ / XS the quants and
// scales -- Q8_0 blocks with XSUM (unless null) their sums, or with K set Q8_K blocks with
// XSUM their sums of 16.
template <bool K>
__global__ __launch_bounds__(kThreads) void rmsnorm_quant_kernel(const float* __restrict__ x, const float* __restrict__ w, float* h, i8* xq,
                                                                 float* xs, int* xsum, int dim, float eps, int f16_scale, int seq) {
  const long row = blockIdx.x;
  const float* xr = x + row * dim;
  float* hr = h ? h + row * dim : nullptr;
  const float nscale = norm_scale(norm_partial(xr, dim), xr, dim, eps, seq);
  if constexpr (K) {
    const int S = dim / 256;
    float4 xfirst[4], nfirst[4];
    load_q8k_pass(xr, S, 0, xfirst);
    load_q8k_pass(w, S, 0, nfirst);
    stage_q8k_from_f32<256>(xr, S, xq + row * dim, xs + row * S, xsum + row * (dim / 16), xfirst, w, nfirst, nscale, hr);
  } else {
    stage_q8_from_f32(xr, dim / 32, f16_scale, xq + row * dim, xs + row * (dim / 32), xsum ? xsum + row * (dim / 32) : nullptr, w, nscale, hr);
  }
}

size_t gemv_smem(int fset, const IltGemvParams& p) {
  const bool q8 = fset == ILT_Q8_0;
  const int S = q8 ? p.cols / 32 : p.cols / 256;
  size_t b = q8 ? (size_t)p.cols : (size_t)S * XP;
  b += (q8 || fset == ILT_IQ2_XXS) ? 0 : (size_t)p.cols / 16 * 4;
  b += 4 * (size_t)S + 8;
  if (fset == ILT_IQ2_XXS) b += 3072;
  return b + (size_t)kWaves * p.batch * S * (q8 ? 1 : 2) * 4 * (p.glu ? 2 : 1);
}

// Workgroups of variant FSET with SMEM bytes of LDS that one CU holds at a time (asked of the
// runtime once per variant and LDS size, kept per device 0..7).
int resident_per_cu(int fset, size_t smem) {
  static int cache[8][6][65];       // [device][variant][LDS KB], 0 = not asked yet
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 8) dev = 0;
  const int v = fset == 0 ? 0 : fset == ILT_Q8_0 ? 1 : fset == ILT_Q4_K ? 2 : fset == ILT_Q6_K ? 3 : fset == ILT_Q2_K ? 4 : 5;
  int& c = cache[dev][v][(smem + 1023) / 1024];
  if (c == 0) {
    int n = 0;
    hipError_t e = hipErrorInvalidValue;
    switch (v) {
      case 0: e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, gemv_kernel<0>, kThreads, smem); break;
      case 1: e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, gemv_kernel<ILT_Q8_0>, kThreads, smem); break;
      case 2: e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, gemv_kernel<ILT_Q4_K>, kThreads, smem); break;
      case 3: e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, gemv_kernel<ILT_Q6_K>, kThreads, smem); break;
      case 4: e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, gemv_kernel<ILT_Q2_K>, kThreads, smem); break;
      default: e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, gemv_kernel<ILT_IQ2_XXS>, kThreads, smem); break;
    }
    c = (e == hipSuccess && n > 0) ? n : 1;
  }
  return c;
}

}  // namespace

// The streamed variant's launch, when the product qualifies: Q4_K / Q6_K matrices on one
// activation vector, or IQ2_XXS / Q2_K experts (nz of them, each on its own vector right after
// the previous one's, or all on one); at most 16 rows a wave over the 3072 row waves of one
// workgroup per CU; everything within a CU's LDS.  Returns hipErrorNotSupported otherwise.
static unsigned long long g_streamed_launches = 0;
unsigned long long ilt_k_streamed_launches() { return g_streamed_launches; }

static hipError_t gemv_stream_launch(IltGemvParams& p, int fset, int nz, hipStream_t st, bool plan_only = false) {
  const char* force = getenv("ILT_GEMV_STREAM");          // "0": never (tests)
  if (force && atoi(force) == 0) return hipErrorNotSupported;
  const bool experts = p.ptrs != nullptr;
  const bool q8 = fset == ILT_Q8_0;
  if (experts ? !(fset == ILT_IQ2_XXS || fset == ILT_Q2_K) : !(fset == 0 || fset == ILT_Q4_K || fset == ILT_Q6_K || q8)) return hipErrorNotSupported;
  if (p.group_rows > 0 || (!experts && nz != 1) || (!experts && !q8 && p.glu > 1) || (experts && (p.norm_w || !(p.x_stride == 0 || p.x_stride == p.cols))))
    return hipErrorNotSupported;
  if (q8 && (p.norm_w || (p.cols / 32) % 2 != 0)) return hipErrorNotSupported;      // the scales go four bytes at a time
  const int S = q8 ? p.cols / 32 : p.cols / 256;
  const int nx = p.x_stride ? nz : 1;
  if (!q8 && (p.xf && p.norm_w ? S > 64 : (long)S * nx > 64 * 3)) return hipErrorNotSupported;
  const int nm = (p.glu || experts) ? 1 : p.nmat;
  long total_rows = 0, bytes = 0;
  for (int i = 0; i < nm; i++) { total_rows += p.mat[i].rows; bytes += (long)p.mat[i].rows * p.mat[i].row_bytes; }
  constexpr int kWavesAll = 256 * kRowWaves;
  // (from half a megabyte on: below that the looping variant's smaller workgroups are as fast)
  if (total_rows * nz > 16L * kWavesAll || bytes * nz * (p.glu ? 2 : 1) < (512L << 10)) return hipErrorNotSupported;
  int nb = 0, batch = 1;
  if (experts) {
    // the waves are shared out evenly over the experts; a batch is rows of one expert
    int nbz = kWavesAll / nz;
    if (nbz < 1) return hipErrorNotSupported;
    if (nbz > p.mat[0].rows) nbz = p.mat[0].rows;
    for (int i = 0; i < p.nmat; i++) {
      p.mat[i].batch0 = 0; p.mat[i].nbat = nbz; p.mat[i].rq = p.mat[0].rows / nbz; p.mat[i].rr = p.mat[0].rows % nbz;
    }
    batch = p.mat[0].rq + (p.mat[0].rr ? 1 : 0);
    nb = nbz * nz;
  } else {
    // every wave one batch: the waves are shared out over the matrices by rows, never more than there are
    int nb_total = (int)min((long)kWavesAll, total_rows);
    if (total_rows >= kWavesAll) {
      // A wave forms its terms 16 blocks (Q8_0: 32) a step, so a wave with 20 blocks takes two steps as one with 30
      // does: two row waves a SIMD with three rows each then take 4 steps a SIMD where three with two rows take 6.
      // Two waves a SIMD where that saves a quarter of the steps and the rows still fit.
      const int gpw = q8 ? 32 : 16;
      auto steps = [&](int waves) { const long r = (total_rows + waves - 1) / waves; return (waves / 1024) * ((r * S + gpw - 1) / gpw); };
      const long r2 = (total_rows + 2047) / 2048;
      const long one2 = q8 ? (r2 * (p.cols + 2 * S) + 15) / 16 * 16 : r2 * S * 224;
      const size_t smem2 = (size_t)S * nx * (XP + 16 * 4 + 4) + 3200 + (size_t)kRowWaves * r2 * S * 2 * 4 * (p.glu ? 2 : 1) + (size_t)kRowWaves * one2 * (p.glu ? 2 : 1);
      if (steps(2048) * 4 <= steps(kWavesAll) * 3 && r2 <= 16 && smem2 <= 150 * 1024) nb_total = 2048;
    }
    int given = 0;
    for (int i = 0; i < nm; i++) {
      int nbi = (int)((long)nb_total * p.mat[i].rows / total_rows);
      if (nbi < 1) nbi = 1;
      p.mat[i].nbat = nbi; given += nbi;
    }
    for (int i = 0; given < nb_total; i = (i + 1) % nm)          // the rounding's leftovers, where rows allow
      if (p.mat[i].nbat < p.mat[i].rows) { p.mat[i].nbat++; given++; }
    if (given > kWavesAll) return hipErrorNotSupported;
    for (int i = 0; i < p.nmat; i++) {
      if (i >= nm) { p.mat[i].batch0 = 0; p.mat[i].nbat = p.mat[0].nbat; p.mat[i].rq = p.mat[0].rq; p.mat[i].rr = p.mat[0].rr; continue; }
      p.mat[i].batch0 = nb;
      p.mat[i].rq = p.mat[i].rows / p.mat[i].nbat;
      p.mat[i].rr = p.mat[i].rows % p.mat[i].nbat;
      batch = max(batch, p.mat[i].rq + (p.mat[i].rr ? 1 : 0));
      nb += p.mat[i].nbat;
    }
  }
  if (batch > 16) return hipErrorNotSupported;
  p.nbatches = nb;
  p.batch = batch;
  p.nz = nz;
  const int nglu = p.glu ? 2 : 1;
  const int lb = fset == ILT_Q4_K ? 144 : fset == ILT_IQ2_XXS ? 80 : fset == ILT_Q2_K ? 96 : 224;      // Q6_K's spread blocks at worst
  // a wave's rows of one matrix (Q8_0: the quants, then the scales, rounded to 16 bytes)
  const long one = q8 ? ((long)batch * (p.cols + 2 * S) + 15) / 16 * 16 : (long)batch * S * lb;
  p.region = (int)(one * nglu);
  const size_t xbytes = q8 ? (size_t)p.cols + (size_t)S * 4
                           : (size_t)S * nx * XP + (fset == ILT_IQ2_XXS ? 3072 : (size_t)S * nx * 16 * 4) + (size_t)S * nx * 4;
  const size_t smem = xbytes + 16 + (size_t)kRowWaves * batch * S * (q8 ? 1 : 2) * 4 * nglu + (size_t)kRowWaves * p.region;
  if (smem > 156 * 1024) return hipErrorNotSupported;
  p.s_magic = (uint32_t)(0x100000000ULL / (uint64_t)S) + 1;
  if (plan_only) return nb >= 256 ? hipSuccess : hipErrorNotSupported;
  static bool attr_set[8] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 8) dev = 0;
  if (!attr_set[dev]) {            // more dynamic LDS than the default 64 KB: asked for once per device
    const void* kernels[11] = { (const void*)gemv_stream_kernel<0>, (const void*)gemv_stream_kernel<ILT_Q4_K>, (const void*)gemv_stream_kernel<ILT_Q6_K>,
                                (const void*)gemv_stream_kernel<ILT_IQ2_XXS>, (const void*)gemv_stream_kernel<ILT_Q2_K>,
                                (const void*)gemv_stream_kernel<ILT_Q8_0>, (const void*)gemv_stream_kernel<0, true>,
                                (const void*)gemv_stream_kernel<ILT_Q4_K, true>, (const void*)gemv_stream_kernel<ILT_Q6_K, true>,
                                (const void*)gemv_stream_kernel<ILT_Q8_0, true>, (const void*)gemv_stream_kernel<ILT_Q8_0, 2> };
    for (int i = 0; i < 11; i++)
      if (hipFuncSetAttribute(kernels[i], hipFuncAttributeMaxDynamicSharedMemorySize, 158 * 1024) != hipSuccess) {
        (void)hipGetLastError();
        return hipErrorNotSupported;
      }
    attr_set[dev] = true;
  }
  const dim3 grid(min(256, nb));                                      // wave w of workgroup g takes batch w * grid + g
  bool early = p.acc != 0;
  for (int i = 0; i < p.nmat; i++) early = early || p.mat[i].bias != nullptr;
  if (p.sum.rows) {                 // (its conditions were checked before the plan was made)
    hipLaunchKernelGGL((gemv_stream_kernel<ILT_Q8_0, 2>), grid, dim3(kStreamThreads), smem, st, p);
    g_streamed_launches++;
    return hipGetLastError();
  }
  early = early && !p.glu && !p.ptrs;
  if (early) {
    switch (fset) {
      case 0: hipLaunchKernelGGL((gemv_stream_kernel<0, true>), grid, dim3(kStreamThreads), smem, st, p); break;
      case ILT_Q4_K: hipLaunchKernelGGL((gemv_stream_kernel<ILT_Q4_K, true>), grid, dim3(kStreamThreads), smem, st, p); break;
      case ILT_Q6_K: hipLaunchKernelGGL((gemv_stream_kernel<ILT_Q6_K, true>), grid, dim3(kStreamThreads), smem, st, p); break;
      case ILT_Q8_0: hipLaunchKernelGGL((gemv_stream_kernel<ILT_Q8_0, true>), grid, dim3(kStreamThreads), smem, st, p); break;
      default: early = false; break;
    }
    if (early) { g_streamed_launches++; return hipGetLastError(); }
  }
  // a routing to carry along goes with the Q8_0 kernel only, for up to 256 experts (four a lane)
  if (p.route.logits) p.route.done = fset == ILT_Q8_0 && p.route.ne <= 256 && p.route.nu <= 64 && p.route.nu <= p.route.ne ? 1 : 0;
  if (p.route.logits && !p.route.done) p.route.logits = nullptr;
  switch (fset) {
    case 0: hipLaunchKernelGGL(gemv_stream_kernel<0>, grid, dim3(kStreamThreads), smem, st, p); break;
    case ILT_Q4_K: hipLaunchKernelGGL(gemv_stream_kernel<ILT_Q4_K>, grid, dim3(kStreamThreads), smem, st, p); break;
    case ILT_Q6_K: hipLaunchKernelGGL(gemv_stream_kernel<ILT_Q6_K>, grid, dim3(kStreamThreads), smem, st, p); break;
    case ILT_IQ2_XXS: hipLaunchKernelGGL(gemv_stream_kernel<ILT_IQ2_XXS>, grid, dim3(kStreamThreads), smem, st, p); break;
    case ILT_Q8_0: hipLaunchKernelGGL(gemv_stream_kernel<ILT_Q8_0>, grid, dim3(kStreamThreads), smem, st, p); break;
    default: hipLaunchKernelGGL(gemv_stream_kernel<ILT_Q2_K>, grid, dim3(kStreamThreads), smem, st, p); break;
  }
  g_streamed_launches++;
  return hipGetLastError();
}

hipError_t ilt_gemv_plan(IltGemvParams& p, int nz) {
  int fset = p.mat[0].fmt;
  for (int i = 1; i < p.nmat; i++) if (p.mat[i].fmt != fset) fset = 0;
  return gemv_stream_launch(p, fset, nz, nullptr, true);
}

void ilt_gemv_rows_of(const IltGemvParams& p, IltRowsAhead& out) {
  out.nm = 0;
  if (p.ptrs) return;
  for (int i = 0; i < p.nmat && i < 4; i++) {
    const IltGemvMat& m = p.mat[i];
    out.m[out.nm++] = {m.w, m.row_bytes, m.rq, m.rr, m.batch0, m.nbat};
  }
}

hipError_t ilt_gemv_launch(IltGemvParams& p, int nz, hipStream_t st) {
  if (p.ahead.a && (p.ahead.nrows <= 0 || (p.ahead.stride & 3) || !p.ahead.b || (((uintptr_t)p.ahead.a | (uintptr_t)p.ahead.b) & 15)))
    p.ahead.a = nullptr;                                   // (rows that 16-byte loads cannot take: no reading ahead)
  int fset = p.mat[0].fmt;
  for (int i = 1; i < p.nmat; i++) if (p.mat[i].fmt != fset) fset = 0;
  if (p.sum.rows) {               // a sum carried along: the streamed Q8_0 launch of one matrix takes it, nothing else does
    bool ok = fset == ILT_Q8_0 && p.nmat == 1 && !p.acc && !p.mat[0].bias && !p.glu && !p.ptrs && p.group_rows == 0 && nz == 1 &&
              p.sum.k >= 1 && p.sum.k <= 8 && p.sum.stride >= p.mat[0].rows;
    if (!ok) return hipErrorNotSupported;
  }
  if (p.counts) {                 // an expert's several rows: the looping variant of the experts' formats, floats in
    if (!p.bases || !p.ptrs || p.sel || !p.xf || p.glu || p.acc || p.norm_w || p.group_rows || p.nmat != 1 || p.mat[0].bias ||
        !(fset == ILT_IQ2_XXS || fset == ILT_Q2_K))
      return hipErrorNotSupported;
  } else {
    const hipError_t e = gemv_stream_launch(p, fset, nz, st);
    if (e != hipErrorNotSupported || p.sum.rows) return e;
  }
  const bool q8 = fset == ILT_Q8_0;
  const int S = q8 ? p.cols / 32 : p.cols / 256;
  const int nm = p.glu ? 1 : p.nmat;
  long total_rows = 0;
  for (int i = 0; i < nm; i++) total_rows += p.mat[i].rows;
  const int ngroups = p.group_rows > 0 ? (int)(total_rows / p.group_rows) : 1;
  const long rows_each = p.group_rows > 0 ? p.group_rows : total_rows;     // rows that share one x
  // The grid is a whole number of workgroups per CU (256 CUs), 1024 workgroups at most, split
  // over grid y and the row groups; every wave gets the same number of batches, and a
  // matrix's batches share its rows out evenly.  A batch is 16 rows at most (one lane each
  // in phase B) and no more than the terms' share of LDS (32 KB) allows.
  const size_t row_terms = (size_t)kWaves * S * (q8 ? 1 : 2) * 4 * (p.glu ? 2 : 1);
  int rb_max = 16;
  if ((size_t)rb_max * row_terms > 32768) rb_max = (int)(32768 / row_terms);
  if (rb_max < 1) rb_max = 1;
  const long all_rows = rows_each * nz * ngroups;
  p.batch = rb_max;
  const size_t smem = gemv_smem(fset, p);
  if (smem > 64 * 1024) return hipErrorInvalidValue;
  // no more workgroups than are resident at once (registers and LDS decide how many a CU
  // holds): a second round of workgroups would start only when the first has finished
  int m = resident_per_cu(fset, smem);
  if (m > 4) m = 4;
  while (m > 1 && all_rows < 3L * 1024 * m) m--;               // at least three rows a wave on average
  int waves_each = 1024 * m / (nz * ngroups) / kWaves * kWaves;  // waves per (grid y, group)
  if (waves_each < kWaves) waves_each = kWaves;
  if (waves_each > rows_each) waves_each = (int)((rows_each + kWaves - 1) / kWaves * kWaves);
  const int rounds = (int)((rows_each + (long)waves_each * rb_max - 1) / ((long)waves_each * rb_max));
  long nb_total = (long)waves_each * rounds;
  if (nb_total > rows_each) nb_total = rows_each;
  int nb = 0;
  for (int i = 0; i < p.nmat; i++) {
    p.mat[i].batch0 = nb;
    if (i >= nm) { p.mat[i].nbat = p.mat[0].nbat; p.mat[i].rq = p.mat[0].rq; p.mat[i].rr = p.mat[0].rr; continue; }
    const long r = p.group_rows > 0 ? p.group_rows : p.mat[i].rows;
    long nbi = (nb_total * r + rows_each - 1) / rows_each;       // this matrix's share of the batches
    if (nbi < (r + rb_max - 1) / rb_max) nbi = (r + rb_max - 1) / rb_max;
    if (nbi > r) nbi = r;
    p.mat[i].nbat = (int)nbi;
    p.mat[i].rq = (int)(r / nbi);
    p.mat[i].rr = (int)(r % nbi);
    nb += (int)nbi;
  }
  p.nbatches = nb;                                                          // per group, per grid y
  p.s_magic = (uint32_t)(0x100000000ULL / (uint64_t)S) + 1;   // floor(f/S) = umulhi(f, magic) while f*S < 2^32
  const int wgs = waves_each / kWaves;
  p.wgs_per_group = wgs;
  dim3 grid(wgs * ngroups, nz);
  if (p.counts) {
    if (fset == ILT_IQ2_XXS) hipLaunchKernelGGL(gemv_rows_kernel<ILT_IQ2_XXS>, grid, dim3(kThreads), smem, st, p);
    else hipLaunchKernelGGL(gemv_rows_kernel<ILT_Q2_K>, grid, dim3(kThreads), smem, st, p);
    return hipGetLastError();
  }
  switch (fset) {
    case 0: hipLaunchKernelGGL(gemv_kernel<0>, grid, dim3(kThreads), smem, st, p); break;
    case ILT_Q8_0: hipLaunchKernelGGL(gemv_kernel<ILT_Q8_0>, grid, dim3(kThreads), smem, st, p); break;
    case ILT_Q4_K: hipLaunchKernelGGL(gemv_kernel<ILT_Q4_K>, grid, dim3(kThreads), smem, st, p); break;
    case ILT_Q6_K: hipLaunchKernelGGL(gemv_kernel<ILT_Q6_K>, grid, dim3(kThreads), smem, st, p); break;
    case ILT_Q2_K: hipLaunchKernelGGL(gemv_kernel<ILT_Q2_K>, grid, dim3(kThreads), smem, st, p); break;
    case ILT_IQ2_XXS: hipLaunchKernelGGL(gemv_kernel<ILT_IQ2_XXS>, grid, dim3(kThreads), smem, st, p); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

hipError_t ilt_k_rmsnorm_quant(int k, const float* x, const float* w, float* h, int8_t* xq, float* xs, int* xsum, int dim,
                               float eps, int f16_scale, int seq, int nrows, hipStream_t st) {
  if (nrows <= 0) return hipSuccess;
  if (k) hipLaunchKernelGGL(rmsnorm_quant_kernel<true>, dim3(nrows), dim3(kThreads), 0, st, x, w, h, xq, xs, xsum, dim, eps, f16_scale, seq);
  else hipLaunchKernelGGL(rmsnorm_quant_kernel<false>, dim3(nrows), dim3(kThreads), 0, st, x, w, h, xq, xs, xsum, dim, eps, f16_scale, seq);
  return hipGetLastError();
}
