// Prefill products on the bf16 matrix cores of gfx950: Y[t][r] = W[r].x_t for many tokens,
// W dequantized from GGUF Q4_K / Q6_K / Q2_K / IQ2_XXS blocks to bf16 on the way into LDS,
// the activations already rounded to bf16 (ilt_k_cvt_bf16), fp32 accumulation in
// v_mfma_f32_32x32x16_bf16.  This is the fast path: its results differ from the CPU path's
// by the bf16 roundings (tolerance 2e-2 relative, against bit-exact for the int8 path in
// kernels_gemm.hip).  Each weight is dequantized exactly as the reference's
// *-row-floats! / kmat-row! do (kquant.lisp:466-497, iquant.lisp:161-230) before rounding.
//
// A workgroup of 2*TM threads computes TM rows x TN tokens (256x256, 128x256 or 128x128,
// the larger the tile the less is fetched and dequantized per product; the smaller ones for
// few tokens and for the expert groups) in steps of 32 columns:
//   - the activations' 32-column slab goes from global memory straight into LDS
//     (global_load_lds_dwordx4), two steps ahead, into a ring of three slabs;
//   - thread (row, e) dequantizes columns 16e..16e+15 of its row in every step.  It holds
//     the raw bytes of half a super-block (four steps) of its row in registers, in two sets
//     loaded four steps before first use; it dequantizes the next step's weights and writes
//     them as bf16 into one of two weight slabs while the current step's MFMAs run;
//   - one barrier per step; wave w multiplies rows 64*(w/2).. by tokens (TN/2)*(w%2)..
//     as patches of 32x32.  The MFMA's M side is the tokens and its N side the rows, so a
//     lane's 16 results of a patch are one row for 16 tokens and a store instruction writes
//     32 consecutive rows of a token.
// Both kinds of slab hold 64 bytes per row as four 16-byte pieces, unpadded and swizzled
// (slab_off): the direct loads write 1 KB per wave instruction contiguously, so the swizzle
// is applied by choosing which global piece each lane fetches.
// Tiles are numbered so that the workgroups resident on one XCD (every eighth workgroup id)
// form a block of 8 row tiles x several token tiles and share W and x slabs through that
// XCD's L2.  The grouped expert product (d4_mm_id_*) walks the token tiles of every
// expert's rows in turn; for the experts' own formats, IQ2_XXS and Q2_K, it has a kernel of
// its own that dequantizes into the MFMA operands without a detour of the weights through LDS
// as bf16 (gemm_bf16_regb_kernel).
// The same pipeline also carries the exact product (gemm_i8p_kernel, further down): scale * quant
// as int8 planes on v_mfma_i32_32x32x32_i8, the bits of the CPU path's MATMUL!.
#include "ilt_device.h"
#include "ilt_iq2xxs_tables.h"
#include "ilt_kernels.h"
#include <stdlib.h>
#include <mutex>
#include <type_traits>

namespace {

typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v2f __attribute__((ext_vector_type(2)));

constexpr int KS = 32;                 // columns per step
constexpr int GR = 8;                  // row tiles per block of tiles sharing an L2

__device__ const u64 bf_grid_dev[256] = { ILT_IQ2XXS_GRID_VALUES };

__device__ __forceinline__ u32 pack_bf16(float a, float b) {
  const v2f v = {a, b};
  const v2bf r = __builtin_convertvector(v, v2bf);
  u32 u; __builtin_memcpy(&u, &r, 4); return u;
}

// The raw bytes a thread needs for four steps (half a super-block, 128 columns) of its row:
// thread (row, e) dequantizes columns 16e..16e+15 of every 32-column step.  Loaded once per
// four steps, so that a load instruction's 32 rows fetch 32 bytes each rather than 16 or 2.
template <int FMT> struct WRaw;
template <> struct WRaw<ILT_Q4_K> { int4 hdr, q[2]; static constexpr int LOADS = 3; };
template <> struct WRaw<ILT_Q6_K> { int4 ql[2], qh; int2 sc; u32 d; static constexpr int LOADS = 5; };
template <> struct WRaw<ILT_Q2_K> { int4 q; int2 sc; u32 dd; static constexpr int LOADS = 3; };
template <> struct WRaw<ILT_IQ2_XXS> { int4 q[2]; u32 d; static constexpr int LOADS = 3; };

// hb: the half super-block (hb>>1 the super-block, c = hb&1 its half)
template <int FMT> __device__ __forceinline__ void load_w(WRaw<FMT>& r, __amdgpu_buffer_rsrc_t rw, u32 rowoff, int hb, int e);

template <> __device__ __forceinline__ void load_w<ILT_Q4_K>(WRaw<ILT_Q4_K>& r, __amdgpu_buffer_rsrc_t rw, u32 rowoff, int hb, int e) {
  const u32 b = rowoff + (u32)(hb >> 1) * 144;
  r.hdr = ilt_bld16(rw, b);
  r.q[0] = ilt_bld16(rw, b + 16 + 64 * (hb & 1) + 16 * e);
  r.q[1] = ilt_bld16(rw, b + 48 + 64 * (hb & 1) + 16 * e);
}
template <> __device__ __forceinline__ void load_w<ILT_Q6_K>(WRaw<ILT_Q6_K>& r, __amdgpu_buffer_rsrc_t rw, u32 rowoff, int hb, int e) {
  const u32 b = rowoff + (u32)(hb >> 1) * ILT_Q6K_STRIDE;
  const int c = hb & 1;
  r.ql[0] = ilt_bld16(rw, b + 64 * c + 16 * e);
  r.ql[1] = ilt_bld16(rw, b + 64 * c + 32 + 16 * e);
  r.qh = ilt_bld16(rw, b + 128 + 32 * c + 16 * e);
  r.sc = ilt_bld8(rw, b + 192 + 8 * c);
  r.d = ilt_bld2(rw, b + 208);
}
template <> __device__ __forceinline__ void load_w<ILT_Q2_K>(WRaw<ILT_Q2_K>& r, __amdgpu_buffer_rsrc_t rw, u32 rowoff, int hb, int e) {
  const u32 b = rowoff + (u32)(hb >> 1) * 84;
  r.q = ilt_bld16(rw, b + 16 + 32 * (hb & 1) + 16 * e);
  r.sc = ilt_bld8(rw, b + 8 * (hb & 1));
  r.dd = ilt_bld4(rw, b + 80);
}
template <> __device__ __forceinline__ void load_w<ILT_IQ2_XXS>(WRaw<ILT_IQ2_XXS>& r, __amdgpu_buffer_rsrc_t rw, u32 rowoff, int hb, int e) {
  const u32 b = rowoff + (u32)(hb >> 1) * 66;
  r.q[0] = ilt_bld16(rw, b + 2 + 32 * (hb & 1));
  r.q[1] = ilt_bld16(rw, b + 18 + 32 * (hb & 1));
  r.d = ilt_bld2(rw, b);
}

__device__ __forceinline__ u32 word_of(const int4& v, int i) { return (u32)(i == 0 ? v.x : i == 1 ? v.y : i == 2 ? v.z : v.w); }

// 16 weights as floats, in column order, each with the CPU dequantizers' value.  Where the CPU
// multiplies then subtracts (d1*q - m1, dl*q - ml) the product is exact in fp32 (a 17-bit
// scale times a 2- or 4-bit integer), and Q6_K's s*(q-32) is one rounding of an exact value;
// so a fused multiply-add gives the same bits in half the instructions.
// j: the step within the half super-block (a constant after unrolling); c: which half.
template <int FMT> __device__ __forceinline__ void dequant16(const WRaw<FMT>& r, int j, int c, int e, float* o);

template <> __device__ __forceinline__ void dequant16<ILT_Q4_K>(const WRaw<ILT_Q4_K>& r, int j, int c, int e, float* o) {
  const int sh = 8 * j, hl = j & 1;              // group g = 4c + j of the super-block
  const u32 x0 = ((u32)r.hdr.y >> sh) & 0xFF, x1 = ((u32)r.hdr.z >> sh) & 0xFF, x2 = ((u32)r.hdr.w >> sh) & 0xFF;
  const u32 sc = c == 0 ? (x0 & 63) : ((x2 & 0xF) | ((x0 >> 6) << 4));
  const u32 mn = c == 0 ? (x1 & 63) : ((x2 >> 4) | ((x1 >> 6) << 4));
  const float d1 = ilt_h2f((u16)(r.hdr.x & 0xFFFF)) * (float)sc, m1 = ilt_h2f((u16)((u32)r.hdr.x >> 16)) * (float)mn;
  const int4& q = r.q[j >> 1];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const u32 v = (word_of(q, i) >> (4 * hl)) & 0x0F0F0F0F;
#pragma unroll
    for (int k = 0; k < 4; k++) o[4 * i + k] = __builtin_fmaf(d1, (float)((v >> (8 * k)) & 0xFF), -m1);   // d1*q is exact in fp32
  }
}

template <> __device__ __forceinline__ void dequant16<ILT_Q6_K>(const WRaw<ILT_Q6_K>& r, int j, int c, int e, float* o) {
  const int h = j >> 1;                          // 32-weight part j of the half: ql[j&1]'s nibble h, qh's bit pair j
  const u32 scw = (u32)(j < 2 ? r.sc.x : r.sc.y) >> (16 * (j & 1) + 8 * e);
  const float s = ilt_h2f((u16)r.d) * (float)(i8)(scw & 0xFF), s32 = -32.0f * s;
  const int4& ql = r.ql[j & 1];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const u32 v = ((word_of(ql, i) >> (4 * h)) & 0x0F0F0F0F) | (((word_of(r.qh, i) >> (2 * j)) & 0x03030303) << 4);
#pragma unroll
    for (int k = 0; k < 4; k++) o[4 * i + k] = __builtin_fmaf(s, (float)((v >> (8 * k)) & 0xFF), s32);   // = RN(s*(q-32)): one rounding either way
  }
}

template <> __device__ __forceinline__ void dequant16<ILT_Q2_K>(const WRaw<ILT_Q2_K>& r, int j, int c, int e, float* o) {
  const u32 scw = ((u32)(j < 2 ? r.sc.x : r.sc.y) >> (16 * (j & 1) + 8 * e)) & 0xFF;
  const float dl = ilt_h2f((u16)(r.dd & 0xFFFF)) * (float)(scw & 15), ml = ilt_h2f((u16)(r.dd >> 16)) * (float)(scw >> 4);
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const u32 v = (word_of(r.q, i) >> (2 * j)) & 0x03030303;
#pragma unroll
    for (int k = 0; k < 4; k++) o[4 * i + k] = __builtin_fmaf(dl, (float)((v >> (8 * k)) & 0xFF), -ml);   // dl*q is exact in fp32
  }
}

// IQ2_XXS has three magnitudes (its codebook's bytes are 0x08, 0x19 and 0x2b), so a unit of 16
// weights takes three products db*8, db*25, db*43 -- each the CPU's (db * mag), rounded to bf16
// -- and every weight is one of those with its sign: a byte permute picks the pair of bf16 for
// two weights, an xor sets their signs.  The permute selectors of a codebook entry and the sign
// masks of a 7-bit sign index (+ parity) come ready-made from two tables in LDS.
struct Iq2Tables {
  u32 sel[256][4];       // entry g: selector for weights (2k, 2k+1) of codebook entry g, k = 0..3
  u32 sgn[128][4];       // entry s: 0x8000 where weight 2k is negative | 0x80000000 where weight 2k+1 is
};
__device__ __forceinline__ void iq2_tables_fill(Iq2Tables& T, int t) {    // threads t = 0..255 of a workgroup; a barrier follows
  const u64 g = bf_grid_dev[t & 255];
#pragma unroll
  for (int k = 0; k < 4; k++) {
    const u32 t0 = ((u32)(g >> (16 * k + 3))) & 6, t1 = ((u32)(g >> (16 * k + 11))) & 6;    // 2 * (byte >> 4): 0, 2, 4
    if (t < 256) T.sel[t][k] = t0 | ((t0 + 1) << 8) | (t1 << 16) | ((t1 + 1) << 24);
  }
  if (t < 128) {
    const u32 sb = (u32)t | ((__popc(t) & 1) << 7);
#pragma unroll
    for (int k = 0; k < 4; k++) T.sgn[t][k] = (((sb >> (2 * k)) & 1) << 15) | (((sb >> (2 * k + 1)) & 1) << 31);
  }
}

// 16 weights as 8 words of two bf16, in column order.
template <int FMT>
__device__ __forceinline__ void dequant16_pk(const WRaw<FMT>& r, int j, int c, int e, const Iq2Tables*, u32* pk) {
  float o[16];
  dequant16<FMT>(r, j, c, e, o);
#pragma unroll
  for (int i = 0; i < 8; i++) pk[i] = pack_bf16(o[2 * i], o[2 * i + 1]);
}
template <>
__device__ __forceinline__ void dequant16_pk<ILT_IQ2_XXS>(const WRaw<ILT_IQ2_XXS>& r, int j, int c, int e, const Iq2Tables* T, u32* pk) {
  const int4& q = r.q[j >> 1];                   // the half's 32-weight group j: 8 bytes
  const u32 g = word_of(q, 2 * (j & 1)) >> (16 * e), aux = word_of(q, 2 * (j & 1) + 1);
  const float db = (ilt_h2f((u16)r.d) * (0.5f + (float)(aux >> 28))) * 0.25f;
  const u32 t01 = pack_bf16(db * 8.0f, db * 25.0f), t2 = pack_bf16(db * 43.0f, 0.0f);
#pragma unroll
  for (int l = 0; l < 2; l++) {
    const int4 sel = ilt_lds_ld16(T->sel[(g >> (8 * l)) & 0xFF]);
    const int4 sg = ilt_lds_ld16(T->sgn[(aux >> (7 * (2 * e + l))) & 127]);
    pk[4 * l + 0] = __builtin_amdgcn_perm(t2, t01, (u32)sel.x) ^ (u32)sg.x;
    pk[4 * l + 1] = __builtin_amdgcn_perm(t2, t01, (u32)sel.y) ^ (u32)sg.y;
    pk[4 * l + 2] = __builtin_amdgcn_perm(t2, t01, (u32)sel.z) ^ (u32)sg.z;
    pk[4 * l + 3] = __builtin_amdgcn_perm(t2, t01, (u32)sel.w) ^ (u32)sg.w;
  }
}

struct BfParams {
  const u8* w;                               // dense
  const u64* ptrs; long long add;            // grouped: expert z's matrix at ptrs[z] + add
  const u32* counts; const u32* bases; int ne;
  int rows, cols; long long row_bytes;
  const u16* x;                              // bf16 activations, cols per token (the gathered rows when grouped)
  const u32* rmap;                           // grouped: row i of the groups is x's row rmap[i] (null: row i)
  float* y; const float* bias; int acc; int ntok;
  long long ldy;                             // floats from a token's results to the next token's in y (rows, unless p covers a part of the rows)
  // several matrices of one format on the same tokens in one launch (gemm_i8p_kernel, dense): matrix m's row tiles follow
  // matrix m-1's; rows = the tiles of all of them together times 128 until the workgroup has found its matrix
  int nmulti; const u8* mw[3]; int mrows[3]; float* my[3]; const float* mbias[3];
  // the grouped gate and up products with the gated activation (gemm_bf16_regb_kernel<FMT, true>): rows = the width of
  // each; up's matrix at ptrs[z] + add + up_delta; mid[i][r] = bf16((silu(gate) * up) * wrow[i]), clamped as d4_swiglu_w does
  unsigned up_delta; const float* wrow; float clamp; u16* mid;
  // the exact product (gemm_i8p_kernel): x = the tokens' Q8_K quants (a byte a column), with their block scales and sums of 16
  const float* xd; const int* bsums;
  // Q8_0 (gemm_i8q_kernel): w = the quants (a byte a weight, rows of cols bytes), wdq their f16 scales, xd the tokens' scales (one per 32)
  const u16* wdq;
  // the planes made beforehand (gemm_i8pp_kernel): w = the hi plane, wlo the lo plane (a byte a weight, rows of cols bytes), wdf = d per row and super-block
  const u8* wlo; const float* wdf;
  // the columns split over workgroups (gemm_bf16_kernel, dense): workgroups from split_from on take the tiles from
  // split_from on, ksplit of them a tile, each a run of the super-blocks, and leave their sums in part (a tile of TM x TN
  // floats each, token after token); bf16_split_sum_kernel adds a tile's parts in order and writes y.  ksplit 0: none
  int ksplit, split_from; float* part;
};

template <int TM, int TN, int NXS, int NWS> struct Smem {
  __align__(16) u8 xs[NXS][TN * KS * 2];
  __align__(16) u8 ws[NWS][TM * KS * 2];
  Iq2Tables iq2;
  u32 scan[256];
  int tile_z, tile_t0, tile_n;
};

// Piece p (16 bytes) of row r of a slab.  Rows are 64 bytes, so 8 consecutive rows span 128
// bytes-wide LDS twice over and 16 rows a 256-byte-wide one four times; the piece index is
// xor-ed with bits of the row such that the same piece of 8 (or 16) consecutive rows falls
// in 8 (or 16) different 16-byte columns.
__device__ __forceinline__ u32 slab_swz(int r) { return (((r >> 1) ^ (r >> 3)) & 1) | (((r >> 2) & 1) << 1); }
__device__ __forceinline__ u32 slab_off(int r, int p) { return (u32)(4 * r + (p ^ slab_swz(r))) * 16; }

// ---- a wave's results to y ----
// Patch (a, b), register r of a lane: token wt0 + 32a + 8*(r/4) + 4*lh + r%4, row wr0 + 32b + l32
// of the tile, so a store instruction writes 32 consecutive rows of two tokens.  With one
// workgroup on a CU nothing else runs while it stores, so the loop is kept to an address add
// and a store per value and has no branches: the stores go through a buffer descriptor that
// ends with the tile's last token, which drops what lies past it, and a lane whose row the
// matrix does not have starts 2 GiB out.  (ldy * 1024 < 2^31, checked by the host.)
template <int NA, int NB, bool BIAS, bool ACC>
__device__ __forceinline__ void store_patches(const v16f (&acc)[NA][NB], const BfParams& p, __amdgpu_buffer_rsrc_t ry, int r0,
                                              int wt0, int wr0, int l32, int lh) {
  const u32 rows4 = (u32)p.ldy * 4;
#pragma unroll
  for (int b = 0; b < NB; b++) {
    const int row = r0 + wr0 + 32 * b + l32;
    const bool ok = row < p.rows;
    const u32 base = ok ? (u32)((wt0 + 4 * lh) * (int)p.ldy + row) * 4 : 0x80000000u;
    float bv = 0.0f;
    if (BIAS) bv = ok ? p.bias[row] : 0.0f;
#pragma unroll
    for (int a = 0; a < NA; a++) {
      float old[16];
      if (ACC) {
#pragma unroll
        for (int r = 0; r < 16; r++)
          old[r] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(ry, base + (u32)(32 * a + 8 * (r >> 2) + (r & 3)) * rows4, 0, 0));
      }
#pragma unroll
      for (int r = 0; r < 16; r++) {
        float v = acc[a][b][r];
        if (BIAS) v = v + bv;
        if (ACC) v = old[r] + v;
        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(u32, v), ry, base + (u32)(32 * a + 8 * (r >> 2) + (r & 3)) * rows4, 0, 0);
      }
    }
  }
}

template <int NA, int NB>
__device__ __forceinline__ void store_tile(const v16f (&acc)[NA][NB], const BfParams& p, long tok0, int ntok, int r0,
                                           int wt0, int wr0, int l32, int lh) {
  // (ntok may come out of LDS: the same in every lane, said so to the compiler)
  const u32 ybytes = ((u32)(__builtin_amdgcn_readfirstlane(ntok) - 1) * (u32)p.ldy + (u32)p.rows) * 4;
  const __amdgpu_buffer_rsrc_t ry = ilt_rsrc(ilt_uniform_ptr(p.y + tok0 * p.ldy), ybytes);
  if (p.bias) {
    if (p.acc) store_patches<NA, NB, true, true>(acc, p, ry, r0, wt0, wr0, l32, lh);
    else store_patches<NA, NB, true, false>(acc, p, ry, r0, wt0, wr0, l32, lh);
  } else {
    if (p.acc) store_patches<NA, NB, false, true>(acc, p, ry, r0, wt0, wr0, l32, lh);
    else store_patches<NA, NB, false, false>(acc, p, ry, r0, wt0, wr0, l32, lh);
  }
}

// Which tile a workgroup takes: row tile rt, tokens tok0 .. tok0+ntok-1 (of expert z's group,
// with w its matrix, when grouped).  Tiles are numbered so that the eight XCDs' workgroups (the
// hardware deals them round-robin) each walk a contiguous run, GR row tiles of one token tile
// after another.  False: none (the grid is rounded up).  S: scan[256], tile_z, tile_t0, tile_n.
// (dense) tile number s of the NT x NR: its row tile and its first token
__device__ __forceinline__ void tile_place(int s, int NT, int NR, int& rt, int& tt) {
  const int rg = s / (GR * NT), rem = s - rg * GR * NT, nr = min(GR, NR - rg * GR);
  tt = rem / nr;
  rt = rg * GR + (rem - tt * nr);
}

// LIMIT >= 0: only the tiles before it are dealt out (a multiple of 8; the workgroups from it on take parts of the rest)
template <int TM, int TN, typename SM>
__device__ __forceinline__ bool pick_tile(const BfParams& p, SM& S, long& tok0, int& ntok, int& rt, const u8*& w, int limit = -1) {
  const int t = threadIdx.x;
  const int NR = (p.rows + TM - 1) / TM;
  int NT;
  if (p.ptrs) {
    if (t < 256) S.scan[t] = t < p.ne ? (p.counts[t] + TN - 1) / TN : 0;
    __syncthreads();
    for (int off = 1; off < 256; off <<= 1) {
      const u32 v = (t < 256 && t >= off) ? S.scan[t - off] : 0;
      __syncthreads();
      if (t < 256) S.scan[t] += v;
      __syncthreads();
    }
    NT = (int)S.scan[255];
  } else {
    NT = (p.ntok + TN - 1) / TN;
  }
  const int total = limit >= 0 ? limit : NT * NR, per = (total + 7) / 8;
  const int L = blockIdx.x, j = L >> 3;
  const int s = (L & 7) * per + j;
  if (j >= per || s >= total) return false;
  int tt;
  tile_place(s, NT, NR, rt, tt);
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
  return true;
}

// TM rows x TN tokens per workgroup; wave w: rows 32*NB*(w/2).., tokens (TN/2)*(w%2)..: NA x NB
// patches of 32x32.  NB = 2: 2*TM threads, two per row (a thread dequantizes 16 weights a step);
// NB = 4: TM threads, one per row (32 weights a step).
template <int TM, int NB> constexpr int bf16_threads() { return 64 * 2 * (TM / (32 * NB)); }

template <int FMT, int TM, int TN, int NB>
__global__ __launch_bounds__((bf16_threads<TM, NB>()), (TM * TN == 65536 ? 1 : TM * TN == 32768 ? 2 : 3)) void gemm_bf16_kernel(BfParams p) {
  __shared__ Smem<TM, TN, 3, 2> S;
  constexpr int THREADS = bf16_threads<TM, NB>();
  constexpr int NE = 2 * TM / THREADS;   // 16-column units of a row a thread dequantizes per step: 1 or 2
  constexpr int NA = TN / 64;            // 32-token patches per wave
  constexpr int NI = 4 * TN / THREADS;   // direct-load instructions per wave and step
  constexpr int WL = WRaw<FMT>::LOADS * NE;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;

  long tok0; int ntok, rt; const u8* w = p.w;
  int sb0 = 0, sb1 = p.cols / 256;                         // the super-blocks this workgroup multiplies
  const bool part = p.ksplit > 1 && (int)blockIdx.x >= p.split_from;
  if (part) {
    const int q = (int)blockIdx.x - p.split_from, ti = q / p.ksplit, ky = q - ti * p.ksplit;
    const int NT = (p.ntok + TN - 1) / TN, NR = (p.rows + TM - 1) / TM;
    if (p.split_from + ti >= NT * NR) return;
    int tt;
    tile_place(p.split_from + ti, NT, NR, rt, tt);
    tok0 = (long)tt * TN;
    ntok = min(TN, p.ntok - (int)tok0);
    sb0 = (int)((long)ky * sb1 / p.ksplit);
    sb1 = (int)((long)(ky + 1) * sb1 / p.ksplit);
  } else if (!pick_tile<TM, TN>(p, S, tok0, ntok, rt, w, p.ksplit > 1 ? p.split_from : -1)) return;
  const int r0 = rt * TM;
  if (FMT == ILT_IQ2_XXS) {
    if (t < 256) iq2_tables_fill(S.iq2, t);
    __syncthreads();
  }

  // ---- this thread's shares of a step ----
  const int wrow = NE == 1 ? t >> 1 : t, e0 = NE == 1 ? t & 1 : 0;   // 16 weights (or all 32) of row wrow
  const __amdgpu_buffer_rsrc_t rw = ilt_rsrc(ilt_uniform_ptr(w), (u32)min((long long)p.rows * p.row_bytes, 0xFFFFFFF0LL));
  const u32 wrowoff = (u32)((long long)min(r0 + wrow, p.rows - 1) * p.row_bytes);
  const u32 wdst = slab_off(wrow, 2 * e0);                 // unit e's two pieces: 2e and 2e+1, at (wdst ^ 32e) and that ^ 16
  const u8* xbase = (const u8*)ilt_uniform_ptr(p.rmap ? p.x : p.x + tok0 * (long)p.cols);
  u32 xoff[NI];                                            // the x pieces it sends to LDS
#pragma unroll
  for (int i = 0; i < NI; i++) {
    const int P = (wave * NI + i) * 64 + lane, tok = P >> 2, kp = (P & 3) ^ (int)slab_swz(tok);
    const int tk = min(tok, ntok - 1);
    xoff[i] = (p.rmap ? p.rmap[tok0 + tk] : (u32)tk) * (u32)p.cols * 2 + 16 * kp;
  }

  v16f acc[NA][NB];
#pragma unroll
  for (int a = 0; a < NA; a++)
#pragma unroll
    for (int b = 0; b < NB; b++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[a][b][r] = 0.0f;

  const int wt0 = (TN / 2) * (wave & 1), wr0 = 32 * NB * (wave >> 1);   // this wave's tokens and rows in the tile
  const int l32 = lane & 31, lh = lane >> 5;
  u32 aoff[NA], boff[NB];                                  // fragment offsets for the step's first 16 columns; the second 16 at ^ 32
#pragma unroll
  for (int a = 0; a < NA; a++) aoff[a] = slab_off(wt0 + 32 * a + l32, lh);
#pragma unroll
  for (int b = 0; b < NB; b++) boff[b] = slab_off(wr0 + 32 * b + l32, lh);

  const int nk = p.cols / KS, nh = nk / 4;                 // steps, half super-blocks
  auto issue_x = [&](int stage, int ks) {
#pragma unroll
    for (int i = 0; i < NI; i++) ilt_g2lds16(xbase + ks * (KS * 2) + xoff[i], S.xs[stage] + (wave * NI + i) * 1024);
  };
  auto dequant_unit = [&](const WRaw<FMT>& raw, int u, int j, int c, u8* ws) {   // 16 weights of step j of a half into a slab
    u32 pk[8];
    dequant16_pk<FMT>(raw, j, c, e0 + u, &S.iq2, pk);
    ilt_lds_st16_untracked(ws + (wdst ^ (32 * u)), pk[0], pk[1], pk[2], pk[3]);
    ilt_lds_st16_untracked(ws + (wdst ^ (32 * u) ^ 16), pk[4], pk[5], pk[6], pk[7]);
  };
  auto dequant_to = [&](const WRaw<FMT>* raw, int j, int c, int slab) {   // step j of a half's weights into a slab
#pragma unroll
    for (int u = 0; u < NE; u++) dequant_unit(raw[u], u, j, c, S.ws[slab]);
  };
  auto load_raw = [&](WRaw<FMT>* raw, int hb) {
#pragma unroll
    for (int u = 0; u < NE; u++) load_w<FMT>(raw[u], rw, wrowoff, hb, e0 + u);
  };

  {
  // Two register sets of raw weights, each a half super-block (4 steps): rawa holds half 0
  // of a super-block, rawb half 1.  Step ks multiplies slab ks while it dequantizes step
  // ks+1's weights into the other weight slab; a set is reloaded, with the half two ahead,
  // right after its last step is dequantized, four steps before it is needed again.
  WRaw<FMT> rawa[NE], rawb[NE];
  load_raw(rawa, 2 * sb0);
  issue_x(0, 8 * sb0);
  load_raw(rawb, 2 * sb0 + 1);
  issue_x(1, 8 * sb0 + 1);
  int st0 = 0, st1 = 1, st2 = 2;                           // ring: the step's slab, the next step's, the one after
  dequant_to(rawa, 0, 0, 0);

  // J: the step's place in its super-block (0..7), a constant in the unrolled body
  auto step = [&](int ks, auto Jc) {
    constexpr int J = decltype(Jc)::value;
    // All loads but the previous step's have landed: this step's x slab has (sent two steps
    // ago).  The barrier also publishes the weight slab written during the previous step,
    // and says that x slab ks-1 and the other weight slab are read no more.
    constexpr int prev = NI + ((J == 0 || J == 4) ? WL : 0);   // steps 3 and 7 of a super-block also reload a set
    asm volatile("s_waitcnt vmcnt(%0)" :: "n"(prev) : "memory");
    ilt_barrier_lds();                                     // no fence: later steps' loads stay in flight
    if (J == 3) load_raw(rawa, min((ks >> 2) + 2, nh - 1));   // rawa's last use was step 2's dequantization
    if (J == 7) load_raw(rawb, min((ks >> 2) + 2, nh - 1));
    issue_x(st2, min(ks + 2, nk - 1));
    __builtin_amdgcn_sched_barrier(0);
    const u8* xs = S.xs[st0];
    const u8* ws = S.ws[J & 1];
    // step ks+1's weights: J+1 = 1..3 from rawa, 4..7 from rawb, 8 = the next super-block's 0 from rawa
    // (past the last step: a slab nobody reads)
    constexpr int J1 = (J + 1) & 7;
#pragma unroll
    for (int kk = 0; kk < 2; kk++) {
      v8bf af[NA], bf[NB];
#pragma unroll
      for (int a = 0; a < NA; a++) af[a] = *(const v8bf*)(xs + (aoff[a] ^ (32 * kk)));
#pragma unroll
      for (int b = 0; b < NB; b++) bf[b] = *(const v8bf*)(ws + (boff[b] ^ (32 * kk)));
      if (kk == 0) dequant_to(J1 < 4 ? rawa : rawb, J1 & 3, J1 >> 2, J1 & 1);
#pragma unroll
      for (int a = 0; a < NA; a++)
#pragma unroll
        for (int b = 0; b < NB; b++) acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[a], bf[b], acc[a][b], 0, 0, 0);
    }
    const int s = st0; st0 = st1; st1 = st2; st2 = s;
  };
  for (int ks = 8 * sb0; ks < 8 * sb1; ks += 8) {     // one super-block of 256 columns
    step(ks + 0, std::integral_constant<int, 0>{});
    step(ks + 1, std::integral_constant<int, 1>{});
    step(ks + 2, std::integral_constant<int, 2>{});
    step(ks + 3, std::integral_constant<int, 3>{});
    step(ks + 4, std::integral_constant<int, 4>{});
    step(ks + 5, std::integral_constant<int, 5>{});
    step(ks + 6, std::integral_constant<int, 6>{});
    step(ks + 7, std::integral_constant<int, 7>{});
  }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the tail's redundant loads: nothing may land in LDS after the workgroup ends

  if (part) {              // the sums of this run of columns, the whole tile (what lies past the matrix or the tokens: never read)
    BfParams q = p;
    q.y = p.part + (long)((int)blockIdx.x - p.split_from) * (TM * TN); q.ldy = TM; q.rows = TM; q.bias = nullptr; q.acc = 0;
    store_tile<NA, NB>(acc, q, 0, TN, 0, wt0, wr0, l32, lh);
  } else {
    store_tile<NA, NB>(acc, p, tok0, ntok, r0, wt0, wr0, l32, lh);
  }
}

// The split tiles' parts added up, part after part, and written to y as store_tile writes a tile (bias, acc).
// Grid (TM * TN / 1024, tiles): a thread four rows of a token.
template <int TM, int TN>
__global__ __launch_bounds__(256) void bf16_split_sum_kernel(BfParams p) {
  const int ti = blockIdx.y, e = ((int)blockIdx.x * 256 + (int)threadIdx.x) * 4, tok = e / TM, row = e - tok * TM;
  const int NT = (p.ntok + TN - 1) / TN, NR = (p.rows + TM - 1) / TM;
  int rt, tt;
  tile_place(p.split_from + ti, NT, NR, rt, tt);
  const long tk = (long)tt * TN + tok;
  if (tk >= p.ntok) return;
  const float* src = p.part + (long)ti * p.ksplit * (TM * TN) + e;
  float4 s = *(const float4*)src;
  for (int k = 1; k < p.ksplit; k++) {
    const float4 v = *(const float4*)(src + (long)k * (TM * TN));
    s.x = s.x + v.x; s.y = s.y + v.y; s.z = s.z + v.z; s.w = s.w + v.w;
  }
  const float o[4] = {s.x, s.y, s.z, s.w};
  float* y = p.y + tk * p.ldy;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int r = rt * TM + row + i;
    if (r < p.rows) {
      float v = o[i];
      if (p.bias) v = v + p.bias[r];
      if (p.acc) v = y[r] + v;
      y[r] = v;
    }
  }
}

// ---- the grouped product with the weights dequantized into MFMA operands ------------------------
// An expert's group of a prefill chunk is a hundred rows of tokens or so: one token tile, so
// every weight is dequantized once whichever way, and the kernel above then spends more of the
// LDS's bandwidth on weights (the slab written, then read by two waves as fragments) than on
// anything else, and its per-lane loads of 16 or 32 bytes from as many rows as lanes ask the
// memory pipeline for a whole line each.  Here
//  - the quantized blocks go to LDS as they are, by direct loads of 16 bytes a lane from
//    consecutive addresses (5 or 6 pieces a block, see RegB), a super-block (8 steps) of the
//    tile's 256 rows at a time into one of two buffers, one load a wave and step;
//  - a wave keeps 64 rows of W to itself, over all of the tile's 128 tokens: lane (l32, lh)
//    dequantizes the 8 weights of a row that make up its share of an MFMA's B operand --
//    columns 16*kk + 8*lh .. + 7 of the step, of row 32*b + l32 -- from the block in LDS straight
//    into registers, and only the activations go through LDS as bf16;
//  - the token patches past the group's last row are skipped (a group of 40 rows takes half
//    the MFMAs of one of 128).
template <int FMT> struct RegB;

// IQ2_XXS in LDS: 80 bytes a block, the 64 bytes of the eight groups first (four pieces from
// byte 2 of the block on), then the block's first 16 bytes, which start with d.  A lane's raw
// set covers two steps (a quarter of a super-block: two groups of 32 weights, 8 bytes each).
template <> struct RegB<ILT_IQ2_XXS> {
  static constexpr int PPB = 5, LB = 80, BB = 66;
  static constexpr int P = 2;                          // steps a set covers
  static __device__ __forceinline__ u32 goff(u32 pc) { return pc == 4 ? 0u : 2 + 16 * pc; }
  struct Raw { int4 q; u32 d; };
  struct Prep { u32 g, sg, t01, t2; };
  // u: the set's place in the super-block
  static __device__ __forceinline__ void load(Raw& r, const u8* blk, int u, int lh) {
    r.q = ilt_lds_ld16(blk + 16 * u);
    r.d = *(const ILT_LDS u16*)(blk + 64);
  }
  // j: the step within the set.  The three magnitudes as dequant16_pk makes them.
  static __device__ __forceinline__ Prep prep(const Raw& r, int j, int lh) {
    const u32 aux = word_of(r.q, 2 * j + 1);
    const float db = (ilt_h2f((u16)r.d) * (0.5f + (float)(aux >> 28))) * 0.25f;
    return { word_of(r.q, 2 * j) >> (8 * lh), aux >> (7 * lh), pack_bf16(db * 8.0f, db * 25.0f), pack_bf16(db * 43.0f, 0.0f) };
  }
  // the lane's 8 weights of unit kk of the step
  static __device__ __forceinline__ v8bf frag(const Raw&, const Prep& pr, int j, int kk, int lh, const Iq2Tables* T) {
    const int4 sel = ilt_lds_ld16(T->sel[(pr.g >> (16 * kk)) & 0xFF]);
    const int4 sm = ilt_lds_ld16(T->sgn[(pr.sg >> (14 * kk)) & 127]);
    u32 pk[4];
    pk[0] = __builtin_amdgcn_perm(pr.t2, pr.t01, (u32)sel.x) ^ (u32)sm.x;
    pk[1] = __builtin_amdgcn_perm(pr.t2, pr.t01, (u32)sel.y) ^ (u32)sm.y;
    pk[2] = __builtin_amdgcn_perm(pr.t2, pr.t01, (u32)sel.z) ^ (u32)sm.z;
    pk[3] = __builtin_amdgcn_perm(pr.t2, pr.t01, (u32)sel.w) ^ (u32)sm.w;
    v8bf out; __builtin_memcpy(&out, pk, 16); return out;
  }
};

// Q2_K in LDS: 96 bytes a block, its first 80 bytes (16 scale bytes, 64 of quants) as five
// pieces, then bytes 68..83, whose last four are d and dmin: they land at 92.
// A 16-weight unit has one scale and one minimum, so its weights take four values,
// fma(dl, q, -ml) for q = 0..3 as the CPU forms them: the lane makes those once for a whole
// unit -- unit lh of the step, both halves of it -- and picks each weight's bf16 with byte
// permutes that take the 2-bit codes as selectors.  Lane (l32, 0) then holds columns 0..15 of
// the step and lane (l32, 1) columns 16..31, where the MFMA wants columns 16*kk + 8*lh ..:
// one swap of the second half of the low lanes with the first half of the high lanes
// (v_permlane32_swap) gives both operands.
template <> struct RegB<ILT_Q2_K> {
  static constexpr int PPB = 6, LB = 96, BB = 84;
  static constexpr int P = 4;
  static __device__ __forceinline__ u32 goff(u32 pc) { return pc == 5 ? 68u : 16 * pc; }
  struct Raw { int4 q; u32 sc, dd; };                  // of a step: the unit's 16 bytes of quants, its scale byte, d and dmin
  // J: the step within the super-block
  static __device__ __forceinline__ void read(Raw& r, const u8* blk, int J, int lh) {
    r.q = ilt_lds_ld16(blk + 16 + 32 * (J >> 2) + 16 * lh);
    r.sc = *(const ILT_LDS u8*)(blk + 2 * J + lh);
    r.dd = *(const ILT_LDS u32*)(blk + 92);
  }
  static __device__ __forceinline__ void make(const Raw& r, int J, v8bf& f0, v8bf& f1) {
    const float dl = ilt_h2f((u16)(r.dd & 0xFFFF)) * (float)(r.sc & 15), ml = ilt_h2f((u16)(r.dd >> 16)) * (float)(r.sc >> 4);
    // (q = 0 and 1 as fma too: -ml and dl - ml but for the sign of a zero)
    const u32 p01 = pack_bf16(__builtin_fmaf(dl, 0.0f, -ml), __builtin_fmaf(dl, 1.0f, -ml));
    const u32 p23 = pack_bf16(__builtin_fmaf(dl, 2.0f, -ml), __builtin_fmaf(dl, 3.0f, -ml));
    const u32 lo4 = __builtin_amdgcn_perm(p23, p01, 0x06040200u), hi4 = __builtin_amdgcn_perm(p23, p01, 0x07050301u);   // the four low bytes, the four high bytes
    u32 pk[8];
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const u32 v = (word_of(r.q, i) >> (2 * (J & 3))) & 0x03030303;       // weights 4i .. 4i+3 of the unit
      const u32 lo = __builtin_amdgcn_perm(lo4, lo4, v), hi = __builtin_amdgcn_perm(hi4, hi4, v);
      pk[2 * i] = __builtin_amdgcn_perm(hi, lo, 0x05010400u);
      pk[2 * i + 1] = __builtin_amdgcn_perm(hi, lo, 0x07030602u);
    }
    u32 o0[4], o1[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
      // lanes 32..63 of the first (columns 16..23) <-> lanes 0..31 of the second (columns 8..15)
      const auto sw = __builtin_amdgcn_permlane32_swap(pk[i], pk[4 + i], false, false);
      o0[i] = sw[0]; o1[i] = sw[1];
    }
    __builtin_memcpy(&f0, o0, 16);
    __builtin_memcpy(&f1, o1, 16);
  }
};

struct TileSel { u32 scan[256]; int tile_z, tile_t0, tile_n, pad; };

// dynamic LDS: the x ring, the two buffers of blocks, the tile choice's scratch, IQ2_XXS's tables
template <int FMT> constexpr size_t regb_smem() {
  return 3 * 128 * KS * 2 + 2 * 256 * RegB<FMT>::LB + sizeof(TileSel) + (FMT == ILT_IQ2_XXS ? sizeof(Iq2Tables) : 0);
}

// GLU: the tile's 256 rows are 128 rows of the gate matrix and the same 128 of the up matrix,
// a wave's row patch 0 gate rows and patch 1 the up rows of the same numbers, so that a lane
// holds both products of a (token, row) and the epilogue writes the gated activation.
template <int FMT, bool GLU>
__global__ __launch_bounds__(256, 2) void gemm_bf16_regb_kernel(BfParams p) {
  constexpr int TM = 256, TN = 128, NA = 4, NB = 2, NI = 2;
  constexpr int TR = GLU ? 128 : 256;                        // rows of a matrix a tile covers
  typedef RegB<FMT> R;
  constexpr int P = R::P, UPS = 8 / P;                       // steps a raw set covers, sets a super-block
  constexpr int NWW = TM * R::PPB / 64 / 4;                  // block loads a wave and super-block: 5 or 6
  constexpr int WPS = P == 4 ? 2 : 1;                        // of which it sends this many a step, from step 0 on
  constexpr int WSTEPS = (NWW + WPS - 1) / WPS;
  constexpr int XS = TN * KS * 2, WS = TM * R::LB;
  extern __shared__ __align__(16) u8 regb_lds[];
  u8* const xsl = regb_lds;                                  // [3][XS]
  u8* const wsl = regb_lds + 3 * XS;                         // [2][WS]
  TileSel& S = *(TileSel*)(regb_lds + 3 * XS + 2 * WS);
  const Iq2Tables* T = (const Iq2Tables*)(regb_lds + 3 * XS + 2 * WS + sizeof(TileSel));
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;

  long tok0; int ntok, rt; const u8* w = p.w;
  if (!pick_tile<TR, TN>(p, S, tok0, ntok, rt, w)) return;
  const int r0 = rt * TR;
  if (FMT == ILT_IQ2_XXS) iq2_tables_fill(*(Iq2Tables*)T, t);     // (a barrier follows, before the first operands are made)

  const int l32 = lane & 31, lh = lane >> 5, wr0 = 64 * wave;
  // the pieces this lane sends to LDS for a super-block: piece 64*(wave + 4*i) + lane of the tile's 256 * PPB
  const u8* wbase = (const u8*)ilt_uniform_ptr(w);
  // (the addresses are made anew for every load: registers are scarcer than instruction slots)
  const u32 wq0 = 64 * wave + lane, wrow_bytes = (u32)p.row_bytes, wlast = (u32)(p.rows - 1 - r0);
  const u8* xbase = (const u8*)ilt_uniform_ptr(p.rmap ? p.x : p.x + tok0 * (long)p.cols);
  u32 xoff[NI];
#pragma unroll
  for (int i = 0; i < NI; i++) {
    const int P_ = (wave * NI + i) * 64 + lane, tok = P_ >> 2, kp = (P_ & 3) ^ (int)slab_swz(tok);
    const int tk = min(tok, ntok - 1);
    xoff[i] = (p.rmap ? p.rmap[tok0 + tk] : (u32)tk) * (u32)p.cols * 2 + 16 * kp;
  }

  v16f acc[NA][NB];
#pragma unroll
  for (int a = 0; a < NA; a++)
#pragma unroll
    for (int b = 0; b < NB; b++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[a][b][r] = 0.0f;
  const u32 aoff0 = slab_off(l32, lh);                        // token 32a + l32: 2048a on (its swizzle is the same)
  const u32 blk0 = (u32)(wr0 + l32) * R::LB;                  // this lane's first row's block in a buffer; the second 32 blocks on

  const int nk = p.cols / KS, nsb = nk / 8;
  auto issue_x = [&](int stage, int ks) {
#pragma unroll
    for (int i = 0; i < NI; i++) ilt_g2lds16(xbase + ks * (KS * 2) + xoff[i], xsl + stage * XS + (wave * NI + i) * 1024);
  };
  auto issue_w = [&](int i, int sb, int buf) {               // load i of super-block sb's blocks
    const u32 q = wq0 + 256 * i, row = __umulhi(q, 0xFFFFFFFFu / R::PPB + 1), pc = q - row * R::PPB;
    // GLU: tile row 64w + 32b + l is row 32w + l of the gate (b = 0) or up (b = 1) matrix's 128
    const u32 mrow = GLU ? ((row >> 6) << 5) | (row & 31) : row;
    const u32 off = __umul24(r0 + min(mrow, wlast), wrow_bytes) + R::goff(pc) + (GLU && (row & 32) ? p.up_delta : 0u);
    ilt_g2lds16(wbase + (u32)sb * R::BB + off, wsl + buf * WS + (wave + 4 * i) * 1024);
  };
#pragma unroll
  for (int i = 0; i < NWW; i++) issue_w(i, 0, 0);
  issue_x(0, 0);
  issue_x(1, 1);
  asm volatile("s_waitcnt vmcnt(%0)" :: "n"(2 * NI) : "memory");
  __syncthreads();

  // what every step starts with: the waits, the barrier, the loads it sends off
  auto step_head = [&](int ks, auto Jc, int st2) {
    constexpr int J = decltype(Jc)::value;                   // the step's place in its super-block
    const int sb = ks >> 3;
    // All loads but the previous step's have landed: this step's x slab has (sent two steps ago).
    constexpr int sent = (J >= 1 && J <= WSTEPS) ? (NWW - (J - 1) * WPS < WPS ? NWW - (J - 1) * WPS : WPS) : 0;   // block loads of the previous step
    asm volatile("s_waitcnt vmcnt(%0)" :: "n"(NI + sent) : "memory");
    ilt_barrier_lds();                                       // no fence: later steps' loads stay in flight
#pragma unroll
    for (int i = J * WPS; i < ((J + 1) * WPS < NWW ? (J + 1) * WPS : NWW); i++) issue_w(i, min(sb + 1, nsb - 1), (sb + 1) & 1);
    issue_x(st2, min(ks + 2, nk - 1));
  };
  auto eight_steps = [&](auto& step) {
    for (int ks = 0; ks < nk; ks += 8) {
      step(ks + 0, std::integral_constant<int, 0>{});
      step(ks + 1, std::integral_constant<int, 1>{});
      step(ks + 2, std::integral_constant<int, 2>{});
      step(ks + 3, std::integral_constant<int, 3>{});
      step(ks + 4, std::integral_constant<int, 4>{});
      step(ks + 5, std::integral_constant<int, 5>{});
      step(ks + 6, std::integral_constant<int, 6>{});
      step(ks + 7, std::integral_constant<int, 7>{});
    }
  };

  if constexpr (FMT == ILT_Q2_K) {
    // Step ks multiplies with the operands made during step ks-1 and makes step ks+1's: its
    // first half row patch 0's (both units), its second half row patch 1's, from raw bytes read
    // out of LDS at the step's start.
    typedef typename R::Raw Raw;
    v8bf bq[2][2][NB];                                       // [step parity][unit][row patch]
    {
      Raw r0_[NB];
#pragma unroll
      for (int b = 0; b < NB; b++) R::read(r0_[b], wsl + blk0 + b * 32 * R::LB, 0, lh);
#pragma unroll
      for (int b = 0; b < NB; b++) R::make(r0_[b], 0, bq[0][0][b], bq[0][1][b]);
    }
    auto run = [&](auto NALc) {
      constexpr int NAL = decltype(NALc)::value;             // token patches that hold rows
      int st0 = 0, st1 = 1, st2 = 2;
      auto step = [&](int ks, auto Jc) {
        constexpr int J = decltype(Jc)::value, J1 = (J + 1) & 7;
        step_head(ks, Jc, st2);
        Raw rn[NB];                                          // (past the last step: the last super-block's again)
        const u8* wnext = wsl + (((ks >> 3) + (J == 7 ? 1 : 0)) & 1) * WS + blk0;
#pragma unroll
        for (int b = 0; b < NB; b++) R::read(rn[b], wnext + b * 32 * R::LB, J1, lh);
        __builtin_amdgcn_sched_barrier(0);
        const u8* xs = xsl + st0 * XS;
#pragma unroll
        for (int kk = 0; kk < 2; kk++) {
          v8bf af[NAL];
#pragma unroll
          for (int a = 0; a < NAL; a++) af[a] = *(const v8bf*)(xs + (aoff0 ^ (32 * kk)) + 2048 * a);
#pragma unroll
          for (int a = 0; a < NAL; a++)
#pragma unroll
            for (int b = 0; b < NB; b++) acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[a], bq[J & 1][kk][b], acc[a][b], 0, 0, 0);
          R::make(rn[kk], J1, bq[J1 & 1][0][kk], bq[J1 & 1][1][kk]);      // row patch kk of the next step
        }
        const int s_ = st0; st0 = st1; st1 = st2; st2 = s_;
      };
      eight_steps(step);
    };
    switch ((ntok + 31) >> 5) {
      case 1: run(std::integral_constant<int, 1>{}); break;
      case 2: run(std::integral_constant<int, 2>{}); break;
      case 3: run(std::integral_constant<int, 3>{}); break;
      default: run(std::integral_constant<int, 4>{}); break;
    }
  } else {
    // Raw sets A and B take turns, P steps each, and are read out of LDS P steps (B) or 2P-1..P
    // (A) before their turn.  Half-step (ks, kk) multiplies with bq[kk] and makes the operands of
    // the half-step after it: (ks, 1) during (ks, 0), (ks+1, 0) during (ks, 1).  Super-block
    // sb+1's blocks are sent for during the first steps of super-block sb, into the buffer that
    // was last read early in super-block sb-1, and have landed when the first set is read from
    // them (step 8-P of sb).
    typedef typename R::Raw Raw;
    typedef typename R::Prep Prep;
    Raw rawa[NB], rawb[NB];
    Prep pr[NB];
    v8bf bq[2][NB];
    auto load_raw = [&](Raw* raw, int unit) {                  // set number unit of the row, out of LDS
      const int sb = unit / UPS;
#pragma unroll
      for (int b = 0; b < NB; b++) R::load(raw[b], wsl + (sb & 1) * WS + blk0 + b * 32 * R::LB, unit - sb * UPS, lh);
    };
    load_raw(rawa, 0);
#pragma unroll
    for (int b = 0; b < NB; b++) { pr[b] = R::prep(rawa[b], 0, lh); bq[0][b] = R::frag(rawa[b], pr[b], 0, 0, lh, T); }

    auto run = [&](auto NALc) {
      constexpr int NAL = decltype(NALc)::value;               // token patches that hold rows
      int st0 = 0, st1 = 1, st2 = 2;
      auto step = [&](int ks, auto Jc) {
        constexpr int J = decltype(Jc)::value;                 // the step's place in its super-block
        constexpr int JJ = J % (2 * P);                        // and in a round of both sets
        step_head(ks, Jc, st2);
        if (JJ == 0) load_raw(rawb, min(ks / P + 1, nk / P - 1));
        if (JJ == P) load_raw(rawa, min(ks / P + 1, nk / P - 1));
        __builtin_amdgcn_sched_barrier(0);
        const u8* xs = xsl + st0 * XS;
        constexpr int J1 = (JJ + 1) % (2 * P);
#pragma unroll
        for (int kk = 0; kk < 2; kk++) {
          v8bf af[NAL];
#pragma unroll
          for (int a = 0; a < NAL; a++) af[a] = *(const v8bf*)(xs + (aoff0 ^ (32 * kk)) + 2048 * a);
          if (kk == 0) {
#pragma unroll
            for (int b = 0; b < NB; b++) bq[1][b] = R::frag(JJ < P ? rawa[b] : rawb[b], pr[b], JJ % P, 1, lh, T);
          }
#pragma unroll
          for (int a = 0; a < NAL; a++)
#pragma unroll
            for (int b = 0; b < NB; b++) acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[a], bq[kk][b], acc[a][b], 0, 0, 0);
          if (kk == 1) {       // (past the last step: operands nobody multiplies with)
#pragma unroll
            for (int b = 0; b < NB; b++) {
              pr[b] = R::prep(J1 < P ? rawa[b] : rawb[b], J1 % P, lh);
              bq[0][b] = R::frag(J1 < P ? rawa[b] : rawb[b], pr[b], J1 % P, 0, lh, T);
            }
          }
        }
        const int s = st0; st0 = st1; st1 = st2; st2 = s;
      };
      eight_steps(step);
    };
    switch ((ntok + 31) >> 5) {
      case 1: run(std::integral_constant<int, 1>{}); break;
      case 2: run(std::integral_constant<int, 2>{}); break;
      case 3: run(std::integral_constant<int, 3>{}); break;
      default: run(std::integral_constant<int, 4>{}); break;
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the tail's redundant loads: nothing may land in LDS after the workgroup ends

  if constexpr (GLU) {
    // register r of patch a: token 32a + 8*(r/4) + 4*lh + r%4 of the tile, row r0 + 32*wave + l32.
    // Through descriptors that end with the tile's last token: a load past it gives 0, a store is dropped.
    const int row = r0 + 32 * wave + l32;
    const u32 nt = (u32)__builtin_amdgcn_readfirstlane(ntok);
    const __amdgpu_buffer_rsrc_t rwt = ilt_rsrc(ilt_uniform_ptr(p.wrow + tok0), nt * 4);
    const __amdgpu_buffer_rsrc_t rm = ilt_rsrc(ilt_uniform_ptr(p.mid + tok0 * (long)p.rows), (nt - 1) * (u32)p.rows * 2 + (u32)p.rows * 2);
    const u32 base = row < p.rows ? (u32)row * 2 : 0x80000000u;
#pragma unroll
    for (int a = 0; a < NA; a++) {
      if (32 * a < ntok) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const u32 tk = (u32)(32 * a + 8 * (r >> 2) + 4 * lh + (r & 3));
          const float wv = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rwt, tk * 4, 0, 0));
          float g = acc[a][0][r], u = acc[a][1][r];
          if (p.clamp > 1e-6f) { g = fminf(g, p.clamp); u = fmaxf(-p.clamp, fminf(u, p.clamp)); }
          const float o = (ilt_silu(g) * u) * wv;
          __builtin_amdgcn_raw_buffer_store_b16((u16)(pack_bf16(o, 0.0f) & 0xFFFF), rm, base + tk * (u32)p.rows * 2, 0, 0);
        }
      }
    }
  } else {
    store_tile<NA, NB>(acc, p, tok0, ntok, r0, 0, wr0, l32, lh);
  }
}

template <int FMT, bool GLU>
hipError_t launch_regb(const BfParams& p, long long token_tiles, hipStream_t st) {
  const long long total = token_tiles * (p.rows / (GLU ? 128 : 256)), per = (total + 7) / 8;
  if (per * 8 > 0x7FFFFFFFLL) return hipErrorInvalidValue;
  static bool attr_set[8] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 8) dev = 0;
  if (!attr_set[dev]) {            // more dynamic LDS than the default 64 KB: asked for once per device
    const hipError_t e = hipFuncSetAttribute((const void*)gemm_bf16_regb_kernel<FMT, GLU>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)regb_smem<FMT>());
    if (e != hipSuccess) return e;
    attr_set[dev] = true;
  }
  hipLaunchKernelGGL((gemm_bf16_regb_kernel<FMT, GLU>), dim3((unsigned)(per * 8)), dim3(256), regb_smem<FMT>(), st, p);
  return hipGetLastError();
}

// ---- the exact product on the same pipeline: Q6_K and Q4_K as two int8 planes -------------------
// Bit for bit the CPU path's MATMUL! (and gemm_i8_kernel's) result: per super-block an integer
// isum = sum over its 256 columns of (scale * quant) * xq, then sum += (d*yd) * float(isum) (and
// Q4_K's term of the minimums before it), block after block (kquant.lisp:180-236).  Any exact
// way to the integer will do, so the products P = sc*(q-32) (Q6_K, 13 bits) or sc*q (Q4_K, 10
// bits) go to the int8 matrix cores as two planes, the bytes of T = P + C0 >= 0 (C0 = 4128 or
// 0): hi = T >> 8 (0..31) and lo = (T & 255) - 128, so
//   isum = 256*(hi.xq) + (lo.xq) + (128 - C0)*(sum of the block's xq),
// the last from the activations' sums of 16.  v_mfma_i32_32x32x32_i8 accumulates both planes
// over the super-block's four steps of 64 columns; the lanes then combine them once per block.
// Four weights are made at a time: the even and the odd bytes of a word as two 16-bit fields
// and one 24-bit multiply(-add) for both fields (each field's total is within 0..65535, so
// borrows between them cancel).  Q4_K's sum of minimum * (sum of 32 quants) over the eight
// groups is one more pair of small products per super-block, the sums of 32 split into planes
// the same way.
typedef int v4i_ __attribute__((ext_vector_type(4)));
typedef int v16i_ __attribute__((ext_vector_type(16)));
typedef int v3i_ __attribute__((ext_vector_type(3)));

template <int FMT> struct I8p;

// Thread (row, q4) makes columns 16*q4.. of its row in every step of 64 columns: part
// 2*jj + q4/2 of half c (jj = the step within the half), weights 16*(q4 & 1).. of the part.
template <> struct I8p<ILT_Q6_K> {
  static constexpr int KCX = 4000;                           // isum = 256*hi + lo - KCX * (sum of xq)
  static constexpr int PLANES = 2, WL = 4;                   // planes; loads of a raw set
  struct Raw { int4 ql, qh; int2 sc; u32 d; };               // a half super-block's share
  static __device__ __forceinline__ void load(Raw& r, __amdgpu_buffer_rsrc_t rw, u32 rowoff, int hb, int q4) {
    const u32 b = rowoff + (u32)(hb >> 1) * ILT_Q6K_STRIDE;
    const int c = hb & 1;
    r.ql = ilt_bld16(rw, b + 64 * c + 16 * q4);              // ql[64c + 32*(part & 1) + l], part & 1 = q4 / 2, l = 16*(q4 & 1)..
    r.qh = ilt_bld16(rw, b + 128 + 32 * c + 16 * (q4 & 1));
    r.sc = ilt_bld8(rw, b + 192 + 8 * c);
    r.d = ilt_bld2(rw, b + 208);
  }
  static __device__ __forceinline__ float d_of(const Raw& r) { return ilt_h2f((u16)r.d); }
  // J: the step within the super-block
  template <typename SM> static __device__ __forceinline__ void planes(const Raw& r, int J, int q4, int* hi, int* lo, const SM&) {
    const int jj = J & 1;
    const int sc = (int)(i8)(((u32)(jj ? r.sc.y : r.sc.x) >> (8 * q4)) & 0xFF);      // scale 8c + 2*part + (q4 & 1)
    const int cpair = (4128 - 32 * sc) * 0x10001;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const u32 v = ((word_of(r.ql, i) >> (4 * jj)) & 0x0F0F0F0F) | (((word_of(r.qh, i) >> (4 * jj + 2 * (q4 >> 1))) & 0x03030303) << 4);
      const u32 te = (u32)(__mul24((int)(v & 0x00FF00FF), sc) + cpair), to = (u32)(__mul24((int)((v >> 8) & 0x00FF00FF), sc) + cpair);
      hi[i] = (int)__builtin_amdgcn_perm(to, te, 0x07030501u);                  // the fields' high bytes, in the weights' order
      lo[i] = (int)(__builtin_amdgcn_perm(to, te, 0x06020400u) ^ 0x80808080u);   // their low bytes - 128
    }
  }
};

// Q4_K: step J of a super-block is groups 2J (low nibbles) and 2J+1 (high nibbles) of qs[32J..32J+31].
template <> struct I8p<ILT_Q4_K> {
  static constexpr int KCX = -128;
  static constexpr int PLANES = 2, WL = 4;
  struct Raw { int4 q[2]; v3i_ s; u32 dd; };                 // a half's two steps of quants (the thread's 16 bytes), the block's 12 scale bytes, d and dmin
  static __device__ __forceinline__ void load(Raw& r, __amdgpu_buffer_rsrc_t rw, u32 rowoff, int hb, int q4) {
    const u32 b = rowoff + (u32)(hb >> 1) * 144;
    r.q[0] = ilt_bld16(rw, b + 16 + 64 * (hb & 1) + 16 * (q4 & 1));
    r.q[1] = ilt_bld16(rw, b + 48 + 64 * (hb & 1) + 16 * (q4 & 1));
    r.s = __builtin_amdgcn_raw_buffer_load_b96(rw, b + 4, 0, 0);
    r.dd = ilt_bld4(rw, b);
  }
  static __device__ __forceinline__ float d_of(const Raw& r) { return ilt_h2f((u16)(r.dd & 0xFFFF)); }
  static __device__ __forceinline__ float dmin_of(const Raw& r) { return ilt_h2f((u16)(r.dd >> 16)); }
  static __device__ __forceinline__ u32 sbyte(const Raw& r, int i) { return ((u32)(i < 4 ? r.s.x : i < 8 ? r.s.y : r.s.z) >> (8 * (i & 3))) & 0xFF; }
  // scale-min-k4 (kquant.lisp:64-72), g a constant
  static __device__ __forceinline__ u32 scale_of(const Raw& r, int g) {
    return g < 4 ? (sbyte(r, g) & 63) : ((sbyte(r, g + 4) & 15) | ((sbyte(r, g - 4) >> 6) << 4));
  }
  static __device__ __forceinline__ u32 min_of(const Raw& r, int g) {
    return g < 4 ? (sbyte(r, g + 4) & 63) : ((sbyte(r, g + 4) >> 4) | ((sbyte(r, g) >> 6) << 4));
  }
  template <typename SM> static __device__ __forceinline__ void planes(const Raw& r, int J, int q4, int* hi, int* lo, const SM&) {
    const int jp = q4 >> 1;                                  // group 2J + jp
    const int sc = (int)(jp ? scale_of(r, 2 * J + 1) : scale_of(r, 2 * J));
    const int4& q = r.q[J & 1];
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const u32 v = (word_of(q, i) >> (4 * jp)) & 0x0F0F0F0F;
      const u32 te = (u32)__mul24((int)(v & 0x00FF00FF), sc), to = (u32)__mul24((int)((v >> 8) & 0x00FF00FF), sc);
      hi[i] = (int)__builtin_amdgcn_perm(to, te, 0x07030501u);
      lo[i] = (int)(__builtin_amdgcn_perm(to, te, 0x06020400u) ^ 0x80808080u);
    }
  }
};

// Q2_K: sc*q is at most 45, one plane.  Step J of a super-block is parts 2*(J&1) and 2*(J&1)+1 of half J/2, all four
// parts of a half in the same 32 bytes of quants, two bits each; the minimums' term over the sixteen groups of 16.
template <> struct I8p<ILT_Q2_K> {
  static constexpr int KCX = 0;
  static constexpr int PLANES = 1, WL = 3;
  struct Raw { int4 q, s; u32 dd; };                         // the thread's 16 bytes of the half's quants, the block's 16 scale bytes, d and dmin
  static __device__ __forceinline__ void load(Raw& r, __amdgpu_buffer_rsrc_t rw, u32 rowoff, int hb, int q4) {
    const u32 b = rowoff + (u32)(hb >> 1) * 84;
    r.q = ilt_bld16(rw, b + 16 + 32 * (hb & 1) + 16 * (q4 & 1));
    r.s = ilt_bld16(rw, b);
    r.dd = ilt_bld4(rw, b + 80);
  }
  static __device__ __forceinline__ float d_of(const Raw& r) { return ilt_h2f((u16)(r.dd & 0xFFFF)); }
  static __device__ __forceinline__ float dmin_of(const Raw& r) { return ilt_h2f((u16)(r.dd >> 16)); }
  template <typename SM> static __device__ __forceinline__ void planes(const Raw& r, int J, int q4, int*, int* lo, const SM&) {
    const int c = J >> 1, jj = J & 1;
    const u32 sc = (word_of(r.s, 2 * c + jj) >> (8 * q4)) & 15;             // scale 8c + 2*part + (q4 & 1), part = 2jj + q4/2
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const u32 v = (word_of(r.q, i) >> (4 * jj + 2 * (q4 >> 1))) & 0x03030303;
      lo[i] = (int)(v * sc);                                  // four products of at most 45: no carries between the bytes
    }
  }
};

template <int TM> struct I8pSmemT {
  __align__(16) u8 xs[3][128 * 64];       // the tokens' quants, 64 columns a step
  __align__(16) u8 wh[2][TM * 64];        // the rows' hi plane, the step's and the next step's
  __align__(16) u8 wl[2][TM * 64];        // lo plane
  float wd[128], wdm[128];                // of the super-block: d (and Q4_K's dmin) of the rows,
  float xd[128];                          //   the tokens' scales
  int cx[128];                            //   and KCX * the sum of their quants
  union {
    // Q4_K's minimums: the rows' eight minimums and their sum; the tokens' eight sums of 32 as planes
    // (U = sum + 4096: U >> 8, and (U & 255) - 128)
    struct { int2 wmn[128]; int wms[128]; int2 bh[128], bl[128]; };
    // IQ2_XXS: the codebook, and for each 7-bit sign index (+ parity) 0xFF in the bytes of the negative weights
    struct { u64 grid[256]; u64 smask[128]; };
  };
  u32 scan[256];
  int tile_z, tile_t0, tile_n;
};
typedef I8pSmemT<128> I8pSmem;

// IQ2_XXS: a block's eight groups of 32 weights add (float(sumi) * (0.5 + scale)) alternately to two sums,
// fa (even groups) and fb (odd), then sum += (d*yd) * (fa + fb) (iquant.lisp:161-215).  Every term is a
// multiple of 1/2, and with the codebook's entries (byte sums of at most 203) twice a sum of four of them
// stays below 2^24 (at most 4 * 31 * 4 * 128 * 203 = 12,888,064): none of those float additions rounds, and
// fa = float(S) * 0.5 for the integer S = sum over the even groups of (2*scale + 1) * sumi.  (Were the
// last addition to round, it would round the exact sum once, as the conversion of S does.)  So the weights go in as (2*scale + 1) * (signed
// magnitude), at most 1333 in absolute value, + 1408 as two planes, and a step's first 32 columns (an even
// group) and second 32 (an odd one) have integer sums of their own.
template <> struct I8p<ILT_IQ2_XXS> {
  static constexpr int KCX = 1280;
  static constexpr int PLANES = 2, WL = 3;
  struct Raw { int2 g[2]; u32 d; };                          // the thread's group of each of the half's two steps (8 bytes: four codebook indices, signs and scale), d
  static __device__ __forceinline__ void load(Raw& r, __amdgpu_buffer_rsrc_t rw, u32 rowoff, int hb, int q4) {
    const u32 b = rowoff + (u32)(hb >> 1) * 66 + 2 + 8 * (4 * (hb & 1) + (q4 >> 1));
    r.g[0] = ilt_bld8(rw, b);
    r.g[1] = ilt_bld8(rw, b + 16);
    r.d = ilt_bld2(rw, rowoff + (u32)(hb >> 1) * 66);
  }
  static __device__ __forceinline__ float d_of(const Raw& r) { return ilt_h2f((u16)r.d); }
  template <typename SM> static __device__ __forceinline__ void planes(const Raw& r, int J, int q4, int* hi, int* lo, const SM& S) {
    const u32 idx = (u32)r.g[J & 1].x, aux = (u32)r.g[J & 1].y;
    const int mult = 2 * (int)(aux >> 28) + 1;
    const u32 c0 = 1408u * 0x10001u;
#pragma unroll
    for (int l2 = 0; l2 < 2; l2++) {
      const int l = 2 * (q4 & 1) + l2;                       // the group's l-th run of 8 weights
      const int2 mag = ilt_lds_ld8(&S.grid[(idx >> (8 * l)) & 0xFF]);
      const int2 neg = ilt_lds_ld8(&S.smask[(aux >> (7 * l)) & 127]);
#pragma unroll
      for (int h = 0; h < 2; h++) {
        const u32 m = (u32)(h ? mag.y : mag.x), nb = (u32)(h ? neg.y : neg.x);
        const u32 pe = (u32)__mul24((int)(m & 0x00FF00FF), mult), po = (u32)__mul24((int)((m >> 8) & 0x00FF00FF), mult);
        const u32 me = __builtin_amdgcn_perm(nb, nb, 0x02020000u), mo = __builtin_amdgcn_perm(nb, nb, 0x03030101u);   // the fields of the negative weights
        const u32 te = (pe ^ me) + (c0 - me), to = (po ^ mo) + (c0 - mo);       // 1408 +- the product, in both fields
        hi[2 * l2 + h] = (int)__builtin_amdgcn_perm(to, te, 0x07030501u);
        lo[2 * l2 + h] = (int)(__builtin_amdgcn_perm(to, te, 0x06020400u) ^ 0x80808080u);
      }
    }
  }
};

__device__ __forceinline__ void ilt_lds_st4_untracked(void* p, u32 v) {
  asm volatile("ds_write_b32 %0, %1" :: "v"((u32)(uintptr_t)(ILT_LDS void*)p), "v"(v) : "memory");
}
__device__ __forceinline__ void ilt_lds_st8_untracked(void* p, u32 a, u32 b) {
  const uint2 v = {a, b};
  asm volatile("ds_write_b64 %0, %1" :: "v"((u32)(uintptr_t)(ILT_LDS void*)p), "v"(v) : "memory");
}

// 128 rows x 128 tokens a workgroup of eight waves (one workgroup a CU, two waves a SIMD: a
// wave's two planes of integer sums, its float sums and the raw bytes leave no room for more);
// wave w: rows 32*(w/2).., tokens 64*(w%2)...  TM 64 (dense): 64 rows x 128 tokens a workgroup of four waves, two or
// three workgroups a CU -- for products whose 128-row tiles are fewer than the CUs, or leave the last round over them
// mostly empty (a prompt's chunk on a small model's matrices); the same sums in the same order.
template <int FMT, bool GROUPED, int TM = 128>
__global__ __launch_bounds__(4 * TM, TM == 128 ? 1 : 2) void gemm_i8p_kernel(BfParams p) {
  typedef I8p<FMT> F;
  typedef typename F::Raw Raw;
  static_assert(TM == 128 || (TM == 64 && !GROUPED), "the grouped wave layout takes eight waves");
  constexpr int TN = 128, NA = 2, THREADS = 4 * TM, NI = 512 / THREADS;
  // Q6_K needs the quants' sum over a block and IQ2_XXS over its even and odd groups (d4_mm_id_iq2_xxs has no argument for
  // the sums of 16 anyway): both are added up from the slabs in LDS, which saves four 16-byte loads a thread and block.
  constexpr bool XSLAB = FMT == ILT_IQ2_XXS || FMT == ILT_Q6_K;
  constexpr int WL = F::WL, XL = XSLAB ? 1 : 5;               // loads of a raw set, of a token's constants
  constexpr bool TWO = F::PLANES == 2;
  constexpr bool SPLIT = FMT == ILT_IQ2_XXS;                 // the first and the second 32 columns of a step have sums of their own
  constexpr int KW = 64;                                     // columns a step
  __shared__ I8pSmemT<TM> S;
  // Q2_K has no hi plane: its room holds the minimums' operands (sixteen groups: 16 bytes a row or token; 6 KB of the
  // hi plane's two slabs, 8 KB at 64 rows)
  int4* const q2_wmn = (int4*)S.wh[0];
  int4* const q2_bh = q2_wmn + 128;
  int4* const q2_bl = q2_bh + 128;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;

  long tok0; int ntok, rt; const u8* w = p.w;
  if (!pick_tile<TM, TN>(p, S, tok0, ntok, rt, w)) return;
  if constexpr (!GROUPED) {
    if (p.nmulti > 1) {                                      // which of the launch's matrices the row tile belongs to
      const int n0 = (p.mrows[0] + TM - 1) / TM, n1 = n0 + (p.mrows[1] + TM - 1) / TM;
      const int m = rt < n0 ? 0 : rt < n1 ? 1 : 2;
      rt -= m == 0 ? 0 : m == 1 ? n0 : n1;
      w = m == 0 ? p.mw[0] : m == 1 ? p.mw[1] : p.mw[2];
      p.rows = m == 0 ? p.mrows[0] : m == 1 ? p.mrows[1] : p.mrows[2];
      p.y = m == 0 ? p.my[0] : m == 1 ? p.my[1] : p.my[2];
      p.bias = m == 0 ? p.mbias[0] : m == 1 ? p.mbias[1] : p.mbias[2];
      p.ldy = p.rows;
    }
  }
  const int r0 = rt * TM;
  int* const cxo = (int*)S.wdm;                              // IQ2_XXS: cx for the even groups, this for the odd ones
  if constexpr (FMT == ILT_IQ2_XXS) {
    if (t < 256) S.grid[t] = bf_grid_dev[t];
    if (t < 128) {
      const u32 sb = (u32)t | ((__popc(t) & 1) << 7);
      u32 m[2] = {0, 0};
#pragma unroll
      for (int j = 0; j < 8; j++) m[j >> 2] |= ((sb >> j) & 1) ? 0xFFu << (8 * (j & 3)) : 0u;
      S.smask[t] = (u64)m[0] | ((u64)m[1] << 32);
    }
    __syncthreads();
  }

  const int wrow = t >> 2, q4 = t & 3;
  const __amdgpu_buffer_rsrc_t rw = ilt_rsrc(ilt_uniform_ptr(w), (u32)min((long long)p.rows * p.row_bytes, 0xFFFFFFF0LL));
  const u32 wrowoff = (u32)((long long)min(r0 + wrow, p.rows - 1) * p.row_bytes);
  const u32 wdst = slab_off(wrow, q4);
  const u8* xbase = (const u8*)ilt_uniform_ptr((const i8*)p.x + tok0 * (long)p.cols);
  u32 xoff[NI];                                              // piece (wave * NI + i) * 64 + lane of a slab: token piece / 4, part piece % 4
#pragma unroll
  for (int i = 0; i < NI; i++) {
    const int P = (wave * NI + i) * 64 + lane;
    xoff[i] = (u32)min(P >> 2, ntok - 1) * (u32)p.cols + 16 * ((P & 3) ^ (int)slab_swz(P >> 2));
  }
  const int nk = p.cols / KW, nsb = p.cols / 256;
  // a token's constants for a super-block, by thread t & 127 (every wave loads, so that all count the same loads)
  const long ctok = tok0 + min(t & 127, ntok - 1);
  const float* xdp = p.xd + ctok * nsb;
  const int4* bsp = (const int4*)(p.bsums + ctok * (p.cols / 16));      // (IQ2_XXS: not read)
  float c_yd; int4 c_bs[4];
  auto load_consts = [&](int sb) {
    c_yd = xdp[sb];
    if constexpr (!XSLAB) {
#pragma unroll
      for (int i = 0; i < 4; i++) c_bs[i] = bsp[4 * sb + i];
    }
  };
  auto store_consts = [&](const Raw& ra) {                   // after a barrier that ends the last block's reads
    if (t < 128) {
      int sx = 0;
      if constexpr (!XSLAB) {
#pragma unroll
        for (int i = 0; i < 4; i++) sx += c_bs[i].x + c_bs[i].y + c_bs[i].z + c_bs[i].w;
      }
      ilt_lds_st4_untracked(&S.xd[t], __builtin_bit_cast(u32, c_yd));
      if constexpr (!XSLAB) ilt_lds_st4_untracked(&S.cx[t], (u32)(F::KCX * sx));
      if constexpr (FMT == ILT_Q4_K) {
        u32 h[2] = {0, 0}, l[2] = {0, 0};
#pragma unroll
        for (int g = 0; g < 8; g++) {                        // the sum of group g's 32 quants
          const int4& bs = c_bs[g >> 1];
          const u32 u = (u32)(((g & 1) ? bs.z + bs.w : bs.x + bs.y) + 4096);
          h[g >> 2] |= (u >> 8) << (8 * (g & 3));
          l[g >> 2] |= ((u & 255) ^ 128) << (8 * (g & 3));
        }
        ilt_lds_st8_untracked(&S.bh[t], h[0], h[1]);
        ilt_lds_st8_untracked(&S.bl[t], l[0], l[1]);
      }
      if constexpr (FMT == ILT_Q2_K) {
        u32 h[4] = {0, 0, 0, 0}, l[4] = {0, 0, 0, 0};
#pragma unroll
        for (int g = 0; g < 16; g++) {                       // the sum of group g's 16 quants + 2048, as planes
          const u32 u = (u32)(word_of(c_bs[g >> 2], g & 3) + 2048);
          h[g >> 2] |= (u >> 8) << (8 * (g & 3));
          l[g >> 2] |= ((u & 255) ^ 128) << (8 * (g & 3));
        }
        ilt_lds_st16_untracked(&q2_bh[t], (int)h[0], (int)h[1], (int)h[2], (int)h[3]);
        ilt_lds_st16_untracked(&q2_bl[t], (int)l[0], (int)l[1], (int)l[2], (int)l[3]);
      }
    }
    if (q4 == 0) {
      ilt_lds_st4_untracked(&S.wd[wrow], __builtin_bit_cast(u32, F::d_of(ra)));
      if constexpr (FMT == ILT_Q4_K) {
        ilt_lds_st4_untracked(&S.wdm[wrow], __builtin_bit_cast(u32, F::dmin_of(ra)));
        u32 m[2] = {0, 0}, ms = 0;
#pragma unroll
        for (int g = 0; g < 8; g++) { const u32 mn = F::min_of(ra, g); m[g >> 2] |= mn << (8 * (g & 3)); ms += mn; }
        ilt_lds_st8_untracked(&S.wmn[wrow], m[0], m[1]);
        ilt_lds_st4_untracked(&S.wms[wrow], ms);
      }
      if constexpr (FMT == ILT_Q2_K) {
        ilt_lds_st4_untracked(&S.wdm[wrow], __builtin_bit_cast(u32, F::dmin_of(ra)));
        u32 m[4], ms = 0;
#pragma unroll
        for (int i = 0; i < 4; i++) {                        // the minimums: the scale bytes' high nibbles
          m[i] = (word_of(ra.s, i) >> 4) & 0x0F0F0F0F;
          ms += (m[i] & 0xFF) + ((m[i] >> 8) & 0xFF) + ((m[i] >> 16) & 0xFF) + (m[i] >> 24);
        }
        ilt_lds_st16_untracked(&q2_wmn[wrow], (int)m[0], (int)m[1], (int)m[2], (int)m[3]);
        ilt_lds_st4_untracked(&S.wms[wrow], ms);
      }
    }
  };
  auto load_raw = [&](Raw& r, int hb) { F::load(r, rw, wrowoff, hb, q4); };       // half super-block hb of the thread's row
  auto issue_x = [&](int stage, int ks) {
#pragma unroll
    for (int i = 0; i < NI; i++) ilt_g2lds16(xbase + ks * KW + xoff[i], S.xs[stage] + (wave * NI + i) * 1024);
  };
  // the thread's 16 weights of step J of a super-block, out of the set that holds its half, into a pair of slabs
  auto dequant_to = [&](const Raw& r, int J, int slab) {
    int hi[4], lo[4];
    F::planes(r, J, q4, hi, lo, S);
    if constexpr (TWO) ilt_lds_st16_untracked(S.wh[slab] + wdst, hi[0], hi[1], hi[2], hi[3]);
    ilt_lds_st16_untracked(S.wl[slab] + wdst, lo[0], lo[1], lo[2], lo[3]);
  };

  v16f sum[NA][1];
  v16i_ ah[SPLIT ? 2 : 1][NA], al[SPLIT ? 2 : 1][NA];
  int xsum[NI] = {};                                         // IQ2_XXS, Q6_K: see the step
#pragma unroll
  for (int a = 0; a < NA; a++)
#pragma unroll
    for (int r = 0; r < 16; r++) sum[a][0][r] = 0.0f;

  // this wave's tokens and rows in the tile.  Grouped: waves 0-3 the first 64 tokens, 4-7 the second, one of each on
  // every SIMD, and a wave whose tokens the group does not have (a group of up to 64 rows) only makes planes.
  const int wt0 = GROUPED ? 64 * (wave >> 2) : 64 * (wave & 1), wr0 = GROUPED ? 32 * (wave & 3) : 32 * (wave >> 1);
  const bool work = !GROUPED || __builtin_amdgcn_readfirstlane(wt0) < ntok;
  const int l32 = lane & 31, lh = lane >> 5;
  u32 aoff[NA];                                              // fragment offsets of the step's first 32 columns (piece lh); the second 32 at ^ 32
#pragma unroll
  for (int a = 0; a < NA; a++) aoff[a] = slab_off(wt0 + 32 * a + l32, lh);
  const u32 boff = slab_off(wr0 + l32, lh);

  // Raw set A holds half 0 of a super-block and B half 1, two steps each; step ks multiplies
  // slab ks while it makes step ks+1's planes, so A is free after step 0 and loaded again (the
  // next block's) in step 1, B after step 2 and loaded in step 3.  The next block's token
  // constants are loaded in step 2 and stored in the next step 0.
  Raw rawa, rawb;
  load_raw(rawa, 0);
  load_consts(0);
  issue_x(0, 0);
  load_raw(rawb, 1);
  issue_x(1, 1);
  int st0 = 0, st1 = 1, st2 = 2;
  dequant_to(rawa, 0, 0);
  store_consts(rawa);

  auto step = [&](int ks, auto Jc) {
    constexpr int J = decltype(Jc)::value;                   // the step's place in its super-block
    // All loads but the previous step's have landed: this step's x slab has (sent two steps ago).
    constexpr int prev = NI + ((J == 0 || J == 2) ? WL : J == 3 ? XL : 0);
    asm volatile("s_waitcnt vmcnt(%0)" :: "n"(prev) : "memory");
    ilt_barrier_lds();                                       // no fence: later steps' loads stay in flight
    const int sb = ks >> 2;
    if (J == 0 && ks > 0) store_consts(rawa);                // (the first block's were stored before the loop)
    if (J == 1) load_raw(rawa, min(2 * sb + 2, 2 * nsb - 1));
    if (J == 2) load_consts(min(sb + 1, nsb - 1));
    if (J == 3) load_raw(rawb, min(2 * sb + 3, 2 * nsb - 1));
    issue_x(st2, min(ks + 2, nk - 1));
    __builtin_amdgcn_sched_barrier(0);
    const u8* xs = S.xs[st0];
    const u8* whs = S.wh[J & 1];
    const u8* wls = S.wl[J & 1];
    const v16i_ zero = {};
    if constexpr (XSLAB) {
      // the sums of the tokens' quants over the block (IQ2_XXS: over its even and its odd groups), from the slabs: thread t
      // adds piece t & 3 of token t / 4 (and of token t / 4 + 64 with four waves); pieces 0 and 1 are the step's even
      // group, 2 and 3 its odd one
#pragma unroll
      for (int i = 0; i < NI; i++) {
        const int4 xv = ilt_lds_ld16(xs + slab_off((t >> 2) + (THREADS / 4) * i, t & 3));
        int sp = __builtin_amdgcn_sdot4(xv.x, 0x01010101, 0, false);
        sp = __builtin_amdgcn_sdot4(xv.y, 0x01010101, sp, false);
        sp = __builtin_amdgcn_sdot4(xv.z, 0x01010101, sp, false);
        sp = __builtin_amdgcn_sdot4(xv.w, 0x01010101, sp, false);
        sp += __shfl_xor(sp, 1);
        if constexpr (!SPLIT) sp += __shfl_xor(sp, 2);
        xsum[i] = J == 0 ? sp : xsum[i] + sp;
      }
    }
#pragma unroll
    for (int kk = 0; kk < 2; kk++) {
      v4i_ af[NA] = {}, bh = {}, bl = {};
      if (work) {
#pragma unroll
        for (int a = 0; a < NA; a++) af[a] = *(const v4i_*)(xs + (aoff[a] ^ (32 * kk)));
        if constexpr (TWO) bh = *(const v4i_*)(whs + (boff ^ (32 * kk)));
        bl = *(const v4i_*)(wls + (boff ^ (32 * kk)));
      }
      if (kk == 0) {       // step ks+1's planes: J+1 = 1 from A, 2 and 3 from B, 4 = the next block's 0 from A (past the last step: planes nobody reads)
        if (J == 0) dequant_to(rawa, 1, 1);
        if (J == 1) dequant_to(rawb, 2, 0);
        if (J == 2) dequant_to(rawb, 3, 1);
        if (J == 3) dequant_to(rawa, 0, 0);
      }
      if (work) {
#pragma unroll
        for (int a = 0; a < NA; a++) {                       // a super-block's first products start its integer sums
          constexpr int ps = 0;
          const int pk = SPLIT ? kk : ps;
          const bool first = J == 0 && (SPLIT || kk == 0);
          if constexpr (TWO) ah[pk][a] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[a], bh, first ? zero : ah[pk][a], 0, 0, 0);
          al[pk][a] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[a], bl, first ? zero : al[pk][a], 0, 0, 0);
        }
      }
    }
    if constexpr (XSLAB) {
      if (J == 3) {        // the block's sums of quants, for everyone's terms below
#pragma unroll
        for (int i = 0; i < NI; i++) {
          if ((t & 3) == 0) ilt_lds_st4_untracked(&S.cx[(t >> 2) + (THREADS / 4) * i], (u32)(F::KCX * xsum[i]));
          if (SPLIT && (t & 3) == 2) ilt_lds_st4_untracked(&cxo[(t >> 2) + (THREADS / 4) * i], (u32)(F::KCX * xsum[i]));
        }
        ilt_barrier_lds();
      }
    }
    if (J == 3 && work) {  // the super-block is complete: its terms, as the CPU path adds them
      const int row = wr0 + l32;
      const float d = S.wd[row];
      if constexpr (FMT == ILT_Q4_K) {
        // im = sum over the groups of minimum * (sum of 32 quants) = 256*(mn.hi) + (mn.lo) - 3968*(sum of mn)
        const float dm = S.wdm[row];
        const int ms = 3968 * S.wms[row];
        const int2 mnb = S.wmn[row];
        const v4i_ bm = { lh ? 0 : mnb.x, lh ? 0 : mnb.y, 0, 0 };
#pragma unroll
        for (int a = 0; a < NA; a++) {
          const int2 th = S.bh[wt0 + 32 * a + l32], tl = S.bl[wt0 + 32 * a + l32];
          const v4i_ fh = { lh ? 0 : th.x, lh ? 0 : th.y, 0, 0 }, fl = { lh ? 0 : tl.x, lh ? 0 : tl.y, 0, 0 };
          const v16i_ mh = __builtin_amdgcn_mfma_i32_32x32x32_i8(fh, bm, zero, 0, 0, 0);
          const v16i_ ml = __builtin_amdgcn_mfma_i32_32x32x32_i8(fl, bm, zero, 0, 0, 0);
#pragma unroll
          for (int r = 0; r < 16; r++) {
            const int tk = wt0 + 32 * a + 8 * (r >> 2) + 4 * lh + (r & 3);
            const float yd = S.xd[tk];
            const int im = 256 * mh[r] + ml[r] - ms;
            const int isum = 256 * ah[0][a][r] + al[0][a][r] - S.cx[tk];
            sum[a][0][r] = sum[a][0][r] - (yd * dm) * (float)im;
            sum[a][0][r] = sum[a][0][r] + (yd * d) * (float)isum;
          }
        }
      } else if constexpr (FMT == ILT_IQ2_XXS) {
#pragma unroll
        for (int a = 0; a < NA; a++) {
#pragma unroll
          for (int r = 0; r < 16; r++) {
            const int tk = wt0 + 32 * a + 8 * (r >> 2) + 4 * lh + (r & 3);
            const float fa = (float)(256 * ah[0][a][r] + al[0][a][r] - S.cx[tk]) * 0.5f;
            const float fb = (float)(256 * ah[1][a][r] + al[1][a][r] - cxo[tk]) * 0.5f;
            sum[a][0][r] = sum[a][0][r] + (d * S.xd[tk]) * (fa + fb);
          }
        }
      } else if constexpr (FMT == ILT_Q2_K) {
        // im = sum over the sixteen groups of minimum * (sum of 16 quants) = 256*(mn.hi) + (mn.lo) - 1920*(sum of mn)
        const float dm = S.wdm[row];
        const int ms = 1920 * S.wms[row];
        const int4 mnb = q2_wmn[row];
        const v4i_ bm = { lh ? 0 : mnb.x, lh ? 0 : mnb.y, lh ? 0 : mnb.z, lh ? 0 : mnb.w };
#pragma unroll
        for (int a = 0; a < NA; a++) {
          const int4 th = q2_bh[wt0 + 32 * a + l32], tl = q2_bl[wt0 + 32 * a + l32];
          const v4i_ fh = { lh ? 0 : th.x, lh ? 0 : th.y, lh ? 0 : th.z, lh ? 0 : th.w };
          const v4i_ fl = { lh ? 0 : tl.x, lh ? 0 : tl.y, lh ? 0 : tl.z, lh ? 0 : tl.w };
          const v16i_ mh = __builtin_amdgcn_mfma_i32_32x32x32_i8(fh, bm, zero, 0, 0, 0);
          const v16i_ ml = __builtin_amdgcn_mfma_i32_32x32x32_i8(fl, bm, zero, 0, 0, 0);
#pragma unroll
          for (int r = 0; r < 16; r++) {
            const int tk = wt0 + 32 * a + 8 * (r >> 2) + 4 * lh + (r & 3);
            const float yd = S.xd[tk];
            const int im = 256 * mh[r] + ml[r] - ms;
            sum[a][0][r] = sum[a][0][r] + ((-yd) * dm) * (float)im;
            sum[a][0][r] = sum[a][0][r] + (yd * d) * (float)al[0][a][r];
          }
        }
      } else {
#pragma unroll
        for (int a = 0; a < NA; a++) {
#pragma unroll
          for (int r = 0; r < 16; r++) {
            const int tk = wt0 + 32 * a + 8 * (r >> 2) + 4 * lh + (r & 3);
            const int isum = 256 * ah[0][a][r] + al[0][a][r] - S.cx[tk];
            sum[a][0][r] = sum[a][0][r] + (d * S.xd[tk]) * (float)isum;
          }
        }
      }
    }
    const int s_ = st0; st0 = st1; st1 = st2; st2 = s_;
  };
  for (int ks = 0; ks < nk; ks += 4) {     // one super-block of 256 columns
    step(ks + 0, std::integral_constant<int, 0>{});
    step(ks + 1, std::integral_constant<int, 1>{});
    step(ks + 2, std::integral_constant<int, 2>{});
    step(ks + 3, std::integral_constant<int, 3>{});
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the tail's redundant loads: nothing may land in LDS after the workgroup ends

  if constexpr (FMT == ILT_IQ2_XXS) {
#pragma unroll
    for (int a = 0; a < NA; a++)
#pragma unroll
      for (int r = 0; r < 16; r++) sum[a][0][r] = 0.25f * sum[a][0][r];
  }
  store_tile<NA, 1>(sum, p, tok0, ntok, r0, wt0, wr0, l32, lh);
}

// ---- the exact Q8_0 product on the same pipeline -------------------------------------------------
// Q8_0 scales every block of 32 in float on either side: sum += float(isum) * (dw * dx), block
// after block (tensor.lisp:329-336), so there is nothing to fold into integers; but the quants
// are int8 as they lie in memory and a v_mfma_i32_32x32x32_i8 is exactly one block deep.  Both
// operands' slabs (64 columns = two blocks a step) come by direct loads, three steps in
// flight; the two scales a row and a token have per step go through registers a step ahead.
struct I8qSmem {
  __align__(16) u8 xs[3][128 * 64];
  __align__(16) u8 ws[3][128 * 64];
  float dw[2][2][128];                    // [step parity][block of the step][row]
  float dx[2][2][128];                    // [step parity][block of the step][token]
  u32 scan[256];
  int tile_z, tile_t0, tile_n;
};

__global__ __launch_bounds__(512, 2) void gemm_i8q_kernel(BfParams p) {
  constexpr int TM = 128, TN = 128, NA = 2, KW = 64;
  __shared__ I8qSmem S;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;

  long tok0; int ntok, rt; const u8* w = p.w;
  if (!pick_tile<TM, TN>(p, S, tok0, ntok, rt, w)) return;
  const int r0 = rt * TM;
  const int nk = p.cols / KW, nb = p.cols / 32;

  // piece t of a slab, of the tokens' and of the rows' quants
  const int prow = t >> 2, pk = (t & 3) ^ (int)slab_swz(prow);
  const u8* xbase = (const u8*)ilt_uniform_ptr((const i8*)p.x + tok0 * (long)p.cols);
  const u8* wbase = (const u8*)ilt_uniform_ptr(w + (long)r0 * p.cols);
  const u32 xoff = (u32)min(prow, ntok - 1) * (u32)p.cols + 16 * pk;
  const u32 woff = (u32)min(prow, p.rows - 1 - r0) * (u32)p.cols + 16 * pk;
  // a scale a thread and step: threads 0..255 a row's (row t/2, block t%2 of the step), 256..511 a token's
  const int sidx = (t & 255) >> 1, sblk = t & 1;
  const bool srow = t < 256;
  const u16* dwp = p.wdq + (long)min(r0 + sidx, p.rows - 1) * nb + sblk;
  const float* dxp = p.xd + (tok0 + min(sidx, ntok - 1)) * nb + sblk;
  auto load_scale = [&](int ks) { return srow ? ilt_h2f(dwp[2 * ks]) : dxp[2 * ks]; };
  auto store_scale = [&](float v, int ks) {
    float* dst = srow ? &S.dw[ks & 1][sblk][sidx] : &S.dx[ks & 1][sblk][sidx];
    asm volatile("ds_write_b32 %0, %1" :: "v"((u32)(uintptr_t)(ILT_LDS void*)dst), "v"(v) : "memory");
  };
  auto issue = [&](int stage, int ks) {
    ilt_g2lds16(xbase + ks * KW + xoff, S.xs[stage] + wave * 1024);
    ilt_g2lds16(wbase + ks * KW + woff, S.ws[stage] + wave * 1024);
  };

  v16f sum[NA][1];
#pragma unroll
  for (int a = 0; a < NA; a++)
#pragma unroll
    for (int r = 0; r < 16; r++) sum[a][0][r] = 0.0f;
  const int wt0 = 64 * (wave & 1), wr0 = 32 * (wave >> 1);  // this wave's tokens and rows in the tile
  const int l32 = lane & 31, lh = lane >> 5;
  u32 aoff[NA];
#pragma unroll
  for (int a = 0; a < NA; a++) aoff[a] = slab_off(wt0 + 32 * a + l32, lh);
  const u32 boff = slab_off(wr0 + l32, lh);

  // Step ks waits for its slabs (sent two steps ago), stores the scales of step ks+1 (loaded a step
  // ago), loads those of step ks+2 and sends for step ks+2's slabs.
  // (in this order: step 0 waits for all but the last three loads)
  store_scale(load_scale(0), 0);
  issue(0, 0);
  float sc_next = load_scale(min(1, nk - 1));
  issue(1, min(1, nk - 1));
  int st0 = 0, st1 = 1, st2 = 2;
  const v16i_ zero = {};
  for (int ks = 0; ks < nk; ks++) {
    asm volatile("s_waitcnt vmcnt(3)" ::: "memory");         // all loads but the previous step's three (its scale and two slabs)
    ilt_barrier_lds();                                       // no fence: later steps' loads stay in flight
    store_scale(sc_next, ks + 1);
    sc_next = load_scale(min(ks + 2, nk - 1));
    issue(st2, min(ks + 2, nk - 1));
    __builtin_amdgcn_sched_barrier(0);
    const u8* xs = S.xs[st0];
    const u8* ws = S.ws[st0];
#pragma unroll
    for (int kk = 0; kk < 2; kk++) {                         // block 2*ks + kk
      const v4i_ bw = *(const v4i_*)(ws + (boff ^ (32 * kk)));
      const float dw = S.dw[ks & 1][kk][wr0 + l32];
#pragma unroll
      for (int a = 0; a < NA; a++) {
        const v4i_ af = *(const v4i_*)(xs + (aoff[a] ^ (32 * kk)));
        const v16i_ d = __builtin_amdgcn_mfma_i32_32x32x32_i8(af, bw, zero, 0, 0, 0);
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const float dx = S.dx[ks & 1][kk][wt0 + 32 * a + 8 * (r >> 2) + 4 * lh + (r & 3)];
          sum[a][0][r] = sum[a][0][r] + (float)d[r] * (dw * dx);
        }
      }
    }
    const int s_ = st0; st0 = st1; st1 = st2; st2 = s_;
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the tail's redundant loads: nothing may land in LDS after the workgroup ends
  store_tile<NA, 1>(sum, p, tok0, ntok, r0, wt0, wr0, l32, lh);
}

// ---- the exact product in two passes: the planes once, then a loop without dequantization -------
// As for bf16: with thousands of tokens (or a matrix multiplied again and again) the two planes
// of a Q6_K matrix are worth writing out once -- a byte a weight each, in slabs of 128 rows x 64
// columns (the row count padded to a multiple of 128), and d per row and super-block as floats -- so that the product's loop holds only direct loads of
// three slabs, fragment reads, MFMAs and the combine per super-block.  The same integers, the
// same float expression per block: the same bits as gemm_i8p_kernel and the CPU path.
template <int FMT>
__global__ __launch_bounds__(256) void planes_i8_kernel(const u8* __restrict__ w, long long row_bytes, int rows, int cols,
                                                        u8* __restrict__ wh, u8* __restrict__ wl, float* __restrict__ wdf) {
  typedef I8p<FMT> F;
  const int nsb = cols / 256;
  const long long u = (long long)blockIdx.x * 256 + threadIdx.x;       // 16 weights: unit q4 of step J of a super-block of a row
  if (u >= (long long)rows * nsb * 16) return;
  const int q4 = (int)(u & 3), J = (int)((u >> 2) & 3);
  const long long sr = u >> 4;
  const int sb = (int)(sr % nsb);
  const long long row = sr / nsb;
  const __amdgpu_buffer_rsrc_t rw = ilt_rsrc(ilt_uniform_ptr(w), (u32)min((long long)rows * row_bytes, 0xFFFFFFF0LL));
  typename F::Raw r;
  F::load(r, rw, (u32)(row * row_bytes), 2 * sb + (J >> 1), q4);
  int hi[4], lo[4];
  const int dummy = 0;
  switch (J) {            // (the step is a constant inside planes)
    case 0: F::planes(r, 0, q4, hi, lo, dummy); break;
    case 1: F::planes(r, 1, q4, hi, lo, dummy); break;
    case 2: F::planes(r, 2, q4, hi, lo, dummy); break;
    default: F::planes(r, 3, q4, hi, lo, dummy); break;
  }
  // slab order: the 64 columns of a step for 128 consecutive rows are 8 KB in one piece (row r of the group at 64*r),
  // the groups' slabs for step 0, 1, ... one after another, so that the product's direct loads read whole lines
  const long long o = ((row >> 7) * (cols / 64) + sb * 4 + J) * 8192 + (row & 127) * 64 + 16 * q4;
  *(int4*)(wh + o) = make_int4(hi[0], hi[1], hi[2], hi[3]);
  *(int4*)(wl + o) = make_int4(lo[0], lo[1], lo[2], lo[3]);
  if (J == 0 && q4 == 0) wdf[row * nsb + sb] = F::d_of(r);
}

// NB row patches a wave: 1 = eight waves of 32 rows x 64 tokens (one workgroup a CU, slabs four steps ahead).
// (2 = four waves of 64 x 64, two workgroups a CU, reads a quarter less from LDS per MFMA but does not fit the
// registers: 27 spilled, 486 against 590 TFLOP/s.)
template <int NB> struct I8ppSmem {
  static constexpr int RING = NB == 1 ? 5 : 3;
  __align__(16) u8 xs[RING][128 * 64];
  __align__(16) u8 wh[RING][128 * 64];
  __align__(16) u8 wl[RING][128 * 64];
  float wd[128], xd[128];                 // of the super-block: d of the rows, the tokens' scales
  int cx[128];                            //   and 4000 * the sum of their quants
  u32 scan[256];
  int tile_z, tile_t0, tile_n, pad;
};

template <int NB>
__global__ __launch_bounds__(512 / NB, 2) void gemm_i8pp_kernel(BfParams p) {
  constexpr int TM = 128, TN = 128, NA = 2, KW = 64;
  constexpr int THREADS = 512 / NB, NWAVES = THREADS / 64, NP = 512 / THREADS;      // NP: pieces of a slab a thread sends for
  constexpr int NL = 3 * NP, XL = 2;                         // loads a step (three slabs), of a super-block's constants
  extern __shared__ __align__(16) u8 i8pp_lds[];
  I8ppSmem<NB>& S = *(I8ppSmem<NB>*)i8pp_lds;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;

  long tok0; int ntok, rt; const u8* w = p.w;
  if (!pick_tile<TM, TN>(p, S, tok0, ntok, rt, w)) return;
  const int r0 = rt * TM;
  const int nk = p.cols / KW, nsb = p.cols / 256;

  const u8* xbase = (const u8*)ilt_uniform_ptr((const i8*)p.x + tok0 * (long)p.cols);
  const u8* hbase = (const u8*)ilt_uniform_ptr(p.w + (long)rt * nk * 8192);       // the row tile's slabs, one a step
  const u8* lbase = (const u8*)ilt_uniform_ptr(p.wlo + (long)rt * nk * 8192);
  u32 xoff[NP], woff[NP];                                    // piece i * THREADS + t of a slab
#pragma unroll
  for (int i = 0; i < NP; i++) {
    const int P_ = i * THREADS + t, prow = P_ >> 2, pk = (P_ & 3) ^ (int)slab_swz(prow);
    xoff[i] = (u32)min(prow, ntok - 1) * (u32)p.cols + 16 * pk;
    woff[i] = (u32)prow * 64 + 16 * pk;
  }
  auto issue = [&](int stage, int ks) {
#pragma unroll
    for (int i = 0; i < NP; i++) {
      ilt_g2lds16(xbase + ks * KW + xoff[i], S.xs[stage] + (i * NWAVES + wave) * 1024);
      ilt_g2lds16(hbase + (long)ks * 8192 + woff[i], S.wh[stage] + (i * NWAVES + wave) * 1024);
      ilt_g2lds16(lbase + (long)ks * 8192 + woff[i], S.wl[stage] + (i * NWAVES + wave) * 1024);
    }
  };
  // a super-block's constants, by thread t & 127 (every wave loads, so that all count the same loads)
  const long ctok = tok0 + min(t & 127, ntok - 1);
  // (the sums of the tokens' quants over a super-block are taken from the slabs in LDS, see the step: the
  // activations' sums of 16 would be 16 more registers held across two steps)
  const float* xdp = p.xd + ctok * nsb;
  const float* wdp = p.wdf + (long)min(r0 + (t & 127), p.rows - 1) * nsb;
  float c_yd, c_d;
  auto load_consts = [&](int sb) {
    c_yd = xdp[sb];
    c_d = wdp[sb];
  };
  auto store_consts = [&]() {                                // after a barrier that ends the last block's reads
    if (t < 128) {
      ilt_lds_st4_untracked(&S.xd[t], __builtin_bit_cast(u32, c_yd));
      ilt_lds_st4_untracked(&S.wd[t], __builtin_bit_cast(u32, c_d));
    }
  };
  int xsum[NP] = {};

  v16f sum[NA][NB];
  v16i_ ah[NA][NB], al[NA][NB];
#pragma unroll
  for (int a = 0; a < NA; a++)
#pragma unroll
    for (int b = 0; b < NB; b++)
#pragma unroll
      for (int r = 0; r < 16; r++) sum[a][b][r] = 0.0f;
  const int wt0 = 64 * (wave & 1), wr0 = 32 * NB * (wave >> 1);       // this wave's tokens and rows in the tile
  const int l32 = lane & 31, lh = lane >> 5;
  u32 aoff[NA], boff[NB];
#pragma unroll
  for (int a = 0; a < NA; a++) aoff[a] = slab_off(wt0 + 32 * a + l32, lh);
#pragma unroll
  for (int b = 0; b < NB; b++) boff[b] = slab_off(wr0 + 32 * b + l32, lh);

  constexpr int D = I8ppSmem<NB>::RING;
  load_consts(0);
  store_consts();
#pragma unroll
  for (int i = 0; i < D - 1; i++) issue(i, min(i, nk - 1));
  int cur = 0;                                               // the step's slabs' place in the rings
  const v16i_ zero = {};
  auto step = [&](int ks, auto Jc) {
    constexpr int J = decltype(Jc)::value;                   // the step's place in its super-block
    // This step's slabs were sent D-1 steps ago: all loads but those of the D-2 steps since have landed
    // (the constants' loads of step 2 of a super-block among them, if that step is one of those).
    constexpr bool consts_since = D == 5 ? J != 2 : J == 3;
    constexpr int prev = (D - 2) * NL + (consts_since ? XL : 0);
    if (ks < D - 1) asm volatile("s_waitcnt vmcnt(%0)" :: "n"((D - 2) * NL) : "memory");     // (no constants' loads before the first super-block's slabs)
    else asm volatile("s_waitcnt vmcnt(%0)" :: "n"(prev) : "memory");
    ilt_barrier_lds();                                       // no fence: later steps' loads stay in flight
    const int sb = ks >> 2;
    if (J == 0 && ks > 0) store_consts();                    // (the first block's were stored before the loop)
    if (J == 2) load_consts(min(sb + 1, nsb - 1));
    issue(cur == 0 ? D - 1 : cur - 1, min(ks + D - 1, nk - 1));         // into the slabs the step before read
    __builtin_amdgcn_sched_barrier(0);
    const u8* xs = S.xs[cur];
    const u8* whs = S.wh[cur];
    const u8* wls = S.wl[cur];
#pragma unroll
    for (int i = 0; i < NP; i++) {                           // the sum of the step's 64 quants of token (i * THREADS + t) / 4, in its four lanes
      const int4 xv = ilt_lds_ld16(xs + slab_off((i * THREADS + t) >> 2, t & 3));
      int sp = __builtin_amdgcn_sdot4(xv.x, 0x01010101, 0, false);
      sp = __builtin_amdgcn_sdot4(xv.y, 0x01010101, sp, false);
      sp = __builtin_amdgcn_sdot4(xv.z, 0x01010101, sp, false);
      sp = __builtin_amdgcn_sdot4(xv.w, 0x01010101, sp, false);
      sp += __shfl_xor(sp, 1);
      sp += __shfl_xor(sp, 2);
      xsum[i] = J == 0 ? sp : xsum[i] + sp;
    }
#pragma unroll
    for (int kk = 0; kk < 2; kk++) {
      v4i_ af[NA], bh[NB], bl[NB];
#pragma unroll
      for (int a = 0; a < NA; a++) af[a] = *(const v4i_*)(xs + (aoff[a] ^ (32 * kk)));
#pragma unroll
      for (int b = 0; b < NB; b++) { bh[b] = *(const v4i_*)(whs + (boff[b] ^ (32 * kk))); bl[b] = *(const v4i_*)(wls + (boff[b] ^ (32 * kk))); }
#pragma unroll
      for (int a = 0; a < NA; a++)
#pragma unroll
        for (int b = 0; b < NB; b++) {                       // a super-block's first products start its integer sums
          ah[a][b] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[a], bh[b], (J == 0 && kk == 0) ? zero : ah[a][b], 0, 0, 0);
          al[a][b] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[a], bl[b], (J == 0 && kk == 0) ? zero : al[a][b], 0, 0, 0);
        }
    }
    if (J == 3) {          // the super-block is complete: sum += (d * yd) * float(isum), as the CPU path adds it
#pragma unroll
      for (int i = 0; i < NP; i++)
        if ((t & 3) == 0) ilt_lds_st4_untracked(&S.cx[(i * THREADS + t) >> 2], (u32)(4000 * xsum[i]));
      ilt_barrier_lds();
      float d[NB];
#pragma unroll
      for (int b = 0; b < NB; b++) d[b] = S.wd[wr0 + 32 * b + l32];
#pragma unroll
      for (int a = 0; a < NA; a++)
#pragma unroll
        for (int r4 = 0; r4 < 4; r4++) {                     // four consecutive tokens' constants at a time
          const int tk = wt0 + 32 * a + 8 * r4 + 4 * lh;
          const float4 yd = *(const float4*)&S.xd[tk];
          const int4 cx = *(const int4*)&S.cx[tk];
          const float ydv[4] = {yd.x, yd.y, yd.z, yd.w};
          const int cxv[4] = {cx.x, cx.y, cx.z, cx.w};
#pragma unroll
          for (int k = 0; k < 4; k++)
#pragma unroll
            for (int b = 0; b < NB; b++) {
              const int r = 4 * r4 + k;
              const int isum = 256 * ah[a][b][r] + al[a][b][r] - cxv[k];
              sum[a][b][r] = sum[a][b][r] + (d[b] * ydv[k]) * (float)isum;
            }
          __builtin_amdgcn_sched_barrier(0);
        }
    }
    cur = cur == D - 1 ? 0 : cur + 1;
  };
  for (int ks = 0; ks < nk; ks += 4) {
    step(ks + 0, std::integral_constant<int, 0>{});
    step(ks + 1, std::integral_constant<int, 1>{});
    step(ks + 2, std::integral_constant<int, 2>{});
    step(ks + 3, std::integral_constant<int, 3>{});
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the tail's redundant loads: nothing may land in LDS after the workgroup ends
  store_tile<NA, NB>(sum, p, tok0, ntok, r0, wt0, wr0, l32, lh);
}

// ---- the two-pass product: W as plain bf16 ------------------------------------------------------
// With thousands of tokens the in-loop dequantization above is repeated for every tile of 256
// tokens and its VALU work competes with the MFMAs for issue slots.  With HBM to spare the
// matrix can instead be dequantized once into a bf16 copy (kept for later products, or made
// per product) and multiplied by a kernel whose loop holds nothing but direct loads to LDS,
// fragment reads and MFMAs.

//
// Both operands of that kernel are stored in slabs: the 32 columns of a step for 128
// consecutive rows (or tokens) are 8 KB in one piece, row r of the group at 64*r, the groups'
// slabs for step 0, 1, ... one after another.  A step's direct loads then read whole 128-byte
// lines of a few DRAM pages instead of 64 bytes from each of 256 rows' pages.  The row count is
// padded to a multiple of 256 (the padding rows hold zeros).
constexpr int SLAB_ROWS = 128, SLAB_BYTES = SLAB_ROWS * KS * 2;
__device__ __forceinline__ long long slab_addr(long long row, int ks, int nk) {     // of the row's 64 bytes of step ks
  return ((row / SLAB_ROWS) * nk + ks) * SLAB_BYTES + (row % SLAB_ROWS) * (KS * 2);
}

// A workgroup: one super-block (256 columns, eight slabs) of a group of 128 rows, so that every
// line of the quantized rows it touches is used up by it; thread (row, e) dequantizes the 2 x 4 x 16
// weights that kernel thread (row, e) dequantizes there and writes 32 bytes into each slab.
// Every eighth workgroup id is one XCD: an XCD takes a run of consecutive super-blocks, whose
// rows' shared lines then meet in its L2.
template <int FMT>
__global__ __launch_bounds__(256) void dequant_bf16_kernel(const u8* __restrict__ w, long long row_bytes, int rows, int cols, u8* __restrict__ out,
                                                           int total) {
  __shared__ Iq2Tables iq2;
  if (FMT == ILT_IQ2_XXS) { iq2_tables_fill(iq2, threadIdx.x); __syncthreads(); }
  const int nsb = cols / 256, nk = cols / KS;
  const int per = (total + 7) / 8, unit = (blockIdx.x & 7) * per + (blockIdx.x >> 3);
  if ((int)(blockIdx.x >> 3) >= per || unit >= total) return;
  const int e = threadIdx.x & 1, rl = threadIdx.x >> 1;
  const int sb = unit % nsb;
  const long long row = (long long)(unit / nsb) * SLAB_ROWS + rl;
  const bool live = row < rows;
  WRaw<FMT> raw[2];
  if (live) {
    // one descriptor for the whole matrix (less than 4 GiB, checked by the host), the row in the lane's offset
    const __amdgpu_buffer_rsrc_t rw = ilt_rsrc(w, (u32)min((long long)rows * row_bytes, 0xFFFFFFF0LL));
    const u32 rowoff = (u32)(row * row_bytes);
    load_w<FMT>(raw[0], rw, rowoff, 2 * sb, e);
    load_w<FMT>(raw[1], rw, rowoff, 2 * sb + 1, e);
  }
#pragma unroll
  for (int c = 0; c < 2; c++) {
#pragma unroll
    for (int j = 0; j < 4; j++) {
      u32 pk[8] = {0, 0, 0, 0, 0, 0, 0, 0};
      if (live) dequant16_pk<FMT>(raw[c], j, c, e, &iq2, pk);
      u8* dst = out + slab_addr(row, 8 * sb + 4 * c + j, nk) + 32 * e;
      *(int4*)dst = make_int4((int)pk[0], (int)pk[1], (int)pk[2], (int)pk[3]);
      *(int4*)(dst + 16) = make_int4((int)pk[4], (int)pk[5], (int)pk[6], (int)pk[7]);
    }
  }
}

// Floats (n tokens of cols) to bf16 in slabs; npad tokens are written, zeros past n.  Thread:
// 8 columns (16 bytes) of a token; a wave: the 64 bytes of 16 consecutive tokens.
__global__ __launch_bounds__(256) void cvt_bf16_slabs_kernel(const float* __restrict__ x, u8* __restrict__ out, int n, long long npad, int cols) {
  const int nk = cols / KS;
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;      // (group, ks, token in group, piece)
  const int piece = (int)(i & 3), tl = (int)((i >> 2) % SLAB_ROWS);
  const long long gk = i / (4 * SLAB_ROWS);
  const int ks = (int)(gk % nk);
  const long long tok = (gk / nk) * SLAB_ROWS + tl;
  if (tok >= npad) return;
  int4 v = make_int4(0, 0, 0, 0);
  if (tok < n) {
    const float4* src = (const float4*)(x + tok * cols + ks * KS + 8 * piece);
    const float4 a = src[0], b = src[1];
    v = make_int4(pack_bf16(a.x, a.y), pack_bf16(a.z, a.w), pack_bf16(b.x, b.y), pack_bf16(b.z, b.w));
  }
  *(int4*)(out + slab_addr(tok, ks, nk) + 16 * piece) = v;
}

template <int T> struct PlainSmem {
  __align__(16) u8 xs[4][T * KS * 2];
  __align__(16) u8 ws[4][T * KS * 2];
};

// T rows x T tokens a workgroup of four waves.  T = 256: a wave alone on its SIMD with 128 x 128
// results in 256 accumulator registers; T = 128 (two workgroups a CU) for the rows left over
// when the 256-tiles do not fill a whole number of rounds over the CUs.  Both operands' 32-column slabs go from global memory straight into
// LDS, three steps ahead, each into a ring of four slabs; a step's fragments are read half a
// step ahead of their MFMAs.  One barrier a step.  p.w, p.x: the operands in slabs.
template <int T>
__global__ __launch_bounds__(256, (T == 256 ? 1 : 2)) void gemm_bf16_plain_kernel(BfParams p) {
  __shared__ PlainSmem<T> S;
  constexpr int NI = T / 64, NP = T / 64;      // direct loads per wave, step and operand; 32 x 32 patches each way per wave
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int NR = (p.rows + T - 1) / T, NT = (p.ntok + T - 1) / T;
  const int total = NT * NR, per = (total + 7) / 8;
  const int L = blockIdx.x, j = L >> 3;
  const int s = (L & 7) * per + j;
  if (j >= per || s >= total) return;
  const int rg = s / (GR * NT), rem = s - rg * GR * NT, nr = min(GR, NR - rg * GR);
  const int tt = rem / nr, rt = rg * GR + (rem - tt * nr);
  const long tok0 = (long)tt * T;
  const int ntok = min(T, p.ntok - (int)tok0), r0 = rt * T;
  const int nk = p.cols / KS;

  const u8* xbase = (const u8*)ilt_uniform_ptr((const u8*)p.x + slab_addr(tok0, 0, nk));
  const u8* wbase = (const u8*)ilt_uniform_ptr(p.w + slab_addr(r0, 0, nk));
  u32 off[NI];                                 // the same place in x's and W's slabs
#pragma unroll
  for (int i = 0; i < NI; i++) {
    const int P = (wave * NI + i) * 64 + lane, r = P >> 2, kp = (P & 3) ^ (int)slab_swz(r);
    off[i] = (u32)slab_addr(r, 0, nk) + 16 * kp;
  }
  v16f acc[NP][NP];
#pragma unroll
  for (int a = 0; a < NP; a++)
#pragma unroll
    for (int b = 0; b < NP; b++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[a][b][r] = 0.0f;
  const int wt0 = (T / 2) * (wave & 1), wr0 = (T / 2) * (wave >> 1);
  const int l32 = lane & 31, lh = lane >> 5;
  u32 aoff[NP], boff[NP];
#pragma unroll
  for (int a = 0; a < NP; a++) { aoff[a] = slab_off(wt0 + 32 * a + l32, lh); boff[a] = slab_off(wr0 + 32 * a + l32, lh); }

  auto issue = [&](int stage, int ks) {
#pragma unroll
    for (int i = 0; i < NI; i++) ilt_g2lds16(xbase + ks * SLAB_BYTES + off[i], S.xs[stage] + (wave * NI + i) * 1024);
#pragma unroll
    for (int i = 0; i < NI; i++) ilt_g2lds16(wbase + ks * SLAB_BYTES + off[i], S.ws[stage] + (wave * NI + i) * 1024);
  };
  issue(0, 0);
  issue(1, min(1, nk - 1));
  issue(2, min(2, nk - 1));
  asm volatile("s_waitcnt vmcnt(%0)" :: "n"(2 * NI) : "memory");     // slabs 0 and 1: step 0 reads both
  ilt_barrier_lds();
  v8bf fa[NP], fb[NP], ga[NP], gb[NP];
#pragma unroll
  for (int a = 0; a < NP; a++) { fa[a] = *(const v8bf*)(S.xs[0] + aoff[a]); fb[a] = *(const v8bf*)(S.ws[0] + boff[a]); }

  // ST: the step's slab, a constant after unrolling
  auto step = [&](int ks, auto Sc) {
    constexpr int ST = decltype(Sc)::value;
    issue((ST + 3) & 3, min(ks + 3, nk - 1));
    __builtin_amdgcn_sched_barrier(0);
    auto half = [&](const u8* xs_next, const u8* ws_next, u32 flip, v8bf* ua, v8bf* ub, v8bf* na, v8bf* nb) {
#pragma unroll
      for (int q = 0; q < NP; q++) {
        na[q] = *(const v8bf*)(xs_next + (aoff[q] ^ flip));
        nb[q] = *(const v8bf*)(ws_next + (boff[q] ^ flip));
#pragma unroll
        for (int b = 0; b < NP; b++) acc[q][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ua[q], ub[b], acc[q][b], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    half(S.xs[ST], S.ws[ST], 32, fa, fb, ga, gb);                          // columns 0..15; reads this step's 16..31
    half(S.xs[(ST + 1) & 3], S.ws[(ST + 1) & 3], 0, ga, gb, fa, fb);        // columns 16..31; reads the next step's 0..15
    // only this step's loads may still be on their way: slab ks+2, which the next step reads
    // from its second half on, has landed; the barrier publishes it and frees slab ks
    asm volatile("s_waitcnt vmcnt(%0)" :: "n"(2 * NI) : "memory");
    ilt_barrier_lds();
  };
  for (int ks = 0; ks < nk; ks += 4) {
    step(ks + 0, std::integral_constant<int, 0>{});
    step(ks + 1, std::integral_constant<int, 1>{});
    step(ks + 2, std::integral_constant<int, 2>{});
    step(ks + 3, std::integral_constant<int, 3>{});
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

  store_tile<NP, NP>(acc, p, tok0, ntok, r0, wt0, wr0, l32, lh);
}

__global__ __launch_bounds__(256) void cvt_bf16_kernel(const float* __restrict__ x, u16* __restrict__ xb, long long n8) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= n8) return;
  const float4 a = ((const float4*)x)[2 * i], b = ((const float4*)x)[2 * i + 1];
  ((int4*)xb)[i] = make_int4(pack_bf16(a.x, a.y), pack_bf16(a.z, a.w), pack_bf16(b.x, b.y), pack_bf16(b.z, b.w));
}

// Q8_K activations (quantize-q8k!'s quants and block scales) as bf16: d * q, the value the CPU path's row dots
// multiply the weights with, rounded to bf16 -- 8 quants a thread.  SLABS: into cvt_bf16_slabs' layout
// (npad tokens written, zeros past n).
template <bool SLABS>
__global__ __launch_bounds__(256) void q8k_bf16_kernel(const i8* __restrict__ xq, const float* __restrict__ xd, u8* __restrict__ out, int n,
                                                       long long npad, int cols) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;      // rows: (token, 8 columns); slabs: (group, ks, token in group, piece)
  long long tok; int c0; u8* dst;
  if (SLABS) {
    const int nk = cols / KS;
    const int piece = (int)(i & 3), tl = (int)((i >> 2) % SLAB_ROWS);
    const long long gk = i / (4 * SLAB_ROWS);
    const int ks = (int)(gk % nk);
    tok = (gk / nk) * SLAB_ROWS + tl; c0 = ks * KS + 8 * piece;
    if (tok >= npad) return;
    dst = out + slab_addr(tok, ks, nk) + 16 * piece;
  } else {
    const int per = cols / 8;
    tok = i / per; c0 = (int)(i % per) * 8;
    if (tok >= n) return;
    dst = out + (tok * cols + c0) * 2;
  }
  int4 v = make_int4(0, 0, 0, 0);
  if (tok < n) {
    const int2 q = *(const int2*)(xq + tok * cols + c0);
    const float d = xd[(tok * cols + c0) >> 8];
    float f[8];
#pragma unroll
    for (int k = 0; k < 4; k++) {
      f[k] = d * (float)(i8)((u32)q.x >> (8 * k));
      f[4 + k] = d * (float)(i8)((u32)q.y >> (8 * k));
    }
    v = make_int4(pack_bf16(f[0], f[1]), pack_bf16(f[2], f[3]), pack_bf16(f[4], f[5]), pack_bf16(f[6], f[7]));
  }
  *(int4*)dst = v;
}

// Room for the split tiles' parts: a buffer per (device, stream) -- launches on two streams may overlap, and each needs
// its parts to itself -- grown when a launch needs more; sixteen of them at most.  A launch that gets no room (a stream
// under capture, the table full, no memory) goes unsplit.
struct PartRoom { int dev; hipStream_t st; float* p; size_t bytes; };
std::mutex g_part_mu;
PartRoom g_part[16] = {};
int g_nparts = 0;
float* part_room(size_t bytes, hipStream_t st) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return nullptr;
  // (a captured launch would keep the room's address while a later launch may grow the room and free it: under capture
  // nothing is split)
  hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(st, &cs) != hipSuccess || cs != hipStreamCaptureStatusNone) { (void)hipGetLastError(); return nullptr; }
  std::lock_guard<std::mutex> lock(g_part_mu);
  PartRoom* r = nullptr;
  for (int i = 0; i < g_nparts; i++) if (g_part[i].dev == dev && g_part[i].st == st) r = &g_part[i];
  if (r && r->bytes >= bytes) return r->p;
  if (!r) {
    if (g_nparts == 16) return nullptr;
    r = &g_part[g_nparts++];
    *r = {dev, st, nullptr, 0};
  }
  if (r->p) {
    if (hipStreamSynchronize(st) != hipSuccess) return nullptr;        // this stream's earlier launches may still use the old room
    (void)hipFree(r->p);
    r->p = nullptr; r->bytes = 0;
  }
  const size_t want = bytes + bytes / 4;
  if (hipMalloc((void**)&r->p, want) != hipSuccess) { (void)hipGetLastError(); r->p = nullptr; return nullptr; }
  r->bytes = want;
  return r->p;
}

// The tiles past the last whole round over the 256 CUs would take a round of their own (272 tiles: two rounds, the second
// one sixteenth full).  They are split instead: KSPLIT workgroups a tile, each a run of the columns' super-blocks, dealt
// over all CUs beside the whole rounds' tiles, and a small kernel adds a tile's parts.  Chosen where the model -- rounds
// of whole tiles plus rounds of parts (split_rounds) -- says it saves a twentieth or more.
// ILT_BF16_SPLITK=0: never (tests).
// (a part: its share of the columns and what every workgroup spends besides its columns, about two super-blocks' worth;
// the parts' round as such -- they start when the whole tiles' last round ends, write their sums, and the adding kernel
// reads them back -- about 0.3 of a tile's time, measured on 17408 x 5120 at 512 to 4096 tokens)
inline double split_rounds(long long full, long long lo, int k, int nsb) {
  return (double)(full / 256) + (double)((lo * k + 255) / 256) * (1.0 / k + 2.0 / nsb) + 0.3;
}
inline int choose_ksplit(long long total, int nsb, long long& split_from) {
  const char* force = getenv("ILT_BF16_SPLITK");
  if (force && atoi(force) == 0) return 0;
  const long long full = total / 256 * 256, lo = total - full;
  if (lo == 0 || nsb < 2) return 0;
  const double plain = (double)((total + 255) / 256);
  double best = plain; int bk = 0;
  for (int k = 2; k <= nsb && k <= 32; k++) {
    const double c = split_rounds(full, lo, k, nsb);
    if (c < best - 1e-9) { best = c; bk = k; }
  }
  if (bk == 0 || best > plain * 0.95) return 0;
  split_from = full;
  return bk;
}

template <int FMT, int TM, int TN, int NB>
hipError_t launch_bf16(const BfParams& p0, long long token_tiles, hipStream_t st) {
  BfParams p = p0;
  const long long total = token_tiles * ((p.rows + TM - 1) / TM), per = (total + 7) / 8;
  if (per * 8 > 0x7FFFFFFFLL) return hipErrorInvalidValue;
  long long split_from = 0;
  const int k = p.ptrs ? 0 : choose_ksplit(total, p.cols / 256, split_from);
  if (k > 1) {
    const long long lo = total - split_from;
    float* room = (size_t)lo * k * TM * TN * 4 <= ((size_t)256 << 20) ? part_room((size_t)lo * k * TM * TN * 4, st) : nullptr;
    if (room) {
      p.ksplit = k; p.split_from = (int)split_from; p.part = room;
      hipLaunchKernelGGL((gemm_bf16_kernel<FMT, TM, TN, NB>), dim3((unsigned)(split_from + lo * k)), dim3(bf16_threads<TM, NB>()), 0, st, p);
      hipLaunchKernelGGL((bf16_split_sum_kernel<TM, TN>), dim3(TM * TN / 1024, (unsigned)lo), dim3(256), 0, st, p);
      return hipGetLastError();
    }
  }
  hipLaunchKernelGGL((gemm_bf16_kernel<FMT, TM, TN, NB>), dim3((unsigned)(per * 8)), dim3(bf16_threads<TM, NB>()), 0, st, p);
  return hipGetLastError();
}

template <int TM, int TN, int NB>
hipError_t dispatch_bf16(int fmt, const BfParams& p, long long token_tiles, hipStream_t st) {
  switch (fmt) {
    case ILT_Q4_K: return launch_bf16<ILT_Q4_K, TM, TN, NB>(p, token_tiles, st);
    case ILT_Q6_K: return launch_bf16<ILT_Q6_K, TM, TN, NB>(p, token_tiles, st);
    case ILT_Q2_K: return launch_bf16<ILT_Q2_K, TM, TN, NB>(p, token_tiles, st);
    case ILT_IQ2_XXS: return launch_bf16<ILT_IQ2_XXS, TM, TN, NB>(p, token_tiles, st);
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

hipError_t ilt_k_q8k_bf16(const int8_t* xq, const float* xd, uint16_t* out, int n, int cols, int slabs, hipStream_t st) {
  if (n <= 0) return hipSuccess;
  if (cols <= 0 || cols % 256 != 0) return hipErrorInvalidValue;
  if (slabs) {
    const long long npad = ((long long)n + 255) / 256 * 256, units = npad * (cols / 8);
    hipLaunchKernelGGL(q8k_bf16_kernel<true>, dim3((unsigned)((units + 255) / 256)), dim3(256), 0, st, (const i8*)xq, xd, (u8*)out, n, npad, cols);
  } else {
    const long long units = (long long)n * (cols / 8);
    hipLaunchKernelGGL(q8k_bf16_kernel<false>, dim3((unsigned)((units + 255) / 256)), dim3(256), 0, st, (const i8*)xq, xd, (u8*)out, n, (long long)n, cols);
  }
  return hipGetLastError();
}

hipError_t ilt_k_gemm_bf16(int fmt, const uint8_t* w, long long row_bytes, int rows, int cols, const uint16_t* xb, int ntok,
                           float* y, const float* bias, int acc, hipStream_t st) {
  if (ntok <= 0 || rows <= 0) return hipSuccess;
  BfParams p = {};
  p.w = w; p.rows = rows; p.cols = cols; p.row_bytes = row_bytes; p.x = xb; p.y = y; p.bias = bias; p.acc = acc; p.ntok = ntok;
  p.ldy = rows;
  // Larger tiles fetch and dequantize less per product but leave more of the last round of
  // workgroups idle.  Cost of a variant: rounds over the 256 CUs x tile area / its measured
  // relative rate (128x128 0.85, 128x256 1.0, 256x256 1.36: a CU's 58-63, 53.7 and 39.5 us for 128 rows x 128 tokens x
  // 5120 columns of Q6_K, with as many workgroups on it as fit).
  const long long t128 = (ntok + 127) / 128, t256 = (ntok + 255) / 256, r256 = (rows + 255) / 256, r128 = (rows + 127) / 128;
  const char* force = getenv("ILT_BF16_TILE");     // "1".."3": that variant whatever the shape (tests)
  int tile = force ? atoi(force) : 0;
  if (tile < 1 || tile > 3) {
    // (rounds: whole ones, and the parts' where the last round's tiles are split, see choose_ksplit)
    auto rounds = [&](long long tiles) {
      long long from = 0;
      const int k = choose_ksplit(tiles, cols / 256, from);
      return k > 1 ? split_rounds(from, tiles - from, k, cols / 256) : (double)((tiles + 255) / 256);
    };
    const double c1 = rounds(t128 * r128) * 1.0 / 0.85;
    const double c2 = rounds(t256 * r128) * 2.0 / 1.0;
    const double c3 = rounds(t256 * r256) * 4.0 / 1.36;
    tile = c3 <= c2 && c3 <= c1 ? 3 : c2 <= c1 ? 2 : 1;
  }
  if (tile == 3) return dispatch_bf16<256, 256, 2>(fmt, p, t256, st);
  if (tile == 2) return dispatch_bf16<128, 256, 2>(fmt, p, t256, st);
  return dispatch_bf16<128, 128, 2>(fmt, p, t128, st);
}

hipError_t ilt_k_gemm_bf16_id(int fmt, const uint64_t* ptrs, long long add, const uint32_t* counts, const uint32_t* bases,
                              int ne, long long row_bytes, int rows, int cols, const uint16_t* xb, const uint32_t* rmap,
                              long long total_rows, float* y, hipStream_t st) {
  if (total_rows <= 0 || rows <= 0 || ne <= 0) return hipSuccess;
  if (ne > 256) return hipErrorInvalidValue;
  BfParams p = {};
  p.ptrs = ptrs; p.add = add; p.counts = counts; p.bases = bases; p.ne = ne;
  p.rows = rows; p.cols = cols; p.row_bytes = row_bytes; p.x = xb; p.rmap = rmap; p.y = y; p.ntok = (int)total_rows;
  p.ldy = rows;
  // 256 rows x 128 tokens a workgroup when the matrices have the rows for it: an expert seldom has
  // more than 128 rows of tokens in a chunk.  The experts' formats go to gemm_bf16_regb_kernel;
  // ILT_BF16_ID_TILE (tests): "2" = that tile in gemm_bf16_kernel (a wave: 128 x 64, a quarter less read
  // from LDS per MFMA than 128 x 128), "1" = 128 x 128 always.
  const char* force = getenv("ILT_BF16_ID_TILE");
  const int forced = force ? atoi(force) : 0;
  if (rows % 256 == 0 && forced == 0 && (fmt == ILT_IQ2_XXS || fmt == ILT_Q2_K)) {      // weights straight into MFMA operands
    if ((long long)rows * row_bytes >= 0x7FFFFFFFLL || row_bytes >= (1 << 24)) return hipErrorInvalidValue;      // the kernel's 32- and 24-bit address arithmetic
    return fmt == ILT_IQ2_XXS ? launch_regb<ILT_IQ2_XXS, false>(p, total_rows / 128 + ne, st) : launch_regb<ILT_Q2_K, false>(p, total_rows / 128 + ne, st);
  }
  if (rows % 256 == 0 && forced != 1) {      // the expert formats (Q4_K / Q6_K raw sets would not fit the registers)
    if (fmt == ILT_IQ2_XXS) return launch_bf16<ILT_IQ2_XXS, 256, 128, 4>(p, total_rows / 128 + ne, st);
    if (fmt == ILT_Q2_K) return launch_bf16<ILT_Q2_K, 256, 128, 4>(p, total_rows / 128 + ne, st);
  }
  return dispatch_bf16<128, 128, 2>(fmt, p, total_rows / 128 + ne, st);
}

hipError_t ilt_k_gemm_bf16_id_glu(int fmt, const uint64_t* ptrs, long long add_gate, long long add_up, const uint32_t* counts,
                                  const uint32_t* bases, int ne, long long row_bytes, int rows, int cols, const uint16_t* xb,
                                  const uint32_t* rmap, long long total_rows, float clamp, const float* wrow, uint16_t* mid,
                                  hipStream_t st) {
  if (total_rows <= 0 || rows <= 0 || ne <= 0) return hipSuccess;
  if (ne > 256 || fmt != ILT_IQ2_XXS || rows % 128 != 0 || add_up < add_gate) return hipErrorInvalidValue;
  // the kernel's 32- and 24-bit address arithmetic
  if ((long long)rows * row_bytes + (add_up - add_gate) >= 0x7FFFFFFFLL || row_bytes >= (1 << 24) || rows >= (1 << 21))
    return hipErrorInvalidValue;
  BfParams p = {};
  p.ptrs = ptrs; p.add = add_gate; p.up_delta = (unsigned)(add_up - add_gate); p.counts = counts; p.bases = bases; p.ne = ne;
  p.rows = rows; p.cols = cols; p.row_bytes = row_bytes; p.x = xb; p.rmap = rmap; p.ntok = (int)total_rows;
  p.wrow = wrow; p.clamp = clamp; p.mid = mid;
  return launch_regb<ILT_IQ2_XXS, true>(p, total_rows / 128 + ne, st);
}

// 64-row tiles (dense) where the 128-row tiles would leave CUs idle: fewer tiles than one and a half rounds over the
// 256 CUs, or a last round less than half full.  ILT_I8P_TM (tests): 64 or 128 whatever the shape.
static int i8p_tile_rows(long long tiles128) {
  const char* force = getenv("ILT_I8P_TM");
  if (force && (atoi(force) == 64 || atoi(force) == 128)) return atoi(force);
  const long long rem = tiles128 % 256;
  return (tiles128 < 384 || (tiles128 < 1024 && rem != 0 && rem < 128)) ? 64 : 128;
}

template <bool GROUPED>
static hipError_t launch_i8p(int fmt, const BfParams& p, long long token_tiles, hipStream_t st, int tm = 128) {
  if ((fmt != ILT_Q6_K && fmt != ILT_Q4_K && fmt != ILT_Q2_K && fmt != ILT_IQ2_XXS) || p.cols % 256 != 0 || (long long)p.rows * 1024 >= 0x7FFFFFFFLL)
    return hipErrorInvalidValue;
  const long long total = token_tiles * ((p.rows + tm - 1) / tm), per = (total + 7) / 8;
  if (per * 8 > 0x7FFFFFFFLL) return hipErrorInvalidValue;
  const dim3 grid((unsigned)(per * 8));
  if constexpr (!GROUPED) {
    if (tm == 64) {
      if (fmt == ILT_Q6_K) hipLaunchKernelGGL((gemm_i8p_kernel<ILT_Q6_K, false, 64>), grid, dim3(256), 0, st, p);
      else if (fmt == ILT_Q4_K) hipLaunchKernelGGL((gemm_i8p_kernel<ILT_Q4_K, false, 64>), grid, dim3(256), 0, st, p);
      else if (fmt == ILT_Q2_K) hipLaunchKernelGGL((gemm_i8p_kernel<ILT_Q2_K, false, 64>), grid, dim3(256), 0, st, p);
      else hipLaunchKernelGGL((gemm_i8p_kernel<ILT_IQ2_XXS, false, 64>), grid, dim3(256), 0, st, p);
      return hipGetLastError();
    }
  }
  if (fmt == ILT_Q6_K) hipLaunchKernelGGL((gemm_i8p_kernel<ILT_Q6_K, GROUPED>), grid, dim3(512), 0, st, p);
  else if (fmt == ILT_Q4_K) hipLaunchKernelGGL((gemm_i8p_kernel<ILT_Q4_K, GROUPED>), grid, dim3(512), 0, st, p);
  else if (fmt == ILT_Q2_K) hipLaunchKernelGGL((gemm_i8p_kernel<ILT_Q2_K, GROUPED>), grid, dim3(512), 0, st, p);
  else hipLaunchKernelGGL((gemm_i8p_kernel<ILT_IQ2_XXS, GROUPED>), grid, dim3(512), 0, st, p);
  return hipGetLastError();
}

hipError_t ilt_k_gemm_i8_planes(int fmt, const uint8_t* w, long long row_bytes, int rows, int cols, const int8_t* xq, const float* xd,
                                const int* bsums, int ntok, float* y, const float* bias, int acc, hipStream_t st, long long ldy) {
  if (ntok <= 0 || rows <= 0) return hipSuccess;
  if (ldy == 0) ldy = rows;
  if (ldy < rows || ldy * 1024 >= 0x7FFFFFFFLL) return hipErrorInvalidValue;
  BfParams p = {};
  p.w = w; p.rows = rows; p.cols = cols; p.row_bytes = row_bytes; p.x = (const u16*)xq; p.xd = xd; p.bsums = bsums;
  p.y = y; p.bias = bias; p.acc = acc; p.ntok = ntok; p.ldy = ldy;
  const long long tt = (ntok + 127) / 128;
  return launch_i8p<false>(fmt, p, tt, st, i8p_tile_rows(tt * ((rows + 127) / 128)));
}

// Up to three matrices of one format (Q6_K, Q4_K, Q2_K) on the same tokens in one launch: their row tiles one after
// another, so that matrices too small to fill the chip on their own share it (Q/K/V, gate and up of a prompt's chunk).
// hipErrorNotSupported: the caller launches them one by one.
hipError_t ilt_k_gemm_i8_planes_n(int fmt, int nmat, const uint8_t* const* ws, const int* rows, float* const* ys, const float* const* biases,
                                  long long row_bytes, int cols, const int8_t* xq, const float* xd, const int* bsums, int ntok, int acc,
                                  hipStream_t st) {
  if (nmat < 2 || nmat > 3 || ntok < 96 || (fmt != ILT_Q6_K && fmt != ILT_Q4_K && fmt != ILT_Q2_K) || cols % 256 != 0) return hipErrorNotSupported;
  BfParams p = {};
  long long tiles128 = 0;
  for (int m = 0; m < nmat; m++) {
    if (rows[m] < 128 || rows[m] >= (1 << 21) || (long long)rows[m] * row_bytes >= 0x7FFFFFFFLL) return hipErrorNotSupported;
    p.mw[m] = ws[m]; p.mrows[m] = rows[m]; p.my[m] = ys[m]; p.mbias[m] = biases ? biases[m] : nullptr;
    tiles128 += (rows[m] + 127) / 128;
  }
  if (tiles128 * 128 >= (1 << 21)) return hipErrorNotSupported;
  const int tm = i8p_tile_rows(tiles128 * ((ntok + 127) / 128));
  long long tiles = 0;
  for (int m = 0; m < nmat; m++) tiles += (rows[m] + tm - 1) / tm;
  p.nmulti = nmat;
  p.w = ws[0]; p.rows = (int)(tiles * tm); p.cols = cols; p.row_bytes = row_bytes; p.x = (const u16*)xq; p.xd = xd; p.bsums = bsums;
  p.y = ys[0]; p.acc = acc; p.ntok = ntok; p.ldy = rows[0];
  return launch_i8p<false>(fmt, p, (ntok + 127) / 128, st, tm);
}

hipError_t ilt_k_planes_i8(int fmt, const uint8_t* w, long long row_bytes, int rows, int cols, uint8_t* wh, uint8_t* wl, float* wdf,
                           hipStream_t st) {
  if (rows <= 0) return hipSuccess;
  if (fmt != ILT_Q6_K || cols % 256 != 0 || (long long)rows * row_bytes >= 0xFFFFFFF0LL) return hipErrorInvalidValue;
  const long long units = (long long)rows * (cols / 256) * 16;
  if ((units + 255) / 256 > 0x7FFFFFFFLL) return hipErrorInvalidValue;
  hipLaunchKernelGGL(planes_i8_kernel<ILT_Q6_K>, dim3((unsigned)((units + 255) / 256)), dim3(256), 0, st, w, row_bytes, rows, cols, wh, wl, wdf);
  return hipGetLastError();
}

hipError_t ilt_k_gemm_i8_pp(const uint8_t* wh, const uint8_t* wl, const float* wdf, int rows, int cols, const int8_t* xq, const float* xd,
                            int ntok, float* y, const float* bias, int acc, hipStream_t st) {
  if (ntok <= 0 || rows <= 0) return hipSuccess;
  if (cols % 256 != 0 || (long long)rows * 1024 >= 0x7FFFFFFFLL || (long long)128 * cols >= 0x7FFFFFFFLL) return hipErrorInvalidValue;
  BfParams p = {};
  p.w = wh; p.wlo = wl; p.wdf = wdf; p.rows = rows; p.cols = cols; p.row_bytes = cols; p.x = (const u16*)xq; p.xd = xd;
  p.y = y; p.bias = bias; p.acc = acc; p.ntok = ntok; p.ldy = rows;
  const long long total = (long long)((ntok + 127) / 128) * ((rows + 127) / 128), per = (total + 7) / 8;
  if (per * 8 > 0x7FFFFFFFLL) return hipErrorInvalidValue;
  static bool attr_set[8] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 8) dev = 0;
  if (!attr_set[dev]) {            // more dynamic LDS than the default 64 KB: asked for once per device
    const hipError_t e = hipFuncSetAttribute((const void*)gemm_i8pp_kernel<1>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)sizeof(I8ppSmem<1>));
    if (e != hipSuccess) return e;
    attr_set[dev] = true;
  }
  hipLaunchKernelGGL(gemm_i8pp_kernel<1>, dim3((unsigned)(per * 8)), dim3(512), sizeof(I8ppSmem<1>), st, p);
  return hipGetLastError();
}

hipError_t ilt_k_gemm_i8_q8(const uint8_t* wq, const uint16_t* wd, int rows, int cols, const int8_t* xq, const float* xs, int ntok,
                            float* y, const float* bias, int acc, hipStream_t st, long long ldy) {
  if (ntok <= 0 || rows <= 0) return hipSuccess;
  if (ldy == 0) ldy = rows;
  if (cols % 64 != 0 || ldy < rows || ldy * 1024 >= 0x7FFFFFFFLL || (long long)128 * cols >= 0x7FFFFFFFLL) return hipErrorInvalidValue;
  BfParams p = {};
  p.w = wq; p.wdq = wd; p.rows = rows; p.cols = cols; p.row_bytes = cols; p.x = (const u16*)xq; p.xd = xs;
  p.y = y; p.bias = bias; p.acc = acc; p.ntok = ntok; p.ldy = ldy;
  const long long total = (long long)((ntok + 127) / 128) * ((rows + 127) / 128), per = (total + 7) / 8;
  if (per * 8 > 0x7FFFFFFFLL) return hipErrorInvalidValue;
  hipLaunchKernelGGL(gemm_i8q_kernel, dim3((unsigned)(per * 8)), dim3(512), 0, st, p);
  return hipGetLastError();
}

hipError_t ilt_k_gemm_i8_planes_id(int fmt, const uint64_t* ptrs, long long add, const uint32_t* counts, const uint32_t* bases, int ne,
                                   long long row_bytes, int rows, int cols, const int8_t* xq, const float* xd, const int* bsums,
                                   long long total_rows, float* y, hipStream_t st) {
  if (total_rows <= 0 || rows <= 0 || ne <= 0) return hipSuccess;
  if (ne > 256) return hipErrorInvalidValue;
  BfParams p = {};
  p.ptrs = ptrs; p.add = add; p.counts = counts; p.bases = bases; p.ne = ne;
  p.rows = rows; p.cols = cols; p.row_bytes = row_bytes; p.x = (const u16*)xq; p.xd = xd; p.bsums = bsums;
  p.y = y; p.ntok = (int)total_rows; p.ldy = rows;
  return launch_i8p<true>(fmt, p, total_rows / 128 + ne, st);
}

hipError_t ilt_k_cvt_bf16_slabs(const float* x, uint16_t* out, int n, int cols, hipStream_t st) {
  if (n <= 0) return hipSuccess;
  const long long npad = (n + 255LL) / 256 * 256, threads = npad * (cols / 8);
  hipLaunchKernelGGL(cvt_bf16_slabs_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, st, x, (u8*)out, n, npad, cols);
  return hipGetLastError();
}

hipError_t ilt_k_dequant_bf16(int fmt, const uint8_t* w, long long row_bytes, int rows, int cols, uint16_t* outp, hipStream_t st) {
  if (rows <= 0) return hipSuccess;
  u8* out = (u8*)outp;
  const long long groups = (rows + 255LL) / 256 * 2;                    // of 128 rows, the padding included
  const long long units = groups * (cols / 256);
  if (units > 0x7FFFFFF0LL) return hipErrorInvalidValue;
  const int total = (int)units;
  const dim3 grid((unsigned)((units + 7) / 8 * 8));
  switch (fmt) {
    case ILT_Q4_K: hipLaunchKernelGGL(dequant_bf16_kernel<ILT_Q4_K>, grid, dim3(256), 0, st, w, row_bytes, rows, cols, out, total); break;
    case ILT_Q6_K: hipLaunchKernelGGL(dequant_bf16_kernel<ILT_Q6_K>, grid, dim3(256), 0, st, w, row_bytes, rows, cols, out, total); break;
    case ILT_Q2_K: hipLaunchKernelGGL(dequant_bf16_kernel<ILT_Q2_K>, grid, dim3(256), 0, st, w, row_bytes, rows, cols, out, total); break;
    case ILT_IQ2_XXS: hipLaunchKernelGGL(dequant_bf16_kernel<ILT_IQ2_XXS>, grid, dim3(256), 0, st, w, row_bytes, rows, cols, out, total); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

template <int T>
static hipError_t launch_plain(const BfParams& p, hipStream_t st) {
  const long long total = (long long)((p.ntok + T - 1) / T) * ((p.rows + T - 1) / T), per = (total + 7) / 8;
  if (per * 8 > 0x7FFFFFFFLL) return hipErrorInvalidValue;
  hipLaunchKernelGGL(gemm_bf16_plain_kernel<T>, dim3((unsigned)(per * 8)), dim3(256), 0, st, p);
  return hipGetLastError();
}

hipError_t ilt_k_gemm_bf16_plain(const uint16_t* wb, int rows, int cols, const uint16_t* xb, int ntok, float* y, const float* bias,
                                 int acc, hipStream_t st) {
  if (ntok <= 0 || rows <= 0) return hipSuccess;
  BfParams p = {};
  p.w = (const uint8_t*)wb; p.rows = rows; p.cols = cols; p.x = xb; p.y = y; p.bias = bias; p.acc = acc; p.ntok = ntok;
  p.ldy = rows;
  // One 256 x 256 tile a CU at a time: tiles beyond a whole number of rounds over the 256 CUs
  // would take a round of their own.  Instead the row tiles that fill whole rounds go to the
  // 256-tiles and the rows left over to 128-tiles (512 a round, a round of them about 0.7 of a
  // big one for half the work); with less than one round of 256-tiles, everything to 128-tiles.
  const long long nt = (ntok + 255) / 256, nr = (rows + 255) / 256, full = nt * nr / 256;
  const char* force = getenv("ILT_BF16_PLAIN_SPLIT");      // "0": 256-tiles only; "128": 128-tiles only (tests)
  long long nr_big = nr;
  if (force ? atoi(force) == 128 : full == 0) nr_big = 0;
  else if (!(force && atoi(force) == 0) && nt * nr % 256 != 0) {
    const long long nr1 = full * 256 / nt, rest = rows - nr1 * 256;
    const long long small_rounds = (((rest + 127) / 128) * ((ntok + 127) / 128) + 511) / 512;
    if (0.7 * (double)small_rounds < 1.0) nr_big = nr1;
  }
  if (nr_big > 0) {
    BfParams q = p;
    q.rows = (int)min((long long)rows, nr_big * 256);
    const hipError_t e = launch_plain<256>(q, st);
    if (e != hipSuccess) return e;
  }
  if (nr_big * 256 < rows) {
    const long long r1 = nr_big * 256;
    BfParams q = p;
    q.rows = rows - (int)r1;
    q.w = p.w + r1 * (long long)cols * 2;                // whole groups of 128 rows: their slabs follow one another
    q.y = y + r1;
    q.bias = bias ? bias + r1 : nullptr;
    return launch_plain<128>(q, st);
  }
  return hipSuccess;
}
