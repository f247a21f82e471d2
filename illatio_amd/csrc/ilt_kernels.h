// Internal interface between the kernel translation units and the C-ABI layer.
#ifndef ILT_KERNELS_H
#define ILT_KERNELS_H

#include <hip/hip_runtime.h>
#include <stdint.h>

// Weight formats, numbered as GGUF numbers them (the reference's src/gguf.lisp:31-40).
#define ILT_Q8_0 8
#define ILT_Q2_K 10
#define ILT_Q4_K 12
#define ILT_Q6_K 14
#define ILT_IQ2_XXS 16

// Q6_K on the device: the 210-byte GGUF block followed by two bytes of padding, so that
// every block (and every 16-byte piece of it) starts on a 4-byte boundary.
#define ILT_Q6K_STRIDE 212

struct IltGemvMat {
  const uint8_t* w;          // the matrix (Q8_0: its int8 quants), rows one after another
  const uint16_t* wd;        // Q8_0 only: the f16 block scales
  float* y;                  // output rows
  const float* bias;         // added after the sum, or null
  long long row_bytes;
  long long add;             // experts: grid y's matrix is at ptrs[y] + add (w unused)
  int rows;
  int fmt;                   // ILT_Q8_0, ILT_Q4_K, ILT_Q6_K (dense); the expert kernels ignore it
  int batch0, nbat;          // this matrix's first batch among the launch's, and how many (set at launch)
  int rq, rr;                // rows / nbat and rows % nbat: batch i is rq rows, one more for the first rr (set at launch)
};

// A token's d4-route carried along by a product launch (the streamed variant, Q8_0): one of the activation waves of the
// first workgroup routes once its own work is done, while the rows stream in.  logits null: none.  done: set by
// ilt_gemv_launch when the launch it made takes the routing along (otherwise the caller launches d4_route itself).
struct IltRouteAlong {
  const float* logits; const float* bias;    // ne logits; ne biases or null
  uint32_t* sel; float* wout;                // nu slots each
  int ne, nu; float scale;
  int done;
};

// KV cache rows read ahead by a product launch's activation waves once their own work is done (the streamed variant):
// the launch after it -- one token's attention -- then finds its keys and values in the L2 of the die that wants them.
// Workgroup g runs on die g % 8; die x reads floats off[x] .. off[x] + width[x] - 1 of each of the nrows rows of a and
// of b (stride floats apart), and every die the three small vectors.  a null: nothing.
struct IltCacheAhead {
  const float* a; const float* b;
  int stride, nrows;
  int off[8], width[8];
  const float* small[3]; int nsmall[3];
};

// The next streamed product's rows, read ahead the same way: that launch's plan (ilt_gemv_plan) says which rows its
// workgroup g -- die g % 8 -- will stream, and this launch's idle waves on that die touch their cache lines, so that
// the next launch streams from L2 instead of HBM.  nm 0: nothing.
struct IltRowsAhead {
  int nm;                                                                       // matrices (a gate/up pair: two, with the same batches)
  struct M { const uint8_t* w; long long row_bytes; int rq, rr, batch0, nbat; } m[4];
};

// The MoE step's sum carried along by its last product (the shared expert's down launch): y[r] becomes
// ((0 + rows[0][r]) + rows[1][r] + ...) + (the product's row r) -- the routed experts' down rows added in order, then
// the shared expert's, as d4-routed! and its caller add them (moe_sum's arithmetic) -- instead of a launch for the
// sum.  rows null: nothing.  Streamed Q8_0 launches without bias or acc only, k <= 8; ilt_gemv_launch returns
// hipErrorNotSupported where the launch cannot take it, and has launched nothing then.
struct IltSumAlong {
  const float* rows;
  long long stride;          // floats from one row to the next
  int k;
};

struct IltGemvParams {
  IltGemvMat mat[4];         // up to four matrices sharing the activations
  int nmat;
  const uint64_t* ptrs;      // experts: grid y's matrices are at ptrs[y] + mat[i].add,
  const uint32_t* sel;       //   or at ptrs[sel[y]] + mat[i].add when sel is given (ptrs = all the slots)
  int cols;
  const int8_t* xq;          // quantized activations ...
  const float* xs;           //   their block scales (per 32 for Q8_0, per 256 otherwise)
  const int* bsums;          //   Q8_K: sums of each 16 quants
  const float* xf;           // ... or the activations as floats, quantized by each workgroup
  const float* norm_w;       //   floats only: quantize rmsnorm!(x) * norm_w instead of x (model.lisp:205-216)
  float eps;                 //   the norm's epsilon
  int norm_seq;              //   1 = always add the squares one after another (the CPU's order) instead of when needed
  int f16_scale;             // Q8_0 from floats: store the scale through fp16 (*q8-f16-scale*)
  int x_stride;              // activations of grid y start at y * x_stride elements
  int y_stride;              // outputs of grid y start at y * y_stride
  int acc;                   // y += result
  int glu;                   // mat[0] = gate, mat[1] = up, into mat[0].y: 1 = swiglu! (model.lisp:364-378),
                             //   2 = d4-routed!/d4-shared!'s (ds4f.lisp:1016-1019): clamp, silu(g)*u, times wts[y]
  float clamp;               // glu 2: g = min(g, clamp), u in [-clamp, clamp] when clamp > 1e-6
  const float* wts;          // glu 2: the weight of grid y's expert, or null
  int group_rows;            // >0: row r reads the activations of group r/group_rows (cols apart)
  int nbatches;              // batches of rows in the launch (per group, per grid y; set at launch)
  int wgs_per_group;         // grouped rows: workgroups sharing one group (set at launch)
  int batch;                 // rows a wave takes through phase A at a time (set at launch)
  int region;                // streamed variant: bytes of LDS per wave for its rows (set at launch)
  int nz;                    // streamed variant: experts taking part (set at launch)
  uint32_t s_magic;          // ceil(2^32 / blocks per row)
  // (what only some waves read, and late, comes last: the fields every wave needs for its first loads then sit in the
  // kernel arguments' first cache lines, where a few scalar loads bring them in)
  IltSumAlong sum;
  IltRouteAlong route;
  IltCacheAhead ahead;
  IltRowsAhead rows_ahead;
  // grid y's expert on several rows of activations (the looping variant only): rows bases[y] .. bases[y] + counts[y] - 1
  // of the activations and of the output, x_stride / y_stride apart, its matrix read from memory once and from the
  // cache for the rows after the first (the counts / bases of the reference's d4_mv_*, ds4f.cu:762-772); null = row y
  const uint32_t* counts;
  const uint32_t* bases;
};

// The kernel is chosen by the matrices' formats (mat[i].fmt): one format, or Q4_K and Q6_K mixed.
hipError_t ilt_gemv_launch(IltGemvParams& p, int nz, hipStream_t st);
// The streamed variant's plan for p without launching (the batches of each matrix): hipSuccess when ilt_gemv_launch
// would take the streamed variant with a grid of 256 workgroups, hipErrorNotSupported otherwise.
hipError_t ilt_gemv_plan(IltGemvParams& p, int nz);
// out = the rows p's launch will stream, for another launch's rows_ahead (p planned by ilt_gemv_plan)
void ilt_gemv_rows_of(const IltGemvParams& p, IltRowsAhead& out);

unsigned long long ilt_k_streamed_launches();      // decode products launched as the streamed variant so far (diagnostic)

hipError_t ilt_k_quant_q8(const float* x, int8_t* xq, float* xs, int* xsum, long long nblocks, int f16_scale, hipStream_t st);
hipError_t ilt_k_quant_q8k(const float* x, int8_t* xq, float* xd, int* bsums, long long nblocks, hipStream_t st);
hipError_t ilt_k_swiglu_quant_q8k(const float* gate, const float* up, int8_t* xq, float* xd, int* bsums, long long nblocks, hipStream_t st);
// ntok rows of cols floats, x_stride floats apart, quantized into packed rows: quantize-q8! (k 0) or quantize-q8k! (k 1)
hipError_t ilt_k_quant_rows(int k, const float* x, int8_t* xq, float* xs, int* bsums, long long ntok, int cols, long long x_stride,
                            int f16_scale, hipStream_t st);
// rmsnorm! then quantize-q8! (k 0; xsum may be null) or quantize-q8k! (k 1), a row of DIM floats a workgroup
hipError_t ilt_k_rmsnorm_quant(int k, const float* x, const float* w, float* h, int8_t* xq, float* xs, int* xsum, int dim,
                               float eps, int f16_scale, int seq, int nrows, hipStream_t st);
hipError_t ilt_k_mm_f16(int ncols, int nrows, int ntok, long long row_halfs, int x_stride, int y_stride, const uint16_t* w, const float* x,
                        float* y, hipStream_t st);
hipError_t ilt_k_repack_q8(const uint8_t* raw, int8_t* qs, uint16_t* d, long long nblocks, hipStream_t st);
hipError_t ilt_k_repack_q6k(const uint8_t* raw, uint8_t* out, long long nblocks, hipStream_t st);
hipError_t ilt_k_copy_bytes(const uint8_t* src, uint8_t* dst, long long bytes, hipStream_t st);
// for each of the nz experts with srcs[z] set: bytes from srcs[z] + add to ptrs[z] + add (d4_read_through, ds4f.cu:742-760)
hipError_t ilt_k_read_through(const unsigned long long* srcs, const unsigned long long* ptrs, int nz, long long add, long long bytes,
                              hipStream_t st);
hipError_t ilt_k_dequant_rows(int fmt, const uint8_t* w, const uint16_t* wd, const int* rows_idx, long long nrows,
                              int cols, long long row_bytes, float* out, hipStream_t st);

hipError_t ilt_k_route(int ne, int nu, int hash, float scale, int has_bias, const float* logits, const float* bias,
                       const int* tid2eid, const uint32_t* tokens, uint32_t* sel, float* wout, int ntok, hipStream_t st);
hipError_t ilt_k_group_zero(int ne, uint32_t* counts, hipStream_t st);
hipError_t ilt_k_group_count(int n, int ne, int nu, const uint32_t* sel, uint32_t* counts, uint32_t* rank, hipStream_t st);
hipError_t ilt_k_group_scan(int n, int ne, int nu, const uint32_t* counts, uint32_t* bases, hipStream_t st);
hipError_t ilt_k_group_scatter(int n, int ne, int nu, const uint32_t* sel, const uint32_t* rank, const uint32_t* bases,
                               const float* w, uint32_t* rmap, uint32_t* smap, float* wrow, hipStream_t st);
hipError_t ilt_k_rows_expert(int n, const uint32_t* sel, const uint32_t* smap, uint32_t* rexp, hipStream_t st);
hipError_t ilt_k_gather_rows(int d, int nrows, const float* src, const uint32_t* map, float* x, hipStream_t st);
hipError_t ilt_k_swiglu_w(int n, int ff, float clamp, const float* g, const float* u, const float* w, float* mid,
                          int8_t* xq, float* xs, hipStream_t st);
hipError_t ilt_k_moe_sum(int d, int k, const float* down, const float* shared_, float* moe, const uint32_t* perm, hipStream_t st);
hipError_t ilt_k_moe_sum_rows(int d, int nu, int ntok, const float* down, const uint32_t* map, const float* shared_,
                              float* moe, hipStream_t st);

// ldy: floats from one token's results to the next token's in y (0: rows)
hipError_t ilt_k_gemm_i8(int fmt, const uint8_t* w, const uint16_t* wd, long long row_bytes, int rows, int cols,
                         const int8_t* xq, const float* xs, const int* bsums, int ntok, float* y, const float* bias,
                         int acc, hipStream_t st, long long ldy = 0);
// Q6_K, Q4_K and Q2_K, exact, on the pipelined kernel (kernels_gemm_bf16.hip): scale * quant as int8 planes
hipError_t ilt_k_gemm_i8_planes(int fmt, const uint8_t* w, long long row_bytes, int rows, int cols, const int8_t* xq, const float* xd,
                                const int* bsums, int ntok, float* y, const float* bias, int acc, hipStream_t st, long long ldy = 0);
hipError_t ilt_k_gemm_i8_planes_n(int fmt, int nmat, const uint8_t* const* ws, const int* rows, float* const* ys, const float* const* biases,
                                  long long row_bytes, int cols, const int8_t* xq, const float* xd, const int* bsums, int ntok, int acc,
                                  hipStream_t st);
// The exact product in two passes (Q6_K): the two int8 planes and d per row and super-block once, then the product from them
hipError_t ilt_k_planes_i8(int fmt, const uint8_t* w, long long row_bytes, int rows, int cols, uint8_t* wh, uint8_t* wl, float* wdf,
                           hipStream_t st);
hipError_t ilt_k_gemm_i8_pp(const uint8_t* wh, const uint8_t* wl, const float* wdf, int rows, int cols, const int8_t* xq, const float* xd,
                            int ntok, float* y, const float* bias, int acc, hipStream_t st);
// Q8_0, exact, on the pipelined kernel (cols a multiple of 64)
hipError_t ilt_k_gemm_i8_q8(const uint8_t* wq, const uint16_t* wd, int rows, int cols, const int8_t* xq, const float* xs, int ntok,
                            float* y, const float* bias, int acc, hipStream_t st, long long ldy = 0);
hipError_t ilt_k_gemm_i8_planes_id(int fmt, const uint64_t* ptrs, long long add, const uint32_t* counts, const uint32_t* bases, int ne,
                                   long long row_bytes, int rows, int cols, const int8_t* xq, const float* xd, const int* bsums,
                                   long long total_rows, float* y, hipStream_t st);
hipError_t ilt_k_gemm_i8_id(int fmt, const uint64_t* ptrs, long long add, const uint32_t* counts, const uint32_t* bases,
                            int ne, long long row_bytes, int rows, int cols, const int8_t* xq, const float* xs,
                            const int* bsums, long long total_rows, float* y, hipStream_t st);

// bf16 matrix-core products on bf16 activations (ilt_k_cvt_bf16 rounds floats, n a multiple
// of 8); weights dequantized to bf16 in LDS: Q4_K, Q6_K (212-byte device blocks), Q2_K,
// IQ2_XXS.  Within 2e-2 of the CPU path.
hipError_t ilt_k_cvt_bf16(const float* x, uint16_t* xb, long long n, hipStream_t st);
// Q8_K quants times their block scales as bf16, n tokens of cols (a multiple of 256): rows of cols, or cvt_bf16_slabs' layout
hipError_t ilt_k_q8k_bf16(const int8_t* xq, const float* xd, uint16_t* out, int n, int cols, int slabs, hipStream_t st);
hipError_t ilt_k_gemm_bf16(int fmt, const uint8_t* w, long long row_bytes, int rows, int cols, const uint16_t* xb, int ntok,
                           float* y, const float* bias, int acc, hipStream_t st);
hipError_t ilt_k_gemm_bf16_id(int fmt, const uint64_t* ptrs, long long add, const uint32_t* counts, const uint32_t* bases,
                              int ne, long long row_bytes, int rows, int cols, const uint16_t* xb, const uint32_t* rmap,
                              long long total_rows, float* y, hipStream_t st);
hipError_t ilt_k_gemm_bf16_id_glu(int fmt, const uint64_t* ptrs, long long add_gate, long long add_up, const uint32_t* counts,
                                  const uint32_t* bases, int ne, long long row_bytes, int rows, int cols, const uint16_t* xb,
                                  const uint32_t* rmap, long long total_rows, float clamp, const float* wrow, uint16_t* mid,
                                  hipStream_t st);
// The two-pass product for many tokens: the matrix dequantized once to bf16, then a plain bf16
// product (cols a multiple of 128).  Both operands in slabs (32 columns of 128 rows are 8 KB in
// one piece), rows and tokens padded to a multiple of 256: 2 * cols * ceil(n / 256) * 256 bytes.
hipError_t ilt_k_cvt_bf16_slabs(const float* x, uint16_t* out, int n, int cols, hipStream_t st);
hipError_t ilt_k_dequant_bf16(int fmt, const uint8_t* w, long long row_bytes, int rows, int cols, uint16_t* out, hipStream_t st);
hipError_t ilt_k_gemm_bf16_plain(const uint16_t* wb, int rows, int cols, const uint16_t* xb, int ntok, float* y, const float* bias,
                                 int acc, hipStream_t st);
hipError_t ilt_k_swiglu_w_bf16(int n, int ff, float clamp, const float* g, const float* u, const float* w, uint16_t* mid, hipStream_t st);

// The dense-forward harness's kernels between the products (kernels_attn.hip)
hipError_t ilt_k_qk_rope(float* q, float* k, const float* v, const float* qn, const float* kn, const float* rope, float* kc, float* vc,
                         int nh, int nkv, int hd, int rd, int pos0, float eps, int neox, int ntok, hipStream_t st);
hipError_t ilt_k_argmax(const float* v, int n, int* out, void* scratch, hipStream_t st);
hipError_t ilt_k_attn_step(const float* q, const float* k, const float* v, const float* qn, const float* kn, const float* rope, float* kc,
                           float* vc, float* out, int nh, int nkv, int hd, int rd, int pos, float eps, int neox, float* scratch, hipStream_t st);
hipError_t ilt_k_attn_giveups(unsigned long long* out);
hipError_t ilt_k_attn_rows(const float* q, const float* kc, const float* vc, float* out, int nh, int nkv, int hd, int pos0, int ntok,
                           float* scratch, hipStream_t st);
hipError_t ilt_k_swiglu_rows(float* a, const float* b, long long n, hipStream_t st);

#endif  // ILT_KERNELS_H
