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

struct IltGemvParams {
  const uint8_t* w;          // the matrix (Q8_0: its int8 quants), rows one after another
  const uint64_t* ptrs;      // or, per grid z, the device address of an expert's slot ...
  long long add;             // ... plus this byte offset into it
  const uint16_t* wd;        // Q8_0 only: the f16 block scales
  int rows, cols, row_bytes;
  const int8_t* xq;          // quantized activations
  const float* xs;           // their block scales (per 32 for Q8_0, per 256 otherwise)
  const int* bsums;          // Q8_K: sums of each 16 quants
  int x_stride;              // activations of grid z start at z * x_stride elements
  float* y;                  // output; grid z's at z * y_stride
  int y_stride;
  const float* bias;         // added after the sum, or null
  int acc;                   // y += result
  int rw;                    // rows per workgroup
  int group_rows;            // >0: row r reads the activations of group r/group_rows (cols apart)
};

int ilt_gemv_pick_rw(int fmt, int rows, int cols, int nz);
hipError_t ilt_gemv_launch(int fmt, const IltGemvParams& p, int nz, hipStream_t st);

hipError_t ilt_k_quant_q8(const float* x, int8_t* xq, float* xs, int* xsum, long long nblocks, int f16_scale, hipStream_t st);
hipError_t ilt_k_quant_q8k(const float* x, int8_t* xq, float* xd, int* bsums, long long nblocks, hipStream_t st);
hipError_t ilt_k_repack_q8(const uint8_t* raw, int8_t* qs, uint16_t* d, long long nblocks, hipStream_t st);
hipError_t ilt_k_copy_bytes(const uint8_t* src, uint8_t* dst, long long bytes, hipStream_t st);
hipError_t ilt_k_dequant_rows(int fmt, const uint8_t* w, const uint16_t* wd, const int* rows_idx, long long nrows,
                              int cols, long long row_bytes, float* out, hipStream_t st);

hipError_t ilt_k_route(int ne, int nu, int hash, float scale, int has_bias, const float* logits, const float* bias,
                       const int* tid2eid, const uint32_t* tokens, uint32_t* sel, float* wout, int ntok, hipStream_t st);
hipError_t ilt_k_group_zero(int ne, uint32_t* counts, hipStream_t st);
hipError_t ilt_k_group_count(int n, int ne, int nu, const uint32_t* sel, uint32_t* counts, uint32_t* rank, hipStream_t st);
hipError_t ilt_k_group_scan(int n, int ne, int nu, const uint32_t* counts, uint32_t* bases, hipStream_t st);
hipError_t ilt_k_group_scatter(int n, int ne, int nu, const uint32_t* sel, const uint32_t* rank, const uint32_t* bases,
                               const float* w, uint32_t* rmap, uint32_t* smap, float* wrow, hipStream_t st);
hipError_t ilt_k_gather_rows(int d, int nrows, const float* src, const uint32_t* map, float* x, hipStream_t st);
hipError_t ilt_k_swiglu_w(int n, int ff, float clamp, const float* g, const float* u, const float* w, float* mid,
                          int8_t* xq, float* xs, hipStream_t st);
hipError_t ilt_k_moe_sum(int d, int k, const float* down, const float* shared_, float* moe, const uint32_t* perm, hipStream_t st);
hipError_t ilt_k_moe_sum_rows(int d, int nu, int ntok, const float* down, const uint32_t* map, const float* shared_,
                              float* moe, hipStream_t st);

hipError_t ilt_k_gemm_i8(int fmt, const uint8_t* w, const uint16_t* wd, long long row_bytes, int rows, int cols,
                         const int8_t* xq, const float* xs, const int* bsums, int ntok, float* y, const float* bias,
                         int acc, hipStream_t st);
hipError_t ilt_k_gemm_i8_id(int fmt, const uint64_t* ptrs, long long add, const uint32_t* counts, const uint32_t* bases,
                            int ne, long long row_bytes, int rows, int cols, const int8_t* xq, const float* xs,
                            const int* bsums, long long total_rows, float* y, hipStream_t st);

#endif  // ILT_KERNELS_H
