/*
 * illatio_hip.h -- C ABI of libillatio_hip.so: illatio's quantized matrix-product path
 * on one MI355X (gfx950).
 *
 * The library stands where the reference binds libcuda + NVRTC through SBCL's alien
 * interface (src/cuda.lisp).  Part 1 mirrors the driver calls that file makes, one
 * function each; part 2 is one typed entry point per kernel on the quantized
 * matrix-product path, named after the reference kernel it replaces and taking that
 * kernel's arguments in that kernel's order (grid and block shapes are chosen here, for
 * 64-lane waves, not by the caller); part 3 launches those kernels by name from the
 * reference's 8-byte-slot argument block, as its LAUNCH does.
 *
 * Conventions (src/cuda.lisp:34-57): every function returns an int, 0 on success,
 * otherwise a HIP error code whose text ilt_error_string gives; nothing aborts or
 * throws across the boundary.  Handles (streams, events) and device addresses are plain
 * 64-bit values.  The library owns no memory: it allocates and frees only on request.
 * Stream 0 is the device's default stream.
 *
 * Numerics.  Results are those of the reference's CPU path (src/tensor.lisp,
 * src/kquant.lisp, src/iquant.lisp, src/ds4f.lisp), not of its CUDA kernels: the
 * decode products and the int8 prefill products return the CPU path's bits.  So the
 * K-quant, IQ2_XXS and Q2_K kernels take Q8_K activations (ilt_quant_q8k), where the
 * reference's CUDA kernels take Q8_0-style blocks or floats.
 */
#ifndef ILLATIO_HIP_H
#define ILLATIO_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ILT_OK 0
#define ILT_NOT_READY 600 /* ilt_event_query: work before the event is still running */

/* Weight formats, numbered as GGUF numbers them (src/gguf.lisp:31-40). */
#define ILT_TYPE_Q8_0 8
#define ILT_TYPE_Q2_K 10
#define ILT_TYPE_Q4_K 12
#define ILT_TYPE_Q6_K 14
#define ILT_TYPE_IQ2_XXS 16

/* ---- 1. the device: what src/cuda.lisp asks of the driver --------------------------- */

/* The fields of the reference's CUDEV (src/cuda.lisp:61-70). arch is reported as 90 so
   that callers' (>= arch 80) tests choose the matrix-core paths (cuda-dense.lisp:218). */
typedef struct ilt_device_info {
  char name[256];
  int arch;
  uint64_t total_memory;
  int max_shared;      /* LDS bytes one workgroup may use */
  int numa_node;       /* -1 when unknown */
  int compute_units;
  int wave_size;
} ilt_device_info;

int ilt_init(void);                                     /* cuInit, cuda.lisp:76 */
int ilt_device_count(int* n);                           /* cuDeviceGetCount, :78 */
int ilt_device_get_info(int index, ilt_device_info* out); /* cuDeviceGet/GetName/GetAttribute/TotalMem, :100-135 */
int ilt_set_device(int index);                          /* cuCtxSetCurrent, :90-92 */
const char* ilt_error_string(int code);                 /* cuGetErrorString, :34-39 */

int ilt_stream_create(uint64_t* stream, unsigned flags); /* cuStreamCreate, :133, :380-386; flags 1 = non-blocking */
int ilt_stream_destroy(uint64_t stream);
int ilt_stream_sync(uint64_t stream);                   /* cuStreamSynchronize, :318-319, :414 */
int ilt_stream_wait_event(uint64_t stream, uint64_t event); /* cuStreamWaitEvent, :408-411 */
int ilt_event_create(uint64_t* event, unsigned flags);  /* cuEventCreate, :388-393; flags 2 = no timing */
int ilt_event_destroy(uint64_t event);                  /* cuEventDestroy, :395-396 */
int ilt_event_record(uint64_t event, uint64_t stream);  /* cuEventRecord, :398-399 */
int ilt_event_query(uint64_t event);                    /* cuEventQuery, :433-440: 0 done, ILT_NOT_READY pending */
int ilt_event_elapsed_ms(uint64_t start, uint64_t stop, float* ms); /* for measurement; no reference counterpart */

int ilt_malloc(uint64_t* dptr, uint64_t bytes);         /* cuMemAlloc, :239-249 (at least 256 bytes) */
int ilt_free(uint64_t dptr);                            /* cuMemFree, :261-267 */
int ilt_memset_async(uint64_t dptr, int byte, uint64_t bytes, uint64_t stream); /* cuMemsetD8Async, :269-273 */
int ilt_mem_info(uint64_t* free_bytes, uint64_t* total_bytes); /* cuMemGetInfo, :275-281 */
int ilt_memcpy_htod_async(uint64_t dst, const void* src, uint64_t bytes, uint64_t stream); /* :283-291, :416-421 */
int ilt_memcpy_dtoh_async(void* dst, uint64_t src, uint64_t bytes, uint64_t stream);       /* :302-309, :430-431 */
int ilt_memcpy_dtod_async(uint64_t dst, uint64_t src, uint64_t bytes, uint64_t stream);    /* :423-428 */
int ilt_host_alloc(uint64_t* hptr, uint64_t bytes, unsigned flags); /* cuMemHostAlloc, :371-378; flags 1 portable, 2 mapped */
int ilt_host_free(uint64_t hptr);                       /* cuMemFreeHost, :380 */
/* cuMemHostRegister / cuMemHostUnregister, :359-369: always hipErrorNotSupported (801) and no runtime call.
   Memory that already exists is not pinned here; take pinned memory from ilt_host_alloc instead. */
int ilt_host_register(void* p, uint64_t bytes, unsigned flags);
int ilt_host_unregister(void* p);

/* ---- 2. the kernels --------------------------------------------------------------------
 * Pointers are device addresses.  "|0" marks an argument that may be null.             */

/* Upload-time repacks (cuda-dense.lisp:87-100).
   repack_q8 (src/cuda/dense.cu:42): GGUF Q8_0 blocks -> int8 quants + f16 scales.
   repack_q6k (src/cuda/kquant.cu:195): the reference pads Q6_K blocks to 224 bytes for
   16-byte alignment; gfx950 only needs 4-byte alignment for full-rate 128-bit loads, so
   the device block is the 210 GGUF bytes plus 2 of padding (ILT_Q6K_DEVICE_BLOCK = 212;
   out needs 212*nblocks bytes, the reference's 224*nblocks is enough).  Every kernel that
   takes a Q6_K matrix takes this layout. */
#define ILT_Q6K_DEVICE_BLOCK 212
int ilt_repack_q8(uint64_t stream, const void* raw, void* qs, void* d, int64_t nblocks);
int ilt_repack_q6k(uint64_t stream, const void* raw, void* out, int64_t nblocks);

/* Activation quantizers.
   quant_q8 (dense.cu:84; CPU: quantize-q8!, tensor.lisp:245-262 with *q8-f16-scale* T):
     blocks of 32, scale stored rounded through fp16; xsum|0 gets each block's integer sum.
   d4_quant (ds4f.cu:35; *q8-f16-scale* NIL, ds4f.lisp:1052-1053): the scale kept a float.
   quant_q8k (no CUDA counterpart; CPU: quantize-q8k!, kquant.lisp:130-167): blocks of
     256, xd one float per block, bsums one int32 per 16 quants. */
int ilt_quant_q8(uint64_t stream, const float* x, int8_t* xq, float* xs, int32_t* xsum, int64_t nblocks);
int ilt_d4_quant(uint64_t stream, const float* x, int8_t* xq, float* xs, int nblocks);
int ilt_quant_q8k(uint64_t stream, const float* x, int8_t* xq, float* xd, int32_t* bsums, int64_t nblocks);

/* Decode products, y[r] = W[r].x (+ bias[r]); acc: y += that.
   mv_q8 (dense.cu:194; CPU: matvec!, tensor.lisp:321-352): W repacked by ilt_repack_q8.
   mv_k (kquant.cu:169; CPU: q4k-row-dot / q6k-row-dot, kquant.lisp:171-236): type 0 Q4_K,
     2 Q6_K (kquant-code, cuda-dense.lisp:18-20); w the GGUF blocks; xq/xd/bsums from
     ilt_quant_q8k.
   mv_q8_3 (dense.cu:210): three products sharing x in one call.
   d4_mvq8 (ds4f.cu:50): Q8_0, row r against the activations of group r/group_rows. */
int ilt_mv_q8(uint64_t stream, const int8_t* wq, const uint16_t* wd, const int8_t* xq, const float* xs, float* out,
              const float* bias, int rows, int cols, int acc);
int ilt_mv_q8_3(uint64_t stream, const int8_t* q0, const uint16_t* d0, const int8_t* q1, const uint16_t* d1,
                const int8_t* q2, const uint16_t* d2, const int8_t* xq, const float* xs, float* o0, float* o1, float* o2,
                const float* b0, const float* b1, const float* b2, int r0, int r1, int r2, int cols);
int ilt_mv_k(uint64_t stream, int type, const void* w, const int8_t* xq, const float* xd, const int32_t* bsums, float* out,
             const float* bias, int rows, int cols, int acc);
int ilt_d4_mvq8(uint64_t stream, int rows, int cols, int group_rows, const int8_t* wq, const uint16_t* wd,
                const int8_t* xq, const float* xs, float* y);
/* d4_mvq8n (ds4f.cu:66; cuda-ds4f-prefill.lisp:89): d4_mvq8 for ntok <= 9 tokens (a speculative
   step's): token t's quantized input at xq + t*x_tstride (its scales at xs + t*x_tstride/32, the
   row's group g at + g*cols within it), its output at y + t*y_tstride; each token's sums are
   decode's. */
int ilt_d4_mvq8n(uint64_t stream, int rows, int cols, int group_rows, int ntok, int x_tstride, int y_tstride, const int8_t* wq,
                 const uint16_t* wd, const int8_t* xq, const float* xs, float* y);

/* Gate and up in one launch ending in swiglu! (model.lisp:364-378): out[r] =
   (g / (1 + exp(-g))) * u with g = gate[r].x, u = up[r].x, each the decode product's bits.
   mv_q8_glu (dense.cu:230), mv_k_glu (kquant.cu:183). */
int ilt_mv_q8_glu(uint64_t stream, const int8_t* gq, const uint16_t* gd, const int8_t* uq, const uint16_t* ud,
                  const int8_t* xq, const float* xs, float* out, int rows, int cols);
int ilt_mv_k_glu(uint64_t stream, int gtype, const void* gw, int utype, const void* uw, const int8_t* xq, const float* xd,
                 const int32_t* bsums, float* out, int rows, int cols);

/* Up to four matrices that share x in one launch (the reference has this for Q8_0 only,
   mv_q8_3; its K-quant QKV is three launches, cuda-dense.lisp:321-323).  All Q8_0, or any mix
   of Q4_K and Q6_K.  The activations come quantized (xq, xs, bsums as for mv_q8 / mv_k), or,
   with xf non-null, as floats that every workgroup quantizes for itself exactly as
   quantize-q8! (scale through fp16 when f16_scale) / quantize-q8k! would: the product then
   needs no quantizer launch before it.  glu: descs[0] = gate, descs[1] = up, result into
   descs[0].y.  No counterpart in the reference beyond mv_q8_3. */
typedef struct ilt_mv_desc {
  int gguf_type;          /* ILT_TYPE_Q8_0, ILT_TYPE_Q4_K or ILT_TYPE_Q6_K */
  int rows;
  const void* w;          /* Q8_0: int8 quants (repacked) */
  const uint16_t* wd;     /* Q8_0: f16 scales; else null */
  float* y;
  const float* bias;      /* or null */
} ilt_mv_desc;
int ilt_mv_multi(uint64_t stream, int nmat, const ilt_mv_desc* descs, int cols, const int8_t* xq, const float* xs,
                 const int32_t* bsums, const float* xf, int f16_scale, int acc, int glu);

/* rmsnorm! (model.lisp:205-216) and the quantizer in one launch, a row of dim floats a
   workgroup, n rows: out = (x * scale) * w with scale = 1 / sqrt(float(sum/dim + eps)), the
   squares rounded to floats and added in double.  h (unless null) gets the floats.
   rmsnorm_q8 (dense.cu:144-160; cuda-dense.lisp:260-264): Q8_0 blocks as quant_q8 makes them,
     xsum|0 their sums; launched by name, rows = grid y.
   rmsnorm_q8k: Q8_K blocks as quant_q8k makes them (no CUDA counterpart: the reference's
     K-quant kernels take the floats).
   ilt_mv_multi_norm: ilt_mv_multi on the floats x, normalized like this by each workgroup
     before it quantizes them: norm, quantizer and products in one launch (the reference:
     rmsnorm_q8 then mv_*, cuda-dense.lisp:401-403, 415-417).
   The bits are the CPU's although the squares are added in parallel: the kernel checks that
   no double within the reordering's error bound of its sum rounds to another float, and
   otherwise (or always, with exact_order 1) adds them again one after another. */
int ilt_rmsnorm_q8(uint64_t stream, const float* x, const float* w, float* h, int8_t* xq, float* xs, int32_t* xsum, int dim,
                   float eps, int n, int exact_order);
int ilt_rmsnorm_q8k(uint64_t stream, const float* x, const float* w, float* h, int8_t* xq, float* xd, int32_t* bsums, int dim,
                    float eps, int n, int exact_order);
int ilt_mv_multi_norm(uint64_t stream, int nmat, const ilt_mv_desc* descs, int cols, const float* x, const float* norm_w,
                      float eps, int exact_order, int f16_scale, int glu);

/* ilt_mv_multi (float activations x; norm_w null) or ilt_mv_multi_norm that also reads the rows of the caller's NEXT
   product ahead while it runs: the next product is only described (next_nmat matrices of next_cols columns, next_glu
   as glu), not launched.  The waves that stage the activations, idle once that is done, touch the cache lines the
   next launch's workgroups on their die will stream, so that those come from L2 instead of HBM.  Worth it where this
   launch is long against the next matrix (a layer's gate/up before its down: 9.0 instead of 9.8 us); results are
   those of the plain calls.  Where either product does not take the streamed variant the call is the plain one.  No
   counterpart in the reference. */
int ilt_mv_multi_ahead(uint64_t stream, int nmat, const ilt_mv_desc* descs, int cols, const float* x, const float* norm_w, float eps,
                       int f16_scale, int acc, int glu, int next_nmat, const ilt_mv_desc* next_descs, int next_cols, int next_glu);

/* Diagnostic: how many decode products this process has launched as the streamed variant (the
   one that sends every wave's rows to LDS at once; chosen by shape for Q8_0 / Q4_K / Q6_K products of
   half a megabyte and more whose share fits a CU's LDS).  No counterpart in the reference. */
uint64_t ilt_streamed_launches(void);

/* The indexed expert products (ds4f.cu:769, 837; CPU: iq2xxs-row-dot, q2k-row-dot,
   iquant.lisp:126-215).  For each z < nz: W = the nrows x ncols matrix at ptrs[z] + add
   (row_bytes apart), x = the Q8_K activations at element z*x_stride, y = dst + z*y_stride.
   The reference's grid z (cuda-ds4f.lisp:937-941) is nz here. */
int ilt_d4_mv_iq2_xxs(uint64_t stream, int ncols, int nrows, int row_bytes, int64_t add, int x_stride, int y_stride,
                      const uint64_t* ptrs, int nz, const int8_t* xq, const float* xd, float* dst);
int ilt_d4_mv_q2_k(uint64_t stream, int ncols, int nrows, int row_bytes, int64_t add, int x_stride, int y_stride,
                   const uint64_t* ptrs, int nz, const int8_t* xq, const float* xd, const int32_t* bsums, float* dst);
/* The same two with the reference kernels' own arguments (ds4f.cu:762-772, 837-840; callers: DK-FFN-TAIL,
   cuda-ds4f.lisp:937-941, and DK-FFN-SMALL, cuda-ds4f-spec.lisp:83-88): x = rows of floats, which the kernel
   quantizes as quantize-act! does (kquant.lisp:511-514), so y has the CPU path's bits.
   srcs (or null): for each z with srcs[z] set, the matrix's nrows * row_bytes bytes are first copied from
     srcs[z] + add (host memory the device can read) to ptrs[z] + add, the expert's slot (d4_read_through,
     ds4f.cu:742-760), as a launch of its own in front of the product.
   counts, bases (both or neither): expert z works on rows bases[z] .. bases[z] + counts[z] - 1 of x and y
     (x_stride / y_stride floats apart), its matrix read from memory once and from the cache after; an expert
     with a count of 0 does nothing.  Without them expert z works on row z (x_stride 0: all on row 0). */
int ilt_d4_mv_rows_iq2_xxs(uint64_t stream, int ncols, int nrows, int row_bytes, int64_t add, int x_stride, int y_stride,
                           const uint64_t* ptrs, const uint64_t* srcs, int nz, const float* x, float* y,
                           const uint32_t* counts, const uint32_t* bases);
int ilt_d4_mv_rows_q2_k(uint64_t stream, int ncols, int nrows, int row_bytes, int64_t add, int x_stride, int y_stride,
                        const uint64_t* ptrs, const uint64_t* srcs, int nz, const float* x, float* y,
                        const uint32_t* counts, const uint32_t* bases);

/* The decode step of d4-routed! / d4-shared! (ds4f.lisp:994-1048; DK-FFN-TAIL, cuda-ds4f.lisp:
   908-956) in fewer launches, with the same bits: the activations come as floats and every
   workgroup quantizes them as quantize-q8k! (experts) or quantize-q8! with a float scale
   (shared expert) does, so no quantizer launch precedes the product.
   With sel given, ptrs is the table of all the expert slots and slot z of the launch is expert
   sel[z] -- d4_route's output on the device, so that no routing result goes through the host
   (the reference's decode path syncs and routes on the CPU in every layer,
   cuda-ds4f.lisp:991-999); with sel null, ptrs[z] is slot z's address as in d4_mv_*.
   d4_mv_glu_iq2_xxs: for each z < nz, gate at ptrs[z] + add_gate, up at ptrs[z] + add_up,
     x at element z*x_stride (0: one x for all), mid[z*y_stride + r] = (silu(g)*u) * wts[z]
     with g = min(g, clamp), u in [-clamp, clamp] when clamp > 1e-6 (d4_swiglu_w's formula;
     wts may be null).  Replaces quant + d4_mv_iq2_xxs over 2k matrices + d4_swiglu_w.
   d4_mv_q2_k_f32: d4_mv_q2_k on float activations (each z's own, x_stride apart).
   d4_mvq8_glu: the shared expert's gate and up (Q8_0, repacked) on float x, the same gated
     activation with weight 1 into mid.  Its down projection is ilt_mv_multi with xf = mid
     and f16_scale 0. */
int ilt_d4_mv_glu_iq2_xxs(uint64_t stream, int ncols, int nrows, int row_bytes, int64_t add_gate, int64_t add_up,
                          int x_stride, int y_stride, const uint64_t* ptrs, const uint32_t* sel, int nz, const float* x,
                          const float* wts, float clamp, float* mid);
int ilt_d4_mv_q2_k_f32(uint64_t stream, int ncols, int nrows, int row_bytes, int64_t add, int x_stride, int y_stride,
                       const uint64_t* ptrs, const uint32_t* sel, int nz, const float* x, float* dst);
int ilt_d4_mvq8_glu(uint64_t stream, int rows, int cols, const int8_t* gq, const uint16_t* gd, const int8_t* uq,
                    const uint16_t* ud, const float* x, float clamp, float* mid);

/* One token's FFN past the router in one call: DK-FFN-HEAD's shared expert and DK-FFN-TAIL
   (cuda-ds4f.lisp:883-956) with the routing left on the device (the reference copies the
   logits out, waits and routes on the CPU in every layer, :991-999).  Four launches on stream:
   d4_mvq8_glu (one of whose waves does d4_route's work while the rows stream in: up to 256 experts and a
   shared expert large enough for the streamed product, else d4_route is a launch of its own),
   d4_mv_glu_iq2_xxs and d4_mv_q2_k_f32 indexed by the routing's sel, and last the shared expert's down
   product, which adds the routed experts' rows in slot order and then its own as it stores them (d4_moe_sum's
   arithmetic; up to 8 slots and a matrix large enough for the streamed product, else the product and d4_moe_sum
   are two launches); moe[d] = the nu routed experts' rows in slot order + the shared
   expert's, with the CPU path's bits (d4-ffn without HC, ds4f.lisp:980-992).  Nothing is
   allocated, freed or waited for.  The intermediate results (sel, weights, the two gated
   activations, the shared expert's row, one down row per slot) live in ws, 256-byte aligned,
   ilt_d4_ffn_step_workspace(nu, d, ff) bytes of device memory that the caller owns (0 for
   sizes the step does not take: nu <= 64, ne <= 1024, d and ff multiples of 256).
   slots: the table of all ne expert slots, each gate | up | down with gate_bytes =
   ff * (d/256) * 66; the shared expert's three Q8_0 matrices repacked by ilt_repack_q8.
   bias may be null.  Calls on one stream that share ws run one after another. */
typedef struct ilt_ffn_step_weights {
  const uint64_t* slots;
  int64_t gate_bytes;
  const int8_t* sgate_q; const uint16_t* sgate_d;
  const int8_t* sup_q; const uint16_t* sup_d;
  const int8_t* sdown_q; const uint16_t* sdown_d;
} ilt_ffn_step_weights;
uint64_t ilt_d4_ffn_step_workspace(int nu, int d, int ff);
int ilt_d4_ffn_step(uint64_t stream, void* ws, uint64_t ws_bytes, int ne, int nu, int d, int ff, float scale, float clamp,
                    const ilt_ffn_step_weights* wt, const float* logits, const float* bias, const float* x, float* moe);
/* Measurement only (no counterpart in the reference): the calling thread's next ilt_d4_ffn_step calls record
   events[i] (ilt_event_create's handles, n <= 8) on the stream before their launch i and the one after their last
   launch behind it, so that a bench can time the step's launches as the step queues them; n = 0 switches it off. */
int ilt_d4_ffn_step_events(const uint64_t* events, int n);

/* ilt_d4_ffn_step without a workspace and without any allocation.  No counterpart in the
   reference: it is for callers that cannot allocate device memory or keep a workspace alive --
   code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  The
   intermediate results live in a device array inside the library, ilt_d4_ffn_step_noalloc_max_bytes()
   = 1 MiB per GPU, held until the process ends; a step whose ilt_d4_ffn_step_workspace(nu, d, ff)
   is larger returns hipErrorInvalidValue (1) and does nothing (config 4's step, nu 6, d 4096,
   ff 2048, takes 172,544 bytes).  The call makes no hipMalloc, hipFree or other allocating call;
   the array's address is asked of the runtime on the first call on each device.  Every call on a
   GPU shares that GPU's array: calls on one stream run one after another and are safe; calls that
   overlap on one GPU (two streams, two threads) race on it.  Same results as ilt_d4_ffn_step. */
uint64_t ilt_d4_ffn_step_noalloc_max_bytes(void);
int ilt_d4_ffn_step_noalloc(uint64_t stream, int ne, int nu, int d, int ff, float scale, float clamp,
                            const ilt_ffn_step_weights* wt, const float* logits, const float* bias, const float* x, float* moe);

/* Rows as floats (dense.cu:53 embed_q8, kquant.cu:202 embed_k; CPU: q8mat-row!, kmat-row!,
   iq2xxs-row-floats!, q2k-row-floats!): out[n] = row tokens[n] (row n when tokens is null)
   of W, bit-exact.  ilt_dequant_rows takes a GGUF type (any of the five; Q8_0 repacked,
   wd its scales). */
int ilt_embed_q8(uint64_t stream, const int8_t* qs, const uint16_t* d, const int32_t* tokens, float* out, int cols, int n);
int ilt_embed_k(uint64_t stream, int type, const void* w, const int32_t* tokens, float* out, int cols, int n);
int ilt_dequant_rows(uint64_t stream, int gguf_type, const void* w, const uint16_t* wd, const int32_t* rows_idx,
                     int64_t nrows, int cols, float* out);

/* The expert path's small kernels (ds4f.cu:645, 902; ds4f_chunk.cu:393-508; CPU:
   d4-route, d4-routed!, ds4f.lisp:950-1037, 1169-1239).  d4_route routes ntok tokens
   (the reference's grid x).  hash 0: top-nu; 1: tid2eid table.  has_bias 0/1/2 as there. */
int ilt_d4_route(uint64_t stream, int ne, int nu, int hash, float scale, int has_bias, const float* logits,
                 const float* bias, const int32_t* tid2eid, const uint32_t* tokens, uint32_t* sel, float* wout, int ntok);
int ilt_d4_group_zero(uint64_t stream, int ne, uint32_t* counts);
int ilt_d4_group_count(uint64_t stream, int n, int ne, int nu, const uint32_t* sel, uint32_t* counts, uint32_t* rank);
int ilt_d4_group_scan(uint64_t stream, int n, int ne, int nu, const uint32_t* counts, uint32_t* bases);
int ilt_d4_group_scatter(uint64_t stream, int n, int ne, int nu, const uint32_t* sel, const uint32_t* rank,
                         const uint32_t* bases, const float* w, uint32_t* rmap, uint32_t* smap, float* wrow);
int ilt_d4_gather_rows(uint64_t stream, int d, int nrows, const float* src, const uint32_t* map, float* x);
/* The expert of every grouped row: rexp[smap[i]] = sel[i] for the n (token, slot) pairs.  With it the indexed
   expert kernels (sel = rexp over the table of all slots, one launch slot a grouped row) take an expert's rows
   one after another, so its matrices come from memory once for all its tokens and from the cache after -- what
   the counts / bases arguments of the reference's d4_mv_* give a short pass (ds4f.cu:762-772,
   cuda-ds4f-spec.lisp:83-88), with the routing and the grouping left on the device. */
int ilt_d4_rows_expert(uint64_t stream, int n, const uint32_t* sel, const uint32_t* smap, uint32_t* rexp);
int ilt_d4_swiglu_w(uint64_t stream, int n, int ff, float clamp, const float* g, const float* u, const float* w,
                    float* mid, int8_t* xq, float* xs);
int ilt_d4_moe_sum(uint64_t stream, int d, int k, const float* down, const float* shared_, float* moe, const uint32_t* perm);
int ilt_d4_moe_sum_rows(uint64_t stream, int d, int nu, int ntok, const float* down, const uint32_t* map,
                        const float* shared_, float* moe);

/* Between the products of a dense decoder layer: what the forward harness (illatio_amd/model.py, the
   reference's cuda-forward-n, cuda-dense.lisp:380-432) runs besides them.  The floats are the CPU path's
   (model.lisp:205-334, 364-378), sum for sum, so a token's logits have the CPU path's bits.
   qk_rope (dense.cu:318-362, the same arguments; tokens = grid y): the head norms where qn / kn are given,
     RoPE from rope (a position's rd/2 cosines then rd/2 sines; rope-table, model.lisp:218-231, made by the
     host), K and V of token t into the caches at position pos0 + t.
   attn_rows: attend-head! for every query head of ntok tokens, token t over positions 0 .. pos0 + t; scores
     in F32-DOT16's order, the softmax's sum in double, the values added position after position.  It stands
     where the reference launches attn_decode + attn_merge / attn_prefill (dense.cu:376-727), whose partial
     sums meet in another order.  scratch: ntok * nh * ((pos0 + ntok + 3) & ~3) floats of the caller's for the raw
     scores (contexts up to 8192 positions: the scores over many workgroups, for several tokens their softmax, then
     the values -- a chunk of tokens with heads of 64 or 128: 64 tokens x 64 positions of scores and 32 tokens x a
     head of values a workgroup, sixteen results a thread; pointers 16-byte aligned for those), or null (one launch,
     a workgroup a head, any context that fits LDS).
   swiglu (dense.cu:307): swiglu! on n values, a = (a / (1 + e^-a)) * b, the exponential through double. */
/* The table qk_rope takes, for positions pos0 .. pos0 + n - 1, written to host memory (n * head_dim floats). */
int ilt_rope_table(int head_dim, int pos0, int n, float base, float* out);
int ilt_qk_rope(uint64_t stream, float* q, float* k, const float* v, const float* qn, const float* kn, const float* rope, float* kc,
                float* vc, int nh, int nkv, int hd, int rd, int pos0, float eps, int neox, int ntok);
int ilt_attn_rows(uint64_t stream, const float* q, const float* kc, const float* vc, float* out, int nh, int nkv, int hd, int pos0, int ntok,
                  float* scratch);
/* ilt_qk_rope and ilt_attn_rows of one token at position pos (< 8192) in fewer launches.  Up to position 1023 with
   heads of 64 or 128: one launch, a workgroup a (query head, 16 columns of the values), each norming and turning its
   head and the token's key itself; where a head's workgroups run on one die (nh a multiple of 8) each takes an eighth
   of the head's scores and they exchange them inside the launch through a buffer of the library's (scratch is not
   touched), else each takes all of them.  Launches of it that overlap on one GPU make each other give that exchange up
   (correct, slower).  Otherwise two: the
   launch that takes the scores norms and turns the query heads and the token's key and writes the caches' rows at
   pos.  Either way out is what ilt_attn_rows gives after ilt_qk_rope, bit for bit; q and k are left as they came
   (not normed, not turned).  scratch: nh * ((pos + 4) & ~3) floats.  nctx: the rows kc and vc hold; pos at or past
   it is refused (the caches' rows at pos are written).  Each stream's launches exchange through a buffer of their
   own (the first eight streams of a device; the rest share one); ilt_attn_giveups counts the workgroups that gave
   an exchange up since the library was loaded (a diagnostic: such a launch is correct and about 200 us longer). */
int ilt_attn_step(uint64_t stream, const float* q, const float* k, const float* v, const float* qn, const float* kn, const float* rope, float* kc,
                  float* vc, float* out, int nh, int nkv, int hd, int rd, int pos, float eps, int neox, float* scratch, int nctx);
int ilt_attn_giveups(uint64_t* out);

/* One token through the whole dense decoder in one call: what the host loop of cuda-forward-n queues for one
   token (cuda-dense.lisp:380-432; the CPU's forward-1, model.lisp:396-462) -- embedding row, then per layer the
   Q/K/V products with the norm inside, ilt_attn_step, wo onto the residual, gate/up with the norm and the gated
   activation inside, down onto the residual, and (want_logits) the output norm and head: 5 launches a layer + 2 while
   the context is at most 1,024 positions, 6 beyond.
   The structs are read on the host during the call; every pointer in them is device memory but `layers`.
   Matrices as dense uploads hold them (Q8_0 split into quants and scales, Q6_K in 212-byte blocks).  pos < 8192
   (the attention's scratch), the caches hold at least pos + 1 positions, rope at least (pos + 1) * rd floats.
   token: one id, on the device.  The results are those of the single calls, bit for bit. */
/* ARGMAX (model.lisp:464-468) on the device: out[0] = the index of the first of the greatest of v's n floats (a NaN
   is never greater; a NaN in front stays the best, as in the reference's scan).  No counterpart among the
   reference's kernels: its host picks the token (cuda-dense.lisp:428-430); with this a greedy decode queues token
   after token without the logits' trip to the host (ilt_dense_decode takes its token from device memory).  scratch:
   2048 bytes of the caller's, 8-byte aligned (128 workgroups leave their bests there for a second launch), or null
   (one workgroup reads everything: several times slower on a vocabulary's logits). */
int ilt_argmax(uint64_t stream, const float* v, int n, int32_t* out, void* scratch);
typedef struct ilt_dense_mat { int gguf_type, rows, cols; const void* w; const uint16_t* wd; } ilt_dense_mat;
typedef struct ilt_dense_layer {
  const float *attn_norm, *q_norm, *k_norm, *ffn_norm;        /* q_norm, k_norm: null when the model has no head norms */
  ilt_dense_mat wq, wk, wv, wo, gate, up, down;
  float *kc, *vc;                                             /* this layer's caches, nkv * hd floats a position */
  const float *bq, *bk, *bv;                                  /* Q, K and V's biases, or null (qwen2 has them) */
} ilt_dense_layer;
typedef struct ilt_dense_model {
  int nl, d, ffn, nh, nkv, hd, rd, neox;
  int nctx;                                                   /* rows of every layer's kc and vc: a token at or past it is refused */
  float eps;
  ilt_dense_mat embd, output;
  const float *output_norm, *rope;
  const ilt_dense_layer* layers;                              /* nl of them, host memory */
  float *x, *q, *k, *v, *att, *fa, *scores, *logits;          /* d, nh*hd, nkv*hd, nkv*hd, nh*hd, ffn, nh*((pos+4)&~3), vocab floats */
} ilt_dense_model;
int ilt_dense_decode(uint64_t stream, const ilt_dense_model* m, const int32_t* token, int pos, int want_logits);
int ilt_swiglu(uint64_t stream, float* a, const float* b, int64_t n);
/* ilt_swiglu followed by ilt_quant_q8k in one launch, for a prompt chunk whose gated activations only the down product
   reads (GLU-MUL's "swiglu" launch, cuda-dense.lisp:338-339, and the quantizing launch that follows it in
   CUDA-FORWARD-N, cuda-dense.lisp:417-418): the blocks are those the two leave, the floats are not written.  gate, up: nblocks * 256 floats, 16-byte aligned. */
int ilt_swiglu_quant_q8k(uint64_t stream, const float* gate, const float* up, int8_t* xq, float* xd, int32_t* bsums, int64_t nblocks);

/* Prefill products on the int8 matrix cores, y[t*rows + r] = W[r].x_t (+ bias[r]) for n
   tokens, each (row, token) with the decode kernel's bits (CPU: MATMUL!, batch.lisp:128-205,
   "bit-identical to feeding the tokens one at a time", :10-12).
   mm_q8 (dense.cu:251, 642, 884 mm_q8 / mm_q8_mma / mm_q8_mma2): W repacked by ilt_repack_q8,
     activations from ilt_quant_q8 (or ilt_d4_quant), token t's at t*cols.
   mm_k (kquant.cu:223, 458-466 mm_k / mm_q4k_mma / mm_q6k_mma): type 0 Q4_K, 2 Q6_K;
     activations from ilt_quant_q8k.
   d4_mm_id_* (ds4f_mm.cu:256-257): the grouped expert product.  Expert z's matrix is at
     ptrs[z] + add; it multiplies rows bases[z] .. bases[z]+counts[z]-1 of the gathered,
     Q8_K-quantized activations (xq/xd/bsums, ncols apart) into the same rows of y (nrows
     apart).  ne experts (at most 256), total_rows = the sum of counts. */
int ilt_mm_q8(uint64_t stream, const int8_t* wq, const uint16_t* wd, const int8_t* xq, const float* xs, float* y,
              const float* bias, int rows, int cols, int n, int acc);
int ilt_mm_k(uint64_t stream, int type, const void* w, const int8_t* xq, const float* xd, const int32_t* bsums, float* y,
             const float* bias, int rows, int cols, int n, int acc);
/* Up to three K-quant matrices of one type on the same tokens in one launch -- for Q4_K / Q6_K what mm_q8_mma2 is
   for Q8_0 (cuda-dense.lisp:250-258: cmat-mul-n; same argument pattern: (w, y, bias, rows) three times, then the
   activations): the row tiles of matrices too small to fill the chip on their own share a launch (Q/K/V, gate and
   up of a prompt's chunk).  type: the reference's kquant code (0 Q4_K, 2 Q6_K).  A matrix of no rows or a null one
   takes no part.  The results are ilt_mm_k's, bit for bit. */
int ilt_mm_k_n(uint64_t stream, int type, const void* w0, float* y0, const float* b0, int rows0, const void* w1, float* y1, const float* b1,
               int rows1, const void* w2, float* y2, const float* b2, int rows2, const int8_t* xq, const float* xd, const int32_t* bsums,
               int cols, int n, int acc);
/* d4_mm_<format> (ds4f_mm.cu:252-255; dk-mm, cuda-ds4f-prefill.lisp:65-68): one matrix on a chunk of
   ntok tokens' FLOAT activations, y[t*y_stride + r] = W[r] . x[t*x_stride ..].  The reference's kernels
   round weights and activations to halves; these give the CPU path's results:
   q8_0 (the shared expert and the attention projections of a chunk; w, wd as ilt_repack_q8 leaves them,
     row_bytes 0 or ncols): every token quantized by quantize-q8! with the scale kept a float, then
     ilt_mm_q8's exact product -- q8mv!'s bits per token (ds4f.lisp:294-297, 1039-1048);
   q2_k, iq2_xxs: quantize-q8k!, then the exact product (the row dots of iquant.lisp:126-215);
   f16 (the router, ds4f.lisp:1175 f32mm!): floats, every dot added up in F32-DOT16's order
     (tensor.lisp:370-378), bit for bit; ncols a multiple of 16.
   x_stride >= ncols and y_stride >= nrows: the reference passes them for the grouped attention output product,
   one call a group on a slice of each token's heads into a slice of its low row, w and wd at offsets into
   their arrays (cuda-ds4f-prefill.lisp:277-281); the K formats want x_stride a multiple of 4.
   The quantized formats keep their quantized activations in a buffer inside the library, one per (GPU, stream), that
   grows to the largest chunk seen and is kept until the process ends: calls that overlap on one GPU are on different
   streams and do not share a buffer (sixteen buffers at most; a call on a seventeenth stream returns
   hipErrorOutOfMemory).  Growing waits for the stream, frees and allocates, and is refused while the stream is being
   captured (hipErrorStreamCaptureUnsupported): ilt_d4_mm_reserve(ntok, ncols) sizes the current GPU's buffers -- those
   there are, and every one made later -- for chunks of up to ntok tokens of ncols columns, and
   ilt_d4_mm_reserve_stream makes and sizes one stream's at once; calls within that size allocate nothing.  Neither has a
   counterpart in the reference (its kernels take the float rows as they are). */
int ilt_d4_mm_reserve(int ntok, int ncols);
int ilt_d4_mm_reserve_stream(uint64_t stream, int ntok, int ncols);
int ilt_d4_mm_q8_0(uint64_t stream, int ncols, int nrows, int ntok, int row_bytes, int x_stride, int y_stride, const int8_t* w,
                   const uint16_t* wd, const float* x, float* y);
int ilt_d4_mm_f16(uint64_t stream, int ncols, int nrows, int ntok, int row_bytes, int x_stride, int y_stride, const uint16_t* w,
                  const float* x, float* y);
int ilt_d4_mm_q2_k(uint64_t stream, int ncols, int nrows, int ntok, int row_bytes, int x_stride, int y_stride, const void* w,
                   const float* x, float* y);
int ilt_d4_mm_iq2_xxs(uint64_t stream, int ncols, int nrows, int ntok, int row_bytes, int x_stride, int y_stride, const void* w,
                      const float* x, float* y);

/* mm_q8_mma2 (dense.cu:884; cuda-dense.lisp:215, 255-258): up to three Q8_0 matrices on the same
   quantized tokens (Q, K, V of a prefill chunk) in one call; a matrix of no rows takes no part.
   Each is ilt_mm_q8's product. */
int ilt_mm_q8_mma2(uint64_t stream, const int8_t* w0, const uint16_t* d0, float* y0, const float* b0, int rows0, const int8_t* w1,
                   const uint16_t* d1, float* y1, const float* b1, int rows1, const int8_t* w2, const uint16_t* d2, float* y2,
                   const float* b2, int rows2, const int8_t* xq, const float* xs, int cols, int n, int acc);
int ilt_d4_mm_id_iq2_xxs(uint64_t stream, int ncols, int nrows, int row_bytes, int64_t add, const uint64_t* ptrs,
                         const uint32_t* counts, const uint32_t* bases, int ne, int64_t total_rows,
                         const int8_t* xq, const float* xd, float* y);
int ilt_d4_mm_id_q2_k(uint64_t stream, int ncols, int nrows, int row_bytes, int64_t add, const uint64_t* ptrs,
                      const uint32_t* counts, const uint32_t* bases, int ne, int64_t total_rows,
                      const int8_t* xq, const float* xd, const int32_t* bsums, float* y);

/* The same products on the bf16 matrix cores: W is dequantized to bf16 value by value as the
   CPU's *-row-floats! do (kquant.lisp:466-497 Q4_K, :530-569 Q6_K, :411-445 Q2_K;
   iquant.lisp:161-230 IQ2_XXS), the activations are floats rounded to bf16 by cvt_bf16
   (in place of an activation quantizer), the accumulation is fp32.  This is the faster
   prefill path; its results are within 2e-2 (relative to the largest output) of the CPU
   path, not bit-exact.
   cvt_bf16: n floats (a multiple of 8, 16-byte aligned) to n bf16.
   mm_k_bf16: gguf_type 10 Q2_K, 12 Q4_K, 14 Q6_K (212-byte device blocks of
     ilt_repack_q6k), 16 IQ2_XXS; xb is n tokens of cols bf16, 16-byte aligned;
     y[t*rows + r] (+= when acc, + bias[r]).  The matrix is at most 4 GiB.
   dequant_bf16 + cvt_bf16_slabs + mm_bf16: the same product in two passes, for thousands of
     tokens or a matrix multiplied again and again.  dequant_bf16 writes the matrix as bf16
     (each weight the value mm_k_bf16 rounds in its loop), cvt_bf16_slabs the activations;
     mm_bf16 multiplies the two copies and returns mm_k_bf16's numbers (the same products
     added in the same order).  Both copies are laid out in slabs -- the 32 columns
     32s..32s+31 of rows 128g..128g+127 are 8 KB in one piece at ((g * cols/32) + s) * 8192,
     row r of the group at 64 * (r % 128) -- with the rows (tokens) padded with zeros to a
     multiple of 256: a copy is 2 * cols * ceil(rows / 256) * 256 bytes, 16-byte aligned;
     cols a multiple of 128 (dequant_bf16: of 256).  With memory to spare the matrix's copy can
     stay resident beside the quantized matrix that decode reads.
   d4_mm_id_bf16: the grouped expert product of ds4f_mm.cu:256-257, same gguf_type codes, other
     arguments as d4_mm_id_*.  Row i of the groups multiplies xb's row rmap[i] (d4_group_scatter's
     row -> token map: the tokens' activations are read in place, no gathered copy), or row i
     itself when rmap is null.
   d4_swiglu_w_bf16: d4_swiglu_w's gated activation rounded to bf16 (ff a multiple of 8).
   d4_mm_id_glu_bf16: the gate and up products of d4_mm_id_bf16 (IQ2_XXS; up's matrix at
     ptrs[z] + add_up, add_up >= add_gate) and d4_swiglu_w_bf16 in one launch: mid[i][r] for the
     groups' row i and r < nrows (a multiple of 128), the bits the three launches give. */
int ilt_cvt_bf16(uint64_t stream, const float* x, uint16_t* xb, int64_t n);
/* The bf16 products on the activations the CPU path multiplies with: quantize-q8k!'s quants times their block
   scales (kquant.lisp:117-167; what q4k-row-dot and the others see of x), rounded to bf16, n tokens of cols (a
   multiple of 256) -- as rows for mm_k_bf16 (slabs 0) or in cvt_bf16_slabs' layout for mm_bf16 (slabs 1).  With
   these the bf16 path shares the CPU path's rounding of the activations to int8 blocks and differs from it by the
   bf16 roundings alone.  No counterpart in the reference's CUDA path (its mm_*_mma kernels multiply integer
   operands, kquant.cu:300-304). */
int ilt_q8k_bf16(uint64_t stream, const int8_t* xq, const float* xd, uint16_t* xb, int n, int cols, int slabs);
int ilt_mm_k_bf16(uint64_t stream, int gguf_type, const void* w, const uint16_t* xb, float* y, const float* bias,
                  int rows, int cols, int n, int acc);
int ilt_cvt_bf16_slabs(uint64_t stream, const float* x, uint16_t* xs, int n, int cols);
int ilt_dequant_bf16(uint64_t stream, int gguf_type, const void* w, uint16_t* wb, int rows, int cols);
int ilt_mm_bf16(uint64_t stream, const uint16_t* wb, const uint16_t* xb, float* y, const float* bias, int rows, int cols, int n,
                int acc);
/* The exact product in two passes (no counterpart in the reference: its GPU prefill does not have the CPU
   path's bits): planes_i8 writes a Q6_K matrix as the two int8 planes of scale * (quant - 32) (slabs of 128
   rows x 64 columns: ceil(rows/128)*128*cols bytes each) and d per row and super-block as floats (rows * cols / 256); mm_i8_planes is mm_k from
   those and the Q8_K quants and scales (it adds the quants up itself: no sums of 16), bit for bit, for a matrix multiplied again and again or by thousands of tokens. */
int ilt_planes_i8(uint64_t stream, int gguf_type, const void* w, int8_t* wh, int8_t* wl, float* wdf, int rows, int cols);
int ilt_mm_i8_planes(uint64_t stream, const int8_t* wh, const int8_t* wl, const float* wdf, const int8_t* xq, const float* xd,
                     float* y, const float* bias, int rows, int cols, int n, int acc);
int ilt_d4_mm_id_bf16(uint64_t stream, int gguf_type, int ncols, int nrows, int row_bytes, int64_t add, const uint64_t* ptrs,
                      const uint32_t* counts, const uint32_t* bases, int ne, int64_t total_rows,
                      const uint16_t* xb, const uint32_t* rmap, float* y);
int ilt_d4_swiglu_w_bf16(uint64_t stream, int n, int ff, float clamp, const float* g, const float* u, const float* w,
                         uint16_t* mid);
int ilt_d4_mm_id_glu_bf16(uint64_t stream, int gguf_type, int ncols, int nrows, int row_bytes, int64_t add_gate, int64_t add_up,
                          const uint64_t* ptrs, const uint32_t* counts, const uint32_t* bases, int ne, int64_t total_rows,
                          const uint16_t* xb, const uint32_t* rmap, float clamp, const float* wrow, uint16_t* mid);

/* ---- 3. launch by name (src/cuda.lisp:323-352) -------------------------------------------
 * params[i] points at argument i's 8-byte slot: a pointer as 64 bits, an int in the low
 * 32 bits, a float in the low 32 bits, a long long as 64 bits.  Kernel names and argument
 * orders are the reference's (its src/cuda/ *.cu); the grid and block passed in are read
 * only where an argument count lives in them (d4_route: tokens = gx; d4_mv_*: experts =
 * gz).  d4_mv_iq2_xxs / d4_mv_q2_k take the reference's twelve slots (ilt_d4_mv_rows_*); as
 * d4_mvq_iq2_xxs / d4_mvq_q2_k the slots "src1, counts, bases" carry Q8_K activations made
 * beforehand, "xq, xd, bsums", and srcs is not read (ilt_d4_mv_iq2_xxs / ilt_d4_mv_q2_k).  mm_q8, mm_q8_mma, mm_k, mm_q4k_mma and
 * mm_q6k_mma take the reference's lists.  d4_mm_id_iq2_xxs / d4_mm_id_q2_k take the
 * reference's eleven slots (ncols, nrows, row_bytes, x_stride, y_stride, add, ptrs, counts,
 * bases, x, y) with x = xq, followed by three more: xd, bsums, total_rows (long long);
 * experts = gz.  Unknown names return hipErrorNotFound. */
int ilt_launch(const char* kernel, unsigned gx, unsigned gy, unsigned gz, unsigned bx, unsigned by, unsigned bz,
               unsigned shared_bytes, uint64_t stream, void** params);

#ifdef __cplusplus
}
#endif
#endif /* ILLATIO_HIP_H */
