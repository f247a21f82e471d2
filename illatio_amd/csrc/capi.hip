// The C ABI of libillatio_hip.so (declared in include/illatio_hip.h): the driver calls the
// reference's src/cuda.lisp makes, typed entry points for the kernels, and launch by name.
// Host code only validates shapes and picks launch geometry; it does no arithmetic on data (ilt_rope_table, a
// model's constants, aside).
#include <mutex>
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include "../../include/illatio_hip.h"
#include "ilt_kernels.h"

#define ILT_TRY(expr) do { hipError_t e_ = (expr); if (e_ != hipSuccess) return (int)e_; } while (0)
#define ILT_MAX_DEVICES 64
#define ILT_REQUIRE(cond) do { if (!(cond)) return (int)hipErrorInvalidValue; } while (0)

static inline hipStream_t S(uint64_t s) { return (hipStream_t)(uintptr_t)s; }
static inline hipEvent_t E(uint64_t e) { return (hipEvent_t)(uintptr_t)e; }

static int block_weights(int fmt) { return fmt == ILT_Q8_0 ? 32 : 256; }
// bytes of one block as the kernels read it (Q6_K: the padded device block)
static int block_bytes(int fmt) {
  switch (fmt) { case ILT_Q8_0: return 34; case ILT_Q2_K: return 84; case ILT_Q4_K: return 144;
                 case ILT_Q6_K: return ILT_Q6K_STRIDE; case ILT_IQ2_XXS: return 66; }
  return 0;
}
// kquant.cu's numbering of the K-quants (cuda-dense.lisp:18-20) -> GGUF's
static int kquant_type(int code) { return code == 0 ? ILT_Q4_K : code == 2 ? ILT_Q6_K : 0; }

namespace {
struct Args {
  void** p;
  template <class T> T ptr(int i) const { return (T)(uintptr_t)(*(const uint64_t*)p[i]); }
  int i32(int i) const { return *(const int32_t*)p[i]; }
  long long i64(int i) const { return *(const int64_t*)p[i]; }
  float f32(int i) const { return *(const float*)p[i]; }
};
}  // namespace

extern "C" {

int ilt_init(void) { return (int)hipInit(0); }

int ilt_device_count(int* n) { ILT_REQUIRE(n); return (int)hipGetDeviceCount(n); }

int ilt_device_get_info(int index, ilt_device_info* out) {
  ILT_REQUIRE(out);
  hipDeviceProp_t p;
  ILT_TRY(hipGetDeviceProperties(&p, index));
  memset(out, 0, sizeof(*out));
  snprintf(out->name, sizeof(out->name), "%s (%s)", p.name, p.gcnArchName);
  out->arch = 90;
  out->total_memory = p.totalGlobalMem;
  out->max_shared = (int)p.sharedMemPerBlock;
  out->compute_units = p.multiProcessorCount;
  out->wave_size = p.warpSize;
  out->numa_node = -1;
  char path[128];
  snprintf(path, sizeof(path), "/sys/bus/pci/devices/%04x:%02x:%02x.0/numa_node", p.pciDomainID, p.pciBusID, p.pciDeviceID);
  if (FILE* f = fopen(path, "r")) { int node; if (fscanf(f, "%d", &node) == 1) out->numa_node = node; fclose(f); }
  return ILT_OK;
}

int ilt_set_device(int index) { return (int)hipSetDevice(index); }

const char* ilt_error_string(int code) {
  if (code == ILT_OK) return "no error";
  return hipGetErrorString((hipError_t)code);
}

int ilt_stream_create(uint64_t* stream, unsigned flags) {
  ILT_REQUIRE(stream);
  hipStream_t s;
  ILT_TRY(hipStreamCreateWithFlags(&s, (flags & 1) ? hipStreamNonBlocking : hipStreamDefault));
  *stream = (uint64_t)(uintptr_t)s;
  return ILT_OK;
}
int ilt_stream_destroy(uint64_t stream) { return (int)hipStreamDestroy(S(stream)); }
int ilt_stream_sync(uint64_t stream) { return (int)hipStreamSynchronize(S(stream)); }
int ilt_stream_wait_event(uint64_t stream, uint64_t event) { return (int)hipStreamWaitEvent(S(stream), E(event), 0); }

int ilt_event_create(uint64_t* event, unsigned flags) {
  ILT_REQUIRE(event);
  hipEvent_t e;
  ILT_TRY(hipEventCreateWithFlags(&e, (flags & 2) ? hipEventDisableTiming : hipEventDefault));
  *event = (uint64_t)(uintptr_t)e;
  return ILT_OK;
}
int ilt_event_destroy(uint64_t event) { return (int)hipEventDestroy(E(event)); }
int ilt_event_record(uint64_t event, uint64_t stream) { return (int)hipEventRecord(E(event), S(stream)); }
int ilt_event_query(uint64_t event) {
  hipError_t e = hipEventQuery(E(event));
  if (e == hipErrorNotReady) { (void)hipGetLastError(); return ILT_NOT_READY; }
  return (int)e;
}
int ilt_event_elapsed_ms(uint64_t start, uint64_t stop, float* ms) { ILT_REQUIRE(ms); return (int)hipEventElapsedTime(ms, E(start), E(stop)); }

int ilt_malloc(uint64_t* dptr, uint64_t bytes) {
  ILT_REQUIRE(dptr);
  void* p = nullptr;
  ILT_TRY(hipMalloc(&p, bytes < 256 ? 256 : bytes));
  *dptr = (uint64_t)(uintptr_t)p;
  return ILT_OK;
}
int ilt_free(uint64_t dptr) { return dptr ? (int)hipFree((void*)(uintptr_t)dptr) : ILT_OK; }
int ilt_memset_async(uint64_t dptr, int byte, uint64_t bytes, uint64_t stream) {
  return (int)hipMemsetAsync((void*)(uintptr_t)dptr, byte, bytes, S(stream));
}
int ilt_mem_info(uint64_t* free_bytes, uint64_t* total_bytes) {
  ILT_REQUIRE(free_bytes && total_bytes);
  size_t f = 0, t = 0;
  ILT_TRY(hipMemGetInfo(&f, &t));
  *free_bytes = f; *total_bytes = t;
  return ILT_OK;
}
int ilt_memcpy_htod_async(uint64_t dst, const void* src, uint64_t bytes, uint64_t stream) {
  return (int)hipMemcpyAsync((void*)(uintptr_t)dst, src, bytes, hipMemcpyHostToDevice, S(stream));
}
int ilt_memcpy_dtoh_async(void* dst, uint64_t src, uint64_t bytes, uint64_t stream) {
  return (int)hipMemcpyAsync(dst, (const void*)(uintptr_t)src, bytes, hipMemcpyDeviceToHost, S(stream));
}
int ilt_memcpy_dtod_async(uint64_t dst, uint64_t src, uint64_t bytes, uint64_t stream) {
  return (int)hipMemcpyAsync((void*)(uintptr_t)dst, (const void*)(uintptr_t)src, bytes, hipMemcpyDeviceToDevice, S(stream));
}
int ilt_host_alloc(uint64_t* hptr, uint64_t bytes, unsigned flags) {
  ILT_REQUIRE(hptr);
  void* p = nullptr;
  unsigned f = 0;
  if (flags & 1) f |= hipHostMallocPortable;
  if (flags & 2) f |= hipHostMallocMapped;
  ILT_TRY(hipHostMalloc(&p, bytes < 64 ? 64 : bytes, f));
  *hptr = (uint64_t)(uintptr_t)p;
  return ILT_OK;
}
int ilt_host_free(uint64_t hptr) { return (int)hipHostFree((void*)(uintptr_t)hptr); }
// Pinning memory that already exists is not offered: the hosts this library is deployed on refuse
// hipHostRegister, and the error it leaves is reported by whichever GPU call comes next.  The caller
// (the reference pins mmap'd expert files, cuda.lisp:359-366) takes pinned memory from ilt_host_alloc
// and reads the file into it; with every expert resident in HBM nothing needs read-through.
int ilt_host_register(void* p, uint64_t bytes, unsigned flags) {
  (void)p; (void)bytes; (void)flags;
  return (int)hipErrorNotSupported;
}
int ilt_host_unregister(void* p) { (void)p; return (int)hipErrorNotSupported; }

// ---- kernels ----------------------------------------------------------------------------------

int ilt_repack_q8(uint64_t stream, const void* raw, void* qs, void* d, int64_t nblocks) {
  ILT_REQUIRE(nblocks >= 0 && (nblocks == 0 || (raw && qs && d)));
  return (int)ilt_k_repack_q8((const uint8_t*)raw, (int8_t*)qs, (uint16_t*)d, nblocks, S(stream));
}

int ilt_repack_q6k(uint64_t stream, const void* raw, void* out, int64_t nblocks) {
  ILT_REQUIRE(nblocks >= 0 && (nblocks == 0 || (raw && out)));
  return (int)ilt_k_repack_q6k((const uint8_t*)raw, (uint8_t*)out, nblocks, S(stream));
}

int ilt_quant_q8(uint64_t stream, const float* x, int8_t* xq, float* xs, int32_t* xsum, int64_t nblocks) {
  ILT_REQUIRE(nblocks >= 0 && (nblocks == 0 || (x && xq && xs)));
  return (int)ilt_k_quant_q8(x, xq, xs, xsum, nblocks, 1, S(stream));
}

int ilt_d4_quant(uint64_t stream, const float* x, int8_t* xq, float* xs, int nblocks) {
  ILT_REQUIRE(nblocks >= 0 && (nblocks == 0 || (x && xq && xs)));
  return (int)ilt_k_quant_q8(x, xq, xs, nullptr, nblocks, 0, S(stream));
}

int ilt_quant_q8k(uint64_t stream, const float* x, int8_t* xq, float* xd, int32_t* bsums, int64_t nblocks) {
  ILT_REQUIRE(nblocks >= 0 && (nblocks == 0 || (x && xq && xd && bsums)));
  ILT_REQUIRE(((uintptr_t)x & 15) == 0 && ((uintptr_t)xq & 3) == 0);      // 16-byte loads, 4-byte stores
  return (int)ilt_k_quant_q8k(x, xq, xd, bsums, nblocks, S(stream));
}

// One launch over up to four dense matrices sharing the activations (given quantized, or
// as floats to be quantized by the kernel).
// The launch's parameters into p; live (may be null) = how many of the matrices have rows (none: nothing to launch)
static int gemv_multi_build(IltGemvParams& p, int* live_out, int nmat, const int* fmts, const void* const* ws, const uint16_t* const* wds,
                            float* const* ys, const float* const* biases, const int* rows, int cols, const int8_t* xq,
                            const float* xs, const int32_t* bsums, const float* xf, int f16_scale, int acc, int glu,
                            int group_rows, const float* norm_w, float eps, int norm_seq) {
  ILT_REQUIRE(nmat >= 1 && nmat <= 4 && cols > 0);
  const bool q8 = fmts[0] == ILT_Q8_0;
  p = IltGemvParams{};
  int live = 0;
  for (int i = 0; i < nmat; i++) {
    const int fmt = fmts[i];
    ILT_REQUIRE((fmt == ILT_Q8_0 || fmt == ILT_Q4_K || fmt == ILT_Q6_K) && (fmt == ILT_Q8_0) == q8);
    ILT_REQUIRE(rows[i] >= 0 && cols % block_weights(fmt) == 0);
    if (rows[i] == 0) { ILT_REQUIRE(!glu); continue; }
    ILT_REQUIRE(ws[i] && ys[i] && ((uintptr_t)ws[i] & 15) == 0 && (fmt != ILT_Q8_0 || wds[i]));
    IltGemvMat& m = p.mat[live++];
    m.w = (const uint8_t*)ws[i]; m.wd = wds[i]; m.y = ys[i]; m.bias = biases ? biases[i] : nullptr;
    m.rows = rows[i]; m.fmt = fmt;
    m.row_bytes = fmt == ILT_Q8_0 ? cols : (long long)cols / 256 * block_bytes(fmt);
  }
  if (live_out) *live_out = live;
  if (live == 0) return ILT_OK;
  if (glu) ILT_REQUIRE(live == 2 && p.mat[0].rows == p.mat[1].rows && !acc);
  if (xf) ILT_REQUIRE(((uintptr_t)xf & 15) == 0 && ((uintptr_t)norm_w & 15) == 0);
  else ILT_REQUIRE(!norm_w && xq && xs && (q8 || bsums) && ((uintptr_t)xq & 15) == 0);
  p.nmat = live; p.cols = cols; p.xq = xq; p.xs = xs; p.bsums = bsums; p.xf = xf; p.f16_scale = f16_scale;
  p.norm_w = norm_w; p.eps = eps; p.norm_seq = norm_seq;
  p.acc = acc; p.glu = glu;
  if (group_rows > 0 && group_rows < p.mat[0].rows) {
    ILT_REQUIRE(live == 1 && p.mat[0].rows % group_rows == 0);
    p.group_rows = group_rows;
  }
  return ILT_OK;
}

static int gemv_multi(uint64_t stream, int nmat, const int* fmts, const void* const* ws, const uint16_t* const* wds,
                      float* const* ys, const float* const* biases, const int* rows, int cols, const int8_t* xq,
                      const float* xs, const int32_t* bsums, const float* xf, int f16_scale, int acc, int glu,
                      int group_rows, const float* norm_w = nullptr, float eps = 0.0f, int norm_seq = 0) {
  IltGemvParams p;
  int live = 0;
  const int e = gemv_multi_build(p, &live, nmat, fmts, ws, wds, ys, biases, rows, cols, xq, xs, bsums, xf, f16_scale, acc, glu, group_rows,
                                 norm_w, eps, norm_seq);
  if (e != ILT_OK || live == 0) return e;
  return (int)ilt_gemv_launch(p, 1, S(stream));
}

static int gemv_dense(uint64_t stream, int fmt, const void* w, const uint16_t* wd, const int8_t* xq, const float* xs,
                      const int32_t* bsums, const float* xf, int f16_scale, float* out, const float* bias, int rows,
                      int cols, int acc, int group_rows) {
  ILT_REQUIRE(fmt);
  return gemv_multi(stream, 1, &fmt, &w, &wd, &out, &bias, &rows, cols, xq, xs, bsums, xf, f16_scale, acc, 0, group_rows);
}

int ilt_mv_q8(uint64_t stream, const int8_t* wq, const uint16_t* wd, const int8_t* xq, const float* xs, float* out,
              const float* bias, int rows, int cols, int acc) {
  return gemv_dense(stream, ILT_Q8_0, wq, wd, xq, xs, nullptr, nullptr, 0, out, bias, rows, cols, acc, 0);
}

int ilt_mv_q8_3(uint64_t stream, const int8_t* q0, const uint16_t* d0, const int8_t* q1, const uint16_t* d1,
                const int8_t* q2, const uint16_t* d2, const int8_t* xq, const float* xs, float* o0, float* o1, float* o2,
                const float* b0, const float* b1, const float* b2, int r0, int r1, int r2, int cols) {
  const int fmts[3] = {ILT_Q8_0, ILT_Q8_0, ILT_Q8_0}, rows[3] = {r0, r1, r2};
  const void* ws[3] = {q0, q1, q2}; const uint16_t* wds[3] = {d0, d1, d2};
  float* ys[3] = {o0, o1, o2}; const float* bs[3] = {b0, b1, b2};
  return gemv_multi(stream, 3, fmts, ws, wds, ys, bs, rows, cols, xq, xs, nullptr, nullptr, 0, 0, 0, 0);
}

int ilt_mv_q8_glu(uint64_t stream, const int8_t* gq, const uint16_t* gd, const int8_t* uq, const uint16_t* ud,
                  const int8_t* xq, const float* xs, float* out, int rows, int cols) {
  const int fmts[2] = {ILT_Q8_0, ILT_Q8_0}, r[2] = {rows, rows};
  const void* ws[2] = {gq, uq}; const uint16_t* wds[2] = {gd, ud};
  float* ys[2] = {out, out};
  return gemv_multi(stream, 2, fmts, ws, wds, ys, nullptr, r, cols, xq, xs, nullptr, nullptr, 0, 0, 1, 0);
}

int ilt_mv_k(uint64_t stream, int type, const void* w, const int8_t* xq, const float* xd, const int32_t* bsums, float* out,
             const float* bias, int rows, int cols, int acc) {
  return gemv_dense(stream, kquant_type(type), w, nullptr, xq, xd, bsums, nullptr, 0, out, bias, rows, cols, acc, 0);
}

int ilt_mv_k_glu(uint64_t stream, int gtype, const void* gw, int utype, const void* uw, const int8_t* xq, const float* xd,
                 const int32_t* bsums, float* out, int rows, int cols) {
  const int fmts[2] = {kquant_type(gtype), kquant_type(utype)}, r[2] = {rows, rows};
  ILT_REQUIRE(fmts[0] && fmts[1]);
  const void* ws[2] = {gw, uw}; const uint16_t* wds[2] = {nullptr, nullptr};
  float* ys[2] = {out, out};
  return gemv_multi(stream, 2, fmts, ws, wds, ys, nullptr, r, cols, xq, xd, bsums, nullptr, 0, 0, 1, 0);
}

int ilt_mv_multi(uint64_t stream, int nmat, const ilt_mv_desc* descs, int cols, const int8_t* xq, const float* xs,
                 const int32_t* bsums, const float* xf, int f16_scale, int acc, int glu) {
  ILT_REQUIRE(descs && nmat >= 1 && nmat <= 4);
  int fmts[4], rows[4]; const void* ws[4]; const uint16_t* wds[4]; float* ys[4]; const float* bs[4];
  for (int i = 0; i < nmat; i++) {
    fmts[i] = descs[i].gguf_type; rows[i] = descs[i].rows; ws[i] = descs[i].w; wds[i] = descs[i].wd;
    ys[i] = descs[i].y; bs[i] = descs[i].bias;
  }
  return gemv_multi(stream, nmat, fmts, ws, wds, ys, bs, rows, cols, xq, xs, bsums, xf, f16_scale, acc, glu, 0);
}

// ilt_mv_multi / ilt_mv_multi_norm on float activations, reading the rows of the caller's next product ahead while it
// runs (norm_w null: no norm).  The next product is described, not launched; where either of the two does not take
// the streamed variant the call is the plain one.
int ilt_mv_multi_ahead(uint64_t stream, int nmat, const ilt_mv_desc* descs, int cols, const float* xf, const float* norm_w, float eps,
                       int f16_scale, int acc, int glu, int next_nmat, const ilt_mv_desc* next_descs, int next_cols, int next_glu) {
  ILT_REQUIRE(descs && nmat >= 1 && nmat <= 4 && xf && (!next_nmat || (next_descs && next_nmat >= 1 && next_nmat <= 4 && next_cols > 0)));
  auto build = [&](IltGemvParams& p, int* live, int n, const ilt_mv_desc* d, int c, const float* x, const float* nw, int a, int g) -> int {
    int fmts[4], rows[4]; const void* ws[4]; const uint16_t* wds[4]; float* ys[4]; const float* bs[4];
    for (int i = 0; i < n; i++) { fmts[i] = d[i].gguf_type; rows[i] = d[i].rows; ws[i] = d[i].w; wds[i] = d[i].wd; ys[i] = d[i].y; bs[i] = d[i].bias; }
    return gemv_multi_build(p, live, n, fmts, ws, wds, ys, bs, rows, c, nullptr, nullptr, nullptr, x, f16_scale, a, g, 0, nw, eps, 0);
  };
  IltGemvParams p, pn;
  int live = 0, live_n = 0;
  const int e = build(p, &live, nmat, descs, cols, xf, norm_w, acc, glu);
  if (e != ILT_OK || live == 0) return e;
  // (the next product's activations do not matter to its plan: this call's stand in for them)
  static const bool rows_on = []{ const char* f = getenv("ILT_ROWS_AHEAD"); return !(f && f[0] == '0'); }();      // ("0": never, for tests)
  if (rows_on && next_nmat && build(pn, &live_n, next_nmat, next_descs, next_cols, xf, nullptr, 0, next_glu) == ILT_OK && live_n &&
      ilt_gemv_plan(p, 1) == hipSuccess && ilt_gemv_plan(pn, 1) == hipSuccess)
    ilt_gemv_rows_of(pn, p.rows_ahead);
  return (int)ilt_gemv_launch(p, 1, S(stream));
}

uint64_t ilt_streamed_launches(void) { return (uint64_t)ilt_k_streamed_launches(); }

int ilt_mv_multi_norm(uint64_t stream, int nmat, const ilt_mv_desc* descs, int cols, const float* x, const float* norm_w,
                      float eps, int exact_order, int f16_scale, int glu) {
  ILT_REQUIRE(descs && nmat >= 1 && nmat <= 4 && x && norm_w);
  int fmts[4], rows[4]; const void* ws[4]; const uint16_t* wds[4]; float* ys[4]; const float* bs[4];
  for (int i = 0; i < nmat; i++) {
    fmts[i] = descs[i].gguf_type; rows[i] = descs[i].rows; ws[i] = descs[i].w; wds[i] = descs[i].wd;
    ys[i] = descs[i].y; bs[i] = descs[i].bias;
  }
  return gemv_multi(stream, nmat, fmts, ws, wds, ys, bs, rows, cols, nullptr, nullptr, nullptr, x, f16_scale, 0, glu, 0,
                    norm_w, eps, exact_order ? 1 : 0);
}

static int rmsnorm_quant(uint64_t stream, int k, const float* x, const float* w, float* h, int8_t* xq, float* xs, int32_t* xsum,
                         int dim, float eps, int n, int exact_order) {
  ILT_REQUIRE(n >= 0 && dim > 0 && dim % (k ? 256 : 32) == 0);
  if (n == 0) return ILT_OK;
  ILT_REQUIRE(x && w && xq && xs && (!k || xsum) && ((uintptr_t)x & 15) == 0 && ((uintptr_t)w & 15) == 0 &&
              ((uintptr_t)h & 15) == 0 && ((uintptr_t)xq & 3) == 0);
  return (int)ilt_k_rmsnorm_quant(k, x, w, h, xq, xs, xsum, dim, eps, 1, exact_order ? 1 : 0, n, S(stream));
}

int ilt_rmsnorm_q8(uint64_t stream, const float* x, const float* w, float* h, int8_t* xq, float* xs, int32_t* xsum, int dim,
                   float eps, int n, int exact_order) {
  return rmsnorm_quant(stream, 0, x, w, h, xq, xs, xsum, dim, eps, n, exact_order);
}

int ilt_rmsnorm_q8k(uint64_t stream, const float* x, const float* w, float* h, int8_t* xq, float* xd, int32_t* bsums, int dim,
                    float eps, int n, int exact_order) {
  return rmsnorm_quant(stream, 1, x, w, h, xq, xd, bsums, dim, eps, n, exact_order);
}

int ilt_d4_mvq8(uint64_t stream, int rows, int cols, int group_rows, const int8_t* wq, const uint16_t* wd,
                const int8_t* xq, const float* xs, float* y) {
  ILT_REQUIRE(group_rows > 0);
  return gemv_dense(stream, ILT_Q8_0, wq, wd, xq, xs, nullptr, nullptr, 0, y, nullptr, rows, cols, 0, group_rows);
}

// add_up >= 0: the gated pair, gate at ptrs[z] + add and up at ptrs[z] + add_up, dst = the gated activation.
// xf: the activations as floats, quantized to Q8_K in the kernel; else xq, xd, bsums.
static int gemv_experts(uint64_t stream, int fmt, int ncols, int nrows, int row_bytes, int64_t add, int64_t add_up,
                        int x_stride, int y_stride, const uint64_t* ptrs, int nz, const int8_t* xq, const float* xd,
                        const int32_t* bsums, const float* xf, const float* wts, float clamp, float* dst,
                        const uint32_t* sel = nullptr, const uint32_t* counts = nullptr, const uint32_t* bases = nullptr) {
  ILT_REQUIRE(nrows >= 0 && nz >= 0 && ncols > 0 && ncols % 256 == 0 && row_bytes == ncols / 256 * block_bytes(fmt));
  if (nrows == 0 || nz == 0) return ILT_OK;
  ILT_REQUIRE(ptrs && dst && add >= 0 && (add & 1) == 0 && (add_up < 0 || (add_up & 1) == 0) && x_stride % 256 == 0 && x_stride >= 0);
  ILT_REQUIRE(!counts || (bases && xf && !sel && add_up < 0));
  if (xf) ILT_REQUIRE(((uintptr_t)xf & 15) == 0);
  else ILT_REQUIRE(xq && xd && (bsums || fmt == ILT_IQ2_XXS) && ((uintptr_t)xq & 15) == 0);
  ILT_REQUIRE(nz <= 65535);
  IltGemvParams p = {};
  p.nmat = 1; p.mat[0].rows = nrows; p.mat[0].row_bytes = row_bytes; p.mat[0].fmt = fmt; p.mat[0].y = dst; p.mat[0].add = add;
  if (add_up >= 0) {
    p.nmat = 2; p.mat[1] = p.mat[0]; p.mat[1].add = add_up;
    p.glu = 2; p.clamp = clamp; p.wts = wts;
  }
  p.ptrs = ptrs; p.sel = sel; p.cols = ncols;
  p.xq = xq; p.xs = xd; p.bsums = bsums; p.xf = xf; p.x_stride = x_stride; p.y_stride = y_stride;
  p.counts = counts; p.bases = bases;
  return (int)ilt_gemv_launch(p, nz, S(stream));
}

// the reference's own arguments (ds4f.cu:762-772): srcs read through first, float rows quantized by the kernel
static int mv_rows(uint64_t stream, int fmt, int ncols, int nrows, int row_bytes, int64_t add, int x_stride, int y_stride,
                   const uint64_t* ptrs, const uint64_t* srcs, int nz, const float* x, float* y, const uint32_t* counts,
                   const uint32_t* bases) {
  ILT_REQUIRE(x && (counts == nullptr) == (bases == nullptr));
  if (srcs && nrows > 0 && nz > 0) {
    ILT_REQUIRE(ptrs && add >= 0 && (add & 1) == 0 && row_bytes > 0 && nz <= 65535);
    ILT_TRY(ilt_k_read_through((const unsigned long long*)srcs, (const unsigned long long*)ptrs, nz, add, (long long)nrows * row_bytes,
                               S(stream)));
  }
  return gemv_experts(stream, fmt, ncols, nrows, row_bytes, add, -1, x_stride, y_stride, ptrs, nz, nullptr, nullptr, nullptr, x,
                      nullptr, 0.0f, y, nullptr, counts, bases);
}

int ilt_d4_mv_rows_iq2_xxs(uint64_t stream, int ncols, int nrows, int row_bytes, int64_t add, int x_stride, int y_stride,
                           const uint64_t* ptrs, const uint64_t* srcs, int nz, const float* x, float* y,
                           const uint32_t* counts, const uint32_t* bases) {
  return mv_rows(stream, ILT_IQ2_XXS, ncols, nrows, row_bytes, add, x_stride, y_stride, ptrs, srcs, nz, x, y, counts, bases);
}

int ilt_d4_mv_rows_q2_k(uint64_t stream, int ncols, int nrows, int row_bytes, int64_t add, int x_stride, int y_stride,
                        const uint64_t* ptrs, const uint64_t* srcs, int nz, const float* x, float* y,
                        const uint32_t* counts, const uint32_t* bases) {
  return mv_rows(stream, ILT_Q2_K, ncols, nrows, row_bytes, add, x_stride, y_stride, ptrs, srcs, nz, x, y, counts, bases);
}

int ilt_d4_mv_iq2_xxs(uint64_t stream, int ncols, int nrows, int row_bytes, int64_t add, int x_stride, int y_stride,
                      const uint64_t* ptrs, int nz, const int8_t* xq, const float* xd, float* dst) {
  return gemv_experts(stream, ILT_IQ2_XXS, ncols, nrows, row_bytes, add, -1, x_stride, y_stride, ptrs, nz, xq, xd,
                      nullptr, nullptr, nullptr, 0.0f, dst);
}

int ilt_d4_mv_q2_k(uint64_t stream, int ncols, int nrows, int row_bytes, int64_t add, int x_stride, int y_stride,
                   const uint64_t* ptrs, int nz, const int8_t* xq, const float* xd, const int32_t* bsums, float* dst) {
  return gemv_experts(stream, ILT_Q2_K, ncols, nrows, row_bytes, add, -1, x_stride, y_stride, ptrs, nz, xq, xd, bsums,
                      nullptr, nullptr, 0.0f, dst);
}

int ilt_d4_mv_glu_iq2_xxs(uint64_t stream, int ncols, int nrows, int row_bytes, int64_t add_gate, int64_t add_up,
                          int x_stride, int y_stride, const uint64_t* ptrs, const uint32_t* sel, int nz, const float* x,
                          const float* wts, float clamp, float* mid) {
  ILT_REQUIRE(add_up >= 0 && x);
  return gemv_experts(stream, ILT_IQ2_XXS, ncols, nrows, row_bytes, add_gate, add_up, x_stride, y_stride, ptrs, nz,
                      nullptr, nullptr, nullptr, x, wts, clamp, mid, sel);
}

int ilt_d4_mv_q2_k_f32(uint64_t stream, int ncols, int nrows, int row_bytes, int64_t add, int x_stride, int y_stride,
                       const uint64_t* ptrs, const uint32_t* sel, int nz, const float* x, float* dst) {
  ILT_REQUIRE(x);
  return gemv_experts(stream, ILT_Q2_K, ncols, nrows, row_bytes, add, -1, x_stride, y_stride, ptrs, nz, nullptr, nullptr,
                      nullptr, x, nullptr, 0.0f, dst, sel);
}

// route: a token's routing for the launch to carry along, or null; its done says whether the launch did
static int mvq8_glu(uint64_t stream, int rows, int cols, const int8_t* gq, const uint16_t* gd, const int8_t* uq,
                    const uint16_t* ud, const float* x, float clamp, float* mid, IltRouteAlong* route) {
  ILT_REQUIRE(rows >= 0 && cols > 0 && cols % 32 == 0);
  if (rows == 0) return ILT_OK;
  ILT_REQUIRE(gq && gd && uq && ud && x && mid && ((uintptr_t)gq & 15) == 0 && ((uintptr_t)uq & 15) == 0 && ((uintptr_t)x & 15) == 0);
  IltGemvParams p = {};
  p.nmat = 2;
  for (int i = 0; i < 2; i++) {
    p.mat[i].w = (const uint8_t*)(i ? uq : gq); p.mat[i].wd = i ? ud : gd; p.mat[i].y = mid;
    p.mat[i].rows = rows; p.mat[i].fmt = ILT_Q8_0; p.mat[i].row_bytes = cols;
  }
  p.cols = cols; p.xf = x; p.f16_scale = 0; p.glu = 2; p.clamp = clamp;
  if (route) { p.route = *route; p.route.done = 0; }
  const int e = (int)ilt_gemv_launch(p, 1, S(stream));
  if (route) route->done = e == ILT_OK ? p.route.done : 0;
  return e;
}

int ilt_d4_mvq8_glu(uint64_t stream, int rows, int cols, const int8_t* gq, const uint16_t* gd, const int8_t* uq,
                    const uint16_t* ud, const float* x, float clamp, float* mid) {
  return mvq8_glu(stream, rows, cols, gq, gd, uq, ud, x, clamp, mid, nullptr);
}

int ilt_dequant_rows(uint64_t stream, int gguf_type, const void* w, const uint16_t* wd, const int32_t* rows_idx,
                     int64_t nrows, int cols, float* out) {
  ILT_REQUIRE(block_bytes(gguf_type) && cols > 0 && cols % block_weights(gguf_type) == 0 && nrows >= 0);
  if (nrows == 0) return ILT_OK;
  ILT_REQUIRE(w && out && (gguf_type != ILT_Q8_0 || wd));
  const long long rb = gguf_type == ILT_Q8_0 ? cols : (long long)cols / 256 * block_bytes(gguf_type);
  return (int)ilt_k_dequant_rows(gguf_type, (const uint8_t*)w, wd, rows_idx, nrows, cols, rb, out, S(stream));
}

int ilt_embed_q8(uint64_t stream, const int8_t* qs, const uint16_t* d, const int32_t* tokens, float* out, int cols, int n) {
  return ilt_dequant_rows(stream, ILT_Q8_0, qs, d, tokens, n, cols, out);
}

int ilt_embed_k(uint64_t stream, int type, const void* w, const int32_t* tokens, float* out, int cols, int n) {
  ILT_REQUIRE(kquant_type(type));
  return ilt_dequant_rows(stream, kquant_type(type), w, nullptr, tokens, n, cols, out);
}

int ilt_d4_route(uint64_t stream, int ne, int nu, int hash, float scale, int has_bias, const float* logits,
                 const float* bias, const int32_t* tid2eid, const uint32_t* tokens, uint32_t* sel, float* wout, int ntok) {
  ILT_REQUIRE(ntok >= 0 && (ntok == 0 || (logits && sel && wout)));
  ILT_REQUIRE(!has_bias || bias);
  ILT_REQUIRE(hash != 1 || (tid2eid && tokens));
  return (int)ilt_k_route(ne, nu, hash, scale, has_bias, logits, bias, tid2eid, tokens, sel, wout, ntok, S(stream));
}

int ilt_d4_group_zero(uint64_t stream, int ne, uint32_t* counts) {
  ILT_REQUIRE(ne > 0 && counts);
  return (int)ilt_k_group_zero(ne, counts, S(stream));
}
int ilt_d4_group_count(uint64_t stream, int n, int ne, int nu, const uint32_t* sel, uint32_t* counts, uint32_t* rank) {
  ILT_REQUIRE(n >= 0 && (n == 0 || (sel && counts && rank)));
  return (int)ilt_k_group_count(n, ne, nu, sel, counts, rank, S(stream));
}
int ilt_d4_group_scan(uint64_t stream, int n, int ne, int nu, const uint32_t* counts, uint32_t* bases) {
  ILT_REQUIRE(ne > 0 && counts && bases);
  return (int)ilt_k_group_scan(n, ne, nu, counts, bases, S(stream));
}
int ilt_d4_group_scatter(uint64_t stream, int n, int ne, int nu, const uint32_t* sel, const uint32_t* rank,
                         const uint32_t* bases, const float* w, uint32_t* rmap, uint32_t* smap, float* wrow) {
  ILT_REQUIRE(n >= 0 && nu > 0 && (n == 0 || (sel && rank && bases && w && rmap && smap && wrow)));
  return (int)ilt_k_group_scatter(n, ne, nu, sel, rank, bases, w, rmap, smap, wrow, S(stream));
}
int ilt_d4_rows_expert(uint64_t stream, int n, const uint32_t* sel, const uint32_t* smap, uint32_t* rexp) {
  ILT_REQUIRE(n >= 0 && (n == 0 || (sel && smap && rexp)));
  return (int)ilt_k_rows_expert(n, sel, smap, rexp, S(stream));
}
int ilt_d4_gather_rows(uint64_t stream, int d, int nrows, const float* src, const uint32_t* map, float* x) {
  ILT_REQUIRE(d > 0 && nrows >= 0 && (nrows == 0 || (src && map && x)));
  return (int)ilt_k_gather_rows(d, nrows, src, map, x, S(stream));
}
int ilt_d4_swiglu_w(uint64_t stream, int n, int ff, float clamp, const float* g, const float* u, const float* w,
                    float* mid, int8_t* xq, float* xs) {
  ILT_REQUIRE(n >= 0 && ff > 0 && (n == 0 || (g && u && w && mid)) && (!xq || xs));
  return (int)ilt_k_swiglu_w(n, ff, clamp, g, u, w, mid, xq, xs, S(stream));
}
int ilt_d4_swiglu_w_bf16(uint64_t stream, int n, int ff, float clamp, const float* g, const float* u, const float* w, uint16_t* mid) {
  ILT_REQUIRE(n >= 0 && ff > 0 && ff % 8 == 0 && (n == 0 || (g && u && w && mid)));
  ILT_REQUIRE((((uintptr_t)g | (uintptr_t)u | (uintptr_t)mid) & 15) == 0);
  return (int)ilt_k_swiglu_w_bf16(n, ff, clamp, g, u, w, mid, S(stream));
}
int ilt_d4_moe_sum(uint64_t stream, int d, int k, const float* down, const float* shared_, float* moe, const uint32_t* perm) {
  ILT_REQUIRE(d > 0 && k >= 0 && down && moe);
  return (int)ilt_k_moe_sum(d, k, down, shared_, moe, perm, S(stream));
}
int ilt_d4_moe_sum_rows(uint64_t stream, int d, int nu, int ntok, const float* down, const uint32_t* map,
                        const float* shared_, float* moe) {
  ILT_REQUIRE(d > 0 && nu > 0 && ntok >= 0 && (ntok == 0 || (down && map && moe)));
  return (int)ilt_k_moe_sum_rows(d, nu, ntok, down, map, shared_, moe, S(stream));
}

// ---- one token's FFN past the router in one call ------------------------------------------------
// The step's intermediate results, 256-byte aligned pieces of one buffer.
namespace {
struct StepLayout { uint64_t sel, w, smid, sout, bm, bd, total; };
inline uint64_t up256(uint64_t v) { return (v + 255) / 256 * 256; }
StepLayout step_layout(int nu, int d, int ff) {
  StepLayout l; uint64_t o = 0;
  l.sel = o; o += up256(4ull * nu);
  l.w = o; o += up256(4ull * nu);
  l.smid = o; o += up256(4ull * ff);
  l.sout = o; o += up256(4ull * d);
  l.bm = o; o += up256(4ull * nu * ff);
  l.bd = o; o += up256(4ull * nu * d);
  l.total = o;
  return l;
}
int step_args_ok(int ne, int nu, int d, int ff, const ilt_ffn_step_weights* wt, const float* logits, const float* x, float* moe) {
  ILT_REQUIRE(wt && logits && x && moe && ne >= 1 && ne <= 1024 && nu >= 1 && nu <= 64 && nu <= ne);
  ILT_REQUIRE(d > 0 && ff > 0 && d % 256 == 0 && ff % 256 == 0 && d <= (1 << 20) && ff <= (1 << 20));
  ILT_REQUIRE(wt->slots && wt->gate_bytes == (int64_t)ff * (d / 256 * 66) && wt->sgate_q && wt->sgate_d && wt->sup_q && wt->sup_d &&
              wt->sdown_q && wt->sdown_d);
  return ILT_OK;
}
// The shared expert's down product as the step's last launch, the step's sum carried along (IltSumAlong): MOE gets
// ((0 + bd[0]) + ... + bd[nu-1]) + W.smid.  hipErrorNotSupported (nothing launched) where the launch cannot take it.
int shared_down_sum(uint64_t stream, int d, int ff, const int8_t* wq, const uint16_t* wd, const float* smid, const float* bd, int nu,
                    float* moe) {
  IltGemvParams p;
  int live = 0, fmt = ILT_Q8_0, rows = d;
  const void* w = wq; const float* nobias = nullptr;
  const int e = gemv_multi_build(p, &live, 1, &fmt, &w, &wd, &moe, &nobias, &rows, ff, nullptr, nullptr, nullptr, smid, 0, 0, 0, 0, nullptr, 0.0f, 0);
  if (e != ILT_OK) return e;
  if (live == 0) return (int)hipErrorNotSupported;
  p.sum = {bd, (long long)d, nu};
  return (int)ilt_gemv_launch(p, 1, S(stream));
}
// A caller's events around the step's launches (ilt_d4_ffn_step_events): event i recorded on the stream before launch
// i, the one after the last launch behind it.  Per thread; none by default.
thread_local const uint64_t* g_step_events = nullptr;
thread_local int g_step_nevents = 0, g_step_marked = 0;
int step_mark(uint64_t stream) {
  if (g_step_events && g_step_marked < g_step_nevents) ILT_TRY(hipEventRecord((hipEvent_t)g_step_events[g_step_marked++], S(stream)));
  return ILT_OK;
}
// Five launches on STREAM, nothing allocated, freed or waited for; ws holds step_layout's bytes.
int step_run(uint64_t stream, uint8_t* ws, int ne, int nu, int d, int ff, float scale, float clamp, const ilt_ffn_step_weights* wt,
             const float* logits, const float* bias, const float* x, float* moe) {
  const StepLayout l = step_layout(nu, d, ff);
  uint32_t* sel = (uint32_t*)(ws + l.sel);
  float *w = (float*)(ws + l.w), *smid = (float*)(ws + l.smid), *sout = (float*)(ws + l.sout);
  float *bm = (float*)(ws + l.bm), *bd = (float*)(ws + l.bd);
  const int grb = d / 256 * 66, drb = ff / 256 * 84;
  // the routing rides along with the shared expert's gate/up launch (one of its waves routes while the rows stream
  // in); where that launch cannot take it, a launch of its own
  IltRouteAlong route = {logits, bias, sel, w, ne, nu, scale, 0};
  g_step_marked = 0;
  ILT_TRY((hipError_t)step_mark(stream));
  ILT_TRY((hipError_t)mvq8_glu(stream, ff, d, wt->sgate_q, wt->sgate_d, wt->sup_q, wt->sup_d, x, clamp, smid, &route));
  if (!route.done) ILT_TRY((hipError_t)ilt_d4_route(stream, ne, nu, 0, scale, bias ? 1 : 0, logits, bias, nullptr, nullptr, sel, w, 1));
  ILT_TRY((hipError_t)step_mark(stream));
  ILT_TRY((hipError_t)ilt_d4_mv_glu_iq2_xxs(stream, d, ff, grb, 0, wt->gate_bytes, 0, ff, wt->slots, sel, nu, x, w, clamp, bm));
  ILT_TRY((hipError_t)step_mark(stream));
  ILT_TRY((hipError_t)ilt_d4_mv_q2_k_f32(stream, ff, d, drb, 2 * wt->gate_bytes, ff, d, wt->slots, sel, nu, bm, bd));
  ILT_TRY((hipError_t)step_mark(stream));
  // the shared expert's down product last, adding the routed experts' rows and its own as it stores them; where
  // that launch cannot (more than eight slots, a matrix too small for the streamed variant): the product, then the sum
  int e = shared_down_sum(stream, d, ff, wt->sdown_q, wt->sdown_d, smid, bd, nu, moe);
  if (e == (int)hipErrorNotSupported) {
    ilt_mv_desc down = {ILT_Q8_0, d, wt->sdown_q, wt->sdown_d, sout, nullptr};
    ILT_TRY((hipError_t)ilt_mv_multi(stream, 1, &down, ff, nullptr, nullptr, nullptr, smid, 0, 0, 0));
    e = ilt_d4_moe_sum(stream, d, nu, bd, sout, moe, nullptr);
  }
  if (e != ILT_OK) return e;
  return step_mark(stream);
}
}  // namespace

int ilt_d4_ffn_step_events(const uint64_t* events, int n) {
  ILT_REQUIRE(n >= 0 && n <= 8 && (n == 0 || events));
  g_step_events = n ? events : nullptr;
  g_step_nevents = n;
  return ILT_OK;
}

uint64_t ilt_d4_ffn_step_workspace(int nu, int d, int ff) {
  if (nu < 1 || d < 1 || ff < 1 || nu > 64 || d > (1 << 20) || ff > (1 << 20)) return 0;
  return step_layout(nu, d, ff).total;
}

int ilt_d4_ffn_step(uint64_t stream, void* ws, uint64_t ws_bytes, int ne, int nu, int d, int ff, float scale, float clamp,
                    const ilt_ffn_step_weights* wt, const float* logits, const float* bias, const float* x, float* moe) {
  ILT_TRY((hipError_t)step_args_ok(ne, nu, d, ff, wt, logits, x, moe));
  ILT_REQUIRE(ws && ((uintptr_t)ws & 255) == 0 && ws_bytes >= step_layout(nu, d, ff).total);
  return step_run(stream, (uint8_t*)ws, ne, nu, d, ff, scale, clamp, wt, logits, bias, x, moe);
}

// ilt_d4_ffn_step for callers that cannot allocate or pass a workspace: the step's intermediate
// results in a device array that is part of the library's code object.  Each GPU the library runs
// on holds its own copy, at its own address, until the process ends.
#define ILT_STEP_SCRATCH_BYTES (1u << 20)
static __device__ __align__(256) __attribute__((used)) unsigned char scratch[ILT_STEP_SCRATCH_BYTES];
// The array's address on each device, asked of the runtime once per device with that device
// current.  In host code the name `scratch` is a stand-in for the symbol, not a device address:
// only these pointers go to kernels.
static void* g_scratch_ptr[ILT_MAX_DEVICES];

static int step_scratch(uint8_t** out) {
  int dev = -1;
  ILT_TRY(hipGetDevice(&dev));
  ILT_REQUIRE(dev >= 0 && dev < ILT_MAX_DEVICES);
  void* p = __atomic_load_n(&g_scratch_ptr[dev], __ATOMIC_ACQUIRE);
  if (!p) {
    ILT_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    ILT_REQUIRE(p && ((uintptr_t)p & 255) == 0);
    __atomic_store_n(&g_scratch_ptr[dev], p, __ATOMIC_RELEASE);       // two threads racing store the same address
  }
  *out = (uint8_t*)p;
  return ILT_OK;
}

uint64_t ilt_d4_ffn_step_noalloc_max_bytes(void) { return ILT_STEP_SCRATCH_BYTES; }

int ilt_d4_ffn_step_noalloc(uint64_t stream, int ne, int nu, int d, int ff, float scale, float clamp,
                            const ilt_ffn_step_weights* wt, const float* logits, const float* bias, const float* x, float* moe) {
  ILT_TRY((hipError_t)step_args_ok(ne, nu, d, ff, wt, logits, x, moe));
  if (step_layout(nu, d, ff).total > ILT_STEP_SCRATCH_BYTES) return (int)hipErrorInvalidValue;    // beyond the array: say so, touch nothing
  uint8_t* ws = nullptr;
  ILT_TRY((hipError_t)step_scratch(&ws));
  // Every piece of the layout is written in full by the launch that produces it before a later
  // launch reads it, so nothing of the previous call's contents has to be cleared.
  return step_run(stream, ws, ne, nu, d, ff, scale, clamp, wt, logits, bias, x, moe);
}

int ilt_mm_q8(uint64_t stream, const int8_t* wq, const uint16_t* wd, const int8_t* xq, const float* xs, float* y,
              const float* bias, int rows, int cols, int n, int acc) {
  ILT_REQUIRE(rows >= 0 && n >= 0 && cols > 0 && cols % 32 == 0);
  if (rows == 0 || n == 0) return ILT_OK;
  ILT_REQUIRE(wq && wd && xq && xs && y && ((uintptr_t)wq & 15) == 0 && ((uintptr_t)xq & 15) == 0 && cols % 16 == 0);
  return (int)ilt_k_gemm_i8(ILT_Q8_0, (const uint8_t*)wq, wd, cols, rows, cols, xq, xs, nullptr, n, y, bias, acc, S(stream));
}

int ilt_mm_q8_mma2(uint64_t stream, const int8_t* w0, const uint16_t* d0, float* y0, const float* b0, int rows0, const int8_t* w1,
                   const uint16_t* d1, float* y1, const float* b1, int rows1, const int8_t* w2, const uint16_t* d2, float* y2,
                   const float* b2, int rows2, const int8_t* xq, const float* xs, int cols, int n, int acc) {
  // a matrix of no rows (or a null one) takes no part, as in the reference's grid
  const int8_t* ws[3] = {w0, w1, w2}; const uint16_t* ds[3] = {d0, d1, d2}; float* ys[3] = {y0, y1, y2};
  const float* bs[3] = {b0, b1, b2}; const int rows[3] = {rows0, rows1, rows2};
  for (int i = 0; i < 3; i++) {
    ILT_REQUIRE(rows[i] >= 0);
    if (rows[i] == 0 || !ws[i]) continue;
    const int e = ilt_mm_q8(stream, ws[i], ds[i], xq, xs, ys[i], bs[i], rows[i], cols, n, acc);
    if (e != ILT_OK) return e;
  }
  return ILT_OK;
}

int ilt_d4_mvq8n(uint64_t stream, int rows, int cols, int group_rows, int ntok, int x_tstride, int y_tstride, const int8_t* wq,
                 const uint16_t* wd, const int8_t* xq, const float* xs, float* y) {
  ILT_REQUIRE(ntok >= 0 && ntok <= 9 && x_tstride >= 0 && x_tstride % 32 == 0 && y_tstride >= 0 && cols > 0 && cols % 32 == 0);
  for (int t = 0; t < ntok; t++) {
    const int e = ilt_d4_mvq8(stream, rows, cols, group_rows, wq, wd, xq + (long long)t * x_tstride, xs + (long long)t * x_tstride / 32,
                              y + (long long)t * y_tstride);
    if (e != ILT_OK) return e;
  }
  return ILT_OK;
}

int ilt_mm_k(uint64_t stream, int type, const void* w, const int8_t* xq, const float* xd, const int32_t* bsums, float* y,
             const float* bias, int rows, int cols, int n, int acc) {
  const int fmt = kquant_type(type);
  ILT_REQUIRE(fmt && rows >= 0 && n >= 0 && cols > 0 && cols % 256 == 0);
  if (rows == 0 || n == 0) return ILT_OK;
  ILT_REQUIRE(w && xq && xd && bsums && y && ((uintptr_t)w & 15) == 0 && ((uintptr_t)xq & 15) == 0);
  return (int)ilt_k_gemm_i8(fmt, (const uint8_t*)w, nullptr, (long long)cols / 256 * block_bytes(fmt), rows, cols, xq, xd,
                            bsums, n, y, bias, acc, S(stream));
}

// Up to three K-quant matrices of one type on the same tokens (what mm_q8_mma2 is for Q8_0, cuda-dense.lisp:250-258):
// one launch when the shapes allow it, else one after another; a matrix of no rows (or a null one) takes no part.
int ilt_mm_k_n(uint64_t stream, int type, const void* w0, float* y0, const float* b0, int rows0, const void* w1, float* y1, const float* b1,
               int rows1, const void* w2, float* y2, const float* b2, int rows2, const int8_t* xq, const float* xd, const int32_t* bsums,
               int cols, int n, int acc) {
  const int fmt = kquant_type(type);
  ILT_REQUIRE(fmt && n >= 0 && cols > 0 && cols % 256 == 0 && rows0 >= 0 && rows1 >= 0 && rows2 >= 0);
  const void* wsrc[3] = {w0, w1, w2}; float* ysrc[3] = {y0, y1, y2}; const float* bsrc[3] = {b0, b1, b2}; const int rsrc[3] = {rows0, rows1, rows2};
  const uint8_t* ws[3]; float* ys[3]; const float* bs[3]; int rows[3], nm = 0;
  for (int i = 0; i < 3; i++) {
    if (rsrc[i] == 0 || !wsrc[i]) continue;
    ILT_REQUIRE(ysrc[i] && ((uintptr_t)wsrc[i] & 15) == 0);
    ws[nm] = (const uint8_t*)wsrc[i]; ys[nm] = ysrc[i]; bs[nm] = bsrc[i]; rows[nm] = rsrc[i]; nm++;
  }
  if (nm == 0 || n == 0) return ILT_OK;
  ILT_REQUIRE(xq && xd && bsums && ((uintptr_t)xq & 15) == 0);
  const long long row_bytes = (long long)cols / 256 * block_bytes(fmt);
  const hipError_t e = ilt_k_gemm_i8_planes_n(fmt, nm, ws, rows, ys, bs, row_bytes, cols, xq, xd, bsums, n, acc, S(stream));
  if (e != hipErrorNotSupported) return (int)e;
  for (int i = 0; i < nm; i++) {
    const int r = ilt_mm_k(stream, type, ws[i], xq, xd, bsums, ys[i], bs[i], rows[i], cols, n, acc);
    if (r != ILT_OK) return r;
  }
  return ILT_OK;
}

static int mm_id(uint64_t stream, int fmt, int ncols, int nrows, int row_bytes, int64_t add, const uint64_t* ptrs,
                 const uint32_t* counts, const uint32_t* bases, int ne, int64_t total_rows, const int8_t* xq,
                 const float* xd, const int32_t* bsums, float* y) {
  ILT_REQUIRE(ncols > 0 && ncols % 256 == 0 && nrows >= 0 && ne >= 0 && ne <= 256 && total_rows >= 0);
  ILT_REQUIRE(row_bytes == ncols / 256 * block_bytes(fmt) && add >= 0 && (add & 1) == 0);
  if (nrows == 0 || ne == 0 || total_rows == 0) return ILT_OK;
  ILT_REQUIRE(ptrs && counts && bases && xq && xd && y && (bsums || fmt == ILT_IQ2_XXS) && ((uintptr_t)xq & 15) == 0);
  return (int)ilt_k_gemm_i8_id(fmt, ptrs, add, counts, bases, ne, row_bytes, nrows, ncols, xq, xd, bsums, total_rows, y, S(stream));
}

int ilt_d4_mm_id_iq2_xxs(uint64_t stream, int ncols, int nrows, int row_bytes, int64_t add, const uint64_t* ptrs,
                         const uint32_t* counts, const uint32_t* bases, int ne, int64_t total_rows,
                         const int8_t* xq, const float* xd, float* y) {
  return mm_id(stream, ILT_IQ2_XXS, ncols, nrows, row_bytes, add, ptrs, counts, bases, ne, total_rows, xq, xd, nullptr, y);
}

int ilt_d4_mm_id_q2_k(uint64_t stream, int ncols, int nrows, int row_bytes, int64_t add, const uint64_t* ptrs,
                      const uint32_t* counts, const uint32_t* bases, int ne, int64_t total_rows,
                      const int8_t* xq, const float* xd, const int32_t* bsums, float* y) {
  return mm_id(stream, ILT_Q2_K, ncols, nrows, row_bytes, add, ptrs, counts, bases, ne, total_rows, xq, xd, bsums, y);
}

// ---- d4_mm_<format>: one matrix on a chunk of tokens' float activations (ds4f_mm.cu:252-255) ----------
// The reference's kernels round weights and activations to halves; these quantize the activations as the CPU
// path does and run the exact products, so the quantized activations need room: a buffer per (device, stream) that
// only ever grows, kept until the process ends -- calls that overlap on one GPU are on different streams, and each
// stream's calls have a buffer to themselves (sixteen of them at most; a seventeenth stream is refused).  Growing frees
// and allocates, which waits for the stream and cannot happen while it is being captured (refused then): a caller that
// captures, or that wants no such stall in its loop, sizes the buffers beforehand -- ilt_d4_mm_reserve for every buffer
// made from then on and the ones there are, ilt_d4_mm_reserve_stream for one stream's at once.
namespace {
struct QRoom { int dev; hipStream_t st; void* p; size_t bytes; };
QRoom g_qroom[16];
int g_nqrooms = 0;
size_t g_qroom_min = 0;
std::mutex g_qroom_mu;
size_t qroom_bytes(int fmt, size_t ntok, size_t ncols) {
  const size_t n = ntok * ncols, bw = fmt == ILT_Q8_0 ? 32 : 256;
  return (n + 255) / 256 * 256 + (n / bw * 4 + 255) / 256 * 256 + (fmt == ILT_Q8_0 ? 0 : (n / 16 * 4 + 255) / 256 * 256);
}
// (the lock held) the stream's buffer grown to BYTES
int qroom_grow(QRoom& q, size_t bytes) {
  if (q.bytes >= bytes) return ILT_OK;
  hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
  ILT_TRY(hipStreamIsCapturing(q.st, &cs));
  if (cs != hipStreamCaptureStatusNone) return (int)hipErrorStreamCaptureUnsupported;
  if (q.p) {
    ILT_TRY(hipStreamSynchronize(q.st));                 // the stream's earlier calls may still read the old buffer
    ILT_TRY(hipFree(q.p));
  }
  q.p = nullptr; q.bytes = 0;
  const size_t want = bytes + bytes / 4 + (1 << 20);
  ILT_TRY(hipMalloc(&q.p, want));
  q.bytes = want;
  return ILT_OK;
}
int qroom(uint64_t stream, size_t bytes, uint8_t** out) {
  int dev = -1;
  ILT_TRY(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(g_qroom_mu);
  QRoom* q = nullptr;
  for (int i = 0; i < g_nqrooms; i++) if (g_qroom[i].dev == dev && g_qroom[i].st == S(stream)) q = &g_qroom[i];
  if (!q) {
    if (g_nqrooms == 16) return (int)hipErrorOutOfMemory;
    q = &g_qroom[g_nqrooms];
    *q = {dev, S(stream), nullptr, 0};
    const int e = qroom_grow(*q, bytes > g_qroom_min ? bytes : g_qroom_min);
    if (e != ILT_OK) return e;
    g_nqrooms++;
  } else {
    const int e = qroom_grow(*q, bytes);
    if (e != ILT_OK) return e;
  }
  if (out) *out = (uint8_t*)q->p;
  return ILT_OK;
}
int d4_mm_quantized(uint64_t stream, int fmt, int ncols, int nrows, int ntok, int row_bytes, int x_stride, int y_stride, const void* w,
                    const uint16_t* wd, const float* x, float* y) {
  const int bw = block_weights(fmt);
  ILT_REQUIRE(ncols > 0 && ncols % bw == 0 && nrows >= 0 && ntok >= 0);
  if (nrows == 0 || ntok == 0) return ILT_OK;
  // a token's ncols floats start x_stride floats after the token before's, its nrows results y_stride floats after
  // (the grouped attention output product reads a slice of each token's heads and writes a slice of its low rows,
  // cuda-ds4f-prefill.lisp:277-281); the quantized activations are packed
  ILT_REQUIRE(w && x && y && ((uintptr_t)w & 15) == 0 && ((uintptr_t)x & 15) == 0);
  ILT_REQUIRE(x_stride >= ncols && y_stride >= nrows && (fmt == ILT_Q8_0 || x_stride % 4 == 0));
  const size_t n = (size_t)ntok * ncols;
  const size_t qb = (n + 255) / 256 * 256, sb = (n / bw * 4 + 255) / 256 * 256, bb = fmt == ILT_Q8_0 ? 0 : (n / 16 * 4 + 255) / 256 * 256;
  uint8_t* room = nullptr;
  ILT_TRY((hipError_t)qroom(stream, qb + sb + bb, &room));
  int8_t* xq = (int8_t*)room; float* xs = (float*)(room + qb); int32_t* bs = (int32_t*)(room + qb + sb);
  if (fmt == ILT_Q8_0) {
    // d4-shared!'s and the attention projections' activations: quantize-q8! with the scale kept a float (ds4f.lisp:1052-1053)
    ILT_REQUIRE(wd && (row_bytes == 0 || row_bytes == ncols));
    ILT_TRY(ilt_k_quant_rows(0, x, xq, xs, nullptr, ntok, ncols, x_stride, 0, S(stream)));
    return (int)ilt_k_gemm_i8(ILT_Q8_0, (const uint8_t*)w, wd, ncols, nrows, ncols, xq, xs, nullptr, ntok, y, nullptr, 0, S(stream), y_stride);
  }
  ILT_REQUIRE(row_bytes == ncols / 256 * block_bytes(fmt));
  ILT_TRY(ilt_k_quant_rows(1, x, xq, xs, bs, ntok, ncols, x_stride, 0, S(stream)));
  return (int)ilt_k_gemm_i8(fmt, (const uint8_t*)w, nullptr, row_bytes, nrows, ncols, xq, xs, bs, ntok, y, nullptr, 0, S(stream), y_stride);
}
}  // namespace

int ilt_d4_mm_reserve(int ntok, int ncols) {
  ILT_REQUIRE(ntok >= 0 && ncols >= 0);
  const size_t bytes = qroom_bytes(ILT_Q2_K, (size_t)ntok, (size_t)ncols);       // the K formats' layout is the larger one
  int dev = -1;
  ILT_TRY(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(g_qroom_mu);
  if (bytes > g_qroom_min) g_qroom_min = bytes;
  for (int i = 0; i < g_nqrooms; i++)
    if (g_qroom[i].dev == dev) {
      const int e = qroom_grow(g_qroom[i], bytes);
      if (e != ILT_OK) return e;
    }
  return ILT_OK;
}

int ilt_d4_mm_reserve_stream(uint64_t stream, int ntok, int ncols) {
  ILT_REQUIRE(ntok >= 0 && ncols >= 0);
  return qroom(stream, qroom_bytes(ILT_Q2_K, (size_t)ntok, (size_t)ncols), nullptr);
}

int ilt_d4_mm_q8_0(uint64_t stream, int ncols, int nrows, int ntok, int row_bytes, int x_stride, int y_stride, const int8_t* w,
                   const uint16_t* wd, const float* x, float* y) {
  return d4_mm_quantized(stream, ILT_Q8_0, ncols, nrows, ntok, row_bytes, x_stride, y_stride, w, wd, x, y);
}
int ilt_d4_mm_q2_k(uint64_t stream, int ncols, int nrows, int ntok, int row_bytes, int x_stride, int y_stride, const void* w,
                   const float* x, float* y) {
  return d4_mm_quantized(stream, ILT_Q2_K, ncols, nrows, ntok, row_bytes, x_stride, y_stride, w, nullptr, x, y);
}
int ilt_d4_mm_iq2_xxs(uint64_t stream, int ncols, int nrows, int ntok, int row_bytes, int x_stride, int y_stride, const void* w,
                      const float* x, float* y) {
  return d4_mm_quantized(stream, ILT_IQ2_XXS, ncols, nrows, ntok, row_bytes, x_stride, y_stride, w, nullptr, x, y);
}
int ilt_d4_mm_f16(uint64_t stream, int ncols, int nrows, int ntok, int row_bytes, int x_stride, int y_stride, const uint16_t* w,
                  const float* x, float* y) {
  ILT_REQUIRE(ncols > 0 && ncols % 16 == 0 && nrows >= 0 && ntok >= 0 && row_bytes >= 2 * ncols && row_bytes % 2 == 0);
  if (nrows == 0 || ntok == 0) return ILT_OK;
  ILT_REQUIRE(w && x && y && x_stride >= ncols && y_stride >= nrows);
  return (int)ilt_k_mm_f16(ncols, nrows, ntok, row_bytes / 2, x_stride, y_stride, w, x, y, S(stream));
}

static int bf16_type(int t) { return (t == ILT_Q2_K || t == ILT_Q4_K || t == ILT_Q6_K || t == ILT_IQ2_XXS) ? t : 0; }

int ilt_cvt_bf16(uint64_t stream, const float* x, uint16_t* xb, int64_t n) {
  ILT_REQUIRE(n >= 0 && n % 8 == 0);
  if (n == 0) return ILT_OK;
  ILT_REQUIRE(x && xb && ((uintptr_t)x & 15) == 0 && ((uintptr_t)xb & 15) == 0);
  return (int)ilt_k_cvt_bf16(x, xb, n, S(stream));
}

int ilt_q8k_bf16(uint64_t stream, const int8_t* xq, const float* xd, uint16_t* xb, int n, int cols, int slabs) {
  ILT_REQUIRE(n >= 0 && cols > 0 && cols % 256 == 0);
  if (n == 0) return ILT_OK;
  ILT_REQUIRE(xq && xd && xb && ((uintptr_t)xq & 7) == 0 && ((uintptr_t)xb & 15) == 0);
  return (int)ilt_k_q8k_bf16(xq, xd, xb, n, cols, slabs, S(stream));
}

int ilt_mm_k_bf16(uint64_t stream, int gguf_type, const void* w, const uint16_t* xb, float* y, const float* bias,
                  int rows, int cols, int n, int acc) {
  const int fmt = bf16_type(gguf_type);
  ILT_REQUIRE(fmt && rows >= 0 && n >= 0 && cols > 0 && cols % 256 == 0);
  if (rows == 0 || n == 0) return ILT_OK;
  const long long row_bytes = (long long)cols / 256 * block_bytes(fmt);
  ILT_REQUIRE(w && xb && y && ((uintptr_t)w & 1) == 0 && ((uintptr_t)xb & 15) == 0);
  ILT_REQUIRE(row_bytes * rows < 0xFFFFFFF0LL && rows < (1 << 21));
  return (int)ilt_k_gemm_bf16(fmt, (const uint8_t*)w, row_bytes, rows, cols, xb, n, y, bias, acc, S(stream));
}

int ilt_cvt_bf16_slabs(uint64_t stream, const float* x, uint16_t* xs, int n, int cols) {
  ILT_REQUIRE(n >= 0 && cols > 0 && cols % 128 == 0);
  if (n == 0) return ILT_OK;
  ILT_REQUIRE(x && xs && ((uintptr_t)x & 15) == 0 && ((uintptr_t)xs & 15) == 0);
  return (int)ilt_k_cvt_bf16_slabs(x, xs, n, cols, S(stream));
}

int ilt_dequant_bf16(uint64_t stream, int gguf_type, const void* w, uint16_t* wb, int rows, int cols) {
  const int fmt = bf16_type(gguf_type);
  ILT_REQUIRE(fmt && rows >= 0 && cols > 0 && cols % 256 == 0);
  if (rows == 0) return ILT_OK;
  ILT_REQUIRE(w && wb && ((uintptr_t)w & 1) == 0 && ((uintptr_t)wb & 15) == 0);
  ILT_REQUIRE((long long)cols / 256 * block_bytes(fmt) * rows < 0xFFFFFFF0LL);
  return (int)ilt_k_dequant_bf16(fmt, (const uint8_t*)w, (long long)cols / 256 * block_bytes(fmt), rows, cols, wb, S(stream));
}

int ilt_planes_i8(uint64_t stream, int gguf_type, const void* w, int8_t* wh, int8_t* wl, float* wdf, int rows, int cols) {
  const int fmt = bf16_type(gguf_type);
  ILT_REQUIRE(fmt == ILT_Q6_K && rows >= 0 && cols > 0 && cols % 256 == 0);
  if (rows == 0) return ILT_OK;
  ILT_REQUIRE(w && wh && wl && wdf && ((uintptr_t)w & 3) == 0 && ((uintptr_t)wh & 15) == 0 && ((uintptr_t)wl & 15) == 0);
  ILT_REQUIRE((long long)cols / 256 * block_bytes(fmt) * rows < 0xFFFFFFF0LL);
  return (int)ilt_k_planes_i8(fmt, (const uint8_t*)w, (long long)cols / 256 * block_bytes(fmt), rows, cols, (uint8_t*)wh, (uint8_t*)wl, wdf, S(stream));
}

int ilt_mm_i8_planes(uint64_t stream, const int8_t* wh, const int8_t* wl, const float* wdf, const int8_t* xq, const float* xd,
                     float* y, const float* bias, int rows, int cols, int n, int acc) {
  ILT_REQUIRE(rows >= 0 && n >= 0 && cols > 0 && cols % 256 == 0 && cols < (1 << 22) && rows < (1 << 21));
  if (rows == 0 || n == 0) return ILT_OK;
  ILT_REQUIRE(wh && wl && wdf && xq && xd && y && ((uintptr_t)wh & 15) == 0 && ((uintptr_t)wl & 15) == 0 && ((uintptr_t)xq & 15) == 0);
  return (int)ilt_k_gemm_i8_pp((const uint8_t*)wh, (const uint8_t*)wl, wdf, rows, cols, xq, xd, n, y, bias, acc, S(stream));
}

int ilt_mm_bf16(uint64_t stream, const uint16_t* wb, const uint16_t* xb, float* y, const float* bias, int rows, int cols, int n,
                int acc) {
  ILT_REQUIRE(rows >= 0 && n >= 0 && cols > 0 && cols % 128 == 0 && cols < (1 << 22) && rows < (1 << 21));
  if (rows == 0 || n == 0) return ILT_OK;
  ILT_REQUIRE(wb && xb && y && ((uintptr_t)wb & 15) == 0 && ((uintptr_t)xb & 15) == 0);
  return (int)ilt_k_gemm_bf16_plain(wb, rows, cols, xb, n, y, bias, acc, S(stream));
}

int ilt_d4_mm_id_bf16(uint64_t stream, int gguf_type, int ncols, int nrows, int row_bytes, int64_t add, const uint64_t* ptrs,
                      const uint32_t* counts, const uint32_t* bases, int ne, int64_t total_rows,
                      const uint16_t* xb, const uint32_t* rmap, float* y) {
  const int fmt = bf16_type(gguf_type);
  ILT_REQUIRE(fmt && ncols > 0 && ncols % 256 == 0 && nrows >= 0 && ne >= 0 && ne <= 256 && total_rows >= 0);
  ILT_REQUIRE(row_bytes == ncols / 256 * block_bytes(fmt) && add >= 0 && (add & 1) == 0);
  if (nrows == 0 || ne == 0 || total_rows == 0) return ILT_OK;
  ILT_REQUIRE(ptrs && counts && bases && xb && y && ((uintptr_t)xb & 15) == 0 && total_rows < (1LL << 31));
  ILT_REQUIRE((long long)row_bytes * nrows < 0xFFFFFFF0LL && nrows < (1 << 21));
  return (int)ilt_k_gemm_bf16_id(fmt, ptrs, add, counts, bases, ne, row_bytes, nrows, ncols, xb, rmap, total_rows, y, S(stream));
}

int ilt_d4_mm_id_glu_bf16(uint64_t stream, int gguf_type, int ncols, int nrows, int row_bytes, int64_t add_gate, int64_t add_up,
                          const uint64_t* ptrs, const uint32_t* counts, const uint32_t* bases, int ne, int64_t total_rows,
                          const uint16_t* xb, const uint32_t* rmap, float clamp, const float* wrow, uint16_t* mid) {
  const int fmt = bf16_type(gguf_type);
  ILT_REQUIRE(fmt == ILT_IQ2_XXS && ncols > 0 && ncols % 256 == 0 && nrows >= 0 && nrows % 128 == 0 && ne >= 0 && ne <= 256 && total_rows >= 0);
  ILT_REQUIRE(row_bytes == ncols / 256 * block_bytes(fmt) && add_gate >= 0 && (add_gate & 1) == 0 && add_up >= add_gate && (add_up & 1) == 0);
  if (nrows == 0 || ne == 0 || total_rows == 0) return ILT_OK;
  ILT_REQUIRE(ptrs && counts && bases && xb && wrow && mid && ((uintptr_t)xb & 15) == 0 && ((uintptr_t)mid & 1) == 0 && total_rows < (1LL << 31));
  ILT_REQUIRE((long long)row_bytes * nrows + (add_up - add_gate) < 0x7FFFFFFFLL && nrows < (1 << 21));
  return (int)ilt_k_gemm_bf16_id_glu(fmt, ptrs, add_gate, add_up, counts, bases, ne, row_bytes, nrows, ncols, xb, rmap, total_rows, clamp,
                                     wrow, mid, S(stream));
}

// ---- launch by name ---------------------------------------------------------------------------
// ---- between the products of a dense layer (the forward harness) ----------------------------------
int ilt_qk_rope(uint64_t stream, float* q, float* k, const float* v, const float* qn, const float* kn, const float* rope, float* kc,
                float* vc, int nh, int nkv, int hd, int rd, int pos0, float eps, int neox, int ntok) {
  ILT_REQUIRE(ntok >= 0 && (ntok == 0 || (q && k && v && rope && kc && vc)) && pos0 >= 0);
  return (int)ilt_k_qk_rope(q, k, v, qn, kn, rope, kc, vc, nh, nkv, hd, rd, pos0, eps, neox, ntok, S(stream));
}
// ilt_qk_rope and ilt_attn_rows for one token at position pos, as two launches instead of three (the first one
// norms and turns the heads where it needs them and writes the caches' rows); q and k are left as they came
int ilt_attn_step(uint64_t stream, const float* q, const float* k, const float* v, const float* qn, const float* kn, const float* rope, float* kc,
                  float* vc, float* out, int nh, int nkv, int hd, int rd, int pos, float eps, int neox, float* scratch, int nctx) {
  // pos < nctx: the caches' rows at pos are written (kc, vc hold nctx rows); 8192: what the tiled values kernel takes
  ILT_REQUIRE(q && k && v && rope && kc && vc && out && scratch && nh > 0 && nkv > 0 && pos >= 0 && pos < nctx && pos < 8192);
  return (int)ilt_k_attn_step(q, k, v, qn, kn, rope, kc, vc, out, nh, nkv, hd, rd, pos, eps, neox, scratch, S(stream));
}
int ilt_attn_giveups(uint64_t* out) {
  ILT_REQUIRE(out);
  unsigned long long v = 0;
  ILT_TRY(ilt_k_attn_giveups(&v));
  *out = v;
  return ILT_OK;
}
// ARGMAX (model.lisp:464-468) of n floats on the device: the index into out[0] (device memory), so that a greedy
// decode can go on without the logits' trip to the host (the reference picks the token on the host, cuda-dense.lisp:428-430)
int ilt_argmax(uint64_t stream, const float* v, int n, int32_t* out, void* scratch) {
  ILT_REQUIRE(v && out && n > 0 && ((uintptr_t)v & 15) == 0 && ((uintptr_t)scratch & 7) == 0);
  return (int)ilt_k_argmax(v, n, out, scratch, S(stream));
}

// ---- one token through the dense decoder: the launches of the single calls, queued in one ----------
static ilt_mv_desc mv_of(const ilt_dense_mat& w, float* y, const float* bias = nullptr) { return {w.gguf_type, w.rows, w.w, w.wd, y, bias}; }
// A product launch of the decoder, made ready first and queued later: the launches of a layer are known before any of
// them runs, so each can read ahead what the next one will stream (ilt_gemv_plan, IltRowsAhead).
struct DecLaunch { IltGemvParams p; int live; bool planned; };
static int dec_build(DecLaunch& L, int nmat, const ilt_mv_desc* descs, int cols, const float* xf, const float* norm, float eps, int acc, int glu) {
  int fmts[4], rows[4]; const void* ws[4]; const uint16_t* wds[4]; float* ys[4]; const float* bs[4];
  for (int i = 0; i < nmat; i++) {
    fmts[i] = descs[i].gguf_type; rows[i] = descs[i].rows; ws[i] = descs[i].w; wds[i] = descs[i].wd; ys[i] = descs[i].y; bs[i] = descs[i].bias;
  }
  ILT_REQUIRE(xf && (norm || !glu));
  const int e = gemv_multi_build(L.p, &L.live, nmat, fmts, ws, wds, ys, bs, rows, cols, nullptr, nullptr, nullptr, xf, 1, acc, glu, 0, norm, eps, 0);
  if (e != ILT_OK) return e;
  L.planned = L.live > 0 && ilt_gemv_plan(L.p, 1) == hipSuccess;
  return ILT_OK;
}
// next: the launch whose rows this one reads ahead, or null
static int dec_run(DecLaunch& L, const DecLaunch* next, uint64_t stream) {
  if (L.live == 0) return ILT_OK;
  static const bool rows_on = []{ const char* f = getenv("ILT_ROWS_AHEAD"); return !(f && f[0] == '0'); }();
  if (rows_on && L.planned && next && next->planned) ilt_gemv_rows_of(next->p, L.p.rows_ahead);
  return (int)ilt_gemv_launch(L.p, 1, S(stream));
}
// Q/K/V with the norm inside: one launch where the three share an activation format (all Q8_0, or K-quants), else one each
static bool qkv_one_launch(const ilt_dense_layer& L) {
  const bool q = L.wq.gguf_type == ILT_TYPE_Q8_0, k = L.wk.gguf_type == ILT_TYPE_Q8_0, v = L.wv.gguf_type == ILT_TYPE_Q8_0;
  return q == k && k == v;
}
static int dec_build_qkv(DecLaunch& Q, const ilt_dense_model* m, const ilt_dense_layer& L) {
  const ilt_mv_desc qkv[3] = {mv_of(L.wq, m->q, L.bq), mv_of(L.wk, m->k, L.bk), mv_of(L.wv, m->v, L.bv)};
  return dec_build(Q, 3, qkv, m->d, m->x, L.attn_norm, m->eps, 0, 0);
}
int ilt_dense_decode(uint64_t stream, const ilt_dense_model* m, const int32_t* token, int pos, int want_logits) {
  ILT_REQUIRE(m && token && m->layers && m->nl > 0 && pos >= 0 && pos < m->nctx && pos < 8192);
  ILT_REQUIRE(m->x && m->q && m->k && m->v && m->att && m->fa && m->scores && m->rope && (!want_logits || (m->logits && m->output_norm)));
  int e;
  if (m->embd.gguf_type == ILT_TYPE_Q8_0) e = ilt_embed_q8(stream, (const int8_t*)m->embd.w, m->embd.wd, token, m->x, m->d, 1);
  else e = ilt_embed_k(stream, m->embd.gguf_type == ILT_TYPE_Q4_K ? 0 : m->embd.gguf_type == ILT_TYPE_Q6_K ? 2 : -1, m->embd.w, token, m->x, m->d, 1);
  if (e) return e;
  DecLaunch qkv = {}, wo = {}, glu = {}, down = {};
  for (int l = 0; l < m->nl; l++) {
    const ilt_dense_layer& L = m->layers[l];
    const bool one = qkv_one_launch(L);
    if (one && (e = dec_build_qkv(qkv, m, L))) return e;
    const ilt_mv_desc dwo = mv_of(L.wo, m->x), dglu[2] = {mv_of(L.gate, m->fa), mv_of(L.up, m->fa)}, ddown = mv_of(L.down, m->x);
    if ((e = dec_build(wo, 1, &dwo, L.wo.cols, m->att, nullptr, 0.0f, 1, 0))) return e;
    if ((e = dec_build(glu, 2, dglu, m->d, m->x, L.ffn_norm, m->eps, 0, 1))) return e;
    if ((e = dec_build(down, 1, &ddown, L.down.cols, m->fa, nullptr, 0.0f, 1, 0))) return e;
    // the attention's keys and values read ahead into the L2 of the die whose workgroups will want them (the one-launch
    // attention deals a die consecutive heads: attn_step_fused_kernel's mapping), with the table's row and the head norms
    IltCacheAhead ahead = {};
    static const bool ahead_on = []{ const char* f = getenv("ILT_CACHE_AHEAD"); return !(f && f[0] == '0'); }();
    const int nwg = m->nh * (m->hd / 16);
    if (ahead_on && pos > 0 && pos < 1024 && (m->hd == 64 || m->hd == 128) && nwg % 8 == 0 && m->nkv > 0 && m->nh % m->nkv == 0) {
      const int ns = m->hd / 16, group = m->nh / m->nkv;
      ahead.a = L.kc; ahead.b = L.vc; ahead.stride = m->nkv * m->hd; ahead.nrows = pos;
      for (int x = 0; x < 8; x++) {
        const int h0 = x * (nwg / 8) / ns, h1 = ((x + 1) * (nwg / 8) - 1) / ns, k0 = h0 / group, k1 = h1 / group;
        ahead.off[x] = k0 * m->hd; ahead.width[x] = (k1 - k0 + 1) * m->hd;
      }
      ahead.small[0] = m->rope + (long long)pos * m->rd; ahead.nsmall[0] = m->rd;
      ahead.small[1] = L.q_norm; ahead.nsmall[1] = m->hd;
      ahead.small[2] = L.k_norm; ahead.nsmall[2] = m->hd;
    }
    if (one) {
      qkv.p.ahead = ahead;
      if ((e = dec_run(qkv, nullptr, stream))) return e;
    } else {
      const ilt_mv_desc d3[3] = {mv_of(L.wq, m->q, L.bq), mv_of(L.wk, m->k, L.bk), mv_of(L.wv, m->v, L.bv)};
      for (int i = 0; i < 3; i++)
        if ((e = ilt_mv_multi_norm(stream, 1, &d3[i], m->d, m->x, L.attn_norm, m->eps, 0, 1, 0))) return e;
    }
    if ((e = ilt_attn_step(stream, m->q, m->k, m->v, L.q_norm, L.k_norm, m->rope, L.kc, L.vc, m->att, m->nh, m->nkv, m->hd, m->rd, pos, m->eps,
                           m->neox, m->scores, m->nctx))) return e;
    // gate/up's launch reads down's rows ahead: it is the one launch long enough after its own rows are in (the terms
    // of both matrices' rows, two sums a row and the gated activation) for the next matrix to arrive meanwhile.  The
    // other links of the chain -- Q/K/V reading wo's rows ahead, wo gate/up's, down the next layer's Q/K/V's -- lengthen
    // the reading launch by more than the next one gains (at the Qwen3-4B shape 541 to 549 tok/s against 555 without any;
    // this link alone: 563)
    if ((e = dec_run(wo, nullptr, stream))) return e;
    if ((e = dec_run(glu, &down, stream))) return e;
    if ((e = dec_run(down, nullptr, stream))) return e;
  }
  if (want_logits) {
    const ilt_mv_desc head = mv_of(m->output, m->logits);
    if ((e = ilt_mv_multi_norm(stream, 1, &head, m->d, m->x, m->output_norm, m->eps, 0, 1, 0))) return e;
  }
  return ILT_OK;
}

// rope-table (model.lisp:218-231) for positions pos0 .. pos0 + n - 1, on the host: a position's head_dim/2 cosines
// then head_dim/2 sines, theta advanced by repeated single-float multiplication, theta-scale, cos and sin through
// double and rounded to single as SBCL evaluates them.  The only float arithmetic this file does: model constants,
// made once and uploaded by the caller; nothing here can overflow or trap.
int ilt_rope_table(int head_dim, int pos0, int n, float base, float* out) {
  ILT_REQUIRE(out && head_dim >= 2 && head_dim % 2 == 0 && pos0 >= 0 && n >= 0 && base > 0.0f);
  const int half = head_dim / 2;
  const float e = -2.0f / (float)head_dim;
  const float theta_scale = (float)pow((double)base, (double)e);
  for (int p = 0; p < n; p++) {
    float theta = (float)(pos0 + p);
    float* row = out + (size_t)p * head_dim;
    for (int i = 0; i < half; i++) {
      row[i] = (float)cos((double)theta); row[half + i] = (float)sin((double)theta);
      const volatile float next = theta * theta_scale;
      theta = next;
    }
  }
  return ILT_OK;
}
int ilt_attn_rows(uint64_t stream, const float* q, const float* kc, const float* vc, float* out, int nh, int nkv, int hd, int pos0, int ntok,
                  float* scratch) {
  ILT_REQUIRE(ntok >= 0 && (ntok == 0 || (q && kc && vc && out)) && nh > 0 && nkv > 0);
  return (int)ilt_k_attn_rows(q, kc, vc, out, nh, nkv, hd, pos0, ntok, scratch, S(stream));
}
int ilt_swiglu(uint64_t stream, float* a, const float* b, int64_t n) {
  ILT_REQUIRE(n >= 0 && (n == 0 || (a && b)));
  return (int)ilt_k_swiglu_rows(a, b, n, S(stream));
}
int ilt_swiglu_quant_q8k(uint64_t stream, const float* gate, const float* up, int8_t* xq, float* xd, int32_t* bsums, int64_t nblocks) {
  ILT_REQUIRE(nblocks >= 0 && (nblocks == 0 || (gate && up && xq && xd && bsums)));
  ILT_REQUIRE(((((uintptr_t)gate) | ((uintptr_t)up)) & 15) == 0);
  return (int)ilt_k_swiglu_quant_q8k(gate, up, xq, xd, bsums, nblocks, S(stream));
}

int ilt_launch(const char* kernel, unsigned gx, unsigned gy, unsigned gz, unsigned bx, unsigned by, unsigned bz,
               unsigned shared_bytes, uint64_t stream, void** params) {
  ILT_REQUIRE(kernel && params);
  (void)bx; (void)by; (void)bz; (void)shared_bytes;
  const Args a = { params };
  typedef const int8_t* ci8; typedef const uint16_t* cu16; typedef const float* cf; typedef const uint32_t* cu32;
#define K(name) if (!strcmp(kernel, name))
  K("repack_q8") return ilt_repack_q8(stream, a.ptr<const void*>(0), a.ptr<void*>(1), a.ptr<void*>(2), a.i64(3));
  K("repack_q6k") return ilt_repack_q6k(stream, a.ptr<const void*>(0), a.ptr<void*>(1), a.i64(2));
  K("quant_q8") return ilt_quant_q8(stream, a.ptr<cf>(0), a.ptr<int8_t*>(1), a.ptr<float*>(2), a.ptr<int32_t*>(3), a.i64(4));
  K("d4_quant") return ilt_d4_quant(stream, a.ptr<cf>(0), a.ptr<int8_t*>(1), a.ptr<float*>(2), a.i32(3));
  K("quant_q8k") return ilt_quant_q8k(stream, a.ptr<cf>(0), a.ptr<int8_t*>(1), a.ptr<float*>(2), a.ptr<int32_t*>(3), a.i64(4));
  K("rmsnorm_q8") return ilt_rmsnorm_q8(stream, a.ptr<cf>(0), a.ptr<cf>(1), a.ptr<float*>(2), a.ptr<int8_t*>(3), a.ptr<float*>(4),
                                        a.ptr<int32_t*>(5), a.i32(6), a.f32(7), (int)gy, 0);
  K("mv_q8") return ilt_mv_q8(stream, a.ptr<ci8>(0), a.ptr<cu16>(1), a.ptr<ci8>(2), a.ptr<cf>(3), a.ptr<float*>(4),
                              a.ptr<cf>(5), a.i32(6), a.i32(7), a.i32(8));
  K("mv_q8_3") return ilt_mv_q8_3(stream, a.ptr<ci8>(0), a.ptr<cu16>(1), a.ptr<ci8>(2), a.ptr<cu16>(3), a.ptr<ci8>(4),
                                  a.ptr<cu16>(5), a.ptr<ci8>(6), a.ptr<cf>(7), a.ptr<float*>(8), a.ptr<float*>(9),
                                  a.ptr<float*>(10), a.ptr<cf>(11), a.ptr<cf>(12), a.ptr<cf>(13), a.i32(14), a.i32(15),
                                  a.i32(16), a.i32(17));
  K("mv_k") return ilt_mv_k(stream, a.i32(0), a.ptr<const void*>(1), a.ptr<ci8>(2), a.ptr<cf>(3), a.ptr<const int32_t*>(4),
                            a.ptr<float*>(5), a.ptr<cf>(6), a.i32(7), a.i32(8), a.i32(9));
  if (!strcmp(kernel, "mm_q8") || !strcmp(kernel, "mm_q8_mma"))
    return ilt_mm_q8(stream, a.ptr<ci8>(0), a.ptr<cu16>(1), a.ptr<ci8>(2), a.ptr<cf>(3), a.ptr<float*>(4), a.ptr<cf>(5),
                     a.i32(6), a.i32(7), a.i32(8), a.i32(9));
  K("mm_q8_mma2")
    return ilt_mm_q8_mma2(stream, a.ptr<ci8>(0), a.ptr<cu16>(1), a.ptr<float*>(2), a.ptr<cf>(3), a.i32(4), a.ptr<ci8>(5), a.ptr<cu16>(6),
                          a.ptr<float*>(7), a.ptr<cf>(8), a.i32(9), a.ptr<ci8>(10), a.ptr<cu16>(11), a.ptr<float*>(12), a.ptr<cf>(13),
                          a.i32(14), a.ptr<ci8>(15), a.ptr<cf>(16), a.i32(17), a.i32(18), a.i32(19));
  K("d4_mvq8n") return ilt_d4_mvq8n(stream, a.i32(0), a.i32(1), a.i32(2), a.i32(3), a.i32(4), a.i32(5), a.ptr<ci8>(6), a.ptr<cu16>(7),
                                    a.ptr<ci8>(8), a.ptr<cf>(9), a.ptr<float*>(10));
  K("mm_k_n")
    return ilt_mm_k_n(stream, a.i32(0), a.ptr<const void*>(1), a.ptr<float*>(2), a.ptr<cf>(3), a.i32(4), a.ptr<const void*>(5), a.ptr<float*>(6),
                      a.ptr<cf>(7), a.i32(8), a.ptr<const void*>(9), a.ptr<float*>(10), a.ptr<cf>(11), a.i32(12), a.ptr<ci8>(13), a.ptr<cf>(14),
                      a.ptr<const int32_t*>(15), a.i32(16), a.i32(17), a.i32(18));
  K("mm_k") return ilt_mm_k(stream, a.i32(0), a.ptr<const void*>(1), a.ptr<ci8>(2), a.ptr<cf>(3), a.ptr<const int32_t*>(4),
                            a.ptr<float*>(5), a.ptr<cf>(6), a.i32(7), a.i32(8), a.i32(9), a.i32(10));
  if (!strcmp(kernel, "mm_q4k_mma") || !strcmp(kernel, "mm_q6k_mma"))
    return ilt_mm_k(stream, kernel[4] == '4' ? 0 : 2, a.ptr<const void*>(0), a.ptr<ci8>(1), a.ptr<cf>(2),
                    a.ptr<const int32_t*>(3), a.ptr<float*>(4), a.ptr<cf>(5), a.i32(6), a.i32(7), a.i32(8), a.i32(9));
  K("q8k_bf16") return ilt_q8k_bf16(stream, a.ptr<ci8>(0), a.ptr<cf>(1), a.ptr<uint16_t*>(2), a.i32(3), a.i32(4), a.i32(5));
  K("cvt_bf16") return ilt_cvt_bf16(stream, a.ptr<cf>(0), a.ptr<uint16_t*>(1), a.i64(2));
  K("mm_k_bf16") return ilt_mm_k_bf16(stream, a.i32(0), a.ptr<const void*>(1), a.ptr<cu16>(2), a.ptr<float*>(3), a.ptr<cf>(4),
                                      a.i32(5), a.i32(6), a.i32(7), a.i32(8));
  K("cvt_bf16_slabs") return ilt_cvt_bf16_slabs(stream, a.ptr<cf>(0), a.ptr<uint16_t*>(1), a.i32(2), a.i32(3));
  K("planes_i8") return ilt_planes_i8(stream, a.i32(0), a.ptr<const void*>(1), a.ptr<int8_t*>(2), a.ptr<int8_t*>(3), a.ptr<float*>(4), a.i32(5), a.i32(6));
  K("mm_i8_planes")
    return ilt_mm_i8_planes(stream, a.ptr<ci8>(0), a.ptr<ci8>(1), a.ptr<cf>(2), a.ptr<ci8>(3), a.ptr<cf>(4), a.ptr<float*>(5),
                            a.ptr<cf>(6), a.i32(7), a.i32(8), a.i32(9), a.i32(10));
  K("dequant_bf16") return ilt_dequant_bf16(stream, a.i32(0), a.ptr<const void*>(1), a.ptr<uint16_t*>(2), a.i32(3), a.i32(4));
  K("mm_bf16") return ilt_mm_bf16(stream, a.ptr<cu16>(0), a.ptr<cu16>(1), a.ptr<float*>(2), a.ptr<cf>(3), a.i32(4), a.i32(5), a.i32(6), a.i32(7));
  K("d4_mm_id_bf16")
    return ilt_d4_mm_id_bf16(stream, a.i32(0), a.i32(1), a.i32(2), a.i32(3), a.i64(4), a.ptr<const uint64_t*>(5), a.ptr<cu32>(6),
                             a.ptr<cu32>(7), a.i32(8), a.i64(9), a.ptr<cu16>(10), a.ptr<cu32>(11), a.ptr<float*>(12));
  K("d4_mm_id_glu_bf16")
    return ilt_d4_mm_id_glu_bf16(stream, a.i32(0), a.i32(1), a.i32(2), a.i32(3), a.i64(4), a.i64(5), a.ptr<const uint64_t*>(6), a.ptr<cu32>(7),
                                 a.ptr<cu32>(8), a.i32(9), a.i64(10), a.ptr<cu16>(11), a.ptr<cu32>(12), a.f32(13), a.ptr<cf>(14), a.ptr<uint16_t*>(15));
  K("d4_swiglu_w_bf16") return ilt_d4_swiglu_w_bf16(stream, a.i32(0), a.i32(1), a.f32(2), a.ptr<cf>(3), a.ptr<cf>(4), a.ptr<cf>(5), a.ptr<uint16_t*>(6));
  K("qk_rope") return ilt_qk_rope(stream, a.ptr<float*>(0), a.ptr<float*>(1), a.ptr<cf>(2), a.ptr<cf>(3), a.ptr<cf>(4), a.ptr<cf>(5), a.ptr<float*>(6),
                                  a.ptr<float*>(7), a.i32(8), a.i32(9), a.i32(10), a.i32(11), a.i32(12), a.f32(13), a.i32(14), (int)gy);
  K("swiglu") return ilt_swiglu(stream, a.ptr<float*>(0), a.ptr<cf>(1), a.i64(2));
  // The reference's attention launches by their names and slots (cuda-dense.lisp:341-364; dense.cu:376, 482, 517, 727),
  // computed in the CPU's float order: attn_decode leaves one token's finished heads in PART (its split of the keys and
  // its partial sums have no counterpart here: chunk, nsplit and scale are read past), attn_merge moves them to ATT and
  // quantizes them for a Q8_0 output projection when XQ is given; attn_prefill / attn_prefill2 are a chunk's attn_rows.
  K("attn_decode") return ilt_attn_rows(stream, a.ptr<cf>(0), a.ptr<cf>(1), a.ptr<cf>(2), a.ptr<float*>(3), a.i32(4), a.i32(5), a.i32(6), a.i32(7), 1, nullptr);
  K("attn_merge") {
    const int nh = a.i32(5), hd = a.i32(6), ntok = gy ? (int)gy : 1;
    ILT_REQUIRE(a.ptr<cf>(0) && a.ptr<float*>(1) && nh > 0 && hd > 0 && (long long)nh * hd % 32 == 0);
    const uint64_t bytes = 4ull * nh * hd * ntok;
    ILT_TRY((hipError_t)ilt_memcpy_dtod_async((uint64_t)(uintptr_t)a.ptr<float*>(1), (uint64_t)(uintptr_t)a.ptr<cf>(0), bytes, stream));
    if (!a.ptr<int8_t*>(2)) return ILT_OK;
    return ilt_quant_q8(stream, a.ptr<cf>(1), a.ptr<int8_t*>(2), a.ptr<float*>(3), a.ptr<int32_t*>(4), (int64_t)nh * hd * ntok / 32);
  }
  if (!strcmp(kernel, "attn_prefill") || !strcmp(kernel, "attn_prefill2"))
    return ilt_attn_rows(stream, a.ptr<cf>(0), a.ptr<cf>(1), a.ptr<cf>(2), a.ptr<float*>(3), a.i32(4), a.i32(5), a.i32(6), a.i32(7), a.i32(8), nullptr);
  K("attn_rows") return ilt_attn_rows(stream, a.ptr<cf>(0), a.ptr<cf>(1), a.ptr<cf>(2), a.ptr<float*>(3), a.i32(4), a.i32(5), a.i32(6), a.i32(7), (int)gy, a.ptr<float*>(8));
  K("argmax") return ilt_argmax(stream, a.ptr<cf>(0), a.i32(1), a.ptr<int32_t*>(2), a.ptr<void*>(3));
  K("attn_step") return ilt_attn_step(stream, a.ptr<cf>(0), a.ptr<cf>(1), a.ptr<cf>(2), a.ptr<cf>(3), a.ptr<cf>(4), a.ptr<cf>(5), a.ptr<float*>(6),
                                      a.ptr<float*>(7), a.ptr<float*>(8), a.i32(9), a.i32(10), a.i32(11), a.i32(12), a.i32(13), a.f32(14), a.i32(15),
                                      a.ptr<float*>(16), a.i32(17));
  K("d4_rows_expert") return ilt_d4_rows_expert(stream, a.i32(0), a.ptr<cu32>(1), a.ptr<cu32>(2), a.ptr<uint32_t*>(3));
  K("d4_mm_q8_0") return ilt_d4_mm_q8_0(stream, a.i32(0), a.i32(1), a.i32(2), a.i32(3), a.i32(4), a.i32(5), a.ptr<ci8>(6), a.ptr<cu16>(7), a.ptr<cf>(8), a.ptr<float*>(9));
  K("d4_mm_f16") return ilt_d4_mm_f16(stream, a.i32(0), a.i32(1), a.i32(2), a.i32(3), a.i32(4), a.i32(5), a.ptr<cu16>(6), a.ptr<cf>(8), a.ptr<float*>(9));
  K("d4_mm_q2_k") return ilt_d4_mm_q2_k(stream, a.i32(0), a.i32(1), a.i32(2), a.i32(3), a.i32(4), a.i32(5), a.ptr<const void*>(6), a.ptr<cf>(8), a.ptr<float*>(9));
  K("d4_mm_iq2_xxs") return ilt_d4_mm_iq2_xxs(stream, a.i32(0), a.i32(1), a.i32(2), a.i32(3), a.i32(4), a.i32(5), a.ptr<const void*>(6), a.ptr<cf>(8), a.ptr<float*>(9));
  K("d4_mm_id_iq2_xxs")
    return ilt_d4_mm_id_iq2_xxs(stream, a.i32(0), a.i32(1), a.i32(2), a.i64(5), a.ptr<const uint64_t*>(6), a.ptr<cu32>(7),
                                a.ptr<cu32>(8), (int)gz, a.i64(13), a.ptr<ci8>(9), a.ptr<cf>(11), a.ptr<float*>(10));
  K("d4_mm_id_q2_k")
    return ilt_d4_mm_id_q2_k(stream, a.i32(0), a.i32(1), a.i32(2), a.i64(5), a.ptr<const uint64_t*>(6), a.ptr<cu32>(7),
                             a.ptr<cu32>(8), (int)gz, a.i64(13), a.ptr<ci8>(9), a.ptr<cf>(11), a.ptr<const int32_t*>(12),
                             a.ptr<float*>(10));
  K("mv_q8_glu") return ilt_mv_q8_glu(stream, a.ptr<ci8>(0), a.ptr<cu16>(1), a.ptr<ci8>(2), a.ptr<cu16>(3), a.ptr<ci8>(4),
                                      a.ptr<cf>(5), a.ptr<float*>(6), a.i32(7), a.i32(8));
  K("mv_k_glu") return ilt_mv_k_glu(stream, a.i32(0), a.ptr<const void*>(1), a.i32(2), a.ptr<const void*>(3), a.ptr<ci8>(4),
                                    a.ptr<cf>(5), a.ptr<const int32_t*>(6), a.ptr<float*>(7), a.i32(8), a.i32(9));
  K("d4_mv_glu_iq2_xxs")
    return ilt_d4_mv_glu_iq2_xxs(stream, a.i32(0), a.i32(1), a.i32(2), a.i64(3), a.i64(4), a.i32(5), a.i32(6),
                                 a.ptr<const uint64_t*>(7), a.ptr<cu32>(8), (int)gz, a.ptr<cf>(9), a.ptr<cf>(10), a.f32(11), a.ptr<float*>(12));
  K("d4_mv_q2_k_f32")
    return ilt_d4_mv_q2_k_f32(stream, a.i32(0), a.i32(1), a.i32(2), a.i64(3), a.i32(4), a.i32(5), a.ptr<const uint64_t*>(6),
                              a.ptr<cu32>(7), (int)gz, a.ptr<cf>(8), a.ptr<float*>(9));
  K("d4_mvq8_glu") return ilt_d4_mvq8_glu(stream, a.i32(0), a.i32(1), a.ptr<ci8>(2), a.ptr<cu16>(3), a.ptr<ci8>(4), a.ptr<cu16>(5),
                                          a.ptr<cf>(6), a.f32(7), a.ptr<float*>(8));
  K("d4_mvq8") return ilt_d4_mvq8(stream, a.i32(0), a.i32(1), a.i32(2), a.ptr<ci8>(3), a.ptr<cu16>(4), a.ptr<ci8>(5),
                                  a.ptr<cf>(6), a.ptr<float*>(7));
  // d4_mv_iq2_xxs / d4_mv_q2_k: the reference's twelve slots (ds4f.cu:769-772, 837-840), float rows in
  K("d4_mv_iq2_xxs")
    return ilt_d4_mv_rows_iq2_xxs(stream, a.i32(0), a.i32(1), a.i32(2), a.i64(3), a.i32(4), a.i32(5), a.ptr<const uint64_t*>(6),
                                  a.ptr<const uint64_t*>(7), (int)gz, a.ptr<cf>(8), a.ptr<float*>(9), a.ptr<cu32>(10), a.ptr<cu32>(11));
  K("d4_mv_q2_k")
    return ilt_d4_mv_rows_q2_k(stream, a.i32(0), a.i32(1), a.i32(2), a.i64(3), a.i32(4), a.i32(5), a.ptr<const uint64_t*>(6),
                               a.ptr<const uint64_t*>(7), (int)gz, a.ptr<cf>(8), a.ptr<float*>(9), a.ptr<cu32>(10), a.ptr<cu32>(11));
  // the same on activations quantized beforehand (quant_q8k): slot 7 unused, slots 8, 10, 11 = xq, xd, bsums
  K("d4_mvq_iq2_xxs")
    return ilt_d4_mv_iq2_xxs(stream, a.i32(0), a.i32(1), a.i32(2), a.i64(3), a.i32(4), a.i32(5), a.ptr<const uint64_t*>(6),
                             (int)gz, a.ptr<ci8>(8), a.ptr<cf>(10), a.ptr<float*>(9));
  K("d4_mvq_q2_k")
    return ilt_d4_mv_q2_k(stream, a.i32(0), a.i32(1), a.i32(2), a.i64(3), a.i32(4), a.i32(5), a.ptr<const uint64_t*>(6),
                          (int)gz, a.ptr<ci8>(8), a.ptr<cf>(10), a.ptr<const int32_t*>(11), a.ptr<float*>(9));
  K("embed_q8") return ilt_embed_q8(stream, a.ptr<ci8>(0), a.ptr<cu16>(1), a.ptr<const int32_t*>(2), a.ptr<float*>(3), a.i32(4), (int)gx);
  K("embed_k") return ilt_embed_k(stream, a.i32(0), a.ptr<const void*>(1), a.ptr<const int32_t*>(2), a.ptr<float*>(3), a.i32(4), (int)gx);
  K("d4_route") return ilt_d4_route(stream, a.i32(0), a.i32(1), a.i32(2), a.f32(3), a.i32(4), a.ptr<cf>(5), a.ptr<cf>(6),
                                    a.ptr<const int32_t*>(7), a.ptr<cu32>(8), a.ptr<uint32_t*>(9), a.ptr<float*>(10), (int)gx);
  K("d4_group_zero") return ilt_d4_group_zero(stream, a.i32(0), a.ptr<uint32_t*>(1));
  K("d4_group_count") return ilt_d4_group_count(stream, a.i32(0), a.i32(1), a.i32(2), a.ptr<cu32>(3), a.ptr<uint32_t*>(4), a.ptr<uint32_t*>(5));
  K("d4_group_scan") return ilt_d4_group_scan(stream, a.i32(0), a.i32(1), a.i32(2), a.ptr<cu32>(3), a.ptr<uint32_t*>(4));
  K("d4_group_scatter") return ilt_d4_group_scatter(stream, a.i32(0), a.i32(1), a.i32(2), a.ptr<cu32>(3), a.ptr<cu32>(4),
                                                    a.ptr<cu32>(5), a.ptr<cf>(6), a.ptr<uint32_t*>(7), a.ptr<uint32_t*>(8), a.ptr<float*>(9));
  K("d4_gather_rows") return ilt_d4_gather_rows(stream, a.i32(0), a.i32(1), a.ptr<cf>(2), a.ptr<cu32>(3), a.ptr<float*>(4));
  K("d4_swiglu_w") return ilt_d4_swiglu_w(stream, a.i32(0), a.i32(1), a.f32(2), a.ptr<cf>(3), a.ptr<cf>(4), a.ptr<cf>(5),
                                          a.ptr<float*>(6), a.ptr<int8_t*>(7), a.ptr<float*>(8));
  K("d4_moe_sum") return ilt_d4_moe_sum(stream, a.i32(0), a.i32(1), a.ptr<cf>(2), a.ptr<cf>(3), a.ptr<float*>(4), a.ptr<cu32>(5));
  K("d4_moe_sum_rows") return ilt_d4_moe_sum_rows(stream, a.i32(0), a.i32(1), a.i32(2), a.ptr<cf>(3), a.ptr<cu32>(4),
                                                  a.ptr<cf>(5), a.ptr<float*>(6));
#undef K
  return (int)hipErrorNotFound;
}

}  // extern "C"
