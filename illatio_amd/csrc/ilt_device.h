// Device-side helpers shared by the gfx950 kernels: wave64 lane exchange through
// DPP, exact fp16 widening, packed int8 dot products.
#ifndef ILT_DEVICE_H
#define ILT_DEVICE_H

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#define ILT_WAVE 64

typedef int8_t i8;
typedef uint8_t u8;
typedef uint16_t u16;
typedef uint32_t u32;
typedef uint64_t u64;

// DPP controls (CDNA ISA): quad_perm 0x00-0xff, row_shl:n 0x100+n (lane i reads lane
// i+n of its 16-lane row), row_shr:n 0x110+n, row_half_mirror 0x141 (reverse within 8).
#define ILT_DPP_XOR1 0xB1
#define ILT_DPP_XOR2 0x4E
#define ILT_DPP_HALF_MIRROR 0x141
#define ILT_DPP_ROW_MIRROR 0x140
#define ILT_DPP_SHL(n) (0x100 + (n))

template <int CTRL>
__device__ __forceinline__ int ilt_dpp(int v) {
  return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, true);
}
template <int CTRL>
__device__ __forceinline__ float ilt_dppf(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}

// Integer sums over aligned groups of 2/4/8/16 lanes; every lane of the group ends
// with the total.  Integers: any order gives the same bits.
__device__ __forceinline__ int ilt_sum2(int v) { return v + ilt_dpp<ILT_DPP_XOR1>(v); }
__device__ __forceinline__ int ilt_sum4(int v) { v = ilt_sum2(v); return v + ilt_dpp<ILT_DPP_XOR2>(v); }
__device__ __forceinline__ int ilt_sum8(int v) { v = ilt_sum4(v); return v + ilt_dpp<ILT_DPP_HALF_MIRROR>(v); }
__device__ __forceinline__ int ilt_sum16(int v) { v = ilt_sum8(v); return v + ilt_dpp<ILT_DPP_ROW_MIRROR>(v); }

__device__ __forceinline__ float ilt_max16(float v) {
  v = fmaxf(v, ilt_dppf<ILT_DPP_XOR1>(v));
  v = fmaxf(v, ilt_dppf<ILT_DPP_XOR2>(v));
  v = fmaxf(v, ilt_dppf<ILT_DPP_HALF_MIRROR>(v));
  v = fmaxf(v, ilt_dppf<ILT_DPP_ROW_MIRROR>(v));
  return v;
}

// A wave's maximum and a wave's sum of doubles, the same in every lane: butterflies over a row's 16 lanes through DPP,
// the four rows through readlane -- a tenth of the trips through LDS that __shfl_xor's permutes make.  All 64 lanes
// must be active.  (The order of the adds is not the CPU's: callers check whether that could show.)
template <int CTRL> __device__ __forceinline__ double dpp_double(double v) {
  return __hiloint2double(ilt_dpp<CTRL>(__double2hiint(v)), ilt_dpp<CTRL>(__double2loint(v)));
}
__device__ __forceinline__ double readlane_double(double v, int lane) {
  return __hiloint2double(__builtin_amdgcn_readlane(__double2hiint(v), lane), __builtin_amdgcn_readlane(__double2loint(v), lane));
}
__device__ __forceinline__ double wave_sum_double(double v) {
  v += dpp_double<ILT_DPP_XOR1>(v);
  v += dpp_double<ILT_DPP_XOR2>(v);
  v += dpp_double<ILT_DPP_HALF_MIRROR>(v);
  v += dpp_double<ILT_DPP_ROW_MIRROR>(v);
  return (readlane_double(v, 0) + readlane_double(v, 16)) + (readlane_double(v, 32) + readlane_double(v, 48));
}
__device__ __forceinline__ float wave_max_float(float v) {
  v = ilt_max16(v);
  const int b = __float_as_int(v);
  return fmaxf(fmaxf(__int_as_float(__builtin_amdgcn_readlane(b, 0)), __int_as_float(__builtin_amdgcn_readlane(b, 16))),
               fmaxf(__int_as_float(__builtin_amdgcn_readlane(b, 32)), __int_as_float(__builtin_amdgcn_readlane(b, 48))));
}

// binary16 bits -> binary32, exact (subnormals included).
__device__ __forceinline__ float ilt_h2f(u16 h) { return __half2float(__ushort_as_half(h)); }

// four int8 x int8 products added to c (v_dot4_i32_i8); exact.
__device__ __forceinline__ int ilt_dot4(int a, int b, int c) { return __builtin_amdgcn_sdot4(a, b, c, false); }

__device__ __forceinline__ int ilt_dot16(const int4& a, const int4& b, int c) {
  c = ilt_dot4(a.x, b.x, c); c = ilt_dot4(a.y, b.y, c); c = ilt_dot4(a.z, b.z, c); return ilt_dot4(a.w, b.w, c);
}

// a * b and a * b + c for a and b that fit 24 bits (signed), at the full rate; a 32-bit multiply takes
// four times as long.  The operands' sign extension from bit 23 is written out: it shows the compiler
// that v_mul_i32_i24 / v_mad_i32_i24 will do, and it goes away where the range is known (known within the
// basic block: an operand that comes out of a branch has lost its range, and the multiply is a 32-bit one
// again).  Not inline assembly: the compiler puts the wait states that a dot instruction's result needs
// before its own instructions only.
__device__ __forceinline__ int ilt_s24(int a) { return (a << 8) >> 8; }
__device__ __forceinline__ int ilt_mul24(int a, int b) { return ilt_s24(a) * ilt_s24(b); }
__device__ __forceinline__ int ilt_mad24(int a, int b, int c) { return ilt_s24(a) * ilt_s24(b) + c; }

// Address spaces spelled out.  A pointer rebuilt from an integer (an expert's slot
// address), or carried through a struct, is "generic" to the compiler; generic loads are
// FLAT instructions, which count against the LDS counter as well as the memory counter and
// so cannot stay in flight across an LDS read.  These helpers load through address space 1
// (global) and store through address space 3 (LDS) whatever the pointer's history.
#define ILT_GLOBAL __attribute__((address_space(1)))
#define ILT_LDS __attribute__((address_space(3)))

typedef int ilt_v4i __attribute__((ext_vector_type(4)));
typedef int ilt_v2i __attribute__((ext_vector_type(2)));
typedef float ilt_v2f __attribute__((ext_vector_type(2)));
// (The pointer goes through its low 32 bits -- a generic pointer into LDS holds the LDS address there --
// because a cast from generic to LDS proper first compares the pointer with null: two more
// instructions on 64-bit values per address, in loops that are bound by their instruction count.)
#define ILT_LDS_PTR(T, p) ((ILT_LDS T*)(unsigned long long)(unsigned)(unsigned long long)(p))
__device__ __forceinline__ int4 ilt_lds_ld16(const void* p) {
  const ilt_v4i v = *ILT_LDS_PTR(const ilt_v4i, p); return make_int4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ int2 ilt_lds_ld8(const void* p) {
  const ilt_v2i v = *ILT_LDS_PTR(const ilt_v2i, p); return make_int2(v.x, v.y);
}
__device__ __forceinline__ float ilt_lds_ldf(const void* p) { return *ILT_LDS_PTR(const float, p); }
__device__ __forceinline__ void ilt_lds_stf(void* p, float v) { *ILT_LDS_PTR(float, p) = v; }
__device__ __forceinline__ void ilt_lds_stf2(void* p, float a, float b) { ilt_v2f v = {a, b}; *ILT_LDS_PTR(ilt_v2f, p) = v; }

// Global loads that may be only 2-byte aligned (GGUF blocks of 34, 66, 84 and 210 bytes are
// not 16-byte multiples); gfx950 performs them in hardware.
__device__ __forceinline__ int4 ilt_ld16(const u8* p) {
  int4 v; __builtin_memcpy(&v, __builtin_assume_aligned(p, 2), 16); return v;
}
__device__ __forceinline__ int2 ilt_ld8(const u8* p) {
  int2 v; __builtin_memcpy(&v, __builtin_assume_aligned(p, 2), 8); return v;
}
__device__ __forceinline__ u32 ilt_ld4(const u8* p) {
  u32 v; __builtin_memcpy(&v, __builtin_assume_aligned(p, 2), 4); return v;
}
__device__ __forceinline__ u16 ilt_ld2(const u8* p) {
  u16 v; __builtin_memcpy(&v, __builtin_assume_aligned(p, 2), 2); return v;
}

// Buffer loads: a wave-uniform descriptor (base, byte count) plus a per-lane byte offset.
// They count against the memory counter only, so they stay in flight across LDS traffic,
// and a read past the byte count returns zeros instead of faulting.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t ilt_rsrc(const void* base, u32 bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, bytes, 0x00020000);
}
// A pointer that is the same in every lane, said so to the compiler (a descriptor built from
// a value it cannot prove uniform is applied lane by lane in a loop).
__device__ __forceinline__ const void* ilt_uniform_ptr(const void* p) {
  const u64 a = (u64)p;
  const u32 lo = __builtin_amdgcn_readfirstlane((u32)a), hi = __builtin_amdgcn_readfirstlane((u32)(a >> 32));
  return (const void*)(((u64)hi << 32) | lo);
}
__device__ __forceinline__ int4 ilt_bld16(__amdgpu_buffer_rsrc_t r, u32 off) {
  const ilt_v4i v = __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 0);
  return make_int4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ int2 ilt_bld8(__amdgpu_buffer_rsrc_t r, u32 off) {
  const ilt_v2i v = __builtin_amdgcn_raw_buffer_load_b64(r, off, 0, 0);
  return make_int2(v.x, v.y);
}
__device__ __forceinline__ u32 ilt_bld4(__amdgpu_buffer_rsrc_t r, u32 off) { return __builtin_amdgcn_raw_buffer_load_b32(r, off, 0, 0); }
__device__ __forceinline__ u16 ilt_bld2(__amdgpu_buffer_rsrc_t r, u32 off) { return __builtin_amdgcn_raw_buffer_load_b16(r, off, 0, 0); }
__device__ __forceinline__ u8 ilt_bld1(__amdgpu_buffer_rsrc_t r, u32 off) { return __builtin_amdgcn_raw_buffer_load_b8(r, off, 0, 0); }

// 16 bytes per lane from global memory straight into LDS, no register in between: lane i's
// piece lands at lds_base + 16*i (lds_base the same in every lane).  Counted by vmcnt.
__device__ __forceinline__ void ilt_g2lds16(const void* src, void* lds_base) {
  __builtin_amdgcn_global_load_lds((const ILT_GLOBAL void*)src, (ILT_LDS void*)lds_base, 16, 0, 0);
}

// A 16-byte LDS store the compiler does not see as one.  After a direct global-to-LDS load
// it makes every LDS store wait for vmcnt(0), i.e. for loads sent off to arrive steps later;
// a kernel that keeps such loads in flight stores through this and waits for its stores
// itself (ilt_barrier_lds) before the barrier that publishes them.
__device__ __forceinline__ void ilt_lds_st16_untracked(void* p, int a, int b, int c, int d) {
  const ilt_v4i v = {a, b, c, d};
  asm volatile("ds_write_b128 %0, %1" :: "v"((u32)(uintptr_t)(ILT_LDS void*)p), "v"(v) : "memory");
}
// This wave's LDS traffic done, then the workgroup barrier -- without __syncthreads()'s fence,
// which would also wait for every global load in flight (vmcnt(0)), the direct-to-LDS ones
// included.  The caller waits (s_waitcnt vmcnt(n)) for the loads the barrier must publish.
// A kernel's arguments sit in device memory that nothing has read yet: the first scalar load from each of their
// 64-byte lines is a trip to memory, and code that reads an argument, branches on it and reads the next makes those
// trips one after another (a launch whose arguments were left in host memory took 3.8 us longer).  This asks for
// one dword of each of the first 7 lines (448 bytes: what every wave of the product kernels reads before its first
// loads) at once and waits for them together; the loads that follow find the lines in the scalar cache.  (All 12
// lines of those kernels' arguments: 0.25 % slower; the later ones are read by few waves, late.)  Loads only.
__device__ __forceinline__ void ilt_kernarg_warm7() {
  const auto k = __builtin_amdgcn_kernarg_segment_ptr();
  unsigned t0, t1, t2, t3, t4, t5, t6;
  asm volatile(
      "s_load_dword %0, %7, 0x0\n\ts_load_dword %1, %7, 0x40\n\ts_load_dword %2, %7, 0x80\n\ts_load_dword %3, %7, 0xc0\n\t"
      "s_load_dword %4, %7, 0x100\n\ts_load_dword %5, %7, 0x140\n\ts_load_dword %6, %7, 0x180\n\t"
      "s_waitcnt lgkmcnt(0)"
      : "=&s"(t0), "=&s"(t1), "=&s"(t2), "=&s"(t3), "=&s"(t4), "=&s"(t5), "=&s"(t6)
      : "s"(k)
      : "memory");
}
__device__ __forceinline__ void ilt_barrier_lds() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// SBCL evaluates single-float exp and log by widening to double, calling libm and
// rounding back (the CPU path's silu, softplus); the kernels do the same.
__device__ __forceinline__ float ilt_expf_via_double(float x) { return (float)exp((double)x); }
__device__ __forceinline__ float ilt_logf_via_double(float x) { return (float)log((double)x); }

__device__ __forceinline__ float ilt_sigmoid(float x) {
  if (x >= 0.0f) return 1.0f / (1.0f + ilt_expf_via_double(-x));
  float e = ilt_expf_via_double(x);
  return e / (1.0f + e);
}
__device__ __forceinline__ float ilt_silu(float x) { return x * ilt_sigmoid(x); }

#endif  // ILT_DEVICE_H
