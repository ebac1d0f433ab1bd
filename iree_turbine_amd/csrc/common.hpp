// Shared device/host helpers for the gfx950 kernels: vector types, MFMA wrappers,
// LDS address-space casts, direct-to-LDS loads and the error plumbing of the C ABI.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdarg.h>
#include <stdio.h>
#include <atomic>
#include "../../include/turbine_mi355.h"

namespace mi355 {

typedef _Float16 half_t;
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef __attribute__((__vector_size__(4 * sizeof(__fp16)))) __fp16 fp16x4_t;
typedef float floatx2 __attribute__((ext_vector_type(2)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef int intx2 __attribute__((ext_vector_type(2)));
typedef int intx4 __attribute__((ext_vector_type(4)));
typedef int intx8 __attribute__((ext_vector_type(8)));
typedef unsigned short ushortx4 __attribute__((ext_vector_type(4)));

#define MI355_LDS(T, p) ((__attribute__((address_space(3))) T*)(p))
#define MI355_GLOBAL(p) ((const __attribute__((address_space(1))) void*)(p))

// One wave copies 64 x 16 bytes from global memory straight into LDS.  Lane l's
// 16 bytes land at lds_wave_base + 16*l: the LDS side is fixed by the lane id,
// so any swizzle is applied by choosing which global address each lane reads.
__device__ __forceinline__ void load_lds_16B(const void* gptr, void* lds_wave_base) {
  __builtin_amdgcn_global_load_lds(MI355_GLOBAL(gptr), MI355_LDS(void, lds_wave_base), 16, 0, 0);
}

// Same copy through a buffer descriptor: address = descriptor base + voffset (per lane) + soffset
// (wave-uniform), all in bytes, so a load costs no 64-bit vector address arithmetic.  Offsets at or
// beyond the descriptor's size read zeros instead of faulting.
typedef __amdgpu_buffer_rsrc_t buffer_rsrc_t;
__device__ __forceinline__ buffer_rsrc_t make_buffer(const void* base, unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ void buffer_load_lds_16B(buffer_rsrc_t rsrc, unsigned voffset, unsigned soffset, void* lds_wave_base) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, MI355_LDS(void, lds_wave_base), 16, (int)voffset, (int)soffset, 0, 0);
}

// The lane id (0..63) recomputed on the spot, opaque to the compiler: what is derived from it is neither hoisted out
// of a loop nor kept in a register across code that has none to spare.
__device__ __forceinline__ int opaque_lane_id() {
  int l;
  asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(l));
  return l;
}

// Timing-only ablations of the streamed GEMM and prefill kernels, for measuring what a part of a kernel costs: a
// library built with one of these (python -m iree_turbine_amd.build -DMI355_ABLATE_... --out other.so) computes WRONG
// results by construction and says so through mi355_build_flags().  The default build defines none of them.
//   MI355_ABLATE_NO_LOADS       the K loop issues no global -> LDS loads (LDS keeps whatever it held)
//   MI355_ABLATE_L1_LOADS       every load of the K loop reads the same few KiB (always an L1 hit)
//   MI355_ABLATE_NO_LOAD_WAITS  the K loop never waits for a load
//   MI355_ABLATE_PLAIN_LOAD_ORDER  (fp16 GEMM) the lanes of a row fetch its 16-byte chunks in ascending order
//   MI355_ABLATE_NO_BARRIERS    the K loop has no workgroup barriers
//   MI355_ABLATE_NO_SCALE_READS / MI355_ABLATE_NO_SCALE_LOADS   (block-scaled GEMMs) no LDS reads / no loads of scales
//   MI355_ABLATE_NO_A_LOADS     (skinny MXFP4 GEMM) no loads of the activation rows
//   MI355_ABLATE_NO_STORES      the streamed kernels' epilogues stage their results and store nothing
//   MI355_ABLATE_NO_EXP / MI355_ABLATE_NO_K_READS / MI355_ABLATE_NO_V_READS   (prefill) no exponentials / fragment reads
#if defined(MI355_ABLATE_NO_BARRIERS)
#define MI355_KLOOP_BARRIER() do {} while (0)
#else
#define MI355_KLOOP_BARRIER() __builtin_amdgcn_s_barrier()
#endif
#if defined(MI355_ABLATE_NO_LOAD_WAITS)
#define MI355_KLOOP_VMCNT(n) 63
#define MI355_KLOOP_VMCNT_STR(n) "63"
#else
#define MI355_KLOOP_VMCNT(n) (n)
#define MI355_KLOOP_VMCNT_STR(n) #n
#endif

__device__ __forceinline__ void wait_vmcnt0() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// One 16-byte global store per lane as ONE instruction, written out: kernels whose later `s_waitcnt vmcnt(n)` counts
// past the stores of an epilogue (stores and loads share the counter, in issue order) need the number of store
// instructions fixed by the source, not left to how the compiler lowers an assignment.
// The two wait states behind the store are the part's rule for a store of more than 8 bytes followed by a vector
// instruction that overwrites its data registers (the store reads them late); the compiler inserts them for stores it
// emits itself and cannot for one inside an assembly statement.  Without them the next conversion into the same
// registers corrupted one value in sixteen.
template <typename T>
__device__ __forceinline__ void store_global_16B(void* p, const T& v) {
  static_assert(sizeof(T) == 16, "store_global_16B stores exactly 16 bytes per lane");
#if defined(MI355_ABLATE_NO_STORES)
  asm volatile("" ::"v"(p), "v"(v) : "memory");
#else
  asm volatile("global_store_dwordx4 %0, %1, off\n\ts_nop 1" ::"v"(p), "v"(v) : "memory");
#endif
}

// D(32x32) += A(32x16) * B(16x32).  Lane l supplies A[l%32][8*(l/32) .. +7] and
// B[8*(l/32) .. +7][l%32]; it receives D[8*(r/4) + 4*(l/32) + r%4][l%32] in register r.
__device__ __forceinline__ floatx16 mfma_32x32x16(half8 a, half8 b, floatx16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}
// D(16x16) += A(16x32) * B(32x16).  Lane l supplies A[l%16][8*(l/16) .. +7] and
// B[8*(l/16) .. +7][l%16]; it receives D[4*(l/16) + r][l%16] in register r.
__device__ __forceinline__ floatx4 mfma_16x16x32(half8 a, half8 b, floatx4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}

// LDS transpose read.  Within each group of 16 lanes, lane i passes the address
// of 4 consecutive halfs; seen as a 4x16 matrix M[k][n] where lane i supplied
// M[i/4][4*(i%4) .. +3], lane i receives the column M[0..3][i].
__device__ __forceinline__ half4 lds_read_tr16(const void* lds_ptr) {
  fp16x4_t t = __builtin_amdgcn_ds_read_tr16_b64_v4f16(MI355_LDS(fp16x4_t, lds_ptr));
  return *(half4*)&t;
}

// fp32 -> bf16 bits, round to nearest even, NaN stays NaN: the hardware conversion (v_cvt_pk_bf16_f32; two values
// per instruction where the caller converts neighbours) instead of six integer operations per value.
__device__ __forceinline__ unsigned short f32_to_bf16_rne(float f) { return __builtin_bit_cast(unsigned short, (__bf16)f); }

// ---- fp16 / bf16 as a template switch ----------------------------------------------------
// Kernels that serve both 16-bit formats carry the data as opaque 16-bit lanes of half_t vectors and take a
// `bool BF` (false = fp16, true = bf16) for the few places where the format matters: the MFMA instruction, the
// conversions from and to fp32, the packed dot product.
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
template <bool BF>
__device__ __forceinline__ floatx16 mfma16(half8 a, half8 b, floatx16 c) {
  if constexpr (BF)
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
  else
    return mfma_32x32x16(a, b, c);
}
template <bool BF>
__device__ __forceinline__ floatx4 mfma16_16x16x32(half8 a, half8 b, floatx4 c) {
  if constexpr (BF)
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
  else
    return mfma_16x16x32(a, b, c);
}
// fp32 -> the 16-bit format (round to nearest even), returned in a half_t-sized container
template <bool BF>
__device__ __forceinline__ half_t cvt16(float f) {
  if constexpr (BF) return __builtin_bit_cast(half_t, (__bf16)f);
  else return (half_t)f;
}
template <bool BF>
__device__ __forceinline__ float to_f32(half_t v) {
  if constexpr (BF) return __builtin_bit_cast(float, (unsigned)__builtin_bit_cast(unsigned short, v) << 16);
  else return (float)v;
}
// two fp32 values rounded to the 16-bit format and packed; dot2_ones adds the two ROUNDED values to acc in fp32
template <bool BF>
__device__ __forceinline__ half2v cvt16x2(float a, float b) {
  if constexpr (BF) {
    bf16x2_t p = {(__bf16)a, (__bf16)b};
    return __builtin_bit_cast(half2v, p);
  } else {
    return half2v{(half_t)a, (half_t)b};
  }
}
template <bool BF>
__device__ __forceinline__ float dot2_ones(half2v p, float acc) {
  if constexpr (BF) {
    const bf16x2_t ones = {(__bf16)1.f, (__bf16)1.f};
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, p), ones, acc, false);
  } else {
    const half2v ones = {(half_t)1.f, (half_t)1.f};
    return __builtin_amdgcn_fdot2(p, ones, acc, false);
  }
}

// ---- host side ---------------------------------------------------------------------------

void set_error(const char* fmt, ...);
int fail(int code, const char* fmt, ...);
int check_launch(const char* kernel, dim3 grid, dim3 block, size_t lds);

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Raises a kernel's dynamic-LDS limit, once per device.  The attribute belongs to the (kernel, device) pair
// and a process may drive several devices, so `done` -- the call site's own record -- holds one bit per device
// ordinal; ordinals past 63 set the attribute on every launch.
inline int allow_lds(const void* kernel, int bytes, std::atomic<uint64_t>& done, const char* name) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev > 63) dev = -1;
  if (dev >= 0 && ((done.load(std::memory_order_relaxed) >> dev) & 1u)) return 0;
  hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e != hipSuccess) {
    set_error("hipFuncSetAttribute(%s, %d bytes of LDS): %s", name, bytes, hipGetErrorString(e));
    return (int)e;
  }
  if (dev >= 0) done.fetch_or(uint64_t(1) << dev, std::memory_order_relaxed);
  return 0;
}

}  // namespace mi355
