// What one load or LDS read per 8 MFMAs (one "step" of the streamed GEMM kernels) adds to a stream of independent
// v_mfma_f32_16x16x32_f16, one wave per SIMD, loads from an L1-resident region: alone, with a workgroup barrier every
// 32 MFMAs (the kernels' interval), and with the load's place in the step differing by wave (four copies of the loop).
// Build and run: python -m iree_turbine_amd.build --probes && iree_turbine_amd/csrc/probes/bin/mfma_load_bubble
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#include "../common.hpp"
using namespace mi355;
#define CK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("err %s line %d\n", hipGetErrorString(e), __LINE__); exit(1);} } while (0)
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
// MODE 0: MFMAs only; 1: one 16B direct-to-LDS load per 8 MFMAs; 2: one ds_read_b128 per 8 MFMAs; 3: load + 3 ds_reads;
// 4: two loads back to back per 16 MFMAs; 5: load to VGPR; 6: one 4B direct-to-LDS load per 8 MFMAs; 7: load with half the lanes
template <int MODE, int BAR, int LDP>
__device__ __forceinline__ void body(const char* src, long long* out, int iters) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const buffer_rsrc_t rs = make_buffer(src + (size_t)blockIdx.x * 65536, 65536);
  const unsigned voff = (unsigned)(lane >> 3) * 128u + (lane & 7) * 16u;
  const unsigned la = (unsigned)(uintptr_t)MI355_LDS(char, lds) + lane * 16 + 32768;
  floatx4 acc[8];
  half8 a = {1, 2, 3, 4, 5, 6, 7, 8}, b = {1, 1, 1, 1, 1, 1, 1, 1};
  for (int i = 0; i < 8; i++) acc[i] = floatx4{0, 0, 0, 0};
  asm volatile("" : "+v"(a), "+v"(b));
  half8 r0, r1, r2;
  typedef int i4 __attribute__((ext_vector_type(4)));
  i4 g;
  __syncthreads();
  long long t0 = clock64();
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int u = 0; u < 8; u++) {
      const unsigned so = ((unsigned)((it * 8 + u) * 4 + wave) * 1024u) & 65535u;
#pragma unroll
      for (int m = 0; m < 8; m++) {
        asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc[m]) : "v"(a), "v"(b));
        if (m == 0 && (MODE == 2 || MODE == 3)) asm volatile("ds_read_b128 %0, %1" : "=v"(r0) : "v"(la));
        if (m == 1 && MODE == 3) asm volatile("ds_read_b128 %0, %1 offset:1024" : "=v"(r1) : "v"(la));
        if (m == 3 && MODE == 3) asm volatile("ds_read_b128 %0, %1 offset:2048" : "=v"(r2) : "v"(la));
        if (m == LDP) {
          if (MODE == 1 || MODE == 3) buffer_load_lds_16B(rs, voff, so, lds + (u & 7) * 4096 + wave * 1024);
          if (MODE == 4 && (u & 1)) { buffer_load_lds_16B(rs, voff, so, lds + (u & 7) * 4096 + wave * 1024); buffer_load_lds_16B(rs, voff, so ^ 512u, lds + ((u - 1) & 7) * 4096 + wave * 1024); }
          if (MODE == 5) asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen" : "=v"(g) : "v"(voff), "s"(rs), "s"(so));
          if (MODE == 6) __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, MI355_LDS(void, lds + (u & 7) * 4096 + wave * 1024), 4, (int)voff, (int)so, 0, 0);
          if (MODE == 7) { if (lane < 32) buffer_load_lds_16B(rs, voff, so, lds + (u & 7) * 4096 + wave * 1024); }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      if (BAR && (u & 3) == 3) { asm volatile("s_waitcnt vmcnt(16) lgkmcnt(0)" ::: "memory"); __builtin_amdgcn_s_barrier(); __builtin_amdgcn_sched_barrier(0); }
    }
    if (MODE == 2 || MODE == 3) asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(r0), "+v"(r1), "+v"(r2));
    if (MODE == 5) asm volatile("s_waitcnt vmcnt(0)" : "+v"(g));
    asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
  }
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
  long long t1 = clock64();
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
  float s = 0;
  for (int i = 0; i < 8; i++) s += acc[i][0];
  if (lane == 0) out[blockIdx.x * 4 + wave] = t1 - t0 + (s == 12345.f ? 1 : 0);
}
template <int MODE, int BAR, int STAG>
__global__ __launch_bounds__(256) void probe(const char* src, long long* out, int iters) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  if (STAG) {
    if (wave == 0) body<MODE, BAR, 1>(src, out, iters);
    else if (wave == 1) body<MODE, BAR, 3>(src, out, iters);
    else if (wave == 2) body<MODE, BAR, 5>(src, out, iters);
    else body<MODE, BAR, 7>(src, out, iters);
  } else body<MODE, BAR, 5>(src, out, iters);
}
template <int MODE, int BAR = 0, int STAG = 0> void run(const char* name, const char* src) {
  long long* d; CK(hipMalloc(&d, 256 * 4 * 8));
  const int iters = 300;
  CK(hipFuncSetAttribute((const void*)probe<MODE, BAR, STAG>, hipFuncAttributeMaxDynamicSharedMemorySize, 65536));
  for (int r = 0; r < 2; r++) probe<MODE, BAR, STAG><<<256, 256, 65536>>>(src, d, iters);
  CK(hipDeviceSynchronize());
  long long h[1024]; CK(hipMemcpy(h, d, sizeof(h), hipMemcpyDeviceToHost));
  double s = 0; for (int i = 0; i < 1024; i++) s += h[i];
  printf("%-48s cycles per 8 MFMAs %.1f\n", name, s / 1024 / (iters * 8.0));
  CK(hipFree(d));
}
int main() {
  char* src; CK(hipMalloc(&src, 64u << 20)); CK(hipMemset(src, 1, 64u << 20));
  run<0, 1>("MFMAs only, barrier every 32", src);
  run<1, 1>("+ load, barrier every 32", src);
  run<3, 1>("+ load + 3 ds_reads, barrier every 32", src);
  run<1, 1, 1>("+ load, barrier every 32, staggered by wave", src);
  run<3, 1, 1>("+ load + 3 ds_reads, barrier, staggered", src);
  run<1, 0, 1>("+ load, no barrier, staggered (code copies)", src);
  run<0>("MFMAs only", src);
  run<1>("+ one 16B direct-to-LDS load", src);
  run<2>("+ one ds_read_b128", src);
  run<3>("+ load + 3 ds_read_b128", src);
  run<4>("+ two loads back to back every 16 MFMAs", src);
  run<5>("+ one 16B load to VGPRs", src);
  run<6>("+ one 4B direct-to-LDS load", src);
  run<7>("+ one 16B direct-to-LDS load, 32 lanes", src);
  return 0;
}
