// Rate of 16-byte-per-lane loads (1 KiB per wave-instruction) global -> LDS directly and global -> registers, from a
// footprint per workgroup that stays in the vector L1 (4 KiB), in L2 (64 KiB x 256 workgroups) or in neither (1 MiB x
// 256): cycles per wave-instruction for a lone wave and for four waves (one per SIMD) of a CU.
// Build and run: python -m iree_turbine_amd.build --probes && iree_turbine_amd/csrc/probes/bin/load_rate
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#include "../common.hpp"
using namespace mi355;
#define CK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("err %s line %d\n", hipGetErrorString(e), __LINE__); exit(1);} } while (0)
// MODE 0: direct-to-LDS 16B; 1: to VGPR 16B; 2: direct-to-LDS 4B; FOOT: bytes of footprint per workgroup
template <int MODE>
__global__ __launch_bounds__(256) void probe(const char* src, long long* out, int iters, unsigned foot_mask, unsigned row_stride) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const buffer_rsrc_t rs = make_buffer(src + (size_t)blockIdx.x * (foot_mask + 1u), foot_mask + 1u);
  // lane = (row l >> 3, chunk l & 7): 8 rows of 128 bytes per wave-load, rows row_stride apart
  const unsigned voff = (unsigned)(lane >> 3) * row_stride + (lane & 7) * 16u;
  typedef int i4 __attribute__((ext_vector_type(4)));
  i4 acc = {0, 0, 0, 0};
  __syncthreads();
  long long t0 = clock64();
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int u = 0; u < 16; u++) {
      const unsigned so = ((unsigned)((it * 16 + u) * 4 + wave) * 8u * row_stride) & foot_mask;
      if (MODE == 0) buffer_load_lds_16B(rs, voff, so, lds + (u & 7) * 4096 + wave * 1024);
      else if (MODE == 1) {
        i4 v;
        asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen" : "=v"(v) : "v"(voff), "s"(rs), "s"(so));
        asm volatile("" : "+v"(v));
        acc += v;
      }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  }
  long long t1 = clock64();
  if (lane == 0) out[blockIdx.x * 4 + wave] = t1 - t0 + (acc[0] == 12345 ? 1 : 0);
}
template <int MODE> void run(const char* name, const char* src, unsigned foot, unsigned row_stride, int nw) {
  long long* d; CK(hipMalloc(&d, 256 * 4 * 8));
  CK(hipMemset(d, 0, 256 * 4 * 8));
  const int iters = 500;
  CK(hipFuncSetAttribute((const void*)probe<MODE>, hipFuncAttributeMaxDynamicSharedMemorySize, 65536));
  for (int r = 0; r < 2; r++) probe<MODE><<<256, nw * 64, 65536>>>(src, d, iters, foot - 1, row_stride);
  CK(hipDeviceSynchronize());
  long long h[1024]; CK(hipMemcpy(h, d, sizeof(h), hipMemcpyDeviceToHost));
  double s = 0; for (int i = 0; i < 256; i++) s += h[i * 4];
  printf("%-28s foot %8u stride %5u waves %d  cycles/instr/wave %.2f  per CU %.2f  -> %.1f B/clk/CU\n", name, foot, row_stride, nw,
         s / 256 / (iters * 16.0), s / 256 / (iters * 16.0) / nw, 1024.0 / (s / 256 / (iters * 16.0) / nw));
  CK(hipFree(d));
}
int main() {
  char* src; CK(hipMalloc(&src, 256u << 20)); CK(hipMemset(src, 1, 256u << 20));
  for (int nw = 1; nw <= 4; nw *= 4) {
    run<0>("direct-to-LDS 16B", src, 4096, 128, nw);      // L1 resident
    run<1>("to VGPR 16B", src, 4096, 128, nw);
    run<0>("direct-to-LDS 16B", src, 1 << 20, 128, nw);   // L2 resident (1 MiB per CU: 256 MiB total > L2: MALL)
    run<1>("to VGPR 16B", src, 1 << 20, 128, nw);
    run<0>("direct-to-LDS 16B", src, 65536, 128, nw);     // 64 KiB per CU = 16 MiB total: L2
    run<1>("to VGPR 16B", src, 65536, 128, nw);
    run<0>("direct-to-LDS 16B rows 8K", src, 65536, 8192, nw);
  }
  return 0;
}
