// LDS read patterns: cycles per wave-instruction, one workgroup of 1 or 4 waves (one per SIMD) per CU, 16 reads in
// flight per wave.  Answers what a narrow read costs beside a 16-byte one and where bank conflicts begin: lanes are
// (row r = lane & 15, group c = lane >> 4) as in the GEMM kernels' fragment and scale reads; a row stride of 16 bytes
// spreads 16 rows over the 64 banks once (no conflict), 32 bytes folds them twice (a true two-way conflict).
// Build and run: python -m iree_turbine_amd.build --probes && iree_turbine_amd/csrc/probes/bin/lds_read_patterns
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#define CK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("err %s line %d\n", hipGetErrorString(e), __LINE__); exit(1);} } while (0)
template <int PAT>
__global__ __launch_bounds__(256) void probe(long long* out, int iters) {
  __shared__ __attribute__((aligned(1024))) char lds[65536];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int i = threadIdx.x; i < 16384; i += 256) ((int*)lds)[i] = i;
  __syncthreads();
  const int r16 = lane & 15, cq = lane >> 4;
  unsigned base = (unsigned)(uintptr_t)(__attribute__((address_space(3))) char*)lds + wave * 4096;
  unsigned addr;
  if (PAT == 0) addr = base + r16 * 16 + cq;
  else if (PAT == 1) addr = base + r16 * 16;
  else if (PAT == 2) addr = base + r16 * 16;
  else if (PAT == 3) addr = base + r16 * 16;
  else if (PAT == 4) addr = base + r16 * 16;
  else if (PAT == 5) addr = base + lane * 4;
  else if (PAT == 6) addr = base + r16 * 16 + 2 * cq;
  else if (PAT == 7) addr = base + lane * 4;
  else if (PAT == 8) addr = base + lane * 16;       // b128 distinct
  else if (PAT == 9) addr = base + r16 * 4 + cq;    // u8, 16 consecutive dwords, 4 bytes each
  else if (PAT == 10) addr = base + r16 * 8 + cq;   // u8, stride 8
  else if (PAT == 11) addr = base + r16 * 32 + cq;  // u8, stride 32
  else addr = base;
  int v[16];
  long long t0 = clock64();
  for (int it = 0; it < iters; it++) {
#define RD(i)                                                                                        \
    if (PAT == 0 || PAT == 1 || PAT == 5 || PAT == 9 || PAT == 10 || PAT == 11) asm volatile("ds_read_u8 %0, %1 offset:%2" : "=v"(v[i]) : "v"(addr), "n"(i * 256)); \
    else if (PAT == 6) asm volatile("ds_read_u16 %0, %1 offset:%2" : "=v"(v[i]) : "v"(addr), "n"(i * 256));        \
    else if (PAT == 2 || PAT == 7) asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(v[i]) : "v"(addr), "n"(i * 256));
    if constexpr (PAT == 3) {
      long long w[16];
#pragma unroll
      for (int i = 0; i < 16; i++) asm volatile("ds_read_b64 %0, %1 offset:%2" : "=v"(w[i]) : "v"(addr), "n"(i * 256));
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
      for (int i = 0; i < 16; i++) asm volatile("" ::"v"(w[i]));
    } else if constexpr (PAT == 4 || PAT == 8) {
      typedef int i4 __attribute__((ext_vector_type(4)));
      i4 w[16];
#pragma unroll
      for (int i = 0; i < 16; i++) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(w[i]) : "v"(addr), "n"(i * 1024 * (PAT == 8 ? 1 : 0) + (PAT == 4 ? i * 256 : 0)));
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
      for (int i = 0; i < 16; i++) asm volatile("" ::"v"(w[i]));
    } else {
      RD(0) RD(1) RD(2) RD(3) RD(4) RD(5) RD(6) RD(7) RD(8) RD(9) RD(10) RD(11) RD(12) RD(13) RD(14) RD(15)
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
      for (int i = 0; i < 16; i++) asm volatile("" ::"v"(v[i]));
    }
  }
  long long t1 = clock64();
  if (lane == 0) out[blockIdx.x * 4 + wave] = t1 - t0;
}
template <int PAT> void run(const char* name, int nw) {
  long long* d; CK(hipMalloc(&d, 256 * 4 * 8));
  const int iters = 2000;
  probe<PAT><<<256, nw * 64>>>(d, iters);
  probe<PAT><<<256, nw * 64>>>(d, iters);
  CK(hipDeviceSynchronize());
  long long h[1024]; CK(hipMemcpy(h, d, sizeof(h), hipMemcpyDeviceToHost));
  double s = 0; for (int i = 0; i < 256; i++) s += h[i * 4];
  // clock64 = s_memtime at 100 MHz constant? report raw ticks per instruction per wave
  printf("%-40s waves %d ticks/instr/wave %.4f  ticks/instr per CU %.4f\n", name, nw, s / 256 / (iters * 16.0), s / 256 / (iters * 16.0) / nw);
  CK(hipFree(d));
}
int main() {
  for (int nw = 1; nw <= 4; nw *= 4) {
    run<0>("u8 row*16+cq (current)", nw);
    run<1>("u8 row*16 (same byte)", nw);
    run<2>("b32 row*16 broadcast", nw);
    run<3>("b64 row*16 broadcast", nw);
    run<4>("b128 row*16 broadcast", nw);
    run<5>("u8 lane*4 distinct banks", nw);
    run<6>("u16 row*16+2cq", nw);
    run<7>("b32 lane*4 distinct", nw);
    run<8>("b128 lane*16 distinct", nw);
    run<9>("u8 row*4+cq", nw);
    run<10>("u8 row*8+cq", nw);
    run<11>("u8 row*32+cq", nw);
  }
  return 0;
}
