// HBM read rate of 128 MiB (8192 rows of 16 KiB, as the weights of a 16 x 8192 x 8192 fp16 product) in three orders, each
// launch on another of six copies so that nothing comes out of the memory-side cache:
//   linear:  workgroup b of W reads its contiguous 128 MiB / W, 8 KiB per step of its 512 threads
//   columns: workgroup b of 256 owns 32 rows and sweeps them together, a 1 KiB window per row and step (wave w takes the
//            128-byte segment w of the window, 8 rows per instruction): the skinny GEMM kernel's order
//   columns, rotated: the same with the sweep started (b >> 3) steps in, i.e. at another place for every workgroup of an XCD
// And the paged decode kernel's gather on its own: two pools of 18432 pages of 32 KiB (16 tokens x 8 kv heads x 256 B; 1.2 GB
// in all), workgroup (list, kv head, split) reads slice `head` (16 rows of 256 B, 2 KiB apart) of each of the 96 pages of its
// list from both pools, pages shuffled, in the kernel's grid order (split fastest) and with the head fastest.
// Build and run: python -m iree_turbine_amd.build --probes && iree_turbine_amd/csrc/probes/bin/hbm_read_patterns
#include <hip/hip_runtime.h>
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>
typedef int intx4 __attribute__((ext_vector_type(4)));
#define CK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("err %s line %d\n", hipGetErrorString(e), __LINE__); exit(1);} } while (0)

template <int U>
__global__ __launch_bounds__(512) void read_linear(const intx4* __restrict__ src, int* __restrict__ out, int iters) {
  const intx4* p = src + (size_t)blockIdx.x * iters * U * 512 + threadIdx.x;
  int s = 0;
  for (int it = 0; it < iters; it++) {
    intx4 v[U];
#pragma unroll
    for (int i = 0; i < U; i++) v[i] = p[(size_t)(it * U + i) * 512];
#pragma unroll
    for (int i = 0; i < U; i++) s += v[i][0] ^ v[i][3];
  }
  if (s == 0x12345) out[blockIdx.x * 512 + threadIdx.x] = s;  // never true for the fill pattern: keeps the loads alive
}

template <int AHEAD, bool ROTATED>
__global__ __launch_bounds__(512) void read_columns(const char* __restrict__ src, int* __restrict__ out) {
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const char* p = src + (size_t)blockIdx.x * 32 * 16384 + (size_t)(lane >> 3) * 16384 + (lane & 7) * 16 + w * 128;
  const int rot = ROTATED ? (int)(blockIdx.x >> 3) : 0;
  int s = 0;
  intx4 v[AHEAD][4];
#pragma unroll
  for (int a = 0; a < AHEAD; a++)
#pragma unroll
    for (int i = 0; i < 4; i++) v[a][i] = *(const intx4*)(p + (size_t)i * 8 * 16384 + ((a + rot) & 15) * 1024);
  for (int j = 0; j < 16; j += AHEAD) {
#pragma unroll
    for (int a = 0; a < AHEAD; a++) {
#pragma unroll
      for (int i = 0; i < 4; i++) s += v[a][i][0] ^ v[a][i][3];
      if (j + a + AHEAD < 16)
#pragma unroll
        for (int i = 0; i < 4; i++) v[a][i] = *(const intx4*)(p + (size_t)i * 8 * 16384 + ((j + a + AHEAD + rot) & 15) * 1024);
    }
  }
  if (s == 0x12345) out[blockIdx.x * 512 + threadIdx.x] = s;
}

// grid: (split, head, list) for ORDER 0, (head, split, list) for ORDER 1; a wave takes pages w, w + 4, ..., two per step
template <int ORDER>
__global__ __launch_bounds__(256) void read_pages(const char* __restrict__ kp, const char* __restrict__ vp, const int* __restrict__ table, int pages,
                                                  int* out) {
  const int split = ORDER == 0 ? blockIdx.x : blockIdx.y, head = ORDER == 0 ? blockIdx.y : blockIdx.x, list = blockIdx.z;
  const int nsplit = ORDER == 0 ? gridDim.x : gridDim.y;
  const int* t = table + ((size_t)list * nsplit + split) * pages;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const size_t lo = (size_t)(lane >> 4) * 2048 + (lane & 15) * 16 + head * 256;  // 4 rows of 256 bytes per instruction
  int s = 0;
  for (int p = w; p < pages; p += 8) {
    intx4 v[16];
    const size_t b0 = (size_t)t[p] * 32768, b1 = (size_t)t[p + 4 < pages ? p + 4 : p] * 32768;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      v[i] = *(const intx4*)(kp + b0 + lo + i * 8192);
      v[4 + i] = *(const intx4*)(vp + b0 + lo + i * 8192);
      v[8 + i] = *(const intx4*)(kp + b1 + lo + i * 8192);
      v[12 + i] = *(const intx4*)(vp + b1 + lo + i * 8192);
    }
#pragma unroll
    for (int i = 0; i < 16; i++) s += v[i][0] ^ v[i][3];
  }
  if (s == 0x12345) out[threadIdx.x] = s;
}

static const size_t kBytes = (size_t)128 << 20;
static const int kSets = 6;

template <typename Launch>
static void timed(const char* what, Launch launch) {
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0));
  CK(hipEventCreate(&e1));
  for (int rep = 0; rep < 20; rep++) launch(rep % kSets);
  CK(hipEventRecord(e0, 0));
  for (int rep = 0; rep < 200; rep++) launch(rep % kSets);
  CK(hipEventRecord(e1, 0));
  CK(hipEventSynchronize(e1));
  float ms;
  CK(hipEventElapsedTime(&ms, e0, e1));
  printf("%-72s %6.2f us per launch  %5.2f TB/s\n", what, ms * 1000 / 200, kBytes / (ms / 200 * 1e-3) / 1e12);
  fflush(stdout);
}

int main() {
  char* src;
  int* out;
  CK(hipMalloc(&src, kBytes * kSets));
  CK(hipMalloc(&out, 4096 * 512 * 4));
  CK(hipMemset(src, 1, kBytes * kSets));
  auto set = [&](int s) { return src + (size_t)s * kBytes; };
  timed("linear, 256 workgroups, 8 loads of 16 bytes per thread in flight", [&](int s) {
    hipLaunchKernelGGL(read_linear<8>, dim3(256), dim3(512), 0, 0, (const intx4*)set(s), out, (int)(kBytes / 16 / 512 / 8 / 256));
  });
  timed("linear, 1024 workgroups, 8 in flight", [&](int s) {
    hipLaunchKernelGGL(read_linear<8>, dim3(1024), dim3(512), 0, 0, (const intx4*)set(s), out, (int)(kBytes / 16 / 512 / 8 / 1024));
  });
  timed("linear, 4096 workgroups, 4 in flight", [&](int s) {
    hipLaunchKernelGGL(read_linear<4>, dim3(4096), dim3(512), 0, 0, (const intx4*)set(s), out, (int)(kBytes / 16 / 512 / 4 / 4096));
  });
  timed("columns (32 rows x 1 KiB window), 1 step ahead", [&](int s) {
    hipLaunchKernelGGL((read_columns<1, false>), dim3(256), dim3(512), 0, 0, set(s), out);
  });
  timed("columns, 2 steps ahead", [&](int s) { hipLaunchKernelGGL((read_columns<2, false>), dim3(256), dim3(512), 0, 0, set(s), out); });
  timed("columns, 4 steps ahead", [&](int s) { hipLaunchKernelGGL((read_columns<4, false>), dim3(256), dim3(512), 0, 0, set(s), out); });
  timed("columns, 2 steps ahead, sweep start rotated by the workgroup's index in its XCD", [&](int s) {
    hipLaunchKernelGGL((read_columns<2, true>), dim3(256), dim3(512), 0, 0, set(s), out);
  });
  timed("columns, 4 steps ahead, rotated", [&](int s) { hipLaunchKernelGGL((read_columns<4, true>), dim3(256), dim3(512), 0, 0, set(s), out); });
  CK(hipFree(src));

  const int lists = 64, nsplit = 3, pages = 96, P = lists * nsplit * pages;
  char *kp, *vp;
  int* table;
  CK(hipMalloc(&kp, (size_t)P * 32768));
  CK(hipMalloc(&vp, (size_t)P * 32768));
  CK(hipMalloc(&table, P * 4));
  CK(hipMemset(kp, 1, (size_t)P * 32768));
  CK(hipMemset(vp, 1, (size_t)P * 32768));
  std::vector<int> perm(P);
  for (int i = 0; i < P; i++) perm[i] = i;
  std::mt19937 gen(1);
  std::shuffle(perm.begin(), perm.end(), gen);
  CK(hipMemcpy(table, perm.data(), P * 4, hipMemcpyHostToDevice));
  for (int order = 0; order < 2; order++) {
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    auto launch = [&]() {
      if (order == 0) hipLaunchKernelGGL(read_pages<0>, dim3(nsplit, 8, lists), dim3(256), 0, 0, kp, vp, table, pages, out);
      else hipLaunchKernelGGL(read_pages<1>, dim3(8, nsplit, lists), dim3(256), 0, 0, kp, vp, table, pages, out);
    };
    for (int r = 0; r < 5; r++) launch();
    CK(hipEventRecord(e0, 0));
    for (int r = 0; r < 20; r++) launch();
    CK(hipEventRecord(e1, 0));
    CK(hipEventSynchronize(e1));
    float ms;
    CK(hipEventElapsedTime(&ms, e0, e1));
    const double bytes = 2.0 * P * 32768;
    printf("%-72s %6.1f us per launch  %5.2f TB/s\n", order ? "decode's page gather (1.2 GB, shuffled pages), kv head fastest in the grid" : "decode's page gather (1.2 GB, shuffled pages), split fastest (the kernel's grid)",
           ms * 1000 / 20, bytes / (ms / 20 * 1e-3) / 1e12);
    fflush(stdout);
  }
  CK(hipFree(out));
  return 0;
}
