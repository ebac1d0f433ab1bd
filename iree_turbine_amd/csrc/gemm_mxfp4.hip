// Block-scaled MXFP4 GEMM for gfx950:  C[M,N] = dq(A) . dq(B)^T, bf16 (or fp32) output.
//
// Codes are two E2M1 values per byte (even k in the low nibble), one E8M0 scale byte per 32
// consecutive k.  The arithmetic is v_mfma_scale_f32_32x32x64_f8f6f4 with both operands in
// fp4 format: the instruction takes the raw codes plus one scale byte per lane and per
// operand and applies 2^(scale-127) in hardware, so nothing is dequantised in software.
//
// Tiling is the fp16 GEMM's with k measured in bytes: a K slab is 256 fp4 values = 128 bytes
// per row = 8 chunks of 16 bytes (one chunk = one 32-element scale block), copied with
// direct-to-LDS loads into a two-stage ring with the same XOR swizzle.  A lane's 16-byte
// fragment is exactly one scale block, so the lane's scale byte is scale[row][slab*8 + 2*ks + h]
// (h = lane / 32); each lane fetches the 8 scale bytes of its row for a slab with one 8-byte
// global load one slab ahead, lanes with h = 1 pre-shift by one byte, and the op_sel field of
// the MFMA picks byte 0 or 2.
#include "common.hpp"

namespace mi355 {

__device__ __forceinline__ void map_tile_mx(int pid, int tiles_m, int tiles_n, int group_m, int& tm, int& tn) {
  const int T = tiles_m * tiles_n;
  const int xcd = pid & 7, loc = pid >> 3;
  const int per = T >> 3, rem = T & 7;
  const int id = xcd * per + (xcd < rem ? xcd : rem) + loc;
  const int width = group_m * tiles_n;
  const int grp = id / width, within = id - grp * width;
  const int first_m = grp * group_m;
  const int gsz = (tiles_m - first_m) < group_m ? (tiles_m - first_m) : group_m;
  tm = first_m + within % gsz;
  tn = within / gsz;
}

template <typename OutT> struct MxOut;
template <> struct MxOut<float> {
  static __device__ __forceinline__ void store4(float* p, float a, float b, float c, float d) {
    floatx4 v = {a, b, c, d};
    *reinterpret_cast<floatx4*>(p) = v;
  }
  static __device__ __forceinline__ void store1(float* p, float a) { *p = a; }
};
template <> struct MxOut<unsigned short> {  // bf16 bits
  static __device__ __forceinline__ void store4(unsigned short* p, float a, float b, float c, float d) {
    ushortx4 v = {f32_to_bf16_rne(a), f32_to_bf16_rne(b), f32_to_bf16_rne(c), f32_to_bf16_rne(d)};
    *reinterpret_cast<ushortx4*>(p) = v;
  }
  static __device__ __forceinline__ void store1(unsigned short* p, float a) { *p = f32_to_bf16_rne(a); }
};

__device__ __forceinline__ floatx16 mfma_fp4_32x32x64(intx4 a, int sa, intx4 b, int sb, floatx16 c, bool odd) {
  intx8 av = {a[0], a[1], a[2], a[3], 0, 0, 0, 0};
  intx8 bv = {b[0], b[1], b[2], b[3], 0, 0, 0, 0};
  if (odd) return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(av, bv, c, 4, 4, 2, sa, 2, sb);
  return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(av, bv, c, 4, 4, 0, sa, 0, sb);
}

template <int BM, int BN, int WM, int WN, typename OutT>
__global__ __launch_bounds__(WM* WN * 64) void gemm_mxfp4_tiled(const uint8_t* __restrict__ A, const uint8_t* __restrict__ As,
                                                                const uint8_t* __restrict__ B, const uint8_t* __restrict__ Bs,
                                                                OutT* __restrict__ C, int M, int N, int K, int tiles_m,
                                                                int tiles_n, int group_m) {
  constexpr int NW = WM * WN;
  constexpr int WTM = BM / WM, WTN = BN / WN;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int A_BYTES = BM * 128, B_BYTES = BN * 128, STAGE = A_BYTES + B_BYTES;
  constexpr int A_GROUPS = BM / 8, B_GROUPS = BN / 8;
  static_assert(A_GROUPS % NW == 0 && B_GROUPS % NW == 0, "loads must split evenly over waves");
  constexpr int LA = A_GROUPS / NW, LB = B_GROUPS / NW;

  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave / WN, wn = wave % WN;
  int tile_m, tile_n;
  map_tile_mx(blockIdx.x, tiles_m, tiles_n, group_m, tile_m, tile_n);

  const int Kb = K >> 1;   // bytes per row of codes
  const int Ksc = K >> 5;  // scale bytes per row
  const int lrow = lane >> 3;
  const int lchunk = (lane & 7) ^ (((wave & 1) << 2) | (lrow >> 1));
  const uint8_t* a_src = A + (size_t)(tile_m * BM + wave * 8 + lrow) * Kb + lchunk * 16;
  const uint8_t* b_src = B + (size_t)(tile_n * BN + wave * 8 + lrow) * Kb + lchunk * 16;
  const size_t row_step = (size_t)NW * 8 * Kb;

  auto issue_loads = [&](int stage) {
    char* dst = lds + stage * STAGE + wave * 1024;
#pragma unroll
    for (int i = 0; i < LA; i++) load_lds_16B(a_src + i * row_step, dst + i * NW * 1024);
#pragma unroll
    for (int i = 0; i < LB; i++) load_lds_16B(b_src + i * row_step, dst + A_BYTES + i * NW * 1024);
    a_src += 128;
    b_src += 128;
  };

  const int r32 = lane & 31, h = lane >> 5;
  const int sw = (h ^ ((r32 >> 1) & 7)) * 16;
  const int a_base = (wm * WTM + r32) * 128 + sw;
  const int b_base = A_BYTES + (wn * WTN + r32) * 128 + sw;

  // scale bytes: 8 per row per slab
  const uint8_t* as_src = As + (size_t)(tile_m * BM + wm * WTM + r32) * Ksc;
  const uint8_t* bs_src = Bs + (size_t)(tile_n * BN + wn * WTN + r32) * Ksc;
  intx2 sa_cur[TM], sb_cur[TN], sa_nxt[TM], sb_nxt[TN];
  auto load_scales = [&](intx2* sa, intx2* sb) {
#pragma unroll
    for (int j = 0; j < TM; j++) sa[j] = *reinterpret_cast<const intx2*>(as_src + (size_t)j * 32 * Ksc);
#pragma unroll
    for (int i = 0; i < TN; i++) sb[i] = *reinterpret_cast<const intx2*>(bs_src + (size_t)i * 32 * Ksc);
    as_src += 8;
    bs_src += 8;
  };

  floatx16 acc[TN][TM];
#pragma unroll
  for (int i = 0; i < TN; i++)
#pragma unroll
    for (int j = 0; j < TM; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

  const int KT = K / 256;
  load_scales(sa_cur, sb_cur);
  issue_loads(0);
  wait_vmcnt0();
  __syncthreads();

  const int shift = 8 * h;
  for (int kt = 0; kt < KT; kt++) {
    if (kt + 1 < KT) {
      issue_loads((kt + 1) & 1);
      load_scales(sa_nxt, sb_nxt);
    }
    const char* st = lds + (kt & 1) * STAGE;
#pragma unroll
    for (int ks = 0; ks < 4; ks++) {
      intx4 fm[TM], fn[TN];
      int sm[TM], sn[TN];
#pragma unroll
      for (int j = 0; j < TM; j++) {
        fm[j] = *reinterpret_cast<const intx4*>(st + ((a_base ^ (ks * 32)) + j * 4096));
        sm[j] = (int)((unsigned)sa_cur[j][ks >> 1] >> shift);
      }
#pragma unroll
      for (int i = 0; i < TN; i++) {
        fn[i] = *reinterpret_cast<const intx4*>(st + ((b_base ^ (ks * 32)) + i * 4096));
        sn[i] = (int)((unsigned)sb_cur[i][ks >> 1] >> shift);
      }
#pragma unroll
      for (int i = 0; i < TN; i++)
#pragma unroll
        for (int j = 0; j < TM; j++) acc[i][j] = mfma_fp4_32x32x64(fn[i], sn[i], fm[j], sm[j], acc[i][j], ks & 1);
    }
    wait_vmcnt0();
    __syncthreads();
#pragma unroll
    for (int j = 0; j < TM; j++) sa_cur[j] = sa_nxt[j];
#pragma unroll
    for (int i = 0; i < TN; i++) sb_cur[i] = sb_nxt[i];
  }

  const int m0 = tile_m * BM + wm * WTM + r32;
  const int n0 = tile_n * BN + wn * WTN + 4 * h;
#pragma unroll
  for (int j = 0; j < TM; j++) {
    OutT* crow = C + (size_t)(m0 + j * 32) * N + n0;
#pragma unroll
    for (int i = 0; i < TN; i++)
#pragma unroll
      for (int q = 0; q < 4; q++)
        MxOut<OutT>::store4(crow + i * 32 + q * 8, acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2],
                            acc[i][j][4 * q + 3]);
  }
}

// Any-shape kernel (K % 32 == 0): 32x32 output tile per wave, 4 waves per workgroup along N,
// operands fetched straight from global memory in fragment layout with bounds checks.
template <typename OutT>
__global__ __launch_bounds__(256) void gemm_mxfp4_generic(const uint8_t* __restrict__ A, const uint8_t* __restrict__ As,
                                                          const uint8_t* __restrict__ B, const uint8_t* __restrict__ Bs,
                                                          OutT* __restrict__ C, int M, int N, int K) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r32 = lane & 31, h = lane >> 5;
  const int m = blockIdx.y * 32 + r32;
  const int n = (blockIdx.x * 4 + wave) * 32 + r32;
  const int Kb = K >> 1, Ksc = K >> 5;
  floatx16 acc;
#pragma unroll
  for (int r = 0; r < 16; r++) acc[r] = 0.f;
  const intx4 zero = {0, 0, 0, 0};
  for (int kb = 0; kb + 1 <= Ksc; kb += 2) {  // two scale blocks (64 elements) per MFMA
    const int blk = kb + h;
    const bool k_ok = blk < Ksc;
    intx4 fa = zero, fb = zero;
    int sa = 127, sb = 127;
    if (m < M && k_ok) {
      fa = *reinterpret_cast<const intx4*>(A + (size_t)m * Kb + blk * 16);
      sa = As[(size_t)m * Ksc + blk];
    }
    if (n < N && k_ok) {
      fb = *reinterpret_cast<const intx4*>(B + (size_t)n * Kb + blk * 16);
      sb = Bs[(size_t)n * Ksc + blk];
    }
    acc = mfma_fp4_32x32x64(fb, sb, fa, sa, acc, false);
  }
  if (m < M) {
    const int nb = (blockIdx.x * 4 + wave) * 32;
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const int nn = nb + 8 * (r >> 2) + 4 * h + (r & 3);
      if (nn < N) MxOut<OutT>::store1(C + (size_t)m * N + nn, acc[r]);
    }
  }
}

// Exact software decode of the format, for checking the device against the closed form.
__global__ __launch_bounds__(256) void mxfp4_dequant_kernel(const uint8_t* __restrict__ codes, const uint8_t* __restrict__ scales,
                                                            float* __restrict__ out, long long rows, int K) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;  // one byte = two elements
  const long long total = rows * (K >> 1);
  if (idx >= total) return;
  const long long row = idx / (K >> 1);
  const int kb = (int)(idx - row * (K >> 1));
  const unsigned byte = codes[idx];
  const unsigned sc = scales[row * (K >> 5) + (kb >> 4)];
  const float scale = sc == 255u ? __builtin_nanf("") : (sc == 0u ? __builtin_bit_cast(float, 0x00400000u) : __builtin_bit_cast(float, sc << 23));
  float v[2];
#pragma unroll
  for (int e = 0; e < 2; e++) {
    const unsigned c = (byte >> (4 * e)) & 15u;
    const unsigned mag = c & 7u;
    // E2M1: 0, 0.5, 1, 1.5, 2, 3, 4, 6
    float f = mag == 0 ? 0.f : mag == 1 ? 0.5f : (float)(2u | (mag & 1u)) * (float)(1u << ((mag >> 1) - 1)) * 0.5f;
    if (c & 8u) f = -f;
    v[e] = f * scale;
  }
  *reinterpret_cast<floatx2*>(out + 2 * idx) = floatx2{v[0], v[1]};
}

struct MxVariant {
  const char* name;
  int bm, bn;
};
static const MxVariant kMxVariants[] = {
    {"tiled_256x256x256_w2x4", 256, 256},
    {"tiled_128x128x256_w2x2", 128, 128},
    {"generic_32x128", 32, 128},
};
constexpr int kNumMxVariants = sizeof(kMxVariants) / sizeof(kMxVariants[0]);
int mxfp4_variant_count() { return kNumMxVariants; }
const char* mxfp4_variant_name(int i) { return (i >= 0 && i < kNumMxVariants) ? kMxVariants[i].name : nullptr; }

template <int BM, int BN, int WM, int WN, typename OutT>
static int launch_mx_tiled(const void* a, const void* as, const void* b, const void* bs, void* c, int M, int N, int K,
                           hipStream_t stream) {
  auto kern = gemm_mxfp4_tiled<BM, BN, WM, WN, OutT>;
  constexpr int lds_bytes = 2 * (BM + BN) * 128;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       lds_bytes);
    if (e != hipSuccess) {
      set_error("hipFuncSetAttribute(gemm_mxfp4_tiled, %d bytes LDS): %s", lds_bytes, hipGetErrorString(e));
      return (int)e;
    }
    attr_set = true;
  }
  const int tiles_m = M / BM, tiles_n = N / BN;
  dim3 grid(tiles_m * tiles_n), block(WM * WN * 64);
  hipLaunchKernelGGL(kern, grid, block, lds_bytes, stream, (const uint8_t*)a, (const uint8_t*)as, (const uint8_t*)b,
                     (const uint8_t*)bs, (OutT*)c, M, N, K, tiles_m, tiles_n, 4);
  return check_launch("gemm_mxfp4_tiled", grid, block, lds_bytes);
}

template <typename OutT>
static int launch_mx(int variant, const void* a, const void* as, const void* b, const void* bs, void* c, int M, int N, int K,
                     hipStream_t stream) {
  switch (variant) {
    case 0: return launch_mx_tiled<256, 256, 2, 4, OutT>(a, as, b, bs, c, M, N, K, stream);
    case 1: return launch_mx_tiled<128, 128, 2, 2, OutT>(a, as, b, bs, c, M, N, K, stream);
    default: {
      dim3 grid((N + 127) / 128, (M + 31) / 32), block(256);
      hipLaunchKernelGGL(gemm_mxfp4_generic<OutT>, grid, block, 0, stream, (const uint8_t*)a, (const uint8_t*)as,
                         (const uint8_t*)b, (const uint8_t*)bs, (OutT*)c, M, N, K);
      return check_launch("gemm_mxfp4_generic", grid, block, 0);
    }
  }
}

}  // namespace mi355

using namespace mi355;

extern "C" int mi355_mxfp4_gemm(const void* a, const void* a_scale, const void* b, const void* b_scale, void* c, int64_t M,
                                int64_t N, int64_t K, int out_dtype, int variant, void* stream) {
  if (!a || !a_scale || !b || !b_scale || !c) return fail(-MI355_E_NULL, "mxfp4_gemm: null pointer");
  if (M <= 0 || N <= 0 || K <= 0 || M > (1 << 30) || N > (1 << 30) || K > (1 << 30))
    return fail(-MI355_E_SHAPE, "mxfp4_gemm: bad shape M=%lld N=%lld K=%lld", (long long)M, (long long)N, (long long)K);
  if (K % 32 != 0) return fail(-MI355_E_SHAPE, "mxfp4_gemm: K=%lld must be a multiple of the 32-element scale block", (long long)K);
  if (out_dtype != MI355_BF16 && out_dtype != MI355_F32)
    return fail(-MI355_E_DTYPE, "mxfp4_gemm: out_dtype %d (want MI355_BF16 or MI355_F32)", out_dtype);
  if (variant >= kNumMxVariants) return fail(-MI355_E_DTYPE, "mxfp4_gemm: variant %d out of range", variant);
  if (!aligned16(a) || !aligned16(b) || !aligned16(c))
    return fail(-MI355_E_ALIGN, "mxfp4_gemm: a, b, c must be 16-byte aligned");
  const bool sc_al = ((reinterpret_cast<uintptr_t>(a_scale) | reinterpret_cast<uintptr_t>(b_scale)) & 7u) == 0;
  auto fits = [&](int v) {
    if (v == kNumMxVariants - 1) return true;
    return sc_al && M % kMxVariants[v].bm == 0 && N % kMxVariants[v].bn == 0 && K % 256 == 0;
  };
  if (variant < 0) {
    if (fits(0) && (M / 256) * (N / 256) >= 128) variant = 0;
    else if (fits(1)) variant = 1;
    else variant = kNumMxVariants - 1;
  } else if (!fits(variant)) {
    return fail(-MI355_E_SHAPE, "mxfp4_gemm: variant %s needs M%%%d==0, N%%%d==0, K%%256==0 and 8-byte aligned scales",
                kMxVariants[variant].name, kMxVariants[variant].bm, kMxVariants[variant].bn);
  }
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (out_dtype == MI355_F32) return launch_mx<float>(variant, a, a_scale, b, b_scale, c, (int)M, (int)N, (int)K, s);
  return launch_mx<unsigned short>(variant, a, a_scale, b, b_scale, c, (int)M, (int)N, (int)K, s);
}

extern "C" int mi355_mxfp4_dequant(const void* codes, const void* scales, float* out, int64_t rows, int64_t K, void* stream) {
  if (!codes || !scales || !out) return fail(-MI355_E_NULL, "mxfp4_dequant: null pointer");
  if (rows <= 0 || K <= 0 || K % 32 != 0 || K > (1 << 30) || rows * (K / 2) > (1ll << 38))
    return fail(-MI355_E_SHAPE, "mxfp4_dequant: bad shape rows=%lld K=%lld (K must be a multiple of 32)", (long long)rows, (long long)K);
  if ((reinterpret_cast<uintptr_t>(out) & 7u) != 0) return fail(-MI355_E_ALIGN, "mxfp4_dequant: out must be 8-byte aligned");
  const long long total = rows * (K / 2);
  dim3 grid((unsigned)((total + 255) / 256)), block(256);
  hipLaunchKernelGGL(mxfp4_dequant_kernel, grid, block, 0, reinterpret_cast<hipStream_t>(stream), (const uint8_t*)codes,
                     (const uint8_t*)scales, out, (long long)rows, (int)K);
  return check_launch("mxfp4_dequant_kernel", grid, block, 0);
}
