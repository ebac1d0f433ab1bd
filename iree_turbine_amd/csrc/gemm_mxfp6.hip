// Block-scaled MXFP6 GEMM for gfx950:  C[M,N] = dq(A) . dq(B)^T, bf16 (or fp32) output.
//
// Elements are OCP 6-bit floats -- E2M3 (sign, 2 exponent bits with bias 1, 3 mantissa bits; largest value 7.5)
// or E3M2 (3 exponent bits with bias 3, 2 mantissa bits; largest value 28) -- with one E8M0 scale byte per 32
// consecutive k.  A row is a little-endian bit stream: element k occupies bits [6k, 6k + 6) of the row, so a
// scale block of 32 elements is 24 bytes and a row K * 3 / 4 bytes.  That is exactly what
// v_mfma_scale_f32_32x32x64_f8f6f4 takes for a 6-bit operand (measured with one-hot operands): lane (r, h)
// supplies block h of the k-step for row r in its first six registers, slot s at bits [6s, 6s + 6), and its own
// scale byte; the last two registers are ignored.
#include <math.h>
#include <type_traits>

#include "common.hpp"

namespace mi355 {

namespace {

template <typename OutT> struct Out6;
template <> struct Out6<float> {
  static __device__ __forceinline__ void store1(float* p, float a) { *p = a; }
};
template <> struct Out6<unsigned short> {  // bf16 bits
  static __device__ __forceinline__ void store1(unsigned short* p, float a) { *p = f32_to_bf16_rne(a); }
};

// FMT: the instruction's format code, 2 = E2M3, 3 = E3M2
template <int FMT>
__device__ __forceinline__ floatx16 mfma_fp6_32x32x64(intx8 a, int sa, intx8 b, int sb, floatx16 c) {
  return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, FMT, FMT, 0, sa, 0, sb);
}

// one 24-byte block (8-byte aligned) as an MFMA operand
__device__ __forceinline__ intx8 load_block(const uint8_t* p) {
  const intx2 d0 = *reinterpret_cast<const intx2*>(p);
  const intx2 d1 = *reinterpret_cast<const intx2*>(p + 8);
  const intx2 d2 = *reinterpret_cast<const intx2*>(p + 16);
  return intx8{d0[0], d0[1], d1[0], d1[1], d2[0], d2[1], 0, 0};
}

}  // namespace

// Any shape with K % 32 == 0: one wave per 32x32 output tile, operands straight from global memory.
template <typename OutT, int FMT>
__global__ __launch_bounds__(256) void gemm_mxfp6_generic(const uint8_t* __restrict__ A, const uint8_t* __restrict__ As,
                                                          const uint8_t* __restrict__ B, const uint8_t* __restrict__ Bs,
                                                          OutT* __restrict__ C, int M, int N, int K) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r32 = lane & 31, h = lane >> 5;
  const int m = blockIdx.y * 32 + r32;
  const int n = (blockIdx.x * 4 + wave) * 32 + r32;
  const int Ksc = K >> 5;
  const size_t row_bytes = (size_t)Ksc * 24;
  floatx16 acc;
#pragma unroll
  for (int r = 0; r < 16; r++) acc[r] = 0.f;
  const intx8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  for (int kb = 0; kb < Ksc; kb += 2) {  // two scale blocks (64 elements) per MFMA
    const int blk = kb + h;
    const bool k_ok = blk < Ksc;  // a lone last block pairs with zeros
    intx8 fa = zero, fb = zero;
    int sa = 127, sb = 127;
    if (m < M && k_ok) {
      fa = load_block(A + (size_t)m * row_bytes + (size_t)blk * 24);
      sa = As[(size_t)m * Ksc + blk];
    }
    if (n < N && k_ok) {
      fb = load_block(B + (size_t)n * row_bytes + (size_t)blk * 24);
      sb = Bs[(size_t)n * Ksc + blk];
    }
    acc = mfma_fp6_32x32x64<FMT>(fb, sb, fa, sa, acc);
  }
  if (m < M) {
    const int nb = (blockIdx.x * 4 + wave) * 32;
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const int nn = nb + 8 * (r >> 2) + 4 * h + (r & 3);
      if (nn < N) Out6<OutT>::store1(C + (size_t)m * N + nn, acc[r]);
    }
  }
}

static const char* kMx6Variants[] = {"generic_32x128"};
constexpr int kNumMx6Variants = 1;
int mxfp6_variant_count() { return kNumMx6Variants; }
const char* mxfp6_variant_name(int i) { return (i >= 0 && i < kNumMx6Variants) ? kMx6Variants[i] : nullptr; }

template <typename OutT, int FMT>
static int launch_mx6(int variant, const void* a, const void* as, const void* b, const void* bs, void* c, int M, int N, int K,
                      hipStream_t stream) {
  (void)variant;
  dim3 grid((N + 127) / 128, (M + 31) / 32), block(256);
  hipLaunchKernelGGL((gemm_mxfp6_generic<OutT, FMT>), grid, block, 0, stream, (const uint8_t*)a, (const uint8_t*)as,
                     (const uint8_t*)b, (const uint8_t*)bs, (OutT*)c, M, N, K);
  return check_launch("gemm_mxfp6_generic", grid, block, 0);
}

}  // namespace mi355

using namespace mi355;

extern "C" int mi355_mxfp6_gemm(const void* a, const void* a_scale, const void* b, const void* b_scale, void* c, int64_t M,
                                int64_t N, int64_t K, int element_format, int out_dtype, int variant, void* stream) {
  if (!a || !a_scale || !b || !b_scale || !c) return fail(-MI355_E_NULL, "mxfp6_gemm: null pointer");
  if (M <= 0 || N <= 0 || K <= 0 || M > (1 << 30) || N > (1 << 30) || K > (1 << 27))
    return fail(-MI355_E_SHAPE, "mxfp6_gemm: bad shape M=%lld N=%lld K=%lld", (long long)M, (long long)N, (long long)K);
  if (K % 32 != 0) return fail(-MI355_E_SHAPE, "mxfp6_gemm: K=%lld must be a multiple of the 32-element scale block", (long long)K);
  if (element_format != MI355_FP6_E2M3 && element_format != MI355_FP6_E3M2)
    return fail(-MI355_E_DTYPE, "mxfp6_gemm: element_format %d (want MI355_FP6_E2M3 or MI355_FP6_E3M2)", element_format);
  if (out_dtype != MI355_BF16 && out_dtype != MI355_F32)
    return fail(-MI355_E_DTYPE, "mxfp6_gemm: out_dtype %d (want MI355_BF16 or MI355_F32)", out_dtype);
  if (variant >= kNumMx6Variants) return fail(-MI355_E_DTYPE, "mxfp6_gemm: variant %d out of range", variant);
  if (!aligned16(a) || !aligned16(b) || !aligned16(c)) return fail(-MI355_E_ALIGN, "mxfp6_gemm: a, b, c must be 16-byte aligned");
  if (variant < 0) variant = 0;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const bool e2m3 = element_format == MI355_FP6_E2M3;
  if (out_dtype == MI355_F32)
    return e2m3 ? launch_mx6<float, 2>(variant, a, a_scale, b, b_scale, c, (int)M, (int)N, (int)K, s)
                : launch_mx6<float, 3>(variant, a, a_scale, b, b_scale, c, (int)M, (int)N, (int)K, s);
  return e2m3 ? launch_mx6<unsigned short, 2>(variant, a, a_scale, b, b_scale, c, (int)M, (int)N, (int)K, s)
              : launch_mx6<unsigned short, 3>(variant, a, a_scale, b, b_scale, c, (int)M, (int)N, (int)K, s);
}
