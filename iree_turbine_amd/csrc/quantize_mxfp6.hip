// MXFP6 quantisation for gfx950: x[rows, K] (fp16 / bf16 / fp32) -> 6-bit codes (E2M3 or E3M2) packed as a
// little-endian bit stream, 24 bytes per block of 32, + one E8M0 scale byte per block: the producer of
// mi355_mxfp6_gemm's operands.  OCP Microscaling Formats v1.0 conversion: shared exponent =
// floor(log2(max |x|)) - emax (2 for E2M3, 4 for E3M2) clamped to [-127, 127] (all-zero block: -127; a block
// with a NaN or infinity: the NaN scale 0xFF and signed-zero codes), every element scaled by 2^-shared exactly
// and rounded to the nearest value with ties to the even code, magnitudes beyond the largest value saturating.
//
// A lane owns one block: 32 consecutive elements in, v_cvt_scalef32_pk32_{fp6,bf6}_* turns them into the six
// dwords the GEMM reads (slot s at bits [6s, 6s + 6) -- the instruction's own packing), three 8-byte stores and
// one scale byte out.  Waves that hold a non-finite value or a block whose exponent is clamped at the bottom of
// the E8M0 range (the scale is no longer a normal float) take a software rounding path instead.
#include "common.hpp"

namespace mi355 {

namespace {

typedef _Float16 halfx32 __attribute__((ext_vector_type(32)));
typedef __bf16 bf16x32 __attribute__((ext_vector_type(32)));
typedef float floatx16q __attribute__((ext_vector_type(16)));
typedef unsigned uintx6 __attribute__((ext_vector_type(6)));

// E2M3: FMT 0, 2 exponent bits, 3 mantissa bits, bias 1, emax 2.  E3M2: FMT 1, 3 / 2 / 3, emax 4.
template <int FMT> struct F6 {
  static constexpr int MB = FMT == 0 ? 3 : 2;
  static constexpr int BIAS = FMT == 0 ? 1 : 3;
  static constexpr int EMAX = FMT == 0 ? 2 : 4;
};

// software rounding of one magnitude y >= 0 (already scaled) to the 5-bit magnitude code
template <int FMT>
__device__ __forceinline__ unsigned round6_sw(float y) {
  constexpr int MB = F6<FMT>::MB, BIAS = F6<FMT>::BIAS;
  const float min_normal = __builtin_amdgcn_ldexpf(1.0f, 1 - BIAS);
  unsigned code;
  if (y < min_normal) {
    // subnormal codes count steps of 2^(1 - BIAS - MB); a tie goes to the even count, and the count 2^MB is the
    // code of the smallest normal value
    code = (unsigned)__builtin_rintf(__builtin_amdgcn_ldexpf(y, MB + BIAS - 1));
  } else {
    unsigned b = __builtin_bit_cast(unsigned, y);
    b += ((1u << (22 - MB)) - 1u) + ((b >> (23 - MB)) & 1u);  // round the mantissa to MB bits, ties to even
    const int e = (int)(b >> 23) - 127;
    code = ((unsigned)(e + BIAS) << MB) | ((b >> (23 - MB)) & ((1u << MB) - 1u));
  }
  return code > 31u ? 31u : code;
}

template <typename T> struct Q6In;
template <bool BF16> struct Q6In16 {
  intx4 w[4];  // 32 elements
  __device__ __forceinline__ void load(const void* p) {
#pragma unroll
    for (int i = 0; i < 4; i++) w[i] = reinterpret_cast<const intx4*>(p)[i];
  }
  __device__ __forceinline__ void zero() {
#pragma unroll
    for (int i = 0; i < 4; i++) w[i] = intx4{0, 0, 0, 0};
  }
  static constexpr unsigned kInf = BF16 ? 0x7f80u : 0x7c00u;
  // |x| bit patterns order like unsigned integers (NaN > inf > finite): the block maximum is a packed maximum
  __device__ __forceinline__ unsigned amax_bits() const {
    typedef unsigned short ushortx2 __attribute__((ext_vector_type(2)));
    ushortx2 m = {0, 0};
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const unsigned u = (unsigned)w[i][j] & 0x7fff7fffu;
        m = __builtin_elementwise_max(m, __builtin_bit_cast(ushortx2, u));
      }
    return m[0] > m[1] ? m[0] : m[1];
  }
  static __device__ __forceinline__ float bits_to_float(unsigned b) {
    if (BF16) return __builtin_bit_cast(float, b << 16);
    return (float)__builtin_bit_cast(half_t, (unsigned short)b);
  }
  __device__ __forceinline__ float element(int i) const {  // i is a compile-time constant after unrolling
    const unsigned u = (unsigned)w[i >> 3][(i >> 1) & 3];
    const unsigned short s = (i & 1) ? (unsigned short)(u >> 16) : (unsigned short)(u & 0xffffu);
    return bits_to_float(s);
  }
  template <int FMT> __device__ __forceinline__ uintx6 convert(float scale) const {
    if constexpr (BF16) {
      bf16x32 v;
      __builtin_memcpy(&v, w, 64);
      if constexpr (FMT == 0) return __builtin_amdgcn_cvt_scalef32_pk32_fp6_bf16(v, scale);
      else return __builtin_amdgcn_cvt_scalef32_pk32_bf6_bf16(v, scale);
    } else {
      halfx32 v;
      __builtin_memcpy(&v, w, 64);
      if constexpr (FMT == 0) return __builtin_amdgcn_cvt_scalef32_pk32_fp6_f16(v, scale);
      else return __builtin_amdgcn_cvt_scalef32_pk32_bf6_f16(v, scale);
    }
  }
};
template <> struct Q6In<half_t> : Q6In16<false> {};
template <> struct Q6In<unsigned short> : Q6In16<true> {};
template <> struct Q6In<float> {
  floatx4 f[8];
  static constexpr unsigned kInf = 0x7f800000u;
  __device__ __forceinline__ void load(const void* p) {
#pragma unroll
    for (int i = 0; i < 8; i++) f[i] = reinterpret_cast<const floatx4*>(p)[i];
  }
  __device__ __forceinline__ void zero() {
#pragma unroll
    for (int i = 0; i < 8; i++) f[i] = floatx4{0.f, 0.f, 0.f, 0.f};
  }
  __device__ __forceinline__ unsigned amax_bits() const {
    unsigned m = 0;
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const float fj = f[i][j];
        const unsigned b = __builtin_bit_cast(unsigned, fj) & 0x7fffffffu;
        m = b > m ? b : m;
      }
    return m;
  }
  static __device__ __forceinline__ float bits_to_float(unsigned b) { return __builtin_bit_cast(float, b); }
  __device__ __forceinline__ float element(int i) const { return f[i >> 2][i & 3]; }
  template <int FMT> __device__ __forceinline__ uintx6 convert(float scale) const {
    // the instruction interleaves its two sources: slot 2i from the first, slot 2i + 1 from the second
    floatx16q lo, hi;
#pragma unroll
    for (int i = 0; i < 16; i++) {
      lo[i] = element(2 * i);
      hi[i] = element(2 * i + 1);
    }
    if constexpr (FMT == 0) return __builtin_amdgcn_cvt_scalef32_2xpk16_fp6_f32(lo, hi, scale);
    else return __builtin_amdgcn_cvt_scalef32_2xpk16_bf6_f32(lo, hi, scale);
  }
};

}  // namespace

template <typename T, int FMT>
__global__ __launch_bounds__(256) void mxfp6_quantize_kernel(const T* __restrict__ x, uint8_t* __restrict__ codes,
                                                             uint8_t* __restrict__ scales, long long n_blocks) {
  const long long blk = (long long)blockIdx.x * 256 + threadIdx.x;
  const bool live = blk < n_blocks;
  Q6In<T> in;
  if (live) in.load(x + blk * 32);
  else in.zero();
  const unsigned mb = in.amax_bits();
  const bool poisoned = mb >= Q6In<T>::kInf;
  const float amax = Q6In<T>::bits_to_float(mb);
  // floor(log2(amax)) = frexp exponent - 1 (also right for subnormal inputs)
  int shared = mb == 0 ? -127 : __builtin_amdgcn_frexp_expf(amax) - 1 - F6<FMT>::EMAX;
  shared = shared < -127 ? -127 : (shared > 127 ? 127 : shared);
  uintx6 out;
  if (__builtin_amdgcn_ballot_w64(live && (poisoned || shared < -126)) != 0) {
    unsigned long long acc = 0;  // bit stream, flushed a dword at a time
    int have = 0, word = 0;
#pragma unroll
    for (int i = 0; i < 32; i++) {
      const float xi = in.element(i);
      const float y = poisoned ? 0.f : __builtin_fabsf(__builtin_amdgcn_ldexpf(xi, -shared));
      const unsigned c = round6_sw<FMT>(y) | ((__builtin_bit_cast(unsigned, xi) >> 31) << 5);
      acc |= (unsigned long long)c << have;
      have += 6;
      if (have >= 32) {
        out[word++] = (unsigned)acc;
        acc >>= 32;
        have -= 32;
      }
    }
  } else {
    out = in.template convert<FMT>(__builtin_amdgcn_ldexpf(1.0f, shared));
  }
  if (live) {
    unsigned long long* dst = reinterpret_cast<unsigned long long*>(codes + blk * 24);
    dst[0] = (unsigned long long)out[0] | ((unsigned long long)out[1] << 32);
    dst[1] = (unsigned long long)out[2] | ((unsigned long long)out[3] << 32);
    dst[2] = (unsigned long long)out[4] | ((unsigned long long)out[5] << 32);
    scales[blk] = (uint8_t)(poisoned ? 255 : shared + 127);
  }
}

}  // namespace mi355

using namespace mi355;

template <int FMT>
static int launch_q6(const void* x, int in_dtype, long long n_blocks, void* codes, void* scales, hipStream_t s) {
  dim3 grid((unsigned)((n_blocks + 255) / 256)), block(256);
  if (in_dtype == MI355_F16)
    hipLaunchKernelGGL((mxfp6_quantize_kernel<half_t, FMT>), grid, block, 0, s, (const half_t*)x, (uint8_t*)codes, (uint8_t*)scales, n_blocks);
  else if (in_dtype == MI355_BF16)
    hipLaunchKernelGGL((mxfp6_quantize_kernel<unsigned short, FMT>), grid, block, 0, s, (const unsigned short*)x, (uint8_t*)codes,
                       (uint8_t*)scales, n_blocks);
  else
    hipLaunchKernelGGL((mxfp6_quantize_kernel<float, FMT>), grid, block, 0, s, (const float*)x, (uint8_t*)codes, (uint8_t*)scales, n_blocks);
  return check_launch("mxfp6_quantize_kernel", grid, block, 0);
}

extern "C" int mi355_mxfp6_quantize(const void* x, int in_dtype, int64_t rows, int64_t K, int element_format, void* codes,
                                    void* scales, void* stream) {
  if (!x || !codes || !scales) return fail(-MI355_E_NULL, "mxfp6_quantize: null pointer");
  if (rows <= 0 || K <= 0 || K % 32 != 0 || rows > (1ll << 40) / K)
    return fail(-MI355_E_SHAPE, "mxfp6_quantize: bad shape rows=%lld K=%lld (K must be a multiple of 32)", (long long)rows,
                (long long)K);
  if (in_dtype != MI355_F32 && in_dtype != MI355_F16 && in_dtype != MI355_BF16)
    return fail(-MI355_E_DTYPE, "mxfp6_quantize: in_dtype %d (want MI355_F32, MI355_F16 or MI355_BF16)", in_dtype);
  if (element_format != MI355_FP6_E2M3 && element_format != MI355_FP6_E3M2)
    return fail(-MI355_E_DTYPE, "mxfp6_quantize: element_format %d (want MI355_FP6_E2M3 or MI355_FP6_E3M2)", element_format);
  if (!aligned16(x) || (reinterpret_cast<uintptr_t>(codes) & 7u))
    return fail(-MI355_E_ALIGN, "mxfp6_quantize: x must be 16-byte aligned and codes 8-byte aligned");
  const long long n_blocks = rows * K / 32;
  if ((n_blocks + 255) / 256 > 0x7fffffffll) return fail(-MI355_E_SHAPE, "mxfp6_quantize: too many blocks for one launch");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  return element_format == MI355_FP6_E2M3 ? launch_q6<0>(x, in_dtype, n_blocks, codes, scales, s)
                                          : launch_q6<1>(x, in_dtype, n_blocks, codes, scales, s);
}
