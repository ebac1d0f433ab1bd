// MXFP4 and MXFP8 quantisation for gfx950 (the fp8 kernel is at the end of the file).  MXFP4: x[rows, K] (fp16 / bf16 / fp32) -> E2M1 codes (two per byte, even k in the
// low nibble) + one E8M0 scale byte per 32 consecutive k.  This is the producer of the block-scaled GEMM's
// operands.  OCP Microscaling Formats v1.0 conversion: shared exponent = floor(log2(max |x|)) - 2 per block
// (clamped to [-127, 127]; an all-zero block takes -127, a block with a NaN or infinity the NaN scale 0xFF),
// every element scaled by 2^-shared exactly and rounded to the nearest E2M1 value with ties to the even code,
// magnitudes beyond 6 saturating to 6.
//
// HBM bound (2 or 4 bytes in, 17/32 byte out per element).  K % 32 == 0, so blocks never straddle rows and
// the whole tensor is one flat run of blocks: a lane takes 8 consecutive elements (one 16-byte load for
// 16-bit inputs), four neighbouring lanes form a block and share the maximum through two lane exchanges; a
// wave covers 16 blocks and writes their 16 scale bytes as four dwords.
//
// Rounding is done by v_cvt_scalef32_pk_fp4_{f16,bf16,f32}, which divides two values by a power-of-two
// scale and rounds them to E2M1 exactly as the format asks (nearest, ties to the even code, saturating;
// checked against the threshold form over every tie and 3400 other magnitudes per scale).  Waves that hold
// a non-finite value or a block whose exponent is clamped at the bottom of the E8M0 range (the scale is no
// longer a normal float) take the threshold form in software instead.
#include "common.hpp"

namespace mi355 {

typedef _Float16 half2v_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef unsigned short ushortx2 __attribute__((ext_vector_type(2)));

// software rounding of 8 fp32 values with the block's exponent (zero magnitudes for a poisoned block)
__device__ __forceinline__ unsigned quantize8_sw(const float* v, int shared, bool poisoned) {
  unsigned packed = 0;
#pragma unroll
  for (int i = 0; i < 8; i++) {
    const float xi = poisoned ? 0.f : v[i];
    const float y = __builtin_fabsf(__builtin_amdgcn_ldexpf(xi, -shared));  // exact power-of-two scaling
    // thresholds halfway between neighbouring values; a tie goes to the even code
    unsigned c = (y > 0.25f) + (y >= 0.75f) + (y > 1.25f) + (y >= 1.75f) + (y > 2.5f) + (y >= 3.5f) + (y > 5.0f);
    c |= (__builtin_bit_cast(unsigned, v[i]) >> 31) << 3;
    packed |= c << (4 * i);
  }
  return packed;
}

template <typename T> struct QIn;
// 16-bit inputs: 8 elements = 4 dwords; |x| bit patterns order like unsigned integers (NaN > inf > finite),
// so the block maximum is a packed unsigned maximum
template <bool BF16> struct QIn16 {
  intx4 w;
  __device__ __forceinline__ void load(const void* p) { w = *reinterpret_cast<const intx4*>(p); }
  __device__ __forceinline__ void zero() { w = intx4{0, 0, 0, 0}; }
  static constexpr unsigned kInf = BF16 ? 0x7f80u : 0x7c00u;
  __device__ __forceinline__ unsigned amax_bits() const {
    ushortx2 m = __builtin_bit_cast(ushortx2, (unsigned)w[0] & 0x7fff7fffu);
#pragma unroll
    for (int i = 1; i < 4; i++) m = __builtin_elementwise_max(m, __builtin_bit_cast(ushortx2, (unsigned)w[i] & 0x7fff7fffu));
    return m[0] > m[1] ? m[0] : m[1];
  }
  static __device__ __forceinline__ float bits_to_float(unsigned b) {
    if (BF16) return __builtin_bit_cast(float, b << 16);
    return (float)__builtin_bit_cast(half_t, (unsigned short)b);
  }
  __device__ __forceinline__ void to_float(float* v) const {
    const unsigned u[4] = {(unsigned)w[0], (unsigned)w[1], (unsigned)w[2], (unsigned)w[3]};
#pragma unroll
    for (int i = 0; i < 4; i++) {
      if (BF16) {
        v[2 * i] = __builtin_bit_cast(float, u[i] << 16);
        v[2 * i + 1] = __builtin_bit_cast(float, u[i] & 0xffff0000u);
      } else {
        v[2 * i] = (float)__builtin_bit_cast(half_t, (unsigned short)(u[i] & 0xffffu));
        v[2 * i + 1] = (float)__builtin_bit_cast(half_t, (unsigned short)(u[i] >> 16));
      }
    }
  }
  __device__ __forceinline__ unsigned convert(float scale) const {
    // the byte selector is the last argument; each source dword is taken out of the vector first
    const unsigned u0 = (unsigned)w[0], u1 = (unsigned)w[1], u2 = (unsigned)w[2], u3 = (unsigned)w[3];
    unsigned r = 0;
    if (BF16) {
      r = __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(r, __builtin_bit_cast(bf16x2_t, u0), scale, 0);
      r = __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(r, __builtin_bit_cast(bf16x2_t, u1), scale, 1);
      r = __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(r, __builtin_bit_cast(bf16x2_t, u2), scale, 2);
      r = __builtin_amdgcn_cvt_scalef32_pk_fp4_bf16(r, __builtin_bit_cast(bf16x2_t, u3), scale, 3);
    } else {
      r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f16(r, __builtin_bit_cast(half2v_t, u0), scale, 0);
      r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f16(r, __builtin_bit_cast(half2v_t, u1), scale, 1);
      r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f16(r, __builtin_bit_cast(half2v_t, u2), scale, 2);
      r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f16(r, __builtin_bit_cast(half2v_t, u3), scale, 3);
    }
    return r;
  }
};
template <> struct QIn<half_t> : QIn16<false> {};
template <> struct QIn<unsigned short> : QIn16<true> {};
template <> struct QIn<float> {
  float f[8];
  static constexpr unsigned kInf = 0x7f800000u;
  __device__ __forceinline__ void load(const void* p) {
    floatx4 a = *reinterpret_cast<const floatx4*>(p), b = *(reinterpret_cast<const floatx4*>(p) + 1);
#pragma unroll
    for (int i = 0; i < 4; i++) {
      f[i] = a[i];
      f[4 + i] = b[i];
    }
  }
  __device__ __forceinline__ void zero() {
#pragma unroll
    for (int i = 0; i < 8; i++) f[i] = 0.f;
  }
  __device__ __forceinline__ unsigned amax_bits() const {
    unsigned m = 0;
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const unsigned b = __builtin_bit_cast(unsigned, f[i]) & 0x7fffffffu;
      m = b > m ? b : m;
    }
    return m;
  }
  static __device__ __forceinline__ float bits_to_float(unsigned b) { return __builtin_bit_cast(float, b); }
  __device__ __forceinline__ void to_float(float* v) const {
#pragma unroll
    for (int i = 0; i < 8; i++) v[i] = f[i];
  }
  __device__ __forceinline__ unsigned convert(float scale) const {
    unsigned r = 0;
    r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(r, f[0], f[1], scale, 0);
    r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(r, f[2], f[3], scale, 1);
    r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(r, f[4], f[5], scale, 2);
    r = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(r, f[6], f[7], scale, 3);
    return r;
  }
};

// A wave covers QU chunks of 512 elements; all of a lane's loads are issued before any is used, which is what
// keeps enough bytes in flight to stream at the memory system's rate.
constexpr int QU = 4;

// scale bytes of one 512-element chunk: block b lives in lanes 4b..4b+3; lanes 0..3 each gather four of them
__device__ __forceinline__ void store_scales(uint8_t* scales, int sbyte, int lane, long long b0, long long n_blocks) {
  unsigned sw = 0;
#pragma unroll
  for (int j = 0; j < 4; j++) sw |= (unsigned)__shfl(sbyte, 16 * (lane & 3) + 4 * j) << (8 * j);
  if (lane < 4) {
    if (b0 + 4 <= n_blocks && ((reinterpret_cast<uintptr_t>(scales) + b0) & 3) == 0) {
      *reinterpret_cast<unsigned*>(scales + b0) = sw;
    } else {
#pragma unroll
      for (int j = 0; j < 4; j++)
        if (b0 + j < n_blocks) scales[b0 + j] = (uint8_t)(sw >> (8 * j));
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void mxfp4_quantize_kernel(const T* __restrict__ x, uint8_t* __restrict__ codes,
                                                             uint8_t* __restrict__ scales, long long n_elems) {
  const int lane = threadIdx.x & 63;
  const long long wave_id = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  QIn<T> in[QU];
#pragma unroll
  for (int u = 0; u < QU; u++) {
    const long long e0 = (wave_id * QU + u) * 512 + lane * 8;  // first of this lane's 8 elements of chunk u
    if (e0 < n_elems) in[u].load(x + e0);  // n_elems is a multiple of 32, so a lane is all in or all out
    else in[u].zero();
  }
#pragma unroll
  for (int u = 0; u < QU; u++) {
    const long long e0 = (wave_id * QU + u) * 512 + lane * 8;
    const bool live = e0 < n_elems;
    // block maximum of |x| over 4 lanes, as a bit pattern: anything at or above infinity poisons the block
    unsigned mb = in[u].amax_bits();
    unsigned o = __shfl_xor(mb, 1);
    mb = o > mb ? o : mb;
    o = __shfl_xor(mb, 2);
    mb = o > mb ? o : mb;
    const bool poisoned = mb >= QIn<T>::kInf;
    const float amax = QIn<T>::bits_to_float(mb);
    // floor(log2(amax)) = frexp exponent - 1 (also right for subnormal inputs)
    int shared = mb == 0 ? -127 : __builtin_amdgcn_frexp_expf(amax) - 1 - 2;
    shared = shared < -127 ? -127 : (shared > 127 ? 127 : shared);
    unsigned packed;
    if (__builtin_amdgcn_ballot_w64(live && (poisoned || shared < -126)) != 0) {
      float v[8];
      in[u].to_float(v);
      packed = quantize8_sw(v, shared, poisoned);
    } else {
      packed = in[u].convert(__builtin_amdgcn_ldexpf(1.0f, shared));
    }
    if (live) *reinterpret_cast<unsigned*>(codes + (e0 >> 1)) = packed;
    store_scales(scales, poisoned ? 255 : shared + 127, lane, (wave_id * QU + u) * 16 + lane * 4, n_elems >> 5);
  }
}

// MXFP8 (E4M3 codes, one byte per element): the same block walk with the element format's emax of 8 -- shared
// exponent floor(log2(max |x|)) - 8 -- and values beyond the largest finite code (448) saturating to it.  The
// scaling by 2^-shared is exact (v_ldexp_f32), the clamp makes every value representable in range, and
// v_cvt_pk_fp8_f32 rounds to the nearest code, ties to even, subnormal codes included (checked against the
// brute-force nearest-code search over every fp16 value).
template <typename T>
__global__ __launch_bounds__(256) void mxfp8_quantize_kernel(const T* __restrict__ x, uint8_t* __restrict__ codes,
                                                             uint8_t* __restrict__ scales, long long n_elems) {
  const int lane = threadIdx.x & 63;
  const long long wave_id = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  QIn<T> in[QU];
#pragma unroll
  for (int u = 0; u < QU; u++) {
    const long long e0 = (wave_id * QU + u) * 512 + lane * 8;
    if (e0 < n_elems) in[u].load(x + e0);
    else in[u].zero();
  }
#pragma unroll
  for (int u = 0; u < QU; u++) {
    const long long e0 = (wave_id * QU + u) * 512 + lane * 8;
    const bool live = e0 < n_elems;
    unsigned mb = in[u].amax_bits();
    unsigned o = __shfl_xor(mb, 1);
    mb = o > mb ? o : mb;
    o = __shfl_xor(mb, 2);
    mb = o > mb ? o : mb;
    const bool poisoned = mb >= QIn<T>::kInf;
    const float amax = QIn<T>::bits_to_float(mb);
    int shared = mb == 0 ? -127 : __builtin_amdgcn_frexp_expf(amax) - 1 - 8;
    shared = shared < -127 ? -127 : (shared > 127 ? 127 : shared);
    float v[8];
    in[u].to_float(v);
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const float y = __builtin_amdgcn_ldexpf(v[i], -shared);
      v[i] = poisoned ? __builtin_copysignf(0.f, v[i]) : __builtin_fminf(__builtin_fmaxf(y, -448.f), 448.f);
    }
    int w0 = __builtin_amdgcn_cvt_pk_fp8_f32(v[0], v[1], 0, false);
    w0 = __builtin_amdgcn_cvt_pk_fp8_f32(v[2], v[3], w0, true);
    int w1 = __builtin_amdgcn_cvt_pk_fp8_f32(v[4], v[5], 0, false);
    w1 = __builtin_amdgcn_cvt_pk_fp8_f32(v[6], v[7], w1, true);
    if (live) *reinterpret_cast<intx2*>(codes + e0) = intx2{w0, w1};
    store_scales(scales, poisoned ? 255 : shared + 127, lane, (wave_id * QU + u) * 16 + lane * 4, n_elems >> 5);
  }
}

}  // namespace mi355

using namespace mi355;

extern "C" int mi355_mxfp4_quantize(const void* x, int in_dtype, int64_t rows, int64_t K, void* codes, void* scales,
                                    void* stream) {
  if (!x || !codes || !scales) return fail(-MI355_E_NULL, "mxfp4_quantize: null pointer");
  if (rows <= 0 || K <= 0 || K % 32 != 0 || rows > (1ll << 40) / K)
    return fail(-MI355_E_SHAPE, "mxfp4_quantize: bad shape rows=%lld K=%lld (K must be a multiple of 32)", (long long)rows,
                (long long)K);
  if (in_dtype != MI355_F32 && in_dtype != MI355_F16 && in_dtype != MI355_BF16)
    return fail(-MI355_E_DTYPE, "mxfp4_quantize: in_dtype %d (want MI355_F32, MI355_F16 or MI355_BF16)", in_dtype);
  if (!aligned16(x) || (reinterpret_cast<uintptr_t>(codes) & 3u))
    return fail(-MI355_E_ALIGN, "mxfp4_quantize: x must be 16-byte aligned and codes 4-byte aligned");
  const long long n = rows * K;
  const long long waves = (n + 512 * QU - 1) / (512 * QU);
  dim3 grid((unsigned)((waves + 3) / 4)), block(256);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (in_dtype == MI355_F16)
    hipLaunchKernelGGL(mxfp4_quantize_kernel<half_t>, grid, block, 0, s, (const half_t*)x, (uint8_t*)codes, (uint8_t*)scales, n);
  else if (in_dtype == MI355_BF16)
    hipLaunchKernelGGL(mxfp4_quantize_kernel<unsigned short>, grid, block, 0, s, (const unsigned short*)x, (uint8_t*)codes,
                       (uint8_t*)scales, n);
  else
    hipLaunchKernelGGL(mxfp4_quantize_kernel<float>, grid, block, 0, s, (const float*)x, (uint8_t*)codes, (uint8_t*)scales, n);
  return check_launch("mxfp4_quantize_kernel", grid, block, 0);
}

extern "C" int mi355_mxfp8_quantize(const void* x, int in_dtype, int64_t rows, int64_t K, void* codes, void* scales,
                                    void* stream) {
  if (!x || !codes || !scales) return fail(-MI355_E_NULL, "mxfp8_quantize: null pointer");
  if (rows <= 0 || K <= 0 || K % 32 != 0 || rows > (1ll << 40) / K)
    return fail(-MI355_E_SHAPE, "mxfp8_quantize: bad shape rows=%lld K=%lld (K must be a multiple of 32)", (long long)rows,
                (long long)K);
  if (in_dtype != MI355_F32 && in_dtype != MI355_F16 && in_dtype != MI355_BF16)
    return fail(-MI355_E_DTYPE, "mxfp8_quantize: in_dtype %d (want MI355_F32, MI355_F16 or MI355_BF16)", in_dtype);
  if (!aligned16(x) || (reinterpret_cast<uintptr_t>(codes) & 7u))
    return fail(-MI355_E_ALIGN, "mxfp8_quantize: x must be 16-byte aligned and codes 8-byte aligned");
  const long long n = rows * K;
  const long long waves = (n + 512 * QU - 1) / (512 * QU);
  dim3 grid((unsigned)((waves + 3) / 4)), block(256);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (in_dtype == MI355_F16)
    hipLaunchKernelGGL(mxfp8_quantize_kernel<half_t>, grid, block, 0, s, (const half_t*)x, (uint8_t*)codes, (uint8_t*)scales, n);
  else if (in_dtype == MI355_BF16)
    hipLaunchKernelGGL(mxfp8_quantize_kernel<unsigned short>, grid, block, 0, s, (const unsigned short*)x, (uint8_t*)codes,
                       (uint8_t*)scales, n);
  else
    hipLaunchKernelGGL(mxfp8_quantize_kernel<float>, grid, block, 0, s, (const float*)x, (uint8_t*)codes, (uint8_t*)scales, n);
  return check_launch("mxfp8_quantize_kernel", grid, block, 0);
}
