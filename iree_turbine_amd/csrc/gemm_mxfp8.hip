// Block-scaled MXFP8 GEMM for gfx950:  C[M,N] = dq(A) . dq(B)^T, bf16 (or fp32) output.
//
// Codes are OCP FP8 E4M3 bytes (one per element), one E8M0 scale byte per 32 consecutive k.  The arithmetic
// is v_mfma_scale_f32_32x32x64_f8f6f4 with both operands in fp8 format: a lane supplies 32 bytes -- exactly
// one scale block -- and its scale byte, and the instruction applies 2^(scale-127) in hardware.
//
// Operand layout of the instruction with 8-bit elements (measured with one-hot operands): of the 64 k of a
// k-step, block 0 (k 0..31) is scaled by the scale of lanes 0..31 and block 1 by that of lanes 32..63, but the
// ELEMENTS of both blocks are split over both lane halves -- lane (r, h) holds elements 16h..16h+15 of block
// 0 in its first 16 bytes and elements 16h..16h+15 of block 1 in its second 16 bytes.
//
// Tiling is the MXFP4 GEMM's with twice the bytes per element: a K slab is 128 elements = 128 bytes per row
// = 8 chunks of 16 bytes = 4 scale blocks = 2 k-steps of 64, copied with direct-to-LDS loads into a two-stage
// ring with the same XOR swizzle.  k-step ks (0, 1) pairs block ks with block 2+ks: a lane reads chunk 2ks+h
// (its half of block ks) and chunk 4+2ks+h (its half of block 2+ks), and supplies byte ks (h = 0) or 2+ks
// (h = 1) of the ONE scale dword a row has per slab; lanes of the upper half shift their dword right by 16
// once, so that op_sel = ks picks the byte for both halves.
#include <math.h>
#include <type_traits>

#include "common.hpp"

namespace mi355 {

namespace {

__device__ __forceinline__ void map_tile8(int pid, int tiles_m, int tiles_n, int group_m, int& tm, int& tn) {
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

template <typename OutT> struct Out8;
template <> struct Out8<float> {
  static __device__ __forceinline__ void store4(float* p, float a, float b, float c, float d) {
    floatx4 v = {a, b, c, d};
    *reinterpret_cast<floatx4*>(p) = v;
  }
  static __device__ __forceinline__ void store1(float* p, float a) { *p = a; }
};
template <> struct Out8<unsigned short> {  // bf16 bits
  static __device__ __forceinline__ void store4(unsigned short* p, float a, float b, float c, float d) {
    ushortx4 v = {f32_to_bf16_rne(a), f32_to_bf16_rne(b), f32_to_bf16_rne(c), f32_to_bf16_rne(d)};
    *reinterpret_cast<ushortx4*>(p) = v;
  }
  static __device__ __forceinline__ void store1(unsigned short* p, float a) { *p = f32_to_bf16_rne(a); }
};

// byte SEL of sa / sb scales the lane's 32-element block of a / b (format code 0 = fp8 E4M3)
template <int SEL>
__device__ __forceinline__ floatx16 mfma_fp8_32x32x64(intx8 a, int sa, intx8 b, int sb, floatx16 c) {
  return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 0, 0, SEL, sa, SEL, sb);
}

}  // namespace

// SCALED = false: plain fp8 GEMM, C = alpha . A . B^T (every block scale is 2^0, no scale traffic).
template <int BM, int BN, int WM, int WN, typename OutT, bool SCALED>
__global__ __launch_bounds__(WM* WN * 64) void gemm_mxfp8_tiled(const uint8_t* __restrict__ A, const uint8_t* __restrict__ As,
                                                                const uint8_t* __restrict__ B, const uint8_t* __restrict__ Bs,
                                                                OutT* __restrict__ C, int M, int N, int K, int tiles_m,
                                                                int tiles_n, int group_m, float alpha) {
  constexpr int NW = WM * WN;
  constexpr int WTM = BM / WM, WTN = BN / WN;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int A_BYTES = BM * 128, B_BYTES = BN * 128, STAGE = A_BYTES + B_BYTES;
  static_assert((BM / 8) % NW == 0 && (BN / 8) % NW == 0 && NW % 2 == 0, "loads must split evenly over an even number of waves");
  constexpr int LA = BM / 8 / NW, LB = BN / 8 / NW;

  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave / WN, wn = wave % WN;
  int tile_m, tile_n;
  map_tile8(blockIdx.x, tiles_m, tiles_n, group_m, tile_m, tile_n);

  const int Ksc = K >> 5;  // scale bytes per row
  const int lrow = lane >> 3;
  // chunk c of row r lives in slot c ^ ((r >> 1) & 7): conflict-free fragment reads on 64 LDS banks
  const int lchunk = (lane & 7) ^ (((wave & 1) << 2) | (lrow >> 1));
  const uint8_t* a_src = A + (size_t)(tile_m * BM + wave * 8) * K;
  const uint8_t* b_src = B + (size_t)(tile_n * BN + wave * 8) * K;
  const unsigned lane_off = (unsigned)lrow * (unsigned)K + (unsigned)lchunk * 16u;
  const size_t row_step = (size_t)NW * 8 * K;
  auto issue_loads = [&](int stage, int slab) {
    char* dst = lds + stage * STAGE + wave * 1024;
    const uint8_t* ap = a_src + slab * 128;
    const uint8_t* bp = b_src + slab * 128;
#pragma unroll
    for (int i = 0; i < LA; i++) load_lds_16B(ap + i * row_step + lane_off, dst + i * NW * 1024);
#pragma unroll
    for (int i = 0; i < LB; i++) load_lds_16B(bp + i * row_step + lane_off, dst + A_BYTES + i * NW * 1024);
  };

  const int r32 = lane & 31, h = lane >> 5;
  const int sw = (h ^ ((r32 >> 1) & 7)) * 16;  // chunk h of the row, swizzled; k-step ks adds 2 ks, the second block 4
  const int a_base = (wm * WTM + r32) * 128 + sw;
  const int b_base = A_BYTES + (wn * WTN + r32) * 128 + sw;
  auto read_frags = [&](const char* st, int ks, intx8* fm, intx8* fn) {
#pragma unroll
    for (int j = 0; j < TM; j++) {
      const int at = (a_base ^ (ks * 32)) + j * 4096;
      const intx4 lo = *reinterpret_cast<const intx4*>(st + at);
      const intx4 hi = *reinterpret_cast<const intx4*>(st + (at ^ 64));
      fm[j] = intx8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    }
#pragma unroll
    for (int i = 0; i < TN; i++) {
      const int at = (b_base ^ (ks * 32)) + i * 4096;
      const intx4 lo = *reinterpret_cast<const intx4*>(st + at);
      const intx4 hi = *reinterpret_cast<const intx4*>(st + (at ^ 64));
      fn[i] = intx8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    }
  };

  // the row's scale dword of a slab (4 blocks), shifted so that byte ks is this lane's block of k-step ks
  const uint8_t* as_src = As + (size_t)(tile_m * BM + wm * WTM + r32) * Ksc;
  const uint8_t* bs_src = Bs + (size_t)(tile_n * BN + wn * WTN + r32) * Ksc;
  auto fetch_scales = [&](int* da, int* db, int slab) {
    if constexpr (SCALED) {
#pragma unroll
      for (int j = 0; j < TM; j++)
        da[j] = (int)(*reinterpret_cast<const unsigned*>(as_src + (size_t)j * 32 * Ksc + slab * 4) >> (16 * h));
#pragma unroll
      for (int i = 0; i < TN; i++)
        db[i] = (int)(*reinterpret_cast<const unsigned*>(bs_src + (size_t)i * 32 * Ksc + slab * 4) >> (16 * h));
    } else {
#pragma unroll
      for (int j = 0; j < TM; j++) da[j] = 0x7f7f7f7f;
#pragma unroll
      for (int i = 0; i < TN; i++) db[i] = 0x7f7f7f7f;
    }
  };

  floatx16 acc[TN][TM];
#pragma unroll
  for (int i = 0; i < TN; i++)
#pragma unroll
    for (int j = 0; j < TM; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;
  auto mfmas = [&](auto ks_tag, const intx8* fm, const intx8* fn, const int* ca, const int* cb) __attribute__((always_inline)) {
    constexpr int KS = decltype(ks_tag)::value;
#pragma unroll
    for (int i = 0; i < TN; i++)
#pragma unroll
      for (int j = 0; j < TM; j++) acc[i][j] = mfma_fp8_32x32x64<KS>(fn[i], cb[i], fm[j], ca[j], acc[i][j]);
  };
  auto interleave = [&]() {  // fragment reads (two per fragment) between the MFMAs of the previous k-step
#pragma unroll
    for (int i = 0; i < TM * TN; i++) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, (2 * (TM + TN) + TM * TN - 1) / (TM * TN), 0);
    }
  };

  const int KT = K / 128;  // even (checked on the host)
  intx8 fm0[TM], fn0[TN], fm1[TM], fn1[TN];
  int sa[2][TM], sb[2][TN];
  using K0 = std::integral_constant<int, 0>;
  using K1 = std::integral_constant<int, 1>;

  issue_loads(0, 0);
  fetch_scales(sa[0], sb[0], 0);
  wait_vmcnt0();
  __syncthreads();
  issue_loads(1, KT > 1 ? 1 : 0);
  read_frags(lds, 0, fm0, fn0);

  // One slab: k-step 0's MFMAs with the reads of k-step 1; the wait + barrier that retire the slab; k-step
  // 1's MFMAs with the loads of the slab after next and the first reads of the next slab.  The scale dwords of
  // the next slab are requested at the top and are the newest loads in flight at the wait, which leaves
  // them outstanding.
  auto slab = [&](auto par_tag, int kt) __attribute__((always_inline)) {
    constexpr int CUR = decltype(par_tag)::value, NXT = CUR ^ 1;
    const char* st = lds + CUR * STAGE;
    __builtin_amdgcn_sched_barrier(0);
    fetch_scales(sa[NXT], sb[NXT], kt + 1 < KT ? kt + 1 : KT - 1);
    read_frags(st, 1, fm1, fn1);
    mfmas(K0{}, fm0, fn0, sa[CUR], sb[CUR]);
    interleave();
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(SCALED ? TM + TN : 0) : "memory");
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
    issue_loads(CUR, kt + 2 < KT ? kt + 2 : KT - 1);
    read_frags(lds + NXT * STAGE, 0, fm0, fn0);
    mfmas(K1{}, fm1, fn1, sa[CUR], sb[CUR]);
#pragma unroll
    for (int i = 0; i < TM * TN; i++) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x010, (LA + LB + TM * TN - 1) / (TM * TN), 0);
      __builtin_amdgcn_sched_group_barrier(0x100, (2 * (TM + TN) + TM * TN - 1) / (TM * TN), 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  for (int kt = 0; kt < KT; kt += 2) {
    slab(K0{}, kt);
    slab(K1{}, kt + 1);
  }
  wait_vmcnt0();  // the speculative loads of the last slabs

  const int m0 = tile_m * BM + wm * WTM + r32;
  const int n0 = tile_n * BN + wn * WTN + 4 * h;
#pragma unroll
  for (int j = 0; j < TM; j++) {
    OutT* crow = C + (size_t)(m0 + j * 32) * N + n0;
#pragma unroll
    for (int i = 0; i < TN; i++)
#pragma unroll
      for (int q = 0; q < 4; q++)
        Out8<OutT>::store4(crow + i * 32 + q * 8, alpha * acc[i][j][4 * q], alpha * acc[i][j][4 * q + 1], alpha * acc[i][j][4 * q + 2],
                           alpha * acc[i][j][4 * q + 3]);
  }
}

// Any shape with K % 32 == 0: one wave per 32x32 output tile, operands straight from global memory.
template <typename OutT, bool SCALED>
__global__ __launch_bounds__(256) void gemm_mxfp8_generic(const uint8_t* __restrict__ A, const uint8_t* __restrict__ As,
                                                          const uint8_t* __restrict__ B, const uint8_t* __restrict__ Bs,
                                                          OutT* __restrict__ C, int M, int N, int K, float alpha) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r32 = lane & 31, h = lane >> 5;
  const int m = blockIdx.y * 32 + r32;
  const int n = (blockIdx.x * 4 + wave) * 32 + r32;
  const int Ksc = K >> 5;
  floatx16 acc;
#pragma unroll
  for (int r = 0; r < 16; r++) acc[r] = 0.f;
  const intx8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  for (int kb = 0; kb < Ksc; kb += 2) {  // two scale blocks (64 elements) per MFMA
    const int blk = kb + h;  // the block this lane's SCALE belongs to; its elements are halves of both blocks
    const bool k_ok = blk < Ksc;
    intx8 fa = zero, fb = zero;
    int sa = 127, sb = 127;
    const bool k1_ok = kb + 1 < Ksc;  // a lone last block pairs with zeros
    if (m < M) {
      const uint8_t* row = A + (size_t)m * K + kb * 32 + 16 * h;
      const intx4 lo = *reinterpret_cast<const intx4*>(row);
      const intx4 hi = k1_ok ? *reinterpret_cast<const intx4*>(row + 32) : intx4{0, 0, 0, 0};
      fa = intx8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      if (SCALED && k_ok) sa = As[(size_t)m * Ksc + blk];
    }
    if (n < N) {
      const uint8_t* row = B + (size_t)n * K + kb * 32 + 16 * h;
      const intx4 lo = *reinterpret_cast<const intx4*>(row);
      const intx4 hi = k1_ok ? *reinterpret_cast<const intx4*>(row + 32) : intx4{0, 0, 0, 0};
      fb = intx8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      if (SCALED && k_ok) sb = Bs[(size_t)n * Ksc + blk];
    }
    acc = mfma_fp8_32x32x64<0>(fb, sb, fa, sa, acc);
  }
  if (m < M) {
    const int nb = (blockIdx.x * 4 + wave) * 32;
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const int nn = nb + 8 * (r >> 2) + 4 * h + (r & 3);
      if (nn < N) Out8<OutT>::store1(C + (size_t)m * N + nn, alpha * acc[r]);
    }
  }
}

static const char* kMx8Variants[] = {"tiled_256x256x128_w2x2", "generic_32x128"};
int mxfp8_variant_count() { return 2; }
const char* mxfp8_variant_name(int i) { return (i >= 0 && i < 2) ? kMx8Variants[i] : nullptr; }

template <typename OutT, bool SCALED>
static int launch_mx8(int variant, const void* a, const void* as, const void* b, const void* bs, void* c, int M, int N, int K,
                      float alpha, hipStream_t stream) {
  if (variant == 0) {
    auto kern = gemm_mxfp8_tiled<256, 256, 2, 2, OutT, SCALED>;
    constexpr int lds_bytes = 2 * 512 * 128;
    static bool attr_set = false;
    if (!attr_set) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
      if (e != hipSuccess) {
        set_error("hipFuncSetAttribute(gemm_mxfp8_tiled, %d bytes LDS): %s", lds_bytes, hipGetErrorString(e));
        return (int)e;
      }
      attr_set = true;
    }
    const int tiles_m = M / 256, tiles_n = N / 256;
    dim3 grid(tiles_m * tiles_n), block(256);
    hipLaunchKernelGGL(kern, grid, block, lds_bytes, stream, (const uint8_t*)a, (const uint8_t*)as, (const uint8_t*)b,
                       (const uint8_t*)bs, (OutT*)c, M, N, K, tiles_m, tiles_n, 4, alpha);
    return check_launch("gemm_mxfp8_tiled", grid, block, lds_bytes);
  }
  dim3 grid((N + 127) / 128, (M + 31) / 32), block(256);
  hipLaunchKernelGGL((gemm_mxfp8_generic<OutT, SCALED>), grid, block, 0, stream, (const uint8_t*)a, (const uint8_t*)as,
                     (const uint8_t*)b, (const uint8_t*)bs, (OutT*)c, M, N, K, alpha);
  return check_launch("gemm_mxfp8_generic", grid, block, 0);
}

}  // namespace mi355

using namespace mi355;

extern "C" int mi355_mxfp8_gemm(const void* a, const void* a_scale, const void* b, const void* b_scale, void* c, int64_t M,
                                int64_t N, int64_t K, int out_dtype, int variant, void* stream) {
  if (!a || !a_scale || !b || !b_scale || !c) return fail(-MI355_E_NULL, "mxfp8_gemm: null pointer");
  if (M <= 0 || N <= 0 || K <= 0 || M > (1 << 30) || N > (1 << 30) || K > (1 << 27))
    return fail(-MI355_E_SHAPE, "mxfp8_gemm: bad shape M=%lld N=%lld K=%lld", (long long)M, (long long)N, (long long)K);
  if (K % 32 != 0) return fail(-MI355_E_SHAPE, "mxfp8_gemm: K=%lld must be a multiple of the 32-element scale block", (long long)K);
  if (out_dtype != MI355_BF16 && out_dtype != MI355_F32)
    return fail(-MI355_E_DTYPE, "mxfp8_gemm: out_dtype %d (want MI355_BF16 or MI355_F32)", out_dtype);
  if (variant > 1) return fail(-MI355_E_DTYPE, "mxfp8_gemm: variant %d out of range", variant);
  if (!aligned16(a) || !aligned16(b) || !aligned16(c)) return fail(-MI355_E_ALIGN, "mxfp8_gemm: a, b, c must be 16-byte aligned");
  const bool sc_al4 = ((reinterpret_cast<uintptr_t>(a_scale) | reinterpret_cast<uintptr_t>(b_scale)) & 3u) == 0;
  const bool fits0 = sc_al4 && M % 256 == 0 && N % 256 == 0 && K % 256 == 0 && K >= 256;  // slabs in pairs, one scale dword per slab
  if (variant < 0) variant = fits0 ? 0 : 1;
  else if (variant == 0 && !fits0)
    return fail(-MI355_E_SHAPE, "mxfp8_gemm: variant %s needs M%%256==0, N%%256==0, K%%256==0 and 4-byte aligned scales", kMx8Variants[0]);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (out_dtype == MI355_F32) return launch_mx8<float, true>(variant, a, a_scale, b, b_scale, c, (int)M, (int)N, (int)K, 1.f, s);
  return launch_mx8<unsigned short, true>(variant, a, a_scale, b, b_scale, c, (int)M, (int)N, (int)K, 1.f, s);
}

extern "C" int mi355_fp8_gemm(const void* a, const void* b, void* c, int64_t M, int64_t N, int64_t K, float alpha, int out_dtype,
                              int variant, void* stream) {
  if (!a || !b || !c) return fail(-MI355_E_NULL, "fp8_gemm: null pointer");
  if (M <= 0 || N <= 0 || K <= 0 || M > (1 << 30) || N > (1 << 30) || K > (1 << 27))
    return fail(-MI355_E_SHAPE, "fp8_gemm: bad shape M=%lld N=%lld K=%lld", (long long)M, (long long)N, (long long)K);
  if (K % 32 != 0) return fail(-MI355_E_SHAPE, "fp8_gemm: K=%lld must be a multiple of 32", (long long)K);
  if (out_dtype != MI355_BF16 && out_dtype != MI355_F32)
    return fail(-MI355_E_DTYPE, "fp8_gemm: out_dtype %d (want MI355_BF16 or MI355_F32)", out_dtype);
  if (variant > 1) return fail(-MI355_E_DTYPE, "fp8_gemm: variant %d out of range", variant);
  if (!isfinite(alpha)) return fail(-MI355_E_SHAPE, "fp8_gemm: alpha must be finite");
  if (!aligned16(a) || !aligned16(b) || !aligned16(c)) return fail(-MI355_E_ALIGN, "fp8_gemm: a, b, c must be 16-byte aligned");
  const bool fits0 = M % 256 == 0 && N % 256 == 0 && K % 256 == 0 && K >= 256;
  if (variant < 0) variant = fits0 ? 0 : 1;
  else if (variant == 0 && !fits0)
    return fail(-MI355_E_SHAPE, "fp8_gemm: variant %s needs M%%256==0, N%%256==0, K%%256==0", kMx8Variants[0]);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (out_dtype == MI355_F32) return launch_mx8<float, false>(variant, a, nullptr, b, nullptr, c, (int)M, (int)N, (int)K, alpha, s);
  return launch_mx8<unsigned short, false>(variant, a, nullptr, b, nullptr, c, (int)M, (int)N, (int)K, alpha, s);
}
