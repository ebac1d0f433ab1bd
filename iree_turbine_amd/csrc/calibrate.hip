// Calibration loops: what the MFMA unit of this board sustains when nothing else is in the way.
//
// Every wave keeps its operands in registers and issues MFMAs back to back: no LDS, no global traffic inside the
// loop.  The rate such a loop sustains depends on the DATA (the board's power limit lowers the clock as more bits
// toggle), so the caller supplies the operand bytes: all zeros reads the issue-rate peak, operands drawn like a
// benchmark's read the ceiling any kernel can reach on that benchmark's data.  A roofline fraction quoted against
// the datasheet peak can then be read against the measured ceiling as well.
#include <type_traits>

#include "common.hpp"

namespace mi355 {

constexpr int CAL_WAVES = 4;      // one wave per SIMD
constexpr int CAL_CHAINS = 8;     // independent accumulator chains per wave: more than the MFMA pipeline is deep

// 32x32x16 fp16 MFMAs: per wave and trip, CAL_CHAINS MFMAs of 32*32*16*2 flop.
__global__ __launch_bounds__(CAL_WAVES * 64) void calibrate_mfma_f16_kernel(const half8* __restrict__ operands, unsigned mask,
                                                                            float* __restrict__ sink, int trips) {
  const unsigned t = threadIdx.x + blockIdx.x * blockDim.x;
  half8 a[4], b[4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    a[i] = operands[(t * 8 + i) & mask];
    b[i] = operands[(t * 8 + 4 + i) & mask];
  }
  floatx16 c[CAL_CHAINS];
#pragma unroll
  for (int i = 0; i < CAL_CHAINS; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) c[i][r] = 0.f;
#pragma unroll 1
  for (int it = 0; it < trips; it++) {
#pragma unroll
    for (int i = 0; i < CAL_CHAINS; i++) c[i] = mfma_32x32x16(a[i & 3], b[(i >> 1) & 3], c[i]);
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < CAL_CHAINS; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) s += c[i][r];
  sink[t] = s;
}

// 16x16x32 fp16 MFMAs (half the output block, twice the depth per instruction): per wave and trip, 2 * CAL_CHAINS
// MFMAs of 16*16*32*2 flop, the same flop per trip as the 32x32x16 loop.
__global__ __launch_bounds__(CAL_WAVES * 64) void calibrate_mfma_f16_16x16x32_kernel(const half8* __restrict__ operands, unsigned mask,
                                                                                     float* __restrict__ sink, int trips) {
  const unsigned t = threadIdx.x + blockIdx.x * blockDim.x;
  half8 a[4], b[4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    a[i] = operands[(t * 8 + i) & mask];
    b[i] = operands[(t * 8 + 4 + i) & mask];
  }
  floatx4 c[2 * CAL_CHAINS];
#pragma unroll
  for (int i = 0; i < 2 * CAL_CHAINS; i++) c[i] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll 1
  for (int it = 0; it < trips; it++) {
#pragma unroll
    for (int i = 0; i < 2 * CAL_CHAINS; i++) c[i] = mfma_16x16x32(a[i & 3], b[(i >> 2) & 3], c[i]);
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 2 * CAL_CHAINS; i++)
#pragma unroll
    for (int r = 0; r < 4; r++) s += c[i][r];
  sink[t] = s;
}

// GEMM-like register loops: 256 accumulators per lane (a 128 x 128 block per wave, as the GEMM kernels hold), eight A
// and eight B operand registers rotated over the trips, and every product subtracted again eight trips later (a negated
// copy of the A operands), so the accumulators wander around zero like the partial sums of a product of zero-mean
// data instead of growing without bound -- the accumulate path sees operands of comparable exponents, as in a real
// GEMM.  WIDE = false: 16 MFMAs 32x32x16 per trip; true: 64 MFMAs 16x16x32 per trip (twice the flop).
template <bool WIDE>
__global__ __launch_bounds__(CAL_WAVES * 64) void calibrate_mfma_f16_walk_kernel(const half8* __restrict__ operands, unsigned mask,
                                                                                 float* __restrict__ sink, int trips) {
  const unsigned t = threadIdx.x + blockIdx.x * blockDim.x;
  half8 a[16], b[8];
#pragma unroll
  for (int i = 0; i < 8; i++) {
    a[i] = operands[(t * 16 + i) & mask];
    a[8 + i] = -a[i];
    b[i] = operands[(t * 16 + 8 + i) & mask];
  }
#pragma unroll
  for (int i = 0; i < 8; i++) asm volatile("" : "+v"(a[8 + i]));  // kept in registers, not recomputed inside the loop
  constexpr int R = WIDE ? 8 : 4;
  typedef typename std::conditional<WIDE, floatx4, floatx16>::type acc_t;
  acc_t c[R][R];
#pragma unroll
  for (int i = 0; i < R; i++)
#pragma unroll
    for (int j = 0; j < R; j++)
#pragma unroll
      for (int r = 0; r < (WIDE ? 4 : 16); r++) c[i][j][r] = 0.f;
#pragma unroll 1
  for (int it = 0; it < trips; it += 16) {
#pragma unroll
    for (int tt = 0; tt < 16; tt++) {
#pragma unroll
      for (int i = 0; i < R; i++)
#pragma unroll
        for (int j = 0; j < R; j++) {
          const half8 av = a[((j + tt) & 7) + (tt >= 8 ? 8 : 0)], bv = b[(i + 3 * tt) & 7];
          if constexpr (WIDE) c[i][j] = mfma_16x16x32(bv, av, c[i][j]);
          else c[i][j] = mfma_32x32x16(bv, av, c[i][j]);
        }
    }
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < R; i++)
#pragma unroll
    for (int j = 0; j < R; j++)
#pragma unroll
      for (int r = 0; r < (WIDE ? 4 : 16); r++) s += c[i][j][r];
  sink[t] = s;
}

// Scaled 32x32x64 MFMAs with fp4 operands (16 bytes per lane; the upper half of the operand registers is unused):
// per wave and trip, CAL_CHAINS MFMAs of 32*32*64*2 flop.  scale_mode 0: every block scale 2^0; 1: E8M0 bytes
// 119..134 derived from the operand bits (exponents spread over [-8, 7] like a block-scaled benchmark's).
__global__ __launch_bounds__(CAL_WAVES * 64) void calibrate_mfma_fp4_kernel(const intx4* __restrict__ operands, unsigned mask,
                                                                            float* __restrict__ sink, int trips, int scale_mode) {
  const unsigned t = threadIdx.x + blockIdx.x * blockDim.x;
  intx8 a[4], b[4];
  int sa[4], sb[4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const intx4 x = operands[(t * 8 + i) & mask], y = operands[(t * 8 + 4 + i) & mask];
    a[i] = intx8{x[0], x[1], x[2], x[3], 0, 0, 0, 0};
    b[i] = intx8{y[0], y[1], y[2], y[3], 0, 0, 0, 0};
    sa[i] = scale_mode ? 119 + ((x[0] >> 3) & 15) : 127;
    sb[i] = scale_mode ? 119 + ((y[1] >> 5) & 15) : 127;
  }
  floatx16 c[CAL_CHAINS];
#pragma unroll
  for (int i = 0; i < CAL_CHAINS; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) c[i][r] = 0.f;
#pragma unroll 1
  for (int it = 0; it < trips; it++) {
#pragma unroll
    for (int i = 0; i < CAL_CHAINS; i++)
      c[i] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[i & 3], b[(i >> 1) & 3], c[i], 4, 4, 0, sa[i & 3], 0, sb[(i >> 1) & 3]);
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < CAL_CHAINS; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) s += c[i][r];
  sink[t] = s;
}

// The GEMM-like loop for the scaled fp4 MFMAs: 256 accumulators, eight A and eight B operand registers (16 bytes of
// codes per lane) with E8M0 scales spread over 2^-8 .. 2^7, rotated over the trips.  fp4 has no exact negation by
// sign flip of a register here (the codes are sign-magnitude nibbles: XOR 0x88888888 flips every sign), so the
// negated A operands are that XOR.  WIDE = false: 16 MFMAs 32x32x64 per trip; true: 64 MFMAs 16x16x128.
template <bool WIDE>
__global__ __launch_bounds__(CAL_WAVES * 64) void calibrate_mfma_fp4_walk_kernel(const intx4* __restrict__ operands, unsigned mask,
                                                                                 float* __restrict__ sink, int trips) {
  const unsigned t = threadIdx.x + blockIdx.x * blockDim.x;
  intx8 a[16], b[8];
  int sa[8], sb[8];
#pragma unroll
  for (int i = 0; i < 8; i++) {
    const intx4 x = operands[(t * 16 + i) & mask], y = operands[(t * 16 + 8 + i) & mask];
    a[i] = intx8{x[0], x[1], x[2], x[3], 0, 0, 0, 0};
    a[8 + i] = intx8{x[0] ^ (int)0x88888888, x[1] ^ (int)0x88888888, x[2] ^ (int)0x88888888, x[3] ^ (int)0x88888888, 0, 0, 0, 0};
    b[i] = intx8{y[0], y[1], y[2], y[3], 0, 0, 0, 0};
    sa[i] = 119 + ((x[0] >> 3) & 15);
    sb[i] = 119 + ((y[1] >> 5) & 15);
  }
#pragma unroll
  for (int i = 0; i < 8; i++) asm volatile("" : "+v"(a[8 + i]));
  constexpr int R = WIDE ? 8 : 4;
  typedef typename std::conditional<WIDE, floatx4, floatx16>::type acc_t;
  acc_t c[R][R];
#pragma unroll
  for (int i = 0; i < R; i++)
#pragma unroll
    for (int j = 0; j < R; j++)
#pragma unroll
      for (int r = 0; r < (WIDE ? 4 : 16); r++) c[i][j][r] = 0.f;
#pragma unroll 1
  for (int it = 0; it < trips; it += 16) {
#pragma unroll
    for (int tt = 0; tt < 16; tt++) {
#pragma unroll
      for (int i = 0; i < R; i++)
#pragma unroll
        for (int j = 0; j < R; j++) {
          const int ai = (j + tt) & 7, bi = (i + 3 * tt) & 7;
          const intx8 av = a[ai + (tt >= 8 ? 8 : 0)], bv = b[bi];
          if constexpr (WIDE) c[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bv, av, c[i][j], 4, 4, 0, sb[bi], 0, sa[ai]);
          else c[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(bv, av, c[i][j], 4, 4, 0, sb[bi], 0, sa[ai]);
        }
    }
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < R; i++)
#pragma unroll
    for (int j = 0; j < R; j++)
#pragma unroll
      for (int r = 0; r < (WIDE ? 4 : 16); r++) s += c[i][j][r];
  sink[t] = s;
}

// The instruction mix of one 64-key tile of the prefill kernel, per wave of 32 queries, out of registers only: 16 score
// MFMAs 32x32x16 (two chains of eight, each starting from one block of addends) with the softmax of the PREVIOUS tile's
// scores placed between them as the prefill kernel pins it -- per MFMA two v_exp_f32, one packed conversion and one
// dot2 -- then 16 MFMAs into four output accumulators that take the packed probabilities as their B operand; before
// them the in-lane v_max3 chain over the 32 scores and its wave-wide test.  No LDS reads, no loads, no barrier: what
// this loop sustains is the ceiling the instruction mix itself sets for the prefill kernel at one (256 workgroups) or
// two (512) waves per SIMD.  MODE 0: the whole mix; 1: without the maximum chain; 2: the MFMAs alone, same
// dependences; 3: the vector work alone.
template <int MODE>
__global__ __launch_bounds__(CAL_WAVES * 64) __attribute__((amdgpu_waves_per_eu(2, 2))) void calibrate_fa_issue_kernel(
    const half8* __restrict__ operands, unsigned mask, float* __restrict__ sink, int trips) {
  constexpr bool MFMAS = MODE != 3, VECTOR = MODE != 2, MAXIMUM = MODE == 0;
  const unsigned t = threadIdx.x + blockIdx.x * blockDim.x;
  half8 kf[4], vf[4], qf[8];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    kf[i] = operands[(t * 16 + i) & mask];
    vf[i] = operands[(t * 16 + 4 + i) & mask];
  }
#pragma unroll
  for (int i = 0; i < 8; i++) qf[i] = operands[(t * 16 + 8 + i) & mask];
  floatx16 oacc[4], negm, sa[2], sb[2];
#pragma unroll
  for (int r = 0; r < 16; r++) {
    negm[r] = -1.f;
#pragma unroll
    for (int i = 0; i < 4; i++) oacc[i][r] = 0.f;
    sa[0][r] = sa[1][r] = sb[0][r] = sb[1][r] = -2.f;
  }
  float l_run = 0.f, grow_thr = 1e30f;
  auto tile = [&](floatx16* s, floatx16* s_next) {
    if constexpr (MAXIMUM) {
      float mx = s[0][0];
#pragma unroll
      for (int tt = 0; tt < 2; tt++)
#pragma unroll
        for (int r = 0; r < 16; r++) mx = fmaxf(mx, s[tt][r]);
      if (__builtin_amdgcn_ballot_w64(mx > grow_thr) != 0) {  // never taken: the threshold is out of reach
#pragma unroll
        for (int r = 0; r < 16; r++) negm[r] -= mx;
      }
    }
    half8 pf[4];
    float psum = 0.f;
    asm volatile("" : "+v"(negm));  // opaque: the score MFMAs are not loop-invariant
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (MFMAS) {
#pragma unroll
      for (int tt = 0; tt < 2; tt++)
#pragma unroll
        for (int ks = 0; ks < 8; ks++) s_next[tt] = mfma_32x32x16(kf[(ks + tt) & 3], qf[ks], ks == 0 ? negm : s_next[tt]);
    }
    if constexpr (VECTOR) {
#pragma unroll
      for (int tt = 0; tt < 2; tt++)
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
          const half2v pp = {(half_t)__builtin_amdgcn_exp2f(s[tt][r]), (half_t)__builtin_amdgcn_exp2f(s[tt][r + 1])};
          psum = __builtin_amdgcn_fdot2(pp, half2v{(half_t)1.f, (half_t)1.f}, psum, false);
          pf[tt * 2 + (r >> 3)][r & 7] = pp[0];
          pf[tt * 2 + (r >> 3)][(r & 7) + 1] = pp[1];
        }
    } else {
      asm volatile("" ::"v"(s[0]), "v"(s[1]));  // the scores count as used
#pragma unroll
      for (int i = 0; i < 4; i++) pf[i] = qf[i];
    }
    if constexpr (MFMAS && VECTOR) {
#pragma unroll
      for (int i = 0; i < 16; i++) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x400, 2, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, 2, 0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    l_run += psum;
    if constexpr (MFMAS) {
#pragma unroll
      for (int i = 0; i < 16; i++) {
        oacc[i & 3] = mfma_32x32x16(vf[(i + (i >> 2)) & 3], pf[i >> 2], oacc[i & 3]);
        __builtin_amdgcn_sched_barrier(0);
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; i++)
#pragma unroll
        for (int e = 0; e < 8; e++) oacc[i][e] += (float)pf[i][e];
    }
    if constexpr (!MFMAS) {  // the next tile's scores: opaque copies, so that their exponentials are computed anew
#pragma unroll
      for (int tt = 0; tt < 2; tt++) {
        s_next[tt] = s[tt];
        asm volatile("" : "+v"(s_next[tt]));
      }
    }
  };
#pragma unroll 1
  for (int it = 0; it < trips; it += 2) {
    tile(sa, sb);
    tile(sb, sa);
  }
  float acc = l_run;
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc += oacc[i][r];
  sink[t] = acc;
}

// The same work per tile with the vector instructions spread over all 32 MFMAs instead of the 16 score MFMAs: one
// exponential behind every score MFMA (the first 32-key half of the tile), two behind each of the first eight output
// MFMAs (the second half; those MFMAs multiply the first half's probabilities), and the maximum chain of the NEXT
// tile's scores behind the last eight.  EXPS_A = exponentials behind each score MFMA (1 or 2: 2 is the order of
// calibrate_fa_issue_kernel written step by step).
template <int EXPS_A>
__global__ __launch_bounds__(CAL_WAVES * 64) __attribute__((amdgpu_waves_per_eu(2, 2))) void calibrate_fa_spread_kernel(
    const half8* __restrict__ operands, unsigned mask, float* __restrict__ sink, int trips) {
  const unsigned t = threadIdx.x + blockIdx.x * blockDim.x;
  half8 kf[4], vf[4], qf[8];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    kf[i] = operands[(t * 16 + i) & mask];
    vf[i] = operands[(t * 16 + 4 + i) & mask];
  }
#pragma unroll
  for (int i = 0; i < 8; i++) qf[i] = operands[(t * 16 + 8 + i) & mask];
  floatx16 oacc[4], negm, sa[2], sb[2];
#pragma unroll
  for (int r = 0; r < 16; r++) {
    negm[r] = -1.f;
#pragma unroll
    for (int i = 0; i < 4; i++) oacc[i][r] = 0.f;
    sa[0][r] = sa[1][r] = sb[0][r] = sb[1][r] = -2.f;
  }
  float l_run = 0.f, grow_thr = 1e30f, mx = -3.f;
  const half2v ones = {(half_t)1.f, (half_t)1.f};
  auto tile = [&](floatx16* s, floatx16* s_next) {
    if (__builtin_amdgcn_ballot_w64(mx > grow_thr) != 0) {  // never taken
#pragma unroll
      for (int r = 0; r < 16; r++) negm[r] -= mx;
    }
    half8 pf[4];
    float psum = 0.f;
    asm volatile("" : "+v"(negm));
    __builtin_amdgcn_sched_barrier(0);
    // exponentials of score pair p (0..15) of the current tile -> pf
    auto softmax_pair = [&](int p) {
      const int tt = p >> 3, r = (p & 7) * 2;
      const half2v pp = {(half_t)__builtin_amdgcn_exp2f(s[tt][r]), (half_t)__builtin_amdgcn_exp2f(s[tt][r + 1])};
      psum = __builtin_amdgcn_fdot2(pp, ones, psum, false);
      pf[tt * 2 + (r >> 3)][r & 7] = pp[0];
      pf[tt * 2 + (r >> 3)][(r & 7) + 1] = pp[1];
    };
    constexpr int PAIRS_A = EXPS_A * 8;  // pairs finished during the score MFMAs
#pragma unroll
    for (int i = 0; i < 16; i++) {
      const int tt = i >> 3, ks = i & 7;
      s_next[tt] = mfma_32x32x16(kf[(ks + tt) & 3], qf[ks], ks == 0 ? negm : s_next[tt]);
      if (EXPS_A == 2) softmax_pair(i);
      else if (i & 1) softmax_pair(i >> 1);
      __builtin_amdgcn_sched_barrier(0);
    }
    float mxn = s_next[0][0];
#pragma unroll
    for (int i = 0; i < 16; i++) {
      oacc[i & 3] = mfma_32x32x16(vf[(i + (i >> 2)) & 3], pf[i >> 2], oacc[i & 3]);
      if (EXPS_A == 1 && i < 8) softmax_pair(PAIRS_A + i);
      if (i >= 8) {
        const int tt = (i - 8) >> 2, r = ((i - 8) & 3) * 4;
        mxn = fmaxf(fmaxf(mxn, s_next[tt][r]), s_next[tt][r + 1]);
        mxn = fmaxf(fmaxf(mxn, s_next[tt][r + 2]), s_next[tt][r + 3]);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    mx = mxn;
    l_run += psum;
  };
#pragma unroll 1
  for (int it = 0; it < trips; it += 2) {
    tile(sa, sb);
    tile(sb, sa);
  }
  float acc = l_run;
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc += oacc[i][r];
  sink[t] = acc;
}

// The same tile with v_mfma_f32_16x16x32_f16 in place of 32x32x16: the same flop, registers and operand bytes per tile --
// 32 score MFMAs (4 key groups x 2 query groups x 4 steps over d; a K fragment serves both query groups) and 32 output
// MFMAs (8 d groups x 2 query groups x 2 steps over the keys) -- with the vector work behind the score MFMAs (one
// exponential each).  VECTOR = false: the MFMAs alone.  Whether the narrower MFMA is cheaper on benchmark-like data
// here as it is in a GEMM's register structure is what this loop answers.
template <bool VECTOR>
__global__ __launch_bounds__(CAL_WAVES * 64) __attribute__((amdgpu_waves_per_eu(2, 2))) void calibrate_fa_issue16_kernel(
    const half8* __restrict__ operands, unsigned mask, float* __restrict__ sink, int trips) {
  const unsigned t = threadIdx.x + blockIdx.x * blockDim.x;
  half8 kf[4], vf[4], qf[8];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    kf[i] = operands[(t * 16 + i) & mask];
    vf[i] = operands[(t * 16 + 4 + i) & mask];
  }
#pragma unroll
  for (int i = 0; i < 8; i++) qf[i] = operands[(t * 16 + 8 + i) & mask];  // [query group][step over d]
  floatx4 oacc[16], negm, sa[8], sb[8];
  negm = floatx4{-1.f, -1.f, -1.f, -1.f};
#pragma unroll
  for (int i = 0; i < 16; i++) oacc[i] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int i = 0; i < 8; i++) sa[i] = sb[i] = floatx4{-2.f, -2.f, -2.f, -2.f};
  float l_run = 0.f;
  const half2v ones = {(half_t)1.f, (half_t)1.f};
  auto tile = [&](floatx4* s, floatx4* s_next) {
    half8 pf[4];  // [query group][key step]: 8 probabilities
    float psum = 0.f;
    asm volatile("" : "+v"(negm));
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < 32; i++) {
      const int kg = i >> 3, ks = (i >> 1) & 3, qg = i & 1;  // a K fragment (kg, ks) feeds both query groups back to back
      s_next[kg * 2 + qg] = mfma_16x16x32(kf[(kg + ks) & 3], qf[qg * 4 + ks], ks == 0 ? negm : s_next[kg * 2 + qg]);
      if constexpr (VECTOR) {
        // one exponential per score MFMA; every second MFMA packs a pair
        const int e = i;  // score e of the tile's 32 per lane: accumulator e / 4, element e % 4
        if (i & 1) {
          const half2v pp = {(half_t)__builtin_amdgcn_exp2f(s[(e - 1) >> 2][(e - 1) & 3]), (half_t)__builtin_amdgcn_exp2f(s[e >> 2][e & 3])};
          psum = __builtin_amdgcn_fdot2(pp, ones, psum, false);
          pf[e >> 3][(e & 7) - 1] = pp[0];
          pf[e >> 3][e & 7] = pp[1];
          asm volatile("" : "+v"(psum));
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (!VECTOR) {
      asm volatile("" ::"v"(s[0]), "v"(s[1]), "v"(s[2]), "v"(s[3]), "v"(s[4]), "v"(s[5]), "v"(s[6]), "v"(s[7]));
#pragma unroll
      for (int i = 0; i < 4; i++) pf[i] = qf[i];
    }
    l_run += psum;
#pragma unroll
    for (int i = 0; i < 32; i++) {
      const int dg = i & 7, qg = (i >> 3) & 1, st = i >> 4;  // V^T fragment (dg, st); accumulators rotate
      oacc[dg * 2 + qg] = mfma_16x16x32(vf[(dg + st) & 3], pf[qg * 2 + st], oacc[dg * 2 + qg]);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
#pragma unroll 1
  for (int it = 0; it < trips; it += 2) {
    tile(sa, sb);
    tile(sb, sa);
  }
  float acc = l_run;
#pragma unroll
  for (int i = 0; i < 16; i++)
#pragma unroll
    for (int r = 0; r < 4; r++) acc += oacc[i][r];
  sink[t] = acc;
}

}  // namespace mi355

using namespace mi355;

// The prefill tile's instruction mix out of registers (calibrate_fa_issue_kernel).  mode 0..3 as documented there;
// 256 workgroups put one wave on every SIMD, 512 two.  flop_per_launch counts the 32 MFMAs of a tile (modes 0..2).
extern "C" int mi355_calibrate_fa_issue(int mode, const void* operands, int64_t operand_bytes, float* sink, int64_t sink_floats,
                                        int64_t workgroups, int64_t trips, double* flop_per_launch, void* stream) {
  if (!operands || !sink) return fail(-MI355_E_NULL, "calibrate_fa_issue: null pointer");
  if (mode < 0 || mode > 7) return fail(-MI355_E_DTYPE, "calibrate_fa_issue: mode %d unknown (0 whole mix, 1 without the maximum chain, 2 MFMAs alone, 3 vector work alone, 4 vector work spread over all 32 MFMAs, 5 the order of mode 0 written step by step, 6 / 7 the tile on 16x16x32 MFMAs: whole mix / MFMAs alone)", mode);
  if (operand_bytes < 16 || (operand_bytes & (operand_bytes - 1)) || operand_bytes > (1ll << 30))
    return fail(-MI355_E_SHAPE, "calibrate_fa_issue: operand_bytes %lld must be a power of two in [16, 2^30]", (long long)operand_bytes);
  if (workgroups <= 0 || workgroups > 65535 || trips <= 0 || trips > (1 << 24))
    return fail(-MI355_E_SHAPE, "calibrate_fa_issue: workgroups %lld / trips %lld out of range", (long long)workgroups, (long long)trips);
  if (sink_floats < workgroups * CAL_WAVES * 64)
    return fail(-MI355_E_SCRATCH, "calibrate_fa_issue: sink needs %lld floats", (long long)(workgroups * CAL_WAVES * 64));
  if (!aligned16(operands)) return fail(-MI355_E_ALIGN, "calibrate_fa_issue: operands must be 16-byte aligned");
  trips = (trips + 1) & ~1ll;
  const unsigned mask = (unsigned)(operand_bytes / 16 - 1);
  dim3 grid((unsigned)workgroups), block(CAL_WAVES * 64);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (flop_per_launch) *flop_per_launch = 32.0 * (2.0 * 32 * 32 * 16) * (double)trips * CAL_WAVES * (double)workgroups;
  switch (mode) {
    case 0: hipLaunchKernelGGL(calibrate_fa_issue_kernel<0>, grid, block, 0, s, (const half8*)operands, mask, sink, (int)trips); break;
    case 1: hipLaunchKernelGGL(calibrate_fa_issue_kernel<1>, grid, block, 0, s, (const half8*)operands, mask, sink, (int)trips); break;
    case 2: hipLaunchKernelGGL(calibrate_fa_issue_kernel<2>, grid, block, 0, s, (const half8*)operands, mask, sink, (int)trips); break;
    case 3: hipLaunchKernelGGL(calibrate_fa_issue_kernel<3>, grid, block, 0, s, (const half8*)operands, mask, sink, (int)trips); break;
    case 4: hipLaunchKernelGGL(calibrate_fa_spread_kernel<1>, grid, block, 0, s, (const half8*)operands, mask, sink, (int)trips); break;
    case 5: hipLaunchKernelGGL(calibrate_fa_spread_kernel<2>, grid, block, 0, s, (const half8*)operands, mask, sink, (int)trips); break;
    case 6: hipLaunchKernelGGL(calibrate_fa_issue16_kernel<true>, grid, block, 0, s, (const half8*)operands, mask, sink, (int)trips); break;
    default: hipLaunchKernelGGL(calibrate_fa_issue16_kernel<false>, grid, block, 0, s, (const half8*)operands, mask, sink, (int)trips); break;
  }
  return check_launch("calibrate_fa_issue", grid, block, 0);
}

// kind 0: fp16 32x32x16; kind 1: fp4 32x32x64 with unit scales; kind 2: fp4 with spread scales; kind 3: fp16 16x16x32;
// kinds 4 / 5: the GEMM-like loops with 32x32x16 / 16x16x32 (trips rounded down to a multiple of 16); kinds 6 / 7: the
// GEMM-like loops with fp4 32x32x64 / 16x16x128.
extern "C" int mi355_calibrate_mfma(int kind, const void* operands, int64_t operand_bytes, float* sink, int64_t sink_floats,
                                    int64_t workgroups, int64_t trips, double* flop_per_launch, void* stream) {
  if (!operands || !sink) return fail(-MI355_E_NULL, "calibrate_mfma: null pointer");
  if (kind < 0 || kind > 7) return fail(-MI355_E_DTYPE, "calibrate_mfma: kind %d unknown (0 fp16 32x32x16, 1 fp4, 2 fp4 with spread scales, 3 fp16 16x16x32, 4 / 5 GEMM-like 32x32x16 / 16x16x32, 6 / 7 GEMM-like fp4 32x32x64 / 16x16x128)", kind);
  if (operand_bytes < 16 || (operand_bytes & (operand_bytes - 1)) || operand_bytes > (1ll << 30))
    return fail(-MI355_E_SHAPE, "calibrate_mfma: operand_bytes %lld must be a power of two in [16, 2^30]", (long long)operand_bytes);
  if (workgroups <= 0 || workgroups > 65535 || trips <= 0 || trips > (1 << 24))
    return fail(-MI355_E_SHAPE, "calibrate_mfma: workgroups %lld / trips %lld out of range", (long long)workgroups, (long long)trips);
  if (sink_floats < workgroups * CAL_WAVES * 64)
    return fail(-MI355_E_SCRATCH, "calibrate_mfma: sink needs %lld floats", (long long)(workgroups * CAL_WAVES * 64));
  if (!aligned16(operands)) return fail(-MI355_E_ALIGN, "calibrate_mfma: operands must be 16-byte aligned");
  const unsigned mask = (unsigned)(operand_bytes / 16 - 1);
  dim3 grid((unsigned)workgroups), block(CAL_WAVES * 64);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const double per_mfma = (kind == 0 || kind == 3) ? 2.0 * 32 * 32 * 16 : 2.0 * 32 * 32 * 64;  // kind 3: per pair of MFMAs
  if (kind >= 4) {
    trips &= ~15ll;
    if (trips <= 0) return fail(-MI355_E_SHAPE, "calibrate_mfma: the GEMM-like loops need trips >= 16");
    if (flop_per_launch) *flop_per_launch = 2.0 * 32 * 32 * 16 * ((kind & 1) ? 32 : 16) * (double)trips * CAL_WAVES * (double)workgroups;
    if (kind >= 6 && flop_per_launch) *flop_per_launch *= 4.0;  // four times the depth per MFMA
    if (kind == 6)
      hipLaunchKernelGGL(calibrate_mfma_fp4_walk_kernel<false>, grid, block, 0, s, (const intx4*)operands, mask, sink, (int)trips);
    else if (kind == 7)
      hipLaunchKernelGGL(calibrate_mfma_fp4_walk_kernel<true>, grid, block, 0, s, (const intx4*)operands, mask, sink, (int)trips);
    else if (kind == 4)
      hipLaunchKernelGGL(calibrate_mfma_f16_walk_kernel<false>, grid, block, 0, s, (const half8*)operands, mask, sink, (int)trips);
    else
      hipLaunchKernelGGL(calibrate_mfma_f16_walk_kernel<true>, grid, block, 0, s, (const half8*)operands, mask, sink, (int)trips);
    return check_launch("calibrate_mfma", grid, block, 0);
  }
  if (flop_per_launch) *flop_per_launch = per_mfma * CAL_CHAINS * (double)trips * CAL_WAVES * (double)workgroups;
  if (kind == 3)
    hipLaunchKernelGGL(calibrate_mfma_f16_16x16x32_kernel, grid, block, 0, s, (const half8*)operands, mask, sink, (int)trips);
  else if (kind == 0)
    hipLaunchKernelGGL(calibrate_mfma_f16_kernel, grid, block, 0, s, (const half8*)operands, mask, sink, (int)trips);
  else
    hipLaunchKernelGGL(calibrate_mfma_fp4_kernel, grid, block, 0, s, (const intx4*)operands, mask, sink, (int)trips, kind == 2);
  return check_launch("calibrate_mfma", grid, block, 0);
}
