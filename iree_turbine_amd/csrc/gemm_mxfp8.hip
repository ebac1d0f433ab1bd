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
//
// The streamed kernel uses v_mfma_scale_f32_16x16x128_f8f6f4 instead, one instruction per 128-element slab row:
// lane (r = l % 16, g = l / 16) supplies bytes 16g..16g+15 and 64+16g..64+16g+15 of row r (measured with
// one-hot operands), and its scale byte is that of block g (k 32g..32g+31) of the slab.
#include <math.h>
#include <type_traits>

#include "common.hpp"
#include "gemm_tiles.hpp"

namespace mi355 {

namespace {

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
  map_tile(blockIdx.x, tiles_m, tiles_n, group_m, tile_m, tile_n);

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
        MxOut<OutT>::store4(crow + i * 32 + q * 8, alpha * acc[i][j][4 * q], alpha * acc[i][j][4 * q + 1], alpha * acc[i][j][4 * q + 2],
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
      if (nn < N) MxOut<OutT>::store1(C + (size_t)m * N + nn, alpha * acc[r]);
    }
  }
}

// Register-staged form: the two-stage direct-to-LDS ring above has only one slab of loads in flight, and a slab's
// 32 MFMAs (about 0.85 us) are shorter than a loaded memory system's round trip, so it runs at the speed of
// the loads.  Here slab s+3 is loaded into VGPRs while slab s computes, slab s+1 is copied from registers into the
// LDS stage that slab s-1 left, and a slab has one barrier, late in its second k-step.  An 8-bit fragment is 8
// registers, so fragments are not double buffered: the four B fragments stay for a k-step and each is re-read
// right behind its last MFMA, the A fragments stream through two registers one row tile ahead.  With 64-cycle
// MFMAs that leaves every read about three MFMAs of latency.  Scales travel as in the staged MXFP4 kernel: a
// lane owns one row and fetches the 8 scale bytes of two slabs, A rows with the even slabs, B rows with the odd
// ones, through four 4 KiB LDS buffers (A / B, group parity) that hold every slab's scale dword twice, plain
// and rotated by 16 bits, so that both lane halves find their two bytes where op_sel looks for them.
// Loads into registers are inline assembly with hand-placed waits, which the compiler cannot see through: the
// kernel must not spill (a register would be stored before its data has arrived; the build checks that).
template <typename OutT, bool SCALED>
__global__ __launch_bounds__(256) void gemm_mxfp8_staged(const uint8_t* __restrict__ A, const uint8_t* __restrict__ As,
                                                         const uint8_t* __restrict__ B, const uint8_t* __restrict__ Bs,
                                                         OutT* __restrict__ C, int M, int N, int K, int tiles_m, int tiles_n,
                                                         int group_m, float alpha) {
  constexpr int BM = 256, BN = 256, WN = 2, NW = 4;
  constexpr int WTM = 128, WTN = 128, TM = 4, TN = 4;
  // LDS, per operand and stage: eight planes, one per 16-byte chunk of the slab's 128-byte rows, each 256 rows x 16
  // bytes plus 32 bytes of padding.  A fragment read is 16 consecutive rows of one plane (conflict free), the
  // chunk a lane wants is a constant plane offset, and the padding spreads the 8 chunks x 2 rows that 16 lanes
  // of a staging write carry over all banks.  Order: A stage 0, A stage 1, B stage 0, B stage 1, so that one
  // address register per operand reaches both stages through the 16-bit instruction offset; then the scale
  // buffers A parity 0, A parity 1, B parity 0, B parity 1, 4 KiB each.
  constexpr int PL = 256 * 16 + 32, OP_BYTES = 8 * PL, B_OFF = 2 * OP_BYTES;
  constexpr int SC_OFF = 17 * 8192;
  static_assert(SC_OFF >= 4 * OP_BYTES && SC_OFF % 8192 == 0, "scale buffers behind the data stages; parity is address bit 12");
  constexpr int NL = SCALED ? 17 : 16;  // loads per slab and lane
  typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
  typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
  typedef int i32x4 __attribute__((ext_vector_type(4)));

  extern __shared__ __attribute__((aligned(1024))) char lds[];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave / WN, wn = wave % WN;
  int tile_m, tile_n;
  map_tile(blockIdx.x, tiles_m, tiles_n, group_m, tile_m, tile_n);

  const unsigned row_bytes = (unsigned)K;
  const unsigned sc_bytes = (unsigned)K >> 5;
  auto make_desc = [&](const uint8_t* base, unsigned bytes) {
    const unsigned long long p = reinterpret_cast<unsigned long long>(base);
    i32x4 d;
    d[0] = __builtin_amdgcn_readfirstlane((int)(unsigned)p);
    d[1] = __builtin_amdgcn_readfirstlane((int)(unsigned)((p >> 32) & 0xFFFFu));
    d[2] = __builtin_amdgcn_readfirstlane((int)bytes);
    d[3] = 0x00020000;
    return d;
  };
  // codes: wave-load i covers rows (i * NW + wave) * 8 .. + 7 of the tile, 8 lanes per 128-byte row piece
  const int lrow = lane >> 3, lc = lane & 7;
  const i32x4 a_src = make_desc(A + (size_t)(tile_m * BM + wave * 8) * row_bytes, (unsigned)(BM - wave * 8) * row_bytes);
  const i32x4 b_src = make_desc(B + (size_t)(tile_n * BN + wave * 8) * row_bytes, (unsigned)(BN - wave * 8) * row_bytes);
  const unsigned g_off = (unsigned)lrow * row_bytes + (unsigned)lc * 16u;
  const unsigned row_step = (unsigned)NW * 8u * row_bytes;
  const int w_off_a = lc * PL + (wave * 8 + lrow) * 16;
  const int w_off_b = w_off_a + B_OFF;
  // scales: lane l of wave w owns row 64 w + l of the tile
  i32x4 as_src = {0, 0, 0, 0}, bs_src = {0, 0, 0, 0};
  if constexpr (SCALED) {
    as_src = make_desc(As + (size_t)(tile_m * BM + wave * 64) * sc_bytes, (unsigned)(BM - wave * 64) * sc_bytes);
    bs_src = make_desc(Bs + (size_t)(tile_n * BN + wave * 64) * sc_bytes, (unsigned)(BN - wave * 64) * sc_bytes);
  }
  const unsigned s_off = (unsigned)lane * sc_bytes;
  int sc_wr = SC_OFF + 4096 + (wave * 64 + lane) * 16;  // where the NEXT group's A scales go (B: + 8192); flips per group

  // staging registers: r[set][n], n < 8 the A row groups, 8..15 the B row groups; rsc[set] the scale row
  u32x4 r[2][16];
  u32x2 rsc[2];
#define MI355_M8_LOAD(S, n, k_off_)                                                                  \
  asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen"                                            \
               : "=v"(r[S][n])                                                                       \
               : "v"(g_off), "s"((n) < 8 ? a_src : b_src), "s"((k_off_) + (unsigned)((n)&7) * row_step) \
               : "memory")
#define MI355_M8_LOAD_SC(S, desc, group_)                                                                                          \
  do {                                                                                                                             \
    if constexpr (SCALED)                                                                                                          \
      asm volatile("buffer_load_dwordx2 %0, %1, %2, %3 offen" : "=v"(rsc[S]) : "v"(s_off), "s"(desc), "s"((unsigned)(group_)*8u) : "memory"); \
  } while (0)
  // `newer` = loads issued after the one that filled the register; they may still be in flight
#define MI355_M8_WRITE(S, n, newer, st_)                                                                                   \
  do {                                                                                                                     \
    asm volatile("s_waitcnt vmcnt(%1)" : "+v"(r[S][n]) : "n"(newer) : "memory");                                           \
    *reinterpret_cast<u32x4*>(lds + ((n) < 8 ? w_off_a : w_off_b) + ((st_)*OP_BYTES + ((n)&7) * NW * 128)) = r[S][n];        \
  } while (0)
#define MI355_M8_WRITE_SC(S, newer, addr_)                                                 \
  do {                                                                                     \
    if constexpr (SCALED) {                                                                \
      asm volatile("s_waitcnt vmcnt(%1)" : "+v"(rsc[S]) : "n"(newer) : "memory");          \
      *reinterpret_cast<u32x4*>(lds + (addr_)) = both_halves(rsc[S]);                      \
    }                                                                                      \
  } while (0)

  // a row's two slab dwords, each followed by itself rotated by 16 bits (what lane half 1 reads)
  auto both_halves = [](u32x2 d) { return u32x4{d[0], (d[0] >> 16) | (d[0] << 16), d[1], (d[1] >> 16) | (d[1] << 16)}; };

  const int r32 = lane & 31, h = lane >> 5;
  // lane half h reads chunks 2 ks + h (its half of block ks) and 4 + 2 ks + h (its half of block 2 + ks)
  const int a_rd = (wm * WTM + r32) * 16 + h * PL;
  const int b_rd = B_OFF + (wn * WTN + r32) * 16 + h * PL;
  // scale dwords of the CURRENT group (parity flips per group); + 8 for the group's second slab.  Lane half h takes
  // the copy whose bytes 0, 1 are blocks 2h, 2h + 1 of the slab: op_sel = ks picks block 2h + ks.
  int sc_rd_a = SC_OFF + (wm * WTM + r32) * 16 + 4 * h;
  int sc_rd_b = SC_OFF + 8192 + (wn * WTN + r32) * 16 + 4 * h;

  floatx16 acc[TN][TM];
#pragma unroll
  for (int i = 0; i < TN; i++)
#pragma unroll
    for (int j = 0; j < TM; j++)
#pragma unroll
      for (int q = 0; q < 16; q++) acc[i][j][q] = 0.f;

  const int KT = K / 128;  // even, >= 4 (checked on the host)
  // B fragments stay for a k-step; A fragments stream through two registers sets, one row tile ahead
  intx8 fa0, fa1, fn[TN];
  int ca[TM], cb[TN];  // one scale dword per row tile: replaced, like the fragments, right after its last use

  // fragment of k-step ks at constant offset `imm` (stage and row tile) from the operand's address register
  auto frag = [&](int at, int ks, int imm) {
    const intx4 lo = *reinterpret_cast<const intx4*>(lds + at + (2 * ks * PL + imm));
    const intx4 hi = *reinterpret_cast<const intx4*>(lds + at + ((4 + 2 * ks) * PL + imm));
    return intx8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  };
  auto scale_dword = [&](int addr) {
    if constexpr (SCALED) return *reinterpret_cast<const int*>(lds + addr);
    else return 0x7f7f7f7f;
  };

#define MI355_M8_LOAD_ALL(S, slab_)                                                                              \
  do {                                                                                                           \
    const unsigned ko_ = (unsigned)(slab_)*128u;                                                                 \
    MI355_M8_LOAD(S, 0, ko_); MI355_M8_LOAD(S, 1, ko_); MI355_M8_LOAD(S, 2, ko_); MI355_M8_LOAD(S, 3, ko_);      \
    MI355_M8_LOAD(S, 4, ko_); MI355_M8_LOAD(S, 5, ko_); MI355_M8_LOAD(S, 6, ko_); MI355_M8_LOAD(S, 7, ko_);      \
    MI355_M8_LOAD(S, 8, ko_); MI355_M8_LOAD(S, 9, ko_); MI355_M8_LOAD(S, 10, ko_); MI355_M8_LOAD(S, 11, ko_);    \
    MI355_M8_LOAD(S, 12, ko_); MI355_M8_LOAD(S, 13, ko_); MI355_M8_LOAD(S, 14, ko_); MI355_M8_LOAD(S, 15, ko_);  \
  } while (0)
  // prologue: slab 0 (+ A scales of group 0) -> set 0 -> stage 0; B scales of group 0 through a spare
  // register; slab 1 (+ B scales of group 1) -> set 1; then slab 2 (+ A scales of group 1) -> set 0
  const int KG = KT / 2;  // scale groups
  u32x2 rs;
  MI355_M8_LOAD_ALL(0, 0);
  MI355_M8_LOAD_SC(0, as_src, 0);
  if constexpr (SCALED) asm volatile("buffer_load_dwordx2 %0, %1, %2, 0 offen" : "=v"(rs) : "v"(s_off), "s"(bs_src) : "memory");
  MI355_M8_LOAD_ALL(1, 1);
  MI355_M8_LOAD_SC(1, bs_src, KG > 1 ? 1 : 0);
  // everything older than set 1's loads has landed once at most NL are outstanding
  MI355_M8_WRITE(0, 0, NL, 0); MI355_M8_WRITE(0, 1, NL, 0); MI355_M8_WRITE(0, 2, NL, 0); MI355_M8_WRITE(0, 3, NL, 0);
  MI355_M8_WRITE(0, 4, NL, 0); MI355_M8_WRITE(0, 5, NL, 0); MI355_M8_WRITE(0, 6, NL, 0); MI355_M8_WRITE(0, 7, NL, 0);
  MI355_M8_WRITE(0, 8, NL, 0); MI355_M8_WRITE(0, 9, NL, 0); MI355_M8_WRITE(0, 10, NL, 0); MI355_M8_WRITE(0, 11, NL, 0);
  MI355_M8_WRITE(0, 12, NL, 0); MI355_M8_WRITE(0, 13, NL, 0); MI355_M8_WRITE(0, 14, NL, 0); MI355_M8_WRITE(0, 15, NL, 0);
  MI355_M8_WRITE_SC(0, NL, sc_wr - 4096);
  if constexpr (SCALED) {
    asm volatile("s_waitcnt vmcnt(%1)" : "+v"(rs) : "n"(NL) : "memory");
    *reinterpret_cast<u32x4*>(lds + sc_wr - 4096 + 8192) = both_halves(rs);
  }
  MI355_M8_LOAD_ALL(0, 2);
  MI355_M8_LOAD_SC(0, as_src, KG > 1 ? 1 : 0);
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __syncthreads();
  fa0 = frag(a_rd, 0, 0);
#pragma unroll
  for (int j = 0; j < TM; j++) {
    fn[j] = frag(b_rd, 0, j * 512);
    ca[j] = scale_dword(sc_rd_a + j * 512);
    cb[j] = scale_dword(sc_rd_b + j * 512);
  }

  // Four MFMAs of A row tile j (fragment FA) against the four B fragments; X0..X3 are what follows each of them:
  // one or two memory instructions, or the re-read of the B fragment just used.
#define MI355_M8_GROUP(KS, j, FA, X0, X1, X2, X3)                                      \
  do {                                                                                 \
    acc[0][j] = mfma_fp8_32x32x64<KS>(fn[0], cb[0], FA, ca[j], acc[0][j]);             \
    X0;                                                                                \
    __builtin_amdgcn_sched_barrier(0);                                                 \
    acc[1][j] = mfma_fp8_32x32x64<KS>(fn[1], cb[1], FA, ca[j], acc[1][j]);             \
    X1;                                                                                \
    __builtin_amdgcn_sched_barrier(0);                                                 \
    acc[2][j] = mfma_fp8_32x32x64<KS>(fn[2], cb[2], FA, ca[j], acc[2][j]);             \
    X2;                                                                                \
    __builtin_amdgcn_sched_barrier(0);                                                 \
    acc[3][j] = mfma_fp8_32x32x64<KS>(fn[3], cb[3], FA, ca[j], acc[3][j]);             \
    X3;                                                                                \
    __builtin_amdgcn_sched_barrier(0);                                                 \
  } while (0)
#define MI355_NOP ((void)0)

  // Slab kt (scales in ca/cb) sits in stage P; set Q = 1 - P holds slab kt+1 and the scale row SCD travels with
  // (written to SCW); each register is reloaded with slab kt+3 (the scale row with group GN) soon after it is
  // written or later in the slab.  In flight when register n is written: the rest of its own round (NL - 1 - n),
  // the NL loads of the other set and the loads of this slab issued so far.
  // The one barrier of the slab stands behind the last read of stage P and before the first read of stage Q, in
  // the last group of k-step 1; the MFMAs around it cover the latency of the reads on both sides.
  // HALF = 8 if slab kt+1 is the second slab of its group.
#define MI355_M8_W(Q, n, issued) MI355_M8_WRITE(Q, n, 2 * NL - 1 - (n) + (issued), Q)
#define MI355_M8_SLAB(P, Q, kt_, SCD, SCW, GN, HALF)                                                                       \
  do {                                                                                                                     \
    constexpr int st = P * OP_BYTES, nst = Q * OP_BYTES;                                                                   \
    const int nxt_ = (kt_) + 3 < KT ? (kt_) + 3 : KT - 1; /* past the end: re-fetch, never used */                         \
    const unsigned ko = (unsigned)nxt_ * 128u;                                                                             \
    const int gn_ = (GN) < KG ? (GN) : KG - 1;                                                                             \
    __builtin_amdgcn_sched_barrier(0);                                                                                     \
    MI355_M8_GROUP(0, 0, fa0, MI355_M8_W(Q, 0, 0); MI355_M8_W(Q, 1, 0), MI355_M8_W(Q, 2, 0); fa1 = frag(a_rd, 0, st + 512),      \
                   MI355_M8_W(Q, 3, 0); MI355_M8_W(Q, 4, 0), MI355_M8_W(Q, 5, 0); MI355_M8_LOAD(Q, 0, ko));                 \
    MI355_M8_GROUP(0, 1, fa1, MI355_M8_W(Q, 6, 1); MI355_M8_W(Q, 7, 1), MI355_M8_W(Q, 8, 1); fa0 = frag(a_rd, 0, st + 2 * 512),  \
                   MI355_M8_W(Q, 9, 1); MI355_M8_W(Q, 10, 1), MI355_M8_W(Q, 11, 1); MI355_M8_LOAD(Q, 1, ko));               \
    MI355_M8_GROUP(0, 2, fa0, MI355_M8_W(Q, 12, 2); MI355_M8_W(Q, 13, 2), MI355_M8_W(Q, 14, 2); fa1 = frag(a_rd, 0, st + 3 * 512), \
                   MI355_M8_W(Q, 15, 2); MI355_M8_WRITE_SC(Q, NL + 2, SCW), MI355_M8_LOAD(Q, 2, ko));                      \
    MI355_M8_GROUP(0, 3, fa1, fn[0] = frag(b_rd, 1, st); fa0 = frag(a_rd, 1, st),                                          \
                   MI355_M8_LOAD(Q, 3, ko); fn[1] = frag(b_rd, 1, st + 512), fn[2] = frag(b_rd, 1, st + 2 * 512),          \
                   fn[3] = frag(b_rd, 1, st + 3 * 512));                                                                   \
    MI355_M8_GROUP(1, 0, fa0, MI355_M8_LOAD(Q, 4, ko), fa1 = frag(a_rd, 1, st + 512), MI355_M8_LOAD(Q, 5, ko),             \
                   MI355_M8_LOAD(Q, 6, ko));                                                                               \
    MI355_M8_GROUP(1, 1, fa1, MI355_M8_LOAD(Q, 7, ko), fa0 = frag(a_rd, 1, st + 2 * 512), MI355_M8_LOAD(Q, 8, ko),         \
                   MI355_M8_LOAD(Q, 9, ko));                                                                               \
    MI355_M8_GROUP(1, 2, fa0, MI355_M8_LOAD(Q, 10, ko), fa1 = frag(a_rd, 1, st + 3 * 512), MI355_M8_LOAD(Q, 11, ko),       \
                   MI355_M8_LOAD(Q, 12, ko));                                                                              \
    if (HALF == 0) { sc_rd_a ^= 4096; sc_rd_b ^= 4096; }                                                                   \
    /* the slab's one barrier: behind the last read of stage P, before the first read of stage Q and of new scales */    \
    MI355_M8_GROUP(1, 3, fa1,                                                                                              \
                   asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); __builtin_amdgcn_s_barrier();                       \
                   fa0 = frag(a_rd, 0, nst); fn[0] = frag(b_rd, 0, nst); cb[0] = scale_dword(sc_rd_b + HALF);              \
                   ca[0] = scale_dword(sc_rd_a + HALF),                                                                    \
                   MI355_M8_LOAD(Q, 13, ko); fn[1] = frag(b_rd, 0, nst + 512); cb[1] = scale_dword(sc_rd_b + HALF + 512);  \
                   ca[1] = scale_dword(sc_rd_a + HALF + 512),                                                              \
                   MI355_M8_LOAD(Q, 14, ko); fn[2] = frag(b_rd, 0, nst + 2 * 512); cb[2] = scale_dword(sc_rd_b + HALF + 1024); \
                   ca[2] = scale_dword(sc_rd_a + HALF + 1024),                                                             \
                   MI355_M8_LOAD(Q, 15, ko); MI355_M8_LOAD_SC(Q, SCD, gn_); fn[3] = frag(b_rd, 0, nst + 3 * 512);          \
                   cb[3] = scale_dword(sc_rd_b + HALF + 1536); ca[3] = scale_dword(sc_rd_a + HALF + 1536));                \
  } while (0)

  for (int kt = 0; kt < KT; kt += 2) {
    const int g0 = kt >> 1;
    // even slab: set 1 carries slab kt+1 and the B scales of group g0+1; reloaded with slab kt+3 and the B scales of g0+2
    MI355_M8_SLAB(0, 1, kt, bs_src, sc_wr + 8192, g0 + 2, 8);
    // odd slab: set 0 carries slab kt+2 and the A scales of group g0+1; reloaded with slab kt+4 and the A scales of g0+2
    MI355_M8_SLAB(1, 0, kt + 1, as_src, sc_wr, g0 + 2, 0);
    sc_wr ^= 4096;
    // The loads of the last slabs fetch nothing that is used, and behind the loop the compiler hands their
    // registers to the epilogue: let them land while the registers still belong to them.
    // The wait names every staging register as an input, so that the registers stay allocated to the loads up to it
    // however the compiler restructures the last iteration.
    if (kt + 2 >= KT) {
      asm volatile("s_waitcnt vmcnt(0)" ::"v"(r[0][0]), "v"(r[0][1]), "v"(r[0][2]), "v"(r[0][3]), "v"(r[0][4]), "v"(r[0][5]), "v"(r[0][6]), "v"(r[0][7]), "v"(r[0][8]), "v"(r[0][9]), "v"(r[0][10]), "v"(r[0][11]), "v"(r[0][12]), "v"(r[0][13]), "v"(r[0][14]), "v"(r[0][15]) : "memory");
      asm volatile("" ::"v"(r[1][0]), "v"(r[1][1]), "v"(r[1][2]), "v"(r[1][3]), "v"(r[1][4]), "v"(r[1][5]), "v"(r[1][6]), "v"(r[1][7]), "v"(r[1][8]), "v"(r[1][9]), "v"(r[1][10]), "v"(r[1][11]), "v"(r[1][12]), "v"(r[1][13]), "v"(r[1][14]), "v"(r[1][15]) : "memory");
    }
  }
#undef MI355_M8_SLAB
#undef MI355_M8_W
#undef MI355_M8_GROUP
#undef MI355_NOP
#undef MI355_M8_LOAD_ALL
#undef MI355_M8_WRITE_SC
#undef MI355_M8_WRITE
#undef MI355_M8_LOAD_SC
#undef MI355_M8_LOAD
  // drain the speculative loads; every wave is past its last fragment read before the epilogue reuses LDS
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
  __syncthreads();

  if constexpr (sizeof(OutT) == 2) {
    // bf16 epilogue through LDS, one wave-private region each, 32 rows per pass: ds_write_b64 of 4 consecutive n
    // (chunk slot c ^ ((m >> 1) & 7)), whole 256-byte rows read back 16 bytes per lane
    constexpr int ROW_B = WTN * 2, CH = WTN / 8;
    char* ep = lds + wave * (32 * ROW_B);
    constexpr int ROWS_PER_IT = 64 / CH;
    const int er = lane / CH, ec = lane % CH;
#pragma unroll
    for (int j = 0; j < TM; j++) {
#pragma unroll
      for (int i = 0; i < TN; i++)
#pragma unroll
        for (int q = 0; q < 4; q++) {
          const int c = i * 4 + q;
          ushortx4 v = {f32_to_bf16_rne(alpha * acc[i][j][4 * q]), f32_to_bf16_rne(alpha * acc[i][j][4 * q + 1]),
                        f32_to_bf16_rne(alpha * acc[i][j][4 * q + 2]), f32_to_bf16_rne(alpha * acc[i][j][4 * q + 3])};
          *reinterpret_cast<ushortx4*>(ep + r32 * ROW_B + ((c ^ ((r32 >> 1) & 7)) * 16) + 8 * h) = v;
        }
      OutT* cbase = C + (size_t)(tile_m * BM + wm * WTM + j * 32) * N + tile_n * BN + wn * WTN + ec * 8;
#pragma unroll
      for (int it = 0; it < 32 / ROWS_PER_IT; it++) {
        const int row = it * ROWS_PER_IT + er;
        const u32x4 v = *reinterpret_cast<const u32x4*>(ep + row * ROW_B + ((ec ^ ((row >> 1) & 7)) * 16));
        *reinterpret_cast<u32x4*>(cbase + (size_t)row * N) = v;
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  } else {
    const int m0 = tile_m * BM + wm * WTM + r32;
    const int n0 = tile_n * BN + wn * WTN + 4 * h;
#pragma unroll
    for (int j = 0; j < TM; j++) {
      OutT* crow = C + (size_t)(m0 + j * 32) * N + n0;
#pragma unroll
      for (int i = 0; i < TN; i++)
#pragma unroll
        for (int q = 0; q < 4; q++)
          MxOut<OutT>::store4(crow + i * 32 + q * 8, alpha * acc[i][j][4 * q], alpha * acc[i][j][4 * q + 1], alpha * acc[i][j][4 * q + 2],
                             alpha * acc[i][j][4 * q + 3]);
    }
  }
}

// Streamed form (see gemm_f16_nt_stream and gemm_mxfp4_stream for the reasoning; the LDS map, the load schedule and the
// tile walk are those of the MXFP4 kernel).  A slab row is 128 bytes = 128 codes = 4 scale blocks = one k step of the
// 16x16x128 MFMA: lane l supplies row l & 15 and the 16-byte chunks (l >> 4) and 4 + (l >> 4) of the row as one
// 32-byte operand, and its scale byte is that of block l >> 4 of the slab.  The B fragments of a slab are held in
// registers (read from LDS during the first two steps of the slab before), the A rows are streamed one 16-row
// fragment per step, two steps ahead; a step is 8 MFMAs (one A fragment against the 8 B fragments).
// LDS (160 KiB): B in a ring of five 16 KiB half buffers (U = rows 0..63, V = rows 64..127 of both 128-row halves), A
// in two 32 KiB buffers freed block by block, 16 KiB for the scales.
// Scales are staged through LDS in groups of four slabs: 16 bytes per row, one lane per row, 8 KiB per group (A rows,
// then B rows), two buffers; a group is loaded in the first two steps of every fourth slab, three slabs before its
// first read.  A lane fetches a scale with a one-byte LDS read (bits 0..7 of a register, as the MFMA wants it): the A
// scale of a step next to its fragment, the 8 B scales of the next slab in steps 2..5.
// One step = 8 MFMAs + LDS reads + two data loads; a barrier every 2 steps (an interval):
//   interval q of slab t loads   A: block q - 1 of slab t + 2 (q = 0: block 3 of slab t + 1)
//                                B: part q of slab t + 3 (parts 0, 1 -> its U half, parts 2, 3 -> its V half)
// At a barrier every wave has waited for its loads older than the newest 15 and for its LDS reads older than the interval.
// SCALED = false: every scale is 2^0 (no scale traffic) and the result is multiplied by alpha.
template <typename OutT, bool SCALED>
__global__ __launch_bounds__(256) void gemm_mxfp8_stream(const uint8_t* __restrict__ A, const uint8_t* __restrict__ As,
                                                         const uint8_t* __restrict__ B, const uint8_t* __restrict__ Bs,
                                                         OutT* __restrict__ C, int M, int N, int K, int tiles_m, int tiles_n,
                                                         int group_m, float alpha) {
  typedef _Float16 half8 __attribute__((ext_vector_type(8)));  // 16 opaque bytes
  constexpr int BM = 256, BN = 256, WN = 2, WTM = 128, WTN = 128;
  constexpr int HALF = 128 * 128, ABUF = 256 * 128, SGRP = 8192;
  constexpr int B_AT = 0, A_AT = 5 * HALF, S_AT = A_AT + 2 * ABUF;
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave / WN, wn = wave % WN;
  const int T = tiles_m * tiles_n, G = (int)gridDim.x;
  int pid = blockIdx.x;
  int tile_m, tile_n;
  map_tile(pid, tiles_m, tiles_n, group_m, tile_m, tile_n);

  // One descriptor per array (each under 4 GiB, checked on the host); tile, slab and row block go into the scalar offset.
  const unsigned row_bytes = (unsigned)K, SK = (unsigned)K / 32u;
  const buffer_rsrc_t a_src = make_buffer(A, (unsigned)(tiles_m * BM) * row_bytes);
  const buffer_rsrc_t b_src = make_buffer(B, (unsigned)(tiles_n * BN) * row_bytes);
  const buffer_rsrc_t sa_src = make_buffer(SCALED ? As : A, (unsigned)(tiles_m * BM) * SK);
  const buffer_rsrc_t sb_src = make_buffer(SCALED ? Bs : B, (unsigned)(tiles_n * BN) * SK);
  const int lrow = lane >> 3;
  // codes: a wave-load covers 8 rows x 128 bytes; lane = (row l >> 3, slot l & 7) fetches chunk slot ^ ((row >> 1) & 7)
  const unsigned g_off = (unsigned)(wave * 8 + lrow) * row_bytes + (unsigned)((lane & 7) ^ (((wave & 1) << 2) | (lrow >> 1))) * 16u;
  // scales: a wave-load covers rows 64 w .. 64 w + 63 of the tile, 16 bytes (four slabs) per lane
  const unsigned gs_off = (unsigned)(wave * 64 + lane) * SK;
  const int KT = K / 128;  // a multiple of 4, >= 8 (checked on the host)
  unsigned a_cur = (unsigned)(tile_m * BM) * row_bytes, b_cur = (unsigned)(tile_n * BN) * row_bytes;
  unsigned a_nxt = a_cur, b_nxt = b_cur;  // the next tile (after the last: itself again; those loads are never used)
  unsigned sa_cur = (unsigned)(tile_m * BM) * SK, sb_cur = (unsigned)(tile_n * BN) * SK, sa_nxt = sa_cur, sb_nxt = sb_cur;
  auto slab_at = [&](int s, unsigned cur, unsigned nxt) { return s < KT ? cur + (unsigned)s * 128u : nxt + (unsigned)(s - KT) * 128u; };
  auto grp_at = [&](int s, unsigned cur, unsigned nxt) { return s < KT ? cur + (unsigned)s * 4u : nxt + (unsigned)(s - KT) * 4u; };
  // offsets of the slabs 1, 2 (A) and 3 (B) ahead and of the scale group after this one; those of the next slab are
  // worked out one per step in the second half of a slab
  unsigned a_off1 = a_cur + 128u, a_off2 = a_cur + 256u, b_off3 = b_cur + 384u, sa_off = sa_cur + 16u, sb_off = sb_cur + 16u;
  unsigned n_a1 = 0, n_a2 = 0, n_b3 = 0, n_sa = 0, n_sb = 0;
  auto load_a = [&](int buf, int h, int blk, unsigned at) {
    buffer_load_lds_16B(a_src, g_off, (unsigned)(h * 128 + blk * 32) * row_bytes + at,
                        lds + A_AT + buf * ABUF + (h * 16 + blk * 4 + wave) * 1024);
  };
  // part p (rows 32 p .. 32 p + 31 of either 128-row half) into the half buffer at byte offset half_at
  auto load_b = [&](int half_at, int h, int part, unsigned at) {
    buffer_load_lds_16B(b_src, g_off, (unsigned)(h * 128 + part * 32) * row_bytes + at,
                        lds + B_AT + half_at + (h * 8 + (part & 1) * 4 + wave) * 1024);
  };
  auto load_scales = [&](bool is_b, int grp_at_lds, unsigned at) {
    buffer_load_lds_16B(is_b ? sb_src : sa_src, gs_off, at, lds + S_AT + grp_at_lds + (is_b ? 4096 : 0) + wave * 1024);
  };

  // fragment reads: lane l takes row l & 15 of a 16-row block, chunks (l >> 4) and 4 + (l >> 4) of the 128-byte row
  const int r16 = lane & 15, cq = lane >> 4;
  const unsigned lds0 = (unsigned)(uintptr_t)MI355_LDS(char, lds);
  const unsigned lane_rd = (unsigned)(r16 * 128 + ((cq ^ (r16 >> 1)) & 7) * 16);  // upper chunk: ^ 64
  unsigned aaddr[2][2];  // [A buffer][lower / upper chunk]
#pragma unroll
  for (int bf = 0; bf < 2; bf++)
#pragma unroll
    for (int kh = 0; kh < 2; kh++) aaddr[bf][kh] = lds0 + A_AT + bf * ABUF + wm * (WTM * 128) + (lane_rd ^ (kh * 64));
  const unsigned b_lane = lds0 + B_AT + wn * (64 * 128) + lane_rd;  // 64 rows of either half per half buffer
  unsigned bU[2], bV[2];  // [lower / upper chunk]: the U and V half buffers read in this slab
  // scale reads: the byte of row (16 rb + r16), slab s, block cq sits at row * 16 + 4 (s & 3) + cq of the slab's group
  const unsigned sa_lane = lds0 + S_AT + (unsigned)((wm * WTM + r16) * 16 + cq);
  const unsigned sb_lane = lds0 + S_AT + 4096 + (unsigned)((wn * WTN + r16) * 16 + cq);
  unsigned sa_rd = sa_lane, sa_rdn = sa_lane + 4, sb_rdn = sb_lane + 4;  // this slab's A scales, the next slab's A and B

  // [n block][m block].  Never cleared: the MFMAs of a tile's first slab take a zero addend instead -- a register write
  // in front of an inline-assembly MFMA would need wait states the compiler does not know to insert.
  floatx4 acc[8][8];
  intx4 fbl0[8], fbh0[8], fbl1[8], fbh1[8];  // B fragments as read (lower, upper chunk) for the two slab parities
  intx8 fb0[8], fb1[8];                       // ... as MFMA operands
  intx4 fal[4], fah[4];                       // A fragments by step
  int sb0[8], sb1[8], sat[4];                 // B scales of the two slab parities; A scales by step
  if constexpr (!SCALED) {
#pragma unroll
    for (int i = 0; i < 8; i++) sb0[i] = sb1[i] = 127;
#pragma unroll
    for (int i = 0; i < 4; i++) sat[i] = 127;
  }

#define MI355_S8_CAT(lo, hi) __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7)
  // MFMAs as inline assembly with the accumulators pinned to AGPRs.  No MFMA here reads an accumulator written fewer
  // than 64 MFMAs earlier.  x, sx: B codes and scale (bits 0..7); y, sy: A codes and scale.
#define MI355_S8_ACC(ZERO, c, x, sx, y, sy)                                                               \
  do {                                                                                                    \
    if constexpr (ZERO)                                                                                   \
      asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, 0, %3, %4 op_sel_hi:[0,0,0]"            \
                   : "=a"(c) : "v"(x), "v"(y), "v"(sx), "v"(sy));                                         \
    else                                                                                                  \
      asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel_hi:[0,0,0]"           \
                   : "+a"(c) : "v"(x), "v"(y), "v"(sx), "v"(sy));                                         \
  } while (0)
  // The first MFMA of a step together with the wait for the step's A fragment and scale (requested two steps earlier;
  // LG = LDS reads issued since).  One statement, with the registers as plain inputs: a separate wait statement that
  // names them as outputs makes the compiler put a wait state in front of their next use.
#define MI355_S8_ACCW(ZERO, LG, c, x, sx, y, sy)                                                                         \
  do {                                                                                                                   \
    if constexpr (ZERO)                                                                                                  \
      asm volatile("s_waitcnt lgkmcnt(%5)\n\tv_mfma_scale_f32_16x16x128_f8f6f4 %0, %3, %1, 0, %4, %2 op_sel_hi:[0,0,0]"   \
                   : "=a"(c) : "v"(y), "v"(sy), "v"(x), "v"(sx), "n"(LG));                                               \
    else                                                                                                                 \
      asm volatile("s_waitcnt lgkmcnt(%5)\n\tv_mfma_scale_f32_16x16x128_f8f6f4 %0, %3, %1, %0, %4, %2 op_sel_hi:[0,0,0]"  \
                   : "+a"(c) : "v"(y), "v"(sy), "v"(x), "v"(sx), "n"(LG));                                               \
  } while (0)
#define MI355_S8_READ(dst, addr, off) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(off))
#define MI355_S8_READ8(dst, addr, off) asm volatile("ds_read_u8 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(off))
#define MI355_S8_TIE8(X) "+v"(X[0]), "+v"(X[1]), "+v"(X[2]), "+v"(X[3]), "+v"(X[4]), "+v"(X[5]), "+v"(X[6]), "+v"(X[7])
#define MI355_S8_TIE4(X) "+v"(X[0]), "+v"(X[1]), "+v"(X[2]), "+v"(X[3])

  // ---- prologue: B0 (half buffers 0, 1), A0, B1 (2, 3), A1 blocks 0..2, scale group 0 ----
#pragma unroll
  for (int x = 0; x < 8; x++) load_b((x >> 2) * HALF, x & 1, x >> 1, b_cur);
#pragma unroll
  for (int x = 0; x < 8; x++) load_a(0, x & 1, x >> 1, a_cur);
#pragma unroll
  for (int x = 0; x < 8; x++) load_b((2 + (x >> 2)) * HALF, x & 1, x >> 1, b_cur + 128u);
#pragma unroll
  for (int x = 0; x < 6; x++) load_a(1, x & 1, x >> 1, a_cur + 128u);
  if constexpr (SCALED) {
    load_scales(false, 0, sa_cur);
    load_scales(true, 0, sb_cur);
  }
  __builtin_amdgcn_sched_barrier(0);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_sched_barrier(0);
  bU[0] = b_lane; bU[1] = b_lane ^ 64;
  bV[0] = b_lane + HALF; bV[1] = bV[0] ^ 64;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    MI355_S8_READ(fbl0[i], bU[0], i * 2048); MI355_S8_READ(fbh0[i], bU[1], i * 2048);
    MI355_S8_READ(fbl0[4 + i], bV[0], i * 2048); MI355_S8_READ(fbh0[4 + i], bV[1], i * 2048);
  }
  MI355_S8_READ(fal[0], aaddr[0][0], 0); MI355_S8_READ(fah[0], aaddr[0][1], 0);
  MI355_S8_READ(fal[1], aaddr[0][0], 2048); MI355_S8_READ(fah[1], aaddr[0][1], 2048);
  asm volatile("s_waitcnt lgkmcnt(0)"
               : MI355_S8_TIE8(fbl0), MI355_S8_TIE8(fbh0), "+v"(fal[0]), "+v"(fah[0]), "+v"(fal[1]), "+v"(fah[1]));
  if constexpr (SCALED) {
#pragma unroll
    for (int i = 0; i < 8; i++) MI355_S8_READ8(sb0[i], sb_lane, i * 256);
    MI355_S8_READ8(sat[0], sa_lane, 0); MI355_S8_READ8(sat[1], sa_lane, 256);
    asm volatile("s_waitcnt lgkmcnt(0)" : MI355_S8_TIE8(sb0), "+v"(sat[0]), "+v"(sat[1]));
  }
#pragma unroll
  for (int i = 0; i < 8; i++) fb0[i] = MI355_S8_CAT(fbl0[i], fbh0[i]);
  __builtin_amdgcn_s_barrier();  // every wave has read B0: its half buffers may receive slab 2's V half (0) and slab 3's U half (1)
  __builtin_amdgcn_sched_barrier(0);
  // B2: U half -> half buffer 4, V half -> half buffer 0
#pragma unroll
  for (int x = 0; x < 8; x++) load_b(((4 + (x >> 2)) % 5) * HALF, x & 1, x >> 1, b_cur + 256u);
  __builtin_amdgcn_sched_barrier(0);

  // B ring: slab t's halves live in half buffers (2 t) % 5 and (2 t + 1) % 5; pos = (2 t) % 5 for the current slab t
  int pos = 0;
  int sg_ld = SGRP;  // LDS offset of the scale group buffer the next group goes to (groups alternate)

  // Step j of slab phase PH (slab index mod 4; A buffer PH & 1): the MFMAs of m block j on fal/fah[j % 4], sat[j % 4]
  // against FB / SB[0..7].  LGKM = LDS reads issued after those of step j - 2 (which filled this step's fragment).
#define MI355_S8_STEP(j, PH, FB, FBNL, FBNH, SB, SBN, LGKM, FIRST)                                                      \
  do {                                                                                                                 \
    constexpr int PAR = (PH)&1, j2 = (j) + 2, nb = j2 >= 8 ? 1 - PAR : PAR, nj = j2 & 7;                                \
    const intx8 ya = MI355_S8_CAT(fal[(j)&3], fah[(j)&3]);                                                             \
    MI355_S8_ACCW(FIRST, LGKM, acc[0][j], FB[0], SB[0], ya, sat[(j)&3]);                                               \
    MI355_S8_READ(fal[j2 & 3], aaddr[nb][0], nj * 2048);                                                               \
    MI355_S8_READ(fah[j2 & 3], aaddr[nb][1], nj * 2048);                                                               \
    __builtin_amdgcn_sched_barrier(0);                                                                                 \
    MI355_S8_ACC(FIRST, acc[1][j], FB[1], SB[1], ya, sat[(j)&3]);                                                      \
    if constexpr (SCALED) {                                                                                            \
      if constexpr (j2 >= 8) MI355_S8_READ8(sat[j2 & 3], sa_rdn, nj * 256);                                            \
      else MI355_S8_READ8(sat[j2 & 3], sa_rd, nj * 256);                                                               \
    }                                                                                                                  \
    __builtin_amdgcn_sched_barrier(0);                                                                                 \
    MI355_S8_ACC(FIRST, acc[2][j], FB[2], SB[2], ya, sat[(j)&3]);                                                      \
    if constexpr ((j) < 2) {                                                                                           \
      MI355_S8_READ(FBNL[4 * (j)], ((j) ? bV : bU)[0], 0 * 2048);                                                      \
      MI355_S8_READ(FBNH[4 * (j)], ((j) ? bV : bU)[1], 0 * 2048);                                                      \
      MI355_S8_READ(FBNL[4 * (j) + 1], ((j) ? bV : bU)[0], 1 * 2048);                                                  \
      MI355_S8_READ(FBNH[4 * (j) + 1], ((j) ? bV : bU)[1], 1 * 2048);                                                  \
    } else if constexpr (SCALED && (j) < 6) {                                                                          \
      MI355_S8_READ8(SBN[2 * ((j)-2)], sb_rdn, (2 * ((j)-2)) * 256);                                                   \
    }                                                                                                                  \
    __builtin_amdgcn_sched_barrier(0);                                                                                 \
    MI355_S8_ACC(FIRST, acc[3][j], FB[3], SB[3], ya, sat[(j)&3]);                                                      \
    if constexpr ((j) < 2) {                                                                                           \
      MI355_S8_READ(FBNL[4 * (j) + 2], ((j) ? bV : bU)[0], 2 * 2048);                                                  \
      MI355_S8_READ(FBNH[4 * (j) + 2], ((j) ? bV : bU)[1], 2 * 2048);                                                  \
      MI355_S8_READ(FBNL[4 * (j) + 3], ((j) ? bV : bU)[0], 3 * 2048);                                                  \
      MI355_S8_READ(FBNH[4 * (j) + 3], ((j) ? bV : bU)[1], 3 * 2048);                                                  \
    } else if constexpr (SCALED && (j) < 6) {                                                                          \
      MI355_S8_READ8(SBN[2 * ((j)-2) + 1], sb_rdn, (2 * ((j)-2) + 1) * 256);                                           \
    }                                                                                                                  \
    __builtin_amdgcn_sched_barrier(0);                                                                                 \
    MI355_S8_ACC(FIRST, acc[4][j], FB[4], SB[4], ya, sat[(j)&3]);                                                      \
    {                                                                                                                  \
      constexpr int q = (j) >> 1;                                                                                      \
      /* the scale group after this one: A rows in step 0, B rows in step 1 of every fourth slab */                   \
      if constexpr (SCALED && (PH) == 0 && (j) == 0) load_scales(false, sg_ld, sa_off);                                \
      if constexpr (SCALED && (PH) == 0 && (j) == 1) load_scales(true, sg_ld, sb_off);                                 \
      if constexpr (((j)&1) == 0) {                                                                                    \
        if constexpr (q == 0) load_a(1 - PAR, 0, 3, a_off1);                                                           \
        else load_a(PAR, 0, q - 1, a_off2);                                                                            \
      } else {                                                                                                         \
        load_b(q < 2 ? ld_u : ld_v, 0, q, b_off3);                                                                     \
      }                                                                                                                \
    }                                                                                                                  \
    __builtin_amdgcn_sched_barrier(0);                                                                                 \
    MI355_S8_ACC(FIRST, acc[5][j], FB[5], SB[5], ya, sat[(j)&3]);                                                      \
    {                                                                                                                  \
      constexpr int q = (j) >> 1;                                                                                      \
      if constexpr (((j)&1) == 0) {                                                                                    \
        if constexpr (q == 0) load_a(1 - PAR, 1, 3, a_off1);                                                           \
        else load_a(PAR, 1, q - 1, a_off2);                                                                            \
      } else {                                                                                                         \
        load_b(q < 2 ? ld_u : ld_v, 1, q, b_off3);                                                                     \
      }                                                                                                                \
    }                                                                                                                  \
    __builtin_amdgcn_sched_barrier(0);                                                                                 \
    if constexpr ((j) == 3) n_a1 = slab_at(kt + 2, a_cur, a_nxt);                                                      \
    if constexpr ((j) == 4) n_a2 = slab_at(kt + 3, a_cur, a_nxt);                                                      \
    if constexpr ((j) == 5) n_b3 = slab_at(kt + 4, b_cur, b_nxt);                                                      \
    if constexpr (SCALED && (PH) == 3 && (j) == 6) n_sa = grp_at(kt + 5, sa_cur, sa_nxt);                              \
    if constexpr (SCALED && (PH) == 3 && (j) == 7) n_sb = grp_at(kt + 5, sb_cur, sb_nxt);                              \
    MI355_S8_ACC(FIRST, acc[6][j], FB[6], SB[6], ya, sat[(j)&3]);                                                      \
    MI355_S8_ACC(FIRST, acc[7][j], FB[7], SB[7], ya, sat[(j)&3]);                                                      \
    __builtin_amdgcn_sched_barrier(0);                                                                                 \
  } while (0)
  // End of an interval: loads older than the newest VMC and LDS reads older than the interval are complete in every wave.
#define MI355_S8_SYNC(RD, VMC)                                                      \
  do {                                                                              \
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(%1)" ::"n"(VMC), "n"(RD) : "memory"); \
    __builtin_amdgcn_s_barrier();                                                   \
    __builtin_amdgcn_sched_barrier(0);                                              \
  } while (0)
  // LDS reads per step: A fragment (2) and scale (1) + 8 for four B fragments in steps 0, 1 or 2 B scales in steps 2..5.
  constexpr int RA = SCALED ? 3 : 2, RB = SCALED ? 2 : 0;
#define MI355_S8_SLAB(PH, FB, FBNL, FBNH, FBN, SB, SBN, FIRST, VMC)                                              \
  do {                                                                                                          \
    {                                                                                                           \
      const int pu = pos + 2 >= 5 ? pos - 3 : pos + 2, pv = pos + 3 >= 5 ? pos - 2 : pos + 3; /* slab t + 1 */   \
      bU[0] = b_lane + (unsigned)(pu * HALF);                                                                   \
      bU[1] = bU[0] ^ 64;                                                                                       \
      bV[0] = b_lane + (unsigned)(pv * HALF);                                                                   \
      bV[1] = bV[0] ^ 64;                                                                                       \
    }                                                                                                           \
    /* slab t + 3: U half -> (2 t + 6) % 5 = pos + 1, V half -> (2 t + 7) % 5 = pos + 2 */                       \
    const int ld_u = (pos + 1 >= 5 ? pos - 4 : pos + 1) * HALF, ld_v = (pos + 2 >= 5 ? pos - 3 : pos + 2) * HALF; \
    MI355_S8_STEP(0, PH, FB, FBNL, FBNH, SB, SBN, RA, FIRST);                                                   \
    MI355_S8_STEP(1, PH, FB, FBNL, FBNH, SB, SBN, RA + 8, FIRST);                                               \
    MI355_S8_SYNC(15, VMC);                                                                                     \
    MI355_S8_STEP(2, PH, FB, FBNL, FBNH, SB, SBN, RA + 8, FIRST);                                               \
    MI355_S8_STEP(3, PH, FB, FBNL, FBNH, SB, SBN, RA + RB, FIRST);                                              \
    MI355_S8_SYNC(2 * (RA + RB), VMC);                                                                          \
    MI355_S8_STEP(4, PH, FB, FBNL, FBNH, SB, SBN, RA + RB, FIRST);                                              \
    MI355_S8_STEP(5, PH, FB, FBNL, FBNH, SB, SBN, RA + RB, FIRST);                                              \
    MI355_S8_SYNC(2 * (RA + RB), VMC);                                                                          \
    MI355_S8_STEP(6, PH, FB, FBNL, FBNH, SB, SBN, RA + RB, FIRST);                                              \
    MI355_S8_STEP(7, PH, FB, FBNL, FBNH, SB, SBN, RA, FIRST);                                                   \
    /* the next slab's B fragments and scales were requested in steps 0..5: they have landed; tie them here */  \
    asm volatile("s_waitcnt vmcnt(%24) lgkmcnt(%25)"                                                            \
                 : MI355_S8_TIE8(FBNL), MI355_S8_TIE8(FBNH), MI355_S8_TIE8(SBN)                                 \
                 : "n"(VMC), "n"(2 * RA) : "memory");                                                           \
    _Pragma("unroll") for (int i_ = 0; i_ < 8; i_++) FBN[i_] = MI355_S8_CAT(FBNL[i_], FBNH[i_]);                \
    __builtin_amdgcn_s_barrier();                                                                               \
    __builtin_amdgcn_sched_barrier(0);                                                                          \
    a_off1 = n_a1;                                                                                              \
    a_off2 = n_a2;                                                                                              \
    b_off3 = n_b3;                                                                                              \
    pos = pos + 2 >= 5 ? pos - 3 : pos + 2;                                                                     \
    /* the scale reads of the slabs after this one: 4 bytes on per slab; slab 4 g starts group g's buffer */    \
    sa_rd = sa_rdn;                                                                                             \
    if constexpr ((PH) == 2) {                                                                                  \
      sa_rdn = sa_lane + (unsigned)sg_ld;                                                                       \
      sb_rdn = sb_lane + (unsigned)sg_ld;                                                                       \
    } else {                                                                                                    \
      sa_rdn = sa_rdn + 4;                                                                                      \
      sb_rdn = sb_rdn + 4;                                                                                      \
    }                                                                                                           \
    if constexpr ((PH) == 3) {                                                                                  \
      sg_ld ^= SGRP;                                                                                            \
      sa_off = n_sa;                                                                                            \
      sb_off = n_sb;                                                                                            \
    }                                                                                                           \
  } while (0)

  for (; pid < T; pid += G) {
    int nxt_m = tile_m, nxt_n = tile_n;
    if (pid + G < T) map_tile(pid + G, tiles_m, tiles_n, group_m, nxt_m, nxt_n);
    a_nxt = (unsigned)(nxt_m * BM) * row_bytes;
    b_nxt = (unsigned)(nxt_n * BN) * row_bytes;
    sa_nxt = (unsigned)(nxt_m * BM) * SK;
    sb_nxt = (unsigned)(nxt_n * BN) * SK;
    // In a tile's first slab the 32 stores of the epilogue before it sit in the queue behind the loads the waits are
    // about (a 32-bit epilogue, 64 stores, drains the queue instead).
    constexpr int VMC_FIRST = sizeof(OutT) == 2 ? 15 + 32 : 15;
    int kt = 0;
    MI355_S8_SLAB(0, fb0, fbl1, fbh1, fb1, sb0, sb1, true, VMC_FIRST);
    kt = 1;
    MI355_S8_SLAB(1, fb1, fbl0, fbh0, fb0, sb1, sb0, false, 15);
    kt = 2;
    MI355_S8_SLAB(2, fb0, fbl1, fbh1, fb1, sb0, sb1, false, 15);
    kt = 3;
    MI355_S8_SLAB(3, fb1, fbl0, fbh0, fb0, sb1, sb0, false, 15);
    for (kt = 4; kt < KT; kt += 4) {
      MI355_S8_SLAB(0, fb0, fbl1, fbh1, fb1, sb0, sb1, false, 15);
      kt++;
      MI355_S8_SLAB(1, fb1, fbl0, fbh0, fb0, sb1, sb0, false, 15);
      kt++;
      MI355_S8_SLAB(2, fb0, fbl1, fbh1, fb1, sb0, sb1, false, 15);
      kt++;
      MI355_S8_SLAB(3, fb1, fbl0, fbh0, fb0, sb1, sb0, false, 15);
      kt -= 3;
    }
    // ---- epilogue ---- (gemm_tiles.hpp).  16-bit results are staged through LDS in a wave-private 2 KiB region while
    // the next tile's slabs are landing; free at this point is block 3 of A buffer 1 (rows 96..127 of either half: twice
    // 4 KiB), which the next loads reach only after the barrier below.
    mx_stream_epilogue<true>(acc, alpha, C + (size_t)(tile_m * BM + wm * WTM) * N + tile_n * BN + wn * WTN, N,
                              lds0 + (unsigned)(A_AT + ABUF + (wave < 2 ? 12 * 1024 + wave * 2048 : 28 * 1024 + (wave - 2) * 2048)));
    a_cur = a_nxt;
    b_cur = b_nxt;
    sa_cur = sa_nxt;
    sb_cur = sb_nxt;
    tile_m = nxt_m;
    tile_n = nxt_n;
    // the waves leave the epilogue together: the next loads reach the LDS the other waves' epilogues use
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
  }
  // the loads issued for a tile that does not exist still target LDS: let them land before the workgroup ends
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" : MI355_S8_TIE4(fal), MI355_S8_TIE4(fah), MI355_S8_TIE4(sat));
#undef MI355_S8_SLAB
#undef MI355_S8_SYNC
#undef MI355_S8_STEP
#undef MI355_S8_TIE4
#undef MI355_S8_TIE8
#undef MI355_S8_READ8
#undef MI355_S8_READ
#undef MI355_S8_ACCW
#undef MI355_S8_ACC
#undef MI355_S8_CAT
}

static const char* kMx8Variants[] = {"tiled_256x256x128_w2x2", "generic_32x128", "staged_256x256x128_w2x2",
                                     "stream_256x256x128_w2x2", "stream_256x256x128_w2x2_walk"};
constexpr int kNumMx8Variants = 5;
int mxfp8_variant_count() { return kNumMx8Variants; }
const char* mxfp8_variant_name(int i) { return (i >= 0 && i < kNumMx8Variants) ? kMx8Variants[i] : nullptr; }

static int mx8_cu_count() {
  static int cached[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (cached[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cached[dev] = n;
  }
  return cached[dev];
}

template <typename OutT, bool SCALED>
static int launch_mx8(int variant, const void* a, const void* as, const void* b, const void* bs, void* c, int M, int N, int K,
                      float alpha, hipStream_t stream) {
  if (variant == 0) {
    auto kern = gemm_mxfp8_tiled<256, 256, 2, 2, OutT, SCALED>;
    constexpr int lds_bytes = 2 * 512 * 128;
    static std::atomic<uint64_t> lds_ok{0};
    if (int rc = allow_lds(reinterpret_cast<const void*>(kern), lds_bytes, lds_ok, "gemm_mxfp8_tiled")) return rc;
    const int tiles_m = M / 256, tiles_n = N / 256;
    dim3 grid(tiles_m * tiles_n), block(256);
    hipLaunchKernelGGL(kern, grid, block, lds_bytes, stream, (const uint8_t*)a, (const uint8_t*)as, (const uint8_t*)b,
                       (const uint8_t*)bs, (OutT*)c, M, N, K, tiles_m, tiles_n, 4, alpha);
    return check_launch("gemm_mxfp8_tiled", grid, block, lds_bytes);
  }
  if (variant == 2) {
    auto kern = gemm_mxfp8_staged<OutT, SCALED>;
    constexpr int lds_bytes = 17 * 8192 + 4 * 4096;  // two padded stages per operand, four scale buffers
    static std::atomic<uint64_t> lds_ok{0};
    if (int rc = allow_lds(reinterpret_cast<const void*>(kern), lds_bytes, lds_ok, "gemm_mxfp8_staged")) return rc;
    const int tiles_m = M / 256, tiles_n = N / 256;
    dim3 grid(tiles_m * tiles_n), block(256);
    hipLaunchKernelGGL(kern, grid, block, lds_bytes, stream, (const uint8_t*)a, (const uint8_t*)as, (const uint8_t*)b,
                       (const uint8_t*)bs, (OutT*)c, M, N, K, tiles_m, tiles_n, 4, alpha);
    return check_launch("gemm_mxfp8_staged", grid, block, lds_bytes);
  }
  if (variant == 3 || variant == 4) {
    auto kern = gemm_mxfp8_stream<OutT, SCALED>;
    constexpr int lds_bytes = 5 * 16384 + 2 * 32768 + 16384;  // five B half buffers, two A buffers, two scale groups
    static std::atomic<uint64_t> lds_ok{0};
    if (int rc = allow_lds(reinterpret_cast<const void*>(kern), lds_bytes, lds_ok, "gemm_mxfp8_stream")) return rc;
    const int tiles_m = M / 256, tiles_n = N / 256;
    int wgs = tiles_m * tiles_n;
    if (variant == 4) {  // one workgroup per CU walks its tiles
      int g = mx8_cu_count() & ~7;  // multiples of 8 keep a workgroup's tiles on the XCD it runs on
      if (g < 8) g = 8;
      if (wgs > g) wgs = g;
    }
    dim3 grid(wgs), block(256);
    hipLaunchKernelGGL(kern, grid, block, lds_bytes, stream, (const uint8_t*)a, (const uint8_t*)as, (const uint8_t*)b,
                       (const uint8_t*)bs, (OutT*)c, M, N, K, tiles_m, tiles_n, 4, alpha);
    return check_launch("gemm_mxfp8_stream", grid, block, lds_bytes);
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
  if (variant >= kNumMx8Variants) return fail(-MI355_E_DTYPE, "mxfp8_gemm: variant %d out of range", variant);
  if (!aligned16(a) || !aligned16(b) || !aligned16(c)) return fail(-MI355_E_ALIGN, "mxfp8_gemm: a, b, c must be 16-byte aligned");
  const bool sc_al4 = ((reinterpret_cast<uintptr_t>(a_scale) | reinterpret_cast<uintptr_t>(b_scale)) & 3u) == 0;
  const bool fits0 = sc_al4 && M % 256 == 0 && N % 256 == 0 && K % 256 == 0 && K >= 256;  // slabs in pairs, one scale dword per slab
  const bool fits2 = fits0 && K >= 512 && K <= (1 << 23);  // four slabs in flight; 32-bit buffer offsets
  // streamed: scale groups of four slabs (16-byte loads), the look-ahead stays within the next tile, one descriptor per array
  const bool sc_al16 = ((reinterpret_cast<uintptr_t>(a_scale) | reinterpret_cast<uintptr_t>(b_scale)) & 15u) == 0;
  const bool fits3 = sc_al16 && M % 256 == 0 && N % 256 == 0 && K % 512 == 0 && K >= 1024 && M * K < (int64_t(1) << 32) &&
                     N * K < (int64_t(1) << 32);
  // streamed, one workgroup per CU walking its tiles: 4096x8192x8192 200 us against 233 for the staged kernel
  if (variant < 0) variant = fits3 ? 4 : fits2 ? 2 : fits0 ? 0 : 1;
  else if ((variant == 3 || variant == 4) && !fits3)
    return fail(-MI355_E_SHAPE,
                "mxfp8_gemm: variant %s needs M%%256==0, N%%256==0, K%%512==0, K >= 1024, 16-byte aligned scales and a, b under 4 GiB",
                kMx8Variants[variant]);
  else if (variant == 0 && !fits0)
    return fail(-MI355_E_SHAPE, "mxfp8_gemm: variant %s needs M%%256==0, N%%256==0, K%%256==0 and 4-byte aligned scales", kMx8Variants[0]);
  else if (variant == 2 && !fits2)
    return fail(-MI355_E_SHAPE, "mxfp8_gemm: variant %s needs M%%256==0, N%%256==0, K%%256==0, 512 <= K <= 2^23 and 4-byte aligned scales",
                kMx8Variants[2]);
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
  if (variant >= kNumMx8Variants) return fail(-MI355_E_DTYPE, "fp8_gemm: variant %d out of range", variant);
  if (!isfinite(alpha)) return fail(-MI355_E_SHAPE, "fp8_gemm: alpha must be finite");
  if (!aligned16(a) || !aligned16(b) || !aligned16(c)) return fail(-MI355_E_ALIGN, "fp8_gemm: a, b, c must be 16-byte aligned");
  const bool fits0 = M % 256 == 0 && N % 256 == 0 && K % 256 == 0 && K >= 256;
  const bool fits2 = fits0 && K >= 512 && K <= (1 << 23);
  const bool fits3 = M % 256 == 0 && N % 256 == 0 && K % 512 == 0 && K >= 1024 && M * K < (int64_t(1) << 32) && N * K < (int64_t(1) << 32);
  // streamed, one workgroup per CU walking its tiles: 4096x8192x8192 200 us against 233 for the staged kernel
  if (variant < 0) variant = fits3 ? 4 : fits2 ? 2 : fits0 ? 0 : 1;
  else if ((variant == 3 || variant == 4) && !fits3)
    return fail(-MI355_E_SHAPE, "fp8_gemm: variant %s needs M%%256==0, N%%256==0, K%%512==0, K >= 1024 and a, b under 4 GiB",
                kMx8Variants[variant]);
  else if (variant == 0 && !fits0)
    return fail(-MI355_E_SHAPE, "fp8_gemm: variant %s needs M%%256==0, N%%256==0, K%%256==0", kMx8Variants[0]);
  else if (variant == 2 && !fits2)
    return fail(-MI355_E_SHAPE, "fp8_gemm: variant %s needs M%%256==0, N%%256==0, K%%256==0 and 512 <= K <= 2^23", kMx8Variants[2]);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (out_dtype == MI355_F32) return launch_mx8<float, false>(variant, a, nullptr, b, nullptr, c, (int)M, (int)N, (int)K, alpha, s);
  return launch_mx8<unsigned short, false>(variant, a, nullptr, b, nullptr, c, (int)M, (int)N, (int)K, alpha, s);
}
