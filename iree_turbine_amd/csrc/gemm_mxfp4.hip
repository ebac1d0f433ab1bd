// Block-scaled MXFP4 GEMM for gfx950:  C[M,N] = dq(A) . dq(B)^T, bf16 (or fp32) output.
//
// Codes are two E2M1 values per byte (even k in the low nibble), one E8M0 scale byte per 32
// consecutive k.  The arithmetic is v_mfma_scale_f32_32x32x64_f8f6f4 with both operands in
// fp4 format: the instruction takes the raw codes plus one scale byte per lane and per
// operand and applies 2^(scale-127) in hardware, so nothing is dequantised in software.
//
// Tiling is the fp16 GEMM's with k measured in bytes: a K slab is 256 fp4 values = 128 bytes
// per row = 8 chunks of 16 bytes (one chunk = one 32-element scale block), copied with
// direct-to-LDS loads into a two-stage ring with the same XOR swizzle and the same rotated,
// software-pipelined k-loop.
//
// A lane's 16-byte fragment is exactly one scale block.  Which two blocks of a slab form a 64-wide
// k-step is free as long as A and B agree, so k-step ks (0..3) pairs block ks (lanes 0..31) with
// block 4+ks (lanes 32..63): a lane then needs bytes ks = 0..3 of ONE dword per row and slab
// (dword h = lane / 32 of the row's 8 scale bytes), fetched one slab ahead, and the op_sel field
// of the MFMA picks the byte: no shifts or permutes in the loop.
#include <type_traits>

#include "common.hpp"
#include "gemm_tiles.hpp"

namespace mi355 {

// byte SEL of sa / sb scales the lane's block of a / b
template <int SEL>
__device__ __forceinline__ floatx16 mfma_fp4_32x32x64(intx4 a, int sa, intx4 b, int sb, floatx16 c) {
  intx8 av = {a[0], a[1], a[2], a[3], 0, 0, 0, 0};
  intx8 bv = {b[0], b[1], b[2], b[3], 0, 0, 0, 0};
  return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(av, bv, c, 4, 4, SEL, sa, SEL, sb);
}

// SCALES_LDS: scale bytes travel through LDS in groups of 4 slabs (32 bytes per row, two buffers behind
// the data stages) instead of one strided 8-byte global load per lane, row tile and slab.  Needs
// K % 1024 == 0.
// SLAB (with SCALES_LDS): the slab form of gemm_f16_nt_pipelined -- four data stages, the fragments and scale dwords
// of a whole slab in one of two register sets, one wait per trip in front of its barrier -- for launches in which a
// workgroup has its CU to itself: its slab time in the k-step form is its load latency.
// RAGGED_M (slab form): M is any number of rows; the loads of A's codes and scales take row min(row, M - 1), the
// epilogue stores the rows below M.
template <int BM, int BN, int WM, int WN, typename OutT, bool SCALES_LDS, bool SLAB = false, bool RAGGED_M = false>
__global__ __launch_bounds__(WM* WN * 64) void gemm_mxfp4_tiled(const uint8_t* __restrict__ A, const uint8_t* __restrict__ As,
                                                                const uint8_t* __restrict__ B, const uint8_t* __restrict__ Bs,
                                                                OutT* __restrict__ C, int M, int N, int K, int tiles_m,
                                                                int tiles_n, int group_m) {
  constexpr int NW = WM * WN;
  constexpr int WTM = BM / WM, WTN = BN / WN;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int A_BYTES = BM * 128, B_BYTES = BN * 128, STAGE = A_BYTES + B_BYTES;
  constexpr int A_GROUPS = BM / 8, B_GROUPS = BN / 8;
  static_assert(A_GROUPS % NW == 0 && B_GROUPS % NW == 0 && NW % 2 == 0, "loads must split evenly over an even number of waves");
  constexpr int LA = A_GROUPS / NW, LB = B_GROUPS / NW;

  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave / WN, wn = wave % WN;
  int tile_m, tile_n;
  map_tile(blockIdx.x, tiles_m, tiles_n, group_m, tile_m, tile_n);

  const int Kb = K >> 1;   // bytes per row of codes
  const int Ksc = K >> 5;  // scale bytes per row
  const int lrow = lane >> 3;
  // chunk c of row r lives in slot c ^ ((r >> 1) & 7): conflict-free fragment reads on 64 LDS banks
  const int lchunk = (lane & 7) ^ (((wave & 1) << 2) | (lrow >> 1));
  // wave-uniform base pointer + one 32-bit per-lane offset shared by every load of the wave
  const uint8_t* a_src = A + (size_t)(tile_m * BM + (RAGGED_M ? 0 : wave * 8)) * Kb;  // RAGGED_M: the tile's first row
  const uint8_t* b_src = B + (size_t)(tile_n * BN + wave * 8) * Kb;
  const unsigned lane_off = (unsigned)lrow * (unsigned)Kb + (unsigned)lchunk * 16u;
  const size_t row_step = (size_t)NW * 8 * Kb;
  static_assert(!RAGGED_M || SLAB, "only the slab form cuts its last tile row");
  // RAGGED_M: byte offset from the tile's first row of A (which exists) of this lane's clamped row in A load i
  unsigned a_off[RAGGED_M ? LA : 1];
  if constexpr (RAGGED_M) {
#pragma unroll
    for (int i = 0; i < LA; i++) {
      const int row = tile_m * BM + wave * 8 + i * NW * 8 + lrow;
      a_off[i] = (unsigned)((row < M ? row : M - 1) - tile_m * BM) * (unsigned)Kb + (unsigned)lchunk * 16u;  // from the tile's first row
    }
  }

  auto issue_loads = [&](int stage, int slab) {
    char* dst = lds + stage * STAGE + wave * 1024;
    const uint8_t* ap = a_src + slab * 128;
    const uint8_t* bp = b_src + slab * 128;
#pragma unroll
    for (int i = 0; i < LA; i++) {
      if constexpr (RAGGED_M) load_lds_16B(ap + a_off[i], dst + i * NW * 1024);
      else load_lds_16B(ap + i * row_step + lane_off, dst + i * NW * 1024);
    }
#pragma unroll
    for (int i = 0; i < LB; i++) load_lds_16B(bp + i * row_step + lane_off, dst + A_BYTES + i * NW * 1024);
  };

  const int r32 = lane & 31, h = lane >> 5;
  const int sw = ((4 * h) ^ ((r32 >> 1) & 7)) * 16;  // chunk ks + 4h of the row, swizzled
  const int a_base = (wm * WTM + r32) * 128 + sw;
  const int b_base = A_BYTES + (wn * WTN + r32) * 128 + sw;

  // scale dwords: bytes 4h..4h+3 of the row's 8 scale bytes of a slab, fetched one slab ahead into the
  // register set the slab after next will not touch
  const uint8_t* as_src = As + (size_t)(tile_m * BM + wm * WTM + r32) * Ksc + 4 * h;
  const uint8_t* bs_src = Bs + (size_t)(tile_n * BN + wn * WTN + r32) * Ksc + 4 * h;
  int sa[2][TM], sb[2][TN];
  // LDS scale buffers: [buffer][A rows then B rows][32 bytes = 4 slabs x 8 blocks]
  constexpr int SC_BUF = (BM + BN) * 32;
  constexpr int STAGES = SLAB ? 4 : 2;
  static_assert(!SLAB || SCALES_LDS, "the slab form stages its scales through LDS");
  char* sc_lds = lds + STAGES * STAGE;
  static_assert(((BM + BN) / 32) % NW == 0, "scale rows must split evenly over waves");
  constexpr int LS = (BM + BN) / 32 / NW;  // wave-loads (32 rows x 32 bytes) per wave per group
  const unsigned sc_lane_off = (unsigned)(lane >> 1) * (unsigned)Ksc + (unsigned)(lane & 1) * 16u;
  auto issue_scale_loads = [&](int group) {
    char* dst = sc_lds + (group & 1) * SC_BUF;
#pragma unroll
    for (int i = 0; i < LS; i++) {
      const int r0 = (wave * LS + i) * 32;  // first of 32 consecutive rows (all in A or all in B: BM % 32 == 0)
      const uint8_t* src = r0 < BM ? As + (size_t)(tile_m * BM + r0) * Ksc : Bs + (size_t)(tile_n * BN + r0 - BM) * Ksc;
      if constexpr (RAGGED_M) {
        const int row = tile_m * BM + r0 + (lane >> 1);
        if (r0 < BM) src = As + (size_t)(row < M ? row : M - 1) * Ksc - (size_t)(lane >> 1) * Ksc;  // this lane's row, clamped
      }
      load_lds_16B(src + group * 32 + sc_lane_off, dst + r0 * 32);
    }
  };
  const int sa_off = (wm * WTM + r32) * 32 + 4 * h, sb_off = (BM + wn * WTN + r32) * 32 + 4 * h;
  auto fetch_scales = [&](int* da, int* db, int slab) {
    if constexpr (SCALES_LDS) {
      const char* buf = sc_lds + ((slab >> 2) & 1) * SC_BUF + (slab & 3) * 8;
#pragma unroll
      for (int j = 0; j < TM; j++) da[j] = *reinterpret_cast<const int*>(buf + sa_off + j * 1024);
#pragma unroll
      for (int i = 0; i < TN; i++) db[i] = *reinterpret_cast<const int*>(buf + sb_off + i * 1024);
    } else {
#pragma unroll
      for (int j = 0; j < TM; j++) da[j] = *reinterpret_cast<const int*>(as_src + (size_t)j * 32 * Ksc + slab * 8);
#pragma unroll
      for (int i = 0; i < TN; i++) db[i] = *reinterpret_cast<const int*>(bs_src + (size_t)i * 32 * Ksc + slab * 8);
    }
  };

  auto read_frags = [&](const char* st, int ks, intx4* fm, intx4* fn) {
#pragma unroll
    for (int j = 0; j < TM; j++) fm[j] = *reinterpret_cast<const intx4*>(st + ((a_base ^ (ks * 16)) + j * 4096));
#pragma unroll
    for (int i = 0; i < TN; i++) fn[i] = *reinterpret_cast<const intx4*>(st + ((b_base ^ (ks * 16)) + i * 4096));
  };

  floatx16 acc[TN][TM];
#pragma unroll
  for (int i = 0; i < TN; i++)
#pragma unroll
    for (int j = 0; j < TM; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

  auto mfmas = [&](auto ks_tag, const intx4* fm, const intx4* fn, const int* ca, const int* cb) __attribute__((always_inline)) {
    constexpr int KS = decltype(ks_tag)::value;
#pragma unroll
    for (int i = 0; i < TN; i++)
#pragma unroll
      for (int j = 0; j < TM; j++) acc[i][j] = mfma_fp4_32x32x64<KS>(fn[i], cb[i], fm[j], ca[j], acc[i][j]);
  };
  auto interleave = [&]() {
#pragma unroll
    for (int i = 0; i < TM + TN; i++) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // 1 MFMA
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // 1 DS read
    }
    __builtin_amdgcn_sched_group_barrier(0x008, TM * TN - (TM + TN), 0);
  };

  const int KT = K / 256;
  const int KG = (KT + 3) >> 2;  // scale groups
  using K0 = std::integral_constant<int, 0>;
  using K1 = std::integral_constant<int, 1>;
  using K2 = std::integral_constant<int, 2>;
  using K3 = std::integral_constant<int, 3>;
  if constexpr (SLAB) {
    // Trip kt: MFMAs of slab kt from the current register set | fragment and scale reads of slab kt+1 into the other
    // set | loads of slab kt+4 into the stage slab kt left (every wave read it a trip ago) and, on every fourth trip,
    // of scale group kt/4 + 1 (its buffer's last reader was trip kt-2).  The wait in front of the barrier leaves the
    // loads of the two newest trips in flight, so a load has three trips to land.
    constexpr int NL = LA + LB, NM = 4 * TM * TN, NR = 5 * (TM + TN);
    constexpr bool PINNED = NM > 4;  // a trip of four MFMAs is too short to spread anything over
    intx4 am[2][4][TM], an[2][4][TN];
    auto read_at = [&](const char* st, const char* scb, int r, intx4(*fm)[TM], intx4(*fn)[TN], int* da, int* db) __attribute__((always_inline)) {
      // read r of a trip: first the scale dwords, then the fragments k-step by k-step
      if (r < TM) da[r] = *reinterpret_cast<const int*>(scb + sa_off + r * 1024);
      else if (r < TM + TN) db[r - TM] = *reinterpret_cast<const int*>(scb + sb_off + (r - TM) * 1024);
      else {
        const int q = r - (TM + TN), rk = q / (TM + TN), f = q % (TM + TN);
        if (f < TM) fm[rk][f] = *reinterpret_cast<const intx4*>(st + ((a_base ^ (rk * 16)) + f * 4096));
        else fn[rk][f - TM] = *reinterpret_cast<const intx4*>(st + ((b_base ^ (rk * 16)) + (f - TM) * 4096));
      }
    };
    auto mfma_at = [&](int m, const intx4(*fm)[TM], const intx4(*fn)[TN], const int* ca, const int* cb) __attribute__((always_inline)) {
      const int ks = m / (TM * TN), i = (m / TM) % TN, j = m % TM;
      if (ks == 0) acc[i][j] = mfma_fp4_32x32x64<0>(fn[0][i], cb[i], fm[0][j], ca[j], acc[i][j]);
      else if (ks == 1) acc[i][j] = mfma_fp4_32x32x64<1>(fn[1][i], cb[i], fm[1][j], ca[j], acc[i][j]);
      else if (ks == 2) acc[i][j] = mfma_fp4_32x32x64<2>(fn[2][i], cb[i], fm[2][j], ca[j], acc[i][j]);
      else acc[i][j] = mfma_fp4_32x32x64<3>(fn[3][i], cb[i], fm[3][j], ca[j], acc[i][j]);
    };
    auto trip = [&](auto kk_tag, int kt) __attribute__((always_inline)) {
      constexpr int KK = decltype(kk_tag)::value;
      constexpr int CUR = KK & 1, NXT = CUR ^ 1;
      constexpr int NLT = NL + (KK == 0 ? LS : 0);  // loads of this trip
      const int nslab = kt + 1;
      const char* st = lds + (nslab & 3) * STAGE;
      const char* scb = sc_lds + ((nslab >> 2) & 1) * SC_BUF + (nslab & 3) * 8;
      const int lslab = kt + 4 < KT ? kt + 4 : KT - 1;
      char* dst = lds + (kt & 3) * STAGE + wave * 1024;
      const uint8_t* ap = a_src + lslab * 128;
      const uint8_t* bp = b_src + lslab * 128;
      const int g = (kt >> 2) + 1 < KG ? (kt >> 2) + 1 : KG - 1;
      auto load_at = [&](int l) __attribute__((always_inline)) {
        if (l < LA) {
          if constexpr (RAGGED_M) load_lds_16B(ap + a_off[l], dst + l * NW * 1024);
          else load_lds_16B(ap + l * row_step + lane_off, dst + l * NW * 1024);
        } else if (l < NL) load_lds_16B(bp + (l - LA) * row_step + lane_off, dst + A_BYTES + (l - LA) * NW * 1024);
        else {
          const int r0 = (wave * LS + (l - NL)) * 32;
          const uint8_t* src = r0 < BM ? As + (size_t)(tile_m * BM + r0) * Ksc : Bs + (size_t)(tile_n * BN + r0 - BM) * Ksc;
          if constexpr (RAGGED_M) {
            const int row = tile_m * BM + r0 + (lane >> 1);
            if (r0 < BM) src = As + (size_t)(row < M ? row : M - 1) * Ksc - (size_t)(lane >> 1) * Ksc;  // this lane's row, clamped
          }
          load_lds_16B(src + g * 32 + sc_lane_off, sc_lds + (g & 1) * SC_BUF + r0 * 32);
        }
      };
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (PINNED) {
#pragma unroll
        for (int m = 0; m < NM; m++) {
          mfma_at(m, am[CUR], an[CUR], sa[CUR], sb[CUR]);
#pragma unroll
          for (int r = m * NR / NM; r < (m + 1) * NR / NM; r++) read_at(st, scb, r, am[NXT], an[NXT], sa[NXT], sb[NXT]);
#pragma unroll
          for (int l = m * NLT / NM; l < (m + 1) * NLT / NM; l++) load_at(l);
          __builtin_amdgcn_sched_barrier(0);
        }
      } else {
#pragma unroll
        for (int r = 0; r < NR; r++) read_at(st, scb, r, am[NXT], an[NXT], sa[NXT], sb[NXT]);
#pragma unroll
        for (int l = 0; l < NLT; l++) load_at(l);
#pragma unroll
        for (int m = 0; m < NM; m++) mfma_at(m, am[CUR], an[CUR], sa[CUR], sb[CUR]);
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, NR, 0);
        __builtin_amdgcn_sched_group_barrier(0x010, NLT, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, NM - 1, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
      // in flight behind the wait: the loads of this trip and of the one before (the scale group rides with trip 0 of
      // a period, so trips 0 and 1 leave LS more)
      asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(2 * NL + (KK <= 1 ? LS : 0)) : "memory");
      __builtin_amdgcn_s_barrier();
    };
    issue_scale_loads(0);
#pragma unroll
    for (int t = 0; t < 3; t++) issue_loads(t, t < KT ? t : KT - 1);
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * NL) : "memory");
    __builtin_amdgcn_s_barrier();  // not __syncthreads(): its fence would wait for every load in flight
#pragma unroll
    for (int r = 0; r < NR; r++) read_at(lds, sc_lds, r, am[0], an[0], sa[0], sb[0]);
    issue_loads(3, 3 < KT ? 3 : KT - 1);
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(2 * NL) : "memory");
    __builtin_amdgcn_s_barrier();
    for (int kt = 0; kt < KT; kt += 4) {  // K % 1024 == 0 on this path
      trip(K0{}, kt);
      trip(K1{}, kt + 1);
      trip(K2{}, kt + 2);
      trip(K3{}, kt + 3);
    }
  } else {
  intx4 fm0[TM], fn0[TN], fm1[TM], fn1[TN];
  if constexpr (SCALES_LDS) issue_scale_loads(0);
  issue_loads(0, 0);
  wait_vmcnt0();
  __syncthreads();
  fetch_scales(sa[0], sb[0], 0);
  if constexpr (SCALES_LDS) issue_scale_loads(KG > 1 ? 1 : 0);
  issue_loads(1, KT > 1 ? 1 : 0);
  read_frags(lds, 0, fm0, fn0);
  if constexpr (!SCALES_LDS) wait_vmcnt0();

  // One slab (rotated k-loop, see gemm_f16_nt_pipelined): fragment reads for k-step s+1 ride between the
  // MFMAs of k-step s; the slab-retiring barrier sits in front of the last k-step's MFMAs, which overlap
  // the global -> LDS loads of slab kt+2 and the first fragment reads of slab kt+1.  With LDS-staged
  // scales the loop is unrolled by the scale-group period (4 slabs, KK = kt & 3 static) so that the body
  // stays one basic block: a branch inside it would end the scheduling region and the fixed
  // MFMA / LDS-read interleave with it.
  auto slab = [&](auto kk_tag, int kt) __attribute__((always_inline)) {
    constexpr int KK = decltype(kk_tag)::value;
    constexpr int CUR = KK & 1, NXT = CUR ^ 1;
    const char* st = lds + (kt & 1) * STAGE;
    __builtin_amdgcn_sched_barrier(0);
    fetch_scales(sa[NXT], sb[NXT], kt + 1 < KT ? kt + 1 : KT - 1);
    read_frags(st, 1, fm1, fn1);
    mfmas(K0{}, fm0, fn0, sa[CUR], sb[CUR]);
    if constexpr (SCALES_LDS) {
#pragma unroll
      for (int i = 0; i < TM + TN; i++) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);  // one fragment, one scale dword
      }
      __builtin_amdgcn_sched_group_barrier(0x008, TM * TN - (TM + TN), 0);
    } else {
      interleave();
    }
    __builtin_amdgcn_sched_barrier(0);
    read_frags(st, 2, fm0, fn0);
    mfmas(K1{}, fm1, fn1, sa[CUR], sb[CUR]);
    interleave();
    __builtin_amdgcn_sched_barrier(0);
    read_frags(st, 3, fm1, fn1);
    mfmas(K2{}, fm0, fn0, sa[CUR], sb[CUR]);
    interleave();
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
    issue_loads(kt & 1, kt + 2 < KT ? kt + 2 : KT - 1);
    if constexpr (SCALES_LDS && KK == 3) {
      // Group g replaces group g-2 in its buffer; the last slab of g-2 is this one, and its scale dwords
      // went into registers during the previous slab, before the barrier above.
      const int g = (kt >> 2) + 2;
      issue_scale_loads(g < KG ? g : KG - 1);
    }
    read_frags(lds + ((kt + 1) & 1) * STAGE, 0, fm0, fn0);
    mfmas(K3{}, fm1, fn1, sa[CUR], sb[CUR]);
    {
      constexpr int NL = LA + LB + (SCALES_LDS && KK == 3 ? LS : 0), NR = TM + TN, NM = TM * TN;
      constexpr int M_FOR_LOADS = NM / 2, L_PER_M = (NL + M_FOR_LOADS - 1) / M_FOR_LOADS;
#pragma unroll
      for (int i = 0; i < M_FOR_LOADS; i++) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x010, L_PER_M, 0);
      }
      constexpr int M_FOR_READS = NM - M_FOR_LOADS - 1, R_PER_M = (NR + M_FOR_READS - 1) / M_FOR_READS;
#pragma unroll
      for (int i = 0; i < M_FOR_READS; i++) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, R_PER_M, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  if constexpr (SCALES_LDS) {
    for (int kt = 0; kt < KT; kt += 4) {  // K % 1024 == 0 on this path
      slab(K0{}, kt);
      slab(K1{}, kt + 1);
      slab(K2{}, kt + 2);
      slab(K3{}, kt + 3);
    }
  } else {
    // scale dwords come straight from global memory (waited for with the slab's loads); two slabs per
    // trip keep the register-set indices static
    int kt = 0;
    for (; kt + 1 < KT; kt += 2) {
      slab(K0{}, kt);
      slab(K1{}, kt + 1);
    }
    if (kt < KT) slab(K0{}, kt);
  }
  }
  wait_vmcnt0();
  __syncthreads();

  if constexpr (sizeof(OutT) == 2) {
    // bf16 epilogue through LDS: each wave transposes its tile privately, then stores full rows
    constexpr int ROW_B = WTN * 2, CH = WTN / 8;
    char* ep = lds + wave * (WTM * ROW_B);
#pragma unroll
    for (int j = 0; j < TM; j++) {
      const int ml = j * 32 + r32;
#pragma unroll
      for (int i = 0; i < TN; i++)
#pragma unroll
        for (int q = 0; q < 4; q++) {
          const int c = i * 4 + q;
          ushortx4 v = {f32_to_bf16_rne(acc[i][j][4 * q]), f32_to_bf16_rne(acc[i][j][4 * q + 1]),
                        f32_to_bf16_rne(acc[i][j][4 * q + 2]), f32_to_bf16_rne(acc[i][j][4 * q + 3])};
          *reinterpret_cast<ushortx4*>(ep + ml * ROW_B + ((c ^ ((ml >> 1) & (CH - 1))) * 16) + 8 * h) = v;
        }
    }
    constexpr int ROWS_PER_IT = 64 / CH;
    const int er = lane / CH, ec = lane % CH;
    OutT* cbase = C + (size_t)(tile_m * BM + wm * WTM) * N + tile_n * BN + wn * WTN + ec * 8;
#pragma unroll
    for (int it = 0; it < WTM / ROWS_PER_IT; it++) {
      const int row = it * ROWS_PER_IT + er;
      intx4 v = *reinterpret_cast<const intx4*>(ep + row * ROW_B + ((ec ^ ((row >> 1) & (CH - 1))) * 16));
      if (!RAGGED_M || tile_m * BM + wm * WTM + row < M) *reinterpret_cast<intx4*>(cbase + (size_t)row * N) = v;
    }
  } else {
    const int m0 = tile_m * BM + wm * WTM + r32;
    const int n0 = tile_n * BN + wn * WTN + 4 * h;
#pragma unroll
    for (int j = 0; j < TM; j++) {
      OutT* crow = C + (size_t)(m0 + j * 32) * N + n0;
      if (RAGGED_M && m0 + j * 32 >= M) continue;
#pragma unroll
      for (int i = 0; i < TN; i++)
#pragma unroll
        for (int q = 0; q < 4; q++)
          MxOut<OutT>::store4(crow + i * 32 + q * 8, acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2],
                              acc[i][j][4 * q + 3]);
    }
  }
}

// Persistent kernel: one workgroup per CU walks its output tiles (ids pid, pid + grid, ...) as one
// continuous sequence of K slabs, so the first slabs and scale groups of the next tile are already in
// flight while a tile finishes, and the epilogue (through its own small LDS region) overlaps them.
// Slab schedule, fragment register sets X, Y, Z rotating with period two slabs:
//   k-step 0: MFMAs | LDS reads of the fragments of k-steps 1 and 2 and of the next slab's scale dwords
//   k-step 1: MFMAs | LDS reads of k-step 3 (into the set k-step 0 just released)
//   wait + barrier: the stage is fully read, the next slab has landed
//   k-step 2: MFMAs | most global -> LDS loads of the slab after next (into the stage just read)
//   k-step 3: MFMAs | LDS reads of k-step 0 of the next slab, remaining loads, every second slab the next
//             group of scale bytes
// Scale bytes are staged in groups of 2 slabs (16 bytes per row, one lane per row, two buffers).  The loop
// body is unrolled by that period so it contains no branch.  Needs K % 512 == 0 and K >= 1024.
template <int BM, int BN, int WM, int WN, typename OutT>
__global__ __launch_bounds__(WM* WN * 64) void gemm_mxfp4_persistent(const uint8_t* __restrict__ A, const uint8_t* __restrict__ As,
                                                                     const uint8_t* __restrict__ B, const uint8_t* __restrict__ Bs,
                                                                     OutT* __restrict__ C, int M, int N, int K, int tiles_m,
                                                                     int tiles_n, int group_m) {
  constexpr int NW = WM * WN;
  constexpr int WTM = BM / WM, WTN = BN / WN;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int A_BYTES = BM * 128, B_BYTES = BN * 128, STAGE = A_BYTES + B_BYTES;
  constexpr int A_GROUPS = BM / 8, B_GROUPS = BN / 8;
  static_assert(A_GROUPS % NW == 0 && B_GROUPS % NW == 0 && NW % 2 == 0, "loads must split evenly over an even number of waves");
  static_assert((BM + BN) == 64 * NW && BM % 64 == 0, "one scale wave-load (64 rows x 16 bytes) per wave and group");
  constexpr int LA = A_GROUPS / NW, LB = B_GROUPS / NW;
  constexpr int SC_BUF = (BM + BN) * 16;  // one scale group: 16 bytes (2 slabs x 8 blocks) per row
  constexpr int SC_BASE = 2 * STAGE, EP_BASE = SC_BASE + 2 * SC_BUF;
  constexpr int EP_WAVE = 32 * 64;  // one epilogue pass of a wave: a 32 x 32 bf16 tile, 64-byte rows

  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave / WN, wn = wave % WN;
  const int T = tiles_m * tiles_n;
  const int G = gridDim.x;
  const int Kb = K >> 1;   // bytes per row of codes
  const int Ksc = K >> 5;  // scale bytes per row
  const int KT = K / 256;  // even, >= 4 (checked by the host)

  const int lrow = lane >> 3;
  const int lchunk = (lane & 7) ^ (((wave & 1) << 2) | (lrow >> 1));
  const unsigned lane_off = (unsigned)lrow * (unsigned)Kb + (unsigned)lchunk * 16u;
  const unsigned row_step = (unsigned)NW * 8u * (unsigned)Kb;
  const unsigned panel_a = (unsigned)(BM - wave * 8) * (unsigned)Kb, panel_b = (unsigned)(BN - wave * 8) * (unsigned)Kb;
  // scale rows: wave w stages rows 64w .. 64w+63 of the tile's BM A rows followed by its BN B rows
  const bool sc_is_a = wave * 64 < BM;
  const unsigned sc_lane_off = (unsigned)lane * (unsigned)Ksc;

  auto tile_src = [&](int pid, buffer_rsrc_t& a_src, buffer_rsrc_t& b_src, buffer_rsrc_t& sc_src, int& tile_m, int& tile_n) {
    map_tile(pid, tiles_m, tiles_n, group_m, tile_m, tile_n);
    a_src = make_buffer(A + (size_t)(tile_m * BM + wave * 8) * Kb, panel_a);
    b_src = make_buffer(B + (size_t)(tile_n * BN + wave * 8) * Kb, panel_b);
    const uint8_t* sp = sc_is_a ? As + (size_t)(tile_m * BM + wave * 64) * Ksc : Bs + (size_t)(tile_n * BN + wave * 64 - BM) * Ksc;
    sc_src = make_buffer(sp, 64u * (unsigned)Ksc);
  };
  auto issue_loads = [&](auto first_tag, auto last_tag, int stage, buffer_rsrc_t ap, buffer_rsrc_t bp, int slab) __attribute__((always_inline)) {
    constexpr int FIRST = decltype(first_tag)::value, LAST = decltype(last_tag)::value;
    char* dst = lds + stage * STAGE + wave * 1024;
    const unsigned k_off = (unsigned)slab * 128u;
#pragma unroll
    for (int i = 0; i < LA; i++)
      if (i >= FIRST && i < LAST) buffer_load_lds_16B(ap, lane_off, k_off + i * row_step, dst + i * NW * 1024);
#pragma unroll
    for (int i = 0; i < LB; i++)
      if (LA + i >= FIRST && LA + i < LAST) buffer_load_lds_16B(bp, lane_off, k_off + i * row_step, dst + A_BYTES + i * NW * 1024);
  };
  auto issue_scale_loads = [&](int buf, buffer_rsrc_t sp, int group) {
    buffer_load_lds_16B(sp, sc_lane_off, (unsigned)group * 16u, lds + SC_BASE + buf * SC_BUF + wave * 1024);
  };

  const int r32 = lane & 31, h = lane >> 5;
  const int sw = ((4 * h) ^ ((r32 >> 1) & 7)) * 16;  // chunk ks + 4h of the row, swizzled
  const int a_base = (wm * WTM + r32) * 128 + sw;
  const int b_base = A_BYTES + (wn * WTN + r32) * 128 + sw;
  auto read_frags = [&](const char* st, int ks, intx4* fm, intx4* fn) {
#pragma unroll
    for (int j = 0; j < TM; j++) fm[j] = *reinterpret_cast<const intx4*>(st + ((a_base ^ (ks * 16)) + j * 4096));
#pragma unroll
    for (int i = 0; i < TN; i++) fn[i] = *reinterpret_cast<const intx4*>(st + ((b_base ^ (ks * 16)) + i * 4096));
  };
  // scale dword (bytes 4h .. 4h+3 of the row's 8 bytes of a slab) of virtual slab v
  const int sa_off = (wm * WTM + r32) * 16 + 4 * h, sb_off = (BM + wn * WTN + r32) * 16 + 4 * h;
  auto fetch_scales = [&](int* da, int* db, int v) {
    const char* buf = lds + SC_BASE + ((v >> 1) & 1) * SC_BUF + (v & 1) * 8;
#pragma unroll
    for (int j = 0; j < TM; j++) da[j] = *reinterpret_cast<const int*>(buf + sa_off + j * 512);
#pragma unroll
    for (int i = 0; i < TN; i++) db[i] = *reinterpret_cast<const int*>(buf + sb_off + i * 512);
  };

  floatx16 acc[TN][TM];
  auto zero_acc = [&]() {
#pragma unroll
    for (int i = 0; i < TN; i++)
#pragma unroll
      for (int j = 0; j < TM; j++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;
  };
  zero_acc();
  auto mfmas = [&](auto ks_tag, const intx4* fm, const intx4* fn, const int* ca, const int* cb) __attribute__((always_inline)) {
    constexpr int KS = decltype(ks_tag)::value;
#pragma unroll
    for (int i = 0; i < TN; i++)
#pragma unroll
      for (int j = 0; j < TM; j++) acc[i][j] = mfma_fp4_32x32x64<KS>(fn[i], cb[i], fm[j], ca[j], acc[i][j]);
  };

  constexpr int NM = TM * TN, NR = TM + TN, NL = LA + LB;
  constexpr int NL2 = NL < NM ? (3 * NL) / 4 : NM - 2;  // loads issued in k-step 2
  static_assert(3 * NR <= 2 * NM + 2 && NL - NL2 + 1 + (NR + 1) / 2 < NM, "k-step regions too small for their memory work");
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  using I2 = std::integral_constant<int, 2>;
  using I3 = std::integral_constant<int, 3>;
  using IL2 = std::integral_constant<int, NL2>;
  using IL = std::integral_constant<int, NL>;

  intx4 fmx[TM], fnx[TN], fmy[TM], fny[TN], fmz[TM], fnz[TN];
  int sa[2][TM], sb[2][TN];

  int pid = blockIdx.x;
  if (pid >= T) return;
  buffer_rsrc_t a_src, b_src, s_src, a_nxt, b_nxt, s_nxt;
  int tile_m, tile_n, nxt_m, nxt_n;
  tile_src(pid, a_src, b_src, s_src, tile_m, tile_n);
  issue_scale_loads(0, s_src, 0);
  issue_scale_loads(1, s_src, 1);
  issue_loads(I0{}, IL{}, 0, a_src, b_src, 0);
  wait_vmcnt0();
  __syncthreads();
  issue_loads(I0{}, IL{}, 1, a_src, b_src, 1);
  fetch_scales(sa[0], sb[0], 0);
  read_frags(lds, 0, fmx, fnx);
  int v = 0;  // slabs retired so far (even at every tile start: KT is even)

  // One slab; PAR = its parity.  Even slabs run k-steps 0..3 on sets X, Y, Z, X and leave the next
  // slab's first fragments in Y; odd slabs run on Y, Z, X, Y and leave them in X.
  auto slab = [&](auto par_tag, int kt, intx4* f0m, intx4* f0n, intx4* f1m, intx4* f1n, intx4* f2m, intx4* f2n) __attribute__((always_inline)) {
    constexpr int PAR = decltype(par_tag)::value;
    const char* st = lds + PAR * STAGE;
    __builtin_amdgcn_sched_barrier(0);
    read_frags(st, 1, f1m, f1n);
    read_frags(st, 2, f2m, f2n);
    fetch_scales(sa[PAR ^ 1], sb[PAR ^ 1], v + 1);
    mfmas(I0{}, f0m, f0n, sa[PAR], sb[PAR]);
#pragma unroll
    for (int i = 0; i < NM; i++) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, (3 * NR + NM - 1) / NM, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    read_frags(st, 3, f0m, f0n);  // k-step 0's set is free again
    mfmas(I1{}, f1m, f1n, sa[PAR], sb[PAR]);
#pragma unroll
    for (int i = 0; i < (NR + 1) / 2; i++) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, NM - (NR + 1) / 2, 0);
    __builtin_amdgcn_sched_barrier(0);
    // retire the slab: every wave's LDS reads of this stage have returned, the next slab has landed
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
    // loads of the slab after next (branch-free: past the end of this tile they belong to the next tile)
    const bool wrap = kt + 2 >= KT;
    const int ls = wrap ? kt + 2 - KT : kt + 2;
    const buffer_rsrc_t la = wrap ? a_nxt : a_src, lb = wrap ? b_nxt : b_src;
    issue_loads(I0{}, IL2{}, PAR, la, lb, ls);
    mfmas(I2{}, f2m, f2n, sa[PAR], sb[PAR]);
#pragma unroll
    for (int i = 0; i < NL2; i++) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x010, 1, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, NM - NL2, 0);
    __builtin_amdgcn_sched_barrier(0);
    // next slab's first fragments: into Y after an even slab (k-step 1's set), into X after an odd one
    // (k-step 2's set) -- both idle by now
    if constexpr (PAR == 0) read_frags(lds + STAGE, 0, f1m, f1n);
    else read_frags(lds, 0, f2m, f2n);
    issue_loads(IL2{}, IL{}, PAR, la, lb, ls);
    if constexpr (PAR == 1) {
      // The group two ahead replaces the group of this slab pair: its dwords went into registers during
      // the previous slab, before the barrier above.
      const int g = (kt >> 1) + 2, KG = KT >> 1;
      const bool gwrap = g >= KG;
      issue_scale_loads((v >> 1) & 1, gwrap ? s_nxt : s_src, gwrap ? g - KG : g);
    }
    mfmas(I3{}, f0m, f0n, sa[PAR], sb[PAR]);
#pragma unroll
    for (int i = 0; i < (NR + 1) / 2; i++) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
    }
#pragma unroll
    for (int i = 0; i < NL - NL2 + PAR; i++) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x010, 1, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, NM - (NR + 1) / 2 - (NL - NL2 + PAR), 0);
    __builtin_amdgcn_sched_barrier(0);
    v++;
  };

  for (; pid < T; pid += G) {
    const int npid = pid + G < T ? pid + G : pid;  // the last tile "continues" into itself; those loads are never used
    tile_src(npid, a_nxt, b_nxt, s_nxt, nxt_m, nxt_n);
    for (int kt = 0; kt < KT; kt += 2) {
      slab(I0{}, kt, fmx, fnx, fmy, fny, fmz, fnz);
      slab(I1{}, kt + 1, fmy, fny, fmz, fnz, fmx, fnx);
    }

    // ---- epilogue of this tile; the next tile's first slabs and scale groups are already in flight ----
    const int m0 = tile_m * BM + wm * WTM, n0 = tile_n * BN + wn * WTN;
    if constexpr (sizeof(OutT) == 2) {
      // one 32 x 32 MFMA tile per pass through a private 2 KiB region: 8-byte writes of 4 consecutive n
      // (chunk slot q ^ ((m>>2)&3)), whole 64-byte rows read back 16 bytes per lane.  LDS operations of a
      // wave execute in order, so passes need no waits between them.
      char* ep = lds + EP_BASE + wave * EP_WAVE;
      const int er = lane >> 2, ec = lane & 3;
#pragma unroll
      for (int j = 0; j < TM; j++)
#pragma unroll
        for (int i = 0; i < TN; i++) {
#pragma unroll
          for (int q = 0; q < 4; q++) {
            ushortx4 pv = {f32_to_bf16_rne(acc[i][j][4 * q]), f32_to_bf16_rne(acc[i][j][4 * q + 1]),
                           f32_to_bf16_rne(acc[i][j][4 * q + 2]), f32_to_bf16_rne(acc[i][j][4 * q + 3])};
            *reinterpret_cast<ushortx4*>(ep + r32 * 64 + ((q ^ ((r32 >> 2) & 3)) * 16) + 8 * h) = pv;
          }
#pragma unroll
          for (int it = 0; it < 2; it++) {
            const int row = it * 16 + er;
            intx4 ov = *reinterpret_cast<const intx4*>(ep + row * 64 + ((ec ^ ((row >> 2) & 3)) * 16));
            *reinterpret_cast<intx4*>(C + (size_t)(m0 + j * 32 + row) * N + n0 + i * 32 + ec * 8) = ov;
          }
          __builtin_amdgcn_sched_barrier(0);  // one pass at a time
        }
    } else {
#pragma unroll
      for (int j = 0; j < TM; j++) {
        OutT* crow = C + (size_t)(m0 + r32 + j * 32) * N + n0 + 4 * h;
#pragma unroll
        for (int i = 0; i < TN; i++)
#pragma unroll
          for (int q = 0; q < 4; q++)
            MxOut<OutT>::store4(crow + i * 32 + q * 8, acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2],
                                acc[i][j][4 * q + 3]);
      }
    }
    zero_acc();
    a_src = a_nxt;
    b_src = b_nxt;
    s_src = s_nxt;
    tile_m = nxt_m;
    tile_n = nxt_n;
  }
  wait_vmcnt0();  // loads issued past the last tile still target LDS: let them land before the block ends
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
    acc = mfma_fp4_32x32x64<0>(fb, sb, fa, sa, acc);
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

// Skinny-M kernel (M <= 32): weight streaming, HBM bound.  One workgroup (8 waves) per 32 rows of B;
// wave w owns 128-byte K segments w, w+8, ... of those rows (at most 4 per pass = 16 KiB of LDS per
// wave).  Everything a wave needs for a pass is requested up front -- B codes by direct-to-LDS loads
// (8 rows x 128 bytes per instruction, fully coalesced), A fragments and both scale sets straight into
// registers -- so that the whole 34 MB problem is in flight at once; then 16 MFMAs per wave, a reduction
// of the 8 partial 32x32 tiles through LDS, and one bf16 store.  Inside a 128-byte segment lane half h
// takes chunks 4h..4h+3 (k-step s' -> chunk 4h+s'): any chunk order is valid as long as A, B and the
// scale bytes agree, and this one makes a lane's scale bytes one aligned dword selected by op_sel.
template <typename OutT>
__global__ __launch_bounds__(512) void gemm_mxfp4_skinny(const uint8_t* __restrict__ A, const uint8_t* __restrict__ As,
                                                         const uint8_t* __restrict__ B, const uint8_t* __restrict__ Bs,
                                                         OutT* __restrict__ C, int M, int N, int K) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r32 = lane & 31, h = lane >> 5;
  const int n0 = blockIdx.x * 32;
  const int Kb = K >> 1, Ksc = K >> 5;
  const int nseg = Kb >> 7;  // 128-byte segments per row
  char* my = lds + wave * 16384;

  floatx16 acc;
#pragma unroll
  for (int r = 0; r < 16; r++) acc[r] = 0.f;

  const int lrow = lane >> 3;
  const bool m_ok = r32 < M;
  char* tr = lds + 8 * 16384 + wave * 4096;  // one A segment (32 rows x 128 bytes) per wave, for the transposition below
  const int m_cl = r32 < M ? r32 : M - 1;    // rows past M repeat the last one: their output columns are never stored
  // The MFMAs as inline assembly: with fp4 operands the instruction takes four registers per source, where the builtin
  // wants eight (the upper four zeroed) and a pass's sixteen such tuples do not fit beside everything else.  ZERO: the
  // first link of a chain takes a zero addend.  Scale byte of the operands' scale registers = LO + 2 HI.
#define MI355_SK_MFMA(LO, HI, ZERO, c, x, sx, y, sy)                                                                      \
  do {                                                                                                                   \
    if (ZERO)                                                                                                            \
      asm volatile("v_mfma_scale_f32_32x32x64_f8f6f4 %0, %1, %2, 0, %3, %4 op_sel:[" #LO "," #LO ",0] op_sel_hi:[" #HI "," #HI \
                   ",0] cbsz:4 blgp:4"                                                                                   \
                   : "=v"(c) : "v"(x), "v"(y), "v"(sx), "v"(sy));                                                        \
    else                                                                                                                 \
      asm volatile("v_mfma_scale_f32_32x32x64_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel:[" #LO "," #LO ",0] op_sel_hi:[" #HI "," #HI \
                   ",0] cbsz:4 blgp:4"                                                                                   \
                   : "+v"(c) : "v"(x), "v"(y), "v"(sx), "v"(sy));                                                        \
  } while (0)
  int seg0 = 0;
  for (; seg0 + 32 <= nseg; seg0 += 32) {  // a full pass covers 32 segments (4 per wave), straight-line
    // The wave takes four CONSECUTIVE segments (32 scale blocks per row), and lane half h the blocks 16 h .. 16 h + 15
    // of them, one per MFMA: k-step t multiplies block t (lanes of half 0) and block 16 + t (half 1).  Any assignment
    // of blocks to lanes and k-steps is valid as long as A, B and the scales agree; this one makes a lane's 16 scale
    // bytes of either operand ONE aligned 16-byte load (op_sel picks the byte of a dword) where a dword per lane and
    // segment took eight loads of 32 cache lines each.
    // A is the same 128 KiB for every workgroup and comes out of L2 -- as many bytes per workgroup as its share of
    // B.  It is fetched like B -- 8 rows x 128 bytes per instruction, lane = (row, chunk) -- FIRST, and while the B
    // loads issued behind it are still in flight it is turned into the MFMA layout through a 4 KiB LDS region (same
    // swizzle as B).
    // The A loads, the wait for them and the LDS instructions of the transposition are inline assembly: the compiler
    // waits for EVERY load in flight before the first use of a loaded register once direct-to-LDS loads are among
    // them, and before any LDS access it can see.  Loads return in order, so "at most the 16 B loads outstanding"
    // means A has landed.  LDS executes a wave's instructions in order, so the reads see the writes and the next
    // pass's writes come after this one's reads.
    // Workgroups start together and walk K in the same order: were wave w of every workgroup to take the same
    // segments, every workgroup of an XCD would ask for the same A lines at the same time.  Ids 8 apart share an XCD,
    // so the rotation is taken from the id's bits above those.
    intx4 fa[4][4];
    const int segw = seg0 + 4 * ((wave + (int)(blockIdx.x >> 3)) & 7);
    intx4 sav, sbv;  // the lane's 16 scale bytes of A and of B
#if defined(MI355_ABLATE_NO_SCALE_LOADS)
    sav = sbv = intx4{0x7f7f7f7f, 0x7f7f7f7f + segw, 0x7f7f7f7f, 0x7f7f7f7f};
#else
    sav = *reinterpret_cast<const intx4*>(As + (size_t)m_cl * Ksc + segw * 8 + 16 * h);
    sbv = *reinterpret_cast<const intx4*>(Bs + (size_t)(n0 + r32) * Ksc + segw * 8 + 16 * h);
#endif
#pragma unroll
    for (int q = 0; q < 4; q++) {
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const int row = i * 8 + lrow;
        const uint8_t* ap = A + (size_t)(row < M ? row : M - 1) * Kb + (segw + q) * 128 + (lane & 7) * 16;
#if defined(MI355_ABLATE_NO_A_LOADS)
        fa[q][i] = intx4{(int)(uintptr_t)ap, lane, q, i};
#else
        asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(fa[q][i]) : "v"(ap) : "memory");
#endif
      }
    }
#pragma unroll
    for (int qo = 0; qo < 4; qo++) {
      const int q = ((qo & 1) << 1) | (qo >> 1);  // segments 0, 2, 1, 3: the first eight k-steps read segments 0 and 2
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const int row = i * 8 + lrow;
        const int chunk = (lane & 7) ^ ((row >> 1) & 7);
#if !defined(MI355_ABLATE_NO_LOADS)
        load_lds_16B(B + (size_t)(n0 + row) * Kb + (segw + q) * 128 + chunk * 16, my + q * 4096 + i * 1024);
#endif
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_waitcnt vmcnt(16)"
                 : "+v"(fa[0][0]), "+v"(fa[0][1]), "+v"(fa[0][2]), "+v"(fa[0][3]), "+v"(fa[1][0]), "+v"(fa[1][1]),
                   "+v"(fa[1][2]), "+v"(fa[1][3]), "+v"(fa[2][0]), "+v"(fa[2][1]), "+v"(fa[2][2]), "+v"(fa[2][3]),
                   "+v"(fa[3][0]), "+v"(fa[3][1]), "+v"(fa[3][2]), "+v"(fa[3][3]));
    const unsigned tr_base = (unsigned)(uintptr_t)MI355_LDS(char, tr);
    const int sw = (r32 >> 1) & 7;
    // The 4 KiB region takes, per pass, four chunks of a segment of lane half 0 (q01) in the first 64 bytes of a row's
    // slots and the same four chunks of the segment of lane half 1 (2 + q01) in the second, so that every lane reads
    // in every pass: written by the lanes that loaded those chunks, read as block t = 8 q01 + 4 ch + cc.
    unsigned wa[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int row = i * 8 + lrow;
      wa[i] = tr_base + row * 128 + (((lane & 3) ^ ((row >> 1) & 7)) * 16);  // slot (lane & 3) of half 0; half 1: ^ 64
    }
    const unsigned ra = tr_base + r32 * 128;
    intx4 ga[16];  // A blocks in MFMA layout: ga[t] = block 16 h + t of the wave's 32
#pragma unroll
    for (int q01 = 0; q01 < 2; q01++) {
#pragma unroll
      for (int ch = 0; ch < 2; ch++) {
        if (((lane >> 2) & 1) == ch) {
#pragma unroll
          for (int i = 0; i < 4; i++) {
            asm volatile("ds_write_b128 %0, %1" ::"v"(wa[i]), "v"(fa[q01][i]) : "memory");
            asm volatile("ds_write_b128 %0, %1" ::"v"(wa[i] ^ 64u), "v"(fa[q01 + 2][i]) : "memory");
          }
        }
#pragma unroll
        for (int cc = 0; cc < 4; cc++)
          asm volatile("ds_read_b128 %0, %1" : "=v"(ga[q01 * 8 + ch * 4 + cc]) : "v"(ra + (unsigned)(((h * 4 + cc) ^ sw) * 16)) : "memory");
      }
    }
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(ga[0]), "+v"(ga[1]), "+v"(ga[2]), "+v"(ga[3]), "+v"(ga[4]), "+v"(ga[5]), "+v"(ga[6]), "+v"(ga[7]),
                   "+v"(ga[8]), "+v"(ga[9]), "+v"(ga[10]), "+v"(ga[11]), "+v"(ga[12]), "+v"(ga[13]), "+v"(ga[14]), "+v"(ga[15]));
    // B lands in order: the first eight k-steps (segments 0 and 2) run while the other half is still in flight.  The
    // fragment reads are assembly like the transposition's (the compiler would wait for every load in front of them).
    // Four chains (k-step t -> chain t % 4), so that no MFMA reads a sum written by one of the three before it.
    // "A" operand = B rows (n), "B" operand = A rows (m): pacc[n][m].
    const unsigned my_b = (unsigned)(uintptr_t)MI355_LDS(char, my) + 2 * h * 4096 + r32 * 128;  // block 16 h + t: segment 2 h + t / 8, chunk t % 8
    floatx16 pacc[4];
#pragma unroll
    for (int half = 0; half < 2; half++) {
      if (half == 0) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
      else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      intx4 fb[8];
#pragma unroll
      for (int c = 0; c < 8; c++)
        asm volatile("ds_read_b128 %0, %1" : "=v"(fb[c]) : "v"(my_b + (unsigned)(half * 4096 + ((c ^ sw) * 16))) : "memory");
      asm volatile("s_waitcnt lgkmcnt(0)"
                   : "+v"(fb[0]), "+v"(fb[1]), "+v"(fb[2]), "+v"(fb[3]), "+v"(fb[4]), "+v"(fb[5]), "+v"(fb[6]), "+v"(fb[7]));
#pragma unroll
      for (int c = 0; c < 8; c++) {
        const int t = half * 8 + c;
        const int sbq = sbv[t >> 2], saq = sav[t >> 2];
        if ((t & 3) == 0) MI355_SK_MFMA(0, 0, t < 4, pacc[0], fb[c], sbq, ga[t], saq);
        if ((t & 3) == 1) MI355_SK_MFMA(1, 0, t < 4, pacc[1], fb[c], sbq, ga[t], saq);
        if ((t & 3) == 2) MI355_SK_MFMA(0, 1, t < 4, pacc[2], fb[c], sbq, ga[t], saq);
        if ((t & 3) == 3) MI355_SK_MFMA(1, 1, t < 4, pacc[3], fb[c], sbq, ga[t], saq);
      }
    }
    // the compiler does not know that these registers were written by MFMAs just now: the wait states an MFMA result
    // needs before a vector instruction may read it, and every sum tied to a statement behind them
    asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15" : "+v"(pacc[0]), "+v"(pacc[1]), "+v"(pacc[2]), "+v"(pacc[3]));
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] += (pacc[0][r] + pacc[1][r]) + (pacc[2][r] + pacc[3][r]);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // this wave's LDS reads are done before the next pass overwrites
  }
  if (seg0 < nseg) {  // the last, partial pass: segments w, w + 8, ... of what is left, operands loaded in the MFMA's own layout
    intx4 fa[4][4];
    int sa[4], sb[4];
    int cnt = 0;
#pragma unroll
    for (int q = 0; q < 4; q++) {
      const int seg = seg0 + wave + 8 * q;
      if (seg < nseg) {
        cnt = q + 1;
        // B codes: 32 rows x 128 bytes -> 4 wave-loads of 8 rows; chunk c of row r in slot c ^ ((r >> 1) & 7)
#pragma unroll
        for (int i = 0; i < 4; i++) {
          const int row = i * 8 + lrow;
          const int chunk = (lane & 7) ^ ((row >> 1) & 7);
          load_lds_16B(B + (size_t)(n0 + row) * Kb + seg * 128 + chunk * 16, my + q * 4096 + i * 1024);
        }
        sb[q] = *reinterpret_cast<const int*>(Bs + (size_t)(n0 + r32) * Ksc + seg * 8 + 4 * h);
        if (m_ok) {
          sa[q] = *reinterpret_cast<const int*>(As + (size_t)r32 * Ksc + seg * 8 + 4 * h);
#pragma unroll
          for (int sp = 0; sp < 4; sp++)
            fa[q][sp] = *reinterpret_cast<const intx4*>(A + (size_t)r32 * Kb + seg * 128 + (4 * h + sp) * 16);
        } else {
          sa[q] = 0x7f7f7f7f;
#pragma unroll
          for (int sp = 0; sp < 4; sp++) fa[q][sp] = intx4{0, 0, 0, 0};
        }
      }
    }
    wait_vmcnt0();
    if (cnt > 0) {
      floatx16 pacc[4];  // one chain per k-step of a segment; segment 0 starts them
#pragma unroll
      for (int q = 0; q < 4; q++) {
        if (q < cnt) {
#pragma unroll
          for (int sp = 0; sp < 4; sp++) {
            const int c = 4 * h + sp;
            const intx4 fb = *reinterpret_cast<const intx4*>(my + q * 4096 + r32 * 128 + ((c ^ ((r32 >> 1) & 7)) * 16));
            // MFMA "A" operand = B rows (n), "B" operand = A rows (m): pacc[n][m]
            if (sp == 0) MI355_SK_MFMA(0, 0, q == 0, pacc[0], fb, sb[q], fa[q][sp], sa[q]);
            if (sp == 1) MI355_SK_MFMA(1, 0, q == 0, pacc[1], fb, sb[q], fa[q][sp], sa[q]);
            if (sp == 2) MI355_SK_MFMA(0, 1, q == 0, pacc[2], fb, sb[q], fa[q][sp], sa[q]);
            if (sp == 3) MI355_SK_MFMA(1, 1, q == 0, pacc[3], fb, sb[q], fa[q][sp], sa[q]);
          }
        }
      }
      asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15" : "+v"(pacc[0]), "+v"(pacc[1]), "+v"(pacc[2]), "+v"(pacc[3]));
#pragma unroll
      for (int r = 0; r < 16; r++) acc[r] += (pacc[0][r] + pacc[1][r]) + (pacc[2][r] + pacc[3][r]);
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  }
#undef MI355_SK_MFMA

  // reduce the 8 partial tiles: lane (m = r32, h) register r holds n = 8*(r/4) + 4h + r%4, i.e. four consecutive n per
  // group of four registers.  Tiles are stored [wave][m][n] with rows of 36 floats: 16-byte writes, and the threads
  // that add up one output element each read consecutive n -- with m as the fastest index every read instruction hit
  // one bank 32 times, and the eight waves' reads, which share the CU's LDS, took 4 us of the kernel's 14.
  __syncthreads();
  constexpr int RED_PITCH = 36;
  float* red = reinterpret_cast<float*>(lds);  // [wave][m 32][RED_PITCH]
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const floatx4 v = {acc[4 * j], acc[4 * j + 1], acc[4 * j + 2], acc[4 * j + 3]};
    *reinterpret_cast<floatx4*>(red + (wave * 32 + r32) * RED_PITCH + 8 * j + 4 * h) = v;
  }
  __syncthreads();
  for (int idx = threadIdx.x; idx < 1024; idx += 512) {
    const int m = idx >> 5, n = idx & 31;
    float v = 0.f;
#pragma unroll
    for (int w = 0; w < 8; w++) v += red[(w * 32 + m) * RED_PITCH + n];
    if (m < M) MxOut<OutT>::store1(C + (size_t)m * N + n0 + n, v);
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

// Register-staged form (see gemm_f16_nt_staged for the reasoning): four waves with 128x128 wave tiles, the
// codes of slab s+3 loaded into VGPRs while slab s computes, slab s+1 copied from registers into the LDS
// stage that slab s-1 left, every memory instruction alone between two MFMAs, one barrier per slab.
// Scales ride along as a 17th staging register: a lane owns one row of the tile and fetches the 16 scale
// bytes of two slabs, A rows with the even slabs (their own group), B rows with the odd slabs (the group that
// starts one slab later); they pass through four 4 KiB LDS buffers (A / B, group parity) from which every
// lane reads one dword per row tile and slab -- bytes 4h..4h+3, picked by op_sel -- one slab ahead.
template <typename OutT>
__global__ __launch_bounds__(256) void gemm_mxfp4_staged(const uint8_t* __restrict__ A, const uint8_t* __restrict__ As,
                                                         const uint8_t* __restrict__ B, const uint8_t* __restrict__ Bs,
                                                         OutT* __restrict__ C, int M, int N, int K, int tiles_m, int tiles_n,
                                                         int group_m) {
  constexpr int BM = 256, BN = 256, WN = 2, NW = 4;
  constexpr int WTM = 128, WTN = 128, TM = 4, TN = 4;
  constexpr int A_BYTES = BM * 128, STAGE = (BM + BN) * 128;
  constexpr int SC_OFF = 2 * STAGE;  // scale buffers: A parity 0, A parity 1, B parity 0, B parity 1, 4 KiB each
  typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
  typedef int i32x4 __attribute__((ext_vector_type(4)));

  extern __shared__ __attribute__((aligned(1024))) char lds[];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave / WN, wn = wave % WN;
  int tile_m, tile_n;
  map_tile(blockIdx.x, tiles_m, tiles_n, group_m, tile_m, tile_n);

  const unsigned row_bytes = (unsigned)K >> 1;  // codes
  const unsigned sc_bytes = (unsigned)K >> 5;   // scale bytes per row
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
  const int w_off = wave * 1024 + lrow * 128 + ((lc ^ (((wave & 1) << 2) | (lrow >> 1))) * 16);
  // scales: lane l of wave w owns row 64 w + l of the tile
  const i32x4 as_src = make_desc(As + (size_t)(tile_m * BM + wave * 64) * sc_bytes, (unsigned)(BM - wave * 64) * sc_bytes);
  const i32x4 bs_src = make_desc(Bs + (size_t)(tile_n * BN + wave * 64) * sc_bytes, (unsigned)(BN - wave * 64) * sc_bytes);
  const unsigned s_off = (unsigned)lane * sc_bytes;
  int sc_wr = SC_OFF + 4096 + (wave * 64 + lane) * 16;  // where the NEXT group's A scales go (B: + 8192); flips per group

  // staging registers: r[set][n], n < 8 the A row groups, 8..15 the B row groups, 16 the scale row
  u32x4 r[2][17];
#define MI355_MX_LOAD(S, n, k_off_)                                                                  \
  asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen"                                            \
               : "=v"(r[S][n])                                                                       \
               : "v"(g_off), "s"((n) < 8 ? a_src : b_src), "s"((k_off_) + (unsigned)((n)&7) * row_step) \
               : "memory")
#define MI355_MX_LOAD_SC(S, desc, group_)                                                            \
  asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen" : "=v"(r[S][16]) : "v"(s_off), "s"(desc), "s"((unsigned)(group_)*16u) : "memory")
  // `newer` = loads issued after the one that filled the register; they may still be in flight
#define MI355_MX_WRITE(S, n, newer, st_)                                                                                   \
  do {                                                                                                                     \
    asm volatile("s_waitcnt vmcnt(%1)" : "+v"(r[S][n]) : "n"(newer) : "memory");                                           \
    *reinterpret_cast<u32x4*>((st_) + w_off + ((n) < 8 ? (n)*NW * 1024 : A_BYTES + ((n)-8) * NW * 1024)) = r[S][n];        \
  } while (0)
#define MI355_MX_WRITE_SC(S, newer, addr_)                                                   \
  do {                                                                                       \
    asm volatile("s_waitcnt vmcnt(%1)" : "+v"(r[S][16]) : "n"(newer) : "memory");            \
    *reinterpret_cast<u32x4*>(lds + (addr_)) = r[S][16];                                     \
  } while (0)

  const int r32 = lane & 31, h = lane >> 5;
  const int sw = ((4 * h) ^ ((r32 >> 1) & 7)) * 16;  // chunk ks + 4h of the row, swizzled
  const int a_base = (wm * WTM + r32) * 128 + sw;
  const int b_base = A_BYTES + (wn * WTN + r32) * 128 + sw;
  // scale dwords of the CURRENT group (parity flips per group); + 8 for the group's second slab
  int sc_rd_a = SC_OFF + (wm * WTM + r32) * 16 + 4 * h;
  int sc_rd_b = SC_OFF + 8192 + (wn * WTN + r32) * 16 + 4 * h;

  floatx16 acc[TN][TM];
#pragma unroll
  for (int i = 0; i < TN; i++)
#pragma unroll
    for (int j = 0; j < TM; j++)
#pragma unroll
      for (int q = 0; q < 16; q++) acc[i][j][q] = 0.f;

  const int KT = K / 256;  // even, >= 4 (checked on the host)
  intx4 fm0[TM], fn0[TN], fm1[TM], fn1[TN];
  int ca0[TM], cb0[TN], ca1[TM], cb1[TN];

#define MI355_MX_LOAD_ALL(S, slab_)                                                                              \
  do {                                                                                                           \
    const unsigned ko_ = (unsigned)(slab_)*128u;                                                                 \
    MI355_MX_LOAD(S, 0, ko_); MI355_MX_LOAD(S, 1, ko_); MI355_MX_LOAD(S, 2, ko_); MI355_MX_LOAD(S, 3, ko_);      \
    MI355_MX_LOAD(S, 4, ko_); MI355_MX_LOAD(S, 5, ko_); MI355_MX_LOAD(S, 6, ko_); MI355_MX_LOAD(S, 7, ko_);      \
    MI355_MX_LOAD(S, 8, ko_); MI355_MX_LOAD(S, 9, ko_); MI355_MX_LOAD(S, 10, ko_); MI355_MX_LOAD(S, 11, ko_);    \
    MI355_MX_LOAD(S, 12, ko_); MI355_MX_LOAD(S, 13, ko_); MI355_MX_LOAD(S, 14, ko_); MI355_MX_LOAD(S, 15, ko_);  \
  } while (0)
  // prologue: slab 0 (+ A scales of group 0) -> set 0 -> stage 0; B scales of group 0 through a spare
  // register; slab 1 (+ B scales of group 1) -> set 1; then slab 2 (+ A scales of group 1) -> set 0
  const int KG = KT / 2;  // scale groups
  u32x4 rs;
  MI355_MX_LOAD_ALL(0, 0);
  MI355_MX_LOAD_SC(0, as_src, 0);
  asm volatile("buffer_load_dwordx4 %0, %1, %2, 0 offen" : "=v"(rs) : "v"(s_off), "s"(bs_src) : "memory");
  MI355_MX_LOAD_ALL(1, 1);
  MI355_MX_LOAD_SC(1, bs_src, KG > 1 ? 1 : 0);
  MI355_MX_WRITE(0, 0, 17, lds); MI355_MX_WRITE(0, 1, 17, lds); MI355_MX_WRITE(0, 2, 17, lds); MI355_MX_WRITE(0, 3, 17, lds);
  MI355_MX_WRITE(0, 4, 17, lds); MI355_MX_WRITE(0, 5, 17, lds); MI355_MX_WRITE(0, 6, 17, lds); MI355_MX_WRITE(0, 7, 17, lds);
  MI355_MX_WRITE(0, 8, 17, lds); MI355_MX_WRITE(0, 9, 17, lds); MI355_MX_WRITE(0, 10, 17, lds); MI355_MX_WRITE(0, 11, 17, lds);
  MI355_MX_WRITE(0, 12, 17, lds); MI355_MX_WRITE(0, 13, 17, lds); MI355_MX_WRITE(0, 14, 17, lds); MI355_MX_WRITE(0, 15, 17, lds);
  MI355_MX_WRITE_SC(0, 17, sc_wr - 4096);
  asm volatile("s_waitcnt vmcnt(17)" : "+v"(rs) : : "memory");
  *reinterpret_cast<u32x4*>(lds + sc_wr - 4096 + 8192) = rs;
  MI355_MX_LOAD_ALL(0, 2);
  MI355_MX_LOAD_SC(0, as_src, KG > 1 ? 1 : 0);
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __syncthreads();
#pragma unroll
  for (int j = 0; j < TM; j++) {
    fm0[j] = *reinterpret_cast<const intx4*>(lds + (a_base + j * 4096));
    fn0[j] = *reinterpret_cast<const intx4*>(lds + (b_base + j * 4096));
    ca0[j] = *reinterpret_cast<const int*>(lds + sc_rd_a + j * 512);
    cb0[j] = *reinterpret_cast<const int*>(lds + sc_rd_b + j * 512);
  }

  // fragment reads of the next k-step: A fragments in groups 0 and 1, B fragments in groups 2 and 3
  auto frag_reads = [&](int g, const char* rst, int rks, intx4* fm_n, intx4* fn_n) {
    if (g < 2) {
      fm_n[2 * g] = *reinterpret_cast<const intx4*>(rst + ((a_base ^ (rks * 16)) + (2 * g) * 4096));
      fm_n[2 * g + 1] = *reinterpret_cast<const intx4*>(rst + ((a_base ^ (rks * 16)) + (2 * g + 1) * 4096));
    } else {
      fn_n[2 * g - 4] = *reinterpret_cast<const intx4*>(rst + ((b_base ^ (rks * 16)) + (2 * g - 4) * 4096));
      fn_n[2 * g - 3] = *reinterpret_cast<const intx4*>(rst + ((b_base ^ (rks * 16)) + (2 * g - 3) * 4096));
    }
  };
  // scale dwords of the next slab (two per group of four MFMAs), `half` = 0 / 8 for the slab within its group
  auto scale_reads = [&](int g, int half, int* ca_n, int* cb_n) {
    if (g < 2) {
      ca_n[2 * g] = *reinterpret_cast<const int*>(lds + sc_rd_a + half + (2 * g) * 512);
      ca_n[2 * g + 1] = *reinterpret_cast<const int*>(lds + sc_rd_a + half + (2 * g + 1) * 512);
    } else {
      cb_n[2 * g - 4] = *reinterpret_cast<const int*>(lds + sc_rd_b + half + (2 * g - 4) * 512);
      cb_n[2 * g - 3] = *reinterpret_cast<const int*>(lds + sc_rd_b + half + (2 * g - 3) * 512);
    }
  };
#define MI355_MX_GROUP(KS, g, fm, fn, ca, cb, READS, W1, W2, LD)                        \
  do {                                                                                  \
    acc[g][0] = mfma_fp4_32x32x64<KS>(fn[g], cb[g], fm[0], ca[0], acc[g][0]);           \
    W1;                                                                                 \
    __builtin_amdgcn_sched_barrier(0);                                                  \
    acc[g][1] = mfma_fp4_32x32x64<KS>(fn[g], cb[g], fm[1], ca[1], acc[g][1]);           \
    W2;                                                                                 \
    __builtin_amdgcn_sched_barrier(0);                                                  \
    acc[g][2] = mfma_fp4_32x32x64<KS>(fn[g], cb[g], fm[2], ca[2], acc[g][2]);           \
    LD;                                                                                 \
    __builtin_amdgcn_sched_barrier(0);                                                  \
    acc[g][3] = mfma_fp4_32x32x64<KS>(fn[g], cb[g], fm[3], ca[3], acc[g][3]);           \
    READS;                                                                              \
    __builtin_amdgcn_sched_barrier(0);                                                  \
  } while (0)
#define MI355_NOP ((void)0)

  // Slab kt (scales in ca/cb) sits in stage P; set Q = 1 - P holds slab kt+1 and the scale row SCD travels
  // with (written to SCW), and is reloaded register by register with slab kt+3 and the scales of group GN.
  // In flight when register n is written: the rest of its own round (16 - n), the 17 loads of the other
  // set, and the loads of this slab issued so far.  HALF = 8 if slab kt+1 is the second slab of its group.
#define MI355_MX_SLAB(P, Q, kt_, ca, cb, ca_n, cb_n, SCD, SCW, GN, HALF)                                                    \
  do {                                                                                                                     \
    const char* st = lds + P * STAGE;                                                                                      \
    char* nst = lds + Q * STAGE;                                                                                           \
    const int nxt_ = (kt_) + 3 < KT ? (kt_) + 3 : KT - 1; /* past the end: re-fetch, never used */                         \
    const unsigned ko = (unsigned)nxt_ * 128u;                                                                             \
    const int gn_ = (GN) < KG ? (GN) : KG - 1;                                                                             \
    __builtin_amdgcn_sched_barrier(0);                                                                                     \
    MI355_MX_GROUP(0, 0, fm0, fn0, ca, cb, frag_reads(0, st, 1, fm1, fn1), MI355_MX_WRITE(Q, 0, 33, nst), MI355_MX_WRITE(Q, 1, 32, nst), MI355_MX_LOAD(Q, 0, ko));   \
    MI355_MX_GROUP(0, 1, fm0, fn0, ca, cb, frag_reads(1, st, 1, fm1, fn1), MI355_MX_WRITE(Q, 2, 32, nst), MI355_NOP, MI355_MX_LOAD(Q, 1, ko));                       \
    MI355_MX_GROUP(0, 2, fm0, fn0, ca, cb, frag_reads(2, st, 1, fm1, fn1), MI355_MX_WRITE(Q, 3, 32, nst), MI355_MX_WRITE(Q, 4, 31, nst), MI355_MX_LOAD(Q, 2, ko));   \
    MI355_MX_GROUP(0, 3, fm0, fn0, ca, cb, frag_reads(3, st, 1, fm1, fn1), MI355_MX_WRITE(Q, 5, 31, nst), MI355_NOP, MI355_MX_LOAD(Q, 3, ko));                       \
    MI355_MX_GROUP(1, 0, fm1, fn1, ca, cb, frag_reads(0, st, 2, fm0, fn0), MI355_MX_WRITE(Q, 6, 31, nst), MI355_MX_WRITE(Q, 7, 30, nst), MI355_MX_LOAD(Q, 4, ko));   \
    MI355_MX_GROUP(1, 1, fm1, fn1, ca, cb, frag_reads(1, st, 2, fm0, fn0), MI355_MX_WRITE(Q, 8, 30, nst), MI355_NOP, MI355_MX_LOAD(Q, 5, ko));                       \
    MI355_MX_GROUP(1, 2, fm1, fn1, ca, cb, frag_reads(2, st, 2, fm0, fn0), MI355_MX_WRITE(Q, 9, 30, nst), MI355_MX_WRITE(Q, 10, 29, nst), MI355_MX_LOAD(Q, 6, ko));  \
    MI355_MX_GROUP(1, 3, fm1, fn1, ca, cb, frag_reads(3, st, 2, fm0, fn0), MI355_MX_WRITE(Q, 11, 29, nst), MI355_NOP, MI355_MX_LOAD(Q, 7, ko));                      \
    MI355_MX_GROUP(2, 0, fm0, fn0, ca, cb, frag_reads(0, st, 3, fm1, fn1), MI355_MX_WRITE(Q, 12, 29, nst), MI355_NOP, MI355_MX_LOAD(Q, 8, ko));                      \
    MI355_MX_GROUP(2, 1, fm0, fn0, ca, cb, frag_reads(1, st, 3, fm1, fn1), MI355_MX_WRITE(Q, 13, 29, nst), MI355_NOP, MI355_MX_LOAD(Q, 9, ko));                      \
    MI355_MX_GROUP(2, 2, fm0, fn0, ca, cb, frag_reads(2, st, 3, fm1, fn1), MI355_MX_WRITE(Q, 14, 29, nst), MI355_NOP, MI355_MX_LOAD(Q, 10, ko));                     \
    MI355_MX_GROUP(2, 3, fm0, fn0, ca, cb, frag_reads(3, st, 3, fm1, fn1), MI355_MX_WRITE(Q, 15, 29, nst), MI355_MX_WRITE_SC(Q, 28, SCW), MI355_MX_LOAD(Q, 11, ko)); \
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");                                                                     \
    __syncthreads();                                                                                                       \
    __builtin_amdgcn_sched_barrier(0);                                                                                     \
    if (HALF == 0) { sc_rd_a ^= 4096; sc_rd_b ^= 4096; }                                                                   \
    MI355_MX_GROUP(3, 0, fm1, fn1, ca, cb, frag_reads(0, nst, 0, fm0, fn0); scale_reads(0, HALF, ca_n, cb_n), MI355_NOP, MI355_NOP, MI355_MX_LOAD(Q, 12, ko)); \
    MI355_MX_GROUP(3, 1, fm1, fn1, ca, cb, frag_reads(1, nst, 0, fm0, fn0); scale_reads(1, HALF, ca_n, cb_n), MI355_NOP, MI355_NOP, MI355_MX_LOAD(Q, 13, ko)); \
    MI355_MX_GROUP(3, 2, fm1, fn1, ca, cb, frag_reads(2, nst, 0, fm0, fn0); scale_reads(2, HALF, ca_n, cb_n), MI355_NOP, MI355_NOP, MI355_MX_LOAD(Q, 14, ko)); \
    MI355_MX_GROUP(3, 3, fm1, fn1, ca, cb, frag_reads(3, nst, 0, fm0, fn0); scale_reads(3, HALF, ca_n, cb_n), MI355_NOP, MI355_NOP,                            \
                   MI355_MX_LOAD(Q, 15, ko); MI355_MX_LOAD_SC(Q, SCD, gn_));                                             \
  } while (0)

  for (int kt = 0; kt < KT; kt += 2) {
    const int g0 = kt >> 1;
    // even slab: set 1 carries slab kt+1 and the B scales of group g0+1; reloaded with slab kt+3 and the B scales of g0+2
    MI355_MX_SLAB(0, 1, kt, ca0, cb0, ca1, cb1, bs_src, sc_wr + 8192, g0 + 2, 8);
    // odd slab: set 0 carries slab kt+2 and the A scales of group g0+1; reloaded with slab kt+4 and the A scales of g0+2
    MI355_MX_SLAB(1, 0, kt + 1, ca1, cb1, ca0, cb0, as_src, sc_wr, g0 + 2, 0);
    sc_wr ^= 4096;
    // The loads of the last slabs fetch nothing that is used, and behind the loop the compiler hands their
    // registers to the epilogue: let them land while the registers still belong to them.
    // The wait names every staging register as an input, so that the registers stay allocated to the loads up to it
    // however the compiler restructures the last iteration.
    if (kt + 2 >= KT) {
      asm volatile("s_waitcnt vmcnt(0)" ::"v"(r[0][0]), "v"(r[0][1]), "v"(r[0][2]), "v"(r[0][3]), "v"(r[0][4]), "v"(r[0][5]), "v"(r[0][6]), "v"(r[0][7]), "v"(r[0][8]), "v"(r[0][9]), "v"(r[0][10]), "v"(r[0][11]), "v"(r[0][12]), "v"(r[0][13]), "v"(r[0][14]), "v"(r[0][15]), "v"(r[0][16]) : "memory");
      asm volatile("" ::"v"(r[1][0]), "v"(r[1][1]), "v"(r[1][2]), "v"(r[1][3]), "v"(r[1][4]), "v"(r[1][5]), "v"(r[1][6]), "v"(r[1][7]), "v"(r[1][8]), "v"(r[1][9]), "v"(r[1][10]), "v"(r[1][11]), "v"(r[1][12]), "v"(r[1][13]), "v"(r[1][14]), "v"(r[1][15]), "v"(r[1][16]) : "memory");
    }
  }
#undef MI355_MX_SLAB
#undef MI355_MX_GROUP
#undef MI355_NOP
#undef MI355_MX_LOAD_ALL
#undef MI355_MX_WRITE_SC
#undef MI355_MX_WRITE
#undef MI355_MX_LOAD_SC
#undef MI355_MX_LOAD
  // drain the speculative loads; every wave is past its last fragment read before the epilogue reuses LDS
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
  __syncthreads();

  // epilogue addresses from a lane id taken behind the drain: derived from `lane` they would be computed ahead of it,
  // in registers that are not free while the staging sets are live
  const int le = opaque_lane_id();
  const int r32e = le & 31, he = le >> 5;
  if constexpr (sizeof(OutT) == 2) {
    // bf16 epilogue through LDS, one wave-private region each, 32 rows per pass: ds_write_b64 of 4 consecutive n
    // (chunk slot c ^ ((m >> 1) & 7)), whole 256-byte rows read back 16 bytes per lane
    constexpr int ROW_B = WTN * 2, CH = WTN / 8;
    char* ep = lds + wave * (32 * ROW_B);
    constexpr int ROWS_PER_IT = 64 / CH;
    const int er = le / CH, ec = le % CH;
#pragma unroll
    for (int j = 0; j < TM; j++) {
#pragma unroll
      for (int i = 0; i < TN; i++)
#pragma unroll
        for (int q = 0; q < 4; q++) {
          const int c = i * 4 + q;
          ushortx4 v = {f32_to_bf16_rne(acc[i][j][4 * q]), f32_to_bf16_rne(acc[i][j][4 * q + 1]),
                        f32_to_bf16_rne(acc[i][j][4 * q + 2]), f32_to_bf16_rne(acc[i][j][4 * q + 3])};
          *reinterpret_cast<ushortx4*>(ep + r32e * ROW_B + ((c ^ ((r32e >> 1) & 7)) * 16) + 8 * he) = v;
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
    const int m0 = tile_m * BM + wm * WTM + r32e;
    const int n0 = tile_n * BN + wn * WTN + 4 * he;
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
}

// Streamed form (see gemm_f16_nt_stream for the reasoning; the code bytes are laid out identically: a slab row is 128
// bytes = 256 codes = 8 scale blocks).  Whole 128-byte rows go global -> LDS directly, about two slabs ahead; the B
// fragments of a slab are held in registers (read from LDS during the first quarter of the slab before), the A rows
// are streamed fragment by fragment, each feeding 8 MFMAs 16x16x128 (a lane's 16 bytes are one scale block: lane l
// supplies row l & 15, block 2 (l >> 4) + kh of the slab in k half kh, so that its two scale bytes of a slab are
// neighbours).  One workgroup per CU walks its tiles as one slab sequence.
// LDS (160 KiB): B in a ring of five 16 KiB half buffers (U = rows 0..63, V = rows 64..127 of both 128-row halves; a
// half is loaded over two intervals, read seven or six intervals later and free one interval after that), A in two 32
// KiB buffers freed block by block, and 16 KiB for the scales.
// Scales are staged through LDS in groups of two slabs: 16 bytes per row, one lane per row, 8 KiB per group (A rows,
// then B rows), two buffers; a group is loaded in the first two steps of an even slab and first read 19 steps later.
// A lane fetches the two scale bytes of a row block and slab with one two-byte LDS read and the MFMA's op_sel picks
// the byte of its k half: the A scales of an m block four steps ahead, with the fragment of its first k half; the 8
// B scale pairs of the next slab in steps 4..11, into the register set the current slab does not use.
// One step = 8 MFMAs + LDS reads (A fragment, on even steps an A scale pair; steps 0..3: four B fragments; steps 4..11:
// one B scale pair) + one data load (+ a scale group load); a barrier every 4 steps.  At a barrier every wave has waited for its loads older
// than the newest 15 (about a slab's worth; the tightest case is B part 3, read 16 loads after its own) and for its LDS
// reads older than the interval:
//   interval q of slab t loads   A: block q - 1 of slab t + 2 (q = 0: block 3 of slab t + 1)
//                                B: part q of slab t + 3 (parts 0, 1 -> its U half, parts 2, 3 -> its V half)
template <typename OutT>
__global__ __launch_bounds__(256) void gemm_mxfp4_stream(const uint8_t* __restrict__ A, const uint8_t* __restrict__ As,
                                                         const uint8_t* __restrict__ B, const uint8_t* __restrict__ Bs,
                                                         OutT* __restrict__ C, int M, int N, int K, int tiles_m, int tiles_n,
                                                         int group_m) {
  typedef _Float16 half8 __attribute__((ext_vector_type(8)));  // 16 opaque bytes of codes
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
  const unsigned row_bytes = (unsigned)K / 2u, SK = (unsigned)K / 32u;
  const buffer_rsrc_t a_src = make_buffer(A, (unsigned)(tiles_m * BM) * row_bytes);
  const buffer_rsrc_t b_src = make_buffer(B, (unsigned)(tiles_n * BN) * row_bytes);
  const buffer_rsrc_t sa_src = make_buffer(As, (unsigned)(tiles_m * BM) * SK);
  const buffer_rsrc_t sb_src = make_buffer(Bs, (unsigned)(tiles_n * BN) * SK);
  const int lrow = lane >> 3;
  // codes: a wave-load covers 8 rows x 128 bytes; lane = (row l >> 3, slot l & 7) fetches chunk slot ^ ((row >> 1) & 7)
  const unsigned g_off = (unsigned)(wave * 8 + lrow) * row_bytes + (unsigned)((lane & 7) ^ (((wave & 1) << 2) | (lrow >> 1))) * 16u;
  // scales: a wave-load covers rows 64 w .. 64 w + 63 of the tile, 16 bytes (two slabs) per lane
  const unsigned gs_off = (unsigned)(wave * 64 + lane) * SK;
  const int KT = K / 256;  // even, >= 4 (checked on the host)
  unsigned a_cur = (unsigned)(tile_m * BM) * row_bytes, b_cur = (unsigned)(tile_n * BN) * row_bytes;
  unsigned a_nxt = a_cur, b_nxt = b_cur;  // the next tile (after the last: itself again; those loads are never used)
  unsigned sa_cur = (unsigned)(tile_m * BM) * SK, sb_cur = (unsigned)(tile_n * BN) * SK, sa_nxt = sa_cur, sb_nxt = sb_cur;
  auto slab_at = [&](int s, unsigned cur, unsigned nxt) { return s < KT ? cur + (unsigned)s * 128u : nxt + (unsigned)(s - KT) * 128u; };
  auto grp_at = [&](int s, unsigned cur, unsigned nxt) { return s < KT ? cur + (unsigned)s * 8u : nxt + (unsigned)(s - KT) * 8u; };
  // offsets of the slabs 1, 2 (A) and 3 (B) ahead and of the scale group after this pair of slabs; those of the next slab
  // are worked out one per step in the second half of a slab
  unsigned a_off1 = a_cur + 128u, a_off2 = a_cur + 256u, b_off3 = b_cur + 384u, sa_off = sa_cur + 16u, sb_off = sb_cur + 16u;
  unsigned n_a1 = 0, n_a2 = 0, n_b3 = 0, n_sa = 0, n_sb = 0;
  auto load_a = [&](int buf, int h, int blk, unsigned at) {
#if !defined(MI355_ABLATE_NO_LOADS)
    buffer_load_lds_16B(a_src, g_off, (unsigned)(h * 128 + blk * 32) * row_bytes + at,
                        lds + A_AT + buf * ABUF + (h * 16 + blk * 4 + wave) * 1024);
#endif
  };
  // part p (rows 32 p .. 32 p + 31 of either 128-row half) into the half buffer at byte offset half_at
  auto load_b = [&](int half_at, int h, int part, unsigned at) {
#if !defined(MI355_ABLATE_NO_LOADS)
    buffer_load_lds_16B(b_src, g_off, (unsigned)(h * 128 + part * 32) * row_bytes + at,
                        lds + B_AT + half_at + (h * 8 + (part & 1) * 4 + wave) * 1024);
#endif
  };
  auto load_scales = [&](bool is_b, int grp_at_lds, unsigned at) {
#if !defined(MI355_ABLATE_NO_LOADS) && !defined(MI355_ABLATE_NO_SCALE_LOADS)
    buffer_load_lds_16B(is_b ? sb_src : sa_src, gs_off, at, lds + S_AT + grp_at_lds + (is_b ? 4096 : 0) + wave * 1024);
#endif
  };

  // fragment reads: lane l takes row l & 15 of a 16-row block, chunk 2 (l >> 4) + kh of the 128-byte row: which scale
  // blocks of a slab meet in a k half is free as long as A and B agree, and this pairing puts a lane's two scale bytes
  // of a slab (k halves 0 and 1) side by side, so one two-byte LDS read fetches both and op_sel picks the byte
  const int r16 = lane & 15, cq = lane >> 4;
  const unsigned lds0 = (unsigned)(uintptr_t)MI355_LDS(char, lds);
  const unsigned lane_rd = (unsigned)(r16 * 128 + (((2 * cq) ^ (r16 >> 1)) & 7) * 16);  // k half 1: ^ 16
  unsigned aaddr[2][2];  // [A buffer][k half]
#pragma unroll
  for (int bf = 0; bf < 2; bf++)
#pragma unroll
    for (int kh = 0; kh < 2; kh++) aaddr[bf][kh] = lds0 + A_AT + bf * ABUF + wm * (WTM * 128) + (lane_rd ^ (kh * 16));
  const unsigned b_lane = lds0 + B_AT + wn * (64 * 128) + lane_rd;  // 64 rows of either half per half buffer
  unsigned bU[2], bV[2];  // [k half]: the U and V half buffers read in this slab
  // scale reads: the bytes of row (16 rb + r16), slab parity sp, blocks 2 cq and 2 cq + 1 sit at row * 16 + 8 sp + 2 cq
  const unsigned sa_lane = lds0 + S_AT + (unsigned)((wm * WTM + r16) * 16 + 2 * cq);
  const unsigned sb_lane = lds0 + S_AT + 4096 + (unsigned)((wn * WTN + r16) * 16 + 2 * cq);
  unsigned sa_rd = sa_lane, sa_rdn = sa_lane + 8, sb_rdn = sb_lane + 8;  // this slab's A scales, the next slab's A and B

  // [n block][m block].  Never cleared: the first MFMA of a tile on each accumulator (slab 0, k half 0) takes a zero
  // addend instead -- a register write in front of an inline-assembly MFMA would need wait states the compiler does not
  // know to insert.
  floatx4 acc[8][8];
  half8 fb0[2][8], fb1[2][8], fa[8];
  // scale registers hold two bytes: k half 0 in bits 0..7, k half 1 in bits 8..15 (the MFMA's op_sel picks one)
  int sb0[8], sb1[8], sat[4];  // B scales [row block] of the two slab parities; A scales by m block (a ring of four)
#if defined(MI355_ABLATE_NO_SCALE_READS)
  for (int i = 0; i < 8; i++) sb0[i] = sb1[i] = 127 * 257;
  for (int i = 0; i < 4; i++) sat[i] = 127 * 257;
#endif

  // MFMAs as inline assembly with the accumulators pinned to AGPRs (64 four-register accumulators: the compiler's own
  // allocation keeps moving some of them between the two register classes inside the loop).  No MFMA here reads an
  // accumulator written fewer than 8 MFMAs earlier.  x, sx: B codes and scales; y, sy: A codes and scales; KH (0 / 1): the
  // k half, which is also the byte of both scale registers that the MFMA applies.
#define MI355_SM_MFMA(KH, c, x, sx, y, sy)                                                                                \
  asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel:[%5,%5,0] op_sel_hi:[0,0,0] cbsz:4 blgp:4" \
               : "+a"(c) : "v"(x), "v"(y), "v"(sx), "v"(sy), "n"(KH))
#define MI355_SM_MFMA0(KH, c, x, sx, y, sy)                                                                               \
  asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, 0, %3, %4 op_sel:[%5,%5,0] op_sel_hi:[0,0,0] cbsz:4 blgp:4"  \
               : "=a"(c) : "v"(x), "v"(y), "v"(sx), "v"(sy), "n"(KH))
#define MI355_SM_ACC(ZERO, KH, c, x, sx, y, sy)              \
  do {                                                       \
    if constexpr (ZERO) MI355_SM_MFMA0(KH, c, x, sx, y, sy); \
    else MI355_SM_MFMA(KH, c, x, sx, y, sy);                 \
  } while (0)
  // The first MFMA of a step together with the wait for the step's A fragment and scale (y, sy: both were requested four
  // steps earlier; LG = LDS reads issued since).  One statement, with the registers as plain inputs: a separate wait
  // statement that names them as outputs makes the compiler put a wait state in front of their next use.  All the
  // statements involved are volatile assembly, which keeps their order.
#define MI355_SM_ACCW(ZERO, KH, LG, c, x, sx, y, sy)                                                                              \
  do {                                                                                                                          \
    if constexpr (ZERO)                                                                                                         \
      asm volatile("s_waitcnt lgkmcnt(%5)\n\tv_mfma_scale_f32_16x16x128_f8f6f4 %0, %3, %1, 0, %4, %2 op_sel:[%6,%6,0] op_sel_hi:[0,0,0] cbsz:4 blgp:4" \
                   : "=a"(c) : "v"(y), "v"(sy), "v"(x), "v"(sx), "n"(LG), "n"(KH));                                             \
    else                                                                                                                        \
      asm volatile("s_waitcnt lgkmcnt(%5)\n\tv_mfma_scale_f32_16x16x128_f8f6f4 %0, %3, %1, %0, %4, %2 op_sel:[%6,%6,0] op_sel_hi:[0,0,0] cbsz:4 blgp:4" \
                   : "+a"(c) : "v"(y), "v"(sy), "v"(x), "v"(sx), "n"(LG), "n"(KH));                                             \
  } while (0)
#define MI355_SM_READ(dst, addr, off) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(off))
#if defined(MI355_ABLATE_NO_SCALE_READS)  // no scale reads: the counted waits shrink by the reads that are gone
#define MI355_SM_READ16(dst, addr, off) do {} while (0)
#define MI355_SM_LG(with_scales, without) without
#define MI355_SM_LG_END "3"
#else
#define MI355_SM_READ16(dst, addr, off) asm volatile("ds_read_u16 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(off))
#define MI355_SM_LG(with_scales, without) with_scales
#define MI355_SM_LG_END "6"
#endif
#define MI355_SM_TIE8(X) "+v"(X[0]), "+v"(X[1]), "+v"(X[2]), "+v"(X[3]), "+v"(X[4]), "+v"(X[5]), "+v"(X[6]), "+v"(X[7])

  // ---- prologue: B0 (half buffers 0, 1), A0, B1 (2, 3), A1 blocks 0..2, scale group 0 ----
#pragma unroll
  for (int x = 0; x < 8; x++) load_b((x >> 2) * HALF, x & 1, x >> 1, b_cur);
#pragma unroll
  for (int x = 0; x < 8; x++) load_a(0, x & 1, x >> 1, a_cur);
#pragma unroll
  for (int x = 0; x < 8; x++) load_b((2 + (x >> 2)) * HALF, x & 1, x >> 1, b_cur + 128u);
#pragma unroll
  for (int x = 0; x < 6; x++) load_a(1, x & 1, x >> 1, a_cur + 128u);
  load_scales(false, 0, sa_cur);
  load_scales(true, 0, sb_cur);
  __builtin_amdgcn_sched_barrier(0);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_sched_barrier(0);
  bU[0] = b_lane; bU[1] = b_lane ^ 16;
  bV[0] = b_lane + HALF; bV[1] = bV[0] ^ 16;
  MI355_SM_READ(fb0[0][0], bU[0], 0 * 2048); MI355_SM_READ(fb0[0][1], bU[0], 1 * 2048);
  MI355_SM_READ(fb0[0][2], bU[0], 2 * 2048); MI355_SM_READ(fb0[0][3], bU[0], 3 * 2048);
  MI355_SM_READ(fb0[0][4], bV[0], 0 * 2048); MI355_SM_READ(fb0[0][5], bV[0], 1 * 2048);
  MI355_SM_READ(fb0[0][6], bV[0], 2 * 2048); MI355_SM_READ(fb0[0][7], bV[0], 3 * 2048);
  MI355_SM_READ(fb0[1][0], bU[1], 0 * 2048); MI355_SM_READ(fb0[1][1], bU[1], 1 * 2048);
  MI355_SM_READ(fb0[1][2], bU[1], 2 * 2048); MI355_SM_READ(fb0[1][3], bU[1], 3 * 2048);
  MI355_SM_READ(fb0[1][4], bV[1], 0 * 2048); MI355_SM_READ(fb0[1][5], bV[1], 1 * 2048);
  MI355_SM_READ(fb0[1][6], bV[1], 2 * 2048); MI355_SM_READ(fb0[1][7], bV[1], 3 * 2048);
  MI355_SM_READ(fa[0], aaddr[0][0], 0); MI355_SM_READ(fa[1], aaddr[0][1], 0);
  MI355_SM_READ(fa[2], aaddr[0][0], 2048); MI355_SM_READ(fa[3], aaddr[0][1], 2048);
  asm volatile("s_waitcnt lgkmcnt(0)" : MI355_SM_TIE8(fb0[0]), MI355_SM_TIE8(fb0[1]), "+v"(fa[0]), "+v"(fa[1]), "+v"(fa[2]), "+v"(fa[3]));
  MI355_SM_READ16(sb0[0], sb_lane, 0 * 256); MI355_SM_READ16(sb0[1], sb_lane, 1 * 256);
  MI355_SM_READ16(sb0[2], sb_lane, 2 * 256); MI355_SM_READ16(sb0[3], sb_lane, 3 * 256);
  MI355_SM_READ16(sb0[4], sb_lane, 4 * 256); MI355_SM_READ16(sb0[5], sb_lane, 5 * 256);
  MI355_SM_READ16(sb0[6], sb_lane, 6 * 256); MI355_SM_READ16(sb0[7], sb_lane, 7 * 256);
  MI355_SM_READ16(sat[0], sa_lane, 0); MI355_SM_READ16(sat[1], sa_lane, 256);
  asm volatile("s_waitcnt lgkmcnt(0)" : MI355_SM_TIE8(sb0), "+v"(sat[0]), "+v"(sat[1]));
  __builtin_amdgcn_s_barrier();  // every wave has read B0: its half buffers may receive slab 2's V half (0) and slab 3's U half (1)
  __builtin_amdgcn_sched_barrier(0);
  // B2: U half -> half buffer 4, V half -> half buffer 0
#pragma unroll
  for (int x = 0; x < 8; x++) load_b(((4 + (x >> 2)) % 5) * HALF, x & 1, x >> 1, b_cur + 256u);
  __builtin_amdgcn_sched_barrier(0);

  // B ring: slab t's halves live in half buffers (2 t) % 5 and (2 t + 1) % 5; pos = (2 t) % 5 for the current slab t
  int pos = 0;
  int sg_ld = SGRP;  // LDS offset of the scale group buffer the next group goes to (groups alternate)

  // Step s of a slab whose A buffer is PAR: MFMAs of (m block s / 2, k half s % 2) on fa[s % 8] and byte s % 2 of
  // sat[(s / 2) % 4] against FB[s % 2][0..7] and byte s % 2 of SB[0..7].  LGKM = LDS reads issued after those of step
  // s - 4 (which filled fa of this step; the m block's scales came with the even step of the pair).
#define MI355_SM_STEP(s, PAR, FB, FBN, SB, SBN, LGKM, FIRST)                                                               \
  do {                                                                                                                     \
    constexpr int s4 = (s) + 4, nb = s4 >= 16 ? 1 - (PAR) : (PAR), ns = s4 & 15, kh = (s)&1, mb = ((s) >> 1) & 3;          \
    MI355_SM_ACCW(FIRST && !kh, kh, LGKM, acc[0][(s) >> 1], FB[kh][0], SB[0], fa[(s)&7], sat[mb]);                          \
    MI355_SM_READ(fa[s4 & 7], aaddr[nb][ns & 1], (ns >> 1) * 2048);                                                        \
    __builtin_amdgcn_sched_barrier(0);                                                                                     \
    MI355_SM_ACC(FIRST && !kh, kh, acc[1][(s) >> 1], FB[kh][1], SB[1], fa[(s)&7], sat[mb]);                                 \
    if constexpr (kh == 0) { /* both scale bytes of m block (s + 4) / 2, two steps before its first use */                \
      if constexpr (s4 >= 16) MI355_SM_READ16(sat[(s4 >> 1) & 3], sa_rdn, (ns >> 1) * 256);                                \
      else MI355_SM_READ16(sat[(s4 >> 1) & 3], sa_rd, (ns >> 1) * 256);                                                    \
    }                                                                                                                      \
    __builtin_amdgcn_sched_barrier(0);                                                                                     \
    MI355_SM_ACC(FIRST && !kh, kh, acc[2][(s) >> 1], FB[kh][2], SB[2], fa[(s)&7], sat[mb]);                                 \
    if constexpr ((s) < 4) {                                                                                               \
      MI355_SM_READ(FBN[(s) >> 1][(4 * (s)) & 7], ((s)&1 ? bV : bU)[(s) >> 1], 0 * 2048);                                  \
      MI355_SM_READ(FBN[(s) >> 1][(4 * (s) + 1) & 7], ((s)&1 ? bV : bU)[(s) >> 1], 1 * 2048);                              \
    } else if constexpr ((s) < 12) {                                                                                       \
      MI355_SM_READ16(SBN[(s)-4], sb_rdn, ((s)-4) * 256); /* the next slab's B scales, one row block per step */           \
    }                                                                                                                      \
    __builtin_amdgcn_sched_barrier(0);                                                                                     \
    MI355_SM_ACC(FIRST && !kh, kh, acc[3][(s) >> 1], FB[kh][3], SB[3], fa[(s)&7], sat[mb]);                                 \
    if constexpr ((s) < 4) {                                                                                               \
      MI355_SM_READ(FBN[(s) >> 1][(4 * (s) + 2) & 7], ((s)&1 ? bV : bU)[(s) >> 1], 2 * 2048);                              \
      MI355_SM_READ(FBN[(s) >> 1][(4 * (s) + 3) & 7], ((s)&1 ? bV : bU)[(s) >> 1], 3 * 2048);                              \
    }                                                                                                                      \
    __builtin_amdgcn_sched_barrier(0);                                                                                     \
    MI355_SM_ACC(FIRST && !kh, kh, acc[4][(s) >> 1], FB[kh][4], SB[4], fa[(s)&7], sat[mb]);                                 \
    MI355_SM_ACC(FIRST && !kh, kh, acc[5][(s) >> 1], FB[kh][5], SB[5], fa[(s)&7], sat[mb]);                                 \
    {                                                                                                                      \
      constexpr int q = (s) >> 2, x = (s)&3;                                                                               \
      /* the scale group after this pair of slabs: A rows in step 0, B rows in step 1 of an even slab */                  \
      if constexpr ((PAR) == 0 && (s) == 0) load_scales(false, sg_ld, sa_off);                                             \
      if constexpr ((PAR) == 0 && (s) == 1) load_scales(true, sg_ld, sb_off);                                              \
      if constexpr (x < 2) {                                                                                               \
        if constexpr (q == 0) load_a(1 - (PAR), x, 3, a_off1);                                                             \
        else load_a(PAR, x, q - 1, a_off2);                                                                                \
      } else {                                                                                                             \
        load_b(q < 2 ? ld_u : ld_v, x - 2, q, b_off3);                                                                     \
      }                                                                                                                    \
    }                                                                                                                      \
    __builtin_amdgcn_sched_barrier(0);                                                                                     \
    if constexpr ((s) == 8) n_a1 = slab_at(kt + 2, a_cur, a_nxt);                                                          \
    if constexpr ((s) == 9) n_a2 = slab_at(kt + 3, a_cur, a_nxt);                                                          \
    if constexpr ((s) == 10) n_b3 = slab_at(kt + 4, b_cur, b_nxt);                                                         \
    if constexpr ((PAR) == 1 && (s) == 11) n_sa = grp_at(kt + 3, sa_cur, sa_nxt);                                          \
    if constexpr ((PAR) == 1 && (s) == 12) n_sb = grp_at(kt + 3, sb_cur, sb_nxt);                                          \
    MI355_SM_ACC(FIRST && !kh, kh, acc[6][(s) >> 1], FB[kh][6], SB[6], fa[(s)&7], sat[mb]);                                 \
    MI355_SM_ACC(FIRST && !kh, kh, acc[7][(s) >> 1], FB[kh][7], SB[7], fa[(s)&7], sat[mb]);                                 \
    __builtin_amdgcn_sched_barrier(0);                                                                                     \
  } while (0)
  // End of an interval: loads older than the newest VMC and LDS reads older than the interval are complete in every wave.
#define MI355_SM_SYNC(RD, VMC)                                                        \
  do {                                                                                \
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(%1)" ::"n"(MI355_KLOOP_VMCNT(VMC)), "n"(RD) : "memory");   \
    MI355_KLOOP_BARRIER();                                                               \
    __builtin_amdgcn_sched_barrier(0);                                                \
  } while (0)
  // LDS reads per step: the A fragment, in even steps the m block's A scales, + 4 B fragments in steps 0..3 or one row
  // block's B scales in steps 4..11: 6 5 6 5 | 3 2 3 2 | 3 2 3 2 | 2 1 2 1.  A step's count is the sum over the three
  // steps before it (at most 15 can be counted); an interval's end waits for the reads older than the interval.
#define MI355_SM_SLAB(PAR, FB, FBN, SB, SBN, FIRST, VMC)                                                         \
  do {                                                                                                          \
    {                                                                                                           \
      const int pu = pos + 2 >= 5 ? pos - 3 : pos + 2, pv = pos + 3 >= 5 ? pos - 2 : pos + 3; /* slab t + 1 */   \
      bU[0] = b_lane + (unsigned)(pu * HALF);                                                                   \
      bU[1] = bU[0] ^ 16;                                                                                       \
      bV[0] = b_lane + (unsigned)(pv * HALF);                                                                   \
      bV[1] = bV[0] ^ 16;                                                                                       \
    }                                                                                                           \
    /* slab t + 3: U half -> (2 t + 6) % 5 = pos + 1, V half -> (2 t + 7) % 5 = pos + 2 */                       \
    const int ld_u = (pos + 1 >= 5 ? pos - 4 : pos + 1) * HALF, ld_v = (pos + 2 >= 5 ? pos - 3 : pos + 2) * HALF; \
    MI355_SM_STEP(0, PAR, FB, FBN, SB, SBN, MI355_SM_LG(4, 3), FIRST);                                          \
    MI355_SM_STEP(1, PAR, FB, FBN, SB, SBN, MI355_SM_LG(9, 7), FIRST);                                         \
    MI355_SM_STEP(2, PAR, FB, FBN, SB, SBN, MI355_SM_LG(12, 11), FIRST);                                        \
    MI355_SM_STEP(3, PAR, FB, FBN, SB, SBN, MI355_SM_LG(15, 15), FIRST);                                        \
    MI355_SM_SYNC(15, VMC);                                                                                     \
    MI355_SM_STEP(4, PAR, FB, FBN, SB, SBN, MI355_SM_LG(15, 15), FIRST);                                        \
    MI355_SM_STEP(5, PAR, FB, FBN, SB, SBN, MI355_SM_LG(14, 15), FIRST);                                        \
    MI355_SM_STEP(6, PAR, FB, FBN, SB, SBN, MI355_SM_LG(10, 11), FIRST);                                        \
    MI355_SM_STEP(7, PAR, FB, FBN, SB, SBN, MI355_SM_LG(8, 7), FIRST);                                         \
    MI355_SM_SYNC(MI355_SM_LG(10, 4), VMC);                                                                                     \
    MI355_SM_STEP(8, PAR, FB, FBN, SB, SBN, MI355_SM_LG(7, 3), FIRST);                                         \
    MI355_SM_STEP(9, PAR, FB, FBN, SB, SBN, MI355_SM_LG(8, 3), FIRST);                                         \
    MI355_SM_STEP(10, PAR, FB, FBN, SB, SBN, MI355_SM_LG(7, 3), FIRST);                                        \
    MI355_SM_STEP(11, PAR, FB, FBN, SB, SBN, MI355_SM_LG(8, 3), FIRST);                                        \
    MI355_SM_SYNC(MI355_SM_LG(10, 4), VMC);                                                                                     \
    MI355_SM_STEP(12, PAR, FB, FBN, SB, SBN, MI355_SM_LG(7, 3), FIRST);                                        \
    MI355_SM_STEP(13, PAR, FB, FBN, SB, SBN, MI355_SM_LG(7, 3), FIRST);                                        \
    MI355_SM_STEP(14, PAR, FB, FBN, SB, SBN, MI355_SM_LG(5, 3), FIRST);                                         \
    MI355_SM_STEP(15, PAR, FB, FBN, SB, SBN, MI355_SM_LG(5, 3), FIRST);                                         \
    /* the next slab's B fragments and scales were requested in steps 0..11: they have landed; tie them here */ \
    asm volatile("s_waitcnt vmcnt(%24) lgkmcnt(" MI355_SM_LG_END ")"                                                              \
                 : MI355_SM_TIE8(FBN[0]), MI355_SM_TIE8(FBN[1]), MI355_SM_TIE8(SBN)                             \
                 : "n"(MI355_KLOOP_VMCNT(VMC)) : "memory");                                                                        \
    MI355_KLOOP_BARRIER();                                                                                         \
    __builtin_amdgcn_sched_barrier(0);                                                                          \
    a_off1 = n_a1;                                                                                              \
    a_off2 = n_a2;                                                                                              \
    b_off3 = n_b3;                                                                                              \
    pos = pos + 2 >= 5 ? pos - 3 : pos + 2;                                                                     \
    /* the scale reads of the next slab: its parity's 8 bytes; an odd slab's successor starts the next group */ \
    if constexpr ((PAR) == 0) {                                                                                 \
      sa_rd = sa_rdn;                                                                                           \
      sa_rdn = sa_lane + (unsigned)sg_ld;        /* slab t + 2: the group being loaded, first 8 bytes */        \
      sb_rdn = sb_lane + (unsigned)sg_ld;                                                                       \
    } else {                                                                                                    \
      sa_rd = sa_rdn;                                                                                           \
      sa_rdn = sa_rd + 8;                                                                                       \
      sb_rdn = sb_rdn + 8;                                                                                      \
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
    MI355_SM_SLAB(0, fb0, fb1, sb0, sb1, true, VMC_FIRST);
    kt = 1;
    MI355_SM_SLAB(1, fb1, fb0, sb1, sb0, false, 15);
    for (kt = 2; kt < KT; kt += 2) {
      MI355_SM_SLAB(0, fb0, fb1, sb0, sb1, false, 15);
      kt++;
      MI355_SM_SLAB(1, fb1, fb0, sb1, sb0, false, 15);
      kt--;
    }
    // ---- epilogue ---- (gemm_tiles.hpp).  16-bit results are staged through LDS in a wave-private 2 KiB region while
    // the next tile's slabs are landing; free at this point is block 3 of A buffer 1 (rows 96..127 of either half: twice
    // 4 KiB), which the next loads reach only after the barrier below.
    mx_stream_epilogue<false>(acc, 1.f, C + (size_t)(tile_m * BM + wm * WTM) * N + tile_n * BN + wn * WTN, N,
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
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" : MI355_SM_TIE8(fa), "+v"(sat[0]), "+v"(sat[1]), "+v"(sat[2]), "+v"(sat[3]));
#undef MI355_SM_SLAB
#undef MI355_SM_SYNC
#undef MI355_SM_STEP
#undef MI355_SM_TIE8
#undef MI355_SM_READ16
#undef MI355_SM_LG
#undef MI355_SM_LG_END
#undef MI355_SM_READ
#undef MI355_SM_ACCW
#undef MI355_SM_ACC
#undef MI355_SM_MFMA0
#undef MI355_SM_MFMA
}

struct MxVariant {
  const char* name;
  int bm, bn;
};
static const MxVariant kMxVariants[] = {
    {"persistent_256x256x256_w2x4", 256, 256},
    {"tiled_256x256x256_w2x4", 256, 256},
    {"tiled_128x128x256_w2x2", 128, 128},
    {"skinny_m32_n32_w8", 32, 32},
    {"staged_256x256x256_w2x2", 256, 256},
    {"stream_256x256x256_w2x2", 256, 256},
    {"stream_256x256x256_w2x2_walk", 256, 256},
    {"tiled_64x64x256_w2x2", 64, 64},
    {"generic_32x128", 32, 128},
};
constexpr int kNumMxVariants = sizeof(kMxVariants) / sizeof(kMxVariants[0]);
int mxfp4_variant_count() { return kNumMxVariants; }
const char* mxfp4_variant_name(int i) { return (i >= 0 && i < kNumMxVariants) ? kMxVariants[i].name : nullptr; }

template <int BM, int BN, int WM, int WN, typename OutT, bool SCALES_LDS, bool SLAB = false, bool RAGGED = false>
static int launch_mx_tiled(const void* a, const void* as, const void* b, const void* bs, void* c, int M, int N, int K,
                           hipStream_t stream) {
  auto kern = gemm_mxfp4_tiled<BM, BN, WM, WN, OutT, SCALES_LDS, SLAB, RAGGED>;
  constexpr int lds_bytes = (SLAB ? 4 : 2) * (BM + BN) * 128 + (SCALES_LDS ? 2 * (BM + BN) * 32 : 0);
  static_assert(lds_bytes <= 160 * 1024, "the stages and the scale buffers fit in LDS");
  static std::atomic<uint64_t> lds_ok{0};
  if (int rc = allow_lds(reinterpret_cast<const void*>(kern), lds_bytes, lds_ok, "gemm_mxfp4_tiled")) return rc;
  const int tiles_m = RAGGED ? (M + BM - 1) / BM : M / BM, tiles_n = N / BN;
  dim3 grid(tiles_m * tiles_n), block(WM * WN * 64);
  hipLaunchKernelGGL(kern, grid, block, lds_bytes, stream, (const uint8_t*)a, (const uint8_t*)as, (const uint8_t*)b,
                     (const uint8_t*)bs, (OutT*)c, M, N, K, tiles_m, tiles_n, 4);
  return check_launch("gemm_mxfp4_tiled", grid, block, lds_bytes);
}

static int mx_cu_count() {
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

template <int BM, int BN, int WM, int WN, typename OutT>
static int launch_mx_persistent(const void* a, const void* as, const void* b, const void* bs, void* c, int M, int N, int K,
                                hipStream_t stream) {
  auto kern = gemm_mxfp4_persistent<BM, BN, WM, WN, OutT>;
  // two data stages, two scale groups of 16 bytes per row, one 2 KiB epilogue pass per wave
  constexpr int lds_bytes = 2 * (BM + BN) * 128 + 2 * (BM + BN) * 16 + WM * WN * 2048;
  static std::atomic<uint64_t> lds_ok{0};
  if (int rc = allow_lds(reinterpret_cast<const void*>(kern), lds_bytes, lds_ok, "gemm_mxfp4_persistent")) return rc;
  const int tiles_m = M / BM, tiles_n = N / BN;
  const int T = tiles_m * tiles_n;
  int g = mx_cu_count() & ~7;  // multiples of 8 keep a workgroup's tiles on the XCD it runs on
  if (g < 8) g = 8;
  dim3 grid(T < g ? T : g), block(WM * WN * 64);
  hipLaunchKernelGGL(kern, grid, block, lds_bytes, stream, (const uint8_t*)a, (const uint8_t*)as, (const uint8_t*)b,
                     (const uint8_t*)bs, (OutT*)c, M, N, K, tiles_m, tiles_n, 4);
  return check_launch("gemm_mxfp4_persistent", grid, block, lds_bytes);
}

template <typename OutT>
static int launch_mx_staged(const void* a, const void* as, const void* b, const void* bs, void* c, int M, int N, int K,
                            hipStream_t stream) {
  auto kern = gemm_mxfp4_staged<OutT>;
  constexpr int lds_bytes = 2 * 512 * 128 + 4 * 4096;  // two data stages, four scale buffers
  static std::atomic<uint64_t> lds_ok{0};
  if (int rc = allow_lds(reinterpret_cast<const void*>(kern), lds_bytes, lds_ok, "gemm_mxfp4_staged")) return rc;
  const int tiles_m = M / 256, tiles_n = N / 256;
  dim3 grid(tiles_m * tiles_n), block(256);
  hipLaunchKernelGGL(kern, grid, block, lds_bytes, stream, (const uint8_t*)a, (const uint8_t*)as, (const uint8_t*)b,
                     (const uint8_t*)bs, (OutT*)c, M, N, K, tiles_m, tiles_n, 4);
  return check_launch("gemm_mxfp4_staged", grid, block, lds_bytes);
}

template <typename OutT>
static int launch_mx_stream(const void* a, const void* as, const void* b, const void* bs, void* c, int M, int N, int K,
                            hipStream_t stream, bool one_per_cu) {
  auto kern = gemm_mxfp4_stream<OutT>;
  constexpr int lds_bytes = 5 * 16384 + 2 * 32768 + 16384;  // five B half buffers, two A buffers, two scale groups
  static std::atomic<uint64_t> lds_ok{0};
  if (int rc = allow_lds(reinterpret_cast<const void*>(kern), lds_bytes, lds_ok, "gemm_mxfp4_stream")) return rc;
  const int tiles_m = M / 256, tiles_n = N / 256;
  int wgs = tiles_m * tiles_n;
  if (one_per_cu) {
    int g = mx_cu_count() & ~7;  // multiples of 8 keep a workgroup's tiles on the XCD it runs on
    if (g < 8) g = 8;
    if (wgs > g) wgs = g;
  }
  dim3 grid(wgs), block(256);
  hipLaunchKernelGGL(kern, grid, block, lds_bytes, stream, (const uint8_t*)a, (const uint8_t*)as, (const uint8_t*)b,
                     (const uint8_t*)bs, (OutT*)c, M, N, K, tiles_m, tiles_n, 4);
  return check_launch("gemm_mxfp4_stream", grid, block, lds_bytes);
}

template <typename OutT>
static int launch_mx(int variant, const void* a, const void* as, const void* b, const void* bs, void* c, int M, int N, int K,
                     hipStream_t stream) {
  switch (variant) {
    case 0: return launch_mx_persistent<256, 256, 2, 4, OutT>(a, as, b, bs, c, M, N, K, stream);
    case 1:
      if (K % 1024 == 0) return launch_mx_tiled<256, 256, 2, 4, OutT, true>(a, as, b, bs, c, M, N, K, stream);
      return launch_mx_tiled<256, 256, 2, 4, OutT, false>(a, as, b, bs, c, M, N, K, stream);
    case 2:
      if (K % 1024 == 0 && (long long)(M / 128) * (N / 128) <= 256)  // every workgroup has a CU to itself: the slab form
        return launch_mx_tiled<128, 128, 2, 2, OutT, true, true>(a, as, b, bs, c, M, N, K, stream);
      if (K % 1024 == 0) return launch_mx_tiled<128, 128, 2, 2, OutT, true>(a, as, b, bs, c, M, N, K, stream);
      return launch_mx_tiled<128, 128, 2, 2, OutT, false>(a, as, b, bs, c, M, N, K, stream);
    case 3: {
      auto kern = gemm_mxfp4_skinny<OutT>;
      constexpr int lds_bytes = 8 * 16384 + 8 * 4096;  // B segments + one A transposition region per wave
      static std::atomic<uint64_t> lds_ok{0};
      if (int rc = allow_lds(reinterpret_cast<const void*>(kern), lds_bytes, lds_ok, "gemm_mxfp4_skinny")) return rc;
      dim3 grid(N / 32), block(512);
      hipLaunchKernelGGL(kern, grid, block, lds_bytes, stream, (const uint8_t*)a, (const uint8_t*)as, (const uint8_t*)b,
                         (const uint8_t*)bs, (OutT*)c, M, N, K);
      return check_launch("gemm_mxfp4_skinny", grid, block, lds_bytes);
    }
    case 4: return launch_mx_staged<OutT>(a, as, b, bs, c, M, N, K, stream);
    case 5: return launch_mx_stream<OutT>(a, as, b, bs, c, M, N, K, stream, false);
    case 6: return launch_mx_stream<OutT>(a, as, b, bs, c, M, N, K, stream, true);
    case 7: return launch_mx_tiled<64, 64, 2, 2, OutT, true, true>(a, as, b, bs, c, M, N, K, stream);  // slab form only
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
  if (M <= 0 || N <= 0 || K <= 0 || M > (1 << 30) || N > (1 << 30) || K > (1 << 28))
    return fail(-MI355_E_SHAPE, "mxfp4_gemm: bad shape M=%lld N=%lld K=%lld", (long long)M, (long long)N, (long long)K);
  if (K % 32 != 0) return fail(-MI355_E_SHAPE, "mxfp4_gemm: K=%lld must be a multiple of the 32-element scale block", (long long)K);
  if (out_dtype != MI355_BF16 && out_dtype != MI355_F32)
    return fail(-MI355_E_DTYPE, "mxfp4_gemm: out_dtype %d (want MI355_BF16 or MI355_F32)", out_dtype);
  if (variant >= kNumMxVariants) return fail(-MI355_E_DTYPE, "mxfp4_gemm: variant %d out of range", variant);
  if (!aligned16(a) || !aligned16(b) || !aligned16(c))
    return fail(-MI355_E_ALIGN, "mxfp4_gemm: a, b, c must be 16-byte aligned");
  const bool sc_al = ((reinterpret_cast<uintptr_t>(a_scale) | reinterpret_cast<uintptr_t>(b_scale)) & 7u) == 0;
  const bool sc_al4 = ((reinterpret_cast<uintptr_t>(a_scale) | reinterpret_cast<uintptr_t>(b_scale)) & 3u) == 0;
  const bool sc_al16 = ((reinterpret_cast<uintptr_t>(a_scale) | reinterpret_cast<uintptr_t>(b_scale)) & 15u) == 0;
  auto fits = [&](int v) {
    if (v == kNumMxVariants - 1) return true;
    if (v == 3) return sc_al4 && M <= 32 && N % 32 == 0 && K % 256 == 0;  // skinny: whole 128-byte segments
    if (v == 7 && K % 1024 != 0) return false;  // scale groups of four slabs
    if ((v == 0 || v == 4) && !(sc_al16 && K % 512 == 0 && K >= 1024 && K <= (1 << 22))) return false;  // 2-slab scale groups
    // streamed: slabs in pairs, four or more; each operand behind one buffer descriptor
    if ((v == 5 || v == 6) && !(sc_al16 && K % 512 == 0 && K >= 1024 && M * (K / 2) < (1ll << 32) && N * (K / 2) < (1ll << 32))) return false;
    return sc_al && M % kMxVariants[v].bm == 0 && N % kMxVariants[v].bn == 0 && K % 256 == 0;
  };
  // Many rows that are no multiple of the 256-row tile against weights the large kernels take: the multiple of 256 and
  // the remainder (the 64x64 tile with a cut last row, or the weight-streaming kernel) as two products on row ranges.
  if (variant < 0 && M >= 512 && M % 256 != 0 && N % 256 == 0 && K % 1024 == 0 && sc_al16) {
    const int64_t m0 = M / 256 * 256;
    const size_t out_bytes = out_dtype == MI355_F32 ? 4 : 2;
    if (int rc = mi355_mxfp4_gemm(a, a_scale, b, b_scale, c, m0, N, K, out_dtype, -1, stream)) return rc;
    return mi355_mxfp4_gemm(static_cast<const char*>(a) + (size_t)m0 * (K / 2), static_cast<const char*>(a_scale) + (size_t)m0 * (K / 32), b,
                            b_scale, static_cast<char*>(c) + (size_t)m0 * N * out_bytes, M - m0, N, K, out_dtype, -1, stream);
  }
  bool cut_rows = false;  // the automatic choice took the 64x64 tile for a ragged M
  if (variant < 0) {
    // M <= 32 is weight streaming and has its own kernel.  The 256x256 tile halves the L2 -> LDS bytes per
    // flop; it is used when there are enough tiles to fill the 256 CUs and the last round of workgroups
    // is at least 85 % full.
    const long long t256 = (M / 256) * (N / 256);
    const long long rounds = (t256 + 255) / 256;
    const bool big = t256 >= 128 && t256 * 100 >= rounds * 256 * 85;
    if (fits(3)) variant = 3;
    else if (big && fits(6)) variant = 6;  // streamed, one workgroup per CU: 4096x8192x8192 124 us against 133 for the persistent kernel
    else if (big && K >= 32768 && fits(4)) variant = 4;  // its epilogue is not overlapped: ahead only from 128 slabs per tile
    else if (big && fits(0)) variant = 0;
    else if (big && fits(1)) variant = 1;
    // Few tiles: what counts is how many CUs pull operands (a lone workgroup moves about 75-100 GB/s through its CU
    // whatever its tile), so up to 320 tiles of 64x64 take those (128x8192x8192: 16.7 us on 128x128 tiles, 10.8 on
    // 64x64; 1024x1024x8192 15.3 -> 10.0; 256x8192x8192, 512 tiles of 64x64: 17.6 against 18.7).
    else if (fits(7) && ((M / 64) * (N / 64) <= 320 || !fits(2))) variant = 7;  // also what divides by 64 and not by 128
    // any number of rows against N % 64 == 0 and K % 1024 == 0 (activations against weights): the 64x64 tile with its
    // last tile row cut, instead of the bounds-checked kernel (100 x 8192 x 8192: 61 -> 12 us)
    else if (M % 64 != 0 && sc_al && N % 64 == 0 && K % 1024 == 0) {
      variant = 7;
      cut_rows = true;
    }
    else if (fits(2)) variant = 2;
    else variant = kNumMxVariants - 1;
  } else if (!fits(variant)) {
    return fail(-MI355_E_SHAPE, "mxfp4_gemm: variant %s does not fit M=%lld N=%lld K=%lld (tile %dx%d, K%%256==0, aligned scales)",
                kMxVariants[variant].name, (long long)M, (long long)N, (long long)K, kMxVariants[variant].bm, kMxVariants[variant].bn);
  }
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (cut_rows) {
    if (out_dtype == MI355_F32) return launch_mx_tiled<64, 64, 2, 2, float, true, true, true>(a, a_scale, b, b_scale, c, (int)M, (int)N, (int)K, s);
    return launch_mx_tiled<64, 64, 2, 2, unsigned short, true, true, true>(a, a_scale, b, b_scale, c, (int)M, (int)N, (int)K, s);
  }
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
