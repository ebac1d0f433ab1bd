// fp16 / bf16 NT GEMM for gfx950:  C[M,N] = A[M,K] . B[N,K]^T with fp32 accumulation.
//
// Kernels in this file, all on the same LDS row format: gemm_f16_nt_stream (the current kernel for large shapes: whole-row
// direct-to-LDS loads two slabs ahead, 16x16x32 MFMAs, a tile walk), gemm_f16_nt_persistent (8 waves, chosen for short
// K), gemm_f16_nt_pipelined (64x64, 128x64, 128x128 and 256x128 tiles: products of up to one round of tiles, any number
// of rows, with or without a K split, and the strip a sparse last round is cut into), gemm_f16_nt_staged (the
// register-staged predecessor of the streamed kernel, kept as the independent comparator of the bit-identity tests),
// gemm_f16_nt_skinny and gemm_f16_nt_skinny_rb (M <= 32 and M <= 128: weight streaming) and a bounds-checked kernel for
// any shape.
//
// LDS row format: K is walked in slabs of 64 halfs; a slab row is 128 bytes = 8 chunks of 16 bytes; both operands are
// K-contiguous, so the same row format serves A and B.  Slabs are copied global -> LDS with direct-to-LDS loads (no VGPR
// staging; the register-staged kernel excepted).  LDS rows are XOR-swizzled at chunk granularity: chunk c of row r lives
// in slot c ^ ((r >> 1) & 7).  LDS has 64 banks of 4 bytes, so two 128-byte rows span the banks once and a
// 16-lane phase of a ds_read_b128 (16 consecutive rows, one chunk each) is conflict-free exactly
// when (r & 1, slot) is distinct over those rows; measured 247 B/clk/CU against 128 for the
// c ^ (r & 7) swizzle and 32 unswizzled.  Because a direct-to-LDS load fixes the LDS slot by lane
// id, the swizzle is applied on the global side (lane -> which chunk it fetches).
//
// In the 32x32x16 kernels the MFMA roles are swapped (B rows feed the "A" operand, A rows feed the "B" operand) so a
// lane ends up owning 4 consecutive n for one m, which turns the epilogue into 8/16-byte
// row-contiguous stores.
//
// Workgroup -> tile mapping is XCD aware: hardware deals consecutive workgroup ids
// round-robin to the 8 XCDs (each with a private L2), so ids are first regrouped into 8
// contiguous ranges and then walked in GROUP_M-tall column-major panels to keep the A/B
// slabs that one XCD touches small.
#include <type_traits>

#include "common.hpp"
#include "gemm_tiles.hpp"

namespace mi355 {

// BF selects the 16-bit input format (false = fp16, true = bf16; mfma16 / cvt16 of the shared header).  Both travel
// through the kernels as opaque 16-bit lanes of half8 / half4 vectors (same tiles, same LDS format, same fragment
// layout); only the MFMA instruction and the conversion of the fp32 sums in the epilogue differ.
template <typename OutT, bool BF> struct OutPack;
template <bool BF> struct OutPack<float, BF> {
  static __device__ __forceinline__ void store4(float* p, float a, float b, float c, float d) {
    floatx4 v = {a, b, c, d};
    *reinterpret_cast<floatx4*>(p) = v;
  }
  static __device__ __forceinline__ void store1(float* p, float a) { *p = a; }
};
template <bool BF> struct OutPack<half_t, BF> {
  static __device__ __forceinline__ void store4(half_t* p, float a, float b, float c, float d) {
    half4 v = {cvt16<BF>(a), cvt16<BF>(b), cvt16<BF>(c), cvt16<BF>(d)};
    *reinterpret_cast<half4*>(p) = v;
  }
  static __device__ __forceinline__ void store1(half_t* p, float a) { *p = cvt16<BF>(a); }
};

// Software-pipelined kernel: a BM x BN output tile per workgroup, slabs copied global -> LDS with
// direct-to-LDS loads into a ring of slabs, 32x32x16 MFMAs.  Two forms of the k-loop:
//  * k-step pipeline, two slabs (SLAB = false; more than 256 tiles of 128x128, where two workgroups of 64 KiB share a
//    CU): the loop is rotated so that (a) the fragments of k-step s+1 are requested from LDS before the MFMAs of
//    k-step s issue, (b) the barrier that retires a slab sits in front of the last k-step's MFMAs, which then overlap
//    the first fragment reads of the next slab, and (c) the global -> LDS loads for slab k+2 are issued right after
//    that barrier into the stage that was just retired.  A load has one slab time to land.
//  * slab pipeline, four slabs (SLAB = true; a workgroup with a CU to itself, and the small tiles): the fragments of
//    a whole slab sit in one of two register sets, so a trip has one wait, in front of its barrier; the reads of slab
//    s+1 and the loads of slab s+4 are slotted between the MFMAs of slab s, and a load has three slab times to land.
//    A lone workgroup's slab time in the k-step form is its load latency plus, on small tiles, the chain of LDS read
//    latencies of four k-steps with one or two MFMAs each to cover them: 64x64 0.22 -> 0.15 us per slab, 128x128
//    0.60 -> 0.42 (what LDS bandwidth allows); 1024^3 on 64x64 tiles 6.7 -> 5.4 us, 1024x1024x4096 19.4 -> 15.9 us.
//  * RAGGED_M: M is any number of rows and N any multiple of 8 columns (the last tile row and the last tile column are
//    cut): the loads of A take row min(row, M - 1) and those of B row min(row, N - 1), so they stay inside the operands,
//    and the epilogue stores the rows below M and the 16-byte chunks left of column N only.  N is then both the row
//    pitch of C and its number of columns.  With a K split M is the number of rows of A, and every row of the stacked
//    partial tiles is stored (the workspace holds whole tiles).
template <int BM, int BN, int WM, int WN, typename OutT, bool BF, bool SLAB = false, bool RAGGED_M = false>
__global__ __launch_bounds__(WM* WN * 64) void gemm_f16_nt_pipelined(const half_t* __restrict__ A,
                                                                     const half_t* __restrict__ B,
                                                                     OutT* __restrict__ C, int M, int N, int K,
                                                                     int tiles_m, int tiles_n, int group_m, int ldk,
                                                                     int split_tiles_m, int ksplit_halfs, int krot_step) {
  // K: the length of the K range a workgroup adds up; ldk: the row pitch of A and B in halfs.  With a K split
  // (split_tiles_m > 0) the tile grid is stacked S times along M: tile row t stands for tile row t % split_tiles_m of A
  // and the K range t / split_tiles_m, ksplit_halfs apart, and C (the workspace) has S times the rows.
  constexpr int NW = WM * WN;
  constexpr int WTM = BM / WM, WTN = BN / WN;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int A_BYTES = BM * 128, B_BYTES = BN * 128, STAGE = A_BYTES + B_BYTES;
  constexpr int A_GROUPS = BM / 8, B_GROUPS = BN / 8;
  static_assert(A_GROUPS % NW == 0 && B_GROUPS % NW == 0 && NW % 2 == 0, "loads must split evenly over an even number of waves");
  constexpr int LA = A_GROUPS / NW, LB = B_GROUPS / NW;
  // A ring of STAGES slabs: slab s+STAGES is requested when slab s retires, so a load has STAGES-1 slab times to land,
  // and the wait that retires a slab leaves the loads of the STAGES-2 newest slabs in flight (loads return in order).
  constexpr int STAGES = !SLAB ? 2 : 4 * (BM + BN) * 128 <= 160 * 1024 ? 4 : 3;  // what 160 KiB of LDS hold
  static_assert((STAGES - 2) * (LA + LB) < 64, "the load counter has six bits");
  constexpr int IN_FLIGHT = (STAGES - 2) * (LA + LB);

  extern __shared__ __attribute__((aligned(1024))) char lds[];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave / WN, wn = wave % WN;
  int tile_m, tile_n;
  map_tile(blockIdx.x, tiles_m, tiles_n, group_m, tile_m, tile_n);

  const int lrow = lane >> 3;
  const int lchunk = (lane & 7) ^ (((wave & 1) << 2) | (lrow >> 1));
  // wave-uniform base pointer + one 32-bit per-lane offset (in halfs) shared by every load of the wave
  int a_tile = tile_m;
  size_t k_at = 0;
  if (split_tiles_m > 0)
    while (a_tile >= split_tiles_m) {  // at most S - 1 turns
      a_tile -= split_tiles_m;
      k_at += (size_t)ksplit_halfs;
    }
  const half_t* a_src = A + (size_t)(a_tile * BM + (RAGGED_M ? 0 : wave * 8)) * ldk + k_at;
  const half_t* b_src = B + (size_t)(tile_n * BN + (RAGGED_M ? 0 : wave * 8)) * ldk + k_at;
  const unsigned lane_off = (unsigned)lrow * (unsigned)ldk + (unsigned)lchunk * 8u;
  const size_t row_step = (size_t)NW * 8 * ldk;
  // RAGGED_M: the offset (in halfs, from the tile's first row) of this lane's row in A load i, the row clamped to M - 1
  unsigned a_off[RAGGED_M ? LA : 1];
  if constexpr (RAGGED_M) {
#pragma unroll
    for (int i = 0; i < LA; i++) {
      const int row = a_tile * BM + wave * 8 + i * NW * 8 + lrow;
      a_off[i] = (unsigned)((row < M ? row : M - 1) - a_tile * BM) * (unsigned)ldk + (unsigned)lchunk * 8u;
    }
  }
  unsigned b_off[RAGGED_M ? LB : 1];  // the same for the rows of B, clamped to N - 1
  if constexpr (RAGGED_M) {
#pragma unroll
    for (int i = 0; i < LB; i++) {
      const int row = tile_n * BN + wave * 8 + i * NW * 8 + lrow;
      b_off[i] = (unsigned)((row < N ? row : N - 1) - tile_n * BN) * (unsigned)ldk + (unsigned)lchunk * 8u;
    }
  }
  auto load_a = [&](const half_t* ap, int i, char* dst) {  // ap: a_src at the slab
    if constexpr (RAGGED_M) load_lds_16B(ap + a_off[i], dst);
    else load_lds_16B(ap + i * row_step + lane_off, dst);
  };
  auto load_b = [&](const half_t* bp, int i, char* dst) {
    if constexpr (RAGGED_M) load_lds_16B(bp + b_off[i], dst);
    else load_lds_16B(bp + i * row_step + lane_off, dst);
  };

  // krot_step != 0 (a few rows of A against many rows of B, which then stream from memory): the workgroups of tile
  // column n start their sweep over K n slabs in.  The rows of B are 2 K bytes apart, and workgroups that all read the
  // same offset of their rows at the same time crowd a few memory channels (128 x 28672 x 8192 with the weights out of
  // every cache: 122.5 -> 100.2 us); the workgroups of a column, which share those rows, still sweep together, and A is
  // small enough to stay in the L2s whatever the order.  With both operands large the rotation loses (the row panels
  // of A are shared by workgroups of different columns).
  const int krot = krot_step ? tile_n % (K / 64) : 0;
  auto rotated = [&](int slab) {
    const int r = slab + krot;
    return r < K / 64 ? r : r - K / 64;
  };
  auto issue_loads = [&](int stage, int slab0) {
    const int slab = rotated(slab0);
    char* dst = lds + stage * STAGE + wave * 1024;
    const half_t* ap = a_src + slab * 64;
    const half_t* bp = b_src + slab * 64;
#pragma unroll
    for (int i = 0; i < LA; i++) load_a(ap, i, dst + i * NW * 1024);
#pragma unroll
    for (int i = 0; i < LB; i++) load_b(bp, i, dst + A_BYTES + i * NW * 1024);
  };

  const int r32 = lane & 31, h = lane >> 5;
  const int sw = (h ^ ((r32 >> 1) & 7)) * 16;
  const int a_base = (wm * WTM + r32) * 128 + sw;
  const int b_base = A_BYTES + (wn * WTN + r32) * 128 + sw;
  auto read_frags = [&](const char* st, int ks, half8* fm, half8* fn) {
#pragma unroll
    for (int j = 0; j < TM; j++) fm[j] = *reinterpret_cast<const half8*>(st + ((a_base ^ (ks * 32)) + j * 4096));
#pragma unroll
    for (int i = 0; i < TN; i++) fn[i] = *reinterpret_cast<const half8*>(st + ((b_base ^ (ks * 32)) + i * 4096));
  };

  floatx16 acc[TN][TM];
#pragma unroll
  for (int i = 0; i < TN; i++)
#pragma unroll
    for (int j = 0; j < TM; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

  auto mfmas = [&](const half8* fm, const half8* fn) {
#pragma unroll
    for (int i = 0; i < TN; i++)
#pragma unroll
      for (int j = 0; j < TM; j++) acc[i][j] = mfma16<BF>(fn[i], fm[j], acc[i][j]);
  };

  const int KT = K / 64;
  if constexpr (SLAB) {
    // The stage slab s left is free at the start of trip s: every wave read it into registers a trip ago.
    half8 am[2][4][TM], an[2][4][TN];
    auto read_slab = [&](const char* st, half8(*fm)[TM], half8(*fn)[TN]) {
#pragma unroll
      for (int ks = 0; ks < 4; ks++) read_frags(st, ks, fm[ks], fn[ks]);
    };
    // A trip in source order, pinned by a scheduling fence behind every MFMA: the MFMA, then its share of the next
    // slab's fragment reads and of the loads (left to itself the compiler issues the loads in one burst, and a wave's
    // load is accepted only every 33 cycles: 1024x2048x4096 on 128x64 tiles 27.1 -> 24.7 us).  A trip of four MFMAs
    // (the 64x64 tile) is too short to spread anything over and is left to the compiler, which puts the reads and the
    // loads behind the first MFMA (pinned: 1024^3 5.4 -> 5.8 us).
    constexpr int NM = 4 * TM * TN, NR = 4 * (TM + TN), NL = LA + LB;
    constexpr bool PINNED = NM > 4;
    int stage = 0;  // kt % STAGES
    auto trip = [&](int kt, half8(*cm)[TM], half8(*cn)[TN], half8(*nm)[TM], half8(*nn)[TN]) {
      const int next = stage + 1 == STAGES ? 0 : stage + 1;
      const char* st = lds + next * STAGE;
      const int slab = rotated(kt + STAGES < KT ? kt + STAGES : KT - 1);
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (PINNED) {
        char* dst = lds + stage * STAGE + wave * 1024;
        const half_t* ap = a_src + slab * 64;
        const half_t* bp = b_src + slab * 64;
#pragma unroll
        for (int m = 0; m < NM; m++) {
          const int ks = m / (TM * TN), i = (m / TM) % TN, j = m % TM;
          acc[i][j] = mfma16<BF>(cn[ks][i], cm[ks][j], acc[i][j]);
#pragma unroll
          for (int r = m * NR / NM; r < (m + 1) * NR / NM; r++) {
            const int rk = r / (TM + TN), f = r % (TM + TN);
            if (f < TM) nm[rk][f] = *reinterpret_cast<const half8*>(st + ((a_base ^ (rk * 32)) + f * 4096));
            else nn[rk][f - TM] = *reinterpret_cast<const half8*>(st + ((b_base ^ (rk * 32)) + (f - TM) * 4096));
          }
#pragma unroll
          for (int l = m * NL / NM; l < (m + 1) * NL / NM; l++) {
            if (l < LA) load_a(ap, l, dst + l * NW * 1024);
            else load_b(bp, l - LA, dst + A_BYTES + (l - LA) * NW * 1024);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      } else {
        read_slab(st, nm, nn);
        issue_loads(stage, kt + STAGES < KT ? kt + STAGES : KT - 1);
#pragma unroll
        for (int ks = 0; ks < 4; ks++) mfmas(cm[ks], cn[ks]);
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, NR, 0);
        __builtin_amdgcn_sched_group_barrier(0x010, NL, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, NM - 1, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
      stage = next;
      asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(IN_FLIGHT) : "memory");
      __builtin_amdgcn_s_barrier();
    };
#pragma unroll
    for (int s = 0; s < STAGES - 1; s++) issue_loads(s, s < KT ? s : KT - 1);
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(IN_FLIGHT) : "memory");
    __builtin_amdgcn_s_barrier();
    read_slab(lds, am[0], an[0]);
    issue_loads(STAGES - 1, STAGES - 1 < KT ? STAGES - 1 : KT - 1);
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(IN_FLIGHT) : "memory");
    __builtin_amdgcn_s_barrier();
    int kt = 0;
    for (; kt + 2 <= KT; kt += 2) {
      trip(kt, am[0], an[0], am[1], an[1]);
      trip(kt + 1, am[1], an[1], am[0], an[0]);
    }
    if (kt < KT) trip(kt, am[0], an[0], am[1], an[1]);
  } else {
  half8 fm0[TM], fn0[TN], fm1[TM], fn1[TN];

#pragma unroll
  for (int s = 0; s < STAGES - 1; s++) issue_loads(s, s < KT ? s : KT - 1);
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(IN_FLIGHT) : "memory");
  __builtin_amdgcn_s_barrier();  // not __syncthreads(): its fence would wait for every load in flight
  issue_loads(STAGES - 1, STAGES - 1 < KT ? STAGES - 1 : KT - 1);
  read_frags(lds, 0, fm0, fn0);

  // One k-step region: the MFMAs of the current fragments with the LDS reads of the next fragments
  // slotted in between them (first instruction is an MFMA, so the wait in front of it only covers
  // reads issued a whole k-step earlier).
  // (Tiles with fewer MFMAs per k-step than fragment reads are left to the compiler's own order.)
  constexpr bool HAND_ORDER = TM * TN >= TM + TN;
  auto interleave = [&]() {
    if constexpr (HAND_ORDER) {
#pragma unroll
      for (int i = 0; i < TM + TN; i++) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // 1 MFMA
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // 1 DS read
      }
      __builtin_amdgcn_sched_group_barrier(0x008, TM * TN - (TM + TN), 0);
    }
  };

  for (int kt = 0; kt < KT; kt++) {
    const char* st = lds + (kt & (STAGES - 1)) * STAGE;
    __builtin_amdgcn_sched_barrier(0);
    read_frags(st, 1, fm1, fn1);
    mfmas(fm0, fn0);
    interleave();
    __builtin_amdgcn_sched_barrier(0);
    read_frags(st, 2, fm0, fn0);
    mfmas(fm1, fn1);
    interleave();
    __builtin_amdgcn_sched_barrier(0);
    read_frags(st, 3, fm1, fn1);
    mfmas(fm0, fn0);
    interleave();
    __builtin_amdgcn_sched_barrier(0);
    // retire the slab: every wave's LDS reads of this stage have returned, next slab has landed
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(IN_FLIGHT) : "memory");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    // The MFMAs of the last k-step need nothing new, so they lead; the loads for slab kt+STAGES (into the
    // stage just retired) and the first fragment reads of slab kt+1 are slotted in between them.
    // Past the end the loads re-fetch the last slab and the reads see stale bytes; neither is used.
    issue_loads(kt & (STAGES - 1), kt + STAGES < KT ? kt + STAGES : KT - 1);
    read_frags(lds + ((kt + 1) & (STAGES - 1)) * STAGE, 0, fm0, fn0);
    mfmas(fm1, fn1);
    if constexpr (HAND_ORDER) {
      constexpr int NL = LA + LB, NR = TM + TN, NM = TM * TN;
      constexpr int M_FOR_LOADS = NM / 2, L_PER_M = (NL + M_FOR_LOADS - 1) / M_FOR_LOADS;
#pragma unroll
      for (int i = 0; i < M_FOR_LOADS; i++) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x010, L_PER_M, 0);  // VMEM (direct-to-LDS loads)
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
  }
  }
  // the speculative loads of the last iterations target LDS: drain them before the epilogue reuses it
  wait_vmcnt0();
  __syncthreads();

  if constexpr (sizeof(OutT) == 2) {
    // fp16 epilogue through LDS (free after the last barrier): each wave transposes its own
    // WTM x WTN tile in a private region (ds_write_b64 of 4 consecutive n, chunk slot c ^ ((m>>1)&7)),
    // then reads whole rows back 16 bytes per lane and stores full 128-byte lines.
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
          half4 v = {cvt16<BF>(acc[i][j][4 * q]), cvt16<BF>(acc[i][j][4 * q + 1]), cvt16<BF>(acc[i][j][4 * q + 2]),
                     cvt16<BF>(acc[i][j][4 * q + 3])};
          *reinterpret_cast<half4*>(ep + ml * ROW_B + ((c ^ ((ml >> 1) & (CH - 1))) * 16) + 8 * h) = v;
        }
    }
    constexpr int ROWS_PER_IT = 64 / CH;
    const int er = lane / CH, ec = lane % CH;
    OutT* cbase = C + (size_t)(tile_m * BM + wm * WTM) * N + tile_n * BN + wn * WTN + ec * 8;
#pragma unroll
    for (int it = 0; it < WTM / ROWS_PER_IT; it++) {
      const int row = it * ROWS_PER_IT + er;
      half8 v = *reinterpret_cast<const half8*>(ep + row * ROW_B + ((ec ^ ((row >> 1) & (CH - 1))) * 16));
      if (!RAGGED_M || ((split_tiles_m > 0 || tile_m * BM + wm * WTM + row < M) && tile_n * BN + wn * WTN + ec * 8 < N))
        *reinterpret_cast<half8*>(cbase + (size_t)row * N) = v;
    }
  } else {
    // fp32 epilogue, the same way (a lane's four consecutive n are one 16-byte chunk; chunk slot c ^ (m & (CH - 1))):
    // stored straight from the accumulators a row would get 32 bytes per instruction, a quarter of a line.
    constexpr int ROW_B = WTN * 4, CH = WTN / 4;
    static_assert(NW * WTM * ROW_B <= STAGES * STAGE, "the waves' output tiles fit in the ring");
    char* ep = lds + wave * (WTM * ROW_B);
#pragma unroll
    for (int j = 0; j < TM; j++) {
      const int ml = j * 32 + r32;
#pragma unroll
      for (int i = 0; i < TN; i++)
#pragma unroll
        for (int q = 0; q < 4; q++) {
          const int c = i * 8 + q * 2 + h;
          floatx4 v = {acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
          *reinterpret_cast<floatx4*>(ep + ml * ROW_B + ((c ^ (ml & (CH - 1))) * 16)) = v;
        }
    }
    constexpr int ROWS_PER_IT = 64 / CH;
    const int er = lane / CH, ec = lane % CH;
    OutT* cbase = C + (size_t)(tile_m * BM + wm * WTM) * N + tile_n * BN + wn * WTN + ec * 4;
#pragma unroll
    for (int it = 0; it < WTM / ROWS_PER_IT; it++) {
      const int row = it * ROWS_PER_IT + er;
      floatx4 v = *reinterpret_cast<const floatx4*>(ep + row * ROW_B + ((ec ^ (row & (CH - 1))) * 16));
      if (!RAGGED_M || ((split_tiles_m > 0 || tile_m * BM + wm * WTM + row < M) && tile_n * BN + wn * WTN + ec * 4 < N))
        *reinterpret_cast<floatx4*>(cbase + (size_t)row * N) = v;
    }
  }
}

// Register-staged form: the slab after next waits in VGPRs instead of LDS.  160 KiB of LDS hold only two
// 64 KiB stages, so a direct-to-LDS load of slab s+2 cannot start before every wave has read slab s: the 16
// loads of a wave then issue in one burst in the last k-step, and a wave that is alone on its SIMD stands
// still while the texture path drains them (measured on the pipelined 4-wave kernel: 30 % of the time).
// Here four waves (512 registers each: 256 accumulators, two fragment sets, two staging sets of 16 x 16
// bytes) load slab s+3 into registers while slab s computes and copy slab s+1 from registers into the LDS
// stage that slab s-1 left, one load and about one ds_write per four MFMAs, evenly over the slab.  A load
// has two slab times to land, and there is still one barrier per slab:
//   k-steps 0..2: MFMAs | fragment reads of the next k-step | ds_write of slab s+1 | loads of slab s+3
//   wait + barrier: slab s+1 is complete in LDS, every wave has read slab s
//   k-step 3:     MFMAs | fragment reads of k-step 0 of slab s+1 | the last loads of slab s+3
// The loads are inline assembly so that the waits for them can be placed by hand (the compiler's vmcnt
// placement merges the loop's entry and back edge pessimistically).  Same LDS format as the other tiled
// kernels; the swizzle is applied by the ds_write address.
template <int BM, int BN, int WM, int WN, typename OutT, bool BF>
__global__ __launch_bounds__(WM* WN * 64) void gemm_f16_nt_staged(const half_t* __restrict__ A, const half_t* __restrict__ B,
                                                                  OutT* __restrict__ C, int M, int N, int K, int tiles_m,
                                                                  int tiles_n, int group_m) {
  constexpr int NW = WM * WN;
  constexpr int WTM = BM / WM, WTN = BN / WN;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int A_BYTES = BM * 128, B_BYTES = BN * 128, STAGE = A_BYTES + B_BYTES;
  constexpr int LA = BM / 8 / NW, LB = BN / 8 / NW;
  static_assert(NW == 4 && TM == 4 && TN == 4 && LA == 8 && LB == 8, "the slab schedule below is written out for a 2x2 grid of 128x128 wave tiles");
  static_assert(A_BYTES + (LB - 1) * NW * 1024 < 65536, "ds_write immediate offsets");
  typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
  typedef int i32x4 __attribute__((ext_vector_type(4)));

  extern __shared__ __attribute__((aligned(1024))) char lds[];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave / WN, wn = wave % WN;
  // The workgroup walks tiles blockIdx.x, blockIdx.x + gridDim.x, ... as ONE slab sequence: launched with one
  // workgroup per tile it is the plain kernel; launched with one workgroup per CU, the loads of a tile's last
  // three slabs fetch the next tile's first three, so only the first tile of a workgroup pays the pipeline fill,
  // and a tile's stores drain under the next tile's MFMAs.
  const int T = tiles_m * tiles_n;
  int pid = blockIdx.x;
  int tile_m, tile_n;
  map_tile(pid, tiles_m, tiles_n, group_m, tile_m, tile_n);

  // global side: wave-load i covers rows (i * NW + wave) * 8 .. + 7 of the tile, 8 lanes per 128-byte row piece
  const unsigned row_bytes = (unsigned)K * 2u;
  // buffer descriptors by hand: base, stride 0, size, raw dword format
  auto make_desc = [&](const half_t* base, unsigned bytes) {
    const unsigned long long p = reinterpret_cast<unsigned long long>(base);
    i32x4 d;
    d[0] = __builtin_amdgcn_readfirstlane((int)(unsigned)p);
    d[1] = __builtin_amdgcn_readfirstlane((int)(unsigned)((p >> 32) & 0xFFFFu));
    d[2] = __builtin_amdgcn_readfirstlane((int)bytes);
    d[3] = 0x00020000;
    return d;
  };
  i32x4 a_src = make_desc(A + (size_t)(tile_m * BM + wave * 8) * K, (unsigned)(BM - wave * 8) * row_bytes);
  i32x4 b_src = make_desc(B + (size_t)(tile_n * BN + wave * 8) * K, (unsigned)(BN - wave * 8) * row_bytes);
  i32x4 a_nxt = a_src, b_nxt = b_src;  // the tile after this one (the last tile: itself; those loads are never used)
  const unsigned row_step = (unsigned)NW * 8u * row_bytes;
  // Per-lane offsets of the K loop.  They are set at the start of every tile from a lane id the compiler cannot see
  // through: as plain loop invariants they would stay live across the epilogue, which has no registers to spare
  // beside the staging sets, and would be spilled to scratch around it.
  unsigned g_off;
  int w_off, a_base, b_base;
  auto lane_offsets = [&]() {
    const int lk = opaque_lane_id();
    const int lrow = lk >> 3, lc = lk & 7;
    g_off = (unsigned)lrow * row_bytes + (unsigned)lc * 16u;
    // LDS side of the staging writes: row r = (i * NW + wave) * 8 + lrow, chunk lc in slot lc ^ ((r >> 1) & 7); NW is
    // even, so the swizzle term does not depend on i
    w_off = wave * 1024 + lrow * 128 + ((lc ^ (((wave & 1) << 2) | (lrow >> 1))) * 16);
    const int r32k = lk & 31, hk = lk >> 5;
    const int sw = (hk ^ ((r32k >> 1) & 7)) * 16;
    a_base = (wm * WTM + r32k) * 128 + sw;
    b_base = A_BYTES + (wn * WTN + r32k) * 128 + sw;
  };
  lane_offsets();

  // staging registers: r[set][n], n < 8 the A row groups, n >= 8 the B row groups
  u32x4 r[2][16];
  // (macros: inline assembly inside a generic lambda cannot name the enclosing function's arrays)
#define MI355_ST_LOAD(S, n, k_off_, da_, db_)                                                        \
  asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen"                                            \
               : "=v"(r[S][n])                                                                       \
               : "v"(g_off), "s"((n) < 8 ? da_ : db_), "s"((k_off_) + (unsigned)((n)&7) * row_step)   \
               : "memory")
  // `newer` = loads issued after the one that filled r[S][n]; they may still be in flight
#define MI355_ST_WRITE(S, n, newer, st_)                                                                                   \
  do {                                                                                                                     \
    asm volatile("s_waitcnt vmcnt(%1)" : "+v"(r[S][n]) : "n"(newer) : "memory");                                           \
    *reinterpret_cast<u32x4*>((st_) + w_off + ((n) < 8 ? (n)*NW * 1024 : A_BYTES + ((n)-8) * NW * 1024)) = r[S][n];        \
  } while (0)

  auto read_frags = [&](const char* st, int ks, half8* fm, half8* fn) {
#pragma unroll
    for (int j = 0; j < TM; j++) fm[j] = *reinterpret_cast<const half8*>(st + ((a_base ^ (ks * 32)) + j * 4096));
#pragma unroll
    for (int i = 0; i < TN; i++) fn[i] = *reinterpret_cast<const half8*>(st + ((b_base ^ (ks * 32)) + i * 4096));
  };

  floatx16 acc[TN][TM];
#pragma unroll
  for (int i = 0; i < TN; i++)
#pragma unroll
    for (int j = 0; j < TM; j++)
#pragma unroll
      for (int q = 0; q < 16; q++) acc[i][j][q] = 0.f;

  const int KT = K / 64;  // even, >= 4 (checked on the host)
  half8 fm0[TM], fn0[TN], fm1[TM], fn1[TN];

  // prologue: slab 0 -> set 0 -> stage 0; slab 1 -> set 1; slab 2 -> set 0
#define MI355_ST_LOAD_ALL(S, slab_)                                       \
  do {                                                                    \
    const unsigned ko_ = (unsigned)(slab_)*128u;                          \
    MI355_ST_LOAD(S, 0, ko_, a_src, b_src); MI355_ST_LOAD(S, 1, ko_, a_src, b_src); MI355_ST_LOAD(S, 2, ko_, a_src, b_src);     \
    MI355_ST_LOAD(S, 3, ko_, a_src, b_src); MI355_ST_LOAD(S, 4, ko_, a_src, b_src); MI355_ST_LOAD(S, 5, ko_, a_src, b_src);     \
    MI355_ST_LOAD(S, 6, ko_, a_src, b_src); MI355_ST_LOAD(S, 7, ko_, a_src, b_src); MI355_ST_LOAD(S, 8, ko_, a_src, b_src);     \
    MI355_ST_LOAD(S, 9, ko_, a_src, b_src); MI355_ST_LOAD(S, 10, ko_, a_src, b_src); MI355_ST_LOAD(S, 11, ko_, a_src, b_src);   \
    MI355_ST_LOAD(S, 12, ko_, a_src, b_src); MI355_ST_LOAD(S, 13, ko_, a_src, b_src); MI355_ST_LOAD(S, 14, ko_, a_src, b_src);  \
    MI355_ST_LOAD(S, 15, ko_, a_src, b_src);                                                                                    \
  } while (0)
  MI355_ST_LOAD_ALL(0, 0);
  MI355_ST_LOAD_ALL(1, 1);
  MI355_ST_WRITE(0, 0, 16, lds); MI355_ST_WRITE(0, 1, 16, lds); MI355_ST_WRITE(0, 2, 16, lds); MI355_ST_WRITE(0, 3, 16, lds);
  MI355_ST_WRITE(0, 4, 16, lds); MI355_ST_WRITE(0, 5, 16, lds); MI355_ST_WRITE(0, 6, 16, lds); MI355_ST_WRITE(0, 7, 16, lds);
  MI355_ST_WRITE(0, 8, 16, lds); MI355_ST_WRITE(0, 9, 16, lds); MI355_ST_WRITE(0, 10, 16, lds); MI355_ST_WRITE(0, 11, 16, lds);
  MI355_ST_WRITE(0, 12, 16, lds); MI355_ST_WRITE(0, 13, 16, lds); MI355_ST_WRITE(0, 14, 16, lds); MI355_ST_WRITE(0, 15, 16, lds);
  MI355_ST_LOAD_ALL(0, 2);
  // every tile starts with all three slabs landed (later tiles: the K loop ends that way), so the first two slabs
  // of a tile never wait for a load
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
  __syncthreads();
  read_frags(lds, 0, fm0, fn0);

  // One group = the four MFMAs of accumulator row g, each followed by one piece of memory work, so that no
  // MFMA waits behind more than one long-issuing instruction (a 1 KiB ds_write takes about 20 cycles to
  // issue, an MFMA keeps the pipe busy for 32): up to two ds_writes, the load, and two fragment reads of the
  // next k-step.  The A fragments (all four are needed by the next k-step's first group) are read in groups
  // 0 and 1, the B fragments in groups 2 and 3: every fragment is requested two groups or more before its use.
  auto frag_reads = [&](int g, const char* rst, int rks, half8* fm_n, half8* fn_n) {
    if (g < 2) {
      fm_n[2 * g] = *reinterpret_cast<const half8*>(rst + ((a_base ^ (rks * 32)) + (2 * g) * 4096));
      fm_n[2 * g + 1] = *reinterpret_cast<const half8*>(rst + ((a_base ^ (rks * 32)) + (2 * g + 1) * 4096));
    } else {
      fn_n[2 * g - 4] = *reinterpret_cast<const half8*>(rst + ((b_base ^ (rks * 32)) + (2 * g - 4) * 4096));
      fn_n[2 * g - 3] = *reinterpret_cast<const half8*>(rst + ((b_base ^ (rks * 32)) + (2 * g - 3) * 4096));
    }
  };
#define MI355_ST_GROUP(g, fm, fn, rst, rks, fm_n, fn_n, W1, W2, LD) \
  do {                                                              \
    acc[g][0] = mfma16<BF>(fn[g], fm[0], acc[g][0]);             \
    W1;                                                             \
    __builtin_amdgcn_sched_barrier(0);                              \
    acc[g][1] = mfma16<BF>(fn[g], fm[1], acc[g][1]);             \
    W2;                                                             \
    __builtin_amdgcn_sched_barrier(0);                              \
    acc[g][2] = mfma16<BF>(fn[g], fm[2], acc[g][2]);             \
    LD;                                                             \
    __builtin_amdgcn_sched_barrier(0);                              \
    acc[g][3] = mfma16<BF>(fn[g], fm[3], acc[g][3]);             \
    frag_reads(g, rst, rks, fm_n, fn_n);                            \
    __builtin_amdgcn_sched_barrier(0);                              \
  } while (0)
#define MI355_NOP ((void)0)

  // Slab kt sits in stage P.  Set Q = 1 - P holds slab kt+1 (loaded during slab kt-2) and is copied to stage Q
  // register by register, each register reloaded with slab kt+3 once it is written out; set P is receiving
  // slab kt+2.  Loads in flight when register n is written: the rest of its own round (15 - n), the 16 of the
  // other set, and the G loads of this slab issued so far.
  // Past the end of the tile the loads belong to the next tile (branch-free: descriptors and slab index are selected).
  // W: 0 = exact waits; 1 = none -- used for the first two slabs behind an epilogue, where every staging register has
  // landed (the K loop ends with vmcnt(0)) and the only operations in flight are the epilogue's stores, which an
  // exact count would wait for.
#define MI355_ST_SLAB(P, Q, kt_, W)                                                                                        \
  do {                                                                                                                     \
    const char* st = lds + P * STAGE;                                                                                      \
    char* nst = lds + Q * STAGE;                                                                                           \
    const bool wrap_ = (kt_) + 3 >= KT;                                                                                    \
    const unsigned ko = (unsigned)(wrap_ ? (kt_) + 3 - KT : (kt_) + 3) * 128u;                                             \
    const i32x4 la = wrap_ ? a_nxt : a_src, lb = wrap_ ? b_nxt : b_src;                                                    \
    __builtin_amdgcn_sched_barrier(0);                                                                                     \
    MI355_ST_GROUP(0, fm0, fn0, st, 1, fm1, fn1, MI355_ST_WRITE(Q, 0, (W) ? 63 : 31, nst), MI355_ST_WRITE(Q, 1, (W) ? 63 : 30, nst), MI355_ST_LOAD(Q, 0, ko, la, lb));   \
    MI355_ST_GROUP(1, fm0, fn0, st, 1, fm1, fn1, MI355_ST_WRITE(Q, 2, (W) ? 63 : 30, nst), MI355_NOP, MI355_ST_LOAD(Q, 1, ko, la, lb));                                  \
    MI355_ST_GROUP(2, fm0, fn0, st, 1, fm1, fn1, MI355_ST_WRITE(Q, 3, (W) ? 63 : 30, nst), MI355_ST_WRITE(Q, 4, (W) ? 63 : 29, nst), MI355_ST_LOAD(Q, 2, ko, la, lb));   \
    MI355_ST_GROUP(3, fm0, fn0, st, 1, fm1, fn1, MI355_ST_WRITE(Q, 5, (W) ? 63 : 29, nst), MI355_NOP, MI355_ST_LOAD(Q, 3, ko, la, lb));                                  \
    MI355_ST_GROUP(0, fm1, fn1, st, 2, fm0, fn0, MI355_ST_WRITE(Q, 6, (W) ? 63 : 29, nst), MI355_ST_WRITE(Q, 7, (W) ? 63 : 28, nst), MI355_ST_LOAD(Q, 4, ko, la, lb));   \
    MI355_ST_GROUP(1, fm1, fn1, st, 2, fm0, fn0, MI355_ST_WRITE(Q, 8, (W) ? 63 : 28, nst), MI355_NOP, MI355_ST_LOAD(Q, 5, ko, la, lb));                                  \
    MI355_ST_GROUP(2, fm1, fn1, st, 2, fm0, fn0, MI355_ST_WRITE(Q, 9, (W) ? 63 : 28, nst), MI355_ST_WRITE(Q, 10, (W) ? 63 : 27, nst), MI355_ST_LOAD(Q, 6, ko, la, lb));  \
    MI355_ST_GROUP(3, fm1, fn1, st, 2, fm0, fn0, MI355_ST_WRITE(Q, 11, (W) ? 63 : 27, nst), MI355_NOP, MI355_ST_LOAD(Q, 7, ko, la, lb));                                 \
    MI355_ST_GROUP(0, fm0, fn0, st, 3, fm1, fn1, MI355_ST_WRITE(Q, 12, (W) ? 63 : 27, nst), MI355_NOP, MI355_ST_LOAD(Q, 8, ko, la, lb));                                 \
    MI355_ST_GROUP(1, fm0, fn0, st, 3, fm1, fn1, MI355_ST_WRITE(Q, 13, (W) ? 63 : 27, nst), MI355_NOP, MI355_ST_LOAD(Q, 9, ko, la, lb));                                 \
    MI355_ST_GROUP(2, fm0, fn0, st, 3, fm1, fn1, MI355_ST_WRITE(Q, 14, (W) ? 63 : 27, nst), MI355_NOP, MI355_ST_LOAD(Q, 10, ko, la, lb));                                \
    MI355_ST_GROUP(3, fm0, fn0, st, 3, fm1, fn1, MI355_ST_WRITE(Q, 15, (W) ? 63 : 27, nst), MI355_NOP, MI355_ST_LOAD(Q, 11, ko, la, lb));                                \
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");                                                                     \
    __syncthreads();                                                                                                       \
    __builtin_amdgcn_sched_barrier(0);                                                                                     \
    MI355_ST_GROUP(0, fm1, fn1, nst, 0, fm0, fn0, MI355_NOP, MI355_NOP, MI355_ST_LOAD(Q, 12, ko, la, lb));                 \
    MI355_ST_GROUP(1, fm1, fn1, nst, 0, fm0, fn0, MI355_NOP, MI355_NOP, MI355_ST_LOAD(Q, 13, ko, la, lb));                 \
    MI355_ST_GROUP(2, fm1, fn1, nst, 0, fm0, fn0, MI355_NOP, MI355_NOP, MI355_ST_LOAD(Q, 14, ko, la, lb));                 \
    MI355_ST_GROUP(3, fm1, fn1, nst, 0, fm0, fn0, MI355_NOP, MI355_NOP, MI355_ST_LOAD(Q, 15, ko, la, lb));                 \
  } while (0)

  const int G = (int)gridDim.x;
  for (; pid < T; pid += G) {
    int nxt_m = tile_m, nxt_n = tile_n;
    if (pid + G < T) {
      map_tile(pid + G, tiles_m, tiles_n, group_m, nxt_m, nxt_n);
      a_nxt = make_desc(A + (size_t)(nxt_m * BM + wave * 8) * K, (unsigned)(BM - wave * 8) * row_bytes);
      b_nxt = make_desc(B + (size_t)(nxt_n * BN + wave * 8) * K, (unsigned)(BN - wave * 8) * row_bytes);
    }
    MI355_ST_SLAB(0, 1, 0, 1);
    MI355_ST_SLAB(1, 0, 1, 1);
    for (int kt = 2; kt < KT; kt += 2) {
      MI355_ST_SLAB(0, 1, kt, 0);
      MI355_ST_SLAB(1, 0, kt + 1, 0);
    }
    // The staging registers now hold the next tile's slabs 1 and 2 (for the last tile: loads that are never used).
    // The code from here to the next slab is scheduled by the compiler, which does not know that such a register may
    // still be receiving its load: let every load land while nothing but the loads owns these registers.
    // The wait names every staging register as an input: the compiler has to keep them allocated to the loads up
    // to this point and cannot hand one to other code while its load (a speculative one past the last slab included)
    // is still in flight.
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::"v"(r[0][0]), "v"(r[0][1]), "v"(r[0][2]), "v"(r[0][3]), "v"(r[0][4]), "v"(r[0][5]), "v"(r[0][6]), "v"(r[0][7]), "v"(r[0][8]), "v"(r[0][9]), "v"(r[0][10]), "v"(r[0][11]), "v"(r[0][12]), "v"(r[0][13]), "v"(r[0][14]), "v"(r[0][15]) : "memory");
    asm volatile("" ::"v"(r[1][0]), "v"(r[1][1]), "v"(r[1][2]), "v"(r[1][3]), "v"(r[1][4]), "v"(r[1][5]), "v"(r[1][6]), "v"(r[1][7]), "v"(r[1][8]), "v"(r[1][9]), "v"(r[1][10]), "v"(r[1][11]), "v"(r[1][12]), "v"(r[1][13]), "v"(r[1][14]), "v"(r[1][15]) : "memory");

    // ---- epilogue of this tile, out of LDS that no stage uses (stage 0 already holds the next tile's slab 0) ----
    // Its addresses are derived from a lane id the compiler cannot see through, or it would compute all of them
    // ahead of the tile loop and keep them in registers that the K loop needs (it then spills to scratch).
    const int le = opaque_lane_id();
    const int r32e = le & 31, he = le >> 5;
    if constexpr (sizeof(OutT) == 2) {
      // 16-bit epilogue through a wave-private LDS region, one 32-row x 64-column piece (two accumulator tiles) per
      // pass: 8-byte writes of 4 consecutive n (chunk slot c ^ ((m >> 1) & 7) of the 128-byte row), whole rows read
      // back 16 bytes per lane and stored as full cache lines.  LDS operations of a wave execute in order, so the
      // passes need no waits between them.  Two tiles per pass, not four: the staging registers stay live across the
      // epilogue (they hold the next tile's slabs) and a wider pass would not fit the remaining registers.
      constexpr int ROW_B = 128;
      char* ep = lds + 2 * STAGE + wave * (32 * ROW_B);
      const int er = le >> 3, ec = le & 7;
      const buffer_rsrc_t c_dst = make_buffer(C + (size_t)(tile_m * BM + wm * WTM) * N + tile_n * BN + wn * WTN,
                                              (unsigned)(((WTM - 1) * (size_t)N + WTN) * 2));
      const int c_lane_off = (er * N + ec * 8) * 2;
#pragma unroll
      for (int j = 0; j < TM; j++) {
#pragma unroll
        for (int ip = 0; ip < TN / 2; ip++) {
#pragma unroll
          for (int ii = 0; ii < 2; ii++)
#pragma unroll
            for (int q = 0; q < 4; q++) {
              const int c = ii * 4 + q, i = 2 * ip + ii;
              half4 v = {cvt16<BF>(acc[i][j][4 * q]), cvt16<BF>(acc[i][j][4 * q + 1]), cvt16<BF>(acc[i][j][4 * q + 2]),
                         cvt16<BF>(acc[i][j][4 * q + 3])};
              *reinterpret_cast<half4*>(ep + r32e * ROW_B + ((c ^ ((r32e >> 1) & 7)) * 16) + 8 * he) = v;
            }
#pragma unroll
          for (int it = 0; it < 4; it++) {
            const int row = it * 8 + er;
            const u32x4 v = *reinterpret_cast<const u32x4*>(ep + row * ROW_B + ((ec ^ ((row >> 1) & 7)) * 16));
            // row j * 32 + it * 8 + er of the wave's 128 x 128 block, columns ip * 64 + ec * 8 .. + 7: one per-lane
            // offset for the whole epilogue, the rest in the scalar offset
            __builtin_amdgcn_raw_buffer_store_b128(v, c_dst, c_lane_off, ((j * 32 + it * 8) * N + ip * 64) * 2, 0);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
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
            OutPack<OutT, BF>::store4(crow + i * 32 + q * 8, acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2],
                                      acc[i][j][4 * q + 3]);
      }
    }
#pragma unroll
    for (int i = 0; i < TN; i++)
#pragma unroll
      for (int j = 0; j < TM; j++)
#pragma unroll
        for (int q = 0; q < 16; q++) acc[i][j][q] = 0.f;
    a_src = a_nxt;
    b_src = b_nxt;
    tile_m = nxt_m;
    tile_n = nxt_n;
    lane_offsets();
    // the next tile's first fragments, read again (stage 0 holds its slab 0): not carrying them across the epilogue
    // leaves the epilogue 32 more registers
    read_frags(lds, 0, fm0, fn0);
  }
#undef MI355_ST_SLAB
#undef MI355_ST_GROUP
#undef MI355_NOP
#undef MI355_ST_LOAD_ALL
#undef MI355_ST_WRITE
#undef MI355_ST_LOAD
}

// Streamed form: whole 128-byte rows of a 64-half slab go global -> LDS directly (8 rows per wave-load), and LDS is
// freed in pieces WITHIN a slab, so that loads run two slabs ahead in 160 KiB with no staging registers and no ds_write:
//  * the B fragments of a slab (128 rows x 64 halfs per wave = 16 registers of 8 halfs) are held in registers for the
//    whole slab and fetched from LDS during the first half of the slab before, so a B buffer is free half a slab after
//    its reads begin; three 32 KiB B buffers;
//  * the A rows are streamed: fragment (16 rows, 32 halfs) by fragment, each feeding 8 MFMAs 16x16x32 against the held
//    B fragments, read from LDS four steps (one interval) ahead; a block of 32 A rows per half is free one interval
//    after it was read; two 32 KiB A buffers, the loads of slab t + 2 follow the reads of slab t block by block.
// One step = 8 MFMAs (m block j = step / 2, k half = step % 2) + one A read + (first half of the slab) two B reads + one
// load; 16 steps per slab, a barrier every 4 steps (an interval).  At a barrier every wave has waited for its loads older
// than one slab and for its LDS reads older than one interval, which is what the reuse below relies on:
//   interval q of slab t loads   A: block q - 1 of slab t + 2 (q = 0: block 3 of slab t + 1)
//                                B: part q + 1 of slab t + 3 (q = 3: part 0 of slab t + 4)
// Reads and waits are inline assembly (with direct-to-LDS loads in flight the compiler would wait for all of them before
// any LDS read it can see); every read's destination is tied to the wait that covers it.
// K split (split_tiles_m > 0): the launch covers S = tiles_m / split_tiles_m partial products of K elements each, stacked
// along M -- tile row tm belongs to split tm / split_tiles_m, reads rows (tm % split_tiles_m) * 256 .. of A and the K
// range starting split * ksplit_bytes into every row of A and B, and writes rows tm * 256 .. of C, which the host
// points at an [S * M, N] workspace.  ldk is the row length of A and B in elements (= K without a split).
template <typename OutT, bool BF>
__global__ __launch_bounds__(256) void gemm_f16_nt_stream(const half_t* __restrict__ A, const half_t* __restrict__ B,
                                                          OutT* __restrict__ C, int ldk, int N, int K, int tiles_m, int tiles_n,
                                                          int group_m, int split_tiles_m, unsigned ksplit_bytes) {
  constexpr int BM = 256, BN = 256, WN = 2, WTM = 128, WTN = 128;
  constexpr int BUF = 256 * 128;                 // one operand, one slab
  constexpr int B_AT = 0, A_AT = 3 * BUF;        // three B buffers, then two A buffers
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave / WN, wn = wave % WN;
  // The workgroup walks tiles blockIdx.x, blockIdx.x + gridDim.x, ... as ONE slab sequence (launched with one workgroup
  // per tile it runs just that tile): loads for slabs past a tile's end fetch the next tile's first slabs, so only a
  // workgroup's first tile pays the pipeline fill, and a tile's stores drain under the next tile's MFMAs.
  const int T = tiles_m * tiles_n, G = (int)gridDim.x;
  int pid = blockIdx.x;
  int tile_m, tile_n;
  map_tile(pid, tiles_m, tiles_n, group_m, tile_m, tile_n);

  // global side: a wave-load covers 8 rows x 128 bytes; wave w loads rows 128 h + 32 blk + 8 w .. + 7 of either operand.
  // lane = (row l >> 3, slot l & 7) fetches chunk slot ^ ((row >> 1) & 7): the row's 8-row group index 16 h + 4 blk + w
  // has the parity of w
  // One descriptor per operand covers all of it (under 4 GiB, checked on the host); the tile, the slab and the row block
  // go into the scalar offset, so that moving on to the next tile changes one scalar.
  const unsigned row_bytes = (unsigned)ldk * 2u;
  const int a_tiles = split_tiles_m > 0 ? split_tiles_m : tiles_m;  // tile rows of A itself
  const buffer_rsrc_t a_src = make_buffer(A, (unsigned)(a_tiles * BM) * row_bytes);
  const buffer_rsrc_t b_src = make_buffer(B, (unsigned)(tiles_n * BN) * row_bytes);
  const int lrow = lane >> 3;
#if defined(MI355_ABLATE_PLAIN_LOAD_ORDER)   // timing only: the lanes of a row fetch its chunks in ascending order (LDS then holds the wrong layout)
  const unsigned g_off = (unsigned)(wave * 8 + lrow) * row_bytes + (unsigned)(lane & 7) * 16u;
#else
  const unsigned g_off = (unsigned)(wave * 8 + lrow) * row_bytes + (unsigned)((lane & 7) ^ (((wave & 1) << 2) | (lrow >> 1))) * 16u;
#endif
  const int KT = K / 64;  // even, >= 4 (checked on the host)
  // byte offsets of a tile's rows in A and B (with a K split: plus the split's K range)
  auto tile_offsets = [&](int tm, int tn, unsigned& a_at, unsigned& b_at) {
    unsigned k_at = 0;
    while (tm >= a_tiles) {  // at most S - 1 turns, none without a split
      tm -= a_tiles;
      k_at += ksplit_bytes;
    }
    a_at = (unsigned)(tm * BM) * row_bytes + k_at;
    b_at = (unsigned)(tn * BN) * row_bytes + k_at;
  };
  unsigned a_cur, b_cur;  // this tile's rows
  tile_offsets(tile_m, tile_n, a_cur, b_cur);
  unsigned a_nxt = a_cur, b_nxt = b_cur;  // the next tile's (after the last tile: its own again; those loads are never used)
  // byte offset of slab kt + d of the walk: past this tile's end it is a slab of the next tile
  auto slab_at = [&](int s, unsigned cur, unsigned nxt) { return s < KT ? cur + (unsigned)s * 128u : nxt + (unsigned)(s - KT) * 128u; };
  // offsets of the slabs 1, 2 (A) and 3, 4 (B) ahead of the current one; those of the next slab are worked out one per
  // step in the second half of a slab (scalar instructions bunched at a slab's start would hold up its first MFMAs)
  unsigned a_off1 = a_cur + 128u, a_off2 = a_cur + 256u, b_off3 = b_cur + 384u, b_off4 = b_cur + 512u;
  unsigned n_a1 = 0, n_a2 = 0, n_b3 = 0, n_b4 = 0;
  // rows 128 h + 32 blk (+ 8 wave) of the slab at byte offset `at` of operand X into the buffer at byte offset buf_at
  auto load = [&](bool is_a, int buf_at, int h, int blk, unsigned at) {
    const unsigned so = (unsigned)(h * 128 + blk * 32) * row_bytes + at;
#if defined(MI355_ABLATE_L1_LOADS)
    buffer_load_lds_16B(is_a ? a_src : b_src, (unsigned)lane * 16u, (so & 1024u) + (unsigned)(blockIdx.x & 31) * 4096u,
                        lds + buf_at + (h * 16 + blk * 4 + wave) * 1024);
#elif !defined(MI355_ABLATE_NO_LOADS)
    buffer_load_lds_16B(is_a ? a_src : b_src, g_off, so, lds + buf_at + (h * 16 + blk * 4 + wave) * 1024);
#endif
  };

  // fragment reads: lane l takes row l & 15 of a 16-row block, chunk 4 kh + (l >> 4) of the 128-byte row
  const int r16 = lane & 15, cq = lane >> 4;
  const unsigned lds0 = (unsigned)(uintptr_t)MI355_LDS(char, lds);
  const unsigned lane_rd = (unsigned)(r16 * 128 + ((cq ^ (r16 >> 1)) & 7) * 16);  // k half 1: ^ 64
  unsigned aaddr[2][2];  // [A buffer][k half]
#pragma unroll
  for (int bf = 0; bf < 2; bf++)
#pragma unroll
    for (int kh = 0; kh < 2; kh++) aaddr[bf][kh] = lds0 + A_AT + bf * BUF + wm * (WTM * 128) + (lane_rd ^ (kh * 64));
  const unsigned b_lane = lds0 + B_AT + wn * (WTN * 128) + lane_rd;
  unsigned baddr[2];  // [k half], of the B buffer being read in this slab

  // [n block][m block].  Never cleared: the first MFMA of a tile on each accumulator (slab 0, k half 0) takes a zero
  // addend instead -- a register write in front of an inline-assembly MFMA would need wait states the compiler does not
  // know to insert.
  floatx4 acc[8][8];
  half8 fb0[2][8], fb1[2][8], fa[8];

  // MFMAs as inline assembly with the accumulators pinned to AGPRs: with 64 four-register accumulators the compiler's
  // own allocation keeps moving some of them between the two register classes inside the loop.  No MFMA here reads an
  // accumulator written fewer than 8 MFMAs earlier, and nothing else touches the accumulators before the loop ends.
#define MI355_SM_MFMA(c, x, y)                                                                                  \
  do {                                                                                                          \
    if constexpr (BF) asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(x), "v"(y));       \
    else asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(x), "v"(y));                     \
  } while (0)
#define MI355_SM_ACC(ZERO, c, x, y)   \
  do {                                \
    if constexpr (ZERO) MI355_SM_MFMA0(c, x, y); \
    else MI355_SM_MFMA(c, x, y);      \
  } while (0)
#define MI355_SM_MFMA0(c, x, y)                                                                                 \
  do {                                                                                                          \
    if constexpr (BF) asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, 0" : "=a"(c) : "v"(x), "v"(y));        \
    else asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, 0" : "=a"(c) : "v"(x), "v"(y));                      \
  } while (0)
  // The first MFMA of a step together with the wait for the step's A fragment y (requested four steps earlier; LG = LDS
  // reads issued since).  One statement, with the fragment as a plain input: a separate wait statement that names it as
  // an output makes the compiler put a wait state in front of its next use.  All the statements involved are volatile
  // assembly, which keeps their order.
#define MI355_SM_ACCW(ZERO, LG, c, x, y)                                                                                         \
  do {                                                                                                                          \
    if constexpr (ZERO && BF) asm volatile("s_waitcnt lgkmcnt(%3)\n\tv_mfma_f32_16x16x32_bf16 %0, %1, %2, 0" : "=a"(c) : "v"(x), "v"(y), "n"(LG)); \
    else if constexpr (ZERO) asm volatile("s_waitcnt lgkmcnt(%3)\n\tv_mfma_f32_16x16x32_f16 %0, %1, %2, 0" : "=a"(c) : "v"(x), "v"(y), "n"(LG)); \
    else if constexpr (BF) asm volatile("s_waitcnt lgkmcnt(%3)\n\tv_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(x), "v"(y), "n"(LG)); \
    else asm volatile("s_waitcnt lgkmcnt(%3)\n\tv_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(x), "v"(y), "n"(LG)); \
  } while (0)
#define MI355_SM_READ(dst, addr, off) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(off))
#define MI355_SM_TIE8(X) "+v"(X[0]), "+v"(X[1]), "+v"(X[2]), "+v"(X[3]), "+v"(X[4]), "+v"(X[5]), "+v"(X[6]), "+v"(X[7])

  // ---- prologue: B0, A0, B1, A1 blocks 0..2, B2 ----
#pragma unroll
  for (int x = 0; x < 8; x++) load(false, B_AT, x & 1, x >> 1, b_cur);
#pragma unroll
  for (int x = 0; x < 8; x++) load(true, A_AT, x & 1, x >> 1, a_cur);
#pragma unroll
  for (int x = 0; x < 8; x++) load(false, B_AT + BUF, x & 1, x >> 1, b_cur + 128u);
#pragma unroll
  for (int x = 0; x < 6; x++) load(true, A_AT + BUF, x & 1, x >> 1, a_cur + 128u);
#pragma unroll
  for (int x = 0; x < 8; x++) load(false, B_AT + 2 * BUF, x & 1, x >> 1, b_cur + 256u);
  __builtin_amdgcn_sched_barrier(0);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  // everything has landed: a tile starts with all loads but those of the interval before it complete (later tiles: the
  // wait in the middle of the epilogue), and its first slab runs without load waits
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_sched_barrier(0);
  baddr[0] = b_lane;
  baddr[1] = b_lane ^ 64;
  MI355_SM_READ(fb0[0][0], baddr[0], 0 * 2048); MI355_SM_READ(fb0[0][1], baddr[0], 1 * 2048);
  MI355_SM_READ(fb0[0][2], baddr[0], 2 * 2048); MI355_SM_READ(fb0[0][3], baddr[0], 3 * 2048);
  MI355_SM_READ(fb0[0][4], baddr[0], 4 * 2048); MI355_SM_READ(fb0[0][5], baddr[0], 5 * 2048);
  MI355_SM_READ(fb0[0][6], baddr[0], 6 * 2048); MI355_SM_READ(fb0[0][7], baddr[0], 7 * 2048);
  MI355_SM_READ(fb0[1][0], baddr[1], 0 * 2048); MI355_SM_READ(fb0[1][1], baddr[1], 1 * 2048);
  MI355_SM_READ(fb0[1][2], baddr[1], 2 * 2048); MI355_SM_READ(fb0[1][3], baddr[1], 3 * 2048);
  MI355_SM_READ(fb0[1][4], baddr[1], 4 * 2048); MI355_SM_READ(fb0[1][5], baddr[1], 5 * 2048);
  MI355_SM_READ(fb0[1][6], baddr[1], 6 * 2048); MI355_SM_READ(fb0[1][7], baddr[1], 7 * 2048);
  MI355_SM_READ(fa[0], aaddr[0][0], 0); MI355_SM_READ(fa[1], aaddr[0][1], 0);
  MI355_SM_READ(fa[2], aaddr[0][0], 2048); MI355_SM_READ(fa[3], aaddr[0][1], 2048);
  asm volatile("s_waitcnt lgkmcnt(0)" : MI355_SM_TIE8(fb0[0]), MI355_SM_TIE8(fb0[1]), "+v"(fa[0]), "+v"(fa[1]), "+v"(fa[2]), "+v"(fa[3]));
  __builtin_amdgcn_s_barrier();  // every wave has read B0: its buffer may receive slab 3
  __builtin_amdgcn_sched_barrier(0);
  load(false, B_AT, 0, 0, b_cur + 384u);
  load(false, B_AT, 1, 0, b_cur + 384u);
  __builtin_amdgcn_sched_barrier(0);

  // B buffer rotation: slab t lives in buffer t % 3
  int b_rd = BUF;       // byte offset of the buffer read during this slab (slab t + 1)
  int b_ld012 = 0;      // buffer loaded in intervals 0..2 (slab t + 3)

  // Step s of a slab whose A buffer is PAR: MFMAs of (m block s / 2, k half s % 2) on fa[s % 8] against FB[s % 2][0..7].
  // LGKM = LDS reads issued after the read that filled fa[s % 8] (they may still be in flight).
#define MI355_SM_STEP(s, PAR, FB, FBN, LGKM, FIRST)                                                                              \
  do {                                                                                                                     \
    constexpr int s4 = (s) + 4, nb = s4 >= 16 ? 1 - (PAR) : (PAR), ns = s4 & 15;                                           \
    MI355_SM_ACCW(FIRST && !((s)&1), LGKM, acc[0][(s) >> 1], FB[(s)&1][0], fa[(s)&7]);                                     \
    MI355_SM_READ(fa[s4 & 7], aaddr[nb][ns & 1], (ns >> 1) * 2048);                                                        \
    __builtin_amdgcn_sched_barrier(0);                                                                                     \
    MI355_SM_ACC(FIRST && !((s)&1), acc[1][(s) >> 1], FB[(s)&1][1], fa[(s)&7]);                                      \
    if constexpr ((s) < 8) MI355_SM_READ(FBN[(s) >> 2][(2 * (s)) & 7], baddr[(s) >> 2], ((2 * (s)) & 7) * 2048);           \
    __builtin_amdgcn_sched_barrier(0);                                                                                     \
    MI355_SM_ACC(FIRST && !((s)&1), acc[2][(s) >> 1], FB[(s)&1][2], fa[(s)&7]);                                      \
    MI355_SM_ACC(FIRST && !((s)&1), acc[3][(s) >> 1], FB[(s)&1][3], fa[(s)&7]);                                      \
    if constexpr ((s) < 8) MI355_SM_READ(FBN[(s) >> 2][(2 * (s) + 1) & 7], baddr[(s) >> 2], ((2 * (s) + 1) & 7) * 2048);   \
    __builtin_amdgcn_sched_barrier(0);                                                                                     \
    MI355_SM_ACC(FIRST && !((s)&1), acc[4][(s) >> 1], FB[(s)&1][4], fa[(s)&7]);                                      \
    MI355_SM_ACC(FIRST && !((s)&1), acc[5][(s) >> 1], FB[(s)&1][5], fa[(s)&7]);                                      \
    {                                                                                                                      \
      constexpr int q = (s) >> 2, x = (s)&3;                                                                               \
      if constexpr (x < 2) {                                                                                               \
        if constexpr (q == 0) load(true, A_AT + (1 - (PAR)) * BUF, x, 3, a_off1);                                          \
        else load(true, A_AT + (PAR) * BUF, x, q - 1, a_off2);                                                             \
      } else {                                                                                                             \
        if constexpr (q == 3) load(false, B_AT + b_rd, x - 2, 0, b_off4);                                                  \
        else load(false, B_AT + b_ld012, x - 2, q + 1, b_off3);                                                            \
      }                                                                                                                    \
    }                                                                                                                      \
    __builtin_amdgcn_sched_barrier(0);                                                                                     \
    if constexpr ((s) == 8) n_a1 = slab_at(kt + 2, a_cur, a_nxt);                                                          \
    if constexpr ((s) == 9) n_a2 = slab_at(kt + 3, a_cur, a_nxt);                                                          \
    if constexpr ((s) == 10) n_b3 = slab_at(kt + 4, b_cur, b_nxt);                                                         \
    if constexpr ((s) == 11) n_b4 = slab_at(kt + 5, b_cur, b_nxt);                                                         \
    MI355_SM_ACC(FIRST && !((s)&1), acc[6][(s) >> 1], FB[(s)&1][6], fa[(s)&7]);                                      \
    MI355_SM_ACC(FIRST && !((s)&1), acc[7][(s) >> 1], FB[(s)&1][7], fa[(s)&7]);                                      \
    __builtin_amdgcn_sched_barrier(0);                                                                                     \
  } while (0)
  // End of an interval: loads older than one slab and LDS reads older than this interval are complete in every wave.
#define MI355_SM_SYNC(RD, VM)                                                    \
  do {                                                                           \
    if constexpr (VM) asm volatile("s_waitcnt vmcnt(" MI355_KLOOP_VMCNT_STR(16) ") lgkmcnt(%0)" ::"n"(RD) : "memory"); \
    else asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(RD) : "memory");             \
    MI355_KLOOP_BARRIER();                                                          \
    __builtin_amdgcn_sched_barrier(0);                                           \
  } while (0)
  // Reads issued in one step: 3 in the first half of a slab (A, B, B), 1 in the second.  The read that fills fa for
  // step s was the first read of step s - 4.
#define MI355_SM_SLAB(PAR, FB, FBN, VM, FIRST)                                                                            \
  do {                                                                                                          \
    baddr[0] = b_lane + (unsigned)b_rd;                                                                         \
    baddr[1] = baddr[0] ^ 64;                                                                                   \
    MI355_SM_STEP(0, PAR, FB, FBN, 3, FIRST);  /* steps 12..15 of the slab before: one read each */                    \
    MI355_SM_STEP(1, PAR, FB, FBN, 5, FIRST);                                                                          \
    MI355_SM_STEP(2, PAR, FB, FBN, 7, FIRST);                                                                          \
    MI355_SM_STEP(3, PAR, FB, FBN, 9, FIRST);                                                                          \
    MI355_SM_SYNC(12, VM);                                                                                        \
    MI355_SM_STEP(4, PAR, FB, FBN, 11, FIRST);                                                                         \
    MI355_SM_STEP(5, PAR, FB, FBN, 11, FIRST);                                                                         \
    MI355_SM_STEP(6, PAR, FB, FBN, 11, FIRST);                                                                         \
    MI355_SM_STEP(7, PAR, FB, FBN, 11, FIRST);                                                                         \
    MI355_SM_SYNC(12, VM);                                                                                        \
    MI355_SM_STEP(8, PAR, FB, FBN, 11, FIRST);                                                                         \
    MI355_SM_STEP(9, PAR, FB, FBN, 9, FIRST);                                                                          \
    MI355_SM_STEP(10, PAR, FB, FBN, 7, FIRST);                                                                         \
    MI355_SM_STEP(11, PAR, FB, FBN, 5, FIRST);                                                                         \
    MI355_SM_SYNC(4, VM);                                                                                        \
    MI355_SM_STEP(12, PAR, FB, FBN, 3, FIRST);                                                                         \
    MI355_SM_STEP(13, PAR, FB, FBN, 3, FIRST);                                                                         \
    MI355_SM_STEP(14, PAR, FB, FBN, 3, FIRST);                                                                         \
    MI355_SM_STEP(15, PAR, FB, FBN, 3, FIRST);                                                                         \
    /* the B fragments of the next slab were all requested in steps 0..7: they have landed; tie them to this point */ \
    if constexpr (VM) asm volatile("s_waitcnt vmcnt(" MI355_KLOOP_VMCNT_STR(16) ") lgkmcnt(4)" : MI355_SM_TIE8(FBN[0]), MI355_SM_TIE8(FBN[1])::"memory"); \
    else asm volatile("s_waitcnt lgkmcnt(4)" : MI355_SM_TIE8(FBN[0]), MI355_SM_TIE8(FBN[1])::"memory");         \
    MI355_KLOOP_BARRIER();                                                                                         \
    __builtin_amdgcn_sched_barrier(0);                                                                          \
    a_off1 = n_a1;                                                                                              \
    a_off2 = n_a2;                                                                                              \
    b_off3 = n_b3;                                                                                              \
    b_off4 = n_b4;                                                                                              \
    b_ld012 = b_rd;                                                                                             \
    b_rd = b_rd == 2 * BUF ? 0 : b_rd + BUF;                                                                    \
  } while (0)

  for (; pid < T; pid += G) {
    int nxt_m = tile_m, nxt_n = tile_n;
    if (pid + G < T) map_tile(pid + G, tiles_m, tiles_n, group_m, nxt_m, nxt_n);
    tile_offsets(nxt_m, nxt_n, a_nxt, b_nxt);
    int kt = 0;
    MI355_SM_SLAB(0, fb0, fb1, false, true);  // everything its reads need landed before the tile began
    kt = 1;
    MI355_SM_SLAB(1, fb1, fb0, true, false);
    for (kt = 2; kt < KT; kt += 2) {
      MI355_SM_SLAB(0, fb0, fb1, true, false);
      kt++;
      MI355_SM_SLAB(1, fb1, fb0, true, false);
      kt--;
    }
    // ---- epilogue ----
    // The MFMAs are inline assembly, so the compiler does not know that the accumulators were written just now: the
    // wait states an MFMA result needs before another instruction may read it are spelled out, and every accumulator is
    // tied to a statement behind them so that no read of it can be scheduled earlier.
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
#pragma unroll
    for (int i = 0; i < 8; i++)
      asm volatile("" : "+a"(acc[i][0]), "+a"(acc[i][1]), "+a"(acc[i][2]), "+a"(acc[i][3]), "+a"(acc[i][4]), "+a"(acc[i][5]),
                        "+a"(acc[i][6]), "+a"(acc[i][7]));
    // lane holds, for m = 16 j + (l & 15): n = 16 i + 4 (l >> 4) + r, r < 4.  The addresses come from a lane id the
    // compiler cannot see through, so that none of them is computed ahead of the K loop and kept across it.
    const int le = opaque_lane_id();
    const int r16e = le & 15, cqe = le >> 4;
    if constexpr (sizeof(OutT) == 2) {
      // 16-bit results go through LDS, one m block (16 rows x 128 columns = 4 KiB) per pass in a wave-private region:
      // 8-byte writes of 4 consecutive n (chunk slot c ^ ((m >> 1) & 7) within each 128-byte half row), whole rows read
      // back 16 bytes per lane and stored as full cache lines.  LDS operations of a wave execute in order, so the passes
      // need no waits between them.  The next tile's slabs are landing in LDS meanwhile; free at this point are parts
      // 1..3 of the B buffer whose part 0 was loaded in the interval before (rows 32..127 of either half: twice 12 KiB),
      // which the next loads reach only after the barrier below.
      // These LDS accesses are inline assembly like the K loop's: a direct-to-LDS load is in flight at this point, and
      // the compiler would wait for all of them in front of an LDS access it can see.
      const unsigned ep = lds0 + (unsigned)(B_AT + b_ld012 + (wave < 3 ? 4096 + wave * 4096 : 16 * 1024 + 4096));
      const int er = le >> 4, ec = le & 15, sw = (r16e >> 1) & 7;
      // write: row r16e, chunk (2 i + (cqe >> 1)) ^ sw, 8-byte half cqe & 1; the chunk's i term is an XOR of the address
      const unsigned wa = ep + (unsigned)(r16e * 256 + ((((cqe >> 1) ^ (sw & 1)) | (sw & 6)) * 16) + 8 * (cqe & 1));
      // read: row 4 it + er, chunk ec ^ ((row >> 1) & 7) = (ec ^ (er >> 1)) ^ 2 it
      const unsigned ra = ep + (unsigned)(er * 256 + ((ec ^ (er >> 1)) * 16));
      OutT* cbase = C + (size_t)(tile_m * BM + wm * WTM + er) * N + tile_n * BN + wn * WTN + ec * 8;
#pragma unroll
      for (int j = 0; j < 8; j++) {
#pragma unroll
        for (int i = 0; i < 8; i++) {
          half4 v = {cvt16<BF>(acc[i][j][0]), cvt16<BF>(acc[i][j][1]), cvt16<BF>(acc[i][j][2]), cvt16<BF>(acc[i][j][3])};
          asm volatile("ds_write_b64 %0, %1" ::"v"(wa ^ (unsigned)(32 * i)), "v"(v) : "memory");
        }
        half8 rv[4];
        asm volatile("ds_read_b128 %0, %1" : "=v"(rv[0]) : "v"(ra));
        asm volatile("ds_read_b128 %0, %1 offset:1024" : "=v"(rv[1]) : "v"(ra ^ 32u));
        asm volatile("ds_read_b128 %0, %1 offset:2048" : "=v"(rv[2]) : "v"(ra ^ 64u));
        asm volatile("ds_read_b128 %0, %1 offset:3072" : "=v"(rv[3]) : "v"(ra ^ 96u));
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(rv[0]), "+v"(rv[1]), "+v"(rv[2]), "+v"(rv[3]));
#pragma unroll
        for (int it = 0; it < 4; it++) store_global_16B(cbase + (size_t)(j * 16 + it * 4) * N, rv[it]);  // one instruction each
        if (j == 3) {
          // Half of the stores are out.  The next tile's first slab runs without load waits: everything it and the
          // first interval after it read was loaded before this tile's last interval, i.e. all but the 4 loads
          // issued since -- which are followed in the queue by the 16 store instructions above.
          asm volatile("s_waitcnt vmcnt(20)" ::: "memory");
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    } else {
      OutT* crow = C + (size_t)(tile_m * BM + wm * WTM + r16e) * N + tile_n * BN + wn * WTN + 4 * cqe;
#pragma unroll
      for (int j = 0; j < 8; j++) {
#pragma unroll
        for (int i = 0; i < 8; i++) {
          static_assert(sizeof(OutT) == 2 || sizeof(OutT) == 4, "16- or 32-bit output");
          const floatx4 v = {acc[i][j][0], acc[i][j][1], acc[i][j][2], acc[i][j][3]};
          store_global_16B(crow + (size_t)(j * 16) * N + i * 16, v);  // one instruction each
        }
        if (j == 3) asm volatile("s_waitcnt vmcnt(36)" ::: "memory");  // as above, behind 32 store instructions
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    a_cur = a_nxt;
    b_cur = b_nxt;
    tile_m = nxt_m;
    tile_n = nxt_n;
    // the waves leave the epilogue together: the first slab's reads rely on the wait above having been made by all
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
  }
  // the loads issued for a tile that does not exist still target LDS: let them land before the workgroup ends
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" : MI355_SM_TIE8(fa));
#undef MI355_SM_SLAB
#undef MI355_SM_SYNC
#undef MI355_SM_STEP
#undef MI355_SM_TIE8
#undef MI355_SM_READ
#undef MI355_SM_ACCW
#undef MI355_SM_ACC
#undef MI355_SM_MFMA0
#undef MI355_SM_MFMA
}

// Persistent kernel: one workgroup per CU walks its share of the output tiles (tile ids pid, pid + grid,
// ...) as ONE continuous sequence of K slabs.  The loads issued during the last two slabs of a tile
// already fetch the first two slabs of the next tile, the fragment reads at the end of the last slab
// already belong to the next tile, and the epilogue runs out of its own LDS region (one 32-row pass at a
// time), so its global stores drain while the next tile computes.
//
// Slab schedule (four k-steps of 16, one fragment register set each):
//   k-step 0: MFMAs of set 0   | LDS reads of sets 1 and 2
//   k-step 1: MFMAs of set 1   | LDS reads of set 3 (front-loaded)
//   wait + barrier: every wave has read the whole stage, the next slab has landed
//   k-step 2: MFMAs of set 2   | most global -> LDS loads of the slab after next (into the stage just read)
//   k-step 3: MFMAs of set 3   | LDS reads of set 0 of the next slab, remaining loads
// Reading a slab's last fragments one k-step early frees its stage half a slab sooner, so the loads
// spread over two k-steps instead of bunching behind the barrier, and they use buffer addressing
// (descriptor + per-lane offset + scalar offset): no vector address arithmetic in the loop.
template <int BM, int BN, int WM, int WN, typename OutT, bool BF>
__global__ __launch_bounds__(WM* WN * 64) void gemm_f16_nt_persistent(const half_t* __restrict__ A,
                                                                      const half_t* __restrict__ B,
                                                                      OutT* __restrict__ C, int M, int N, int K,
                                                                      int tiles_m, int tiles_n, int group_m) {
  constexpr int NW = WM * WN;
  constexpr int WTM = BM / WM, WTN = BN / WN;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int A_BYTES = BM * 128, B_BYTES = BN * 128, STAGE = A_BYTES + B_BYTES;
  constexpr int A_GROUPS = BM / 8, B_GROUPS = BN / 8;
  static_assert(A_GROUPS % NW == 0 && B_GROUPS % NW == 0 && NW % 2 == 0, "loads must split evenly over an even number of waves");
  constexpr int LA = A_GROUPS / NW, LB = B_GROUPS / NW;
  constexpr int EP_ROW = WTN * 2;        // bytes of one fp16 output row of a wave's tile
  constexpr int EP_WAVE = 32 * EP_ROW;   // one epilogue pass of a wave: 32 rows
  constexpr int EP_CH = EP_ROW / 16;     // 16-byte chunks per row
  constexpr int EP_RPB = EP_ROW >= 256 ? 1 : 256 / EP_ROW;  // rows per 256 bytes (= per sweep of the 64 banks)

  extern __shared__ __attribute__((aligned(1024))) char lds[];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave / WN, wn = wave % WN;
  const int T = tiles_m * tiles_n;
  const int G = gridDim.x;
  const int KT = K / 64;  // >= 2 (checked by the host)

  const int lrow = lane >> 3;
  const int lchunk = (lane & 7) ^ (((wave & 1) << 2) | (lrow >> 1));
  // byte offsets inside a tile's row panel: per lane (row of the 8-row group, swizzled chunk) and per
  // wave-load (8 * NW rows further down); the host keeps BM * K * 2 below 2^31
  const unsigned lane_off = ((unsigned)lrow * (unsigned)K + (unsigned)lchunk * 8u) * 2u;
  const unsigned row_step = (unsigned)NW * 8u * (unsigned)K * 2u;
  const unsigned panel_a = (unsigned)(BM - wave * 8) * (unsigned)K * 2u, panel_b = (unsigned)(BN - wave * 8) * (unsigned)K * 2u;

  // buffer descriptors over the rows of a tile that this wave copies (its first row onwards)
  auto tile_src = [&](int pid, buffer_rsrc_t& a_src, buffer_rsrc_t& b_src, int& tile_m, int& tile_n) {
    map_tile(pid, tiles_m, tiles_n, group_m, tile_m, tile_n);
    a_src = make_buffer(A + (size_t)(tile_m * BM + wave * 8) * K, panel_a);
    b_src = make_buffer(B + (size_t)(tile_n * BN + wave * 8) * K, panel_b);
  };
  // wave-loads FIRST .. LAST-1 of a slab (A groups first, then B groups)
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

  const int r32 = lane & 31, h = lane >> 5;
  const int sw = (h ^ ((r32 >> 1) & 7)) * 16;
  const int a_base = (wm * WTM + r32) * 128 + sw;
  const int b_base = A_BYTES + (wn * WTN + r32) * 128 + sw;
  auto read_frags = [&](const char* st, int ks, half8* fm, half8* fn) {
#pragma unroll
    for (int j = 0; j < TM; j++) fm[j] = *reinterpret_cast<const half8*>(st + ((a_base ^ (ks * 32)) + j * 4096));
#pragma unroll
    for (int i = 0; i < TN; i++) fn[i] = *reinterpret_cast<const half8*>(st + ((b_base ^ (ks * 32)) + i * 4096));
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
  auto mfmas = [&](const half8* fm, const half8* fn) {
#pragma unroll
    for (int i = 0; i < TN; i++)
#pragma unroll
      for (int j = 0; j < TM; j++) acc[i][j] = mfma16<BF>(fn[i], fm[j], acc[i][j]);
  };

  constexpr int NM = TM * TN;       // MFMAs per k-step
  constexpr int NR = TM + TN;       // fragment reads per k-step
  constexpr int NL = LA + LB;       // wave-loads per slab
  constexpr int NL2 = NL < NM ? (3 * NL) / 4 : NM - 2;  // loads issued in k-step 2
  static_assert(2 * NR <= 2 * NM && NR / 2 + 1 <= NM && NL - NL2 + (NR + 1) / 2 < NM, "k-step regions too small for their memory work");
  using I0 = std::integral_constant<int, 0>;
  using IL2 = std::integral_constant<int, NL2>;
  using IL = std::integral_constant<int, NL>;

  half8 fm0[TM], fn0[TN], fm1[TM], fn1[TN], fm2[TM], fn2[TN], fm3[TM], fn3[TN];

  int pid = blockIdx.x;
  if (pid >= T) return;
  buffer_rsrc_t a_src, b_src, a_nxt, b_nxt;
  int tile_m, tile_n, nxt_m, nxt_n;
  tile_src(pid, a_src, b_src, tile_m, tile_n);
  issue_loads(I0{}, IL{}, 0, a_src, b_src, 0);
  wait_vmcnt0();
  __syncthreads();
  issue_loads(I0{}, IL{}, 1, a_src, b_src, 1);
  read_frags(lds, 0, fm0, fn0);
  int v = 0;  // slabs retired so far: selects the LDS stage across tile boundaries

  for (; pid < T; pid += G) {
    // the tile after this one (the last tile "continues" into itself: its first slabs are fetched again
    // and never used)
    const int npid = pid + G < T ? pid + G : pid;
    tile_src(npid, a_nxt, b_nxt, nxt_m, nxt_n);

    for (int kt = 0; kt < KT; kt++, v++) {
      const char* st = lds + (v & 1) * STAGE;
      __builtin_amdgcn_sched_barrier(0);
      read_frags(st, 1, fm1, fn1);
      read_frags(st, 2, fm2, fn2);
      mfmas(fm0, fn0);
#pragma unroll
      for (int i = 0; i < (2 * NR) % NM; i++) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, (2 * NR) / NM + 1, 0);
      }
#pragma unroll
      for (int i = (2 * NR) % NM; i < NM; i++) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, (2 * NR) / NM, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
      read_frags(st, 3, fm3, fn3);
      mfmas(fm1, fn1);
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
      // loads of the slab after next (branch-free: past the end of this tile they are the next tile's
      // slabs 0 and 1)
      const bool wrap = kt + 2 >= KT;
      const int ls = wrap ? kt + 2 - KT : kt + 2;
      const buffer_rsrc_t la = wrap ? a_nxt : a_src, lb = wrap ? b_nxt : b_src;
      issue_loads(I0{}, IL2{}, v & 1, la, lb, ls);
      mfmas(fm2, fn2);
#pragma unroll
      for (int i = 0; i < NL2; i++) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x010, 1, 0);  // VMEM (direct-to-LDS load)
      }
      __builtin_amdgcn_sched_group_barrier(0x008, NM - NL2, 0);
      __builtin_amdgcn_sched_barrier(0);
      read_frags(lds + ((v + 1) & 1) * STAGE, 0, fm0, fn0);
      issue_loads(IL2{}, IL{}, v & 1, la, lb, ls);
      mfmas(fm3, fn3);
#pragma unroll
      for (int i = 0; i < (NR + 1) / 2; i++) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
      }
#pragma unroll
      for (int i = 0; i < NL - NL2; i++) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x010, 1, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, NM - (NR + 1) / 2 - (NL - NL2), 0);
      __builtin_amdgcn_sched_barrier(0);
    }

    // ---- epilogue of this tile; the next tile's first two slabs are already in flight ----
    if constexpr (sizeof(OutT) == 2) {
      // 32 rows per pass through a private region behind the two stages: ds_write_b64 of 4 consecutive n
      // (swizzled 16-byte chunk slots), whole rows read back 16 bytes per lane and stored as full lines.
      // LDS operations of a wave execute in order, so passes need no waits between them.
      char* ep = lds + 2 * STAGE + wave * EP_WAVE;
      constexpr int ROWS_PER_IT = 64 / EP_CH;
      const int er = lane / EP_CH, ec = lane % EP_CH;
      OutT* cbase = C + (size_t)(tile_m * BM + wm * WTM) * N + tile_n * BN + wn * WTN + ec * 8;
#pragma unroll
      for (int j = 0; j < TM; j++) {
#pragma unroll
        for (int i = 0; i < TN; i++)
#pragma unroll
          for (int q = 0; q < 4; q++) {
            const int c = i * 4 + q;
            half4 hv = {cvt16<BF>(acc[i][j][4 * q]), cvt16<BF>(acc[i][j][4 * q + 1]), cvt16<BF>(acc[i][j][4 * q + 2]),
                        cvt16<BF>(acc[i][j][4 * q + 3])};
            *reinterpret_cast<half4*>(ep + r32 * EP_ROW + ((c ^ ((r32 / EP_RPB) & (EP_CH - 1))) * 16) + 8 * h) = hv;
          }
#pragma unroll
        for (int it = 0; it < 32 / ROWS_PER_IT; it++) {
          const int row = it * ROWS_PER_IT + er;
          half8 ov = *reinterpret_cast<const half8*>(ep + row * EP_ROW + ((ec ^ ((row / EP_RPB) & (EP_CH - 1))) * 16));
          *reinterpret_cast<half8*>(cbase + (size_t)(j * 32 + row) * N) = ov;
        }
        __builtin_amdgcn_sched_barrier(0);  // one pass at a time: keeps the converted values of later passes out of registers
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
            OutPack<OutT, BF>::store4(crow + i * 32 + q * 8, acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2],
                                  acc[i][j][4 * q + 3]);
      }
    }
    zero_acc();
    a_src = a_nxt;
    b_src = b_nxt;
    tile_m = nxt_m;
    tile_n = nxt_n;
  }
  // the loads issued for a tile that does not exist still target LDS: let them land before the block ends
  wait_vmcnt0();
}

// Skinny-M kernel (M <= 32, the decode-shaped product): weight streaming, HBM bound.  One workgroup of 8 waves per
// 32 rows of B; wave w owns the 64-half K segments w, w + 8, ... of those rows and walks them through a private
// double buffer in LDS (2 x (4 KiB of B + 4 KiB of A)): the direct-to-LDS loads of segment j + 1 -- 8 rows x 128
// bytes per instruction for both operands -- are issued before segment j is consumed.  Rows of A past M repeat row
// M - 1 (same cache lines; their output columns are never stored).  The 8 partial 32 x 32 tiles are summed through
// LDS at the end.
// Nothing loaded is carried in registers across iterations, and the waits and the LDS fragment reads are inline
// assembly: with direct-to-LDS loads in flight the compiler waits for ALL of them before any LDS access it can
// see, which would serialise the two segments.  Loads return in order, so "at most the 8 loads of the next segment
// outstanding" means this one has landed.
template <typename OutT, bool BF>
__global__ __launch_bounds__(512) void gemm_f16_nt_skinny(const half_t* __restrict__ A, const half_t* __restrict__ B,
                                                          OutT* __restrict__ C, int M, int N, int K) {
  extern __shared__ __attribute__((aligned(16384))) char lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r32 = lane & 31, h = lane >> 5;
  const int n0 = blockIdx.x * 32;
  const int nseg = K >> 6;
  const int mine = wave < nseg ? (nseg - wave + 7) >> 3 : 0;  // segments of this wave
  char* my = lds + wave * 16384;
  const unsigned my_lds = (unsigned)(uintptr_t)MI355_LDS(char, my);

  floatx16 acc;
#pragma unroll
  for (int r = 0; r < 16; r++) acc[r] = 0.f;

  // global side of the loads: instruction i covers rows 8i .. 8i + 7, lane = (row, slot); the chunk it fetches is
  // slot ^ ((row >> 1) & 7), the swizzle of the tiled kernels
  const int lrow = lane >> 3;
  const half_t* b_src[4];
  const half_t* a_src[4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int row = i * 8 + lrow;
    const int chunk = (lane & 7) ^ ((row >> 1) & 7);
    b_src[i] = B + (size_t)(n0 + row) * K + chunk * 8;
    a_src[i] = A + (size_t)(row < M ? row : M - 1) * K + chunk * 8;
  }
  // fragment reads: row r32, chunk 2 * ks + h
  unsigned rd[4];
#pragma unroll
  for (int ks = 0; ks < 4; ks++) rd[ks] = my_lds + r32 * 128 + (((2 * ks + h) ^ ((r32 >> 1) & 7)) * 16);

  // The workgroups of an XCD start their sweep over K at different places: rows are 2 K bytes apart, so 256 workgroups
  // that all read the same offset of their 32 rows at the same time crowd a few memory channels (a plain read of the
  // same 128 MiB in this order: 27.6 us whatever the prefetch depth; with the start rotated by the workgroup's index
  // within its XCD: 23.2 us, as fast as a linear sweep; this kernel on 16 x 8192 x 8192: 31.2 -> 24.5 us).
  const int rot = mine > 0 ? (int)(blockIdx.x >> 3) % mine : 0;
  auto issue = [&](int j) {
    const int jr = j + rot < mine ? j + rot : j + rot - mine;
    const int seg = wave + 8 * jr;
    char* dst = my + (j & 1) * 8192;
#pragma unroll
    for (int i = 0; i < 4; i++) load_lds_16B(b_src[i] + seg * 64, dst + i * 1024);
#pragma unroll
    for (int i = 0; i < 4; i++) load_lds_16B(a_src[i] + seg * 64, dst + 4096 + i * 1024);
    __builtin_amdgcn_sched_barrier(0);
  };
  if (mine > 0) issue(0);
  for (int j = 0; j < mine; j++) {
    if (j + 1 < mine) {
      issue(j + 1);
      asm volatile("s_waitcnt vmcnt(8)");
    } else {
      asm volatile("s_waitcnt vmcnt(0)");
    }
    const unsigned bo = (unsigned)(j & 1) << 13;
    half8 fb[4], fa[4];
#pragma unroll
    for (int ks = 0; ks < 4; ks++) {
      asm volatile("ds_read_b128 %0, %1" : "=v"(fb[ks]) : "v"(rd[ks] + bo));
      asm volatile("ds_read_b128 %0, %1 offset:4096" : "=v"(fa[ks]) : "v"(rd[ks] + bo));
    }
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(fb[0]), "+v"(fb[1]), "+v"(fb[2]), "+v"(fb[3]), "+v"(fa[0]), "+v"(fa[1]), "+v"(fa[2]), "+v"(fa[3]));
#pragma unroll
    for (int ks = 0; ks < 4; ks++) acc = mfma16<BF>(fb[ks], fa[ks], acc);  // acc[n][m]
    __builtin_amdgcn_sched_barrier(0);
  }

  // reduce the 8 partial tiles: lane (m = r32, h) register r holds n = 8*(r/4) + 4h + r%4
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
  __syncthreads();
  // Tiles are stored [wave][m][n] with rows of 36 floats (a lane's registers 4 j .. 4 j + 3 are four consecutive n: 16-byte
  // writes), and the threads that add up one output element each read consecutive n.  With m as the fastest index every
  // read instruction hit one bank 32 times, and the eight waves' reads share the CU's LDS: about 3 us of the kernel.
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
    if (m < M) OutPack<OutT, BF>::store1(C + (size_t)m * N + n0 + n, v);
  }
}

// The skinny kernel for more than 32 rows in one launch (launches of the kernel above for 32 rows each would read the
// weights once each): the same decomposition and B path (segments through a private two-stage LDS ring), RB 32-row
// blocks of A, NW waves that split K.  A wave's LDS holds B's two stages (8 KiB) and ONE stage of A (RB x 4 KiB: two
// would not fit): the A segment j + 1 is requested as soon as the fragments of A segment j sit in registers, in front of
// the step's MFMAs, and comes out of L2 while they run and while the wave waits for B, which comes from memory and was
// requested a step earlier.  (A fragments loaded straight into registers, 32 lines per instruction instead of 8, made
// the load path the bottleneck: 64 x 8192 x 8192 in 43.5 us against 35.7.)  RB = 2 with 8 waves (33 to 64 rows, 128 KiB
// of LDS), RB = 4 with 4 waves (65 to 128 rows, 96 KiB).  Loads return in order, and a step's B loads are issued behind
// the A loads of the step before, so "at most the 4 newest loads outstanding" means B and A of this step have landed.
// Same rotation of the sweep's start.
template <typename OutT, bool BF, int RB, int NW>
__global__ __launch_bounds__(NW * 64) void gemm_f16_nt_skinny_rb(const half_t* __restrict__ A, const half_t* __restrict__ B,
                                                                OutT* __restrict__ C, int M, int N, int K) {
  constexpr int WAVE_LDS = 8192 + RB * 4096;  // B stage 0 | B stage 1 | A (RB x 4 KiB)
  constexpr int RED_PITCH = 36;
  static_assert(NW * WAVE_LDS <= 160 * 1024 && NW * 32 * RB * RED_PITCH * 4 <= NW * WAVE_LDS, "stages and the reduction fit");
  extern __shared__ __attribute__((aligned(16384))) char lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r32 = lane & 31, h = lane >> 5;
  const int n0 = blockIdx.x * 32;
  const int nseg = K >> 6;
  const int mine = wave < nseg ? (nseg - wave + NW - 1) / NW : 0;  // segments of this wave
  char* my = lds + wave * WAVE_LDS;
  const unsigned my_lds = (unsigned)(uintptr_t)MI355_LDS(char, my);

  floatx16 acc[RB];
#pragma unroll
  for (int b = 0; b < RB; b++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc[b][r] = 0.f;

  const int lrow = lane >> 3;
  const half_t* b_src[4];
  const half_t* a_src[4 * RB];
#pragma unroll
  for (int i = 0; i < 4 * RB; i++) {
    const int row = i * 8 + lrow;
    const int chunk = (lane & 7) ^ ((row >> 1) & 7);
    if (i < 4) b_src[i] = B + (size_t)(n0 + row) * K + chunk * 8;
    a_src[i] = A + (size_t)(row < M ? row : M - 1) * K + chunk * 8;
  }
  unsigned rd[4];
#pragma unroll
  for (int ks = 0; ks < 4; ks++) rd[ks] = my_lds + r32 * 128 + (((2 * ks + h) ^ ((r32 >> 1) & 7)) * 16);

  const int rot = mine > 0 ? (int)(blockIdx.x >> 3) % mine : 0;
  auto segment = [&](int j) {
    const int jr = j + rot < mine ? j + rot : j + rot - mine;
    return wave + NW * jr;
  };
  auto issue_b = [&](int j) {
    const int seg = segment(j);
    char* dst = my + (j & 1) * 4096;
#pragma unroll
    for (int i = 0; i < 4; i++) load_lds_16B(b_src[i] + seg * 64, dst + i * 1024);
    __builtin_amdgcn_sched_barrier(0);
  };
  auto issue_a = [&](int j) {
    const int seg = segment(j);
#pragma unroll
    for (int i = 0; i < 4 * RB; i++) load_lds_16B(a_src[i] + seg * 64, my + 8192 + i * 1024);
    __builtin_amdgcn_sched_barrier(0);
  };
  if (mine > 0) {
    issue_b(0);
    issue_a(0);
  }
  for (int j = 0; j < mine; j++) {
    if (j + 1 < mine) {
      issue_b(j + 1);
      asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
    } else {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    const unsigned bo = (unsigned)(j & 1) << 12;
    half8 fb[4], fa[RB][4];
#pragma unroll
    for (int ks = 0; ks < 4; ks++) {
      asm volatile("ds_read_b128 %0, %1" : "=v"(fb[ks]) : "v"(rd[ks] + bo));
#pragma unroll
      for (int b = 0; b < RB; b++) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(fa[b][ks]) : "v"(rd[ks]), "n"(8192 + 4096 * b));
    }
    // one wait for all of them; the fragments are named so that no use moves above it
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(fb[0]), "+v"(fb[1]), "+v"(fb[2]), "+v"(fb[3])::"memory");
#pragma unroll
    for (int b = 0; b < RB; b++) asm volatile("" : "+v"(fa[b][0]), "+v"(fa[b][1]), "+v"(fa[b][2]), "+v"(fa[b][3])::"memory");
    __builtin_amdgcn_sched_barrier(0);
    if (j + 1 < mine) issue_a(j + 1);  // the A stage is free: its fragments sit in registers
#pragma unroll
    for (int ks = 0; ks < 4; ks++)
#pragma unroll
      for (int b = 0; b < RB; b++) acc[b] = mfma16<BF>(fb[ks], fa[b][ks], acc[b]);  // acc[n][m]
    __builtin_amdgcn_sched_barrier(0);
  }

  // reduce the NW partial tiles of each row block, as above
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
  __syncthreads();
  float* red = reinterpret_cast<float*>(lds);  // [wave][m 32 RB][RED_PITCH]
#pragma unroll
  for (int b = 0; b < RB; b++)
#pragma unroll
    for (int q = 0; q < 4; q++) {
      const floatx4 v = {acc[b][4 * q], acc[b][4 * q + 1], acc[b][4 * q + 2], acc[b][4 * q + 3]};
      *reinterpret_cast<floatx4*>(red + (wave * 32 * RB + 32 * b + r32) * RED_PITCH + 8 * q + 4 * h) = v;
    }
  __syncthreads();
  for (int idx = threadIdx.x; idx < 1024 * RB; idx += NW * 64) {
    const int m = idx >> 5, n = idx & 31;
    float v = 0.f;
#pragma unroll
    for (int w = 0; w < NW; w++) v += red[(w * 32 * RB + m) * RED_PITCH + n];
    if (m < M) OutPack<OutT, BF>::store1(C + (size_t)m * N + n0 + n, v);
  }
}

// Any-shape kernel: 64x64 tile, 4 waves, bounds-checked staging through registers.  Used for
// shapes the tiled kernel does not divide (and as an independent implementation in tests).
template <typename OutT, bool BF>
__global__ __launch_bounds__(256) void gemm_f16_nt_generic(const half_t* __restrict__ A, const half_t* __restrict__ B,
                                                           OutT* __restrict__ C, int M, int N, int K) {
  constexpr int PITCH = 40;  // halfs per LDS row: 32 data + 8 pad keeps 16-byte alignment, spreads banks
  __shared__ __attribute__((aligned(16))) half_t sA[64 * PITCH];
  __shared__ __attribute__((aligned(16))) half_t sB[64 * PITCH];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int row0_m = blockIdx.y * 64, row0_n = blockIdx.x * 64;
  const int lr = tid >> 2, lk = (tid & 3) * 8;
  const bool vec_ok = (K % 8) == 0;
  floatx16 acc;
#pragma unroll
  for (int r = 0; r < 16; r++) acc[r] = 0.f;
  const int r32 = lane & 31, h = lane >> 5;

  for (int k0 = 0; k0 < K; k0 += 32) {
    half8 va, vb;
    {
      const int gm = row0_m + lr, gn = row0_n + lr, gk = k0 + lk;
      if (gm < M && vec_ok && gk + 8 <= K) {
        va = *reinterpret_cast<const half8*>(A + (size_t)gm * K + gk);
      } else {
#pragma unroll
        for (int e = 0; e < 8; e++) va[e] = (gm < M && gk + e < K) ? A[(size_t)gm * K + gk + e] : (half_t)0;
      }
      if (gn < N && vec_ok && gk + 8 <= K) {
        vb = *reinterpret_cast<const half8*>(B + (size_t)gn * K + gk);
      } else {
#pragma unroll
        for (int e = 0; e < 8; e++) vb[e] = (gn < N && gk + e < K) ? B[(size_t)gn * K + gk + e] : (half_t)0;
      }
    }
    __syncthreads();  // previous slab fully consumed
    *reinterpret_cast<half8*>(sA + lr * PITCH + lk) = va;
    *reinterpret_cast<half8*>(sB + lr * PITCH + lk) = vb;
    __syncthreads();
#pragma unroll
    for (int ks = 0; ks < 2; ks++) {
      half8 fm = *reinterpret_cast<const half8*>(sA + (wm * 32 + r32) * PITCH + ks * 16 + h * 8);
      half8 fn = *reinterpret_cast<const half8*>(sB + (wn * 32 + r32) * PITCH + ks * 16 + h * 8);
      acc = mfma16<BF>(fn, fm, acc);
    }
  }
  const int m = row0_m + wm * 32 + r32;
  if (m < M) {
#pragma unroll
    for (int r = 0; r < 16; r++) {
      const int n = row0_n + wn * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
      if (n < N) OutPack<OutT, BF>::store1(C + (size_t)m * N + n, acc[r]);
    }
  }
}

// ---- host side ----------------------------------------------------------------------------

// Sum of the S partial products of a K split (an [S * plane_rows, N] fp32 workspace, split s in rows s * plane_rows ..;
// plane_rows >= M: with a cut last tile row the planes hold whole tiles): four columns per lane, the partials added in
// split order, the sum converted as the kernels' own epilogues convert theirs.
template <typename OutT, bool BF>
__global__ __launch_bounds__(256) void gemm_ksplit_merge(const float* __restrict__ ws, OutT* __restrict__ C, int M, int N, int ldc,
                                                         int S, int plane_rows) {
  const size_t idx = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
  const size_t plane = (size_t)plane_rows * N;
  if (idx >= (size_t)M * N) return;
  floatx4 acc = *reinterpret_cast<const floatx4*>(ws + idx);
  for (int sp = 1; sp < S; sp++) acc += *reinterpret_cast<const floatx4*>(ws + sp * plane + idx);
  const size_t r = idx / (size_t)N, c = idx - r * (size_t)N;
  OutPack<OutT, BF>::store4(C + r * (size_t)ldc + c, acc[0], acc[1], acc[2], acc[3]);
}

struct GemmVariant {
  const char* name;
  int bm, bn, threads;
};
static const GemmVariant kGemmVariants[] = {
    {"persistent_256x256x64_w2x4", 256, 256, 512},
    {"pipelined_128x128x64_w2x2", 128, 128, 256},
    {"staged_256x256x64_w2x2", 256, 256, 256},
    {"skinny_m32_n32_w8", 32, 32, 512},
    {"stream_256x256x64_w2x2", 256, 256, 256},
    {"stream_256x256_tail_128x128", 256, 256, 256},
    {"stream_256x256x64_w2x2_walk", 256, 256, 256},
    {"pipelined_64x64x64_w2x2", 64, 64, 256},
    {"pipelined_128x64x64_w2x2", 128, 64, 256},
    {"pipelined_256x128x64_w2x2", 256, 128, 256},
    {"generic_64x64x32", 64, 64, 256},
};
// indices of the table above
enum { V_PERSISTENT = 0, V_PIPELINED_128 = 1, V_STAGED = 2, V_SKINNY = 3, V_STREAM = 4, V_STREAM_TAIL = 5, V_STREAM_WALK = 6,
       V_PIPELINED_64 = 7, V_PIPELINED_128x64 = 8, V_PIPELINED_256x128 = 9 };
constexpr int kNumGemmVariants = sizeof(kGemmVariants) / sizeof(kGemmVariants[0]);

int gemm_variant_count() { return kNumGemmVariants; }
const char* gemm_variant_name(int i) { return (i >= 0 && i < kNumGemmVariants) ? kGemmVariants[i].name : nullptr; }

// number of CUs of the device the stream's context is on (cached per device)
static int cu_count() {
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

// The pipelined kernel's slab form needs 128 bytes of LDS per tile row and column four times over: the 128x128 tile
// takes it when every workgroup has a CU to itself (with 320 tiles the lost co-residency costs 20 %), the smaller
// tiles (64 and 96 KiB: two and one workgroup per CU) always.
static bool pipelined_slab_form(long long tiles, int bm_plus_bn) { return bm_plus_bn != 256 || tiles <= 256; }

// Whether the workgroups of a tile column start their K sweep at another place (the kernel's krot_step): A at most 4 MiB
// (it stays in the L2s in any order), B at least 16 MiB (it streams).
static int pipelined_krot(long long M, long long N, long long K) { return M * K * 2 <= (4 << 20) && N * K * 2 >= (16 << 20); }

// RAGGED: M is any number of rows and N any multiple of 8 (the pipelined kernel's slab form only: the caller has
// checked pipelined_slab_form); C is then N columns wide (ldc == N)
template <int BM, int BN, int WM, int WN, typename OutT, int KIND, bool BF, bool RAGGED = false>  // KIND: 1 pipelined, 2 register-staged
static int launch_tiled(const void* a, const void* b, void* c, int M, int N, int K, int ldc, hipStream_t stream) {
  // the kernels use their N argument only as the row stride of C, so a column range of a wider C is the
  // same launch with ldc in its place
  static_assert(KIND == 1 || KIND == 2, "pipelined or register-staged");
  static_assert(!RAGGED || KIND == 1, "only the pipelined kernel cuts its last tile row");
  const int tiles_m = RAGGED ? (M + BM - 1) / BM : M / BM, tiles_n = RAGGED ? (N + BN - 1) / BN : N / BN;
  if (RAGGED && (ldc != N || N % 8)) return fail(-MI355_E_SHAPE, "gemm_f16_nt: a cut tile column needs N %% 8 == 0 and a C of N columns");
  int group_m = 4;
  dim3 grid(tiles_m * tiles_n), block(WM * WN * 64);
  if constexpr (KIND == 2) {
    // the register-staged kernel keeps its epilogue out of the stages: 32 rows x 128 bytes per wave
    constexpr int lds_bytes = 2 * (BM + BN) * 128 + WM * WN * 32 * 128;
    static std::atomic<uint64_t> lds_ok{0};
    auto kern = gemm_f16_nt_staged<BM, BN, WM, WN, OutT, BF>;
    if (int rc = allow_lds(reinterpret_cast<const void*>(kern), lds_bytes, lds_ok, "gemm_f16_nt")) return rc;
    hipLaunchKernelGGL(kern, grid, block, lds_bytes, stream, (const half_t*)a, (const half_t*)b, (OutT*)c, M, ldc, K, tiles_m,
                       tiles_n, group_m);
    return check_launch("gemm_f16_nt_staged", grid, block, lds_bytes);
  } else {
    auto go = [&](auto kern, int lds_bytes, std::atomic<uint64_t>& lds_ok) {
      if (int rc = allow_lds(reinterpret_cast<const void*>(kern), lds_bytes, lds_ok, "gemm_f16_nt")) return rc;
      hipLaunchKernelGGL(kern, grid, block, lds_bytes, stream, (const half_t*)a, (const half_t*)b, (OutT*)c, M, ldc, K, tiles_m,
                         tiles_n, group_m, K, 0, 0, pipelined_krot(M, N, K));
      return check_launch("gemm_f16_nt_pipelined", grid, block, lds_bytes);
    };
    static std::atomic<uint64_t> lds_ok2{0}, lds_ok4{0};
    constexpr int slab_stages = 4 * (BM + BN) * 128 <= 160 * 1024 ? 4 : 3;  // as the kernel picks them
    if constexpr (RAGGED) {
      static std::atomic<uint64_t> lds_okr{0};
      return go(gemm_f16_nt_pipelined<BM, BN, WM, WN, OutT, BF, true, true>, slab_stages * (BM + BN) * 128, lds_okr);
    }
    if (pipelined_slab_form((long long)tiles_m * tiles_n, BM + BN))
      return go(gemm_f16_nt_pipelined<BM, BN, WM, WN, OutT, BF, true>, slab_stages * (BM + BN) * 128, lds_ok4);
    if constexpr (BM + BN == 256) return go(gemm_f16_nt_pipelined<BM, BN, WM, WN, OutT, BF, false>, 2 * (BM + BN) * 128, lds_ok2);
    return fail(-MI355_E_SHAPE, "gemm_f16_nt: no k-step form of this tile");  // not reached: pipelined_slab_form
  }
}

// K split on the pipelined kernel, for products too small for 256x256 tiles to spread over the chip: S K ranges
// of k_part each, fp32 partial tiles stacked along M in the workspace (row pitch N).  ragged: any M, N % 8 == 0 (the
// slab form only); a range's partial products are then ceil(M / BM) whole tiles of rows, and the kernel takes M as the
// number of rows of A.
template <bool BF, int BM = 128, int BN = 128>
static int launch_pipelined_ksplit(const half_t* a, const half_t* b, float* ws, int M, int N, int K, int S, hipStream_t stream,
                                   bool ragged = false) {
  const int k_part = K / S;
  const int rows_of_tiles = ragged ? (M + BM - 1) / BM : M / BM;
  const int tiles_m = rows_of_tiles * S, tiles_n = ragged ? (N + BN - 1) / BN : N / BN;
  dim3 grid(tiles_m * tiles_n), block(256);
  auto go = [&](auto kern, int lds_bytes, std::atomic<uint64_t>& lds_ok) {
    if (int rc = allow_lds(reinterpret_cast<const void*>(kern), lds_bytes, lds_ok, "gemm_f16_nt")) return rc;
    hipLaunchKernelGGL(kern, grid, block, lds_bytes, stream, a, b, ws, ragged ? M : M * S, N, k_part, tiles_m, tiles_n, 4, K,
                       rows_of_tiles, k_part, pipelined_krot(M, N, K));
    return check_launch("gemm_f16_nt_pipelined (K split)", grid, block, lds_bytes);
  };
  static std::atomic<uint64_t> lds_ok2{0}, lds_ok4{0};
  if (ragged) {
    static std::atomic<uint64_t> lds_okr{0};
    if (N % 8 || !pipelined_slab_form(grid.x, BM + BN)) return fail(-MI355_E_SHAPE, "gemm_f16_nt: no K split with cut tiles for this shape");
    return go(gemm_f16_nt_pipelined<BM, BN, 2, 2, float, BF, true, true>, 4 * (BM + BN) * 128, lds_okr);
  }
  if (pipelined_slab_form(grid.x, BM + BN)) return go(gemm_f16_nt_pipelined<BM, BN, 2, 2, float, BF, true>, 4 * (BM + BN) * 128, lds_ok4);
  if constexpr (BM + BN == 256) return go(gemm_f16_nt_pipelined<BM, BN, 2, 2, float, BF, false>, 2 * (BM + BN) * 128, lds_ok2);
  return fail(-MI355_E_SHAPE, "gemm_f16_nt: no k-step form of this tile");  // not reached: pipelined_slab_form
}

template <int BM, int BN, int WM, int WN, typename OutT, bool BF>
static int launch_persistent(const void* a, const void* b, void* c, int M, int N, int K, hipStream_t stream) {
  auto kern = gemm_f16_nt_persistent<BM, BN, WM, WN, OutT, BF>;
  constexpr int lds_bytes = 2 * (BM + BN) * 128 + WM * WN * 32 * (BN / WN) * 2;  // two stages + one epilogue pass per wave
  static std::atomic<uint64_t> lds_ok{0};
  if (int rc = allow_lds(reinterpret_cast<const void*>(kern), lds_bytes, lds_ok, "gemm_f16_nt_persistent")) return rc;
  const int tiles_m = M / BM, tiles_n = N / BN;
  const int T = tiles_m * tiles_n;
  // one workgroup per CU (the LDS footprint allows no more), in multiples of 8 so that a workgroup's tile
  // ids pid + k * grid all fall on the XCD the hardware placed it on
  int g = cu_count() & ~7;
  if (g < 8) g = 8;
  dim3 grid(T < g ? T : g), block(WM * WN * 64);
  hipLaunchKernelGGL(kern, grid, block, lds_bytes, stream, (const half_t*)a, (const half_t*)b, (OutT*)c, M, N, K, tiles_m,
                     tiles_n, 4);
  return check_launch("gemm_f16_nt_persistent", grid, block, lds_bytes);
}

// ksplit > 1: M, N, K describe the whole product; c is an [ksplit * M, N] workspace of OutT = float partial products.
template <typename OutT, bool BF>
static int launch_stream(const void* a, const void* b, void* c, int M, int N, int K, int ldc, hipStream_t stream,
                         bool one_per_cu = false, int ksplit = 1) {
  auto kern = gemm_f16_nt_stream<OutT, BF>;
  constexpr int lds_bytes = 5 * 256 * 128;  // three B buffers and two A buffers of 32 KiB
  static std::atomic<uint64_t> lds_ok{0};
  if (int rc = allow_lds(reinterpret_cast<const void*>(kern), lds_bytes, lds_ok, "gemm_f16_nt_stream")) return rc;
  const int tiles_m = (M / 256) * ksplit, tiles_n = N / 256, k_part = K / ksplit;
  int wgs = tiles_m * tiles_n;
  // The walk looks up to five slabs ahead and knows one tile ahead: a tile needs six slabs or more.
  if (one_per_cu && k_part >= 384) {
    // one workgroup per CU walking tiles pid, pid + grid, ...; a multiple of 8 keeps a workgroup's tiles on its XCD
    int g = cu_count() & ~7;
    if (g < 8) g = 8;
    if (wgs > g) wgs = g;
  }
  dim3 grid(wgs), block(256);
  hipLaunchKernelGGL(kern, grid, block, lds_bytes, stream, (const half_t*)a, (const half_t*)b, (OutT*)c, K, ldc, k_part, tiles_m,
                     tiles_n, 4, ksplit > 1 ? M / 256 : 0, ksplit > 1 ? (unsigned)k_part * 2u : 0u);
  return check_launch("gemm_f16_nt_stream", grid, block, lds_bytes);
}

// Register-staged kernel with a finer-grained last round.  256x256 tiles go to the 256 CUs in rounds; when the
// last round would leave most CUs idle and its tiles form whole tile columns (or rows) of the grid, that
// strip is computed by the 128x128 kernel instead (four times the workgroups, so the strip spreads over the
// whole chip) in a second launch on the same stream.  Shapes that do not split this way run the staged
// kernel alone.
static bool tail_split(int M, int N, int& main_m, int& main_n) {
  const int tm = M / 256, tn = N / 256;
  const long long t = (long long)tm * tn;
  const int rem = (int)(t % 256);
  main_m = M;
  main_n = N;
  if (t <= 256 || rem == 0 || rem > 96) return false;  // one round, a full last round, or one that is busy enough
  if (rem % tm == 0) main_n = N - (rem / tm) * 256;
  else if (rem % tn == 0) main_m = M - (rem / tn) * 256;
  else return false;
  return true;
}

// K split: a product with too few 256x256 tiles for the 256 CUs is cut into S K ranges, every (tile, range) pair a unit
// of the streamed kernel's walk, fp32 partial products in a caller-provided workspace, one merge launch behind it.
// S doubles while the units still fit one round of the chip and a range keeps 1024 or more of K in whole slab pairs.
// The partial products cost a write and a read of 256 KiB per unit, so short K only splits when the units are few
// (measured, one tile's time in us for K = 4096 / 8192 against the 128x128 kernel: 64 tiles 47.8 / 70.1 against
// 45.5 / 82.7, 16 tiles 35.1 / 36.4 against 39.4 / 68.8, 128 tiles in two ranges 70.8 / 115.6 against 72.2 / 135.3).
static int ksplit_factor(long long tiles, int K) {
  if (K < 4096 || (K < 6144 && tiles > 32)) return 1;
  int s = 1;
  while (s < 8 && 2ll * s * tiles <= 256 && (K / (2 * s)) % 128 == 0 && K / (2 * s) >= 1024) s *= 2;
  return s;
}

template <typename OutT, bool BF>
static int launch_ksplit(const half_t* a, const half_t* b, OutT* c, int M, int N, int K, int ldc, int S, float* ws, hipStream_t stream) {
  if (int rc = launch_stream<float, BF>(a, b, ws, M, N, K, N, stream, true, S)) return rc;
  const long long lanes = (long long)M * N / 4;
  dim3 grid((unsigned)((lanes + 255) / 256)), block(256);
  hipLaunchKernelGGL((gemm_ksplit_merge<OutT, BF>), grid, block, 0, stream, (const float*)ws, c, M, N, ldc, S, M);
  return check_launch("gemm_ksplit_merge", grid, block, 0);
}

template <typename OutT, bool BF, int BM = 128, int BN = 128>
static int launch_ksplit128(const half_t* a, const half_t* b, OutT* c, int M, int N, int K, int ldc, int S, float* ws, hipStream_t stream,
                            bool ragged = false) {
  if (int rc = launch_pipelined_ksplit<BF, BM, BN>(a, b, ws, M, N, K, S, stream, ragged)) return rc;
  const long long lanes = (long long)M * N / 4;
  dim3 grid((unsigned)((lanes + 255) / 256)), block(256);
  hipLaunchKernelGGL((gemm_ksplit_merge<OutT, BF>), grid, block, 0, stream, (const float*)ws, c, M, N, ldc, S,
                     ragged ? (M + BM - 1) / BM * BM : M);
  return check_launch("gemm_ksplit_merge", grid, block, 0);
}

// K split on 128x128 tiles, for products that are small even for that: S doubles while the (tile, range) units still
// number <= 256 and a range keeps 512 of K (1024 beyond 64 units).  Measured against the 256x256 split and the plain
// kernels (us, graph-timed; best S in brackets): 256x256x8192 14.4 [16] against 30.3, 512x512x4096 15.2 [8] against 30.2,
// 512x1024x8192 22.6 [8] against 33.5, 1024x1024x4096 22.6 [4] against 33.9, 384x640x8192 18.7 [8] against 73.6; no gain
// from K = 1024, nor beyond 64 tiles except for 4096 <= K < 6144, where two ranges are level to ahead of the 256x256
// split (1024x2048x4096: 31.9 against 36.0).
static int ksplit128_factor(long long t128, int K) {
  if (K % 128 != 0) return 1;
  return (t128 > 128 && t128 <= 160 && K >= 4096 && K < 6144) ? 2 : 1;  // up to 128 tiles: small_plan below
}

// Products of at most 128 tiles of 128x128 (M * N <= 2 Mi): the tile shape and the K split that a cost model prices
// lowest.  These launches are bound by what their busiest CU moves through its LDS: per 64-wide slab a workgroup writes
// (BM + BN) * 128 bytes into LDS and its four waves read twice that back, at 128 bytes per clock: 0.15 us on a 64x64
// tile, 0.25 on 128x64, 0.42 on 128x128 (0.20 / 0.33 / 0.42 with all 256 CUs asking the L2s at once) against 0.05 /
// 0.11 / 0.21 us of MFMA work.  So the time of a launch is its fixed part (2.5 us: launch, first loads, epilogue) plus
// the operand bytes of its busiest CU at that rate, and what shortens it is more CUs at work: smaller tiles (more
// operand bytes in total, which the L2s serve) or K ranges (a merge launch: 2.3 us plus the partial tiles written and
// read at about 4.5 TB/s, half that beyond 8 MiB).  Against a sweep of 30 shapes (256^2 to 1408^2 and 1024x2048,
// K 512 to 8192, three tile shapes, 1 to 8 ranges, every plan timed) the model's times are within 15 % (median 4 %)
// and its choice within 4 % of the best measured plan.  1024^3: 10.4 -> 5.5 us (vendor library 7.8); 512x512x4096:
// 15.8 -> 9.6 (10.1); 1024x2048x2048: 18.3 -> 13.1 (15.9); 1024x1024x4096: 21.1 -> 15.3 (18.6).
// 129 to 256 tiles of 256x128 (257 to 512 of 128x128: more than one round of those, half a round of 256x256): one
// round of the pipelined kernel's 256x128 tile.  2048x2560x4096 59.5 (128x128) / 72.1 (256x256) -> 54.1 us, 2048x4096x4096
// 75.8 / 77.7 -> 67.2, 1024x8192x2048 40.7 / 44.6 -> 38.0 (vendor library 48.3, 66.4, 38.0); level with the K split on
// 256x256 tiles at K = 8192.  Short K as well: 2048x4096x1024 22.9 (128x128) / 26.3 (256x256) -> 21.5 us, 1024x8192x512
// 14.2 / 17.0 -> 14.1, 2048x2560x256 8.7 / 11.1 -> 8.5.
static bool takes_256x128(int64_t M, int64_t N, int64_t K) {
  if (M % 256 || N % 128 || K % 64 || K < 256 || K >= 8192) return false;
  const int64_t units = (M / 256) * (N / 128);
  return units > 128 && units <= 256;
}

struct SmallPlan {
  int bm = 0, bn = 0, S = 1;  // bm == 0: not a small product
  bool ragged = false;        // M is no multiple of bm or N none of bn: the last tile row or column is cut
  int64_t ws_bytes() const { return S > 1 ? (int64_t)S * plane_rows * cols * 4 : 0; }
  int64_t plane_rows = 0, cols = 0;  // rows (whole tiles) and columns of one K range's partial products
};
static SmallPlan small_plan(int64_t M, int64_t N, int64_t K, int64_t ws_bytes) {
  SmallPlan best;
  // any number of rows, any multiple of 8 columns (a cut last tile row or column costs what a whole one does, and
  // nothing is padded or copied)
  if (N % 8 || K % 64 || ((M + 63) / 64 * 64) * ((N + 63) / 64 * 64) > (1ll << 21) || K > (1 << 21)) return best;
  double best_us = 0;
  static const int kTiles[3][2] = {{64, 64}, {128, 64}, {128, 128}};
  for (const auto& t : kTiles) {
    const int bm = t[0], bn = t[1];
    const bool ragged = M % bm != 0 || N % bn != 0;
    const int64_t tiles = ((M + bm - 1) / bm) * ((N + bn - 1) / bn);
    const int64_t plane_rows = (M + bm - 1) / bm * bm;  // a cut tile row's partial products are whole tiles
    for (int S = 1; S <= 8; S *= 2) {
      const int64_t units = tiles * S, k_part = K / S;
      if (units > 512 || K % (64 * S)) break;
      if (ragged && !pipelined_slab_form(units, bm + bn)) break;  // cut tiles: the slab form only
      if (S > 1 && (k_part < 512 || S * plane_rows * N * 4 > ws_bytes)) break;
      const double per_cu_kib = (double)((units + 255) / 256) * (bm + bn) * 2 * k_part / 1024.0;
      double us_per_kib;
      if (bm + bn == 256) us_per_kib = pipelined_slab_form(units, 256) ? 0.013 : 0.0188;
      else us_per_kib = 0.0095 + 0.0035 * (units <= 128 ? 0.0 : units >= 256 ? 1.0 : (units - 128) / 128.0);
      double us = 2.5 + per_cu_kib * us_per_kib;
      if (S > 1) {
        const double partial_bytes = (double)S * plane_rows * N * 8;
        us += 2.3 + partial_bytes / 4.5e6 + (partial_bytes > (8 << 20) ? (partial_bytes - (8 << 20)) / 4.5e6 : 0.0);
      }
      if (best.bm == 0 || us < best_us) {
        best_us = us;
        best.bm = bm, best.bn = bn, best.S = S, best.ragged = ragged, best.plane_rows = plane_rows, best.cols = N;
      }
    }
  }
  return best;
}
static int ksplit128_plan(int M, int N, int K) {
  if (M % 128 || N % 128) return 1;
  return ksplit128_factor((long long)(M / 128) * (N / 128), K);
}

// The sub-problem that would take a K split on 256x256 tiles under the automatic choice, if any: the strip a sparse
// last round is cut into, or the whole product when it has at most 128 tiles (and the 128x128 split above does not
// take it).  Returns S (1: none) and the sub-problem's M and N.
static int ksplit_plan(int M, int N, int K, int& sub_m, int& sub_n) {
  sub_m = M;
  sub_n = N;
  if (M % 256 || N % 256) return 1;
  const long long t256 = (long long)(M / 256) * (N / 256);
  int mm, mn;
  if (t256 > 128) {
    if (!tail_split(M, N, mm, mn)) return 1;
    if (mn < N) sub_n = N - mn;
    else sub_m = M - mm;
    return ksplit_factor((long long)(sub_m / 256) * (sub_n / 256), K);
  }
  if (ksplit128_plan(M, N, K) > 1) return 1;
  return t256 >= 1 ? ksplit_factor(t256, K) : 1;
}

template <typename OutT, bool BF>
static int launch_split(const void* a, const void* b, void* c, int M, int N, int K, hipStream_t stream, float* ws = nullptr,
                        size_t ws_bytes = 0) {
  auto main_part = [&](int m, int n) { return launch_stream<OutT, BF>(a, b, c, m, n, K, N, stream, true); };  // one workgroup per CU
  const half_t* ah = (const half_t*)a;
  const half_t* bh = (const half_t*)b;
  OutT* ch = (OutT*)c;
  int mm, mn;
  if (!tail_split(M, N, mm, mn)) {
    int sm, sn;
    const int S = ws ? ksplit_plan(M, N, K, sm, sn) : 1;
    if (S > 1 && ws_bytes >= (size_t)S * M * N * 4) return launch_ksplit<OutT, BF>(ah, bh, ch, M, N, K, N, S, ws, stream);
    return main_part(M, N);
  }
  int rc = main_part(mm, mn);
  if (rc) return rc;
  // the strip: K split over 256x256 tiles when the caller brought a workspace, else the 128x128 kernel
  const int sm = mn < N ? M : M - mm, sn = mn < N ? N - mn : N;
  const half_t* sa = mn < N ? ah : ah + (size_t)mm * K;
  const half_t* sb = mn < N ? bh + (size_t)mn * K : bh;
  OutT* sc = mn < N ? ch + mn : ch + (size_t)mm * N;
  const int S = ws ? ksplit_factor((long long)(sm / 256) * (sn / 256), K) : 1;
  if (S > 1 && ws_bytes >= (size_t)S * sm * sn * 4) return launch_ksplit<OutT, BF>(sa, sb, sc, sm, sn, K, N, S, ws, stream);
  return launch_tiled<128, 128, 2, 2, OutT, 1, BF>(sa, sb, sc, sm, sn, K, N, stream);
}

template <typename OutT, bool BF>
static int launch_variant(int variant, const void* a, const void* b, void* c, int M, int N, int K, hipStream_t stream,
                          float* ws = nullptr, size_t ws_bytes = 0) {
  switch (variant) {
    case V_PERSISTENT: return launch_persistent<256, 256, 2, 4, OutT, BF>(a, b, c, M, N, K, stream);
    case V_PIPELINED_128: return launch_tiled<128, 128, 2, 2, OutT, 1, BF>(a, b, c, M, N, K, N, stream);
    case V_STAGED: return launch_tiled<256, 256, 2, 2, OutT, 2, BF>(a, b, c, M, N, K, N, stream);
    case V_SKINNY: {
      auto kern = gemm_f16_nt_skinny<OutT, BF>;
      constexpr int lds_bytes = 8 * 16384;
      static std::atomic<uint64_t> lds_ok{0};
      if (int rc = allow_lds(reinterpret_cast<const void*>(kern), lds_bytes, lds_ok, "gemm_f16_nt_skinny")) return rc;
      dim3 grid(N / 32), block(512);
      if (M > 64) {  // 65 to 128 rows: four row blocks, four waves
        auto kern = gemm_f16_nt_skinny_rb<OutT, BF, 4, 4>;
        constexpr int lds128 = 4 * (8192 + 4 * 4096);
        static std::atomic<uint64_t> lds_ok128{0};
        if (int rc = allow_lds(reinterpret_cast<const void*>(kern), lds128, lds_ok128, "gemm_f16_nt_skinny_rb")) return rc;
        hipLaunchKernelGGL(kern, grid, dim3(256), lds128, stream, (const half_t*)a, (const half_t*)b, (OutT*)c, M, N, K);
        return check_launch("gemm_f16_nt_skinny_rb", grid, dim3(256), lds128);
      }
      if (M > 32) {  // 33 to 64 rows: two row blocks, eight waves; the weights are read once
        auto kern64 = gemm_f16_nt_skinny_rb<OutT, BF, 2, 8>;
        static std::atomic<uint64_t> lds_ok64{0};
        if (int rc = allow_lds(reinterpret_cast<const void*>(kern64), lds_bytes, lds_ok64, "gemm_f16_nt_skinny_rb")) return rc;
        hipLaunchKernelGGL(kern64, grid, block, lds_bytes, stream, (const half_t*)a, (const half_t*)b, (OutT*)c, M, N, K);
        return check_launch("gemm_f16_nt_skinny_rb", grid, block, lds_bytes);
      }
      for (int m0 = 0; m0 < M; m0 += 32) {
        const int rows = M - m0 < 32 ? M - m0 : 32;
        hipLaunchKernelGGL(kern, grid, block, lds_bytes, stream, (const half_t*)a + (size_t)m0 * K, (const half_t*)b,
                           (OutT*)c + (size_t)m0 * N, rows, N, K);
        if (int rc = check_launch("gemm_f16_nt_skinny", grid, block, lds_bytes)) return rc;
      }
      return 0;
    }
    case V_STREAM: return launch_stream<OutT, BF>(a, b, c, M, N, K, N, stream);
    case V_STREAM_TAIL: return launch_split<OutT, BF>(a, b, c, M, N, K, stream, ws, ws_bytes);
    case V_STREAM_WALK: return launch_stream<OutT, BF>(a, b, c, M, N, K, N, stream, true);
    case V_PIPELINED_64: return launch_tiled<64, 64, 2, 2, OutT, 1, BF>(a, b, c, M, N, K, N, stream);
    case V_PIPELINED_128x64: return launch_tiled<128, 64, 2, 2, OutT, 1, BF>(a, b, c, M, N, K, N, stream);
    case V_PIPELINED_256x128: return launch_tiled<256, 128, 2, 2, OutT, 1, BF>(a, b, c, M, N, K, N, stream);
    default: {
      dim3 grid((N + 63) / 64, (M + 63) / 64), block(256);
      hipLaunchKernelGGL((gemm_f16_nt_generic<OutT, BF>), grid, block, 0, stream, (const half_t*)a, (const half_t*)b, (OutT*)c,
                         M, N, K);
      return check_launch("gemm_f16_nt_generic", grid, block, 0);
    }
  }
}

}  // namespace mi355

using namespace mi355;

// Many rows that are no multiple of the 256-row tile (and more than one round of smaller tiles covers): the automatic
// choice runs the multiple of 256 and the remainder as two products on row ranges of A and C.  Against padded copies
// of A and of the result: 4100x4096x4096 162 -> 110 us, 9000x8192x2048 321 -> 243, 5000x8192x8192 598 -> 517.
// whether a product of M rows (any number) against N % 8 == 0, K % 64 == 0 is one the tiled or weight-streaming kernels
// take whole: the small-product rule, one round of 128x128 or of 256x128 tiles, or up to 128 rows of a decode shape
static bool one_round_of_rows(int64_t M, int64_t N, int64_t K) {
  if (((M + 63) / 64 * 64) * ((N + 63) / 64 * 64) <= (1ll << 21)) return true;
  if ((M + 127) / 128 * ((N + 127) / 128) <= 256) return true;
  if (K >= 256 && K < 8192 && (M + 255) / 256 * ((N + 127) / 128) <= 256) return true;
  return M <= 128 && N % 32 == 0 && N >= 2048 && K >= 512;
}
static bool splits_rows(int64_t M, int64_t N, int64_t K) {
  if (M < 512 || M % 256 == 0 || N % 128 || K % 64) return false;
  return !one_round_of_rows(M, N, K) && one_round_of_rows(M % 256, N, K);  // the remainder must have a fast kernel
}

// fp16 and bf16 share everything but the kernel instantiation; `bf` also names the 16-bit output format
static int gemm_nt_entry(bool bf, const void* a, const void* b, void* c, int64_t M, int64_t N, int64_t K, int out_dtype, int variant,
                         void* stream, void* workspace = nullptr, int64_t workspace_bytes = 0) {
  if (!a || !b || !c) return fail(-MI355_E_NULL, "gemm_f16_nt: null pointer (a=%p b=%p c=%p)", a, b, c);
  if (M <= 0 || N <= 0 || K <= 0 || M > (1 << 30) || N > (1 << 30) || K > (1 << 27))
    return fail(-MI355_E_SHAPE, "gemm_f16_nt: bad shape M=%lld N=%lld K=%lld", (long long)M, (long long)N, (long long)K);
  if (out_dtype != MI355_F32 && out_dtype != (bf ? MI355_BF16 : MI355_F16))
    return fail(-MI355_E_DTYPE, "gemm_f16_nt: out_dtype %d (want MI355_F32 or %s)", out_dtype, bf ? "MI355_BF16" : "MI355_F16");
  if (variant >= kNumGemmVariants) return fail(-MI355_E_DTYPE, "gemm_f16_nt: variant %d out of range", variant);
  const bool al = aligned16(a) && aligned16(b) && aligned16(c);
  auto fits = [&](int v) {
    if (v == kNumGemmVariants - 1) return true;
    const bool streamed = v == V_STREAM || v == V_STREAM_TAIL || v == V_STREAM_WALK;
    if (v == V_PERSISTENT && (K < 128 || K > (1 << 21))) return false;  // prefetches two slabs ahead; 32-bit byte offsets inside a 256-row panel
    if (v == V_STAGED && N > (1 << 22)) return false;  // 32-bit byte offsets inside a wave's 128 rows of C
    if (v == V_STAGED && (K < 256 || K % 128 != 0 || K > (1 << 21))) return false;  // slabs in pairs, three in flight
    // the streamed kernel addresses each operand through one buffer descriptor
    if (streamed && (M * K * 2 >= (1ll << 32) || N * K * 2 >= (1ll << 32))) return false;
    if (streamed && (K < 256 || K % 128 != 0 || K > (1 << 21))) return false;  // slabs in pairs; 32-bit byte offsets inside a 256-row panel
    if (v == V_SKINNY) return al && M <= 128 && N % 32 == 0 && K % 64 == 0;  // a tile is 32 rows of B; 64-half K segments
    return al && M % kGemmVariants[v].bm == 0 && N % kGemmVariants[v].bn == 0 && K % 64 == 0;
  };
  if (variant < 0 && al && splits_rows(M, N, K)) {
    const int64_t m0 = M / 256 * 256;
    const size_t out_bytes = out_dtype == MI355_F32 ? 4 : 2;
    if (int rc = gemm_nt_entry(bf, a, b, c, m0, N, K, out_dtype, -1, stream, workspace, workspace_bytes)) return rc;
    return gemm_nt_entry(bf, static_cast<const char*>(a) + (size_t)m0 * K * 2, b, static_cast<char*>(c) + (size_t)m0 * N * out_bytes,
                         M - m0, N, K, out_dtype, -1, stream, workspace, workspace_bytes);
  }
  int split128 = 1;  // K ranges of the 128x128 split, when the automatic choice takes it
  SmallPlan small;   // tile shape and K ranges of a small product, when the automatic choice takes it
  int cut_rows = 0;  // 1 / 2: a product beyond the small rule on 128x128 / 256x128 tiles with a cut last tile row or column
  if (variant < 0) {
    // Large problems take the 256x256 tile; when that leaves most of the 256 CUs idle the
    // 128x128 tile (4x the workgroups) wins; everything else goes to the bounds-checked kernel.
    const long long t256 = (M / 256) * (N / 256);
    const long long rounds = (t256 + 255) / 256;  // 256 CUs, one 256x256 workgroup each
    // The streamed kernel with its sparse last round cut off from K = 1024 up: 8192^3 1460 against 1295
    // TFLOP/s for the register-staged kernel and 1285 for the persistent one, 4096^3 1405 / 1240 / 1244,
    // 2048x10240x8192 1285 / 1180 / 1044, 8192x8192x1024 1174 / 1064 / 1167.  Shorter K: the persistent kernel, which
    // hides each tile's prologue and epilogue under its neighbours (8192x8192x512: 978 against 854), as long as its
    // last round is >= 85% busy.
    const bool full_rounds = t256 * 100 >= rounds * 256 * 85;
    const int s128 = (workspace && fits(V_PIPELINED_128)) ? ksplit128_plan((int)M, (int)N, (int)K) : 1;
    // decode-shaped: stream the weights once.  Up to 64 rows always; 65 to 128 rows when M is no multiple of 64 (such
    // products went to the bounds-checked kernel: 65 x 8192 x 8192 149 -> 36.5 us; at 128 rows the 64x64 tiles of the
    // small-product rule are ahead, 43.9 against 47.9 us, and far ahead with many columns).
    if (fits(V_SKINNY) && (M <= 64 || M % 64 != 0) && N >= 2048 && K >= 512) variant = V_SKINNY;
    else if (al && (small = small_plan(M, N, K, INT64_MAX)).bm) {
      // a workspace short of what the plan asks for is no workspace (not a plan with fewer ranges)
      if (small.S > 1 && (!workspace || workspace_bytes < small.ws_bytes())) small = small_plan(M, N, K, 0);
      variant = small.bm == 64 ? V_PIPELINED_64 : small.bn == 64 ? V_PIPELINED_128x64 : V_PIPELINED_128;
    }
    else if (al && takes_256x128(M, N, K)) variant = V_PIPELINED_256x128;
    else if (s128 > 1 && workspace_bytes >= (int64_t)s128 * M * N * 4) {  // a small product: K split on 128x128 tiles
      variant = V_PIPELINED_128;
      split128 = s128;
    }
    // any number of rows and any multiple of 8 columns beyond the small rule, as long as one round of workgroups covers
    // the product: the last tile row and column of 128x128 tiles (up to 256 of them) or of 256x128 tiles (129 to 256)
    // are cut inside the kernel
    else if (al && N % 8 == 0 && K % 64 == 0 && (M % 128 != 0 || N % 128 != 0) && ((M + 127) / 128) * ((N + 127) / 128) <= 256) {
      variant = V_PIPELINED_128;
      cut_rows = 1;
    } else if (al && N % 8 == 0 && K % 64 == 0 && (M % 256 != 0 || N % 128 != 0) && K >= 256 && K < 8192 &&
               ((M + 127) / 128) * ((N + 127) / 128) > 256 && ((M + 255) / 256) * ((N + 127) / 128) <= 256) {
      variant = V_PIPELINED_256x128;
      cut_rows = 2;
    }
    else if (K < 1024 && t256 <= 2048 && fits(V_PERSISTENT) && t256 >= 128 && full_rounds) variant = V_PERSISTENT;
    else if (t256 <= 128 && fits(V_STREAM_TAIL) && workspace && [&] {  // too few tiles for the chip, and a workspace to split K into
               int sm, sn;
               const int S = ksplit_plan((int)M, (int)N, (int)K, sm, sn);
               return S > 1 && workspace_bytes >= (int64_t)S * sm * sn * 4;
             }())
      variant = V_STREAM_TAIL;
    else if (fits(V_STREAM_TAIL) && t256 >= 128) variant = V_STREAM_TAIL;
    else if (fits(V_PERSISTENT) && t256 >= 128 && full_rounds) variant = V_PERSISTENT;
    else if (fits(V_PIPELINED_128)) variant = V_PIPELINED_128;
    else if (fits(V_PIPELINED_128x64)) variant = V_PIPELINED_128x64;  // larger products that divide by 64 and not by 128
    else if (fits(V_PIPELINED_64)) variant = V_PIPELINED_64;
    else variant = kNumGemmVariants - 1;
  } else if (!fits(variant) && variant == V_SKINNY) {
    return fail(-MI355_E_SHAPE, "gemm_f16_nt: variant %s needs M<=128, N%%32==0, K%%64==0 and 16-byte aligned pointers",
                kGemmVariants[variant].name);
  } else if (!fits(variant)) {
    return fail(-MI355_E_SHAPE, "gemm_f16_nt: variant %s needs M%%%d==0, N%%%d==0, K%%64==0 and 16-byte aligned pointers",
                kGemmVariants[variant].name, kGemmVariants[variant].bm, kGemmVariants[variant].bn);
  }
  if (variant == kNumGemmVariants - 1 && ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) & 15u) && K % 8 == 0) {
    return fail(-MI355_E_ALIGN, "gemm_f16_nt: a and b must be 16-byte aligned when K %% 8 == 0");
  }
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  float* ws = static_cast<float*>(workspace);
  const size_t wsb = workspace_bytes > 0 ? (size_t)workspace_bytes : 0;
  if (ws && !aligned16(ws)) return fail(-MI355_E_ALIGN, "gemm_f16_nt: workspace must be 16-byte aligned");
  if ((small.ragged && small.S == 1) || cut_rows) {
    const int m = (int)M, n = (int)N, k = (int)K;
    auto tiled = [&](auto out, auto is_bf) {
      using OutT = decltype(out);
      constexpr bool BF = decltype(is_bf)::value;
      if (cut_rows == 2) return launch_tiled<256, 128, 2, 2, OutT, 1, BF, true>(a, b, c, m, n, k, n, s);
      if (cut_rows == 1) return launch_tiled<128, 128, 2, 2, OutT, 1, BF, true>(a, b, c, m, n, k, n, s);
      if (small.bm == 64) return launch_tiled<64, 64, 2, 2, OutT, 1, BF, true>(a, b, c, m, n, k, n, s);
      if (small.bn == 64) return launch_tiled<128, 64, 2, 2, OutT, 1, BF, true>(a, b, c, m, n, k, n, s);
      return launch_tiled<128, 128, 2, 2, OutT, 1, BF, true>(a, b, c, m, n, k, n, s);
    };
    if (bf) return out_dtype == MI355_F32 ? tiled(float{}, std::true_type{}) : tiled(half_t{}, std::true_type{});
    return out_dtype == MI355_F32 ? tiled(float{}, std::false_type{}) : tiled(half_t{}, std::false_type{});
  }
  if (small.S > 1) {
    const half_t *ah = (const half_t*)a, *bh = (const half_t*)b;
    const int m = (int)M, n = (int)N, k = (int)K, S = small.S;
    auto tiled = [&](auto out, auto is_bf) {
      using OutT = decltype(out);
      constexpr bool BF = decltype(is_bf)::value;
      if (small.bm == 64) return launch_ksplit128<OutT, BF, 64, 64>(ah, bh, (OutT*)c, m, n, k, n, S, ws, s, small.ragged);
      if (small.bn == 64) return launch_ksplit128<OutT, BF, 128, 64>(ah, bh, (OutT*)c, m, n, k, n, S, ws, s, small.ragged);
      return launch_ksplit128<OutT, BF, 128, 128>(ah, bh, (OutT*)c, m, n, k, n, S, ws, s, small.ragged);
    };
    if (bf) return out_dtype == MI355_F32 ? tiled(float{}, std::true_type{}) : tiled(half_t{}, std::true_type{});
    return out_dtype == MI355_F32 ? tiled(float{}, std::false_type{}) : tiled(half_t{}, std::false_type{});
  }
  if (split128 > 1) {
    const half_t *ah = (const half_t*)a, *bh = (const half_t*)b;
    const int m = (int)M, n = (int)N, k = (int)K;
    if (bf) {
      if (out_dtype == MI355_F32) return launch_ksplit128<float, true>(ah, bh, (float*)c, m, n, k, n, split128, ws, s);
      return launch_ksplit128<half_t, true>(ah, bh, (half_t*)c, m, n, k, n, split128, ws, s);
    }
    if (out_dtype == MI355_F32) return launch_ksplit128<float, false>(ah, bh, (float*)c, m, n, k, n, split128, ws, s);
    return launch_ksplit128<half_t, false>(ah, bh, (half_t*)c, m, n, k, n, split128, ws, s);
  }
  if (bf) {
    if (out_dtype == MI355_F32) return launch_variant<float, true>(variant, a, b, c, (int)M, (int)N, (int)K, s, ws, wsb);
    return launch_variant<half_t, true>(variant, a, b, c, (int)M, (int)N, (int)K, s, ws, wsb);
  }
  if (out_dtype == MI355_F32) return launch_variant<float, false>(variant, a, b, c, (int)M, (int)N, (int)K, s, ws, wsb);
  return launch_variant<half_t, false>(variant, a, b, c, (int)M, (int)N, (int)K, s, ws, wsb);
}

// Bytes of workspace with which the automatic choice would split K for this shape (0: it would not).
static int64_t gemm_nt_workspace_bytes(int64_t M, int64_t N, int64_t K) {
  if (M > 0 && N > 0 && K > 0 && splits_rows(M, N, K)) {  // two products, one after the other, on one workspace
    const int64_t main = gemm_nt_workspace_bytes(M / 256 * 256, N, K), rest = gemm_nt_workspace_bytes(M % 256, N, K);
    return main > rest ? main : rest;
  }
  if (M <= 0 || N <= 0 || K <= 0 || M > (1 << 30) || N > (1 << 30) || K > (1 << 21) || K < 256 || K % 128 != 0) return 0;
  if (M * K * 2 >= (1ll << 32) || N * K * 2 >= (1ll << 32)) return 0;  // the streamed kernel's one descriptor per operand
  if (M <= 64 && N % 32 == 0 && N >= 2048 && K >= 512) return 0;        // the weight-streaming kernel's shapes
  const SmallPlan sp = small_plan(M, N, K, INT64_MAX);
  if (sp.bm) return sp.ws_bytes();
  if (takes_256x128(M, N, K)) return 0;
  const int s128 = (K % 64 == 0) ? ksplit128_plan((int)M, (int)N, (int)K) : 1;
  if (s128 > 1) return (int64_t)s128 * M * N * 4;
  int sm, sn;
  const int S = ksplit_plan((int)M, (int)N, (int)K, sm, sn);
  return S > 1 ? (int64_t)S * sm * sn * 4 : 0;
}

extern "C" int mi355_gemm_f16_nt(const void* a, const void* b, void* c, int64_t M, int64_t N, int64_t K, int out_dtype,
                                 int variant, void* stream) {
  return gemm_nt_entry(false, a, b, c, M, N, K, out_dtype, variant, stream);
}

extern "C" int mi355_gemm_bf16_nt(const void* a, const void* b, void* c, int64_t M, int64_t N, int64_t K, int out_dtype,
                                  int variant, void* stream) {
  return gemm_nt_entry(true, a, b, c, M, N, K, out_dtype, variant, stream);
}

extern "C" int64_t mi355_gemm_nt_workspace_bytes(int64_t M, int64_t N, int64_t K) { return gemm_nt_workspace_bytes(M, N, K); }

extern "C" int mi355_gemm_f16_nt_ws(const void* a, const void* b, void* c, int64_t M, int64_t N, int64_t K, int out_dtype,
                                    int variant, void* workspace, int64_t workspace_bytes, void* stream) {
  return gemm_nt_entry(false, a, b, c, M, N, K, out_dtype, variant, stream, workspace, workspace_bytes);
}

extern "C" int mi355_gemm_bf16_nt_ws(const void* a, const void* b, void* c, int64_t M, int64_t N, int64_t K, int out_dtype,
                                     int variant, void* workspace, int64_t workspace_bytes, void* stream) {
  return gemm_nt_entry(true, a, b, c, M, N, K, out_dtype, variant, stream, workspace, workspace_bytes);
}
