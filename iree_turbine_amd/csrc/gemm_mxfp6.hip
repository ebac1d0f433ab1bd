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
#include "gemm_tiles.hpp"

namespace mi355 {

namespace {

// FMT: the instruction's format code, 2 = E2M3, 3 = E3M2
template <int FMT>
__device__ __forceinline__ floatx16 mfma_fp6_32x32x64(intx8 a, int sa, intx8 b, int sb, floatx16 c) {
  return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, FMT, FMT, 0, sa, 0, sb);
}

// byte SEL of sa / sb scales the lane's block
template <int FMT, int SEL>
__device__ __forceinline__ floatx16 mfma_fp6_sel(intx8 a, int sa, intx8 b, int sb, floatx16 c) {
  return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, FMT, FMT, SEL, sa, SEL, sb);
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
      if (nn < N) MxOut<OutT>::store1(C + (size_t)m * N + nn, acc[r]);
    }
  }
}

// Register-staged tiled kernel, the design of gemm_mxfp8_staged for 96-byte slab rows: 256x256 tile, 4 waves with
// 128x128 wave tiles, a K slab of 128 elements = 96 bytes per row = 6 chunks of 16 bytes = 4 scale blocks = 2
// k-steps.  Slab s+3 is loaded into VGPRs while slab s computes, slab s+1 is copied from registers into the LDS
// stage that slab s-1 left; one barrier per slab.  LDS holds a stage as six chunk planes (256 rows x 16 bytes, 48
// bytes of padding).  A 24-byte block is a chunk and half of its neighbour, and which half comes first depends on
// the block's parity; a k-step therefore pairs blocks of EQUAL parity -- k-step 0 takes blocks 0 (lane half 0)
// and 2 (half 1), each a ds_read_b128 of chunk 3h and a ds_read_b64 of the low half of chunk 3h + 1; k-step 1
// blocks 1 and 3, the high half of chunk 3h + 1 and chunk 3h + 2 -- so both lane halves run the same
// instructions.  The row's scale dword per slab is stored plain and rotated by 16 bits, as for MXFP8: lane half h
// reads the copy whose bytes 0, 1 are blocks 2h, 2h + 1 and op_sel = ks picks the block.
// The loads into registers are inline assembly with hand-placed waits: the kernel must not spill.
template <typename OutT, int FMT>
__global__ __launch_bounds__(256) void gemm_mxfp6_staged(const uint8_t* __restrict__ A, const uint8_t* __restrict__ As,
                                                         const uint8_t* __restrict__ B, const uint8_t* __restrict__ Bs,
                                                         OutT* __restrict__ C, int M, int N, int K, int tiles_m, int tiles_n,
                                                         int group_m) {
  constexpr int BM = 256, BN = 256, WN = 2;
  constexpr int WTM = 128, WTN = 128, TM = 4, TN = 4;
  // LDS: A stage 0, A stage 1, B stage 0, B stage 1, then the scale buffers A parity 0, A parity 1, B parity 0,
  // B parity 1 (4 KiB each; parity is address bit 12)
  constexpr int PL = 256 * 16 + 48, OP_BYTES = 6 * PL, B_OFF = 2 * OP_BYTES;
  constexpr int SC_OFF = 13 * 8192;
  static_assert(SC_OFF >= 4 * OP_BYTES && SC_OFF % 8192 == 0, "scale buffers behind the data stages");
  constexpr int NL = 13;  // loads per slab and lane: 6 chunks of A, 6 of B, one scale row
  typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
  typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
  typedef int i32x4 __attribute__((ext_vector_type(4)));

  extern __shared__ __attribute__((aligned(1024))) char lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WN, wn = wave % WN;
  int tile_m, tile_n;
  map_tile(blockIdx.x, tiles_m, tiles_n, group_m, tile_m, tile_n);

  const unsigned row_bytes = ((unsigned)K >> 2) * 3u;
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
  // codes: the 128 rows x 6 chunks of half a tile are 768 chunks = 3 per thread, thread t taking chunks t,
  // t + 256, t + 512 in row-major order (6 consecutive lanes cover one 96-byte row piece); load n < 6 is chunk
  // (n % 3) of the upper (n < 3) or lower half of the A tile, 6..11 the same of the B tile
  unsigned g_off[3];
  int w_off[3];
#pragma unroll
  for (int j = 0; j < 3; j++) {
    const int q = j * 256 + tid, row = q / 6, ch = q - row * 6;
    g_off[j] = (unsigned)row * row_bytes + (unsigned)ch * 16u;
    w_off[j] = ch * PL + row * 16;
  }
  const i32x4 a_src = make_desc(A + (size_t)(tile_m * BM) * row_bytes, (unsigned)BM * row_bytes);
  const i32x4 b_src = make_desc(B + (size_t)(tile_n * BN) * row_bytes, (unsigned)BN * row_bytes);
  const unsigned half_step = 128u * row_bytes;
  // scales: lane l of wave w owns row 64 w + l of the tile
  const i32x4 as_src = make_desc(As + (size_t)(tile_m * BM + wave * 64) * sc_bytes, (unsigned)(BM - wave * 64) * sc_bytes);
  const i32x4 bs_src = make_desc(Bs + (size_t)(tile_n * BN + wave * 64) * sc_bytes, (unsigned)(BN - wave * 64) * sc_bytes);
  const unsigned s_off = (unsigned)lane * sc_bytes;
  int sc_wr = SC_OFF + 4096 + (wave * 64 + lane) * 16;  // where the NEXT group's A scales go (B: + 8192); flips per group

  u32x4 r[2][12];
  u32x2 rsc[2];
#define MI355_M6_LOAD(S, n, k_off_)                                                                              \
  asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen"                                                        \
               : "=v"(r[S][n])                                                                                   \
               : "v"(g_off[(n) % 3]), "s"((n) < 6 ? a_src : b_src), "s"((k_off_) + (unsigned)(((n) % 6) / 3) * half_step) \
               : "memory")
#define MI355_M6_LOAD_SC(S, desc, group_) \
  asm volatile("buffer_load_dwordx2 %0, %1, %2, %3 offen" : "=v"(rsc[S]) : "v"(s_off), "s"(desc), "s"((unsigned)(group_)*8u) : "memory")
  // `newer` = loads issued after the one that filled the register; they may still be in flight
#define MI355_M6_WRITE(S, n, newer, st_)                                                                                   \
  do {                                                                                                                     \
    asm volatile("s_waitcnt vmcnt(%1)" : "+v"(r[S][n]) : "n"(newer) : "memory");                                           \
    *reinterpret_cast<u32x4*>(lds + w_off[(n) % 3] + (((n) < 6 ? 0 : B_OFF) + (st_)*OP_BYTES + (((n) % 6) / 3) * 2048)) = r[S][n]; \
  } while (0)
#define MI355_M6_WRITE_SC(S, newer, addr_)                                           \
  do {                                                                               \
    asm volatile("s_waitcnt vmcnt(%1)" : "+v"(rsc[S]) : "n"(newer) : "memory");      \
    *reinterpret_cast<u32x4*>(lds + (addr_)) = both_halves(rsc[S]);                  \
  } while (0)

  // a row's two slab dwords, each followed by itself rotated by 16 bits (what lane half 1 reads)
  auto both_halves = [](u32x2 d) { return u32x4{d[0], (d[0] >> 16) | (d[0] << 16), d[1], (d[1] >> 16) | (d[1] << 16)}; };

  const int r32 = lane & 31, h = lane >> 5;
  const int a_rd = (wm * WTM + r32) * 16 + h * 3 * PL;
  const int b_rd = B_OFF + (wn * WTN + r32) * 16 + h * 3 * PL;
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
  // B fragments stay for a k-step; A fragments stream through two register sets, one row tile ahead
  intx8 fa0, fa1, fn[TN];
  int ca[TM], cb[TN];

  // fragment of k-step ks at constant offset `imm` (stage and row tile) from the operand's address register
  auto frag = [&](int at, int ks, int imm) {
    if (ks == 0) {
      const intx4 lo = *reinterpret_cast<const intx4*>(lds + at + imm);
      const intx2 hi = *reinterpret_cast<const intx2*>(lds + at + (PL + imm));
      return intx8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], 0, 0};
    }
    const intx2 lo = *reinterpret_cast<const intx2*>(lds + at + (PL + 8 + imm));
    const intx4 hi = *reinterpret_cast<const intx4*>(lds + at + (2 * PL + imm));
    return intx8{lo[0], lo[1], hi[0], hi[1], hi[2], hi[3], 0, 0};
  };
  auto scale_dword = [&](int addr) { return *reinterpret_cast<const int*>(lds + addr); };

#define MI355_M6_LOAD_ALL(S, slab_)                                                                              \
  do {                                                                                                           \
    const unsigned ko_ = (unsigned)(slab_)*96u;                                                                  \
    MI355_M6_LOAD(S, 0, ko_); MI355_M6_LOAD(S, 1, ko_); MI355_M6_LOAD(S, 2, ko_); MI355_M6_LOAD(S, 3, ko_);      \
    MI355_M6_LOAD(S, 4, ko_); MI355_M6_LOAD(S, 5, ko_); MI355_M6_LOAD(S, 6, ko_); MI355_M6_LOAD(S, 7, ko_);      \
    MI355_M6_LOAD(S, 8, ko_); MI355_M6_LOAD(S, 9, ko_); MI355_M6_LOAD(S, 10, ko_); MI355_M6_LOAD(S, 11, ko_);    \
  } while (0)
  // prologue: slab 0 (+ A scales of group 0) -> set 0 -> stage 0; B scales of group 0 through a spare
  // register; slab 1 (+ B scales of group 1) -> set 1; then slab 2 (+ A scales of group 1) -> set 0
  const int KG = KT / 2;  // scale groups
  u32x2 rs;
  MI355_M6_LOAD_ALL(0, 0);
  MI355_M6_LOAD_SC(0, as_src, 0);
  asm volatile("buffer_load_dwordx2 %0, %1, %2, 0 offen" : "=v"(rs) : "v"(s_off), "s"(bs_src) : "memory");
  MI355_M6_LOAD_ALL(1, 1);
  MI355_M6_LOAD_SC(1, bs_src, KG > 1 ? 1 : 0);
  // everything older than set 1's loads has landed once at most NL are outstanding
  MI355_M6_WRITE(0, 0, NL, 0); MI355_M6_WRITE(0, 1, NL, 0); MI355_M6_WRITE(0, 2, NL, 0); MI355_M6_WRITE(0, 3, NL, 0);
  MI355_M6_WRITE(0, 4, NL, 0); MI355_M6_WRITE(0, 5, NL, 0); MI355_M6_WRITE(0, 6, NL, 0); MI355_M6_WRITE(0, 7, NL, 0);
  MI355_M6_WRITE(0, 8, NL, 0); MI355_M6_WRITE(0, 9, NL, 0); MI355_M6_WRITE(0, 10, NL, 0); MI355_M6_WRITE(0, 11, NL, 0);
  MI355_M6_WRITE_SC(0, NL, sc_wr - 4096);
  asm volatile("s_waitcnt vmcnt(%1)" : "+v"(rs) : "n"(NL) : "memory");
  *reinterpret_cast<u32x4*>(lds + sc_wr - 4096 + 8192) = both_halves(rs);
  MI355_M6_LOAD_ALL(0, 2);
  MI355_M6_LOAD_SC(0, as_src, KG > 1 ? 1 : 0);
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __syncthreads();
  fa0 = frag(a_rd, 0, 0);
#pragma unroll
  for (int j = 0; j < TM; j++) {
    fn[j] = frag(b_rd, 0, j * 512);
    ca[j] = scale_dword(sc_rd_a + j * 512);
    cb[j] = scale_dword(sc_rd_b + j * 512);
  }

  // Four MFMAs of A row tile j (fragment FA) against the four B fragments; X0..X3 are what follows each of them
#define MI355_M6_GROUP(KS, j, FA, X0, X1, X2, X3)                                       \
  do {                                                                                  \
    acc[0][j] = mfma_fp6_sel<FMT, KS>(fn[0], cb[0], FA, ca[j], acc[0][j]);              \
    X0;                                                                                 \
    __builtin_amdgcn_sched_barrier(0);                                                  \
    acc[1][j] = mfma_fp6_sel<FMT, KS>(fn[1], cb[1], FA, ca[j], acc[1][j]);              \
    X1;                                                                                 \
    __builtin_amdgcn_sched_barrier(0);                                                  \
    acc[2][j] = mfma_fp6_sel<FMT, KS>(fn[2], cb[2], FA, ca[j], acc[2][j]);              \
    X2;                                                                                 \
    __builtin_amdgcn_sched_barrier(0);                                                  \
    acc[3][j] = mfma_fp6_sel<FMT, KS>(fn[3], cb[3], FA, ca[j], acc[3][j]);              \
    X3;                                                                                 \
    __builtin_amdgcn_sched_barrier(0);                                                  \
  } while (0)
#define MI355_NOP ((void)0)

  // Slab kt (scales in ca/cb) sits in stage P; set Q = 1 - P holds slab kt+1 and the scale row SCD travels with
  // (written to SCW); each register is reloaded with slab kt+3 (the scale row with group GN) after it is written.
  // In flight when register n is written: the rest of its own round (NL - 1 - n), the NL loads of the other set
  // and the loads of this slab issued so far.  The slab's one barrier stands behind the last read of stage P and
  // before the first read of stage Q, in the last group of k-step 1.  HALF = 8 if slab kt+1 is the second slab
  // of its scale group.
#define MI355_M6_W(Q, n, issued) MI355_M6_WRITE(Q, n, 2 * NL - 1 - (n) + (issued), Q)
#define MI355_M6_SLAB(P, Q, kt_, SCD, SCW, GN, HALF)                                                                       \
  do {                                                                                                                     \
    constexpr int st = P * OP_BYTES, nst = Q * OP_BYTES;                                                                   \
    const int nxt_ = (kt_) + 3 < KT ? (kt_) + 3 : KT - 1; /* past the end: re-fetch, never used */                         \
    const unsigned ko = (unsigned)nxt_ * 96u;                                                                              \
    const int gn_ = (GN) < KG ? (GN) : KG - 1;                                                                             \
    __builtin_amdgcn_sched_barrier(0);                                                                                     \
    MI355_M6_GROUP(0, 0, fa0, MI355_M6_W(Q, 0, 0); MI355_M6_W(Q, 1, 0), MI355_M6_W(Q, 2, 0); fa1 = frag(a_rd, 0, st + 512), \
                   MI355_M6_W(Q, 3, 0), MI355_M6_W(Q, 4, 0); MI355_M6_LOAD(Q, 0, ko));                                      \
    MI355_M6_GROUP(0, 1, fa1, MI355_M6_W(Q, 5, 1); MI355_M6_W(Q, 6, 1), MI355_M6_W(Q, 7, 1); fa0 = frag(a_rd, 0, st + 2 * 512), \
                   MI355_M6_W(Q, 8, 1), MI355_M6_W(Q, 9, 1); MI355_M6_LOAD(Q, 1, ko));                                      \
    MI355_M6_GROUP(0, 2, fa0, MI355_M6_W(Q, 10, 2); MI355_M6_W(Q, 11, 2), MI355_M6_WRITE_SC(Q, NL + 2, SCW); fa1 = frag(a_rd, 0, st + 3 * 512), \
                   MI355_M6_LOAD(Q, 2, ko), MI355_M6_LOAD(Q, 3, ko));                                                      \
    MI355_M6_GROUP(0, 3, fa1, fn[0] = frag(b_rd, 1, st); fa0 = frag(a_rd, 1, st),                                          \
                   MI355_M6_LOAD(Q, 4, ko); fn[1] = frag(b_rd, 1, st + 512), fn[2] = frag(b_rd, 1, st + 2 * 512),          \
                   fn[3] = frag(b_rd, 1, st + 3 * 512));                                                                   \
    MI355_M6_GROUP(1, 0, fa0, MI355_M6_LOAD(Q, 5, ko), fa1 = frag(a_rd, 1, st + 512), MI355_M6_LOAD(Q, 6, ko),             \
                   MI355_M6_LOAD(Q, 7, ko));                                                                               \
    MI355_M6_GROUP(1, 1, fa1, MI355_M6_LOAD(Q, 8, ko), fa0 = frag(a_rd, 1, st + 2 * 512), MI355_M6_LOAD(Q, 9, ko),         \
                   MI355_M6_LOAD(Q, 10, ko));                                                                              \
    MI355_M6_GROUP(1, 2, fa0, MI355_M6_LOAD(Q, 11, ko), fa1 = frag(a_rd, 1, st + 3 * 512), MI355_M6_LOAD_SC(Q, SCD, gn_),  \
                   MI355_NOP);                                                                                             \
    if (HALF == 0) { sc_rd_a ^= 4096; sc_rd_b ^= 4096; }                                                                   \
    MI355_M6_GROUP(1, 3, fa1,                                                                                              \
                   asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); __builtin_amdgcn_s_barrier();                       \
                   fa0 = frag(a_rd, 0, nst); fn[0] = frag(b_rd, 0, nst); cb[0] = scale_dword(sc_rd_b + HALF);              \
                   ca[0] = scale_dword(sc_rd_a + HALF),                                                                    \
                   fn[1] = frag(b_rd, 0, nst + 512); cb[1] = scale_dword(sc_rd_b + HALF + 512);                            \
                   ca[1] = scale_dword(sc_rd_a + HALF + 512),                                                              \
                   fn[2] = frag(b_rd, 0, nst + 2 * 512); cb[2] = scale_dword(sc_rd_b + HALF + 1024);                       \
                   ca[2] = scale_dword(sc_rd_a + HALF + 1024),                                                             \
                   fn[3] = frag(b_rd, 0, nst + 3 * 512); cb[3] = scale_dword(sc_rd_b + HALF + 1536);                       \
                   ca[3] = scale_dword(sc_rd_a + HALF + 1536));                                                            \
  } while (0)

  for (int kt = 0; kt < KT; kt += 2) {
    const int g0 = kt >> 1;
    // even slab: set 1 carries slab kt+1 and the B scales of group g0+1; reloaded with slab kt+3 and the B scales of g0+2
    MI355_M6_SLAB(0, 1, kt, bs_src, sc_wr + 8192, g0 + 2, 8);
    // odd slab: set 0 carries slab kt+2 and the A scales of group g0+1; reloaded with slab kt+4 and the A scales of g0+2
    MI355_M6_SLAB(1, 0, kt + 1, as_src, sc_wr, g0 + 2, 0);
    sc_wr ^= 4096;
    // The loads of the last slabs fetch nothing that is used, and behind the loop the compiler hands their
    // registers to the epilogue: let them land while the registers still belong to them.
    // The wait names every staging register as an input, so that the registers stay allocated to the loads up to it
    // however the compiler restructures the last iteration.
    if (kt + 2 >= KT) {
      asm volatile("s_waitcnt vmcnt(0)" ::"v"(r[0][0]), "v"(r[0][1]), "v"(r[0][2]), "v"(r[0][3]), "v"(r[0][4]), "v"(r[0][5]), "v"(r[0][6]), "v"(r[0][7]), "v"(r[0][8]), "v"(r[0][9]), "v"(r[0][10]), "v"(r[0][11]) : "memory");
      asm volatile("" ::"v"(r[1][0]), "v"(r[1][1]), "v"(r[1][2]), "v"(r[1][3]), "v"(r[1][4]), "v"(r[1][5]), "v"(r[1][6]), "v"(r[1][7]), "v"(r[1][8]), "v"(r[1][9]), "v"(r[1][10]), "v"(r[1][11]) : "memory");
    }
  }
#undef MI355_M6_SLAB
#undef MI355_M6_W
#undef MI355_M6_GROUP
#undef MI355_NOP
#undef MI355_M6_LOAD_ALL
#undef MI355_M6_WRITE_SC
#undef MI355_M6_WRITE
#undef MI355_M6_LOAD_SC
#undef MI355_M6_LOAD
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
          ushortx4 v = {f32_to_bf16_rne(acc[i][j][4 * q]), f32_to_bf16_rne(acc[i][j][4 * q + 1]),
                        f32_to_bf16_rne(acc[i][j][4 * q + 2]), f32_to_bf16_rne(acc[i][j][4 * q + 3])};
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
      float* crow = C + (size_t)(m0 + j * 32) * N + n0;
#pragma unroll
      for (int i = 0; i < TN; i++)
#pragma unroll
        for (int q = 0; q < 4; q++)
          *reinterpret_cast<floatx4*>(crow + i * 32 + q * 8) =
              floatx4{acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
    }
  }
}

static const char* kMx6Variants[] = {"generic_32x128", "staged_256x256x128_w2x2"};
constexpr int kNumMx6Variants = 2;
int mxfp6_variant_count() { return kNumMx6Variants; }
const char* mxfp6_variant_name(int i) { return (i >= 0 && i < kNumMx6Variants) ? kMx6Variants[i] : nullptr; }

template <typename OutT, int FMT>
static int launch_mx6(int variant, const void* a, const void* as, const void* b, const void* bs, void* c, int M, int N, int K,
                      hipStream_t stream) {
  if (variant == 1) {
    {
      auto kern = gemm_mxfp6_staged<OutT, FMT>;
      constexpr int lds_bytes = 13 * 8192 + 4 * 4096;  // two padded stages per operand, four scale buffers
      static std::atomic<uint64_t> lds_ok{0};
      if (int rc = allow_lds(reinterpret_cast<const void*>(kern), lds_bytes, lds_ok, "gemm_mxfp6_staged")) return rc;
      const int tiles_m = M / 256, tiles_n = N / 256;
      dim3 grid(tiles_m * tiles_n), block(256);
      hipLaunchKernelGGL(kern, grid, block, lds_bytes, stream, (const uint8_t*)a, (const uint8_t*)as, (const uint8_t*)b,
                         (const uint8_t*)bs, (OutT*)c, M, N, K, tiles_m, tiles_n, 4);
      return check_launch("gemm_mxfp6_staged", grid, block, lds_bytes);
    }
  }
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
  const bool sc_al4 = ((reinterpret_cast<uintptr_t>(a_scale) | reinterpret_cast<uintptr_t>(b_scale)) & 3u) == 0;
  // slabs of 128 elements in pairs, four in flight; 32-bit buffer offsets
  const bool fits1 = sc_al4 && M % 256 == 0 && N % 256 == 0 && K % 256 == 0 && K >= 512 && K <= (1 << 23);
  if (variant < 0) variant = fits1 ? 1 : 0;
  else if (variant == 1 && !fits1)
    return fail(-MI355_E_SHAPE, "mxfp6_gemm: variant %s needs M%%256==0, N%%256==0, K%%256==0, 512 <= K <= 2^23 and 4-byte aligned scales",
                kMx6Variants[1]);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const bool e2m3 = element_format == MI355_FP6_E2M3;
  if (out_dtype == MI355_F32)
    return e2m3 ? launch_mx6<float, 2>(variant, a, a_scale, b, b_scale, c, (int)M, (int)N, (int)K, s)
                : launch_mx6<float, 3>(variant, a, a_scale, b, b_scale, c, (int)M, (int)N, (int)K, s);
  return e2m3 ? launch_mx6<unsigned short, 2>(variant, a, a_scale, b, b_scale, c, (int)M, (int)N, (int)K, s)
              : launch_mx6<unsigned short, 3>(variant, a, a_scale, b, b_scale, c, (int)M, (int)N, (int)K, s);
}
