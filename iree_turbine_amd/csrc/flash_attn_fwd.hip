// Flash-attention forward (prefill) for gfx950, head dim 128, fp16 in/out, fp32 softmax.
//
// One workgroup = 4 waves = 128 queries of one (batch, head); each wave owns 32 queries and
// keeps, in registers, its Q fragments (32 VGPRs), the running max / sum of every query, and
// the 32 x 128 fp32 output accumulator (64 VGPRs).  K and V are streamed in 64-key tiles
// through a two-stage LDS ring filled by direct-to-LDS loads.
//
// Both contractions are computed transposed so that the softmax never leaves registers:
//   S^T[key][query]  = K . Q^T     (MFMA A operand = K rows from LDS, B operand = Q in registers)
//   O^T[d][query]   += V^T . P^T   (A operand = V^T via LDS transpose reads, B operand = P)
// With v_mfma_f32_32x32x16_f16 a lane owns one query column of S^T (16 keys per 32-key tile,
// the other 16 sit in lane^32), so row max / sum are in-lane reductions plus one cross-lane
// exchange, and the exponentiated scores are already laid out as the B operand of the second
// MFMA.  The order in which keys are fed to that MFMA is whatever the S^T register order
// dictates; V^T is fetched with the matching order by ds_read_b64_tr_b16.
//
// LDS swizzles (16-byte chunks, 256-byte rows): K chunk c of row r -> slot c ^ (r & 15);
// V chunk c of row r -> slot c ^ (2 * (r & 7)).  As in the GEMM, the swizzle is applied on the
// global side of the direct-to-LDS loads.
#include "common.hpp"
#include <math.h>
#include <type_traits>

namespace mi355 {

constexpr int FA_BLOCK_M = 128;
constexpr int FA_BLOCK_N = 64;
constexpr int FA_STAGE = 2 * FA_BLOCK_N * 256;  // K tile + V tile, bytes

// Where each operand's (batch, head, row) lives, in elements; the 128 elements of a row are contiguous.
// `group` query heads share one K/V head (1 = plain multi-head attention).
struct FaLayout {
  int64_t q_b, q_h, k_b, k_h, v_b, v_h, o_b, o_h;
  unsigned q_r, k_r, v_r, o_r;
  int H, group;
};

template <bool CAUSAL, bool BF>
__global__ __launch_bounds__(256) void fa_fwd_d128(const half_t* __restrict__ Q, const half_t* __restrict__ K,
                                                   const half_t* __restrict__ V, half_t* __restrict__ O, int BH, int Sq,
                                                   int Sk, float scale_log2e, int q_blocks, FaLayout lay) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r32 = lane & 31, h = lane >> 5;

  // workgroup -> (batch*head, query block).  Consecutive ids land on different XCDs; keep all
  // query blocks of one head on one XCD so its K/V stay in that XCD's L2.
  int bh, qb;
  {
    const int pid = blockIdx.x;
    if (((BH / lay.group) & 7) == 0) {
      // all query blocks of the `group` query heads that share one K/V head sit on one XCD
      const int xcd = pid & 7, loc = pid >> 3, per_kv = q_blocks * lay.group;
      const int w = loc % per_kv;
      bh = ((loc / per_kv) * 8 + xcd) * lay.group + w / q_blocks;
      qb = w % q_blocks;
    } else {
      bh = pid / q_blocks;
      qb = pid % q_blocks;
    }
    if (CAUSAL) qb = q_blocks - 1 - qb;  // longest rows first
  }
  const int causal_off = Sk - Sq;  // query i sees keys <= i + causal_off
  const int q0 = qb * FA_BLOCK_M;
  const int wq0 = q0 + wave * 32;  // first query of this wave
  const int q_row = wq0 + r32;
  const bool q_ok = q_row < Sq;

  const int b_idx = bh / lay.H, h_idx = bh - b_idx * lay.H, hk_idx = h_idx / lay.group;
  const half_t* Qb = Q + b_idx * lay.q_b + h_idx * lay.q_h;
  const half_t* Kb = K + b_idx * lay.k_b + hk_idx * lay.k_h;
  const half_t* Vb = V + b_idx * lay.v_b + hk_idx * lay.v_h;
  half_t* Ob = O + b_idx * lay.o_b + h_idx * lay.o_h;

  // number of key tiles this workgroup walks
  int k_end = Sk;
  if (CAUSAL) {
    int last_q = q0 + FA_BLOCK_M - 1;
    if (last_q > Sq - 1) last_q = Sq - 1;
    int lim = last_q + causal_off + 1;
    if (lim < k_end) k_end = lim;
  }
  const int n_tiles = k_end > 0 ? (k_end + FA_BLOCK_N - 1) / FA_BLOCK_N : 0;

  // ---- Q fragments (MFMA B operand): lane (query r32, half h) holds d = 16*ks + 8*h .. +7 ----
  half8 qf[8];
#pragma unroll
  for (int ks = 0; ks < 8; ks++) {
    if (q_ok) {
      qf[ks] = *reinterpret_cast<const half8*>(Qb + (size_t)q_row * lay.q_r + ks * 16 + h * 8);
    } else {
#pragma unroll
      for (int e = 0; e < 8; e++) qf[ks][e] = (half_t)0;
    }
  }

  // ---- global -> LDS: a wave-load moves 4 rows of 256 bytes; lane l: row l/16, slot l%16 ----
  const int lrow = lane >> 4, lslot = lane & 15;
  const int k_chunk = lslot ^ (wave * 4 + lrow);           // group g = wave + 4*i, so (row & 15) = 4*wave + lrow
  const int v_chunk = lslot ^ (2 * ((wave & 1) * 4 + lrow));  // (row & 7) = 4*(wave&1) + lrow
  auto issue_loads = [&](int tile, int stage) {
    char* dst = lds + stage * FA_STAGE + wave * 1024;
    const int key0 = tile * FA_BLOCK_N;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      int row = key0 + (wave + 4 * i) * 4 + lrow;
      if (row > Sk - 1) row = Sk - 1;  // clamp: the tail rows are masked out of the softmax
      load_lds_16B(Kb + (size_t)row * lay.k_r + k_chunk * 8, dst + i * 4096);
      load_lds_16B(Vb + (size_t)row * lay.v_r + v_chunk * 8, dst + FA_BLOCK_N * 256 + i * 4096);
    }
  };

  // ---- LDS read addresses ----
  const int k_base = r32 * 256 + ((h ^ (lane & 15)) * 16);  // ^ (ks*32), + t*8192
  const int i16 = lane & 15, g16 = lane >> 4;
  const int v_row = 4 * (g16 >> 1) + (i16 >> 2);
  const int v_cl = 2 * (g16 & 1) + ((i16 & 3) >> 1);
  const int v_base = FA_BLOCK_N * 256 + v_row * 256 + ((v_cl ^ (2 * (v_row & 7))) * 16) + (i16 & 1) * 8;  // ^ (dt*64), + t16*4096, + {0,2048}

  floatx16 oacc[4];
#pragma unroll
  for (int dt = 0; dt < 4; dt++)
#pragma unroll
    for (int r = 0; r < 16; r++) oacc[dt][r] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  if (n_tiles > 0) {
    issue_loads(0, 0);
    wait_vmcnt0();
    __syncthreads();
  }

  for (int j = 0; j < n_tiles; j++) {
    if (j + 1 < n_tiles) issue_loads(j + 1, (j + 1) & 1);
    const char* st = lds + (j & 1) * FA_STAGE;
    const int key0 = j * FA_BLOCK_N;
    // a wave whose every query is before this tile has nothing to do here (causal only)
    const bool active = !CAUSAL || (key0 <= wq0 + 31 + causal_off);
    if (active) {
      floatx16 s[2];
#pragma unroll
      for (int t = 0; t < 2; t++) {
#pragma unroll
        for (int r = 0; r < 16; r++) s[t][r] = 0.f;
#pragma unroll
        for (int ks = 0; ks < 8; ks++) {
          half8 kf = *reinterpret_cast<const half8*>(st + ((k_base ^ (ks * 32)) + t * 8192));
          s[t] = mfma16<BF>(kf, qf[ks], s[t]);
        }
      }
      const bool need_mask = (CAUSAL && (key0 + FA_BLOCK_N - 1 > wq0 + causal_off)) || (key0 + FA_BLOCK_N > Sk);
      if (need_mask) {
        const int lim = CAUSAL ? (q_row + causal_off < Sk - 1 ? q_row + causal_off : Sk - 1) : Sk - 1;  // last visible key
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
          for (int r = 0; r < 16; r++) {
            const int key = key0 + 32 * t + 8 * (r >> 2) + 4 * h + (r & 3);
            if (key > lim) s[t][r] = -INFINITY;
          }
      }
      float mx = s[0][0];
#pragma unroll
      for (int t = 0; t < 2; t++)
#pragma unroll
        for (int r = 0; r < 16; r++) mx = fmaxf(mx, s[t][r]);
      mx = fmaxf(mx, __shfl_xor(mx, 32));
      const float m_new = fmaxf(m_run, mx);
      const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
      const float alpha = exp2f((m_run - m_use) * scale_log2e);
      const float mc = m_use * scale_log2e;
      m_run = m_new;
      float psum = 0.f;
      half8 pf[4];
#pragma unroll
      for (int t = 0; t < 2; t++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const float p = exp2f(s[t][r] * scale_log2e - mc);
          psum += p;
          pf[t * 2 + (r >> 3)][r & 7] = cvt16<BF>(p);
        }
      l_run = l_run * alpha + psum;
#pragma unroll
      for (int dt = 0; dt < 4; dt++)
#pragma unroll
        for (int r = 0; r < 16; r++) oacc[dt][r] *= alpha;
      // O^T += V^T P^T
#pragma unroll
      for (int t16 = 0; t16 < 4; t16++) {
#pragma unroll
        for (int dt = 0; dt < 4; dt++) {
          const char* va = st + ((v_base ^ (dt * 64)) + t16 * 4096);
          half4 lo = lds_read_tr16(va);
          half4 hi = lds_read_tr16(va + 2048);
          half8 vf = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
          oacc[dt] = mfma16<BF>(vf, pf[t16], oacc[dt]);
        }
      }
    }
    wait_vmcnt0();
    __syncthreads();
  }

  // ---- epilogue ----
  const float l_tot = l_run + __shfl_xor(l_run, 32);
  const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
  if (q_ok) {
    half_t* orow = Ob + (size_t)q_row * lay.o_r + 4 * h;
#pragma unroll
    for (int dt = 0; dt < 4; dt++)
#pragma unroll
      for (int q = 0; q < 4; q++) {
        half4 v = {cvt16<BF>(oacc[dt][4 * q] * inv), cvt16<BF>(oacc[dt][4 * q + 1] * inv), cvt16<BF>(oacc[dt][4 * q + 2] * inv),
                   cvt16<BF>(oacc[dt][4 * q + 3] * inv)};
        *reinterpret_cast<half4*>(orow + dt * 32 + q * 8) = v;
      }
  }
}

// Paged K/V (the PAGED form of fa_fwd_d128_m16): the keys and values of sequence b are the first seq_lens[b] token rows of the
// pages block_table[b][0..], 16 << page_shift tokens per page, laid out [page][token][kv head][128].  The kernel
// walks 16-token blocks; a page is 1 << page_shift consecutive blocks.
struct FaPaged {
  const int* block_table;  // [batch][max_pages]
  const int* seq_lens;     // [batch]
  int max_pages, num_pages, page_shift;
};

// body(std::integral_constant<int, 0>{}), ..., body(std::integral_constant<int, N - 1>{}): a loop whose index is a
// constant expression in the body (instruction immediates of inline assembly need one).
template <int I, int N, typename F>
__device__ __forceinline__ void static_for(F&& body) {
  if constexpr (I < N) {
    body(std::integral_constant<int, I>{});
    static_for<I + 1, N>(body);
  }
}

// Software-pipelined form.  Same tiling and register layout, but the score MFMAs run one key tile
// ahead of the softmax: in trip j a wave issues S^T(j+1) = K(j+1) . Q^T, exponentiates the scores of
// tile j on the VALU while those MFMAs execute, then issues O^T += V(j)^T . P(j)^T.  K and V sit in
// separate two-deep LDS rings, K one tile ahead of V; the trip is written twice (scores ping-pong
// between two register sets, ring slots become compile-time constants) so nothing is copied.
// The running maximum is only raised -- and O rescaled -- when some query's maximum grew by more than
// 2^8; until then exponentials are taken against the stale maximum (they stay below 2^8, and O / l is
// the same quotient), which keeps the 64-register rescale off the common path.
// V swizzle: chunk c of row r -> slot c ^ (4 * (r & 3)), which keeps the four 64-byte row pieces that a
// half-wave transpose read touches on distinct banks (measured conflict-free; c ^ 2(r & 7) is not).
// NW = waves per workgroup: 4 (128 queries, two workgroups per CU) or 8 (256 queries, one workgroup per CU: the two
// wave quartets of a CU then share ONE copy of every K / V tile instead of loading one each -- half the LDS writes
// and half the L2 reads for the same fragment reads).
template <bool CAUSAL, bool BF, int NW = 4>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(2, 2))) void fa_fwd_d128_pipe(
    const half_t* __restrict__ Q, const half_t* __restrict__ K, const half_t* __restrict__ V, half_t* __restrict__ O, int BH,
    int Sq, int Sk, float scale_log2e, int q_blocks, FaLayout lay) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  static_assert(NW == 4 || NW == 8, "four or eight waves");
  constexpr int BLOCK_M = NW * 32;          // queries per workgroup
  constexpr int NI = 16 / NW;               // wave-loads per wave and tile (a wave-load = 4 rows of 256 bytes)
  constexpr int TILE_B = FA_BLOCK_N * 256;  // bytes of one K or V tile
  // (A three-slot ring for the 8-wave form -- tiles loaded two trips ahead, a trip waiting only for the loads of the
  // trip before -- measured 5 % slower than two slots: load latency is not what the trips wait for, and ring slots
  // that are not compile-time constants cost address arithmetic.)
  constexpr int VBUF = 2 * TILE_B;          // K ring at 0, V ring behind it
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r32 = lane & 31, h = lane >> 5;

  // Workgroup -> (batch * head, unit).  A unit is one 128-query block; with the causal mask it is a pair of
  // blocks, the i-th from the end and the i-th from the start, processed one after the other, so that every
  // workgroup walks the same number of key tiles (q_blocks + 1) and the grid has no long tail.
  const int units = CAUSAL ? (q_blocks + 1) / 2 : q_blocks;
  int bh, unit;
  {
    const int pid = blockIdx.x;
    if (((BH / lay.group) & 7) == 0) {
      // all units of the `group` query heads that share one K/V head sit on one XCD
      const int xcd = pid & 7, loc = pid >> 3, per_kv = units * lay.group;
      const int w = loc % per_kv;
      bh = ((loc / per_kv) * 8 + xcd) * lay.group + w / units;
      unit = w % units;
    } else {
      bh = pid / units;
      unit = pid % units;
    }
  }
  const int b_idx = bh / lay.H;
  const int h_idx = bh - b_idx * lay.H, hk_idx = h_idx / lay.group;
  const int causal_off = Sk - Sq;
  const half_t* Qb = Q + b_idx * lay.q_b + h_idx * lay.q_h;
  const half_t* Kb = K + b_idx * lay.k_b + hk_idx * lay.k_h;
  const half_t* Vb = V + b_idx * lay.v_b + hk_idx * lay.v_h;
  half_t* Ob = O + b_idx * lay.o_b + h_idx * lay.o_h;

  // LDS addresses of the eight K fragment reads of a 32-key half tile (ks = 0..7), formed once: left to the
  // compiler inside the pass loop, the offsets are hoisted as integers and each read then adds the LDS base to
  // one again, vector instructions that upset the pinned MFMA / softmax interleave
  typedef const __attribute__((address_space(3))) half8* lds_half8_t;
  unsigned k_frag[8];
  {
    const int kb0 = r32 * 256 + ((h ^ (lane & 15)) * 16);
#pragma unroll
    for (int ks = 0; ks < 8; ks++) {
      k_frag[ks] = (unsigned)(uintptr_t)MI355_LDS(char, lds + (kb0 ^ (ks * 32)));
      asm volatile("" : "+v"(k_frag[ks]));  // one opaque value per read: nothing to re-derive it from
    }
  }
  // LDS addresses of the V^T transpose reads (slot 0 of the V ring; dt = 0..3), same treatment
  unsigned v_frag[4];
  {
    const int i16 = lane & 15, g16 = lane >> 4;
    const int v_row = 4 * (g16 >> 1) + (i16 >> 2);
    const int vb0 = VBUF + v_row * 256 + (i16 >> 2) * 64 + (2 * (g16 & 1) + ((i16 & 3) >> 1)) * 16 + (i16 & 1) * 8;
#pragma unroll
    for (int dt = 0; dt < 4; dt++) {
      v_frag[dt] = (unsigned)(uintptr_t)MI355_LDS(char, lds + (vb0 ^ (dt * 64)));
      asm volatile("" : "+v"(v_frag[dt]));
    }
  }
  for (int pass = 0; pass < (CAUSAL ? 2 : 1); pass++) {
  const int qb = CAUSAL ? (pass == 0 ? q_blocks - 1 - unit : unit) : unit;
  if (CAUSAL && pass == 1 && 2 * unit == q_blocks - 1) break;  // the middle block of an odd count has no partner
  const int q0 = qb * BLOCK_M;
  const int wq0 = q0 + wave * 32;
  const int q_row = wq0 + r32;
  const bool q_ok = q_row < Sq;

  int k_end = Sk;
  if (CAUSAL) {
    int last_q = q0 + BLOCK_M - 1;
    if (last_q > Sq - 1) last_q = Sq - 1;
    int lim = last_q + causal_off + 1;
    if (lim < k_end) k_end = lim;
  }
  const int n_tiles = k_end > 0 ? (k_end + FA_BLOCK_N - 1) / FA_BLOCK_N : 0;

  half8 qf[8];
#pragma unroll
  for (int ks = 0; ks < 8; ks++) {
    if (q_ok) {
      // scale . log2(e) is folded into Q (rounded to the 16-bit format again: a relative error of 2^-11 per
      // element for fp16, 2^-8 for bf16 -- the same size as the rounding of P), so the MFMA delivers exponents of
      // 2 directly
      const half8 raw = *reinterpret_cast<const half8*>(Qb + (size_t)q_row * lay.q_r + ks * 16 + h * 8);
#pragma unroll
      for (int e = 0; e < 8; e++) qf[ks][e] = cvt16<BF>(to_f32<BF>(raw[e]) * scale_log2e);
    } else {
#pragma unroll
      for (int e = 0; e < 8; e++) qf[ks][e] = (half_t)0;
    }
  }

  const int lrow = lane >> 4, lslot = lane & 15;
  const int k_chunk = lslot ^ ((wave * 4 + lrow) & 15);
  const int v_chunk = lslot ^ (4 * lrow);
  // Global -> LDS through a buffer descriptor rebuilt per tile on the scalar unit (base = first row of the tile,
  // size = up to the end of the tile's last valid row): the per-lane byte offset is loop-invariant, rows at or
  // beyond Sk read zeros (they are masked out of the softmax), and no 64-bit vector address arithmetic is left.
  const unsigned k_rb = lay.k_r * 2, v_rb = lay.v_r * 2;  // row strides in bytes
  const unsigned k_voff = (wave * 4 + lrow) * k_rb + k_chunk * 16;
  const unsigned v_voff = (wave * 4 + lrow) * v_rb + v_chunk * 16;
  auto issue_kv = [&](const half_t* base, unsigned rb, unsigned voff, int tile, int lds_off) {
    char* dst = lds + lds_off + wave * 1024;
    const int row0 = tile * FA_BLOCK_N;
    int rem = Sk - row0;
    rem = rem > FA_BLOCK_N ? FA_BLOCK_N : rem;
    const buffer_rsrc_t rs = make_buffer(reinterpret_cast<const char*>(base) + (size_t)row0 * rb, (unsigned)(rem - 1) * rb + 256u);
#pragma unroll
    for (int i = 0; i < NI; i++) buffer_load_lds_16B(rs, voff + (unsigned)(i * NW * 4) * rb, 0, dst + i * NW * 1024);
  };

  floatx16 oacc[4];
#pragma unroll
  for (int dt = 0; dt < 4; dt++)
#pragma unroll
    for (int r = 0; r < 16; r++) oacc[dt][r] = 0.f;
  // The running maximum m of a query lives negated in all 16 registers of `negm`, which every score MFMA chain
  // starts from: the accumulators then hold log2-domain scores relative to m and feed v_exp_f32 unchanged.
  // (A lane owns one query column of S^T, so the 16 values of a lane are equal.)
  floatx16 negm;
#pragma unroll
  for (int r = 0; r < 16; r++) negm[r] = 0.f;
  float l_run = 0.f;
  // m is raised -- and O rescaled -- only when a score exceeds it by more than 2^8; -inf until the query has
  // seen its first unmasked key, so that the first one always sets m
  float grow_thr = -INFINITY;
  constexpr float kRescaleThreshold = 8.f;

  auto wave_active = [&](int tile) { return !CAUSAL || (tile * FA_BLOCK_N <= wq0 + 31 + causal_off); };

  // S^T = K(slot) . Q^T, 16 MFMAs
  auto scores = [&](int koff, floatx16* s) {
#pragma unroll
    for (int t = 0; t < 2; t++) {
#pragma unroll
      for (int ks = 0; ks < 8; ks++) {
        half8 kf = *(lds_half8_t)(uintptr_t)(k_frag[ks] + (unsigned)(koff + t * 8192));
        s[t] = mfma16<BF>(kf, qf[ks], ks == 0 ? negm : s[t]);
      }
    }
  };

  // softmax of tile `tile` (scores in s) and O^T += V(slot)^T . P^T
  auto softmax_pv = [&](auto masked_tag, int tile, auto voff_tag, floatx16* s, int koff_next, floatx16* s_next) {
    constexpr bool MASKED = decltype(masked_tag)::value;
    constexpr int VOFF = decltype(voff_tag)::value;  // byte offset of the V ring slot to read
    if (MASKED) {
      const int key0 = tile * FA_BLOCK_N;
      const bool need_mask = (CAUSAL && (key0 + FA_BLOCK_N - 1 > wq0 + causal_off)) || (key0 + FA_BLOCK_N > Sk);
      if (need_mask) {
        const int lim = CAUSAL ? (q_row + causal_off < Sk - 1 ? q_row + causal_off : Sk - 1) : Sk - 1;
        const int rel = lim - key0 - 4 * h;  // last visible key, relative to the tile and to this lane's rows
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
          for (int r = 0; r < 16; r++)
          {
            // -inf where the key is beyond `rel`, by bit selection: a compare-and-select per score would hold
            // a scalar register pair per score and push loop-invariant scalars out of the register file
            const unsigned hide = (unsigned)((rel - (32 * t + 8 * (r >> 2) + (r & 3))) >> 31);
            const float sv = s[t][r];  // (bit_cast straight from a vector element miscompiles)
            s[t][r] = __builtin_bit_cast(float, (hide & 0xFF800000u) | (~hide & __builtin_bit_cast(unsigned, sv)));
          }
      }
    }
    float mx = s[0][0];
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
      for (int r = 0; r < 16; r++) mx = fmaxf(mx, s[t][r]);
    if (__builtin_amdgcn_ballot_w64(mx > grow_thr) != 0) {
      // rare: some query's scores outgrew its maximum (or it saw its first key).  The other half of a query's
      // keys sits in lane ^ 32; both lanes take the same decision.
      const float mxx = fmaxf(mx, __shfl_xor(mx, 32));
      const bool fresh = grow_thr == -INFINITY;
      const float delta = fresh ? (mxx == -INFINITY ? 0.f : mxx) : fmaxf(mxx, 0.f);
      const float alpha = fresh ? 1.f : __builtin_amdgcn_exp2f(-delta);
      if (mxx != -INFINITY) grow_thr = kRescaleThreshold;
      l_run *= alpha;
#pragma unroll
      for (int dt = 0; dt < 4; dt++)
#pragma unroll
        for (int r = 0; r < 16; r++) oacc[dt][r] *= alpha;
#pragma unroll
      for (int t = 0; t < 2; t++)
#pragma unroll
        for (int r = 0; r < 16; r++) s[t][r] -= delta;
#pragma unroll
      for (int r = 0; r < 16; r++) negm[r] -= delta;
    }
    half8 pf[4];
    float psum = 0.f;
    // Scores of the next tile and exponentials of this one in one straight-line block: a wave issues in
    // order, so only VALU work placed between two MFMAs runs while the first occupies the matrix pipe.
    // (Past the last tile the scores are computed from stale LDS bytes and never used.)
    __builtin_amdgcn_sched_barrier(0);
    scores(koff_next, s_next);
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
      for (int r = 0; r < 16; r += 2) {
        const half2v pp = cvt16x2<BF>(__builtin_amdgcn_exp2f(s[t][r]), __builtin_amdgcn_exp2f(s[t][r + 1]));
        psum = dot2_ones<BF>(pp, psum);  // sums what the second MFMA multiplies
        pf[t * 2 + (r >> 3)][r & 7] = pp[0];
        pf[t * 2 + (r >> 3)][(r & 7) + 1] = pp[1];
      }
    // order: 3 K fragment reads up front, then per score MFMA one more read and the work of two scores
    // (two exp, one cvt_pk, one dot2) -- a fragment is requested two MFMAs before its use
    __builtin_amdgcn_sched_group_barrier(0x100, 3, 0);
#pragma unroll
    for (int i = 0; i < 13; i++) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x400, 2, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, 2, 0);
    }
#pragma unroll
    for (int i = 0; i < 3; i++) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x400, 2, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, 2, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  
    l_run += psum;
    // O^T += V^T P^T: 16 MFMAs, each V^T fragment (two transpose reads) requested two MFMAs ahead.
    // The reads and their waits are inline assembly: a transpose read the compiler can see makes it wait for
    // EVERY direct-to-LDS load in flight first (it cannot tell that the loads fill other ring slots), which put a
    // vmcnt(0) -- the loads issued at the head of this trip -- in the middle of every trip.  In this block nothing
    // else counts in lgkmcnt: LDS returns in order, so MFMA i may run once at most the reads of fragments i + 1
    // and i + 2 (two each) are outstanding.  Each wait names the fragment's registers, so no use moves above it.
    half4 vlo[3], vhi[3];
    auto vr = [&](auto itag) {  // i = t16*4 + dt
      constexpr int i = decltype(itag)::value;
      constexpr int off = VOFF + (i >> 2) * 4096;
      half4 &lo = vlo[i % 3], &hi = vhi[i % 3];  // (operands of an assembly statement do not capture by themselves)
      const unsigned addr = v_frag[i & 3];
      asm volatile("ds_read_b64_tr_b16 %0, %2 offset:%3\n\tds_read_b64_tr_b16 %1, %2 offset:%4"
                   : "=&v"(lo), "=&v"(hi)
                   : "v"(addr), "n"(off), "n"(off + 2048));
    };
    vr(std::integral_constant<int, 0>{});
    vr(std::integral_constant<int, 1>{});
    static_for<0, 16>([&](auto itag) {
      constexpr int i = decltype(itag)::value;
      if constexpr (i + 2 < 16) vr(std::integral_constant<int, i + 2>{});
      half4 &lo = vlo[i % 3], &hi = vhi[i % 3];
      if constexpr (i + 2 < 16)
        asm volatile("s_waitcnt lgkmcnt(4)" : "+v"(lo), "+v"(hi));
      else if constexpr (i + 1 < 16)
        asm volatile("s_waitcnt lgkmcnt(2)" : "+v"(lo), "+v"(hi));
      else
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(lo), "+v"(hi));
      const half8 vf = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      oacc[i & 3] = mfma16<BF>(vf, pf[i >> 2], oacc[i & 3]);
      __builtin_amdgcn_sched_barrier(0);
    });
  };

  floatx16 sa[2], sb[2];
  if (n_tiles > 0) {
    issue_kv(Kb, k_rb, k_voff, 0, 0);
    issue_kv(Vb, v_rb, v_voff, 0, VBUF);
    if (n_tiles > 1) issue_kv(Kb, k_rb, k_voff, 1, TILE_B);
    wait_vmcnt0();
    __syncthreads();
    if (wave_active(0)) scores(0, sa);
    // trip 0 overwrites the K(0) slot with K(2): every wave must have read its K(0) fragments first
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __syncthreads();
  }

  // trip j (PAR = j & 1): loads for K(j+2) and V(j+1); scores of tile j+1; softmax + PV of tile j
  auto trip = [&](auto par_tag, int j, floatx16* s_cur, floatx16* s_next) {
    constexpr int PAR = decltype(par_tag)::value;
    constexpr int K_CUR = PAR * TILE_B, K_NEXT = (1 - PAR) * TILE_B, V_CUR = PAR * TILE_B, V_NEXT = VBUF + (1 - PAR) * TILE_B;
    if (j + 2 < n_tiles) issue_kv(Kb, k_rb, k_voff, j + 2, K_CUR);
    if (j + 1 < n_tiles) issue_kv(Vb, v_rb, v_voff, j + 1, V_NEXT);
    if (wave_active(j)) softmax_pv(std::true_type{}, j, std::integral_constant<int, V_CUR>{}, s_cur, K_NEXT, s_next);  // idle from here on otherwise
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __syncthreads();
  };
  for (int j = 0; j < n_tiles; j += 2) {
    trip(std::integral_constant<int, 0>{}, j, sa, sb);
    if (j + 1 < n_tiles) trip(std::integral_constant<int, 1>{}, j + 1, sb, sa);
  }

  const float l_tot = l_run + __shfl_xor(l_run, 32);
  const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
  {
    // Output through LDS (the K / V rings are idle: the last trip ended with a barrier): a lane holds 64 of its query's 128
    // values in 4-value pieces; each wave assembles its 32 rows x 256 bytes in a private region (chunk c of row r in
    // slot c ^ (r & 15)), reads whole 16-byte chunks back and stores full rows -- 8 stores of 16 bytes per lane instead
    // of 16 of 8 bytes that each touch 32 rows.
    char* ep = lds + wave * 8192;
    // (the lane id is taken afresh: addresses derived from the kernel's own `lane` are invariant over the passes of a
    // causal pair, get hoisted in front of the pass loop and then occupy registers all through the key walk)
    const int el = CAUSAL ? opaque_lane_id() : lane;
    const int e32 = el & 31, eh = el >> 5;
#pragma unroll
    for (int dt = 0; dt < 4; dt++)
#pragma unroll
      for (int q = 0; q < 4; q++) {
        half4 v = {cvt16<BF>(oacc[dt][4 * q] * inv), cvt16<BF>(oacc[dt][4 * q + 1] * inv), cvt16<BF>(oacc[dt][4 * q + 2] * inv),
                   cvt16<BF>(oacc[dt][4 * q + 3] * inv)};
        *reinterpret_cast<half4*>(ep + e32 * 256 + (((dt * 4 + q) ^ (e32 & 15)) * 16) + 8 * eh) = v;
      }
    const int er = el >> 4, ec = el & 15;
#pragma unroll
    for (int it = 0; it < 8; it++) {
      const int row = it * 4 + er;
      const half8 v = *reinterpret_cast<const half8*>(ep + row * 256 + ((ec ^ (row & 15)) * 16));
      if (wq0 + row < Sq) *reinterpret_cast<half8*>(Ob + (size_t)(wq0 + row) * lay.o_r + ec * 8) = v;
    }
    if (CAUSAL) __syncthreads();  // the next pass loads K / V tiles over these regions
  }
  }  // pass
}


// The pipelined form on v_mfma_f32_16x16x32 (variant "..._m16").  Same tiles, rings, loads, passes and barriers as
// fa_fwd_d128_pipe; what changes is the MFMA shape and with it every fragment layout.  On benchmark-like data a
// 16x16x32 MFMA costs the board less energy per flop than a 32x32x16 (register-only loops with this tile's structure:
// 0.75 against 0.66 of the datasheet peak for the MFMAs alone, 0.60 against 0.57 with the softmax), and the prefill
// kernel runs against the power limit.
// A wave's 32 queries are two groups of 16 (qg), a 64-key tile four groups of 16 keys (kg), d = 128 four steps of 32 (ks),
// eight groups of 16 (dg).  With q16 = lane & 15, g = lane >> 4:
//   S^T(kg, qg) = K(kg) . Q(qg)^T:  A = K rows kg*16 + q16, d = 32 ks + 8 g .. + 7 (one 16-byte chunk from LDS, shared by
//       both query groups); B = Q row qg*16 + q16, same d (registers); the lane receives keys kg*16 + 4 g + r, r < 4, of
//       query qg*16 + q16: it owns one query per group and a quarter of the tile's keys.
//   O^T(dg, qg) += V(dg)^T . P(qg)^T over two steps of 32 keys (key groups 2 st, 2 st + 1): the lane's eight probabilities
//       (4 of either key group) are the B operand as they stand; A = V^T rows d = dg*16 + q16 for those same keys: two
//       transpose reads, each a 4 x 16 block (keys 4 g .. 4 g + 3 of one key group, 16 consecutive d) per 16 lanes.
// LDS: K chunk c of row r in slot c ^ (r & 15) as before; V chunk c of row r in slot c ^ 2 (r & 7): the 8 rows a half
// wave's transpose read touches (32 bytes each) then fall on 8 distinct 32-byte bank groups.
// SPREAD: the exponentials of a tile's second key step run behind the first key step's output MFMAs instead of behind
// the score MFMAs (vector work behind 48 of the trip's 64 MFMAs instead of 32).  Measured on 2 x 32 x 4096: ahead with
// eight waves (unmasked 475 against 484 us), behind with four (causal 268 against 263); each form is built the way it
// runs faster.
template <bool CAUSAL, bool BF, int NW, bool SPREAD, bool PAGED = false>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(2, 2))) void fa_fwd_d128_m16(
    const half_t* __restrict__ Q, const half_t* __restrict__ K, const half_t* __restrict__ V, half_t* __restrict__ O, int BH,
    int Sq, int Sk_arg, float scale_log2e, int q_blocks, FaLayout lay, FaPaged pg) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  static_assert(NW == 4 || !PAGED, "the paged form maps one page to one wave-load of a 4-wave workgroup");
  constexpr int BLOCK_M = NW * 32, NI = 16 / NW;
  constexpr int TILE_B = FA_BLOCK_N * 256, VBUF = 2 * TILE_B;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int q16 = lane & 15, g = lane >> 4;

  const int units = CAUSAL ? (q_blocks + 1) / 2 : q_blocks;
  int bh, unit;
  {
    const int pid = blockIdx.x;
    if (((BH / lay.group) & 7) == 0) {
      const int xcd = pid & 7, loc = pid >> 3, per_kv = units * lay.group;
      const int w = loc % per_kv;
      bh = ((loc / per_kv) * 8 + xcd) * lay.group + w / units;
      unit = w % units;
    } else {
      bh = pid / units;
      unit = pid % units;
    }
  }
  int b_idx = bh / lay.H;
  const int h_idx = bh - b_idx * lay.H, hk_idx = h_idx / lay.group;
  int Sk = Sk_arg;
  if constexpr (PAGED) {
    // Sequences differ in length and workgroups are dispatched in grid order: take the sequences longest first,
    // so that the short ones make up the tail.  Thread t counts the sequences that come before sequence t.
    const int num_seqs = BH / lay.H;
    if (num_seqs > 1 && num_seqs <= 256) {
      int* pick = reinterpret_cast<int*>(lds);
      const int t = threadIdx.x;
      if (t < num_seqs) {
        const int mine = pg.seq_lens[t];
        int rank = 0;
        for (int j = 0; j < num_seqs; j++) {
          const int other = pg.seq_lens[j];
          rank += (other > mine) || (other == mine && j < t);
        }
        if (rank == b_idx) *pick = t;
      }
      __syncthreads();
      b_idx = __builtin_amdgcn_readfirstlane(*pick);
      __syncthreads();  // the slot is part of the K ring
    }
    Sk = __builtin_amdgcn_readfirstlane(pg.seq_lens[b_idx]);
    const int cap = (pg.max_pages * 16) << pg.page_shift;
    Sk = Sk < 0 ? 0 : (Sk > cap ? cap : Sk);
  }
  const int causal_off = Sk - Sq;
  const half_t* Qb = Q + b_idx * lay.q_b + h_idx * lay.q_h;
  const half_t* Kb = K + (PAGED ? 0 : b_idx * lay.k_b) + hk_idx * lay.k_h;
  const half_t* Vb = V + (PAGED ? 0 : b_idx * lay.v_b) + hk_idx * lay.v_h;
  half_t* Ob = O + b_idx * lay.o_b + h_idx * lay.o_h;

  // fragment read addresses, opaque (see fa_fwd_d128_pipe): K by step over d, V by d group
  typedef const __attribute__((address_space(3))) half8* lds_half8_t;
  unsigned k_frag[4], v_frag[8];
  {
#pragma unroll
    for (int ks = 0; ks < 4; ks++) {
      k_frag[ks] = (unsigned)(uintptr_t)MI355_LDS(char, lds + q16 * 256 + (((ks * 4 + g) ^ q16) * 16));
      asm volatile("" : "+v"(k_frag[ks]));
    }
    // lane i of a 16-lane group hands in row i / 4, halfs 4 (i % 4) .. + 3 of the 4 x 16 block
    const int row = 4 * g + (q16 >> 2), rr = row & 7;
    const int vb0 = VBUF + row * 256 + (rr << 5) + 16 * ((q16 & 3) >> 1) + 8 * (q16 & 1);
#pragma unroll
    for (int dg = 0; dg < 8; dg++) {
      v_frag[dg] = (unsigned)(uintptr_t)MI355_LDS(char, lds + (vb0 ^ (dg << 5)));
      asm volatile("" : "+v"(v_frag[dg]));
    }
  }

  for (int pass = 0; pass < (CAUSAL ? 2 : 1); pass++) {
  const int qb = CAUSAL ? (pass == 0 ? q_blocks - 1 - unit : unit) : unit;
  if (CAUSAL && pass == 1 && 2 * unit == q_blocks - 1) break;
  const int q0 = qb * BLOCK_M;
  const int wq0 = q0 + wave * 32;

  int k_end = Sk;
  if (CAUSAL) {
    int last_q = q0 + BLOCK_M - 1;
    if (last_q > Sq - 1) last_q = Sq - 1;
    int lim = last_q + causal_off + 1;
    if (lim < k_end) k_end = lim;
  }
  const int n_tiles = k_end > 0 ? (k_end + FA_BLOCK_N - 1) / FA_BLOCK_N : 0;

  // Q fragments [query group][step over d], scale . log2(e) folded in and rounded to the 16-bit format again
  half8 qf[2][4];
#pragma unroll
  for (int qg = 0; qg < 2; qg++) {
    const int q_row = wq0 + qg * 16 + q16;
#pragma unroll
    for (int ks = 0; ks < 4; ks++) {
      if (q_row < Sq) {
        const half8 raw = *reinterpret_cast<const half8*>(Qb + (size_t)q_row * lay.q_r + ks * 32 + g * 8);
#pragma unroll
        for (int e = 0; e < 8; e++) qf[qg][ks][e] = cvt16<BF>(to_f32<BF>(raw[e]) * scale_log2e);
      } else {
#pragma unroll
        for (int e = 0; e < 8; e++) qf[qg][ks][e] = (half_t)0;
      }
    }
  }

  const int lrow = lane >> 4, lslot = lane & 15;
  const int k_chunk = lslot ^ ((wave * 4 + lrow) & 15);
  const int v_chunk = lslot ^ (2 * (((wave & 1) << 2) | lrow));
  const unsigned k_rb = lay.k_r * 2, v_rb = lay.v_r * 2;
  const unsigned k_voff = (wave * 4 + lrow) * k_rb + k_chunk * 16;
  const unsigned v_voff = (wave * 4 + lrow) * v_rb + v_chunk * 16;
  // paged form: page ids come through the scalar cache (constant address space: the table is not written while the
  // kernel runs), one tile ahead of their use, so that no K/V load waits for a table read
  typedef const int __attribute__((address_space(4)))* table_ptr_t;
  const table_ptr_t table_row =
      PAGED ? (table_ptr_t)(unsigned long long)(pg.block_table + (size_t)b_idx * pg.max_pages) : (table_ptr_t)0;
  auto load_ids = [&](int tile, int* ids) {
    if constexpr (PAGED) {
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const int blk = tile * 4 + i, page = blk >> pg.page_shift;  // 16-token block -> its page and place in it
        const int e = page < pg.max_pages ? table_row[page] : -1;
        ids[i] = (e >= 0 && e < pg.num_pages) ? (e << pg.page_shift) + (blk & ((1 << pg.page_shift) - 1)) : -1;
      }
    }
  };
  auto issue_kv = [&](const half_t* base, unsigned rb, unsigned voff, int tile, int lds_off, const int* ids) {
    char* dst = lds + lds_off + wave * 1024;
    const int row0 = tile * FA_BLOCK_N;
    int rem = Sk - row0;
    rem = rem > FA_BLOCK_N ? FA_BLOCK_N : rem;
    if constexpr (PAGED) {
      // wave-load i covers rows 16 i .. 16 i + 15 of the tile = 16-token block 4 tile + i of the sequence: one descriptor
      // per block, sized to its valid rows (none for a block beyond the sequence or an id outside the cache)
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const int id = ids[i];
        int rows = rem - 16 * i;
        rows = rows > 16 ? 16 : rows;
        const bool ok = rows > 0 && id >= 0;
        const buffer_rsrc_t rs = make_buffer(reinterpret_cast<const char*>(base) + (size_t)(ok ? id : 0) * 16u * rb,
                                             ok ? (unsigned)(rows - 1) * rb + 256u : 0u);
        buffer_load_lds_16B(rs, voff, 0, dst + i * 4096);
      }
    } else {
      const buffer_rsrc_t rs = make_buffer(reinterpret_cast<const char*>(base) + (size_t)row0 * rb, (unsigned)(rem - 1) * rb + 256u);
#pragma unroll
      for (int i = 0; i < NI; i++) {
#if !defined(MI355_ABLATE_NO_LOADS)
        buffer_load_lds_16B(rs, voff + (unsigned)(i * NW * 4) * rb, 0, dst + i * NW * 1024);
#endif
      }
    }
  };

  floatx4 oacc[8][2];  // [d group][query group]
#pragma unroll
  for (int dg = 0; dg < 8; dg++)
#pragma unroll
    for (int qg = 0; qg < 2; qg++) oacc[dg][qg] = floatx4{0.f, 0.f, 0.f, 0.f};
  // the negated running maximum of the lane's query in either group, four equal values: the addend of every score chain
  floatx4 negm[2] = {floatx4{0.f, 0.f, 0.f, 0.f}, floatx4{0.f, 0.f, 0.f, 0.f}};
  float l_run[2] = {0.f, 0.f};
  float grow_thr[2] = {-INFINITY, -INFINITY};
  constexpr float kRescaleThreshold = 8.f;

  auto wave_active = [&](int tile) { return !CAUSAL || (tile * FA_BLOCK_N <= wq0 + 31 + causal_off); };
  auto kread = [&](int f, int koff) {  // K fragment f = kg * 4 + ks of the slot at koff
#if defined(MI355_ABLATE_NO_K_READS)
    half8 stale = qf[0][f & 3];
    asm volatile("" : "+v"(stale));
    return stale;
#else
    return *(lds_half8_t)(uintptr_t)(k_frag[f & 3] + (unsigned)(koff + (f >> 2) * 4096));
#endif
  };
  // S^T of one tile, no softmax beside it (a pass's first tile)
  auto scores = [&](int koff, floatx4 (*s)[2]) {
#pragma unroll
    for (int f = 0; f < 16; f++) {
      const int kg = f >> 2, ks = f & 3;
      const half8 kf = kread(f, koff);
#pragma unroll
      for (int qg = 0; qg < 2; qg++) s[kg][qg] = mfma16_16x16x32<BF>(kf, qf[qg][ks], ks == 0 ? negm[qg] : s[kg][qg]);
    }
  };

  auto softmax_pv = [&](int tile, auto voff_tag, floatx4 (*s)[2], int koff_next, floatx4 (*s_next)[2]) {
    constexpr int VOFF = decltype(voff_tag)::value;
    {
      const int key0 = tile * FA_BLOCK_N;
      const bool need_mask = (CAUSAL && (key0 + FA_BLOCK_N - 1 > wq0 + causal_off)) || (key0 + FA_BLOCK_N > Sk);
      if (need_mask) {
#pragma unroll
        for (int qg = 0; qg < 2; qg++) {
          const int q_row = wq0 + qg * 16 + q16;
          const int lim = CAUSAL ? (q_row + causal_off < Sk - 1 ? q_row + causal_off : Sk - 1) : Sk - 1;  // last visible key
          const int rel = lim - key0 - 4 * g;
#pragma unroll
          for (int kg = 0; kg < 4; kg++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
              const unsigned hide = (unsigned)((rel - (16 * kg + r)) >> 31);
              const float sv = s[kg][qg][r];
              s[kg][qg][r] = __builtin_bit_cast(float, (hide & 0xFF800000u) | (~hide & __builtin_bit_cast(unsigned, sv)));
            }
        }
      }
    }
    float mx[2];
#pragma unroll
    for (int qg = 0; qg < 2; qg++) {
      mx[qg] = s[0][qg][0];
#pragma unroll
      for (int kg = 0; kg < 4; kg++)
#pragma unroll
        for (int r = 0; r < 4; r++) mx[qg] = fmaxf(mx[qg], s[kg][qg][r]);
    }
    if (__builtin_amdgcn_ballot_w64(mx[0] > grow_thr[0] || mx[1] > grow_thr[1]) != 0) {
      // rare: some query's scores outgrew its maximum (or it saw its first key).  A query's keys are spread over the
      // four lanes q16 + 16 g; they take the same decision.
#pragma unroll
      for (int qg = 0; qg < 2; qg++) {
        float mxx = fmaxf(mx[qg], __shfl_xor(mx[qg], 16));
        mxx = fmaxf(mxx, __shfl_xor(mxx, 32));
        if (mxx > grow_thr[qg]) {
          const bool fresh = grow_thr[qg] == -INFINITY;
          const float delta = fresh ? mxx : fmaxf(mxx, 0.f);  // (mxx > -inf here)
          const float alpha = fresh ? 1.f : __builtin_amdgcn_exp2f(-delta);
          grow_thr[qg] = kRescaleThreshold;
          l_run[qg] *= alpha;
#pragma unroll
          for (int dg = 0; dg < 8; dg++)
#pragma unroll
            for (int r = 0; r < 4; r++) oacc[dg][qg][r] *= alpha;
#pragma unroll
          for (int kg = 0; kg < 4; kg++)
#pragma unroll
            for (int r = 0; r < 4; r++) s[kg][qg][r] -= delta;
#pragma unroll
          for (int r = 0; r < 4; r++) negm[qg][r] -= delta;
        }
      }
    }
    // Scores of the next tile and the softmax of this one, step by step.  Step i = MFMA (kg, ks, qg) = (i / 8, (i / 2) % 4,
    // i % 2) of the next tile -- a K fragment serves both query groups back to back and is requested three fragments
    // ahead -- and one exponential of this tile, taken in the order the output MFMAs want the probabilities: key step,
    // query group, key group of the pair, r.  Every second step packs a pair; its dot2 (the row sum of what the second
    // contraction multiplies) runs one pair behind.  The empty statements tie the vector work to its step.
    half8 pf[2][2];  // [query group][key step]
    float psum[2] = {0.f, 0.f};
    half2v pp_prev = {(half_t)0, (half_t)0};
    // exponential e of the tile (0..31), in the order the output MFMAs want the probabilities: key step e / 16, query group
    // (e / 8) % 2, key group of the pair (e / 4) % 2, r = e % 4.  Every second one packs a pair; the pair's dot2 (the row
    // sum of what the second contraction multiplies) runs one pair behind.  The empty statements tie the work to its step.
    float e_even = 0.f;
    auto expo = [&](int e) {
      const int st = e >> 4, eq = (e >> 3) & 1, ekg = 2 * st + ((e >> 2) & 1), r = e & 3;
#if defined(MI355_ABLATE_NO_EXP)
      const float ev = s[ekg][eq][r];
#else
      const float ev = __builtin_amdgcn_exp2f(s[ekg][eq][r]);
#endif
      if (e & 1) {
        if (e > 1) psum[((e - 2) >> 3) & 1] = dot2_ones<BF>(pp_prev, psum[((e - 2) >> 3) & 1]);
        half2v pp = cvt16x2<BF>(e_even, ev);
        asm volatile("" : "+v"(pp), "+v"(psum[0]), "+v"(psum[1]));
        pf[eq][st][((e >> 2) & 1) * 4 + r - 1] = pp[0];
        pf[eq][st][((e >> 2) & 1) * 4 + r] = pp[1];
        pp_prev = pp;
      } else {
        e_even = ev;
        asm volatile("" : "+v"(e_even));
      }
    };
    // Scores of the next tile, step by step: step i = MFMA (kg, ks, qg) = (i / 8, (i / 2) % 4, i % 2) -- a K fragment serves
    // both query groups back to back and is requested three fragments ahead -- with the exponentials of this tile's
    // FIRST key step behind every second MFMA; those of the second key step run behind the first key step's output
    // MFMAs below, so that the vector work is spread over 48 of the trip's 64 MFMAs.
    __builtin_amdgcn_sched_barrier(0);
    {
      half8 kf[4];
      kf[0] = kread(0, koff_next);
      kf[1] = kread(1, koff_next);
      kf[2] = kread(2, koff_next);
#pragma unroll
      for (int i = 0; i < 32; i++) {
        const int f = i >> 1, kg = f >> 2, ks = f & 3, qg = i & 1;
        if (qg == 0 && f + 3 < 16) kf[(f + 3) & 3] = kread(f + 3, koff_next);
        s_next[kg][qg] = mfma16_16x16x32<BF>(kf[f & 3], qf[qg][ks], ks == 0 ? negm[qg] : s_next[kg][qg]);
        if (SPREAD) {
          if (i & 1) expo(i >> 1);
        } else {
          expo(i);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // O^T += V^T P^T: step f = (key step, d group) = (f / 8, f % 8), two MFMAs (one per query group) on one V^T fragment
    // (two transpose reads, in assembly with their waits, see fa_fwd_d128_pipe), requested two fragments ahead.
    half4 vlo[3], vhi[3];
    auto vr = [&](auto ftag) {  // fragment f = st * 8 + dg
      constexpr int f = decltype(ftag)::value;
      constexpr int off = VOFF + (f >> 3) * 8192;  // key groups 2 st and 2 st + 1: 16 rows of 256 bytes apart
      half4 &lo = vlo[f % 3], &hi = vhi[f % 3];
      const unsigned addr = v_frag[f & 7];
#if defined(MI355_ABLATE_NO_V_READS)
      asm volatile("" : "=&v"(lo), "=&v"(hi) : "v"(addr));
#else
      asm volatile("ds_read_b64_tr_b16 %0, %2 offset:%3\n\tds_read_b64_tr_b16 %1, %2 offset:%4"
                   : "=&v"(lo), "=&v"(hi)
                   : "v"(addr), "n"(off), "n"(off + 4096));
#endif
    };
    vr(std::integral_constant<int, 0>{});
    vr(std::integral_constant<int, 1>{});
    static_for<0, 16>([&](auto ftag) {
      constexpr int f = decltype(ftag)::value;
      constexpr int st = f >> 3, dg = f & 7;
      if constexpr (f + 2 < 16) vr(std::integral_constant<int, f + 2>{});
      half4 &lo = vlo[f % 3], &hi = vhi[f % 3];
      if constexpr (f + 2 < 16)
        asm volatile("s_waitcnt lgkmcnt(4)" : "+v"(lo), "+v"(hi));
      else if constexpr (f + 1 < 16)
        asm volatile("s_waitcnt lgkmcnt(2)" : "+v"(lo), "+v"(hi));
      else
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(lo), "+v"(hi));
      const half8 vf = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      oacc[dg][0] = mfma16_16x16x32<BF>(vf, pf[0][st], oacc[dg][0]);
      if constexpr (SPREAD && f < 8) expo(16 + 2 * f);
      __builtin_amdgcn_sched_barrier(0);
      oacc[dg][1] = mfma16_16x16x32<BF>(vf, pf[1][st], oacc[dg][1]);
      if constexpr (SPREAD && f < 8) expo(16 + 2 * f + 1);
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (f == 7 || (!SPREAD && f == 0)) {  // the last pair's dot2 (it belongs to query group 1)
        if (SPREAD || f == 0) {
          psum[1] = dot2_ones<BF>(pp_prev, psum[1]);
          l_run[0] += psum[0];
          l_run[1] += psum[1];
        }
      }
    });
  };

  floatx4 sa[4][2], sb[4][2];  // scores [key group][query group], two tiles
  int k_ids[4] = {-1, -1, -1, -1}, v_ids[4] = {-1, -1, -1, -1};  // paged form: ids of the next K tile and the next V tile to fetch
  if (n_tiles > 0) {
    load_ids(0, k_ids);
    issue_kv(Kb, k_rb, k_voff, 0, 0, k_ids);
    issue_kv(Vb, v_rb, v_voff, 0, VBUF, k_ids);
    load_ids(1, v_ids);
    if (n_tiles > 1) issue_kv(Kb, k_rb, k_voff, 1, TILE_B, v_ids);
    load_ids(2, k_ids);  // what trip 0 issues: K(2) and V(1)
    wait_vmcnt0();
    __syncthreads();
    if (wave_active(0)) scores(0, sa);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __syncthreads();
  }
  auto trip = [&](auto par_tag, int j, floatx4 (*s_cur)[2], floatx4 (*s_next)[2]) {
    constexpr int PAR = decltype(par_tag)::value;
    constexpr int K_CUR = PAR * TILE_B, K_NEXT = (1 - PAR) * TILE_B, V_CUR = VBUF + PAR * TILE_B, V_NEXT = VBUF + (1 - PAR) * TILE_B;
    if (j + 2 < n_tiles) issue_kv(Kb, k_rb, k_voff, j + 2, K_CUR, k_ids);
    if (j + 1 < n_tiles) issue_kv(Vb, v_rb, v_voff, j + 1, V_NEXT, v_ids);
    if constexpr (PAGED) {
      // the next trip fetches V(j+2) -- the tile whose ids K just used -- and K(j+3)
#pragma unroll
      for (int i = 0; i < 4; i++) v_ids[i] = k_ids[i];
      load_ids(j + 3, k_ids);
    }
    if (wave_active(j)) softmax_pv(j, std::integral_constant<int, V_CUR - VBUF>{}, s_cur, K_NEXT, s_next);
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
#if !defined(MI355_ABLATE_NO_BARRIERS)
    __syncthreads();
#endif
  };
  for (int j = 0; j < n_tiles; j += 2) {
    trip(std::integral_constant<int, 0>{}, j, sa, sb);
    if (j + 1 < n_tiles) trip(std::integral_constant<int, 1>{}, j + 1, sb, sa);
  }

  {
    // Output through LDS (the rings are idle: the last trip ended with a barrier): each wave assembles its 32 rows x 256
    // bytes in a private region (chunk c of row r in slot c ^ (r & 15)) from 8-byte pieces -- the lane holds d = 16 dg +
    // 4 g .. + 3 of its query in either group -- and stores whole rows, 16 bytes per lane.
    char* ep = lds + wave * 8192;
    const int el = CAUSAL ? opaque_lane_id() : lane;  // (see fa_fwd_d128_pipe)
    const int e16 = el & 15, eg = el >> 4;
#pragma unroll
    for (int qg = 0; qg < 2; qg++) {
      float l_tot = l_run[qg] + __shfl_xor(l_run[qg], 16);
      l_tot += __shfl_xor(l_tot, 32);
      const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
#pragma unroll
      for (int dg = 0; dg < 8; dg++) {
        const half4 v = {cvt16<BF>(oacc[dg][qg][0] * inv), cvt16<BF>(oacc[dg][qg][1] * inv), cvt16<BF>(oacc[dg][qg][2] * inv),
                         cvt16<BF>(oacc[dg][qg][3] * inv)};
        *reinterpret_cast<half4*>(ep + (qg * 16 + e16) * 256 + (((dg * 2 + (eg >> 1)) ^ e16) * 16) + 8 * (eg & 1)) = v;
      }
    }
    const int er = el >> 4, ec = el & 15;
#pragma unroll
    for (int it = 0; it < 8; it++) {
      const int row = it * 4 + er;
      const half8 v = *reinterpret_cast<const half8*>(ep + row * 256 + ((ec ^ (row & 15)) * 16));
      if (wq0 + row < Sq) *reinterpret_cast<half8*>(Ob + (size_t)(wq0 + row) * lay.o_r + ec * 8) = v;
    }
    if (CAUSAL) __syncthreads();  // the next pass loads K / V tiles over these regions
  }
  }  // pass
}

// Persistent form of fa_fwd_d128_pipe ("walk"): one workgroup per CU slot runs its passes (a pass = one block of
// NW * 32 queries of one head against its keys) one after the other -- units dealt round-robin (unit = workgroup +
// i * grid), a causal unit being a pair of blocks as above -- and overlaps what a pass costs beside its key tiles:
//  * the next pass's Q rows and first tiles (K 0, K 1, V 0) are requested in front of the current pass's LAST tile when
//    that tile has odd number (a pass of an even tile count): both K slots and V slot 0 are free from there on, the Q
//    rows land in registers that would hold the scores of a following tile (the last tile computes none), and nothing
//    waits for any of it before the finished pass has been normalised and staged.  Otherwise they are requested right
//    after the last trip;
//  * the output goes through a staging region of its own (the rings are being filled) and is stored behind the barrier
//    that opens the next pass; the stores are not waited for: they drain under the next pass's first trip, whose
//    closing wait covers them.
// A pass has at least two key tiles (the launcher checks Sk >= 128, and Sq == Sk with the mask).  The arithmetic per
// query is that of fa_fwd_d128_pipe, instruction for instruction: results are bit-identical.
template <bool CAUSAL, bool BF, int NW>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(2, 2))) void fa_fwd_d128_walk(
    const half_t* __restrict__ Q, const half_t* __restrict__ K, const half_t* __restrict__ V, half_t* __restrict__ O, int BH,
    int Sq, int Sk, float scale_log2e, int q_blocks, FaLayout lay) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  constexpr int BLOCK_M = NW * 32, NI = 16 / NW;
  constexpr int TILE_B = FA_BLOCK_N * 256, VBUF = 2 * TILE_B, STG = 4 * TILE_B;  // K ring, V ring, output staging
  constexpr int STG_ROWS = NW == 8 ? 32 : 8;  // rows a wave stages per round: 8 KiB (one round) or 2 KiB (four) per wave
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r32 = lane & 31, h = lane >> 5;
  const int causal_off = Sk - Sq;
  const int units = CAUSAL ? (q_blocks + 1) / 2 : q_blocks;
  const int total_units = BH * units;
  const bool xcd_map = ((BH / lay.group) & 7) == 0;  // the launcher makes the grid a multiple of 8 then

  // ---- passes of this workgroup, by ordinal: unit = blockIdx.x + (ord / passes per unit) * gridDim.x ----
  struct Pass {
    int ord;  // < 0: there is no such pass
    int b, hq, hk, qb, n;  // batch, query head, K/V head, query block, key tiles
  };
  auto pass_at = [&](int ord) {  // the first existing pass with ordinal >= ord
    Pass ps;
    for (;;) {
      const int pid = (int)blockIdx.x + (CAUSAL ? (ord >> 1) : ord) * (int)gridDim.x;
      if (pid >= total_units) {
        ps.ord = -1, ps.b = ps.hq = ps.hk = ps.qb = 0, ps.n = 2;
        return ps;
      }
      int bh, unit;
      if (xcd_map) {
        const int xcd = pid & 7, loc = pid >> 3, per_kv = units * lay.group;
        const int w = loc % per_kv;
        bh = ((loc / per_kv) * 8 + xcd) * lay.group + w / units;
        unit = w % units;
      } else {
        bh = pid / units;
        unit = pid % units;
      }
      const bool second = CAUSAL && (ord & 1);
      if (second && 2 * unit == q_blocks - 1) {  // the middle block of an odd count has no partner
        ord++;
        continue;
      }
      ps.ord = ord;
      ps.qb = CAUSAL ? (second ? unit : q_blocks - 1 - unit) : unit;
      ps.b = bh / lay.H;
      ps.hq = bh - ps.b * lay.H;
      ps.hk = ps.hq / lay.group;
      int k_end = Sk;
      if (CAUSAL) {
        int last_q = ps.qb * BLOCK_M + BLOCK_M - 1;
        if (last_q > Sq - 1) last_q = Sq - 1;
        const int lim = last_q + causal_off + 1;
        if (lim < k_end) k_end = lim;
      }
      ps.n = (k_end + FA_BLOCK_N - 1) / FA_BLOCK_N;
      // (the divisions run on the vector unit; the fields are wave-uniform and belong in scalar registers)
      ps.qb = __builtin_amdgcn_readfirstlane(ps.qb), ps.b = __builtin_amdgcn_readfirstlane(ps.b);
      ps.hq = __builtin_amdgcn_readfirstlane(ps.hq), ps.hk = __builtin_amdgcn_readfirstlane(ps.hk);
      ps.n = __builtin_amdgcn_readfirstlane(ps.n);
      return ps;
    }
  };

  // ---- per-lane constants ----
  const int lrow = lane >> 4, lslot = lane & 15;
  const int k_chunk = lslot ^ ((wave * 4 + lrow) & 15);
  const int v_chunk = lslot ^ (4 * lrow);
  const unsigned k_rb = lay.k_r * 2, v_rb = lay.v_r * 2;  // row strides in bytes
  const unsigned k_voff = (wave * 4 + lrow) * k_rb + k_chunk * 16;
  const unsigned v_voff = (wave * 4 + lrow) * v_rb + v_chunk * 16;
  typedef const __attribute__((address_space(3))) half8* lds_half8_t;
  unsigned k_frag[8], v_frag[4];  // LDS addresses of the fragment reads, opaque (see fa_fwd_d128_pipe)
  {
    const int kb0 = r32 * 256 + ((h ^ (lane & 15)) * 16);
#pragma unroll
    for (int ks = 0; ks < 8; ks++) {
      k_frag[ks] = (unsigned)(uintptr_t)MI355_LDS(char, lds + (kb0 ^ (ks * 32)));
      asm volatile("" : "+v"(k_frag[ks]));
    }
    const int i16 = lane & 15, g16 = lane >> 4;
    const int v_row = 4 * (g16 >> 1) + (i16 >> 2);
    const int vb0 = VBUF + v_row * 256 + (i16 >> 2) * 64 + (2 * (g16 & 1) + ((i16 & 3) >> 1)) * 16 + (i16 & 1) * 8;
#pragma unroll
    for (int dt = 0; dt < 4; dt++) {
      v_frag[dt] = (unsigned)(uintptr_t)MI355_LDS(char, lds + (vb0 ^ (dt * 64)));
      asm volatile("" : "+v"(v_frag[dt]));
    }
  }

  half8 qf[8];
  // Q rows of pass ps: requested as they lie in memory (rows at or beyond Sq: zeros), later scaled by scale . log2(e),
  // rounded to the 16-bit format again and kept as the B operands of the score MFMAs
  auto request_q = [&](const Pass& ps, half8* raw) {
    const int ql = opaque_lane_id();  // (addresses derived from `lane` would be held in registers through the key walk)
    const int q_row = ps.qb * BLOCK_M + wave * 32 + (ql & 31);
    const half_t* qp = Q + ps.b * lay.q_b + ps.hq * lay.q_h + (size_t)q_row * lay.q_r + (ql >> 5) * 8;
    if (q_row < Sq) {
#pragma unroll
      for (int ks = 0; ks < 8; ks++) raw[ks] = *reinterpret_cast<const half8*>(qp + ks * 16);
    } else {
#pragma unroll
      for (int ks = 0; ks < 8; ks++)
#pragma unroll
        for (int e = 0; e < 8; e++) raw[ks][e] = (half_t)0;
    }
  };
  auto convert_q = [&](const half8* raw) {
#pragma unroll
    for (int ks = 0; ks < 8; ks++)
#pragma unroll
      for (int e = 0; e < 8; e++) qf[ks][e] = cvt16<BF>(to_f32<BF>(raw[ks][e]) * scale_log2e);
  };

  Pass cur = pass_at(0);
  if (cur.ord < 0) return;  // (the launcher starts no more workgroups than units)
  bool tiles_requested = false;  // K 0, K 1, V 0 of `cur` already requested (by the pass before)

  for (;;) {  // passes
  Pass nxt;  // looked up behind trip 0 (its divisions then run beside the other waves' work, not between two passes)
  nxt.ord = -1, nxt.b = nxt.hq = nxt.hk = nxt.qb = 0, nxt.n = 2;
  const int q0 = cur.qb * BLOCK_M;
  const int wq0 = q0 + wave * 32;
  const int q_row = wq0 + r32;
  const int n_tiles = cur.n;
  const half_t* Kb = K + cur.b * lay.k_b + cur.hk * lay.k_h;
  const half_t* Vb = V + cur.b * lay.v_b + cur.hk * lay.v_h;

  auto issue_kv = [&](const half_t* base, unsigned rb, unsigned voff, int tile, int lds_off) {
    char* dst = lds + lds_off + wave * 1024;
    const int row0 = tile * FA_BLOCK_N;
    int rem = Sk - row0;
    rem = rem > FA_BLOCK_N ? FA_BLOCK_N : rem;
    const buffer_rsrc_t rs = make_buffer(reinterpret_cast<const char*>(base) + (size_t)row0 * rb, (unsigned)(rem - 1) * rb + 256u);
#pragma unroll
    for (int i = 0; i < NI; i++) buffer_load_lds_16B(rs, voff + (unsigned)(i * NW * 4) * rb, 0, dst + i * NW * 1024);
  };

  floatx16 oacc[4];
#pragma unroll
  for (int dt = 0; dt < 4; dt++)
#pragma unroll
    for (int r = 0; r < 16; r++) oacc[dt][r] = 0.f;
  floatx16 negm;
#pragma unroll
  for (int r = 0; r < 16; r++) negm[r] = 0.f;
  float l_run = 0.f;
  float grow_thr = -INFINITY;
  constexpr float kRescaleThreshold = 8.f;

  auto wave_active = [&](int tile) { return !CAUSAL || (tile * FA_BLOCK_N <= wq0 + 31 + causal_off); };

  auto scores = [&](int koff, floatx16* s) {
#pragma unroll
    for (int t = 0; t < 2; t++) {
#pragma unroll
      for (int ks = 0; ks < 8; ks++) {
        half8 kf = *(lds_half8_t)(uintptr_t)(k_frag[ks] + (unsigned)(koff + t * 8192));
        s[t] = mfma16<BF>(kf, qf[ks], ks == 0 ? negm : s[t]);
      }
    }
  };

  // softmax of tile `tile` (scores in s) and O^T += V(slot)^T . P^T, with the scores of the following tile computed between
  // the exponentials; LAST: there is no following tile
  auto softmax_pv = [&](int tile, auto voff_tag, auto last_tag, floatx16* s, int koff_next, floatx16* s_next) {
    constexpr int VOFF = decltype(voff_tag)::value;
    constexpr bool LAST = decltype(last_tag)::value;
    {
      const int key0 = tile * FA_BLOCK_N;
      const bool need_mask = (CAUSAL && (key0 + FA_BLOCK_N - 1 > wq0 + causal_off)) || (key0 + FA_BLOCK_N > Sk);
      if (need_mask) {
        const int lim = CAUSAL ? (q_row + causal_off < Sk - 1 ? q_row + causal_off : Sk - 1) : Sk - 1;
        const int rel = lim - key0 - 4 * h;
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
          for (int r = 0; r < 16; r++) {
            const unsigned hide = (unsigned)((rel - (32 * t + 8 * (r >> 2) + (r & 3))) >> 31);
            const float sv = s[t][r];
            s[t][r] = __builtin_bit_cast(float, (hide & 0xFF800000u) | (~hide & __builtin_bit_cast(unsigned, sv)));
          }
      }
    }
    float mx = s[0][0];
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
      for (int r = 0; r < 16; r++) mx = fmaxf(mx, s[t][r]);
    if (__builtin_amdgcn_ballot_w64(mx > grow_thr) != 0) {
      const float mxx = fmaxf(mx, __shfl_xor(mx, 32));
      const bool first = grow_thr == -INFINITY;
      const float delta = first ? (mxx == -INFINITY ? 0.f : mxx) : fmaxf(mxx, 0.f);
      const float alpha = first ? 1.f : __builtin_amdgcn_exp2f(-delta);
      if (mxx != -INFINITY) grow_thr = kRescaleThreshold;
      l_run *= alpha;
#pragma unroll
      for (int dt = 0; dt < 4; dt++)
#pragma unroll
        for (int r = 0; r < 16; r++) oacc[dt][r] *= alpha;
#pragma unroll
      for (int t = 0; t < 2; t++)
#pragma unroll
        for (int r = 0; r < 16; r++) s[t][r] -= delta;
#pragma unroll
      for (int r = 0; r < 16; r++) negm[r] -= delta;
    }
    half8 pf[4];
    float psum = 0.f;
    // Scores of the next tile and the softmax of this one, step by step: score MFMA i, the K fragment of MFMA i + 3
    // requested, and the work of score pair i (two exponentials, one packed conversion, one dot2) behind it.  A
    // scheduling barrier after every step pins the order (a wave issues in order: only vector work placed between two
    // MFMAs runs while the first occupies the matrix pipe).
    __builtin_amdgcn_sched_barrier(0);
    {
      half8 kf[4];
      half2v pp_prev = {(half_t)0, (half_t)0};
      auto kread = [&](int i) { return *(lds_half8_t)(uintptr_t)(k_frag[i & 7] + (unsigned)(koff_next + (i >> 3) * 8192)); };
      if constexpr (!LAST) {
        kf[0] = kread(0);
        kf[1] = kread(1);
        kf[2] = kread(2);
      }
#pragma unroll
      for (int i = 0; i < 16; i++) {
        const int t = i >> 3, ks = i & 7, r = 2 * ks;
        if constexpr (!LAST) {
          if (i + 3 < 16) kf[(i + 3) & 3] = kread(i + 3);
          s_next[t] = mfma16<BF>(kf[i & 3], qf[ks], ks == 0 ? negm : s_next[t]);
        }
        // (the empty statement ties the pair's arithmetic to this step: without side effects of its own it is placed
        // wherever instruction selection likes, scheduling barriers or not)
        float e0 = __builtin_amdgcn_exp2f(s[t][r]), e1 = __builtin_amdgcn_exp2f(s[t][r + 1]);
        if (i > 0) psum = dot2_ones<BF>(pp_prev, psum);  // (one step behind its conversion, as in fa_fwd_d128_pipe)
        half2v pp = cvt16x2<BF>(e0, e1);
        asm volatile("" : "+v"(pp), "+v"(psum));
        pf[t * 2 + (r >> 3)][r & 7] = pp[0];
        pf[t * 2 + (r >> 3)][(r & 7) + 1] = pp[1];
        pp_prev = pp;
        __builtin_amdgcn_sched_barrier(0);
      }
      psum = dot2_ones<BF>(pp_prev, psum);
    }
    l_run += psum;
    half4 vlo[3], vhi[3];  // V^T reads and their waits in assembly, as in fa_fwd_d128_pipe
    auto vr = [&](auto itag) {
      constexpr int i = decltype(itag)::value;
      constexpr int off = VOFF + (i >> 2) * 4096;
      half4 &lo = vlo[i % 3], &hi = vhi[i % 3];
      const unsigned addr = v_frag[i & 3];
      asm volatile("ds_read_b64_tr_b16 %0, %2 offset:%3\n\tds_read_b64_tr_b16 %1, %2 offset:%4"
                   : "=&v"(lo), "=&v"(hi)
                   : "v"(addr), "n"(off), "n"(off + 2048));
    };
    vr(std::integral_constant<int, 0>{});
    vr(std::integral_constant<int, 1>{});
    static_for<0, 16>([&](auto itag) {
      constexpr int i = decltype(itag)::value;
      if constexpr (i + 2 < 16) vr(std::integral_constant<int, i + 2>{});
      half4 &lo = vlo[i % 3], &hi = vhi[i % 3];
      if constexpr (i + 2 < 16)
        asm volatile("s_waitcnt lgkmcnt(4)" : "+v"(lo), "+v"(hi));
      else if constexpr (i + 1 < 16)
        asm volatile("s_waitcnt lgkmcnt(2)" : "+v"(lo), "+v"(hi));
      else
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(lo), "+v"(hi));
      const half8 vf = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      oacc[i & 3] = mfma16<BF>(vf, pf[i >> 2], oacc[i & 3]);
      __builtin_amdgcn_sched_barrier(0);
    });
  };

  floatx16 sa[2], sb[2];
  if (!tiles_requested) {
    half8 raw[8];
    request_q(cur, raw);
    issue_kv(Kb, k_rb, k_voff, 0, 0);
    issue_kv(Vb, v_rb, v_voff, 0, VBUF);
    issue_kv(Kb, k_rb, k_voff, 1, TILE_B);
    convert_q(raw);
    wait_vmcnt0();
    __syncthreads();
  }
  scores(0, sa);  // every wave sees keys in a pass's first tile
  // trip 0 overwrites the K(0) slot with K(2): every wave must have read its K(0) fragments first
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __syncthreads();

  // trip j (PAR = j & 1): loads for K(j+2) and V(j+1); scores of tile j+1; softmax + PV of tile j
  auto trip = [&](auto par_tag, int j, floatx16* s_cur, floatx16* s_next) {
    constexpr int PAR = decltype(par_tag)::value;
    constexpr int K_CUR = PAR * TILE_B, K_NEXT = (1 - PAR) * TILE_B, V_CUR = PAR * TILE_B, V_NEXT = VBUF + (1 - PAR) * TILE_B;
    if (j + 2 < n_tiles) issue_kv(Kb, k_rb, k_voff, j + 2, K_CUR);
    if (j + 1 < n_tiles) issue_kv(Vb, v_rb, v_voff, j + 1, V_NEXT);
    if (wave_active(j)) softmax_pv(j, std::integral_constant<int, V_CUR>{}, std::false_type{}, s_cur, K_NEXT, s_next);  // idle from here on otherwise
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __syncthreads();
  };
  // A pass of an even tile count runs its last tile (an odd trip) apart, behind the requests for the next pass: there are
  // no loads and no scores left for this pass, neither K slot is read again and V slot 0 was last read by the trip before.
  // A pass of an odd count ends with an ordinary trip and the requests follow it.
  const int n_plain = (n_tiles & 1) ? n_tiles : n_tiles - 1;
  for (int j = 0; j < n_plain; j += 2) {
    trip(std::integral_constant<int, 0>{}, j, sa, sb);
    if (j == 0) nxt = pass_at(cur.ord + 1);  // (two tiles at least: trip 0 is never the last)
    if (j + 1 < n_plain) trip(std::integral_constant<int, 1>{}, j + 1, sb, sa);
  }

  // ---- between passes ----
  half8 qraw[8];
  request_q(nxt.ord >= 0 ? nxt : cur, qraw);  // (unconditional, and converted unconditionally below: the old Q fragments are dead from here on)
  if (nxt.ord >= 0) {
    const half_t* Kn = K + nxt.b * lay.k_b + nxt.hk * lay.k_h;
    const half_t* Vn = V + nxt.b * lay.v_b + nxt.hk * lay.v_h;
    issue_kv(Kn, k_rb, k_voff, 0, 0);
    issue_kv(Vn, v_rb, v_voff, 0, VBUF);
    issue_kv(Kn, k_rb, k_voff, 1, TILE_B);
  }
  if (n_plain < n_tiles) {
    if (wave_active(n_tiles - 1)) softmax_pv(n_tiles - 1, std::integral_constant<int, TILE_B>{}, std::true_type{}, sb, 0, sa);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  }
  const float l_tot = l_run + __shfl_xor(l_run, 32);
  const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
  half8 orow[32 / 4];  // the rows this lane stores: 16-byte chunk ec of rows er, er + 4, ...
  const int el = opaque_lane_id();
  const int er = el >> 4, ec = el & 15;
  {
    // Output through the wave's staging region, STG_ROWS rows per round (chunk c of row r in slot c ^ (r & 15)): a lane
    // holds 4-value pieces of one row; whole 16-byte chunks are read back, to be stored as full rows
    char* ep = lds + STG + wave * (STG_ROWS * 256);
    const int e32 = el & 31, eh = el >> 5;
#pragma unroll
    for (int round = 0; round < 32 / STG_ROWS; round++) {
      if (STG_ROWS == 32 || (e32 / STG_ROWS) == round) {
#pragma unroll
        for (int dt = 0; dt < 4; dt++)
#pragma unroll
          for (int q = 0; q < 4; q++) {
            const half4 v = {cvt16<BF>(oacc[dt][4 * q] * inv), cvt16<BF>(oacc[dt][4 * q + 1] * inv), cvt16<BF>(oacc[dt][4 * q + 2] * inv),
                             cvt16<BF>(oacc[dt][4 * q + 3] * inv)};
            *reinterpret_cast<half4*>(ep + (e32 % STG_ROWS) * 256 + (((dt * 4 + q) ^ (e32 & 15)) * 16) + 8 * eh) = v;
          }
      }
#pragma unroll
      for (int it = 0; it < STG_ROWS / 4; it++) {
        const int lr = it * 4 + er, row = round * STG_ROWS + lr;
        orow[round * (STG_ROWS / 4) + it] = *reinterpret_cast<const half8*>(ep + lr * 256 + ((ec ^ (row & 15)) * 16));
      }
    }
  }
  convert_q(qraw);  // (the oldest of the requests)
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");  // the next pass's first tiles
  __syncthreads();
  {
    // the stores are left in flight: they drain under the next pass's first trip, whose closing wait covers them
    half_t* Ob = O + cur.b * lay.o_b + cur.hq * lay.o_h;
#pragma unroll
    for (int it = 0; it < 8; it++) {
      const int row = it * 4 + er;
      if (wq0 + row < Sq) *reinterpret_cast<half8*>(Ob + (size_t)(wq0 + row) * lay.o_r + ec * 8) = orow[it];
    }
  }
  if (nxt.ord < 0) break;
  tiles_requested = true;
  cur = nxt;
  }  // passes
}

static const char* kFaVariants[] = {"d128_bm128_bn64_w4_pipelined", "d128_bm128_bn64_w4", "d128_bm256_bn64_w8_pipelined",
                                    "d128_bm256_bn64_w8_walk", "d128_bm128_bn64_w4_walk", "d128_bm128_bn64_w4_m16",
                                    "d128_bm256_bn64_w8_m16"};
int fa_variant_count() { return 7; }
const char* fa_variant_name(int i) { return (i >= 0 && i < 7) ? kFaVariants[i] : nullptr; }

}  // namespace mi355

using namespace mi355;

// number of CUs of the current device (cached per device)
static int fa_cu_count() {
  static std::atomic<int> cached[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  int n = cached[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cached[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

template <bool BF>
static int fa_launch(const void* q, const void* k, const void* v, void* o, int64_t B, int64_t H, int64_t Hkv, int64_t Sq,
                     int64_t Sk, int64_t D, const FaLayout& lay, float scale, int is_causal, int variant, void* stream,
                     const char* who) {
  if (!q || !k || !v || !o) return fail(-MI355_E_NULL, "%s: null pointer", who);
  if (D != 128) return fail(-MI355_E_SHAPE, "%s: head dim %lld not supported (only 128)", who, (long long)D);
  if (B <= 0 || H <= 0 || Sq <= 0 || Sk <= 0 || B * H > (1 << 24) || Sq > (1 << 24) || Sk > (1 << 24))
    return fail(-MI355_E_SHAPE, "%s: bad shape B=%lld H=%lld Sq=%lld Sk=%lld", who, (long long)B, (long long)H, (long long)Sq,
                (long long)Sk);
  if (Hkv <= 0 || H % Hkv != 0)
    return fail(-MI355_E_SHAPE, "%s: %lld query heads over %lld key/value heads", who, (long long)H, (long long)Hkv);
  if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(o))
    return fail(-MI355_E_ALIGN, "%s: q, k, v, o must be 16-byte aligned", who);
  if (variant > 6) return fail(-MI355_E_DTYPE, "%s: variant %d out of range", who, variant);
  if (!(scale > 0.f) || !isfinite(scale)) return fail(-MI355_E_SHAPE, "%s: scale must be positive and finite", who);
  const int BH = (int)(B * H);
  const int q_blocks = (int)((Sq + FA_BLOCK_M - 1) / FA_BLOCK_M);
  const int lds_bytes = 2 * FA_STAGE;
  static std::atomic<uint64_t> lds_ok[4] = {};
  const void* kernels[4] = {reinterpret_cast<const void*>(fa_fwd_d128<true, BF>), reinterpret_cast<const void*>(fa_fwd_d128<false, BF>),
                            reinterpret_cast<const void*>(fa_fwd_d128_pipe<true, BF>),
                            reinterpret_cast<const void*>(fa_fwd_d128_pipe<false, BF>)};
  for (int i = 0; i < 4; i++)
    if (int rc = allow_lds(kernels[i], lds_bytes, lds_ok[i], "fa_fwd_d128")) return rc;
  const float scale_log2e = scale * 1.4426950408889634f;
  // Without a mask, and with enough 256-query blocks for every CU, the 8-wave form is ahead (2 x 32 x 4096: 503 against
  // 514 us); with the causal mask the two are level and the 4-wave form has the finer-grained tail.
  // The automatic choice is the 16x16x32 form: eight waves (with the exponentials spread into the output MFMAs) for
  // unmasked shapes with enough 256-query blocks for every CU (2 x 32 x 4096: 475 us against 483 for the 32x32x16 form
  // on the same box), four waves otherwise (causal 2 x 32 x 4096: 263 against 269; the finer-grained tail).
  if (variant < 0) variant = (!is_causal && (int64_t)BH * ((Sq + 255) / 256) >= 512) ? 6 : 5;
  if (variant == 5 || variant == 6) {
    // the pipelined forms on 16x16x32 MFMAs, 4 waves (128-query blocks) or 8 (256)
    const bool w8 = variant == 6;
    const int bm = w8 ? 256 : 128;
    const int qbm = (int)((Sq + bm - 1) / bm);
    const void* kern = w8 ? (is_causal ? (const void*)fa_fwd_d128_m16<true, BF, 8, true> : (const void*)fa_fwd_d128_m16<false, BF, 8, true>)
                          : (is_causal ? (const void*)fa_fwd_d128_m16<true, BF, 4, false> : (const void*)fa_fwd_d128_m16<false, BF, 4, false>);
    static std::atomic<uint64_t> okm[4] = {};
    if (int rc = allow_lds(kern, lds_bytes, okm[(w8 ? 2 : 0) + (is_causal ? 1 : 0)], "fa_fwd_d128_m16")) return rc;
    dim3 grid(BH * (is_causal ? (qbm + 1) / 2 : qbm)), block(w8 ? 512 : 256);
    const half_t *qp = (const half_t*)q, *kp = (const half_t*)k, *vp = (const half_t*)v;
    half_t* op = (half_t*)o;
    int bh_i = BH, sq_i = (int)Sq, sk_i = (int)Sk, qb_i = qbm;
    FaLayout lay_v = lay;
    float sc = scale_log2e;
    FaPaged no_pages{nullptr, nullptr, 0, 0, 0};
    void* args[] = {&qp, &kp, &vp, &op, &bh_i, &sq_i, &sk_i, &sc, &qb_i, &lay_v, &no_pages};
    hipError_t e = hipLaunchKernel(kern, grid, block, args, lds_bytes, reinterpret_cast<hipStream_t>(stream));
    if (e != hipSuccess) return fail((int)e, "%s: launch of fa_fwd_d128_m16 failed: %s", who, hipGetErrorString(e));
    return check_launch("fa_fwd_d128_m16", grid, block, lds_bytes);
  }
  if (variant == 3 || variant == 4) {
    // the persistent forms: every pass needs two key tiles, and the masked form a square mask (no pass without keys)
    const bool w8 = variant == 3;
    const int bm = w8 ? 256 : 128;
    const int qbw = (int)((Sq + bm - 1) / bm);
    const int64_t units_w = (int64_t)BH * (is_causal ? (qbw + 1) / 2 : qbw);
    if (Sk < 128 || (is_causal && Sq != Sk) || units_w >= (1ll << 30))
      return fail(-MI355_E_SHAPE, "%s: the persistent form needs Sk >= 128%s (Sq=%lld Sk=%lld)", who, is_causal ? " and Sq == Sk" : "",
                  (long long)Sq, (long long)Sk);
    const void* kern = w8 ? (is_causal ? (const void*)fa_fwd_d128_walk<true, BF, 8> : (const void*)fa_fwd_d128_walk<false, BF, 8>)
                          : (is_causal ? (const void*)fa_fwd_d128_walk<true, BF, 4> : (const void*)fa_fwd_d128_walk<false, BF, 4>);
    static std::atomic<uint64_t> okw[4] = {};
    const int ldsw = 4 * FA_BLOCK_N * 256 + (w8 ? 8 * 8192 : 4 * 2048);  // K and V rings + output staging
    if (int rc = allow_lds(kern, ldsw, okw[(w8 ? 2 : 0) + (is_causal ? 1 : 0)], "fa_fwd_d128_walk")) return rc;
    int g = fa_cu_count() * (w8 ? 1 : 2);  // workgroups resident at once
    if (((BH / lay.group) & 7) == 0) g &= ~7;  // units of one K/V head stay on the XCD that a workgroup runs on
    if (g < 1) g = 1;
    if (units_w < g) g = (int)units_w;
    dim3 grid(g), block(w8 ? 512 : 256);
    const half_t *qp = (const half_t*)q, *kp = (const half_t*)k, *vp = (const half_t*)v;
    half_t* op = (half_t*)o;
    int bh_i = BH, sq_i = (int)Sq, sk_i = (int)Sk;
    FaLayout lay_v = lay;
    float sc = scale_log2e;
    int qb_i = qbw;
    void* args[] = {&qp, &kp, &vp, &op, &bh_i, &sq_i, &sk_i, &sc, &qb_i, &lay_v};
    hipError_t e = hipLaunchKernel(kern, grid, block, args, ldsw, reinterpret_cast<hipStream_t>(stream));
    if (e != hipSuccess) return fail((int)e, "%s: launch of fa_fwd_d128_walk failed: %s", who, hipGetErrorString(e));
    return check_launch("fa_fwd_d128_walk", grid, block, ldsw);
  }
  if (variant == 2) {
    // eight waves: 256-query blocks, one workgroup per CU
    auto kern = is_causal ? fa_fwd_d128_pipe<true, BF, 8> : fa_fwd_d128_pipe<false, BF, 8>;
    static std::atomic<uint64_t> ok8[2] = {};
    const int lds8 = lds_bytes;
    if (int rc = allow_lds(reinterpret_cast<const void*>(kern), lds8, ok8[is_causal ? 1 : 0], "fa_fwd_d128_pipe<8>")) return rc;
    const int qb8 = (int)((Sq + 255) / 256);
    dim3 grid(BH * (is_causal ? (qb8 + 1) / 2 : qb8)), block(512);
    hipLaunchKernelGGL(kern, grid, block, lds8, reinterpret_cast<hipStream_t>(stream), (const half_t*)q, (const half_t*)k,
                       (const half_t*)v, (half_t*)o, BH, (int)Sq, (int)Sk, scale_log2e, qb8, lay);
    return check_launch("fa_fwd_d128_pipe<8 waves>", grid, block, lds8);
  }
  // the pipelined causal kernel takes a pair of query blocks per workgroup
  const int units = (variant != 1 && is_causal) ? (q_blocks + 1) / 2 : q_blocks;
  dim3 grid(BH * units), block(256);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (variant == 1) {
    auto kern = is_causal ? fa_fwd_d128<true, BF> : fa_fwd_d128<false, BF>;
    hipLaunchKernelGGL(kern, grid, block, lds_bytes, s, (const half_t*)q, (const half_t*)k, (const half_t*)v, (half_t*)o, BH,
                       (int)Sq, (int)Sk, scale_log2e, q_blocks, lay);
  } else {
    auto kern = is_causal ? fa_fwd_d128_pipe<true, BF> : fa_fwd_d128_pipe<false, BF>;
    hipLaunchKernelGGL(kern, grid, block, lds_bytes, s, (const half_t*)q, (const half_t*)k, (const half_t*)v, (half_t*)o, BH,
                       (int)Sq, (int)Sk, scale_log2e, q_blocks, lay);
  }
  return check_launch(variant == 1 ? "fa_fwd_d128" : "fa_fwd_d128_pipe", grid, block, lds_bytes);
}

template <bool BF>
static int fa_contiguous(const void* q, const void* k, const void* v, void* o, int64_t B, int64_t H, int64_t Sq, int64_t Sk,
                         int64_t D, float scale, int is_causal, int variant, void* stream) {
  FaLayout lay;
  lay.q_b = H * Sq * 128, lay.q_h = Sq * 128, lay.q_r = 128;
  lay.o_b = lay.q_b, lay.o_h = lay.q_h, lay.o_r = 128;
  lay.k_b = lay.v_b = H * Sk * 128, lay.k_h = lay.v_h = Sk * 128, lay.k_r = lay.v_r = 128;
  lay.H = (int)H, lay.group = 1;
  return fa_launch<BF>(q, k, v, o, B, H, H, Sq, Sk, D, lay, scale, is_causal, variant, stream,
                       BF ? "flash_attn_fwd_bf16" : "flash_attn_fwd");
}

extern "C" int mi355_flash_attn_fwd(const void* q, const void* k, const void* v, void* o, int64_t B, int64_t H, int64_t Sq,
                                    int64_t Sk, int64_t D, float scale, int is_causal, int variant, void* stream) {
  return fa_contiguous<false>(q, k, v, o, B, H, Sq, Sk, D, scale, is_causal, variant, stream);
}

extern "C" int mi355_flash_attn_fwd_bf16(const void* q, const void* k, const void* v, void* o, int64_t B, int64_t H, int64_t Sq,
                                         int64_t Sk, int64_t D, float scale, int is_causal, int variant, void* stream) {
  return fa_contiguous<true>(q, k, v, o, B, H, Sq, Sk, D, scale, is_causal, variant, stream);
}

template <bool BF>
static int fa_strided(const void* q, const void* k, const void* v, void* o, int64_t B, int64_t H, int64_t Hkv, int64_t Sq,
                      int64_t Sk, int64_t D, const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                      const int64_t* o_strides, float scale, int is_causal, int variant, void* stream) {
  const char* who = BF ? "flash_attn_fwd_strided_bf16" : "flash_attn_fwd_strided";
  if (!q_strides || !k_strides || !v_strides || !o_strides) return fail(-MI355_E_NULL, "%s: null stride array", who);
  const int64_t* all[4] = {q_strides, k_strides, v_strides, o_strides};
  for (const int64_t* st : all) {
    for (int i = 0; i < 3; i++)
      if (st[i] < 0 || (st[i] & 7)) return fail(-MI355_E_ALIGN, "%s: strides must be non-negative multiples of 8 elements", who);
    if (st[2] < 128 || st[2] >= (1ll << 24))
      return fail(-MI355_E_SHAPE, "%s: row stride %lld outside [128, 2^24)", who, (long long)st[2]);
  }
  if ((B > 1 && o_strides[0] == 0) || (H > 1 && o_strides[1] == 0)) return fail(-MI355_E_SHAPE, "%s: output batch / head strides must not be 0", who);
  FaLayout lay;
  lay.q_b = q_strides[0], lay.q_h = q_strides[1], lay.q_r = (unsigned)q_strides[2];
  lay.k_b = k_strides[0], lay.k_h = k_strides[1], lay.k_r = (unsigned)k_strides[2];
  lay.v_b = v_strides[0], lay.v_h = v_strides[1], lay.v_r = (unsigned)v_strides[2];
  lay.o_b = o_strides[0], lay.o_h = o_strides[1], lay.o_r = (unsigned)o_strides[2];
  lay.H = (int)H, lay.group = Hkv > 0 ? (int)(H / Hkv) : 1;
  return fa_launch<BF>(q, k, v, o, B, H, Hkv, Sq, Sk, D, lay, scale, is_causal, variant, stream, who);
}

extern "C" int mi355_flash_attn_fwd_strided(const void* q, const void* k, const void* v, void* o, int64_t B, int64_t H,
                                            int64_t Hkv, int64_t Sq, int64_t Sk, int64_t D, const int64_t* q_strides,
                                            const int64_t* k_strides, const int64_t* v_strides, const int64_t* o_strides,
                                            float scale, int is_causal, int variant, void* stream) {
  return fa_strided<false>(q, k, v, o, B, H, Hkv, Sq, Sk, D, q_strides, k_strides, v_strides, o_strides, scale, is_causal, variant,
                           stream);
}

extern "C" int mi355_flash_attn_fwd_strided_bf16(const void* q, const void* k, const void* v, void* o, int64_t B, int64_t H,
                                                 int64_t Hkv, int64_t Sq, int64_t Sk, int64_t D, const int64_t* q_strides,
                                                 const int64_t* k_strides, const int64_t* v_strides, const int64_t* o_strides,
                                                 float scale, int is_causal, int variant, void* stream) {
  return fa_strided<true>(q, k, v, o, B, H, Hkv, Sq, Sk, D, q_strides, k_strides, v_strides, o_strides, scale, is_causal, variant,
                          stream);
}

template <bool BF>
static int fa_paged_prefill(const void* q, const void* k_cache, const void* v_cache, const void* block_table, const void* seq_lens,
                            void* out, int64_t num_seqs, int64_t num_new, int64_t num_q_heads, int64_t num_kv_heads, int64_t D,
                            int64_t page_size, int64_t max_pages_per_seq, int64_t num_pages, float scale, void* stream) {
  const char* who = BF ? "paged_prefill_attn_bf16" : "paged_prefill_attn";
  if (!q || !k_cache || !v_cache || !block_table || !seq_lens || !out) return fail(-MI355_E_NULL, "%s: null pointer", who);
  if (D != 128) return fail(-MI355_E_SHAPE, "%s: head dim %lld not supported (only 128)", who, (long long)D);
  int page_shift = -1;
  for (int sh = 0; sh <= 4; sh++)
    if (page_size == (16ll << sh)) page_shift = sh;
  if (page_shift < 0) return fail(-MI355_E_SHAPE, "%s: page size %lld not supported (16, 32, 64, 128 or 256)", who, (long long)page_size);
  if (num_seqs <= 0 || num_new <= 0 || num_q_heads <= 0 || num_kv_heads <= 0 || max_pages_per_seq <= 0 || num_pages <= 0 ||
      num_seqs * num_q_heads > (1 << 24) || num_new > (1 << 20) || max_pages_per_seq > (1 << 20) || num_pages > (1 << 24) ||
      (max_pages_per_seq * page_size) > (1 << 24))
    return fail(-MI355_E_SHAPE, "%s: bad shape seqs=%lld new=%lld q_heads=%lld kv_heads=%lld max_pages=%lld pages=%lld", who,
                (long long)num_seqs, (long long)num_new, (long long)num_q_heads, (long long)num_kv_heads,
                (long long)max_pages_per_seq, (long long)num_pages);
  if (num_q_heads % num_kv_heads != 0)
    return fail(-MI355_E_SHAPE, "%s: %lld query heads over %lld key/value heads", who, (long long)num_q_heads, (long long)num_kv_heads);
  if (num_kv_heads * 128 >= (1 << 24)) return fail(-MI355_E_SHAPE, "%s: too many key/value heads", who);
  if (!aligned16(q) || !aligned16(k_cache) || !aligned16(v_cache) || !aligned16(out))
    return fail(-MI355_E_ALIGN, "%s: q, k_cache, v_cache, out must be 16-byte aligned", who);
  if (!(scale > 0.f) || !isfinite(scale)) return fail(-MI355_E_SHAPE, "%s: scale must be positive and finite", who);
  FaLayout lay;
  lay.q_b = num_new * num_q_heads * 128, lay.q_h = 128, lay.q_r = (unsigned)(num_q_heads * 128);
  lay.o_b = lay.q_b, lay.o_h = 128, lay.o_r = lay.q_r;
  lay.k_b = lay.v_b = 0, lay.k_h = lay.v_h = 128, lay.k_r = lay.v_r = (unsigned)(num_kv_heads * 128);
  lay.H = (int)num_q_heads, lay.group = (int)(num_q_heads / num_kv_heads);
  const int BH = (int)(num_seqs * num_q_heads);
  const int q_blocks = (int)((num_new + FA_BLOCK_M - 1) / FA_BLOCK_M);
  const int lds_bytes = 2 * FA_STAGE;
  auto kern = fa_fwd_d128_m16<true, BF, 4, false, true>;
  static std::atomic<uint64_t> lds_ok{0};
  if (int rc = allow_lds(reinterpret_cast<const void*>(kern), lds_bytes, lds_ok, "fa_fwd_d128_m16<paged>")) return rc;
  dim3 grid(BH * ((q_blocks + 1) / 2)), block(256);
  const FaPaged pg{static_cast<const int*>(block_table), static_cast<const int*>(seq_lens), (int)max_pages_per_seq, (int)num_pages,
                   page_shift};
  hipLaunchKernelGGL(kern, grid, block, lds_bytes, reinterpret_cast<hipStream_t>(stream), (const half_t*)q, (const half_t*)k_cache,
                     (const half_t*)v_cache, (half_t*)out, BH, (int)num_new, 0, scale * 1.4426950408889634f, q_blocks, lay, pg);
  return check_launch("fa_fwd_d128_m16<paged>", grid, block, lds_bytes);
}

extern "C" int mi355_paged_prefill_attn(const void* q, const void* k_cache, const void* v_cache, const void* block_table,
                                        const void* seq_lens, void* out, int64_t num_seqs, int64_t num_new, int64_t num_q_heads,
                                        int64_t num_kv_heads, int64_t D, int64_t page_size, int64_t max_pages_per_seq,
                                        int64_t num_pages, float scale, void* stream) {
  return fa_paged_prefill<false>(q, k_cache, v_cache, block_table, seq_lens, out, num_seqs, num_new, num_q_heads, num_kv_heads, D,
                                 page_size, max_pages_per_seq, num_pages, scale, stream);
}

extern "C" int mi355_paged_prefill_attn_bf16(const void* q, const void* k_cache, const void* v_cache, const void* block_table,
                                             const void* seq_lens, void* out, int64_t num_seqs, int64_t num_new,
                                             int64_t num_q_heads, int64_t num_kv_heads, int64_t D, int64_t page_size,
                                             int64_t max_pages_per_seq, int64_t num_pages, float scale, void* stream) {
  return fa_paged_prefill<true>(q, k_cache, v_cache, block_table, seq_lens, out, num_seqs, num_new, num_q_heads, num_kv_heads, D,
                                page_size, max_pages_per_seq, num_pages, scale, stream);
}
