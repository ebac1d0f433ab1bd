// Paged GQA decode attention for gfx950 (one query token per sequence, head dim 128,
// 16-token pages, fp16 KV cache laid out [page][token][kv_head][128]).
//
// The op is HBM bound: every K and V byte is read exactly once, so the kernel is organised
// around keeping many page reads in flight and doing the arithmetic on the side.
//
// Phase 0: one workgroup (4 waves) per (sequence, kv head, kv split).  The waves take the
// split's pages round-robin, two pages (32 tokens) per step, and never synchronise with each
// other until the end: every wave owns a private LDS ring.
//   - K pages go global -> registers, already in MFMA A-operand layout (lane = token, 16-byte
//     chunks of the head row), and S^T[token][q head] = K . Q^T is one v_mfma_f32_16x16x32_f16
//     chain per page with all q heads of the group in the MFMA N dimension.
//   - V pages go global -> LDS by direct-to-LDS loads (fully coalesced 256-byte rows), and
//     O^T[d][q head] += V^T . P^T fetches V^T with LDS transpose reads.  The token order inside
//     that contraction is the order S^T leaves the scores in registers.
//   - The next step's K and V are requested before the current step is computed; the wait is
//     on the loads of the current step only (vmcnt counts loads in order).
//   The four waves' (max, sum, acc) are merged through LDS and written as one fp32 partial per
//   (seq, q head, split) -- or, with a single split, normalised and written as fp16 directly.
// Phase 1: merges the splits of every (seq, q head).
#include "common.hpp"
#include <math.h>

namespace mi355 {

constexpr int PD_WAVES = 4;
constexpr int PD_WAVE_LDS = 2 * 8192;  // two stages of two 4 KiB V pages

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Merge of the kv splits of one (sequence, q head) for output element d: the one statement of this arithmetic,
// used by the merge kernel and by the last-arriving workgroup of the one-launch form, so that both give the same
// bits.  COHERENT: read with device-scope loads (partials written by other workgroups of the running kernel,
// possibly through another XCD's L2).
template <bool COHERENT>
__device__ __forceinline__ float pd_load(const float* p) {
  if constexpr (COHERENT) return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  else return *p;
}
template <bool COHERENT>
__device__ __forceinline__ float merge_splits(const float* part_acc, const float* part_ml, size_t row, int d, int num_splits) {
  const float* ml = part_ml + row * num_splits * 2;
  float m_tot = -INFINITY;
  for (int s = 0; s < num_splits; s++) m_tot = fmaxf(m_tot, pd_load<COHERENT>(ml + 2 * s));
  float acc = 0.f, l = 0.f;
  if (m_tot > -INFINITY) {
    for (int s = 0; s < num_splits; s++) {
      const float ms = pd_load<COHERENT>(ml + 2 * s);
      if (ms > -INFINITY) {
        const float w = fast_exp2(ms - m_tot);
        acc = __builtin_fmaf(w, pd_load<COHERENT>(part_acc + (row * num_splits + s) * 128 + d), acc);
        l = __builtin_fmaf(w, pd_load<COHERENT>(ml + 2 * s + 1), l);
      }
    }
  }
  float r = acc * (l > 0.f ? 1.f / l : 0.f);
  // keep the product a rounded fp32 value in both users: left alone, the compiler fuses it with a following
  // conversion to fp16 into one mixed-precision instruction with a single rounding where it can, and not elsewhere
  asm volatile("" : "+v"(r));
  return r;
}

// Exclusive prefix sum of one int per thread over the 256 threads of the workgroup (wave scans by shuffles, the
// four wave totals through `tmp`, 4 ints of LDS); every thread also gets the grand total.
__device__ __forceinline__ int block_exclusive_scan(int v, int* tmp, int& total) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int incl = v;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int n = __shfl_up(incl, d);
    if (lane >= d) incl += n;
  }
  if (lane == 63) tmp[wave] = incl;
  __syncthreads();
  int base = 0;
  total = 0;
#pragma unroll
  for (int w = 0; w < PD_WAVES; w++) {
    const int tw = tmp[w];
    base += w < wave ? tw : 0;
    total += tw;
  }
  __syncthreads();
  return base + incl - v;
}

template <int G, bool BF>  // G = q heads per kv head (<= 16); BF = bf16 instead of fp16 operands and output
__global__ __launch_bounds__(PD_WAVES * 64) void paged_decode_phase0(
    const half_t* __restrict__ Q, const half_t* __restrict__ Kc, const half_t* __restrict__ Vc,
    const int* __restrict__ block_table, const int* __restrict__ seq_lens, float* __restrict__ part_acc,
    float* __restrict__ part_ml, half_t* __restrict__ out, half_t* __restrict__ final_out, int num_kv_heads, int max_pages_per_seq, int num_splits,
    float scale_log2e, int window, int page_shift, int num_pages, int* __restrict__ arrivals, unsigned epoch) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int split = blockIdx.x, kvh = blockIdx.y;
  // Workgroups are dispatched in grid order and a ragged batch ends with whatever is dispatched last: walking
  // the sequences longest first leaves the short ones for the tail.  Each workgroup finds "the sequence with
  // rank blockIdx.z" itself -- thread t counts the sequences that come before sequence t -- which costs a
  // few hundred cached loads for the batch sizes where the tail matters; larger batches keep their order.
  int seq = blockIdx.z;
  const int num_seqs = (int)gridDim.z;
  if (num_seqs > 1 && num_seqs <= PD_WAVES * 64) {
    int* pick = reinterpret_cast<int*>(lds);
    const int t = threadIdx.x;
    if (t < num_seqs) {
      const int mine = seq_lens[t];
      int rank = 0;
      for (int j = 0; j < num_seqs; j++) {
        const int other = seq_lens[j];
        rank += (other > mine) || (other == mine && j < t);
      }
      if (rank == (int)blockIdx.z) *pick = t;
    }
    __syncthreads();
    seq = *pick;
    __syncthreads();  // the slot is part of the V ring
  } else if (num_seqs > PD_WAVES * 64 && num_seqs <= 16384) {
    // Larger batches: an exact rank would cost num_seqs^2 / 256 loads per thread.  Sequences are instead put into 256
    // buckets by length (longest first) with a counting pass, the workgroup finds the bucket that holds rank
    // blockIdx.z, and takes the sequence at that offset inside the bucket in thread-major order -- a bijection from
    // ranks to sequences that is ordered by length down to 1/256 of the longest possible length, for a few loads
    // per thread and two block scans.
    int* hist = reinterpret_cast<int*>(lds);  // [256] sequences per bucket
    int* tmp = hist + 256;                    // [4] scan scratch
    int* res = tmp + 4;                       // bucket, offset inside it, chosen sequence
    const int t = threadIdx.x;
    const int reach = (max_pages_per_seq << page_shift) * 16;
    auto bucket_of = [&](int len) {
      len = len < 0 ? 0 : (len > reach ? reach : len);
      return 255 - (int)(((long long)len * 255) / (reach > 0 ? reach : 1));
    };
    hist[t] = 0;
    __syncthreads();
    for (int j = t; j < num_seqs; j += PD_WAVES * 64) atomicAdd(&hist[bucket_of(seq_lens[j])], 1);
    __syncthreads();
    int total;
    const int mine = hist[t];
    const int first = block_exclusive_scan(mine, tmp, total);
    const int z = (int)blockIdx.z;
    if (first <= z && z < first + mine) {
      res[0] = t;
      res[1] = z - first;
    }
    __syncthreads();
    const int bkt = res[0], off = res[1];
    int hits = 0;
    for (int j = t; j < num_seqs; j += PD_WAVES * 64) hits += bucket_of(seq_lens[j]) == bkt;
    const int before = block_exclusive_scan(hits, tmp, total);
    if (before <= off && off < before + hits) {
      int k = off - before;
      for (int j = t; j < num_seqs; j += PD_WAVES * 64)
        if (bucket_of(seq_lens[j]) == bkt && k-- == 0) res[2] = j;
    }
    __syncthreads();
    seq = res[2];
    __syncthreads();  // the area is part of the V ring
  }
  const int num_q_heads = num_kv_heads * G;
  // a length beyond what the block table can address is cut to the table's reach
  const int max_tokens = (max_pages_per_seq << page_shift) * 16;
  const int L_in = seq_lens[seq];
  const int L = L_in < 0 ? 0 : (L_in > max_tokens ? max_tokens : L_in);
  // sliding window: only the last `window` tokens take part (window <= 0: all of them); pages wholly in
  // front of the window are never touched and the splits divide the pages that remain
  const int lo = (window > 0 && L > window) ? L - window : 0;
  const int p_lo = lo >> 4;
  const int p_hi = (L + 15) >> 4;
  const int pps = (p_hi - p_lo + num_splits - 1) / num_splits;
  const int p_begin = p_lo + split * pps;
  const int p_end = (p_begin + pps < p_hi) ? p_begin + pps : p_hi;
  const int n_steps = p_end > p_begin ? (p_end - p_begin + 1) >> 1 : 0;
  const int* bt = block_table + (size_t)seq * max_pages_per_seq;

  const int i16 = lane & 15, g = lane >> 4;
  // Q^T fragments (MFMA B operand): lane (head i16, chunk g) holds d = 32*ks + 8*g .. +7
  half8 qf[4];
#pragma unroll
  for (int ks = 0; ks < 4; ks++) {
    if (i16 < G) {
      qf[ks] = *reinterpret_cast<const half8*>(Q + ((size_t)seq * num_q_heads + kvh * G + i16) * 128 + ks * 32 + g * 8);
    } else {
#pragma unroll
      for (int e = 0; e < 8; e++) qf[ks][e] = (half_t)0;
    }
  }

  char* my_lds = lds + wave * PD_WAVE_LDS;
  const size_t tok_stride = (size_t)num_kv_heads * 128;  // halfs between consecutive tokens of a page
  const half_t* k_lane = Kc + (size_t)kvh * 128 + i16 * tok_stride + g * 8;
  // V direct-to-LDS: wave-load i moves rows 4i .. 4i+3; lane: row 4i + lane/16, slot lane%16
  const int vl_row = lane >> 4, vl_slot = lane & 15;
  const half_t* v_lane = Vc + (size_t)kvh * 128 + vl_row * tok_stride;
  // V transpose reads: lane (i16, g) reads row 4g + i16/4, bytes 32*dt + 8*(i16%4) of the row
  const int vr_row = 4 * g + (i16 >> 2);
  const int vr_base = vr_row * 256 + ((((i16 & 3) >> 1) ^ (2 * (vr_row & 7))) * 16) + (i16 & 1) * 8;  // ^ (dt*32)

  half8 kf[2][2][4];  // [buffer][page][ks]
  // A table entry outside [0, num_pages) (a stale or padding id inside a sequence's live range) must not become an
  // address: such a block is fetched from page 0 instead and bad[buffer] remembers to drop it -- its scores become
  // -inf and its V rows zero, so it contributes nothing.  Wave-uniform, so the flags live in scalar registers.
  int bad[2] = {0, 0};  // bit x: block x of the step in this buffer is dropped
  auto issue = [&](int step, int buf) {
    const int pa = p_begin + 2 * (wave + PD_WAVES * step);
    // the kernel walks 16-token blocks; a page of 16 << page_shift tokens is that many consecutive blocks
    const int sub = (1 << page_shift) - 1;
    int id0 = bt[pa >> page_shift];
    int id1 = (pa + 1 < p_end) ? bt[(pa + 1) >> page_shift] : id0;
    const int drop0 = (unsigned)id0 >= (unsigned)num_pages, drop1 = (unsigned)id1 >= (unsigned)num_pages;
    id0 = drop0 ? 0 : id0;
    id1 = drop1 ? 0 : id1;
    bad[buf] = drop0 | (drop1 << 1);
    const int pg0 = (id0 << page_shift) + (pa & sub);
    const int pg1 = (pa + 1 < p_end) ? (id1 << page_shift) + ((pa + 1) & sub) : pg0;
    char* dst = my_lds + buf * 8192;
#pragma unroll
    for (int x = 0; x < 2; x++) {
      const size_t page_off = (size_t)(x ? pg1 : pg0) * 16 * tok_stride;
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const int chunk = vl_slot ^ (2 * ((4 * (i & 1) + vl_row) & 7));
        load_lds_16B(v_lane + page_off + (size_t)(4 * i) * tok_stride + chunk * 8, dst + x * 4096 + i * 1024);
      }
    }
#pragma unroll
    for (int x = 0; x < 2; x++) {
      const size_t page_off = (size_t)(x ? pg1 : pg0) * 16 * tok_stride;
#pragma unroll
      for (int ks = 0; ks < 4; ks++) kf[buf][x][ks] = *reinterpret_cast<const half8*>(k_lane + page_off + ks * 32);
    }
  };

  floatx4 oacc[8];
#pragma unroll
  for (int dt = 0; dt < 8; dt++) oacc[dt] = floatx4{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY, l_run = 0.f;

  const int my_steps = n_steps > wave ? (n_steps - wave + PD_WAVES - 1) / PD_WAVES : 0;
  if (my_steps > 0) issue(0, 0);
#pragma unroll 1
  for (int u = 0; u < my_steps; u += 2) {
    // two steps per trip so that the register buffers are indexed statically
#pragma unroll
    for (int b = 0; b < 2; b++) {
      const int step = u + b;
      if (step < my_steps) {
        if (step + 1 < my_steps) {
          issue(step + 1, b ^ 1);
          asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
        } else {
          asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
        const int pa = p_begin + 2 * (wave + PD_WAVES * step);
        const bool drop0 = bad[b] & 1;
        const bool has1 = pa + 1 < p_end && !(bad[b] & 2);
        floatx4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < 4; ks++) s0 = mfma16_16x16x32<BF>(kf[b][0][ks], qf[ks], s0);
#pragma unroll
        for (int ks = 0; ks < 4; ks++) s1 = mfma16_16x16x32<BF>(kf[b][1][ks], qf[ks], s1);
        // lane (head i16, g) holds tokens 4g + r of each page
        const int tok0 = pa * 16 + 4 * g;
        const bool ragged = pa * 16 + 32 > L || bad[b] != 0;  // wave-uniform: this step reaches past the sequence end or drops a block
#pragma unroll
        for (int r = 0; r < 4; r++) {
          if (drop0 || tok0 + r >= L || tok0 + r < lo) s0[r] = -INFINITY;
          if (!has1 || tok0 + 16 + r >= L) s1[r] = -INFINITY;  // the second page of a step lies behind `lo`
        }
        float mx = fmaxf(fmaxf(fmaxf(s0[0], s0[1]), fmaxf(s0[2], s0[3])), fmaxf(fmaxf(s1[0], s1[1]), fmaxf(s1[2], s1[3])));
        mx = fmaxf(mx, __shfl_xor(mx, 16));
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        // block pa holds a valid token (the window's first or its own first) unless it was dropped: m_new may still be
        // -inf then, and (-inf) - (-inf) must not reach the exponentials
        const float m_new = fmaxf(m_run, mx);
        const bool none_yet = m_new == -INFINITY;
        const float alpha = none_yet ? 1.f : fast_exp2((m_run - m_new) * scale_log2e);
        const float mc = none_yet ? 0.f : m_new * scale_log2e;
        m_run = m_new;
        half8 pf;
        float psum = 0.f;
#pragma unroll
        for (int r = 0; r < 4; r++) {
          const float p0 = fast_exp2(s0[r] * scale_log2e - mc);
          const float p1 = fast_exp2(s1[r] * scale_log2e - mc);
          psum += p0 + p1;
          pf[r] = cvt16<BF>(p0);
          pf[4 + r] = cvt16<BF>(p1);
        }
        l_run = l_run * alpha + psum;
        const char* vst = my_lds + b * 8192;
#pragma unroll
        for (int dt = 0; dt < 8; dt++) {
          half4 lo = lds_read_tr16(vst + (vr_base ^ (dt * 32)));
          half4 hi = lds_read_tr16(vst + 4096 + (vr_base ^ (dt * 32)));
          if (ragged) {  // tokens at or beyond L may hold anything (NaN included): 0 * garbage must stay 0
#pragma unroll
            for (int e = 0; e < 4; e++) {
              if (drop0 || tok0 + e >= L) lo[e] = (half_t)0;
              if (!has1 || tok0 + 16 + e >= L) hi[e] = (half_t)0;
            }
          }
          half8 vf = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
          oacc[dt] = oacc[dt] * alpha;
          oacc[dt] = mfma16_16x16x32<BF>(vf, pf, oacc[dt]);
        }
      }
    }
  }

  // ---- merge the four waves through LDS ----
  l_run += __shfl_xor(l_run, 16);
  l_run += __shfl_xor(l_run, 32);
  __syncthreads();  // every wave is done with its V ring
  float* sm = reinterpret_cast<float*>(lds);              // [wave][G]
  float* sl = sm + PD_WAVES * 16;                         // [wave][G]
  float* sacc = sl + PD_WAVES * 16;                       // [wave][G][128]
  if (i16 < G) {
    if (g == 0) {
      sm[wave * 16 + i16] = m_run;
      sl[wave * 16 + i16] = l_run;
    }
#pragma unroll
    for (int dt = 0; dt < 8; dt++)
      *reinterpret_cast<floatx4*>(sacc + ((wave * G + i16) * 128 + dt * 16 + 4 * g)) = oacc[dt];
  }
  __syncthreads();
  for (int idx = threadIdx.x; idx < G * 128; idx += PD_WAVES * 64) {
    const int hd = idx >> 7, d = idx & 127;
    float m_tot = -INFINITY;
#pragma unroll
    for (int w = 0; w < PD_WAVES; w++) m_tot = fmaxf(m_tot, sm[w * 16 + hd]);
    float acc = 0.f, l = 0.f;
    if (m_tot > -INFINITY) {
#pragma unroll
      for (int w = 0; w < PD_WAVES; w++) {
        const float mw = sm[w * 16 + hd];
        const float wgt = mw > -INFINITY ? fast_exp2((mw - m_tot) * scale_log2e) : 0.f;
        acc += wgt * sacc[(w * G + hd) * 128 + d];
        l += wgt * sl[w * 16 + hd];
      }
    }
    const int qh = kvh * G + hd;
    if (out) {
      out[((size_t)seq * num_q_heads + qh) * 128 + d] = cvt16<BF>(l > 0.f ? acc / l : 0.f);
    } else {
      const size_t pidx = ((size_t)seq * num_q_heads + qh) * num_splits + split;
      // device-scope stores: written through to where every XCD sees them, so the merging workgroup needs no
      // cache-wide write-back or invalidate (one of those per workgroup cost 3x the kernel's time)
      __hip_atomic_store(part_acc + pidx * 128 + d, acc, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (d == 0) {
        __hip_atomic_store(part_ml + pidx * 2, m_tot * scale_log2e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(part_ml + pidx * 2 + 1, l, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
  }
  if (out || !arrivals) return;

  // ---- merge of the splits by whichever workgroup of this (sequence, kv head) finishes last ----
  // Every workgroup waits until its partials are written, then counts itself in on the (sequence, kv head) counter;
  // the one that completes the count merges the splits (what paged_decode_phase1 does in a launch of its own) and puts
  // the counter back to zero.
  // Ordering.  The partials are written with device-scope stores: they go through to the memory every XCD sees (no
  // dirty line stays behind in this XCD's L2).  vmcnt(0) returns once all of them are acknowledged there, and only
  // then is the counter's read-modify-write issued, itself at device scope, so it executes behind the stores in the
  // one place all workgroups' accesses to that word are ordered.  A workgroup that observes the completed count
  // therefore runs after every other workgroup's partials are in memory, and reads them with device-scope loads,
  // which do not hit in a cache that could hold an older copy.  That is release (stores, wait, RMW) and acquire (RMW,
  // then loads) spelled with a wait and cache-bypassing accesses instead of cache-wide write-back and invalidate
  // operations: one of those per workgroup tripled the kernel's time.
  // The counter word is (epoch << 12) | count.  A word that carries another epoch -- whatever an earlier call that
  // did not run to its end, or memory that was never cleared, left behind -- counts as zero, so a call does not
  // depend on what it finds; epochs are handed out per call by the launcher (1 .. 2^20 - 1, cyclic).
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  int* flag = reinterpret_cast<int*>(lds);
  if (threadIdx.x == 0) {
    unsigned* ctr = reinterpret_cast<unsigned*>(arrivals) + (size_t)seq * num_kv_heads + kvh;
    unsigned seen = __hip_atomic_load(ctr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    unsigned count;
    do {  // at most num_splits workgroups contend for the word
      count = ((seen >> 12) == epoch ? (seen & 0xFFFu) : 0u) + 1u;
    } while (!__hip_atomic_compare_exchange_strong(ctr, &seen, (epoch << 12) | count, __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                                   __HIP_MEMORY_SCOPE_AGENT));
    const int last = count == (unsigned)num_splits;
    if (last) __hip_atomic_store(ctr, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    *flag = last;
  }
  __syncthreads();
  if (!*flag) return;
  for (int idx = threadIdx.x; idx < G * 128; idx += PD_WAVES * 64) {
    const int hd = idx >> 7, d = idx & 127;
    const size_t row = (size_t)seq * num_q_heads + kvh * G + hd;
    final_out[row * 128 + d] = cvt16<BF>(merge_splits<true>(part_acc, part_ml, row, d, num_splits));
  }
}

// Phase 1: one wave per (seq, q head); lane handles d = 2*lane, 2*lane + 1.
template <bool BF>
__global__ __launch_bounds__(64) void paged_decode_phase1(const float* __restrict__ part_acc,
                                                          const float* __restrict__ part_ml, half_t* __restrict__ out,
                                                          int num_splits) {
  const size_t row = blockIdx.x;
  const int lane = threadIdx.x;
  half2v o;
  if (num_splits <= 8) {
    // the usual case: every load of the row is issued before the first is used (one memory round trip instead of
    // one per split); the arithmetic is merge_splits' own, operation for operation
    const float* ml = part_ml + row * num_splits * 2;
    float m[8], ls[8];
    floatx2 a[8];
#pragma unroll
    for (int s = 0; s < 8; s++) {
      const bool on = s < num_splits;
      m[s] = on ? ml[2 * s] : -INFINITY;
      ls[s] = on ? ml[2 * s + 1] : 0.f;
      a[s] = on ? *reinterpret_cast<const floatx2*>(part_acc + (row * num_splits + s) * 128 + 2 * lane) : floatx2{0.f, 0.f};
    }
    float m_tot = -INFINITY;
#pragma unroll
    for (int s = 0; s < 8; s++) m_tot = fmaxf(m_tot, m[s]);
    float acc0 = 0.f, acc1 = 0.f, l = 0.f;
    if (m_tot > -INFINITY) {
#pragma unroll
      for (int s = 0; s < 8; s++) {
        if (m[s] > -INFINITY) {
          const float w = fast_exp2(m[s] - m_tot);
          acc0 = __builtin_fmaf(w, a[s][0], acc0);
          acc1 = __builtin_fmaf(w, a[s][1], acc1);
          l = __builtin_fmaf(w, ls[s], l);
        }
      }
    }
    const float inv = l > 0.f ? 1.f / l : 0.f;
    float r0 = acc0 * inv, r1 = acc1 * inv;
    asm volatile("" : "+v"(r0), "+v"(r1));  // rounded fp32 products, as in merge_splits
    o = half2v{cvt16<BF>(r0), cvt16<BF>(r1)};
  } else {
    o = half2v{cvt16<BF>(merge_splits<false>(part_acc, part_ml, row, 2 * lane, num_splits)),
               cvt16<BF>(merge_splits<false>(part_acc, part_ml, row, 2 * lane + 1, num_splits))};
  }
  *reinterpret_cast<half2v*>(out + row * 128 + 2 * lane) = o;
}

static const char* kDecodeVariants[] = {"d128_p16_w4_2pages"};
int decode_variant_count() { return 1; }
const char* decode_variant_name(int i) { return i == 0 ? kDecodeVariants[0] : nullptr; }

// A fresh tag for the arrival counters of the one-launch form, 1 .. 2^20 - 1, per call and process-wide.
static unsigned next_decode_epoch() {
  static std::atomic<unsigned> counter{0};
  return counter.fetch_add(1, std::memory_order_relaxed) % ((1u << 20) - 1u) + 1u;
}

template <int G, bool BF>
static int launch_phase0(const void* q, const void* kc, const void* vc, const int32_t* bt, const int32_t* sl, float* pacc,
                         float* pml, void* out, void* final_out, int32_t* arrivals, int num_seqs, int num_kv_heads, int max_pages,
                         int num_splits, float scale, int window, int page_shift, int num_pages, hipStream_t stream) {
  auto kern = paged_decode_phase0<G, BF>;
  constexpr int lds_bytes = PD_WAVES * PD_WAVE_LDS;
  static_assert(lds_bytes >= (int)((2 * PD_WAVES * 16 + PD_WAVES * G * 128) * sizeof(float)), "merge area must fit");
  static std::atomic<uint64_t> lds_ok{0};
  if (int rc = allow_lds(reinterpret_cast<const void*>(kern), lds_bytes, lds_ok, "paged_decode_phase0")) return rc;
  dim3 grid(num_splits, num_kv_heads, num_seqs), block(PD_WAVES * 64);
  hipLaunchKernelGGL(kern, grid, block, lds_bytes, stream, (const half_t*)q, (const half_t*)kc, (const half_t*)vc, bt, sl,
                     pacc, pml, (half_t*)out, (half_t*)final_out, num_kv_heads, max_pages, num_splits, scale * 1.4426950408889634f, window,
                     page_shift, num_pages, arrivals, arrivals ? next_decode_epoch() : 0u);
  return check_launch("paged_decode_phase0", grid, block, lds_bytes);
}

// 16 << shift tokens per page, shift 0..4; -1 for any other size
static int page_shift_of(int64_t page_size) {
  for (int sh = 0; sh <= 4; sh++)
    if (page_size == (16ll << sh)) return sh;
  return -1;
}

static int check_decode_args(const char* fn, int64_t num_seqs, int64_t hq, int64_t hkv, int64_t D, int64_t page_size,
                             int64_t max_pages, int64_t num_pages, int64_t num_splits, float scale) {
  if (D != 128) return fail(-MI355_E_SHAPE, "%s: head dim %lld not supported (only 128)", fn, (long long)D);
  if (page_shift_of(page_size) < 0)
    return fail(-MI355_E_SHAPE, "%s: page size %lld not supported (16, 32, 64, 128 or 256)", fn, (long long)page_size);
  if (num_pages > (1 << 26)) return fail(-MI355_E_SHAPE, "%s: too many pages", fn);
  if (num_seqs <= 0 || hq <= 0 || hkv <= 0 || max_pages <= 0 || num_pages <= 0 || num_seqs > 65535 || hkv > 65535)
    return fail(-MI355_E_SHAPE, "%s: bad sizes seqs=%lld hq=%lld hkv=%lld max_pages=%lld num_pages=%lld", fn,
                (long long)num_seqs, (long long)hq, (long long)hkv, (long long)max_pages, (long long)num_pages);
  if (hq % hkv != 0) return fail(-MI355_E_SHAPE, "%s: q heads %lld not a multiple of kv heads %lld", fn, (long long)hq, (long long)hkv);
  const int64_t G = hq / hkv;
  if (G != 1 && G != 2 && G != 4 && G != 8 && G != 16)
    return fail(-MI355_E_SHAPE, "%s: q heads per kv head = %lld, supported: 1, 2, 4, 8, 16", fn, (long long)G);
  if (num_splits < 1 || num_splits > 1024) return fail(-MI355_E_SHAPE, "%s: num_splits %lld out of range [1, 1024]", fn, (long long)num_splits);
  if (max_pages > (1 << 22)) return fail(-MI355_E_SHAPE, "%s: block table too wide (%lld pages per sequence)", fn, (long long)max_pages);
  if (!(scale > 0.f) || !isfinite(scale)) return fail(-MI355_E_SHAPE, "%s: scale must be positive and finite", fn);
  return 0;
}

template <bool BF>
static int run_phase0(const void* q, const void* kc, const void* vc, const int32_t* bt, const int32_t* sl, float* pacc,
                      float* pml, void* out, void* final_out, int32_t* arrivals, int64_t num_seqs, int64_t hq, int64_t hkv,
                      int64_t max_pages,
                      int64_t num_splits, float scale, int window, int page_shift, int64_t num_pages, hipStream_t stream) {
  const int G = (int)(hq / hkv);
#define MI355_PD_CASE(GG) \
  case GG: return launch_phase0<GG, BF>(q, kc, vc, bt, sl, pacc, pml, out, final_out, arrivals, (int)num_seqs, (int)hkv, (int)max_pages, (int)num_splits, scale, window, page_shift, (int)num_pages, stream)
  switch (G) {
    MI355_PD_CASE(1);
    MI355_PD_CASE(2);
    MI355_PD_CASE(4);
    MI355_PD_CASE(8);
    MI355_PD_CASE(16);
  }
#undef MI355_PD_CASE
  return fail(-MI355_E_SHAPE, "paged_decode: unsupported group size %d", G);
}

}  // namespace mi355

using namespace mi355;

template <bool BF>
static int phase0_entry(const void* q, const void* k_cache, const void* v_cache, const int32_t* block_table,
                        const int32_t* seq_lens, float* part_acc, float* part_ml, int64_t num_seqs, int64_t num_q_heads,
                        int64_t num_kv_heads, int64_t D, int64_t page_size, int64_t max_pages_per_seq, int64_t num_pages,
                        int64_t num_splits, float scale, void* stream) {
  if (!q || !k_cache || !v_cache || !block_table || !seq_lens) return fail(-MI355_E_NULL, "paged_decode_phase0: null pointer");
  if (int rc = check_decode_args("paged_decode_phase0", num_seqs, num_q_heads, num_kv_heads, D, page_size, max_pages_per_seq,
                                 num_pages, num_splits, scale))
    return rc;
  if (!part_acc || !part_ml) return fail(-MI355_E_SCRATCH, "paged_decode_phase0: part_acc / part_ml scratch is required");
  if (!aligned16(q) || !aligned16(k_cache) || !aligned16(v_cache) || !aligned16(part_acc))
    return fail(-MI355_E_ALIGN, "paged_decode_phase0: q, k_cache, v_cache, part_acc must be 16-byte aligned");
  return run_phase0<BF>(q, k_cache, v_cache, block_table, seq_lens, part_acc, part_ml, nullptr, nullptr, nullptr, num_seqs,
                        num_q_heads, num_kv_heads, max_pages_per_seq, num_splits, scale, 0, page_shift_of(page_size), num_pages,
                           reinterpret_cast<hipStream_t>(stream));
}

extern "C" int mi355_paged_decode_phase0(const void* q, const void* k_cache, const void* v_cache, const int32_t* block_table,
                                         const int32_t* seq_lens, float* part_acc, float* part_ml, int64_t num_seqs,
                                         int64_t num_q_heads, int64_t num_kv_heads, int64_t D, int64_t page_size,
                                         int64_t max_pages_per_seq, int64_t num_pages, int64_t num_splits, float scale,
                                         void* stream) {
  return phase0_entry<false>(q, k_cache, v_cache, block_table, seq_lens, part_acc, part_ml, num_seqs, num_q_heads, num_kv_heads, D,
                             page_size, max_pages_per_seq, num_pages, num_splits, scale, stream);
}

extern "C" int mi355_paged_decode_phase0_bf16(const void* q, const void* k_cache, const void* v_cache,
                                              const int32_t* block_table, const int32_t* seq_lens, float* part_acc,
                                              float* part_ml, int64_t num_seqs, int64_t num_q_heads, int64_t num_kv_heads,
                                              int64_t D, int64_t page_size, int64_t max_pages_per_seq, int64_t num_pages,
                                              int64_t num_splits, float scale, void* stream) {
  return phase0_entry<true>(q, k_cache, v_cache, block_table, seq_lens, part_acc, part_ml, num_seqs, num_q_heads, num_kv_heads, D,
                            page_size, max_pages_per_seq, num_pages, num_splits, scale, stream);
}

template <bool BF>
static int run_phase1(const float* part_acc, const float* part_ml, void* out, int64_t num_seqs, int64_t num_q_heads, int64_t D,
                      int64_t num_splits, void* stream) {
  if (!part_acc || !part_ml || !out) return fail(-MI355_E_NULL, "paged_decode_phase1: null pointer");
  if (D != 128) return fail(-MI355_E_SHAPE, "paged_decode_phase1: head dim %lld not supported (only 128)", (long long)D);
  if (num_seqs <= 0 || num_q_heads <= 0 || num_splits < 1 || num_splits > 1024 || num_seqs * num_q_heads > (1ll << 30))
    return fail(-MI355_E_SHAPE, "paged_decode_phase1: bad sizes");
  dim3 grid((unsigned)(num_seqs * num_q_heads)), block(64);
  hipLaunchKernelGGL(paged_decode_phase1<BF>, grid, block, 0, reinterpret_cast<hipStream_t>(stream), part_acc, part_ml,
                     (half_t*)out, (int)num_splits);
  return check_launch("paged_decode_phase1", grid, block, 0);
}

extern "C" int mi355_paged_decode_phase1(const float* part_acc, const float* part_ml, void* out, int64_t num_seqs,
                                         int64_t num_q_heads, int64_t D, int64_t num_splits, void* stream) {
  return run_phase1<false>(part_acc, part_ml, out, num_seqs, num_q_heads, D, num_splits, stream);
}

extern "C" int mi355_paged_decode_phase1_bf16(const float* part_acc, const float* part_ml, void* out, int64_t num_seqs,
                                              int64_t num_q_heads, int64_t D, int64_t num_splits, void* stream) {
  return run_phase1<true>(part_acc, part_ml, out, num_seqs, num_q_heads, D, num_splits, stream);
}

template <bool BF>
static int decode_attn(const char* fn, const void* q, const void* k_cache, const void* v_cache, const int32_t* block_table,
                       const int32_t* seq_lens, void* out, float* part_acc, float* part_ml, int32_t* arrivals, int64_t num_seqs,
                       int64_t num_q_heads, int64_t num_kv_heads, int64_t D, int64_t page_size, int64_t max_pages_per_seq,
                       int64_t num_pages, int64_t num_splits, float scale, int64_t window, void* stream) {
  if (!q || !k_cache || !v_cache || !block_table || !seq_lens || !out) return fail(-MI355_E_NULL, "%s: null pointer", fn);
  if (int rc = check_decode_args(fn, num_seqs, num_q_heads, num_kv_heads, D, page_size, max_pages_per_seq, num_pages,
                                 num_splits, scale))
    return rc;
  if (window < 0 || window > (1ll << 30)) return fail(-MI355_E_SHAPE, "%s: window %lld out of range [0, 2^30]", fn, (long long)window);
  if (!aligned16(q) || !aligned16(k_cache) || !aligned16(v_cache) || !aligned16(out))
    return fail(-MI355_E_ALIGN, "%s: q, k_cache, v_cache, out must be 16-byte aligned", fn);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (num_splits == 1)
    return run_phase0<BF>(q, k_cache, v_cache, block_table, seq_lens, nullptr, nullptr, out, nullptr, nullptr, num_seqs, num_q_heads,
                          num_kv_heads, max_pages_per_seq, 1, scale, (int)window, page_shift_of(page_size), num_pages, s);
  if (!part_acc || !part_ml) return fail(-MI355_E_SCRATCH, "%s: num_splits > 1 needs part_acc / part_ml scratch", fn);
  if (!aligned16(part_acc)) return fail(-MI355_E_ALIGN, "%s: part_acc must be 16-byte aligned", fn);
  // One launch, the last workgroup of every (sequence, kv head) merging, pays a store acknowledgement and an atomic
  // round trip (about 3 us) at the end of EVERY workgroup, during which its LDS keeps the next workgroup off the CU.
  // With all workgroups resident at once (two per CU) that wait is hidden behind nothing and still costs less than
  // a second launch (1 sequence x 32768 tokens: one launch is ahead); with several rounds of workgroups it adds up
  // to more than the merge kernel's 5 us (the 64-sequence benchmark batch: 216 us against 211), so those grids keep
  // the two launches.
  const bool one_launch = arrivals && num_splits * num_kv_heads * num_seqs <= 2 * 256;
  if (one_launch)
    return run_phase0<BF>(q, k_cache, v_cache, block_table, seq_lens, part_acc, part_ml, nullptr, out, arrivals, num_seqs,
                          num_q_heads, num_kv_heads, max_pages_per_seq, num_splits, scale, (int)window, page_shift_of(page_size),
                          num_pages, s);
  if (int rc = run_phase0<BF>(q, k_cache, v_cache, block_table, seq_lens, part_acc, part_ml, nullptr, nullptr, nullptr, num_seqs,
                              num_q_heads, num_kv_heads, max_pages_per_seq, num_splits, scale, (int)window,
                              page_shift_of(page_size), num_pages, s))
    return rc;
  return run_phase1<BF>(part_acc, part_ml, out, num_seqs, num_q_heads, D, num_splits, stream);
}

extern "C" int mi355_paged_decode_attn_fused(const void* q, const void* k_cache, const void* v_cache,
                                             const int32_t* block_table, const int32_t* seq_lens, void* out, float* part_acc,
                                             float* part_ml, int32_t* arrivals, int64_t num_seqs, int64_t num_q_heads,
                                             int64_t num_kv_heads, int64_t D, int64_t page_size, int64_t max_pages_per_seq,
                                             int64_t num_pages, int64_t num_splits, float scale, int64_t window, int dtype,
                                             void* stream) {
  const char* fn = "paged_decode_attn_fused";
  if (dtype != MI355_F16 && dtype != MI355_BF16) return fail(-MI355_E_DTYPE, "%s: dtype %d (MI355_F16 or MI355_BF16)", fn, dtype);
  if (dtype == MI355_BF16)
    return decode_attn<true>(fn, q, k_cache, v_cache, block_table, seq_lens, out, part_acc, part_ml, arrivals, num_seqs, num_q_heads,
                             num_kv_heads, D, page_size, max_pages_per_seq, num_pages, num_splits, scale, window, stream);
  return decode_attn<false>(fn, q, k_cache, v_cache, block_table, seq_lens, out, part_acc, part_ml, arrivals, num_seqs, num_q_heads,
                            num_kv_heads, D, page_size, max_pages_per_seq, num_pages, num_splits, scale, window, stream);
}

extern "C" int mi355_paged_decode_attn(const void* q, const void* k_cache, const void* v_cache, const int32_t* block_table,
                                       const int32_t* seq_lens, void* out, float* part_acc, float* part_ml, int64_t num_seqs,
                                       int64_t num_q_heads, int64_t num_kv_heads, int64_t D, int64_t page_size,
                                       int64_t max_pages_per_seq, int64_t num_pages, int64_t num_splits, float scale,
                                       void* stream) {
  return decode_attn<false>("paged_decode_attn", q, k_cache, v_cache, block_table, seq_lens, out, part_acc, part_ml, nullptr, num_seqs,
                     num_q_heads, num_kv_heads, D, page_size, max_pages_per_seq, num_pages, num_splits, scale, 0, stream);
}

extern "C" int mi355_paged_decode_attn_window(const void* q, const void* k_cache, const void* v_cache,
                                              const int32_t* block_table, const int32_t* seq_lens, void* out, float* part_acc,
                                              float* part_ml, int64_t num_seqs, int64_t num_q_heads, int64_t num_kv_heads,
                                              int64_t D, int64_t page_size, int64_t max_pages_per_seq, int64_t num_pages,
                                              int64_t num_splits, float scale, int64_t window, void* stream) {
  return decode_attn<false>("paged_decode_attn_window", q, k_cache, v_cache, block_table, seq_lens, out, part_acc, part_ml, nullptr,
                            num_seqs, num_q_heads, num_kv_heads, D, page_size, max_pages_per_seq, num_pages, num_splits, scale,
                            window, stream);
}

extern "C" int mi355_paged_decode_attn_window_bf16(const void* q, const void* k_cache, const void* v_cache,
                                                   const int32_t* block_table, const int32_t* seq_lens, void* out,
                                                   float* part_acc, float* part_ml, int64_t num_seqs, int64_t num_q_heads,
                                                   int64_t num_kv_heads, int64_t D, int64_t page_size,
                                                   int64_t max_pages_per_seq, int64_t num_pages, int64_t num_splits,
                                                   float scale, int64_t window, void* stream) {
  return decode_attn<true>("paged_decode_attn_window_bf16", q, k_cache, v_cache, block_table, seq_lens, out, part_acc, part_ml, nullptr,
                           num_seqs, num_q_heads, num_kv_heads, D, page_size, max_pages_per_seq, num_pages, num_splits, scale,
                           window, stream);
}

// ---- decode for callers that cannot allocate --------------------------------------------------------------
// The split-K partials live in a file-scope device array instead of caller memory.  Every GPU the library runs on
// holds its own copy of the array (at its own address) until the process ends; the address is looked up once per
// device, with that device current, and kept.
constexpr int64_t PD_STATIC_MAX_ROWS = 32768;  // num_seqs * num_q_heads * num_splits
static __device__ __align__(256) float scratch[PD_STATIC_MAX_ROWS * (128 + 2)];  // 16.25 MiB: part_acc, then part_ml

static std::atomic<float*> g_scratch_ptr[64];  // per device ordinal; host code uses these, never the array's name

static int static_scratch(const char* fn, float** ptr) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) {
    set_error("%s: hipGetDevice: %s", fn, hipGetErrorString(e));
    return (int)e;
  }
  if (dev < 0 || dev >= 64) return fail(-MI355_E_SHAPE, "%s: device ordinal %d not supported (0..63)", fn, dev);
  float* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!p) {
    e = hipGetSymbolAddress(reinterpret_cast<void**>(&p), HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) {
      set_error("%s: hipGetSymbolAddress(scratch) on device %d: %s", fn, dev, hipGetErrorString(e));
      return e != hipSuccess ? (int)e : (int)hipErrorInvalidSymbol;
    }
    g_scratch_ptr[dev].store(p, std::memory_order_release);  // two threads racing here store the same address
  }
  *ptr = p;
  return 0;
}

extern "C" int mi355_paged_decode_attn_static(const void* q, const void* k_cache, const void* v_cache,
                                              const int32_t* block_table, const int32_t* seq_lens, void* out,
                                              int64_t num_seqs, int64_t num_q_heads, int64_t num_kv_heads, int64_t D,
                                              int64_t page_size, int64_t max_pages_per_seq, int64_t num_pages,
                                              int64_t num_splits, float scale, void* stream) {
  const char* fn = "paged_decode_attn_static";
  if (num_splits <= 1)  // a single split needs no partials at all
    return decode_attn<false>(fn, q, k_cache, v_cache, block_table, seq_lens, out, nullptr, nullptr, nullptr, num_seqs, num_q_heads,
                              num_kv_heads, D, page_size, max_pages_per_seq, num_pages, num_splits, scale, 0, stream);
  if (num_seqs <= 0 || num_q_heads <= 0 || num_seqs > PD_STATIC_MAX_ROWS || num_q_heads > PD_STATIC_MAX_ROWS ||
      num_splits > PD_STATIC_MAX_ROWS || num_seqs * num_q_heads * num_splits > PD_STATIC_MAX_ROWS)
    return fail(-MI355_E_SCRATCH, "%s: num_seqs * num_q_heads * num_splits = %lld x %lld x %lld exceeds the built-in scratch "
                "of %lld rows; use mi355_paged_decode_attn with caller-owned scratch", fn, (long long)num_seqs,
                (long long)num_q_heads, (long long)num_splits, (long long)PD_STATIC_MAX_ROWS);
  float* base = nullptr;
  if (int rc = static_scratch(fn, &base)) return rc;
  // Phase 0 writes every (seq, q head, split) row of both arrays -- an empty split writes (-inf, 0, zeros) -- so
  // nothing of the previous call's contents is read and nothing needs clearing.
  float* part_acc = base;
  float* part_ml = base + num_seqs * num_q_heads * num_splits * 128;
  return decode_attn<false>(fn, q, k_cache, v_cache, block_table, seq_lens, out, part_acc, part_ml, nullptr, num_seqs, num_q_heads,
                            num_kv_heads, D, page_size, max_pages_per_seq, num_pages, num_splits, scale, 0, stream);
}

// ---- KV-cache append: the step in front of decode -------------------------------------------------------
// Writes tokens start_pos[s] .. start_pos[s] + n_new - 1 of every sequence into its pages.  A token's kv
// heads are contiguous both in the source ([seq][token][head][128]) and in a page slot, so one token is one
// contiguous run of num_kv_heads * 256 bytes: one wave per token, 16 bytes per lane and pass.
__global__ __launch_bounds__(256) void kv_cache_append_kernel(const half_t* __restrict__ k_new, const half_t* __restrict__ v_new,
                                                              half_t* __restrict__ k_cache, half_t* __restrict__ v_cache,
                                                              const int* __restrict__ block_table,
                                                              const int* __restrict__ start_pos, int n_new, int num_kv_heads,
                                                              int max_pages_per_seq, int num_pages, long long n_tokens,
                                                              int page_bits) {
  const int lane = threadIdx.x & 63;
  const long long tok = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);  // flat (seq, new token) index
  if (tok >= n_tokens) return;
  const int seq = (int)(tok / n_new), t = (int)(tok - (long long)seq * n_new);
  const int pos = start_pos[seq] + t;
  if (pos < 0) return;
  const int pidx = pos >> page_bits;  // page_bits = log2(tokens per page)
  if (pidx >= max_pages_per_seq) return;  // no table entry for this position: nothing is written
  const int page = block_table[(size_t)seq * max_pages_per_seq + pidx];
  if (page < 0 || page >= num_pages) return;  // padded entry
  const int row_halfs = num_kv_heads * 128;
  const size_t src = (size_t)tok * row_halfs;
  const size_t dst = (((size_t)page << page_bits) + (pos & ((1 << page_bits) - 1))) * row_halfs;
  for (int c = lane * 8; c < row_halfs; c += 512) {
    *reinterpret_cast<half8*>(k_cache + dst + c) = *reinterpret_cast<const half8*>(k_new + src + c);
    *reinterpret_cast<half8*>(v_cache + dst + c) = *reinterpret_cast<const half8*>(v_new + src + c);
  }
}

extern "C" int mi355_kv_cache_append(const void* k_new, const void* v_new, void* k_cache, void* v_cache,
                                     const int32_t* block_table, const int32_t* start_pos, int64_t num_seqs, int64_t n_new,
                                     int64_t num_kv_heads, int64_t D, int64_t page_size, int64_t max_pages_per_seq,
                                     int64_t num_pages, void* stream) {
  if (!k_new || !v_new || !k_cache || !v_cache || !block_table || !start_pos) return fail(-MI355_E_NULL, "kv_cache_append: null pointer");
  if (D != 128) return fail(-MI355_E_SHAPE, "kv_cache_append: head dim %lld not supported (only 128)", (long long)D);
  if (page_shift_of(page_size) < 0)
    return fail(-MI355_E_SHAPE, "kv_cache_append: page size %lld not supported (16, 32, 64, 128 or 256)", (long long)page_size);
  if (num_seqs <= 0 || n_new <= 0 || num_kv_heads <= 0 || max_pages_per_seq <= 0 || num_pages <= 0 || n_new > (1 << 24) ||
      num_kv_heads > 65535 || num_seqs * n_new > (1ll << 40))
    return fail(-MI355_E_SHAPE, "kv_cache_append: bad sizes seqs=%lld n_new=%lld hkv=%lld max_pages=%lld num_pages=%lld",
                (long long)num_seqs, (long long)n_new, (long long)num_kv_heads, (long long)max_pages_per_seq, (long long)num_pages);
  if (!aligned16(k_new) || !aligned16(v_new) || !aligned16(k_cache) || !aligned16(v_cache))
    return fail(-MI355_E_ALIGN, "kv_cache_append: k_new, v_new, k_cache, v_cache must be 16-byte aligned");
  const long long n_tokens = num_seqs * n_new;
  dim3 grid((unsigned)((n_tokens + 3) / 4)), block(256);
  hipLaunchKernelGGL(kv_cache_append_kernel, grid, block, 0, reinterpret_cast<hipStream_t>(stream), (const half_t*)k_new,
                     (const half_t*)v_new, (half_t*)k_cache, (half_t*)v_cache, block_table, start_pos, (int)n_new,
                     (int)num_kv_heads, (int)max_pages_per_seq, (int)num_pages, n_tokens, 4 + page_shift_of(page_size));
  return check_launch("kv_cache_append_kernel", grid, block, 0);
}
