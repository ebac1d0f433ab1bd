// Pieces the GEMM kernels of every operand format share: the workgroup -> tile map, the output conversions of the
// block-scaled kernels, and the epilogue of the streamed block-scaled kernels (MXFP4 and MXFP8 use one LDS map).
#pragma once
#include "common.hpp"

namespace mi355 {

// workgroup -> tile: eight consecutive ids run on eight XCDs, so each XCD (one L2) gets a contiguous run of tiles,
// walked in groups of group_m tile rows
__device__ __forceinline__ void map_tile(int pid, int tiles_m, int tiles_n, int group_m, int& tm, int& tn) {
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

// output element types of the block-scaled GEMMs: fp32, or bf16 as its 16 bits
template <typename OutT> struct MxOut;
template <> struct MxOut<float> {
  static __device__ __forceinline__ void store4(float* p, float a, float b, float c, float d) {
    floatx4 v = {a, b, c, d};
    *reinterpret_cast<floatx4*>(p) = v;
  }
  static __device__ __forceinline__ void store1(float* p, float a) { *p = a; }
};
template <> struct MxOut<unsigned short> {  // bf16 bits
  static __device__ __forceinline__ void store4(unsigned short* p, float a, float b, float c, float d) {
    ushortx4 v = {f32_to_bf16_rne(a), f32_to_bf16_rne(b), f32_to_bf16_rne(c), f32_to_bf16_rne(d)};
    *reinterpret_cast<ushortx4*>(p) = v;
  }
  static __device__ __forceinline__ void store1(unsigned short* p, float a) { *p = f32_to_bf16_rne(a); }
};

// Epilogue of the streamed block-scaled kernels (256x256 tile, 4 waves of 128x128, acc[n block][m block] in AGPRs
// written by inline-assembly MFMAs).  tile_c points at the wave's first output element, N is the row pitch of C, ep
// the LDS address of the wave's private 2 KiB staging region (free until the workgroup's next barrier).  ALPHA:
// every sum is multiplied by alpha first.
template <bool ALPHA, typename OutT>
__device__ __forceinline__ void mx_stream_epilogue(floatx4 (&acc)[8][8], float alpha, OutT* tile_c, int N, unsigned ep) {
  // The MFMAs are inline assembly, so the compiler does not know that the accumulators were written just now: the
  // wait states an MFMA result needs before another instruction may read it are spelled out, and every accumulator is
  // tied to a statement behind them so that no read of it can be scheduled earlier.
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
#pragma unroll
  for (int i = 0; i < 8; i++)
    asm volatile("" : "+a"(acc[i][0]), "+a"(acc[i][1]), "+a"(acc[i][2]), "+a"(acc[i][3]), "+a"(acc[i][4]), "+a"(acc[i][5]),
                      "+a"(acc[i][6]), "+a"(acc[i][7]));
  auto val = [&](float x) { return ALPHA ? alpha * x : x; };
  // lane holds, for m = 16 j + (l & 15): n = 16 i + 4 (l >> 4) + r, r < 4.  The addresses come from a lane id the
  // compiler cannot see through, so that none of them is computed ahead of the K loop and kept across it.
  const int le = opaque_lane_id();
  const int r16e = le & 15, cqe = le >> 4;
  if constexpr (sizeof(OutT) == 2) {
    // bf16 results go through LDS, 16 rows x 64 columns (2 KiB) per pass: 8-byte writes of 4 consecutive n (chunk slot
    // c ^ ((m >> 1) & 7) of the 128-byte row), whole rows read back 16 bytes per lane and stored as full cache lines.
    // LDS operations of a wave execute in order, so the passes need no waits between them.  Inline assembly like the
    // K loop's LDS accesses: direct-to-LDS loads of the next tile are in flight, and the compiler would wait for all
    // of them in front of an LDS access it can see.
    const int er = le >> 3, ec = le & 7, sw = (r16e >> 1) & 7;
    // write: row r16e, chunk (2 (i & 3) + (cqe >> 1)) ^ sw, 8-byte half cqe & 1; the i term is an XOR of the address
    const unsigned wa = ep + (unsigned)(r16e * 128 + ((((cqe >> 1) ^ (sw & 1)) | (sw & 6)) * 16) + 8 * (cqe & 1));
    // read: row 8 it + er, chunk ec ^ ((row >> 1) & 7) = (ec ^ (er >> 1)) ^ 4 it
    const unsigned ra = ep + (unsigned)(er * 128 + ((ec ^ (er >> 1)) * 16));
    OutT* cbase = tile_c + (size_t)er * N + ec * 8;
#pragma unroll
    for (int j = 0; j < 8; j++) {
#pragma unroll
      for (int ih = 0; ih < 2; ih++) {
#pragma unroll
        for (int ii = 0; ii < 4; ii++) {
          const int i = ih * 4 + ii;
          ushortx4 v = {f32_to_bf16_rne(val(acc[i][j][0])), f32_to_bf16_rne(val(acc[i][j][1])),
                        f32_to_bf16_rne(val(acc[i][j][2])), f32_to_bf16_rne(val(acc[i][j][3]))};
          asm volatile("ds_write_b64 %0, %1" ::"v"(wa ^ (unsigned)(32 * ii)), "v"(v) : "memory");
        }
        half8 rv[2];
        asm volatile("ds_read_b128 %0, %1" : "=v"(rv[0]) : "v"(ra));
        asm volatile("ds_read_b128 %0, %1 offset:1024" : "=v"(rv[1]) : "v"(ra ^ 64u));
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(rv[0]), "+v"(rv[1]));
#pragma unroll
        for (int it = 0; it < 2; it++)  // one store instruction each: the next tile's first waits count past these 32
          store_global_16B(cbase + (size_t)(j * 16 + it * 8) * N + ih * 64, rv[it]);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  } else {
    OutT* crow = tile_c + (size_t)r16e * N + 4 * cqe;
#pragma unroll
    for (int j = 0; j < 8; j++) {
#pragma unroll
      for (int i = 0; i < 8; i++)
        MxOut<OutT>::store4(crow + (size_t)(j * 16) * N + i * 16, val(acc[i][j][0]), val(acc[i][j][1]), val(acc[i][j][2]),
                            val(acc[i][j][3]));
      __builtin_amdgcn_sched_barrier(0);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // 64 stores: more than a wait can count past
  }
}

}  // namespace mi355
