/*
 * turbine_mi355.h -- C ABI of the MI355X (gfx950) dense-kernel library.
 *
 * One shared object, libturbine_mi355.so, exports the functions below.  Every
 * function takes raw device pointers, plain integer sizes and the HIP stream
 * to launch on (a hipStream_t passed as void*; NULL = the legacy default
 * stream).  Nothing here allocates or synchronises, and the caller owns all
 * memory, including split-K scratch.  Two entry points keep state of their own
 * and say so where they are declared: mi355_paged_decode_attn_static (its
 * scratch is a device array inside the library image, one copy per GPU) and
 * mi355_paged_decode_attn_fused (arrival counters in caller memory, tagged
 * with a per-call number the library hands out).
 *
 * Return value: 0 on success; a negative MI355_E_* code when the arguments
 * violate the kernel's contract (nothing was launched); a positive value is
 * the hipError_t reported by the launch.  mi355_last_error() returns a
 * thread-local text describing the most recent failure on this thread.
 *
 * Reference interfaces these entry points stand behind (paths relative to the
 * iree-turbine checkout):
 *   - the eager custom-op hook CustomOp.eager_execute,
 *     iree/turbine/runtime/op_reg/base.py:221-232 and the dispatcher
 *     trampoline at base.py:1061-1072;
 *   - the callable-kernel protocol Launchable.__call__,
 *     iree/turbine/runtime/launch.py:203-272 (contiguous tensors, one device,
 *     launch ordered on torch's current stream, runtime/device.py:336-361);
 *   - the reference itself reaches HIP through ctypes on libamdhip64
 *     (iree/turbine/runtime/device.py:86-150); this header is the same kind
 *     of boundary one level up.
 */
#ifndef TURBINE_MI355_H_
#define TURBINE_MI355_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MI355_ABI_VERSION 1

/* contract-violation codes (returned negated: e.g. -MI355_E_SHAPE) */
#define MI355_E_NULL 1      /* a required pointer is NULL */
#define MI355_E_SHAPE 2     /* a size is non-positive or not supported by any kernel variant */
#define MI355_E_ALIGN 3     /* a pointer is not aligned as the kernel requires (16 bytes) */
#define MI355_E_DTYPE 4     /* unknown out_dtype / variant selector */
#define MI355_E_SCRATCH 5   /* split-K scratch missing or too small */

/* output element types */
#define MI355_F32 0
#define MI355_F16 1
#define MI355_BF16 2

int mi355_abi_version(void);
const char* mi355_last_error(void);
/* "" for the product build.  A library built with timing-only ablation switches (-DMI355_ABLATE_..., see
 * csrc/common.hpp) names them here: such a build computes wrong results on purpose and exists to measure what a part
 * of a kernel costs.  No counterpart in the reference. */
const char* mi355_build_flags(void);

/* Number of kernel variants of a family and the name of variant i
 * (family: "gemm_f16_nt" -- shared by the bf16 entry --, "flash_attn_fwd", "paged_decode",
 * "mxfp4_gemm", "mxfp8_gemm" -- shared by mi355_fp8_gemm --, "mxfp6_gemm"). */
int mi355_variant_count(const char* family);
const char* mi355_variant_name(const char* family, int i);

/*
 * fp16 NT GEMM:  C[M,N] = A[M,K] . B[N,K]^T, fp32 accumulation.
 * A, B: fp16 row-major (K contiguous).  C: row-major, out_dtype MI355_F32 or
 * MI355_F16.  variant < 0 selects by shape; otherwise a variant index.
 * Replaces: BOO GEMMForward with transpose_b (torch.mm(a, b.t())),
 * iree/turbine/kernel/boo/op_exports/gemm.py:217-230, and the TK tiled GEMM
 * of tests/kernel/vector_codegen_test.py:71-100.
 */
int mi355_gemm_f16_nt(const void* a, const void* b, void* c,
                      int64_t M, int64_t N, int64_t K,
                      int out_dtype, int variant, void* stream);

/*
 * The same GEMM with bf16 operands: A, B bf16 row-major (K contiguous), fp32
 * accumulation, C out_dtype MI355_F32 or MI355_BF16 (round to nearest even).
 * Same kernels, variants and shape rules as mi355_gemm_f16_nt.
 * Replaces: aten::mm / aten::addmm signatures with bf16 operands
 * (iree/turbine/kernel/boo/op_exports/aten.py:44-49, dtype names parsed at
 * iree/turbine/kernel/boo/op_exports/aten.py:101-144) and nn.Linear in bf16
 * under the BOO backend (iree/turbine/kernel/boo/ops/graph.py:171-182).
 */
int mi355_gemm_bf16_nt(const void* a, const void* b, void* c,
                       int64_t M, int64_t N, int64_t K,
                       int out_dtype, int variant, void* stream);

/*
 * The same two GEMMs with a caller-provided workspace, which lets the automatic choice (variant < 0) split K:
 * a product with too few 256x256 tiles for the 256 CUs -- the whole product when it has at most 128 such tiles
 * (on 128x128, 128x64 or 64x64 tiles when it is smaller still), or the strip a sparse last round of tiles is cut into -- is computed
 * as S partial products over K ranges (fp32, in the workspace) and one merge launch.  mi355_gemm_nt_workspace_bytes returns the size with which a shape would
 * take that path (0: it would not; the plain entry points do the same work then).  A NULL or smaller workspace is
 * not an error: the call runs as mi355_gemm_f16_nt would.  The workspace is scratch: nothing in it is read before
 * the same call has written it, so one buffer serves any sequence of calls on a stream (calls that overlap on
 * other streams need their own).  Results differ from the plain entry in summation order only (fp32 partial sums
 * added in split order).  Same reference interfaces as mi355_gemm_f16_nt / mi355_gemm_bf16_nt; the workspace
 * arguments have no counterpart there.
 */
int64_t mi355_gemm_nt_workspace_bytes(int64_t M, int64_t N, int64_t K);
int mi355_gemm_f16_nt_ws(const void* a, const void* b, void* c,
                         int64_t M, int64_t N, int64_t K,
                         int out_dtype, int variant,
                         void* workspace, int64_t workspace_bytes, void* stream);
int mi355_gemm_bf16_nt_ws(const void* a, const void* b, void* c,
                          int64_t M, int64_t N, int64_t K,
                          int out_dtype, int variant,
                          void* workspace, int64_t workspace_bytes, void* stream);

/*
 * Flash-attention forward (prefill): O = softmax(scale . Q K^T [+ causal mask]) V.
 * q, o: [B, H, Sq, D]; k, v: [B, H, Sk, D]; all fp16 contiguous; D == 128.
 * fp32 online softmax, fp16 output.  is_causal: query i attends keys
 * j <= i + (Sk - Sq) (lower-right aligned; equals lower-triangular when Sq == Sk).
 * Replaces: aten::scaled_dot_product_attention as canonicalised by
 * iree/turbine/kernel/boo/fusion/replacement.py:275-284, and the TK fused
 * attention of tests/kernel/fused_attention_test.py:25-77.
 */
int mi355_flash_attn_fwd(const void* q, const void* k, const void* v, void* o,
                         int64_t B, int64_t H, int64_t Sq, int64_t Sk, int64_t D,
                         float scale, int is_causal, int variant, void* stream);

/*
 * The same computation on strided operands and with grouped K/V heads, so that
 * a caller holding [B, S, H, D] projections (the `x.view(B, S, H, D).transpose(1, 2)`
 * views a model hands to scaled_dot_product_attention) needs no copies.
 * q, o: logical [B, H, Sq, D]; k, v: logical [B, Hkv, Sk, D] with H % Hkv == 0:
 * query head h reads K/V head h / (H / Hkv)  (enable_gqa semantics).
 * *_strides: {batch, head, row} strides in ELEMENTS; the D elements of a row are
 * contiguous.  Every stride is a non-negative multiple of 8 (16-byte rows), row
 * strides lie in [128, 2^24); a 0 batch or head stride on q, k or v broadcasts.
 * Replaces: the same SDPA root as above for the non-contiguous operands that the
 * reference makes contiguous before every launch
 * (iree/turbine/runtime/op_reg/eager.py:119-132).
 */
int mi355_flash_attn_fwd_strided(const void* q, const void* k, const void* v, void* o,
                                 int64_t B, int64_t H, int64_t Hkv, int64_t Sq, int64_t Sk, int64_t D,
                                 const int64_t* q_strides, const int64_t* k_strides,
                                 const int64_t* v_strides, const int64_t* o_strides,
                                 float scale, int is_causal, int variant, void* stream);

/*
 * bf16 forms of the two entries above: q, k, v, o bf16, fp32 online softmax, the
 * probabilities rounded to bf16 for the second product, bf16 output.  Same kernels
 * (instantiated with the bf16 MFMA), shapes, strides and variants.
 * Replaces: the same SDPA root for bf16 operands -- the reference's signature
 * parser takes the dtype from the tensor type names,
 * iree/turbine/kernel/boo/op_exports/aten.py:101-144.
 */
int mi355_flash_attn_fwd_bf16(const void* q, const void* k, const void* v, void* o,
                              int64_t B, int64_t H, int64_t Sq, int64_t Sk, int64_t D,
                              float scale, int is_causal, int variant, void* stream);
int mi355_flash_attn_fwd_strided_bf16(const void* q, const void* k, const void* v, void* o,
                                      int64_t B, int64_t H, int64_t Hkv, int64_t Sq, int64_t Sk, int64_t D,
                                      const int64_t* q_strides, const int64_t* k_strides,
                                      const int64_t* v_strides, const int64_t* o_strides,
                                      float scale, int is_causal, int variant, void* stream);

/*
 * Paged GQA decode attention, one query token per sequence.
 * q:           [num_seqs, num_q_heads, D]                 fp16
 * k_cache,
 * v_cache:     [num_pages, page_size, num_kv_heads, D]    fp16
 * block_table: [num_seqs, max_pages_per_seq]              int32 page ids; entries at or
 *              beyond ceil(seq_len/page_size) are never read
 * seq_lens:    [num_seqs]                                 int32, >= 0
 * out:         [num_seqs, num_q_heads, D]                 fp16
 * Requirements: D == 128, page_size 16, 32, 64, 128 or 256, num_q_heads == 4 * num_kv_heads or
 * any ratio in {1, 2, 4, 8, 16}.
 *
 * Split-K: phase 0 writes, for every (seq, q head, split), an unnormalised
 * fp32 partial output and its (running max in log2 units, running sum);
 * phase 1 merges the splits.  part_acc: [num_seqs, num_q_heads, num_splits, D]
 * fp32; part_ml: [num_seqs, num_q_heads, num_splits, 2] fp32.
 * mi355_paged_decode_attn runs both phases (num_splits == 1 needs no scratch).
 * No reference counterpart survives in the checkout; semantics follow the GQA
 * KV-cache attention of tests/dynamo/llama_test.py:82-91,160-181.
 */
int mi355_paged_decode_phase0(const void* q, const void* k_cache, const void* v_cache,
                              const int32_t* block_table, const int32_t* seq_lens,
                              float* part_acc, float* part_ml,
                              int64_t num_seqs, int64_t num_q_heads, int64_t num_kv_heads,
                              int64_t D, int64_t page_size, int64_t max_pages_per_seq,
                              int64_t num_pages, int64_t num_splits, float scale, void* stream);
int mi355_paged_decode_phase1(const float* part_acc, const float* part_ml, void* out,
                              int64_t num_seqs, int64_t num_q_heads, int64_t D,
                              int64_t num_splits, void* stream);

/* The two phases with q, k_cache, v_cache (phase 0) and out (phase 1) in bf16; the fp32
 * partial results between them have the same layout and meaning. */
int mi355_paged_decode_phase0_bf16(const void* q, const void* k_cache, const void* v_cache,
                                   const int32_t* block_table, const int32_t* seq_lens,
                                   float* part_acc, float* part_ml,
                                   int64_t num_seqs, int64_t num_q_heads, int64_t num_kv_heads,
                                   int64_t D, int64_t page_size, int64_t max_pages_per_seq,
                                   int64_t num_pages, int64_t num_splits, float scale, void* stream);
int mi355_paged_decode_phase1_bf16(const float* part_acc, const float* part_ml, void* out,
                                   int64_t num_seqs, int64_t num_q_heads, int64_t D,
                                   int64_t num_splits, void* stream);
int mi355_paged_decode_attn(const void* q, const void* k_cache, const void* v_cache,
                            const int32_t* block_table, const int32_t* seq_lens, void* out,
                            float* part_acc, float* part_ml,
                            int64_t num_seqs, int64_t num_q_heads, int64_t num_kv_heads,
                            int64_t D, int64_t page_size, int64_t max_pages_per_seq,
                            int64_t num_pages, int64_t num_splits, float scale, void* stream);

/*
 * Paged decode in ONE launch: as mi355_paged_decode_attn_window (window == 0: all tokens), for fp16
 * or bf16 tensors (dtype = MI355_F16 | MI355_BF16), with the merge of the kv splits done inside the
 * phase-0 kernel by whichever workgroup of a (sequence, kv head) finishes last, instead of by a second
 * launch -- when the whole grid is resident at once (num_seqs * num_kv_heads * num_splits <= 512);
 * larger grids run the two launches, which is faster there, and leave `arrivals` untouched.
 * arrivals: int32 [num_seqs * num_kv_heads] of device memory, the per-(sequence, kv head) arrival
 * counters.  Every call tags the words it counts in with a number of its own (handed out inside the
 * library, 1 .. 2^20 - 1, cyclic) and treats a word that carries another tag as zero, so a call does
 * not depend on the buffer's contents: an earlier call that did not run to its end, or memory that was
 * never cleared, does no harm (short of a stale word that happens to carry this call's tag).  A call
 * that completes leaves its words zero.  One buffer serves every call ordered after this one; calls
 * that may overlap need a buffer each.  A captured graph replays one tag: its replays rely on the words
 * being left zero by the replay before.  arrivals == NULL selects the two launches whatever the
 * grid (for a caller that cannot provide counters, e.g. a first call under stream capture).
 * num_splits <= 512 on this path.  No counterpart in the reference (GQA semantics
 * tests/dynamo/llama_test.py:82-91).
 */
int mi355_paged_decode_attn_fused(const void* q, const void* k_cache, const void* v_cache,
                                  const int32_t* block_table, const int32_t* seq_lens, void* out,
                                  float* part_acc, float* part_ml, int32_t* arrivals,
                                  int64_t num_seqs, int64_t num_q_heads, int64_t num_kv_heads,
                                  int64_t D, int64_t page_size, int64_t max_pages_per_seq,
                                  int64_t num_pages, int64_t num_splits, float scale,
                                  int64_t window, int dtype, void* stream);

/*
 * mi355_paged_decode_attn for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference,
 * whose runtime allocates its results itself (iree/turbine/runtime/op_reg/eager.py:195-199).
 * Same arguments, kernels and results as mi355_paged_decode_attn, fp16, without part_acc / part_ml:
 * the split-K partials go to a 16.25 MiB array that is part of the library's device image (one copy
 * per GPU the library is used on, held until the process ends).  The call allocates nothing and
 * frees nothing.  Limit: num_seqs * num_q_heads * num_splits <= 32768, otherwise -MI355_E_SCRATCH
 * (nothing launched).  Every call on a GPU uses that GPU's one array: calls that may overlap on
 * one GPU (different streams or threads) race on it and must be serialised by the caller; calls
 * on one stream are ordered.  The first call on a device looks up the array's address.
 */
int mi355_paged_decode_attn_static(const void* q, const void* k_cache, const void* v_cache,
                                   const int32_t* block_table, const int32_t* seq_lens, void* out,
                                   int64_t num_seqs, int64_t num_q_heads, int64_t num_kv_heads,
                                   int64_t D, int64_t page_size, int64_t max_pages_per_seq,
                                   int64_t num_pages, int64_t num_splits, float scale, void* stream);

/*
 * Paged decode with a sliding window: as mi355_paged_decode_attn, but a query
 * attends only to the last `window` cached tokens of its sequence (window == 0:
 * all of them).  Pages wholly in front of the window are not read.  Same masking
 * convention as the causal mask of tests/dynamo/llama_test.py:160-181 restricted
 * to a band; the reference has no paged form.
 */
int mi355_paged_decode_attn_window(const void* q, const void* k_cache, const void* v_cache,
                                   const int32_t* block_table, const int32_t* seq_lens, void* out,
                                   float* part_acc, float* part_ml,
                                   int64_t num_seqs, int64_t num_q_heads, int64_t num_kv_heads,
                                   int64_t D, int64_t page_size, int64_t max_pages_per_seq,
                                   int64_t num_pages, int64_t num_splits, float scale,
                                   int64_t window, void* stream);

/*
 * The same with q, k_cache, v_cache and out in bf16 (window == 0: plain paged
 * decode).  The fp32 split-K scratch has the same layout.  For the bf16 KV cache
 * of a bf16 model (the llama of tests/dynamo/llama_test.py runs in the dtype of
 * its weights); mi355_kv_cache_append moves 16-bit elements and serves both.
 */
int mi355_paged_decode_attn_window_bf16(const void* q, const void* k_cache, const void* v_cache,
                                        const int32_t* block_table, const int32_t* seq_lens, void* out,
                                        float* part_acc, float* part_ml,
                                        int64_t num_seqs, int64_t num_q_heads, int64_t num_kv_heads,
                                        int64_t D, int64_t page_size, int64_t max_pages_per_seq,
                                        int64_t num_pages, int64_t num_splits, float scale,
                                        int64_t window, void* stream);

/*
 * KV-cache append, the step in front of decode: the paged form of
 *   cache_k[:bsz, start_pos : start_pos + seqlen] = xk   (tests/dynamo/llama_test.py:165-166)
 * with a start position per sequence.
 * k_new, v_new: [num_seqs, n_new, num_kv_heads, D] fp16 or bf16 (16-bit elements are moved as they are); token t of sequence s is
 * written at position start_pos[s] + t, i.e. page block_table[s][pos / page_size],
 * slot pos % page_size of k_cache / v_cache ([num_pages, page_size, num_kv_heads, D]).
 * Positions without a table entry (pos / page_size >= max_pages_per_seq) or whose
 * entry is outside [0, num_pages) are skipped.  D == 128, page_size 16, 32, 64, 128 or 256.
 */
int mi355_kv_cache_append(const void* k_new, const void* v_new, void* k_cache, void* v_cache,
                          const int32_t* block_table, const int32_t* start_pos,
                          int64_t num_seqs, int64_t n_new, int64_t num_kv_heads, int64_t D,
                          int64_t page_size, int64_t max_pages_per_seq, int64_t num_pages,
                          void* stream);

/*
 * Prefill over a paged KV cache (chunked / prefix prefill, the step between append and decode):
 * the num_new latest tokens of every sequence attend to that sequence's cached keys and values,
 * causally -- query t (0-based among the new tokens) of sequence s sees cache positions
 * j <= seq_lens[s] - num_new + t, the mask of tests/dynamo/llama_test.py:285-290 shifted by the
 * cached prefix.  The new tokens' own K/V are expected in the cache already
 * (mi355_kv_cache_append), so seq_lens counts them.
 * q, out:      [num_seqs, num_new, num_q_heads, D]        fp16
 * k_cache,
 * v_cache:     [num_pages, page_size, num_kv_heads, D]    fp16
 * block_table: [num_seqs, max_pages_per_seq] int32; entries at or beyond
 *              ceil(seq_len/page_size) are never read, ids outside [0, num_pages) read as zeros
 * seq_lens:    [num_seqs] int32 (clamped to [0, max_pages_per_seq * page_size]); queries with
 *              no visible key produce zeros
 * D == 128, page_size 16, 32, 64, 128 or 256, num_q_heads % num_kv_heads == 0.  Same kernel as
 * mi355_flash_attn_fwd (fp32 online softmax, fp16 output), K/V tiles fetched page by page.
 * Replaces: the prefill call of the attention in tests/dynamo/llama_test.py:144-182 when the
 * cache is paged (no surviving paged counterpart in the reference).
 */
int mi355_paged_prefill_attn(const void* q, const void* k_cache, const void* v_cache,
                             const void* block_table, const void* seq_lens, void* out,
                             int64_t num_seqs, int64_t num_new, int64_t num_q_heads,
                             int64_t num_kv_heads, int64_t D, int64_t page_size,
                             int64_t max_pages_per_seq, int64_t num_pages, float scale, void* stream);

/* The same with q, k_cache, v_cache and out in bf16. */
int mi355_paged_prefill_attn_bf16(const void* q, const void* k_cache, const void* v_cache,
                                  const void* block_table, const void* seq_lens, void* out,
                                  int64_t num_seqs, int64_t num_new, int64_t num_q_heads,
                                  int64_t num_kv_heads, int64_t D, int64_t page_size,
                                  int64_t max_pages_per_seq, int64_t num_pages, float scale, void* stream);

/*
 * Block-scaled MXFP4 GEMM: C[M,N] = dq(A) . dq(B)^T, fp32 accumulation, bf16 out.
 * a: uint8 [M, K/2], b: uint8 [N, K/2]  -- two E2M1 codes per byte, element 2i
 *    in the low nibble, element 2i+1 in the high nibble;
 * a_scale: uint8 [M, K/32], b_scale: uint8 [N, K/32] -- E8M0 (value 2^(byte-127)),
 *    one per 32 consecutive K elements.
 * dq(x)[r,k] = E2M1(code[r,k]) * 2^(scale[r,k/32] - 127).  K % 32 == 0.
 * Format names: iree/turbine/kernel/_support/dtype.py:117,119 (f8e8m0fnu,
 * f4e2m1fn); scale symbols iree/turbine/kernel/lang/global_symbols.py:33-35.
 */
int mi355_mxfp4_gemm(const void* a, const void* a_scale, const void* b, const void* b_scale,
                     void* c, int64_t M, int64_t N, int64_t K,
                     int out_dtype, int variant, void* stream);

/*
 * Block-scaled MXFP8 GEMM: C[M,N] = dq(A) . dq(B)^T, fp32 accumulation, bf16 or fp32 out.
 * a: uint8 [M, K], b: uint8 [N, K] -- OCP FP8 E4M3 codes (sign, 4 exponent bits of bias 7,
 *    3 mantissa bits, no infinities, NaN = S.1111.111), one per element;
 * a_scale: uint8 [M, K/32], b_scale: uint8 [N, K/32] -- E8M0, one per 32 consecutive K elements.
 * dq(x)[r,k] = E4M3(code[r,k]) * 2^(scale[r,k/32] - 127).  K % 32 == 0.
 * The wider element format at the boundary of mi355_mxfp4_gemm: same scales, same layout, one byte per
 * element.  Format names: iree/turbine/kernel/_support/dtype.py:115,117 (f8e4m3fn, f8e8m0fnu).
 */
int mi355_mxfp8_gemm(const void* a, const void* a_scale, const void* b, const void* b_scale,
                     void* c, int64_t M, int64_t N, int64_t K,
                     int out_dtype, int variant, void* stream);

/*
 * Block-scaled MXFP6 GEMM: C[M,N] = dq(A) . dq(B)^T, fp32 accumulation, bf16 or fp32 out.
 * a: uint8 [M, K*3/4], b: uint8 [N, K*3/4] -- OCP 6-bit codes packed as a little-endian bit stream per row:
 *    element k occupies bits [6k, 6k+6) of the row, a scale block of 32 elements is 24 bytes.
 *    element_format MI355_FP6_E2M3: sign, 2 exponent bits (bias 1), 3 mantissa bits, values up to 7.5
 *    (the reference's f6E2M3FN, iree/turbine/kernel/_support/dtype.py:118);
 *    MI355_FP6_E3M2: sign, 3 exponent bits (bias 3), 2 mantissa bits, values up to 28.  No NaN or infinity codes.
 * a_scale: uint8 [M, K/32], b_scale: uint8 [N, K/32] -- E8M0, one per 32 consecutive K elements.
 * dq(x)[r,k] = FP6(code[r,k]) * 2^(scale[r,k/32] - 127).  K % 32 == 0.
 */
#define MI355_FP6_E2M3 0
#define MI355_FP6_E3M2 1
int mi355_mxfp6_gemm(const void* a, const void* a_scale, const void* b, const void* b_scale,
                     void* c, int64_t M, int64_t N, int64_t K, int element_format,
                     int out_dtype, int variant, void* stream);

/*
 * MXFP6 quantisation, the producer of mi355_mxfp6_gemm's operands: x [rows, K] in fp16 / bf16 / fp32 ->
 * codes uint8 [rows, K*3/4] (8-byte aligned, the bit-stream layout above) and scales uint8 [rows, K/32].
 * Per block of 32: scale exponent floor(log2(max|x|)) - emax (emax 2 for E2M3, 4 for E3M2) clamped to
 * [-127, 127] (all-zero block: -127; a NaN or infinity in the block: scale 0xFF and signed-zero codes),
 * elements rounded to the nearest value, ties to the even code, saturating at the largest value (7.5 / 28)
 * (OCP Microscaling Formats v1.0).  K % 32 == 0.
 */
int mi355_mxfp6_quantize(const void* x, int in_dtype, int64_t rows, int64_t K, int element_format,
                         void* codes, void* scales, void* stream);

/*
 * Plain fp8 GEMM (no block scales): C[M,N] = alpha . A . B^T with A [M, K], B [N, K] OCP FP8 E4M3 codes,
 * fp32 accumulation, bf16 or fp32 out; alpha carries the product of the per-tensor scales a caller
 * quantised with.  The kernels of mi355_mxfp8_gemm with every block scale fixed at 2^0.  K % 32 == 0.
 * Replaces: GEMMForward (iree/turbine/kernel/boo/op_exports/gemm.py:217-230) for fp8 operands
 * (dtype iree/turbine/kernel/_support/dtype.py:115, f8e4m3fn).
 */
int mi355_fp8_gemm(const void* a, const void* b, void* c, int64_t M, int64_t N, int64_t K,
                   float alpha, int out_dtype, int variant, void* stream);

/*
 * MXFP4 dequantisation on the device (used to show that the device decodes
 * the format bit-exactly): out[r,k] = E2M1(code) * 2^(scale-127) as fp32.
 * codes: uint8 [rows, K/2]; scales: uint8 [rows, K/32]; out: fp32 [rows, K].
 */
int mi355_mxfp4_dequant(const void* codes, const void* scales, float* out,
                        int64_t rows, int64_t K, void* stream);

/*
 * MXFP4 quantisation, the producer of mi355_mxfp4_gemm's operands: x [rows, K] in
 * fp16 / bf16 / fp32 (in_dtype MI355_F16 / MI355_BF16 / MI355_F32) ->
 * codes uint8 [rows, K/2] and scales uint8 [rows, K/32] in the layout above.
 * Per block of 32: scale exponent floor(log2(max|x|)) - 2 clamped to [-127, 127]
 * (all-zero block: -127; a NaN or infinity in the block: scale 0xFF), elements
 * rounded to the nearest E2M1 value, ties to the even code, saturating at 6
 * (OCP Microscaling Formats v1.0).  K % 32 == 0.  The reference has no producer
 * for these dtypes; it only declares them (iree/turbine/kernel/_support/dtype.py:117,119).
 */
int mi355_mxfp4_quantize(const void* x, int in_dtype, int64_t rows, int64_t K,
                         void* codes, void* scales, void* stream);

/*
 * MXFP8 quantisation, the producer of mi355_mxfp8_gemm's operands: x [rows, K] in
 * fp16 / bf16 / fp32 -> codes uint8 [rows, K] (OCP E4M3, 8-byte aligned) and
 * scales uint8 [rows, K/32].  Per block of 32: scale exponent
 * floor(log2(max|x|)) - 8 clamped to [-127, 127] (all-zero block: -127; a NaN or
 * infinity in the block: scale 0xFF and signed-zero codes), elements rounded to
 * the nearest E4M3 value, ties to the even code, saturating at 448 (OCP
 * Microscaling Formats v1.0).  K % 32 == 0.  As for MXFP4 the reference only
 * declares the element dtype (iree/turbine/kernel/_support/dtype.py:115,117).
 */
int mi355_mxfp8_quantize(const void* x, int in_dtype, int64_t rows, int64_t K,
                         void* codes, void* scales, void* stream);

/*
 * Calibration, not part of the path: a register-only MFMA loop (no LDS, no memory traffic inside the
 * loop) on caller-supplied operand bytes, to measure what the MFMA unit of the board sustains on a
 * given data distribution -- the ceiling that the roofline fractions of the GEMM and attention
 * kernels can be read against beside the datasheet peak.  No counterpart in the reference; it plays
 * the part of the plain-copy workload for the HBM figures.
 * kind 0: v_mfma_f32_32x32x16_f16; 1: v_mfma_scale_f32_32x32x64_f8f6f4 with fp4 operands and unit
 * scales; 2: the same with E8M0 scales spread over 2^-8 .. 2^7; 3: v_mfma_f32_16x16x32_f16 (two per
 * 32x32x16's worth of flop); 4 / 5: loops with a GEMM's register structure (256 accumulators per lane,
 * eight A and eight B operands rotated, every product subtracted again eight trips later) on
 * 32x32x16 / 16x16x32 fp16 MFMAs, trips rounded down to a multiple of 16; 6 / 7: the same structure on
 * scaled fp4 MFMAs 32x32x64 / 16x16x128.  operands: operand_bytes (a power of
 * two >= 16) of device memory read once before the loop; sink: >= workgroups * 256 floats, written
 * once after it; *flop_per_launch (optional, host memory) receives the flop count of the launch.
 */
int mi355_calibrate_mfma(int kind, const void* operands, int64_t operand_bytes, float* sink,
                         int64_t sink_floats, int64_t workgroups, int64_t trips,
                         double* flop_per_launch, void* stream);

/*
 * Calibration, not part of the path and without a counterpart in the reference: the instruction mix of one
 * 64-key tile of the prefill kernel per wave of 32 queries (32 MFMAs 32x32x16, 32 v_exp_f32, 16 packed
 * conversions, 16 dot2, the v_max3 chain and its wave-wide test), out of registers only -- no LDS reads,
 * loads or barriers.  What it sustains is the ceiling that instruction issue sets for the prefill kernel.
 * mode 0: the whole mix; 1: without the maximum chain; 2: the MFMAs alone, same dependences; 3: the vector
 * work alone.  256 workgroups (of 256 threads) put one wave on every SIMD, 512 two.  operands, sink and
 * flop_per_launch as for mi355_calibrate_mfma; the flop count is that of the tile's 32 MFMAs.
 */
int mi355_calibrate_fa_issue(int mode, const void* operands, int64_t operand_bytes, float* sink,
                             int64_t sink_floats, int64_t workgroups, int64_t trips,
                             double* flop_per_launch, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* TURBINE_MI355_H_ */
