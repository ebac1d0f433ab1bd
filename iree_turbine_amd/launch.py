"""Out-variant launchers: checked tensors in, C-ABI call on torch's current stream, output tensors
written in place.  Both the custom ops (ops.py) and the template kernels (templates/) go through
these functions; they are the only callers of the C ABI, and each one runs the kernel's shape / dtype
contract (contract.py) on its tensors before it takes a single device pointer."""

from __future__ import annotations

import ctypes
import math

import torch
from torch import Tensor

from . import _lib, contract


def _dev(*tensors: Tensor) -> torch.device:
    dev = tensors[0].device
    for t in tensors[1:]:
        if t.device != dev:
            # same rule and wording as Launchable.__call__, iree/turbine/runtime/launch.py:220-225
            raise RuntimeError(f"Cannot launch with tensors from multiple devices: {t.device} vs {dev}")
    if dev.type != "cuda":
        raise RuntimeError(f"the kernels run on an MI355X only; got tensors on {dev} (there is no CPU fallback)")
    return dev


def _half_dtype(name: str, *tensors: Tensor) -> torch.dtype:
    """The one 16-bit float format (fp16 or bf16) that all of `tensors` share; the kernels exist for both."""
    dt = tensors[0].dtype
    if dt not in (torch.float16, torch.bfloat16) or any(t.dtype != dt for t in tensors):
        raise ValueError(f"{name}: tensors must all be float16 or all bfloat16, got {[str(t.dtype) for t in tensors]}")
    return dt


def _contig_out(t: Tensor, name: str) -> None:
    if not t.is_contiguous():
        raise ValueError(f"{name}: output tensors must be contiguous")  # runtime/launch.py:246


_PAD_MIN_FLOPS = 0.0  # the tiled kernels on padded copies beat the bounds-checked kernel at every size measured (from 2e7 flop)


def _one_round_of_rows(M: int, N: int, K: int) -> bool:
    """A product of any M rows against N % 8 == 0, K % 64 == 0 that the library's tiled or weight-streaming kernels
    take whole (the library's rule of the same name)."""
    up = lambda x, t: -(-x // t)
    if up(M, 64) * 64 * up(N, 64) * 64 <= (1 << 21) or up(M, 128) * up(N, 128) <= 256:
        return True
    if 256 <= K < 8192 and up(M, 256) * up(N, 128) <= 256:
        return True
    return M <= 128 and N % 32 == 0 and N >= 2048 and K >= 512


def _ragged_rows_fit(M: int, N: int, K: int) -> bool:
    """Shapes whose ragged M (and N, in multiples of 8) the library handles itself: a cut last tile row or column where
    one round of tiles covers the product, two products on row ranges beyond that (N a multiple of 128 then)."""
    if N % 8 or K % 64:
        return False
    if _one_round_of_rows(M, N, K):
        return True
    return N % 128 == 0 and M >= 512 and M % 256 != 0 and _one_round_of_rows(M % 256, N, K)


def _skinny_fits(M: int, N: int, K: int) -> bool:
    """The shapes the library's weight-streaming kernel takes by itself (decode-shaped products: few rows of A
    against a large B); padding A to a tile would multiply their work by 128 / M."""
    return M <= 64 and N % 32 == 0 and K % 64 == 0 and N >= 2048 and K >= 512


def gemm_nt_out(a: Tensor, b: Tensor, c: Tensor, variant: int = -1) -> Tensor:
    contract.check_gemm_operands("gemm_nt", a, b)
    dev = _dev(a, b, c)
    a, b = a.contiguous(), b.contiguous()
    _contig_out(c, "gemm_nt")
    M, K = a.shape
    N = b.shape[0]
    if tuple(c.shape) != (M, N):
        raise ValueError(f"gemm_nt: c is {tuple(c.shape)}, expected {(M, N)}")
    if c.dtype not in (torch.float32, a.dtype):
        raise ValueError(f"gemm_nt: c must be float32 or {a.dtype}, got {c.dtype}")
    lib = _lib.load()
    entry = lib.mi355_gemm_bf16_nt if a.dtype == torch.bfloat16 else lib.mi355_gemm_f16_nt
    a_k, b_k, c_k = a, b, c
    if variant < 0 and 2.0 * M * N * K >= _PAD_MIN_FLOPS and (M % 128 or N % 128 or K % 64) and not _skinny_fits(M, N, K) \
            and not _ragged_rows_fit(M, N, K):
        # Ragged sizes would go to the bounds-checked 64x64 kernel (about a fifth of the tiled kernels' rate).  Zero
        # padding changes no sum, so the ragged operands are copied into tile-aligned buffers and the result cut
        # out again: three extra passes over memory against a 4-5x faster product (3000x5000x4104: 508 -> 190 us).
        tile = 256 if ((M + 255) // 256) * ((N + 255) // 256) >= 128 else 128
        Mp, Np, Kp = -(-M // tile) * tile, -(-N // tile) * tile, -(-K // 64) * 64
        if (Mp, Kp) != (M, K):
            a_k = torch.zeros((Mp, Kp), dtype=a.dtype, device=dev)
            a_k[:M, :K] = a
        if (Np, Kp) != (N, K):
            b_k = torch.zeros((Np, Kp), dtype=b.dtype, device=dev)
            b_k[:N, :K] = b
        if (Mp, Np) != (M, N):
            c_k = torch.empty((Mp, Np), dtype=c.dtype, device=dev)
    # A shape with too few 256x256 tiles for the chip (or with a sparse last round of them) splits K when it gets a
    # workspace for the fp32 partial products; the library says how large.  torch's caching allocator makes the
    # allocation cheap and safe under graph capture.
    ws_bytes = lib.mi355_gemm_nt_workspace_bytes(c_k.shape[0], c_k.shape[1], a_k.shape[1]) if variant < 0 else 0
    with torch.cuda.device(dev):
        if ws_bytes > 0:
            ws = torch.empty(ws_bytes // 4, dtype=torch.float32, device=dev)
            entry_ws = lib.mi355_gemm_bf16_nt_ws if a.dtype == torch.bfloat16 else lib.mi355_gemm_f16_nt_ws
            rc = entry_ws(a_k.data_ptr(), b_k.data_ptr(), c_k.data_ptr(), c_k.shape[0], c_k.shape[1], a_k.shape[1],
                          _lib.dtype_code(c.dtype), variant, ws.data_ptr(), ws_bytes, _lib.current_stream_ptr(dev))
        else:
            rc = entry(a_k.data_ptr(), b_k.data_ptr(), c_k.data_ptr(), c_k.shape[0], c_k.shape[1], a_k.shape[1],
                       _lib.dtype_code(c.dtype), variant, _lib.current_stream_ptr(dev))
    _lib.check(rc, f"gemm_nt M={M} N={N} K={K} in={a.dtype} out={c.dtype} variant={variant}")
    if c_k is not c:
        c.copy_(c_k[:M, :N])
    return c


def _fa_strides(t: Tensor):
    """{batch, head, row} element strides if the kernel can read `t` in place, else None."""
    sb, sh, sr, sd = t.stride()
    if t.size(3) != 1 and sd != 1:
        return None
    if t.size(0) == 1:
        sb = 0
    if t.size(1) == 1:
        sh = 0
    if t.size(2) == 1:
        sr = 128
    if min(sb, sh) < 0 or sr < 128 or sr >= 2**24 or (sb | sh | sr) & 7 or t.data_ptr() & 15:
        return None
    return (sb, sh, sr)


def flash_attn_fwd_out(q: Tensor, k: Tensor, v: Tensor, o: Tensor, is_causal: bool, scale: float, variant: int = -1) -> Tensor:
    """q, o: [B, H, Sq, 128]; k, v: [B, Hkv, Sk, 128] with H % Hkv == 0.  Operands whose rows are contiguous and
    16-byte aligned (any batch / head / row strides, e.g. transposed [B, S, H, D] views) are read in place; others
    are copied first.  `o` must be such a tensor."""
    contract.check_attention_operands("flash_attn_fwd", q, k, v)
    dev = _dev(q, k, v, o)
    B, H, Sq, D = q.shape
    Hkv, Sk = k.shape[1], k.shape[2]
    dt = _half_dtype("flash_attn_fwd", q, k, v, o)
    if o.shape != q.shape:
        raise ValueError("flash_attn_fwd: o must have q's shape")
    if scale is None or scale <= 0:
        scale = 1.0 / math.sqrt(D)
    ins = []
    for t in (q, k, v):
        st = _fa_strides(t)
        if st is None:
            t = t.contiguous()
            st = _fa_strides(t)
        ins.append((t, st))
    o_st = _fa_strides(o)
    if o_st is None or (B > 1 and o_st[0] == 0) or (H > 1 and o_st[1] == 0):
        raise ValueError("flash_attn_fwd: output rows must be contiguous, 16-byte aligned and not overlapping")  # runtime/launch.py:246
    arr = lambda st: (ctypes.c_int64 * 3)(*st)
    lib = _lib.load()
    entry = lib.mi355_flash_attn_fwd_strided_bf16 if dt == torch.bfloat16 else lib.mi355_flash_attn_fwd_strided
    with torch.cuda.device(dev):
        rc = entry(ins[0][0].data_ptr(), ins[1][0].data_ptr(), ins[2][0].data_ptr(), o.data_ptr(), B, H, Hkv, Sq, Sk, D,
                   arr(ins[0][1]), arr(ins[1][1]), arr(ins[2][1]), arr(o_st), scale, int(bool(is_causal)), variant,
                   _lib.current_stream_ptr(dev))
    _lib.check(rc, f"flash_attn_fwd {dt} B={B} H={H} Hkv={Hkv} Sq={Sq} Sk={Sk} D={D} causal={is_causal}")
    return o


def paged_decode_phase0_out(q, k_cache, v_cache, block_table, seq_lens, part_acc, part_ml, scale: float) -> None:
    contract.check_paged_args("paged_decode_phase0", q, k_cache, v_cache, block_table, seq_lens, bf16_ok=True)
    ns = contract.check_decode_partials("paged_decode_phase0", part_acc, part_ml, q.shape[0], q.shape[1])
    dev = _dev(q, k_cache, v_cache, block_table, seq_lens, part_acc, part_ml)
    q, k_cache, v_cache = q.contiguous(), k_cache.contiguous(), v_cache.contiguous()
    block_table, seq_lens = block_table.contiguous(), seq_lens.contiguous()
    _contig_out(part_acc, "paged_decode_phase0")
    _contig_out(part_ml, "paged_decode_phase0")
    dt = _half_dtype("paged_decode_phase0", q, k_cache, v_cache)
    S, Hq, D = q.shape
    P, page, Hkv, _ = k_cache.shape
    if scale is None or scale <= 0:
        scale = 1.0 / math.sqrt(D)
    lib = _lib.load()
    entry = lib.mi355_paged_decode_phase0_bf16 if dt == torch.bfloat16 else lib.mi355_paged_decode_phase0
    with torch.cuda.device(dev):
        rc = entry(q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), block_table.data_ptr(), seq_lens.data_ptr(),
                   part_acc.data_ptr(), part_ml.data_ptr(), S, Hq, Hkv, D, page, block_table.shape[1], P, ns, scale,
                   _lib.current_stream_ptr(dev))
    _lib.check(rc, f"paged_decode_phase0 seqs={S} hq={Hq} hkv={Hkv} splits={ns}")


def paged_decode_phase1_out(part_acc: Tensor, part_ml: Tensor, out: Tensor) -> Tensor:
    contract.require(part_acc.dim() == 4, "paged_decode_phase1: part_acc must be fp32 [S, Hq, splits, 128]")
    contract.check_decode_partials("paged_decode_phase1", part_acc, part_ml, part_acc.shape[0], part_acc.shape[1])
    dev = _dev(part_acc, part_ml, out)
    part_acc, part_ml = part_acc.contiguous(), part_ml.contiguous()
    _contig_out(out, "paged_decode_phase1")
    S, Hq, ns, D = part_acc.shape
    if tuple(out.shape) != (S, Hq, D) or out.dtype not in (torch.float16, torch.bfloat16):
        raise ValueError("paged_decode_phase1: out must be float16 or bfloat16 [S, Hq, D]")
    lib = _lib.load()
    entry = lib.mi355_paged_decode_phase1_bf16 if out.dtype == torch.bfloat16 else lib.mi355_paged_decode_phase1
    with torch.cuda.device(dev):
        rc = entry(part_acc.data_ptr(), part_ml.data_ptr(), out.data_ptr(), S, Hq, D, ns, _lib.current_stream_ptr(dev))
    _lib.check(rc, f"paged_decode_phase1 seqs={S} hq={Hq} splits={ns}")
    return out


_ARRIVALS: dict[tuple[int, int], Tensor] = {}  # (device index, stream) -> int32 arrival counters, grown on demand


def _arrival_counters(dev: torch.device, n: int) -> Tensor | None:
    """The per-(sequence, kv head) arrival counters of the one-launch decode: one buffer per stream (launches on one
    stream are ordered; two streams never share a buffer), zeroed when it is created.  Under stream capture a fill
    would be recorded instead of run, so a stream that meets its first call (or a larger batch than any before) while
    it is being captured gets no counters: that call takes the two-launch form, which needs none."""
    key = (dev.index if dev.index is not None else torch.cuda.current_device(), torch.cuda.current_stream(dev).cuda_stream)
    buf = _ARRIVALS.get(key)
    if buf is None or buf.numel() < n:
        if torch.cuda.is_current_stream_capturing():
            return None
        buf = torch.zeros(max(n, 4096), dtype=torch.int32, device=dev)
        _ARRIVALS[key] = buf
    return buf


def paged_decode_attn_out(q, k_cache, v_cache, block_table, seq_lens, out, scale: float, num_kv_splits: int,
                          part_acc: Tensor | None = None, part_ml: Tensor | None = None, window: int = 0) -> Tensor:
    contract.check_paged_args("paged_decode_attn", q, k_cache, v_cache, block_table, seq_lens, bf16_ok=True)
    contract.require(1 <= num_kv_splits <= 1024, f"paged_decode_attn: num_kv_splits must be in [1, 1024], got {num_kv_splits}")
    contract.require(window >= 0, f"paged_decode_attn: window must be >= 0, got {window}")
    if num_kv_splits > 1 and part_acc is not None and part_ml is not None:  # caller-owned scratch
        contract.check_decode_partials("paged_decode_attn", part_acc, part_ml, q.shape[0], q.shape[1], num_kv_splits)
    dev = _dev(q, k_cache, v_cache, block_table, seq_lens, out)
    q, k_cache, v_cache = q.contiguous(), k_cache.contiguous(), v_cache.contiguous()
    block_table, seq_lens = block_table.contiguous(), seq_lens.contiguous()
    _contig_out(out, "paged_decode_attn")
    S, Hq, D = q.shape
    P, page, Hkv, _ = k_cache.shape
    dt = _half_dtype("paged_decode_attn", q, k_cache, v_cache, out)
    if out.shape != q.shape:
        raise ValueError("paged_decode_attn: out must have q's shape")
    if scale is None or scale <= 0:
        scale = 1.0 / math.sqrt(D)
    if num_kv_splits > 1:
        if part_acc is None:
            part_acc = torch.empty((S, Hq, num_kv_splits, D), dtype=torch.float32, device=dev)
        if part_ml is None:
            part_ml = torch.empty((S, Hq, num_kv_splits, 2), dtype=torch.float32, device=dev)
        _dev(q, part_acc, part_ml)
        contract.check_decode_partials("paged_decode_attn", part_acc, part_ml, S, Hq, num_kv_splits)
        _contig_out(part_acc, "paged_decode_attn")
        _contig_out(part_ml, "paged_decode_attn")
    pa = part_acc.data_ptr() if num_kv_splits > 1 else None
    pm = part_ml.data_ptr() if num_kv_splits > 1 else None
    counters = _arrival_counters(dev, S * Hkv) if num_kv_splits > 1 else None
    arrivals = counters.data_ptr() if counters is not None else None
    with torch.cuda.device(dev):
        rc = _lib.load().mi355_paged_decode_attn_fused(q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), block_table.data_ptr(),
                                                       seq_lens.data_ptr(), out.data_ptr(), pa, pm, arrivals, S, Hq, Hkv, D, page,
                                                       block_table.shape[1], P, num_kv_splits, scale, window, _lib.dtype_code(dt),
                                                       _lib.current_stream_ptr(dev))
    _lib.check(rc, f"paged_decode_attn {dt} seqs={S} hq={Hq} hkv={Hkv} pages={P} splits={num_kv_splits} window={window}")
    return out


def kv_cache_append(k_new, v_new, k_cache, v_cache, block_table, start_pos) -> None:
    """Writes k_new / v_new [S, n_new, Hkv, 128] into the paged caches in place (see mi355_kv_cache_append)."""
    contract.check_kv_append("kv_cache_append", k_new, v_new, k_cache, v_cache, block_table, start_pos)
    dev = _dev(k_new, v_new, k_cache, v_cache, block_table, start_pos)
    k_new, v_new = k_new.contiguous(), v_new.contiguous()
    block_table, start_pos = block_table.contiguous(), start_pos.contiguous()
    _contig_out(k_cache, "kv_cache_append")
    _contig_out(v_cache, "kv_cache_append")
    _half_dtype("kv_cache_append", k_new, v_new, k_cache, v_cache)  # 16-bit elements are moved as they are
    S, n_new, Hkv, D = k_new.shape
    P, page = k_cache.shape[0], k_cache.shape[1]
    with torch.cuda.device(dev):
        rc = _lib.load().mi355_kv_cache_append(k_new.data_ptr(), v_new.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                                               block_table.data_ptr(), start_pos.data_ptr(), S, n_new, Hkv, D, page,
                                               block_table.shape[1], P, _lib.current_stream_ptr(dev))
    _lib.check(rc, f"kv_cache_append seqs={S} n_new={n_new} hkv={Hkv} pages={P}")


def paged_prefill_attn_out(q: Tensor, k_cache: Tensor, v_cache: Tensor, block_table: Tensor, seq_lens: Tensor, out: Tensor,
                           scale: float) -> Tensor:
    """q, out [S, n_new, Hq, 128]; caches [P, page, Hkv, 128]; seq_lens counts the new tokens (see mi355_paged_prefill_attn)."""
    contract.check_paged_prefill("paged_prefill_attn", q, k_cache, v_cache, block_table, seq_lens)
    dev = _dev(q, k_cache, v_cache, block_table, seq_lens, out)
    q, k_cache, v_cache = q.contiguous(), k_cache.contiguous(), v_cache.contiguous()
    block_table, seq_lens = block_table.contiguous(), seq_lens.contiguous()
    _contig_out(out, "paged_prefill_attn")
    S, n_new, Hq, D = q.shape
    P, page, Hkv = k_cache.shape[0], k_cache.shape[1], k_cache.shape[2]
    dt = _half_dtype("paged_prefill_attn", q, k_cache, v_cache, out)
    if out.shape != q.shape:
        raise ValueError("paged_prefill_attn: out must have q's shape")
    if scale is None or scale <= 0:
        scale = 1.0 / math.sqrt(D)
    lib = _lib.load()
    entry = lib.mi355_paged_prefill_attn_bf16 if dt == torch.bfloat16 else lib.mi355_paged_prefill_attn
    with torch.cuda.device(dev):
        rc = entry(q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), block_table.data_ptr(), seq_lens.data_ptr(),
                   out.data_ptr(), S, n_new, Hq, Hkv, D, page, block_table.shape[1], P, scale, _lib.current_stream_ptr(dev))
    _lib.check(rc, f"paged_prefill_attn seqs={S} n_new={n_new} hq={Hq} hkv={Hkv} pages={P}")
    return out


def _check_mx_out(op: str, c: Tensor) -> None:
    if c.dtype not in (torch.bfloat16, torch.float32):
        raise ValueError(f"{op}: c must be bfloat16 or float32, got {c.dtype}")


def mxfp4_gemm_out(a, a_scale, b, b_scale, c: Tensor, variant: int = -1) -> Tensor:
    contract.check_mx_pair("mxfp4_gemm", a, a_scale, b, b_scale, per_byte=2)
    _check_mx_out("mxfp4_gemm", c)
    dev = _dev(a, a_scale, b, b_scale, c)
    a, a_scale, b, b_scale = a.contiguous(), a_scale.contiguous(), b.contiguous(), b_scale.contiguous()
    _contig_out(c, "mxfp4_gemm")
    M, N, K = a.shape[0], b.shape[0], a.shape[1] * 2
    if tuple(c.shape) != (M, N):
        raise ValueError(f"mxfp4_gemm: c is {tuple(c.shape)}, expected {(M, N)}")
    with torch.cuda.device(dev):
        rc = _lib.load().mi355_mxfp4_gemm(a.data_ptr(), a_scale.data_ptr(), b.data_ptr(), b_scale.data_ptr(), c.data_ptr(), M, N,
                                          K, _lib.dtype_code(c.dtype), variant, _lib.current_stream_ptr(dev))
    _lib.check(rc, f"mxfp4_gemm M={M} N={N} K={K} out={c.dtype} variant={variant}")
    return c


def mxfp8_gemm_out(a, a_scale, b, b_scale, c: Tensor, variant: int = -1) -> Tensor:
    contract.check_mx_pair("mxfp8_gemm", a, a_scale, b, b_scale, per_byte=1)
    _check_mx_out("mxfp8_gemm", c)
    dev = _dev(a, a_scale, b, b_scale, c)
    a, a_scale, b, b_scale = a.contiguous(), a_scale.contiguous(), b.contiguous(), b_scale.contiguous()
    _contig_out(c, "mxfp8_gemm")
    M, N, K = a.shape[0], b.shape[0], a.shape[1]
    if tuple(c.shape) != (M, N):
        raise ValueError(f"mxfp8_gemm: c is {tuple(c.shape)}, expected {(M, N)}")
    with torch.cuda.device(dev):
        rc = _lib.load().mi355_mxfp8_gemm(a.data_ptr(), a_scale.data_ptr(), b.data_ptr(), b_scale.data_ptr(), c.data_ptr(), M, N,
                                          K, _lib.dtype_code(c.dtype), variant, _lib.current_stream_ptr(dev))
    _lib.check(rc, f"mxfp8_gemm M={M} N={N} K={K} out={c.dtype} variant={variant}")
    return c


FP6_FORMATS = {"e2m3": 0, "e3m2": 1}  # MI355_FP6_E2M3, MI355_FP6_E3M2


def mxfp6_gemm_out(a, a_scale, b, b_scale, c: Tensor, element_format: str = "e2m3", variant: int = -1) -> Tensor:
    dev = _dev(a, a_scale, b, b_scale, c)
    if element_format not in FP6_FORMATS:
        raise ValueError(f"mxfp6_gemm: element_format must be one of {sorted(FP6_FORMATS)}, got {element_format!r}")
    contract.check_mxfp6_pair("mxfp6_gemm", a, a_scale, b, b_scale)
    _check_mx_out("mxfp6_gemm", c)
    a, a_scale, b, b_scale = a.contiguous(), a_scale.contiguous(), b.contiguous(), b_scale.contiguous()
    _contig_out(c, "mxfp6_gemm")
    M, N, K = a.shape[0], b.shape[0], a_scale.shape[1] * 32
    if tuple(c.shape) != (M, N):
        raise ValueError(f"mxfp6_gemm: c is {tuple(c.shape)}, expected {(M, N)}")
    with torch.cuda.device(dev):
        rc = _lib.load().mi355_mxfp6_gemm(a.data_ptr(), a_scale.data_ptr(), b.data_ptr(), b_scale.data_ptr(), c.data_ptr(), M, N,
                                          K, FP6_FORMATS[element_format], _lib.dtype_code(c.dtype), variant,
                                          _lib.current_stream_ptr(dev))
    _lib.check(rc, f"mxfp6_gemm M={M} N={N} K={K} format={element_format} out={c.dtype} variant={variant}")
    return c


def fp8_gemm_out(a, b, c: Tensor, alpha: float = 1.0, variant: int = -1) -> Tensor:
    contract.check_fp8_operands("fp8_gemm", a, b)
    _check_mx_out("fp8_gemm", c)
    dev = _dev(a, b, c)
    a, b = a.contiguous(), b.contiguous()
    _contig_out(c, "fp8_gemm")
    M, N, K = a.shape[0], b.shape[0], a.shape[1]
    if tuple(c.shape) != (M, N):
        raise ValueError(f"fp8_gemm: c is {tuple(c.shape)}, expected {(M, N)}")
    with torch.cuda.device(dev):
        rc = _lib.load().mi355_fp8_gemm(a.data_ptr(), b.data_ptr(), c.data_ptr(), M, N, K, float(alpha), _lib.dtype_code(c.dtype),
                                        variant, _lib.current_stream_ptr(dev))
    _lib.check(rc, f"fp8_gemm M={M} N={N} K={K} out={c.dtype} variant={variant}")
    return c


def mxfp4_dequant_out(codes: Tensor, scales: Tensor, out: Tensor) -> Tensor:
    contract.check_mx_operand("mxfp4_dequant", "codes", codes, scales)
    dev = _dev(codes, scales, out)
    codes, scales = codes.contiguous(), scales.contiguous()
    _contig_out(out, "mxfp4_dequant")
    rows, K = codes.shape[0], codes.shape[1] * 2
    if tuple(out.shape) != (rows, K) or out.dtype != torch.float32:
        raise ValueError("mxfp4_dequant: out must be float32 [rows, K]")
    with torch.cuda.device(dev):
        rc = _lib.load().mi355_mxfp4_dequant(codes.data_ptr(), scales.data_ptr(), out.data_ptr(), rows, K,
                                             _lib.current_stream_ptr(dev))
    _lib.check(rc, f"mxfp4_dequant rows={rows} K={K}")
    return out


def mxfp4_quantize_out(x: Tensor, codes: Tensor, scales: Tensor) -> tuple[Tensor, Tensor]:
    contract.check_quantize_input("mxfp4_quantize", x)
    dev = _dev(x, codes, scales)
    x = x.contiguous()
    _contig_out(codes, "mxfp4_quantize")
    _contig_out(scales, "mxfp4_quantize")
    rows, K = x.shape
    if tuple(codes.shape) != (rows, K // 2) or tuple(scales.shape) != (rows, K // 32) or codes.dtype != torch.uint8 \
            or scales.dtype != torch.uint8:
        raise ValueError("mxfp4_quantize: codes must be uint8 [rows, K/2] and scales uint8 [rows, K/32]")
    with torch.cuda.device(dev):
        rc = _lib.load().mi355_mxfp4_quantize(x.data_ptr(), _lib.dtype_code(x.dtype), rows, K, codes.data_ptr(),
                                              scales.data_ptr(), _lib.current_stream_ptr(dev))
    _lib.check(rc, f"mxfp4_quantize rows={rows} K={K} in={x.dtype}")
    return codes, scales


def mxfp6_quantize_out(x: Tensor, codes: Tensor, scales: Tensor, element_format: str = "e2m3") -> tuple[Tensor, Tensor]:
    dev = _dev(x, codes, scales)
    if element_format not in FP6_FORMATS:
        raise ValueError(f"mxfp6_quantize: element_format must be one of {sorted(FP6_FORMATS)}, got {element_format!r}")
    contract.check_quantize_input("mxfp6_quantize", x)
    x = x.contiguous()
    _contig_out(codes, "mxfp6_quantize")
    _contig_out(scales, "mxfp6_quantize")
    rows, K = x.shape
    if tuple(codes.shape) != (rows, K // 4 * 3) or tuple(scales.shape) != (rows, K // 32) or codes.dtype != torch.uint8 \
            or scales.dtype != torch.uint8:
        raise ValueError("mxfp6_quantize: codes must be uint8 [rows, K*3/4] and scales uint8 [rows, K/32]")
    with torch.cuda.device(dev):
        rc = _lib.load().mi355_mxfp6_quantize(x.data_ptr(), _lib.dtype_code(x.dtype), rows, K, FP6_FORMATS[element_format],
                                              codes.data_ptr(), scales.data_ptr(), _lib.current_stream_ptr(dev))
    _lib.check(rc, f"mxfp6_quantize rows={rows} K={K} in={x.dtype} format={element_format}")
    return codes, scales


def mxfp8_quantize_out(x: Tensor, codes: Tensor, scales: Tensor) -> tuple[Tensor, Tensor]:
    contract.check_quantize_input("mxfp8_quantize", x)
    dev = _dev(x, codes, scales)
    x = x.contiguous()
    _contig_out(codes, "mxfp8_quantize")
    _contig_out(scales, "mxfp8_quantize")
    rows, K = x.shape
    if tuple(codes.shape) != (rows, K) or tuple(scales.shape) != (rows, K // 32) or codes.dtype != torch.uint8 \
            or scales.dtype != torch.uint8:
        raise ValueError("mxfp8_quantize: codes must be uint8 [rows, K] and scales uint8 [rows, K/32]")
    with torch.cuda.device(dev):
        rc = _lib.load().mi355_mxfp8_quantize(x.data_ptr(), _lib.dtype_code(x.dtype), rows, K, codes.data_ptr(),
                                              scales.data_ptr(), _lib.current_stream_ptr(dev))
    _lib.check(rc, f"mxfp8_quantize rows={rows} K={K} in={x.dtype}")
    return codes, scales
