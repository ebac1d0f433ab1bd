"""CPU-side tests of the boundary: the C-ABI library loads and exports every declared symbol, the
custom ops have Meta kernels and contract checks, nothing falls back to the CPU, and the template /
launchable surface behaves like the reference's (no kernel is launched here)."""

import re
from pathlib import Path

import pytest
import sympy
import torch

import iree_turbine_amd as ita
from iree_turbine_amd import _lib, lang, op_reg
from iree_turbine_amd.templates import (AttentionShape, get_gemm_kernel, get_mxfp4_gemm_kernel,
                                         get_paged_decode_attention_kernels, get_vanilla_attention_kernel,
                                         paged_decode_attention_shape)

ROOT = Path(__file__).resolve().parent.parent


def test_library_exports_every_declared_symbol():
    header = (ROOT / "include" / "turbine_mi355.h").read_text()
    declared = set(re.findall(r"\b(mi355_[a-z0-9_]+)\s*\(", header))
    assert declared == set(_lib.EXPORTED_SYMBOLS), declared ^ set(_lib.EXPORTED_SYMBOLS)
    lib = _lib.load()
    for name in declared:
        assert getattr(lib, name) is not None
    assert lib.mi355_abi_version() == 1
    assert _lib.variants("gemm_f16_nt")[0].startswith("persistent_256x256")
    assert _lib.variants("no_such_family") == []


def test_c_abi_rejects_bad_arguments_without_a_gpu():
    lib = _lib.load()
    assert lib.mi355_gemm_f16_nt(None, None, None, 16, 16, 16, 0, -1, None) == -1  # MI355_E_NULL
    assert "null pointer" in _lib.last_error()
    assert lib.mi355_gemm_f16_nt(16, 16, 16, 0, 16, 16, 0, -1, None) == -2  # MI355_E_SHAPE
    assert lib.mi355_gemm_f16_nt(16, 16, 16, 16, 16, 16, 7, -1, None) == -4  # MI355_E_DTYPE
    assert lib.mi355_flash_attn_fwd(16, 16, 16, 16, 1, 1, 8, 8, 64, 1.0, 0, -1, None) == -2  # D != 128
    assert lib.mi355_flash_attn_fwd(16, 16, 16, 24, 1, 1, 8, 8, 128, 1.0, 0, -1, None) == -3  # misaligned o
    assert lib.mi355_mxfp4_gemm(16, 16, 16, 16, 16, 4, 4, 48, 2, -1, None) == -2  # K % 32
    assert lib.mi355_paged_decode_attn(16, 16, 16, 16, 16, 16, None, None, 2, 8, 2, 128, 16, 4, 9, 4, 1.0, None) == -5  # scratch
    assert lib.mi355_paged_decode_attn(16, 16, 16, 16, 16, 16, None, None, 2, 8, 2, 128, 8, 4, 9, 1, 1.0, None) == -2  # page 8
    with pytest.raises(ValueError, match="contract violation"):
        _lib.check(-2, "x")
    with pytest.raises(_lib.KernelLibraryError, match="HIP error"):
        _lib.check(1, "x")


def test_ops_registered_with_meta_kernels():
    for name in ("gemm_nt", "flash_attn_fwd", "paged_decode_attn", "paged_decode_phase0", "paged_decode_phase1",
                 "mxfp4_gemm", "mxfp4_dequant"):
        assert f"mi355.{name}" in op_reg.ALL_CUSTOM_OP_REGS
    a = torch.empty(64, 32, dtype=torch.float16, device="meta")
    b = torch.empty(48, 32, dtype=torch.float16, device="meta")
    c = torch.ops.mi355.gemm_nt(a, b, "float32", -1)
    assert c.shape == (64, 48) and c.dtype == torch.float32 and c.device.type == "meta"
    q = torch.empty(2, 4, 100, 128, dtype=torch.float16, device="meta")
    k = torch.empty(2, 4, 77, 128, dtype=torch.float16, device="meta")
    assert torch.ops.mi355.flash_attn_fwd(q, k, k, True, 0.0).shape == q.shape
    u8 = lambda *s: torch.empty(*s, dtype=torch.uint8, device="meta")
    o = torch.ops.mi355.mxfp4_gemm(u8(32, 64), u8(32, 4), u8(16, 64), u8(16, 4), "bfloat16", -1)
    assert o.shape == (32, 16) and o.dtype == torch.bfloat16
    assert torch.ops.mi355.mxfp4_dequant(u8(8, 16), u8(8, 1)).shape == (8, 32)


def test_op_contract_errors_on_meta():
    h = lambda *s: torch.empty(*s, dtype=torch.float16, device="meta")
    with pytest.raises(ValueError, match="K mismatch"):
        torch.ops.mi355.gemm_nt(h(4, 8), h(4, 16), "float32", -1)
    with pytest.raises(ValueError, match="out_dtype"):
        torch.ops.mi355.gemm_nt(h(4, 8), h(4, 8), "bfloat16", -1)
    with pytest.raises(ValueError, match="head dim"):
        torch.ops.mi355.flash_attn_fwd(h(1, 1, 8, 64), h(1, 1, 8, 64), h(1, 1, 8, 64), False, 0.0)
    bt = torch.empty(2, 4, dtype=torch.int32, device="meta")
    sl = torch.empty(2, dtype=torch.int32, device="meta")
    with pytest.raises(ValueError, match="page size"):
        torch.ops.mi355.paged_decode_attn(h(2, 8, 128), h(9, 48, 2, 128), h(9, 48, 2, 128), bt, sl, 0.0, 1)  # 48 is not 16 * 2^n
    with pytest.raises(ValueError, match="q heads"):
        torch.ops.mi355.paged_decode_attn(h(2, 6, 128), h(9, 16, 4, 128), h(9, 16, 4, 128), bt, sl, 0.0, 1)


def test_no_cpu_fallback():
    a = torch.zeros(16, 16, dtype=torch.float16)
    with pytest.raises(NotImplementedError):
        torch.ops.mi355.gemm_nt(a, a, "float32", -1)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        ita.launch.gemm_nt_out(a, a, torch.zeros(16, 16), -1)
    # the product never imports the oracle
    for py in (ROOT / "iree_turbine_amd").rglob("*.py"):
        assert "oracle" not in py.read_text(), py


def test_duplicate_registration_raises():
    with pytest.raises(RuntimeError, match="Duplicate turbine custom op registration"):
        @op_reg.CustomOp.register
        class gemm_nt(op_reg.CustomOp):  # noqa: F811
            signature = "gemm_nt(Tensor a) -> Tensor"

            def select(self, sel):
                pass


def test_spec_key_format():
    op = op_reg.ALL_CUSTOM_OP_REGS["mi355.gemm_nt"]
    a = torch.empty(64, 32, dtype=torch.float16, device="meta")
    sel = op_reg.KernelSelection(op, [a, a, "float16", -1])
    op.select(sel)
    assert sel.spec_key == ("mi355.DEF::gemm_nt::default(tensor[2:torch.float16]<[64, 32]>,tensor[2:torch.float16]<[64, 32]>,"
                            "attr(float16),attr(-1))->(tensor[2:torch.float16]<[64, 64]>)")


def test_symbols_and_bindings():
    assert lang.sym.BLOCK_M == sympy.Symbol("BLOCK_M", integer=True, nonnegative=True)
    b = lang.SymbolBindings({lang.sym.M: 4})
    b.bind_constant(lang.sym.M, 4)
    with pytest.raises(ValueError, match="Attempt to bind symbol M=5 conflicts with previous 4"):
        b.bind_constant(lang.sym.M, 5)
    assert b.get_static_value(lang.sym.M * 4) == 16 and b.get_static_value(lang.sym.N) is None
    assert lang.f4e2m1fn.bitwidth() == 4 and lang.f8e8m0fnu.bitwidth() == 8 and lang.f16.bitwidth() == 16


def test_template_getters_and_launchable_rules():
    k, hp = get_gemm_kernel((8192, 8192, 8192))
    assert hp[lang.sym.BLOCK_M] == 256 and hp[lang.sym.M] == 8192
    assert get_gemm_kernel((1024, 1024, 1024))[1][lang.sym.BLOCK_M] == 128
    assert lang.sym.M not in get_gemm_kernel((33, 65, 17), dynamic_dims=True)[1]
    run = ita.wave_compile(ita.WaveCompileOptions(subs=hp), k)
    with pytest.raises(RuntimeError, match="without any Tensor args"):
        run()
    with pytest.raises(RuntimeError, match="multiple devices"):
        run(torch.zeros(2, 2), torch.zeros(2, 2, device="meta"), torch.zeros(2, 2))
    with pytest.raises(ValueError, match="specialised for M=8192"):
        run(torch.zeros(4, 4).half(), torch.zeros(4, 4).half(), torch.zeros(4, 4))
    with pytest.raises(ValueError, match="conflicts with previous"):
        ita.wave_compile(ita.WaveCompileOptions(subs={lang.sym.M: 1}), run)
    with pytest.raises(ValueError, match="float16"):
        get_gemm_kernel((64, 64, 64), dtype=torch.float32)
    shape = AttentionShape(num_query_heads=32, num_kv_heads=32, head_size=128, head_size_kv=128, query_seq_len=4096, kv_seq_len=4096)
    fa, fhp = get_vanilla_attention_kernel(shape, is_causal=True)
    assert fhp == {lang.sym.BLOCK_M: 128, lang.sym.BLOCK_N: 64} and "causal" in fa.name
    with pytest.raises(ValueError, match="head size 128"):
        get_vanilla_attention_kernel(AttentionShape(8, 8, 64, 64))
    dshape = paged_decode_attention_shape(32, 8, 128, 128, 16, 64)
    p0, p1, hp0, hp1 = get_paged_decode_attention_kernels(dshape, num_kv_splits=8, k_shape=(100, 16, 8, 128))
    assert p0.num_outputs == 2 and p1.num_outputs == 1 and hp0[lang.sym.U] == 8
    assert get_paged_decode_attention_kernels(paged_decode_attention_shape(32, 8, 128, 128, 32, 64))[2][lang.sym.BLOCK_SIZE] == 32
    with pytest.raises(ValueError, match="pages of 16, 32, 64, 128 or 256"):
        get_paged_decode_attention_kernels(paged_decode_attention_shape(32, 8, 128, 128, 48, 64))
    mk, mhp = get_mxfp4_gemm_kernel((4096, 8192, 8192))
    assert mhp[lang.sym.BLOCK_K] == 256
    with pytest.raises(ValueError, match="multiple of 32"):
        get_mxfp4_gemm_kernel((32, 32, 48))
