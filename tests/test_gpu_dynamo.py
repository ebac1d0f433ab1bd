"""GPU: `torch.compile(..., backend="mi355")` routes linear layers and attention to the MI355X kernels and gives
what eager PyTorch gives.  The model is the attention + feed-forward block of the reference's dynamo test
(tests/dynamo/llama_test.py:94-248) with the attention written as `scaled_dot_product_attention`, the form the
reference's fusion schema roots at (iree/turbine/kernel/boo/fusion/schema.py:116-135)."""

import pytest
import torch
import torch.nn.functional as F
from torch import nn

from conftest import announce

pytestmark = pytest.mark.gpu


class Block(nn.Module):
    def __init__(self, dim=512, n_heads=4, n_kv_heads=4, hidden=1024, bias=False):
        super().__init__()
        self.h, self.hkv, self.d = n_heads, n_kv_heads, dim // n_heads
        self.wq = nn.Linear(dim, n_heads * self.d, bias=bias)
        self.wk = nn.Linear(dim, n_kv_heads * self.d, bias=bias)
        self.wv = nn.Linear(dim, n_kv_heads * self.d, bias=bias)
        self.wo = nn.Linear(n_heads * self.d, dim, bias=bias)
        self.w1 = nn.Linear(dim, hidden, bias=bias)
        self.w2 = nn.Linear(hidden, dim, bias=bias)
        self.w3 = nn.Linear(dim, hidden, bias=bias)
        self.norm1 = nn.LayerNorm(dim)
        self.norm2 = nn.LayerNorm(dim)

    def forward(self, x):
        B, S, _ = x.shape
        y = self.norm1(x)
        q = self.wq(y).view(B, S, self.h, self.d).transpose(1, 2)
        k = self.wk(y).view(B, S, self.hkv, self.d).transpose(1, 2)
        v = self.wv(y).view(B, S, self.hkv, self.d).transpose(1, 2)
        a = F.scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=self.h != self.hkv)
        x = x + self.wo(a.transpose(1, 2).reshape(B, S, -1))
        y = self.norm2(x)
        return x + self.w2(F.silu(self.w1(y)) * self.w3(y))


@pytest.mark.parametrize("bias,hkv", [(False, 4), (True, 4), (False, 2)])
def test_compiled_block_matches_eager(dev, bias, hkv):
    import iree_turbine_amd.dynamo as mdyn

    announce(f"torch.compile backend=mi355 bias={bias} hkv={hkv}")
    torch.manual_seed(3)
    torch._dynamo.reset()
    model = Block(bias=bias, n_kv_heads=hkv).to(dev).half().eval()
    x = torch.randn(2, 192, 512, device=dev).half()
    with torch.no_grad():
        want = model(x)
        mdyn.LAST_SUBSTITUTIONS.clear()
        got = torch.compile(model, backend="mi355")(x)
        again = torch.compile(model, backend="mi355")(x)
    torch.cuda.synchronize()
    counts = dict(mdyn.LAST_SUBSTITUTIONS)
    if hkv == 4:  # with grouped heads PyTorch may pick a decomposed attention; the products are routed either way
        assert counts["sdpa"] == 1, counts
    assert counts["mm"] + counts["addmm"] == 7, counts
    assert (counts["addmm"] == 7) if bias else (counts["mm"] == 7), counts
    torch.testing.assert_close(got.float(), want.float(), rtol=1e-2, atol=1e-2)
    assert torch.equal(got, again)


def test_compiled_bf16_block_routes_its_linear_layers(dev):
    """In bf16 the seven linear layers go to the bf16 GEMM and attention to the bf16 attention kernel; the result
    is what eager gives, to bf16's 8 bits."""
    import iree_turbine_amd.dynamo as mdyn

    announce("torch.compile backend=mi355 bf16")
    torch.manual_seed(4)
    torch._dynamo.reset()
    model = Block(bias=True).to(dev).bfloat16().eval()
    x = torch.randn(2, 192, 512, device=dev).bfloat16()
    with torch.no_grad():
        want = model(x)
        mdyn.LAST_SUBSTITUTIONS.clear()
        got = torch.compile(model, backend="mi355")(x)
    torch.cuda.synchronize()
    counts = dict(mdyn.LAST_SUBSTITUTIONS)
    assert counts["addmm"] == 7 and counts["sdpa"] == 1, counts
    assert got.dtype == torch.bfloat16
    torch.testing.assert_close(got.float(), want.float(), rtol=5e-2, atol=5e-2)


def test_compiled_training_step_keeps_attention_in_pytorch(dev):
    """With gradients the log-sum-exp of the attention is consumed by the backward graph, so the attention stays
    with PyTorch; the matrix products of both the forward and the backward graph still go to the kernels."""
    import iree_turbine_amd.dynamo as mdyn

    announce("torch.compile backend=mi355 training step")
    torch.manual_seed(4)
    torch._dynamo.reset()
    model = Block().to(dev).half()
    ref = Block().to(dev).half()
    ref.load_state_dict(model.state_dict())
    x = torch.randn(1, 128, 512, device=dev).half()
    mdyn.LAST_SUBSTITUTIONS.clear()
    torch.compile(model, backend="mi355")(x).float().square().mean().backward()
    ref(x).float().square().mean().backward()
    torch.cuda.synchronize()
    assert mdyn.LAST_SUBSTITUTIONS["mm"] > 0
    for (n, p), (_, r) in zip(model.named_parameters(), ref.named_parameters()):
        scale = r.grad.float().abs().max().item() + 1e-6
        assert (p.grad.float() - r.grad.float()).abs().max().item() <= 2e-2 * scale, n


def test_causal_attention_with_unequal_lengths_keeps_pytorch(dev):
    """aten's causal mask is aligned to the first key, the kernel's to the last: for Sq != Sk the pass must leave
    the call alone, and the compiled result must equal eager PyTorch's."""
    import torch.nn.functional as F

    import iree_turbine_amd.dynamo as mdyn

    announce("torch.compile causal Sq != Sk")
    torch.manual_seed(5)
    torch._dynamo.reset()
    q = torch.randn(1, 4, 128, 128, device=dev).half()
    k = torch.randn(1, 4, 320, 128, device=dev).half()
    v = torch.randn(1, 4, 320, 128, device=dev).half()

    def attn(q, k, v):
        return F.scaled_dot_product_attention(q, k, v, is_causal=True) * 2.0

    with torch.no_grad():
        want = attn(q, k, v)
        mdyn.LAST_SUBSTITUTIONS.clear()
        got = torch.compile(attn, backend="mi355")(q, k, v)
    torch.cuda.synchronize()
    assert mdyn.LAST_SUBSTITUTIONS.get("sdpa", 0) == 0
    torch.testing.assert_close(got.float(), want.float(), rtol=1e-3, atol=2e-3)
