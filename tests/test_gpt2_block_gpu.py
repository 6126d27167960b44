"""A GPT-2 style transformer block assembled from the hexmi operators (layer norm -> QKV matmul -> causal
attention -> projection -> residual -> layer norm -> MLP with GELU-tanh -> residual), checked against the same
block in PyTorch on the CPU in fp32. Stands in for the reference's model-level flow
(test/python/torch-mlir: gpt2lmheadmodel) at the level of one block; weights are random (no checkpoint)."""
import math

import pytest
import torch
import torch.nn.functional as F

pytestmark = pytest.mark.gpu


def _block_torch(x, p, heads):
    B, S, E = x.shape
    h = F.layer_norm(x, (E,), p["ln1_w"], p["ln1_b"], 1e-5)
    qkv = h @ p["w_qkv"] + p["b_qkv"]
    q, k, v = (t.view(B, S, heads, E // heads).transpose(1, 2) for t in qkv.split(E, dim=-1))
    a = F.scaled_dot_product_attention(q, k, v, is_causal=True)
    a = a.transpose(1, 2).reshape(B, S, E)
    x = x + a @ p["w_o"] + p["b_o"]
    h = F.layer_norm(x, (E,), p["ln2_w"], p["ln2_b"], 1e-5)
    m = F.gelu(h @ p["w_fc"] + p["b_fc"], approximate="tanh")
    return x + m @ p["w_proj"] + p["b_proj"]


def _block_hexmi(hexmi, x, p, heads):
    """Ten launches: every bias add and both residual adds ride in the epilogue of the matmul that produces their
    operand (`hexmi_gemm_ex`)."""
    B, S, E = x.shape
    D = E // heads
    rows = x.reshape(B * S, E)
    h = hexmi.layer_norm(rows, p["ln1_w"], p["ln1_b"], 1e-5)
    qkv = hexmi.matmul(h, p["w_qkv"], bias=p["b_qkv"])
    q, k, v = (t.reshape(B, S, heads, D).transpose(1, 2).contiguous() for t in qkv.split(E, dim=-1))
    a = hexmi.flash_attention(q, k, v, 1.0 / math.sqrt(D), True)
    a = a.transpose(1, 2).reshape(B * S, E).contiguous()
    rows = hexmi.matmul(a, p["w_o"], bias=p["b_o"], residual=rows)
    h = hexmi.layer_norm(rows, p["ln2_w"], p["ln2_b"], 1e-5)
    m = hexmi.gelu(hexmi.matmul(h, p["w_fc"], bias=p["b_fc"]))
    out = hexmi.matmul(m, p["w_proj"], bias=p["b_proj"], residual=rows)
    return out.reshape(B, S, E)


def _block_hexmi_unfused(hexmi, x, p, heads):
    """The same block with every bias and residual add as its own launch (seven more)."""
    B, S, E = x.shape
    D = E // heads
    rows = x.reshape(B * S, E)
    h = hexmi.layer_norm(rows, p["ln1_w"], p["ln1_b"], 1e-5)
    qkv = hexmi.binary("add", hexmi.matmul(h, p["w_qkv"]), p["b_qkv"].expand(B * S, 3 * E).contiguous())
    q, k, v = (t.reshape(B, S, heads, D).transpose(1, 2).contiguous() for t in qkv.split(E, dim=-1))
    a = hexmi.flash_attention(q, k, v, 1.0 / math.sqrt(D), True)
    a = a.transpose(1, 2).reshape(B * S, E).contiguous()
    rows = hexmi.binary("add", rows, hexmi.binary("add", hexmi.matmul(a, p["w_o"]),
                                                  p["b_o"].expand(B * S, E).contiguous()))
    h = hexmi.layer_norm(rows, p["ln2_w"], p["ln2_b"], 1e-5)
    m = hexmi.gelu(hexmi.binary("add", hexmi.matmul(h, p["w_fc"]), p["b_fc"].expand(B * S, 4 * E).contiguous()))
    out = hexmi.binary("add", rows, hexmi.binary("add", hexmi.matmul(m, p["w_proj"]),
                                                 p["b_proj"].expand(B * S, E).contiguous()))
    return out.reshape(B, S, E)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_gpt2_block(hexmi, dtype):
    B, S, E, heads = 2, 256, 768, 12                                  # GPT-2 small: 12 heads of 64
    g = torch.Generator().manual_seed(50)
    std = 0.02
    p = {"ln1_w": 1 + 0.1 * torch.randn(E, generator=g), "ln1_b": 0.1 * torch.randn(E, generator=g),
         "ln2_w": 1 + 0.1 * torch.randn(E, generator=g), "ln2_b": 0.1 * torch.randn(E, generator=g),
         "w_qkv": std * torch.randn(E, 3 * E, generator=g), "b_qkv": std * torch.randn(3 * E, generator=g),
         "w_o": std * torch.randn(E, E, generator=g), "b_o": std * torch.randn(E, generator=g),
         "w_fc": std * torch.randn(E, 4 * E, generator=g), "b_fc": std * torch.randn(4 * E, generator=g),
         "w_proj": std * torch.randn(4 * E, E, generator=g), "b_proj": std * torch.randn(E, generator=g)}
    x = torch.randn(B, S, E, generator=g)
    pl = {k: v.to(dtype) for k, v in p.items()}                       # the values both sides compute with
    want = _block_torch(x.to(dtype).float(), {k: v.float() for k, v in pl.items()}, heads)
    got = _block_hexmi(hexmi, x.to(dtype).cuda(), {k: v.cuda() for k, v in pl.items()}, heads).cpu().float()
    err = (got - want).abs().max().item()
    assert err <= (3e-2 if dtype == torch.float16 else 2e-1), err
    assert torch.isfinite(got).all()
    # fused epilogues round once where the separate adds round two or three times: no further from the fp32 block
    sep = _block_hexmi_unfused(hexmi, x.to(dtype).cuda(), {k: v.cuda() for k, v in pl.items()}, heads).cpu().float()
    assert err <= (sep - want).abs().max().item() * 1.25 + 1e-3
