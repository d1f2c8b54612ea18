"""The custom-op wrappers the vLLM-Omni plugin installs: same results as the direct C-ABI calls, valid
under torch's op checks, and traceable as one graph by ``torch.compile`` (the reference compiles its
repeated blocks, vllm_omni/diffusion/compile.py:11-41)."""

import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

from oracle import ops

pytestmark = pytest.mark.gpu


def _rand(*shape, seed=0, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g).to(dtype)


def test_ops_equal_the_direct_calls_and_pass_opcheck(gpu):
    from vllm_omni_amd import kernels, torch_ops  # noqa: F401
    from vllm_omni_amd._lib import ODIT_NORM_NONE

    q, k, v = (_rand(2, 130, 4, 64, seed=s).to(gpu) for s in (1, 2, 3))
    mask = torch.ones(2, 130, dtype=torch.bool, device=gpu)
    mask[1, 100:] = False
    for m in (None, mask):
        assert torch.equal(torch.ops.omni_dit.attention(q, k, v, 0.125, m), kernels.attn_fwd(q, k, v, 0.125, key_mask=m))
    x, mod = _rand(2, 130, 256, seed=4).to(gpu), _rand(2, 768, seed=5).to(gpu)
    shift, scale, _ = mod.chunk(3, dim=-1)
    assert torch.equal(torch.ops.omni_dit.adaln_modulate(x, shift, scale, 1e-6),
                       kernels.adaln_modulate(x, shift, scale, eps=1e-6))
    ang = torch.rand(130, 32, generator=torch.Generator().manual_seed(6)) * 6.0
    cos, sin = ang.cos().to(gpu), ang.sin().to(gpu)
    want = torch.empty_like(q)
    kernels.qknorm_rope(q, None, None, want, None, None, None, None, cos, sin, norm_mode=ODIT_NORM_NONE, neox=False)
    assert torch.equal(torch.ops.omni_dit.rotary(q, cos, sin, False), want)
    checks = ("test_schema", "test_faketensor", "test_aot_dispatch_static")
    torch.library.opcheck(torch.ops.omni_dit.attention.default, (q, k, v, 0.125, mask), test_utils=checks)
    torch.library.opcheck(torch.ops.omni_dit.adaln_modulate.default, (x, shift, scale, 1e-6), test_utils=checks)
    torch.library.opcheck(torch.ops.omni_dit.rotary.default, (q, cos, sin, False), test_utils=checks)


class _Layer(nn.Module):
    """Stand-in for a reference CustomOp layer: ``forward`` goes to ``forward_hip``."""

    def forward(self, *a, **kw):
        return self.forward_hip(*a, **kw)


class _AdaLN(_Layer):
    def __init__(self, C):
        super().__init__()
        self.eps, self.hidden_size = 1e-6, C
        self.layernorm = nn.LayerNorm(C, elementwise_affine=False, eps=1e-6)


class _Rope(_Layer):
    is_neox_style = False


class _MiniBlock(nn.Module):
    """One image-only block wired the way the reference wires its layers: adaLN -> qkv -> rotary ->
    attention -> projection -> gated residual."""

    def __init__(self, C=256, H=4):
        super().__init__()
        from vllm_omni_amd import plugin, torch_ops

        self.H, self.D = H, C // H
        self.norm, self.rope = _AdaLN(C), _Rope()
        _AdaLN.forward_hip = torch_ops.adaln_forward_hip
        _Rope.forward_hip = torch_ops.rope_forward_hip
        self.attn = plugin.CompiledHipFlashAttentionBackend.get_impl_cls()(
            num_heads=H, head_size=self.D, softmax_scale=self.D ** -0.5, causal=False, num_kv_heads=H)
        self.qkv, self.out = nn.Linear(C, 3 * C), nn.Linear(C, C)

    def forward(self, x, mod, cos, sin):
        h, gate = self.norm(x, mod)
        q, k, v = (t.unflatten(-1, (self.H, self.D)) for t in self.qkv(h).chunk(3, dim=-1))
        o = self.attn.forward(self.rope(q, cos, sin), self.rope(k, cos, sin), v)
        return x + gate * self.out(o.flatten(2, 3))


def test_compiled_block_is_one_graph_and_matches_eager_and_oracle(gpu):
    torch.manual_seed(0)
    blk = _MiniBlock().to(gpu).bfloat16()
    S = 96
    x, mod = _rand(2, S, 256, seed=7).to(gpu), (_rand(2, 768, seed=8) * 0.3).to(gpu)
    ang = torch.rand(S, 32, generator=torch.Generator().manual_seed(9)) * 6.0
    cos, sin = ang.cos().to(gpu), ang.sin().to(gpu)
    with torch.inference_mode():
        eager = blk(x, mod, cos, sin)
        compiled = torch.compile(blk, backend="aot_eager", fullgraph=True, dynamic=True)  # fullgraph: a break raises
        got = compiled(x, mod, cos, sin)
        got2 = compiled(x[:, :64], mod, cos[:64], sin[:64])   # another length through the same dynamic graph
        eager2 = blk(x[:, :64].contiguous(), mod, cos[:64], sin[:64])
    assert torch.equal(got, eager)
    assert torch.equal(got2, eager2)
    # and the whole thing is the reference arithmetic: fp32 oracle of the same wiring
    w = {k: v.float().cpu() for k, v in blk.state_dict().items()}
    xf, mf = x.float().cpu(), mod.float().cpu()
    h, gate = ops.ada_layer_norm(xf, mf, None, 1e-6)
    q, k, v = (t.unflatten(-1, (4, 64)) for t in F.linear(h, w["qkv.weight"], w["qkv.bias"]).chunk(3, dim=-1))
    o = ops.sdpa(ops.apply_rotary(q, ang.cos(), ang.sin()), ops.apply_rotary(k, ang.cos(), ang.sin()), v, 64 ** -0.5)
    want = xf + gate * F.linear(o.flatten(2, 3), w["out.weight"], w["out.bias"])
    assert (got.float().cpu() - want).abs().max().item() <= 3e-2
