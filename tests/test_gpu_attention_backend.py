"""The reference's own two attention-backend tests (tests/diffusion/attention/test_flash_attn.py:60-147 and
153-261), run against this package's backend classes: same shapes (8 heads x 64, 48 + 16 tokens padded by 10
each), same seeds (42, 123), same thresholds. Inputs are drawn on the CPU so the vectors do not depend on the
device's generator."""

import pytest
import torch

pytestmark = pytest.mark.gpu

HIDDEN, ENCODER, PAD, HEADS, DIM = 48, 16, 10, 8, 64


def _mask(batch, seq_len, valid, device):
    m = torch.zeros(batch, seq_len, dtype=torch.bool, device=device)
    m[:, :valid] = True
    return m


def _pad(t, target):
    b, s, h, d = t.shape
    return torch.cat([t, torch.zeros(b, target - s, h, d, dtype=t.dtype, device=t.device)], dim=1)


def _valid(out):
    return torch.cat([out[:, :HIDDEN], out[:, HIDDEN + PAD:HIDDEN + PAD + ENCODER]], dim=1)


def test_padding_equivalence(gpu):
    """Case 1: batch 1; unpadded without a mask against padded with the [B,S] key-padding mask."""
    from vllm_omni_amd.attention.backends.abstract import AttentionMetadata
    from vllm_omni_amd.attention.backends.hip_flash import HipFlashAttentionImpl

    impl = HipFlashAttentionImpl(num_heads=HEADS, head_size=DIM, softmax_scale=1.0 / (DIM ** 0.5), causal=False)
    torch.manual_seed(42)
    hidden = torch.randn(1, HIDDEN, HEADS, DIM).bfloat16().to(gpu)
    encoder = torch.randn(1, ENCODER, HEADS, DIM).bfloat16().to(gpu)
    qa = torch.cat([hidden, encoder], dim=1)
    out_a = impl.forward(query=qa, key=qa.clone(), value=qa.clone(), attn_metadata=AttentionMetadata(attn_mask=None))
    qb = torch.cat([_pad(hidden, HIDDEN + PAD), _pad(encoder, ENCODER + PAD)], dim=1)
    mask = torch.cat([_mask(1, HIDDEN + PAD, HIDDEN, gpu), _mask(1, ENCODER + PAD, ENCODER, gpu)], dim=1)
    out_b = impl.forward(query=qb, key=qb.clone(), value=qb.clone(), attn_metadata=AttentionMetadata(attn_mask=mask))
    diff = (out_a - _valid(out_b)).abs()
    print(f"padding equivalence: max {diff.max().item():.2e} mean {diff.float().mean().item():.2e}", flush=True)
    assert diff.max().item() < 0.1 and diff.float().mean().item() < 0.01   # the reference's thresholds
    # the padding moves keys to other tiles, so sums re-associate: one bf16 ulp of an O(1) value at most
    assert diff.max().item() <= 2 ** -7


def test_hip_flash_vs_sdpa(gpu):
    """Case 2: batch 2 with padding; the HIP backend with the 2-D mask against the SDPA backend with the
    additive 4-D mask the reference test builds for it."""
    from vllm_omni_amd.attention.backends.abstract import AttentionMetadata
    from vllm_omni_amd.attention.backends.hip_flash import HipFlashAttentionImpl
    from vllm_omni_amd.attention.backends.sdpa import SDPAImpl

    kw = dict(num_heads=HEADS, head_size=DIM, softmax_scale=1.0 / (DIM ** 0.5), causal=False)
    fa, sdpa = HipFlashAttentionImpl(**kw), SDPAImpl(**kw)
    torch.manual_seed(123)
    hidden = torch.randn(2, HIDDEN, HEADS, DIM).bfloat16().to(gpu)
    encoder = torch.randn(2, ENCODER, HEADS, DIM).bfloat16().to(gpu)
    q = torch.cat([_pad(hidden, HIDDEN + PAD), _pad(encoder, ENCODER + PAD)], dim=1)
    mask = torch.cat([_mask(2, HIDDEN + PAD, HIDDEN, gpu), _mask(2, ENCODER + PAD, ENCODER, gpu)], dim=1)
    out_fa = fa.forward(query=q.clone(), key=q.clone(), value=q.clone(), attn_metadata=AttentionMetadata(attn_mask=mask))
    mask4 = mask[:, None, None, :]
    additive = torch.zeros_like(mask4, dtype=torch.bfloat16).masked_fill_(~mask4, float("-inf"))
    out_sdpa = sdpa.forward(query=q.clone(), key=q.clone(), value=q.clone(),
                            attn_metadata=AttentionMetadata(attn_mask=additive))
    diff = (_valid(out_fa) - _valid(out_sdpa)).abs()
    print(f"hip flash vs sdpa: max {diff.max().item():.2e} mean {diff.float().mean().item():.2e}", flush=True)
    assert diff.max().item() < 0.01 and diff.float().mean().item() < 0.001   # the reference's thresholds


def test_what_the_kernel_does_not_take_goes_to_sdpa(gpu):
    """The backends this one replaces take causal attention, any head size and masks of any broadcastable shape
    (vllm_omni/diffusion/attention/backends/sdpa.py:73-92): such calls run on the SDPA route and give what
    torch's scaled_dot_product_attention gives for the permuted tensors."""
    from vllm_omni_amd import kernels
    from vllm_omni_amd.attention.backends.abstract import AttentionMetadata
    from vllm_omni_amd.attention.backends.hip_flash import HipFlashAttentionImpl

    def sdpa(q, k, v, mask=None, causal=False):
        o = torch.nn.functional.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2),
                                                             attn_mask=mask, is_causal=causal, scale=q.shape[-1] ** -0.5)
        return o.transpose(1, 2)

    calls = []
    orig = kernels.attn_fwd
    kernels.attn_fwd = lambda *a, **kw: (calls.append(1), orig(*a, **kw))[1]
    try:
        torch.manual_seed(7)
        q, k, v = (torch.randn(2, 40, 4, 64).bfloat16().to(gpu) for _ in range(3))
        kw = dict(num_heads=4, head_size=64, softmax_scale=64 ** -0.5)
        # the 4-D additive mask the reference's SDPA test builds
        keep = torch.ones(2, 1, 1, 40, dtype=torch.bool, device=gpu)
        keep[:, :, :, 33:] = False
        additive = torch.zeros(2, 1, 1, 40, dtype=torch.bfloat16, device=gpu).masked_fill_(~keep, float("-inf"))
        impl = HipFlashAttentionImpl(causal=False, **kw)
        got = impl.forward(query=q, key=k, value=v, attn_metadata=AttentionMetadata(attn_mask=additive))
        torch.testing.assert_close(got.float(), sdpa(q, k, v, additive).float(), atol=2e-2, rtol=2e-2)
        # a full [B,H,Sq,Sk] boolean mask
        full = (torch.rand(2, 4, 40, 40, device=gpu) > 0.3)
        full[..., 0] = True
        got = impl.forward(query=q, key=k, value=v, attn_metadata=AttentionMetadata(attn_mask=full))
        torch.testing.assert_close(got.float(), sdpa(q, k, v, full).float(), atol=2e-2, rtol=2e-2)
        # causal
        got = HipFlashAttentionImpl(causal=True, **kw).forward(query=q, key=k, value=v)
        torch.testing.assert_close(got.float(), sdpa(q, k, v, causal=True).float(), atol=2e-2, rtol=2e-2)
        # a head size outside the kernel's
        q96, k96, v96 = (torch.randn(1, 24, 2, 96).bfloat16().to(gpu) for _ in range(3))
        got = HipFlashAttentionImpl(num_heads=2, head_size=96, softmax_scale=96 ** -0.5).forward(query=q96, key=k96, value=v96)
        torch.testing.assert_close(got.float(), sdpa(q96, k96, v96).float(), atol=2e-2, rtol=2e-2)
        assert not calls, "none of these may reach the HIP kernel"
        # and the [B,Sk] boolean mask does
        m2 = keep[:, 0, 0, :]
        got = impl.forward(query=q, key=k, value=v, attn_metadata=AttentionMetadata(attn_mask=m2))
        torch.testing.assert_close(got.float(), sdpa(q, k, v, keep).float(), atol=2e-2, rtol=2e-2)
        assert len(calls) == 1
    finally:
        kernels.attn_fwd = orig
