"""Host-side logic of the product package against the oracle and against closed forms (CPU only)."""

import math

import numpy as np
import pytest
import torch
import torch.nn as nn

from oracle import denoise as odn
from oracle import teacache as otc
from vllm_omni_amd import denoise
from vllm_omni_amd.attention.backends.registry import DiffusionAttentionBackendEnum, register_diffusion_backend
from vllm_omni_amd.attention.selector import get_attn_backend
from vllm_omni_amd.cache.teacache.config import _MODEL_COEFFICIENTS, TeaCacheConfig
from vllm_omni_amd.cache.teacache.hook import TeaCacheHook, rel_l1_from_sums
from vllm_omni_amd.cache.teacache.state import TeaCacheState
from vllm_omni_amd.hooks.base import HookRegistry, ModelHook, StateManager


# ----------------------------------------------------------------------------------- TeaCache
def test_coefficients_are_the_references():
    for k, v in otc.COEFFICIENTS.items():
        assert _MODEL_COEFFICIENTS[k] == v
    assert TeaCacheConfig().rel_l1_thresh == 0.2
    with pytest.raises(ValueError):
        TeaCacheConfig(rel_l1_thresh=0.0)
    with pytest.raises(KeyError):
        TeaCacheConfig(transformer_type="Nope")
    with pytest.raises(ValueError):
        TeaCacheConfig(coefficients=[1.0, 2.0])


def _run_decider(rels, coeffs, thresh):
    hook = TeaCacheHook(TeaCacheConfig(rel_l1_thresh=thresh, coefficients=coeffs))
    st = TeaCacheState()
    out = []
    for r in rels:
        out.append(hook._decide(st, r))
        st.cnt += 1
    return out


def test_decision_sequence_hand_built():
    # |p(r)| = 0.1 per step with p(x) = x, threshold 0.25: compute, skip, skip, compute(reset), skip, skip, compute
    coeffs = [0.0, 0.0, 0.0, 1.0, 0.0]
    got = _run_decider([None] + [0.1] * 6, coeffs, 0.25)
    assert got == [True, False, False, True, False, False, True]
    # exact threshold hit computes (strict <)
    assert _run_decider([None, 0.25], coeffs, 0.25) == [True, True]


def test_decision_matches_oracle_on_random_trajectories():
    rng = np.random.default_rng(0)
    for name in ("QwenImageTransformer2DModel", "FluxTransformer2DModel"):
        coeffs = otc.COEFFICIENTS[name]
        for thresh in (0.1, 0.25, 0.6):
            rels = [None] + list(rng.uniform(0.0, 0.35, size=40))
            st = otc.BranchState()
            ref = []
            for r in rels:
                ref.append(otc.decide(st, r, coeffs, thresh))
                st.cnt += 1
            assert _run_decider(rels, coeffs, thresh) == ref


def test_rel_l1_from_sums_reproduces_torch_rounding():
    g = torch.Generator().manual_seed(3)
    for dtype in (torch.bfloat16, torch.float16, torch.float32):
        prev = torch.randn(2048, generator=g).to(dtype)
        cur = (prev.float() * 1.05 + 0.02 * torch.randn(2048, generator=g)).to(dtype)
        want = ((cur - prev).abs().mean() / (prev.abs().mean() + 1e-8)).item()
        sd = (cur - prev).abs().double().sum().item()
        sp = prev.abs().double().sum().item()
        got = rel_l1_from_sums(sd, sp, 2048, dtype)
        assert got == pytest.approx(want, rel=1e-6 if dtype == torch.float32 else 0)


# ----------------------------------------------------------------------------------- hooks
class _Toy(nn.Module):
    def forward(self, x, k=1):
        return x * 2 + k


def test_hook_registry_dispatch_rules():
    m = _Toy()
    reg = HookRegistry.get_or_create(m)
    assert HookRegistry.get_or_create(m) is reg
    assert m(3) == 7  # no hooks: original forward

    class AddOne(ModelHook):
        def post_forward(self, module, output):
            return output + 1

    class TimesTen(ModelHook):
        def pre_forward(self, module, *args, **kwargs):
            return (args[0] * 10,), kwargs

    reg.register_hook("a", AddOne())
    assert m(3) == 8
    reg.register_hook("b", TimesTen())
    assert m(3, k=0) == 61  # pre hooks in name order, post hooks reversed
    reg.remove_hook("a")
    reg.remove_hook("b")
    assert m(3) == 7

    class Replace(ModelHook):
        def new_forward(self, module, *args, **kwargs):
            return "replaced"

    reg.register_hook("r", Replace())
    assert m(1) == "replaced"


def test_state_manager_contexts():
    sm = StateManager(TeaCacheState)
    sm.set_context("teacache_positive")
    a = sm.get_state()
    a.cnt = 5
    sm.set_context("teacache_negative")
    assert sm.get_state().cnt == 0
    sm.set_context("teacache_positive")
    assert sm.get_state() is a and sm.current_context == "teacache_positive"
    sm.reset()
    assert sm.get_state().cnt == 0


def test_hook_route_is_rebuilt_when_the_hook_set_changes():
    m = _Toy()
    reg = HookRegistry.get_or_create(m)
    calls = []

    class Skip(ModelHook):
        def initialize_hook(self, module):
            calls.append("init")
            return module

        def new_forward(self, module, *args, **kwargs):
            return module._original_forward(*args, **kwargs) if args[0] else "skipped"

        def reset_state(self, module):
            calls.append("reset")
            return module

    reg.register_hook("skip", Skip())
    assert calls == ["init"] and m(0) == "skipped" and m(2) == 5 and reg.dispatch(2) == 5
    reg.reset_hook("skip")
    reg.reset_hook("absent")
    assert calls == ["init", "reset"] and isinstance(reg.get_hook("skip"), Skip) and reg.get_hook("absent") is None
    reg.remove_hook("absent")
    reg.remove_hook("skip")
    assert m(0) == 1 and m._hook_registry is reg and m._original_forward(1) == 3


def test_qwen_rotary_tables_from_integer_positions_equal_the_oracles():
    from oracle import qwen_image as oq
    from vllm_omni_amd.blocks.qwen_image import QwenEmbedLayer3DRope, QwenEmbedRope

    cfg = oq.tiny_config()
    cases = [(False, [(1, 4, 6)]), (False, [(1, 5, 3)]), (False, [(1, 4, 4), (1, 6, 2), (2, 3, 5)]),
             (True, [(1, 2, 2)] * 5 + [(1, 2, 3)]), (True, [(1, 3, 3)]), (False, [(1, 64, 64)])]
    for layer3d, shapes in cases:
        rope = (QwenEmbedLayer3DRope if layer3d else QwenEmbedRope)(
            theta=cfg.theta, axes_dim=list(cfg.axes_dims_rope), scale_rope=True)
        vid, txt = rope(shapes, [3, 5], "cpu")
        want_v, want_t = oq.qwen_rope_freqs_images(cfg, shapes, txt_len=5, layer3d=layer3d)
        assert vid.dtype == torch.complex64 and torch.equal(vid, want_v) and torch.equal(txt, want_t)
    # built under a non-default device context (as bench.py builds the model) the tables still come from the host
    with torch.device("meta"):
        rope_meta = QwenEmbedRope(theta=cfg.theta, axes_dim=list(cfg.axes_dims_rope), scale_rope=True)
    vid_m, txt_m = rope_meta([(1, 4, 6)], [5], "cpu")
    want_v, want_t = oq.qwen_rope_freqs_images(cfg, [(1, 4, 6)], txt_len=5)
    assert torch.equal(vid_m, want_v) and torch.equal(txt_m, want_t)
    # without centring rows and columns count from zero and text starts after the full extent
    plain = QwenEmbedRope(theta=10000, axes_dim=[4, 6, 6], scale_rope=False)
    vid, txt = plain((1, 2, 3), [2], "cpu")
    inv = 1.0 / np.power(10000.0, np.arange(0, 6, 2) / 6)
    np.testing.assert_allclose(vid[5, 2:5].numpy(), np.exp(1j * 1 * inv), atol=1e-6)   # token (0, 1, 2): row 1
    np.testing.assert_allclose(vid[5, 5:8].numpy(), np.exp(1j * 2 * inv), atol=1e-6)   # column 2
    np.testing.assert_allclose(txt[1, 5:8].numpy(), np.exp(1j * 4 * inv), atol=1e-6)   # start 3, second token


# ----------------------------------------------------------------------------------- registry / selector
def test_backend_registry_and_selector(monkeypatch):
    E = DiffusionAttentionBackendEnum
    with pytest.raises(ValueError, match="Unknown diffusion attention backend"):
        E["NOPE"]
    with pytest.raises(ValueError, match="must be registered"):
        E.SAGE_ATTN.get_path()
    assert E.FLASH_ATTN.get_class().get_name() == "HIP_FLASH_ATTN"
    assert E.TORCH_SDPA.get_class().get_name() == "SDPA"
    register_diffusion_backend(E.TORCH_SDPA, E.FLASH_ATTN.value)
    try:
        assert E.TORCH_SDPA.is_overridden() and E.TORCH_SDPA.get_class().get_name() == "HIP_FLASH_ATTN"
    finally:
        E.TORCH_SDPA.clear_override()
    get_attn_backend.cache_clear()
    assert get_attn_backend(-1).get_name() == "HIP_FLASH_ATTN"
    get_attn_backend.cache_clear()
    monkeypatch.setenv("DIFFUSION_ATTENTION_BACKEND", "TORCH_SDPA")
    assert get_attn_backend(-1).get_name() == "SDPA"
    get_attn_backend.cache_clear()
    cls = get_attn_backend.__wrapped__(-1).get_impl_cls()
    from vllm_omni_amd.attention.backends.hip_flash import HipFlashAttentionImpl

    # what the kernel does not take is routed to SDPA, as the backends this one replaces take it
    # (vllm_omni/diffusion/attention/backends/sdpa.py:73-92); on the CPU that route runs as it is
    causal = HipFlashAttentionImpl(4, 64, 0.125, causal=True)
    assert not causal.kernel_takes_layer and not HipFlashAttentionImpl(2, 96, 0.1).kernel_takes_layer
    assert HipFlashAttentionImpl(4, 64, 0.125).kernel_takes_layer
    q = torch.randn(1, 6, 4, 64)
    want = torch.nn.functional.scaled_dot_product_attention(q.transpose(1, 2), q.transpose(1, 2), q.transpose(1, 2),
                                                            is_causal=True, scale=0.125).transpose(1, 2)
    assert torch.allclose(causal.forward(q, q, q), want, atol=1e-6)
    takes = HipFlashAttentionImpl.kernel_takes_mask
    assert takes(None, 2, 8) and takes(torch.ones(2, 8, dtype=torch.bool), 2, 8)
    assert not takes(torch.zeros(2, 8), 2, 8) and not takes(torch.ones(2, 1, 1, 8, dtype=torch.bool), 2, 8)
    assert not takes(torch.ones(8, 8, dtype=torch.bool), 2, 8)
    assert cls is not None


# ----------------------------------------------------------------------------------- denoise harness
def test_schedule_matches_oracle_and_closed_form():
    for n, s in ((4, 256), (20, 4096), (28, 1024)):
        a, b = denoise.flow_match_sigmas(n, s), odn.shifted_sigmas(n, s)
        assert np.array_equal(a, b) and a[-1] == 0.0 and len(a) == n + 1
        assert np.all(np.diff(a) < 0)
    # mu endpoints: 0.5 at 256 tokens, 1.15 at 4096; sigma=1 is a fixed point of the shift
    assert math.isclose(denoise.calculate_shift(256), 0.5) and math.isclose(denoise.calculate_shift(4096), 1.15)
    assert denoise.flow_match_sigmas(10, 4096)[0] == 1.0
    # shift formula at one interior point, by hand: s = 0.5, mu = 1.15 -> e/(e+1)
    sig = denoise.flow_match_sigmas(2, 4096)
    e = math.exp(1.15)
    assert math.isclose(float(sig[1]), e / (e + 1.0), rel_tol=1e-6)


def test_cfg_combine_and_euler_closed_forms():
    g = torch.Generator().manual_seed(0)
    pos, neg = torch.randn(1, 8, 4, generator=g), torch.randn(1, 8, 4, generator=g)
    assert torch.allclose(denoise.combine_cfg_noise(pos, neg, 1.0), pos, atol=1e-6)
    assert torch.allclose(denoise.combine_cfg_noise(pos, neg, 0.0), neg)
    out = denoise.combine_cfg_noise(pos, neg, 4.0, cfg_normalize=True)
    assert torch.allclose(out.norm(dim=-1), pos.norm(dim=-1), atol=1e-5)
    assert torch.allclose(out, odn.combine_cfg(pos, neg, 4.0, True))
    # Euler on a constant velocity field integrates exactly: x_end = x0 - v (sigma goes 1 -> 0)
    sig = denoise.flow_match_sigmas(7, 1024)
    x = torch.zeros(1, 3, 2)
    v = torch.full((1, 3, 2), 2.5)
    for i in range(7):
        x = denoise.euler_step(x, v, float(sig[i]), float(sig[i + 1]))
    assert torch.allclose(x, -v, atol=1e-5)
    # Euler on the linear field v = x / sigma keeps x / sigma constant: x_i = x_0 * sigma_i
    x = torch.ones(1, 2, 2)
    for i in range(6):
        x = denoise.euler_step(x, x / float(sig[i]), float(sig[i]), float(sig[i + 1]))
        assert torch.allclose(x, torch.full_like(x, float(sig[i + 1])), atol=1e-5)


# ----------------------------------------------------------------------------- checkpoint loading
def _split_qkv(flat, fused_suffix, names):
    """Turn fused [q;k;v] entries of a flat state into three separately stored tensors."""
    out = {}
    for k, v in flat.items():
        hit = next((f for f in fused_suffix if f in k), None)
        if hit is None:
            out[k] = v
            continue
        for part, t in zip(names[hit], v.chunk(3, dim=0)):
            out[k.replace(hit, part)] = t
    return out


def test_load_weights_stacks_qkv_and_renames_like_the_reference():
    from oracle import flux as ofx
    from oracle import qwen_image as oq
    from oracle import wan as ow
    from vllm_omni_amd.blocks.flux import FluxTransformer2DModel
    from vllm_omni_amd.blocks.qwen_image import QwenImageTransformer2DModel
    from vllm_omni_amd.blocks.wan import WanTransformer3DModel

    joint = {".to_qkv.": (".to_q.", ".to_k.", ".to_v."),
             ".add_kv_proj.": (".add_q_proj.", ".add_k_proj.", ".add_v_proj.")}
    # Qwen-Image: diffusers stores attn.to_out.0
    cfg = oq.tiny_config()
    flat = oq.init_params(cfg, seed=3, bias_std=0.02)
    stored = {k.replace(".attn.to_out.", ".attn.to_out.0."): v for k, v in _split_qkv(flat, list(joint), joint).items()}
    m = QwenImageTransformer2DModel(in_channels=cfg.in_channels, out_channels=cfg.out_channels,
                                    num_layers=cfg.num_layers, attention_head_dim=cfg.head_dim,
                                    num_attention_heads=cfg.num_heads, joint_attention_dim=cfg.joint_attention_dim,
                                    axes_dims_rope=cfg.axes_dims_rope)
    loaded = m.load_weights(stored.items())
    assert set(stored) <= loaded
    for k, p in m.named_parameters():
        assert torch.equal(p, flat[k]), k
    # Flux
    fcfg = ofx.tiny_config()
    fflat = ofx.init_params(fcfg, seed=4, bias_std=0.02)
    fm = FluxTransformer2DModel(in_channels=fcfg.in_channels, out_channels=fcfg.out_channels,
                                num_layers=fcfg.num_layers, num_single_layers=fcfg.num_single_layers,
                                attention_head_dim=fcfg.head_dim, num_attention_heads=fcfg.num_heads,
                                joint_attention_dim=fcfg.joint_attention_dim,
                                pooled_projection_dim=fcfg.pooled_projection_dim, axes_dims_rope=fcfg.axes_dims_rope)
    fm.load_weights(_split_qkv(fflat, list(joint), joint).items())
    for k, p in fm.named_parameters():
        assert torch.equal(p, fflat[k]), k
    # Wan: only attn1 is fused; ffn.net.N and the top-level scale_shift_table are renamed; extras are skipped
    wcfg = ow.tiny_config()
    wflat = ow.init_params(wcfg, seed=5, bias_std=0.02, norm_jitter=0.1)
    a1 = {".attn1.to_qkv.": (".attn1.to_q.", ".attn1.to_k.", ".attn1.to_v.")}
    wstored = {}
    for k, v in _split_qkv(wflat, list(a1), a1).items():
        k = k.replace(".ffn.net_0.", ".ffn.net.0.").replace(".ffn.net_2.", ".ffn.net.2.")
        k = k.replace(".to_out.", ".to_out.0.")
        if k == "output_scale_shift_prepare.scale_shift_table":
            k = "scale_shift_table"
        wstored[k] = v
    wstored["not.a.parameter"] = torch.zeros(1)
    wm = WanTransformer3DModel(patch_size=wcfg.patch_size, num_attention_heads=wcfg.num_heads,
                               attention_head_dim=wcfg.head_dim, in_channels=wcfg.in_channels,
                               out_channels=wcfg.out_channels, text_dim=wcfg.text_dim, ffn_dim=wcfg.ffn_dim,
                               num_layers=wcfg.num_layers, rope_max_seq_len=wcfg.rope_max_seq_len)
    loaded = wm.load_weights(wstored.items())
    assert "not.a.parameter" not in loaded
    for k, p in wm.named_parameters():
        assert torch.equal(p, wflat[k]), k
    # a shard of the wrong size is an error, not a silent partial copy
    with pytest.raises(ValueError):
        m.load_weights([("transformer_blocks.0.attn.to_q.weight", torch.zeros(3, cfg.dim))])
    with pytest.raises(KeyError):
        m.load_weights([("transformer_blocks.0.nothing.weight", torch.zeros(1))])


# ------------------------------------------------------------------------------ vLLM-Omni plugin
def _stub_vllm_omni(monkeypatch):
    """A stand-in for the four reference modules the plugin touches, with the interfaces they have there:
    a closed enum + override registry (attention/backends/registry.py:38-152), ``register_extractor``
    (cache/teacache/extractors.py:585-615) and the two CustomOp classes."""
    import enum
    import sys
    import types

    import torch.nn as nn

    class DiffusionAttentionBackendEnum(enum.Enum):
        FLASH_ATTN = "vllm_omni.diffusion.attention.backends.flash_attn.FlashAttentionBackend"
        TORCH_SDPA = "vllm_omni.diffusion.attention.backends.sdpa.SDPABackend"
        SAGE_ATTN = "vllm_omni.diffusion.attention.backends.sage_attn.SageAttentionBackend"

    overrides, extractors = {}, {}

    def register_diffusion_backend(backend, class_path=None):
        assert isinstance(backend, DiffusionAttentionBackendEnum) and class_path
        overrides[backend] = class_path
        return lambda x: x

    class AdaLayerNorm(nn.Module):
        def forward_hip(self, x, mod_params, index=None):
            raise AssertionError("reference path")

    class RotaryEmbedding(nn.Module):
        def forward_hip(self, x, cos, sin):
            raise AssertionError("reference path")

    tree = {
        "vllm_omni": {}, "vllm_omni.diffusion": {}, "vllm_omni.diffusion.attention": {},
        "vllm_omni.diffusion.attention.backends": {},
        "vllm_omni.diffusion.attention.backends.registry": {
            "DiffusionAttentionBackendEnum": DiffusionAttentionBackendEnum,
            "register_diffusion_backend": register_diffusion_backend},
        "vllm_omni.diffusion.cache": {}, "vllm_omni.diffusion.cache.teacache": {},
        "vllm_omni.diffusion.cache.teacache.extractors": {
            "register_extractor": lambda name, fn: extractors.__setitem__(name, fn)},
        "vllm_omni.diffusion.layers": {},
        "vllm_omni.diffusion.layers.adalayernorm": {"AdaLayerNorm": AdaLayerNorm},
        "vllm_omni.diffusion.layers.rope": {"RotaryEmbedding": RotaryEmbedding},
    }
    for name, attrs in tree.items():
        mod = types.ModuleType(name)
        mod.__path__ = []
        for k, v in attrs.items():
            setattr(mod, k, v)
        monkeypatch.setitem(sys.modules, name, mod)
    return DiffusionAttentionBackendEnum, overrides, extractors, AdaLayerNorm, RotaryEmbedding


def test_plugin_needs_vllm_omni():
    import sys

    from vllm_omni_amd import plugin

    assert "vllm_omni" not in sys.modules
    with pytest.raises(ImportError, match="vllm-omni"):
        plugin.register()


def test_plugin_registers_backend_layers_and_extractor(monkeypatch):
    import importlib

    from vllm_omni_amd import plugin, torch_ops
    from vllm_omni_amd.cache.teacache.extractors import extract_flux_context

    E, overrides, extractors, AdaLN, Rope = _stub_vllm_omni(monkeypatch)
    plugin.register()
    plugin.register()  # loaded once per process at least; twice must be harmless
    assert overrides == {E.FLASH_ATTN: plugin.BACKEND_PATH, E.TORCH_SDPA: plugin.BACKEND_PATH}
    mod, cls = plugin.BACKEND_PATH.rsplit(".", 1)
    backend = getattr(importlib.import_module(mod), cls)   # how the reference's selector resolves it
    assert backend.get_name() == "HIP_FLASH_ATTN" and backend.supports_attention_mask()
    assert backend.supports_head_size(128) and not backend.supports_head_size(96)
    impl = backend.get_impl_cls()(num_heads=4, head_size=64, softmax_scale=0.125, causal=False, num_kv_heads=4)
    assert type(impl).forward_hip is torch_ops.attention_forward_hip
    assert AdaLN.forward_hip is torch_ops.adaln_forward_hip and Rope.forward_hip is torch_ops.rope_forward_hip
    assert extractors == {"FluxTransformer2DModel": extract_flux_context}
    with pytest.raises(TypeError, match="FluxTransformer2DModel"):
        extract_flux_context(type("Other", (), {"transformer_blocks": [0]})(), None)


def test_custom_ops_trace_with_fake_tensors():
    """Shape propagation of the three ops without any device: what torch.compile's tracer sees."""
    from torch._subclasses.fake_tensor import FakeTensorMode

    from vllm_omni_amd import torch_ops  # noqa: F401  (defines torch.ops.omni_dit)

    with FakeTensorMode():
        q = torch.empty(2, 70, 4, 64, dtype=torch.bfloat16, device="cuda")
        k = torch.empty(2, 90, 4, 64, dtype=torch.bfloat16, device="cuda")
        o = torch.ops.omni_dit.attention(q, k, k, 0.125, torch.ones(2, 90, dtype=torch.bool, device="cuda"))
        assert o.shape == q.shape and o.dtype == q.dtype and o.device.type == "cuda"
        x = torch.empty(2, 70, 256, dtype=torch.bfloat16, device="cuda")
        m = torch.empty(2, 256, dtype=torch.bfloat16, device="cuda")
        assert torch.ops.omni_dit.adaln_modulate(x, m, m, 1e-6).shape == x.shape
        t = torch.empty(70, 32, device="cuda")
        assert torch.ops.omni_dit.rotary(q, t, t, False).shape == q.shape


def test_models_take_the_reference_constructor_calls():
    """Pipelines build ``Model(od_config=od_config, **transformer_kwargs)`` (pipeline_qwen_image_edit.py:253):
    the config object is accepted, a parallel degree above one is refused, Wan exposes ``.config``."""
    from types import SimpleNamespace as NS

    from vllm_omni_amd.blocks.flux import FluxTransformer2DModel
    from vllm_omni_amd.blocks.qwen_image import QwenImageTransformer2DModel
    from vllm_omni_amd.blocks.wan import WanTransformer3DModel

    one = NS(parallel_config=NS(tensor_parallel_size=1, sequence_parallel_size=None, ulysses_degree=1, ring_degree=1,
                                cfg_parallel_size=1), tf_model_config=NS(num_layers=1))
    tiny = dict(num_layers=2, attention_head_dim=64, num_attention_heads=2, joint_attention_dim=32)
    m = QwenImageTransformer2DModel(od_config=one, zero_cond_t=True, use_additional_t_cond=True, use_layer3d_rope=True,
                                    guidance_embeds=False, quant_config=None, **tiny)
    assert m.parallel_config is one.parallel_config and len(m.transformer_blocks) == 2
    assert m.dtype == torch.float32 and m.in_channels == 64 and m.guidance_embeds is False and m.do_true_cfg is False
    assert m.time_text_embed.addition_t_embedding.weight.shape == (2, 128) and m.pos_embed.layer3d
    f = FluxTransformer2DModel(od_config=one, num_single_layers=1, pooled_projection_dim=16, **tiny)
    assert len(f.transformer_blocks) == 1   # tf_model_config.num_layers wins, as in the reference
    assert f.dtype == torch.float32 and f.guidance_embeds is True
    two = NS(parallel_config=NS(tensor_parallel_size=1, ulysses_degree=2))
    for cls in (QwenImageTransformer2DModel, FluxTransformer2DModel):
        with pytest.raises(NotImplementedError, match="ulysses_degree"):
            cls(od_config=two, **tiny)
    with pytest.raises(NotImplementedError, match="quantised"):
        QwenImageTransformer2DModel(quant_config=object(), **tiny)
    w = WanTransformer3DModel(num_attention_heads=2, attention_head_dim=64, ffn_dim=64, num_layers=1, text_dim=32)
    assert w.config.patch_size == (1, 2, 2) and w.config.num_layers == 1 and w.config.image_dim is None


# ------------------------------------------------------- cache backends, after the reference's own tests
def test_cache_backend_and_selector_like_the_reference_tests(monkeypatch):
    """tests/diffusion/cache/test_cache_backends.py:126-222 of the reference, against this package:
    TeaCacheBackend init / enable / enable with coefficients / refresh, and the selector."""
    from unittest.mock import Mock

    from vllm_omni_amd.cache.base import DiffusionCacheConfig
    from vllm_omni_amd.cache.selector import get_cache_backend
    from vllm_omni_amd.cache.teacache import backend as backend_mod
    from vllm_omni_amd.cache.teacache.backend import TeaCacheBackend

    backend = TeaCacheBackend(DiffusionCacheConfig(rel_l1_thresh=0.3))
    assert backend.config.rel_l1_thresh == 0.3 and backend.enabled is False and backend.is_enabled() is False

    def pipeline():
        p, t = Mock(), Mock()
        p.__class__.__name__ = "QwenImagePipeline"
        t.__class__.__name__ = "QwenImageTransformer2DModel"
        p.transformer = t
        return p, t

    for cfg in (DiffusionCacheConfig(rel_l1_thresh=0.3),
                DiffusionCacheConfig(rel_l1_thresh=0.3, coefficients=[1.0, 0.5, 0.2, 0.1, 0.05])):
        applied = Mock()
        monkeypatch.setattr(backend_mod, "apply_teacache_hook", applied)
        backend = TeaCacheBackend(cfg)
        p, t = pipeline()
        backend.enable(p)
        assert backend.enabled is True
        applied.assert_called_once()
        module, tc = applied.call_args[0]
        assert module is t and tc.transformer_type == "QwenImageTransformer2DModel" and tc.rel_l1_thresh == 0.3
        assert list(tc.coefficients) == (cfg.coefficients or [-4.5e2, 2.8e2, -4.5e1, 3.2, -2.0e-2])
        assert backend.config is cfg   # the given object stays the backend's config
    # a transformer class without coefficients is a configuration error, reported as ValueError
    p, t = pipeline()
    t.__class__.__name__ = "SomethingElse"
    with pytest.raises(ValueError, match="Invalid TeaCache configuration"):
        TeaCacheBackend(DiffusionCacheConfig()).enable(p)
    # refresh resets the hook through the registry
    p, t = pipeline()
    t._hook_registry = Mock()
    backend = TeaCacheBackend(DiffusionCacheConfig())
    backend.enable(p)
    backend.refresh(p, num_inference_steps=50)
    t._hook_registry.reset_hook.assert_called_once()
    # selector
    assert get_cache_backend(None, None) is None and get_cache_backend("none", None) is None
    b = get_cache_backend("tea_cache", {"rel_l1_thresh": 0.3, "Fn_compute_blocks": 4})
    assert isinstance(b, TeaCacheBackend) and b.config.rel_l1_thresh == 0.3
    with pytest.raises(ValueError, match="Unsupported cache backend"):
        get_cache_backend("invalid_backend", {})
    with pytest.raises(NotImplementedError):
        get_cache_backend("cache_dit", {})
    assert DiffusionCacheConfig.from_dict({}).rel_l1_thresh == 0.2


# ----------------------------------------------------------------------------------- CFG mixin
class _RowMixer(torch.nn.Module):
    """A per-sample token mixer (softmax over a sample's own positions): what one sample yields does
    not depend on which other samples share its batch, as for a DiT."""

    def __init__(self, channels: int = 4, width: int = 128, seed: int = 42):
        super().__init__()
        g = torch.Generator().manual_seed(seed)
        self.w_in = torch.nn.Parameter(torch.randn(channels, width, generator=g) * 0.3)
        self.w_qk = torch.nn.Parameter(torch.randn(width, width, generator=g) * 0.1)
        self.w_out = torch.nn.Parameter(torch.randn(width, channels, generator=g) * 0.3)

    def forward(self, x: torch.Tensor, **kwargs):
        b, c, h, w = x.shape
        s = x.flatten(2).transpose(1, 2) @ self.w_in
        p = torch.softmax((s @ self.w_qk) @ s.transpose(1, 2) / s.shape[-1] ** 0.5, dim=-1)
        s = torch.nn.functional.layer_norm(s + p @ s, (s.shape[-1],))
        return ((s @ self.w_out).transpose(1, 2).reshape(b, c, h, w),)


class _Pipe(denoise.CFGParallelMixin):
    def __init__(self, batch_branches: bool):
        self.transformer = _RowMixer().double().eval()
        self.batch_cfg_branches = batch_branches


@pytest.mark.parametrize("cfg_normalize", [False, True])
def test_predict_noise_maybe_with_cfg_batched_equals_sequential(cfg_normalize):
    """The reference's test of its mixin (tests/diffusion/distributed/test_cfg_parallel.py:293-372: batch 2,
    4 channels, 16x16, width 128, scale 7.5, seeds 42/123, both settings of cfg_normalize) with the one-call
    schedule in the place of the two-rank one; the sequential result is also checked against the formula."""
    x_pos = torch.randn(2, 4, 16, 16, dtype=torch.float64, generator=torch.Generator().manual_seed(123))
    x_neg = torch.randn(2, 4, 16, 16, dtype=torch.float64, generator=torch.Generator().manual_seed(124))
    outs = []
    for batched in (True, False):
        pipe = _Pipe(batched)
        calls = []
        pipe.transformer.register_forward_hook(lambda m, a, kw, o: calls.append(kw["x"].shape[0]), with_kwargs=True)
        with torch.no_grad():
            outs.append(pipe.predict_noise_maybe_with_cfg(True, 7.5, {"x": x_pos}, {"x": x_neg}, cfg_normalize))
        assert calls == ([4] if batched else [2, 2])
    assert outs[0].shape == x_pos.shape
    torch.testing.assert_close(outs[0], outs[1], atol=1e-12, rtol=1e-12)
    with torch.no_grad():
        p, n = pipe.transformer(x=x_pos)[0], pipe.transformer(x=x_neg)[0]
    want = n + 7.5 * (p - n)
    if cfg_normalize:
        want = want * (p.norm(dim=-1, keepdim=True) / want.norm(dim=-1, keepdim=True))
        torch.testing.assert_close(outs[1].norm(dim=-1), p.norm(dim=-1))
    torch.testing.assert_close(outs[1], want, atol=1e-12, rtol=1e-12)


def test_predict_noise_without_cfg():
    """do_true_cfg = False: the positive prediction alone, one call, negative arguments untouched
    (test_cfg_parallel.py:375-431), and output_slice keeps the leading positions of axis 1."""
    pipe = _Pipe(True)
    x = torch.randn(1, 4, 16, 16, dtype=torch.float64, generator=torch.Generator().manual_seed(123))
    with torch.no_grad():
        got = pipe.predict_noise_maybe_with_cfg(False, 7.5, {"x": x}, None)
        want = pipe.transformer(x=x)[0]
        cut = pipe.predict_noise_maybe_with_cfg(False, 7.5, {"x": x}, None, output_slice=3)
    assert torch.equal(got, want) and torch.equal(cut, want[:, :3])


def test_batch_cfg_kwargs_pads_and_masks_prompts():
    lat = torch.randn(1, 6, 8)
    pos = {"hidden_states": lat, "timestep": torch.tensor([0.5]), "guidance": None,
           "encoder_hidden_states": torch.randn(1, 5, 3), "encoder_hidden_states_mask": None,
           "img_shapes": [[(1, 2, 3)]], "txt_seq_lens": [5], "return_dict": False}
    neg = dict(pos, encoder_hidden_states=torch.randn(1, 2, 3), txt_seq_lens=[2])
    both = denoise.batch_cfg_kwargs(pos, neg)
    assert both["hidden_states"].shape == (2, 6, 8) and torch.equal(both["hidden_states"][1], lat[0])
    assert both["timestep"].tolist() == [0.5, 0.5] and both["guidance"] is None and both["return_dict"] is False
    assert both["img_shapes"] == [[(1, 2, 3)], [(1, 2, 3)]] and both["txt_seq_lens"] == [5, 5]
    text, mask = both["encoder_hidden_states"], both["encoder_hidden_states_mask"]
    assert text.shape == (2, 5, 3) and torch.equal(text[1, :2], neg["encoder_hidden_states"][0])
    assert torch.count_nonzero(text[1, 2:]) == 0
    assert mask.tolist() == [[True] * 5, [True, True, False, False, False]]
    # equal lengths and no masks: nothing to mask
    same = denoise.batch_cfg_kwargs(pos, dict(pos))
    assert same["encoder_hidden_states_mask"] is None and same["img_shapes"] == [[(1, 2, 3)]] * 2
    # a given mask is kept and extended by the padding
    neg_m = dict(neg, encoder_hidden_states_mask=torch.tensor([[1, 0]]))
    assert denoise.batch_cfg_kwargs(pos, neg_m)["encoder_hidden_states_mask"][1].tolist() == [True, False, False, False, False]
    # what cannot be stacked is left to two calls
    assert denoise.batch_cfg_kwargs(pos, dict(pos, hidden_states=torch.randn(1, 7, 8))) is None
    assert denoise.batch_cfg_kwargs(pos, dict(pos, return_dict=True)) is None
    assert denoise.batch_cfg_kwargs(pos, {"hidden_states": lat}) is None


def test_flow_match_scheduler_follows_the_sigma_table():
    n, s_img = 9, 1024
    sched = denoise.FlowMatchEulerScheduler()
    sched.set_timesteps(sigmas=np.linspace(1.0, 1.0 / n, n), mu=denoise.calculate_shift(s_img))
    sig = denoise.flow_match_sigmas(n, s_img)
    np.testing.assert_allclose(sched.sigmas, sig, rtol=1e-6)
    np.testing.assert_allclose(sched.timesteps.numpy(), sig[:-1] * 1000, rtol=1e-6)
    x = torch.randn(1, 5, 4, generator=torch.Generator().manual_seed(2))
    want = x.clone()
    sched.set_begin_index(0)
    for i, t in enumerate(sched.timesteps):
        v = torch.full_like(x, float(i + 1))
        x = sched.step(v, t, x, return_dict=False)[0]
        want = want + (float(sig[i + 1]) - float(sig[i])) * v
    torch.testing.assert_close(x, want)
    # constant velocity: the steps telescope to x0 - sigma_0 v
    sched.set_begin_index(0)
    y = torch.zeros(3)
    for t in sched.timesteps:
        y = sched.step(torch.ones(3), t, y, return_dict=False)[0]
    torch.testing.assert_close(y, torch.full((3,), -1.0))


def test_qwen_mixin_diffuse_feeds_the_transformer_like_the_reference():
    """Arguments per step (cfg_parallel.py:86-123 of the reference's qwen_image package): timestep / 1000 in
    the latent dtype, latents joined with the image latents on axis 1 and the prediction cut back to the
    latents' length, scheduler restarted at index 0."""
    seen = []

    class Net(torch.nn.Module):
        def forward(self, hidden_states, timestep, encoder_hidden_states, **kw):
            seen.append((hidden_states.shape, timestep.clone(), encoder_hidden_states.shape, kw))
            return (hidden_states * 0 + encoder_hidden_states.mean(dim=(1, 2), keepdim=True),)

    class Pipe(denoise.QwenImageCFGParallelMixin):
        pass

    pipe = Pipe()
    pipe.transformer, pipe.scheduler = Net(), denoise.FlowMatchEulerScheduler()
    pipe.scheduler.set_timesteps(3)
    pipe.scheduler.set_begin_index(2)
    lat, cond = torch.zeros(1, 4, 2), torch.ones(1, 3, 2)
    pos, neg = torch.full((1, 5, 2), 2.0), torch.full((1, 2, 2), -1.0)
    out = pipe.diffuse(pos, None, neg, None, lat, [[(1, 2, 2), (1, 1, 3)]], [5], [2], pipe.scheduler.timesteps,
                       True, None, 2.0, image_latents=cond, cfg_normalize=False,
                       additional_transformer_kwargs={"return_dict": False})
    assert len(seen) == 3 and pipe.transformer.do_true_cfg is True
    shape, t, tshape, kw = seen[0]
    assert shape == (2, 7, 2) and tshape == (2, 5, 2) and t.tolist() == [1.0, 1.0]
    assert kw["txt_seq_lens"] == [5, 5] and kw["return_dict"] is False and kw["guidance"] is None
    assert kw["encoder_hidden_states_mask"].sum(dim=1).tolist() == [5, 2]
    assert out.shape == lat.shape
    # velocity per branch: mean of the (padded) prompt = 2 and -2/5; combined -0.4 + 2 * 2.4 = 4.4; sum of dsigma = -1
    torch.testing.assert_close(out, torch.full_like(lat, -4.4))


def test_profile_records_name_the_launches_they_were_measured_on():
    """bench.py quotes HBM traffic and matrix-pipe counters from profiles/*.txt only for the launch plan those
    files were measured on (vllm_omni_amd/profiling.py)."""
    from vllm_omni_amd import profiling

    traffic = profiling.read_record(profiling.TRAFFIC_FILE)
    counters = profiling.read_record(profiling.COUNTERS_FILE)
    plan = traffic["attention_plan"]
    assert plan == counters["attention_plan"] and "attn_fwd_dma_kernel<T, 128, 8, 0>" in plan
    fig = profiling.attention_figures(plan)
    assert fig["traffic_bytes"] == traffic["traffic_bytes"] > 213.9e6          # at least the algorithmic bytes
    assert 0.3 < fig["mfma_busy_frac"] < 1.0 and 1000 < fig["clock_MHz"] < 2500
    assert "attn_fwd_dma_kernel" in fig["profiled_kernel"]
    with pytest.raises(RuntimeError, match="re-run the counter passes"):
        profiling.attention_figures(plan.replace("units=768", "units=769"))
    assert profiling._plan_kernels(plan) == ["attn_fwd_dma_kernel<T, 128, 8, 0>", "attn_fwd_dma_kernel<T, 128, 8, 1>",
                                             "attn_merge_kernel<T, 128, 256>"]
    assert profiling._is_kernel("attn_merge_kernel<T, 128, 256>", "void odit::attn_merge_kernel<odit::bf16_t, 128, 256>(odit::AttnParams, int)")
    assert not profiling._is_kernel("attn_fwd_dma_kernel<T, 128, 8, 1>", "void odit::attn_fwd_dma_kernel<odit::bf16_t, 128, 8, 0>(odit::AttnParams)")
