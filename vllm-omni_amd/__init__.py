"""MI355X-native kernels for the per-step DiT transformer-block forward of vLLM-Omni's diffusion
stack, behind the reference's own attention-backend / CustomOp / TeaCache interfaces.

Layout
  csrc/                 HIP kernels + the C ABI (include/omni_dit.h), built into libomni_dit_hip.so
  _lib.py, kernels.py   ctypes binding and tensor-level wrappers
  platforms.py          the one platform this package targets (ROCm, gfx950)
  attention/            AttentionBackend / AttentionImpl / Attention layer, backend registry + selector
  layers/               CustomOp, AdaLayerNorm, RotaryEmbedding, RMSNorm
  hooks/, cache/        HookRegistry / ModelHook and the TeaCache hook, state, config, extractors
  blocks/               Qwen-Image dual-stream block and transformer composed from the kernels
  denoise.py            CFG-batched flow-matching Euler loop that drives the transformer
"""

__version__ = "0.1.0"
