"""CPU oracle for the DiT transformer-block hot path — TEST INFRASTRUCTURE ONLY.

A clean-room, plain-PyTorch restatement (CPU, fp32 or the tensor dtype, one torch op per reference op,
same dtype casts) of the reference's torch path for the per-step DiT block forward. Only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may import this package, and
only as the checker or the timed CPU baseline; the product package never does.

The reference (Flink-ddd/vllm-omni) is pure Python and cannot be imported where this runs (vllm and
diffusers are absent), so there is no compiled ``oracle/_ref``. Each function cites the reference
lines it follows. How each function is pinned independently of its own formula (closed forms,
library routines, brute force, invariants) is listed in ``tests/test_oracle_*.py``.

Parity status of arithmetic that lives in third-party wheels absent from the reference tree
(**parity unpinned** at that boundary — upstream conventions adopted, not verifiable here):
  * ``rms_norm_head``      vllm RMSNorm cast order (fp32 normalise -> cast -> x weight); vllm==0.16.0 / 0.14.0+rocm700
  * ``ada_layer_norm_continuous``, ``timestep_embedding`` + ``TimestepEmbedding`` MLP,
    ``flow_match_euler_step`` / sigma shifting    diffusers>=0.36.0 (AdaLayerNormContinuous chunk
    order scale,shift; FlowMatchEulerDiscreteScheduler). The sinusoid of ``timestep_embedding`` is pinned
    by closed forms and, in its ``cast_freqs`` form, follows the in-tree function at
    pipeline_qwen_image.py:141-190; that the transformers' ``Timesteps`` keeps fp32 frequencies is the
    upstream convention.
  * Flux: ``AdaLayerNormZero`` / ``AdaLayerNormZeroSingle`` chunk orders, the combined
    timestep/guidance/pooled-text embedding, ``get_1d_rotary_pos_embed``; Wan: ``FP32LayerNorm``,
    ``PixArtAlphaTextProjection`` (diffusers>=0.36.0; see ``oracle/flux.py``, ``oracle/wan.py``).
The reference tree itself restates three of these conventions in code of other models, which is what the
oracle's choice is checked against (``tests/test_oracle_heads.py``):
  * vllm_omni/model_executor/models/qwen3_tts/modeling_qwen3_tts.py:584-598 (``Qwen3TTSRMSNorm``):
    fp32 normalise, cast to the input dtype, THEN multiply by the weight — the cast order of ``rms_norm_head``;
  * .../qwen3_tts/tokenizer_25hz/modeling_qwen3_tts_tokenizer_v1.py:473-488 (``AdaLayerNormZero``):
    chunk(6) = shift_msa, scale_msa, gate_msa, shift_mlp, scale_mlp, gate_mlp, LN(x)(1 + scale_msa) + shift_msa;
  * same file :492-507 (``AdaLayerNormZero_Final``): chunk(2) = scale, shift, LN(x)(1 + scale) + shift — the
    order of ``ada_layer_norm_continuous``.
Everything else (attention, interleaved/NeoX rotary, AdaLayerNorm, gated residual, rel-L1, TeaCache
decision logic, Qwen rope tables, block wiring, CFG combine) follows code present in the reference.
"""
