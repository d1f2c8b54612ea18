"""Headline benchmark: denoise steps/s of the Qwen-Image-shape MMDiT at 1024x1024 on one MI355X.

One "step" = one CFG-batched (B=2) transformer forward — stem, 60 dual-stream blocks, head — plus the
CFG combine and the Euler update, on synthetic inputs already resident in HBM. Prints ONE JSON line:
steps/s, the attention kernel's live-measured roofline fraction (bf16 MFMA), per-kernel GB/s and
TFLOP/s for the other kernels on the path, and the CPU oracle timed on the host cores.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--blocks N] [--no-cpu] [--no-kernels] [--no-in-step] [--no-teacache]
  python bench.py --workload flux|wan [--steps K] [--warmup W]     (the other block families, same protocol)
  python bench.py --workload flux --teacache 0.25                  (adds the 28-step TeaCache trajectory: skip rate, steps/s)
"""

from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_MFMA_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA, vendor figure
PEAK_HBM_GBS = 8000.0            # MI355X HBM3E, vendor figure
# HBM traffic, MFMA-busy share and in-kernel clock of the attention call come from the committed counter
# summaries under profiles/ (vllm_omni_amd.profiling.attention_figures), which name the launches they were
# measured on: a build that dispatches other launches for the headline shape makes bench.py stop.

# Qwen-Image shape at 1024x1024 (BASELINE.json configs[2])
LAYERS, HEADS, HEAD_DIM, MLP_RATIO = 60, 24, 128, 4
C = HEADS * HEAD_DIM
S_IMG, S_TXT, TEXT_DIM, IN_CH = 4096, 256, 3584, 64
IMG_SHAPE = (1, 64, 64)
B = 2


def _events(torch):
    return torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)


def _time_op(torch, fn, iters=20, warmup=3):
    """Average duration (ms) of fn() from HIP events on the current stream."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    a, b = _events(torch)
    a.record()
    for _ in range(iters):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / iters


class AttnTimer:
    """Brackets every attention launch of the timed region with HIP events on the launch stream."""

    def __init__(self, torch, kernels):
        self.torch, self.kernels = torch, kernels
        self.orig = kernels.attn_fwd
        self.pairs = []
        self.flops = []
        self.active = False

    def __enter__(self):
        def timed(*a, **kw):
            if not self.active:
                return self.orig(*a, **kw)
            s, e = _events(self.torch)
            s.record()
            out = self.orig(*a, **kw)
            e.record()
            q, k = a[0], a[1]
            self.pairs.append((s, e))
            self.flops.append(4.0 * q.shape[0] * q.shape[2] * q.shape[1] * k.shape[1] * q.shape[3])
            return out

        self.kernels.attn_fwd = timed
        return self

    def __exit__(self, *exc):
        self.kernels.attn_fwd = self.orig

    def mean_ms(self):
        return sum(s.elapsed_time(e) for s, e in self.pairs) / max(len(self.pairs), 1)

    def dominant(self):
        """(mean ms, flop per launch, launches) of the launches with the largest flop count."""
        top = max(self.flops)
        ms = [s.elapsed_time(e) for (s, e), f in zip(self.pairs, self.flops) if f == top]
        return sum(ms) / len(ms), top, len(ms)


class StepKernelTimer:
    """HIP-event brackets around the hand-written kernels and the GEMMs of whole denoise steps run AFTER the timed
    region (same process, chip in the state the timed steps left it in): what each kernel achieves on the data
    the step hands it, as opposed to the rotating-buffer microbenchmarks of ``kernel_rooflines``. The brackets
    cost a few microseconds each, which is why they stay out of the timed steps."""

    def __init__(self, torch, kernels):
        self.torch, self.kernels = torch, kernels
        self.records = {}   # label -> [events..., work, unit]
        self.saved = []

    def _bracket(self, label, work, unit, fn, a, kw):
        s, e = _events(self.torch)
        s.record()
        out = fn(*a, **kw)
        e.record()
        rec = self.records.setdefault(label, {"pairs": [], "work": work, "unit": unit})
        rec["pairs"].append((s, e))
        return out

    def __enter__(self):
        k, F = self.kernels, self.torch.nn.functional
        esz = lambda t: t.element_size()  # noqa: E731

        def adaln_pair(first, second, **kw):
            byt = sum(2 * p[0].numel() * esz(p[0]) for p in (first, second))
            return self._bracket("adaln_modulate_pair(img+txt)", byt, "B", orig["adaln_modulate_pair"], (first, second), kw)

        def qknorm_pair(first, second, q_out, k_out, v_out, **kw):
            byt = sum(2 * (p[0].numel() + (p[1].numel() if p[1] is not None else 0) +
                           (p[2].numel() if p[2] is not None else 0)) * esz(p[0]) for p in (first, second))
            return self._bracket("qknorm_rope_pair(img+txt)", byt, "B", orig["qknorm_rope_pair"],
                                 (first, second, q_out, k_out, v_out), kw)

        def linear(x, weight, bias=None, **kw):
            if kw.get("plan_only") or kw.get("tune_iters"):
                return orig["linear"](x, weight, bias, **kw)
            M, (N, K) = x.numel() // x.shape[-1], weight.shape
            plan_kw = {a: b for a, b in kw.items() if a != "out"}
            own = orig["linear"](x, weight, bias, plan_only=True, **plan_kw)[0]
            tail = "gelu" if kw.get("activation") else ("gated_residual" if kw.get("residual") is not None else "bias")
            label = f"linear {M}x{N}x{K} {tail} [{'hand-written' if own else 'hipBLASLt'}]"
            return self._bracket(label, 2.0 * M * N * K, "FLOP", orig["linear"], (x, weight, bias), kw)

        def f_linear(x, weight, bias=None):
            M, (N, K) = x.numel() // x.shape[-1], weight.shape
            if M * N * K < 1 << 30:
                return orig["F.linear"](x, weight, bias)
            return self._bracket(f"torch linear {M}x{N}x{K} [hipBLASLt]", 2.0 * M * N * K, "FLOP", orig["F.linear"],
                                 (x, weight, bias), {})

        def attn(*a, **kw):
            q, kk = a[0], a[1]
            fl = 4.0 * q.shape[0] * q.shape[2] * q.shape[1] * kk.shape[1] * q.shape[3]
            return self._bracket(f"attn_fwd B={q.shape[0]} S={q.shape[1]}x{kk.shape[1]} {q.shape[2]}x{q.shape[3]}", fl, "FLOP",
                                 orig["attn_fwd"], a, kw)

        orig = {"adaln_modulate_pair": k.adaln_modulate_pair, "qknorm_rope_pair": k.qknorm_rope_pair,
                "linear": k.linear, "attn_fwd": k.attn_fwd, "F.linear": F.linear}
        self.saved = [(k, "adaln_modulate_pair", k.adaln_modulate_pair), (k, "qknorm_rope_pair", k.qknorm_rope_pair),
                      (k, "linear", k.linear), (k, "attn_fwd", k.attn_fwd), (F, "linear", F.linear)]
        k.adaln_modulate_pair, k.qknorm_rope_pair, k.linear, k.attn_fwd, F.linear = adaln_pair, qknorm_pair, linear, attn, f_linear
        return self

    def __exit__(self, *exc):
        for mod, name, fn in self.saved:
            setattr(mod, name, fn)

    def report(self, steps):
        out = {}
        for label, rec in self.records.items():
            us = [s.elapsed_time(e) * 1e3 for s, e in rec["pairs"]]
            mean = sum(us) / len(us)
            row = {"calls_per_step": len(us) / steps, "avg_us": mean, "ms_per_step": sum(us) / steps / 1e3}
            if rec["unit"] == "B":
                row["GB/s"] = rec["work"] / mean / 1e3
                row["frac_hbm"] = row["GB/s"] / PEAK_HBM_GBS
                row["algorithmic_bytes"] = rec["work"]
            else:
                row["TFLOP/s"] = rec["work"] / mean / 1e6
                row["frac_mfma"] = row["TFLOP/s"] / PEAK_MFMA_BF16_TFLOPS
            out[label] = row
        return dict(sorted(out.items(), key=lambda kv: -kv[1]["ms_per_step"]))


def max_engine_clock_mhz():
    """Highest 'Max Clock Freq. (MHz)' that rocminfo lists for a GPU agent, or None when it cannot be read."""
    import re
    import subprocess

    try:
        text = subprocess.run(["rocminfo"], capture_output=True, text=True, timeout=30).stdout
    except (OSError, subprocess.SubprocessError):
        return None
    best = None
    for agent in text.split("*******")[1:]:
        if "Device Type:             GPU" in agent or re.search(r"Device Type:\s+GPU", agent):
            m = re.search(r"Max Clock Freq\. \(MHz\):\s+(\d+)", agent)
            if m:
                best = max(best or 0, int(m.group(1)))
    return float(best) if best else None


def build_model(torch, layers, fuse_epilogues=True):
    from vllm_omni_amd.blocks.qwen_image import QwenImageTransformer2DModel

    prev = torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)
    try:
        with torch.device("cuda"):
            model = QwenImageTransformer2DModel(num_layers=layers, attention_head_dim=HEAD_DIM,
                                                num_attention_heads=HEADS, joint_attention_dim=TEXT_DIM,
                                                in_channels=IN_CH, out_channels=16, mlp_ratio=MLP_RATIO,
                                                fuse_epilogues=fuse_epilogues)
    finally:
        torch.set_default_dtype(prev)
    g = torch.Generator(device="cuda").manual_seed(0)
    with torch.no_grad():
        for name, p in model.named_parameters():
            if name.endswith("norm_q.weight") or name.endswith("norm_k.weight") or name == "txt_norm.weight":
                p.fill_(1.0)
            elif name.endswith(".bias"):
                p.zero_()
            else:
                p.normal_(0.0, 0.02, generator=g)
    model.fuse_modulation()
    return model.eval()


def _init_synthetic(torch, model, seed=0):
    g = torch.Generator(device="cuda").manual_seed(seed)
    with torch.no_grad():
        for name, p in model.named_parameters():
            if name.endswith(("norm_q.weight", "norm_k.weight", "norm2.weight", "txt_norm.weight")):
                p.fill_(1.0)
            elif name.endswith(".bias"):
                p.zero_()
            elif name.endswith("scale_shift_table"):
                p.normal_(0.0, p.shape[-1] ** -0.5, generator=g)
            else:
                p.normal_(0.0, 0.02, generator=g)


def flux_workload(torch, layers=None):
    """BASELINE.json configs[4]: Flux shape, 19 dual + 38 single blocks, B=1, 512 text + 4096 image tokens."""
    from vllm_omni_amd.blocks.flux import FluxTransformer2DModel
    from vllm_omni_amd.denoise import euler_step, flow_match_sigmas

    n_dual, n_single = (19, 38) if layers is None else (max(layers // 3, 1), max(layers - layers // 3, 1))
    prev = torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)
    try:
        with torch.device("cuda"):
            model = FluxTransformer2DModel(num_layers=n_dual, num_single_layers=n_single)
    finally:
        torch.set_default_dtype(prev)
    _init_synthetic(torch, model)
    model.fuse_modulation()
    model.eval()
    dev = torch.device("cuda:0")
    g = torch.Generator(device="cuda").manual_seed(1)
    s_txt, side = 512, 64
    lat0 = torch.randn(1, side * side, 64, device=dev, generator=g).bfloat16()
    text = torch.randn(1, s_txt, 4096, device=dev, generator=g).bfloat16()
    pooled = torch.randn(1, 768, device=dev, generator=g).bfloat16()
    ids = torch.zeros(side, side, 3, device=dev)
    ids[..., 1] += torch.arange(side, device=dev)[:, None]
    ids[..., 2] += torch.arange(side, device=dev)[None, :]
    img_ids, txt_ids = ids.reshape(-1, 3), torch.zeros(s_txt, 3, device=dev)
    guidance = torch.full((1,), 3.5, device=dev)
    sig = flow_match_sigmas(28, side * side)

    def step(i, lat):
        t = torch.full((1,), float(sig[i % 28]), device=dev, dtype=torch.bfloat16)
        out = model(hidden_states=lat, encoder_hidden_states=text, pooled_projections=pooled, timestep=t,
                    img_ids=img_ids, txt_ids=txt_ids, guidance=guidance, return_dict=False)[0]
        return euler_step(lat, out, float(sig[i % 28]), float(sig[i % 28 + 1]))

    Cf, S = 3072, s_txt + side * side
    gemm = 2.0 * S * Cf * Cf * (n_dual * (3 + 1 + 8) + n_single * (3 + 4 + 5))
    name = (f"Flux-shape MMDiT denoise step: {n_dual} dual + {n_single} single blocks, hidden 3072, 24 heads x 128, "
            f"{s_txt} text + {side * side} image tokens, batch 1 (guidance-distilled), random weights N(0,0.02)")
    def trajectory(steps):
        """One whole guidance-distilled denoise trajectory of `steps` Euler steps from lat0 (what TeaCache's
        decisions are defined on: every step compares its modulated input with the previous step's)."""
        sg = flow_match_sigmas(steps, side * side)
        lat = lat0
        for i in range(steps):
            t = torch.full((1,), float(sg[i]), device=dev, dtype=torch.bfloat16)
            out = model(hidden_states=lat, encoder_hidden_states=text, pooled_projections=pooled, timestep=t,
                        img_ids=img_ids, txt_ids=txt_ids, guidance=guidance, return_dict=False)[0]
            lat = euler_step(lat, out, float(sg[i]), float(sg[i + 1]))
        return lat

    step.trajectory = trajectory
    return model, step, lat0, name, gemm, (n_dual, n_single) == (19, 38)


def wan_workload(torch, layers=None):
    """BASELINE.json configs[3]: Wan2.1-14B shape, 40 blocks, B=2, 21x30x52 = 32760 video tokens, 512 text tokens."""
    from vllm_omni_amd.blocks.wan import WanTransformer3DModel
    from vllm_omni_amd.denoise import combine_cfg_noise, euler_step

    n = 40 if layers is None else layers
    prev = torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)
    try:
        with torch.device("cuda"):
            model = WanTransformer3DModel(num_layers=n)
    finally:
        torch.set_default_dtype(prev)
    _init_synthetic(torch, model)
    model.eval()
    dev = torch.device("cuda:0")
    g = torch.Generator(device="cuda").manual_seed(1)
    lat0 = torch.randn(1, 16, 21, 60, 104, device=dev, generator=g).bfloat16()
    text = torch.randn(2, 512, 4096, device=dev, generator=g).bfloat16()

    def step(i, lat):
        t = torch.full((2,), 900.0 - 40.0 * i, device=dev)
        out = model(lat.expand(2, -1, -1, -1, -1), t, text, return_dict=False)[0]
        noise = combine_cfg_noise(out[0:1], out[1:2], 5.0, False)
        return euler_step(lat, noise, 1.0 - 0.04 * i, 1.0 - 0.04 * (i + 1))

    Cw, Fw, S, T = 5120, 13824, 32760, 512
    gemm = n * 2.0 * 2 * (S * (3 * Cw * Cw + Cw * Cw + Cw * Cw + Cw * Cw + 2 * Cw * Fw) + T * 2 * Cw * Cw)
    name = (f"Wan2.1-14B-shape video DiT denoise step: {n} blocks, hidden 5120, 40 heads x 128, FFN 13824, "
            "21x30x52 = 32760 video tokens, 512 text tokens, CFG batch 2, random weights N(0,0.02)")
    return model, step, lat0, name, gemm, n == 40


def run_secondary(torch, kernels, args):
    """Flux / Wan shapes: same timing protocol as the headline line, one JSON line, no CPU leg."""
    make = flux_workload if args.workload == "flux" else wan_workload
    model, step, lat, name, gemm_flop, valid = make(torch, None if args.blocks == LAYERS else args.blocks)
    with torch.inference_mode(), AttnTimer(torch, kernels) as timer:
        if args.autotune > 0:
            kernels.set_linear_autotune(args.autotune)
            step(0, lat)
            kernels.set_linear_autotune(0)
        for i in range(args.warmup):
            lat = step(i, lat)
        torch.cuda.synchronize()
        timer.active = True
        t0 = time.perf_counter()
        for i in range(args.warmup, args.warmup + args.steps):
            lat = step(i, lat)
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
        timer.active = False
    assert bool(torch.isfinite(lat.float()).all()), "non-finite latents"
    ms, flop, n = timer.dominant()
    tf = flop / ms / 1e9
    attn_total = sum(timer.flops) / args.steps
    in_step = None
    if not args.no_in_step:   # as for the headline workload: extra steps outside the timed region, kernel by kernel
        n_extra = 1 if args.workload == "wan" else 2
        with torch.inference_mode(), StepKernelTimer(torch, kernels) as kt:
            for i in range(n_extra):
                lat = step(i, lat)
            torch.cuda.synchronize()
        in_step = kt.report(n_extra)
    teacache = None
    if args.teacache is not None:
        if args.workload != "flux":
            sys.exit("bench.py: --teacache is measured at the Flux shape (BASELINE.json configs[4]): use --workload flux")
        teacache = teacache_trajectory(torch, model, step, args.teacache, args.steps / elapsed)
    print(json.dumps({
        "metric": f"DiT denoise steps/s, {args.workload} shape (1 GPU)", "value": args.steps / elapsed,
        "unit": "steps/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": elapsed * 1e3 / args.steps, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic", "config": {"workload": name, "valid": valid},
        "roofline": {"kernel": "attn_fwd (largest attention shape of the step)", "bound": "mfma", "achieved": tf,
                     "peak": PEAK_MFMA_BF16_TFLOPS, "unit": "TFLOP/s", "frac": tf / PEAK_MFMA_BF16_TFLOPS,
                     "traffic": None, "launches_timed": n, "avg_ms": ms, "flop_per_launch": flop},
        "step_flop": {"gemm": gemm_flop, "attention": attn_total,
                      "achieved_TFLOP/s": (gemm_flop + attn_total) / (elapsed / args.steps) / 1e12},
        "teacache": teacache,
        "kernels_in_step": None if in_step is None else {
            "what": "per-kernel averages over extra steps run right after the timed region, each call between its own "
                    "HIP events (not part of `value`)", "kernels": in_step},
    }))


def teacache_trajectory(torch, model, step, thresh, plain_steps_per_s, steps=28, first_trajectory_decisions=None):
    """BASELINE.json configs[4]: the 28-step trajectory with the TeaCache hook on (relative-L1 threshold `thresh`
    on the modulated first-block input, the reference's 4th-order polynomial for this model): one untimed
    trajectory, then the same trajectory timed. Steps/s counts every denoise step, skipped or computed."""
    from vllm_omni_amd.cache.teacache import TeaCacheBackend

    class Pipe:
        transformer = model

    backend = TeaCacheBackend({"rel_l1_thresh": float(thresh)})
    backend.enable(Pipe)
    with torch.inference_mode():
        backend.refresh(Pipe, steps)
        step.trajectory(steps)
        torch.cuda.synchronize()
        if first_trajectory_decisions is not None:
            first_trajectory_decisions.extend(dict(d) for d in TeaCacheBackend.hook_of(Pipe).decisions)
        backend.refresh(Pipe, steps)
        t0 = time.perf_counter()
        lat = step.trajectory(steps)
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
    hook = TeaCacheBackend.hook_of(Pipe)
    decisions = [bool(d["compute"]) for d in hook.decisions]
    margins = [abs(d["acc"] - float(thresh)) for d in hook.decisions if d["rel"] is not None and d["acc"] > 0]
    assert len(decisions) == steps and bool(torch.isfinite(lat.float()).all())
    skipped = decisions.count(False)
    return {"rel_l1_thresh": float(thresh), "steps": steps, "skipped": skipped, "skip_rate": skipped / steps,
            "steps/s": steps / elapsed, "ms_per_step": elapsed * 1e3 / steps, "steps/s_without_cache": plain_steps_per_s,
            "speedup": steps / elapsed / plain_steps_per_s, "compute_pattern": "".join("C" if c else "s" for c in decisions),
            "min_distance_to_threshold": min(margins) if margins else None,
            "data": "synthetic latents, random weights: the skip pattern is this trajectory's, not a trained model's"}


def teacache_flux(torch, kernels):
    """BASELINE.json configs[4] inside the default run: the Flux-shape model (19 dual + 38 single blocks, 512 text +
    4096 image tokens, bf16), 28 Euler steps under the TeaCache hook at threshold 0.25, next to the uncached rate.
    During the untimed first trajectory the operands of the first three relative-L1 reductions are copied to the
    host, and the scalar the hook thresholded is checked, bit for bit, against the reference's own expression
    (vllm_omni/diffusion/cache/teacache/hook.py:214-221) evaluated by torch on the host in the tensors' dtype,
    outside every timed region."""
    model, step, lat0, name, _gemm, valid = flux_workload(torch)
    captured = []
    orig = kernels.rel_l1_sums

    def capturing(cur, prev, **kw):
        if len(captured) < 3:
            captured.append((cur.detach().cpu(), prev.detach().cpu()))
        return orig(cur, prev, **kw)

    with torch.inference_mode():
        lat = lat0
        for i in range(2):
            lat = step(i, lat)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        n_plain = 4
        for i in range(2, 2 + n_plain):
            lat = step(i, lat)
        torch.cuda.synchronize()
        plain = n_plain / (time.perf_counter() - t0)
    kernels.rel_l1_sums = capturing
    try:
        out = teacache_trajectory(torch, model, step, 0.25, plain, first_trajectory_decisions=(first := []))
    finally:
        kernels.rel_l1_sums = orig
    rels = [d["rel"] for d in first if d["rel"] is not None][:len(captured)]
    checks = []
    for (cur, prev), got in zip(captured, rels):
        want = ((cur - prev).abs().mean() / (prev.abs().mean() + 1e-8)).item()
        checks.append({"hook": got, "host": want, "equal": got == want})
    assert checks and all(c["equal"] for c in checks), f"relative-L1 scalars differ from the host expression's: {checks}"
    out["workload"] = name
    out["valid"] = valid
    out["rel_l1_checked_against_host_expression"] = {"decisions": len(checks), "bit_identical": True,
                                                     "values": [c["hook"] for c in checks]}
    del model
    return out


def _time_rot(torch, fns, iters=40, warmup=4):
    """Average duration (ms) of the closures in `fns`, called round-robin: each closure works on its
    own buffers, and together the sets exceed the 256 MB last-level cache, so the figure is HBM
    traffic, not cache hits."""
    n = len(fns)
    for i in range(warmup):
        fns[i % n]()
    torch.cuda.synchronize()
    a, b = _events(torch)
    a.record()
    for i in range(iters):
        fns[i % n]()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / iters


def kernel_rooflines(torch):
    """Achieved GB/s (bandwidth-bound kernels) and TFLOP/s (attention, GEMM) at the config shapes.
    Bytes are the ALGORITHMIC bytes of each kernel (inputs read once + outputs written once)."""
    from vllm_omni_amd import kernels
    from vllm_omni_amd._lib import ODIT_NORM_HEAD

    dev = "cuda"
    bf = torch.bfloat16
    out = {}
    NSET = 8  # 8 x (>= 100 MB) per kernel

    def bw(name, fns, byt):
        ms = _time_rot(torch, fns)
        out[name] = {"ms": ms, "GB/s": byt / ms / 1e6, "frac_hbm": byt / ms / 1e6 / PEAK_HBM_GBS,
                     "algorithmic_bytes": byt}

    xs = [torch.randn(B, S_IMG, C, device=dev, dtype=bf) for _ in range(NSET)]
    ys = [torch.randn(B, S_IMG, C, device=dev, dtype=bf) for _ in range(NSET)]
    os_ = [torch.empty(B, S_IMG, C, device=dev, dtype=bf) for _ in range(NSET)]
    mod = torch.randn(B, 3 * C, device=dev, dtype=bf)
    shift, scale, gate = mod.chunk(3, dim=-1)
    n_el = xs[0].numel()
    bw("adaln_modulate", [lambda i=i: kernels.adaln_modulate(xs[i], shift, scale, out=os_[i]) for i in range(NSET)],
       2 * n_el * 2)
    bw("gated_residual", [lambda i=i: kernels.gated_residual(xs[i], ys[i], gate, out=os_[i]) for i in range(NSET)],
       3 * n_el * 2)
    bw("rel_l1", [lambda i=i: kernels.rel_l1_sums(xs[i], ys[i]) for i in range(NSET)], 2 * n_el * 2)
    # reference point, not a kernel of the path: what a plain device copy of the same 50 MB tensors reaches on
    # this box with the same rotation of buffers (torch's copy kernel; gated residual with a gate of ones is
    # this library's own streaming pass over three such tensors)
    bw("reference_copy_50MB", [lambda i=i: os_[i].copy_(xs[i]) for i in range(NSET)], 2 * n_el * 2)
    del ys
    qkvs = [torch.randn(B, S_IMG, 3, HEADS, HEAD_DIM, device=dev, dtype=bf) for _ in range(NSET)]
    jqs = [[torch.empty(B, S_IMG + S_TXT, HEADS, HEAD_DIM, device=dev, dtype=bf) for _ in range(3)] for _ in range(NSET)]
    w = torch.ones(HEAD_DIM, device=dev, dtype=bf)
    cos = torch.rand(S_IMG, HEAD_DIM // 2, device=dev)
    sin = torch.rand(S_IMG, HEAD_DIM // 2, device=dev)
    # as in the step: q and k are normalised, rotated and written to the joint buffers; v stays where the
    # projection left it (the attention kernel reads it there), so it is no traffic of this kernel
    bw("qknorm_rope",
       [lambda i=i: kernels.qknorm_rope(qkvs[i][:, :, 0], qkvs[i][:, :, 1], None, jqs[i][0], jqs[i][1],
                                        None, w, w, cos, sin, out_seq_offset=S_TXT, norm_mode=ODIT_NORM_HEAD)
        for i in range(NSET)], 2 * (2 * qkvs[0].numel() // 3) * 2)
    bw("qknorm_rope_with_v_copy",
       [lambda i=i: kernels.qknorm_rope(qkvs[i][:, :, 0], qkvs[i][:, :, 1], qkvs[i][:, :, 2], jqs[i][0], jqs[i][1],
                                        jqs[i][2], w, w, cos, sin, out_seq_offset=S_TXT, norm_mode=ODIT_NORM_HEAD)
        for i in range(NSET)], 2 * qkvs[0].numel() * 2)
    del qkvs, jqs, xs, os_
    us = [torch.randn(B * S_IMG, MLP_RATIO * C, device=dev, dtype=bf) for _ in range(4)]
    bw("gelu_tanh", [lambda i=i: kernels.gelu_tanh(us[i], out=us[i]) for i in range(4)], 2 * us[0].numel() * 2)
    del us
    S = S_IMG + S_TXT
    q = torch.randn(B, S, HEADS, HEAD_DIM, device=dev, dtype=bf)
    k, v = torch.randn_like(q), torch.randn_like(q)
    sc = 1.0 / math.sqrt(HEAD_DIM)
    ms = _time_op(torch, lambda: kernels.attn_fwd(q, k, v, sc))
    fl = 4.0 * B * HEADS * S * S * HEAD_DIM
    out["attn_fwd"] = {"ms": ms, "TFLOP/s": fl / ms / 1e9, "frac_mfma": fl / ms / 1e9 / PEAK_MFMA_BF16_TFLOPS}
    # the same launch on constant inputs: the matrix pipe is power-limited, and operand data that does
    # not toggle lets it hold its clock - the difference to the line above is the chip, not the kernel
    q1 = torch.ones_like(q)
    ms1 = _time_op(torch, lambda: kernels.attn_fwd(q1, q1, q1, sc))
    out["attn_fwd_constant_inputs"] = {"ms": ms1, "TFLOP/s": fl / ms1 / 1e9,
                                       "frac_mfma": fl / ms1 / 1e9 / PEAK_MFMA_BF16_TFLOPS}
    del q1
    xm = torch.randn(B * S_IMG, C, device=dev, dtype=bf)
    wm = torch.randn(MLP_RATIO * C, C, device=dev, dtype=bf)
    bm = torch.zeros(MLP_RATIO * C, device=dev, dtype=bf)
    ms = _time_op(torch, lambda: torch.nn.functional.linear(xm, wm, bm))
    fl = 2.0 * xm.shape[0] * C * MLP_RATIO * C
    out["gemm_mlp_up(hipBLASLt)"] = {"ms": ms, "TFLOP/s": fl / ms / 1e9,
                                     "frac_mfma": fl / ms / 1e9 / PEAK_MFMA_BF16_TFLOPS}
    # the text stream's MLP down-projection with its gated residual (M = B * S_TXT rows, one gate vector per
    # batch row) on the hand-written stream-K kernel and on the library, weights rotating so each call reads cold ones
    del xm, wm, bm
    n_w = 8
    xt = torch.randn(B, S_TXT, MLP_RATIO * C, device=dev, dtype=bf)
    wts = [torch.randn(C, MLP_RATIO * C, device=dev, dtype=bf) * 0.02 for _ in range(n_w)]
    bt = torch.zeros(C, device=dev, dtype=bf)
    res, gt = torch.randn(B, S_TXT, C, device=dev, dtype=bf), torch.randn(B, C, device=dev, dtype=bf)
    ot = torch.empty_like(res)
    fl = 2.0 * B * S_TXT * C * MLP_RATIO * C
    for engine, label in (("handwritten", "gemm_text_mlp_down(stream-K, hand-written)"),
                          ("library", "gemm_text_mlp_down(hipBLASLt, one launch per batch row)")):
        ms = _time_rot(torch, [lambda w=w: kernels.linear(xt, w, bt, residual=res, gate=gt, out=ot, engine=engine)
                               for w in wts])
        out[label] = {"ms": ms, "TFLOP/s": fl / ms / 1e9, "frac_mfma": fl / ms / 1e9 / PEAK_MFMA_BF16_TFLOPS}
    del xt, wts, res, ot
    # the image stream's MLP up-projection with its GELU epilogue, hand-written tile kernel against the library,
    # weights rotating (four 75 MB weights and the 201 MB output exceed the last-level cache)
    xm = torch.randn(B * S_IMG, C, device=dev, dtype=bf)
    wms = [torch.randn(MLP_RATIO * C, C, device=dev, dtype=bf) * 0.02 for _ in range(4)]
    bm = torch.zeros(MLP_RATIO * C, device=dev, dtype=bf)
    om = torch.empty(B * S_IMG, MLP_RATIO * C, device=dev, dtype=bf)
    fl = 2.0 * B * S_IMG * C * MLP_RATIO * C
    for engine, label in (("handwritten", "gemm_img_mlp_up_gelu(tile kernel, hand-written)"),
                          ("library", "gemm_img_mlp_up_gelu(hipBLASLt)")):
        ms = _time_rot(torch, [lambda w=w: kernels.linear(xm, w, bm, activation="gelu_tanh", out=om, engine=engine)
                               for w in wms], iters=16)
        out[label] = {"ms": ms, "TFLOP/s": fl / ms / 1e9, "frac_mfma": fl / ms / 1e9 / PEAK_MFMA_BF16_TFLOPS}
    return out


def counter_probe(torch, kernels, dev):
    """Three launches of each kernel of the path at the headline shapes on N(0,1) data, nothing else: short
    enough for a hardware-counter pass (counters serialise the dispatches)."""
    from vllm_omni_amd._lib import ODIT_NORM_HEAD

    bf = torch.bfloat16
    S = S_IMG + S_TXT
    q = torch.randn(B, S, HEADS, HEAD_DIM, device=dev, dtype=bf)
    k, v = torch.randn_like(q), torch.randn_like(q)
    x = torch.randn(B, S_IMG, C, device=dev, dtype=bf)
    y, o = torch.randn_like(x), torch.empty_like(x)
    shift, scale, gate = torch.randn(B, 3 * C, device=dev, dtype=bf).chunk(3, dim=-1)
    qkv = torch.randn(B, S_IMG, 3, HEADS, HEAD_DIM, device=dev, dtype=bf)
    jq, jk = torch.empty_like(q), torch.empty_like(q)
    w = torch.ones(HEAD_DIM, device=dev, dtype=bf)
    cos, sin = torch.rand(S_IMG, HEAD_DIM // 2, device=dev), torch.rand(S_IMG, HEAD_DIM // 2, device=dev)
    x2 = x.view(B * S_IMG, C)
    w_up = torch.randn(MLP_RATIO * C, C, device=dev, dtype=bf) * 0.02
    b_up = torch.zeros(MLP_RATIO * C, device=dev, dtype=bf)
    w_qkv = torch.randn(3 * C, C, device=dev, dtype=bf) * 0.02
    b_qkv = torch.zeros(3 * C, device=dev, dtype=bf)
    # text stream's MLP down-projection with its gated residual (the hand-written stream-K GEMM)
    t_in = torch.randn(B, S_TXT, MLP_RATIO * C, device=dev, dtype=bf)
    t_res = torch.randn(B, S_TXT, C, device=dev, dtype=bf)
    w_dn = torch.randn(C, MLP_RATIO * C, device=dev, dtype=bf) * 0.02
    g32 = torch.randn(B, C, device=dev)
    assert kernels.linear(t_in, w_dn, None, residual=t_res, gate=g32, gate_bias=g32 * 0.1, prescaled=True, plan_only=True)[0]
    for _ in range(3):
        kernels.attn_fwd(q, k, v, 1.0 / math.sqrt(HEAD_DIM))
        kernels.qknorm_rope(qkv[:, :, 0], qkv[:, :, 1], None, jq, jk, None, w, w, cos, sin, out_seq_offset=S_TXT,
                            norm_mode=ODIT_NORM_HEAD)
        kernels.adaln_modulate(x, shift, scale, out=o)
        kernels.gated_residual(x, y, gate, out=o)
        kernels.rel_l1_sums(x, y)
        kernels.linear(x2, w_up, b_up, activation="gelu_tanh")
        kernels.linear(x2, w_up, b_up, activation="gelu_tanh", engine="handwritten")   # the tile kernel on the same problem
        torch.nn.functional.linear(x2, w_qkv, b_qkv)
        kernels.linear(t_in, w_dn, None, residual=t_res, gate=g32, gate_bias=g32 * 0.1, prescaled=True)
    torch.cuda.synchronize()
    print(json.dumps({"probe": "attention, qknorm+rope, adaLN, gated residual, rel-L1, MLP-up GEMM (GELU epilogue), "
                               "QKV GEMM, text MLP-down GEMM (stream-K, gated residual) at the Qwen-Image shape, 3 launches each",
                      "attention_plan": kernels.attn_plan(B, S, S, HEADS, HEAD_DIM),
                      "text_mlp_down_flop": 2.0 * B * S_TXT * C * MLP_RATIO * C,
                      "attention_flop": 4.0 * B * HEADS * S * S * HEAD_DIM,
                      "mlp_up_flop": 2.0 * B * S_IMG * C * MLP_RATIO * C, "qkv_flop": 2.0 * B * S_IMG * C * 3 * C}))


def mfma_ceiling(torch):
    """Sustained rate of the bf16 MFMA this path uses with nothing else in the loop, for constant and for
    random operand data (the part is power-limited: the two differ by about 30 %)."""
    import ctypes as C

    from vllm_omni_amd import _lib

    path = _lib.LIB_PATH.with_name("libomni_dit_probe.so")   # a measurement aid, kept out of the product library
    if not path.exists():
        return {"error": f"{path.name} not built"}
    lib = C.CDLL(os.fspath(path))
    lib.odit_probe_mfma.restype = C.c_int
    lib.odit_probe_mfma.argtypes = [C.c_int, C.c_int, C.c_int, C.c_void_p, C.POINTER(C.c_double), C.c_void_p]
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    sink = torch.empty(cus * 512, device="cuda", dtype=torch.float32)
    st = torch.cuda.current_stream().cuda_stream
    out = {}
    for name, rnd in (("constant_operands", 0), ("random_operands", 1)):
        flop = C.c_double(0.0)
        assert lib.odit_probe_mfma(rnd, 2000, cus, sink.data_ptr(), C.byref(flop), st) == 0
        torch.cuda.synchronize()
        best = 0.0
        for _ in range(3):
            a, b = _events(torch)
            a.record()
            assert lib.odit_probe_mfma(rnd, 20000, cus, sink.data_ptr(), C.byref(flop), st) == 0
            b.record()
            torch.cuda.synchronize()
            best = max(best, flop.value / a.elapsed_time(b) / 1e9)
        out[name] = {"TFLOP/s": best, "frac_of_nominal_peak": best / PEAK_MFMA_BF16_TFLOPS}
    return out


def cpu_baseline(torch):
    """The CPU oracle (plain-torch restatement of the reference path) on the host cores: ONE block of
    the 60 at the full B=2 shape, in fp32 and in bf16, the faster of the two extrapolated to a step."""
    from oracle import qwen_image as oq

    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    cfg = oq.QwenConfig(num_layers=1)
    w = oq.init_params(cfg, seed=0, dtype=torch.float32)
    g = torch.Generator().manual_seed(0)
    img = torch.randn(B, S_IMG, C, generator=g)
    txt = torch.randn(B, S_TXT, C, generator=g)
    temb = torch.randn(B, C, generator=g)
    vf, tf = oq.qwen_rope_freqs(cfg, *IMG_SHAPE, txt_len=S_TXT)
    with torch.inference_mode():
        oq.block_forward(w, 0, cfg, img[:, :256], txt, temb, vf[:256], tf)  # page in / warm threads
        reps, t0 = 0, time.perf_counter()
        while reps < 3 or (time.perf_counter() - t0 < 12.0 and reps < 12):  # about 12-20 s of CPU work
            oq.block_forward(w, 0, cfg, img, txt, temb, vf, tf)
            reps += 1
        total = time.perf_counter() - t0
    dt = total / reps
    # the same block in bf16, the dtype the GPU path computes in. Which of the two the CPU runs faster depends
    # on the host (bf16 matmul instructions or not): the faster one is the baseline, both are reported
    wb = {k: v.bfloat16() for k, v in w.items()}
    ib, tb, eb = img.bfloat16(), txt.bfloat16(), temb.bfloat16()
    with torch.inference_mode():
        reps16, t0 = 0, time.perf_counter()
        while reps16 < 1 or (time.perf_counter() - t0 < 6.0 and reps16 < 6):
            oq.block_forward(wb, 0, cfg, ib, tb, eb, vf, tf)
            reps16 += 1
        dt16 = (time.perf_counter() - t0) / reps16
    best, best_name = (dt, "fp32") if dt <= dt16 else (dt16, "bf16")
    return {"value": 1.0 / (best * LAYERS), "unit": "steps/s", "cores": cores, "kind": "port", "cpu_dtype": best_name,
            "fp32": {"value": 1.0 / (dt * LAYERS), "block_seconds": dt, "repetitions": reps},
            "bf16": {"value": 1.0 / (dt16 * LAYERS), "block_seconds": dt16, "repetitions": reps16},
            "sample": f"1 of {LAYERS} blocks at the full B=2, 4096+256-token shape, plain torch on {cores} threads: "
                      f"fp32 {reps} repetitions in {total:.1f} s, bf16 {reps16} repetitions of {dt16:.2f} s; the faster "
                      f"({best_name}) is the baseline; step time extrapolated as {LAYERS} x block (stem/head < 0.5%)",
            "block_seconds": best}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--blocks", type=int, default=LAYERS, help="debug only: fewer blocks (result is then marked invalid)")
    ap.add_argument("--workload", choices=("qwen", "flux", "wan"), default="qwen",
                    help="qwen = the headline metric; flux / wan = the other block families at their config shapes")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="launch only the headline attention shape and a plain 512 MiB copy, a few times each: the "
                         "program to run under `rocprofv3 --pmc FETCH_SIZE` / `--pmc WRITE_SIZE`")
    ap.add_argument("--counter-probe", action="store_true",
                    help="launch each hand-written kernel and the two large GEMMs at the headline shapes three "
                         "times: the program to run under `rocprofv3 --pmc <SQ counters>`")
    ap.add_argument("--unfused-epilogues", action="store_true",
                    help="A/B switch: GELU and gated residuals as separate kernels after plain GEMMs")
    ap.add_argument("--autotune", type=int, default=0,
                    help="time the library's kernels for each fused-epilogue GEMM in an untimed first step")
    ap.add_argument("--linear-engine", choices=("auto", "library", "handwritten"), default="auto",
                    help="A/B switch for the fused-epilogue projections: auto = the hand-written stream-K kernel where "
                         "it is expected (or was tuned) to win and the library elsewhere; library = hipBLASLt always")
    ap.add_argument("--teacache", type=float, default=None, metavar="THRESH",
                    help="with --workload flux: also run the 28-step trajectory under the TeaCache hook with this "
                         "relative-L1 threshold and report skip rate and steps/s")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-kernels", action="store_true")
    ap.add_argument("--no-in-step", action="store_true",
                    help="skip the two extra, untimed steps whose kernels are bracketed one by one (kernels_in_step)")
    ap.add_argument("--no-teacache", action="store_true",
                    help="skip the Flux-shape TeaCache trajectory (BASELINE.json configs[4]) that follows the headline measurement")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: this build runs the DiT step on ONE GPU (CFG branches are batched on it; "
                 "there are no collectives). Run with --gpus 1.")

    import torch

    from vllm_omni_amd import _lib, kernels
    from vllm_omni_amd.denoise import combine_cfg_noise, euler_step, flow_match_sigmas

    _lib.load()
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    from vllm_omni_amd import gemm_tuning

    tuned = gemm_tuning.enable()  # hipBLASLt solution ids picked offline for this model's GEMM shapes
    kernels.set_linear_engine(args.linear_engine)
    torch.cuda.set_device(0)
    dev = torch.device("cuda:0")
    if args.traffic_probe:
        S = S_IMG + S_TXT
        q = torch.randn(B, S, HEADS, HEAD_DIM, device=dev, dtype=torch.bfloat16)
        k, v = torch.randn_like(q), torch.randn_like(q)
        src = torch.empty(512 << 20, device=dev, dtype=torch.uint8).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(4):
            kernels.attn_fwd(q, k, v, 1.0 / math.sqrt(HEAD_DIM))
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"probe": "attention B=2 S=4352 24x128 bf16 x4, copy 512 MiB x4",
                          "attention_plan": kernels.attn_plan(B, S, S, HEADS, HEAD_DIM),
                          "attention_min_bytes": 4 * q.numel() * 2, "copy_bytes_each_way": src.numel()}))
        return
    if args.counter_probe:
        return counter_probe(torch, kernels, dev)
    if args.workload != "qwen":
        return run_secondary(torch, kernels, args)
    model = build_model(torch, args.blocks, fuse_epilogues=not args.unfused_epilogues)
    g = torch.Generator(device="cuda").manual_seed(1)
    latents = torch.randn(1, S_IMG, IN_CH, device=dev, generator=g).bfloat16()
    text = torch.randn(B, S_TXT, TEXT_DIM, device=dev, generator=g).bfloat16()
    total_steps = args.steps + args.warmup
    sig = flow_match_sigmas(max(total_steps, 20), S_IMG)

    def step(i, lat):
        t = torch.full((B,), float(sig[i]), device=dev, dtype=torch.bfloat16)
        out = model(hidden_states=lat.expand(B, -1, -1), encoder_hidden_states=text, encoder_hidden_states_mask=None,
                    timestep=t, img_shapes=[IMG_SHAPE], txt_seq_lens=[S_TXT] * B, return_dict=False)[0]
        noise = combine_cfg_noise(out[0:1], out[1:2], 4.0, True)
        return euler_step(lat, noise, float(sig[i]), float(sig[i + 1]))

    with torch.inference_mode(), AttnTimer(torch, kernels) as timer:
        lat = latents
        if args.autotune > 0:   # untimed: pick the library kernel for each fused-epilogue GEMM
            kernels.set_linear_autotune(args.autotune)
            step(0, lat)
            kernels.set_linear_autotune(0)
        for i in range(args.warmup):
            lat = step(i, lat)
        torch.cuda.synchronize()
        timer.active = True
        t0 = time.perf_counter()
        for i in range(args.warmup, total_steps):
            lat = step(i, lat)
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
        timer.active = False
        attn_ms = timer.mean_ms()
        n_attn = len(timer.pairs)
    assert bool(torch.isfinite(lat.float()).all()), "non-finite latents"
    in_step = None
    if not args.no_in_step:
        # two more steps, outside the timed region, every hand-written kernel and GEMM between its own events
        n_extra = 2
        with torch.inference_mode(), StepKernelTimer(torch, kernels) as kt:
            for i in range(n_extra):
                lat = step(i, lat)
            torch.cuda.synchronize()
        in_step = kt.report(n_extra)
    ms_per_step = elapsed * 1e3 / args.steps
    S = S_IMG + S_TXT
    attn_flop = 4.0 * B * HEADS * S * S * HEAD_DIM
    attn_tflops = attn_flop / attn_ms / 1e9
    from vllm_omni_amd import profiling

    plan = kernels.attn_plan(B, S, S, HEADS, HEAD_DIM)
    try:
        prof = profiling.attention_figures(plan)
    except (RuntimeError, ValueError, OSError) as e:
        # the committed counter summaries were measured on other launches than this build makes: quote none
        prof = {"traffic_bytes": None, "mfma_busy_frac": None, "clock_MHz": None, "profiled_kernel": None,
                "stale": str(e)}
    result = {
        "metric": "DiT denoise steps/s @1024² Qwen-Image shape (1 GPU); attn % bf16 MFMA peak",
        "value": args.steps / elapsed,
        "unit": "steps/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": f"Qwen-Image-shape MMDiT denoise step: {args.blocks} dual-stream blocks, hidden {C}, "
                               f"{HEADS} heads x {HEAD_DIM}, MLP {MLP_RATIO * C}, {S_IMG} image + {S_TXT} text tokens, "
                               "CFG batch 2, random weights N(0,0.02)",
                   "valid": args.blocks == LAYERS, "gemm": "hipBLASLt via torch" + (" (tuned solution table)" if tuned else "") +
                           ("" if args.linear_engine == "library" else "; text-stream MLP down-projection on the hand-written "
                            "stream-K MFMA kernel") +
                           ("; GELU and gated residuals as separate kernels" if args.unfused_epilogues else
                            "; GELU and gated residuals in the GEMM epilogues (odit_linear)")},
        "roofline": {"kernel": f"joint attention, B=2, 24x128, S=4352; one call = {plan} (timed together)", "bound": "mfma",
                     "achieved": attn_tflops, "peak": PEAK_MFMA_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": attn_tflops / PEAK_MFMA_BF16_TFLOPS,
                     "traffic": prof["traffic_bytes"],
                     "counters": {"mfma_busy_frac_of_cycles": prof["mfma_busy_frac"], "clock_MHz_in_kernel": prof["clock_MHz"],
                                  "kernel": prof["profiled_kernel"], "stale": prof.get("stale"),
                                  "source": "profiles/" + profiling.COUNTERS_FILE + " and profiles/" + profiling.TRAFFIC_FILE +
                                            " (rocprofv3 --pmc passes over bench.py --counter-probe / --traffic-probe, not live; "
                                            "launch plan checked against this build)"},
                     "launches_timed": n_attn, "avg_ms": attn_ms, "flop_per_launch": attn_flop},
        "step_flop": None,
    }
    gemm_flop = 2.0 * (B * S_IMG + B * S_TXT) * (3 * C * C + C * C + 2 * MLP_RATIO * C * C) * args.blocks
    result["step_flop"] = {"gemm": gemm_flop, "attention": attn_flop * args.blocks,
                           "achieved_TFLOP/s": (gemm_flop + attn_flop * args.blocks) / elapsed * args.steps / 1e12}
    if in_step is not None:
        result["kernels_in_step"] = {
            "what": "per-kernel averages over two extra steps run right after the timed region, each call between its "
                    "own HIP events (not part of `value`): the rate on the data the step hands the kernel",
            "kernels": in_step}
    if not args.no_kernels:
        with torch.inference_mode():
            result["kernels"] = kernel_rooflines(torch)
            result["mfma_ceiling"] = mfma_ceiling(torch)
            result["roofline"]["frac_of_measured_mfma_ceiling_random_data"] = (
                attn_tflops / result["mfma_ceiling"]["random_operands"]["TFLOP/s"])
    props = torch.cuda.get_device_properties(0)
    mhz = max_engine_clock_mhz()
    result["device"] = {
        "name": props.name, "gcn_arch": getattr(props, "gcnArchName", None), "compute_units": props.multi_processor_count,
        "max_engine_clock_MHz": mhz, "hbm_GiB": props.total_memory / 2 ** 30,
        # 4 SIMDs x one 32x32x16 bf16 MFMA (32768 FLOP) per 32 cycles = 4096 FLOP per clock per CU
        "bf16_mfma_peak_from_clock_TFLOP/s": (props.multi_processor_count * mhz * 1e6 * 4096 / 1e12) if mhz else None,
        "peaks_used": {"bf16_mfma_TFLOP/s": PEAK_MFMA_BF16_TFLOPS, "hbm_GB/s": PEAK_HBM_GBS},
    }
    del model
    torch.cuda.empty_cache()
    if not args.no_teacache and args.blocks == LAYERS:
        result["teacache_flux"] = teacache_flux(torch, kernels)
        torch.cuda.empty_cache()
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(torch)
        result["gpu_over_cpu"] = result["value"] / result["cpu_baseline"]["value"]
    print(json.dumps(result))


if __name__ == "__main__":
    main()
