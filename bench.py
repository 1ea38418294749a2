#!/usr/bin/env python3
"""Benchmark of the MTA forward path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline] [--no-extras]

A step is one full Multi-Token-Attention forward (MTAAttentionTriton.forward) at the
configuration the headline metric is quoted on: B=2, H=16, S=4096, D=128, bf16, causal,
6x11 pre-softmax conv (N(0,0.05) + identity tap), identity pre-softmax head weights,
identity 3x3 post-softmax conv, post-softmax head mixing in groups of 4 (I + N(0,0.1)).
Inputs are synthetic, seeded, and resident in HBM before the timed region.  Prints ONE
JSON line.  `value` is the latency of one forward in ms.  Defaults: 60 warm-up steps, 100
timed ones.  The first forty or so forwards after the device has been idle run up to 20 %
slower than the ones that follow (0.62-0.68 ms against 0.565 ms): every timed loop here is
therefore preceded by 80 ms of the same work (`ramp`), then by the W warm-up steps, then by
exactly K timed steps.

The `roofline` object is for the slowest hand-written kernel of the step; its duration
is measured live with events recorded on the stream the kernels run on.  `kernels` adds
the standalone operators at their own configurations (conv alone, head-mix alone, fused
conv-attention).  `cpu_baseline` times the oracle (a torch restatement of the
reference's PyTorch module) on the host cores, on a bounded sample.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0      # MI355X HBM3E, published
MFMA_BF16_PEAK_TF = 2500.0  # MI355X dense bf16, published


def tri(s: int) -> int:
    return s * (s + 1) // 2


def score_pass_bytes(b, h, s, esize):
    """Algorithmic bytes of one causal pass over a (B,H,S,S) tensor: read the lower triangle, write everything."""
    return b * h * (tri(s) + s * s) * esize


def stage_model(name, b, h, s, d, r=6, sk=11, esize=2):
    """Algorithmic HBM bytes and useful matrix flops of one stage of the forward at (B,H,S,D).

    A stage reads what it needs of the lower triangle and writes what its consumer reads:
      qk_conv          reads q,k; writes the lower triangle of the scores (QK^T, scale and conv fused)
      mix_softmax_mix  reads the lower triangle, writes the lower triangle (P V below never reads above it)
      pv               reads the lower triangle of P and V, writes O
      conv_pre / mix_* / softmax / conv_post (unfused route) read the triangle and write the full tensor
      qk, pv_gemm      library GEMMs over the full square
    """
    t, full, qkv = b * h * tri(s) * esize, b * h * s * s * esize, b * h * s * d * esize
    if name == "qk_conv":
        return 2 * qkv + t, 2 * b * h * tri(s) * d + 2 * r * sk * b * h * tri(s)
    if name == "mix_softmax_mix":
        return 2 * t, 0
    if name == "pv":
        return t + 2 * qkv, 2 * b * h * tri(s) * d
    if name in ("qk", "pv_gemm"):
        return 2 * qkv + full, 2 * b * h * s * s * d
    return t + full, 0


# Which kernel runs a stage of the headline forward, as rocprofv3 names it in profiles/mta_forward_c4_hbm_traffic.txt
STAGE_KERNEL = {"qk_conv": "conv_attn_fwd_mfma<bf16_t, 128, 6, 11, true, 4, false>",
                "mix_softmax_mix": "mix_softmax_mix_packed<bf16_t, 4, 1, false, true, 512, 8, false>",
                "pv": "causal_pv_kernel<bf16_t, 128, 1>"}
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "mta_forward_c4_hbm_traffic.txt")


def kernel_sources_digest():
    """sha256 over the kernel sources the library is built from: names the build a counter profile belongs to."""
    import hashlib
    d = os.path.join(ROOT, "multitokenatention_triton_amd", "csrc")
    h = hashlib.sha256()
    for name in sorted(os.listdir(d)):
        if name.endswith((".hip", ".hpp")):
            h.update(name.encode())
            with open(os.path.join(d, name), "rb") as f:
                h.update(f.read())
    return h.hexdigest()[:16]


def measured_traffic(stage):
    """HBM bytes per launch of the stage's kernel from the committed rocprofv3 counter summary (FETCH_SIZE and
    WRITE_SIZE, each scaled by what the same counter reads for a plain 1 GiB device copy; the summary states the
    factors) -- or None when the summary was taken from other kernel sources than the ones in this tree."""
    pat = STAGE_KERNEL.get(stage)
    try:
        lines = open(TRAFFIC_PROFILE).read().splitlines()
    except OSError:
        return None
    digest = [ln.split(":", 1)[1].strip() for ln in lines if ln.startswith("kernel sources sha256")]
    if not pat or not digest or digest[0] != kernel_sources_digest():
        return None
    for ln in lines:
        f = ln.split(None, 5)
        if len(f) == 6 and pat in f[5]:
            try:
                return float(f[4]) * 1e6
            except ValueError:
                pass
    return None


def build_c4(torch, mta, O, device, b=2, h=16, s=4096, d=128, dtype=None, nsets=3):
    dtype = dtype or torch.bfloat16
    g = torch.Generator().manual_seed(125)
    cfg = mta.MTAConfig(query_kernel_size=6, key_kernel_size=11)
    mod = mta.MTAAttentionTriton(h, cfg, dropout=0.0, causal=True).to(dtype)
    with torch.no_grad():
        mod.mta_conv_triton.weight.copy_(O.seeded_conv_weight(h, 6, 11, 0.05, dtype))
        mod.wpsm_triton.weight.copy_(torch.eye(h))
        mod.mta_conv_after_sm_triton.weight.copy_(O.identity_conv_kernel(h, 3, 3, dtype))
        mod.wposm_triton.weight.copy_(O.block_diag_head_weight(h, 4, 0.1, g, dtype))
    mod = mod.to(device).eval().requires_grad_(False)
    # the configuration states the structure (identity wpsm and post conv, groups of 4): read it off the weights once
    mod.infer_weight_structure()
    sets = [tuple(t.to(device) for t in O.seeded_qkv(b, h, s, d, dtype, seed=123 + i)) for i in range(nsets)]
    return mod, sets


def build_general(torch, mta, O, device, b=1, h=16, s=4096, d=128, nsets=2, train=False, dtype=None, ks=(7, 7)):
    """The closest shapes to the reference's published rows (benchmark_seq_len_results.jsonl: H16 D128 fp16, 7x7 conv
    before and after the softmax; benchmark_mta_attention.py: bf16, 11x15; benchmark_seq_len.py: 128 heads) with all four
    weights non-trivial -- random kernels, dense random head weights (the reference's scripts run identity weights
    through kernels that take no advantage of them)."""
    dtype = dtype or torch.float16
    g = torch.Generator().manual_seed(321)
    cfg = mta.MTAConfig(query_kernel_size=ks[0], key_kernel_size=ks[1], after_sm_query_kernel_size=ks[0],
                        after_sm_key_kernel_size=ks[1])
    mod = mta.MTAAttentionTriton(h, cfg, dropout=0.0, causal=True).to(dtype)
    with torch.no_grad():
        mod.mta_conv_triton.weight.copy_(O.seeded_conv_weight(h, ks[0], ks[1], 0.05, dtype, seed=5))
        mod.mta_conv_after_sm_triton.weight.copy_(O.seeded_conv_weight(h, ks[0], ks[1], 0.05, dtype, seed=6))
        mod.wpsm_triton.weight.copy_(torch.eye(h) + 0.1 * torch.randn(h, h, generator=g))
        mod.wposm_triton.weight.copy_(torch.eye(h) + 0.1 * torch.randn(h, h, generator=g))
    mod = mod.to(device)                                 # dense weights: nothing is assumed about their structure
    mod = mod.train() if train else mod.eval().requires_grad_(False)
    sets = [tuple(t.to(device).requires_grad_(train) for t in O.seeded_qkv(b, h, s, d, dtype, seed=400 + i))
            for i in range(nsets)]
    return mod, sets


RAMP_MS = 80.0


def ramp(torch, fn, nsets, min_ms=RAMP_MS):
    """Keep the device busy with the work that is about to be timed for `min_ms` of wall time.  After an idle spell
    (the host preparing inputs takes seconds) the first 25 ms or so of kernels run up to 20 % slower than what follows;
    the W warm-up steps of the contract come after this and are too few to cover it when W is small."""
    t0 = time.perf_counter()
    i = 0
    while (time.perf_counter() - t0) * 1e3 < min_ms:
        for _ in range(10):
            fn(i % nsets)
            i += 1
        torch.cuda.synchronize()


def time_steps(torch, fn, nsets, warmup, steps):
    ramp(torch, fn, nsets)
    for i in range(warmup):
        fn(i % nsets)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        fn(i % nsets)
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / steps


def time_launches(torch, fn, nsets, warmup, steps):
    """Average duration of one launch of a single-kernel operator: an event pair around every launch, on the stream
    the kernel is launched on (what `rocprofv3 --kernel-trace` reports per dispatch, plus the event overhead; the
    wall clock over a loop of launches also counts the gaps between them)."""
    ramp(torch, fn, nsets)
    for i in range(warmup):
        fn(i % nsets)
    torch.cuda.synchronize()
    pairs = []
    for i in range(steps):
        e0 = _record(torch)
        fn(i % nsets)
        pairs.append((e0, _record(torch)))
    torch.cuda.synchronize()
    return sum(a.elapsed_time(b) for a, b in pairs) / steps


def stage_breakdown(torch, mod, sets, steps):
    """Average duration of each stage of forward(), from events on the kernels' own stream."""
    marks = []
    mod._stage_hook = lambda name: marks.append((name, _record(torch)))
    per_step = []
    for i in range(steps):
        marks.clear()
        mod(*sets[i % len(sets)], None, None)
        per_step.append(list(marks))
    torch.cuda.synchronize()
    mod._stage_hook = None
    acc = {}
    for m in per_step:
        for (name, ev), (_, nxt) in zip(m[:-1], m[1:]):
            acc.setdefault(name, []).append(ev.elapsed_time(nxt))
    return {k: sum(v) / len(v) for k, v in acc.items()}


def _record(torch):
    ev = torch.cuda.Event(enable_timing=True)
    ev.record()  # on the current stream, the one ops.py hands to the library
    return ev


def bench_kernels(torch, mta, O, device, steps, warmup):
    """Standalone operators at their own BASELINE configurations."""
    out = {}
    bf16 = torch.bfloat16
    g = torch.Generator().manual_seed(7)
    # conv alone: (2,16,2048,2048) bf16, 6x11 N(0,0.05), causal
    n, c, s = 2, 16, 2048
    w = O.seeded_conv_weight(c, 6, 11, 0.05, bf16, identity_tap=False).to(device)
    xs = [torch.tril(torch.randn(n, c, s, s, generator=g).to(bf16)).to(device) for _ in range(3)]
    ys = [torch.empty_like(x) for x in xs]
    ms = time_launches(torch, lambda i: mta.ops.conv2d_causal(xs[i], w, True, out=ys[i]), 3, warmup, steps)
    by = score_pass_bytes(n, c, s, 2)
    out["conv2d_6x11_bf16_2x16x2048x2048"] = {"ms": ms, "algorithmic_bytes": by, "GBps": by / ms / 1e6,
                                              "frac_hbm_peak": by / ms / 1e6 / HBM_PEAK_GBS}
    del ys
    # its two gradients at the same shape (convolution_2d_trit.py:336-378): dx reads the lower triangle of dy and
    # writes all of dx; dw reads the lower triangles of x and dy
    ms = time_launches(torch, lambda i: mta.ops.conv2d_bwd_input(xs[i], w, True), 3, warmup, steps)
    out["conv2d_bwd_input_6x11_bf16_2x16x2048x2048"] = {"ms": ms, "algorithmic_bytes": by, "GBps": by / ms / 1e6,
                                                        "frac_hbm_peak": by / ms / 1e6 / HBM_PEAK_GBS}
    by2 = 2 * n * c * tri(s) * 2
    ms = time_launches(torch, lambda i: mta.ops.conv2d_bwd_weight(xs[i], xs[(i + 1) % 3], (6, 11), True), 3, warmup, steps)
    out["conv2d_bwd_weight_6x11_bf16_2x16x2048x2048"] = {"ms": ms, "algorithmic_bytes": by2, "GBps": by2 / ms / 1e6,
                                                         "frac_hbm_peak": by2 / ms / 1e6 / HBM_PEAK_GBS}
    del xs
    # head-mix alone: (2,32,2048,2048) bf16, groups of 4
    n, c, s = 2, 32, 2048
    wm = O.block_diag_head_weight(c, 4, 0.1, g, bf16).to(device)
    xs = []
    for _ in range(2):
        logits = torch.randn(n, c, s, s, generator=g)
        logits.masked_fill_(torch.triu(torch.ones(s, s, dtype=torch.bool), 1), float("-inf"))
        xs.append(torch.softmax(logits, -1).to(bf16).to(device))
        del logits
    ys = [torch.empty_like(x) for x in xs]
    by = score_pass_bytes(n, c, s, 2)
    for label, grp in (("headmix_g4_bf16_2x32x2048x2048", 4), ("headmix_dense_bf16_2x32x2048x2048", None)):
        ms = time_launches(torch, lambda i: mta.ops.headmix(xs[i], wm, True, 0.0, group_size=grp, out=ys[i]), 2, warmup, steps)
        out[label] = {"ms": ms, "algorithmic_bytes": by, "GBps": by / ms / 1e6, "frac_hbm_peak": by / ms / 1e6 / HBM_PEAK_GBS}
    del ys
    # its two gradients (triton_linear_head.py:322-370): dx = W^T dy (groups of 4), dW = dy x^T over the attended positions
    ms = time_launches(torch, lambda i: mta.ops.headmix_bwd_input(xs[i], wm, True, group_size=4), 2, warmup, steps)
    out["headmix_bwd_input_g4_bf16_2x32x2048x2048"] = {"ms": ms, "algorithmic_bytes": by, "GBps": by / ms / 1e6,
                                                       "frac_hbm_peak": by / ms / 1e6 / HBM_PEAK_GBS}
    by2 = 2 * n * c * tri(s) * 2
    ms = time_launches(torch, lambda i: mta.ops.headmix_bwd_weight(xs[i], xs[1 - i], True), 2, warmup, steps)
    out["headmix_bwd_weight_bf16_2x32x2048x2048"] = {"ms": ms, "algorithmic_bytes": by2, "GBps": by2 / ms / 1e6,
                                                     "frac_hbm_peak": by2 / ms / 1e6 / HBM_PEAK_GBS}
    # the softmax gradient of the training route from the stored probabilities (what torch's autograd through
    # mta_attention_triton.py:79 is replaced by): reads p and dp below the diagonal, writes dx everywhere
    ms = time_launches(torch, lambda i: mta.ops.softmax_bwd(xs[i], xs[1 - i], True), 2, warmup, steps)
    by3 = 2 * n * c * tri(s) * 2 + n * c * s * s * 2
    out["softmax_bwd_bf16_2x32x2048x2048"] = {"ms": ms, "algorithmic_bytes": by3, "GBps": by3 / ms / 1e6,
                                              "frac_hbm_peak": by3 / ms / 1e6 / HBM_PEAK_GBS}
    del xs
    # fused conv-attention: B1 H32 S8192 D128 bf16, 6x11
    b, h, s, d = 1, 32, 8192, 128
    sets = [tuple(t.to(device) for t in O.seeded_qkv(b, h, s, d, bf16, seed=200 + i)) for i in range(2)]
    wc = O.seeded_conv_weight(h, 6, 11, 0.05, bf16).to(device)
    os_ = [torch.empty_like(sets[0][0]) for _ in range(2)]
    ms = time_launches(torch, lambda i: mta.ops.conv_attn_fwd(*sets[i], wc, True, None, out=os_[i]), 2, min(warmup, 10),
                    max(2, steps // 4))
    mfma_flops = 4 * b * h * tri(s) * d
    out["conv_attn_fused_bf16_1x32x8192x128"] = {"ms": ms, "mfma_useful_flops": mfma_flops,
                                                 "TFLOPs": mfma_flops / ms / 1e9,
                                                 "frac_mfma_peak": mfma_flops / ms / 1e9 / MFMA_BF16_PEAK_TF}
    del sets, os_
    # the general four-stage forward (all MTA weights non-trivial), B1 H16 S4096 D128 fp16, 7x7 conv pre and post
    mod, sets = build_general(torch, mta, O, device)
    ms = time_steps(torch, lambda i: mod(*sets[i], None, None), len(sets), min(warmup, 30), max(3, steps // 2))
    stages = stage_breakdown(torch, mod, sets, 3)
    out["mta_forward_general_fp16_1x16x4096x128_7x7_pre_post_dense"] = {
        "ms": ms, "stages_ms": stages,
        "note": "forward only; the reference's published row for this shape (Triton 11.345 ms, PyTorch 43.795 ms, "
                "hardware unstated) is context, not a baseline"}
    # the same module under a 1024-key sliding-window mask tensor: band masks behind a post-softmax conv
    mod.use_mask = True
    s_len = sets[0][0].size(2)
    pos = torch.arange(s_len, device=device)
    window = ((pos[None, :] <= pos[:, None]) & (pos[None, :] > pos[:, None] - 1024))[None, None]
    ms = time_steps(torch, lambda i: mod(*sets[i], window, None), len(sets), min(warmup, 30), max(3, steps // 2))
    stages = []
    mod._stage_hook = stages.append
    mod(*sets[0], window, None)
    mod._stage_hook = None
    out["mta_forward_general_fp16_1x16x4096x128_7x7_pre_post_dense_window1024_mask"] = {
        "ms": ms, "stages": stages,
        "note": "the general configuration with use_mask=True and a sliding-window mask tensor; not a row of the reference's"}
    del mod, sets, window
    # two more of the reference's own benchmark shapes, forward only: its benchmark script's configuration (bf16, 11x15
    # kernels before and after the softmax, B1 H16 S4096 D64: benchmark_mta_attention.py:12-38) and the 128-head sweep's
    # first row (B1 H128 S2048 D64 fp16 7x7: benchmark_seq_len.py:22-30, benchmark_seq_len_results.jsonl:198)
    for label, kw, note in (
            ("mta_forward_general_bf16_1x16x4096x64_11x15_pre_post_dense",
             dict(b=1, h=16, s=4096, d=64, dtype=torch.bfloat16, ks=(11, 15)),
             "the reference's benchmark script runs this shape (benchmark_mta_attention.py:12-38); it publishes no number for it"),
            ("mta_forward_general_fp16_1x128x2048x64_7x7_pre_post_dense",
             dict(b=1, h=128, s=2048, d=64, dtype=torch.float16, ks=(7, 7)),
             "the reference's published row for this shape (Triton 22.579 ms, PyTorch 115.382 ms, hardware unstated) is "
             "context, not a baseline"),
            # fp32, the dtype of most of the reference's published rows: no one-kernel scores stage and no triangle-only
            # P V (library GEMMs), fp32-FMA conv kernels (benchmark_seq_len_results.jsonl:1)
            ("mta_forward_general_fp32_1x16x1024x64_11x15_pre_post_dense",
             dict(b=1, h=16, s=1024, d=64, dtype=torch.float32, ks=(11, 15)),
             "the reference's published row for this shape (Triton 1.887 ms, PyTorch 4.203 ms, hardware unstated) is "
             "context, not a baseline")):
        mod, sets = build_general(torch, mta, O, device, **kw)
        ms = time_steps(torch, lambda i: mod(*sets[i], None, None), len(sets), min(warmup, 10), max(3, steps // 5))
        out[label] = {"ms": ms, "stages_ms": stage_breakdown(torch, mod, sets, 3), "note": "forward only; " + note}
        del mod, sets
    # the headline forward under a sliding-window mask (each row sees its last 1024 keys), given to the module as a
    # (1,1,S,S) boolean mask tensor: it travels to the kernels as one int32 per (batch entry, row)
    mod, sets = build_c4(torch, mta, O, device)
    mod.use_mask = True
    s_len = sets[0][0].size(2)
    pos = torch.arange(s_len, device=device)
    window = ((pos[None, :] <= pos[:, None]) & (pos[None, :] > pos[:, None] - 1024))[None, None]
    ms = time_steps(torch, lambda i: mod(*sets[i], window, None), len(sets), min(warmup, 30), max(3, steps // 2))
    stages = []
    mod._stage_hook = stages.append
    mod(*sets[0], window, None)
    mod._stage_hook = None
    out["mta_forward_bf16_2x16x4096x128_window1024_mask"] = {
        "ms": ms, "stages": stages,
        "note": "the headline configuration with use_mask=True and a sliding-window mask tensor; not a row of the reference's"}
    # ... and under a key-padding mask of the batch (the second sequence is 3000 tokens long), given as a (B,1,S,S) boolean
    # mask tensor: it travels to the kernels as one fp32 value per (batch entry, key)
    lengths = torch.tensor([s_len, 3000], device=device)
    padded = ((pos[None, :] < lengths[:, None])[:, None, None, :] & (pos[None, :] <= pos[:, None])[None, None])
    ms = time_steps(torch, lambda i: mod(*sets[i], padded, None), len(sets), min(warmup, 30), max(3, steps // 2))
    stages = []
    mod._stage_hook = stages.append
    mod(*sets[0], padded, None)
    mod._stage_hook = None
    out["mta_forward_bf16_2x16x4096x128_key_padding_mask"] = {
        "ms": ms, "stages": stages,
        "note": "the headline configuration with use_mask=True and a key-padding mask tensor (lengths 4096 and 3000); not a row of the reference's"}
    # ... and under a mask of arbitrary content (a fifth of the keys below the diagonal hidden at random, the diagonal
    # kept), given as a (1,1,S,S) boolean mask tensor: the single-stage kernels with three mask passes between them
    gen = torch.Generator(device=device).manual_seed(11)
    holes = ((torch.rand(s_len, s_len, device=device, generator=gen) > 0.2) | (pos[None, :] == pos[:, None])) & (pos[None, :] <= pos[:, None])
    holes = holes[None, None]
    ms = time_steps(torch, lambda i: mod(*sets[i], holes, None), len(sets), min(warmup, 5), max(3, steps // 5))
    stages = []
    mod._stage_hook = stages.append
    mod(*sets[0], holes, None)
    mod._stage_hook = None
    out["mta_forward_bf16_2x16x4096x128_random_holes_mask"] = {
        "ms": ms, "stages": stages,
        "note": "the headline configuration with use_mask=True and a mask tensor with holes; not a row of the reference's"}
    del mod, sets, window, padded, holes
    # the first module and shape in training: forward operator by operator (each with its HIP backward kernels; the two
    # matrix products, the softmax and the dropout are torch's) and backward to q, k, v and the four weights
    mod, sets = build_general(torch, mta, O, device, train=True)
    params = [p for p in mod.parameters()]
    gout = torch.randn(sets[0][0].shape, generator=torch.Generator().manual_seed(9)).to(sets[0][0].dtype).to(device)
    gout = gout.transpose(1, 2)

    def train_step(i):
        for t in params + list(sets[i]):
            t.grad = None
        with torch.enable_grad():
            mod(*sets[i], None, None).backward(gout)

    ms = time_steps(torch, train_step, len(sets), min(warmup, 5), max(3, steps // 10))
    out["mta_forward_backward_general_fp16_1x16x4096x128_7x7_pre_post_dense"] = {
        "ms": ms,
        "note": "forward + backward; the reference's published row for this shape (Triton 39.090 ms, PyTorch 253.350 ms, "
                "hardware unstated) is context, not a baseline"}
    # ... and the same training step under mask tensors (use_mask=True): a sliding window of 1024 keys and a key-padding
    # mask, both recognised and run through the same differentiable kernel operators
    mod.use_mask = True
    s_len = sets[0][0].size(2)
    pos = torch.arange(s_len, device=device)
    lower = pos[None, :] <= pos[:, None]
    masks = {"window1024_mask": (lower & (pos[None, :] > pos[:, None] - 1024))[None, None],
             "key_padding_mask": ((pos < 3000)[None, :] & lower)[None, None]}
    for name, mask in masks.items():
        def masked_step(i, mask=mask):
            for t in params + list(sets[i]):
                t.grad = None
            with torch.enable_grad():
                mod(*sets[i], mask, None).backward(gout)

        ms = time_steps(torch, masked_step, len(sets), min(warmup, 5), max(3, steps // 10))
        out["mta_forward_backward_general_fp16_1x16x4096x128_7x7_pre_post_dense_" + name] = {
            "ms": ms, "note": "forward + backward with use_mask=True and a mask tensor; not a row of the reference's"}
    return out


def cpu_baseline(torch, O, b, h, s, d, budget_s=12.0):
    """The oracle's torch MTA forward on all host cores, on a bounded sample of the same workload."""
    threads = os.cpu_count() or 1
    torch.set_num_threads(threads)
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(125)
    w_pre = O.seeded_conv_weight(h, 6, 11, 0.05, dtype).unsqueeze(1)
    w_post = O.identity_conv_kernel(h, 3, 3, dtype).unsqueeze(1)
    wpsm = torch.eye(h, dtype=dtype)
    wposm = O.block_diag_head_weight(h, 4, 0.1, g, dtype)

    def run(ss):
        q, k, v = O.seeded_qkv(1, h, ss, d, dtype)
        t0 = time.perf_counter()
        with torch.no_grad():
            O.mta_forward(q, k, v, w_pre, wpsm, w_post, wposm)
        return time.perf_counter() - t0

    probe_s = 256
    t_probe = min(run(probe_s), run(probe_s))
    ss = probe_s
    while ss * 2 <= s and t_probe * ((ss * 2) / probe_s) ** 2 <= budget_s:
        ss *= 2
    t = run(ss) if ss != probe_s else t_probe
    factor = (b * s * s) / (1 * ss * ss)
    return {"value": t * 1e3 * factor, "unit": "ms", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"oracle.mta_forward bf16 on B=1,H={h},S={ss},D={d} took {t * 1e3:.1f} ms; "
                      f"scaled by {factor:.0f} (score-tensor elements) to B={b},S={s}",
            "host_cpu_count": os.cpu_count(), "torch_threads": torch.get_num_threads(), "cpu_model": _cpu_model()}


def cpu_baselines_other(torch, O):
    """The oracle on the host cores for the other configurations: C1 at its full size, one batch element of the
    conv-alone and head-mix-alone configurations, and a row slab of the fused conv-attention one.  A few seconds each."""
    threads = os.cpu_count() or 1
    torch.set_num_threads(threads)
    out = {}
    with torch.no_grad():
        # C1: B1 H4 S256 D64 fp32, conv 3x5, full size, 10 repetitions
        q, k, v = O.seeded_qkv(1, 4, 256, 64, torch.float32)
        g = torch.Generator().manual_seed(125)
        w_pre = O.seeded_conv_weight(4, 3, 5, 0.1, torch.float32).unsqueeze(1)
        w_post = O.identity_conv_kernel(4, 3, 3, torch.float32).unsqueeze(1)
        wpsm, wposm = O.block_diag_head_weight(4, 2, 0.1, g), O.block_diag_head_weight(4, 2, 0.1, g)
        O.mta_forward(q, k, v, w_pre, wpsm, w_post, wposm)
        t0 = time.perf_counter()
        for _ in range(10):
            O.mta_forward(q, k, v, w_pre, wpsm, w_post, wposm)
        out["mta_forward_fp32_1x4x256x64"] = {"value": (time.perf_counter() - t0) * 100.0, "unit": "ms", "cores": threads,
                                              "kind": "port", "sample": "full size, mean of 10 repetitions"}
        # C2: conv alone (2,16,2048,2048) bf16 6x11: one batch element, scaled by 2
        bf16 = torch.bfloat16
        gg = torch.Generator().manual_seed(7)
        x = torch.tril(torch.randn(1, 16, 2048, 2048, generator=gg)).to(bf16)
        w = O.seeded_conv_weight(16, 6, 11, 0.05, bf16, identity_tap=False)
        t0 = time.perf_counter()
        O.depthwise_conv(x, w, True)
        t = time.perf_counter() - t0
        out["conv2d_6x11_bf16_2x16x2048x2048"] = {"value": t * 2e3, "unit": "ms", "cores": threads, "kind": "port",
                                                  "sample": f"one of the two batch elements took {t * 1e3:.0f} ms; scaled by 2"}
        del x
        # C3: head-mix alone (2,32,2048,2048) bf16 groups of 4: one batch element, scaled by 2
        x = torch.softmax(torch.randn(1, 32, 2048, 2048, generator=gg).masked_fill(
            torch.triu(torch.ones(2048, 2048, dtype=torch.bool), 1), float("-inf")), -1).to(bf16)
        wm = O.block_diag_head_weight(32, 4, 0.1, gg, bf16)
        t0 = time.perf_counter()
        O.head_linear(x, wm, True, 0.0)
        t = time.perf_counter() - t0
        out["headmix_g4_bf16_2x32x2048x2048"] = {"value": t * 2e3, "unit": "ms", "cores": threads, "kind": "port",
                                                 "sample": f"one of the two batch elements took {t * 1e3:.0f} ms; scaled by 2"}
        del x
        # C5: fused conv-attention B1 H32 S8192 D128 bf16: 256 query rows in the middle of the sequence against all
        # keys, 8 of the 32 heads; scaled by rows and heads (the work per row grows with the row index: the middle
        # slab stands for the average row)
        q, k, v = O.seeded_qkv(1, 8, 8192, 128, bf16, seed=200)
        wc = O.seeded_conv_weight(8, 6, 11, 0.05, bf16)
        t0 = time.perf_counter()
        O.conv_attention_rows(q, k, v, wc, 3968, 4224, True)
        t = time.perf_counter() - t0
        out["conv_attn_fused_bf16_1x32x8192x128"] = {
            "value": t * 1e3 * (8192 / 256) * (32 / 8), "unit": "ms", "cores": threads, "kind": "port",
            "sample": f"query rows 3968..4223 of 8 heads took {t * 1e3:.0f} ms; scaled by 32 (rows) x 4 (heads)"}
    return out


def _cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=60)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="only run a plain device copy of 1 GiB five times (scales the FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")

    import torch

    import multitokenatention_triton_amd as mta
    from oracle import mta_oracle as O

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    device = torch.device("cuda:0")
    if args.copy_calibration:
        src = torch.ones(1 << 29, dtype=torch.bfloat16, device=device)   # 1 GiB read + 1 GiB written per copy
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_calibration_bytes_each_way": src.numel() * 2, "copies": 5}))
        return
    b, h, s, d = 2, 16, 4096, 128
    mod, sets = build_c4(torch, mta, O, device, b, h, s, d)

    with torch.no_grad():
        ms = time_steps(torch, lambda i: mod(*sets[i], None, None), len(sets), args.warmup, args.steps)
        stages = stage_breakdown(torch, mod, sets, max(3, min(args.steps, 10)))
        ran_own_pv = "qk" not in stages  # the fused route ends in mta_causal_pv_fwd, the unfused one in a library GEMM
        hip_stages = {k: v for k, v in stages.items() if k != "qk" and (k != "pv" or ran_own_pv)}
        dom = max(hip_stages, key=hip_stages.get)
        dom_bytes, dom_flops = stage_model(dom, b, h, s, d)
        achieved = dom_bytes / hip_stages[dom] / 1e6
        per_stage = {}
        for k, v in stages.items():
            by, fl = stage_model(k if (k != "pv" or ran_own_pv) else "pv_gemm", b, h, s, d)
            per_stage[k] = {"ms": v, "algorithmic_bytes": by, "GBps": by / v / 1e6, "frac_hbm_peak": by / v / 1e6 / HBM_PEAK_GBS,
                            "useful_TFLOPs": fl / v / 1e9}
        kernels = {} if args.no_extras else bench_kernels(torch, mta, O, device, args.steps, args.warmup)

    result = {
        "metric": "MTA fwd latency (ms) + conv/head-mix HBM GB/s, H16 S4096 D128 bf16",
        "value": ms, "unit": "ms", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms,
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "full MTA forward B=2 H=16 S=4096 D=128 bf16 causal, conv 6x11 pre-softmax, "
                               "identity post-softmax conv, head-mix groups of 4 (BASELINE configs[3])",
                   "global_batch": b, "seq_len": s},
        "roofline": {"bound": "hbm", "kernel": dom, "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": measured_traffic(dom),
                     "algorithmic_bytes": dom_bytes, "avg_kernel_ms": hip_stages[dom],
                     "useful_matrix_TFLOPs": dom_flops / hip_stages[dom] / 1e9},
        "stages_ms": stages,
        "stages": per_stage,
        "kernels": kernels,
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(torch, O, b, h, s, d)
        if not args.no_extras:
            result["cpu_baselines_other_configs"] = cpu_baselines_other(torch, O)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
