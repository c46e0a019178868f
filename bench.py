#!/usr/bin/env python3
"""Benchmark of the quantised-KV decode-attention hot path on one MI355X.

A "step" is one fused decode-attention layer call (the reference's decode
branch, patch_internvl.py:344-436) on a synthetic InternVL2.5-8B-shaped layer:
batch 64, 32 query / 8 KV heads, head_dim 128, 3 328 packed image tokens plus a
128-row bf16 residual window.  Inputs are resident in HBM before the timed
region; the call rotates over several distinct buffer sets (> 256 MB in total)
so the packed codes are not served from the Infinity Cache.

Prints ONE JSON line.  `value` is the
average duration of one layer call in microseconds; `roofline` prices the
algorithmic bytes of that call against the 8 TB/s HBM peak; `cpu_baseline` is
the C port of the oracle timed on this host's cores on a bounded sample.

Before the W warm-up steps the same calls run untimed for `--settle-ms`
(default 300 ms): the device takes that long under this load to reach its
steady state (a run of 20 steps straight after the inputs are built reads
about 10 % slower than one of 4 000), and the steady state is what a decode
loop of thousands of layer calls per second sees.  `config.settle_ms` states it.
The timed block of K steps is repeated `--blocks` times (default 25) and the
median block is `value` / `ms_per_step` (`config.timed_blocks`); the figure of a
cold process - W warm-up steps and one block of K steps with no settling run -
is reported beside it as `value_unsettled_us`.
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

HBM_PEAK_GBPS = 8000.0
METRIC = "1-bit decode-attn µs/layer + HBM GB/s %peak; InternVL2.5-8B decode tok/s"

WORKLOADS = {
    # name: (B, Hq, Hkv, D, T, R, S)
    "internvl2.5-8b-layer-b64-kv3328+128": (64, 32, 8, 128, 3328, 128, 0),
    "long-context-b8-kv32768": (8, 32, 8, 128, 32768, 0, 0),
    "wide-batch-b256-kv3328": (256, 32, 8, 128, 3328, 0, 0),
    "internvl2.5-26b-layer-b16-kv9984+64": (16, 48, 8, 128, 9984, 64, 0),
}
DEFAULT_WORKLOAD = "internvl2.5-8b-layer-b64-kv3328+128"


def algorithmic_bytes(B, Hq, Hkv, D, T, R, bits, elt=2):
    """Each byte counted once: K+V codes, per-channel K and V statistics,
    fp residual K+V, q in and out."""
    codes = 2 * B * Hkv * T * D * bits // 8
    stats = 4 * B * Hkv * D * elt
    resid = 2 * B * Hkv * R * D * elt
    qo = 2 * B * Hq * D * elt
    return codes + stats + resid + qo


def measured_traffic(workload, bits):
    """HBM bytes per launch measured with rocprofv3 byte counters (profiles/decode_kernel_traffic.json),
    or None when that workload has not been profiled."""
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", "decode_kernel_traffic.json")
    try:
        with open(path) as f:
            return json.load(f).get(f"{workload}/bits{bits}", {}).get("traffic_bytes")
    except OSError:
        return None


def build_sets(torch, ops, shape, bits, nsets, seed):
    """Synthetic layer state, generated on the GPU with a seeded device
    generator: K/V ~ N(0,1), four key channels per kv-head scaled by |t3|+1
    (Student-t, nu=3), quantised and packed by the prefill kernel."""
    B, Hq, Hkv, D, T, R, S = shape
    dev = torch.device("cuda:0")
    torch.manual_seed(seed)
    g = torch.Generator(device=dev).manual_seed(seed)
    cpu_rng = torch.Generator().manual_seed(seed)
    clip_k, clip_v = (0.5, 0.3) if bits == 1 else (1.0, 1.0)
    sets = []
    for _ in range(nsets):
        k = torch.randn((B, T, Hkv, D), generator=g, device=dev)
        v = torch.randn((B, T, Hkv, D), generator=g, device=dev)
        for h in range(Hkv):
            ch = torch.randperm(D, generator=cpu_rng)[:4].to(dev)
            t3 = torch.distributions.StudentT(3.0).sample((4,)).abs().to(dev) + 1.0
            k[:, :, h, ch] *= t3
        k, v = k.to(torch.bfloat16), v.to(torch.bfloat16)
        ck, sk, zk = ops.quantize_pack(k, bits, clip_k)
        cv, sv, zv = ops.quantize_pack(v, bits, clip_v)
        del k, v
        q = torch.randn((B, Hq, D), generator=g, device=dev).to(torch.bfloat16)
        kr = torch.randn((B, Hkv, max(R, 1), D), generator=g, device=dev).to(torch.bfloat16)[:, :, :R]
        vr = torch.randn((B, Hkv, max(R, 1), D), generator=g, device=dev).to(torch.bfloat16)[:, :, :R]
        sets.append(dict(q=q, ck=ck, cv=cv, sk=sk, zk=zk, sv=sv, zv=zv, kr=kr if R else None, vr=vr if R else None))
    return sets


def settle(torch, run, ms):
    """Run `run(i)` untimed for about `ms` milliseconds of device time."""
    if ms <= 0:
        return
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for i in range(8):
        run(i)
    end.record()
    torch.cuda.synchronize()
    per = max(start.elapsed_time(end) / 8, 1e-3)
    for i in range(int(ms / per)):
        run(i)
    torch.cuda.synchronize()


def time_block(torch, calls, steps):
    """One timed block: exactly `steps` calls between two events, synchronised on both sides; ms per call."""
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for i in range(steps):
        calls[i % len(calls)].run()
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / steps


def time_calls(torch, calls, steps, warmup, settle_ms=0.0, blocks=1):
    """`warmup` untimed calls, then `blocks` timed blocks of exactly `steps` calls each; the median block
    is the figure (a single block of 20 calls lasts under a millisecond and reads a few per cent high or
    low from one run to the next).  Returns (median ms per call, [every block's ms per call])."""
    settle(torch, lambda i: calls[i % len(calls)].run(), settle_ms)
    for i in range(warmup):
        calls[i % len(calls)].run()
    per = sorted(time_block(torch, calls, steps) for _ in range(max(1, blocks)))
    return per[len(per) // 2], per


def time_fp16_kv(torch, shape, steps, warmup, nsets):
    """Full-precision-KV attention over the same tokens with torch's fused SDPA."""
    B, Hq, Hkv, D, T, R, S = shape
    dev = torch.device("cuda:0")
    N = T + R
    sets = []
    for _ in range(nsets):
        q = torch.randn((B, Hq, 1, D), device=dev, dtype=torch.bfloat16)
        k = torch.randn((B, Hkv, N, D), device=dev, dtype=torch.bfloat16)
        v = torch.randn((B, Hkv, N, D), device=dev, dtype=torch.bfloat16)
        sets.append((q, k, v))
    F = torch.nn.functional

    def run(i):
        q, k, v = sets[i % nsets]
        return F.scaled_dot_product_attention(q, k, v, enable_gqa=True)

    for i in range(warmup):
        run(i)
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for i in range(steps):
        run(i)
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / steps


def time_fp16_kv_own(torch, ops, shape, steps, warmup, nsets):
    """Full-precision-KV attention over the same tokens with this library's own kernel: every
    token a row of the full-precision window (no packed part)."""
    B, Hq, Hkv, D, T, R, S = shape
    dev = torch.device("cuda:0")
    N = T + R
    calls = []
    for _ in range(nsets):
        q = torch.randn((B, Hq, D), device=dev, dtype=torch.bfloat16)
        k = torch.randn((B, Hkv, N, D), device=dev, dtype=torch.bfloat16)
        v = torch.randn((B, Hkv, N, D), device=dev, dtype=torch.bfloat16)
        calls.append(ops.DecodeCall(q, None, None, None, None, None, None, k, v, sprompt_len=0, bits=1))
    it = [0]

    def run():
        calls[it[0] % nsets].run()
        it[0] += 1

    return _time_fn(torch, run, steps, warmup)


def _time_fn(torch, fn, steps, warmup):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(steps):
        fn()
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / steps


def prefill_leg(torch, ops, shape, bits, steps=40, warmup=10, contiguous=False, rope=True):
    """Prefill quantise-and-pack of one K tensor of the layer shape: read as the strided key block of
    a fused projection output (what the attention forward hands over), or as a contiguous (B, T, H, D)
    tensor; priced against the read-once roofline."""
    B, Hq, Hkv, D, T, R, S = shape
    dev = torch.device("cuda:0")
    G = Hq // Hkv
    if contiguous:
        k_view = torch.randn((B, T, Hkv, D), device=dev, dtype=torch.bfloat16)
    else:
        proj = torch.randn((B, T, Hkv, G + 2, D), device=dev, dtype=torch.bfloat16)
        k_view = proj[..., -2, :]
    clip = 0.5 if bits == 1 else 1.0
    ms = _time_fn(torch, lambda: ops.quantize_pack(k_view, bits, clip), steps, warmup)
    rd = B * T * Hkv * D * 2 + B * Hkv * T * D * bits // 8
    res = {"us_per_tensor": round(ms * 1e3, 1), "algorithmic_bytes": rd, "achieved_GBps": round(rd / ms / 1e6, 1),
           "frac_of_hbm_peak": round(rd / ms / 1e6 / HBM_PEAK_GBPS, 4), "bits": bits,
           "input": "contiguous (B, T, H, D)" if contiguous else "key block of the fused projection output"}
    if rope and T <= ops.ROPE_FUSED_MAX_T:
        # keys: rotary embedding fused into the pass (un-rotated keys read once, rotated rows written once)
        t = torch.arange(T + 41, device=dev, dtype=torch.float32)
        inv = 1.0 / (1e6 ** (torch.arange(0, D, 2, device=dev).float() / D))
        emb = torch.cat([torch.outer(t, inv)] * 2, dim=-1)
        cos, sin = emb.cos().to(torch.bfloat16), emb.sin().to(torch.bfloat16)
        k_rot = ops.empty_token_rows(B, T, Hkv, D, torch.bfloat16, dev)   # as the patched forward allocates it
        ms_f = _time_fn(torch, lambda: ops.rope_quantize_pack(k_view, cos, sin, 41, k_rot, bits, clip), steps, warmup)
        ms_r = _time_fn(torch, lambda: ops.rope_rows(k_view, cos, sin, 41, out=k_rot), steps, warmup)
        ms_q = _time_fn(torch, lambda: ops.quantize_pack(k_rot, bits, clip), steps, warmup)
        rdf = rd + B * T * Hkv * D * 2      # + the rotated rows written once
        res["with_rotary_embedding"] = {
            "fused_us_per_tensor": round(ms_f * 1e3, 1), "algorithmic_bytes": rdf,
            "achieved_GBps": round(rdf / ms_f / 1e6, 1), "frac_of_hbm_peak": round(rdf / ms_f / 1e6 / HBM_PEAK_GBPS, 4),
            "two_step_us_per_tensor": round((ms_r + ms_q) * 1e3, 1),
            "note": "fused: cq_rope_quantize_pack; two-step: cq_rope_rows, then cq_quantize_pack on the rotated tensor"}
    return res


def side_legs(torch, ops, shape, bits, sets, settle_ms=0.0, only_token=False):
    """Figures next to the headline one, same layer shape: the prefill quantise-and-pack of one
    K tensor read as the strided key block of a fused projection output (read-once roofline),
    and the decode kernel on per-token values (`v_mode = token`)."""
    B, Hq, Hkv, D, T, R, S = shape
    dev = torch.device("cuda:0")
    G = Hq // Hkv
    res = {}
    if not only_token:
        res["prefill_quantize_pack"] = prefill_leg(torch, ops, shape, bits)
    proj = torch.randn((B, T, Hkv, G + 2, D), device=dev, dtype=torch.bfloat16)
    k_view, v_view = proj[..., -2, :], proj[..., -1, :]
    ms_t = _time_fn(torch, lambda: ops.quantize_pack_token(v_view, bits), 40, 10)
    # per-token values: every buffer set gets values of its own, so the calls rotate over as many
    # distinct code buffers as the headline measurement does
    calls = []
    for i, x in enumerate(sets):
        vv = torch.randn((B, T, Hkv, D), device=dev, dtype=torch.bfloat16)
        words, vsc, vmn = ops.quantize_pack_token(vv, bits)
        del vv
        calls.append(ops.DecodeCall(x["q"], x["ck"], words, x["sk"], x["zk"], vsc, vmn, x["kr"], x["vr"],
                                    sprompt_len=S, bits=bits, v_mode="token"))
    del proj, k_view, v_view
    ms_d, _ = time_calls(torch, calls, 200, 20, settle_ms, 5)
    nb = algorithmic_bytes(B, Hq, Hkv, D, T, R, bits) - 2 * B * Hkv * D * 2 + 2 * B * Hkv * T * (D // 32) * 2
    res["per_token_values"] = {"quantize_pack_token_us": round(ms_t * 1e3, 1), "decode_us_layer": round(ms_d * 1e3, 2),
                               "algorithmic_bytes": nb, "achieved_GBps": round(nb / ms_d / 1e6, 1),
                               "frac_of_hbm_peak": round(nb / ms_d / 1e6 / HBM_PEAK_GBPS, 4),
                               "launch_plan": calls[0].plan(), "note": f"{len(calls)} buffer sets"}
    del calls
    if only_token:
        return res
    # the other bit width of the same layer shape (the benchmark's layer configuration names b = 1 and b = 2)
    ob = 2 if bits == 1 else 1
    osets = build_sets(torch, ops, shape, ob, 2 if ob == 2 else len(sets), 4321)
    ocalls = [ops.DecodeCall(x["q"], x["ck"], x["cv"], x["sk"], x["zk"], x["sv"], x["zv"], x["kr"], x["vr"],
                             sprompt_len=S, bits=ob) for x in osets]
    ms_o, _ = time_calls(torch, ocalls, 200, 20, settle_ms, 5)
    nbo = algorithmic_bytes(B, Hq, Hkv, D, T, R, ob)
    res[f"decode_{ob}bit"] = {"us_layer": round(ms_o * 1e3, 2), "algorithmic_bytes": nbo,
                              "achieved_GBps": round(nbo / ms_o / 1e6, 1),
                              "frac_of_hbm_peak": round(nbo / ms_o / 1e6 / HBM_PEAK_GBPS, 4),
                              "launch_plan": ocalls[0].plan(), "note": f"{len(osets)} buffer sets"}
    return res


def cpu_baseline(torch, sets, shape, bits, budget_s=12.0):
    """C port of the oracle on this host's cores, on a bounded sample: the
    first `bs` batch rows of the workload; the per-layer figure is scaled
    linearly to the full batch (batch rows are independent)."""
    from oracle import c_port
    c_port.build()
    B, Hq, Hkv, D, T, R, S = shape
    bs = min(B, 4)
    s0 = sets[0]
    f = lambda t: None if t is None else t[:bs].float().cpu().numpy()  # noqa: E731
    args = (f(s0["q"]), s0["ck"][:bs].cpu().numpy(), s0["cv"][:bs].cpu().numpy(), f(s0["sk"]), f(s0["zk"]),
            f(s0["sv"]), f(s0["zv"]), f(s0["kr"]), f(s0["vr"]), S, bits)
    cores = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    t0 = time.perf_counter()
    c_port.decode_attention(*args)
    first = time.perf_counter() - t0
    reps = max(3, min(50, int(budget_s / max(first, 1e-3))))
    times = []
    for _ in range(reps):
        t0 = time.perf_counter()
        c_port.decode_attention(*args)
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    return {"value": round(med * 1e6 * B / bs, 1), "unit": "us/layer", "cores": cores, "kind": "port",
            "sample": f"oracle/cq_oracle.c (OpenMP) on {bs} of {B} batch rows, median of {reps} runs, "
                      f"scaled x{B // bs} to the full batch"}


def cpu_reference_config(torch, ops, seed=1234):
    """The CPU-runnable reference configuration, CPU and GPU side by side: batch 1, 32 query / 8 KV
    heads, head_dim 128, 1 024 tokens, fp16, K / V ~ N(0,1) with four key channels per kv-head scaled
    x10, 1-bit codes (clip 0.5 / 0.3), calibration offsets (-3, 0), no window.  The C port of the
    oracle on the host cores and the HIP path on the GPU run on the same packed state."""
    import numpy as np
    from oracle import c_port, cq_oracle as O
    B, Hq, Hkv, D, T = 1, 32, 8, 128, 1024
    k, v = O.synth_kv(B, T, Hkv, D, "fp16", seed=seed, outliers=4, outlier_kind="x10")
    q = O.round_to(np.random.default_rng(seed + 1).standard_normal((B, Hq, D), dtype=np.float32), "fp16")
    g = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(torch.float16).cuda()  # noqa: E731
    ck, sk, zk = ops.quantize_pack(g(k), 1, 0.5)
    cv, sv, zv = ops.quantize_pack(g(v), 1, 0.3)
    call = ops.DecodeCall(g(q), ck, cv, sk, zk, sv, zv, None, None, sprompt_len=0, bits=1)
    gpu_ms = _time_fn(torch, call.run, 200, 20)
    out = call.run().float().cpu().numpy()
    f = lambda t: t.float().cpu().numpy()  # noqa: E731
    args = (q, ck.cpu().numpy(), cv.cpu().numpy(), f(sk), f(zk), f(sv), f(zv), None, None, 0, 1)
    c_port.build()
    want = c_port.decode_attention(*args)
    times = []
    for _ in range(30):
        t0 = time.perf_counter()
        c_port.decode_attention(*args)
        times.append(time.perf_counter() - t0)
    times.sort()
    err = np.abs(out - want)
    return {"workload": "cpu-reference-config-b1-kv1024-fp16", "cpu_us_layer": round(times[len(times) // 2] * 1e6, 1),
            "gpu_us_layer": round(gpu_ms * 1e3, 2), "launch_plan": call.plan(),
            "max_abs_gpu_vs_cpu": float(err.max()), "mean_abs_gpu_vs_cpu": float(err.mean()),
            "sample": "whole configuration, median of 30 CPU runs"}


def model_leg(torch, batch=64, tiles=13, sys_len=41, text_len=23, new_tokens=128, seed=1234, model_name="8b"):
    """InternVL2.5-8B-shaped decode (InternLM2.5-7B language model: 32 layers, hidden 4096, 32/8
    heads, head_dim 128, vocab 92 553; InternViT-300M-shaped vision tower), random-init bf16 weights,
    synthetic uniform-noise tiles: tokens/s of `new_tokens` greedy steps at `batch`, prefill
    excluded, 1-bit KV (patched attention) vs full-precision KV (unpatched) on the same weights."""
    from calibquant_amd import patch_internvl as pi
    from calibquant_amd.internlm2 import InternLM2Attention, InternLM2Config, InternVLChatStandIn
    dev = torch.device("cuda:0")
    torch.manual_seed(seed)
    prev = torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)
    try:
        with torch.device(dev):
            from calibquant_amd.internvit import InternViTConfig
            cfg = InternLM2Config.internvl2_5_26b() if model_name == "26b" else InternLM2Config.internvl2_5_8b()
            vit = InternViTConfig.internvit_6b() if model_name == "26b" else InternViTConfig.internvit_300m()
            model = InternVLChatStandIn(cfg, vit=vit).eval()
    finally:
        torch.set_default_dtype(prev)
    T = tiles * 256
    N = sys_len + T + text_len
    ids = torch.randint(0, 90000, (batch, N), device=dev)
    ids[:, sys_len:sys_len + T] = model.img_context_token_id
    fp_forward, fp_generate = InternLM2Attention.forward, InternVLChatStandIn.generate
    res = {"model": "internvl2.5-" + model_name + "-shaped", "prompt_tokens": N, "image_tokens": T,
           "new_tokens": new_tokens, "batch": batch,
           "vision_tower": "internvit-6b-shaped" if model_name == "26b" else "internvit-300m-shaped"}

    def features():
        vis = []
        # vision features tile-chunked per sample to bound the pixel tensor
        for b0 in range(0, batch, 8):
            pix = torch.rand((8 * tiles, 3, 448, 448), device=dev, dtype=torch.bfloat16)
            vis.append(model.extract_feature(pix))
        return torch.cat(vis, 0)

    def drop_state():
        for layer in model.language_model.model.layers:      # drop the KV state before the next run
            for name in ("_kv", "_cq_window", "_cq_call", "_cq_step", "_cq_stats", "encoded_features_k", "encoded_features_v"):
                if hasattr(layer.attention, name):
                    delattr(layer.attention, name)
        torch.cuda.empty_cache()

    def run_eager(tag, patched):
        """The reference's way: an eager host loop, one launch sequence per layer per token."""
        stamps = []

        def on_step(i):
            if i == 0 or i == new_tokens - 1:     # only the two ends of the decode loop synchronise
                torch.cuda.synchronize()
                stamps.append(time.perf_counter())

        with torch.no_grad():
            vit = features()
            if patched:
                out = pi.custom_generate(model, pixel_values=torch.empty(0), input_ids=ids, visual_features=vit,
                                         max_new_tokens=new_tokens, on_step=on_step)
            else:
                emb = model.language_model.get_input_embeddings()(ids)
                emb[ids == model.img_context_token_id] = vit.reshape(-1, emb.shape[-1])
                out = model.language_model.generate(inputs_embeds=emb, max_new_tokens=new_tokens, on_step=on_step)
        assert out.shape == (batch, new_tokens)
        # stamps[0] closes the prefill; the decode steps are the intervals after it
        dt = stamps[-1] - stamps[0]
        res[tag + "_eager_decode_tok_s"] = round(batch * (new_tokens - 1) / dt, 1)
        res[tag + "_eager_ms_per_token_step"] = round(dt / (new_tokens - 1) * 1e3, 3)
        drop_state()

    def run_graph(tag, patched, fp_kernel=False):
        """The decode step recorded once as a HIP graph and replayed per token; timed over the
        replays only (the first decode step runs eagerly and the recording follows it)."""
        from calibquant_amd.graph_decode import StaticDecoder
        stamps = []
        first_replay = 2

        def on_step(i):
            if i == first_replay or i == new_tokens - 1:
                torch.cuda.synchronize()
                stamps.append(time.perf_counter())

        lm = model.language_model
        with torch.no_grad():
            vit = features()
            emb = lm.get_input_embeddings()(ids)
            emb[ids == model.img_context_token_id] = vit.reshape(-1, emb.shape[-1])
            if patched:
                for layer in lm.model.layers:
                    layer.attention.cq_image_token_num = T
            pos = torch.arange(N, device=dev)[None].expand(batch, N)
            logits, past = lm.forward_step(emb, pos, None)
            del emb, vit
            first = logits[:, -1].argmax(-1)
            dec = StaticDecoder(lm, past, N, new_tokens, fp_kernel=fp_kernel)
            del past
            drop_state()
            out = dec.generate(first, new_tokens, use_graph=True, on_step=on_step)
        assert out.shape == (batch, new_tokens)
        steps = new_tokens - 1 - first_replay
        dt = stamps[-1] - stamps[0]
        res[tag + "_decode_tok_s"] = round(batch * steps / dt, 1)
        res[tag + "_ms_per_token_step"] = round(dt / steps * 1e3, 3)
        del dec
        drop_state()

    try:
        # Full-precision KV runs eagerly only: its step is bound by the attention kernel's HBM
        # reads (not by the host), and torch's attention over a fixed-capacity cache with a
        # length mask - what a recorded step would need - falls back to a much slower kernel.
        run_eager("fp16_kv", False)
        res["fp16_kv_decode_tok_s"] = res["fp16_kv_eager_decode_tok_s"]
        # ... and the same full-precision cache read by this library's own attention kernel (every
        # token a row of its full-precision window), step recorded as a HIP graph: the stronger baseline
        run_graph("fp16_kv_own_kernel", False, fp_kernel=True)
        import contextlib, io
        with contextlib.redirect_stdout(io.StringIO()):
            pi.patch_model(model, "calibquant")
        run_eager("kv_1bit", True)
        run_graph("kv_1bit", True)
    finally:
        InternLM2Attention.forward, InternVLChatStandIn.generate = fp_forward, fp_generate
    res["note"] = ("kv_1bit_decode_tok_s: decode step replayed as a HIP graph; *_eager_*: eager host loop through the "
                   "patched forward (1-bit: one call into the host shim per layer and token; fp16: torch SDPA, bound by "
                   "that attention kernel); fp16_kv_own_kernel_*: full-precision cache through this library's attention "
                   "kernel, HIP graph")
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--bits", type=int, default=1, choices=(1, 2))
    ap.add_argument("--workload", default=DEFAULT_WORKLOAD, choices=sorted(WORKLOADS))
    ap.add_argument("--sets", type=int, default=4, help="distinct input buffer sets rotated through")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-fp16kv", action="store_true", help="skip the fp16-KV comparison leg")
    ap.add_argument("--no-model", action="store_true", help="skip the full-model decode tok/s leg")
    ap.add_argument("--model", default="8b", choices=("8b", "26b"),
                    help="language-model shape of the full-model leg (26b: 48 layers, hidden 6144, 48/8 heads)")
    ap.add_argument("--no-side", action="store_true", help="skip the prefill / per-token-value side figures")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also launch three 256 MiB device copies (known traffic, for scaling profiler byte counters)")
    ap.add_argument("--settle-ms", type=float, default=300.0,
                    help="untimed run of the same calls before the warm-up steps, in ms of device time")
    ap.add_argument("--blocks", type=int, default=25,
                    help="timed blocks of --steps calls each; the median block is reported")
    ap.add_argument("--only", default=None, choices=("prefill", "prefill-contiguous", "token-values"),
                    help="run one side figure alone (for profiling it) and print its JSON")
    ap.add_argument("--seed", type=int, default=1234)
    a = ap.parse_args()
    if a.gpus != 1:
        print(f"bench.py: this build measures one GPU only (asked for {a.gpus}); "
              "the path shards over batch rows and kv-heads without any exchange between GPUs", file=sys.stderr)
        sys.exit(2)

    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)
    from calibquant_amd import ops

    shape = WORKLOADS[a.workload]
    B, Hq, Hkv, D, T, R, S = shape
    if a.copy_calibration:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda").random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    if a.only in ("prefill", "prefill-contiguous"):
        print(json.dumps(prefill_leg(torch, ops, shape, a.bits, a.steps, a.warmup, a.only == "prefill-contiguous")))
        return
    sets = build_sets(torch, ops, shape, a.bits, a.sets, a.seed)
    if a.only == "token-values":
        print(json.dumps(side_legs(torch, ops, shape, a.bits, sets, a.settle_ms, only_token=True)))
        return
    calls = [ops.DecodeCall(s["q"], s["ck"], s["cv"], s["sk"], s["zk"], s["sv"], s["zv"], s["kr"], s["vr"],
                            sprompt_len=S, bits=a.bits) for s in sets]
    # the same K steps after W warm-up calls straight after the inputs were built (no settling run, one
    # block): the protocol of a cold process, reported next to the steady-state figure
    ms_cold, _ = time_calls(torch, calls, a.steps, a.warmup, 0.0, 1)
    ms, per_block = time_calls(torch, calls, a.steps, a.warmup, a.settle_ms, a.blocks)
    plan = calls[0].plan()
    nbytes = algorithmic_bytes(B, Hq, Hkv, D, T, R, a.bits)
    gbps = nbytes / (ms * 1e-3) / 1e9

    out = {
        "metric": METRIC,
        "value": round(ms * 1e3, 3),
        "unit": "us/layer",
        "n_gpus": 1,
        "steps": a.steps,
        "warmup": a.warmup,
        "ms_per_step": round(ms, 6),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": a.workload, "batch": B, "q_heads": Hq, "kv_heads": Hkv, "head_dim": D,
                   "kv_packed_tokens": T, "kv_residual_rows": R, "bits": a.bits, "storage_dtype": "bf16",
                   "buffer_sets": a.sets, "settle_ms": a.settle_ms, "timed_blocks": a.blocks,
                   "timing": f"median of {a.blocks} timed blocks of {a.steps} steps each, after {a.settle_ms:g} ms of "
                             f"the same calls untimed and {a.warmup} warm-up steps",
                   "launches_per_step": plan["launches"], "launch_plan": plan},
        "value_unsettled_us": round(ms_cold * 1e3, 3),
        "value_blocks_us": {"min": round(per_block[0] * 1e3, 3), "max": round(per_block[-1] * 1e3, 3)},
        "roofline": {"bound": "hbm", "achieved": round(gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(gbps / HBM_PEAK_GBPS, 4), "traffic": measured_traffic(a.workload, a.bits),
                     "traffic_source": "profiles/decode_kernel_traffic.json (rocprofv3 FETCH_SIZE / WRITE_SIZE of an "
                                       "earlier run of this workload, scaled by a 256 MiB copy; not measured by this run)",
                     "algorithmic_bytes": nbytes},
    }
    if not a.no_fp16kv:
        try:
            fp_ms = time_fp16_kv(torch, shape, max(20, a.steps // 4), max(5, a.warmup // 4), a.sets)
            out["fp16_kv_us_layer"] = round(fp_ms * 1e3, 2)
            out["speedup_vs_fp16_kv"] = round(fp_ms / ms, 2)
            own_ms = time_fp16_kv_own(torch, ops, shape, max(20, a.steps // 4), max(5, a.warmup // 4), a.sets)
            out["fp16_kv_own_kernel_us_layer"] = round(own_ms * 1e3, 2)
            out["speedup_vs_fp16_kv_own_kernel"] = round(own_ms / ms, 2)
        except Exception as e:  # the comparison leg must not sink the measurement
            out["fp16_kv_us_layer"] = None
            out["fp16_kv_error"] = repr(e)[:200]
    if not a.no_cpu:
        out["cpu_baseline"] = cpu_baseline(torch, sets, shape, a.bits)
        try:
            out["cpu_baseline"]["reference_config"] = cpu_reference_config(torch, ops, a.seed)
        except Exception as e:  # must not sink the measurement
            out["cpu_baseline"]["reference_config"] = {"error": repr(e)[:200]}
    if not a.no_side:
        try:
            out["side_legs"] = side_legs(torch, ops, shape, a.bits, sets, a.settle_ms)
        except Exception as e:  # side figures must not sink the measurement
            out["side_legs"] = {"error": repr(e)[:300]}
    if not a.no_model and a.workload == DEFAULT_WORKLOAD and a.bits == 1:
        del sets, calls
        torch.cuda.empty_cache()
        try:
            if a.model == "26b":   # InternLM2-20B-shaped: 3 images = 39 tiles, 41 + 23 text tokens, batch 16, 64 new tokens
                out["model_decode"] = model_leg(torch, batch=16, tiles=39, new_tokens=64, model_name="26b")
            else:
                out["model_decode"] = model_leg(torch)
        except Exception as e:  # the model leg must not sink the kernel measurement
            out["model_decode"] = {"error": repr(e)[:300]}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
