#!/usr/bin/env python3
"""Benchmark of the quantized-KV decode-attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2|c2-paged|c2-prologue|c2-ragged|c1|c4|c4-prologue|b1-32k|b4-16k|d256-int8|d256-fp8|d64-int8|c3|c3-prompt|c3-fp8|c3-d256|c3-d64|c3-b1|c3-b1-shadow|c3-prologue|c3-shadow|c3-fp8-shadow|c5-decode|c5-decode-layer|c5-decode-layer-3calls|c5-prefill|c5-prefill-norm|c5-prefill-layer|c5-prefill-recurrent]

One "step" is one pass of the hot path over one batch: quantize-on-write of one new token per
sequence into the int8 cache, then dequant-fused GQA decode attention over the whole context
(one attention layer).  The default workload is the headline configuration: batch 64, 32 query
heads, 8 KV heads, head_dim 128, every context 8192, int8 KV with per-token-per-head fp32 scales,
K/V source N(0,1) with 1 % outliers at 8 sigma, seeded synthetic data generated on the device.

The timed region starts with all inputs resident in HBM.  Four copies of the cache at different
addresses are rotated through so that no launch finds its data in the last-level cache.

Prints ONE JSON line.  `value` is algorithmic HBM bytes per step / step time (GB/s); the line also
carries tokens/s, the roofline of the dominant kernel (HIP events around that kernel alone, on the
stream it runs on) and the CPU baseline: the reference's libtorch op sequence (dequantize, GQA
expand, fp32 matmul/softmax/matmul) timed on this machine's host cores on a bounded sample.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E peak


def settle(torch, step, window=20, min_launches=300, max_launches=4000, tol=0.01):
    """Untimed settling phase, independent of --warmup: the first few hundred launches after set-up run a few per
    cent slower (clocks and memory settle).  Runs `step(i)` in windows of `window` launches, each window timed with
    a pair of events on the launch stream, until at least `min_launches` have run and three consecutive windows
    agree within `tol` (or `max_launches` is reached).  Returns (launches run, last window's us per launch)."""
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    hist, n = [], 0
    while n < max_launches:
        e0.record()
        for i in range(window):
            step(n + i)
        e1.record()
        e1.synchronize()
        n += window
        hist.append(e0.elapsed_time(e1) / window * 1e3)
        if n >= min_launches and len(hist) >= 3:
            last = hist[-3:]
            if max(last) - min(last) <= tol * min(last):
                break
    return n, hist[-1]

WORKLOADS = {
    # name: (B, Hq, Hkv, D, T, ragged, fp8, sigma, outliers)
    "c2": (64, 32, 8, 128, 8192, False, False, 1.0, True),
    "c2-ragged": (64, 32, 8, 128, 8192, True, False, 1.0, True),
    "c1": (1, 32, 8, 128, 2048, False, False, 1.0, False),
    "c4": (32, 64, 8, 128, 32768, False, True, 0.5, False),
    # one sequence with a long context: the reference's usual serving shape (a single stream), split-K over 512 workgroups
    "b1-32k": (1, 32, 8, 128, 32768, False, False, 1.0, True),
    "b4-16k": (4, 32, 8, 128, 16384, False, False, 1.0, True),
    # the head shape of Qwen3.5's full-attention layers (16 query / 4 KV heads of 256), same cache bytes as c2 / half of c4
    "d256-int8": (64, 16, 4, 256, 8192, False, False, 1.0, True),
    "d256-fp8": (32, 16, 4, 256, 32768, False, True, 0.5, False),
    # 64-wide heads (the reference's paged-cache tests use them), same cache bytes as c2
    "d64-int8": (64, 32, 16, 64, 8192, False, False, 1.0, True),
    # c2 with the cache in 256-token blocks scattered through a pool (the reference's BlockPool geometry,
    # kv_cache.rs:477): the same bytes, every wavefront step resolved through the block table
    "c2-paged": (64, 32, 8, 128, 8192, False, False, 1.0, True),
    # c2 with q and the new K row arriving as projected: per-head QK-norm (Llama flavour) and the rotary embedding run
    # inside the decode-step launch (hs_decode_step_int8_prologue)
    "c2-prologue": (64, 32, 8, 128, 8192, False, False, 1.0, True),
    # c4 the same way over the FP8 cache (hs_decode_step_fp8_prologue): the step a Qwen3-style layer runs
    "c4-prologue": (32, 64, 8, 128, 32768, False, True, 0.5, False),
}


def make_source(torch, gen, shape, sigma, outliers, dev):
    x = torch.randn(shape, generator=gen, device=dev, dtype=torch.float32) * sigma
    if outliers:
        m = torch.rand(shape, generator=gen, device=dev) < 0.01
        x = torch.where(m, torch.sign(x) * (8.0 * sigma), x)
    return x.to(torch.bfloat16)


def cpu_baseline(torch, name, caches, q, lens, Hq, fp8, seconds_budget=12.0):
    """Reference op sequence on the host cores, on the first rows of the same workload."""
    from oracle import reference_path as ref
    B = q.shape[0]
    T = int(lens.max())
    bs = min(B, 4 if T <= 8192 else 1)
    kc, vc, ks, vs = caches
    kc_h = kc[:bs, :, :T].permute(0, 2, 1, 3).contiguous().cpu()
    vc_h = vc[:bs, :, :T].permute(0, 2, 1, 3).contiguous().cpu()
    if fp8:
        ks_h, vs_h = ks[:bs].cpu(), vs[:bs].cpu()
    else:
        ks_h = ks[:bs, :, :T].permute(0, 2, 1).contiguous().cpu()
        vs_h = vs[:bs, :, :T].permute(0, 2, 1).contiguous().cpu()
    q_h = q[:bs].cpu().unsqueeze(1)
    lens_h = [int(x) for x in lens[:bs].cpu()]
    ragged = len(set(lens_h)) > 1 or lens_h[0] != T

    def run():
        if fp8:
            return ref.decode_attention_fp8(q_h, kc_h, vc_h, ks_h, vs_h)
        return ref.decode_attention_int8(q_h, kc_h, vc_h, ks_h, vs_h, lens_h if ragged else None)

    run()  # warm-up
    times = []
    t_start = time.perf_counter()
    while len(times) < 64 and (time.perf_counter() - t_start < seconds_budget or len(times) < 3):  # about ten seconds of host work
        t0 = time.perf_counter()
        out = run()
        times.append(time.perf_counter() - t0)
    med = float(np.median(times))
    from hyprstream_amd import workloads as wl
    Hkv, D = kc.shape[1], kc.shape[3]
    nbytes = (wl.decode_bytes_fp8 if fp8 else wl.decode_bytes_int8)(np.array(lens_h), Hq, Hkv, D)
    cpu_model = "unknown"
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    cpu_model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    return {
        "value": nbytes / med / 1e9, "unit": "GB/s", "cores": int(torch.get_num_threads()), "kind": "port",
        "nproc": int(os.cpu_count() or 0), "intra_op_threads": int(torch.get_num_threads()), "cpu_model": cpu_model,
        "sample": "first %d of %d sequences of workload %s (T=%d): libtorch CPU dequantize + GQA expand + fp32 "
                  "matmul/softmax/matmul, median of %d runs, %.1f ms per call, %.1f tokens/s"
                  % (bs, B, name, T, len(times), med * 1e3, bs / med),
        "tokens_per_s": bs / med, "ms_per_call": med * 1e3,
    }, out


def bench_prefill(args, torch, hb, wl, C=512, fp8=False, d256=False, d64=False, b1=False, prologue=False, shadow=False):
    """Config 3: chunked causal prefill, B=4 x 4096 tokens in 512-token chunks, Hq 32 / Hkv 8, D 128.
    One step = all eight chunk calls of one layer (attention + quantize-on-write of every chunk).
    Variants: C = 4096 (the whole prompt in one call), fp8 = an e4m3fn cache with per-head scales, d256 = the head
    shape of Qwen3.5's full-attention layers (Hq 16 / Hkv 4, D 256: the same flops and bytes), prologue = q and k arrive
    as projected and every chunk call is preceded by the QK-norm + rotary pre-pass (hs_qk_prologue_apply, Llama-flavour
    norm, whole-head rotation); the pre-pass is inside the timed step, the roofline figure stays the attention kernel's;
    shadow = the calls also keep a bf16 operand-order copy of the prompt's dequantized K/V (hs_kv_layout.prefill_shadow,
    2 x the int8 bytes, for the duration of the prompt) and read the history from it instead of converting codes."""
    dev = "cuda:0"
    B, T, Hq, Hkv, D = (4, 4096, 16, 4, 256) if d256 else (4, 4096, 32, 8, 64) if d64 else (1 if b1 else 4, 4096, 32, 8, 128)
    gen = torch.Generator(device=dev)
    gen.manual_seed(wl.SEED)
    sigma = 0.5 if fp8 else 1.0
    q = torch.randn(B, T, Hq, D, generator=gen, device=dev, dtype=torch.float32).to(torch.bfloat16)
    k = (sigma * torch.randn(B, T, Hkv, D, generator=gen, device=dev, dtype=torch.float32)).to(torch.bfloat16)
    v = (sigma * torch.randn(B, T, Hkv, D, generator=gen, device=dev, dtype=torch.float32)).to(torch.bfloat16)
    chunks = [(q[:, i:i + C].contiguous(), k[:, i:i + C].contiguous(), v[:, i:i + C].contiguous()) for i in range(0, T, C)]
    lay = hb.contiguous_layout(Hkv, T, D)
    kc = torch.zeros(B, Hkv, T, D, dtype=torch.uint8 if fp8 else torch.int8, device=dev)
    vc = torch.zeros_like(kc)
    if fp8:
        ks = torch.zeros(B, Hkv, dtype=torch.float32, device=dev)
        vs = torch.zeros_like(ks)
        hb.kv_fp8_calibrate(chunks[0][1], chunks[0][2], ks, vs)  # per-head scales from the first chunk
    else:
        ks = torch.zeros(B, Hkv, lay.scale_stride_head, dtype=torch.float32, device=dev)
        vs = torch.zeros_like(ks)
    outs = [torch.empty(B, C, Hq, D, dtype=torch.bfloat16, device=dev) for _ in chunks]
    scale = 1.0 / float(np.sqrt(D))
    # scratch for the key split of calls with few query tiles (the library decides per call; --key-splits 1 = never)
    split_ws = hb.prefill_split_workspace(B, C, Hq, Hkv, D)
    shadow_buf = hb.prefill_shadow(B, Hkv, D, T) if shadow else None
    if prologue:
        inv = 1.0 / (10000.0 ** (torch.arange(0, D, 2, device=dev, dtype=torch.float32) / D))
        ang = torch.arange(T, device=dev, dtype=torch.float32)[:, None] * inv[None, :]
        sin, cos = ang.sin().to(torch.bfloat16).contiguous(), ang.cos().to(torch.bfloat16).contiguous()
        qw = (1.0 + 0.1 * torch.randn(D, generator=gen, device=dev)).to(torch.bfloat16)
        kw = (1.0 + 0.1 * torch.randn(D, generator=gen, device=dev)).to(torch.bfloat16)
        pro = hb.qk_prologue(hb.QKNORM_LLAMA, 1e-6, qw, kw, sin, cos)
        # The projections of a prompt give q and k for all of its tokens at once (llama.rs:560-611 runs norm and rotation
        # on the whole [B, T, H, D] tensors before cache.update), so the pre-pass is ONE launch over the prompt: the eight
        # chunks' rows laid end to end as 8 B "sequences" of C tokens whose first positions are 0, C, 2C, ...; the chunk
        # calls read their slices of its output.  --prologue-fused-q sends only k through the pre-pass and lets the
        # chunk launches normalise and rotate q themselves (hs_kv_layout.prefill_q_prologue); --prologue-per-chunk runs
        # the q + k pre-pass in front of every chunk call instead of once (eight launches of an eighth of the rows).
        nch = len(chunks)
        q_all = torch.cat([c[0] for c in chunks], 0).contiguous()   # [nch * B, C, Hq, D]
        k_all = torch.cat([c[1] for c in chunks], 0).contiguous()
        q_rot, k_rot = torch.empty_like(q_all), torch.empty_like(k_all)
        first_pos = (torch.arange(nch * B, device=dev, dtype=torch.int32) // B * C).contiguous()
    q_prepass = not args.prologue_fused_q or args.prologue_per_chunk

    def step(write=True, with_prologue=True):
        if prologue and with_prologue and not args.prologue_per_chunk:
            if q_prepass:
                hb.qk_prologue_apply(q_all, k_all, pro, q_rot, k_rot, first_pos, 0)
            else:
                hb.qk_prologue_apply(None, k_all, pro, None, k_rot, first_pos, 0)
        for i, (qc, kcn, vcn) in enumerate(chunks):
            fused = None
            if prologue and with_prologue:
                kcn = k_rot[i * B:(i + 1) * B]
                if q_prepass:
                    qc = q_rot[i * B:(i + 1) * B]
                    if args.prologue_per_chunk:
                        hb.qk_prologue_apply(chunks[i][0], chunks[i][1], pro, qc, kcn, None, i * C)
                else:
                    fused = pro
            hb.prefill_attn(qc, kcn, vcn, kc, vc, ks, vs, lay, i * C, outs[i], scale, write, fp8=fp8, q_prologue=fused,
                            split_workspace=split_ws, key_splits=args.key_splits, shadow=shadow_buf)

    settle(torch, lambda i: step(), window=10, min_launches=100, max_launches=1000)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / args.steps * 1e3
    flops = 4 * B * Hq * D * T * (T + 1) // 2  # causal half, QK^T + PV
    # attention kernel alone (no quantize-on-write), HIP events on its stream
    n_ev = 50
    e0 = [torch.cuda.Event(enable_timing=True) for _ in range(n_ev)]
    e1 = [torch.cuda.Event(enable_timing=True) for _ in range(n_ev)]
    for i in range(n_ev):
        e0[i].record()
        step(write=shadow, with_prologue=False)  # (the copy is appended by the cache write: with it the write stays in)
        e1[i].record()
    torch.cuda.synchronize()
    kms = float(np.mean([a.elapsed_time(b) for a, b in zip(e0, e1)]))
    peak = 2500.0
    res = {
        "metric": "prefill-attn TFLOP/s (%% bf16 MFMA peak) + tokens/s, B=%d x 4096 in %d-chunks, Llama-3-8B shape" % (B, C),
        "value": flops / (ms * 1e-3) / 1e12, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": ("bf16 MFMA (new tokens; history from the bf16 copy of the dequantized %s cache), f32 accumulate" if shadow else
                  "bf16 MFMA (new tokens) + f16 MFMA over %s codes (history), f32 accumulate") % ("fp8" if fp8 else "int8"),
        "data": "synthetic (seeded, generated on device)",
        "config": {"workload": "c3%s: chunked causal prefill B=%d T=4096 chunk=%d Hq=%d Hkv=%d D=%d, %s cache of earlier "
                               "chunks + own bf16 K/V, quantize-on-write, one layer"
                               % ("-b1-shadow" if shadow and b1 else "-fp8-shadow" if shadow and fp8 else "-prologue with the prompt copy" if shadow and prologue else "-shadow" if shadow else "-prologue" if prologue else "-d256" if d256 else "-d64" if d64 else "-b1" if b1 else "-fp8" if fp8 else "-prompt" if C == T else "", B, C, Hq, Hkv, D,
                                  "fp8 e4m3fn" if fp8 else "int8"),
                   "algorithmic_flops_per_step": int(flops)},
        "tokens_per_s": B * T / (ms * 1e-3),
        "roofline": {"bound": "mfma", "kernel": "prefill_attn_kernel (%d chunk launches)" % len(chunks), "achieved": flops / (kms * 1e-3) / 1e12,
                     "peak": peak, "unit": "TFLOP/s", "frac": flops / (kms * 1e-3) / 1e12 / peak, "traffic": None,
                     "avg_us_all_launches": kms * 1e3},
    }
    print(json.dumps(res))


def bench_deltanet(args, torch, hb, wl, prefill, recurrent=False, norm=None):
    """Config 5: gated DeltaNet, nk 16 / nv 32, dk = dv = 128.  Decode: B = 64, one token, fp32 state read and
    written once (HBM bound).  Prefill: B = 4 x 4096 tokens in chunks of 64 on the matrix pipe (c5-prefill), or
    through the token-by-token fp32 recurrence (c5-prefill-recurrent).  norm: the chunked prefill followed by the layer's
    gated RMSNorm as one call (hs_deltanet_forward_chunked_gated_norm, c5-prefill-norm); norm = "layer": the prompt branch
    of the whole layer between its projections, conv1d + SiLU + gates included (hs_deltanet_prefill_layer, c5-prefill-layer)."""
    dev = "cuda:0"
    nk, nv, d = 16, 32, 128
    B, T = (args.batch or 4, 4096) if prefill else (args.batch or 64, 1)
    gen = torch.Generator(device=dev)
    gen.manual_seed(wl.SEED)
    nrm = lambda x: (x / x.norm(dim=-1, keepdim=True).clamp_min(1e-3)).to(torch.bfloat16)
    q = nrm(torch.randn(B, T, nk, d, generator=gen, device=dev))
    k = nrm(torch.randn(B, T, nk, d, generator=gen, device=dev))
    v = torch.randn(B, T, nv, d, generator=gen, device=dev).to(torch.bfloat16)
    g = -torch.nn.functional.softplus(torch.randn(B, T, nv, generator=gen, device=dev))
    beta = torch.sigmoid(torch.randn(B, T, nv, generator=gen, device=dev))
    ncopies = 1 if prefill else max(1, args.copies)
    states = [torch.randn(B, nv, d, d, generator=gen, device=dev) * 0.1 for _ in range(ncopies)]
    out = torch.empty(B, T, nv, d, dtype=torch.float32, device=dev)
    qs = 1.0 / float(np.sqrt(d))

    chunked = prefill and not recurrent
    ws_bytes = (hb.deltanet_chunked_gated_norm_workspace_bytes if norm else hb.deltanet_chunked_workspace_bytes)(B, T, nk, nv)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev) if chunked else None

    if norm:
        z = torch.randn(B, T, nv, d, generator=gen, device=dev).to(torch.bfloat16)
        nw = torch.rand(d, generator=gen, device=dev) + 0.5
        out_n = torch.empty(B, T, nv, d, dtype=torch.bfloat16, device=dev)
    if norm == "layer":
        C = 2 * nk * d + nv * d
        rn = lambda *sh: torch.randn(*sh, generator=gen, device=dev)
        lx, lw, lcs = rn(B, T, C).to(torch.bfloat16), (0.5 * rn(C, 4)).to(torch.bfloat16), rn(B, C, 3).to(torch.bfloat16)
        la, lb = (2 * rn(B, T, nv)).to(torch.bfloat16), (2 * rn(B, T, nv)).to(torch.bfloat16)
        lnae, ldtb = -rn(nv).exp(), rn(nv)
        lws = None

    def step(i):
        if norm == "layer":
            nonlocal lws
            lws = hb.deltanet_prefill_layer(lx, lw, lcs, la, lb, lnae, ldtb, z, nw, 1e-6, states[i % ncopies], nk, nv, d, d, qs, True,
                                            workspace=lws)[2]
        elif norm:
            hb.deltanet_forward_chunked_gated_norm(q, k, v, g, beta, states[i % ncopies], z, nw, 1e-6, out_n, qs, False, workspace=ws)
        elif chunked:
            hb.deltanet_forward_chunked(q, k, v, g, beta, states[i % ncopies], out, qs, False, workspace=ws)
        else:
            hb.deltanet_forward(q, k, v, g, beta, states[i % ncopies], out, qs, False)

    settle(torch, step, window=10 if prefill else 20, min_launches=100 if prefill else 300, max_launches=2000)
    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(i)
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / args.steps * 1e3
    n_ev = 100
    e0 = [torch.cuda.Event(enable_timing=True) for _ in range(n_ev)]
    e1 = [torch.cuda.Event(enable_timing=True) for _ in range(n_ev)]
    for i in range(n_ev):
        e0[i].record()
        step(i)
        e1[i].record()
    torch.cuda.synchronize()
    kms = float(np.mean([a.elapsed_time(b) for a, b in zip(e0, e1)]))
    state_bytes = 2 * B * nv * d * d * 4
    io_bytes = B * T * (2 * nk * d * 2 + nv * d * 2 + 2 * nv * 4 + (nv * d * 2 * 2 if norm else nv * d * 4))
    if norm == "layer":  # mixed q|k|v in, z in, bf16 rows out, the gate inputs, the conv state both ways
        io_bytes = B * T * ((2 * nk * d + nv * d) * 2 + 2 * nv * d * 2 + 2 * nv * 2) + 2 * B * (2 * nk * d + nv * d) * 3 * 2
    nbytes = state_bytes + io_bytes
    res = {
        "metric": "deltanet %s HBM GB/s + tokens/s, nk=16 nv=32 dk=dv=128" % ("prefill" if prefill else "decode"),
        "value": nbytes / (ms * 1e-3) / 1e9, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16 MFMA operands, f32 accumulation, triangular solve and state; bf16 q/k/v" if chunked else "f32 state and arithmetic, bf16 q/k/v",
        "data": "synthetic (seeded, generated on device)",
        "config": {"workload": "c5-%s: gated delta rule B=%d T=%d nk=16 nv=32 dk=dv=128, fp32 state [B,32,128,128]%s%s"
                               % (("prefill-layer" if norm == "layer" else "prefill-norm" if norm else "prefill") if prefill else "decode", B, T,
                                  ", chunk size 64" if chunked else (", token recurrence" if prefill else ""),
                                  ", between conv1d + SiLU + gates and the gated RMSNorm (one call)" if norm == "layer" else
                                  ", then the gated RMSNorm (same call)" if norm else ""),
                   "algorithmic_bytes_per_step": int(nbytes)},
        "tokens_per_s": B * T / (ms * 1e-3),
        "roofline": {"bound": "hbm", "kernel": (("deltanet_conv8 + gates + " if norm == "layer" else "") + "deltanet_chunk_factor_kernel + deltanet_chunk_walk_kernel" + (" + gated_rmsnorm_rows_kernel" if norm else "") if chunked else "deltanet_prefill_kernel") if prefill else "deltanet_decode_kernel", "achieved": nbytes / (kms * 1e-3) / 1e9,
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": nbytes / (kms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                     "traffic": None, "avg_kernel_us": kms * 1e3},
    }
    tpath = os.path.join(ROOT, "profiles", "deltanet_traffic.json")
    wname = ("c5-prefill-layer" if norm == "layer" else "c5-prefill-norm" if norm else "c5-prefill") if chunked else None
    if wname and os.path.exists(tpath):  # both kernels' FETCH_SIZE + WRITE_SIZE per step, recorded under rocprofv3
        try:
            t = json.load(open(tpath)).get(wname)
        except (OSError, ValueError):
            t = None
        if t is not None:
            res["roofline"]["traffic"] = t
            res["roofline"]["traffic_source"] = "recorded rocprofv3 counters: profiles/deltanet_traffic.json (not measured in this run)"
    print(json.dumps(res))


def bench_deltanet_layer(args, torch, hb, wl, fused):
    """The decode branch of a gated-DeltaNet layer between its two projections (Config 5's shape, B = 64 unless --batch):
    conv1d + SiLU + gates for the new token, the recurrent step, the gated RMSNorm.  c5-decode-layer: one launch
    (hs_deltanet_decode_layer); c5-decode-layer-3calls: hs_deltanet_prepare + hs_deltanet_forward + hs_deltanet_gated_norm
    (four launches), the same results bit for bit.  Bytes: the fp32 state read and written once plus the step's
    activations, conv state and weights."""
    dev = "cuda:0"
    nk, nv, d = 16, 32, 128
    B = args.batch or 64
    C = 2 * nk * d + nv * d
    gen = torch.Generator(device=dev)
    gen.manual_seed(wl.SEED)
    rn = lambda *s: torch.randn(*s, generator=gen, device=dev)
    x, w = rn(B, 1, C).to(torch.bfloat16), (0.5 * rn(C, 4)).to(torch.bfloat16)
    cs = [rn(B, C, 3).to(torch.bfloat16), torch.empty(B, C, 3, dtype=torch.bfloat16, device=dev)]
    a_in, b_in = (2 * rn(B, 1, nv)).to(torch.bfloat16), (2 * rn(B, 1, nv)).to(torch.bfloat16)
    nae, dtb = -rn(nv).exp(), rn(nv)
    z, nw = rn(B, 1, nv, d).to(torch.bfloat16), rn(d)
    ncopies = max(1, args.copies)
    states = [rn(B, nv, d, d) * 0.1 for _ in range(ncopies)]
    out = torch.empty(B, 1, nv, d, dtype=torch.bfloat16, device=dev)
    o32 = torch.empty(B, 1, nv, d, dtype=torch.float32, device=dev)
    qs = 1.0 / float(np.sqrt(d))

    def step(i):
        src, dst = cs[i & 1], cs[(i + 1) & 1]
        if fused:
            hb.deltanet_decode_layer(x, w, src, a_in, b_in, nae, dtb, z, nw, 1e-6, states[i % ncopies], nk, nv, d, d, qs, True,
                                     out=out, conv_state_out=dst)
        else:
            q, k, v, g, beta, _ = hb.deltanet_prepare(x, w, src, a_in, b_in, nae, dtb, nk, nv, d, d)
            hb.deltanet_forward(q, k, v, g, beta, states[i % ncopies], o32, qs, True)
            hb.deltanet_gated_norm(o32, z, nw, 1e-6)

    settle(torch, step, window=20, min_launches=300, max_launches=2000)
    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(i)
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / args.steps * 1e3
    n_ev = 100
    e0 = [torch.cuda.Event(enable_timing=True) for _ in range(n_ev)]
    e1 = [torch.cuda.Event(enable_timing=True) for _ in range(n_ev)]
    for i in range(n_ev):
        e0[i].record()
        step(i)
        e1[i].record()
    torch.cuda.synchronize()
    kms = float(np.mean([a_.elapsed_time(b_) for a_, b_ in zip(e0, e1)]))
    nbytes = 2 * B * nv * d * d * 4 + B * (C * 2 + 2 * C * 3 * 2 + 2 * nv * 2 + 2 * nv * d * 2) + C * 4 * 2
    res = {
        "metric": "deltanet decode layer (conv + gates + step + gated norm) HBM GB/s + tokens/s, nk=16 nv=32 dk=dv=128",
        "value": nbytes / (ms * 1e-3) / 1e9, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32 state and arithmetic, bf16 activations", "data": "synthetic (seeded, generated on device)",
        "config": {"workload": "c5-decode-layer%s: gated-DeltaNet layer decode step B=%d nk=16 nv=32 dk=dv=128, %s"
                               % ("" if fused else "-3calls", B, "one launch" if fused else "prepare + step + gated norm (four launches)"),
                   "algorithmic_bytes_per_step": int(nbytes)},
        "tokens_per_s": B / (ms * 1e-3),
        "roofline": {"bound": "hbm", "kernel": "deltanet_decode_kernel<true>" if fused else "deltanet_conv8 + gates + deltanet_decode_kernel<false> + gated_rmsnorm_rows",
                     "achieved": nbytes / (kms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": nbytes / (kms * 1e-3) / 1e9 / HBM_PEAK_GBS, "traffic": None, "avg_kernel_us": kms * 1e3},
    }
    print(json.dumps(res))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=200)  # the first launches after set-up run a few % slower (clocks settle)
    ap.add_argument("--workload", default="c2", choices=sorted(WORKLOADS) + ["c3", "c3-prompt", "c3-fp8", "c3-d256", "c3-d64", "c3-b1", "c3-b1-shadow", "c3-prologue", "c3-shadow", "c3-fp8-shadow", "c5-decode", "c5-decode-layer", "c5-decode-layer-3calls", "c5-prefill", "c5-prefill-norm", "c5-prefill-layer", "c5-prefill-recurrent"])
    ap.add_argument("--copies", type=int, default=4, help="cache copies rotated through (defeats the last-level cache)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--block-tokens", type=int, default=256, help="tokens per pool block of the c2-paged workload")
    ap.add_argument("--cap-pad", type=int, default=0, help="decode workloads: cache capacity = context length + this many tokens")
    ap.add_argument("--prefill-columns", type=int, default=0, choices=[0, 16, 32, 128, 256],
                    help="prefill workloads: fix the (query, head) columns a workgroup owns (0 = the library's choice)")
    ap.add_argument("--key-splits", type=int, default=0,
                    help="prefill workloads: runs the keys of a query tile are cut into (0 = the library decides, 1 = never)")
    ap.add_argument("--prologue-fused-q", action="store_true",
                    help="c3-prologue: only k goes through the pre-pass, the chunk launches normalise and rotate q themselves")
    ap.add_argument("--prompt-copy", action="store_true",
                    help="c3 workloads: keep the bf16 copy of the prompt's K/V and read the history from it (what the -shadow workloads do)")
    ap.add_argument("--prologue-per-chunk", action="store_true",
                    help="c3-prologue: run the QK-norm + rotary pre-pass in front of every chunk call instead of once over the prompt")
    ap.add_argument("--chunk-tokens", type=int, default=0, choices=[0, 256, 512, 1024, 2048, 4096],
                    help="prefill workloads: tokens per chunk call (0 = the workload's own: 512, c3-prompt 4096)")
    ap.add_argument("--batch", type=int, default=0, help="c5 workloads: sequences in the batch (0 = the configuration's 64 for decode, 4 for prefill)")
    ap.add_argument("--graph", action="store_true", help="replay the decode steps from a captured HIP graph")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="run only a plain 1 GiB device-to-device copy, the reference point for scaling "
                         "rocprofv3's FETCH_SIZE / WRITE_SIZE counters")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU's share of the path; --gpus must be 1 (this build has no multi-GPU leg)",
              file=sys.stderr)
        sys.exit(2)

    import torch
    from hyprstream_amd import bindings as hb
    from hyprstream_amd import workloads as wl
    hb.PREFILL_COLUMNS = args.prefill_columns

    if not torch.cuda.is_available():
        print("no GPU visible: bench.py needs an MI355X", file=sys.stderr)
        sys.exit(1)
    hb.lib()  # fail loudly if the HIP library is not built
    dev = "cuda:0"
    if args.calibrate_copy:
        src = torch.randint(0, 255, (1 << 30,), dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(max(1, args.steps)):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"calibrate_copy_bytes": 1 << 30, "launches": max(1, args.steps)}))
        return
    if args.workload.startswith("c3"):
        return bench_prefill(args, torch, hb, wl, C=args.chunk_tokens or (4096 if args.workload == "c3-prompt" else 512),
                             fp8=args.workload.startswith("c3-fp8"), d256=args.workload == "c3-d256", d64=args.workload == "c3-d64", b1=args.workload.startswith("c3-b1"), prologue=args.workload == "c3-prologue", shadow=args.workload.endswith("-shadow") or args.prompt_copy)
    if args.workload.startswith("c5-decode-layer"):
        return bench_deltanet_layer(args, torch, hb, wl, fused=args.workload == "c5-decode-layer")
    if args.workload.startswith("c5"):
        return bench_deltanet(args, torch, hb, wl, "prefill" in args.workload, recurrent=args.workload.endswith("recurrent"),
                              norm="layer" if args.workload == "c5-prefill-layer" else args.workload == "c5-prefill-norm")
    B, Hq, Hkv, D, T, ragged, fp8, sigma, outliers = WORKLOADS[args.workload]
    gen = torch.Generator(device=dev)
    gen.manual_seed(wl.SEED)

    ncopies = max(1, args.copies)
    cap = T + args.cap_pad  # tokens the cache has room for (the reference allocates max_seq_len, not the current length)
    layout = hb.contiguous_layout(Hkv, cap, D)
    cdt = torch.uint8 if fp8 else torch.int8
    caches = []
    for c in range(ncopies):
        kc = torch.empty(B, Hkv, cap, D, dtype=cdt, device=dev)
        vc = torch.empty(B, Hkv, cap, D, dtype=cdt, device=dev)
        if fp8:
            ks = torch.empty(B, Hkv, dtype=torch.float32, device=dev)
            vs = torch.empty(B, Hkv, dtype=torch.float32, device=dev)
        else:
            ks = torch.empty(B, Hkv, layout.scale_stride_head, dtype=torch.float32, device=dev)
            vs = torch.empty(B, Hkv, layout.scale_stride_head, dtype=torch.float32, device=dev)
        caches.append((kc, vc, ks, vs))
    # fill copy 0 through the library's own quantize-on-write path (a prefill-sized write), sequence by sequence
    kc0, vc0, ks0, vs0 = caches[0]
    one = hb.contiguous_layout(Hkv, cap, D)
    tchunk = min(T, 8192)
    for b in range(B):
        for t0 in range(0, T, tchunk):
            ksrc = make_source(torch, gen, (1, tchunk, Hkv, D), sigma, outliers, dev)
            vsrc = make_source(torch, gen, (1, tchunk, Hkv, D), sigma, outliers, dev)
            if fp8:
                if t0 == 0:
                    hb.kv_fp8_calibrate(ksrc, vsrc, ks0[b:b + 1], vs0[b:b + 1])
                hb.kv_quantize_fp8(ksrc, vsrc, kc0[b:b + 1], vc0[b:b + 1], ks0[b:b + 1], vs0[b:b + 1], one, None, t0)
            else:
                hb.kv_quantize_int8(ksrc, vsrc, kc0[b:b + 1], vc0[b:b + 1], ks0[b:b + 1], vs0[b:b + 1], one, None, t0)
    for c in range(1, ncopies):
        for dst, src in zip(caches[c], caches[0]):
            dst.copy_(src)
    paged = args.workload == "c2-paged"
    if paged and args.cap_pad:
        sys.exit("--cap-pad is for the contiguous cache layouts")
    if paged:
        # every cache copy becomes a pool of 256-token blocks in a random order; K and V blocks of a sequence come from
        # one pool (ids 0..n-1 for K, n..2n-1 for V before the shuffle), as PagedLayerKVCache takes them
        BT = args.block_tokens
        nb = T // BT
        perm = torch.randperm(2 * B * nb, generator=torch.Generator().manual_seed(wl.SEED)).to(torch.int32)
        k_tab = perm[: B * nb].reshape(B, nb).contiguous().to(dev)
        v_tab = perm[B * nb:].reshape(B, nb).contiguous().to(dev)
        pools = []
        for kc, vc, ks, vs in caches:
            pc = torch.empty(2 * B * nb, Hkv, BT, D, dtype=cdt, device=dev)
            ps = torch.empty(2 * B * nb, Hkv, BT, dtype=torch.float32, device=dev)
            pc[k_tab.long().reshape(-1)] = kc.reshape(B, Hkv, nb, BT, D).permute(0, 2, 1, 3, 4).reshape(B * nb, Hkv, BT, D)
            pc[v_tab.long().reshape(-1)] = vc.reshape(B, Hkv, nb, BT, D).permute(0, 2, 1, 3, 4).reshape(B * nb, Hkv, BT, D)
            ps[k_tab.long().reshape(-1)] = ks[:, :, :T].reshape(B, Hkv, nb, BT).permute(0, 2, 1, 3).reshape(B * nb, Hkv, BT)
            ps[v_tab.long().reshape(-1)] = vs[:, :, :T].reshape(B, Hkv, nb, BT).permute(0, 2, 1, 3).reshape(B * nb, Hkv, BT)
            pools.append((pc, pc, ps, ps))
        flat_caches, caches = caches, pools
        layout = hb.paged_layout(Hkv, BT, D, k_tab, v_tab)
    if ragged:
        lens = torch.randint(512, T + 1, (B,), generator=gen, device=dev, dtype=torch.int32)
    else:
        lens = torch.full((B,), T, dtype=torch.int32, device=dev)
    pos = (lens - 1).contiguous()
    q = torch.randn(B, Hq, D, generator=gen, device=dev, dtype=torch.float32).to(torch.bfloat16)
    k_new = make_source(torch, gen, (B, 1, Hkv, D), sigma, outliers, dev)
    v_new = make_source(torch, gen, (B, 1, Hkv, D), sigma, outliers, dev)
    out = torch.empty(B, Hq, D, dtype=torch.bfloat16, device=dev)
    max_len = T
    if ragged:  # the host built the lengths, so it can tell the library how many tokens the batch holds
        layout.total_tokens_hint = int(lens.sum().item())
    ws = torch.empty(hb.decode_workspace_bytes(B, Hq, Hkv, D, max_len), dtype=torch.uint8, device=dev)
    scale = 1.0 / float(np.sqrt(D))
    quant = hb.kv_quantize_fp8 if fp8 else hb.kv_quantize_int8

    pro = None
    if args.workload in ("c2-prologue", "c4-prologue"):
        inv = 1.0 / (10000.0 ** (torch.arange(0, D, 2, device=dev, dtype=torch.float32) / D))
        ang = torch.arange(T, device=dev, dtype=torch.float32)[:, None] * inv[None, :]
        rope = (ang.sin().to(torch.bfloat16).contiguous(), ang.cos().to(torch.bfloat16).contiguous())
        qw = (1.0 + 0.1 * torch.randn(D, generator=gen, device=dev)).to(torch.bfloat16)
        kw = (1.0 + 0.1 * torch.randn(D, generator=gen, device=dev)).to(torch.bfloat16)
        pro = hb.qk_prologue(hb.QKNORM_LLAMA, 1e-6, qw, kw, rope[0], rope[1])

    def step(i):
        kc, vc, ks, vs = caches[i % ncopies]
        if pro is not None:
            hb.decode_step_prologue(q, k_new, v_new, pro, kc, vc, ks, vs, layout, lens, out, ws, Hkv, max_len, scale, fp8=fp8)
        else:
            hb.decode_step(q, k_new, v_new, kc, vc, ks, vs, layout, lens, out, ws, Hkv, max_len, scale, fp8=fp8)

    settled, settled_us = settle(torch, step)
    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    graph = None
    if args.graph:
        # one HIP graph holding `ncopies` consecutive steps (one per cache copy), replayed steps/ncopies times
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for i in range(ncopies):
                step(i)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for i in range(ncopies):
                step(i)
        graph.replay()
        torch.cuda.synchronize()
        args.steps = max(ncopies, args.steps // ncopies * ncopies)
    t0 = time.perf_counter()
    if graph is not None:
        for i in range(args.steps // ncopies):
            graph.replay()
    else:
        for i in range(args.steps):
            step(i)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt / args.steps * 1e3

    lens_h = lens.cpu().numpy()
    step_bytes = (wl.decode_bytes_fp8 if fp8 else wl.decode_bytes_int8)(lens_h, Hq, Hkv, D)
    gbs = step_bytes / (ms_per_step * 1e-3) / 1e9

    # ---- roofline of the dominant kernel alone: HIP events (torch's, recorded on the stream the library
    # launches on) around each launch.  When every sequence is one chunk the whole step IS that one launch
    # (new-token write + attention + output); otherwise the split-K kernel is timed without the merge.
    nchunks = hb.decode_num_chunks(B, Hkv, max_len, layout.total_tokens_hint)
    single = nchunks == 1
    write_bytes = B * Hkv * D * (2 * 2 + 2 * 1) + (0 if fp8 else B * Hkv * 2 * 4)
    kern_bytes = step_bytes if single else step_bytes - write_bytes
    n_ev = 200  # independent of --steps: a short timed region must not shorten the kernel statistics
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n_ev)]
    for i in range(n_ev):
        kc, vc, ks, vs = caches[i % ncopies]
        if single:
            evs[i][0].record()
            hb.decode_step(q, k_new, v_new, kc, vc, ks, vs, layout, lens, out, ws, Hkv, max_len, scale, fp8=fp8)
            evs[i][1].record()
        else:
            quant(k_new, v_new, kc, vc, ks, vs, layout, pos, 0)
            evs[i][0].record()
            hb.decode_attn(q, kc, vc, ks, vs, layout, lens, out, ws, Hkv, max_len, scale, fp8=fp8, phases=1)
            evs[i][1].record()
            hb.decode_attn(q, kc, vc, ks, vs, layout, lens, out, ws, Hkv, max_len, scale, fp8=fp8, phases=2)
    torch.cuda.synchronize()
    kt = np.array([a.elapsed_time(b) for a, b in evs])  # ms
    k_avg_ms = float(kt.mean())
    achieved = kern_bytes / (k_avg_ms * 1e-3) / 1e9

    # HBM bytes per launch are a recorded counter figure (two rocprofv3 --pmc runs, FETCH_SIZE and WRITE_SIZE, scaled
    # by a plain copy of known size), not something this run measures: the source file is named beside the number.
    traffic, traffic_source = None, None
    tpath = os.path.join(ROOT, "profiles", "decode_attn_traffic.json")
    if os.path.exists(tpath):
        try:
            traffic = json.load(open(tpath)).get(args.workload)
            if traffic is not None:
                traffic_source = "recorded rocprofv3 counters: profiles/decode_attn_traffic.json (not measured in this run)"
        except Exception:
            traffic = None

    result = {
        "metric": "decode-attn HBM GB/s (% peak) + tokens/s, B=64 ctx 8K int8 KV, Llama-3-8B shape",
        "value": gbs, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp8_e4m3 codes, f16 MFMA, f32 accumulate" if fp8 else "int8 codes, f16 MFMA, f32 accumulate",
        "data": "synthetic (seeded, generated on device)",
        "config": {"workload": "%s: B=%d Hq=%d Hkv=%d D=%d T=%s %s KV, 1 new token/seq quantized on write, one layer"
                               % (args.workload, B, Hq, Hkv, D, "U[512,%d]" % T if ragged else str(T),
                                  "fp8-e4m3 per-head-scale" if fp8 else "int8 per-token-per-head-scale"),
                   "cache_copies_rotated": ncopies, "algorithmic_bytes_per_step": int(step_bytes)},
        "pct_of_hbm_peak": 100.0 * gbs / HBM_PEAK_GBS,
        "tokens_per_s": B / (ms_per_step * 1e-3),
        "roofline": {"bound": "hbm", "kernel": "decode_attn_kernel", "achieved": achieved, "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS, "traffic": traffic,
                     "traffic_source": traffic_source, "settle_launches": settled, "settled_us_per_launch": settled_us,
                     "avg_kernel_us": k_avg_ms * 1e3, "min_kernel_us": float(kt.min()) * 1e3,
                     "algorithmic_bytes_per_launch": int(kern_bytes), "launches_timed": n_ev},
    }
    if not args.no_cpu_baseline:
        cb, _ = cpu_baseline(torch, args.workload, (flat_caches if paged else caches)[0], q, lens, Hq, fp8)
        if args.workload == "c2":
            # the reference's own CPU-runnable configuration (one sequence, 2048 tokens, int8), whole, same op sequence
            T1 = 2048
            one = tuple(t[:1, :, :T1].contiguous() for t in (flat_caches if paged else caches)[0])
            c1, _ = cpu_baseline(torch, "c1", one, q[:1], torch.full((1,), T1, dtype=torch.int32), Hq, False, seconds_budget=3.0)
            cb["single_sequence_2048"] = {k: c1[k] for k in ("value", "unit", "ms_per_call", "tokens_per_s")}
        result["cpu_baseline"] = cb
    print(json.dumps(result))


if __name__ == "__main__":
    main()
