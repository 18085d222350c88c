#!/usr/bin/env python3
"""Benchmark of the MI355X hot path on ONE GPU.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A "step" is one pass of the headline workload over one synthetic batch: bf16 causal self-attention forward
AND backward at B=4, H=16, S=4096, D=128 (the second benchmark configuration), inputs resident in HBM before
the timed region.  `value` is the attention TFLOP/s over that step with the FlashAttention flop convention
(forward 4*B*H*S^2*D/2, backward 2.5x forward).  The same JSON line also carries, under "extra", the other
figures the metric names: fused AdamW GB/s on the LLaMA-50M flat buffers and LLaMA-50M train-step tokens/s.

"roofline" describes the dominant kernel of the step (the one with the largest summed kernel time, measured
live with HIP events on the launch stream through the library's timing hooks); "cpu_baseline" times the CPU
oracle on a bounded sample of the same workload on the host cores.  Prints exactly one JSON line on stdout.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16 matrix peak
HBM_PEAK_GBPS = 8000.0          # MI355X HBM3E peak
PROFILES = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles")


def measured_hbm_traffic():
    """HBM bytes per launch of each attention kernel on the headline workload: profiles/attn_cfg2_hbm_traffic.json, the
    figures of profiles/attn_cfg2_hbm_traffic.md (two rocprofv3 --pmc runs of this script, FETCH_SIZE, then WRITE_SIZE,
    each scaled by the same counter over the --calibrate-traffic kernel).  Counters cannot be read from inside the timed
    run; a missing file gives null figures."""
    try:
        with open(os.path.join(PROFILES, "attn_cfg2_hbm_traffic.json")) as f:
            return {k: v["hbm_bytes_per_launch"] for k, v in json.load(f)["kernels"].items()}
    except (OSError, KeyError, ValueError):
        return {}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--skip-extra", action="store_true", help="only the headline attention workload")
    ap.add_argument("--skip-cpu", action="store_true", help="omit the CPU baseline legs")
    ap.add_argument("--only", default=None, help="run only this leg of `extra` (for profiling one part of the run)")
    ap.add_argument("--calibrate-traffic", action="store_true",
                    help="only launch the streaming kernel of known size (mlts_scale over 1 GiB of fp32: 1 GiB read, "
                         "1 GiB written per launch) that the FETCH_SIZE / WRITE_SIZE counters are scaled against")
    return ap.parse_args()


def attention_inputs(torch, dev, B, H, S, D, seed=1234):
    gen = torch.Generator().manual_seed(seed)
    return [torch.randn(B, H, S, D, generator=gen).bfloat16().to(dev) for _ in range(4)]


PREHEAT_S = 0.25
LLAMA_PREHEAT_STEPS = 25  # untimed training steps in front of the warm-up steps of the LLaMA legs


def preheat(torch, fn, seconds=PREHEAT_S):
    """Untimed calls of the step for `seconds` of wall time, in front of the W warm-up steps: an idle GPU raises its
    clocks over the first ~50 ms of load, which is longer than five warm-up steps of a 1.3 ms step (the first twenty
    steps after five warm-up steps run 5 % slower than the twenty after them)."""
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(4):
            fn()
        torch.cuda.synchronize()


def timed(torch, fn, steps, warmup, preheat_steps=None):
    """Mean seconds per call.  The interpreter's cyclic garbage collector is held off during the timed calls (as
    timeit does): one full collection is a 50-100 ms pause, which in a launch-bound loop of ten steps is the result.
    preheat_steps: a fixed number of untimed calls in place of the wall-time pre-heat, for steps that change state
    (training steps: legs that are compared afterwards must have taken the same number of optimizer steps)."""
    import gc
    gc.collect()  # before the pre-heat: a collection behind it would leave the GPU idle long enough to drop its clocks
    gc.disable()
    try:
        if preheat_steps is None:
            preheat(torch, fn)
        else:
            for _ in range(preheat_steps):
                fn()
            torch.cuda.synchronize()
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps
    finally:
        gc.enable()


def bench_attention(torch, ops, _lib, dev, steps, warmup, shape=(4, 16, 4096, 128)):
    B, H, S, D = shape
    q, k, v, do = attention_inputs(torch, dev, B, H, S, D)
    fwd_flops = 4.0 * B * H * S * S * D / 2.0
    flops = {"fwd": fwd_flops, "bwd": 2.5 * fwd_flops}
    state = {}

    def step():
        o, lse = ops.attention_forward(q, k, v, mask_mode=ops.MASK_CAUSAL)
        state["grads"] = ops.attention_backward(do, q, k, v, o, lse, mask_mode=ops.MASK_CAUSAL)

    preheat(torch, step)
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    _lib.kernel_timing(True)
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    sec = (time.perf_counter() - t0) / steps
    kernels = {}
    for name in ("attn_fwd", "attn_bwd_dkdv", "attn_bwd_dq"):
        total_ms, launches = _lib.kernel_time_ms(name)
        if launches:
            kernels[name] = {"ms": total_ms / launches, "launches_per_step": launches / steps}
    delta_time = _lib.kernel_time_ms("attn_delta")
    _lib.kernel_timing(False)
    # algorithmic flops per launch of each kernel (FlashAttention convention: 2 GEMMs forward, 5 backward: S, dP, dV,
    # dK, dQ, each fwd_flops / 2)
    # both backward kernels recompute S and dP; the five conventional products are credited 3 : 2 (dV, dK, + S | dQ, + dP)
    kernel_flops = {"attn_fwd": fwd_flops, "attn_bwd_dkdv": 2.5 * fwd_flops * 0.6, "attn_bwd_dq": 2.5 * fwd_flops * 0.4}
    for name, rec in kernels.items():
        rec["tflops"] = kernel_flops[name] / (rec["ms"] * 1e-3) / 1e12
    # the row-wise delta = sum(dO * O) pass in front of the backward kernels: memory bound, reads dO and O once
    total_ms, launches = delta_time
    if launches:
        nbytes = 2 * 2 * B * H * S * D + 4 * B * H * S
        kernels["attn_delta"] = {"ms": total_ms / launches, "launches_per_step": launches / steps,
                                 "gbps": nbytes / (total_ms / launches * 1e-3) / 1e9}
    return sec, flops, kernels, kernel_flops


def bench_attention_d64(torch, ops, _lib, dev, steps, warmup):
    """The attention of the LLaMA-50M step alone: B=8, H=8, S=2048, head_dim 64, causal, bf16."""
    sec, flops, kernels, _ = bench_attention(torch, ops, _lib, dev, steps, warmup, shape=(8, 8, 2048, 64))
    value = (flops["fwd"] + flops["bwd"]) / sec / 1e12
    return {"workload": "causal self-attention fwd+bwd, B=8 H=8 S=2048 D=64, bf16", "value": value, "unit": "TFLOP/s",
            "frac_of_mfma_peak": value / MFMA_BF16_PEAK_TFLOPS, "ms_per_step": sec * 1e3, "kernels": kernels}


def packed_rows(torch, B, S, gen):
    """Documents of uniform length in [64, 2048] until the row is full, the last one cut (configuration 3); returns
    positions, sequence ids and sum over documents of L^2 / 2."""
    pos = torch.zeros(B, S, dtype=torch.long)
    seq = torch.zeros(B, S, dtype=torch.long)
    work = 0
    for b in range(B):
        i = d = 0
        while i < S:
            L = min(int(torch.randint(64, 2049, (1,), generator=gen)), S - i)
            pos[b, i:i + L] = torch.arange(L)
            seq[b, i:i + L] = d
            work += L * L / 2.0
            i, d = i + L, d + 1
    return pos, seq, work


def bench_cfg3_packed_gqa(torch, ops, _lib, dev, steps, warmup):
    """Configuration 3: packed documents, grouped-query attention (32 query heads on 8 KV heads), forward + backward;
    TFLOP/s on the score elements the drawn documents actually have (sum of L^2 / 2 per head)."""
    B, S, Hq, Hkv, D = 2, 8192, 32, 8, 128
    gen = torch.Generator().manual_seed(1234)
    pos, seq, work = packed_rows(torch, B, S, gen)
    q = torch.randn(B, Hq, S, D, generator=gen).bfloat16().to(dev)
    k = torch.randn(B, Hkv, S, D, generator=gen).bfloat16().to(dev)
    v = torch.randn(B, Hkv, S, D, generator=gen).bfloat16().to(dev)
    do = torch.randn(B, Hq, S, D, generator=gen).bfloat16().to(dev)
    # int32 ids, as the C-ABI takes them: converted once per batch (every layer's attention shares them), not per call
    ids = dict(q_pos=pos.int().to(dev), k_pos=pos.int().to(dev), q_seq=seq.int().to(dev), k_seq=seq.int().to(dev))

    def step():
        # the mask plan (tile statistics, visibility bits, block orders) is built once per step, in the forward, and
        # serves the backward: what one attention layer pays.  Left alone, the plan would be kept from step to step
        # (and, in a model, from layer to layer) for as long as the id tensors do not change.
        ops.clear_doc_plan_cache()
        o, lse = ops.attention_forward(q, k, v, mask_mode=ops.MASK_DOC, **ids)
        ops.attention_backward(do, q, k, v, o, lse, mask_mode=ops.MASK_DOC, **ids)

    sec = timed(torch, step, steps, warmup)

    def step_plan_kept():  # what every layer but the first pays: the plan of the unchanged ids is found in ops' cache
        o, lse = ops.attention_forward(q, k, v, mask_mode=ops.MASK_DOC, **ids)
        ops.attention_backward(do, q, k, v, o, lse, mask_mode=ops.MASK_DOC, **ids)

    sec_kept = timed(torch, step_plan_kept, steps, warmup)
    flops = 3.5 * 4.0 * Hq * D * work
    return {"workload": "packed documents (lengths uniform in [64, 2048]) causal attention fwd+bwd, B=2 S=8192 Hq=32 Hkv=8 D=128, bf16; "
                        "one document-mask plan built per step",
            "score_elements_per_head": work, "flops_per_step": flops, "ms_per_step": sec * 1e3,
            "ms_per_step_plan_kept": sec_kept * 1e3,
            "value": flops / sec / 1e12, "unit": "TFLOP/s", "frac_of_mfma_peak": flops / sec / 1e12 / MFMA_BF16_PEAK_TFLOPS}


def bench_cfg4_ring_rank(torch, dev, steps, warmup, rank=1):
    """Configuration 4: one rank's share of zigzag ring attention at CP=4 over 32768 tokens (local Q of 8192 tokens against
    the four KV chunks, all resident; block kernels + fp32 LSE merges forward, then the backward with the global O / LSE).
    4 balanced blocks = 134,217,728 score elements per head: 3.848 TFLOP per rank."""
    from maltos_amd.ring_attention import zigzag_ring_attention
    from maltos_amd.ring_layout import expected_zigzag_ring_positions

    W, H, S_loc, D = 4, 16, 8192, 128
    gen = torch.Generator().manual_seed(1234)
    gq, gk, gv, gdo = (torch.randn(1, H, W * S_loc, D, generator=gen).bfloat16().to(dev) for _ in range(4))
    pos = [expected_zigzag_ring_positions(S_loc, rank=r, world_size=W, device=dev) for r in range(W)]
    q = gq.index_select(2, pos[rank]).requires_grad_(True)
    do = gdo.index_select(2, pos[rank])
    chunks = [(gk.index_select(2, p_).requires_grad_(True), gv.index_select(2, p_).requires_grad_(True)) for p_ in pos]
    del gq, gk, gv, gdo

    def step():
        out = zigzag_ring_attention(q, chunks, rank=rank, world_size=W)
        out.backward(do)
        q.grad = None
        for kc, vc in chunks:
            kc.grad = vc.grad = None

    sec = timed(torch, step, steps, warmup)
    flops = 3.5 * 4.0 * H * D * (W * S_loc * S_loc / 2.0)
    return {"workload": f"zigzag ring attention fwd+bwd, rank {rank} of CP=4 over 32768 tokens, local Q 8192, H=16 D=128, bf16, merges included",
            "flops_per_step": flops, "ms_per_step": sec * 1e3, "value": flops / sec / 1e12, "unit": "TFLOP/s",
            "frac_of_mfma_peak": flops / sec / 1e12 / MFMA_BF16_PEAK_TFLOPS}


def parity_cfg2(torch, ops, dev):
    """Largest absolute and relative-to-largest-value differences of O, LSE, dQ, dK, dV on the headline inputs (first
    batch element, all heads) against the library routine the configuration names: PyTorch SDPA, math backend, fp32,
    differentiated by autograd."""
    import torch.nn.functional as F
    from torch.nn.attention import SDPBackend, sdpa_kernel

    B, H, S, D = 4, 16, 4096, 128
    q, k, v, do = (t[:1] for t in attention_inputs(torch, dev, B, H, S, D))
    qg, kg, vg = (t.clone().requires_grad_(True) for t in (q, k, v))
    o, lse = ops.attention(qg, kg, vg, mask_mode=ops.MASK_CAUSAL, return_lse=True)
    o.backward(do)
    qf, kf, vf = (t.float().requires_grad_(True) for t in (q, k, v))
    with sdpa_kernel(SDPBackend.MATH):
        want = F.scaled_dot_product_attention(qf, kf, vf, is_causal=True)
    want.backward(do.float())
    out = {}
    for name, got, ref in (("O", o, want), ("dQ", qg.grad, qf.grad), ("dK", kg.grad, kf.grad), ("dV", vg.grad, vf.grad)):
        err = (got.float() - ref.detach()).abs().max().item()
        out[name] = {"max_abs": err, "rel": err / ref.detach().abs().max().item()}
    scores = (qf.detach() @ kf.detach().transpose(-1, -2)) * D ** -0.5
    scores.masked_fill_(~torch.ones(S, S, dtype=torch.bool, device=dev).tril(), float("-inf"))
    want_lse = torch.logsumexp(scores, dim=-1)
    err = (lse - want_lse).abs().max().item()
    out["LSE"] = {"max_abs": err, "rel": err / want_lse.abs().max().item()}
    out["reference"] = "torch SDPA math backend in fp32 on the bf16-rounded inputs, batch element 0 of configuration 2"
    out["bound"] = "2e-2 max-abs (O, dQ, dK, dV), 1e-4 (LSE)"
    return out


def _parity_update(out, name, got, ref):
    err = (got.float() - ref.float()).abs().max().item()
    rec = out.setdefault(name, {"max_abs": 0.0, "largest_value": 0.0})
    rec["max_abs"] = max(rec["max_abs"], err)
    rec["largest_value"] = max(rec["largest_value"], ref.float().abs().max().item())


def _parity_finish(out, reference, bound):
    for rec in out.values():
        rec["rel"] = rec["max_abs"] / rec.pop("largest_value")
    out["reference"] = reference
    out["bound"] = bound
    return out


def parity_cfg3(torch, ops, dev):
    """Largest differences of O, LSE, dQ, dK, dV of configuration 3 (first batch row, every document, all heads) against
    the oracle: causal attention of each document alone in fp32, differentiated by autograd, on the GPU tensors."""
    from oracle import attention as oa

    B, S, Hq, Hkv, D = 1, 8192, 32, 8, 128
    gen = torch.Generator().manual_seed(1234)
    pos, seq, _ = packed_rows(torch, B, S, gen)
    q = torch.randn(B, Hq, S, D, generator=gen).bfloat16().to(dev)
    k = torch.randn(B, Hkv, S, D, generator=gen).bfloat16().to(dev)
    v = torch.randn(B, Hkv, S, D, generator=gen).bfloat16().to(dev)
    do = torch.randn(B, Hq, S, D, generator=gen).bfloat16().to(dev)
    qg, kg, vg = (t.clone().requires_grad_(True) for t in (q, k, v))
    ids = dict(q_pos=pos.to(dev), k_pos=pos.to(dev), q_seq=seq.to(dev), k_seq=seq.to(dev))
    o, lse = ops.attention(qg, kg, vg, mask_mode=ops.MASK_DOC, return_lse=True, **ids)
    o.backward(do)
    out = {}
    starts = (seq[0, 1:] != seq[0, :-1]).nonzero().flatten().add(1).tolist()
    for a, b in zip([0] + starts, starts + [S]):
        sl = slice(a, b)
        qf, kf, vf = (t[:, :, sl].float().requires_grad_(True) for t in (q, k, v))
        want_o, want_lse = oa.attention_with_lse(qf, kf, vf, oa.causal_mask(b - a, b - a, dev))
        want_o.backward(do[:, :, sl].float())
        for name, got, ref in (("O", o[:, :, sl], want_o), ("LSE", lse[:, :, sl], want_lse), ("dQ", qg.grad[:, :, sl], qf.grad),
                               ("dK", kg.grad[:, :, sl], kf.grad), ("dV", vg.grad[:, :, sl], vf.grad)):
            _parity_update(out, name, got, ref.detach())
    return _parity_finish(out, "oracle.attention (fp32) per document on the bf16-rounded inputs, batch row 0 of configuration 3's shapes, "
                               f"{len(starts) + 1} documents",
                          "2e-2 + 2^-8 |value| (O, dQ, dK, dV; dK and dV are sums over four query heads, their half ulp exceeds 2e-2 "
                          "where |value| > 5), 1e-4 (LSE)")


def parity_cfg4(torch, dev, rank=1, heads=(0, 15)):
    """Largest differences of O, LSE, dQ and the four chunks' dK, dV of configuration 4 (one rank's ring share) against
    the oracle: ONE pass of causal attention over all 32768 tokens in fp32 with dO zero outside the rank, on `heads`."""
    from maltos_amd.ring_attention import zigzag_ring_attention
    from maltos_amd.ring_layout import expected_zigzag_ring_positions
    from oracle import attention as oa

    W, H, S_loc, D = 4, 16, 8192, 128
    total = W * S_loc
    gen = torch.Generator().manual_seed(1234)
    gq, gk, gv, gdo = (torch.randn(1, H, total, D, generator=gen).bfloat16().to(dev) for _ in range(4))
    pos = [expected_zigzag_ring_positions(S_loc, rank=r, world_size=W, device=dev) for r in range(W)]
    q = gq.index_select(2, pos[rank]).requires_grad_(True)
    chunks = [(gk.index_select(2, p_).requires_grad_(True), gv.index_select(2, p_).requires_grad_(True)) for p_ in pos]
    o, lse = zigzag_ring_attention(q, chunks, rank=rank, world_size=W, return_lse=True)
    o.backward(gdo.index_select(2, pos[rank]))
    do_masked = torch.zeros_like(gdo)
    do_masked[:, :, pos[rank]] = gdo[:, :, pos[rank]]
    mask = oa.causal_mask(total, total, dev)
    out = {}
    for h in heads:
        qf, kf, vf = (t[:, h:h + 1].float().requires_grad_(True) for t in (gq, gk, gv))
        want_o, want_lse = oa.attention_with_lse(qf, kf, vf, mask)
        want_o.backward(do_masked[:, h:h + 1].float())
        _parity_update(out, "O", o[:, h:h + 1], want_o.detach()[:, :, pos[rank]])
        _parity_update(out, "LSE", lse[:, h:h + 1], want_lse.detach()[:, :, pos[rank]])
        _parity_update(out, "dQ", q.grad[:, h:h + 1], qf.grad[:, :, pos[rank]])
        for src, (kc, vc) in enumerate(chunks):
            _parity_update(out, "dK", kc.grad[:, h:h + 1], kf.grad[:, :, pos[src]])
            _parity_update(out, "dV", vc.grad[:, h:h + 1], vf.grad[:, :, pos[src]])
        del qf, kf, vf, want_o, want_lse
    return _parity_finish(out, f"oracle.attention (fp32): one causal pass over all 32768 tokens, rank {rank}, heads {list(heads)}",
                          "2e-2 max-abs (O, dQ, dK, dV), 1e-4 (LSE)")


def bench_adamw(torch, ops, _lib, dev, steps, warmup):
    n = 58_073_600  # LLaMA-50M parameters
    p = torch.randn(n, device=dev)
    g = torch.randn(n, device=dev) * 0.01
    m = torch.zeros(n, device=dev)
    v = torch.zeros(n, device=dev)
    lowp = torch.empty(n, dtype=torch.bfloat16, device=dev)
    hp = dict(lr=3e-4, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.1)
    state = {"t": 0}

    def step():
        state["t"] += 1
        ops.adamw_step_(p, g, m, v, step=state["t"], p_lowp=lowp, **hp)

    preheat(torch, step, 0.1)
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    _lib.kernel_timing(True)
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    total_ms, launches = _lib.kernel_time_ms("adamw")
    _lib.kernel_timing(False)
    ms = total_ms / max(1, launches)
    bytes_per_launch = 30.0 * n  # read p,g,m,v (16 B) + write p,m,v (12 B) + bf16 model copy (2 B)
    return {"params": n, "bytes_per_param": 30, "kernel_ms": ms, "gbps": bytes_per_launch / (ms * 1e-3) / 1e9,
            "frac_of_hbm_peak": bytes_per_launch / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS}


def bench_hbm_kernels(torch, ops, _lib, dev, reps=20):
    """The memory-bound kernels of the step, each alone at its LLaMA-50M shape (merge: at the ring configuration's), timed
    with the library's HIP events: microseconds per call, algorithmic bytes (every operand read once, every result
    written once), GB/s and the fraction of the HBM peak."""
    N, h, I, V = 8 * 2048, 512, 1376, 32000
    bf = torch.bfloat16
    g = torch.Generator().manual_seed(1234)
    rnd = lambda *shape: torch.randn(*shape, generator=g).to(bf).to(dev)
    x, res, dy, dres = rnd(N, h), rnd(N, h), rnd(N, h), rnd(N, h)
    w = torch.ones(h, dtype=bf, device=dev)
    _, rstd = torch.ops.maltos.rmsnorm_fwd(x, w, 1e-5)
    gate, up, dh = rnd(N, I), rnd(N, I), rnd(N, I)
    q = rnd(8, 2048, 8, 64).transpose(1, 2)                      # the projection output's [B, H, S, D] view
    ang = torch.arange(2048, dtype=torch.float32)[:, None] * (10000.0 ** (-torch.arange(0, 64, 2, dtype=torch.float32) / 64))[None, :]
    cos, sin = torch.cos(ang).to(bf).to(dev), torch.sin(ang).to(bf).to(dev)
    logits = rnd(N, V)
    logits_own = rnd(N, V)                                          # overwritten by its own gradient, call after call
    q2 = rnd(8, 2048, 8, 64).transpose(1, 2)
    labels = torch.randint(0, V, (N,), generator=g).to(dev)
    n_par = 58_073_600
    gsrc = torch.randn(n_par, device=dev).to(bf)
    gdst = torch.empty(n_par, device=dev)
    sq = torch.empty((), dtype=torch.float64, device=dev)
    B4, H4, S4, D4 = 1, 16, 8192, 128
    out_acc = torch.zeros(B4, H4, S4, D4, device=dev)
    lse_acc = torch.zeros(B4, H4, S4, device=dev)
    o_blk = torch.randn(B4, H4, S4, D4, device=dev).to(bf)
    lse_blk = torch.randn(B4, H4, S4, device=dev)
    e = 2
    cases = [
        ("rmsnorm_fwd", "rmsnorm_fwd", 2 * N * h * e, lambda: torch.ops.maltos.rmsnorm_fwd(x, w, 1e-5)),
        ("rmsnorm_bwd", "rmsnorm_bwd", 3 * N * h * e, lambda: torch.ops.maltos.rmsnorm_bwd(dy, x, w, rstd)),
        ("add_rmsnorm_fwd", "rmsnorm_fwd", 4 * N * h * e, lambda: torch.ops.maltos.add_rmsnorm_fwd(x, res, w, 1e-5)),
        ("add_rmsnorm_bwd", "rmsnorm_bwd", 4 * N * h * e, lambda: torch.ops.maltos.add_rmsnorm_bwd(dy, dres, x, w, rstd)),
        ("rope", "rope", 2 * e * q.numel(), lambda: ops.rope(q, cos, sin)),
        ("swiglu_fwd", "swiglu_fwd", 3 * N * I * e, lambda: torch.ops.maltos.swiglu_fwd(gate, up)),
        ("swiglu_bwd", "swiglu_bwd", 5 * N * I * e, lambda: torch.ops.maltos.swiglu_bwd(dh, gate, up)),
        ("cross_entropy_fwd_bwd", "ce", 2 * N * V * e, lambda: torch.ops.maltos.ce_fwd_bwd(logits, labels, -100)),
        # the form the model uses for the logits it owns: the gradient takes their place (one buffer instead of two)
        ("cross_entropy_fwd_bwd_over_logits", "ce", 2 * N * V * e, lambda: ops._ce_fwd_bwd(logits_own, labels, -100, overwrite=True)),
        ("rope_pair_q_and_k", "rope", 2 * 2 * e * q.numel(), lambda: ops.rope_pair(q, q2, cos, sin)),
        ("grad_to_f32_with_norm", "grad_to_f32", 6 * n_par, lambda: ops.grad_to_f32_(gdst, gsrc, sq_out=sq)),
        ("attn_merge", "attn_merge", 10 * B4 * H4 * S4 * D4 + 12 * B4 * H4 * S4,
         lambda: ops.attention_merge_(out_acc, lse_acc, o_blk, lse_blk)),
    ]

    out = {}
    with torch.no_grad():
        for label, timer, nbytes, fn in cases:
            preheat(torch, fn, 0.05)
            for _ in range(3):
                fn()
            torch.cuda.synchronize()
            _lib.kernel_timing(True)
            for _ in range(reps):
                fn()
            torch.cuda.synchronize()
            total_ms, launches = _lib.kernel_time_ms(timer)
            _lib.kernel_timing(False)
            us = total_ms / max(1, launches) * 1e3
            gbps = nbytes / (us * 1e-6) / 1e9
            out[label] = {"us": us, "algorithmic_bytes": nbytes, "gbps": gbps, "frac_of_hbm_peak": gbps / HBM_PEAK_GBPS}
        # yardstick: what a plain device-to-device copy (torch's copy kernel) reaches when it moves as many bytes as the
        # small kernels above, timed the same way (an event pair around every launch): launches this short are bounded by
        # how fast a grid starts and drains, whatever they compute
        for label, n_elem in (("plain_copy_moving_33.6MB", N * h), ("plain_copy_moving_67.1MB", 2 * N * h)):
            src = torch.randn(n_elem, generator=g).to(bf).to(dev)
            dst = torch.empty_like(src)
            fn = lambda: dst.copy_(src)
            preheat(torch, fn, 0.05)
            pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(reps)]
            torch.cuda.synchronize()
            for a, b in pairs:
                a.record()
                fn()
                b.record()
            torch.cuda.synchronize()
            us = sum(a.elapsed_time(b) for a, b in pairs) / reps * 1e3
            nbytes = 2 * n_elem * e
            out[label] = {"us": us, "algorithmic_bytes": nbytes, "gbps": nbytes / (us * 1e-6) / 1e9,
                          "frac_of_hbm_peak": nbytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBPS}
    return out


def bench_llama50m(torch, dev, steps, warmup, zero1=False, graph=False, no_tuned_gemms=False, zero2=False):
    """graph=True: forward + backward replayed from one HIP graph (clip, AdamW and the gradient clear stay eager).
    zero1=True: the same step with the parameters in the ZeRO-1 flat buffers (world size 1): one optimizer launch
    per 25 MiB bucket on the bucket's local shard, the clip applied on the device as in the flat legs, gather back into
    the flat data buffer.
    zero2=True: ZeRO-2's per-bucket gradient buffers instead of one: every bucket's shard is taken when its last
    gradient has arrived, inside the backward pass."""
    zero1 = zero1 or zero2
    from maltos_amd.gemm_tuning import tuned_gemms_off, use_tuned_gemms
    from maltos_amd.grad_clip import clip_grad_norm_fused_
    from maltos_amd.llama import LlamaConfig, LlamaForCausalLM, set_grad_accumulation_into_buffers
    from maltos_amd.optim import FusedAdamW, MasterWeightsOptimizer

    # the linear layers' products run on the vendor GEMM libraries; which of their kernels serves which shape comes from
    # the selection the package ships for gfx950 (0: the file was recorded with other library versions and is not used)
    gemm_shapes = 0 if no_tuned_gemms else use_tuned_gemms()
    cfg = LlamaConfig(vocab_size=32000, hidden_size=512, intermediate_size=1376, num_hidden_layers=8,
                      num_attention_heads=8, max_position_embeddings=2048, rms_norm_eps=1e-5)
    torch.manual_seed(1234)
    model = LlamaForCausalLM(cfg)
    with torch.no_grad():
        for p in model.parameters():
            if p.dim() >= 2:
                p.normal_(0.0, 0.02)
    model = model.to(dev).to(torch.bfloat16)
    set_grad_accumulation_into_buffers(model)  # gradients live in flat buffers that are cleared in place: dW adds into them
    factory = lambda params: MasterWeightsOptimizer(params, optimizer_factory=lambda ps: FusedAdamW(
        ps, lr=3e-4, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1))
    if zero1:
        from maltos_amd.zero1 import Zero1FlatBuffers
        from maltos_amd.zero2 import Zero2FlatBuffers
        z = (Zero2FlatBuffers if zero2 else Zero1FlatBuffers)(model, optimizer_factory=factory, bucket_mb_size=25)
    else:
        opt = factory(model.parameters())
    gen = torch.Generator().manual_seed(1234)
    ids = torch.randint(0, cfg.vocab_size, (8, 2049), generator=gen).to(dev)
    batch = {"input_ids": ids[:, :-1].contiguous(), "labels": ids[:, 1:].contiguous()}
    out = {}

    def step():
        loss = model(batch)
        loss.backward()
        out["sq"] = clip_grad_norm_fused_(opt, 1.0)  # flat fp32 grads, global-norm clip at 1.0, no host sync
        opt.step()
        opt.zero_grad(set_to_none=True)
        out["loss"] = loss

    if graph:
        from maltos_amd.graph_step import CapturedForwardBackward
        captured = CapturedForwardBackward(model, batch, embed=model.embed_tokens, clear_grads=lambda: opt.zero_grad(set_to_none=True))

    def step_graph():
        out["loss"] = captured(batch)
        out["sq"] = clip_grad_norm_fused_(opt, 1.0)
        opt.step()
        opt.zero_grad(set_to_none=True)

    def step_zero1():
        z.reset_grads()
        loss = model(batch)
        loss.backward()
        out["norm"] = z.step(1.0, clip_on_device=True)   # the sum of squares, left on the device as in the flat legs
        out["loss"] = loss

    # a fixed number of untimed steps (~0.3 s) in front: the three legs then report loss and gradient norm of the same
    # optimizer step, and they agree when the layouts compute the same thing
    sec = timed(torch, step_zero1 if zero1 else step_graph if graph else step, steps, warmup, preheat_steps=LLAMA_PREHEAT_STEPS)
    tuned_gemms_off()
    tokens = 8 * 2048
    res = {"ms_per_step": sec * 1e3, "tokens_per_sec": tokens / sec, "loss_last": float(out["loss"].detach()),
           "grad_norm_last": float(out["norm"].sqrt()) if zero1 else float(out["sq"].sqrt()),
           "optimizer_steps_taken": LLAMA_PREHEAT_STEPS + warmup + steps,
           "params": sum(p.numel() for p in model.parameters()),
           "tflops_reference_estimator": tokens * model.flops_per_token() / sec / 1e12,
           "gemm_kernels": (f"per-shape selection of maltos_amd/tuned/gemm_gfx950.csv ({gemm_shapes} shapes)" if gemm_shapes
                            else "the GEMM libraries' own choice")}
    if zero1:
        res["buckets"] = len(z.buckets)
    return res


def cpu_baseline(torch):
    """CPU oracle (plain PyTorch fp32 restatement) on a bounded sample of the headline workload."""
    from oracle import attention as oa

    threads = os.cpu_count() or 1
    torch.set_num_threads(threads)
    B, H, S, D = 1, 2, 4096, 128  # one slice: 1/32 of the B=4, H=16 workload, same S and D
    gen = torch.Generator().manual_seed(1234)
    q, k, v, do = (torch.randn(B, H, S, D, generator=gen).bfloat16().float() for _ in range(4))
    mask = oa.causal_mask(S, S, "cpu")
    flops = 3.5 * 4.0 * B * H * S * S * D / 2.0

    def step():
        qf, kf, vf = (t.clone().requires_grad_(True) for t in (q, k, v))
        o, _ = oa.attention_with_lse(qf, kf, vf, mask)
        o.backward(do)

    # the whole B=4, H=16 workload is 32 such slices; the oracle materialises an S x S score matrix per head, so it walks
    # them one after the other (same arithmetic, 1/32 of the memory)
    slices = 32
    step()
    passes, t0 = 0, time.perf_counter()
    while passes < 1 or (time.perf_counter() - t0 < 10.0 and passes < 3):
        for _ in range(slices):
            step()
        passes += 1
    sec = (time.perf_counter() - t0) / passes
    return {"value": slices * flops / sec / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"oracle.attention (fp32 PyTorch restatement) fwd+bwd over the full workload, walked as {slices} slices of "
                      f"B={B},H={H},S={S},D={D}: {passes} pass(es), {sec:.2f} s each (1 warm-up slice)"}


def llama_cfg_inputs(torch, cfg_dict, batch, seq, seed=1234):
    """Initial weights (matrices N(0, 0.02), norm weights 1, in named_parameters order) and token ids of a LLaMA
    configuration, drawn from one CPU generator."""
    from collections import OrderedDict

    from oracle import llama as ol

    cfg = ol.OracleLlamaConfig(**cfg_dict)
    gen = torch.Generator().manual_seed(seed)
    params = OrderedDict()
    for name, shape in ol.param_shapes(cfg).items():
        params[name] = torch.randn(shape, generator=gen) * 0.02 if len(shape) >= 2 else torch.ones(shape)
    ids = torch.randint(0, cfg.vocab_size, (batch, seq + 1), generator=gen)
    return cfg, params, ids[:, :-1].contiguous(), ids[:, 1:].contiguous()


CFG1 = dict(vocab_size=8192, hidden_size=256, intermediate_size=688, num_hidden_layers=4, num_attention_heads=4,
            max_position_embeddings=256, rms_norm_eps=1e-5, rope_theta=10000.0)
CFG5 = dict(vocab_size=32000, hidden_size=512, intermediate_size=1376, num_hidden_layers=8, num_attention_heads=8,
            max_position_embeddings=2048, rms_norm_eps=1e-5, rope_theta=10000.0)


def cpu_baseline_llama(torch, dev, which):
    """One full train step (forward, backward, clip for configuration 5, stock AdamW on fp32 masters) of the CPU oracle
    on the host cores at full size, next to the same first step through the HIP path from identical weights and
    tokens: time, tokens/s and the parity of loss and gradient norm."""
    from maltos_amd.grad_clip import clip_grad_norm_, clip_grad_norm_fused_
    from maltos_amd.llama import LlamaConfig, LlamaForCausalLM, set_grad_accumulation_into_buffers
    from maltos_amd.optim import FusedAdamW, MasterWeightsOptimizer
    from oracle import llama as ol

    cfg_dict, batch, seq, dtype, max_norm = ((CFG1, 8, 256, torch.float32, None) if which == "cfg1"
                                             else (CFG5, 8, 2048, torch.bfloat16, 1.0))
    cfg, params, inp, lab = llama_cfg_inputs(torch, cfg_dict, batch, seq)
    threads = os.cpu_count() or 1
    torch.set_num_threads(threads)
    rounded = {n: p.to(dtype).float() for n, p in params.items()}   # the oracle evaluates the rounded network in fp32
    timed_steps = 2 if which == "cfg1" else 1
    ol.train_step(rounded, cfg, inp, lab, max_norm=max_norm) if which == "cfg1" else None   # warm-up (small case only)
    t0 = time.perf_counter()
    for _ in range(timed_steps):
        want_loss, want_norm, _ = ol.train_step(rounded, cfg, inp, lab, max_norm=max_norm)
    cpu_sec = (time.perf_counter() - t0) / timed_steps
    model = LlamaForCausalLM(LlamaConfig(**cfg_dict)).to(dev)
    with torch.no_grad():
        for n, p in model.named_parameters():
            p.copy_(params[n])
    model = model.to(dtype)
    if dtype != torch.float32:
        set_grad_accumulation_into_buffers(model)   # as the llama50m_train_step leg: dW adds into the flat gradient buffer
    adam = lambda ps: FusedAdamW(ps, lr=3e-4, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
    opt = MasterWeightsOptimizer(model.parameters(), optimizer_factory=adam) if dtype != torch.float32 else adam(model.parameters())
    data = {"input_ids": inp.to(dev), "labels": lab.to(dev)}
    first = {}

    def step(timed_step=True):
        loss = model(data)
        loss.backward()
        if not timed_step:   # the first step: the norm is read back for the parity figures (one host round trip)
            first["norm"] = float(clip_grad_norm_(opt, max_norm if max_norm is not None else float("inf")))   # inf: the norm only
            first["loss"] = float(loss.detach())
        elif max_norm is not None:   # the timed steps clip on the device, as the llama50m_train_step leg does
            clip_grad_norm_fused_(opt, max_norm)
        opt.step()
        opt.zero_grad(set_to_none=True)

    from maltos_amd.gemm_tuning import tuned_gemms_off, use_tuned_gemms
    gemm_shapes = use_tuned_gemms() if which == "cfg5" else 0   # as the llama50m_train_step leg; the parity step below too
    step(timed_step=False)
    gpu_sec = timed(torch, step, 10, 3, preheat_steps=LLAMA_PREHEAT_STEPS)
    tuned_gemms_off()
    tokens = batch * seq
    return {"workload": f"{'tiny LLaMA fp32 (configuration 1)' if which == 'cfg1' else 'LLaMA-50M bf16 (configuration 5)'} full train step, "
                        f"batch {batch} x {seq}",
            "cpu": {"ms": cpu_sec * 1e3, "tokens_per_sec": tokens / cpu_sec, "cores": torch.get_num_threads(), "kind": "port",
                    "sample": f"oracle.llama.train_step (fp32 PyTorch restatement, stock AdamW) at full size, {timed_steps} timed step(s)"
                              + (", 1 warm-up" if which == "cfg1" else ", no warm-up")},
            "gpu": {"ms": gpu_sec * 1e3, "tokens_per_sec": tokens / gpu_sec,
                    "gemm_kernels": (f"per-shape selection of maltos_amd/tuned/gemm_gfx950.csv ({gemm_shapes} shapes)" if gemm_shapes
                                     else "the GEMM libraries' own choice"),
                    "clip": "none (the configuration has no clip)" if max_norm is None else
                            "global-norm clip at 1.0 applied on the device (no host read): the eager step of extra.llama50m_train_step"},
            "parity": {"loss": {"hip": first["loss"], "oracle": want_loss, "rel": abs(first["loss"] - want_loss) / abs(want_loss)},
                       "grad_norm": {"hip": first["norm"], "oracle": want_norm, "rel": abs(first["norm"] - want_norm) / abs(want_norm)},
                       "bound": "1e-4 relative (fp32)" if which == "cfg1" else "1e-3 relative (bf16)"}}


def main() -> int:
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU only (got --gpus {args.gpus}); every figure here is a single-GPU figure.",
              file=sys.stderr)
        return 2
    import torch

    from maltos_amd import _lib, ops

    if not torch.cuda.is_available():
        print("bench.py needs a GPU: the HIP path has no CPU fallback.", file=sys.stderr)
        return 2
    dev = torch.device("cuda:0")
    if args.calibrate_traffic:
        x = torch.ones(1 << 28, device=dev)
        for _ in range(3):
            ops.scale_(x, 1.0001)
        torch.cuda.synchronize()
        print(json.dumps({"calibration_kernel": "scale_kernel", "launches": 3, "read_bytes_per_launch": 1 << 30,
                          "written_bytes_per_launch": 1 << 30}))
        return 0
    sec, flops, kernels, kernel_flops = bench_attention(torch, ops, _lib, dev, args.steps, args.warmup)
    total_flops = flops["fwd"] + flops["bwd"]
    value = total_flops / sec / 1e12
    dominant = max(kernels, key=lambda n: kernels[n]["ms"] * kernels[n]["launches_per_step"])
    dom = kernels[dominant]
    result = {
        "metric": "attn fwd+bwd TFLOP/s (% MFMA peak) S=4096; train tokens/sec LLaMA-50M, 1 GPU",
        "value": value,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": sec * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "causal self-attention fwd+bwd, B=4 H=16 S=4096 D=128, bf16 (configuration 2)",
                   "flops_per_step": total_flops, "frac_of_mfma_peak": value / MFMA_BF16_PEAK_TFLOPS,
                   "preheat": f"{PREHEAT_S} s of untimed steps before the warm-up steps (clock ramp of an idle GPU)"},
        "roofline": {"bound": "mfma", "kernel": dominant, "achieved": dom["tflops"], "peak": MFMA_BF16_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": dom["tflops"] / MFMA_BF16_PEAK_TFLOPS,
                     "traffic": measured_hbm_traffic().get(dominant),
                     "kernel_ms": dom["ms"], "algorithmic_flops_per_launch": kernel_flops[dominant]},
        "kernels": kernels,
    }
    if not args.skip_extra:
        extra = {}

        def leg(name, fn):
            # a secondary figure that cannot be produced is reported as such; the headline line is still printed
            if args.only is not None and name != args.only:
                return
            try:
                extra[name] = fn()
            except Exception as exc:  # noqa: BLE001
                extra[name] = {"error": f"{type(exc).__name__}: {exc}"[:500]}
                torch.cuda.synchronize()

        half = max(5, args.steps // 2)
        leg("parity_cfg2", lambda: parity_cfg2(torch, ops, dev))
        leg("attn_d64", lambda: bench_attention_d64(torch, ops, _lib, dev, args.steps, args.warmup))
        leg("cfg3_packed_gqa", lambda: bench_cfg3_packed_gqa(torch, ops, _lib, dev, half, args.warmup))
        leg("parity_cfg3", lambda: parity_cfg3(torch, ops, dev))
        leg("cfg4_ring_rank", lambda: bench_cfg4_ring_rank(torch, dev, half, 3))
        leg("parity_cfg4", lambda: parity_cfg4(torch, dev))
        leg("adamw_flat_fp32", lambda: bench_adamw(torch, ops, _lib, dev, max(10, args.steps), args.warmup))
        leg("hbm_kernels", lambda: bench_hbm_kernels(torch, ops, _lib, dev))
        leg("llama50m_train_step", lambda: bench_llama50m(torch, dev, half, max(10, args.warmup)))
        leg("llama50m_train_step_graph", lambda: bench_llama50m(torch, dev, half, max(10, args.warmup), graph=True))
        leg("llama50m_train_step_graph_library_gemm_choice",
            lambda: bench_llama50m(torch, dev, half, max(10, args.warmup), graph=True, no_tuned_gemms=True))
        leg("llama50m_train_step_zero1_layout", lambda: bench_llama50m(torch, dev, half, max(10, args.warmup), zero1=True))
        leg("llama50m_train_step_zero2_layout", lambda: bench_llama50m(torch, dev, half, max(10, args.warmup), zero2=True))
        if not args.skip_cpu:
            leg("cfg1_tiny_llama_step_vs_cpu", lambda: cpu_baseline_llama(torch, dev, "cfg1"))
            leg("cfg5_llama50m_step_vs_cpu", lambda: cpu_baseline_llama(torch, dev, "cfg5"))
        result["extra"] = extra
    if not args.skip_cpu:
        result["cpu_baseline"] = cpu_baseline(torch)
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
