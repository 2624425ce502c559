#!/usr/bin/env python3
"""Benchmark of the quantized attention path on one MI355X.

A step is one full pass of the path over one batch of synthetic q/k/v already resident in HBM:
quantize Q, quantize K (mean, Hadamard, int8), quantize V (fp8), fused attention - the same
kernel sequence ``ksana_sage_forward`` enqueues, issued stage by stage so HIP events on the
launch stream can bracket the attention kernel inside the timed region.

Prints ONE JSON line.  ``value`` is attention flops (4*B*H*L^2*D) per second of whole-step time.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

METRIC = "Sage-attn effective TFLOPS & % INT8/FP8 MFMA peak, Wan-14B 480p (L=32760)"
MFMA_PEAK_TFLOPS = 5000.0  # MI355X dense INT8 (POP/s) = dense FP8 (PFLOP/s) = 5.0e15 /s
HBM_PEAK_GBS = 8000.0
# HBM bytes per launch of the attention kernel at the headline workload: 2.0 x FETCH_SIZE + 1.0 x WRITE_SIZE from
# two rocprofv3 --pmc runs, factors from a 1 GiB device copy in the same runs.  A constant from that profile, not a
# counter read in this run (counters need rocprofv3 around the process).
ATTN_TRAFFIC_BYTES = {"wan14b_480p": 1808505 * 1024}
ATTN_TRAFFIC_SOURCE = "profiles/sage_attn_fwd_kernel_wan14b_480p.md (rocprofv3 --pmc, not this run)"


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default=None, help="one of ksanadit_amd.workloads.WORKLOADS (default: headline)")
    ap.add_argument("--pwl-exp2", action="store_true", help="piecewise-linear e4m3 code instead of exp2 on the transcendental unit (faster, less accurate)")
    ap.add_argument("--calib-copy-mib", type=int, default=0, help="also run one plain device copy of this many MiB (reference point for HBM traffic counters)")
    ap.add_argument("--skip-extra", action="store_true", help="leave out the block-sparse and norm+RoPE legs (they run after the timed steps)")
    ap.add_argument("--skip-block-sparse", action="store_true", help="leave out the block-sparse leg only")
    ap.add_argument("--skip-sla", action="store_true", help="leave out the sparse-linear backend's leg")
    ap.add_argument("--skip-causal", action="store_true", help="leave out the causal leg only (it launches the same kernel instantiation as the block-sparse leg)")
    ap.add_argument("--skip-other-workloads", action="store_true", help="leave out the attention timings at the other measured shapes")
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="target length of the CPU SDPA sample; 0 skips it")
    return ap.parse_args()


def cpu_baseline(workload, target_s: float):
    """The oracle's SDPA (ksana/operations/attention/backends/sdpa.py:47-79 restated) on the host
    cores, on a head-subsample of the same workload sized to about ``target_s`` seconds."""
    from ksanadit_amd.workloads import make_inputs
    from oracle.sdpa_ref import sdpa_ref

    cores = torch.get_num_threads()
    per_head = workload.flops / workload.H

    def timed(heads, seq=None):
        q, k, v = make_inputs(workload, heads=heads, seq=seq)
        t0 = time.perf_counter()
        sdpa_ref(q, k, v)
        return time.perf_counter() - t0

    probe_seq = min(workload.L, 4096)
    timed(1, probe_seq)  # warm the thread pool
    t_probe = timed(1, probe_seq)
    rate = 4.0 * workload.B * probe_seq * probe_seq * workload.D / t_probe
    heads = int(max(1, min(workload.H, target_s * rate / per_head)))
    t = timed(heads)
    flops = per_head * heads
    model = "unknown"
    try:
        with open("/proc/cpuinfo") as f:
            model = next((line.split(":", 1)[1].strip() for line in f if line.startswith("model name")), model)
    except OSError:
        pass
    return {
        "value": round(flops / t / 1e12, 4),
        "unit": "TFLOP/s",
        "cores": cores,
        "cpu_model": model,
        "kind": "port",
        "sample": f"{workload.name}: {heads} of {workload.H} heads at full L={workload.L}, bf16, one call, {t:.2f} s",
        "ms_per_call_extrapolated": round(t / heads * workload.H * 1e3, 1),
    }


def pctl(xs, q):
    xs = sorted(xs)
    return xs[min(len(xs) - 1, max(0, int(round(q * (len(xs) - 1)))))]


def spread(xs, digits=4):
    """median, 10th and 90th percentile of a list of per-step times"""
    return {"median": round(pctl(xs, 0.5), digits), "p10": round(pctl(xs, 0.1), digits), "p90": round(pctl(xs, 0.9), digits)}


def device_inputs(w, dev, Lq=None, Lk=None):
    """q, k, v of a workload's distributions drawn on the device (seeded): for legs whose timing, not whose values,
    is reported - drawing 3 x 387 M values on the host would take longer than everything else together."""
    g = torch.Generator(device=dev).manual_seed(w.seed)
    Lq = w.L if Lq is None else Lq
    Lk = w.L if Lk is None else Lk

    def draw(L, offset, outliers):
        x = torch.randn((w.B, L, w.H, w.D), generator=g, device=dev, dtype=torch.float32)
        if w.text_tokens:
            x[:, : min(w.text_tokens, L)] *= w.text_std
        if offset:
            x += torch.randn((w.H, w.D), generator=g, device=dev) * w.k_offset_std
        if outliers and w.outlier_p > 0:
            m = torch.rand(x.shape, generator=g, device=dev) < w.outlier_p
            x = torch.where(m, x * w.outlier_gain, x)
        return x.to(torch.bfloat16)

    return draw(Lq, False, True), draw(Lk, True, True), draw(Lk, False, False)


def time_attention(sage_ops, ws, out, iters, **kw):
    """median / p10 / p90 of the attention call on the operands in ``ws`` (HIP events on the launch stream)"""
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(2)] for _ in range(iters)]
    sage_ops.attn_fwd(ws, out, **kw)
    torch.cuda.synchronize()
    for e in ev:
        e[0].record()
        sage_ops.attn_fwd(ws, out, **kw)
        e[1].record()
    torch.cuda.synchronize()
    return [e[0].elapsed_time(e[1]) for e in ev]


def mfma_probe(dev, iters=5):
    """What the matrix pipe sustains on the attention kernel's own MFMA mix with nothing else running."""
    import ctypes as C

    from ksanadit_amd import _capi

    lib = _capi.load()
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    scratch = torch.empty(cus * 512, dtype=torch.float32, device=dev)
    ops = C.c_double(0.0)
    stream = C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    times = []
    for i in range(iters + 1):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        _capi.check(lib.ksana_sage_mfma_probe(scratch.data_ptr(), scratch.numel() * 4, cus, 20000, stream, C.byref(ops)),
                    "ksana_sage_mfma_probe")
        e1.record()
        torch.cuda.synchronize()
        if i:
            times.append(e0.elapsed_time(e1))
    return round(ops.value / (pctl(times, 0.5) * 1e-3) / 1e12, 1)


def op_end_to_end(w, q, k, v, iters=7):
    """One call through KsanaAttentionOp as a model block makes it: backend adaptor, workspace from torch's allocator,
    three quantizers, attention, output tensor."""
    from ksanadit_amd import KsanaAttentionBackend, KsanaAttentionConfig, pick_attn_op

    op = pick_attn_op(KsanaAttentionConfig(backend=KsanaAttentionBackend.SAGE_ATTN))(num_heads=w.H, head_size=w.D)
    op(q, k, v)
    torch.cuda.synchronize()
    times = []
    for _ in range(iters):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        o = op(q, k, v)
        e1.record()
        torch.cuda.synchronize()
        times.append(e0.elapsed_time(e1))
        del o
    res = spread(times)
    # the same calls issued back to back, as a model issues them: the host side of a call (allocator, ctypes, five
    # launches) then runs while the GPU works on the call before, and only the GPU time is left
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        o = op(q, k, v)
        del o
    e1.record()
    torch.cuda.synchronize()
    res["back_to_back"] = round(e0.elapsed_time(e1) / iters, 4)
    return res


def other_workloads(sage_ops, dev, pwl, iters=7):
    """Attention-kernel time at the other measured shapes (parity-test shapes; values drawn on the device)."""
    from ksanadit_amd.workloads import WORKLOADS, Workload

    cases = [(WORKLOADS[n], None, None) for n in ("wan5b_720p", "wan14b_720p", "qwen_cfg")]
    # WanCrossAttention: every video token attends to the 512 text tokens (wan_model.py:233-251, text_len 512)
    cases.append((Workload("wan14b_480p_cross_attn", 1006, 1, 40, 32760), 32760, 512))
    res = {}
    for w, Lq, Lk in cases:
        q, k, v = device_inputs(w, dev, Lq, Lk)
        ws = sage_ops.workspace_for(q, k)
        out = torch.empty_like(q)
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
        sm = w.D**-0.5
        sage_ops.quant_q(q, ws, sm), sage_ops.quant_k(k, ws, True), sage_ops.quant_v(v, ws)
        torch.cuda.synchronize()
        ev[0].record()
        sage_ops.quant_q(q, ws, sm), sage_ops.quant_k(k, ws, True), sage_ops.quant_v(v, ws)
        ev[1].record()
        times = time_attention(sage_ops, ws, out, iters, pwl_exp2=pwl)
        flops = 4.0 * w.B * w.H * q.shape[1] * k.shape[1] * w.D
        ms = pctl(times, 0.5)
        res[w.name] = {"shape": f"B={w.B} H={w.H} Lq={q.shape[1]} Lk={k.shape[1]} D={w.D}", "attn_kernel_ms": spread(times),
                       "attn_kernel_tflops": round(flops / (ms * 1e-3) / 1e12, 1),
                       "frac_of_mfma_peak": round(flops / (ms * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS, 4),
                       "quantizer_ms": round(ev[0].elapsed_time(ev[1]), 4)}
        if w.name == "wan14b_720p":
            # tile lists of more than 1 024 entries (1 182 key tiles): a radial-style mask and causal masking
            mask = radial_style_mask(w.L, WAN_GRIDS[w.name]).to(dev)
            density = float(mask.float().mean())
            t_mask = pctl(time_attention(sage_ops, ws, out, 3, pwl_exp2=pwl, block_mask=mask), 0.5)
            t_causal = pctl(time_attention(sage_ops, ws, out, 3, pwl_exp2=pwl, causal=True), 0.5)
            res[w.name]["block_sparse"] = {"density": round(density, 4), "attn_kernel_ms": round(t_mask, 4),
                                           "kept_block_rate_vs_dense": round(density * ms / t_mask, 3)}
            res[w.name]["causal"] = {"attn_kernel_ms": round(t_causal, 4),
                                     "kept_pair_rate_vs_dense": round((w.L + 1) / (2.0 * w.L) * ms / t_causal, 3)}
        del q, k, v, ws, out
        torch.cuda.empty_cache()
    # Head size 64 (no BASELINE model has it; the backend interface serves it): the headline shape's token count
    d64 = Workload("wan14b_480p_head_size_64", 1008, 1, 40, 32760)
    q, k, v = device_inputs(d64, dev)
    q, k, v = (t[..., :64].contiguous() for t in (q, k, v))
    ws = sage_ops.workspace_for(q, k)
    out = torch.empty_like(q)
    sage_ops.quant_q(q, ws, 64**-0.5), sage_ops.quant_k(k, ws, True), sage_ops.quant_v(v, ws)
    times = time_attention(sage_ops, ws, out, iters, pwl_exp2=pwl)
    wide = pctl(time_attention(sage_ops, ws, out, iters, tile_skip=True), 0.5) if not pwl else None
    ms = pctl(times, 0.5)
    flops = 4.0 * d64.B * d64.H * d64.L * d64.L * 64
    res[d64.name] = {"shape": f"B={d64.B} H={d64.H} L={d64.L} D=64", "attn_kernel_ms": spread(times),
                     "attn_kernel_tflops": round(flops / (ms * 1e-3) / 1e12, 1),
                     "frac_of_mfma_peak": round(flops / (ms * 1e-3) / 1e12 / MFMA_PEAK_TFLOPS, 4),
                     "attn_kernel_ms_full_width_code": None if wide is None else round(wide, 4),
                     "note": "operands zero-extended to 128 channels; the matrix instructions cover the lower 64 only (the upper 64 repeat them after the Hadamard transform)"}
    del q, k, v, ws, out
    torch.cuda.empty_cache()
    # Peaked attention, made on purpose: the headline distributions with q scaled by 4 (every score 4 times as far from
    # its row's mean), with and without the tile skip (KSANA_SAGE_FLAG_TILE_SKIP: same bits, see the header)
    if not pwl:
        w = WORKLOADS["wan14b_480p"]
        q, k, v = device_inputs(w, dev)
        q = (q.float() * 4.0).to(torch.bfloat16)
        ws = sage_ops.workspace_for(q, k)
        out, out2 = torch.empty_like(q), torch.empty_like(q)
        sage_ops.quant_q(q, ws, w.D**-0.5), sage_ops.quant_k(k, ws, True), sage_ops.quant_v(v, ws)
        full = pctl(time_attention(sage_ops, ws, out, iters), 0.5)
        skip = pctl(time_attention(sage_ops, ws, out2, iters, tile_skip=True), 0.5)
        res["wan14b_480p_scores_x4"] = {"shape": f"B={w.B} H={w.H} L={w.L} D={w.D}, q x 4", "attn_kernel_ms": round(full, 4),
                                        "attn_kernel_ms_tile_skip": round(skip, 4), "same_bits": bool(torch.equal(out, out2))}
        del q, k, v, ws, out, out2
        torch.cuda.empty_cache()
    return res


def radial_leg(sage_ops, dev, pwl, iters=5):
    """The block-sparse call with the mask the radial backend builds (backends/radial_mask.py, which reproduces the
    reference's generator bit for bit) on a latent grid that backend accepts: height and width multiples of 16
    (radial_sage_attn.py:123-124), here 21 frames of 64 x 112 -> 32 x 56 tokens, L = 37632, H = 40."""
    from ksanadit_amd.backends.radial_mask import kernel_block_mask, radial_block_mask
    from ksanadit_amd.config import KsanaRadialSageAttentionConfig
    from ksanadit_amd.workloads import Workload

    cfg = KsanaRadialSageAttentionConfig()
    frames, tpf = 21, 32 * 56
    w = Workload("wan14b_radial_grid", 1007, 1, 40, frames * tpf, outlier_p=1e-3)
    q, k, v = device_inputs(w, dev)
    ws = sage_ops.workspace_for(q, k)
    out = torch.empty_like(q)
    sm = w.D**-0.5
    sage_ops.quant_q(q, ws, sm), sage_ops.quant_k(k, ws, True), sage_ops.quant_v(v, ws)
    pattern = radial_block_mask(w.L, w.L, frames, cfg.block_size, cfg.decay_factor)
    mask = kernel_block_mask(pattern, cfg.block_size, w.L).to(dev)
    density = float(mask.float().mean())
    dense = pctl(time_attention(sage_ops, ws, out, iters, pwl_exp2=pwl), 0.5)
    times = time_attention(sage_ops, ws, out, iters, pwl_exp2=pwl, block_mask=mask)
    ms = pctl(times, 0.5)
    return {"mask": f"radial_block_mask(L={w.L}, frames={frames}, block_size={cfg.block_size}, decay_factor={cfg.decay_factor})",
            "shape": f"B=1 H=40 L={w.L} D=128", "density": round(density, 4), "attn_kernel_ms": spread(times),
            "dense_attn_kernel_ms": round(dense, 4),
            "tflops_on_kept_blocks": round(w.flops * density / (ms * 1e-3) / 1e12, 2),
            "kept_block_rate_vs_dense": round((w.flops * density / ms) / (w.flops / dense), 3)}


# (frames, height, width) of the latent token grid behind each Wan workload's sequence length
WAN_GRIDS = {"cpu_plumbing": (3, 20, 26), "wan5b_720p": (31, 22, 40), "wan14b_480p": (21, 30, 52),
             "wan14b_720p": (21, 45, 80)}


def radial_style_mask(L, grid, blk_q=128, blk_k=64):
    """A block mask with the structure of the reference's radial masks (attn_mask.py:45-110): every query sees
    the first frame and its own; the band of allowed in-frame distances halves each time the frame distance
    doubles.  Built here for timing; it is not the reference's generator."""
    f, h, wd = grid
    tpf = h * wd
    nq, nk = -(-L // blk_q), -(-L // blk_k)
    qpos = torch.arange(nq) * blk_q + blk_q // 2
    kpos = torch.arange(nk) * blk_k + blk_k // 2
    qf, kf = (qpos // tpf).clamp(max=f - 1), (kpos // tpf).clamp(max=f - 1)
    qi, ki = qpos % tpf, kpos % tpf
    dist = (qf[:, None] - kf[None, :]).abs()
    group = torch.where(dist > 0, torch.floor(torch.log2(dist.clamp(min=1).float())) + 1, torch.zeros(()))
    width = torch.where(dist == 0, torch.full((), float(tpf)), (tpf / 2.0) / torch.pow(2.0, group - 1)).clamp(min=blk_q)
    mask = (qi[:, None] - ki[None, :]).abs() <= width
    mask |= (kf == 0)[None, :]
    return mask.to(torch.int8)


def block_sparse_leg(sage_ops, w, ws, out, grid, pwl, iters):
    """Outside the timed step: the attention kernel driven by a radial-style block mask (128 x 64 blocks)."""
    mask = radial_style_mask(w.L, grid).to(out.device)
    density = float(mask.float().mean())
    pairs = mask[: mask.shape[0] // 2 * 2].view(-1, 2, mask.shape[1]).amax(dim=1)  # what a 256-row workgroup walks
    density_wg = float(pairs.float().mean())
    times = time_attention(sage_ops, ws, out, iters, pwl_exp2=pwl, block_mask=mask)
    ms = pctl(times, 0.5)
    return {
        "mask": "radial-style, 128x64 blocks, broadcast over heads",
        "density": round(density, 4),
        "density_per_256_row_workgroup": round(density_wg, 4),
        "attn_kernel_ms": round(ms, 4),
        "attn_kernel_ms_spread": spread(times),
        "tflops_on_kept_blocks": round(w.flops * density / (ms * 1e-3) / 1e12, 2),
    }


def causal_leg(sage_ops, w, ws, out, pwl, iters):
    """Outside the timed step: the same kernel with causal masking (half of the score matrix)."""
    times = time_attention(sage_ops, ws, out, iters, causal=True, pwl_exp2=pwl)
    ms = pctl(times, 0.5)
    kept = (w.L + 1) / (2.0 * w.L)  # fraction of (query, key) pairs on or below the diagonal
    return {"attn_kernel_ms": round(ms, 4), "tflops_on_kept_pairs": round(w.flops * kept / (ms * 1e-3) / 1e12, 2)}


def prep_quantizer_leg(sage_ops, w, q, k, v, ws, sm_scale, grid, dev, iters):
    """Outside the timed step: the quantizer with the block's RMSNorm + RoPE applied on the fly
    (q and k taken as the raw projections).  Same 9 N algorithmic bytes as the plain quantizer; what a
    separate norm kernel and a separate rotation kernel would add is 8 N more for each of q and k."""
    g = torch.Generator().manual_seed(7)
    wq = (1.0 + 0.2 * torch.randn(w.H * w.D, generator=g)).to(dev)
    wk = (1.0 + 0.2 * torch.randn(w.H * w.D, generator=g)).to(dev)
    d = w.D

    def table(rows, dim):  # exp(i * pos * theta^(-2j/dim)), complex128
        f = torch.outer(torch.arange(rows), 1.0 / torch.pow(10000.0, torch.arange(0, dim, 2).to(torch.float64).div(dim)))
        return torch.polar(torch.ones_like(f), f)

    freqs = torch.cat([table(1024, d - 4 * (d // 6)), table(1024, 2 * (d // 6)), table(1024, 2 * (d // 6))], dim=1).to(dev)
    prep = sage_ops.WanPrep(wq, wk, 1e-6, freqs, [grid])
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(2)] for _ in range(iters)]

    def run(e=None):
        if e:
            e[0].record()
        sage_ops.quant_qk(q, k, ws, sm_scale, True, prep=prep)
        sage_ops.quant_v(v, ws)
        if e:
            e[1].record()

    run()
    torch.cuda.synchronize()
    for e in ev:
        run(e)
    torch.cuda.synchronize()
    ms = sum(e[0].elapsed_time(e[1]) for e in ev) / iters
    nbytes = 9.0 * w.elements
    gbs = nbytes / (ms * 1e-3) / 1e9

    def eager_norm_rope(x, weight):
        """The same step as the model block runs it, with torch's own kernels on this GPU: RMSNorm in fp32
        (ksana/operations/ops.py:62-72), then the rotation in complex128 (ksana/utils/rope.py:103-128)."""
        B, L, H, D = x.shape
        xf = x.reshape(B, L, H * D).float()
        y = ((xf * torch.rsqrt(xf.pow(2).mean(dim=-1, keepdim=True) + 1e-6)) * weight).type_as(x).view(B, L, H, D)
        f, h, wd = grid
        parts = freqs.split([D // 2 - 2 * (D // 2 // 3), D // 2 // 3, D // 2 // 3], dim=1)
        tab = torch.cat([parts[0][:f].view(f, 1, 1, -1).expand(f, h, wd, -1), parts[1][:h].view(1, h, 1, -1).expand(f, h, wd, -1),
                         parts[2][:wd].view(1, 1, wd, -1).expand(f, h, wd, -1)], dim=-1).reshape(f * h * wd, 1, -1)
        n = f * h * wd
        z = torch.view_as_complex(y[0, :n].to(torch.float64).reshape(n, H, -1, 2))
        z = torch.view_as_real(z * tab).flatten(2)
        return torch.stack([torch.cat([z, y[0, n:]])]).type_as(x)

    eager_norm_rope(q, wq)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    eager_norm_rope(q, wq)
    eager_norm_rope(k, wk)
    e1.record()
    torch.cuda.synchronize()
    eager_ms = e0.elapsed_time(e1)
    return {
        "what": "quantizer with RMSNorm(row of H*D) and 3-axis RoPE on q, k (q and k in one call; row statistics taken inside q's kernel); V as before",
        "grid": list(grid),
        "ms": round(ms, 4),
        "bound": "hbm",
        "achieved": round(gbs, 1),
        "peak": HBM_PEAK_GBS,
        "unit": "GB/s",
        "frac": round(gbs / HBM_PEAK_GBS, 4),
        "algorithmic_bytes": nbytes,
        "eager_norm_rope_ms": round(eager_ms, 3),
        "eager_note": "norm + rotation of q and k as the model block issues them (torch kernels on this GPU), to be added "
                      "to quantizer_ms for the path without the on-the-fly step",
    }


def sla_leg(sage_ops, w, q, k, v, ws, dev, iters, topk=0.1):
    """Outside the timed step: the sparse-linear backend at the headline shape, part by part (HIP events): the block
    map (block averages taken along by the quantizers of q and k, then scores + top-k), the block-sparse attention on that map,
    the linear branch with the block's linear layer and the final sum folded in (HIP), and - for scale - the same
    branch as the reference issues it (five torch kernels plus the layer plus the sum)."""
    from ksanadit_amd.backends import sage_sla
    from ksanadit_amd.config import KsanaSageSLAConfig
    from ksanadit_amd import pick_attn_op

    def timed(fn):
        fn()
        torch.cuda.synchronize()
        ev = [[torch.cuda.Event(enable_timing=True) for _ in range(2)] for _ in range(iters)]
        for e in ev:
            e[0].record()
            fn()
            e[1].record()
        torch.cuda.synchronize()
        return pctl([e[0].elapsed_time(e[1]) for e in ev], 0.5)

    proj = torch.nn.Linear(w.D, w.D, bias=True).to(dev).to(q.dtype)
    sm = w.D**-0.5
    # (the legs before this one left other operands in the workspace)
    pq, pk = sage_ops.quant_qk_pooled(q, k, ws, sm)
    sage_ops.quant_v(v, ws)
    bm, kept = sage_sla.block_map_from_pooled(pq, pk, topk)
    out = torch.empty_like(q)
    # the block averages ride in the quantizers of q and k: what they add to those two, and the map kernel itself
    plain_ms = timed(lambda: (sage_ops.quant_q(q, ws, sm), sage_ops.quant_k(k, ws, True)))
    pooled_ms = timed(lambda: sage_ops.quant_qk_pooled(q, k, ws, sm))
    map_ms = timed(lambda: sage_sla.block_map_from_pooled(pq, pk, topk))
    pool_ms = timed(lambda: (sage_ops.block_means(q, 128), sage_ops.block_means(k, 64, centre=ws.k_mean)))
    attn_ms = timed(lambda: sage_ops.attn_fwd(ws, out, block_mask=bm))
    with torch.no_grad():
        lin_ms = timed(lambda: sage_ops.sla_linear(q, k, v, proj.weight, proj.bias, add=out, out=out))
        qh, kh, vh = (t.transpose(1, 2) for t in (q, k, v))

        def eager():
            o_l = sage_sla.linear_branch(qh, kh, vh)
            with torch.amp.autocast("cuda", dtype=q.dtype):
                o_l = proj(o_l)
            return (out.transpose(1, 2) + o_l).to(q.dtype).transpose(1, 2)

        eager_ms = timed(eager)
        op = pick_attn_op(KsanaSageSLAConfig(topk=topk))(num_heads=w.H, head_size=w.D, causal=False)
        e2e_ms = timed(lambda: op(q, k, v, proj_l=proj))
    nb = w.elements * 2.0
    return {
        "what": "SageSLA backend, topk share %.2f: block map + block-sparse attention + linear branch (layer and sum folded in)" % topk,
        "kept_key_blocks": f"{kept} of {bm.shape[-1]}",
        "block_map_ms": round(map_ms + pooled_ms - plain_ms, 4),
        "block_map_note": "scores + top-k kernel, plus what the block averages add to the quantizers of q and k they ride in",
        "block_averages_in_quantizers_ms": round(pooled_ms - plain_ms, 4),
        "block_averages_as_own_passes_ms": round(pool_ms, 4),
        "sparse_attn_ms": round(attn_ms, 4),
        "sparse_attn_tflops_on_kept_blocks": round(w.flops * kept / bm.shape[-1] / (attn_ms * 1e-3) / 1e12, 1),
        "linear_branch_ms": round(lin_ms, 4),
        "linear_branch_gbs": round(5.0 * nb / (lin_ms * 1e-3) / 1e9, 1),
        "linear_branch_note": "algorithmic bytes 5 x 2N: q, k, v and the sparse result read once, the sum written once",
        "linear_branch_torch_ms": round(eager_ms, 4),
        "op_e2e_ms": round(e2e_ms, 4),
    }


def main() -> int:
    args = parse()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported (every run here has exactly one MI355X)", file=sys.stderr)
        return 2
    if not torch.cuda.is_available():
        print("bench.py needs a HIP device", file=sys.stderr)
        return 2

    from ksanadit_amd import sage_ops
    from ksanadit_amd.workloads import HEADLINE, WORKLOADS, make_inputs

    w = WORKLOADS[args.workload or HEADLINE]
    dev = torch.device("cuda:0")
    q, k, v = make_inputs(w, device=dev)
    ws = sage_ops.workspace_for(q, k)
    out = torch.empty_like(q)
    sm_scale = w.D**-0.5

    def step(ev=None):
        if ev:
            ev[0].record()
        sage_ops.quant_q(q, ws, sm_scale)
        sage_ops.quant_k(k, ws, True)
        sage_ops.quant_v(v, ws)
        if ev:
            ev[1].record()
        sage_ops.attn_fwd(ws, out, pwl_exp2=args.pwl_exp2)
        if ev:
            ev[2].record()

    if args.calib_copy_mib:
        src = torch.empty(args.calib_copy_mib << 20, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        dst.copy_(src)  # reads and writes calib_copy_mib MiB once each
        torch.cuda.synchronize()
        del src, dst
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    events = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(args.steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for ev in events:
        step(ev)
    torch.cuda.synchronize()
    t1 = time.perf_counter()

    ms_step = (t1 - t0) * 1e3 / args.steps
    quant_times = [e[0].elapsed_time(e[1]) for e in events]
    attn_times = [e[1].elapsed_time(e[2]) for e in events]
    step_times = [e[0].elapsed_time(e[2]) for e in events]
    quant_ms = sum(quant_times) / args.steps
    attn_ms = sum(attn_times) / args.steps
    attn_tflops = w.flops / (attn_ms * 1e-3) / 1e12
    n = w.elements
    quant_bytes = 9.0 * n  # q, k, v read once as 16-bit, written once as 8-bit
    quant_gbs = quant_bytes / (quant_ms * 1e-3) / 1e9

    rec = {
        "metric": METRIC,
        "value": round(w.flops / (ms_step * 1e-3) / 1e12, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8+fp8",
        "data": "synthetic",
        "config": {"workload": f"{w.name}: B={w.B} H={w.H} L={w.L} D={w.D} bf16 non-causal, seed {w.seed}",
                   "exp2": "piecewise-linear e4m3 code" if args.pwl_exp2 else "exact"},
        "attn_kernel_ms": round(attn_ms, 4),
        "attn_kernel_tflops": round(attn_tflops, 2),
        "pct_mfma_peak": round(100.0 * attn_tflops / MFMA_PEAK_TFLOPS, 2),
        "quantizer_ms": round(quant_ms, 4),
        # per-step times between HIP events on the launch stream: the means above, and how the steps scatter
        "step_ms_spread": spread(step_times),
        "attn_kernel_ms_spread": spread(attn_times),
        "quantizer_ms_spread": spread(quant_times),
        "roofline": {
            "kernel": "sage_attn_fwd_kernel",
            "bound": "mfma",
            "achieved": round(attn_tflops, 2),
            "peak": MFMA_PEAK_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(attn_tflops / MFMA_PEAK_TFLOPS, 4),
            "traffic": ATTN_TRAFFIC_BYTES.get(w.name),
            "traffic_source": ATTN_TRAFFIC_SOURCE if w.name in ATTN_TRAFFIC_BYTES else None,
        },
        "quantizer_roofline": {
            "kernels": "quant_q; col_partial + k_mean_finalize + quant_k; quant_v_fused (one read of V)",
            "bound": "hbm",
            "achieved": round(quant_gbs, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(quant_gbs / HBM_PEAK_GBS, 4),
            "algorithmic_bytes": quant_bytes,
        },
    }
    grid = WAN_GRIDS.get(w.name)
    if args.skip_extra:
        grid = None
    else:
        # the matrix pipe alone, same process, same clocks
        rec["mfma_microbench_tflops"] = mfma_probe(dev)
        rec["roofline"]["frac_of_mfma_microbench"] = round(attn_tflops / rec["mfma_microbench_tflops"], 4)
        # what a model block pays per call: the op, its adaptor, workspace allocation, quantizers, attention
        rec["op_e2e_ms"] = op_end_to_end(w, q, k, v)
    if grid is not None and w.L <= 131072:
        if not args.skip_block_sparse:
            rec["block_sparse"] = block_sparse_leg(sage_ops, w, ws, out, grid, args.pwl_exp2, max(3, args.steps // 2))
        if not args.skip_causal:
            rec["causal"] = causal_leg(sage_ops, w, ws, out, args.pwl_exp2, max(3, args.steps // 2))
    if grid is not None and w.B == 1:
        rec["prep_quantizer"] = prep_quantizer_leg(sage_ops, w, q, k, v, ws, sm_scale, grid, dev, max(3, args.steps // 2))
    if grid is not None and w.B == 1 and not args.skip_sla:
        rec["sla"] = sla_leg(sage_ops, w, q, k, v, ws, dev, max(3, args.steps // 2))
    if not args.skip_extra and not args.skip_other_workloads:
        del q, k, v, ws, out
        torch.cuda.empty_cache()
        if not args.skip_block_sparse:
            rec["block_sparse_radial"] = radial_leg(sage_ops, dev, args.pwl_exp2)
        rec["other_workloads"] = other_workloads(sage_ops, dev, args.pwl_exp2)
    if args.cpu_seconds > 0:
        rec["cpu_baseline"] = cpu_baseline(w, args.cpu_seconds)
    print(json.dumps(rec))
    return 0


if __name__ == "__main__":
    sys.exit(main())
