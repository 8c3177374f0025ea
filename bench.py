#!/usr/bin/env python3
"""Benchmark of the per-layer padding-removal hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2] [--no-cpu] [--no-extra] [--step-only]

A step is one pass of
    depad -> transpose_pad -> QK^T -> scale_mask_softmax -> PV -> transpose_depad -> residual + LayerNorm
over one synthetic batch whose inputs are already resident in HBM.  The timed form is the one
layer.padding_removal_layer runs when the caller names none (`step_form` in the line): for 16-bit storage two
launches -- fused attention that addresses the packed projections and the packed context through per-sequence row
offsets (so neither transpose is a launch of its own and no score tensor exists), then the LayerNorm, which takes
its residual rows straight from the padded activations (so depad is not a launch either); for fp32 QK^T, softmax
and PV as three kernels on the same packed operands plus that LayerNorm.  The three-kernel form, the reference's
seven ops through one call and the unchanged caller's seven Python calls are timed beside it.  The headline
value is tokens/s of that pass on the workload named by --workload (default c3,
the OPT-30B-shaped layer: the largest of the five that fits one GPU -- 1.9 GB of
scores, 45 GFLOP per contraction -- and the one whose kernels are bound by HBM
bandwidth rather than by launch cost); the other workloads, the per-kernel
bandwidths, the PyTorch-ROCm eager pipeline and the CPU oracle are reported beside
it in the same JSON line.

The line also carries
  roofline      achieved vs peak for the kernel that takes the largest share of the step,
                from algorithmic bytes (or FLOPs) per launch and the kernel's launch-to-launch
                time measured with events on the launch stream;
  cpu_baseline  the CPU oracle (a port of the reference's eager path) timed on
                this box's host cores on a bounded sample of the same workload.
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

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
MFMA_PEAK_TFLOPS = {"f16": 2500.0, "bf16": 2500.0, "f32": 157.3}
PROFILES = os.path.join(ROOT, "profiles")


def library_source_hash() -> str:
    """Digest of the sources libenergon_hip.so was compiled from (en_source_hash)."""
    from energonai_amd import _lib
    return _lib.load().en_source_hash().decode()


def measured_traffic(workload: str, form: str = "default"):
    """HBM bytes per launch of each kernel of the step, from the counter summary kept under profiles/
    (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this file, scaled by what the same counters read for
    en_copy_bytes of known size; written by bench_profiles.py).  Counters cannot be read from inside the
    benchmark, so the figures of the last profiled tree are reported beside the live timing.  Returns
    (bytes by op, digest of the library sources the summary was measured on or None); ({}, None) when the
    summary is not there."""
    tag = "" if form == "default" else f"_{form}"
    path = os.path.join(PROFILES, f"bench_{workload}{tag}_hbm_traffic.md")
    out, digest = {}, None
    try:
        with open(path) as f:
            for line in f:
                if line.startswith("Library sources"):
                    parts = line.split("`")
                    digest = parts[-2] if len(parts) >= 3 else None
                cells = [c.strip() for c in line.strip().strip("|").split("|")]
                if len(cells) >= 3 and cells[0].startswith("`") and cells[0].endswith("`"):
                    try:
                        out[cells[0].strip("`")] = float(cells[-3]) * 1e6      # column "traffic MB"
                    except ValueError:
                        pass
    except OSError:
        pass
    return out, digest


DTYPE_NAME = {"torch.float16": "f16", "torch.bfloat16": "bf16", "torch.float32": "f32"}
PREHEAT_S = 0.1      # untimed load before the warm-up steps, so that the timed steps run at the settled clock


def _event_time_ms(fn, iters, torch):
    """Average time of fn() over iters back-to-back launches, events on the current stream."""
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(iters):
        fn()
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) / iters


def _median_step_ms(fn, iters, torch):
    """Median of per-step event timings (used for the eager baseline, as its definition asks)."""
    times = []
    for _ in range(iters):
        s = torch.cuda.Event(enable_timing=True)
        e = torch.cuda.Event(enable_timing=True)
        s.record()
        fn()
        e.record()
        e.synchronize()
        times.append(s.elapsed_time(e))
    times.sort()
    return times[len(times) // 2]


# ---------------------------------------------------------------------------
# PyTorch-ROCm eager pipeline: the same seven steps with stock torch ops
# ---------------------------------------------------------------------------
def eager_prefill_step(torch, w, d):
    import torch.nn.functional as F
    B, S, H, D = w.batch, w.seq, w.heads, w.head_dim
    lens = d["lens_list"]
    hp = d["hidden_padded"]
    # depad: the reference's cat loop (energonai/kernel/cuda_native/transpose_pad.py:30-37)
    if w.left_padded:
        x = torch.cat([hp[i:i + 1, S - lens[i]:S, :] for i in range(B)], dim=1)
    else:
        x = torch.cat([hp[i:i + 1, 0:lens[i], :] for i in range(B)], dim=1)
    # pad: zeros + index copy + permute
    qkv = torch.zeros(B * S, H, 3 * D, dtype=hp.dtype, device=hp.device)
    qkv.index_copy_(0, d["valid_rows"], d["qkv_packed"][0])
    qkv = qkv.view(B, S, H, 3 * D).permute(0, 2, 1, 3).contiguous()
    q, k, v = torch.chunk(qkv, 3, dim=-1)
    s = torch.matmul(q, k.transpose(-1, -2)) * w.scale
    if w.causal:
        s = torch.where(d["tri"], s, d["neg"])
    s = s + d["key_mask"]
    p = torch.softmax(s, -1, dtype=torch.float).to(hp.dtype)
    ctx = torch.matmul(p, v)
    ctx = ctx.permute(0, 2, 1, 3).reshape(B * S, H * D).index_select(0, d["valid_rows"]).unsqueeze(0)
    attn_out = ctx if d["dense_out"] is None else d["dense_out"]
    return F.layer_norm(attn_out + x, (w.hidden,), d["gamma"], d["beta"], 1e-5)


def eager_decode_step(torch, w, d):
    import torch.nn.functional as F
    s = torch.matmul(d["q"], d["k_cache"].transpose(-1, -2)) * w.scale
    s = s + d["key_mask"]
    p = torch.softmax(s, -1, dtype=torch.float).to(d["q"].dtype)
    ctx = torch.matmul(p, d["v_cache_clean"])
    ctx = ctx.permute(0, 2, 1, 3).reshape(1, w.batch, w.heads * w.head_dim)
    return F.layer_norm(d["dense_out"] + d["residual"], (w.hidden,), d["gamma"], d["beta"], 1e-5), ctx


def add_eager_aux(torch, w, d, device):
    lens = d["lens_list"]
    B, S = w.batch, w.seq
    pos = torch.arange(S, device=device)
    lens_t = torch.tensor(lens, device=device)
    key_ok = pos.view(1, S) < lens_t.view(B, 1)
    d["key_mask"] = ((~key_ok).to(w.dtype) * -10000.0).view(B, 1, 1, S)
    if not w.decode:
        rows = torch.cat([torch.arange(n, device=device) + b * S for b, n in enumerate(lens)])
        d["valid_rows"] = rows
        d["tri"] = torch.tril(torch.ones(S, S, dtype=torch.bool, device=device)).view(1, 1, S, S)
        d["neg"] = torch.tensor(-1e4, dtype=w.dtype, device=device)
    else:
        d["v_cache_clean"] = d["v_cache"]


# ---------------------------------------------------------------------------
# whole transformer block (projections and MLP included): Block1D of this package on packed
# tokens against the reference block's forward (energonai/model/endecoder.py:48-70,
# attention.py:56-136 without the past cache) written with stock torch ops on the padded batch
# ---------------------------------------------------------------------------
def eager_block_forward(torch, blk, x, mask, heads, causal_tri, neg):
    import torch.nn.functional as F
    B, S, hid = x.shape
    D = hid // heads
    n1, n2, at, mlp = blk.norm1, blk.norm2, blk.attn, blk.mlp
    h = F.layer_norm(x, (hid,), n1.weight, n1.bias, n1.eps)
    k, v, q = torch.chunk(at.query_key_value(h), 3, dim=-1)
    sp = lambda t: t.reshape(B, S, heads, D).permute(0, 2, 1, 3)
    q, k, v = sp(q) * (D ** -0.5), sp(k), sp(v)
    sc = torch.where(causal_tri, torch.matmul(q, k.transpose(-1, -2)), neg) + mask
    pr = torch.softmax(sc, -1, dtype=torch.float).to(x.dtype)
    ctx = torch.matmul(pr, v).transpose(1, 2).reshape(B, S, hid)
    s1 = x + at.dense(ctx)
    h2 = F.layer_norm(s1, (hid,), n2.weight, n2.bias, n2.eps)
    return s1 + mlp.dense_2(mlp.activation(mlp.dense_1(h2)))


def run_block(torch, w, steps, warmup):
    """Prefill of one pre-LN OPT decoder block (ReLU MLP) at the workload's shape (left-padded batch in, padded batch out)."""
    from energonai_amd import workloads
    from energonai_amd.model import Block1D, set_gemm_tuning
    from energonai_amd.seqinfo import seq_info
    dev = torch.device("cuda")
    B, S, hid, H = w.batch, w.seq, w.heads * w.head_dim, w.heads
    lens = workloads.make_lens(w)
    ll = [int(v) for v in lens]
    g = torch.Generator().manual_seed(3000 + w.index)
    import torch.nn.functional as F
    blk = Block1D(hid, H, 4.0, activation=F.relu, dtype=w.dtype, max_seq_len=S, disable_past_cache=True).to(dev)   # OPT: ReLU
    with torch.no_grad():
        for name, prm in blk.named_parameters():
            if prm.dim() == 2:
                prm.copy_((0.02 * torch.randn(prm.shape, generator=g)).to(w.dtype))
    x = torch.randn(B, S, hid, generator=g).to(w.dtype)
    valid = torch.zeros(B, S)
    for b, n in enumerate(ll):
        valid[b, S - n:] = 1
    x = (x * valid.unsqueeze(-1).to(w.dtype)).to(dev)
    mask = ((1.0 - valid) * -10000.0).to(w.dtype).view(B, 1, 1, S).to(dev)
    tri = torch.tril(torch.ones(S, S, dtype=torch.bool, device=dev)).view(1, 1, S, S)
    neg = torch.tensor(-1e4, dtype=w.dtype, device=dev)
    info = seq_info(lens.to(dev), B, dev)
    tokens = info.total
    with torch.no_grad():
        ours = lambda: blk(x, seq_lens=info)
        ref = lambda: eager_block_forward(torch, blk, x, mask, H, tri, neg)
        a, b_ = ours(), ref()
        rows = valid.bool().to(dev)
        err = (a[rows].float() - b_[rows].float()).abs().max().item()
        for _ in range(warmup):
            ours()
        torch.cuda.synchronize()
        ms = _event_time_ms(ours, steps, torch)
        # the same block with every projection on the fastest hipBLASLt candidate for its shape
        set_gemm_tuning(True)
        try:
            c = ours()
            err_tuned = (c[rows].float() - b_[rows].float()).abs().max().item()
            for _ in range(max(2, warmup // 2)):
                ours()
            torch.cuda.synchronize()
            ms_tuned = _event_time_ms(ours, steps, torch)
        finally:
            set_gemm_tuning(False)
        for _ in range(max(2, warmup // 2)):
            ref()
        torch.cuda.synchronize()
        ms_ref = _median_step_ms(ref, max(5, steps // 2), torch)
    del blk
    torch.cuda.empty_cache()
    return {"shape": f"{w.name}: hidden {hid}, {H} heads, batch {B}, bucket {S}, {tokens} valid tokens, left-padded",
            "ms_per_block": ms, "tokens_per_s": tokens / (ms * 1e-3), "ms_per_block_tuned_gemms": ms_tuned,
            "eager_padded_ms_per_block": ms_ref, "speedup_vs_eager_padded": ms_ref / ms,
            "max_abs_diff_vs_eager_on_valid_rows": err, "max_abs_diff_vs_eager_tuned_gemms": err_tuned}


def run_block_decode(torch, w, steps, warmup):
    """Incremental decode of one pre-LN OPT block at the decode workload's shape: prefill a left-padded batch
    with first_cache=True, then time single-token steps.  Baseline: the same block with stock torch ops and a
    padded [B,H,Smax,D] K/V cache (scatter of the new row, masked single-query attention over the whole cache)."""
    import torch.nn.functional as F
    from energonai_amd import workloads
    from energonai_amd.model import Block1D, set_gemm_tuning
    dev = torch.device("cuda")
    B, hid, H, D = w.batch, w.heads * w.head_dim, w.heads, w.head_dim
    lens = workloads.make_lens(w)
    S = int(lens.max())
    total = warmup + 2 * steps + 6                # decode steps taken below: warm-up, timed, tuned
    smax = w.seq + max(64, total + 2)
    g = torch.Generator().manual_seed(4000 + w.index)
    blk = Block1D(hid, H, 4.0, activation=F.relu, dtype=w.dtype, max_seq_len=smax).to(dev)
    with torch.no_grad():
        for name, prm in blk.named_parameters():
            if prm.dim() == 2:
                prm.copy_((0.02 * torch.randn(prm.shape, generator=g)).to(w.dtype))
        buf = torch.zeros(B, S + total, hid, dtype=w.dtype, device=dev)      # the padded batch, one column per step
        valid = (torch.arange(S).view(1, S) >= (S - lens.view(B, 1))).to(dev)
        buf[:, :S] = torch.randn(B, S, hid, device=dev, dtype=w.dtype) * valid.unsqueeze(-1)
        buf[:, S:] = torch.randn(B, total, hid, device=dev, dtype=w.dtype)
        lens_dev = lens.to(dev)
        blk(buf[:, :S], seq_lens=lens_dev, first_cache=True)
        torch.cuda.synchronize()
        pos = [S]

        def ours():
            pos[0] += 1
            return blk(buf[:, :pos[0]], first_cache=False)
        for _ in range(warmup):
            ours()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            ours()
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / steps

        # the same steps with every projection on the fastest hipBLASLt candidate for its (skinny) shape
        set_gemm_tuning(True)
        try:
            for _ in range(2):
                ours()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(steps):
                ours()
            torch.cuda.synchronize()
            ms_tuned = (time.perf_counter() - t0) * 1e3 / steps
        finally:
            set_gemm_tuning(False)

        # baseline: padded cache [B,H,smax,D], positions as in the left-padded batch
        at, mlp, n1, n2 = blk.attn, blk.mlp, blk.norm1, blk.norm2
        kc = torch.randn(B, H, smax, D, device=dev, dtype=w.dtype)
        vc = torch.randn(B, H, smax, D, device=dev, dtype=w.dtype)
        cur = [S]
        key_pos = torch.arange(smax, device=dev).view(1, 1, 1, smax)
        first = (S - lens_dev).view(B, 1, 1, 1)

        def ref():
            x = buf[:, cur[0]:cur[0] + 1]
            h = F.layer_norm(x, (hid,), n1.weight, n1.bias, n1.eps)
            k, v, q = torch.chunk(at.query_key_value(h), 3, dim=-1)
            kc[:, :, cur[0]] = k.view(B, H, D)
            vc[:, :, cur[0]] = v.view(B, H, D)
            cur[0] += 1
            mask = ((key_pos >= first) & (key_pos < cur[0])).to(w.dtype)
            sc = torch.matmul(q.view(B, H, 1, D) * (D ** -0.5), kc.transpose(-1, -2)) + (1.0 - mask) * -10000.0
            pr = torch.softmax(sc, -1, dtype=torch.float).to(w.dtype)
            ctx = torch.matmul(pr, vc).transpose(1, 2).reshape(B, 1, hid)
            s1 = x + at.dense(ctx)
            h2 = F.layer_norm(s1, (hid,), n2.weight, n2.bias, n2.eps)
            return s1 + mlp.dense_2(F.relu(mlp.dense_1(h2)))
        for _ in range(max(2, warmup // 2)):
            ref()
        torch.cuda.synchronize()
        n_ref = max(5, steps // 2)
        t0 = time.perf_counter()
        for _ in range(n_ref):
            ref()
        torch.cuda.synchronize()
        ms_ref = (time.perf_counter() - t0) * 1e3 / n_ref
    del blk, buf, kc, vc
    torch.cuda.empty_cache()
    return {"shape": f"{w.name}: hidden {hid}, {H} heads, batch {B}, cached lengths {int(lens.min())}..{S}, one new token each",
            "ms_per_step": ms, "tokens_per_s": B / (ms * 1e-3), "ms_per_step_tuned_gemms": ms_tuned,
            "eager_padded_cache_ms_per_step": ms_ref,
            "speedup_vs_eager_padded_cache": ms_ref / ms}


# ---------------------------------------------------------------------------
# one workload on the GPU
# ---------------------------------------------------------------------------
def run_workload(torch, w, steps, warmup, want_eager=True, want_kernels=True, step_only=False, form="default"):
    from energonai_amd import kernel as K
    from energonai_amd import layer, workloads
    from energonai_amd.seqinfo import seq_info
    dev = torch.device("cuda", 0)
    res = {"title": w.title, "dtype": DTYPE_NAME[str(w.dtype)]}
    if w.decode:
        d = workloads.make_decode_inputs(w, device=dev, cache_on_device=True)
        info = seq_info(d["lens"], w.batch, dev)
        tokens = w.batch
        res["step_form"] = "single_pass"       # decode_attn (QK^T, softmax, PV in one pass over the caches) + LayerNorm

        def step():
            return layer.decode_layer(d["q"], d["k_cache"], d["v_cache"], info, d["residual"], d["gamma"], d["beta"],
                                      workloads.EPS, w.scale, dense_out=d["dense_out"])
    else:
        d = workloads.make_inputs(w, device=dev)
        info = seq_info(d["lens"], w.batch, dev)
        tokens = d["total"]
        three = layer.three_kernel_form(w.causal, w.dtype, w.seq)
        # "default": whatever padding_removal_layer runs when the caller names no form (the product's own choice);
        # "three_kernel": QK^T, softmax and PV as separate kernels on packed operands (for profiles of those kernels)
        step_form_name = layer.default_attention_form(w.causal, w.dtype, w.seq, w.head_dim, w.scale) \
            if form == "default" else three
        res["step_form"] = step_form_name

        def step():
            return layer.padding_removal_layer(d["hidden_padded"], d["qkv_packed"], info, w.heads, w.head_dim,
                                               d["gamma"], d["beta"], workloads.EPS, w.scale, w.causal,
                                               w.left_padded, dense_out=d["dense_out"], sum_seq=tokens,
                                               fused_attention=None if form == "default" else three)
    res["tokens"] = tokens
    if not w.decode and not step_only:
        # what is built once per batch outside the timed step and reused by every layer: prefix sum, row offsets of
        # the folded depad, workgroup order of the attention kernels (one small kernel each)
        from energonai_amd import _lib
        stream = _lib.stream_of(info.lens)
        tab = torch.empty_like(info.tile_table(w.heads, w.seq))
        offs = torch.empty_like(info.row_offsets(w.seq, w.left_padded))
        cu = torch.empty_like(info.cu_seqlens)
        per_batch = {
            "prefix_sum": lambda: _lib.check(_lib.fn.en_prefix_sum(info.lens.data_ptr(), 0, w.batch, cu.data_ptr(), None, stream), "prefix_sum"),
            "padding_offsets": lambda: _lib.check(_lib.fn.en_padding_offsets(info.lens.data_ptr(), w.batch, w.seq, int(w.left_padded),
                                                                            offs.data_ptr(), stream), "padding_offsets"),
            "attn_tile_table": lambda: _lib.check(_lib.fn.en_attn_tile_table(info.lens.data_ptr(), w.batch, w.heads, w.seq, 0, 128,
                                                                            tab.data_ptr(), stream), "attn_tile_table"),
        }
        res["per_batch_setup_us"] = {}
        for name, fn in per_batch.items():
            for _ in range(3):
                fn()
            torch.cuda.synchronize()
            res["per_batch_setup_us"][name] = _event_time_ms(fn, 20, torch) * 1e3
    # the GPU raises its clocks only after some tens of milliseconds of load (measured: 332 us/step after 10 steps,
    # 295 us after 100, 294 us after 1000): the step is run untimed for PREHEAT_S first, then the W warm-up steps
    t_heat = time.perf_counter()
    while time.perf_counter() - t_heat < PREHEAT_S:
        for _ in range(10):
            step()
        torch.cuda.synchronize()
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    res["ms_per_step"] = wall_ms
    res["tokens_per_s"] = tokens / (wall_ms * 1e-3)

    # the same step as an unchanged caller of the reference API issues it (examples/bert/bert.py:100-132): seven
    # Python calls with the reference's semantics -- transpose_pad writes zeros into the padding rows, the
    # softmax zeroes the whole tail of every row -- next to the one-call form above
    if not w.decode and not step_only:
        def step_api():
            T = tokens
            x = K.depad(d["hidden_padded"], w.batch, info, left_padded=w.left_padded, sum_seq=T)
            qkv = K.transpose_pad(d["qkv_packed"], w.batch, w.seq, info, w.heads, 3 * w.head_dim)
            q, k, v = torch.chunk(qkv, 3, dim=-1)
            scores = K.attn_qk(q, k, info, causal=w.causal)
            probs = K.scale_mask_softmax(w.batch, w.seq, w.heads, scores, info, scale=w.scale, causal=w.causal)
            ctx = K.attn_pv(probs, v, info, causal=w.causal)
            ctx_packed = K.transpose_depad(ctx, w.batch, T, w.seq, info, w.heads, w.head_dim)
            attn_out = ctx_packed.view(1, T, w.heads * w.head_dim) if d["dense_out"] is None else d["dense_out"]
            return K.layer_norm_forward(attn_out, d["gamma"], d["beta"], (w.hidden,), workloads.EPS, residual=x)
        for _ in range(max(2, warmup // 2)):
            step_api()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            step_api()
        torch.cuda.synchronize()
        res["api_sequence_ms_per_step"] = (time.perf_counter() - t0) * 1e3 / steps

    # other forms of the same step through the one-call entry point, for comparison; never the headline:
    #   reference_ops_one_call   the seven ops of the reference's sequence (padded tensors, both transposes, depad)
    #   three_kernel             QK^T, softmax, PV as three kernels on packed operands, depad folded into the LayerNorm
    #                            (the default where the fused kernel does not apply), scores in the layout
    #                            layer.three_kernel_form picks; three_kernel_other_scores: the other score layout
    #   fused_attention ...      QK^T + softmax + PV in one kernel: on the padded buffer, on the packed projections,
    #                            and with depad folded into the LayerNorm as well (the default where it applies)
    if not w.decode and not step_only:
        forms = [("reference_ops_one_call_ms_per_step", False, False), ("three_kernel_ms_per_step", three, True)]
        if w.dtype != torch.float32:
            if w.causal:
                forms += [("three_kernel_other_scores_ms_per_step",
                           "varlen" if three == "varlen_packed" else "varlen_packed", True)]
            forms += [("fused_attention_ms_per_step", True, False),
                      ("packed_fused_attention_ms_per_step", "packed", False),
                      ("packed_fused_folded_depad_ms_per_step", "packed", True)]
        for key, fform, fold in forms:
            def step_form():
                return layer.padding_removal_layer(d["hidden_padded"], d["qkv_packed"], info, w.heads, w.head_dim,
                                                   d["gamma"], d["beta"], workloads.EPS, w.scale, w.causal,
                                                   w.left_padded, dense_out=d["dense_out"], sum_seq=tokens,
                                                   fused_attention=fform, fold_depad=fold)
            for _ in range(max(2, warmup // 2)):
                step_form()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(steps):
                step_form()
            torch.cuda.synchronize()
            res[key] = (time.perf_counter() - t0) * 1e3 / steps

    # the same step replayed from a HIP graph (launch overhead removed); reported, never the headline
    try:
        if step_only:
            raise RuntimeError("skipped (--step-only)")
        g = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step()
            with torch.cuda.graph(g, stream=side):
                step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        for _ in range(3):
            g.replay()
        res["graph_ms_per_step"] = _event_time_ms(g.replay, steps, torch)
        del g
    except Exception as exc:  # graph capture is a convenience measurement only
        res["graph_ms_per_step"] = None
        res["graph_error"] = str(exc)[:200]
    torch.cuda.synchronize()

    if want_kernels:
        res["step_kernels"], res["three_kernel_step_kernels"], res["kernels"] = kernel_table(
            torch, K, layer, workloads, w, d, info, steps, step_only, res.get("step_form"))
    if want_eager:
        add_eager_aux(torch, w, d, dev)
        fn = (lambda: eager_decode_step(torch, w, d)) if w.decode else (lambda: eager_prefill_step(torch, w, d))
        try:
            for _ in range(min(warmup, 10)):
                fn()
            torch.cuda.synchronize()
            ms = _median_step_ms(fn, max(5, min(steps, 50)), torch)
            res["eager_gpu_ms_per_step"] = ms
            res["speedup_vs_eager_gpu"] = ms / wall_ms
        except Exception as exc:
            res["eager_gpu_ms_per_step"] = None
            res["eager_error"] = str(exc)[:200]
    del d
    torch.cuda.empty_cache()
    return res


def kernel_table(torch, K, layer, workloads, w, d, info, steps, step_only=False, step_form=None):
    """Launch-to-launch time of every kernel on its real operands -> GB/s, TFLOP/s, fraction of peak.

    Three tables: `step` holds the kernels the timed step launches, in its form (prefill default: fused attention
    on the packed projections, LayerNorm taking its residual rows from the padded activations); `three` holds the
    kernels of the three-kernel form of the step (QK^T and PV on the packed projections with row offsets, scores in
    the packed causal layout where that applies, the same LayerNorm) -- it is the `step` table when that form is
    the one timed, and is left out of a --step-only run otherwise; `api` holds every op of the reference's sequence
    in the form its public function launches it (padded [B,H,S,*] tensors, zero-filled padding, whole-row softmax
    tails).
    """
    dt = DTYPE_NAME[str(w.dtype)]
    es = torch.empty(0, dtype=w.dtype).element_size()
    alg = workloads.algorithmic_bytes(w, d["lens_list"])
    flops = workloads.algorithmic_flops(w, d["lens_list"])
    H, D, S, B = w.heads, w.head_dim, w.seq, w.batch
    api, step, three = {}, {}, {}
    if w.decode:
        # the step: one pass over the caches (QK^T, softmax and PV in one kernel), then the LayerNorm; the three
        # separate decode ops stay public and are timed in the `kernels` table
        ctx = torch.empty((B, H, 1, D), dtype=w.dtype, device=d["q"].device)
        step["decode_attn"] = lambda: K.decode_attn(d["q"], d["k_cache"], d["v_cache"], info, scale=w.scale, out=ctx)
        step["layernorm_residual"] = lambda: K.layer_norm_forward(d["dense_out"], d["gamma"], d["beta"], (w.hidden,),
                                                                  workloads.EPS, residual=d["residual"])
        if not step_only:
            ones = layer._ones_info(B, d["q"].device)
            keep = layer.decode_layer(d["q"], d["k_cache"], d["v_cache"], info, d["residual"], d["gamma"], d["beta"],
                                      workloads.EPS, w.scale, dense_out=d["dense_out"], keep=True, single_pass=False)
            scores = torch.empty((B, H, 1, S), dtype=w.dtype, device=d["q"].device)
            probs = keep["scores_probs"]
            api["decode_qk"] = lambda: K.decode_qk(d["q"], d["k_cache"], info, out=scores)
            api["scale_mask_softmax"] = lambda: K.scale_mask_softmax(B, 1, H, probs, info, scale=w.scale, k_seq_len=S,
                                                                     q_len_list=ones)
            api["decode_pv"] = lambda: K.decode_pv(probs, d["v_cache"], info, out=ctx)
            # the single pass over the same cache contents kept in pages of 64 positions, page ids shuffled over a pool
            P = 64
            pages = B * (S // P)
            perm = torch.randperm(pages, device=d["q"].device)
            table = perm.view(B, S // P).to(torch.int32).contiguous()

            def paged(cache):
                pool = torch.empty((pages, H, P, D), dtype=w.dtype, device=cache.device)
                pool[perm] = cache.view(B, H, S // P, P, D).permute(0, 2, 1, 3, 4).reshape(pages, H, P, D)
                return pool
            k_pool, v_pool = paged(d["k_cache"]), paged(d["v_cache"])
            ctx_paged = K.decode_attn_paged(d["q"], k_pool, v_pool, info, table, scale=w.scale)
            if not torch.equal(ctx_paged, K.decode_attn(d["q"], d["k_cache"], d["v_cache"], info, scale=w.scale)):
                raise RuntimeError("decode_attn_paged and decode_attn disagree on the same cache contents")
            api["decode_attn_paged"] = lambda: K.decode_attn_paged(d["q"], k_pool, v_pool, info, table, scale=w.scale,
                                                                   out=ctx_paged)
            alg["decode_attn_paged"] = alg["decode_attn"]
    else:
        T = d["total"]
        # ---- the kernels of the three-kernel form
        packed_scores = layer.three_kernel_form(w.causal, w.dtype, S) == "varlen_packed"
        qv, kv, vv = torch.chunk(d["qkv_packed"].view(T, H, 3 * D), 3, dim=-1)
        ctx_step = torch.empty((1, T, H, D), dtype=w.dtype, device="cuda")
        offs = info.row_offsets(S, w.left_padded)
        attn_out_step = ctx_step.view(1, T, H * D) if d["dense_out"] is None else d["dense_out"]
        fused_step = step_form == "packed"
        if not (step_only and fused_step):
            n_scores = K.packed_scores_elems(B, H, S, w.dtype) if packed_scores else B * H * S * S
            s_step = torch.empty(n_scores, dtype=w.dtype, device="cuda")
            three["attn_qk"] = lambda: K.attn_qk_varlen(qv, kv, B, S, info, causal=w.causal, packed_scores=packed_scores,
                                                        out=s_step)
            if packed_scores:
                three["scale_mask_softmax"] = lambda: K.scale_mask_softmax_packed(B, S, H, s_step, info, scale=w.scale)
            else:
                three["scale_mask_softmax"] = lambda: K.scale_mask_softmax(B, S, H, s_step.view(B, H, S, S), info,
                                                                           scale=w.scale, causal=w.causal,
                                                                           tail_rows=layer.SOFTMAX_TAIL_ROWS)
            three["attn_pv"] = lambda: K.attn_pv_varlen(s_step, vv, B, S, info, causal=w.causal,
                                                        packed_scores=packed_scores, out=ctx_step)
        ln_step = lambda: K.layer_norm_forward(attn_out_step, d["gamma"], d["beta"], (w.hidden,), workloads.EPS,
                                               residual=d["hidden_padded"], residual_row_offsets=offs)
        alg["scale_mask_softmax"] = alg.pop("scale_mask_softmax")       # keep the key order readable
        step_alg = dict(attn_qk=alg["attn_qk"], scale_mask_softmax=alg["scale_mask_softmax_no_tail"],
                        attn_pv=alg["attn_pv"], layernorm_residual=alg["layernorm_residual"],
                        attn_fused_packed=4 * T * H * D * es)   # q, k, v in; ctx out
        if fused_step:
            # ---- the kernels of the default form: fused attention on the packed projections, then the LayerNorm
            step["attn_fused_packed"] = lambda: K.attn_fused_packed(d["qkv_packed"], B, S, info, H, D, scale=w.scale,
                                                                    causal=w.causal, out=ctx_step)
            step["layernorm_residual"] = ln_step
            if three:
                three["layernorm_residual"] = ln_step
        else:
            three["layernorm_residual"] = ln_step
            step, three = three, {}
        if not step_only:
            # ---- the reference's sequence of ops, each as its public function launches it
            keep = layer.padding_removal_layer(d["hidden_padded"], d["qkv_packed"], info, H, D, d["gamma"], d["beta"],
                                               workloads.EPS, w.scale, w.causal, w.left_padded,
                                               dense_out=d["dense_out"], sum_seq=T, keep=True)
            q, k, v = torch.chunk(keep["qkv"], 3, dim=-1)
            scores = keep["probs"]
            ctx = keep["ctx"]
            attn_out = keep["ctx_packed"].view(1, T, H * D) if d["dense_out"] is None else d["dense_out"]
            api["depad"] = lambda: K.depad(d["hidden_padded"], B, info, left_padded=w.left_padded, sum_seq=T)
            api["transpose_pad"] = lambda: K.transpose_pad(d["qkv_packed"], B, S, info, H, 3 * D)
            # without the zero fill of the padding rows (readers bounded by the lengths need none)
            alg["transpose_pad_valid_rows"] = 2 * T * H * 3 * D * es
            api["transpose_pad_valid_rows"] = lambda: K.transpose_pad(d["qkv_packed"], B, S, info, H, 3 * D,
                                                                      zero_padding=False)
            api["attn_qk"] = lambda: K.attn_qk(q, k, info, causal=w.causal, out=scores)
            api["scale_mask_softmax"] = lambda: K.scale_mask_softmax(B, S, H, scores, info, scale=w.scale,
                                                                     causal=w.causal)
            api["scale_mask_softmax_no_tail"] = lambda: K.scale_mask_softmax(B, S, H, scores, info, scale=w.scale,
                                                                           causal=w.causal,
                                                                           tail_rows=layer.SOFTMAX_TAIL_ROWS)
            api["attn_pv"] = lambda: K.attn_pv(scores, v, info, causal=w.causal, out=ctx)
            if w.dtype != torch.float32:
                alg["attn_fused"] = 4 * T * H * D * es   # q, k, v in; ctx out
                api["attn_fused"] = lambda: K.attn_fused(q, k, v, info, scale=w.scale, causal=w.causal, out=ctx)
                alg["attn_fused_packed"] = alg["attn_fused"]
                ctx_pk = torch.empty(1, T, H * D, dtype=w.dtype, device="cuda")
                api["attn_fused_packed"] = lambda: K.attn_fused_packed(d["qkv_packed"], B, S, info, H, D,
                                                                       scale=w.scale, causal=w.causal, out=ctx_pk)
                if D > 64:
                    # the same op with 64 queries per wave (256-row tiles): built, measured, not what the step runs
                    alg["attn_fused_packed_wide"] = alg["attn_fused"]
                    api["attn_fused_packed_wide"] = lambda: K.attn_fused_packed(d["qkv_packed"], B, S, info, H, D,
                                                                                scale=w.scale, causal=w.causal, out=ctx_pk,
                                                                                query_tile=256)
            api["transpose_depad"] = lambda: K.transpose_depad(ctx, B, T, S, info, H, D)
            api["layernorm_residual"] = lambda: K.layer_norm_forward(attn_out, d["gamma"], d["beta"], (w.hidden,),
                                                                     workloads.EPS, residual=keep["x"])

    yard = {} if step_only else workload_yardsticks(torch, w, d, info,
                                                    (not w.decode) and layer.three_kernel_form(w.causal, w.dtype, S) == "varlen_packed")

    def measure(fns, bytes_of, layout="padded"):
        table = {}
        for name, fn in fns.items():
            _preheat(torch, fn)       # each row at the settled clock, like the timed steps themselves
            ms = _event_time_ms(fn, steps, torch)
            row = {"us": ms * 1e3, "alg_MB": bytes_of[name] / 1e6, "GBps": bytes_of[name] / (ms * 1e-3) / 1e9}
            row["hbm_frac"] = row["GBps"] / HBM_PEAK_GBS
            if name in ("attn_qk", "attn_pv", "decode_qk", "decode_pv", "decode_attn", "decode_attn_paged", "attn_fused",
                        "attn_fused_packed", "attn_fused_packed_wide"):
                row["TFLOPs"] = (2 if name.startswith("attn_fused") or name.startswith("decode_attn") else 1) * flops / (ms * 1e-3) / 1e12
                row["mfma_frac"] = row["TFLOPs"] / MFMA_PEAK_TFLOPS[dt]
            # what a kernel that only moves the bytes reaches in this kernel's access pattern, and this kernel's share of it
            key = YARDSTICK_OF.get(name)
            if key is not None and key.startswith("prefix_"):
                key = f"{key}_{layout}"
            if key in yard:
                row["yardstick_GBps"] = yard[key]
                row["yardstick_pattern"] = key
                row["frac_of_yardstick"] = row["GBps"] / yard[key]
            # PV: also against the same bytes read tile by tile along the keys, its own walk, three workgroups per CU
            walk = f"prefix_read_tile_walk_3_per_cu_{layout}"
            if name == "attn_pv" and walk in yard:
                row["tile_walk_yardstick_GBps"] = yard[walk]
                row["frac_of_tile_walk_yardstick"] = row["GBps"] / yard[walk]
            table[name] = row
        return table
    step_layout = "packed" if ("prefix_read_packed" in yard) else "padded"
    step_table = measure(step, alg if w.decode else step_alg, step_layout)
    three_table = measure(three, alg if w.decode else step_alg, step_layout)
    api_table = measure(api, alg, "padded")
    return step_table, three_table, api_table


# ---------------------------------------------------------------------------
# CPU baseline: the oracle on this box's host cores, bounded sample
# ---------------------------------------------------------------------------
def host_cpu():
    """(threads the process may use, os.cpu_count(), CPU model).  A one-GPU box exports OMP_NUM_THREADS for its
    share of the host's cores; that is what the baseline runs on, and the machine's full count is printed beside it."""
    total = os.cpu_count() or 1
    granted = total
    try:
        granted = max(1, min(total, int(os.environ.get("OMP_NUM_THREADS", total))))
    except ValueError:
        pass
    model = "unknown"
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    return granted, total, model


def cpu_baseline(torch, w, full_batch, passes=3):
    """The oracle's layer (a torch-eager restatement of the reference path) in fp32 on the host cores: the whole
    batch for the fp32 workload, for the small fp16 one and for the headline workload, the first sequences of
    the others; one warm-up pass, then the median of `passes` timed ones."""
    from energonai_amd import workloads
    from oracle import eager
    threads, total, model = host_cpu()
    torch.set_num_threads(threads)
    if w.decode:
        nb = w.batch if full_batch else 8
        lens = workloads.make_lens(w)[:nb]
        sub = workloads.Workload(w.index, w.name, w.title, torch.float32, nb, w.seq, w.heads, w.head_dim, w.hidden,
                                 w.len_lo, w.len_hi, w.causal, w.left_padded, decode=True)
        d = workloads.make_decode_inputs(sub, dtype=torch.float32, lens=lens)
        tokens = nb

        def step():
            eager.decode_attention(d["q"], d["k_cache"], d["v_cache"], d["lens_list"], w.scale)
            eager.layer_norm(d["dense_out"], d["gamma"], d["beta"], workloads.EPS, residual=d["residual"])
    else:
        nb = w.batch if (full_batch or w.name in ("c1", "c2")) else 4
        lens = workloads.make_lens(w)[:nb]
        sub = workloads.Workload(w.index, w.name, w.title, torch.float32, nb, w.seq, w.heads, w.head_dim, w.hidden,
                                 w.len_lo, w.len_hi, w.causal, w.left_padded)
        d = workloads.make_inputs(sub, dtype=torch.float32, lens=lens)
        tokens = d["total"]

        def step():
            eager.layer_unpadded(d["hidden_padded"], d["qkv_packed"], d["lens_list"], w.heads, w.head_dim, d["gamma"],
                                 d["beta"], workloads.EPS, w.scale, w.causal, w.left_padded,
                                 dense_out=d["dense_out"])
    which = "all" if nb == w.batch else f"the first {nb} of the"
    unit = "sequences (one new token each)" if w.decode else f"sequences ({tokens} tokens)"
    step()  # warm-up (first touch of the fp32 score tensors)
    times = []
    for _ in range(passes):
        t0 = time.perf_counter()
        step()
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    return {"value": tokens / med, "unit": "tokens/s", "cores": threads, "kind": "port",
            "host_cpu_count": total, "cpu_model": model,
            "sample": f"{w.name}: {which} {w.batch} {unit}, fp32 on the CPU"
                      f"{'' if w.dtype == torch.float32 else ' (the GPU path stores ' + DTYPE_NAME[str(w.dtype)] + ')'}; "
                      f"median of {len(times)} passes after one warm-up, {med * 1e3:.1f} ms each; "
                      f"{threads} threads on a host of {total} ({model}); "
                      f"oracle.eager.layer_unpadded, the torch-eager restatement of the reference path"}


def copy_yardstick(torch, iters):
    """en_copy_bytes at 64 MiB, 256 MiB and 1 GiB (read n + write n bytes per launch); with it the stream and
    causal-prefix yardsticks (see stream_yardsticks)."""
    from energonai_amd import _lib
    out = {"kernel": "copy_kernel", "unit": "GB/s", "sizes": {}}
    stream = torch.cuda.current_stream().cuda_stream
    for mib in (64, 256, 1024):
        n = mib << 20
        a = torch.empty(n, dtype=torch.uint8, device="cuda")
        b = torch.empty_like(a)
        a.fill_(1)
        fn = lambda: _lib.check(_lib.fn.en_copy_bytes(a.data_ptr(), b.data_ptr(), n, stream), "copy")
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        ms = _event_time_ms(fn, max(5, iters), torch)
        out["sizes"][f"{mib}MiB"] = {"bytes_read": n, "bytes_written": n, "us": ms * 1e3, "GBps": 2 * n / (ms * 1e-3) / 1e9}
        del a, b
    return out


def decode_sizes(torch, iters):
    """The single-pass decode attention at batch sizes from one sequence up (72 heads of 128 channels, fp16, every
    cache full): one workgroup per (batch, head) unit, the keys of a unit shared between workgroups (what the call
    does for fewer than 512 units), and the same cache contents in pages of 64 positions shuffled over a pool."""
    from energonai_amd import kernel as K
    from energonai_amd.seqinfo import seq_info
    H, D, P = 72, 128, 64
    rows = []
    for B in (1, 2, 4, 8, 16, 64):
        for S in (2048, 8192):
            if 2 * B * H * S * D * 2 > 6e9:
                continue
            dev = torch.device("cuda")
            q = torch.randn(B, H, 1, D, device=dev, dtype=torch.float16)
            kc = torch.randn(B, H, S, D, device=dev, dtype=torch.float16)
            vc = torch.randn_like(kc)
            info = seq_info(torch.full((B,), S, dtype=torch.int32, device=dev), B, dev)
            out = torch.empty(B, H, 1, D, device=dev, dtype=torch.float16)
            pages = B * (S // P)
            perm = torch.randperm(pages, device=dev)
            table = perm.view(B, S // P).to(torch.int32).contiguous()
            k_pool = torch.empty((pages, H, P, D), dtype=kc.dtype, device=dev)
            v_pool = torch.empty_like(k_pool)
            k_pool[perm] = kc.view(B, H, S // P, P, D).permute(0, 2, 1, 3, 4).reshape(pages, H, P, D)
            v_pool[perm] = vc.view(B, H, S // P, P, D).permute(0, 2, 1, 3, 4).reshape(pages, H, P, D)
            need = K.decode_attn_workspace_bytes(B, H, S, D)
            ws = torch.empty(max(need, 16), dtype=torch.uint8, device=dev)
            fns = {"one_workgroup_per_unit": lambda: K.decode_attn(q, kc, vc, info, out=out, split=False),
                   "as_called": lambda: K.decode_attn(q, kc, vc, info, out=out, workspace=ws),
                   "paged": lambda: K.decode_attn_paged(q, k_pool, v_pool, info, table, out=out, workspace=ws)}
            nbytes = 2 * B * H * S * D * 2
            row = {"batch": B, "cached_positions": S, "units": B * H, "cache_MB": nbytes / 1e6,
                   "shares_per_unit": (need // (B * H * (D + 2) * 4)) if need else 1}
            for name, fn in fns.items():
                _preheat(torch, fn)
                us = _event_time_ms(fn, max(10, iters), torch) * 1e3
                row[name] = {"us": us, "GBps": nbytes / us / 1e3}
            rows.append(row)
            del kc, vc, k_pool, v_pool
    return {"heads": H, "size_per_head": D, "page": P, "dtype": "f16", "rows": rows}


STREAM_MODES = {"copy": 0, "read": 1, "write": 2, "inplace": 0}
PREFIX_MODES = {"inplace": 0, "write": 1, "read": 2, "out_of_place": 3,
                # read only, a 128-row tile at a time along the keys in 128- or 256-byte pieces per row (how PV walks its
                # probabilities); "_3_per_cu": with the three workgroups per CU the attention kernels have
                "read_tile_walk": 4, "read_tile_walk_3_per_cu": 5, "read_tile_walk_256B": 6,
                "read_tile_walk_256B_3_per_cu": 7}


def _preheat(torch, fn):
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < PREHEAT_S:
        for _ in range(5):
            fn()
        torch.cuda.synchronize()


def stream_yardstick_GBps(torch, nbytes, mode, nt, iters=10):
    """en_stream_yardstick over one contiguous range: bytes moved per second (a copy moves 2 x nbytes)."""
    from energonai_amd import _lib
    nbytes = max(16, (int(nbytes) // 16) * 16)
    a = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    b = torch.empty(nbytes if mode in ("copy", "write") else 16, dtype=torch.uint8, device="cuda")
    a.fill_(1)
    stream = torch.cuda.current_stream().cuda_stream
    dst = a if mode == "inplace" else b
    fn = lambda: _lib.check(_lib.fn.en_stream_yardstick(a.data_ptr(), dst.data_ptr(), nbytes, STREAM_MODES[mode], int(nt),
                                                        stream), "stream_yardstick")
    _preheat(torch, fn)
    ms = _event_time_ms(fn, iters, torch)
    return (2 if mode in ("copy", "inplace") else 1) * nbytes / (ms * 1e-3) / 1e9


def prefix_yardstick_GBps(torch, lens_dev, lens_list, B, H, S, dtype, packed, mode, nt, iters=10):
    """en_prefix_yardstick over the causal prefixes of a batch's score tensor: bytes of the visible prefixes
    (H x element size x sum n(n+1)/2, once per direction moved) per second."""
    from energonai_amd import _lib
    from energonai_amd.kernel.attention import packed_scores_elems
    es = torch.empty(0, dtype=dtype).element_size()
    n = packed_scores_elems(B, H, S, dtype) if packed else B * H * S * S
    a = torch.zeros(n, dtype=dtype, device="cuda")
    b = torch.zeros(n, dtype=dtype, device="cuda") if mode == "out_of_place" else None
    vis = H * es * sum(m * (m + 1) // 2 for m in lens_list)
    stream = torch.cuda.current_stream().cuda_stream
    fn = lambda: _lib.check(_lib.fn.en_prefix_yardstick(a.data_ptr(), _lib.ptr(b), lens_dev.data_ptr(), B, H, S, int(packed),
                                                        PREFIX_MODES[mode], int(nt), es, stream), "prefix_yardstick")
    _preheat(torch, fn)
    ms = _event_time_ms(fn, iters, torch)
    return (2 if mode in ("inplace", "out_of_place") else 1) * vis / (ms * 1e-3) / 1e9


def stream_yardsticks(torch, iters):
    """Every yardstick at the sizes and sequence lengths of the two large prefill workloads and of the decode
    workload: what a kernel that does nothing but move the bytes reaches in each access pattern."""
    from energonai_amd import workloads
    out = {"unit": "GB/s", "stream": {}, "prefix": {}}
    for mib in (128, 512, 2048):
        row = {}
        for mode in STREAM_MODES:
            for nt in (0, 1):
                row[f"{mode}{'_nt' if nt else ''}"] = stream_yardstick_GBps(torch, mib << 20, mode, nt, iters)
        out["stream"][f"{mib}MiB"] = row
    for name in ("c3", "c4"):
        w = workloads.BY_NAME[name]
        lens = workloads.make_lens(w)
        ll = [int(v) for v in lens]
        lens_dev = lens.to("cuda")
        for packed in (0, 1):
            row = {}
            for mode in PREFIX_MODES:
                for nt in (0, 1):
                    row[f"{mode}{'_nt' if nt else ''}"] = prefix_yardstick_GBps(torch, lens_dev, ll, w.batch, w.heads, w.seq,
                                                                                w.dtype, packed, mode, nt, iters)
            out["prefix"][f"{name}_{'packed' if packed else 'padded'}"] = row
    return out


# which yardstick speaks for which kernel row of the tables (prefix patterns: causal prefill workloads only)
YARDSTICK_OF = {"depad": "copy", "transpose_pad": "copy", "transpose_pad_valid_rows": "copy", "transpose_depad": "copy",
                "layernorm_residual": "copy", "scale_mask_softmax": "prefix_inplace",
                "scale_mask_softmax_no_tail": "prefix_inplace", "attn_qk": "prefix_write", "attn_pv": "prefix_read",
                "decode_qk": "read", "decode_pv": "read", "decode_attn": "read", "decode_attn_paged": "read"}


def workload_yardsticks(torch, w, d, info, packed_scores):
    """The yardsticks of one workload, best of plain and non-temporal accesses: {"copy", "read",
    "prefix_*_packed", "prefix_*_padded"} -> GB/s."""
    es = torch.empty(0, dtype=w.dtype).element_size()
    y = {}
    if w.decode:
        nbytes = w.heads * sum(d["lens_list"]) * w.head_dim * es
        y["read"] = max(stream_yardstick_GBps(torch, nbytes, "read", nt) for nt in (0, 1))
        y["copy"] = max(stream_yardstick_GBps(torch, 64 << 20, "copy", nt) for nt in (0, 1))
        return y
    nbytes = max(d["total"] * w.hidden * es, 1 << 20)
    y["copy"] = max(stream_yardstick_GBps(torch, nbytes, "copy", nt) for nt in (0, 1))
    if w.causal:
        for layout, packed in (("padded", 0), ("packed", 1)):
            if packed and not packed_scores:
                continue
            for mode in ("inplace", "write", "read", "read_tile_walk_3_per_cu"):
                y[f"prefix_{mode}_{layout}"] = max(
                    prefix_yardstick_GBps(torch, info.lens, d["lens_list"], w.batch, w.heads, w.seq, w.dtype, packed, mode, nt)
                    for nt in (0, 1))
    return y


def roofline_of(res, workload_name, form="default"):
    """Roofline object of the kernel that takes the largest share of a workload's step, in the form the step
    launches it: algorithmic bytes (or FLOPs) per launch over the launch-to-launch time measured above.
    Fused attention reads q, k, v and writes ctx (4 T H D e bytes) and does 4 D FLOPs per visible score: which roof
    bounds it follows from its FLOPs per byte against the machine's (peak FLOP/s over peak bytes/s); c3 (short
    sequences, 170 FLOP/B against 312) sits under the HBM roof, c4 (355 FLOP/B) under the matrix roof.  Both
    fractions are in the object whichever one `frac` is.  `traffic` comes from the counter summary under profiles/
    (None when there is none for this workload, or when it was measured on other sources than this library's)."""
    kt = res["step_kernels"]
    dom = max(kt, key=lambda n: kt[n]["us"])
    row = kt[dom]
    by_op, digest = measured_traffic(workload_name, form)
    traffic = by_op.get(dom)
    if "mfma_frac" in row and dom.startswith("attn_fused"):
        peak_tf = MFMA_PEAK_TFLOPS[res["dtype"]]
        flops = row["TFLOPs"] * 1e12 * row["us"] * 1e-6
        intensity = flops / (row["alg_MB"] * 1e6)
        balance = peak_tf * 1e12 / (HBM_PEAK_GBS * 1e9)
        roofline = {"kernel": dom, "traffic": traffic, "us_per_launch": row["us"],
                    "alg_flops_per_launch": flops, "alg_bytes_per_launch": row["alg_MB"] * 1e6,
                    "flops_per_byte": intensity, "machine_flops_per_byte": balance,
                    "hbm_frac": row["hbm_frac"], "mfma_frac": row["mfma_frac"]}
        if intensity < balance:
            roofline.update({"bound": "hbm", "achieved": row["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": row["hbm_frac"]})
        else:
            roofline.update({"bound": "mfma", "achieved": row["TFLOPs"], "peak": peak_tf, "unit": "TFLOP/s", "frac": row["mfma_frac"]})
    else:
        roofline = {"kernel": dom, "bound": "hbm", "achieved": row["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                    "frac": row["GBps"] / HBM_PEAK_GBS, "traffic": traffic, "us_per_launch": row["us"],
                    "alg_bytes_per_launch": row["alg_MB"] * 1e6}
    # the counter summary speaks for the sources it was measured on: say whether those are this library's
    roofline["traffic_measured_on_sources"] = digest
    roofline["traffic_is_of_this_library"] = None if traffic is None else (digest == library_source_hash())
    return roofline


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="c3", choices=["c1", "c2", "c3", "c4", "c5"])
    ap.add_argument("--form", default="default", choices=["default", "three_kernel"],
                    help="the step that is timed: the product's default form, or QK^T / softmax / PV as three kernels")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="only the headline workload, no eager / other workloads")
    ap.add_argument("--step-only", action="store_true",
                    help="with --no-extra: launch nothing but the step and its own kernels (for profiles)")
    ap.add_argument("--copy-yardstick", action="store_true",
                    help="instead of the benchmark, time en_copy_bytes (plain 128-bit copy) at known sizes (used to "
                         "calibrate the FETCH_SIZE / WRITE_SIZE counters) and the stream and causal-prefix yardsticks: "
                         "copy / read only / write only with plain and non-temporal accesses, and in-place, write-only, "
                         "read-only and out-of-place passes over the causal prefixes of the c3 and c4 score tensors in "
                         "the [B,H,S,S] and the packed layout")
    ap.add_argument("--decode-sizes", action="store_true",
                    help="instead of the benchmark, time the single-pass decode attention from one sequence to 64 "
                         "(keys of a unit shared between workgroups or not; contiguous caches and pages)")
    ns = ap.parse_args(argv)
    if ns.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU's share of the path; --gpus must be 1 "
              "(the path shards by head / by sequence with no exchange step, nothing here uses a second GPU)",
              file=sys.stderr)
        return 2

    import torch
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2
    torch.cuda.set_device(0)
    from energonai_amd import build as hip_build
    hip_build.ensure_built()      # loads what is built; compiles only when nothing is
    from energonai_amd import workloads

    if ns.copy_yardstick:
        out = copy_yardstick(torch, ns.steps)
        if not ns.step_only:      # --step-only: the plain copy alone (the counter calibration run of bench_profiles.py)
            out["yardsticks"] = stream_yardsticks(torch, max(5, ns.steps))
        out["library_source_hash"] = library_source_hash()
        print(json.dumps(out))
        return 0

    if ns.decode_sizes:
        out = decode_sizes(torch, ns.steps)
        out["library_source_hash"] = library_source_hash()
        print(json.dumps(out))
        return 0

    w = workloads.BY_NAME[ns.workload]
    torch.cuda.synchronize()
    if ns.step_only:
        ns.no_extra = True
    head = run_workload(torch, w, ns.steps, ns.warmup, want_eager=not ns.no_extra, want_kernels=True,
                        step_only=ns.step_only, form=ns.form)
    torch.cuda.synchronize()

    kt = head["step_kernels"]
    roofline = roofline_of(head, w.name, ns.form)

    out = {
        "metric": "per_layer_tokens_per_s", "value": head["tokens_per_s"], "unit": "tokens/s", "n_gpus": 1,
        "steps": ns.steps, "warmup": ns.warmup, "ms_per_step": head["ms_per_step"], "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": head["dtype"], "data": "synthetic",
        "library_source_hash": library_source_hash(),
        "config": {"workload": f"{w.name}: {w.title}; batch {w.batch}, bucket {w.seq}, {w.heads}x{w.head_dim} heads, "
                               f"LayerNorm width {w.hidden}, {head['tokens']} valid tokens"},
        "roofline": roofline,
        "step_form": head.get("step_form"), "preheat_ms": PREHEAT_S * 1e3,
        "per_batch_setup_us": head.get("per_batch_setup_us"),
        "three_kernel_ms_per_step": head.get("three_kernel_ms_per_step"),
        "three_kernel_other_scores_ms_per_step": head.get("three_kernel_other_scores_ms_per_step"),
        "api_sequence_ms_per_step": head.get("api_sequence_ms_per_step"),
        "reference_ops_one_call_ms_per_step": head.get("reference_ops_one_call_ms_per_step"),
        "graph_ms_per_step": head.get("graph_ms_per_step"),
        "fused_attention_ms_per_step": head.get("fused_attention_ms_per_step"),
        "packed_fused_attention_ms_per_step": head.get("packed_fused_attention_ms_per_step"),
        "packed_fused_folded_depad_ms_per_step": head.get("packed_fused_folded_depad_ms_per_step"),
        "eager_gpu_ms_per_step": head.get("eager_gpu_ms_per_step"),
        "speedup_vs_eager_gpu": head.get("speedup_vs_eager_gpu"),
        "step_kernels": kt,
        "three_kernel_step_kernels": head["three_kernel_step_kernels"],
        "kernels": head["kernels"],
    }
    if not ns.no_extra:
        others = {}
        for ow in workloads.WORKLOADS:
            if ow.name == w.name:
                continue
            try:
                others[ow.name] = run_workload(torch, ow, max(5, ns.steps // 2), max(2, ns.warmup // 2))
                others[ow.name]["roofline"] = roofline_of(others[ow.name], ow.name)
            except Exception as exc:
                others[ow.name] = {"error": str(exc)[:300]}
        out["workloads"] = others
        blocks = {}
        for name in ("c2", "c3"):
            try:
                blocks[name] = run_block(torch, workloads.BY_NAME[name], max(5, ns.steps // 2), max(2, ns.warmup // 2))
            except Exception as exc:
                blocks[name] = {"error": str(exc)[:300]}
        out["model_block_prefill"] = blocks
        try:
            out["model_block_decode"] = run_block_decode(torch, workloads.BY_NAME["c5"], max(5, ns.steps // 2), 3)
        except Exception as exc:
            out["model_block_decode"] = {"error": str(exc)[:300]}
    if not ns.no_cpu:
        # every GPU tensor is gone by now; the CPU leg runs last so that it cannot disturb the GPU timings
        out["cpu_baseline"] = cpu_baseline(torch, w, full_batch=True)
        if not ns.no_extra:
            out["cpu_baselines"] = {w.name: out["cpu_baseline"]}
            for ow in workloads.WORKLOADS:
                if ow.name != w.name:
                    try:
                        out["cpu_baselines"][ow.name] = cpu_baseline(torch, ow, full_batch=False)
                    except Exception as exc:
                        out["cpu_baselines"][ow.name] = {"error": str(exc)[:300]}
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
