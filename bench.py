#!/usr/bin/env python3
"""Benchmark of the sparse-attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload north_star|north_star_bs64|north_star_global|north_star_bf16|dense_phase|dense_phase_d64|config1|config1_b256|config2|config3|config4|config5|config5_fp32]

A step is one forward+backward of the drop-in sparse attention module (``CUDABlockAttention``:
layout preparation, the C-ABI forward, the C-ABI backward) on seeded synthetic inputs that are
already resident in HBM.  The default workload is the north-star configuration: B=32, H=2, L=4096,
d=32, 32x32 blocks, diagonal band of 3 plus random blocks up to 10 % block density, fp32.

Prints ONE JSON line.  ``value`` is the effective TFLOP/s of the step (algorithmic FLOPs
12*n*d*NB divided by the step time); ``roofline`` describes the slowest kernel (its share of the
algorithmic FLOPs over its own HIP-event time); ``cpu_baseline`` is the dense PyTorch statement of
the same semantics (the oracle) timed on the host cores over a bounded sample of the batch.
``window_ms`` holds five further 20-step timings of the same step and their median.  The default run
adds the other measured workloads as sub-objects of the same line (``config1``, ``config4``,
``config5``, ``config5_fp32``, ``config2``, ``dense_phase``: step time, windows and roofline of each; ``--no-config1``
and ``--no-extra`` leave them out); their CPU baselines are part of their own ``--workload`` runs.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_FP32_MFMA_TFLOPS = 157.3
PEAK_HBM_GBS = 8000.0
PEAK_BF16_MFMA_TFLOPS = 2500.0


def _event_ms(fn, iters, warm=3):
    """Average duration of fn() in ms from HIP events on the current (= the library's) stream."""
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(iters):
        fn()
    end.record()
    end.synchronize()
    return start.elapsed_time(end) / iters


def _spin_up(step, min_ms=300.0):
    """Untimed repetitions of ``step`` for at least ``min_ms`` of wall time, in batches separated by a
    synchronisation.  The shader clock of an idle MI355X needs some tens of milliseconds of continuous load to
    reach its steady value; without this a short run (few warm-up steps) is timed on the ramp.  Returns the
    wall time spent, in ms."""
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    while True:
        for _ in range(20):
            step()
        torch.cuda.synchronize()
        el = 1e3 * (time.perf_counter() - t0)
        if el >= min_ms:
            return el


def _timed_steps(step, steps, warmup):
    """``warmup`` untimed steps, then exactly ``steps`` timed ones between two synchronisations: ms per step."""
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    return 1e3 * (time.perf_counter() - t0) / steps


def _windows(step, n_windows=5, per=20):
    """Five back-to-back windows of 20 steps each, every one between two synchronisations: the ms per step of each
    window and their median, so that one line shows how much a single timing of this step moves."""
    out = []
    for _ in range(n_windows):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(per):
            step()
        torch.cuda.synchronize()
        out.append(1e3 * (time.perf_counter() - t0) / per)
    return {"windows": [round(x, 4) for x in out], "median": round(float(np.median(out)), 4), "steps_per_window": per}


def _profiled_traffic_bytes(kernel):
    """HBM bytes per launch of ``kernel`` on the north-star workload as measured with rocprofv3 --pmc
    (FETCH_SIZE / WRITE_SIZE scaled by a copy kernel of known size): the 'HBM MiB/launch' column of the
    committed summary profiles/north_star_tile_kernels.txt.  None if the summary has no such row."""
    path = os.path.join(ROOT, "profiles", "north_star_tile_kernels.txt")
    try:
        in_table = False
        for line in open(path):
            if line.startswith("kernel") and "HBM MiB/launch" in line:
                in_table = True
                continue
            if in_table:
                if not line.strip():
                    break
                if line.startswith(kernel):
                    return float(line.split()[-1]) * 1048576.0
    except OSError:
        pass
    return None


def build_workload(name):
    from spion_amd import workloads
    from spion_amd.csr import block_mask_to_csr_host

    if name in ("north_star", "north_star_bs64", "north_star_global"):
        # bs64: the block size the reference uses on its L = 4000 tasks (config.py:99,181), same density
        # global: plus one block row and one block column that span the sequence (as configuration 5 has)
        B, H, L, d, bs = 32, 2, 4096, 32, 64 if name == "north_star_bs64" else 32
        mat = workloads.north_star_mask(bs)
        if name == "north_star_global":
            mat[0, :] = 1.0
            mat[:, 0] = 1.0
        scale = 1.0
    elif name in ("config1", "config1_b256"):
        # b256: the same layer at the batch size the reference trains its L = 1024 tasks with (config.py:60)
        B, H, L, d, bs = 256 if name == "config1_b256" else 8, 2, 1024, 32, 32
        mat = workloads.config1_mask()
        scale = 1.0 / np.sqrt(32.0)
    elif name == "config4":
        B, H, L, d, bs = 32, 2, 4096, 32, 1
        mat = None
        scale = 1.0
    elif name == "config5_fp32":
        # shape of the scale-up configuration (L=16384, d=64, 64x64 blocks, band + global row/column
        # + 1 % random blocks) run through the fp32 path, for comparison with the bf16 one ("config5")
        B, H, L, d, bs = 4, 8, 16384, 64, 64
        mat = workloads.config5_mask()
        scale = 1.0 / 8.0
    else:
        raise SystemExit(f"unknown workload {name}")
    wl = dict(name=name, B=B, H=H, L=L, d=d, bs=bs, mat=mat, scale=scale)
    if mat is not None:
        sm, off, col = block_mask_to_csr_host(mat, bs)
        wl["block_density"] = float(mat.mean())
    else:
        sm, off, col = workloads.window_random_csr(L, 64, 205, seed=3)
        wl["block_density"] = None
    wl.update(sum_mat=sm, offsets=off, columns=col, nnz=int(off[-1]))
    return wl


def cpu_baseline(wl, budget_s=20.0):
    """The oracle's dense PyTorch statement (forward + autograd backward) on the host cores, on as many
    whole samples of the batch as fit in the time budget."""
    from oracle import sparse_attention as osa
    from spion_amd import workloads

    cores = os.cpu_count() or 1
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)
    H, L, d = wl["H"], wl["L"], wl["d"]
    if L > 8192:
        H = 1  # an [H, L, L] fp32 buffer per head is 1 GiB at L = 16384: one head is the bounded sample
    rows = osa.csr_row_index(wl["offsets"])
    pat = torch.zeros(L, L)
    pat[torch.from_numpy(rows), torch.from_numpy(wl["columns"].astype(np.int64))] = 1.0
    key_mask = workloads.valid_length_mask(1, L, L // 2, L, seed=5) if wl["name"] == "config4" else None
    q, k, v, do = workloads.qkv(1, H, L, d, scale=wl["scale"], seed=0)
    for t in (q, k, v):
        t.requires_grad_()

    def one():
        for t in (q, k, v):
            t.grad = None
        o, _ = osa.dense_masked_attention(q, k, v, pat, key_mask)
        o.backward(do)

    one()  # warm-up
    t0 = time.perf_counter()
    n = 0
    while True:
        one()
        n += 1
        el = time.perf_counter() - t0
        if el > budget_s or n >= wl["B"]:
            break
    flops = 12.0 * wl["nnz"] * d * H * n
    return dict(value=flops / el / 1e12, unit="TFLOP/s", cores=cores, kind="port",
                ms_per_sample=1e3 * el / n,
                sample=f"{n} of {wl['B']} samples (H={H}, L={L}, d={d}) of the same workload, dense masked "
                       f"softmax attention forward+autograd backward in PyTorch fp32; effective rate on the "
                       f"algorithmic 12*n*d FLOPs (dense FLOPs actually executed: {12.0 * L * L * d * H * n:.3e})")


def bench_pattern_discovery(args, dev):
    """Configuration 2: two 1024x1024 score maps -> 31x31 diagonal filter, 32x32 pooling, q = 0.90, path walk.
    HBM-bound: 4*L*L bytes read per map.  CPU baseline: the oracle's PyTorch-CPU route on the same maps."""
    import spion_amd
    from oracle import pattern as op
    from spion_amd import workloads

    L, bs, q, n_maps = 1024, 32, 0.90, 2
    maps_cpu = workloads.score_maps_config2(n_maps, L, 32, seed=0)
    maps = maps_cpu.to(dev)

    def step():
        return spion_amd.discover_block_masks(maps, bs, mode="conv_ff", threshold=q)

    spinup_ms = _spin_up(step, args.spinup_ms)
    ms_step = _timed_steps(step, args.steps, args.warmup)
    window_ms = _windows(step)
    t_evt = _event_ms(step, max(10, args.steps))
    bytes_read = 4.0 * L * L * n_maps
    cpu = None
    if not args.no_cpu_baseline:
        t1 = time.perf_counter()
        reps = 0
        while time.perf_counter() - t1 < 10.0:
            for i in range(n_maps):
                op.generate_mask_conv_ff(maps_cpu[i].numpy(), bs, q, route="torch")
            reps += 1
        cpu_ms = 1e3 * (time.perf_counter() - t1) / reps
        cpu = {"value": n_maps / (cpu_ms / 1e3), "unit": "maps/s", "cores": min(os.cpu_count() or 1, torch.get_num_threads()),
               "kind": "port", "sample": f"the same {n_maps} maps, {reps} repetitions of the PyTorch-CPU route "
                                         "(F.conv2d, avg_pool2d, quantile) plus the iterative walk"}
    result = {
        "metric": "pattern discovery (conv filter + block pool + quantile + path walk), maps per second, 1 GPU",
        "value": n_maps / (ms_step / 1e3), "unit": "maps/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_step, "window_ms": window_ms, "spinup_ms": round(spinup_ms, 1), "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f64",
        "data": "synthetic (seeded softmax(QK^T) maps with a diagonal band boost)",
        "config": {"workload": f"config2: {n_maps} score maps {L}x{L}, 31x31 diagonal filter, {bs}x{bs} pooling, q={q}"},
        "roofline": {"bound": "hbm", "kernel": "conv_pool_cols_kernel + threshold_walk_kernel", "achieved": bytes_read / t_evt / 1e6,
                     "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": bytes_read / t_evt / 1e6 / PEAK_HBM_GBS, "traffic": None,
                     "event_ms": t_evt},
    }
    if cpu:
        result["cpu_baseline"] = cpu
    return result


def bench_encoder_step(args, dev):
    """Configuration 3: one training step (forward, backward, AdamW update) of the 2-layer sparse encoder,
    batch 256, L=1024, d_model 64, FFN 128, H=2, d_head 32, masks discovered from the model's own dense phase.
    The model around the attention layers is plain torch.nn (tests/encoder_harness.py)."""
    import spion_amd
    from tests import encoder_harness as eh

    torch.manual_seed(0)
    cfg = eh.model_config(L=1024, batch=256, block_size=32, key_mask=False, threshold=0.90)
    ids, mask, labels = eh.synthetic_batch(cfg, seed=1, device=dev)
    model = eh.EncoderForSC(cfg, spion_amd.Attention).to(dev)
    with torch.no_grad():
        _, attn_lst = model(ids, mask, labels, None, is_attn=True)
    mat_lst = spion_amd.generate_pattern_conv_ff(attn_lst, cfg)
    density = [float(m.mean()) for m in mat_lst[0]]
    del attn_lst
    torch.cuda.empty_cache()
    for layer in model.layers:
        layer.mha.reconstruct_for_blocksparse(cfg)
    opt = eh.make_optimizer(model)

    def step():
        opt.zero_grad(set_to_none=True)
        loss, _ = model(ids, mask, labels, mat_lst)
        loss.mean().backward()
        opt.step()

    spinup_ms = _spin_up(step, args.spinup_ms)
    ms_step = _timed_steps(step, args.steps, args.warmup)
    window_ms = _windows(step)

    # attention share: the two layers' C-ABI kernels, from HIP events around a forward+backward of one layer's
    # attention core at the same shape
    B, H, L, d = cfg["batch_size"], cfg["num_head"], cfg["max_seq_len"], cfg["head_dim"]
    core_mod = model.layers[0].mha.block_attn
    q, k, v, do = (torch.randn(B, H, L, d, device=dev) for _ in range(4))
    for t in (q, k, v):
        t.requires_grad_()

    def attn_only():
        out, _ = core_mod(q, k, v, mask, mat_lst[0][0])
        out.backward(do)

    t_attn = _event_ms(attn_only, max(10, args.steps))
    return {
        "metric": "2-layer sparse encoder training step (fwd+bwd+AdamW), samples per second, 1 GPU",
        "value": B / (ms_step / 1e3), "unit": "samples/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_step, "window_ms": window_ms, "spinup_ms": round(spinup_ms, 1), "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic (uniform token ids, uniform labels, random-init weights)",
        "config": {"workload": f"config3: 2-layer encoder step, batch {B}, L={L}, d_model 64, FFN 128, H={H}, d_head {d}, "
                               f"block {cfg['block_size']}, discovered block densities {[round(x, 3) for x in density]}"},
        "attention_core_ms_per_layer": t_attn,
        "attention_share_of_step": 2.0 * t_attn / ms_step,
    }


def bench_bf16_scale_up(args, dev, shape="config5"):
    """Configuration 5 (``shape="north_star"``: the north-star shape and mask with bf16 tensors instead): bf16 tensors, fp32 accumulation and softmax, B=4, H=8, L=16384, d=64, 64x64 blocks (band +
    one global block row and column + 1 % random blocks), Q, K, V ~ N(0,1)/8.  A step is forward + backward of the
    ``BlockAttentionBF16`` module.  The probabilities are never written to memory, so the algorithmic bytes are the
    eleven [NB, L, d] bf16 tensors plus the fp32 row statistics; the roofline is HBM (ridge of bf16 MFMA: 310 flop/B,
    this workload: 12*n*d / (22*L*d) = 268 flop/B)."""
    import spion_amd
    from spion_amd import _lib, workloads
    from spion_amd.csr import block_mask_to_csr_host

    if shape == "north_star":
        B, H, L, d, bs, in_scale = 32, 2, 4096, 32, 32, 1.0
        mat_np = workloads.north_star_mask(bs)
    else:
        B, H, L, d, bs, in_scale = 4, 8, 16384, 64, 64, 1.0 / 8.0
        mat_np = workloads.config5_mask()
    NB = B * H
    _, off, _ = block_mask_to_csr_host(mat_np, bs)
    nnz = int(off[-1])
    mat = torch.from_numpy(mat_np).to(dev)
    q, k, v, do = (t.to(torch.bfloat16) for t in workloads.qkv(B, H, L, d, scale=in_scale, seed=0, device=dev))
    for t in (q, k, v):
        t.requires_grad_()
    cfg = dict(head_dim=d, num_head=H, max_seq_len=L, batch_size=B, block_size=bs)
    module = spion_amd.BlockAttentionBF16(cfg)
    ones = torch.ones(B, L, device=dev)

    def step():
        for t in (q, k, v):
            t.grad = None
        out, _ = module(q, k, v, ones, mat)
        out.backward(do)

    spinup_ms = _spin_up(step, args.spinup_ms)
    ms_step = _timed_steps(step, args.steps, args.warmup)
    window_ms = _windows(step)

    core = _lib.core()
    idx = module.csr_cache.get(mat, bs)
    Q, K, V, dO = (t.detach().reshape(NB, L, d).contiguous() for t in (q, k, v, do))
    O, dQ, dK, dV = (torch.empty_like(Q) for _ in range(4))
    lse = torch.empty(NB, L, device=dev)
    tail = (idx.offsets.data_ptr(), idx.columns.data_ptr(), idx.sum_mat.data_ptr(), nnz)

    def fwd():
        core.spion_block_bf16_attn_forward(module.attn_handle, Q.data_ptr(), K.data_ptr(), V.data_ptr(), None,
                                           O.data_ptr(), lse.data_ptr(), *tail)

    def bwd():
        core.spion_block_bf16_attn_backward(module.attn_handle, Q.data_ptr(), K.data_ptr(), V.data_ptr(), None,
                                            O.data_ptr(), lse.data_ptr(), dO.data_ptr(), dQ.data_ptr(), dK.data_ptr(),
                                            dV.data_ptr(), *tail)

    it = max(10, args.steps)
    t_fwd = _event_ms(fwd, it)
    t_bwd = _event_ms(bwd, it)
    core.spion_set_backward_passes(module.attn_handle, 1)
    t_row = _event_ms(bwd, it)
    core.spion_set_backward_passes(module.attn_handle, 2)
    t_col = _event_ms(bwd, it)
    core.spion_set_backward_passes(module.attn_handle, 3)
    _lib.check_error("bench bf16 kernels")

    alg_flops = workloads.sparse_flops(nnz, d, NB)
    tensor = 2.0 * L * d * NB  # one [NB, L, d] bf16 tensor
    stat = 4.0 * L * NB        # one [NB, L] fp32 row statistic
    # forward: read Q, K, V, write O, lse; row pass: read Q, K, V, dO, O, lse, write dQ, -g; column pass: read
    # Q, K, V, dO, lse, -g, write dK, dV
    kbytes = {"bf16_fwd_kernel": 4 * tensor + stat, "bf16_bwd_row_kernel": 6 * tensor + 2 * stat,
              "bf16_bwd_col_kernel": 6 * tensor + 2 * stat}
    alg_bytes = 11 * tensor + 2 * stat  # each tensor once (11 of them) plus the statistic written and read back
    kernels = dict(zip(kbytes, (t_fwd, t_row, t_col)))
    dom = max(kernels, key=kernels.get)
    roof = dict(bound="hbm", kernel=dom, achieved=kbytes[dom] / kernels[dom] / 1e6, peak=PEAK_HBM_GBS, unit="GB/s",
                traffic=None)
    roof["frac"] = roof["achieved"] / roof["peak"]
    roof["kernel_ms"] = {k_: round(v_, 4) for k_, v_ in kernels.items()}
    roof["mfma_frac_of_bf16_peak"] = (alg_flops / 3.0) / kernels[dom] / 1e9 / PEAK_BF16_MFMA_TFLOPS
    result = {
        "metric": "sparse-attn fwd+bwd effective TFLOP/s (12*n*d*NB algorithmic FLOPs / step time), 1 GPU",
        "value": alg_flops / ms_step / 1e9, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_step, "window_ms": window_ms, "spinup_ms": round(spinup_ms, 1), "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": f"synthetic (seeded N(0,1)*{in_scale:g} tensors rounded to bf16, seeded block mask)",
        "config": {"workload": f"{shape}{'_bf16' if shape != 'config5' else ''}: bf16 sparse attention fwd+bwd, B={B} H={H} L={L} d={d}, block {bs}, "
                               f"nnz/head={nnz}, block density={round(float(mat_np.mean()), 4)}",
                   "kernel_path": "mfma-bf16-tile"},
        "abi_ms": {"attn_forward": round(t_fwd, 4), "attn_backward": round(t_bwd, 4),
                   "fwd_plus_bwd": round(t_fwd + t_bwd, 4)},
        "abi_effective_tflops": alg_flops / (t_fwd + t_bwd) / 1e9,
        "abi_effective_hbm_gbs": alg_bytes / (t_fwd + t_bwd) / 1e6,
        "algorithmic": {"gflop": alg_flops / 1e9, "mbytes": alg_bytes / 1e6},
        "roofline": roof,
    }
    if not args.no_cpu_baseline:
        wl = build_workload("config5_fp32" if shape == "config5" else "north_star")
        result["cpu_baseline"] = cpu_baseline(wl)
    return result


def bench_dense_phase(args, dev, d=32):
    """Dense-phase attention (the phase that feeds pattern discovery) at configuration 3's layer shape: B=256, H=2,
    L=1024, d=32, fp32, forward + backward of the ``CUDAAttention`` module, which materialises the full
    [B, H, L, L] probability map (2.1 GB) as the reference does.  FLOPs 12*L*L*d*NB; MFMA-bound.
    d=64 (``dense_phase_d64``): the same FLOPs with half the batch."""
    import spion_amd
    from oracle import sparse_attention as osa
    from spion_amd import _lib, workloads
    from spion_amd.attention import Attention

    B, H, L = (256 if d == 32 else 128), 2, 1024
    NB = B * H
    cfg = dict(head_dim=d, num_head=H, max_seq_len=L, batch_size=B, block_size=32)
    cpp = Attention._cuda_compile_module()
    handle = cpp.init(d, L, NB)
    _lib.check_error("init")
    module = spion_amd.CUDAAttention(cfg, cpp, handle)
    q, k, v, do = workloads.qkv(B, H, L, d, scale=1.0, seed=0, device=dev)
    for t in (q, k, v):
        t.requires_grad_()
    ones = torch.ones(B, L, device=dev)

    def step():
        for t in (q, k, v):
            t.grad = None
        out, _ = module(q, k, v, ones)
        out.backward(do)

    spinup_ms = _spin_up(step, args.spinup_ms)
    ms_step = _timed_steps(step, args.steps, args.warmup)
    window_ms = _windows(step)
    # the same step through the reference's ABI (feature-major operands: four transposes a step)
    module.reads_views = False
    for _ in range(max(3, args.warmup // 4)):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(max(5, args.steps // 4)):
        step()
    torch.cuda.synchronize()
    ms_step_abi = 1e3 * (time.perf_counter() - t0) / max(5, args.steps // 4)
    module.reads_views = True

    # the kernels the module runs: row-major operands at the strided entry points
    import ctypes
    core = _lib.core()
    Qr, Kr, Vr, dOr = (t.detach().contiguous() for t in (q, k, v, do))
    out_r = torch.empty_like(Qr)
    attn = torch.empty(NB, L, L, device=dev)
    gq, gk, gv = (torch.empty_like(Qr) for _ in range(3))
    lay = _lib.head_layout(Qr)
    A = ctypes.addressof(lay)
    t_fwd_rm = _event_ms(lambda: core.spion_dense_forward_strided(
        handle, Qr.data_ptr(), Kr.data_ptr(), Vr.data_ptr(), None, attn.data_ptr(), out_r.data_ptr(), H, A, A),
        max(10, args.steps // 4))
    _lib.check_error("dense forward (row-major)")
    t_bwd_rm = _event_ms(lambda: core.spion_dense_backward_strided(
        handle, Qr.data_ptr(), Kr.data_ptr(), Vr.data_ptr(), attn.data_ptr(), out_r.data_ptr(), dOr.data_ptr(),
        gq.data_ptr(), gk.data_ptr(), gv.data_ptr(), H, A, A, A), max(10, args.steps // 4))
    _lib.check_error("dense backward (row-major)")
    # the same forward leaving the mean of all maps as well (what pattern discovery reads)
    mean_map = torch.empty(L, L, device=dev)
    t_fwd_mean = None
    if d == 32:  # the mean-emitting forward is served for head dimension 32
        t_fwd_mean = _event_ms(lambda: core.spion_dense_forward_strided_mean(
            handle, Qr.data_ptr(), Kr.data_ptr(), Vr.data_ptr(), None, attn.data_ptr(), out_r.data_ptr(),
            mean_map.data_ptr(), H, A, A), max(10, args.steps // 4))
        _lib.check_error("dense forward with mean (row-major)")
    del Qr, Kr, Vr, dOr, out_r, gq, gk, gv, mean_map

    # forward kernel alone at the C ABI (operands in the layouts it takes: Qt, Vt feature-major)
    Qt = _lib.transpose_last2(q.detach().reshape(NB, L, d))
    Vt = _lib.transpose_last2(v.detach().reshape(NB, L, d))
    K = k.detach().reshape(NB, L, d).contiguous()
    out_t = torch.empty(NB, d, L, device=dev)
    t_fwd = _event_ms(lambda: cpp.attn_forward(handle, Qt.data_ptr(), K.data_ptr(), Vt.data_ptr(), attn.data_ptr(),
                                               out_t.data_ptr()), max(10, args.steps // 4))
    _lib.check_error("dense forward")
    # the two backward kernels together (operands: Qt, Kt, V, the map, dOt)
    Kt = _lib.transpose_last2(k.detach().reshape(NB, L, d))
    V = v.detach().reshape(NB, L, d).contiguous()
    dOt = _lib.transpose_last2(do.reshape(NB, L, d))
    dq, dk, dv = (torch.empty(NB, d, L, device=dev) for _ in range(3))
    t_bwd = _event_ms(lambda: cpp.attn_backward(handle, Qt.data_ptr(), Kt.data_ptr(), V.data_ptr(), attn.data_ptr(),
                                                dOt.data_ptr(), None, None, None, dq.data_ptr(), dk.data_ptr(),
                                                dv.data_ptr()), max(10, args.steps // 4))
    _lib.check_error("dense backward")
    alg_flops = 12.0 * L * L * d * NB
    k_fwd = "dense_fwd_reg_kernel" if d == 32 else "dense_fwd_reg64_kernel"
    k_bwd = f"dense_bwd_row{d}_kernel + dense_bwd_col{d}_kernel"
    roof = dict(bound="mfma", kernel=k_fwd, achieved=alg_flops / 3.0 / t_fwd_rm / 1e9,
                peak=PEAK_FP32_MFMA_TFLOPS, unit="TFLOP/s", traffic=None)
    roof["frac"] = roof["achieved"] / roof["peak"]
    roof["kernel_ms"] = {k_fwd: round(t_fwd_rm, 4), k_bwd: round(t_bwd_rm, 4)}
    roof["backward_frac"] = alg_flops * 2.0 / 3.0 / t_bwd_rm / 1e9 / PEAK_FP32_MFMA_TFLOPS
    if t_fwd_mean is not None:
        roof["forward_with_mean_ms"] = round(t_fwd_mean, 4)  # spion_dense_forward_strided_mean: maps + their mean
    # the feature-major ABI: the same kernels at d = 32, the two-sweep kernels with operand-layout loads at d = 64
    roof["reference_abi_kernel_ms"] = {
        k_fwd if d == 32 else "dense_fwd_kernel": round(t_fwd, 4),
        k_bwd if d == 32 else "dense_bwd_row_kernel + dense_bwd_col_kernel": round(t_bwd, 4)}
    result = {
        "metric": "dense-phase attn fwd+bwd effective TFLOP/s (12*L*L*d*NB FLOPs / step time), 1 GPU",
        "value": alg_flops / ms_step / 1e9, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_step, "window_ms": window_ms, "spinup_ms": round(spinup_ms, 1), "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic (seeded N(0,1) tensors)",
        "config": {"workload": f"dense_phase: softmax attention fwd+bwd with the full probability map, B={B} H={H} L={L} d={d}"},
        "algorithmic": {"gflop": alg_flops / 1e9, "map_gbytes": 4.0 * NB * L * L / 1e9},
        "reference_abi_step_ms": round(ms_step_abi, 4),
        "roofline": roof,
    }
    if not args.no_cpu_baseline:
        cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1)))
        torch.set_num_threads(cores)
        qc, kc, vc, doc = workloads.qkv(1, H, L, d, scale=1.0, seed=0)
        for t in (qc, kc, vc):
            t.requires_grad_()
        pat = torch.ones(L, L)
        n, t1 = 0, time.perf_counter()
        while time.perf_counter() - t1 < 10.0:
            for t in (qc, kc, vc):
                t.grad = None
            o, _ = osa.dense_masked_attention(qc, kc, vc, pat, None)
            o.backward(doc)
            n += 1
        el = time.perf_counter() - t1
        result["cpu_baseline"] = dict(value=12.0 * L * L * d * H * n / el / 1e12, unit="TFLOP/s", cores=cores, kind="port",
                                      ms_per_sample=1e3 * el / n,
                                      sample=f"{n} repetitions of one sample (H={H}, L={L}, d={d}): dense softmax attention "
                                             "forward + autograd backward in PyTorch fp32 (the oracle's dense statement; its "
                                             "off-pattern term vanishes on a full pattern)")
    return result


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--workload", default="north_star")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-config1", action="store_true", help="north_star only: leave out the L = 1024 sub-object")
    ap.add_argument("--no-extra", action="store_true",
                    help="north_star only: leave out the config4 / config5 / config5_fp32 / config2 / dense_phase sub-objects")
    ap.add_argument("--spinup-ms", type=float, default=300.0,
                    help="untimed repetitions of the step for this long before the warm-up (clock ramp)")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run a plain 256 MiB device copy a few times (calibrates rocprofv3 byte counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")
    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs a GPU; there is no CPU fallback")
    torch.cuda.set_device(0)
    dev = torch.device("cuda:0")

    import spion_amd
    from spion_amd import _lib, workloads
    from spion_amd.attention import Attention

    if args.copy_probe:
        src = torch.ones(64 * 1024 * 1024, dtype=torch.float32, device=dev)  # 256 MiB read + 256 MiB written
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    if args.workload == "config2":
        print(json.dumps(bench_pattern_discovery(args, dev)))
        return
    if args.workload == "config3":
        print(json.dumps(bench_encoder_step(args, dev)))
        return
    if args.workload == "config5":
        print(json.dumps(bench_bf16_scale_up(args, dev)))
        return
    if args.workload in ("dense_phase", "dense_phase_d64"):
        print(json.dumps(bench_dense_phase(args, dev, 32 if args.workload == "dense_phase" else 64)))
        return
    if args.workload == "north_star_bf16":
        print(json.dumps(bench_bf16_scale_up(args, dev, "north_star")))
        return

    result = bench_sparse_layer(args, dev, args.workload, full=True)
    if args.workload == "north_star":
        # the other measured workloads ride in the same line, each as a sub-object with its own step time, windows and
        # roofline (CPU baselines only in their own --workload runs, so that the default run stays within minutes)
        keep = ("metric", "value", "unit", "ms_per_step", "window_ms", "spinup_ms", "dtype", "config", "hip_graph",
                "rowmajor_abi_ms", "abi_ms", "kernels_effective_tflops", "roofline", "algorithmic")
        sub = argparse.Namespace(**vars(args))
        sub.no_cpu_baseline = True
        extra = []
        if not args.no_config1:
            # the metric is quoted at L = 1024 and L = 4096: the L = 1024 point is configuration 1
            extra.append(("config1", lambda: bench_sparse_layer(sub, dev, "config1", full=False)))
        if not args.no_extra:
            extra += [("config4", lambda: bench_sparse_layer(sub, dev, "config4", full=False)),
                      ("config5", lambda: bench_bf16_scale_up(sub, dev)),
                      ("config5_fp32", lambda: bench_sparse_layer(sub, dev, "config5_fp32", full=False)),
                      ("config2", lambda: bench_pattern_discovery(sub, dev)),
                      ("dense_phase", lambda: bench_dense_phase(sub, dev))]
        for name, run in extra:
            r = run()
            result[name] = {k_: r[k_] for k_ in keep if k_ in r}
            torch.cuda.empty_cache()
    print(json.dumps(result))


def bench_sparse_layer(args, dev, workload, full=True):
    """Forward + backward of the drop-in sparse attention module on one of the fp32 workloads.  ``full`` adds the
    legs that only describe the default workload further (reference-ABI timings, projection views, CPU baseline)."""
    import spion_amd
    from spion_amd import _lib, workloads
    from spion_amd.attention import Attention

    wl = build_workload(workload)
    B, H, L, d, bs, nnz = wl["B"], wl["H"], wl["L"], wl["d"], wl["bs"], wl["nnz"]
    NB = B * H
    q, k, v, do = workloads.qkv(B, H, L, d, scale=wl["scale"], seed=0, device=dev)
    for t in (q, k, v):
        t.requires_grad_()
    with_mask = wl["name"] == "config4"
    cfg = dict(head_dim=d, num_head=H, max_seq_len=L, batch_size=B, block_size=bs)
    if with_mask:
        cpp = Attention._blockcuda_mask_compile_module()
        mod_cls = spion_amd.CUDABlockMaskAttention
        key_mask = workloads.valid_length_mask(B, L, L // 2, L, seed=5).to(dev)
        pattern = torch.zeros(L, L)
        rows = np.repeat(np.arange(L), wl["sum_mat"])
        pattern[torch.from_numpy(rows), torch.from_numpy(wl["columns"].astype(np.int64))] = 1.0
        mat = pattern.to(dev)
    else:
        cpp = Attention._blockcuda_compile_module()
        mod_cls = spion_amd.CUDABlockAttention
        key_mask = torch.ones(B, L, device=dev)
        mat = torch.from_numpy(wl["mat"]).to(dev)
    handle = cpp.init(d, L, NB, bs)
    _lib.check_error("init")
    module = mod_cls(cfg, cpp, handle)

    def step():
        for t in (q, k, v):
            t.grad = None
        out, _ = module(q, k, v, key_mask, mat)
        out.backward(do)

    spinup_ms = _spin_up(step, args.spinup_ms)
    ms_step = _timed_steps(step, args.steps, args.warmup)
    window_ms = _windows(step)
    path = _lib.core().spion_last_path(handle)

    # ---- the same step recorded once as a HIP graph and replayed (what a launch-bound caller would do) ----------
    graph_ms = None
    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        for t in (q, k, v):
            t.grad = None
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            out_g, _ = module(q, k, v, key_mask, mat)
            out_g.backward(do)
        _spin_up(graph.replay, min(args.spinup_ms, 100.0))
        graph_ms = _timed_steps(graph.replay, args.steps, args.warmup)
        del graph, out_g
    except Exception as e:  # the eager figures above stand on their own
        graph_ms = f"capture failed: {type(e).__name__}: {e}"
    for t in (q, k, v):
        t.grad = None
    _lib.use_current_stream(module, dev)  # the capture left the handle on its own stream
    # ---- the same step with the heads as the layer hands them over: views of [B, L, H*d] projections ------
    views = None
    if full and getattr(module, "reads_views", False):
        qv, kv, vv = (t.detach().transpose(1, 2).contiguous().transpose(1, 2).requires_grad_() for t in (q, k, v))
        dov = do.transpose(1, 2).contiguous().transpose(1, 2)

        def step_views():
            for t in (qv, kv, vv):
                t.grad = None
            o, _ = module(qv, kv, vv, key_mask, mat)
            o.backward(dov)

        views = {}
        for name, flag in (("in_place_ms", True), ("with_copies_ms", False)):
            module.reads_views = flag
            views[name] = round(_timed_steps(step_views, args.steps, args.warmup), 4)
        module.reads_views = True
        views["what"] = ("module step on heads that are views of [B,L,H*d] projections: read and written in place "
                         "by the strided entry points, against the reference's contiguous copies first")
        del qv, kv, vv, dov
    # the module hands the forward's output to the backward itself; a caller of the reference's ABI cannot, so
    # the timings below run with the library's kept copies of Out, as such a caller would
    _lib.core().spion_use_output_cache(handle, 1)

    # ---- per-kernel times at the C ABI, HIP events on the library's stream -----------------------
    core = _lib.core()
    idx = module.csr_cache.get(mat, bs)
    Q = q.detach().reshape(NB, L, d).contiguous()
    K = k.detach().reshape(NB, L, d).contiguous()
    V = v.detach().reshape(NB, L, d).contiguous()
    dO = do.reshape(NB, L, d).contiguous()
    Kt = K.transpose(1, 2).contiguous()
    Vt = V.transpose(1, 2).contiguous()
    P = torch.empty(NB * nnz, device=dev)
    O = torch.empty_like(Q)
    dP = torch.empty(NB * nnz, device=dev)
    dS = torch.empty(NB * nnz, device=dev)
    dQ, dK, dV = torch.empty_like(Q), torch.empty_like(Q), torch.empty_like(Q)
    pen = (1e6 * (1.0 - key_mask.repeat(1, H))).contiguous() if with_mask else None

    def fwd():
        a = [handle, Q.data_ptr(), Kt.data_ptr(), V.data_ptr()] + ([pen.data_ptr()] if with_mask else [])
        cpp.attn_forward(*a, P.data_ptr(), O.data_ptr(), idx.offsets.data_ptr(), idx.columns.data_ptr(),
                         idx.sum_mat.data_ptr(), nnz)

    def bwd():
        cpp.attn_backward(handle, Q.data_ptr(), K.data_ptr(), Vt.data_ptr(), P.data_ptr(), dO.data_ptr(),
                          dP.data_ptr(), dS.data_ptr(), dQ.data_ptr(), dK.data_ptr(), dV.data_ptr(),
                          idx.offsets.data_ptr(), idx.columns.data_ptr(), idx.sum_mat.data_ptr(), nnz)

    # what the module runs: every operand row-major, the forward's output handed to the backward
    def fwd_rm():
        core.spion_attn_forward_rowmajor(handle, Q.data_ptr(), K.data_ptr(), V.data_ptr(),
                                         pen.data_ptr() if with_mask else None, P.data_ptr(), O.data_ptr(),
                                         idx.offsets.data_ptr(), idx.columns.data_ptr(), idx.sum_mat.data_ptr(), nnz)

    def bwd_rm():
        core.spion_attn_backward_rowmajor(handle, Q.data_ptr(), K.data_ptr(), V.data_ptr(), P.data_ptr(), O.data_ptr(),
                                          dO.data_ptr(), dS.data_ptr(), dQ.data_ptr(), dK.data_ptr(), dV.data_ptr(),
                                          idx.offsets.data_ptr(), idx.columns.data_ptr(), idx.sum_mat.data_ptr(), nnz)

    it = max(10, args.steps)
    # the reference's ABI (transposed K / V operands, no output in the backward: the library keeps copies)
    t_fwd_abi = _event_ms(fwd, it)
    t_bwd_abi = _event_ms(bwd, it)
    t_seq_abi = _event_ms(lambda: (fwd(), bwd()), it)  # the order a training step runs them in
    # the three kernels as the module launches them
    core.spion_use_output_cache(handle, 0)
    t_fwd = _event_ms(fwd_rm, it)
    t_bwd = _event_ms(bwd_rm, it)
    t_seq = _event_ms(lambda: (fwd_rm(), bwd_rm()), it)
    core.spion_set_backward_passes(handle, 1)
    t_row = _event_ms(bwd_rm, it)
    core.spion_set_backward_passes(handle, 2)
    t_col = _event_ms(bwd_rm, it)
    core.spion_set_backward_passes(handle, 3)
    _lib.check_error("bench kernels")

    alg_flops = workloads.sparse_flops(nnz, d, NB)
    alg_bytes = workloads.sparse_bytes(nnz, L, d, NB)
    third = alg_flops / 3.0  # forward, row pass and column pass carry 4*n*d*NB each
    names = {1: ("tile_fwd_kernel", "tile_bwd_row_kernel", "tile_bwd_col_kernel"),
             2: ("elem_fwd_kernel", "elem_bwd_row_kernel", "elem_bwd_col_kernel"),
             # hybrid: dense window tiles on the MFMA units + gathered remainder; each phase is two or three launches
             3: ("hyb_rem_logits_lds_kernel + hyb_tile_fwd_kernel + hyb_rem_pv_lds_kernel"
                 if L % 1024 == 0 and NB * (L // 1024) >= 256 and "SPION_HYB_GATHER" not in os.environ
                 else "hyb_rem_logits_kernel + hyb_tile_fwd_kernel + hyb_rem_pv_kernel",
                 "hyb_tile_bwd_row_kernel + hyb_rem_bwd_row_kernel",
                 "hyb_tile_bwd_col_kernel + " + ("hyb_rem_bwd_col_lds_kernel" if L % 1024 == 0 and NB * (L // 256) >= 256
                                                  and "SPION_HYB_GATHER" not in os.environ else "hyb_rem_bwd_col_kernel"))}[path]
    kernels = dict(zip(names, (t_fwd, t_row, t_col)))
    dom = max(kernels, key=kernels.get)
    dom_ms = kernels[dom]
    if path == 1:
        roof = dict(bound="mfma", kernel=dom, achieved=third / dom_ms / 1e9, peak=PEAK_FP32_MFMA_TFLOPS,
                    unit="TFLOP/s", traffic=None)
    else:
        # element path: HBM-bound by design; the slowest kernel's share of the algorithmic bytes
        share = {names[0]: 4.0 * (4 * L * d + nnz) * NB, names[1]: 4.0 * (4 * L * d + nnz) * NB,
                 names[2]: 4.0 * (3 * L * d) * NB}[dom]
        roof = dict(bound="hbm", kernel=dom, achieved=share / dom_ms / 1e6, peak=PEAK_HBM_GBS, unit="GB/s",
                    traffic=None)
    roof["frac"] = roof["achieved"] / roof["peak"]
    if wl["name"] == "north_star":  # the workload the committed byte counters were taken on
        roof["traffic"] = _profiled_traffic_bytes(dom)
    roof["kernel_ms"] = {k_: round(v_, 4) for k_, v_ in kernels.items()}
    if path == 2:
        # what the element kernels actually move: per pattern entry two gathered rows of d floats (K and V in the
        # forward and the row pass, Q and dO in the column pass), served by the caches, not by HBM
        gbytes = 2.0 * 4.0 * d * nnz * NB
        roof["gathered_rows"] = {
            "gbytes_per_kernel": round(gbytes / 1e9, 2),
            "tbytes_per_s": {k_: round(gbytes / v_ / 1e9, 2) for k_, v_ in kernels.items()},
            "what": "bytes of gathered operand rows per kernel over its time; for scale, 256 CUs x 64 B per clock "
                    "at 2.4 GHz of vector L1 bandwidth would be 39 TB/s"}
    if path == 1:
        # MFMA work a tile costs each kernel against its algorithmic share: the column pass recomputes dP (1.5x);
        # the forward is taken in its register-resident form (1x; its two-sweep form for very long rows is 1.5x)
        executed = {"tile_fwd_kernel": 1.0, "tile_bwd_row_kernel": 1.0, "tile_bwd_col_kernel": 1.5}
        roof["frac_per_kernel"] = {k_: round(third / v_ / 1e9 / PEAK_FP32_MFMA_TFLOPS, 4) for k_, v_ in kernels.items()}
        roof["frac_on_executed_mfma"] = {k_: round(executed[k_] * third / v_ / 1e9 / PEAK_FP32_MFMA_TFLOPS, 4)
                                         for k_, v_ in kernels.items()}

    result = {
        "metric": "sparse-attn fwd+bwd effective TFLOP/s (12*n*d*NB algorithmic FLOPs / step time), 1 GPU",
        "value": alg_flops / ms_step / 1e9,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_step,
        "window_ms": window_ms,
        "spinup_ms": round(spinup_ms, 1),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic (seeded N(0,1) tensors, seeded block mask)",
        "config": {"workload": f"{wl['name']}: sparse attention fwd+bwd, B={B} H={H} L={L} d={d}, "
                               f"block {bs}, nnz/head={nnz}, block density="
                               f"{wl['block_density'] if wl['block_density'] is None else round(wl['block_density'], 4)}",
                   "kernel_path": {1: "mfma-tile", 2: "element", 3: "hybrid (mfma tiles + gathered remainder)"}[path]},
        "rowmajor_abi_ms": {"attn_forward": round(t_fwd, 4), "attn_backward": round(t_bwd, 4),
                            "fwd_plus_bwd": round(t_fwd + t_bwd, 4), "fwd_then_bwd_sequence": round(t_seq, 4),
                            "what": "spion_attn_forward_rowmajor / spion_attn_backward_rowmajor, the entry points "
                                    "the module calls; kernel_ms are these kernels"},
        "abi_ms": {"attn_forward": round(t_fwd_abi, 4), "attn_backward": round(t_bwd_abi, 4),
                   "fwd_plus_bwd": round(t_fwd_abi + t_bwd_abi, 4), "fwd_then_bwd_sequence": round(t_seq_abi, 4),
                   "what": "the reference's ABI: transposed K / V operands, kept copies of Out"},
        "kernels_effective_tflops": alg_flops / (t_fwd + t_bwd) / 1e9,
        "kernels_fraction_of_fp32_mfma_peak": alg_flops / (t_fwd + t_bwd) / 1e9 / PEAK_FP32_MFMA_TFLOPS,
        "kernels_effective_hbm_gbs": alg_bytes / (t_fwd + t_bwd) / 1e6,
        "abi_effective_tflops": alg_flops / (t_fwd_abi + t_bwd_abi) / 1e9,
        "abi_fraction_of_fp32_mfma_peak": alg_flops / (t_fwd_abi + t_bwd_abi) / 1e9 / PEAK_FP32_MFMA_TFLOPS,
        "algorithmic": {"gflop": alg_flops / 1e9, "mbytes": alg_bytes / 1e6},
        "roofline": roof,
    }
    if isinstance(graph_ms, float):
        result["hip_graph"] = {"ms_per_step": graph_ms, "value": alg_flops / graph_ms / 1e9,
                               "what": "the module's forward + backward recorded once as a HIP graph and replayed"}
    else:
        result["hip_graph"] = {"error": graph_ms}
    if views:
        result["projection_views"] = views
    if full and not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(wl)
    cpp.destroy(handle)
    return result


if __name__ == "__main__":
    main()
