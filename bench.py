#!/usr/bin/env python3
"""Benchmark of the memory-rule hot path on one MI355X.

A step is one forward + backward pass of the workload over one batch of
synthetic input that is already resident in HBM.  Prints ONE JSON line.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

Workloads (BASELINE.json `configs`):
  titans_chunkwise_c3  configs[2] (default; the metric's d=512, L=4096): Titans LMM
                    chunkwise training, chunk 64, 8 heads x 64, batch 16, seq 4096,
                    bf16 k/v/q, fp32 accumulate and state; matrix-core kernels.
  titans_exact_c2   configs[1]: Titans LMM exact recurrence, 8 heads x 64
                    (d=512), batch 8, seq 2048, fp32, state checkpoints every 64
                    tokens (checkpointed forward + fused checkpointed backward).
  swa_c5            the attention branch of configs[4]: sliding-window attention, window 512,
                    8 heads x 64, bf16 storage, fp32 softmax, batch 8, seq 4096, fwd+bwd.
  swa_stats_c5      the same attention through the pair that keeps two softmax statistics per query
                    instead of the weight tensor (what the layer calls).
  mag_layer_c5      configs[4]: the full layer — CMS of k=4 Titans levels (periods 1, 8, 64, 512;
                    chunkwise rule, chunk 64) gating sliding-window attention (window 512), 8 heads
                    x 64, batch 8, seq 4096: forward + backward + frequency-aware AdamW step.
  adamw_c5          the optimizer step of configs[4]: frequency-aware AdamW over the layer's
                    parameter set (d=512, k=4 levels, all levels firing), gradient-norm clip
                    + update in two launches; here a "token" is a parameter.
  hope_selfref_c4   configs[3]: HOPE self-referential memory, 8 heads x 64, batch 8,
                    seq 2048, fp32, self-generated values, frozen snapshots per
                    64-token chunk; grads to x and to the six initial memories.
  hebbian_c2        the Hebbian rule (M <- (1 - alpha) M + v k^T) at the shape of configs[1]:
                    full-trajectory forward + whole-sequence segment backward.
"""
import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "Titans LMM fwd+bwd tokens/s (d=512, L=4096, 1 GPU); % of HBM/MFMA roofline"

# Published MI355X peaks used as roofline denominators.
PEAK_HBM_GBS = 8000.0
PEAK_FP32_TFLOPS = 157.3
PEAK_BF16_TFLOPS = 2500.0

# Algorithmic work per head-token at d=64 (fp32): forward 9 d^2 flop
# (M k, S update, M update, M q), backward 30 d^2 flop (one replay + reverse
# sweep); compulsory HBM bytes forward 1548, backward 2328.
D_HEAD = 64
FLOP_FWD = 9 * D_HEAD * D_HEAD
FLOP_BWD = 30 * D_HEAD * D_HEAD
# The checkpointed backward in chunk-parallel matrix form executes more than the token loop's 30 d^2: per 64-token
# chunk, in 64^3 products (2 * 64^3 flop each, block-sparse ones counted by the blocks they issue): chunk-local pass
# 15.6 (Gram and state products 4, (W.P)^T dY 1, blocked inverse 0.35, T R and T (m.K) 2.25, scan matrices 4, additive
# terms 4), gradient pass 15.75, adjoint scan 4.
EXACT_MM_PRODUCTS = {"ex_local_kernel": 15.6, "ex_grads_kernel": 15.75, "ex_scan_kernel": 4.0}
FLOP_EXACT_MM = {k: v * 2 * 64 ** 3 / 64 for k, v in EXACT_MM_PRODUCTS.items()}   # per head-token
FLOP_BWD_MM = sum(FLOP_EXACT_MM.values())
BYTES_FWD = 1548
BYTES_BWD = 2328


def make_inputs(B, s, d, seed):
    import torch
    g = torch.Generator(device="cpu").manual_seed(seed)
    rn = lambda *shape: torch.randn(*shape, generator=g, dtype=torch.float32)
    k, q, v, dy = rn(B, s, d), rn(B, s, d), rn(B, s, d), rn(B, s, d)
    k = k / k.norm(dim=-1, keepdim=True)
    q = q / q.norm(dim=-1, keepdim=True)
    alpha, theta, eta = (torch.sigmoid(rn(B, s)) for _ in range(3))
    x = dict(k=k, v=v, q=q, dy=dy, alpha=alpha, theta=theta, eta=eta,
             m0=torch.zeros(B, d, d), s0=torch.zeros(B, d, d))
    return {n: t.contiguous() for n, t in x.items()}


# HOPE self-referential memory, per head-token at d=64, counted on the update
# equations as the reference evaluates them: forward 54 d^2 flop (5 projections,
# read, and per memory: target, error, update), forward + backward 260 d^2.
FLOP_HOPE_FWD = 54 * D_HEAD * D_HEAD
FLOP_HOPE_BWD = 206 * D_HEAD * D_HEAD
# What the kernels execute per head-token (M_c,t = F_c G_t + H_t, self-generated values: H = 0), d = 64,
# chunks of 64.  Forward: 8 matrix-vector products (g = G x, p = G q, five with F_c g, y = F_mem p) 16 d^2,
# the rank-1 update of G 2 d^2, and M_c = F_c G_L for six memories once per chunk 12 d^3 / 64 = 12 d^2.
# Backward: sweep 15 d^2 on the vector units (w = dG k, z = dG^T u, dg from three F^T products, the rank-2
# update of dG), 8 d^2 of outer products into dF and 16 d^3 / 64 = 16 d^2 of chunk-boundary products on the
# fp32 matrix cores; the chunk-parallel kernels before and after it 14 d^2 + 3 d^2 on the matrix cores (their
# MOPS counters) and about 2 d^2 beside them.
FLOP_HOPE_EXEC_FWD = 30 * D_HEAD * D_HEAD
FLOP_HOPE_EXEC_BWD = 58 * D_HEAD * D_HEAD
BYTES_HOPE_FWD = 2 * 4 * D_HEAD + 6 * D_HEAD * D_HEAD * 4 // 64   # x, y; snapshots written once per 64 tokens
BYTES_HOPE_BWD = 2 * 4 * D_HEAD + 6 * D_HEAD * D_HEAD * 4 // 64   # dy, d_x; snapshots read


def cpu_baseline(x, heads, budget_s=12.0):
    """C restatement of the reference's Rust loops (oracle), one thread, on a
    bounded sample of the same inputs: whole batch elements (8 chains each)
    until the time budget is used."""
    from oracle import pyoracle as orc
    B, s, d = x["k"].shape
    npx = {n: t.numpy() for n, t in x.items()}
    done = 0
    t_start = time.perf_counter()
    while done < B:
        for b in range(done, done + heads):
            a = [npx[n][b] for n in ("k", "v", "q", "alpha", "theta", "eta")]
            y, ms, ss = orc.titans_forward(*a, npx["m0"][b], npx["s0"][b])
            orc.titans_backward(*a, ms, ss, npx["dy"][b])
        done += heads
        if time.perf_counter() - t_start > budget_s:
            break
    el = time.perf_counter() - t_start
    tokens = (done // heads) * s
    return {"value": tokens / el, "unit": "tokens/s", "cores": 1, "kind": "port",
            "sample": f"{done} of {B} chains ({done // heads} sequences of {s} tokens, all {heads} heads), "
                      f"full-trajectory forward + backward, {el:.1f} s"}


def host_threads():
    """Threads for the all-cores CPU leg: the host cores this process may use (the GPU boxes export
    their CPU share as OMP_NUM_THREADS)."""
    n = os.cpu_count() or 1
    try:
        n = min(n, int(os.environ.get("OMP_NUM_THREADS", n)))
    except ValueError:
        pass
    return max(1, n)


def cpu_all_cores(chain_fn, n_chains, seq_len, chains_per_token_row, what, budget_s=10.0):
    """The same oracle over whole chains on every host core: chains are independent, the oracle is a C
    library called through ctypes (the interpreter lock is released during a call), so a thread pool
    scales like the reference's loops would under a chain-parallel driver.  Chains are handed out until
    the time budget is used."""
    from concurrent.futures import ThreadPoolExecutor
    n_thr = host_threads()
    done = 0
    t_start = time.perf_counter()
    with ThreadPoolExecutor(n_thr) as pool:
        while done < n_chains and time.perf_counter() - t_start < budget_s:
            batch = list(range(done, min(n_chains, done + n_thr)))
            list(pool.map(chain_fn, batch))
            done += len(batch)
    el = time.perf_counter() - t_start
    return {"value": done * seq_len / chains_per_token_row / el, "unit": "tokens/s", "cores": n_thr, "kind": "port",
            "sample": f"{done} of {n_chains} chains of {seq_len} tokens ({chains_per_token_row} chains = one sequence "
                      f"of d=512), {what}, {n_thr} threads, {el:.1f} s"}


# Chunkwise (matrix form), per head-token at d=64, C=64: compulsory HBM bytes forward 1164
# (bf16 k,v,q, gates, fp32 y, chunk states), backward 1944; flops forward 57 344, backward ~143 k.
BYTES_CW_FWD, BYTES_CW_BWD = 1164, 1944
FLOP_CW_FWD, FLOP_CW_BWD = 57344, 143360


def cpu_baseline_chunkwise(x, C, budget_s=12.0):
    """Oracle of the frozen-M0 chunkwise rule, one thread, whole chains until the budget is used."""
    from oracle import pyoracle as orc
    B, s, d = x["k"].shape
    npx = {n: t.float().numpy() for n, t in x.items()}
    done = 0
    t_start = time.perf_counter()
    while done < B and time.perf_counter() - t_start < budget_s:
        a = [npx[n][done] for n in ("k", "v", "q", "alpha", "theta", "eta")]
        y, mc, sc = orc.chunkwise_forward(*a, npx["m0"][done], npx["s0"][done], C, True)
        orc.chunkwise_backward(*a, mc, sc, npx["dy"][done], C, True)
        done += 1
    el = time.perf_counter() - t_start
    return {"value": done * s / 8 / el, "unit": "tokens/s", "cores": 1, "kind": "port",
            "sample": f"{done} of {B} chains of {s} tokens (8 chains = one sequence of d=512), chunkwise "
                      f"forward + backward, {el:.1f} s"}


def cpu_baseline_hope(mems, x, dy, C, budget_s=12.0):
    """Same oracle, HOPE path: whole chains until the time budget is used."""
    from oracle import pyoracle as orc
    B, s, d = x.shape
    done = 0
    t_start = time.perf_counter()
    while done < B and time.perf_counter() - t_start < budget_s:
        _, _, c = orc.selfref_forward(mems[done].numpy(), x[done].numpy(), C, True)
        orc.selfref_backward(c, dy[done].numpy())
        done += 1
    el = time.perf_counter() - t_start
    return {"value": done * s / 8 / el, "unit": "tokens/s", "cores": 1, "kind": "port",
            "sample": f"{done} of {B} chains of {s} tokens (8 chains = one sequence of d=512), "
                      f"forward + backward, {el:.1f} s"}


def setup_titans_exact_c2(torch, D, lib, m_norm_max=None):
    """m_norm_max: None = no bound (the largest float, as BASELINE configs[1] states it); a number = the bound the
    reference's shipped configurations pass (cli/configs/gear1_d1024_gpu1.json:14 has 100)."""
    bs, heads, d, s, C = 8, 8, 64, 2048, 64
    B = bs * heads
    x = make_inputs(B, s, d, 0x5EED0002)
    dv = {n: t.cuda() for n, t in x.items()}
    n_ck = 1 + sum(1 for t in range(s) if (t + 1) % C == 0 or t + 1 == s)
    z = lambda *shape: torch.zeros(*shape, dtype=torch.float32, device="cuda")
    mc, sc, y = z(B, n_ck, d, d), z(B, n_ck, d, d), z(B, s, d)
    g = dict(dk=z(B, s, d), dv=z(B, s, d), dq=z(B, s, d), da=z(B, s), dt=z(B, s), de=z(B, s),
             dm=z(d, d), ds=z(d, d))
    F32_MAX = float(np.finfo(np.float32).max) if m_norm_max is None else float(m_norm_max)

    def fwd():
        D.call("titans_forward_ckpt_batched_f32_rocm", dv["k"], dv["v"], dv["q"], dv["alpha"],
               dv["theta"], dv["eta"], dv["m0"], dv["s0"], mc, sc, y, s, d, B, C, 0.0, F32_MAX)

    def bwd():
        D.call("titans_backward_ckpt_f32_rocm", dv["k"], dv["v"], dv["q"], dv["alpha"], dv["theta"],
               dv["eta"], mc, sc, dv["dy"], g["dk"], g["dv"], g["dq"], g["da"], g["dt"], g["de"],
               g["dm"], g["ds"], s, d, B, C, 0.0, F32_MAX)

    def chain(b):
        from oracle import pyoracle as orc
        a = [x[n][b].numpy() for n in ("k", "v", "q", "alpha", "theta", "eta")]
        y, ms, ss = orc.titans_forward(*a, x["m0"][b].numpy(), x["s0"][b].numpy())
        orc.titans_backward(*a, ms, ss, x["dy"][b].numpy())

    return dict(
        fwd=fwd, bwd=bwd, tokens=bs * s, head_tokens=B * s,
        # the backward runs in chunk-parallel matrix form (csrc/exact_mm.hip): roofline.frac is priced on the flops its
        # kernels execute, the figure on the token loop's count sits beside it (on_reference_flops)
        flop_fwd=FLOP_FWD, flop_bwd=FLOP_BWD_MM, flop_ref_fwd=FLOP_FWD, flop_ref_bwd=FLOP_BWD,
        bytes_fwd=BYTES_FWD, bytes_bwd=BYTES_BWD,
        # flops per head-token that each instrumented kernel executes
        kernel_work=dict(FLOP_EXACT_MM, rule_fwd_kernel=FLOP_FWD, rule_bwd_fused_kernel=FLOP_BWD),
        kernel_names={"forward": "forward_ckpt", "backward": "backward_ckpt_matrix_form"},
        cpu_all=lambda: cpu_all_cores(chain, B, s, heads, "full-trajectory forward + backward"),
        config={"workload": "BASELINE configs[1]: Titans LMM exact recurrence, 8 heads x 64 (d=512), "
                            "batch 8, seq 2048, fp32 state, checkpoints every 64 tokens, fwd+bwd" +
                            ("" if m_norm_max is None else f", m_norm_max = {m_norm_max:g} (never reached)"),
                "batch": bs, "heads": heads, "head_dim": d, "seq_len": s, "checkpoint_interval": C},
        cpu=lambda: cpu_baseline(x, heads))


def setup_titans_chunkwise_c3(torch, D, lib, mode="bf16"):
    """mode: "bf16" (the bf16 pair), "bf16_mnorm" (the same through the entry points that take the reference's
    error_clip / m_norm_max, with m_norm_max = 100 as cli/configs/gear1_d1024_gpu1.json ships it), "f32_mnorm"
    (float tokens through the reference-named symbols titans_chunkwise_*_f32_cuda with m_norm_max = 100)."""
    bs, heads, d, s, C = 16, 8, 64, 4096, 64
    B = bs * heads
    x = make_inputs(B, s, d, 0x5EED0003)
    for n in ("k", "v", "q"):
        x[n] = x[n].to(torch.bfloat16)
        if mode == "f32_mnorm":
            x[n] = x[n].to(torch.float32)
    dv = {n: t.cuda() for n, t in x.items()}
    mnorm = 100.0
    nc = s // C
    z = lambda *shape: torch.zeros(*shape, dtype=torch.float32, device="cuda")
    mc, sc, y = z(B, nc + 1, d, d), z(B, nc + 1, d, d), z(B, s, d)
    g = dict(dk=z(B, s, d), dv=z(B, s, d), dq=z(B, s, d), da=z(B, s), dt=z(B, s), de=z(B, s),
             dm=z(d, d), ds=z(d, d))

    tail = () if mode == "bf16" else (0.0, mnorm)
    f_name, b_name = {"bf16": ("titans_chunkwise_forward_bf16_rocm", "titans_chunkwise_backward_bf16_rocm"),
                      "bf16_mnorm": ("titans_chunkwise_forward_bf16_guarded_rocm", "titans_chunkwise_backward_bf16_guarded_rocm"),
                      "f32_mnorm": ("titans_chunkwise_forward_f32_cuda", "titans_chunkwise_backward_f32_cuda")}[mode]

    def fwd():
        D.call(f_name, dv["k"], dv["v"], dv["q"], dv["alpha"], dv["theta"],
               dv["eta"], dv["m0"], dv["s0"], mc, sc, y, s, d, B, C, *tail)

    def bwd():
        D.call(b_name, dv["k"], dv["v"], dv["q"], dv["alpha"], dv["theta"],
               dv["eta"], mc, sc, dv["dy"], g["dk"], g["dv"], g["dq"], g["da"], g["dt"], g["de"],
               g["dm"], g["ds"], s, d, B, C, *tail)

    def chain(b):
        from oracle import pyoracle as orc
        a = [x[n][b].float().numpy() for n in ("k", "v", "q", "alpha", "theta", "eta")]
        y, mco, sco = orc.chunkwise_forward(*a, x["m0"][b].numpy(), x["s0"][b].numpy(), C, True)
        orc.chunkwise_backward(*a, mco, sco, x["dy"][b].numpy(), C, True)

    what = {"bf16": "bf16 k/v/q with fp32 accumulate and fp32 M/S, fwd+bwd",
            "bf16_mnorm": "bf16 k/v/q with fp32 accumulate and fp32 M/S, fwd+bwd, through the entry points that take the "
                          "reference's couplings, m_norm_max = 100 (never reached: the matrix form serves the call behind a "
                          "device-side test, one stream synchronisation per direction)",
            "f32_mnorm": "float k/v/q through the reference-named symbols titans_chunkwise_{forward,backward}_f32_cuda with "
                         "m_norm_max = 100 (never reached: the fp32 matrix form serves the call behind a device-side test)"}[mode]
    return dict(
        fwd=fwd, bwd=bwd, tokens=bs * s, head_tokens=B * s, bound="hbm", dtype="bf16" if mode != "f32_mnorm" else "f32",
        flop_fwd=FLOP_CW_FWD, flop_bwd=FLOP_CW_BWD, bytes_fwd=BYTES_CW_FWD, bytes_bwd=BYTES_CW_BWD,
        matrix="bf16_matrix", matrix_peak=PEAK_BF16_TFLOPS,
        # each kernel's OWN compulsory bytes per head-token (what it must read and write given its role in
        # the split; intermediates between kernels count for both sides, so these do not add up to 3108):
        #   forward chain: the forward's 1164
        #   adjoint scan: k, q 256 + dY 256 + gates 12 + adjoint snapshots (bf16) 2 x 8192 / 64
        #   gradients: k, v, q 384 + dY 256 + gates 12 + states 512 + adjoints (bf16) 256 + d_k, d_v, d_q 768
        #              + d_theta 4 + per-token terms for the gate pass 256 + 16
        #   gate sweeps: those 256 + 16, gates 8, d_alpha, d_eta 8
        kernel_work={"cw_chain_fwd_kernel": BYTES_CW_FWD, "cw_adjoint_chain_kernel": 780,
                     "cw_grads_bf16_kernel": 2464, "cw_gates_sweep_kernel": 288},
        kernel_names={"forward": "chunkwise_forward_bf16", "backward": "chunkwise_backward_bf16"},
        cpu_all=lambda: cpu_all_cores(chain, B, s, heads, "chunkwise forward + backward"),
        config={"workload": "BASELINE configs[2]: Titans LMM chunkwise training, chunk 64, 8 heads x 64 (d=512), "
                            "batch 16, seq 4096, " + what,
                "batch": bs, "heads": heads, "head_dim": d, "seq_len": s, "chunk_size": C},
        cpu=lambda: cpu_baseline_chunkwise(x, C))


# SWA per head-token at window 512, hd 64: forward 4*ws*hd flop, backward ~2.5x; compulsory bytes
# bf16 q,k,v,out 512 + weights 2*1024 + fp32 d_out,dq,dk,dv 1024.
FLOP_SWA_FWD, FLOP_SWA_BWD = 4 * 512 * 64, 10 * 512 * 64
BYTES_SWA_FWD = 4 * 128 + 1024           # q, k, v in, out and the weights out
BYTES_SWA_BWD = 3 * 128 + 1024 + 4 * 256


def cpu_baseline_swa(q, k, v, d_out, window, heads, budget_s=12.0):
    """Oracle SWA forward + backward, one thread, on leading tokens of one sequence."""
    from oracle import pyoracle as orc
    n = 512
    bits = lambda t: t[:1, :n].contiguous().view(__import__("torch").uint16).numpy()
    t_start = time.perf_counter()
    reps = 0
    while time.perf_counter() - t_start < budget_s:
        out, aw = orc.swa_forward(bits(q), bits(k), bits(v), window, heads, 0)
        orc.swa_backward(bits(q), bits(k), bits(v), aw, d_out[:1, :n].numpy(), window, heads, 0)
        reps += 1
    el = time.perf_counter() - t_start
    return {"value": reps * n / el, "unit": "tokens/s", "cores": 1, "kind": "port",
            "sample": f"{reps} x the first {n} tokens of one sequence (all {heads} heads; windows are partly "
                      f"filled, so this overstates the CPU rate), forward + backward, {el:.1f} s"}


def setup_swa_c5(torch, D, lib, lse=False, heads=8, hd=64):
    bs, s, window = 8, 4096, 512
    td = heads * hd
    g = torch.Generator(device="cpu").manual_seed(0x5EED0005)
    q, k, v = (torch.randn(bs, s, td, generator=g).to(torch.bfloat16) for _ in range(3))
    d_out = torch.randn(bs, s, td, generator=g)
    qd, kd, vd, dod = q.cuda(), k.cuda(), v.cuda(), d_out.cuda()
    out = torch.zeros(bs, s, td, dtype=torch.bfloat16, device="cuda")
    aw = torch.zeros(bs, heads, s, window, dtype=torch.bfloat16, device="cuda")
    dq, dk, dv = (torch.zeros(bs, s, td, dtype=torch.float32, device="cuda") for _ in range(3))

    stats = torch.zeros(bs, heads, s, 2, dtype=torch.float32, device="cuda")

    def fwd():
        if lse:
            D.call("swa_forward_lse_bf16_rocm", qd, kd, vd, out, stats, s, heads, hd, window, bs)
        else:
            D.call("swa_forward_f32_cuda", qd, kd, vd, out, aw, s, heads, hd, window, bs, 0)

    def bwd():
        dk.zero_(); dv.zero_()
        if lse:
            D.call("swa_backward_lse_bf16_rocm", qd, kd, vd, stats, dod, dq, dk, dv, s, heads, hd, window, bs)
        else:
            D.call("swa_backward_f32_cuda", qd, kd, vd, aw, dod, dq, dk, dv, s, heads, hd, window, bs, 0)

    # the statistics pair moves 8 bytes per head-token where the contract pair moves the 1024-byte weight row
    wbytes = 8 if lse else 1024
    return dict(
        fwd=fwd, bwd=bwd, tokens=bs * s, head_tokens=bs * heads * s, bound="hbm", dtype="bf16",
        flop_fwd=4 * window * hd, flop_bwd=10 * window * hd + (4 * window * hd if lse else 0),
        bytes_fwd=4 * 2 * hd + wbytes, bytes_bwd=3 * 2 * hd + wbytes + 4 * 4 * hd,
        matrix="bf16_matrix", matrix_peak=PEAK_BF16_TFLOPS,
        kernel_names={"forward": "swa_forward", "backward": "swa_backward"},
        config={"workload": f"BASELINE configs[4], attention branch: sliding-window attention, window 512, {heads} heads x {hd}, "
                            "bf16 storage with fp32 softmax, batch 8, seq 4096, fwd+bwd"
                            + (", per-query softmax statistics kept instead of the weight tensor" if lse else ""),
                "batch": bs, "heads": heads, "head_dim": hd, "seq_len": s, "window": window},
        cpu=lambda: cpu_baseline_swa(q, k, v, d_out, window, heads))


def cpu_baseline_mag_layer(bs, s, d, heads, k, window):
    """The layer's CPU cost as the sum of its parts, each on a bounded sample, one thread: the chunkwise
    rule (oracle, k levels x heads chains), sliding-window attention (oracle), the dense projections
    (numpy fp32 GEMMs held to one BLAS thread) and AdamW (oracle) amortised over the step's tokens.
    The glue between them (row norms, gate dot products, head transposes) is left out: the figure
    overstates the CPU rate."""
    import torch
    from threadpoolctl import threadpool_limits
    from oracle import pyoracle as orc
    hd, C, n = d // heads, 64, 1024
    xin = make_inputs(k * heads, n, hd, 0x5EED0009)
    npx = {nm: t.numpy() for nm, t in xin.items()}
    t0 = time.perf_counter()
    for b in range(k * heads):
        a = [npx[nm][b] for nm in ("k", "v", "q", "alpha", "theta", "eta")]
        y, mc, sc = orc.chunkwise_forward(*a, npx["m0"][b], npx["s0"][b], C, True)
        orc.chunkwise_backward(*a, mc, sc, npx["dy"][b], C, True)
    t_rule = (time.perf_counter() - t0) / n
    g = torch.Generator(device="cpu").manual_seed(0x5EED000A)
    ns = 1024
    q, kk, v = (torch.randn(1, ns, d, generator=g).to(torch.bfloat16).view(torch.uint16).numpy() for _ in range(3))
    do = torch.randn(1, ns, d, generator=g).numpy()
    t0 = time.perf_counter()
    out, aw = orc.swa_forward(q, kk, v, window, heads, 0)
    orc.swa_backward(q, kk, v, aw, do, window, heads, 0)
    t_swa = (time.perf_counter() - t0) / ns
    rs = np.random.default_rng(5)
    xm, wm = rs.standard_normal((n, d), dtype=np.float32), rs.standard_normal((d, d), dtype=np.float32)
    n_proj = 3 + 3 * k + 1            # q, k, v, per level k, v, q, and W_o
    with threadpool_limits(limits=1):
        t0 = time.perf_counter()
        for _ in range(n_proj):
            yv = xm @ wm.T            # forward
            _ = yv @ wm               # input gradient
            _ = yv.T @ xm             # weight gradient
        t_proj = (time.perf_counter() - t0) / n
    n_par = (4 + 3 * k) * d * d + 3 * k * (2 * d + 1)
    w, gr, m, vv = (rs.standard_normal(n_par, dtype=np.float32) for _ in range(4))
    vv = np.abs(vv)
    t0 = time.perf_counter()
    orc.grad_norm_clip([gr], 1.0)
    orc.adamw_step(w, gr, m, vv, 3e-4, 0.9, 0.95, 1e-8, 10.0, 20.0, 0.1)
    t_opt = (time.perf_counter() - t0) / (bs * s)
    per_token = t_rule + t_swa + t_proj + t_opt
    return {"value": 1.0 / per_token, "unit": "tokens/s", "cores": 1, "kind": "port",
            "sample": f"sum of parts per token: chunkwise rule {k} levels x {heads} heads on {n} tokens "
                      f"({t_rule * 1e6:.0f} us/token), attention on {ns} tokens ({t_swa * 1e6:.0f}), {n_proj} projection "
                      f"GEMM triples on {n} tokens ({t_proj * 1e6:.0f}), AdamW over {n_par} parameters per step of "
                      f"{bs * s} tokens ({t_opt * 1e6:.1f}); glue kernels not counted"}


def setup_mag_layer_c5(torch, D, lib, precision="bf16x3"):
    from nl_hecate_amd.mag_layer import MagLayer, MagTrainer
    bs, heads, d, s, k, window = 8, 8, 512, 4096, 4, 512
    layer = MagLayer(d, heads, k, window, [1, 8, 64, 512], rule="chunkwise", chunk=64, seed=0x5EED0007,
                     precision=precision)
    tr = MagTrainer(layer, lr=3e-4, beta1=0.9, beta2=0.95, weight_decay=0.1)
    g = torch.Generator(device="cpu").manual_seed(0x5EED0008)
    x = (torch.randn(bs, s, d, generator=g) / d ** 0.5).cuda()
    d_out = torch.randn(bs, s, d, generator=g).cuda()
    st = {}

    def fwd():
        st["out"], st["cache"] = layer.forward(x)

    def bwd():
        layer.backward(st["cache"], d_out, tr.grads)
        tr.opt.step(st["cache"]["pulse"], tr.lr, tr.max_grad_norm, tr.scale)

    # the timed step replays forward + backward from a HIP graph (the eager pair above, some 330
    # launches, is launch-bound on the host) and runs AdamW eagerly
    # (the synthetic batch is written once into the buffers the graph reads, as a device-side producer would do
    # every step: no copy of the inputs inside the timed step)
    def step():
        bufs = tr.graph_inputs(x.shape)
        if bufs is None:
            tr.step_graphed(x, d_out)
        else:
            if "static" not in st:
                bufs[0].copy_(x)
                bufs[1].copy_(d_out)
                st["static"] = True
            tr.step_graphed(*bufs)

    # per token: 4 levels x 8 heads x chunkwise memory + 8 heads x SWA (algorithmic bytes / flops of the parts)
    return dict(
        fwd=fwd, bwd=bwd, step=step, tokens=bs * s, head_tokens=bs * s, bound="hbm", dtype="bf16",
        flop_fwd=4 * 8 * FLOP_CW_FWD + 8 * FLOP_SWA_FWD, flop_bwd=4 * 8 * FLOP_CW_BWD + 8 * FLOP_SWA_BWD,
        bytes_fwd=4 * 8 * BYTES_CW_FWD + 8 * BYTES_SWA_FWD, bytes_bwd=4 * 8 * BYTES_CW_BWD + 8 * BYTES_SWA_BWD,
        step_eager=lambda: (fwd(), bwd()),
        kernel_names={"forward": "layer_forward", "backward": "layer_backward_and_adamw"},
        config={"workload": "BASELINE configs[4]: full layer, CMS k=4 Titans levels at periods [1,8,64,512] (chunkwise "
                            "rule, chunk 64, bf16 k/v/q) with MAG sigmoid gating over sliding-window attention "
                            "(window 512, bf16, fp32 softmax), 8 heads x 64 (d=512), batch 8, seq 4096, x ~ N(0,1/d), "
                            "Xavier weights; forward + backward (replayed from a HIP graph) + AdamW (lr 3e-4, betas "
                            "0.9/0.95, wd 0.1); " + (
                                "projections: x and the weights rounded once to bf16, fp32 accumulation (own MFMA kernel with "
                                "the norm / gate / head-split epilogue forward, library GEMMs backward), every step a call "
                                "into the C ABI" if precision == "bf16" else
                                "projections: hi + lo bf16 splits, three products per GEMM (fp32-grade), library GEMMs"),
                "batch": bs, "heads": heads, "d_model": d, "seq_len": s, "levels": k, "window": window},
        cpu=lambda: cpu_baseline_mag_layer(bs, s, d, heads, k, window))


def cpu_baseline_adamw(tensors, budget_s=12.0):
    from oracle import pyoracle as orc
    host = [(w.cpu().numpy().copy(), g.cpu().numpy(), m.cpu().numpy().copy(), v.cpu().numpy().copy())
            for w, g, m, v in tensors]
    n = sum(w.size for w, _, _, _ in host)
    t_start = time.perf_counter()
    reps = 0
    while time.perf_counter() - t_start < budget_s:
        orc.grad_norm_clip([g for _, g, _, _ in host], 1.0)
        for w, g, m, v in host:
            orc.adamw_step(w, g, m, v, 3e-4, 0.9, 0.95, 1e-8, 10.0, 20.0, 0.1)
        reps += 1
    el = time.perf_counter() - t_start
    return {"value": reps * n / el, "unit": "params/s", "cores": 1, "kind": "port",
            "sample": f"{reps} optimizer steps over all {n} parameters (clip + update), {el:.1f} s"}


def setup_adamw_c5(torch, D, lib):
    from nl_hecate_amd.cms import FrequencyAwareAdamW, Pulse
    d, k = 512, 4
    g = torch.Generator(device="cpu").manual_seed(0x5EED0006)
    opt = FrequencyAwareAdamW(k, 0.9, 0.95, 1e-8, 0.1)
    tensors = []

    def add(group, *shape):
        w = (torch.randn(*shape, generator=g) * 0.02).cuda()
        gr = torch.randn(*shape, generator=g).cuda()
        m, v = torch.zeros_like(w), torch.zeros_like(w)
        opt.add_tensor(group, w, gr, m, v)
        tensors.append((w, gr, m, v))

    for _ in range(4):                # attention branch: W_q, W_k, W_v, W_o
        add(-1, d, d)
    for level in range(k):            # per level: three memory projections, three gate vectors + biases
        for _ in range(3):
            add(level, d, d)
        for _ in range(3):
            add(level, 2 * d)
            add(level, 1)
    n = sum(w.numel() for w, _, _, _ in tensors)
    pulse = Pulse(0, [True] * k)
    scale = torch.zeros(2, dtype=torch.float32, device="cuda")

    def fwd():
        pass

    def bwd():
        opt.step(pulse, 3e-4, 1.0, scale)

    return dict(
        fwd=fwd, bwd=bwd, tokens=n, head_tokens=n, bound="hbm", dtype="f32", unit="params/s",
        flop_fwd=0, flop_bwd=12, bytes_fwd=0, bytes_bwd=28,
        kernel_names={"forward": "none", "backward": "adamw_step"},
        config={"workload": "BASELINE configs[4], optimizer step: frequency-aware AdamW (lr 3e-4, betas 0.9/0.95, wd 0.1) "
                            "with gradient-norm clip over the layer's parameters, d=512, k=4 levels, all firing",
                "parameters": n, "tensors": len(tensors)},
        cpu=lambda: cpu_baseline_adamw(tensors))


def setup_hope_selfref_c4(torch, D, lib):
    from nl_hecate_amd import selfref as SR
    bs, heads, d, s, C = 8, 8, 64, 2048, 64
    B = bs * heads
    g = torch.Generator(device="cpu").manual_seed(0x5EED0004)
    lim = (6.0 / (2 * d)) ** 0.5
    mems = (torch.rand(B, 6, d, d, generator=g) * 2 - 1) * lim
    mems[:, 5] = 0.0
    x = torch.randn(B, s, d, generator=g) / (heads * d) ** 0.5
    dy = torch.randn(B, s, d, generator=g)
    m0, xd, dyd = mems.cuda(), x.cuda(), dy.cuda()
    st = {}

    def fwd():
        m = m0.clone()
        st["y"], st["cache"] = SR.chunkwise_self_ref_step(m, xd, C, True)

    def bwd():
        st["g"] = SR.chunkwise_self_ref_step_backward(st["cache"], dyd)

    return dict(
        fwd=fwd, bwd=bwd, tokens=bs * s, head_tokens=B * s,
        # the roofline is priced on the flops the kernels execute; the count on the reference's update
        # equations (1.8x / 3.6x more) is reported beside it
        flop_fwd=FLOP_HOPE_EXEC_FWD, flop_bwd=FLOP_HOPE_EXEC_BWD, bytes_fwd=BYTES_HOPE_FWD, bytes_bwd=BYTES_HOPE_BWD,
        flop_ref_fwd=FLOP_HOPE_FWD, flop_ref_bwd=FLOP_HOPE_BWD,
        kernel_names={"forward": "selfref_forward", "backward": "selfref_backward"},
        config={"workload": "BASELINE configs[3]: HOPE self-referential memory, 8 heads x 64 (d=512), "
                            "batch 8, seq 2048, fp32, self-generated values, frozen snapshots per 64 tokens, fwd+bwd.  With the "
                            "configuration's inputs (x ~ N(0, 1/d), M_mem = 0) the decay gate sits at 1/2, every memory is "
                            "exactly zero in fp32 after about 150 tokens and y = 0 throughout; the timing does not depend on "
                            "the values, and the full-size value test uses engineered non-degenerate memories instead",
                "batch": bs, "heads": heads, "head_dim": d, "seq_len": s, "chunk_size": C},
        cpu=lambda: cpu_baseline_hope(mems, x, dy, C))


# Hebbian rule, per head-token at d=64 with the full trajectory the contract asks for: forward
# k,v,q 768 + alpha 4 + y 256 + M_{t+1} 16 384 = 17 412 B, 6 d^2 flop; backward k,v,q,dY 1024 + alpha 4 +
# grads 772 + the states the chunk-parallel form needs (one per 64 tokens: 16 384 / 64 = 256) = 2 056 B
# (the reference's sequential backward reads M_t per token: 18 184 B), 12 d^2 flop.
BYTES_HEB_FWD, BYTES_HEB_BWD = 17412, 2056
FLOP_HEB_FWD, FLOP_HEB_BWD = 6 * 64 * 64, 12 * 64 * 64


def cpu_baseline_hebbian(x, heads, budget_s=12.0):
    """Oracle of the Hebbian rule (dispatch.rs:1566-1660), one thread, whole sequences until the budget is used."""
    from oracle import pyoracle as orc
    B, s, d = x["k"].shape
    npx = {n: t.numpy() for n, t in x.items()}
    done = 0
    t_start = time.perf_counter()
    while done < B and time.perf_counter() - t_start < budget_s:
        for b in range(done, done + heads):
            a = [npx[n][b] for n in ("k", "v", "q", "alpha")]
            y, ms = orc.hebbian_forward(*a, npx["m0"][b])
            orc.hebbian_backward(*a, ms, npx["dy"][b])
        done += heads
    el = time.perf_counter() - t_start
    return {"value": (done // heads) * s / el, "unit": "tokens/s", "cores": 1, "kind": "port",
            "sample": f"{done} of {B} chains ({done // heads} sequences of {s} tokens, all {heads} heads), "
                      f"full-trajectory forward + backward, {el:.1f} s"}


def setup_hebbian_c2(torch, D, lib):
    bs, heads, d, s = 8, 8, 64, 2048
    B = bs * heads
    x = make_inputs(B, s, d, 0x5EED0006)
    dv = {n: t.cuda() for n, t in x.items()}
    z = lambda *shape: torch.zeros(*shape, dtype=torch.float32, device="cuda")
    ms, y = z(B, s + 1, d, d), z(B, s, d)
    g = dict(dk=z(B, s, d), dv=z(B, s, d), dq=z(B, s, d), da=z(B, s), dm=z(B, d, d), seed=z(B, d, d))

    def fwd():
        D.hebbian_forward_dd(dv["k"], dv["v"], dv["q"], dv["alpha"], dv["m0"], ms, y, s, d, B, s, d * d)

    def bwd():
        D.hebbian_backward_dd_segment(dv["k"], dv["v"], dv["q"], dv["alpha"], ms, dv["dy"], g["seed"],
                                      g["dk"], g["dv"], g["dq"], g["da"], g["dm"], 0, s, d, B, s)

    return dict(
        fwd=fwd, bwd=bwd, tokens=bs * s, head_tokens=B * s, bound="hbm",
        flop_fwd=FLOP_HEB_FWD, flop_bwd=FLOP_HEB_BWD, bytes_fwd=BYTES_HEB_FWD, bytes_bwd=BYTES_HEB_BWD,
        kernel_names={"forward": "hebbian_forward", "backward": "hebbian_backward_segment"},
        config={"workload": "Hebbian rule at the shape of BASELINE configs[1]: 8 heads x 64 (d=512), batch 8, "
                            "seq 2048, fp32, full M trajectory, forward + whole-sequence segment backward",
                "batch": bs, "heads": heads, "head_dim": d, "seq_len": s},
        cpu=lambda: cpu_baseline_hebbian(x, heads))


WORKLOADS = {"titans_chunkwise_c3": setup_titans_chunkwise_c3, "titans_exact_c2": setup_titans_exact_c2,
             "hope_selfref_c4": setup_hope_selfref_c4, "swa_c5": setup_swa_c5,
             "swa_stats_c5": lambda torch, D, lib: setup_swa_c5(torch, D, lib, lse=True),
             "swa_c5_hd32": lambda torch, D, lib: setup_swa_c5(torch, D, lib, heads=16, hd=32),
             "swa_stats_c5_hd32": lambda torch, D, lib: setup_swa_c5(torch, D, lib, lse=True, heads=16, hd=32),
             "adamw_c5": setup_adamw_c5, "hebbian_c2": setup_hebbian_c2,
             "mag_layer_c5": lambda torch, D, lib: setup_mag_layer_c5(torch, D, lib, precision="bf16"),
             "mag_layer_c5_bf16x3": lambda torch, D, lib: setup_mag_layer_c5(torch, D, lib, precision="bf16x3"),
             "hbm_copy": None, "mfma_peak": None,
             "titans_chunkwise_c3_mnorm": lambda torch, D, lib: setup_titans_chunkwise_c3(torch, D, lib, mode="bf16_mnorm"),
             "titans_chunkwise_c3_f32_mnorm": lambda torch, D, lib: setup_titans_chunkwise_c3(torch, D, lib, mode="f32_mnorm"),
             "titans_exact_c2_mnorm": lambda torch, D, lib: setup_titans_exact_c2(torch, D, lib, m_norm_max=100.0)}


# The kernel sources each workload's launches come from: a traffic profile is stamped with a hash of THESE files
# (and the headers they include), so an edit elsewhere in the library does not make it look stale, and an edit
# here does until the profile is measured again.
_CW_BF16 = ["chunkwise_chain.hip", "chunkwise_adjoint.hip", "chunkwise_grads.hip", "chunkwise_gates.hip", "chunkwise_mm.hip"]
_SWA = ["swa_mfma.hip", "swa.hip"]
WORKLOAD_SOURCES = {
    "titans_chunkwise_c3": _CW_BF16,
    "titans_chunkwise_c3_mnorm": _CW_BF16 + ["chunkwise_guard.hip"],
    "titans_chunkwise_c3_f32_mnorm": ["chunkwise_mm.hip", "chunkwise_gates.hip", "chunkwise_guard.hip", "memory_rules.hip"],
    "titans_exact_c2": ["memory_rules.hip", "exact_mm.hip", "chunkwise_gates.hip"],
    "titans_exact_c2_mnorm": ["memory_rules.hip", "exact_mm.hip", "chunkwise_gates.hip", "chunkwise_guard.hip"],
    "hope_selfref_c4": ["selfref.hip"],
    "swa_c5": _SWA, "swa_stats_c5": _SWA, "swa_c5_hd32": _SWA, "swa_stats_c5_hd32": _SWA,
    "adamw_c5": ["optim.hip", "cms.hip"],
    "hebbian_c2": ["hebbian.hip"],
    "mag_layer_c5": _CW_BF16 + _SWA + ["level_step.hip", "layer_glue.hip", "cms.hip", "optim.hip"],
    "mag_layer_c5_bf16x3": _CW_BF16 + _SWA + ["layer_glue.hip", "cms.hip", "optim.hip", "elementwise.hip"],
    "hbm_copy": ["roof_probes.hip"], "mfma_peak": ["roof_probes.hip"],
}


def workload_files(workload):
    """The kernel sources of a workload and the library headers they include, directly or through one another
    (the C ABI header is left out: a new declaration changes no kernel)."""
    import re
    csrc = os.path.join(ROOT, "nl_hecate_amd", "csrc")
    todo, seen = list(WORKLOAD_SOURCES[workload]), []
    while todo:
        f = todo.pop()
        if f in seen or not os.path.exists(os.path.join(csrc, f)):
            continue
        seen.append(f)
        todo += re.findall(r'#include "([A-Za-z0-9_]+\.h)"', open(os.path.join(csrc, f)).read())
    return sorted(seen)


def source_hash(workload):
    """sha256 over the kernel sources of a workload and the headers they include."""
    import hashlib
    h = hashlib.sha256()
    for f in workload_files(workload):
        h.update(f.encode())
        h.update(open(os.path.join(ROOT, "nl_hecate_amd", "csrc", f), "rb").read())
    return h.hexdigest()


def git_head():
    import subprocess
    try:
        return subprocess.check_output(["git", "-C", ROOT, "rev-parse", "--short=12", "HEAD"],
                                       stderr=subprocess.DEVNULL).decode().strip()
    except Exception:
        return None


def profile_sidecar(workload):
    """profiles/<workload>.json, written by `bench.py --write-profile` from rocprofv3 counter runs:
    per-kernel FETCH_SIZE / WRITE_SIZE bytes per launch, stamped with the sources they were measured on."""
    path = os.path.join(ROOT, "profiles", workload + ".json")
    if not os.path.exists(path):
        return None
    with open(path) as f:
        return json.load(f)


def short_kernel_name(n):
    n = n.replace("void ", "").replace("nlh::(anonymous namespace)::", "").replace("nlh::", "")
    return n.split("(")[0]


def write_profile(workload, raw):
    """Summarise the rocprofv3 runs found under `raw` (trace_<w>/, pmc_FETCH_SIZE_<w>/, pmc_WRITE_SIZE_<w>/,
    pmc_FETCH_SIZE_calib/, pmc_WRITE_SIZE_calib/, optional pmc_MFMA_<w>/) into
    profiles/<workload>_kernels_and_hbm_traffic.txt and the sidecar profiles/<workload>.json."""
    import collections
    import csv
    import glob

    def find(sub, name):
        hits = glob.glob(os.path.join(raw, sub, "**", name), recursive=True)
        if not hits:
            sys.exit(f"--write-profile: {name} not found under {os.path.join(raw, sub)}")
        return hits[0]

    def pmc(path):
        agg = collections.defaultdict(lambda: [0, 0.0])
        for row in csv.DictReader(open(path)):
            k = (row["Kernel_Name"], row["Counter_Name"])
            agg[k][0] += 1
            agg[k][1] += float(row["Counter_Value"])
        return {k: v / n for k, (n, v) in agg.items()}

    if workload in ("hbm_copy", "mfma_peak"):
        # the probes: the kernel trace and the line bench.py printed in the same session (<raw>/bench_<workload>.json)
        stats = list(csv.DictReader(open(find("trace_" + workload, "t_kernel_stats.csv"))))
        cmd = f"python3 bench.py --workload {workload}"
        lines = [f"{workload}: what the probe kernels (csrc/roof_probes.hip) sustain on one MI355X (rocprofv3, ROCm 7.2)", "",
                 f"commands (from /tmp, TMPDIR=/tmp): {cmd} > <out>/bench_{workload}.json; rocprofv3 --kernel-trace --stats "
                 f"--output-format csv -d <out>/trace_{workload} -o t -- {cmd}", "",
                 f"sources: git {git_head()}, sha256 of {', '.join('csrc/' + f for f in workload_files(workload))} "
                 f"{source_hash(workload)[:16]}", "",
                 f"{'probe':44s} {'ms':>9s} {'achieved':>10s} {'unit':>8s} {'of data-sheet peak':>19s}"]
        res = json.load(open(os.path.join(raw, f"bench_{workload}.json")))
        for pr in res["probes"]:
            nm = pr["name"] + (f", {pr['waves_per_simd']} wave(s) per SIMD" if "waves_per_simd" in pr else "")
            lines.append(f"{nm[:44]:44s} {pr['ms']:9.4f} {pr['achieved']:10.1f} {pr['unit']:>8s} {pr['frac']:19.3f}")
        lines += ["", "kernel trace of the same command", f"{'kernel':62s} {'calls':>6s} {'total_us':>11s} {'avg_us':>10s}"]
        for r in stats[:8]:
            lines.append(f"{short_kernel_name(r['Name'])[:62]:62s} {int(r['Calls']):6d} {float(r['TotalDurationNs']) / 1e3:11.1f} "
                         f"{float(r['AverageNs']) / 1e3:10.2f}")
        with open(os.path.join(ROOT, "profiles", workload + "_probe_kernels.txt"), "w") as f:
            f.write("\n".join(lines) + "\n")
        with open(os.path.join(ROOT, "profiles", workload + ".json"), "w") as f:
            json.dump({"workload": workload, "git_head": git_head(), "source_sha256": source_hash(workload),
                       "sources": workload_files(workload), "probes": res["probes"]}, f, indent=1, sort_keys=True)
            f.write("\n")
        print("\n".join(lines))
        return
    cal_f = [v for (k, c), v in pmc(find("pmc_FETCH_SIZE_calib", "p_counter_collection.csv")).items() if "map_kernel" in k][0]
    cal_w = [v for (k, c), v in pmc(find("pmc_WRITE_SIZE_calib", "p_counter_collection.csv")).items() if "map_kernel" in k][0]
    kib = 262144.0
    ff, fw = kib / cal_f, kib / cal_w
    stats = list(csv.DictReader(open(find("trace_" + workload, "t_kernel_stats.csv"))))
    pf = pmc(find("pmc_FETCH_SIZE_" + workload, "p_counter_collection.csv"))
    pw = pmc(find("pmc_WRITE_SIZE_" + workload, "p_counter_collection.csv"))
    cmd = f"python3 bench.py --workload {workload}"
    lines = [f"{workload}: per-kernel time and HBM traffic on one MI355X (rocprofv3, ROCm 7.2)", "",
             "commands (from /tmp, TMPDIR=/tmp; one run each; the summary below was written by "
             f"`python3 bench.py --workload {workload} --write-profile <dir holding the runs' output>`):",
             f"  rocprofv3 --kernel-trace --stats --output-format csv -d <out>/trace_{workload} -o t -- {cmd} --steps 10 --warmup 3 --no-cpu-baseline",
             f"  rocprofv3 --pmc FETCH_SIZE --output-format csv -d <out>/pmc_FETCH_SIZE_{workload} -o p -- {cmd} --steps 2 --warmup 1 --no-cpu-baseline",
             f"  rocprofv3 --pmc WRITE_SIZE --output-format csv -d <out>/pmc_WRITE_SIZE_{workload} -o p -- {cmd} --steps 2 --warmup 1 --no-cpu-baseline",
             "  rocprofv3 --pmc FETCH_SIZE (then WRITE_SIZE) --output-format csv -d <out>/pmc_<counter>_calib -o p -- python3 bench.py --calibrate-copy"
             "   (plain map kernel: 262144 KiB read, 262144 KiB written per launch)", "",
             f"sources: git {git_head()}, sha256 of {', '.join('csrc/' + f for f in workload_files(workload))} "
             f"{source_hash(workload)[:16]}", "",
             "kernel trace (warm-up + timed steps + the per-entry-point and per-kernel timing launches of bench.py)",
             f"{'kernel':62s} {'calls':>6s} {'total_us':>11s} {'avg_us':>10s} {'pct':>6s}"]
    kernels = {}
    for r in stats[:24]:
        nm = short_kernel_name(r["Name"])
        lines.append(f"{nm[:62]:62s} {int(r['Calls']):6d} {float(r['TotalDurationNs']) / 1e3:11.1f} "
                     f"{float(r['AverageNs']) / 1e3:10.2f} {float(r['Percentage']):6.2f}")
        kernels.setdefault(nm, {})["avg_us"] = float(r["AverageNs"]) / 1e3
    lines += ["", f"counter calibration: the map kernel reads FETCH_SIZE={cal_f:.1f} for 262144 KiB read (factor {ff:.3f}) "
                  f"and WRITE_SIZE={cal_w:.1f} for 262144 KiB written (factor {fw:.3f})", "",
              f"{'kernel':62s} {'FETCH_SIZE':>12s} {'WRITE_SIZE':>12s} {'read_MiB':>10s} {'written_MiB':>11s}"]
    # every kernel of the run, the library's own and the GEMM library's (those carry generated names)
    names = sorted({k for (k, c) in pf}, key=lambda k: -pf[(k, "FETCH_SIZE")])
    counts = collections.Counter(row["Kernel_Name"] for row in csv.DictReader(open(find("pmc_FETCH_SIZE_" + workload,
                                                                                          "p_counter_collection.csv"))))
    own = [counts[k] for k in names if "nlh::" in k]
    runs = collections.Counter(own).most_common(1)[0][0] if own else 1   # launches of a once-per-step kernel = steps in that run
    step_bytes = 0.0
    for k in names:
        a, b = pf[(k, "FETCH_SIZE")], pw.get((k, "WRITE_SIZE"), 0.0)
        nm = short_kernel_name(k)
        step_bytes += (a * ff + b * fw) * 1024 * counts[k] / runs
        if "nlh::" not in k and (a * ff + b * fw) < 1024:   # below 1 MiB per launch and not ours: fills and the like
            continue
        lines.append(f"{nm[:62]:62s} {a:12.1f} {b:12.1f} {a * ff / 1024:10.1f} {b * fw / 1024:11.1f}")
        kernels.setdefault(nm, {}).update(fetch_bytes=int(a * ff * 1024), write_bytes=int(b * fw * 1024))
    lines += ["", f"HBM traffic per step, every kernel of the run x its launches per step ({runs} steps' worth of launches in the "
                  f"counter run): {step_bytes / 1e9:.3f} GB"]
    mp = glob.glob(os.path.join(raw, "pmc_MFMA_" + workload, "**", "p_counter_collection.csv"), recursive=True)
    if mp:
        pm = pmc(mp[0])
        lines += ["", "matrix-core counters (one more run): rocprofv3 --pmc SQ_VALU_MFMA_BUSY_CYCLES SQ_BUSY_CYCLES "
                      "SQ_INSTS_VALU_MFMA_MOPS_BF16 SQ_INSTS_VALU_MFMA_MOPS_F32 GRBM_GUI_ACTIVE --output-format csv "
                      f"-d <out>/pmc_MFMA_{workload} -o p -- {cmd} --steps 2 --warmup 1 --no-cpu-baseline",
                  "per launch; GRBM_GUI_ACTIVE is summed over the 8 XCDs, SQ_VALU_MFMA_BUSY_CYCLES over the 1024 SIMDs; "
                  "MOPS counters are in units of 512 flop; mfma_busy = MFMA_BUSY / 1024 / (GUI_ACTIVE / 8)",
                  f"{'kernel':62s} {'GUI_ACTIVE':>12s} {'MFMA_BUSY':>13s} {'MOPS_BF16':>12s} {'MOPS_F32':>12s} {'mfma_busy':>10s}"]
        for k in sorted({k for (k, c) in pm if "nlh::" in k}, key=lambda k: -pm.get((k, "GRBM_GUI_ACTIVE"), 0)):
            ga = pm.get((k, "GRBM_GUI_ACTIVE"), 0)
            if ga <= 0:
                continue
            mb = pm.get((k, "SQ_VALU_MFMA_BUSY_CYCLES"), 0)
            nm = short_kernel_name(k)
            lines.append(f"{nm[:62]:62s} {ga:12.0f} {mb:13.0f} {pm.get((k, 'SQ_INSTS_VALU_MFMA_MOPS_BF16'), 0):12.0f} "
                         f"{pm.get((k, 'SQ_INSTS_VALU_MFMA_MOPS_F32'), 0):12.0f} {mb / 1024 / (ga / 8):10.3f}")
            kernels.setdefault(nm, {})["mfma_busy"] = mb / 1024 / (ga / 8)
    out_txt = os.path.join(ROOT, "profiles", workload + "_kernels_and_hbm_traffic.txt")
    with open(out_txt, "w") as f:
        f.write("\n".join(lines) + "\n")
    side = {"workload": workload, "git_head": git_head(), "source_sha256": source_hash(workload),
            "sources": workload_files(workload), "step_traffic_bytes": int(step_bytes),
            "calibration": {"fetch_factor": ff, "write_factor": fw,
                            "note": "counter KiB per dispatch x factor = KiB moved; factors from a map kernel of known size"},
            "kernels": kernels}
    with open(os.path.join(ROOT, "profiles", workload + ".json"), "w") as f:
        json.dump(side, f, indent=1, sort_keys=True)
        f.write("\n")
    print(open(out_txt).read())


def run_probe(which, torch, lib, steps, warmup):
    """What the box sustains, from kernels of the simplest shape (csrc/roof_probes.hip): streaming copies at 1 : 1 and
    3 : 2 read : write, and the matrix cores' issue peak for the two instructions the library uses."""
    res = {"metric": "sustained rate of the probe kernels", "n_gpus": 1, "steps": steps, "warmup": warmup,
           "data": "synthetic", "higher_is_better": True, "config": {"workload": which}, "probes": []}

    def timed(fn):
        for _ in range(warmup):
            fn()
        lib.nlh_timer_start()
        for _ in range(steps):
            fn()
        return lib.nlh_timer_stop_ms() / steps

    if which == "hbm_copy":
        n = 64 << 20   # floats per stream: 256 MiB, far beyond the 256 MB Infinity Cache once several streams are in play
        for reads, writes in ((1, 1), (3, 2)):
            a = torch.randn(reads * n, dtype=torch.float32, device="cuda")
            b = torch.empty(writes * n, dtype=torch.float32, device="cuda")
            ms = timed(lambda: lib.nlh_probe_stream_rocm(a.data_ptr(), b.data_ptr(), n, reads, writes))
            gbs = 4 * n * (reads + writes) / (ms * 1e-3) / 1e9
            res["probes"].append({"name": f"stream {reads} read : {writes} write", "bytes": 4 * n * (reads + writes), "ms": ms,
                                  "achieved": gbs, "unit": "GB/s", "peak": PEAK_HBM_GBS, "frac": gbs / PEAK_HBM_GBS})
            del a, b
        res.update(value=res["probes"][0]["achieved"], unit="GB/s", dtype="f32")
    else:
        cus = torch.cuda.get_device_properties(0).multi_processor_count
        out = torch.empty(cus * 8 * 256, dtype=torch.float32, device="cuda")
        for kind, name, flop, per_iter, peak in ((0, "v_mfma_f32_16x16x32_bf16", 16384, 8, PEAK_BF16_TFLOPS),
                                                 (2, "v_mfma_f32_32x32x16_bf16", 32768, 4, PEAK_BF16_TFLOPS),
                                                 (1, "v_mfma_f32_16x16x4_f32", 2048, 8, PEAK_FP32_TFLOPS)):
            for wps in (1, 2, 4):
                iters = 20000
                ms = timed(lambda: lib.nlh_probe_mfma_rocm(kind, iters, wps, out.data_ptr()))
                tf = flop * per_iter * iters * cus * 4 * wps / (ms * 1e-3) / 1e12
                res["probes"].append({"name": name, "waves_per_simd": wps, "ms": ms, "achieved": tf, "unit": "TFLOP/s",
                                      "peak": peak, "frac": tf / peak})
        res.update(value=max(p["achieved"] for p in res["probes"]), unit="TFLOP/s", dtype="bf16")
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="titans_chunkwise_c3", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="launch a plain map kernel (256 MiB read, 256 MiB written) 5 times and exit: "
                         "the known-size reference for scaling FETCH_SIZE / WRITE_SIZE counters")
    ap.add_argument("--write-profile", metavar="DIR",
                    help="no GPU work: summarise the rocprofv3 runs of this workload found under DIR into "
                         "profiles/<workload>_kernels_and_hbm_traffic.txt and profiles/<workload>.json")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (--gpus must be 1).")
    if args.write_profile:
        write_profile(args.workload, args.write_profile)
        return

    import torch
    from nl_hecate_amd import dispatch as D
    from nl_hecate_amd.ffi import lib

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU (the HIP library has no CPU fallback).")
    torch.cuda.set_device(0)
    lib.load()

    if args.calibrate_copy:
        n = 64 << 20
        a = torch.randn(n, dtype=torch.float32, device="cuda")
        b = torch.empty_like(a)
        for _ in range(5):
            D.call("sigmoid_cuda", a, b, n)
        torch.cuda.synchronize()
        print(json.dumps({"calibration_kernel": "map_kernel (sigmoid_cuda)", "launches": 5,
                          "read_bytes_per_launch": 4 * n, "written_bytes_per_launch": 4 * n}))
        return

    if args.workload in ("hbm_copy", "mfma_peak"):
        print(json.dumps(run_probe(args.workload, torch, lib, args.steps, args.warmup)))
        return

    w = WORKLOADS[args.workload](torch, D, lib)
    fwd, bwd = w["fwd"], w["bwd"]

    step = w.get("step") or (lambda: (fwd(), bwd()))
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()

    # timed region: exactly K steps, bracketed by synchronisation on both sides
    t0 = time.perf_counter()
    lib.nlh_timer_start()
    for _ in range(args.steps):
        step()
    ev_ms = lib.nlh_timer_stop_ms()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    ms_per_step = wall_ms / args.steps
    value = w["tokens"] / (ms_per_step * 1e-3)
    ev_step_ms = ev_ms / args.steps

    # per-entry-point durations with events on the launch stream (outside the timed region)
    def avg_ms(fn, n=10):
        lib.nlh_timer_start()
        for _ in range(n):
            fn()
        return lib.nlh_timer_stop_ms() / n
    fwd_ms, bwd_ms = avg_ms(fwd), avg_ms(bwd)
    # every instrumented kernel on its own: event pairs around its launches inside the entry points
    reps = 5
    lib.nlh_kernel_timer_enable(1)
    buf = ctypes.create_string_buffer(8192)
    timed = {}
    for _ in range(reps):
        (w.get("step_eager") or (lambda: (fwd(), bwd())))()
        assert lib.nlh_kernel_timer_report(buf, len(buf)) >= 0
        for item in buf.value.decode().split(";"):
            if item:
                nm, launches, ms = item.rsplit(":", 2)
                t = timed.setdefault(nm, [0, 0.0])
                t[0] += int(launches)
                t[1] += float(ms)
    lib.nlh_kernel_timer_enable(0)

    head_tokens = w["head_tokens"]
    hbm_bound = w.get("bound") == "hbm"
    peak = PEAK_HBM_GBS if hbm_bound else PEAK_FP32_TFLOPS
    unit = "GB/s" if hbm_bound else "TFLOP/s"
    per_ht = (lambda b, f: b) if hbm_bound else (lambda b, f: f)   # algorithmic work per head-token: bytes or flops
    scale = 1e9 if hbm_bound else 1e12

    def rate(work_per_ht, ms):
        return work_per_ht * head_tokens / (max(ms, 1e-9) * 1e-3) / scale

    side = profile_sidecar(args.workload)
    stale = None if side is None else side.get("source_sha256") != source_hash(args.workload)
    side_k = {} if side is None else side["kernels"]

    def kernel_traffic(nm):   # bytes per launch from the sidecar: the profile's kernel whose name starts with nm
        for pn, rec in side_k.items():
            if pn.startswith(nm) and "fetch_bytes" in rec:
                return rec["fetch_bytes"] + rec.get("write_bytes", 0)
        return None

    kernels = []
    for nm, (launches, ms) in sorted(timed.items(), key=lambda kv: -kv[1][1]):
        own = w.get("kernel_work", {}).get(nm)
        rec = {"name": nm, "launches_per_step": launches / reps, "avg_launch_ms": ms / launches,
               "ms_per_step": ms / reps, "traffic": kernel_traffic(nm)}
        if own is not None:
            rec.update(algorithmic=own * head_tokens, achieved=rate(own, ms / reps),
                       frac=rate(own, ms / reps) / peak, unit=unit)
        kernels.append(rec)
    step_traffic = None if side is None else side.get("step_traffic_bytes")
    if step_traffic is None and kernels and all(k["traffic"] is not None for k in kernels):
        step_traffic = int(sum(k["traffic"] * k["launches_per_step"] for k in kernels))
    work_step = per_ht(w.get("bytes_fwd", 0) + w["bytes_bwd"], w["flop_fwd"] + w["flop_bwd"])
    work_bwd = per_ht(w["bytes_bwd"], w["flop_bwd"])
    work_fwd = per_ht(w.get("bytes_fwd", 0), w["flop_fwd"])
    roofline = {
        "unit_timed": "the whole step (every kernel of the forward and backward entry points), HIP events on the "
                      "launch stream around the timed steps",
        "bound": "hbm" if hbm_bound else "mfma",
        "achieved": rate(work_step, ev_step_ms), "peak": peak, "unit": unit,
        "frac": rate(work_step, ev_step_ms) / peak,
        "algorithmic": work_step * head_tokens,
        "algorithmic_unit": "bytes per step" if hbm_bound else "flop per step",
        "avg_launch_ms": ev_step_ms,
        "traffic": step_traffic,
        "traffic_unit": "HBM bytes per step: sum over kernels of (FETCH_SIZE + WRITE_SIZE per launch, scaled by a copy "
                        "kernel) x launches per step, from profiles/" + args.workload + ".json",
        "traffic_stale": stale,
        "traffic_measured_at": None if side is None else side.get("git_head"),
        "entry_points": {
            "forward": {"ms": fwd_ms, "achieved": rate(work_fwd, fwd_ms), "frac": rate(work_fwd, fwd_ms) / peak},
            "backward": {"ms": bwd_ms, "achieved": rate(work_bwd, bwd_ms), "frac": rate(work_bwd, bwd_ms) / peak}},
        "kernels": kernels,
        "dominant_kernel": kernels[0] if kernels else None,
    }
    if "matrix" in w:   # matrix-core rate of the whole step beside the memory figure
        tf = (w["flop_fwd"] + w["flop_bwd"]) * head_tokens / (ev_step_ms * 1e-3) / 1e12
        roofline[w["matrix"]] = {"achieved": tf, "peak": w["matrix_peak"], "unit": "TFLOP/s", "frac": tf / w["matrix_peak"]}
    if "flop_ref_fwd" in w:   # the same step priced on the flops of the reference's formulation
        tf = (w["flop_ref_fwd"] + w["flop_ref_bwd"]) * head_tokens / (ev_step_ms * 1e-3) / 1e12
        roofline["flops_counted"] = "executed by the kernels"
        roofline["on_reference_flops"] = {"achieved": tf, "peak": peak, "unit": "TFLOP/s", "frac": tf / peak,
                                          "flop_per_step": (w["flop_ref_fwd"] + w["flop_ref_bwd"]) * head_tokens}
    if not hbm_bound:
        gbs = (w.get("bytes_fwd", 0) + w["bytes_bwd"]) * head_tokens / (ev_step_ms * 1e-3) / 1e9
        roofline["hbm"] = {"achieved": gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": gbs / PEAK_HBM_GBS}
    out = {
        "metric": METRIC, "value": value, "unit": w.get("unit", "tokens/s"), "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": w.get("dtype", "f32"), "data": "synthetic",
        "config": w["config"],
        "event_ms_per_step": ev_step_ms,
        "kernels_ms": {w["kernel_names"]["forward"]: fwd_ms, w["kernel_names"]["backward"]: bwd_ms},
        "roofline": roofline,
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = w["cpu"]()
        if "cpu_all" in w:
            out["cpu_baseline_all_cores"] = w["cpu_all"]()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
