#!/usr/bin/env python3
"""Benchmark of the Megalodon fused-op hot path on one MI355X.

Headline (`value`): one full Megalodon-7B-style block, forward + backward, at
L = 32768 (BASELINE config 4: D=4096, EMA ndim 16, z 1024, value 8192, 4 heads,
chunk 4096, FFN 11008 SwiGLU, bf16 weights and activations, fp32 norm / EMA
state), in tokens/s.  A step is one forward + backward of the block on
synthetic, seeded inputs that are resident in HBM before the timed region.

Beside it, in the same JSON line:
  roofline      the dominant kernel of the CEMA + convolution sub-layer
                (config 1: B=1, L=32768, D=4096, ndim=16, x / dy bf16), timed
                live with device events on the launch stream around twenty
                launches back to back
  cema_layer    the config-1 step (layer forward + backward) on the default
                path (chunked recurrence on the matrix cores, float32-equivalent
                arithmetic) and on the two FFT-convolution engines
  other_ops     TimestepNorm (config 2) and chunk attention (config 3)
  cpu_baseline  the block on the host cores through the reference's CPU
                formulation, on a bounded sample; per-op baselines in cpu_ops
Prints one JSON line.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E
# HBM bytes one backward launch of the CEMA recurrence moves at config 1: FETCH_SIZE x 2.0 +
# WRITE_SIZE x 1.0 from two rocprofv3 --pmc passes of this script (--cema-only --copy-calibration),
# the factors being what the same counters read for a plain copy of 2^30 bytes.  A measured
# constant (profiles/cema_scan_config1_hbm_traffic.txt): counters cannot be read from in here.
CEMA_BWD_TRAFFIC_BYTES = 8.091e8

CFG4 = dict(model_dim=4096, z_dim=1024, value_dim=8192, num_heads=4, cema_ndim=16, chunk_size=4096,
            ffn_hidden_dim=11008, norm_num_groups=32)


def host_cores():
    """Threads for the CPU baselines: the cores this process may run on (OMP_NUM_THREADS, when the
    environment sets it, is the share of the box a job is given and wins)."""
    env = os.environ.get("OMP_NUM_THREADS")
    if env:
        return int(env)
    try:
        return len(os.sched_getaffinity(0))
    except AttributeError:
        return os.cpu_count() or 1


def host_info():
    model = "unknown"
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    return {"nproc": os.cpu_count(), "cpu_model": model, "omp_num_threads_env": os.environ.get("OMP_NUM_THREADS")}


# --------------------------------------------------------------------------- CPU baselines
def _timed(fn, budget_s, max_reps=3):
    t0 = time.perf_counter()
    fn()
    one = time.perf_counter() - t0
    reps = max(1, min(max_reps, int(budget_s / max(one, 1e-3)) - 1))
    t0 = time.perf_counter()
    for _ in range(reps):
        fn()
    return (time.perf_counter() - t0) / reps, reps


def cpu_cema(B, D, N, L, seed, cores, budget_s=12.0):
    """Config 1 through the reference's CPU formulation: ema_parameters by the
    C/OpenMP restatement of its loop nest (csrc/ops/ema_parameters.cc), the
    convolution by torch.fft on CPU tensors (fused_ops/fftconv.py:30-75)."""
    import torch
    from megalodon_amd import synthetic
    from oracle import native
    lib = native.port()
    Ds = 1024
    prm = synthetic.cema_params(D, N, seed)
    io = synthetic.cema_inputs(B, Ds, L, seed, torch.bfloat16)
    p, lq, g, om = prm["p"][:Ds], prm["q"][:Ds].log(), prm["gamma"][:Ds], prm["omega"][:Ds]

    def step():
        k = native.ema_weight_fwd(lib, "oracle_", p, lq, g, L)
        x = io["x"].float()
        n = 2 * (L if (L & (L - 1)) == 0 else (1 << L.bit_length()))
        x_f = torch.fft.rfft(x, n=n)
        k_f = torch.fft.rfft(k, n=n, norm="forward")
        y = torch.fft.irfft(x_f * k_f, n=n, norm="forward")[..., :L].to(torch.bfloat16)
        out = y + io["x"] * om
        dy = io["dy"].float()
        dy_f = torch.fft.rfft(dy.flip(dims=(-1,)), n=n)
        dx = torch.fft.irfft(dy_f * k_f, n=n, norm="forward")[..., :L].flip(dims=(-1,)).to(torch.bfloat16)
        dk = torch.fft.irfft((dy_f * x_f).sum(dim=0), n=n)[..., :L].flip(dims=(-1,))
        dx = dx + io["dy"] * om
        dom = (io["dy"].float() * x).sum(dim=(0, 2))
        return out, dx, dom, native.ema_weight_bwd(lib, "oracle_", dk, p, lq, g)

    dt, reps = _timed(step, budget_s)
    return {"value": B * L / (dt * D / Ds), "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": f"{Ds} of {D} channels, {reps} rep(s) of the fwd+bwd step at L={L}, {dt:.2f} s each, "
                      f"scaled by D/{Ds}"}


def cpu_timestep_norm(cores, budget_s=12.0):
    """Config 2 through the C/OpenMP restatement of GroupTimestepNormCPUFwd/Bwd
    (csrc/ops/timestep_norm.cc:218-450; the scan runs over the batch only, as there)."""
    import torch
    from megalodon_amd import synthetic
    from oracle import native
    lib = native.port()
    B, L, D, G = 4, 8192, 4096, 32
    Ls = L
    io = {k: (v[:, :Ls].contiguous() if v.dim() >= 2 and v.shape[1] == L else v)
          for k, v in synthetic.timestep_norm_inputs(B, L, D, G, 1002).items()}
    f = {k: (v.float() if v.is_floating_point() else v) for k, v in io.items()}

    def step():
        y, count, mean, var, cm, cr = native.group_timestep_norm_fwd(
            lib, "oracle_", f["x"], f["prev_count"], f["prev_mean"], f["prev_var"], f["gamma"], f["beta"],
            f["mask"], G, 1e-5)
        native.group_timestep_norm_bwd(lib, "oracle_", f["dy"], f["dmean"], f["dvar"], f["x"], f["prev_mean"],
                                       count, cm, cr, f["gamma"], f["mask"], G)

    dt, reps = _timed(step, budget_s, max_reps=30)
    return {"value": B * Ls / dt, "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": f"the whole config (all {Ls} steps of all {B} sequences), {reps} rep(s), {dt:.2f} s each"}


def cpu_attention(cores, budget_s=12.0):
    """Config 3 through the reference's unfused branch: matmul + causal mask +
    float32 softmax + matmul, backward by autograd
    (modules/moving_average_gated_attention.py:116-129)."""
    import torch
    from megalodon_amd import synthetic
    C, H1, H2 = 4096, 256, 2048
    io = synthetic.attention_inputs(1, C, 1, H1, H2, 1003)
    q, k, v = (io[n].float().transpose(1, 2).requires_grad_(True) for n in ("q", "k", "v"))
    dy = io["dy"].float().transpose(1, 2)
    mask = torch.full((C, C), float("-inf")).triu(1)

    def step():
        for t in (q, k, v):
            t.grad = None
        s = torch.matmul(q, k.transpose(2, 3)) + mask
        out = torch.matmul(torch.softmax(s, dim=-1, dtype=torch.float32), v)
        out.backward(dy)

    dt, reps = _timed(step, budget_s, max_reps=30)
    pairs = 32  # 8 chunks x 4 heads
    return {"value": 32768 / (dt * pairs), "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": f"1 of {pairs} (chunk, head) pairs (they are independent), {reps} rep(s), {dt:.2f} s each, "
                      f"scaled by {pairs}"}


def cpu_block_forward(p, x, cfg):
    """One block on CPU tensors in float32, the reference's CPU arithmetic: TimestepNorm and the CEMA
    kernel row through the C/OpenMP restatements of its loop nests (csrc/ops/timestep_norm.cc:218-450,
    csrc/ops/ema_parameters.cc:17-98), the convolution through torch.fft (fused_ops/fftconv.py:30-75),
    attention as matmul + causal mask + float32 softmax + matmul
    (modules/moving_average_gated_attention.py:116-129), projections and norms through
    torch.nn.functional; differentiable.  `p` is keyed like MegaBlock.named_parameters(); x (1, L, D)
    with L at most one chunk."""
    import math
    import torch
    import torch.nn.functional as F
    from oracle import native
    lib = native.port()
    _, Ls, D = x.shape
    Z, H = cfg["z_dim"], cfg["value_dim"]
    N, NH, G = cfg["cema_ndim"], cfg["num_heads"], cfg["norm_num_groups"]
    assert x.shape[0] == 1 and Ls <= cfg["chunk_size"]
    pc, pm, pv = torch.zeros(1, dtype=torch.int64), torch.zeros(1, G), torch.ones(1, G)

    class TimestepNormCPU(torch.autograd.Function):
        @staticmethod
        def forward(ctx, x_, gamma, beta):
            y, count, mean, var, cm, cr = native.group_timestep_norm_fwd(lib, "oracle_", x_, pc, pm, pv, gamma, beta,
                                                                         None, G, 1e-5)
            ctx.save_for_backward(x_, count, cm, cr, gamma)
            return y

        @staticmethod
        def backward(ctx, gy):
            x_, count, cm, cr, gamma = ctx.saved_tensors
            dx, _, _, dgam, dbet = native.group_timestep_norm_bwd(lib, "oracle_", gy.contiguous(), torch.zeros(1, G),
                                                                  torch.zeros(1, G), x_, pm, count, cm, cr, gamma, None, G)
            return dx, dgam, dbet

    class EmaWeightCPU(torch.autograd.Function):
        @staticmethod
        def forward(ctx, pp, q, gam):
            ctx.save_for_backward(pp, q, gam)
            return native.ema_weight_fwd(lib, "oracle_", pp, q.log(), gam, Ls)

        @staticmethod
        def backward(ctx, gk):
            pp, q, gam = ctx.saved_tensors
            # the operator returns the gradients with respect to (p, q, gamma), as the reference's does
            dp, dq, dg = native.ema_weight_bwd(lib, "oracle_", gk.contiguous(), pp, q.log(), gam)
            return dp.view_as(pp), dq.view_as(q), dg.view_as(gam)

    rms = lambda t, w: t * torch.rsqrt((t * t).mean(-1, keepdim=True) + 1e-5) * (1.0 if w is None else w + 1.0)
    tsn = TimestepNormCPU.apply(x, p["mega.timenorm.weight"] + 1.0, p["mega.timenorm.bias"])
    pp = torch.sigmoid(p["mega.cema.alpha"])
    ang = torch.sigmoid(p["mega.cema.theta"]) * (2 * math.pi / N) * torch.arange(1, N + 1).view(1, N, 1)
    q = torch.polar(1.0 - pp * torch.sigmoid(p["mega.cema.delta"]), ang)
    k = EmaWeightCPU.apply(pp, q.squeeze(-1), torch.view_as_complex(p["mega.cema.gamma"]) * math.sqrt(1.0 / N))
    xt = tsn.transpose(1, 2)
    n = 2 * (Ls if (Ls & (Ls - 1)) == 0 else (1 << Ls.bit_length()))
    conv = torch.fft.irfft(torch.fft.rfft(xt, n=n) * torch.fft.rfft(k, n=n, norm="forward"), n=n, norm="forward")[..., :Ls]
    mx = rms((conv + xt * p["mega.cema.omega"]).transpose(1, 2), p["mega.rmsnorm.weight"])
    zh = Z // NH
    z = rms(F.linear(mx, p["mega.wz.weight"], p["mega.wz.bias"]).view(1, Ls, NH, zh), None).view(1, Ls, Z)
    z = z.unsqueeze(2) * ((p["mega.gamma"] + 1.0) / math.sqrt(zh)) + p["mega.beta"]
    qq, kk = (t.reshape(1, Ls, NH, zh).transpose(1, 2) for t in torch.unbind(z, dim=2))
    v = F.silu(F.linear(tsn, p["mega.wv.weight"], p["mega.wv.bias"])).view(1, Ls, NH, H // NH).transpose(1, 2)
    rr = F.silu(F.linear(mx, p["mega.wr.weight"], p["mega.wr.bias"]))
    mask = torch.full((Ls, Ls), float("-inf")).triu(1)
    prob = torch.softmax(torch.matmul(qq, kk.transpose(2, 3)) + mask, dim=-1, dtype=torch.float32)
    attn = torch.matmul(prob, v).transpose(1, 2).reshape(1, Ls, H) * rr
    y1 = F.linear(mx, p["mega.wh1.weight"], p["mega.wh1.bias"]) + F.linear(attn, p["mega.wh2.weight"]) + x
    nn_ = F.layer_norm(y1, (D,), p["nffn.norm.weight"] + 1.0, p["nffn.norm.bias"], 1e-5)
    hid = F.silu(F.linear(nn_, p["nffn.fc1.weight"])) * F.linear(nn_, p["nffn.fc3.weight"])
    return F.linear(hid, p["nffn.fc2.weight"]) + x


def cpu_block(cores, budget_s=25.0):
    """Config 4 on the host in float32 (cpu_block_forward, backward by autograd) on a prefix of the
    sequence: every stage but attention is linear in L and attention is cheaper per token below one
    chunk, so the figure flatters the CPU."""
    import torch
    Ls = 1024
    g = torch.Generator().manual_seed(1004)
    D, Z, H, F_ = CFG4["model_dim"], CFG4["z_dim"], CFG4["value_dim"], CFG4["ffn_hidden_dim"]
    N = CFG4["cema_ndim"]
    r = lambda *s: (torch.randn(*s, generator=g) * 0.02).requires_grad_(True)
    p = {"mega.timenorm.weight": r(D), "mega.timenorm.bias": r(D), "mega.cema.alpha": r(D, N, 1),
         "mega.cema.delta": r(D, N, 1), "mega.cema.theta": r(D, 1, 1), "mega.cema.gamma": r(D, N, 2),
         "mega.cema.omega": r(D, 1), "mega.rmsnorm.weight": r(D), "mega.wz.weight": r(Z, D), "mega.wz.bias": r(Z),
         "mega.wv.weight": r(H, D), "mega.wv.bias": r(H), "mega.wr.weight": r(H, D), "mega.wr.bias": r(H),
         "mega.wh1.weight": r(D, D), "mega.wh1.bias": r(D), "mega.wh2.weight": r(D, H), "mega.gamma": r(2, Z),
         "mega.beta": r(2, Z), "nffn.norm.weight": r(D), "nffn.norm.bias": r(D), "nffn.fc1.weight": r(F_, D),
         "nffn.fc2.weight": r(D, F_), "nffn.fc3.weight": r(F_, D)}
    x = (torch.rand(1, Ls, D, generator=g) * 2 - 1).requires_grad_(True)
    dy = torch.randn(1, Ls, D, generator=g)

    def step():
        for t in list(p.values()) + [x]:
            t.grad = None
        cpu_block_forward(p, x, CFG4).backward(dy)

    dt, reps = _timed(step, budget_s, max_reps=3)
    return {"value": Ls / dt, "unit": "tokens/s", "cores": cores, "kind": "port", "dtype": "f32", **host_info(),
            "sample": f"the first {Ls} of 32768 tokens of the block in float32 (C/OpenMP restatements of the reference's "
                      f"TimestepNorm and ema_parameters loop nests, torch.fft convolution, matmul + softmax attention, "
                      f"F.linear projections; autograd backward), {reps} rep(s), {dt:.2f} s each"}


# --------------------------------------------------------------------------- GPU legs
def dev_ms(torch, fn, n, warm=1):
    # `warm` untimed calls first: the first milliseconds after an idle device run below the clocks
    # the kernels sustain (attention forward: 1.62 ms over calls 2-6, 1.33 ms over calls 11-110)
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(n):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / n


def block_leg(torch, dev, steps, warmup):
    from megalodon_amd.modules import MegaBlock
    torch.manual_seed(1004)
    blk = MegaBlock(**CFG4).to(dev).bfloat16()
    gb = torch.Generator().manual_seed(1004)
    bx = (torch.rand(1, 32768, 4096, generator=gb) * 2 - 1).bfloat16().to(dev).requires_grad_(True)
    bdy = torch.randn(1, 32768, 4096, generator=gb).bfloat16().to(dev)

    def step():
        bx.grad = None
        for prm in blk.parameters():
            prm.grad = None
        o, _ = blk(bx)
        o.backward(bdy)

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps
    # outside the timed region: a TimestepNorm tile that gave up its bounded wait would have
    # written NaN; the status word turns that into an error instead of a quietly wrong number
    from megalodon_amd import extension as ops
    ops.timestep_norm_status(dev)
    if not torch.isfinite(bx.grad.float()).all():
        raise RuntimeError("bench: the block's input gradient is not finite")
    del blk, bx, bdy
    torch.cuda.empty_cache()
    return dt


def cema_leg(torch, dev, steps, warmup, copy_calibration):
    """Config 1: layer forward + backward; per-kernel device times of the default path."""
    from megalodon_amd import _lib, synthetic
    from megalodon_amd.modules import MultiHeadComplexEMA
    B, D, N, L, seed = 1, 4096, 16, 32768, 1001
    layer = MultiHeadComplexEMA(D, N).to(dev).train()
    io = synthetic.cema_inputs(B, D, L, seed, torch.bfloat16)
    x = io["x"].to(dev).requires_grad_(True)
    dy = io["dy"].to(dev)

    def step():
        x.grad = None
        for prm in layer.parameters():
            prm.grad = None
        out, _ = layer(x, None, False)
        out.backward(dy)

    def timed(n):
        for _ in range(warmup):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n):
            step()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / n

    for _ in range(warmup):
        step()
    log = {"mega_cema_scan_fwd": [], "mega_cema_scan_bwd_state": [], "mega_cema_coeffs_fwd": [], "mega_cema_coeffs_bwd": []}
    _lib.set_event_log(log)
    dt = timed(steps)
    _lib.set_event_log(None)
    avg = {k: (sum(a.elapsed_time(b) for a, b in v) / max(1, len(v))) for k, v in log.items()}
    E = B * D * L
    # the two recurrence kernels launched back to back on the layer's own operands, device events
    # around the run: the launch duration without the host's time to issue it (inside a step the
    # device is idle when the first event of a call is recorded, so `kernels_ms` above holds the
    # 10-25 us the host takes to launch as well)
    from megalodon_amd import extension as ops
    n_k = 20 if steps >= 5 else max(1, steps)
    with torch.no_grad():
        cp, clq, cgm = ops.cema_coeffs_fwd(layer.alpha.float(), layer.delta.float(), layer.theta.float(),
                                           layer.gamma.float())
        xd = x.detach()
        ms_f = dev_ms(torch, lambda: ops.cema_scan_fwd(xd, cp, clq, cgm, layer.omega), n_k, warm=min(3, n_k))
        ms_b = dev_ms(torch, lambda: ops.cema_scan_bwd(dy, xd, cp, clq, cgm, layer.omega), n_k, warm=min(3, n_k))
    res = {"ms_per_step": dt * 1e3, "tokens_per_s": B * L / dt,
           "GBps_on_10E": 10 * E / dt / 1e9, "frac_hbm_on_10E": 10 * E / dt / 1e9 / HBM_PEAK_GBS,
           "kernels_ms": avg,
           "scan_launch_ms": {"fwd": ms_f, "bwd": ms_b, "launches": n_k},
           "scan_fwd_GBps": 4 * E / (ms_f * 1e-3) / 1e9,
           "scan_bwd_GBps": 6 * E / (ms_b * 1e-3) / 1e9}
    # the same step on the FFT-convolution operators: float32 transforms, then the fp16-stage engine
    n_alt = max(1, min(5, steps))
    os.environ["MEGA_CEMA_FFT"] = "1"
    try:
        res["fft_conv_fp32_engine"] = {"ms_per_step": timed(n_alt) * 1e3, "steps": n_alt}
        os.environ["MEGA_FFTCONV_F16_STAGES"] = "1"
        res["fft_conv_f16_stage_engine"] = {"ms_per_step": timed(n_alt) * 1e3, "steps": n_alt}
    finally:
        os.environ.pop("MEGA_CEMA_FFT", None)
        os.environ.pop("MEGA_FFTCONV_F16_STAGES", None)
    # the same layer step on float32 rows: the recurrence kernels on two bfloat16 pieces per tensor
    # (16 significant bits, parameter gradients within 1e-4), three backward launches
    x32 = io["x"].float().to(dev).requires_grad_(True)
    dy32 = io["dy"].float().to(dev)

    def step32():
        x32.grad = None
        for prm in layer.parameters():
            prm.grad = None
        out, _ = layer(x32, None, False)
        out.backward(dy32)

    for _ in range(2):
        step32()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(n_alt):
        step32()
    torch.cuda.synchronize()
    res["float32_rows"] = {"ms_per_step": (time.perf_counter() - t0) / n_alt * 1e3, "steps": n_alt}
    del x32, dy32
    if copy_calibration:
        src = torch.ones(1 << 29, dtype=torch.bfloat16, device=dev)
        dst = torch.empty_like(src)
        torch.mul(src, 1.0, out=dst)  # reads 2^30 bytes, writes 2^30 bytes
        torch.cuda.synchronize()
        del src, dst
    roofline = {
        "bound": "hbm",
        "kernel": "cema_scan_bwd_kernel<bf16> (one launch = backward of the CEMA layer for all B*D rows: dx and the "
                  "gradients of p, q, gamma, omega from dy and x; the longest kernel of the config-1 step)",
        "achieved": res["scan_bwd_GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
        "frac": res["scan_bwd_GBps"] / HBM_PEAK_GBS, "traffic": CEMA_BWD_TRAFFIC_BYTES,
        "algorithmic_bytes": 6 * E,
    }
    return res, roofline


def other_ops(torch, dev):
    """TimestepNorm (config 2) and chunk attention (config 3), timed with device events."""
    from megalodon_amd import extension as ops, synthetic
    other = {}
    tB, tL, tD, tG = 4, 8192, 4096, 32
    tio = {k_: v_.to(dev) for k_, v_ in synthetic.timestep_norm_inputs(tB, tL, tD, tG, 1002).items()}
    tE = tB * tL * tD
    # GBps / frac_hbm price the op at its 4E (6E) algorithmic bytes; padding rows are written
    # (zeros) but never read, so GBps_moved counts them once less.  Timed as the module runs it
    # (the saved statistics time-last, (B, G, L): they go to the backward and nowhere else) and,
    # beside it, as the operator-level call returns them (the reference's (B, L, G))
    live = 1.0 - float(tio["mask"].float().mean())
    # The forward leg that is timed first after the other legs of this program reads 6-7 % slower
    # than the same leg timed after a backward leg (which leaves x in the memory-side cache), so the
    # two layouts are timed in two rounds -- ref, module, ref, module -- and the second round, where
    # both have the same predecessor, is what is reported.
    for rnd in range(2):
        for time_last, tag, note in ((False, "_ref_layout", "statistics (B, L, G) (operator-level call)"),
                                     (True, "", "statistics kept (B, G, L) (module path)")):
            fwd = lambda: ops.group_timestep_norm_fwd(tio["x"], tio["prev_count"], tio["prev_mean"], tio["prev_var"],
                                                      tio["gamma"], tio["beta"], tio["mask"], tG, 1e-5,
                                                      stats_time_last=time_last)
            ty, tcount, tmean, tvar, tcm, tcr = fwd()
            ms = dev_ms(torch, fwd, 50, warm=5)
            other["timestep_norm_fwd" + tag] = {"ms": ms, "GBps": 4 * tE / ms / 1e6,
                                                "frac_hbm": 4 * tE / ms / 1e6 / HBM_PEAK_GBS, "unmasked_steps": live,
                                                "GBps_moved": (2 + 2 * live) * tE / ms / 1e6, "statistics": note}
            ms = dev_ms(torch, lambda: ops.group_timestep_norm_bwd(tio["dy"], tio["dmean"], tio["dvar"], tio["x"],
                                                                   tio["prev_mean"], tcount, tcm, tcr, tio["gamma"],
                                                                   tio["mask"], tG, stats_time_last=time_last), 50, warm=5)
            other["timestep_norm_bwd" + tag] = {"ms": ms, "GBps": 6 * tE / ms / 1e6,
                                                "frac_hbm": 6 * tE / ms / 1e6 / HBM_PEAK_GBS, "unmasked_steps": live,
                                                "GBps_moved": (2 + 4 * live) * tE / ms / 1e6, "statistics": note}
    ops.timestep_norm_status(dev)
    if not torch.isfinite(bx.grad.float()).all():
        raise RuntimeError("bench: the block's input gradient is not finite")
    del blk, bx, bdy
    torch.cuda.empty_cache()
    return dt


def cema_leg(torch, dev, steps, warmup, copy_calibration):
    """Config 1: layer forward + backward; per-kernel device times of the default path."""
    from megalodon_amd import _lib, synthetic
    from megalodon_amd.modules import MultiHeadComplexEMA
    B, D, N, L, seed = 1, 4096, 16, 32768, 1001
    layer = MultiHeadComplexEMA(D, N).to(dev).train()
    io = synthetic.cema_inputs(B, D, L, seed, torch.bfloat16)
    x = io["x"].to(dev).requires_grad_(True)
    dy = io["dy"].to(dev)

    def step():
        x.grad = None
        for prm in layer.parameters():
            prm.grad = None
        out, _ = layer(x, None, False)
        out.backward(dy)

    def timed(n):
        for _ in range(warmup):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n):
            step()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / n

    for _ in range(warmup):
        step()
    log = {"mega_cema_scan_fwd": [], "mega_cema_scan_bwd_state": [], "mega_cema_coeffs_fwd": [], "mega_cema_coeffs_bwd": []}
    _lib.set_event_log(log)
    dt = timed(steps)
    _lib.set_event_log(None)
    avg = {k: (sum(a.elapsed_time(b) for a, b in v) / max(1, len(v))) for k, v in log.items()}
    E = B * D * L
    # the two recurrence kernels launched back to back on the layer's own operands, device events
    # around the run: the launch duration without the host's time to issue it (inside a step the
    # device is idle when the first event of a call is recorded, so `kernels_ms` above holds the
    # 10-25 us the host takes to launch as well)
    from megalodon_amd import extension as ops
    n_k = 20 if steps >= 5 else max(1, steps)
    with torch.no_grad():
        cp, clq, cgm = ops.cema_coeffs_fwd(layer.alpha.float(), layer.delta.float(), layer.theta.float(),
                                           layer.gamma.float())
        xd = x.detach()
        ms_f = dev_ms(torch, lambda: ops.cema_scan_fwd(xd, cp, clq, cgm, layer.omega), n_k, warm=min(3, n_k))
        ms_b = dev_ms(torch, lambda: ops.cema_scan_bwd(dy, xd, cp, clq, cgm, layer.omega), n_k, warm=min(3, n_k))
    res = {"ms_per_step": dt * 1e3, "tokens_per_s": B * L / dt,
           "GBps_on_10E": 10 * E / dt / 1e9, "frac_hbm_on_10E": 10 * E / dt / 1e9 / HBM_PEAK_GBS,
           "kernels_ms": avg,
           "scan_launch_ms": {"fwd": ms_f, "bwd": ms_b, "launches": n_k},
           "scan_fwd_GBps": 4 * E / (ms_f * 1e-3) / 1e9,
           "scan_bwd_GBps": 6 * E / (ms_b * 1e-3) / 1e9}
    # the same step on the FFT-convolution operators: float32 transforms, then the fp16-stage engine
    n_alt = max(1, min(5, steps))
    os.environ["MEGA_CEMA_FFT"] = "1"
    try:
        res["fft_conv_fp32_engine"] = {"ms_per_step": timed(n_alt) * 1e3, "steps": n_alt}
        os.environ["MEGA_FFTCONV_F16_STAGES"] = "1"
        res["fft_conv_f16_stage_engine"] = {"ms_per_step": timed(n_alt) * 1e3, "steps": n_alt}
    finally:
        os.environ.pop("MEGA_CEMA_FFT", None)
        os.environ.pop("MEGA_FFTCONV_F16_STAGES", None)
    # the same layer step on float32 rows: the recurrence kernels on two bfloat16 pieces per tensor
    # (16 significant bits, parameter gradients within 1e-4), three backward launches
    x32 = io["x"].float().to(dev).requires_grad_(True)
    dy32 = io["dy"].float().to(dev)

    def step32():
        x32.grad = None
        for prm in layer.parameters():
            prm.grad = None
        out, _ = layer(x32, None, False)
        out.backward(dy32)

    for _ in range(2):
        step32()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(n_alt):
        step32()
    torch.cuda.synchronize()
    res["float32_rows"] = {"ms_per_step": (time.perf_counter() - t0) / n_alt * 1e3, "steps": n_alt}
    del x32, dy32
    if copy_calibration:
        src = torch.ones(1 << 29, dtype=torch.bfloat16, device=dev)
        dst = torch.empty_like(src)
        torch.mul(src, 1.0, out=dst)  # reads 2^30 bytes, writes 2^30 bytes
        torch.cuda.synchronize()
        del src, dst
    roofline = {
        "bound": "hbm",
        "kernel": "cema_scan_bwd_kernel<bf16> (one launch = backward of the CEMA layer for all B*D rows: dx and the "
                  "gradients of p, q, gamma, omega from dy and x; the longest kernel of the config-1 step)",
        "achieved": res["scan_bwd_GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
        "frac": res["scan_bwd_GBps"] / HBM_PEAK_GBS, "traffic": CEMA_BWD_TRAFFIC_BYTES,
        "algorithmic_bytes": 6 * E,
    }
    return res, roofline


def other_ops(torch, dev):
    """TimestepNorm (config 2) and chunk attention (config 3), timed with device events."""
    from megalodon_amd import extension as ops, synthetic
    other = {}
    tB, tL, tD, tG = 4, 8192, 4096, 32
    tio = {k_: v_.to(dev) for k_, v_ in synthetic.timestep_norm_inputs(tB, tL, tD, tG, 1002).items()}
    tE = tB * tL * tD
    # GBps / frac_hbm price the op at its 4E (6E) algorithmic bytes; padding rows are written
    # (zeros) but never read, so GBps_moved counts them once less.  Timed as the module runs it
    # (the saved statistics time-last, (B, G, L): they go to the backward and nowhere else) and,
    # beside it, as the operator-level call returns them (the reference's (B, L, G))
    live = 1.0 - float(tio["mask"].float().mean())
    # whichever forward leg is timed first after the other legs of this program reads 7 % slower
    # than when it is timed second; forty untimed calls first take that out of both
    for _ in range(40):
        ops.group_timestep_norm_fwd(tio["x"], tio["prev_count"], tio["prev_mean"], tio["prev_var"], tio["gamma"],
                                    tio["beta"], tio["mask"], tG, 1e-5)
    for time_last, tag, note in ((False, "_ref_layout", "statistics (B, L, G) (operator-level call)"),
                                 (True, "", "statistics kept (B, G, L) (module path)")):
        fwd = lambda: ops.group_timestep_norm_fwd(tio["x"], tio["prev_count"], tio["prev_mean"], tio["prev_var"],
                                                  tio["gamma"], tio["beta"], tio["mask"], tG, 1e-5,
                                                  stats_time_last=time_last)
        ty, tcount, tmean, tvar, tcm, tcr = fwd()
        ms = dev_ms(torch, fwd, 100, warm=20)
        other["timestep_norm_fwd" + tag] = {"ms": ms, "GBps": 4 * tE / ms / 1e6,
                                            "frac_hbm": 4 * tE / ms / 1e6 / HBM_PEAK_GBS, "unmasked_steps": live,
                                            "GBps_moved": (2 + 2 * live) * tE / ms / 1e6, "statistics": note}
        ms = dev_ms(torch, lambda: ops.group_timestep_norm_bwd(tio["dy"], tio["dmean"], tio["dvar"], tio["x"],
                                                               tio["prev_mean"], tcount, tcm, tcr, tio["gamma"],
                                                               tio["mask"], tG, stats_time_last=time_last), 100, warm=20)
        other["timestep_norm_bwd" + tag] = {"ms": ms, "GBps": 6 * tE / ms / 1e6,
                                            "frac_hbm": 6 * tE / ms / 1e6 / HBM_PEAK_GBS, "unmasked_steps": live,
                                            "GBps_moved": (2 + 4 * live) * tE / ms / 1e6, "statistics": note}
    ops.timestep_norm_status(dev)
    del tio, ty, tcm, tcr
    # what a kernel that only moves the same streams reaches: one read + one write stream of 2E
    # bytes each (the forward passes), two reads + one write (the backward passes)
    a = torch.empty(2 * tE, dtype=torch.uint8, device=dev).random_()
    b = torch.empty_like(a).random_()
    ceiling = {}
    for name, second, streams in (("read1_write1", None, 2), ("read2_write1", b, 3)):
        best = None
        for wgs in (2048, 4096, 8192, 16384, 32768):
            for nt in (False, True):
                ms = dev_ms(torch, lambda: ops.stream_copy(a, second, wgs, nt), 10)
                if best is None or ms < best[0]:
                    best = (ms, wgs, nt)
        ceiling[name] = {"ms": best[0], "GBps": streams * 2 * tE / best[0] / 1e6,
                         "frac_hbm": streams * 2 * tE / best[0] / 1e6 / HBM_PEAK_GBS, "workgroups": best[1], "nontemporal": best[2]}
    other["stream_copy_ceiling"] = ceiling
    del a, b
    aio = {k_: v_.to(dev) for k_, v_ in synthetic.attention_inputs(8, 4096, 4, 256, 2048, 1003).items()}
    pairs = 4096 * 4097 // 2
    f_fwd, f_bwd = 2 * pairs * (256 + 2048) * 32, 2 * pairs * (2 * 256 + 2 * 2048) * 32
    # forward as the modules run it (w goes to the backward pass only: the zeros right of the diagonal
    # block stay unwritten), and as the operator-level call returns it (every row of w written to its
    # end, as the reference's softmax does: 0.55 GB of zeros more)
    ay, aw = ops.attention_fwd(aio["q"], aio["k"], aio["v"], 1.0, 0.0, True, lower_only=True)
    ms = dev_ms(torch, lambda: ops.attention_fwd(aio["q"], aio["k"], aio["v"], 1.0, 0.0, True, lower_only=True), 50, warm=10)
    other["attention_fwd"] = {"ms": ms, "TFLOPs": f_fwd / ms / 1e9, "frac_mfma_bf16": f_fwd / ms / 1e9 / 2516.6,
                              "w": "lower blocks only (module path)"}
    ms = dev_ms(torch, lambda: ops.attention_fwd(aio["q"], aio["k"], aio["v"], 1.0, 0.0, True), 50, warm=10)
    other["attention_fwd_full_w"] = {"ms": ms, "TFLOPs": f_fwd / ms / 1e9, "frac_mfma_bf16": f_fwd / ms / 1e9 / 2516.6,
                                     "w": "every row to its end (operator-level call)"}
    ms = dev_ms(torch, lambda: ops.attention_bwd(aio["dy"], aio["q"], aio["k"], aio["v"], aw, 1.0, True), 50, warm=10)
    other["attention_bwd"] = {"ms": ms, "TFLOPs": f_bwd / ms / 1e9, "frac_mfma_bf16": f_bwd / ms / 1e9 / 2516.6}
    del aio, ay, aw
    torch.cuda.empty_cache()
    return other


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cema-only", action="store_true",
                    help="time only the config-1 layer step (short runs under a profiler)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also launch one plain elementwise copy of 1 GiB in, 1 GiB out "
                         "(reference point for scaling FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (every op shards "
              "without communication along channels / batch / heads); run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    import torch
    from megalodon_amd import _lib

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    _lib.load()  # fails loudly when the HIP library is missing
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    cema, roofline = cema_leg(torch, dev, args.steps, args.warmup, args.copy_calibration)
    if args.cema_only:
        print(json.dumps({"cema_layer": cema, "roofline": roofline}), flush=True)
        return
    other = other_ops(torch, dev)
    dt = block_leg(torch, dev, args.steps, args.warmup)

    result = {
        "metric": "Megalodon layer fwd+bwd tokens/s at L=32K, 1 GPU; CEMA+FFT-conv HBM GB/s (% peak)",
        "value": 32768 / dt,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": dt * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16 (fp32 accumulation; CEMA recurrence, norm statistics and softmax in fp32)",
        "data": "synthetic",
        "config": {"workload": "configs[4]: one Megalodon-7B-style block forward+backward, B=1 L=32768 D=4096, "
                               "EMA ndim 16, z 1024, value 8192, 4 heads, chunk 4096, FFN 11008 SwiGLU, bf16 weights "
                               "and activations, fp32 norm / EMA parameters; TimestepNorm -> CEMA -> gated chunk "
                               "attention -> normalized FFN",
                   "global_batch": 1, "seq_len": 32768},
        "roofline": roofline,
        "cema_layer": cema,
        "other_ops": other,
    }
    if not args.no_cpu_baseline:
        cores = host_cores()
        torch.set_num_threads(cores)
        os.environ.setdefault("OMP_NUM_THREADS", str(cores))
        result["cpu_baseline"] = cpu_block(cores)
        result["host"] = host_info()
        result["cpu_ops"] = {"cema_conv_config1": cpu_cema(1, 4096, 16, 32768, 1001, cores),
                             "timestep_norm_config2": cpu_timestep_norm(cores),
                             "attention_config3": cpu_attention(cores)}
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
