#!/usr/bin/env python3
"""Benchmark of the Megalodon fused-op hot path on one MI355X.

A step is one CEMA layer forward+backward at the 7B layer width (BASELINE
config 1): k = ema_parameters(p, q, gamma) -> y = fftconv(x, k) + x*omega, then
backward through both ops to dx, d(alpha, delta, theta, gamma, omega), with
B=1, L=32768, D=4096, ndim=16, x and the upstream gradient in bf16.  The
convolution's DFT stages run on the matrix cores (fp16 operands, fp32
accumulation; twiddles, the spectral product and every sum in fp32); the same
step through the all-fp32 VALU convolution engine is timed beside it
("fp32_fft_engine").  Inputs are synthetic, seeded, and resident in HBM before
the timed region.  Prints one JSON line.
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
# HBM bytes one forward convolution launch moves at config 1 (1.11e9 of them the spectra kept for the backward): FETCH_SIZE x 2.0 + WRITE_SIZE x 1.0 from
# two rocprofv3 --pmc passes of this script, the factors being what the same counters read for a plain
# copy of 2^30 bytes (--copy-calibration).  A measured constant: counters cannot be read from in here.
FFTCONV_TRAFFIC_BYTES = 2.49e9


def cpu_baseline(B, D, N, L, seed, budget_s=25.0):
    """The same step on the host cores through the reference's CPU formulation:
    ema_parameters by the C/OpenMP restatement of its C++ loop nest, the
    convolution by torch.fft on CPU tensors (which is the reference's CPU
    path), on a bounded slice of the channels (every loop nest is linear in D).
    """
    import torch
    from megalodon_amd import synthetic
    from oracle import native, fftconv as offt

    cores = os.cpu_count() or 1
    cores = min(cores, 16) if os.environ.get("OMP_NUM_THREADS") is None else int(os.environ["OMP_NUM_THREADS"])
    torch.set_num_threads(cores)
    os.environ.setdefault("OMP_NUM_THREADS", str(cores))
    lib = native.port()
    Ds = 512
    prm = synthetic.cema_params(D, N, seed)
    io = synthetic.cema_inputs(B, Ds, L, seed, torch.bfloat16)
    p, lq, g = prm["p"][:Ds], prm["q"][:Ds].log(), prm["gamma"][:Ds]
    om = prm["omega"][:Ds]

    def step():
        k = native.ema_weight_fwd(lib, "oracle_", p, lq, g, L)
        x = io["x"].float()
        L_ = x.shape[-1]
        n = 2 * (L_ if (L_ & (L_ - 1)) == 0 else (1 << L_.bit_length()))
        x_f = torch.fft.rfft(x, n=n)
        k_f = torch.fft.rfft(k, n=n, norm="forward")
        y = torch.fft.irfft(x_f * k_f, n=n, norm="forward")[..., :L_].to(torch.bfloat16)
        out = y + io["x"] * om
        dy = io["dy"].float()
        dy_f = torch.fft.rfft(dy.flip(dims=(-1,)), n=n)
        dx = torch.fft.irfft(dy_f * k_f, n=n, norm="forward")[..., :L_].flip(dims=(-1,)).to(torch.bfloat16)
        dk = torch.fft.irfft((dy_f * x_f).sum(dim=0), n=n)[..., :L_].flip(dims=(-1,))
        dx = dx + io["dy"] * om
        dom = (io["dy"].float() * x).sum(dim=(0, 2))
        grads = native.ema_weight_bwd(lib, "oracle_", dk, p, lq, g)
        return out, dx, dom, grads

    t0 = time.perf_counter()
    step()
    one = time.perf_counter() - t0
    reps = max(1, min(5, int(budget_s / max(one, 1e-3)) - 1))
    t0 = time.perf_counter()
    for _ in range(reps):
        step()
    dt = (time.perf_counter() - t0) / reps
    tokens_per_s = B * L / (dt * D / Ds)
    return {
        "value": tokens_per_s, "unit": "tokens/s", "cores": cores, "kind": "port",
        "sample": f"{Ds} of {D} channels, {reps} rep(s) of the full fwd+bwd step at L={L}, "
                  f"{dt:.3f} s each, scaled by D/{Ds}",
    }


def other_ops(torch, dev, synthetic):
    """TimestepNorm (config 2), chunk attention (config 3) and one block (config 4),
    timed with device events; reported beside the config-1 step."""
    def dev_ms(fn, n):
        fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / n

    from megalodon_amd import extension as ops
    other = {}
    tB, tL, tD, tG = 4, 8192, 4096, 32
    tio = {k_: v_.to(dev) for k_, v_ in synthetic.timestep_norm_inputs(tB, tL, tD, tG, 1002).items()}
    tE = tB * tL * tD
    fwd = lambda: ops.group_timestep_norm_fwd(tio["x"], tio["prev_count"], tio["prev_mean"], tio["prev_var"],
                                              tio["gamma"], tio["beta"], tio["mask"], tG, 1e-5)
    ty, tcount, tmean, tvar, tcm, tcr = fwd()
    ms = dev_ms(fwd, 10)
    # GBps / frac_hbm price the op at its 4E (6E) algorithmic bytes; padding rows
    # are written (zeros) but never read, so GBps_moved counts them once less
    live = 1.0 - float(tio["mask"].float().mean()) if tio.get("mask") is not None else 1.0
    other["timestep_norm_fwd"] = {"ms": ms, "GBps": 4 * tE / ms / 1e6, "frac_hbm": 4 * tE / ms / 1e6 / HBM_PEAK_GBS,
                                  "unmasked_steps": live, "GBps_moved": (2 + 2 * live) * tE / ms / 1e6}
    ms = dev_ms(lambda: ops.group_timestep_norm_bwd(tio["dy"], tio["dmean"], tio["dvar"], tio["x"], tio["prev_mean"],
                                                    tcount, tcm, tcr, tio["gamma"], tio["mask"], tG), 10)
    other["timestep_norm_bwd"] = {"ms": ms, "GBps": 6 * tE / ms / 1e6, "frac_hbm": 6 * tE / ms / 1e6 / HBM_PEAK_GBS,
                                  "unmasked_steps": live, "GBps_moved": (2 + 4 * live) * tE / ms / 1e6}
    del tio, ty, tcm, tcr
    aio = {k_: v_.to(dev) for k_, v_ in synthetic.attention_inputs(8, 4096, 4, 256, 2048, 1003).items()}
    pairs = 4096 * 4097 // 2
    f_fwd, f_bwd = 2 * pairs * (256 + 2048) * 32, 2 * pairs * (2 * 256 + 2 * 2048) * 32
    ay, aw = ops.attention_fwd(aio["q"], aio["k"], aio["v"], 1.0, 0.0, True)
    ms = dev_ms(lambda: ops.attention_fwd(aio["q"], aio["k"], aio["v"], 1.0, 0.0, True), 3)
    other["attention_fwd"] = {"ms": ms, "TFLOPs": f_fwd / ms / 1e9, "frac_mfma_bf16": f_fwd / ms / 1e9 / 2516.6}
    ms = dev_ms(lambda: ops.attention_bwd(aio["dy"], aio["q"], aio["k"], aio["v"], aw, 1.0, True), 3)
    other["attention_bwd"] = {"ms": ms, "TFLOPs": f_bwd / ms / 1e9, "frac_mfma_bf16": f_bwd / ms / 1e9 / 2516.6}
    del aio, ay, aw
    torch.cuda.empty_cache()

    # config 4: one full 7B-style block forward+backward (random init std 0.02, bf16)
    from megalodon_amd.modules import MegaBlock
    torch.manual_seed(1004)
    blk = MegaBlock(model_dim=4096, z_dim=1024, value_dim=8192, num_heads=4, cema_ndim=16, chunk_size=4096,
                    ffn_hidden_dim=11008, norm_num_groups=32).to(dev).bfloat16()
    gb = torch.Generator().manual_seed(1004)
    bx = (torch.rand(1, 32768, 4096, generator=gb) * 2 - 1).bfloat16().to(dev).requires_grad_(True)
    bdy = torch.randn(1, 32768, 4096, generator=gb).bfloat16().to(dev)

    def block_step():
        bx.grad = None
        for prm in blk.parameters():
            prm.grad = None
        o, _ = blk(bx)
        o.backward(bdy)

    block_step()
    torch.cuda.synchronize()
    tb0 = time.perf_counter()
    for _ in range(3):
        block_step()
    torch.cuda.synchronize()
    bms = (time.perf_counter() - tb0) / 3 * 1e3
    other["block_config4_fwd_bwd"] = {"ms": bms, "tokens_per_s": 32768 / (bms * 1e-3)}
    del blk, bx, bdy
    torch.cuda.empty_cache()
    return other


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--skip-other-ops", action="store_true",
                    help="time only the config-1 step (short runs under a profiler)")
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
    from megalodon_amd import _lib, synthetic
    from megalodon_amd.modules import MultiHeadComplexEMA

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    _lib.load()  # fails loudly when the HIP library is missing
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    B, D, N, L, seed = 1, 4096, 16, 32768, 1001

    layer = MultiHeadComplexEMA(D, N).to(dev)
    layer.train()
    io = synthetic.cema_inputs(B, D, L, seed, torch.bfloat16)
    x = io["x"].to(dev).requires_grad_(True)
    dy = io["dy"].to(dev)

    def step():
        x.grad = None
        for prm in layer.parameters():
            prm.grad = None
        out, _ = layer(x, None, False)
        out.backward(dy.to(out.dtype))

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()

    log = {"mega_fftconv_residual_fwd_saving": [], "mega_fftconv_residual_bwd_saved": [],
           "mega_ema_weight_fwd": [], "mega_ema_weight_bwd": []}
    _lib.set_event_log(log)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    _lib.set_event_log(None)

    def avg_ms(name):
        ev = log[name]
        return sum(a.elapsed_time(b) for a, b in ev) / max(1, len(ev))

    E = B * D * L
    ms_step = dt / args.steps * 1e3
    conv_ms = avg_ms("mega_fftconv_residual_fwd_saving")  # one launch of the convolution kernel
    conv_bytes = 8 * E  # x 2E + k 4E in, y 2E out (bf16 rows, fp32 kernel); the saved spectra are not counted
    achieved = conv_bytes / (conv_ms * 1e-3) / 1e9
    kernels = {
        "fftconv_fwd_ms": conv_ms,
        "fftconv_bwd_ms": avg_ms("mega_fftconv_residual_bwd_saved"),
        "ema_weight_fwd_ms": avg_ms("mega_ema_weight_fwd"),
        "ema_weight_bwd_ms": avg_ms("mega_ema_weight_bwd"),
    }
    # dy 2E in, dx 2E + dk 4E out; x and k are not read again (their spectra are: not counted)
    kernels["fftconv_bwd_GBps"] = 8 * E / (kernels["fftconv_bwd_ms"] * 1e-3) / 1e9
    kernels["ema_weight_fwd_GBps"] = 4 * E / (kernels["ema_weight_fwd_ms"] * 1e-3) / 1e9
    kernels["ema_weight_bwd_GBps"] = 4 * E / (kernels["ema_weight_bwd_ms"] * 1e-3) / 1e9

    # the same step with every FFT butterfly in fp32 on the vector ALUs
    fp32_engine = None
    if not args.skip_other_ops:
        os.environ["MEGA_FFTCONV_VALU"] = "1"
        try:
            step()
            torch.cuda.synchronize()
            n32 = max(1, min(5, args.steps))
            t1 = time.perf_counter()
            for _ in range(n32):
                step()
            torch.cuda.synchronize()
            dt32 = (time.perf_counter() - t1) / n32
        finally:
            os.environ.pop("MEGA_FFTCONV_VALU", None)
        fp32_engine = {"ms_per_step": dt32 * 1e3, "tokens_per_s": B * L / dt32, "steps": n32}

    if args.copy_calibration:
        src = torch.ones(1 << 29, dtype=torch.bfloat16, device=dev)
        dst = torch.empty_like(src)
        torch.mul(src, 1.0, out=dst)  # reads 2^30 bytes, writes 2^30 bytes
        torch.cuda.synchronize()
        del src, dst

    other = {}
    if not args.skip_other_ops:
        other = other_ops(torch, dev, synthetic)
    result = {
        "metric": "Megalodon layer fwd+bwd tokens/s at L=32K, 1 GPU; CEMA+FFT-conv HBM GB/s (% peak)",
        "value": B * L / (dt / args.steps),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16*f16+f32",
        "data": "synthetic",
        "config": {"workload": "configs[1]: CEMA + causal FFT convolution forward+backward, "
                               "B=1 L=32768 D=4096 ndim=16, x/dy bf16, k/dk fp32; DFT stages fp16 operands "
                               "with fp32 accumulation on the matrix cores, everything else fp32",
                   "global_batch": B, "seq_len": L},
        "roofline": {
            "bound": "hbm", "kernel": "fftconv_mfma_kernel<bf16, MODE=0> (one launch = forward conv of all rows, skip term "
                                      "included, spectra of x and k kept for the backward launch)",
            "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBS, "traffic": FFTCONV_TRAFFIC_BYTES,
        },
        "kernels": kernels,
        "fp32_fft_engine": fp32_engine,
        "other_ops": other,
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(B, D, N, L, seed)
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
