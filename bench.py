#!/usr/bin/env python3
"""Benchmark of the SFNO spectral hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload sht_pair|spectral_block|sfno8l|rollout|fft2_pair|pointwise_backward|train_step]

Default workload (the configuration the headline metric is quoted on): forward + inverse
real SHT at 721x1440 (equiangular, lmax = mmax = 721), batch 1, 73 channels, float32,
through the reference-layout module interface (RealSHT.forward then
InverseRealSHT.forward).  One step = one such pair with the input already resident in
HBM.  Prints ONE JSON line; `roofline` describes the dominant kernel (the Legendre
contraction) from HIP-event timings taken in this run, `cpu_baseline` is the PyTorch-CPU
restatement of the reference op sequence timed on this host on the whole workload
(--quick: on a channel sample).  The default run appends the other configurations of the
metric as extra keys, each with its own roofline and CPU baseline: the SFNO-8L forward
(configs[3], with every kernel class timed at its in-model shape), one spectral block
(configs[2], fp32 and bf16), the batch-4 rollout (configs[4]) and the Legendre stage on the
fp32 matrix instruction.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "modulus-makani_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

PEAK_FP32_MFMA_TFLOPS = 157.3
PEAK_BF16_MFMA_TFLOPS = 2500.0       # dense bf16 and fp16
PEAK_HBM_GBS = 8000.0


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="sht_pair", choices=["sht_pair", "spectral_block", "sfno8l", "rollout", "fft2_pair", "pointwise_backward", "train_step"])
    ap.add_argument("--no-sfno", action="store_true", help="skip the SFNO-8L forward timing appended to the default run")
    ap.add_argument("--compute", default="fp32", choices=["fp32", "fp32_bf16x3", "bf16", "fp32_mfma"],
                    help="arithmetic of the Legendre and dhconv contractions: fp32 (reference precision: operands scaled and cut into two fp16 parts, "
                         "three products on the fp16 matrix pipe), fp32_bf16x3 (three exact bf16 parts, six products), fp32_mfma (transform pair only: "
                         "the fp32 matrix instruction) or bf16 MFMA inputs with fp32 accumulation")
    ap.add_argument("--no-extras", action="store_true", help="skip the spectral-block, rollout and fp32-MFMA figures appended to the default run")
    ap.add_argument("--quick", action="store_true", help="CPU baselines on a channel sample (scaled) instead of the whole workload")
    ap.add_argument("--rollout-steps", type=int, default=12, help="autoregressive steps timed by --workload rollout")
    ap.add_argument("--rollout-warmup", type=int, default=2)
    ap.add_argument("--batch", type=int, default=1, help="--workload spectral_block: samples per step (configs[2] is batch 1)")
    ap.add_argument("--backward", action="store_true", help="--workload spectral_block: time forward + backward (input and weight gradients)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-library-leg", action="store_true", help="--workload train_step: skip the same step with PyTorch's library convolutions")
    ap.add_argument("--yardstick", action="store_true",
                    help="also run one plain 256 MiB elementwise copy (mul by 1): the known-size reference for FETCH_SIZE/WRITE_SIZE runs")
    ap.add_argument("--cpu-sample-channels", type=int, default=4)
    return ap.parse_args()


def event_time_ms(fn, iters, stream):
    """Average duration of fn() over `iters` launches, HIP events on the launch stream."""
    import torch

    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    fn()
    torch.cuda.synchronize()
    start.record(stream)
    for _ in range(iters):
        fn()
    stop.record(stream)
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / iters


def triangular_count(lmax, mmax):
    return sum(max(0, lmax - m) for m in range(mmax))


def make_fields(isht, channels, device):
    """Band-limited Gaussian random fields: spectral coefficients with ~l^-2 power, unit variance per channel."""
    import torch

    lmax, mmax = isht.lmax, isht.mmax
    coeffs = torch.zeros(1, channels, lmax, mmax, dtype=torch.complex64)
    scale = 1.0 / (torch.arange(lmax, dtype=torch.float32) + 1.0)
    tri = torch.tril(torch.ones(lmax, mmax))          # m <= l
    for c in range(channels):
        g = torch.Generator().manual_seed(1000 + c)
        a = torch.complex(torch.randn(lmax, mmax, generator=g), torch.randn(lmax, mmax, generator=g)) / (2.0 ** 0.5)
        a = a * scale[:, None] * tri
        a[:, 0] = a[:, 0].real.to(torch.complex64)
        if mmax == isht.nlon // 2 + 1:
            a[:, -1] = 0
        coeffs[0, c] = a
    x = isht(coeffs.to(device))
    x = x - x.mean(dim=(-2, -1), keepdim=True)
    x = x / x.std(dim=(-2, -1), keepdim=True)
    return x.contiguous()


def csrc_hash():
    """sha256 over the kernel and host sources the library is built from (file names and contents, sorted)."""
    import hashlib

    h = hashlib.sha256()
    csrc = os.path.join(ROOT, "modulus-makani_amd", "csrc")
    files = sorted(os.path.join(csrc, f) for f in os.listdir(csrc)) + [os.path.join(ROOT, "include", "sfno_spectral.h")]
    for f in files:
        h.update(os.path.basename(f).encode())
        with open(f, "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()[:16]


def read_traffic(key, note=None):
    """HBM bytes per launch from the committed rocprofv3 counter summary -- only if that summary was taken on the kernel
    sources this run was built from (profiles/traffic.json records their hash); otherwise None, with the reason in `note`."""
    path = os.path.join(ROOT, "profiles", "traffic.json")
    try:
        with open(path) as f:
            t = json.load(f)
    except (OSError, ValueError):
        return None
    entry = t.get(key)
    if entry is None:
        return None
    if not isinstance(entry, dict) or entry.get("csrc_sha") != csrc_hash():
        if note is not None:
            note.append(f"profiles/traffic.json[{key}] was measured on other kernel sources "
                        f"({entry.get('csrc_sha') if isinstance(entry, dict) else 'no hash recorded'} != {csrc_hash()}): not reported")
        return None
    return entry.get("bytes")


def cpu_threads():
    import torch

    torch.set_num_threads(os.cpu_count() if (os.cpu_count() or 1) <= 64 else 64)
    return torch.get_num_threads()


def cpu_baseline_sht_pair(nlat, nlon, lmax, mmax, grid, channels, sample=None):
    """Times the reference op sequence (dense fp32 tables, torch.fft + torch.einsum) on the host cores: the whole workload
    (all channels), or -- sample = n -- n channels scaled by n / channels."""
    import torch
    from oracle.torch_ref import TorchRefSHT

    cores = cpu_threads()
    ref = TorchRefSHT(nlat, nlon, lmax, mmax, grid)
    n = channels if not sample else min(sample, channels)
    x = torch.randn(1, n, nlat, nlon, generator=torch.Generator().manual_seed(7))
    times = []
    for it in range(4):
        t0 = time.perf_counter()
        y = ref.inverse(ref.forward(x))
        dt = time.perf_counter() - t0
        if it:
            times.append(dt)
    assert y.shape == x.shape
    t = min(times)
    times.sort()
    what = (f"the whole workload: {channels} channels" if n == channels else
            f"{n} of {channels} channels, scaled by {n}/{channels} (the pair is linear in the number of channels)")
    return {
        "value": (1.0 / t) * (n / channels),
        "unit": "pairs/s",
        "cores": cores,
        "kind": "port",
        "sample": f"{what}, full {nlat}x{nlon} grid, all orders, dense fp32 tables; best of 3 after 1 warm-up "
                  f"({t:.3f} s, median {times[1]:.3f} s)",
    }


def cpu_baseline_spectral_block(nlat, nlon, L, M, grid, C, weight, sample=None):
    """configs[2] on the host cores: rfft -> two einsums -> the dhconv einsum (contractions.py:134) -> two einsums -> irfft."""
    import torch
    from oracle.torch_ref import TorchRefSHT

    cores = cpu_threads()
    ref = TorchRefSHT(nlat, nlon, L, M, grid)
    w = weight.detach().cpu()
    x = torch.randn(1, C, nlat, nlon, generator=torch.Generator().manual_seed(2))
    times = []
    for it in range(3):
        t0 = time.perf_counter()
        y = ref.inverse(torch.einsum("bixy,iox->boxy", ref.forward(x), w))
        if it:
            times.append(time.perf_counter() - t0)
    assert y.shape == x.shape
    return {"value": 1.0 / min(times), "unit": "blocks/s", "cores": cores, "kind": "port",
            "sample": f"the whole block ({C} channels, {nlat}x{nlon}), best of 2 after 1 warm-up ({min(times):.3f} s)"}


def bench_sht_pair(args):
    import torch
    import makani_amd as ma
    from makani_amd._lib import lib, check

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    nlat, nlon, lmax, mmax, grid, C = 721, 1440, 721, 721, "equiangular", 73
    sht = ma.RealSHT(nlat, nlon, lmax=lmax, mmax=mmax, grid=grid, compute=args.compute)
    isht = ma.InverseRealSHT(nlat, nlon, lmax=lmax, mmax=mmax, grid=grid, compute=args.compute)
    x = make_fields(isht, C, dev)
    torch.cuda.synchronize()

    def step():
        return isht(sht(x))

    if args.yardstick:
        src = torch.ones(64 * 1024 * 1024, dtype=torch.float32, device=dev)
        dst = torch.mul(src, 1.0)            # reads 256 MiB, writes 256 MiB
        del src, dst
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        y = step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt / args.steps * 1e3
    assert torch.isfinite(y).all()

    # ---- per-stage timings (HIP events on the launch stream) ----------------------------------
    stream = torch.cuda.current_stream(dev)
    sp = ctypes.c_void_p(stream.cuda_stream)
    rows = C
    pf, pi = sht.plan(dev).handle, isht.plan(dev).handle
    xm = torch.empty(lib.sfno_fourier_elems(pf, rows), dtype=torch.float32, device=dev)
    spec = torch.empty(lib.sfno_spectral_elems(pf, rows), dtype=torch.float32, device=dev)
    coeffs = torch.empty(1, C, lmax, mmax, dtype=torch.complex64, device=dev)
    out = torch.empty_like(x)
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    stages = {
        "rfft": lambda: check(lib.sfno_rfft(pf, P(x), 0, P(xm), rows, sp), "rfft"),
        "legendre_analysis": lambda: check(lib.sfno_legendre_analysis(pf, P(xm), P(spec), rows, sp), "legendre_analysis"),
        "spectral_to_coeffs": lambda: check(lib.sfno_spectral_to_coeffs(P(spec), P(coeffs), rows, lmax, mmax, 1, sp), "to_coeffs"),
        "coeffs_to_spectral": lambda: check(lib.sfno_coeffs_to_spectral(P(coeffs), P(spec), rows, lmax, mmax, 1, sp), "to_spectral"),
        "legendre_synthesis": lambda: check(lib.sfno_legendre_synthesis(pi, P(spec), P(xm), rows, sp), "legendre_synthesis"),
        "irfft": lambda: check(lib.sfno_irfft(pi, P(xm), P(out), 0, rows, sp), "irfft"),
    }
    stage_ms = {}
    for name, fn in stages.items():      # run in pipeline order so every buffer holds real data
        stage_ms[name] = event_time_ms(fn, max(5, args.steps), stream)

    T = triangular_count(lmax, mmax)
    leg_flops = 4.0 * rows * nlat * T                 # 2 flop/MAC, Re and Im
    dom = max(("legendre_analysis", "legendre_synthesis"), key=lambda k: stage_ms[k])
    achieved = leg_flops / (stage_ms[dom] * 1e-3) / 1e12
    # algorithmic bytes of the Legendre stage: Fourier panel + triangular table (fp32 or bf16 entries) + triangular coefficients
    Tp = sum(min(l + 1, mmax) for l in range(lmax))
    leg_bytes = rows * nlat * mmax * 8 + T * nlat * (2 if args.compute == "bf16" else 4) + rows * Tp * 8
    hbm_gbs = leg_bytes / (stage_ms[dom] * 1e-3) / 1e9
    mfma_view = {"achieved": achieved, "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s", "frac": achieved / PEAK_FP32_MFMA_TFLOPS,
                 "algorithmic_flops_per_launch": leg_flops}
    kname = f"{'legendre_f16_kernel' if args.compute == 'fp32' else 'legendre_fold_kernel'} ({dom})"
    if args.compute == "fp32_mfma":
        # contraction on the fp32 matrix instruction: 45 flop per byte, above the fp32 ridge (19.7)
        roofline = {"kernel": kname, "bound": "mfma", **mfma_view, "traffic": None,
                    "avg_launch_ms": stage_ms[dom],
                    "note": "algorithmic (triangular) fp32 flops over the kernel's time; the kernel executes half of those MACs (equator fold)"}
    else:
        # contraction on the fp16 / bf16 matrix pipe (fp32 operands cut into two fp16 or three bf16 parts, or bf16 operands): 45 flop per
        # byte is far below that pipe's ridge (312), so HBM is the roofline that bounds the kernel
        tnote = []
        # what the matrix pipe executes: half the algorithmic MACs (equator fold), each as three fp16 / six bf16 products (one in bf16 mode)
        products = {"fp32": 3, "fp32_bf16x3": 6, "bf16": 1}[args.compute]
        executed = leg_flops / 2 * products
        how = {"fp32": " and forms every fp32 product from three fp16 MFMA partial products of operands scaled by powers of two and cut into two fp16 "
                       "parts (4-byte table entries)",
               "fp32_bf16x3": " and forms every fp32 product from six bf16 MFMA partial products of exactly split operands (6-byte table entries)",
               "bf16": ""}[args.compute]
        roofline = {"kernel": kname, "bound": "hbm", "achieved": hbm_gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                    "frac": hbm_gbs / PEAK_HBM_GBS, "traffic": read_traffic(dom, tnote) if args.compute == "fp32" else None,
                    "algorithmic_bytes_per_launch": leg_bytes,
                    "avg_launch_ms": stage_ms[dom], "against_fp32_mfma_peak": mfma_view,
                    "executed_on_matrix_pipe": {"products_per_mac": products, "flops_per_launch": executed,
                                                "achieved_TFLOPs": executed / (stage_ms[dom] * 1e-3) / 1e12,
                                                "peak_TFLOPs": PEAK_BF16_MFMA_TFLOPS, "frac": executed / (stage_ms[dom] * 1e-3) / 1e12 / PEAK_BF16_MFMA_TFLOPS},
                    "traffic_note": tnote[0] if tnote else None,
                    "note": ("algorithmic bytes = Fourier panel + triangular table at the reference's element size + triangular coefficients, "
                             "each moved once; the kernel folds the equator (half the MACs and table entries)" + how
                             + (f", which takes the contraction off the fp32 matrix roofline: against that peak the same launch reads "
                                f"{achieved:.0f} of {PEAK_FP32_MFMA_TFLOPS} TFLOP/s" if products > 1 else ""))}
    fft_bytes = rows * nlat * nlon * 4 + rows * nlat * mmax * 8
    result = {
        "metric": "SHT fwd+inv/s @721x1440",
        "value": args.steps / dt,
        "unit": "pairs/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32" if args.compute != "bf16" else "bf16 MFMA inputs, f32 accumulate (FFT f32)",
        "data": "synthetic",
        "compute": args.compute,
        "config": {
            "workload": "configs[1]: RealSHT + InverseRealSHT, equiangular 721x1440, lmax=mmax=721, batch 1, 73 channels, "
                        "band-limited Gaussian random fields (l^-2 power, unit variance)",
            "nlat": nlat, "nlon": nlon, "lmax": lmax, "mmax": mmax, "batch": 1, "channels": C,
        },
        "roofline": roofline,
        "stages_ms": stage_ms,
        "fft_hbm": {
            "rfft_GBps": fft_bytes / (stage_ms["rfft"] * 1e-3) / 1e9,
            "irfft_GBps": fft_bytes / (stage_ms["irfft"] * 1e-3) / 1e9,
            "rfft_frac": fft_bytes / (stage_ms["rfft"] * 1e-3) / 1e9 / PEAK_HBM_GBS,
            "irfft_frac": fft_bytes / (stage_ms["irfft"] * 1e-3) / 1e9 / PEAK_HBM_GBS,
            "peak_GBps": PEAK_HBM_GBS,
            "algorithmic_bytes_per_launch": fft_bytes,
        },
    }
    if not args.no_cpu_baseline:
        del xm, spec, coeffs, out
        result["cpu_baseline"] = cpu_baseline_sht_pair(nlat, nlon, lmax, mmax, grid, C, args.cpu_sample_channels if args.quick else None)
    return result


def bench_fft2_pair(args):
    """The planar pair RealFFT2 + InverseRealFFT2 (layers.py:219-287) at the full-resolution shape of configs[1], 720x1440."""
    import torch
    import makani_amd as ma
    from makani_amd._lib import lib, check

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    nlat, nlon, C = 720, 1440, 73
    fwd, inv = ma.RealFFT2(nlat, nlon), ma.InverseRealFFT2(nlat, nlon)
    lmax, mmax = fwd.lmax, fwd.mmax
    x = torch.randn(1, C, nlat, nlon, device=dev, generator=torch.Generator(dev).manual_seed(3))

    def step():
        return inv(fwd(x))

    if args.yardstick:
        src = torch.ones(64 * 1024 * 1024, dtype=torch.float32, device=dev)
        dst = torch.mul(src, 1.0)            # reads 256 MiB, writes 256 MiB
        del src, dst
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        y = step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    assert float((y - x).abs().max()) < 1e-4

    stream = torch.cuda.current_stream(dev)
    sp = ctypes.c_void_p(stream.cuda_stream)
    rows = C
    pf, pi = fwd.plan(dev).handle, inv.plan(dev).handle
    xm = torch.empty(lib.sfno_fourier_elems(pf, rows), dtype=torch.float32, device=dev)
    spec = torch.empty(lib.sfno_spectral_elems(pf, rows), dtype=torch.float32, device=dev)
    coeffs = torch.empty(1, C, lmax, mmax, dtype=torch.complex64, device=dev)
    out = torch.empty_like(x)
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    stages = {
        "rfft": lambda: check(lib.sfno_rfft(pf, P(x), 0, P(xm), rows, sp), "rfft"),
        "latitude_fft": lambda: check(lib.sfno_legendre_analysis(pf, P(xm), P(spec), rows, sp), "latitude_fft"),
        "spectral_to_coeffs": lambda: check(lib.sfno_spectral_to_coeffs(P(spec), P(coeffs), rows, lmax, mmax, 0, sp), "to_coeffs"),
        "coeffs_to_spectral": lambda: check(lib.sfno_coeffs_to_spectral(P(coeffs), P(spec), rows, lmax, mmax, 0, sp), "to_spectral"),
        "latitude_ifft": lambda: check(lib.sfno_legendre_synthesis(pi, P(spec), P(xm), rows, sp), "latitude_ifft"),
        "irfft": lambda: check(lib.sfno_irfft(pi, P(xm), P(out), 0, rows, sp), "irfft"),
    }
    stage_ms = {name: event_time_ms(fn, max(5, args.steps), stream) for name, fn in stages.items()}
    dom = max(("latitude_fft", "latitude_ifft"), key=lambda k: stage_ms[k])
    lat_bytes = rows * mmax * (nlat + lmax) * 8          # every Fourier coefficient read once and every kept coefficient written once
    gbs = lat_bytes / (stage_ms[dom] * 1e-3) / 1e9
    result = {
        "metric": "FFT2 fwd+inv/s @720x1440",
        "value": args.steps / dt,
        "unit": "pairs/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": dt / args.steps * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "RealFFT2 + InverseRealFFT2 (spectral_transform='fft'), 720x1440, all modes, batch 1, 73 channels, Gaussian random fields"},
        "roofline": {"kernel": f"latfft_kernel ({dom})", "bound": "hbm", "achieved": gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": gbs / PEAK_HBM_GBS, "traffic": read_traffic("fft2_" + dom), "algorithmic_bytes_per_launch": lat_bytes,
                     "avg_launch_ms": stage_ms[dom]},
        "stages_ms": stage_ms,
    }
    if not args.no_cpu_baseline:
        from oracle.torch_ref import TorchRefFFT2

        cpu_threads()
        ref = TorchRefFFT2(nlat, nlon)
        xs = (x[:, : 2 * args.cpu_sample_channels] if args.quick else x).cpu()
        times = []
        for it in range(4):
            t0 = time.perf_counter()
            ys = ref.inverse(ref.forward(xs))
            if it:
                times.append(time.perf_counter() - t0)
        t = min(times)
        n = xs.shape[1]
        result["cpu_baseline"] = {"value": (1.0 / t) * (n / C), "unit": "pairs/s", "cores": torch.get_num_threads(), "kind": "port",
                                  "sample": f"{n} of {C} channels, torch.fft.rfft2 + irfft2 (the reference's own ops) in float32, best of 3 after "
                                            f"1 warm-up ({t:.3f} s), scaled by {n}/{C}"}
    return result


def bench_spectral_block(args):
    """configs[2]: forward SHT -> dhconv -> inverse SHT on a 241x480 Legendre-Gauss grid, 384 channels."""
    import torch
    import makani_amd as ma

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    nlat, nlon, L, M, C = 241, 480, 241, 241, 384
    sht = ma.RealSHT(nlat, nlon, lmax=L, mmax=M, grid="legendre-gauss", compute=args.compute)
    isht = ma.InverseRealSHT(nlat, nlon, lmax=L, mmax=M, grid="legendre-gauss", compute=args.compute)
    conv = ma.SpectralConv(sht, isht, C, C, operator_type="dhconv", compute=args.compute).to(dev)
    g = torch.Generator().manual_seed(3)
    w = torch.complex(torch.randn(C, C, L, generator=g), torch.randn(C, C, L, generator=g)) / (2.0 ** 0.5) * (1.0 / C) ** 0.5
    with torch.no_grad():
        conv.weight.copy_(w.to(dev))
    B = max(1, args.batch)
    R = B * C                               # rows of the transforms
    x = torch.randn(B, C, nlat, nlon, generator=torch.Generator().manual_seed(2)).to(dev)
    Tp = sum(min(l + 1, M) for l in range(L))
    dh_flops = 8.0 * B * C * C * Tp
    leg_flops = 4.0 * R * nlat * triangular_count(L, M)
    if args.backward:
        # forward + backward (input and weight gradients) through the adjoint kernels: twice the transform work and
        # three times the channel mix of the forward pass
        x.requires_grad_(True)
        gy = torch.randn(B, C, nlat, nlon, generator=torch.Generator().manual_seed(6)).to(dev)

        def step():
            conv.weight.grad = None
            x.grad = None
            y, _ = conv(x)
            y.backward(gy)
            return y

        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            y = step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        assert torch.isfinite(x.grad).all() and torch.isfinite(torch.view_as_real(conv.weight.grad)).all()
        flops = 3 * dh_flops + 4 * leg_flops
        return {
            "metric": "spectral block fwd+bwd/s @241x480x384",
            "value": args.steps / dt,
            "unit": "blocks/s",
            "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": dt / args.steps * 1e3,
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "f32" if args.compute != "bf16" else "bf16 MFMA inputs, f32 accumulate (FFT f32)", "data": "synthetic",
            "config": {"workload": "configs[2] with its backward pass: SHT -> dhconv -> inverse SHT, gradients of the input and of the weight"},
            "useful_TFLOPs_per_step": flops / 1e12,
            "achieved_TFLOPs": flops / (dt / args.steps) / 1e12,
        }
    if args.yardstick:
        src = torch.ones(64 * 1024 * 1024, dtype=torch.float32, device=dev)
        dst = torch.mul(src, 1.0)            # reads 256 MiB, writes 256 MiB
        del src, dst
    with torch.no_grad():
        for _ in range(args.warmup):
            conv(x)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            y, _ = conv(x)
        torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    assert torch.isfinite(y).all()
    # the five kernels of the block, each timed on its own through the C ABI on the block's own plans and weight
    from makani_amd._lib import lib, check
    from makani_amd.contractions import dhconv_spectral

    stream = torch.cuda.current_stream(dev)
    sp = ctypes.c_void_p(stream.cuda_stream)
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    pf, pi = sht.plan(dev).handle, isht.plan(dev).handle
    xm = torch.empty(lib.sfno_fourier_elems(pf, R), dtype=torch.float32, device=dev)
    spec = torch.empty(lib.sfno_spectral_elems(pf, R), dtype=torch.float32, device=dev)
    out = torch.empty_like(x)
    iters = max(5, args.steps)
    with torch.no_grad():
        stages = {
            "rfft": event_time_ms(lambda: check(lib.sfno_rfft(pf, P(x), 0, P(xm), R, sp), "rfft"), iters, stream),
            "legendre_analysis": event_time_ms(lambda: check(lib.sfno_legendre_analysis(pf, P(xm), P(spec), R, sp), "analysis"), iters, stream),
            "dhconv": event_time_ms(lambda: dhconv_spectral(spec, conv.weight, B, M, compute=args.compute), iters, stream),
            "legendre_synthesis": event_time_ms(lambda: check(lib.sfno_legendre_synthesis(pi, P(spec), P(xm), R, sp), "synthesis"), iters, stream),
            "irfft": event_time_ms(lambda: check(lib.sfno_irfft(pi, P(xm), P(out), 0, R, sp), "irfft"), iters, stream),
        }
    wbytes = 4 if args.compute == "bf16" else 8
    work = {   # algorithmic bytes per launch
        "rfft": R * nlat * nlon * 4 + R * nlat * M * 8, "irfft": R * nlat * nlon * 4 + R * nlat * M * 8,
        "legendre_analysis": R * nlat * M * 8 + triangular_count(L, M) * nlat * (2 if args.compute == "bf16" else 4) + R * Tp * 8,
        "dhconv": C * C * L * wbytes + 2 * R * Tp * 8,
    }
    work["legendre_synthesis"] = work["legendre_analysis"]
    dom = max(stages, key=lambda k: stages[k])
    gbs = work[dom] / (stages[dom] * 1e-3) / 1e9
    res = {
        "metric": "spectral block fwd/s @241x480x384",
        "value": args.steps / dt,
        "batch": B,
        "unit": "blocks/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": dt / args.steps * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32" if args.compute != "bf16" else "bf16 MFMA inputs, f32 accumulate (FFT f32)", "data": "synthetic", "compute": args.compute,
        "config": {"workload": f"configs[2]: SHT -> dhconv -> inverse SHT, legendre-gauss 241x480, lmax=mmax=241, batch {B}, 384 channels"},
        "useful_TFLOPs_per_step": (dh_flops + 2 * leg_flops) / 1e12,
        "achieved_TFLOPs": (dh_flops + 2 * leg_flops) / (dt / args.steps) / 1e12,
        "stages_ms": stages,
        # at batch 1 every kernel of the block is below the ridge of the matrix pipe it runs on: HBM bounds it
        "roofline": {"kernel": dom, "bound": "hbm", "achieved": gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": gbs / PEAK_HBM_GBS,
                     "traffic": read_traffic(("block_" if B == 1 else f"block_b{B}_") + dom) if args.compute == "fp32" else None,
                     "algorithmic_bytes_per_launch": work[dom],
                     "avg_launch_ms": stages[dom],
                     "per_stage_frac": {k: work[k] / (stages[k] * 1e-3) / 1e9 / PEAK_HBM_GBS for k in stages}},
    }
    if not args.no_cpu_baseline and B == 1:
        del xm, spec, out
        res["cpu_baseline"] = cpu_baseline_spectral_block(nlat, nlon, L, M, "legendre-gauss", C, conv.weight)
    return res


def build_sfno8l(dev, compute="fp32"):
    """SFNO-linear, 8 layers, embed 384, scale factor 3, 73 channels in/out (config/sfnonet.yaml:24-40,149-174), random init."""
    import torch
    from makani_amd.sfnonet import SphericalFourierNeuralOperatorNet

    torch.manual_seed(4)
    net = SphericalFourierNeuralOperatorNet(inp_shape=(721, 1440), out_shape=(721, 1440), scale_factor=3, inp_chans=73, out_chans=73,
                                            embed_dim=384, num_layers=8, use_mlp=True, mlp_ratio=2.0, activation_function="gelu",
                                            normalization_layer="instance_norm", big_skip=True, operator_type="dhconv", filter_type="linear",
                                            spectral_compute=compute)
    return net.to(dev).eval()


def time_sfno_forward(batch, iters, warmup, dev, compute="fp32"):
    """Median forward time (ms) of the SFNO-8L under bf16 autocast, inference mode, HIP events."""
    import torch

    net = build_sfno8l(dev, compute)
    x = torch.randn(batch, 73, 721, 1440, generator=torch.Generator().manual_seed(5)).to(dev)
    times = []
    with torch.inference_mode(), torch.autocast("cuda", dtype=torch.bfloat16):
        for _ in range(warmup):
            y = net(x)
        torch.cuda.synchronize()
        for _ in range(iters):
            s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s.record()
            y = net(x)
            e.record()
            torch.cuda.synchronize()
            times.append(s.elapsed_time(e))
    assert torch.isfinite(y.float()).all()
    times.sort()
    return times[len(times) // 2], times[0], net, x


def sfno_kernel_classes(dev, net, iters=10):
    """Every kernel class of the SFNO-8L forward (batch 1) timed on its own at its in-model shape with HIP events, next to the
    work the class does per launch and the roofline that bounds it.  Transform stages go through the C ABI on the network's own
    plans, the 1x1 convolutions through the fused kernels on the network's own weights.  Returns {class: {...}} with calls per
    forward, so that sum(calls * ms) can be held against the measured forward time."""
    import torch
    import makani_amd.pointwise as pw
    from makani_amd import _lib
    from makani_amd._lib import lib, check

    stream = torch.cuda.current_stream(dev)
    sp = ctypes.c_void_p(stream.cuda_stream)
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    C = net.embed_dim
    out = {}

    def hbm(name, calls, ms, nbytes):
        out[name] = {"calls": calls, "ms": ms, "bound": "hbm", "algorithmic_bytes": nbytes, "achieved_GBps": nbytes / ms / 1e6,
                     "frac": nbytes / ms / 1e6 / PEAK_HBM_GBS}

    def mfma(name, calls, ms, flops, nbytes):
        # bf16 matrix pipe; at these shapes the byte stream is the binding roof when bytes / 8 TB/s exceeds flops / 2.5 PFLOP/s
        t_hbm, t_pipe = nbytes / (PEAK_HBM_GBS * 1e9), flops / (PEAK_BF16_MFMA_TFLOPS * 1e12)
        bound = "hbm" if t_hbm >= t_pipe else "mfma"
        out[name] = {"calls": calls, "ms": ms, "bound": bound, "algorithmic_bytes": nbytes, "algorithmic_flops": flops,
                     "achieved_GBps": nbytes / ms / 1e6, "achieved_TFLOPs": flops / ms / 1e9,
                     "frac": max(t_hbm, t_pipe) / (ms * 1e-3)}

    big, small = net.trans_down, net.trans
    nl = len(net.blocks)
    for tag, fwd, inv, n_r, n_i in (("721x1440", net.trans_down, net.itrans_up, 1, 2), ("240x480", net.trans, net.itrans, nl - 1, nl)):
        nlat, nlon, lmax, mmax = fwd.nlat, fwd.nlon, fwd.lmax, fwd.mmax
        pf, pi = fwd.plan(dev).handle, inv.plan(dev).handle
        x = torch.randn(C, nlat, nlon, device=dev).to(torch.bfloat16)
        xm = torch.empty(lib.sfno_fourier_elems(pf, C), dtype=torch.float32, device=dev)
        spec = torch.empty(lib.sfno_spectral_elems(pf, C), dtype=torch.float32, device=dev)
        fft_bytes = C * nlat * nlon * 2 + C * nlat * mmax * 8
        T = triangular_count(lmax, mmax)
        Tp = sum(min(l + 1, mmax) for l in range(lmax))
        leg_bytes = C * nlat * mmax * 8 + T * nlat * 4 + C * Tp * 8
        leg_flops = 4.0 * C * nlat * T / 2 * 3          # executed: equator fold, three fp16 products per fp32 product
        t = event_time_ms(lambda: check(lib.sfno_rfft(pf, P(x), _lib.DTYPE_BF16, P(xm), C, sp), "rfft"), iters, stream)
        hbm(f"rfft {tag} bf16 in", n_r, t, fft_bytes)
        t = event_time_ms(lambda: check(lib.sfno_legendre_analysis(pf, P(xm), P(spec), C, sp), "analysis"), iters, stream)
        mfma(f"legendre analysis {tag}", n_r, t, leg_flops, leg_bytes)
        t = event_time_ms(lambda: check(lib.sfno_legendre_synthesis(pi, P(spec), P(xm), C, sp), "synthesis"), iters, stream)
        mfma(f"legendre synthesis {tag}", n_i, t, leg_flops, leg_bytes)
        t = event_time_ms(lambda: check(lib.sfno_irfft(pi, P(xm), P(x), _lib.DTYPE_BF16, C, sp), "irfft"), iters, stream)
        hbm(f"irfft {tag} bf16 out", n_i, t, fft_bytes)
        if tag == "240x480":
            from makani_amd.contractions import dhconv_spectral
            w = net.blocks[1].filter.filter.weight
            t = event_time_ms(lambda: dhconv_spectral(spec, w, 1, mmax), iters, stream)
            mfma("dhconv 384x384x240", nl, t, 8.0 * C * C * Tp * 3, C * C * lmax * 8 + 2 * C * Tp * 8)      # executed: three fp16 products per real product
        del x, xm, spec
    # 1x1 convolutions of the pointwise tail: (name, module weight, bias, act, addend?, resolution, calls)
    hw_big, hw_small = net.inp_shape, (net.h, net.w)
    blk, last = net.blocks[1], net.blocks[-1]
    # the last block's skip convolution and the decoder's first convolution run as one convolution over two tensors where the
    # network merges them
    merged = 1 if net._decoder_merge_ok() else 0
    # likewise the decoder's last convolution and the convolution of the big skip
    tail = 1 if net._tail_cat_ok() else 0
    convs = [("conv 73->384 +GELU 721x1440", net.encoder.fwd[0], "gelu", False, hw_big, 1),
             # the encoder's last convolution runs only where the network does not fold it into the first block's spectral weight
             ("conv 384->384 721x1440", net.encoder.fwd[2], None, False, hw_big, 0 if net._encoder_fold() is not None else 1),
             ("conv 384->768 +GELU 240x480", blk.mlp.fwd[0], "gelu", False, hw_small, nl - 1),
             ("conv 768->384 240x480", blk.mlp.fwd[3], None, False, hw_small, nl - 1),
             ("conv 384->384 +addend 240x480", blk.outer_skip, None, True, hw_small, nl - 1),
             ("conv 384->768 +GELU 721x1440", last.mlp.fwd[0], "gelu", False, hw_big, 1),
             ("conv 768->384 721x1440", last.mlp.fwd[3], None, False, hw_big, 1),
             ("conv 384->384 +addend 721x1440", last.outer_skip, None, True, hw_big, 1 - merged),
             ("conv 384->384 +GELU 721x1440", net.decoder.fwd[0], "gelu", False, hw_big, 1 - merged),
             ("conv 384->73 +addend 721x1440", net.decoder.fwd[2], None, True, hw_big, 1 - tail),
             ("conv 73->73 721x1440", net.residual_transform, None, False, hw_big, 1 - tail)]
    for name, mod, act, add, (h, w_), calls in convs:
        O, K = mod.weight.shape[0], mod.weight.shape[1]
        xin = torch.randn(1, K, h, w_, device=dev).to(torch.bfloat16)
        addend = torch.randn(1, O, h, w_, device=dev).to(torch.bfloat16) if add else None
        sc = torch.ones(1, O, device=dev) if add else None
        sh = torch.zeros(1, O, device=dev) if add else None
        t = event_time_ms(lambda: pw.conv1x1(xin, mod.weight, mod.bias, act, addend, sc, sh), iters, stream)
        npx = h * w_
        mfma(name, calls, t, 2.0 * K * O * npx, 2 * npx * (K + O + (O if add else 0)))
        del xin, addend
    if True:
        h, w_ = hw_big
        O, K = net.decoder.fwd[0].weight.shape[0], net.decoder.fwd[0].weight.shape[1]
        x1 = torch.randn(1, K, h, w_, device=dev).to(torch.bfloat16)
        x2 = torch.randn(1, K, h, w_, device=dev).to(torch.bfloat16)
        wcat = torch.randn(O, 2 * K, device=dev) / (2 * K) ** 0.5
        bias = torch.zeros(O, device=dev)
        t = event_time_ms(lambda: pw.conv1x1_cat(x1, x2, wcat, bias, "gelu"), iters, stream)
        mfma("conv (384+384)->384 +GELU 721x1440, two inputs", merged, t, 2.0 * 2 * K * O * h * w_, 2 * h * w_ * (2 * K + O))
        del x1, x2
        O, K, K2 = net.decoder.fwd[2].weight.shape[0], net.decoder.fwd[2].weight.shape[1], net.residual_transform.weight.shape[1]
        x1 = torch.randn(1, K, h, w_, device=dev).to(torch.bfloat16)
        x2 = torch.randn(1, K2, h, w_, device=dev).to(torch.bfloat16)
        wcat = torch.randn(O, K + K2, device=dev) / (K + K2) ** 0.5
        t = event_time_ms(lambda: pw.conv1x1_cat(x1, x2, wcat, None, None), iters, stream)
        mfma("conv (384+73)->73 721x1440, two inputs", tail, t, 2.0 * (K + K2) * O * h * w_, 2 * h * w_ * (K + K2 + O))
        del x1, x2
    # instance-norm statistics and the scale/shift/GELU pass
    for tag, (h, w_), calls in (("240x480", hw_small, nl - 1), ("721x1440", hw_big, 1)):
        xin = torch.randn(1, C, h, w_, device=dev).to(torch.bfloat16)
        t = event_time_ms(lambda: pw.instance_norm_coeffs(xin), iters, stream)
        hbm(f"instance-norm statistics {tag}", calls, t, 2 * C * h * w_)
        sc, sh = pw.instance_norm_coeffs(xin)
        t = event_time_ms(lambda: pw.scale_shift_act(xin, sc, sh, "gelu"), iters, stream)
        hbm(f"scale+shift+GELU {tag}", calls, t, 4 * C * h * w_)
        del xin
    return out


def bench_sfno8l(args):
    import torch

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    med, best, net, xin = time_sfno_forward(1, max(args.steps, 5), args.warmup, dev, args.compute)
    del xin
    torch.cuda.empty_cache()
    with torch.inference_mode():
        classes = sfno_kernel_classes(dev, net) if args.compute == "fp32" else None
    return {
        "metric": "SFNO-L8 fwd ms/sample", "value": med, "unit": "ms/sample", "n_gpus": 1, "steps": max(args.steps, 5), "warmup": args.warmup,
        "ms_per_step": med, "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16 pointwise / f32 spectral" if args.compute != "bf16" else "bf16 pointwise / bf16-MFMA spectral contractions",
        "data": "synthetic",
        "config": {"workload": "configs[3]: SFNO-linear 8 layers, embed 384, scale factor 3 (721x1440 -> 240x480), 73 channels, batch 1, "
                               "bf16 autocast forward, random-init weights, N(0,1) inputs"},
        "best_ms": best,
        "kernel_classes_ms_sum": sum(c["calls"] * c["ms"] for c in classes.values()) if classes else None,
        "kernel_classes": classes,
    }


def bench_rollout(args):
    """configs[4]: batch 4, 12 autoregressive steps x_{t+1} = model(x_t) (makani/utils/inferencer.py:144-177, n_history = 0)."""
    import torch

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    net = build_sfno8l(dev, args.compute)
    x0 = torch.randn(4, 73, 721, 1440, generator=torch.Generator().manual_seed(5)).to(dev)
    nsteps = args.rollout_steps
    with torch.inference_mode(), torch.autocast("cuda", dtype=torch.bfloat16):
        x = x0
        for _ in range(args.rollout_warmup):
            x = net(x).float()
        torch.cuda.synchronize()
        x = x0
        t0 = time.perf_counter()
        for _ in range(nsteps):
            x = net(x).float()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
    finite = bool(torch.isfinite(x).all())
    # HBM bytes per rollout step, all kernels, from the FETCH_SIZE / WRITE_SIZE counter runs summarised under profiles/
    traffic = read_traffic("rollout_step_batch4") if args.compute == "fp32" else None
    return {
        "metric": "SFNO-L8 rollout ms/step", "value": dt / nsteps * 1e3, "unit": "ms/step", "n_gpus": 1, "steps": nsteps, "warmup": args.rollout_warmup,
        "ms_per_step": dt / nsteps * 1e3, "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16 pointwise / f32 spectral", "data": "synthetic",
        "config": {"workload": "configs[4]: SFNO-8L, batch 4, 12-step autoregressive rollout, bf16 autocast"},
        "ms_per_sample_step": dt / nsteps / 4 * 1e3, "finite": finite,
        "hbm_traffic_bytes_per_step": traffic, "hbm_traffic_bytes_total": traffic * nsteps if traffic else None,
        # the whole step as one HBM stream: measured bytes of all its kernels (rocprofv3 FETCH_SIZE + WRITE_SIZE, profiles/) over its time
        "roofline": ({"kernel": "all kernels of one rollout step (batch 4)", "bound": "hbm", "achieved": traffic / (dt / nsteps) / 1e9, "peak": PEAK_HBM_GBS,
                      "unit": "GB/s", "frac": traffic / (dt / nsteps) / 1e9 / PEAK_HBM_GBS, "traffic": traffic,
                      "note": "measured traffic, not algorithmic bytes: the per-kernel algorithmic figures are in sfno_l8_fwd_ms_per_sample.kernel_classes"}
                     if traffic else None),
        "cpu_baseline": {"value": None, "unit": "ms/step", "cores": os.cpu_count(), "kind": "port",
                         "sample": "skipped: budget (one sample of the 8-layer network is 4.5 TFLOP of fp32 convolutions on the host; the transform "
                                   "pair and the spectral block carry the CPU comparison)"},
    }


def bench_pointwise_backward(args):
    """Backward of the 1x1 convolutions of the SFNO-8L tail at their in-model shapes (bf16): weight + bias gradient and input
    gradient on the HIP kernels, with the kernels PyTorch picks for the same F.conv2d gradients beside them."""
    import torch
    import torch.nn.functional as F
    from makani_amd import pointwise as pw

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    stream = torch.cuda.current_stream(dev)
    iters = max(args.steps, 5)
    shapes = [("fc1 384->768 240x480", 384, 768, 240, 480), ("fc2 768->384 240x480", 768, 384, 240, 480), ("skip 384->384 240x480", 384, 384, 240, 480),
              ("fc1 384->768 721x1440", 384, 768, 721, 1440), ("encoder 73->384 721x1440", 73, 384, 721, 1440), ("decoder 384->73 721x1440", 384, 73, 721, 1440)]
    out, total = {}, 0.0
    for name, K, O, H, W in shapes:
        x = torch.randn(1, K, H, W, device=dev).bfloat16()
        gy = torch.randn(1, O, H, W, device=dev).bfloat16()
        w = torch.randn(O, K, 1, 1, device=dev) / K ** 0.5
        wt = w.reshape(O, K).t().contiguous()
        wb = w.bfloat16().requires_grad_(True)
        xr = x.clone().requires_grad_(True)
        y = F.conv2d(xr, wb)
        for f in (lambda: pw.conv1x1_weight_grad(gy, x, True), lambda: pw.conv1x1(gy, wt)):
            for _ in range(3):
                f()
        t_w = event_time_ms(lambda: pw.conv1x1_weight_grad(gy, x, True), iters, stream)
        t_x = event_time_ms(lambda: pw.conv1x1(gy, wt), iters, stream)
        for _ in range(3):
            torch.autograd.grad(y, (wb, xr), gy, retain_graph=True)
        t_lw = event_time_ms(lambda: torch.autograd.grad(y, wb, gy, retain_graph=True), iters, stream)
        t_lx = event_time_ms(lambda: torch.autograd.grad(y, xr, gy, retain_graph=True), iters, stream)
        nbytes = 2.0 * H * W * (K + O)
        out[name] = {"weight_grad_ms": t_w, "input_grad_ms": t_x, "weight_grad_frac_hbm": nbytes / (t_w * 1e-3) / 1e9 / PEAK_HBM_GBS,
                     "input_grad_frac_hbm": nbytes / (t_x * 1e-3) / 1e9 / PEAK_HBM_GBS, "library_weight_grad_ms": t_lw, "library_input_grad_ms": t_lx}
        total += t_w + t_x
        del x, gy, y, xr
    return {"metric": "1x1 convolution backward, sum over the listed shapes", "value": total, "unit": "ms", "n_gpus": 1, "steps": iters, "warmup": 3,
            "ms_per_step": total, "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
            "config": {"workload": "weight/bias and input gradients of the SFNO-8L tail's 1x1 convolutions, batch 1, bf16, N(0,1) operands"},
            "shapes": out}


def bench_train_step(args):
    """One training step of the SFNO-8L network (configs[3] shapes, batch 1) under bf16 autocast: forward, mean-square loss,
    backward, SGD update (so that every packed weight copy is rebuilt each step, as in training).  The transforms, dhconv and
    the 1x1 convolutions run on the HIP kernels in both directions; GELU and the instance norms are PyTorch's.  The same
    step with the convolutions left to PyTorch's library kernels is timed beside it."""
    import torch
    from makani_amd import pointwise as pw

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    net = build_sfno8l(dev, args.compute).train()
    opt = torch.optim.SGD(net.parameters(), lr=1e-6)
    x = torch.randn(1, 73, 721, 1440, generator=torch.Generator().manual_seed(5)).to(dev)
    tgt = torch.randn(1, 73, 721, 1440, generator=torch.Generator().manual_seed(6)).to(dev)

    def step():
        opt.zero_grad(set_to_none=True)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            y = net(x)
        loss = ((y.float() - tgt) ** 2).mean()
        loss.backward()
        opt.step()
        return loss

    def timed():
        for _ in range(max(args.warmup, 2)):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            loss = step()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / args.steps * 1e3, float(loss.detach())

    ms, loss = timed()
    peak = torch.cuda.max_memory_allocated() / 1e9
    ms_lib = None
    if not args.no_library_leg:
        saved = pw.trainable_active
        pw.trainable_active = lambda t: False
        try:
            ms_lib, _ = timed()
        finally:
            pw.trainable_active = saved
    return {"metric": "SFNO-L8 training step ms/sample", "value": ms, "unit": "ms", "n_gpus": 1, "steps": args.steps, "warmup": max(args.warmup, 2),
            "ms_per_step": ms, "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "bf16 pointwise / f32 spectral", "data": "synthetic",
            "config": {"workload": "SFNO-linear 8 layers, embed 384, 721x1440 -> 240x480, 73 channels, batch 1: forward + backward + SGD update, bf16 autocast"},
            "ms_per_step_with_library_convolutions": ms_lib, "loss_finite": loss == loss and abs(loss) != float("inf"), "peak_memory_GB": peak}


def legendre_fp32_mfma_figure(iters=10):
    """The Legendre stage of configs[1] on the fp32 matrix instruction (compute="fp32_mfma"): time per direction and algorithmic
    (triangular) flops over it against the fp32 MFMA peak."""
    import torch
    import makani_amd as ma
    from makani_amd._lib import lib, check

    dev = torch.device("cuda:0")
    nlat, nlon, lmax, mmax, C = 721, 1440, 721, 721, 73
    sht = ma.RealSHT(nlat, nlon, lmax=lmax, mmax=mmax, grid="equiangular", compute="fp32_mfma")
    isht = ma.InverseRealSHT(nlat, nlon, lmax=lmax, mmax=mmax, grid="equiangular", compute="fp32_mfma")
    x = make_fields(isht, C, dev)
    stream = torch.cuda.current_stream(dev)
    sp = ctypes.c_void_p(stream.cuda_stream)
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    pf, pi = sht.plan(dev).handle, isht.plan(dev).handle
    xm = torch.empty(lib.sfno_fourier_elems(pf, C), dtype=torch.float32, device=dev)
    spec = torch.empty(lib.sfno_spectral_elems(pf, C), dtype=torch.float32, device=dev)
    check(lib.sfno_rfft(pf, P(x), 0, P(xm), C, sp), "rfft")
    ana = event_time_ms(lambda: check(lib.sfno_legendre_analysis(pf, P(xm), P(spec), C, sp), "analysis"), iters, stream)
    syn = event_time_ms(lambda: check(lib.sfno_legendre_synthesis(pi, P(spec), P(xm), C, sp), "synthesis"), iters, stream)
    flops = 4.0 * C * nlat * triangular_count(lmax, mmax)
    fig = lambda ms: {"ms": ms, "TFLOPs": flops / ms / 1e9, "frac": flops / ms / 1e9 / PEAK_FP32_MFMA_TFLOPS}
    return {"analysis": fig(ana), "synthesis": fig(syn), "peak_TFLOPs": PEAK_FP32_MFMA_TFLOPS, "algorithmic_flops_per_launch": flops,
            "note": "v_mfma_f32_32x32x2_f32 on fp32 tables; algorithmic (triangular) flops, of which the kernel executes half (equator fold)"}


def main():
    args = parse()
    if args.gpus != 1:
        print(f"bench.py measures one GPU: --gpus {args.gpus} is not supported (the spectral path has no multi-GPU part)", file=sys.stderr)
        sys.exit(2)
    import torch

    if not torch.cuda.is_available():
        print("bench.py needs a HIP device", file=sys.stderr)
        sys.exit(1)
    if args.compute == "fp32_mfma" and (args.workload != "sht_pair" or not args.no_sfno):
        print("--compute fp32_mfma exists for the transform pair only: use it with --workload sht_pair --no-sfno", file=sys.stderr)
        sys.exit(2)
    if args.workload == "sht_pair":
        res = bench_sht_pair(args)
        if not args.no_sfno:
            # the second headline figure of the metric, measured in the same run
            torch.cuda.empty_cache()
            med, best, net, xin = time_sfno_forward(1, 10, 3, torch.device("cuda:0"))
            del xin
            torch.cuda.empty_cache()
            with torch.inference_mode():
                classes = sfno_kernel_classes(torch.device("cuda:0"), net)
            res["sfno_l8_fwd_ms_per_sample"] = {"value": med, "best": best, "batch": 1, "dtype": "bf16 pointwise / f32 spectral",
                                                "config": "configs[3]: SFNO-linear 8 layers, embed 384, 721x1440, 73 channels, bf16 autocast",
                                                "kernel_classes_ms_sum": sum(c["calls"] * c["ms"] for c in classes.values()),
                                                "kernel_classes": classes}
            del net, classes
        if not args.no_extras and args.compute == "fp32":
            import copy
            import gc

            def sub(workload, compute, steps, warmup):
                a = copy.copy(args)
                a.workload, a.compute, a.steps, a.warmup, a.backward = workload, compute, steps, warmup, False
                gc.collect()
                torch.cuda.empty_cache()
                return a

            keep = ("value", "unit", "ms_per_step", "dtype", "compute", "config", "stages_ms", "roofline", "cpu_baseline", "achieved_TFLOPs",
                    "ms_per_sample_step", "finite", "hbm_traffic_bytes_per_step", "hbm_traffic_bytes_total", "steps", "warmup")
            pick = lambda r: {k: r[k] for k in keep if k in r}
            # configs[2] in both variants, configs[4], and the Legendre stage on the fp32 matrix instruction
            res["spectral_block"] = {"fp32": pick(bench_spectral_block(sub("spectral_block", "fp32", 20, 5)))}
            a = sub("spectral_block", "bf16", 20, 5)
            a.no_cpu_baseline = True          # same host computation as the fp32 variant
            res["spectral_block"]["bf16"] = pick(bench_spectral_block(a))
            res["rollout"] = pick(bench_rollout(sub("rollout", "fp32", 12, 2)))
            gc.collect()
            torch.cuda.empty_cache()
            res["legendre_fp32_mfma"] = legendre_fp32_mfma_figure()
    elif args.workload == "fft2_pair":
        res = bench_fft2_pair(args)
    elif args.workload == "spectral_block":
        res = bench_spectral_block(args)
    elif args.workload == "sfno8l":
        res = bench_sfno8l(args)
    elif args.workload == "pointwise_backward":
        res = bench_pointwise_backward(args)
    elif args.workload == "train_step":
        res = bench_train_step(args)
    else:
        res = bench_rollout(args)
    print(json.dumps(res), flush=True)


if __name__ == "__main__":
    main()
