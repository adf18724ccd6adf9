#!/usr/bin/env python3
"""Benchmark of the quaternion Conv2D hot path on one MI355X.

A step is one pass of the hot path over one batch of synthetic input: forward, input-gradient and
filter-gradient of one quaternion convolution, inputs resident in HBM.  The default workload is the
pointwise fp32 configuration (N=32, 64->64 quaternion channels, 56x56); --workload selects the
others.  Prints ONE JSON line: real-equivalent TFLOP/s (16 real multiply-adds per quaternion
multiply-add, for either product mode), the roofline of the dominant kernel and the reference's CPU
algorithm timed on the host cores of the same box.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "quaternion conv TFLOP/s (real-equiv, % MFMA peak) + q-ResNet-50 fwd+bwd img/s"
PEAK_TFLOPS = {"f32": 157.3, "f16": 2500.0}  # MI355X dense MFMA peaks

WORKLOADS = {
    # name: (n, ci, co, h, w, k, padding, dtype, policy)
    "c2_pw_f32": (32, 64, 64, 56, 56, 1, "VALID", "f32", "fp32"),
    "c3_k3_f32": (64, 64, 64, 56, 56, 3, "SAME", "f32", "fp32"),
    "c4_k3_f16_128_28": (128, 128, 128, 28, 28, 3, "SAME", "f16", "full16"),
    "c4_k3_f16_256_14": (128, 256, 256, 14, 14, 3, "SAME", "f16", "full16"),
    "c4_pw_f16_128_28": (128, 128, 128, 28, 28, 1, "VALID", "f16", "full16"),
    "c4_pw_f16_256_14": (128, 256, 256, 14, 14, 1, "VALID", "f16", "full16"),
}
RESNET = "c5_qresnet50"  # quaternion ResNet-50 forward+backward, N=64, 224x224, fp16 full16 policy

# HBM bytes per launch of the main kernel of each pass, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of
# this script (summaries under profiles/): (FETCH_SIZE * 2 KiB + WRITE_SIZE * 1 KiB), the unit sizes being
# what the same counters read for a plain 256 MiB device copy.  Configurations not profiled report null.
KIB = 1024.0
MEASURED_TRAFFIC = {
    ("c2_pw_f32", 8): {"fwd": (66673.9 * 2 + 131712.0) * KIB, "bwd_data": (66610.1 * 2 + 131712.0) * KIB,
                       "bwd_weights": (100555.4 * 2 + 32768.0) * KIB},
    ("c3_k3_f32", 8): {"fwd": (150715.1 * 2 + 244946.0) * KIB, "bwd_data": (161077.9 * 2 + 246386.3) * KIB,
                       "bwd_weights": (379051.4 * 2 + 32256.0) * KIB},
    ("c4_k3_f16_128_28", 16): {"fwd": (86388.7 * 2 + 111692.5) * KIB, "bwd_data": (86388.7 * 2 + 111692.5) * KIB,
                               "bwd_weights": (180024.9 * 2 + 48384.0) * KIB},
    ("c4_k3_f16_128_28", 8): {"fwd": (122328.1 * 2 + 112062.2) * KIB, "bwd_data": (121113.6 * 2 + 112644.7) * KIB,
                              "bwd_weights": (180008.1 * 2 + 48384.0) * KIB},
}


def executed_share(kernel_name):
    """Executed / real-equivalent arithmetic of a kernel: the factorized (8-product) kernels run half the
    multiplications.  The product mode asks for a formulation; on fp16 matrix cores the library runs the
    pointwise passes and the filter gradient of the 8-product mode on 16-product kernels (faster there), so
    the share is read off the kernel that actually ran."""
    return 0.5 if "_p8_" in kernel_name else 1.0


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="c2_pw_f32", choices=sorted(WORKLOADS) + [RESNET])
    ap.add_argument("--mode", type=int, default=0, choices=[0, 8, 16],
                    help="product formulation; 0 = from UPSTRIDE_MEMORY_OPTIMIZED like the reference (default 8)")
    ap.add_argument("--policy", default=None, help="override UPSTRIDE_CONV_FP16_POLICY for fp16 workloads")
    ap.add_argument("--batch", type=int, default=64, help="images per step of the ResNet workload")
    ap.add_argument("--torch-bn", action="store_true",
                    help="ResNet workload: torch.nn.BatchNorm2d + ReLU (MIOpen) instead of the library's batch-norm kernels")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also launch a plain 256 MiB device copy (untimed), the yardstick for HBM byte counters")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="CPU time budget of the cpu_baseline leg")
    return ap.parse_args()


def cpu_baseline(cfg, mode, seconds):
    """The reference's CPU algorithm (lane decomposition + scalar oneDNN convolutions through
    torch's CPU backend) on a bounded sample of the same workload."""
    import torch
    import oracle
    from oracle import torch_cpu_path as tcp
    n, ci, co, h, w, k, padding, _, _ = cfg
    threads = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(threads)
    n_s = max(1, n // 8)
    g = oracle.make_geom(n_s, ci, co, h, w, k, k, 1, 1, padding)
    gen = torch.Generator().manual_seed(0x5EED)
    x = torch.randn(4 * n_s, ci, h, w, generator=gen)
    wt = torch.randn(4, co, ci, k, k, generator=gen) * (2.0 / (ci * k * k)) ** 0.5
    gr = torch.randn(4 * n_s, co, g.ho, g.wo, generator=gen)
    name = "factorized" if mode == 8 else "generic"
    flops = 3 * 2 * 16 * n_s * co * ci * g.ho * g.wo * k * k

    def step():
        tcp.conv2d_fwd(g, x, wt, None, name)
        tcp.conv2d_bwd(g, x, wt, gr, name)

    step()  # warm-up (primitive creation)
    times = []
    t_end = time.perf_counter() + seconds
    while len(times) < 3 or (time.perf_counter() < t_end and len(times) < 50):
        t0 = time.perf_counter()
        step()
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    return {
        "value": flops / med / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
        "sample": "%d of %d images of the same workload, fwd+dgrad+wgrad, %s path, scalar convs by torch %s CPU "
                  "(oneDNN), fp32, median of %d runs" % (n_s, n, name, torch.__version__, len(times)),
        "ms_per_step_sample": med * 1e3,
    }


def resnet_flops(n):
    """Real-equivalent forward FLOPs of the 53 convolutions + head (2*16*N*Co*Ci*Ho*Wo*Kh*Kw each)."""
    total, size = 0.0, 224
    def conv(ci, co, k, s, hin):
        ho = (hin + s - 1) // s
        return 2.0 * 16 * n * co * ci * ho * ho * k * k, ho
    f, size = conv(3, 16, 7, 2, size)
    total += f
    size = (size + 1) // 2  # max-pool
    cin = 16
    for width, cout, count, stride in ((16, 64, 3, 1), (32, 128, 4, 2), (64, 256, 6, 2), (128, 512, 3, 2)):
        for i in range(count):
            s = stride if i == 0 else 1
            total += conv(cin, width, 1, 1, size)[0]
            f, out = conv(width, width, 3, s, size)
            total += f + conv(width, cout, 1, 1, out)[0]
            if s != 1 or cin != cout:
                total += conv(cin, cout, 1, s, size)[0]
            size, cin = out, cout
    return total + 2.0 * 16 * n * 250 * 512


def bench_resnet(args):
    import torch
    import phoenix_core_amd as phx
    from phoenix_core_amd import capi
    policy = args.policy or "full16"
    env = {"UPSTRIDE_CONV_FP16_POLICY": policy}
    if args.mode == 16 or (args.mode == 0 and phx.Context().memory_optimized):
        env["UPSTRIDE_MEMORY_OPTIMIZED"] = "1"
    ctx = phx.Context(env)
    mode = 16 if ctx.memory_optimized else 8
    n = args.batch
    dev = torch.device("cuda:0")
    torch.manual_seed(0x5EED + 5)
    model = phx.QResNet50(1000, dtype=torch.float16, context=ctx, fused_bn=not args.torch_bn).to(dev).train()
    images = torch.randn(n, 3, 224, 224, device=dev).half()
    labels = torch.randint(0, 1000, (n,), device=dev)

    def step():
        model.zero_grad(set_to_none=True)
        loss = torch.nn.functional.cross_entropy(model(images).float(), labels)
        loss.backward()
        return loss

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    ncalls = 3 * 54
    capi.profile_enable(ncalls * args.steps)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        loss = step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    kernel_ms = capi.profile_collect(ncalls * args.steps)
    capi.profile_enable(0)
    ms_per_step = elapsed / args.steps * 1e3
    fwd_flops = resnet_flops(n)
    conv_ms = sum(kernel_ms) / args.steps
    out = {
        "metric": METRIC, "value": n / (ms_per_step * 1e-3), "unit": "img/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": "%s: quaternion ResNet-50 forward+backward (no optimizer step, as the metric names), "
                               "N=%d real images (4N=%d quaternion rows after the real-input stem), 224x224, 53 quaternion convs + "
                               "quaternion dense head; batch-norm (with the ReLU behind it) by %s, residual add, "
                               "pooling and cross-entropy by PyTorch"
                               % (RESNET, n, 4 * n, "torch.nn.BatchNorm2d (MIOpen)" if args.torch_bn else
                                  "the library's streaming kernels (include/phx_bn.h)"),
                   "product_mode": mode, "fp16_policy": policy, "batch_norm": "torch" if args.torch_bn else "library"},
        "real_equiv_tflops": 3 * fwd_flops / (ms_per_step * 1e-3) / 1e12,
        "quaternion_kernel_ms_per_step": conv_ms, "loss": float(loss.detach()),
    }
    print(json.dumps(out))
    return 0


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (--gpus %d refused)" % args.gpus,
              file=sys.stderr)
        return 2
    if args.workload == RESNET:
        return bench_resnet(args)

    import torch
    import phoenix_core_amd as phx
    from phoenix_core_amd import capi

    cfg = WORKLOADS[args.workload]
    n, ci, co, h, w, k, padding, dt, policy = cfg
    if args.policy:
        policy = args.policy
    env = {"UPSTRIDE_CONV_FP16_POLICY": policy}
    if args.mode == 16 or (args.mode == 0 and phx.Context().memory_optimized):
        env["UPSTRIDE_MEMORY_OPTIMIZED"] = "1"
    ctx = phx.Context(env)
    mode = 16 if ctx.memory_optimized else 8
    dtype = torch.float32 if dt == "f32" else torch.float16

    dev = torch.device("cuda:0")
    torch.manual_seed(0x5EED + sorted(WORKLOADS).index(args.workload))
    scale = 1.0 if dt == "f32" else 0.5
    x = (scale * torch.randn(4 * n, ci, h, w, device=dev)).to(dtype)
    wt = (scale * torch.randn(4, co, ci, k, k, device=dev) * (2.0 / (ci * k * k)) ** 0.5).to(dtype)
    desc = phx.Conv2DDescriptor(x.shape, wt.shape, 1, 1, padding, dtype=dtype, context=ctx)
    gr = (scale * torch.randn(desc.output_shape, device=dev)).to(dtype)
    ho, wo = desc.output_shape[2:]
    y = torch.empty(desc.output_shape, dtype=dtype, device=dev)
    dx = torch.empty_like(x)
    dw = torch.empty_like(wt)
    L = capi.lib()
    sizes = [desc.workspace_bytes(p) for p in (capi.PHX_PASS_FWD, capi.PHX_PASS_BWD_DATA, capi.PHX_PASS_BWD_WEIGHTS)]
    ws = torch.empty(max(sizes), dtype=torch.uint8, device=dev)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    d = ctypes.byref(desc.c)
    names = {}

    def step():
        capi.check(L.phx_qconv2d_fwd(d, stream, P(x), P(wt), None, P(y), P(ws), sizes[0]), "fwd")
        names.setdefault("fwd", capi.last_kernel_name())
        capi.check(L.phx_qconv2d_bwd_data(d, stream, P(gr), P(wt), P(dx), P(ws), sizes[1]), "bwd_data")
        names.setdefault("bwd_data", capi.last_kernel_name())
        capi.check(L.phx_qconv2d_bwd_weights(d, stream, P(x), P(gr), P(dw), P(ws), sizes[2]), "bwd_weights")
        names.setdefault("bwd_weights", capi.last_kernel_name())

    if args.copy_calibration:
        src = torch.empty(64 << 20, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)  # reads 256 MiB, writes 256 MiB
        del src, dst
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    capi.profile_enable(3 * args.steps)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    kernel_ms = capi.profile_collect(3 * args.steps)
    capi.profile_enable(0)

    flops_pass = 2.0 * 16 * n * co * ci * ho * wo * k * k
    ms_per_step = elapsed / args.steps * 1e3
    value = 3 * flops_pass / (ms_per_step * 1e-3) / 1e12
    per_pass = {}
    for i, key in enumerate(("fwd", "bwd_data", "bwd_weights")):
        vals = kernel_ms[i::3]
        per_pass[key] = sum(vals) / max(1, len(vals))
    dominant = max(per_pass, key=per_pass.get)
    compute = "f32" if (dt == "f32" or policy == "fp32" or (policy == "backward32" and dominant != "fwd")) else "f16"
    achieved = flops_pass / (per_pass[dominant] * 1e-3) / 1e12
    esize = 4 if dt == "f32" else 2
    # algorithmic bytes of a pass: read the activations (or the gradient), read the filters, write the result
    bytes_pass = {
        "fwd": esize * (x.numel() + wt.numel() + y.numel()),
        "bwd_data": esize * (gr.numel() + wt.numel() + dx.numel()),
        "bwd_weights": esize * (x.numel() + gr.numel() + dw.numel()),
    }
    traffic = MEASURED_TRAFFIC.get((args.workload, mode), {}).get(dominant)
    out = {
        "metric": METRIC, "value": value, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dt, "data": "synthetic",
        "config": {"workload": "%s: quaternion conv %dx%d stride 1, N=%d (4N=%d rows), %d->%d q-channels, %dx%d, "
                               "fwd+input-grad+filter-grad" % (args.workload, k, k, n, 4 * n, ci, co, h, w),
                   "product_mode": mode, "fp16_policy": policy, "padding": padding},
        "images_per_s": n / (ms_per_step * 1e-3),
        "frac_of_mfma_peak": value / PEAK_TFLOPS[compute],
        "executed_tflops": value * sum(executed_share(names[k]) for k in names) / len(names),
        "kernel_ms": per_pass, "kernels": names,
        "algorithmic_hbm_gb_s": {k: bytes_pass[k] / (per_pass[k] * 1e-3) / 1e9 for k in per_pass},
        "roofline": {"bound": "mfma", "kernel": names[dominant], "achieved": achieved, "peak": PEAK_TFLOPS[compute],
                     "unit": "TFLOP/s", "frac": achieved / PEAK_TFLOPS[compute], "traffic": traffic,
                     "algorithmic_bytes": bytes_pass[dominant],
                     "executed": achieved * executed_share(names[dominant])},
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(cfg, mode, args.cpu_seconds)
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
