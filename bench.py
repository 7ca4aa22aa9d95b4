#!/usr/bin/env python3
"""Benchmark of the MI355X backend for Z-Ant's tensor-math hot path.

Workload (N=1 GPU): the reference's README CNN (Conv32-ReLU-MaxPool-Conv64-ReLU-MaxPool-Flatten-Dense512-ReLU-
Dense10-Softmax, f32) at batch 4096 -- the configuration the headline metric "batched inferences/sec at batch
4096" is quoted on.  One step = one forward pass over one resident batch.  Prints ONE JSON line.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline] [--no-operators] [--no-networks]

`value` is inferences/s with inputs resident in HBM; `roofline` is measured live with HIP events around the
dominant kernel of the pass; `cpu_baseline` times the CPU oracle (a restatement of the reference's algorithm:
the reference is Zig-only and no Zig toolchain exists here) on the host, one image at a time on one core, which
is how the reference's generated predict() runs.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# HBM bytes per launch of the pass's kernels at batch 4096, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this
# file scaled by a 256 MiB copy (summary and commands: profiles/cnn_f32_b4096_hbm_traffic.md).  Counters cannot be read
# from inside the process, so `roofline.traffic` reports the figure of that run -- keyed by the device function the
# profile names, and reported only when the kernel this run launched for the dominant node is that same function
# (otherwise null: the figure would describe a kernel that no longer runs).
MEASURED_HBM_BYTES = {
    "conv_f32_mfma_kernel<4,2,2,4,9,true,true>": 119.79e6,
    "conv_f32_c1k3_pool_mfma_kernel<true,true>": 103.63e6,
    "gemm_f32_dma_kernel<1,4,2,0,0,5>": 60.91e6,  # the model's first Gemm (B packed at load)
    "gemm_f32_dma_kernel<1,4,2,0,3,5>": 60.93e6,  # the same shape through gemm_lean (B row-major)
    "gemm_f32_skinny_kernel<3>": 8.88e6,
}
PEAK_F32_MFMA_TFLOPS = 157.3
PEAK_I8_MFMA_TOPS = 5030.0
PEAK_HBM_GBS = 8000.0
BATCH = 4096


def kernel_avg_ms(ctx, fn, iters):
    """Average duration of the main kernel of `fn` (HIP events recorded by the library around that launch)."""
    ctx.kernel_timing(True)
    tot = 0.0
    for _ in range(iters):
        fn()
        tot += ctx.kernel_ms()
    ctx.kernel_timing(False)
    return tot / iters


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-operators", action="store_true", help="skip the standalone operator figures (configs 2a, 2b, 3)")
    ap.add_argument("--no-networks", action="store_true", help="skip the int8 network figures (configs 4, 5)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 256 MiB device copy (3x): the known-size reference for scaling the "
                         "FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run of this command")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build targets ONE MI355X; the forward pass shards by batch with no collectives "
                 "and no multi-GPU figure is produced. Run with --gpus 1.")

    import numpy as np
    import torch
    import __graft_entry__ as ge

    za = ge.load_package()  # raises if libzant_hip.so is not built: there is no fallback path
    tm = za.tensor_math
    from zant_amd import networks

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    ctx = tm.context()
    params = networks.readme_cnn_params(seed=0)
    model = networks.build_readme_cnn_model(ctx, BATCH, params)  # what is timed: one zant_model_run per step
    g = np.random.default_rng(1)
    x_host = g.random((BATCH, 1, 28, 28), dtype=np.float32)  # ~U[0,1)
    ctx.check(za.lib.zant_hip_upload(ctx.handle, model.input_ptr, x_host.ctypes.data, x_host.nbytes))  # resident input

    # ---- parity gate on the first images of the batch (the oracle is only the checker) ----
    model.run()
    out_host = np.zeros((BATCH, 10), np.float32)
    ctx.check(za.lib.zant_hip_download(ctx.handle, out_host.ctypes.data, model.output_ptr, out_host.nbytes))
    from oracle import oracle as zo

    def oracle_forward(img):
        y = zo.ReLU(zo.Conv(img, params["w1"], params["b1"], [1, 1], None, None, 1, None))
        y = zo.onnx_maxpool(y, [2, 2], [2, 2], [1, 1], [0, 0, 0, 0])
        y = zo.ReLU(zo.Conv(y, params["w2"], params["b2"], [1, 1], None, None, 1, None))
        y = zo.onnx_maxpool(y, [2, 2], [2, 2], [1, 1], [0, 0, 0, 0])
        y = zo.ReLU(zo.gemm(y.reshape(1, 1, 1, 1600), params["g1"], params["c1"], 1.0, 1.0, False, False))
        y = zo.gemm(y, params["g2"], params["c2"], 1.0, 1.0, False, False)
        return zo.softmax(y.reshape(1, 10))

    ref = np.concatenate([oracle_forward(x_host[i:i + 1]) for i in (0, 1, 2, BATCH - 1)])
    np.testing.assert_allclose(out_host[[0, 1, 2, BATCH - 1]], ref, rtol=1e-4, atol=1e-5)

    # ---- timed region: W warm-up steps, then exactly K steps between synchronisations ----
    # The shader clock needs some 15 ms of continuous work to settle (0.268 ms per pass measured after 5 passes of a cold
    # start, 0.257 after 50, 0.256 after 200): about 30 ms of untimed passes first, whatever W is, so that the W warm-up
    # steps and the K timed ones run at the clock a busy device runs at.
    for _ in range(120):
        model.run()
    ctx.sync()
    for _ in range(args.warmup):
        model.run()
    ctx.sync()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ctx.timer_start()
    for _ in range(args.steps):
        model.run()
    ev_ms = ctx.timer_stop()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    ms_per_step = max(ev_ms, wall_ms) / args.steps  # the host clock includes the final synchronisation
    value = BATCH / (ms_per_step * 1e-3)
    # the result of the LAST timed step must be the first step's, bit for bit (the input stays resident and intact)
    last_host = np.zeros_like(out_host)
    ctx.check(za.lib.zant_hip_download(ctx.handle, last_host.ctypes.data, model.output_ptr, last_host.nbytes))
    assert np.array_equal(last_host, out_host), "the last timed step differs from the gated first step"

    if args.copy_calibration:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # ---- per-kernel durations of the pass: HIP events around the main kernel of every launching node ----
    flops = networks.readme_cnn_flops_per_inference()
    kit = max(5, min(args.steps, 20))
    acc = None
    for _ in range(kit):
        prof = model.profile()
        acc = prof if acc is None else [(n, a[1] + p[1], o, b) for a, p, (n, _, o, b) in zip(acc, prof, prof)]
    per_kernel = {}
    for i, (name, ms_sum, ops, nbytes) in enumerate(acc):
        ms = ms_sum / kit
        key = f"{i}:{name}"
        # the roofline that bounds each node: arithmetic intensity against the f32 MFMA / HBM ridge (157.3 TF / 8 TB/s)
        mfma_bound = ops > 0 and ops / nbytes > PEAK_F32_MFMA_TFLOPS * 1e12 / (PEAK_HBM_GBS * 1e9)
        if mfma_bound:
            ach = ops / (ms * 1e-3) / 1e12
            per_kernel[key] = {"ms": round(ms, 4), "bound": "mfma", "achieved_tflops": round(ach, 2),
                               "frac": round(ach / PEAK_F32_MFMA_TFLOPS, 4), "flop": ops, "bytes": nbytes}
        else:
            ach = nbytes / (ms * 1e-3) / 1e9
            per_kernel[key] = {"ms": round(ms, 4), "bound": "hbm", "achieved_gbs": round(ach, 1),
                               "frac": round(ach / PEAK_HBM_GBS, 4), "flop": ops, "bytes": nbytes}
    launched = model.launch_kernels()
    for i, key in enumerate(per_kernel):
        per_kernel[key]["kernel"] = launched[i]
    dominant = max(per_kernel, key=lambda k: per_kernel[k]["ms"])
    dk = per_kernel[dominant]
    traffic = MEASURED_HBM_BYTES.get(dk["kernel"])
    if dk["bound"] == "mfma":
        roofline = {"kernel": dominant, "device_function": dk["kernel"], "bound": "mfma", "achieved": dk["achieved_tflops"],
                    "peak": PEAK_F32_MFMA_TFLOPS, "unit": "TFLOP/s", "frac": dk["frac"], "traffic": traffic, "avg_ms": dk["ms"]}
    else:
        roofline = {"kernel": dominant, "device_function": dk["kernel"], "bound": "hbm", "achieved": dk["achieved_gbs"],
                    "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": dk["frac"], "traffic": traffic, "avg_ms": dk["ms"]}

    # ---- the per-operator path: what a binding that calls one lean operator per node pays (no fusion of the pools, one
    # launch per node, weights packed on every call), against the fused zant_model_run the headline times ----
    lean = networks.ReadmeCNN(BATCH, params)
    xt = torch.from_numpy(x_host).to(dev)
    lean_out = lean.forward(xt)
    ctx.sync()
    np.testing.assert_allclose(lean_out[[0, 1, 2, BATCH - 1]].cpu().numpy(), ref, rtol=1e-4, atol=1e-5)
    for _ in range(3):
        lean.forward(xt)
    ctx.sync()
    ctx.timer_start()
    for _ in range(kit):
        lean.forward(xt)
    lean_ms = ctx.timer_stop() / kit
    lean_path = {"ms_per_step": round(lean_ms, 4), "inferences_per_s": round(BATCH / lean_ms * 1e3, 1), "calls_per_step": 8,
                 "what": "conv_lean(+relu) / onnx_maxpool_lean / conv_lean(+relu) / onnx_maxpool_lean / gemm_lean(+relu) / "
                         "gemm_lean / softmax_lean through the C ABI on preallocated tensors"}
    # the same eight calls with prepared-weights handles for the two convolutions (zant_hip_conv2d_f32_prepack): what a
    # binding that keeps its weights pays once they are packed
    lean.prepare()
    np.testing.assert_allclose(lean.forward(xt)[[0, 1, 2, BATCH - 1]].cpu().numpy(), ref, rtol=1e-4, atol=1e-5)
    for _ in range(3):
        lean.forward(xt)
    ctx.sync()
    ctx.timer_start()
    for _ in range(kit):
        lean.forward(xt)
    lean_path["ms_per_step_prepared_weights"] = round(ctx.timer_stop() / kit, 4)
    # ... and with the two Conv -> ReLU -> MaxPool chains as one prepared call each (fuse_pool), which is what a code
    # generator that peephole-fuses the chain emits: six calls, the pooled activations the only ones that exist
    lean.prepare(fuse_pool=True)
    np.testing.assert_allclose(lean.forward(xt)[[0, 1, 2, BATCH - 1]].cpu().numpy(), ref, rtol=1e-4, atol=1e-5)
    for _ in range(3):
        lean.forward(xt)
    ctx.sync()
    ctx.timer_start()
    for _ in range(kit):
        lean.forward(xt)
    lean_path["ms_per_step_prepared_fused_pools"] = round(ctx.timer_stop() / kit, 4)
    del lean, xt, lean_out

    # ---- standalone operator figures (the "conv TOPS" half of the metric): configs 2a, 2b, 3 ----
    operators = None
    if not args.no_operators:
        operators = {}
        torch.manual_seed(0)
        xa = torch.randn(256, 64, 56, 56, device=dev)
        wa = torch.randn(64, 64, 3, 3, device=dev) * (2.0 / 576) ** 0.5
        ba = torch.randn(64, device=dev) * 0.1
        ya = torch.zeros(256, 64, 56, 56, device=dev)
        fn = lambda: tm.conv_lean(xa, wa, ya, ba, [1, 1], [1, 1, 1, 1], [1, 1], 1, "NOTSET")
        fn(); ms = kernel_avg_ms(ctx, fn, kit)
        fl = 2 * 256 * 64 * 56 * 56 * 64 * 9
        operators["conv_f32_N256_C64_56x56_K64_3x3"] = {"ms": round(ms, 4), "tflops": round(fl / ms / 1e9, 2),
                                                        "frac_f32_mfma_peak": round(fl / ms / 1e9 / PEAK_F32_MFMA_TFLOPS, 4)}
        # parity gate on the timed tensors (first and last image), which is also the one-core oracle sample
        pick = [0, 255]
        xs, wsl, bs = xa[pick].cpu().numpy(), wa.cpu().numpy(), ba.cpu().numpy()
        t0 = time.perf_counter()
        ref_a = zo.Conv(xs, wsl, bs, [1, 1], [1, 1, 1, 1], [1, 1], 1, "NOTSET")
        dt = time.perf_counter() - t0
        np.testing.assert_allclose(ya[pick].cpu().numpy(), ref_a, rtol=1e-4, atol=1e-5)
        operators["conv_f32_N256_C64_56x56_K64_3x3"]["parity_gate"] = "images 0 and 255 of the timed output against the oracle, rtol 1e-4 atol 1e-5"
        if not args.no_cpu_baseline:
            operators["conv_f32_N256_C64_56x56_K64_3x3"]["cpu_oracle_1core"] = {
                "gflops": round(fl * 2 / 256 / dt / 1e9, 2), "sample": f"2 of 256 images, {dt:.1f} s"}
        del xa, ya
        ga = torch.randn(1, 1, 4096, 1600, device=dev)
        gb = torch.randn(1, 1, 1600, 512, device=dev) * (2.0 / 1600) ** 0.5
        gc = torch.randn(1, 1, 1, 512, device=dev) * 0.1
        gy = torch.zeros(1, 1, 4096, 512, device=dev)
        fn = lambda: tm.gemm_lean(ga, gb, gc, 1.0, 1.0, False, False, gy)
        fn(); ms = kernel_avg_ms(ctx, fn, kit)
        fl = 2 * 4096 * 1600 * 512
        operators["gemm_f32_4096x1600x512"] = {"ms": round(ms, 4), "tflops": round(fl / ms / 1e9, 2),
                                               "frac_f32_mfma_peak": round(fl / ms / 1e9 / PEAK_F32_MFMA_TFLOPS, 4)}
        rows = np.r_[0:128, 4096 - 128:4096]  # the first and the last row block
        gas = ga[:, :, rows].cpu().numpy()
        t0 = time.perf_counter()
        ref_g = zo.gemm(gas, gb.cpu().numpy(), gc.cpu().numpy(), 1.0, 1.0, False, False)
        dt = time.perf_counter() - t0
        np.testing.assert_allclose(gy[:, :, rows].cpu().numpy(), ref_g, rtol=1e-4, atol=1e-5)
        operators["gemm_f32_4096x1600x512"]["parity_gate"] = "rows 0..127 and 3968..4095 of the timed output against the oracle, rtol 1e-4 atol 1e-5"
        if not args.no_cpu_baseline:
            operators["gemm_f32_4096x1600x512"]["cpu_oracle_1core"] = {
                "gflops": round(fl * 256 / 4096 / dt / 1e9, 2), "sample": f"256 of 4096 rows, {dt:.1f} s"}
        xq = torch.randint(0, 256, (128, 128, 28, 28), dtype=torch.uint8, device=dev)
        wq = torch.randint(-127, 128, (128, 128, 3, 3), dtype=torch.int8, device=dev)
        ws = torch.rand(128, device=dev) * 0.009 + 0.001
        bq = torch.randint(-1000, 1001, (128,), dtype=torch.int32, device=dev)
        yq = torch.zeros(128, 128, 28, 28, dtype=torch.uint8, device=dev)
        fn = lambda: tm.qlinearconv_lean(xq, 0.02, 128, wq, ws, None, 0.05, 128, bq, yq, [1, 1], [1, 1, 1, 1], [1, 1])
        fn(); ms = kernel_avg_ms(ctx, fn, kit)
        q_kernel = ctx.kernel_name()
        # the whole lean call as a per-operator binding pays it: weight packing included (the kernel regroups the NCHW
        # input into 16-channel units itself; its time above includes that)
        ctx.sync(); ctx.timer_start()
        for _ in range(kit):
            fn()
        call_ms = ctx.timer_stop() / kit
        op = 2 * 128 * 128 * 28 * 28 * 128 * 9
        operators["qlinearconv_u8i8_N128_C128_28x28_K128_3x3"] = {"ms": round(ms, 4), "tops": round(op / ms / 1e9, 2),
                                                                  "frac_i8_mfma_peak": round(op / ms / 1e9 / PEAK_I8_MFMA_TOPS, 5),
                                                                  "kernel": q_kernel, "whole_call_ms": round(call_ms, 4)}
        # with a prepared-weights handle (zant_hip_qlinearconv_prepack): NCHW tensors, and channel-blocked tensors on both
        # sides (no regrouping of the input, no staging of the output: what a chain of convolutions pays per layer)
        qop = operators["qlinearconv_u8i8_N128_C128_28x28_K128_3x3"]
        plan = tm.QConvPlan(xq.shape, 0.02, 128, wq, ws, None, 0.05, 128, bq, [1, 1], [1, 1, 1, 1], [1, 1])
        yq2 = torch.zeros_like(yq)
        plan(xq, yq2)
        assert torch.equal(yq2, yq), "config 3: the prepared call differs from the plain one"
        ctx.sync(); ctx.timer_start()
        for _ in range(kit):
            plan(xq, yq2)
        qop["prepared_call_ms"] = round(ctx.timer_stop() / kit, 4)
        plan.close()
        planb = tm.QConvPlan(xq.shape, 0.02, 128, wq, ws, None, 0.05, 128, bq, [1, 1], [1, 1, 1, 1], [1, 1],
                             x_layout=tm.BLOCKED16, y_layout=tm.BLOCKED16)
        xb = tm.to_blocked16(xq)
        yb = planb(xb)
        assert torch.equal(tm.from_blocked16(yb, yq.shape), yq), "config 3: the blocked prepared call differs from the plain one"
        ctx.sync(); ctx.timer_start()
        for _ in range(kit):
            planb(xb, yb)
        qop["prepared_blocked_call_ms"] = round(ctx.timer_stop() / kit, 4)
        qop["prepared_blocked_kernel_ms"] = round(kernel_avg_ms(ctx, lambda: planb(xb, yb), kit), 4)
        planb.close()
        del xb, yb, yq2
        pick = [0, 127]
        t0 = time.perf_counter()
        ref_q = zo.qlinearconv(xq[pick].cpu().numpy(), 0.02, 128, wq.cpu().numpy(), ws.cpu().numpy(), None, 0.05, 128,
                               bq.cpu().numpy(), [1, 1], [1, 1, 1, 1], [1, 1])
        dt = time.perf_counter() - t0
        assert np.array_equal(yq[pick].cpu().numpy(), ref_q), "config 3: timed output differs from the oracle"
        operators["qlinearconv_u8i8_N128_C128_28x28_K128_3x3"]["parity_gate"] = "images 0 and 127 of the timed output against the oracle, bit-exact"
        if not args.no_cpu_baseline:
            operators["qlinearconv_u8i8_N128_C128_28x28_K128_3x3"]["cpu_oracle_1core"] = {
                "gops": round(op * 2 / 128 / dt / 1e9, 2), "sample": f"2 of 128 images, {dt:.1f} s"}
        # the same layer at batch 1024: eight tiles per compute unit instead of one, which shows the rate of the
        # kernel's tile pipeline apart from launch, first fill and the last epilogue
        del xq, yq
        xq8 = torch.randint(0, 256, (1024, 128, 28, 28), dtype=torch.uint8, device=dev)
        yq8 = torch.zeros(1024, 128, 28, 28, dtype=torch.uint8, device=dev)
        fn8 = lambda: tm.qlinearconv_lean(xq8, 0.02, 128, wq, ws, None, 0.05, 128, bq, yq8, [1, 1], [1, 1, 1, 1], [1, 1])
        fn8(); ms8 = kernel_avg_ms(ctx, fn8, kit)
        k8 = ctx.kernel_name()
        ctx.sync(); ctx.timer_start()
        for _ in range(kit):
            fn8()
        call8 = ctx.timer_stop() / kit
        planb8 = tm.QConvPlan(xq8.shape, 0.02, 128, wq, ws, None, 0.05, 128, bq, [1, 1], [1, 1, 1, 1], [1, 1],
                              x_layout=tm.BLOCKED16, y_layout=tm.BLOCKED16)
        xb8 = tm.to_blocked16(xq8)
        yb8 = planb8(xb8)
        assert torch.equal(tm.from_blocked16(yb8, yq8.shape), yq8), "config 3 at batch 1024: the blocked prepared call differs from the plain one"
        for _ in range(5):
            planb8(xb8, yb8)
        ctx.sync(); ctx.timer_start()
        for _ in range(kit):
            planb8(xb8, yb8)
        blocked8 = ctx.timer_stop() / kit
        planb8.close()
        del xb8, yb8
        ref8 = zo.qlinearconv(xq8[[0, 1023]].cpu().numpy(), 0.02, 128, wq.cpu().numpy(), ws.cpu().numpy(), None, 0.05, 128,
                              bq.cpu().numpy(), [1, 1], [1, 1, 1, 1], [1, 1])
        assert np.array_equal(yq8[[0, 1023]].cpu().numpy(), ref8), "config 3 at batch 1024: timed output differs from the oracle"
        operators["qlinearconv_u8i8_N1024_C128_28x28_K128_3x3"] = {
            "ms": round(ms8, 4), "tops": round(8 * op / ms8 / 1e9, 2), "frac_i8_mfma_peak": round(8 * op / ms8 / 1e9 / PEAK_I8_MFMA_TOPS, 5),
            "kernel": k8, "whole_call_ms": round(call8, 4), "prepared_blocked_call_ms": round(blocked8, 4),
            "prepared_blocked_frac_i8_mfma_peak": round(8 * op / blocked8 / 1e9 / PEAK_I8_MFMA_TOPS, 5), "parity_gate": "images 0 and 1023 of the timed output against the oracle, bit-exact"}
        del xq8, yq8

    # ---- HBM-bound operators (pool / activation / requantisation / residual add): algorithmic bytes / kernel time ----
    if operators is not None:
        # What the machine gives a plain device-to-device copy moving the same number of bytes (half read, half
        # written), measured here with HIP events: the practical ceiling of a streaming kernel of that size, beside the
        # fraction of the 8 TB/s peak.
        copy_cache = {}

        def copy_gbs(nbytes):
            half = max(int(nbytes) // 2 // 256 * 256, 256)
            if half not in copy_cache:
                src = torch.empty(half, dtype=torch.uint8, device=dev).fill_(1)
                dst = torch.empty_like(src)
                for _ in range(3):
                    dst.copy_(src)
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                torch.cuda.synchronize()
                e0.record()
                for _ in range(10):
                    dst.copy_(src)
                e1.record()
                torch.cuda.synchronize()
                copy_cache[half] = 2 * half / (e0.elapsed_time(e1) / 10) / 1e6
                del src, dst
            return copy_cache[half]

        def hbm(name, fn, nbytes):
            # Timed like the copy beside it: ten launches back to back between two events.  Events around every single
            # launch (kernel_event_ms) add two to three microseconds of record and dispatch time to each, a fifth of a
            # 15 us kernel and nothing the copy's figure carries.
            fn()
            ev_ms = kernel_avg_ms(ctx, fn, 5)
            ctx.sync(); ctx.timer_start()
            for _ in range(10):
                fn()
            ms = ctx.timer_stop() / 10
            operators[name] = {"ms": round(ms, 4), "kernel_event_ms": round(ev_ms, 4), "gbs": round(nbytes / ms / 1e6, 1),
                               "frac_hbm_peak": round(nbytes / ms / 1e6 / PEAK_HBM_GBS, 4),
                               "plain_copy_same_bytes_gbs": round(copy_gbs(nbytes), 1)}

        xf = torch.randn(4096, 32, 26, 26, device=dev)
        yf = torch.empty_like(xf)
        hbm("relu_f32_4096x32x26x26", lambda: tm.ReLU_lean(xf, yf), 2 * xf.numel() * 4)
        hbm("leaky_relu_f32_4096x32x26x26", lambda: tm.leakyReLU_lean(xf, 0.1, yf), 2 * xf.numel() * 4)
        yp = torch.empty(4096, 32, 13, 13, device=dev)
        hbm("maxpool2x2_f32_4096x32x26x26", lambda: tm.onnx_maxpool_lean(xf, yp, [2, 2], [2, 2], [1, 1], [0, 0, 0, 0]),
            xf.numel() * 5)
        hbm("avgpool2x2_f32_4096x32x26x26", lambda: tm.avgpool_lean(xf, yp, [2, 2], [2, 2]), xf.numel() * 5)
        bn = [torch.rand(32, device=dev) + 0.5 for _ in range(4)]
        hbm("batchnorm_f32_4096x32x26x26", lambda: tm.batchnorm(xf, bn[0], bn[1], bn[2], bn[3], 1e-5, out=yf), 2 * xf.numel() * 4)
        bf = torch.randn(4096, 32, 26, 26, device=dev)
        hbm("add_f32_same_shape", lambda: tm.sum_tensors_lean(xf, bf, yf), 3 * xf.numel() * 4)
        bc = torch.randn(32, 1, 1, device=dev)
        hbm("add_f32_per_channel_broadcast", lambda: tm.sum_tensors_lean(xf, bc, yf), 2 * xf.numel() * 4)
        hbm("sigmoid_f32_4096x32x26x26", lambda: tm.sigmoid_lean(xf, yf), 2 * xf.numel() * 4)
        del bf, yp
        gx = torch.randn(256, 64, 56, 56, device=dev)
        gy = torch.empty(256, 64, 1, 1, device=dev)
        hbm("reduce_mean_hw_f32_256x64x56x56", lambda: tm.reduce_mean_lean(gx, gy, [2, 3], True), gx.numel() * 4 + gy.numel() * 4)
        cy = torch.empty(256, 128, 56, 56, device=dev)
        hbm("concat_channels_f32_2x256x64x56x56", lambda: tm.lean_concatenate([gx, gx], 1, cy), 2 * cy.numel() * 4)
        del cy
        rx = torch.randn(256, 64, 28, 28, device=dev)
        ry = torch.empty(256, 64, 56, 56, device=dev)
        hbm("resize_nearest_x2_f32_256x64x28x28", lambda: tm.resize(rx, "nearest", [1.0, 1.0, 2.0, 2.0], None, "asymmetric", out=ry),
            5 * rx.numel() * 4)
        del gx, gy, rx, ry
        sm = torch.randn(1 << 20, 10, device=dev)
        so = torch.empty_like(sm)
        hbm("softmax_f32_1Mx10", lambda: tm.softmax_lean(sm, so), 2 * sm.numel() * 4)
        del sm, so, xf, yf
        qa = torch.randint(0, 256, (1024, 96, 48, 48), dtype=torch.uint8, device=dev)
        qb = torch.randint(0, 256, qa.shape, dtype=torch.uint8, device=dev)
        qo = torch.empty_like(qa)
        hbm("qlinear_relu6_u8_1024x96x48x48", lambda: tm.qlinear_act(qa, 0.05, 128, "relu6", 0.0, 0.03, 0, out=qo), 2 * qa.numel())
        hbm("qlinear_add_u8_1024x96x48x48", lambda: tm.qlinear_add(qa, 0.05, 128, qb, 0.04, 120, 0.07, 100, out=qo), 3 * qa.numel())
        qp = torch.empty(1024, 96, 24, 24, dtype=torch.uint8, device=dev)
        hbm("maxpool2x2_u8_1024x96x48x48", lambda: tm.onnx_maxpool_lean(qa, qp, [2, 2], [2, 2], [1, 1], [0, 0, 0, 0]),
            qa.numel() * 5 // 4)
        qg = torch.empty(1024, 96, 1, 1, dtype=torch.uint8, device=dev)
        hbm("qlinear_global_avgpool_u8_1024x96x48x48", lambda: tm.qlinear_global_avgpool(qa, 0.05, 128, 0.05, 128, out=qg), qa.numel())
        ff = torch.randn(1024, 96, 48, 48, device=dev)
        s1 = torch.tensor([0.05], device=dev)
        z1 = torch.tensor([128], dtype=torch.uint8, device=dev)
        fo = torch.empty_like(ff)
        hbm("quantize_linear_f32_u8", lambda: tm.quantize_linear(ff, s1, z1, 1, out=qo), ff.numel() * 5)
        hbm("dequantize_linear_u8_f32", lambda: tm.dequantize_linear(qa, s1, z1, 1, out=fo), ff.numel() * 5)
        del qa, qb, qp, ff, qo, fo, qg
        # depthwise 3x3 between channel-blocked tensors (the layout the executor keeps int8 activations in), timed as a
        # node of a small model: dense 3x3 -> depthwise 3x3 -> dense 3x3 keeps it out of the fused-block pattern
        from zant_amd.model import Model, U8
        gd = np.random.default_rng(3)
        DN, DC, DH = 1024, 96, 48
        dm = Model(ctx)
        dt = dm.input((DN, 16, DH, DH), U8, 0.02, 128)
        dws = gd.uniform(0.001, 0.01, DC).astype(np.float32)
        dt = dm.qlinearconv(dt, gd.integers(-127, 128, (DC, 16, 3, 3), dtype=np.int8), dws, gd.integers(-99, 99, DC, dtype=np.int32),
                            0.05, 128, [1, 1], [1, 1, 1, 1])
        dt = dm.qlinearconv(dt, gd.integers(-127, 128, (DC, 1, 3, 3), dtype=np.int8), dws, gd.integers(-99, 99, DC, dtype=np.int32),
                            0.05, 128, [1, 1], [1, 1, 1, 1], [1, 1], DC)
        dt = dm.qlinearconv(dt, gd.integers(-127, 128, (16, DC, 3, 3), dtype=np.int8), dws[:16], gd.integers(-99, 99, 16, dtype=np.int32),
                            0.05, 128, [1, 1], [1, 1, 1, 1])
        dm.finalize()
        dm.profile()
        dw_ms = sum(dm.profile()[1][1] for _ in range(5)) / 5
        dw_bytes = 2 * DN * DC * DH * DH + 9 * DC + 8 * DC
        operators["qlinearconv_depthwise3x3_u8_blocked_1024x96x48x48"] = {
            "ms": round(dw_ms, 4), "gbs": round(dw_bytes / dw_ms / 1e6, 1), "frac_hbm_peak": round(dw_bytes / dw_ms / 1e6 / PEAK_HBM_GBS, 4)}
        dm.close()

    # ---- int8 networks (configs 4 and 5): whole-network throughput with the calibrated scales of the golden fixture ----
    nets_out = None
    if not args.no_networks:
        nets_out = {}
        gold = json.load(open(os.path.join(ROOT, "tests", "golden", "int8_networks.json")))
        for name, arch, nb in (("tiny_yolo_int8", networks.tiny_yolo_arch(), 512),
                               ("mobilenet_v2_035_int8", networks.mobilenet_v2_035_arch(), 1024)):
            qparams = networks.int8_params(arch, seed=gold[name]["param_seed"])
            qm = networks.build_int8_model(ctx, arch, qparams, gold[name]["quant"], nb)
            xq = np.random.default_rng(2).integers(0, 256, (nb,) + tuple(arch["input"]), dtype=np.uint8)
            # parity gate: the two golden images at the head of the batch must reproduce the oracle's bytes
            xg = np.random.default_rng(gold[name]["input_seed"]).integers(0, 256, (2,) + tuple(arch["input"]), dtype=np.uint8)
            xq[:2] = xg
            yq = qm.predict_host(xq)
            assert np.array_equal(yq[:2].ravel(), np.array(gold[name]["expected_u8"], np.uint8)), name
            for _ in range(3):
                qm.run()
            ctx.sync()
            ctx.timer_start()
            for _ in range(kit):
                qm.run()
            ms = ctx.timer_stop() / kit
            macs = gold[name]["macs_per_inference"]
            # the two floors of the pass: its integer operations at the int8 matrix-core peak, and the algorithmic
            # bytes of its launches (inputs + parameters + output of each, once) at the HBM peak
            prof = qm.profile()
            nets_out[name] = {"batch": nb, "ms_per_step": round(ms, 4), "inferences_per_s": round(nb / ms * 1e3, 1),
                              "tops": round(2.0 * macs * nb / ms / 1e9, 2), "launches_per_step": qm.num_launches,
                              "arena_bytes": qm.arena_bytes,
                              "mfma_floor_ms": round(2.0 * macs * nb / (PEAK_I8_MFMA_TOPS * 1e12) * 1e3, 4),
                              "hbm_floor_ms": round(sum(pb for _, _, _, pb in prof) / (PEAK_HBM_GBS * 1e9) * 1e3, 4),
                              "kernel_ms": [round(pm, 4) for _, pm, _, _ in prof]}
            qm.close()

    # ---- CPU baseline: the oracle on one host core, one image at a time, over a bounded sample ----
    cpu = None
    if not args.no_cpu_baseline:
        sample = 3 * BATCH  # about 15 s of CPU work
        t0 = time.perf_counter()
        for i in range(sample):
            oracle_forward(x_host[i % BATCH:i % BATCH + 1])
        dt = time.perf_counter() - t0
        cpu = {"value": round(sample / dt, 2), "unit": "inferences/s", "cores": 1, "kind": "port",
               "host_cores": os.cpu_count(),
               "sample": f"{sample} images (the batch, three times over), batch 1 per call (how the reference's predict() runs), "
                         f"{dt:.1f} s of CPU time; each image is nine calls from a Python loop into the C oracle through ctypes, "
                         "with numpy allocating every output: the interpreter and allocation overhead is inside the figure"}

    line = {
        "metric": "batched inferences/sec + conv TOPS (% of MI355X peak) at batch 4096",
        "value": round(value, 1), "unit": "inferences/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "config 1: README f32 CNN (Conv32-ReLU-Pool-Conv64-ReLU-Pool-Gemm512-ReLU-Gemm10-Softmax), "
                               "input 4096x1x28x28 ~U[0,1), He-normal weights, seed 0", "batch": BATCH,
                   "flop_per_inference_executed": flops["executed"], "flop_per_inference_graph": flops["total"],
                   "launches_per_step": model.num_launches,
                   "arena_bytes": model.arena_bytes, "unfused_activation_bytes": model.unfused_bytes,
                   # executed work: the fused pass computes conv2 at 10x10 (the pool drops row / column 10)
                   "tflops": round(flops["executed"] * BATCH / (ms_per_step * 1e-3) / 1e12, 2),
                   "tflops_graph_flop": round(flops["total"] * BATCH / (ms_per_step * 1e-3) / 1e12, 2),
                   "lean_call_path": lean_path},
        "roofline": roofline,
        "cpu_baseline": cpu,
        "kernels": per_kernel,
        "operators": operators,
        "networks": nets_out,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
