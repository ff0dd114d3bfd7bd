#!/usr/bin/env python3
"""Benchmark of the activation-compression hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One step = one pass of the hot path over benchmark config 2: minimax -> pack_mixed_precision
(in-kernel Philox) -> unpack_mixed_precision on a resident fp32 activation [256,256,56,56]
(ResNet-50 layer1), per-sample bits from the greedy allocation at an average of 2.0 bits,
groups of 256.  `value` is algorithmic bytes per step / time per step.  The JSON line also
carries the roofline figures of every kernel (HIP-event timed), the other single-GPU configs
(ReLU / max-pool masks on fp16, fixed-width pack, fused QLinear weight gradient, the ResNet-50
L3 step when the host layer is importable) and the CPU baseline (the oracle's restatement of
the reference's config.simulate quantiser on this box's host cores).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
MFMA_BF16_PEAK_TFLOPS = 2500.0  # dense bf16, published

# HBM bytes per launch measured with rocprofv3 --pmc (FETCH_SIZE, then WRITE_SIZE, each scaled by
# what the same counter reads for actnn_stream_copy of a known size); see profiles/.  None = not
# measured yet.
MEASURED_TRAFFIC_BYTES = {"minimax": 828536830, "pack_mixed": 892254308, "unpack_mixed": 886732426}


def _event_time_ms(fn, reps, warmup=3):
    """Average duration of fn() over `reps` launches, HIP events on the current stream (the
    stream every kernel of this library is launched on)."""
    import torch
    for _ in range(warmup):
        fn()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(reps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / reps


def make_config2(device, N=256, C=256, H=56, W=56, seed=0):
    """fp32 activation of benchmark config 2 and its per-sample bits (greedy at avg 2.0 bits)."""
    import torch
    import actnn_amd.cpp_extension.calc_precision as ext_cp
    import actnn_amd.cpp_extension.minimax as ext_minimax
    import actnn_amd.cpp_extension.quantization as ext_q
    g = torch.Generator(device=device).manual_seed(seed)
    s_c = torch.exp(torch.randn(C, generator=g, device=device))
    x = torch.randn(N, C, H, W, generator=g, device=device)
    x = torch.relu_(x).mul_(s_c.view(1, C, 1, 1))
    # samples differ in range (LogNormal(0, 0.7) per sample): with identically distributed samples
    # the greedy allocation hands every sample the same width and the mixed-width path is not used
    x.mul_(torch.exp(0.7 * torch.randn(N, generator=g, device=device)).view(N, 1, 1, 1))
    gs = 256
    G = C * H * W // gs
    xg = x.view(N, G, gs)
    mn, mx = ext_minimax.minimax(xg.view(-1, gs))
    mn, mx = mn.view(N, G, 1), mx.view(N, G, 1)
    # sensitivity and greedy allocation as the reference's scheme does (qscheme.py:80-88) with
    # num_locations = 1 and grad_sum = 1
    num_pixels = H * W
    range_sqr = torch.norm((mx - mn).view(N, -1), dim=1).float().square() * (gs / num_pixels)
    Cs = (1 / 4 * range_sqr).to(torch.float32).cpu()
    b = torch.ones(N, dtype=torch.int32) * 8
    w = torch.ones(N, dtype=torch.int32)
    b = ext_cp.calc_precision(b, Cs, w, int(2 * N))
    bits = ext_q.attach_bits_host(b.to(device), b)
    return xg, mn, mx, bits, b


def algorithmic_bytes(n, esize, avg_bits, gs=256):
    groups = n // gs
    return {
        "minimax": n * esize + 2 * groups * esize,
        "pack_mixed": n * esize + 2 * groups * esize + avg_bits * n / 8 + groups * esize,
        "unpack_mixed": avg_bits * n / 8 + 2 * groups * esize + n * esize,
    }


def cpu_baseline(budget_s=15.0):
    """The oracle's restatement of the reference's config.simulate quantise+dequantise
    (actnn/actnn/ops.py:22-41,55-57) on benchmark config 1, all host cores."""
    import torch
    from oracle import simulate
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    torch.manual_seed(0)
    x = torch.relu(torch.randn(32, 64, 56, 56)).view(32, 784, 256)
    noise = torch.rand(32, 784, 256, generator=torch.Generator().manual_seed(1)) - 0.5
    mn, mx = x.min(2, keepdim=True)[0], x.max(2, keepdim=True)[0]

    def run():
        q, s = simulate.quantize_simulate(x.clone(), 2, mn, mx, noise)
        return simulate.dequantize_simulate(q, s, mn)

    for _ in range(3):
        run()
    times = []
    t_end = time.perf_counter() + budget_s
    while len(times) < 10 or (time.perf_counter() < t_end and len(times) < 200):
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    n = x.numel()
    return {"value": round(4 * n / med / 1e9, 3), "unit": "GB/s", "cores": torch.get_num_threads(),
            "kind": "port", "elements_per_s": round(n / med, 1), "median_ms": round(med * 1e3, 3),
            "sample": f"config.simulate quantise+dequantise of fp32 [32,64,56,56] (n={n}), 2 bits, "
                      f"median of {len(times)} repetitions; GB/s over 4n input bytes"}


def other_configs(device, reps):
    """ReLU / max-pool on fp16 [256,64,112,112] (config 3) and fixed-width pack on fp16 [8192,4096]."""
    import torch
    import actnn_amd.cpp_extension.minimax as ext_minimax
    import actnn_amd.cpp_extension.quantization as ext_q
    out = {}
    x = torch.randn(256, 64, 112, 112, device=device, dtype=torch.float16)
    g = torch.randn_like(x)
    n = x.numel()
    y, mask = ext_q.relu_forward(x)
    t = _event_time_ms(lambda: ext_q.relu_forward(x), reps)
    b = 2 * n + 2 * n + n / 8
    out["relu_forward_f16"] = {"ms": t, "GB/s": b / t / 1e6, "frac": b / t / 1e6 / HBM_PEAK_GBS}
    t = _event_time_ms(lambda: ext_q.relu_backward(g, mask), reps)
    out["relu_backward_f16"] = {"ms": t, "GB/s": b / t / 1e6, "frac": b / t / 1e6 / HBM_PEAK_GBS}
    _, keep = ext_q.dropout_forward(x, 0.25)
    t = _event_time_ms(lambda: ext_q.dropout_forward(x, 0.25), reps)
    out["dropout_forward_f16"] = {"ms": t, "GB/s": b / t / 1e6, "frac": b / t / 1e6 / HBM_PEAK_GBS}
    t = _event_time_ms(lambda: ext_q.dropout_backward(g, keep, 0.25), reps)
    out["dropout_backward_f16"] = {"ms": t, "GB/s": b / t / 1e6, "frac": b / t / 1e6 / HBM_PEAK_GBS}
    del keep
    k, s, p = (3, 3), (2, 2), (1, 1)
    yp, idx = ext_q.max_pool2d_forward(x, k, s, p, (1, 1))
    gp = torch.randn_like(yp)
    b = 2 * n + 2 * n / 4 + n / 4
    t = _event_time_ms(lambda: ext_q.max_pool2d_forward(x, k, s, p, (1, 1)), reps)
    out["max_pool2d_forward_f16"] = {"ms": t, "GB/s": b / t / 1e6, "frac": b / t / 1e6 / HBM_PEAK_GBS}
    t = _event_time_ms(lambda: ext_q.max_pool2d_backward(gp, idx, x.shape, k, s, p), reps)
    out["max_pool2d_backward_f16"] = {"ms": t, "GB/s": b / t / 1e6, "frac": b / t / 1e6 / HBM_PEAK_GBS}
    del y, mask, yp, idx, gp
    # training-mode batch norm on the same tensor, in both layouts: forward (statistics + normalise;
    # with the quantiser's group min/max from the statistics pass; with the 2-bit pack in the
    # normalising pass), backward from the full-precision input and straight from the 2-bit stream
    import actnn_amd.cpp_extension.backward_func as ext_bf
    from actnn_amd.ops import _Quantized
    from actnn_amd.utils import memory_order
    C = x.shape[1]
    w = torch.rand(C, device=device) + 0.5
    bias = torch.randn(C, device=device)
    Nb, Gb = x.shape[0], n // x.shape[0] // 256
    host_bits = torch.full((Nb,), 2, dtype=torch.int32)
    bits2 = ext_q.attach_bits_host(host_bits.to(device), host_bits)
    for tag, fmt in (("", torch.contiguous_format), ("_channels_last", torch.channels_last)):
        xb, gb = x.contiguous(memory_format=fmt), g.contiguous(memory_format=fmt)

        def rate(name, nbytes, fn):
            t = _event_time_ms(fn, reps)
            out[name + tag + "_f16"] = {"ms": t, "GB/s": nbytes / t / 1e6, "frac": nbytes / t / 1e6 / HBM_PEAK_GBS}
        rate("batch_norm_forward", 3 * 2 * n, lambda: ext_bf.hip_batch_norm_forward(xb, w, bias, None, None, 0.1, 1e-5))
        rate("batch_norm_forward_with_group_minmax", 3 * 2 * n + 2 * 2 * n / 256,
             lambda: ext_bf.hip_batch_norm_forward(xb, w, bias, None, None, 0.1, 1e-5, minmax=True))
        ws, mean, invstd, lo, hi = ext_bf.hip_batch_norm_forward_stats(xb, w, bias, None, None, 0.1, 1e-5)
        lo3, hi3 = lo.view(Nb, Gb, 1), hi.view(Nb, Gb, 1)
        # statistics + min/max, then normalise + 2-bit pack: x twice, y, stream, min/max/scale
        rate("batch_norm_forward_with_pack", 3 * 2 * n + 2 * n / 8 + 5 * 2 * n / 256,
             lambda: ext_bf.hip_batch_norm_forward_apply(
                 xb, ext_bf.hip_batch_norm_forward_stats(xb, w, bias, None, None, 0.1, 1e-5)[0], bits2, lo3, hi3))
        rate("batch_norm_backward", 5 * 2 * n, lambda: ext_bf.hip_batch_norm_backward(xb, gb, w, mean, invstd))
        q_in, q_scale = ext_q.pack_mixed_precision(memory_order(xb).reshape(Nb, Gb, 256), lo3, hi3, bits2, True)
        quantized = _Quantized((q_in, bits2, q_scale, lo3))
        quantized.memory_format = None if fmt == torch.contiguous_format else fmt
        # dy twice, dx once; stream, scale, min twice
        rate("batch_norm_backward_from_2bit_stream", 3 * 2 * n + 2 * (2 * n / 8 + 2 * 2 * n / 256),
             lambda: ext_bf.hip_batch_norm_backward_packed(xb.shape, quantized, gb, w, mean, invstd))
        del xb, gb
    del x, g, q_in, q_scale, quantized, lo, hi
    # config 4 input through the fixed-width path (2 bits)
    M, I = 8192, 4096
    xs = torch.randn(M, I // 256, 256, device=device, dtype=torch.float16)
    mn, mx = ext_minimax.minimax(xs.view(-1, 256))
    mn, mx = mn.view(M, -1, 1), mx.view(M, -1, 1)
    packed, scale = ext_q.pack_single_precision(xs, mn, mx, 2, True)
    ns = xs.numel()
    b = 2 * ns + 3 * 2 * ns / 256 + ns / 4
    t = _event_time_ms(lambda: ext_q.pack_single_precision(xs, mn, mx, 2, True), reps)
    out["pack_single_2bit_f16"] = {"ms": t, "GB/s": b / t / 1e6, "frac": b / t / 1e6 / HBM_PEAK_GBS}
    t = _event_time_ms(lambda: ext_q.unpack_single_precision(packed, 2, scale, mn, M, I // 256, 256), reps)
    out["unpack_single_2bit_f16"] = {"ms": t, "GB/s": b / t / 1e6, "frac": b / t / 1e6 / HBM_PEAK_GBS}
    # config 4: fused dequant + grad_weight GEMM (MFMA roofline), and the unfused path beside it
    O = 4096
    go = torch.randn(M, O, device=device, dtype=torch.float16)
    flops = 2.0 * M * O * I
    t = _event_time_ms(lambda: ext_q.linear_grad_weight_q2(go, packed, scale, mn, I), reps)
    out["linear_grad_weight_q2_fused"] = {"ms": t, "TFLOP/s": flops / t / 1e9,
                                          "frac_mfma_bf16": flops / t / 1e9 / MFMA_BF16_PEAK_TFLOPS}

    def unfused():
        x = ext_q.unpack_single_precision(packed, 2, scale, mn, M, I // 256, 256).view(M, I)
        return go.t().mm(x)
    t = _event_time_ms(unfused, reps)
    out["linear_grad_weight_unfused_unpack_plus_mm"] = {"ms": t, "TFLOP/s": flops / t / 1e9,
                                                        "frac_mfma_bf16": flops / t / 1e9 / MFMA_BF16_PEAK_TFLOPS}
    return {k_: {kk: round(vv, 4) for kk, vv in v.items()} for k_, v in out.items()}


def _heartbeat(period=30.0):
    """Progress lines on stderr while the long legs run (MIOpen's solver search during the first
    ResNet-50 step is silent for minutes); stdout stays the single JSON line."""
    import threading
    t0 = time.time()

    def beat():
        while True:
            time.sleep(period)
            print(f"[bench] running, {time.time() - t0:.0f} s", file=sys.stderr, flush=True)
    threading.Thread(target=beat, daemon=True).start()


def main():
    _heartbeat()
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--skip-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--skip-extra", action="store_true", help="only the config-2 hot path")
    ap.add_argument("--only", choices=["other", "resnet50", "resnet50_channels_last", "resnet50_fp32", "resnet50_levels", "batch_norm_shapes"],
                    default=None,
                    help="profiling aid: run just the other single-GPU configs (ReLU, max-pool, "
                         "fixed-width pack, fused GEMM), just the ResNet-50 L3 step, the fp32 "
                         "(no autocast) ResNet-50 pair of the reference's own protocol, every "
                         "optimisation level (channels-last, bf16), or the fused "
                         "batch-norm passes on every batch-norm shape of ResNet-50; print their JSON")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: the hot path shards by sample with no exchange step, "
                 "and this build runs on single-GPU boxes only (--gpus must be 1).")

    import torch
    import actnn_amd.cpp_extension.minimax as ext_minimax
    import actnn_amd.cpp_extension.quantization as ext_q
    from actnn_amd import _lib
    lib = _lib.load()

    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    if args.only == "other":
        print(json.dumps({"other_configs": other_configs(device, max(10, args.steps // 2))}))
        return
    if args.only == "resnet50":
        import bench_extra
        print(json.dumps({"resnet50_L3": bench_extra.resnet50_step(device, "L3", warmup=2, steps=3)}))
        return
    if args.only == "resnet50_channels_last":
        import bench_extra
        print(json.dumps({"resnet50_L3_channels_last": bench_extra.resnet50_step(
            device, "L3", warmup=2, steps=3, channels_last=True)}))
        return
    if args.only == "resnet50_fp32":
        import bench_extra
        out = {}
        for key, level, cl in (("resnet50_fp32_exact", "exact", False), ("resnet50_fp32_L3", "L3", False),
                               ("resnet50_fp32_exact_channels_last", "exact", True),
                               ("resnet50_fp32_L3_channels_last", "L3", True)):
            torch.cuda.empty_cache()
            torch.cuda.reset_peak_memory_stats()
            out[key] = bench_extra.resnet50_step(device, level, warmup=2, steps=5, autocast=False, channels_last=cl)
        print(json.dumps(out))
        return
    if args.only == "resnet50_levels":
        import bench_extra
        out = {}
        for level in ("exact", "L0", "L1", "L2", "L3", "L3.1", "L4", "swap"):
            torch.cuda.empty_cache()
            torch.cuda.reset_peak_memory_stats()
            out["resnet50_" + level] = bench_extra.resnet50_step(device, level, warmup=2, steps=5, channels_last=True)
            print("[bench] %s done" % level, file=sys.stderr, flush=True)
        print(json.dumps(out))
        return
    if args.only == "batch_norm_shapes":
        import bench_extra
        print(json.dumps({"batch_norm_shapes": [bench_extra.batch_norm_shapes(device, channels_last=cl)
                                                for cl in (True, False)]}))
        return
    xg, mn, mx, bits, bits_host = make_config2(device)
    N, G, gs = xg.shape
    n = xg.numel()
    avg_bits = float(bits_host.float().mean())
    ab = algorithmic_bytes(n, 4, avg_bits)

    def step():
        lo, hi = ext_minimax.minimax(xg.view(-1, gs))
        packed, scale = ext_q.pack_mixed_precision(xg, lo.view(N, G, 1), hi.view(N, G, 1), bits, True)
        return ext_q.unpack_mixed_precision(packed, bits, scale, lo.view(N, G, 1), N, G, gs)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    step_bytes = ab["minimax"] + ab["pack_mixed"] + ab["unpack_mixed"]
    value = step_bytes / ms_per_step / 1e6

    # per-kernel timing (HIP events on the launch stream)
    reps = max(20, args.steps)
    packed, scale = ext_q.pack_mixed_precision(xg, mn, mx, bits, True)
    kern = {
        "minimax": _event_time_ms(lambda: ext_minimax.minimax(xg.view(-1, gs)), reps),
        "pack_mixed": _event_time_ms(lambda: ext_q.pack_mixed_precision(xg, mn, mx, bits, True), reps),
        "unpack_mixed": _event_time_ms(lambda: ext_q.unpack_mixed_precision(packed, bits, scale, mn, N, G, gs), reps),
    }
    # plain copy of the same footprint: what a streaming kernel reaches on this box
    dst = torch.empty_like(xg)
    copy_ms = _event_time_ms(lambda: _lib.check(lib.actnn_stream_copy(
        xg.data_ptr(), dst.data_ptr(), n * 4, torch.cuda.current_stream().cuda_stream), "copy"), reps)
    del dst
    kernels = {k: {"ms": round(v, 4), "GB/s": round(ab[k] / v / 1e6, 1),
                   "frac": round(ab[k] / v / 1e6 / HBM_PEAK_GBS, 4), "algorithmic_bytes": int(ab[k])}
               for k, v in kern.items()}
    kernels["stream_copy"] = {"ms": round(copy_ms, 4), "GB/s": round(2 * n * 4 / copy_ms / 1e6, 1),
                              "frac": round(2 * n * 4 / copy_ms / 1e6 / HBM_PEAK_GBS, 4)}
    pair_ms = kern["minimax"] + kern["pack_mixed"]
    pair = {"ms": round(pair_ms, 4), "GB/s": round((ab["minimax"] + ab["pack_mixed"]) / pair_ms / 1e6, 1),
            "frac": round((ab["minimax"] + ab["pack_mixed"]) / pair_ms / 1e6 / HBM_PEAK_GBS, 4)}

    dom = "pack_mixed"
    roofline = {"bound": "hbm", "kernel": dom, "achieved": kernels[dom]["GB/s"], "peak": HBM_PEAK_GBS,
                "unit": "GB/s", "frac": kernels[dom]["frac"],
                "traffic": MEASURED_TRAFFIC_BYTES.get(dom)}

    result = {
        "metric": "pack+unpack GB/s & % HBM peak at avg 2-bit; R50 L3 train images/sec",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "configs[1]: minimax + pack_mixed_precision + unpack_mixed_precision, "
                               "fp32 [256,256,56,56], group 256, greedy bits at avg "
                               f"{avg_bits:.3f} (min {int(bits_host.min())}, max {int(bits_host.max())}), "
                               "in-kernel Philox",
                   "bytes_per_step": int(step_bytes)},
        "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4),
        "roofline": roofline,
        "kernels": kernels,
        "minimax_plus_pack": pair,
    }
    if not args.skip_extra:
        del packed, scale
        torch.cuda.empty_cache()
        try:
            result["other_configs"] = other_configs(device, max(10, args.steps // 2))
        except Exception as e:                       # keep the headline line even if an extra fails
            result["other_configs"] = {"error": repr(e)}
        try:
            import bench_extra
            result.update(bench_extra.run(device))
        except ImportError:
            pass
        except Exception as e:
            result["extra_error"] = repr(e)
    if not args.skip_cpu:
        result["cpu_baseline"] = cpu_baseline()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
