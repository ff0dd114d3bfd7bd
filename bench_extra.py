"""Extra benchmark legs used by bench.py: the ResNet-50 training step under QModule at L3
(benchmark config 5) with the reference's speed and memory protocols
(mem_speed_benchmark/train.py:363-397 memory, :422-438 speed)."""
import sys
import gc
import time

import torch
import torch.nn.functional as F

from actnn_amd import QBNScheme, QModule, QScheme, config, set_optimization_level
from actnn_amd.resnet import resnet50
from actnn_amd.utils import compute_tensor_bytes, get_memory_usage


def resnet50_step(device, level="L3", batch=512, warmup=3, steps=10, autocast=True, channels_last=False):
    """images/s = batch / median step time over `steps` steps after `warmup`; activation memory =
    allocated before backward - allocated after the data is loaded - bytes(loss, output)."""
    config.reset()
    QScheme.reset()
    QBNScheme.reset()
    model = resnet50()
    if level != "exact":
        set_optimization_level(level)
        model = QModule(model)
    model = model.to(device).train()
    if channels_last:
        model = model.to(memory_format=torch.channels_last)
    opt = torch.optim.SGD(model.parameters(), lr=0.1, momentum=0.9, weight_decay=1e-4)
    g = torch.Generator(device=device).manual_seed(0)
    images = torch.randn(batch, 3, 224, 224, generator=g, device=device)
    if channels_last:
        images = images.contiguous(memory_format=torch.channels_last)
    target = torch.randint(0, 1000, (batch,), generator=g, device=device)
    times, act_mem, peak = [], None, None
    for it in range(warmup + steps):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        init_mem = get_memory_usage()
        with torch.autocast("cuda", dtype=torch.bfloat16, enabled=autocast):
            output = model(images)
            loss = F.cross_entropy(output, target)
        if it == warmup:
            torch.cuda.synchronize()
            before_backward = get_memory_usage()
            act_mem = before_backward - init_mem - compute_tensor_bytes([loss, output])
        opt.zero_grad(set_to_none=True)
        loss.backward()
        opt.step()
        del loss, output
        torch.cuda.synchronize()
        if it >= warmup:
            times.append(time.perf_counter() - t0)
        # progress on stderr: the first steps of a fresh process spend minutes in the convolution
        # library's solver search, and a silent process looks hung to whoever supervises it
        print(f"[bench] resnet50 {level} {'channels_last' if channels_last else 'contiguous'} "
              f"autocast={autocast} step {it + 1}/{warmup + steps}: {time.perf_counter() - t0:.3f} s",
              file=sys.stderr, flush=True)
    peak = torch.cuda.max_memory_allocated()
    times.sort()
    med = times[len(times) // 2]
    config.reset()
    QScheme.reset()
    QBNScheme.reset()
    return {"images_per_s": round(batch / med, 1), "ms_per_step": round(med * 1e3, 2),
            "activation_mem_MB": round(act_mem / 2 ** 20, 1), "peak_mem_MB": round(peak / 2 ** 20, 1),
            "batch": batch, "level": level, "autocast_bf16": autocast,
            "memory_format": "channels_last" if channels_last else "contiguous", "warmup": warmup, "steps": steps}


def run(device):
    """ResNet-50, batch 512, bf16 autocast: L3 and the unquantised model, in the channels-last
    layout (what this GPU's convolution kernels work in natively) and in the default one."""
    out = {}
    for key, level, channels_last in (("resnet50_L3_channels_last", "L3", True),
                                      ("resnet50_exact_channels_last", "exact", True),
                                      ("resnet50_L3", "L3", False),
                                      ("resnet50_exact", "exact", False)):
        torch.cuda.empty_cache()
        torch.cuda.reset_peak_memory_stats()
        out[key] = resnet50_step(device, level, channels_last=channels_last)
    torch.cuda.empty_cache()
    return out


# ResNet-50's batch-norm inputs: (channels, height = width, how many layers have this shape)
RESNET50_BN_SHAPES = [(64, 112, 1), (64, 56, 6), (256, 56, 4), (128, 56, 1), (128, 28, 7), (512, 28, 5),
                      (256, 28, 1), (256, 14, 11), (1024, 14, 7), (512, 14, 1), (512, 7, 5), (2048, 7, 4)]


def batch_norm_shapes(device, channels_last=True, batch=512, reps=10, keep=()):
    """The three fused batch-norm steps of an L3 training step (statistics + group min/max;
    normalise + 2-bit pack; backward from the packed input with the gradient norm), timed with
    events - the calls queued behind other work, so that the device sets the pace - on every
    batch-norm shape of ResNet-50 in bf16: ms and GB/s of algorithmic bytes per
    shape, and the totals weighted by the number of layers.  `keep`: (C, H) pairs to restrict the run
    to (for counter runs on single shapes)."""
    import actnn_amd.cpp_extension.backward_func as bf
    from actnn_amd.cpp_extension.quantization import attach_bits_total
    from actnn_amd.ops import _Quantized

    worst = []      # slowest run over the median run, per timed call
    # Work that keeps the device busy (about 2 ms) while the timed calls are queued behind it: the
    # passes of the small planes run 10-40 us, less than a call takes to issue from Python, and timed
    # one by one on an idle device they would show the caller's pace.  In the training step the host is
    # ahead of the device (28 ms of host time in a 67 ms step at this batch size) and the passes run
    # back to back, which is what the queue reproduces.
    blocker = torch.zeros(256 << 20, dtype=torch.uint8, device=device)

    def timed(fn, batches=5):
        for _ in range(3):
            fn()
        torch.cuda.synchronize(device)
        # `batches` runs of `reps` calls, each run between two events (an event between every two
        # calls is a barrier packet of its own, several microseconds on passes that last ten); the
        # median run counts and the slowest is reported.  The stalls of tens of milliseconds once seen
        # here were CPython's full garbage collection (40 ms with torch loaded, timed through
        # gc.callbacks; in a kernel trace a gap between two dispatches with no HIP call inside), which
        # started wherever the allocation counters said so: the timed loop collects first and keeps
        # the collector off.
        marks = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(batches)]
        gc.collect()
        gc.disable()
        try:
            for start, stop in marks:
                for _ in range(24):
                    blocker.add_(1)
                start.record()
                for _ in range(reps):
                    fn()
                stop.record()
            torch.cuda.synchronize(device)
        finally:
            gc.enable()
        each = sorted(start.elapsed_time(stop) / reps for start, stop in marks)
        worst.append((each[-1] / each[batches // 2], each[-1]))
        return each[batches // 2]

    rows, totals = [], [0.0, 0.0, 0.0]
    shapes = [sh for sh in RESNET50_BN_SHAPES if not keep or sh[:2] in keep]
    for C, H, count in shapes:
        x = torch.randn(batch, C, H, H, device=device, dtype=torch.bfloat16)
        dy = torch.randn_like(x)
        if channels_last:
            x = x.contiguous(memory_format=torch.channels_last)
            dy = dy.contiguous(memory_format=torch.channels_last)
        w, b = torch.rand(C, device=device) + 0.5, torch.randn(C, device=device)
        n = x.numel()
        bits = attach_bits_total(torch.full((batch,), 2, dtype=torch.int32, device=device), 2 * batch)
        ws, mean, invstd, mn, mx = bf.hip_batch_norm_forward_stats(x, w, b, None, None, 0.1, 1e-5)
        _, packed, scale = bf.hip_batch_norm_forward_apply(x, ws, bits, mn, mx)
        quantized = _Quantized((packed, bits, scale, mn.view(batch, -1, 1)))
        quantized.native_bf16 = True
        quantized.memory_format = torch.channels_last if channels_last else None
        t = [timed(lambda: bf.hip_batch_norm_forward_stats(x, w, b, None, None, 0.1, 1e-5)),
             timed(lambda: bf.hip_batch_norm_forward_apply(x, ws, bits, mn, mx)),
             timed(lambda: bf.hip_batch_norm_backward_packed(x.shape, quantized, dy, w, mean, invstd, sumsq=True))]
        nbytes = [2 * n + 4 * n / 256, 4 * n + n / 4 + 2 * n / 256, 3 * 2 * n + 2 * (n / 4 + 4 * n / 256)]
        rows.append({"shape": [C, H, H], "layers": count, "ms": [round(v, 4) for v in t],
                     "GB/s": [round(nb / v / 1e6) for nb, v in zip(nbytes, t)]})
        for k in range(3):
            totals[k] += count * t[k]
    return {"steps": ["statistics+minmax", "normalise+pack", "backward_from_2bit_stream"], "batch": batch,
            "memory_format": "channels_last" if channels_last else "contiguous", "shapes": rows,
            "ms_per_training_step": [round(v, 3) for v in totals],
            # (three timed calls per shape, in the order of `steps`)
            "slowest_run": {"over_median": round(max(worst)[0], 2), "ms": round(max(worst)[1], 3),
                                   "shape": shapes[worst.index(max(worst)) // 3][:2],
                                   "step": worst.index(max(worst)) % 3}}
