"""Layer-level behaviour on the GPU: the compressed autograd functions against stock torch layers
(the reference checks the same things in tests/test_act_quantized_ops.py:318-447 and
tests/test_linear.py)."""
import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

import actnn_amd
from actnn_amd import QBNScheme, QModule, QScheme, config, set_optimization_level
from actnn_amd.ops import dequantize_activation, quantize_saved
from actnn_amd.resnet import resnet50
from _util import DEV

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def fresh_config():
    config.reset()
    QScheme.reset()
    QBNScheme.reset()
    yield
    config.reset()
    QScheme.reset()
    QBNScheme.reset()


def _grads(layer, x, g):
    x = x.clone().requires_grad_(True)
    y = layer(x)
    y.backward(g)
    return y.detach(), x.grad, [p.grad.clone() for p in layer.parameters()]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_conv2d_8bit_close_to_exact(dtype):
    # per-group 8-bit quantisation of the saved input: gradients within the reference's 8-bit
    # tolerance of the exact ones (tests/test_act_quantized_ops.py:403-447 uses 1e-1)
    config.activation_compression_bits = [8]
    config.initial_bits = 8
    config.perlayer = False
    torch.manual_seed(0)
    N, Cc, H, W = 4, 256, 28, 28
    q = actnn_amd.QConv2d(Cc, 64, 3, padding=1).to(DEV).to(dtype)
    ref = nn.Conv2d(Cc, 64, 3, padding=1).to(DEV).to(dtype)
    ref.load_state_dict(q.state_dict())
    x = torch.randn(N, Cc, H, W, device=DEV, dtype=dtype)
    g = torch.randn(N, 64, H, W, device=DEV, dtype=dtype)
    yq, gxq, gpq = _grads(q, x, g)
    yr, gxr, gpr = _grads(ref, x, g)
    # forward is the stock convolution (MIOpen may pick a different algorithm per call)
    assert torch.allclose(yq.float(), yr.float(), atol=2e-3 if dtype == torch.float32 else 2e-2, rtol=1e-2)
    tol = 1e-1
    assert torch.allclose(gxq.float(), gxr.float(), atol=tol, rtol=tol)
    for a, b in zip(gpq, gpr):
        rel = (a.float() - b.float()).norm() / b.float().norm()
        assert rel < 2e-2


def test_simulate_and_kernel_paths_agree_statistically():
    # config.simulate vs the kernels on the same layer (reference: tests/test_act_quantized_ops.py:360-400)
    config.activation_compression_bits = [8]
    config.initial_bits = 8
    config.perlayer = False
    torch.manual_seed(0)
    q = actnn_amd.QConv2d(64, 32, 3, padding=1).to(DEV)
    x = torch.randn(4, 64, 28, 28, device=DEV)
    g = torch.randn(4, 32, 28, 28, device=DEV)
    res = []
    for sim in (True, False):
        config.simulate = sim
        q.zero_grad()
        res.append(_grads(q, x, g))
    (y0, gx0, gp0), (y1, gx1, gp1) = res
    assert torch.allclose(y0, y1, atol=2e-3) and torch.allclose(gx0, gx1, atol=2e-3)
    for a, b in zip(gp0, gp1):
        assert (a - b).norm() / b.norm() < 2e-2


def test_quantize_dequantize_glue_shapes_and_padding():
    # 300 features per sample -> padded to 512 (2 groups), un-padded on the way back; fp32 keeps
    # scale/min as bf16 (ops.py:115-116)
    set_optimization_level("L2")
    x = torch.randn(6, 3, 10, 10, device=DEV)
    qd = quantize_saved(x, None)
    q_input, q_bits, q_scale, q_min = qd
    assert q_bits == 4 and q_input.dtype == torch.int8
    assert q_scale.dtype == torch.bfloat16 and q_scale.shape == (6, 2, 1)
    back = dequantize_activation(qd, x.shape)
    assert back.shape == x.shape and back.dtype == torch.float32 and back.is_contiguous()
    rng = (x.view(6, -1).max(1)[0] - x.view(6, -1).min(1)[0]).max()
    assert (back - x).abs().max() < rng / 15 * 1.1 + 0.05      # one 4-bit step (+ bf16 scale/min rounding)


def test_batch_norm_without_compression_matches_torch():
    config.compress_activation = False
    torch.manual_seed(0)
    q = actnn_amd.QBatchNorm2d(16).to(DEV)
    ref = nn.BatchNorm2d(16).to(DEV)
    x = torch.randn(8, 16, 14, 14, device=DEV)
    g = torch.randn_like(x)
    yq, gxq, gpq = _grads(q, x, g)
    yr, gxr, gpr = _grads(ref, x, g)
    assert torch.allclose(yq, yr, atol=1e-3) and torch.allclose(gxq, gxr, atol=1e-3)
    for a, b in zip(gpq, gpr):
        assert torch.allclose(a, b, atol=1e-3, rtol=1e-3)
    assert torch.allclose(q.running_mean, ref.running_mean, atol=1e-5)
    assert torch.allclose(q.running_var, ref.running_var, atol=1e-5)


def test_linear_without_compression_matches_torch():
    config.compress_activation = False
    torch.manual_seed(0)
    q = actnn_amd.QLinear(100, 10).to(DEV)
    ref = nn.Linear(100, 10).to(DEV)
    ref.load_state_dict(q.state_dict())
    x = torch.randn(32, 100, device=DEV)
    g = torch.randn(32, 10, device=DEV)
    yq, gxq, gpq = _grads(q, x, g)
    yr, gxr, gpr = _grads(ref, x, g)
    assert torch.allclose(yq, yr, atol=1e-5) and torch.allclose(gxq, gxr, atol=1e-5)
    for a, b in zip(gpq, gpr):
        assert torch.allclose(a, b, atol=1e-4, rtol=1e-4)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_qlinear_fused_weight_gradient_path(dtype):
    # fixed 2-bit width (no adaptive scheme): linear.backward takes the fused GEMM; the result must
    # agree with the unfused path (unpack + mm) run on the same packed input
    config.activation_compression_bits = [2]
    config.adaptive_conv_scheme = False
    torch.manual_seed(0)
    q = actnn_amd.QLinear(512, 264).to(DEV).to(dtype)
    x = torch.randn(64, 512, device=DEV, dtype=dtype)
    g = torch.randn(64, 264, device=DEV, dtype=dtype)
    from actnn_amd import ops
    torch.cuda.manual_seed(7)
    _, gx_f, gp_f = _grads(q, x, g)
    q.zero_grad()
    saved = ops._fused_grad_weight_ok
    ops._fused_grad_weight_ok = lambda *a: False
    try:
        torch.cuda.manual_seed(7)                 # same Philox stream -> same packed input
        _, gx_u, gp_u = _grads(q, x, g)
    finally:
        ops._fused_grad_weight_ok = saved
    assert torch.equal(gx_f, gx_u)
    assert (gp_f[0].float() - gp_u[0].float()).norm() / gp_u[0].float().norm() < 1e-2
    assert torch.equal(gp_f[1], gp_u[1])


@pytest.mark.parametrize("level,bits,mode,stream", [("L2", 2, True, int), ("L2", 4, True, None), ("L3", 2, True, None),
                                                     ("L2", 4, "always", int), ("L3", 2, "always", torch.Tensor)])
def test_qlinear_takes_the_fused_gemm_where_it_is_the_faster_path(level, bits, mode, stream, monkeypatch):
    # under bf16 autocast a QLinear's weight gradient comes from the fused kernel when its input was
    # saved as the 2-bit fixed-width stream; the 4-bit stream of L1 / L2 and the per-sample stream
    # of L3 take unpack + mm unless config.fused_linear_grad_weight == "always".  Where the fused
    # kernel runs, its result agrees with the unfused path on the same packed input
    import actnn_amd.cpp_extension.quantization as ext_q
    set_optimization_level(level)
    config.activation_compression_bits = [bits] + config.activation_compression_bits[1:]
    config.fused_linear_grad_weight = mode
    torch.manual_seed(0)
    q = actnn_amd.QLinear(2048, 1000).to(DEV)
    x = torch.randn(128, 2048, device=DEV)
    calls = []
    fused = ext_q.linear_grad_weight
    monkeypatch.setattr(ext_q, "linear_grad_weight", lambda *a: calls.append(type(a[2])) or fused(*a))

    def step():
        q.zero_grad()
        with torch.autocast("cuda", dtype=torch.bfloat16):
            y = q(x.clone().requires_grad_(True))
        y.float().square().mean().backward()
        return q.weight.grad.clone()
    step()                                          # first step: degenerate widths at L3
    torch.cuda.manual_seed(5)
    gw_fused = step()
    if stream is None:
        assert calls == []
        return
    assert len(calls) == 2 and calls[0] is stream
    config.fused_linear_grad_weight = False
    torch.cuda.manual_seed(5)
    gw_unfused = step()
    assert len(calls) == 2
    assert (gw_fused - gw_unfused).norm() / gw_unfused.norm() < 1e-2


def test_l3_first_step_uses_the_degenerate_allocation_then_rebalances():
    # gradient scale starts at 0 (qscheme.py:24): the first forward gives 8 bits to the first
    # samples and 1 to the rest; after one backward the scale is positive and bits follow C
    torch.manual_seed(0)
    model = QModule(nn.Sequential(nn.Conv2d(8, 8, 3, padding=1), nn.BatchNorm2d(8), nn.ReLU(),
                                  nn.Conv2d(8, 8, 3, padding=1))).to(DEV)
    x = torch.randn(16, 8, 16, 16, device=DEV)
    model(x).square().mean().backward()
    s0 = QScheme.layers[0]
    assert s0.b.tolist() == [8, 8, 3] + [1] * 13            # target 32 = 8 + 8 + 3 + 13
    assert float(s0.scales) > 0
    budgets = [float(s.bits) for s in QScheme.layers]         # set by the per-layer re-balancing
    assert abs(sum(budgets) / 2 - 2.0) < 0.26                 # both layers have the same size
    model(x)
    assert int(s0.b.sum()) <= int(budgets[0] * 16) and int(s0.b.min()) >= 1


@pytest.mark.parametrize("one_call", [False, True])
def test_sensitivities_reach_the_host_in_one_transfer_per_step(one_call):
    """The widths are made on the device; the sensitivities of all layers travel in one pool.  What
    the host reads per layer equals what the layer's own kernel computes from its input's ranges,
    one step after another, and a change of the batch size makes a new pool - whether the layer's
    sequence goes through one library call or step by step."""
    from actnn_amd import qscheme
    from actnn_amd.cpp_extension import minimax as ext_minimax, quantization as ext_q
    config.fused_quantize = one_call
    torch.manual_seed(0)
    model = QModule(nn.Sequential(nn.Conv2d(8, 8, 3, padding=1), nn.ReLU(), nn.Conv2d(8, 8, 3, padding=1),
                                  nn.ReLU(), nn.Conv2d(8, 4, 1))).to(DEV)
    seen = []
    start, call = QScheme.start_quantization_bits, ext_q.quantize_activation_device

    def spy_start(self, input, known_minmax=None):
        groups, mn, mx, num_pixels = qscheme.group_min_max(input, known_minmax)
        seen.append((self, self.sensitivity(mn, mx, input.shape[0], num_pixels).clone()))
        return start(self, input, known_minmax)

    def spy_call(rows, N, known_minmax, alloc):
        mn, mx = ext_minimax.minimax(rows)
        seen.append((QScheme.layers[alloc.pending.index], ext_minimax.range_sqr(mn, mx, N, alloc.factor, alloc.mult)))
        return call(rows, N, known_minmax, alloc)

    QScheme.start_quantization_bits, ext_q.quantize_activation_device = spy_start, spy_call
    try:
        for step, n in enumerate((16, 16, 8)):
            seen.clear()
            x = torch.randn(n, 8, 16, 16, device=DEV)
            model(x).square().mean().backward()
            pool = QScheme.sensitivity_pool
            assert pool is not None and pool.dev.shape == (3, n) and not pool.dirty
            assert len(seen) == 3
            for scheme, expected in seen:
                assert scheme.C.shape == (n,)
                assert torch.equal(scheme.C, expected.cpu()), (step, scheme.name)
    finally:
        QScheme.start_quantization_bits, ext_q.quantize_activation_device = start, call


@pytest.mark.parametrize("channels_last", [False, True])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_one_library_call_per_layer_equals_the_step_by_step_sequence(channels_last, dtype):
    """config.fused_quantize puts min/max (or the batch-norm statistics), the widths and the pack of a
    layer behind one library call.  Same kernels on the same generator state: outputs, gradients,
    widths and sensitivities of three training steps (per-layer re-balancing included) are those
    of the step-by-step sequence bit for bit."""
    from actnn_amd.cpp_extension import backward_func as bf, quantization as q

    from actnn_amd import ops
    plain_tuple = ops._Quantized

    def run(fused):
        config.reset(); QScheme.reset(); QBNScheme.reset()
        set_optimization_level("L3")
        config.fused_quantize = fused
        torch.manual_seed(0)
        model = QModule(nn.Sequential(nn.Conv2d(8, 16, 3, padding=1), nn.BatchNorm2d(16), nn.ReLU(),
                                      nn.Conv2d(16, 16, 3, padding=1), nn.BatchNorm2d(16), nn.ReLU(),
                                      nn.Conv2d(16, 8, 1))).to(DEV)
        if channels_last:
            model = model.to(memory_format=torch.channels_last)
        torch.cuda.manual_seed(77)
        calls = {"bn": 0, "conv": 0}
        saved = []
        real_bn, real_conv = bf.hip_batch_norm_forward_quantize, q.quantize_activation_device

        def count_bn(*a, **k):
            calls["bn"] += 1
            return real_bn(*a, **k)

        def count_conv(*a, **k):
            calls["conv"] += 1
            return real_conv(*a, **k)

        class Recorded(plain_tuple):                      # every tuple a layer saves for its backward
            def __new__(cls, items):
                self = plain_tuple.__new__(cls, items)
                saved.append(self)
                return self

        bf.hip_batch_norm_forward_quantize, q.quantize_activation_device = count_bn, count_conv
        ops._Quantized = Recorded
        out = []
        try:
            # (the weights stay as they are: MIOpen's weight-gradient kernels add with atomics, and
            # what is compared here must not depend on their order)
            for step in range(3):
                g = torch.Generator(device=DEV).manual_seed(step)
                x = torch.randn(16, 8, 16, 16, device=DEV, generator=g)
                if channels_last:
                    x = x.contiguous(memory_format=torch.channels_last)
                model.zero_grad()
                del saved[:]
                with torch.autocast("cuda", dtype=torch.bfloat16, enabled=dtype == torch.bfloat16):
                    y = model(x)
                assert len(saved) == 5
                kept = [t.clone() for tup in saved for t in tup] + \
                       [torch.as_tensor([tup.native_bf16, tup.memory_format is not None]) for tup in saved]
                y.float().square().mean().backward()
                out.append([y.detach().clone()] + kept + [p.grad.clone() for p in model.parameters() if p.dim() == 1]
                           + [l.b.clone() for l in QScheme.layers] + [l.C.clone() for l in QScheme.layers]
                           + [torch.as_tensor(float(l.bits)) for l in QScheme.layers + QBNScheme.layers])
        finally:
            bf.hip_batch_norm_forward_quantize, q.quantize_activation_device = real_bn, real_conv
            ops._Quantized = plain_tuple
        return out, calls

    (slow, slow_calls), (fast, fast_calls) = run(False), run(True)
    assert slow_calls == {"bn": 0, "conv": 0}
    assert fast_calls == {"bn": 6, "conv": 9}            # every batch norm and every convolution, every step
    for step, (a, b) in enumerate(zip(slow, fast)):
        assert len(a) == len(b)
        for i, (u, v) in enumerate(zip(a, b)):
            assert torch.equal(u.cpu(), v.cpu()), (step, i)


@pytest.mark.parametrize("channels_last", [False, True])
def test_small_model_trains_at_l3(channels_last):
    # the same toy problem with stock layers and with 2-bit compressed activations: the loss
    # curves must track each other (the quantisation noise is unbiased), in both memory layouts
    def make():
        torch.manual_seed(0)
        return nn.Sequential(nn.Conv2d(3, 16, 3, padding=1), nn.BatchNorm2d(16), nn.ReLU(), nn.MaxPool2d(2),
                             nn.Conv2d(16, 32, 3, padding=1), nn.BatchNorm2d(32), nn.ReLU(),
                             nn.AdaptiveAvgPool2d(1), nn.Flatten(), nn.Linear(32, 10))
    torch.manual_seed(1)
    y = torch.randint(0, 10, (64,), device=DEV)
    pattern = torch.randn(10, 3, 32, 32, device=DEV)
    x = torch.randn(64, 3, 32, 32, device=DEV) + pattern[y]

    if channels_last:
        x = x.contiguous(memory_format=torch.channels_last)

    def run(model):
        model = model.to(DEV)
        if channels_last:
            model = model.to(memory_format=torch.channels_last)
        opt = torch.optim.SGD(model.parameters(), lr=0.05, momentum=0.9)
        losses = []
        for _ in range(40):
            opt.zero_grad()
            loss = F.cross_entropy(model(x), y)
            loss.backward()
            opt.step()
            losses.append(loss.item())
        return losses

    exact = make()
    quant = QModule(make())
    quant.load_state_dict(exact.state_dict())
    le, lq = run(exact), run(quant)
    assert lq[-1] < lq[0] - 0.1
    assert abs(lq[-1] - le[-1]) < 0.05 and max(abs(a - b) for a, b in zip(le, lq)) < 0.1


@pytest.mark.parametrize("channels_last", [False, True])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_converted_add_relu_is_the_addition_followed_by_relu(channels_last, dtype):
    """QModule swaps AddReLU for the fused layer: output and both gradients are those of the
    unfused modules, in either memory layout; a 16-bit output of whole 2048-element tiles carries the
    group min / max for the convolution that compresses it next."""
    from actnn_amd import AddReLU, QAddReLU
    from actnn_amd.layers import known_group_minmax

    class Block(nn.Module):
        def __init__(self):
            super().__init__()
            self.close = AddReLU()

        def forward(self, a, b):
            return self.close(a, b)

    torch.manual_seed(5)
    a = torch.randn(8, 32, 8, 8, device=DEV).to(dtype)
    b = torch.randn(8, 32, 8, 8, device=DEV).to(dtype)
    b[:, ::2] = -a[:, ::2]
    if channels_last:
        a, b = (t.contiguous(memory_format=torch.channels_last) for t in (a, b))
    g = torch.randn_like(a)
    plain, fused = Block(), QModule(Block())
    assert isinstance(fused.model.close, QAddReLU)
    outs = []
    for model in (plain, fused):
        a1, b1 = a.clone().requires_grad_(True), b.clone().requires_grad_(True)
        out = model(a1, b1)
        out.backward(g)
        outs.append((out.detach(), a1.grad, b1.grad, out))
    for u, v in zip(outs[0][:3], outs[1][:3]):
        assert torch.equal(u, v)
    assert outs[1][0].is_contiguous(memory_format=torch.channels_last if channels_last else torch.contiguous_format)
    known = known_group_minmax(outs[1][3])
    if dtype == torch.bfloat16:
        from actnn_amd.utils import memory_order
        groups = memory_order(outs[1][0]).reshape(-1, 256)
        assert known is not None
        assert torch.equal(known[0], groups.min(1).values) and torch.equal(known[1], groups.max(1).values)
    else:
        assert known is None
    # operands that do not share a layout take the unfused path, with the same result
    if channels_last:
        a1 = a.contiguous().requires_grad_(True)
        out = fused(a1, b)
        assert torch.equal(out, outs[0][0])


@pytest.mark.parametrize("autocast", [False, True])
def test_resnet50_step_runs(autocast):
    torch.manual_seed(0)
    model = QModule(resnet50()).to(DEV)
    x = torch.randn(8, 3, 64, 64, device=DEV)
    y = torch.randint(0, 1000, (8,), device=DEV)
    for _ in range(2):
        model.zero_grad()
        with torch.autocast("cuda", dtype=torch.bfloat16, enabled=autocast):
            loss = F.cross_entropy(model(x), y)
        loss.backward()
    assert torch.isfinite(loss)
    grads = [p.grad for p in model.parameters()]
    assert all(g is not None and torch.isfinite(g).all() for g in grads)
    assert all(g.dtype == torch.float32 for g in grads)


def test_activation_memory_shrinks():
    # saved-for-backward bytes of one conv+bn+relu stage: L3 (2 bits) vs L0 (masks only)
    def saved_bytes(level):
        config.reset(); QScheme.reset(); QBNScheme.reset()
        set_optimization_level(level)
        torch.manual_seed(0)
        model = QModule(nn.Sequential(nn.Conv2d(64, 64, 3, padding=1), nn.BatchNorm2d(64), nn.ReLU(),
                                      nn.Conv2d(64, 64, 3, padding=1))).to(DEV)
        x = torch.randn(32, 64, 56, 56, device=DEV)
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated()
        out = model(x)
        torch.cuda.synchronize()
        held = torch.cuda.memory_allocated() - before - out.numel() * 4
        out.sum().backward()
        return held
    full, packed = saved_bytes("L0"), saved_bytes("L3")
    assert packed < full / 6


def _cl(model):
    return model.to(DEV).to(memory_format=torch.channels_last)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_channels_last_block_8bit_close_to_exact_and_stays_channels_last(dtype):
    """A channels-last model is compressed in memory order (no transposes): with 8 bits the
    gradients of conv + BN + ReLU + max-pool + conv match the exact ones as in the default layout,
    and activations and gradients keep the channels-last strides throughout."""
    config.activation_compression_bits = [8]
    config.initial_bits = 8
    config.perlayer = False

    def make():
        torch.manual_seed(0)
        return nn.Sequential(nn.Conv2d(16, 32, 3, padding=1, bias=False), nn.BatchNorm2d(32), nn.ReLU(),
                             nn.MaxPool2d(3, 2, 1), nn.Conv2d(32, 64, 3, padding=1, bias=False),
                             nn.BatchNorm2d(64), nn.ReLU(), nn.Dropout(0.0))
    exact = _cl(make()).to(dtype)
    quant = _cl(QModule(make())).to(dtype)
    quant.load_state_dict(exact.state_dict())
    x = torch.randn(8, 16, 32, 32, device=DEV, dtype=dtype).contiguous(memory_format=torch.channels_last)
    g = torch.randn(8, 64, 16, 16, device=DEV, dtype=dtype).contiguous(memory_format=torch.channels_last)
    res = []
    for model in (exact, quant):
        xi = x.clone(memory_format=torch.preserve_format).requires_grad_(True)
        y = model(xi)
        assert y.is_contiguous(memory_format=torch.channels_last)
        y.backward(g)
        assert xi.grad.is_contiguous(memory_format=torch.channels_last)
        res.append((y.detach().float(), xi.grad.float(), [p.grad.float() for p in model.parameters()]))
    (ye, gxe, gpe), (yq, gxq, gpq) = res
    tol = 2e-3 if dtype == torch.float32 else 6e-2
    assert torch.allclose(yq, ye, atol=tol, rtol=tol)
    assert (gxq - gxe).norm() / gxe.norm() < 3e-2
    for a, b in zip(gpq, gpe):
        assert (a - b).norm() / (b.norm() + 1e-6) < 3e-2


def test_channels_last_saved_activation_round_trip():
    """quantize_saved / dequantize_activation on a channels-last tensor: groups follow memory
    order, the rebuilt tensor has the logical shape, channels-last strides and 8-bit accuracy;
    the packed stream equals the one of the same memory seen as a default-layout tensor."""
    config.activation_compression_bits = [8]
    torch.manual_seed(0)
    x = torch.randn(4, 64, 12, 8, device=DEV).contiguous(memory_format=torch.channels_last)
    torch.cuda.manual_seed(3)
    q = quantize_saved(x, None)
    assert q.memory_format == torch.channels_last
    back = dequantize_activation(q, x.shape)
    assert back.shape == x.shape and back.is_contiguous(memory_format=torch.channels_last)
    # one 8-bit step, plus the bfloat16 rounding of the stored scale / minimum of an fp32 activation
    assert (back - x).abs().max() < (x.max() - x.min()) / 255 + 2.0 ** -6 * x.abs().max()
    torch.cuda.manual_seed(3)
    q2 = quantize_saved(x.permute(0, 2, 3, 1).contiguous(), None)       # same memory, default layout
    # (the fixed-width stream ends in one spare byte that no kernel writes, .cu:268)
    assert torch.equal(q[0][:-1], q2[0][:-1]) and torch.equal(q[2], q2[2])


def test_resnet50_channels_last_step_runs():
    torch.manual_seed(0)
    model = _cl(QModule(resnet50()))
    x = torch.randn(8, 3, 64, 64, device=DEV).contiguous(memory_format=torch.channels_last)
    y = torch.randint(0, 1000, (8,), device=DEV)
    for _ in range(2):
        model.zero_grad()
        with torch.autocast("cuda", dtype=torch.bfloat16):
            loss = F.cross_entropy(model(x), y)
        loss.backward()
    assert torch.isfinite(loss)
    assert all(p.grad is not None and torch.isfinite(p.grad).all() for p in model.parameters())


@pytest.mark.parametrize("dims", [1, 2, 3])
def test_conv_transpose_8bit_close_to_exact(dims):
    """QConvTranspose1d/2d/3d (layers.py:101-191 of the reference): forward is the stock operator,
    gradients from the 8-bit saved input are within the reference's 8-bit tolerance of the exact
    ones; QModule converts the stock layers."""
    config.activation_compression_bits = [8]
    config.initial_bits = 8
    config.perlayer = False
    torch.manual_seed(dims)
    stock = {1: nn.ConvTranspose1d, 2: nn.ConvTranspose2d, 3: nn.ConvTranspose3d}[dims]
    quant = {1: actnn_amd.QConvTranspose1d, 2: actnn_amd.QConvTranspose2d, 3: actnn_amd.QConvTranspose3d}[dims]
    spatial = {1: (64,), 2: (16, 16), 3: (4, 8, 8)}[dims]
    ref = stock(32, 16, 3, stride=2, padding=1, output_padding=1).to(DEV)
    q = quant(32, 16, 3, stride=2, padding=1, output_padding=1).to(DEV)
    q.load_state_dict(ref.state_dict())
    wrapped = QModule(nn.Sequential(stock(32, 16, 3, stride=2, padding=1, output_padding=1)))
    assert isinstance(wrapped.model[0], quant)
    x = torch.randn(4, 32, *spatial, device=DEV)
    g = torch.randn(4, 16, *[2 * s for s in spatial], device=DEV)
    yq, gxq, gpq = _grads(q, x, g)
    yr, gxr, gpr = _grads(ref, x, g)
    assert torch.allclose(yq, yr, atol=2e-3, rtol=1e-2)
    assert torch.allclose(gxq, gxr, atol=1e-1, rtol=1e-1)
    for a, b in zip(gpq, gpr):
        assert (a - b).norm() / b.norm() < 2e-2


@pytest.mark.parametrize("channels_last", [False, True])
def test_batch_norm_fused_and_unfused_paths_save_the_same_stream(channels_last):
    """QBatchNorm2d at L3: the fused sequence (statistics + min/max, allocation, normalise + pack;
    backward from the stream) and the reference's sequence (minimax, pack, library batch norm;
    unpack + backward) save bit-identical tuples for the same generator state, with the widths
    allocated on the device or on the host, and give matching outputs and gradients."""
    def run(fused, device_allocation):
        config.reset(); QScheme.reset(); QBNScheme.reset()
        config.fused_bn_pack = config.fused_bn_backward = fused
        config.device_allocation = device_allocation
        config.perlayer = False
        torch.manual_seed(0)
        conv = actnn_amd.QConv2d(16, 64, 3, padding=1).to(DEV)        # gives the BN scheme its predecessor
        bn = actnn_amd.QBatchNorm2d(64).to(DEV)
        x = torch.randn(24, 16, 16, 16, device=DEV)
        if channels_last:
            conv, bn = conv.to(memory_format=torch.channels_last), bn.to(memory_format=torch.channels_last)
            x = x.contiguous(memory_format=torch.channels_last)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            h = conv(x)
            torch.cuda.manual_seed(11)
            y = bn(h)
        saved = y.grad_fn.saved[0]
        g = torch.randn_like(y)
        gh, gw = torch.autograd.grad(y, [h, bn.weight], g)        # the saved tuple is released by backward
        return y, saved, gh, gw
    ref = run(False, False)
    for fused, dev_alloc in ((True, True), (True, False), (False, True)):
        y, saved, gh, gw = run(fused, dev_alloc)
        assert torch.equal(saved[1].cpu(), ref[1][1].cpu())                       # widths
        assert torch.equal(saved[0], ref[1][0]) and torch.equal(saved[2], ref[1][2]) and torch.equal(saved[3], ref[1][3])
        assert torch.allclose(y.float(), ref[0].float(), atol=2e-2, rtol=2e-2)
        assert torch.allclose(gh.float(), ref[2].float(), atol=3e-2, rtol=3e-2)
        assert torch.allclose(gw, ref[3], rtol=2e-2, atol=2e-1)


def test_batch_norm_1d_on_rows_takes_the_fused_passes():
    """QBatchNorm1d on [N, C] inputs (layers.py:270-310 serves them through the same Function): the
    fused sequence - statistics + group min/max, allocation, normalise + pack, backward from the
    stream - runs on the library's kernels and saves the same tuple as the reference's sequence;
    a width that is not a whole number of groups takes minimax + pack and the plain kernels."""
    import actnn_amd.cpp_extension.backward_func as ext_bf

    def run(fused, C):
        config.reset(); QScheme.reset(); QBNScheme.reset()
        config.fused_bn_pack = config.fused_bn_backward = fused
        config.perlayer = False
        torch.manual_seed(0)
        lin = actnn_amd.QLinear(64, C).to(DEV)
        bn = actnn_amd.QBatchNorm1d(C).to(DEV)
        x = torch.randn(96, 64, device=DEV)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            h = lin(x)
            torch.cuda.manual_seed(11)
            y = bn(h)
        saved = y.grad_fn.saved[0]
        g = torch.randn_like(y)
        gh, gw = torch.autograd.grad(y, [h, bn.weight], g)
        return y, saved, gh, gw, h
    for C in (512, 104):
        ref = run(False, C)
        y, saved, gh, gw, h = run(True, C)
        assert ext_bf.hip_batch_norm_applies(h, None, None, None, None)
        assert ext_bf.hip_batch_norm_minmax_applies(h, None, None, None, None) == (C % 256 == 0)
        assert torch.equal(saved[1].cpu(), ref[1][1].cpu())
        assert torch.equal(saved[0], ref[1][0]) and torch.equal(saved[2], ref[1][2]) and torch.equal(saved[3], ref[1][3])
        assert torch.allclose(y.float(), ref[0].float(), atol=2e-2, rtol=2e-2)
        assert torch.allclose(gh.float(), ref[2].float(), atol=3e-2, rtol=3e-2)
        assert torch.allclose(gw, ref[3], rtol=2e-2, atol=2e-1)
        exact = torch.nn.functional.batch_norm(h.float(), None, None, None, None, True, 0.1, 1e-5)
        assert torch.allclose(y.float(), exact * 1.0, atol=3e-2, rtol=3e-2)


@pytest.mark.parametrize("channels_last", [False, True])
@pytest.mark.parametrize("level", ["L0", "L1", "L2", "L3", "L3.1", "L4", "swap"])
def test_every_optimization_level_trains_a_step(level, channels_last):
    """All levels of set_optimization_level (conf.py:5-36) run two training steps of a small
    conv / BN / ReLU / max-pool / dropout / linear model in both memory layouts, with finite
    gradients close to the exact model's at the levels that keep 4 bits or more."""
    def make():
        torch.manual_seed(0)
        return nn.Sequential(nn.Conv2d(8, 32, 3, padding=1, bias=False), nn.BatchNorm2d(32), nn.ReLU(),
                             nn.MaxPool2d(3, 2, 1), nn.Conv2d(32, 64, 1), nn.BatchNorm2d(64), nn.ReLU(),
                             nn.Dropout(0.0), nn.AdaptiveAvgPool2d(1), nn.Flatten(), nn.Linear(64, 10))
    set_optimization_level(level)
    if level == "L3.1":
        config.pipeline_threshold = 1 << 16                 # force the micro-batched conv backward
    exact = make().to(DEV)
    quant = QModule(make()).to(DEV)
    quant.load_state_dict(exact.state_dict())
    x = torch.randn(16, 8, 32, 32, device=DEV)
    if channels_last:
        exact, quant = exact.to(memory_format=torch.channels_last), quant.to(memory_format=torch.channels_last)
        x = x.contiguous(memory_format=torch.channels_last)
    y = torch.randint(0, 10, (16,), device=DEV)
    for model in (exact, quant):
        for _ in range(2):
            model.zero_grad()
            F.cross_entropy(model(x), y).backward()
    for (name, p), q in zip(exact.named_parameters(), quant.parameters()):
        assert q.grad is not None and torch.isfinite(q.grad).all(), name
        if level in ("L0", "L1", "L2", "swap"):
            assert (q.grad - p.grad).norm() <= 0.25 * p.grad.norm() + 1e-3, name


def test_qmodule_channels_last_option():
    torch.manual_seed(0)
    net = nn.Sequential(nn.Conv2d(8, 32, 3, padding=1), nn.BatchNorm2d(32), nn.ReLU(), nn.Conv2d(32, 16, 1))
    model = QModule(net, channels_last=True).to(DEV)
    assert all(p.is_contiguous(memory_format=torch.channels_last) for p in model.parameters() if p.dim() == 4)
    x = torch.randn(4, 8, 16, 16, device=DEV, requires_grad=True)          # default-layout input
    y = model(x)
    assert y.is_contiguous(memory_format=torch.channels_last)
    y.sum().backward()
    assert x.grad.shape == x.shape and torch.isfinite(x.grad).all()


def test_swap_space_round_trip_and_prefetch():
    """Tensors parked on the host come back bit-identical in last-in first-out order (the order of
    the backward pass), whether they were transferred ahead of time or on demand."""
    from actnn_amd.utils import swap_space, swap_to_cpu, swap_to_device
    swap_space.reset()
    g = torch.Generator(device=DEV).manual_seed(0)
    originals = [torch.randint(-2 ** 31, 2 ** 31 - 1, (1 << (12 + i % 5),), generator=g, device=DEV, dtype=torch.int64).int()
                 for i in range(12)]
    hosts = [swap_to_cpu(t) for t in originals]
    assert all(h.device.type == "cpu" and h.is_pinned() for h in hosts)
    for k in range(11, -1, -1):
        back = swap_to_device(hosts[k])
        assert back.is_cuda and torch.equal(back, originals[k])
        if k >= 1:
            assert hosts[k - 1]._actnn_swap["ahead"] is not None          # already on its way
    assert swap_space.parked == []
    # on demand, out of order
    hosts = [swap_to_cpu(t) for t in originals[:4]]
    for k in (2, 0, 3, 1):
        assert torch.equal(swap_to_device(hosts[k]), originals[k])


@pytest.mark.parametrize("channels_last", [False, True])
def test_relu_hands_group_min_max_to_the_next_convolution(channels_last):
    """QReLU -> QConv2d: with the hand-off the convolution saves the same stream, widths, scales
    and minima as when it reduces its input itself; a tensor changed in place after the ReLU, or a
    cast one, is not trusted."""
    from actnn_amd.layers import known_group_minmax
    def run(share):
        config.reset(); QScheme.reset(); QBNScheme.reset()
        config.share_relu_min_max = share
        config.perlayer = False
        torch.manual_seed(0)
        relu, conv = actnn_amd.QReLU(), actnn_amd.QConv2d(64, 32, 3, padding=1).to(DEV)
        x = torch.randn(16, 64, 16, 16, device=DEV).bfloat16()
        if channels_last:
            conv = conv.to(memory_format=torch.channels_last)
            x = x.contiguous(memory_format=torch.channels_last)
        x.requires_grad_(True)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            h = relu(x)
            assert (known_group_minmax(h) is not None) == share
            torch.cuda.manual_seed(4)
            y = conv(h)
        saved = y.grad_fn.saved[0]
        (gx,) = torch.autograd.grad(y, x, torch.ones_like(y))
        return h, saved, gx
    h0, s0, g0 = run(False)
    h1, s1, g1 = run(True)
    assert torch.equal(h0, h1)
    assert all(torch.equal(a, b) for a, b in zip(s0, s1))
    # the gradient passes through MIOpen's backward-data kernel, which may add in no fixed order
    # before rounding to bf16: one rounding step of slack
    a, b = g0.float(), g1.float()
    assert ((a - b).abs() <= 2.0 ** -7 * torch.maximum(a.abs(), b.abs()) + 1e-3 * a.abs().max()).all()
    h1.add_(1.0)
    assert known_group_minmax(h1) is None                    # changed in place: the version moved on
    assert known_group_minmax(h0.float()) is None


@pytest.mark.parametrize("channels_last", [False, True])
def test_batch_norm_backward_hands_the_gradient_norm_to_the_convolution(channels_last):
    """QConv2d -> QBatchNorm2d: the convolution's running gradient statistic (qscheme.py:47-55) is
    the same whether batch-norm backward leaves sum(dx^2) or the convolution reduces its incoming
    gradient itself (fp32 sums in different orders: rtol 1e-5), and the gradients agree."""
    def run(share):
        config.reset(); QScheme.reset(); QBNScheme.reset()
        config.share_grad_sqnorm = share
        config.perlayer = False
        torch.manual_seed(0)
        conv = actnn_amd.QConv2d(16, 64, 3, padding=1, bias=False).to(DEV)
        bn = actnn_amd.QBatchNorm2d(64).to(DEV)
        x = torch.randn(16, 16, 16, 16, device=DEV).bfloat16()
        if channels_last:
            conv, bn = conv.to(memory_format=torch.channels_last), bn.to(memory_format=torch.channels_last)
            x = x.contiguous(memory_format=torch.channels_last)
        x.requires_grad_(True)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            torch.cuda.manual_seed(4)
            y = bn(conv(x))
        g = torch.randn_like(y)
        grads = torch.autograd.grad(y, [x, conv.weight, bn.weight], g)
        return conv.scheme.scales, grads
    s0, g0 = run(False)
    s1, g1 = run(True)
    assert torch.equal(g0[2], g1[2])                # batch norm's own weight gradient: same kernels, same bits
    for a, b in zip(g0[:2], g1[:2]):                # through MIOpen's convolution backward, whose split-K
        a, b = a.float(), b.float()                 # kernels add in no fixed order before the result is
        bound = 2.0 ** -7 * torch.maximum(a.abs(), b.abs()) + 1e-3 * a.abs().max()    # rounded to bf16
        assert ((a - b).abs() <= bound).all()
    s0, s1 = float(s0), float(s1)
    assert s0 > 0 and abs(s0 - s1) <= 1e-5 * s0
    # the statistic really came from the hand-off: without the attribute set_scale reduces itself
    import actnn_amd.cpp_extension.backward_func as ext_bf
    seen = []
    original = ext_bf.known_sumsq
    ext_bf.known_sumsq = lambda grad: seen.append(original(grad)) or seen[-1]
    try:
        run(True)
    finally:
        ext_bf.known_sumsq = original
    assert len(seen) == 1 and seen[0] is not None


def test_per_sample_gradient_statistics_with_the_index_yielding_loader():
    """config.use_gradient (qscheme.py:20-22,37-55): every layer keeps one running squared gradient
    norm per dataset entry; the loader supplies the entries of each batch.  The table lives on the
    device, holds 0.5 * ||grad_n||^2 after an entry's first visit (running value from 0), leaves
    entries not yet visited at zero, and entries not yet visited borrow the batch mean when the
    widths are allocated."""
    from torch.utils.data import TensorDataset
    from actnn_amd.dataloader import DataLoader
    torch.manual_seed(0)
    data = TensorDataset(torch.randn(48, 8, 16, 16) * torch.linspace(0.2, 3.0, 48).view(48, 1, 1, 1),
                         torch.randint(0, 4, (48,)))
    config.use_gradient = True
    QScheme.num_samples = len(data)
    model = QModule(nn.Sequential(nn.Conv2d(8, 8, 3, padding=1), nn.BatchNorm2d(8), nn.ReLU(),
                                  nn.Conv2d(8, 4, 3, padding=1), nn.AdaptiveAvgPool2d(1), nn.Flatten())).to(DEV)
    first, last = QScheme.layers[0], QScheme.layers[1]
    assert first.scales.shape == (48,)
    grads = {}
    model.model[3].register_full_backward_hook(lambda m, gi, go: grads.__setitem__("last", go[0].detach().clone()))
    loader = DataLoader(data, batch_size=16, shuffle=True, generator=torch.Generator().manual_seed(1))
    seen = []
    for step, (indices, (x, y)) in enumerate(loader):
        QScheme.batch = indices
        F.cross_entropy(model(x.to(DEV)), y.to(DEV)).backward()
        seen += indices
        assert last.scales.is_cuda and first.scales.is_cuda
        want = 0.5 * grads["last"].double().flatten(1).square().sum(1)
        got = last.scales[torch.tensor(indices, device=DEV)].double()
        assert torch.allclose(got, want, rtol=1e-5, atol=0)
        rest = sorted(set(range(48)) - set(seen))
        assert (last.scales[torch.tensor(rest, device=DEV, dtype=torch.long)] == 0).all()
        if step == 1:
            break
    # second visit: running value, and a batch with unseen entries borrows the mean for them
    QScheme.batch = seen[:8] + rest[:8]
    scale = last.get_scale(torch.device(DEV))
    table = last.scales[torch.tensor(QScheme.batch, device=DEV)]
    assert torch.equal(scale[:8], table[:8]) and (table[8:] == 0).all()
    assert torch.allclose(scale[8:], (table.mean() + 1e-9).expand(8))
    before = last.scales.clone()
    x, y = data[QScheme.batch]
    F.cross_entropy(model(x.to(DEV)), y.to(DEV)).backward()
    want = 0.5 * before[torch.tensor(QScheme.batch, device=DEV)].double() \
        + 0.5 * grads["last"].double().flatten(1).square().sum(1)
    assert torch.allclose(last.scales[torch.tensor(QScheme.batch, device=DEV)].double(), want, rtol=1e-5, atol=0)
    assert int(last.b.min()) >= 1 and int(last.b.sum()) <= int(last.bits * 16) and len(set(last.b.tolist())) > 1


def test_sync_batch_norm_of_one_process_is_batch_norm(monkeypatch):
    """QSyncBatchNorm without peers (no process group, or a group of one rank) takes the path of
    QBatchNorm2d (layers.py:444-455): same output, gradients and saved stream; with peers it
    refuses, since the statistics exchange is not part of this build."""
    import torch.distributed as dist
    def run(cls):
        config.reset(); QScheme.reset(); QBNScheme.reset()
        torch.manual_seed(0)
        bn = cls(64).to(DEV)
        x = torch.randn(8, 64, 16, 16, device=DEV, requires_grad=True)
        torch.cuda.manual_seed(3)
        y = bn(x)
        saved = y.grad_fn.saved[0]
        grads = torch.autograd.grad(y, [x, bn.weight, bn.bias], torch.ones_like(y) * x.detach())
        return y, saved, grads, bn
    y0, s0, g0, _ = run(actnn_amd.QBatchNorm2d)
    y1, s1, g1, bn = run(actnn_amd.QSyncBatchNorm)
    assert torch.equal(y0, y1) and all(torch.equal(a, b) for a, b in zip(g0, g1))
    assert all(torch.equal(a, b) for a, b in zip(s0, s1))
    assert int(bn.num_batches_tracked) == 1 and isinstance(bn, nn.SyncBatchNorm)
    with pytest.raises(ValueError):
        bn(torch.randn(8, 64, 4, 4))                                   # host tensor, as the reference
    bn.eval()
    assert torch.allclose(bn(y0.detach()), F.batch_norm(y0.detach(), bn.running_mean, bn.running_var,
                                                        bn.weight, bn.bias, False, 0.1, bn.eps), atol=1e-5)
    bn.train()
    monkeypatch.setattr(dist, "is_initialized", lambda: True)
    monkeypatch.setattr(dist, "get_world_size", lambda group=None: 1)
    assert torch.equal(bn(y0.detach()), actnn_amd.QSyncBatchNorm(64).to(DEV)(y0.detach()))
    monkeypatch.setattr(dist, "get_world_size", lambda group=None: 2)
    with pytest.raises(NotImplementedError):
        bn(y0.detach())


def test_layer_norm_re_exports_against_torch():
    """backward_func's three layer-norm names (backward_func.cc:83-85) against F.layer_norm and
    autograd."""
    import actnn_amd.cpp_extension.backward_func as ext_bf
    torch.manual_seed(0)
    x = torch.randn(6, 5, 32, 8, device=DEV, requires_grad=True)
    w = (torch.rand(32, 8, device=DEV) + 0.5).requires_grad_(True)
    b = torch.randn(32, 8, device=DEV, requires_grad=True)
    X, gamma, beta, M, N = ext_bf.prepare_layer_norm_inputs(x.detach(), (32, 8), w.detach(), b.detach())
    assert (M, N) == (30, 256)
    Y, mean, rstd = ext_bf.layer_norm_cuda(X, gamma, beta, M, N, 1e-5)
    ref = F.layer_norm(x, (32, 8), w, b, 1e-5)
    assert torch.allclose(Y, ref, atol=1e-5)
    assert torch.allclose(mean, x.detach().reshape(30, 256).mean(1), atol=1e-5)
    dY = torch.randn_like(ref)
    gx, gw, gb = torch.autograd.grad(ref, [x, w, b], dY)
    dX, dgamma, dbeta = ext_bf.layer_norm_backward_cuda(dY, X, mean, rstd, gamma, M, N, [True, True, True])
    assert torch.allclose(dX, gx, atol=1e-4) and torch.allclose(dgamma, gw, atol=1e-4)
    assert torch.allclose(dbeta, gb, atol=1e-4)
    with pytest.raises(RuntimeError):
        ext_bf.prepare_layer_norm_inputs(x.detach(), (8,), w.detach(), None)      # weight shape
    with pytest.raises(RuntimeError):
        ext_bf.prepare_layer_norm_inputs(x.detach(), (16, 8), None, None)         # trailing dims


@pytest.mark.parametrize("channels_last", [False, True])
def test_fixed_width_batch_norm_takes_the_fused_passes(channels_last):
    """Levels without per-sample allocation (L2: 4 bits everywhere, no scheme): batch norm still
    writes the packed copy of its input in its normalising pass - the per-sample stream at one
    width - and reads it back in the backward kernels.  Output identical to the unfused sequence,
    saved input within one quantisation step, gradients those of the dequantised input."""
    def run(fused):
        config.reset(); QScheme.reset(); QBNScheme.reset()
        set_optimization_level("L2")
        config.fused_bn_pack = fused
        config.fused_bn_backward = fused
        torch.manual_seed(0)
        bn = actnn_amd.QBatchNorm2d(64).to(DEV)
        assert bn.scheme is None
        x = torch.randn(16, 64, 14, 14, device=DEV).bfloat16()
        if channels_last:
            bn = bn.to(memory_format=torch.channels_last)
            x = x.contiguous(memory_format=torch.channels_last)
        x.requires_grad_(True)
        torch.cuda.manual_seed(2)
        y = bn(x)
        quantized, _, _, _, save_mean, save_invstd = y.grad_fn.saved[:6]
        back = dequantize_activation(quantized, x.shape)
        g = torch.randn_like(y)
        grads = torch.autograd.grad(y, [x, bn.weight, bn.bias], g)
        return x, y, quantized, back, g, grads, (bn.weight.detach(), save_mean, save_invstd)
    x, y1, q1, back1, g, grads1, stats = run(True)
    _, y0, q0, back0, _, grads0, _ = run(False)
    assert isinstance(q1[1], torch.Tensor) and q1[1].tolist() == [4] * 16 and isinstance(q0[1], int)
    assert q1[0].numel() * 4 == x.numel() * 4 // 8                       # int32 words: 4 bits per element
    assert torch.equal(y0, y1)
    span = (x.detach().float().max() - x.detach().float().min()).item()
    for back in (back0, back1):
        assert back.shape == x.shape and (back.float() - x.detach().float()).abs().max().item() <= span / 15 + 0.05
    # the backward kernels rebuild x exactly as the unpack kernel does: same gradients, bit for bit,
    # as the plain backward pass on the dequantised tensor
    import actnn_amd.cpp_extension.backward_func as ext_bf
    want = ext_bf.hip_batch_norm_backward(back1, g, *stats)
    assert all(torch.equal(a, b) for a, b in zip(grads1, want))
    assert torch.equal(grads1[2], grads0[2])                             # the bias gradient never sees x
    # and the quantisation noise is unbiased: the input gradient stays close to the exact layer's
    ref = nn.BatchNorm2d(64).to(DEV)
    xr = x.detach().float().requires_grad_(True)
    (gx,) = torch.autograd.grad(ref(xr), xr, g.float())
    assert (grads1[0].float() - gx).abs().max() <= 0.05 * gx.abs().max() + 0.05


@pytest.mark.parametrize("level", ["L3", "L2"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("channels,size,folded", [(64, 8, True), (128, 4, True), (256, 8, True), (32, 8, True),
                                                  (512, 4, True), (1024, 2, True), (96, 8, False), (768, 4, False)])
def test_relu_folded_into_the_batch_norm_pass_equals_the_two_layers(dtype, channels, size, folded, level):
    """layers.bn_relu hands a converted batch norm and the ReLU after it over together: where the
    shape allows (channels-last, 16-bit, C a divisor of 256 or a multiple of 512) the ReLU runs inside the normalise +
    pack pass, and the backward passes apply the ReLU's mask to the gradient as they read it.
    Output, group min / max left for the next layer, running statistics, the compressed input and
    every gradient are those of the two layers, bit for bit - also with only the forward folded, and
    at the level with one width for all (L2) as with per-sample widths (L3); other shapes take the
    two layers."""
    from actnn_amd import ops
    from actnn_amd.layers import QBatchNorm2d, QReLU, bn_relu, known_group_minmax
    calls = []
    real = ops.batch_norm_relu.forward

    def run(fold, fold_backward=True):
        config.reset(); QScheme.reset(); QBNScheme.reset()
        set_optimization_level(level)
        config.fused_bn_relu = fold
        config.fused_bn_relu_backward = fold_backward
        torch.manual_seed(3)
        bn, relu = QBatchNorm2d(channels).to(DEV).train(), QReLU()
        with torch.no_grad():
            bn.weight.uniform_(-1.0, 1.5)
            bn.bias.normal_()
        g = torch.Generator(device=DEV).manual_seed(9)
        x = (torch.randn(16, channels, size, size, device=DEV, generator=g) * 2 + 0.3).to(dtype)
        x = x.contiguous(memory_format=torch.channels_last).requires_grad_(True)
        go = torch.randn(16, channels, size, size, device=DEV, generator=g).to(dtype).contiguous(memory_format=torch.channels_last)
        torch.cuda.manual_seed(21)
        out = bn_relu(bn, relu, x)
        known = known_group_minmax(out)
        out.backward(go)
        return [out.detach(), x.grad, bn.weight.grad, bn.bias.grad, bn.running_mean.clone(), bn.running_var.clone()] + \
               (list(known) if known is not None else [])

    def spy(*a, **k):
        calls.append(1)
        return real(*a, **k)

    ops.batch_norm_relu.forward = staticmethod(spy)
    try:
        two, one, half = run(False), run(True), run(True, False)
    finally:
        ops.batch_norm_relu.forward = staticmethod(real)
    assert len(calls) == (2 if folded else 0)
    assert len(two) == len(one) == len(half)
    for i, (u, v, w) in enumerate(zip(two, one, half)):
        assert torch.equal(u, v) and torch.equal(u, w), i
    assert one[0].is_contiguous(memory_format=torch.channels_last) and float(one[0].min()) == 0.0


@pytest.mark.parametrize("level", ["L3", "L2"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("channels,size,folded", [(256, 8, True), (64, 8, True), (512, 4, True), (2048, 2, True),
                                                  (96, 8, False)])
def test_closing_step_of_a_residual_block_in_the_batch_norm_pass(dtype, channels, size, folded, level):
    """layers.bn_add_relu: relu(bn(x) + identity) with the addition and the ReLU inside the batch norm's
    normalise + pack pass.  Output, group min / max, running statistics and the gradients of x, of the
    identity and of the batch norm's parameters are those of QBatchNorm2d, the tensor addition and
    QReLU (through QAddReLU) one after the other, bit for bit; a residual in another layout, and
    shapes the pass does not take, go through the separate layers."""
    from actnn_amd import ops
    from actnn_amd.layers import QAddReLU, QBatchNorm2d, bn_add_relu, known_group_minmax
    calls = []
    real = ops.batch_norm_add_relu.forward

    def run(fold, residual_layout=torch.channels_last):
        config.reset(); QScheme.reset(); QBNScheme.reset()
        set_optimization_level(level)
        config.fused_bn_relu = fold
        torch.manual_seed(4)
        bn, close = QBatchNorm2d(channels).to(DEV).train(), QAddReLU()
        with torch.no_grad():
            bn.weight.uniform_(-1.0, 1.5)
            bn.bias.normal_()
        g = torch.Generator(device=DEV).manual_seed(10)
        x = (torch.randn(8, channels, size, size, device=DEV, generator=g) * 2 + 0.3).to(dtype)
        x = x.contiguous(memory_format=torch.channels_last).requires_grad_(True)
        res = torch.randn(8, channels, size, size, device=DEV, generator=g).to(dtype)
        res = res.contiguous(memory_format=residual_layout).requires_grad_(True)
        go = torch.randn(8, channels, size, size, device=DEV, generator=g).to(dtype).contiguous(memory_format=torch.channels_last)
        torch.cuda.manual_seed(22)
        out = bn_add_relu(bn, close, x, res)
        known = known_group_minmax(out)
        out.backward(go)
        return [out.detach(), x.grad, res.grad, bn.weight.grad, bn.bias.grad, bn.running_mean.clone(),
                bn.running_var.clone()] + (list(known) if known is not None else [])

    def spy(*a, **k):
        calls.append(1)
        return real(*a, **k)

    ops.batch_norm_add_relu.forward = staticmethod(spy)
    try:
        two, one = run(False), run(True)
        other_layout = run(True, torch.contiguous_format)
    finally:
        ops.batch_norm_add_relu.forward = staticmethod(real)
    assert len(calls) == (1 if folded else 0)
    assert len(two) == len(one)
    for i, (u, v) in enumerate(zip(two, one)):
        assert torch.equal(u, v), i
    for i, (u, v) in enumerate(zip(two[:7], other_layout[:7])):
        assert torch.equal(u, v), i


@pytest.mark.parametrize("level", ["L3", "L2"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("identity_from", ["input", "batch_norm"])
@pytest.mark.parametrize("channels,size", [(256, 8), (512, 4), (96, 8)])
def test_skip_connection_gradient_in_one_pass_equals_mask_then_addition(dtype, channels, size, level, identity_from):
    """layers.skip_connection ties a residual block's two uses of its input together: the closing
    step leaves the output's gradient and its ReLU mask, and the input's gradient is the gradient from
    the block's layers plus the masked one, made in one pass.  The input's gradient, the batch norm's
    parameter gradients, the output and the shared group min / max are those of the untied block (the
    mask applied first, autograd adding the two), bit for bit; a shape the fold does not take, and an
    unconverted closing layer, get the input twice.  The same for an identity that is a batch norm's
    output (a downsample branch): that batch norm's backward passes then mask the gradient as they
    read it, and nothing is written for the identity."""
    from actnn_amd import ops
    from actnn_amd.layers import (AddReLU, QAddReLU, QBatchNorm2d, QReLU, bn_add_relu, bn_relu, known_group_minmax,
                                  skip_connection)
    handed = []
    real = ops.SkipGradient.hand_over

    def spy(self, *a):
        handed.append(1)
        return real(self, *a)

    def run(tied):
        config.reset(); QScheme.reset(); QBNScheme.reset()
        set_optimization_level(level)
        config.fused_skip_gradient = tied
        torch.manual_seed(4)
        bn1, relu1 = QBatchNorm2d(channels).to(DEV).train(), QReLU()
        bn3, close = QBatchNorm2d(channels).to(DEV).train(), QAddReLU()
        bn_ds = QBatchNorm2d(channels).to(DEV).train()
        with torch.no_grad():
            for bn in (bn1, bn3, bn_ds):                              # either sign, none near zero: a channel that is
                bn.weight.uniform_(0.4, 1.5)                   # almost constant turns 2-bit noise into overflowing
                bn.weight.mul_(torch.where(torch.rand_like(bn.weight) < 0.3, -1.0, 1.0))     # float16 gradients
                bn.bias.normal_()
        g = torch.Generator(device=DEV).manual_seed(10)
        leaf = (torch.randn(8, channels, size, size, device=DEV, generator=g) * 2 + 0.3).to(dtype)
        leaf = leaf.contiguous(memory_format=torch.channels_last).requires_grad_(True)
        go = torch.randn(8, channels, size, size, device=DEV, generator=g).to(dtype).contiguous(memory_format=torch.channels_last)
        torch.cuda.manual_seed(22)
        x = QReLU()(leaf)                                      # a block input that carries its group min / max
        if identity_from == "input":
            main, identity = skip_connection(close, x)
            assert (known_group_minmax(main) is None) == (known_group_minmax(x) is None)
        else:
            main, identity = x, bn_ds(x * 0.5)
        out = bn_add_relu(bn3, close, bn_relu(bn1, relu1, main * 0.75), identity)
        known = known_group_minmax(out)
        out.backward(go)
        return [out.detach(), leaf.grad, bn1.weight.grad, bn1.bias.grad, bn3.weight.grad, bn3.bias.grad] + (
            [bn_ds.weight.grad, bn_ds.bias.grad] if identity_from == "batch_norm" else []) + (
            list(known) if known is not None else [])

    ops.SkipGradient.hand_over = spy
    try:
        untied, tied = run(False), run(True)
    finally:
        ops.SkipGradient.hand_over = real
    assert len(handed) == (1 if channels != 96 else 0)
    assert len(untied) == len(tied)
    for i, (u, v) in enumerate(zip(untied, tied)):
        assert torch.isfinite(u).all(), i
        assert torch.equal(u, v), i
    x = torch.randn(2, 8, 4, 4, device=DEV, requires_grad=True)
    main, identity = skip_connection(AddReLU(), x)
    assert main is x and identity is x



def test_an_identity_of_two_closing_steps_and_of_another_use_keeps_every_gradient():
    """One tensor as the identity of two closing steps, and used once more besides: the first
    closing step hands its gradient over, the second finds the place taken and returns its masked
    gradient the ordinary way, the other use's gradient arrives as usual.  Output and parameter
    gradients are those of the untied graph bit for bit; the input's gradient is a sum of five bf16
    terms whose order of addition differs between the two graphs, so it agrees to the rounding of
    those additions (no term lost: dropping any one of them is an error of order one)."""
    from actnn_amd.layers import QAddReLU, QBatchNorm2d, QReLU, bn_add_relu, skip_connection

    def run(tied):
        config.reset(); QScheme.reset(); QBNScheme.reset()
        set_optimization_level("L3")
        config.fused_skip_gradient = tied
        torch.manual_seed(4)
        bns = [QBatchNorm2d(64).to(DEV).train() for _ in range(2)]
        close = QAddReLU()
        g = torch.Generator(device=DEV).manual_seed(10)
        leaf = torch.randn(8, 64, 8, 8, device=DEV, generator=g).to(torch.bfloat16)
        leaf = leaf.contiguous(memory_format=torch.channels_last).requires_grad_(True)
        go = torch.randn(8, 64, 8, 8, device=DEV, generator=g).to(torch.bfloat16).contiguous(memory_format=torch.channels_last)
        torch.cuda.manual_seed(22)
        x = QReLU()(leaf)
        main, identity = skip_connection(close, x)
        out = bn_add_relu(bns[0], close, main * 0.75, identity) + bn_add_relu(bns[1], close, main * 1.25, identity) \
            + identity * 0.5
        out.backward(go)
        return [out.detach(), leaf.grad] + [p.grad for bn in bns for p in bn.parameters()]

    for i, (u, v) in enumerate(zip(run(False), run(True))):
        assert torch.isfinite(u).all(), i
        if i == 1:
            assert ((u.float() - v.float()).abs() <= 2.0 ** -6 * (u.float().abs() + 1.0)).all()
        else:
            assert torch.equal(u, v), i
