"""Host-side logic that needs no GPU: configuration levels, model conversion, state-dict
prefix handling, memory accounting, argument checks of the bindings."""
import pytest
import torch
import torch.nn as nn

import actnn_amd
from actnn_amd import QBNScheme, QModule, QScheme, config, set_optimization_level
from actnn_amd.resnet import resnet50


@pytest.fixture(autouse=True)
def fresh_config():
    config.reset()
    QScheme.reset()
    QBNScheme.reset()
    yield
    config.reset()
    QScheme.reset()
    QBNScheme.reset()


def test_defaults_and_levels():
    assert config.activation_compression_bits == [2, 8, 8] and config.initial_bits == 8
    assert config.group_size == 256 and config.stochastic and config.compress_activation
    set_optimization_level("L0")
    assert not config.compress_activation and not config.adaptive_conv_scheme
    config.reset()
    set_optimization_level("L1")
    assert config.activation_compression_bits == [4] and not config.enable_quantized_bn
    config.reset()
    set_optimization_level("L2")
    assert config.activation_compression_bits == [4] and config.enable_quantized_bn
    assert not config.adaptive_bn_scheme
    config.reset()
    set_optimization_level("L3.1")
    assert config.pipeline_threshold == 3 * 1024 ** 3 and config.empty_cache_threshold == 0.2
    config.reset()
    set_optimization_level("L4")
    assert config.swap and config.compress_activation
    config.reset()
    set_optimization_level("swap")
    assert config.swap and not config.compress_activation
    with pytest.raises(ValueError):
        set_optimization_level("L9")


def test_resnet50_conversion_counts():
    # 53 convs + 1 fc carry a QScheme, 53 batch norms a QBNScheme, 49 ReLU sites, 1 max-pool
    model = QModule(resnet50())
    kinds = [type(m).__name__ for m in model.modules()]
    assert kinds.count("QConv2d") == 53 and kinds.count("QBatchNorm2d") == 53
    assert kinds.count("QLinear") == 1 and kinds.count("QReLU") == 49 and kinds.count("QMaxPool2d") == 1
    assert not any(k in ("Conv2d", "BatchNorm2d", "ReLU", "MaxPool2d", "Linear") for k in kinds)
    assert len(QScheme.layers) == 54 and len(QBNScheme.layers) == 53
    # kernel positions feed the sensitivity: 7x7 stem, 3x3 and 1x1 convs
    locs = sorted({s.num_locations for s in QScheme.layers})
    assert locs == [1, 9, 49]
    # every BN scheme remembers the conv built just before it
    assert all(b.prev_linear is not None for b in QBNScheme.layers)


def test_l1_leaves_batch_norm_alone():
    set_optimization_level("L1")
    model = QModule(nn.Sequential(nn.Conv2d(3, 8, 3), nn.BatchNorm2d(8), nn.ReLU()))
    kinds = [type(m).__name__ for m in model.model]
    assert kinds == ["QConv2d", "BatchNorm2d", "QReLU"]
    assert model.model[0].scheme is None          # no adaptive scheme at L1


def test_state_dict_has_no_wrapper_prefix_and_round_trips():
    plain = nn.Sequential(nn.Conv2d(3, 4, 3), nn.BatchNorm2d(4), nn.ReLU(), nn.Flatten(), nn.Linear(4, 2))
    keys = list(plain.state_dict().keys())
    model = QModule(plain)
    sd = model.state_dict()
    assert list(sd.keys()) == keys
    sd = {k: torch.randn_like(v) if v.is_floating_point() else v for k, v in sd.items()}
    model.load_state_dict(sd)
    assert torch.equal(model.model[0].weight, sd["0.weight"])


def test_train_eval_toggle_config():
    model = QModule(nn.Sequential(nn.Linear(4, 4)))
    model.eval()
    assert not config.training
    y = model(torch.randn(2, 4))                  # eval path is plain nn.Linear: runs on CPU
    assert y.shape == (2, 4)
    model.train()
    assert config.training


def test_compute_tensor_bytes_counts_like_the_reference():
    ts = [torch.zeros(10), torch.zeros(10, dtype=torch.int32), torch.zeros(10, dtype=torch.bfloat16),
          torch.zeros(10, dtype=torch.float16), torch.zeros(10, dtype=torch.int8),
          torch.zeros(10, dtype=torch.float64), None, 4]
    assert actnn_amd.compute_tensor_bytes(ts) == 40 + 40 + 20 + 20 + 10
    assert actnn_amd.compute_tensor_bytes(torch.zeros(3, 5)) == 60


def test_bindings_reject_host_tensors():
    import actnn_amd.cpp_extension.minimax as ext_minimax
    import actnn_amd.cpp_extension.quantization as ext_q
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        ext_minimax.minimax(torch.randn(4, 256))
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        ext_q.act_quantized_relu(torch.randn(4))
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        ext_q.pack_single_precision(torch.randn(2, 2, 256), torch.randn(2, 2, 1), torch.randn(2, 2, 1), 2, True)
    import actnn_amd.cpp_extension.calc_precision as ext_cp
    with pytest.raises(RuntimeError):
        ext_cp.calc_precision(torch.ones(4), torch.ones(4), torch.ones(4, dtype=torch.int32), 8)   # b dtype


def test_calc_precision_binding_mutates_and_returns_b():
    import actnn_amd.cpp_extension.calc_precision as ext_cp
    b = torch.ones(256, dtype=torch.int32) * 8
    out = ext_cp.calc_precision(b, torch.zeros(256), torch.ones(256, dtype=torch.int32), 512)
    assert out is b and int(b.sum()) == 512 and int(b[36]) == 5


def test_perlayer_allocation_on_host():
    # three fake layers with very different sensitivities: bits must follow C, average stays 2
    class L:
        weight = nn.Parameter(torch.zeros(1))
    schemes = [QScheme(L()) for _ in range(3)]
    N = 16
    for s, c, d in zip(schemes, (1e-3, 1.0, 1e3), (1000, 1000, 1000)):
        s.C = torch.full((N,), c)
        s.dim = d
    QScheme.allocate_perlayer()
    bits = [float(s.bits) for s in schemes]
    assert bits[0] <= bits[1] <= bits[2] and bits[0] < bits[2]
    assert abs(sum(bits) / 3 - 2.0) < 0.05
    b1 = QBNScheme()
    QBNScheme.allocate_perlayer()
    assert float(b1.bits) == bits[2]              # BN copies the preceding layer's budget


@pytest.mark.parametrize("layers,N", [(54, 512), (54, 128), (3, 7), (1, 1), (9, 8192)])
def test_perlayer_mean_widths_in_one_operation_equal_the_per_layer_expression(layers, N):
    # allocate_perlayer takes every layer's mean width from one reduction over [layers, N]; the
    # reference's expression is a mean over each layer's slice (qscheme.py:127-128): same values, bit for bit
    g = torch.Generator().manual_seed(layers * 1000 + N)
    b = torch.randint(1, 9, (layers * N,), generator=g, dtype=torch.int32)
    together = b.view(layers, N).float().mean(1)
    for i in range(layers):
        one = b[i * N:(i + 1) * N].float().mean()
        assert one.dtype == together[i].dtype and one.shape == together[i].shape
        assert torch.equal(one, together[i])
    dims = torch.randint(1, 10 ** 6, (layers,), generator=g, dtype=torch.int32)
    assert torch.equal(dims.repeat_interleave(N),
                       torch.cat([torch.ones(N, dtype=torch.int32) * int(d) for d in dims], 0))


def test_adaptive_avg_pool2d_keeps_only_the_shape():
    import torch.nn.functional as F
    from actnn_amd.ops import adaptive_avg_pool2d
    x = torch.randn(3, 5, 7, 4, dtype=torch.float64, requires_grad=True)
    y = adaptive_avg_pool2d.apply(x, (1, 1))
    ref = F.adaptive_avg_pool2d(x, (1, 1))
    assert torch.allclose(y, ref)
    g = torch.randn_like(ref)
    (gx,) = torch.autograd.grad(y, x, g)
    (gr,) = torch.autograd.grad(ref, x, g)
    assert torch.allclose(gx, gr) and y.grad_fn.saved == x.shape
    with pytest.raises(AssertionError):
        adaptive_avg_pool2d.apply(x, (2, 2))


class _FakeLib:
    """Stands in for the C-ABI library where a test only needs to see which calls are made."""

    def __init__(self):
        self.prefix_calls = 0

    def actnn_bits_prefix(self, bits_ptr, prefix_ptr, N, stream):
        self.prefix_calls += 1
        return 0


def test_bits_cache_follows_the_version_counter(monkeypatch):
    # the sum / prefix / host copy attached to a `bits` tensor must not outlive an in-place change
    import actnn_amd.cpp_extension._glue as glue
    import actnn_amd.cpp_extension.quantization as ext_q
    fake = _FakeLib()
    monkeypatch.setattr(glue, "lib", lambda: fake)
    monkeypatch.setattr(glue, "stream_ptr", lambda device: 0)
    host = torch.tensor([2, 2, 3, 1], dtype=torch.int32)
    bits = ext_q.attach_bits_host(host.clone(), host)
    total, prefix = ext_q._bits_info(bits)
    assert total == 8 and fake.prefix_calls == 1
    assert ext_q._bits_info(bits)[1] is prefix and fake.prefix_calls == 1        # cache hit
    bits[0] = 8                                                                  # in-place: version moves on
    total2, prefix2 = ext_q._bits_info(bits)
    assert total2 == 14 and prefix2 is not prefix and fake.prefix_calls == 2      # re-read, not the stale sum
    bits[1] = 9                                                                  # out of range now
    with pytest.raises(RuntimeError, match="1..8 bits"):
        ext_q._bits_info(bits)
    # a total attached by the device allocation is dropped the same way
    b2 = ext_q.attach_bits_total(torch.full((4,), 2, dtype=torch.int32), 8, prefix=torch.zeros(5, dtype=torch.int32))
    assert ext_q._bits_info(b2)[0] == 8 and fake.prefix_calls == 2               # prefix came attached
    b2.fill_(4)
    assert ext_q._bits_info(b2)[0] == 16 and fake.prefix_calls == 3


@pytest.mark.parametrize("padding,kernel", [("same", 3), ("same", 4), ("valid", 3), (1, 3)])
def test_qconv_string_padding_matches_torch(padding, kernel):
    # with compression off the Q-layer's training path (custom Function, explicit backward
    # operator) runs on the CPU: outputs and all three gradients must equal nn.Conv2d's
    from actnn_amd.layers import QConv2d
    set_optimization_level("L0")
    torch.manual_seed(0)
    ref = nn.Conv2d(3, 5, kernel, padding=padding)
    q = QModule(nn.Sequential(nn.Conv2d(3, 5, kernel, padding=padding)))
    assert isinstance(q.model[0], QConv2d) and q.model[0].padding == ref.padding
    q.model[0].load_state_dict(ref.state_dict())
    x = torch.randn(2, 3, 9, 8, requires_grad=True)
    xr = x.detach().clone().requires_grad_(True)
    y, yr = q(x), ref(xr)
    assert torch.allclose(y, yr, atol=1e-6)
    g = torch.randn_like(yr)
    y.backward(g)
    yr.backward(g)
    assert torch.allclose(x.grad, xr.grad, atol=1e-5)
    assert torch.allclose(q.model[0].weight.grad, ref.weight.grad, atol=1e-5)
    assert torch.allclose(q.model[0].bias.grad, ref.bias.grad, atol=1e-5)


def test_no_scheme_path_keeps_group_ranges_whatever_pergroup_says():
    # the reference's fixed-width path (ops.py:77-96) never reads config.pergroup
    from actnn_amd.ops import no_scheme_compute_quantization_bits
    from actnn_amd.qscheme import group_min_max
    x = torch.randn(2, 4, 8, 16)                     # 512 features: two groups per sample
    rows = x.view(-1, 256)
    known = (rows.min(1)[0], rows.max(1)[0])
    config.pergroup = False
    config.activation_compression_bits = [4]
    groups, bits, mn, mx = no_scheme_compute_quantization_bits(x, known)
    assert bits == 4 and torch.equal(mn.view(-1), known[0]) and torch.equal(mx.view(-1), known[1])
    _, mn_s, mx_s, _ = group_min_max(x, known)        # the schemes' rule: one range for the tensor
    assert bool((mn_s == x.min()).all()) and bool((mx_s == x.max()).all())


def test_skip_connection_hand_over_and_ordinary_accumulation():
    """The tie between a residual block's two uses of its input, on the host side: host tensors and
    unconverted closing layers get the input twice; the autograd node adds the two gradients like
    the engine would when nothing was handed over; a hand-over is taken exactly once."""
    from actnn_amd import ops
    from actnn_amd.layers import AddReLU, QAddReLU, skip_connection
    x = torch.randn(2, 4, 3, 3, requires_grad=True)
    for closing in (AddReLU(), QAddReLU()):
        main, identity = skip_connection(closing, x)                 # a host tensor is never tied
        assert main is x and identity is x
    tie = ops.SkipGradient()
    assert tie.take() == (None, None, None)
    assert tie.hand_over("g", "m", torch.channels_last) and not tie.hand_over("g2", "m2", None)
    assert tie.take() == ("g", "m", torch.channels_last) and tie.take() == (None, None, None)
    # nothing handed over: the node is the plain sum of what arrives on its two outputs
    tie = ops.SkipGradient()
    main, identity = ops.skip_connection.apply(x, tie)
    (main * 2.0 + identity * 3.0).sum().backward()
    assert torch.equal(x.grad, torch.full_like(x, 5.0))
    x.grad = None
    main, identity = ops.skip_connection.apply(x, ops.SkipGradient())
    (identity * 3.0).sum().backward()                                # only one of the two used
    assert torch.equal(x.grad, torch.full_like(x, 3.0))
