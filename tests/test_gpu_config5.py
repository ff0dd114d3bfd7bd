"""Benchmark config 5 at its stated size under `-m gpu`: ResNet-50 under QModule at L3, batch 512,
224 x 224, fp32 weights with bf16 autocast, SGD - the step of the reference's
mem_speed_benchmark/train.py:357-438 - in both memory layouts, with the activation-memory protocol
of train.py:363-397 checked against the closed form of the saved tensors; and, at a batch a
comparison can afford, the weight gradients of the compressed model against the exact model's."""
import pytest
import torch
import torch.nn.functional as F

from actnn_amd import QBNScheme, QModule, QScheme, config, set_optimization_level
from actnn_amd.resnet import resnet50
from actnn_amd.utils import compute_tensor_bytes, get_memory_usage
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
    torch.cuda.empty_cache()


# Saved tensors of ResNet-50 v1.5 at 224 x 224 per sample, (channels, height = width, count), written
# down from the public architecture (not read off the model under test):
CONV_INPUTS = [(3, 224, 1), (64, 56, 8), (256, 56, 4), (128, 56, 1), (512, 28, 5), (128, 28, 7), (256, 28, 1),
               (1024, 14, 7), (256, 14, 11), (512, 14, 1), (2048, 7, 2), (512, 7, 5)]
BN_INPUTS = [(64, 112, 1), (64, 56, 6), (256, 56, 4), (128, 56, 1), (128, 28, 7), (512, 28, 5), (256, 28, 1),
             (256, 14, 11), (1024, 14, 7), (512, 14, 1), (512, 7, 5), (2048, 7, 4)]
# ReLU outputs (one 1-bit mask each): stem, then per bottleneck relu1, relu2 (after the stride) and relu3
RELU_OUTPUTS = [(64, 112, 1), (64, 56, 6), (256, 56, 3), (128, 56, 1), (128, 28, 7), (512, 28, 4),
                (256, 28, 1), (256, 14, 11), (1024, 14, 6), (512, 14, 1), (512, 7, 5), (2048, 7, 3)]
FC_INPUT = 2048
POOL_OUTPUT = (64, 56)


def _elems(shapes):
    return sum(c * h * h * k for c, h, k in shapes)


QUANTISED_ELEMS = _elems(CONV_INPUTS) + _elems(BN_INPUTS) + FC_INPUT      # per sample
MASK_AND_INDEX_BYTES = _elems(RELU_OUTPUTS) // 8 + POOL_OUTPUT[0] * POOL_OUTPUT[1] ** 2 // 2
assert QUANTISED_ELEMS == 21_778_432 and QUANTISED_ELEMS % 256 == 0 and _elems(RELU_OUTPUTS) == 9_608_704


def compressed_bytes_per_sample(avg_bits=2):
    """Quantised conv / batch-norm / fc inputs at `avg_bits` with one bf16 scale and one bf16 minimum
    per group of 256."""
    return QUANTISED_ELEMS * avg_bits // 8 + QUANTISED_ELEMS // 256 * 2 * 2


def closed_form_bytes_per_sample(avg_bits=2):
    """Bytes the L3 model keeps per sample for the backward pass: the compressed inputs, 1-bit ReLU
    masks, max-pool indices at two per byte."""
    return compressed_bytes_per_sample(avg_bits) + MASK_AND_INDEX_BYTES


@pytest.mark.timeout(900)
@pytest.mark.parametrize("channels_last", [True, False])
def test_resnet50_l3_batch512_bf16_step(channels_last):
    batch = 512
    set_optimization_level("L3")
    torch.manual_seed(0)
    model = QModule(resnet50()).to(DEV).train()
    if channels_last:
        model = model.to(memory_format=torch.channels_last)
    opt = torch.optim.SGD(model.parameters(), lr=0.1, momentum=0.9, weight_decay=1e-4)
    g = torch.Generator(device=DEV).manual_seed(0)
    images = torch.randn(batch, 3, 224, 224, generator=g, device=DEV)
    if channels_last:
        images = images.contiguous(memory_format=torch.channels_last)
    target = torch.randint(0, 1000, (batch,), generator=g, device=DEV)
    print(f"[config5] channels_last={channels_last}: model built", flush=True)

    # what the conv / batch-norm / linear layers keep: dtype and bytes of every piece of every saved tuple
    saved_dtypes = set()
    saved_bytes = [0]
    import actnn_amd.ops as ops
    mark_saved = ops._mark_saved

    def spy(q, input):
        saved_dtypes.update((i, t.dtype) for i, t in enumerate(q) if isinstance(t, torch.Tensor))
        saved_bytes[0] += compute_tensor_bytes(list(q))
        return mark_saved(q, input)
    ops._mark_saved = spy
    try:
        for step in range(3):
            budgets = [float(s.bits) for s in QScheme.layers]     # per-layer budgets this step runs with
            saved_bytes[0] = 0
            torch.cuda.synchronize()
            init_mem = get_memory_usage()
            with torch.autocast("cuda", dtype=torch.bfloat16):
                output = model(images)
                loss = F.cross_entropy(output, target)
            torch.cuda.synchronize()
            act_mem = get_memory_usage() - init_mem - compute_tensor_bytes([loss, output])
            # per-sample widths of every conv / linear input: within 1..8 and summing to the layer's
            # budget int(bits * N) (qscheme.py:86-88)
            for s, budget in zip(QScheme.layers, budgets):
                b = s.b
                assert b.numel() == batch and int(b.min()) >= 1 and int(b.max()) <= 8
                assert int(b.sum()) == int(budget * batch), (s.name, int(b.sum()), budget)
            opt.zero_grad(set_to_none=True)
            loss.backward()
            opt.step()
            assert torch.isfinite(loss), step
            print(f"[config5] step {step}: loss {loss.item():.4f}, activation memory {act_mem / 2**30:.3f} GiB",
                  flush=True)
            if step == 0:
                # first step: no gradient statistic yet, every layer runs at 2 bits per sample
                assert all(b == 2 for b in budgets)
            else:
                # re-balanced budgets: the greedy pass over all layers keeps the dim-weighted average at 2
                dims = [s.dim for s in QScheme.layers]
                avg = sum(b * d for b, d in zip(budgets, dims)) / sum(dims)
                assert 1.9 < avg <= 2.0 + 1e-6, avg
            # The reference's protocol (train.py:363-397).  Besides the compressed inputs the layers'
            # contexts hold the 1-bit ReLU masks, the 4-bit pool indices and the bf16 copies of the
            # weights that autocast makes (25.6 M parameters).
            weights_bf16 = sum(p.numel() for p in model.parameters() if p.dim() > 1) * 2
            if step == 0:
                # every layer at 2 bits: the closed form of the saved tensors
                expect = closed_form_bytes_per_sample(2) * batch + weights_bf16
                assert abs(act_mem - expect) / expect < 0.05, (act_mem, expect)
                assert abs(saved_bytes[0] - compressed_bytes_per_sample(2) * batch) < 0.01 * saved_bytes[0]
            # every step (batch-norm inputs take the width of the convolution before them,
            # qbnscheme.py:54-60, so after the first re-balancing the total is not fixed by the 2-bit
            # budget): what is held is the compressed tuples and nothing else - no full-precision copy
            # of any activation survives the forward pass
            expect = saved_bytes[0] + MASK_AND_INDEX_BYTES * batch + weights_bf16
            assert abs(act_mem - expect) / expect < 0.05, (step, act_mem, expect)
            del loss, output
    finally:
        ops._mark_saved = mark_saved
    grads = [p.grad for p in model.parameters()]
    assert all(gr is not None and torch.isfinite(gr).all() for gr in grads)
    assert all(gr.dtype == torch.float32 for gr in grads)
    # (q_input, q_bits, q_scale, q_min): int32 stream and widths, bf16 scale / minimum - the dtypes
    # compute_tensor_bytes counts (utils.py:26-40)
    assert saved_dtypes == {(0, torch.int32), (1, torch.int32), (2, torch.bfloat16), (3, torch.bfloat16)}


@pytest.mark.timeout(600)
@pytest.mark.parametrize("channels_last", [False, True])
def test_resnet50_8bit_weight_gradients_match_the_exact_model(channels_last):
    """Compression only touches what is kept for the backward pass: the forward results are the
    exact model's, and with 8 bits per value every layer's weight gradient stays close to the exact
    one (fp32, no autocast, so that the only difference is the quantisation of the saved inputs)."""
    batch = 8
    torch.manual_seed(0)
    exact = resnet50().to(DEV).train()
    config.activation_compression_bits = [8, 8, 8]
    config.initial_bits = 8
    config.perlayer = False
    quant = QModule(resnet50()).to(DEV).train()
    quant.load_state_dict(exact.state_dict())
    if channels_last:
        exact = exact.to(memory_format=torch.channels_last)
        quant = quant.to(memory_format=torch.channels_last)
    x = torch.randn(batch, 3, 224, 224, device=DEV)
    if channels_last:
        x = x.contiguous(memory_format=torch.channels_last)
    y = torch.randint(0, 1000, (batch,), device=DEV)
    le = F.cross_entropy(exact(x), y)
    le.backward()
    lq = F.cross_entropy(quant(x), y)
    lq.backward()
    assert abs(le.item() - lq.item()) < 1e-3 * abs(le.item())
    worst = 0.0
    for (name, pe), (_, pq) in zip(exact.named_parameters(), quant.model.named_parameters()):
        if pe.dim() < 2:
            continue
        rel = float((pq.grad - pe.grad).norm() / pe.grad.norm())
        worst = max(worst, rel)
        assert rel < 0.1, (name, rel)
    print(f"[config5] worst relative weight-gradient error at 8 bits: {worst:.4f}", flush=True)
