"""Greedy allocation on the device vs the host routine (itself pinned against the oracle, brute
force and the reference's own calc_precision.cc in tests/test_oracle_calc_precision.py): the
widths must be identical, ties and zero sensitivities included."""
import numpy as np
import pytest
import torch

import actnn_amd.cpp_extension.calc_precision as ext_cp
from _util import DEV

pytestmark = pytest.mark.gpu


def _host(C, initial, target):
    N = C.numel()
    b = torch.ones(N, dtype=torch.int32) * initial
    return ext_cp.calc_precision(b, C.clone(), torch.ones(N, dtype=torch.int32), float(target))


def _cases():
    g = torch.Generator().manual_seed(0)
    yield "lognormal", torch.exp(3 * torch.randn(512, generator=g)), 8, 2 * 512
    yield "uniform", torch.rand(300, generator=g), 8, int(2.5 * 300)
    yield "all_zero", torch.zeros(16), 8, 32                  # first training step: every delta is -0
    yield "some_zero", torch.cat([torch.zeros(7), torch.rand(9, generator=g)]), 8, 40
    yield "duplicates", torch.tensor([1.0, 2.0, 1.0, 2.0, 1.0, 0.5, 0.5, 4.0] * 8), 8, 3 * 64
    yield "one_item", torch.tensor([3.0]), 8, 2
    yield "nothing_to_take", torch.rand(10, generator=g), 4, 40
    yield "over_budget", torch.rand(10, generator=g), 4, 50
    yield "everything_taken", torch.rand(10, generator=g), 8, 10
    yield "below_floor", torch.rand(10, generator=g), 8, 3    # cannot go below one bit each
    yield "initial_2", torch.rand(100, generator=g), 2, 150
    yield "initial_1", torch.rand(9, generator=g), 1, 9
    yield "huge_range", torch.tensor([1e-30, 1e30, 1.0, 1e-10, 1e10] * 20), 8, 250
    yield "max_candidates", torch.exp(torch.randn(1170, generator=g)), 8, 2 * 1170
    for seed in range(20):
        gg = torch.Generator().manual_seed(100 + seed)
        N = int(torch.randint(1, 600, (1,), generator=gg))
        initial = int(torch.randint(2, 9, (1,), generator=gg))
        avg = float(torch.rand(1, generator=gg)) * (initial - 1) + 1
        C = torch.exp(2 * torch.randn(N, generator=gg)).round(decimals=int(seed % 3))   # coarse values: ties
        yield f"random{seed}", C, initial, int(avg * N)


@pytest.mark.parametrize("name,C,initial,target", list(_cases()), ids=lambda v: v if isinstance(v, str) else "")
def test_device_allocation_equals_host(name, C, initial, target):
    C = C.float().contiguous()
    exp = _host(C, initial, target)
    got = ext_cp.calc_precision_device(C.to(DEV), initial, target)
    assert got.dtype == torch.int32 and got.is_cuda
    assert np.array_equal(got.cpu().numpy(), exp.numpy()), name


def test_device_allocation_rejects_what_does_not_fit():
    with pytest.raises(RuntimeError):
        ext_cp.calc_precision_device(torch.rand(1171, device=DEV), 8, 2000)      # 8197 candidates
    with pytest.raises(RuntimeError):
        ext_cp.calc_precision_device(torch.rand(8, device=DEV), 9, 16)
    with pytest.raises(RuntimeError):
        ext_cp.calc_precision_device(torch.rand(8), 8, 16)                        # host tensor
    assert ext_cp.calc_precision_device(torch.rand(0, device=DEV), 8, 0).numel() == 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("N,G", [(512, 49), (37, 3136), (8, 1)])
def test_allocation_in_one_call_equals_the_three_calls(N, G, dtype):
    import actnn_amd.cpp_extension.minimax as ext_minimax
    from actnn_amd.cpp_extension.quantization import _bits_info
    g = torch.Generator(device=DEV).manual_seed(N + G)
    mn = -torch.rand(N * G, generator=g, device=DEV).to(dtype)
    mx = (torch.rand(N * G, generator=g, device=DEV) * torch.exp(torch.randn(N, 1, generator=g, device=DEV)).expand(N, G).reshape(-1)).to(dtype)
    mult = torch.rand(N, generator=g, device=DEV) + 0.5
    for m in (None, mult, mult[:1].reshape(())):
        sens, bits, prefix = ext_cp.allocate_bits_device(mn, mx, N, 0.37, m, 8, 2 * N)
        sens_ref = ext_minimax.range_sqr(mn, mx, N, 0.37, m)
        bits_ref = ext_cp.calc_precision_device(sens_ref, 8, 2 * N)
        assert torch.equal(sens, sens_ref) and torch.equal(bits, bits_ref)
        assert torch.equal(prefix, _bits_info(bits_ref)[1])
        assert int(prefix[-1]) == int(bits.sum()) == 2 * N
    # also where the ranking takes nothing (every width stays 8), everything (every width 1), or
    # does not run at all (start width 1)
    for initial, target in ((8, 8 * N), (8, N), (1, N), (4, 3 * N)):
        sens, bits, prefix = ext_cp.allocate_bits_device(mn, mx, N, 0.37, None, initial, target)
        assert int(bits.sum()) == target and int(bits.min()) >= 1 and int(bits.max()) <= initial
        assert torch.equal(prefix[1:], torch.cumsum(bits, 0).to(torch.int32)) and int(prefix[0]) == 0


@pytest.mark.parametrize("N", [1, 2, 3, 100, 512, 1170])
def test_allocation_in_one_call_from_dirty_buffers(N):
    """The output buffers may hold anything on entry, and every repetition gives the same widths and
    the prefix of exactly those widths."""
    from actnn_amd import _lib
    lib = _lib.load()
    g = torch.Generator(device=DEV).manual_seed(N)
    G = 7
    mn = -torch.rand(N * G, generator=g, device=DEV)
    mx = torch.rand(N * G, generator=g, device=DEV) * torch.exp(torch.randn(N, 1, generator=g, device=DEV)).expand(N, G).reshape(-1)
    first = None
    for rep in range(20):
        sens = torch.empty(N, device=DEV)
        bits = torch.full((N,), -7, dtype=torch.int32, device=DEV)
        prefix = torch.full((N + 1,), 0x7fffffff - rep, dtype=torch.int32, device=DEV)
        rc = lib.actnn_allocate_bits_device(mn.data_ptr(), mx.data_ptr(), 0.5, None, 0, sens.data_ptr(),
                                            bits.data_ptr(), prefix.data_ptr(), N, G, 8, 2 * N, 0, None)
        assert rc == 0
        assert int(prefix[0]) == 0
        assert torch.equal(prefix[1:], torch.cumsum(bits, 0).to(torch.int32))
        assert int(prefix[-1]) == 2 * N
        if first is None:
            first = bits.clone()
        assert torch.equal(bits, first)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("known", [False, True])
def test_quantise_an_activation_in_one_call_equals_the_three_calls(dtype, known):
    """actnn_quantize_activation is [minimax] -> allocation -> pack_mixed on one stream: stream, scale,
    min, widths, prefix and sensitivities are those of the separate calls on the same generator state."""
    import actnn_amd.cpp_extension.minimax as ext_minimax
    import actnn_amd.cpp_extension.quantization as ext_q
    from actnn_amd.qscheme import AllocationArgs
    N, G = 24, 13
    g = torch.Generator(device=DEV).manual_seed(5)
    rows = (torch.randn(N * G, 256, generator=g, device=DEV)
            * torch.exp(torch.randn(N, 1, 1, generator=g, device=DEV)).expand(N, G, 256).reshape(N * G, 256)).to(dtype)
    per_sample = torch.rand(N, generator=g, device=DEV) + 0.5
    for mult in (None, per_sample[:1].reshape(()), per_sample):
        sens_row = torch.empty(N, device=DEV)
        alloc = AllocationArgs(N, 0.37, mult, 8, 2.25, sens_row)
        mn, mx = ext_minimax.minimax(rows)
        torch.cuda.manual_seed(11)
        packed, bits, scale, mn_out = ext_q.quantize_activation_device(rows, N, (mn, mx) if known else None, alloc)
        torch.cuda.manual_seed(11)
        sens_ref, bits_ref, prefix_ref = ext_cp.allocate_bits_device(mn, mx, N, 0.37, mult, 8, int(2.25 * N))
        ext_q.attach_bits_total(bits_ref, alloc.total, prefix_ref)
        packed_ref, scale_ref = ext_q.pack_mixed_precision(rows.view(N, G, 256), mn.view(N, G, 1), mx.view(N, G, 1),
                                                           bits_ref, True)
        assert torch.equal(bits, bits_ref) and int(bits.sum()) == alloc.total == int(2.25 * N)
        assert torch.equal(ext_q._bits_info(bits)[1], prefix_ref)
        assert torch.equal(sens_row, sens_ref) and torch.equal(mn_out, mn)
        assert torch.equal(packed, packed_ref) and torch.equal(scale, scale_ref)


def test_one_call_entry_points_reject_what_their_steps_reject():
    from actnn_amd import _lib
    lib = _lib.load()
    N, G = 4, 2
    rows = torch.randn(N * G, 256, device=DEV)
    mn, mx = torch.empty(N * G, device=DEV), torch.empty(N * G, device=DEV)
    sens, bits, prefix = torch.empty(N, device=DEV), torch.empty(N, dtype=torch.int32, device=DEV), torch.empty(N + 1, dtype=torch.int32, device=DEV)
    scale, packed = torch.empty(N * G, device=DEV), torch.empty(8 * N * G * 8, dtype=torch.int32, device=DEV)

    def call(**k):
        a = dict(data=rows.data_ptr(), mn=mn.data_ptr(), mx=mx.data_ptr(), known=0, sens=sens.data_ptr(),
                 bits=bits.data_ptr(), prefix=prefix.data_ptr(), initial=8, target=2 * N, scale=scale.data_ptr(),
                 packed=packed.data_ptr(), N=N, G=G, dtype=0)
        a.update(k)
        return lib.actnn_quantize_activation(a["data"], a["mn"], a["mx"], a["known"], 1.0, None, 0, a["sens"], a["bits"],
                                             a["prefix"], a["initial"], a["target"], a["scale"], a["packed"], 1, 0,
                                             a["N"], a["G"], a["dtype"], None)
    assert call() == 0
    for bad in (dict(data=None), dict(mn=None), dict(prefix=None), dict(packed=None), dict(N=0), dict(G=0),
                dict(initial=9), dict(dtype=7), dict(data=rows.data_ptr() + 4)):
        assert call(**bad) != 0, bad
    # batch norm: every output is required, whole groups of 256 only
    x = torch.randn(4, 8, 8, 8, device=DEV)
    y = torch.empty_like(x)
    ws_bytes = lib.actnn_batch_norm_workspace_bytes(4, 8, 64, 0, 0)
    ws = torch.empty(ws_bytes // 4, device=DEV)
    sm, si = torch.empty(8, device=DEV), torch.empty(8, device=DEV)

    def bn(**k):
        a = dict(y=y.data_ptr(), mn=mn.data_ptr(), packed=packed.data_ptr(), HW=64)
        a.update(k)
        return lib.actnn_batch_norm_forward_quantize(
            x.data_ptr(), None, None, None, None, a["y"], sm.data_ptr(), si.data_ptr(), a["mn"], mx.data_ptr(),
            ws.data_ptr(), ws_bytes, 1.0, None, 0, sens.data_ptr(), bits.data_ptr(), prefix.data_ptr(), 8, 2 * N,
            scale.data_ptr(), a["packed"], 1, 0, a.get("mask"), None, None, a.get("residual"), 4, 8, a["HW"], 0.1,
            1e-5, 0, 0, None)
    assert bn() == 0
    for bad in (dict(y=None), dict(mn=None), dict(packed=None), dict(HW=63), dict(mask=packed.data_ptr()), dict(residual=x.data_ptr())):
        assert bn(**bad) != 0, bad
    torch.cuda.synchronize()
