"""actnn_batch_norm_forward_static - the forward batch norm whose scratch memory is a fixed device
array inside the library, for callers that cannot allocate - against actnn_batch_norm_forward with
a caller-provided workspace: bit-identical outputs, on two calls in a row, the second with a
smaller input (the array keeps the first call's contents), through the C ABI."""
import pytest
import torch

from actnn_amd import _lib
from _util import DEV

pytestmark = pytest.mark.gpu

CODE = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}


def _forward(lib, static, x, w, b, N, C, HW, channels_last, minmax):
    dev = x.device
    y = torch.empty_like(x)
    mean = torch.empty(C, device=dev)
    invstd = torch.empty(C, device=dev)
    run_mean = torch.zeros(C, device=dev)
    run_var = torch.ones(C, device=dev)
    groups = x.numel() // 256
    mn = torch.empty(groups, dtype=x.dtype, device=dev) if minmax else None
    mx = torch.empty(groups, dtype=x.dtype, device=dev) if minmax else None
    ptr = lambda t: t.data_ptr() if t is not None else None
    stream = torch.cuda.current_stream().cuda_stream
    if static:
        rc = lib.actnn_batch_norm_forward_static(
            ptr(x), ptr(w), ptr(b), ptr(run_mean), ptr(run_var), ptr(y), ptr(mean), ptr(invstd), ptr(mn), ptr(mx),
            N, C, HW, 0.1, 1e-5, CODE[x.dtype], int(channels_last), stream)
    else:
        nbytes = lib.actnn_batch_norm_workspace_bytes(N, C, HW, CODE[x.dtype], int(channels_last))
        assert nbytes > 0
        ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        rc = lib.actnn_batch_norm_forward(
            ptr(x), ptr(w), ptr(b), ptr(run_mean), ptr(run_var), ptr(y), ptr(mean), ptr(invstd), ptr(mn), ptr(mx),
            ptr(ws), nbytes, N, C, HW, 0.1, 1e-5, CODE[x.dtype], int(channels_last), stream)
    assert rc == 0, lib.actnn_strerror(rc)
    torch.cuda.synchronize()
    return [y, mean, invstd, run_mean, run_var] + ([mn, mx] if minmax else [])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("channels_last", [False, True])
def test_static_scratch_forward_matches_workspace_forward(dtype, channels_last):
    lib = _lib.load()
    torch.manual_seed(0)
    # two calls in a row on the same GPU array: a large problem, then a smaller one
    for (N, C, H), minmax in (((64, 256, 28), True), ((8, 64, 14), False), ((16, 128, 7), False)):
        HW = H * H
        x = (torch.randn(N, C, H, H, device=DEV) * 2 + 0.5).to(dtype)
        if channels_last:
            x = x.permute(0, 2, 3, 1).contiguous()       # [N, H, W, C] in memory
        w = torch.rand(C, device=DEV) + 0.5
        b = torch.randn(C, device=DEV)
        print(f"[no-alloc] {dtype} channels_last={channels_last} N={N} C={C} H={H}", flush=True)
        want = _forward(lib, False, x, w, b, N, C, HW, channels_last, minmax)
        got = _forward(lib, True, x, w, b, N, C, HW, channels_last, minmax)
        for a, e in zip(got, want):
            assert torch.equal(a, e)


def test_static_scratch_forward_allocates_nothing():
    lib = _lib.load()
    assert lib.actnn_batch_norm_forward_static_limit() > 0         # the set-up call resolves the array
    N, C, H = 32, 128, 14
    x = torch.randn(N, C, H, H, device=DEV).to(torch.bfloat16)
    w, b = torch.rand(C, device=DEV) + 0.5, torch.randn(C, device=DEV)
    y, mean, invstd = torch.empty_like(x), torch.empty(C, device=DEV), torch.empty(C, device=DEV)
    stream = torch.cuda.current_stream().cuda_stream

    def call():
        return lib.actnn_batch_norm_forward_static(
            x.data_ptr(), w.data_ptr(), b.data_ptr(), None, None, y.data_ptr(), mean.data_ptr(),
            invstd.data_ptr(), None, None, N, C, H * H, 0.1, 1e-5, 2, 0, stream)
    assert call() == 0
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    torch_alloc0, torch_reserved0 = torch.cuda.memory_allocated(), torch.cuda.memory_reserved()
    for _ in range(10):
        assert call() == 0
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0                                           # no device memory taken from the driver
    assert torch.cuda.memory_allocated() == torch_alloc0 and torch.cuda.memory_reserved() == torch_reserved0


def test_static_scratch_rejects_what_does_not_fit():
    lib = _lib.load()
    limit = lib.actnn_batch_norm_forward_static_limit()
    assert limit == 16 << 20
    N, C, HW = 64, 1 << 20, 8
    assert lib.actnn_batch_norm_workspace_bytes(N, C, HW, 2, 1) > limit      # 20 MiB
    rc = lib.actnn_batch_norm_forward_static(None, None, None, None, None, None, None, None, None, None,
                                             N, C, HW, 0.1, 1e-5, 2, 1, None)
    assert rc == -5 and b"scratch" in lib.actnn_strerror(rc)
