"""The allocation-free head entry point (fstu_head_argmax_static) against fstu_head_argmax: identical logits and picks,
through the C ABI, on two calls in a row (the second with a smaller input: the static array keeps no trace of the
first)."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _both(hip, x, W, temperature):
    lib = hip.load()
    rows, K = x.shape
    N = W.shape[0]
    dt = hip.FSTU_BF16 if x.dtype == torch.bfloat16 else hip.FSTU_F32
    st = torch.cuda.current_stream().cuda_stream
    ws = torch.zeros(16 * 64, dtype=torch.int64, device="cuda")
    tok_a = torch.full((rows, 3), -7, dtype=torch.int64, device="cuda")
    tok_b = torch.full((rows, 3), -7, dtype=torch.int64, device="cuda")
    la = torch.empty(rows, N, dtype=x.dtype, device="cuda")
    lb = torch.empty(rows, N, dtype=x.dtype, device="cuda")
    hip._check(lib.fstu_head_argmax(x.data_ptr(), K, W.data_ptr(), la.data_ptr(), N, rows, N, K, temperature, ws.data_ptr(),
                                    tok_a[:, 1].data_ptr(), 3, dt, st), "fstu_head_argmax")
    free_before = None
    for _ in range(2):      # the runtime may set up its own queues on a kernel's first launch: watch the second call
        lb.zero_()
        tok_b.fill_(-7)
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        hip._check(lib.fstu_head_argmax_static(x.data_ptr(), K, W.data_ptr(), lb.data_ptr(), N, rows, N, K, temperature,
                                               tok_b[:, 1].data_ptr(), 3, dt, st), "fstu_head_argmax_static")
        torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before, "the allocation-free entry point changed the free device memory"
    assert torch.equal(la, lb)
    assert torch.equal(tok_a, tok_b)
    assert bool((tok_b[:, [0, 2]] == -7).all()) and bool((tok_b[:, 1] >= 0).all()) and bool((tok_b[:, 1] < N).all())
    return tok_b[:, 1].clone()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_head_argmax_static_equals_head_argmax_on_two_calls_in_a_row(dtype):
    from flash_stu import _hip as hip
    g = torch.Generator().manual_seed(5)
    x1 = torch.randn(16, 768, generator=g).to(dtype).cuda()
    W1 = (torch.randn(50257, 768, generator=g) / 16).to(dtype).cuda()
    t1 = _both(hip, x1, W1, 0.8)
    # second call, smaller in every dimension: fewer rows, fewer features, shorter K
    x2 = torch.randn(3, 256, generator=g).to(dtype).cuda()
    W2 = (torch.randn(1000, 256, generator=g) / 16).to(dtype).cuda()
    W2[900] = W2[17]
    x2[0] = W2[17].float().sign().to(dtype) * 3          # tie between ids 17 and 900 is the maximum of row 0
    t2 = _both(hip, x2, W2, 1.0)
    assert int(t2[0]) == 17
    ref = (x2.float() @ W2.float().t()).to(dtype).float().argmax(-1)
    assert torch.equal(t2[1:].cpu(), ref[1:].cpu())
    assert t1.shape[0] == 16


def test_head_argmax_static_rejects_more_rows_than_the_scratch_holds():
    from flash_stu import _hip as hip
    lib = hip.load()
    x = torch.zeros(17, 64, dtype=torch.bfloat16, device="cuda")
    W = torch.zeros(32, 64, dtype=torch.bfloat16, device="cuda")
    out = torch.zeros(17, 32, dtype=torch.bfloat16, device="cuda")
    tok = torch.zeros(17, dtype=torch.int64, device="cuda")
    rc = lib.fstu_head_argmax_static(x.data_ptr(), 64, W.data_ptr(), out.data_ptr(), 32, 17, 32, 64, 1.0, tok.data_ptr(), 1,
                                     hip.FSTU_BF16, torch.cuda.current_stream().cuda_stream)
    assert rc == -3 and b"static scratch" in lib.fstu_last_error()
