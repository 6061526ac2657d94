"""The entry point that allocates nothing: the greedy pick over an LM head with the library's own scratch array,
through the C ABI, against the entry point that takes a caller's workspace: same indices and the same winning
logits bit for bit, on two calls in a row, the second with a smaller input (the array keeps the first call's
contents)."""
import pytest
import torch

from merak_amd import _lib, ops

pytestmark = pytest.mark.gpu


def _both(x, w):
    lib = _lib.lib()
    B, K = x.shape
    N = w.shape[0]
    dev = x.device
    stream = torch.cuda.current_stream(dev).cuda_stream
    idx_a = torch.full((B,), -1, dtype=torch.int64, device=dev)
    val_a = torch.zeros(B, dtype=torch.float32, device=dev)
    _lib.check(lib.mtp_gemv_argmax_noalloc(x.data_ptr(), w.data_ptr(), idx_a.data_ptr(), val_a.data_ptr(), B, N, K,
                                           _lib.MTP_BF16, stream), "mtp_gemv_argmax_noalloc")
    need = lib.mtp_gemv_argmax_workspace_bytes(B, N, K)
    ws = torch.empty(need, dtype=torch.uint8, device=dev)
    idx_b = torch.full((B,), -1, dtype=torch.int64, device=dev)
    val_b = torch.zeros(B, dtype=torch.float32, device=dev)
    _lib.check(lib.mtp_gemv_argmax(x.data_ptr(), w.data_ptr(), idx_b.data_ptr(), val_b.data_ptr(), ws.data_ptr(), need,
                                   B, N, K, _lib.MTP_BF16, stream), "mtp_gemv_argmax")
    torch.cuda.synchronize()
    return idx_a, val_a, idx_b, val_b


def test_gemv_argmax_noalloc_matches_the_workspace_entry_point(gpu):
    g = torch.Generator().manual_seed(77)
    lib = _lib.lib()
    assert lib.mtp_gemv_argmax_noalloc_max_bytes() == 4 << 20
    for (b, n, k) in ((32, 128256, 4096), (5, 1000, 512)):        # the second call is the smaller one
        x = torch.randn(b, k, generator=g).bfloat16().to(gpu)
        w = (torch.randn(n, k, generator=g) * 0.02).bfloat16().to(gpu)
        idx_a, val_a, idx_b, val_b = _both(x, w)
        assert torch.equal(idx_a, idx_b) and torch.equal(val_a, val_b)
        ref = torch.nn.functional.linear(x.float(), w.float()).argmax(-1)
        assert (idx_a == ref).float().mean() > 0.9                 # bf16 products: near ties may differ from fp32
    # a shape beyond the library's array is refused with a clear error, nothing is launched
    rc = lib.mtp_gemv_argmax_noalloc(x.data_ptr(), w.data_ptr(), idx_a.data_ptr(), None, 32, 1 << 20, 512, _lib.MTP_BF16, None)
    assert rc == -4 and b"scratch" in lib.mtp_last_error()
