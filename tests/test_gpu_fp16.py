"""GPU parity of the IEEE-half path (the reference's own reduced precision: ``--fp16`` makes ``params_dtype``
torch.half, Merak/merak_args/args.py:584-585) through the C ABI: linears forward / backward with their fused
epilogues, activation backward, embedding gradient, cross entropy, and a small model end to end.

Tolerance 2e-3 relative (norm-wise) against the fp32 oracle on the same fp16 inputs: fp16 carries 11 bits of
mantissa against bf16's 8, products are accumulated in fp32, results rounded once.
"""
import pytest
import torch
import torch.nn.functional as F

from merak_amd import mpu, ops, set_args
from oracle import tp_reference as R

pytestmark = pytest.mark.gpu
TOL_F16 = 2e-3
H = torch.float16


def rel(got, ref):
    got, ref = got.detach().double().cpu(), ref.detach().double().cpu()
    return ((got - ref).norm() / ref.norm().clamp_min(1e-300)).item()


def gen(seed):
    return torch.Generator().manual_seed(9000 + seed)


def _inputs(m, n, k, seed):
    x = torch.randn(m, k, generator=gen(seed)).to(H)
    w = (torch.randn(n, k, generator=gen(seed + 1)) * 0.02).to(H)
    b = (torch.randn(n, generator=gen(seed + 2)) * 0.02).to(H)
    dy = (torch.randn(m, n, generator=gen(seed + 3)) * 0.1).to(H)
    return x, w, b, dy


@pytest.mark.parametrize("m,n,k", [(512, 6144, 4096), (256, 4096, 14336), (1024, 3072, 768), (300, 520, 136),
                                   (64, 50, 27), (1, 8, 8), (257, 255, 72)])     # MFMA kernel and the general one
def test_linear_fwd_bwd_fp16(gpu, m, n, k):
    x, w, b, dy = _inputs(m, n, k, 1)
    xf, wf, bf, dyf = x.float(), w.float(), b.float(), dy.float()
    y, _ = ops.linear_fwd(x.to(gpu), w.to(gpu), b.to(gpu), ops.EPI_BIAS)
    assert y.dtype == H and rel(y, R.column_parallel_linear_forward(xf, wf, bf)[0]) < TOL_F16
    y0, _ = ops.linear_fwd(x.to(gpu), w.to(gpu), None, ops.EPI_NONE)
    assert rel(y0, R.row_parallel_linear_forward(xf, wf, None)[0]) < TOL_F16
    rdx, rdw, rdb = R.linear_backward(xf, wf, dyf, True)
    assert rel(ops.linear_dgrad(dy.to(gpu), w.to(gpu)), rdx) < TOL_F16
    dw, db = ops.linear_wgrad(dy.to(gpu), x.to(gpu), True)
    assert dw.dtype == H and db.dtype == H and rel(dw, rdw) < TOL_F16 and rel(db, rdb) < TOL_F16
    acc, accb = torch.ones(n, k, device=gpu), torch.ones(n, device=gpu)          # fp32 main gradients
    ops.linear_wgrad(dy.to(gpu), x.to(gpu), True, dw=acc, db=accb, accumulate=True)
    assert rel(acc - 1, rdw) < 1e-3 and rel(accb - 1, rdb) < 1e-3


@pytest.mark.parametrize("m,n,k", [(512, 3072, 768), (100, 260, 72)])
def test_gelu_and_swiglu_epilogues_fp16(gpu, m, n, k):
    x, w, b, dy = _inputs(m, n, k, 5)
    pre = F.linear(x.float(), w.float(), b.float()).to(H).float()      # the activation sees the rounded value
    y, act = ops.linear_fwd(x.to(gpu), w.to(gpu), b.to(gpu), ops.EPI_BIAS_GELU, want_pre=True)
    assert rel(y, pre) < TOL_F16 and rel(act, R.gelu_new(pre)) < TOL_F16
    dpre = ops.activation_bwd(dy.to(gpu), y, ops.EPI_BIAS_GELU)
    assert rel(dpre, dy.float() * R.gelu_new_grad(y.float().cpu())) < TOL_F16
    pre2 = F.linear(x.float(), w.float()).to(H).float()
    y2, act2 = ops.linear_fwd(x.to(gpu), w.to(gpu), None, ops.EPI_SWIGLU, want_pre=True)
    assert act2.shape == (m, n // 2) and rel(act2, R.swiglu(pre2)) < TOL_F16
    dact = dy[:, : n // 2].contiguous()
    d2 = ops.activation_bwd(dact.to(gpu), y2, ops.EPI_SWIGLU)
    assert rel(d2, R.swiglu_backward(dact.float(), y2.float().cpu())) < TOL_F16


@pytest.mark.parametrize("n,v", [(64, 50257), (33, 1000), (16, 128256)])
def test_cross_entropy_fp16(gpu, n, v):
    g = gen(9)
    logits = (torch.randn(n, v, generator=g) * 2).to(H)
    t = torch.randint(0, v, (n,), generator=g)
    t[0] = -100                                                      # not an ignore index in the reference
    go = torch.rand(n, generator=g) + 0.5
    ref_loss, ref_grad = R.cross_entropy_fp32(logits, t, 0, go)
    lg = logits.to(gpu).requires_grad_(True)
    loss = mpu.vocab_parallel_cross_entropy(lg * 1, t.to(gpu))
    assert loss.dtype == torch.float32 and rel(loss, ref_loss) < 1e-5
    (loss * go.to(gpu)).sum().backward()
    assert lg.grad.dtype == H and rel(lg.grad, ref_grad) < TOL_F16
    # one launch for forward and backward (the trainer's mean)
    lg2 = logits.to(gpu).requires_grad_(True)
    mean = mpu.vocab_loss_fn(lg2 * 1, t.to(gpu))
    mean.backward()
    _, ref_mean_grad = R.cross_entropy_fp32(logits, t, 0, torch.full((n,), 1.0 / n))
    assert abs(mean.item() - ref_loss.mean().item()) < 1e-5 * abs(ref_loss.mean().item()) + 1e-6
    # gradients of the mean are ~1e-5 per element: fp16 stores them as subnormals, so compare after scaling
    lg3 = logits.to(gpu).requires_grad_(True)
    (mpu.vocab_loss_fn(lg3 * 1, t.to(gpu), loss_scale=1024.0) * 1024.0).backward()      # the hint, then the scaling itself
    assert rel(lg3.grad.float() / 1024.0, ref_mean_grad) < TOL_F16


def test_embedding_fp16(gpu):
    g = gen(11)
    table = torch.randn(500, 192, generator=g).to(H)
    ids = torch.randint(0, 500, (6, 40), generator=g)
    assert torch.equal(ops.embedding_gather(ids.to(gpu), table.to(gpu), 0, 500).cpu(), table[ids])
    dout = torch.randn(6, 40, 192, generator=g).to(H)
    ref = R.embedding_backward(ids, dout.float(), 500, 0, 500)
    d16 = ops.embedding_bwd(ids.to(gpu), dout.to(gpu), 500, 0, 500)
    assert d16.dtype == H and rel(d16, ref) < TOL_F16
    d32 = ops.embedding_bwd(ids.to(gpu), dout.to(gpu), 500, 0, 500, dtype=torch.float32)
    assert rel(d32, ref) < 1e-5


def test_fp16_params_dtype_model_trains_like_stock_torch(gpu):
    """``params_dtype = torch.half`` (what ``--fp16`` sets): embedding -> column(gelu_new) -> row -> LM head ->
    loss, one scaled step, against stock torch in fp32 on the same fp16-rounded parameters."""
    set_args(use_cpu_initialization=True, params_dtype=H)
    torch.manual_seed(13)
    init = lambda t_: torch.nn.init.normal_(t_, 0.0, 0.02)
    emb = mpu.VocabParallelEmbedding(300, 128, init_method=init)
    col = mpu.ColumnParallelLinear(128, 512, gather_output=False, init_method=init, activation="gelu_new")
    row = mpu.RowParallelLinear(512, 128, input_is_parallel=True, init_method=init)
    head = mpu.ColumnParallelLinear(128, 300, bias=False, gather_output=False, init_method=init)
    mods = torch.nn.ModuleDict({"emb": emb, "col": col, "row": row, "head": head})
    assert all(p.dtype == H for p in mods.parameters())
    ref = {k: v.detach().float().clone().requires_grad_(True) for k, v in mods.state_dict().items()}
    mods.to(gpu)
    ids = torch.randint(0, 300, (4, 9), generator=gen(14))
    labels = torch.randint(0, 300, (4, 9), generator=gen(15))
    scale = 256.0                                                            # fp16 training scales the loss
    h = emb(ids.to(gpu))
    h = h + row(col(h)[0])[0]
    loss = mpu.vocab_loss_fn(head(h), labels.to(gpu), loss_scale=scale) * scale
    loss.backward()
    hr = F.embedding(ids, ref["emb.weight"])
    hr = hr + F.linear(R.gelu_new(F.linear(hr, ref["col.weight"], ref["col.bias"])), ref["row.weight"], ref["row.bias"])
    want = F.cross_entropy(F.linear(hr, ref["head.weight"]).view(-1, 300), labels.view(-1)) * scale
    want.backward()
    assert abs(loss.item() - want.item()) < 5e-3 * abs(want.item())
    for name, p_ in mods.named_parameters():
        assert p_.grad.dtype == H and torch.isfinite(p_.grad).all(), name
        assert rel(p_.grad, ref[name].grad) < 1e-2, name                    # fp16 activations through three layers
