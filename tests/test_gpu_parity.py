"""Parity of the HIP path with the CPU oracle, through the C ABI (ctypes) on an MI355X.

Tolerances (relative error = ||got - ref|| / ||ref|| unless stated):
  embedding gather, argmax indices ........ bit-exact
  fp32 paths .............................. 1e-4
  bf16 GEMM outputs and gradients ......... 1e-2 against the fp32 oracle
  cross-entropy loss ...................... 1e-5 (bf16 logits are upcast; the oracle runs the reference
                                            algorithm in fp32 on the same bf16 values)
"""
import json
import os

import pytest
import torch
import torch.nn.functional as F

from merak_amd import mpu, ops, set_args
from merak_amd.inference import DecodeStep, greedy_from_logits, greedy_next_token
from oracle import tp_reference as R

pytestmark = pytest.mark.gpu
G = os.path.join(os.path.dirname(__file__), "golden")

TOL_F32, TOL_BF16, TOL_LOSS = 1e-4, 1e-2, 1e-5


def rel(got, ref):
    got, ref = got.detach().double().cpu(), ref.detach().double().cpu()
    return ((got - ref).norm() / ref.norm().clamp_min(1e-300)).item()


def gen(seed):
    return torch.Generator().manual_seed(1234 + seed)


# =============================================================================== cross entropy
@pytest.mark.parametrize("case", json.load(open(os.path.join(G, "ce_small.json"))),
                         ids=lambda c: f"start{c['vocab_start']}_t{c['target']}")
@pytest.mark.parametrize("dtype", [torch.float32])
def test_ce_golden_vectors(gpu, case, dtype):
    x = torch.tensor(case["logits"], dtype=dtype, device=gpu)
    t = torch.tensor(case["target"], device=gpu)
    loss, m, s, pred = ops.vocab_ce_fwd(x, t, case["vocab_start"])
    assert rel(loss, torch.tensor(case["loss"])) < TOL_LOSS
    g = torch.tensor(case["grad_output"], dtype=torch.float32, device=gpu)
    ops.vocab_ce_bwd_(x, t, m, s, g, case["vocab_start"])
    assert rel(x, torch.tensor(case["grad"])) < TOL_F32


@pytest.mark.parametrize("dtype,n,v", [
    (torch.float32, 64, 50257),     # GPT-2 vocab: rows are not 16-byte aligned
    (torch.bfloat16, 64, 128256),   # Llama-3 vocab
    (torch.float32, 7, 1), (torch.float32, 3, 5), (torch.bfloat16, 5, 9), (torch.bfloat16, 4, 1031),
    (torch.float32, 2, 2048 + 3), (torch.bfloat16, 1, 40000),
])
def test_ce_forward_backward_vs_oracle(gpu, dtype, n, v):
    x = torch.randn(n, v, generator=gen(1)).to(dtype)
    t = torch.randint(0, v, (n,), generator=gen(2))
    t[torch.randperm(n, generator=gen(3))[: max(1, n // 20)]] = -100      # 5% "ignore" labels
    g = torch.full((n,), 1.0 / n)
    ref_loss, ref_grad = R.cross_entropy_fp32(x, t, 0, g)
    xg = x.to(gpu)
    loss, m, s, pred = ops.vocab_ce_fwd(xg, t.to(gpu), 0)
    assert torch.equal(xg.cpu(), x), "forward must not modify the logits"
    # 1e-5 relative; a vocabulary of one gives an exactly zero loss, so an absolute floor of 1e-6 is allowed
    assert (loss.cpu() - ref_loss).abs().max() <= TOL_LOSS * max(ref_loss.abs().max().item(), 0.1)
    assert rel(loss, ref_loss) < TOL_LOSS or v == 1
    assert torch.equal(m.cpu(), x.float().max(-1).values)
    out = ops.vocab_ce_bwd_(xg, t.to(gpu), m, s, g.to(gpu), 0)
    assert out.data_ptr() == xg.data_ptr(), "gradient must reuse the logits storage"
    assert rel(xg, ref_grad) < (TOL_F32 if dtype == torch.float32 else TOL_BF16)


def test_ce_autograd_function_matches_reference_semantics(gpu):
    n, v = 48, 50257
    x = torch.randn(4, 12, v, generator=gen(4))
    t = torch.randint(0, v, (4, 12), generator=gen(5))
    t[0, 0] = -100
    ref_loss, ref_grad = R.cross_entropy_fp32(x.view(n, v), t.view(n), 0, torch.full((n,), 1.0 / n))
    xg = x.to(gpu).requires_grad_(True)
    logits = xg * 1.0                                   # a non-leaf, as the LM head's output would be
    loss = mpu.vocab_parallel_cross_entropy(logits, t.to(gpu))
    assert loss.shape == t.shape and loss.dtype == torch.float32
    torch.mean(loss.view(-1)).backward()                # merak_trainer.py:323-325
    assert rel(loss.view(-1), ref_loss) < TOL_LOSS
    assert rel(xg.grad.view(n, v), ref_grad) < TOL_F32
    # opt-in: reproduce the reference's side effect (caller's logits end up holding the softmax)
    y = x.to(gpu).clone()
    l2 = mpu.vocab_parallel_cross_entropy(y, t.to(gpu), materialize_softmax=True)
    assert rel(y.view(n, v), torch.softmax(x.view(n, v), -1)) < TOL_F32 and rel(l2.view(-1), ref_loss) < TOL_LOSS


@pytest.mark.parametrize("v", [4096, 40000])   # rows walked in steps / rows held in registers by the backward
def test_ce_bf16_loss_dtype_flag_and_materialized_backward(gpu, v):
    n = 16
    x = torch.randn(n, v, generator=gen(6)).bfloat16()
    t = torch.randint(0, v, (n,), generator=gen(7))
    g = torch.rand(n, generator=gen(8))
    ref_loss, ref_grad = R.cross_entropy_fp32(x, t, 0, g)
    xg = x.to(gpu).requires_grad_(True)
    lg = xg * 1
    loss = mpu.vocab_parallel_cross_entropy(lg, t.to(gpu), loss_in_logits_dtype=True, materialize_softmax=True)
    assert loss.dtype == torch.bfloat16                 # cross_entropy.py:77 returns the logits dtype
    (loss.float() * g.to(gpu)).sum().backward()
    assert rel(xg.grad, ref_grad) < 2 * TOL_BF16        # softmax was rounded to bf16 once more on the way


def test_ce_one_rank_share_combines_to_full(gpu):
    """8 vocab slices, each through the kernel with its [start, end); MAX/SUM/SUM on the host."""
    n, v, p = 32, 8 * 1002, 8
    x = torch.randn(n, v, generator=gen(9)).bfloat16()
    t = torch.randint(0, v, (n,), generator=gen(10))
    t[3] = -100
    full_loss, full_grad = R.cross_entropy_fp32(x, t, 0, torch.ones(n))
    mpu.set_model_parallel_world_size(p)
    parts, slices = [], []
    for r in range(p):
        mpu.set_model_parallel_rank(r)
        sl = x[:, r * 1002:(r + 1) * 1002].contiguous().to(gpu)
        m, s, pr = mpu.vocab_parallel_cross_entropy_partials(sl, t.to(gpu))
        om, os_, opr, inr = R.cross_entropy_partials(x[:, r * 1002:(r + 1) * 1002], t, r * 1002)
        assert torch.equal(m.cpu(), om) and rel(s, os_) < TOL_LOSS and torch.equal(pr.cpu(), opr)
        parts.append((m.cpu(), s.cpu(), pr.cpu(), inr))
        slices.append(sl)
    loss, gm, gs = R.combine_partials(*zip(*parts))
    assert rel(loss, full_loss) < TOL_LOSS
    for r in range(p):
        mpu.set_model_parallel_rank(r)
        mpu.vocab_parallel_cross_entropy_backward_(slices[r], t.to(gpu), gm.to(gpu), gs.to(gpu), torch.ones(n, device=gpu))
        assert rel(slices[r], full_grad[:, r * 1002:(r + 1) * 1002]) < TOL_BF16


def test_ce_empty_and_errors(gpu):
    loss, *_ = ops.vocab_ce_fwd(torch.empty(0, 17, device=gpu), torch.empty(0, dtype=torch.int64, device=gpu), 0)
    assert loss.numel() == 0
    with pytest.raises(TypeError):
        ops.vocab_ce_fwd(torch.randn(2, 4, device=gpu), torch.zeros(2, dtype=torch.int32, device=gpu), 0)
    with pytest.raises(ValueError, match="contiguous"):
        ops.vocab_ce_fwd(torch.randn(4, 8, device=gpu)[:, ::2], torch.zeros(4, dtype=torch.int64, device=gpu), 0)
    with pytest.raises(TypeError):
        ops.vocab_ce_fwd(torch.randn(2, 4, device=gpu).double(), torch.zeros(2, dtype=torch.int64, device=gpu), 0)


def test_ce_full_size_llama_vocab(gpu):
    """[8192, 128256] bf16 with 5% -100 labels: oracle on a sample of rows; whole-tensor properties."""
    n, v = 8192, 128256
    x = torch.empty(n, v, dtype=torch.bfloat16, device=gpu).normal_(generator=torch.Generator(device=gpu).manual_seed(1238))
    t = torch.randint(0, v, (n,), generator=gen(11))
    t[torch.randperm(n, generator=gen(12))[: n // 20]] = -100
    tg = t.to(gpu)
    loss, m, s, pred = ops.vocab_ce_fwd(x, tg, 0)
    rows = torch.randperm(n, generator=gen(13))[:48]
    rows[0] = (t == -100).nonzero()[0, 0]
    xs = x[rows.to(gpu)].cpu()
    g = torch.full((n,), 1.0 / n)
    ref_loss, ref_grad = R.cross_entropy_fp32(xs, t[rows], 0, g[rows])
    assert rel(loss.cpu()[rows], ref_loss) < TOL_LOSS
    assert bool(torch.isfinite(loss).all()) and float(loss.min()) > 0
    ops.vocab_ce_bwd_(x, tg, m, s, g.to(gpu), 0)
    assert rel(x[rows.to(gpu)], ref_grad) < TOL_BF16
    # each gradient row sums to g_i * (1 - [target in range])  (softmax sums to one, minus the one-hot)
    rowsum = x.float().sum(-1).cpu() * n
    expect = (t == -100).float()
    assert (rowsum - expect).abs().max() < 0.05


def test_ce_full_size_gpt2_vocab(gpu):
    """[8192, 50257] fp32 (rows not 16-byte aligned), uniform labels: oracle on a sample of rows; every gradient
    row sums to zero (softmax sums to one, minus the one-hot)."""
    n, v = 8192, 50257
    x = torch.empty(n, v, device=gpu).normal_(generator=torch.Generator(device=gpu).manual_seed(1239))
    t = torch.randint(0, v, (n,), generator=gen(14))
    tg = t.to(gpu)
    loss, m, s, pred = ops.vocab_ce_fwd(x, tg, 0)
    rows = torch.randperm(n, generator=gen(15))[:48]
    xs = x[rows.to(gpu)].cpu()
    g = torch.full((n,), 1.0 / n)
    ref_loss, ref_grad = R.cross_entropy_fp32(xs, t[rows], 0, g[rows])
    assert rel(loss.cpu()[rows], ref_loss) < TOL_LOSS
    assert bool(torch.isfinite(loss).all()) and float(loss.min()) > 0
    ops.vocab_ce_bwd_(x, tg, m, s, g.to(gpu), 0)
    assert rel(x[rows.to(gpu)], ref_grad) < TOL_F32
    assert (x.double().sum(-1).cpu() * n).abs().max() < 1e-3


@pytest.mark.parametrize("dtype,n,v", [
    (torch.float32, 64, 50257), (torch.bfloat16, 64, 128256), (torch.float32, 7, 1), (torch.float32, 3, 5),
    (torch.bfloat16, 5, 9), (torch.bfloat16, 4, 1031), (torch.float32, 2, 2048 + 3), (torch.bfloat16, 3, 40000),
    (torch.float32, 2, 81920), (torch.bfloat16, 2, 163840),     # the longest rows that stay in registers
    (torch.bfloat16, 3, 8192 * 4 + 5), (torch.float32, 5, 4096 * 4 + 1), (torch.bfloat16, 6, 8192 * 12 - 3),
])
def test_ce_one_launch_forward_backward(gpu, dtype, n, v):
    """mtp_vocab_ce_fwd_bwd against the oracle and against the two-launch path on the same inputs."""
    x = torch.randn(n, v, generator=gen(14)).to(dtype)
    t = torch.randint(0, v, (n,), generator=gen(15))
    t[torch.randperm(n, generator=gen(16))[: max(1, n // 20)]] = -100
    gr = torch.rand(n, generator=gen(17)) + 0.5
    scale = 0.25
    ref_loss, ref_grad = R.cross_entropy_fp32(x, t, 0, gr * scale)
    tol_g = TOL_F32 if dtype == torch.float32 else TOL_BF16
    a, b = x.to(gpu), x.to(gpu)
    loss, m, s, pred = ops.vocab_ce_fwd_bwd_(a, t.to(gpu), 0, gr.to(gpu), scale)
    loss2, m2, s2, pred2 = ops.vocab_ce_fwd(b, t.to(gpu), 0)
    ops.vocab_ce_bwd_(b, t.to(gpu), m2, s2, (gr * scale).to(gpu), 0)
    assert (loss.cpu() - ref_loss).abs().max() <= TOL_LOSS * max(ref_loss.abs().max().item(), 0.1)
    assert torch.equal(m, m2) and torch.equal(pred, pred2) and rel(s, s2) < TOL_LOSS
    assert rel(a, ref_grad) < tol_g and rel(a, b) < tol_g
    # no per-row gradient: g = grad_scale for every row
    c = x.to(gpu)
    ops.vocab_ce_fwd_bwd_(c, t.to(gpu), 0, None, 1.0 / n)
    assert rel(c, R.cross_entropy_fp32(x, t, 0, torch.full((n,), 1.0 / n))[1]) < tol_g


@pytest.mark.parametrize("dtype,n,v", [(torch.bfloat16, 700, 40000), (torch.float32, 523, 4 * 4096 + 1),
                                        (torch.bfloat16, 257, 8192 * 8 - 3), (torch.float16, 300, 32768)])
def test_ce_row_kernels_walk_their_rows(gpu, set_tuning, dtype, n, v):
    """The register-resident kernels (one-launch forward+backward, row backward) either take one row per workgroup
    or walk rows b, b + 256, ... as persistent workgroups, asking for the next row behind the stores of the current
    one (the default depends on the kernel and the element size; MTP_CE_PERSIST forces either): more rows than
    workgroups (two or three per workgroup, the last round part empty), rows whose 16-byte alignment changes from
    row to row.  Against the oracle, and the same bits in every form."""
    x = torch.randn(n, v, generator=gen(114)).to(dtype)
    t = torch.randint(0, v, (n,), generator=gen(115))
    t[torch.randperm(n, generator=gen(116))[: n // 20]] = -100
    gr = torch.rand(n, generator=gen(117)) + 0.5
    ref_loss, ref_grad = R.cross_entropy_fp32(x, t, 0, gr * 0.5)
    tol_g = TOL_F32 if dtype == torch.float32 else TOL_BF16
    outs = []
    for persist in (None, 0, 1, 2):
        set_tuning("MTP_CE_PERSIST", persist)
        a, b = x.to(gpu), x.to(gpu)
        loss, m, s, pred = ops.vocab_ce_fwd_bwd_(a, t.to(gpu), 0, gr.to(gpu), 0.5)
        _, m2, s2, _ = ops.vocab_ce_fwd(b, t.to(gpu), 0)
        ops.vocab_ce_bwd_(b, t.to(gpu), m2, s2, (gr * 0.5).to(gpu), 0)
        outs.append((a, b, loss, m, s, pred))
    a, b, loss = outs[0][:3]
    assert (loss.cpu() - ref_loss).abs().max() <= TOL_LOSS * max(ref_loss.abs().max().item(), 0.1)
    assert rel(a, ref_grad) < tol_g and rel(b, ref_grad) < tol_g
    for other in outs[1:]:
        for p, q in zip(outs[0], other):
            assert torch.equal(p, q)


def test_ce_one_launch_vocab_slice_and_limits(gpu):
    n, v, start = 8, 1002, 3006
    x = torch.randn(n, v, generator=gen(18)).bfloat16()
    t = torch.randint(0, 8 * v, (n,), generator=gen(19))
    t[0], t[1] = start, start + v - 1                    # first and last id of this slice
    om, os_, opr, inr = R.cross_entropy_partials(x, t, start)
    xg = x.to(gpu)
    _, m, s, pr = ops.vocab_ce_fwd_bwd_(xg, t.to(gpu), start, None, 1.0)
    assert torch.equal(m.cpu(), om) and rel(s, os_) < TOL_LOSS and torch.equal(pr.cpu(), opr)
    sm = torch.softmax(x.float(), -1)
    onehot = torch.zeros(n, v)
    onehot[inr, (t - start)[inr]] = 1.0
    assert rel(xg, sm - onehot) < TOL_BF16
    # rows too long for the registers: the C entry point says so, the module falls back to two launches
    for dtype in (torch.float32, torch.bfloat16):
        lim = ops.vocab_ce_fused_max_vocab(dtype)
        assert lim == {torch.float32: 81920, torch.bfloat16: 163840}[dtype]
        big = torch.zeros(1, lim + 1, dtype=dtype, device=gpu)
        with pytest.raises(RuntimeError, match="does not fit"):
            ops.vocab_ce_fwd_bwd_(big, torch.zeros(1, dtype=torch.int64, device=gpu), 0)
    big = torch.randn(2, 81920 + 7, generator=gen(20))
    bt = torch.tensor([5, 81920])
    bg = big.to(gpu).requires_grad_(True)
    mpu.vocab_loss_fn(bg * 1.0, bt.to(gpu)).backward()
    assert rel(bg.grad, R.cross_entropy_fp32(big, bt, 0, torch.full((2,), 0.5))[1]) < TOL_F32
    empty = ops.vocab_ce_fwd_bwd_(torch.empty(0, 17, device=gpu), torch.empty(0, dtype=torch.int64, device=gpu), 0)
    assert empty[0].numel() == 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_ce_vocab_loss_fn_autograd(gpu, dtype):
    """The trainer's mean loss (merak_trainer.py:313-326) through the one-launch kernel: the assumed upstream
    gradient 1/n is what autograd delivers; a different one (loss scaling, per-position masks) is corrected."""
    n, v = 48, 50257
    x = torch.randn(4, 12, v, generator=gen(21)).to(dtype)
    t = torch.randint(0, v, (4, 12), generator=gen(22))
    t[0, 0] = -100
    tol_g = TOL_F32 if dtype == torch.float32 else TOL_BF16
    ref_loss, ref_grad = R.cross_entropy_fp32(x.view(n, v), t.view(n), 0, torch.full((n,), 1.0 / n))
    xg = x.to(gpu).requires_grad_(True)
    loss = mpu.vocab_loss_fn((xg * 1.0,), (t.to(gpu),))
    assert loss.dim() == 0 and abs(loss.item() - ref_loss.mean().item()) < TOL_LOSS * ref_loss.mean().item() * 10
    loss.backward()
    assert rel(xg.grad.view(n, v), ref_grad) < tol_g
    # upstream gradient differs from the assumption: scaled loss and a per-position mask
    mask = (torch.rand(4, 12, generator=gen(23)) > 0.3).float()
    xg2 = x.to(gpu).requires_grad_(True)
    losses = mpu.vocab_parallel_cross_entropy(xg2 * 1.0, t.to(gpu), fused_backward_scale=1.0 / n)
    assert rel(losses.view(-1), ref_loss) < TOL_LOSS
    (1024.0 * (losses * mask.to(gpu)).sum() / mask.sum()).backward()
    ref2 = R.cross_entropy_fp32(x.view(n, v), t.view(n), 0, 1024.0 * mask.view(n) / mask.sum())[1]
    assert rel(xg2.grad.view(n, v), ref2) < 2 * tol_g       # bf16: rounded once more by the rescale
    assert bool((xg2.grad.view(n, v)[mask.view(n) == 0] == 0).all())


def test_ce_vocab_loss_fn_leaves_logits_alone_without_grad(gpu):
    """Evaluation: under no_grad, or for logits that take no gradient, the loss is the same and the logits the
    caller gets back are still logits (the reference's eval_batch returns them after the loss)."""
    n, v = 37, 5000
    x = torch.randn(n, v, generator=gen(90)).bfloat16()
    t = torch.randint(0, v, (n,), generator=gen(91))
    ref, _ = R.cross_entropy_fp32(x, t, 0, torch.full((n,), 1.0 / n))
    for mode in ("no_grad", "no_requires_grad"):
        xg = x.to(gpu)
        if mode == "no_grad":
            xg.requires_grad_(True)
            with torch.no_grad():
                loss = mpu.vocab_loss_fn((xg, None), t.to(gpu))
        else:
            loss = mpu.vocab_loss_fn(xg, t.to(gpu))
        assert abs(loss.item() - ref.mean().item()) < 1e-4
        assert torch.equal(xg.detach().cpu(), x), mode
    # training: the forward consumes the logits, and autograd knows they changed
    xg = x.to(gpu).requires_grad_(True)
    y = xg * 1.0
    v0 = y._version
    mpu.vocab_loss_fn(y, t.to(gpu)).backward()
    assert y._version > v0 and not torch.equal(y.detach().cpu(), x)


def test_ce_one_launch_full_size_llama_vocab(gpu):
    n, v = 8192, 128256
    x = torch.empty(n, v, dtype=torch.bfloat16, device=gpu).normal_(generator=torch.Generator(device=gpu).manual_seed(1239))
    t = torch.randint(0, v, (n,), generator=gen(24))
    t[torch.randperm(n, generator=gen(25))[: n // 20]] = -100
    rows = torch.randperm(n, generator=gen(26))[:48]
    rows[0] = (t == -100).nonzero()[0, 0]
    xs = x[rows.to(gpu)].cpu()
    ref_loss, ref_grad = R.cross_entropy_fp32(xs, t[rows], 0, torch.full((48,), 1.0 / n))
    loss, m, s, pred = ops.vocab_ce_fwd_bwd_(x, t.to(gpu), 0, None, 1.0 / n)
    assert rel(loss.cpu()[rows], ref_loss) < TOL_LOSS
    assert bool(torch.isfinite(loss).all()) and float(loss.min()) > 0
    assert rel(x[rows.to(gpu)], ref_grad) < TOL_BF16
    rowsum = x.float().sum(-1).cpu() * n
    assert (rowsum - (t == -100).float()).abs().max() < 0.05
    before = x[:64].clone()
    ops.vocab_ce_rescale_(x, torch.full((n,), 1.0 / n, device=gpu), 1.0 / n)      # equal: must not touch anything
    assert torch.equal(x[:64], before)


@pytest.mark.parametrize("dtype,n,k,v,chunk,has_bias", [(torch.bfloat16, 300, 256, 5000, 128, False),
                                                        (torch.bfloat16, 1023, 512, 32000, 512, True),
                                                        (torch.float32, 96, 64, 1000, 40, True)])
def test_lm_head_cross_entropy_chunked(gpu, dtype, n, k, v, chunk, has_bias):
    """LM head + cross entropy per row chunk (the full logits never exist) against the oracle's F.linear
    followed by the reference cross entropy, forward and both of the head's gradients."""
    set_args(use_cpu_initialization=True, params_dtype=dtype)
    torch.manual_seed(4)
    head = mpu.ColumnParallelLinear(k, v, bias=has_bias, gather_output=False,
                                    init_method=lambda t: torch.nn.init.normal_(t, 0.0, 0.05))
    if has_bias:
        with torch.no_grad():
            head.bias.normal_(0, 0.05)
    h = torch.randn(3, n // 3, k, generator=gen(110)).to(dtype)
    t = torch.randint(0, v, (3, n // 3), generator=gen(111))
    t[0, 0] = -100
    hr = h.float().clone().requires_grad_(True)
    wr = head.weight.detach().float().requires_grad_(True)
    br = head.bias.detach().float().requires_grad_(True) if has_bias else None
    logits = R.column_parallel_linear_forward(hr, wr, br)[0]
    if dtype == torch.bfloat16:                    # the head stores bf16 logits before the loss reads them
        logits = logits + (logits.detach().bfloat16().float() - logits.detach())
    ref_loss, _ = R.cross_entropy_fp32(logits.detach().reshape(n, v), t.view(-1), 0, torch.ones(n))
    lse = torch.logsumexp(logits.reshape(n, v), -1)
    inr = t.view(-1) >= 0
    picked = logits.reshape(n, v)[torch.arange(n), t.view(-1).clamp_min(0)]
    # out-of-range targets: loss = lse - max, and the reference's backward (cross_entropy.py:92-104) is softmax * g,
    # i.e. the max term is a constant there
    closed = torch.where(inr, lse - picked, lse - logits.reshape(n, v).max(-1).values.detach())
    assert rel(closed.detach(), ref_loss) < 1e-5
    (3.0 * closed.mean()).backward()
    head.to(gpu)
    hg = h.to(gpu).requires_grad_(True)
    losses = mpu.lm_head_cross_entropy(hg, head, t.to(gpu), loss_scale=3.0, chunk_rows=chunk)
    assert losses.shape == t.shape and losses.dtype == torch.float32
    assert rel(losses.view(-1), ref_loss) < (TOL_LOSS if dtype == torch.float32 else 1e-4)
    (3.0 * losses.mean()).backward()
    tol = TOL_F32 * 5 if dtype == torch.float32 else 2 * TOL_BF16
    assert rel(hg.grad, hr.grad) < tol and rel(head.weight.grad, wr.grad) < tol
    if has_bias:
        assert rel(head.bias.grad, br.grad) < tol
    # another common factor is rescaled in backward; per-position weights are refused
    hg2 = h.to(gpu).requires_grad_(True)
    head.weight.grad = None
    l2 = mpu.lm_head_cross_entropy(hg2, head, t.to(gpu), chunk_rows=chunk)
    (5.0 * l2.sum()).backward(retain_graph=True)
    assert rel(hg2.grad, hr.grad * (5.0 * n / 3.0)) < tol
    hg2.grad = None
    (5.0 * l2.sum()).backward()                    # a second pass over the retained graph scales once, not twice
    assert rel(hg2.grad, hr.grad * (5.0 * n / 3.0)) < tol
    with pytest.raises(RuntimeError, match="one upstream gradient"):
        l3 = mpu.lm_head_cross_entropy(h.to(gpu).requires_grad_(True), head, t.to(gpu), chunk_rows=chunk)
        (l3.view(-1) * torch.arange(n, device=gpu)).sum().backward()


@pytest.mark.parametrize("accum", [None, torch.float32])
def test_lm_head_cross_entropy_many_chunks(gpu, accum):
    """32 chunks of 256 tokens: the weight gradient summed across chunks in the weight's dtype (one rounding per
    chunk, as the reference's .grad sums micro-batches) stays within twice the one-piece tolerance, and within it
    when summed in fp32; the two differ from the unfused layers only by that rounding."""
    n, k, v, chunk = 8192, 512, 2048, 256
    g = gen(120)
    h = torch.randn(n, k, generator=g).bfloat16()
    w = (torch.randn(v, k, generator=g) * 0.05).bfloat16()
    b = (torch.randn(v, generator=g) * 0.05).bfloat16()
    t = torch.randint(0, v, (n,), generator=g)
    t[::50] = -100
    hr, wr, br = h.float().requires_grad_(True), w.float().requires_grad_(True), b.float().requires_grad_(True)
    logits = F.linear(hr, wr, br)
    logits = logits + (logits.detach().bfloat16().float() - logits.detach())
    lse = torch.logsumexp(logits, -1)
    picked = logits[torch.arange(n), t.clamp_min(0)]
    closed = torch.where(t >= 0, lse - picked, lse - logits.max(-1).values.detach())
    closed.mean().backward()
    hg = h.to(gpu).requires_grad_(True)
    wg = w.to(gpu).requires_grad_(True)
    bg = b.to(gpu).requires_grad_(True)
    head = type("Head", (torch.nn.Module,), {})()
    head.weight, head.bias = wg, bg
    losses = mpu.lm_head_cross_entropy(hg, head, t.to(gpu), chunk_rows=chunk, grad_accum_dtype=accum)
    assert rel(losses, closed.detach()) < 1e-4
    losses.mean().backward()
    assert wg.grad.dtype == torch.bfloat16 and bg.grad.dtype == torch.bfloat16
    tol = 2 * TOL_BF16 if accum is None else TOL_BF16
    assert rel(hg.grad, hr.grad) < TOL_BF16 and rel(wg.grad, wr.grad) < tol and rel(bg.grad, br.grad) < tol
    # a head whose weight takes no gradient: the bias gradient alone, no weight-sized temporary
    wf = w.to(gpu)
    bg2 = b.to(gpu).requires_grad_(True)
    head.weight, head.bias = wf, bg2
    before = torch.cuda.max_memory_allocated()
    torch.cuda.reset_peak_memory_stats()
    l2 = mpu.lm_head_cross_entropy(h.to(gpu), head, t.to(gpu), chunk_rows=chunk, grad_accum_dtype=accum)
    l2.mean().backward()
    assert rel(bg2.grad, br.grad) < tol


# =============================================================================== embedding
@pytest.mark.parametrize("dtype,v,h", [(torch.bfloat16, 1000, 4096), (torch.float32, 777, 33), (torch.bfloat16, 50, 7),
                                        (torch.float32, 64, 1)])
def test_embedding_exact(gpu, dtype, v, h):
    table = torch.randn(v, h, generator=gen(20)).to(dtype)
    ids = torch.randint(0, v, (3, 11), generator=gen(21))
    out = ops.embedding_gather(ids.to(gpu), table.to(gpu), 0, v)
    assert out.shape == (3, 11, h) and torch.equal(out.cpu(), R.vocab_parallel_embedding_forward(ids, table, 0, v, 1))
    lo, hi = v // 4, v // 2                                   # one rank's slice: outside ids give exact zeros
    shard = table[lo:hi].contiguous()
    out = ops.embedding_gather(ids.to(gpu), shard.to(gpu), lo, hi)
    assert torch.equal(out.cpu(), R.vocab_parallel_embedding_forward(ids, shard, lo, hi, 4))


def test_embedding_module_forward_backward(gpu):
    set_args(use_cpu_initialization=True, params_dtype=torch.bfloat16)
    torch.manual_seed(0)
    emb = mpu.VocabParallelEmbedding(512, 64, init_method=torch.nn.init.normal_).to(gpu)
    ids = torch.randint(0, 512, (4, 33), generator=gen(22))
    ids[0, :5] = 7                                            # repeated ids accumulate
    out = emb(ids.to(gpu))
    assert torch.equal(out.cpu(), emb.weight.detach().cpu()[ids])
    dout = torch.randn(4, 33, 64, generator=gen(23)).bfloat16()
    out.backward(dout.to(gpu))
    ref = R.embedding_backward(ids, dout, 512, 0, 512)
    assert emb.weight.grad.dtype == torch.bfloat16 and rel(emb.weight.grad, ref) < TOL_BF16
    dt = ops.embedding_bwd(ids.to(gpu), dout.to(gpu), 512, 0, 512, dtype=torch.float32)
    assert dt.dtype == torch.float32 and rel(dt, ref) < TOL_F32
    empty = ops.embedding_gather(torch.empty(0, dtype=torch.int64, device=gpu), emb.weight.detach(), 0, 512)
    assert empty.shape == (0, 64)
    oob = torch.zeros(1, dtype=torch.int32, device=gpu)
    ops.embedding_gather(torch.tensor([1, 600, -3], device=gpu), emb.weight.detach(), 0, 512, oob)
    assert oob.item() == 2


@pytest.mark.parametrize("dtype,n,v,h,lo,hi", [
    (torch.bfloat16, 4096, 1000, 4096, 0, 1000),      # many repeats per id
    (torch.float32, 513, 64, 77, 0, 64),              # row length not a multiple of 4
    (torch.bfloat16, 700, 4000, 1030, 1000, 2000),    # one rank's vocabulary slice: ids outside it contribute nothing
    (torch.bfloat16, 300, 16, 8, 0, 16),
])
def test_embedding_backward_reproducible(gpu, dtype, n, v, h, lo, hi):
    ids = torch.randint(0, v, (n,), generator=gen(27))
    ids[: n // 3] = lo + 1                                     # one id carried by a third of the tokens
    dout = torch.randn(n, h, generator=gen(28)).to(dtype)
    ref = R.embedding_backward(ids, dout, hi - lo, lo, hi)
    a = ops.embedding_bwd(ids.to(gpu), dout.to(gpu), hi - lo, lo, hi, dtype=torch.float32)
    b = ops.embedding_bwd(ids.to(gpu), dout.to(gpu), hi - lo, lo, hi, dtype=torch.float32)
    assert rel(a, ref) < TOL_F32 and torch.equal(a, b), "same inputs, same bits"
    # the documented order: ascending token index in fp32; an id carried by more than 32 tokens: the same inside
    # blocks of 32 of its tokens, the block sums in ascending order inside blocks of 32 blocks, those in ascending order
    mine = (ids == lo + 1).nonzero().flatten().tolist()
    def running(rows):
        acc = torch.zeros(h)
        for r in rows:
            acc += r
        return acc
    if len(mine) > 32:
        blocks = [running([dout[i].float() for i in mine[b:b + 32]]) for b in range(0, len(mine), 32)]
        seq = running([running(blocks[b:b + 32]) for b in range(0, len(blocks), 32)])
    else:
        seq = running([dout[i].float() for i in mine])
    assert torch.equal(a[1].cpu(), seq)
    # accumulation onto an existing gradient (tied LM head), in the table's own dtype
    base = torch.randn(hi - lo, h, generator=gen(29)).to(dtype)
    tied = ops.embedding_bwd(ids.to(gpu), dout.to(gpu), hi - lo, lo, hi, out=base.to(gpu))
    assert tied.dtype == dtype and rel(tied, ref + base.float()) < (TOL_F32 if dtype == torch.float32 else TOL_BF16)
    untouched = torch.ones(hi - lo, dtype=torch.bool)
    untouched[ids[(ids >= lo) & (ids < hi)] - lo] = False
    assert torch.equal(tied.cpu()[untouched], base[untouched])


def test_embedding_backward_padded_batch(gpu):
    """Half of 8192 tokens carry one id (a padded batch), a few more ids are carried by 33-200 tokens, the rest are
    Zipf-like: parity with the oracle, the same bits on every run, and a bounded time (the chain of the common id is
    walked in blocks of 32, not token by token)."""
    n, v, h = 8192, 32000, 4096
    g = gen(30)
    ids = (torch.rand(n, generator=g) ** 4 * v).long().clamp_max(v - 1)
    ids[torch.randperm(n, generator=g)[: n // 2]] = 2                      # pad id
    for k, c in ((7, 33), (11, 64), (13, 200), (17, 32)):
        ids[torch.randperm(n, generator=g)[:c]] = k
    dout = torch.randn(n, h, generator=g).bfloat16()
    ref = R.embedding_backward(ids, dout, v, 0, v)
    a = ops.embedding_bwd(ids.to(gpu), dout.to(gpu), v, 0, v, dtype=torch.float32)
    b = ops.embedding_bwd(ids.to(gpu), dout.to(gpu), v, 0, v, dtype=torch.float32)
    assert rel(a, ref) < TOL_F32 and torch.equal(a, b)
    for k in (2, 7, 11, 13, 17):
        assert rel(a[k], ref[k]) < TOL_F32, k
    idg, dg, out = ids.to(gpu), dout.to(gpu), torch.zeros(v, h, device=gpu)
    ops.embedding_bwd(idg, dg, v, 0, v, out=out)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(5):
        ops.embedding_bwd(idg, dg, v, 0, v, out=out)
    e1.record()
    torch.cuda.synchronize()
    assert e0.elapsed_time(e1) / 5 < 2.0, "a common id must not be walked token by token (milliseconds)"


def test_embedding_full_size_llama_table(gpu):
    v, h, n = 128256, 4096, 8192
    table = torch.empty(v, h, dtype=torch.bfloat16, device=gpu).normal_(0, 0.02, generator=torch.Generator(device=gpu).manual_seed(1239))
    ids = torch.randint(0, v, (n,), generator=gen(24))
    out = ops.embedding_gather(ids.to(gpu), table, 0, v)
    pick = torch.randperm(n, generator=gen(25))[:256]
    host_rows = table[ids[pick].to(gpu)].cpu()                # plain copies of the source rows to the host
    assert torch.equal(out.cpu()[pick], R.vocab_parallel_embedding_forward(torch.arange(256), host_rows, 0, 256, 1))
    # checksum of checksums: a pure gather preserves every row's bit pattern
    src = table.view(torch.int16).to(torch.int64).sum(-1)[ids.to(gpu)]
    assert torch.equal(out.view(torch.int16).to(torch.int64).sum(-1), src)


# =============================================================================== linear layers
def _lin_inputs(m, n, k, dtype, seed, bias=True):
    x = torch.randn(m, k, generator=gen(seed)).to(dtype)
    w = (torch.randn(n, k, generator=gen(seed + 1)) * 0.02).to(dtype)
    b = (torch.randn(n, generator=gen(seed + 2)) * 0.02).to(dtype) if bias else None
    dy = torch.randn(m, n, generator=gen(seed + 3)).to(dtype)
    return x, w, b, dy


@pytest.mark.parametrize("dtype,m,n,k", [
    (torch.float32, 1024, 3072, 768),       # GPT-2-small column layer, fewer tokens
    (torch.float32, 1024, 768, 3072),       # GPT-2-small row layer
    (torch.bfloat16, 512, 6144, 4096),      # Llama-3-8B QKV
    (torch.bfloat16, 256, 4096, 14336),     # Llama-3-8B down
    (torch.bfloat16, 512, 1280, 8192),      # Llama-70B tp=8 QKV shard
    (torch.bfloat16, 512, 8192, 1024),      # Llama-70B tp=8 o-proj shard
    (torch.bfloat16, 300, 520, 136), (torch.bfloat16, 64, 50, 27), (torch.bfloat16, 1, 8, 8),
    (torch.float32, 100, 77, 33), (torch.float32, 1, 1, 1), (torch.bfloat16, 257, 255, 72),
    (torch.float32, 300, 520, 136), (torch.float32, 129, 132, 20), (torch.float32, 64, 8, 4), (torch.float32, 3, 260, 4100),
    # k long enough for the forward kernel's register-staged pairs of k-tiles, with ragged m, n and end of k
    (torch.bfloat16, 300, 520, 1000), (torch.bfloat16, 257, 255, 456), (torch.bfloat16, 129, 1000, 200),
    (torch.bfloat16, 1000, 264, 232), (torch.bfloat16, 31, 700, 192), (torch.float16, 300, 520, 1000),
])
def test_linear_fwd_bwd_vs_oracle(gpu, dtype, m, n, k):
    tol = TOL_F32 if dtype == torch.float32 else TOL_BF16
    x, w, b, dy = _lin_inputs(m, n, k, dtype, 30)
    xf, wf, bf, dyf = x.float(), w.float(), b.float(), dy.float()
    ref, _ = R.column_parallel_linear_forward(xf, wf, bf)
    y, _ = ops.linear_fwd(x.to(gpu), w.to(gpu), b.to(gpu), ops.EPI_BIAS)
    assert rel(y, ref) < tol
    y0, _ = ops.linear_fwd(x.to(gpu), w.to(gpu), None, ops.EPI_NONE)
    assert rel(y0, R.row_parallel_linear_forward(xf, wf, None)[0]) < tol
    rdx, rdw, rdb = R.linear_backward(xf, wf, dyf, True)
    assert rel(ops.linear_dgrad(dy.to(gpu), w.to(gpu)), rdx) < tol
    dw, db = ops.linear_wgrad(dy.to(gpu), x.to(gpu), True)
    assert dw.dtype == dtype and rel(dw, rdw) < tol and rel(db, rdb) < tol
    if dtype == torch.bfloat16:                       # fp32 main-gradient accumulation
        acc = torch.ones(n, k, device=gpu)
        accb = torch.ones(n, device=gpu)
        ops.linear_wgrad(dy.to(gpu), x.to(gpu), True, dw=acc, db=accb, accumulate=True)
        assert rel(acc - 1, rdw) < TOL_F32 * 10 and rel(accb - 1, rdb) < TOL_F32 * 10


def _every_product_once(gpu, dtype, m, n, k, seed):
    """Every 16-bit product and epilogue of the linear layers on one shape, as a dict of device tensors."""
    x, w, b, dy = _lin_inputs(m, n, k, dtype, seed)
    xg, wg, bg, dyg = x.to(gpu), w.to(gpu), b.to(gpu), dy.to(gpu)
    out = {}
    out["y"], _ = ops.linear_fwd(xg, wg, bg, ops.EPI_BIAS)
    out["pre"], out["gelu"] = ops.linear_fwd(xg, wg, bg, ops.EPI_BIAS_GELU)
    out["spre"], out["swiglu"] = ops.linear_fwd(xg, wg, None, ops.EPI_SWIGLU)
    out["dx"] = ops.linear_dgrad(dyg, wg)
    out["dw"], out["db"] = ops.linear_wgrad(dyg, xg, True)
    acc, accb = torch.ones(n, k, device=gpu), torch.ones(n, device=gpu)
    ops.linear_wgrad(dyg, xg, True, dw=acc, db=accb, accumulate=True)
    out["acc"], out["accb"] = acc, accb
    # accumulation in the tensor dtype (how `.grad` sums micro-batches), onto a gradient of the same size
    acc16 = out["dw"].clone()
    ops.linear_wgrad(dyg, xg, False, dw=acc16, accumulate=True)
    out["acc16"] = acc16
    return (x, w, b, dy), out


def _check_every_product(inputs, out, tol, what):
    x, w, b, dy = (t.float() for t in inputs)
    pre = R.column_parallel_linear_forward(x, w, b)[0]
    assert rel(out["y"], pre) < tol and rel(out["pre"], pre) < tol, what
    assert rel(out["gelu"], R.gelu_new(pre)) < tol, what
    assert rel(out["spre"], F.linear(x, w)) < tol, what
    assert rel(out["swiglu"], R.swiglu(out["spre"].float().cpu())) < tol, what
    rdx, rdw, rdb = R.linear_backward(x, w, dy, True)
    assert rel(out["dx"], rdx) < tol and rel(out["dw"], rdw) < tol and rel(out["db"], rdb) < tol, what
    assert rel(out["acc"] - 1, rdw) < TOL_F32 * 10 and rel(out["accb"] - 1, rdb) < TOL_F32 * 10, what
    assert rel(out["acc16"], 2 * rdw) < tol, what


# k, n and m multiples of 64 (every product can take the 64-deep loop), then ragged in all three
# (the third has 33 k-tiles of 64 forward; the fourth gives the weight gradient 17 k-tiles and ragged tiles of every width)
_CFG_SHAPES = [(320, 576, 448), (300, 520, 200), (1100, 1304, 2112), (1088, 1000, 648)]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("cfg", list(range(14)))
def test_every_tile_configuration_vs_oracle(gpu, set_tuning, dtype, cfg):
    """Each tile configuration forced in turn (one that cannot serve a shape or epilogue falls back to the
    automatic choice): every product and epilogue against the oracle, and the same bits on a second run."""
    set_tuning("MTP_GEMM_CFG", cfg)
    for (m, n, k) in _CFG_SHAPES:
        inputs, out = _every_product_once(gpu, dtype, m, n, k, 300 + cfg)
        _check_every_product(inputs, out, TOL_BF16, (cfg, m, n, k))
        _, again = _every_product_once(gpu, dtype, m, n, k, 300 + cfg)
        for name in out:
            assert torch.equal(out[name], again[name]), (cfg, m, n, k, name)


def test_linear_scratch_is_allocated_only_for_shapes_that_use_it(gpu):
    """The wrappers ask the library how much scratch a product can use and allocate none for the (many) shapes that
    never touch it; a shape stream-K is taken for gets the buffer, per device and stream, until it is released."""
    from merak_amd import _lib
    ops.release_workspaces()
    x, w, _, dy = _lin_inputs(512, 1024, 512, torch.bfloat16, 33, bias=False)      # every product has under 32 k-tiles
    y, _ = ops.linear_fwd(x.to(gpu), w.to(gpu), None, ops.EPI_NONE)
    ops.linear_bwd(dy.to(gpu), x.to(gpu), w.to(gpu), False)
    assert not ops._linear_ws_cache and rel(y, F.linear(x.float(), w.float())) < TOL_BF16
    x, w, _, _ = _lin_inputs(256, 512, 4096, torch.bfloat16, 34, bias=False)       # 2 tiles, 64 k-tiles each
    y, _ = ops.linear_fwd(x.to(gpu), w.to(gpu), None, ops.EPI_NONE)
    assert rel(y, F.linear(x.float(), w.float())) < TOL_BF16
    assert [t.numel() for t in ops._linear_ws_cache.values()] == [_lib.lib().mtp_linear_workspace_bytes()]
    ops.release_workspaces()
    assert not ops._linear_ws_cache


@pytest.mark.parametrize("mode", [0, 1, 2])
@pytest.mark.parametrize("cfg", [8, None])
def test_stream_k_forced_vs_oracle(gpu, set_tuning, mode, cfg):
    """Stream-K switched off, taken wherever the last round is part empty, and with every tile going through its
    kernel: against the oracle, the same bits on every run (the pieces are summed in k order by a second kernel,
    no atomics), and the three modes within rounding of one another."""
    set_tuning("MTP_GEMM_SK", mode)
    set_tuning("MTP_GEMM_CFG", cfg)
    for (m, n, k) in _CFG_SHAPES + [(256, 512, 4096), (512, 768, 8192)]:
        inputs, out = _every_product_once(gpu, torch.bfloat16, m, n, k, 330)
        _check_every_product(inputs, out, TOL_BF16, (mode, cfg, m, n, k))
        for _ in range(2):
            _, again = _every_product_once(gpu, torch.bfloat16, m, n, k, 330)
            for name in out:
                assert torch.equal(out[name], again[name]), (mode, cfg, m, n, k, name)


@pytest.mark.parametrize("slices", [1, 2, 4, 8, None])
def test_fp32_products_cut_along_k(gpu, set_tuning, slices):
    """fp32 products with few output tiles and a long k are cut into slices along k (one workgroup per tile and
    slice, a second kernel adds the slices in slice order): switched off, forced to 2 / 4 / 8 and as chosen, against
    the oracle, with bias, bias gradient and accumulation, ragged shapes included, and the same bits on every run."""
    set_tuning("MTP_GEMM_F32_SLICES", slices)
    for (m, n, k) in ((4096, 768, 256), (8192, 384, 132), (2100, 260, 520)):
        x, w, b, dy = _lin_inputs(m, n, k, torch.float32, 350)
        xg, wg, bg, dyg = x.to(gpu), w.to(gpu), b.to(gpu), dy.to(gpu)
        rdx, rdw, rdb = R.linear_backward(x, w, dy, True)
        outs = []
        for _ in range(2):
            dw, db = ops.linear_wgrad(dyg, xg, True)                      # k of this product = m tokens
            acc, accb = torch.ones(n, k, device=gpu), torch.ones(n, device=gpu)
            ops.linear_wgrad(dyg, xg, True, dw=acc, db=accb, accumulate=True)
            y, _ = ops.linear_fwd(dyg, wg.t().contiguous(), None, ops.EPI_NONE)   # [m, k] = dy w: k of the product = n
            outs.append((dw, db, acc, accb, y))
        dw, db, acc, accb, y = outs[0]
        assert rel(dw, rdw) < TOL_F32 and rel(db, rdb) < TOL_F32, (slices, m, n, k)
        assert rel(acc - 1, rdw) < TOL_F32 * 10 and rel(accb - 1, rdb) < TOL_F32 * 10, (slices, m, n, k)
        assert rel(y, rdx) < TOL_F32, (slices, m, n, k)
        for a, b2 in zip(outs[0], outs[1]):
            assert torch.equal(a, b2), (slices, m, n, k)
    # a product with a bias whose k is long: forward of a narrow layer over many features
    x, w, b, _ = _lin_inputs(96, 200, 4096, torch.float32, 351)
    y, _ = ops.linear_fwd(x.to(gpu), w.to(gpu), b.to(gpu), ops.EPI_BIAS)
    assert rel(y, R.column_parallel_linear_forward(x, w, b)[0]) < TOL_F32


@pytest.mark.parametrize("mixed", [None, 0])
def test_mixed_tiling_vs_oracle(gpu, set_tuning, mixed):
    """One and a half rounds of 256x256 tiles are launched as one round on the 64-deep loop plus one round of
    half-size tiles on the ring loop (columns for the forward product, rows for the weight gradient): with it
    and with it switched off, against the oracle on sampled rows and columns of both parts, ragged edges, bias +
    GELU, bias gradient and accumulation; the same bits on every run."""
    set_tuning("MTP_GEMM_MIXED", mixed)
    m, n, k = 4096, 6100, 4096          # 16 x 24 tiles forward, 24 x 16 for the weight gradient
    g = torch.Generator(device=gpu).manual_seed(1242)
    x = torch.empty(m, k, device=gpu).normal_(generator=g).bfloat16()
    w = torch.empty(n, k, device=gpu).normal_(0, 0.02, generator=g).bfloat16()
    b = torch.empty(n, device=gpu).normal_(0, 0.5, generator=g).bfloat16()
    dy = torch.empty(m, n, device=gpu).normal_(generator=g).bfloat16()
    rm = torch.randperm(m, generator=gen(74))[:24].to(gpu)
    rn = torch.cat([torch.randperm(n, generator=gen(75))[:20], torch.tensor([0, 4095, 4096, 4097, n - 1])]).to(gpu)
    xs, ws, bs = x[rm].cpu().float(), w.cpu().float(), b.cpu().float()
    runs = []
    for _ in range(2):
        y, act = ops.linear_fwd(x, w, b, ops.EPI_BIAS_GELU)
        dw, db = ops.linear_wgrad(dy, x, True)
        acc, accb = torch.ones(n, k, device=gpu), torch.ones(n, device=gpu)
        ops.linear_wgrad(dy, x, True, dw=acc, db=accb, accumulate=True)
        runs.append((y, act, dw, db, acc, accb))
    y, act, dw, db, acc, accb = runs[0]
    pre = R.column_parallel_linear_forward(xs, ws, bs)[0]
    assert rel(y[rm], pre) < TOL_BF16 and rel(act[rm], R.gelu_new(y[rm].float().cpu())) < TOL_BF16
    ref_dw = dy[:, rn].cpu().float().t() @ x.cpu().float()
    ref_db = dy.cpu().float().sum(0)
    assert rel(dw[rn], ref_dw) < TOL_BF16 and rel(db, ref_db) < TOL_BF16
    assert rel(acc[rn] - 1, ref_dw) < TOL_F32 * 10 and rel(accb - 1, ref_db) < TOL_F32 * 10
    for a, c in zip(runs[0], runs[1]):
        assert torch.equal(a, c)


@pytest.mark.parametrize("name,m,n,k", [("llama8b_down", 4096, 4096, 14336), ("llama70b_tp8_oproj", 8192, 8192, 1024),
                                         ("llama70b_tp8_qkv", 8192, 1280, 8192),     # the weight gradient's long tiles go first
                                         ("ragged", 1792, 2304, 3000), ("small", 300, 520, 448)])
def test_layer_backward_in_one_call(gpu, set_tuning, name, m, n, k):
    """mtp_linear_bwd: input and weight gradient of a layer as one call — one launch where the tiles of the two
    products together fill fewer rounds of workgroups (the first two shapes, and 84 + 108 tiles of the third,
    whose outputs end inside a tile), two launches otherwise.  The same bits as the two separate calls without scratch, with bias gradient, fp32
    accumulation into existing gradients, and on every run; the oracle on sampled rows."""
    g = torch.Generator(device=gpu).manual_seed(1243)
    x = torch.empty(m, k, device=gpu).normal_(generator=g).bfloat16()
    w = torch.empty(n, k, device=gpu).normal_(0, 0.02, generator=g).bfloat16()
    dy = torch.empty(m, n, device=gpu).normal_(generator=g).bfloat16()
    set_tuning("MTP_GEMM_PAIR", 0)
    set_tuning("MTP_GEMM_SK", 0)             # the pair never cuts a tile along k
    dx0, dw0, db0 = ops.linear_bwd(dy, x, w, True)
    acc0, accb0 = torch.ones(n, k, device=gpu), torch.ones(n, device=gpu)
    ops.linear_bwd(dy, x, w, True, dw=acc0, db=accb0, accumulate=True)
    set_tuning("MTP_GEMM_PAIR", None)
    set_tuning("MTP_GEMM_SK", None)
    runs = []
    for _ in range(2):
        dx, dw, db = ops.linear_bwd(dy, x, w, True)
        acc, accb = torch.ones(n, k, device=gpu), torch.ones(n, device=gpu)
        dx2, _, _ = ops.linear_bwd(dy, x, w, True, dw=acc, db=accb, accumulate=True)
        _, dw_nodb, none = ops.linear_bwd(dy, x, w, False)
        assert none is None and torch.equal(dx2, dx) and torch.equal(dw_nodb, dw)
        runs.append((dx, dw, db, acc, accb))
    for a, b in zip(runs[0], runs[1]):
        assert torch.equal(a, b), name                      # the same bits on every run
    # against the two separate launches: the same sums, possibly in another tile configuration's order
    for a, b, tol in ((dx, dx0, 3e-3), (dw, dw0, 3e-3), (db, db0, 3e-3), (acc, acc0, 1e-5), (accb, accb0, 1e-5)):
        assert rel(a, b) < tol, name
    rm = torch.randperm(m, generator=gen(76))[:16].to(gpu)
    rn = torch.randperm(n, generator=gen(77))[:16].to(gpu)
    ws = w.cpu().float()
    assert rel(dx[rm], dy[rm].cpu().float() @ ws) < TOL_BF16
    assert rel(dw[rn], dy[:, rn].cpu().float().t() @ x.cpu().float()) < TOL_BF16
    assert rel(db, dy.cpu().float().sum(0)) < TOL_BF16
    _whole_gradients_by_blocks(x, w, dy, dx, dw, name)


def test_measurement_switches_are_not_in_the_shipped_library(gpu, set_tuning):
    """MTP_GEMM_DEBUG turns parts of the product off in a measurement build (-DMTP_MEASURE).  The library that
    ships must not know the variable: with it set, results still match the oracle and are the bits of a run
    without it."""
    inputs, plain = _every_product_once(gpu, torch.bfloat16, 320, 576, 448, 340)
    for value in (1, 2, 4, 255):
        set_tuning("MTP_GEMM_DEBUG", value)
        _, out = _every_product_once(gpu, torch.bfloat16, 320, 576, 448, 340)
        _check_every_product(inputs, out, TOL_BF16, value)
        for name in out:
            assert torch.equal(out[name], plain[name]), (value, name)


@pytest.mark.parametrize("nbytes", [16, 16 * 1023, 16384, 16384 * 7 + 48, 16 * (4096 * 64 * 3 + 1025)])
def test_reference_copy_kernel_copies_every_byte(gpu, nbytes):
    """mtp_stream_copy (the bandwidth reference bench.py quotes): whole 16 KiB pieces and what is left of the last."""
    from merak_amd import _lib
    src = torch.randint(0, 256, (nbytes,), dtype=torch.uint8, generator=gen(77)).to(gpu)
    dst = torch.zeros(nbytes + 64, dtype=torch.uint8, device=gpu)
    st = torch.cuda.current_stream().cuda_stream
    _lib.check(_lib.lib().mtp_stream_copy(src.data_ptr(), dst.data_ptr(), nbytes, st), "copy")
    assert torch.equal(dst[:nbytes], src) and int(dst[nbytes:].sum()) == 0


@pytest.mark.parametrize("dtype,m,n,k", [(torch.float32, 512, 3072, 768), (torch.bfloat16, 512, 3072, 768),
                                          (torch.bfloat16, 200, 136, 72), (torch.float32, 33, 20, 10)])
def test_bias_gelu_epilogue(gpu, dtype, m, n, k):
    tol = TOL_F32 if dtype == torch.float32 else TOL_BF16
    x, w, b, dy = _lin_inputs(m, n, k, dtype, 40)
    pre = R.column_parallel_linear_forward(x.float(), w.float(), b.float())[0]
    y, act = ops.linear_fwd(x.to(gpu), w.to(gpu), b.to(gpu), ops.EPI_BIAS_GELU)
    assert rel(y, pre) < tol and rel(act, R.gelu_new(pre)) < tol
    _, act_only = ops.linear_fwd(x.to(gpu), w.to(gpu), b.to(gpu), ops.EPI_BIAS_GELU, want_pre=False)
    assert torch.equal(act_only, act)
    d = ops.activation_bwd(dy.to(gpu), y, ops.EPI_BIAS_GELU)
    assert rel(d, dy.float() * R.gelu_new_grad(y.float().cpu())) < tol


@pytest.mark.parametrize("dtype,m,n,k", [(torch.bfloat16, 512, 2 * 14336, 4096), (torch.bfloat16, 512, 2 * 3584, 8192),
                                          (torch.bfloat16, 130, 2 * 100, 72), (torch.float32, 65, 2 * 24, 40),
                                          (torch.bfloat16, 40, 2 * 13, 16),
                                          # ragged halves and end of k behind the staged pairs of k-tiles
                                          (torch.bfloat16, 130, 2 * 300, 1000), (torch.bfloat16, 257, 2 * 136, 264)])
def test_swiglu_epilogue(gpu, dtype, m, n, k):
    tol = TOL_F32 if dtype == torch.float32 else TOL_BF16
    x, w, _, _ = _lin_inputs(m, n, k, dtype, 50, bias=False)
    pre = F.linear(x.float(), w.float())
    y, act = ops.linear_fwd(x.to(gpu), w.to(gpu), None, ops.EPI_SWIGLU)
    assert act.shape == (m, n // 2) and rel(y, pre) < tol
    assert rel(act, R.swiglu(y.float().cpu())) < tol     # activation of the stored (rounded) pre-activation
    dact = torch.randn(m, n // 2, generator=gen(54)).to(dtype)
    d = ops.activation_bwd(dact.to(gpu), y, ops.EPI_SWIGLU)
    assert rel(d, R.swiglu_backward(dact.float(), y.float().cpu())) < tol


@pytest.mark.parametrize("dtype,m,h", [(torch.bfloat16, 1, 8), (torch.bfloat16, 3, 4096), (torch.float32, 5001, 24),
                                       (torch.bfloat16, 9000, 40), (torch.float16, 777, 2056), (torch.bfloat16, 300, 7)])
def test_swiglu_backward_row_and_column_split(gpu, dtype, m, h):
    """One row, more rows than row groups (several steps and an odd one left), rows wider than one column
    block, unaligned rows."""
    y = torch.randn(m, 2 * h, generator=gen(58)).to(dtype)
    dact = torch.randn(m, h, generator=gen(59)).to(dtype)
    d = ops.activation_bwd(dact.to(gpu), y.to(gpu), ops.EPI_SWIGLU)
    assert rel(d, R.swiglu_backward(dact.float(), y.float())) < (TOL_F32 if dtype == torch.float32 else TOL_BF16)


def test_gpt2_small_fp32_full_size(gpu):
    """Config 1 in full: Column 768->3072 bias+GeLU, Row 3072->768 bias, 8x1024 tokens, fp32, via the modules."""
    set_args(use_cpu_initialization=True, params_dtype=torch.float32)
    torch.manual_seed(1)
    init = lambda t: torch.nn.init.normal_(t, 0.0, 0.02)
    col = mpu.ColumnParallelLinear(768, 3072, gather_output=False, init_method=init, activation="gelu_new")
    row = mpu.RowParallelLinear(3072, 768, input_is_parallel=True, init_method=init)
    with torch.no_grad():
        col.bias.normal_(0, 0.02); row.bias.normal_(0, 0.02)
    x = torch.randn(8, 1024, 768, generator=gen(60))
    dy = torch.randn(8, 1024, 768, generator=gen(61))
    # oracle chain on the host (reference op order), autograd for the backward
    xr = x.clone().requires_grad_(True)
    wc, bc, wr, br = (p.detach().clone().requires_grad_(True) for p in (col.weight, col.bias, row.weight, row.bias))
    h = R.gelu_new(R.column_parallel_linear_forward(xr, wc, bc)[0])
    out_ref, none = R.row_parallel_linear_forward(h, wr, br)
    out_ref.backward(dy)
    col.to(gpu); row.to(gpu)
    xg = x.to(gpu).requires_grad_(True)
    hg, b1 = col(xg)
    out, b2 = row(hg)
    assert b1 is None and b2 is None and out.shape == (8, 1024, 768)
    out.backward(dy.to(gpu))
    assert rel(out, out_ref) < TOL_F32 and rel(xg.grad, xr.grad) < TOL_F32
    for p, r in ((col.weight, wc), (col.bias, bc), (row.weight, wr), (row.bias, br)):
        assert rel(p.grad, r.grad) < TOL_F32


def _whole_gradients_by_blocks(x, w, dy, dx, dw, what, blk=32):
    """Every element of both gradients in a checked number.  Sums over blocks of `blk` rows commute with the products:
    dX summed over the rows of a block = (dY summed over those rows) W, and dW summed over the columns of a block =
    dY^T (X summed over those columns).  Both sides in fp32 on the device (torch's fp32 matmul on the small side), compared
    per blk x blk block of the output, so that one wrong tile anywhere shows as a block far beyond the rounding of the
    16-bit gradients (2^-9 per element)."""
    m, k = x.shape
    n = w.shape[0]
    mb, kb = m // blk, k // blk
    xf, wf, dyf = x.float(), w.float(), dy.float()
    got_dx = dx.float()[: mb * blk].view(mb, blk, k).sum(1)                      # [m/blk, k]
    ref_dx = dyf[: mb * blk].view(mb, blk, n).sum(1) @ wf
    got_dw = dw.float()[:, : kb * blk].view(n, kb, blk).sum(2)                   # [n, k/blk]
    ref_dw = dyf.t() @ xf[:, : kb * blk].view(m, kb, blk).sum(2)
    for name, got, ref, axis in (("dx", got_dx[:, : kb * blk].reshape(mb, kb, blk), ref_dx[:, : kb * blk].reshape(mb, kb, blk), 2),
                                 ("dw", got_dw[: n // blk * blk].reshape(n // blk, blk, kb), ref_dw[: n // blk * blk].reshape(n // blk, blk, kb), 1)):
        err = (got - ref).double().norm(dim=axis)
        mag = ref.double().norm(dim=axis)
        # a block's reference can be small by chance: measure against the typical block as well
        worst = (err / torch.maximum(mag, mag.median())).max().item()
        assert worst < 2 * TOL_BF16, (what, name, worst)



@pytest.mark.parametrize("name,m,k,n", [("llama8b_qkv", 4096, 4096, 6144), ("llama8b_down", 4096, 14336, 4096),
                                         ("llama70b_tp8_qkv", 8192, 8192, 1280), ("llama70b_tp8_oproj", 8192, 1024, 8192),
                                         ("llama70b_tp8_down", 8192, 3584, 8192)])
def test_linear_full_size_sampled(gpu, name, m, k, n):
    """Full Llama-3-8B and Llama-70B tp=8 shard shapes: oracle on sampled rows of Y, dX and dW; linearity in X over the whole output."""
    g = torch.Generator(device=gpu).manual_seed(1240)
    x = torch.empty(m, k, device=gpu).normal_(generator=g).bfloat16()
    w = torch.empty(n, k, device=gpu).normal_(0, 0.02, generator=g).bfloat16()
    dy = torch.empty(m, n, device=gpu).normal_(generator=g).bfloat16()
    y, _ = ops.linear_fwd(x, w, None, ops.EPI_NONE)
    dx = ops.linear_dgrad(dy, w)
    dw, _ = ops.linear_wgrad(dy, x, False)
    rm = torch.randperm(m, generator=gen(70))[:32].to(gpu)
    rn = torch.randperm(n, generator=gen(71))[:32].to(gpu)
    xs, ws, dys = x[rm].cpu().float(), w.cpu().float(), dy[rm].cpu().float()
    assert rel(y[rm], R.row_parallel_linear_forward(xs, ws, None)[0]) < TOL_BF16
    assert rel(dx[rm], R.linear_backward(xs, ws, dys, False)[0]) < TOL_BF16
    ref_dw = R.linear_backward(x.cpu().float(), ws[rn.cpu()], dy[:, rn].cpu().float(), False)[1]
    assert rel(dw[rn], ref_dw) < TOL_BF16
    _whole_gradients_by_blocks(x, w, dy, dx, dw, name)
    y2, _ = ops.linear_fwd((x.float() * 2).bfloat16(), w, None, ops.EPI_NONE)     # exact in bf16: scaling by 2
    assert torch.equal(y2.float(), y.float() * 2)


@pytest.mark.parametrize("name,m,k,half", [("llama8b_gate_up", 4096, 4096, 14336), ("llama70b_tp8_gate_up", 8192, 8192, 3584)])
def test_swiglu_full_size_sampled(gpu, name, m, k, half):
    """Gate/up column layers with the fused SwiGLU at their full token counts: oracle on sampled rows of the
    pre-activation, the activation, dX and dW; the pre-activation is linear in X over the whole output."""
    n = 2 * half
    g = torch.Generator(device=gpu).manual_seed(1241)
    x = torch.empty(m, k, device=gpu).normal_(generator=g).bfloat16()
    w = torch.empty(n, k, device=gpu).normal_(0, 0.02, generator=g).bfloat16()
    dact = torch.empty(m, half, device=gpu).normal_(generator=g).bfloat16()
    y, act = ops.linear_fwd(x, w, None, ops.EPI_SWIGLU)
    assert y.shape == (m, n) and act.shape == (m, half)
    rm = torch.randperm(m, generator=gen(72))[:32].to(gpu)
    rn = torch.randperm(n, generator=gen(73))[:32].to(gpu)
    xs, ws = x[rm].cpu().float(), w.cpu().float()
    assert rel(y[rm], F.linear(xs, ws)) < TOL_BF16
    assert rel(act[rm], R.swiglu(y[rm].float().cpu())) < TOL_BF16      # activation of the stored pre-activation
    _, act_only = ops.linear_fwd(x, w, None, ops.EPI_SWIGLU, want_pre=False)
    assert torch.equal(act_only, act)
    dy = ops.activation_bwd(dact, y, ops.EPI_SWIGLU)
    assert rel(dy[rm], R.swiglu_backward(dact[rm].float().cpu(), y[rm].float().cpu())) < TOL_BF16
    dx = ops.linear_dgrad(dy, w)
    dw, _ = ops.linear_wgrad(dy, x, False)
    dys = dy[rm].cpu().float()
    assert rel(dx[rm], R.linear_backward(xs, ws, dys, False)[0]) < TOL_BF16
    ref_dw = R.linear_backward(x.cpu().float(), ws[rn.cpu()], dy[:, rn].cpu().float(), False)[1]
    assert rel(dw[rn], ref_dw) < TOL_BF16
    _whole_gradients_by_blocks(x, w, dy, dx, dw, name)
    y2, _ = ops.linear_fwd((x.float() * 2).bfloat16(), w, None, ops.EPI_SWIGLU)   # exact in bf16: scaling by 2
    assert torch.equal(y2.float(), y.float() * 2)


def test_module_surface_on_gpu(gpu):
    set_args(use_cpu_initialization=True, params_dtype=torch.bfloat16)
    torch.manual_seed(2)
    col = mpu.ColumnParallelLinear(256, 512, skip_bias_add=True, gather_output=False).to(gpu)
    x = torch.randn(2, 5, 256, generator=gen(80)).bfloat16()
    out, ob = col(x.to(gpu).transpose(0, 1))                    # non-contiguous (seq, batch, hidden) view
    assert ob is col.bias and out.shape == (5, 2, 512)
    ref = R.column_parallel_linear_forward(x.float().transpose(0, 1), col.weight.detach().cpu().float(),
                                           col.bias.detach().cpu().float(), True)[0]
    assert rel(out, ref) < TOL_BF16
    row = mpu.RowParallelLinear(512, 256, bias=True, input_is_parallel=True, skip_bias_add=True).to(gpu)
    o2, b2 = row(out)
    assert b2 is row.bias and o2.shape == (5, 2, 256)
    set_args(use_cpu_initialization=False, params_dtype=torch.float32)
    dev_layer = mpu.ColumnParallelLinear(64, 64, init_method=lambda t: torch.nn.init.normal_(t, 0, 0.02))
    assert dev_layer.weight.is_cuda and dev_layer.bias.is_cuda
    empty, _ = dev_layer(torch.empty(0, 64, device=gpu))
    assert empty.shape == (0, 64)


def test_model_parallel_rng_on_the_device(gpu):
    """The device path of the weight initialisation (layers.py:44-53): shards drawn on the GPU under the
    model-parallel generator state: the same shard for one rank seeded twice, different shards for two ranks of one
    group, the device's default generator state (and the host's) left where it was."""
    from merak_amd.mpu.layers import _initialize_affine_weight_gpu

    def shard(rank, seed=1234):
        mpu.set_model_parallel_world_size(2)
        mpu.set_model_parallel_rank(rank)
        mpu.model_parallel_manual_seed(seed)
        before_gpu, before_cpu = torch.cuda.get_rng_state(gpu), torch.get_rng_state()
        w = torch.empty(8, 16, device=gpu)
        _initialize_affine_weight_gpu(w, torch.nn.init.normal_, 0)
        assert torch.equal(torch.cuda.get_rng_state(gpu), before_gpu) and torch.equal(torch.get_rng_state(), before_cpu)
        return w

    a, b, a2 = shard(0), shard(1), shard(0)
    assert not torch.equal(a, b) and torch.equal(a, a2)
    # host-resident weights on a machine with a GPU draw under the same tracker
    mpu.model_parallel_manual_seed(99)
    c1 = torch.empty(4, 4)
    _initialize_affine_weight_gpu(c1, torch.nn.init.normal_, 0)
    mpu.model_parallel_manual_seed(99)
    c2 = torch.empty(4, 4)
    _initialize_affine_weight_gpu(c2, torch.nn.init.normal_, 0)
    assert torch.equal(c1, c2)


def test_one_launch_ce_marks_the_layer_logits_as_overwritten(gpu):
    """The one-launch cross entropy overwrites the logits with their gradient during forward.  The logits a
    ColumnParallelLinear returns own their storage (no view), so the overwrite is recorded: another function that
    saved those logits for its own backward fails loudly instead of using gradients as if they were logits."""
    set_args(use_cpu_initialization=True, params_dtype=torch.bfloat16)
    col = mpu.ColumnParallelLinear(64, 512, bias=False, gather_output=False).to(gpu)
    x = torch.randn(4, 8, 64, generator=gen(90)).bfloat16().to(gpu).requires_grad_(True)
    tgt = torch.randint(0, 512, (4, 8), generator=gen(91)).to(gpu)
    logits, _ = col(x)
    assert logits.shape == (4, 8, 512) and not logits._is_view()
    other = (logits * logits).sum()             # saves the logits for its backward
    loss = mpu.vocab_loss_fn(logits, tgt)       # overwrites them
    with pytest.raises(RuntimeError, match="modified by an inplace operation"):
        other.backward(retain_graph=True)
    loss.backward()
    assert x.grad is not None and torch.isfinite(x.grad.float()).all()


def test_modules_cast_to_bf16_after_construction(gpu):
    """The reference builds its parameters in fp32 (or fp16) and turns the model to bf16 afterwards with
    ``module.bfloat16()`` (amp_engine.py:130-139, pipeline/module.py:189-190): the layers, embedding and loss
    must work on parameters that changed dtype after the constructor ran."""
    set_args(use_cpu_initialization=True, params_dtype=torch.float32)
    torch.manual_seed(3)
    init = lambda t: torch.nn.init.normal_(t, 0.0, 0.02)

    class Tiny(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.emb = mpu.VocabParallelEmbedding(300, 128, init_method=init)
            self.col = mpu.ColumnParallelLinear(128, 512, gather_output=False, init_method=init)
            self.row = mpu.RowParallelLinear(512, 128, input_is_parallel=True, init_method=init)
            self.head = mpu.ColumnParallelLinear(128, 300, bias=False, gather_output=False, init_method=init)

        def forward(self, ids, labels):
            h = self.emb(ids)
            h = h + self.row(F.gelu(self.col(h)[0], approximate="tanh"))[0]
            return mpu.vocab_parallel_cross_entropy(self.head(h)[0], labels).mean()

    m = Tiny()
    assert m.col.weight.dtype == torch.float32
    ref = {k: v.detach().clone() for k, v in m.state_dict().items()}
    m = m.to(gpu).bfloat16()
    assert all(p.dtype == torch.bfloat16 and p.is_cuda for p in m.parameters())
    ids = torch.randint(0, 300, (4, 9), generator=gen(81))
    labels = torch.randint(0, 300, (4, 9), generator=gen(82))
    loss = m(ids.to(gpu), labels.to(gpu))
    loss.backward()
    # stock torch on the bf16-rounded weights, fp32 arithmetic
    w = {k: v.bfloat16().float().requires_grad_(True) for k, v in ref.items()}
    h = F.embedding(ids, w["emb.weight"])
    h = h + F.linear(F.gelu(F.linear(h, w["col.weight"], w["col.bias"]), approximate="tanh"), w["row.weight"], w["row.bias"])
    want = F.cross_entropy(F.linear(h, w["head.weight"]).view(-1, 300), labels.view(-1))
    want.backward()
    assert abs(loss.item() - want.item()) < 2e-2 * abs(want.item())
    for name, p_ in m.named_parameters():
        assert p_.grad is not None and p_.grad.dtype == torch.bfloat16, name
        assert rel(p_.grad, w[name].grad) < 3 * TOL_BF16, name          # bf16 activations through three layers


# =============================================================================== decode
@pytest.mark.parametrize("b,n,k", [(1, 64, 256), (8, 1000, 512), (32, 4096, 1024), (5, 130, 4104), (17, 77, 40),
                                    (32, 6144, 4096), (8, 4096, 14336)])
def test_gemv_and_fused_argmax(gpu, b, n, k):
    x = torch.randn(b, k, generator=gen(90)).bfloat16()
    w = (torch.randn(n, k, generator=gen(91)) * 0.02).bfloat16()
    ref = F.linear(x.float(), w.float())
    y = ops.gemv(x.to(gpu), w.to(gpu))
    assert rel(y, ref) < TOL_BF16
    idx, val = ops.gemv_argmax(x.to(gpu), w.to(gpu))
    assert idx.dtype == torch.int64 and torch.equal(idx.cpu(), R.greedy_argmax(ref))
    assert rel(val, ref.max(-1).values) < TOL_F32
    assert torch.equal(greedy_from_logits(ref.to(gpu)).cpu(), R.greedy_argmax(ref))


@pytest.mark.parametrize("b,n,k,epi,force,cut", [
    (32, 4096, 14336, "none", None, True), (17, 4096, 14336, "bias", None, True), (9, 1280, 8192, "none", None, True),
    (32, 4096, 4096, "none", None, False), (8, 4096, 14336, "none", None, False),      # small k / small batch: uncut
    (32, 6144, 4096, "bias", "4", True), (32, 2048, 4096, "swiglu", "8", True), (24, 1000, 1024, "none", "2", True),
    (3, 4096, 4096, "none", "8", True)])
def test_gemv_cut_along_k_with_workspace(gpu, set_tuning, b, n, k, epi, force, cut):
    """Few-row matrices with a long k run, above 8 batch rows, as k slices whose partial sums meet in a
    workspace (other shapes only when forced): same numbers as the oracle, the same bits on every run, and a
    workspace that can be used again as it is left."""
    if force:
        set_tuning("MTP_GEMV_S", force)
    g = gen(31)
    x = torch.randn(b, k, generator=g).bfloat16()
    w = (torch.randn(n, k, generator=g) * 0.02).bfloat16()
    bias = (torch.randn(n, generator=g) * 0.1).bfloat16() if epi == "bias" else None
    e = {"none": ops.EPI_NONE, "bias": ops.EPI_BIAS, "swiglu": ops.EPI_SWIGLU}[epi]
    ref = F.linear(x.float(), w.float(), None if bias is None else bias.float())
    if epi == "swiglu":
        ref = R.swiglu(ref.bfloat16().float())
    ws = ops.gemv_workspace(b, n, k, e, gpu)
    assert (ws is not None) == cut
    xg, wg, bg = x.to(gpu), w.to(gpu), None if bias is None else bias.to(gpu)
    y1 = ops.gemv(xg, wg, bg, e, workspace=ws)
    y2 = ops.gemv(xg, wg, bg, e, workspace=ws)
    assert rel(y1, ref) < TOL_BF16
    assert torch.equal(y1, y2)
    if ws is not None:
        assert rel(ops.gemv(xg, wg, bg, e), y1) < TOL_BF16 / 4        # against the uncut form
        assert int(ws[:4 * ((n + 15) // 16)].count_nonzero()) == 0       # counters are back at zero


def test_gemv_one_workspace_for_shapes_in_turn(gpu):
    """Two cut shapes with different numbers of rows alternate on one zeroed workspace: the counters sit at a
    fixed place, so the partial sums of the matrix with few rows never land in the other one's counters."""
    g = gen(33)
    b = 16
    shapes = [(1024, 8192), (8192, 8192), (1280, 8192), (4096, 14336)]
    need = max(_lib_bytes(b, n, k) for n, k in shapes)
    assert need > 0 and min(_lib_bytes(b, n, k) for n, k in shapes) > 0, "every shape here is cut"
    ws = torch.zeros(need, dtype=torch.uint8, device=gpu)
    mats = [((torch.randn(n, k, generator=g) * 0.02).bfloat16().to(gpu), torch.randn(b, k, generator=g).bfloat16().to(gpu))
            for n, k in shapes]
    for rep in range(2):
        for w, x in mats:
            y = ops.gemv(x, w, workspace=ws)
            assert rel(y, F.linear(x.float(), w.float())) < TOL_BF16
    assert int(ws[:8192].view(torch.int32).abs().sum()) == 0


def test_argmax_one_workspace_for_shapes_in_turn(gpu):
    """One workspace serves greedy picks of different shapes in turn (nothing in it needs clearing): fewer workgroups
    than batch rows, thousands of them, two batch tiles."""
    shapes = [(3, 48, 64), (32, 128256, 512), (7, 5000, 256), (20, 40000, 128), (1, 70000, 64), (32, 1000, 72)]
    ws = ops.argmax_workspace(32, 128256, 512, gpu)
    ws.fill_(0xA5)
    for rep in range(2):
        for (b, n, k) in shapes:
            x = torch.randn(b, k, generator=gen(190 + b)).bfloat16()
            w = (torch.randn(n, k, generator=gen(191 + b)) * 0.02).bfloat16()
            ref = F.linear(x.float(), w.float())
            idx, val = ops.gemv_argmax(x.to(gpu), w.to(gpu), ws)
            idx2, val2 = ops.gemv_argmax(x.to(gpu), w.to(gpu))
            assert torch.equal(idx, idx2) and torch.equal(val, val2), (rep, b, n, k)
            # bf16 products: a near tie may fall the other way than in fp32, the winning value may not
            assert rel(val, ref.max(-1).values) < TOL_F32 and (idx.cpu() == ref.argmax(-1)).float().mean() >= 0.9


@pytest.mark.parametrize("b,n1,half,k,bias", [(32, 6144, 14336, 4096, False), (17, 1000, 4096, 1024, True),
                                               (8, 6144, 14336, 4096, False), (32, 130, 200, 264, True),
                                               (20, 1280, 3584, 8192, False), (25, 6100, 14000, 4096, True),
                                               (32, 3000, 14336, 4096, False), (5, 6100, 14000, 4096, True),
                                               (16, 3000, 14336, 4096, False), (32, 6090, 14336, 4096, False),
                                               (2, 4097, 14336, 4096, True)])
def test_gemv_pair_is_the_two_products(gpu, set_tuning, b, n1, half, k, bias):
    """mtp_gemv_pair: QKV-like and gate/up-like products over the same rows in one call — one grid above 16 rows
    for the shapes it takes (the first product's rows as one or two more row groups in the loop of the mixed
    groups, ragged ends included, or as a block in front of the loop: MTP_GEMV_PAIR = 2), two launches otherwise:
    the results of the two separate calls, and the oracle."""
    x = torch.randn(b, k, generator=gen(290)).bfloat16()
    w1 = (torch.randn(n1, k, generator=gen(291)) * 0.02).bfloat16()
    w2 = (torch.randn(2 * half, k, generator=gen(292)) * 0.02).bfloat16()
    b1 = (torch.randn(n1, generator=gen(293)) * 0.1).bfloat16() if bias else None
    b2 = (torch.randn(2 * half, generator=gen(294)) * 0.1).bfloat16() if bias else None
    dev = lambda t: None if t is None else t.to(gpu)
    xg, w1g, w2g, b1g, b2g = dev(x), dev(w1), dev(w2), dev(b1), dev(b2)
    y1 = ops.gemv(xg, w1g, b1g, ops.EPI_BIAS if bias else ops.EPI_NONE)
    a2 = ops.gemv(xg, w2g, b2g, ops.EPI_SWIGLU)
    for pair in (None, 2, 0):
        set_tuning("MTP_GEMV_PAIR", pair)
        p1, p2 = ops.gemv_pair(xg, w1g, w2g, b1g, b2g)
        # Above 16 rows the second product runs in the configuration it has on its own: the same bits.  Up to 16
        # rows its up rows walk in step with the gate rows in the one grid (half a row ahead on its own), and the
        # first product's rows are cut into other blocks in either: other orders of the sums along k, the same
        # values to rounding.
        assert rel(p1, y1) < 3e-3 and rel(p2, a2) < 3e-3, pair
        q1, q2 = ops.gemv_pair(xg, w1g, w2g, b1g, b2g)              # fixed summation orders: the same bits every run
        assert torch.equal(p1, q1) and torch.equal(p2, q2), pair
        if b > 16 or pair == 0:
            assert torch.equal(p2, a2), pair
        if pair == 0:
            assert torch.equal(p1, y1)
    ref1 = F.linear(x.float(), w1.float(), None if b1 is None else b1.float())
    pre = F.linear(x.float(), w2.float(), None if b2 is None else b2.float()).bfloat16().float()
    assert rel(y1, ref1) < TOL_BF16 and rel(a2, R.swiglu(pre)) < TOL_BF16


def _lib_bytes(b, n, k):
    from merak_amd import _lib
    return _lib.lib().mtp_gemv_workspace_bytes(b, n, k, _lib.EPI_NONE)


def test_argmax_ties_and_nan(gpu):
    k, n = 256, 999
    x = torch.randn(4, k, generator=gen(92)).bfloat16()
    w = (torch.randn(n, k, generator=gen(93)) * 0.02).bfloat16()
    ref = F.linear(x.float(), w.float())
    best = ref.argmax(-1)
    for b in range(4):                      # duplicate each winner's weight row at a lower and a higher index
        w[5 + b] = w[best[b]]
        w[900 + b] = w[best[b]]
    ref = F.linear(x.float(), w.float())
    idx, _ = ops.gemv_argmax(x.to(gpu), w.to(gpu))
    assert torch.equal(idx.cpu(), R.greedy_argmax(ref))     # exact ties: the first index wins
    assert all(int(i) <= 5 + 3 or int(i) == int(best[b]) for b, i in enumerate(idx.cpu()))
    # an all-zero activation row makes every logit equal: index 0, for every batch size class and k layout
    for bb, kk in ((1, 256), (20, 256), (3, 264)):
        wz = (torch.randn(n, kk, generator=gen(95)) * 0.02).bfloat16()
        xz = torch.randn(bb, kk, generator=gen(96)).bfloat16()
        xz[bb // 2] = 0
        iz, vz = ops.gemv_argmax(xz.to(gpu), wz.to(gpu))
        assert torch.equal(iz.cpu(), R.greedy_argmax(F.linear(xz.float(), wz.float()))) and int(iz[bb // 2]) == 0
        assert float(vz[bb // 2]) == 0.0
    logits = ref.clone()
    logits[1, 700] = float("nan"); logits[1, 800] = float("nan"); logits[2, 3] = float("inf")
    assert torch.equal(greedy_from_logits(logits.to(gpu)).cpu(), R.greedy_argmax(logits))
    assert torch.equal(greedy_from_logits(logits.bfloat16().to(gpu)).cpu(), R.greedy_argmax(logits.bfloat16()))


@pytest.mark.parametrize("b", [1, 8, 32])
def test_decode_step_llama8b_full_size(gpu, b):
    """Config 5: QKV 4096->6144, gate/up 4096->2x14336 (+SwiGLU), down 14336->4096, LM head 4096->128256."""
    g = torch.Generator(device=gpu).manual_seed(1241)
    mk = lambda n, k: torch.empty(n, k, device=gpu).normal_(0, 0.02, generator=g).bfloat16()
    wq, wg, wd, wl = mk(6144, 4096), mk(2 * 14336, 4096), mk(4096, 14336), mk(128256, 4096)
    x = torch.randn(b, 4096, generator=gen(94)).bfloat16()
    step = DecodeStep(wq, wg, wd, wl)
    qkv, out, tok = step(x.to(gpu))
    rq, ro, rlogits, rtok = R.decode_step(x, wq.cpu(), wg.cpu(), wd.cpu(), wl.cpu())
    assert rel(qkv, rq.float()) < TOL_BF16 and rel(out, ro.float()) < TOL_BF16
    # the greedy pick is compared on identical inputs to the LM head: feed the kernel's own `out`
    ref_tok = R.greedy_argmax(F.linear(out.cpu().float(), wl.cpu().float()))
    assert torch.equal(tok.cpu(), ref_tok)
    assert torch.equal(greedy_next_token(out, wl).cpu(), ref_tok)


# =============================================================================== sampling tail
@pytest.mark.parametrize("dtype,b,v,temp,top_k,top_p", [
    (torch.float32, 4, 1000, 1.0, 0, 0.0), (torch.float32, 4, 1000, 0.7, 10, 0.0), (torch.float32, 4, 1000, 1.3, 0, 0.9),
    (torch.float32, 8, 50257, 0.9, 50, 0.95), (torch.bfloat16, 8, 128256, 0.8, 40, 0.9),
    (torch.bfloat16, 3, 128256, 1.0, 0, 0.5), (torch.float32, 2, 7, 1.0, 3, 0.6), (torch.float32, 5, 1, 1.0, 1, 0.9),
    (torch.float32, 3, 300, 1.0, 300, 0.9999), (torch.bfloat16, 32, 32000, 0.6, 1, 0.0),
])
def test_sampling_filter_and_draw_vs_oracle(gpu, dtype, b, v, temp, top_k, top_p):
    """mtp_sample_top_k_top_p against the restated top_k_logits + softmax + inverse CDF: the filtered logits bit
    for bit (bf16 logits give many exactly equal values: a tie that straddles the top-p boundary is kept whole
    here, in part by the reference, so only such ties may differ), the drawn token for the same uniforms."""
    x = (torch.randn(b, v, generator=gen(100)) * 2.5).to(dtype)
    u = torch.rand(b, generator=gen(101))
    ref_tok, ref_probs = R.sample_tail(x.clone(), temp, top_k, top_p, u)
    ref_f = R.top_k_logits(x.float() / temp, top_k=top_k, top_p=top_p)
    tok, filt = ops.sample_top_k_top_p(x.to(gpu), temp, top_k, top_p, u.to(gpu), want_filtered=True)
    filt, tok = filt.cpu(), tok.cpu()
    kept, ref_kept = filt > -float("inf"), ref_f > -float("inf")
    assert torch.equal(filt[kept], (x.float() / temp)[kept]), "kept logits are float(x) / temperature, untouched"
    for r in range(b):
        diff = kept[r] != ref_kept[r]
        if diff.any():      # only members of the tie at the boundary value, and only kept in addition
            vals = (x.float() / temp)[r][diff]
            assert top_p > 0 and bool((vals == vals[0]).all()) and bool(kept[r][diff].all())
            assert float(vals[0]) == float(filt[r][kept[r]].min())
        else:
            assert int(tok[r]) == int(ref_tok[r]) or _near_cdf_step(ref_probs[r], float(u[r]))
        assert kept[r][tok[r]], "the drawn token is one that was kept"
    tok2, filt2 = ops.sample_top_k_top_p(x.to(gpu), temp, top_k, top_p, u.to(gpu), want_filtered=True)
    assert torch.equal(tok2.cpu(), tok) and torch.equal(filt2.cpu(), filt), "same inputs, same bits"


def _near_cdf_step(probs, u, eps=1e-5):
    cdf = torch.cumsum(probs, -1)
    return bool(((cdf - u * cdf[-1]).abs() < eps).any())


def test_sampling_follows_the_distribution_and_api(gpu):
    from merak_amd.inference import sample_next_token, top_k_logits
    x = torch.randn(1, 40, generator=gen(102))
    n = 32768
    xs = x.expand(n, 40).contiguous().to(gpu)
    us = torch.rand(n, generator=gen(103)).to(gpu)
    toks = sample_next_token(xs, temperature=0.9, top_k=12, top_p=0.0, uniforms=us)
    probs = R.sample_tail(x.clone(), 0.9, 12, 0.0, torch.zeros(1))[1][0]
    freq = torch.bincount(toks.cpu(), minlength=40).double() / n
    assert (freq - probs).abs().max() < 0.012 and bool((freq[probs == 0] == 0).all())
    # u = 0 draws the first kept token, u just below 1 the last one
    kept = (probs > 0).nonzero().flatten()
    ends = sample_next_token(xs[:2], 0.9, 12, 0.0, torch.tensor([0.0, 0.99999994], device=gpu)).cpu()
    assert int(ends[0]) == int(kept[0]) and int(ends[1]) == int(kept[-1])
    f = top_k_logits(xs[:3], top_k=5)
    assert torch.equal(f.cpu(), R.top_k_logits(x.expand(3, 40).clone(), top_k=5))
    assert sample_next_token(xs[:4], generator=torch.Generator(device=gpu).manual_seed(1)).shape == (4,)
    with pytest.raises(RuntimeError, match="temperature"):
        ops.sample_top_k_top_p(xs[:1], 0.0, 0, 0.0, us[:1])
    with pytest.raises(RuntimeError, match="out of range"):        # torch.topk's complaint in the reference
        ops.sample_top_k_top_p(xs[:1], 1.0, 41, 0.0, us[:1])
    with pytest.raises(ValueError):
        ops.sample_top_k_top_p(xs[:1])
    assert ops.sample_top_k_top_p(torch.empty(0, 9, device=gpu), 1.0, 0, 0.0, torch.empty(0, device=gpu))[0].numel() == 0


# =============================================================================== seeded shape sweeps
def _sweep_shapes(seed, count, lo, hi, mult):
    g = torch.Generator().manual_seed(seed)
    out = []
    for _ in range(count):
        m, n, k = (int(torch.randint(lo, hi, (1,), generator=g)) for _ in range(3))
        out.append((m, max(mult, n // mult * mult), max(mult, k // mult * mult)))
    return out


@pytest.mark.parametrize("dtype,mult", [(torch.bfloat16, 8), (torch.float32, 4), (torch.float32, 1), (torch.bfloat16, 1)])
def test_linear_shape_sweep(gpu, dtype, mult):
    """24 seeded shapes per case around the tile edges of every kernel (fast kernels take n, k multiples of
    8 / 4; anything else goes through the general kernel): forward with bias, dgrad, wgrad with bias gradient."""
    tol = TOL_F32 if dtype == torch.float32 else TOL_BF16
    for (m, n, k) in _sweep_shapes(7 + mult, 24, 1, 700, mult):
        x, w, b, dy = _lin_inputs(m, n, k, dtype, 200 + m + n + k)
        xf, wf, bf, dyf = x.float(), w.float(), b.float(), dy.float()
        y, _ = ops.linear_fwd(x.to(gpu), w.to(gpu), b.to(gpu), ops.EPI_BIAS)
        assert rel(y, R.column_parallel_linear_forward(xf, wf, bf)[0]) < tol, (m, n, k)
        rdx, rdw, rdb = R.linear_backward(xf, wf, dyf, True)
        assert rel(ops.linear_dgrad(dy.to(gpu), w.to(gpu)), rdx) < tol, (m, n, k)
        dw, db = ops.linear_wgrad(dy.to(gpu), x.to(gpu), True)
        assert rel(dw, rdw) < tol and rel(db, rdb) < tol, (m, n, k)


def test_gemv_shape_sweep(gpu):
    g = torch.Generator().manual_seed(11)
    for _ in range(24):
        b = int(torch.randint(1, 33, (1,), generator=g))
        n = int(torch.randint(1, 3000, (1,), generator=g))
        k = int(torch.randint(1, 300, (1,), generator=g)) * 8
        x = torch.randn(b, k, generator=g).bfloat16()
        w = (torch.randn(n, k, generator=g) * 0.05).bfloat16()
        ref = F.linear(x.float(), w.float())
        assert rel(ops.gemv(x.to(gpu), w.to(gpu)), ref) < TOL_BF16, (b, n, k)
        idx, val = ops.gemv_argmax(x.to(gpu), w.to(gpu))
        assert torch.equal(idx.cpu(), R.greedy_argmax(ref)), (b, n, k)
        if n % 2 == 0:
            sw = ops.gemv(x.to(gpu), w.to(gpu), None, ops.EPI_SWIGLU)
            y = ref.bfloat16().float()
            assert rel(sw, F.silu(y[:, : n // 2]) * y[:, n // 2:]) < TOL_BF16, (b, n, k)


def test_ce_shape_sweep(gpu):
    g = torch.Generator().manual_seed(12)
    for i in range(16):
        dtype = torch.bfloat16 if i % 2 else torch.float32
        n = int(torch.randint(1, 40, (1,), generator=g))
        v = int(torch.randint(1, 70000, (1,), generator=g))
        start = int(torch.randint(0, 3, (1,), generator=g)) * v
        x = (torch.randn(n, v, generator=g) * 3).to(dtype)
        t = torch.randint(0, 3 * v, (n,), generator=g)
        gr = torch.rand(n, generator=g)
        ref_loss, ref_grad = R.cross_entropy_fp32(x, t, start, gr)
        tol = TOL_F32 if dtype == torch.float32 else TOL_BF16
        a = x.to(gpu)
        loss, m, s, _ = ops.vocab_ce_fwd(a, t.to(gpu), start)
        ops.vocab_ce_bwd_(a, t.to(gpu), m, s, gr.to(gpu), start)
        b2 = x.to(gpu)
        loss2, *_ = ops.vocab_ce_fwd_bwd_(b2, t.to(gpu), start, gr.to(gpu), 1.0)
        for lo, gx in ((loss, a), (loss2, b2)):
            assert (lo.cpu() - ref_loss).abs().max() <= TOL_LOSS * max(ref_loss.abs().max().item(), 0.1), (n, v, dtype)
            assert rel(gx, ref_grad) < tol, (n, v, dtype)


# =============================================================================== a small training loop
class _TorchBlock(torch.nn.Module):
    """The same tiny model in stock PyTorch fp32: embedding -> Linear+gelu_new -> Linear -> LM head -> cross entropy."""

    def __init__(self, v, h, f):
        super().__init__()
        self.emb = torch.nn.Embedding(v, h)
        self.fc = torch.nn.Linear(h, f)
        self.proj = torch.nn.Linear(f, h)
        self.head = torch.nn.Linear(h, v, bias=False)

    def forward(self, ids, labels):
        x = self.emb(ids)
        x = x + self.proj(R.gelu_new(self.fc(x)))
        logits = self.head(x)
        return F.cross_entropy(logits.view(-1, logits.shape[-1]), labels.view(-1))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_training_loop_matches_stock_pytorch(gpu, dtype):
    """Six SGD steps of a small block built from this package's layers the way Merak builds them (tagged nn.Linear
    -> build_layers -> ColPara / RowPara, VocabParallelEmbedding, vocab-parallel LM head, vocab_loss_fn) against
    the same block in stock PyTorch fp32 on the CPU, from identical initial weights and batches: the loss
    curves must agree (fp32: to 1e-4; bf16 parameters: to bf16 training noise)."""
    from merak_amd.tensor_parallel import build_layers
    v, h, f, b, s = 1000, 128, 512, 4, 24
    set_args(use_cpu_initialization=True, params_dtype=dtype)
    torch.manual_seed(11)
    ref = _TorchBlock(v, h, f)
    init = lambda t: torch.nn.init.normal_(t, 0.0, 0.02)
    fc, proj = torch.nn.Linear(h, f), torch.nn.Linear(f, h)
    fc.mp_attr, proj.mp_attr = "col_mlp", "row_mlp"
    col, row = build_layers("fc", fc, 1, init, init), build_layers("proj", proj, 1, init, init)
    emb = mpu.VocabParallelEmbedding(v, h, init_method=init)
    head = mpu.ColumnParallelLinear(h, v, bias=False, gather_output=False, init_method=init)
    with torch.no_grad():       # identical starting point
        emb.weight.copy_(ref.emb.weight); head.weight.copy_(ref.head.weight)
        col.weight.copy_(ref.fc.weight); col.bias.copy_(ref.fc.bias)
        row.weight.copy_(ref.proj.weight); row.bias.copy_(ref.proj.bias)
        if dtype == torch.bfloat16:   # the reference starts from the same rounded values
            for p, q in ((ref.emb.weight, emb.weight), (ref.head.weight, head.weight), (ref.fc.weight, col.weight),
                         (ref.fc.bias, col.bias), (ref.proj.weight, row.weight), (ref.proj.bias, row.bias)):
                p.copy_(q.float())
    mods = torch.nn.ModuleList([emb, col, row, head]).to(gpu)
    assert set(dict(col.named_parameters())) == {"col_linear.weight", "col_linear.bias"}
    opt_ref = torch.optim.SGD(ref.parameters(), lr=0.5)
    opt = torch.optim.SGD(mods.parameters(), lr=0.5)
    g = gen(120)
    losses, ref_losses = [], []
    for step in range(6):
        ids = torch.randint(0, v, (b, s), generator=g)
        labels = torch.randint(0, v, (b, s), generator=g)
        opt_ref.zero_grad(); lr_ = ref(ids, labels); lr_.backward(); opt_ref.step(); ref_losses.append(lr_.item())
        opt.zero_grad()
        x = emb(ids.to(gpu))
        x = x + row(R.gelu_new(col(x)))                 # ColPara / RowPara return the output only (mp_layers.py:121,176)
        logits, _ = head(x)
        loss = mpu.vocab_loss_fn((logits,), (labels.to(gpu),))
        loss.backward(); opt.step(); losses.append(loss.item())
    tol = 1e-4 if dtype == torch.float32 else 3e-2
    assert all(abs(a - b_) <= tol * abs(b_) for a, b_ in zip(losses, ref_losses)), (losses, ref_losses)
    assert ref_losses[-1] < ref_losses[0] - 0.05, "the reference loop itself must be learning"


def test_tagged_model_rebuilt_onto_the_gfx950_layers(gpu):
    """The reference's sequence (feature lists -> set_mp_attr -> module rebuild, mp_attrs.py:43-202,
    model_parallel.py:87-99) at tensor-parallel degree 1: the rebuilt MLP, given the original weights, computes
    what the stock torch modules compute, forward and backward."""
    from merak_amd.tensor_parallel import (set_tp_layer_lists, set_mp_attr, rebuild_module, reset_tp_layer_lists,
                                           init_method_normal, scaled_init_method_normal, ColPara, RowPara)

    class MLP(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.fc_in, self.fc_out = torch.nn.Linear(256, 1024), torch.nn.Linear(1024, 256)

        def forward(self, x):
            return self.fc_out(F.gelu(self.fc_in(x), approximate="tanh"))

    torch.manual_seed(5)
    stock = MLP()
    x = torch.randn(3, 50, 256)
    xs = x.clone().requires_grad_(True)
    ref = stock(xs)
    ref.backward(torch.ones_like(ref))
    reset_tp_layer_lists()
    set_tp_layer_lists(col_para_list=["fc_in"], row_para_list=["fc_out"])
    set_args(use_cpu_initialization=True, params_dtype=torch.float32)
    mine = rebuild_module(set_mp_attr(MLP(), 1), 1, init_method_normal(0.02), scaled_init_method_normal(0.02, 1))
    reset_tp_layer_lists()
    assert isinstance(mine.fc_in, ColPara) and isinstance(mine.fc_out, RowPara)
    missing = mine.load_state_dict({k.replace("fc_in.", "fc_in.col_linear.").replace("fc_out.", "fc_out.row_linear."): v
                                    for k, v in stock.state_dict().items()})
    assert not missing.missing_keys and not missing.unexpected_keys
    mine.to(gpu)
    xg = x.to(gpu).requires_grad_(True)
    out = mine(xg)
    out.backward(torch.ones_like(out))
    assert rel(out, ref) < TOL_F32 and rel(xg.grad, xs.grad) < TOL_F32
    assert rel(mine.fc_in.weight.grad, stock.fc_in.weight.grad) < TOL_F32
    assert rel(mine.fc_out.bias.grad, stock.fc_out.bias.grad) < TOL_F32


def test_greedy_pick_over_a_vocab_sharded_lm_head(gpu):
    """Eight ranks' vocab slices of an LM head, each through the fused GEMV + argmax: one (max value, local index)
    pair per row and rank, combined on the host the way an all-gather would allow (largest value, lowest rank on
    equality), gives the full head's pick."""
    g = gen(77)
    B, V, K, p = 8, 8 * 1003, 512, 8
    x = torch.randn(B, K, generator=g).bfloat16()
    w = (torch.randn(V, K, generator=g) * 0.05).bfloat16()
    w[5000] = w[1200]                                            # an exact tie across two ranks' slices
    x[3] = (w[1200].float() * 4).bfloat16()                      # row 3 picks the tied rows
    full_idx, full_val = ops.gemv_argmax(x.to(gpu), w.to(gpu))
    vals, idxs = [], []
    for r in range(p):
        lo, hi = R.vocab_range_from_global_vocab_size(V, r, p)
        i, v = ops.gemv_argmax(x.to(gpu), w[lo:hi].contiguous().to(gpu))
        vals.append(v.cpu())
        idxs.append(i.cpu() + lo)
    vals, idxs = torch.stack(vals), torch.stack(idxs)            # [ranks, B]
    win = vals.argmax(0)                                         # first (lowest) rank among equal maxima
    got = idxs[win, torch.arange(B)]
    ref = R.greedy_argmax(F.linear(x.float(), w.float()))
    clear = torch.ones(B, dtype=torch.bool)
    clear[3] = False
    assert torch.equal(got[clear], ref[clear]) and torch.equal(full_idx.cpu()[clear], ref[clear])
    assert int(got[3]) in (1200, 5000) and int(ref[3]) == 1200   # the tie: equal to rounding across workgroups
    assert torch.allclose(vals.max(0).values, full_val.cpu(), rtol=1e-5)


@pytest.mark.parametrize("mix", ["1", "2", "3", "4", "5", "6", "7", None])
@pytest.mark.parametrize("b,half,k,with_bias", [(1, 14336, 4096, False), (8, 1000, 1024, True), (16, 56, 512, False),
                                                (3, 3584, 8192, False), (32, 14336, 4096, False), (17, 1000, 1024, True),
                                                (25, 100, 512, False)])
def test_gemv_swiglu_mixed_row_groups(gpu, set_tuning, mix, b, half, k, with_bias):
    """SwiGLU GEMV whose 16-row tiles hold 8 gate rows and their 8 up rows, for every number of groups per
    workgroup (forced) and for the automatic choice: same result as the oracle, ragged ends included, with one
    batch tile (up rows half a row ahead of the gate rows, two products per tile) and with two (rows in step)."""
    if mix is not None:
        set_tuning("MTP_GEMV_MIX", mix)
    g = gen(41)
    x = torch.randn(b, k, generator=g).bfloat16()
    w = (torch.randn(2 * half, k, generator=g) * 0.03).bfloat16()
    bias = (torch.randn(2 * half, generator=g) * 0.1).bfloat16() if with_bias else None
    pre = F.linear(x.float(), w.float(), None if bias is None else bias.float()).bfloat16().float()
    y = ops.gemv(x.to(gpu), w.to(gpu), None if bias is None else bias.to(gpu), ops.EPI_SWIGLU)
    assert y.shape == (b, half) and rel(y, R.swiglu(pre)) < TOL_BF16
    assert torch.equal(y, ops.gemv(x.to(gpu), w.to(gpu), None if bias is None else bias.to(gpu), ops.EPI_SWIGLU))


def test_gemv_swiglu_seeded_sweep(gpu):
    """30 seeded SwiGLU GEMV shapes (any batch up to 32, ragged halves, k multiples of 8) against the oracle."""
    g = gen(43)
    for case in range(30):
        b = int(torch.randint(1, 33, (1,), generator=g))
        half = int(torch.randint(1, 3000, (1,), generator=g))
        k = 8 * int(torch.randint(1, 600, (1,), generator=g))
        if case % 3 == 0:
            k = 512 * int(torch.randint(1, 9, (1,), generator=g))           # the shapes the mixed row groups take
        x = torch.randn(b, k, generator=g).bfloat16()
        w = (torch.randn(2 * half, k, generator=g) * 0.03).bfloat16()
        pre = F.linear(x.float(), w.float()).bfloat16().float()
        y = ops.gemv(x.to(gpu), w.to(gpu), None, ops.EPI_SWIGLU)
        assert rel(y, R.swiglu(pre)) < TOL_BF16, (case, b, half, k)


def test_wrappers_reject_mismatched_shapes_before_any_launch(gpu):
    """Pointers carry no shape: the tensor-level wrappers are where a mismatch must stop."""
    bf = dict(device=gpu, dtype=torch.bfloat16)
    x, w = torch.zeros(4, 64, **bf), torch.zeros(32, 64, **bf)
    with pytest.raises(ValueError, match="bias"):
        ops.linear_fwd(x, w, torch.zeros(31, **bf), ops.EPI_BIAS)
    with pytest.raises(ValueError, match="even"):
        ops.linear_fwd(x, torch.zeros(31, 64, **bf), None, ops.EPI_SWIGLU)
    with pytest.raises(ValueError):
        ops.linear_fwd(x.view(2, 2, 64), w, None)
    with pytest.raises(ValueError, match="db"):
        ops.linear_wgrad(torch.zeros(4, 32, **bf), x, True, dw=torch.zeros(32, 64, **bf), db=torch.zeros(8, **bf))
    with pytest.raises(ValueError, match="dact"):
        ops.activation_bwd(torch.zeros(4, 32, **bf), torch.zeros(4, 32, **bf), ops.EPI_SWIGLU)
    ids = torch.zeros(6, dtype=torch.int64, device=gpu)
    with pytest.raises(ValueError, match="gradient rows"):
        ops.embedding_bwd(ids, torch.zeros(5, 16, **bf), 10, 0, 10)
    with pytest.raises(ValueError, match="vocab range"):
        ops.embedding_bwd(ids, torch.zeros(6, 16, **bf), 12, 0, 10)
    with pytest.raises(ValueError, match=r"\[B, K\]"):
        ops.gemv(torch.zeros(2, 32, **bf), w)
    with pytest.raises(ValueError, match="bias"):
        ops.gemv(torch.zeros(2, 64, **bf), w, torch.zeros(16, **bf), ops.EPI_BIAS)
    with pytest.raises(ValueError, match=r"\[B, K\]"):
        ops.gemv_argmax(torch.zeros(2, 128, **bf), w)
    lg, t = torch.zeros(4, 8, device=gpu), torch.zeros(4, dtype=torch.int64, device=gpu)
    with pytest.raises(ValueError, match="row_max"):
        ops.vocab_ce_bwd_(lg, t, torch.zeros(3, device=gpu), torch.zeros(4, device=gpu), None, 0)
    with pytest.raises(ValueError, match="grad_out"):
        ops.vocab_ce_bwd_(lg, t, None, None, torch.zeros(5, device=gpu), 0)
    with pytest.raises(TypeError):
        ops.vocab_ce_bwd_(lg, t.int(), None, None, None, 0)
