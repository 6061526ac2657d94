"""Seeded random shapes through the linear, decode and cross-entropy entry points against the CPU oracle.

The fixed cases of test_gpu_parity.py sit on tile and vector boundaries chosen by hand; these draw M, N, K,
batch and vocabulary sizes at random (fixed seeds) so that any combination of ragged edges meets every
epilogue and element type.  Tolerances: fp32 1e-4, bf16 1.2e-2, fp16 3e-3 (relative Frobenius error against
the fp32 oracle on the same rounded inputs), argmax indices exact wherever the oracle's top two logits are
further apart than the 16-bit rounding of the product.
"""
import random

import pytest
import torch

from merak_amd import mpu, ops
from oracle import tp_reference as R

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-4, torch.bfloat16: 1.2e-2, torch.float16: 3e-3}


def rel(got, ref):
    got, ref = got.detach().double().cpu(), ref.detach().double().cpu()
    return ((got - ref).norm() / ref.norm().clamp_min(1e-300)).item()


def _dim(rng):
    r = rng.random()
    if r < 0.3:
        return rng.randint(1, 64)
    if r < 0.8:
        return rng.randint(1, 700)
    return rng.choice([255, 256, 257, 511, 512, 513, 768, 1023, 1024, 1025, 1280])


@pytest.mark.parametrize("seed", range(6))
def test_linear_random_shapes(gpu, seed):
    rng = random.Random(100 + seed)
    g = torch.Generator().manual_seed(500 + seed)
    for case in range(10):
        dt = rng.choice([torch.bfloat16, torch.bfloat16, torch.float16, torch.float32])
        M, N, K = _dim(rng), _dim(rng), _dim(rng)
        if rng.random() < 0.7:
            K = max(8, K // 8 * 8)
        epi = rng.choice([ops.EPI_NONE, ops.EPI_BIAS, ops.EPI_BIAS_GELU, ops.EPI_SWIGLU, ops.EPI_GELU])
        if epi == ops.EPI_SWIGLU:
            N = max(2, N // 2 * 2)
        tag = f"seed {seed} case {case}: {dt} M={M} N={N} K={K} epilogue={epi}"
        x = torch.randn(M, K, generator=g).to(dt)
        w = (torch.randn(N, K, generator=g) * 0.05).to(dt)
        b = (torch.randn(N, generator=g) * 0.1).to(dt) if epi in (ops.EPI_BIAS, ops.EPI_BIAS_GELU) else None
        dy = torch.randn(M, N, generator=g).to(dt)
        # oracle: the reference's op order in fp32 on the same rounded values
        ref_y, _ = R.column_parallel_linear_forward(x.float(), w.float(), None if b is None else b.float())
        ref_pre = ref_y.to(dt).float()     # the activation sees the stored (rounded) pre-activation
        ref_dx, ref_dw, ref_db = R.linear_backward(x.float(), w.float(), dy.float(), True)

        xg, wg, dyg = x.to(gpu), w.to(gpu), dy.to(gpu)
        y, act = ops.linear_fwd(xg, wg, None if b is None else b.to(gpu), epi, want_pre=True)
        errs = {"y": rel(y, ref_y)}
        if epi in (ops.EPI_BIAS_GELU, ops.EPI_GELU):
            errs["act"] = rel(act, R.gelu_new(ref_pre))
        if epi == ops.EPI_SWIGLU:
            errs["act"] = rel(act, R.swiglu(ref_pre))
        errs["dx"] = rel(ops.linear_dgrad(dyg, wg), ref_dx)
        out_dtype = rng.choice([None, torch.float32])
        dw, db = ops.linear_wgrad(dyg, xg, True, out_dtype=out_dtype)
        errs["dw"], errs["db"] = rel(dw, ref_dw), rel(db, ref_db)
        if out_dtype is torch.float32:
            # main-gradient form: a second micro-batch accumulates into the fp32 buffers
            ops.linear_wgrad(dyg, xg, True, dw=dw, db=db, accumulate=True)
            errs["dw_acc"], errs["db_acc"] = rel(dw, 2 * ref_dw), rel(db, 2 * ref_db)
        assert max(errs.values()) < TOL[dt], (tag, errs)


@pytest.mark.parametrize("seed", range(4))
def test_decode_products_random_shapes(gpu, seed):
    rng = random.Random(200 + seed)
    g = torch.Generator().manual_seed(600 + seed)
    for case in range(10):
        dt = rng.choice([torch.bfloat16, torch.bfloat16, torch.float16])
        B = rng.choice([1, 2, 3, 7, 8, 9, 15, 16, 17, 31, 32])
        N = rng.choice([rng.randint(1, 300), rng.randint(1, 5000), 4096, 1280, 2 * rng.randint(1, 3000)])
        K = rng.choice([rng.randint(1, 64) * 8, rng.randint(1, 40) * 64, 4096, 8192, 3584, rng.randint(1, 2000) * 8])
        epi = rng.choice([ops.EPI_NONE, ops.EPI_NONE, ops.EPI_BIAS, ops.EPI_SWIGLU])
        if epi == ops.EPI_SWIGLU:
            N = max(2, N // 2 * 2)
        tag = f"seed {seed} case {case}: {dt} B={B} N={N} K={K} epilogue={epi}"
        x = torch.randn(B, K, generator=g).to(dt)
        w = (torch.randn(N, K, generator=g) * 0.05).to(dt)
        b = (torch.randn(N, generator=g) * 0.1).to(dt) if epi == ops.EPI_BIAS else None
        ref, _ = R.column_parallel_linear_forward(x.float(), w.float(), None if b is None else b.float())
        ref_out = R.swiglu(ref.to(dt).float()) if epi == ops.EPI_SWIGLU else ref
        xg, wg = x.to(gpu), w.to(gpu)
        ws = ops.gemv_workspace(B, N, K, epi, gpu) if rng.random() < 0.5 else None
        for launch in range(2 if ws is not None else 1):   # a workspace comes back clean for the next launch
            y = ops.gemv(xg, wg, None if b is None else b.to(gpu), epi, workspace=ws)
            assert rel(y, ref_out) < TOL[dt], (tag, launch)
        logits = x.float() @ w.float().t()
        idx, val = ops.gemv_argmax(xg, wg)
        assert rel(val, logits.max(-1).values) < TOL[dt], tag
        top2 = logits.topk(min(2, N), dim=-1).values
        clear = (top2[:, 0] - top2[:, -1]) > 1e-3 * top2[:, 0].abs().clamp_min(1e-3) if N > 1 else torch.ones(B, dtype=torch.bool)
        assert bool(((idx.cpu() == R.greedy_argmax(logits)) | ~clear).all()), tag


@pytest.mark.parametrize("seed", range(3))
def test_product_pair_random_shapes(gpu, seed):
    """mtp_gemv_pair on drawn shapes: second products that fill the chip with mixed SwiGLU groups (one grid, the
    first product's rows as one or two more row groups in the loop, or more rows than that holds: two launches) and
    ones that do not, every batch size class, ragged row counts, with and without biases."""
    rng = random.Random(300 + seed)
    g = torch.Generator(device=gpu).manual_seed(700 + seed)
    for case in range(8):
        dt = rng.choice([torch.bfloat16, torch.bfloat16, torch.float16])
        B = rng.choice([1, 5, 8, 16, 17, 24, 32])
        K = rng.choice([512, 1024, 2048, 1536, 520])
        wgs = rng.choice([200, 230, 250, 256, 100])
        half = 56 * wgs - rng.choice([0, 0, 3, 17, 55])
        if rng.random() < 0.25:
            half = rng.randint(1, 3000)
        n1 = rng.choice([rng.randint(1, 16 * wgs), rng.randint(16 * wgs, 32 * wgs), rng.randint(32 * wgs, 40 * wgs)])
        bias = rng.random() < 0.4
        tag = f"seed {seed} case {case}: {dt} B={B} K={K} half={half} n1={n1} bias={bias}"
        x = torch.randn(B, K, device=gpu, generator=g).to(dt)
        w1 = (torch.randn(n1, K, device=gpu, generator=g) * 0.03).to(dt)
        w2 = (torch.randn(2 * half, K, device=gpu, generator=g) * 0.03).to(dt)
        b1 = (torch.randn(n1, device=gpu, generator=g) * 0.1).to(dt) if bias else None
        b2 = (torch.randn(2 * half, device=gpu, generator=g) * 0.1).to(dt) if bias else None
        y1, a2 = ops.gemv_pair(x, w1, w2, b1, b2)
        assert y1.shape == (B, n1) and a2.shape == (B, half), tag
        cpu = lambda t: None if t is None else t.cpu().float()
        r1, _ = R.column_parallel_linear_forward(cpu(x), cpu(w1), cpu(b1))
        pre, _ = R.column_parallel_linear_forward(cpu(x), cpu(w2), cpu(b2))
        assert rel(y1, r1) < TOL[dt] and rel(a2, R.swiglu(pre.to(dt).float())) < TOL[dt], tag


@pytest.mark.parametrize("seed", range(3))
def test_cross_entropy_random_shapes(gpu, seed):
    rng = random.Random(300 + seed)
    g = torch.Generator().manual_seed(700 + seed)
    for case in range(12):
        dt = rng.choice([torch.float32, torch.bfloat16, torch.float16])
        n = rng.choice([1, 2, 5, 64, 300])
        v = rng.choice([2, 7, 100, 1000, 4097, 32000, 50257, rng.randint(2, 70000)])
        tag = f"seed {seed} case {case}: {dt} n={n} v={v}"
        logits = (torch.randn(n, v, generator=g) * 3).to(dt)
        t = torch.randint(-5, v + 5, (n,), generator=g)      # a few targets outside the vocabulary
        t[rng.randrange(n)] = -100
        go = torch.randn(n, generator=g)
        ref_loss, ref_grad = R.cross_entropy_fp32(logits, t, 0, go)
        lg = logits.to(gpu).requires_grad_(True)
        loss = mpu.vocab_parallel_cross_entropy(lg * 1.0, t.to(gpu))
        loss.backward(go.to(gpu).to(loss.dtype))
        assert rel(loss, ref_loss) < 1e-5, tag
        assert rel(lg.grad, ref_grad) < TOL[dt], tag
