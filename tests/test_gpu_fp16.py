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


# ---- the decode kernels in IEEE half ----
@pytest.mark.parametrize("b,n,k,epi", [(1, 4096, 4096, "none"), (8, 1000, 512, "bias"), (32, 2048, 1024, "swiglu"),
                                       (32, 4096, 14336, "none"), (5, 130, 4104, "none")])
def test_gemv_and_fused_argmax_fp16(gpu, b, n, k, epi):
    g = gen(21)
    x = torch.randn(b, k, generator=g).to(H)
    w = (torch.randn(n, k, generator=g) * 0.02).to(H)
    bias = (torch.randn(n, generator=g) * 0.1).to(H) if epi == "bias" else None
    e = {"none": ops.EPI_NONE, "bias": ops.EPI_BIAS, "swiglu": ops.EPI_SWIGLU}[epi]
    ref = F.linear(x.float(), w.float(), None if bias is None else bias.float())
    ws = ops.gemv_workspace(b, n, k, e, gpu)
    y = ops.gemv(x.to(gpu), w.to(gpu), None if bias is None else bias.to(gpu), e, workspace=ws)
    assert y.dtype == H and rel(y, R.swiglu(ref.to(H).float()) if epi == "swiglu" else ref) < TOL_F16
    if epi == "none":
        idx, val = ops.gemv_argmax(x.to(gpu), w.to(gpu))
        top2 = ref.topk(2, dim=-1).values
        clear = (top2[:, 0] - top2[:, 1]) > 1e-3 * top2[:, 0].abs()
        assert torch.equal(idx.cpu()[clear], ref.argmax(-1)[clear])
        assert torch.allclose(val.cpu(), ref.max(-1).values, rtol=1e-3, atol=1e-4)
    with pytest.raises(TypeError):
        ops.gemv(x.to(gpu), w.bfloat16().to(gpu))                 # mixed 16-bit dtypes


@pytest.mark.parametrize("b", [4, 32])
def test_gemv_pair_fp16(gpu, b):
    """QKV-like and gate/up-like products in one grid (the first product's rows inside the loop of the mixed SwiGLU
    groups), one and two batch tiles, ragged row counts, in IEEE half: against the oracle."""
    g = gen(27)
    n1, half, k = 3016, 14000, 2048
    x = torch.randn(b, k, generator=g).to(H)
    w1 = (torch.randn(n1, k, generator=g) * 0.02).to(H)
    w2 = (torch.randn(2 * half, k, generator=g) * 0.02).to(H)
    y1, a2 = ops.gemv_pair(x.to(gpu), w1.to(gpu), w2.to(gpu))
    assert y1.dtype == H and a2.dtype == H
    assert rel(y1, F.linear(x.float(), w1.float())) < TOL_F16
    assert rel(a2, R.swiglu(F.linear(x.float(), w2.float()).to(H).float())) < TOL_F16


def test_rmsnorm_rope_attention_fp16(gpu):
    from merak_amd.inference import rope_tables
    g = gen(22)
    x, r = (torch.randn(4, 4096, generator=g) * 2).to(H), torch.randn(4, 4096, generator=g).to(H)
    wn = (torch.rand(4096, generator=g) + 0.5).to(H)
    y, h = ops.rmsnorm(x.to(gpu), wn.to(gpu), 1e-5, r.to(gpu), want_residual=True)
    ref_y, _ = R.rms_norm(x.float(), wn.float(), 1e-5, r.float())
    assert torch.equal(h.cpu(), r + x) and rel(y, ref_y) < TOL_F16
    B, n_q, n_kv, d, L = 3, 8, 2, 128, 700
    qkv = torch.randn(B, (n_q + 2 * n_kv) * d, generator=g).to(H)
    kc0, vc0 = torch.randn(B, n_kv, L, d, generator=g).to(H), torch.randn(B, n_kv, L, d, generator=g).to(H)
    cos, sin = rope_tables(d, L, 500000.0, dtype=H)
    pos = torch.tensor([699, 0, 300])
    heads = qkv.float().view(B, n_q + 2 * n_kv, d)
    cf, sf = cos.float()[pos], sin.float()[pos]
    kf, vf = kc0.float(), vc0.float()
    for b in range(B):
        kf[b, :, pos[b]] = R.apply_rope(heads[:, n_q:n_q + n_kv], cf, sf)[b]
        vf[b, :, pos[b]] = heads[b, n_q + n_kv:]
    want = R.attn_decode(R.apply_rope(heads[:, :n_q], cf, sf), kf, vf, pos + 1)
    k1, v1, k2, v2 = kc0.to(gpu), vc0.to(gpu), kc0.to(gpu), vc0.to(gpu)
    out = ops.attn_decode_append(qkv.to(gpu), cos.to(gpu), sin.to(gpu), pos.to(gpu), k1, v1, n_q)
    assert out.dtype == H and rel(out, want) < TOL_F16
    q = ops.rope_kv_append(qkv.to(gpu), cos.to(gpu), sin.to(gpu), pos.to(gpu), k2, v2, n_q)
    assert torch.equal(k1, k2) and torch.equal(v1, v2)
    assert rel(ops.attn_decode(q, k2, v2, (pos + 1).to(gpu)), want) < TOL_F16


def test_sampling_and_argmax_rows_fp16(gpu):
    g = gen(23)
    logits = (torch.randn(4, 5000, generator=g) * 3).to(H)
    u = torch.rand(4, generator=g)
    ref_tok, ref_probs = R.sample_tail(logits.clone(), 0.7, 40, 0.9, u)
    tok, filt = ops.sample_top_k_top_p(logits.to(gpu), 0.7, 40, 0.9, u.to(gpu), want_filtered=True)
    ref_filt = R.top_k_logits(logits.float() / 0.7, 40, 0.9)
    kept, ref_kept = filt.cpu() > -float("inf"), ref_filt > -float("inf")
    assert (kept | ~ref_kept).all()                                  # ties at the top-p boundary may only add
    assert torch.equal(filt.cpu()[ref_kept], ref_filt[ref_kept])
    assert int((tok.cpu() == ref_tok).sum()) >= 3
    assert torch.equal(ops.argmax_rows(logits.to(gpu)).cpu(), logits.float().argmax(-1))


def test_llama_decoder_fp16_matches_full_sequence_forward(gpu):
    """The cached decoder on an fp16 model against the fp32 full-sequence forward of the library model."""
    from transformers import LlamaConfig, LlamaForCausalLM
    from merak_amd.inference import LlamaDecoder
    torch.manual_seed(31)
    cfg = LlamaConfig(hidden_size=512, intermediate_size=1024, num_attention_heads=4, num_key_value_heads=2,
                      head_dim=128, num_hidden_layers=2, vocab_size=1000, max_position_embeddings=128,
                      rope_theta=10000.0, rms_norm_eps=1e-5, attn_implementation="eager", tie_word_embeddings=False)
    model = LlamaForCausalLM(cfg).eval()
    for p_ in model.parameters():
        if p_.dim() == 1:
            p_.data.uniform_(0.5, 1.5)
        p_.data = p_.data.to(H).float()
    ids = torch.randint(0, cfg.vocab_size, (2, 24), generator=gen(31))
    with torch.no_grad():
        full = model(input_ids=ids).logits
    dec = LlamaDecoder.from_hf(model.half().to(gpu), max_len=32, batch=2)
    worst = 0.0
    for t in range(24):
        lg = dec.logits(ids[:, t].to(gpu))
        assert lg.dtype == H
        worst = max(worst, rel(lg, full[:, t]))
    assert worst < 4 * TOL_F16, worst
