"""GPU parity of the cached single-position step (RMSNorm, rotary + cache append, attention over the cache,
the whole Llama block and model) against the CPU oracle, through the C ABI.

Tolerances: bf16 results 1e-2 relative (norm-wise) against the oracle's fp32 arithmetic on the same bf16
inputs; fp32 RMSNorm 1e-4; copies (the value rows of the cache, untouched cache rows) bit-exact.
"""
import os

import pytest
import torch

from merak_amd import ops
from merak_amd.inference import LlamaDecoder, rope_tables
from oracle import tp_reference as R

pytestmark = pytest.mark.gpu
TOL_F32, TOL_BF16 = 1e-4, 1e-2


def rel(got, ref):
    got, ref = got.detach().double().cpu(), ref.detach().double().cpu()
    return ((got - ref).norm() / ref.norm().clamp_min(1e-300)).item()


def gen(seed):
    return torch.Generator().manual_seed(4321 + seed)


@pytest.mark.parametrize("dtype,rows,dim", [(torch.bfloat16, 1, 4096), (torch.bfloat16, 32, 4096), (torch.bfloat16, 5, 1000),
                                            (torch.float32, 3, 768), (torch.bfloat16, 2, 8192), (torch.float32, 1, 7)])
def test_rmsnorm(gpu, dtype, rows, dim):
    g = gen(1)
    x = (torch.randn(rows, dim, generator=g) * 3).to(dtype)
    r = torch.randn(rows, dim, generator=g).to(dtype)
    w = (torch.rand(dim, generator=g) + 0.5).to(dtype)
    tol = TOL_F32 if dtype == torch.float32 else TOL_BF16
    y = ops.rmsnorm(x.to(gpu), w.to(gpu), 1e-5)
    assert y.dtype == dtype and rel(y, R.rms_norm(x.float(), w.float(), 1e-5)[0]) < tol
    y, h = ops.rmsnorm(x.to(gpu), w.to(gpu), 1e-5, r.to(gpu), want_residual=True)
    ref_y, ref_h = R.rms_norm(x.float(), w.float(), 1e-5, r.float())
    assert torch.equal(h.cpu(), (r + x))            # the sum is rounded as the tensor expression rounds it
    assert rel(y, ref_y) < tol
    with pytest.raises(ValueError):
        ops.rmsnorm(x.to(gpu), w[:-1].to(gpu), 1e-5)


@pytest.mark.parametrize("B,n_q,n_kv", [(1, 32, 8), (5, 8, 1), (32, 4, 4)])
def test_rope_kv_append(gpu, B, n_q, n_kv):
    g = gen(2)
    d, L = 128, 64
    qkv = torch.randn(B, (n_q + 2 * n_kv) * d, generator=g).bfloat16()
    cos, sin = rope_tables(d, L, 500000.0, dtype=torch.bfloat16)
    pos = torch.randint(0, L, (B,), generator=g)
    kc0 = torch.randn(B, n_kv, L, d, generator=g).bfloat16()
    vc0 = torch.randn(B, n_kv, L, d, generator=g).bfloat16()
    kc, vc = kc0.to(gpu), vc0.to(gpu)
    q = ops.rope_kv_append(qkv.to(gpu), cos.to(gpu), sin.to(gpu), pos.to(gpu), kc, vc, n_q)
    heads = qkv.float().view(B, n_q + 2 * n_kv, d)
    cf, sf = cos.float()[pos], sin.float()[pos]
    assert rel(q, R.apply_rope(heads[:, :n_q], cf, sf)) < TOL_BF16
    ref_k = R.apply_rope(heads[:, n_q:n_q + n_kv], cf, sf)
    kc, vc = kc.cpu(), vc.cpu()
    for b in range(B):
        p = int(pos[b])
        assert rel(kc[b, :, p], ref_k[b]) < TOL_BF16
        assert torch.equal(vc[b, :, p], qkv.view(B, -1, d)[b, n_q + n_kv:])        # values are copied
        keep = torch.ones(L, dtype=torch.bool)
        keep[p] = False
        assert torch.equal(kc[b][:, keep], kc0[b][:, keep]) and torch.equal(vc[b][:, keep], vc0[b][:, keep])
    # a position outside the cache leaves everything as it was
    kc, vc = kc0.to(gpu), vc0.to(gpu)
    ops.rope_kv_append(qkv.to(gpu), cos.to(gpu), sin.to(gpu), torch.full((B,), L, dtype=torch.int64, device=gpu), kc, vc,
                       n_q)
    assert torch.equal(kc.cpu(), kc0) and torch.equal(vc.cpu(), vc0)


def _attn_case(gpu, B, n_q, n_kv, max_len, lens, seed, scale_v=1.0):
    g = gen(seed)
    d = 128
    q = torch.randn(B, n_q, d, generator=g).bfloat16()
    kc = torch.randn(B, n_kv, max_len, d, generator=g).bfloat16()
    vc = (torch.randn(B, n_kv, max_len, d, generator=g) * scale_v).bfloat16()
    lens = torch.tensor(lens, dtype=torch.int64)
    ref = R.attn_decode(q.float(), kc.float(), vc.float(), lens)
    # whatever lies behind the valid prefix must not be read into the result
    for b in range(B):
        kc[b, :, int(lens[b]):] = float("nan")
        vc[b, :, int(lens[b]):] = float("nan")
    return q.to(gpu), kc.to(gpu), vc.to(gpu), lens.to(gpu), ref


@pytest.mark.parametrize("n_q,n_kv", [(32, 8), (8, 1), (16, 16), (16, 1)])
@pytest.mark.parametrize("lens", [[1], [31], [32], [33], [128], [777], [2048]])
def test_attn_decode_lengths_and_groups(gpu, n_q, n_kv, lens):
    q, kc, vc, dl, ref = _attn_case(gpu, 1, n_q, n_kv, 2048, lens, seed=3)
    out = ops.attn_decode(q, kc, vc, dl, len_bound=max(lens))
    assert out.shape == q.shape and out.dtype == torch.bfloat16
    assert rel(out, ref) < TOL_BF16


@pytest.mark.parametrize("splits", ["1", "3", "16", "64"])
def test_attn_decode_ragged_batch_any_split_count(gpu, splits, set_tuning):
    lens = [1000, 1, 0, 64, 513, 37]
    q, kc, vc, dl, ref = _attn_case(gpu, 6, 32, 8, 1024, lens, seed=4)
    set_tuning("MTP_ATTN_SPLITS", splits)
    out = ops.attn_decode(q, kc, vc, dl)
    assert torch.count_nonzero(out[2]) == 0                      # no tokens: zeros
    for b in range(6):
        if lens[b]:
            assert rel(out[b], ref[b]) < TOL_BF16, (b, lens[b])
    # one token: exactly its value row
    assert torch.equal(out[1].cpu().view(8, 4, 128), vc[1, :, 0].cpu()[:, None, :].expand(8, 4, 128))


def test_attn_decode_sharp_and_flat_softmax(gpu):
    """A query that matches one key far better than the rest returns that key's value; zero queries average."""
    g = gen(5)
    B, n_q, n_kv, L, d = 2, 8, 2, 500, 128
    kc = torch.randn(B, n_kv, L, d, generator=g).bfloat16()
    vc = torch.randn(B, n_kv, L, d, generator=g).bfloat16()
    q = torch.zeros(B, n_q, d).bfloat16()
    q[0] = (kc[0, :, 321].float() * 8).bfloat16().repeat_interleave(4, 0)      # scores ~ 8 |k|^2 / sqrt(d) ~ 90
    lens = torch.tensor([L, L])
    out = ops.attn_decode(q.to(gpu), kc.to(gpu), vc.to(gpu), lens.to(gpu)).cpu()
    assert rel(out[0], vc[0, :, 321].repeat_interleave(4, 0)) < TOL_BF16
    assert rel(out[1], vc[1].float().mean(1).repeat_interleave(4, 0)) < TOL_BF16
    ref = R.attn_decode(q.float(), kc.float(), vc.float(), lens)
    assert rel(out, ref) < TOL_BF16


def test_attn_decode_llama8b_shape_long_context(gpu):
    """32 sequences of up to 8192 tokens, 32 q / 8 kv heads: checked on a sample of (sequence, head) pairs
    against the oracle, and through invariance: permuting the cached tokens of a sequence (keys and values
    together) must not change its output beyond rounding."""
    g = gen(6)
    B, n_q, n_kv, L, d = 32, 32, 8, 8192, 128
    kc = torch.randn(B, n_kv, L, d, generator=g, dtype=torch.bfloat16).to(gpu)
    vc = torch.randn(B, n_kv, L, d, generator=g, dtype=torch.bfloat16).to(gpu)
    q = torch.randn(B, n_q, d, generator=g).bfloat16().to(gpu)
    lens = torch.randint(4000, L + 1, (B,), generator=g)
    lens[0], lens[1] = L, 4097
    out = ops.attn_decode(q, kc, vc, lens.to(gpu))
    for b in (0, 1, 17, 31):
        ref = R.attn_decode(q[b:b + 1].float().cpu(), kc[b:b + 1].float().cpu(), vc[b:b + 1].float().cpu(), lens[b:b + 1])
        assert rel(out[b], ref[0]) < TOL_BF16, b
    n = int(lens[5])
    perm = torch.randperm(n, generator=g).to(gpu)
    kc[5, :, :n] = kc[5][:, perm]
    vc[5, :, :n] = vc[5][:, perm]
    again = ops.attn_decode(q, kc, vc, lens.to(gpu))
    assert rel(again[5], out[5]) < TOL_BF16
    assert torch.equal(again[6], out[6])                     # untouched sequences: bit for bit the same


@pytest.mark.parametrize("B,n_q,n_kv,L", [(1, 32, 8, 2048), (7, 8, 1, 300), (32, 32, 8, 1024), (3, 16, 16, 64)])
def test_attn_decode_append_equals_append_then_attend(gpu, B, n_q, n_kv, L):
    """The one-launch form against rotary/append followed by attention (and so, through the tests of those,
    against the oracle): same cache contents bit for bit, same attention output up to summation order."""
    g = gen(9)
    d = 128
    qkv = torch.randn(B, (n_q + 2 * n_kv) * d, generator=g).bfloat16().to(gpu)
    cos, sin = (t.to(gpu) for t in rope_tables(d, L, 500000.0, dtype=torch.bfloat16))
    pos = torch.randint(0, L, (B,), generator=g)
    pos[0] = L - 1
    if B > 2:
        pos[1], pos[2] = 0, L                      # nothing cached yet; outside the cache
    kc0 = torch.randn(B, n_kv, L, d, generator=g).bfloat16()
    vc0 = torch.randn(B, n_kv, L, d, generator=g).bfloat16()
    k1, v1, k2, v2 = kc0.to(gpu), vc0.to(gpu), kc0.to(gpu), vc0.to(gpu)
    q = ops.rope_kv_append(qkv, cos, sin, pos.to(gpu), k1, v1, n_q)
    ref = ops.attn_decode(q, k1, v1, (pos + 1).clamp_max(L).to(gpu))
    ws = ops.attn_workspace(B, n_q, n_kv, L, gpu)
    for _ in range(2):                              # the workspace is reusable as the launch leaves it
        out = ops.attn_decode_append(qkv, cos, sin, pos.to(gpu), k2, v2, n_q, workspace=ws)
        assert torch.equal(k1, k2) and torch.equal(v1, v2)
        for b in range(B):
            if int(pos[b]) < L:
                assert rel(out[b], ref[b]) < TOL_BF16, (b, int(pos[b]))
            else:
                assert torch.count_nonzero(out[b]) == 0
    if B > 2:
        assert torch.equal(out[1].cpu().view(n_kv, n_q // n_kv, d),
                           qkv[1].view(-1, d)[n_q + n_kv:].cpu()[:, None, :].expand(n_kv, n_q // n_kv, d))
    # and straight against the oracle for one row
    heads = qkv[0].float().cpu().view(1, n_q + 2 * n_kv, d)
    cf, sf = cos.float().cpu()[pos[:1]], sin.float().cpu()[pos[:1]]
    kf, vf = kc0[:1].float(), vc0[:1].float()
    kf[0, :, pos[0]] = R.apply_rope(heads[:, n_q:n_q + n_kv], cf, sf)[0]
    vf[0, :, pos[0]] = heads[0, n_q + n_kv:]
    want = R.attn_decode(R.apply_rope(heads[:, :n_q], cf, sf), kf, vf, pos[:1] + 1)
    assert rel(out[0], want[0]) < TOL_BF16


def test_attn_decode_rejects_bad_arguments(gpu):
    q = torch.zeros(2, 8, 128, dtype=torch.bfloat16, device=gpu)
    kc = torch.zeros(2, 2, 64, 128, dtype=torch.bfloat16, device=gpu)
    lens = torch.ones(2, dtype=torch.int64, device=gpu)
    ops.attn_decode(q, kc, kc.clone(), lens)
    with pytest.raises(ValueError):
        ops.attn_decode(q, kc, kc.clone()[:, :, :32], lens)                      # cache shapes differ
    with pytest.raises(ValueError):
        ops.attn_decode(q, kc, kc.clone(), lens.int())                            # lens must be int64
    with pytest.raises(RuntimeError, match="head_dim"):
        ops.attn_decode(q[:, :, :64].contiguous(), kc[..., :64].contiguous(), kc[..., :64].contiguous(), lens)
    with pytest.raises(RuntimeError, match="q heads per kv head"):
        ops.attn_decode(torch.zeros(2, 34, 128, dtype=torch.bfloat16, device=gpu), kc, kc.clone(), lens)
    with pytest.raises(RuntimeError, match="len_bound"):
        ops.attn_decode(q, kc, kc.clone(), lens, len_bound=65)


def _tiny_model(seed):
    from transformers import LlamaConfig, LlamaForCausalLM
    torch.manual_seed(seed)
    cfg = LlamaConfig(hidden_size=512, intermediate_size=1024, num_attention_heads=4, num_key_value_heads=2,
                      head_dim=128, num_hidden_layers=2, vocab_size=1000, max_position_embeddings=128,
                      rope_theta=10000.0, rms_norm_eps=1e-5, attn_implementation="eager", tie_word_embeddings=False)
    model = LlamaForCausalLM(cfg).eval()
    for p_ in model.parameters():
        if p_.dim() == 1:
            p_.data.uniform_(0.5, 1.5)
        p_.data = p_.data.bfloat16().float()          # values a bf16 copy holds exactly
    return cfg, model


@pytest.mark.parametrize("fused", [False, True])
def test_llama_decoder_matches_full_sequence_forward(gpu, fused):
    """Token by token with the cache on the GPU == what the generation loop computes: the full-sequence forward
    of the library model (fp32, CPU, same bf16-representable weights), row context_length-1 (:223)."""
    cfg, model = _tiny_model(7)
    B, T = 3, 40
    ids = torch.randint(0, cfg.vocab_size, (B, T), generator=gen(7))
    with torch.no_grad():
        full = model(input_ids=ids).logits                              # [B, T, V] fp32
    dec = LlamaDecoder.from_hf(model.bfloat16().to(gpu), max_len=64, batch=B, fused=fused)
    assert dec.fused == fused
    worst = 0.0
    for t in range(T):
        logits = dec.logits(ids[:, t].to(gpu))
        worst = max(worst, rel(logits, full[:, t]))
    assert worst < 2 * TOL_BF16, worst            # two blocks of bf16 rounding on top of each other
    assert dec.lens.tolist() == [T] * B
    # greedy pick of the fused LM head == argmax of the materialised logits of the same step
    dec.reset()
    for t in range(5):
        tok = dec.step(ids[:, t].to(gpu))
        dec.lens -= 1                                 # run the same position again, now with logits written
        dec.host_len_bound -= 1
        lg = dec.logits(ids[:, t].to(gpu))
        top2 = lg.float().topk(2, dim=-1).values
        clear = (top2[:, 0] - top2[:, 1]) > 1e-2 * top2[:, 0].abs()
        assert torch.equal(tok[clear].cpu(), lg.argmax(-1)[clear].cpu())


def test_block_step_vs_oracle_llama8b_shape(gpu):
    """One Llama-3-8B block (H 4096, 32/8 heads, I 14336), 8 sequences with 1000-3000 cached tokens."""
    g = gen(8)
    B, H, n_q, n_kv, d, I, L = 8, 4096, 32, 8, 128, 14336, 3072
    def w(*shape, std=0.02):
        return (torch.randn(*shape, generator=g) * std).bfloat16()
    wt = {"input_norm": (torch.rand(H, generator=g) + 0.5).bfloat16(), "qkv": w((n_q + 2 * n_kv) * d, H),
          "o": w(H, n_q * d), "post_norm": (torch.rand(H, generator=g) + 0.5).bfloat16(), "gate_up": w(2 * I, H),
          "down": w(H, I)}
    x, res = torch.randn(B, H, generator=g).bfloat16(), torch.randn(B, H, generator=g).bfloat16()
    kc, vc = torch.randn(B, n_kv, L, d, generator=g).bfloat16(), torch.randn(B, n_kv, L, d, generator=g).bfloat16()
    pos = torch.randint(1000, 3000, (B,), generator=g)
    cos, sin = rope_tables(d, L, 500000.0, dtype=torch.bfloat16)
    kf, vf = kc.float(), vc.float()
    ref_x, ref_res = R.llama_block_step(x.float(), res.float(), pos, pos + 1, {k: v.float() for k, v in wt.items()}, kf,
                                        vf, cos.float(), sin.float(), n_q, 1e-5)
    G = {k: v.to(gpu) for k, v in wt.items()}
    kc, vc = kc.to(gpu), vc.to(gpu)
    h, r1 = ops.rmsnorm(x.to(gpu), G["input_norm"], 1e-5, res.to(gpu), want_residual=True)
    q = ops.rope_kv_append(ops.gemv(h, G["qkv"]), cos.to(gpu), sin.to(gpu), pos.to(gpu), kc, vc, n_q)
    a = ops.attn_decode(q, kc, vc, (pos + 1).to(gpu), len_bound=3000)
    o = ops.gemv(a.view(B, -1), G["o"])
    h2, r2 = ops.rmsnorm(o, G["post_norm"], 1e-5, r1, want_residual=True)
    out = ops.gemv(ops.gemv(h2, G["gate_up"], None, ops.EPI_SWIGLU), G["down"])
    assert rel(r2, ref_res) < TOL_BF16
    assert rel(out, ref_x) < 2 * TOL_BF16
    for b in range(B):
        assert rel(kc[b, :, int(pos[b])], kf[b, :, int(pos[b])]) < TOL_BF16


def test_negative_rotation_knobs_are_clamped(gpu, set_tuning):
    """The measurement knobs that rotate the walk order are taken modulo a count on the device: negative values
    from the environment are clamped on the host (they used to turn into negative offsets)."""
    set_tuning("MTP_GEMV_ROT", "-3")
    set_tuning("MTP_ATTN_ROT", "-5")
    g = gen(12)
    x = torch.randn(4, 1024, generator=g).bfloat16()
    w = (torch.randn(512, 1024, generator=g) * 0.05).bfloat16()
    assert rel(ops.gemv(x.to(gpu), w.to(gpu)), torch.nn.functional.linear(x.float(), w.float())) < TOL_BF16
    q, kc, vc, dl, ref = _attn_case(gpu, 2, 8, 2, 512, [512, 100], seed=12)
    assert rel(ops.attn_decode(q, kc, vc, dl), ref) < TOL_BF16


@pytest.mark.parametrize("fused", [False, True])
def test_llama_decoder_graph_replay_matches_eager(gpu, fused):
    """A step recorded into a HIP graph, replayed for every position with eager work and synchronisations in
    between, gives what the eager launches give (the split count of the attention differs, so equal to
    rounding), on every replay."""
    cfg, model = _tiny_model(9)
    B, T = 2, 12
    ids = torch.randint(0, cfg.vocab_size, (B, T), generator=gen(9)).to(gpu)
    model = model.bfloat16().to(gpu)
    eager = LlamaDecoder.from_hf(model, max_len=64, batch=B, fused=fused)
    graphed = LlamaDecoder.from_hf(model, max_len=64, batch=B, fused=fused)
    for t in range(3):                                  # a prefix before the capture: the graph starts mid-sequence
        eager.logits(ids[:, t])
        graphed.logits(ids[:, t])
    graphed.capture()
    assert graphed.lens.tolist() == [3] * B
    for t in range(3, T):
        le = eager.logits(ids[:, t]).float()
        lg = graphed.logits(ids[:, t]).float()
        torch.cuda.synchronize()
        assert rel(lg, le) < TOL_BF16, t
        assert torch.equal(graphed.lens, eager.lens)
        scratch = torch.randn(256, 256, device=gpu) @ torch.randn(256, 256, device=gpu)   # unrelated eager work
        assert torch.isfinite(scratch).all()
    for c_e, c_g in zip(eager.k_cache + eager.v_cache, graphed.k_cache + graphed.v_cache):
        assert torch.equal(c_e[:, :, :T], c_g[:, :, :T])
    # greedy tokens out of the graph: the argmax of the eager logits of the same step, where that is clear-cut
    le = eager.logits(ids[:, 0]).float()
    tok_g = graphed.step(ids[:, 0])
    top2 = le.topk(2, dim=-1).values
    clear = (top2[:, 0] - top2[:, 1]) > 1e-2 * top2[:, 0].abs()
    assert tok_g.shape == (B,) and torch.equal(tok_g[clear], le.argmax(-1)[clear])


def _sumsq16(x):
    """fp32 [B, K/16]: sums of squares per 16 elements, what the producing linear hands to the norm prologue"""
    return x.float().pow(2).view(x.shape[0], -1, 16).sum(-1).contiguous()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,N,K", [(1, 4096, 4096), (5, 4096, 14336), (16, 1024, 512), (32, 4096, 14336), (32, 6144, 1024),
                                   (3, 1000, 520)])
def test_gemv_residual_epilogue(gpu, dtype, B, N, K):
    """y = dtype(dtype(x W^T) + residual), bit for bit what the plain product followed by the tensor add gives,
    and the sums of squares of y per 16 rows (also through the k-sliced form, which B = 32 x 14336 takes)."""
    g = gen(60)
    x = torch.randn(B, K, generator=g).to(dtype).to(gpu)
    w = (torch.randn(N, K, generator=g) * 0.03).to(dtype).to(gpu)
    res = torch.randn(B, N, generator=g).to(dtype).to(gpu)
    ws = ops.gemv_workspace(B, N, K, ops.EPI_NONE, gpu)
    plain = ops.gemv(x, w, workspace=ws)
    y, ss = ops.gemv_fused(x, w, residual=res, want_sumsq=True, workspace=ws)
    assert torch.equal(y, plain + res)
    pad = (-N) % 16
    ref_ss = torch.nn.functional.pad(y.float().pow(2), (0, pad)).view(B, -1, 16).sum(-1)
    assert ss.shape == (B, (N + 15) // 16) and torch.allclose(ss, ref_ss, rtol=1e-5, atol=1e-30)
    y2 = res.clone()                                     # in place on the residual stream
    ops.gemv_fused(x, w, residual=y2, out=y2, workspace=ws)
    assert torch.equal(y2, y)
    assert torch.equal(ops.gemv_fused(x, w, workspace=ws), plain)            # nothing fused: the plain product
    y3, ss3 = ops.gemv_fused(x, w, want_sumsq=True, workspace=ws)          # sums of squares without a residual
    assert torch.equal(y3, plain) and torch.allclose(
        ss3, torch.nn.functional.pad(plain.float().pow(2), (0, pad)).view(B, -1, 16).sum(-1), rtol=1e-5, atol=1e-30)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,N,K,epi", [(1, 6144, 4096, "none"), (8, 6144, 4096, "none"), (5, 4096, 4096, "none"),
                                       (1, 28672, 4096, "swiglu"), (8, 28672, 4096, "swiglu"), (3, 28672, 4096, "swiglu"),
                                       (4, 8192, 512, "swiglu"), (3, 2048, 512, "swiglu"), (8, 2048, 1024, "swiglu"),
                                       (2, 1280, 8192, "none"), (4, 1280, 8192, "none"), (4, 512, 5120, "none"),
                                       (8, 256, 1024, "none"), (1, 1000, 512, "none")])
def test_gemv_norm_prologue(gpu, dtype, B, N, K, epi):
    """The product with RMSNorm(x) taken inside the linear against (a) the stand-alone norm kernel followed by
    the plain product and (b) the oracle in fp32.  The two GPU forms add the squares in different orders, so a
    row's scale may differ in its last bit and a few normalised elements by one unit of the tensor dtype."""
    g = gen(61)
    E = ops.EPI_SWIGLU if epi == "swiglu" else ops.EPI_NONE
    x = (torch.randn(B, K, generator=g) * 2).to(dtype)
    nw = (torch.rand(K, generator=g) + 0.5).to(dtype)
    w = (torch.randn(N, K, generator=g) * 0.03).to(dtype)
    xg, nwg, wg = x.to(gpu), nw.to(gpu), w.to(gpu)
    fused = ops.gemv_fused(xg, wg, None, E, norm_weight=nwg, sumsq_in=_sumsq16(xg), eps=1e-5)
    two = ops.gemv(ops.rmsnorm(xg, nwg, 1e-5), wg, None, E)
    tol = TOL_BF16 if dtype == torch.bfloat16 else 2e-3
    assert fused.shape == two.shape and rel(fused, two) < tol / 4
    hn = R.rms_norm(x.float(), nw.float(), 1e-5)[0]
    hn = hn.to(dtype).float()                                   # the normalised row as the tensor dtype holds it
    ref = torch.nn.functional.linear(hn, w.float())
    if epi == "swiglu":
        gate, up = ref[:, :N // 2].to(dtype).float(), ref[:, N // 2:].to(dtype).float()
        ref = torch.nn.functional.silu(gate) * up
    assert rel(fused, ref) < tol


@pytest.mark.parametrize("groups", [1, 2, 3, 4, 5, 6, 7])
def test_gemv_norm_prologue_every_mixed_group_count(gpu, groups, set_tuning):
    set_tuning("MTP_GEMV_MIX", str(groups))
    g = gen(62)
    B, N, K = 6, 2 * 1288, 1024
    x = torch.randn(B, K, generator=g).bfloat16().to(gpu)
    nw = (torch.rand(K, generator=g) + 0.5).bfloat16().to(gpu)
    w = (torch.randn(N, K, generator=g) * 0.03).bfloat16().to(gpu)
    fused = ops.gemv_fused(x, w, None, ops.EPI_SWIGLU, norm_weight=nw, sumsq_in=_sumsq16(x), eps=1e-6)
    two = ops.gemv(ops.rmsnorm(x, nw, 1e-6), w, None, ops.EPI_SWIGLU)
    assert rel(fused, two) < TOL_BF16 / 4
    plain = ops.gemv(x, w, None, ops.EPI_SWIGLU)                # the two-set main loop without the norm
    set_tuning("MTP_GEMV_MIX", "0")
    assert rel(plain, ops.gemv(x, w, None, ops.EPI_SWIGLU)) < TOL_BF16 / 4


def test_gemv_fused_chain_is_a_block(gpu):
    """o product (+ residual, sums of squares) -> gate/up product with the norm inside -> down product
    (+ residual): the second half of a Llama-3-8B block against the oracle, at B = 1, 8 and 32."""
    g = gen(63)
    H, I = 4096, 14336
    wo = (torch.randn(H, H, generator=g) * 0.02).bfloat16()
    wgu = (torch.randn(2 * I, H, generator=g) * 0.02).bfloat16()
    wd = (torch.randn(H, I, generator=g) * 0.02).bfloat16()
    nw = (torch.rand(H, generator=g) + 0.5).bfloat16()
    G = [t.to(gpu) for t in (wo, wgu, wd, nw)]
    for B in (1, 8, 32):
        a = torch.randn(B, H, generator=g).bfloat16()
        res = torch.randn(B, H, generator=g).bfloat16()
        ws = ops.gemv_workspace(B, H, I, ops.EPI_NONE, gpu)
        r1, ss = ops.gemv_fused(a.to(gpu), G[0], residual=res.to(gpu), want_sumsq=True, workspace=ws)
        assert ops.gemv_norm_fits(B, H) == (B <= 8)
        if B <= 8:
            act = ops.gemv_fused(r1, G[1], None, ops.EPI_SWIGLU, norm_weight=G[3], sumsq_in=ss, eps=1e-5)
        else:       # more rows than the norm prologue holds: the stand-alone norm in between
            act = ops.gemv(ops.rmsnorm(r1, G[3], 1e-5), G[1], None, ops.EPI_SWIGLU)
        r2 = ops.gemv_fused(act, G[2], residual=r1, workspace=ws)
        # oracle, rounding to bf16 where the tensors of the model are bf16
        bf = lambda t: t.bfloat16().float()
        o = bf(torch.nn.functional.linear(a.float(), wo.float()))
        ref_r1 = bf(o + res.float())
        hn = bf(R.rms_norm(ref_r1, nw.float(), 1e-5)[0])
        gu = bf(torch.nn.functional.linear(hn, wgu.float()))
        ref_act = bf(torch.nn.functional.silu(gu[:, :I]) * gu[:, I:])
        ref_r2 = bf(bf(torch.nn.functional.linear(ref_act, wd.float())) + ref_r1)
        assert rel(r1, ref_r1) < TOL_BF16 and rel(act, ref_act) < TOL_BF16 and rel(r2, ref_r2) < TOL_BF16, B


def test_gemv_fused_rejects_bad_arguments(gpu):
    x = torch.zeros(2, 1024, dtype=torch.bfloat16, device=gpu)
    w = torch.zeros(64, 1024, dtype=torch.bfloat16, device=gpu)
    nw = torch.ones(1024, dtype=torch.bfloat16, device=gpu)
    ss = _sumsq16(x)
    with pytest.raises(ValueError, match="sumsq_in"):
        ops.gemv_fused(x, w, norm_weight=nw)                                        # the norm needs the sums
    with pytest.raises(ValueError, match="sumsq_in"):
        ops.gemv_fused(x, w, norm_weight=nw, sumsq_in=ss[:, :-1].contiguous())
    with pytest.raises(ValueError, match="norm_weight"):
        ops.gemv_fused(x, w, norm_weight=nw[:-8].contiguous(), sumsq_in=ss)
    with pytest.raises(RuntimeError, match="512"):                                  # K = 576: not a multiple of 512
        ops.gemv_fused(x[:, :576].contiguous(), w[:, :576].contiguous(), norm_weight=nw[:576].contiguous(),
                       sumsq_in=ss[:, :36].contiguous())
    with pytest.raises(RuntimeError, match="plain stores"):                         # residual with SwiGLU
        ops.gemv_fused(x, w, None, ops.EPI_SWIGLU, residual=torch.zeros(2, 32, dtype=torch.bfloat16, device=gpu))
    with pytest.raises(ValueError, match="residual"):
        ops.gemv_fused(x, w, residual=torch.zeros(2, 63, dtype=torch.bfloat16, device=gpu))
    sq = torch.zeros(2, 1024, dtype=torch.bfloat16, device=gpu)
    with pytest.raises(RuntimeError, match="must not be the input"):                # in place on the input
        ops.gemv_fused(sq, torch.zeros(1024, 1024, dtype=torch.bfloat16, device=gpu), out=sq)
    with pytest.raises(RuntimeError, match="8 x 4096"):                             # 9 rows do not fit
        x9 = torch.zeros(9, 1024, dtype=torch.bfloat16, device=gpu)
        ops.gemv_fused(x9, w, norm_weight=nw, sumsq_in=_sumsq16(x9))
    assert ops.gemv_norm_fits(8, 4096) and ops.gemv_norm_fits(4, 8192) and not ops.gemv_norm_fits(2, 16384)
    assert not ops.gemv_norm_fits(9, 512) and not ops.gemv_norm_fits(5, 8192) and not ops.gemv_norm_fits(1, 576)
    with pytest.raises(ValueError, match="fused=True"):
        LlamaDecoder(torch.zeros(10, 640, dtype=torch.bfloat16, device=gpu), [], nw, w, 4, 2, fused=True)
    with pytest.raises(ValueError, match="fused=True"):
        LlamaDecoder(torch.zeros(10, 1024, dtype=torch.bfloat16, device=gpu), [], nw, w, 4, 2, batch=16, fused=True)


def test_attn_decode_seeded_sweep(gpu):
    """40 seeded cases over batch, head grouping, cache capacity, ragged lengths and dtype, plain and appending
    forms, against the oracle."""
    g = gen(50)
    worst = 0.0
    for case in range(40):
        B = int(torch.randint(1, 9, (1,), generator=g))
        group = [1, 2, 4, 8, 16][int(torch.randint(0, 5, (1,), generator=g))]
        n_kv = int(torch.randint(1, 5, (1,), generator=g))
        n_q = n_kv * group
        max_len = int(torch.randint(1, 1200, (1,), generator=g))
        dt = torch.bfloat16 if case % 2 == 0 else torch.float16
        tol = TOL_BF16 if dt == torch.bfloat16 else 2e-3
        lens = torch.randint(0, max_len + 1, (B,), generator=g)
        q = torch.randn(B, n_q, 128, generator=g).to(dt)
        kc = torch.randn(B, n_kv, max_len, 128, generator=g).to(dt)
        vc = torch.randn(B, n_kv, max_len, 128, generator=g).to(dt)
        ref = R.attn_decode(q.float(), kc.float(), vc.float(), lens)
        out = ops.attn_decode(q.to(gpu), kc.to(gpu), vc.to(gpu), lens.to(gpu))
        for b in range(B):
            if int(lens[b]) == 0:
                assert torch.count_nonzero(out[b]) == 0, (case, b)
            else:
                e = rel(out[b], ref[b])
                worst = max(worst, e / tol)
                assert e < tol, (case, b, B, n_q, n_kv, max_len, int(lens[b]), dt)
        # the appending form at positions lens - 1 reproduces the same output when the cache row and qkv agree
        pos = (lens - 1).clamp_min(0)
        heads = torch.cat([q, torch.stack([kc[b, :, pos[b]] for b in range(B)]),
                           torch.stack([vc[b, :, pos[b]] for b in range(B)])], dim=1)       # [B, n_q + 2 n_kv, 128]
        ident_cos = torch.ones(max_len, 128).to(dt)                                         # rotation by zero
        ident_sin = torch.zeros(max_len, 128).to(dt)
        k2, v2 = kc.to(gpu), vc.to(gpu)
        out2 = ops.attn_decode_append(heads.reshape(B, -1).to(gpu), ident_cos.to(gpu), ident_sin.to(gpu), pos.to(gpu),
                                      k2, v2, n_q)
        assert torch.equal(k2.cpu(), kc) and torch.equal(v2.cpu(), vc)                      # rewrote the same rows
        for b in range(B):
            if int(lens[b]) > 0:
                assert rel(out2[b], ref[b]) < tol, ("append", case, b)
    assert worst < 1.0
