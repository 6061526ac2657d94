"""Pins the CPU oracle (oracle/tp_reference.py) against things it was not written from:
hand-computed golden vectors, library routines, closed forms, autograd in fp64, brute force.
A dropped term, a wrong sign, a transposed operand or an off-by-one index fails at least one test."""
import json
import math
import os

import pytest
import torch
import torch.nn.functional as F

from oracle import tp_reference as R

G = os.path.join(os.path.dirname(__file__), "golden")


def _load(name):
    with open(os.path.join(G, name)) as f:
        return json.load(f)


# ------------------------------------------------------------------ cross entropy
@pytest.mark.parametrize("case", _load("ce_small.json"), ids=lambda c: f"start{c['vocab_start']}_t{c['target']}")
def test_ce_golden(case):
    x = torch.tensor(case["logits"], dtype=torch.float64)
    t = torch.tensor(case["target"], dtype=torch.int64)
    v = x.shape[1]
    loss, sm, mask, mt = R.vocab_parallel_cross_entropy_forward(x.clone(), t, case["vocab_start"],
                                                                case["vocab_start"] + v)
    assert torch.allclose(loss, torch.tensor(case["loss"], dtype=torch.float64), rtol=1e-12, atol=1e-12)
    g = R.vocab_parallel_cross_entropy_backward(sm, mask, mt, torch.tensor(case["grad_output"], dtype=torch.float64))
    assert torch.allclose(g, torch.tensor(case["grad"], dtype=torch.float64), rtol=1e-10, atol=1e-12)


def test_ce_matches_library_in_range():
    torch.manual_seed(1)
    x = torch.randn(64, 1000, dtype=torch.float64) * 3
    t = torch.randint(0, 1000, (64,))
    loss, *_ = R.vocab_parallel_cross_entropy_forward(x.clone(), t, 0, 1000)
    assert torch.allclose(loss, F.cross_entropy(x, t, reduction="none"), rtol=1e-12, atol=1e-12)


def test_ce_out_of_range_is_lse_minus_max():
    torch.manual_seed(2)
    x = torch.randn(16, 333, dtype=torch.float64)
    t = torch.tensor([-100, 333, 400, -1] * 4)
    loss, sm, *_ = R.vocab_parallel_cross_entropy_forward(x.clone(), t, 0, 333)
    assert torch.allclose(loss, torch.logsumexp(x, -1) - x.max(-1).values, rtol=1e-12)
    assert torch.allclose(sm, torch.softmax(x, -1), rtol=1e-12)  # and the input now holds the softmax


def test_ce_is_in_place_and_shaped_like_target():
    x = torch.randn(3, 5, 11)
    t = torch.randint(0, 11, (3, 5))
    buf = x.clone()
    loss, sm, *_ = R.vocab_parallel_cross_entropy_forward(buf, t, 0, 11)
    assert loss.shape == t.shape and sm.data_ptr() == buf.data_ptr()
    assert torch.allclose(buf, torch.softmax(x, -1), atol=1e-6)


def test_ce_backward_is_autograd_of_closed_form():
    torch.manual_seed(3)
    x = torch.randn(12, 50, dtype=torch.float64, requires_grad=True)
    t = torch.randint(0, 50, (12,))
    t[::4] = -100
    g = torch.rand(12, dtype=torch.float64)
    inr = (t >= 0) & (t < 50)
    closed = torch.where(inr, torch.logsumexp(x, -1) - x.gather(1, t.clamp(0, 49)[:, None])[:, 0],
                         torch.logsumexp(x, -1) - x.max(-1).values.detach())
    (ref,) = torch.autograd.grad((closed * g).sum(), x)
    loss, grad = R.cross_entropy_fp32(x.detach(), t, 0, g)
    assert torch.allclose(loss.double(), closed.detach(), rtol=1e-5, atol=1e-6)
    assert torch.allclose(grad.double(), ref, rtol=1e-4, atol=1e-7)


def test_ce_partials_over_8_slices_combine_to_full():
    torch.manual_seed(4)
    n, v, p = 10, 64, 8
    x = torch.randn(n, v) * 2
    t = torch.randint(0, v, (n,))
    t[0] = -100
    full, _ = R.cross_entropy_fp32(x, t, 0)
    parts = [R.cross_entropy_partials(x[:, r * 8:(r + 1) * 8], t, r * 8) for r in range(p)]
    loss, gm, gs = R.combine_partials(*zip(*parts))
    assert torch.allclose(loss, full, rtol=1e-6, atol=1e-6)
    assert torch.equal(gm, x.max(-1).values)


# ------------------------------------------------------------------ activations
def test_activation_golden():
    a = _load("activations.json")
    x = torch.tensor(a["x"], dtype=torch.float64)
    assert torch.allclose(R.gelu_new(x), torch.tensor(a["gelu_new"], dtype=torch.float64), rtol=1e-12, atol=1e-15)
    y = torch.cat([x, torch.ones_like(x)])
    assert torch.allclose(R.swiglu(y), torch.tensor(a["silu"], dtype=torch.float64), rtol=1e-12, atol=1e-15)


def test_activation_derivatives_are_autograd():
    x = torch.linspace(-5, 5, 101, dtype=torch.float64, requires_grad=True)
    (g,) = torch.autograd.grad(R.gelu_new(x).sum(), x)
    assert torch.allclose(R.gelu_new_grad(x.detach()), g, rtol=1e-10, atol=1e-12)
    y = torch.randn(7, 10, dtype=torch.float64, requires_grad=True)
    d = torch.randn(7, 5, dtype=torch.float64)
    (gy,) = torch.autograd.grad((R.swiglu(y) * d).sum(), y)
    assert torch.allclose(R.swiglu_backward(d, y.detach()), gy, rtol=1e-10, atol=1e-12)
    # the library's tanh-approximate GELU is the same function
    assert torch.allclose(R.gelu_new(x.detach()), F.gelu(x.detach(), approximate="tanh"), rtol=1e-10, atol=1e-12)


# ------------------------------------------------------------------ linear
def test_linear_forward_brute_force_and_tuple_contract():
    torch.manual_seed(5)
    x = torch.randn(2, 3, 4, dtype=torch.float64)
    w = torch.randn(5, 4, dtype=torch.float64)
    b = torch.randn(5, dtype=torch.float64)
    brute = torch.zeros(2, 3, 5, dtype=torch.float64)
    for i in range(2):
        for j in range(3):
            for n in range(5):
                brute[i, j, n] = sum(x[i, j, k] * w[n, k] for k in range(4)) + b[n]
    out, ob = R.column_parallel_linear_forward(x, w, b)
    assert ob is None and torch.allclose(out, brute, rtol=1e-12)
    out, ob = R.column_parallel_linear_forward(x, w, b, skip_bias_add=True)
    assert ob is b and torch.allclose(out, brute - b, rtol=1e-12)
    out, ob = R.row_parallel_linear_forward(x, w, b)
    assert ob is None and torch.allclose(out, brute, rtol=1e-12)
    out, ob = R.row_parallel_linear_forward(x, w, b, skip_bias_add=True)
    assert ob is b and torch.allclose(out, brute - b, rtol=1e-12)
    out, ob = R.row_parallel_linear_forward(x, w, None)
    assert ob is None and torch.allclose(out, brute - b, rtol=1e-12)


def test_linear_backward_is_autograd():
    torch.manual_seed(6)
    x = torch.randn(4, 3, 6, dtype=torch.float64, requires_grad=True)
    w = torch.randn(5, 6, dtype=torch.float64, requires_grad=True)
    b = torch.randn(5, dtype=torch.float64, requires_grad=True)
    dy = torch.randn(4, 3, 5, dtype=torch.float64)
    gx, gw, gb = torch.autograd.grad((F.linear(x, w, b) * dy).sum(), (x, w, b))
    dx, dw, db = R.linear_backward(x.detach(), w.detach(), dy, True)
    assert torch.allclose(dx, gx) and torch.allclose(dw, gw) and torch.allclose(db, gb)
    assert dw.shape == w.shape and dx.shape == x.shape  # a transposed operand would change these


# ------------------------------------------------------------------ embedding
def test_embedding_forward_exact_and_shard_zero_rows():
    torch.manual_seed(7)
    table = torch.randn(32, 6)
    ids = torch.randint(0, 32, (3, 7))
    assert torch.equal(R.vocab_parallel_embedding_forward(ids, table, 0, 32, 1), table[ids])
    full = torch.zeros(3, 7, 6)
    for r in range(4):  # 4 ranks of 8 rows: sum of the masked partial outputs is the full lookup
        part = R.vocab_parallel_embedding_forward(ids, table[8 * r:8 * r + 8], 8 * r, 8 * r + 8, 4)
        outside = (ids < 8 * r) | (ids >= 8 * r + 8)
        assert torch.equal(part[outside], torch.zeros_like(part[outside]))
        full += part
    assert torch.equal(full, table[ids])


def test_embedding_backward_is_autograd_and_brute_force():
    torch.manual_seed(8)
    table = torch.randn(16, 4, requires_grad=True)
    ids = torch.tensor([[1, 1, 5], [15, 0, 1]])
    dout = torch.randn(2, 3, 4)
    (g,) = torch.autograd.grad((F.embedding(ids, table) * dout).sum(), table)
    assert torch.allclose(R.embedding_backward(ids, dout, 16, 0, 16), g, atol=1e-6)
    shard = R.embedding_backward(ids, dout, 8, 0, 8)  # rank 0 of 2: id 15 is not ours
    brute = torch.zeros(8, 4)
    for i in range(2):
        for j in range(3):
            if ids[i, j] < 8:
                brute[ids[i, j]] += dout[i, j]
    assert torch.allclose(shard, brute, atol=1e-6)


# ------------------------------------------------------------------ sharding, integers, argmax
def test_shard_master_weight_golden_table():
    s = _load("shard_table.json")
    master = torch.tensor([[10.0 * r + c for c in range(s["in"])] for r in range(s["out"])])
    for rank in range(s["world"]):
        for stride, key in ((1, "column_stride1"), (2, "column_stride2")):
            got = R.shard_master_weight(master, s["out"] // s["world"], 0, stride, rank, s["world"])
            assert torch.equal(got, master[s[key][str(rank)]])
    master = torch.tensor([[10.0 * r + c for c in range(s["row_in"])] for r in range(4)])
    for rank in range(s["row_world"]):
        got = R.shard_master_weight(master, s["row_in"] // s["row_world"], 1, 1, rank, s["row_world"])
        assert torch.equal(got, master[:, s["row_stride1"][str(rank)]])


def test_vocab_ranges_and_divide():
    assert R.vocab_range_from_global_vocab_size(128256, 3, 8) == (3 * 16032, 4 * 16032)
    assert R.vocab_range_from_per_partition_vocab_size(10, 2, 99) == (20, 30)
    with pytest.raises(AssertionError, match="50257 is not divisible by 8"):
        R.vocab_range_from_global_vocab_size(50257, 0, 8)
    covered = []
    for r in range(4):
        a, b = R.vocab_range_from_global_vocab_size(1000, r, 4)
        covered += list(range(a, b))
    assert covered == list(range(1000))


def test_greedy_argmax_first_index_on_ties():
    x = torch.tensor([[1.0, 5.0, 5.0, 2.0], [7.0, 7.0, 7.0, 7.0], [-1.0, -3.0, -0.5, -0.5]])
    assert R.greedy_argmax(x).tolist() == [1, 0, 2]
    torch.manual_seed(9)
    y = torch.randn(5, 1000)
    brute = [max(range(1000), key=lambda j: (y[i, j].item(), -j)) for i in range(5)]
    assert R.greedy_argmax(y).tolist() == brute
    assert R.greedy_argmax(y).dtype == torch.int64


def test_decode_step_reduces_to_plain_linears():
    torch.manual_seed(10)
    x = torch.randn(3, 16).bfloat16()
    wq, wg, wd, wl = (torch.randn(*s).bfloat16() * 0.1 for s in ((24, 16), (64, 16), (16, 32), (100, 16)))
    qkv, out, logits, tok = R.decode_step(x, wq, wg, wd, wl)
    assert torch.equal(qkv, F.linear(x.float(), wq.float()).bfloat16())
    y = F.linear(x.float(), wg.float()).bfloat16().float()
    h = (F.silu(y[:, :32]) * y[:, 32:]).bfloat16()
    assert torch.equal(out, F.linear(h.float(), wd.float()).bfloat16())
    assert torch.equal(tok, F.linear(out.float(), wl.float()).argmax(-1))


# ------------------------------------------------------------------------------- sampling tail
def test_top_k_top_p_filter_hand_cases():
    """Worked by hand from text_generation_inference.py:48-68.  probs 0.5/0.3/0.15/0.05 (logits = log p)."""
    lp = torch.tensor([[0.3, 0.05, 0.5, 0.15]]).log()
    inf = float("inf")
    # top_k = 2: the 2nd largest is log 0.3; everything below it goes
    assert torch.equal(R.top_k_logits(lp.clone(), top_k=2) == -inf, torch.tensor([[False, True, False, True]]))
    # top_p = 0.7: sorted cumulative 0.5, 0.8, 0.95, 1.0 -> "> 0.7" from the 2nd on, shifted right by one: the
    # token that crosses the threshold stays, the rest goes
    assert torch.equal(R.top_k_logits(lp.clone(), top_p=0.7) == -inf, torch.tensor([[False, True, False, True]]))
    # top_p = 0.4: even the first token is above the threshold, and is kept regardless (:65)
    assert torch.equal(R.top_k_logits(lp.clone(), top_p=0.4) == -inf, torch.tensor([[True, True, False, True]]))
    # top_p = 0.85: cumulative 0.5, 0.8 <= 0.85 < 0.95: three tokens stay
    assert torch.equal(R.top_k_logits(lp.clone(), top_p=0.85) == -inf, torch.tensor([[False, True, False, False]]))
    # ties with the k-th value stay (strict "<" at :50)
    t = torch.tensor([[1.0, 3.0, 2.0, 2.0, 0.0]])
    assert torch.equal(R.top_k_logits(t.clone(), top_k=2) == -inf, torch.tensor([[True, False, False, False, True]]))
    # kept values are untouched; the function edits its argument
    x = lp.clone()
    y = R.top_k_logits(x, top_k=3)
    assert y is x and torch.equal(x[0, [0, 2, 3]], lp[0, [0, 2, 3]])


def test_top_k_top_p_filter_matches_library_warpers():
    """Same rule as transformers' TopK/TopP warpers away from exact threshold equality."""
    from transformers.generation.logits_process import TopKLogitsWarper, TopPLogitsWarper
    g = torch.Generator().manual_seed(5)
    x = torch.randn(6, 997, generator=g) * 3
    for k in (1, 5, 50):
        assert torch.equal(R.top_k_logits(x.clone(), top_k=k), TopKLogitsWarper(top_k=k)(None, x.clone()))
    for p in (0.1, 0.5, 0.9, 0.999):
        assert torch.equal(R.top_k_logits(x.clone(), top_p=p), TopPLogitsWarper(top_p=p)(None, x.clone()))
    both = TopPLogitsWarper(top_p=0.8)(None, TopKLogitsWarper(top_k=40)(None, x.clone()))
    assert torch.equal(R.top_k_logits(x.clone(), top_k=40, top_p=0.8), both)


def test_sample_tail_is_inverse_cdf_and_follows_the_distribution():
    import numpy as np
    g = torch.Generator().manual_seed(6)
    x = torch.randn(4, 50, generator=g) * 2
    u = torch.rand(4, generator=g)
    tok, probs = R.sample_tail(x, 0.7, 10, 0.9, u)
    ref_probs = F.softmax(R.top_k_logits(x.float() / 0.7, 10, 0.9).double(), -1)
    assert torch.allclose(probs, ref_probs)
    for b in range(4):        # numpy's searchsorted on the cumulative distribution
        cdf = np.cumsum(probs[b].numpy())
        assert int(tok[b]) == int(np.searchsorted(cdf, float(u[b].double()) * cdf[-1], side="right"))
        assert probs[b, tok[b]] > 0
    # frequencies over many uniforms approach the probabilities (8 kept tokens, 40000 draws)
    one = torch.randn(1, 30, generator=g)
    us = torch.rand(40000, generator=g)
    toks, pr = R.sample_tail(one.expand(40000, 30).clone(), 1.0, 8, 0.0, us)
    freq = torch.bincount(toks, minlength=30).double() / 40000
    assert (freq - pr[0]).abs().max() < 0.01 and int((pr[0] > 0).sum()) == 8


# ---- one position against a key/value cache: pinned on transformers' own Llama block over the full sequence ----
ROPE_THETA = 10000.0


def _tiny_llama(seed=11, layers=2):
    from transformers import LlamaConfig
    from transformers.models.llama import modeling_llama as ML
    torch.manual_seed(seed)
    cfg = LlamaConfig(hidden_size=256, intermediate_size=384, num_attention_heads=4, num_key_value_heads=2,
                      head_dim=64, num_hidden_layers=layers, vocab_size=211, max_position_embeddings=64,
                      rope_theta=ROPE_THETA, rms_norm_eps=1e-5, attn_implementation="eager", attention_bias=False,
                      mlp_bias=False)
    model = ML.LlamaModel(cfg).eval()
    for p_ in model.parameters():      # norm weights away from 1 so that a dropped weight would show
        if p_.dim() == 1:
            p_.data.uniform_(0.5, 1.5)
    return cfg, model


def _block_weights(layer):
    a, m = layer.self_attn, layer.mlp
    return {"input_norm": layer.input_layernorm.weight.data,
            "qkv": torch.cat([a.q_proj.weight, a.k_proj.weight, a.v_proj.weight]).data,
            "o": a.o_proj.weight.data, "post_norm": layer.post_attention_layernorm.weight.data,
            "gate_up": torch.cat([m.gate_proj.weight, m.up_proj.weight]).data, "down": m.down_proj.weight.data}


def test_cached_step_equals_full_sequence_forward_of_the_library_model():
    """Stepping position by position with a cache gives, at every position, the row the full-sequence forward
    of transformers' LlamaModel gives there (rows of two different lengths in one batch)."""
    cfg, model = _tiny_llama()
    B, T = 2, 9
    ids = torch.randint(0, cfg.vocab_size, (B, T), generator=torch.Generator().manual_seed(3))
    with torch.no_grad():
        full = model(input_ids=ids).last_hidden_state                        # [B, T, H]
    d, n_q, n_kv = cfg.head_dim, cfg.num_attention_heads, cfg.num_key_value_heads
    cos_t, sin_t = R.rope_tables(d, 64, ROPE_THETA)
    kc = [torch.zeros(B, n_kv, 16, d) for _ in model.layers]
    vc = [torch.zeros(B, n_kv, 16, d) for _ in model.layers]
    with torch.no_grad():
        for t in range(T):
            pos = torch.full((B,), t, dtype=torch.int64)
            x, res = model.embed_tokens(ids[:, t]), None
            for li, layer in enumerate(model.layers):
                x, res = R.llama_block_step(x, res, pos, pos + 1, _block_weights(layer), kc[li], vc[li], cos_t,
                                            sin_t, n_q, cfg.rms_norm_eps)
            y, _ = R.rms_norm(x, model.norm.weight.data, cfg.rms_norm_eps, res)
            assert torch.allclose(y, full[:, t], atol=2e-5, rtol=1e-4), t


def test_cached_step_pieces_against_library_routines():
    from transformers.models.llama import modeling_llama as ML
    cfg, model = _tiny_llama(layers=1)
    g = torch.Generator().manual_seed(4)
    # RMSNorm: the library module; the residual is added first
    x, r = torch.randn(3, 256, generator=g), torch.randn(3, 256, generator=g)
    norm = model.layers[0].input_layernorm
    y, h = R.rms_norm(x, norm.weight.data, cfg.rms_norm_eps, r)
    assert torch.equal(h, r + x) and torch.allclose(y, norm(r + x))
    # closed form on a constant row: every element c -> weight * c / sqrt(c^2 + eps)
    c = torch.full((1, 256), 3.0)
    assert torch.allclose(R.rms_norm(c, norm.weight.data, 1e-5)[0], norm.weight.data * 3.0 / math.sqrt(9.0 + 1e-5))
    # rotary tables and rotation: the library's rotary module and apply_rotary_pos_emb
    rot = ML.LlamaRotaryEmbedding(cfg)
    pos = torch.tensor([[0, 5, 17]])
    cos, sin = rot(torch.zeros(1, 3, 256), pos)
    cos_t, sin_t = R.rope_tables(cfg.head_dim, 64, ROPE_THETA)
    assert torch.allclose(cos[0], cos_t[pos[0]]) and torch.allclose(sin[0], sin_t[pos[0]])
    q = torch.randn(1, 4, 3, 64, generator=g)                             # [batch, heads, positions, d]
    k = torch.randn(1, 2, 3, 64, generator=g)
    qe, ke = ML.apply_rotary_pos_emb(q, k, cos, sin)
    mine = R.apply_rope(q[0].transpose(0, 1), cos_t[pos[0]], sin_t[pos[0]])   # rows = positions
    assert torch.allclose(mine, qe[0].transpose(0, 1), atol=1e-6)
    # a rotation keeps the norm of every (i, i + d/2) pair; position 0 is the identity
    assert torch.allclose(mine.norm(dim=-1), q[0].transpose(0, 1).norm(dim=-1), rtol=1e-5)
    assert torch.equal(R.apply_rope(q[0, :, :1].transpose(0, 1), cos_t[:1], sin_t[:1]), q[0, :, :1].transpose(0, 1))
    # attention: torch's scaled_dot_product_attention over the valid prefix, kv heads repeated per group
    B, n_q, n_kv, d, L = 3, 8, 2, 32, 20
    qq = torch.randn(B, n_q, d, generator=g)
    kc, vc = torch.randn(B, n_kv, L, d, generator=g), torch.randn(B, n_kv, L, d, generator=g)
    lens = torch.tensor([20, 1, 7])
    got = R.attn_decode(qq, kc, vc, lens)
    for b in range(B):
        n = int(lens[b])
        kk = kc[b, :, :n].repeat_interleave(n_q // n_kv, 0)
        vv = vc[b, :, :n].repeat_interleave(n_q // n_kv, 0)
        ref = F.scaled_dot_product_attention(qq[b][:, None], kk, vv)[:, 0]
        assert torch.allclose(got[b], ref, atol=1e-5)
    assert torch.allclose(got[1], vc[1, :, 0].repeat_interleave(4, 0))     # one token: its value comes back
    # junk beyond lens must not matter
    kc2, vc2 = kc.clone(), vc.clone()
    kc2[2, :, 7:], vc2[2, :, 7:] = 1e4, float("nan")
    assert torch.equal(R.attn_decode(qq, kc2, vc2, lens)[2], got[2])
