"""Host-side behaviour of the drop-in layers: constructor contract, attributes, parameter tags,
state-dict names, weight sharding, the plug-in boundary (build_layers), and the refusal to run
anywhere but on the GPU kernels.  No GPU needed."""
import json
import os

import pytest
import torch
import torch.nn as nn
from hypothesis import given, settings, strategies as st

from merak_amd import mpu, set_args, get_args
from merak_amd.tensor_parallel import (ColPara, RowPara, build_layers, init_method_normal,
                                       scaled_init_method_normal)
from oracle import tp_reference as R

G = os.path.join(os.path.dirname(__file__), "golden")


def test_column_parallel_contract():
    l = mpu.ColumnParallelLinear(12, 20)
    assert l.weight.shape == (20, 12) and l.bias.shape == (20,)
    assert l.gather_output is True and l.skip_bias_add is False  # class defaults, layers.py:193-196
    assert l.input_size == 12 and l.output_size == 20 and l.output_size_per_partition == 20
    assert l.weight.model_parallel and l.weight.partition_dim == 0 and l.weight.partition_stride == 1
    assert l.bias.model_parallel and l.bias.partition_dim == 0 and l.bias.stride == 1
    assert torch.count_nonzero(l.bias) == 0
    assert l.master_weight is None
    assert repr(l) == "ColumnParallelLinear(in_features=12, out_features=20, bias=True)"
    nb = mpu.ColumnParallelLinear(12, 20, bias=False)
    assert nb.bias is None and [n for n, _ in nb.named_parameters()] == ["weight"]
    pos = mpu.ColumnParallelLinear(12, 20, True, False, nn.init.xavier_normal_)  # model_parallel.py:143-156
    assert pos.gather_output is False


def test_row_parallel_contract():
    l = mpu.RowParallelLinear(12, 20, input_is_parallel=True)
    assert l.weight.shape == (20, 12) and l.bias.shape == (20,)
    assert l.weight.partition_dim == 1 and not hasattr(l.bias, "model_parallel")  # row bias is not sharded
    assert l.input_size_per_partition == 12
    assert repr(l) == "RowParallelLinear(in_features=12, out_features=20, bias=True)"


def test_shard_shapes_at_tp8_match_llama70b_rank():
    mpu.set_model_parallel_world_size(8)
    mpu.set_model_parallel_rank(3)
    set_args(use_cpu_initialization=True, params_dtype=torch.bfloat16)
    col = mpu.ColumnParallelLinear(64, 8 * 1280, bias=False, gather_output=False)
    row = mpu.RowParallelLinear(8 * 3584, 64, bias=False, input_is_parallel=True)
    emb = mpu.VocabParallelEmbedding(128256, 8)
    assert col.weight.shape == (1280, 64) and col.weight.dtype == torch.bfloat16
    assert row.weight.shape == (64, 3584)
    assert (emb.vocab_start_index, emb.vocab_end_index) == (3 * 16032, 4 * 16032)
    assert emb.weight.shape == (16032, 8)
    with pytest.raises(AssertionError, match="50257 is not divisible by 8"):
        mpu.VocabParallelEmbedding(50257, 8)


def test_cpu_init_shards_like_the_reference():
    s = json.load(open(os.path.join(G, "shard_table.json")))

    def arange_init(t):
        with torch.no_grad():
            t.copy_(torch.tensor([[10.0 * r + c for c in range(t.shape[1])] for r in range(t.shape[0])]))
        return t

    mpu.set_model_parallel_world_size(s["world"])
    for rank in range(s["world"]):
        mpu.set_model_parallel_rank(rank)
        for stride, key in ((1, "column_stride1"), (2, "column_stride2")):
            l = mpu.ColumnParallelLinear(s["in"], s["out"], bias=False, init_method=arange_init, stride=stride,
                                         keep_master_weight_for_test=True)
            assert l.master_weight.shape == (s["out"], s["in"])
            assert torch.equal(l.weight.data, l.master_weight[s[key][str(rank)]])
            assert l.weight.partition_stride == stride
    mpu.set_model_parallel_world_size(s["row_world"])
    for rank in range(s["row_world"]):
        mpu.set_model_parallel_rank(rank)
        l = mpu.RowParallelLinear(s["row_in"], 4, bias=False, init_method=arange_init,
                                  keep_master_weight_for_test=True)
        assert torch.equal(l.weight.data, l.master_weight[:, s["row_stride1"][str(rank)]])


def test_params_dtype_and_init_methods():
    set_args(use_cpu_initialization=True, params_dtype=torch.bfloat16)
    torch.manual_seed(0)
    l = mpu.ColumnParallelLinear(256, 512, init_method=init_method_normal(0.02))
    assert l.weight.dtype == torch.bfloat16 and l.bias.dtype == torch.bfloat16
    assert abs(l.weight.float().std().item() - 0.02) < 2e-3
    r = mpu.RowParallelLinear(256, 512, init_method=scaled_init_method_normal(0.02, 8))
    assert abs(r.weight.float().std().item() - 0.02 / 4.0) < 1e-3
    assert abs(scaled_init_method_normal(0.02, {"a": 4, "b": 4})(torch.empty(512, 512)).std().item() - 0.005) < 1e-3


def test_state_dict_names_and_boundary():
    lin = nn.Linear(16, 8)          # as set_mp_attr leaves it at mp=2: out_features already divided
    lin.mp_attr = "col"
    mpu.set_model_parallel_world_size(2)
    mpu.set_model_parallel_rank(1)
    col = build_layers("q_proj", lin, 2, init_method_normal(0.02), scaled_init_method_normal(0.02, 2))
    assert isinstance(col, ColPara) and col.col_linear.output_size == 16 and col.weight.shape == (8, 16)
    assert sorted(col.state_dict()) == ["col_linear.bias", "col_linear.weight"]
    assert col.col_linear.gather_output is False and col.need_permute is False
    lin2 = nn.Linear(8, 16, bias=False)
    lin2.mp_attr = "row_mlp"
    row = build_layers("down_proj", lin2, 2, init_method_normal(0.02), scaled_init_method_normal(0.02, 2))
    assert isinstance(row, RowPara) and row.row_linear.input_size == 16 and row.weight.shape == (16, 8)
    assert sorted(row.state_dict()) == ["row_linear.weight"] and row.bias is None
    assert row.row_linear.input_is_parallel is True
    plain = nn.Linear(4, 4)
    assert build_layers("x", plain, 2, None, None) is plain        # untagged: returned unchanged
    assert build_layers("ln", nn.LayerNorm(4), 2, None, None) is None
    set_args(use_cpu_initialization=True, tp_overlapping_level=2)
    with pytest.raises(NotImplementedError):
        ColPara(4, 4, init_method_normal(0.02))


def test_forward_refuses_cpu_tensors_and_other_dtypes():
    l = mpu.ColumnParallelLinear(8, 8)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        l(torch.randn(2, 8))
    e = mpu.VocabParallelEmbedding(16, 4)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        e(torch.tensor([1, 2]))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        mpu.vocab_parallel_cross_entropy(torch.randn(2, 8), torch.tensor([1, 2]))


def test_mappings_and_groups_at_size_one_and_above():
    x = torch.randn(2, 6)
    for f in (mpu.copy_to_model_parallel_region, mpu.reduce_from_model_parallel_region,
              mpu.scatter_to_model_parallel_region, mpu.gather_from_model_parallel_region):
        assert f(x) is x                       # every collective is bypassed at world size 1 (mappings.py:36,53,89)
    assert mpu.get_model_parallel_world_size() == 1 and mpu.get_model_parallel_rank() == 0
    mpu.set_model_parallel_world_size(3)
    mpu.set_model_parallel_rank(2)
    assert torch.equal(mpu.scatter_to_model_parallel_region(x), x[:, 4:6])
    with pytest.raises(RuntimeError, match="other tensor-parallel ranks"):
        mpu.gather_from_model_parallel_region(x)
    with pytest.raises(RuntimeError, match="MAX/SUM/SUM"):
        mpu.vocab_parallel_cross_entropy(torch.randn(2, 8), torch.tensor([1, 2]))


def test_split_tensor_along_last_dim():
    x = torch.arange(24.).view(2, 12)
    parts = mpu.split_tensor_along_last_dim(x, 3)
    assert [p.shape for p in parts] == [(2, 4)] * 3 and not parts[1].is_contiguous()
    assert all(p.is_contiguous() for p in mpu.split_tensor_along_last_dim(x, 3, True))
    with pytest.raises(AssertionError, match="12 is not divisible by 5"):
        mpu.split_tensor_along_last_dim(x, 5)


@settings(max_examples=200, deadline=None)
@given(per=st.integers(1, 10 ** 6), world=st.integers(1, 64), data=st.data())
def test_vocab_utility_matches_oracle(per, world, data):
    rank = data.draw(st.integers(0, world - 1))
    got = mpu.VocabUtility.vocab_range_from_global_vocab_size(per * world, rank, world)
    assert got == R.vocab_range_from_global_vocab_size(per * world, rank, world) == (rank * per, rank * per + per)
    assert mpu.divide(per * world, world) == per


def test_rope_tables_default_and_llama3_scaling_match_the_library():
    """cos / sin tables of the decoder against transformers' LlamaRotaryEmbedding (default rope type and the
    Llama-3.1 frequency rescale)."""
    from transformers import LlamaConfig
    from transformers.models.llama.modeling_llama import LlamaRotaryEmbedding
    from merak_amd.inference import rope_tables
    scaling = {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
               "original_max_position_embeddings": 8192, "rope_theta": 500000.0}
    pos = torch.tensor([[0, 1, 17, 4095, 8191, 20000]])
    for params in ({"rope_type": "default", "rope_theta": 10000.0}, scaling):
        cfg = LlamaConfig(hidden_size=512, num_attention_heads=4, head_dim=128, num_hidden_layers=1, vocab_size=32,
                          intermediate_size=64, max_position_embeddings=32768, rope_parameters=dict(params))
        cos, sin = LlamaRotaryEmbedding(cfg)(torch.zeros(1, pos.shape[1], 512), pos)
        mine_cos, mine_sin = rope_tables(128, 20001, params["rope_theta"],
                                         params if params["rope_type"] != "default" else None)
        assert torch.allclose(mine_cos[pos[0]], cos[0], atol=2e-4), params["rope_type"]
        assert torch.allclose(mine_sin[pos[0]], sin[0], atol=2e-4), params["rope_type"]
    with pytest.raises(NotImplementedError):
        rope_tables(128, 16, 10000.0, {"rope_type": "yarn"})


# ---- feature lists -> tags -> rebuilt layers (mp_attrs.py:43-202, model_parallel.py:87-99) ----
class _ToyAttn(nn.Module):
    def __init__(self, h):
        super().__init__()
        self.c_attn, self.c_proj = nn.Linear(h, 3 * h), nn.Linear(h, h)
        self.num_heads, self.split_size = 4, h


class _ToyMLP(nn.Module):
    def __init__(self, h):
        super().__init__()
        self.fc_in, self.fc_out = nn.Linear(h, 4 * h), nn.Linear(4 * h, h, bias=False)

    def forward(self, x):
        return self.fc_out(torch.nn.functional.gelu(self.fc_in(x), approximate="tanh"))


class _ToyModel(nn.Module):
    def __init__(self, h=64, v=100):
        super().__init__()
        self.wte = nn.Embedding(v, h)
        self.blocks = nn.ModuleList([nn.ModuleDict({"attn": _ToyAttn(h), "mlp": _ToyMLP(h)}) for _ in range(2)])
        self.head_scale = nn.Parameter(torch.ones(8, h))


def test_feature_lists_tag_and_rebuild_like_the_reference():
    from merak_amd.tensor_parallel import (set_tp_layer_lists, set_mp_attr, rebuild_module, mp_is_setted,
                                           get_tp_attr_list, reset_tp_layer_lists)
    reset_tp_layer_lists()
    assert not mp_is_setted()
    with pytest.raises(AssertionError, match="at least one kind of tp list"):
        set_tp_layer_lists(col_para_list=["c_attn"])                 # column names need row names (:181-183)
    set_tp_layer_lists(col_para_list=["c_attn", "fc_in"], row_para_list=["c_proj", "fc_out"],
                       weight_change_list=[("wte", 0), ("head_scale", 0)])
    assert mp_is_setted() and get_tp_attr_list() == []
    m = set_mp_attr(_ToyModel(), 2)
    b0 = m.blocks[0]
    assert (b0["attn"].c_attn.mp_attr, b0["attn"].c_attn.out_features, b0["attn"].c_attn.in_features) == ("col", 96, 64)
    assert (b0["attn"].c_proj.mp_attr, b0["attn"].c_proj.in_features) == ("row", 32)
    assert (b0["mlp"].fc_in.mp_attr, b0["mlp"].fc_in.out_features) == ("col", 128)
    assert (b0["mlp"].fc_out.mp_attr, b0["mlp"].fc_out.in_features) == ("row", 128)
    assert (b0["attn"].num_heads, b0["attn"].split_size) == (2, 32)         # default attribute list (:26-27)
    assert m.wte.weight.shape == (50, 64) and m.wte.num_embeddings == 50    # module weight cut along dim 0
    assert m.head_scale.shape == (4, 64)                                    # bare parameter cut along dim 0
    mpu.set_model_parallel_world_size(2)
    mpu.set_model_parallel_rank(1)
    rebuild_module(m, 2, init_method_normal(0.02), scaled_init_method_normal(0.02, 2))
    for blk in m.blocks:
        assert isinstance(blk["attn"].c_attn, ColPara) and isinstance(blk["mlp"].fc_in, ColPara)
        assert isinstance(blk["attn"].c_proj, RowPara) and isinstance(blk["mlp"].fc_out, RowPara)
        assert blk["attn"].c_attn.weight.shape == (96, 64) and blk["attn"].c_proj.weight.shape == (64, 32)
        assert blk["mlp"].fc_in.weight.shape == (128, 64) and blk["mlp"].fc_out.weight.shape == (64, 128)
        assert blk["mlp"].fc_out.bias is None and blk["mlp"].fc_in.bias.shape == (128,)
    assert "blocks.1.mlp.fc_in.col_linear.weight" in m.state_dict()
    # attributes that do not divide are refused with the reference's message (:140-141)
    reset_tp_layer_lists()
    set_tp_layer_lists(col_para_list=["c_attn"], row_para_list=["c_proj"], tp_attr_list=["num_heads"])
    with pytest.raises(AssertionError, match="mp attr set error, num_heads"):
        set_mp_attr(_ToyModel(), 3)
    reset_tp_layer_lists()


def test_input_output_ratio_table_tags_linear_and_conv1d():
    from transformers.pytorch_utils import Conv1D
    from merak_amd.tensor_parallel import set_tp_layer_lists, set_mp_attr, reset_tp_layer_lists, rebuild_module
    reset_tp_layer_lists()
    set_tp_layer_lists(input_output_mapping=[(1, 4, "col"), (4, 1, "row"), (1, 3, "col")])

    class GPT2ish(nn.Module):
        def __init__(self):
            super().__init__()
            self.c_fc, self.c_proj, self.c_attn = Conv1D(256, 64), Conv1D(64, 256), Conv1D(192, 64)   # (nf, nx)
            self.lin_up, self.lin_same = nn.Linear(64, 256), nn.Linear(64, 64)

    m = set_mp_attr(GPT2ish(), 4)
    assert (m.c_fc.mp_attr, m.c_fc.in_features, m.c_fc.out_features) == ("col", 64, 64)
    assert (m.c_proj.mp_attr, m.c_proj.in_features, m.c_proj.out_features) == ("row", 64, 64)
    assert (m.c_attn.mp_attr, m.c_attn.out_features) == ("col", 48)
    assert (m.lin_up.mp_attr, m.lin_up.out_features) == ("col", 64) and not hasattr(m.lin_same, "mp_attr")
    mpu.set_model_parallel_world_size(4)
    rebuild_module(m, 4, init_method_normal(0.02), scaled_init_method_normal(0.02, 1))
    assert isinstance(m.c_fc, ColPara) and m.c_fc.weight.shape == (64, 64)          # [out/p, in]
    assert isinstance(m.c_proj, RowPara) and m.c_proj.weight.shape == (64, 64)      # [out, in/p]
    assert isinstance(m.c_attn, ColPara) and m.c_attn.weight.shape == (48, 64)
    assert isinstance(m.lin_same, nn.Linear)                                        # untagged: left alone
    reset_tp_layer_lists()


def test_model_parallel_rng_gives_ranks_different_shards():
    """Device-side initialisation draws under the model-parallel generator state (layers.py:52-53): two ranks of one
    tensor-parallel group, seeded alike, get different shards; one rank seeded twice gets the same shard; the
    default generator is left where it was."""
    from merak_amd.mpu.layers import _initialize_affine_weight_gpu
    from merak_amd.mpu.random import get_rng_tracker

    def shard(rank, seed=1234):
        mpu.set_model_parallel_world_size(2)
        mpu.set_model_parallel_rank(rank)
        mpu.model_parallel_manual_seed(seed)
        before = torch.get_rng_state()
        w = torch.empty(8, 16)
        _initialize_affine_weight_gpu(w, torch.nn.init.normal_, 0)
        assert torch.equal(torch.get_rng_state(), before)          # the fork restores the caller's state
        assert w.model_parallel and w.partition_dim == 0 and w.partition_stride == 1
        return w

    a, b, a2 = shard(0), shard(1), shard(0)
    assert not torch.equal(a, b) and torch.equal(a, a2)
    # a second draw under the same state continues the stream, as the reference's fork does
    w1, w2 = torch.empty(4), torch.empty(4)
    mpu.model_parallel_manual_seed(7)
    _initialize_affine_weight_gpu(w1, torch.nn.init.normal_, 0)
    _initialize_affine_weight_gpu(w2, torch.nn.init.normal_, 0)
    assert not torch.equal(w1, w2)
    # an explicit context wins; without a seeded tracker the current generator is used
    get_rng_tracker().reset()
    torch.manual_seed(5)
    w3 = torch.empty(4)
    _initialize_affine_weight_gpu(w3, torch.nn.init.normal_, 0)
    torch.manual_seed(5)
    assert torch.equal(w3, torch.empty(4).normal_())
    with pytest.raises(Exception, match="already exists"):
        t = mpu.RNGStatesTracker()
        t.add("a", 1)
        t.add("b", 1)
