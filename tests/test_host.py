"""CPU tests of the host logic and of the C ABI's symbol table (no GPU, no compute calls)."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

from oracle import llama_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_loads_and_exports_every_declared_symbol():
    from easyllm_amd import _lib
    header = open(os.path.join(ROOT, "include", "ezl.h")).read()
    declared = sorted(set(re.findall(r"\b(ezl_[a-z0-9_]+)\s*\(", header)))
    assert len(declared) >= 25
    lib = _lib.load()
    for name in declared:
        assert hasattr(lib, name), "libezl.so does not export %s" % name
    assert sorted(_lib.exported_symbols()) == declared  # the Python binding covers exactly the header
    assert lib.ezl_version() >= 100
    assert isinstance(lib.ezl_last_error(), bytes)


def test_bad_arguments_are_rejected_without_a_gpu():
    """Argument validation happens on the host before any launch, so it is testable here."""
    from easyllm_amd import _lib
    lib = _lib.load()
    null = ctypes.c_void_p(None)
    rc = lib.ezl_rmsnorm_fwd(null, null, null, null, null, null, 4, 12, 1e-6, null)  # h % 8 != 0
    assert rc == -2 and b"h % 8" in lib.ezl_last_error()
    rc = lib.ezl_gemm_bf16(null, null, null, 8, 8, 8, 8, 8, 8, 1, 1, 0, 0, null, 0, null)  # null operands
    assert rc == -1
    strides = (ctypes.c_int64 * 8)(*([8] * 8))
    rc = lib.ezl_attn_fwd(null, null, null, null, null, null, 1, 16, 16, 4, 4, 96, 0.1, strides, null)  # head dim 96
    assert rc == -2 and b"head dim" in lib.ezl_last_error()
    rc = lib.ezl_ce_fused(null, null, null, null, null, null, 4, 30, 0, 0, null)  # vocab % 8 != 0
    assert rc == -2


def test_forward_without_gpu_fails_loudly():
    from easyllm_amd import kernels
    with pytest.raises(ValueError):
        kernels.swiglu_fwd(torch.zeros(8, dtype=torch.bfloat16), torch.zeros(8, dtype=torch.bfloat16))


def _tiny_kwargs(**over):
    kw = dict(num_layers=2, hidden_size=64, num_attention_heads=4, vocab_size=128, seq_length=16, bf16=True,
              use_cpu_initialization=True)
    kw.update(over)
    return kw


def test_registry_builds_model_with_reference_state_dict_layout():
    from easyllm_amd.runner import build_model
    m = build_model({"type": "llama_custom", "kwargs": _tiny_kwargs(num_kv_attention_heads=2, intermediate_size=96)})
    sd = m.state_dict()
    L = 2
    expect = {"1.word_embeddings.weight": (128, 64), "%d.weight" % (L + 4): (64,), "%d.word_embeddings.weight" % (L + 5): (128, 64)}
    for i in range(L):
        p = "%d." % (i + 3)
        expect.update({p + "input_layernorm.weight": (64,), p + "self_attn.q_proj.weight": (64, 64),
                       p + "self_attn.k_proj.weight": (32, 64), p + "self_attn.v_proj.weight": (32, 64),
                       p + "self_attn.o_proj.weight": (64, 64), p + "self_attn.rotary_emb.inv_freq": (8,),
                       p + "post_attention_layernorm.weight": (64,), p + "mlp.gate_proj.weight": (96, 64),
                       p + "mlp.up_proj.weight": (96, 64), p + "mlp.down_proj.weight": (64, 96)})
    assert {k: tuple(v.shape) for k, v in sd.items()} == expect
    assert all(v.dtype == torch.bfloat16 for k, v in sd.items() if "inv_freq" not in k)
    w = m.get_submodule("3").self_attn.q_proj.weight
    assert w.tensor_model_parallel and w.partition_dim == 0 and w.partition_stride == 1
    assert m.get_submodule("3").self_attn.o_proj.weight.partition_dim == 1
    assert m.model_kwargs == {"num_layers": 2, "checkpoint_activations": True}
    assert m.transformer_layer_params["glu_activation"] == "silu" and m.loss_fn.is_prefix is False
    assert torch.equal(sd["3.self_attn.rotary_emb.inv_freq"], O.rope_inv_freq(16))


def test_config_defaulting_rules():
    from easyllm_amd.default_cfg import update_model_cfg
    cfg = update_model_cfg(_tiny_kwargs(hidden_size=256, some_unknown_key=1))
    t = cfg["transformer_layer_params"]
    assert t["intermediate_size"] == 768 and t["kv_channels"] == 64 and t["num_kv_attention_heads"] == 4  # ceil256(8h/3)
    assert t["layer_norm"]["type"] == "rms_norm" and t["layer_norm"]["kwargs"]["eps"] == 1e-6
    assert t["output_initializer"]["kwargs"]["num_layers"] == 2 and t["params_dtype"] == "bfloat16"
    assert "some_unknown_key" not in cfg  # silently dropped, as in the reference
    assert cfg["loss_params"] == {"type": "softmax_cross_entropy", "kwargs": {"is_prefix": False}}
    cfg = update_model_cfg(_tiny_kwargs(hidden_size=4096, num_attention_heads=32))
    assert cfg["transformer_layer_params"]["intermediate_size"] == 11008
    cfg = update_model_cfg(_tiny_kwargs(vocab_size=130, unpad_vocab_size=128, loss_params={"kwargs": {"align_vocab_size_strict": True}}))
    assert cfg["loss_params"]["kwargs"]["cut_size"] == 2
    with pytest.raises(AssertionError):
        update_model_cfg(_tiny_kwargs(kv_channels=8))


def test_presets_and_key_conflicts():
    from easyllm_amd.llama import _LLAMA_MODELS, check_keys_mapping
    from easyllm_amd.registry import MODULE_ZOO_REGISTRY
    for name in ["llama_custom", "llama_7b", "llama_13b", "llama_20b", "llama_65b", "llama2_7b", "llama2_13b", "llama2_70b",
                 "codellama_7b", "codellama_13b", "codellama_34b"]:
        assert name in MODULE_ZOO_REGISTRY
    assert _LLAMA_MODELS["llama2_70b"]["num_kv_attention_heads"] == 8 and _LLAMA_MODELS["llama2_7b"]["intermediate_size"] == 11008
    with pytest.raises(AssertionError):
        check_keys_mapping(_LLAMA_MODELS["llama2_7b"], {"hidden_size": 1})


@pytest.mark.parametrize("seq_len", [1000, 4096, 4097, 16384, 32768, 40000])
def test_dynamic_checkpoint_rule_matches_oracle(seq_len):
    from easyllm_amd.runner import build_model
    dc = {"enabled": True, "size_map": {4096: 0, 8192: 2, 16384: 4, 32768: 8}}
    m = build_model({"type": "llama_custom", "kwargs": _tiny_kwargs(num_layers=8, dynamic_checkpoint=dc)})
    m.skip_checkpoint_layer_range = m.start_checkpoint_layer_idx + m.get_checkpoint_range(seq_len)
    got = [m._is_checkpointable([f]) for f in m.forward_funcs if f.__class__.__name__ == "ParallelTransformerLayerPipe"]
    assert got == O.checkpointed_layers(8, seq_len, True, dc)
    # embedding / norm / head / plain functions are never checkpointed
    others = [f for f in m.forward_funcs if f.__class__.__name__ != "ParallelTransformerLayerPipe"]
    assert not any(m._is_checkpointable([f]) for f in others)


def test_static_checkpoint_settings():
    from easyllm_amd.runner import build_model
    m = build_model({"type": "llama_custom", "kwargs": _tiny_kwargs()})  # checkpoint_activations default True, no size_map
    layers = [f for f in m.forward_funcs if f.__class__.__name__ == "ParallelTransformerLayerPipe"]
    assert m.activation_checkpoint_interval == 1 and all(m._is_checkpointable([f]) for f in layers)
    m = build_model({"type": "llama_custom", "kwargs": _tiny_kwargs(checkpoint_activations=False)})
    assert m.activation_checkpoint_interval == 0
    # a chunk that mixes a layer with a non-layer is not checkpointable (interval > 1)
    m = build_model({"type": "llama_custom", "kwargs": _tiny_kwargs(checkpoint_num_layers=2)})
    assert not m._is_checkpointable(m.forward_funcs[2:4]) and m._is_checkpointable(m.forward_funcs[3:5])


def test_packed_input_producers_match_oracle():
    from easyllm_amd import data
    rng = np.random.RandomState(0)
    for _ in range(20):
        toks = rng.randint(0, 5, size=rng.randint(1, 40))
        cu = data.get_cu_seqlens(toks, 2)
        assert cu == O.get_cu_seqlens(toks, 2)
        assert data.get_position_ids(cu) == O.get_position_ids(cu)
    assert data.get_cu_seqlens(np.array([7, 7, 2, 7, 7, 2, 7, 7]), 2) == [0, 3, 6, 8]
    flat = data.flatten_cu_seqlens([[0, 3, 6, 8], [0, 5, 9]], 8)
    assert flat.tolist() == O.flatten_cu_seqlens([[0, 3, 6, 8], [0, 5, 9]], 8).tolist() == [0, 3, 6, 8, 13, 16]
    assert data.packed_doc_lengths(16384, 64, 4096, 1005) == O.packed_doc_lengths(16384, 64, 4096, 1005)


def test_batch_tuple_layouts():
    from easyllm_amd import data
    tokens = torch.tensor([[5, 6, 9, 9]])
    labels = torch.tensor([[6, 9, -100, -100]])
    (t, pos, mask), (lab, lm) = data.flash_batch(tokens, labels, pad_token_id=9)
    assert pos.tolist() == [[0, 1, 2, 3]] and lm.dtype == torch.bool and lm.tolist() == [[True, True, False, False]]
    (t, pos, mask), (lab, lm) = data.json_batch(tokens, labels, pad_token_id=9)
    assert lm.dtype == torch.float32 and lm.tolist() == [[1.0, 1.0, 0.0, 0.0]]
    cu = torch.tensor([0, 2, 4])
    out = data.flash_batch(tokens, labels, 9, cu_seqlens=cu, position_ids=torch.tensor([[0, 1, 0, 1]]))
    assert len(out[0]) == 4 and out[0][3] is cu


def test_workload_flops_and_inputs():
    from easyllm_amd import workloads as W
    assert abs(W.step_flops(W.WORKLOADS["C2"]) / O.step_flops(dict(num_layers=4, hidden_size=4096, num_attention_heads=32,
               num_kv_attention_heads=32, head_dim=128, intermediate_size=11008, vocab_size=32000), 1, 4096) - 1) < 1e-12
    inputs, (labels, lm), doc_lens = W.make_inputs(W.WORKLOADS["C5"])
    assert sum(doc_lens) == 16384 and inputs[3][-1] == 16384 and inputs[1].shape == (1, 16384)
    _, (labels, _), _ = W.make_inputs(W.WORKLOADS["C4"])
    frac = (labels == -100).float().mean().item()
    assert 0.08 < frac < 0.12


def test_checkpoint_function_recomputes_and_matches(monkeypatch):
    """The recompute wrapper itself is device independent: same grads with and without it."""
    from easyllm_amd.checkpointing import checkpoint
    lin = torch.nn.Linear(8, 8)
    calls = {"n": 0}

    def chunk(x, aux):
        calls["n"] += 1
        return torch.tanh(lin(x)) * 2.0, aux

    x = torch.randn(4, 8, requires_grad=True)
    aux = torch.arange(3)
    y, aux_out = checkpoint(chunk, x, aux)
    assert torch.equal(aux_out, aux) and calls["n"] == 1
    y.sum().backward()
    assert calls["n"] == 2  # forward ran again inside backward
    g1, gw1 = x.grad.clone(), lin.weight.grad.clone()
    x.grad = None
    lin.weight.grad = None
    chunk(x, aux)[0].sum().backward()
    assert torch.equal(g1, x.grad) and torch.equal(gw1, lin.weight.grad)


def test_weight_decay_split_and_optimizer_config_errors():
    """optimizer_helper.py:19-51,70-72: biases and MixedFusedLayerNorm modules get no decay (RMSNorm weights do, as in
    the reference); cpu_optimizer is refused."""
    import torch
    from easyllm_amd import optimizer
    from easyllm_amd.layers import RMSNorm

    class MixedFusedLayerNorm(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.weight = torch.nn.Parameter(torch.ones(4))

    class Toy(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.lin = torch.nn.Linear(4, 4, bias=True)
            self.norm = RMSNorm(True, 4)
            self.ln = MixedFusedLayerNorm()
            self.frozen = torch.nn.Linear(4, 4, bias=False)
            self.frozen.weight.requires_grad = False

    toy = Toy()
    decay, no_decay = optimizer.get_params_for_weight_decay_optimization(toy)
    assert {id(p) for p in decay["params"]} == {id(toy.lin.weight), id(toy.frozen.weight), id(toy.norm.weight)}
    assert {id(p) for p in no_decay["params"]} == {id(toy.lin.bias), id(toy.ln.weight)} and no_decay["weight_decay"] == 0.0
    groups = optimizer.filter_freeze_param_groups([{"params": [toy.frozen.weight]}, decay])
    assert len(groups) == 1 and groups[0] is decay
    with pytest.raises(NotImplementedError):
        optimizer.build_optimizer({"type": "FusedAdam", "cpu_optimizer": True, "kwargs": {}}, toy)
    with pytest.raises(NotImplementedError):
        optimizer.build_optimizer({"type": "SophiaG", "kwargs": {}}, toy)
    with pytest.raises(RuntimeError):
        optimizer.FusedAdam([toy.lin.weight], amsgrad=True)
    with pytest.raises(ValueError):  # parameters without fp32 gradient buffers are rejected before any GPU work
        optimizer.FusedAdam([toy.lin.weight])
