"""Model kwargs -> per-module parameter dicts (reference: llama/default_cfg.py:11-256).

Accepted top-level keys are those of SHARED_DEFAULTS and MODEL_DEFAULTS plus the five nested dicts
(`word_embedings_params`, `layer_norm_params`, `transformer_layer_params`, `lm_head_params`,
`loss_params`).  As in the reference, unknown top-level keys do not raise: the reference's check at
:57 compares the merged dict with itself, and the keep-list at :85-88 then drops what the pipe
constructor does not take.
"""
import copy

from .layers import check_torch_dtype

SHARED_DEFAULTS = {
    "num_layers": None, "vocab_size": None, "unpad_vocab_size": None, "kv_channels": None,
    "num_attention_heads": None, "num_kv_attention_heads": None, "intermediate_size": None, "seq_length": None,
    "hidden_size": None, "hidden_dropout": 0, "position_embedding_type": "rotary", "position_embedding_kwargs": None,
    "params_dtype": None, "pretrain_causal_attention": True, "use_cpu_initialization": False, "parallel_output": True,
    "sync_tp_duplicated_parameters": True, "sequence_parallel": False, "fp16": False, "bf16": False,
    "attn_mask_type": "causal", "fp32_residual_connection": False, "micro_batch_size": 1, "use_flash_attn": True,
}
MODEL_DEFAULTS = {
    "checkpoint_activations": True, "checkpoint_num_layers": 1, "dynamic_checkpoint": None,
    "pp_partition_method": "type:transformer|embedding",
    # not in the reference: False leaves the logits in bf16 for the loss kernel (which reads bf16 and
    # accumulates in fp32) instead of materialising the fp32 copy of llama.py:187-188
    "fp32_logits": True,
}
PIPE_KWARGS = ("num_layers", "parallel_output", "fp16", "bf16", "fp32_residual_connection", "pretrain_causal_attention",
               "checkpoint_activations", "checkpoint_num_layers", "dynamic_checkpoint", "pp_partition_method",
               "sequence_parallel", "fp32_logits")
EMBEDDING_DEFAULTS = {
    "num_tokentypes": 0, "max_position_embeddings": None, "use_bnb_optimizer": False,
    "initializer": {"type": "normal", "kwargs": {"sigma": 0.02}},
}
LAYER_NORM_DEFAULTS = {"eps": 1e-6}
TRANSFORMER_LAYER_DEFAULTS = {
    "layer_type": "encoder", "layer_norm": None, "apply_residual_connection_post_layernorm": False,
    "apply_query_key_layer_scaling": True, "attention_softmax_in_fp32": False, "masked_softmax_fusion": True,
    "attention_dropout": 0, "bias_gelu_fusion": False, "glu_activation": "silu", "use_openai_gelu": False,
    "onnx_safe": None, "bias_dropout_fusion": True,
    "initializer": {"type": "normal", "kwargs": {"sigma": 0.02}},
    "output_initializer": {"type": "scaled_normal", "kwargs": {"sigma": 0.02, "num_layers": 32}},
    "qkv_pack": False, "attention_qkv_bias": False, "attention_o_bias": False,
}


def update_shared_config(cfg):
    shared = copy.deepcopy(SHARED_DEFAULTS)
    merged = copy.deepcopy(MODEL_DEFAULTS)
    merged.update(cfg)
    for key, value in merged.items():
        if key in shared:
            shared[key] = value
    shared["params_dtype"] = check_torch_dtype(shared["params_dtype"], shared["fp16"], shared["bf16"])
    if shared["fp32_residual_connection"]:
        assert shared["fp16"] or shared["bf16"], "residual connection in fp32 only supported when using fp16 or bf16."
    assert shared["num_layers"] is not None and shared["hidden_size"] is not None and shared["num_attention_heads"] is not None
    assert shared["hidden_size"] % shared["num_attention_heads"] == 0
    per_head = shared["hidden_size"] // shared["num_attention_heads"]
    if shared["kv_channels"] is None:
        shared["kv_channels"] = per_head
    else:
        assert shared["kv_channels"] == per_head
    if shared["intermediate_size"] is None:  # ceil256(8h/3), :77-78
        shared["intermediate_size"] = ((int(2 * (4 * shared["hidden_size"]) / 3) + 255) // 256) * 256
    if shared["num_kv_attention_heads"] is None:
        shared["num_kv_attention_heads"] = shared["num_attention_heads"]
    merged.update(shared)
    pipe_cfg = {k: v for k, v in merged.items() if k in PIPE_KWARGS}
    return pipe_cfg, shared


def update_embeding_config(cfg, shared, as_head=False):
    out = copy.deepcopy(EMBEDDING_DEFAULTS)
    mapping = {"hidden_size": "hidden_size", "vocab_size": "vocab_size", "embedding_dropout_prob": "hidden_dropout",
               "position_embedding_type": "position_embedding_type", "params_dtype": "params_dtype",
               "pretrain_causal_attention": "pretrain_causal_attention", "use_cpu_initialization": "use_cpu_initialization",
               "sequence_parallel": "sequence_parallel"}
    if as_head:
        mapping["parallel_output"] = "parallel_output"
    for key, src in mapping.items():
        out[key] = shared[src]
    out.update(cfg)
    if shared["position_embedding_type"] in ("absolute", "alibi"):
        assert out["max_position_embeddings"] is not None
        if shared["seq_length"] is not None:
            assert out["max_position_embeddings"] >= shared["seq_length"]
    else:
        assert out["max_position_embeddings"] is None
    return out


def update_ln_config(cfg, shared):
    out = copy.deepcopy(LAYER_NORM_DEFAULTS)
    for key, src in {"sync_tp_duplicated_parameters": "sync_tp_duplicated_parameters", "normalized_shape": "hidden_size",
                     "use_flash_attn": "use_flash_attn", "bf16": "bf16", "sequence_parallel": "sequence_parallel"}.items():
        out[key] = shared[src]
    out.update(cfg)
    return out


def update_transformer_layer_config(cfg, shared, ln_cfg, num_layers):
    out = copy.deepcopy(TRANSFORMER_LAYER_DEFAULTS)
    mapping = {"self_attn_mask_type": "attn_mask_type"}
    for key in ("position_embedding_type", "position_embedding_kwargs", "params_dtype", "fp16", "bf16",
                "fp32_residual_connection", "kv_channels", "num_attention_heads", "num_kv_attention_heads", "hidden_size",
                "use_cpu_initialization", "sync_tp_duplicated_parameters", "sequence_parallel", "use_flash_attn",
                "hidden_dropout", "intermediate_size", "seq_length", "micro_batch_size"):
        mapping[key] = key
    for key, src in mapping.items():
        out[key] = shared[src]
    out.update(cfg)
    if out["layer_norm"] is None:
        out["layer_norm"] = ln_cfg
    if out["output_initializer"]["kwargs"].get("num_layers", None):
        out["output_initializer"]["kwargs"]["num_layers"] = num_layers
    if out["glu_activation"] is not None and out["bias_gelu_fusion"]:
        raise ValueError("if glu-activation is used, please set bias-gelu-fusion to false")
    return out


def update_loss_config(cfg, shared):
    cfg.update({"is_prefix": shared["attn_mask_type"] == "prefix"})
    if cfg.pop("align_vocab_size_strict", False):
        if shared["vocab_size"] != shared["unpad_vocab_size"]:
            cfg.update({"cut_size": shared["vocab_size"] - shared["unpad_vocab_size"]})
    return cfg


def update_model_cfg(cfg):
    word_embedings_cfg = cfg.pop("word_embedings_params", {})
    layer_norm_cfg = cfg.pop("layer_norm_params", {})
    transformer_layer_cfg = cfg.pop("transformer_layer_params", {})
    lm_head_cfg = cfg.pop("lm_head_params", {})
    loss_cfg = cfg.pop("loss_params", {})
    cfg, shared = update_shared_config(cfg)
    word_embedings_cfg = update_embeding_config(word_embedings_cfg, shared, as_head=False)
    layer_norm_cfg["type"] = layer_norm_cfg.get("type", "rms_norm")
    layer_norm_cfg["kwargs"] = update_ln_config(layer_norm_cfg.get("kwargs", {}), shared)
    transformer_layer_cfg = update_transformer_layer_config(transformer_layer_cfg, shared, layer_norm_cfg,
                                                            num_layers=cfg["num_layers"])
    lm_head_cfg = update_embeding_config(lm_head_cfg, shared, as_head=True)
    loss_cfg["type"] = loss_cfg.get("type", "softmax_cross_entropy")
    loss_cfg["kwargs"] = update_loss_config(loss_cfg.get("kwargs", {}), shared)
    cfg["word_embedings_params"] = word_embedings_cfg
    cfg["layer_norm_params"] = layer_norm_cfg
    cfg["transformer_layer_params"] = transformer_layer_cfg
    cfg["lm_head_params"] = lm_head_cfg
    cfg["loss_params"] = loss_cfg
    return cfg
