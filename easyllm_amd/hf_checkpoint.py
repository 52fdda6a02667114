"""Loading Hugging Face-format checkpoints into the Megatron-layout llama stack, and writing them back.

Counterpart of llm/models/mg_models/llama/utils.py:58-350 of the reference: the key maps `hf_to_megatron_llama`
(:158-219), `qwen_to_llama` (:58-110), `internlm2_to_llama2` (:113-155), the tensor-parallel slicing rule of
`load_func` (:233-303, with `get_start_end` :222-231) and the directory loader `load_llama_from_hf_format` (:307-350).
Target keys are the kept state-dict layout: `1.word_embeddings.weight`, `{i+3}.self_attn.q_proj.weight`, ...,
`{L+4}.weight`, `{L+5}.word_embeddings.weight` (the reference addresses the same modules through its engine wrapper
as `module.<key>`; both spellings are accepted when copying).  `megatron_to_hf_llama` is the inverse map for export.

Pickle-based `.bin` shards are read with `torch.load(..., weights_only=True)` only; object-store (`.ceph`) listings
and LoRA adapters are not supported.
"""
import glob
import logging
import os

import torch

from .layers import ColumnParallelLinear, RowParallelLinear, VocabParallelEmbedding

logger = logging.getLogger(__name__)

# HF llama parameter name inside `model.layers.<i>.` -> name inside layer module `<i+3>.`
_LLAMA_LAYER_KEYS = {
    "self_attn.q_proj": "self_attn.q_proj", "self_attn.k_proj": "self_attn.k_proj", "self_attn.v_proj": "self_attn.v_proj",
    "self_attn.o_proj": "self_attn.o_proj", "mlp.gate_proj": "mlp.gate_proj", "mlp.down_proj": "mlp.down_proj",
    "mlp.up_proj": "mlp.up_proj", "post_attention_layernorm": "post_attention_layernorm", "input_layernorm": "input_layernorm",
}


def _num_layers(model):
    return model.model_kwargs["num_layers"]


def _layer_id(key):
    return int(key.split(".")[2])


def hf_to_megatron_llama(dt, model, pack=False):
    """LlamaForCausalLM names -> stack names.  pack=True gathers q/k/v into one `wqkv` entry holding the list [q, k, v]
    (sliced per rank before concatenation by `copy_into_model`)."""
    L = _num_layers(model)
    out = {}
    for key, value in dt.items():
        if "model.embed_tokens" in key:
            out["1.word_embeddings.weight"] = value
        elif "model.norm" in key:
            out["%d.weight" % (L + 4)] = value
        elif "lm_head" in key:
            out["%d.word_embeddings.weight" % (L + 5)] = value
        elif "layers" in key:
            prefix = "%d." % (_layer_id(key) + 3)
            kind = "weight" if "weight" in key else "bias"
            for hf_name, name in _LLAMA_LAYER_KEYS.items():
                if hf_name not in key:
                    continue
                if pack and hf_name in ("self_attn.k_proj", "self_attn.v_proj"):
                    continue  # carried by the q_proj entry
                if pack and hf_name == "self_attn.q_proj":
                    k_key, v_key = key.replace("q_proj", "k_proj"), key.replace("q_proj", "v_proj")
                    assert k_key in dt and v_key in dt, \
                        "Pack mode only suport q_proj, k_proj, v_proj in one checkpoint, please re-formula your checkpoint file."
                    out[prefix + "self_attn.wqkv." + kind] = [value, dt[k_key], dt[v_key]]
                elif hf_name.startswith("self_attn"):
                    out[prefix + name + "." + kind] = value
                else:  # MLP and norm entries are weights only (utils.py:206-215)
                    out[prefix + name + ".weight"] = value
        else:
            logger.info("unuse keys %s", key)
    return out


def qwen_to_llama(dt, model):
    """Qwen (v1) names: fused `c_attn` split into thirds; `w2` is the gate, `w1` the up projection (utils.py:99-104)."""
    L = _num_layers(model)
    hid = model.transformer_layer_params["hidden_size"]
    out = {}
    for key, value in dt.items():
        if "wte.weight" in key:
            out["1.word_embeddings.weight"] = value
        elif "ln_f.weight" in key:
            out["%d.weight" % (L + 4)] = value
        elif "lm_head.weight" in key:
            out["%d.word_embeddings.weight" % (L + 5)] = value
        elif "transformer.h" in key:
            prefix = "%d." % (_layer_id(key) + 3)
            if "attn.c_attn.weight" in key:
                for name, part in zip("qkv", torch.chunk(value, 3, dim=0)):
                    out[prefix + "self_attn.%s_proj.weight" % name] = part.reshape(-1, hid)
            if "attn.c_attn.bias" in key:
                for name, part in zip("qkv", torch.chunk(value, 3, dim=0)):
                    out[prefix + "self_attn.%s_proj.bias" % name] = part.reshape(-1)
            if "attn.c_proj" in key:
                out[prefix + "self_attn.o_proj.weight"] = value
            if "mlp.w2.weight" in key:
                out[prefix + "mlp.gate_proj.weight"] = value
            if "mlp.c_proj.weight" in key:
                out[prefix + "mlp.down_proj.weight"] = value
            if "mlp.w1.weight" in key:
                out[prefix + "mlp.up_proj.weight"] = value
            if "ln_2.weight" in key:
                out[prefix + "post_attention_layernorm.weight"] = value
            if "ln_1.weight" in key:
                out[prefix + "input_layernorm.weight"] = value
        else:
            logger.info("unuse keys %s", key)
    return out


def internlm2_to_llama2(dt, model, pack=False):
    """InternLM2 names: `wqkv` rows are grouped per KV head as [gs query heads, key, value] (utils.py:127-133)."""
    L = _num_layers(model)
    p = model.transformer_layer_params
    n_heads, n_kv, hid = p["num_attention_heads"], p["num_kv_attention_heads"], p["hidden_size"]
    gs, head_dim = n_heads // n_kv, hid // n_heads
    out = {}
    for key, value in dt.items():
        if "tok_embeddings" in key:
            out["1.word_embeddings.weight"] = value
        elif "model.norm.weight" in key:
            out["%d.weight" % (L + 4)] = value
        elif "output" in key:
            out["%d.word_embeddings.weight" % (L + 5)] = value
        elif "layers" in key:
            prefix = "%d." % (_layer_id(key) + 3)
            if "attention.wqkv" in key:
                grouped = value.reshape(-1, gs + 2, head_dim, hid)
                q = grouped[:, :gs].reshape(-1, hid)
                k = grouped[:, -2].reshape(-1, hid)
                v = grouped[:, -1].reshape(-1, hid)
                if pack:
                    out[prefix + "self_attn.wqkv.weight"] = [q, k, v]
                else:
                    out[prefix + "self_attn.q_proj.weight"], out[prefix + "self_attn.k_proj.weight"] = q, k
                    out[prefix + "self_attn.v_proj.weight"] = v
            for src, dst in (("attention.wo", "self_attn.o_proj"), ("feed_forward.w1", "mlp.gate_proj"),
                             ("feed_forward.w2", "mlp.down_proj"), ("feed_forward.w3", "mlp.up_proj"),
                             ("ffn_norm.weight", "post_attention_layernorm"), ("attention_norm.weight", "input_layernorm")):
                if src in key:
                    out[prefix + dst + ".weight"] = value
        else:
            logger.info("unuse keys %s", key)
    return out


def megatron_to_hf_llama(state_dict, num_layers):
    """Inverse of `hf_to_megatron_llama` (unpacked form) for export; `inv_freq` buffers are dropped."""
    out = {}
    for key, value in state_dict.items():
        key = key[len("module."):] if key.startswith("module.") else key
        if "inv_freq" in key:
            continue
        idx, _, rest = key.partition(".")
        idx = int(idx)
        if idx == 1:
            out["model.embed_tokens.weight"] = value
        elif idx == num_layers + 4:
            out["model.norm.weight"] = value
        elif idx == num_layers + 5:
            out["lm_head.weight"] = value
        elif 3 <= idx < num_layers + 3:
            if "wqkv" in rest:
                raise NotImplementedError("export of packed wqkv weights: split them with the model's head counts first")
            out["model.layers.%d.%s" % (idx - 3, rest)] = value
        else:
            raise KeyError("unexpected key %s" % key)
    return out


def get_start_end(size, tp_world_size, tp_rank):
    """[begin, end) of rank tp_rank when every rank owns `size` consecutive rows (utils.py:222-231)."""
    assert 0 <= tp_rank < tp_world_size
    return [size * tp_rank, size * (tp_rank + 1)]


def slice_for_rank(value, module, param_shape, tp_rank, tp_world_size):
    """The part of a full checkpoint tensor that belongs to this rank's parameter (utils.py:262-286)."""
    if isinstance(module, VocabParallelEmbedding):
        start, stop = get_start_end(param_shape[0], tp_world_size, tp_rank)
        return value[start:stop]
    if isinstance(module, ColumnParallelLinear):
        if isinstance(value, (list, tuple)):  # packed [q, k, v]: slice each, then concatenate
            parts = []
            for t in value:
                start, stop = get_start_end(t.shape[0] // tp_world_size, tp_world_size, tp_rank)
                parts.append(t[start:stop])
            return torch.cat(parts, dim=0)
        start, stop = get_start_end(param_shape[0], tp_world_size, tp_rank)
        return value[start:stop]
    if isinstance(module, RowParallelLinear):
        if len(param_shape) == 1:  # bias: replicated
            return value
        start, stop = get_start_end(param_shape[1], tp_world_size, tp_rank)
        return value[:, start:stop]
    return value[:]


def _find_param(name, model):
    for candidate in (name, name[len("module."):] if name.startswith("module.") else "module." + name):
        mod_name, _, attr = candidate.rpartition(".")
        try:
            module = model.get_submodule(mod_name)
        except AttributeError:
            continue
        param = getattr(module, attr, None)
        if isinstance(param, torch.Tensor):
            return param, module
    return None, None


def copy_into_model(dt, model, tp_rank=0, tp_world_size=1, init_set=None):
    """Copies converted tensors into the model's parameters; returns the set of names that were initialised.
    A parameter with more rows than the checkpoint (padded vocabulary) keeps the checkpoint rows and fills the rest with
    0.1 x the checkpoint row of smallest sum, as the reference does (utils.py:290-296)."""
    init_set = set() if init_set is None else init_set
    for name, value in dt.items():
        param, module = _find_param(name, model)
        if param is None:
            continue
        tensor = slice_for_rank(value, module, tuple(param.shape), tp_rank, tp_world_size)
        with torch.no_grad():
            if tuple(param.shape) != tuple(tensor.shape):
                if param.dim() != 2 or tensor.dim() != 2 or tensor.shape[0] > param.shape[0] or tensor.shape[1] != param.shape[1]:
                    raise ValueError("Name %s -- current %s and got %s" % (name, tuple(param.shape), tuple(tensor.shape)))
                padded = param.data.clone()
                padded[:tensor.size(0)] = tensor.to(padded.dtype)
                donor = int(value.float().sum(1).argmin())
                padded[tensor.size(0):] = (value[donor].float() * 0.1).to(padded.dtype)
                param.data.copy_(padded)
            else:
                param.data.copy_(tensor.to(param.dtype))
        init_set.add(name)
    return init_set


_CONVERTERS = {
    "llama": lambda dt, model: hf_to_megatron_llama(dt, model, pack=False),
    "llama_pack": lambda dt, model: hf_to_megatron_llama(dt, model, pack=True),
    "internlm2": lambda dt, model: internlm2_to_llama2(dt, model, pack=False),
    "internlm2_pack": lambda dt, model: internlm2_to_llama2(dt, model, pack=True),
    "qwen": qwen_to_llama,
}


def load_shard(filename):
    if filename.endswith(".safetensors"):
        from safetensors.torch import load_file
        return load_file(filename)
    return torch.load(filename, map_location="cpu", weights_only=True)


def load_llama_from_hf_format(load_dir, model, optimizer=None, num_layers=None, lora_mode=False, worker=8, pretrain_type="llama",
                              tp_rank=0, tp_world_size=1):
    """Reads every `*.bin` (else `*.safetensors`) shard of load_dir into `model`; False when there is none
    (utils.py:307-350).  Returns True after logging the parameters no shard initialised."""
    if lora_mode:
        raise NotImplementedError("LoRA checkpoints are not supported")
    if pretrain_type not in _CONVERTERS:
        raise ValueError("%s is not be supported" % pretrain_type)
    filenames = sorted(glob.glob(os.path.join(load_dir, "*.bin"))) or sorted(glob.glob(os.path.join(load_dir, "*.safetensors")))
    if not filenames:
        return False
    init_set = set()
    for filename in filenames:  # shards are independent; read sequentially (`worker` kept for call compatibility)
        logger.info("loadding %s", filename)
        copy_into_model(_CONVERTERS[pretrain_type](load_shard(filename), model), model, tp_rank, tp_world_size, init_set)
    known = {k[len("module."):] if k.startswith("module.") else k for k in init_set}
    missing = {k for k in model.state_dict().keys() if "inv_freq" not in k and k not in known}
    logger.info("not init set %s", missing)
    if optimizer is not None and hasattr(optimizer, "refresh_fp32_params"):
        optimizer.refresh_fp32_params()
    return True
