"""LlamaModelPipe: the flat spec list of the reference (llama/llama.py:22-190), its dynamic
activation-checkpoint rule (:97-137), the size presets (:193-266) and the registry entry points
(:269-349, llama/__init__.py:14-19).

The reference subclasses DeepSpeed's PipelineModule; DeepSpeed is not part of this build, so the two
things the step needs from it are restated here: modules are registered under their spec index (state
dict keys `3.self_attn.q_proj.weight`, ...), and `forward` walks the list in chunks of
`activation_checkpoint_interval`, checkpointing a chunk iff `_is_checkpointable(chunk)`.
"""
import math

import torch

from . import dist_env
from . import functional as F_
from .checkpointing import checkpoint
from .default_cfg import update_model_cfg
from .layers import LayerSpec, build_layer_norm
from .lm_head import EmbedddingPipeNoTied
from .registry import LOSS_REGISTRY, MODULE_ZOO_REGISTRY
from .transformer import ParallelTransformerLayerPipe
from .word_embedings import EmbeddingPipe
from . import losses as _losses  # noqa: F401  (registers 'softmax_cross_entropy')


def fp32_to_float16(val, convertor):
    """Casts fp32 floating tensors of a (nested) tuple; ids and masks pass untouched (fp16_module.py:24-33)."""
    if isinstance(val, (tuple, list)):
        out = [fp32_to_float16(v, convertor) for v in val]
        return tuple(out) if isinstance(val, tuple) else out
    if torch.is_tensor(val) and val.dtype == torch.float32:
        return convertor(val)
    return val


def float16_to_fp32(val):
    """Casts bf16/fp16 tensors of a (nested) tuple to fp32 (fp16_module.py:36-45)."""
    if isinstance(val, (tuple, list)):
        out = [float16_to_fp32(v) for v in val]
        return tuple(out) if isinstance(val, tuple) else out
    if torch.is_tensor(val) and val.dtype == torch.bfloat16:
        return F_.to_fp32(val)
    if torch.is_tensor(val) and val.dtype == torch.float16:
        return val.float()
    return val


class LlamaModelPipe(torch.nn.Module):
    def __init__(self, num_layers, parallel_output=True, fp16=False, bf16=True, fp32_residual_connection=False,
                 pretrain_causal_attention=False, checkpoint_activations=True, checkpoint_num_layers=1,
                 pp_partition_method="type:transformer|embedding", sequence_parallel=False, dynamic_checkpoint=None,
                 word_embedings_params=None, transformer_layer_params=None, layer_norm_params=None, lm_head_params=None,
                 loss_params=None, fp32_logits=True):
        super().__init__()
        self.parallel_output = parallel_output
        self.sequence_parallel = sequence_parallel
        self.fp32_logits = fp32_logits  # False: leave bf16 logits for the loss kernel to read directly
        self._set_model_kwargs(num_layers, checkpoint_activations)
        self.word_embedings_params = word_embedings_params
        self.transformer_layer_params = transformer_layer_params
        self.layer_norm_params = layer_norm_params
        self.lm_head_params = lm_head_params
        self.loss_params = loss_params
        self.specs = self.build_specs(num_layers, fp16, bf16, fp32_residual_connection, pretrain_causal_attention)
        self.loss_fn = LOSS_REGISTRY.build(self.loss_params)
        self.activation_checkpoint_interval = checkpoint_num_layers if checkpoint_activations else 0
        self.size_map = None
        self.skip_checkpoint_layer_range = -1
        if dynamic_checkpoint is not None and dynamic_checkpoint["enabled"]:
            self.size_map = dynamic_checkpoint["size_map"]
        self.num_layers_per_pp = math.ceil(num_layers / dist_env.get_pipeline_model_parallel_world_size())
        self.start_checkpoint_layer_idx = self.num_layers_per_pp * dist_env.get_pipeline_model_parallel_rank()
        self.skip_checkpoint_layer_range += self.start_checkpoint_layer_idx
        self.activation_checkpoint_func = checkpoint
        self.recompute_count = 0  # chunks re-run in backward during the last forward (for tests / logs)
        self.forward_funcs = []
        for idx, spec in enumerate(self.specs):
            if isinstance(spec, LayerSpec):
                module = spec.build()
                self.add_module(str(idx), module)
                self.forward_funcs.append(module)
            elif isinstance(spec, torch.nn.Module):
                self.add_module(str(idx), spec)
                self.forward_funcs.append(spec)
            else:
                self.forward_funcs.append(spec)

    # ---- dynamic checkpoint rule ------------------------------------------------------------
    def _is_checkpointable(self, funcs):
        if self.skip_checkpoint_layer_range < self.start_checkpoint_layer_idx:
            return all("ParallelTransformerLayerPipe" in f.__class__.__name__ for f in funcs)
        flag = True
        for f in funcs:
            flag = flag and ("ParallelTransformerLayerPipe" in f.__class__.__name__)
            if hasattr(f, "layer_number"):
                flag = flag and (f.layer_number < self.skip_checkpoint_layer_range)
        return flag

    def get_checkpoint_range(self, seq_len):
        for item in sorted(self.size_map.keys()):
            if seq_len <= item:
                return self.size_map[item]
        return -1

    def get_seq_len(self, forward_input):
        return forward_input[0].shape[1]  # first (and only) pipeline stage: tokens [b, s]

    def forward(self, forward_input):
        seq_len = self.get_seq_len(forward_input)
        if self.size_map is not None:
            self.skip_checkpoint_layer_range = self.start_checkpoint_layer_idx + self.get_checkpoint_range(seq_len)
        return self._forward_specs(forward_input)

    def _forward_specs(self, x):
        funcs_all = self.forward_funcs
        n = len(funcs_all)

        def exec_range(start, end):
            def run(*inputs):
                inputs = inputs[0] if len(inputs) == 1 else inputs
                for f in funcs_all[start:end]:
                    inputs = f(inputs)
                return inputs
            return run

        self.recompute_count = 0
        interval = self.activation_checkpoint_interval
        if interval == 0:
            return exec_range(0, n)(x)
        for start in range(0, n, interval):
            end = min(start + interval, n)
            funcs = funcs_all[start:end]
            if not isinstance(x, tuple):
                x = (x,)
            if self._is_checkpointable(funcs) and torch.is_grad_enabled():
                self.recompute_count += 1
                x = self.activation_checkpoint_func(exec_range(start, end), *x)
            else:
                x = exec_range(start, end)(*x)
        return x

    def _set_model_kwargs(self, num_layers, checkpoint_activations):
        self.model_kwargs = {"num_layers": num_layers, "checkpoint_activations": checkpoint_activations}

    def build_specs(self, num_layers, fp16, bf16, fp32_residual_connection, pretrain_causal_attention):
        if fp16:
            raise NotImplementedError("the HIP path computes in bf16; fp16 is not built")
        if not bf16:
            raise NotImplementedError("the HIP path computes in bf16 (set bf16=True); fp32 end-to-end is the CPU oracle's job")
        specs = []

        def _to_float16(inputs):
            return fp32_to_float16(inputs, lambda v: v.bfloat16())
        specs.append(_to_float16)
        specs.append(LayerSpec(EmbeddingPipe, **self.word_embedings_params))

        def transpose(x):  # [b, s, h] -> [s, b, h]
            if isinstance(x, (tuple, list)):
                return (F_.transpose01(x[0]), *x[1:])
            return F_.transpose01(x)
        specs.append(transpose)
        for layer_idx in range(num_layers):
            self.transformer_layer_params.update({"layer_number": layer_idx})
            specs.append(LayerSpec(ParallelTransformerLayerPipe, **self.transformer_layer_params))

        def undo(x):  # [s, b, h] -> [b, s, h]
            if isinstance(x, (tuple, list)):
                x = x[0]
            return F_.transpose01(x)
        specs.append(undo)
        specs.append(build_layer_norm(self.layer_norm_params, layer_spec=True))
        specs.append(LayerSpec(EmbedddingPipeNoTied, **self.lm_head_params))
        if self.fp32_logits:
            specs.append(float16_to_fp32)
        return specs


_LLAMA_MODELS = {
    "llama_7b": {"num_layers": 32, "hidden_size": 4096, "num_attention_heads": 32},
    "llama_13b": {"num_layers": 40, "hidden_size": 5120, "num_attention_heads": 40},
    "llama_20b": {"num_layers": 60, "hidden_size": 5120, "num_attention_heads": 40},
    "llama_65b": {"num_layers": 80, "hidden_size": 8192, "num_attention_heads": 64},
    "llama2_7b": {"num_layers": 32, "hidden_size": 4096, "intermediate_size": 11008, "num_attention_heads": 32,
                  "num_kv_attention_heads": 32},
    "llama2_13b": {"num_layers": 40, "hidden_size": 5120, "intermediate_size": 13824, "num_attention_heads": 40,
                   "num_kv_attention_heads": 40},
    "llama2_70b": {"num_layers": 80, "hidden_size": 8192, "intermediate_size": 28672, "num_attention_heads": 64,
                   "num_kv_attention_heads": 8},
    "codellama_7b": {"num_layers": 32, "hidden_size": 4096, "intermediate_size": 11008, "num_attention_heads": 32,
                     "num_kv_attention_heads": 32, "position_embedding_kwargs": {"base": 1.e6}},
    "codellama_13b": {"num_layers": 40, "hidden_size": 5120, "intermediate_size": 13824, "num_attention_heads": 40,
                      "num_kv_attention_heads": 40, "position_embedding_kwargs": {"base": 1.e6}},
    # `ffn_hidden_size` is not a key any config reads (it is dropped); ceil256(8h/3) happens to give 22016
    "codellama_34b": {"num_layers": 48, "hidden_size": 8192, "ffn_hidden_size": 22016, "num_attention_heads": 64,
                      "num_kv_attention_heads": 8, "position_embedding_kwargs": {"base": 1.e6}},
}


def check_keys_mapping(cfg_a, cfg_b):
    for key in cfg_a:
        if key in cfg_b:
            assert cfg_a[key] == cfg_b[key], "the value of key {} of two configs do not match".format(key)


def llama_custom(**cfg_model):
    cfg_model = update_model_cfg(cfg_model)
    return LlamaModelPipe(**cfg_model)


def _preset(name):
    def build(**cfg_model):
        preset = _LLAMA_MODELS[name]
        check_keys_mapping(preset, cfg_model)
        cfg_model.update(preset)
        return llama_custom(**cfg_model)
    build.__name__ = name
    return build


MODULE_ZOO_REGISTRY.register("llama_custom", llama_custom)
for _name in _LLAMA_MODELS:
    globals()[_name] = _preset(_name)
    MODULE_ZOO_REGISTRY.register(_name, globals()[_name])
