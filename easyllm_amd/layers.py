"""Host-side mirror of the reference's base layers, backed by the HIP kernels:

  RMSNorm / build_layer_norm ....... base_modules/layers/fused_layer_norm.py:20-71, 143-155
  ColumnParallelLinear ............. base_modules/layers/column_parallel_linear.py:158-266
  RowParallelLinear ................ base_modules/layers/row_parallel_linear.py:13-132
  VocabParallelEmbedding ........... base_modules/layers/vocab_parallel_emb.py:30-137
  GLU_ACTIVATIONS['silu'] .......... base_modules/layers/glu_activations.py:56-78
  initializers / dtype helpers ..... base_modules/utils.py:11-96, llm/utils/model/initializer.py:41-48

Same class names, constructor kwargs, forward signatures/returns and state-dict keys; TP size is 1.
"""
import math
import numbers

import torch
from torch.nn.parameter import Parameter

from . import dist_env
from . import functional as F_


def _param_device():
    return torch.device("cuda", torch.cuda.current_device()) if torch.cuda.is_available() else torch.device("cpu")


# ---- initializers (base_modules/utils.py:11-38) ---------------------------------------------
def init_method_normal(sigma):
    def init_(tensor):
        return torch.nn.init.normal_(tensor, mean=0.0, std=sigma)
    return init_


def scaled_init_method_normal(sigma, num_layers):
    std = sigma / math.sqrt(2.0 * num_layers)

    def init_(tensor):
        return torch.nn.init.normal_(tensor, mean=0.0, std=std)
    return init_


def get_initializer_from_cfg(cfg):
    if cfg is None:
        return init_method_normal(sigma=0.02)
    if cfg["type"] == "normal":
        return init_method_normal(**cfg["kwargs"])
    if cfg["type"] == "scaled_normal":
        return scaled_init_method_normal(**cfg["kwargs"])
    raise NotImplementedError(cfg["type"])


_DTYPES = {"half": torch.half, "float": torch.float, "float16": torch.float16, "float32": torch.float32,
           "bfloat16": torch.bfloat16}


def get_torch_dtype(v):
    return v if isinstance(v, torch.dtype) else _DTYPES[v]


def check_torch_dtype(params_dtype, fp16=False, bf16=False):  # base_modules/utils.py:40-59
    if params_dtype is None:
        assert not (fp16 and bf16)
        return "half" if fp16 else ("bfloat16" if bf16 else "float")
    assert params_dtype in _DTYPES
    if params_dtype in ("half", "float16"):
        assert fp16 and not bf16
    elif params_dtype == "bfloat16":
        assert bf16 and not fp16
    else:
        assert not bf16 and not fp16
    return params_dtype


def set_tensor_model_parallel_attributes(tensor, is_parallel, dim, stride):  # initializer.py:41-48
    for attribute in ("tensor_model_parallel", "partition_dim", "partition_stride"):
        assert not hasattr(tensor, attribute)
    tensor.tensor_model_parallel = is_parallel
    tensor.partition_dim = dim
    tensor.partition_stride = stride


def _require_bf16(t, what):
    if t.dtype != torch.bfloat16:
        raise TypeError("%s: the HIP path computes in bf16 (got %s); build the model with bf16=True" % (what, t.dtype))


# ---- RMSNorm ----------------------------------------------------------------------------------
class RMSNorm(torch.nn.Module):
    def __init__(self, sync_tp_duplicated_parameters, normalized_shape, eps=1e-6, use_flash_attn=False, bf16=True,
                 hf_mode=False, sequence_parallel=False, params_dtype=None):
        super().__init__()
        if isinstance(normalized_shape, numbers.Integral):
            normalized_shape = (normalized_shape,)
        self.normalized_shape = torch.Size(normalized_shape)
        self.eps = eps
        self.use_flash_attn = use_flash_attn
        self.bf16 = bf16
        self.hf_mode = hf_mode
        dtype = get_torch_dtype(params_dtype) if params_dtype is not None else (torch.bfloat16 if bf16 else torch.float32)
        self.weight = Parameter(torch.ones(*normalized_shape, dtype=dtype, device=_param_device()))
        self.layernorm_tp_auto_sync = sync_tp_duplicated_parameters
        self.sequence_parallel = sequence_parallel

    def reset_parameters(self):
        torch.nn.init.ones_(self.weight)

    def forward(self, input):
        if self.layernorm_tp_auto_sync or self.sequence_parallel:
            dist_env.sync_tp_duplicated_parameter(self.weight)  # AVG over a 1-rank group (:51-54)
        _require_bf16(input, "RMSNorm")
        return F_.rmsnorm(input, self.weight, self.eps)

    def forward_keep_input(self, x):
        """(x, norm(x)): x is returned as the residual branch so that its gradient is fused into the norm's backward."""
        if self.layernorm_tp_auto_sync or self.sequence_parallel:
            dist_env.sync_tp_duplicated_parameter(self.weight)
        _require_bf16(x, "RMSNorm")
        return F_.rmsnorm_pass(x, self.weight, self.eps)

    def forward_with_residual(self, x, residual):
        """(x + residual, norm(x + residual)) in one kernel -- transformer.py:786-787 fused."""
        if self.layernorm_tp_auto_sync or self.sequence_parallel:
            dist_env.sync_tp_duplicated_parameter(self.weight)
        _require_bf16(x, "RMSNorm")
        return F_.add_rmsnorm(x, residual, self.weight, self.eps)


class LayerSpec(object):
    """Deferred constructor, the shape of deepspeed.pipe.LayerSpec used by llama/llama.py:142-190."""

    def __init__(self, typename, *module_args, **module_kwargs):
        self.typename = typename
        self.module_args = module_args
        self.module_kwargs = module_kwargs

    def build(self):
        return self.typename(*self.module_args, **self.module_kwargs)


def build_layer_norm(cfg_ln, layer_spec=False):
    if cfg_ln["type"] == "rms_norm":
        if layer_spec:
            return LayerSpec(RMSNorm, **cfg_ln["kwargs"])
        return RMSNorm(**cfg_ln["kwargs"])
    # 'mixed_fused_norm' (LayerNorm with bias) is never selected by the llama configs
    raise NotImplementedError(cfg_ln["type"])


# ---- linears ----------------------------------------------------------------------------------
class ColumnParallelLinear(torch.nn.Module):
    """Y = X A^T (+ b); weight [output_size, input_size]; returns (output, bias_if_skip_bias_add)."""

    def __init__(self, input_size, output_size, bias=True, gather_output=True, init_method=torch.nn.init.xavier_normal_,
                 stride=1, keep_master_weight_for_test=False, skip_bias_add=False, use_cpu_initialization=False,
                 params_dtype=torch.half, sequence_parallel=False):
        super().__init__()
        self.input_size, self.output_size = input_size, output_size
        self.use_bias = bias
        self.gather_output = gather_output
        self.init_method = init_method
        self.stride = stride
        self.params_dtype = params_dtype
        world_size = dist_env.get_tensor_model_parallel_world_size()
        assert output_size % world_size == 0, "{} is not divisible by {}".format(output_size, world_size)
        self.output_size_per_partition = output_size // world_size
        self.skip_bias_add = skip_bias_add
        dev = torch.device("cpu") if use_cpu_initialization else _param_device()
        self.weight = Parameter(torch.empty(self.output_size_per_partition, input_size, device=dev, dtype=params_dtype))
        set_tensor_model_parallel_attributes(self.weight, True, 0, stride)
        with torch.no_grad():
            init_method(self.weight)
        if bias:
            self.bias = Parameter(torch.zeros(self.output_size_per_partition, device=dev, dtype=params_dtype))
            set_tensor_model_parallel_attributes(self.bias, True, 0, stride)
        else:
            self.register_parameter("bias", None)
        self.sequence_parallel = sequence_parallel

    def forward(self, input_):
        _require_bf16(input_, "ColumnParallelLinear")
        input_parallel = input_ if self.sequence_parallel else dist_env.copy_to_tensor_model_parallel_region(input_)
        output = F_.linear(input_parallel, self.weight)
        if self.bias is not None and not self.skip_bias_add:
            output = F_.bias_add(output, self.bias)
        if self.gather_output:
            assert not self.sequence_parallel
            output = dist_env.gather_from_tensor_model_parallel_region(output)
        return output, (self.bias if self.skip_bias_add else None)


class RowParallelLinear(torch.nn.Module):
    """Y = X A^T (+ b) with A split along its input dimension (whole at TP=1)."""

    def __init__(self, input_size, output_size, bias=True, input_is_parallel=False, init_method=torch.nn.init.xavier_normal_,
                 stride=1, keep_master_weight_for_test=False, skip_bias_add=False, use_cpu_initialization=False,
                 params_dtype=torch.half, sync_tp_duplicated_parameters=False, sequence_parallel=False):
        super().__init__()
        self.input_size, self.output_size = input_size, output_size
        self.use_bias = bias
        self.input_is_parallel = input_is_parallel
        self.init_method = init_method
        self.stride = stride
        self.params_dtype = params_dtype
        world_size = dist_env.get_tensor_model_parallel_world_size()
        assert input_size % world_size == 0, "{} is not divisible by {}".format(input_size, world_size)
        self.input_size_per_partition = input_size // world_size
        self.skip_bias_add = skip_bias_add
        self.sequence_parallel = sequence_parallel
        dev = torch.device("cpu") if use_cpu_initialization else _param_device()
        self.weight = Parameter(torch.empty(output_size, self.input_size_per_partition, device=dev, dtype=params_dtype))
        set_tensor_model_parallel_attributes(self.weight, True, 1, stride)
        with torch.no_grad():
            init_method(self.weight)
        if bias:
            self.bias = Parameter(torch.zeros(output_size, device=dev, dtype=params_dtype))
        else:
            self.register_parameter("bias", None)
        self.bias_tp_auto_sync = sync_tp_duplicated_parameters

    def forward(self, input_):
        _require_bf16(input_, "RowParallelLinear")
        if not self.input_is_parallel:
            assert not self.sequence_parallel
            input_ = dist_env.scatter_to_tensor_model_parallel_region(input_)
        output_ = dist_env.reduce_from_tensor_model_parallel_region(F_.linear(input_, self.weight))
        if self.bias_tp_auto_sync and self.bias is not None:
            dist_env.sync_tp_duplicated_parameter(self.bias)
        if not self.skip_bias_add:
            output = F_.bias_add(output_, self.bias) if self.bias is not None else output_
            return output, None
        return output_, self.bias


# ---- embedding --------------------------------------------------------------------------------
class VocabParallelEmbedding(torch.nn.Module):
    def __init__(self, num_embeddings, embedding_dim, init_method=torch.nn.init.xavier_normal_, use_bnb_optimizer=False,
                 use_cpu_initialization=False, params_dtype=None):
        super().__init__()
        self.num_embeddings = num_embeddings
        self.embedding_dim = embedding_dim
        self.init_method = init_method
        self.padding_idx = None
        self.tensor_model_parallel_size = dist_env.get_tensor_model_parallel_world_size()
        self.vocab_start_index, self.vocab_end_index = 0, num_embeddings
        self.num_embeddings_per_partition = num_embeddings
        self.params_dtype = params_dtype
        if use_bnb_optimizer:
            raise NotImplementedError("bitsandbytes embeddings are outside the decoder-layer step")
        dev = torch.device("cpu") if use_cpu_initialization else _param_device()
        self.weight = Parameter(torch.empty(num_embeddings, embedding_dim, device=dev, dtype=params_dtype))
        set_tensor_model_parallel_attributes(self.weight, True, 0, 1)
        with torch.no_grad():
            init_method(self.weight)

    def forward(self, input_):
        # the range check of :107-109 happens inside the gather kernel (flag -> ValueError)
        return dist_env.reduce_from_tensor_model_parallel_region(F_.embedding(input_, self.weight))


# ---- GLU activations --------------------------------------------------------------------------
class _SiLUGate(object):
    """`GLU_ACTIVATIONS['silu']` of the reference is silu(gate); the product with `up` follows in
    ParallelMLP.forward (transformer.py:222).  Here both run in one kernel via `fused_mul`."""

    @staticmethod
    def fused_mul(gate, up):
        return F_.swiglu(gate, up)


GLU_ACTIVATIONS = {"silu": _SiLUGate}
