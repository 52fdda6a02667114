"""Decoder layer, host side: same classes, constructor kwargs, forward signatures and state-dict keys as
the reference's llama/transformer.py, with every op routed to the HIP kernels.

  FlashAttention ................ transformer.py:65-143
  ParallelMLP ................... transformer.py:146-225
  ParallelAttention ............. transformer.py:228-597  (flash path only; the baddbmm/softmax/bmm
                                  branch :492-592 is the definition the CPU oracle restates)
  ParallelTransformerLayer[Pipe]  transformer.py:625-867

Differences that are deliberate and invisible in the results: activations stay in [s, b, h] from end
to end (the attention kernels take token strides, so the reference's `s b ... -> b s ...` copies at
:478/:491 do not exist); the residual add of :786 is fused into the RMSNorm that follows it; the
SiLU and the product with `up` (:222) are one kernel.
"""
import math

import torch

from . import dist_env
from . import functional as F_
from .layers import (ColumnParallelLinear, RowParallelLinear, GLU_ACTIVATIONS, build_layer_norm,
                     get_initializer_from_cfg, get_torch_dtype)
from .positional_embeddings import RotaryEmbedding, apply_rotary_pos_emb

_POSITION_TYPES = ("rotary", "absolute", "alibi", "flash", "dynamicntk")
_MASK_TYPES = ("causal", "padding", "prefix", "custom")


class FlashAttention(torch.nn.Module):
    """Causal softmax(q k^T * scale) v over packed documents (the flash_attn_varlen_* seam)."""

    def __init__(self, causal=False, softmax_scale=None, attention_dropout=0.0):
        super().__init__()
        self.softmax_scale = softmax_scale
        self.dropout_p = attention_dropout
        self.causal = causal

    def forward(self, q, k, v, key_padding_mask=None, cu_seqlens=None):
        """q [b, s, nq, d], k/v [b, s, nk, d] (any token strides) -> [b, s, nq, d]."""
        assert q.dtype in [torch.float16, torch.bfloat16]
        assert q.is_cuda
        out = self.forward_sb(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1), key_padding_mask, cu_seqlens)
        return out.transpose(0, 1)

    def forward_sb(self, q, k, v, key_padding_mask=None, cu_seqlens=None):
        """Same on [s, b, heads, d] tensors; returns contiguous [s, b, nq, d]."""
        if not self.causal:
            raise NotImplementedError("only causal attention is built")
        if self.training and self.dropout_p != 0.0:
            raise NotImplementedError("attention dropout is 0 in every llama config")
        if q.dtype != torch.bfloat16:
            raise TypeError("the HIP attention computes in bf16")
        if key_padding_mask is not None:  # :117-141: unpad, attend among the kept tokens of each row, pad back with zeros
            if tuple(key_padding_mask.shape) != (q.shape[1], q.shape[0]):
                raise ValueError("key_padding_mask must be [b, s]")
            return F_.flash_attention_unpadded(q, k, v, key_padding_mask.bool(), self.softmax_scale)
        if cu_seqlens is not None:
            cu_seqlens = cu_seqlens.view(-1).int()  # :103
        return F_.flash_attention(q, k, v, cu_seqlens, self.softmax_scale)


class ParallelMLP(torch.nn.Module):
    """down_proj(silu(gate_proj(x)) * up_proj(x)); returns (output, output_bias)."""

    def __init__(self, init_method, output_layer_init_method, hidden_size=1024, intermediate_size=4096,
                 use_cpu_initialization=False, params_dtype=torch.half, bias_gelu_fusion=False, glu_activation=None,
                 use_openai_gelu=False, onnx_safe=False, sync_tp_duplicated_parameters=True, sequence_parallel=False):
        super().__init__()
        self.sequence_parallel = sequence_parallel
        common = dict(gather_output=False, init_method=init_method, skip_bias_add=True, bias=False,
                      use_cpu_initialization=use_cpu_initialization, params_dtype=params_dtype,
                      sequence_parallel=sequence_parallel)
        self.gate_proj = ColumnParallelLinear(hidden_size, intermediate_size, **common)
        self.up_proj = ColumnParallelLinear(hidden_size, intermediate_size, **common)
        if glu_activation not in GLU_ACTIVATIONS:
            raise NotImplementedError("glu_activation=%r: the llama step uses 'silu' (default_cfg.py:163)" % (glu_activation,))
        self.activation_func = GLU_ACTIVATIONS[glu_activation]
        self.down_proj = RowParallelLinear(intermediate_size, hidden_size, input_is_parallel=True,
                                           init_method=output_layer_init_method, skip_bias_add=True, bias=False,
                                           use_cpu_initialization=use_cpu_initialization, params_dtype=params_dtype,
                                           sync_tp_duplicated_parameters=sync_tp_duplicated_parameters,
                                           sequence_parallel=sequence_parallel)

    def forward(self, hidden_states):
        # gate_proj and up_proj share their input: one fan-out op (input gradient accumulated in the GEMM)
        h1, h2 = F_.fan_out_linear(hidden_states, self.gate_proj.weight, self.up_proj.weight)
        h1 = self.activation_func.fused_mul(h1, h2)
        return self.down_proj(h1)


class ParallelAttention(torch.nn.Module):
    """Self-attention: q/k/v (or packed wqkv) projections, rotary, causal flash attention, o_proj."""

    def __init__(self, init_method, output_layer_init_method, layer_number, attention_type="self_attn",
                 attn_mask_type="padding", fp16=False, bf16=True, position_embedding_type=None,
                 position_embedding_kwargs=None, apply_query_key_layer_scaling=False, attention_softmax_in_fp32=False,
                 kv_channels=0, num_attention_heads=1, num_kv_attention_heads=1, hidden_size=2048,
                 masked_softmax_fusion=False, attention_dropout=0, params_dtype=torch.half, use_cpu_initialization=False,
                 sync_tp_duplicated_parameters=True, sequence_parallel=False, use_flash_attn=False, use_matmul=False,
                 qkv_pack=False, qkv_bias=False, o_bias=False):
        super().__init__()
        self.fp16, self.bf16 = fp16, bf16
        self.position_embedding_type = position_embedding_type
        # query-key layer scaling only rescales the non-flash branch and cancels exactly (:354-357)
        self.apply_query_key_layer_scaling = apply_query_key_layer_scaling
        self.layer_number = max(1, layer_number)
        assert attention_type in ("self_attn", None) or str(attention_type).endswith("self_attn"), \
            "Not implementented for cross-attention"
        self.attn_mask_type = attn_mask_type
        self.sequence_parallel = sequence_parallel
        if not use_flash_attn:
            raise NotImplementedError("only the flash-attention branch of ParallelAttention is built (use_flash_attn=True)")
        self.use_flash_attn = True
        assert attention_dropout == 0, "attention dropout is 0 in every llama config"
        projection_size = kv_channels * num_attention_heads
        projection_size_kv = kv_channels * num_kv_attention_heads
        world_size = dist_env.get_tensor_model_parallel_world_size()

        def partition(proj_size, num_heads):  # :287-298
            assert proj_size % world_size == 0, "{} is not divisible by {}".format(proj_size, world_size)
            assert proj_size % num_heads == 0, "{} is not divisible by {}".format(proj_size, num_heads)
            assert num_heads % world_size == 0, "{} is not divisible by {}".format(num_heads, world_size)
            return proj_size // world_size, proj_size // num_heads, num_heads // world_size

        (self.hidden_size_per_partition, self.hidden_size_per_attention_head,
         self.num_attention_heads_per_partition) = partition(projection_size, num_attention_heads)
        (self.hidden_size_kv_per_partition, self.hidden_size_per_kv_attention_head,
         self.num_kv_attention_heads_per_partition) = partition(projection_size_kv, num_kv_attention_heads)
        assert self.num_attention_heads_per_partition % self.num_kv_attention_heads_per_partition == 0

        self.qkv_pack = qkv_pack
        self.q_size = projection_size // world_size
        self.kv_size = projection_size_kv // world_size
        col = dict(gather_output=False, init_method=init_method, bias=qkv_bias, use_cpu_initialization=use_cpu_initialization,
                   params_dtype=params_dtype, sequence_parallel=sequence_parallel)
        if not qkv_pack:
            self.q_proj = ColumnParallelLinear(hidden_size, projection_size, **col)
            self.k_proj = ColumnParallelLinear(hidden_size, projection_size_kv, **col)
            self.v_proj = ColumnParallelLinear(hidden_size, projection_size_kv, **col)
        else:
            self.wqkv = ColumnParallelLinear(hidden_size, projection_size + 2 * projection_size_kv, **col)
        self.norm_factor = math.sqrt(self.hidden_size_per_attention_head)
        self.core_attention_flash = FlashAttention(causal=True, attention_dropout=attention_dropout)
        self.o_proj = RowParallelLinear(projection_size, hidden_size, input_is_parallel=True,
                                        init_method=output_layer_init_method, skip_bias_add=True, bias=o_bias,
                                        use_cpu_initialization=use_cpu_initialization, params_dtype=params_dtype,
                                        sync_tp_duplicated_parameters=sync_tp_duplicated_parameters,
                                        sequence_parallel=sequence_parallel)
        if position_embedding_type == "rotary":
            self.rotary_emb = RotaryEmbedding(self.hidden_size_per_attention_head, precision=params_dtype,
                                              **(position_embedding_kwargs or {}))
        else:
            raise NotImplementedError("position_embedding_type=%r: the llama step uses 'rotary' (default_cfg.py:22)"
                                      % (position_embedding_type,))

    def forward(self, hidden_states, attention_mask, cu_seqlens=None, position_ids=None, layer_past=None,
                get_key_value=False, alibi=None):
        # hidden_states [s, b, h]
        if layer_past is not None or get_key_value:
            raise NotImplementedError("KV-cache inference is outside the training step")
        if not self.qkv_pack and self.q_proj.bias is None:
            query_layer, key_layer, value_layer = F_.fan_out_linear(hidden_states, self.q_proj.weight, self.k_proj.weight,
                                                                    self.v_proj.weight)
        elif not self.qkv_pack:
            query_layer, _ = self.q_proj(hidden_states)
            key_layer, _ = self.k_proj(hidden_states)
            value_layer, _ = self.v_proj(hidden_states)
        else:
            qkv_layer, _ = self.wqkv(hidden_states)  # q | k | v along the last dim (:427-429)
            query_layer = qkv_layer[..., :self.q_size]
            key_layer = qkv_layer[..., self.q_size:(self.q_size + self.kv_size)]
            value_layer = qkv_layer[..., (self.q_size + self.kv_size):]
        sq, bs = query_layer.shape[0], query_layer.shape[1]
        nq, nk = self.num_attention_heads_per_partition, self.num_kv_attention_heads_per_partition
        d = self.hidden_size_per_attention_head
        q = query_layer.view(sq, bs, nq, d) if not self.qkv_pack else query_layer.unflatten(-1, (nq, d))
        k = key_layer.view(sq, bs, nk, d) if not self.qkv_pack else key_layer.unflatten(-1, (nk, d))
        v = value_layer.view(sq, bs, nk, d) if not self.qkv_pack else value_layer.unflatten(-1, (nk, d))
        cos, sin = self.rotary_emb.tables(sq, q.device)
        q, k = apply_rotary_pos_emb(q, k, cos, sin, position_ids)
        if attention_mask is None or cu_seqlens is not None:  # :480-488: document boundaries replace the padding mask
            qk_mask = None
        elif attention_mask.dim() == 2:
            qk_mask = attention_mask
        else:
            qk_mask = ~attention_mask[:, 0, :, 0]
        with dist_env.get_cuda_rng_tracker().fork():
            context_layer = self.core_attention_flash.forward_sb(q, k, v, qk_mask, cu_seqlens)
        context_layer = context_layer.view(sq, bs, nq * d)  # 's b (h d)', already contiguous
        return self.o_proj(context_layer)


class ParallelTransformerLayer(torch.nn.Module):
    """Pre-norm residual block: x1 = x + attn(ln1(x)); y = x1 + mlp(ln2(x1))."""

    def __init__(self, layer_number, layer_type="encoder", self_attn_mask_type="padding", position_embedding_type=None,
                 position_embedding_kwargs=None, params_dtype="half", layer_norm=None, fp16=False, bf16=True,
                 fp32_residual_connection=False, apply_residual_connection_post_layernorm=False,
                 apply_query_key_layer_scaling=False, attention_softmax_in_fp32=False, kv_channels=0, num_attention_heads=0,
                 num_kv_attention_heads=0, hidden_size=2048, masked_softmax_fusion=False, attention_dropout=0,
                 use_cpu_initialization=None, bias_gelu_fusion=False, glu_activation=None, use_openai_gelu=False,
                 onnx_safe=None, sync_tp_duplicated_parameters=False, hidden_dropout=0, bias_dropout_fusion=False,
                 intermediate_size=4096, seq_length=1024, micro_batch_size=1, sequence_parallel=False, use_flash_attn=False,
                 initializer=None, output_initializer=None, use_matmul=False, qkv_pack=False, attention_qkv_bias=False,
                 attention_o_bias=False):
        super().__init__()
        assert layer_type in ("encoder", "decoder")
        assert position_embedding_type in _POSITION_TYPES and self_attn_mask_type in _MASK_TYPES
        self.layer_number = layer_number
        self.layer_type = layer_type
        params_dtype = get_torch_dtype(params_dtype)
        self.apply_residual_connection_post_layernorm = apply_residual_connection_post_layernorm
        self.bf16 = bf16
        if fp32_residual_connection:
            raise NotImplementedError("fp32 residual stream is not built (default_cfg.py:32 default is False)")
        self.fp32_residual_connection = False
        self.sequence_parallel = sequence_parallel
        assert hidden_dropout == 0, "hidden dropout is 0 in every llama config (default_cfg.py:21)"
        self.hidden_dropout = hidden_dropout
        self.bias_dropout_fusion = bias_dropout_fusion
        self.input_layernorm = build_layer_norm(layer_norm)
        self.self_attn = ParallelAttention(
            init_method=get_initializer_from_cfg(initializer),
            output_layer_init_method=get_initializer_from_cfg(output_initializer), layer_number=layer_number,
            attention_type="self_attn", attn_mask_type=self_attn_mask_type, fp16=fp16, bf16=bf16,
            position_embedding_type=position_embedding_type, position_embedding_kwargs=position_embedding_kwargs,
            apply_query_key_layer_scaling=apply_query_key_layer_scaling, attention_softmax_in_fp32=attention_softmax_in_fp32,
            kv_channels=kv_channels, num_attention_heads=num_attention_heads, num_kv_attention_heads=num_kv_attention_heads,
            hidden_size=hidden_size, masked_softmax_fusion=masked_softmax_fusion, attention_dropout=attention_dropout,
            params_dtype=params_dtype, use_cpu_initialization=use_cpu_initialization,
            sync_tp_duplicated_parameters=sync_tp_duplicated_parameters, sequence_parallel=sequence_parallel,
            use_flash_attn=use_flash_attn, use_matmul=use_matmul, qkv_pack=qkv_pack, qkv_bias=attention_qkv_bias,
            o_bias=attention_o_bias)
        self.post_attention_layernorm = build_layer_norm(layer_norm)
        self.mlp = ParallelMLP(
            init_method=get_initializer_from_cfg(initializer),
            output_layer_init_method=get_initializer_from_cfg(output_initializer), hidden_size=hidden_size,
            intermediate_size=intermediate_size, use_cpu_initialization=use_cpu_initialization, params_dtype=params_dtype,
            bias_gelu_fusion=bias_gelu_fusion, glu_activation=glu_activation, use_openai_gelu=use_openai_gelu,
            onnx_safe=onnx_safe, sync_tp_duplicated_parameters=sync_tp_duplicated_parameters,
            sequence_parallel=sequence_parallel)
        self.alibi = None

    def forward(self, hidden_states, attention_mask, cu_seqlens=None, position_ids=None, layer_past=None,
                get_key_value=False):
        hidden_states, layernorm_output = self.input_layernorm.forward_keep_input(hidden_states)
        attention_output, attention_bias = self.self_attn(layernorm_output, attention_mask, cu_seqlens, position_ids,
                                                          layer_past=layer_past, get_key_value=get_key_value, alibi=self.alibi)
        if attention_bias is not None:
            attention_output = F_.bias_add(attention_output, attention_bias)
        if self.apply_residual_connection_post_layernorm:
            layernorm_input = F_.add(attention_output, layernorm_output)
            layernorm_output = self.post_attention_layernorm(layernorm_input)
            residual = layernorm_output
        else:
            # residual add (:786) + post-attention RMSNorm (:787) in one kernel
            layernorm_input, layernorm_output = self.post_attention_layernorm.forward_with_residual(attention_output,
                                                                                                     hidden_states)
            residual = layernorm_input
        mlp_output, _ = self.mlp(layernorm_output)
        return F_.add(mlp_output, residual)  # :797


class ParallelTransformerLayerPipe(ParallelTransformerLayer):
    """Threads (hidden, mask[, cu_seqlens, position_ids]) through the spec list unchanged (:854-867)."""

    def forward(self, inputs, **kwargs):
        assert torch.is_tensor(inputs) or isinstance(inputs, tuple)
        if torch.is_tensor(inputs) or len(inputs) == 1:
            hidden_states = inputs if torch.is_tensor(inputs) else inputs[0]
            return super().forward(hidden_states, None, **kwargs)
        if len(inputs) == 2:
            return super().forward(*inputs, **kwargs), inputs[1]
        if len(inputs) == 4:
            hidden_states, attention_mask, cu_seqlens, position_ids = inputs
            return super().forward(hidden_states, attention_mask, cu_seqlens, position_ids, **kwargs), attention_mask, \
                cu_seqlens, position_ids
        raise RuntimeError("Received more inputs than understood.")
