"""Inputs of the golden fixture `hf_llama_tiny.npz`: a tiny GQA llama (2 layers, h 256, 4 query / 2 kv heads of 64,
f 688, V 512) with seeded, bf16-exact weights and one seeded batch [2, 64] with a few ignored labels.

Shared by the script that writes the fixture (expected values come from transformers' LlamaForCausalLM, an independent
implementation) and by the tests that check the CPU oracle and the HIP path against it.  Parameter names are those of the
layer stack (llama/utils.py:158-210 of the reference: 1 = embedding, 3.. = decoder layers, L+4 = final norm, L+5 = head).
"""
import torch

CFG = dict(num_layers=2, hidden_size=256, num_attention_heads=4, num_kv_attention_heads=2, head_dim=64,
           intermediate_size=688, vocab_size=512, eps=1e-6, rope_base=10000.0)
SEQ, BATCH, SEED = 64, 2, 20240607
IGNORE_INDEX = -100

_LAYER_PARAMS = ("input_layernorm.weight", "self_attn.q_proj.weight", "self_attn.k_proj.weight", "self_attn.v_proj.weight",
                 "self_attn.o_proj.weight", "post_attention_layernorm.weight", "mlp.gate_proj.weight", "mlp.up_proj.weight",
                 "mlp.down_proj.weight")


def make_weights():
    """fp32 tensors whose values are exactly representable in bf16."""
    g = torch.Generator().manual_seed(SEED)
    c = CFG
    h, d, f, V = c["hidden_size"], c["head_dim"], c["intermediate_size"], c["vocab_size"]
    nq, nk, L = c["num_attention_heads"], c["num_kv_attention_heads"], c["num_layers"]
    shapes = {"input_layernorm.weight": (h,), "self_attn.q_proj.weight": (nq * d, h), "self_attn.k_proj.weight": (nk * d, h),
              "self_attn.v_proj.weight": (nk * d, h), "self_attn.o_proj.weight": (h, nq * d),
              "post_attention_layernorm.weight": (h,), "mlp.gate_proj.weight": (f, h), "mlp.up_proj.weight": (f, h),
              "mlp.down_proj.weight": (h, f)}

    def draw(shape):
        if len(shape) == 1:  # norm weights around 1 so that their gradients matter
            w = 1.0 + 0.1 * torch.randn(shape, generator=g)
        else:
            w = 0.05 * torch.randn(shape, generator=g)
        return w.bfloat16().float()

    W = {"1.word_embeddings.weight": draw((V, h))}
    for i in range(L):
        for name in _LAYER_PARAMS:
            W["%d.%s" % (i + 3, name)] = draw(shapes[name])
    W["%d.weight" % (L + 4)] = draw((h,))
    W["%d.word_embeddings.weight" % (L + 5)] = draw((V, h))
    return W


def make_batch():
    g = torch.Generator().manual_seed(SEED + 1)
    tokens = torch.randint(0, CFG["vocab_size"], (BATCH, SEQ), generator=g)
    labels = torch.randint(0, CFG["vocab_size"], (BATCH, SEQ), generator=g)
    labels[torch.rand(BATCH, SEQ, generator=g) < 0.1] = IGNORE_INDEX
    return tokens, labels


def to_hf_state_dict(W):
    L = CFG["num_layers"]
    sd = {"model.embed_tokens.weight": W["1.word_embeddings.weight"], "model.norm.weight": W["%d.weight" % (L + 4)],
          "lm_head.weight": W["%d.word_embeddings.weight" % (L + 5)]}
    for i in range(L):
        for name in _LAYER_PARAMS:
            sd["model.layers.%d.%s" % (i, name)] = W["%d.%s" % (i + 3, name)]
    return sd


def from_hf_name(name):
    """HF parameter name -> stack name."""
    L = CFG["num_layers"]
    if name == "model.embed_tokens.weight":
        return "1.word_embeddings.weight"
    if name == "model.norm.weight":
        return "%d.weight" % (L + 4)
    if name == "lm_head.weight":
        return "%d.word_embeddings.weight" % (L + 5)
    _, _, i, rest = name.split(".", 3)
    return "%d.%s" % (int(i) + 3, rest)


def grad_block(t):
    """The slice of a gradient the fixture keeps: leading 8 x 8 block (first 32 entries of a vector)."""
    return t[:8, :8] if t.dim() == 2 else t[:32]
