"""The five synthetic workloads of the benchmark (shapes, seeds, input recipes) and the algorithmic
FLOP count of one fwd+bwd step (causal attention = lower triangle only; recompute not counted)."""
import numpy as np
import torch

from . import data

WORKLOADS = {
    "C1": dict(desc="tiny llama (L2 h256 4x64 MHA f688 V32000 s512 b2)", num_layers=2, hidden_size=256,
               num_attention_heads=4, num_kv_attention_heads=4, intermediate_size=688, vocab_size=32000, seq=512, batch=2,
               seed=1001),
    "C2": dict(desc="Llama-2-7B-shaped stack (L4 h4096 32x128 MHA f11008 V32000 s4096 b1)", num_layers=4, hidden_size=4096,
               num_attention_heads=32, num_kv_attention_heads=32, intermediate_size=11008, vocab_size=32000, seq=4096,
               batch=1, seed=1002),
    "C3": dict(desc="Llama-2-70B-shaped GQA stack (L2 h8192 64q/8kv x128 f28672 V32000 s4096 b1)", num_layers=2,
               hidden_size=8192, num_attention_heads=64, num_kv_attention_heads=8, intermediate_size=28672, vocab_size=32000,
               seq=4096, batch=1, seed=1003),
    "C4": dict(desc="Qwen-14B-shaped large-vocab stack (L2 h5120 40x128 f13696 V152064 s2048 b2, 10% labels ignored)",
               num_layers=2, hidden_size=5120, num_attention_heads=40, num_kv_attention_heads=40, intermediate_size=13696,
               vocab_size=152064, seq=2048, batch=2, seed=1004, ignore_frac=0.1),
    "C5": dict(desc="packed 16384-token batch on the 7B shape (L8, docs log-uniform [64,4096], dynamic checkpoint k=4)",
               num_layers=8, hidden_size=4096, num_attention_heads=32, num_kv_attention_heads=32, intermediate_size=11008,
               vocab_size=32000, seq=16384, batch=1, seed=1005, packed=(64, 4096),
               dynamic_checkpoint={"enabled": True, "size_map": {4096: 0, 8192: 2, 16384: 4, 32768: 8}}),
}


def model_kwargs(w, **overrides):
    """kwargs for MODULE_ZOO_REGISTRY.build({'type': 'llama_custom', 'kwargs': ...})."""
    kw = dict(num_layers=w["num_layers"], hidden_size=w["hidden_size"], num_attention_heads=w["num_attention_heads"],
              num_kv_attention_heads=w["num_kv_attention_heads"], intermediate_size=w["intermediate_size"],
              vocab_size=w["vocab_size"], seq_length=w["seq"], micro_batch_size=w["batch"], bf16=True,
              checkpoint_activations="dynamic_checkpoint" in w, dynamic_checkpoint=w.get("dynamic_checkpoint"),
              fp32_logits=False)
    kw.update(overrides)
    return kw


def make_inputs(w, device="cpu"):
    """Seeded token ids / labels (uniform over the vocab) in the reference's batch tuple layout."""
    g = torch.Generator().manual_seed(w["seed"])
    b, s, V = w["batch"], w["seq"], w["vocab_size"]
    tokens = torch.randint(0, V, (b, s), generator=g)
    labels = torch.randint(0, V, (b, s), generator=g)
    if w.get("ignore_frac"):
        labels[torch.rand(b, s, generator=g) < w["ignore_frac"]] = data.IGNORE_INDEX
    loss_mask = torch.ones(b, s, dtype=torch.float32)
    position_ids = torch.arange(s).unsqueeze(0).expand(b, s).contiguous()
    doc_lens = None
    if "packed" in w:
        lo, hi = w["packed"]
        doc_lens = data.packed_doc_lengths(b * s, lo, hi, w["seed"])
        cu = np.concatenate([[0], np.cumsum(doc_lens)])
        cu_seqlens = torch.tensor(cu, dtype=torch.int64)
        position_ids = torch.tensor([data.get_position_ids(cu.tolist())], dtype=torch.int64)
        inputs = (tokens.to(device), position_ids.to(device), None, cu_seqlens.to(device))
    else:
        inputs = (tokens.to(device), position_ids.to(device), None)
    return inputs, (labels.to(device), loss_mask.to(device)), doc_lens


def step_flops(w, doc_lens=None):
    b, s = w["batch"], w["seq"]
    T = b * s
    L, h, V = w["num_layers"], w["hidden_size"], w["vocab_size"]
    nq, nk, f = w["num_attention_heads"], w["num_kv_attention_heads"], w["intermediate_size"]
    d = h // nq
    proj = 2 * T * h * nq * d + 4 * T * h * nk * d + 2 * T * nq * d * h
    mlp = 6 * T * h * f
    lens = doc_lens if doc_lens is not None else [s] * b
    attn = 2 * nq * d * sum(l * l for l in lens)
    head = 2 * T * h * V
    return 3 * (L * (proj + mlp + attn) + head)
