"""Writes tests/golden/bf16_floor_c2_widths.json: how far transformers' LlamaForCausalLM run in bf16 lands from its own
fp32 run at the widths of the headline workload (4 layers, hidden 4096, 32 heads of 128, FFN 11008, vocabulary 32000;
one sequence of 256 tokens), for the logits, the loss and every parameter gradient.  Numbers only: relative L2 distance,
cosine and largest error over largest reference magnitude per tensor.

The model is built from a local config object (nothing is downloaded); the weights are the seeded N(0, 0.02) bf16-exact
matrices of oracle.llama_oracle.init_weights (RMSNorm weights drawn around 1 so that their gradients carry information),
so the test that reads the fixture can rebuild them without transformers.  Both runs happen on the CPU.

Attention goes through transformers' "sdpa" implementation (torch's fused CPU kernel, which like the flash-attention seam of
the reference keeps scores and probabilities in fp32 inside the kernel).  The "eager" implementation stores the bf16-rounded
scores before the softmax, an error of up to 2^-9 |s| in the exponent, and lands several times farther from fp32; its logits
distance is recorded beside the other as `logits_eager_attention` for comparison and is not what the test checks.

Run from the repository root:  python tests/golden/make_bf16_floor_fixture.py      (about two minutes, 30 GB of memory)
"""
import json
import os
import sys

import torch
import torch.nn.functional as F

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
sys.path.insert(0, HERE)
import hf_llama_recipe as R  # noqa: E402

CFG = dict(num_layers=4, hidden_size=4096, num_attention_heads=32, num_kv_attention_heads=32, head_dim=128,
           intermediate_size=11008, vocab_size=32000, eps=1e-6, rope_base=10000.0)
SEQ, SEED = 256, 20250301


def make_weights():
    """The stack's fp32 weights, every value a bf16 number.  Kept here (not in the oracle) so that the recipe is part of
    the fixture: the test imports this function."""
    from oracle import llama_oracle as O
    W = O.init_weights(CFG, seed=SEED, round_to_bf16=True)
    g = torch.Generator().manual_seed(SEED + 1)
    for k in W:
        if W[k].dim() == 1:
            W[k] = (1.0 + 0.1 * torch.randn(W[k].shape, generator=g)).bfloat16().float()
    return W


def make_batch():
    g = torch.Generator().manual_seed(SEED + 2)
    tokens = torch.randint(0, CFG["vocab_size"], (1, SEQ), generator=g)
    labels = torch.randint(0, CFG["vocab_size"], (1, SEQ), generator=g)
    return tokens, labels


def distance(a, ref):
    """(relative L2, cosine, max |a - ref| / max |ref|) in fp64."""
    a, ref = a.detach().double().reshape(-1), ref.detach().double().reshape(-1)
    rn = ref.norm().item()
    return [(a - ref).norm().item() / rn, torch.dot(a, ref).item() / (a.norm().item() * rn),
            (a - ref).abs().max().item() / ref.abs().max().item()]


def to_hf_state_dict(W):
    L = CFG["num_layers"]
    sd = {"model.embed_tokens.weight": W["1.word_embeddings.weight"], "model.norm.weight": W["%d.weight" % (L + 4)],
          "lm_head.weight": W["%d.word_embeddings.weight" % (L + 5)]}
    for i in range(L):
        for name in R._LAYER_PARAMS:
            sd["model.layers.%d.%s" % (i, name)] = W["%d.%s" % (i + 3, name)]
    return sd


def from_hf_name(name):
    L = CFG["num_layers"]
    if name == "model.embed_tokens.weight":
        return "1.word_embeddings.weight"
    if name == "model.norm.weight":
        return "%d.weight" % (L + 4)
    if name == "lm_head.weight":
        return "%d.word_embeddings.weight" % (L + 5)
    _, _, i, rest = name.split(".", 3)
    return "%d.%s" % (int(i) + 3, rest)


def run(hf, tokens, labels):
    hf.zero_grad(set_to_none=True)
    logits = hf(input_ids=tokens).logits
    loss = F.cross_entropy(logits.float().reshape(-1, CFG["vocab_size"]), labels.reshape(-1))
    loss.backward()
    return logits.detach().float(), loss.item(), {from_hf_name(n): p.grad.detach().float().clone() for n, p in hf.named_parameters()}


def build(attn, W):
    from transformers import LlamaConfig, LlamaForCausalLM
    c = CFG
    hf_cfg = LlamaConfig(vocab_size=c["vocab_size"], hidden_size=c["hidden_size"], intermediate_size=c["intermediate_size"],
                         num_hidden_layers=c["num_layers"], num_attention_heads=c["num_attention_heads"],
                         num_key_value_heads=c["num_kv_attention_heads"], head_dim=c["head_dim"], rms_norm_eps=c["eps"],
                         rope_theta=c["rope_base"], max_position_embeddings=SEQ, tie_word_embeddings=False,
                         attention_bias=False, mlp_bias=False, hidden_act="silu", attn_implementation=attn)
    hf = LlamaForCausalLM(hf_cfg).float()
    missing, unexpected = hf.load_state_dict(to_hf_state_dict(W), strict=False)
    assert not unexpected and all("rotary" in m or "inv_freq" in m for m in missing), (missing, unexpected)
    return hf


def to_bf16(hf):
    """module.bfloat16() also rounds the rotary frequencies (a buffer), which no bf16 training path does -- with them in bf16
    the phase error grows with the position and the logits land 7 % from fp32 instead of 2.5 %.  They are kept in fp32, as
    when a bf16 checkpoint is loaded into a freshly built model; the cos / sin values are still rounded to bf16 per use."""
    inv_freq = hf.model.rotary_emb.inv_freq.clone()
    hf = hf.bfloat16()
    hf.model.rotary_emb.inv_freq = inv_freq
    return hf


def main():
    W = make_weights()
    tokens, labels = make_batch()
    hf = build("sdpa", W)
    l32, loss32, g32 = run(hf, tokens, labels)
    hf = to_bf16(hf)
    l16, loss16, g16 = run(hf, tokens, labels)
    del hf
    with torch.no_grad():
        eager16 = to_bf16(build("eager", W))(input_ids=tokens).logits.float()
    out = {"what": "transformers LlamaForCausalLM, bf16 run against its own fp32 run, CPU; [relative L2, cosine, max-rel]",
           "transformers": __import__("transformers").__version__, "torch": torch.__version__,
           "cfg": CFG, "seq": SEQ, "seed": SEED,
           "weights_abs_sum": sum(v.double().abs().sum().item() for v in W.values()),
           "loss_fp32": loss32, "loss_bf16": loss16,
           "logits_fp32_probe": [l32[0, i, j].item() for i, j in ((0, 0), (17, 4242), (255, 31999))],
           "logits": distance(l16, l32), "logits_eager_attention": distance(eager16, l32), "grads": {k: distance(g16[k], g32[k]) for k in sorted(g32)}}
    path = os.path.join(HERE, "bf16_floor_c2_widths.json")
    with open(path, "w") as fh:
        json.dump(out, fh, indent=1, sort_keys=True)
    print("wrote", path, "loss fp32 %.6f bf16 %.6f logits" % (loss32, loss16), out["logits"])


if __name__ == "__main__":
    main()
