"""Writes tests/golden/hf_llama_tiny.npz: loss, logits and parameter gradients of the tiny llama described in
hf_llama_recipe.py as computed in fp32 on the CPU by transformers' LlamaForCausalLM (built from a local config object;
nothing is downloaded).  Run from the repository root:  python tests/golden/make_hf_llama_fixture.py
"""
import os
import sys

import numpy as np
import torch
import torch.nn.functional as F

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import hf_llama_recipe as R  # noqa: E402


def main():
    from transformers import LlamaConfig, LlamaForCausalLM
    c = R.CFG
    hf_cfg = LlamaConfig(vocab_size=c["vocab_size"], hidden_size=c["hidden_size"], intermediate_size=c["intermediate_size"],
                         num_hidden_layers=c["num_layers"], num_attention_heads=c["num_attention_heads"],
                         num_key_value_heads=c["num_kv_attention_heads"], head_dim=c["head_dim"], rms_norm_eps=c["eps"],
                         rope_theta=c["rope_base"], max_position_embeddings=R.SEQ, tie_word_embeddings=False,
                         attention_bias=False, mlp_bias=False, hidden_act="silu", attn_implementation="eager")
    hf = LlamaForCausalLM(hf_cfg).float()
    W = R.make_weights()
    missing, unexpected = hf.load_state_dict(R.to_hf_state_dict(W), strict=False)
    assert not unexpected and all("rotary" in m or "inv_freq" in m for m in missing), (missing, unexpected)
    tokens, labels = R.make_batch()
    logits = hf(input_ids=tokens).logits  # [b, s, V] fp32
    # mean over the labels that are not ignored (llama/losses.py:53-55 of the reference with loss_mask == 1)
    loss = F.cross_entropy(logits.reshape(-1, c["vocab_size"]), labels.reshape(-1), ignore_index=R.IGNORE_INDEX)
    loss.backward()
    out = {"tokens": tokens.numpy(), "labels": labels.numpy(), "loss": np.float64(loss.item()),
           "logits_slice": logits.detach()[:, ::4, ::8].numpy().copy(),
           "weights_abs_sum": np.float64(sum(v.double().abs().sum().item() for v in W.values()))}
    for name, p in hf.named_parameters():
        key = R.from_hf_name(name)
        out["gnorm/" + key] = np.float64(p.grad.double().norm().item())
        out["gblock/" + key] = R.grad_block(p.grad).numpy().copy()
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "hf_llama_tiny.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes; loss", loss.item())


if __name__ == "__main__":
    main()
