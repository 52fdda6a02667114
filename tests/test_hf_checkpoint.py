"""HF-format checkpoint key maps, tensor-parallel slicing and the directory loader (CPU), plus one GPU end-to-end check:
a transformers LlamaForCausalLM saved to safetensors, loaded into the stack, must give the same logits."""
import os

import pytest
import torch

from easyllm_amd import hf_checkpoint as H


class _FakeModel:
    def __init__(self, num_layers, hidden, nq, nk):
        self.model_kwargs = {"num_layers": num_layers}
        self.transformer_layer_params = {"hidden_size": hidden, "num_attention_heads": nq, "num_kv_attention_heads": nk}


def _hf_llama_state(L, h, nq, nk, f, V, bias=False):
    g = torch.Generator().manual_seed(3)
    d = h // nq
    sd = {"model.embed_tokens.weight": torch.randn(V, h, generator=g), "model.norm.weight": torch.randn(h, generator=g),
          "lm_head.weight": torch.randn(V, h, generator=g)}
    for i in range(L):
        p = "model.layers.%d." % i
        sd[p + "self_attn.q_proj.weight"] = torch.randn(nq * d, h, generator=g)
        sd[p + "self_attn.k_proj.weight"] = torch.randn(nk * d, h, generator=g)
        sd[p + "self_attn.v_proj.weight"] = torch.randn(nk * d, h, generator=g)
        sd[p + "self_attn.o_proj.weight"] = torch.randn(h, nq * d, generator=g)
        if bias:
            for n, rows in (("q", nq * d), ("k", nk * d), ("v", nk * d)):
                sd[p + "self_attn.%s_proj.bias" % n] = torch.randn(rows, generator=g)
        sd[p + "mlp.gate_proj.weight"] = torch.randn(f, h, generator=g)
        sd[p + "mlp.up_proj.weight"] = torch.randn(f, h, generator=g)
        sd[p + "mlp.down_proj.weight"] = torch.randn(h, f, generator=g)
        sd[p + "input_layernorm.weight"] = torch.randn(h, generator=g)
        sd[p + "post_attention_layernorm.weight"] = torch.randn(h, generator=g)
        sd[p + "self_attn.rotary_emb.inv_freq"] = torch.randn(d // 2, generator=g)  # old checkpoints carry it; ignored
    return sd


def test_llama_key_map_round_trip_and_pack():
    L, h, nq, nk, f, V = 2, 16, 4, 2, 24, 32
    sd = _hf_llama_state(L, h, nq, nk, f, V, bias=True)
    m = _FakeModel(L, h, nq, nk)
    conv = H.hf_to_megatron_llama(sd, m)
    assert conv["1.word_embeddings.weight"] is sd["model.embed_tokens.weight"]
    assert conv["%d.weight" % (L + 4)] is sd["model.norm.weight"] and conv["%d.word_embeddings.weight" % (L + 5)] is sd["lm_head.weight"]
    assert conv["4.self_attn.k_proj.bias"] is sd["model.layers.1.self_attn.k_proj.bias"]
    assert conv["3.mlp.down_proj.weight"] is sd["model.layers.0.mlp.down_proj.weight"]
    assert len(conv) == 3 + L * 12 and not any("inv_freq" in k or "rotary" in k for k in conv)
    back = H.megatron_to_hf_llama(conv, L)
    assert set(back) == {k for k in sd if "rotary" not in k} and all(back[k] is sd[k] for k in back)
    packed = H.hf_to_megatron_llama(sd, m, pack=True)
    w = packed["3.self_attn.wqkv.weight"]
    assert isinstance(w, list) and w[0] is sd["model.layers.0.self_attn.q_proj.weight"] and w[2] is sd["model.layers.0.self_attn.v_proj.weight"]
    assert packed["4.self_attn.wqkv.bias"][1] is sd["model.layers.1.self_attn.k_proj.bias"]
    assert "3.self_attn.q_proj.weight" not in packed and "3.self_attn.k_proj.weight" not in packed
    del sd["model.layers.0.self_attn.v_proj.weight"]
    with pytest.raises(AssertionError):
        H.hf_to_megatron_llama(sd, m, pack=True)


def test_qwen_key_map_splits_c_attn_in_thirds():
    L, h = 1, 8
    m = _FakeModel(L, h, 2, 2)
    c_attn = torch.arange(3 * h * h, dtype=torch.float32).reshape(3 * h, h)
    c_bias = torch.arange(3 * h, dtype=torch.float32)
    sd = {"transformer.wte.weight": torch.zeros(4, h), "transformer.ln_f.weight": torch.ones(h), "lm_head.weight": torch.ones(4, h),
          "transformer.h.0.attn.c_attn.weight": c_attn, "transformer.h.0.attn.c_attn.bias": c_bias,
          "transformer.h.0.attn.c_proj.weight": torch.full((h, h), 2.0), "transformer.h.0.mlp.w1.weight": torch.full((12, h), 3.0),
          "transformer.h.0.mlp.w2.weight": torch.full((12, h), 4.0), "transformer.h.0.mlp.c_proj.weight": torch.full((h, 12), 5.0),
          "transformer.h.0.ln_1.weight": torch.full((h,), 6.0), "transformer.h.0.ln_2.weight": torch.full((h,), 7.0)}
    conv = H.qwen_to_llama(sd, m)
    assert torch.equal(conv["3.self_attn.q_proj.weight"], c_attn[:h]) and torch.equal(conv["3.self_attn.v_proj.weight"], c_attn[2 * h:])
    assert torch.equal(conv["3.self_attn.k_proj.bias"], c_bias[h:2 * h])
    assert float(conv["3.mlp.gate_proj.weight"][0, 0]) == 4.0 and float(conv["3.mlp.up_proj.weight"][0, 0]) == 3.0  # w2 = gate, w1 = up
    assert float(conv["3.mlp.down_proj.weight"][0, 0]) == 5.0 and float(conv["3.input_layernorm.weight"][0]) == 6.0
    assert float(conv["3.post_attention_layernorm.weight"][0]) == 7.0 and "5.weight" in conv and "6.word_embeddings.weight" in conv


def test_internlm2_wqkv_is_grouped_per_kv_head():
    L, nq, nk, d = 1, 4, 2, 2
    h, gs = nq * d, nq // nk
    m = _FakeModel(L, h, nq, nk)
    # row r of wqkv carries the code 1000*kv_group + 100*slot + head_dim_index in every column
    rows = []
    for g_ in range(nk):
        for slot in range(gs + 2):
            for j in range(d):
                rows.append(torch.full((h,), 1000.0 * g_ + 100.0 * slot + j))
    wqkv = torch.stack(rows)
    sd = {"model.tok_embeddings.weight": torch.zeros(3, h), "model.norm.weight": torch.ones(h), "output.weight": torch.ones(3, h),
          "model.layers.0.attention.wqkv.weight": wqkv, "model.layers.0.attention.wo.weight": torch.ones(h, h),
          "model.layers.0.feed_forward.w1.weight": torch.full((6, h), 1.0), "model.layers.0.feed_forward.w3.weight": torch.full((6, h), 3.0),
          "model.layers.0.feed_forward.w2.weight": torch.full((h, 6), 2.0),
          "model.layers.0.attention_norm.weight": torch.ones(h), "model.layers.0.ffn_norm.weight": torch.ones(h)}
    conv = H.internlm2_to_llama2(sd, m)
    q, k, v = conv["3.self_attn.q_proj.weight"], conv["3.self_attn.k_proj.weight"], conv["3.self_attn.v_proj.weight"]
    assert q.shape == (nq * d, h) and k.shape == (nk * d, h) and v.shape == (nk * d, h)
    assert q[:, 0].tolist() == [0, 1, 100, 101, 1000, 1001, 1100, 1101]     # query heads 0,1 of group 0, then of group 1
    assert k[:, 0].tolist() == [200, 201, 1200, 1201] and v[:, 0].tolist() == [300, 301, 1300, 1301]
    assert float(conv["3.mlp.gate_proj.weight"][0, 0]) == 1.0 and float(conv["3.mlp.up_proj.weight"][0, 0]) == 3.0
    packed = H.internlm2_to_llama2(sd, m, pack=True)["3.self_attn.wqkv.weight"]
    assert torch.equal(packed[0], q) and torch.equal(packed[1], k) and torch.equal(packed[2], v)


def test_tensor_parallel_slicing_rule():
    from easyllm_amd.layers import ColumnParallelLinear, RowParallelLinear, VocabParallelEmbedding
    assert H.get_start_end(5, 4, 0) == [0, 5] and H.get_start_end(5, 4, 3) == [15, 20]
    col = ColumnParallelLinear.__new__(ColumnParallelLinear)
    row = RowParallelLinear.__new__(RowParallelLinear)
    emb = VocabParallelEmbedding.__new__(VocabParallelEmbedding)
    full = torch.arange(8 * 6, dtype=torch.float32).reshape(8, 6)
    assert torch.equal(H.slice_for_rank(full, col, (4, 6), 1, 2), full[4:8])          # output rows split
    assert torch.equal(H.slice_for_rank(full, row, (8, 3), 1, 2), full[:, 3:6])       # input columns split
    assert torch.equal(H.slice_for_rank(full[:, 0], row, (8,), 1, 2), full[:, 0])     # row-parallel bias replicated
    assert torch.equal(H.slice_for_rank(full, emb, (2, 6), 3, 4), full[6:8])          # vocabulary rows split
    q, k, v = full[:4], full[4:6] + 100, full[6:8] + 200
    packed = H.slice_for_rank([q, k, v], col, (4, 6), 1, 2)                            # each of q, k, v split, then joined
    assert torch.equal(packed, torch.cat([q[2:4], k[1:2], v[1:2]]))
    assert torch.equal(H.slice_for_rank(full, object(), (8, 6), 0, 2), full)


def _tiny_model(L=2, h=64, nq=4, nk=2, f=96, V=128, device=None, **extra):
    from easyllm_amd import runner
    kwargs = dict(num_layers=L, hidden_size=h, num_attention_heads=nq, num_kv_attention_heads=nk, intermediate_size=f,
                  vocab_size=V, seq_length=256, micro_batch_size=2, bf16=True, fp32_logits=False)
    kwargs.update(extra)
    return runner.build_model({"type": "llama_custom", "kwargs": kwargs})


def test_copy_into_model_and_padded_vocabulary(tmp_path):
    L, h, nq, nk, f, V = 2, 64, 4, 2, 96, 128
    model = _tiny_model(L, h, nq, nk, f, V + 8)  # model vocabulary padded by 8 rows
    sd = _hf_llama_state(L, h, nq, nk, f, V)
    from safetensors.torch import save_file
    save_file({k: v.contiguous() for k, v in sd.items() if "rotary" not in k}, os.path.join(tmp_path, "model.safetensors"))
    assert H.load_llama_from_hf_format(str(tmp_path / "nothing_here"), model) is False
    assert H.load_llama_from_hf_format(str(tmp_path), model, pretrain_type="llama") is True
    msd = model.state_dict()
    assert torch.equal(msd["3.self_attn.q_proj.weight"].float(), sd["model.layers.0.self_attn.q_proj.weight"].to(msd["3.self_attn.q_proj.weight"].dtype).float())
    emb, src = msd["1.word_embeddings.weight"].float(), sd["model.embed_tokens.weight"]
    assert torch.equal(emb[:V], src.to(msd["1.word_embeddings.weight"].dtype).float())
    donor = int(src.sum(1).argmin())
    assert torch.allclose(emb[V:], (src[donor] * 0.1).expand(8, h), rtol=1e-2, atol=1e-3)
    with pytest.raises(ValueError):
        H.load_llama_from_hf_format(str(tmp_path), model, pretrain_type="baichuan")
    with pytest.raises(ValueError):  # a tensor that cannot belong to the parameter is an error, not a silent copy
        H.copy_into_model({"3.mlp.down_proj.weight": torch.zeros(h + 1, f)}, model)


@pytest.mark.gpu
def test_hf_llama_checkpoint_gives_the_same_logits(gpu_device, tmp_path):
    from transformers import LlamaConfig, LlamaForCausalLM
    print("hf checkpoint -> stack", flush=True)
    L, h, nq, nk, f, V = 2, 256, 4, 2, 512, 1024
    torch.manual_seed(11)
    hf = LlamaForCausalLM(LlamaConfig(vocab_size=V, hidden_size=h, intermediate_size=f, num_hidden_layers=L, num_attention_heads=nq,
                                      num_key_value_heads=nk, rms_norm_eps=1e-6, rope_theta=10000.0, max_position_embeddings=256,
                                      tie_word_embeddings=False, attention_bias=False, hidden_act="silu",
                                      attn_implementation="eager")).bfloat16().float().eval()  # weights exactly representable in bf16
    hf.save_pretrained(str(tmp_path), safe_serialization=True)
    model = _tiny_model(L, h, nq, nk, f, V)
    assert H.load_llama_from_hf_format(str(tmp_path), model, pretrain_type="llama") is True
    tokens = torch.randint(0, V, (2, 160))
    with torch.no_grad():
        ref = hf(input_ids=tokens).logits
        out = model((tokens.to(gpu_device), None, None)).float().cpu()
    err = (out - ref).abs().max().item()
    assert err <= 2e-2 * ref.abs().max().item(), err
    cos = torch.nn.functional.cosine_similarity(out.reshape(-1), ref.reshape(-1), dim=0).item()
    assert cos >= 0.9999, cos
    back = H.megatron_to_hf_llama(model.state_dict(), L)
    assert all(torch.equal(back[k].float().cpu(), v.float()) for k, v in hf.state_dict().items() if "rotary" not in k)
