"""GPU parity of the whole decoder-layer training step (model classes -> autograd wrappers -> C ABI ->
HIP kernels) against the fp32 CPU oracle on identical seeded inputs and (bf16-rounded) weights.

Tolerances (stated by the task): loss within 1e-3 relative; logits and parameter gradients
max |a - ref| <= 2e-2 * max |ref| and cosine >= 0.9999; token gather and label masking bit-exact.
"""
import pytest
import torch

from oracle import llama_oracle as O

pytestmark = pytest.mark.gpu


def close(a, ref, name, rel=2e-2, cos=0.9999):
    a = a.detach().float().cpu().reshape(-1)
    ref = ref.detach().float().cpu().reshape(-1)
    assert a.shape == ref.shape, name
    assert torch.isfinite(a).all(), name + ": non-finite"
    denom = ref.abs().max().item()
    err = (a - ref).abs().max().item()
    assert err <= rel * max(denom, 1e-30), "%s: max err %.3e vs max ref %.3e" % (name, err, denom)
    if denom > 0:
        c = (torch.dot(a, ref) / (a.norm() * ref.norm() + 1e-30)).item()
        assert c >= cos, "%s: cosine %.6f" % (name, c)


def oracle_cfg(w):
    return dict(num_layers=w["num_layers"], hidden_size=w["hidden_size"], num_attention_heads=w["num_attention_heads"],
                num_kv_attention_heads=w["num_kv_attention_heads"], head_dim=w["hidden_size"] // w["num_attention_heads"],
                intermediate_size=w["intermediate_size"], vocab_size=w["vocab_size"])


def build_pair(w, dev, **overrides):
    """HIP model on the GPU + oracle weights holding the same (bf16-rounded) values."""
    from easyllm_amd import runner, workloads as W
    model = runner.build_model({"type": "llama_custom", "kwargs": W.model_kwargs(w, **overrides)})
    Wt = O.init_weights(oracle_cfg(w), seed=w["seed"], round_to_bf16=True)
    for k in list(Wt):  # non-trivial norm weights so that their gradients are exercised
        if "layernorm" in k or k.endswith(".weight") and Wt[k].dim() == 1:
            g = torch.Generator().manual_seed(len(k))
            Wt[k] = (1.0 + 0.1 * torch.randn(Wt[k].shape, generator=g)).bfloat16().float()
    sd = {k: v.to(torch.bfloat16) for k, v in Wt.items()}
    missing, unexpected = model.load_state_dict(sd, strict=False)
    assert not unexpected and all("inv_freq" in m for m in missing), (missing, unexpected)
    model.to(dev)
    runner.attach_main_grads(model)
    return model, Wt


def oracle_step(Wt, w, inputs, labels, loss_mask):
    Wg = {k: v.clone().requires_grad_(True) for k, v in Wt.items()}
    pos = inputs[1] if len(inputs) == 4 else None
    cu = inputs[3] if len(inputs) == 4 else None
    logits = O.model_forward(Wg, oracle_cfg(w), inputs[0], pos, cu)
    loss = O.cross_entropy_loss(logits, labels, loss_mask)
    loss.backward()
    return logits.detach(), loss.item(), {k: v.grad for k, v in Wg.items()}


def to_dev(t, dev):
    return tuple(None if x is None else x.to(dev) for x in t)


def check_step(model, Wt, w, inputs, labels, loss_mask, dev):
    from easyllm_amd import runner
    ref_logits, ref_loss, ref_grads = oracle_step(Wt, w, inputs, labels, loss_mask)
    runner.zero_main_grads(model)
    logits = model(to_dev(inputs, dev))
    close(logits, ref_logits, "logits")
    loss = model.loss_fn(logits, (labels.to(dev), loss_mask.to(dev)))
    loss.backward()
    assert abs(loss.item() - ref_loss) <= 1e-3 * abs(ref_loss), "loss %.6f vs %.6f" % (loss.item(), ref_loss)
    for name, p in model.named_parameters():
        close(p.main_grad, ref_grads[name], "grad " + name)
    return loss.item()


def test_c1_tiny_llama_full_step(gpu_device):
    """Config 1 (the CPU-runnable case): 2 layers, h256, 4x64 MHA, f688, V32000, s512, b2."""
    from easyllm_amd import workloads as W
    w = W.WORKLOADS["C1"]
    model, Wt = build_pair(w, gpu_device)
    inputs, (labels, loss_mask), _ = W.make_inputs(w)
    print("C1 step", flush=True)
    check_step(model, Wt, w, inputs, labels, loss_mask, gpu_device)


def test_gqa_packed_dynamic_checkpoint_step(gpu_device):
    """Small GQA stack with a packed batch (cu_seqlens + restarting position ids), 10% ignored labels
    and the dynamic checkpoint rule active; checks parity with the oracle AND that loss and every
    gradient are bit-identical whatever number of layers is recomputed."""
    from easyllm_amd import data, workloads as W
    w = dict(num_layers=3, hidden_size=512, num_attention_heads=4, num_kv_attention_heads=2, intermediate_size=1024,
             vocab_size=4096, seq=768, batch=1, seed=77, ignore_frac=0.1,
             dynamic_checkpoint={"enabled": True, "size_map": {256: 0, 512: 1, 1024: 2, 2048: 3}})
    model, Wt = build_pair(w, gpu_device)
    inputs, (labels, loss_mask), _ = W.make_inputs(w)
    doc_lens = [1, 200, 63, 257, 247]
    cu = [0]
    for l in doc_lens:
        cu.append(cu[-1] + l)
    pos = torch.tensor([data.get_position_ids(cu)])
    inputs = (inputs[0], pos, None, torch.tensor(cu, dtype=torch.int64))
    loss_mask[0, 5] = 0.0
    print("packed GQA step, k=2", flush=True)
    base = check_step(model, Wt, w, inputs, labels, loss_mask, gpu_device)
    assert model.recompute_count == 2  # seq 768 -> size_map key 1024 -> first 2 layers
    ref = {n: p.main_grad.clone() for n, p in model.named_parameters()}
    from easyllm_amd import runner
    for k in (0, 3):
        model.size_map = {4096: k}
        runner.zero_main_grads(model)
        loss = runner.forward_step(model, to_dev(inputs, gpu_device), (labels.to(gpu_device), loss_mask.to(gpu_device)))
        assert model.recompute_count == k
        assert loss.item() == base
        for n, p in model.named_parameters():
            assert torch.equal(p.main_grad, ref[n]), n  # every kernel, the embedding scatter included, sums in a fixed order


def test_batched_mha_with_bool_loss_mask_and_accumulation(gpu_device):
    """b=2 exercises the [b,s,h] <-> [s,b,h] moves; two micro-batches accumulate into main_grad (linearity)."""
    from easyllm_amd import runner, workloads as W
    w = dict(num_layers=2, hidden_size=256, num_attention_heads=2, num_kv_attention_heads=2, intermediate_size=512,
             vocab_size=1024, seq=160, batch=2, seed=5)
    model, Wt = build_pair(w, gpu_device)
    inputs, (labels, loss_mask), _ = W.make_inputs(w)
    loss_mask = torch.rand(2, 160, generator=torch.Generator().manual_seed(3)) < 0.9  # bool, as flash_batch_pipe emits
    check_step(model, Wt, w, inputs, labels, loss_mask, gpu_device)
    one = {n: p.main_grad.clone() for n, p in model.named_parameters()}
    runner.forward_step(model, to_dev(inputs, gpu_device), (labels.to(gpu_device), loss_mask.to(gpu_device)))  # accumulates
    for n, p in model.named_parameters():
        close(p.main_grad, 2 * one[n], "accumulated " + n, rel=1e-3)


def test_packed_samples_from_the_token_cache_through_the_step(gpu_device, tmp_path):
    """The data path of the packed workload end to end: a token cache on disk built from tokenised json lines ->
    `MMapIndexJsonDataset(with_cu_lens=True)` samples (llm/data/nlp_dataset.py:596-646) -> `BatchAlignCollector`'s shift
    and boundary flattening (nlp_dataloader.py:131-187) -> `flash_batch_pipe`'s tuple (nlp_batch_fn.py:181-205) -> the HIP
    step; loss, logits and every gradient against the oracle fed the same batch."""
    import json
    import numpy as np
    from easyllm_amd import data as D, mmap_dataset as M
    V, pad, eos, seq, b = 1008, 1007, 2, 256, 2

    class Tok:
        vocab_size, eos_token_id = V, eos

    rng = np.random.RandomState(21)
    with open(tmp_path / "train.jsonl", "w") as f:
        for _ in range(80):
            f.write(json.dumps({"input_ids": rng.randint(3, 1000, size=int(rng.randint(5, 120))).tolist() + [eos]}) + "\n")
    ds = M.MMapIndexJsonDataset(str(tmp_path), seed=9, total_samples=6, max_seq_length=seq, json_file=str(tmp_path / "train.jsonl"),
                                tokenizer=Tok(), cache_worker=1, with_cu_lens=True)
    items = [ds[1], ds[4]]
    batch = D.batch_align_collate(items, pad_token_id=pad, max_seq_length=seq, pretrain=True)
    inputs, (labels, loss_mask) = D.flash_batch_from(batch, pad_token_id=pad, pretrain=True)
    tokens, position_ids, attention_mask, cu_seqlens = inputs
    assert tuple(tokens.shape) == (b, seq) and cu_seqlens[-1].item() == b * seq and len(cu_seqlens) > 4
    assert position_ids[0, :5].tolist() == [0, 1, 2, 3, 4] and (position_ids == 0).sum().item() == len(cu_seqlens) - 1
    w = dict(num_layers=2, hidden_size=512, num_attention_heads=8, num_kv_attention_heads=2, intermediate_size=1024,
             vocab_size=V, seq=seq, batch=b, seed=31)
    model, Wt = build_pair(w, gpu_device)
    print("step on packed samples of a token cache:", len(cu_seqlens) - 1, "documents", flush=True)
    check_step(model, Wt, w, inputs, labels, loss_mask, gpu_device)


def test_loss_paths_agree_and_reference_api(gpu_device):
    from easyllm_amd.losses import CrossEntropy, vocab_parallel_cross_entropy
    g = torch.Generator().manual_seed(9)
    logits = (torch.randn(2, 40, 2048, generator=g) * 2).bfloat16()
    labels = torch.randint(0, 2048, (2, 40), generator=g)
    labels[0, 3] = -100
    lm = torch.ones(2, 40)
    lm[1, 7] = 0
    la = logits.to(gpu_device).requires_grad_(True)
    lb = logits.to(gpu_device).requires_grad_(True)
    fused = CrossEntropy(is_prefix=False)(la, (labels.to(gpu_device), lm.to(gpu_device)))
    plain = CrossEntropy(is_prefix=False, fused=False)(lb, (labels.to(gpu_device), lm.to(gpu_device)))
    ref = O.cross_entropy_loss(logits.float(), labels, lm)
    assert abs(fused.item() - ref.item()) <= 1e-3 * ref.item() and abs(plain.item() - ref.item()) <= 1e-3 * ref.item()
    (fused * 3.0).backward()  # exercises the upstream-gradient scaling of the fused path
    (plain * 3.0).backward()
    close(la.grad, lb.grad, "fused vs unfused grad", rel=1e-2)
    per_tok = vocab_parallel_cross_entropy(logits.float().to(gpu_device), labels.to(gpu_device))  # fp32 logits, as the reference calls it
    assert torch.allclose(per_tok.cpu(), O.vocab_parallel_cross_entropy(logits.float(), labels), rtol=1e-4, atol=1e-4)


def test_bad_token_id_raises_value_error(gpu_device):
    from easyllm_amd.layers import VocabParallelEmbedding, init_method_normal
    emb = VocabParallelEmbedding(100, 64, init_method=init_method_normal(0.02), params_dtype=torch.bfloat16)
    ids = torch.tensor([[1, 2, 100]], device=gpu_device)
    with pytest.raises(ValueError):
        emb(ids)
    out = emb(torch.tensor([[1, 2, 99]], device=gpu_device))
    assert torch.equal(out[0, 2], emb.weight[99])  # gather is bit-exact
    # deferred mode: same error, raised when the flag is examined instead of inside the call
    from easyllm_amd import functional
    functional.set_input_check("deferred")
    try:
        emb(torch.tensor([[1, 2, 99]], device=gpu_device))
        functional.flush_input_checks()
        emb(ids)
        with pytest.raises(ValueError):
            functional.flush_input_checks()
        functional.flush_input_checks()  # nothing left pending
    finally:
        functional._PENDING_CHECKS.clear()
        functional.set_input_check("sync")


def test_position_id_beyond_the_rotary_table_raises_index_error(gpu_device):
    """The reference indexes its cos / sin tables (one row per sequence position) with the position ids; an id past the
    table is an indexing error there (positional_embeddings.py:109-117).  Same here, from the embedding stage."""
    from easyllm_amd import workloads as W
    w = dict(num_layers=1, hidden_size=256, num_attention_heads=2, num_kv_attention_heads=2, intermediate_size=512,
             vocab_size=1024, seq=64, batch=1, seed=8)
    model, _ = build_pair(w, gpu_device)
    inputs, (labels, loss_mask), _ = W.make_inputs(w)
    cu = torch.tensor([0, 40, 64])
    good = torch.tensor([list(range(40)) + list(range(24))])
    model(to_dev((inputs[0], good, None, cu), gpu_device))
    bad = good.clone()
    bad[0, 50] = 64
    with pytest.raises(IndexError):
        model(to_dev((inputs[0], bad, None, cu), gpu_device))
    bad[0, 50] = -1
    with pytest.raises(IndexError):
        model(to_dev((inputs[0], bad, None, cu), gpu_device))


def test_qkv_pack_and_bias_variants(gpu_device):
    """wqkv (q|k|v packed, transformer.py:427-429) with qkv bias: parity of one layer against the oracle."""
    from easyllm_amd.transformer import ParallelTransformerLayer
    h, nq, nk, d, f, s, b = 256, 4, 2, 64, 512, 96, 2
    ln = {"type": "rms_norm", "kwargs": dict(sync_tp_duplicated_parameters=True, normalized_shape=h, eps=1e-6,
                                             use_flash_attn=True, bf16=True, sequence_parallel=False)}
    layer = ParallelTransformerLayer(0, self_attn_mask_type="causal", position_embedding_type="rotary", params_dtype="bfloat16",
                                     layer_norm=ln, bf16=True, kv_channels=d, num_attention_heads=nq, num_kv_attention_heads=nk,
                                     hidden_size=h, glu_activation="silu", intermediate_size=f, use_flash_attn=True,
                                     qkv_pack=True, attention_qkv_bias=True).to(gpu_device)
    with torch.no_grad():
        layer.self_attn.wqkv.bias.normal_(0, 0.02)
    Wt = {"3." + k: v.detach().float().cpu() for k, v in layer.state_dict().items()}
    x = (torch.randn(s, b, h, generator=torch.Generator().manual_seed(1))).bfloat16()
    cfg = dict(num_attention_heads=nq, num_kv_attention_heads=nk, head_dim=d)
    xr = x.float().requires_grad_(True)
    Wg = {k: v.clone().requires_grad_(True) for k, v in Wt.items()}
    ref = O.decoder_layer(xr, Wg, "3.", cfg)
    dy = torch.randn(s, b, h, generator=torch.Generator().manual_seed(2)).bfloat16()
    ref.backward(dy.float())
    xg = x.to(gpu_device).requires_grad_(True)
    out = layer(xg, None)
    close(out, ref, "packed layer out")
    out.backward(dy.to(gpu_device))
    close(xg.grad, xr.grad, "packed layer dx")
    close(layer.self_attn.wqkv.weight.grad, Wg["3.self_attn.wqkv.weight"].grad, "wqkv grad")
    close(layer.self_attn.wqkv.bias.grad, Wg["3.self_attn.wqkv.bias"].grad, "wqkv bias grad")
