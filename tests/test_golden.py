"""The committed golden fixture (tests/golden/hf_llama_tiny.npz, written by tests/golden/make_hf_llama_fixture.py from
transformers' LlamaForCausalLM in fp32) against the CPU oracle, and against the HIP path on a GPU.

Tolerances: oracle vs fixture is fp32 vs fp32 (1e-5 on the loss, 2e-4 absolute on logits, 1e-3 relative on gradient norms);
HIP vs fixture is the bf16 bar: loss within 1e-3 relative, tensors max |a - ref| <= 2e-2 max |ref|.
"""
import os
import sys

import numpy as np
import pytest
import torch

from oracle import llama_oracle as O

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
sys.path.insert(0, GOLDEN)
import hf_llama_recipe as R  # noqa: E402


@pytest.fixture(scope="module")
def fixture():
    data = np.load(os.path.join(GOLDEN, "hf_llama_tiny.npz"))
    W = R.make_weights()
    # the seeded recipe reproduces the weights the fixture was computed with
    assert abs(sum(v.double().abs().sum().item() for v in W.values()) - float(data["weights_abs_sum"])) < 1e-6
    tokens, labels = R.make_batch()
    assert np.array_equal(tokens.numpy(), data["tokens"]) and np.array_equal(labels.numpy(), data["labels"])
    return data, W, tokens, labels


def test_oracle_reproduces_the_fixture(fixture):
    data, W, tokens, labels = fixture
    Wg = {k: v.clone().requires_grad_(True) for k, v in W.items()}
    logits = O.model_forward(Wg, R.CFG, tokens)
    loss = O.cross_entropy_loss(logits, labels, torch.ones(labels.shape))
    loss.backward()
    assert abs(loss.item() - float(data["loss"])) < 1e-5
    assert np.allclose(logits.detach()[:, ::4, ::8].numpy(), data["logits_slice"], atol=2e-4, rtol=1e-4)
    for k, v in Wg.items():
        ref_norm = float(data["gnorm/" + k])
        assert abs(v.grad.double().norm().item() - ref_norm) <= 1e-3 * ref_norm, k
        ref_block = data["gblock/" + k]
        assert np.allclose(R.grad_block(v.grad).numpy(), ref_block, atol=1e-3 * np.abs(ref_block).max() + 1e-7), k


@pytest.mark.gpu
def test_hip_step_reproduces_the_fixture(fixture, gpu_device):
    from easyllm_amd import runner
    data, W, tokens, labels = fixture
    c = R.CFG
    model = runner.build_model({"type": "llama_custom", "kwargs": dict(
        num_layers=c["num_layers"], hidden_size=c["hidden_size"], num_attention_heads=c["num_attention_heads"],
        num_kv_attention_heads=c["num_kv_attention_heads"], intermediate_size=c["intermediate_size"],
        vocab_size=c["vocab_size"], seq_length=R.SEQ, micro_batch_size=R.BATCH, bf16=True, use_flash_attn=True)})
    missing, unexpected = model.load_state_dict({k: v.bfloat16() for k, v in W.items()}, strict=False)
    assert not unexpected and all("inv_freq" in m for m in missing), (missing, unexpected)
    model.to(gpu_device)
    runner.attach_main_grads(model)
    from easyllm_amd import data as D
    inputs, (lab, loss_mask) = D.json_batch(tokens.to(gpu_device), labels.to(gpu_device), pad_token_id=-1)
    output = model(inputs)
    loss = model.loss_fn(output, (lab, loss_mask))
    loss.backward()
    ref_loss = float(data["loss"])
    assert abs(loss.item() - ref_loss) <= 1e-3 * abs(ref_loss)
    logits = output.detach().float().cpu()
    ref = data["logits_slice"]
    assert np.abs(logits[:, ::4, ::8].numpy() - ref).max() <= 2e-2 * np.abs(ref).max()
    grads = {k: p.main_grad for k, p in model.named_parameters()}
    for k in W:
        ref_norm = float(data["gnorm/" + k])
        assert abs(grads[k].double().norm().item() - ref_norm) <= 2e-2 * ref_norm, k
        ref_block = data["gblock/" + k]
        got = R.grad_block(grads[k]).float().cpu().numpy()
        # the kept block is a small corner: bound its error by the scale of the whole gradient
        scale = ref_norm / np.sqrt(grads[k].numel())
        assert np.abs(got - ref_block).max() <= 2e-2 * max(np.abs(ref_block).max(), 4 * scale), k
