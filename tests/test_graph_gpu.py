"""The captured step must reproduce the eager step bit for bit on every replay, with eager work and synchronisations of
the program's own in between, and with new inputs copied into its static buffers."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_graphed_step_matches_eager_on_every_replay(gpu_device):
    from easyllm_amd import runner, workloads as W
    print("graphed step", flush=True)
    w = dict(num_layers=2, hidden_size=256, num_attention_heads=4, num_kv_attention_heads=2, intermediate_size=512,
             vocab_size=1024, seq=256, batch=2, seed=17)
    torch.manual_seed(w["seed"])
    model = runner.build_model({"type": "llama_custom", "kwargs": W.model_kwargs(w)})
    runner.attach_main_grads(model)
    batches = []
    for seed in (17, 18, 19):
        w2 = dict(w, seed=seed)
        batches.append(W.make_inputs(w2, device=gpu_device)[:2])

    def eager(inputs, labels):
        runner.zero_main_grads(model)
        loss = runner.forward_step(model, inputs, labels)
        return loss.item(), {n: p.main_grad.clone() for n, p in model.named_parameters()}

    expected = [eager(i, l) for i, l in batches]
    step = runner.GraphedStep(model, *batches[0])
    for rnd in range(2):
        for (inputs, labels), (loss_ref, grads_ref) in zip(batches, expected):
            loss = step(inputs, labels)
            torch.cuda.synchronize()
            assert loss.item() == loss_ref, (rnd, loss.item(), loss_ref)
            for n, p in model.named_parameters():
                assert torch.equal(p.main_grad, grads_ref[n]), (rnd, n)
            # eager work of the program's own between replays
            l2, _ = eager(*batches[1])
            assert l2 == expected[1][0]
    # an out-of-range token id surfaces as the same ValueError, one call late
    bad = batches[0][0][0].clone()
    bad[0, 3] = w["vocab_size"]
    step((bad,) + tuple(batches[0][0][1:]), batches[0][1])
    with pytest.raises(ValueError):
        step.flush()


def test_graphed_accumulating_step_adds_to_what_the_buffers_hold(gpu_device):
    """Eager micro-batch A, then a replay of a graph captured with accumulate=True on micro-batch B: the fp32 buffers
    must hold exactly what eager A followed by eager B (accumulating) leaves, bit for bit -- the warm-up passes that
    precede the capture may not leak into them -- and a buffer marked fresh starts the replay from zero."""
    from easyllm_amd import runner, workloads as W
    print("graphed accumulating step", flush=True)
    w = dict(num_layers=2, hidden_size=256, num_attention_heads=4, num_kv_attention_heads=2, intermediate_size=512,
             vocab_size=1024, seq=256, batch=2, seed=23)
    torch.manual_seed(w["seed"])
    model = runner.build_model({"type": "llama_custom", "kwargs": W.model_kwargs(w)})
    runner.attach_main_grads(model)
    A = W.make_inputs(dict(w, seed=23), device=gpu_device)[:2]
    B = W.make_inputs(dict(w, seed=24), device=gpu_device)[:2]

    def grads():
        return {n: p.main_grad.clone() for n, p in model.named_parameters()}

    runner.zero_main_grads(model)
    runner.forward_step(model, *A)
    runner.forward_step(model, *B)
    expect_ab = grads()
    runner.zero_main_grads(model)
    runner.forward_step(model, *B)
    expect_b = grads()

    runner.zero_main_grads(model)
    runner.forward_step(model, *A)
    held = grads()
    step = runner.GraphedStep(model, *B, accumulate=True)
    for n, p in model.named_parameters():  # building the graph left the buffers as they were
        assert torch.equal(p.main_grad, held[n]), n
    step()
    torch.cuda.synchronize()
    for n, p in model.named_parameters():
        assert torch.equal(p.main_grad, expect_ab[n]), n
    # second round with the same graph: zero, eager A, replay B
    runner.zero_main_grads(model)
    runner.forward_step(model, *A)
    step()
    torch.cuda.synchronize()
    for n, p in model.named_parameters():
        assert torch.equal(p.main_grad, expect_ab[n]), n
    # buffers marked fresh: the replay alone leaves B's gradients
    runner.zero_main_grads(model)
    step()
    torch.cuda.synchronize()
    for n, p in model.named_parameters():
        assert torch.equal(p.main_grad, expect_b[n]), n
