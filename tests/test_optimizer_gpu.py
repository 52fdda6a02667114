"""Optimizer step through the C ABI against the CPU oracle (and torch.optim.AdamW as a second witness)."""
import pytest
import torch

from oracle import llama_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def K():
    from easyllm_amd import kernels
    return kernels


@pytest.mark.parametrize("n", [1, 7, 4096, 100003])
def test_sumsq_and_clip_coef(K, gpu_device, n):
    print("sumsq", n, flush=True)
    x = torch.randn(n, generator=torch.Generator().manual_seed(n)) * 3
    partials = torch.full((2, K.sumsq_partials()), 7.0, dtype=torch.float32, device=gpu_device)  # every slot is overwritten
    K.sumsq(x.to(gpu_device), partials[0])
    K.sumsq(torch.zeros(0, dtype=torch.float32, device=gpu_device), partials[1])
    assert float(partials[1].abs().max()) == 0.0
    norm = O.global_grad_norm([x])
    for max_norm in (1.0, 1e9, 0.0):
        out = K.clip_coef(partials.view(-1), max_norm).cpu()
        assert abs(float(out[0]) - norm) <= 2e-6 * norm
        assert abs(float(out[1]) - O.clip_coefficient(norm, max_norm)) <= 2e-6
    again = torch.empty_like(partials[0])
    K.sumsq(x.to(gpu_device), again)
    assert torch.equal(again, partials[0])  # fixed reduction order


@pytest.mark.parametrize("n,wd,bc", [(8, 0.0, True), (1027, 0.1, True), (65536 + 3, 0.01, False)])
def test_adamw_kernel_matches_oracle(K, gpu_device, n, wd, bc):
    print("adamw", n, wd, bc, flush=True)
    g = torch.Generator().manual_seed(31)
    p0 = torch.randn(n, generator=g).bfloat16().float()
    master, m, v = p0.clone(), torch.zeros(n), torch.zeros(n)
    dm, de, dv = p0.to(gpu_device), torch.zeros(n, device=gpu_device), torch.zeros(n, device=gpu_device)
    param = p0.bfloat16().to(gpu_device)
    coef = torch.tensor([123.0, 0.25], device=gpu_device)
    lr, b1, b2, eps = 1e-2, 0.9, 0.95, 1e-8
    for step in range(1, 5):
        grad = torch.randn(n, generator=g) * (0.05 if step % 2 else 4.0)
        use_coef = step >= 3
        master, m, v = O.adamw_step(master, m, v, grad * (0.25 if use_coef else 1.0), lr, b1, b2, eps, wd, step, bc)
        K.adamw_step(dm, de, dv, grad.to(gpu_device), param, lr, b1, b2, eps, wd, step, bc, coef if use_coef else None)
        assert torch.allclose(dm.cpu(), master, rtol=2e-6, atol=1e-6), step  # fp32 rounding of fused multiply-adds
        assert torch.allclose(de.cpu(), m, rtol=2e-6, atol=1e-6) and torch.allclose(dv.cpu(), v, rtol=2e-6, atol=1e-6)
        assert torch.equal(param, dm.bfloat16())  # bf16 weight = round-to-nearest-even of the master value


def test_fused_adam_on_a_model_matches_torch_adamw(gpu_device):
    """Two steps of build_optimizer(...).step(clip_grad=1.0) on a tiny stack against torch.optim.AdamW +
    clip_grad_norm_ run on fp32 CPU copies fed with the same main_grads; checks the reference's weight-decay split."""
    from easyllm_amd import optimizer, runner, workloads as W
    w = dict(num_layers=2, hidden_size=256, num_attention_heads=4, num_kv_attention_heads=2, intermediate_size=512,
             vocab_size=512, seq=128, batch=2, seed=9)
    torch.manual_seed(w["seed"])
    model = runner.build_model({"type": "llama_custom", "kwargs": W.model_kwargs(w)})
    runner.attach_main_grads(model)
    opt = optimizer.build_optimizer({"type": "FusedAdam", "kwargs": {"lr": 1e-3, "weight_decay": 0.1, "betas": [0.9, 0.95],
                                                                     "eps": 1e-8}}, model)
    names = {p: n for n, p in model.named_parameters()}
    (decay,) = opt.param_groups  # the empty no-decay group (no biases, no MixedFusedLayerNorm here) is filtered out
    assert decay["weight_decay"] == 0.1 and len(decay["params"]) == len(names)
    ref = {n: torch.nn.Parameter(p.detach().float().cpu()) for n, p in model.named_parameters()}
    ref_opt = torch.optim.AdamW([ref[names[p]] for p in decay["params"]], lr=1e-3, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
    inputs, labels, _ = W.make_inputs(w, device=gpu_device)
    for step in range(2):
        opt.zero_grad()
        runner.forward_step(model, inputs, labels)
        for n, p in model.named_parameters():
            ref[n].grad = p.main_grad.detach().cpu().clone() * (50.0 if step == 0 else 1.0)
            if step == 0:
                p.main_grad.mul_(50.0)  # force the clip to bite in the first step
        total = float(torch.nn.utils.clip_grad_norm_(list(ref.values()), max_norm=1.0))
        norm_coef = opt.step(clip_grad=1.0).cpu()
        ref_opt.step()
        assert abs(float(norm_coef[0]) - total) <= 1e-4 * total
        assert (float(norm_coef[1]) < 1.0) == (total > 1.0)
        for n, p in model.named_parameters():
            assert torch.allclose(opt.state[p]["master"].cpu(), ref[n].detach(), rtol=1e-4, atol=1e-6), (step, n)
            assert torch.equal(p.detach(), opt.state[p]["master"].bfloat16()), n
