"""Step driver: forward -> loss -> backward for one micro-batch, with fp32 main-grad buffers.

Counterpart of `BaseRunner.forward_step` -> DeepSpeed `train_batch` (llm/runners/base_llm_runner.py:236-245)
for what lies inside this build: `loss = loss_fn(model(inputs), labels); loss.backward()`, weight
gradients landing in fp32 `main_grad` buffers (DeepSpeed's bf16 optimizer accumulates in fp32).
The optimizer step, gradient clipping, loss scaling by accumulation steps and ZeRO are DeepSpeed's
and are not reproduced.
"""
import torch

from .registry import MODULE_ZOO_REGISTRY
from . import llama as _llama  # noqa: F401  (registers the model builders)


def build_model(cfg):
    """cfg = {'type': 'llama_custom' | 'llama2_7b' | ..., 'kwargs': {...}} as in the reference's yaml `model:` node."""
    return MODULE_ZOO_REGISTRY.build(cfg)


def attach_main_grads(model):
    """One fp32 gradient buffer per parameter; marks them fresh (first write overwrites)."""
    for p in model.parameters():
        if p.requires_grad:
            p.main_grad = torch.zeros(p.shape, dtype=torch.float32, device=p.device)
            p.main_grad_fresh = True


def zero_main_grads(model):
    """zero_grad without a memset: the next gradient written to each buffer overwrites it."""
    for p in model.parameters():
        if getattr(p, "main_grad", None) is not None:
            p.main_grad_fresh = True
        p.grad = None


def forward_step(model, inputs, labels):
    """One micro-batch: returns the loss tensor after backward has run."""
    output = model(inputs)
    loss = model.loss_fn(output, labels)
    loss.backward()
    return loss
