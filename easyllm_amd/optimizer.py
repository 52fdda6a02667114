"""Optimizer step for the decoder stack: AdamW on fp32 master weights with global-norm gradient clipping.

Mirrors what the reference's Megatron path runs after backward:

* `build_optimizer(cfg_optim, model)` (llm/utils/model/optimizer_helper.py:70-98) with the weight-decay split of
  `_get_params_for_weight_decay_optimization` (:19-51) and `filter_freeze_param_groups` (:60-67).  The split is
  restated literally: only modules whose class is named `MixedFusedLayerNorm` and parameters named `bias` are exempt
  from decay, so the `RMSNorm` weights of the llama stack DO decay when `weight_decay` is non-zero (the shipped
  configs set it to 0);
* apex `FusedAdam(params, lr, bias_correction=True, betas, eps, adam_w_mode=True, weight_decay)` as configured by
  configs/megatron/llama_7b_sft.yaml:106-112;
* DeepSpeed's bf16 optimizer around it: fp32 master copy of every bf16 weight, fp32 gradient accumulation (the
  `main_grad` buffers of this build), `gradient_clipping: 1.0` (llama_7b_sft.yaml:13) on the global L2 norm.

apex and DeepSpeed are not part of the reference tree; the arithmetic is their published AdamW / clipping rule and is
pinned in the tests against torch.optim.AdamW + torch.nn.utils.clip_grad_norm_.  Everything runs in HIP kernels on
the current stream; the clip coefficient never leaves the device.
"""
import torch

from . import kernels as K

NO_DECAY_MODULES = ("MixedFusedLayerNorm",)


def get_params_for_weight_decay_optimization(model):
    """-> (decay group, no-decay group); optimizer_helper.py:19-51 without the apex work-around that halves the first
    group (:41-49; the split changes nothing in the arithmetic)."""
    decay, no_decay = {"params": []}, {"params": [], "weight_decay": 0.0}
    for module_ in model.modules():
        own = [(n, p) for n, p in module_._parameters.items() if p is not None]
        if module_.__class__.__name__ in NO_DECAY_MODULES:
            no_decay["params"].extend(p for _, p in own)
        else:
            decay["params"].extend(p for n, p in own if n != "bias")
            no_decay["params"].extend(p for n, p in own if n == "bias")
    return decay, no_decay


def filter_freeze_param_groups(param_groups):
    """optimizer_helper.py:60-67: groups without a trainable parameter are dropped."""
    return [g for g in param_groups if any(p.requires_grad for p in g["params"])]


class FusedAdam:
    """apex.optimizers.FusedAdam's constructor surface (AdamW mode) over bf16 weights with fp32 master copies.

    Gradients are read from `param.main_grad` (fp32).  `step(clip_grad=c)` clips by the global L2 norm first when
    c > 0 and returns the device tensor (norm, coefficient)."""

    def __init__(self, params, lr=1e-3, bias_correction=True, betas=(0.9, 0.999), eps=1e-8, adam_w_mode=True,
                 weight_decay=0.0, amsgrad=False, set_grad_none=True):
        if amsgrad:
            raise RuntimeError("FusedAdam does not support the AMSGrad variant.")  # apex raises the same
        if not adam_w_mode:
            raise NotImplementedError("only the AdamW mode (decoupled weight decay) is built")
        params = list(params)
        if params and not isinstance(params[0], dict):
            params = [{"params": params}]
        self.defaults = dict(lr=lr, bias_correction=bias_correction, betas=tuple(betas), eps=eps, weight_decay=weight_decay)
        self.param_groups = []
        for g in params:
            group = dict(self.defaults)
            group.update(g)
            group["params"] = [p for p in group["params"] if p.requires_grad]
            group["step"] = 0
            self.param_groups.append(group)
        self.state = {}
        for group in self.param_groups:
            for p in group["params"]:
                if getattr(p, "main_grad", None) is None:
                    raise ValueError("every optimised parameter needs an fp32 main_grad buffer (runner.attach_main_grads)")
                self.state[p] = {"master": p.detach().float().contiguous(), "exp_avg": torch.zeros_like(p, dtype=torch.float32),
                                 "exp_avg_sq": torch.zeros_like(p, dtype=torch.float32)}
        n = sum(len(g["params"]) for g in self.param_groups)
        dev = self.param_groups[0]["params"][0].device if n else torch.device("cpu")
        self._partials = torch.zeros(max(n, 1), K.sumsq_partials(), dtype=torch.float32, device=dev) if n else None
        self._norm_coef = torch.ones(2, dtype=torch.float32, device=dev) if n else None

    def _all_params(self):
        for group in self.param_groups:
            for p in group["params"]:
                yield group, p

    def global_grad_norm(self, max_norm):
        """(norm, coefficient) of all main_grads as a device tensor; max_norm <= 0 disables clipping (coefficient 1)."""
        for i, (_, p) in enumerate(self._all_params()):
            K.sumsq(p.main_grad.view(-1), self._partials[i])
        return K.clip_coef(self._partials.view(-1), max_norm, out=self._norm_coef)

    def step(self, clip_grad=0.0):
        norm_coef = self.global_grad_norm(clip_grad) if clip_grad and clip_grad > 0 else None
        for group in self.param_groups:
            if not group["params"]:
                continue
            group["step"] += 1
            b1, b2 = group["betas"]
            for p in group["params"]:
                st = self.state[p]
                K.adamw_step(st["master"].view(-1), st["exp_avg"].view(-1), st["exp_avg_sq"].view(-1), p.main_grad.view(-1),
                             p.data.view(-1) if p.dtype == torch.bfloat16 else None, group["lr"], b1, b2, group["eps"],
                             group["weight_decay"], group["step"], group["bias_correction"], norm_coef)
                if p.dtype != torch.bfloat16:
                    p.data.copy_(st["master"])
        return norm_coef

    def refresh_fp32_params(self):
        """Re-reads the fp32 master copies from the model weights (called after a checkpoint was loaded into them)."""
        for _, p in self._all_params():
            self.state[p]["master"].copy_(p.detach().float())

    def zero_grad(self, set_to_none=True):
        """No memset: the next gradient written to each main_grad overwrites it."""
        for _, p in self._all_params():
            p.main_grad_fresh = True
            p.grad = None


def build_optimizer(cfg_optim, model, deepspeed=True):
    """cfg_optim = {'type': 'FusedAdam', 'kwargs': {lr, weight_decay, betas, eps}} as in the reference's yaml `optimizer:`."""
    if cfg_optim.get("cpu_optimizer", False):
        raise NotImplementedError("need to add cpu adam")  # same refusal as optimizer_helper.py:71-72
    if cfg_optim["type"] not in ("FusedAdam", "AdamW"):
        raise NotImplementedError("optimizer type %s is not built; FusedAdam / AdamW are" % cfg_optim["type"])
    groups = filter_freeze_param_groups(list(get_params_for_weight_decay_optimization(model)))
    kwargs = dict(cfg_optim.get("kwargs", {}))
    kwargs.pop("params", None)
    return FusedAdam(groups, **kwargs)
