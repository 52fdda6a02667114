"""Loss of the llama step (reference: llama/losses.py:11-56, base_modules/functions/cross_entropy.py:115-117)."""
import torch

from . import functional as F_
from .registry import LOSS_REGISTRY

IGNORE_INDEX = -100  # llm/data/nlp_dataset.py:20

vocab_parallel_cross_entropy = F_.vocab_parallel_cross_entropy


@LOSS_REGISTRY.register("softmax_cross_entropy")
class CrossEntropy(object):
    """loss = sum(per_token * mask) / N, mask = loss_mask * (labels != -100), N = sum(mask).

    `fused=True` (default) computes the loss and d loss / d logits in one visit of the bf16 (or fp32)
    logits; `fused=False` goes through `vocab_parallel_cross_entropy` plus torch reductions exactly as
    the reference composes them (:51-55).  Both give the same value.  Only the causal, non-prefix
    normalisation (default_cfg.py:220-222) is built.
    """

    def __init__(self, loss_on_targets_only=False, reweight_loss_based_on_position_frequency=False, is_prefix=True,
                 cut_size=None, fused=True, **kwargs):
        self.loss_on_targets_only = loss_on_targets_only
        self.reweight_loss_based_on_position_frequency = reweight_loss_based_on_position_frequency
        self.is_prefix = is_prefix
        self.cut_size = cut_size
        self.fused = fused

    def get_expected_number_of_tokens(self, labels, loss_mask):
        if self.is_prefix:
            raise NotImplementedError("prefix-LM normalisation is not part of the causal llama step")
        ignore_mask = labels == IGNORE_INDEX
        loss_mask = loss_mask.view(-1) * (~ignore_mask.view(-1))
        return loss_mask.sum(), loss_mask

    def __call__(self, output, labels):
        labels, loss_mask = labels[0], labels[1]
        if self.is_prefix:
            raise NotImplementedError("prefix-LM normalisation is not part of the causal llama step")
        if self.fused:
            return F_.fused_cross_entropy_loss(output, labels, loss_mask, self.cut_size, IGNORE_INDEX)
        losses = vocab_parallel_cross_entropy(output.contiguous(), labels, self.cut_size)
        expected_number_of_tokens, loss_mask = self.get_expected_number_of_tokens(labels, loss_mask)
        return torch.sum(losses.view(-1) * loss_mask) / expected_number_of_tokens
