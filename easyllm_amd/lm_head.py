"""Untied LM head (reference: llama/lm_head.py:49-104; the LoRA branch :10-46 is out of scope)."""
from . import dist_env
from . import functional as F_
from .word_embedings import EmbeddingPipe


def parallel_lm_logits(input_, word_embeddings_weight, parallel_output, bias=None, sequence_parallel=False):
    """logits = input @ W^T with W [V, h]; TP=1 so no gather is needed either way (:68-71)."""
    if sequence_parallel:
        input_parallel = dist_env.gather_from_sequence_parallel_region(input_, tensor_parallel_output_grad=True)
    else:
        input_parallel = dist_env.copy_to_tensor_model_parallel_region(input_)
    logits_parallel = F_.linear(input_parallel, word_embeddings_weight)
    if bias is not None:
        logits_parallel = F_.bias_add(logits_parallel, bias)
    if parallel_output:
        return logits_parallel
    return dist_env.gather_from_tensor_model_parallel_region(logits_parallel)


class EmbedddingPipeNoTied(EmbeddingPipe):
    def __init__(self, *args, parallel_output=True, **kwargs):
        super().__init__(*args, **kwargs)
        self.parallel_output = parallel_output

    def forward(self, lm_output, **kwargs):
        return parallel_lm_logits(lm_output, self.word_embeddings_weight, self.parallel_output,
                                  sequence_parallel=self.sequence_parallel)
