"""Token embedding stage (reference: llama/word_embedings.py:11-177)."""
import torch

from . import dist_env
from . import functional as F_
from .layers import VocabParallelEmbedding, get_initializer_from_cfg, get_torch_dtype


class Embedding(torch.nn.Module):
    def __init__(self, vocab_size, hidden_size, embedding_dropout_prob, num_tokentypes=0, position_embedding_type=None,
                 max_position_embeddings=None, params_dtype=None, pretrain_causal_attention=False, use_bnb_optimizer=False,
                 use_cpu_initialization=False, initializer=None, sequence_parallel=False):
        super().__init__()
        self.hidden_size = hidden_size
        self.init_method = get_initializer_from_cfg(initializer)
        self.num_tokentypes = num_tokentypes
        self.position_embedding_type = position_embedding_type
        self.pretrain_causal_attention = pretrain_causal_attention
        if position_embedding_type == "absolute":
            raise NotImplementedError("learned absolute positions are not used by the llama configs (rotary)")
        assert embedding_dropout_prob == 0, "embedding dropout is 0 in every llama config"
        self.word_embeddings = VocabParallelEmbedding(vocab_size, hidden_size, init_method=self.init_method,
                                                      use_bnb_optimizer=use_bnb_optimizer,
                                                      use_cpu_initialization=use_cpu_initialization,
                                                      params_dtype=get_torch_dtype(params_dtype))
        self.position_embeddings = None
        self.sequence_parallel = sequence_parallel

    def forward(self, input_ids, position_ids):
        embeddings = self.word_embeddings(input_ids)  # [b, s, h]
        if self.sequence_parallel:
            embeddings = dist_env.scatter_to_sequence_parallel_region(embeddings)
        return embeddings


class EmbeddingPipe(Embedding):
    def forward(self, inputs, **kwargs):
        input_ids, position_ids, attention_mask = inputs[0], inputs[1], inputs[2]
        embeddings = super().forward(input_ids, position_ids)
        if len(inputs) == 4:
            # the layers index their rotary tables (one row per sequence position) with these ids
            F_.check_position_ids(position_ids, input_ids.shape[1])
            return embeddings, attention_mask, inputs[3], position_ids
        # with a 3-tuple the mask and the position ids are dropped here, as in the reference (:169-172)
        return embeddings

    @property
    def word_embeddings_weight(self):
        return self.word_embeddings.weight
