"""Integer producers of the packed-sequence inputs and the batch tuple layout the model consumes.

Reference: `get_cu_seqlens` / `get_position_ids` (llm/data/nlp_transforms.py:40-55), the per-batch
flattening of cu_seqlens in `BatchAlignCollector._pad_func` (llm/data/nlp_dataloader.py:172-187) and
the tuple layouts of `json_batch_pipe` / `flash_batch_pipe` (llm/data/nlp_batch_fn.py:131-205).
Host-side numpy/torch integer code; nothing here is in the timed region.
"""
import numpy as np
import torch

IGNORE_INDEX = -100


def get_cu_seqlens(tokens, eos_token_id):
    """Document boundaries of one packed sample: 0, the position after every EOS, and the length."""
    tokens = np.asarray(tokens)
    ends = (np.flatnonzero(tokens == eos_token_id) + 1).tolist()
    if not ends or ends[-1] != len(tokens):
        ends.append(len(tokens))
    return [0] + ends


def get_position_ids(cu_seqlens):
    """Positions restart at 0 at every document boundary."""
    out = []
    for a, e in zip(cu_seqlens[:-1], cu_seqlens[1:]):
        out.extend(range(e - a))
    return out


def flatten_cu_seqlens(cu_list, max_seq_length):
    """Per-sample boundaries -> boundaries in the flattened (b s) token order: each sample's list is
    clamped to max_seq_length and shifted by its row offset; the leading 0 of rows > 0 is dropped."""
    parts = []
    for bidx, cu in enumerate(cu_list):
        c = torch.clamp(torch.as_tensor(cu, dtype=torch.int64), max=max_seq_length) + bidx * max_seq_length
        parts.append(c if bidx == 0 else c[1:])
    return torch.cat(parts)


def flash_batch(tokens, labels, pad_token_id, cu_seqlens=None, position_ids=None):
    """((tokens, position_ids, attention_mask[, cu_seqlens]), (labels, loss_mask)) as `flash_batch_pipe` emits it."""
    attention_mask = tokens.ne(pad_token_id)
    loss_mask = attention_mask.clone()
    if cu_seqlens is None:
        s = tokens.shape[1]
        position_ids = torch.arange(s, dtype=torch.long, device=tokens.device).unsqueeze(0).expand_as(tokens)
        return (tokens, position_ids, attention_mask), (labels, loss_mask)
    return (tokens, position_ids, attention_mask, cu_seqlens), (labels, loss_mask)


def json_batch(tokens, labels, pad_token_id):
    """`json_batch_pipe` layout: float loss mask (1 except on pad tokens), positions 0..s-1, no cu_seqlens."""
    s = tokens.shape[1]
    position_ids = torch.arange(s, dtype=torch.long, device=tokens.device).unsqueeze(0).expand_as(tokens)
    loss_mask = torch.ones(tokens.shape, dtype=torch.float, device=tokens.device)
    loss_mask[tokens == pad_token_id] = 0.0
    attention_mask = None
    return (tokens, position_ids, attention_mask), (labels, loss_mask)


def packed_doc_lengths(total, lo, hi, seed):
    """Document lengths drawn log-uniform in [lo, hi] until they cover `total` tokens (last truncated)."""
    rng = np.random.RandomState(seed)
    lens, acc = [], 0
    while acc < total:
        ln = int(round(np.exp(rng.uniform(np.log(lo), np.log(hi)))))
        ln = max(1, min(ln, total - acc))
        lens.append(ln)
        acc += ln
    return lens
