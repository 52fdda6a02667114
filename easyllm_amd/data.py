"""Integer producers of the packed-sequence inputs and the batch tuple layout the model consumes.

Reference: `get_cu_seqlens` / `get_position_ids` (llm/data/nlp_transforms.py:40-55), the collator
`BatchAlignCollector` (llm/data/nlp_dataloader.py:110-187: next-token shift, padding, per-batch
flattening of cu_seqlens) and the tuple layouts of `json_batch_pipe` / `flash_batch_pipe`
(llm/data/nlp_batch_fn.py:131-205).
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


def _pad_with_alignment(items, padding_value, max_seq_length, alignment, offset_label, is_label):
    """nlp_dataloader.py:147-170: rows padded to the batch's longest item (rounded up to `alignment`, capped at
    max_seq_length); with offset_label the inputs drop their last token and the labels their first (next-token shift)."""
    new_size = -(-max(len(it) for it in items) // alignment) * alignment
    rows = []
    for it in items:
        row = torch.full((min(max_seq_length, new_size),), padding_value, dtype=torch.int64)
        o_size = it.size(0) - 1
        if offset_label:
            row[:o_size] = it[1:] if is_label else it[:-1]
        else:
            row[:o_size + 1] = it[:max_seq_length]
        rows.append(row)
    return torch.stack(rows)


def batch_align_collate(instances, pad_token_id, max_seq_length, alignment=1, ignore_idx=IGNORE_INDEX, offset_label=True,
                        pretrain=False):
    """`BatchAlignCollector.__call__` (nlp_dataloader.py:131-145): dataset items -> dict of batch tensors.  With
    `pretrain`, items carry `cu_seqlens` / `position_ids` (packed samples) and the batch gets the flattened boundaries."""
    input_ids = _pad_with_alignment([i["input_ids"] for i in instances], pad_token_id, max_seq_length, alignment, offset_label, False)
    labels = _pad_with_alignment([i["labels"] for i in instances], ignore_idx, max_seq_length, alignment, offset_label, True)
    batch = dict(input_ids=input_ids, labels=labels, attention_mask=input_ids.ne(pad_token_id))
    if pretrain:
        batch["position_ids"] = _pad_with_alignment([i["position_ids"] for i in instances], 0, max_seq_length, alignment,
                                                    offset_label, False)
        batch["cu_seqlens"] = flatten_cu_seqlens([i["cu_seqlens"] for i in instances], max_seq_length)
    return batch


def flash_batch_from(batch, pad_token_id, pretrain=False):
    """`FlashBatchFunction.__call__` (nlp_batch_fn.py:181-205) on a collated batch dict."""
    if pretrain:
        return flash_batch(batch["input_ids"].long(), batch["labels"].long(), pad_token_id, batch["cu_seqlens"], batch["position_ids"])
    return flash_batch(batch["input_ids"].long(), batch["labels"].long(), pad_token_id)


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
