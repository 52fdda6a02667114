"""Rotary position embedding, host side (reference: llama/positional_embeddings.py:5-36, 94-122).

`inv_freq` is a registered buffer exactly as in the reference (it appears in the state dict as
`...self_attn.rotary_emb.inv_freq`).  The cos/sin cache is kept as fp32 half tables [S, d/2] -- the
reference rounds its tables to bf16 when precision is bf16 (:33-35); keeping fp32 is closer to the
exact rotation and is what the parity tests compare against.
"""
import torch

from . import functional as F_
from . import kernels as K


class RotaryEmbedding(torch.nn.Module):
    def __init__(self, dim, base=10000, precision=torch.half, scale_factor=1.0):
        super().__init__()
        inv_freq = 1.0 / (base ** (torch.arange(0, dim, 2).float() / dim))
        self.register_buffer("inv_freq", inv_freq)
        self.dim = dim
        self.max_seq_len_cached = None
        self.cos_half = None
        self.sin_half = None
        self.precision = precision
        self.scale_factor = scale_factor

    def tables(self, seq_len, device):
        """fp32 (cos, sin) half tables [>= seq_len, dim/2] on `device`, built by the HIP table kernel."""
        if self.max_seq_len_cached is None or seq_len > self.max_seq_len_cached or self.cos_half.device != device:
            inv = self.inv_freq.to(device=device, dtype=torch.float32).contiguous()
            self.cos_half, self.sin_half = K.rope_table(inv, int(seq_len), self.scale_factor)
            self.max_seq_len_cached = int(seq_len)
        return self.cos_half, self.sin_half

    def forward(self, x, seq_dim=1, seq_len=None):
        """Reference-shaped return value: (cos, sin) of shape [seq_len, 1, dim] in `precision`."""
        if seq_len is None:
            seq_len = x.shape[seq_dim]
        c, s = self.tables(seq_len, x.device)
        cos = torch.cat((c[:seq_len], c[:seq_len]), dim=-1)[:, None, :]
        sin = torch.cat((s[:seq_len], s[:seq_len]), dim=-1)[:, None, :]
        if self.precision == torch.bfloat16:
            cos, sin = cos.bfloat16(), sin.bfloat16()
        return cos, sin


def apply_rotary_pos_emb(q, k, cos_half, sin_half, position_ids=None):
    """q [s, b, nq, d], k [s, b, nk, d] -> rotated (q, k); position_ids int64 [b, s] or None
    (positions = sequence index), cf. apply_rotary_pos_emb_torch (:105-122)."""
    return F_.apply_rotary_pair(q, k, cos_half, sin_half, position_ids)
