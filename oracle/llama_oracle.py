"""fp32 CPU restatement of the reference's Megatron llama decoder-layer training step (TP=1).

TEST INFRASTRUCTURE ONLY -- the checker, never the thing measured or shipped.  Imported by
``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py``; the product
package never imports it.

Every function cites the reference lines (relative to ``/root/reference``) it restates.  The
reference cannot run here (DeepSpeed / flash-attn are hard imports and absent) and its test suite
holds no golden vectors for this path, so each function is pinned in ``tests/test_oracle.py``
against library routines, closed forms and invariants:

  embedding ............ pinned (``torch.nn.functional.embedding``, index_add brute force)
  rmsnorm .............. pinned (``F.rms_norm``, scale invariance, fp64 gradcheck of the closed-form bwd)
  linear ............... pinned (``F.linear``)
  rope ................. pinned (complex-rotation closed form, relative-position property,
                                transformers' ``apply_rotary_pos_emb``)
  attention ............ pinned (``F.scaled_dot_product_attention`` causal + GQA, per-document split,
                                brute-force python loops on tiny inputs; the key-padding-mask form against a
                                brute-force loop over kept tokens and, for right-padded rows, the truncated rows)
  swiglu ............... pinned (``F.silu``, closed-form derivative vs autograd)
  layer / model wiring . pinned (``transformers.LlamaForCausalLM`` built from a local config, live and through the
                                committed fixture tests/golden/hf_llama_tiny.npz: loss, logits, every gradient)
  cross entropy ........ pinned (``F.cross_entropy``, uniform-logits ln V, shift invariance)
  dynamic-ckpt rule .... pinned (table-driven known answers written from the reference text)
  packed inputs ........ pinned (hand-worked known answers)
  sample locations ..... pinned (the reference's own helpers.cpp compiled into oracle/_ref by oracle/build_ref.py, and
                                slicing the concatenated token stream by brute force)
  bf16-storage mode .... pinned (storage off is bit-identical to the fp32 functions; the rounding helper equals
                                ``x.bfloat16().float()`` in both directions; a linear chain worked by hand)
  optimizer step ....... pinned (``torch.optim.AdamW`` over several steps with and without weight decay,
                                ``torch.nn.utils.clip_grad_norm_``); apex / DeepSpeed themselves are absent, so
                                their rounding order inside the update is parity unpinned

Parity unpinned (defined by code that is neither under /root/reference nor installed): DeepSpeed's
micro-batch loss scaling / bf16-optimizer accumulation / checkpoint internals, and flash-attn 2.2.5's
internal rounding points.  Only "recompute gives the same numbers" is restated for the former; for
the latter the fp32 definition below is the target, within the stated bf16 tolerances.

All math is done in the dtype of the inputs (fp32 by default; fp64 for gradcheck).
"""
import math

import numpy as np
import torch

IGNORE_INDEX = -100  # llm/data/nlp_dataset.py:20


# --------------------------------------------------------------------------------------------
# storage rounding of the reference's bf16 path
# --------------------------------------------------------------------------------------------
class _RoundTrip(torch.autograd.Function):
    """Rounds a tensor to `dtype` and back, and does the same to the gradient that flows back through
    it: a tensor the reference materialises in bf16 has a bf16 gradient as well."""

    @staticmethod
    def forward(ctx, x, dtype):
        ctx.dtype = dtype
        return x.to(dtype).to(x.dtype)

    @staticmethod
    def backward(ctx, g):
        return g.to(ctx.dtype).to(g.dtype), None


def stored(x, storage_dtype=None):
    """`x` as the reference's 16-bit path holds it in memory: all arithmetic stays in the dtype of `x`
    (fp32), only the result is rounded to `storage_dtype` (None: no rounding, `x` itself is returned)."""
    if storage_dtype is None:
        return x
    return _RoundTrip.apply(x, storage_dtype)


# --------------------------------------------------------------------------------------------
# B. embedding   (base_modules/layers/vocab_parallel_emb.py:106-137, TP=1 branch)
# --------------------------------------------------------------------------------------------
def embedding(ids, weight):
    if bool((ids >= weight.shape[0]).any()):  # vocab_parallel_emb.py:107-109
        raise ValueError("There is an input id in the input that is greater than the highest possible input id.")
    return weight[ids]  # F.embedding with no padding_idx / max_norm == row gather (:124-127)


def embedding_bwd(ids, grad_out, vocab_size):
    """Scatter-add of the row gradients into a zero [V, h] matrix (autograd of F.embedding)."""
    gw = torch.zeros(vocab_size, grad_out.shape[-1], dtype=grad_out.dtype)
    gw.index_add_(0, ids.reshape(-1), grad_out.reshape(-1, grad_out.shape[-1]))
    return gw


# --------------------------------------------------------------------------------------------
# D. RMSNorm   (base_modules/layers/fused_layer_norm.py:43-47,56-71; fp32-accumulate form)
# --------------------------------------------------------------------------------------------
def rmsnorm(x, w, eps=1e-6):
    return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w


def rmsnorm_bwd(x, w, dy, eps=1e-6):
    """Closed-form backward: returns (dx, dw)."""
    h = x.shape[-1]
    rstd = torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)
    xhat = x * rstd
    g = dy * w
    dx = rstd * (g - xhat * (g * xhat).sum(-1, keepdim=True) / h)
    dw = (dy * xhat).reshape(-1, h).sum(0)
    return dx, dw


# --------------------------------------------------------------------------------------------
# E/F/L. linears   (column_parallel_linear.py:42,68,99-100; row_parallel_linear.py:113; lm_head.py:62)
# --------------------------------------------------------------------------------------------
def linear(x, w, b=None):
    y = x @ w.t()
    return y if b is None else y + b


def linear_bwd(x, w, dy, has_bias=False):
    dx = dy @ w  # column_parallel_linear.py:68
    dy2 = dy.reshape(-1, dy.shape[-1])
    x2 = x.reshape(-1, x.shape[-1])
    dw = dy2.t() @ x2  # :99
    db = dy2.sum(0) if has_bias else None  # :100
    return dx, dw, db


# --------------------------------------------------------------------------------------------
# G. rotary embedding   (llama/positional_embeddings.py:7-36, 94-96, 105-122)
# --------------------------------------------------------------------------------------------
def rope_inv_freq(dim, base=10000.0, dtype=torch.float32):
    return 1.0 / (base ** (torch.arange(0, dim, 2).float() / dim)).to(dtype)  # :9


def rope_cos_sin(positions, dim, base=10000.0, scale_factor=1.0, dtype=torch.float32):
    """cos/sin of shape positions.shape + [dim]; table math follows :21-31 (no bf16 rounding)."""
    inv_freq = rope_inv_freq(dim, base, dtype)
    t = positions.to(dtype) / scale_factor
    freqs = t[..., None] * inv_freq
    emb = torch.cat((freqs, freqs), dim=-1)
    return emb.cos(), emb.sin()


def rotate_half(x):  # :94-96
    x1, x2 = x[..., : x.shape[-1] // 2], x[..., x.shape[-1] // 2:]
    return torch.cat((-x2, x1), dim=-1)


def apply_rope(x, cos, sin):  # :121  (x [..., heads, d]; cos/sin broadcast over heads)
    return x * cos + rotate_half(x) * sin


def apply_rope_bwd(dy, cos, sin):
    """Transpose of the rotation = rotation by the negative angle."""
    return dy * cos - rotate_half(dy) * sin


def positions_sb(s, b, position_ids=None):
    """[s, b] position of every token: arange(s) (:107-108) or position_ids.T (:110-113)."""
    if position_ids is None:
        return torch.arange(s)[:, None].expand(s, b)
    return position_ids.transpose(0, 1)


# --------------------------------------------------------------------------------------------
# H / H'. attention   (llama/transformer.py:83-143 semantics, :492-592 definition;
#                      fused_softmax.py:211-233; base_modules/utils.py:123-125)
# --------------------------------------------------------------------------------------------
def attention_unpadded(q, k, v, key_padding_mask, scale=None):
    """The key_padding_mask branch of FlashAttention.forward (llama/transformer.py:117-141): each batch row is compressed
    to the tokens its mask keeps (unpad_input), those attend causally among themselves in their compressed order, and the
    result is scattered back with zero rows at the dropped positions (pad_input).  key_padding_mask: bool [b, s]."""
    b, s, nq, d = q.shape
    out = torch.zeros_like(q)
    for i in range(b):
        keep = torch.nonzero(key_padding_mask[i]).reshape(-1)
        if keep.numel() == 0:
            continue
        out[i, keep] = attention(q[i:i + 1, keep], k[i:i + 1, keep], v[i:i + 1, keep], None, scale)[0]
    return out


def attention(q, k, v, cu_seqlens=None, scale=None):
    """Causal softmax(q k^T * scale) v.

    q [b, s, nq, d]; k, v [b, s, nk, d]; returns [b, s, nq, d].  Tokens are flattened to (b s)
    (transformer.py:96-98); documents are the rows of the batch (cu = arange(0,(b+1)s,s), :101) or
    the given cu_seqlens (:103), attention is causal *within* each document.  kv head of query head
    i is i // (nq // nk) (flash-attn's GQA convention, :110-115).
    """
    b, s, nq, d = q.shape
    nk = k.shape[2]
    if scale is None:
        scale = 1.0 / math.sqrt(d)  # softmax_scale=None -> 1/sqrt(d), :373-375
    if cu_seqlens is None:
        cu = list(range(0, (b + 1) * s, s))
    else:
        cu = [int(c) for c in cu_seqlens.reshape(-1).tolist()]
    qf = q.reshape(b * s, nq, d)
    kf = k.reshape(b * s, nk, d).repeat_interleave(nq // nk, dim=1)
    vf = v.reshape(b * s, nk, d).repeat_interleave(nq // nk, dim=1)
    out = torch.zeros_like(qf)
    for a, e in zip(cu[:-1], cu[1:]):
        if e <= a:
            continue
        qd = qf[a:e].transpose(0, 1)  # [nq, l, d]
        kd = kf[a:e].transpose(0, 1)
        vd = vf[a:e].transpose(0, 1)
        scores = (qd @ kd.transpose(1, 2)) * scale
        ln = e - a
        mask = torch.triu(torch.ones(ln, ln, dtype=torch.bool), diagonal=1)
        scores = scores.masked_fill(mask, torch.finfo(scores.dtype).min)  # utils.py:123-125
        probs = torch.softmax(scores, dim=-1)
        out[a:e] = (probs @ vd).transpose(0, 1)
    return out.reshape(b, s, nq, d)


# --------------------------------------------------------------------------------------------
# I. SwiGLU activation   (llama/transformer.py:220-222; glu_activations.py:56-61)
# --------------------------------------------------------------------------------------------
def swiglu(gate, up):
    return torch.nn.functional.silu(gate) * up


def swiglu_bwd(gate, up, dout):
    sig = torch.sigmoid(gate)
    dgate = dout * up * sig * (1.0 + gate * (1.0 - sig))
    dup = dout * gate * sig
    return dgate, dup


# --------------------------------------------------------------------------------------------
# J. decoder layer   (llama/transformer.py:410-491,595; :756-802)
# --------------------------------------------------------------------------------------------
def decoder_layer(x, W, prefix, cfg, position_ids=None, cu_seqlens=None, storage_dtype=None):
    """x [s, b, h] -> [s, b, h].  W maps state-dict names (llama/utils.py:158-210) to tensors.

    storage_dtype=torch.bfloat16 rounds every tensor that the reference's bf16 path writes to memory -- the output of
    each norm (fused_layer_norm.py:56-57), of each linear (column_parallel_linear.py:42, row_parallel_linear.py:113),
    of the rotation (positional_embeddings.py:121), of the attention seam (transformer.py:106-115), of silu and of its
    product with `up` (transformer.py:220-222) and of both residual adds (:786, :797) -- and their gradients, while the
    arithmetic that produces each of them stays fp32.  The rotary tables stay fp32 (the reference rounds them too,
    positional_embeddings.py:33-35; the kernels under test do not)."""
    st = lambda t: stored(t, storage_dtype)  # noqa: E731
    s, b, h = x.shape
    nq, nk, d = cfg["num_attention_heads"], cfg["num_kv_attention_heads"], cfg["head_dim"]
    eps = cfg.get("eps", 1e-6)
    a = st(rmsnorm(x, W[prefix + "input_layernorm.weight"], eps))  # :766
    if (prefix + "self_attn.wqkv.weight") in W:  # qkv_pack, :426-429 (q | k | v along the output dim)
        qkv = st(linear(a, W[prefix + "self_attn.wqkv.weight"], W.get(prefix + "self_attn.wqkv.bias")))
        q, k, v = qkv[..., : nq * d], qkv[..., nq * d: (nq + nk) * d], qkv[..., (nq + nk) * d:]
    else:
        q = st(linear(a, W[prefix + "self_attn.q_proj.weight"], W.get(prefix + "self_attn.q_proj.bias")))  # :422
        k = st(linear(a, W[prefix + "self_attn.k_proj.weight"], W.get(prefix + "self_attn.k_proj.bias")))
        v = st(linear(a, W[prefix + "self_attn.v_proj.weight"], W.get(prefix + "self_attn.v_proj.bias")))
    pos = positions_sb(s, b, position_ids)  # [s, b]
    cos, sin = rope_cos_sin(pos, d, cfg.get("rope_base", 10000.0), dtype=x.dtype)  # [s, b, d]
    q = st(apply_rope(q.reshape(s, b, nq, d), cos[:, :, None, :], sin[:, :, None, :]))  # :437-448
    k = st(apply_rope(k.reshape(s, b, nk, d), cos[:, :, None, :], sin[:, :, None, :]))
    v = v.reshape(s, b, nk, d)
    ctx = st(attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1), cu_seqlens))  # :475-490
    ctx = ctx.transpose(0, 1).reshape(s, b, nq * d)  # :491
    x1 = st(x + st(linear(ctx, W[prefix + "self_attn.o_proj.weight"])))  # :595, :786
    m = st(rmsnorm(x1, W[prefix + "post_attention_layernorm.weight"], eps))  # :787
    gate = st(linear(m, W[prefix + "mlp.gate_proj.weight"]))
    up = st(linear(m, W[prefix + "mlp.up_proj.weight"]))
    if storage_dtype is None:
        act = swiglu(gate, up)
    else:
        act = st(st(torch.nn.functional.silu(gate)) * up)  # glu_activations.py:56-61 then transformer.py:222
    return st(x1 + st(linear(act, W[prefix + "mlp.down_proj.weight"])))  # :789-797


# --------------------------------------------------------------------------------------------
# model = spec list of llama/llama.py:142-190
# --------------------------------------------------------------------------------------------
def layer_prefix(i):
    return "%d." % (i + 3)  # specs 0 cast, 1 embedding, 2 transpose, 3.. layers


def model_forward(W, cfg, tokens, position_ids=None, cu_seqlens=None, storage_dtype=None):
    """tokens i64 [b, s] -> fp32 logits [b, s, V].

    With no cu_seqlens (3-tuple input) the reference drops position_ids and the mask after the
    embedding (word_embedings.py:169-172): positions are arange(s) and attention is purely causal.
    storage_dtype: see decoder_layer; the logits are rounded as well (lm_head.py:62 produces bf16, llama.py:187-188
    widens them again for the loss).
    """
    L = cfg["num_layers"]
    if cu_seqlens is None:
        position_ids = None
    x = stored(embedding(tokens, W["1.word_embeddings.weight"]), storage_dtype)  # [b, s, h]
    x = x.transpose(0, 1).contiguous()  # llama.py:157-168
    for i in range(L):
        x = decoder_layer(x, W, layer_prefix(i), cfg, position_ids, cu_seqlens, storage_dtype)
    x = x.transpose(0, 1).contiguous()  # :175-179
    x = stored(rmsnorm(x, W["%d.weight" % (L + 4)], cfg.get("eps", 1e-6)), storage_dtype)  # :182
    return stored(linear(x, W["%d.word_embeddings.weight" % (L + 5)]), storage_dtype)  # lm_head.py:62, untied


def init_weights(cfg, seed, sigma=0.02, dtype=torch.float32, round_to_bf16=False):
    """N(0, sigma) matrices (output projections included -- the benchmark configs say plain
    N(0, 0.02)), RMSNorm weights 1; names/shapes per llama/utils.py:158-210."""
    g = torch.Generator().manual_seed(seed)
    L, h, V = cfg["num_layers"], cfg["hidden_size"], cfg["vocab_size"]
    nq, nk, d, f = cfg["num_attention_heads"], cfg["num_kv_attention_heads"], cfg["head_dim"], cfg["intermediate_size"]

    def normal(*shape):
        w = torch.randn(*shape, generator=g, dtype=torch.float32) * sigma
        if round_to_bf16:
            w = w.bfloat16().float()
        return w.to(dtype)

    W = {"1.word_embeddings.weight": normal(V, h)}
    for i in range(L):
        p = layer_prefix(i)
        W[p + "input_layernorm.weight"] = torch.ones(h, dtype=dtype)
        W[p + "self_attn.q_proj.weight"] = normal(nq * d, h)
        W[p + "self_attn.k_proj.weight"] = normal(nk * d, h)
        W[p + "self_attn.v_proj.weight"] = normal(nk * d, h)
        W[p + "self_attn.o_proj.weight"] = normal(h, nq * d)
        W[p + "post_attention_layernorm.weight"] = torch.ones(h, dtype=dtype)
        W[p + "mlp.gate_proj.weight"] = normal(f, h)
        W[p + "mlp.up_proj.weight"] = normal(f, h)
        W[p + "mlp.down_proj.weight"] = normal(h, f)
    W["%d.weight" % (L + 4)] = torch.ones(h, dtype=dtype)
    W["%d.word_embeddings.weight" % (L + 5)] = normal(V, h)
    return W


# --------------------------------------------------------------------------------------------
# M. vocab-parallel cross entropy, TP=1   (base_modules/functions/cross_entropy.py:24-112)
# --------------------------------------------------------------------------------------------
def label_masking(target, vocab_size, cut_size=None):
    """Integer part of the loss (bit-exact contract): (target_mask, masked_target), :42-53."""
    end = vocab_size - (cut_size or 0)
    target_mask = (target < 0) | (target >= end)
    masked_target = target.clone()
    masked_target[target_mask] = 0
    return target_mask, masked_target


def vocab_parallel_cross_entropy(logits, target, cut_size=None):
    """Per-token loss [b, s] (no masking: a label outside [0, V) contributes pred = 0, :65)."""
    V = logits.shape[-1]
    end = V - (cut_size or 0)
    x = logits - logits[..., :end].max(dim=-1, keepdim=True)[0]  # :31-39
    target_mask, masked_target = label_masking(target, V, cut_size)
    pred = torch.gather(x, -1, masked_target[..., None])[..., 0]  # :58-63
    pred = pred.masked_fill(target_mask, 0.0)  # :65
    sum_exp = x.exp()[..., :end].sum(-1)  # :72-77
    return sum_exp.log() - pred  # :83


def vocab_parallel_cross_entropy_bwd(logits, target, grad_out, cut_size=None):
    """Closed form of :91-112: (softmax - onehot[valid]) * grad_out, softmax normalised by the
    sum over the un-cut columns but evaluated on every column (:72-76, 86)."""
    V = logits.shape[-1]
    end = V - (cut_size or 0)
    x = logits - logits[..., :end].max(dim=-1, keepdim=True)[0]
    e = x.exp()
    g = e / e[..., :end].sum(-1, keepdim=True)
    target_mask, masked_target = label_masking(target, V, cut_size)
    g.scatter_add_(-1, masked_target[..., None], -(1.0 - target_mask.to(g.dtype))[..., None])  # :106-107
    return g * grad_out[..., None]  # :110


# --------------------------------------------------------------------------------------------
# N. CrossEntropy loss   (llama/losses.py:20-56, non-prefix branch)
# --------------------------------------------------------------------------------------------
def loss_weights(labels, loss_mask):
    """mask = loss_mask.view(-1) * (labels != -100) (:21-23) and N = mask.sum() (:45)."""
    w = loss_mask.reshape(-1).to(torch.float32) * (labels.reshape(-1) != IGNORE_INDEX).to(torch.float32)
    return w, w.sum()


def cross_entropy_loss(logits, labels, loss_mask, cut_size=None):
    losses = vocab_parallel_cross_entropy(logits.float() if logits.dtype != torch.float64 else logits,
                                          labels, cut_size)  # :51-52
    w, n = loss_weights(labels, loss_mask)
    return torch.sum(losses.reshape(-1) * w.to(losses.dtype)) / n.to(losses.dtype)  # :55


# --------------------------------------------------------------------------------------------
# K. dynamic activation-checkpoint rule   (llama/llama.py:62-73, 97-137)
# --------------------------------------------------------------------------------------------
def get_checkpoint_range(size_map, seq_len):  # :113-118
    for key in sorted(size_map.keys()):
        if seq_len <= key:
            return size_map[key]
    return -1


def checkpointed_layers(num_layers, seq_len, checkpoint_activations=True, dynamic_checkpoint=None,
                        pp_rank=0, pp_size=1):
    """List[bool] per decoder layer: is its forward re-run in backward?

    interval = checkpoint_num_layers if checkpoint_activations else 0 (:62-65): 0 => nothing is
    ever checkpointed.  start = ceil(L/pp)*pp_rank (:71-72); range = start + (-1 | k) (:67,73,135-136).
    range < start => every transformer layer (:100-102); else layer_number < range (:104-110).
    """
    if not checkpoint_activations:
        return [False] * num_layers
    start = math.ceil(num_layers / pp_size) * pp_rank
    rng = -1 + start
    if dynamic_checkpoint is not None and dynamic_checkpoint.get("enabled"):
        rng = start + get_checkpoint_range(dynamic_checkpoint["size_map"], seq_len)
    if rng < start:
        return [True] * num_layers
    return [i < rng for i in range(num_layers)]


# --------------------------------------------------------------------------------------------
# P. packed-sequence inputs   (llm/data/nlp_transforms.py:40-55; nlp_dataloader.py:172-187)
# --------------------------------------------------------------------------------------------
def get_cu_seqlens(tokens, eos_token_id):  # nlp_transforms.py:40-49
    tokens = np.asarray(tokens)
    cu = (np.where(tokens == eos_token_id)[0] + 1).tolist()
    if len(cu) == 0 or cu[-1] != len(tokens):
        cu.append(len(tokens))
    cu.insert(0, 0)
    return cu


def get_position_ids(cu_seqlens):  # :51-55
    pos = []
    for i in range(1, len(cu_seqlens)):
        pos.extend(range(cu_seqlens[i] - cu_seqlens[i - 1]))
    return pos


def flatten_cu_seqlens(cu_list, max_seq_length):  # nlp_dataloader.py:177-184
    flat = []
    for bidx, cu in enumerate(cu_list):
        c = np.minimum(np.asarray(cu, dtype=np.int64), max_seq_length) + bidx * max_seq_length
        flat.append(c if bidx == 0 else c[1:])
    return np.concatenate(flat)


def packed_doc_lengths(total, lo, hi, seed):
    """Document lengths drawn log-uniform in [lo, hi] until they cover `total` tokens (last one
    truncated) -- the synthetic packed-batch recipe of the dynamic-checkpoint workload."""
    rng = np.random.RandomState(seed)
    lens, acc = [], 0
    while acc < total:
        ln = int(round(math.exp(rng.uniform(math.log(lo), math.log(hi)))))
        ln = max(1, min(ln, total - acc))
        lens.append(ln)
        acc += ln
    return lens


# --------------------------------------------------------------------------------------------
# packed-sequence sample locations (llm/data/cores/helpers.cpp:36-122, nlp_dataset.py:424-463)
# --------------------------------------------------------------------------------------------
def build_location_idx(sizes, doc_idx, seq_length, num_epochs, tokens_per_epoch):
    """Closed form: samples of seq_length + 1 tokens overlap by one token, so sample k starts at token k * seq_length
    of the documents laid end to end in doc_idx order; row k = (position in doc_idx, offset inside that document)."""
    sizes, doc_idx = np.asarray(sizes, dtype=np.int64), np.asarray(doc_idx, dtype=np.int64)
    num_samples = (num_epochs * tokens_per_epoch - 1) // seq_length
    ends = np.cumsum(sizes[doc_idx])                                  # one past each document's last token
    starts = np.arange(num_samples + 1, dtype=np.int64) * seq_length
    where = np.searchsorted(ends, starts, side="right")               # first document whose end lies beyond the token
    before = np.concatenate(([0], ends))[where]
    return np.stack([where, starts - before], axis=1).astype(np.int32)


# --------------------------------------------------------------------------------------------
# optimizer step (apex FusedAdam in AdamW mode + DeepSpeed global-norm clipping;
# llm/utils/model/optimizer_helper.py:70-98, configs/megatron/llama_7b_sft.yaml:13,106-112)
# --------------------------------------------------------------------------------------------
def global_grad_norm(grads):
    """L2 norm over all gradient tensors."""
    return math.sqrt(sum(float((g.double() ** 2).sum()) for g in grads))


def clip_coefficient(total_norm, max_norm):
    """DeepSpeed: clip_coef = max_norm / (total_norm + 1e-6), applied only when below one."""
    if max_norm <= 0:
        return 1.0
    c = max_norm / (total_norm + 1e-6)
    return c if c < 1.0 else 1.0


def adamw_step(p, m, v, g, lr, beta1, beta2, eps, weight_decay, step, bias_correction=True):
    """One AdamW update (decoupled weight decay); returns new (p, m, v).  step counts from 1."""
    m = beta1 * m + (1.0 - beta1) * g
    v = beta2 * v + (1.0 - beta2) * g * g
    bc1 = 1.0 - beta1 ** step if bias_correction else 1.0
    bc2 = 1.0 - beta2 ** step if bias_correction else 1.0
    denom = (v / bc2).sqrt() + eps
    p = p - lr * ((m / bc1) / denom + weight_decay * p)
    return p, m, v


# --------------------------------------------------------------------------------------------
# algorithmic FLOPs of one fwd+bwd step (causal attention counts the lower triangle only)
# --------------------------------------------------------------------------------------------
def step_flops(cfg, b, s, doc_lens=None):
    T = b * s
    L, h, V = cfg["num_layers"], cfg["hidden_size"], cfg["vocab_size"]
    nq, nk, d, f = cfg["num_attention_heads"], cfg["num_kv_attention_heads"], cfg["head_dim"], cfg["intermediate_size"]
    proj = 2 * T * h * nq * d + 4 * T * h * nk * d + 2 * T * nq * d * h
    mlp = 6 * T * h * f
    if doc_lens is None:
        doc_lens = [s] * b
    attn = 2 * nq * d * sum(l * l for l in doc_lens)
    head = 2 * T * h * V
    return 3 * (L * (proj + mlp + attn) + head)
