"""torch.autograd.Function wrappers that route forward AND backward through the HIP kernels.

Backward runs on PyTorch's autograd worker thread; the C ABI is re-entrant and every launch goes to
the current HIP stream, so nothing else is needed for that.

Weight gradients: if a parameter carries an fp32 ``main_grad`` buffer (Megatron's gradient
accumulation fusion; the reference leaves this to DeepSpeed's bf16 optimizer), the gradient is
accumulated straight into it by the kernel and autograd receives ``None``; otherwise a bf16
gradient is returned as usual.  ``param.main_grad_fresh = True`` makes the next write overwrite the
buffer instead of adding to it (a zero_grad without a memset).
"""
import torch

from . import kernels as K


def _main_grad_target(param):
    """(buffer or None, accumulate flag) for a parameter, consuming its 'fresh' mark."""
    mg = getattr(param, "main_grad", None)
    if mg is None:
        return None, False
    fresh = getattr(param, "main_grad_fresh", False)
    if fresh:
        param.main_grad_fresh = False
    return mg, not fresh


# --------------------------------------------------------------------------------------------
# linear: base_modules/layers/column_parallel_linear.py:13-106, row_parallel_linear.py:113
# --------------------------------------------------------------------------------------------
class LinearFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight):
        x2d = x.reshape(-1, x.shape[-1])
        y = K.linear_fwd(x2d, weight)
        ctx.save_for_backward(x, weight)
        return y.view(*x.shape[:-1], weight.shape[0])

    @staticmethod
    def backward(ctx, dy):
        x, weight = ctx.saved_tensors
        dy2d = dy.reshape(-1, dy.shape[-1])
        if not dy2d.is_contiguous():
            dy2d = dy2d.contiguous()
        dx = None
        if ctx.needs_input_grad[0]:
            dx = K.linear_dgrad(dy2d, weight).view(x.shape)
        dw = None
        if ctx.needs_input_grad[1]:
            x2d = x.reshape(-1, x.shape[-1])
            mg, acc = _main_grad_target(weight)
            if mg is not None:
                K.linear_wgrad(dy2d, x2d, out=mg, accumulate=acc)
            else:
                dw = K.linear_wgrad(dy2d, x2d)
        return dx, dw


def linear(x, weight):
    return LinearFunction.apply(x, weight)


class FanOutLinearFunction(torch.autograd.Function):
    """One input through several bias-free linears (q/k/v, or gate/up): y_i = x W_i^T.  The input gradient
    sum_i dy_i W_i is one GEMM whose reduction runs over all (dy_i, W_i) pairs (fp32 sum, one rounding) instead of one
    matmul per linear plus add kernels."""

    @staticmethod
    def forward(ctx, x, *weights):
        x2d = x.reshape(-1, x.shape[-1])
        ctx.save_for_backward(x, *weights)
        return tuple(K.linear_fwd(x2d, w).view(*x.shape[:-1], w.shape[0]) for w in weights)

    @staticmethod
    def backward(ctx, *dys):
        x, *weights = ctx.saved_tensors
        x2d = x.reshape(-1, x.shape[-1])
        dx = None
        grads = []
        dy2ds = []
        for dy in dys:
            if dy is None:
                dy2ds.append(None)
                continue
            dy2d = dy.reshape(-1, dy.shape[-1])
            dy2ds.append(dy2d if dy2d.is_contiguous() else dy2d.contiguous())
        if ctx.needs_input_grad[0]:
            pairs = [(dy2d, w) for dy2d, w in zip(dy2ds, weights) if dy2d is not None]
            if pairs:
                dx = K.linear_dgrad_multi([a for a, _ in pairs], [b for _, b in pairs])
        for i, (dy2d, w) in enumerate(zip(dy2ds, weights)):
            if dy2d is None:
                grads.append(None)
                continue
            dw = None
            if ctx.needs_input_grad[1 + i]:
                mg, acc = _main_grad_target(w)
                if mg is not None:
                    K.linear_wgrad(dy2d, x2d, out=mg, accumulate=acc)
                else:
                    dw = K.linear_wgrad(dy2d, x2d)
            grads.append(dw)
        return (None if dx is None else dx.view(x.shape),) + tuple(grads)


def fan_out_linear(x, *weights):
    return FanOutLinearFunction.apply(x, *weights)


class BiasAddFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, bias):
        ctx.bias = bias
        return K.bias_add(x.contiguous(), bias)

    @staticmethod
    def backward(ctx, dy):
        mg, acc = _main_grad_target(ctx.bias)
        db = K.bias_grad(dy.contiguous(), main_grad=mg, accumulate=acc)
        return dy, db


def bias_add(x, bias):
    return BiasAddFunction.apply(x, bias)


# --------------------------------------------------------------------------------------------
# RMSNorm (+ fused residual add): base_modules/layers/fused_layer_norm.py:49-71, transformer.py:786
# --------------------------------------------------------------------------------------------
class RMSNormFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, eps):
        xc = x.contiguous()
        y, rstd, _ = K.rmsnorm_fwd(xc, weight, eps)
        ctx.save_for_backward(xc, weight, rstd)
        return y

    @staticmethod
    def backward(ctx, dy):
        x, weight, rstd = ctx.saved_tensors
        mg, acc = _main_grad_target(weight)
        dx, dw = K.rmsnorm_bwd(dy.contiguous(), x, weight, rstd, main_grad=mg, accumulate=acc)
        return dx, dw, None


class AddRMSNormFunction(torch.autograd.Function):
    """(x, residual) -> (sum, rmsnorm(sum) * w): the residual add and the norm that follows it."""

    @staticmethod
    def forward(ctx, x, residual, weight, eps):
        y, rstd, s = K.rmsnorm_fwd(x.contiguous(), weight, eps, residual=residual.contiguous())
        ctx.save_for_backward(s, weight, rstd)
        return s, y

    @staticmethod
    def backward(ctx, dsum, dy):
        s, weight, rstd = ctx.saved_tensors
        mg, acc = _main_grad_target(weight)
        dx, dw = K.rmsnorm_bwd(dy.contiguous(), s, weight, rstd, dresidual=dsum.contiguous(), main_grad=mg, accumulate=acc)
        return dx, dx, dw, None


class RMSNormPassFunction(torch.autograd.Function):
    """x -> (x, rmsnorm(x) * w): the pre-norm block keeps x as its residual, so the gradient arriving on the
    residual branch is added inside the norm's backward kernel instead of by a separate add."""

    @staticmethod
    def forward(ctx, x, weight, eps):
        xc = x.contiguous()
        y, rstd, _ = K.rmsnorm_fwd(xc, weight, eps)
        ctx.save_for_backward(xc, weight, rstd)
        return xc.view_as(xc), y

    @staticmethod
    def backward(ctx, dres, dy):
        x, weight, rstd = ctx.saved_tensors
        mg, acc = _main_grad_target(weight)
        dx, dw = K.rmsnorm_bwd(dy.contiguous(), x, weight, rstd, dresidual=None if dres is None else dres.contiguous(),
                               main_grad=mg, accumulate=acc)
        return dx, dw, None


def rmsnorm(x, weight, eps):
    return RMSNormFunction.apply(x, weight, eps)


def rmsnorm_pass(x, weight, eps):
    return RMSNormPassFunction.apply(x, weight, eps)


def add_rmsnorm(x, residual, weight, eps):
    return AddRMSNormFunction.apply(x, residual, weight, eps)


# --------------------------------------------------------------------------------------------
# SwiGLU: llama/transformer.py:220-222
# --------------------------------------------------------------------------------------------
class SwiGLUFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, gate, up):
        ctx.save_for_backward(gate, up)
        return K.swiglu_fwd(gate, up)

    @staticmethod
    def backward(ctx, dout):
        gate, up = ctx.saved_tensors
        return K.swiglu_bwd(dout.contiguous(), gate, up)


def swiglu(gate, up):
    return SwiGLUFunction.apply(gate.contiguous(), up.contiguous())


# --------------------------------------------------------------------------------------------
# rotary embedding: llama/positional_embeddings.py:105-122
# --------------------------------------------------------------------------------------------
class RotaryFunction(torch.autograd.Function):
    """x [s, b, heads, d] -> rotated copy; backward rotates the gradient by the negative angle."""

    @staticmethod
    def forward(ctx, x, cos, sin, position_ids):
        ctx.save_for_backward(cos, sin, position_ids)
        return K.rope_apply(x, cos, sin, position_ids)

    @staticmethod
    def backward(ctx, dy):
        cos, sin, position_ids = ctx.saved_tensors
        if dy.stride(3) != 1 or dy.stride(2) != dy.shape[3]:
            dy = dy.contiguous()
        return K.rope_apply(dy, cos, sin, position_ids, backward=True), None, None, None


def apply_rotary(x, cos, sin, position_ids=None):
    return RotaryFunction.apply(x, cos, sin, position_ids)


class RotaryPairFunction(torch.autograd.Function):
    """(q, k) -> rotated copies in one launch; backward rotates both gradients by the negative angle in one launch."""

    @staticmethod
    def forward(ctx, q, k, cos, sin, position_ids):
        ctx.save_for_backward(cos, sin, position_ids)
        return K.rope_apply_pair(q, k, cos, sin, position_ids)

    @staticmethod
    def backward(ctx, dq, dk):
        cos, sin, position_ids = ctx.saved_tensors
        if dq.stride(3) != 1 or dq.stride(2) != dq.shape[3]:
            dq = dq.contiguous()
        if dk.stride(3) != 1 or dk.stride(2) != dk.shape[3]:
            dk = dk.contiguous()
        gq, gk = K.rope_apply_pair(dq, dk, cos, sin, position_ids, backward=True)
        return gq, gk, None, None, None


def apply_rotary_pair(q, k, cos, sin, position_ids=None):
    return RotaryPairFunction.apply(q, k, cos, sin, position_ids)


# --------------------------------------------------------------------------------------------
# attention: llama/transformer.py:83-143
# --------------------------------------------------------------------------------------------
class FlashAttnFunction(torch.autograd.Function):
    """q [s, b, nq, d], k/v [s, b, nk, d] -> [s, b, nq, d]; causal inside each document."""

    @staticmethod
    def forward(ctx, q, k, v, cu_seqlens, scale):
        out, lse = K.attn_fwd(q, k, v, cu_seqlens, scale)
        ctx.save_for_backward(q, k, v, out, lse, cu_seqlens)
        ctx.scale = scale
        return out

    @staticmethod
    def backward(ctx, dout):
        q, k, v, out, lse, cu_seqlens = ctx.saved_tensors
        if dout.stride(3) != 1 or dout.stride(2) != dout.shape[3]:
            dout = dout.contiguous()
        dq, dk, dv = K.attn_bwd(q, k, v, out, dout, lse, cu_seqlens, ctx.scale)
        return dq, dk, dv, None, None


def flash_attention(q, k, v, cu_seqlens=None, scale=None):
    return FlashAttnFunction.apply(q, k, v, cu_seqlens, scale)


class RowsGatherFunction(torch.autograd.Function):
    """x [s, b, heads, d] -> [s', b', heads, d] whose rows (in (b s) order) are x's rows picked by `idx` (zeros where idx
    is negative).  `idx_back` is the inverse selection: the gradient is the same gather the other way round.  With the
    indices of `kernels.mask_compact` this is unpad_input / pad_input of llama/transformer.py:121-141."""

    @staticmethod
    def forward(ctx, x, idx, idx_back, out_sb):
        ctx.save_for_backward(idx_back)
        ctx.in_sb = (x.shape[0], x.shape[1])
        return K.rows_gather(x, idx, out_sb)

    @staticmethod
    def backward(ctx, dy):
        (idx_back,) = ctx.saved_tensors
        if dy.stride(3) != 1 or dy.stride(2) != dy.shape[3]:
            dy = dy.contiguous()
        return K.rows_gather(dy, idx_back, ctx.in_sb), None, None, None


def flash_attention_unpadded(q, k, v, key_padding_mask, scale=None):
    """Attention over the tokens a [b, s] key-padding mask keeps (llama/transformer.py:117-141): every batch row is
    compressed to its kept tokens, which attend causally among themselves; dropped positions come back as zero rows."""
    s, b = q.shape[0], q.shape[1]
    idx, inv, cu = K.mask_compact(key_padding_mask.contiguous())
    n = s * b
    qc = RowsGatherFunction.apply(q, idx, inv, (n, 1))
    kc = RowsGatherFunction.apply(k, idx, inv, (n, 1))
    vc = RowsGatherFunction.apply(v, idx, inv, (n, 1))
    oc = FlashAttnFunction.apply(qc, kc, vc, cu, scale)
    return RowsGatherFunction.apply(oc, inv, idx, (s, b))


# --------------------------------------------------------------------------------------------
# embedding: base_modules/layers/vocab_parallel_emb.py:106-137
# --------------------------------------------------------------------------------------------
class EmbeddingFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, ids, weight):
        ids = ids.contiguous()
        out, flag = K.embed_gather(ids, weight)
        ctx.save_for_backward(ids, weight)
        ctx.mark_non_differentiable(flag)
        return out, flag

    @staticmethod
    def backward(ctx, dout, _dflag):
        ids, weight = ctx.saved_tensors
        mg, acc = _main_grad_target(weight)
        if mg is not None:
            K.embed_scatter_add(ids, dout.contiguous(), mg, accumulate=acc)
            return None, None
        buf = torch.empty(weight.shape, dtype=torch.float32, device=weight.device)
        K.embed_scatter_add(ids, dout.contiguous(), buf, accumulate=False)
        return None, K.cast_f32_to_bf16(buf)


def _raise_for_id_flag(bad, ids, num_embeddings):
    if isinstance(num_embeddings, tuple):  # ("position", table length): the rotary tables' index check
        if bad:
            raise IndexError("position id outside the rotary table [0, %d)" % num_embeddings[1])
        return
    if bad & 1:
        raise ValueError("There is an input id in the input that is greater than the highest possible input id.\n"
                         "Input: {}\nnum_embeddings: {}".format(ids, num_embeddings))
    if bad & 2:
        raise IndexError("negative token id in the input")


# "sync": the check blocks on the gather, like the reference's host-side comparison (:107-109).
# "deferred": the flag is copied to pinned host memory behind the gather and examined at the next
# embedding call or flush_input_checks(); the launch queue never drains, the error surfaces one call late.
_INPUT_CHECK = "sync"
_PENDING_CHECKS = []
CAPTURED_ID_FLAGS = []


def set_input_check(mode):
    assert mode in ("sync", "deferred"), mode
    global _INPUT_CHECK
    flush_input_checks()
    _INPUT_CHECK = mode


def flush_input_checks(wait=True):
    """Raise for any earlier embedding call whose out-of-range flag has arrived (all of them with wait=True)."""
    while _PENDING_CHECKS:
        ev, host, ids, n = _PENDING_CHECKS[0]
        if not wait and not ev.query():
            return
        ev.synchronize()
        _PENDING_CHECKS.pop(0)
        _raise_for_id_flag(int(host.item()), ids, n)


def _dispatch_flag(flag, ids, limit_tag):
    """Examines a device flag according to the input-check mode (see set_input_check)."""
    if torch.cuda.is_current_stream_capturing():
        CAPTURED_ID_FLAGS.append((flag, limit_tag))
        return
    if _INPUT_CHECK == "deferred":
        flush_input_checks(wait=False)
        host = torch.empty(1, dtype=torch.int32, pin_memory=True)
        host.copy_(flag, non_blocking=True)
        ev = torch.cuda.Event()
        ev.record()
        _PENDING_CHECKS.append((ev, host, ids, limit_tag))
        return
    _raise_for_id_flag(int(flag.item()), ids, limit_tag)


def check_position_ids(position_ids, table_len):
    """IndexError for a position id outside [0, table_len), as indexing the reference's cos / sin tables would give
    (positional_embeddings.py:109-117); sync or deferred like the token-id check."""
    _dispatch_flag(K.ids_in_range_flag(position_ids.contiguous(), table_len), position_ids, ("position", int(table_len)))


def embedding(ids, weight):
    """Row gather; raises ValueError for an id >= vocab like the reference (:107-109)."""
    out, flag = EmbeddingFunction.apply(ids, weight)
    # inside a graph capture nothing may synchronise: the flag tensor is handed to whoever captures (runner.GraphedStep),
    # which reads it back after each replay
    _dispatch_flag(flag, ids, weight.shape[0])
    return out


# --------------------------------------------------------------------------------------------
# layout / dtype plumbing: llama/llama.py:145-188
# --------------------------------------------------------------------------------------------
class Transpose01Function(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x):
        return K.transpose01(x.contiguous())

    @staticmethod
    def backward(ctx, dy):
        return K.transpose01(dy.contiguous())


def transpose01(x):
    """[d0, d1, ...] -> contiguous [d1, d0, ...]; a free view when either extent is 1."""
    if x.shape[0] == 1 or x.shape[1] == 1:
        return x.contiguous().view((x.shape[1], x.shape[0]) + tuple(x.shape[2:]))
    return Transpose01Function.apply(x)


class AddFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, a, b):
        return K.add(a.contiguous(), b.contiguous())

    @staticmethod
    def backward(ctx, dy):
        return dy, dy


def add(a, b):
    return AddFunction.apply(a, b)


class ToFp32Function(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x):
        return K.cast_bf16_to_f32(x.contiguous())

    @staticmethod
    def backward(ctx, dy):
        return K.cast_f32_to_bf16(dy.contiguous())


def to_fp32(x):
    return ToFp32Function.apply(x)


# --------------------------------------------------------------------------------------------
# loss: base_modules/functions/cross_entropy.py:24-117, llama/losses.py:20-56
# --------------------------------------------------------------------------------------------
class VocabParallelCrossEntropyFunction(torch.autograd.Function):
    """Per-token loss with the reference's semantics (no masking, no reduction)."""

    @staticmethod
    def forward(ctx, logits, target, cut_size):
        logits = logits.contiguous()
        target = target.contiguous()
        loss, lse = K.ce_fwd(logits, target, cut_size or 0)
        ctx.save_for_backward(logits, target, lse)
        ctx.cut_size = cut_size or 0
        return loss

    @staticmethod
    def backward(ctx, grad_out):
        logits, target, lse = ctx.saved_tensors
        g = K.ce_bwd(logits, target, lse, grad_out.contiguous().float(), ctx.cut_size)
        return g, None, None


def vocab_parallel_cross_entropy(vocab_parallel_logits, target, cut_size=None):
    return VocabParallelCrossEntropyFunction.apply(vocab_parallel_logits, target, cut_size)


class FusedCrossEntropyLossFunction(torch.autograd.Function):
    """sum(loss_i * w_i) / sum(w), w = loss_mask * (label != -100), with d loss / d logits produced
    in the same visit of the logits (written to a new buffer, or over the logits when `inplace`)."""

    @staticmethod
    def forward(ctx, logits, labels, loss_mask, cut_size, ignore_index, inplace):
        logits = logits.contiguous()
        labels = labels.contiguous()
        weights, count = K.ce_prepare(labels, None if loss_mask is None else loss_mask.contiguous(), ignore_index)
        loss_rows, grad = K.ce_fused(logits, labels, weights, count, cut_size or 0, inplace=inplace)
        ctx.save_for_backward(grad)
        return K.ce_reduce(loss_rows, weights, count)

    @staticmethod
    def backward(ctx, grad_out):
        (grad,) = ctx.saved_tensors
        K.scale_by_scalar_(grad, grad_out.reshape(1).float().contiguous())
        return grad, None, None, None, None, None


def fused_cross_entropy_loss(logits, labels, loss_mask=None, cut_size=None, ignore_index=-100, inplace=False):
    return FusedCrossEntropyLossFunction.apply(logits, labels, loss_mask, cut_size, ignore_index, inplace)
