"""Thin tensor-level wrappers over the C ABI (no autograd here; see functional.py).

torch is used only for device memory and the current HIP stream.  Every wrapper validates what the
kernel and its grid assume (device, dtype, contiguity) before launching.
"""
import ctypes

import torch

from . import _lib

BF16 = torch.bfloat16


def _p(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _need(cond, msg):
    if not cond:
        raise ValueError(msg)


def _bf16c(t, name):
    _need(t.is_cuda and t.dtype == BF16 and t.is_contiguous(), "%s must be a contiguous bf16 GPU tensor" % name)


# ------------------------------------------------------------------------------------- RMSNorm
def rmsnorm_fwd(x, weight, eps, residual=None):
    """x [..., h] -> (y, rstd, sum) ; sum = x + residual (bf16) when residual is given, else None."""
    _bf16c(x, "x"); _bf16c(weight, "weight")
    h = x.shape[-1]
    rows = x.numel() // h
    _need(weight.numel() == h, "weight size mismatch")
    y = torch.empty_like(x)
    rstd = torch.empty(rows, dtype=torch.float32, device=x.device)
    s = None
    if residual is not None:
        _bf16c(residual, "residual")
        _need(residual.shape == x.shape, "residual shape mismatch")
        s = torch.empty_like(x)
    _lib.call("ezl_rmsnorm_fwd", _p(x), _p(residual), _p(weight), _p(y), _p(s), _p(rstd), rows, h, float(eps), _stream())
    return y, rstd, s


def rmsnorm_bwd(dy, x, weight, rstd, dresidual=None, main_grad=None, accumulate=False, dx=None, dw=None, builtin_scratch=False):
    """Returns (dx, dw): dw is a bf16 [h] tensor, or None when it was written into main_grad (fp32).
    builtin_scratch: go through the entry point that keeps its partial sums in the library's own device array; with `dx`
    (and `dw` when there is no main_grad) passed in, the call then allocates nothing."""
    _bf16c(dy, "dy"); _bf16c(x, "x"); _bf16c(weight, "weight")
    h = x.shape[-1]
    rows = x.numel() // h
    _need(dy.shape == x.shape and rstd.numel() == rows and rstd.dtype == torch.float32, "rmsnorm_bwd: shape mismatch")
    if dresidual is not None:
        _bf16c(dresidual, "dresidual")
        _need(dresidual.shape == x.shape, "dresidual shape mismatch")
    if dx is None:
        dx = torch.empty_like(x)
    else:
        _bf16c(dx, "dx")
        _need(dx.shape == x.shape, "dx shape mismatch")
    if main_grad is None:
        if dw is None:
            dw = torch.empty(h, dtype=BF16, device=x.device)
        _bf16c(dw, "dw")
        _need(dw.numel() == h, "dw size mismatch")
    else:
        dw = None
        _need(main_grad.dtype == torch.float32 and main_grad.is_contiguous() and main_grad.numel() == h, "bad main_grad")
    if builtin_scratch:
        _lib.call("ezl_rmsnorm_bwd_noalloc", _p(dy), _p(x), _p(weight), _p(rstd), _p(dresidual), _p(dx), _p(dw), _p(main_grad),
                  1 if accumulate else 0, rows, h, _stream())
        return dx, dw
    ws_bytes = _lib.rmsnorm_bwd_workspace_bytes(rows, h)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device)
    _lib.call("ezl_rmsnorm_bwd", _p(dy), _p(x), _p(weight), _p(rstd), _p(dresidual), _p(dx), _p(dw), _p(main_grad),
              1 if accumulate else 0, _p(ws), ws_bytes, rows, h, _stream())
    return dx, dw


# ------------------------------------------------------------------------------------- SwiGLU
def swiglu_fwd(gate, up):
    _bf16c(gate, "gate"); _bf16c(up, "up")
    _need(gate.shape == up.shape, "gate/up shape mismatch")
    out = torch.empty_like(gate)
    _lib.call("ezl_swiglu_fwd", _p(gate), _p(up), _p(out), gate.numel(), _stream())
    return out


def swiglu_bwd(dout, gate, up):
    _bf16c(dout, "dout"); _bf16c(gate, "gate"); _bf16c(up, "up")
    _need(gate.shape == up.shape == dout.shape, "swiglu_bwd shape mismatch")
    dgate, dup = torch.empty_like(gate), torch.empty_like(up)
    _lib.call("ezl_swiglu_bwd", _p(dout), _p(gate), _p(up), _p(dgate), _p(dup), gate.numel(), _stream())
    return dgate, dup


# ------------------------------------------------------------------------------------- RoPE
def rope_table(inv_freq, npos, scale_factor=1.0):
    _need(inv_freq.is_cuda and inv_freq.dtype == torch.float32 and inv_freq.is_contiguous(), "inv_freq must be fp32 on the GPU")
    half = inv_freq.numel()
    cos = torch.empty(npos, half, dtype=torch.float32, device=inv_freq.device)
    sin = torch.empty_like(cos)
    _lib.call("ezl_rope_table", _p(inv_freq), _p(cos), _p(sin), npos, half, float(scale_factor), _stream())
    return cos, sin


def rope_apply(x, cos, sin, position_ids=None, backward=False, out=None):
    """x [s, b, nheads, d] (token rows may be strided, heads*d contiguous).  Returns a contiguous result
    unless `out` (may be x itself, for in-place) is given."""
    _need(x.is_cuda and x.dtype == BF16 and x.dim() == 4, "x must be a bf16 [s, b, heads, d] GPU tensor")
    s, b, nh, d = x.shape
    _need(x.stride(3) == 1 and x.stride(2) == d and (b == 1 or x.stride(0) == b * x.stride(1)),
          "rope_apply: unsupported strides")
    row_stride = x.stride(1) if b > 1 else x.stride(0)
    if out is None:
        out = torch.empty((s, b, nh, d), dtype=BF16, device=x.device)
    _need(out.stride(3) == 1 and out.stride(2) == d and (b == 1 or out.stride(0) == b * out.stride(1)),
          "rope_apply: unsupported out strides")
    out_stride = out.stride(1) if b > 1 else out.stride(0)
    if position_ids is not None:
        _need(position_ids.is_cuda and position_ids.dtype == torch.int64 and position_ids.is_contiguous()
              and tuple(position_ids.shape) == (b, s), "position_ids must be int64 [b, s]")
    _need(cos.shape == sin.shape and cos.shape[1] == d // 2 and cos.dtype == torch.float32, "bad cos/sin table")
    _lib.call("ezl_rope_apply", _p(x), _p(out), _p(cos), _p(sin), _p(position_ids), s, b, nh, d, row_stride, out_stride,
              cos.shape[0], 1 if backward else 0, _stream())
    return out


def _rope_side(x, out):
    """(row stride of x, out tensor, row stride of out) for a [s, b, heads, d] tensor with contiguous heads*d."""
    s, b, nh, d = x.shape
    _need(x.is_cuda and x.dtype == BF16 and x.dim() == 4, "x must be a bf16 [s, b, heads, d] GPU tensor")
    _need(x.stride(3) == 1 and x.stride(2) == d and (b == 1 or x.stride(0) == b * x.stride(1)), "rope_apply: unsupported strides")
    if out is None:
        out = torch.empty((s, b, nh, d), dtype=BF16, device=x.device)
    _need(out.stride(3) == 1 and out.stride(2) == d and (b == 1 or out.stride(0) == b * out.stride(1)),
          "rope_apply: unsupported out strides")
    return (x.stride(1) if b > 1 else x.stride(0)), out, (out.stride(1) if b > 1 else out.stride(0))


def rope_apply_pair(q, k, cos, sin, position_ids=None, backward=False):
    """Rotates q [s, b, nq, d] and k [s, b, nk, d] in one launch; returns contiguous results."""
    s, b, nq, d = q.shape
    _need(k.shape[0] == s and k.shape[1] == b and k.shape[3] == d, "rope_apply_pair: q / k shapes differ")
    qs, qo, qos = _rope_side(q, None)
    ks, ko, kos = _rope_side(k, None)
    if position_ids is not None:
        _need(position_ids.is_cuda and position_ids.dtype == torch.int64 and position_ids.is_contiguous()
              and tuple(position_ids.shape) == (b, s), "position_ids must be int64 [b, s]")
    _need(cos.shape == sin.shape and cos.shape[1] == d // 2 and cos.dtype == torch.float32, "bad cos/sin table")
    _lib.call("ezl_rope_apply_pair", _p(q), _p(qo), nq, qs, qos, _p(k), _p(ko), k.shape[2], ks, kos, _p(cos), _p(sin),
              _p(position_ids), s, b, d, cos.shape[0], 1 if backward else 0, _stream())
    return qo, ko


def ids_in_range_flag(ids, limit):
    """-> int32 [1] GPU flag: bit 0 set if some id >= limit, bit 1 if some id < 0."""
    _need(ids.is_cuda and ids.dtype == torch.int64 and ids.is_contiguous(), "ids must be contiguous int64 on the GPU")
    flag = torch.zeros(1, dtype=torch.int32, device=ids.device)
    _lib.call("ezl_ids_in_range", _p(ids), ids.numel(), int(limit), _p(flag), _stream())
    return flag


# ------------------------------------------------------------------------------------- embedding
def embed_gather(ids, weight):
    _need(ids.is_cuda and ids.dtype == torch.int64 and ids.is_contiguous(), "ids must be contiguous int64 on the GPU")
    _bf16c(weight, "weight")
    V, h = weight.shape
    out = torch.empty(tuple(ids.shape) + (h,), dtype=BF16, device=weight.device)
    flag = torch.zeros(1, dtype=torch.int32, device=weight.device)
    _lib.call("ezl_embed_gather", _p(ids), _p(weight), _p(out), _p(flag), ids.numel(), h, V, _stream())
    return out, flag


def embed_scatter_add(ids, dy, dweight_f32, accumulate=True):
    """dweight_f32[id] (+)= sum of the dy rows of that id, in row order.  accumulate=False overwrites the buffer: rows of
    ids that do not occur come back zero."""
    _need(ids.is_cuda and ids.dtype == torch.int64 and ids.is_contiguous(), "ids must be contiguous int64 on the GPU")
    _bf16c(dy, "dy")
    V, h = dweight_f32.shape
    _need(dweight_f32.dtype == torch.float32 and dweight_f32.is_contiguous() and dy.shape[-1] == h, "bad dweight")
    ws_bytes = _lib.embed_scatter_add_workspace_bytes(ids.numel(), V)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dy.device)
    _lib.call("ezl_embed_scatter_add", _p(ids), _p(dy), _p(dweight_f32), _p(ws), ws_bytes, ids.numel(), h, V, 1 if accumulate else 0, _stream())


# ------------------------------------------------------------------------------------- plumbing
def transpose01(x):
    _bf16c(x, "x")
    _need(x.dim() >= 3, "transpose01 needs [d0, d1, ...]")
    d0, d1 = x.shape[0], x.shape[1]
    inner = x.numel() // max(d0 * d1, 1) if d0 * d1 else int(torch.Size(x.shape[2:]).numel())
    y = torch.empty((d1, d0) + tuple(x.shape[2:]), dtype=BF16, device=x.device)
    _lib.call("ezl_transpose01", _p(x), _p(y), d0, d1, inner, _stream())
    return y


def add(a, b):
    _bf16c(a, "a"); _bf16c(b, "b")
    _need(a.shape == b.shape, "add shape mismatch")
    out = torch.empty_like(a)
    _lib.call("ezl_add", _p(a), _p(b), _p(out), a.numel(), _stream())
    return out


def cast_bf16_to_f32(x):
    _bf16c(x, "x")
    out = torch.empty(x.shape, dtype=torch.float32, device=x.device)
    _lib.call("ezl_cast_bf16_to_f32", _p(x), _p(out), x.numel(), _stream())
    return out


def cast_f32_to_bf16(x):
    _need(x.is_cuda and x.dtype == torch.float32 and x.is_contiguous(), "x must be contiguous fp32 on the GPU")
    out = torch.empty(x.shape, dtype=BF16, device=x.device)
    _lib.call("ezl_cast_f32_to_bf16", _p(x), _p(out), x.numel(), _stream())
    return out


# ------------------------------------------------------------------------------------- GEMM
def _rows_ld(t, name):
    _need(t.is_cuda and t.dtype == BF16 and t.dim() == 2 and t.stride(1) == 1 and t.stride(0) >= t.shape[1],
          "%s must be a bf16 2-D GPU tensor with unit inner stride" % name)
    return t.stride(0)


def gemm(A, B, M, N, K, lda, ldb, a_kc, b_kc, out=None, out_dtype=BF16, accumulate=False):
    return _gemm(A, B, M, N, K, lda, ldb, a_kc, b_kc, out, out_dtype, accumulate)


def _span(t):
    """Elements from the tensor's first element to one past its last (views of a wider matrix included)."""
    if t.numel() == 0:
        return 0
    return 1 + sum((n - 1) * st for n, st in zip(t.shape, t.stride()))


def _extent_ok(t, rows, cols, ld):
    """True when a [rows x cols] operand with leading dimension ld lies inside tensor t."""
    if rows == 0 or cols == 0:
        return True
    return ld >= cols and _span(t) >= (rows - 1) * ld + cols


def _gemm(A, B, M, N, K, lda, ldb, a_kc, b_kc, out, out_dtype, accumulate):
    _need(not (accumulate and out is None), "GEMM: accumulate needs the buffer to add to (out=...)")
    for t, name in ((A, "A"), (B, "B")):
        _need(t.is_cuda and t.dtype == BF16 and t.stride(-1) == 1, "GEMM operand %s must be a bf16 GPU tensor with unit inner stride" % name)
    # A is M x K stored [m][k] (a_kc) or [k][m]; B is N x K stored [n][k] (b_kc) or [k][n]
    _need(_extent_ok(A, M, K, lda) if a_kc else _extent_ok(A, K, M, lda), "GEMM: A is smaller than M x K with this leading dimension")
    _need(_extent_ok(B, N, K, ldb) if b_kc else _extent_ok(B, K, N, ldb), "GEMM: B is smaller than N x K with this leading dimension")
    if out is None:
        out = torch.empty(M, N, dtype=out_dtype, device=A.device)
    _need(out.is_cuda and out.dim() == 2 and out.stride(1) == 1 and tuple(out.shape) == (M, N), "bad GEMM output")
    _need(out.dtype in (BF16, torch.float32), "GEMM output must be bf16 or fp32")
    ws, ws_bytes = _gemm_workspace(M, N, K, A.device)
    _lib.call("ezl_gemm_bf16", _p(A), _p(B), _p(out), M, N, K, lda, ldb, out.stride(0), 1 if a_kc else 0, 1 if b_kc else 0,
              0 if out.dtype == BF16 else 1, 1 if accumulate else 0, _p(ws), ws_bytes, _stream())
    return out


def _gemm_workspace(M, N, K, device):
    """fp32 partial tiles for shapes whose last round of output tiles would leave most of the chip idle (None otherwise)."""
    nbytes = _lib.gemm_workspace_bytes(M, N, K)
    return (torch.empty(nbytes, dtype=torch.uint8, device=device), nbytes) if nbytes else (None, 0)


def linear_fwd(x2d, w):
    """y[T, out] = x[T, in] @ w[out, in]^T"""
    lda, ldb = _rows_ld(x2d, "x"), _rows_ld(w, "w")
    _need(x2d.shape[1] == w.shape[1], "linear_fwd: inner dimensions differ")
    return gemm(x2d, w, x2d.shape[0], w.shape[0], x2d.shape[1], lda, ldb, True, True)


def linear_dgrad(dy2d, w, out=None, accumulate=False):
    """dx[T, in] (=|+=) dy[T, out] @ w[out, in]"""
    lda, ldb = _rows_ld(dy2d, "dy"), _rows_ld(w, "w")
    _need(dy2d.shape[1] == w.shape[0], "linear_dgrad: inner dimensions differ")
    return gemm(dy2d, w, dy2d.shape[0], w.shape[1], w.shape[0], lda, ldb, True, False, out=out, accumulate=accumulate)


def linear_dgrad_multi(dy2ds, ws, out=None, accumulate=False):
    """dx[T, in] (=|+=) sum_i dy_i[T, out_i] @ w_i[out_i, in]: the input gradient of linears that share their input.
    One launch when the dy_i share a row stride and the w_i theirs; otherwise one accumulating GEMM per pair."""
    import ctypes
    n = len(dy2ds)
    _need(n == len(ws) and n >= 1, "linear_dgrad_multi: list lengths differ")
    _need(not (accumulate and out is None), "linear_dgrad_multi: accumulate needs the buffer to add to (out=...)")
    ldas = [_rows_ld(dy, "dy") for dy in dy2ds]
    ldbs = [_rows_ld(w, "w") for w in ws]
    T, n_in = dy2ds[0].shape[0], ws[0].shape[1]
    for dy, w in zip(dy2ds, ws):
        _need(dy.shape[1] == w.shape[0] and dy.shape[0] == T and w.shape[1] == n_in, "linear_dgrad: dimensions differ")
    if len(set(ldas)) != 1 or len(set(ldbs)) != 1 or n > 3:
        for i, (dy, w) in enumerate(zip(dy2ds, ws)):
            out = linear_dgrad(dy, w, out=out, accumulate=accumulate or i > 0)
        return out
    if out is None:
        out = torch.empty(T, n_in, dtype=BF16, device=dy2ds[0].device)
    _need(out.is_cuda and out.dim() == 2 and out.stride(1) == 1 and tuple(out.shape) == (T, n_in) and out.dtype == BF16, "bad GEMM output")
    wsp, wsp_bytes = _gemm_workspace(T, n_in, sum(w.shape[0] for w in ws), out.device)
    _lib.call("ezl_gemm_bf16_ksplit", n, (ctypes.c_void_p * n)(*[_p(dy) for dy in dy2ds]), (ctypes.c_void_p * n)(*[_p(w) for w in ws]),
              _p(out), T, n_in, (ctypes.c_int64 * n)(*[w.shape[0] for w in ws]), ldas[0], ldbs[0], out.stride(0), 1, 0, 0,
              1 if accumulate else 0, _p(wsp), wsp_bytes, _stream())
    return out


def linear_wgrad(dy2d, x2d, out=None, accumulate=False):
    """dw[out, in] (=|+=) dy[T, out]^T @ x[T, in]; `out` may be an fp32 main-grad buffer."""
    lda, ldb = _rows_ld(dy2d, "dy"), _rows_ld(x2d, "x")
    _need(dy2d.shape[0] == x2d.shape[0], "linear_wgrad: token counts differ")
    return gemm(dy2d, x2d, dy2d.shape[1], x2d.shape[1], dy2d.shape[0], lda, ldb, False, False, out=out, accumulate=accumulate)


def bias_add(x, bias):
    _bf16c(x, "x"); _bf16c(bias, "bias")
    n = x.shape[-1]
    _need(bias.numel() == n, "bias size mismatch")
    out = torch.empty_like(x)
    _lib.call("ezl_bias_add", _p(x), _p(bias), _p(out), x.numel() // n, n, _stream())
    return out


def bias_grad(dy, main_grad=None, accumulate=False):
    """Column sum of dy [rows, n]: bf16 [n], or written into an fp32 main_grad (then returns None)."""
    _bf16c(dy, "dy")
    n = dy.shape[-1]
    rows = dy.numel() // n
    ws_bytes = _lib.bias_grad_workspace_bytes(rows, n)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dy.device)
    db = None if main_grad is not None else torch.empty(n, dtype=BF16, device=dy.device)
    _lib.call("ezl_bias_grad", _p(dy), _p(db), _p(main_grad), 1 if accumulate else 0, _p(ws), ws_bytes, rows, n, _stream())
    return db


# ------------------------------------------------------------------------------------- attention
def _tok_strides(t, b):
    """(seq_stride, batch_stride) of a [s, b, heads, d] tensor whose heads*d block is contiguous."""
    _need(t.is_cuda and t.dtype == BF16 and t.dim() == 4 and t.stride(3) == 1 and t.stride(2) == t.shape[3],
          "attention tensors must be bf16 [s, b, heads, d] with contiguous heads*d")
    return t.stride(0), (t.stride(1) if b > 1 else 0)


def _cu_arg(cu_seqlens, b):
    if cu_seqlens is None:
        return None, b
    _need(cu_seqlens.is_cuda and cu_seqlens.dtype == torch.int32 and cu_seqlens.is_contiguous() and cu_seqlens.dim() == 1
          and cu_seqlens.numel() >= 2, "cu_seqlens must be a contiguous int32 GPU vector")
    return cu_seqlens, cu_seqlens.numel() - 1


def attn_fwd(q, k, v, cu_seqlens=None, scale=None):
    """q [s, b, nq, d], k/v [s, b, nk, d] -> (out [s, b, nq, d] contiguous, lse fp32 [nq, b*s])."""
    s, b, nq, d = q.shape
    nk = k.shape[2]
    _need(k.shape == v.shape and k.shape[0] == s and k.shape[1] == b and k.shape[3] == d, "attn_fwd: k/v shape mismatch")
    out = torch.empty((s, b, nq, d), dtype=BF16, device=q.device)
    lse = torch.empty((nq, b * s), dtype=torch.float32, device=q.device)
    st = []
    for t in (q, k, v, out):
        st.extend(_tok_strides(t, b))
    strides = (ctypes.c_int64 * 8)(*st)
    cu, ndocs = _cu_arg(cu_seqlens, b)
    if scale is None:
        scale = d ** -0.5
    _lib.call("ezl_attn_fwd", _p(q), _p(k), _p(v), _p(out), _p(lse), _p(cu), ndocs, b * s, s, nq, nk, d, float(scale), strides,
              _stream())
    return out, lse


def attn_bwd(q, k, v, out, dout, lse, cu_seqlens=None, scale=None):
    s, b, nq, d = q.shape
    nk = k.shape[2]
    dq = torch.empty((s, b, nq, d), dtype=BF16, device=q.device)
    dk = torch.empty((s, b, nk, d), dtype=BF16, device=q.device)
    dv = torch.empty((s, b, nk, d), dtype=BF16, device=q.device)
    delta = torch.empty((nq, b * s), dtype=torch.float32, device=q.device)
    _need(lse.dtype == torch.float32 and tuple(lse.shape) == (nq, b * s) and lse.is_contiguous(), "bad lse")
    st = []
    for t in (q, k, v, out, dout, dq, dk, dv):
        st.extend(_tok_strides(t, b))
    strides = (ctypes.c_int64 * 16)(*st)
    cu, ndocs = _cu_arg(cu_seqlens, b)
    if scale is None:
        scale = d ** -0.5
    ws_bytes = _lib.attn_bwd_workspace_bytes(b * s, ndocs, nq, nk, d)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device) if ws_bytes else None
    _lib.call("ezl_attn_bwd", _p(q), _p(k), _p(v), _p(out), _p(dout), _p(lse), _p(delta), _p(dq), _p(dk), _p(dv), _p(cu), ndocs,
              b * s, s, nq, nk, d, float(scale), strides, _p(ws), ws_bytes, _stream())
    return dq, dk, dv


# ------------------------------------------------------------------------------------- unpadding
def mask_compact(mask):
    """mask [b, s] (bool / uint8, non-zero = keep) -> (idx int32 [b*s], inv int32 [b*s], cu_seqlens int32 [b+1])."""
    _need(mask.is_cuda and mask.dim() == 2 and mask.dtype in (torch.bool, torch.uint8) and mask.is_contiguous(),
          "key padding mask must be a contiguous bool / uint8 [b, s] GPU tensor")
    b, s = mask.shape
    idx = torch.empty(b * s, dtype=torch.int32, device=mask.device)
    inv = torch.empty(b * s, dtype=torch.int32, device=mask.device)
    cu = torch.empty(b + 1, dtype=torch.int32, device=mask.device)
    _lib.call("ezl_mask_compact", _p(mask), b, s, _p(idx), _p(inv), _p(cu), _stream())
    return idx, inv, cu


def rows_gather(src, idx, out_shape_sb):
    """src [s, b, heads, d] (token strides arbitrary) read as rows in (b s) order; out [s', b', heads, d] contiguous whose
    row r (in (b' s') order) is src row idx[r], or zeros where idx[r] < 0."""
    _need(idx.is_cuda and idx.dtype == torch.int32 and idx.is_contiguous(), "idx must be a contiguous int32 GPU vector")
    s, b, nh, d = src.shape
    so, bo = out_shape_sb
    _need(idx.numel() == so * bo, "one index per output row")
    ss, sb = _tok_strides(src, b)
    out = torch.empty((so, bo, nh, d), dtype=BF16, device=src.device)
    os_, ob = _tok_strides(out, bo)
    _lib.call("ezl_rows_gather", _p(src), _p(idx), _p(out), so * bo, nh * d, s * b, s, ss, sb, so, os_, ob, _stream())
    return out


# ------------------------------------------------------------------------------------- cross entropy
_MASK_DTYPES = {torch.float32: 1, torch.bool: 2, torch.uint8: 2, torch.int64: 3, BF16: 4}


def _logits_dtype(logits):
    _need(logits.is_cuda and logits.is_contiguous() and logits.dtype in (BF16, torch.float32),
          "logits must be contiguous bf16 or fp32 on the GPU")
    return 0 if logits.dtype == BF16 else 1


def _labels(labels, rows):
    _need(labels.is_cuda and labels.dtype == torch.int64 and labels.is_contiguous() and labels.numel() == rows,
          "labels must be contiguous int64 on the GPU, one per logits row")


def ce_prepare(labels, loss_mask, ignore_index=-100):
    """-> (weights fp32 [n], count fp32 [1])"""
    n = labels.numel()
    _labels(labels, n)
    code = 0
    if loss_mask is not None:
        _need(loss_mask.is_cuda and loss_mask.is_contiguous() and loss_mask.numel() == n and loss_mask.dtype in _MASK_DTYPES,
              "loss_mask must be a contiguous GPU tensor (fp32, bool, uint8, int64 or bf16) matching labels")
        code = _MASK_DTYPES[loss_mask.dtype]
    weights = torch.empty(n, dtype=torch.float32, device=labels.device)
    count = torch.empty(1, dtype=torch.float32, device=labels.device)
    _lib.call("ezl_ce_prepare", _p(labels), _p(loss_mask), code, ignore_index, _p(weights), _p(count), n, _stream())
    return weights, count


def ce_fwd(logits, labels, cut_size=0):
    V = logits.shape[-1]
    rows = logits.numel() // V
    _labels(labels, rows)
    loss = torch.empty(labels.shape, dtype=torch.float32, device=logits.device)
    lse = torch.empty(rows, dtype=torch.float32, device=logits.device)
    _lib.call("ezl_ce_fwd", _p(logits), _p(labels), _p(loss), _p(lse), rows, V, cut_size or 0, _logits_dtype(logits), _stream())
    return loss, lse


def ce_bwd(logits, labels, lse, grad_out, cut_size=0, out=None):
    V = logits.shape[-1]
    rows = logits.numel() // V
    _labels(labels, rows)
    _need(grad_out.is_cuda and grad_out.dtype == torch.float32 and grad_out.is_contiguous() and grad_out.numel() == rows,
          "grad_out must be contiguous fp32, one per row")
    if out is None:
        out = torch.empty_like(logits)
    _lib.call("ezl_ce_bwd", _p(logits), _p(labels), _p(lse), _p(grad_out), _p(out), rows, V, cut_size or 0,
              _logits_dtype(logits), _stream())
    return out


def ce_fused(logits, labels, weights, count, cut_size=0, inplace=True):
    """-> (loss_rows fp32 [rows], grad) ; grad aliases logits when inplace."""
    V = logits.shape[-1]
    rows = logits.numel() // V
    _labels(labels, rows)
    loss_rows = torch.empty(rows, dtype=torch.float32, device=logits.device)
    grad = logits if inplace else torch.empty_like(logits)
    _lib.call("ezl_ce_fused", _p(logits), _p(labels), _p(weights), _p(count), _p(loss_rows), _p(grad), rows, V, cut_size or 0,
              _logits_dtype(logits), _stream())
    return loss_rows, grad


def ce_reduce(loss_rows, weights, count):
    out = torch.empty((), dtype=torch.float32, device=loss_rows.device)
    _lib.call("ezl_ce_reduce", _p(loss_rows), _p(weights), _p(count), _p(out), loss_rows.numel(), _stream())
    return out


def scale_by_scalar_(x, scalar):
    _need(scalar.is_cuda and scalar.dtype == torch.float32 and scalar.numel() == 1, "scalar must be one fp32 value on the GPU")
    _need(x.is_contiguous() and x.dtype in (BF16, torch.float32), "x must be contiguous bf16/fp32")
    _lib.call("ezl_scale_by_scalar", _p(x), _p(scalar), x.numel(), 0 if x.dtype == BF16 else 1, _stream())
    return x


# ------------------------------------------------------------------------------------- optimizer step
def _f32c(t, name):
    _need(t.is_cuda and t.dtype == torch.float32 and t.is_contiguous(), "%s must be a contiguous fp32 GPU tensor" % name)


def sumsq_partials():
    return int(_lib.sumsq_partials())


def sumsq(x, partials_row):
    """partials_row (fp32 [sumsq_partials()]) <- per-block sums of x^2."""
    _f32c(x, "x"); _f32c(partials_row, "partials")
    _need(partials_row.numel() == sumsq_partials(), "partials row has the wrong length")
    _lib.call("ezl_sumsq_f32", _p(x), x.numel(), _p(partials_row), _stream())


def clip_coef(partials, max_norm, out=None):
    """-> fp32 [2] on the GPU: (global L2 norm, clip coefficient)."""
    _f32c(partials, "partials")
    if out is None:
        out = torch.empty(2, dtype=torch.float32, device=partials.device)
    _lib.call("ezl_clip_coef", _p(partials), partials.numel(), float(max_norm), _p(out), _stream())
    return out


def adamw_step(master, exp_avg, exp_avg_sq, grad, param, lr, beta1, beta2, eps, weight_decay, step, bias_correction=True,
               norm_coef=None):
    """In-place AdamW update of (master, exp_avg, exp_avg_sq) from fp32 grad; param (bf16 or None) is refreshed from master."""
    for t, n in ((master, "master"), (exp_avg, "exp_avg"), (exp_avg_sq, "exp_avg_sq"), (grad, "grad")):
        _f32c(t, n)
        _need(t.numel() == master.numel(), "%s size mismatch" % n)
    if param is not None:
        _bf16c(param, "param")
        _need(param.numel() == master.numel(), "param size mismatch")
    if norm_coef is not None:
        _f32c(norm_coef, "norm_coef")
        _need(norm_coef.numel() == 2, "norm_coef must hold (norm, coefficient)")
    _lib.call("ezl_adamw_step", _p(master), _p(exp_avg), _p(exp_avg_sq), _p(grad), _p(param), master.numel(), float(lr),
              float(beta1), float(beta2), float(eps), float(weight_decay), int(step), 1 if bias_correction else 0,
              _p(norm_coef), _stream())
