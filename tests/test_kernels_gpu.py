"""GPU parity tests: every HIP kernel, called through the C ABI, against the CPU oracle on the same
seeded inputs.  Tolerances for floating-point outputs (stated by the task): max |a - ref| <= 2e-2 *
max |ref| and cosine >= 0.9999 against the fp32 oracle evaluated on the same bf16-rounded inputs;
integer work (token gather, label masking, layout moves) is bit-exact.
"""
import math

import pytest
import torch

from oracle import llama_oracle as O

pytestmark = pytest.mark.gpu

REL = 2e-2
COS = 0.9999


def close(a, ref, name, rel=REL, cos=COS):
    a = a.detach().float().cpu().reshape(-1)
    ref = ref.detach().float().cpu().reshape(-1)
    assert a.shape == ref.shape, name
    assert torch.isfinite(a).all(), name + ": non-finite values"
    denom = ref.abs().max().item()
    err = (a - ref).abs().max().item()
    assert err <= rel * max(denom, 1e-30), "%s: max err %.3e vs max ref %.3e" % (name, err, denom)
    if denom > 0:
        c = torch.dot(a, ref) / (a.norm() * ref.norm() + 1e-30)
        assert c.item() >= cos, "%s: cosine %.6f" % (name, c.item())


def bf(t):
    return t.bfloat16()


def rnd(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).bfloat16()


@pytest.fixture(scope="module")
def K(gpu_device):
    from easyllm_amd import kernels
    return kernels


# ------------------------------------------------------------------------------------- RMSNorm
@pytest.mark.parametrize("rows,h", [(7, 256), (1024, 688), (515, 4096), (64, 8192), (3, 8), (1537, 5120), (1030, 6144),
                                    (2051, 8192), (5, 4104), (300, 8200), (513, 16384), (70, 32768)])
def test_rmsnorm_fwd_bwd(K, gpu_device, rows, h):
    print("rmsnorm", rows, h, flush=True)
    x, w, dy = rnd(rows, h, seed=1), (1 + 0.1 * torch.randn(h)).bfloat16(), rnd(rows, h, seed=2)
    y, rstd, _ = K.rmsnorm_fwd(x.to(gpu_device), w.to(gpu_device), 1e-6)
    close(y, O.rmsnorm(x.float(), w.float(), 1e-6), "rmsnorm y")
    dx, dw = K.rmsnorm_bwd(dy.to(gpu_device), x.to(gpu_device), w.to(gpu_device), rstd)
    rdx, rdw = O.rmsnorm_bwd(x.float(), w.float(), dy.float(), 1e-6)
    close(dx, rdx, "rmsnorm dx")
    close(dw, rdw, "rmsnorm dw")
    # fp32 main-grad accumulation
    mg = torch.ones(h, dtype=torch.float32, device=gpu_device)
    K.rmsnorm_bwd(dy.to(gpu_device), x.to(gpu_device), w.to(gpu_device), rstd, main_grad=mg, accumulate=True)
    close(mg, rdw + 1.0, "rmsnorm dw accumulate", rel=2e-3)


@pytest.mark.parametrize("rows,h", [(130, 4096), (1201, 8192), (77, 5120), (259, 12288)])
def test_add_rmsnorm_fused(K, gpu_device, rows, h):
    x, r, w = rnd(rows, h, seed=3), rnd(rows, h, seed=4), (1 + 0.1 * torch.randn(h)).bfloat16()
    y, rstd, s = K.rmsnorm_fwd(x.to(gpu_device), w.to(gpu_device), 1e-6, residual=r.to(gpu_device))
    ssum = (x.float() + r.float()).bfloat16()
    assert torch.equal(s.cpu(), ssum)  # one bf16 rounding of the fp32 sum
    close(y, O.rmsnorm(ssum.float(), w.float(), 1e-6), "add+rmsnorm y")
    dy, dres = rnd(rows, h, seed=5), rnd(rows, h, seed=6)
    dx, _ = K.rmsnorm_bwd(dy.to(gpu_device), s, w.to(gpu_device), rstd, dresidual=dres.to(gpu_device))
    rdx, _ = O.rmsnorm_bwd(ssum.float(), w.float(), dy.float(), 1e-6)
    close(dx, rdx + dres.float(), "add+rmsnorm dx")


# ------------------------------------------------------------------------------------- SwiGLU
def test_swiglu(K, gpu_device):
    g, u, do = rnd(333, 688, seed=1, scale=2.0), rnd(333, 688, seed=2), rnd(333, 688, seed=3)
    out = K.swiglu_fwd(g.to(gpu_device), u.to(gpu_device))
    close(out, O.swiglu(g.float(), u.float()), "swiglu")
    dg, du = K.swiglu_bwd(do.to(gpu_device), g.to(gpu_device), u.to(gpu_device))
    rdg, rdu = O.swiglu_bwd(g.float(), u.float(), do.float())
    close(dg, rdg, "swiglu dgate")
    close(du, rdu, "swiglu dup")


# ------------------------------------------------------------------------------------- RoPE
@pytest.mark.parametrize("s,b,nh,d,use_pos", [(33, 2, 4, 64, False), (40, 1, 8, 128, False), (24, 2, 2, 128, True)])
def test_rope(K, gpu_device, s, b, nh, d, use_pos):
    x = rnd(s, b, nh, d, seed=7)
    inv = O.rope_inv_freq(d)
    cos_t, sin_t = K.rope_table(inv.to(gpu_device), s)
    rc, rs = O.rope_cos_sin(torch.arange(s), d)
    assert torch.allclose(cos_t.cpu(), rc[:, : d // 2], atol=2e-6) and torch.allclose(sin_t.cpu(), rs[:, : d // 2], atol=2e-6)
    pid = None
    if use_pos:
        pid = torch.randint(0, s, (b, s), generator=torch.Generator().manual_seed(1))
    pos = O.positions_sb(s, b, pid)
    c, sn = O.rope_cos_sin(pos, d)
    ref = O.apply_rope(x.float(), c[:, :, None, :], sn[:, :, None, :])
    out = K.rope_apply(x.to(gpu_device), cos_t, sin_t, None if pid is None else pid.to(gpu_device))
    close(out, ref, "rope fwd", rel=1e-2)
    back = K.rope_apply(x.to(gpu_device), cos_t, sin_t, None if pid is None else pid.to(gpu_device), backward=True)
    close(back, O.apply_rope_bwd(x.float(), c[:, :, None, :], sn[:, :, None, :]), "rope bwd", rel=1e-2)
    # strided input (q sliced out of a packed qkv row) and in-place output
    packed = rnd(s, b, 3 * nh * d, seed=8).to(gpu_device)
    qv = packed.view(s, b, 3 * nh, d)[:, :, :nh]
    ref2 = O.apply_rope(qv.float().cpu(), c[:, :, None, :], sn[:, :, None, :])
    K.rope_apply(qv, cos_t, sin_t, None if pid is None else pid.to(gpu_device), out=qv)
    close(qv, ref2, "rope in place, strided", rel=1e-2)


def test_rope_pair_equals_two_single_launches(K, gpu_device):
    """q and k of a layer through one launch: bit-identical to rotating each on its own, forward and backward form, with
    strided inputs (slices of a packed qkv projection) and position ids."""
    s, b, nq, nk, d = 37, 2, 4, 2, 128
    qkv = rnd(s, b, (nq + 2 * nk) * d, seed=31).to(gpu_device)
    q = qkv[..., :nq * d].unflatten(-1, (nq, d))
    k = qkv[..., nq * d:(nq + nk) * d].unflatten(-1, (nk, d))
    inv = O.rope_inv_freq(d).to(gpu_device)
    cos, sin = K.rope_table(inv, 64)
    pos = torch.randint(0, 64, (b, s), generator=torch.Generator().manual_seed(2)).to(gpu_device)
    for p_ids in (None, pos):
        for backward in (False, True):
            qo, ko = K.rope_apply_pair(q, k, cos, sin, p_ids, backward=backward)
            assert torch.equal(qo, K.rope_apply(q, cos, sin, p_ids, backward=backward))
            assert torch.equal(ko, K.rope_apply(k, cos, sin, p_ids, backward=backward))


# ------------------------------------------------------------------------------------- embedding
def test_embedding_gather_exact_and_flag(K, gpu_device):
    V, h = 1000, 256
    W = rnd(V, h, seed=9)
    ids = torch.randint(0, V, (2, 77), generator=torch.Generator().manual_seed(2))
    out, flag = K.embed_gather(ids.to(gpu_device), W.to(gpu_device))
    assert torch.equal(out.cpu(), O.embedding(ids, W))  # bit-exact
    assert flag.item() == 0
    bad = ids.clone()
    bad[1, 5] = V
    _, flag = K.embed_gather(bad.to(gpu_device), W.to(gpu_device))
    assert flag.item() == 1
    with pytest.raises(ValueError):
        O.embedding(bad, W)


@pytest.mark.parametrize("V,h,shape", [(50, 64, (3, 200)), (7, 4096, (1, 700)), (300, 8200, (2, 150)), (9001, 64, (2, 3000))])
def test_embedding_scatter_add(K, gpu_device, V, h, shape):
    """Heavy id collisions (V << rows); the sum per id runs in row order in fp32, so the result is bit-exact
    against a sequential fp32 loop, adds onto what the buffer already holds, and repeats identically."""
    print("embed scatter", V, h, shape, flush=True)
    ids = torch.randint(0, V, shape, generator=torch.Generator().manual_seed(3))
    dy = rnd(*shape, h, seed=10)
    init = torch.randn(V, h, generator=torch.Generator().manual_seed(4))
    dW = init.to(gpu_device)
    K.embed_scatter_add(ids.to(gpu_device), dy.to(gpu_device), dW)
    ref = O.embedding_bwd(ids, dy.float(), V)
    assert torch.allclose(dW.cpu() - init, ref, rtol=1e-4, atol=1e-4)
    seq = torch.zeros(V, h)
    seen = set()
    flat_ids, flat_dy = ids.reshape(-1).tolist(), dy.float().reshape(-1, h)
    for r, i in enumerate(flat_ids):  # first occurrence starts the sum, later rows add in order
        seq[i] = flat_dy[r] if i not in seen else seq[i] + flat_dy[r]
        seen.add(i)
    assert torch.equal(dW.cpu(), init + seq)
    dW2 = init.to(gpu_device)
    K.embed_scatter_add(ids.to(gpu_device), dy.to(gpu_device), dW2)
    assert torch.equal(dW2, dW)


def test_embedding_scatter_add_packed_batch_with_frequent_tokens(K, gpu_device):
    """16384 rows as in the packed workload, ids drawn so that every bucket path runs: most ids once, many a few times
    (sorted in LDS), one id 700 times and one 3000 times (beyond the LDS sort).  Row-order fp32 sums, bit for bit."""
    T, V, h = 16384, 32000, 512
    g = torch.Generator().manual_seed(5)
    ids = torch.randint(0, V, (T,), generator=g)
    ids[torch.randperm(T, generator=g)[:3000]] = 17
    ids[torch.randperm(T, generator=g)[:700]] = 31999
    ids[torch.randint(0, T, (2000,), generator=g)] = torch.randint(100, 140, (2000,), generator=g)
    dy = rnd(T, h, seed=11)
    print("embed scatter, packed batch", flush=True)
    dW = torch.zeros(V, h, device=gpu_device)
    K.embed_scatter_add(ids.view(1, T).to(gpu_device), dy.view(1, T, h).to(gpu_device), dW)
    seq = torch.zeros(V, h)
    dyf = dy.float()
    for r, i in enumerate(ids.tolist()):
        seq[i] += dyf[r]
    assert torch.equal(dW.cpu(), seq)
    dW2 = torch.zeros(V, h, device=gpu_device)
    K.embed_scatter_add(ids.view(1, T).to(gpu_device), dy.view(1, T, h).to(gpu_device), dW2)
    assert torch.equal(dW2, dW)
    # overwrite mode: whatever the buffer held is gone, ids that do not occur get zero rows
    dW3 = torch.full((V, h), 3.5, device=gpu_device)
    K.embed_scatter_add(ids.view(1, T).to(gpu_device), dy.view(1, T, h).to(gpu_device), dW3, accumulate=False)
    assert torch.equal(dW3, dW)


def test_embedding_scatter_add_with_an_id_that_fills_most_of_a_long_batch(K, gpu_device):
    """20000 rows of which 11000 carry one id (a padding token): ten 2048-row windows of the ordering bitmap, most of them
    more than half full, and a second id with 1500 rows.  Row-order fp32 sums, bit for bit, in both modes."""
    T, V, h = 20000, 1000, 264
    g = torch.Generator().manual_seed(6)
    ids = torch.randint(0, V, (T,), generator=g)
    ids[torch.randperm(T, generator=g)[:11000]] = 999
    ids[torch.randperm(T, generator=g)[:1500]] = 0
    dy = rnd(T, h, seed=12)
    print("embed scatter, frequent id", flush=True)
    seq = torch.zeros(V, h)
    dyf = dy.float()
    for r, i in enumerate(ids.tolist()):
        seq[i] += dyf[r]
    dW = torch.full((V, h), -1.25, device=gpu_device)
    K.embed_scatter_add(ids.view(1, T).to(gpu_device), dy.view(1, T, h).to(gpu_device), dW, accumulate=False)
    assert torch.equal(dW.cpu(), seq)
    init = torch.randn(V, h, generator=g)
    dW = init.to(gpu_device)
    K.embed_scatter_add(ids.view(1, T).to(gpu_device), dy.view(1, T, h).to(gpu_device), dW)
    assert torch.equal(dW.cpu(), init + seq)


# ------------------------------------------------------------------------------------- plumbing
def test_transpose_add_cast_exact(K, gpu_device):
    x = rnd(5, 3, 64, seed=11)
    assert torch.equal(K.transpose01(x.to(gpu_device)).cpu(), x.transpose(0, 1).contiguous())
    y = rnd(5, 3, 64, seed=12)
    assert torch.equal(K.add(x.to(gpu_device), y.to(gpu_device)).cpu(), (x.float() + y.float()).bfloat16())
    assert torch.equal(K.cast_bf16_to_f32(x.to(gpu_device)).cpu(), x.float())
    f = torch.randn(5, 3, 64)
    assert torch.equal(K.cast_f32_to_bf16(f.to(gpu_device)).cpu(), f.bfloat16())


# ------------------------------------------------------------------------------------- GEMM
@pytest.mark.parametrize("T,n_in,n_out", [(256, 64, 256), (300, 72, 264), (1024, 256, 688), (512, 688, 256), (77, 1024, 520)])
def test_gemm_three_forms(K, gpu_device, T, n_in, n_out):
    print("gemm", T, n_in, n_out, flush=True)
    x, w, dy = rnd(T, n_in, seed=13), rnd(n_out, n_in, seed=14, scale=0.05), rnd(T, n_out, seed=15)
    xg, wg, dyg = x.to(gpu_device), w.to(gpu_device), dy.to(gpu_device)
    close(K.linear_fwd(xg, wg), O.linear(x.float(), w.float()), "gemm fwd")
    rdx, rdw, _ = O.linear_bwd(x.float(), w.float(), dy.float())
    close(K.linear_dgrad(dyg, wg), rdx, "gemm dgrad")
    close(K.linear_wgrad(dyg, xg), rdw, "gemm wgrad bf16")
    mg = torch.full((n_out, n_in), 0.5, dtype=torch.float32, device=gpu_device)
    K.linear_wgrad(dyg, xg, out=mg, accumulate=True)
    close(mg, rdw + 0.5, "gemm wgrad fp32 accumulate", rel=2e-3)
    K.linear_wgrad(dyg, xg, out=mg, accumulate=False)
    close(mg, rdw, "gemm wgrad fp32 overwrite", rel=2e-3)


@pytest.mark.parametrize("T,n_in,n_outs", [(512, 256, (256, 256, 256)), (300, 136, (128, 192)), (256, 256, (64, 1024, 64)),
                                           (130, 64, (72, 64)), (256, 128, (128, 64))])
def test_gemm_input_gradient_over_several_linears(K, gpu_device, T, n_in, n_outs):
    """dx = sum_i dy_i W_i as one GEMM over all pairs (first three cases), and through the per-pair fallback (a reduction
    length that is not a multiple of 64; dy_i with different row strides): against the fp32 sum, and `accumulate`."""
    print("gemm dgrad multi", T, n_in, n_outs, flush=True)
    ws = [rnd(n, n_in, seed=41 + i, scale=0.05) for i, n in enumerate(n_outs)]
    dys = [rnd(T, n, seed=51 + i) for i, n in enumerate(n_outs)]
    ref = sum(dy.float() @ w.float() for dy, w in zip(dys, ws))
    wg, dyg = [w.to(gpu_device) for w in ws], [dy.to(gpu_device) for dy in dys]
    dx = K.linear_dgrad_multi(dyg, wg)
    close(dx, ref, "dgrad over several linears")
    base = rnd(T, n_in, seed=61)
    out = base.to(gpu_device).clone()
    K.linear_dgrad_multi(dyg, wg, out=out, accumulate=True)
    close(out, ref + base.float(), "dgrad over several linears, accumulate")
    # the same call twice gives the same bits
    assert torch.equal(dx, K.linear_dgrad_multi(dyg, wg))


def _gemm_raw(gpu_device, A, B, M, N, Kd, a_kc, b_kc, out, accumulate, with_workspace):
    """ezl_gemm_bf16 straight through the C ABI, with or without the workspace that enables the split last round."""
    import ctypes
    from easyllm_amd import _lib
    p = lambda t: None if t is None else ctypes.c_void_p(t.data_ptr())  # noqa: E731
    nbytes = _lib.gemm_workspace_bytes(M, N, Kd) if with_workspace else 0
    ws = torch.empty(nbytes, dtype=torch.uint8, device=gpu_device) if nbytes else None
    _lib.call("ezl_gemm_bf16", p(A), p(B), p(out), M, N, Kd, A.stride(0), B.stride(0), out.stride(0), int(a_kc), int(b_kc),
              0 if out.dtype == torch.bfloat16 else 1, int(accumulate), p(ws), nbytes, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    return nbytes


@pytest.mark.parametrize("T,n_in,n_out", [(4096, 2048, 5120), (1000, 4096, 520), (4096, 8192, 1024), (4096, 3072, 5120)])
def test_gemm_with_a_split_last_round_of_tiles(K, gpu_device, T, n_in, n_out):
    """Tile counts that leave the last round of 256 workgroups mostly empty (320 tiles; 12 tiles with ragged edges; 64 tiles):
    with the workspace the reduction of those tiles is split over several workgroups.  All three operand forms against the
    fp32 product, against the unsplit launch of the same kernel (same products, fp32 sums grouped differently), with
    accumulation onto an existing fp32 / bf16 result, and bit-identical when repeated."""
    print("gemm split", T, n_in, n_out, flush=True)
    x, w, dy = rnd(T, n_in, seed=71), rnd(n_out, n_in, seed=72, scale=0.05), rnd(T, n_out, seed=73)
    xg, wg, dyg = x.to(gpu_device), w.to(gpu_device), dy.to(gpu_device)
    # forward: M = T, N = n_out, K = n_in
    y0 = torch.empty(T, n_out, dtype=torch.bfloat16, device=gpu_device)
    y1 = torch.empty_like(y0)
    assert _gemm_raw(gpu_device, xg, wg, T, n_out, n_in, True, True, y0, False, False) == 0
    used = _gemm_raw(gpu_device, xg, wg, T, n_out, n_in, True, True, y1, False, True)
    assert used > 0, "this shape is meant to take the split path"
    close(y1, x.float() @ w.float().t(), "split gemm fwd")
    d = (y1.double() - y0.double()).abs().max().item()
    assert d <= 8e-3 * y0.double().abs().max().item()  # one bf16 ulp where a rounding flips ...
    assert (y1 != y0).float().mean().item() < 0.02      # ... which is rare: the fp32 sums differ in the last bits
    y2 = torch.empty_like(y0)
    _gemm_raw(gpu_device, xg, wg, T, n_out, n_in, True, True, y2, False, True)
    assert torch.equal(y1, y2)
    base = rnd(T, n_out, seed=74).to(gpu_device)
    y3 = base.clone()
    _gemm_raw(gpu_device, xg, wg, T, n_out, n_in, True, True, y3, True, True)
    close(y3, y0.float() + base.float(), "split gemm fwd accumulate", rel=8e-3)
    # through the tensor-level wrappers (which pass the workspace): input gradient and fp32 weight gradient
    assert torch.equal(K.linear_fwd(xg, wg), y1), "the wrapper takes the same path"
    rdx, rdw, _ = O.linear_bwd(x.float(), w.float(), dy.float())
    close(K.linear_dgrad(dyg, wg), rdx, "split gemm dgrad")
    mg = torch.full((n_out, n_in), 0.5, dtype=torch.float32, device=gpu_device)
    K.linear_wgrad(dyg, xg, out=mg, accumulate=True)
    close(mg, rdw + 0.5, "split gemm wgrad fp32 accumulate", rel=2e-3)
    K.linear_wgrad(dyg, xg, out=mg, accumulate=False)
    close(mg, rdw, "split gemm wgrad fp32 overwrite", rel=2e-3)


def test_gemm_input_gradient_over_several_linears_with_a_split_last_round(K, gpu_device):
    """The three-pair input gradient at 320 output tiles: the split shares of the reduction (8 K tiles each) straddle the
    boundaries between the pairs (K tiles 5 and 16)."""
    T, n_in, n_outs = 4096, 5120, (320, 704, 1024)
    ws = [rnd(n, n_in, seed=81 + i, scale=0.05) for i, n in enumerate(n_outs)]
    dys = [rnd(T, n, seed=91 + i) for i, n in enumerate(n_outs)]
    ref = sum(dy.float() @ w.float() for dy, w in zip(dys, ws))
    wg, dyg = [w.to(gpu_device) for w in ws], [dy.to(gpu_device) for dy in dys]
    from easyllm_amd import _lib
    assert _lib.gemm_workspace_bytes(T, n_in, sum(n_outs)) > 0
    dx = K.linear_dgrad_multi(dyg, wg)
    close(dx, ref, "dgrad over three linears, split last round")
    assert torch.equal(dx, K.linear_dgrad_multi(dyg, wg))


def test_gemm_forward_with_unaligned_output_width(K, gpu_device):
    """out features not a multiple of 4: the epilogue falls back from vector to element stores; K = 128 and 192 are the
    shortest reductions of the direct-to-LDS kernel (2 and 3 K tiles), K = 64 goes through the register-staged one."""
    for T, n_in, n_out in ((130, 128, 250), (257, 192, 31), (64, 64, 7)):
        print("gemm odd width", T, n_in, n_out, flush=True)
        x, w = rnd(T, n_in, seed=17), rnd(n_out, n_in, seed=18, scale=0.05)
        y = K.linear_fwd(x.to(gpu_device), w.to(gpu_device))
        assert tuple(y.shape) == (T, n_out)
        close(y, x.float() @ w.float().t(), "gemm fwd odd width")


@pytest.mark.parametrize("T,n_in,n_out", [(512, 3072, 512), (300, 3136, 520), (1000, 4096, 264), (257, 8192, 1032)])
def test_gemm_forward_over_long_reductions(K, gpu_device, T, n_in, n_out):
    """The forward form (both operands k-contiguous) from 48 K tiles on runs the 4-wave kernel when the output allows 16-byte
    stores: whole and ragged tiles, bf16 and fp32 results, overwrite and accumulate, an odd number of K tiles (3136 = 49 x 64),
    against the fp64 product of the same bf16 operands; and bit-equal with the 8-wave kernel, which adds the K tiles in the
    same order (reached here through an output whose row stride rules out 16-byte stores)."""
    print("gemm long forward", T, n_in, n_out, flush=True)
    x, w = rnd(T, n_in, seed=91), rnd(n_out, n_in, seed=92, scale=0.05)
    xg, wg = x.to(gpu_device), w.to(gpu_device)
    ref = (x.double() @ w.double().t())
    y = torch.empty(T, n_out, dtype=torch.bfloat16, device=gpu_device)
    _gemm_raw(gpu_device, xg, wg, T, n_out, n_in, 1, 1, y, False, False)
    close(y, ref.float(), "long forward bf16")
    base = rnd(T, n_out, seed=93)
    y2 = base.to(gpu_device).clone()
    _gemm_raw(gpu_device, xg, wg, T, n_out, n_in, 1, 1, y2, True, False)
    close(y2, (ref + base.double()).float(), "long forward bf16 accumulate")
    f = torch.full((T, n_out), 0.25, dtype=torch.float32, device=gpu_device)
    _gemm_raw(gpu_device, xg, wg, T, n_out, n_in, 1, 1, f, True, False)
    assert (f.double().cpu() - (ref + 0.25)).abs().max().item() <= 2e-3 * ref.abs().max().item(), "long forward fp32 accumulate"
    _gemm_raw(gpu_device, xg, wg, T, n_out, n_in, 1, 1, f, False, False)
    assert (f.double().cpu() - ref).abs().max().item() <= 2e-3 * ref.abs().max().item(), "long forward fp32"
    # 8-wave kernel: a row stride of n_out + 4 elements is not a multiple of 8
    wide = torch.zeros(T, n_out + 4, dtype=torch.bfloat16, device=gpu_device)
    y8 = wide[:, :n_out]
    _gemm_raw(gpu_device, xg, wg, T, n_out, n_in, 1, 1, y8, False, False)
    assert torch.equal(y8, y), "4-wave and 8-wave kernels differ"
    assert float(wide[:, n_out:].abs().max()) == 0.0, "wrote past the output's columns"


@pytest.mark.parametrize("T,n_in,n_out", [(3072, 512, 512), (3136, 520, 264), (8192, 264, 1032)])
def test_gemm_fp32_weight_gradient_over_many_tokens(K, gpu_device, T, n_in, n_out):
    """The fp32 weight gradient (both operands k-strided) over 48 K tiles or more runs the 4-wave kernel: whole and ragged
    tiles, an odd number of K tiles, overwrite and accumulate, against the fp64 product of the same bf16 operands; and
    bit-equal with the 8-wave kernel (same order of the K tiles), reached through a row stride that rules out 16-byte stores."""
    print("gemm long wgrad", T, n_in, n_out, flush=True)
    x, dy = rnd(T, n_in, seed=95), rnd(T, n_out, seed=96)
    xg, dyg = x.to(gpu_device), dy.to(gpu_device)
    ref = dy.double().t() @ x.double()
    tol = 2e-3 * ref.abs().max().item()
    g = torch.full((n_out, n_in), 0.5, dtype=torch.float32, device=gpu_device)
    _gemm_raw(gpu_device, dyg, xg, n_out, n_in, T, 0, 0, g, True, False)
    assert (g.double().cpu() - (ref + 0.5)).abs().max().item() <= tol, "accumulate"
    _gemm_raw(gpu_device, dyg, xg, n_out, n_in, T, 0, 0, g, False, False)
    assert (g.double().cpu() - ref).abs().max().item() <= tol, "overwrite"
    wide = torch.zeros(n_out, n_in + 2, dtype=torch.float32, device=gpu_device)  # row stride not a multiple of 4: 8-wave kernel
    g8 = wide[:, :n_in]
    _gemm_raw(gpu_device, dyg, xg, n_out, n_in, T, 0, 0, g8, False, False)
    assert torch.equal(g8, g), "4-wave and 8-wave kernels differ"
    assert float(wide[:, n_in:].abs().max()) == 0.0, "wrote past the output's columns"


def test_gemm_linearity_large(K, gpu_device):
    """Size-independent property at a full-size shape: a column block of the result equals the GEMM on that block of W --
    bit for bit where both launches sum in the same order, and to one bf16 ulp on a rare element where the narrow launch
    (48 tiles: its reduction is split over several workgroups) groups the fp32 sum differently."""
    T, n_in, n_out = 4096, 4096, 11008
    g = torch.Generator(device="cpu").manual_seed(16)
    x1 = (torch.randn(T, n_in, generator=g)).bfloat16().to(gpu_device)
    w = (torch.randn(n_out, n_in, generator=g) * 0.02).bfloat16().to(gpu_device)
    y = K.linear_fwd(x1, w)
    yb = K.linear_fwd(x1, w[5000:5520])
    blk = y[:, 5000:5520].double().cpu()
    assert (blk - yb.double().cpu()).abs().max().item() <= 8e-3 * blk.abs().max().item()
    assert (y[:, 5000:5520] != yb).float().mean().item() < 0.02
    yc = K.linear_fwd(x1[:, :448], w[5000:5520, :448])  # 7 K tiles: too short a reduction to split
    yd = K.linear_fwd(x1[:, :448], w[:, :448])
    assert torch.equal(yd[:, 5000:5520], yc)
    ref = (x1[:64].float() @ w.float().t()).cpu()
    close(y[:64], ref, "gemm big slice")


def test_gemm_wrapper_refuses_what_would_read_or_add_out_of_place(K, gpu_device):
    x, w = rnd(64, 128, seed=1).to(gpu_device), rnd(256, 128, seed=2).to(gpu_device)
    with pytest.raises(ValueError):
        K.linear_wgrad(rnd(64, 256, seed=3).to(gpu_device), x, accumulate=True)  # nothing to add to
    with pytest.raises(ValueError):
        K.linear_dgrad_multi([rnd(64, 256, seed=3).to(gpu_device)], [w], accumulate=True)
    with pytest.raises(ValueError):
        K.gemm(x, w, 128, 256, 128, 128, 128, True, True)  # claims 128 rows of x, there are 64
    with pytest.raises(ValueError):
        K.gemm(x, w, 64, 256, 256, 128, 128, True, True)  # reduction longer than the rows
    with pytest.raises(ValueError):
        K.gemm(x.float(), w, 64, 256, 128, 128, 128, True, True)


def test_gemm_all_forms_at_full_size_reductions(K, gpu_device):
    """The 7B-shape MLP linears, every form against the fp32 product of the same bf16 operands on the host:
    forward (K = 4096), input gradient (K = 11008), fp32 weight gradient over K = T = 4096 tokens written and then
    accumulated, and the input gradient of three linears that share their input as one launch (K = 3 x 4096)."""
    T, n_in, n_out = 4096, 4096, 11008
    x, w, dy = rnd(T, n_in, seed=71), rnd(n_out, n_in, seed=72, scale=0.02), rnd(T, n_out, seed=73)
    xg, wg, dyg = x.to(gpu_device), w.to(gpu_device), dy.to(gpu_device)
    xf, wf, dyf = x.float(), w.float(), dy.float()
    print("gemm full size: forward", flush=True)
    close(K.linear_fwd(xg, wg), xf @ wf.t(), "gemm fwd 4096x11008x4096")
    print("gemm full size: dgrad", flush=True)
    close(K.linear_dgrad(dyg, wg), dyf @ wf, "gemm dgrad 4096x4096x11008")
    print("gemm full size: wgrad fp32", flush=True)
    rdw = dyf.t() @ xf
    mg = torch.empty(n_out, n_in, dtype=torch.float32, device=gpu_device)
    K.linear_wgrad(dyg, xg, out=mg, accumulate=False)
    close(mg, rdw, "gemm wgrad fp32 11008x4096x4096", rel=2e-3, cos=0.999999)
    K.linear_wgrad(dyg, xg, out=mg, accumulate=True)
    close(mg, 2 * rdw, "gemm wgrad fp32 accumulated twice", rel=2e-3, cos=0.999999)
    close(K.linear_wgrad(dyg, xg), rdw, "gemm wgrad bf16 11008x4096x4096")
    print("gemm full size: dgrad over q/k/v", flush=True)
    ws = [rnd(4096, n_in, seed=74 + i, scale=0.02) for i in range(3)]
    dys = [rnd(T, 4096, seed=77 + i) for i in range(3)]
    ref = sum(a.float() @ b.float() for a, b in zip(dys, ws))
    close(K.linear_dgrad_multi([a.to(gpu_device) for a in dys], [b.to(gpu_device) for b in ws]), ref,
          "gemm dgrad over three linears, K = 12288")


def test_gemm_operand_beyond_two_to_the_31_elements(K, gpu_device):
    """d logits of a packed 16384-token batch over a 152064-entry vocabulary is 2.5e9 elements (5 GB): the input gradient
    (that matrix as the row operand) and the weight gradient (as the transposed operand) must address all of it.
    Checked on the first and last rows / columns against fp32 on the host."""
    T, V, h = 16384, 152064, 256
    print("gemm, operand of %.2e elements" % (T * V), flush=True)
    torch.manual_seed(91)
    dy = torch.empty(T, V, dtype=torch.bfloat16, device=gpu_device)
    for r0 in range(0, T, 2048):  # filled in pieces: the generator's fp32 temporaries stay small
        dy[r0:r0 + 2048] = torch.randn(2048, V, device=gpu_device).bfloat16()
    w = (torch.randn(V, h, device=gpu_device) * 0.02).bfloat16()
    x = torch.randn(T, h, device=gpu_device).bfloat16()
    dx = K.linear_dgrad(dy, w)
    rows = torch.cat([torch.arange(0, 8), torch.arange(T // 2 - 4, T // 2 + 4), torch.arange(T - 8, T)])
    close(dx[rows.to(gpu_device)], dy[rows.to(gpu_device)].float().cpu() @ w.float().cpu(), "dgrad rows of a 5 GB operand")
    dw = torch.empty(V, h, dtype=torch.float32, device=gpu_device)
    K.linear_wgrad(dy, x, out=dw)
    cols = torch.cat([torch.arange(0, 8), torch.arange(V // 2 - 4, V // 2 + 4), torch.arange(V - 8, V)])
    ref = dy[:, cols.to(gpu_device)].float().cpu().t() @ x.float().cpu()
    close(dw[cols.to(gpu_device)], ref, "wgrad rows from a 5 GB operand", rel=2e-3)
    del dy, dw
    torch.cuda.empty_cache()


# ------------------------------------------------------------------------------------- attention
def _attn_case(K, dev, s, b, nq, nk, d, cu, seed):
    q, k, v, do = rnd(s, b, nq, d, seed=seed), rnd(s, b, nk, d, seed=seed + 1), rnd(s, b, nk, d, seed=seed + 2), rnd(s, b, nq, d, seed=seed + 3)
    qf, kf, vf = [t.float().requires_grad_(True) for t in (q, k, v)]
    cu_t = None if cu is None else torch.tensor(cu, dtype=torch.int32)
    ref = O.attention(qf.transpose(0, 1), kf.transpose(0, 1), vf.transpose(0, 1), cu_t).transpose(0, 1)
    ref.backward(do.float())
    cug = None if cu is None else cu_t.to(dev)
    out, lse = K.attn_fwd(q.to(dev), k.to(dev), v.to(dev), cug)
    close(out, ref, "attn out")
    dq, dk, dv = K.attn_bwd(q.to(dev), k.to(dev), v.to(dev), out, do.to(dev), lse, cug)
    close(dq, qf.grad, "attn dq")
    close(dk, kf.grad, "attn dk")
    close(dv, vf.grad, "attn dv")


@pytest.mark.parametrize("s,b,nq,nk,d", [(512, 2, 4, 4, 64), (384, 1, 8, 2, 128), (100, 2, 2, 1, 128), (1, 1, 2, 2, 64)])
def test_attention_dense(K, gpu_device, s, b, nq, nk, d):
    print("attention", s, b, nq, nk, d, flush=True)
    _attn_case(K, gpu_device, s, b, nq, nk, d, None, 20)


@pytest.mark.parametrize("d,nq,nk", [(128, 4, 4), (64, 4, 2)])
def test_attention_varlen_ragged(K, gpu_device, d, nq, nk):
    cu = [0, 1, 64, 65, 200, 333, 333, 640]  # lengths 1, 63, 1, 135, 133, 0 (empty), 307
    print("attention varlen", d, nq, nk, flush=True)
    _attn_case(K, gpu_device, 640, 1, nq, nk, d, cu, 30)


def test_attention_varlen_across_batch_rows(K, gpu_device):
    # flattened (b s) documents as the collator builds them: cu + bidx * s, leading 0 dropped
    cu = O.flatten_cu_seqlens([[0, 100, 256], [0, 31, 256]], 256).tolist()
    _attn_case(K, gpu_device, 256, 2, 4, 4, 128, cu, 40)


@pytest.mark.parametrize("s,nq,nk", [(4096, 2, 2), (4096, 8, 1)])
def test_attention_at_full_sequence_length(K, gpu_device, s, nq, nk):
    """seq 4096, d 128: 64 key tiles of online softmax per query block, MHA and a GQA group of 8 (the 70B shape's group),
    forward and backward against the fp32 oracle."""
    print("attention full length", s, nq, nk, flush=True)
    _attn_case(K, gpu_device, s, 1, nq, nk, 128, None, 50)


def test_attention_64_query_heads_on_8_kv_heads(K, gpu_device):
    """The 70B head layout (64 q / 8 kv): with a multiple of 8 kv heads the workgroup renumbering deals whole kv heads to
    the 8 L2 domains; short sequence so that the host finishes quickly."""
    print("attention 64q/8kv", flush=True)
    _attn_case(K, gpu_device, 320, 1, 64, 8, 128, None, 60)
    _attn_case(K, gpu_device, 200, 2, 64, 8, 128, None, 61)


def test_attention_packed_16k_tokens(K, gpu_device):
    """The packed workload's token count and document recipe (16384 tokens, lengths log-uniform in [64, 4096]) on 2 heads:
    block-diagonal causal attention over ~17 documents, forward and backward against the oracle."""
    lens = O.packed_doc_lengths(16384, 64, 4096, 1005)
    cu = [0]
    for l in lens:
        cu.append(cu[-1] + l)
    print("attention packed 16k,", len(lens), "documents", flush=True)
    _attn_case(K, gpu_device, 16384, 1, 2, 2, 128, cu, 70)
    _attn_case(K, gpu_device, 16384, 1, 4, 1, 128, cu, 71)


def test_attention_forward_with_drifting_and_jumping_maxima(K, gpu_device):
    """The forward kernel moves the reference point of its exponentials only when a row's maximum has outgrown it by a
    factor 2^8.  Scores here grow along the keys: slowly for most rows (many tiles pass between two moves, probabilities
    far above 1 in between), in jumps for the keys after position 700; output and logsumexp against the oracle in fp32."""
    s, nq, d = 1024, 2, 128
    g = torch.Generator().manual_seed(77)
    q = torch.randn(s, 1, nq, d, generator=g) * 0.3 + 1.0
    ramp = torch.linspace(0.2, 2.2, s).view(s, 1, 1, 1)
    k = torch.randn(s, 1, nq, d, generator=g) * 0.3 + ramp * 0.5
    k[700:] *= 1.8
    v = torch.randn(s, 1, nq, d, generator=g)
    q, k, v = q.bfloat16(), k.bfloat16(), v.bfloat16()
    scores = torch.einsum("qhd,khd->hqk", q[:, 0].float(), k[:, 0].float()) / d ** 0.5
    scores = scores.masked_fill(torch.triu(torch.ones(s, s, dtype=torch.bool), 1), float("-inf"))
    # the case is what the docstring says: row maxima keep rising, by more than 2^8 in total
    run_max = scores.cummax(-1).values
    rise = (run_max[..., -1] - run_max[..., 64]) * 1.4427  # in powers of two
    assert rise[:, 768:].min() > 16 and 2 < rise[:, 300:700].min() and rise[:, 300:700].max() < 16
    ref_lse = torch.logsumexp(scores, -1)
    ref = torch.einsum("hqk,khd->qhd", torch.softmax(scores, -1), v[:, 0].float())
    out, lse = K.attn_fwd(q.to(gpu_device), k.to(gpu_device), v.to(gpu_device), None)
    close(out[:, 0], ref, "attn out (rising maxima)")
    assert torch.allclose(lse.cpu().view(nq, s), ref_lse, rtol=1e-4, atol=2e-3)


def test_mask_compaction_is_exact(K, gpu_device):
    for b, s, seed in ((3, 700, 1), (1, 64, 2), (5, 1500, 3), (2, 8, 4)):
        mask = torch.rand(b, s, generator=torch.Generator().manual_seed(seed)) < 0.6
        if b > 2:
            mask[1] = False  # a row with nothing kept
            mask[2] = True
        idx, inv, cu = K.mask_compact(mask.to(gpu_device))
        flat = mask.reshape(-1)
        kept = torch.nonzero(flat).reshape(-1)
        want_idx = torch.full((b * s,), -1, dtype=torch.int32)
        want_idx[:kept.numel()] = kept.int()
        want_inv = torch.where(flat, torch.cumsum(flat.int(), 0) - 1, torch.full((b * s,), -1)).int()
        want_cu = torch.cat([torch.zeros(1, dtype=torch.int64), torch.cumsum(mask.sum(1), 0)]).int()
        assert torch.equal(idx.cpu(), want_idx) and torch.equal(inv.cpu(), want_inv) and torch.equal(cu.cpu(), want_cu)


@pytest.mark.parametrize("s,b,nq,nk,d", [(200, 3, 4, 2, 128), (333, 2, 2, 2, 64)])
def test_attention_unpadded_by_key_padding_mask(K, gpu_device, s, b, nq, nk, d):
    """The key_padding_mask branch: gather the kept tokens of every row, attend causally among them, scatter back with zero
    rows; forward and backward (through the autograd wrappers) against the oracle."""
    from easyllm_amd.transformer import FlashAttention
    print("attention unpadded", s, b, nq, nk, d, flush=True)
    mask = torch.rand(b, s, generator=torch.Generator().manual_seed(7)) < 0.7
    mask[0, s // 2:] = False  # right padding
    if b > 2:
        mask[2] = False       # nothing kept
    q, k, v, do = rnd(s, b, nq, d, seed=80), rnd(s, b, nk, d, seed=81), rnd(s, b, nk, d, seed=82), rnd(s, b, nq, d, seed=83)
    qf, kf, vf = [t.float().requires_grad_(True) for t in (q, k, v)]
    ref = O.attention_unpadded(qf.transpose(0, 1), kf.transpose(0, 1), vf.transpose(0, 1), mask).transpose(0, 1)
    ref.backward(do.float())
    qg, kg, vg = [t.to(gpu_device).requires_grad_(True) for t in (q, k, v)]
    attn = FlashAttention(causal=True)
    out = attn(qg.transpose(0, 1), kg.transpose(0, 1), vg.transpose(0, 1), key_padding_mask=mask.to(gpu_device)).transpose(0, 1)
    close(out, ref, "unpadded attn out")
    dropped = ~mask.t()  # [s, b]
    assert torch.count_nonzero(out.detach().cpu()[dropped]) == 0
    out.backward(do.to(gpu_device))
    close(qg.grad, qf.grad, "unpadded attn dq")
    close(kg.grad, kf.grad, "unpadded attn dk")
    close(vg.grad, vf.grad, "unpadded attn dv")
    for gr in (qg.grad, kg.grad, vg.grad):
        assert torch.count_nonzero(gr.cpu()[dropped]) == 0


# ------------------------------------------------------------------------------------- cross entropy
@pytest.mark.parametrize("rows,V,dtype,cut", [(33, 32000, torch.bfloat16, 0), (5, 152064, torch.bfloat16, 0),
                                              (17, 4096, torch.float32, 0), (9, 32000, torch.float32, 0),
                                              (12, 1024, torch.bfloat16, 24),
                                              # rows kept on chip in LDS + registers (one read of the logits): more rows than
                                              # blocks, so every block walks several rows and refills its slots; a row length
                                              # whose last register vector is mostly past the end; cut columns; and the lengths
                                              # either side of that kernel's range
                                              (300, 152064, torch.bfloat16, 0), (270, 73736, torch.bfloat16, 0),
                                              (40, 152064, torch.bfloat16, 64), (6, 180224, torch.bfloat16, 0),
                                              (6, 73720, torch.bfloat16, 0), (6, 180232, torch.bfloat16, 0)])
def test_cross_entropy_all_paths(K, gpu_device, rows, V, dtype, cut):
    print("ce", rows, V, dtype, cut, flush=True)
    g = torch.Generator().manual_seed(50)
    logits = (torch.randn(rows, V, generator=g) * 2).to(dtype)
    labels = torch.randint(0, V - cut, (rows,), generator=g)
    labels[1] = -100
    if rows > 4:
        labels[4] = V - 1 if cut else -100
    lf = logits.float()
    ref_loss = O.vocab_parallel_cross_entropy(lf[None], labels[None], cut or None)[0]
    lg, tg = logits.to(gpu_device), labels.to(gpu_device)
    loss, lse = K.ce_fwd(lg, tg, cut)
    assert torch.allclose(loss.cpu(), ref_loss, rtol=1e-4, atol=1e-4)
    go = torch.rand(rows, generator=g) + 0.5
    grad = K.ce_bwd(lg, tg, lse, go.to(gpu_device), cut)
    ref_grad = O.vocab_parallel_cross_entropy_bwd(lf[None], labels[None], go[None], cut or None)[0]
    close(grad, ref_grad, "ce bwd")
    # fused mean loss + grad
    mask = (torch.rand(rows, generator=g) < 0.8)
    w, n = K.ce_prepare(tg, mask.to(gpu_device))
    rw, rn = O.loss_weights(labels, mask)
    assert torch.equal(w.cpu(), rw) and n.item() == rn.item()  # label masking is exact
    ref_total = O.cross_entropy_loss(lf[None], labels[None], mask[None], cut or None)
    loss_rows, gfused = K.ce_fused(lg.clone(), tg, w, n, cut, inplace=True)
    total = K.ce_reduce(loss_rows, w, n)
    assert abs(total.item() - ref_total.item()) <= 1e-3 * abs(ref_total.item())
    # rows with weight 0 have exactly zero gradient; the others follow the reference's hand-written
    # backward (cross_entropy.py:91-112) with grad_out = weight / count
    zero_rows = (rw == 0)
    assert torch.count_nonzero(gfused.cpu()[zero_rows]) == 0
    ref_fused = O.vocab_parallel_cross_entropy_bwd(lf[None], labels[None], (rw / rn)[None], cut or None)[0]
    close(gfused.cpu()[~zero_rows], ref_fused[~zero_rows], "ce fused grad")
    if not cut:  # without a cut the hand-written backward is the true gradient of the mean loss
        lref = lf.clone().requires_grad_(True)
        O.cross_entropy_loss(lref[None], labels[None], mask[None], None).backward()
        valid = (labels >= 0) & ~zero_rows
        close(gfused.cpu()[valid], lref.grad[valid], "ce fused grad vs autograd")


def test_ce_scale_by_scalar(K, gpu_device):
    x = rnd(16, 64, seed=60).to(gpu_device)
    y = x.clone()
    K.scale_by_scalar_(y, torch.ones(1, device=gpu_device))
    assert torch.equal(x, y)
    K.scale_by_scalar_(y, torch.full((1,), 0.5, device=gpu_device))
    assert torch.equal(y.cpu(), (x.float().cpu() * 0.5).bfloat16())


# ------------------------------------------------------------------------------------- empty inputs
def test_empty_inputs_are_accepted_everywhere(K, gpu_device):
    """Zero tokens (an empty micro-batch shard): every entry point returns empty results without launching on garbage."""
    dev = gpu_device
    h, f, V = 64, 96, 128
    e = lambda *shape, dtype=torch.bfloat16: torch.empty(*shape, dtype=dtype, device=dev)  # noqa: E731
    w = torch.ones(h, dtype=torch.bfloat16, device=dev)
    y, rstd, _ = K.rmsnorm_fwd(e(0, h), w, 1e-6)
    assert y.shape == (0, h) and rstd.numel() == 0
    dx, dw = K.rmsnorm_bwd(e(0, h), e(0, h), w, rstd)
    assert dx.shape == (0, h) and float(dw.float().abs().max()) == 0.0   # no rows: a zero weight gradient
    assert K.swiglu_fwd(e(0, f), e(0, f)).numel() == 0
    dg, du = K.swiglu_bwd(e(0, f), e(0, f), e(0, f))
    assert dg.numel() == 0 and du.numel() == 0
    assert K.add(e(0, h), e(0, h)).numel() == 0
    assert K.transpose01(e(0, 2, h)).shape == (2, 0, h)
    out, flag = K.embed_gather(torch.empty(1, 0, dtype=torch.int64, device=dev), torch.zeros(V, h, dtype=torch.bfloat16, device=dev))
    assert out.shape == (1, 0, h) and flag.item() == 0
    dW = torch.ones(V, h, dtype=torch.float32, device=dev)
    K.embed_scatter_add(torch.empty(0, dtype=torch.int64, device=dev), e(0, h), dW)
    assert float(dW.min()) == 1.0
    wt = torch.zeros(f, h, dtype=torch.bfloat16, device=dev)
    assert K.linear_fwd(e(0, h), wt).shape == (0, f)
    assert K.linear_dgrad(e(0, f), wt).shape == (0, h)
    gw = K.linear_wgrad(e(0, f), e(0, h))                               # K = 0 tokens: the gradient is exactly zero
    assert gw.shape == (f, h) and float(gw.float().abs().max()) == 0.0
    lg = e(0, V)
    lb = torch.empty(0, dtype=torch.int64, device=dev)
    wts, n = K.ce_prepare(lb, None)
    assert float(n) == 0.0
    loss_rows, grad = K.ce_fused(lg, lb, wts, n, inplace=False)
    assert loss_rows.numel() == 0 and grad.numel() == 0
    q, kv = e(0, 1, 4, 64), e(0, 1, 2, 64)
    out, lse = K.attn_fwd(q, kv, kv)
    assert out.shape == (0, 1, 4, 64) and lse.numel() == 0
    dq, dk, dv = K.attn_bwd(q, kv, kv, out, e(0, 1, 4, 64), lse)
    assert dq.numel() == 0 and dk.numel() == 0 and dv.numel() == 0
    inv = 1.0 / (10000 ** (torch.arange(0, 64, 2, device=dev).float() / 64))
    cos, sin = K.rope_table(inv, 8)
    assert K.rope_apply(q, cos, sin).shape == (0, 1, 4, 64)
