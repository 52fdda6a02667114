"""The workspace-free RMSNorm backward (ezl_rmsnorm_bwd_noalloc: partial sums in a device array built into the library)
against ezl_rmsnorm_bwd, through the C ABI: same kernels, so dx and dw must agree bit for bit -- on two calls in a row, the
second on a smaller input (the array still holds the first call's partials), then with the residual gradient and fp32
accumulation, and a width beyond the built-in limit must be refused before anything is launched."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _p(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _both(lib, dev, rows, h, seed, with_res, f32_dw):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(rows, h, generator=g).bfloat16().to(dev)
    dy = torch.randn(rows, h, generator=g).bfloat16().to(dev)
    w = (1.0 + 0.1 * torch.randn(h, generator=g)).bfloat16().to(dev)
    rstd = torch.rsqrt(x.float().pow(2).mean(-1) + 1e-6).contiguous()
    dres = torch.randn(rows, h, generator=g).bfloat16().to(dev) if with_res else None
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    outs = []
    for noalloc in (False, True):
        dx = torch.full((rows, h), 7.0, dtype=torch.bfloat16, device=dev)
        dw16 = None if f32_dw else torch.full((h,), 7.0, dtype=torch.bfloat16, device=dev)
        dw32 = torch.full((h,), 0.25, dtype=torch.float32, device=dev) if f32_dw else None
        if noalloc:
            lib.call("ezl_rmsnorm_bwd_noalloc", _p(dy), _p(x), _p(w), _p(rstd), _p(dres), _p(dx), _p(dw16), _p(dw32),
                     1 if f32_dw else 0, rows, h, stream)
        else:
            nbytes = lib.rmsnorm_bwd_workspace_bytes(rows, h)
            ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
            lib.call("ezl_rmsnorm_bwd", _p(dy), _p(x), _p(w), _p(rstd), _p(dres), _p(dx), _p(dw16), _p(dw32),
                     1 if f32_dw else 0, _p(ws), nbytes, rows, h, stream)
        torch.cuda.synchronize()
        outs.append((dx, dw32 if f32_dw else dw16))
    (dx_a, dw_a), (dx_b, dw_b) = outs
    assert torch.equal(dx_a, dx_b) and torch.equal(dw_a, dw_b), (rows, h)
    assert torch.isfinite(dx_b.float()).all() and dw_b.float().abs().max().item() > 0
    return dw_b


def test_rmsnorm_bwd_without_workspace_matches_the_workspace_entry_point(gpu_device):
    from easyllm_amd import _lib as lib, kernels as K
    from oracle import llama_oracle as O
    lib.load()
    assert lib.load().ezl_rmsnorm_bwd_noalloc_max_h() == 8192
    print("no-alloc rmsnorm backward: 4096 x 4096, then 515 x 1024", flush=True)
    _both(lib, gpu_device, 4096, 4096, 1, False, False)   # 256 blocks of partials
    _both(lib, gpu_device, 515, 1024, 2, False, False)    # smaller: fewer blocks, narrower rows, same array
    _both(lib, gpu_device, 1000, 8192, 3, True, True)     # widest rows, residual gradient, fp32 dw accumulated onto 0.25
    _both(lib, gpu_device, 3, 8, 4, False, True)
    # against the oracle as well (the workspace entry point is, in test_kernels_gpu.py), through the tensor-level wrapper
    g = torch.Generator().manual_seed(9)
    x, dy = torch.randn(300, 2048, generator=g).bfloat16(), torch.randn(300, 2048, generator=g).bfloat16()
    w = (1.0 + 0.1 * torch.randn(2048, generator=g)).bfloat16()
    rstd = torch.rsqrt(x.float().pow(2).mean(-1) + 1e-6)
    rdx, rdw = O.rmsnorm_bwd(x.float(), w.float(), dy.float())
    dx, dw = K.rmsnorm_bwd(dy.to(gpu_device), x.to(gpu_device), w.to(gpu_device), rstd.to(gpu_device), builtin_scratch=True)
    for a, r in ((dx, rdx), (dw, rdw)):
        a, r = a.float().cpu().reshape(-1), r.reshape(-1)
        assert (a - r).abs().max() <= 2e-2 * r.abs().max() and torch.dot(a, r) / (a.norm() * r.norm()) >= 0.9999
    # beyond the built-in scratch: refused, nothing launched
    big = torch.zeros(2, 8200, dtype=torch.bfloat16, device=gpu_device)
    with pytest.raises(RuntimeError):
        lib.call("ezl_rmsnorm_bwd_noalloc", _p(big), _p(big), _p(big[0]), _p(torch.zeros(2, device=gpu_device)), None, _p(big),
                 _p(big[1]), None, 0, 2, 8200, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
