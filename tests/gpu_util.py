"""Helpers shared by the GPU parity tests: move numpy data through the C ABI."""
import numpy as np
import torch

from nntrainer_amd import capi

TOL = 1e-4  # max|gpu - ref| / max|ref| per matrix, the bar the path is judged at


def stream():
    return torch.cuda.current_stream().cuda_stream


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def rel_err(got, ref):
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    return float(np.abs(got - ref).max() / max(np.abs(ref).max(), 1e-30))


def gpu_matmul(w, a):
    """a fp32 numpy [M, K] -> numpy [M, N] through hipq_matmul on device buffers."""
    m = a.shape[0]
    da = dev(a.astype(np.float32))
    dc = torch.full((m, w.n), float("nan"), device="cuda", dtype=torch.float32)
    capi.matmul(w, da, m, dc, stream=stream())
    torch.cuda.synchronize()
    return dc.cpu().numpy()


def gpu_quantize(kind, x, variant="row"):
    """x fp32 numpy [M, K] -> canonical activation blocks uint8 [M, rowbytes]."""
    m, k = x.shape
    nbytes, blk = (34, 32) if kind == "q8_0" else (292, 256)
    dx = dev(x.astype(np.float32))
    out = torch.zeros((m, (k // blk) * nbytes), device="cuda", dtype=torch.uint8)
    if kind == "q8_0":
        capi.quantize_q8_0(dx, m, k, out, stream=stream())
    else:
        capi.quantize_q8_K(dx, m, k, out, variant=capi.Q8K_MAT if variant == "mat" else capi.Q8K_ROW,
                           stream=stream())
    torch.cuda.synchronize()
    return out.cpu().numpy()
