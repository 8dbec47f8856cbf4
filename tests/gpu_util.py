"""Helpers shared by the GPU parity tests: every call goes through the C ABI binding."""
import ctypes

import numpy as np
import torch

import ipex_llm.ggml.model.llama.llama_cpp as ggml

Q4_0, Q4_1, Q8_0, NF4, FP8 = 2, 3, 8, 10, 15
ALL = [Q4_0, Q4_1, Q8_0, NF4, FP8]
NAMES = {2: "sym_int4", 3: "asym_int4", 8: "sym_int8", 10: "nf4", 15: "fp8_e4m3"}
DT = {torch.float16: ggml.DT_F16, torch.bfloat16: ggml.DT_BF16, torch.float32: ggml.DT_F32}


def stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def weights(seed, shape, std=0.02, outliers=True):
    r = np.random.default_rng(seed)
    w = (r.standard_normal(shape) * std).astype(np.float32)
    if outliers:
        mask = r.random(shape) < 0.001
        w[mask] = np.where(r.random(int(mask.sum())) < 0.5, 0.5, -0.5)
    return w


def acts(seed, m, k, dtype):
    r = np.random.default_rng(seed)
    return torch.from_numpy(r.standard_normal((m, k)).astype(np.float32)).to(dtype)


def dev_quantize(w_np, qtype, layout):
    n, k = w_np.shape
    src = torch.from_numpy(w_np).cuda()
    dst = torch.empty(ggml.lowbit_blob_bytes(qtype, n * k), dtype=torch.uint8, device="cuda")
    ggml.lowbit_quantize(src.data_ptr(), dst.data_ptr(), qtype, n, k, layout, stream())
    torch.cuda.synchronize()
    return dst


def dev_relayout(blob, qtype, n, k, src_layout):
    dst = torch.empty_like(blob)
    ggml.lowbit_relayout(blob.data_ptr(), dst.data_ptr(), qtype, n, k, src_layout, stream())
    torch.cuda.synchronize()
    return dst


def dev_dequantize(blob, qtype, n, k, layout, dtype):
    out = torch.empty((n, k), dtype=dtype, device="cuda")
    ggml.lowbit_dequantize(blob.data_ptr(), out.data_ptr(), qtype, n, k, layout, DT[dtype], stream())
    torch.cuda.synchronize()
    return out


def dev_matmul(x, blob, qtype, layout, n, fn="forward", waves=0):
    m, k = x.shape
    xd = x.cuda().contiguous()
    y = torch.full((m, n), float("nan"), dtype=x.dtype, device="cuda")
    args = (xd.data_ptr(), blob.data_ptr(), y.data_ptr(), qtype, layout, DT[x.dtype], m, n, k)
    if fn == "forward":
        ggml.lowbit_forward(*args, stream())
    elif fn == "gemv":
        ggml.lowbit_gemv(*args, waves, stream())
    elif fn == "narrow":
        ggml.lowbit_gemm_narrow(*args, stream())
    else:
        ggml.lowbit_gemm(*args, stream())
    torch.cuda.synchronize()
    return y.float().cpu().numpy()
