"""The batch-sized product (lowbit_gemm_ring) against the CPU oracle, through the C ABI, on a real MI355X."""
import numpy as np
import pytest
import torch

import ipex_llm.ggml.model.llama.llama_cpp as ggml
import lowbit_oracle as orc
from gpu_util import ALL, DT, NF4, Q4_0, Q4_1, Q8_0, acts, dev_matmul, dev_quantize, stream, weights

pytestmark = pytest.mark.gpu

GGML, TILED = 0, 1


def _ring(x, blob, qtype, n, wgs, ws=None, ws_bytes=None):
    m, k = x.shape
    xd = x.cuda().contiguous()
    y = torch.full((m, n), float("nan"), dtype=x.dtype, device="cuda")
    ggml.lowbit_gemm_ring(xd.data_ptr(), blob.data_ptr(), y.data_ptr(), qtype, TILED, DT[x.dtype], m, n, k,
                          ws.data_ptr() if ws is not None else None,
                          (ws.numel() if ws_bytes is None else ws_bytes) if ws is not None else 0, wgs, stream())
    torch.cuda.synchronize()
    return y.float().cpu().numpy()


def _tol(dtype):
    return 2e-3 if dtype == torch.float16 else 8e-3


# (m, n, k, wgs): one step of one tile; a tail tile with one tile row; runs that end inside a tile; 128-row
# blocks with empty rows; three row tiles; more workgroups than there are units; the library's choice
CASES = [(17, 256, 128, 1), (33, 272, 384, 2), (64, 1008, 1024, 3), (100, 528, 2048, 5), (300, 768, 512, 11),
         (32, 512, 256, 64), (24, 4096, 1024, 0)]


@pytest.mark.parametrize("qtype", ALL)
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("m,n,k,wgs", CASES)
def test_ring_against_oracle(qtype, dtype, m, n, k, wgs):
    w = weights(7000 + qtype + m, (n, k))
    x = acts(7001 + m, m, k, dtype)
    blob = dev_quantize(w, qtype, TILED)
    ws = torch.empty(64 << 20, dtype=torch.uint8, device="cuda")
    y = _ring(x, blob, qtype, n, wgs, ws)
    y_exact = orc.mul_mat_exact(orc.quantize(w, qtype), x.float().numpy(), (n, k), qtype)
    assert np.isfinite(y).all() and np.abs(y - y_exact).max() <= _tol(dtype) * np.abs(y_exact).max()


@pytest.mark.parametrize("qtype,dtype", [(Q4_0, torch.float16), (Q8_0, torch.bfloat16), (NF4, torch.float16)])
def test_ring_runs_that_span_several_tiles(qtype, dtype):
    # 8 tiles of 2 steps dealt to 3 workgroups: runs of 5, 5 and 6 units cross two tile boundaries each, so a
    # run holds whole tiles (written straight to y) between two partial ones (summed from the workspace)
    m, n, k = 32, 2048, 256
    w = weights(7100 + qtype, (n, k))
    x = acts(7101, m, k, dtype)
    blob = dev_quantize(w, qtype, TILED)
    ws = torch.empty(16 << 20, dtype=torch.uint8, device="cuda")
    y_exact = orc.mul_mat_exact(orc.quantize(w, qtype), x.float().numpy(), (n, k), qtype)
    for wgs in (3, 5, 7, 16):
        y = _ring(x, blob, qtype, n, wgs, ws)
        assert np.isfinite(y).all() and np.abs(y - y_exact).max() <= _tol(dtype) * np.abs(y_exact).max(), wgs


def test_ring_without_or_with_too_small_a_workspace_takes_whole_tiles():
    m, n, k, qtype = 48, 1024, 2048, Q4_1
    w = weights(7200, (n, k))
    x = acts(7201, m, k, torch.float16)
    blob = dev_quantize(w, qtype, TILED)
    y_exact = orc.mul_mat_exact(orc.quantize(w, qtype), x.float().numpy(), (n, k), qtype)
    y_none = _ring(x, blob, qtype, n, 0)
    assert np.abs(y_none - y_exact).max() <= 2e-3 * np.abs(y_exact).max()
    ws = torch.empty(1 << 20, dtype=torch.uint8, device="cuda")
    ws.fill_(0xff)                                              # NaN patterns: must stay unread
    y_small = _ring(x, blob, qtype, n, 0, ws, 4096)
    assert np.array_equal(y_small, y_none)
    # whole tiles are the plain accumulation order of the tiled GEMM
    assert np.array_equal(y_none, dev_matmul(x, blob, qtype, TILED, n, fn="gemm"))


def test_forward_ws_at_batch_sizes_against_oracle():
    # whichever kernel lowbit_forward_ws picks between M = 17 and 512, with the workspace it asks for
    qtype, n, k = Q4_0, 4096, 4096
    w = weights(7300, (n, k))
    blob = dev_quantize(w, qtype, TILED)
    q = orc.quantize(w, qtype)
    for m in (17, 40, 64, 129, 512):
        x = acts(7301 + m, m, k, torch.float16)
        need = ggml.lowbit_workspace_bytes(m, n, k)
        ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
        y = torch.full((m, n), float("nan"), dtype=torch.float16, device="cuda")
        ggml.lowbit_forward_ws(x.cuda().data_ptr(), blob.data_ptr(), y.data_ptr(), qtype, TILED, 0, m, n, k,
                               ws.data_ptr(), need, stream())
        torch.cuda.synchronize()
        y_exact = orc.mul_mat_exact(q, x.float().numpy(), (n, k), qtype)
        assert np.abs(y.float().cpu().numpy() - y_exact).max() <= 2e-3 * np.abs(y_exact).max(), m


def test_ring_full_size_agrees_with_the_decode_kernel():
    # Llama-2-7B gate projection at batch 32 and 128: too large for the oracle in a test, so the two
    # independent kernels are compared with each other (different summation orders: a few ulps of fp16)
    qtype, n, k = Q4_0, 11008, 4096
    w = torch.randn((n, k), device="cuda") * 0.02
    blob = torch.empty(ggml.lowbit_blob_bytes(qtype, n * k), dtype=torch.uint8, device="cuda")
    ggml.lowbit_quantize(w.data_ptr(), blob.data_ptr(), qtype, n, k, TILED, stream())
    ws = torch.empty(64 << 20, dtype=torch.uint8, device="cuda")
    for m in (32, 128):
        x = (torch.randn((m, k), device="cuda")).half()
        y_ring = torch.empty((m, n), dtype=torch.float16, device="cuda")
        y_gemv = torch.empty_like(y_ring)
        ggml.lowbit_gemm_ring(x.data_ptr(), blob.data_ptr(), y_ring.data_ptr(), qtype, TILED, 0, m, n, k, ws.data_ptr(),
                              ws.numel(), 0, stream())
        ggml.lowbit_gemv(x.data_ptr(), blob.data_ptr(), y_gemv.data_ptr(), qtype, TILED, 0, m, n, k, 0, stream())
        torch.cuda.synchronize()
        d = (y_ring.float() - y_gemv.float()).abs().max().item()
        assert d <= 2e-3 * y_gemv.float().abs().max().item()


def test_ring_vocabulary_sized_weight_agrees_with_the_decode_kernel():
    # an lm_head: 125 tiles of 256 rows dealt to 256 workgroups, and K = 11008 (86 steps) with a row
    # count that leaves the last 32-row block of x partly empty
    qtype = Q4_0
    ws = torch.empty(96 << 20, dtype=torch.uint8, device="cuda")
    for m, n, k in ((40, 32000, 4096), (100, 4096, 11008)):
        w = torch.randn((n, k), device="cuda") * 0.02
        blob = torch.empty(ggml.lowbit_blob_bytes(qtype, n * k), dtype=torch.uint8, device="cuda")
        ggml.lowbit_quantize(w.data_ptr(), blob.data_ptr(), qtype, n, k, TILED, stream())
        x = (torch.randn((m, k), device="cuda")).bfloat16()
        y_ring = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
        y_gemv = torch.empty_like(y_ring)
        ggml.lowbit_gemm_ring(x.data_ptr(), blob.data_ptr(), y_ring.data_ptr(), qtype, TILED, 1, m, n, k, ws.data_ptr(),
                              ws.numel(), 0, stream())
        ggml.lowbit_gemv(x.data_ptr(), blob.data_ptr(), y_gemv.data_ptr(), qtype, TILED, 1, m, n, k, 0, stream())
        torch.cuda.synchronize()
        d = (y_ring.float() - y_gemv.float()).abs().max().item()
        assert d <= 8e-3 * y_gemv.float().abs().max().item()


def test_ring_rejects_bad_arguments():
    m, n, k, qtype = 32, 256, 256, Q4_0
    w = weights(7400, (n, k))
    x = acts(7401, m, k, torch.float16).cuda()
    tiled = dev_quantize(w, qtype, TILED)
    flat = dev_quantize(w, qtype, GGML)
    y = torch.empty((m, n + 1), dtype=torch.float16, device="cuda")
    ok = (x.data_ptr(), tiled.data_ptr(), y.data_ptr(), qtype, TILED, 0, m, n, k, None, 0, 0, stream())

    def bad(i, v, match):
        a = list(ok)
        a[i] = v
        with pytest.raises(RuntimeError, match=match):
            ggml.lowbit_gemm_ring(*a)
    bad(4, GGML, "tiled")                                       # the ggml layout has no tiles to fetch
    bad(1, flat.data_ptr() + 2, "misaligned")
    bad(2, y.data_ptr() + 2, "8-byte")
    bad(11, -1, "wgs")
    bad(5, 2, "f16 or bf16")
    bad(9, x.data_ptr() + 4, "workspace")
    ggml.lowbit_gemm_ring(*ok)
    torch.cuda.synchronize()


def test_forward_ws_random_shapes_against_oracle():
    # whatever kernel the library picks for 40 seeded random problems (all qtypes, both activation types,
    # M from 1 to 600, ragged N and K in tile units), with the workspace it asks for
    rng = np.random.default_rng(77)
    for case in range(40):
        qtype = ALL[case % len(ALL)]
        dtype = (torch.float16, torch.bfloat16)[(case // len(ALL)) % 2]
        m = int(rng.choice([1, 3, 16, 17, 31, 33, 64, 65, 100, 128, 129, 200, 257, 400, 512, 600]))
        n = 16 * int(rng.integers(1, 65))
        k = 128 * int(rng.integers(1, 17))
        w = weights(9000 + case, (n, k))
        x = acts(9100 + case, m, k, dtype)
        blob = dev_quantize(w, qtype, TILED)
        need = ggml.lowbit_workspace_bytes(m, n, k)
        ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
        y = torch.full((m, n), float("nan"), dtype=dtype, device="cuda")
        ggml.lowbit_forward_ws(x.cuda().data_ptr(), blob.data_ptr(), y.data_ptr(), qtype, TILED, DT[dtype], m, n, k,
                               ws.data_ptr(), need, stream())
        torch.cuda.synchronize()
        y_exact = orc.mul_mat_exact(orc.quantize(w, qtype), x.float().numpy(), (n, k), qtype)
        got = y.float().cpu().numpy()
        assert np.isfinite(got).all(), (case, qtype, m, n, k)
        assert np.abs(got - y_exact).max() <= _tol(dtype) * np.abs(y_exact).max(), (case, qtype, m, n, k)
