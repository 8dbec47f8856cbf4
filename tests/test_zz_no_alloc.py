"""lowbit_forward_noalloc (the entry point that allocates nothing) against lowbit_forward_ws, through the C ABI.

Both run the same kernels; one takes its workspace from the caller, the other from the scratch array inside
the library.  The outputs must be identical bit for bit, on consecutive calls that share the scratch (the
second smaller than the first, so that stale partial tiles of the first call lie beyond what it writes),
and the parity bar against the CPU oracle holds for the no-alloc result itself.
"""
import numpy as np
import pytest
import torch

import ipex_llm.ggml.model.llama.llama_cpp as ggml
import lowbit_oracle as orc
from gpu_util import DT, NF4, Q4_0, Q8_0, acts, dev_quantize, stream, weights

pytestmark = pytest.mark.gpu

TILED = 1


def _both(x, blob, qtype, n):
    m, k = x.shape
    xd = x.cuda().contiguous()
    need = ggml.lowbit_workspace_bytes(m, n, k)
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
    y_ws = torch.full((m, n), float("nan"), dtype=x.dtype, device="cuda")
    y_na = torch.full((m, n), float("nan"), dtype=x.dtype, device="cuda")
    ggml.lowbit_forward_ws(xd.data_ptr(), blob.data_ptr(), y_ws.data_ptr(), qtype, TILED, DT[x.dtype], m, n, k,
                           ws.data_ptr() if need else None, need, stream())
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    ggml.lowbit_forward_noalloc(xd.data_ptr(), blob.data_ptr(), y_na.data_ptr(), qtype, TILED, DT[x.dtype], m, n, k,
                                stream())
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before        # the driver handed out no memory during the call
    return y_ws, y_na, need


# (qtype, dtype, m, n, k) in call order: a batch-sized product whose tiles are cut along K (partial tiles
# through the scratch), then a smaller one, then a prefill-sized one that splits K, then one that needs no
# workspace at all
CALLS = [(Q4_0, torch.float16, 128, 11008, 4096), (Q4_0, torch.float16, 40, 8192, 2048),
         (Q8_0, torch.bfloat16, 520, 1024, 4096), (NF4, torch.bfloat16, 100, 528, 2048),
         (Q4_0, torch.float16, 4, 1024, 512)]


def test_noalloc_equals_forward_ws_on_consecutive_calls():
    assert ggml.lowbit_noalloc_scratch_bytes() == 64 << 20
    used_scratch = 0
    for i, (qtype, dtype, m, n, k) in enumerate(CALLS):
        w = weights(9600 + i, (n, k))
        x = acts(9700 + i, m, k, dtype)
        blob = dev_quantize(w, qtype, TILED)
        y_ws, y_na, need = _both(x, blob, qtype, n)
        used_scratch += need > 0
        assert not torch.isnan(y_na).any()
        assert torch.equal(y_ws, y_na), (i, qtype, m, n, k)
        # the parity bar itself, on sampled rows of W so that the oracle stays fast
        rows = np.unique(np.linspace(0, n - 1, 96).astype(np.int64))
        blob_rows = orc.quantize(w[rows], qtype)
        xf = x.float().numpy()[: min(m, 16)]
        got = y_na[: min(m, 16)][:, torch.from_numpy(rows).cuda()].float().cpu().numpy()
        exact = orc.mul_mat_exact(blob_rows, xf, (len(rows), k), qtype)
        ref = orc.mul_mat_q(blob_rows, xf, (len(rows), k), qtype)
        tol = 2e-3 if dtype == torch.float16 else 8e-3
        assert np.abs(got - exact).max() <= tol * np.abs(exact).max()
        assert np.abs(got - ref).max() <= 1e-2 * np.abs(ref).max()
    assert used_scratch >= 3                                  # the cases above do go through the scratch


def test_noalloc_rejects_a_shape_beyond_its_scratch():
    m, n, k = 768, 8192, 28672
    assert ggml.lowbit_workspace_bytes(m, n, k) > ggml.lowbit_noalloc_scratch_bytes()
    blob = torch.zeros(ggml.lowbit_blob_bytes(Q4_0, n * k), dtype=torch.uint8, device="cuda")
    x = torch.zeros((m, k), dtype=torch.float16, device="cuda")
    y = torch.zeros((m, n), dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError, match="scratch"):
        ggml.lowbit_forward_noalloc(x.data_ptr(), blob.data_ptr(), y.data_ptr(), Q4_0, TILED, DT[torch.float16], m, n, k,
                                    stream())
    torch.cuda.synchronize()
