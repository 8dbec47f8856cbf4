"""Every BASELINE configuration at its FULL size against the CPU oracle, through the C ABI.

The oracle cannot finish a full-size product in seconds, so each case checks a sample: the weight is
drawn and quantized on the GPU at full size, `N_ROWS` of its rows are re-quantized by the oracle from the
same fp32 values (their bytes must equal the corresponding rows of the GPU blob), and the oracle's
products of those rows with `M_ROWS` rows of x are compared with the same entries of the full GPU result.
The ggml blob is row-major, so a row slice of it is a valid blob of the sliced weight.

Tolerances: max-abs error <= 2e-3 (fp16) / 8e-3 (bf16) of max|y| against the exact product of the
dequantized weights, and <= 1e-2 * max|y_ref| against the reference-style CPU matmul (activations rounded
to int8 blocks, python/llm/src/ipex_llm/transformers/low_bit_linear.py:462-497).
"""
import numpy as np
import pytest
import torch

import ipex_llm.ggml.model.llama.llama_cpp as ggml
import lowbit_oracle as orc
from gpu_util import DT, FP8, NF4, Q4_0, Q4_1, Q8_0, stream

pytestmark = pytest.mark.gpu

GGML, TILED = 0, 1
N_ROWS, M_ROWS = 192, 24


def _gpu_weight(seed, n, k, std, outliers):
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    w = torch.randn((n, k), generator=g, device="cuda", dtype=torch.float32) * std
    if outliers:                                            # 0.1 % at +-0.5
        u = torch.rand((n, k), generator=g, device="cuda")
        w = torch.where(u < 0.0005, torch.full_like(w, 0.5), torch.where(u > 0.9995, torch.full_like(w, -0.5), w))
    return w


def _quantize_full(w, qtype):
    n, k = w.shape
    blob = torch.empty(ggml.lowbit_blob_bytes(qtype, n * k), dtype=torch.uint8, device="cuda")
    ggml.lowbit_quantize(w.data_ptr(), blob.data_ptr(), qtype, n, k, TILED, stream())
    flat = torch.empty_like(blob)
    ggml.lowbit_relayout(blob.data_ptr(), flat.data_ptr(), qtype, n, k, TILED, stream())
    torch.cuda.synchronize()
    return blob, flat


def _sample(seed, total, count):
    r = np.random.default_rng(seed)
    count = min(count, total)
    picks = set(r.choice(total, size=count, replace=False).tolist()) | {0, total - 1}
    return np.array(sorted(picks))


def _oracle_rows(w, flat, qtype, rows):
    """The oracle's blob of the sampled weight rows; asserts that the GPU wrote the same bytes."""
    n, k = w.shape
    row_bytes = orc.blob_bytes(qtype, k)
    want = orc.quantize(w[torch.from_numpy(rows).cuda()].cpu().numpy(), qtype)
    got = flat.view(n, row_bytes)[torch.from_numpy(rows).cuda()].cpu().numpy().reshape(-1)
    assert np.array_equal(got, want), "quantized bytes of the sampled rows differ from the oracle"
    return want


def _check(y, x, blob_rows, qtype, rows, m_rows, k, dtype, what):
    xf = x[torch.from_numpy(m_rows).cuda()].float().cpu().numpy()
    ys = y[torch.from_numpy(m_rows).cuda()][:, torch.from_numpy(rows).cuda()].float().cpu().numpy()
    exact = orc.mul_mat_exact(blob_rows, xf, (len(rows), k), qtype)
    ref = orc.mul_mat_q(blob_rows, xf, (len(rows), k), qtype)
    tol = 2e-3 if dtype == torch.float16 else 8e-3
    assert np.isfinite(ys).all(), what
    assert np.abs(ys - exact).max() <= tol * np.abs(exact).max(), what
    assert np.abs(ys - ref).max() <= 1e-2 * np.abs(ref).max(), what


def _forward(x, blob, qtype, n, dtype):
    """lowbit_forward_ws with the workspace the library asks for: what LowBitLinear.forward runs."""
    m, k = x.shape
    y = torch.full((m, n), float("nan"), dtype=dtype, device="cuda")
    ws_bytes = max(16, ggml.lowbit_workspace_bytes(m, n, k))
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")
    ggml.lowbit_forward_ws(x.data_ptr(), blob.data_ptr(), y.data_ptr(), qtype, TILED, DT[dtype], m, n, k,
                           ws.data_ptr(), ws_bytes, stream())
    torch.cuda.synchronize()
    assert not torch.isnan(y).any()
    return y


def _acts(seed, m, k, dtype):
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    return torch.randn((m, k), generator=g, device="cuda", dtype=torch.float32).to(dtype)


def _linear_case(seed, qtype, n, k, ms, dtype, std, outliers):
    w = _gpu_weight(seed, n, k, std, outliers)
    blob, flat = _quantize_full(w, qtype)
    rows = _sample(seed + 1, n, N_ROWS)
    blob_rows = _oracle_rows(w, flat, qtype, rows)
    del w, flat
    for m in ms:
        x = _acts(seed + 2 + m, m, k, dtype)
        y = _forward(x, blob, qtype, n, dtype)
        _check(y, x, blob_rows, qtype, rows, _sample(seed + 3, m, M_ROWS), k, dtype, (qtype, n, k, m))


# configs[1]: Llama-2-7B decode linears, sym_int4, fp16, M in {1, 4, 8}; weights N(0, 0.02) + 0.1 % outliers
@pytest.mark.parametrize("n,k", [(4096, 4096), (11008, 4096), (4096, 11008)])
def test_llama2_7b_decode_linears(n, k):
    _linear_case(9100 + n // 100 + k, Q4_0, n, k, (1, 4, 8), torch.float16, 0.02, True)


# configs[2]: the same shapes at prefill, M in {512, 2048}, sym_int4 and asym_int4, fp16
@pytest.mark.parametrize("qtype", [Q4_0, Q4_1])
@pytest.mark.parametrize("n,k", [(4096, 4096), (11008, 4096), (4096, 11008)])
def test_llama2_7b_prefill_linears(qtype, n, k):
    _linear_case(9200 + qtype + n // 100 + k, qtype, n, k, (512, 2048), torch.float16, 0.02, True)


# The gate and up projections of a Llama-2-7B MLP at prefill through the fused launch (lowbit_mlp_forward beyond
# 4 rows: what a converted model's MLP runs from 32 rows on): SiLU(x Wg^T) * (x Wu^T) against the oracle's exact
# products of sampled rows, one rounding of the result.
@pytest.mark.parametrize("qtype,dtype", [(Q4_0, torch.float16), (Q4_1, torch.bfloat16)])
def test_llama2_7b_prefill_fused_gate_up(qtype, dtype):
    n, k = 11008, 4096
    seed = 9250 + qtype
    wg, wu = _gpu_weight(seed, n, k, 0.02, True), _gpu_weight(seed + 1, n, k, 0.02, True)
    (bg, fg), (bu, fu) = _quantize_full(wg, qtype), _quantize_full(wu, qtype)
    rows = _sample(seed + 2, n, N_ROWS)
    rg, ru = _oracle_rows(wg, fg, qtype, rows), _oracle_rows(wu, fu, qtype, rows)
    del wg, wu, fg, fu
    for m in (40, 512, 2048):
        x = _acts(seed + 3 + m, m, k, dtype)
        y = torch.full((m, n), float("nan"), dtype=dtype, device="cuda")
        ggml.lowbit_mlp_forward(x.data_ptr(), bg.data_ptr(), bu.data_ptr(), y.data_ptr(), qtype, DT[dtype], m, n, k, 0, stream())
        torch.cuda.synchronize()
        assert not torch.isnan(y).any()
        m_rows = _sample(seed + 4, m, M_ROWS)
        xf = x[torch.from_numpy(m_rows).cuda()].float().cpu().numpy()
        ys = y[torch.from_numpy(m_rows).cuda()][:, torch.from_numpy(rows).cuda()].float().cpu().numpy()
        g = orc.mul_mat_exact(rg, xf, (len(rows), k), qtype)
        u = orc.mul_mat_exact(ru, xf, (len(rows), k), qtype)
        want = g / (1.0 + np.exp(-g)) * u
        tol = 2e-3 if dtype == torch.float16 else 8e-3
        assert np.abs(ys - want).max() <= tol * np.abs(want).max(), (qtype, m)


# configs[3]: Llama-3-70B linears, nf4 and sym_int8, bf16, M in {1, 16, 1024}; weights N(0, 0.015)
@pytest.mark.parametrize("qtype", [NF4, Q8_0])
@pytest.mark.parametrize("n,k", [(8192, 8192), (1024, 8192), (28672, 8192), (8192, 28672)])
def test_llama3_70b_linears(qtype, n, k):
    _linear_case(9300 + qtype + n // 100 + k, qtype, n, k, (1, 16, 1024), torch.bfloat16, 0.015, False)


# configs[4]: Mixtral-8x7B expert FFN, fp8_e4m3, 8 experts, 512 tokens, top-2, bf16, at full size as
# moe_ffn_grouped runs it: the fused gate/up launch (SiLU in its epilogue), then the down projection with the
# K-split workspace; the gate and up products also as plain grouped launches.  Every expert's sampled rows
# against the oracle on rows of x routed to it.
def test_mixtral_expert_ffn_full_size():
    n_exp, hid, ffn, tokens, top_k = 8, 4096, 14336, 512, 2
    dtype = torch.bfloat16
    g = torch.Generator(device="cuda")
    g.manual_seed(9400)
    logits = torch.randn((tokens, n_exp), generator=g, device="cuda")
    hidden = torch.randn((tokens, hid), generator=g, device="cuda").to(dtype)
    _, experts = torch.topk(torch.softmax(logits, dim=-1), top_k, dim=-1)
    flat_e = experts.reshape(-1)
    order = torch.argsort(flat_e, stable=True)
    counts = torch.bincount(flat_e, minlength=n_exp)
    offsets = torch.zeros(n_exp + 1, dtype=torch.int32, device="cuda")
    offsets[1:] = torch.cumsum(counts, 0).to(torch.int32)
    offs = offsets.cpu().numpy()
    rows_total = tokens * top_k
    xs = hidden[torch.div(order, top_k, rounding_mode="floor")].contiguous()

    def experts_of(n, k, seed):
        blobs, checks = [], []
        for e in range(n_exp):
            w = _gpu_weight(seed + e, n, k, 0.02, False)
            blob, flat = _quantize_full(w, FP8)
            rows = _sample(seed + 100 + e, n, 64)
            checks.append((rows, _oracle_rows(w, flat, FP8, rows)))
            blobs.append(blob)
            del w, flat
        ptrs = torch.tensor([b.data_ptr() for b in blobs], dtype=torch.int64, device="cuda")
        return blobs, ptrs, checks

    def m_sample(seed, e):
        r0, r1 = int(offs[e]), int(offs[e + 1])
        return r0 + _sample(seed + 200 + e, r1 - r0, 8) if r1 > r0 else None

    def plain(x, ptrs, checks, n, k, seed, with_workspace):
        y = torch.full((rows_total, n), float("nan"), dtype=dtype, device="cuda")
        if with_workspace:
            ws_bytes = ggml.lowbit_grouped_workspace_bytes(n_exp, rows_total, n, k)
            ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device="cuda")
            ggml.lowbit_grouped_forward_ws(x.data_ptr(), ptrs.data_ptr(), y.data_ptr(), offsets.data_ptr(), n_exp,
                                           rows_total, FP8, DT[dtype], n, k, ws.data_ptr(), ws_bytes, stream())
        else:
            ggml.lowbit_grouped_forward(x.data_ptr(), ptrs.data_ptr(), y.data_ptr(), offsets.data_ptr(), n_exp,
                                        rows_total, FP8, DT[dtype], n, k, stream())
        torch.cuda.synchronize()
        assert not torch.isnan(y).any()
        for e, (rows, blob_rows) in enumerate(checks):
            m_rows = m_sample(seed, e)
            if m_rows is not None:
                _check(y, x, blob_rows, FP8, rows, m_rows, k, dtype, ("expert", e, n, k, with_workspace))
        return y

    b1, p1, c1 = experts_of(ffn, hid, 9410)                    # w1 (gate)
    # w3 (up): the same sampled rows as w1, so that the fused output can be checked entry by entry
    b3, c3 = [], []
    for e in range(n_exp):
        w = _gpu_weight(9430 + e, ffn, hid, 0.02, False)
        blob, flat = _quantize_full(w, FP8)
        c3.append((c1[e][0], _oracle_rows(w, flat, FP8, c1[e][0])))
        b3.append(blob)
        del w, flat
    p3 = torch.tensor([b.data_ptr() for b in b3], dtype=torch.int64, device="cuda")
    plain(xs, p1, c1, ffn, hid, 9410, False)
    plain(xs, p3, c3, ffn, hid, 9430, False)

    h = torch.full((rows_total, ffn), float("nan"), dtype=dtype, device="cuda")
    ggml.lowbit_grouped_mlp_forward(xs.data_ptr(), p1.data_ptr(), p3.data_ptr(), h.data_ptr(), offsets.data_ptr(), n_exp,
                                    rows_total, FP8, DT[dtype], ffn, hid, 0, stream())
    torch.cuda.synchronize()
    assert not torch.isnan(h).any()
    for e in range(n_exp):
        m_rows = m_sample(9410, e)
        if m_rows is None:
            continue
        rows = c1[e][0]
        xf = xs[torch.from_numpy(m_rows).cuda()].float().cpu().numpy()
        gate = orc.mul_mat_exact(c1[e][1], xf, (len(rows), hid), FP8)
        up = orc.mul_mat_exact(c3[e][1], xf, (len(rows), hid), FP8)
        want = gate / (1.0 + np.exp(-gate)) * up
        got = h[torch.from_numpy(m_rows).cuda()][:, torch.from_numpy(rows).cuda()].float().cpu().numpy()
        assert np.abs(got - want).max() <= 8e-3 * np.abs(want).max(), ("fused gate/up, expert", e)
    del b1, b3

    b2, p2, c2 = experts_of(hid, ffn, 9450)                    # w2 (down), K = 14336
    assert ggml.lowbit_grouped_workspace_bytes(n_exp, rows_total, hid, ffn) > 0      # this shape splits K
    plain(h, p2, c2, hid, ffn, 9450, True)
    plain(h, p2, c2, hid, ffn, 9450, False)
