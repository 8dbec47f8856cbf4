"""HIP path against the CPU oracle, through the C ABI, on a real MI355X."""
import numpy as np
import pytest
import torch

import ipex_llm.ggml.model.llama.llama_cpp as ggml
import lowbit_oracle as orc
from gpu_util import (ALL, DT, FP8, NF4, Q4_0, Q4_1, Q8_0, acts, dev_dequantize, dev_matmul, dev_quantize,
                      dev_relayout, stream, weights)

pytestmark = pytest.mark.gpu

GGML, TILED = 0, 1


# ------------------------------------------------------------------ quantizer: bit exact

@pytest.mark.parametrize("qtype", ALL)
@pytest.mark.parametrize("shape", [(16, 128), (64, 512), (3, 128), (272, 1408), (1024, 4096)])
def test_quantize_bytes_match_oracle(qtype, shape):
    w = weights(1000 + qtype + shape[0], shape)
    got = dev_quantize(w, qtype, GGML).cpu().numpy()
    want = orc.quantize(w, qtype)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("qtype", ALL)
def test_quantize_edge_blocks(qtype):
    qk = orc.qk_size(qtype)
    rows = []
    rows.append(np.zeros(qk))                                   # all zero
    rows.append(np.full(qk, 0.75))                              # constant
    r = np.random.default_rng(5)
    a = r.standard_normal(qk) * 0.02
    a[3], a[qk - 2] = 0.4, -0.4                                 # +max first, same |.| later
    rows.append(a)
    b = a.copy()
    b[3], b[qk - 2] = -0.4, 0.4
    rows.append(b)
    rows.append(np.tile(np.arange(-8, 8), qk // 16) * 0.125)    # exact ramp
    rows.append(r.standard_normal(qk) * 1e-7)                   # tiny: fp16 subnormal scale
    rows.append(r.standard_normal(qk) * 3e4)                    # huge: scale near fp16 max
    c = np.zeros(qk)
    c[0] = 1.0
    c[1:9] = (np.arange(8) + 0.5) / 8.0                         # exact .5 ties for sym_int4
    rows.append(c)
    w = np.stack(rows).astype(np.float32)
    got = dev_quantize(w, qtype, GGML).cpu().numpy()
    assert np.array_equal(got, orc.quantize(w, qtype))


@pytest.mark.parametrize("qtype", ALL)
def test_tiled_quantize_equals_relayout_and_round_trips(qtype):
    n, k = 48, 640
    w = weights(2000 + qtype, (n, k))
    g = dev_quantize(w, qtype, GGML)
    t = dev_quantize(w, qtype, TILED)
    t2 = dev_relayout(g, qtype, n, k, GGML)
    assert torch.equal(t, t2)
    assert not torch.equal(t, g)
    back = dev_relayout(t, qtype, n, k, TILED)
    assert torch.equal(back, g)
    assert np.array_equal(back.cpu().numpy(), orc.quantize(w, qtype))


# ---------------------------------------------------------------- dequantizer

@pytest.mark.parametrize("qtype", ALL)
@pytest.mark.parametrize("layout", [GGML, TILED])
def test_dequantize_fp32_bit_exact(qtype, layout):
    n, k = 32, 512
    w = weights(3000 + qtype, (n, k))
    blob = dev_quantize(w, qtype, layout)
    got = dev_dequantize(blob, qtype, n, k, layout, torch.float32).cpu().numpy()
    want = orc.dequantize(orc.quantize(w, qtype), qtype, (n, k))
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("qtype", ALL)
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_dequantize_half_types_are_rounded_fp32(qtype, dtype):
    n, k = 16, 256
    w = weights(3100 + qtype, (n, k))
    blob = dev_quantize(w, qtype, TILED)
    got = dev_dequantize(blob, qtype, n, k, TILED, dtype).cpu()
    want = torch.from_numpy(orc.dequantize(orc.quantize(w, qtype), qtype, (n, k))).to(dtype)
    assert torch.equal(got, want)


# -------------------------------------------------------------------- matmul

def _tol(dtype, qtype):
    # output rounding (2^-11 / 2^-8 of |y|) plus accumulation order; nf4 in bf16 also rounds its
    # code book to 8 bits.  All far inside the 1e-2 * max|y| budget of the parity bar.
    if dtype == torch.float16:
        return 1.5e-3
    return 8e-3 if qtype == NF4 else 6e-3


@pytest.mark.parametrize("qtype", ALL)
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("m", [1, 2, 4, 5, 8, 9, 16])
def test_gemv_tiled_against_oracle(qtype, dtype, m):
    n, k = 96, 1024
    w = weights(4000 + qtype, (n, k))
    x = acts(4100 + m, m, k, dtype)
    blob_np = orc.quantize(w, qtype)
    blob = dev_quantize(w, qtype, TILED)
    y = dev_matmul(x, blob, qtype, TILED, n, fn="gemv")
    xf = x.float().numpy()
    y_exact = orc.mul_mat_exact(blob_np, xf, (n, k), qtype)
    y_ref = orc.mul_mat_q(blob_np, xf, (n, k), qtype)       # the reference's CPU low-bit matmul
    assert np.isfinite(y).all()
    assert np.abs(y - y_exact).max() <= _tol(dtype, qtype) * np.abs(y_exact).max()
    assert np.abs(y - y_ref).max() <= 1e-2 * np.abs(y_ref).max()


@pytest.mark.parametrize("qtype", ALL)
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("m", [1, 2, 3, 4])
def test_gemv_four_tiles_per_wave_against_oracle(qtype, dtype, m):
    """Up to four rows of x on a weight with at least 8192 rows and K <= 4096 take the shape of the kernel with four
    tiles per wave (the metric's [11008 x 4096] does): K = 640 leaves a wave's last tiles past the end."""
    n, k = 8192, 640
    w = weights(4400 + qtype, (n, k))
    x = acts(4500 + m, m, k, dtype)
    blob_np = orc.quantize(w, qtype)
    blob = dev_quantize(w, qtype, TILED)
    y = dev_matmul(x, blob, qtype, TILED, n, fn="gemv")
    y_exact = orc.mul_mat_exact(blob_np, x.float().numpy(), (n, k), qtype)
    assert np.isfinite(y).all()
    assert np.abs(y - y_exact).max() <= _tol(dtype, qtype) * np.abs(y_exact).max()


@pytest.mark.parametrize("qtype", ALL)
@pytest.mark.parametrize("waves", [1, 3, 16])
def test_gemv_any_wave_count(qtype, waves):
    n, k = 32, 896      # 7 tiles along K: uneven split over the waves
    w = weights(4200 + qtype, (n, k))
    x = acts(4300, 3, k, torch.float16)
    blob = dev_quantize(w, qtype, TILED)
    y = dev_matmul(x, blob, qtype, TILED, n, fn="gemv", waves=waves)
    y_exact = orc.mul_mat_exact(orc.quantize(w, qtype), x.float().numpy(), (n, k), qtype)
    assert np.abs(y - y_exact).max() <= 1.5e-3 * np.abs(y_exact).max()


@pytest.mark.parametrize("qtype", ALL)
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_generic_kernel_on_untileable_shapes(qtype, dtype):
    qk = orc.qk_size(qtype)
    n, k = 37, qk * 3
    w = weights(4400 + qtype, (n, k))
    x = acts(4500, 5, k, dtype)
    blob = dev_quantize(w, qtype, GGML)
    y = dev_matmul(x, blob, qtype, GGML, n)
    y_exact = orc.mul_mat_exact(orc.quantize(w, qtype), x.float().numpy(), (n, k), qtype)
    assert np.abs(y - y_exact).max() <= _tol(dtype, qtype) * np.abs(y_exact).max()


@pytest.mark.parametrize("qtype", ALL)
def test_forward_m_above_16(qtype):
    n, k = 64, 512
    w = weights(4600 + qtype, (n, k))
    x = acts(4700, 40, k, torch.float16)
    blob = dev_quantize(w, qtype, TILED)
    y = dev_matmul(x, blob, qtype, TILED, n)
    y_exact = orc.mul_mat_exact(orc.quantize(w, qtype), x.float().numpy(), (n, k), qtype)
    assert np.abs(y - y_exact).max() <= 1.5e-3 * np.abs(y_exact).max()


def test_headline_shape_sym_int4_m1():
    # BASELINE configs[0]: [4096, 4096] sym_int4, M = 1, fp16
    n = k = 4096
    w = weights(1001, (n, k), outliers=False)
    x = acts(1002, 1, k, torch.float16)
    blob = dev_quantize(w, Q4_0, TILED)
    blob_np = orc.quantize(w, Q4_0)
    assert np.array_equal(dev_relayout(blob, Q4_0, n, k, TILED).cpu().numpy(), blob_np)
    y = dev_matmul(x, blob, Q4_0, TILED, n)
    xf = x.float().numpy()
    y_exact = orc.mul_mat_exact(blob_np, xf, (n, k), Q4_0)
    y_ref = orc.mul_mat_q(blob_np, xf, (n, k), Q4_0)
    assert np.abs(y - y_exact).max() <= 1.5e-3 * np.abs(y_exact).max()
    assert np.abs(y - y_ref).max() <= 1e-2 * np.abs(y_ref).max()


# ------------------------------------------------------------------ MFMA GEMM (prefill)

@pytest.mark.parametrize("qtype", ALL)
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("m,n,k", [(17, 64, 128), (128, 256, 512), (200, 272, 384), (513, 512, 1024)])
def test_gemm_against_oracle(qtype, dtype, m, n, k):
    w = weights(5000 + qtype + m, (n, k))
    x = acts(5100 + m, m, k, dtype)
    blob_np = orc.quantize(w, qtype)
    blob = dev_quantize(w, qtype, TILED)
    y = dev_matmul(x, blob, qtype, TILED, n, fn="gemm")
    xf = x.float().numpy()
    y_exact = orc.mul_mat_exact(blob_np, xf, (n, k), qtype)
    assert np.isfinite(y).all()
    tol = 2e-3 if dtype == torch.float16 else 8e-3
    assert np.abs(y - y_exact).max() <= tol * np.abs(y_exact).max()
    if m <= 128:
        y_ref = orc.mul_mat_q(blob_np, xf, (n, k), qtype)
        assert np.abs(y - y_ref).max() <= 1e-2 * np.abs(y_ref).max()


# (m, n, k): half tiles with a tail (65 rows: 64 + 1), a weight of one narrow tile and a half, full tiles with an
# odd number of K steps, three row tiles with a tail of 44 rows, more narrow tiles than the half-tile limit
NARROW_CASES = [(65, 144, 256), (128, 192, 128), (100, 272, 384), (300, 1008, 1024), (513, 2064, 512)]


@pytest.mark.parametrize("qtype", ALL)
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("m,n,k", NARROW_CASES)
def test_gemm_narrow_tiles_against_oracle(qtype, dtype, m, n, k):
    w = weights(5600 + qtype + m, (n, k))
    x = acts(5601 + m, m, k, dtype)
    blob_np = orc.quantize(w, qtype)
    blob = dev_quantize(w, qtype, TILED)
    y = dev_matmul(x, blob, qtype, TILED, n, fn="narrow")
    y_exact = orc.mul_mat_exact(blob_np, x.float().numpy(), (n, k), qtype)
    assert np.isfinite(y).all()
    tol = 2e-3 if dtype == torch.float16 else 8e-3
    assert np.abs(y - y_exact).max() <= tol * np.abs(y_exact).max()


def test_gemm_narrow_tiles_at_full_size_agree_with_the_decode_kernel():
    # [4096 x 4096] at M = 512 and 1024 (256 half tiles; 256 tiles): where lowbit_forward_ws picks this form
    n = k = 4096
    w = weights(5610, (n, k))
    blob = dev_quantize(w, Q4_0, TILED)
    for m in (512, 1024):
        x = acts(5611 + m, m, k, torch.float16)
        y = dev_matmul(x, blob, Q4_0, TILED, n, fn="narrow")
        rows = [0, 63, 64, 127, 128, m - 1]
        yv = dev_matmul(x[rows], blob, Q4_0, TILED, n, fn="gemv")
        assert np.abs(y[rows] - yv).max() <= 2e-3 * np.abs(yv).max()


def test_gemm_prefill_shape_sym_and_asym_int4():
    # one Llama-2-7B linear at prefill length: [4096 x 4096], M = 512, fp16 (BASELINE configs[2])
    n = k = 4096
    m = 512
    x = acts(5201, m, k, torch.float16)
    for qtype in (Q4_0, Q4_1):
        w = weights(5200 + qtype, (n, k))
        blob_np = orc.quantize(w, qtype)
        blob = dev_quantize(w, qtype, TILED)
        y = dev_matmul(x, blob, qtype, TILED, n)
        # oracle on a slice of the outputs keeps the CPU side to seconds
        rows = np.arange(0, m, 37)
        wd = orc.dequantize(blob_np, qtype, (n, k)).astype(np.float64)
        y_exact = x.float().numpy()[rows].astype(np.float64) @ wd.T
        assert np.abs(y[rows] - y_exact).max() <= 2e-3 * np.abs(y_exact).max()


@pytest.mark.parametrize("qtype,dtype", [(Q4_0, torch.float16), (Q4_1, torch.bfloat16), (Q8_0, torch.float16),
                                         (NF4, torch.bfloat16), (FP8, torch.bfloat16)])
def test_gemm_with_more_tiles_than_cus_against_oracle(qtype, dtype):
    # 10 x 28 = 280 tiles of 128 x 256: the form of the GEMM with two workgroups per CU; M leaves a tail
    # tile of 48 rows (two 32-row blocks), K = 384 is an odd number of 128-column steps
    m, n, k = 1200, 7168, 384
    w = weights(5300 + qtype, (n, k))
    x = acts(5301, m, k, dtype)
    blob_np = orc.quantize(w, qtype)
    blob = dev_quantize(w, qtype, TILED)
    y = dev_matmul(x, blob, qtype, TILED, n, fn="gemm")
    y_exact = orc.mul_mat_exact(blob_np, x.float().numpy(), (n, k), qtype)
    assert np.isfinite(y).all()
    tol = 2e-3 if dtype == torch.float16 else 8e-3
    assert np.abs(y - y_exact).max() <= tol * np.abs(y_exact).max()


def test_gemm_tail_tile_of_at_most_32_rows():
    m, n, k = 1040, 7168, 256            # 8 full row tiles + one of 16 rows: the one-block copy of the loop
    w = weights(5310, (n, k))
    x = acts(5311, m, k, torch.float16)
    blob = dev_quantize(w, Q4_0, TILED)
    y = dev_matmul(x, blob, Q4_0, TILED, n, fn="gemm")
    y_exact = orc.mul_mat_exact(orc.quantize(w, Q4_0), x.float().numpy(), (n, k), Q4_0)
    assert np.abs(y - y_exact).max() <= 2e-3 * np.abs(y_exact).max()


def test_full_size_prefill_agrees_with_the_decode_kernel_and_is_linear():
    """BASELINE configs[2] at full size ([11008 x 4096], M = 2048), where the oracle would take
    minutes: the GEMM must agree with the (oracle-checked) GEMV on sampled rows, and be linear in x."""
    n, k, m = 11008, 4096, 2048
    w = weights(5320, (n, k))
    blob = dev_quantize(w, Q4_0, TILED)
    x = acts(5321, m, k, torch.float16)
    y = dev_matmul(x, blob, Q4_0, TILED, n, fn="gemm")
    rows = [0, 1, 127, 128, 1000, 2047]
    yv = dev_matmul(x[rows], blob, Q4_0, TILED, n, fn="gemv")
    assert np.abs(y[rows] - yv).max() <= 2e-3 * np.abs(yv).max()
    # power-of-two scalings and the sign of x commute with the product up to rounding: the MFMA's
    # internal fp32 accumulation is not sign-symmetric (seen as ~1e-7 differences where the sum cancels
    # to almost nothing), so allow that plus the final fp16 rounding step
    slack = 2 * np.maximum(np.abs(y) * 2.0 ** -10, 2.0 ** -24) + 1e-6 * np.abs(y).max()
    y2 = dev_matmul(x * 2, blob, Q4_0, TILED, n, fn="gemm")
    assert (np.abs(y2 - 2 * y) <= 2 * slack).all() and (y2 == 2 * y).mean() > 0.999
    yn = dev_matmul(-x, blob, Q4_0, TILED, n, fn="gemm")
    assert (np.abs(yn + y) <= slack).all() and (yn == -y).mean() > 0.999
    # a row of the oracle for good measure
    want = orc.mul_mat_exact(orc.quantize(w, Q4_0), x[5:6].float().numpy(), (n, k), Q4_0)
    assert np.abs(y[5:6] - want).max() <= 2e-3 * np.abs(want).max()


def test_device_entry_points_reject_bad_arguments():
    blob = dev_quantize(weights(5330, (32, 256)), Q4_0, TILED)
    x = acts(5331, 2, 256, torch.float16).cuda()
    y = torch.empty((2, 32), dtype=torch.float16, device="cuda")
    ok = (x.data_ptr(), blob.data_ptr(), y.data_ptr(), Q4_0, TILED, DT[torch.float16], 2, 32, 256)
    ggml.lowbit_forward(*ok, stream())
    bad = {"qtype": (3, 99), "layout": (4, 7), "dtype": (5, 2), "M": (6, -1), "K": (8, 250), "x": (0, 0),
           "x alignment": (0, x.data_ptr() + 2)}
    for what, (pos, val) in bad.items():
        args = list(ok)
        args[pos] = val
        with pytest.raises(RuntimeError):
            ggml.lowbit_forward(*args, stream())
    with pytest.raises(RuntimeError, match="tiled"):           # 24 rows cannot be tiled
        ggml.lowbit_forward(x.data_ptr(), blob.data_ptr(), y.data_ptr(), Q4_0, TILED, DT[torch.float16], 2, 24, 256,
                            stream())
    # the dequantizers store 16 bytes per lane: a misaligned destination is refused, not mis-stored
    out = torch.empty(32 * 256 + 8, dtype=torch.float16, device="cuda")
    rows = torch.zeros(4, dtype=torch.int64, device="cuda")
    ggml.lowbit_dequantize(blob.data_ptr(), out.data_ptr(), Q4_0, 32, 256, TILED, DT[torch.float16], stream())
    with pytest.raises(RuntimeError, match="misaligned"):
        ggml.lowbit_dequantize(blob.data_ptr(), out.data_ptr() + 2, Q4_0, 32, 256, TILED, DT[torch.float16], stream())
    with pytest.raises(RuntimeError, match="misaligned"):
        ggml.lowbit_dequantize_rows(blob.data_ptr(), rows.data_ptr(), 4, out.data_ptr() + 8, Q4_0, 32, 256, TILED,
                                    DT[torch.float16], stream())
    # empty problems are no-ops
    ggml.lowbit_forward(x.data_ptr(), blob.data_ptr(), y.data_ptr(), Q4_0, TILED, DT[torch.float16], 0, 32, 256, stream())
    ggml.lowbit_forward(x.data_ptr(), blob.data_ptr(), y.data_ptr(), Q4_0, TILED, DT[torch.float16], 2, 0, 256, stream())
    torch.cuda.synchronize()


@pytest.mark.parametrize("qtype,n,k", [(NF4, 8192, 28672), (Q8_0, 28672, 8192), (NF4, 1024, 8192)])
@pytest.mark.parametrize("m", [1, 16])
def test_llama3_70b_shapes_decode_against_oracle(qtype, n, k, m):
    # BASELINE configs[3] at full size (bf16 activations); long K runs several rounds of the K walk
    w = weights(5400 + qtype, (n, k), std=0.015, outliers=False)
    x = acts(5401 + m, m, k, torch.bfloat16)
    blob = dev_quantize(w, qtype, TILED)
    y = dev_matmul(x, blob, qtype, TILED, n)
    y_exact = orc.mul_mat_exact(orc.quantize(w, qtype), x.float().numpy(), (n, k), qtype)
    assert np.abs(y - y_exact).max() <= 8e-3 * np.abs(y_exact).max()


@pytest.mark.parametrize("qtype,dtype", [(Q4_0, torch.float16), (Q8_0, torch.bfloat16), (NF4, torch.bfloat16)])
@pytest.mark.parametrize("m,n,k,splits", [(48, 1024, 4096, 8), (200, 272, 1408, 3), (512, 4096, 2048, 2),
                                          (130, 11008, 1024, 4), (300, 7168, 896, 7), (96, 512, 4096, 16)])
def test_split_k_gemm_against_oracle(qtype, dtype, m, n, k, splits):
    # K split over several workgroups per tile, partial sums through a workspace; ragged splits
    # (11 steps in 3, 7 steps in 7), both forms of the kernel, tail row tiles
    w = weights(5500 + qtype + m, (n, k))
    x = acts(5501 + m, m, k, dtype)
    blob = dev_quantize(w, qtype, TILED)
    xd = x.cuda()
    ws_bytes = splits * -(-m // 128) * -(-n // 256) * 128 * 256 * 4
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")

    def run(entry, *tail):
        y = torch.full((m, n), float("nan"), dtype=dtype, device="cuda")
        entry(xd.data_ptr(), blob.data_ptr(), y.data_ptr(), qtype, TILED, DT[dtype], m, n, k, *tail, stream())
        torch.cuda.synchronize()
        return y.float().cpu().numpy()
    y = run(ggml.lowbit_gemm_ws, ws.data_ptr(), ws_bytes, splits)
    y_exact = orc.mul_mat_exact(orc.quantize(w, qtype), x.float().numpy(), (n, k), qtype)
    tol = 2e-3 if dtype == torch.float16 else 8e-3
    assert np.isfinite(y).all() and np.abs(y - y_exact).max() <= tol * np.abs(y_exact).max()
    # one split is the plain kernel, bit for bit; an automatic choice and forward agree with the oracle too
    assert np.array_equal(run(ggml.lowbit_gemm_ws, ws.data_ptr(), ws_bytes, 1), dev_matmul(x, blob, qtype, TILED, n, fn="gemm"))
    for y_auto in (run(ggml.lowbit_gemm_ws, ws.data_ptr(), ws_bytes, 0), run(ggml.lowbit_forward_ws, ws.data_ptr(), ws_bytes)):
        assert np.abs(y_auto - y_exact).max() <= tol * np.abs(y_exact).max()
    with pytest.raises(RuntimeError, match="workspace"):
        run(ggml.lowbit_gemm_ws, ws.data_ptr(), ws_bytes - 16, splits)


def test_workspace_query_is_consistent():
    for m, n, k in [(256, 4096, 11008), (64, 28672, 8192), (2048, 11008, 4096), (8, 4096, 4096)]:
        b = ggml.lowbit_workspace_bytes(m, n, k)
        assert b % (32 * 256 * 4) == 0                              # whole partial tiles of either kernel
    assert ggml.lowbit_workspace_bytes(256, 4096, 11008) > 0        # 32 tiles, 86 steps: worth splitting
    assert ggml.lowbit_workspace_bytes(2048, 11008, 4096) == 0      # 688 tiles fill the machine


@pytest.mark.parametrize("qtype,dtype", [(Q4_0, torch.float16), (Q4_1, torch.float16), (Q8_0, torch.bfloat16),
                                         (NF4, torch.bfloat16), (FP8, torch.bfloat16)])
@pytest.mark.parametrize("m,n,k", [(1024, 16384, 256), (512, 33024, 384), (768, 22016, 128)])
def test_gemm_tall_row_tiles_against_oracle(qtype, dtype, m, n, k):
    """Shapes whose 256 x 256 tiles fill every CU at least once take the form of the GEMM with 256-row tiles on
    the left columns and the 128-row form on the columns left over (one column tile of 33024 = 129 * 256, 22
    of 22016 = 86 * 256 at three row tiles); K of one, two and three 128-column steps.  Oracle on sampled rows
    of W and x."""
    w = weights(5600 + qtype + m, (n, k), outliers=False)
    x = acts(5601 + m, m, k, dtype)
    blob = dev_quantize(w, qtype, TILED)
    y = dev_matmul(x, blob, qtype, TILED, n, fn="gemm")
    assert np.isfinite(y).all()
    rows = np.unique(np.concatenate([np.arange(0, n, 61), np.arange(n - 300, n)]))      # incl. the last column tiles
    ms = np.unique(np.concatenate([np.arange(0, m, 37), [255, 256, m - 1]]))
    y_exact = orc.mul_mat_exact(orc.quantize(w[rows], qtype), x.float().numpy()[ms], (len(rows), k), qtype)
    tol = 2e-3 if dtype == torch.float16 else 8e-3
    assert np.abs(y[np.ix_(ms, rows)] - y_exact).max() <= tol * np.abs(y_exact).max()


def test_gemm_tile_line_covers_every_tile_for_any_tile_counts():
    """The GEMM deals its output tiles to the XCDs in equal shares of one line of tiles; every (row tile, column
    tile) must be computed exactly once whatever the counts.  Random M / N / K (1 to 13 row tiles, 1 to 12 column
    tiles, with and without tails; both forms of the kernel, with and without K splits) against the product with
    the weights the library's own dequantizer returns (the dequantizer is bit-exact against the oracle), on a y
    that starts as NaN."""
    rng = np.random.default_rng(77)
    for case in range(24):
        qtype = [Q4_0, FP8, Q8_0, NF4][case % 4]
        dtype = torch.float16 if case % 2 == 0 else torch.bfloat16
        m = int(rng.integers(17, 1700))
        n = 16 * int(rng.integers(1, 190))
        k = 128 * int(rng.integers(1, 7))
        if case % 5 == 0:
            m = 128 * int(rng.integers(1, 14))             # whole row tiles
        w = weights(6000 + case, (n, k))
        x = acts(6100 + case, m, k, dtype).cuda()
        blob = dev_quantize(w, qtype, TILED)
        wd = dev_dequantize(blob, qtype, n, k, TILED, torch.float32)
        want = x.float() @ wd.t()
        splits = int(rng.integers(1, 4)) if k >= 512 else 1
        ws_bytes = max(16, splits * ((m + 127) // 128) * ((n + 255) // 256) * 128 * 1024)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")
        y = torch.full((m, n), float("nan"), dtype=dtype, device="cuda")
        ggml.lowbit_gemm_ws(x.data_ptr(), blob.data_ptr(), y.data_ptr(), qtype, TILED, DT[dtype], m, n, k, ws.data_ptr(),
                            ws_bytes, splits, stream())
        torch.cuda.synchronize()
        assert not torch.isnan(y).any(), (case, qtype, m, n, k, splits)
        tol = 2e-3 if dtype == torch.float16 else 8e-3
        assert (y.float() - want).abs().max() <= tol * want.abs().max(), (case, qtype, m, n, k, splits)


@pytest.mark.gpu
@pytest.mark.parametrize("qtype,dtype", [(Q4_0, torch.float16), (Q4_1, torch.bfloat16), (Q8_0, torch.float16),
                                         (FP8, torch.bfloat16)])
def test_gemm_half_tiles_cover_every_row(qtype, dtype):
    """A launch without a workspace whose tiles leave most compute units idle (at most 96 tiles of 128 x 256) goes
    out in half tiles of 64 rows.  Row counts on both sides of a half (a last row tile of 1, 64, 65 rows), tile counts
    on both sides of the limit (96 and 98 tiles), on a y that starts as NaN, against the product with the weights the
    library's own dequantizer returns (bit-exact against the oracle)."""
    k = 256
    for case, (m, n) in enumerate([(65, 512), (128, 2048), (129, 784), (192, 12288), (193, 6144), (320, 8192),
                                   (200, 12544), (1000, 3072)]):
        w = weights(6300 + case, (n, k))
        x = acts(6350 + case, m, k, dtype).cuda()
        blob = dev_quantize(w, qtype, TILED)
        want = x.float() @ dev_dequantize(blob, qtype, n, k, TILED, torch.float32).t()
        y = torch.full((m, n), float("nan"), dtype=dtype, device="cuda")
        ggml.lowbit_gemm(x.data_ptr(), blob.data_ptr(), y.data_ptr(), qtype, TILED, DT[dtype], m, n, k, stream())
        torch.cuda.synchronize()
        assert not torch.isnan(y).any(), (m, n)
        tol = 2e-3 if dtype == torch.float16 else 8e-3
        assert (y.float() - want).abs().max() <= tol * want.abs().max(), (m, n)


@pytest.mark.gpu
def test_gemm_output_off_16_byte_alignment_equals_aligned_output():
    """With y 16-byte aligned the GEMM lays a wave's rows out in LDS and stores whole cache lines; any other y takes
    the stores straight from the accumulator layout.  Both must give the same bits, tails in M and N included, in
    both forms of the kernel.  (A y that is not 8-byte aligned is refused.)"""
    for case, (qtype, dtype, m, n, k) in enumerate([(Q4_0, torch.float16, 200, 528, 256), (NF4, torch.bfloat16, 512, 8192 + 16, 256),
                                                    (FP8, torch.bfloat16, 2048, 8192, 128), (Q8_0, torch.float16, 77, 48, 384)]):
        w = weights(6400 + case, (n, k))
        x = acts(6500 + case, m, k, dtype).cuda()
        blob = dev_quantize(w, qtype, TILED)
        y0 = torch.full((m, n), float("nan"), dtype=dtype, device="cuda")
        ggml.lowbit_gemm(x.data_ptr(), blob.data_ptr(), y0.data_ptr(), qtype, TILED, DT[dtype], m, n, k, stream())
        for shift in (4,):                                    # 8 bytes off: the least the GEMM entry points accept
            flat = torch.full((m * n + 8,), float("nan"), dtype=dtype, device="cuda")
            y1 = flat[shift:shift + m * n].view(m, n)
            assert y1.data_ptr() % 16 == 2 * shift
            ggml.lowbit_gemm(x.data_ptr(), blob.data_ptr(), y1.data_ptr(), qtype, TILED, DT[dtype], m, n, k, stream())
            torch.cuda.synchronize()
            assert not torch.isnan(y0).any()
            assert torch.equal(y0, y1), (qtype, m, n, k, shift)
            assert torch.isnan(flat[:shift]).all() and torch.isnan(flat[shift + m * n:]).all()
        with pytest.raises(RuntimeError, match="8-byte aligned"):
            ggml.lowbit_gemm(x.data_ptr(), blob.data_ptr(), y0.data_ptr() + 2, qtype, TILED, DT[dtype], m, n, k, stream())


@pytest.mark.gpu
def test_forward_takes_any_y_alignment_through_the_gemv():
    """lowbit_forward accepts a y at any 2-byte boundary: the MFMA kernels store 8 bytes and more, so such a y goes
    through the streaming GEMV in 16-row passes, whatever M."""
    qtype, dtype, m, n, k = Q4_0, torch.float16, 40, 256, 512
    w = weights(6600, (n, k))
    x = acts(6601, m, k, dtype).cuda()
    blob = dev_quantize(w, qtype, TILED)
    want = torch.empty((m, n), dtype=dtype, device="cuda")
    ggml.lowbit_gemv(x.data_ptr(), blob.data_ptr(), want.data_ptr(), qtype, TILED, DT[dtype], m, n, k, 0, stream())
    flat = torch.full((m * n + 8,), float("nan"), dtype=dtype, device="cuda")
    y = flat[1:1 + m * n].view(m, n)
    assert y.data_ptr() % 8 == 2
    ggml.lowbit_forward(x.data_ptr(), blob.data_ptr(), y.data_ptr(), qtype, TILED, DT[dtype], m, n, k, stream())
    torch.cuda.synchronize()
    assert torch.equal(y, want)
    assert torch.isnan(flat[:1]).all() and torch.isnan(flat[1 + m * n:]).all()
