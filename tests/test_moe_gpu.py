"""Grouped expert GEMM (BASELINE configs[4], scaled down) against the per-expert LowBitLinear
loop that is the reference's behaviour, and against the CPU oracle."""
import numpy as np
import pytest
import torch

import lowbit_oracle as orc
from ipex_llm.ggml.quantize import ggml_tensor_qtype as Q
from ipex_llm.transformers.low_bit_linear import FP4Params, LowBitLinear
from ipex_llm.transformers.moe import (ExpertWeights, grouped_forward, moe_ffn_grouped, moe_ffn_reference,
                                       route_top_k)
from gpu_util import weights

pytestmark = pytest.mark.gpu


def _experts(n_exp, n, k, qtype, seed):
    out, raw = [], []
    for e in range(n_exp):
        w = weights(seed + e, (n, k))
        lin = LowBitLinear(k, n, qtype, bias=False)
        lin.weight = FP4Params(torch.from_numpy(w), qtype=qtype).to("cuda")
        out.append(lin.eval())
        raw.append(w)
    return out, raw


@pytest.mark.parametrize("qname,dtype", [("fp8_e4m3", torch.bfloat16), ("sym_int4", torch.float16),
                                         ("nf4", torch.bfloat16), ("sym_int8", torch.float16)])
def test_grouped_forward_matches_oracle_per_group(qname, dtype):
    qtype = Q[qname]
    n_exp, n, k = 8, 272, 384                          # 3 steps of 128 columns: an odd count
    lins, raw = _experts(n_exp, n, k, qtype, 8000)
    # empty group, single row, tiles of 1 / 2 / 3 / 4 row blocks, a full tile plus one row
    counts = [130, 0, 1, 17, 129, 40, 64, 97]
    rows = sum(counts)
    torch.manual_seed(1)
    x = torch.randn(rows, k).to(dtype).cuda()
    offs = torch.tensor(np.concatenate([[0], np.cumsum(counts)]), dtype=torch.int32, device="cuda")
    y = grouped_forward(x, offs, ExpertWeights(lins)).float().cpu().numpy()
    r0 = 0
    for e, c in enumerate(counts):
        if c:
            blob = orc.quantize(raw[e], qtype)
            want = orc.mul_mat_exact(blob, x[r0:r0 + c].float().cpu().numpy(), (n, k), qtype)
            tol = 2e-3 if dtype == torch.float16 else 8e-3
            assert np.abs(y[r0:r0 + c] - want).max() <= tol * np.abs(want).max(), (e, c)
        r0 += c


@pytest.mark.parametrize("qname,dtype", [("fp8_e4m3", torch.bfloat16), ("sym_int4", torch.float16)])
def test_moe_ffn_grouped_equals_per_expert_loop(qname, dtype):
    qtype = Q[qname]
    n_exp, hidden, ffn, tokens = 8, 256, 512, 77
    w1, _ = _experts(n_exp, ffn, hidden, qtype, 8100)
    w3, _ = _experts(n_exp, ffn, hidden, qtype, 8200)
    w2, _ = _experts(n_exp, hidden, ffn, qtype, 8300)
    torch.manual_seed(2)
    x = torch.randn(tokens, hidden).to(dtype).cuda()
    logits = torch.randn(tokens, n_exp).cuda()
    wts, exp = route_top_k(logits, 2)
    assert torch.allclose(wts.sum(-1), torch.ones(tokens, device="cuda"))
    ref = moe_ffn_reference(x, logits, w1, w3, w2).float()
    got = moe_ffn_grouped(x, logits, ExpertWeights(w1), ExpertWeights(w3), ExpertWeights(w2)).float()
    assert (got - ref).abs().max() <= 1e-2 * ref.abs().max()


@pytest.mark.parametrize("qname,dtype", [("sym_int4", torch.float16), ("fp8_e4m3", torch.bfloat16),
                                         ("nf4", torch.bfloat16)])
def test_moe_forward_vec_equals_the_per_expert_decode_loop(qname, dtype):
    from ipex_llm.transformers.moe import moe_forward_vec
    qtype = Q[qname]
    n_exp, hidden, ffn, top_k = 6, 256, 640, 3         # 5 tiles per expert: slots straddle a wave's tiles
    w1, r1 = _experts(n_exp, ffn, hidden, qtype, 8400)
    w3, r3 = _experts(n_exp, ffn, hidden, qtype, 8500)
    w2, r2 = _experts(n_exp, hidden, ffn, qtype, 8600)
    torch.manual_seed(4)
    x = torch.randn(1, hidden).to(dtype).cuda()
    ids = torch.tensor([[4, 0, 5]], device="cuda")
    wts = torch.tensor([[0.5, 0.3, 0.2]], device="cuda")
    got = moe_forward_vec(x, ids, wts, ExpertWeights(w1), ExpertWeights(w3), ExpertWeights(w2)).float().cpu().numpy()
    # the loop of the reference (models/deepseek.py:317-327), in exact arithmetic on the oracle's weights
    xf = x.float().cpu().numpy()
    want = np.zeros((1, hidden), dtype=np.float64)
    for e, wt in zip(ids[0].tolist(), wts[0].tolist()):
        g = orc.mul_mat_exact(orc.quantize(r1[e], qtype), xf, (ffn, hidden), qtype).astype(np.float64)
        u = orc.mul_mat_exact(orc.quantize(r3[e], qtype), xf, (ffn, hidden), qtype).astype(np.float64)
        h = (g / (1.0 + np.exp(-g)) * u).astype(np.float32)
        want += wt * orc.mul_mat_exact(orc.quantize(r2[e], qtype), h, (hidden, ffn), qtype)
    assert np.abs(got - want).max() <= 1e-2 * np.abs(want).max()
    # and against the modules themselves
    loop = sum(wt * w2[e](torch.nn.functional.silu(w1[e](x)) * w3[e](x)).float()
               for e, wt in zip(ids[0].tolist(), wts[0].tolist())).cpu().numpy()
    assert np.abs(got - loop).max() <= 1e-2 * np.abs(loop).max()
