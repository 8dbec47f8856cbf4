"""Fused gate/up projection (xe_linear.mlp_forward_xpu) and row-gather dequantization
(xe_linear.dequantize_rows / LowBitEmbedding) against the CPU oracle, through the C ABI."""
import numpy as np
import pytest
import torch
from torch import nn

import lowbit_oracle as orc
import ipex_llm.ggml.model.llama.llama_cpp as ggml
from ipex_llm.ggml.quantize import ggml_tensor_qtype as Q
from ipex_llm.transformers.embedding import LowBitEmbedding
from ipex_llm.transformers.low_bit_linear import (FP4Params, LowBitLinear, dequantize_rows, mlp_forward_xpu)
from ipex_llm.transformers.models.common import fuse_mlp_base, mlp_gelu_forward, mlp_silu_forward
from ipex_llm.transformers.models.utils import GELU, SILU, mlp_fusion_check
from gpu_util import ALL, NAMES, acts, dev_quantize, dev_relayout, weights

pytestmark = pytest.mark.gpu


def _silu(g):
    return g / (1.0 + np.exp(-g))


def _gelu_tanh(g):
    return 0.5 * g * (1.0 + np.tanh(0.7978845608028654 * (g + 0.044715 * g ** 3)))


@pytest.mark.parametrize("qtype", ALL)
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("m,act", [(1, SILU), (3, GELU), (4, SILU), (5, GELU), (8, SILU), (13, GELU), (16, SILU),
                                   (17, GELU), (31, SILU), (32, GELU), (40, SILU), (130, SILU), (300, GELU)])
def test_mlp_forward_matches_the_exact_gated_product(qtype, dtype, m, act):
    n, k = 304, 640                      # 19 tile rows, K not a multiple of a full round of waves
    wg, wu = weights(9000 + qtype, (n, k)), weights(9100 + qtype, (n, k))
    x = acts(9200 + m, m, k, dtype)
    bg, bu = dev_quantize(wg, qtype, ggml.LAYOUT_TILED), dev_quantize(wu, qtype, ggml.LAYOUT_TILED)
    y = mlp_forward_xpu(x.cuda(), bg, bu, m, k, n, act, qtype).float().cpu().numpy()
    xf = x.float().numpy()
    g = orc.mul_mat_exact(orc.quantize(wg, qtype), xf, (n, k), qtype)
    u = orc.mul_mat_exact(orc.quantize(wu, qtype), xf, (n, k), qtype)
    want = (_silu(g) if act == SILU else _gelu_tanh(g)) * u
    tol = 2e-3 if dtype == torch.float16 else 8e-3       # one rounding of the result to fp16 / bf16
    assert np.abs(y - want).max() <= tol * np.abs(want).max()


def test_mlp_forward_whose_row_tiles_are_a_single_round():
    # nine row tiles of 256 rows by three column tiles: few enough for one round of workgroups, where a row tile's
    # column tiles stay on one XCD (the other tile order of the fused launch); the last row tile holds 37 rows
    m, n, k = 2048 + 37, 272, 256
    wg, wu = weights(9300, (n, k)), weights(9301, (n, k))
    x = acts(9302, m, k, torch.float16)
    bg, bu = dev_quantize(wg, 2, ggml.LAYOUT_TILED), dev_quantize(wu, 2, ggml.LAYOUT_TILED)
    y = mlp_forward_xpu(x.cuda(), bg, bu, m, k, n, SILU, 2).float().cpu().numpy()
    xf = x.float().numpy()
    g = orc.mul_mat_exact(orc.quantize(wg, 2), xf, (n, k), 2)
    u = orc.mul_mat_exact(orc.quantize(wu, 2), xf, (n, k), 2)
    want = _silu(g) * u
    assert np.isfinite(y).all()
    assert np.abs(y - want).max() <= 2e-3 * np.abs(want).max()


def test_mlp_forward_rejects_what_it_cannot_fuse():
    n, k = 32, 128
    b = dev_quantize(weights(1, (n, k)), 2, ggml.LAYOUT_TILED)
    x = acts(2, 5, k, torch.float16).cuda()
    with pytest.raises(RuntimeError, match="activation"):
        mlp_forward_xpu(x[:1], b, b, 1, k, n, 7, 2)
    with pytest.raises(RuntimeError, match="activation"):
        mlp_forward_xpu(x, b, b, 5, k, n, 7, 2)
    with pytest.raises(RuntimeError, match="shape"):
        mlp_forward_xpu(x, b, b, 4, k, n, SILU, 2)


class _GatedMlp(nn.Module):
    def __init__(self, hidden, ffn, act):
        super().__init__()
        self.gate_proj = nn.Linear(hidden, ffn, bias=False)
        self.up_proj = nn.Linear(hidden, ffn, bias=False)
        self.down_proj = nn.Linear(ffn, hidden, bias=False)
        self.act_fn = act

    def forward(self, x):
        return self.down_proj(self.act_fn(self.gate_proj(x)) * self.up_proj(x))


@pytest.mark.parametrize("low_bit,act,fwd", [("sym_int4", nn.SiLU(), mlp_silu_forward),
                                             ("fp8_e4m3", nn.GELU(approximate="tanh"), mlp_gelu_forward)])
def test_optimize_model_patches_gated_mlps_and_the_fused_path_agrees(low_bit, act, fwd):
    from ipex_llm import optimize_model
    torch.manual_seed(11)
    ref = _GatedMlp(256, 512, act).eval()

    class _Wrap(nn.Module):                      # the patch looks for classes named *MLP
        def __init__(self, mlp):
            super().__init__()
            self.mlp = mlp

        def forward(self, x):
            return self.mlp(x)
    _GatedMlp.__name__ = "ToyMLP"
    try:
        model = optimize_model(_Wrap(ref), low_bit=low_bit).to("cuda")
        assert model.mlp.forward.__func__ is fwd
        x1 = torch.randn(1, 1, 256).half().cuda()
        assert mlp_fusion_check(x1, Q[low_bit], False)
        with torch.no_grad():
            fused = model(x1).float()
            m = model.mlp
            plain = m.down_proj(m.act_fn(m.gate_proj(x1)) * m.up_proj(x1)).float()
            assert fused.shape == plain.shape == (1, 1, 256)
            assert (fused - plain).abs().max() <= 1e-2 * plain.abs().max()
            x8 = torch.randn(3, 8, 256).cuda()                   # float32 above 4 rows: the unfused branch
            assert not mlp_fusion_check(x8, Q[low_bit], False)
            y8 = model(x8)
            assert y8.shape == (3, 8, 256) and y8.dtype == torch.float32
            assert torch.equal(y8, m.down_proj(m.act_fn(m.gate_proj(x8)) * m.up_proj(x8)))
            for rows in (16, 24):                                # the streaming kernel's fused launch, one and two passes
                xr = torch.randn(rows // 8, 8, 256).half().cuda()
                assert mlp_fusion_check(xr, Q[low_bit], False)
                yr = model(xr).float()
                plain = m.down_proj(m.act_fn(m.gate_proj(xr)) * m.up_proj(xr)).float()
                assert (yr - plain).abs().max() <= 1e-2 * plain.abs().max()
            x80 = torch.randn(2, 40, 256).half().cuda()          # a prefill batch: the fused GEMM
            assert mlp_fusion_check(x80, Q[low_bit], False) and not mlp_fusion_check(x80.float(), Q[low_bit], False)
            y80 = model(x80).float()
            plain = m.down_proj(m.act_fn(m.gate_proj(x80)) * m.up_proj(x80)).float()
            assert y80.shape == plain.shape == (2, 40, 256)
            assert (y80 - plain).abs().max() <= 1e-2 * plain.abs().max()
    finally:
        _GatedMlp.__name__ = "_GatedMlp"


@pytest.mark.parametrize("qtype", ALL)
@pytest.mark.parametrize("layout", [ggml.LAYOUT_GGML, ggml.LAYOUT_TILED])
def test_dequantize_rows_is_bit_exact_and_zero_fills_bad_indices(qtype, layout):
    n, k = 48, 256
    w = weights(9300 + qtype, (n, k))
    blob = dev_quantize(w, qtype, layout)
    table = orc.dequantize(orc.quantize(w, qtype), qtype, (n, k))
    idx = torch.tensor([[0, 47, 5], [5, 17, 31]], dtype=torch.int64)
    got = dequantize_rows(idx.cuda(), blob, qtype, k, n, layout=layout)
    assert got.dtype == torch.float32 and got.shape == (2, 3, k)
    assert np.array_equal(got.cpu().numpy(), table[idx.numpy()])
    bad = torch.tensor([3, -1, n, 7], dtype=torch.int32).cuda()
    got = dequantize_rows(bad, blob, qtype, k, n, layout=layout).cpu().numpy()
    assert np.array_equal(got[[0, 3]], table[[3, 7]]) and not got[[1, 2]].any()
    assert dequantize_rows(torch.empty(0, dtype=torch.int64).cuda(), blob, qtype, k, n, layout=layout).shape == (0, k)


@pytest.mark.parametrize("qname", ["sym_int4", "nf4", "fp8_e4m3"])
def test_lowbit_embedding_looks_up_dequantized_rows(qname):
    qtype = Q[qname]
    torch.manual_seed(3)
    emb = nn.Embedding(320, 128).half()
    low = LowBitEmbedding.from_embedding(emb, False, qtype)
    assert low.weight.numel() == 0 and not low.qweight.quantized
    with pytest.raises(RuntimeError, match="only supports GPU"):
        low(torch.tensor([1]))
    low = low.to("cuda")
    assert isinstance(low.qweight, FP4Params) and low.qweight.quantized and low.qweight.device.type == "cuda"
    ids = torch.randint(0, 320, (2, 7))
    out = low(ids.cuda())
    assert out.dtype == torch.float16 and out.shape == (2, 7, 128)
    w = emb.weight.detach().float().numpy()
    table = orc.dequantize(orc.quantize(w, qtype), qtype, w.shape)
    assert np.array_equal(out.float().cpu().numpy(), table[ids.numpy()].astype(np.float16).astype(np.float32))
    # back on the CPU the blob is the ggml blob of the table
    assert np.array_equal(low.to("cpu").qweight.data.view(torch.uint8).numpy(), orc.quantize(w, qtype))


def test_from_pretrained_with_embedding_qtype_and_fused_mlp(tmp_path):
    transformers = pytest.importorskip("transformers")
    from ipex_llm.transformers import AutoModelForCausalLM
    cfg = transformers.LlamaConfig(hidden_size=128, intermediate_size=256, num_hidden_layers=2,
                                   num_attention_heads=4, num_key_value_heads=4, vocab_size=320,
                                   max_position_embeddings=64)
    torch.manual_seed(5)
    hf = transformers.LlamaForCausalLM(cfg).eval()
    src = tmp_path / "fp"
    hf.save_pretrained(str(src))
    model = AutoModelForCausalLM.from_pretrained(str(src), load_in_low_bit="sym_int4", embedding_qtype="sym_int8",
                                                 modules_to_not_convert=["lm_head"])
    assert isinstance(model.model.embed_tokens, LowBitEmbedding)
    assert model.model.layers[0].mlp.forward.__func__ is mlp_silu_forward
    ids = torch.randint(0, 320, (1, 1))                       # one token: the fused MLP launch
    with torch.no_grad():
        want = hf(ids).logits
        got = model.to("cuda")(ids.cuda()).logits.float().cpu()
    assert (got - want).abs().mean() / want.abs().mean() < 0.2
    out = tmp_path / "lowbit"
    model.save_low_bit(str(out))
    again = AutoModelForCausalLM.load_low_bit(str(out), embedding_qtype="sym_int8")
    assert isinstance(again.model.embed_tokens, LowBitEmbedding)
    with torch.no_grad():
        got2 = again.to("cuda")(ids.cuda()).logits.float().cpu()
    assert torch.equal(got, got2)


# ------------------------------------------------------------------ merged q/k/v projection

@pytest.mark.parametrize("qname,dtype", [("sym_int4", torch.float16), ("nf4", torch.bfloat16), ("sym_int8", torch.bfloat16)])
@pytest.mark.parametrize("m", [1, 4, 40])
def test_merged_qkv_projection_equals_the_three_separate_ones(qname, dtype, m):
    """The merge of q_proj / k_proj / v_proj (convert.py:996-999 of the reference) is a row concatenation
    before quantization; blocks never straddle rows, so the merged blob is the concatenation of the three
    blobs and every output column must come out as from the separate layers: against the oracle on the
    separate weights, and bit for bit where both calls run the same kernel variant."""
    from ipex_llm.transformers.models.common import merge_qkv_base
    qtype = Q[qname]
    hidden, nq, nkv = 1024, 1024, 256

    class Attention(nn.Module):                      # q/k/v as in a grouped-query attention block
        def __init__(self):
            super().__init__()
            self.q_proj = nn.Linear(hidden, nq, bias=False)
            self.k_proj = nn.Linear(hidden, nkv, bias=False)
            self.v_proj = nn.Linear(hidden, nkv, bias=False)

    torch.manual_seed(17)
    attn = Attention().eval()
    ws = [getattr(attn, n).weight.detach().clone() for n in ("q_proj", "k_proj", "v_proj")]
    separate = []
    for w in ws:
        lin = LowBitLinear(hidden, w.shape[0], qtype, bias=False).eval()
        lin.weight = FP4Params(w.clone(), qtype=qtype).to("cuda")
        separate.append(lin)
    merge_qkv_base(attn, Attention)
    merged = LowBitLinear(hidden, nq + 2 * nkv, qtype, bias=False).eval()
    merged.weight = FP4Params(attn.qkv_proj.weight.detach().clone(), qtype=qtype).to("cuda")
    attn.qkv_proj = merged
    # bytes: merged blob == concatenated blobs (ggml layout, as saved)
    cat = np.concatenate([orc.quantize(w.numpy(), qtype) for w in ws])
    assert np.array_equal(merged.weight.to("cpu").data.view(torch.uint8).numpy(), cat)
    x = acts(9900 + m, m, hidden, dtype).cuda()
    with torch.no_grad():
        q, k, v = attn.q_proj(x), attn.k_proj(x), attn.v_proj(x)          # one launch, two cache reads
        sep = [lin(x) for lin in separate]
        own_rows = attn.v_proj(x.clone())                                  # not the cached tensor: own rows only
    tol = 2e-3 if dtype == torch.float16 else 8e-3
    for got, lin_out, w in zip((q, k, v), sep, ws):
        want = orc.mul_mat_exact(orc.quantize(w.numpy(), qtype), x.float().cpu().numpy(), w.shape, qtype)
        assert np.abs(got.float().cpu().numpy() - want).max() <= tol * np.abs(want).max()
        # same rows through a differently shaped launch: fp32 sums may be associated differently, the rounded
        # results agree to the last place or two
        diff = (got.float() - lin_out.float()).abs().max().item()
        assert diff <= 2.0 ** (-9 if dtype == torch.float16 else -6) * lin_out.float().abs().max().item()
    assert torch.equal(own_rows, sep[2])                                   # same shape, same kernel: bit for bit
