"""Grouped expert GEMM (BASELINE configs[4], scaled down) against the per-expert LowBitLinear
loop that is the reference's behaviour, and against the CPU oracle."""
import numpy as np
import pytest
import torch

import lowbit_oracle as orc
from ipex_llm.ggml.quantize import ggml_tensor_qtype as Q
from ipex_llm.transformers.low_bit_linear import FP4Params, LowBitLinear
from ipex_llm.transformers.moe import (ExpertWeights, grouped_forward, grouped_mlp_forward, moe_ffn_grouped,
                                       moe_ffn_reference, route_top_k)
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


# Row counts that put the launch on the 256-row form (more than 96 rows per group on average): a tile for
# every count of 32-row blocks from 1 to 8, whole tiles, a whole tile plus a short one, an empty group.
TALL_COUNTS = [257, 0, 1, 33, 65, 97, 129, 161, 193, 225, 256, 300]


def _offsets(counts):
    return torch.tensor(np.concatenate([[0], np.cumsum(counts)]), dtype=torch.int32, device="cuda")


@pytest.mark.parametrize("qname,dtype", [("fp8_e4m3", torch.bfloat16), ("sym_int4", torch.float16),
                                         ("asym_int4", torch.bfloat16), ("nf4", torch.bfloat16),
                                         ("sym_int8", torch.float16)])
@pytest.mark.parametrize("k", [384, 2048])
def test_grouped_forward_tall_form_matches_oracle_per_group(qname, dtype, k):
    """K = 2048 with 272 columns splits K over the workspace (2 splits of 8 steps), K = 384 does not; both also
    through the entry point without a workspace."""
    import ipex_llm.ggml.model.llama.llama_cpp as ggml
    from gpu_util import DT, stream
    qtype = Q[qname]
    n = 272
    counts = TALL_COUNTS
    lins, raw = _experts(len(counts), n, k, qtype, 8600)
    rows = sum(counts)
    assert (ggml.lowbit_grouped_workspace_bytes(len(counts), rows, n, k) > 0) == (k == 2048)
    torch.manual_seed(3)
    x = torch.randn(rows, k).to(dtype).cuda()
    offs = _offsets(counts)
    table = ExpertWeights(lins)
    y_ws = grouped_forward(x, offs, table)
    y_plain = torch.full((rows + 3, n), float("nan"), dtype=dtype, device="cuda")      # three rows that no group owns
    ggml.lowbit_grouped_forward(x.data_ptr(), table.ptrs.data_ptr(), y_plain.data_ptr(), offs.data_ptr(), len(counts),
                                rows, qtype, DT[dtype], n, k, stream())
    torch.cuda.synchronize()
    assert torch.isnan(y_plain[rows:]).all() and not torch.isnan(y_plain[:rows]).any()
    r0 = 0
    for e, c in enumerate(counts):
        if c:
            blob = orc.quantize(raw[e], qtype)
            want = orc.mul_mat_exact(blob, x[r0:r0 + c].float().cpu().numpy(), (n, k), qtype)
            tol = 2e-3 if dtype == torch.float16 else 8e-3
            for got in (y_ws, y_plain):
                err = np.abs(got[r0:r0 + c].float().cpu().numpy() - want).max()
                assert err <= tol * np.abs(want).max(), (e, c)
        r0 += c


@pytest.mark.parametrize("qname,dtype,act", [("fp8_e4m3", torch.bfloat16, 0), ("sym_int4", torch.float16, 0),
                                             ("nf4", torch.bfloat16, 1), ("sym_int8", torch.float16, 1),
                                             ("asym_int4", torch.float16, 0)])
@pytest.mark.parametrize("counts", [TALL_COUNTS, [130, 0, 1, 17, 129, 40, 64, 97]])
def test_grouped_mlp_forward_matches_oracle_per_group(qname, dtype, act, counts):
    """act(x Wg^T) * (x Wu^T) of every group in one launch; 272 columns = two workgroup tiles and 16 columns."""
    qtype = Q[qname]
    n, k = 272, 384
    gate, raw_g = _experts(len(counts), n, k, qtype, 8700)
    up, raw_u = _experts(len(counts), n, k, qtype, 8800)
    rows = sum(counts)
    torch.manual_seed(4)
    x = torch.randn(rows, k).to(dtype).cuda()
    h = grouped_mlp_forward(x, _offsets(counts), ExpertWeights(gate), ExpertWeights(up), act).float().cpu().numpy()
    r0 = 0
    for e, c in enumerate(counts):
        if c:
            xe = x[r0:r0 + c].float().cpu().numpy()
            g = orc.mul_mat_exact(orc.quantize(raw_g[e], qtype), xe, (n, k), qtype)
            u = orc.mul_mat_exact(orc.quantize(raw_u[e], qtype), xe, (n, k), qtype)
            if act == 0:
                want = g / (1.0 + np.exp(-g)) * u
            else:
                want = 0.5 * g * (1.0 + np.tanh(0.7978845608028654 * (g + 0.044715 * g ** 3))) * u
            tol = 2e-3 if dtype == torch.float16 else 8e-3
            assert np.abs(h[r0:r0 + c] - want).max() <= tol * np.abs(want).max(), (e, c)
        r0 += c


def _many_counts(n_groups, mean_rows, seed):
    """Row counts for many groups: a quarter empty, single rows, counts either side of a whole tile, a long tail."""
    rng = np.random.default_rng(seed)
    counts = rng.poisson(mean_rows, n_groups)
    counts[rng.random(n_groups) < 0.25] = 0
    counts[0], counts[-1] = 1, 2 * mean_rows + 1           # first and last group take part
    counts[n_groups // 2] = 257
    return [int(c) for c in counts]


@pytest.mark.parametrize("n_groups", [64, 65, 100])
@pytest.mark.parametrize("mean_rows", [24, 140])
def test_grouped_launches_find_their_tiles_among_many_groups(n_groups, mean_rows):
    """Up to 64 groups a workgroup finds its row tile with one lane per group, beyond that by walking the offsets;
    both forms of tile (up to 96 rows per group on average: 128-row tiles, above: 256-row tiles), plain and fused."""
    qtype, dtype = Q["sym_int4"], torch.float16
    n, k = 272, 256
    counts = _many_counts(n_groups, mean_rows, 100 * n_groups + mean_rows)
    gate, raw_g = _experts(n_groups, n, k, qtype, 9100)
    up, raw_u = _experts(n_groups, n, k, qtype, 9300)
    rows = sum(counts)
    torch.manual_seed(6)
    x = torch.randn(rows, k).to(dtype).cuda()
    offs = _offsets(counts)
    y = grouped_forward(x, offs, ExpertWeights(gate)).float().cpu().numpy()
    h = grouped_mlp_forward(x, offs, ExpertWeights(gate), ExpertWeights(up), 0).float().cpu().numpy()
    r0 = 0
    for e, c in enumerate(counts):
        if c:
            xe = x[r0:r0 + c].float().cpu().numpy()
            g = orc.mul_mat_exact(orc.quantize(raw_g[e], qtype), xe, (n, k), qtype)
            u = orc.mul_mat_exact(orc.quantize(raw_u[e], qtype), xe, (n, k), qtype)
            assert np.abs(y[r0:r0 + c] - g).max() <= 2e-3 * np.abs(g).max(), (e, c)
            want = g / (1.0 + np.exp(-g)) * u
            assert np.abs(h[r0:r0 + c] - want).max() <= 2e-3 * np.abs(want).max(), (e, c)
        r0 += c


def test_grouped_ffn_replays_correctly_from_a_hip_graph():
    """The fused gate/up launch and the down projection with its K-split workspace, captured once and replayed
    with new activations and a new routing (static buffers), with eager work and synchronizations between the
    replays; every replay must equal the eager result bit for bit."""
    qtype = Q["fp8_e4m3"]
    n_exp, hidden, ffn, rows = 6, 256, 2048, 6 * 150
    w1, _ = _experts(n_exp, ffn, hidden, qtype, 9000)
    w3, _ = _experts(n_exp, ffn, hidden, qtype, 9100)
    w2, _ = _experts(n_exp, hidden, ffn, qtype, 9200)
    g1, g3, g2 = ExpertWeights(w1), ExpertWeights(w3), ExpertWeights(w2)
    import ipex_llm.ggml.model.llama.llama_cpp as ggml
    assert ggml.lowbit_grouped_workspace_bytes(n_exp, rows, hidden, ffn) > 0        # the down projection splits K
    static_x = torch.zeros(rows, hidden, dtype=torch.bfloat16, device="cuda")
    static_offs = _offsets([150] * n_exp)

    def ffn_of(x, offs):
        return grouped_forward(grouped_mlp_forward(x, offs, g1, g3), offs, g2)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        ffn_of(static_x, static_offs)                      # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_y = ffn_of(static_x, static_offs)
    torch.manual_seed(5)
    for step, counts in enumerate([[150] * 6, [300, 0, 1, 299, 170, 130], [33, 257, 160, 129, 200, 121], [150] * 6]):
        x = torch.randn(rows, hidden, device="cuda").bfloat16()
        offs = _offsets(counts)
        want = ffn_of(x, offs)                             # eager work between the replays
        torch.cuda.synchronize()
        static_x.copy_(x)
        static_offs.copy_(offs)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(static_y, want), step


def test_grouped_entry_points_refuse_bad_arguments():
    import ipex_llm.ggml.model.llama.llama_cpp as ggml
    from gpu_util import stream
    lins, _ = _experts(2, 32, 128, Q["sym_int4"], 8900)
    table = ExpertWeights(lins)
    x = torch.zeros(4, 128, dtype=torch.float16, device="cuda")
    y = torch.zeros(4, 32, dtype=torch.float16, device="cuda")
    offs = _offsets([2, 2])
    args = (x.data_ptr(), table.ptrs.data_ptr(), table.ptrs.data_ptr(), y.data_ptr(), offs.data_ptr(), 2, 4,
            Q["sym_int4"], 0, 32, 128)
    with pytest.raises(RuntimeError, match="activation"):
        ggml.lowbit_grouped_mlp_forward(*args, 7, stream())
    with pytest.raises(RuntimeError, match="null"):
        ggml.lowbit_grouped_mlp_forward(x.data_ptr(), table.ptrs.data_ptr(), None, y.data_ptr(), offs.data_ptr(), 2, 4,
                                        Q["sym_int4"], 0, 32, 128, 0, stream())
    with pytest.raises(RuntimeError, match="f16 or bf16"):
        ggml.lowbit_grouped_forward_ws(x.data_ptr(), table.ptrs.data_ptr(), y.data_ptr(), offs.data_ptr(), 2, 4,
                                       Q["sym_int4"], 2, 32, 128, None, 0, stream())
    assert ggml.lowbit_grouped_workspace_bytes(0, 4, 32, 128) == 0


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


def _mixtral_block(n_exp, hidden, inter, top_k, qtype, seed):
    """A Hugging Face MixtralSparseMoeBlock whose expert weights already are what the oracle dequantizes them to,
    so that the dense block and its low-bit conversion compute with the same numbers."""
    transformers = pytest.importorskip("transformers")
    from transformers.models.mixtral.modeling_mixtral import MixtralSparseMoeBlock
    cfg = transformers.MixtralConfig(hidden_size=hidden, intermediate_size=inter, num_local_experts=n_exp,
                                     num_experts_per_tok=top_k, num_hidden_layers=1, num_attention_heads=4,
                                     num_key_value_heads=4, vocab_size=64)
    torch.manual_seed(seed)
    block = MixtralSparseMoeBlock(cfg).eval()
    with torch.no_grad():
        for p, shape in ((block.experts.gate_up_proj, (2 * inter, hidden)), (block.experts.down_proj, (hidden, inter))):
            for e in range(n_exp):
                w = weights(seed + 10 * e + shape[0], shape)
                p[e] = torch.from_numpy(orc.dequantize(orc.quantize(w, qtype), qtype, shape))
        for p in block.gate.parameters():
            p.copy_(torch.randn_like(p))
    return block


@pytest.mark.parametrize("qname,dtype", [("fp8_e4m3", torch.bfloat16), ("sym_int4", torch.float16)])
def test_low_bit_experts_take_the_place_of_the_fused_experts_module(qname, dtype):
    import copy
    from ipex_llm.transformers.convert import _replace_with_low_bit_linear
    from ipex_llm.transformers.moe import LowBitExperts
    qtype = Q[qname]
    block = _mixtral_block(8, 256, 512, 2, qtype, 9300)
    dense = copy.deepcopy(block).to(dtype).cuda()
    low, replaced = _replace_with_low_bit_linear(block, qtype, modules_to_not_convert=["gate"])
    assert replaced and isinstance(low.experts, LowBitExperts) and isinstance(low.gate, type(dense.gate))
    low = low.to(dtype).to("cuda")
    torch.manual_seed(6)
    for tokens in (300, 1):                                 # grouped launches / the two launches of one decode token
        x = torch.randn(1, tokens, 256, device="cuda").to(dtype)
        with torch.no_grad():
            want = dense(x.clone()).float()
            got = low(x.clone()).float()
        assert got.shape == want.shape
        assert (got - want).abs().max() <= 1e-2 * want.abs().max(), tokens


def test_from_pretrained_tiny_mixtral_and_low_bit_round_trip(tmp_path):
    transformers = pytest.importorskip("transformers")
    from ipex_llm.transformers import AutoModelForCausalLM
    from ipex_llm.transformers.moe import LowBitExperts
    cfg = transformers.MixtralConfig(hidden_size=128, intermediate_size=256, num_hidden_layers=2, num_attention_heads=4,
                                     num_key_value_heads=4, vocab_size=320, max_position_embeddings=64,
                                     num_local_experts=4, num_experts_per_tok=2)
    torch.manual_seed(5)
    hf = transformers.MixtralForCausalLM(cfg).eval()
    src = tmp_path / "fp"
    hf.save_pretrained(str(src))
    model = AutoModelForCausalLM.from_pretrained(str(src), load_in_low_bit="sym_int4", modules_to_not_convert=["lm_head"])
    experts = [m for m in model.modules() if isinstance(m, LowBitExperts)]
    assert len(experts) == 2 and experts[0].gate[0].weight.quantized
    ids = torch.randint(0, 320, (1, 9))
    with torch.no_grad():
        want = hf(ids).logits
        got = model.to("cuda")(ids.cuda()).logits.float().cpu()
    assert (got - want).abs().mean() / want.abs().mean() < 0.25
    out = tmp_path / "lowbit"
    model.save_low_bit(str(out))
    again = AutoModelForCausalLM.load_low_bit(str(out))
    with torch.no_grad():
        got2 = again.to("cuda")(ids.cuda()).logits.float().cpu()
    assert torch.equal(got, got2)
