"""The drop-in Python layer on a real MI355X: LowBitLinear / FP4Params / optimize_model /
from_pretrained, compared with the CPU oracle and with dense layers holding the dequantized
weights (the A/B style of the reference's own GPU tests, test/inference_gpu/*)."""
import ctypes

import numpy as np
import pytest
import torch
from torch import nn

import lowbit_oracle as orc
import ipex_llm.ggml.model.llama.llama_cpp as ggml
from ipex_llm.ggml.quantize import ggml_tensor_qtype as Q
from ipex_llm.transformers.low_bit_linear import (FP4Params, LowBitLinear, dequant, ggml_convert_fp32,
                                                  ggml_convert_qtype, ggml_matmul_src1_x_src0_t)
from gpu_util import ALL, NAMES, weights

pytestmark = pytest.mark.gpu


def _layer(w, qtype, bias=None, **kw):
    n, k = w.shape
    layer = LowBitLinear(k, n, qtype, bias=bias is not None, **kw)
    layer.weight = FP4Params(torch.from_numpy(w), qtype=qtype)
    if bias is not None:
        layer.bias.data = torch.from_numpy(bias)
    return layer.eval()


@pytest.mark.parametrize("qtype", ALL)
def test_fp4params_device_round_trip_keeps_the_ggml_bytes(qtype):
    w = weights(7000 + qtype, (64, 256))
    p = FP4Params(torch.from_numpy(w), qtype=qtype)
    g = p.to("cuda")
    assert g.quantized and g.device.type == "cuda" and tuple(g._shape) == (64, 256)
    c = g.to("cpu")
    blob = c.data.view(torch.uint8).numpy()
    assert np.array_equal(blob, orc.quantize(w, qtype))
    # quantizing on the host path (staged through the GPU) gives the same blob
    h = FP4Params(torch.from_numpy(w), qtype=qtype).to("cpu")
    assert h.quantized and np.array_equal(h.data.view(torch.uint8).numpy(), blob)
    # and a quantized CPU blob moved to the GPU equals the directly quantized one
    assert torch.equal(h.to("cuda").data.view(torch.uint8), g.data.view(torch.uint8))


def test_convert_qtype_blob_dtypes_and_dequant_entry_points():
    w = weights(7100, (32, 256))
    for qtype in ALL:
        blob = ggml_convert_qtype(torch.from_numpy(w), qtype, device="cpu")
        assert blob.dtype == (torch.bfloat16 if qtype == Q["nf4"] else torch.uint8)
        want = orc.dequantize(orc.quantize(w, qtype), qtype, w.shape)
        got = ggml_convert_fp32(blob.view(torch.uint8), w.shape, w.size, qtype)
        assert np.array_equal(got.numpy(), want)
        dev = FP4Params(torch.from_numpy(w), qtype=qtype).to("cuda")
        flat = dequant(torch.empty(0, dtype=torch.float32, device="cuda"), dev.data, qtype, shape=w.shape)
        assert np.array_equal(flat.reshape(w.shape).cpu().numpy(), want)


@pytest.mark.parametrize("qtype", ALL)
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_lowbitlinear_forward_matches_dense_layer_of_dequantized_weights(qtype, dtype):
    n, k = 96, 256
    w = weights(7200 + qtype, (n, k))
    bias = (np.random.default_rng(1).standard_normal(n) * 0.1).astype(np.float32)
    layer = _layer(w, qtype, bias).to("cuda")
    wd = torch.from_numpy(orc.dequantize(orc.quantize(w, qtype), qtype, w.shape))
    dense = nn.Linear(k, n)
    dense.weight.data, dense.bias.data = wd, torch.from_numpy(bias)
    torch.manual_seed(3)
    for shape in [(1, 1, k), (2, 5, k), (3, k), (2, 40, k)]:
        x = torch.randn(shape).to(dtype)
        y = layer(x.cuda())
        assert y.dtype == dtype and y.shape == shape[:-1] + (n,) and y.device.type == "cuda"
        ref = dense(x.float())
        tol = 3e-3 if dtype != torch.bfloat16 else 1.2e-2
        assert (y.float().cpu() - ref).abs().max() <= tol * ref.abs().max()


def test_lm_head_slice_act_order_and_no_bias():
    n, k = 64, 128
    w = weights(7300, (n, k))
    layer = _layer(w, Q["sym_int4"], optimize_lm_head=True, act_order=True).to("cuda")
    perm = torch.randperm(k)
    layer.g_idx_map = perm.cuda()
    wd = torch.from_numpy(orc.dequantize(orc.quantize(w, 2), 2, w.shape))
    x = torch.randn(2, 12, k).half()
    y = layer(x.cuda()).float().cpu()
    assert y.shape == (2, 1, n)                       # a prefill keeps its last position only
    ref = x[:, -1:, :].float()[..., perm] @ wd.T
    assert (y - ref).abs().max() <= 3e-3 * ref.abs().max()


def test_cpu_resident_weight_uses_the_host_pointer_matmul():
    n, k = 48, 256
    w = weights(7400, (n, k))
    layer = _layer(w, Q["sym_int4"])
    layer.weight = layer.weight.to("cpu")             # quantized, still on the host
    x = torch.randn(3, k)
    y = layer(x)
    assert y.device.type == "cpu" and y.dtype == torch.float32
    blob = orc.quantize(w, 2)
    ref = orc.mul_mat_q(blob, x.numpy(), (n, k), 2)    # the reference's CPU low-bit matmul
    assert np.abs(y.numpy() - ref).max() <= 1e-2 * np.abs(ref).max()
    y2 = ggml_matmul_src1_x_src0_t(layer.weight.data, x, (n, k), 2)
    assert torch.equal(y, y2)
    with pytest.raises(RuntimeError, match="not supported on CPU"):
        l2 = _layer(w, Q["nf4"])
        l2.weight = l2.weight.to("cpu")
        l2(x)


def test_host_pointer_abi_quantize_dequantize():
    w = weights(7500, (16, 384))
    for qtype in ALL:
        src = np.ascontiguousarray(w)
        dst = np.zeros(ggml.lowbit_blob_bytes(qtype, w.size), dtype=np.uint8)
        hist = (ctypes.c_int64 * 16)()
        n = ggml.ggml_quantize_tensor(src.ctypes.data_as(ctypes.POINTER(ctypes.c_float)),
                                      ctypes.c_void_p(dst.ctypes.data), qtype, w.size, w.shape[1], hist, False)
        assert n == dst.size and np.array_equal(dst, orc.quantize(w, qtype))
        out = np.zeros(w.size, dtype=np.float32)
        ggml.ggml_dequantize(ctypes.c_void_p(dst.ctypes.data), ctypes.c_void_p(out.ctypes.data), w.size, qtype)
        assert np.array_equal(out.reshape(w.shape), orc.dequantize(dst, qtype, w.shape))
    # scale_search (the closed binary's search; the reference's caller ignores the return value) does not leave
    # the blob unwritten: the symbol falls back to the plain block scale
    dst2 = np.zeros(orc.blob_bytes(2, w.size), dtype=np.uint8)
    n = ggml.ggml_quantize_tensor(src.ctypes.data_as(ctypes.POINTER(ctypes.c_float)),
                                  ctypes.c_void_p(dst2.ctypes.data), 2, w.size, w.shape[1], hist, True)
    assert n == dst2.size and np.array_equal(dst2, orc.quantize(w, 2))


class _Mlp(nn.Module):
    def __init__(self):
        super().__init__()
        self.up = nn.Linear(128, 256)
        self.down = nn.Linear(256, 128, bias=False)
        self.skip = nn.Linear(128, 128)

    def forward(self, x):
        return self.skip(self.down(torch.relu(self.up(x))))


@pytest.mark.parametrize("low_bit", ["sym_int4", "asym_int4", "sym_int8", "nf4", "fp8_e4m3"])
def test_optimize_model_save_and_load_low_bit(low_bit, tmp_path):
    from ipex_llm import optimize_model
    from ipex_llm.optimize import load_low_bit
    torch.manual_seed(11)
    ref = _Mlp().eval()
    model = _Mlp().eval()
    model.load_state_dict(ref.state_dict())
    model = optimize_model(model, low_bit=low_bit, modules_to_not_convert=["skip"])
    assert isinstance(model.up, LowBitLinear) and type(model.skip) is nn.Linear
    assert model._bigdl_config["bigdl_transformers_low_bit"] == low_bit
    x = torch.randn(4, 128)
    model = model.to("cuda")
    y = model(x.cuda()).cpu()
    want = ref(x)
    rel = (y - want).abs().max() / want.abs().max()
    assert rel < (0.15 if "4" in low_bit else 0.05)          # quantization noise, not kernel error
    model.save_low_bit(str(tmp_path))
    fresh = load_low_bit(_Mlp().eval(), str(tmp_path))
    assert isinstance(fresh.up, LowBitLinear) and fresh.up.weight.quantized
    blob_saved = fresh.up.weight.data.view(torch.uint8).numpy()
    assert np.array_equal(blob_saved, orc.quantize(ref.up.weight.detach().numpy(), Q[low_bit]))
    y2 = fresh.to("cuda")(x.cuda()).cpu()
    assert torch.equal(y, y2)


def test_from_pretrained_tiny_llama_and_low_bit_round_trip(tmp_path):
    transformers = pytest.importorskip("transformers")
    from ipex_llm.transformers import AutoModelForCausalLM
    cfg = transformers.LlamaConfig(hidden_size=128, intermediate_size=256, num_hidden_layers=2,
                                   num_attention_heads=4, num_key_value_heads=4, vocab_size=320,
                                   max_position_embeddings=64)
    torch.manual_seed(5)
    hf = transformers.LlamaForCausalLM(cfg).eval()
    src = tmp_path / "fp"
    hf.save_pretrained(str(src))
    model = AutoModelForCausalLM.from_pretrained(str(src), load_in_low_bit="sym_int4",
                                                 modules_to_not_convert=["lm_head"])
    assert model.config.bigdl_transformers_low_bit == "sym_int4"
    lin = model.model.layers[0].mlp.gate_proj
    assert isinstance(lin, LowBitLinear) and lin.weight.quantized
    assert type(model.lm_head) is nn.Linear
    # q_proj / k_proj / v_proj were merged before quantization, as the reference does for Llama
    attn = model.model.layers[0].self_attn
    assert isinstance(attn.qkv_proj, LowBitLinear) and attn.qkv_proj.out_len == 3 * 128
    ids = torch.randint(0, 320, (1, 9))
    with torch.no_grad():
        want = hf(ids).logits
        got = model.to("cuda")(ids.cuda()).logits.float().cpu()
    assert (got - want).abs().mean() / want.abs().mean() < 0.2
    out = tmp_path / "lowbit"
    model.save_low_bit(str(out))
    with pytest.raises(RuntimeError, match="load_low_bit"):
        AutoModelForCausalLM.from_pretrained(str(out), load_in_4bit=True)
    again = AutoModelForCausalLM.load_low_bit(str(out))
    with torch.no_grad():
        got2 = again.to("cuda")(ids.cuda()).logits.float().cpu()
    assert torch.equal(got, got2)


def test_host_resident_weight_takes_the_reference_cpu_routes():
    """A LowBitLinear whose blob stays on the host (reference: low_bit_linear.py:683-715): few rows go through the
    ggml-style host-pointer matmul, BIGDL_LLM_LINEAR_THRESHOLD rows and more of sym_int4 through one dequantization
    and a dense fp32 product, a training step through MatMulLowBitCPU; all three equal the dense layer of the
    oracle's dequantized weight."""
    from ipex_llm.transformers import low_bit_linear as lbl
    n, k = 96, 256
    w = weights(7300, (n, k))
    layer = _layer(w, Q["sym_int4"])
    layer.weight = layer.weight.to("cpu")                     # quantized, still on the host
    assert layer.weight.data.device.type == "cpu" and layer.weight.quantized
    wd = torch.from_numpy(orc.dequantize(orc.quantize(w, Q["sym_int4"]), Q["sym_int4"], (n, k)))
    x_small = torch.randn(5, k)
    x_large = torch.randn(lbl.TORCH_LINEAR_THRESHOLD, k)
    for x in (x_small, x_large):
        y = layer(x)
        want = x @ wd.t()
        assert y.shape == want.shape and y.dtype == x.dtype
        assert (y - want).abs().max() <= 1e-2 * want.abs().max()
    assert torch.allclose(layer(x_large), x_large @ wd.t(), atol=1e-4)          # the dense route is exact fp32
    layer.train()
    xg = torch.randn(3, k, requires_grad=True)
    y = layer(xg)
    go = torch.randn_like(y)
    y.backward(go)
    assert torch.allclose(xg.grad, go @ wd, atol=1e-4)


def test_tiny_llama_generates_under_inference_mode(tmp_path):
    """Callers of the reference run `generate` inside `torch.inference_mode()`: activations are inference
    tensors there (no version counter) and nothing of a layer's merged q/k/v product may outlive the layer."""
    transformers = pytest.importorskip("transformers")
    from ipex_llm.transformers import AutoModelForCausalLM
    cfg = transformers.LlamaConfig(hidden_size=128, intermediate_size=256, num_hidden_layers=2,
                                   num_attention_heads=4, num_key_value_heads=2, vocab_size=320,
                                   max_position_embeddings=64)
    torch.manual_seed(6)
    hf = transformers.LlamaForCausalLM(cfg).eval()
    src = tmp_path / "fp"
    hf.save_pretrained(str(src))
    model = AutoModelForCausalLM.from_pretrained(str(src), load_in_low_bit="sym_int4").to("cuda")
    ids = torch.randint(0, 320, (2, 9)).cuda()
    with torch.no_grad():
        want = model(ids).logits
        tokens_want = model.generate(ids, max_new_tokens=4, do_sample=False)
    with torch.inference_mode():
        got = model(ids).logits
        tokens = model.generate(ids, max_new_tokens=4, do_sample=False)
    assert torch.equal(got, want) and torch.equal(tokens, tokens_want) and tokens.shape == (2, 13)
    for layer in model.model.layers:
        assert layer.self_attn.__dict__.get("_qkv_cache") is None


@pytest.mark.parametrize("qname,dtype", [("nf4", torch.bfloat16), ("sym_int4", torch.float16)])
def test_training_backward_is_grad_out_times_the_dequantized_weight(qname, dtype):
    """MatMulLowBit.backward (reference: low_bit_linear.py:520-541), the QLoRA gradient path."""
    qtype = Q[qname]
    n, k = 96, 256
    w = weights(7100, (n, k))
    layer = _layer(w, qtype).to("cuda").train()
    x = torch.randn(2, 5, k).to(dtype).cuda().requires_grad_(True)
    y = layer(x)
    assert y.requires_grad and y.shape == (2, 5, n)
    go = torch.randn_like(y)
    y.backward(go)
    wd = torch.from_numpy(orc.dequantize(orc.quantize(w, qtype), qtype, (n, k))).to(dtype).cuda()
    want = (go.float().view(-1, n) @ wd.float()).view(2, 5, k)
    assert x.grad.shape == x.shape and x.grad.dtype == dtype
    assert (x.grad.float() - want).abs().max() <= 1e-2 * want.abs().max()
    assert layer.weight.grad is None


def test_lowbit_linears_replay_correctly_from_a_hip_graph():
    """Decode and small-prefill calls captured once and replayed with new inputs (static buffers), with
    eager work and synchronizations between the replays; every replay must equal the eager result."""
    torch.manual_seed(9)
    lins = [_layer(weights(7200 + i, (n, k)), Q["sym_int4"]).to("cuda") for i, (n, k) in
            enumerate([(512, 256), (256, 512)])]
    emb_like = _layer(weights(7210, (4096, 256)), Q["sym_int8"]).to("cuda")      # many tiles, short K walk
    tail = _layer(weights(7220, (1024, 4096)), Q["nf4"]).to("cuda")              # few tiles, long K walk: cut tiles

    def net(x):
        return tail(emb_like(lins[1](torch.nn.functional.silu(lins[0](x)))))
    for rows in (1, 48):                                   # GEMV path / batch-size kernel with partial tiles in a workspace
        static_x = torch.zeros(rows, 256, dtype=torch.float16, device="cuda")
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            net(static_x)                                  # warm-up outside the capture
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            static_y = net(static_x)
        for step in range(4):
            x = torch.randn(rows, 256, device="cuda").half()
            want = net(x)                                  # eager work between the replays
            torch.cuda.synchronize()
            static_x.copy_(x)
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(static_y, want), (rows, step)


@pytest.mark.parametrize("qname", ["sym_int4", "nf4"])
def test_module_cuda_and_cpu_keep_the_residency_rule(qname):
    """model.cuda() calls Tensor.cuda on every parameter, not .to(): the blob must still arrive tiled, and
    model.cpu() must bring the ggml bytes back."""
    qtype = Q[qname]
    torch.manual_seed(21)
    w = torch.randn(64, 256) * 0.02
    lin = LowBitLinear(256, 64, qtype, bias=False).eval()
    lin.weight = FP4Params(w.clone(), qtype=qtype)
    net = nn.Sequential(lin).cuda()
    p = net[0].weight
    assert p.quantized and p.data.device.type == "cuda" and p.blob_layout == ggml.LAYOUT_TILED
    blob = orc.quantize(w.numpy(), qtype)
    x = torch.randn(5, 256).half()
    y = net(x.cuda()).float().cpu().numpy()
    want = orc.mul_mat_exact(blob, x.float().numpy(), (64, 256), qtype)
    assert np.abs(y - want).max() <= 2e-3 * np.abs(want).max()
    # a quantized CPU blob through .cuda() as well (not only an unquantized weight)
    back = net.cpu()
    assert np.array_equal(back[0].weight.data.view(torch.uint8).numpy(), blob)
    again = back.cuda()
    assert np.array_equal(again(x.cuda()).float().cpu().numpy(), y)
    # FP4Params built from a ggml blob that already lives on the GPU
    born = FP4Params(torch.from_numpy(blob).cuda() if qname != "nf4" else torch.from_numpy(blob).cuda().view(torch.bfloat16),
                     quantized=True, _shape=torch.Size((64, 256)), qtype=qtype)
    assert torch.equal(born.data.view(torch.uint8), again[0].weight.data.view(torch.uint8))
    # quantize(device) lands tiled too
    direct = FP4Params(w.clone(), qtype=qtype).quantize("cuda")
    assert torch.equal(direct.data.view(torch.uint8), born.data.view(torch.uint8))


# ------------------------------------------------------------------ fp32 activations

@pytest.mark.parametrize("qname", ["sym_int4", "asym_int4", "sym_int8", "nf4", "fp8_e4m3"])
@pytest.mark.parametrize("m,n,k", [(1, 96, 1024), (3, 272, 384), (20, 64, 512), (2, 37, 256)])
def test_forward_f32_keeps_range_and_precision(qname, m, n, k):
    """lowbit_forward_f32 (fp32 in, fp32 out): activations of magnitude 1e5 must neither overflow nor lose
    more than the parity bar allows, and the result carries far more than half precision."""
    from ipex_llm.transformers.low_bit_linear import forward_new
    qtype = Q[qname]
    if k % orc.qk_size(qtype):
        pytest.skip("row length is no multiple of the block")
    rng = np.random.default_rng(300 + m)
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    x = (rng.standard_normal((m, k)) * 1e5).astype(np.float32)          # far beyond fp16's 65504
    blob = orc.quantize(w, qtype)
    p = FP4Params(torch.from_numpy(w), qtype=qtype).to("cuda")
    y = forward_new(torch.from_numpy(x).cuda(), p.data, qtype, n, layout=p.blob_layout, keep_fp32=True)
    assert y.dtype == torch.float32
    y = y.cpu().numpy()
    ref = orc.mul_mat_q(blob, x, (n, k), qtype)
    exact = orc.mul_mat_exact(blob, x, (n, k), qtype)
    assert np.isfinite(y).all()
    assert np.abs(y - ref).max() <= 1e-2 * np.abs(ref).max()
    assert np.abs(y - exact).max() <= 3e-5 * np.abs(exact).max()           # two bf16 planes: 16 mantissa bits


def test_lowbitlinear_float32_input_follows_the_reference_rules():
    """low_bit_linear.py:657-668 of the reference: float32 x goes to half precision only at inference with
    conver_to_half and more than one row outside the small-batch range."""
    torch.manual_seed(8)
    w = torch.randn(64, 256) * 0.02
    blob = orc.quantize(w.numpy(), Q["sym_int4"])

    def layer(conver_to_half):
        lin = LowBitLinear(256, 64, Q["sym_int4"], bias=False, conver_to_half=conver_to_half).eval()
        lin.weight = FP4Params(w.clone(), qtype=Q["sym_int4"])
        return lin.to("cuda")
    big = 3.0e5                                                            # overflows fp16
    # (up to 48 rows, 64 here with K % 256 == 0 and out_len % 64 == 0, are the small-batch range: :272-307)
    for rows, conv, stays_fp32 in ((1, True, True), (4, True, True), (40, True, True), (64, True, True), (65, True, False),
                                   (65, False, True)):
        x = torch.randn(rows, 256) * (big if stays_fp32 else 1.0)
        y = layer(conv)(x.cuda())
        assert y.dtype == torch.float32 and torch.isfinite(y).all()
        exact = orc.mul_mat_exact(blob, x.numpy(), (64, 256), Q["sym_int4"])
        tol = 3e-5 if stays_fp32 else 2e-3
        assert np.abs(y.cpu().numpy() - exact).max() <= tol * np.abs(exact).max(), (rows, conv)


def test_cpu_resident_matmul_is_fp32_in_and_out():
    """ggml_compute_forward_mul_mat_q_fp32 (the reference's CPU branch, low_bit_linear.py:462-497): |x| up to
    1e5 and |y| far above 65504 stay finite and within the parity bar of the reference-style CPU matmul."""
    from ipex_llm.transformers.low_bit_linear import ggml_matmul_src1_x_src0_t
    rng = np.random.default_rng(9)
    for qname in ("sym_int4", "asym_int4", "sym_int8"):
        qtype = Q[qname]
        w = (rng.standard_normal((48, 512)) * 0.5).astype(np.float32)
        x = (rng.standard_normal((5, 512)) * 1e5).astype(np.float32)
        blob = orc.quantize(w, qtype)
        y = ggml_matmul_src1_x_src0_t(torch.from_numpy(blob), torch.from_numpy(x), torch.Size((48, 512)), qtype).numpy()
        ref = orc.mul_mat_q(blob, x, (48, 512), qtype)
        assert np.isfinite(y).all() and np.abs(ref).max() > 65504
        assert np.abs(y - ref).max() <= 1e-2 * np.abs(ref).max()
