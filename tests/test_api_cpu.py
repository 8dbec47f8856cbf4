"""Host logic of the drop-in Python layer and the C ABI surface; no GPU needed."""
import ctypes
import os
import re

import numpy as np

import pytest
import torch
from torch import nn

import ipex_llm.ggml.model.llama.llama_cpp as ggml
from ipex_llm.ggml.quantize import ggml_tensor_qtype
from ipex_llm.transformers.convert import _replace_with_low_bit_linear, ggml_convert_low_bit
from ipex_llm.transformers.low_bit_linear import (FP16Linear, FP4Params, LowBitLinear, ggml_convert_qtype,
                                                  reshape_lm_head_input, use_batch_forward)

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
Q = ggml_tensor_qtype


def test_qtype_table_matches_reference_integers():
    # python/llm/src/ipex_llm/ggml/quantize.py:28-57
    assert (Q["sym_int4"], Q["asym_int4"], Q["sym_int8"], Q["nf4"], Q["fp8_e4m3"]) == (2, 3, 8, 10, 15)
    assert (Q["fp16"], Q["bf16"], Q["fp8"], Q["fp8_e5m2"], Q["woq_int4"]) == (12, 20, 19, 19, 34)


def test_library_exports_every_declared_symbol():
    hdr = open(os.path.join(ROOT, "include", "lowbit_abi.h")).read()
    hdr = re.sub(r"/\*.*?\*/", "", hdr, flags=re.S)
    names = re.findall(r"\b((?:lowbit|ggml|llama)_\w+)\s*\(", hdr)
    assert len(set(names)) >= 18
    lib = ctypes.CDLL(os.path.join(ROOT, "ipex-llm_amd", "ipex_llm", "libs", "liblowbit_hip.so"))
    for n in set(names):
        assert hasattr(lib, n), n
    assert lib.lowbit_abi_version() == 1


def test_block_geometry_through_the_abi():
    got = [(ggml.ggml_qk_size(q), ggml.ggml_type_size(q)) for q in (2, 3, 8, 10, 15)]
    assert got == [(32, 18), (32, 20), (32, 34), (64, 34), (128, 132)]
    assert ggml.ggml_qk_size(Q["q4_k"]) == 0
    assert ggml.lowbit_blob_bytes(2, 4096 * 4096) == 9437184
    assert ggml.lowbit_blob_bytes(2, 11008 * 4096) == 25362432
    assert ggml.lowbit_tileable(2, 4096, 11008) and not ggml.lowbit_tileable(2, 4096, 4544)
    assert not ggml.lowbit_tileable(2, 100, 4096)


def test_abi_rejects_bad_arguments_without_touching_the_gpu():
    lib = ggml._lib
    assert lib.lowbit_quantize(None, None, 99, 16, 128, 0, None) == -2
    assert b"qtype" in lib.lowbit_last_error()
    assert lib.lowbit_quantize(None, None, 2, 16, 100, 0, None) == -5
    assert lib.lowbit_quantize(None, None, 2, 8, 128, 1, None) == -5       # not tileable
    assert lib.lowbit_quantize(None, None, 2, 16, 128, 0, None) == -1      # null pointers
    assert lib.lowbit_gemv(None, None, None, 2, 0, 2, 1, 16, 128, 0, None) == -4   # fp32 activations
    assert lib.lowbit_relayout(ctypes.c_void_p(4096), ctypes.c_void_p(4096 + 16), 2, 16, 128, 0, None) == -1
    assert b"overlap" in lib.lowbit_last_error()
    assert lib.lowbit_quantize(None, None, 2, 0, 128, 0, None) == 0        # empty tensor is fine
    with pytest.raises(RuntimeError):
        ggml.lowbit_quantize(None, None, 99, 16, 128, 0, None)


def test_unsupported_quantizers_raise():
    for f in (ggml.ggml_quantize_tensor_rtn, ggml.ggml_quantize_tensor_with_weights):
        with pytest.raises(RuntimeError):
            f()


@pytest.mark.parametrize("name,per_block", [("sym_int4", (32, 18)), ("asym_int4", (32, 20)),
                                            ("sym_int8", (32, 34)), ("fp8_e4m3", (128, 132))])
def test_convert_qtype_shape_only(name, per_block):
    w = torch.empty(8, 256, dtype=torch.float32, device="meta")
    out = ggml_convert_qtype(w, Q[name], device="meta")
    assert out.dtype == torch.uint8 and out.dim() == 1
    assert out.numel() == 8 * 256 // per_block[0] * per_block[1]
    out2 = ggml_convert_qtype(torch.zeros(8, 256), Q[name], device="cpu", convert_shape_only=True)
    assert out2.shape == out.shape and out2.device.type == "cpu"


def test_convert_qtype_nf4_is_declared_bfloat16():
    # low_bit_linear.py:132-138 of the reference: half as many bf16 elements as bytes
    out = ggml_convert_qtype(torch.empty(4, 128, device="meta"), Q["nf4"], device="meta")
    assert out.dtype == torch.bfloat16 and out.numel() == 4 * 128 // 64 * 34 // 2


def test_convert_qtype_input_checks():
    with pytest.raises(RuntimeError, match="float32"):
        ggml_convert_qtype(torch.zeros(2, 64, dtype=torch.float16), Q["sym_int4"], device="meta")
    with pytest.raises(RuntimeError, match="multiple of 32"):
        ggml_convert_qtype(torch.zeros(2, 48), Q["sym_int4"], device="meta")
    with pytest.raises(RuntimeError, match="multiple of 128"):
        ggml_convert_qtype(torch.zeros(2, 64), Q["fp8_e4m3"], device="meta")
    with pytest.raises(RuntimeError, match="no MI355X kernel"):
        ggml_convert_qtype(torch.zeros(2, 256), Q["q4_k"], device="meta")
    with pytest.raises(RuntimeError, match="scale_search"):
        ggml_convert_qtype(torch.zeros(2, 256), Q["fp8_e4m3"], device="meta", enable_scale_search=True)


def test_fp4params_meta_quantize_keeps_shape_bookkeeping():
    p = FP4Params(torch.empty(16, 128, device="meta"), qtype=Q["sym_int4"])
    q = p.to("meta")
    assert q.quantized and tuple(q._shape) == (16, 128) and q.qtype == 2
    assert q.data.numel() == 16 * 128 // 32 * 18 and q.get_shape() == q._shape
    assert not q.requires_grad


class _Toy(nn.Module):
    def __init__(self):
        super().__init__()
        self.embed = nn.Embedding(10, 128)
        self.block = nn.Sequential(nn.Linear(128, 256, bias=True), nn.ReLU(), nn.Linear(256, 128, bias=False))
        self.odd = nn.Linear(100, 64)          # in_features % 64 != 0 -> kept
        self.keep_me = nn.Linear(128, 128)
        self.lm_head = nn.Linear(128, 10, bias=False)


def test_replace_with_low_bit_linear_rules():
    with torch.device("meta"):
        m = _Toy()
    m.eval()
    m, replaced = _replace_with_low_bit_linear(m, Q["sym_int4"], modules_to_not_convert=["keep_me"],
                                               convert_shape_only=True)
    assert replaced
    assert isinstance(m.block[0], LowBitLinear) and isinstance(m.block[2], LowBitLinear)
    assert type(m.odd) is nn.Linear and type(m.keep_me) is nn.Linear and type(m.embed) is nn.Embedding
    assert m.block[0].bias is not None and m.block[2].bias is None
    assert m.block[0].weight.quantized and tuple(m.block[0].weight._shape) == (256, 128)
    assert m.block[0].weight.data.numel() == 256 * 128 // 32 * 18
    assert not m.block[0].training and not m.block[0].weight.requires_grad
    assert m.lm_head.optimize_lm_head and not m.block[0].optimize_lm_head
    assert (m.block[0].in_len, m.block[0].out_len, m.block[0].weight_shape) == (128, 256, (256, 128))
    # converting twice leaves LowBitLinear layers alone
    m, replaced = _replace_with_low_bit_linear(m, Q["sym_int4"], modules_to_not_convert=["keep_me"],
                                               convert_shape_only=True)
    assert isinstance(m.block[0], LowBitLinear)


def test_convert_low_bit_fp16_and_warning():
    m = nn.Sequential(nn.Linear(64, 64))
    m = ggml_convert_low_bit(m, Q["fp16"])
    assert isinstance(m[0], FP16Linear) and m[0].weight.dtype == torch.float16
    with pytest.warns(UserWarning, match="No linear modules"):
        ggml_convert_low_bit(nn.Sequential(nn.ReLU()), Q["sym_int4"])


def test_optimize_model_argument_checks():
    from ipex_llm import optimize_model
    with pytest.raises(RuntimeError, match="Unknown load_in_low_bit"):
        optimize_model(nn.Linear(64, 64), low_bit="int3")
    with pytest.raises(RuntimeError, match="torch.nn.Module"):
        optimize_model(object())


def test_lm_head_input_keeps_last_position_of_a_prefill():
    x = torch.arange(2 * 12 * 4, dtype=torch.float32).reshape(2, 12, 4)
    y = reshape_lm_head_input(x)
    assert y.shape == (2, 1, 4) and torch.equal(y[:, 0], x[:, -1])
    assert reshape_lm_head_input(x[:, :10]).shape == (2, 10, 4)


def test_forward_of_an_empty_activation():
    layer = LowBitLinear(128, 64, Q["sym_int4"], bias=False)
    y = layer(torch.empty(1, 0, 128, dtype=torch.float16))
    assert y.shape == (1, 0, 64) and y.dtype == torch.float16


def test_use_batch_forward_window():
    """The reference's predicate (low_bit_linear.py:272-307) on a device outside its per-device clauses."""
    x = torch.zeros(4, 256, dtype=torch.half)
    assert use_batch_forward(x, 2, 64) and not use_batch_forward(x[:1], 2, 64)
    assert use_batch_forward(torch.zeros(48, 128, dtype=torch.half), 2, 48)
    assert not use_batch_forward(torch.zeros(49, 128, dtype=torch.half), 2, 64)         # 49..64 rows need K % 256 == 0
    assert use_batch_forward(torch.zeros(64, 256, dtype=torch.float), 3, 128)
    assert not use_batch_forward(torch.zeros(64, 256, dtype=torch.half), 2, 96)         # ... and out_len % 64 == 0
    assert not use_batch_forward(torch.zeros(65, 256, dtype=torch.half), 2, 64)
    assert not use_batch_forward(torch.zeros(4, 192, dtype=torch.half), 2, 64)
    assert not use_batch_forward(torch.zeros(4, 256, dtype=torch.bfloat16), 2, 64)      # float32 and half only
    assert use_batch_forward(x, Q["fp8_e4m3"], 64)
    assert not use_batch_forward(x, Q["sym_int8"], 64) and not use_batch_forward(x, Q["nf4"], 64)


@pytest.mark.skipif(torch.cuda.is_available(), reason="checks the no-GPU failure mode")
def test_real_quantization_without_a_gpu_fails_loudly():
    with pytest.raises(RuntimeError, match="MI355X|failed"):
        ggml_convert_qtype(torch.zeros(2, 64), Q["sym_int4"], device="cpu")


# every name python/llm/src/ipex_llm/ggml/model/llama/llama_cpp.py resolves on the library at import
# (`_lib.<name>.argtypes = ...` / `.restype = ...`, lines 228-1193): a missing one raises AttributeError there
REFERENCE_IMPORT_SYMBOLS = [
    "ggml_quantize_tensor", "ggml_quantize_tensor_with_weights", "ggml_quantize_tensor_rtn",
    "ggml_quantize_tensor_rtn_with_weights", "ggml_type_size", "ggml_qk_size", "ggml_dequantize_q4_0",
    "ggml_quantize_q4_0", "ggml_dequantize", "ggml_q_format_convet_cpu2xpu", "ggml_q_format_convet_xpu2cpu",
    "ggml_compute_forward_mul_mat_q_fp32", "llama_init_backend",
    "llama_apply_lora_from_file", "llama_context_default_params", "llama_copy_state_data", "llama_eval",
    "llama_free", "llama_get_embeddings", "llama_get_kv_cache_token_count", "llama_get_logits",
    "llama_get_state_size", "llama_init_candidates", "llama_init_from_file", "llama_load_session_file",
    "llama_mlock_supported", "llama_mmap_supported", "llama_model_quantize", "llama_n_ctx", "llama_n_embd",
    "llama_n_vocab", "llama_print_system_info", "llama_print_timings", "llama_reset_timings",
    "llama_sample_frequency_and_presence_penalties", "llama_sample_repetition_penalty", "llama_sample_softmax",
    "llama_sample_tail_free", "llama_sample_temperature", "llama_sample_token", "llama_sample_token_greedy",
    "llama_sample_token_mirostat", "llama_sample_token_mirostat_v2", "llama_sample_top_k", "llama_sample_top_p",
    "llama_sample_typical", "llama_save_session_file", "llama_set_rng_seed", "llama_set_state_data",
    "llama_time_us", "llama_token_bos", "llama_token_eos", "llama_token_nl", "llama_token_to_str",
    "llama_tokenize",
]


def test_library_exports_every_symbol_the_reference_resolves_at_import():
    assert len(set(REFERENCE_IMPORT_SYMBOLS)) == 55
    lib = ctypes.CDLL(os.path.join(ROOT, "ipex-llm_amd", "ipex_llm", "libs", "liblowbit_hip.so"))
    for n in REFERENCE_IMPORT_SYMBOLS:
        assert hasattr(lib, n), n


def test_quantizers_outside_the_path_fail_with_a_message():
    lib = ctypes.CDLL(os.path.join(ROOT, "ipex-llm_amd", "ipex_llm", "libs", "liblowbit_hip.so"))
    lib.lowbit_last_error.restype = ctypes.c_char_p
    lib.ggml_quantize_tensor_with_weights.restype = ctypes.c_size_t
    lib.ggml_quantize_tensor_with_weights.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int,
                                                      ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
    assert lib.ggml_quantize_tensor_with_weights(None, None, Q["q4_k"], 1, 256, None, None) == 0
    assert b"not implemented" in lib.lowbit_last_error()
    lib.ggml_quantize_tensor_rtn.restype = ctypes.c_size_t
    lib.ggml_quantize_tensor_rtn.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int,
                                             ctypes.c_size_t, ctypes.c_int, ctypes.c_void_p, ctypes.c_bool]
    assert lib.ggml_quantize_tensor_rtn(None, None, None, 2, 4096, 64, None, False) == 0
    assert b"NPU" in lib.lowbit_last_error()


def test_optimize_pre_merges_qkv_and_the_stock_attention_forward_still_works():
    """convert.py:996-999 / models/common.py:40-52 of the reference: q_proj, k_proj, v_proj become qkv_proj.
    Dense weights on the CPU here (the merge happens before quantization)."""
    transformers = pytest.importorskip("transformers")
    from ipex_llm.transformers.convert import _optimize_pre
    from ipex_llm.transformers.models.common import MergedProjectionSlice
    cfg = transformers.LlamaConfig(hidden_size=64, intermediate_size=128, num_hidden_layers=2,
                                   num_attention_heads=4, num_key_value_heads=2, vocab_size=50,
                                   max_position_embeddings=32)
    torch.manual_seed(3)
    model = transformers.LlamaForCausalLM(cfg).eval()
    attn = model.model.layers[0].self_attn
    wq, wk, wv = (getattr(attn, n).weight.detach().clone() for n in ("q_proj", "k_proj", "v_proj"))
    ids = torch.randint(0, 50, (2, 7))
    with torch.no_grad():
        want = model(ids).logits
    n_params = sum(p.numel() for p in model.parameters())
    model = _optimize_pre(model)
    attn = model.model.layers[0].self_attn
    assert torch.equal(attn.qkv_proj.weight, torch.cat([wq, wk, wv]))
    assert (attn.qkv_proj.in_features, attn.qkv_proj.out_features) == (64, 64 + 32 + 32)
    assert all(isinstance(getattr(attn, n), MergedProjectionSlice) for n in ("q_proj", "k_proj", "v_proj"))
    assert (attn.k_proj.start, attn.k_proj.length, attn.v_proj.start) == (64, 32, 96)
    assert sum(p.numel() for p in model.parameters()) == n_params          # nothing is held twice
    assert not any("q_proj" in k for k in model.state_dict())
    with torch.no_grad():
        got = model(ids).logits
    assert torch.allclose(got, want, atol=1e-5, rtol=1e-5)
    # a slice called on a tensor the merged product was not run on computes its own rows
    x = torch.randn(3, 64)
    assert torch.allclose(attn.v_proj(x), x @ wv.t(), atol=1e-5)
    # merging twice changes nothing; other model types are left alone
    again = _optimize_pre(model)
    assert again.model.layers[0].self_attn.qkv_proj is attn.qkv_proj
    gpt = transformers.GPT2LMHeadModel(transformers.GPT2Config(n_layer=1, n_head=2, n_embd=32, vocab_size=40))
    assert _optimize_pre(gpt) is gpt


def test_merged_qkv_slices_under_inference_mode_and_cache_lifetime():
    """Inference tensors carry no version counter; the merged product is dropped once q, k and v have read
    it; a model whose k/v see another tensor than q (cross-attention) stops running the merged product;
    stock attention code reads `q_proj.weight.dtype` and `q_proj.bias`."""
    transformers = pytest.importorskip("transformers")
    from ipex_llm.transformers.convert import _optimize_pre
    cfg = transformers.LlamaConfig(hidden_size=64, intermediate_size=128, num_hidden_layers=2,
                                   num_attention_heads=4, num_key_value_heads=2, vocab_size=50,
                                   max_position_embeddings=32, attention_bias=True)
    torch.manual_seed(4)
    model = transformers.LlamaForCausalLM(cfg).eval()
    ids = torch.randint(0, 50, (2, 7))
    with torch.no_grad():
        want = model(ids).logits
    attn = model.model.layers[0].self_attn
    wq, wk, bq = attn.q_proj.weight.detach().clone(), attn.k_proj.weight.detach().clone(), attn.q_proj.bias.detach().clone()
    model = _optimize_pre(model)
    with torch.inference_mode():
        got = model(ids).logits
        out = model.generate(ids, max_new_tokens=3, do_sample=False)
    assert torch.allclose(got, want, atol=1e-5, rtol=1e-5) and out.shape == (2, 10)
    for layer in model.model.layers:
        assert layer.self_attn.__dict__.get("_qkv_cache") is None          # no activation stays pinned
    attn = model.model.layers[0].self_attn
    assert attn.q_proj.weight.dtype == torch.float32 and torch.equal(attn.q_proj.weight, wq)
    assert torch.equal(attn.k_proj.weight, wk) and torch.equal(attn.q_proj.bias, bq)
    # cross-attention: q on one tensor, k and v on another
    calls = []
    inner = attn.qkv_proj.forward
    attn.qkv_proj.forward = lambda t: (calls.append(t.shape), inner(t))[1]
    a, b = torch.randn(3, 64), torch.randn(5, 64)
    with torch.inference_mode():
        for _ in range(2):
            q, k, v = attn.q_proj(a), attn.k_proj(b), attn.v_proj(b)
    assert torch.allclose(q, a @ wq.t() + bq, atol=1e-5) and torch.allclose(k, b @ wk.t() + attn.k_proj.bias, atol=1e-5)
    assert v.shape == (5, 32) and attn.__dict__["_qkv_cache"] is None and attn.__dict__["_qkv_apart"]
    assert len(calls) == 1             # merged once; every later call multiplies its own rows only


def test_linears_whose_row_length_is_no_multiple_of_the_block_stay_dense():
    # fp8_e4m3 blocks hold 128 weights: 192 input features pass the reference's % 64 rule but cannot be quantized
    with torch.device("meta"):
        m = nn.Sequential(nn.Linear(192, 64), nn.Linear(256, 64))
    m, replaced = _replace_with_low_bit_linear(m, Q["fp8_e4m3"], convert_shape_only=True)
    assert replaced and type(m[0]) is nn.Linear and isinstance(m[1], LowBitLinear)


def test_fused_mlp_refuses_weights_that_are_not_tiled_blobs_next_to_x():
    """A raw pointer only reaches the fused gate/up kernel after the checks forward_new makes; anything else
    takes the module's own forward."""
    from ipex_llm.transformers.low_bit_linear import mlp_forward_xpu
    from ipex_llm.transformers.models.common import fuse_mlp_base
    x = torch.zeros(1, 128, dtype=torch.half)
    blob = torch.zeros(64 * 128 // 32 * 18, dtype=torch.uint8)
    with pytest.raises(RuntimeError, match="GPU"):
        mlp_forward_xpu(x, blob, blob, 1, 128, 64, 0, 2)                  # x on the CPU

    class Mlp(nn.Module):
        def __init__(self):
            super().__init__()
            self.gate_proj = nn.Linear(128, 64, bias=False)
            self.up_proj = nn.Linear(128, 64, bias=False)
            self.down_proj = nn.Linear(64, 128, bias=False)
            self.act_fn = nn.SiLU()
            self.calls = 0

        def forward(self, x):
            self.calls += 1
            return 2.0 * self.down_proj(self.act_fn(self.gate_proj(x)) * self.up_proj(x))   # not the plain form

    from ipex_llm.transformers.convert import convert_forward
    from ipex_llm.transformers.models.common import mlp_silu_forward
    m = Mlp().eval()
    xf = torch.randn(2, 128)
    want = m(xf)
    convert_forward(m, Mlp, mlp_silu_forward)
    got = m(xf)                                                           # dense CPU weights: cannot be fused
    assert torch.equal(got, want) and m.calls == 2                        # the class's own forward ran
    assert fuse_mlp_base(m, 0, xf).shape == (2, 128)


def test_kernel_choice_boundaries_are_pinned():
    """Which kernel lowbit_forward / lowbit_forward_ws picks is decided by constants fitted on MI355X
    (abi.hip, gemm.hip, gemm_ring.hip).  This table pins today's choices for the BASELINE shapes so that a
    re-fit cannot silently route a shape to another kernel: whoever changes a constant re-measures and edits
    the table.  Host arithmetic only (lowbit_forward_plan)."""
    G, R, M, S, N = ggml.PLAN_GEMV, ggml.PLAN_RING, ggml.PLAN_GEMM, ggml.PLAN_GEMM_SPLIT, ggml.PLAN_GEMM_NARROW

    def plans(qtype, n, k, ms):
        with_ws = [ggml.lowbit_forward_plan(qtype, 1, m, n, k, True, ggml.lowbit_workspace_bytes(m, n, k)) for m in ms]
        without = [ggml.lowbit_forward_plan(qtype, 1, m, n, k, False) for m in ms]
        return with_ws, without
    ms = (1, 16, 17, 32, 64, 128, 256, 511, 512, 1024, 2048)
    #                         1  16  17  32  64 128 256 511 512 1024 2048
    table = {
        (2, 4096, 4096):   ([G, G, G, G, R, S, S, S, S, N, M], [G, G, G, G, G, N, N, N, N, N, M]),
        (2, 11008, 4096):  ([G, G, R, R, R, S, S, M, M, M, M], [G, G, G, G, N, N, N, M, M, M, M]),
        (2, 4096, 11008):  ([G, G, R, R, R, S, S, S, S, S, M], [G, G, G, G, G, G, N, M, M, M, M]),
        (3, 11008, 4096):  ([G, G, R, R, R, S, S, M, M, M, M], [G, G, G, G, N, N, N, M, M, M, M]),
        (10, 8192, 8192):  ([G, G, R, R, R, R, R, S, S, S, M], [G, G, G, G, G, N, N, N, N, N, M]),
        (10, 1024, 8192):  ([G, G, R, R, R, R, R, R, R, R, R], [G, G, G, G, G, G, N, N, N, N, N]),
        (10, 28672, 8192): ([G, G, R, R, R, S, S, M, M, M, M], [G, G, G, G, N, N, N, M, M, M, M]),
        (10, 8192, 28672): ([G, G, R, R, R, S, S, S, S, S, M], [G, G, G, G, G, N, N, N, N, N, M]),
        (8, 28672, 8192):  ([G, G, R, R, R, S, M, M, M, M, M], [G, G, N, N, N, N, M, M, M, M, M]),
        (8, 8192, 28672):  ([G, G, R, R, R, S, S, S, S, S, M], [G, G, G, G, G, N, N, N, N, M, M]),
        (15, 14336, 4096): ([G, G, R, R, R, S, N, M, M, M, M], [G, G, G, G, N, N, N, M, M, M, M]),
    }
    for (qtype, n, k), want in table.items():
        assert plans(qtype, n, k, ms) == (want[0], want[1]), (qtype, n, k, plans(qtype, n, k, ms))
    # the rules that do not depend on fitted constants
    for qtype in (2, 3, 8, 10, 15):
        assert ggml.lowbit_forward_plan(qtype, 1, 16, 4096, 4096, True, 1 << 30) == G        # one streaming pass
        assert ggml.lowbit_forward_plan(qtype, 0, 4096, 4096, 4096, True, 1 << 30) == G      # ggml layout: any-shape kernel
    assert ggml.lowbit_forward_plan(99, 1, 1, 64, 128, False) < 0


class _FusedExperts(nn.Module):
    """The shape of MixtralExperts in current transformers: all experts in two 3-D parameters."""

    def __init__(self, n_exp, hidden, inter):
        super().__init__()
        self.gate_up_proj = nn.Parameter(torch.empty(n_exp, 2 * inter, hidden))
        self.down_proj = nn.Parameter(torch.empty(n_exp, hidden, inter))
        self.act_fn = nn.SiLU()


def test_fused_experts_module_is_replaced_expert_by_expert():
    from ipex_llm.transformers.moe import LowBitExperts

    class Block(nn.Module):
        def __init__(self, hidden, inter):
            super().__init__()
            self.gate = nn.Linear(hidden, 4, bias=False)
            self.experts = _FusedExperts(4, hidden, inter)
    with torch.device("meta"):
        m = nn.Sequential(Block(128, 256)).eval()
    m, replaced = _replace_with_low_bit_linear(m, Q["sym_int4"], convert_shape_only=True)
    ex = m[0].experts
    assert replaced and isinstance(ex, LowBitExperts) and not ex.training
    assert (ex.num_experts, ex.hidden_dim, ex.intermediate_dim) == (4, 128, 256)
    for e in range(4):
        assert tuple(ex.gate[e].weight._shape) == (256, 128) and tuple(ex.up[e].weight._shape) == (256, 128)
        assert tuple(ex.down[e].weight._shape) == (128, 256) and ex.down[e].weight.quantized
        assert ex.gate[e].weight.data.numel() == 256 * 128 // 32 * 18 and not ex.gate[e].weight.requires_grad
    keys = set(m.state_dict().keys())
    assert {"0.experts.gate.0.weight", "0.experts.up.3.weight", "0.experts.down.2.weight"} <= keys
    assert not any("gate_up_proj" in k for k in keys)
    # rows that do not divide into fp8_e4m3's blocks of 128: the module stays as it is
    with torch.device("meta"):
        m2 = nn.Sequential(Block(192, 256)).eval()
    m2, _ = _replace_with_low_bit_linear(m2, Q["fp8_e4m3"], convert_shape_only=True)
    assert isinstance(m2[0].experts, _FusedExperts)


def test_grouped_split_workspace_holds_a_tile_for_every_workgroup():
    """Every workgroup of a K-split grouped launch writes one 256 x 256 fp32 tile at its own index: the workspace
    the library asks for must hold splits x workgroups of them, whatever tile order the launch takes (a grid that
    grew with the tile order once overran a workspace sized from the tile count).  Host arithmetic only."""
    rng = np.random.default_rng(11)
    tile = 256 * 256 * 4
    shapes = [(12, 1917, 272, 2048), (8, 1024, 4096, 14336), (8, 1024, 14336, 4096), (8, 256, 4096, 14336), (1, 40, 512, 8192)]
    shapes += [(int(rng.integers(1, 70)), int(rng.integers(1, 5000)), 16 * int(rng.integers(1, 1200)), 128 * int(rng.integers(1, 120)))
               for _ in range(300)]
    split_seen = False
    for n_groups, rows, n, k in shapes:
        need = ggml.lowbit_grouped_workspace_bytes(n_groups, rows, n, k)
        for ws in {need, need // 2, 0}:
            tall, splits, waves, grid = ggml.lowbit_grouped_forward_plan(n_groups, rows, n, k, ws > 0, ws)
            assert splits >= 1 and waves in (4, 8) and grid % 8 == 0 and grid >= 8
            if splits > 1:
                split_seen = True
                assert tall == 1 and splits * grid * tile <= ws, (n_groups, rows, n, k, ws, splits, grid)
        assert (need == 0) == (ggml.lowbit_grouped_forward_plan(n_groups, rows, n, k, True, 1 << 40)[1] == 1)
    assert split_seen


def test_layout_converters_take_the_reference_signature():
    """ggml_q_format_convet_cpu2xpu(tensor, num_elem, qtype) as the reference calls it (low_bit_linear.py:178-233)
    does what the C symbol of that name does: a copy that stays in the ggml layout."""
    from ipex_llm.transformers.low_bit_linear import ggml_q_format_convet_cpu2xpu, ggml_q_format_convet_xpu2cpu
    blob = torch.arange(18 * 8, dtype=torch.uint8)
    for fn in (ggml_q_format_convet_cpu2xpu, ggml_q_format_convet_xpu2cpu):
        out = fn(blob, 256, Q["sym_int4"])
        assert torch.equal(out, blob) and out.data_ptr() != blob.data_ptr()
    with pytest.raises(RuntimeError, match="uint8"):
        ggml_q_format_convet_cpu2xpu(blob.float(), 256, Q["sym_int4"])


def test_workspace_query_with_a_budget_names_what_the_plan_uses():
    """lowbit_workspace_bytes_for(qtype, layout, M, N, K, budget): never above the budget, zero where the plan has
    no partial tiles, and the plan made with exactly that many bytes is the plan made with the whole budget."""
    G, R, D, S = ggml.PLAN_GEMV, ggml.PLAN_RING, ggml.PLAN_GEMM, ggml.PLAN_GEMM_SPLIT
    for qtype in (2, 3, 8, 10, 15):
        for n, k in ((4096, 4096), (11008, 4096), (4096, 11008), (1024, 8192), (28672, 8192)):
            for m in (1, 16, 24, 64, 128, 512, 2048):
                for budget in (0, 1 << 20, 64 << 20, 256 << 20, 1 << 40):
                    need = ggml.lowbit_workspace_bytes_for(qtype, 1, m, n, k, budget)
                    assert need <= budget
                    plan = ggml.lowbit_forward_plan(qtype, 1, m, n, k, budget >= 16, budget)
                    assert (need > 0) == (plan in (R, S)), (qtype, m, n, k, budget, need, plan)
                    assert ggml.lowbit_forward_plan(qtype, 1, m, n, k, need > 0, need) == (plan if need else ggml.lowbit_forward_plan(qtype, 1, m, n, k, False))
                assert ggml.lowbit_workspace_bytes_for(qtype, 1, m, n, k, 1 << 40) <= ggml.lowbit_workspace_bytes(m, n, k)
        assert ggml.lowbit_workspace_bytes_for(qtype, 0, 512, 4096, 4096, 1 << 30) == 0      # ggml layout: any-shape kernel
