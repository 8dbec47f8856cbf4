"""GPTQ / AWQ -> asym_int4 repack (reference: transformers/convert.py:379-453): the codes are kept,
only the packing changes, so the expected blob and weights follow from the definition
w[o, i] = scale[g, o] * (q[i, o] - zero[g, o])."""
import numpy as np
import pytest
import torch
from torch import nn

import np_formats as npf
from ipex_llm.ggml.quantize import ggml_tensor_qtype as Q
from ipex_llm.transformers.convert import _replace_with_low_bit_linear, convert_gptq, is_gptq_linear

ORDER_GPTQ = list(range(8))
ORDER_AWQ = [0, 4, 1, 5, 2, 6, 3, 7]       # AutoAWQ's interleave: nibble j holds column ORDER[j]


def _pack(vals, axis, order=ORDER_GPTQ):
    """8 consecutive 4-bit values along `axis` -> one int32 (value `order[j]` in nibble j)."""
    v = np.moveaxis(vals.astype(np.int64), axis, -1)
    v = v.reshape(*v.shape[:-1], -1, 8)
    word = np.zeros(v.shape[:-1], dtype=np.int64)
    for j in range(8):
        word |= v[..., order[j]] << (4 * j)
    word = np.where(word >= 2 ** 31, word - 2 ** 32, word).astype(np.int32)
    return torch.from_numpy(np.moveaxis(word, -1, axis).copy())


class FakeQuantLinear(nn.Module):
    """Tensors of AutoGPTQ's QuantLinear (bits=4)."""

    def __init__(self, q, zeros, scales, group, g_idx=None, bias=None):
        super().__init__()
        in_f, out_f = q.shape
        self.bits, self.group_size, self.infeatures, self.outfeatures = 4, group, in_f, out_f
        self.register_buffer("qweight", _pack(q, 0))                       # [in / 8, out]
        self.register_buffer("qzeros", _pack(zeros - 1, 1))                # [groups, out / 8], zero - 1
        self.register_buffer("scales", torch.from_numpy(scales))           # [groups, out] fp16
        self.register_buffer("g_idx", torch.from_numpy(g_idx if g_idx is not None
                                                       else np.arange(in_f) // group).to(torch.int32))
        self.register_buffer("wf", torch.arange(0, 32, 4, dtype=torch.int32))
        self.bias = None if bias is None else nn.Parameter(torch.from_numpy(bias))


def _case(seed, in_f=256, out_f=48, group=128):
    r = np.random.default_rng(seed)
    q = r.integers(0, 16, (in_f, out_f))
    zeros = r.integers(1, 17, (in_f // group, out_f))
    scales = (r.random((in_f // group, out_f)) * 0.02 + 0.001).astype(np.float16)
    return q, zeros, scales


def _expected(q, zeros, scales, group):
    d = np.repeat(scales.T, group // 32, axis=1)                            # [out, blocks] fp16
    z = np.repeat(zeros.T, group // 32, axis=1).astype(np.float16)
    m = -(z * d)                                                            # fp16 product, one rounding
    codes = q.T.reshape(q.shape[1], -1, 32)
    w = codes * d[..., None].astype(np.float32) + m[..., None].astype(np.float32)
    return d, m, codes, w.reshape(q.shape[1], q.shape[0])


def test_gptq_repack_gives_the_q4_1_blob_of_the_same_codes():
    q, zeros, scales = _case(1)
    mod = FakeQuantLinear(q, zeros, scales, 128)
    assert is_gptq_linear(mod) and not is_gptq_linear(nn.Linear(8, 8))
    blob, g_map = convert_gptq(mod)
    assert g_map is None and blob.dtype == torch.uint8 and blob.numel() == 48 * 256 // 32 * 20
    d, m, codes, w = _expected(q, zeros, scales, 128)
    got = blob.numpy().reshape(48, 8, 20)
    assert np.array_equal(got[..., 0:2].copy().view(np.float16)[..., 0], d)
    assert np.array_equal(got[..., 2:4].copy().view(np.float16)[..., 0], m)
    assert np.array_equal(got[..., 4:] & 15, codes[..., :16]) and np.array_equal(got[..., 4:] >> 4, codes[..., 16:])
    # the decoder restated from the reference's gguf reader sees the weights of the definition
    assert np.array_equal(npf.decode_q4_1(blob.numpy(), (48, 256)), w.astype(np.float32))
    true_w = (q.T - np.repeat(zeros.T, 128, axis=1)) * np.repeat(scales.T, 128, axis=1).astype(np.float32)
    assert np.abs(w - true_w).max() <= 16 * 0.021 * 2.0 ** -10


def test_act_order_sorts_rows_by_group_and_returns_the_map():
    q, zeros, scales = _case(2)
    r = np.random.default_rng(3)
    g_idx = np.repeat(np.arange(2), 128)
    r.shuffle(g_idx)
    blob, g_map = convert_gptq(FakeQuantLinear(q, zeros, scales, 128, g_idx=g_idx), act_order=True)
    assert np.array_equal(np.sort(g_idx), g_idx[g_map.numpy()])
    _, _, _, w_sorted = _expected(q[g_map.numpy()], zeros, scales, 128)
    assert np.array_equal(npf.decode_q4_1(blob.numpy(), (48, 256)), w_sorted.astype(np.float32))
    # x[..., g_map] @ W_sorted^T == x @ W^T with W in the original input order
    w_orig = np.empty_like(w_sorted)
    w_orig[:, g_map.numpy()] = w_sorted
    true_w = (q.T - zeros.T[:, g_idx]) * scales.T[:, g_idx].astype(np.float32)
    assert np.abs(w_orig - true_w).max() <= 16 * 0.021 * 2.0 ** -10


def test_awq_repack_uses_the_modules_shift_table_and_plain_zeros():
    q, zeros, scales = _case(4)
    zeros = zeros - 1                                                       # AWQ stores the zero itself (0 .. 15)

    class FakeWQLinear(nn.Module):
        def __init__(self):
            super().__init__()
            self.w_bit, self.group_size, self.in_features, self.out_features = 4, 128, 256, 48
            self.register_buffer("qweight", _pack(q, 1, ORDER_AWQ))           # [in, out / 8]
            self.register_buffer("qzeros", _pack(zeros, 1, ORDER_AWQ))
            self.register_buffer("scales", torch.from_numpy(scales))
            # shift that recovers column j: column ORDER[n] sits in nibble n
            self.register_buffer("wf", torch.tensor([4 * ORDER_AWQ.index(j) for j in range(8)], dtype=torch.int32))
            self.bias = None
    blob, _ = convert_gptq(FakeWQLinear(), awq=True)
    _, _, _, w = _expected(q, zeros, scales, 128)
    assert np.array_equal(npf.decode_q4_1(blob.numpy(), (48, 256)), w.astype(np.float32))


@pytest.mark.gpu
def test_converted_gptq_layer_runs_on_the_gpu():
    from ipex_llm.transformers.low_bit_linear import LowBitLinear
    q, zeros, scales = _case(5, in_f=256, out_f=64)
    bias = np.linspace(-1, 1, 64).astype(np.float32)

    class Net(nn.Module):
        def __init__(self):
            super().__init__()
            self.proj = FakeQuantLinear(q, zeros, scales, 128, bias=bias)
    net, replaced = _replace_with_low_bit_linear(Net(), Q["asym_int4"])
    assert replaced and isinstance(net.proj, LowBitLinear) and net.proj.weight.quantized
    _, _, _, w = _expected(q, zeros, scales, 128)
    x = torch.randn(3, 256).half()
    y = net.to("cuda").proj(x.cuda()).float().cpu().numpy()
    want = x.float().numpy() @ w.T.astype(np.float32) + bias
    assert np.abs(y - want).max() <= 2e-3 * np.abs(want).max()


@pytest.mark.gpu
def test_gptq_layer_converted_while_already_on_the_gpu():
    """The packed tensors of the source layer sit on the GPU, so the repacked blob is born there in the ggml
    layout; the parameter has to re-tile it (nothing passes through FP4Params.to from the CPU here)."""
    import lowbit_oracle as orc
    from ipex_llm.transformers.low_bit_linear import LowBitLinear
    import ipex_llm.ggml.model.llama.llama_cpp as ggml
    q, zeros, scales = _case(6, in_f=256, out_f=64)

    class Net(nn.Module):
        def __init__(self):
            super().__init__()
            self.proj = FakeQuantLinear(q, zeros, scales, 128)
    blob_cpu, _ = convert_gptq(FakeQuantLinear(q, zeros, scales, 128))
    net, replaced = _replace_with_low_bit_linear(Net().to("cuda"), Q["asym_int4"])
    assert replaced and isinstance(net.proj, LowBitLinear)
    wp = net.proj.weight
    assert wp.data.device.type == "cuda" and wp.blob_layout == ggml.LAYOUT_TILED
    assert not torch.equal(wp.data.cpu(), blob_cpu)                       # tiled on the device ...
    assert torch.equal(wp.to("cpu").data, blob_cpu)                        # ... the ggml bytes again on the host
    x = torch.randn(3, 256).half()
    y = net.proj(x.cuda()).float().cpu().numpy()
    want = orc.mul_mat_exact(blob_cpu.numpy(), x.float().numpy(), (64, 256), Q["asym_int4"])
    assert np.abs(y - want).max() <= 2e-3 * np.abs(want).max()
