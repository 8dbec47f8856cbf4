"""Low-bit linear layer on one MI355X.

Host-side mirror of python/llm/src/ipex_llm/transformers/low_bit_linear.py:
same public names (ggml_convert_qtype, FP4Params, LowBitLinear, FP16Linear,
BF16Linear, MatMulLowBit, ...), same argument meaning and error behaviour, but
every byte of arithmetic is done by liblowbit_hip.so through its C ABI.

Weight residency rule used throughout: a blob on the CPU is in the ggml layout
(what the reference saves to disk); a blob on the GPU is in the device layout,
i.e. 16x128 tiles whenever out_features % 16 == 0 and in_features % 128 == 0 and
the ggml layout otherwise.  FP4Params enforces the rule on every way a blob can
reach the GPU (to(), cuda(), construction from a blob that is already there) and
converts back on the way to the CPU, as the reference does with
ggml_q_format_convet_cpu2xpu / _xpu2cpu.
"""
import ctypes
import os
from functools import reduce
from operator import mul

import torch
import torch.nn.functional as F
from torch import nn

import ipex_llm.ggml.model.llama.llama_cpp as ggml
from ipex_llm.ggml.quantize import ggml_tensor_qtype
from ipex_llm.utils.common import invalidInputError

TORCH_LINEAR_THRESHOLD = int(os.getenv("BIGDL_LLM_LINEAR_THRESHOLD", "512"))
SYM_INT4 = ggml_tensor_qtype["sym_int4"]
ASYM_INT4 = ggml_tensor_qtype["asym_int4"]
SYM_INT8 = ggml_tensor_qtype["sym_int8"]
NF4 = ggml_tensor_qtype["nf4"]
NF3 = ggml_tensor_qtype["nf3"]
FP8E4 = ggml_tensor_qtype["fp8_e4m3"]
FP4 = ggml_tensor_qtype["fp4"]
MOFQ4 = ggml_tensor_qtype["mixed_fp4"]
MOFQ8 = ggml_tensor_qtype["mixed_fp8"]
FP8E5 = ggml_tensor_qtype["fp8_e5m2"]
FP6 = ggml_tensor_qtype["fp6"]
FP16 = ggml_tensor_qtype["fp16"]
BF16 = ggml_tensor_qtype["bf16"]

_ACCEL = "cuda"   # device.type of an MI355X under PyTorch-ROCm
_WORKSPACE_CAP = 256 << 20   # most that forward_new borrows for split-K partial sums
_DT = {torch.float16: ggml.DT_F16, torch.bfloat16: ggml.DT_BF16, torch.float32: ggml.DT_F32}


def _stream(device=None):
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def _require_gpu(what):
    invalidInputError(torch.cuda.is_available(),
                      f"{what} needs an MI355X: the low-bit kernels have no CPU implementation.")


def get_block_size(qtype: str):
    return ggml.ggml_qk_size(ggml_tensor_qtype[qtype])


def get_qk_size(qtype: int):
    return ggml.ggml_qk_size(qtype)


def device_layout(qtype: int, weight_shape) -> int:
    """Layout of a weight of this shape while it lives on the GPU."""
    n, k = int(weight_shape[0]), int(weight_shape[-1])
    return ggml.LAYOUT_TILED if ggml.lowbit_tileable(qtype, n, k) else ggml.LAYOUT_GGML


def _blob_like(dst_size, qtype, device):
    # nf4 blobs are declared bfloat16 (half as many elements) as in low_bit_linear.py:132-138 of
    # the reference, so that every parameter of a model shares one dtype under ZeRO-3.
    if qtype == NF4:
        return torch.empty(dst_size // 2, dtype=torch.bfloat16, device=device)
    return torch.empty(dst_size, dtype=torch.uint8, device=device)


def ggml_convert_qtype(tensor: torch.Tensor, qtype: int,
                       device=None, convert_shape_only=False,
                       imatrix: torch.Tensor = None,
                       in_features: int = None,
                       enable_scale_search: bool = False,
                       layout: int = None):
    """fp32 [.., K] -> 1-D packed blob (reference: low_bit_linear.py:104-175).

    The blob is in the ggml layout unless `layout` asks for the tiled one (only meaningful
    for a GPU destination).  A CUDA source is quantized where it is; a CPU source is staged
    through the GPU by ggml_quantize_tensor.
    """
    QK = ggml.ggml_qk_size(qtype)
    block_size_in_bytes = ggml.ggml_type_size(qtype)
    invalidInputError(QK > 0, f"qtype {qtype} has no MI355X kernel in this build "
                              "(supported: sym_int4, asym_int4, sym_int8, nf4, fp8_e4m3)")
    invalidInputError(tensor.dtype == torch.float, "Input tensor must be float32")
    invalidInputError(imatrix is None, "imatrix-weighted quantization is not supported")
    invalidInputError(not enable_scale_search, "enable_scale_search is not supported")
    n = tensor.numel()
    k = tensor.shape[-1]
    invalidInputError(k % QK == 0, f"Last dim of input tensor must be multiple of {QK}")

    dst_size = (n // QK) * block_size_in_bytes
    meta = convert_shape_only or (device is not None and torch.device(device).type == "meta")
    if meta:
        return _blob_like(dst_size, qtype, device)
    if layout is None:
        layout = ggml.LAYOUT_GGML

    if tensor.device.type == _ACCEL:
        src = tensor.contiguous()
        dst = _blob_like(dst_size, qtype, src.device)
        if n:
            with torch.cuda.device(src.device):
                ggml.lowbit_quantize(src.data_ptr(), dst.data_ptr(), qtype, n // k, k, layout, _stream())
        return dst if device is None else dst.to(device)

    invalidInputError(layout == ggml.LAYOUT_GGML, "a CPU source can only produce the ggml layout")
    _require_gpu("ggml_convert_qtype")
    src = tensor.contiguous()
    dst = _blob_like(dst_size, qtype, "cpu")
    if n:
        hist = (ctypes.c_int64 * 16)()
        ggml.ggml_quantize_tensor(ctypes.cast(src.data_ptr(), ctypes.POINTER(ctypes.c_float)),
                                  ctypes.c_void_p(dst.data_ptr()), qtype, n, k, hist, enable_scale_search)
    return dst if device is None else dst.to(device)


def _check_blob_dtype(tensor, qtype):
    if qtype == NF4:
        invalidInputError(tensor.dtype == torch.bfloat16, "NF4 Input tensor must be bfloat16")
    else:
        invalidInputError(tensor.dtype == torch.uint8, "Input tensor except NF4 must be uint8")


def _relayout(tensor, qtype, shape, src_layout):
    """Converts a blob between the ggml and the tiled layout; CPU blobs take a round trip
    through the GPU.  Shapes that cannot be tiled come back unchanged."""
    if device_layout(qtype, shape) == ggml.LAYOUT_GGML:
        return tensor
    _require_gpu("layout conversion")
    src = tensor if tensor.device.type == _ACCEL else tensor.to(_ACCEL)
    src = src.contiguous()
    dst = torch.empty_like(src)
    with torch.cuda.device(src.device):
        ggml.lowbit_relayout(src.data_ptr(), dst.data_ptr(), qtype, int(shape[0]), int(shape[-1]),
                             src_layout, _stream())
    return dst if tensor.device.type == _ACCEL else dst.to(tensor.device)


def ggml_q_format_convet_cpu2xpu(tensor: torch.Tensor, num_elem: int, qtype: int, shape=None):
    """ggml layout -> device layout (reference: low_bit_linear.py:178-204).

    `shape` = (out_features, in_features) is an addition: the tiled device layout interleaves
    16 rows, which the reference's (num_elem, qtype) pair cannot describe.  Called with the reference's
    three arguments it does what the C symbol of the same name does: a copy that stays in the ggml
    layout, which is a valid device weight (layout 0, the any-shape kernels)."""
    _check_blob_dtype(tensor, qtype)
    if shape is None:
        return tensor.clone()
    invalidInputError(reduce(mul, shape, 1) == num_elem, "shape does not hold num_elem weights")
    return _relayout(tensor, qtype, shape, ggml.LAYOUT_GGML)


def ggml_q_format_convet_xpu2cpu(tensor: torch.Tensor, num_elem: int, qtype: int, shape=None):
    """device layout -> ggml layout (reference: low_bit_linear.py:207-233).  Without `shape` the blob
    is taken to be in the ggml layout already (what the three-argument cpu2xpu call leaves): a copy."""
    _check_blob_dtype(tensor, qtype)
    if shape is None:
        return tensor.clone()
    invalidInputError(reduce(mul, shape, 1) == num_elem, "shape does not hold num_elem weights")
    return _relayout(tensor, qtype, shape, ggml.LAYOUT_TILED)


def ggml_convert_fp32(tensor: torch.Tensor, weight_shape: tuple, k: int, qtype: int):
    """ggml blob -> fp32 weight (reference: low_bit_linear.py:249-259)."""
    invalidInputError(tensor.dtype == torch.uint8 or (qtype == NF4 and tensor.dtype == torch.bfloat16),
                      "Input tensor must be uint8")
    if tensor.device.type == _ACCEL:
        return dequant(torch.empty(0, dtype=torch.float32, device=tensor.device), tensor, qtype,
                       layout=ggml.LAYOUT_GGML, shape=(k // weight_shape[-1], weight_shape[-1])
                       ).reshape(weight_shape)
    _require_gpu("ggml_convert_fp32")
    src = tensor.contiguous()
    dst_tensor = torch.empty(weight_shape, dtype=torch.float)
    ggml.ggml_dequantize(ctypes.c_void_p(src.data_ptr()), ctypes.c_void_p(dst_tensor.data_ptr()), k, qtype)
    return dst_tensor


def ggml_int4_convert_fp32(tensor: torch.Tensor, weight_shape: tuple, k: int):
    """sym_int4 ggml blob -> fp32 weight (reference: low_bit_linear.py:236-246)."""
    return ggml_convert_fp32(tensor, weight_shape, k, SYM_INT4)


def reshape_lm_head_input(x):
    # reference: low_bit_linear.py:262-269 - a prefill only needs the logits of its last position
    if x.dim() > 3:
        x = x.reshape([-1, x.shape[-2], x.shape[-1]])
    shape = list(x.size())
    if shape[1] > 10:
        shape[1] = 1
        x = x[:, -1, :].view(shape)
    return x


def use_batch_forward(x: torch.Tensor, qtype: int, output_len: int):
    """Whether LowBitLinear.forward hands this call to batch_forward (reference: low_bit_linear.py:272-307).

    The reference's window for a device that none of its per-device clauses names (they list Intel GPUs: arc,
    pvc, mtl, arl, lnl, bmg): float32 or half x with K a multiple of 128, a 4-bit integer or fp8 weight, up to
    48 rows - 64 when K is a multiple of 256 and the output length one of 64 - and more than one row.  What differs
    between the two branches here is what it is in the reference: batch_forward takes x in the dtype it has (a
    float32 x stays float32), forward_new at more than one row computes in half precision.  The kernels behind
    both are chosen by the row count alone (up to 16 rows one pass of the streaming kernel, then the ring kernel,
    then the tiled GEMM)."""
    batch_size = x.shape[0]
    hard_condition = (
        x.dtype in (torch.float, torch.half)
        and x.shape[1] % 128 == 0
        and qtype in (SYM_INT4, ASYM_INT4, FP8E5, FP8E4)
        and (batch_size <= 48 or (batch_size <= 64 and x.shape[1] % 256 == 0 and output_len % 64 == 0))
    )
    return hard_condition and batch_size > 1


# ------------------------------------------------------------------ device ops
# Stand-ins for the torch ops of the reference (transformers/xpu_ops.py:23-62).

def _as_u8(w):
    return w.view(torch.uint8) if w.dtype != torch.uint8 else w


def forward_new(x: torch.Tensor, w: torch.Tensor, qtype: int, output_size: int, layout: int = None,
                keep_fp32: bool = False):
    """xe_linear.forward_new: y[M, out] = x[M, K] @ dequant(w)[out, K]^T in x.dtype.

    A float32 x is computed in half precision (what LowBitLinear asks for at M > 1, low_bit_linear.py:660-665
    of the reference) unless keep_fp32 is set: then x and y stay fp32 through lowbit_forward_f32."""
    invalidInputError(x.dim() == 2 and x.device.type == _ACCEL and w.device == x.device,
                      "forward_new expects a 2-D activation and a weight on the same GPU")
    invalidInputError(x.dtype in _DT, f"unsupported activation dtype {x.dtype}")
    m, k = x.shape
    if layout is None:
        layout = device_layout(qtype, (output_size, k))
    w = _as_u8(w)
    invalidInputError(w.numel() == ggml.lowbit_blob_bytes(qtype, output_size * k),
                      f"weight blob has {w.numel()} bytes, expected "
                      f"{ggml.lowbit_blob_bytes(qtype, output_size * k)} for [{output_size}, {k}]")
    if keep_fp32 and x.dtype == torch.float32:
        xc = x.contiguous()
        y = torch.empty((m, output_size), dtype=torch.float32, device=x.device)
        if m and output_size:
            with torch.cuda.device(x.device):
                ws_bytes = ggml.lowbit_forward_f32_workspace_bytes(m, output_size, k)
                ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device)
                ggml.lowbit_forward_f32(xc.data_ptr(), w.data_ptr(), y.data_ptr(), qtype, layout, m, output_size, k,
                                        ws.data_ptr(), ws_bytes, _stream())
        return y
    xc = x if x.dtype != torch.float32 else x.half()
    xc = xc.contiguous()
    y = torch.empty((m, output_size), dtype=xc.dtype, device=x.device)
    if m and output_size:
        with torch.cuda.device(x.device):
            # workspace for the fp32 partial tiles of the batch-size kernel and of the GEMM when it
            # splits K; taken from torch's caching allocator, so steady-state calls do not allocate
            # (the library is told the budget and says what the plan it makes within it needs)
            ws_bytes = ggml.lowbit_workspace_bytes_for(qtype, layout, m, output_size, k, _WORKSPACE_CAP)
            if ws_bytes:
                ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device)
                ggml.lowbit_forward_ws(xc.data_ptr(), w.data_ptr(), y.data_ptr(), qtype, layout, _DT[xc.dtype],
                                       m, output_size, k, ws.data_ptr(), ws_bytes, _stream())
            else:
                ggml.lowbit_forward(xc.data_ptr(), w.data_ptr(), y.data_ptr(), qtype, layout, _DT[xc.dtype],
                                    m, output_size, k, _stream())
    return y if y.dtype == x.dtype else y.to(x.dtype)


def batch_forward(x: torch.Tensor, w: torch.Tensor, qtype: int, output_size: int = None, layout: int = None):
    """xe_batch.batch_forward: same product for the row counts of use_batch_forward.  The reference hands it
    x in the dtype it has (low_bit_linear.py:657-659), so a float32 x stays fp32."""
    if output_size is None:
        k = x.shape[1]
        output_size = _as_u8(w).numel() // ggml.ggml_type_size(qtype) * ggml.ggml_qk_size(qtype) // k
    return forward_new(x, w, qtype, output_size, layout, keep_fp32=True)


def dequant(x: torch.Tensor, w: torch.Tensor, qtype: int, layout: int = None, shape=None):
    """xe_linear.dequant: whole weight in x.dtype, flat (reference use: low_bit_linear.py:534-538)."""
    w = _as_u8(w)
    n_w = w.numel() // ggml.ggml_type_size(qtype) * ggml.ggml_qk_size(qtype)
    if shape is None:
        invalidInputError(layout in (None, ggml.LAYOUT_GGML),
                          "dequant of a tiled weight needs shape=(out, in)")
        shape = (n_w // ggml.ggml_qk_size(qtype), ggml.ggml_qk_size(qtype))
        layout = ggml.LAYOUT_GGML
    elif layout is None:
        layout = device_layout(qtype, shape)
    invalidInputError(x.dtype in _DT, f"unsupported dtype {x.dtype}")
    out = torch.empty(n_w, dtype=x.dtype, device=w.device)
    if n_w:
        with torch.cuda.device(w.device):
            ggml.lowbit_dequantize(w.data_ptr(), out.data_ptr(), qtype, int(shape[0]), int(shape[-1]), layout,
                                   _DT[x.dtype], _stream())
    return out


def dequantize_rows(x: torch.Tensor, w: torch.Tensor, qtype: int, state_size: int, output_size: int,
                    layout: int = None):
    """xe_linear.dequantize_rows (embedding.py:218-221, xpu_ops.py:59-62): fp32 [*x.shape, state_size],
    row i = dequantized row x[i] of the [output_size, state_size] weight."""
    invalidInputError(x.device.type == _ACCEL and w.device == x.device,
                      "dequantize_rows expects indices and weight on the same GPU")
    invalidInputError(x.dtype in (torch.int64, torch.int32), "indices must be int64 or int32")
    if layout is None:
        layout = device_layout(qtype, (output_size, state_size))
    w = _as_u8(w)
    invalidInputError(w.numel() == ggml.lowbit_blob_bytes(qtype, output_size * state_size),
                      "weight blob does not match [output_size, state_size]")
    rows = x.contiguous().view(-1).to(torch.int64)
    out = torch.empty((rows.numel(), state_size), dtype=torch.float32, device=x.device)
    if rows.numel():
        with torch.cuda.device(x.device):
            ggml.lowbit_dequantize_rows(w.data_ptr(), rows.data_ptr(), rows.numel(), out.data_ptr(), qtype,
                                        output_size, state_size, layout, ggml.DT_F32, _stream())
    return out.view(*x.shape, state_size)


def mlp_forward_xpu(x: torch.Tensor, weight1: torch.Tensor, weight2: torch.Tensor, batch_size: int,
                    state_size: int, output_size: int, act_type: int, qtype: int):
    """xe_linear.mlp_forward_xpu (models/common.py:152-156, xpu_ops.py:34-37):
    act(x @ W1^T) * (x @ W2^T) in one launch; act_type 0 = SiLU, 1 = GELU (tanh form).  Any number of rows:
    up to 16 run the streaming kernel, more the fused gate/up form of the tiled GEMM (made for prefill batches)."""
    invalidInputError(x.dim() == 2 and x.shape == (batch_size, state_size) and x.device.type == _ACCEL,
                      "mlp_forward_xpu expects x of shape [batch_size, state_size] on the GPU")
    invalidInputError(ggml.lowbit_tileable(qtype, output_size, state_size),
                      "mlp_forward_xpu needs output_size % 16 == 0 and state_size % 128 == 0")
    invalidInputError(x.dtype in _DT, f"unsupported activation dtype {x.dtype}")
    want = ggml.lowbit_blob_bytes(qtype, output_size * state_size)
    for name, w in (("weight1", weight1), ("weight2", weight2)):
        invalidInputError(isinstance(w, torch.Tensor) and w.device == x.device,
                          f"mlp_forward_xpu: {name} must be a quantized blob on the same GPU as x")
        invalidInputError(w.is_contiguous() and _as_u8(w).numel() == want,
                          f"mlp_forward_xpu: {name} has {_as_u8(w).numel()} bytes, expected {want} for "
                          f"[{output_size}, {state_size}]")
        invalidInputError(getattr(w, "blob_layout", ggml.LAYOUT_TILED) == ggml.LAYOUT_TILED,
                          f"mlp_forward_xpu: {name} is not in the tiled device layout")
    xc = (x if x.dtype != torch.float32 else x.half()).contiguous()
    y = torch.empty((batch_size, output_size), dtype=xc.dtype, device=x.device)
    with torch.cuda.device(x.device):
        ggml.lowbit_mlp_forward(xc.data_ptr(), _as_u8(weight1).data_ptr(), _as_u8(weight2).data_ptr(), y.data_ptr(),
                                qtype, _DT[xc.dtype], batch_size, output_size, state_size, act_type, _stream())
    return y if y.dtype == x.dtype else y.to(x.dtype)


# ------------------------------------------------------------------ FP4Params

class FP4Params(torch.nn.Parameter):
    """Parameter holding either the original weight or its packed blob
    (reference: low_bit_linear.py:312-459)."""

    def __new__(cls,
                data=None,
                requires_grad=False,
                quantized=False,
                _shape=None,
                convert_shape_only=False,
                qtype=None,
                imatrix=None,
                in_features=None,
                enable_scale_search=False,
                blob_layout=None):
        if data is None:
            data = torch.empty(0)
        if quantized and blob_layout is None and data.device.type == _ACCEL and _shape is not None \
                and data.numel() and not convert_shape_only:
            # A quantized blob handed to the constructor is in the ggml layout by contract (it is what CPU
            # tensors and checkpoints hold).  One that already lives on the GPU is re-tiled here, so that no
            # GPU-resident FP4Params ever holds a ggml blob of a tileable shape.
            data = _relayout(data, qtype, _shape, ggml.LAYOUT_GGML)
        self = torch.Tensor._make_subclass(cls, data, requires_grad)
        self.data = data
        self.quantized = quantized
        self._shape = _shape
        self.qtype = qtype
        self.convert_shape_only = convert_shape_only
        self.imatrix = imatrix
        self.in_features = in_features
        self.enable_scale_search = enable_scale_search
        return self

    def ggml_mse(self, w, ggml_qtype, device):
        w_quant = ggml_convert_qtype(w, ggml_qtype, device=device,
                                     convert_shape_only=self.convert_shape_only,
                                     enable_scale_search=self.enable_scale_search)
        w_dequant = ggml_convert_fp32(w_quant, w.shape, reduce(mul, w.shape, 1), ggml_qtype)
        return F.mse_loss(w_dequant.to(w.device), w), w_quant

    def quantize(self, device=None):
        """In-place quantization to a ggml-layout blob on `device`."""
        if not self.quantized:
            w = self.data.contiguous().float()
            qtype = self.qtype
            if qtype in (MOFQ4, MOFQ8):
                # mixture-of-formats needs fp4 / picks between two encodings
                # (low_bit_linear.py:351-386); only its integer member has a kernel here
                invalidInputError(device == "meta" or str(device) == "meta",
                                  "mixed_fp4 / mixed_fp8 need the fp4 quantizer, which has no MI355X kernel")
                qtype = SYM_INT4 if qtype == MOFQ4 else SYM_INT8
                self.qtype = qtype
            self.data = ggml_convert_qtype(w, qtype, device=device,
                                           convert_shape_only=self.convert_shape_only,
                                           imatrix=self.imatrix, in_features=self.in_features,
                                           enable_scale_search=self.enable_scale_search)
            if self.data.device.type == _ACCEL:
                self.data = _relayout(self.data, qtype, w.shape, ggml.LAYOUT_GGML)   # residency rule
            self.quantized = True
            self._shape = w.shape
        return self

    def get_shape(self):
        return self._shape

    @property
    def blob_layout(self):
        """Layout of the blob as it is held right now: ggml on the CPU / meta device, the device layout of
        its shape on the GPU.  Derived, not stored: nn.Module._apply swaps `.data` under an existing
        parameter object, which would leave a stored value behind."""
        if not self.quantized or self.data.device.type != _ACCEL or self._shape is None:
            return ggml.LAYOUT_GGML
        return device_layout(self.qtype, self._shape)

    def _clone_with(self, data):
        # `data` already obeys the residency rule: say so, or the constructor would re-tile it
        return FP4Params(data, requires_grad=self.requires_grad, quantized=self.quantized,
                         _shape=self._shape, qtype=self.qtype,
                         enable_scale_search=self.enable_scale_search,
                         blob_layout=device_layout(self.qtype, self._shape)
                         if self.quantized and self._shape is not None and data.device.type == _ACCEL
                         else ggml.LAYOUT_GGML)

    def cuda(self, device=None, non_blocking=False, **kwargs):
        # Tensor.cuda() would copy the bytes as they are: a ggml blob would land on the GPU untiled
        if device is None:
            device = torch.device(_ACCEL, torch.cuda.current_device())
        elif isinstance(device, int):
            device = torch.device(_ACCEL, device)
        return self.to(device=device, non_blocking=non_blocking)

    def cpu(self, **kwargs):
        return self.to(device="cpu")

    def to(self, *args, **kwargs):
        device, dtype, non_blocking, _ = torch._C._nn._parse_to(*args, **kwargs)
        cur = self.data.device.type
        if device is not None and device.type == "cpu" and cur == "cpu":
            return self.quantize(device.type)
        if device is not None and device.type == "meta" and cur == "meta":
            return self.quantize(device.type)
        if device is not None and device.type == _ACCEL and cur == "cpu":
            # upload first, then quantize / re-tile on the GPU: one H2D copy, no CPU arithmetic
            if not self.quantized:
                invalidInputError(self.qtype not in (MOFQ4, MOFQ8), "mixed formats are not supported")
                w = self.data.to(device).contiguous().float()
                self._shape = w.shape
                blob = ggml_convert_qtype(w, self.qtype, layout=device_layout(self.qtype, w.shape),
                                          enable_scale_search=self.enable_scale_search)
                self.quantized = True
            else:
                blob = ggml_q_format_convet_cpu2xpu(self.data.to(device), reduce(mul, self._shape, 1),
                                                    self.qtype, shape=self._shape)
            return self._clone_with(blob)
        if device is not None and device.type == "cpu" and cur == _ACCEL:
            data = self.data
            if self.quantized:
                data = ggml_q_format_convet_xpu2cpu(data, reduce(mul, self._shape, 1), self.qtype,
                                                    shape=self._shape)
            return self._clone_with(data.to(device))
        if device is not None and device.type == _ACCEL and cur == _ACCEL and not self.quantized:
            w = self.data.to(device).contiguous().float()
            self._shape = w.shape
            blob = ggml_convert_qtype(w, self.qtype, layout=device_layout(self.qtype, w.shape))
            self.quantized = True
            return self._clone_with(blob)
        return self._clone_with(super().to(device=device, dtype=None if self.quantized else dtype,
                                           non_blocking=non_blocking))


def ggml_matmul_src1_x_src0_t(src0: torch.Tensor, src1: torch.Tensor, src0_shape: torch.Size, src0_qtype: int):
    """x [M, K] times a CPU-resident ggml blob [N, K] (reference: low_bit_linear.py:462-497).
    Host pointers in, fp32 out; the library stages the operands through the GPU."""
    if src1.dtype != torch.float32:
        src1 = src1.float()
    src1 = src1.contiguous()
    src0 = src0.contiguous()
    result_t = torch.empty((src1.shape[0], src0_shape[0]), dtype=torch.float32)
    src_0_ne = (ctypes.c_int64 * 2)(*tuple(reversed(src0_shape)))
    src_1_ne = (ctypes.c_int64 * 2)(*tuple(reversed(src1.shape)))
    _require_gpu("ggml_matmul_src1_x_src0_t")
    ggml.ggml_compute_forward_mul_mat_q_fp32(src_0_ne, ctypes.c_void_p(src0.data_ptr()), src0_qtype,
                                             src_1_ne, ctypes.c_void_p(src1.data_ptr()),
                                             ctypes.c_void_p(result_t.data_ptr()))
    return result_t


class MatMulLowBit(torch.autograd.Function):
    """forward = fused low-bit product; backward = dequantize + dense matmul for grad_A
    (reference: low_bit_linear.py:500-541)."""

    @staticmethod
    def forward(ctx, A, weight, output_size):
        result = forward_new(A, weight.data, weight.qtype, output_size, layout=weight.blob_layout)
        ctx.tensors = (A, weight) if any(ctx.needs_input_grad[:2]) else (None, None)
        return result

    @staticmethod
    def backward(ctx, grad_output):
        A, weight = ctx.tensors
        grad_A = None
        if ctx.needs_input_grad[0]:
            dequant_weight = dequant(A, weight.data, weight.qtype, layout=weight.blob_layout, shape=weight._shape)
            grad_A = torch.matmul(grad_output.to(A.dtype), dequant_weight.reshape(weight._shape))
        return grad_A, None, None


class MatMulLowBitCPU(torch.autograd.Function):
    """The same for a weight blob that lives on the host (reference: low_bit_linear.py:544-570): forward through
    the ggml-style host-pointer matmul, backward = grad_out times the dequantized weight."""

    @staticmethod
    def forward(ctx, A, weight):
        ctx.tensors = (A, weight) if any(ctx.needs_input_grad[:2]) else (None, None)
        x_2d = A.detach().reshape(-1, A.shape[-1])
        result = ggml_matmul_src1_x_src0_t(weight.data, x_2d.cpu(), weight._shape, weight.qtype)
        return result.view(A.shape[:-1] + (weight._shape[0],)).to(A.device)

    @staticmethod
    def backward(ctx, grad_output):
        A, weight = ctx.tensors
        grad_A = None
        if ctx.needs_input_grad[0]:
            dequant_weight = ggml_convert_fp32(weight.data, weight._shape, weight._shape[0] * weight._shape[1], weight.qtype)
            grad_A = torch.matmul(grad_output, dequant_weight.to(grad_output.dtype).to(grad_output.device))
        return grad_A, None


class LowBitLinear(nn.Linear):
    """nn.Linear whose weight is a packed low-bit blob (reference: low_bit_linear.py:573-715)."""

    def __init__(self, input_features, output_features, qtype, bias=True,
                 conver_to_half=True, mp_group=None,
                 optimize_lm_head=False, act_order=False,
                 enable_scale_search=False):
        super().__init__(input_features, output_features, bias)
        self.weight = FP4Params(self.weight.data,
                                requires_grad=False,
                                quantized=False, _shape=None, qtype=qtype,
                                enable_scale_search=enable_scale_search)
        self.in_len = input_features
        self.out_len = output_features
        self.weight_shape = (self.out_len, self.in_len)
        self.weight_length = self.out_len * self.in_len
        self.qtype = qtype
        self.conver_to_half = conver_to_half
        self.mp_group = mp_group
        self.compute_dtype = None  # only for training
        self.optimize_lm_head = optimize_lm_head
        self.device = None
        self.is_lm_head = self.in_len * self.out_len >= 32000 * 4096 and self.bias is None
        self.low_memory_mode = self.is_lm_head
        self.act_order = act_order
        if act_order:
            self.register_buffer("g_idx_map", torch.arange(self.in_len, dtype=torch.int64))

    def forward(self, x: torch.Tensor):
        if self.device is None:
            self.device = "mi355x" if self.weight.data.device.type == _ACCEL else "cpu"
            # 288 GB of HBM: the cache flush around lm_head is opt-in only
            self.low_memory_mode = self.low_memory_mode and os.environ.get("IPEX_LLM_LOW_MEM", None) == "1"
        is_training = self.training and not torch.is_inference_mode_enabled()
        if is_training and self.compute_dtype is not None and x.device.type == _ACCEL:
            x = x.to(self.compute_dtype)

        if self.bias is not None and self.bias.dtype != x.dtype:
            self.bias.data = self.bias.data.to(x.dtype)

        if self.optimize_lm_head:
            x = reshape_lm_head_input(x)

        new_shape = x.shape[:-1] + (self.out_len,)
        if 0 in x.shape:
            return torch.empty(new_shape, dtype=x.dtype, device=x.device)

        if self.act_order:
            x = x[..., self.g_idx_map]

        x_2d = x.contiguous().view(-1, x.shape[-1])

        if self.weight.device.type == _ACCEL:
            if is_training and x_2d.requires_grad:
                result = MatMulLowBit.apply(x_2d, self.weight, self.out_len)
            else:
                do_empty_cache = self.low_memory_mode and x_2d.shape[0] >= 1024
                if do_empty_cache:
                    torch.cuda.empty_cache()
                w = self.weight.data
                layout = self.weight.blob_layout
                if use_batch_forward(x_2d, self.weight.qtype, self.out_len):
                    result = batch_forward(x_2d, w, self.qtype, self.out_len, layout=layout)
                else:
                    # A float32 x is computed in half precision only where the reference does so: at inference
                    # with conver_to_half and more than one row (low_bit_linear.py:660-665).  One row, or a layer
                    # built with conver_to_half=False, keeps fp32 in and out (:666-668).
                    to_half = not is_training and self.conver_to_half and x_2d.shape[0] > 1
                    result = forward_new(x_2d, w, self.qtype, self.out_len, layout=layout, keep_fp32=not to_half)
                if do_empty_cache:
                    torch.cuda.empty_cache()
            result = result.view(new_shape)
            invalidInputError(self.mp_group is None,
                              "mp_group (tensor parallel all-reduce) is outside this single-GPU build")
            if self.bias is not None:
                result += self.bias
        else:
            # weight blob still on the host: same refusal as the reference for the float formats
            invalidInputError(self.qtype not in (NF3, NF4, FP8E4, FP4, FP8E5),
                              "NF3, NF4, FP4 and FP8 quantization are currently not supported on CPU")
            invalidInputError(self.weight.quantized, "the weight has not been quantized yet: call .to() first")
            if is_training and x.requires_grad:
                result = MatMulLowBitCPU.apply(x, self.weight)
            elif self.qtype == SYM_INT4 and x_2d.shape[0] >= TORCH_LINEAR_THRESHOLD:
                # many rows against a host-resident weight: dequantize once and let the dense fp32 product
                # run where x is (reference: low_bit_linear.py:699-702) - every 16 rows would otherwise cost a
                # pass over the weight behind a copy of x and y across PCIe
                x0_fp32 = ggml_int4_convert_fp32(self.weight.data, self.weight_shape, self.weight_length)
                result = F.linear(x.to(dtype=x0_fp32.dtype), x0_fp32.to(x.device))
            else:
                result = ggml_matmul_src1_x_src0_t(self.weight.data, x_2d.cpu(), self.weight_shape, self.qtype)
                result = result.view(new_shape).to(x.device)
            invalidInputError(self.mp_group is None,
                              "mp_group (tensor parallel all-reduce) is outside this single-GPU build")
            if self.bias is not None:
                result += self.bias
        return result.to(x.dtype)


class FP16Linear(nn.Linear):
    """Dense fp16 linear for load_in_low_bit="fp16" (reference: low_bit_linear.py:718-835)."""

    def __init__(self, input_features, output_features, bias=True,
                 mp_group=None, weight_type=1, optimize_lm_head=False):
        super().__init__(input_features, output_features, bias)
        self.in_len = input_features
        self.out_len = output_features
        self.weight_shape = (self.out_len, self.in_len)
        self.weight_length = self.out_len * self.in_len
        self.qtype = FP16
        self.mp_group = mp_group
        self.weight_type = weight_type
        self.optimize_lm_head = optimize_lm_head
        self.compute_dtype = None
        self.disable_fp16_opt = False

    def forward(self, x: torch.Tensor):
        if self.optimize_lm_head:
            x = reshape_lm_head_input(x)
        invalidInputError(self.mp_group is None, "mp_group is outside this single-GPU build")
        w = self.weight if self.weight.dtype == torch.float16 else self.weight.half()
        b = None if self.bias is None else self.bias.to(torch.float16)
        return F.linear(x.to(torch.float16), w, b).to(x.dtype)


class BF16Linear(nn.Linear):
    """Dense bf16 linear for load_in_low_bit="bf16" (reference: low_bit_linear.py:838-873)."""

    def __init__(self, input_features, output_features, bias=True,
                 mp_group=None, compute_dtype=None, optimize_lm_head=False):
        super().__init__(input_features, output_features, bias)
        self.in_len = input_features
        self.out_len = output_features
        self.weight_shape = (self.out_len, self.in_len)
        self.weight_length = self.out_len * self.in_len
        self.qtype = BF16
        self.mp_group = mp_group
        self.compute_dtype = compute_dtype
        self.optimize_lm_head = optimize_lm_head

    def forward(self, x: torch.Tensor):
        if self.optimize_lm_head:
            x = reshape_lm_head_input(x)
        invalidInputError(self.mp_group is None, "mp_group is outside this single-GPU build")
        w = self.weight if self.weight.dtype == torch.bfloat16 else self.weight.to(torch.bfloat16)
        b = None if self.bias is None else self.bias.to(torch.bfloat16)
        return F.linear(x.to(torch.bfloat16), w, b).to(x.dtype)
