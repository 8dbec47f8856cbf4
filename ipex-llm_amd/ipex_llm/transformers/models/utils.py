"""The part of the reference's transformers/models/utils.py that belongs to the low-bit linear
path: when the gate and up projections of a gated MLP may be fused into one launch."""
import torch

from ipex_llm.ggml.quantize import ggml_tensor_qtype

SILU = 0
GELU = 1

SYM_INT4 = ggml_tensor_qtype["sym_int4"]
ASYM_INT4 = ggml_tensor_qtype["asym_int4"]
SYM_INT8 = ggml_tensor_qtype["sym_int8"]
NF4 = ggml_tensor_qtype["nf4"]
FP8E4 = ggml_tensor_qtype["fp8_e4m3"]


def mlp_fusion_check(x: torch.Tensor, qtype, training: bool) -> bool:
    """models/utils.py:246-259 of the reference, with this library's limits: any number of rows (the reference:
    exactly 1) - the streaming kernel fuses gate and up at decode batch sizes, the tiled GEMM beyond (measured on
    MI355X against two products plus the activation as elementwise kernels: ahead or level at every row count) - in
    fp16 / bf16 above 4 rows, and every qtype that has a kernel here."""
    rows = x.numel() // x.size(-1) if x.numel() else 0
    if rows == 0:
        return False
    if rows > 4 and x.dtype not in (torch.float16, torch.bfloat16):
        return False
    if x.device.type != "cuda":
        return False
    if qtype not in (SYM_INT4, ASYM_INT4, SYM_INT8, NF4, FP8E4):
        return False
    if training or x.requires_grad:
        return False
    return True
