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


# Up to this many rows the fused launch is the streaming kernel's (one pass over both weights).
MLP_FUSION_DECODE_ROWS = 16
# From this many rows on the fused gate/up form of the tiled GEMM beats two products plus the activation as an
# elementwise kernel (measured on MI355X: level at 32 rows for the integer formats and fp8_e4m3, ahead by 18 % with
# nf4; at 17 .. 24 rows two passes of the batch-size kernel win).
MLP_FUSION_PREFILL_ROWS = 32


def mlp_fusion_check(x: torch.Tensor, qtype, training: bool) -> bool:
    """models/utils.py:246-259 of the reference, with this library's limits: the streaming kernel serves up
    to 16 rows (the reference: exactly 1), the fused GEMM a prefill batch, both in fp16 / bf16 above 4 rows, and
    every qtype that has a kernel here."""
    rows = x.numel() // x.size(-1) if x.numel() else 0
    if rows == 0 or MLP_FUSION_DECODE_ROWS < rows < MLP_FUSION_PREFILL_ROWS:
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
