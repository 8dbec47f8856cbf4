"""Per-layer qtype routing helpers (reference: transformers/utils.py:286-356, 380-398)."""
import logging

from ipex_llm.ggml.quantize import ggml_tensor_qtype

logging.basicConfig(level=logging.INFO)
logger = logging.getLogger(__name__)


def get_cur_qtype_and_imatrix(qtype, full_module_name, imatrix_data, model_config=None):
    """The importance-matrix / k-quant mixtures of the reference re-route some layers; for the
    five qtypes of this build the routing is the identity and there is never an imatrix."""
    return qtype, None


def check_hidden_size(qtype, hidden_size):
    """k-quants need in_features % 256 == 0 and fall back otherwise (transformers/utils.py:380-398).
    None of them has a kernel here, so only the fall-back targets can come out."""
    if hidden_size % 256 != 0:
        fallback = {ggml_tensor_qtype["q4_k"]: "asym_int4", ggml_tensor_qtype["q6_k"]: "sym_int8"}
        if qtype in fallback:
            logger.info(f"hidden size {hidden_size} is not divisible by 256 - using {fallback[qtype]}")
            return ggml_tensor_qtype[fallback[qtype]]
    return qtype


def get_xpu_device_name(device):
    """Device family string (reference: transformers/utils.py:176-183)."""
    return "mi355x" if getattr(device, "type", str(device)) == "cuda" else "cpu"
