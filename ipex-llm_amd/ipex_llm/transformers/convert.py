"""Module surgery: nn.Linear -> LowBitLinear.

Mirror of the Linear-swap part of the reference's transformers/convert.py
(is_linear_module :138-232, _replace_with_low_bit_linear :469-748,
ggml_convert_low_bit :1079-1171, convert_bigdl_other_module :1174-1182).  The
per-architecture forward patches (_optimize_pre / _optimize_post) belong to the
attention / norm path and are not part of this build.
"""
import logging
import os
import warnings

import torch
from torch import nn

from ipex_llm.ggml.quantize import ggml_tensor_qtype
from ipex_llm.transformers.utils import check_hidden_size, get_cur_qtype_and_imatrix
from ipex_llm.utils.common import invalidInputError

logger = logging.getLogger(__name__)


def is_deepspeed_available():
    return False   # tensor parallel all-reduce is outside this single-GPU build


def get_use_vllm():
    return False


def is_lm_head(name, model_config, out_features):
    return name == "lm_head" or getattr(model_config, "vocab_size", None) == out_features


def is_linear_module(module):
    """(is_linear, (in_features, out_features, mp_group)) - plain nn.Linear only; the vLLM /
    DeepSpeed / GPTQ / AWQ layer classes of the reference are not handled."""
    if isinstance(module, nn.Linear):
        return True, (module.in_features, module.out_features, None)
    return False, (None, None, None)


def use_scale_search(model_config, qtype):
    """The reference searches the block scale for fp6 and most fp8_e4m3 models
    (convert.py:456-466); that search lives in its closed binary and is not reproduced, so
    every layer uses the plain absmax scale."""
    return False


class _empty_init:
    """Stand-in for accelerate.init_empty_weights: parameters created inside live on `meta`."""

    def __enter__(self):
        try:
            from accelerate import init_empty_weights
            self._cm = init_empty_weights()
        except Exception:  # noqa: BLE001
            self._cm = torch.device("meta")
        return self._cm.__enter__()

    def __exit__(self, *exc):
        return self._cm.__exit__(*exc)


def _replace_with_low_bit_linear(model, qtype, modules_to_not_convert=None,
                                 convert_shape_only=False,
                                 cpu_embedding=False,
                                 prefix_name='',
                                 imatrix_data=None, embedding_qtype=None,
                                 model_config=None, torch_dtype=torch.float32,
                                 mixed_precision=False,
                                 act_order=False,
                                 enable_scale_search=False,
                                 ):
    from ipex_llm.transformers.low_bit_linear import BF16Linear, FP16Linear, FP4Params, LowBitLinear
    modules_to_not_convert = modules_to_not_convert or []
    has_been_replaced = False

    for name, module in model.named_children():
        is_linear, linear_args = is_linear_module(module)
        full_module_name = prefix_name + '.' + name if prefix_name != '' else name

        # sub-string match, as in the reference: "0" also matches "10"
        if any(key in full_module_name for key in modules_to_not_convert):
            continue

        if is_linear and not isinstance(module, (LowBitLinear, FP16Linear, BF16Linear)):
            in_features, out_features, mp_group = linear_args
            optimize_lm_head = (is_lm_head(name, model_config, out_features)
                                and os.environ.get("IPEX_LLM_LAST_LM_HEAD", None) != "0")
            new_linear = None
            if qtype not in (ggml_tensor_qtype["fp16"], ggml_tensor_qtype["bf16"]):
                if in_features % 64 != 0:
                    continue   # the kernels need in_features to be a multiple of 64
                cur_qtype, cur_imatrix = get_cur_qtype_and_imatrix(qtype, full_module_name,
                                                                   imatrix_data, model_config)
                cur_qtype = check_hidden_size(cur_qtype, in_features)
                with _empty_init():
                    new_linear = LowBitLinear(in_features, out_features, cur_qtype,
                                              module.bias is not None, mp_group=mp_group,
                                              optimize_lm_head=optimize_lm_head,
                                              enable_scale_search=enable_scale_search)
                device = module.weight.data.device
                paramsLowBit = FP4Params(data=module.weight.data,
                                         requires_grad=False,
                                         quantized=False,
                                         _shape=None,
                                         convert_shape_only=convert_shape_only,
                                         qtype=cur_qtype,
                                         imatrix=cur_imatrix,
                                         in_features=in_features,
                                         enable_scale_search=enable_scale_search).to(device)
                new_linear._parameters['weight'] = paramsLowBit
                if module.bias is not None:
                    new_linear._parameters['bias'] = nn.Parameter(module.bias.data).to(device)
            else:
                half = torch.float16 if qtype == ggml_tensor_qtype["fp16"] else torch.bfloat16
                cls = FP16Linear if qtype == ggml_tensor_qtype["fp16"] else BF16Linear
                module.to(half)
                with _empty_init():
                    new_linear = cls(in_features, out_features, module.bias is not None,
                                     mp_group=mp_group, optimize_lm_head=optimize_lm_head)
                device = module.weight.data.device
                new_linear._parameters['weight'] = nn.Parameter(module.weight)
                if module.bias is not None:
                    new_linear._parameters['bias'] = nn.Parameter(module.bias.data).to(device)

            if new_linear is not None:
                if not module.training:
                    new_linear.eval()
                model._modules[name] = new_linear
                has_been_replaced = True
                model._modules[name].requires_grad_(False)
                module.weight = None

        elif embedding_qtype is not None and type(module) == nn.Embedding:
            # convert.py:726-729 of the reference
            from ipex_llm.transformers.embedding import LowBitEmbedding
            model._modules[name] = LowBitEmbedding.from_embedding(module, convert_shape_only, embedding_qtype)

        if len(list(module.children())) > 0:
            _, _flag = _replace_with_low_bit_linear(
                module, qtype, modules_to_not_convert, convert_shape_only, cpu_embedding,
                prefix_name=full_module_name, imatrix_data=imatrix_data,
                embedding_qtype=embedding_qtype, model_config=model_config, torch_dtype=torch_dtype,
                mixed_precision=mixed_precision, act_order=act_order,
                enable_scale_search=enable_scale_search)
            has_been_replaced = _flag or has_been_replaced
    return model, has_been_replaced


def _optimize_pre(model, qtype=None):
    return model    # q/k/v merging and friends: attention path, not built here


def convert_forward(m, target_m, new_forward):
    """Bind new_forward to every sub-module of class target_m (convert.py:1185-1193 of the reference)."""
    from types import MethodType
    if m.__class__ == target_m:
        m.forward = MethodType(new_forward, m)
    for _, sub_m in m.named_children():
        convert_forward(sub_m, target_m, new_forward)


def _optimize_post(model):
    """Of the reference's per-architecture patches only the gated-MLP fusion belongs to the low-bit
    linear path (its kernel is xe_linear.mlp_forward_xpu).  The reference wires it per model class
    (convert.py:1298, 1720-1739 ...); here every `*MLP` module with low-bit gate / up / down
    projections and a SiLU or tanh-GELU activation gets it."""
    from ipex_llm.transformers.low_bit_linear import LowBitLinear
    from ipex_llm.transformers.models.common import mlp_gelu_forward, mlp_silu_forward
    seen = set()
    for module in model.modules():
        cls = module.__class__
        if cls in seen or not cls.__name__.endswith("MLP"):
            continue
        projs = [getattr(module, n, None) for n in ("gate_proj", "up_proj", "down_proj")]
        act = getattr(module, "act_fn", None)
        if not all(isinstance(p, LowBitLinear) for p in projs) or act is None:
            continue
        act_name = act.__class__.__name__
        if isinstance(act, nn.SiLU) or act_name in ("SiLUActivation", "SiLU"):
            seen.add(cls)
            convert_forward(model, cls, mlp_silu_forward)
        elif (isinstance(act, nn.GELU) and act.approximate == "tanh") or act_name in ("PytorchGELUTanh", "GELUTanh",
                                                                                      "NewGELUActivation"):
            seen.add(cls)
            convert_forward(model, cls, mlp_gelu_forward)
    return model


def ggml_convert_low_bit(model, qtype, optimize_model=True,
                         convert_shape_only=False, device="cpu",
                         modules_to_not_convert=None,
                         cpu_embedding=False,
                         torch_dtype="auto",
                         imatrix_data=None,
                         embedding_qtype=None,
                         mixed_precision=False,
                         disable_optimize_pre=False):
    if qtype in ggml_tensor_qtype.values():
        index = list(ggml_tensor_qtype.values()).index(qtype)
        logger.info(f"Converting the current model to {list(ggml_tensor_qtype.keys())[index]} format......")
    invalidInputError(not cpu_embedding and imatrix_data is None and not mixed_precision,
                      "cpu_embedding / imatrix / mixed_precision are outside the low-bit linear path built here")
    modules_to_not_convert = [] if modules_to_not_convert is None else modules_to_not_convert

    if optimize_model and not disable_optimize_pre:
        model = _optimize_pre(model, qtype)

    model_config = getattr(model, "config", None)
    enable_scale_search = use_scale_search(model_config, qtype)

    if qtype is not None:
        model, has_been_replaced = _replace_with_low_bit_linear(
            model, qtype, modules_to_not_convert, convert_shape_only, cpu_embedding,
            imatrix_data=imatrix_data, embedding_qtype=embedding_qtype, model_config=model_config,
            torch_dtype=torch_dtype, mixed_precision=mixed_precision, act_order=False,
            enable_scale_search=enable_scale_search)
        if not has_been_replaced:
            warnings.warn("No linear modules were found in your model. This can happen for some "
                          "architectures such as gpt2 that uses Conv1D instead of Linear layers.")
        elif device == "cpu" and not convert_shape_only:
            convert_bigdl_other_module(model, torch.float32 if torch_dtype == "auto" else torch_dtype)

    if optimize_model:
        model = _optimize_post(model)
    return model


def convert_bigdl_other_module(model, dtype):
    """Every leaf that is not one of our linears follows `dtype` (convert.py:1174-1182)."""
    from ipex_llm.transformers.low_bit_linear import BF16Linear, FP16Linear, LowBitLinear
    for module in model.modules():
        if list(module.children()) == []:
            if not isinstance(module, (LowBitLinear, FP16Linear, BF16Linear)):
                module.to(dtype)


def convert_forward(m, target_m, new_forward):
    """Re-binds `forward` of every sub-module of class target_m (convert.py:1185-1193)."""
    import types
    if m.__class__ == target_m:
        m.forward = types.MethodType(new_forward, m)
    for _, sub_m in m.named_children():
        convert_forward(sub_m, target_m, new_forward)
