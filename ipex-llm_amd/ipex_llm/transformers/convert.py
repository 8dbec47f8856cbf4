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


def is_gptq_linear(module) -> bool:
    """A 4-bit GPTQ / AWQ linear as AutoGPTQ's QuantLinear or AutoAWQ's WQLinear_GEMM lay it out.
    The reference tests the classes of those packages (convert.py:98-105, 512-513); they are not a
    dependency here, so the layer is recognised by its tensors."""
    return (all(hasattr(module, a) for a in ("qweight", "qzeros", "scales", "group_size", "wf"))
            and getattr(module, "bits", getattr(module, "w_bit", None)) == 4)


def is_linear_module(module):
    """(is_linear, (in_features, out_features, mp_group)): nn.Linear and 4-bit GPTQ / AWQ layers; the
    vLLM / DeepSpeed layer classes of the reference (convert.py:138-232) are not handled."""
    if isinstance(module, nn.Linear):
        return True, (module.in_features, module.out_features, None)
    if is_gptq_linear(module):
        inf = getattr(module, "infeatures", None) or module.in_features
        outf = getattr(module, "outfeatures", None) or module.out_features
        return True, (inf, outf, None)
    return False, (None, None, None)


def _unpack_int32(packed: torch.Tensor, wf: torch.Tensor, axis: int) -> torch.Tensor:
    """Splits every int32 of `packed` into len(wf) 4-bit values (shifts wf) along `axis`:
    the size of that axis grows by len(wf), value j of word r lands at index r * len(wf) + j."""
    n = wf.numel()
    shape = [1] * (packed.dim() + 1)
    shape[axis + 1] = n
    vals = torch.bitwise_and(torch.bitwise_right_shift(packed.unsqueeze(axis + 1), wf.reshape(shape)), 15)
    out_shape = list(packed.shape)
    out_shape[axis] *= n
    return vals.reshape(out_shape).to(torch.uint8)


def convert_gptq(module, awq=False, llm_awq=False, act_order=False):
    """Repacks a 4-bit GPTQ / AWQ layer into an asym_int4 (ggml Q4_1) blob without touching the codes
    (reference: convert.py:379-453).  w[o, i] = scale[g, o] * (q[i, o] - zero[g, o]) becomes
    q * d + m with d = scale and m = -(zero * scale), both fp16; GPTQ stores zero - 1.
    Returns (blob uint8 1-D in the ggml layout, g_id_map or None)."""
    bits = getattr(module, "bits", getattr(module, "w_bit", None))
    invalidInputError(bits == 4, "only 4-bit GPTQ / AWQ layers map onto asym_int4")
    group = int(module.group_size)
    invalidInputError(group % 32 == 0, "group_size must be a multiple of the 32-weight block")
    wf = module.wf.to(torch.int32).reshape(-1)
    scales = module.scales
    zeros = _unpack_int32(module.qzeros, wf, 1).to(torch.int16)             # [groups, out]
    if not awq:
        zeros = zeros + 1
    if awq:
        q = _unpack_int32(module.qweight, wf, 1)                              # [in, out] (llm-awq: [out, in])
        if llm_awq:
            q = q.t()
    else:
        q = _unpack_int32(module.qweight, wf, 0)                              # [in, out]
    g_id_map = None
    if act_order and not awq:
        invalidInputError(module.g_idx.shape[0] == q.shape[0], "g_idx and weight shape mismatch")
        _, g_id_map = torch.sort(module.g_idx)
        q = q[g_id_map, :]
    if llm_awq:
        real = module.in_features // group
        zeros, scales = zeros[:, :real].t(), scales[:, :real].t()
    in_f, out_f = q.shape
    zeros = zeros.reshape(-1, out_f)[: in_f // group]
    scales = scales.reshape(-1, out_f)[: in_f // group]
    # codes: [out, blocks, 32] -> byte j = code j | code j+16 << 4
    qb = q.t().contiguous().reshape(out_f, in_f // 32, 2, 16)
    codes = torch.bitwise_or(qb[:, :, 0, :], torch.bitwise_left_shift(qb[:, :, 1, :], 4))
    # one (d, m) per 32-weight block: every group covers group / 32 consecutive blocks
    d = scales.t().to(torch.float16).repeat_interleave(group // 32, dim=1).contiguous()   # [out, blocks]
    z = zeros.t().to(torch.float16).repeat_interleave(group // 32, dim=1).contiguous()
    m = -(z * d)
    blob = torch.cat([d.unsqueeze(-1).view(torch.uint8), m.unsqueeze(-1).view(torch.uint8), codes], dim=-1)
    return blob.reshape(-1), g_id_map


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
            if is_gptq_linear(module):
                # convert.py:511-545 of the reference: the codes are kept, only the packing changes
                invalidInputError(qtype == ggml_tensor_qtype["asym_int4"],
                                  "GPTQ / AWQ layers convert to asym_int4 only")
                is_awq = hasattr(module, "w_bit")
                has_bias = module.bias is not None and module.bias.abs().sum() != 0
                device = module.qweight.data.device
                invalidInputError(device.type != "meta", "converting from meta device is not supported")
                with _empty_init():
                    new_linear = LowBitLinear(in_features, out_features, qtype, has_bias, mp_group=mp_group,
                                              optimize_lm_head=optimize_lm_head, act_order=act_order)
                weight, g_idx_map = convert_gptq(module, awq=is_awq,
                                                 llm_awq=is_awq and "LLMAWQ" in str(getattr(module, "backend", "")),
                                                 act_order=act_order)
                if act_order:
                    new_linear.g_idx_map = g_idx_map
                new_linear._parameters['weight'] = FP4Params(data=weight, requires_grad=False, quantized=True,
                                                             _shape=(out_features, in_features),
                                                             convert_shape_only=convert_shape_only,
                                                             qtype=qtype).to(device)
                if has_bias:
                    new_linear._parameters['bias'] = nn.Parameter(module.bias.data).to(device)
            elif qtype not in (ggml_tensor_qtype["fp16"], ggml_tensor_qtype["bf16"]):
                if in_features % 64 != 0:
                    continue   # the kernels need in_features to be a multiple of 64
                cur_qtype, cur_imatrix = get_cur_qtype_and_imatrix(qtype, full_module_name,
                                                                   imatrix_data, model_config)
                cur_qtype = check_hidden_size(cur_qtype, in_features)
                from ipex_llm.transformers.low_bit_linear import get_qk_size
                if get_qk_size(cur_qtype) and in_features % get_qk_size(cur_qtype) != 0:
                    continue   # rows that do not divide into blocks (fp8_e4m3: 128 weights) stay dense
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
                if isinstance(module, nn.Linear):
                    module.weight = None

        elif is_fused_experts(module) and qtype not in (ggml_tensor_qtype["fp16"], ggml_tensor_qtype["bf16"]):
            # Current transformers keep the experts of a mixture-of-experts block in one module with 3-D
            # parameters instead of the nn.Linear layers per expert that the reference converts one by one
            # (convert.py:469-748 on transformers 4.37): the whole module is replaced.
            from ipex_llm.transformers.low_bit_linear import get_qk_size
            from ipex_llm.transformers.moe import LowBitExperts
            _, two_i, hidden = module.gate_up_proj.shape
            qk = get_qk_size(qtype)
            if hidden % 64 == 0 and (two_i // 2) % 64 == 0 and (not qk or (hidden % qk == 0 and (two_i // 2) % qk == 0)):
                model._modules[name] = LowBitExperts.from_fused(module, qtype, convert_shape_only=convert_shape_only,
                                                                enable_scale_search=enable_scale_search)
                module.gate_up_proj = None
                module.down_proj = None
                has_been_replaced = True
                continue

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


def is_fused_experts(module):
    """A module that holds all experts of a mixture-of-experts block as two 3-D parameters (MixtralExperts and its
    siblings in current transformers): gate_up_proj [E, 2 I, H], down_proj [E, H, I], and an activation."""
    gate_up, down = getattr(module, "gate_up_proj", None), getattr(module, "down_proj", None)
    return (isinstance(gate_up, nn.Parameter) and isinstance(down, nn.Parameter) and gate_up.dim() == 3 and down.dim() == 3
            and gate_up.shape[0] == down.shape[0] and gate_up.shape[1] == 2 * down.shape[2]
            and gate_up.shape[2] == down.shape[1] and hasattr(module, "act_fn"))


# model types whose attention modules hold q_proj / k_proj / v_proj and get them merged by the reference's
# _optimize_pre (convert.py:954-1008)
_MERGE_QKV_MODEL_TYPES = ("llama", "mistral", "qwen2", "gemma", "gemma2", "minicpm", "stablelm", "mllama")


def _optimize_pre(model, qtype=None):
    """Of the reference's pre-conversion passes (convert.py:880-1076) the one that belongs to the linear
    path: q_proj / k_proj / v_proj become one `qkv_proj`, so that a decode step streams them in one launch
    (convert.py:996-999 for Llama; the merge itself is models/common.py:40-52).  GPTQ checkpoints are left
    alone, as in the reference (convert.py:954-960)."""
    config = getattr(model, "config", None)
    model_type = getattr(config, "model_type", None)
    if model_type not in _MERGE_QKV_MODEL_TYPES:
        return model
    qcfg = getattr(config, "quantization_config", None)
    if (qcfg.get("quant_method") if isinstance(qcfg, dict) else getattr(qcfg, "quant_method", None)) == "gptq":
        return model
    from ipex_llm.transformers.models.common import merge_qkv_base
    for module in list(model.modules()):
        if module.__class__.__name__.endswith("Attention"):
            merge_qkv_base(module, module.__class__)
    return model


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
    """Re-binds `forward` of every sub-module of class target_m (convert.py:1185-1193).  The forward it
    replaces stays reachable as `_forward_before_fusion`: the fused MLP forwards call it whenever a call
    cannot be fused, so that a class whose own forward does more than the plain gated product keeps doing it."""
    import types
    if m.__class__ == target_m:
        if "_forward_before_fusion" not in m.__dict__:
            m.__dict__["_forward_before_fusion"] = m.forward
        m.forward = types.MethodType(new_forward, m)
    for _, sub_m in m.named_children():
        convert_forward(sub_m, target_m, new_forward)
