"""AutoModel* shells: from_pretrained(load_in_low_bit=...), save_low_bit, load_low_bit.

Mirror of the API surface of the reference's transformers/model.py (from_pretrained :111-388,
load_convert :411-528, save_low_bit :59-103, load_low_bit :532-785), re-expressed with the
public Hugging Face API of the installed transformers release.  Only local directories can
be loaded (no hub access here).  The on-disk format is the reference's: a `pytorch_model.bin`
holding 1-D uint8 blobs in the ggml layout, config.json stamped with
`bigdl_transformers_low_bit`, and `load_keys.json`.
"""
import json
import logging
import os
import types

import torch

from ipex_llm.ggml.quantize import ggml_tensor_qtype
from ipex_llm.utils.common import invalidInputError

logger = logging.getLogger(__name__)

PYTORCH_MODEL_NAME = "pytorch_model.bin"


def save_low_bit(self, *args, **kwargs):
    """Writes the low-bit model: config.json (stamped), pytorch_model.bin, load_keys.json."""
    invalidInputError(self.config.to_dict().get("bigdl_transformers_low_bit", False),
                      "Detected this model is not a low-bit model, please use from_pretrained's"
                      " load_in_4bit or load_in_low_bit parameter to load a 4-bit model first.")
    save_dir = args[0] if args else kwargs["save_directory"]
    os.makedirs(save_dir, exist_ok=True)
    from ipex_llm.optimize import _cpu_state
    state = {k: v.detach().to("cpu").contiguous() for k, v in _cpu_state(self).items()}
    self.config.save_pretrained(save_dir)
    if getattr(self, "generation_config", None) is not None:
        try:
            self.generation_config.save_pretrained(save_dir)
        except Exception:  # noqa: BLE001
            pass
    torch.save(state, os.path.join(save_dir, PYTORCH_MODEL_NAME))
    with open(os.path.join(save_dir, "load_keys.json"), "w") as json_file:
        json.dump({"all_checkpoint_keys": list(state.keys())}, json_file)


class _BaseAutoModelClass:
    HF_Model = None

    @classmethod
    def from_pretrained(cls, *args, **kwargs):
        """Hugging Face from_pretrained plus load_in_4bit / load_in_low_bit / optimize_model /
        modules_to_not_convert (reference: transformers/model.py:111-388)."""
        from transformers import PretrainedConfig
        pretrained_model_name_or_path = kwargs.get("pretrained_model_name_or_path", None) \
            if len(args) == 0 else args[0]
        model_hub = kwargs.pop("model_hub", "huggingface")
        invalidInputError(model_hub in ["huggingface", "modelscope"],
                          "The parameter `model_hub` is supposed to be `huggingface` or "
                          f"`modelscope`, but got {model_hub}.")
        invalidInputError(model_hub == "huggingface", "only local Hugging Face directories can be loaded here")
        invalidInputError(not (kwargs.get('device_map') and 'cuda' in str(kwargs['device_map'])),
                          "Please do not use `device_map` with a GPU value as an argument. "
                          "Use model.to('cuda') instead.")
        config_dict, _ = PretrainedConfig.get_config_dict(pretrained_model_name_or_path)
        bigdl_transformers_low_bit = config_dict.pop("bigdl_transformers_low_bit", False)
        invalidInputError(not bigdl_transformers_low_bit,
                          f"Detected model is a low-bit({bigdl_transformers_low_bit}) model, "
                          f"Please use load_low_bit to load this model.")

        load_in_4bit = kwargs.pop("load_in_4bit", False)
        load_in_low_bit = kwargs.pop("load_in_low_bit", None)
        optimize_model = kwargs.pop("optimize_model", True)
        user_quantization_config = kwargs.pop("quantization_config", None)
        speculative = kwargs.pop("speculative", False)
        pipeline_parallel_stages = kwargs.pop("pipeline_parallel_stages", 1)
        torch_dtype = kwargs.pop("torch_dtype", None)
        embedding_qtype = kwargs.pop("embedding_qtype", None)
        invalidInputError(user_quantization_config is None and not speculative
                          and pipeline_parallel_stages == 1,
                          "quantization_config / speculative / pipeline_parallel_stages "
                          "are outside the low-bit linear path built here")

        if load_in_4bit or load_in_low_bit:
            if load_in_low_bit == "fp16":
                invalidInputError(torch_dtype is None or torch_dtype == torch.float16,
                                  "Please use torch_dtype=torch.float16 when setting load_in_low_bit='fp16'.")
                kwargs["torch_dtype"] = torch.float16
            elif load_in_low_bit == "bf16":
                invalidInputError(torch_dtype is None or torch_dtype == torch.bfloat16,
                                  "Please use torch_dtype=torch.bfloat16 when setting load_in_low_bit='bf16'.")
                kwargs["torch_dtype"] = torch.bfloat16
            else:
                kwargs["torch_dtype"] = torch_dtype or "auto"
            q_k = load_in_low_bit if load_in_low_bit else "sym_int4"
            invalidInputError(q_k not in ["sym_int4_rtn", "sym_int8_rtn"],
                              f"The dtype {q_k} is specified for NPU and cannot be used on CPU and GPU")
            invalidInputError(kwargs.pop("imatrix", None) is None, "imatrix quantization is not supported")
            kwargs["embedding_qtype"] = embedding_qtype
            model = cls.load_convert(q_k, optimize_model, *args, **kwargs)
        else:
            if torch_dtype is not None:
                kwargs["torch_dtype"] = torch_dtype
            kwargs.pop("modules_to_not_convert", None)
            model = cls.HF_Model.from_pretrained(*args, **kwargs)
        return model

    @classmethod
    def load_convert(cls, q_k, optimize_model, *args, **kwargs):
        from ipex_llm.transformers.convert import ggml_convert_low_bit
        invalidInputError(q_k in ggml_tensor_qtype,
                          f"Unknown load_in_low_bit value: {q_k}, expected:"
                          f" sym_int4, asym_int4, sym_int8, nf4, fp8_e4m3, fp16 or bf16.")
        qtype = ggml_tensor_qtype[q_k]
        modules_to_not_convert = kwargs.pop("modules_to_not_convert", None)
        cpu_embedding = kwargs.pop("cpu_embedding", False)
        disk_embedding = kwargs.pop("disk_embedding", False)
        mixed_precision = kwargs.pop("mixed_precision", False)
        disable_optimize_pre = kwargs.pop("disable_optimize_pre", False)
        embedding_qtype = kwargs.pop("embedding_qtype", None)
        if embedding_qtype is not None:
            # the reference documents 'q2_k' / 'q4_k' here (model.py:148); any qtype with a kernel works
            invalidInputError(embedding_qtype in ("sym_int4", "asym_int4", "sym_int8", "nf4", "fp8_e4m3"),
                              f"embedding_qtype {embedding_qtype} has no MI355X kernel")
            embedding_qtype = ggml_tensor_qtype[embedding_qtype]
        invalidInputError(not disk_embedding, "disk_embedding is outside the path built here")
        kwargs.pop('device_map', None)
        torch_dtype = kwargs.pop("torch_dtype", "auto")
        hf_kwargs = dict(kwargs)
        hf_kwargs["dtype"] = torch_dtype
        try:
            model = cls.HF_Model.from_pretrained(*args, **hf_kwargs)
        except TypeError:
            hf_kwargs.pop("dtype")
            hf_kwargs["torch_dtype"] = torch_dtype
            model = cls.HF_Model.from_pretrained(*args, **hf_kwargs)

        model = model.to("cpu")
        model = ggml_convert_low_bit(model, qtype, optimize_model,
                                     modules_to_not_convert=modules_to_not_convert,
                                     cpu_embedding=cpu_embedding,
                                     torch_dtype=torch_dtype,
                                     embedding_qtype=embedding_qtype,
                                     mixed_precision=mixed_precision,
                                     disable_optimize_pre=disable_optimize_pre)
        model.config.update({"bigdl_transformers_low_bit": q_k, "bigdl_disk_embedding": False})
        model.config.update({"tie_word_embeddings": False})
        model.save_low_bit = types.MethodType(save_low_bit, model)
        return model

    @classmethod
    def load_low_bit(cls, pretrained_model_name_or_path, *model_args, **kwargs):
        """Rebuilds a model saved by save_low_bit: the skeleton is created on the meta device,
        its linears are swapped shape-only, then the saved tensors are assigned."""
        from transformers import AutoConfig
        from ipex_llm.optimize import _assign
        from ipex_llm.transformers.convert import ggml_convert_low_bit
        optimize_model = kwargs.pop("optimize_model", True)
        modules_to_not_convert = kwargs.pop("modules_to_not_convert", None)
        torch_dtype = kwargs.pop("torch_dtype", "auto")
        embedding_qtype = kwargs.pop("embedding_qtype", None)     # as in the reference (model.py:588)
        if embedding_qtype is not None:
            embedding_qtype = ggml_tensor_qtype[embedding_qtype]
        config = AutoConfig.from_pretrained(pretrained_model_name_or_path)
        low_bit = config.to_dict().get("bigdl_transformers_low_bit", None)
        invalidInputError(low_bit,
                          "Detect this model is not a low-bit model, Please use from_pretrained"
                          " with load_in_4bit or load_in_low_bit to get a low-bit model , and "
                          " serialize the model using save_low_bit first.")
        invalidInputError(low_bit in ggml_tensor_qtype, f"Unknown bigdl_transformers_low_bit value: {low_bit}")
        qtype = ggml_tensor_qtype[low_bit]
        from ipex_llm.optimize import unconverted_linears
        state_dict = torch.load(os.path.join(pretrained_model_name_or_path, PYTORCH_MODEL_NAME),
                                weights_only=True)
        with torch.device("meta"):
            model = cls.HF_Model.from_config(config)
        skip = list(modules_to_not_convert or []) + unconverted_linears(state_dict)
        model = ggml_convert_low_bit(model, qtype, optimize_model, device="meta",
                                     convert_shape_only=True, modules_to_not_convert=skip,
                                     embedding_qtype=embedding_qtype)
        keys_file = os.path.join(pretrained_model_name_or_path, "load_keys.json")
        if os.path.isfile(keys_file):
            with open(keys_file) as f:
                expected = json.load(f)["all_checkpoint_keys"]
            invalidInputError(set(expected) == set(state_dict.keys()),
                              "pytorch_model.bin does not hold the keys listed in load_keys.json")
        for name, tensor in state_dict.items():
            _assign(model, name, tensor)
        left = [n for n, p in model.named_parameters() if p.device.type == "meta"]
        invalidInputError(not left, f"parameters missing from the saved low-bit model: {left[:5]}")
        if torch_dtype != "auto":
            from ipex_llm.transformers.convert import convert_bigdl_other_module
            convert_bigdl_other_module(model, torch_dtype)
        model.eval()
        model.save_low_bit = types.MethodType(save_low_bit, model)
        return model


def _hf(name):
    import transformers
    return getattr(transformers, name)


class AutoModelForCausalLM(_BaseAutoModelClass):
    pass


class AutoModel(_BaseAutoModelClass):
    pass


class AutoModelForSeq2SeqLM(_BaseAutoModelClass):
    pass


class AutoModelForSequenceClassification(_BaseAutoModelClass):
    pass


def _bind():
    for cls in (AutoModelForCausalLM, AutoModel, AutoModelForSeq2SeqLM, AutoModelForSequenceClassification):
        try:
            cls.HF_Model = _hf(cls.__name__)
        except Exception:  # noqa: BLE001
            cls.HF_Model = None


_bind()
