"""optimize_model / save_low_bit / load_low_bit for plain PyTorch models
(reference: python/llm/src/ipex_llm/optimize.py:37-57, 137-267)."""
import json
import os
import types
import warnings
from contextlib import contextmanager

import torch

from ipex_llm.ggml.quantize import ggml_tensor_qtype
from ipex_llm.utils.common import invalidInputError

PYTORCH_MODEL_NAME = "pytorch_model.bin"
CONFIG_NAME = "bigdl_config.json"


def _save_low_bit(self, save_dir, *args, **kwargs):
    invalidInputError(self._bigdl_config.get("bigdl_transformers_low_bit", False),
                      "Detected this model is not a low-bit model, please use from_pretrained's"
                      " load_in_4bit or load_in_low_bit parameter to load a 4-bit model first.")
    os.makedirs(save_dir, exist_ok=True)
    # blobs are written in the ggml layout: GPU-resident weights go back through .to("cpu")
    state = {k: v.detach().to("cpu") for k, v in _cpu_state(self).items()}
    torch.save(state, os.path.join(save_dir, PYTORCH_MODEL_NAME))
    with open(os.path.join(save_dir, CONFIG_NAME), "w") as json_file:
        json.dump(self._bigdl_config, json_file)


def _cpu_state(model):
    from ipex_llm.transformers.low_bit_linear import FP4Params
    out = {}
    for name, p in list(model.named_parameters()) + list(model.named_buffers()):
        if isinstance(p, FP4Params):
            out[name] = p.to("cpu").data
        else:
            out[name] = p.data
    return out


def low_bit_sanity_check(model_path):
    invalidInputError(os.path.isdir(model_path), "model_path should be a valid directory path.")
    invalidInputError(os.path.isfile(os.path.join(model_path, CONFIG_NAME)),
                      "bigdl_config.json should be under your model directory, "
                      "please check your input path.")
    with open(os.path.join(model_path, CONFIG_NAME), 'r') as f:
        _config = json.load(f)
    low_bit = _config.get("bigdl_transformers_low_bit", None)
    if low_bit is None:
        warnings.warn("bigdl_transformers_low_bit not found in bigdl_config.json, "
                      "model is regarded as a normal pytorch model.")
    return low_bit


@contextmanager
def low_memory_init():
    """Builds a model on the meta device (no storage); load_low_bit fills it afterwards."""
    with torch.device("meta"):
        yield


def _assign(model, name, tensor):
    from ipex_llm.transformers.low_bit_linear import FP4Params
    mod = model
    *path, leaf = name.split(".")
    for p in path:
        mod = getattr(mod, p)
    if leaf in mod._parameters:
        old = mod._parameters[leaf]
        if isinstance(old, FP4Params):
            shape = old._shape
            if shape is None and hasattr(mod, "num_embeddings"):      # LowBitEmbedding skeleton
                shape = torch.Size((mod.num_embeddings, mod.embedding_dim))
            mod._parameters[leaf] = FP4Params(tensor, requires_grad=False, quantized=True,
                                              _shape=shape, qtype=old.qtype)
        else:
            mod._parameters[leaf] = torch.nn.Parameter(tensor, requires_grad=False)
    elif leaf in mod._buffers:
        mod._buffers[leaf] = tensor
    else:
        invalidInputError(False, f"unexpected key {name} in the saved low-bit model")


def unconverted_linears(state_dict):
    """Module names whose saved weight is still a dense matrix: they were excluded from the
    conversion when the model was saved and must be excluded again when it is rebuilt."""
    return [k[:-len(".weight")] for k, v in state_dict.items()
            if k.endswith(".weight") and v.dim() == 2 and v.numel() > 0 and v.dtype != torch.uint8]


def load_low_bit(model, model_path):
    """Turns `model` (on cpu or meta) into the low-bit model saved under model_path."""
    low_bit = low_bit_sanity_check(model_path)
    invalidInputError(isinstance(model, torch.nn.Module),
                      f"model should be a instance of `torch.nn.Module`, but got {type(model)} at last.")
    # the file holds tensors only: the safe loader is enough
    state_dict = torch.load(os.path.join(model_path, PYTORCH_MODEL_NAME), weights_only=True)
    if low_bit:
        from ipex_llm.transformers.convert import ggml_convert_low_bit
        qtype = ggml_tensor_qtype[low_bit]
        model = ggml_convert_low_bit(model, qtype=qtype, convert_shape_only=True,
                                     modules_to_not_convert=unconverted_linears(state_dict))
    for param_name, param in state_dict.items():
        _assign(model, param_name, param)
    if low_bit:
        model._bigdl_config = {"bigdl_transformers_low_bit": low_bit}
        model.save_low_bit = types.MethodType(_save_low_bit, model)
    return model


def optimize_model(model, low_bit='sym_int4', optimize_llm=True, modules_to_not_convert=None,
                   cpu_embedding=False, **kwargs):
    """Replaces every nn.Linear of a PyTorch model by its low-bit counterpart
    (reference: optimize.py:199-267; same arguments)."""
    invalidInputError(low_bit is None or low_bit in ggml_tensor_qtype,
                      f"Unknown load_in_low_bit value: {low_bit}, expected:"
                      f" sym_int4, asym_int4, sym_int5, asym_int5 or sym_int8.")
    invalidInputError(isinstance(model, torch.nn.Module),
                      f"model should be an instance of `torch.nn.Module`, but got {type(model)} at last.")
    if hasattr(model, 'device'):
        invalidInputError(model.device.type in ('cpu', 'meta'),
                          f"Expect model on device `cpu` or `meta`, but got device type {model.device.type}")
    if kwargs.pop("replace_embedding", False):
        warnings.warn("replace_embedding is deprecated, please use cpu_embedding instead.", FutureWarning)
        cpu_embedding = True
    if low_bit == "fp16":
        torch_dtype = kwargs.get("torch_dtype", None)
        invalidInputError(torch_dtype is None or torch_dtype == torch.float16,
                          "Please use torch_dtype=torch.float16 when setting low_bit='fp16'.")
        torch_dtype = torch.float16
    else:
        torch_dtype = kwargs.get("torch_dtype", "auto")
    from ipex_llm.transformers.convert import ggml_convert_low_bit
    qtype = ggml_tensor_qtype[low_bit] if low_bit is not None else None
    model = ggml_convert_low_bit(model, qtype=qtype, torch_dtype=torch_dtype,
                                 optimize_model=optimize_llm,
                                 modules_to_not_convert=modules_to_not_convert,
                                 cpu_embedding=cpu_embedding,
                                 disable_optimize_pre=kwargs.pop("disable_optimize_pre", False))
    model._bigdl_config = dict()
    model._bigdl_config["bigdl_transformers_low_bit"] = low_bit
    model.save_low_bit = types.MethodType(_save_low_bit, model)
    return model
