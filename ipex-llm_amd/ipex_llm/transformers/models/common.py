"""q/k/v merge and fused gated-MLP forward (reference: transformers/models/common.py:22-52, 145-170)."""
import warnings
import weakref
from typing import List

import torch

import ipex_llm.ggml.model.llama.llama_cpp as ggml


def merge_linear(linears: List[torch.nn.Linear]) -> torch.nn.Linear:
    """One linear whose weight (and bias) is the row-wise concatenation of `linears`
    (reference: models/common.py:22-37).  GPTQ layers (no `weight`) give None."""
    if not all(isinstance(lin, torch.nn.Linear) and hasattr(lin, "weight") for lin in linears):
        return None
    new_weight = torch.cat([lin.weight.data for lin in linears], dim=0)
    has_bias = linears[0].bias is not None
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")                     # "Initializing zero-element tensors is a no-op"
        new_linear = torch.nn.Linear(0, 0, bias=has_bias)
    if has_bias:
        new_linear.bias = torch.nn.Parameter(torch.cat([lin.bias.data for lin in linears], dim=0), requires_grad=False)
    new_linear.weight = torch.nn.Parameter(new_weight, requires_grad=False)
    new_linear.in_features = new_weight.size(1)
    new_linear.out_features = new_weight.size(0)
    if not linears[0].training:
        new_linear.eval()
    return new_linear


class MergedProjectionSlice(torch.nn.Module):
    """Stands where q_proj / k_proj / v_proj stood after the merge and returns its rows of `qkv_proj(x)`.

    The reference deletes q_proj / k_proj / v_proj and rewrites every attention forward to call
    `self.qkv_proj` (models/common.py:40-52 and the per-model forwards).  Attention forwards are not part of
    the low-bit linear path, so here the stock Hugging Face forward keeps calling the three projections and
    the first call on a tensor runs the merged product, the other two read the rows they need from its result.
    A slice called on a tensor the merged product was not run on (cross-attention keys, say) computes only
    its own rows: the rows of a merged weight are contiguous in both layouts, so a zero-copy view of the blob
    is a valid weight.  The slice owns no parameters; the attention module is kept as a plain attribute, not as
    a registered sub-module, so that the module tree has no cycle through it."""

    def __init__(self, owner: torch.nn.Module, start: int, length: int, leader: bool, last: bool = False):
        super().__init__()
        self.__dict__["_owner"] = owner
        self.start, self.length, self.leader, self.last = start, length, leader, last
        self.out_features = length

    @property
    def in_features(self):
        return self._owner.qkv_proj.in_features

    @property
    def weight(self):
        """This slice's rows of a dense merged weight; the merged low-bit parameter itself otherwise (callers
        read `.dtype` / `.device` of it, as they would of a `LowBitLinear`'s packed weight)."""
        w = self._owner.qkv_proj.weight
        if getattr(w, "quantized", False) or w.dim() != 2 or w.size(0) < self.start + self.length:
            return w
        return w[self.start:self.start + self.length]

    @property
    def bias(self):
        b = self._owner.qkv_proj.bias
        return None if b is None else b[self.start:self.start + self.length]

    def forward(self, x: torch.Tensor):
        owner = self._owner
        cache = owner.__dict__.get("_qkv_cache")
        if cache is not None and cache[0]() is x and cache[1] == _version_of(x):
            y = cache[2]
            if self.last:
                owner.__dict__["_qkv_cache"] = None        # q, k and v have read it: nothing is kept alive
            return y[..., self.start:self.start + self.length]
        if not self.leader:
            if cache is not None:
                # the merged product was run on another tensor (cross-attention): from now on the leader
                # computes its own rows only
                owner.__dict__["_qkv_cache"] = None
                owner.__dict__["_qkv_apart"] = True
            return _project_rows(owner.qkv_proj, x, self.start, self.length)
        if owner.__dict__.get("_qkv_apart", False):
            return _project_rows(owner.qkv_proj, x, self.start, self.length)
        y = owner.qkv_proj(x)
        owner.__dict__["_qkv_cache"] = (weakref.ref(x), _version_of(x), y)
        return y[..., self.start:self.start + self.length]


def _version_of(x: torch.Tensor) -> int:
    """In-place edits bump `_version`; inference tensors do not count them (reading it raises)."""
    return 0 if x.is_inference() else x._version


def _project_rows(linear: torch.nn.Module, x: torch.Tensor, start: int, length: int):
    """x @ W[start : start + length]^T (+ bias) for a dense or a low-bit linear."""
    from ipex_llm.transformers.low_bit_linear import LowBitLinear, forward_new
    bias = None if linear.bias is None else linear.bias[start:start + length]
    if isinstance(linear, LowBitLinear) and linear.weight.data.device.type == "cuda" and start % 16 == 0 \
            and length % 16 == 0 and not linear.training:
        w = linear.weight
        blob = w.data.view(torch.uint8)
        row_bytes = blob.numel() // linear.out_len
        x_2d = x.contiguous().view(-1, x.shape[-1])
        y = forward_new(x_2d, blob[start * row_bytes:(start + length) * row_bytes], w.qtype, length,
                        layout=w.blob_layout)
        y = y.view(*x.shape[:-1], length)
        return y if bias is None else y + bias.to(y.dtype)
    if type(linear) is torch.nn.Linear:
        return torch.nn.functional.linear(x, linear.weight[start:start + length], bias)
    return linear(x)[..., start:start + length]


def merge_qkv_base(module: torch.nn.Module, attention_class):
    """Merges q_proj / k_proj / v_proj of every `attention_class` module into `qkv_proj`
    (reference: models/common.py:40-52)."""
    if (
        isinstance(attention_class, str) and module.__class__.__name__ == attention_class
        or not isinstance(attention_class, str) and isinstance(module, attention_class)
    ):
        projs = [getattr(module, n, None) for n in ("q_proj", "k_proj", "v_proj")]
        if any(p is None for p in projs):
            return
        if len({p.in_features for p in projs if hasattr(p, "in_features")}) != 1 or \
                len({p.bias is None for p in projs if hasattr(p, "bias")}) != 1:
            return
        qkv_proj = merge_linear(projs)
        if qkv_proj is not None:
            sizes = [p.out_features for p in projs]
            del module.q_proj, module.k_proj, module.v_proj
            module.qkv_proj = qkv_proj
            start = 0
            for i, (name, size) in enumerate(zip(("q_proj", "k_proj", "v_proj"), sizes)):
                setattr(module, name, MergedProjectionSlice(module, start, size, leader=(i == 0), last=(i == 2)))
                start += size


def fuse_mlp_base(module: torch.nn.Module, act: int, x: torch.Tensor):
    from ipex_llm.transformers.low_bit_linear import LowBitLinear, mlp_forward_xpu
    from ipex_llm.transformers.models.utils import mlp_fusion_check
    gate, up = module.gate_proj, module.up_proj
    qtype = getattr(gate, "qtype", None)
    fusable = (isinstance(gate, LowBitLinear) and isinstance(up, LowBitLinear)
               and gate.bias is None and up.bias is None
               and gate.weight.quantized and up.weight.quantized
               and gate.weight.data.device == x.device and up.weight.data.device == x.device
               and gate.weight.blob_layout == ggml.LAYOUT_TILED and up.weight.blob_layout == ggml.LAYOUT_TILED
               and gate.in_len == up.in_len == x.size(-1)
               and up.qtype == qtype and gate.out_len == up.out_len
               and x.dtype in (torch.float16, torch.bfloat16, torch.float32)
               and mlp_fusion_check(x, qtype, module.training)
               and ggml.lowbit_tileable(qtype, gate.out_len, x.size(-1)))
    if fusable:
        x_2d = x.contiguous().view(-1, x.size(-1))
        output = module.down_proj(
            mlp_forward_xpu(x_2d, gate.weight.data, up.weight.data, x_2d.size(0), x_2d.size(1), gate.out_len,
                            act, qtype))
        return output.view(*x.shape[:-1], output.size(-1))
    original = module.__dict__.get("_forward_before_fusion")
    if original is not None:
        return original(x)                    # whatever this class does besides the plain gated product
    return module.down_proj(module.act_fn(module.gate_proj(x)) * module.up_proj(x))


def mlp_silu_forward(self, x: torch.Tensor):
    from ipex_llm.transformers.models.utils import SILU
    return fuse_mlp_base(self, SILU, x)


def mlp_gelu_forward(self, x: torch.Tensor):
    from ipex_llm.transformers.models.utils import GELU
    return fuse_mlp_base(self, GELU, x)
