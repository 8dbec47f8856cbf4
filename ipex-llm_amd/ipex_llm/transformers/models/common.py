"""Fused gated-MLP forward (reference: transformers/models/common.py:145-170)."""
import torch

import ipex_llm.ggml.model.llama.llama_cpp as ggml


def fuse_mlp_base(module: torch.nn.Module, act: int, x: torch.Tensor):
    from ipex_llm.transformers.low_bit_linear import LowBitLinear, mlp_forward_xpu
    from ipex_llm.transformers.models.utils import mlp_fusion_check
    gate, up = module.gate_proj, module.up_proj
    qtype = getattr(gate, "qtype", None)
    fusable = (isinstance(gate, LowBitLinear) and isinstance(up, LowBitLinear)
               and gate.bias is None and up.bias is None
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
    return module.down_proj(module.act_fn(module.gate_proj(x)) * module.up_proj(x))


def mlp_silu_forward(self, x: torch.Tensor):
    from ipex_llm.transformers.models.utils import SILU
    return fuse_mlp_base(self, SILU, x)


def mlp_gelu_forward(self, x: torch.Tensor):
    from ipex_llm.transformers.models.utils import GELU
    return fuse_mlp_base(self, GELU, x)
