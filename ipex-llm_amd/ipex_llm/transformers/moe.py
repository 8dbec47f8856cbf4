"""Mixture-of-experts feed-forward on low-bit experts.

The reference has no fused path for a Mixtral-style block at prefill: the Hugging Face block
loops over the experts and calls each expert's (converted) LowBitLinear on the rows routed to
it, then index_adds the weighted result (the same pattern as the reference's own
transformers/models/qwen2_moe.py:375-430).  `moe_ffn_reference` is that loop;
`moe_ffn_grouped` computes the same thing with two grouped launches over the rows sorted by expert:
the fused gate/up projection with the activation in its epilogue, then the down projection.
"""
import ctypes

import torch
import torch.nn as nn
import torch.nn.functional as F

import ipex_llm.ggml.model.llama.llama_cpp as ggml
from ipex_llm.transformers.low_bit_linear import _DT, _as_u8, _stream
from ipex_llm.utils.common import invalidInputError


def route_top_k(router_logits: torch.Tensor, top_k: int = 2):
    """softmax over experts in fp32, top-k, renormalised (Hugging Face Mixtral semantics)."""
    probs = F.softmax(router_logits.float(), dim=-1)
    weights, experts = torch.topk(probs, top_k, dim=-1)
    weights = weights / weights.sum(dim=-1, keepdim=True)
    return weights, experts


class ExpertWeights:
    """Device pointers of one projection of every expert ([N, K] tiled blobs of one qtype)."""

    def __init__(self, linears):
        invalidInputError(len(linears) > 0, "no experts")
        l0 = linears[0]
        self.qtype, self.out_len, self.in_len = l0.qtype, l0.out_len, l0.in_len
        for lin in linears:
            invalidInputError(lin.weight.device.type == "cuda" and lin.weight.quantized
                              and (lin.qtype, lin.out_len, lin.in_len) == (self.qtype, self.out_len, self.in_len),
                              "experts must be quantized, on the GPU and of one shape / qtype")
        invalidInputError(ggml.lowbit_tileable(self.qtype, self.out_len, self.in_len),
                          "grouped experts need out_features % 16 == 0 and in_features % 128 == 0")
        want = ggml.lowbit_blob_bytes(self.qtype, self.out_len * self.in_len)
        for lin in linears:
            invalidInputError(lin.weight.data.device == l0.weight.data.device
                              and lin.weight.blob_layout == ggml.LAYOUT_TILED
                              and _as_u8(lin.weight.data).numel() == want and lin.weight.data.is_contiguous(),
                              "every expert must hold a tiled blob of the common shape on one GPU")
        self.linears = list(linears)
        self.blobs = [_as_u8(lin.weight.data) for lin in linears]        # keeps the storage alive
        self.ptrs = torch.tensor([b.data_ptr() for b in self.blobs], dtype=torch.int64, device=l0.weight.device)

    def check(self, device):
        """The pointer table is a snapshot: refuse to launch if a layer was moved or re-quantized since."""
        for lin, blob in zip(self.linears, self.blobs):
            invalidInputError(lin.weight.data.data_ptr() == blob.data_ptr() and blob.device == device,
                              "an expert weight was moved or replaced after ExpertWeights was built; build it again")


def _check_grouped(x_sorted, group_offsets, experts):
    invalidInputError(x_sorted.dim() == 2 and x_sorted.shape[1] == experts.in_len and x_sorted.dtype in _DT
                      and x_sorted.dtype != torch.float32, "x must be [rows, K] in fp16 / bf16")
    invalidInputError(group_offsets.dtype == torch.int32 and group_offsets.numel() == len(experts.blobs) + 1
                      and group_offsets.device == x_sorted.device, "group_offsets must be int32 [E + 1] on the GPU")
    experts.check(x_sorted.device)


def grouped_forward(x_sorted: torch.Tensor, group_offsets: torch.Tensor, experts: ExpertWeights):
    """y[r] = x_sorted[r] @ dequant(W[e])^T for group_offsets[e] <= r < group_offsets[e+1]."""
    _check_grouped(x_sorted, group_offsets, experts)
    x_sorted = x_sorted.contiguous()
    rows = x_sorted.shape[0]
    y = torch.empty((rows, experts.out_len), dtype=x_sorted.dtype, device=x_sorted.device)
    if rows:
        n_exp = len(experts.blobs)
        ws_bytes = ggml.lowbit_grouped_workspace_bytes(n_exp, rows, experts.out_len, experts.in_len)
        ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=x_sorted.device)
        with torch.cuda.device(x_sorted.device):
            ggml.lowbit_grouped_forward_ws(x_sorted.data_ptr(), experts.ptrs.data_ptr(), y.data_ptr(),
                                           group_offsets.data_ptr(), n_exp, rows, experts.qtype, _DT[x_sorted.dtype],
                                           experts.out_len, experts.in_len, ws.data_ptr(), ws_bytes, _stream())
    return y


def grouped_mlp_forward(x_sorted: torch.Tensor, group_offsets: torch.Tensor, gates: ExpertWeights,
                        ups: ExpertWeights, act: int = 0):
    """h[r] = act(x_sorted[r] @ Wg[e]^T) * (x_sorted[r] @ Wu[e]^T) for the rows of group e, in one launch
    (act: 0 = SiLU, 1 = tanh-GELU, as in mlp_forward_xpu)."""
    _check_grouped(x_sorted, group_offsets, gates)
    invalidInputError((ups.qtype, ups.out_len, ups.in_len) == (gates.qtype, gates.out_len, gates.in_len)
                      and len(ups.blobs) == len(gates.blobs), "gate and up experts do not fit together")
    ups.check(x_sorted.device)
    x_sorted = x_sorted.contiguous()
    rows = x_sorted.shape[0]
    h = torch.empty((rows, gates.out_len), dtype=x_sorted.dtype, device=x_sorted.device)
    if rows:
        with torch.cuda.device(x_sorted.device):
            ggml.lowbit_grouped_mlp_forward(x_sorted.data_ptr(), gates.ptrs.data_ptr(), ups.ptrs.data_ptr(),
                                            h.data_ptr(), group_offsets.data_ptr(), len(gates.blobs), rows,
                                            gates.qtype, _DT[x_sorted.dtype], gates.out_len, gates.in_len, act,
                                            _stream())
    return h


def moe_forward_vec(x: torch.Tensor, topk_ids: torch.Tensor, topk_weight: torch.Tensor, gates: ExpertWeights,
                    ups: ExpertWeights, downs: ExpertWeights, act: int = 0):
    """xe_linear.moe_forward_vec (models/deepseek.py:290-315 of the reference): one token through its top-k
    experts in two launches.  Nothing is read back to the host: the expert ids stay on the GPU.
    x [1, hidden]; topk_ids / topk_weight [1, top_k]; returns [1, hidden]."""
    hidden, inter = gates.in_len, gates.out_len
    invalidInputError(x.dim() == 2 and x.shape == (1, hidden) and x.dtype in (torch.float16, torch.bfloat16),
                      "moe_forward_vec expects one fp16 / bf16 row of x")
    invalidInputError((ups.qtype, ups.out_len, ups.in_len) == (gates.qtype, inter, hidden)
                      and (downs.qtype, downs.out_len, downs.in_len) == (gates.qtype, hidden, inter),
                      "gate / up / down experts do not fit together")
    for table in (gates, ups, downs):
        table.check(x.device)
    top_k = topk_ids.numel()
    ids = topk_ids.reshape(-1).to(torch.int32)
    rw = topk_weight.reshape(-1).to(torch.float32)
    xc = x.contiguous()
    work = torch.empty((top_k, inter), dtype=x.dtype, device=x.device)
    y = torch.empty((1, hidden), dtype=x.dtype, device=x.device)
    with torch.cuda.device(x.device):
        ggml.lowbit_moe_forward(xc.data_ptr(), ids.data_ptr(), rw.data_ptr(), top_k, len(gates.blobs),
                                gates.ptrs.data_ptr(), ups.ptrs.data_ptr(), downs.ptrs.data_ptr(), work.data_ptr(),
                                y.data_ptr(), gates.qtype, _DT[x.dtype], hidden, inter, act, _stream())
    return y


def moe_ffn_reference(hidden, router_logits, w1, w3, w2, top_k=2):
    """The per-expert loop: w1/w3/w2 are lists of LowBitLinear (gate, up, down)."""
    weights, experts = route_top_k(router_logits, top_k)
    out = torch.zeros_like(hidden)
    for e in range(len(w1)):
        tok, slot = torch.where(experts == e)
        if tok.numel() == 0:
            continue
        xe = hidden[tok]
        he = F.silu(w1[e](xe)) * w3[e](xe)
        ye = w2[e](he) * weights[tok, slot].unsqueeze(-1).to(hidden.dtype)
        out.index_add_(0, tok, ye.to(hidden.dtype))
    return out


def moe_ffn_grouped(hidden, router_logits, g1: ExpertWeights, g3: ExpertWeights, g2: ExpertWeights, top_k=2):
    """Same result with two grouped launches over the (token, expert) pairs sorted by expert."""
    n_exp = len(g1.blobs)
    weights, experts = route_top_k(router_logits, top_k)
    flat_e = experts.reshape(-1)
    order = torch.argsort(flat_e, stable=True)
    tok = torch.div(order, top_k, rounding_mode="floor")
    counts = torch.bincount(flat_e, minlength=n_exp)
    offsets = torch.zeros(n_exp + 1, dtype=torch.int32, device=hidden.device)
    offsets[1:] = torch.cumsum(counts, 0).to(torch.int32)
    xs = hidden[tok]
    h = grouped_mlp_forward(xs, offsets, g1, g3)
    y = grouped_forward(h, offsets, g2) * weights.reshape(-1)[order].unsqueeze(-1).to(hidden.dtype)
    out = torch.zeros_like(hidden)
    out.index_add_(0, tok, y)
    return out


def activation_code(act_fn):
    """0 (SiLU) / 1 (tanh-GELU) for the activations the fused kernels know, None for any other."""
    name = act_fn.__class__.__name__
    if isinstance(act_fn, nn.SiLU) or name in ("SiLUActivation", "SiLU"):
        return 0
    if (isinstance(act_fn, nn.GELU) and act_fn.approximate == "tanh") or name in ("PytorchGELUTanh", "GELUTanh",
                                                                               "NewGELUActivation"):
        return 1
    return None


class LowBitExperts(nn.Module):
    """The experts of a sparse mixture-of-experts block with low-bit weights.

    With the transformers version the reference pins (4.37) every expert is a small module of three nn.Linear
    layers, which its `_replace_with_low_bit_linear` turns into LowBitLinear one by one (convert.py:469-748) and
    the block's Python loop calls in turn.  Current transformers keep all experts of a block in one module with two
    3-D parameters, `gate_up_proj` [E, 2 I, H] and `down_proj` [E, H, I], and the call
    `experts(hidden_states [T, H], top_k_index [T, k], top_k_weights [T, k]) -> [T, H]` (MixtralExperts and its
    siblings).  This module takes that one's place: each expert's three weights become LowBitLinear layers
    (`gate[e]`, `up[e]`, `down[e]`, so that save_low_bit / load_low_bit carry them like any other), and on the GPU the
    call runs as two grouped launches over the (token, expert) pairs sorted by expert, or, for one token, as the two
    launches of `moe_forward_vec`.  Anywhere else it is the per-expert loop over the LowBitLinear layers."""

    def __init__(self, num_experts, hidden_dim, intermediate_dim, qtype, act_fn, enable_scale_search=False):
        super().__init__()
        from ipex_llm.transformers.low_bit_linear import LowBitLinear
        self.num_experts, self.hidden_dim, self.intermediate_dim, self.qtype = num_experts, hidden_dim, intermediate_dim, qtype
        self.act_fn = act_fn

        def layers(in_f, out_f):
            return nn.ModuleList([LowBitLinear(in_f, out_f, qtype, bias=False, enable_scale_search=enable_scale_search)
                                  for _ in range(num_experts)])
        self.gate, self.up = layers(hidden_dim, intermediate_dim), layers(hidden_dim, intermediate_dim)
        self.down = layers(intermediate_dim, hidden_dim)
        self.__dict__["_tables"] = None

    @classmethod
    def from_fused(cls, module, qtype, convert_shape_only=False, enable_scale_search=False):
        """From a module that holds `gate_up_proj` [E, 2 I, H], `down_proj` [E, H, I] and `act_fn`."""
        from ipex_llm.transformers.low_bit_linear import FP4Params
        gate_up, down = module.gate_up_proj.data, module.down_proj.data
        n_exp, two_i, hidden = gate_up.shape
        inter = two_i // 2
        invalidInputError(tuple(down.shape) == (n_exp, hidden, inter), "gate_up_proj / down_proj shapes do not fit together")
        new = cls(n_exp, hidden, inter, qtype, module.act_fn, enable_scale_search)
        device = gate_up.device

        def param(w, in_features):
            return FP4Params(data=w.contiguous() if w.device.type != "meta" else w, requires_grad=False, quantized=False,
                             _shape=None, convert_shape_only=convert_shape_only, qtype=qtype, in_features=in_features,
                             enable_scale_search=enable_scale_search).to(device)
        for e in range(n_exp):
            new.gate[e]._parameters["weight"] = param(gate_up[e, :inter], hidden)
            new.up[e]._parameters["weight"] = param(gate_up[e, inter:], hidden)
            new.down[e]._parameters["weight"] = param(down[e], inter)
        if not module.training:
            new.eval()
        new.requires_grad_(False)
        return new

    def _expert_tables(self, device):
        """Pointer tables of the three projections; built on first use and again when a weight has moved."""
        tables = self.__dict__["_tables"]
        if tables is not None:
            try:
                for t in tables:
                    t.check(device)
                return tables
            except RuntimeError:
                pass
        tables = tuple(ExpertWeights(list(layers)) for layers in (self.gate, self.up, self.down))
        self.__dict__["_tables"] = tables
        return tables

    def _grouped_ok(self, x):
        w = self.gate[0].weight
        return (x.device.type == "cuda" and x.dtype in (torch.float16, torch.bfloat16) and not self.training
                and activation_code(self.act_fn) is not None and w.quantized and w.data.device == x.device
                and ggml.lowbit_tileable(self.qtype, self.intermediate_dim, self.hidden_dim)
                and ggml.lowbit_tileable(self.qtype, self.hidden_dim, self.intermediate_dim))

    def forward(self, hidden_states, top_k_index, top_k_weights):
        tokens, top_k = top_k_index.shape
        if tokens == 0:
            return torch.zeros_like(hidden_states)
        if not self._grouped_ok(hidden_states):
            return self._loop(hidden_states, top_k_index, top_k_weights)
        act = activation_code(self.act_fn)
        g1, g3, g2 = self._expert_tables(hidden_states.device)
        if tokens == 1:
            return moe_forward_vec(hidden_states, top_k_index, top_k_weights, g1, g3, g2, act)
        flat_e = top_k_index.reshape(-1)
        order = torch.argsort(flat_e, stable=True)
        tok = torch.div(order, top_k, rounding_mode="floor")
        offsets = torch.zeros(self.num_experts + 1, dtype=torch.int32, device=hidden_states.device)
        offsets[1:] = torch.cumsum(torch.bincount(flat_e, minlength=self.num_experts)[:self.num_experts], 0).to(torch.int32)
        h = grouped_mlp_forward(hidden_states[tok], offsets, g1, g3, act)
        y = grouped_forward(h, offsets, g2) * top_k_weights.reshape(-1)[order].unsqueeze(-1).to(hidden_states.dtype)
        out = torch.zeros_like(hidden_states)
        out.index_add_(0, tok, y)
        return out

    def _loop(self, hidden_states, top_k_index, top_k_weights):
        out = torch.zeros_like(hidden_states)
        for e in range(self.num_experts):
            tok, slot = torch.where(top_k_index == e)
            if tok.numel() == 0:
                continue
            xe = hidden_states[tok]
            he = self.down[e](self.act_fn(self.gate[e](xe)) * self.up[e](xe))
            out.index_add_(0, tok, (he * top_k_weights[tok, slot, None]).to(out.dtype))
        return out
