"""ctypes binding of liblowbit_hip.so.

Takes the place of the reference module of the same name
(python/llm/src/ipex_llm/ggml/model/llama/llama_cpp.py:71-109 for the loader,
:945-1185 for the ggml_* prototypes).  The ggml_* functions keep their
signatures; the lowbit_* functions are the device-pointer entry points that
stand where the reference calls the xe_linear / xe_batch torch ops.

There is no CPU implementation behind this module: if the HIP library cannot
be loaded, importing it raises RuntimeError, exactly as the reference does when
libllama-api.so is missing.
"""
import ctypes
import os
import pathlib

from ipex_llm.utils.common import invalidInputError
from ipex_llm.utils.utils import get_shared_lib_info

LAYOUT_GGML = 0
LAYOUT_TILED = 1
DT_F16, DT_BF16, DT_F32 = 0, 1, 2


def _load_shared_library(lib_base_name: str):
    _base_path, _lib_paths = get_shared_lib_info(lib_base_name=lib_base_name)
    if "LLAMA_CPP_LIB" in os.environ:
        _lib = pathlib.Path(os.environ["LLAMA_CPP_LIB"])
        _lib_paths = [_lib.resolve()]
    for _lib_path in _lib_paths:
        if _lib_path.exists():
            try:
                return ctypes.CDLL(str(_lib_path))
            except Exception as e:  # noqa: BLE001
                invalidInputError(False, f"Failed to load shared library '{_lib_path}': {e}.")
    invalidInputError(False,
                      f"Shared library with base name '{lib_base_name}' not found "
                      f"(looked for {[str(p) for p in _lib_paths]}); build it with "
                      "`make -C ipex-llm_amd/csrc`. There is no CPU fallback.")


_lib_base_name = "lowbit_hip"
_lib = _load_shared_library(_lib_base_name)

c_void_p, c_int, c_int64, c_size_t = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_size_t

_lib.lowbit_abi_version.argtypes = []
_lib.lowbit_abi_version.restype = c_int
_lib.lowbit_last_error.argtypes = []
_lib.lowbit_last_error.restype = ctypes.c_char_p


_lib.lowbit_device_info.argtypes = [ctypes.c_char_p, c_size_t, ctypes.POINTER(c_int), ctypes.POINTER(c_int),
                                    ctypes.POINTER(c_int), ctypes.POINTER(c_int)]
_lib.lowbit_device_info.restype = c_int


def lowbit_device_info() -> dict:
    """Name, CU count, maximum clocks and bus width of the current device as the HIP runtime reports them."""
    name = ctypes.create_string_buffer(256)
    cus, sclk, mclk, bus = c_int(), c_int(), c_int(), c_int()
    _check(_lib.lowbit_device_info(name, 256, ctypes.byref(cus), ctypes.byref(sclk), ctypes.byref(mclk),
                                   ctypes.byref(bus)), "lowbit_device_info")
    return {"name": name.value.decode("utf-8", "replace"), "compute_units": cus.value,
            "max_shader_clock_mhz": sclk.value / 1e3, "max_memory_clock_mhz": mclk.value / 1e3,
            "memory_bus_bits": bus.value}


def last_error() -> str:
    return (_lib.lowbit_last_error() or b"").decode("utf-8", "replace")


def _check(rc: int, what: str):
    invalidInputError(rc == 0, f"{what} failed ({rc}): {last_error()}")


def _check_void(what: str):
    msg = last_error()
    invalidInputError(msg == "", f"{what} failed: {msg}")


# ------------------------------------------------------------------ ggml_* (host pointers)

_lib.ggml_quantize_tensor.argtypes = [ctypes.POINTER(ctypes.c_float), c_void_p, c_int, c_size_t, c_int,
                                      ctypes.POINTER(c_int64), ctypes.c_bool]
_lib.ggml_quantize_tensor.restype = c_size_t


def ggml_quantize_tensor(src, dst, qtype, n, k, hist, scale_search) -> int:
    written = _lib.ggml_quantize_tensor(src, dst, qtype, n, k, hist, scale_search)
    if n:
        _check_void("ggml_quantize_tensor")
    return written


def _unsupported(name):
    def f(*args, **kwargs):
        invalidInputError(False, f"{name} is not provided by the MI355X low-bit library "
                                 "(k-quant / NPU round-to-nearest quantizers are outside its scope).")
    f.__name__ = name
    return f


ggml_quantize_tensor_with_weights = _unsupported("ggml_quantize_tensor_with_weights")
ggml_quantize_tensor_rtn = _unsupported("ggml_quantize_tensor_rtn")
ggml_quantize_tensor_rtn_with_weights = _unsupported("ggml_quantize_tensor_rtn_with_weights")

_lib.ggml_type_size.argtypes = [c_int]
_lib.ggml_type_size.restype = c_size_t
_lib.ggml_qk_size.argtypes = [c_int]
_lib.ggml_qk_size.restype = c_int


def ggml_type_size(qtype) -> int:
    return _lib.ggml_type_size(qtype)


def ggml_qk_size(qtype) -> int:
    return _lib.ggml_qk_size(qtype)


_lib.ggml_dequantize_q4_0.argtypes = [c_void_p, c_void_p, c_size_t]
_lib.ggml_dequantize_q4_0.restype = None
_lib.ggml_dequantize.argtypes = [c_void_p, c_void_p, c_size_t, c_int]
_lib.ggml_dequantize.restype = None


def ggml_dequantize_q4_0(src, dst, k):
    _lib.ggml_dequantize_q4_0(src, dst, k)
    _check_void("ggml_dequantize_q4_0")


def ggml_dequantize(src, dst, k, qtype):
    _lib.ggml_dequantize(src, dst, k, qtype)
    _check_void("ggml_dequantize")


_lib.ggml_q_format_convet_cpu2xpu.argtypes = [c_void_p, c_void_p, c_size_t, c_int]
_lib.ggml_q_format_convet_cpu2xpu.restype = None
_lib.ggml_q_format_convet_xpu2cpu.argtypes = [c_void_p, c_void_p, c_size_t, c_int]
_lib.ggml_q_format_convet_xpu2cpu.restype = None


def ggml_q_format_convet_cpu2xpu(src, dst, n, qtype):
    _lib.ggml_q_format_convet_cpu2xpu(src, dst, n, qtype)
    _check_void("ggml_q_format_convet_cpu2xpu")


def ggml_q_format_convet_xpu2cpu(src, dst, n, qtype):
    _lib.ggml_q_format_convet_xpu2cpu(src, dst, n, qtype)
    _check_void("ggml_q_format_convet_xpu2cpu")


_lib.ggml_compute_forward_mul_mat_q_fp32.argtypes = [ctypes.POINTER(c_int64), c_void_p, c_int,
                                                     ctypes.POINTER(c_int64), c_void_p, c_void_p]
_lib.ggml_compute_forward_mul_mat_q_fp32.restype = None


def ggml_compute_forward_mul_mat_q_fp32(src_0_ne, src_0_data, src_0_qtype, src_1_ne, src_1_data, result):
    _lib.ggml_compute_forward_mul_mat_q_fp32(src_0_ne, src_0_data, src_0_qtype, src_1_ne, src_1_data, result)
    _check_void("ggml_compute_forward_mul_mat_q_fp32")


_lib.llama_init_backend.argtypes = []
_lib.llama_init_backend.restype = None


def llama_init_backend():
    _lib.llama_init_backend()


# ---------------------------------------------------------------- lowbit_* (device pointers)

_lib.lowbit_blob_bytes.argtypes = [c_int, c_int64]
_lib.lowbit_blob_bytes.restype = c_size_t
_lib.lowbit_tileable.argtypes = [c_int, c_int64, c_int64]
_lib.lowbit_tileable.restype = c_int
_lib.lowbit_quantize.argtypes = [c_void_p, c_void_p, c_int, c_int64, c_int64, c_int, c_void_p]
_lib.lowbit_quantize.restype = c_int
_lib.lowbit_relayout.argtypes = [c_void_p, c_void_p, c_int, c_int64, c_int64, c_int, c_void_p]
_lib.lowbit_relayout.restype = c_int
_lib.lowbit_dequantize.argtypes = [c_void_p, c_void_p, c_int, c_int64, c_int64, c_int, c_int, c_void_p]
_lib.lowbit_dequantize.restype = c_int
_lib.lowbit_forward.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int64, c_int64, c_int64,
                                c_void_p]
_lib.lowbit_forward.restype = c_int
_lib.lowbit_gemv.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int64, c_int64, c_int64,
                             c_int, c_void_p]
_lib.lowbit_gemv.restype = c_int
_lib.lowbit_gemm.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int64, c_int64, c_int64,
                             c_void_p]
_lib.lowbit_gemm.restype = c_int


_lib.lowbit_workspace_bytes.argtypes = [c_int64, c_int64, c_int64]
_lib.lowbit_workspace_bytes.restype = c_size_t
_lib.lowbit_forward_ws.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int64, c_int64, c_int64,
                                   c_void_p, c_size_t, c_void_p]
_lib.lowbit_forward_ws.restype = c_int
_lib.lowbit_gemm_ws.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int64, c_int64, c_int64,
                                c_void_p, c_size_t, c_int, c_void_p]
_lib.lowbit_gemm_ws.restype = c_int
_lib.lowbit_gemm_ring.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int64, c_int64, c_int64,
                                  c_void_p, c_size_t, c_int, c_void_p]
_lib.lowbit_gemm_ring.restype = c_int


_lib.lowbit_gemm_narrow.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int64, c_int64, c_int64, c_void_p]
_lib.lowbit_gemm_narrow.restype = c_int


_lib.lowbit_forward_plan.argtypes = [c_int, c_int, c_int64, c_int64, c_int64, c_int, c_size_t]
_lib.lowbit_forward_plan.restype = c_int
PLAN_GEMV, PLAN_RING, PLAN_GEMM, PLAN_GEMM_SPLIT, PLAN_GEMM_NARROW = 0, 1, 2, 3, 4


_lib.lowbit_workspace_bytes_for.argtypes = [c_int, c_int, c_int64, c_int64, c_int64, c_size_t]
_lib.lowbit_workspace_bytes_for.restype = c_size_t


def lowbit_workspace_bytes_for(qtype, layout, m, n, k, max_bytes) -> int:
    """Bytes of workspace lowbit_forward_ws uses for this format when it may have at most max_bytes."""
    return int(_lib.lowbit_workspace_bytes_for(qtype, layout, m, n, k, max_bytes))


def lowbit_forward_plan(qtype, layout, m, n, k, have_workspace, workspace_bytes=0) -> int:
    """PLAN_* code of the kernel lowbit_forward (have_workspace False) / lowbit_forward_ws would run."""
    return _lib.lowbit_forward_plan(qtype, layout, m, n, k, int(bool(have_workspace)), workspace_bytes)


def lowbit_workspace_bytes(m, n, k) -> int:
    return _lib.lowbit_workspace_bytes(m, n, k)


def lowbit_forward_ws(x, w, y, qtype, layout, act_dtype, m, n, k, workspace, workspace_bytes, stream):
    _check(_lib.lowbit_forward_ws(x, w, y, qtype, layout, act_dtype, m, n, k, workspace, workspace_bytes, stream),
           "lowbit_forward_ws")


def lowbit_gemm_ws(x, w, y, qtype, layout, act_dtype, m, n, k, workspace, workspace_bytes, splits, stream):
    _check(_lib.lowbit_gemm_ws(x, w, y, qtype, layout, act_dtype, m, n, k, workspace, workspace_bytes, splits, stream),
           "lowbit_gemm_ws")


def lowbit_gemm_ring(x, w, y, qtype, layout, act_dtype, m, n, k, workspace, workspace_bytes, wgs, stream):
    _check(_lib.lowbit_gemm_ring(x, w, y, qtype, layout, act_dtype, m, n, k, workspace, workspace_bytes, wgs,
                                 stream), "lowbit_gemm_ring")


def lowbit_gemm_narrow(x, w, y, qtype, layout, act_dtype, m, n, k, stream):
    _check(_lib.lowbit_gemm_narrow(x, w, y, qtype, layout, act_dtype, m, n, k, stream), "lowbit_gemm_narrow")


_lib.lowbit_forward_f32_workspace_bytes.argtypes = [c_int64, c_int64, c_int64]
_lib.lowbit_forward_f32_workspace_bytes.restype = c_size_t
_lib.lowbit_forward_f32.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int64, c_int64, c_int64, c_void_p,
                                    c_size_t, c_void_p]
_lib.lowbit_forward_f32.restype = c_int


def lowbit_forward_f32_workspace_bytes(m, n, k) -> int:
    return _lib.lowbit_forward_f32_workspace_bytes(m, n, k)


def lowbit_forward_f32(x, w, y, qtype, layout, m, n, k, workspace, workspace_bytes, stream):
    _check(_lib.lowbit_forward_f32(x, w, y, qtype, layout, m, n, k, workspace, workspace_bytes, stream),
           "lowbit_forward_f32")


_lib.lowbit_noalloc_scratch_bytes.argtypes = []
_lib.lowbit_noalloc_scratch_bytes.restype = c_size_t
_lib.lowbit_forward_noalloc.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int64, c_int64, c_int64,
                                        c_void_p]
_lib.lowbit_forward_noalloc.restype = c_int


def lowbit_noalloc_scratch_bytes() -> int:
    return _lib.lowbit_noalloc_scratch_bytes()


def lowbit_forward_noalloc(x, w, y, qtype, layout, act_dtype, m, n, k, stream):
    _check(_lib.lowbit_forward_noalloc(x, w, y, qtype, layout, act_dtype, m, n, k, stream), "lowbit_forward_noalloc")


_lib.lowbit_grouped_forward.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int, c_int,
                                        c_int64, c_int64, c_void_p]
_lib.lowbit_grouped_forward.restype = c_int


def lowbit_grouped_forward(x, w_ptrs, y, group_offsets, n_groups, total_rows, qtype, act_dtype, n, k, stream):
    _check(_lib.lowbit_grouped_forward(x, w_ptrs, y, group_offsets, n_groups, total_rows, qtype, act_dtype,
                                       n, k, stream), "lowbit_grouped_forward")


_lib.lowbit_grouped_workspace_bytes.argtypes = [c_int, c_int64, c_int64, c_int64]
_lib.lowbit_grouped_workspace_bytes.restype = c_size_t
_lib.lowbit_grouped_forward_ws.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int, c_int,
                                           c_int64, c_int64, c_void_p, c_size_t, c_void_p]
_lib.lowbit_grouped_forward_ws.restype = c_int
_lib.lowbit_grouped_mlp_forward.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int,
                                            c_int, c_int64, c_int64, c_int, c_void_p]
_lib.lowbit_grouped_mlp_forward.restype = c_int


def lowbit_grouped_workspace_bytes(n_groups, total_rows, n, k):
    return int(_lib.lowbit_grouped_workspace_bytes(n_groups, total_rows, n, k))


_lib.lowbit_grouped_forward_plan.argtypes = [c_int, c_int64, c_int64, c_int64, c_int, c_size_t, ctypes.POINTER(c_int)]
_lib.lowbit_grouped_forward_plan.restype = c_int


def lowbit_grouped_forward_plan(n_groups, total_rows, n, k, have_workspace, workspace_bytes=0):
    """(tall, splits, waves, workgroups per split) of a plain grouped product; host arithmetic only."""
    out = (c_int * 4)()
    _check(_lib.lowbit_grouped_forward_plan(n_groups, total_rows, n, k, int(bool(have_workspace)), workspace_bytes, out),
           "lowbit_grouped_forward_plan")
    return tuple(out)


def lowbit_grouped_forward_ws(x, w_ptrs, y, group_offsets, n_groups, total_rows, qtype, act_dtype, n, k, workspace,
                              workspace_bytes, stream):
    _check(_lib.lowbit_grouped_forward_ws(x, w_ptrs, y, group_offsets, n_groups, total_rows, qtype, act_dtype,
                                          n, k, workspace, workspace_bytes, stream), "lowbit_grouped_forward_ws")


def lowbit_grouped_mlp_forward(x, gate_ptrs, up_ptrs, y, group_offsets, n_groups, total_rows, qtype, act_dtype, n, k,
                               act, stream):
    _check(_lib.lowbit_grouped_mlp_forward(x, gate_ptrs, up_ptrs, y, group_offsets, n_groups, total_rows, qtype,
                                           act_dtype, n, k, act, stream), "lowbit_grouped_mlp_forward")


_lib.lowbit_dequantize_rows.argtypes = [c_void_p, c_void_p, c_int64, c_void_p, c_int, c_int64, c_int64, c_int, c_int,
                                        c_void_p]
_lib.lowbit_dequantize_rows.restype = c_int
_lib.lowbit_mlp_forward.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int64, c_int64, c_int64,
                                    c_int, c_void_p]
_lib.lowbit_mlp_forward.restype = c_int


_lib.lowbit_moe_forward.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                                    c_void_p, c_int, c_int, c_int64, c_int64, c_int, c_void_p]
_lib.lowbit_moe_forward.restype = c_int


def lowbit_moe_forward(x, topk_ids, topk_weight, top_k, n_experts, gates, ups, downs, workspace, y, qtype, act_dtype,
                       hidden, inter, act, stream):
    _check(_lib.lowbit_moe_forward(x, topk_ids, topk_weight, top_k, n_experts, gates, ups, downs, workspace, y, qtype,
                                   act_dtype, hidden, inter, act, stream), "lowbit_moe_forward")


def lowbit_dequantize_rows(w, rows, n_rows, dst, qtype, n, k, layout, out_dtype, stream):
    _check(_lib.lowbit_dequantize_rows(w, rows, n_rows, dst, qtype, n, k, layout, out_dtype, stream),
           "lowbit_dequantize_rows")


def lowbit_mlp_forward(x, w_gate, w_up, y, qtype, act_dtype, m, n, k, act, stream):
    _check(_lib.lowbit_mlp_forward(x, w_gate, w_up, y, qtype, act_dtype, m, n, k, act, stream), "lowbit_mlp_forward")


def lowbit_blob_bytes(qtype, n_weights) -> int:
    return _lib.lowbit_blob_bytes(qtype, n_weights)


def lowbit_tileable(qtype, n, k) -> bool:
    return bool(_lib.lowbit_tileable(qtype, n, k))


def lowbit_quantize(src, dst, qtype, n, k, layout, stream):
    _check(_lib.lowbit_quantize(src, dst, qtype, n, k, layout, stream), "lowbit_quantize")


def lowbit_relayout(src, dst, qtype, n, k, src_layout, stream):
    _check(_lib.lowbit_relayout(src, dst, qtype, n, k, src_layout, stream), "lowbit_relayout")


def lowbit_dequantize(w, dst, qtype, n, k, layout, out_dtype, stream):
    _check(_lib.lowbit_dequantize(w, dst, qtype, n, k, layout, out_dtype, stream), "lowbit_dequantize")


def lowbit_forward(x, w, y, qtype, layout, act_dtype, m, n, k, stream):
    _check(_lib.lowbit_forward(x, w, y, qtype, layout, act_dtype, m, n, k, stream), "lowbit_forward")


def lowbit_gemv(x, w, y, qtype, layout, act_dtype, m, n, k, waves, stream):
    _check(_lib.lowbit_gemv(x, w, y, qtype, layout, act_dtype, m, n, k, waves, stream), "lowbit_gemv")


def lowbit_gemm(x, w, y, qtype, layout, act_dtype, m, n, k, stream):
    _check(_lib.lowbit_gemm(x, w, y, qtype, layout, act_dtype, m, n, k, stream), "lowbit_gemm")


llama_init_backend()
