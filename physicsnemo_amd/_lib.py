"""ctypes binding of libphysattn.so (see include/physattn.h for the contract of every symbol).

PyTorch is used for device memory and streams only.  There is no fallback: if the library is not
built, or a call returns an error code, a RuntimeError is raised.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, Structure, c_char_p, c_float, c_int, c_int64, c_void_p

import torch  # noqa: F401  (must be imported first: its HIP runtime is the one the library binds to)

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libphysattn.so")

PA_F32, PA_BF16, PA_BF16_W8 = 0, 1, 2

EXPORTED = [
    "pa_version", "pa_set_compute_units", "pa_status_string", "pa_workspace_bytes", "pa_query_path", "pa_project_inputs",
    "pa_slice_softmax", "pa_reduce_partial_count", "pa_slice_reduce", "pa_slice_attention",
    "pa_deslice_project", "pa_layer_forward", "pa_mfma_buffer_bytes", "pa_mfma_pack_params",
    "pa_mfma_project_softmax", "pa_mfma_slice_reduce", "pa_mfma_project_softmax_reduce", "pa_mfma_partial_groups",
     "pa_mfma_combine_attention", "pa_mfma_deslice_project", "pa_mlp_query", "pa_mlp_workspace_bytes", "pa_mlp_forward", "pa_mlp_pack", "pa_mlp_pack_e4m3", "pa_mlp_input_ln_query", "pa_mlp_forward_packed_ln",
     "pa_mlp_forward_packed",
    "pa_rows_gemm", "pa_slice_weighted_sum", "pa_backward_query", "pa_backward_point_tiles",
    "pa_slice_attention_backward", "pa_slice_softmax_backward", "pa_slice_softmax_plus",
    "pa_backward_point_tiles_plus", "pa_slice_softmax_plus_backward", "pa_slice_cross_attention_mix",
    "pa_mfma_pack_tokens", "pa_flare_column_max_chunks", "pa_flare_column_weights", "pa_flare_softmax_rows",
    "pa_flare_backward_points", "pa_deslice", "pa_cols_gemm_f32_chunks", "pa_cols_gemm_f32", "pa_ball_query", "pa_ball_query_cells", "pa_layer_forward_plus_supported",
    "pa_layer_forward_plus_workspace_bytes", "pa_layer_forward_plus", "pa_flare_forward_mfma_supported",
    "pa_flare_forward_mfma_workspace_bytes", "pa_flare_forward_mfma",
    "pa_mfma_backward_query", "pa_rows_gemm_packed", "pa_mfma_slice_weighted_sum", "pa_mfma_deslice",
    "pa_mfma_backward_tables_bytes", "pa_mfma_backward_groups", "pa_mfma_slice_softmax_backward",
    "pa_cols_gemm_chunks", "pa_cols_gemm", "pa_residual_layernorm",
    "pa_mfma_layer_forward", "pa_rows_gemm_act", "pa_layernorm_backward_groups", "pa_layernorm_backward",
    "pa_static_scratch_bytes", "pa_slice_reduce_static",
    "pa_preprocess_query", "pa_preprocess_workspace_bytes", "pa_preprocess_forward",
    "pa_block_query", "pa_block_workspace_bytes", "pa_block_forward", "pa_markers_enabled",
    "pa_mfma_project_softmax_reduce_clocked",
]

PA_BUF_BLOB, PA_BUF_FX_PACK, PA_BUF_W_PACK, PA_BUF_PARTIALS, PA_BUF_TOKP = range(5)


class PaShape(Structure):
    _fields_ = [(n, c_int64) for n in ("B", "N", "C", "H", "D", "S", "grid_h", "grid_w", "conv_k", "grid_d",
                                        "conv_tap_major")]


class PaParams(Structure):
    _fields_ = [(n, c_void_p) for n in (
        "in_project_x_weight", "in_project_x_bias", "in_project_fx_weight", "in_project_fx_bias",
        "in_project_slice_weight", "in_project_slice_bias", "temperature", "qkv_project_weight",
        "out_linear_weight", "out_linear_bias", "in_project_x_scale", "in_project_fx_scale", "out_linear_scale")]


class PaMlpParams(Structure):
    _fields_ = [(n, c_void_p) for n in ("w1", "b1", "w2", "b2")]


class PaInputLn(Structure):
    _fields_ = [("gamma", c_void_p), ("beta", c_void_p), ("eps", c_float)]


class PaBlockMlp(Structure):
    _fields_ = [("ln_gamma", c_void_p), ("ln_beta", c_void_p), ("ln_eps", c_float), ("w1", c_void_p), ("b1", c_void_p),
                ("w2", c_void_p), ("b2", c_void_p), ("F", c_int64)]


class PaBlockHead(Structure):
    _fields_ = [("weight", c_void_p), ("bias", c_void_p), ("O", c_int64), ("out", c_void_p)]


class PaPlusParams(Structure):
    _fields_ = [(n, c_void_p) for n in ("proj_temperature_0_weight", "proj_temperature_0_bias",
                                        "proj_temperature_2_weight", "proj_temperature_2_bias")]


class PaGaleParams(Structure):
    _fields_ = [(n, c_void_p) for n in ("cross_q_weight", "cross_q_bias", "cross_k_weight", "cross_k_bias",
                                        "cross_v_weight", "cross_v_bias", "state_mixing", "concat_project_weight",
                                        "concat_project_bias")]


class PaBlockTail(Structure):
    _fields_ = [("residual", c_void_p), ("ln_gamma", c_void_p), ("ln_beta", c_void_p), ("ln_eps", c_float),
                ("ln_out", c_void_p)]


_lib = None


def load() -> ctypes.CDLL:
    """Load the shared library once; raise if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m physicsnemo_amd.build` "
            "(hipcc, gfx950). There is no fallback path.")
    lib = ctypes.CDLL(LIB_PATH)
    ps, pp, pt = POINTER(PaShape), POINTER(PaParams), POINTER(PaBlockTail)
    lib.pa_version.restype = c_int
    lib.pa_version.argtypes = []
    lib.pa_set_compute_units.restype = c_int
    lib.pa_set_compute_units.argtypes = [c_int]
    lib.pa_markers_enabled.restype = c_int
    lib.pa_markers_enabled.argtypes = []
    lib.pa_status_string.restype = c_char_p
    lib.pa_status_string.argtypes = [c_int]
    lib.pa_workspace_bytes.restype = c_int64
    lib.pa_workspace_bytes.argtypes = [c_int, ps]
    lib.pa_query_path.restype = c_int
    lib.pa_query_path.argtypes = [c_int, ps]
    lib.pa_project_inputs.restype = c_int
    lib.pa_project_inputs.argtypes = [c_int, ps, pp, c_void_p, c_void_p, c_void_p, c_void_p]
    lib.pa_slice_softmax.restype = c_int
    lib.pa_slice_softmax.argtypes = [c_int, ps, pp, c_void_p, c_void_p, c_void_p]
    lib.pa_reduce_partial_count.restype = c_int64
    lib.pa_reduce_partial_count.argtypes = [ps]
    lib.pa_slice_reduce.restype = c_int
    lib.pa_slice_reduce.argtypes = [c_int, ps, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]
    lib.pa_static_scratch_bytes.restype = c_int64
    lib.pa_static_scratch_bytes.argtypes = []
    lib.pa_slice_reduce_static.restype = c_int
    lib.pa_slice_reduce_static.argtypes = [c_int, ps, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]
    lib.pa_slice_attention.restype = c_int
    lib.pa_slice_attention.argtypes = [ps, pp, c_void_p, c_void_p, c_void_p]
    lib.pa_deslice_project.restype = c_int
    lib.pa_deslice_project.argtypes = [c_int, ps, pp, c_void_p, c_void_p, c_void_p, c_void_p, pt, c_void_p]
    lib.pa_layer_forward.restype = c_int
    lib.pa_layer_forward.argtypes = [c_int, ps, pp, c_void_p, c_void_p, pt, c_void_p, c_void_p, c_int64, c_void_p]
    lib.pa_mfma_buffer_bytes.restype = c_int64
    lib.pa_mfma_buffer_bytes.argtypes = [ps, c_int]
    lib.pa_mfma_pack_params.restype = c_int
    lib.pa_mfma_pack_params.argtypes = [ps, pp, c_void_p, c_void_p]
    lib.pa_mfma_project_softmax.restype = c_int
    lib.pa_mfma_project_softmax.argtypes = [ps, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]
    lib.pa_mfma_slice_reduce.restype = c_int
    lib.pa_mfma_slice_reduce.argtypes = [ps, c_void_p, c_void_p, c_void_p, c_void_p]
    lib.pa_mfma_combine_attention.restype = c_int
    lib.pa_mfma_combine_attention.argtypes = [ps, pp, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]
    lib.pa_mfma_project_softmax_reduce.restype = c_int
    lib.pa_mfma_project_softmax_reduce.argtypes = [ps, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]
    lib.pa_mfma_project_softmax_reduce_clocked.restype = c_int
    lib.pa_mfma_project_softmax_reduce_clocked.argtypes = [ps, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]
    lib.pa_mfma_partial_groups.restype = c_int64
    lib.pa_mfma_partial_groups.argtypes = [ps, c_int]
    lib.pa_mfma_deslice_project.restype = c_int
    lib.pa_mfma_deslice_project.argtypes = [ps, c_void_p, c_void_p, c_void_p, c_void_p, pt, c_void_p]
    lib.pa_mlp_query.restype = c_int
    lib.pa_mlp_query.argtypes = [c_int, c_int64, c_int64, c_int64]
    lib.pa_mlp_workspace_bytes.restype = c_int64
    lib.pa_mlp_workspace_bytes.argtypes = [c_int, c_int64, c_int64, c_int64]
    lib.pa_mlp_pack.restype = c_int
    lib.pa_mlp_pack.argtypes = [c_int, c_int64, c_int64, POINTER(PaMlpParams), c_void_p, c_int64, c_void_p]
    lib.pa_mlp_input_ln_query.restype = c_int
    lib.pa_mlp_input_ln_query.argtypes = [c_int, c_int64, c_int64, c_int64]
    lib.pa_mlp_forward_packed_ln.restype = c_int
    lib.pa_mlp_forward_packed_ln.argtypes = [c_int, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_void_p,
                                             POINTER(PaInputLn), c_void_p, c_void_p, POINTER(PaBlockTail), c_void_p]
    lib.pa_mlp_pack_e4m3.restype = c_int
    lib.pa_mlp_pack_e4m3.argtypes = [c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_void_p]
    lib.pa_mlp_forward_packed.restype = c_int
    lib.pa_mlp_forward_packed.argtypes = [c_int, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_void_p,
                                          c_void_p, pt, c_void_p]
    lib.pa_mlp_forward.restype = c_int
    lib.pa_mlp_forward.argtypes = [c_int, c_int64, c_int64, c_int64, POINTER(PaMlpParams), c_void_p, c_void_p, pt, c_void_p,
                                   c_int64, c_void_p]
    lib.pa_block_query.restype = c_int
    lib.pa_block_query.argtypes = [c_int, ps, c_int64]
    lib.pa_block_workspace_bytes.restype = c_int64
    lib.pa_block_workspace_bytes.argtypes = [c_int, ps, c_int64]
    lib.pa_block_forward.restype = c_int
    lib.pa_block_forward.argtypes = [c_int, ps, POINTER(PaParams), POINTER(PaBlockMlp), c_void_p, c_void_p, c_void_p, pt,
                                     POINTER(PaBlockHead), c_void_p, c_int64, c_void_p]
    lib.pa_preprocess_query.restype = c_int
    lib.pa_preprocess_query.argtypes = [c_int, c_int64, c_int64, c_int64, c_int64]
    lib.pa_preprocess_workspace_bytes.restype = c_int64
    lib.pa_preprocess_workspace_bytes.argtypes = [c_int, c_int64, c_int64, c_int64, c_int64]
    lib.pa_preprocess_forward.restype = c_int
    lib.pa_preprocess_forward.argtypes = [c_int, c_int64, c_int64, c_int64, c_int64, POINTER(PaMlpParams), c_void_p,
                                          c_void_p, pt, c_void_p, c_int64, c_void_p]
    lib.pa_rows_gemm.restype = c_int
    lib.pa_rows_gemm.argtypes = [c_int, ps, c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]
    lib.pa_slice_weighted_sum.restype = c_int
    lib.pa_slice_weighted_sum.argtypes = [c_int, ps, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]
    lib.pa_backward_query.restype = c_int
    lib.pa_backward_query.argtypes = [c_int, ps]
    lib.pa_backward_point_tiles.restype = c_int64
    lib.pa_backward_point_tiles.argtypes = [ps]
    lib.pa_slice_attention_backward.restype = c_int
    lib.pa_slice_attention_backward.argtypes = [ps, pp] + [c_void_p] * 8
    lib.pa_slice_softmax_backward.restype = c_int
    lib.pa_slice_softmax_backward.argtypes = [c_int, ps, pp] + [c_void_p] * 11
    lib.pa_slice_softmax_plus.restype = c_int
    lib.pa_slice_softmax_plus.argtypes = [c_int, ps, pp, POINTER(PaPlusParams)] + [c_void_p] * 5
    lib.pa_backward_point_tiles_plus.restype = c_int64
    lib.pa_backward_point_tiles_plus.argtypes = [ps]
    lib.pa_slice_softmax_plus_backward.restype = c_int
    lib.pa_slice_softmax_plus_backward.argtypes = [c_int, ps, pp, POINTER(PaPlusParams)] + [c_void_p] * 13
    lib.pa_slice_cross_attention_mix.restype = c_int
    lib.pa_slice_cross_attention_mix.argtypes = [ps, POINTER(PaGaleParams), c_int64, c_int64] + [c_void_p] * 6
    lib.pa_mfma_pack_tokens.restype = c_int
    lib.pa_mfma_pack_tokens.argtypes = [ps] + [c_void_p] * 3
    lib.pa_flare_column_max_chunks.restype = c_int64
    lib.pa_flare_column_max_chunks.argtypes = [ps]
    lib.pa_flare_column_weights.restype = c_int
    lib.pa_flare_column_weights.argtypes = [c_int, ps] + [c_void_p] * 5
    lib.pa_flare_softmax_rows.restype = c_int
    lib.pa_flare_softmax_rows.argtypes = [c_int, ps, c_void_p, c_void_p]
    lib.pa_flare_backward_points.restype = c_int
    lib.pa_flare_backward_points.argtypes = [c_int, ps] + [c_void_p] * 10
    lib.pa_deslice.restype = c_int
    lib.pa_deslice.argtypes = [c_int, ps] + [c_void_p] * 4
    lib.pa_flare_forward_mfma_supported.restype = c_int
    lib.pa_flare_forward_mfma_supported.argtypes = [ps]
    lib.pa_flare_forward_mfma_workspace_bytes.restype = c_int64
    lib.pa_flare_forward_mfma_workspace_bytes.argtypes = [ps]
    lib.pa_flare_forward_mfma.restype = c_int
    lib.pa_flare_forward_mfma.argtypes = [ps] + [c_void_p] * 8 + [POINTER(PaBlockTail), c_void_p, c_int64, c_void_p]
    lib.pa_layer_forward_plus_supported.restype = c_int
    lib.pa_layer_forward_plus_supported.argtypes = [c_int, ps]
    lib.pa_layer_forward_plus_workspace_bytes.restype = c_int64
    lib.pa_layer_forward_plus_workspace_bytes.argtypes = [c_int, ps]
    lib.pa_layer_forward_plus.restype = c_int
    lib.pa_layer_forward_plus.argtypes = [c_int, ps, pp, POINTER(PaPlusParams), c_void_p, c_void_p, c_void_p,
                                          POINTER(PaBlockTail), c_void_p, c_void_p, c_int64, c_void_p]
    lib.pa_ball_query.restype = c_int
    lib.pa_ball_query.argtypes = [c_int64, c_int64, c_int64, c_int64, c_float, c_void_p, c_void_p, c_void_p,
                                  c_void_p, c_void_p, c_void_p, c_void_p]
    lib.pa_ball_query_cells.restype = c_int
    lib.pa_ball_query_cells.argtypes = [c_int64, c_int64, c_int64, c_int64, c_float, c_int64] + [c_void_p] * 11
    lib.pa_cols_gemm_f32_chunks.restype = c_int64
    lib.pa_cols_gemm_f32_chunks.argtypes = [c_int64, c_int64, c_int64]
    lib.pa_cols_gemm_f32.restype = c_int
    lib.pa_cols_gemm_f32.argtypes = [c_int64, c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_void_p,
                                     c_void_p]
    lib.pa_mfma_backward_query.restype = c_int
    lib.pa_mfma_backward_query.argtypes = [ps]
    lib.pa_rows_gemm_packed.restype = c_int
    lib.pa_rows_gemm_packed.argtypes = [ps, c_int64] + [c_void_p] * 6
    lib.pa_mfma_slice_weighted_sum.restype = c_int
    lib.pa_mfma_slice_weighted_sum.argtypes = [ps] + [c_void_p] * 5
    lib.pa_mfma_deslice.restype = c_int
    lib.pa_mfma_deslice.argtypes = [ps] + [c_void_p] * 4
    lib.pa_mfma_backward_tables_bytes.restype = c_int64
    lib.pa_mfma_backward_tables_bytes.argtypes = [ps]
    lib.pa_mfma_backward_groups.restype = c_int64
    lib.pa_mfma_backward_groups.argtypes = [ps]
    lib.pa_mfma_slice_softmax_backward.restype = c_int
    lib.pa_mfma_slice_softmax_backward.argtypes = [ps, pp] + [c_void_p] * 12
    lib.pa_cols_gemm_chunks.restype = c_int64
    lib.pa_cols_gemm_chunks.argtypes = [c_int64, c_int64]
    lib.pa_cols_gemm.restype = c_int
    lib.pa_cols_gemm.argtypes = [c_int64, c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_void_p, c_void_p]
    lib.pa_residual_layernorm.restype = c_int
    lib.pa_residual_layernorm.argtypes = [c_int, c_int64, c_int64, c_void_p, pt, c_void_p]
    lib.pa_mfma_layer_forward.restype = c_int
    lib.pa_mfma_layer_forward.argtypes = [ps, pp, c_void_p, c_void_p, c_void_p, pt, c_void_p, c_void_p, c_int64, c_void_p]
    lib.pa_rows_gemm_act.restype = c_int
    lib.pa_rows_gemm_act.argtypes = [c_int, ps, c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p]
    lib.pa_layernorm_backward_groups.restype = c_int64
    lib.pa_layernorm_backward_groups.argtypes = [c_int64]
    lib.pa_layernorm_backward.restype = c_int
    lib.pa_layernorm_backward.argtypes = [c_int, c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_void_p,
                                          c_void_p]
    _lib = lib
    return lib


def check(code: int, what: str) -> None:
    """Turn a non-zero return code into a RuntimeError."""
    if code != 0:
        msg = load().pa_status_string(int(code)).decode()
        raise RuntimeError(f"{what} failed: {msg} (code {code})")


def dtype_code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return PA_F32
    if dtype == torch.bfloat16:
        return PA_BF16
    raise TypeError(f"physicsnemo_amd kernels take float32 or bfloat16 activations, got {dtype}")


def current_stream_ptr(device: torch.device) -> int:
    return int(torch.cuda.current_stream(device).cuda_stream)


def ptr(t) -> int | None:
    return None if t is None else int(t.data_ptr())
