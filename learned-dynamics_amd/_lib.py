"""ctypes binding of libmanagan_hip.so (the C ABI declared in include/managan_hip.h).

The library is the only compute path: if it is missing the import fails with
instructions to build it; there is no CPU or PyTorch fallback.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmanagan_hip.so")
EXT_PATH = os.path.join(_HERE, "managan_torch_ext.so")

c_float_p = ctypes.c_void_p   # device pointers travel as integers
c_int_p = ctypes.c_void_p
vp = ctypes.c_void_p
i32 = ctypes.c_int
i64 = ctypes.c_long
f32 = ctypes.c_float
PtrArray13 = ctypes.c_void_p * 13

MG_OK = 0
MG_ERR_INVALID_ARGUMENT = 1
MG_ERR_HIP = 2
MG_ERR_BOX_TOO_SMALL = 3
MG_ERR_WORKSPACE = 4
MG_ERR_UNSUPPORTED = 5

_SIGNATURES = {
    "mg_neighbour_ndiv": [f32, f32, f32, f32, ctypes.POINTER(i32 * 3)],
    "mg_neighbour_workspace_bytes": [i32, i32, f32, f32, f32, f32, ctypes.POINTER(ctypes.c_size_t)],
    "mg_neighbour_count": [vp, i32, i32, f32, f32, f32, f32, vp, ctypes.c_size_t, vp, vp, vp, vp],
    "mg_neighbour_fill": [vp, ctypes.c_size_t, i32, i32, f32, f32, f32, f32, vp, i32, vp, vp, vp],
    "mg_neighbour_edges": [vp, i32, i32, f32, f32, f32, f32, vp, ctypes.c_size_t, vp, vp, vp, i32, vp, vp, vp],
    "mg_neighbour_edges_static": [vp, i32, i32, f32, f32, f32, f32, vp, vp, vp, i32, vp, vp, vp],
    "mg_neighbour_cell_order": [vp, ctypes.c_size_t, i32, i32, f32, f32, f32, f32, vp, vp],
    "mg_neighbour_wrap_cells": [vp, i32, i32, f32, f32, f32, f32, vp, vp, vp],
    "mg_neighbour_pad": [vp, vp, i32, i32, i32, vp, vp, vp],
    "mg_padded_edges_read": [vp, vp, vp, i32, i32, i32, i32, vp, vp],
    "mg_padded_edges_reduce": [vp, vp, i32, i32, i32, i32, vp, vp],
    "mg_edge_vectors": [vp, vp, vp, i64, f32, f32, f32, vp, vp, vp],
    "mg_segment_row_ptr": [vp, i32, i64, i32, vp, vp],
    "mg_segment_sum_csr": [vp, vp, i32, i32, vp, vp],
    "mg_segment_sum_csr_perm": [vp, vp, vp, i32, i32, vp, vp],
    "mg_gather_rows": [vp, vp, i32, i64, i32, i32, vp, vp],
    "mg_bee_fwd": [vp, vp, vp, vp, vp, vp, i64, i32, ctypes.POINTER(PtrArray13), vp],
    "mg_bee_bwd": [i32, vp, vp, vp, ctypes.POINTER(PtrArray13), i64, i32, vp, vp, vp, vp],
    "mg_bee_indexed_supported": [i32],
    "mg_bee_fwd_indexed": [vp, vp, vp, vp, i64, vp, vp, vp, i64, i32, ctypes.POINTER(PtrArray13), vp],
    "mg_bee_bwd_indexed": [i32, vp, vp, vp, vp, i64, ctypes.POINTER(PtrArray13), vp, i64, ctypes.c_uint, i64, i32, vp, vp,
                           vp, vp],
    "mg_cow_o0_fwd": [vp, vp, vp, vp, i64, i32, vp, vp, vp],
    "mg_cow_o1_fwd": [vp, vp, vp, vp, i64, i32, vp, vp, vp, vp],
    "mg_cow_o0_bwd": [i32, vp, vp, vp, vp, i64, i32, vp, vp, vp],
    "mg_cow_o1_bwd": [i32, vp, vp, vp, vp, vp, i64, i32, vp, vp, vp],
    "mg_tensor_prod_bare": [i32, i32, i32, vp, vp, i64, i32, vp, vp],
    "mg_tensor_prods_avd": [vp, vp, vp, i64, i32, vp, vp, vp, vp],
    "mg_tensor_prods_supported": [i32, i32, i32, i32, i32, i32, i32],
    "mg_tensor_prods": [i32, i32, i32, vp, i64, vp, i64, vp, i64, vp, vp, i64, i32, i32, i32, i32, vp, vp],
    "mg_tensor_linear": [i32, vp, i64, i64, vp, i64, i32, i32, vp, i32, i32, vp, vp],
    "mg_tensor_linear_wgrad_workspace_bytes": [i64, i32, i32, ctypes.POINTER(ctypes.c_size_t)],
    "mg_tensor_linear_wgrad": [i32, vp, vp, i64, i32, i32, vp, vp, vp],
    "mg_tensor_linear_wgrad_f16x2_supported": [i64, i32, i32],
    "mg_tensor_linear_wgrad_f16x2": [vp, vp, vp, i64, vp, i64, i64, i32, i32, vp, vp, vp, vp],
    "mg_tensor_linear_layout": [i32, vp, i64, i64, vp, i64, i32, i32, vp, i32, i32, i32, i32, vp, vp],
    "mg_bee_edge_geometry": [vp, i64, f32, vp, vp, vp],
    "mg_bee_message": [vp, vp, vp, i32, i64, vp, vp, vp, vp, vp, i32, vp, vp, vp, vp, vp, vp, vp, vp],
    "mg_bee_node_products_rank2": [i64, i32, vp, vp, vp, vp, vp, vp, vp, i32, vp, vp, vp, vp, vp, vp, vp, i32, vp],
    "mg_bee_message_rank2_supported": [i32, i32],
    "mg_bee_rank2_weight_bytes": [i32, vp],
    "mg_bee_pack_rank2_weight": [vp, i64, i32, i32, vp, vp],
    "mg_bee_message_rank2": [vp, vp, vp, i32, i64, vp, vp, vp, vp, vp, i32, vp, vp, vp, i32, vp, vp, vp, i32, vp, vp, vp],
    "mg_linear_packed_weight_bytes": [i32, i32, ctypes.POINTER(ctypes.c_size_t)],
    "mg_linear_pack_weight": [vp, i64, i64, i32, i32, vp, vp],
    "mg_tensor_linear_packed": [vp, vp, i64, i32, i32, vp, i32, i32, i32, vp, vp],
    "mg_linear_f16x2_packed_weight_bytes": [i32, i32, ctypes.POINTER(ctypes.c_size_t)],
    "mg_linear_f16x2_pack_weight": [vp, i64, i64, i32, i32, vp, vp],
    "mg_row_absmax": [vp, i64, i32, vp, vp],
    "mg_linear_f64": [vp, vp, vp, i64, i32, i32, i32, vp, vp],
    "mg_tensor_linear_f16x2_rowmax_parts": [i64, i32, i32],
    "mg_tensor_linear_f16x2": [vp, vp, vp, i32, i64, i64, i64, i32, i32, vp, i32, i32, i32, vp, vp, vp],
    "mg_tensor_linear_f16x2_scaled_bound": [vp, vp, vp, i32, i64, i64, i64, i32, i32, vp, i32, i32, i32, vp, vp,
                                            ctypes.c_float, ctypes.c_float, vp],
    "mg_ant16_fwd": [i32, i32, ctypes.POINTER(i32), ctypes.POINTER(vp), ctypes.POINTER(vp), vp, vp, vp, i64, i32, i32, i32,
                     i32, i32, vp, vp],
    "mg_ant16_grad_x": [i32, i32, ctypes.POINTER(i32), ctypes.POINTER(vp), ctypes.POINTER(vp), vp, vp, vp, i64, i32, i32, i32,
                        i32, i32, vp, vp],
    "mg_ant16_grad_left": [i32, vp, vp, vp, i64, i32, i32, i32, i32, vp, vp],
    "mg_ant16_grad_weight_workspace_bytes": [i64, i32, i32, i32, ctypes.POINTER(ctypes.c_size_t)],
    "mg_ant16_grad_weight": [i32, vp, vp, vp, i64, i32, i32, i32, i32, vp, vp, vp],
    "mg_set_linear_mode": [i32],
    "mg_get_linear_mode": [],
    "mg_group_norm_scratch_bytes": [i32, i32, ctypes.POINTER(ctypes.c_size_t)],
    "mg_group_norm": [i32, vp, i64, vp, i64, i32, i32, i32, i32, i32, f32, vp, vp, vp, i64, vp, vp, vp, vp],
    "mg_tens_sigmoid": [i32, vp, i64, vp, vp],
    "mg_painn_update_pre": [vp, i32, vp, i64, i32, vp, vp, vp, vp],
    "mg_painn_update_vec": [vp, i32, vp, vp, i64, i32, vp, vp],
    "mg_radial_encode": [i32, vp, i64, i32, f32, vp, vp],
    "mg_bee_node_products": [i64, i32, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp],
    "mg_bee_node_products_bf16": [i64, i32, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp],
    "mg_tensor_linear_bf16": [vp, vp, i64, i32, i32, vp, i32, i32, i32, i32, vp, vp],
    "mg_bee_message_bf16": [vp, vp, vp, i32, i64, vp, vp, vp, vp, vp, i32, vp, vp, vp, vp, vp, vp],
    "mg_segment_sum_csr_bf16": [vp, vp, i32, i32, f32, vp, vp],
    "mg_painn_radial_encode": [vp, i64, i32, f32, vp, vp],
    "mg_painn_radial_linear": [vp, i64, i32, f32, vp, i64, i64, vp, i32, i32, vp, vp],
    "mg_painn_table_message": [vp, vp, vp, i32, i64, vp, vp, i32, f32, vp, vp, i32, f32, vp, vp, vp, vp, vp],
    "mg_painn_edge_records": [vp, i64, i32, f32, f32, vp, vp],
    "mg_painn_table_message_sliced": [vp, vp, vp, i32, i64, vp, vp, i32, vp, vp, i32, vp, vp, vp, vp, vp],
    "mg_painn_combine_supported": [i32],
    "mg_silu_order": [vp, vp, i64, i32, vp, vp],
    "mg_bee_edge_filters_fwd": [vp, vp, i64, i32, vp, vp, vp],
    "mg_bee_edge_filters_bwd": [vp, vp, vp, vp, i64, i32, vp, vp, vp],
    "mg_painn_table_interp_supported": [i32, i32],
    "mg_painn_table_interp_fwd": [vp, i32, i32, f32, vp, i64, i32, vp, vp],
    "mg_painn_table_buckets": [vp, i64, i32, f32, vp, vp],
    "mg_painn_table_interp_bwd_workspace_bytes": [i32, i32, ctypes.POINTER(ctypes.c_size_t)],
    "mg_painn_table_interp_bwd": [vp, vp, i32, i32, f32, vp, vp, vp, i64, i32, vp, vp, vp, vp],
    "mg_painn_combine_fwd": [vp, vp, vp, vp, vp, i64, i64, i32, i32, vp, vp, vp],
    "mg_painn_combine_fwd_rows": [vp, vp, vp, vp, vp, i64, vp, i64, i64, i32, i32, vp, vp, vp],
    "mg_painn_combine_bwd": [vp, vp, vp, vp, vp, i64, vp, vp, vp, i64, i64, i32, i32, vp, vp, vp, vp, vp],
    "mg_painn_combine_bwd_rows": [vp, vp, i32, f32, vp, vp, vp, vp, vp, vp, i64, vp, vp, vp, i64, i64, i32, i32, vp, vp, vp,
                                  vp, vp],
    "mg_painn_combine_bwd_grid": [vp, i32, f32, vp, vp, vp, vp, vp, i64, vp, vp, vp, i64, i64, i32, i32, vp, vp, vp, vp, vp],
    "mg_painn_message": [vp, vp, vp, i32, i64, vp, vp, vp, vp, i32, f32, vp, vp, vp, vp, vp],
    "mg_tensor_linear_bf16_rowsum_workspace_bytes": [i64, i32, ctypes.POINTER(ctypes.c_size_t)],
    "mg_tensor_linear_bf16_rowsum": [vp, vp, i64, i32, i32, vp, i32, vp, vp, i64, f32, vp, vp, vp, vp],
    "mg_mlp_chain_bf16_workspace_bytes": [i64, ctypes.POINTER(ctypes.c_size_t)],
    "mg_mlp_chain_bf16": [vp, i64, i32, vp, vp, vp, vp, vp, i32, vp, vp, i64, vp, vp, vp, vp],
    "mg_repel5_sim": [vp, vp, vp, f32, f32, i32, i32, i32, ctypes.c_uint64, ctypes.c_uint32, vp],
    "mg_displacement_sums": [vp, i64, i64, vp, vp, i32, f32, vp, vp, vp, vp],
    "mg_tens_group_norm_bf16_scratch_bytes": [i32, i32, ctypes.POINTER(ctypes.c_size_t)],
    "mg_tens_group_norm_bf16": [vp, vp, i32, i32, i32, i32, i32, f32, vp, vp, vp, vp],
    "mg_components_to_rows": [vp, i64, i32, i32, i32, vp, vp, vp],
    "mg_bee_products_linear": [i32, vp, vp, vp, vp, vp, vp, vp, i64, i32, vp, i32, i32, vp, vp],
    "mg_tensor_linear_f16x2_rowsum_workspace_bytes": [i64, i32, ctypes.POINTER(ctypes.c_size_t)],
    "mg_tensor_linear_f16x2_rowsum": [vp, vp, vp, i32, i64, i64, i32, i32, vp, i32, vp, vp, i64, f32, vp, vp, vp, vp],
    "mg_tensor_linear_f16x2_rowsum_scaled_bound": [vp, vp, vp, i32, i64, i64, i32, i32, vp, i32, vp, vp, i64, f32, vp, vp,
                                                   vp, f32, f32, vp],
    "mg_painn_filter_hidden": [vp, i64, f32, vp, i64, i64, vp, vp, vp, i32, vp, vp, vp],
    "mg_painn_filter_message_workspace_bytes": [i64, i32, ctypes.POINTER(ctypes.c_size_t)],
    "mg_painn_filter_message": [vp, vp, vp, vp, i32, i64, i32, vp, vp, vp, vp, vp, vp, i64, i64, i32, f32, vp, vp, vp, vp, vp, vp],
}

_lib = None


def load():
    """Load the library once; raise if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python learned-dynamics_amd/build.py` "
            "(hipcc, --offload-arch=gfx950). There is no fallback path.")
    lib = ctypes.CDLL(LIB_PATH)
    for name, argtypes in _SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = ctypes.c_int
    lib.mg_status_string.restype = ctypes.c_char_p
    lib.mg_status_string.argtypes = [ctypes.c_int]
    lib.mg_last_error.restype = ctypes.c_char_p
    lib.mg_last_error.argtypes = []
    lib.mg_abi_version.restype = ctypes.c_int
    lib.mg_abi_version.argtypes = []
    _lib = lib
    return lib


_ext = None


def load_torch_ext():
    """The PyTorch C++ binding of the library (csrc/torch_binding.cpp): the reference's extension functions with
    at::Tensor arguments.  Raises if it has not been built."""
    global _ext
    if _ext is None:
        load()                                              # the library it links to, by its path
        if not os.path.exists(EXT_PATH):
            raise ImportError(f"{EXT_PATH} is missing: build it with `python learned-dynamics_amd/build.py`")
        import importlib.util

        import torch  # noqa: F401  (the binding links to torch's libraries)
        spec = importlib.util.spec_from_file_location("managan_torch_ext", EXT_PATH)
        module = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(module)
        _ext = module
    return _ext


def check(status):
    """Turn a non-zero mg_status into the Python exception the reference would raise."""
    if status == MG_OK:
        return
    lib = load()
    text = lib.mg_last_error().decode(errors="replace")
    if status == MG_ERR_BOX_TOO_SMALL:
        raise RuntimeError("box dimension must be greater than 3*cutoff")
    kind = lib.mg_status_string(status).decode()
    raise RuntimeError(f"{kind}: {text}" if text else kind)


def exported_symbols():
    return sorted(_SIGNATURES) + ["mg_status_string", "mg_last_error", "mg_abi_version"]
