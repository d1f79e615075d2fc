"""ctypes binding of libptv3_hip.so (the C ABI declared in include/ptv3_hip.h).

There is no fallback: if the library is missing or a call fails, an exception is raised.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libptv3_hip.so")

_vp, _i64, _i32, _f32, _sz = (ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float,
                              ctypes.c_size_t)

# name -> (restype, argtypes); mirrors include/ptv3_hip.h one to one
SIGNATURES = {
    "ptv3_version": (_i32, []),
    "ptv3_strerror": (ctypes.c_char_p, [_i32]),
    "ptv3_encode": (_i32, [_vp, _vp, _i64, _i32, _vp, _i32, _vp, _vp]),
    "ptv3_decode": (_i32, [_vp, _i64, _i32, _i32, _vp, _vp, _vp]),
    "ptv3_grid_max": (_i32, [_vp, _i64, _vp, _vp]),
    "ptv3_voxelize_workspace_bytes": (_sz, [_i64, _i32]),
    "ptv3_voxelize": (_i32, [_vp, _i64, _vp, _i32, _f32, _vp, _vp, _vp, _vp, _vp, ctypes.c_uint32, _vp, _sz, _vp]),
    "ptv3_offset2batch": (_i32, [_vp, _i32, _i64, _vp, _vp]),
    "ptv3_argsort_workspace_bytes": (_sz, [_i64, _i32]),
    "ptv3_argsort": (_i32, [_vp, _i64, _i32, _i32, _vp, _vp, _vp, _sz, _vp]),
    "ptv3_pad_sizes": (_i32, [_vp, _i32, _i64, _vp, _vp]),
    "ptv3_pad_index_workspace_bytes": (_sz, [_i32]),
    "ptv3_pad_index": (_i32, [_vp, _i32, _i64, _i64, _i64, _i64, _vp, _vp, _vp, _vp, _sz, _vp]),
    "ptv3_attn_slots": (_i32, [_vp, _vp, _vp, _vp, _i64, _vp, _vp, _vp]),
    "ptv3_patch_attn_fwd": (_i32, [_vp, _i32, _i64, _i32, _i32, _vp, _vp, _vp, _i64, _i64, _f32,
                                   _vp, _vp]),
    "ptv3_patch_attn_rpe_fwd": (_i32, [_vp, _i64, _i32, _i32, _vp, _vp, _vp, _i64, _i64, _f32, _vp, _vp, _i32, _f32,
                                       ctypes.c_uint32, _vp, _vp]),
    "ptv3_patch_attn_bwd_workspace_bytes": (_sz, [_i32, _i64, _i32, _i32]),
    "ptv3_patch_attn_fwd_lse": (_i32, [_vp, _i32, _i64, _i32, _i32, _vp, _vp, _vp, _i64, _i64, _i64, _f32, _f32,
                                       ctypes.c_uint32, _vp, _vp, _vp]),
    "ptv3_patch_attn_bwd": (_i32, [_vp, _vp, _vp, _i32, _i64, _i32, _i32, _vp, _vp, _vp, _i64, _i64, _i64, _f32, _vp,
                                   _f32, ctypes.c_uint32, _vp, _vp, _sz, _vp]),
    "ptv3_patch_attn_rpe_bwd": (_i32, [_vp, _vp, _vp, _i32, _i64, _i32, _i32, _vp, _vp, _vp, _i64, _i64, _i64, _f32, _vp,
                                       _f32, ctypes.c_uint32, _vp, _vp, _i32, _vp, _vp, _vp, _sz, _vp]),
    "ptv3_kmap_workspace_bytes": (_sz, [_i64]),
    "ptv3_kmap_build": (_i32, [_vp, _i64, _i32, _i32, _vp, _vp, _sz, _vp]),
    "ptv3_subm_conv_fwd": (_i32, [_vp, _i32, _i64, _i32, _vp, _i32, _i32, _vp, _vp, _i32, _vp, _vp]),
    "ptv3_subm_conv_wgrad_workspace_bytes": (_sz, [_i32, _i64, _i32, _i32, _i32]),
    "ptv3_subm_conv_wgrad": (_i32, [_vp, _vp, _i32, _i64, _i32, _i32, _vp, _i32, _vp, _vp, _vp, _sz, _vp]),
    "ptv3_conv_plan_workspace_bytes": (_sz, [_i64, _i32]),
    "ptv3_conv_plan_count": (_i32, [_vp, _i64, _i32, _i32, _vp, _vp, _vp, _sz, _vp]),
    "ptv3_conv_plan_fill": (_i32, [_vp, _i64, _i32, _i32, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "ptv3_kmap_plan_workspace_bytes": (_sz, [_i64, _i32]),
    "ptv3_kmap_plan_count": (_i32, [_vp, _i64, _i32, _vp, _vp, _vp, _sz, _vp]),
    "ptv3_kmap_plan_fill": (_i32, [_vp, _i64, _i32, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "ptv3_kmap_plan_inner_count": (_i32, [_vp, _i64, _vp, _sz, _vp, _vp, _vp, _vp, _vp]),
    "ptv3_kmap_plan_inner_fill": (_i32, [_vp, _vp, _vp, _vp, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _vp]),
    "ptv3_conv_plan_slots": (_i32, [_vp, _i32, _vp, _vp, _i64, _vp, _vp]),
    "ptv3_conv_plan_tile_count": (_i64, [_i64]),
    "ptv3_conv_plan_tiles": (_i32, [_vp, _vp, _i64, _i32, _vp, _vp, _vp, _vp]),
    "ptv3_subm_conv_pack_weight": (_i32, [_vp, _i32, _i32, _i32, _vp, _vp]),
    "ptv3_subm_conv_tiles_fwd": (_i32, [_vp, _i32, _i64, _i32, _i32, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "ptv3_conv_plan_tile_count_sized": (_i64, [_i64, _i32]),
    "ptv3_conv_plan_tiles_sized": (_i32, [_vp, _vp, _i64, _i32, _i32, _vp, _vp, _vp, _vp]),
    "ptv3_subm_conv_tiles_fwd_sized": (_i32, [_vp, _i32, _i64, _i32, _i32, _i32, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "ptv3_subm_conv_pack_weight_blocks": (_i64, [_i32, _i32]),
    "ptv3_subm_conv_pack_weight_batch": (_i32, [_vp, _i32, _i64, _vp]),
    "ptv3_subm_conv_sparse_fwd": (_i32, [_vp, _i32, _i64, _i32, _i32, _vp, _vp, _vp, _vp, _vp, _vp]),
    "ptv3_subm_conv_pairs_fwd": (_i32, [_vp, _i32, _i64, _i32, _i32, _i64, _vp, _vp, _vp, _vp, _vp, _vp,
                                        _i32, _vp, _vp, _vp]),
    "ptv3_pool_clusters_workspace_bytes": (_sz, [_i64]),
    "ptv3_pool_clusters": (_i32, [_vp, _vp, _i64, _i32, _vp, _i32, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "ptv3_pool_clusters_static_max_points": (_i64, []),
    "ptv3_pool_clusters_static": (_i32, [_vp, _vp, _i64, _i32, _vp, _i32, _vp, _vp, _vp, _vp, _vp]),
    "ptv3_pool_gather": (_i32, [_vp, _i64, _i32, _i32, _vp, _i32, _vp, _vp, _i64, _vp, _vp, _vp, _vp, _vp,
                                _vp]),
    "ptv3_pool_orders_workspace_bytes": (_sz, [_i64, _i32]),
    "ptv3_pool_orders": (_i32, [_vp, _vp, _i64, _i32, _i64, _vp, _vp, _vp, _vp, _sz, _vp]),
    "ptv3_segment_reduce": (_i32, [_vp, _i32, _i64, _i32, _vp, _vp, _i64, _i32, _vp, _vp]),
    "ptv3_segment_reduce_bwd": (_i32, [_vp, _vp, _vp, _i32, _i64, _i32, _vp, _vp, _i64, _i32, _vp, _vp]),
    "ptv3_unpool_add": (_i32, [_vp, _vp, _i32, _i64, _i32, _vp, _i64, _vp, _vp]),
    "ptv3_bn_act": (_i32, [_vp, _vp, _vp, _i32, _vp, _vp, _i32, _i64, _i32, _f32, _i32, _vp, _vp]),
    "ptv3_linear_fwd": (_i32, [_vp, _vp, _vp, _i32, _i64, _i32, _i32, _i32, _vp, _vp]),
    "ptv3_linear_wide_fwd": (_i32, [_vp, _vp, _vp, _i32, _i64, _i32, _i32, _i32, _vp, _vp]),
    "ptv3_linear_gemm_fwd": (_i32, [_vp, _vp, _vp, _vp, _i32, _i64, _i32, _i32, _vp, _vp]),
    "ptv3_linear_any_fwd": (_i32, [_vp, _vp, _vp, _vp, _i32, _i64, _i32, _i32, _i32, _vp, _vp]),
    "ptv3_linear_bn_act_fwd": (_i32, [_vp, _vp, _vp, _vp, _vp, _i32, _vp, _vp, _f32, _i32, _i64, _i32, _i32, _i32, _vp, _vp]),
    "ptv3_add_layer_norm_fwd": (_i32, [_vp, _i32, _vp, _i32, _vp, _i32, _vp, _vp, _i32, _i64, _i32, _f32, _vp, _i32,
                                       _vp, _i32, _vp, _vp, _f32, _vp]),
    "ptv3_add_layer_norm_bwd": (_i32, [_vp, _i32, _vp, _i32, _vp, _i32, _vp, _i32, _vp, _i32, _i64, _i32, _f32, _vp,
                                       _i32, _vp, _i32, _vp, _vp, _vp, _i32, _vp, _f32, _vp, _vp, _vp]),
    "ptv3_batch_norm_stats": (_i32, [_vp, _i32, _i64, _i32, _f32, _f32, _vp, _vp, _vp, _vp, _vp]),
    "ptv3_batch_norm_bwd": (_i32, [_vp, _i32, _vp, _i32, _vp, _vp, _vp, _i32, _i64, _i32, _i32, _i32, _vp, _i32, _vp,
                                   _vp]),
    "ptv3_linear_gelu_fwd": (_i32, [_vp, _vp, _vp, _i32, _i64, _i32, _i32, _vp, _vp, _vp]),
    "ptv3_linear_gelu_bwd": (_i32, [_vp, _vp, _vp, _i32, _i64, _i32, _i32, _vp, _vp]),
    "ptv3_scaled_add": (_i32, [_vp, _i32, _vp, _i32, _vp, _i32, _i64, _i32, _vp, _i32, _vp]),
    "ptv3_conv_plan_pair_out": (_i32, [_vp, _vp, _i64, _i64, _vp, _vp]),
    "ptv3_subm_conv_wgrad_pairs": (_i32, [_vp, _vp, _i32, _i64, _i32, _i32, _vp, _vp, _vp, _i32, _vp, _vp, _vp, _sz, _vp]),
    "ptv3_cast_params_blocks": (_i64, [_i32, _i32, _i32, _i32]),
    "ptv3_cast_params": (_i32, [_vp, _i32, _i64, _i32, _vp]),
    "ptv3_linear_wgrad_workspace_bytes": (_sz, [_i64, _i32, _i32]),
    "ptv3_linear_wgrad": (_i32, [_vp, _vp, _i32, _i64, _i32, _i32, _vp, _vp, _vp, _sz, _vp]),
    "ptv3_linear_ln_fwd": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _i64, _i32, _i32, _f32, _vp, _vp, _vp]),
    "ptv3_mlp_fused": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _i32, _i64, _i32, _i32, _vp, _vp]),
    "ptv3_mlp_pack_weights": (_i32, [_vp, _vp, _i32, _i32, _vp, _vp]),
    "ptv3_mlp_pack_weights_blocks": (_i64, [_i32]),
    "ptv3_mlp_pack_weights_batch": (_i32, [_vp, _i32, _i64, _vp]),
    "ptv3_mlp_fused_packed": (_i32, [_vp, _vp, _vp, _vp, _vp, _i32, _i64, _i32, _vp, _vp]),
    "ptv3_linear_pack_weights_blocks": (_i64, [_i32]),
    "ptv3_block_head_wide": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _f32, _vp, _vp, _f32, _vp, _i32, _i64, _i32, _vp, _vp, _vp]),
    "ptv3_block_tail_wide": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _f32, _vp, _vp, _vp, _i32, _i64, _i32, _vp, _vp]),
    "ptv3_block_head_fused": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _f32, _vp, _vp, _f32, _vp, _vp, _i32, _i64, _i32,
                                     _vp, _vp, _vp]),
    "ptv3_block_tail_fused": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _f32, _vp, _vp, _vp, _vp, _i32, _i64, _i32, _i32,
                                     _vp, _vp]),
    "ptv3_layer_norm": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _i64, _i32, _f32, _i32, _vp, _vp, _vp]),
}

_lib = None


class Ptv3Error(RuntimeError):
    pass


def load():
    """Load the shared library once; raise if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise Ptv3Error(
                f"{LIB_PATH} not found: build it with `make -C pointtransformerv3_amd/csrc` "
                "(hipcc --offload-arch=gfx950). There is no CPU fallback.")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)  # AttributeError if the ABI and the header disagree
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def check(rc, what):
    if rc != 0:
        msg = load().ptv3_strerror(rc).decode()
        raise Ptv3Error(f"{what} failed with code {rc}: {msg}")
