"""MI355X-native fused CP4-decomposed Conv2d (forward, backward-data,
backward-filter) behind a C ABI.

This Python package is only the loader/binding of ``csrc/libcp4conv.so`` used
by the tests and the bench; the product is the shared library and the C++ host
layer under ``csrc/host``.  There is no CPU or PyTorch fallback: importing
``paralleltnnlayers_amd.capi`` without the built library raises.
"""
from .capi import (Shape, Geometry, geometry, conv2d_forward_ex, conv2d_backward_data_ex,
                   conv2d_backward_filter_ex, backward_ex_workspace_bytes, Cp4Error, lib, library_path, conv2d_forward, conv2d_forward_bias_act, conv2d_forward_bf16,
                   conv2d_backward_data_bf16, conv2d_backward_filter_bf16, bf16_supported,
                   conv2d_forward_f16, conv2d_backward_data_f16, conv2d_backward_filter_f16, rcp_conv2d_forward,
                   rcp_conv2d_backward_data, rcp_conv2d_backward_filter,
                   conv2d_backward_data, conv2d_backward_filter, conv2d_backward_filter_noalloc,
                   conv2d_backward_filter_full, backward_filter_workspace_bytes,
                   time_forward, time_forward_sets, time_backward_data, time_backward_filter,
                   tune_forward, tune_backward_data, tune_backward_filter, tuned_choice, plan_query,
                   set_tuned_choice, tuned_table, tuned_filter_table, set_tuned_filter_choice,
                   backward_filter_variants, save_tuned, load_tuned, tune_clear, device_status, device_status_detail, set_spin_limit, set_backward_filter_tile_kernel,
                   forward_variants, default_variant, recompose, count_exceeding,
                   random_uniform, time_copy, cp3_shape_for, cp3_expand_factors,
                   cp3_fold_gradients, cp3_conv2d_forward, cp3_conv2d_backward_data,
                   cp3_conv2d_backward_filter)

__all__ = [n for n in dir() if not n.startswith("_")]
