"""ctypes loader of the native library (``libdarknet_hip.so``).

The library is the product; there is no Python or CPU fallback.  ``load()`` raises if the
shared object is missing, and every entry point declared in ``include/darknet_hip.h`` and
``include/darknet_amd.h`` is bound here, so a missing symbol fails at load time, not mid-run.
"""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libdarknet_hip.so")

F = C.POINTER(C.c_float)
I = C.POINTER(C.c_int)
U = C.POINTER(C.c_uint)
V = C.c_void_p
i, f, z = C.c_int, C.c_float, C.c_size_t

# name -> (restype, argtypes); kept in the order of the two public headers
SIGNATURES = {
    # ---- darknet_hip.h: device shim
    "hip_set_device": (None, [i]), "hip_get_device": (i, []), "hip_check_error": (None, [i]),
    "hip_make_array": (V, [F, z]), "hip_make_int_array": (V, [I, z]), "hip_free": (None, [V]),
    "hip_push_array": (None, [V, F, z]), "hip_pull_array": (None, [V, F, z]),
    "hip_mag_array": (f, [V, z]), "hip_compare": (f, [V, F, z, C.c_char_p]),
    "hip_random": (None, [V, z]), "cuda_random": (None, [V, z]),
    "forward_batchnorm_gpu": (None, [V] * 6 + [i, i, i]),
    "hip_pull_int_array": (None, [V, I, z]), "hip_push_int_array": (None, [V, I, z]),
    "hip_synchronize": (None, []),
    "hip_get_stream": (V, []), "hip_set_stream": (None, [V]), "hip_device_name": (C.c_char_p, []),
    "cuda_set_device": (None, [i]), "cuda_get_device": (i, []), "cuda_make_array": (V, [F, z]),
    "cuda_make_int_array": (V, [I, z]), "cuda_free": (None, [V]),
    "cuda_push_array": (None, [V, F, z]), "cuda_pull_array": (None, [V, F, z]),
    "cuda_mag_array": (f, [V, z]), "cuda_compare": (f, [V, F, z, C.c_char_p]),
    "hip_event_create": (V, []), "hip_event_record": (None, [V]),
    "hip_event_elapsed_ms": (f, [V, V]), "hip_event_destroy": (None, [V]),
    # ---- darknet_hip.h: element-wise helpers
    "fill_gpu": (None, [i, f, V, i]), "copy_gpu": (None, [i, V, i, V, i]),
    "copy_gpu_offset": (None, [i, V, i, i, V, i, i]), "activate_array_gpu": (None, [V, i, i]),
    "normalize_gpu": (None, [V, V, V, i, i, i]), "scale_bias_gpu": (None, [V, V, i, i, i]),
    "add_bias_gpu": (None, [V, V, i, i, i]),
    "shortcut_gpu": (None, [i, i, i, i, V, i, i, i, f, f, V]),
    "upsample_gpu": (None, [V, i, i, i, i, i, i, f, V]),
    "softmax_gpu": (None, [V, i, i, i, i, i, i, f, V]),
    "im2col_gpu": (None, [V, i, i, i, i, i, i, V]),
    "binarize_gpu": (None, [V, i, V]), "binarize_weights_gpu": (None, [V, i, i, V]),
    # ---- darknet_hip.h: fused layer forwards
    "forward_convolutional_gpu": (None, [V] * 8 + [i] * 11),
    "forward_convolutional_shortcut_gpu": (None, [V] * 8 + [i] * 11 + [V, V, f, f, i]),
    "forward_convolutional_noalloc_gpu": (i, [V] * 8 + [i] * 11),
    "forward_convolutional_yolo_gpu": (None, [V] * 8 + [i] * 11 + [V, i, i]),
    "conv_packed_floats": (z, [i, i, i, i]), "conv_pack_weights_gpu": (None, [V, V, i, i, i, i]),
    "conv_packed_cached_gpu": (V, [V, i, i, i, i]), "conv_packed_forget": (None, [V]),
    "conv_packed_cached_count": (i, []),
    "conv_set_algo": (None, [i]), "conv_set_ksplit": (None, [i, i]), "conv_set_bands": (None, [i]), "conv_first_set_shape": (None, [i]),
    "xnor_weight_words": (z, [i, i, i]), "xnor_input_words": (z, [i, i, i, i]),
    "xnor_pack_weights_gpu": (None, [V, V, V, i, i, i]),
    "xnor_pack_input_gpu": (None, [V, V, i, i, i, i]),
    "forward_convolutional_xnor_gpu": (None, [V] * 10 + [i] * 10),
    "forward_convolutional_xnor_packed_gpu": (None, [V] * 9 + [i] * 10),
    "forward_convolutional_xnor_fused_gpu": (None, [V] * 4 + [i] + [V] * 7 + [i] * 10),
    "conv_maxpool_fusable": (i, [i] * 10),
    "forward_convolutional_maxpool_gpu": (None, [V] * 9 + [i] * 11),
    "forward_maxpool_gpu": (None, [V, V, V] + [i] * 7),
    "forward_route_gpu": (None, [C.POINTER(V), I, i, V, i]),
    "forward_shortcut_gpu": (None, [V, V, V] + [i] * 7 + [f, f, i]),
    "forward_yolo_gpu": (None, [V, V] + [i] * 5),
    "forward_avgpool_gpu": (None, [V, V] + [i] * 4),
    # ---- darknet_amd.h: layer / network API
    "parse_network_cfg": (V, [C.c_char_p]), "load_network": (V, [C.c_char_p, C.c_char_p, i]),
    "load_weights": (None, [V, C.c_char_p]), "load_weights_upto": (None, [V, C.c_char_p, i, i]),
    "save_weights": (None, [V, C.c_char_p]), "save_weights_upto": (None, [V, C.c_char_p, i]),
    "get_activation": (i, [C.c_char_p]), "get_activation_string": (C.c_char_p, [i]),
    "get_layer_string": (C.c_char_p, [i]),
    "reorg_gpu": (None, [V, i, i, i, i, i, i, V]), "flatten_gpu": (None, [V, i, i, i, i, V]),
    "forward_crop_gpu": (None, [V, V, i, i, i, i, i, i, i]),
    "resize_image_gpu": (None, [V, i, i, i, V, i, i]), "letterbox_image_gpu": (None, [V, i, i, i, V, i, i]),
    "network_pull_outputs": (None, [V]),
    "yolo_decode_gpu": (None, [V, i, i, i, i, F, i, i, i, i, i, f, V, i, V]),
    "nms_sort_gpu": (None, [V, i, i, f]),
    "region_decode_gpu": (None, [V, i, i, i, i, i, i, F, i, i, i, i, i, f, V, i, V]),
    "forward_region_gpu": (None, [V, V, i, i, i, i, i, i, i, i]),
    "forward_local_gpu": (None, [V, V, V, V, i, i, i, i, i, i, i, i, i]),
    "local_set_patch_budget": (None, [C.c_long]),
    "forward_connected_stream_gpu": (None, [V, V, V, V, i, i, i, i]),
    "detection_decode_gpu": (None, [V, i, i, i, i, i, i, f, V, i, V]),
    "num_detections": (i, [V, f]), "make_network_boxes": (V, [V, f, I]),
    "fill_network_boxes": (None, [V, i, i, f, f, I, i, V]),
    "get_network_boxes": (V, [V, i, i, f, f, I, i, I]), "free_detections": (None, [V, i]),
    "do_nms_sort": (None, [V, i, i, f]),
    "get_network_boxes_image": (V, [V, i, i, i, f, i, f, I]),
    "network_decode_image_gpu": (i, [V, i, i, i, f, i]),
    "make_network": (V, [i]), "free_network": (None, [V]), "forward_network": (None, [V]),
    "forward_network_gpu": (None, [V]), "network_predict": (F, [V, F]),
    "set_batch_network": (None, [V, i]), "network_output": (F, [V]),
    "pull_network_output": (None, [V]), "network_width": (i, [V]), "network_height": (i, [V]),
    "forward_network_device": (None, [V]), "forward_network_profiled": (f, [V, F]),
    "network_set_fusion": (None, [i]),
    "network_layer_runs_fused": (i, [V, i]), "network_layer_output_skipped": (i, [V, i]),
    "network_predict_submit": (None, [V, F]), "network_predict_collect": (F, [V]),
    "network_collected_output": (F, [V, i]), "network_predict_in_flight": (i, [V]),
    "forward_network_profiled_kernels": (f, [V, F, F]),
    "hip_set_parse_only": (None, [i]), "hip_parse_only": (i, []),
    "hip_host_alloc": (F, [z]), "hip_host_free": (None, [F]),
    "conv_set_precision": (None, [i]), "conv_get_precision": (i, []),
    "conv_profile_next": (None, [V, V]), "conv_profile_pending": (i, []),
    "conv_kernel_name": (C.c_char_p, [i, i, i, i]),
    "conv_kernel_name_columns": (C.c_char_p, [i, i, i, i, C.c_long]),
    "conv_kernel_name_geometry": (C.c_char_p, [i] * 9), "layer_output_host": (F, [V, i]),
    "layer_indexes_host": (I, [V, i]), "network_set_verbose": (None, [i]),
    "network_set_conv": (None, [V, i, F, F, F, F, F]),
    "network_layer_info": (None, [V, i, I, F]), "network_route_inputs": (i, [V, i, I, I, i]),
    "network_num_layers": (i, [V]), "network_input_gpu": (V, [V]), "network_info": (None, [V, I]),
    "network_conv_flops": (C.c_double, [V]),
}

# exported but taking structs by value (bound by reference C code, not through ctypes)
STRUCT_BY_VALUE = [
    "make_convolutional_layer", "make_maxpool_layer", "make_route_layer", "make_shortcut_layer",
    "make_upsample_layer", "make_yolo_layer", "make_avgpool_layer", "make_softmax_layer", "free_layer",
    "forward_convolutional_layer_gpu", "forward_maxpool_layer_gpu", "forward_route_layer_gpu",
    "forward_shortcut_layer_gpu", "forward_upsample_layer_gpu", "forward_yolo_layer_gpu",
    "forward_avgpool_layer_gpu", "forward_softmax_layer_gpu", "push_convolutional_layer",
    "pull_convolutional_layer", "get_network_output_layer",
    "make_connected_layer", "make_dropout_layer", "make_reorg_layer", "make_crop_layer", "make_cost_layer",
    "forward_connected_layer_gpu", "forward_dropout_layer_gpu", "forward_reorg_layer_gpu",
    "forward_crop_layer_gpu", "forward_cost_layer_gpu", "push_connected_layer", "pull_connected_layer",
    "make_region_layer", "forward_region_layer_gpu",
    "make_local_layer", "forward_local_layer_gpu", "push_local_layer", "pull_local_layer",
    "make_detection_layer", "forward_detection_layer_gpu",
    "make_batchnorm_layer", "forward_batchnorm_layer_gpu", "push_batchnorm_layer", "pull_batchnorm_layer",
    "make_image", "make_empty_image", "free_image", "resize_image", "letterbox_image", "network_predict_image",
    "network_letterbox_input",
]

_lib = None


def load() -> C.CDLL:
    """Load the library and bind every exported entry point; raise if anything is missing."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m darknet_amd.build` "
            "(there is no fallback implementation)")
    lib = C.CDLL(LIB_PATH)  # RTLD_LOCAL: the reference-compatible names stay private to this handle
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.restype = res
        fn.argtypes = args
    for name in STRUCT_BY_VALUE:
        getattr(lib, name)
    C.c_int.in_dll(lib, "gpu_index")
    lib.network_set_verbose(0)
    _lib = lib
    return lib
