"""ctypes binding of libconvlogic_amd.so (the C ABI declared in include/convlogic_amd.h).

The library is loaded on first use.  If it has not been built this raises: there is no
fallback implementation behind the "cuda" code paths.
"""
import ctypes
import os

import torch

_PKG = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB_PATH = os.path.join(_PKG, "libconvlogic_amd.so")

CLG_F32, CLG_F64, CLG_F16 = 0, 1, 2
_DTYPES = {torch.float32: CLG_F32, torch.float64: CLG_F64}
_DTYPES_FC = {**_DTYPES, torch.float16: CLG_F16}       # LogicLayer forward / backward_w / backward_x also store half

_p, _i, _i64, _f64 = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_double


class ConvGeom(ctypes.Structure):
    _fields_ = [(k, ctypes.c_int32) for k in
                ("n", "c_in", "h", "w", "c_out", "stride_h", "stride_w", "pad_h", "pad_w", "kernel_h", "kernel_w")]


_GP = ctypes.POINTER(ConvGeom)

# name -> (restype, argtypes); every symbol include/convlogic_amd.h declares
SIGNATURES = {
    "clg_last_error": (ctypes.c_char_p, []),
    "clg_abi_version": (_i, []),
    "clg_reload_knobs": (None, []),
    "clg_gate_argmax": (_i, [_i, _p, _p, _i64, _p]),
    "clg_fc_forward": (_i, [_i, _p, _p, _p, _p, _p, _i64, _i64, _i64, _p]),
    "clg_fc_backward_w": (_i, [_i, _p, _p, _p, _p, _p, _i64, _i64, _i64, _p]),
    "clg_fc_backward_logits": (_i, [_i, _p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _p]),
    "clg_fc_fold": (_i, [_i, _i, _p, _p, _p, _i64, _p]),
    "clg_fc_forward_folded": (_i, [_i, _p, _p, _p, _p, _p, _i64, _i64, _i64, _p]),
    "clg_fc_backward_x_folded": (_i, [_i, _p, _p, _p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _p]),
    "clg_fc_backward_sole": (_i, [_i, _p, _p, _p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _p]),
    "clg_fc_backward_sole_classes": (_i, [_i, _p, _p, _p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _f64, _p]),
    "clg_fc_forward_logits": (_i, [_i, _p, _p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _p]),
    "clg_fc_backward_fused_fits": (_i, [_i, _i64]),
    "clg_fc_backward_fused": (_i, [_i, _p, _p, _p, _p, _p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _p]),
    "clg_fc_backward_fused_ex": (_i, [_i, _p, _p, _p, _p, _p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _i, _p, _p]),
    "clg_fc_forward_logits_ex": (_i, [_i, _p, _p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _i, _p, _p]),
    "clg_fold_many": (_i, [_i, _i, _p, _p, _p, _p, _p]),
    "clg_group_sum_scratch_bytes": (_i64, [_i, _i64, _i64, _i64]),
    "clg_group_sum": (_i, [_i, _p, _p, _p, _i64, _i64, _i64, _f64, _p]),
    "clg_group_sum_once_fits": (_i, [_i64, _i64, _i64]),
    "clg_group_sum_once": (_i, [_i, _p, _p, _i64, _i64, _i64, _f64, _p]),
    "clg_group_sum_static_max_bytes": (_i64, []),
    "clg_group_sum_static_init": (_i, []),
    "clg_group_sum_static": (_i, [_i, _p, _p, _i64, _i64, _i64, _f64, _p]),
    "clg_group_sum_backward": (_i, [_i, _p, _p, _i64, _i64, _i64, _f64, _p]),
    "clg_fc_backward_x": (_i, [_i, _p, _p, _p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _p]),
    "clg_transpose_2d": (_i, [_i, _p, _p, _i64, _i64, _p]),
    "clg_pack_bits": (_i, [_p, _p, _i64, _i64, _i, _p]),
    "clg_pack_bits_sample_major": (_i, [_p, _p, _i64, _i64, _i, _p]),
    "clg_fc_eval_packed": (_i, [_i, _p, _p, _p, _p, _p, _i64, _i64, _i64, _p]),
    "clg_fc_eval_plan": (_i, [_p, _p, _i64, _i64, _p]),
    "clg_fc_eval_packed_planned": (_i, [_i, _p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _p]),
    "clg_fc_eval_walk_fits": (_i, [_i, _p, _p, _i64]),
    "clg_fc_eval_packed_planned_logits": (_i, [_i, _p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _p]),
    "clg_group_bit_sum": (_i, [_i, _p, _p, _i64, _i64, _i64, _i64, _p]),
    "clg_conv4_forward": (_i, [_i, _GP, _p, _p, _p, _p, _p]),
    "clg_conv4_backward_x": (_i, [_i, _GP, _p, _p, _p, _p, _p, _p]),
    "clg_conv4_backward_w": (_i, [_i, _GP, _p, _p, _p, _p, _p, _p]),
    "clg_conv4_backward_w_scratch_bytes": (_i64, [_i, _GP]),
    "clg_tree_forward": (_i, [_i, _p, _p, _p, _i64, _i64, _i64, _i64, _p]),
    "clg_tree_backward_x": (_i, [_i, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _p]),
    "clg_tree_backward_w": (_i, [_i, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _p]),
    "clg_tree_backward_w_scratch_bytes": (_i64, [_i, _i64, _i64, _i64, _i64]),
    "clg_convblock_forward": (_i, [_i, _GP, _p, _p, _p, _p, _p, _p]),
    "clg_threshold_images": (_i, [_p, _p, _p, _i64, _i64, _i64, _i64, _p]),
    "clg_threshold_pack_images": (_i, [_p, _p, _p, _i64, _i64, _i64, _i64, _p]),
    "clg_convblock_eval_packed": (_i, [_GP, _p, _p, _p, _p, _p]),
    "clg_convblock_eval_packed_ws": (_i, [_GP, _p, _p, _p, _p, _p, _p]),
    "clg_convblock_eval_packed_scratch_bytes": (_i64, [_GP]),
    "clg_convblock_forward_ws": (_i, [_i, _GP, _p, _p, _p, _p, _p, _p, _p]),
    "clg_convblock_forward_scratch_bytes": (_i64, [_i, _GP]),
    "clg_convblock_intermediates": (_i, [_i, _GP, _p, _p, _p, _p, _p, _p]),
    "clg_convblock_backward_x": (_i, [_i, _GP, _p, _p, _p, _p, _p, _p, _p, _p]),
    "clg_convblock_backward_x_scratch_bytes": (_i64, [_i, _GP]),
    "clg_convblock_backward_w": (_i, [_i, _GP, _p, _p, _p, _p, _p, _p, _p, _p]),
    "clg_convblock_backward_w_scratch_bytes": (_i64, [_i, _GP]),
    "clg_convblock_backward": (_i, [_i, _GP, _p, _p, _p, _p, _p, _p, _p, _p, _p]),
    "clg_convblock_backward_logits": (_i, [_i, _GP, _p, _p, _p, _p, _p, _p, _p, _p, _p]),
    "clg_convblock_fm_supported": (_i, [_i, _GP]),
    "clg_convblock_forward_ex": (_i, [_i, _GP, _p, _p, _p, _p, _p, _p, _i, _p, _p]),
    "clg_convblock_padded_elems": (_i64, [_i, _GP, _i]),
    "clg_convblock_forward_padded": (_i, [_i, _GP, _p, _p, _p, _p, _p, _p, _i, _p, _p, _p]),
    "clg_convblock_eval_packed_fm_supported": (_i, [_GP]),
    "clg_convblock_eval_packed_fm": (_i, [_GP, _p, _p, _p, _p, _p]),
    "clg_convblock_forward_fm": (_i, [_i, _GP, _p, _p, _p, _p, _p, _p, _p]),
    "clg_convblock_backward_fm": (_i, [_i, _GP, _p, _p, _p, _p, _p, _p, _p, _i, _p, _p]),
    "clg_convblock_backward_scratch_bytes": (_i64, [_i, _GP]),
    "clg_convblock_plan_bytes": (_i64, [_i, _GP]),
    "clg_convblock_plan": (_i, [_i, _GP, _p, _p, _p, _p]),
    "clg_convblock_backward_planned": (_i, [_i, _GP, _p, _p, _p, _p, _p, _p, _p, _i64, _p, _p, _i, _p, _p]),
    "clg_convblock_backward_planned_padded": (_i, [_i, _GP, _p, _p, _p, _p, _p, _p, _p, _p, _i64, _p, _p, _i, _p, _p]),
    "clg_convblock_bin_supported": (_i, [_i, _GP]),
    "clg_convblock_bin_ctx_bytes": (_i64, [_i, _GP]),
    "clg_convblock_bin_forward": (_i, [_i, _GP, _p, _p, _p, _p, _p, _p, _i, _p, _p]),
    "clg_convblock_bin_backward_scratch_bytes": (_i64, [_i, _GP]),
    "clg_convblock_bin_backward": (_i, [_i, _GP, _p, _p, _p, _p, _p, _i, _p, _p]),
    "clg_host_flag_device_pointer": (_i, [_p, _p]),
}

_lib = None


def load():
    """Loads the shared library and declares all signatures (no GPU needed for this)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"convlogic_amd: {LIB_PATH} is missing. Build it with `python -m convlogic_amd.build` "
                "(needs hipcc); there is no fallback for the 'cuda' implementation.")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib


def available():
    return os.path.exists(LIB_PATH)


_knob_generation = 0


def reload_knobs():
    """Makes the library read its CLG_* environment knobs again (it reads them once per process) and invalidates what
    was derived under the old values (the per-layer backward plans are keyed on knob_generation())."""
    global _knob_generation
    load().clg_reload_knobs()
    _knob_generation += 1


def knob_generation():
    return _knob_generation


def check(rc):
    if rc != 0:
        raise RuntimeError(load().clg_last_error().decode())


def dtype_code(t, half_ok=False):
    try:
        return (_DTYPES_FC if half_ok else _DTYPES)[t.dtype]
    except KeyError:
        kinds = "float32, float64 and float16" if half_ok else "float32 and float64"
        raise RuntimeError(f"convlogic_amd: this kernel supports {kinds}, got {t.dtype}") from None


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_ptr(t):
    """hipStream_t of torch's current stream on the tensor's device, as an integer."""
    if _raw_stream is not None:
        return _raw_stream(t.device.index if t.device.index is not None else torch.cuda.current_device())
    return torch.cuda.current_stream(t.device).cuda_stream


def check_input(t, name, dtype=None, shape=None):
    """Same contract as the reference's CHECK_INPUT (src/common/cuda_utils.cuh:9-13); with dtype / shape also what its
    typed packed_accessor<scalar_t, N> arguments enforce: the kernels read raw pointers, so a tensor of another
    element type or size would be read out of bounds instead of raising."""
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor")
    if not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")
    if dtype is not None and t.dtype != dtype:
        raise RuntimeError(f"{name} must have dtype {dtype}, got {t.dtype}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise RuntimeError(f"{name} must have shape {tuple(shape)}, got {tuple(t.shape)}")
    return t


def check_same_device(ref, *tensors):
    for t in tensors:
        if t is not None and t.device != ref.device:
            raise RuntimeError(f"all tensors must be on one device, got {ref.device} and {t.device}")
