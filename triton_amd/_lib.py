"""ctypes binding of libtriton_amd.so (the C ABI declared in include/triton_amd.h).

There is no CPU fallback: if the library is missing or a call fails, this module
raises.  Tensors are torch allocations; the library only enqueues kernels on the
current HIP stream.
"""
import ctypes as C
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("TAMD_LIB") or os.path.join(_HERE, "libtriton_amd.so")  # TAMD_LIB: another build of the same ABI

# element type codes (include/triton_amd.h)
F32, F16, BF16, FP8_E4M3, FP8_E5M2, MXFP4 = 0, 1, 2, 3, 4, 5
ACT_NONE, ACT_SWIGLU = 0, 1
SCALE_STRIDED, SCALE_CDNA4 = 0, 1
W_STRIDED, W_CDNA4_BLOCKS = 0, 1
E_INVALID, E_UNSUPPORTED, E_ALIGNMENT, E_TOO_LARGE = -1, -2, -3, -4

_TORCH_CODE = {
    torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16,
    torch.float8_e4m3fn: FP8_E4M3, torch.float8_e5m2: FP8_E5M2,
}


def dtype_code(dt: torch.dtype) -> int:
    try:
        return _TORCH_CODE[dt]
    except KeyError:
        raise NotImplementedError(f"dtype {dt} is not supported by the gfx950 kernels") from None


class MatmulArgs(C.Structure):
    """Mirror of `tamd_matmul_args`."""
    _fields_ = [
        ("x", C.c_void_p), ("x_dtype", C.c_int), ("x_stride_m", C.c_int64), ("x_scale", C.c_void_p),
        ("w", C.c_void_p), ("w_dtype", C.c_int),
        ("w_stride_e", C.c_int64), ("w_stride_k", C.c_int64), ("w_stride_n", C.c_int64),
        ("w_scale", C.c_void_p), ("w_mx_scale", C.c_void_p),
        ("w_mx_stride_e", C.c_int64), ("w_mx_stride_k", C.c_int64), ("w_mx_stride_n", C.c_int64),
        ("bias", C.c_void_p), ("bias_dtype", C.c_int), ("bias_stride_e", C.c_int64),
        ("betas", C.c_void_p), ("gammas", C.c_void_p), ("out_alpha", C.c_float),
        ("y", C.c_void_p), ("y_dtype", C.c_int), ("y_stride_m", C.c_int64),
        ("M", C.c_int), ("N", C.c_int), ("K", C.c_int), ("n_experts", C.c_int),
        ("gather_indx", C.c_void_p), ("scatter_indx", C.c_void_p),
        ("slice_sizes", C.c_void_p), ("slice_offs", C.c_void_p),
        ("block_offs", C.c_void_p), ("block_schedule", C.c_void_p),
        ("block_m", C.c_int), ("grid_m", C.c_int),
        ("x_stride_z", C.c_int64), ("y_stride_z", C.c_int64),
        ("activation", C.c_int), ("act_alpha", C.c_float), ("act_limit", C.c_float), ("act_has_limit", C.c_int),
        ("force_variant", C.c_int), ("x_rows", C.c_int64),
        ("y_expected_scale", C.c_void_p), ("y_actual_scale", C.c_void_p), ("y_saturate_inf", C.c_int),
        ("w_mx_layout", C.c_int),
        ("x_mx_scale", C.c_void_p), ("x_mx_stride_m", C.c_int64), ("x_mx_stride_z", C.c_int64),
        ("y_mx_scale", C.c_void_p), ("y_mx_stride_m", C.c_int64), ("y_mx_stride_z", C.c_int64),
        ("w_layout", C.c_int),
    ]


class MatmulArgBag:
    """Plain attribute bag with the fields of `tamd_matmul_args` (all zero / NULL until set): the host code of
    `matmul` fills it like the ctypes structure, and `pack()` turns it into one in a single struct.pack call --
    a third of the time of fifty ctypes field stores."""
    _names = tuple(n for n, _ in MatmulArgs._fields_)
    _get = None
    _struct = None

    def pack(self):
        cls = MatmulArgBag
        if cls._struct is None:
            import operator
            import struct
            code = {C.c_void_p: "P", C.c_int: "i", C.c_int64: "q", C.c_float: "f"}
            cls._struct = struct.Struct("@" + "".join(code[t] for _, t in MatmulArgs._fields_) + "0P")
            assert cls._struct.size == C.sizeof(MatmulArgs)
            cls._get = operator.attrgetter(*cls._names)
        return MatmulArgs.from_buffer_copy(cls._struct.pack(*[v or 0 for v in cls._get(self)]))


for _n in MatmulArgBag._names:
    setattr(MatmulArgBag, _n, 0)


class ReduceArgs(C.Structure):
    """Mirror of `tamd_reduce_args`."""
    _fields_ = [
        ("x", C.c_void_p), ("x_dtype", C.c_int), ("S0", C.c_int64), ("R", C.c_int64), ("S1", C.c_int64),
        ("xs0", C.c_int64), ("xsr", C.c_int64), ("xs1", C.c_int64),
        ("x_mx_scale", C.c_void_p), ("xms0", C.c_int64), ("xmsr", C.c_int64), ("xms1", C.c_int64),
        ("x_flex_scale", C.c_void_p), ("x_global_scale", C.c_void_p),
        ("mask", C.c_void_p), ("ms0", C.c_int64), ("msr", C.c_int64), ("ms1", C.c_int64),
        ("scale", C.c_void_p), ("ss0", C.c_int64), ("ssr", C.c_int64), ("ss1", C.c_int64),
        ("postprocess", C.c_int), ("pp_arg0", C.c_float), ("pp_arg1", C.c_float), ("pp_has_arg1", C.c_int),
        ("y", C.c_void_p), ("y_dtype", C.c_int), ("ys0", C.c_int64), ("ys1", C.c_int64),
        ("y_expected_scale", C.c_void_p), ("y_actual_scale", C.c_void_p), ("y_saturate_inf", C.c_int),
        ("y_mx_scale", C.c_void_p), ("yms0", C.c_int64), ("yms1", C.c_int64),
        ("unpadded_batch_size", C.c_void_p),
    ]


PP_NONE, PP_SWIGLU, PP_PLUS_A_PAIRSUM = 0, 1, 2

_I64, _INT, _PTR, _F = C.c_int64, C.c_int, C.c_void_p, C.c_float
_SIGNATURES = {
    "tamd_version": ([], C.c_int),
    "tamd_error_string": ([_INT], C.c_char_p),
    "tamd_downcast_mxfp": ([_PTR, _INT, _I64, _I64, _I64, _I64, _I64, _I64, _PTR, _INT, _I64, _I64, _PTR, _I64, _I64,
                            _INT, _PTR], C.c_int),
    "tamd_upcast_mxfp": ([_PTR, _INT, _I64, _I64, _PTR, _I64, _I64, _PTR, _INT, _I64, _I64, _I64, _I64, _I64, _I64,
                          _PTR], C.c_int),
    "tamd_widen_mxfp4_rows": ([_PTR, _I64, _I64, _I64, _PTR, _I64, _PTR], C.c_int),
    "tamd_topk_forward": ([_PTR, _INT, _I64, _INT, _INT, _INT, _INT, _INT, _PTR, _PTR, _I64, _PTR, _I64, _I64, _PTR],
                          C.c_int),
    "tamd_bitmatrix_metadata_workspace": ([_I64, _INT], C.c_int64),
    "tamd_bitmatrix_metadata": ([_PTR, _INT, _I64, _INT, _PTR, _PTR, _PTR, _PTR, _PTR], C.c_int),
    "tamd_ragged_metadata": ([_PTR, _INT, _PTR, _I64, _PTR, _I64, _INT, _PTR], C.c_int),
    "tamd_routing_metadata": ([_PTR, _INT, _I64, _INT, _INT, _PTR, _PTR, _PTR, _PTR, _PTR, _I64, _PTR, _I64, _INT,
                               _PTR, _PTR], C.c_int),
    "tamd_routing_metadata_static_init": ([], C.c_int),
    "tamd_routing_metadata_static_max_workspace": ([], C.c_int64),
    "tamd_routing_metadata_static": ([_PTR, _INT, _I64, _INT, _INT, _PTR, _PTR, _PTR, _PTR, _PTR, _I64, _PTR, _I64,
                                      _INT, _PTR], C.c_int),
    "tamd_routing": ([_PTR, _INT, _I64, _INT, _INT, _INT, _PTR, _PTR, _PTR, _I64, _I64, _PTR, _PTR, _PTR, _PTR, _PTR,
                      _I64, _PTR, _I64, _INT, _PTR, _PTR], C.c_int),
    "tamd_matmul": ([C.POINTER(MatmulArgs), _PTR], C.c_int),
    "tamd_reduce": ([_PTR, _INT, _I64, _I64, _I64, _I64, _I64, _I64, _PTR, _I64, _I64, _I64, _PTR, _I64, _I64, _I64,
                     _PTR, _INT, _I64, _I64, _PTR], C.c_int),
    "tamd_reduce_ex": ([C.POINTER(ReduceArgs), _PTR], C.c_int),
    "tamd_swiglu": ([_PTR, _INT, _I64, _I64, _I64, _PTR, _I64, _F, _F, _INT, _PTR], C.c_int),
}

EXPORTS = tuple(_SIGNATURES)
_lib = None


def lib():
    """Loads the shared library on first use; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: build it with `python -m triton_amd.build` "
                               "(there is no CPU fallback)")
        handle = C.CDLL(LIB_PATH)
        for name, (argtypes, restype) in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.argtypes = argtypes
            fn.restype = restype
        _lib = handle
    return _lib


def check(rc: int, what: str):
    """Maps a C ABI return code to the exception the reference raises for the same misuse."""
    if rc == 0:
        return
    msg = f"{what}: {lib().tamd_error_string(rc).decode()} (code {rc})"
    if rc == E_UNSUPPORTED:
        raise NotImplementedError(msg)
    if rc in (E_INVALID, E_ALIGNMENT, E_TOO_LARGE):
        raise ValueError(msg)
    raise RuntimeError(msg)


def ptr(t):
    return None if t is None else C.c_void_p(t.data_ptr())


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_ptr(device=None):
    """The current HIP stream of `device` as a void*.  torch's raw-stream accessor when it is there (a tenth of the
    time of building a torch.cuda.Stream object per call)."""
    if _raw_stream is not None:
        idx = device.index if isinstance(device, torch.device) else device
        if idx is None:
            idx = torch.cuda.current_device()
        return C.c_void_p(_raw_stream(idx))
    return C.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def require_gpu(t: torch.Tensor, name: str):
    if not t.is_cuda:
        raise RuntimeError(f"{name} must live on the GPU: the gfx950 kernels have no CPU path")
