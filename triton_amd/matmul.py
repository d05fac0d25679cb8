"""`matmul` (alias `matmul_ogs`): gather -> grouped / dense GEMM -> bias, fused
activation, gamma -> scatter (matmul.py:243-749 of the reference), over the
gfx950 kernels.  Argument names, defaults and error behaviour follow the
reference; combinations that are not built raise NotImplementedError."""
import ctypes
import math
import weakref
from dataclasses import dataclass
from typing import Callable, Optional

import torch

from . import _lib
from .matmul_details import opt_flags as _opt_flags
from .matmul_details.opt_flags import (InapplicableConstraint, OptFlags, make_opt_flags, scoped_opt_flags,
                                       scoped_opt_flags_constraints)
from .numerics import InFlexData, OutFlexData
from .specialize import FnSpecs
from .tensor import FP4, RaggedTensorMetadata, Tensor, wrap_torch_tensor
from .tensor_details.layout import CDNA4MXScaleLayout, CDNA4MXValueLayout

__all__ = ["matmul", "matmul_ogs", "PrecisionConfig", "FlexCtx", "FusedActivation", "Epilogue", "FnSpecs",
           "InFlexData", "OutFlexData", "InapplicableConstraint", "OptFlags", "scoped_opt_flags",
           "scoped_opt_flags_constraints"]

MXFP_BLOCK_SIZE = 32


@dataclass(frozen=True)
class FusedActivation:
    specs: FnSpecs = FnSpecs.default()
    fn_args: tuple = tuple()


@dataclass(frozen=True)
class Epilogue:
    specs: FnSpecs = FnSpecs.default()
    fn_arg_values_matmul: tuple = tuple()
    fn_arg_values_finalize: tuple = tuple()
    effective_itemsize: Optional[float] = None


@dataclass(frozen=True)
class FlexCtx:
    lhs_data: InFlexData = InFlexData()
    rhs_data: InFlexData = InFlexData()
    out_data: OutFlexData = OutFlexData()
    acc_data: InFlexData = InFlexData()


@dataclass
class PrecisionConfig:
    max_num_imprecise_acc: Optional[int] = None
    allow_tf32: bool = True
    flex_ctx: FlexCtx = FlexCtx()
    acc_scale: float = 1.0
    flexpoint_saturate_inf: bool = False
    report_quantization_err_fn: Optional[Callable] = None
    a_mx_scale: Optional[torch.Tensor] = None
    a_mx_tensor_scale: Optional[torch.Tensor] = None
    a_microblock_size: Optional[int] = None
    b_mx_scale: Optional[torch.Tensor] = None
    b_mx_tensor_scale: Optional[torch.Tensor] = None
    b_microblock_size: Optional[int] = None
    c_mx_scale: Optional[torch.Tensor] = None
    c_microblock_size: Optional[int] = None
    c_value_pack_factor: int = 1
    out_dtype: Optional[torch.dtype] = None
    intermediate_out_dtype: Optional[torch.dtype] = None
    enforce_bitwise_invariance: bool = False


# what `matmul` uses for arguments left out; never written to (c_microblock_size is only filled in for a caller's
# own config with c_mx_scale)
_DEFAULT_PRECISION = PrecisionConfig()
_DEFAULT_ACTIVATION = FusedActivation(FnSpecs.default(), tuple())
_DEFAULT_EPILOGUE = Epilogue(FnSpecs.default(), tuple(), tuple(), False)


def _data(t):
    return t.storage.data if isinstance(t, Tensor) else t


def _widen_mxfp4_activations(a_raw):
    """MXFP4 activations (packed e2m1 codes along K with one e8m0 byte per 32, matmul.py:131-136 of the reference)
    against MXFP4 weights: the codes are widened -- exactly: every e2m1 number is a float8_e4m3fn number -- and take
    the MXFP8 path of the kernels with the same scales."""
    _lib.require_gpu(a_raw, "a")
    assert a_raw.stride(-1) == 1, "packed activations must be contiguous along K"
    rows = a_raw.numel() // a_raw.shape[-1]
    src = a_raw if a_raw.is_contiguous() else a_raw.contiguous()
    out = torch.empty((*a_raw.shape[:-1], 2 * a_raw.shape[-1]), dtype=torch.float8_e4m3fn, device=a_raw.device)
    rc = _lib.lib().tamd_widen_mxfp4_rows(_lib.ptr(src), rows, src.shape[-1], src.shape[-1], _lib.ptr(out),
                                          out.shape[-1], _lib.stream_ptr(a_raw.device))
    _lib.check(rc, "matmul (MXFP4 activations)")
    return out


_TURNED = {}  # id(weights) -> (weak reference to them, their version counter, the copy with unit stride along K)


def _k_contiguous_cached(w):
    key = id(w)
    hit = _TURNED.get(key)
    if hit is not None and hit[0]() is w and hit[1] == w._version:
        return hit[2]
    turned = w.transpose(-1, -2).contiguous().transpose(-1, -2)
    if len(_TURNED) >= 64:
        _TURNED.clear()
    _TURNED[key] = (weakref.ref(w, lambda _, key=key: _TURNED.pop(key, None)), w._version, turned)
    return turned


def matmul(a, b, bias, a_ragged_metadata: Optional[RaggedTensorMetadata] = None,
           b_ragged_metadata: Optional[RaggedTensorMetadata] = None, gather_indx: Optional[torch.Tensor] = None,
           scatter_indx: Optional[torch.Tensor] = None, precision_config: Optional[PrecisionConfig] = None,
           betas: Optional[torch.Tensor] = None, gammas: Optional[torch.Tensor] = None,
           out_alpha: Optional[float] = None, c: Optional[torch.Tensor] = None, fused_comm=None,
           fused_activation: Optional[FusedActivation] = None, epilogue: Optional[Epilogue] = None,
           c_acc_in: Optional[torch.Tensor] = None):
    """
    Y[dst(r), :] = act((X[src(r), :] @ W[e]) + bias[e] * betas[r]) * gammas[r]   for the rows r of every slice e

    a: [M, K] activations (bf16 / fp16, or float8_e4m3fn / float8_e5m2 with flex_ctx.lhs_data.scale), or [B, M, K] batched.
    b: [E, K, N] weights; MXFP4 weights are uint8 with two codes per byte along K
       (storage [E, K/2, N] with unit stride along K) and precision_config.b_mx_scale
       holds their e8m0 scales [E, K/32, N].
    a_ragged_metadata: rows of `a` (after gather) are grouped by slice.
    gather_indx / scatter_indx: int32 row maps (scatter -1 drops the row).
    """
    if precision_config is None:
        precision_config = _DEFAULT_PRECISION
    if fused_activation is None:
        fused_activation = _DEFAULT_ACTIVATION
    if epilogue is None:
        epilogue = _DEFAULT_EPILOGUE
    is_input_batched = a.ndim == 3
    if is_input_batched:
        assert gather_indx is None, "gather not supported in batched mode"
        assert scatter_indx is None, "scatter not supported in batched mode"
        assert b_ragged_metadata is None, "w cannot be ragged in batched mode"
        assert a_ragged_metadata is None, "x cannot be ragged in batched mode"
        assert fused_comm is None, "fused comm is not supported in batched mode"
        assert b.ndim == 3 and b.shape[0] == a.shape[0]
    if b_ragged_metadata is not None:
        raise NotImplementedError("K-ragged matmul is not built for gfx950")
    if fused_comm is not None:
        raise NotImplementedError("fused communication needs more than one GPU")
    if c_acc_in is not None:
        raise NotImplementedError("accumulator input is not built")
    # quantising epilogue: MXFP8 (float8_e4m3fn values, e8m0 scale per 32 output columns), tests/test_matmul.py:547-561
    c_mx_scale = precision_config.c_mx_scale
    mx_out = c_mx_scale is not None
    if epilogue.specs.name.lower() not in ("dflt", "quantize_mxfp8") or (epilogue.specs.name != "dflt") != mx_out:
        raise NotImplementedError(f"epilogue {epilogue.specs.name!r} / c_mx_scale combination is not built (MXFP8 is)")
    if mx_out:
        c_mx_scale = _data(c_mx_scale)
        if c_mx_scale.dtype != torch.uint8 or (precision_config.c_microblock_size or MXFP_BLOCK_SIZE) != MXFP_BLOCK_SIZE:
            raise NotImplementedError("output scales are built as e8m0 bytes per 32 columns")
        if precision_config.c_value_pack_factor != 1:
            raise NotImplementedError("packed output values (c_value_pack_factor != 1) are not built")
        if precision_config.c_microblock_size is None:
            precision_config.c_microblock_size = MXFP_BLOCK_SIZE  # filled in for the caller, as matmul.py:362-363 does
    # fields that change the result and have no kernel here must not be dropped silently
    if precision_config.a_mx_tensor_scale is not None or precision_config.b_mx_tensor_scale is not None:
        raise NotImplementedError("per-tensor scales on top of microscales (NVFP4-style) are not built")
    if precision_config.acc_scale != 1.0:
        raise NotImplementedError("acc_scale other than 1.0 is not built")
    a_mx_scale = precision_config.a_mx_scale
    if a_mx_scale is not None:
        a_mx_scale = _data(a_mx_scale)
        a_raw = a.storage.data if isinstance(a, Tensor) else a
        a_fp4 = a_raw.dtype == torch.uint8 and (not isinstance(a, Tensor) or a.dtype == FP4)
        if not (a_fp4 or a_raw.dtype == torch.float8_e4m3fn) or a_mx_scale.dtype != torch.uint8:
            raise NotImplementedError("microscaled activations are built for float8_e4m3fn or packed e2m1 values "
                                      "with e8m0 scales")
        mb = precision_config.a_microblock_size
        assert mb is None or mb == MXFP_BLOCK_SIZE, "Unsupported microscale block size"
        b_raw = _data(b)
        b_packed = b.dtype == FP4 if isinstance(b, Tensor) else b_raw.dtype == torch.uint8
        if not (precision_config.b_mx_scale is not None and b_packed):
            # weights that are not MXFP4 (16-bit, or MXFP8, which is dequantised to bfloat16 below): the activations are
            # dequantised, as the reference's own reference path does (matmul.py:772-778) -- exactly, to the type the
            # product is computed in -- and take the kernel for 16-bit operands; no block scales are left
            from .numerics_details.mxfp import upcast_from_mxfp
            _lib.require_gpu(a_raw, "a")
            a = upcast_from_mxfp(a_raw, a_mx_scale, torch.float16 if b_raw.dtype == torch.float16 else torch.bfloat16,
                                 axis=-1)
            a_mx_scale = None
        elif a_fp4:
            a = _widen_mxfp4_activations(a_raw)
    flex = precision_config.flex_ctx
    if flex.acc_data.scale is not None:
        raise NotImplementedError("accumulator flex scale is not built")
    if flex.out_data.checksum_scale is not None:
        raise NotImplementedError("flexpoint checksum is not built")
    for sc in (flex.out_data.expected_scale, flex.out_data.actual_scale):
        if sc is not None and (sc.numel() != 1 or sc.dtype != torch.float32):
            raise NotImplementedError("per-batch flexpoint output scales are not built (one float32 value expected)")
    # ---- weights
    b_scale = precision_config.b_mx_scale
    # weights: storage tensor, whether they are packed e2m1 codes, logical shape (a packed axis counts twice)
    b_blocks = isinstance(b, Tensor) and isinstance(b.storage.layout, CDNA4MXValueLayout)  # the kernels' own value layout
    if isinstance(b, Tensor):
        b_data, b_fp4, b_shape = b.storage.data, b.dtype == FP4, list(b.shape)
    else:
        b_data, b_fp4, b_shape = b, b.dtype == torch.uint8, list(b.shape)
        if b_fp4:
            b_shape[b.stride().index(1)] *= 2
    if b_scale is not None:
        assert precision_config.b_microblock_size is not None, \
            "precision_config.b_microblock_size is required when precision_config.b_mx_scale is set"
        assert precision_config.b_microblock_size == MXFP_BLOCK_SIZE, "Unsupported microscale block size"
        b_scale_cdna4 = isinstance(b_scale, Tensor) and isinstance(b_scale.storage.layout, CDNA4MXScaleLayout)
        b_scale_shape = list(b_scale.shape)
        b_scale = _data(b_scale)
        assert b_scale.dtype == torch.uint8, f"Unsupported microscale dtype {b_scale.dtype}"
    if isinstance(a, Tensor):
        a = a.storage.data
    if b_scale is not None and not b_fp4:
        # MXFP8 weights: dequantised to bfloat16 by the library's upcast kernel, as the reference's torch path does
        # (matmul.py:788-794), and multiplied by the kernel for unquantised weights
        w8 = b_data
        if w8.dtype not in (torch.float8_e4m3fn, torch.float8_e5m2) or b_scale_cdna4:
            raise NotImplementedError("microscaled weights are built as MXFP4, or MXFP8 with scales in the strided layout")
        if a.dtype != torch.bfloat16:
            raise NotImplementedError("MXFP8 weights are built for bfloat16 or microscaled activations")
        from .numerics_details.mxfp import upcast_from_mxfp
        b_data = upcast_from_mxfp(w8, b_scale, torch.bfloat16, axis=-2)
        b_shape = list(b_data.shape)
        b_scale = None
    a = flex.lhs_data.reinterpret(a)
    w = flex.rhs_data.reinterpret(b_data)
    a_dtype = a.dtype  # the type the output defaults to
    fp8_types = (torch.float8_e4m3fn, torch.float8_e5m2)
    if not b_fp4 and w.dtype in fp8_types and a.dtype in fp8_types and a_mx_scale is None:
        # fp8 x fp8 with per-tensor scales (tests/test_matmul.py:150-154 of the reference): every fp8 number is a
        # bfloat16 number, so both operands are widened (exactly) and multiplied by the kernel for 16-bit weights; the
        # flex scales enter in its epilogue as they do for any other pair of types
        a, w = a.to(torch.bfloat16), w.to(torch.bfloat16)
    if not b_fp4 and w.stride(-1) == 1 and (w.shape[-1] * w.element_size()) % 16 != 0 \
            and (w.shape[-2] * w.element_size()) % 16 == 0:
        # unquantised weights with unit stride along N whose rows do not start on 16-byte boundaries: the kernel copies
        # 16 bytes at a time, so they are laid out with unit stride along K instead (same values)
        w = w.transpose(-1, -2).contiguous().transpose(-1, -2)
    if not b_fp4 and w.ndim == 2 and w.shape[-1] <= 128 and w.stride(-2) != 1 and w.shape[-2] % 8 == 0 \
            and a_ragged_metadata is None and gather_indx is None and scatter_indx is None:
        # a narrow dense product (the gate matmul: hidden -> expert logits): the kernel for it reads both operands
        # along K, so weights stored with unit stride along N are turned (a few hundred KB); the turned copy is kept
        # for as long as the caller's tensor lives and is not written to, so a layer that holds N-contiguous gate
        # weights pays for the copy once
        w = _k_contiguous_cached(w)
    _lib.require_gpu(a, "a")
    _lib.require_gpu(w, "b")
    assert a.stride(-1) == 1 or a.shape[-1] == 1, "a must be contiguous along K"
    # ---- shapes
    K = a.shape[-1]
    K_W, N = b_shape[-2:]
    assert K == K_W, f"inner dimensions differ: {K} vs {K_W}"
    ragged = a_ragged_metadata is not None
    M = a.shape[-2] if gather_indx is None else gather_indx.shape[0]
    if ragged:
        n_slices, batch = a_ragged_metadata.n_slices, 1
    elif len(b_shape) == 3:
        n_slices = batch = b_shape[0]
    else:
        n_slices = batch = 1
    red_n = fused_activation.specs.reduction_n
    # microscaled activations stand for bf16 numbers (the reference dequantises them to bf16, matmul.py:772-778)
    out_dtype = precision_config.out_dtype or (torch.bfloat16 if precision_config.a_mx_scale is not None else a_dtype)
    if mx_out:
        out_dtype = precision_config.out_dtype or (c.dtype if c is not None else torch.float8_e4m3fn)
        if out_dtype != torch.float8_e4m3fn:
            raise NotImplementedError("MXFP8 output needs float8_e4m3fn values")
        if flex.out_data.expected_scale is not None or flex.out_data.actual_scale is not None:
            raise NotImplementedError("flexpoint output scales together with MX output scales are not built")
    if out_dtype.itemsize == 1 and out_dtype not in (torch.float8_e4m3fn, torch.float8_e5m2):
        raise NotImplementedError(f"{out_dtype} outputs are not built (float8_e4m3fn and float8_e5m2 are)")
    rows_out = M
    if gather_indx is not None:
        rows_out = gather_indx.shape[0]
    if scatter_indx is not None:
        rows_out = scatter_indx.shape[0]
    out_shape = (batch, rows_out, N // red_n)
    if c is None:
        out = torch.empty(out_shape, dtype=out_dtype, device=a.device)
    else:
        out = c[None] if c.ndim == 2 else c
        assert tuple(out.shape) == out_shape, f"output shape {tuple(out.shape)} != {out_shape}"
        assert out.stride(-1) == 1
    squeeze = not is_input_batched

    def finish():
        return out.squeeze(0) if squeeze else out

    if batch * M * N == 0:
        return finish()
    # ---- activation
    act, act_alpha, act_limit, has_limit = _lib.ACT_NONE, 0.0, 0.0, 0
    if fused_activation.specs.name == "swiglu":
        assert red_n == 2
        named = dict(zip(fused_activation.specs.fn_arg_names, fused_activation.fn_args))
        act = _lib.ACT_SWIGLU
        act_alpha = float(named.get("alpha", fused_activation.fn_args[0]))
        limit = named.get("limit", fused_activation.fn_args[1] if len(fused_activation.fn_args) > 1 else None)
        has_limit = int(limit is not None)
        act_limit = float(limit) if limit is not None else 0.0
    elif fused_activation.specs.name != "dflt":
        raise NotImplementedError(f"fused activation {fused_activation.specs.name!r} is not built")
    # ---- tile choice
    flags = make_opt_flags(M, N, K, n_slices, ragged,
                           a_ragged_metadata.expected_slice_size if ragged else None,
                           fp8_rows=a.dtype in fp8_types and b_fp4)
    args = _lib.MatmulArgBag()
    args.x, args.x_dtype = a.data_ptr(), _lib.dtype_code(a.dtype)
    args.x_stride_m = a.stride(-2)
    args.x_stride_z = a.stride(0) if a.ndim == 3 else 0
    args.x_scale = None if flex.lhs_data.scale is None else flex.lhs_data.scale.data_ptr()
    if a_mx_scale is not None:
        want = (*a.shape[:-1], K // MXFP_BLOCK_SIZE)
        assert tuple(a_mx_scale.shape) == want, f"a_mx_scale shape {tuple(a_mx_scale.shape)} != {want}"
        assert a_mx_scale.stride(-1) == 1 or a_mx_scale.shape[-1] == 1, "a_mx_scale must be contiguous along K"
        args.x_mx_scale = a_mx_scale.data_ptr()
        args.x_mx_stride_m = a_mx_scale.stride(-2)
        args.x_mx_stride_z = a_mx_scale.stride(0) if a_mx_scale.ndim == 3 else 0
    if b_blocks:
        # storage [B, ceil(N/64), ceil(K/128) * 4096]: strips of 4 KB blocks, one matrix after the other
        assert b_fp4 and w.ndim == 3 and w.is_contiguous(), "block-layout weights are packed e2m1 codes"
        want_b = math.prod(b_shape[:-2])
        assert list(w.shape) == CDNA4MXValueLayout().storage_shape([want_b, K_W, N]), \
            f"storage {tuple(w.shape)} does not match the block layout of weights {b_shape}"
        args.w_layout = _lib.W_CDNA4_BLOCKS
        wd = w
    else:
        wd = w if w.ndim == 3 else w[None]
    args.w = wd.data_ptr()
    if b_fp4:
        assert b_scale is not None, "MXFP4 weights need precision_config.b_mx_scale"
        args.w_dtype = _lib.MXFP4
        want = [wd.shape[0], K // MXFP_BLOCK_SIZE, N]
        if b_scale_cdna4:
            # pre-shuffled storage [E, K_SCALE_pad * 32, N_pad / 32], block after block in memory
            assert b_scale_shape[-2:] == want[-2:] and math.prod(b_scale_shape[:-2]) == want[0], \
                f"b_mx_scale shape {b_scale_shape} != {want}"
            assert list(b_scale.shape) == CDNA4MXScaleLayout().storage_shape(want) and \
                (b_scale.numel() == 0 or (b_scale.stride(1) == 1 and b_scale.stride(2) == b_scale.shape[1])), \
                "b_mx_scale storage does not match the CDNA4 scale layout"
            args.w_mx_scale = b_scale.data_ptr()
            args.w_mx_layout = _lib.SCALE_CDNA4
            args.w_mx_stride_e, args.w_mx_stride_k, args.w_mx_stride_n = b_scale.stride(0), 0, 0
        else:
            sd = b_scale if b_scale.ndim == 3 else b_scale[None]
            assert list(sd.shape) == want, f"b_mx_scale shape {tuple(sd.shape)} != {tuple(want)}"
            args.w_mx_scale = sd.data_ptr()
            args.w_mx_stride_e, args.w_mx_stride_k, args.w_mx_stride_n = sd.stride()
    else:
        args.w_dtype = _lib.dtype_code(w.dtype)
    if b_blocks:
        args.w_stride_e, args.w_stride_k, args.w_stride_n = wd.stride(0), 1, 0
    else:
        args.w_stride_e, args.w_stride_k, args.w_stride_n = wd.stride()
    args.w_scale = None if flex.rhs_data.scale is None else flex.rhs_data.scale.data_ptr()
    if bias is not None:
        bb = bias if bias.ndim == 2 else bias[None]
        assert bb.stride(-1) == 1 and bb.shape[-1] == N
        args.bias, args.bias_dtype, args.bias_stride_e = bb.data_ptr(), _lib.dtype_code(bb.dtype), bb.stride(0)
    keep = []  # temporaries that must outlive the launch call

    def f32(t):
        if t is None:
            return None
        t = t if t.dtype == torch.float32 and t.is_contiguous() else t.to(torch.float32).contiguous()
        keep.append(t)
        return t.data_ptr()

    def i32(t):
        if t is None:
            return None
        t = t if t.dtype == torch.int32 and t.is_contiguous() else t.to(torch.int32).contiguous()
        keep.append(t)
        return t.data_ptr()

    args.betas, args.gammas = f32(betas), f32(gammas)
    args.out_alpha = 1.0 if out_alpha is None else float(out_alpha)
    args.y, args.y_dtype = out.data_ptr(), _lib.dtype_code(out.dtype)
    args.y_stride_m, args.y_stride_z = out.stride(1), out.stride(0)
    args.M, args.N, args.K, args.n_experts = M, N, K, n_slices
    args.x_rows = a.shape[-2]
    if flex.out_data.expected_scale is not None:
        args.y_expected_scale = flex.out_data.expected_scale.data_ptr()
    if flex.out_data.actual_scale is not None:
        args.y_actual_scale = flex.out_data.actual_scale.data_ptr()
    args.y_saturate_inf = int(precision_config.flexpoint_saturate_inf)
    if mx_out:
        n_groups = -(-(N // red_n) // MXFP_BLOCK_SIZE)
        cs = c_mx_scale if c_mx_scale.ndim == 3 else c_mx_scale[None]
        assert tuple(cs.shape) == (batch, rows_out, n_groups), \
            f"c_mx_scale shape {tuple(c_mx_scale.shape)} != {(rows_out, n_groups)}"
        assert cs.stride(-1) == 1 or cs.shape[-1] == 1, "c_mx_scale must be contiguous along its last axis"
        args.y_mx_scale, args.y_mx_stride_m, args.y_mx_stride_z = cs.data_ptr(), cs.stride(1), cs.stride(0)
    args.gather_indx, args.scatter_indx = i32(gather_indx), i32(scatter_indx)
    if ragged:
        md = a_ragged_metadata
        args.slice_sizes, args.slice_offs = md.slice_sizes.data_ptr(), md.slice_offs.data_ptr()
        args.block_offs = md.block_offs(flags.block_m).data_ptr()
        args.block_schedule = md.block_schedule(flags.block_m).data_ptr()
        args.block_m = flags.block_m
        args.grid_m = RaggedTensorMetadata.n_blocks(md.n_slices, M, flags.block_m)
        # the kernels read up to grid_m entries of the schedule: metadata made for fewer rows than the matmul has is a
        # caller's mistake that must not become a read past the table
        if args.grid_m > md.block_schedule(flags.block_m).shape[-1]:
            raise ValueError(f"a_ragged_metadata was made for fewer rows than the matmul has ({M}): its block schedule "
                             f"holds {md.block_schedule(flags.block_m).shape[-1]} entries, {args.grid_m} are needed")
    else:
        args.force_variant = flags.block_m if "block_m" in _opt_flags._constraints() else 0
    args.activation, args.act_alpha, args.act_limit, args.act_has_limit = act, act_alpha, act_limit, has_limit
    split_k = flags.split_k
    if (split_k == 1 and _opt_flags._constraints().get("split_k") is None and _opt_flags._opt_flags.get() is None
            and not ragged and batch == 1 and M <= 256 and K >= 8192 and scatter_indx is None and not mx_out
            and not args.y_expected_scale and not args.y_actual_scale and out.dtype.itemsize > 1
            and args.w_mx_layout != _lib.SCALE_CDNA4 and not b_blocks):
        # few rows and a long K: a tile's K loop is bound by the latency of its stages and there are too few
        # tiles to hide it, so the ranges of a split run side by side (16 x 16384 x 512: 144 us -> 50 us)
        split_k = next((s for s in (8, 4, 2) if K % (s * 128) == 0 and K // s >= 1024), 1)
    if split_k > 1:
        flags = OptFlags(block_m=flags.block_m, split_k=split_k)
        _matmul_split_k(args.pack(), flags.split_k, a, wd, b_fp4, out, fused_activation, bias, flex.out_data,
                        precision_config.flexpoint_saturate_inf)
        return finish()
    rc = _lib.lib().tamd_matmul(ctypes.byref(args.pack()), _lib.stream_ptr(a.device))
    _lib.check(rc, "matmul")
    return finish()


def _matmul_split_k(args, split_k, a, wd, w_is_fp4, out, fused_activation, bias, out_flex, saturate_inf):
    """K cut into `split_k` ranges (whole multiples of 128) whose float32 partial results [split_k, B, M, N] are
    summed afterwards (matmul.py:180-183, 471-472, 711-737 of the reference).  Every range applies the scales,
    betas, out_alpha and gammas (all linear), only the first adds the bias (_matmul.py:523-528), and the
    activation runs after the sum.

    A plain [M, K] x [K, N] problem whose K divides evenly runs its ranges as the entries of one batched launch
    (range s = batch entry s: activations, weights and scales advanced by s ranges, a bias that is zero for
    s > 0), so that they share the machine; anything else gets one launch per range."""
    from .reduce import reduce
    if args.scatter_indx or args.y_mx_scale:
        raise InapplicableConstraint("split_k cannot be combined with a scatter or a microscaled output")
    if args.w_mx_layout == _lib.SCALE_CDNA4 or args.w_layout == _lib.W_CDNA4_BLOCKS:
        raise InapplicableConstraint("split_k needs weights and weight scales in the strided layouts")
    K, N = args.K, args.N
    if not w_is_fp4 and K % 64 != 0:
        # the kernel for 16-bit weights bounds its K tail by the end of the expert's weights, which a range
        # that starts inside them would move
        raise InapplicableConstraint("split_k with 16-bit weights needs K to be a multiple of 64")
    align = 128 if w_is_fp4 else 64  # whole stages of the kernel that runs the ranges
    chunk = -(-(-(-K // split_k)) // align) * align
    n_split = -(-K // chunk)
    batch, rows = out.shape[0], out.shape[1]
    scratch = torch.empty((n_split, batch, rows, N), dtype=torch.float32, device=out.device)
    w_esz = 1 if w_is_fp4 else wd.element_size()
    one_launch = args.n_experts == 1 and not args.block_schedule and batch == 1 and K % chunk == 0
    if one_launch:
        kq = chunk // 2 if w_is_fp4 else chunk
        part = type(args).from_buffer_copy(args)
        part.K, part.n_experts = chunk, n_split
        part.x_stride_z = chunk
        part.w_stride_e = kq * args.w_stride_k
        if args.w_mx_scale:
            part.w_mx_stride_e = (chunk // MXFP_BLOCK_SIZE) * args.w_mx_stride_k
        if args.x_mx_scale:
            part.x_mx_stride_z = chunk // MXFP_BLOCK_SIZE
        if bias is not None:
            bias_s = torch.zeros((n_split, N), dtype=torch.float32, device=out.device)
            bias_s[0] = bias.reshape(-1)
            part.bias, part.bias_dtype, part.bias_stride_e = bias_s.data_ptr(), _lib.F32, N
        part.activation = _lib.ACT_NONE
        part.y, part.y_dtype = scratch.data_ptr(), _lib.F32
        part.y_stride_m, part.y_stride_z = scratch.stride(2), scratch.stride(0)
        part.y_expected_scale = part.y_actual_scale = None
        part.force_variant = 0
        rc = _lib.lib().tamd_matmul(ctypes.byref(part), _lib.stream_ptr(out.device))
        _lib.check(rc, "matmul (split_k ranges as a batch)")
    for s in range(0 if one_launch else n_split):
        k0 = s * chunk
        part = type(args).from_buffer_copy(args)
        part.K = min(chunk, K - k0)
        part.x = args.x + k0 * a.element_size()
        part.w = args.w + (k0 // 2 if w_is_fp4 else k0) * args.w_stride_k * w_esz
        if args.w_mx_scale:
            part.w_mx_scale = args.w_mx_scale + (k0 // MXFP_BLOCK_SIZE) * args.w_mx_stride_k
        if args.x_mx_scale:
            part.x_mx_scale = args.x_mx_scale + k0 // MXFP_BLOCK_SIZE
        if s > 0:
            part.bias = None
        part.activation = _lib.ACT_NONE
        part.y, part.y_dtype = scratch[s].data_ptr(), _lib.F32
        part.y_stride_m, part.y_stride_z = scratch.stride(2), scratch.stride(1)
        part.y_expected_scale = part.y_actual_scale = None
        rc = _lib.lib().tamd_matmul(ctypes.byref(part), _lib.stream_ptr(out.device))
        _lib.check(rc, "matmul (split_k range)")
    # one finalising launch, as in the reference (matmul.py:711-737): sum of the partial results, the fused activation
    # as the reduction's post-processing function, the output's flexpoint scales, the cast
    from .reduce import PostprocessFn
    parts = scratch.view(n_split, batch * rows, N)
    pp = PostprocessFn(fused_activation.specs, fused_activation.fn_args) if fused_activation.specs.name != "dflt" else None
    dst = out if out.is_contiguous() else torch.empty(out.shape, dtype=out.dtype, device=out.device)
    reduce(parts, dim=0, y=dst.view(batch * rows, -1), y_dtype=out.dtype, y_flex=out_flex, y_flex_saturate_inf=saturate_inf,
           postprocess_fn1=pp)
    if dst is not out:
        out.copy_(dst)


matmul_ogs = matmul
