"""Host-side logic that needs no GPU: storage layouts (literals of the reference's tests/test_tensor.py:32-35,
76-99), the opt-flags constraint API (matmul_details/opt_flags.py:405-455 of the reference), the block-count
bound, dataclass defaults and the errors raised before any launch."""
import threading

import pytest
import torch

from triton_amd.matmul import FnSpecs, FusedActivation, PrecisionConfig, matmul
from triton_amd.matmul_details import opt_flags as OF
from triton_amd.numerics import InFlexData
from triton_amd.tensor import FP4, UINT8, RaggedTensorMetadata, convert_layout, empty, wrap_torch_tensor
from triton_amd.tensor_details.layout import StridedLayout
from oracle import routing_ref as RR


@pytest.mark.parametrize("logical,is_fp4,layout,storage", [
    ((3, 258, 514), True, StridedLayout(-2), [3, 129, 514]),
    ((0, 64), True, StridedLayout(-2), [0, 64]),
    ((3, 258, 514), True, StridedLayout(-1), [3, 258, 257]),
    ((3, 70, 65), False, StridedLayout(-2), [3, 70, 65]),
])
def test_storage_shapes(logical, is_fp4, layout, storage):
    assert layout.storage_shape(list(logical), is_fp4) == storage
    t = empty(logical, FP4 if is_fp4 else UINT8, "meta", layout)
    assert list(t.storage.data.shape) == storage
    assert t.shape == list(logical)
    if 0 not in storage:
        assert t.storage.data.stride(layout.major_dim % len(storage)) == 1


@pytest.mark.parametrize("major_dim", [-1, -2])
def test_odd_fp4_packing_axis_rejected(major_dim):
    shape = [2, 2]
    shape[major_dim] = 1
    with pytest.raises(ValueError):
        StridedLayout(major_dim).storage_shape(shape, True)


@pytest.mark.parametrize("transpose,layout", [(False, StridedLayout(-1)), (False, StridedLayout(1)),
                                              (True, StridedLayout(-2)), (True, StridedLayout(0))])
def test_convert_layout_noop(transpose, layout):
    data = torch.randn(7, 11)
    t = wrap_torch_tensor(data.T if transpose else data)
    assert convert_layout(t, layout) is t


def test_wrap_fp4_doubles_the_packed_axis():
    t = wrap_torch_tensor(torch.zeros(4, 10, 6, dtype=torch.uint8).transpose(1, 2), dtype=FP4)
    assert t.shape == [4, 12, 10] and t.storage.layout.major_dim % 3 == 1
    t2 = wrap_torch_tensor(torch.zeros(4, 6, 10, dtype=torch.uint8), dtype=FP4)
    assert t2.shape == [4, 6, 20]


def test_convert_layout_repacks_fp4_codes():
    g = torch.Generator().manual_seed(0)
    codes = torch.randint(0, 16, (2, 8, 6), generator=g, dtype=torch.uint8)       # logical [2, 8, 6]
    along_last = codes[..., 0::2] | (codes[..., 1::2] << 4)                        # packed along axis -1
    t = wrap_torch_tensor(along_last, dtype=FP4)
    assert t.shape == [2, 8, 6]
    out = convert_layout(t, StridedLayout(-2))
    want = codes[:, 0::2, :] | (codes[:, 1::2, :] << 4)                            # packed along axis -2
    assert list(out.storage.data.shape) == [2, 4, 6] and out.storage.data.stride(1) == 1
    assert torch.equal(out.storage.data, want)


def test_n_blocks_matches_oracle_and_literal():
    assert RaggedTensorMetadata.n_blocks(128, 16384, 16) == 1144
    assert RaggedTensorMetadata.block_sizes() == [16, 32, 64, 128, 256]
    for S, R, b in [(4, 159, 16), (8, 5, 32), (128, 256, 16), (1, 0, 16), (32, 65536, 128)]:
        assert RaggedTensorMetadata.n_blocks(S, R, b) == RR.n_blocks(S, R, b)
    assert RaggedTensorMetadata.max_n_blocks(4, 159) == RR.n_blocks(4, 159, 16)


def test_opt_flags_constraints_scope_and_errors():
    OF.reset_opt_flags_constraints()
    assert OF.make_opt_flags(16384, 5760, 2880, 128, True).block_m == 128
    assert OF.make_opt_flags(256, 5760, 2880, 128, True).block_m == 16
    assert OF.make_opt_flags(256, 4096, 2048, 1, False).block_m == 128
    assert OF.make_opt_flags(1000, 64, 64, 10, True, expected_slice_size=40).block_m == 64
    # the block covers the mean slice and two standard deviations of a Poisson-like size: 16 + 8 -> 32, 64 + 16 -> 128,
    # 2 + 2.8 -> 16 (decode); fp8 rows never take the 16-row block (the streaming kernel would widen them to 16 bits)
    assert OF.make_opt_flags(2048, 5760, 2880, 128, True).block_m == 32
    assert OF.make_opt_flags(8192, 5760, 2880, 128, True).block_m == 128
    assert OF.make_opt_flags(256, 5760, 2880, 128, True, fp8_rows=True).block_m == 32
    assert OF.make_opt_flags(256, 5760, 2880, 1, False, fp8_rows=True).block_m == 128  # dense: rows as they are
    with OF.scoped_opt_flags_constraints({"block_m": 32}):
        assert OF.make_opt_flags(16384, 5760, 2880, 128, True).block_m == 32
        with OF.scoped_opt_flags_constraints({"block_m": 64}):
            assert OF.make_opt_flags(16384, 5760, 2880, 128, True).block_m == 64
        assert OF.make_opt_flags(16384, 5760, 2880, 128, True).block_m == 32
    assert OF.make_opt_flags(16384, 5760, 2880, 128, True).block_m == 128
    with OF.scoped_opt_flags_constraints({"block_m": 48}):
        with pytest.raises(OF.InapplicableConstraint):
            OF.make_opt_flags(100, 64, 64, 1, False)
    with OF.scoped_opt_flags_constraints({"split_k": 4}):
        assert OF.make_opt_flags(100, 64, 64, 1, False).split_k == 4
    assert OF.make_opt_flags(100, 64, 64, 1, False).split_k == 1
    with OF.scoped_opt_flags_constraints({"split_k": 0}):
        with pytest.raises(OF.InapplicableConstraint):
            OF.make_opt_flags(100, 64, 64, 1, False)
    with OF.scoped_opt_flags_constraints({"is_persistent": True}):
        with pytest.raises(OF.InapplicableConstraint):
            OF.make_opt_flags(100, 64, 64, 1, False)
    OF.update_opt_flags_constraints({"block_m": 16})
    assert OF.make_opt_flags(16384, 5760, 2880, 128, True).block_m == 16
    OF.reset_opt_flags_constraints()
    assert OF.make_opt_flags(16384, 5760, 2880, 128, True).block_m == 128


def test_opt_flags_constraint_keys_are_validated():
    """Unknown keys are a caller's mistake (AssertionError, matmul_details/opt_flags.py:71-73 of the reference); known
    keys must hold for the flags that come out (:46-50), so values the fixed tile cannot honour raise instead of
    being dropped."""
    OF.reset_opt_flags_constraints()
    with OF.scoped_opt_flags_constraints({"blok_m": 64}):
        with pytest.raises(AssertionError, match="unsupported constraint"):
            OF.make_opt_flags(100, 64, 64, 1, False)
    for key, bad, good in (("block_n", 128, 256), ("block_k", 64, 128), ("num_warps", 8, 4), ("epilogue_subtile", 2, 1),
                           ("idle_sms", 4, 0)):
        with OF.scoped_opt_flags_constraints({key: bad}):
            with pytest.raises(OF.InapplicableConstraint, match=key):
                OF.make_opt_flags(100, 64, 64, 1, False)
        with OF.scoped_opt_flags_constraints({key: good}):
            flags = OF.make_opt_flags(100, 64, 64, 1, False)
            assert getattr(flags, key, good) == good
        with OF.scoped_opt_flags_constraints({key: None}):
            OF.make_opt_flags(100, 64, 64, 1, False)
    with OF.scoped_opt_flags_constraints({"disable_mx4_block_swap": True, "is_persistent": False}):
        OF.make_opt_flags(100, 64, 64, 1, False)
    # max_allowable_mn switches a requested split_k off once the output is large (opt_flags.py:37-43, 114-117)
    with OF.scoped_opt_flags_constraints({"split_k": 4, "max_allowable_mn": 100 * 64}):
        assert OF.make_opt_flags(100, 64, 4096, 1, False).split_k == 1
        assert OF.make_opt_flags(99, 64, 4096, 1, False).split_k == 4


def test_opt_flags_constraints_are_per_thread():
    OF.reset_opt_flags_constraints()
    seen = {}

    def other():
        seen["block_m"] = OF.make_opt_flags(16384, 64, 64, 128, True).block_m

    with OF.scoped_opt_flags_constraints({"block_m": 16}):
        th = threading.Thread(target=other)
        th.start()
        th.join()
        assert OF.make_opt_flags(16384, 64, 64, 128, True).block_m == 16
    assert seen["block_m"] == 128


def test_dataclass_defaults_follow_the_reference():
    pc = PrecisionConfig()
    assert pc.b_mx_scale is None and pc.out_dtype is None and pc.acc_scale == 1.0 and pc.allow_tf32
    assert FnSpecs.default().name == "dflt" and FnSpecs.default().reduction_n == 1
    fa = FusedActivation(FnSpecs("swiglu", None, ("alpha", "limit"), reduction_n=2), (1.702, 7.0))
    assert fa.specs.reduction_n == 2 and fa.fn_args == (1.702, 7.0)
    assert not InFlexData().is_per_batch


def test_errors_before_launch():
    x = torch.zeros(4, 64, dtype=torch.bfloat16)
    w = torch.zeros(1, 64, 8, dtype=torch.bfloat16)
    with pytest.raises(NotImplementedError):
        matmul(x, w, None, fused_comm=object())
    with pytest.raises(NotImplementedError):
        matmul(x, w, None, c_acc_in=torch.zeros(4, 8))
    with pytest.raises(NotImplementedError):
        matmul(x, w, None, precision_config=PrecisionConfig(a_mx_scale=torch.zeros(4, 2, dtype=torch.uint8)))
    with pytest.raises(AssertionError):
        matmul(torch.zeros(2, 4, 64), torch.zeros(2, 64, 8), None, gather_indx=torch.zeros(4, dtype=torch.int32))
    with pytest.raises((RuntimeError, NotImplementedError)):
        matmul(x, w, None)  # CPU tensors: no CPU path exists


def test_build_reports_kernels_in_scratch_memory():
    # the build refuses a kernel that fell out of registers: it would still be right, and several times slower
    from triton_amd.build import _scratch_users
    remarks = """
x.h:1:1: remark: Function Name: _ZN4tamd1aEv [-Rpass-analysis=kernel-resource-usage]
x.h:1:1: remark:     VGPRs: 242 [-Rpass-analysis=kernel-resource-usage]
x.h:1:1: remark:     ScratchSize [bytes/lane]: 704 [-Rpass-analysis=kernel-resource-usage]
x.h:9:1: remark: Function Name: _ZN4tamd1bEv [-Rpass-analysis=kernel-resource-usage]
x.h:9:1: remark:     ScratchSize [bytes/lane]: 0 [-Rpass-analysis=kernel-resource-usage]
"""
    assert _scratch_users(remarks) == [("_ZN4tamd1aEv", 704)]
    assert _scratch_users("") == []


def test_turned_gate_weights_are_cached_per_tensor_and_version():
    """Weights with unit stride along N are turned once for the narrow-output kernel: the copy is reused while the
    caller's tensor is alive and unmodified, redone after an in-place write, dropped with the tensor."""
    import gc
    import torch
    from triton_amd import matmul as mm
    w = torch.randn(64, 16)
    t1 = mm._k_contiguous_cached(w)
    assert t1.stride() == (1, 64) and torch.equal(t1, w)
    assert mm._k_contiguous_cached(w) is t1
    w.mul_(2.0)
    t2 = mm._k_contiguous_cached(w)
    assert t2 is not t1 and torch.equal(t2, w)
    key = id(w)
    assert key in mm._TURNED
    del w
    gc.collect()
    assert key not in mm._TURNED
