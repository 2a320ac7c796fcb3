"""Host rule set of grouped_mm, checked on the CPU.

The rules (reference api.py:61-163) only look at dtype, rank, sizes, strides and
device, so a small stand-in object can play the tensor and every rule -- also
those behind the "GPU-only" check -- can be exercised without a GPU.  The
expected texts are the reference's, character for character.
"""
import pytest
import torch

from grouped_mm_bf16_amd import api, grouped_mm


class T:
    """Just enough of a tensor for the rule set."""

    def __init__(self, shape, dtype=torch.bfloat16, strides=None, device="cuda:0", cuda=True):
        self.shape = tuple(shape)
        self.dtype = dtype
        if strides is None:
            strides, acc = [], 1
            for s in reversed(self.shape):
                strides.insert(0, acc)
                acc *= max(s, 1)
        self._strides = tuple(strides)
        self.device = torch.device(device)
        self.is_cuda = cuda

    def dim(self):
        return len(self.shape)

    def size(self, i=None):
        return self.shape if i is None else self.shape[i]

    def stride(self, i=None):
        return self._strides if i is None else self._strides[i]

    def numel(self):
        n = 1
        for s in self.shape:
            n *= s
        return n

    def t(self):
        assert self.dim() >= 2
        shp = list(self.shape)
        st = list(self._strides)
        shp[-1], shp[-2] = shp[-2], shp[-1]
        st[-1], st[-2] = st[-2], st[-1]
        return T(shp, self.dtype, st, str(self.device), self.is_cuda)


def offs_t(n, dtype=torch.int32, **kw):
    return T((n,), dtype, **kw)


def fails(msg, a, b, offs=None, bias=None, out_dtype=None):
    with pytest.raises(RuntimeError) as e:
        api.validate_inputs(a, b, offs, bias, out_dtype)
    assert str(e.value) == msg


def test_dtype_rules():
    fails("Expected mat_a to be Float32, BFloat16 or Float16 matrix, got torch.float64",
          T((4, 4), torch.float64), T((4, 4)))
    fails("Expected mat_b to be Float32, BFloat16 or Float16 matrix, got torch.int8",
          T((4, 4)), T((4, 4), torch.int8))
    # mat_a's dtype is reported first even when both are wrong
    fails("Expected mat_a to be Float32, BFloat16 or Float16 matrix, got torch.int32",
          T((4, 4), torch.int32), T((4, 4), torch.int8))
    fails("mat_a and mat_b must have the same dtype", T((4, 4), torch.float16), T((4, 4), torch.bfloat16))


def test_rank_rules():
    fails("mat_a has to be 2 or 3d", T((4,)), T((4, 4)))
    fails("mat_b has to be 2 or 3d", T((4, 4)), T((1, 1, 4, 4)))
    # rank is checked before the dtype match
    fails("mat_a has to be 2 or 3d", T((4,), torch.float16), T((4, 4), torch.float32))


def test_contraction_rule():
    msg = "contraction dimension of mat_a and mat_b must match"
    fails(msg, T((8, 5)), T((2, 6, 3)), offs_t(2))
    fails(msg, T((2, 8, 5)), T((2, 6, 3)))
    fails(msg, T((8, 5)), T((6, 3)), offs_t(2))
    fails(msg, T((2, 8, 5)), T((6, 3)), offs_t(2))


def test_device_rules():
    fails("grouped_mm_bf16 is GPU-only (CUDA/HIP); CPU tensors are not supported",
          T((4, 4), device="cpu", cuda=False), T((4, 4)), offs_t(1))
    fails("mat_a and mat_b must be on the same device", T((4, 4)), T((4, 4), device="cuda:1"), offs_t(1))
    # the device check comes after the contraction check
    fails("contraction dimension of mat_a and mat_b must match",
          T((4, 5), device="cpu", cuda=False), T((4, 4)), offs_t(1))


def test_real_cpu_tensors_are_rejected():
    with pytest.raises(RuntimeError, match="GPU-only"):
        grouped_mm(torch.randn(4, 4), torch.randn(4, 4), offs=torch.tensor([4], dtype=torch.int32))


def test_stride_rule():
    assert api.is_row_major(T((4, 8))) is True
    assert api.is_row_major(T((4, 8)).t()) is False          # column-major view
    assert api.is_row_major(T((4, 8), strides=(16, 1))) is True  # padded rows are fine
    assert api.is_row_major(T((3, 4, 8), strides=(1000, 8, 1))) is True  # batch stride is free
    assert api.is_row_major(T((3, 4, 8), strides=(32, 1, 4))) is False
    with pytest.raises(RuntimeError) as e:
        api.is_row_major(T((4, 8), strides=(16, 2)))
    assert str(e.value) == "Invalid strides/sizes, got (16, 2) for strides and (4, 8) for sizes"
    with pytest.raises(RuntimeError):
        api.is_row_major(T((4, 8), strides=(4, 1)))  # rows overlap
    fails("Invalid strides/sizes, got (16, 2) for strides and (4, 8) for sizes",
          T((4, 8), strides=(16, 2)), T((8, 4)), offs_t(1))
    # no 16-byte alignment rule: odd sizes are valid (reference tests use K=33, N=29)
    api.validate_inputs(T((10, 33)), T((3, 33, 29)), offs_t(3), None, None)


def test_offs_rules():
    msg = "Have to provide offsets if there is a 2d matrix, or no offset if both matrices are 3d"
    fails(msg, T((8, 4)), T((2, 4, 3)))
    fails(msg, T((2, 8, 4)), T((2, 4, 3)), offs_t(2))
    fails("offs must be a CUDA/HIP tensor (CPU offs are not supported)",
          T((8, 4)), T((2, 4, 3)), offs_t(2, device="cpu", cuda=False))
    fails("offs must be on the same device as inputs", T((8, 4)), T((2, 4, 3)), offs_t(2, device="cuda:1"))
    fails("offs has to be 1D", T((8, 4)), T((2, 4, 3)), T((2, 1), torch.int32))
    fails("Offsets have to be int32", T((8, 4)), T((2, 4, 3)), offs_t(2, torch.int64))
    fails("Can't process more than 1024 groups", T((8, 4)), T((1024, 4, 3)), offs_t(1024))
    api.validate_inputs(T((8, 4)), T((1023, 4, 3)), offs_t(1023), None, None)


def test_bias_and_out_dtype_rules():
    fails("Bias not supported yet", T((8, 4)), T((2, 4, 3)), offs_t(2), bias=T((3,)))
    fails("Grouped gemm output dtype must match `mat_a` dtype", T((8, 4)), T((2, 4, 3)), offs_t(2),
          out_dtype=torch.float32)
    # bias is reported before out_dtype
    fails("Bias not supported yet", T((8, 4)), T((2, 4, 3)), offs_t(2), bias=T((3,)), out_dtype=torch.float32)
    got = api.validate_inputs(T((8, 4)), T((2, 4, 3)), offs_t(2), None, torch.bfloat16)
    assert got == api.Checked(True, False, torch.bfloat16)
    got = api.validate_inputs(T((2, 8, 4), torch.float32), T((2, 4, 3), torch.float32), None, None, None)
    assert got == api.Checked(False, False, torch.float32)


def test_output_shapes_and_group_count_rules():
    assert api.output_shape(T((8, 4)), T((2, 4, 3)), offs_t(2)) == (8, 3)
    assert api.output_shape(T((2, 8, 4)), T((2, 4, 3)), None) == (2, 8, 3)
    assert api.output_shape(T((8, 40)), T((40, 3)), offs_t(5)) == (5, 8, 3)
    assert api.output_shape(T((5, 8, 4)), T((4, 30)), offs_t(5)) == (8, 30)
    for a, b, o in [(T((8, 4)), T((2, 4, 3)), offs_t(3)), (T((5, 8, 4)), T((4, 30)), offs_t(4))]:
        with pytest.raises(RuntimeError) as e:
            api.output_shape(a, b, o)
        assert str(e.value) == "matrix batch sizes have to match"
    with pytest.raises(RuntimeError) as e:
        api.output_shape(T((2, 8, 4)), T((3, 4, 3)), None)
    assert str(e.value) == "batched dimension has to match"


def test_signature_is_the_reference_one():
    import inspect
    sig = inspect.signature(grouped_mm)
    assert list(sig.parameters) == ["mat_a", "mat_b", "offs", "bias", "out_dtype"]
    assert [p.default for p in sig.parameters.values()][2:] == [None, None, None]
    assert all(p.kind is inspect.Parameter.POSITIONAL_OR_KEYWORD for p in sig.parameters.values())
