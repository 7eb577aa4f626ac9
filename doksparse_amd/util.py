"""Small host helpers with the names and behaviour of the reference's ``sparse_dok/util.py``."""
import torch

_STR2DTYPE = {
    "bool": torch.bool,
    "uint8": torch.uint8, "char": torch.uint8,
    "int8": torch.int8, "byte": torch.int8,
    "int16": torch.int16, "short": torch.int16,
    "int32": torch.int32, "int": torch.int32,
    "int64": torch.int64, "long": torch.int64,
    "float16": torch.float16, "half": torch.float16,
    "bfloat16": torch.bfloat16,
    "float32": torch.float32, "float": torch.float32,
    "float64": torch.float64, "double": torch.float64,
}

_DTYPE2CTYPE = {
    torch.bool: "bool", torch.uint8: "uint8_t", torch.int8: "int8_t", torch.int16: "int16_t",
    torch.int32: "int32_t", torch.int64: "int64_t", torch.float16: "half",
    torch.bfloat16: "bfloat16", torch.float32: "float", torch.float64: "double",
}


def str2dtype(s):
    """dtype from a name or a dtype (reference: util.py:72-100)."""
    if isinstance(s, torch.dtype):
        return s
    if isinstance(s, str):
        try:
            return _STR2DTYPE[s]
        except KeyError:
            raise ValueError(f"unrecognized type string {s}")
    raise RuntimeError


def dtype2ctype(dtype):
    """C type name of a dtype (reference: util.py:102-123)."""
    return _DTYPE2CTYPE.get(str2dtype(dtype))


def next_power_of_2(n):
    """n if it is a power of two, else the next one; 0 -> 1 (reference: util.py:125-137)."""
    n = int(n)
    if n > 0 and (n & (n - 1)) == 0:
        return n
    return 1 << n.bit_length() if n > 0 else 1


def shape_to_stride(shape):
    """C-contiguous element strides of a shape (reference: util.py:289-293)."""
    shape = tuple(int(s) for s in shape)
    strides = []
    acc = 1
    for s in reversed(shape):
        strides.append(acc)
        acc *= s
    return tuple(reversed(strides))


def get_tensor_accessor_argument_array(*tensors, shape=None, stride=None):
    """[len(tensors), 1 + 2*ndim] int64 rows of (data_ptr, sizes, strides)
    (reference: util.py:295-310)."""
    assert all(isinstance(t, torch.Tensor) for t in tensors)
    assert all(t.shape == tensors[0].shape for t in tensors), "all tensors must have the same shape"
    ndim = tensors[0].dim()
    rows = []
    for t in tensors:
        sizes = tuple(t.shape) if shape is None else tuple(shape)
        strides = tuple(t.stride()) if stride is None else tuple(stride)
        rows.append([t.data_ptr(), *sizes, *strides])
    return torch.tensor(rows, dtype=torch.long).reshape(len(tensors), 1 + 2 * ndim)
