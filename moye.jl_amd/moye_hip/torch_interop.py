"""PyTorch as plumbing only: device memory and streams for tests and the benchmark."""
import torch

from . import _lib

_DT = {torch.float32: _lib.F32, torch.float16: _lib.F16, torch.bfloat16: _lib.BF16, torch.float64: _lib.F64,
       torch.uint8: _lib.U8, torch.int8: _lib.U8, torch.int16: _lib.U16, torch.int32: _lib.U32,
       torch.int64: _lib.U64}
if hasattr(torch, "float8_e4m3fn"):
    _DT[torch.float8_e4m3fn] = _lib.F8E4M3


# moye dtype -> torch dtype (the first torch type registered for it)
TORCH_DTYPES = {}
for _t, _m in _DT.items():
    TORCH_DTYPES.setdefault(_m, _t)


def dtype_of(t):
    return _DT[t.dtype]


def tensor_of(t, shape=None, stride=None, dtype=None):
    """moye_tensor over a torch tensor's storage.  By default the tensor's own sizes and strides
    (torch's are already in elements); pass shape/stride to impose a MoYe layout on the buffer."""
    if shape is None:
        shape, stride = tuple(t.shape), tuple(t.stride())
    return _lib.make_tensor(t.data_ptr(), dtype if dtype is not None else _DT[t.dtype], shape, stride)


def current_stream():
    return torch.cuda.current_stream().cuda_stream
