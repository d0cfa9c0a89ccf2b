"""ctypes view of the DLPack-level entry points (include/tvmkv_dlpack.h).

``tensor(t)`` wraps a torch tensor as a ``DLTensor``; ``view(base, byte_offset, shape)`` describes an
array that lives inside another tensor the way the reference's auxiliary arrays live inside one merged
buffer: ``data`` is the base tensor's address and the array starts ``byte_offset`` bytes further on
(src/runtime/vm/attn_utils.h:1027-1035 of the reference).  ``call(name, *args)`` invokes
``tvmkv_dl_<name>`` with DLTensor / scalar arguments in the reference's slot order."""
import ctypes

from ._lib import check, lib

kDLROCM = 10
kDLInt, kDLFloat = 0, 2


class DLDevice(ctypes.Structure):
    _fields_ = [("device_type", ctypes.c_int32), ("device_id", ctypes.c_int32)]


class DLDataType(ctypes.Structure):
    _fields_ = [("code", ctypes.c_uint8), ("bits", ctypes.c_uint8), ("lanes", ctypes.c_uint16)]


class DLTensor(ctypes.Structure):
    _fields_ = [("data", ctypes.c_void_p), ("device", DLDevice), ("ndim", ctypes.c_int32), ("dtype", DLDataType),
                ("shape", ctypes.POINTER(ctypes.c_int64)), ("strides", ctypes.POINTER(ctypes.c_int64)),
                ("byte_offset", ctypes.c_uint64)]


class RopeScaling(ctypes.Structure):
    """struct tvmkv_rope_scaling of include/tvmkv.h."""
    _fields_ = [("rope_type", ctypes.c_int32), ("rotary_dim", ctypes.c_int32), ("factor", ctypes.c_double),
                ("low_freq_factor", ctypes.c_double), ("high_freq_factor", ctypes.c_double),
                ("beta_fast", ctypes.c_double), ("beta_slow", ctypes.c_double),
                ("max_position_embeddings", ctypes.c_int64), ("original_max_position_embeddings", ctypes.c_int64)]

    TYPES = {"default": 0, "llama3": 1, "longrope": 2, "yarn": 3, "gptj": 4, "llama4": 5}

    @classmethod
    def from_dict(cls, rope_scaling):
        """From the reference's ``rope_scaling`` dictionary (position_embedding.py:258-299)."""
        out = cls()
        out.rope_type = cls.TYPES[rope_scaling.get("rope_type", "default")]
        for key in ("rotary_dim", "factor", "low_freq_factor", "high_freq_factor", "beta_fast", "beta_slow",
                    "max_position_embeddings", "original_max_position_embeddings"):
            if key in rope_scaling:
                setattr(out, key, rope_scaling[key])
        return out


def _dtype_of(torch_dtype):
    import torch
    table = {torch.float16: (kDLFloat, 16), torch.float32: (kDLFloat, 32), torch.int32: (kDLInt, 32),
             torch.int64: (kDLInt, 64), torch.bfloat16: (4, 16)}
    code, bits = table[torch_dtype]
    return DLDataType(code, bits, 1)


class Holder:
    """A DLTensor plus the Python objects that keep its pointers alive."""

    def __init__(self, dl, keep):
        self.dl = dl
        self._keep = keep

    @property
    def pointer(self):
        return ctypes.addressof(self.dl)


def view(base, byte_offset, shape, dtype=None, device_type=kDLROCM, strides=None):
    """`shape` elements of `dtype` (default: the base tensor's) starting byte_offset bytes into `base`."""
    shape_arr = (ctypes.c_int64 * max(len(shape), 1))(*[int(x) for x in shape])
    strides_arr = None
    if strides is not None:
        strides_arr = (ctypes.c_int64 * max(len(strides), 1))(*[int(x) for x in strides])
    dl = DLTensor()
    dl.data = base.data_ptr()
    index = base.device.index
    dl.device = DLDevice(device_type, 0 if index is None else index)
    dl.ndim = len(shape)
    dl.dtype = _dtype_of(dtype or base.dtype)
    dl.shape = ctypes.cast(shape_arr, ctypes.POINTER(ctypes.c_int64))
    dl.strides = ctypes.cast(strides_arr, ctypes.POINTER(ctypes.c_int64)) if strides_arr is not None else None
    dl.byte_offset = int(byte_offset)
    return Holder(dl, (base, shape_arr, strides_arr))


def tensor(t):
    """A contiguous torch tensor as a DLTensor (byte_offset 0)."""
    assert t.is_contiguous()
    return view(t, 0, tuple(t.shape))


def call(name, *args, stream=None):
    """tvmkv_dl_<name>(*args, stream).  Holders pass as DLTensor*, None as NULL, RopeScaling by address."""
    fn = getattr(lib(), "tvmkv_dl_" + name)
    converted = []
    for a in args:
        if isinstance(a, Holder):
            converted.append(ctypes.c_void_p(a.pointer))
        elif isinstance(a, RopeScaling):
            converted.append(ctypes.c_void_p(ctypes.addressof(a)))
        else:
            converted.append(a)
    if stream is None:
        import torch
        stream = torch.cuda.current_stream().cuda_stream
    check(fn(*converted, ctypes.c_void_p(stream)))
