"""ctypes binding of libdtas_packed.so: the reference's own host interface (TVM PackedFunc C signature over
DLTensor handles, experiment/dtas_tuned/elementwise/add/float16/top1_256/host.cc:38-63) in front of the C ABI.
DLTensor / TVMValue are declared here field for field as include/dtas_packed.h declares them."""
import ctypes
import os

from . import _lib

PACKED_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libdtas_packed.so")
FUNCTIONS = ("add", "copy", "cast", "fused_layer_norm_cast1", "fused_softmax_cast", "fused_NT_matmul4_add1",
             "fused_NT_matmul10_add5", "fused_NT_matmul_add", "fused_NT_matmul6_add4",
             # the fused-epilogue GEMMs (prefill and decode names)
             "fused_NT_matmul2_add1_add3_add3", "fused_NT_matmul2_add1_add3_add3_cast", "fused_NT_matmul3_add2_gelu",
             "fused_NT_matmul8_add5_add7_add7", "fused_NT_matmul8_add5_add7_add7_cast5", "fused_NT_matmul9_add6_gelu1",
             # attention: scores and P.V, under the names of both model files
             "fused_NT_matmul1_divide_maximum_minimum_cast2", "fused_NT_matmul7_divide1_maximum1_minimum1_cast7",
             "fused_NT_matmul1_divide1_maximum_minimum_cast2", "fused_NT_matmul7_divide2_maximum1_minimum1_cast7",
             "matmul8", "matmul10", "matmul9", "matmul1",
             # 8-bit weights
             "fused_fused_decode2_fused_NT_matmul_add", "fused_fused_decode2_fused_NT_matmul6_add4",
             "fused_fused_decode4_fused_NT_matmul3_add2_gelu", "fused_fused_decode4_fused_NT_matmul9_add6_gelu1",
             "fused_fused_decode5_fused_NT_matmul4_add1", "fused_fused_decode5_fused_NT_matmul10_add5")
TCODE_OPAQUE_HANDLE, TCODE_NULLPTR, TCODE_DLTENSOR_HANDLE, TCODE_NDARRAY_HANDLE = 3, 4, 7, 13
KDLCUDA, KDLROCM = 2, 10


class DLDevice(ctypes.Structure):
    _fields_ = [("device_type", ctypes.c_int32), ("device_id", ctypes.c_int32)]


class DLDataType(ctypes.Structure):
    _fields_ = [("code", ctypes.c_uint8), ("bits", ctypes.c_uint8), ("lanes", ctypes.c_uint16)]


class DLTensor(ctypes.Structure):
    _fields_ = [("data", ctypes.c_void_p), ("device", DLDevice), ("ndim", ctypes.c_int32), ("dtype", DLDataType),
                ("shape", ctypes.POINTER(ctypes.c_int64)), ("strides", ctypes.POINTER(ctypes.c_int64)),
                ("byte_offset", ctypes.c_uint64)]


class TVMValue(ctypes.Union):
    _fields_ = [("v_int64", ctypes.c_int64), ("v_float64", ctypes.c_double), ("v_handle", ctypes.c_void_p)]


DTYPES = {"float16": (2, 16), "float32": (2, 32), "int8": (0, 8), "int32": (0, 32), "uint32": (1, 32), "float64": (2, 64)}
_handle = None


def lib() -> ctypes.CDLL:
    global _handle
    if _handle is None:
        _lib.lib()  # libdtas_gfx950.so first: the packed library links against it
        if not os.path.exists(PACKED_PATH):
            raise ImportError(f"{PACKED_PATH} is missing: build it with `make -C {os.path.join(os.path.dirname(PACKED_PATH), 'csrc')}`")
        h = ctypes.CDLL(PACKED_PATH)
        for name in FUNCTIONS:
            fn = getattr(h, name)
            fn.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_int32), ctypes.c_int32, ctypes.c_void_p,
                           ctypes.POINTER(ctypes.c_int32), ctypes.c_void_p]
            fn.restype = ctypes.c_int32
        h.dtas_packed_set_stream.argtypes = [ctypes.c_void_p]
        h.dtas_packed_set_stream.restype = None
        h.dtas_packed_last_error.argtypes = []
        h.dtas_packed_last_error.restype = ctypes.c_char_p
        _handle = h
    return _handle


def last_error() -> str:
    return lib().dtas_packed_last_error().decode("utf-8", "replace")


def make_tensor(data_ptr: int, shape, dtype: str, device_id: int = 0, strides=None, device_type: int = KDLROCM,
                byte_offset: int = 0) -> DLTensor:
    """A DLTensor over memory the caller owns.  The shape (and strides) arrays are kept alive on the object."""
    t = DLTensor()
    t.data = data_ptr
    t.device = DLDevice(device_type, device_id)
    t.ndim = len(shape)
    code, bits = DTYPES[dtype]
    t.dtype = DLDataType(code, bits, 1)
    t._shape = (ctypes.c_int64 * len(shape))(*shape)
    t.shape = ctypes.cast(t._shape, ctypes.POINTER(ctypes.c_int64))
    if strides is not None:
        t._strides = (ctypes.c_int64 * len(strides))(*strides)
        t.strides = ctypes.cast(t._strides, ctypes.POINTER(ctypes.c_int64))
    t.byte_offset = byte_offset
    return t


def call(name: str, tensors, codes=None, num_args=None) -> int:
    """Calls `name(args, type_codes, num_args, NULL, NULL, NULL)` as TVM's runtime would."""
    values = (TVMValue * max(1, len(tensors)))()
    for i, t in enumerate(tensors):
        values[i].v_handle = ctypes.addressof(t) if t is not None else None
    tc = (ctypes.c_int32 * max(1, len(tensors)))(*(codes if codes is not None else [TCODE_DLTENSOR_HANDLE] * len(tensors)))
    return getattr(lib(), name)(ctypes.cast(values, ctypes.c_void_p), tc, len(tensors) if num_args is None else num_args, None, None, None)
