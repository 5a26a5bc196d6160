"""ctypes mirror of include/xla_ffi_min.h and a small call-frame builder: the fake XLA host the
FFI handlers are tested against."""
import ctypes as C

BUFFER, SCALAR = 1, 3
PRED, S32, S64, U32, F16, F32, F64, BF16, F8E4M3FN = 1, 4, 5, 8, 10, 11, 12, 16, 20
EXECUTE = 3


class ExtBase(C.Structure):
    pass


ExtBase._fields_ = [("struct_size", C.c_size_t), ("type", C.c_int), ("next", C.POINTER(ExtBase))]


class ApiVersion(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("extension_start", C.c_void_p), ("major_version", C.c_int),
                ("minor_version", C.c_int)]


class Buffer(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("extension_start", C.c_void_p), ("dtype", C.c_int),
                ("data", C.c_void_p), ("rank", C.c_int64), ("dims", C.POINTER(C.c_int64))]


class ByteSpan(C.Structure):
    _fields_ = [("ptr", C.c_char_p), ("len", C.c_size_t)]


class Scalar(C.Structure):
    _fields_ = [("dtype", C.c_int), ("value", C.c_void_p)]


class Args(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("extension_start", C.c_void_p), ("size", C.c_int64),
                ("types", C.POINTER(C.c_int)), ("args", C.POINTER(C.c_void_p))]


class Attrs(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("extension_start", C.c_void_p), ("size", C.c_int64),
                ("types", C.POINTER(C.c_int)), ("names", C.POINTER(C.POINTER(ByteSpan))),
                ("attrs", C.POINTER(C.c_void_p))]


class ErrorCreateArgs(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("extension_start", C.c_void_p), ("message", C.c_char_p),
                ("errc", C.c_int)]


class StreamGetArgs(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("extension_start", C.c_void_p), ("ctx", C.c_void_p),
                ("stream", C.c_void_p)]


class HandlerBundle(C.Structure):
    _fields_ = [("instantiate", C.c_void_p), ("prepare", C.c_void_p), ("initialize", C.c_void_p),
                ("execute", C.c_void_p)]


class HandlerRegisterArgs(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("extension_start", C.c_void_p), ("name", ByteSpan),
                ("platform", ByteSpan), ("bundle", HandlerBundle), ("traits", C.c_uint32)]


class DeviceMemoryAllocateArgs(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("extension_start", C.c_void_p), ("ctx", C.c_void_p),
                ("size", C.c_size_t), ("alignment", C.c_size_t), ("data", C.c_void_p)]


class DeviceMemoryFreeArgs(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("extension_start", C.c_void_p), ("ctx", C.c_void_p),
                ("size", C.c_size_t), ("data", C.c_void_p)]


ERROR_CREATE = C.CFUNCTYPE(C.c_void_p, C.POINTER(ErrorCreateArgs))
DEVICE_ALLOC = C.CFUNCTYPE(C.c_void_p, C.POINTER(DeviceMemoryAllocateArgs))
DEVICE_FREE = C.CFUNCTYPE(C.c_void_p, C.POINTER(DeviceMemoryFreeArgs))
STREAM_GET = C.CFUNCTYPE(C.c_void_p, C.POINTER(StreamGetArgs))
HANDLER_REGISTER = C.CFUNCTYPE(C.c_void_p, C.POINTER(HandlerRegisterArgs))


class Api(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("extension_start", C.c_void_p), ("api_version", ApiVersion),
                ("internal_api", C.c_void_p), ("XLA_FFI_Error_Create", ERROR_CREATE),
                ("XLA_FFI_Error_GetMessage", C.c_void_p), ("XLA_FFI_Error_Destroy", C.c_void_p),
                ("XLA_FFI_Handler_Register", HANDLER_REGISTER), ("XLA_FFI_Stream_Get", STREAM_GET),
                ("XLA_FFI_TypeId_Register", C.c_void_p), ("XLA_FFI_ExecutionContext_Get", C.c_void_p),
                ("XLA_FFI_State_Set", C.c_void_p), ("XLA_FFI_State_Get", C.c_void_p),
                ("XLA_FFI_DeviceMemory_Allocate", DEVICE_ALLOC), ("XLA_FFI_DeviceMemory_Free", DEVICE_FREE)]


class CallFrame(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("extension_start", C.POINTER(ExtBase)), ("api", C.POINTER(Api)),
                ("ctx", C.c_void_p), ("stage", C.c_int), ("args", Args), ("rets", Args), ("attrs", Attrs),
                ("future", C.c_void_p)]


class Metadata(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("api_version", ApiVersion), ("traits", C.c_uint32)]


class MetadataExtension(C.Structure):
    _fields_ = [("extension_base", ExtBase), ("metadata", C.POINTER(Metadata))]


class FakeHost:
    """XLA_FFI_Api with Error_Create, Stream_Get and Handler_Register implemented in Python, and
    DeviceMemory_Allocate / Free when an ``allocator`` (size, alignment) -> (device pointer, keep-alive
    object) is given; without one the table ends at Stream_Get, as an older host's would."""

    def __init__(self, stream=0, allocator=None):
        self.errors = []      # (code, message) of every error created
        self.registered = []  # (name, platform, execute pointer)
        self.stream = stream
        self._keep = []

        def error_create(a):
            self.errors.append((a.contents.errc, a.contents.message.decode()))
            return 0x1000 + len(self.errors)  # opaque non-null handle

        def stream_get(a):
            a.contents.stream = self.stream
            return None

        def handler_register(a):
            r = a.contents
            self.registered.append((C.string_at(r.name.ptr, r.name.len).decode(),
                                    C.string_at(r.platform.ptr, r.platform.len).decode(), r.bundle.execute))
            return None

        self.allocations = []  # (size, alignment) of every scratch request
        self.freed = []        # sizes handed back
        self._live = {}

        def device_alloc(a):
            r = a.contents
            ptr, keep = allocator(r.size, r.alignment)
            self.allocations.append((r.size, r.alignment))
            self._live[ptr] = keep
            r.data = ptr
            return None

        def device_free(a):
            r = a.contents
            self.freed.append(r.size)
            # the tensor is kept until the host object dies: the work that uses it is only enqueued
            self._keep.append(self._live.pop(r.data, None))
            return None

        self._cbs = (ERROR_CREATE(error_create), STREAM_GET(stream_get), HANDLER_REGISTER(handler_register),
                     DEVICE_ALLOC(device_alloc), DEVICE_FREE(device_free))
        self.api = Api()
        self.api.struct_size = C.sizeof(Api) if allocator else Api.XLA_FFI_TypeId_Register.offset
        if allocator:
            self.api.XLA_FFI_DeviceMemory_Allocate = self._cbs[3]
            self.api.XLA_FFI_DeviceMemory_Free = self._cbs[4]
        self.api.api_version = ApiVersion(C.sizeof(ApiVersion), None, 0, 1)
        self.api.XLA_FFI_Error_Create = self._cbs[0]
        self.api.XLA_FFI_Stream_Get = self._cbs[1]
        self.api.XLA_FFI_Handler_Register = self._cbs[2]

    def _buffers(self, bufs):
        n = len(bufs)
        types = (C.c_int * max(n, 1))(*([BUFFER] * n))
        ptrs = (C.c_void_p * max(n, 1))()
        for i, (dtype, data, dims) in enumerate(bufs):
            d = (C.c_int64 * max(len(dims), 1))(*dims)
            b = Buffer(C.sizeof(Buffer), None, dtype, data, len(dims), C.cast(d, C.POINTER(C.c_int64)))
            self._keep += [d, b]
            ptrs[i] = C.addressof(b)
        self._keep += [types, ptrs]
        return Args(C.sizeof(Args), None, n, C.cast(types, C.POINTER(C.c_int)), C.cast(ptrs, C.POINTER(C.c_void_p)))

    def frame(self, args, rets, attrs, stage=EXECUTE):
        """args / rets: lists of (dtype, device pointer, dims); attrs: {name: (dtype, python value)}."""
        f = CallFrame()
        f.struct_size = C.sizeof(CallFrame)
        f.api = C.pointer(self.api)
        f.stage = stage
        f.args = self._buffers(args)
        f.rets = self._buffers(rets)
        names = sorted(attrs)
        n = len(names)
        types = (C.c_int * max(n, 1))(*([SCALAR] * n))
        nptrs = (C.POINTER(ByteSpan) * max(n, 1))()
        aptrs = (C.c_void_p * max(n, 1))()
        ctype = {S32: C.c_int32, S64: C.c_int64, F32: C.c_float, F64: C.c_double, PRED: C.c_uint8}
        for i, name in enumerate(names):
            dtype, value = attrs[name]
            v = ctype[dtype](value)
            s = Scalar(dtype, C.addressof(v))
            raw = name.encode()
            span = ByteSpan(raw, len(raw))
            self._keep += [v, s, raw, span]
            nptrs[i] = C.pointer(span)
            aptrs[i] = C.addressof(s)
        self._keep += [types, nptrs, aptrs]
        f.attrs = Attrs(C.sizeof(Attrs), None, n, C.cast(types, C.POINTER(C.c_int)),
                        C.cast(nptrs, C.POINTER(C.POINTER(ByteSpan))), C.cast(aptrs, C.POINTER(C.c_void_p)))
        self._keep.append(f)
        return f


def gemm_attrs(m, n, k, dtype_in, dtype_out, *, lhs_col_major=False, rhs_col_major=False, out_col_major=False,
               alpha=1.0, beta=0.0, epilogue=None, batch=1):
    """The attribute dictionary XLA attaches to a GEMM custom call (keys as read by the reference's
    RunGemm): row/column counts are those of the logical matrices, the order says how they are stored."""
    a = {
        "lhs_order": (S32, int(lhs_col_major)), "rhs_order": (S32, int(rhs_col_major)),
        "output_order": (S32, int(out_col_major)),
        "lhs_num_rows": (S64, m), "lhs_num_cols": (S64, k), "rhs_num_rows": (S64, k), "rhs_num_cols": (S64, n),
        "output_num_rows": (S64, m), "output_num_cols": (S64, n),
        "lhs_batch_stride": (S64, m * k), "rhs_batch_stride": (S64, k * n), "output_batch_stride": (S64, m * n),
        "lhs_leading_dim_stride": (S64, m if lhs_col_major else k),
        "rhs_leading_dim_stride": (S64, k if rhs_col_major else n),
        "output_leading_dim_stride": (S64, m if out_col_major else n),
        "batch_size": (S64, batch), "alpha": (F32, alpha), "beta": (F32, beta), "algorithm": (S64, -6),
        "lhs_layout_dtype": (S32, dtype_in), "rhs_layout_dtype": (S32, dtype_in),
        "output_layout_dtype": (S32, dtype_out),
    }
    if epilogue is not None:
        a["epilogue"] = (S32, epilogue)
    return a
