"""ctypes model of an XLA-FFI call frame, for driving the handlers without XLA.

Field order follows the OpenXLA FFI C ABI, version 0.2 (xla/ffi/api/c_api.h).  The
fake API table supplies the two callbacks the handlers use: error creation (records
the message and code) and the stream query.
"""

import ctypes as C

S32, U8, F16, F32, F64 = 4, 6, 10, 11, 12
ERR_INVALID_ARGUMENT, ERR_UNIMPLEMENTED, ERR_INTERNAL = 3, 12, 13


class ExtensionBase(C.Structure):
    pass


ExtensionBase._fields_ = [("struct_size", C.c_size_t), ("type", C.c_int32),
                          ("next", C.POINTER(ExtensionBase))]


class ApiVersion(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("extension_start", C.c_void_p),
                ("major_version", C.c_int), ("minor_version", C.c_int)]


class ByteSpan(C.Structure):
    _fields_ = [("ptr", C.c_char_p), ("len", C.c_size_t)]


class Scalar(C.Structure):
    _fields_ = [("dtype", C.c_int32), ("value", C.c_void_p)]


class Buffer(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("extension_start", C.c_void_p), ("dtype", C.c_int32),
                ("data", C.c_void_p), ("rank", C.c_int64), ("dims", C.POINTER(C.c_int64))]


class Args(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("extension_start", C.c_void_p), ("size", C.c_int64),
                ("types", C.POINTER(C.c_int32)), ("args", C.POINTER(C.c_void_p))]


class Attrs(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("extension_start", C.c_void_p), ("size", C.c_int64),
                ("types", C.POINTER(C.c_int32)), ("names", C.POINTER(C.POINTER(ByteSpan))),
                ("attrs", C.POINTER(C.c_void_p))]


class ErrorCreateArgs(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("extension_start", C.c_void_p),
                ("message", C.c_char_p), ("errc", C.c_int32)]


class StreamGetArgs(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("extension_start", C.c_void_p), ("ctx", C.c_void_p),
                ("stream", C.c_void_p)]


ERROR_CREATE = C.CFUNCTYPE(C.c_void_p, C.POINTER(ErrorCreateArgs))
STREAM_GET = C.CFUNCTYPE(C.c_void_p, C.POINTER(StreamGetArgs))


class DeviceMemoryAllocateArgs(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("extension_start", C.c_void_p), ("ctx", C.c_void_p),
                ("size", C.c_size_t), ("alignment", C.c_size_t), ("data", C.c_void_p)]


class DeviceMemoryFreeArgs(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("extension_start", C.c_void_p), ("ctx", C.c_void_p),
                ("size", C.c_size_t), ("data", C.c_void_p)]


DEVICE_ALLOCATE = C.CFUNCTYPE(C.c_void_p, C.POINTER(DeviceMemoryAllocateArgs))
DEVICE_FREE = C.CFUNCTYPE(C.c_void_p, C.POINTER(DeviceMemoryFreeArgs))


class Api(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("extension_start", C.c_void_p),
                ("api_version", ApiVersion), ("internal_api", C.c_void_p),
                ("error_create", ERROR_CREATE), ("error_get_message", C.c_void_p),
                ("error_destroy", C.c_void_p), ("handler_register", C.c_void_p),
                ("stream_get", STREAM_GET), ("type_register", C.c_void_p),
                ("execution_context_get", C.c_void_p), ("state_set", C.c_void_p), ("state_get", C.c_void_p),
                ("device_memory_allocate", DEVICE_ALLOCATE), ("device_memory_free", DEVICE_FREE)] + \
               [(f"unused{n}", C.c_void_p) for n in range(7)]


class CallFrame(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("extension_start", C.POINTER(ExtensionBase)),
                ("api", C.POINTER(Api)), ("ctx", C.c_void_p), ("stage", C.c_int32),
                ("args", Args), ("rets", Args), ("attrs", Attrs), ("future", C.c_void_p)]


class Metadata(C.Structure):
    _fields_ = [("struct_size", C.c_size_t), ("api_version", ApiVersion), ("traits", C.c_uint32),
                ("state_type_id", C.c_int64)]


class MetadataExtension(C.Structure):
    _fields_ = [("base", ExtensionBase), ("metadata", C.POINTER(Metadata))]


class FakeXla:
    """Builds frames and records the errors the handler creates."""

    def __init__(self, stream: int = 0):
        self.errors = []
        self.stream = stream
        self._keep = []

        def error_create(args):
            self.errors.append((args.contents.errc, args.contents.message.decode()))
            return 0xE000 + len(self.errors)

        def stream_get(args):
            args.contents.stream = self.stream
            return None

        #: device scratch handed out through the allocation callbacks: address -> buffer; `allocate`
        #: is a callable `(nbytes) -> object with data_ptr()` (None: the runtime has no memory to give)
        self.allocate = None
        self.scratch = {}
        self.allocations = 0

        def device_allocate(args):
            if self.allocate is None:
                return 0xA110C
            buf = self.allocate(int(args.contents.size) + int(args.contents.alignment))
            base = buf.data_ptr()
            align = max(int(args.contents.alignment), 1)
            aligned = (base + align - 1) // align * align
            self.scratch[aligned] = buf
            self.allocations += 1
            args.contents.data = aligned
            return None

        def device_free(args):
            self.scratch.pop(args.contents.data)   # KeyError: freed what was never handed out
            return None

        self._cb = (ERROR_CREATE(error_create), STREAM_GET(stream_get), DEVICE_ALLOCATE(device_allocate),
                    DEVICE_FREE(device_free))
        self.api = Api(struct_size=C.sizeof(Api), error_create=self._cb[0], stream_get=self._cb[1],
                       device_memory_allocate=self._cb[2], device_memory_free=self._cb[3])
        self.api.api_version = ApiVersion(C.sizeof(ApiVersion), None, 0, 2)

    def buffer(self, dtype: int, data_ptr: int, dims) -> Buffer:
        arr = (C.c_int64 * max(len(dims), 1))(*dims)
        buf = Buffer(C.sizeof(Buffer), None, dtype, data_ptr, len(dims), arr)
        self._keep += [arr, buf]
        return buf

    def _pack(self, buffers):
        n = len(buffers)
        types = (C.c_int32 * max(n, 1))(*([1] * n))
        ptrs = (C.c_void_p * max(n, 1))(*[C.addressof(b) for b in buffers])
        self._keep += [types, ptrs]
        return Args(C.sizeof(Args), None, n, types, ptrs)

    def frame(self, args, rets, attrs: dict, stage: int = 3) -> CallFrame:
        """attrs: name -> (dtype code, ctypes scalar); passed sorted by name, as XLA does."""
        names = sorted(attrs)
        n = len(names)
        types = (C.c_int32 * max(n, 1))(*([3] * n))
        spans = [ByteSpan(name.encode(), len(name)) for name in names]
        span_ptrs = (C.POINTER(ByteSpan) * max(n, 1))(*[C.pointer(s) for s in spans])
        scalars = [Scalar(attrs[name][0], C.addressof(attrs[name][1])) for name in names]
        scalar_ptrs = (C.c_void_p * max(n, 1))(*[C.addressof(s) for s in scalars])
        self._keep += [types, spans, span_ptrs, scalars, scalar_ptrs, attrs]
        frame = CallFrame(struct_size=C.sizeof(CallFrame), extension_start=None,
                          api=C.pointer(self.api), ctx=None, stage=stage,
                          args=self._pack(args), rets=self._pack(rets),
                          attrs=Attrs(C.sizeof(Attrs), None, n, types, span_ptrs, scalar_ptrs),
                          future=None)
        self._keep.append(frame)
        return frame

    def metadata_frame(self):
        md = Metadata(struct_size=C.sizeof(Metadata))
        md.api_version = ApiVersion(C.sizeof(ApiVersion), None, -1, -1)
        md.traits = 99
        md.state_type_id = 77
        ext = MetadataExtension(ExtensionBase(C.sizeof(MetadataExtension), 1, None), C.pointer(md))
        frame = CallFrame(struct_size=C.sizeof(CallFrame),
                          extension_start=C.cast(C.pointer(ext), C.POINTER(ExtensionBase)),
                          api=C.pointer(self.api), stage=0)
        self._keep += [md, ext, frame]
        return frame, md
