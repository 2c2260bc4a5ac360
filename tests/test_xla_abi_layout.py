"""The two hand-written mirrors of the OpenXLA FFI C ABI (`e3j_amd/csrc/xla_ffi_abi.h` for the
handlers, the ctypes classes of `tests/xla_frame.py` for the test frames) against the header the
reference vendors, `lib/e3j_ops/xla/ffi/api/c_api.h`: one translation unit includes the
reference's header and the library's, with a static assertion on the size of every mirrored
structure, the offset of every field and the value of every constant; the same program prints
the reference's layout, which the ctypes classes must reproduce.  Skipped where the reference
tree is absent."""

import ctypes as C
import json
import os
import shutil
import subprocess

import pytest

from tests import xla_frame as F

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REFERENCE_HEADER = "/root/reference/lib/e3j_ops/xla/ffi/api/c_api.h"

pytestmark = pytest.mark.skipif(not os.path.exists(REFERENCE_HEADER) or shutil.which("g++") is None,
                                reason="needs the reference's vendored c_api.h and g++")

#: (structure of xla_ffi_abi.h, structure of c_api.h, ctypes class, [(field here, field there, ctypes field)])
PAIRS = [
    ("XlaExtensionBase", "XLA_FFI_Extension_Base", F.ExtensionBase,
     [("struct_size",) * 3, ("type",) * 3, ("next",) * 3]),
    ("XlaApiVersion", "XLA_FFI_Api_Version", F.ApiVersion,
     [("struct_size",) * 3, ("extension_start",) * 3, ("major_version",) * 3, ("minor_version",) * 3]),
    ("XlaByteSpan", "XLA_FFI_ByteSpan", F.ByteSpan, [("ptr",) * 3, ("len",) * 3]),
    ("XlaScalar", "XLA_FFI_Scalar", F.Scalar, [("dtype",) * 3, ("value",) * 3]),
    ("XlaBuffer", "XLA_FFI_Buffer", F.Buffer,
     [("struct_size",) * 3, ("extension_start",) * 3, ("dtype",) * 3, ("data",) * 3, ("rank",) * 3, ("dims",) * 3]),
    ("XlaArgs", "XLA_FFI_Args", F.Args,
     [("struct_size",) * 3, ("extension_start",) * 3, ("size",) * 3, ("types",) * 3, ("args",) * 3]),
    ("XlaRets", "XLA_FFI_Rets", F.Args,
     [("struct_size",) * 3, ("extension_start",) * 3, ("size",) * 3, ("types",) * 3, ("rets", "rets", "args")]),
    ("XlaAttrs", "XLA_FFI_Attrs", F.Attrs,
     [("struct_size",) * 3, ("extension_start",) * 3, ("size",) * 3, ("types",) * 3, ("names",) * 3, ("attrs",) * 3]),
    ("XlaCallFrame", "XLA_FFI_CallFrame", F.CallFrame,
     [("struct_size",) * 3, ("extension_start",) * 3, ("api",) * 3, ("ctx",) * 3, ("stage",) * 3, ("args",) * 3,
      ("rets",) * 3, ("attrs",) * 3, ("future",) * 3]),
    ("XlaErrorCreateArgs", "XLA_FFI_Error_Create_Args", F.ErrorCreateArgs,
     [("struct_size",) * 3, ("extension_start",) * 3, ("message",) * 3, ("errc",) * 3]),
    ("XlaStreamGetArgs", "XLA_FFI_Stream_Get_Args", F.StreamGetArgs,
     [("struct_size",) * 3, ("extension_start",) * 3, ("ctx",) * 3, ("stream",) * 3]),
    ("XlaMetadata", "XLA_FFI_Metadata", F.Metadata,
     [("struct_size",) * 3, ("api_version",) * 3, ("traits",) * 3, ("state_type_id",) * 3]),
    ("XlaMetadataExtension", "XLA_FFI_Metadata_Extension", F.MetadataExtension,
     [("base", "extension_base", "base"), ("metadata",) * 3]),
    ("XlaApi", "XLA_FFI_Api", F.Api,
     [("struct_size",) * 3, ("extension_start",) * 3, ("api_version",) * 3, ("internal_api",) * 3,
      ("error_create", "XLA_FFI_Error_Create", "error_create"),
      ("error_get_message", "XLA_FFI_Error_GetMessage", "error_get_message"),
      ("error_destroy", "XLA_FFI_Error_Destroy", "error_destroy"),
      ("handler_register", "XLA_FFI_Handler_Register", "handler_register"),
      ("stream_get", "XLA_FFI_Stream_Get", "stream_get"),
      ("type_register", "XLA_FFI_Type_Register", "type_register"),
      ("execution_context_get", "XLA_FFI_ExecutionContext_Get", "execution_context_get"),
      ("state_set", "XLA_FFI_State_Set", "state_set"), ("state_get", "XLA_FFI_State_Get", "state_get"),
      ("device_memory_allocate", "XLA_FFI_DeviceMemory_Allocate", "device_memory_allocate"),
      ("device_memory_free", "XLA_FFI_DeviceMemory_Free", "device_memory_free")]),
    ("XlaDeviceMemoryAllocateArgs", "XLA_FFI_DeviceMemory_Allocate_Args", F.DeviceMemoryAllocateArgs,
     [("struct_size",) * 3, ("extension_start",) * 3, ("ctx",) * 3, ("size",) * 3, ("alignment",) * 3, ("data",) * 3]),
    ("XlaDeviceMemoryFreeArgs", "XLA_FFI_DeviceMemory_Free_Args", F.DeviceMemoryFreeArgs,
     [("struct_size",) * 3, ("extension_start",) * 3, ("ctx",) * 3, ("size",) * 3, ("data",) * 3]),
]
#: constants of xla_ffi_abi.h and the enumerators they restate
CONSTANTS = [
    ("kXlaFfiApiMajor", "XLA_FFI_API_MAJOR"), ("kXlaFfiApiMinor", "XLA_FFI_API_MINOR"),
    ("kXlaExtMetadata", "XLA_FFI_Extension_Metadata"), ("kXlaArgBuffer", "XLA_FFI_ArgType_BUFFER"),
    ("kXlaRetBuffer", "XLA_FFI_RetType_BUFFER"), ("kXlaAttrArray", "XLA_FFI_AttrType_ARRAY"),
    ("kXlaAttrDictionary", "XLA_FFI_AttrType_DICTIONARY"), ("kXlaAttrScalar", "XLA_FFI_AttrType_SCALAR"),
    ("kXlaAttrString", "XLA_FFI_AttrType_STRING"), ("kXlaStageExecute", "XLA_FFI_ExecutionStage_EXECUTE"),
    ("kXlaS32", "XLA_FFI_DataType_S32"), ("kXlaS64", "XLA_FFI_DataType_S64"), ("kXlaU8", "XLA_FFI_DataType_U8"),
    ("kXlaF16", "XLA_FFI_DataType_F16"), ("kXlaF32", "XLA_FFI_DataType_F32"), ("kXlaF64", "XLA_FFI_DataType_F64"),
    ("kXlaErrInvalidArgument", "XLA_FFI_Error_Code_INVALID_ARGUMENT"),
    ("kXlaErrUnimplemented", "XLA_FFI_Error_Code_UNIMPLEMENTED"), ("kXlaErrInternal", "XLA_FFI_Error_Code_INTERNAL"),
]


def _program() -> str:
    lines = ["#include <cstddef>", "#include <cstdio>", f'#include "{REFERENCE_HEADER}"',
             f'#include "{os.path.join(ROOT, "e3j_amd", "csrc", "xla_ffi_abi.h")}"', ""]
    for mine, theirs, _, fields in PAIRS:
        if mine != "XlaApi":   # the library's table stops after the last entry it calls
            lines.append(f'static_assert(sizeof({mine}) == sizeof({theirs}), "size of {mine}");')
        for a, b, _ in fields:
            lines.append(f'static_assert(offsetof({mine}, {a}) == offsetof({theirs}, {b}), "{mine}.{a}");')
            lines.append(f'static_assert(sizeof((({mine} *)0)->{a}) == sizeof((({theirs} *)0)->{b}), "{mine}.{a} size");')
    for mine, theirs in CONSTANTS:
        lines.append(f'static_assert((int){mine} == (int){theirs}, "{mine}");')
    lines += ["", "int main() {", '    std::printf("{");']
    first = True
    for _, theirs, _, fields in PAIRS:
        sep = "" if first else ", "
        first = False
        lines.append(f'    std::printf("{sep}\\"{theirs}\\": {{\\"sizeof\\": %zu", sizeof({theirs}));')
        for _, b, _ in fields:
            lines.append(f'    std::printf(", \\"{b}\\": [%zu, %zu]", offsetof({theirs}, {b}), sizeof((({theirs} *)0)->{b}));')
        lines.append('    std::printf("}");')
    lines += ['    std::printf("}\\n");', "    return 0;", "}", ""]
    return "\n".join(lines)


@pytest.fixture(scope="module")
def reference_layout(tmp_path_factory):
    work = tmp_path_factory.mktemp("xla_abi")
    src, exe = work / "layout.cc", work / "layout"
    src.write_text(_program())
    proc = subprocess.run(["g++", "-std=c++17", "-Wno-invalid-offsetof", str(src), "-o", str(exe)],
                          capture_output=True, text=True)
    assert proc.returncode == 0, "xla_ffi_abi.h disagrees with the vendored c_api.h:\n" + proc.stderr
    return json.loads(subprocess.run([str(exe)], capture_output=True, text=True, check=True).stdout)


def test_library_header_matches_the_vendored_c_api(reference_layout):
    """Compiling the program is the check: every static assertion compares the two headers."""
    assert set(reference_layout) == {theirs for _, theirs, _, _ in PAIRS}


def test_ctypes_frames_match_the_vendored_c_api(reference_layout):
    for _, theirs, cls, fields in PAIRS:
        layout = reference_layout[theirs]
        if theirs != "XLA_FFI_Api":
            assert C.sizeof(cls) == layout["sizeof"], theirs
        else:
            assert C.sizeof(cls) == layout["sizeof"], "the fake function table has every slot of the real one"
        for _, b, c in fields:
            field = getattr(cls, c)
            assert [field.offset, field.size] == layout[b], f"{theirs}.{b}"
