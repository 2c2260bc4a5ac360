// Minimal description of the OpenXLA FFI C ABI (API version 0.2), written for
// this library: only the structures a handler touches, in the field order the
// ABI fixes (OpenXLA xla/ffi/api/c_api.h; the copy the reference vendors is
// lib/e3j_ops/xla/ffi/api/c_api.h:52-56,96-101,150-155,228-236,277-286,
// 403-454,577-583,595-620,722-739,749-773).  Function-table slots that this library
// never calls are typed as opaque pointers.
#ifndef E3J_AMD_CSRC_XLA_FFI_ABI_H_
#define E3J_AMD_CSRC_XLA_FFI_ABI_H_

#include <stddef.h>
#include <stdint.h>

extern "C" {

enum { kXlaFfiApiMajor = 0, kXlaFfiApiMinor = 2 };
enum { kXlaExtMetadata = 1 };
enum { kXlaArgBuffer = 1, kXlaRetBuffer = 1 };
enum { kXlaAttrArray = 1, kXlaAttrDictionary = 2, kXlaAttrScalar = 3, kXlaAttrString = 4 };
enum { kXlaStageExecute = 3 };
// element types (xla::PrimitiveType numbering)
enum { kXlaS32 = 4, kXlaS64 = 5, kXlaU8 = 6, kXlaF16 = 10, kXlaF32 = 11, kXlaF64 = 12 };
// error codes (absl::StatusCode numbering)
enum { kXlaErrInvalidArgument = 3, kXlaErrUnimplemented = 12, kXlaErrInternal = 13 };

struct XlaExtensionBase {
    size_t struct_size;
    int32_t type;
    XlaExtensionBase *next;
};

struct XlaApiVersion {
    size_t struct_size;
    XlaExtensionBase *extension_start;
    int major_version;
    int minor_version;
};

struct XlaByteSpan {
    const char *ptr;
    size_t len;
};

struct XlaScalar {
    int32_t dtype;
    void *value;
};

struct XlaBuffer {
    size_t struct_size;
    XlaExtensionBase *extension_start;
    int32_t dtype;
    void *data;
    int64_t rank;
    int64_t *dims;
};

struct XlaArgs {
    size_t struct_size;
    XlaExtensionBase *extension_start;
    int64_t size;
    int32_t *types;
    void **args;
};

struct XlaRets {
    size_t struct_size;
    XlaExtensionBase *extension_start;
    int64_t size;
    int32_t *types;
    void **rets;
};

struct XlaAttrs {
    size_t struct_size;
    XlaExtensionBase *extension_start;
    int64_t size;
    int32_t *types;
    XlaByteSpan **names;
    void **attrs;
};

struct XlaApi;

struct XlaCallFrame {
    size_t struct_size;
    XlaExtensionBase *extension_start;
    const XlaApi *api;
    void *ctx;
    int32_t stage;
    XlaArgs args;
    XlaRets rets;
    XlaAttrs attrs;
    void *future;
};

struct XlaErrorCreateArgs {
    size_t struct_size;
    XlaExtensionBase *extension_start;
    const char *message;
    int32_t errc;
};

struct XlaStreamGetArgs {
    size_t struct_size;
    XlaExtensionBase *extension_start;
    void *ctx;
    void *stream;  // out
};

struct XlaDeviceMemoryAllocateArgs {
    size_t struct_size;
    XlaExtensionBase *extension_start;
    void *ctx;
    size_t size;
    size_t alignment;
    void *data;  // out
};

struct XlaDeviceMemoryFreeArgs {
    size_t struct_size;
    XlaExtensionBase *extension_start;
    void *ctx;
    size_t size;
    void *data;
};

struct XlaMetadata {
    size_t struct_size;
    XlaApiVersion api_version;
    uint32_t traits;
    int64_t state_type_id;
};

struct XlaMetadataExtension {
    XlaExtensionBase base;
    XlaMetadata *metadata;
};

struct XlaApi {
    size_t struct_size;
    XlaExtensionBase *extension_start;
    XlaApiVersion api_version;
    const void *internal_api;
    void *(*error_create)(XlaErrorCreateArgs *);
    void *error_get_message;
    void *error_destroy;
    void *handler_register;
    void *(*stream_get)(XlaStreamGetArgs *);
    void *type_register;
    void *execution_context_get;
    void *state_set;
    void *state_get;
    void *(*device_memory_allocate)(XlaDeviceMemoryAllocateArgs *);
    void *(*device_memory_free)(XlaDeviceMemoryFreeArgs *);
    // thread_pool_schedule, thread_pool_num_threads, future_create, future_set_available,
    // future_set_error, run_id_get, device_ordinal_get follow; unused.
};

}  // extern "C"
#endif
