// XLA-FFI handlers: decode an XLA_FFI_CallFrame and call the launchers.
//
// Operand order of the reference's targets (lib/e3j_ops/ffi/e3j_ops.h:457-472,575-594):
//   "convolution":      coef, x, y, s, sender, receiver_ptr [, coef_ranges]   -> out
//   "convolution_bwd":  coef, x, y, s, dm, sender_t, receiver_ptr_t, edge_perm [, coef_ranges]
//                                                                   -> dx, dy, ds
// `coef_ranges` is accepted and ignored.  `coef` of "convolution_bwd" may be the
// forward table (rank 2) or the reference's stack of three transposed tables
// (3, nnz, numel) / (3*nnz, numel) flagged by the attribute coef_stacked = 1;
// the first of the three, sorted for dx with columns (j, i, k, l), is then used.
// A third target, "convolution_bwd_receiver", takes the forward's receiver CSR:
//   coef, x, y, s, dm, sender, receiver_ptr, edge_perm -> dx, dy, ds;
// a fourth, "convolution_bwd_ordered", the same operands and a scratch buffer as a fourth
// result (the atomic-free, bit-reproducible backward).
// Attributes: num_nodes, debug (reference); layout, signature, coef_scale, y_flip,
// coef_stacked (optional).  Without `signature` the handler finds the kernels of the table the
// frame carries (see TableResolver: a read-back of the table and a host wait per call; frames that
// name `signature` wait for nothing).  Handlers are re-entrant (the only shared state is the map
// of tables already looked up, behind a mutex), allocate nothing themselves ("convolution_bwd" borrows scratch from the
// runtime through XLA_FFI_DeviceMemory_Allocate when it runs the unrolled kernels, and so does a
// table-driven call for the plan of its table; a runtime without such memory leaves the latter to
// the stream's pool) and enqueue
// on the stream XLA hands over; they answer the metadata query.
//
// The row-wise tensor product (lib/e3j_ops/ffi/e3j_ops.h:124-253,258-372):
//   "tensor_product":      coef, x, y [, coef_ranges] -> z;  attrs num_out, mode, layout, debug
//   "tensor_product_bwd":  coef (2, nnz, numel), x, y, dz [, coef_ranges] -> dx, dy;  attrs mode, layout, debug
// plus the optional attributes signature, coef_scale and coef_sorted (default 1).

#include <cstring>
#include <map>
#include <memory>
#include <mutex>
#include <tuple>
#include <vector>

#include "common.h"
#include "xla_ffi_abi.h"

namespace e3j_amd {
namespace {

void *make_error(const XlaCallFrame *frame, int code, const std::string &msg) {
    XlaErrorCreateArgs args;
    args.struct_size = sizeof(XlaErrorCreateArgs);
    args.extension_start = nullptr;
    args.message = msg.c_str();
    args.errc = code == E3J_AMD_INVALID_ARGUMENT ? kXlaErrInvalidArgument
              : code == E3J_AMD_UNIMPLEMENTED    ? kXlaErrUnimplemented
                                                 : kXlaErrInternal;
    return frame->api->error_create(&args);
}

void *status_to_error(const XlaCallFrame *frame, int rc) {
    return rc == E3J_AMD_OK ? nullptr : make_error(frame, rc, e3j_amd_last_error());
}

// Returns true when the frame is a metadata query (and answers it).
bool answer_metadata(XlaCallFrame *frame) {
    XlaExtensionBase *ext = frame->extension_start;
    if (ext == nullptr || ext->type != kXlaExtMetadata) return false;
    XlaMetadata *md = reinterpret_cast<XlaMetadataExtension *>(ext)->metadata;
    md->api_version.major_version = kXlaFfiApiMajor;
    md->api_version.minor_version = kXlaFfiApiMinor;
    md->traits = 0;
    if (md->struct_size >= offsetof(XlaMetadata, state_type_id) + sizeof(int64_t))
        md->state_type_id = 0;  // stateless handler
    return true;
}

const XlaBuffer *arg(const XlaCallFrame *f, int64_t i) {
    if (i >= f->args.size || f->args.types[i] != kXlaArgBuffer) return nullptr;
    return static_cast<const XlaBuffer *>(f->args.args[i]);
}
const XlaBuffer *ret(const XlaCallFrame *f, int64_t i) {
    if (i >= f->rets.size || f->rets.types[i] != kXlaRetBuffer) return nullptr;
    return static_cast<const XlaBuffer *>(f->rets.rets[i]);
}
size_t dtype_bytes(int32_t dtype) {
    switch (dtype) {
        case kXlaU8: return 1;
        case kXlaF16: return 2;
        case kXlaS32: case kXlaF32: return 4;
        case kXlaS64: case kXlaF64: return 8;
        default: return 1;  // unknown element types are counted as bytes
    }
}

int64_t count(const XlaBuffer *b) {
    int64_t n = 1;
    for (int64_t d = 0; d < b->rank; d++) n *= b->dims[d];
    return n;
}

// Scalar attribute by name; `found` reports presence.
template <typename T>
T attr(const XlaCallFrame *f, const char *name, int32_t dtype, T fallback, bool *found = nullptr) {
    if (found) *found = false;
    const size_t len = std::strlen(name);
    for (int64_t i = 0; i < f->attrs.size; i++) {
        const XlaByteSpan *nm = f->attrs.names[i];
        if (nm->len != len || std::memcmp(nm->ptr, name, len) != 0) continue;
        if (f->attrs.types[i] != kXlaAttrScalar) return fallback;
        const XlaScalar *sc = static_cast<const XlaScalar *>(f->attrs.attrs[i]);
        if (sc->dtype != dtype) return fallback;
        if (found) *found = true;
        T v;
        std::memcpy(&v, sc->value, sizeof(T));
        return v;
    }
    return fallback;
}

// ---- which unrolled kernels serve the table of a frame ----------------------------------------
// The reference's frames carry the coefficient table as a device buffer and no kernel id
// (src/e3j/ops/convolution.py:229-242,433-452).  The handler reads the table back (a few KB) and
// looks it up among the signatures; the answer is remembered under the table's BYTES, never under
// its address (a buffer can be rewritten or reused for a table of the same shape with another
// scale or other signs).  The read runs on a stream of the calling thread that first waits for the
// work already enqueued on the caller's stream (an event), so a table still being written there is
// read after that write; the host waits for the copy.  Frames that carry the attributes
// `signature`, `coef_scale` and `y_flip` skip all of this: that is the path without a host wait.
// Under stream capture nothing can be read back, and nothing is assumed about the buffer: such a
// frame runs the table-driven kernels, which read the table on the device at every replay.
struct ResolvedTable {
    int32_t signature = -1;
    float scale = 1.0f;
    uint32_t flip = 0;
    // float64 tables: the coefficient classes the float64 kernels read (shared with the calls that
    // use them, so that clearing the cache never pulls them away from a call)
    std::shared_ptr<const F64Coefs> classes;
};

class TableResolver {
  public:
    ResolvedTable resolve(const void *device_table, int32_t num_coef, int32_t idx_bytes, bool columns_ji,
                          const e3j_amd_conv_params &p, hipStream_t caller_stream) {
        ResolvedTable none;
        const bool f64 = p.val_dtype == E3J_AMD_F64, f16 = p.val_dtype == E3J_AMD_F16;
        if (num_coef <= 0 || device_table == nullptr) return none;
        // (the float64 and float16 kernels serve the trailing layout)
        if ((f64 || f16) && p.layout != E3J_AMD_LAYOUT_TRAILING) return none;
        const size_t item = f64   ? (idx_bytes == 1 ? sizeof(Coef4D<uint8_t, double>) : sizeof(Coef4D<int32_t, double>))
                            : f16 ? (idx_bytes == 1 ? sizeof(Coef4D<uint8_t, half_t>) : sizeof(Coef4D<int32_t, half_t>))
                                  : (idx_bytes == 1 ? sizeof(Coef4D<uint8_t, float>) : sizeof(Coef4D<int32_t, float>));
        const size_t bytes = item * (size_t)num_coef;
        const Shape shape{num_coef, idx_bytes + (f64 ? 16 : f16 ? 32 : 0), columns_ji ? 1 : 0, p.num_x, p.num_y, p.num_out,
                          p.num_scalars, p.channels, p.layout};
        hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(caller_stream, &capture) != hipSuccess) {
            (void)hipGetLastError();
            return none;
        }
        if (capture != hipStreamCaptureStatusNone) return none;
        int device = 0;
        if (hipGetDevice(&device) != hipSuccess) return none;
        // per thread and device: concurrent handler calls do not share a stream or an event
        thread_local std::map<int, ReadBack> read_backs;
        ReadBack &rb = read_backs[device];
        if (rb.stream == nullptr) {
            if (hipStreamCreateWithFlags(&rb.stream, hipStreamNonBlocking) != hipSuccess ||
                hipEventCreateWithFlags(&rb.after_caller, hipEventDisableTiming) != hipSuccess) {
                rb = ReadBack{};
                (void)hipGetLastError();
                return none;
            }
        }
        std::vector<unsigned char> host(bytes);
        if (hipEventRecord(rb.after_caller, caller_stream) != hipSuccess ||
            hipStreamWaitEvent(rb.stream, rb.after_caller, 0) != hipSuccess ||
            hipMemcpyAsync(host.data(), device_table, bytes, hipMemcpyDeviceToHost, rb.stream) != hipSuccess ||
            hipStreamSynchronize(rb.stream) != hipSuccess) {
            (void)hipGetLastError();
            return none;
        }
        auto key = std::make_pair(shape, std::move(host));
        {
            std::lock_guard<std::mutex> lock(mutex_);
            auto seen = by_content_.find(key);
            if (seen != by_content_.end()) return seen->second.signature == kNoKernel ? none : seen->second;
        }
        // the lookup itself runs without the lock (two threads may do the same one; both find the same)
        ResolvedTable entry;
        if (f64) {
            auto classes = std::make_shared<F64Coefs>();
            entry.signature = match_signature_f64(key.second.data(), idx_bytes, num_coef, p.num_x, p.num_y, p.num_out,
                                                  p.num_scalars, p.channels, p.layout, columns_ji, classes->v,
                                                  &entry.flip);
            entry.classes = std::move(classes);
        } else if (f16) {
            entry.signature = match_signature_f16(key.second.data(), idx_bytes, num_coef, p.num_x, p.num_y, p.num_out,
                                                  p.num_scalars, p.channels, p.layout, columns_ji, &entry.scale,
                                                  &entry.flip);
        } else {
            const std::vector<TableEntry> entries = unpack_entries(key.second.data(), idx_bytes, num_coef, columns_ji);
            entry.signature = match_signature(entries, p.num_x, p.num_y, p.num_out, p.num_scalars, p.channels,
                                              p.layout, &entry.scale, &entry.flip);
        }
        if (entry.signature < 0) entry.signature = kNoKernel;
        {
            std::lock_guard<std::mutex> lock(mutex_);
            if (by_content_.size() > 1024) by_content_.clear();
            by_content_[std::move(key)] = entry;
        }
        return entry.signature == kNoKernel ? none : entry;
    }

  private:
    using Shape = std::tuple<int32_t, int32_t, int32_t, int32_t, int32_t, int32_t, int32_t, int32_t, int32_t>;
    struct ReadBack {
        hipStream_t stream = nullptr;
        hipEvent_t after_caller = nullptr;
    };
    static constexpr int32_t kNoKernel = -2;  // looked up, nothing matches
    std::mutex mutex_;  // guards by_content_ only
    std::map<std::pair<Shape, std::vector<unsigned char>>, ResolvedTable> by_content_;
};

TableResolver &resolver() {
    static TableResolver r;
    return r;
}

struct Decoded {
    e3j_amd_conv_params p;
    hipStream_t stream;
    std::shared_ptr<const F64Coefs> classes;  // what p.coef_classes points to, for the length of the call
};

// Uses the id the frame names, or finds the kernels of the table the frame carries.  float64
// frames are always looked up: their kernels need the table's values (coef_classes), which no
// attribute carries.
void *choose_kernels(XlaCallFrame *f, const char *op, const XlaBuffer *coef, bool columns_ji,
                     Decoded *d, hipStream_t stream) {
    e3j_amd_conv_params *p = &d->p;
    bool named = false;
    (void)attr<int32_t>(f, "signature", kXlaS32, -1, &named);
    if (p->val_dtype == E3J_AMD_F64) {
        named = false;
        p->signature = -1;
        p->y_flip = 0;
    }
    if (named) {
        // an id chosen by the host: at least the table sizes must agree with the operand
        if (p->signature >= 0 && p->signature < e3j_amd_num_signatures() &&
            signature(p->signature).num_coef != p->num_coef)
            return make_error(f, E3J_AMD_INVALID_ARGUMENT,
                              std::string(op) + ": attribute signature names kernels of a table with " +
                                  std::to_string(signature(p->signature).num_coef) + " entries, the coef operand has " +
                                  std::to_string(p->num_coef));
        return nullptr;
    }
    const ResolvedTable found = resolver().resolve(coef->data, p->num_coef, p->coef_idx_bytes, columns_ji, *p, stream);
    if (found.signature >= 0 && (p->val_dtype != E3J_AMD_F64 || found.classes)) {
        p->signature = found.signature;
        p->coef_scale = found.scale;
        p->y_flip = found.flip;
        d->classes = found.classes;
        p->coef_classes = found.classes ? found.classes->v : nullptr;
    }
    return nullptr;
}

// Fills sizes from the buffers, following the reference's handler
// (lib/e3j_ops/ffi/e3j_ops.h:393-414,496-519).  Returns an XLA error or nullptr.
void *decode_common(XlaCallFrame *f, const char *op, const XlaBuffer *coef, const XlaBuffer *x,
                    const XlaBuffer *y, const XlaBuffer *s, const XlaBuffer *node_rows, Decoded *d) {
    const std::string name(op);
    if (!coef || !x || !y || !s || !node_rows)
        return make_error(f, E3J_AMD_INVALID_ARGUMENT, name + ": missing or non-buffer operand");
    if (x->rank < 2 || x->rank > 3 || y->rank < 2 || s->rank < 2 || node_rows->rank < 2)
        return make_error(f, E3J_AMD_INVALID_ARGUMENT, name + ": operand rank");
    e3j_amd_conv_params &p = d->p;
    std::memset(&p, 0, sizeof(p));
    bool has_nodes = false;
    p.num_nodes = attr<int32_t>(f, "num_nodes", kXlaS32, 0, &has_nodes);
    if (!has_nodes) return make_error(f, E3J_AMD_INVALID_ARGUMENT, name + ": attribute num_nodes (i32) is required");
    p.debug = attr<int32_t>(f, "debug", kXlaS32, 0);
    p.layout = attr<int32_t>(f, "layout", kXlaS32, E3J_AMD_LAYOUT_TRAILING);
    p.signature = attr<int32_t>(f, "signature", kXlaS32, -1);
    p.coef_scale = attr<float>(f, "coef_scale", kXlaF32, 1.0f);
    p.y_flip = (uint32_t)attr<int32_t>(f, "y_flip", kXlaS32, 0);
    p.num_edges = y->dims[0];
    p.num_y = (int32_t)y->dims[1];
    if (y->rank == 3 && y->dims[2] != 1)
        return make_error(f, E3J_AMD_UNIMPLEMENTED, name + ": RHS y should have only one channel.");
    const bool leading = p.layout == E3J_AMD_LAYOUT_LEADING;
    if (x->rank == 2) {
        p.channels = 1;
        p.num_x = (int32_t)x->dims[1];
        p.num_scalars = (int32_t)s->dims[1];
        p.num_out = (int32_t)node_rows->dims[1];
    } else {
        p.channels = (int32_t)(leading ? x->dims[1] : x->dims[2]);
        p.num_x = (int32_t)(leading ? x->dims[2] : x->dims[1]);
        p.num_scalars = (int32_t)(s->rank == 3 ? (leading ? s->dims[2] : s->dims[1]) : s->dims[1]);
        p.num_out = (int32_t)(node_rows->rank == 3 ? (leading ? node_rows->dims[2] : node_rows->dims[1])
                                                    : node_rows->dims[1]);
    }
    if (x->dims[0] != p.num_nodes || node_rows->dims[0] != p.num_nodes)
        return make_error(f, E3J_AMD_INVALID_ARGUMENT, name + ": node operands must have num_nodes rows");
    if (s->dims[0] != p.num_edges)
        return make_error(f, E3J_AMD_INVALID_ARGUMENT, name + ": y and s must have one row per edge");
    if (coef->dtype == kXlaU8) p.coef_idx_bytes = 1;
    else if (coef->dtype == kXlaS32) p.coef_idx_bytes = 4;
    else return make_error(f, E3J_AMD_INVALID_ARGUMENT, "unsupported (IDX, VAL) dtype pair");
    if (x->dtype == kXlaF32) p.val_dtype = E3J_AMD_F32;
    else if (x->dtype == kXlaF64) p.val_dtype = E3J_AMD_F64;
    else if (x->dtype == kXlaF16) p.val_dtype = E3J_AMD_F16;
    else return make_error(f, E3J_AMD_INVALID_ARGUMENT, "unsupported (IDX, VAL) dtype pair");
    if (y->dtype != x->dtype || s->dtype != x->dtype || node_rows->dtype != x->dtype)
        return make_error(f, E3J_AMD_INVALID_ARGUMENT, name + ": value operands must share one dtype");

    XlaStreamGetArgs sg;
    sg.struct_size = sizeof(XlaStreamGetArgs);
    sg.extension_start = nullptr;
    sg.ctx = f->ctx;
    sg.stream = nullptr;
    if (void *err = f->api->stream_get(&sg)) return err;
    d->stream = static_cast<hipStream_t>(sg.stream);
    return nullptr;
}

bool is_s32_vector(const XlaBuffer *b) { return b && b->dtype == kXlaS32 && b->rank == 1; }

enum class Backward { kSenderRows, kReceiverRows, kReceiverRowsOrdered };

size_t align256(size_t n) { return (n + 255) / 256 * 256; }

// Scratch memory of the runtime for the length of a handler call (XLA_FFI_DeviceMemory_Allocate /
// _Free; the runtime's allocator orders the reuse of the block after the work enqueued on the
// call's stream).  `data` stays null when the runtime offers none or nothing is asked for.
struct RuntimeScratch {
    XlaCallFrame *frame;
    void *data = nullptr;
    size_t size;
    RuntimeScratch(XlaCallFrame *f, size_t bytes) : frame(f), size(bytes) {
        const XlaApi *api = f->api;
        if (bytes == 0 || api->struct_size < offsetof(XlaApi, device_memory_free) + sizeof(void *) ||
            api->device_memory_allocate == nullptr || api->device_memory_free == nullptr)
            return;
        XlaDeviceMemoryAllocateArgs get;
        get.struct_size = sizeof(get);
        get.extension_start = nullptr;
        get.ctx = f->ctx;
        get.size = bytes;
        get.alignment = 256;
        get.data = nullptr;
        if (api->device_memory_allocate(&get) == nullptr) data = get.data;
    }
    ~RuntimeScratch() {
        if (data == nullptr) return;
        XlaDeviceMemoryFreeArgs give;
        give.struct_size = sizeof(give);
        give.extension_start = nullptr;
        give.ctx = frame->ctx;
        give.size = size;
        give.data = data;
        (void)frame->api->device_memory_free(&give);
    }
    RuntimeScratch(const RuntimeScratch &) = delete;
    RuntimeScratch &operator=(const RuntimeScratch &) = delete;
};

// The plan of a table-driven call in the runtime's memory: the library then allocates nothing and
// the planned kernels also run while the runtime records the stream into a graph.
struct TablePlanMemory : RuntimeScratch {
    TablePlanMemory(XlaCallFrame *f, e3j_amd_conv_params *p)
        : RuntimeScratch(f, p->signature < 0 ? e3j_amd_table_plan_bytes(p) : 0) {
        p->table_plan = static_cast<int32_t *>(data);
    }
};

// "convolution_bwd" as the reference sends it (receiver_t per position of the sender-grouped
// adjacency, sender_ptr, edge_perm) on the receiver-grouped unrolled kernels: positions are
// sorted by receiver (stable), which gives sender per position, receiver_ptr and, composed with
// edge_perm, the row of y / s / dy / ds of every position.  `done` is left false when the
// runtime hands out no scratch memory.
void *backward_on_receiver_rows(XlaCallFrame *f, const char *op, Decoded *d, const XlaBuffer *coef, bool stacked,
                                const XlaBuffer *x, const XlaBuffer *y, const XlaBuffer *s, const XlaBuffer *dm,
                                const XlaBuffer *receiver_t, const XlaBuffer *sender_ptr, const int32_t *perm,
                                const XlaBuffer *dx, const XlaBuffer *dy, const XlaBuffer *ds, bool *done) {
    *done = false;
    const XlaApi *api = f->api;
    if (api->struct_size < offsetof(XlaApi, device_memory_free) + sizeof(void *) ||
        api->device_memory_allocate == nullptr || api->device_memory_free == nullptr)
        return nullptr;
    const e3j_amd_conv_params &p = d->p;
    const size_t e = (size_t)p.num_edges, n = (size_t)p.num_nodes;
    const size_t vec = align256(4 * e);
    const size_t csr = align256(e3j_amd_csr_workspace_bytes(p.num_nodes, p.num_edges));
    const size_t total = 4 * vec + align256(4 * (n + 1)) + csr;
    XlaDeviceMemoryAllocateArgs get;
    get.struct_size = sizeof(get);
    get.extension_start = nullptr;
    get.ctx = f->ctx;
    get.size = total;
    get.alignment = 256;
    get.data = nullptr;
    if (void *err = api->device_memory_allocate(&get)) {
        (void)err;  // ownership of the error object stays with the runtime's bookkeeping
        return nullptr;
    }
    if (get.data == nullptr) return nullptr;
    unsigned char *base = static_cast<unsigned char *>(get.data);
    int32_t *senders = reinterpret_cast<int32_t *>(base);
    int32_t *by_receiver = reinterpret_cast<int32_t *>(base + vec);
    int32_t *sender_sorted = reinterpret_cast<int32_t *>(base + 2 * vec);
    int32_t *edge_rows = reinterpret_cast<int32_t *>(base + 3 * vec);
    int32_t *receiver_ptr = reinterpret_cast<int32_t *>(base + 4 * vec);
    void *workspace = base + 4 * vec + align256(4 * (n + 1));
    hipStream_t stream = d->stream;
    int rc = launch_expand_rows(static_cast<const int32_t *>(sender_ptr->data), p.num_nodes, p.num_edges, senders,
                                stream);
    if (rc == E3J_AMD_OK)
        rc = e3j_amd_sort_edges(static_cast<const int32_t *>(receiver_t->data), senders, p.num_edges, p.num_nodes,
                                by_receiver, sender_sorted, receiver_ptr, workspace, stream);
    if (rc == E3J_AMD_OK) rc = launch_compose_perm(by_receiver, perm, p.num_edges, edge_rows, stream);
    if (rc == E3J_AMD_OK)
        rc = run_backward(&p, true, coef->data, x->data, y->data, s->data, dm->data, sender_sorted, receiver_ptr,
                          edge_rows, dx->data, dy->data, ds->data, stream, stacked);
    // the runtime's allocator orders the reuse of the block after the work enqueued on this stream
    XlaDeviceMemoryFreeArgs give;
    give.struct_size = sizeof(give);
    give.extension_start = nullptr;
    give.ctx = f->ctx;
    give.size = total;
    give.data = get.data;
    void *free_err = api->device_memory_free(&give);
    *done = true;
    if (rc != E3J_AMD_OK) return status_to_error(f, rc);
    return free_err;
    (void)op;
}

void *backward_handler(XlaCallFrame *f, Backward mode) {
    const bool group_is_receiver = mode != Backward::kSenderRows;
    const bool ordered = mode == Backward::kReceiverRowsOrdered;
    const char *op = ordered ? "convolution_bwd_ordered"
                             : group_is_receiver ? "convolution_bwd_receiver" : "convolution_bwd";
    if (answer_metadata(f)) return nullptr;
    if (f->stage != kXlaStageExecute) return nullptr;
    if (f->args.size < 8 || f->rets.size != (ordered ? 4 : 3))
        return make_error(f, E3J_AMD_INVALID_ARGUMENT,
                          std::string(op) + (ordered ? ": expected 8 operands and 4 results (dx, dy, ds, workspace)"
                                                     : ": expected 8 or 9 operands and 3 results"));
    const XlaBuffer *coef = arg(f, 0), *x = arg(f, 1), *y = arg(f, 2), *s = arg(f, 3), *dm = arg(f, 4);
    const XlaBuffer *other = arg(f, 5), *row_ptr = arg(f, 6), *perm = arg(f, 7);
    const XlaBuffer *dx = ret(f, 0), *dy = ret(f, 1), *ds = ret(f, 2);
    Decoded d;
    if (void *err = decode_common(f, op, coef, x, y, s, dm, &d)) return err;
    if (!is_s32_vector(other) || !is_s32_vector(row_ptr) || !is_s32_vector(perm) || !dx || !dy || !ds)
        return make_error(f, E3J_AMD_INVALID_ARGUMENT, std::string(op) + ": adjacency operands must be S32 vectors");
    if (count(other) != d.p.num_edges || count(row_ptr) != (int64_t)d.p.num_nodes + 1 ||
        (count(perm) != 0 && count(perm) != d.p.num_edges))
        return make_error(f, E3J_AMD_INVALID_ARGUMENT, std::string(op) + ": adjacency operand sizes");
    if (count(dx) != count(x) || count(dy) != count(y) || count(ds) != count(s))
        return make_error(f, E3J_AMD_INVALID_ARGUMENT, std::string(op) + ": result shapes");
    const int32_t stacked = attr<int32_t>(f, "coef_stacked", kXlaS32, coef->rank == 3 ? 1 : 0);
    const int64_t numel = coef->dims[coef->rank - 1];
    d.p.num_coef = (int32_t)(count(coef) / numel / (stacked ? 3 : 1));
    const int32_t *perm_ptr = count(perm) ? static_cast<const int32_t *>(perm->data) : nullptr;
    if (void *err = choose_kernels(f, op, coef, stacked != 0, &d, d.stream)) return err;
    // The reference's operands: the adjacency grouped by sender.  The unrolled kernels of that
    // grouping (trailing layout; a row owns its dx) pay a gather of dm rows per edge: faster than
    // a rebuild of the receiver rows (a dozen small launches) plus the receiver-grouped kernel on
    // graphs below about a quarter of a million edges (150k edges, 64 channels: 0.36 against
    // 0.44 ms), slower above (960k edges, 64 channels: 4.07 against 3.62 + 0.2 ms).  Large graphs
    // therefore get their receiver CSR rebuilt in scratch memory of the runtime; without such
    // memory run_backward keeps the sender rows (unrolled in the trailing layout, else table-driven).
    // (the sender-grouped unrolled kernels are float32 kernels: other dtypes always go by receiver rows)
    const bool small_graph = d.p.layout == E3J_AMD_LAYOUT_TRAILING && d.p.num_edges < (1 << 18) &&
                             d.p.val_dtype == E3J_AMD_F32;
    if (mode == Backward::kSenderRows && d.p.signature >= 0 && !small_graph) {
        bool done = false;
        void *err = backward_on_receiver_rows(f, op, &d, coef, stacked != 0, x, y, s, dm, other, row_ptr, perm_ptr,
                                              dx, dy, ds, &done);
        if (err != nullptr || done) return err;
    }
    if (mode == Backward::kSenderRows && d.p.val_dtype != E3J_AMD_F32) {
        // no scratch to rebuild receiver rows in, and the float64 / float16 unrolled kernels walk
        // receiver rows only: the sender rows stay with the table-driven kernel
        d.p.signature = -1;
        d.p.y_flip = 0;
    }
    if (ordered) {
        // the scratch of the atomic-free backward travels as a fourth result buffer (any dtype)
        const XlaBuffer *workspace = ret(f, 3);
        if (!workspace || workspace->data == nullptr ||
            (size_t)count(workspace) * dtype_bytes(workspace->dtype) <
                e3j_amd_convolution_bwd_ordered_workspace_bytes(&d.p))
            return make_error(f, E3J_AMD_INVALID_ARGUMENT,
                              std::string(op) + ": the workspace result is smaller than "
                                                "e3j_amd_convolution_bwd_ordered_workspace_bytes");
        const int rc = e3j_amd_convolution_bwd_ordered(
            &d.p, coef->data, x->data, y->data, s->data, dm->data, static_cast<const int32_t *>(other->data),
            static_cast<const int32_t *>(row_ptr->data), perm_ptr, dx->data, dy->data, ds->data,
            workspace->data, d.stream);
        return status_to_error(f, rc);
    }
    const TablePlanMemory plan(f, &d.p);
    const int rc = run_backward(&d.p, group_is_receiver, coef->data, x->data, y->data, s->data, dm->data,
                                static_cast<const int32_t *>(other->data),
                                static_cast<const int32_t *>(row_ptr->data), perm_ptr, dx->data,
                                dy->data, ds->data, d.stream, stacked != 0);
    return status_to_error(f, rc);
}

// Sizes of the tensor product from the buffer shapes (lib/e3j_ops/ffi/e3j_ops.h:146-187,285-309).
void *decode_tensor_product(XlaCallFrame *f, const char *op, const XlaBuffer *coef, const XlaBuffer *x,
                            const XlaBuffer *y, e3j_amd_tp_params *p, hipStream_t *stream) {
    const std::string name(op);
    if (!coef || !x || !y) return make_error(f, E3J_AMD_INVALID_ARGUMENT, name + ": missing or non-buffer operand");
    if (x->rank < 2 || x->rank > 3 || y->rank < 2 || y->rank > 3 || coef->rank < 2)
        return make_error(f, E3J_AMD_INVALID_ARGUMENT, name + ": operand rank");
    std::memset(p, 0, sizeof(*p));
    bool has_mode = false, has_layout = false;
    p->mode = attr<int32_t>(f, "mode", kXlaS32, 0, &has_mode);
    p->layout = attr<int32_t>(f, "layout", kXlaS32, 0, &has_layout);
    if (!has_mode || !has_layout)
        return make_error(f, E3J_AMD_INVALID_ARGUMENT, name + ": attributes mode and layout (i32) are required");
    p->debug = attr<int32_t>(f, "debug", kXlaS32, 0);
    p->signature = attr<int32_t>(f, "signature", kXlaS32, -1);
    p->coef_scale = attr<float>(f, "coef_scale", kXlaF32, 1.0f);
    p->coef_sorted = attr<int32_t>(f, "coef_sorted", kXlaS32, 1);
    const bool leading = p->layout == E3J_AMD_LAYOUT_LEADING;
    p->num_rows = x->dims[0];
    p->num_x = (int32_t)(x->rank == 3 && !leading ? x->dims[1] : x->dims[x->rank - 1]);
    p->num_y = (int32_t)(y->rank == 3 && !leading ? y->dims[1] : y->dims[y->rank - 1]);
    p->channels_x = (int32_t)(x->rank == 3 ? (leading ? x->dims[1] : x->dims[2]) : 1);
    p->channels_y = (int32_t)(y->rank == 3 ? (leading ? y->dims[1] : y->dims[2]) : 1);
    if (y->dims[0] != p->num_rows)
        return make_error(f, E3J_AMD_INVALID_ARGUMENT, name + ": x and y must have as many rows");
    if (coef->dtype == kXlaU8) p->coef_idx_bytes = 1;
    else if (coef->dtype == kXlaS32) p->coef_idx_bytes = 4;
    else return make_error(f, E3J_AMD_INVALID_ARGUMENT, "unsupported (IDX, VAL) dtype pair");
    if (x->dtype == kXlaF32) p->val_dtype = E3J_AMD_F32;
    else if (x->dtype == kXlaF64) p->val_dtype = E3J_AMD_F64;
    else if (x->dtype == kXlaF16) p->val_dtype = E3J_AMD_F16;
    else return make_error(f, E3J_AMD_INVALID_ARGUMENT, "unsupported (IDX, VAL) dtype pair");
    if (y->dtype != x->dtype)
        return make_error(f, E3J_AMD_INVALID_ARGUMENT, name + ": value operands must share one dtype");
    XlaStreamGetArgs sg;
    sg.struct_size = sizeof(XlaStreamGetArgs);
    sg.extension_start = nullptr;
    sg.ctx = f->ctx;
    sg.stream = nullptr;
    if (void *err = f->api->stream_get(&sg)) return err;
    *stream = static_cast<hipStream_t>(sg.stream);
    return nullptr;
}

int64_t tp_out_count(const e3j_amd_tp_params &p) {
    const int64_t chans = p.mode == E3J_AMD_MODE_OUTER ? (int64_t)p.channels_x * p.channels_y
                        : p.mode == E3J_AMD_MODE_INNER ? 1 : p.channels_x;
    return p.num_rows * p.num_out * chans;
}

}  // namespace
}  // namespace e3j_amd

using namespace e3j_amd;

extern "C" {

void *e3j_amd_xla_convolution(void *call_frame) {
    XlaCallFrame *f = static_cast<XlaCallFrame *>(call_frame);
    if (answer_metadata(f)) return nullptr;
    if (f->stage != kXlaStageExecute) return nullptr;
    if (f->args.size < 6 || f->rets.size != 1)
        return make_error(f, E3J_AMD_INVALID_ARGUMENT, "convolution: expected 6 to 8 operands and 1 result");
    const XlaBuffer *coef = arg(f, 0), *x = arg(f, 1), *y = arg(f, 2), *s = arg(f, 3);
    const XlaBuffer *sender = arg(f, 4), *row_ptr = arg(f, 5), *out = ret(f, 0);
    // operand 6 is the reference's coef_ranges (ignored); operand 7, if present, an edge permutation
    const XlaBuffer *perm = f->args.size >= 8 ? arg(f, 7) : nullptr;
    Decoded d;
    if (void *err = decode_common(f, "convolution", coef, x, y, s, out, &d)) return err;
    if (!is_s32_vector(sender) || !is_s32_vector(row_ptr) || (f->args.size >= 8 && !is_s32_vector(perm)))
        return make_error(f, E3J_AMD_INVALID_ARGUMENT, "convolution: adjacency operands must be S32 vectors");
    if (count(sender) != d.p.num_edges || count(row_ptr) != (int64_t)d.p.num_nodes + 1 ||
        (perm && count(perm) != 0 && count(perm) != d.p.num_edges))
        return make_error(f, E3J_AMD_INVALID_ARGUMENT, "convolution: adjacency operand sizes");
    d.p.num_coef = (int32_t)coef->dims[0];
    if (void *err = choose_kernels(f, "convolution", coef, false, &d, d.stream)) return err;
    const int32_t *perm_ptr = (perm && count(perm)) ? static_cast<const int32_t *>(perm->data) : nullptr;
    const TablePlanMemory plan(f, &d.p);
    const int rc = e3j_amd_convolution_fwd(&d.p, coef->data, x->data, y->data, s->data,
                                           static_cast<const int32_t *>(sender->data),
                                           static_cast<const int32_t *>(row_ptr->data), perm_ptr,
                                           out->data, d.stream);
    return status_to_error(f, rc);
}

void *e3j_amd_xla_tensor_product(void *call_frame) {
    XlaCallFrame *f = static_cast<XlaCallFrame *>(call_frame);
    if (answer_metadata(f)) return nullptr;
    if (f->stage != kXlaStageExecute) return nullptr;
    if (f->args.size < 3 || f->args.size > 4 || f->rets.size != 1)
        return make_error(f, E3J_AMD_INVALID_ARGUMENT, "tensor_product: expected 3 or 4 operands and 1 result");
    const XlaBuffer *coef = arg(f, 0), *x = arg(f, 1), *y = arg(f, 2), *z = ret(f, 0);
    e3j_amd_tp_params p;
    hipStream_t stream;
    if (void *err = decode_tensor_product(f, "tensor_product", coef, x, y, &p, &stream)) return err;
    bool has_out = false;
    p.num_out = attr<int32_t>(f, "num_out", kXlaS32, 0, &has_out);
    if (!has_out) return make_error(f, E3J_AMD_INVALID_ARGUMENT, "tensor_product: attribute num_out (i32) is required");
    p.num_coef = (int32_t)coef->dims[0];
    if (!z || z->dtype != x->dtype || count(z) != tp_out_count(p))
        return make_error(f, E3J_AMD_INVALID_ARGUMENT, "tensor_product: result shape or dtype");
    return status_to_error(f, e3j_amd_tensor_product_fwd(&p, coef->data, x->data, y->data, z->data, stream));
}

void *e3j_amd_xla_tensor_product_bwd(void *call_frame) {
    XlaCallFrame *f = static_cast<XlaCallFrame *>(call_frame);
    if (answer_metadata(f)) return nullptr;
    if (f->stage != kXlaStageExecute) return nullptr;
    if (f->args.size < 4 || f->args.size > 5 || f->rets.size != 2)
        return make_error(f, E3J_AMD_INVALID_ARGUMENT, "tensor_product_bwd: expected 4 or 5 operands and 2 results");
    const XlaBuffer *coef = arg(f, 0), *x = arg(f, 1), *y = arg(f, 2), *dz = arg(f, 3);
    const XlaBuffer *dx = ret(f, 0), *dy = ret(f, 1);
    e3j_amd_tp_params p;
    hipStream_t stream;
    if (void *err = decode_tensor_product(f, "tensor_product_bwd", coef, x, y, &p, &stream)) return err;
    if (!dz || dz->rank < 2 || dz->dtype != x->dtype)
        return make_error(f, E3J_AMD_INVALID_ARGUMENT, "tensor_product_bwd: cotangent operand");
    // the two transposed tables arrive stacked; sizes as the reference takes them (e3j_ops.h:279-283,298-300)
    const int64_t numel = coef->dims[coef->rank - 1];
    p.num_coef = (int32_t)(count(coef) / (2 * numel));
    const bool leading = p.layout == E3J_AMD_LAYOUT_LEADING;
    p.num_out = (int32_t)(dz->rank == 2 || leading ? dz->dims[dz->rank - 1] : dz->dims[1]);
    if (dz->dims[0] != p.num_rows || count(dz) != tp_out_count(p))
        return make_error(f, E3J_AMD_INVALID_ARGUMENT, "tensor_product_bwd: cotangent shape");
    if (!dx || !dy || count(dx) != count(x) || count(dy) != count(y) || dx->dtype != x->dtype || dy->dtype != x->dtype)
        return make_error(f, E3J_AMD_INVALID_ARGUMENT, "tensor_product_bwd: result shapes");
    return status_to_error(f, e3j_amd_tensor_product_bwd(&p, coef->data, x->data, y->data, dz->data, dx->data,
                                                         dy->data, stream));
}

void *e3j_amd_xla_convolution_bwd(void *call_frame) {
    return backward_handler(static_cast<XlaCallFrame *>(call_frame), Backward::kSenderRows);
}

void *e3j_amd_xla_convolution_bwd_receiver(void *call_frame) {
    return backward_handler(static_cast<XlaCallFrame *>(call_frame), Backward::kReceiverRows);
}

void *e3j_amd_xla_convolution_bwd_ordered(void *call_frame) {
    return backward_handler(static_cast<XlaCallFrame *>(call_frame), Backward::kReceiverRowsOrdered);
}

}  // extern "C"
