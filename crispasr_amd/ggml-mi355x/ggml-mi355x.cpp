// ggml-mi355x: a minimal ggml backend that claims GGML_OP_FLASH_ATTN_EXT (and the copies it needs) and runs
// it through libmi355x_fattn.so; every other op stays on ggml-cpu, routed by ggml_backend_sched.
//
// NOT COMPILED IN THIS REPOSITORY: ggml's headers (ggml.h, ggml-backend.h, ggml-backend-impl.h) are an empty
// submodule in the reference tree.  The vtables below are filled member by member, by name, from the v0.17 API as
// recalled (the buffer vtable's members are the ones the reference's own initialiser names,
// src/core/gguf_loader.cpp:332-344): a member that the real headers do not have, or spell differently, fails to
// compile instead of shifting function pointers into the wrong slots.  Build, once ggml is available:
//   g++ -std=c++17 -fPIC -shared -DGGML_BACKEND_DL -I$GGML/include -I$GGML/src -I../../include \
//       ggml-mi355x.cpp -L.. -lmi355x_fattn -o libggml-mi355x.so
// and let ggml_backend_load_all() pick it up (examples/cli/cli.cpp:2416).
#include "ggml-backend-impl.h"
#include "ggml-backend.h"
#include "ggml.h"

#include "mi355x_fattn.h"

#include <cstdlib>
#include <cstring>
#include <string>

// ---- helpers ---------------------------------------------------------------------------------------------

static mi355x_tensor to_mi(const ggml_tensor * t) {
    mi355x_tensor m;
    m.data = t->data;
    m.type = (int32_t)t->type;                  // GGML_TYPE_F32 = 0, F16 = 1, Q4_0 = 2, Q4_1 = 3, Q5_0 = 6, Q5_1 = 7, Q8_0 = 8: the ids the library uses
    for (int i = 0; i < 4; i++) { m.ne[i] = t->ne[i]; m.nb[i] = t->nb[i]; }
    return m;
}

// The same at planning time (supports_op runs before the graph is allocated, data may still be NULL): the library only
// looks at the alignment of data pointers there, so it gets the low bits the address will have.  Buffers of this backend
// start on 256 bytes (buft_align) and the allocator places tensors on that alignment; a view adds its offset into the
// tensor it views.
static mi355x_tensor to_mi_planning(const ggml_tensor * t) {
    mi355x_tensor m = to_mi(t);
    size_t low = 0;
    if (t->data) {
        low = (size_t)(uintptr_t)t->data % 256;
    } else {
        for (const ggml_tensor * v = t; v && v->view_src; v = v->view_src) low += v->view_offs;
        low %= 256;
    }
    m.data = (void *)(uintptr_t)low;            // never dereferenced by mi355x_*_supports
    return m;
}

static mi355x_fattn_params fa_params(const ggml_tensor * node) {
    mi355x_fattn_params p;
    std::memset(&p, 0, sizeof(p));
    std::memcpy(&p.scale,         (const float *)node->op_params + 0, sizeof(float));
    std::memcpy(&p.max_bias,      (const float *)node->op_params + 1, sizeof(float));
    std::memcpy(&p.logit_softcap, (const float *)node->op_params + 2, sizeof(float));
    p.prec = ((const int32_t *)node->op_params)[3];
    // GGML_MI355X_MATCH_CPU=1: quantise the query rows to Q8_0 when K is Q8_0, the arithmetic ggml-cpu is recalled to
    // use there - for comparison runs (test-backend-ops, transcript diffs), not for production
    static const bool match_cpu = getenv("GGML_MI355X_MATCH_CPU") != nullptr;
    if (match_cpu && node->src[1]->type == GGML_TYPE_Q8_0 && node->src[0]->ne[0] % 32 == 0) p.q_quant = MI355X_TYPE_Q8_0;
    return p;
}

// ---- buffer type: pinned, GPU-mapped host memory ------------------------------------------------------------
// The runtimes place weights and KV caches in the first GPU device's default buffer type
// (src/crispasr.cpp:1940-1944, 3942-3971; src/core/gguf_loader.cpp:722-741).  For ggml-cpu to keep running
// every other op on those tensors the buffer must be host memory (is_host = true); the GPU addresses the same
// pages.  A KV cache in such a buffer does not cross the host link on every attention call: the library gives the
// buffer a mirror in HBM when the graph's first KV write (a CPY or SET_ROWS node whose destination lies in it - this
// backend is the first one that supports both the buffer and the op, so the scheduler hands those nodes here) reaches
// it, keeps both copies equal on every write that goes through its entry points - which is every call of the buffer
// vtable below - and reads K and V from the mirror (mi355x_fattn.h, mi355x_host_buffer_alloc).  Nothing here has to
// know: the vtable passes host pointers.  A second buffer type in plain HBM exists for callers that ask for it by name.

struct mi355x_buffer_ctx { void * base; bool device; };

static void   buf_free(ggml_backend_buffer_t b) {
    auto * c = (mi355x_buffer_ctx *)b->context;
    if (c->device) mi355x_buffer_free(c->base); else mi355x_host_buffer_free(c->base);
    delete c;
}
static void * buf_base(ggml_backend_buffer_t b) { return ((mi355x_buffer_ctx *)b->context)->base; }
static enum ggml_status buf_init_tensor(ggml_backend_buffer_t, ggml_tensor *) { return GGML_STATUS_SUCCESS; }
static void buf_memset(ggml_backend_buffer_t, ggml_tensor * t, uint8_t v, size_t off, size_t n) {
    mi355x_buffer_memset((char *)t->data + off, v, n, nullptr);
    mi355x_stream_synchronize(nullptr);
}
static void buf_set(ggml_backend_buffer_t, ggml_tensor * t, const void * d, size_t off, size_t n) {
    mi355x_buffer_set((char *)t->data + off, d, n, nullptr);
}
static void buf_get(ggml_backend_buffer_t, const ggml_tensor * t, void * d, size_t off, size_t n) {
    mi355x_buffer_get(d, (const char *)t->data + off, n, nullptr);
}
static bool buf_cpy(ggml_backend_buffer_t, const ggml_tensor * src, ggml_tensor * dst) {
    if (!ggml_backend_buffer_is_host(src->buffer) && src->buffer->iface.get_base != buf_base) return false;
    mi355x_buffer_copy(dst->data, src->data, ggml_nbytes(src), nullptr);
    mi355x_stream_synchronize(nullptr);
    return true;
}
static void buf_clear(ggml_backend_buffer_t b, uint8_t v) {
    mi355x_buffer_memset(buf_base(b), v, b->size, nullptr);
    mi355x_stream_synchronize(nullptr);
}

static ggml_backend_buffer_i make_buffer_iface() {
    ggml_backend_buffer_i i = {};
    i.free_buffer   = buf_free;
    i.get_base      = buf_base;
    i.init_tensor   = buf_init_tensor;
    i.memset_tensor = buf_memset;
    i.set_tensor    = buf_set;
    i.get_tensor    = buf_get;
    i.cpy_tensor    = buf_cpy;
    i.clear         = buf_clear;
    return i;                                   // set_tensor_2d, get_tensor_2d, reset: NULL (optional)
}
static const ggml_backend_buffer_i mi355x_buffer_iface = make_buffer_iface();

template <bool DEVICE>
static ggml_backend_buffer_t buft_alloc(ggml_backend_buffer_type_t buft, size_t size) {
    void * p = nullptr;
    const int rc = DEVICE ? mi355x_buffer_alloc(size, &p) : mi355x_host_buffer_alloc(size, &p);
    if (rc != MI355X_OK) return nullptr;                      // allocation failures are NULL returns (src/voxtral.cpp:1138-1142)
    return ggml_backend_buffer_init(buft, mi355x_buffer_iface, new mi355x_buffer_ctx{p, DEVICE}, size);
}
static const char * buft_host_name(ggml_backend_buffer_type_t) { return "MI355X_Host"; }
static const char * buft_dev_name(ggml_backend_buffer_type_t)  { return "MI355X"; }
static size_t buft_align(ggml_backend_buffer_type_t) { return 256; }
static size_t buft_max(ggml_backend_buffer_type_t)   { return SIZE_MAX; }
static size_t buft_alloc_size(ggml_backend_buffer_type_t, const ggml_tensor * t) { return ggml_nbytes(t); }
static bool   buft_is_host(ggml_backend_buffer_type_t)  { return true; }
static bool   buft_not_host(ggml_backend_buffer_type_t) { return false; }

static ggml_backend_dev_t g_dev();
template <bool DEVICE>
static ggml_backend_buffer_type make_buft() {
    ggml_backend_buffer_type t = {};
    t.iface.get_name       = DEVICE ? buft_dev_name : buft_host_name;
    t.iface.alloc_buffer   = buft_alloc<DEVICE>;
    t.iface.get_alignment  = buft_align;
    t.iface.get_max_size   = buft_max;
    t.iface.get_alloc_size = buft_alloc_size;
    t.iface.is_host        = DEVICE ? buft_not_host : buft_is_host;
    t.device  = g_dev();
    t.context = nullptr;
    return t;
}
static ggml_backend_buffer_type_t mi355x_host_buft() {
    static ggml_backend_buffer_type t = make_buft<false>();
    return &t;
}
static ggml_backend_buffer_type_t mi355x_dev_buft() {
    static ggml_backend_buffer_type t = make_buft<true>();
    return &t;
}

// ---- supports_op: FLASH_ATTN_EXT and the copies it needs, nothing else ----------------------------------------

static bool dev_supports_op(ggml_backend_dev_t, const ggml_tensor * op) {
    switch (op->op) {
        case GGML_OP_FLASH_ATTN_EXT: {
            if (op->src[4]) return false;                      // sinks
            // a view that would fail the library's alignment checks at launch is refused here, so that the scheduler
            // leaves the node on the CPU instead of getting GGML_STATUS_FAILED from graph_compute
            const mi355x_tensor q = to_mi_planning(op->src[0]), k = to_mi_planning(op->src[1]), v = to_mi_planning(op->src[2]),
                                d = to_mi_planning(op);
            mi355x_tensor m;
            if (op->src[3]) m = to_mi_planning(op->src[3]);
            const mi355x_fattn_params p = fa_params(op);
            return mi355x_fattn_supports(&q, &k, &v, op->src[3] ? &m : nullptr, &d, &p) == MI355X_OK;
        }
        case GGML_OP_CPY: case GGML_OP_CONT: case GGML_OP_DUP: {
            const mi355x_tensor s = to_mi_planning(op->src[0]), d = to_mi_planning(op);
            return mi355x_cpy_supports(&s, &d) == MI355X_OK;
        }
        case GGML_OP_SET_ROWS: {                                // the write into a quantised KV cache (src/core/attention.h:366-376)
            const ggml_tensor * src = op->src[0], * idx = op->src[1];
            if (idx->type != GGML_TYPE_I64 && idx->type != GGML_TYPE_I32) return false;
            const mi355x_tensor s = to_mi_planning(src), d = to_mi_planning(op);
            const int64_t ine[3] = {idx->ne[0], idx->ne[1], idx->ne[2]};
            return mi355x_set_rows_supports(&s, idx->type == GGML_TYPE_I64 ? 64 : 32, ine, &d) == MI355X_OK;   // the library's own shape checks
        }
        case GGML_OP_NONE: case GGML_OP_RESHAPE: case GGML_OP_VIEW: case GGML_OP_PERMUTE: case GGML_OP_TRANSPOSE:
            return true;                                        // no-ops on any backend
        default:
            return false;
    }
}
static bool dev_supports_buft(ggml_backend_dev_t, ggml_backend_buffer_type_t buft) {
    return buft == mi355x_host_buft() || buft == mi355x_dev_buft();
}
// keep CPY/CONT on the CPU unless their destination already lives in one of our buffers
static bool dev_offload_op(ggml_backend_dev_t, const ggml_tensor * op) { return op->op == GGML_OP_FLASH_ATTN_EXT; }

// ---- backend: graph_compute walks the split's nodes ---------------------------------------------------------------

static const char * be_name(ggml_backend_t) { return "MI355X"; }
static void be_free(ggml_backend_t b) { delete b; }
static void be_sync(ggml_backend_t) { mi355x_stream_synchronize(nullptr); }

static enum ggml_status be_graph_compute(ggml_backend_t, ggml_cgraph * g) {
    for (int i = 0; i < ggml_graph_n_nodes(g); i++) {
        ggml_tensor * n = ggml_graph_node(g, i);
        int rc = MI355X_OK;
        switch (n->op) {
            case GGML_OP_FLASH_ATTN_EXT: {
                const mi355x_tensor q = to_mi(n->src[0]), k = to_mi(n->src[1]), v = to_mi(n->src[2]), d = to_mi(n);
                mi355x_tensor m;
                if (n->src[3]) m = to_mi(n->src[3]);
                const mi355x_fattn_params p = fa_params(n);
                rc = mi355x_flash_attn_ext(&q, &k, &v, n->src[3] ? &m : nullptr, &d, &p, nullptr);
                break;
            }
            case GGML_OP_CPY: case GGML_OP_CONT: case GGML_OP_DUP: {
                const mi355x_tensor s = to_mi(n->src[0]), d = to_mi(n);
                rc = mi355x_cpy(&s, &d, nullptr);
                break;
            }
            case GGML_OP_SET_ROWS: {                            // the node is a view of the destination; src[0] = rows, src[1] = indices
                const ggml_tensor * idx = n->src[1];
                const mi355x_tensor s = to_mi(n->src[0]), d = to_mi(n);
                const int64_t ine[3] = {idx->ne[0], idx->ne[1], idx->ne[2]};
                const size_t  inb[3] = {idx->nb[0], idx->nb[1], idx->nb[2]};
                rc = mi355x_set_rows(&s, idx->data, idx->type == GGML_TYPE_I64 ? 64 : 32, ine, inb, &d, nullptr);
                break;
            }
            default:
                break;                                          // views and reshapes
        }
        if (rc != MI355X_OK) {
            GGML_LOG_ERROR("ggml-mi355x: %s failed: %s\n", ggml_op_name(n->op), mi355x_last_error());
            return GGML_STATUS_FAILED;                          // callers only test == GGML_STATUS_SUCCESS (src/crispasr.cpp:273)
        }
    }
    // inputs may be overwritten by the caller as soon as compute returns (src/canary_ctc.cpp:959-963)
    return mi355x_stream_synchronize(nullptr) == MI355X_OK ? GGML_STATUS_SUCCESS : GGML_STATUS_FAILED;
}

static ggml_backend_i make_backend_iface() {
    ggml_backend_i i = {};                      // every optional member (async copies, graph plans, events, graph_optimize) stays NULL
    i.get_name      = be_name;
    i.free          = be_free;
    i.synchronize   = be_sync;
    i.graph_compute = be_graph_compute;
    return i;
}
static const ggml_backend_i mi355x_backend_iface = make_backend_iface();

static ggml_guid_t mi355x_guid() {
    static ggml_guid guid = {0x6d, 0x69, 0x33, 0x35, 0x35, 0x78, 0x2d, 0x66, 0x61, 0x74, 0x74, 0x6e, 0x00, 0x00, 0x00, 0x01};
    return &guid;
}

// ---- device + registry ---------------------------------------------------------------------------------------------

static const char * dev_name(ggml_backend_dev_t) { return "MI355X0"; }
static const char * dev_desc(ggml_backend_dev_t) {
    static mi355x_device_info info;
    static bool once = (mi355x_device_get_info(0, &info), true);
    (void)once;
    return info.name;
}
static void dev_memory(ggml_backend_dev_t, size_t * free, size_t * total) {
    mi355x_device_info info;
    mi355x_device_get_info(0, &info);
    *free = info.free_memory; *total = info.total_memory;
}
static enum ggml_backend_dev_type dev_type(ggml_backend_dev_t) { return GGML_BACKEND_DEVICE_TYPE_GPU; }   // the runtimes only look at GPU|IGPU (src/core/gpu_backend_pref.h:116-163)
static void dev_props(ggml_backend_dev_t d, ggml_backend_dev_props * p) {
    p->name = dev_name(d); p->description = dev_desc(d); p->type = dev_type(d);
    dev_memory(d, &p->memory_free, &p->memory_total);
    p->caps = {};
    p->caps.async                = false;
    p->caps.host_buffer          = true;
    p->caps.buffer_from_host_ptr = false;
    p->caps.events               = false;
}
static ggml_backend_t dev_init(ggml_backend_dev_t d, const char *) {
    if (mi355x_set_device(0) != MI355X_OK) return nullptr;     // callers fall back to the CPU backend (src/voxtral.cpp:842-845)
    ggml_backend * be = new ggml_backend();
    be->guid    = mi355x_guid();
    be->iface   = mi355x_backend_iface;
    be->device  = d;
    be->context = nullptr;
    return be;
}
static ggml_backend_buffer_type_t dev_buft(ggml_backend_dev_t)      { return mi355x_host_buft(); }
static ggml_backend_buffer_type_t dev_host_buft(ggml_backend_dev_t) { return mi355x_host_buft(); }

static ggml_backend_device_i make_device_iface() {
    ggml_backend_device_i i = {};               // buffer_from_host_ptr and the event members stay NULL
    i.get_name             = dev_name;
    i.get_description      = dev_desc;
    i.get_memory           = dev_memory;
    i.get_type             = dev_type;
    i.get_props            = dev_props;
    i.init_backend         = dev_init;
    i.get_buffer_type      = dev_buft;
    i.get_host_buffer_type = dev_host_buft;
    i.supports_op          = dev_supports_op;
    i.supports_buft        = dev_supports_buft;
    i.offload_op           = dev_offload_op;
    return i;
}
static const ggml_backend_device_i mi355x_device_iface = make_device_iface();

static const char * reg_name(ggml_backend_reg_t) { return "MI355X"; }
static size_t reg_count(ggml_backend_reg_t) {
    // a library built from another revision of the header than this file offers no device: its structs may differ
    if (mi355x_api_version() != MI355X_FATTN_API_VERSION) {
        GGML_LOG_ERROR("ggml-mi355x: libmi355x_fattn has API version %d, this backend was built against %d\n",
                       mi355x_api_version(), MI355X_FATTN_API_VERSION);
        return 0;
    }
    int n = 0;
    mi355x_device_count(&n);
    return n > 0 ? 1 : 0;
}
static ggml_backend_dev_t reg_dev(ggml_backend_reg_t, size_t) { return g_dev(); }
static void * reg_proc(ggml_backend_reg_t, const char *) { return nullptr; }

extern "C" ggml_backend_reg_t ggml_backend_mi355x_reg(void) {
    static ggml_backend_reg reg = [] {
        ggml_backend_reg r = {};
        r.api_version            = GGML_BACKEND_API_VERSION;
        r.iface.get_name         = reg_name;
        r.iface.get_device_count = reg_count;
        r.iface.get_device       = reg_dev;
        r.iface.get_proc_address = reg_proc;
        r.context                = nullptr;
        return r;
    }();
    return &reg;
}
static ggml_backend_dev_t g_dev() {
    static ggml_backend_device dev = [] {
        ggml_backend_device d = {};
        d.iface   = mi355x_device_iface;
        d.reg     = ggml_backend_mi355x_reg();
        d.context = nullptr;
        return d;
    }();
    return &dev;
}

#ifdef GGML_BACKEND_DL
GGML_BACKEND_DL_IMPL(ggml_backend_mi355x_reg)
#endif
