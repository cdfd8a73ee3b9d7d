// extern "C" entry points of libmi355x_fattn.so: validation, kernel choice, scratch, launches.
#include "fattn_common.h"

#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <mutex>
#include <vector>

// Scratch of the allocation-free entry point: one array per GPU, part of the library's code object, so that it exists
// once the library is loaded on a device and no call ever has to allocate it.  Host code never uses the array's name as
// an address (here it is only a handle for the lookup below): each device holds its own copy at its own address.
static __device__ __align__(256) unsigned char scratch[MI355X_NOALLOC_SCRATCH_BYTES];

// Counters of launches that merge their split-KV partials in the kernel (FattnArgs::counters): zero when the library is
// loaded, and left at zero by every launch.  Set 0 serves calls that run on the library's own scratch block, set 1 the
// allocation-free entry point: each of the two is one-call-at-a-time per GPU by its contract, and a call of one may
// overlap a call of the other.  A call on a caller's workspace may overlap anything and merges in a launch of its own.
constexpr int MERGE_COUNTERS = 16384;
static __device__ __align__(256) unsigned merge_counters[2 * MERGE_COUNTERS];

namespace {

thread_local char g_err[512] = "";

int fail(int status, const char * fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return status;
}

int hip_fail(hipError_t e, const char * what) {
    (void)hipGetLastError();      // reported here: the launchers read the last error after each launch and must not see this one again
    return fail(MI355X_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
}

#define HIP_TRY(expr)                                   \
    do {                                                \
        hipError_t e_ = (expr);                         \
        if (e_ != hipSuccess) return hip_fail(e_, #expr); \
    } while (0)

size_t type_size(int t) {
    switch (t) {
        case MI355X_TYPE_F32:  return 4;
        case MI355X_TYPE_F16:  return 2;
        default:               return (size_t)fattn_block_bytes(t);      // 0 for a type this library does not know
    }
}
int64_t block_size(int t) { return FATTN_IS_BLOCK_TYPE(t) ? FATTN_QK8_0 : 1; }
// Q4_0, Q4_1, Q5_0, Q5_1: read natively by the vector kernel, through f16 copies by the tile kernel
bool narrow_quant(int t) { return FATTN_IS_BLOCK_TYPE(t) && t != MI355X_TYPE_Q8_0; }

bool is_contiguous(const mi355x_tensor * t) {
    const size_t ts = type_size(t->type);
    if (!ts) return false;
    size_t nb = ts;
    if (t->nb[0] != nb) return false;
    nb *= (size_t)(t->ne[0] / block_size(t->type));
    for (int i = 1; i < 4; i++) {
        if (t->ne[i] != 1 && t->nb[i] != nb) return false;
        nb *= (size_t)t->ne[i];
    }
    return true;
}

struct DeviceCache {
    int  cus = 0;
    bool init = false;
};
DeviceCache g_dev[64];
std::mutex  g_mu;

int device_cus() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    std::lock_guard<std::mutex> lk(g_mu);
    if (!g_dev[dev].init) {
        int cus = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
        g_dev[dev].cus  = cus;
        g_dev[dev].init = true;
    }
    return g_dev[dev].cus;
}

// Extents a kernel can index: none negative, each below 2^31, their product below 2^62 (n = that product).
bool sane_extents(const mi355x_tensor * t, int64_t * n) {
    int64_t p = 1;
    for (int i = 0; i < 4; i++) {
        if (t->ne[i] < 0 || t->ne[i] > 0x7fffffff) return false;
        if (t->ne[i] > 0 && p > ((int64_t)1 << 62) / t->ne[i]) return false;
        p *= t->ne[i];
    }
    if (n) *n = p;
    return true;
}

// Library-owned scratch for the split-KV partials: one growing allocation per device.
// Outgrown blocks stay allocated until the process ends, so launches still in flight on
// other streams keep valid memory.
struct Scratch {
    void * ptr  = nullptr;
    size_t size = 0;
};
Scratch g_scratch[64];

int get_scratch(size_t bytes, void ** out, hipStream_t st) {
    int dev = 0;
    HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= 64) return fail(MI355X_ERR_HIP, "device index %d out of range", dev);
    std::lock_guard<std::mutex> lk(g_mu);
    Scratch & s = g_scratch[dev];
    if (s.size < bytes) {
        // growing means hipMalloc: not while the stream is being recorded into a graph
        hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(st, &cs) != hipSuccess) (void)hipGetLastError();
        else if (cs != hipStreamCaptureStatusNone)
            return fail(MI355X_ERR_WORKSPACE, "this call needs %zu bytes of workspace and the library holds %zu: pass one, or make the call "
                        "once before capturing", bytes, s.size);
        size_t want = s.size ? s.size : (size_t)(8u << 20);
        while (want < bytes) want *= 2;
        void * p = nullptr;
        HIP_TRY(hipMalloc(&p, want));
        s.ptr  = p;          // the previous block is deliberately kept alive
        s.size = want;
    }
    *out = s.ptr;
    return MI355X_OK;
}

void * g_noalloc_scratch[64];      // per device: the address hipGetSymbolAddress gave for `scratch`

// the current device's copy of `scratch`, looked up once per device
int noalloc_scratch(void ** out) {
    int dev = 0;
    HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= 64) return fail(MI355X_ERR_HIP, "device index %d out of range", dev);
    std::lock_guard<std::mutex> lk(g_mu);
    if (!g_noalloc_scratch[dev]) {
        void * ptr = nullptr;
        const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return hip_fail(e, "hipGetSymbolAddress(scratch)");
        if (!ptr) return fail(MI355X_ERR_HIP, "hipGetSymbolAddress(scratch) returned no address");
        g_noalloc_scratch[dev] = ptr;
    }
    *out = g_noalloc_scratch[dev];
    return MI355X_OK;
}

unsigned * g_merge_counters[64];   // per device: the address of merge_counters there
bool       g_merge_counters_failed[64];
const bool g_no_fused_merge = getenv("MI355X_NO_FUSED_MERGE") != nullptr;      // comparison runs: always the merge launch

// the current device's counters of set `set`, or nullptr (then the caller merges in a launch of its own)
unsigned * merge_counter_set(int set) {
    if (set < 0 || g_no_fused_merge) return nullptr;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
        (void)hipGetLastError();
        return nullptr;
    }
    std::lock_guard<std::mutex> lk(g_mu);
    if (!g_merge_counters[dev] && !g_merge_counters_failed[dev]) {
        void * ptr = nullptr;
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(merge_counters)) != hipSuccess || !ptr) {
            (void)hipGetLastError();
            g_merge_counters_failed[dev] = true;
        }
        g_merge_counters[dev] = (unsigned *)ptr;
    }
    return g_merge_counters[dev] ? g_merge_counters[dev] + (size_t)set * MERGE_COUNTERS : nullptr;
}

// ---- host-visible buffers and their mirrors in HBM ---------------------------------------------------------------
// A buffer from mi355x_host_buffer_alloc is pinned host memory that the CPU backend works on in place.  What the GPU
// reads from it again and again - a KV cache - would cross the host link on every call, so such a buffer grows a mirror:
// an HBM allocation of the same size, created by the first KV write into the buffer.  The host copy stays complete and
// authoritative; a page of the mirror is VALID when it holds the same bytes.  Every write that goes through this library
// (copy / set_rows kernels, memset, set, copy) stores to both copies, after bringing the pages it touches up to date, so
// pages that are VALID stay so; attention reads K and V from the mirror, bringing stale pages up to date first.  In the
// steady state of a decoder loop nothing but the new rows (to the host copy), Q and the result cross the link.
constexpr size_t MIRROR_PAGE = 64 * 1024;
struct HostBuf {
    char * base   = nullptr;
    size_t size   = 0;
    char * mirror = nullptr;
    int    dev    = -1;                // the device that holds the mirror: calls made with another device current use the host copy
    std::vector<uint8_t> valid;        // per page
    size_t uploaded = 0;               // bytes brought up to date so far (statistics)
};
std::vector<HostBuf *> g_hostbufs;     // guarded by g_mu
const bool g_no_mirror = getenv("MI355X_NO_MIRROR") != nullptr;      // comparison runs: every read and write goes to the host copy

// the registered buffer that holds [p, p + n), or nullptr (g_mu held)
HostBuf * hostbuf_of(const void * p, size_t n) {
    for (HostBuf * b : g_hostbufs)
        if ((const char *)p >= b->base && (const char *)p + n <= b->base + b->size) return b;
    return nullptr;
}

// first and one-past-last byte that a view touches, relative to its data pointer
void view_span(const mi355x_tensor * t, size_t * bytes) {
    size_t hi = 0;
    bool   empty = false;
    for (int i = 0; i < 4; i++) empty = empty || t->ne[i] <= 0;
    if (!empty) {
        hi = (size_t)(t->ne[0] / block_size(t->type)) * t->nb[0];
        for (int i = 1; i < 4; i++) hi += (size_t)(t->ne[i] - 1) * t->nb[i];
    }
    *bytes = hi;
}

// bring the mirror's pages that overlap [off, off + n) up to date (g_mu held)
int mirror_make_valid(HostBuf * b, size_t off, size_t n, hipStream_t st) {
    if (!b->mirror || n == 0) return MI355X_OK;
    const size_t p0 = off / MIRROR_PAGE, p1 = (off + n + MIRROR_PAGE - 1) / MIRROR_PAGE;
    size_t run = (size_t)-1;
    for (size_t p = p0; p <= p1; p++) {
        const bool stale = p < p1 && !b->valid[p];
        if (stale && run == (size_t)-1) run = p;
        if (!stale && run != (size_t)-1) {
            const size_t lo = run * MIRROR_PAGE, hi = p * MIRROR_PAGE < b->size ? p * MIRROR_PAGE : b->size;
            HIP_TRY(hipMemcpyAsync(b->mirror + lo, b->base + lo, hi - lo, hipMemcpyHostToDevice, st));
            b->uploaded += hi - lo;
            for (size_t k = run; k < p; k++) b->valid[k] = 1;
            run = (size_t)-1;
        }
    }
    return MI355X_OK;
}

// pages that lie inside [off, off + n) altogether have just been written in both copies
void mirror_mark_written(HostBuf * b, size_t off, size_t n) {
    if (!b->mirror) return;
    const size_t p0 = (off + MIRROR_PAGE - 1) / MIRROR_PAGE;
    const size_t end = off + n == b->size ? (b->size + MIRROR_PAGE - 1) / MIRROR_PAGE : (off + n) / MIRROR_PAGE;
    for (size_t p = p0; p < end; p++) b->valid[p] = 1;
}

// A kernel is about to write the view `dst`.  If it lies in a host buffer: create that buffer's mirror if need be (never
// while the stream is being captured: the write then goes to the host copy alone and the pages turn stale), bring the
// pages of the view's span up to date, and return the distance from the host copy to the mirror (0: write the view only).
int mirror_for_write(const mi355x_tensor * dst, hipStream_t st, int64_t * delta) {
    *delta = 0;
    if (g_no_mirror || !dst->data) return MI355X_OK;
    size_t n = 0;
    view_span(dst, &n);
    std::lock_guard<std::mutex> lk(g_mu);
    HostBuf * b = hostbuf_of(dst->data, n);
    if (!b) return MI355X_OK;
    const size_t off = (size_t)((const char *)dst->data - b->base);
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(st, &cs) != hipSuccess) (void)hipGetLastError();
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess) (void)hipGetLastError();
    if (!b->mirror) {
        void * m = nullptr;
        if (cs != hipStreamCaptureStatusNone || dev < 0 || hipMalloc(&m, b->size) != hipSuccess) {
            (void)hipGetLastError();
            return MI355X_OK;                        // no mirror: the buffer stays a plain host buffer
        }
        b->mirror = (char *)m;
        b->dev    = dev;
        b->valid.assign((b->size + MIRROR_PAGE - 1) / MIRROR_PAGE, 0);
    }
    if (cs != hipStreamCaptureStatusNone || dev != b->dev) {
        // a captured write would be replayed without this bookkeeping, and another GPU cannot store into this one's
        // memory: keep the write to the host copy, the pages become stale
        const size_t p0 = off / MIRROR_PAGE, p1 = (off + n + MIRROR_PAGE - 1) / MIRROR_PAGE;
        for (size_t p = p0; p < p1; p++) b->valid[p] = 0;
        return MI355X_OK;
    }
    const int rc = mirror_make_valid(b, off, n, st);
    if (rc) return rc;
    *delta = b->mirror - b->base;
    return MI355X_OK;
}

// A kernel is about to read the view `t` many times over (K or V).  If it lies in a host buffer that has a mirror, bring
// the span's pages up to date and return the view's address in the mirror; otherwise the address it has.
int mirror_for_read(const mi355x_tensor * t, hipStream_t st, void ** data) {
    *data = t->data;
    if (g_no_mirror || !t->data) return MI355X_OK;
    size_t n = 0;
    view_span(t, &n);
    std::lock_guard<std::mutex> lk(g_mu);
    HostBuf * b = hostbuf_of(t->data, n);
    if (!b || !b->mirror) return MI355X_OK;
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess) (void)hipGetLastError();
    if (dev != b->dev) return MI355X_OK;             // the mirror lives on another GPU
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(st, &cs) != hipSuccess) (void)hipGetLastError();
    const size_t off = (size_t)((const char *)t->data - b->base);
    if (cs != hipStreamCaptureStatusNone) {
        // under capture only pages that are up to date already may be read from the mirror
        for (size_t p = off / MIRROR_PAGE; p < (off + n + MIRROR_PAGE - 1) / MIRROR_PAGE; p++)
            if (!b->valid[p]) return MI355X_OK;
    } else {
        const int rc = mirror_make_valid(b, off, n, st);
        if (rc) return rc;
    }
    *data = b->mirror + off;
    return MI355X_OK;
}

// A kernel is about to write the view `t` through its host address alone (an attention result, a mask): should the
// buffer have a mirror, the pages of the view's span are stale from now on.
void mirror_note_host_write(const mi355x_tensor * t) {
    if (g_no_mirror || !t || !t->data) return;
    size_t n = 0;
    view_span(t, &n);
    std::lock_guard<std::mutex> lk(g_mu);
    HostBuf * b = hostbuf_of(t->data, n);
    if (!b || !b->mirror || n == 0) return;
    const size_t off = (size_t)((const char *)t->data - b->base);
    for (size_t p = off / MIRROR_PAGE; p < (off + n + MIRROR_PAGE - 1) / MIRROR_PAGE; p++) b->valid[p] = 0;
}

// a mask argument with no extent is the same as no mask
bool has_mask(const mi355x_tensor * mask) { return mask && mask->ne[0] > 0; }

struct Plan {
    int     kernel;
    int     n_splits;
    int     keys_per_split;
    size_t  workspace;       // bytes in all: [f16 copies of K and V][split partials]
    size_t  ws_partials;     // offset of the split partials inside the workspace
    int64_t merge_sets;      // > 0: the kernel can merge its splits itself, given this many counters
    bool    kv_to_f16;       // K and V are rounded to f16 copies in the workspace first (F32 / quantised K/V before the tile kernel; a
                             // K and a V of different types before any kernel)
    int     pad;             // 0, or the head size (64 / 128) the copies' rows are zero-padded to for the tile kernel
};

// the call as the kernels see it when the plan pads the head: D the padded size, Dv the real one
void apply_pad(FattnArgs & a, const Plan & plan) {
    if (plan.pad) {
        a.Dv = a.D;
        a.D  = plan.pad;
    }
}

int check(const mi355x_tensor * q, const mi355x_tensor * k, const mi355x_tensor * v,
          const mi355x_tensor * mask, const mi355x_tensor * dst, const mi355x_fattn_params * p) {
    if (!q || !k || !v || !p) return fail(MI355X_ERR_INVALID, "null argument");
    if (!sane_extents(q, nullptr) || !sane_extents(k, nullptr) || !sane_extents(v, nullptr) ||
        (mask && !sane_extents(mask, nullptr)) || (dst && !sane_extents(dst, nullptr)))
        return fail(MI355X_ERR_INVALID, "negative or oversized extent");
    if (q->type != MI355X_TYPE_F32) return fail(MI355X_ERR_UNSUPPORTED, "q must be F32 (type %d)", q->type);
    if (!type_size(k->type)) return fail(MI355X_ERR_UNSUPPORTED, "K type %d not covered", k->type);
    if (!type_size(v->type)) return fail(MI355X_ERR_UNSUPPORTED, "V type %d not covered", v->type);

    const int64_t D = q->ne[0], Nq = q->ne[1], Hq = q->ne[2], B = q->ne[3];
    const int64_t Nkv = k->ne[1], Hkv = k->ne[2], Bk = k->ne[3];
    if (k->ne[0] != D) return fail(MI355X_ERR_INVALID, "k.ne0 %lld != q.ne0 %lld", (long long)k->ne[0], (long long)D);
    if (v->ne[1] != Nkv || v->ne[2] != Hkv || v->ne[3] != Bk) return fail(MI355X_ERR_INVALID, "k and v shapes differ");
    if (Hkv <= 0 || Bk <= 0 || Hq % Hkv || B % Bk) return fail(MI355X_ERR_INVALID, "q heads/batch not a multiple of kv heads/batch");
    if (v->ne[0] != D) return fail(MI355X_ERR_UNSUPPORTED, "DV %lld != DK %lld", (long long)v->ne[0], (long long)D);
    // (multiples of 8 everywhere; 36 and 52 - the decoder cross-attention of src/core/cross_attn.h:119-153 in the smaller
    //  Moonshine models - and the like run on the vector kernel)
    if (D <= 0 || D % 4 || D > 256) return fail(MI355X_ERR_UNSUPPORTED, "head size %lld (need a multiple of 4, <= 256)", (long long)D);
    if ((FATTN_IS_BLOCK_TYPE(k->type) || FATTN_IS_BLOCK_TYPE(v->type)) && D % FATTN_QK8_0) return fail(MI355X_ERR_INVALID, "quantised rows need D %% 32 == 0");
    if (D % 8 && k->type != v->type) return fail(MI355X_ERR_UNSUPPORTED, "head size %lld with K and V of different types", (long long)D);
    if (Nq < 0 || Nkv < 0 || Hq <= 0 || B <= 0) return fail(MI355X_ERR_INVALID, "negative or zero extent");
    if (q->nb[0] != 4) return fail(MI355X_ERR_UNSUPPORTED, "q rows must be contiguous (nb0 = %zu)", q->nb[0]);
    if (k->nb[0] != type_size(k->type) || v->nb[0] != type_size(v->type))
        return fail(MI355X_ERR_UNSUPPORTED, "k/v rows must be contiguous");
    const size_t alk = k->type == MI355X_TYPE_F32 ? 4 : 2, alv = v->type == MI355X_TYPE_F32 ? 4 : 2;
    for (int i = 1; i < 4; i++) {
        if (q->nb[i] % 4 || k->nb[i] % alk || v->nb[i] % alv) return fail(MI355X_ERR_UNSUPPORTED, "misaligned strides");
    }
    if (((uintptr_t)q->data % 4) || ((uintptr_t)k->data % alk) || ((uintptr_t)v->data % alv))
        return fail(MI355X_ERR_UNSUPPORTED, "misaligned data pointers");
    if (has_mask(mask)) {
        if (mask->type != MI355X_TYPE_F16) return fail(MI355X_ERR_UNSUPPORTED, "mask must be F16 (type %d)", mask->type);
        if (mask->nb[0] != 2) return fail(MI355X_ERR_INVALID, "mask rows must be contiguous");
        if (mask->ne[0] < Nkv || mask->ne[1] < Nq) return fail(MI355X_ERR_INVALID, "mask smaller than [Nkv, Nq]");
        if (mask->ne[2] <= 0 || mask->ne[3] <= 0 || Hq % mask->ne[2] || B % mask->ne[3])
            return fail(MI355X_ERR_INVALID, "mask broadcast extents do not divide q's");
        for (int i = 1; i < 4; i++) if (mask->nb[i] % 2) return fail(MI355X_ERR_UNSUPPORTED, "misaligned mask strides");
    } else if (p->max_bias > 0.0f) {
        return fail(MI355X_ERR_INVALID, "max_bias > 0 needs a mask");
    }
    if (dst) {
        if (dst->type != MI355X_TYPE_F32) return fail(MI355X_ERR_INVALID, "dst must be F32");
        if (dst->ne[0] != D || dst->ne[1] != Hq || dst->ne[2] != Nq || dst->ne[3] != B)
            return fail(MI355X_ERR_INVALID, "dst must be [DV, Hq, Nq, B]");
        if (!is_contiguous(dst)) return fail(MI355X_ERR_UNSUPPORTED, "dst must be contiguous");
        if ((uintptr_t)dst->data % 16) return fail(MI355X_ERR_UNSUPPORTED, "dst must be 16-byte aligned (128-bit stores)");
    }
    if (Nq * Hq * B > (int64_t)1 << 26 || Nkv > (int64_t)1 << 30) return fail(MI355X_ERR_UNSUPPORTED, "problem too large");
    if (p->prec != 0 && p->prec != 10) return fail(MI355X_ERR_INVALID, "unknown prec %d", p->prec);
    if (p->q_quant != 0 && p->q_quant != MI355X_TYPE_Q8_0) return fail(MI355X_ERR_INVALID, "unknown q_quant %d", p->q_quant);
    if (p->q_quant == MI355X_TYPE_Q8_0 && q->ne[0] % FATTN_QK8_0) return fail(MI355X_ERR_INVALID, "q_quant needs D %% 32 == 0");
    return MI355X_OK;
}

void fill_args(FattnArgs & a, const mi355x_tensor * q, const mi355x_tensor * k, const mi355x_tensor * v,
               const mi355x_tensor * mask, float * dst, const mi355x_fattn_params * p) {
    memset(&a, 0, sizeof(a));
    a.q = (const char *)q->data; a.k = (const char *)k->data; a.v = (const char *)v->data;
    a.mask = has_mask(mask) ? (const char *)mask->data : nullptr;
    a.dst = dst;
    a.D = (int)q->ne[0]; a.Nq = (int)q->ne[1]; a.Hq = (int)q->ne[2]; a.B = (int)q->ne[3];
    a.Dv = a.D;
    a.Nkv = (int)k->ne[1]; a.Hkv = (int)k->ne[2]; a.Bk = (int)k->ne[3];
    a.gqa = a.Hq / a.Hkv; a.bq = a.B / a.Bk;
    a.q_chunks = (int32_t)(((int64_t)a.Nq * a.gqa + 15) / 16);
    a.nbq1 = q->nb[1]; a.nbq2 = q->nb[2]; a.nbq3 = q->nb[3];
    a.nbk1 = k->nb[1]; a.nbk2 = k->nb[2]; a.nbk3 = k->nb[3];
    a.nbv1 = v->nb[1]; a.nbv2 = v->nb[2]; a.nbv3 = v->nb[3];
    a.Hm = 1; a.Bm = 1;
    bool q16 = !((uintptr_t)q->data % 16);
    bool kv16 = !((uintptr_t)k->data % 16) && !((uintptr_t)v->data % 16);
    for (int i = 1; i < 4; i++) {
        q16  = q16 && !(q->nb[i] % 16);
        kv16 = kv16 && !(k->nb[i] % 16) && !(v->nb[i] % 16);
    }
    a.q_aligned16 = q16 ? 1 : 0;
    a.kv_aligned16 = kv16 ? 1 : 0;
    bool kv4 = !((uintptr_t)k->data % 4) && !((uintptr_t)v->data % 4);
    for (int i = 1; i < 4; i++) kv4 = kv4 && !(k->nb[i] % 4) && !(v->nb[i] % 4);
    a.kv_aligned4 = kv4 ? 1 : 0;
    bool kv2 = !((uintptr_t)k->data % 2) && !((uintptr_t)v->data % 2);
    for (int i = 1; i < 4; i++) kv2 = kv2 && !(k->nb[i] % 2) && !(v->nb[i] % 2);
    a.kv_aligned2 = kv2 ? 1 : 0;
    const bool al16 = q16 && kv16;
    a.masked = has_mask(mask) ? 1 : 0;
    if (a.masked) {
        a.Hm = (int)mask->ne[2]; a.Bm = (int)mask->ne[3];
        a.nbm1 = mask->nb[1]; a.nbm2 = mask->nb[2]; a.nbm3 = mask->nb[3];
        bool m8 = !((uintptr_t)mask->data % 8);
        for (int i = 1; i < 4; i++) m8 = m8 && !(mask->nb[i] % 8);
        a.mask_al8 = m8 ? 1 : 0;
        bool m4 = !((uintptr_t)mask->data % 4);
        for (int i = 1; i < 4; i++) m4 = m4 && !(mask->nb[i] % 4);
        a.mask_al4 = m4 ? 1 : 0;
    }
    a.aligned16 = al16 ? 1 : 0;
    a.n_cus = device_cus();
    a.tile_variant = p->tile_variant;
    a.softcap = p->logit_softcap;
    a.scale   = p->logit_softcap != 0.0f ? p->scale / p->logit_softcap : p->scale;
    a.max_bias = p->max_bias;
    // ALiBi slope bases, as ggml derives them from the head count
    const uint32_t n2 = 1u << (uint32_t)floorf(log2f((float)a.Hq));
    a.n_head_log2 = (int)n2;
    a.m0 = powf(2.0f, -(p->max_bias) / n2);
    a.m1 = powf(2.0f, -(p->max_bias / 2.0f) / n2);
    a.n_splits = 1;
    a.keys_per_split = a.Nkv;
    a.part_acc = a.part_ml = nullptr;
    a.counters = nullptr;
}

// the same call on the f16 copies of K and V that kv_to_f16_launch leaves at ws: contiguous [D, Nkv, Hkv, Bk], V behind K
void use_f16_copies(FattnArgs & a, void * ws) {
    const size_t half = (size_t)a.D * a.Nkv * a.Hkv * a.Bk * sizeof(uint16_t);
    a.k = (const char *)ws;
    a.v = (const char *)ws + half;
    a.nbk1 = a.nbv1 = (size_t)a.D * 2;
    a.nbk2 = a.nbv2 = a.nbk1 * a.Nkv;
    a.nbk3 = a.nbv3 = a.nbk2 * a.Hkv;
    a.kv_aligned16 = a.kv_aligned4 = a.kv_aligned2 = 1;
    a.aligned16 = a.q_aligned16;
}

// A K and a V of different storage types (CRISPASR_KV_QUANT_K / _V, src/core/attention.h:132-137) are both rounded to f16
// copies first, whatever the kernel: the call is then planned and run as an F16 one.

// (padded: a0.D is the padded head size and the copies are needed whatever the types)
void make_plan_core(const FattnArgs & a0, int ktype, int vtype, const mi355x_fattn_params * p, bool padded, Plan & plan) {
    FattnArgs a = a0;
    const bool mixed = ktype != vtype || padded;
    if (mixed) {
        use_f16_copies(a, nullptr);
        ktype = MI355X_TYPE_F16;
    }
    int kernel = p->kernel;
    if (kernel == MI355X_FATTN_AUTO) {
        // The decode kernel takes the Nq * gqa rows that share a KV head 16 at a time, each chunk streaming the head's K/V
        // again.  Up to 16 rows that is the whole job.  Beyond, it still beats the tile kernel on a short prompt against
        // a short Q8_0 cache (Canary's decoder reads its quantised cache directly, src/canary.cpp:966-972): no conversion
        // pass, one round of workgroups (measured at 128 x 128 and 256 x 256, 32 q / 8 kv heads: 14.0 -> 8.6 and
        // 18.0 -> 14.3 us; 24 x 300, 8 heads: 14.2 -> 10.9 us; at 407 x 407, 816 chunks, the tile kernel wins 29 to 31).
        // With f16 K/V the two are within a microsecond of each other and the tile kernel keeps the shape.
        const int64_t chunk_wgs = (int64_t)a.q_chunks * a.Hkv * a.B;
        bool          chunked   = ktype == MI355X_TYPE_Q8_0 && chunk_wgs <= 2 * (int64_t)device_cus() && a.Nkv <= 1024;
        // (f16: only the smallest calls - up to one chunk per CU against 64 keys, or 256 keys at 64-wide heads - where the
        //  decode kernel's single round is 1 to 2 us shorter than the tile kernel's 6 to 9: 64 queries x 32 q / 8 kv heads
        //  against 256 keys 8.8 -> 6.9 us)
        if (ktype == MI355X_TYPE_F16 && a.q_chunks > 1 && chunk_wgs <= device_cus() && (a.Nkv <= 64 || (a.D == 64 && a.Nkv <= 256)))
            chunked = true;
        // A longer Q8_0 cache under fewer than 128 queries: the tile kernel would dequantise every tile in its loop, once per
        // query head (1.7 us per 64-key tile at 64-wide heads, 2.1 at 128-wide; 5 sequences x 32 q / 8 kv heads x 16 queries
        // against 4096 keys: 111 us, the decode kernel 29), so the two are priced - the tile kernel's tiles per workgroup
        // after its own key split, the decode kernel's chunks x keys at its measured rate - and the decode kernel has to
        // win by 1.4 (its rate drops with a mask row per query row).
        if (!chunked && ktype == MI355X_TYPE_Q8_0 && a.q_chunks > 1 && a.Nq < 128 && a.Nkv > 1024) {
            const int     cus     = device_cus();
            const int     n_tiles = (a.Nkv + 63) / 64;
            const int64_t wgs     = (int64_t)a.Hq * a.B;
            int ns = 1;
            if (wgs * 4 <= cus) {
                ns = (int)(cus / wgs);
                if (ns > n_tiles / 4) ns = n_tiles / 4;
                if (ns < 1) ns = 1;
            } else if (wgs * 2 <= cus && n_tiles >= 16) {
                ns = 2;
            }
            const double rounds = (double)wgs * ns > 2.0 * cus ? (double)wgs * ns / (2.0 * cus) : 1.0;
            const double tile   = (double)((n_tiles + ns - 1) / ns) * (a.D == 64 ? 1.73 : 2.1) * rounds + (ns > 1 ? 5.0 : 0.0);
            const double decode = (double)chunk_wgs * a.Nkv * (a.D == 64 ? 20.7e-6 : 39.0e-6) + 12.0;
            chunked = decode * 1.4 < tile;
        }
        // The MFMA kernels round F32 and Q8_0 K/V to f16 (2^-12 relative per element).  Over many keys that averages out;
        // a row that sees a handful of keys keeps it (up to 1e-3 on |v| = 4, measured 2.01e-3 in all at 7 keys), so
        // such calls go to the vector kernel, which works on the exact values - and has nothing to gain from MFMA there.
        const bool few_keys = a.Nkv <= 16 && ktype != MI355X_TYPE_F16;
        // 9 to 16 rows per KV head over an f16 cache: the decode kernel's waves merge their rows 8 at a time at 128-wide
        // heads, and its partial rows and merge grow with the rows, while the tile kernel (cut into key ranges of its own)
        // does not care: 128-wide 16 rows x 8 heads against 256 keys 12.2 against 9.7 us, against 4096 keys 17.9 against
        // 13.6; 64-wide from 2048 keys on (20 heads x 16 rows against 4096: 17.1 against 12.8).  Up to 8 rows, and over Q8_0
        // caches, the decode kernel stays ahead or level.
        // (Rows that are several query heads of few queries stay: the tile kernel would walk the keys once per query head -
        //  4 queries x 32 q / 8 kv heads x 5 sequences against 1024 keys 26.8 us there, 14.2 here.)
        const bool tile_rows = ktype == MI355X_TYPE_F16 && a.gqa == 1 && a.Nq > 8 && (a.D == 128 || a.Nkv >= 2048) &&
                               fattn_mma_supported(a, ktype);
        if (few_keys)                                                              kernel = MI355X_FATTN_VEC;
        else if (narrow_quant(ktype))     // up to 16 rows per KV head read the blocks in the decode kernel; more rows share one conversion to f16
            kernel = fattn_decode_supported(a, ktype) && a.q_chunks <= 1                  ? MI355X_FATTN_DECODE_MMA
                     : a.Nq >= 16 && (a.D == 64 || a.D == 128) && a.q_aligned16 ? MI355X_FATTN_MMA
                                                                                : MI355X_FATTN_VEC;
        else if (fattn_decode_supported(a, ktype) && ((a.q_chunks <= 1 && !tile_rows) || chunked)) kernel = MI355X_FATTN_DECODE_MMA;
        else if ((a.Nq >= 16 || tile_rows) && fattn_mma_supported(a, ktype)) kernel = MI355X_FATTN_MMA;
        // F32 K/V under 2 .. 15 queries (the decode kernel does not read F32): the vector kernel streams the keys once per
        // query row, the tile kernel once per head - worth its padding from about 40k (row, key) pairs on at 64-wide heads
        // and 100k at 128-wide ones (4 queries x 32 heads x 5 sequences against 256 keys: 20.1 -> 10.0 us and 30.7 -> 17.8)
        else if (ktype == MI355X_TYPE_F32 && a.Nq >= 2 && fattn_mma_supported(a, ktype) &&
                 (int64_t)a.Nq * a.Hq * a.B * a.Nkv >= (a.D == 64 ? 40000 : 100000))
                                                              kernel = MI355X_FATTN_MMA;
        else                                                  kernel = MI355X_FATTN_VEC;
    }
    plan.kernel = kernel;
    plan.n_splits = 1;
    plan.keys_per_split = a.Nkv;
    plan.workspace = 0;
    plan.kv_to_f16 = false;
    plan.ws_partials = 0;
    plan.merge_sets = 0;
    plan.pad = 0;
    // nothing to launch (no query rows) or nothing to read (no keys: the result is zeros): one range, no workspace
    if ((int64_t)a.Nq * a.Hq * a.B == 0 || a.Nkv == 0) return;
    // The tile kernel rounds F32 and Q8_0 K/V to f16 on their way into LDS anyway.  With enough queries to share the work it
    // is cheaper to do that once, in a copy of its own, and let the f16 path (which moves tiles global->LDS without
    // touching registers) read the result: same values, same rounding.
    plan.ws_partials = 0;
    const bool convertible = (ktype == MI355X_TYPE_F32 && a.kv_aligned16) || (ktype == MI355X_TYPE_Q8_0 && a.kv_aligned2);
    // (F32 rows of 128-wide heads are the costliest to stage through registers - that form still spills - so they are
    //  converted from 0.4 GFLOP of work on, whatever the number of queries: 100 queries x 700 keys x 32 heads 30.9 -> 20.8 us,
    //  127 x 127 x 64 heads 16.6 -> 15.2 us, 100 x 100 x 64 heads 13.5 us either way, 48 x 48 x 64 heads 8.3 against 11.6)
    const bool heavy_f32 = ktype == MI355X_TYPE_F32 && a.D == 128 && (int64_t)a.Nq * a.Nkv * a.Hq * a.B >= 800000;
    if (mixed || (kernel == MI355X_FATTN_MMA && ((convertible && (a.Nq >= 128 || heavy_f32)) || narrow_quant(ktype)))) {
        plan.kv_to_f16 = true;
        plan.workspace = ((size_t)2 * a.D * a.Nkv * a.Hkv * a.Bk * sizeof(uint16_t) + 255) / 256 * 256;
        plan.ws_partials = plan.workspace;
    }
    if (kernel == MI355X_FATTN_MMA) {
        // Very few query tiles and many keys (a short prompt against a long cache): split the keys into ranges of whole
        // 64-key tiles, one workgroup per CU.  Every split repeats the Q load and writes a partial per row, and the merge
        // is a launch of its own, so grids below a quarter of the CUs are split into ranges of at least four tiles, and
        // grids below half of the CUs in two when a workgroup would otherwise walk 16 tiles or more (measured: the
        // Whisper-base encoder, 96 workgroups x 24 key tiles, 25.0 -> 22.0 us in two ranges and slower again in three;
        // a 407-token prefill, 128 workgroups x 7 tiles, loses 2.5 us to any split).
        const int64_t rows    = (int64_t)a.Nq * a.Hq * a.B;
        FattnArgs b  = a;
        int       kt = ktype;
        if (plan.kv_to_f16 && !mixed) {
            use_f16_copies(b, nullptr);
            kt = MI355X_TYPE_F16;
        }
        FattnMmaVariant var;
        fattn_mma_variant(b, kt, var);
        const int     qpw     = var.queries_per_workgroup < 128 ? var.queries_per_workgroup : 128;   // as measured: 128-query units
        const int64_t wgs     = (int64_t)((a.Nq + qpw - 1) / qpw) * a.Hq * a.B;
        const int     n_tiles = (a.Nkv + 63) / 64;
        int ns = p->n_splits;
        if (ns <= 0) {
            // (revised after a sweep of 32 .. 256 queries x 1 .. 40 heads against 1024 .. 8192 keys, ten forced counts each:
            //  tiny grids, one workgroup per CU as before, go down to two tiles per range - 32 queries x 8 heads against 1024
            //  keys under a causal mask 10.7 -> 9.4 us in 8 ranges instead of 4 - but not past 16 ranges, whose merge then
            //  costs more than the shorter loop gains; grids of a quarter to three quarters of the CUs, which were left whole or
            //  cut in two, are cut towards two workgroups per CU in ranges of at least 16 tiles: 256 queries x 40 heads of
            //  128 against 8192 keys, 160 workgroups, 146 -> 81 us in 3 ranges; the Whisper-base encoder's 24 tiles stay whole.)
            ns = 1;
            const int cus = device_cus();
            // (the key-split form of 64-wide heads without a mask walks tiles of 128 keys and more)
            const int nt = var.key_split == 2 && a.D == 64 && !a.masked ? (a.Nkv + 127) / 128 : n_tiles;
            if (wgs * 4 <= cus) {
                int want = (int)(cus / wgs);
                const int by_tiles = nt >= 16 ? nt / 2 : nt / 4;      // (short loops: as before the sweep, which began at 16 tiles)
                if (want > by_tiles) want = by_tiles;
                if (want > 16) want = 16;
                if (want >= 2) ns = want;
            } else if (wgs * 4 <= 3 * (int64_t)cus) {                        // (measured up to 160 workgroups; 320 lose 20% cut in two)
                int want = (int)((4 * (int64_t)cus / wgs + 1) / 2);          // 2 * cus / wgs, rounded
                if (want > nt / 16) want = nt / 16;
                if (want >= 2) ns = want;
            }
        }
        if (ns > n_tiles) ns = n_tiles;
        if (ns < 1) ns = 1;
        if (ns > 64) ns = 64;
        const int tps = (n_tiles + ns - 1) / ns;
        ns = (n_tiles + tps - 1) / tps;
        plan.n_splits = ns;
        plan.keys_per_split = ns > 1 ? tps * 64 : a.Nkv;
        if (ns > 1) plan.workspace += (size_t)rows * ns * (a.D + 2) * sizeof(float);
    }
    if (kernel == MI355X_FATTN_VEC || kernel == MI355X_FATTN_DECODE_MMA) {
        const int64_t rows = (int64_t)a.Nq * a.Hq * a.B;
        // workgroups that exist before splitting, and the fewest keys worth a split
        const int64_t groups   = kernel == MI355X_FATTN_VEC ? rows : (int64_t)a.Hkv * a.B * a.q_chunks;
        // decode kernel: a split must be worth the merge launch (about 2.5 us): measured on Whisper cross-attention
        // (64-wide heads, 1500 keys: best at 8 splits) and a Q8_0 LLM cache (128-wide, 663 keys: best at 6 to 8),
        // while 224 keys are fastest unsplit
        // vector kernel (one workgroup per row and range; sweep of 1 and 2 queries x 8 .. 128 heads x sequences against 224 ..
        // 4096 F32 keys, twelve forced counts each, also with K/V that no cache holds): 1.5 workgroups per CU in all, a power
        // of two per row; ranges of at least 128 keys, for heads wider than 64 of 56 keys up to 448 keys and 112 beyond;
        // at most 8 ranges (16 from 4096 keys on: every range costs its row's merge 0.5 us)
        // (32 heads of 128 against 4096 keys: 29.0 us in 32 ranges, 21.9 in 16; 2 x 128 rows against 1024 keys: 32.8 us in 4, 29.5 in 2)
        const int     min_keys = kernel == MI355X_FATTN_VEC ? (a.D > 64 ? (a.Nkv > 448 ? 112 : 56) : 128) : (a.D <= 64 ? 128 : 64);
        int ns = p->n_splits;
        if (ns <= 0) {
            const int64_t target = kernel == MI355X_FATTN_VEC ? (int64_t)device_cus() * 3 / 2 : (int64_t)device_cus() * 2;
            // whole splits only while they still fit the target: past it a split doubles the grid and adds the merge
            ns = kernel == MI355X_FATTN_VEC ? (int)((target + groups - 1) / (groups > 0 ? groups : 1))
                                            : (int)(target / (groups > 0 ? groups : 1));
            // (decode kernel: to the nearest count - 1500 keys are faster in 8 ranges of 192 than in 7 of 224, 663 in 7 of 96
            //  than in 6 of 128, by 2-3%)
            const int max_by_keys = kernel == MI355X_FATTN_VEC ? (a.Nkv < 2 * min_keys ? 1 : (a.Nkv + min_keys - 1) / min_keys)
                                                               : (a.Nkv + min_keys / 2) / min_keys;
            if (ns > max_by_keys) ns = max_by_keys;
            if (kernel == MI355X_FATTN_VEC) {
                // the workgroup budget rounds down to a power of two
                int by_wgs = 1;
                const int64_t streams = groups / a.gqa > 0 ? groups / a.gqa : 1;      // the rows of a GQA group read the same keys
                while (by_wgs * 2 <= (int)((target + streams - 1) / streams)) by_wgs *= 2;
                ns = by_wgs < max_by_keys ? by_wgs : max_by_keys;
                const int cap = a.Nkv >= 4096 ? 16 : 8;
                if (ns > cap) ns = cap;
            }
            // Decode kernel, long caches under few heads: those bounds alone give 40 to 64 ranges, and every range costs the
            // set's merge (0.2 us each for one row, 0.45 us for sixteen: 4096 f16 keys x 8 heads of 128 took 16 us in
            // 43 ranges and 12 us in 16).  Of the counts up to that bound, take the one a small model likes best -
            // the longer of the cache's pass through HBM (at 5 TB/s) and a wave's chain of 32-key steps (four of them 0.7 us
            // on 64-wide heads, 1.3 us on wider ones, more where workgroups share a CU), plus 1 us for the merge and a
            // share for every range - and the larger count among near-equals (663 keys stay at 7 ranges, 1500 at 8).
            // With K/V that no cache holds, 2 ranges were almost never the best count and up to 384 keys (256 under
            // 128-wide heads) no split was: the fixed microsecond is what keeps those whole.  Against the best of ten forced counts on 192 shapes (1024 .. 8192 keys, 8 .. 40 KV
            // heads x sequences, 1 .. 64 rows each, f16 and Q8_0) this is 5% off in the geometric mean, 35% at worst;
            // the bounds alone were 20% and 2x.
            if (kernel == MI355X_FATTN_DECODE_MMA && ns > 1) {
                const double rows   = (double)(a.Nq * a.gqa < 16 ? a.Nq * a.gqa : 16);
                const double per    = 0.25 + 0.017 * rows;
                double t_hbm = ((double)a.Hkv * a.B * a.Nkv *
                                (double)(a.D / block_size(ktype) * type_size(ktype) + a.D / block_size(vtype) * type_size(vtype)) - 8.0e6) / 5.0e6;
                if (t_hbm < 0.0) t_hbm = 0.0;       // (the first megabytes are a matter of latency, which the chain prices)
                double best = 1e30;
                int    pick = ns;
                for (int pass = 0; pass < 2; pass++)
                    for (int n = 1; n <= ns; n++) {
                        const int kps_n = ((a.Nkv + n - 1) / n + 31) / 32 * 32;
                        if ((a.Nkv + kps_n - 1) / kps_n != n) continue;             // not a count that whole steps give
                        double chain = kps_n / 128.0;
                        if (chain < 1.0) chain = 1.0;
                        chain *= a.D <= 64 ? 0.7 : 1.3;
                        const double per_cu = (double)groups * n / device_cus();     // workgroups sharing a CU share its steps
                        if (per_cu > 1.0) chain *= per_cu;
                        const double est = (chain > t_hbm ? chain : t_hbm) + (n > 1 ? 1.0 + n * per : 0.0);
                        if (pass == 0) { if (est < best) best = est; }
                        else if (est <= best * 1.10) pick = n;
                    }
                ns = pick;
            }
        }
        if (ns > a.Nkv) ns = a.Nkv;
        if (ns < 1) ns = 1;
        if (ns > 256) ns = 256;
        int kps = (a.Nkv + ns - 1) / ns;
        if (kernel == MI355X_FATTN_DECODE_MMA) kps = (kps + 31) / 32 * 32;     // whole wave steps
        if (kps < 1) kps = 1;
        ns = a.Nkv > 0 ? (a.Nkv + kps - 1) / kps : 1;
        plan.n_splits = ns;
        plan.keys_per_split = a.Nkv > 0 ? kps : 0;
        if (ns > 1) plan.workspace += (size_t)rows * ns * (a.D + 2) * sizeof(float);
        if (ns > 1 && groups <= MERGE_COUNTERS) plan.merge_sets = groups;      // (vector kernel: one set per row)
    }
}

// Head sizes the MFMA kernels have no form for (multiples of 8 below 128 other than 64: 32 and 48, 80 and 96 of other
// Whisper-like towers, ...) can still run on them, as the next larger of 64 and 128 with zeros behind the head's own
// elements: the products over the padding are exact zeros, so the result is what the head size itself would give.
//  - The tile kernel: the launch that makes f16 copies of K and V pads their rows, the kernel reads Dv elements of every q
//    row and writes Dv of every dst row.  The cost is the padded share of the MFMA work and the copy.
//  - The decode kernel, over F16 caches: it reads the rows where they lie and pads in its registers.  No copy.
// The vector kernel, which takes any head size, keeps what neither takes: few query rows over F32 and quantised caches,
// and calls too small to pay for the copy launch.
void make_plan(const FattnArgs & a0, int ktype, int vtype, const mi355x_fattn_params * p, Plan & plan) {
    static const bool no_pad = getenv("MI355X_FATTN_NO_PAD") != nullptr;        // comparison runs
    const int pad = a0.D >= 8 && a0.D < 128 && a0.D != 64 && a0.D % 8 == 0 ? (a0.D < 64 ? 64 : 128) : 0;
    // The decode kernel reads f16 rows of such a head size where they lie (no copies): the chunks of a row behind the head's
    // own are zeros in its registers.  It takes the calls the plan at the padded size would give it (5 queries x 16 heads of
    // 80 against 1500 keys: 17.2 us in the vector kernel; 20 heads of 64 take 8.2 us, 10 heads of 128 10.5).
    if (pad && !no_pad && ktype == MI355X_TYPE_F16 && vtype == MI355X_TYPE_F16 &&
        (p->kernel == MI355X_FATTN_AUTO || p->kernel == MI355X_FATTN_DECODE_MMA)) {
        FattnArgs b = a0;
        b.Dv = a0.D;
        b.D  = pad;
        make_plan_core(b, ktype, vtype, p, false, plan);
        // In place the decode kernel has no copy launch to pay for, so it keeps calls further than it does at 64 and 128
        // (decode against vector and padded tile kernel over 1 .. 1024 queries x 4 .. 64 heads x 64 .. 4096 keys at head
        // sizes 32, 48, 80, 96; 864 shapes):
        //  - up to 16 rows per KV head: always, whatever the plan at the padded size says of 9 .. 16 rows (the tile kernel
        //    would need the copies; the vector kernel is level at 64 keys and 1 - 2 us behind from 256 on);
        //  - more rows: up to 64 chunks of 16 per KV head, each of which streams the head's K/V again, in up to three rounds
        //    of workgroups, while a head's chunks see no more than 64k keys between them and all chunks 512k.
        // These rules are 1% off the fastest of the three in the geometric mean (1.5x at worst); the tile kernel alone is
        // 11-19% off on the shapes of more than 16 rows, the vector kernel 2 to 10 times slower from 1024 keys on.
        if (p->kernel == MI355X_FATTN_AUTO && fattn_decode_supported(b, ktype)) {
            bool dec = plan.kernel == MI355X_FATTN_DECODE_MMA;
            if (a0.q_chunks <= 1) {
                dec = true;
            } else if (!dec) {
                const int64_t chunk_wgs = (int64_t)a0.q_chunks * a0.Hkv * a0.B;
                dec = a0.q_chunks <= 64 && chunk_wgs <= 3 * (int64_t)device_cus() &&
                      (int64_t)a0.q_chunks * a0.Nkv <= (1 << 16) && chunk_wgs * a0.Nkv <= (1 << 19);
            }
            if (dec && plan.kernel != MI355X_FATTN_DECODE_MMA) {
                mi355x_fattn_params by_name = *p;
                by_name.kernel = MI355X_FATTN_DECODE_MMA;
                make_plan_core(b, ktype, vtype, &by_name, false, plan);
            }
            if (!dec) plan.kernel = MI355X_FATTN_AUTO;          // (not this kernel: the tile kernel on copies, or the vector kernel)
        }
        if (plan.kernel == MI355X_FATTN_DECODE_MMA && fattn_decode_supported(b, ktype)) {
            plan.pad = pad;
            return;
        }
    }
    if (pad && !no_pad && (p->kernel == MI355X_FATTN_AUTO || p->kernel == MI355X_FATTN_MMA)) {
        FattnArgs b = a0;
        b.Dv = a0.D;
        b.D  = pad;
        make_plan_core(b, ktype, vtype, p, true, plan);
        const int64_t pairs = (int64_t)a0.Nq * a0.Hq * a0.B * a0.Nkv;
        // (vector against padded tile kernel over 2 .. 1500 queries x 4 .. 64 heads x 64 .. 1500 keys at head sizes 32, 48, 80
        //  and 96, f16 and F32 K/V, the choice against the faster of the two: from 16 queries and 100k (query row, key)
        //  pairs on the copy launch and the padding pay - 1 to 3% off in the geometric mean, where the vector kernel alone
        //  is 27 to 71% off and 16 to 44 times slower at worst; above 64 also for 2 .. 15 queries from 150k pairs on, as
        //  for F32 caches of the sizes the tile kernel has forms for)
        // (where the padded plan would take the decode kernel - 16 queries or more in 16-row chunks over F32 or quantised
        //  K/V, which that kernel does not pad - the tile kernel stands in: the vector kernel is 2 to 4 times slower there)
        bool want = p->kernel == MI355X_FATTN_MMA;
        if (!want) {
            want = (pairs >= 100000 && (plan.kernel == MI355X_FATTN_MMA || (plan.kernel == MI355X_FATTN_DECODE_MMA && a0.Nq >= 16))) ||
                   (pad == 128 && a0.Nq >= 2 && a0.Nq < 16 && pairs >= 150000);
        }
        bool tile = want;
        if (want && p->kernel == MI355X_FATTN_AUTO) {
            if (plan.kernel != MI355X_FATTN_MMA) {
                mi355x_fattn_params by_name = *p;
                by_name.kernel = MI355X_FATTN_MMA;
                make_plan_core(b, ktype, vtype, &by_name, true, plan);
            }
            FattnArgs c = b;
            use_f16_copies(c, nullptr);
            tile = fattn_mma_supported(c, MI355X_TYPE_F16);
        }
        if (tile) {
            plan.pad = pad;
            return;
        }
    }
    make_plan_core(a0, ktype, vtype, p, false, plan);
}

// q_quant: the query rows rounded to Q8_0 and back, as contiguous F32 [D, Nq, Hq, B] at ws + q8_bytes
size_t qq_q8_bytes(const mi355x_tensor * q) {
    return ((size_t)q->ne[0] / FATTN_QK8_0 * FATTN_Q8_0_BYTES * q->ne[1] * q->ne[2] * q->ne[3] + 255) / 256 * 256;
}
size_t qq_f32_bytes(const mi355x_tensor * q) {
    return ((size_t)q->ne[0] * q->ne[1] * q->ne[2] * q->ne[3] * sizeof(float) + 255) / 256 * 256;
}
void qq_view(const mi355x_tensor * q, void * data, mi355x_tensor * out) {
    *out = *q;
    out->data = data;
    out->nb[0] = sizeof(float);
    out->nb[1] = (size_t)q->ne[0] * sizeof(float);
    out->nb[2] = out->nb[1] * (size_t)q->ne[1];
    out->nb[3] = out->nb[2] * (size_t)q->ne[2];
}
int qq_run(const mi355x_tensor * q, void * ws, hipStream_t st) {
    CpyArgs c;
    memset(&c, 0, sizeof(c));
    int64_t blocks = 1;
    for (int i = 0; i < 4; i++) { c.sne[i] = c.dne[i] = q->ne[i]; c.snb[i] = (int64_t)q->nb[i]; }
    const int64_t rs = q->ne[0] / FATTN_QK8_0 * FATTN_Q8_0_BYTES;
    c.dnb[0] = FATTN_Q8_0_BYTES; c.dnb[1] = rs; c.dnb[2] = rs * q->ne[1]; c.dnb[3] = c.dnb[2] * q->ne[2];
    blocks = q->ne[0] / FATTN_QK8_0 * q->ne[1] * q->ne[2] * q->ne[3];
    c.src = (const char *)q->data; c.dst = (char *)ws; c.n = blocks;
    int e = cpy_launch(c, MI355X_TYPE_F32, MI355X_TYPE_Q8_0, st);
    if (e) return hip_fail((hipError_t)e, "query quantisation launch");
    CpyArgs d;
    memset(&d, 0, sizeof(d));
    for (int i = 0; i < 4; i++) { d.sne[i] = d.dne[i] = q->ne[i]; d.snb[i] = c.dnb[i]; }
    d.dnb[0] = 4; d.dnb[1] = 4 * q->ne[0]; d.dnb[2] = d.dnb[1] * q->ne[1]; d.dnb[3] = d.dnb[2] * q->ne[2];
    d.src = (const char *)ws; d.dst = (char *)ws + qq_q8_bytes(q); d.n = blocks;
    e = cpy_launch(d, MI355X_TYPE_Q8_0, MI355X_TYPE_F32, st);
    if (e) return hip_fail((hipError_t)e, "query dequantisation launch");
    return MI355X_OK;
}

}  // namespace

extern "C" {

int mi355x_api_version(void) { return MI355X_FATTN_API_VERSION; }

const char * mi355x_status_string(int status) {
    switch (status) {
        case MI355X_OK:              return "ok";
        case MI355X_ERR_UNSUPPORTED: return "unsupported";
        case MI355X_ERR_INVALID:     return "invalid argument";
        case MI355X_ERR_HIP:         return "HIP runtime error";
        case MI355X_ERR_NO_DEVICE:   return "no device";
        case MI355X_ERR_WORKSPACE:   return "workspace too small";
        default:                     return "unknown status";
    }
}

const char * mi355x_last_error(void) { return g_err; }

int mi355x_device_count(int * count) {
    if (!count) return fail(MI355X_ERR_INVALID, "null argument");
    int n = 0;
    const hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) {
        *count = 0;
        (void)hipGetLastError();
        return fail(MI355X_ERR_NO_DEVICE, "hipGetDeviceCount: %s", hipGetErrorString(e));
    }
    *count = n;
    return MI355X_OK;
}

int mi355x_device_get_info(int device, mi355x_device_info * info) {
    if (!info) return fail(MI355X_ERR_INVALID, "null argument");
    hipDeviceProp_t prop;
    HIP_TRY(hipGetDeviceProperties(&prop, device));
    memset(info, 0, sizeof(*info));
    snprintf(info->name, sizeof(info->name), "%s", prop.name);
    snprintf(info->arch, sizeof(info->arch), "%s", prop.gcnArchName);
    info->compute_units       = prop.multiProcessorCount;
    info->clock_khz           = prop.clockRate;
    info->memory_clock_khz    = prop.memoryClockRate;
    info->memory_bus_bits     = prop.memoryBusWidth;
    info->total_memory        = prop.totalGlobalMem;
    info->lds_bytes_per_block = (int32_t)prop.sharedMemPerBlock;
    info->wavefront_size      = prop.warpSize;
    int cur = 0;
    HIP_TRY(hipGetDevice(&cur));
    HIP_TRY(hipSetDevice(device));
    size_t fr = 0, tot = 0;
    const hipError_t e = hipMemGetInfo(&fr, &tot);
    (void)hipSetDevice(cur);
    if (e != hipSuccess) return hip_fail(e, "hipMemGetInfo");
    info->free_memory = fr;
    return MI355X_OK;
}

int mi355x_set_device(int device) {
    HIP_TRY(hipSetDevice(device));
    // Set-up of mi355x_flash_attn_ext_noalloc for this device happens here when the caller comes this way - as a courtesy:
    // a failed lookup must not cost the caller the device (most never use that entry point, which reports the failure itself
    // on its first call).
    void * ptr = nullptr;
    if (noalloc_scratch(&ptr) != MI355X_OK) g_err[0] = 0;
    return MI355X_OK;
}

int mi355x_stream_synchronize(void * stream) {
    HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
    return MI355X_OK;
}

int mi355x_fattn_supports(const mi355x_tensor * q, const mi355x_tensor * k, const mi355x_tensor * v,
                          const mi355x_tensor * mask, const mi355x_tensor * dst,
                          const mi355x_fattn_params * params) {
    return check(q, k, v, mask, dst, params);
}

int mi355x_fattn_plan(const mi355x_tensor * q, const mi355x_tensor * k, const mi355x_tensor * v,
                      const mi355x_tensor * mask, const mi355x_fattn_params * params,
                      int32_t * kernel, int32_t * n_splits) {
    const int rc = check(q, k, v, mask, nullptr, params);
    if (rc) return rc;
    FattnArgs a;
    fill_args(a, q, k, v, mask, nullptr, params);
    Plan plan;
    make_plan(a, k->type, v->type, params, plan);
    if (kernel) *kernel = plan.kernel;
    if (n_splits) *n_splits = plan.n_splits;
    return MI355X_OK;
}

int mi355x_fattn_plan_details(const mi355x_tensor * q, const mi355x_tensor * k, const mi355x_tensor * v,
                              const mi355x_tensor * mask, const mi355x_fattn_params * params,
                              mi355x_fattn_plan_info * info) {
    if (!info) return fail(MI355X_ERR_INVALID, "null argument");
    const int rc = check(q, k, v, mask, nullptr, params);
    if (rc) return rc;
    FattnArgs a;
    fill_args(a, q, k, v, mask, nullptr, params);
    Plan plan;
    make_plan(a, k->type, v->type, params, plan);
    memset(info, 0, sizeof(*info));
    info->kernel         = plan.kernel;
    info->n_splits       = plan.n_splits;
    info->keys_per_split = plan.keys_per_split;
    info->kv_to_f16      = plan.kv_to_f16 ? 1 : 0;
    info->workspace      = plan.workspace;
    info->head_pad       = plan.pad;
    info->merge_in_kernel = plan.merge_sets > 0 && !params->workspace && !g_no_fused_merge ? 1 : 0;
    if (plan.kernel == MI355X_FATTN_MMA) {
        // the order of the call itself: the f16 copies first, then the question whether the tile kernel takes the shape
        int ktype = k->type;
        apply_pad(a, plan);
        if (plan.kv_to_f16) {
            use_f16_copies(a, nullptr);
            ktype = MI355X_TYPE_F16;
        }
        if (!fattn_mma_supported(a, ktype)) return MI355X_OK;
        a.n_splits = plan.n_splits;
        a.keys_per_split = plan.keys_per_split;
        FattnMmaVariant var;
        fattn_mma_variant(a, ktype, var);
        info->queries_per_workgroup = var.queries_per_workgroup;
        info->query_blocks = var.query_blocks;
        info->key_split    = var.key_split;
        info->direct       = var.direct ? 1 : 0;
        info->mask_dma     = var.mask_dma ? 1 : 0;
    }
    return MI355X_OK;
}

int mi355x_fattn_workspace_size(const mi355x_tensor * q, const mi355x_tensor * k, const mi355x_tensor * v,
                                const mi355x_tensor * mask, const mi355x_fattn_params * params,
                                size_t * bytes) {
    if (!bytes) return fail(MI355X_ERR_INVALID, "null argument");
    const int rc = check(q, k, v, mask, nullptr, params);
    if (rc) return rc;
    FattnArgs a;
    fill_args(a, q, k, v, mask, nullptr, params);
    Plan plan;
    make_plan(a, k->type, v->type, params, plan);
    *bytes = plan.workspace + (params->q_quant ? qq_q8_bytes(q) + qq_f32_bytes(q) : 0);
    return MI355X_OK;
}

// counter_set: which of the library's counter sets a launch that merges its splits in the kernel may use (-1: none)
static int flash_attn_run(const mi355x_tensor * q, const mi355x_tensor * k, const mi355x_tensor * v,
                          const mi355x_tensor * mask, const mi355x_tensor * dst,
                          const mi355x_fattn_params * params, void * stream, int counter_set) {
    if (!dst) return fail(MI355X_ERR_INVALID, "null dst");
    int rc = check(q, k, v, mask, dst, params);
    if (rc) return rc;
    if (q->ne[1] != 0 && (!q->data || !k->data || !v->data || !dst->data || (has_mask(mask) && !mask->data)))
        return fail(MI355X_ERR_INVALID, "null data pointer");
    if (params->q_quant && (int64_t)q->ne[1] * q->ne[2] * q->ne[3] > 0) {
        // the rounded query rows go to the head of the workspace; the call proper runs on them with what is left of it
        const size_t qb = qq_q8_bytes(q) + qq_f32_bytes(q);
        mi355x_fattn_params inner = *params;
        inner.q_quant = 0;
        size_t need = 0;
        rc = mi355x_fattn_workspace_size(q, k, v, mask, &inner, &need);
        if (rc) return rc;
        void * ws = params->workspace;
        if (ws) {
            if (params->workspace_size < qb + need)
                return fail(MI355X_ERR_WORKSPACE, "workspace %zu < %zu bytes", params->workspace_size, qb + need);
            if ((uintptr_t)ws % 16) return fail(MI355X_ERR_WORKSPACE, "workspace must be 16-byte aligned");
        } else {
            rc = get_scratch(qb + need, &ws, (hipStream_t)stream);
            if (rc) return rc;
        }
        rc = qq_run(q, ws, (hipStream_t)stream);
        if (rc) return rc;
        mi355x_tensor qd;
        qq_view(q, (char *)ws + qq_q8_bytes(q), &qd);
        inner.workspace      = need ? (char *)ws + qb : nullptr;
        inner.workspace_size = need;
        return flash_attn_run(&qd, k, v, mask, dst, &inner, stream, counter_set);
    }
    // K and V of a cache that lives in a host buffer are read from that buffer's mirror in HBM
    mi355x_tensor km = *k, vm = *v;
    if ((int64_t)q->ne[1] * q->ne[2] * q->ne[3] > 0 && k->ne[1] > 0) {
        rc = mirror_for_read(k, (hipStream_t)stream, &km.data);
        if (rc) return rc;
        rc = mirror_for_read(v, (hipStream_t)stream, &vm.data);
        if (rc) return rc;
    }
    k = &km;
    v = &vm;
    mirror_note_host_write(dst);
    FattnArgs a;
    fill_args(a, q, k, v, mask, (float *)dst->data, params);
    if ((int64_t)a.Nq * a.Hq * a.B == 0) return MI355X_OK;

    Plan plan;
    make_plan(a, k->type, v->type, params, plan);
    apply_pad(a, plan);
    hipStream_t st = (hipStream_t)stream;

    int ktype = k->type;
    if (plan.kernel == MI355X_FATTN_MMA) {
        FattnArgs b = a;
        if (plan.kv_to_f16) use_f16_copies(b, nullptr);
        if (!fattn_mma_supported(b, plan.kv_to_f16 ? MI355X_TYPE_F16 : ktype))
            return fail(MI355X_ERR_UNSUPPORTED, "shape not covered by the MFMA kernel");
    } else if (plan.kernel == MI355X_FATTN_DECODE_MMA) {
        FattnArgs b = a;
        if (plan.kv_to_f16) use_f16_copies(b, nullptr);
        if (!fattn_decode_supported(b, plan.kv_to_f16 ? MI355X_TYPE_F16 : ktype))
            return fail(MI355X_ERR_UNSUPPORTED, "shape not covered by the decode kernel");
    } else if (plan.kernel != MI355X_FATTN_VEC) {
        return fail(MI355X_ERR_UNSUPPORTED, "kernel %d not available", plan.kernel);
    }
    void * ws = nullptr;
    if (plan.workspace) {
        ws = params->workspace;
        if (ws) {
            if (params->workspace_size < plan.workspace)
                return fail(MI355X_ERR_WORKSPACE, "workspace %zu < %zu bytes", params->workspace_size, plan.workspace);
            if ((uintptr_t)ws % 16) return fail(MI355X_ERR_WORKSPACE, "workspace must be 16-byte aligned");
        } else {
            rc = get_scratch(plan.workspace, &ws, st);
            if (rc) return rc;
        }
    }
    if (plan.kv_to_f16) {
        const int e = kv_to_f16_launch(a, k->type, v->type, ws, st);
        if (e) return hip_fail((hipError_t)e, "K/V conversion launch");
        use_f16_copies(a, ws);
        ktype = MI355X_TYPE_F16;
    }
    a.n_splits = plan.n_splits;
    a.keys_per_split = plan.keys_per_split;
    if (plan.n_splits > 1) {
        const size_t rows = (size_t)a.Nq * a.Hq * a.B;
        a.part_acc = (float *)((char *)ws + plan.ws_partials);
        a.part_ml  = a.part_acc + rows * plan.n_splits * a.D;
        if (plan.merge_sets > 0) a.counters = merge_counter_set(counter_set);
    }
    int e = plan.kernel == MI355X_FATTN_MMA   ? fattn_mma_launch(a, ktype, st)
            : plan.kernel == MI355X_FATTN_VEC ? fattn_vec_launch(a, ktype, st)
                                              : fattn_decode_launch(a, ktype, st);
    if (e) return hip_fail((hipError_t)e, "attention kernel launch");
    if (plan.n_splits > 1 && !a.counters) {
        e = fattn_merge_launch(a, st);
        if (e) return hip_fail((hipError_t)e, "fattn_merge launch");
    }
    return MI355X_OK;
}

int mi355x_flash_attn_ext(const mi355x_tensor * q, const mi355x_tensor * k, const mi355x_tensor * v,
                          const mi355x_tensor * mask, const mi355x_tensor * dst,
                          const mi355x_fattn_params * params, void * stream) {
    // on the library's scratch block (one call at a time per GPU by contract) the kernel may merge its splits itself
    return flash_attn_run(q, k, v, mask, dst, params, stream, params && !params->workspace ? 0 : -1);
}

int mi355x_flash_attn_ext_noalloc(const mi355x_tensor * q, const mi355x_tensor * k, const mi355x_tensor * v,
                                  const mi355x_tensor * mask, const mi355x_tensor * dst,
                                  const mi355x_fattn_params * params, void * stream) {
    if (!params) return fail(MI355X_ERR_INVALID, "null argument");
    void * ptr = nullptr;
    int rc = noalloc_scratch(&ptr);
    if (rc) return rc;
    size_t need = 0;
    rc = mi355x_fattn_workspace_size(q, k, v, mask, params, &need);
    if (rc) return rc;
    if (need > (size_t)MI355X_NOALLOC_SCRATCH_BYTES)
        return fail(MI355X_ERR_WORKSPACE, "this call needs %zu bytes of scratch; the allocation-free entry point holds %zu",
                    need, (size_t)MI355X_NOALLOC_SCRATCH_BYTES);
    mi355x_fattn_params inner = *params;
    inner.workspace      = ptr;          // the kernels take the array's device address as they take any workspace
    inner.workspace_size = (size_t)MI355X_NOALLOC_SCRATCH_BYTES;
    return flash_attn_run(q, k, v, mask, dst, &inner, stream, 1);
}

// ---- copies ------------------------------------------------------------------------------

static int cpy_check(const mi355x_tensor * src, const mi355x_tensor * dst) {
    if (!src || !dst) return fail(MI355X_ERR_INVALID, "null argument");
    const int s = src->type, d = dst->type;
    const bool sb = FATTN_IS_BLOCK_TYPE(s), db = FATTN_IS_BLOCK_TYPE(d);
    const bool ok = (s == MI355X_TYPE_F32 && (d == MI355X_TYPE_F32 || d == MI355X_TYPE_F16 || db)) ||
                    (s == MI355X_TYPE_F16 && (d == MI355X_TYPE_F16 || d == MI355X_TYPE_F32)) ||
                    (sb && (d == MI355X_TYPE_F32 || d == s));
    if (!ok) return fail(MI355X_ERR_UNSUPPORTED, "copy %d -> %d not covered", s, d);
    int64_t ns = 1, nd = 1;
    if (!sane_extents(src, &ns) || !sane_extents(dst, &nd)) return fail(MI355X_ERR_INVALID, "negative or oversized extent");
    if (ns != nd) return fail(MI355X_ERR_INVALID, "element counts differ (%lld vs %lld)", (long long)ns, (long long)nd);
    if (dst->nb[0] != type_size(d)) return fail(MI355X_ERR_UNSUPPORTED, "dst rows must be contiguous");
    if (sb && src->nb[0] != type_size(s)) return fail(MI355X_ERR_UNSUPPORTED, "src blocks must be contiguous");
    if (sb || db) {
        if (src->ne[0] % FATTN_QK8_0 || dst->ne[0] % FATTN_QK8_0)
            return fail(MI355X_ERR_INVALID, "quantised copies need ne0 %% 32 == 0 on both sides");
    }
    // every access is at least element-wide (Q8_0 blocks are read and written in 2-byte units)
    const size_t sal = s == MI355X_TYPE_F32 ? 4 : 2, dal = d == MI355X_TYPE_F32 ? 4 : 2;
    if ((uintptr_t)src->data % sal || (uintptr_t)dst->data % dal) return fail(MI355X_ERR_UNSUPPORTED, "misaligned data pointers");
    for (int i = 0; i < 4; i++)
        if (src->nb[i] % sal || dst->nb[i] % dal) return fail(MI355X_ERR_UNSUPPORTED, "misaligned strides");
    return MI355X_OK;
}

// ---- FastConformer relative-position mask --------------------------------------------------------------------

static bool aligned16_view(const mi355x_tensor * t) {
    if ((uintptr_t)t->data % 16) return false;
    for (int i = 1; i < 4; i++)
        if (t->ne[i] > 1 && t->nb[i] % 16) return false;
    return true;
}

static int relpos_check(const mi355x_tensor * qv, const mi355x_tensor * r, const mi355x_tensor * add,
                        const mi355x_tensor * dst) {
    if (!qv || !r || !dst) return fail(MI355X_ERR_INVALID, "null argument");
    if (!sane_extents(qv, nullptr) || !sane_extents(r, nullptr) || !sane_extents(dst, nullptr) || (add && !sane_extents(add, nullptr)))
        return fail(MI355X_ERR_INVALID, "negative or oversized extent");
    if (qv->type != MI355X_TYPE_F32 || qv->nb[0] != 4) return fail(MI355X_ERR_UNSUPPORTED, "q_v must be F32 with unit element stride");
    if (r->type != MI355X_TYPE_F32 && r->type != MI355X_TYPE_F16) return fail(MI355X_ERR_UNSUPPORTED, "r type %d not covered", r->type);
    if (r->nb[0] != type_size(r->type)) return fail(MI355X_ERR_UNSUPPORTED, "r rows must be contiguous");
    if (dst->type != MI355X_TYPE_F16 || dst->nb[0] != 2) return fail(MI355X_ERR_INVALID, "dst must be F16 with contiguous rows");
    const int64_t D = qv->ne[0], Nq = qv->ne[1], H = qv->ne[2], B = qv->ne[3];
    const int64_t Nkv = dst->ne[0];
    if (D != 64 && D != 128) return fail(MI355X_ERR_UNSUPPORTED, "head size %lld not covered (64, 128)", (long long)D);
    if (dst->ne[1] != Nq || dst->ne[2] != H || dst->ne[3] != B) return fail(MI355X_ERR_INVALID, "dst shape does not match q_v");
    if (Nq < 0 || Nkv < 0 || H <= 0 || B <= 0) return fail(MI355X_ERR_INVALID, "bad extents");
    if (Nq > 0 && Nkv > 0 && (r->ne[0] != D || r->ne[1] != Nq + Nkv - 1))
        return fail(MI355X_ERR_INVALID, "r must be [D, Nq+Nkv-1, ..]: got [%lld, %lld], want [%lld, %lld]",
                    (long long)r->ne[0], (long long)r->ne[1], (long long)D, (long long)(Nq + Nkv - 1));
    if (r->ne[2] <= 0 || r->ne[3] <= 0 || H % r->ne[2] || B % r->ne[3]) return fail(MI355X_ERR_INVALID, "r heads / batch do not divide q_v's");
    if (Nq + Nkv > (1 << 24) || H * B > (1 << 24)) return fail(MI355X_ERR_UNSUPPORTED, "extent too large");
    const uint64_t lim = (uint64_t)1 << 31;      // the kernel keeps 32-bit offsets inside a (head, batch) plane
    if ((uint64_t)Nq * qv->nb[1] >= lim || (uint64_t)(Nq + Nkv) * D * 2 >= lim || (uint64_t)Nq * dst->nb[1] >= lim ||
        (add && add->ne[0] > 0 && (uint64_t)Nq * add->nb[1] >= lim))
        return fail(MI355X_ERR_UNSUPPORTED, "a (head, batch) plane exceeds 2 GiB");
    if (qv->data && !aligned16_view(qv)) return fail(MI355X_ERR_UNSUPPORTED, "q_v must be 16-byte aligned");
    if (r->data && !aligned16_view(r)) return fail(MI355X_ERR_UNSUPPORTED, "r must be 16-byte aligned");
    if (dst->nb[1] < (size_t)Nkv * 2 || (dst->nb[1] & 1) || (dst->nb[2] & 1) || (dst->nb[3] & 1)) return fail(MI355X_ERR_INVALID, "bad dst strides");
    if (add && add->ne[0] > 0) {
        if (add->type != MI355X_TYPE_F32 && add->type != MI355X_TYPE_F16) return fail(MI355X_ERR_UNSUPPORTED, "add type %d not covered", add->type);
        if (add->nb[0] != type_size(add->type)) return fail(MI355X_ERR_UNSUPPORTED, "add rows must be contiguous");
        if (add->ne[0] < Nkv || add->ne[1] < Nq) return fail(MI355X_ERR_INVALID, "add is smaller than [Nkv, Nq]");
        if (add->ne[2] <= 0 || add->ne[3] <= 0 || H % add->ne[2] || B % add->ne[3]) return fail(MI355X_ERR_INVALID, "add heads / batch do not divide q_v's");
        const size_t es = type_size(add->type);
        if ((add->data && (uintptr_t)add->data % es) || add->nb[1] % es || add->nb[2] % es || add->nb[3] % es) return fail(MI355X_ERR_UNSUPPORTED, "add is not element-aligned");
    }
    return MI355X_OK;
}

// bytes of the contiguous f16 copy the kernel reads (0 for an F16 table with contiguous rows, which is read in place)
static size_t relpos_table_bytes(const mi355x_tensor * r) {
    if (r->type == MI355X_TYPE_F16 && r->nb[1] == (size_t)r->ne[0] * 2) return 0;
    return ((size_t)r->ne[0] * r->ne[1] * r->ne[2] * r->ne[3] * 2 + 255) / 256 * 256;
}

// r16: room for relpos_table_bytes(r), or NULL to take it from the library's scratch
static int relpos_run(const mi355x_tensor * qv, const mi355x_tensor * r, const mi355x_tensor * add,
                      const mi355x_tensor * dst, float scale, void * r16, hipStream_t st) {
    RelposArgs a;
    memset(&a, 0, sizeof(a));
    a.D = (int)qv->ne[0]; a.Nq = (int)qv->ne[1]; a.H = (int)qv->ne[2]; a.B = (int)qv->ne[3];
    a.Nkv = (int)dst->ne[0];
    if ((int64_t)a.Nq * a.Nkv * a.H * a.B == 0) return MI355X_OK;
    const bool has_add = add && add->ne[0] > 0;
    if (!qv->data || !r->data || !dst->data || (has_add && !add->data)) return fail(MI355X_ERR_INVALID, "null data pointer");
    a.qv = (const char *)qv->data; a.nbq1 = qv->nb[1]; a.nbq2 = qv->nb[2]; a.nbq3 = qv->nb[3];
    a.r  = (const char *)r->data;  a.nbr1 = r->nb[1];  a.nbr2 = r->nb[2];  a.nbr3 = r->nb[3];
    a.Hr = (int)r->ne[2]; a.Br = (int)r->ne[3];
    if (relpos_table_bytes(r)) {
        // the kernel multiplies f16 values anyway: round the table once, into a contiguous [D, NR, Hr, Br] copy
        if (!r16) {
            const int rc = get_scratch(relpos_table_bytes(r), &r16, st);
            if (rc) return rc;
        }
        CpyArgs c;
        memset(&c, 0, sizeof(c));
        c.src = (const char *)r->data;
        c.dst = (char *)r16;
        int64_t nb = 2;
        c.n = 1;
        for (int i = 0; i < 4; i++) {
            c.sne[i] = c.dne[i] = r->ne[i];
            c.snb[i] = (int64_t)r->nb[i];
            c.dnb[i] = nb;
            nb *= r->ne[i];
            c.n *= r->ne[i];
        }
        const int e = cpy_launch(c, r->type, MI355X_TYPE_F16, st);
        if (e) return hip_fail((hipError_t)e, "table conversion launch");
        a.r = (const char *)r16;
        a.nbr1 = (size_t)a.D * 2; a.nbr2 = a.nbr1 * (size_t)r->ne[1]; a.nbr3 = a.nbr2 * (size_t)r->ne[2];
    }
    a.Ha = a.Ba = 1;
    if (has_add) {
        a.add = (const char *)add->data; a.nba1 = add->nb[1]; a.nba2 = add->nb[2]; a.nba3 = add->nb[3];
        a.Ha = (int)add->ne[2]; a.Ba = (int)add->ne[3];
        a.add_f16 = add->type == MI355X_TYPE_F16;
    }
    mirror_note_host_write(dst);
    a.out = (char *)dst->data; a.nbo1 = dst->nb[1]; a.nbo2 = dst->nb[2]; a.nbo3 = dst->nb[3];
    a.out_al4 = !((uintptr_t)dst->data % 4) && !(dst->nb[1] % 4) && !(dst->nb[2] % 4) && !(dst->nb[3] % 4);
    a.scale = scale;
    a.n_cus = device_cus();
    const int e = relpos_bias_launch(a, MI355X_TYPE_F16, st);
    if (e) return hip_fail((hipError_t)e, "relpos_bias launch");
    return MI355X_OK;
}

int mi355x_relpos_bias_supports(const mi355x_tensor * q_v, const mi355x_tensor * r, const mi355x_tensor * add,
                                const mi355x_tensor * dst) {
    return relpos_check(q_v, r, add, dst);
}

int mi355x_relpos_bias_workspace_size(const mi355x_tensor * r, size_t * bytes) {
    if (!r || !bytes) return fail(MI355X_ERR_INVALID, "null argument");
    if (!sane_extents(r, nullptr) || !type_size(r->type)) return fail(MI355X_ERR_INVALID, "bad table");
    *bytes = relpos_table_bytes(r);
    return MI355X_OK;
}

int mi355x_relpos_bias(const mi355x_tensor * q_v, const mi355x_tensor * r, const mi355x_tensor * add,
                       const mi355x_tensor * dst, float scale, void * workspace, size_t workspace_size, void * stream) {
    const int rc = relpos_check(q_v, r, add, dst);
    if (rc) return rc;
    const size_t need = relpos_table_bytes(r);
    if (workspace && need) {
        if (workspace_size < need) return fail(MI355X_ERR_WORKSPACE, "workspace %zu < %zu bytes", workspace_size, need);
        if ((uintptr_t)workspace % 16) return fail(MI355X_ERR_WORKSPACE, "workspace must be 16-byte aligned");
    }
    return relpos_run(q_v, r, add, dst, scale, need ? workspace : nullptr, (hipStream_t)stream);
}

// the mask the fused call keeps in its workspace: [Nkv, Nq, H, B] with rows padded to whole 128-byte lines
static void relpos_mask_view(const mi355x_tensor * q_u, const mi355x_tensor * k, void * data, mi355x_tensor * m) {
    memset(m, 0, sizeof(*m));
    m->data = data;
    m->type = MI355X_TYPE_F16;
    m->ne[0] = k->ne[1]; m->ne[1] = q_u->ne[1]; m->ne[2] = q_u->ne[2]; m->ne[3] = q_u->ne[3];
    m->nb[0] = 2;
    m->nb[1] = ((size_t)k->ne[1] * 2 + 127) / 128 * 128;
    m->nb[2] = m->nb[1] * (size_t)q_u->ne[1];
    m->nb[3] = m->nb[2] * (size_t)q_u->ne[2];
}

static int relpos_fused_check(const mi355x_tensor * q_u, const mi355x_tensor * q_v, const mi355x_tensor * k,
                              const mi355x_tensor * v, const mi355x_tensor * r, const mi355x_tensor * add,
                              const mi355x_tensor * dst, const mi355x_fattn_params * params, mi355x_tensor * m,
                              size_t * mask_bytes, size_t * inner_bytes) {
    if (!q_u || !q_v || !k || !v || !r || !params) return fail(MI355X_ERR_INVALID, "null argument");
    if (params->max_bias != 0.0f || params->logit_softcap != 0.0f)
        return fail(MI355X_ERR_UNSUPPORTED, "relative-position attention takes neither max_bias nor logit_softcap");
    for (int i = 0; i < 4; i++)
        if (q_u->ne[i] != q_v->ne[i]) return fail(MI355X_ERR_INVALID, "q_u and q_v shapes differ");
    relpos_mask_view(q_u, k, nullptr, m);
    int rc = relpos_check(q_v, r, add, m);
    if (rc) return rc;
    rc = check(q_u, k, v, m, dst, params);
    if (rc) return rc;
    *mask_bytes = (m->nb[3] * (size_t)q_u->ne[3] + 255) / 256 * 256 + relpos_table_bytes(r);      // the mask, then the f16 table
    FattnArgs a;
    fill_args(a, q_u, k, v, m, nullptr, params);
    Plan plan;
    make_plan(a, k->type, v->type, params, plan);
    *inner_bytes = plan.workspace;
    return MI355X_OK;
}

// The one-kernel form: taken when no kernel is asked for by name and the shape fits it.  Workspace: f16 copies of K and V
// (unless they are f16 with 16-byte rows already), then the f16 table (unless it is read in place).
struct RelposFused {
    bool   ok;
    bool   kv_copy;
    size_t kv_bytes, table_bytes;
};
static RelposFused relpos_fused_plan(const mi355x_tensor * q_u, const mi355x_tensor * q_v, const mi355x_tensor * k,
                                     const mi355x_tensor * v, const mi355x_tensor * r, const mi355x_tensor * add,
                                     const mi355x_fattn_params * params) {
    RelposFused f = {false, false, 0, 0};
    static const bool off = getenv("MI355X_RELPOS_TWO_LAUNCHES") != nullptr;        // comparison runs
    if (off || params->kernel != MI355X_FATTN_AUTO || params->n_splits > 1 || params->q_quant) return f;
    const int64_t D = q_u->ne[0];
    if ((D != 64 && D != 128) || q_u->ne[1] < 1 || k->ne[1] < 1) return f;
    FattnArgs a;
    fill_args(a, q_u, k, v, nullptr, nullptr, params);
    if (!a.q_aligned16 || !aligned16_view(q_v)) return f;
    if (add && add->ne[0] > 0) {
        const size_t es = type_size(add->type);
        if (add->nb[0] != es) return f;
    }
    if (k->type == MI355X_TYPE_F16 && v->type == MI355X_TYPE_F16 && a.kv_aligned16) {
        f.kv_copy = false;
    } else if (k->type != v->type || (k->type == MI355X_TYPE_F32 && a.kv_aligned16) || (FATTN_IS_BLOCK_TYPE(k->type) && a.kv_aligned2)) {
        f.kv_copy  = true;
        f.kv_bytes = ((size_t)2 * a.D * a.Nkv * a.Hkv * a.Bk * sizeof(uint16_t) + 255) / 256 * 256;
    } else {
        return f;
    }
    f.table_bytes = relpos_table_bytes(r);
    if (!f.table_bytes && !aligned16_view(r)) return f;
    // the kernel keeps 32-bit byte offsets inside a (head, batch) plane of K, V and the table
    const uint64_t lim = (uint64_t)1 << 31;
    const uint64_t kpitch = f.kv_copy ? (uint64_t)a.D * 2 : (uint64_t)k->nb[1], vpitch = f.kv_copy ? (uint64_t)a.D * 2 : (uint64_t)v->nb[1];
    const uint64_t rpitch = f.table_bytes ? (uint64_t)a.D * 2 : (uint64_t)r->nb[1];
    if ((uint64_t)a.Nkv * kpitch >= lim || (uint64_t)a.Nkv * vpitch >= lim || (uint64_t)r->ne[1] * rpitch >= lim) return f;
    // A workgroup of the one-kernel form walks all keys of its head by itself.  A single long utterance leaves most CUs
    // without one, and then the mask kernel + the tile kernel - which cuts the keys of a small grid into ranges - is
    // ahead: 8 heads x 128, one sequence of 750 frames (48 workgroups) 54.4 against 45.8 us, 4 heads 51.9 against 38.1,
    // 1500 frames 90 against 80; up to 375 frames and from 8 sequences on the one kernel wins everywhere (60 against 67 us
    // at 4 heads x 750 frames x 8, 21 against 26 at 100 frames).
    static const bool one_kernel = getenv("MI355X_RELPOS_ONE_KERNEL") != nullptr;     // comparison runs
    const int64_t wgs = (int64_t)((a.Nq + 127) / 128) * a.Hq * a.B;
    if (!one_kernel && wgs * 8 <= 3 * (int64_t)device_cus() && a.Nkv >= 512) return f;
    f.ok = true;
    return f;
}

static int relpos_fused_run(const mi355x_tensor * q_u, const mi355x_tensor * q_v, const mi355x_tensor * k,
                            const mi355x_tensor * v, const mi355x_tensor * r, const mi355x_tensor * add,
                            const mi355x_tensor * dst, const mi355x_fattn_params * params, const RelposFused & f,
                            void * ws, hipStream_t st) {
    FattnArgs a;
    fill_args(a, q_u, k, v, nullptr, (float *)dst->data, params);
    if (!q_v->data || !r->data) return fail(MI355X_ERR_INVALID, "null data pointer");
    // an F32 table with aligned rows is rounded by the launch that rounds K and V
    bool table_done = false;
    if (f.kv_copy) {
        F32Rider x;
        memset(&x, 0, sizeof(x));
        if (f.table_bytes && r->type == MI355X_TYPE_F32 && aligned16_view(r) && k->type == v->type) {
            x.src = (const char *)r->data;
            x.dst = (char *)ws + f.kv_bytes;
            x.ne1 = r->ne[1]; x.ne2 = r->ne[2];
            x.nb1 = (int64_t)r->nb[1]; x.nb2 = (int64_t)r->nb[2]; x.nb3 = (int64_t)r->nb[3];
            x.n   = (int64_t)(a.D / 8) * r->ne[1] * r->ne[2] * r->ne[3];
            table_done = true;
        }
        const int e = kv_to_f16_launch(a, k->type, v->type, ws, st, table_done ? &x : nullptr);
        if (e) return hip_fail((hipError_t)e, "K/V conversion launch");
        use_f16_copies(a, ws);
    }
    FattnRelposArgs g;
    memset(&g, 0, sizeof(g));
    g.qu = a.q; g.nbu1 = a.nbq1; g.nbu2 = a.nbq2; g.nbu3 = a.nbq3;
    g.qv = (const char *)q_v->data; g.nbw1 = (int64_t)q_v->nb[1]; g.nbw2 = (int64_t)q_v->nb[2]; g.nbw3 = (int64_t)q_v->nb[3];
    g.k = a.k; g.nbk1 = a.nbk1; g.nbk2 = a.nbk2; g.nbk3 = a.nbk3;
    g.v = a.v; g.nbv1 = a.nbv1; g.nbv2 = a.nbv2; g.nbv3 = a.nbv3;
    g.r = (const char *)r->data; g.nbr1 = (int64_t)r->nb[1]; g.nbr2 = (int64_t)r->nb[2]; g.nbr3 = (int64_t)r->nb[3];
    g.Hr = (int)r->ne[2]; g.Br = (int)r->ne[3];
    if (f.table_bytes) {
        char * r16 = (char *)ws + f.kv_bytes;
        if (!table_done) {
            CpyArgs c;
            memset(&c, 0, sizeof(c));
            c.src = (const char *)r->data;
            c.dst = r16;
            int64_t nb = 2;
            c.n = 1;
            for (int i = 0; i < 4; i++) {
                c.sne[i] = c.dne[i] = r->ne[i];
                c.snb[i] = (int64_t)r->nb[i];
                c.dnb[i] = nb;
                nb *= r->ne[i];
                c.n *= r->ne[i];
            }
            const int e = cpy_launch(c, r->type, MI355X_TYPE_F16, st);
            if (e) return hip_fail((hipError_t)e, "table conversion launch");
        }
        g.r = r16;
        g.nbr1 = (int64_t)a.D * 2; g.nbr2 = g.nbr1 * r->ne[1]; g.nbr3 = g.nbr2 * r->ne[2];
    }
    g.Ha = g.Ba = 1;
    if (add && add->ne[0] > 0) {
        if (!add->data) return fail(MI355X_ERR_INVALID, "null data pointer");
        g.add = (const char *)add->data; g.nba1 = (int64_t)add->nb[1]; g.nba2 = (int64_t)add->nb[2]; g.nba3 = (int64_t)add->nb[3];
        g.Ha = (int)add->ne[2]; g.Ba = (int)add->ne[3];
        g.add_f16 = add->type == MI355X_TYPE_F16;
    }
    mirror_note_host_write(dst);
    g.dst = (float *)dst->data;
    g.D = a.D; g.Nq = a.Nq; g.Nkv = a.Nkv; g.H = a.Hq; g.B = a.B; g.gqa = a.gqa; g.bq = a.bq;
    g.scale = params->scale;
    g.n_cus = a.n_cus;
    if (!fattn_relpos_supported(g)) return fail(MI355X_ERR_UNSUPPORTED, "shape not covered by the one-kernel form");
    const int e = fattn_relpos_launch(g, st);
    if (e) return hip_fail((hipError_t)e, "relative-position attention launch");
    return MI355X_OK;
}

int mi355x_fattn_relpos_workspace_size(const mi355x_tensor * q_u, const mi355x_tensor * q_v, const mi355x_tensor * k,
                                       const mi355x_tensor * v, const mi355x_tensor * r, const mi355x_tensor * add,
                                       const mi355x_fattn_params * params, size_t * bytes) {
    if (!bytes) return fail(MI355X_ERR_INVALID, "null argument");
    mi355x_tensor m;
    size_t mb = 0, ib = 0;
    const int rc = relpos_fused_check(q_u, q_v, k, v, r, add, nullptr, params, &m, &mb, &ib);
    if (rc) return rc;
    // Which form a call takes depends on the alignment of its data pointers, and a size query may come before those exist
    // (NULL looks aligned): the answer covers both forms, so that a workspace of this size never turns out too small.
    const RelposFused f = relpos_fused_plan(q_u, q_v, k, v, r, add, params);
    const size_t one = f.kv_bytes + f.table_bytes, two = mb + ib;
    *bytes = f.ok && one > two ? one : two;
    return MI355X_OK;
}

int mi355x_flash_attn_relpos(const mi355x_tensor * q_u, const mi355x_tensor * q_v, const mi355x_tensor * k,
                             const mi355x_tensor * v, const mi355x_tensor * r, const mi355x_tensor * add,
                             const mi355x_tensor * dst, const mi355x_fattn_params * params, void * stream) {
    if (!dst) return fail(MI355X_ERR_INVALID, "null dst");
    mi355x_tensor m;
    size_t mb = 0, ib = 0;
    int rc = relpos_fused_check(q_u, q_v, k, v, r, add, dst, params, &m, &mb, &ib);
    if (rc) return rc;
    if ((int64_t)q_u->ne[1] * q_u->ne[2] * q_u->ne[3] == 0) return MI355X_OK;
    const RelposFused f = relpos_fused_plan(q_u, q_v, k, v, r, add, params);
    if (f.ok) {
        if (!q_u->data || !k->data || !v->data || !dst->data) return fail(MI355X_ERR_INVALID, "null data pointer");
        const size_t need = f.kv_bytes + f.table_bytes;
        void * ws = params->workspace;
        if (need) {
            if (ws) {
                if (params->workspace_size < need) return fail(MI355X_ERR_WORKSPACE, "workspace %zu < %zu bytes", params->workspace_size, need);
                if ((uintptr_t)ws % 16) return fail(MI355X_ERR_WORKSPACE, "workspace must be 16-byte aligned");
            } else {
                rc = get_scratch(need, &ws, (hipStream_t)stream);
                if (rc) return rc;
            }
        }
        return relpos_fused_run(q_u, q_v, k, v, r, add, dst, params, f, ws, (hipStream_t)stream);
    }
    void * ws = params->workspace;
    if (ws) {
        if (params->workspace_size < mb + ib)
            return fail(MI355X_ERR_WORKSPACE, "workspace %zu < %zu bytes", params->workspace_size, mb + ib);
        if ((uintptr_t)ws % 16) return fail(MI355X_ERR_WORKSPACE, "workspace must be 16-byte aligned");
    } else {
        rc = get_scratch(mb + ib, &ws, (hipStream_t)stream);
        if (rc) return rc;
    }
    m.data = ws;
    rc = relpos_run(q_v, r, add, &m, params->scale, (char *)ws + mb - relpos_table_bytes(r), (hipStream_t)stream);
    if (rc) return rc;
    mi355x_fattn_params inner = *params;
    inner.workspace      = ib ? (char *)ws + mb : nullptr;      // never the library scratch again: the mask lives there
    inner.workspace_size = ib;
    return mi355x_flash_attn_ext(q_u, k, v, &m, dst, &inner, stream);
}

int mi355x_cpy_supports(const mi355x_tensor * src, const mi355x_tensor * dst) { return cpy_check(src, dst); }

int mi355x_cpy(const mi355x_tensor * src, const mi355x_tensor * dst, void * stream) {
    const int rc = cpy_check(src, dst);
    if (rc) return rc;
    CpyArgs a;
    memset(&a, 0, sizeof(a));
    a.src = (const char *)src->data;
    a.dst = (char *)dst->data;
    int64_t n = 1;
    for (int i = 0; i < 4; i++) {
        a.sne[i] = src->ne[i]; a.dne[i] = dst->ne[i];
        a.snb[i] = (int64_t)src->nb[i]; a.dnb[i] = (int64_t)dst->nb[i];
        n *= src->ne[i];
    }
    const bool blocks = FATTN_IS_BLOCK_TYPE(src->type) || FATTN_IS_BLOCK_TYPE(dst->type);
    a.n = blocks ? n / FATTN_QK8_0 : n;
    if (a.n == 0) return MI355X_OK;
    if (!a.src || !a.dst) return fail(MI355X_ERR_INVALID, "null data pointer");
    if (a.n > ((int64_t)1 << 38)) return fail(MI355X_ERR_UNSUPPORTED, "copy too large");
    const int rm = mirror_for_write(dst, (hipStream_t)stream, &a.mirror);
    if (rm) return rm;
    {   // a source inside a mirrored buffer (ggml_cont of a cache slice, src/core/attention.h:919-920) is read from HBM
        void * sdata = nullptr;
        const int rs = mirror_for_read(src, (hipStream_t)stream, &sdata);
        if (rs) return rs;
        a.src = (const char *)sdata;
    }
    const int e = cpy_launch(a, src->type, dst->type, (hipStream_t)stream);
    if (e) return hip_fail((hipError_t)e, "cpy launch");
    return MI355X_OK;
}

int mi355x_set_rows_supports(const mi355x_tensor * src, int32_t idx_type, const int64_t idx_ne[3], const mi355x_tensor * dst) {
    if (!src || !dst || !idx_ne) return fail(MI355X_ERR_INVALID, "null argument");
    if (!sane_extents(src, nullptr) || !sane_extents(dst, nullptr)) return fail(MI355X_ERR_INVALID, "negative or oversized extent");
    if (src->type != MI355X_TYPE_F32) return fail(MI355X_ERR_UNSUPPORTED, "set_rows source must be F32");
    if (!type_size(dst->type)) return fail(MI355X_ERR_UNSUPPORTED, "set_rows destination type %d", dst->type);
    if (idx_type != 64 && idx_type != 32) return fail(MI355X_ERR_INVALID, "index type must be 32 or 64");
    if (src->ne[0] != dst->ne[0] || src->ne[2] != dst->ne[2] || src->ne[3] != dst->ne[3])
        return fail(MI355X_ERR_INVALID, "set_rows shapes do not match");
    if (idx_ne[0] != src->ne[1] || idx_ne[1] <= 0 || idx_ne[2] <= 0 || src->ne[2] % idx_ne[1] || src->ne[3] % idx_ne[2])
        return fail(MI355X_ERR_INVALID, "set_rows index shape does not match");
    if (src->nb[0] % 4) return fail(MI355X_ERR_UNSUPPORTED, "misaligned strides");
    if (dst->nb[0] != type_size(dst->type)) return fail(MI355X_ERR_UNSUPPORTED, "dst rows must be contiguous");
    if (block_size(dst->type) > 1 && src->ne[0] % block_size(dst->type)) return fail(MI355X_ERR_INVALID, "quantised rows need ne0 %% 32 == 0");
    const size_t dal = dst->type == MI355X_TYPE_F32 ? 4 : 2;
    if ((uintptr_t)src->data % 4 || (uintptr_t)dst->data % dal) return fail(MI355X_ERR_UNSUPPORTED, "misaligned data pointers");
    for (int i = 1; i < 4; i++)
        if (src->nb[i] % 4 || dst->nb[i] % dal) return fail(MI355X_ERR_UNSUPPORTED, "misaligned strides");
    return MI355X_OK;
}

int mi355x_set_rows(const mi355x_tensor * src, const void * idx, int32_t idx_type,
                    const int64_t idx_ne[3], const size_t idx_nb[3],
                    const mi355x_tensor * dst, void * stream) {
    if (!idx_nb) return fail(MI355X_ERR_INVALID, "null argument");
    const int rc = mi355x_set_rows_supports(src, idx_type, idx_ne, dst);
    if (rc) return rc;
    CpyArgs a;
    memset(&a, 0, sizeof(a));
    a.src = (const char *)src->data;
    a.dst = (char *)dst->data;
    a.idx = (const char *)idx;
    a.idx_is_i64 = idx_type == 64;
    int64_t n = 1;
    for (int i = 0; i < 4; i++) {
        a.sne[i] = src->ne[i]; a.dne[i] = dst->ne[i];
        a.snb[i] = (int64_t)src->nb[i]; a.dnb[i] = (int64_t)dst->nb[i];
        n *= src->ne[i];
    }
    for (int i = 0; i < 3; i++) { a.ine[i] = idx_ne[i]; a.inb[i] = (int64_t)idx_nb[i]; }
    a.n = FATTN_IS_BLOCK_TYPE(dst->type) ? n / FATTN_QK8_0 : n;
    if (a.n == 0) return MI355X_OK;
    if (!a.src || !a.dst || !a.idx) return fail(MI355X_ERR_INVALID, "null data pointer");
    const int rm = mirror_for_write(dst, (hipStream_t)stream, &a.mirror);
    if (rm) return rm;
    const int e = set_rows_launch(a, dst->type, (hipStream_t)stream);
    if (e) return hip_fail((hipError_t)e, "set_rows launch");
    return MI355X_OK;
}

// ---- buffers -----------------------------------------------------------------------------

int mi355x_buffer_alloc(size_t size, void ** ptr) {
    if (!ptr) return fail(MI355X_ERR_INVALID, "null argument");
    *ptr = nullptr;
    HIP_TRY(hipMalloc(ptr, size ? size : 1));
    return MI355X_OK;
}

int mi355x_buffer_free(void * ptr) {
    if (ptr) HIP_TRY(hipFree(ptr));
    return MI355X_OK;
}

int mi355x_host_buffer_alloc(size_t size, void ** ptr) {
    if (!ptr) return fail(MI355X_ERR_INVALID, "null argument");
    *ptr = nullptr;
    HIP_TRY(hipHostMalloc(ptr, size ? size : 1, hipHostMallocMapped | hipHostMallocCoherent));
    HostBuf * b = new HostBuf();
    b->base = (char *)*ptr;
    b->size = size ? size : 1;
    std::lock_guard<std::mutex> lk(g_mu);
    g_hostbufs.push_back(b);
    return MI355X_OK;
}

int mi355x_host_buffer_free(void * ptr) {
    if (!ptr) return MI355X_OK;
    HostBuf * b = nullptr;
    {
        std::lock_guard<std::mutex> lk(g_mu);
        for (size_t i = 0; i < g_hostbufs.size(); i++)
            if (g_hostbufs[i]->base == (char *)ptr) {
                b = g_hostbufs[i];
                g_hostbufs.erase(g_hostbufs.begin() + i);
                break;
            }
    }
    if (b) {
        if (b->mirror) HIP_TRY(hipFree(b->mirror));
        delete b;
    }
    HIP_TRY(hipHostFree(ptr));
    return MI355X_OK;
}

int mi355x_host_buffer_mirror_stats(const void * ptr, size_t * mirror_bytes, size_t * valid_bytes, size_t * uploaded_bytes) {
    std::lock_guard<std::mutex> lk(g_mu);
    HostBuf * b = hostbuf_of(ptr, 1);
    if (!b) return fail(MI355X_ERR_INVALID, "not inside a buffer of mi355x_host_buffer_alloc");
    size_t valid = 0;
    for (size_t p = 0; p < b->valid.size(); p++)
        if (b->valid[p]) valid += (p + 1) * MIRROR_PAGE <= b->size ? MIRROR_PAGE : b->size - p * MIRROR_PAGE;
    if (mirror_bytes)   *mirror_bytes   = b->mirror ? b->size : 0;
    if (valid_bytes)    *valid_bytes    = valid;
    if (uploaded_bytes) *uploaded_bytes = b->uploaded;
    return MI355X_OK;
}

int mi355x_host_buffer_invalidate(void * ptr, size_t size) {
    if (size == 0) return MI355X_OK;
    std::lock_guard<std::mutex> lk(g_mu);
    HostBuf * b = hostbuf_of(ptr, size);
    if (!b) return fail(MI355X_ERR_INVALID, "not inside a buffer of mi355x_host_buffer_alloc");
    if (!b->mirror) return MI355X_OK;
    const size_t off = (size_t)((char *)ptr - b->base);
    for (size_t p = off / MIRROR_PAGE; p < (off + size + MIRROR_PAGE - 1) / MIRROR_PAGE; p++) b->valid[p] = 0;
    return MI355X_OK;
}

// The place of [ptr, ptr + size) in the mirror of the host buffer that holds it, if that buffer has one (g_mu held).  The
// callers below write the same bytes to both copies: a page they cover only in part keeps its state - up to date stays up
// to date, stale stays stale and is fetched whole from the host copy when it is next needed.
static int mirror_of_range(void * ptr, size_t size, hipStream_t st, HostBuf ** buf, char ** mirror) {
    *buf = nullptr;
    *mirror = nullptr;
    if (g_no_mirror) return MI355X_OK;
    HostBuf * b = hostbuf_of(ptr, size);
    if (!b || !b->mirror) return MI355X_OK;
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(st, &cs) != hipSuccess) (void)hipGetLastError();
    const size_t off = (size_t)((char *)ptr - b->base);
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess) (void)hipGetLastError();
    // replays would bypass the bookkeeping, and a call made with another GPU current must not touch this one's memory:
    // host copy only, pages stale
    if (cs != hipStreamCaptureStatusNone || dev != b->dev) {
        for (size_t p = off / MIRROR_PAGE; p < (off + size + MIRROR_PAGE - 1) / MIRROR_PAGE; p++) b->valid[p] = 0;
        return MI355X_OK;
    }
    *buf = b;
    *mirror = b->mirror + off;
    return MI355X_OK;
}

int mi355x_buffer_memset(void * ptr, int value, size_t size, void * stream) {
    if (size == 0) return MI355X_OK;
    if (!ptr) return fail(MI355X_ERR_INVALID, "null argument");
    // a fill kernel, not hipMemsetAsync: safe to record into a graph the caller captures
    int e = fill_launch(ptr, value, size, (hipStream_t)stream);
    if (e) return hip_fail((hipError_t)e, "fill launch");
    std::lock_guard<std::mutex> lk(g_mu);
    HostBuf * b; char * m;
    const int rc = mirror_of_range(ptr, size, (hipStream_t)stream, &b, &m);
    if (rc || !m) return rc;
    e = fill_launch(m, value, size, (hipStream_t)stream);
    if (e) return hip_fail((hipError_t)e, "fill launch");
    mirror_mark_written(b, (size_t)((char *)ptr - b->base), size);      // (pages covered in part keep their state: both copies got the same bytes)
    return MI355X_OK;
}

// The copies below name no direction: a buffer is HBM or pinned host memory and the runtime tells them apart by address.
int mi355x_buffer_set(void * dst, const void * host_src, size_t size, void * stream) {
    if (size == 0) return MI355X_OK;
    if (!dst || !host_src) return fail(MI355X_ERR_INVALID, "null argument");
    HIP_TRY(hipMemcpyAsync(dst, host_src, size, hipMemcpyDefault, (hipStream_t)stream));
    {
        std::lock_guard<std::mutex> lk(g_mu);
        HostBuf * b; char * m;
        const int rc = mirror_of_range(dst, size, (hipStream_t)stream, &b, &m);
        if (rc) return rc;
        if (m) {
            HIP_TRY(hipMemcpyAsync(m, host_src, size, hipMemcpyDefault, (hipStream_t)stream));
            mirror_mark_written(b, (size_t)((char *)dst - b->base), size);
        }
    }
    HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
    return MI355X_OK;
}

int mi355x_buffer_get(void * host_dst, const void * src, size_t size, void * stream) {
    if (size == 0) return MI355X_OK;
    if (!host_dst || !src) return fail(MI355X_ERR_INVALID, "null argument");
    HIP_TRY(hipMemcpyAsync(host_dst, src, size, hipMemcpyDefault, (hipStream_t)stream));
    HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
    return MI355X_OK;
}

int mi355x_buffer_copy(void * dst, const void * src, size_t size, void * stream) {
    if (size == 0) return MI355X_OK;
    if (!dst || !src) return fail(MI355X_ERR_INVALID, "null argument");
    HIP_TRY(hipMemcpyAsync(dst, src, size, hipMemcpyDefault, (hipStream_t)stream));
    std::lock_guard<std::mutex> lk(g_mu);
    HostBuf * b; char * m;
    const int rc = mirror_of_range(dst, size, (hipStream_t)stream, &b, &m);
    if (rc || !m) return rc;
    // from the source's own mirror where that is up to date (a cache snapshot then never leaves HBM), else from the source
    const void * from = src;
    HostBuf * sb = hostbuf_of(src, size);
    if (sb && sb->mirror) {
        const size_t so = (size_t)((const char *)src - sb->base);
        bool ok = true;
        for (size_t p = so / MIRROR_PAGE; p < (so + size + MIRROR_PAGE - 1) / MIRROR_PAGE; p++) ok = ok && sb->valid[p];
        if (ok) from = sb->mirror + so;
    }
    HIP_TRY(hipMemcpyAsync(m, from, size, hipMemcpyDefault, (hipStream_t)stream));
    mirror_mark_written(b, (size_t)((char *)dst - b->base), size);
    return MI355X_OK;
}

}  // extern "C"
