/*
 * mi355x_fattn.h - C ABI of the MI355X (gfx950) attention library.
 *
 * This is the launcher layer a ggml backend ("ggml-mi355x") binds for
 * GGML_OP_FLASH_ATTN_EXT and for the tensor copies that op needs.  Plain pointers,
 * sizes and scalars only: no ggml, HIP or torch types cross this boundary.  All data
 * pointers are device pointers (hipMalloc / hipMallocManaged / hipHostMalloc-mapped
 * memory the GPU can address); `stream` is a hipStream_t passed as void* (NULL = the
 * default stream).  Calls are asynchronous on `stream` unless stated otherwise.
 *
 * Every entry point returns an mi355x_status; on a non-zero status
 * mi355x_last_error() holds a message for the calling thread.
 *
 * Reference interfaces replaced (paths relative to the CrispASR tree):
 *   - the op node built by ggml_flash_attn_ext(ctx, q, k, v, mask, scale, max_bias,
 *     logit_softcap) at src/crispasr.cpp:2821, :3220, :3280, src/core/attention.h:992,
 *     src/core/fastconformer.h:924-934, src/core/cross_attn.h:119-153, src/canary.cpp:966-972
 *     and executed by whichever backend ggml_backend_sched assigned
 *     (src/crispasr.cpp:256-280 -> ggml_backend_sched_graph_compute);
 *   - the KV-cache writes ggml_cpy(F32 -> cache view) at src/crispasr.cpp:2810-2811,
 *     3185-3203, 2956-2973 and src/core/attention.h:342-378;
 *   - the buffer vtable a backend fills (member order pinned by the reference's own
 *     initialiser, src/core/gguf_loader.cpp:332-344): memset_tensor / set_tensor /
 *     get_tensor / cpy_tensor / clear.
 */
#ifndef MI355X_FATTN_H
#define MI355X_FATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MI355X_FATTN_API_VERSION 6

/* ggml type ids of the storage types this path meets */
enum mi355x_type {
    MI355X_TYPE_F32  = 0,
    MI355X_TYPE_F16  = 1,
    /* the block-32 cache types CRISPASR_KV_QUANT can name (src/core/attention.h:79-105).  Element j < 16 of a block is the
     * low nibble of qs[j], element j + 16 the high nibble; qh holds the fifth bit of element e in bit e (little-endian).
     * ggml itself is not part of the reference's tree: the four narrow layouts and their scalar quantisers are ggml's as
     * recalled (scale from the signed value of largest magnitude, q = min(15, trunc(x/d + 8.5)) and siblings). */
    MI355X_TYPE_Q4_0 = 2,  /* fp16 d, qs[16]: 18 bytes, x = (q - 8) * d */
    MI355X_TYPE_Q4_1 = 3,  /* fp16 d, fp16 m, qs[16]: 20 bytes, x = q * d + m */
    MI355X_TYPE_Q5_0 = 6,  /* fp16 d, qh[4], qs[16]: 22 bytes, x = (q - 16) * d */
    MI355X_TYPE_Q5_1 = 7,  /* fp16 d, fp16 m, qh[4], qs[16]: 24 bytes, x = q * d + m */
    MI355X_TYPE_Q8_0 = 8   /* fp16 scale d + 32 x int8, 34 bytes, x = q*d */
};

enum mi355x_status {
    MI355X_OK              = 0,
    MI355X_ERR_UNSUPPORTED = 1,   /* valid op, but outside what these kernels cover: route to CPU */
    MI355X_ERR_INVALID     = 2,   /* breaks the op's contract (ggml would assert) */
    MI355X_ERR_HIP         = 3,   /* a HIP runtime call failed */
    MI355X_ERR_NO_DEVICE   = 4,
    MI355X_ERR_WORKSPACE   = 5    /* caller-provided workspace too small */
};

/* The fields of ggml_tensor the kernels read: data, type, ne (elements per dimension,
 * dimension 0 fastest), nb (byte strides; nb[0] is the element - or block - size). */
typedef struct mi355x_tensor {
    void *  data;
    int32_t type;
    int64_t ne[4];
    size_t  nb[4];
} mi355x_tensor;

enum mi355x_fattn_kernel {
    MI355X_FATTN_AUTO       = 0,
    MI355X_FATTN_VEC        = 1,  /* split-KV vector kernel: any supported shape */
    MI355X_FATTN_MMA        = 2,  /* f16 MFMA tile kernel: prefill / encoder shapes */
    MI355X_FATTN_DECODE_MMA = 3   /* split-KV MFMA kernel: the query rows of a KV head 16 at a time (decode steps, short prompts) */
};

/* op_params of the node (scale, max_bias, logit_softcap as f32, prec as i32) plus
 * launch overrides used by the tests and the benchmark. */
typedef struct mi355x_fattn_params {
    float   scale;
    float   max_bias;
    float   logit_softcap;
    int32_t prec;            /* GGML_PREC_DEFAULT = 0, GGML_PREC_F32 = 10; accumulation is f32 either way */
    int32_t kernel;          /* mi355x_fattn_kernel */
    int32_t n_splits;        /* 0 = choose; forces the KV split count of the split-KV kernels */
    void *  workspace;       /* NULL = library-owned scratch: one block per device, grown with hipMalloc when needed and
                              * shared by every call that passes NULL, so such calls (and replays of graphs that recorded
                              * them) belong on one stream at a time; while its stream is capturing, a call that would
                              * have to grow the block is refused with MI355X_ERR_WORKSPACE instead.  (Such a call of the
                              * split-KV decode or vector kernel also merges its partial results inside the kernel - the last workgroup
                              * to finish a set of key ranges does it - where a call on a caller's workspace, which may overlap
                              * others, uses a second launch: same arithmetic, same bits.)
                              * Else 16-byte aligned.  With a caller's workspace of mi355x_fattn_workspace_size bytes the call allocates nothing
                              * and launches kernels only (no memset or copy nodes): it may be recorded into a HIP graph. */
    size_t  workspace_size;
    int32_t q_quant;         /* 0 = the query rows as they are.  MI355X_TYPE_Q8_0 = round every query row to Q8_0 blocks first
                              * (d = amax/127 per 32 values), which is what ggml-cpu is recalled to do when K is Q8_0 (the
                              * vec_dot_type of Q8_0 is Q8_0): a comparison mode for runs against ggml-cpu, two small extra
                              * launches and D % 32 == 0; never needed for correctness. */
    int32_t tile_variant;    /* 0 = choose.  Else 16 * key_split + query_blocks (see mi355x_fattn_plan_info) forces that
                              * instantiation of the tile kernel where it exists (tests, tuning); otherwise ignored. */
} mi355x_fattn_params;

typedef struct mi355x_device_info {
    char     name[128];
    char     arch[32];           /* gcnArchName, e.g. "gfx950:sramecc+:xnack-" */
    int32_t  compute_units;
    int32_t  clock_khz;
    int32_t  memory_clock_khz;
    int32_t  memory_bus_bits;
    uint64_t total_memory;
    uint64_t free_memory;
    int32_t  lds_bytes_per_block;
    int32_t  wavefront_size;
} mi355x_device_info;

/* ---- library / device ---------------------------------------------------------------- */

int          mi355x_api_version(void);
const char * mi355x_status_string(int status);
const char * mi355x_last_error(void);

/* ggml_backend_reg_i::get_device_count / ggml_backend_device_i::get_props, get_memory */
int mi355x_device_count(int * count);
int mi355x_device_get_info(int device, mi355x_device_info * info);
int mi355x_set_device(int device);
/* ggml_backend_i::synchronize */
int mi355x_stream_synchronize(void * stream);

/* ---- GGML_OP_FLASH_ATTN_EXT ------------------------------------------------------------ */

/*
 * dst[DV, Hq, Nq, B] (f32, contiguous, 16-byte aligned) = softmax(scale * q.k^T [soft-capped] + slope(h) * mask) . v
 *
 *   q    F32  [D,  Nq,  Hq,  B ]   any strides with nb[0] == 4
 *   k    F16 | F32 | Q8_0 | Q4_0 | Q4_1 | Q5_0 | Q5_1 [D,  Nkv, Hkv, Bk]   rows contiguous (nb[0] == type size)
 *   v    any of k's types [DV, Nkv, Hkv, Bk]   DV == D.  A V of another type than K's (CRISPASR_KV_QUANT_K / _V,
 *        src/core/attention.h:132-137) costs one conversion of both to f16 copies in the workspace before the kernel.
 *        (Q4_0 .. Q5_1: up to 16 query rows per KV head read the blocks in the decode kernel (head sizes 64 and 128, no
 *         soft cap; other shapes in the vector kernel); more rows go through one conversion of K and V to f16 in the
 *         workspace and the tile kernel)
 *   mask NULL, or F16 [>=Nkv, >=Nq, Hm, Bm], rows contiguous; head h reads h % Hm,
 *        batch b reads b % Bm; -inf entries exclude the key
 *   Hq % Hkv == 0 (query head h reads KV head h / (Hq/Hkv)), B % Bk == 0.
 *   D: a multiple of 4 up to 256.  64 and 128 run on the MFMA kernels.  So do the other multiples of 8 below 128 (32, 48,
 *   80, 96 ...; mi355x_fattn_plan_info.head_pad; the result is that of the head size itself): decode-shaped calls over
 *   F16 caches on the decode kernel, which reads the rows where they lie and fills a row's registers behind the head's
 *   own elements with zeros; calls with 16 queries or more and 100000 (query row, key) pairs or more on the tile kernel, on
 *   f16 copies of K and V in the workspace whose rows are zero-padded to 64 or 128.  Smaller calls of those sizes, few
 *   query rows over F32 or quantised caches, larger multiples of 8 and - with F16 or F32 K/V of one type - multiples of 4
 *   such as the 36 and 52 of src/core/cross_attn.h:119-153's smaller callers run on the vector kernel.
 *   A row whose keys are all excluded (or Nkv == 0) yields zeros.
 *   An excluded key contributes nothing whatever its K/V bytes are - NaN, inf, a Q8_0 block whose scale is NaN - as in
 *   ggml-cpu, which skips it: cache slots that were never written may be masked out instead of cleared
 *   (src/core/attention.h:680-683).  (The MFMA kernels multiply such a key by a probability of exactly zero, look at each
 *   row's result before storing it, and compute a row that came out non-finite again with the excluded keys unread.)
 *
 * mi355x_fattn_supports is the predicate the backend's supports_op mirrors: it returns
 * MI355X_OK, MI355X_ERR_UNSUPPORTED or MI355X_ERR_INVALID without touching the device.
 * Data pointers are never dereferenced there: they may be NULL (graph planning happens before allocation), or carry
 * just the low bits the address will have (say offset-into-buffer modulo 256 for buffers that start on 256 bytes), so
 * that a view whose address would fail the alignment rules above at launch is answered MI355X_ERR_UNSUPPORTED at
 * planning already (the strides are always checked).  The same holds for the other *_supports predicates.
 */
int mi355x_fattn_supports(const mi355x_tensor * q, const mi355x_tensor * k, const mi355x_tensor * v,
                          const mi355x_tensor * mask, const mi355x_tensor * dst,
                          const mi355x_fattn_params * params);

int mi355x_flash_attn_ext(const mi355x_tensor * q, const mi355x_tensor * k, const mi355x_tensor * v,
                          const mi355x_tensor * mask, const mi355x_tensor * dst,
                          const mi355x_fattn_params * params, void * stream);

/*
 * The same call for callers that cannot allocate (code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc).  No counterpart in the reference: ggml backends allocate their pools as they go.
 * Whatever scratch the kernels need (split-KV partials, f16 copies of F32 / Q8_0 K and V, the q_quant staging) is taken
 * from a static device array of MI355X_NOALLOC_SCRATCH_BYTES that is part of the library's image on every GPU it is
 * loaded on; params->workspace and workspace_size are ignored.  The call itself never calls hipMalloc, hipFree or any
 * allocating routine and launches kernels only; a call that would need more scratch than the array holds returns
 * MI355X_ERR_WORKSPACE and launches nothing (mi355x_fattn_workspace_size tells beforehand).
 * All calls on one GPU share that GPU's array: calls that overlap in time on one GPU (two streams, two threads) race -
 * serialise them, or give the overlapping ones their own workspace through mi355x_flash_attn_ext.  Nothing in the array
 * has to start at zero: every byte a call reads has been written by that call's own kernels before.  (Split-KV
 * calls that merge inside the kernel count their workgroups in a second static array, 128 KiB of counters per GPU that
 * starts at zero when the library is loaded and that every launch leaves at zero; this entry point and the calls on the
 * library's scratch block use separate halves of it.)
 * The array's address is looked up once per device, on the first call there (or in mi355x_set_device).
 */
#define MI355X_NOALLOC_SCRATCH_BYTES (32u << 20)
int mi355x_flash_attn_ext_noalloc(const mi355x_tensor * q, const mi355x_tensor * k, const mi355x_tensor * v,
                                  const mi355x_tensor * mask, const mi355x_tensor * dst,
                                  const mi355x_fattn_params * params, void * stream);

/* bytes of scratch the call above would use with these shapes (0 when none) */
int mi355x_fattn_workspace_size(const mi355x_tensor * q, const mi355x_tensor * k, const mi355x_tensor * v,
                                const mi355x_tensor * mask, const mi355x_fattn_params * params,
                                size_t * bytes);

/* which kernel and split count AUTO resolves to (for logs, tests and the benchmark) */
int mi355x_fattn_plan(const mi355x_tensor * q, const mi355x_tensor * k, const mi355x_tensor * v,
                      const mi355x_tensor * mask, const mi355x_fattn_params * params,
                      int32_t * kernel, int32_t * n_splits);

/* The same, with the instantiation of the tile kernel the call takes: tests assert on it that a shape reaches the kernel
 * it is meant to reach, the benchmark names the kernel it times.  (The variant depends on the mask's address too: plan
 * with the data pointers the call will have.) */
typedef struct mi355x_fattn_plan_info {
    int32_t kernel;                  /* mi355x_fattn_kernel */
    int32_t n_splits;
    int32_t keys_per_split;
    int32_t kv_to_f16;               /* 1: F32 / quantised K and V are rounded to f16 copies in the workspace first */
    size_t  workspace;               /* bytes, as mi355x_fattn_workspace_size reports (without the q_quant part) */
    /* tile kernel only (0 otherwise) */
    int32_t queries_per_workgroup;   /* 256, 128 or 64 */
    int32_t query_blocks;            /* 32-query blocks per wave: 1 or 2 */
    int32_t key_split;               /* 2: the waves of a workgroup pair up over the two halves of every 64-key tile */
    int32_t direct;                  /* K/V tiles move global -> LDS without passing registers */
    int32_t mask_dma;                /* the mask takes the same road */
    int32_t merge_in_kernel;         /* 1: the split-KV partials are merged by the last workgroup to finish each set of ranges (no
                                      * merge launch): calls on the library's scratch (params->workspace == NULL); the
                                      * allocation-free entry point does the same for the same shapes */
    int32_t head_pad;                /* 0, or 64 / 128: the head size is neither, and the kernel runs the form for this size - the
                                      * tile kernel on f16 copies of K and V whose rows are zero-padded to it (kv_to_f16 is 1), the
                                      * decode kernel on the F16 rows themselves (kv_to_f16 is 0) */
} mi355x_fattn_plan_info;
int mi355x_fattn_plan_details(const mi355x_tensor * q, const mi355x_tensor * k, const mi355x_tensor * v,
                              const mi355x_tensor * mask, const mi355x_fattn_params * params,
                              mi355x_fattn_plan_info * info);

/* ---- FastConformer relative-position attention (src/core/fastconformer.h:876-935) ---------- */

/*
 * The mask that core_conformer::build_block computes for its flash_attn_ext call, as one launch:
 *
 *   dst[j, i, h, b] = f16( scale * <q_v[:, i, h, b], r[:, Nq-1+j-i, h % Hr, b % Br]>  +  add[j, i, h % Ha, b % Ba] )
 *
 * It replaces the graph nodes  mul_mat(cont(R), Q_v) -> rel_shift view (fastconformer.h:98-102) -> cont -> scale
 * -> add(local_attn_mask) -> cast F16  (fastconformer.h:880-895, 918); dst is the BD_mask tensor of that graph.
 *
 *   q_v  F32 [D, Nq, H, B]            nb[0] == 4, base and strides multiples of 16 bytes; D = 64 or 128
 *   r    F32 | F16 [D, Nq+Nkv-1, Hr, Br]   rows contiguous and 16-byte aligned; H % Hr == 0, B % Br == 0
 *   add  NULL, or F32 | F16 [>=Nkv, >=Nq, Ha, Ba]  (0 / -inf / -1e9 pad and window masks), rows contiguous
 *   dst  F16 [Nkv, Nq, H, B]          rows contiguous (nb[0] == 2); nb[1] may exceed 2*Nkv
 *
 * The dot products take f16-rounded inputs and accumulate in f32; scale, add and the rounding to f16 follow the
 * graph (f32 multiply, f32 add, round to nearest even, overflow to -inf).
 * An F16 table with contiguous rows is read in place.  An F32 (or strided) table is first copied to contiguous f16
 * in the library's per-device scratch block (2 bytes per element; see mi355x_fattn_params.workspace for when that
 * block may be shared); a table that does not change between calls - it depends on the layer and on T only - is
 * best converted once by the caller (mi355x_cpy to F16) and passed as F16.
 */
int mi355x_relpos_bias_supports(const mi355x_tensor * q_v, const mi355x_tensor * r, const mi355x_tensor * add,
                                const mi355x_tensor * dst);
/* workspace: room for the f16 copy of an F32 or strided table (mi355x_relpos_bias_workspace_size bytes, 16-byte aligned;
 * 0 for an F16 table with contiguous rows), or NULL to use the library's per-device scratch block under the rules of
 * mi355x_fattn_params.workspace (one stream at a time, never grown while the stream is capturing). */
int mi355x_relpos_bias_workspace_size(const mi355x_tensor * r, size_t * bytes);
int mi355x_relpos_bias(const mi355x_tensor * q_v, const mi355x_tensor * r, const mi355x_tensor * add,
                       const mi355x_tensor * dst, float scale, void * workspace, size_t workspace_size, void * stream);

/*
 * The whole flash branch of that block (fastconformer.h:915-934) in one call:
 *   dst = softmax(scale * q_u.k^T + mask) . v,   mask[j, i] = f16(scale * <q_v[i], r[Nq-1+j-i]> + add[j, i])
 * q_u, k, v, dst, params as for mi355x_flash_attn_ext (max_bias and logit_softcap must be 0); Nkv = k->ne[1].
 * With params->kernel = MI355X_FATTN_AUTO and head size 64 or 128 the position term is computed inside the attention
 * kernel, tile by tile, and never written out: the workspace then holds only f16 copies of K and V (unless they are F16
 * with 16-byte aligned rows already) and of the table (unless it is read in place); key tiles at the end of the range whose
 * additive mask is -inf for every query (a padded batch) are not walked.  With a kernel asked for by name - or a shape
 * the one-kernel form does not cover - the call is mi355x_relpos_bias into the workspace (rows padded to whole 128-byte
 * lines) followed by mi355x_flash_attn_ext with that mask: the same bits as the two calls made separately.  The two
 * forms round the same mask values and differ by the summation order of their matrix products only.
 */
int mi355x_flash_attn_relpos(const mi355x_tensor * q_u, const mi355x_tensor * q_v, const mi355x_tensor * k,
                             const mi355x_tensor * v, const mi355x_tensor * r, const mi355x_tensor * add,
                             const mi355x_tensor * dst, const mi355x_fattn_params * params, void * stream);
/* bytes of workspace that are enough for the call above in either form (the larger of the two needs: which form a call takes
 * depends on the alignment of its data pointers, which a size query made before allocation cannot know) */
int mi355x_fattn_relpos_workspace_size(const mi355x_tensor * q_u, const mi355x_tensor * q_v, const mi355x_tensor * k,
                                       const mi355x_tensor * v, const mi355x_tensor * r, const mi355x_tensor * add,
                                       const mi355x_fattn_params * params, size_t * bytes);

/* ---- GGML_OP_CPY / CONT / DUP with the destination in a device buffer --------------------- */

/*
 * dst[i] = convert(src[i]) for tensors of equal ne.  Supported: F32 -> F32 | F16 | any block type,
 * F16 -> F16 | F32, block type -> F32 | the same block type.  F32 -> F16 rounds to nearest even; F32 -> Q8_0
 * uses d = amax/127, q = round-to-nearest-even(x * (1/d)) per block of 32 along
 * dimension 0: the rounding of ggml-cpu's vectorised quantiser as the reference describes it
 * (tools/upstream-prs/09-metal-q8_0-bit-match.md:24-28, rint / vcvtnq); ggml's scalar reference quantiser is recalled to
 * round halves away from zero instead, so a value that lands exactly on a tie (x/d = k + 0.5) may differ by one step from
 * a cache written by a backend that follows the scalar code - tie behaviour is not pinned by anything in the reference.
 * F32 -> Q4_0 | Q4_1 | Q5_0 | Q5_1 follow ggml's scalar quantisers as recalled (see mi355x_type), every product and sum a
 * single f32 operation; dequantisation is q*d (exact) or q*d + m (product, then sum, each rounded to f32).
 * src may have any strides; dst rows (dimension 0) must be contiguous.
 */
int mi355x_cpy_supports(const mi355x_tensor * src, const mi355x_tensor * dst);
int mi355x_cpy(const mi355x_tensor * src, const mi355x_tensor * dst, void * stream);

/*
 * GGML_OP_SET_ROWS, the write into a quantised KV cache (src/core/attention.h:366-376):
 * dst[:, idx[i1, i2 % I1, i3 % I2], i2, i3] = convert(src[:, i1, i2, i3]).
 * src F32 [n0, n_rows, n2, n3]; idx I64 (idx_type 64) or I32 (idx_type 32) with
 * ne = {n_rows, I1, I2} and byte strides idx_nb; dst F32 | F16 | any block type [n0, rows, n2, n3].
 */
/* Rows whose index lies outside [0, rows) are not written (ggml-cpu asserts on them): a stale or uninitialised index
 * tensor cannot become a write outside the cache.  mi355x_set_rows_supports is the planning predicate (shapes, types,
 * alignment; data pointers as for mi355x_fattn_supports). */
int mi355x_set_rows_supports(const mi355x_tensor * src, int32_t idx_type, const int64_t idx_ne[3], const mi355x_tensor * dst);
int mi355x_set_rows(const mi355x_tensor * src, const void * idx, int32_t idx_type,
                    const int64_t idx_ne[3], const size_t idx_nb[3],
                    const mi355x_tensor * dst, void * stream);

/* ---- buffer vtable helpers (ggml_backend_buffer_i / ggml_backend_buffer_type_i) ------------ */

int mi355x_buffer_alloc(size_t size, void ** ptr);                 /* alloc_buffer (256-byte aligned) */
int mi355x_buffer_free(void * ptr);                                /* free_buffer */
/* pinned host memory the GPU can address at the same pointer (hipHostMalloc, mapped + coherent): the
 * is_host buffer type a one-op backend needs so that ggml-cpu keeps running every other op on it.
 *
 * The runtimes put their KV caches into the first GPU device's default buffer type (src/crispasr.cpp:3942-3971,
 * src/voxtral.cpp:1137-1145), i.e. into such a buffer, and attention reads them on every call.  So that those reads do not
 * cross the host link each time, a buffer grows a MIRROR in HBM - an allocation of its own size - when mi355x_cpy or
 * mi355x_set_rows first writes into it (the KV writes of the graphs).  From then on:
 *   - the host copy stays complete and authoritative; the mirror is kept page by page (64 KiB), a page being up to date or
 *     stale.  Every write through this library - mi355x_cpy, mi355x_set_rows, mi355x_buffer_memset / _set / _copy -
 *     stores the same bytes to both copies (the kernels store twice; no second launch), having fetched the stale pages it
 *     touches from the host copy first;
 *   - mi355x_flash_attn_ext reads a K or V that lies in the buffer from the mirror (stale pages of the view's span are
 *     fetched first, once), and mi355x_cpy a source that lies there; Q, the mask and the result stay where they are;
 *   - nothing but this library may write into the buffer's memory once it has a mirror - a caller that lets the CPU store
 *     into it directly (or another device) says so with mi355x_host_buffer_invalidate before the next call;
 *   - all calls that touch one buffer belong on one stream at a time (the bookkeeping is done when a call is enqueued).
 *     While a stream is being captured into a HIP graph, writes go to the host copy alone (their pages turn stale) and
 *     reads take the mirror only where it is up to date already: replays bypass the bookkeeping.  The mirror lives on the
 *     GPU that was current at the buffer's first KV write; a call made with another GPU current treats the buffer the
 *     same way (host copy only).
 * MI355X_NO_MIRROR=1 in the environment switches mirrors off (comparison runs). */
int mi355x_host_buffer_alloc(size_t size, void ** ptr);
int mi355x_host_buffer_free(void * ptr);
/* ptr: any address inside a host buffer.  mirror_bytes: 0 while the buffer has no mirror, else its size; valid_bytes:
 * bytes of pages that are up to date; uploaded_bytes: bytes fetched from the host copy so far.  Any of the three may be NULL. */
int mi355x_host_buffer_mirror_stats(const void * ptr, size_t * mirror_bytes, size_t * valid_bytes, size_t * uploaded_bytes);
/* [ptr, ptr + size) of a host buffer has been written behind the library's back: its pages are stale */
int mi355x_host_buffer_invalidate(void * ptr, size_t size);
/* memset_tensor / clear: asynchronous on the stream, done by a fill kernel (no memset node if the caller captures a graph) */
int mi355x_buffer_memset(void * ptr, int value, size_t size, void * stream);
int mi355x_buffer_set(void * dst, const void * host_src, size_t size, void * stream);   /* set_tensor  (sync) */
int mi355x_buffer_get(void * host_dst, const void * src, size_t size, void * stream);   /* get_tensor  (sync) */
int mi355x_buffer_copy(void * dst, const void * src, size_t size, void * stream);      /* cpy_tensor D2D */

#ifdef __cplusplus
}
#endif
#endif /* MI355X_FATTN_H */
