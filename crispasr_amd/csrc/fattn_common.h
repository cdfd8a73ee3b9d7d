// Shared between the gfx950 attention kernels and their launchers (internal).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <atomic>

#include "../../include/mi355x_fattn.h"

#define FATTN_QK8_0 32
#define FATTN_Q8_0_BYTES 34
#define FATTN_IS_BLOCK_TYPE(t) ((t) == MI355X_TYPE_Q8_0 || (t) == MI355X_TYPE_Q4_0 || (t) == MI355X_TYPE_Q4_1 || (t) == MI355X_TYPE_Q5_0 || (t) == MI355X_TYPE_Q5_1)

// Everything a kernel needs about one FLASH_ATTN_EXT node, by value.
struct FattnArgs {
    const char * q;      // F32  [D, Nq, Hq, B]
    const char * k;      // K/V storage type [D, Nkv, Hkv, Bk]
    const char * v;
    const char * mask;   // F16 [>=Nkv, >=Nq, Hm, Bm] or nullptr
    float *      dst;    // F32 [D, Hq, Nq, B] contiguous

    int32_t D, Nq, Hq, B, Nkv, Hkv, Bk;
    int32_t Dv;          // elements of a q row and of a dst row; = D, except when the tile kernel runs a head size it has no
                         // form for on f16 copies of K/V whose rows are zero-padded to D (64 or 128): then the real head size
    int32_t gqa;         // Hq / Hkv
    int32_t bq;          // B / Bk
    int32_t q_chunks;    // decode kernel: 16-row chunks of the Nq * gqa query rows that share a KV head
    int32_t Hm, Bm;      // mask broadcast extents
    int32_t masked;      // the call has a mask (planning looks here: `mask` may still be null when a call is only being sized)

    int64_t nbq1, nbq2, nbq3;
    int64_t nbk1, nbk2, nbk3;
    int64_t nbv1, nbv2, nbv3;
    int64_t nbm1, nbm2, nbm3;

    float scale;         // already divided by logit_softcap when that is non-zero
    float softcap;
    float max_bias, m0, m1;
    int32_t n_head_log2;

    int32_t aligned16;   // q, k and v bases and strides are all multiples of 16 bytes
    int32_t q_aligned16; // q alone
    int32_t kv_aligned16; // k and v alone
    int32_t kv_aligned4;
    int32_t kv_aligned2;  // k and v: base and strides even (what the Q8_0 halfword reads need)
    int32_t mask_al8;    // mask base and strides are multiples of 8 bytes
    int32_t mask_al4;    // ... of 4 bytes
    int32_t n_cus;       // compute units of the device
    int32_t tile_variant; // 0, or 16 * key_split + query_blocks forced by the caller

    // split-KV
    int32_t n_splits;
    int32_t keys_per_split;
    float * part_acc;    // [rows, n_splits, D]  unnormalised accumulators
    float * part_ml;     // [rows, n_splits, 2]  running max, running sum
    // nullptr: the partials are merged by fattn_merge_kernel, a launch of its own.  Else one counter per set of
    // workgroups that share output rows (zero between launches): every workgroup adds one when its partials are out, and
    // the one that finds the set complete merges the rows itself and leaves the counter at zero again.
    unsigned * counters;
};

// Workgroups that use more than 64 KiB of dynamic LDS need hipFuncAttributeMaxDynamicSharedMemorySize raised, and that
// attribute belongs to the (kernel, device) pair: `done` is the launcher's own record per kernel instantiation, one bit
// per device.  Racing callers at worst set the attribute twice.
static inline hipError_t fattn_allow_lds(const void * kernel, int lds_bytes, std::atomic<uint64_t> & done) {
    if (lds_bytes <= 64 * 1024) return hipSuccess;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    const uint64_t bit = dev >= 0 && dev < 64 ? (uint64_t)1 << dev : 0;      // devices past 63: set on every launch
    if (bit && (done.load(std::memory_order_relaxed) & bit)) return hipSuccess;
    e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    if (e == hipSuccess && bit) done.fetch_or(bit, std::memory_order_relaxed);
    return e;
}

static __device__ __forceinline__ float fattn_slope(const FattnArgs & a, int h) {
    if (a.max_bias <= 0.0f) return 1.0f;
    return h < a.n_head_log2 ? powf(a.m0, (float)(h + 1)) : powf(a.m1, (float)(2 * (h - a.n_head_log2) + 1));
}

// A load marked non-temporal, for data that a launch reads once: it leaves the rest of L2 alone and streams faster (a
// read-only sweep of 2 GiB reaches 7.0-7.1 TB/s with it against 5.7-6.2 TB/s with plain loads; a copy gains 5%).  T is
// a scalar or an ext_vector_type.  Not for lines that the same launch touches again (64-byte pieces of mask rows and
// per-lane pieces of block rows were slower with it), nor for a source that the previous launch has just written (the
// F32 -> f16 pass over fresh K/V lost 4% with it).
template <typename T>
static __device__ __forceinline__ T stream_load(const void * p) { return __builtin_nontemporal_load((const T *)p); }

// a * b + c with the product and the sum each rounded to f32, as two graph nodes (or two scalar statements) round them.
// hipcc contracts a * b + c into one fused multiply-add by default, also when it is spelled __fadd_rn(__fmul_rn(a, b), c):
// those inline as contractible operations.  Only operations compiled under "contract(off)" stay apart.
static __device__ __forceinline__ float mul_then_add(float a, float b, float c) {
#pragma clang fp contract(off)
    const float p = a * b;
    return p + c;
}

static __device__ __forceinline__ float h2f_bits(uint16_t h) {
    return (float)__builtin_bit_cast(_Float16, h);
}

// ---- DPP wavefront reductions -------------------------------------------------------
// Butterfly sums over aligned groups of lanes; every lane of a group ends with the total.
template <int CTRL>
static __device__ __forceinline__ float dpp_mov(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, true));
}

static __device__ __forceinline__ float xor_shuffle(float x, int mask) {
    return __shfl_xor(x, mask, 64);
}

template <int GROUP>
static __device__ __forceinline__ float group_sum(float x) {
    static_assert(GROUP == 4 || GROUP == 8 || GROUP == 16 || GROUP == 32 || GROUP == 64, "group size");
    x += dpp_mov<0xB1>(x);                        // quad_perm [1,0,3,2]
    x += dpp_mov<0x4E>(x);                        // quad_perm [2,3,0,1]
    if (GROUP >= 8)  x += dpp_mov<0x141>(x);      // row_half_mirror: pairs the two quads of 8 lanes
    if (GROUP >= 16) x += dpp_mov<0x140>(x);      // row_mirror: pairs the two halves of a row of 16
    if (GROUP >= 32) x += xor_shuffle(x, 16);
    if (GROUP >= 64) x += xor_shuffle(x, 32);
    return x;
}

template <int GROUP>
static __device__ __forceinline__ float group_max(float x) {
    x = fmaxf(x, dpp_mov<0xB1>(x));
    x = fmaxf(x, dpp_mov<0x4E>(x));
    if (GROUP >= 8)  x = fmaxf(x, dpp_mov<0x141>(x));
    if (GROUP >= 16) x = fmaxf(x, dpp_mov<0x140>(x));
    if (GROUP >= 32) x = fmaxf(x, xor_shuffle(x, 16));
    if (GROUP >= 64) x = fmaxf(x, xor_shuffle(x, 32));
    return x;
}

// ---- merging split-KV partials ---------------------------------------------------------
// Loads and stores that are coherent across the whole device while the kernel runs (the L2 caches of the chip's eight
// dies are not, for ordinary accesses): what workgroups of one launch hand to each other goes through these.
static __device__ __forceinline__ void device_store(float * p, float v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
static __device__ __forceinline__ float2 device_load2(const float2 * p) {
    const uint64_t u = __hip_atomic_load((const uint64_t *)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return __builtin_bit_cast(float2, u);
}
static __device__ __forceinline__ float4 device_load4(const float4 * p) {
    const float2 lo = device_load2((const float2 *)p), hi = device_load2((const float2 *)p + 1);
    return make_float4(lo.x, lo.y, hi.x, hi.y);
}

// out[row] = sum_s acc_s * exp(m_s - M) / sum_s l_s * exp(m_s - M), for the four values d4*4 .. d4*4+3 of the row.
// The (m, l) pairs and the accumulators of FATTN_MERGE_BATCH splits are requested together, and the next batch is
// requested before the current one is folded in: a row costs about one memory round trip however many splits it has
// (folded in split order, one batch after the other, whatever is in flight).  DEVICE: the partials come from other
// workgroups of this launch.
constexpr int FATTN_MERGE_BATCH = 8;
template <bool DEVICE>
static __device__ __forceinline__ void fattn_merge_row(const FattnArgs & a, int64_t row, int d4) {
    constexpr int NB = FATTN_MERGE_BATCH;
    const int lpr = a.D / 4;
    const float2 * pm = (const float2 *)(a.part_ml + (size_t)row * a.n_splits * 2);
    const float4 * pa = (const float4 *)(a.part_acc + (size_t)row * a.n_splits * a.D) + d4;
    float4 out = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    float  M = -INFINITY, L = 0.0f;
    auto request = [&](int s0, float2 (&ml)[NB], float4 (&v)[NB]) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < NB; i++) {
            const int s = min(s0 + i, a.n_splits - 1);          // (past the end: a second look at the last one, not used)
            ml[i] = DEVICE ? device_load2(pm + s) : pm[s];
            v[i]  = DEVICE ? device_load4(pa + (size_t)s * lpr) : pa[(size_t)s * lpr];
            if (s0 + i >= a.n_splits) ml[i] = make_float2(-INFINITY, 0.0f);
        }
    };
    auto fold = [&](const float2 (&ml)[NB], const float4 (&v)[NB]) __attribute__((always_inline)) {
        float Mb = M;
#pragma unroll
        for (int i = 0; i < NB; i++) Mb = fmaxf(Mb, ml[i].x);
        if (Mb == -INFINITY) return;                // nothing visible so far
        const float f = __expf(M - Mb);             // M = -inf gives 0
        L *= f; out.x *= f; out.y *= f; out.z *= f; out.w *= f;
        M = Mb;
#pragma unroll
        for (int i = 0; i < NB; i++) {
            // a split that saw no key carries m = -inf and an accumulator that must not be touched (select, not multiply)
            const bool  seen = ml[i].x != -INFINITY;
            const float w    = seen ? __expf(ml[i].x - M) : 0.0f;
            L     += seen ? ml[i].y * w : 0.0f;
            out.x += seen ? v[i].x * w : 0.0f;
            out.y += seen ? v[i].y * w : 0.0f;
            out.z += seen ? v[i].z * w : 0.0f;
            out.w += seen ? v[i].w * w : 0.0f;
        }
    };
    float2 ml0[NB], ml1[NB];
    float4 v0[NB], v1[NB];
    request(0, ml0, v0);
    for (int s0 = 0; s0 < a.n_splits; s0 += 2 * NB) {
        const bool more1 = s0 + NB < a.n_splits, more2 = s0 + 2 * NB < a.n_splits;
        if (more1) request(s0 + NB, ml1, v1);
        fold(ml0, v0);
        if (!more1) break;
        if (more2) request(s0 + 2 * NB, ml0, v0);
        fold(ml1, v1);
    }
    const float inv = L > 0.0f ? 1.0f / L : 0.0f;
    out.x *= inv; out.y *= inv; out.z *= inv; out.w *= inv;
    // (dst rows are Dv floats - the head size - also where the partial rows are those of a head zero-padded to D)
    if (d4 * 4 < a.Dv) *((float4 *)(a.dst + (size_t)row * a.Dv) + d4) = out;
}

// The end of a workgroup that has stored its partials, when the launch merges in the kernel (a.counters): true for the
// one workgroup of set `group` that finds the other n - 1 done.  The partials were stored by device_store (a thread that
// used ordinary stores says so with `wrote_plain`, and pays for a write-back of its die's whole L2): every thread waits
// for its stores to be acknowledged before the workgroup counts itself done, and the merging workgroup reads by
// device_load.  All threads of the workgroup must call this; `flag` is a word of LDS that nothing else uses from here on.
// The counter is zero again when the set is complete.
static __device__ __forceinline__ bool fattn_last_of_set(const FattnArgs & a, int64_t group, int n, int * flag, bool wrote_plain) {
    if (wrote_plain) __threadfence();
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) {
        const unsigned old = __hip_atomic_fetch_add(a.counters + group, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const bool     all = old == (unsigned)(n - 1);
        if (all) __hip_atomic_store(a.counters + group, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        *flag = all;
    }
    __syncthreads();
    return *flag != 0;
}

template <int GROUP>
static __device__ __forceinline__ float group_min(float x) { return -group_max<GROUP>(-x); }

// ---- block-32 storage types ------------------------------------------------------------
// BYTES per block, offsets of the quants (QS), of the fifth bits (QH, 0 = none) and whether a minimum follows the scale
template <int TYPE> struct BlockFormat;
template <> struct BlockFormat<MI355X_TYPE_Q4_0> { static constexpr int BYTES = 18, QS = 2, QH = 0, LEVELS = 16; static constexpr bool HAS_M = false; };
template <> struct BlockFormat<MI355X_TYPE_Q4_1> { static constexpr int BYTES = 20, QS = 4, QH = 0, LEVELS = 16; static constexpr bool HAS_M = true;  };
template <> struct BlockFormat<MI355X_TYPE_Q5_0> { static constexpr int BYTES = 22, QS = 6, QH = 2, LEVELS = 32; static constexpr bool HAS_M = false; };
template <> struct BlockFormat<MI355X_TYPE_Q5_1> { static constexpr int BYTES = 24, QS = 8, QH = 4, LEVELS = 32; static constexpr bool HAS_M = true;  };
template <> struct BlockFormat<MI355X_TYPE_Q8_0> { static constexpr int BYTES = 34, QS = 2, QH = 0, LEVELS = 256; static constexpr bool HAS_M = false; };

static inline __host__ __device__ int fattn_block_bytes(int type) {
    switch (type) {
        case MI355X_TYPE_Q4_0: return 18;
        case MI355X_TYPE_Q4_1: return 20;
        case MI355X_TYPE_Q5_0: return 22;
        case MI355X_TYPE_Q5_1: return 24;
        case MI355X_TYPE_Q8_0: return 34;
        default:               return 0;
    }
}

// elements j0 .. j0+7 (j0 = 0, 8, 16 or 24) of one block as f32: q*d is exact, q*d + m is one product and one sum,
// each rounded to f32 (not fused).  Blocks are only 2-byte aligned: halfword reads.
template <int TYPE>
static __device__ __forceinline__ void dequant8(const char * blk, int j0, float (&out)[8]) {
    typedef BlockFormat<TYPE> F;
    const float d = h2f_bits(*(const uint16_t *)blk);
    if (TYPE == MI355X_TYPE_Q8_0) {
        const uint16_t * qs = (const uint16_t *)(blk + 2 + j0);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint16_t w = qs[i];
            out[2 * i]     = (float)(int8_t)(w & 0xff) * d;
            out[2 * i + 1] = (float)(int8_t)(w >> 8) * d;
        }
        return;
    }
    const float m = F::HAS_M ? h2f_bits(*(const uint16_t *)(blk + 2)) : 0.0f;
    const uint16_t * qs = (const uint16_t *)(blk + F::QS + (j0 & 8));       // elements j and j + 16 share a byte
    const int sh = (j0 & 16) ? 4 : 0;
    uint32_t hb = 0;
    if (F::QH) {
        const uint16_t * qh = (const uint16_t *)(blk + F::QH);
        hb = (((uint32_t)qh[0] | (uint32_t)qh[1] << 16) >> j0) & 0xffu;
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t w  = qs[i];
        const int      q0 = (int)(((w >> sh) & 15u) | (((hb >> (2 * i)) & 1u) << 4));
        const int      q1 = (int)(((w >> (8 + sh)) & 15u) | (((hb >> (2 * i + 1)) & 1u) << 4));
        if (F::HAS_M) {
            out[2 * i]     = mul_then_add((float)q0, d, m);
            out[2 * i + 1] = mul_then_add((float)q1, d, m);
        } else {
            out[2 * i]     = (float)(q0 - F::LEVELS / 2) * d;
            out[2 * i + 1] = (float)(q1 - F::LEVELS / 2) * d;
        }
    }
}

// One CPY / SET_ROWS node.
struct CpyArgs {
    const char * src;
    char *       dst;
    int64_t sne[4], dne[4];
    int64_t snb[4], dnb[4];
    int64_t n;                 // elements (or blocks of 32 when a side is a block type)
    int64_t mirror;            // 0, or the distance in bytes from dst to a second copy that gets the same stores
    // SET_ROWS only
    const char * idx;
    int32_t idx_is_i64;
    int64_t ine[3], inb[3];
};

// The relative-position mask of a FastConformer attention block (relpos.hip).
struct RelposArgs {
    const char * qv;  size_t nbq1, nbq2, nbq3;                  // F32 [D, Nq, H, B]
    const char * r;   size_t nbr1, nbr2, nbr3; int32_t Hr, Br;   // F32 | F16 [D, Nq+Nkv-1, Hr, Br]
    const char * add; size_t nba1, nba2, nba3; int32_t Ha, Ba;   // optional F32 | F16 [>=Nkv, >=Nq, Ha, Ba]
    int32_t add_f16;
    char *       out; size_t nbo1, nbo2, nbo3;                  // F16 [Nkv, Nq, H, B], rows contiguous
    int32_t out_al4;                                            // out base and strides are multiples of 4 bytes
    int32_t D, Nq, Nkv, H, B;
    float   scale;
    int32_t n_cus;                                              // CUs of the device (0 = unknown)
    int32_t n_qblocks, n_chunks, chunk_tiles;                   // filled in by the launcher
};

// FastConformer's relative-position attention in one kernel (fattn_relpos.hip): K, V and the table are f16
struct FattnRelposArgs {
    const char * qu;  int64_t nbu1, nbu2, nbu3;                  // F32 [D, Nq, H, B]: q + pos_bias_u
    const char * qv;  int64_t nbw1, nbw2, nbw3;                  // F32 [D, Nq, H, B]: q + pos_bias_v
    const char * k;   int64_t nbk1, nbk2, nbk3;                  // F16 [D, Nkv, H / gqa, B / bq]
    const char * v;   int64_t nbv1, nbv2, nbv3;
    const char * r;   int64_t nbr1, nbr2, nbr3; int32_t Hr, Br;   // F16 [D, Nq+Nkv-1, Hr, Br]
    const char * add; int64_t nba1, nba2, nba3; int32_t Ha, Ba;   // optional F32 | F16 [>=Nkv, >=Nq, Ha, Ba]
    int32_t add_f16;
    float *      dst;                                            // F32 [D, H, Nq, B] contiguous
    int32_t D, Nq, Nkv, H, B, gqa, bq;
    int32_t n_cus;
    float   scale;
};

// Launchers implemented next to their kernels; all return hipError_t as int.
int fattn_vec_launch(const FattnArgs & a, int ktype, hipStream_t stream);
int fattn_merge_launch(const FattnArgs & a, hipStream_t stream);
int fattn_mma_launch(const FattnArgs & a, int ktype, hipStream_t stream);
// the instantiation of the tile kernel a call takes
struct FattnMmaVariant {
    int  query_blocks;            // 32-query blocks per wave (1 or 2)
    int  key_split;               // 2: the waves of a workgroup pair up over the two halves of every key tile
    int  queries_per_workgroup;
    bool direct;                  // K/V tiles move global -> LDS without passing registers
    bool mask_dma;                // so does the mask
};
void fattn_mma_variant(const FattnArgs & a, int ktype, FattnMmaVariant & v);
bool fattn_mma_supported(const FattnArgs & a, int ktype);
int fattn_decode_launch(const FattnArgs & a, int ktype, hipStream_t stream);
bool fattn_decode_supported(const FattnArgs & a, int ktype);
int cpy_launch(const CpyArgs & a, int stype, int dtype, hipStream_t stream);
int set_rows_launch(const CpyArgs & a, int dtype, hipStream_t stream);
int fill_launch(void * ptr, int value, size_t size, hipStream_t stream);      // memset by a kernel
int relpos_bias_launch(RelposArgs a, int rtype, hipStream_t stream);
int fattn_relpos_launch(const FattnRelposArgs & a, hipStream_t stream);
bool fattn_relpos_supported(const FattnRelposArgs & a);
// an F32 tensor [D, ne1, ne2, ne3] (D = the attention call's head size, rows 16-byte aligned) converted to a contiguous f16
// copy by the same launch; n = its 8-element chunks
// (kv_to_f16_launch: K and V, of any storage type each and any strides, -> contiguous f16 [D, Nkv, Hkv, Bk] at dst and right
//  behind it; the rider only beside a K and V of one type)
struct F32Rider {
    const char * src;
    char *       dst;
    int64_t ne1, ne2, nb1, nb2, nb3, n;
};
int kv_to_f16_launch(const FattnArgs & a, int ktype, int vtype, void * dst, hipStream_t stream, const F32Rider * rider = nullptr);
