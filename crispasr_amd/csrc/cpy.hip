// GGML_OP_CPY / CONT / DUP / SET_ROWS with the destination in device memory: the KV-cache
// writes that feed FLASH_ATTN_EXT (src/crispasr.cpp:2810-2811, 3185-3203, 2956-2973;
// src/core/attention.h:342-378) and the dequantising reads (src/core/attention.h:917-920).
// HBM-bound byte work: one element (or one element of a block of 32) per lane, coalesced along
// dimension 0.  Source and destination may have different shapes with equal element
// counts (the reference copies a [n_state, n_ctx] tensor into a 1-D cache view).
#include "fattn_common.h"

#include <string.h>

// The quantisers must round every product and every sum on its own, as the reference's scalar code does: hipcc's default
// contraction turns x * id + c into one fused multiply-add (so do __fmul_rn / __fadd_rn, which inline as contractible), and
// an element whose sum lands within half an ulp of an integer then truncates to the neighbouring level.
#pragma clang fp contract(off)

namespace {

// byte offset of unit i, where a unit is `unit0` elements along dimension 0 and one step of
// nb[0] covers `per_nb0` elements (32 for a Q8_0 tensor, 1 otherwise)
__device__ __forceinline__ int64_t offset_of(int64_t i, const int64_t (&ne)[4], const int64_t (&nb)[4],
                                             int64_t unit0, int64_t per_nb0 = 1) {
    const int64_t n0 = ne[0] / unit0;
    const int64_t i0 = i % n0;  i /= n0;
    const int64_t i1 = i % ne[1]; i /= ne[1];
    const int64_t i2 = i % ne[2];
    const int64_t i3 = i / ne[2];
    return i0 * (unit0 / per_nb0) * nb[0] + i1 * nb[1] + i2 * nb[2] + i3 * nb[3];
}

template <typename TS, typename TD>
__global__ void __launch_bounds__(256) cpy_scalar_kernel(const CpyArgs a) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= a.n) return;
    const TS x = *(const TS *)(a.src + offset_of(i, a.sne, a.snb, 1));
    char * dp = a.dst + offset_of(i, a.dne, a.dnb, 1);
    *(TD *)dp = (TD)x;                                          // f32 -> f16 is round-to-nearest-even
    if (a.mirror) *(TD *)(dp + a.mirror) = (TD)x;
}

// 8 consecutive elements of dimension 0 per lane: 128-bit loads and stores for f16 <-> f32 and same-type copies.
// Launched only when both sides have ne0 % 8 == 0, unit element stride and 16-byte aligned rows.
template <typename TS, typename TD>
__global__ void __launch_bounds__(256) cpy_vec8_kernel(const CpyArgs a) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= a.n) return;
    const TS * sp = (const TS *)(a.src + offset_of(i, a.sne, a.snb, 8));
    TD *       dp = (TD *)(a.dst + offset_of(i, a.dne, a.dnb, 8));
    typedef TS vs8 __attribute__((ext_vector_type(8)));
    typedef TD vd8 __attribute__((ext_vector_type(8)));
    const vs8 x = *(const vs8 *)sp;
    vd8 y;
#pragma unroll
    for (int e = 0; e < 8; e++) y[e] = (TD)x[e];
    *(vd8 *)dp = y;
    if (a.mirror) *(vd8 *)((char *)dp + a.mirror) = y;
}

// quantise one block of 32 held one element per lane (32 consecutive lanes) and store it
// (called by every lane of the wave: the reductions run before any divergence).
//   Q8_0: d = amax/127 (f32), q = rne(x * (1/d)), d stored as fp16
//   Q4_0 / Q5_0: d = (signed value of largest magnitude, the first one) / -8 (-16), q = min(15 (31), trunc(x/d + 8.5 (16.5)))
//   Q4_1 / Q5_1: d = (max - min) / 15 (31), m = min, q = min(15 (31), trunc((x - min)/d + 0.5))
// every product and sum is a single f32 operation, none fused.
// mirror: 0, or the distance to a second copy of the destination that gets the same bytes
template <int TYPE>
__device__ __forceinline__ void quantize_block_store(float x, char * blk, int e, bool ok, int64_t mirror) {
    typedef BlockFormat<TYPE> F;
    const int copies = mirror ? 2 : 1;
    if (TYPE == MI355X_TYPE_Q8_0) {
        const float amax = group_max<32>(fabsf(x));
        const float d    = amax / 127.0f;
        const float id   = d != 0.0f ? 1.0f / d : 0.0f;
        const int   qi   = (int)rintf(x * id);
        if (ok) {
            for (int c = 0; c < copies; c++, blk += mirror) {
                ((int8_t *)(blk + 2))[e] = (int8_t)qi;
                if (e == 0) *(_Float16 *)blk = (_Float16)d;
            }
        }
        return;
    }
    const int half = (threadIdx.x & 32);                 // which 32 lanes of the wave hold this block
    float d, m = 0.0f;
    int   qi;
    if (!F::HAS_M) {
        const float    amax  = group_max<32>(fabsf(x));
        const uint32_t who   = (uint32_t)(__ballot(fabsf(x) == amax) >> half);
        const int      first = who ? __ffs(who) - 1 : 0;
        float ext = __shfl(x, half + first, 64);
        if (!(amax > 0.0f)) ext = 0.0f;
        d = ext / (float)(-(F::LEVELS / 2));
        const float id = d != 0.0f ? 1.0f / d : 0.0f;
        const float x0 = x * id;
        qi = (int)(int8_t)(int)(x0 + ((float)(F::LEVELS / 2) + 0.5f));
    } else {
        m = group_min<32>(x);
        const float mx = group_max<32>(x);
        d = (mx - m) / (float)(F::LEVELS - 1);
        const float id = d != 0.0f ? 1.0f / d : 0.0f;
        const float x0 = (x - m) * id;
        qi = (int)(uint8_t)(int)(x0 + 0.5f);
    }
    qi = qi < F::LEVELS - 1 ? qi : F::LEVELS - 1;
    const int      hi = __shfl(qi, half + (e & 15) + 16, 64);       // the element that shares this lane's byte
    const uint32_t qh = (uint32_t)(__ballot((qi & 0x10) != 0) >> half);
    if (ok) {
        for (int c = 0; c < copies; c++, blk += mirror) {
            if (e < 16) ((uint8_t *)(blk + F::QS))[e] = (uint8_t)((qi & 15) | ((hi & 15) << 4));
            if (e == 16) *(_Float16 *)blk = (_Float16)d;
            if (F::HAS_M && e == 17) *(_Float16 *)(blk + 2) = (_Float16)m;
            if (F::QH && e == 18) *(uint16_t *)(blk + F::QH) = (uint16_t)qh;
            if (F::QH && e == 19) *(uint16_t *)(blk + F::QH + 2) = (uint16_t)(qh >> 16);
        }
    }
}

// F32 -> block type; one block per 32 lanes
template <int TYPE>
__global__ void __launch_bounds__(256) cpy_f32_block_kernel(const CpyArgs a) {
    const int64_t blk = (int64_t)blockIdx.x * 8 + (threadIdx.x >> 5);
    const int     e   = threadIdx.x & 31;
    const bool    ok  = blk < a.n;
    const int64_t bc  = ok ? blk : 0;                       // keep all lanes in the reductions
    const char *  sp  = a.src + offset_of(bc, a.sne, a.snb, FATTN_QK8_0) + e * a.snb[0];
    const float   x   = ok ? *(const float *)sp : 0.0f;
    char * dp = a.dst + offset_of(bc, a.dne, a.dnb, FATTN_QK8_0, FATTN_QK8_0);
    quantize_block_store<TYPE>(x, dp, e, ok, a.mirror);
}

// block type -> F32; 8 elements per lane, four lanes per block
template <int TYPE>
__global__ void __launch_bounds__(256) cpy_block_f32_kernel(const CpyArgs a) {
    const int64_t t   = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t blk = t >> 2;
    const int     j0  = (int)(t & 3) * 8;
    if (blk >= a.n) return;
    const char * sp = a.src + offset_of(blk, a.sne, a.snb, FATTN_QK8_0, FATTN_QK8_0);
    float y[8];
    dequant8<TYPE>(sp, j0, y);
    char * dp = a.dst + offset_of(blk, a.dne, a.dnb, FATTN_QK8_0) + j0 * a.dnb[0];
#pragma unroll
    for (int i = 0; i < 8; i++) *(float *)(dp + i * a.dnb[0]) = y[i];
    if (a.mirror) {
#pragma unroll
        for (int i = 0; i < 8; i++) *(float *)(dp + a.mirror + i * a.dnb[0]) = y[i];
    }
}

// same block type on both sides: move the blocks as halfwords
template <int TYPE>
__global__ void __launch_bounds__(256) cpy_block_block_kernel(const CpyArgs a) {
    constexpr int HW = BlockFormat<TYPE>::BYTES / 2;
    const int64_t t   = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t blk = t / HW;
    const int     w   = (int)(t % HW);
    if (blk >= a.n) return;
    const uint16_t * sp = (const uint16_t *)(a.src + offset_of(blk, a.sne, a.snb, FATTN_QK8_0, FATTN_QK8_0));
    uint16_t *       dp = (uint16_t *)(a.dst + offset_of(blk, a.dne, a.dnb, FATTN_QK8_0, FATTN_QK8_0));
    dp[w] = sp[w];
    if (a.mirror) *(uint16_t *)((char *)(dp + w) + a.mirror) = sp[w];
}

// SET_ROWS: dst[:, idx[i1, i2 % ine1, i3 % ine2], i2, i3] = convert(src[:, i1, i2, i3]), src F32
template <int DTYPE>
__global__ void __launch_bounds__(256) set_rows_kernel(const CpyArgs a) {
    // one unit = 32 elements of a source row (block types) or 1 element (F16/F32)
    constexpr bool BLOCKS = FATTN_IS_BLOCK_TYPE(DTYPE);
    constexpr int  UNIT   = BLOCKS ? FATTN_QK8_0 : 1;
    int64_t u;
    int     e = 0;
    if (UNIT == 1) {
        u = (int64_t)blockIdx.x * 256 + threadIdx.x;
    } else {
        u = (int64_t)blockIdx.x * 8 + (threadIdx.x >> 5);
        e = threadIdx.x & 31;
    }
    const bool ok = u < a.n;
    int64_t    r  = ok ? u : 0;
    const int64_t n0 = a.sne[0] / UNIT;
    const int64_t i0 = r % n0;      r /= n0;
    const int64_t i1 = r % a.sne[1]; r /= a.sne[1];
    const int64_t i2 = r % a.sne[2];
    const int64_t i3 = r / a.sne[2];
    const char * ip = a.idx + i1 * a.inb[0] + (i2 % a.ine[1]) * a.inb[1] + (i3 % a.ine[2]) * a.inb[2];
    const int64_t drow = a.idx_is_i64 ? *(const int64_t *)ip : (int64_t)*(const int32_t *)ip;
    // A row index outside the destination writes nothing (ggml-cpu asserts 0 <= idx < ne1 instead): a stale or
    // uninitialised index tensor must not become a write outside the cache.  The lanes stay in the block's reduction.
    const bool inside = ok && drow >= 0 && drow < a.dne[1];
    const char * sp = a.src + (i0 * UNIT + e) * a.snb[0] + i1 * a.snb[1] + i2 * a.snb[2] + i3 * a.snb[3];
    const float  x  = ok ? *(const float *)sp : 0.0f;
    char * dp = a.dst + i0 * a.dnb[0] + (inside ? drow : 0) * a.dnb[1] + i2 * a.dnb[2] + i3 * a.dnb[3];
    if constexpr (BLOCKS) {
        quantize_block_store<DTYPE>(x, dp, e, inside, a.mirror);
    } else if (inside) {
        for (int c = 0; c < (a.mirror ? 2 : 1); c++, dp += a.mirror) {
            if (DTYPE == MI355X_TYPE_F16) *(_Float16 *)dp = (_Float16)x;
            else                          *(float *)dp = x;
        }
    }
}

// K and V of one attention call -> two contiguous f16 tensors [D, Nkv, Hkv, Bk] (K first, V right behind it), one
// launch for both.  One lane per 8 elements of a row: two 128-bit loads (F32) or 8 quants and the block's scale
// (Q8_0), one 128-bit store.  Rounding is the tile kernel's own: f32 -> f16 round-to-nearest-even, q*d exact in f32
// and then rounded once.
// An F32 table [D, n1, n2, n3] with 16-byte aligned rows may ride along (the relative-position table of a FastConformer
// block, rounded for the same call): the threads behind K's and V's write its contiguous f16 copy.
template <int TYPE>
__global__ void __launch_bounds__(256) kv_to_f16_kernel(const FattnArgs a, char * dst, const F32Rider x) {
    const int     cpr  = a.D / 8;                                  // chunks per row
    const int64_t half = (int64_t)cpr * a.Nkv * a.Hkv * a.Bk;      // chunks per tensor
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= 2 * half) {
        i -= 2 * half;
        if (i >= x.n) return;
        const int c = (int)(i % cpr);
        int64_t   r = i / cpr;
        const int64_t i1 = r % x.ne1;  r /= x.ne1;
        const int64_t i2 = r % x.ne2;
        const int64_t i3 = r / x.ne2;
        const char * row = x.src + i1 * x.nb1 + i2 * x.nb2 + i3 * x.nb3;
        const float4 x0 = *(const float4 *)(row + c * 32);
        const float4 x1 = *(const float4 *)(row + c * 32 + 16);
        typedef _Float16 h8 __attribute__((ext_vector_type(8)));
        h8 y;
        y[0] = (_Float16)x0.x; y[1] = (_Float16)x0.y; y[2] = (_Float16)x0.z; y[3] = (_Float16)x0.w;
        y[4] = (_Float16)x1.x; y[5] = (_Float16)x1.y; y[6] = (_Float16)x1.z; y[7] = (_Float16)x1.w;
        *(h8 *)(x.dst + i * 16) = y;
        return;
    }
    const bool is_v = i >= half;
    if (is_v) i -= half;
    const int     c = (int)(i % cpr);
    int64_t       r = i / cpr;
    const int64_t j = r % a.Nkv;  r /= a.Nkv;
    const int64_t h = r % a.Hkv;
    const int64_t b = r / a.Hkv;
    const char * row = is_v ? a.v + j * a.nbv1 + h * a.nbv2 + b * a.nbv3
                            : a.k + j * a.nbk1 + h * a.nbk2 + b * a.nbk3;
    typedef _Float16 h8 __attribute__((ext_vector_type(8)));
    h8 y;
    if constexpr (TYPE == MI355X_TYPE_F32) {
        const float4 x0 = *(const float4 *)(row + c * 32);
        const float4 x1 = *(const float4 *)(row + c * 32 + 16);
        y[0] = (_Float16)x0.x; y[1] = (_Float16)x0.y; y[2] = (_Float16)x0.z; y[3] = (_Float16)x0.w;
        y[4] = (_Float16)x1.x; y[5] = (_Float16)x1.y; y[6] = (_Float16)x1.z; y[7] = (_Float16)x1.w;
    } else {
        float f[8];
        dequant8<TYPE>(row + (c >> 2) * fattn_block_bytes(TYPE), (c & 3) * 8, f);
#pragma unroll
        for (int e = 0; e < 8; e++) y[e] = (_Float16)f[e];
    }
    *(h8 *)(dst + ((is_v ? half : 0) + i) * 16) = y;
}

// The same for a K and a V of different storage types (CRISPASR_KV_QUANT_K / _V, src/core/attention.h:132-137; the
// Canary decoder hands both cache views to the op as they are, src/canary.cpp:953-972): the type is looked up per
// tensor at run time.  Scalar loads: such rows are only as aligned as their type.
// It is also the launch that pads: the copies' rows are a.D elements long, the first a.Dv of them the source row's
// (a multiple of 8), zeros behind - how the tile kernel, which has forms for 64- and 128-wide heads, gets the others.
__global__ void __launch_bounds__(256) kv_to_f16_mixed_kernel(const FattnArgs a, const int ktype, const int vtype, char * dst) {
    const int     cpr  = a.D / 8;
    const int64_t half = (int64_t)cpr * a.Nkv * a.Hkv * a.Bk;
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= 2 * half) return;
    const bool is_v = i >= half;
    if (is_v) i -= half;
    const int     c = (int)(i % cpr);
    if (c * 8 >= a.Dv) {
        *(uint4 *)(dst + ((is_v ? half : 0) + i) * 16) = uint4{0u, 0u, 0u, 0u};
        return;
    }
    int64_t       r = i / cpr;
    const int64_t j = r % a.Nkv;  r /= a.Nkv;
    const int64_t h = r % a.Hkv;
    const int64_t b = r / a.Hkv;
    const char * row = is_v ? a.v + j * a.nbv1 + h * a.nbv2 + b * a.nbv3
                            : a.k + j * a.nbk1 + h * a.nbk2 + b * a.nbk3;
    float f[8];
    const char * blk = row + (c >> 2) * fattn_block_bytes(is_v ? vtype : ktype);
    switch (is_v ? vtype : ktype) {
        case MI355X_TYPE_F32:
#pragma unroll
            for (int e = 0; e < 8; e++) f[e] = ((const float *)row)[c * 8 + e];
            break;
        case MI355X_TYPE_F16:
#pragma unroll
            for (int e = 0; e < 8; e++) f[e] = h2f_bits(((const uint16_t *)row)[c * 8 + e]);
            break;
        case MI355X_TYPE_Q8_0: dequant8<MI355X_TYPE_Q8_0>(blk, (c & 3) * 8, f); break;
        case MI355X_TYPE_Q4_0: dequant8<MI355X_TYPE_Q4_0>(blk, (c & 3) * 8, f); break;
        case MI355X_TYPE_Q4_1: dequant8<MI355X_TYPE_Q4_1>(blk, (c & 3) * 8, f); break;
        case MI355X_TYPE_Q5_0: dequant8<MI355X_TYPE_Q5_0>(blk, (c & 3) * 8, f); break;
        default:               dequant8<MI355X_TYPE_Q5_1>(blk, (c & 3) * 8, f); break;
    }
    typedef _Float16 h8 __attribute__((ext_vector_type(8)));
    h8 y;
#pragma unroll
    for (int e = 0; e < 8; e++) y[e] = (_Float16)f[e];
    *(h8 *)(dst + ((is_v ? half : 0) + i) * 16) = y;
}

// memset as a kernel: a memset node recorded into a captured graph is what a fill kernel avoids.
// 16-byte stores over the aligned middle, single bytes for the (< 16-byte) head and tail.
__global__ void __launch_bounds__(256) fill_kernel(unsigned char * p, unsigned value, size_t head, size_t n16, size_t tail) {
    typedef unsigned u4 __attribute__((ext_vector_type(4)));
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    const unsigned w = value * 0x01010101u;
    if (i < n16) *(u4 *)(p + head + i * 16) = u4{w, w, w, w};
    if (i < head) p[i] = (unsigned char)value;
    if (i < tail) p[head + n16 * 16 + i] = (unsigned char)value;
}

}  // namespace

int fill_launch(void * ptr, int value, size_t size, hipStream_t stream) {
    if (size == 0) return 0;
    size_t head = (16 - (uintptr_t)ptr % 16) % 16;
    if (head > size) head = size;
    const size_t n16  = (size - head) / 16;
    const size_t tail = size - head - n16 * 16;
    const size_t threads = n16 > 16 ? n16 : 16;                    // head and tail are below 16 bytes each
    if ((threads + 255) / 256 > 0x7fffffffu) return (int)hipErrorInvalidValue;
    hipLaunchKernelGGL(fill_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, stream,
                       (unsigned char *)ptr, (unsigned)(value & 0xff), head, n16, tail);
    return (int)hipGetLastError();
}

int kv_to_f16_launch(const FattnArgs & a, int ktype, int vtype, void * dst, hipStream_t stream, const F32Rider * rider) {
    F32Rider x;
    memset(&x, 0, sizeof(x));
    if (rider) x = *rider;
    const int64_t n = 2 * (int64_t)(a.D / 8) * a.Nkv * a.Hkv * a.Bk + x.n;
    if (n == 0) return 0;
    if ((n + 255) / 256 > 0x7fffffff) return (int)hipErrorInvalidValue;
    const unsigned g = (unsigned)((n + 255) / 256);
    if (ktype != vtype || a.Dv != a.D) {
        if (rider) return (int)hipErrorInvalidValue;
        hipLaunchKernelGGL(kv_to_f16_mixed_kernel, dim3(g), dim3(256), 0, stream, a, ktype, vtype, (char *)dst);
        return (int)hipGetLastError();
    }
    switch (ktype) {
#define KV16(T) case T: hipLaunchKernelGGL((kv_to_f16_kernel<T>), dim3(g), dim3(256), 0, stream, a, (char *)dst, x); break
        KV16(MI355X_TYPE_F32);
        KV16(MI355X_TYPE_Q8_0);
        KV16(MI355X_TYPE_Q4_0);
        KV16(MI355X_TYPE_Q4_1);
        KV16(MI355X_TYPE_Q5_0);
        KV16(MI355X_TYPE_Q5_1);
#undef KV16
        default: return (int)hipErrorInvalidValue;
    }
    return (int)hipGetLastError();
}

static bool vec8_ok(const CpyArgs & a, int stype, int dtype) {
    if (FATTN_IS_BLOCK_TYPE(stype) || FATTN_IS_BLOCK_TYPE(dtype)) return false;
    const int64_t ss = stype == MI355X_TYPE_F32 ? 4 : 2, ds = dtype == MI355X_TYPE_F32 ? 4 : 2;
    if (a.sne[0] % 8 || a.dne[0] % 8 || a.snb[0] != ss || a.dnb[0] != ds) return false;
    if (((uintptr_t)a.src % (8 * ss)) || ((uintptr_t)a.dst % (8 * ds))) return false;
    for (int i = 1; i < 4; i++) {
        if ((a.sne[i] > 1 && a.snb[i] % (8 * ss)) || (a.dne[i] > 1 && a.dnb[i] % (8 * ds))) return false;
    }
    return true;
}

int cpy_launch(const CpyArgs & a, int stype, int dtype, hipStream_t stream) {
    if (a.n == 0) return 0;
    if (vec8_ok(a, stype, dtype)) {
        CpyArgs v = a;
        v.n = a.n / 8;
        const unsigned g = (unsigned)((v.n + 255) / 256);
        if (stype == MI355X_TYPE_F32 && dtype == MI355X_TYPE_F32)      hipLaunchKernelGGL((cpy_vec8_kernel<float, float>), dim3(g), dim3(256), 0, stream, v);
        else if (stype == MI355X_TYPE_F32 && dtype == MI355X_TYPE_F16) hipLaunchKernelGGL((cpy_vec8_kernel<float, _Float16>), dim3(g), dim3(256), 0, stream, v);
        else if (stype == MI355X_TYPE_F16 && dtype == MI355X_TYPE_F16) hipLaunchKernelGGL((cpy_vec8_kernel<_Float16, _Float16>), dim3(g), dim3(256), 0, stream, v);
        else                                                          hipLaunchKernelGGL((cpy_vec8_kernel<_Float16, float>), dim3(g), dim3(256), 0, stream, v);
        return (int)hipGetLastError();
    }
    const unsigned g256 = (unsigned)((a.n + 255) / 256);
    const unsigned g8   = (unsigned)((a.n + 7) / 8);
    if (stype == MI355X_TYPE_F32 && dtype == MI355X_TYPE_F32)
        hipLaunchKernelGGL((cpy_scalar_kernel<float, float>), dim3(g256), dim3(256), 0, stream, a);
    else if (stype == MI355X_TYPE_F32 && dtype == MI355X_TYPE_F16)
        hipLaunchKernelGGL((cpy_scalar_kernel<float, _Float16>), dim3(g256), dim3(256), 0, stream, a);
    else if (stype == MI355X_TYPE_F16 && dtype == MI355X_TYPE_F16)
        hipLaunchKernelGGL((cpy_scalar_kernel<_Float16, _Float16>), dim3(g256), dim3(256), 0, stream, a);
    else if (stype == MI355X_TYPE_F16 && dtype == MI355X_TYPE_F32)
        hipLaunchKernelGGL((cpy_scalar_kernel<_Float16, float>), dim3(g256), dim3(256), 0, stream, a);
#define BLOCK_CASES(T)                                                                                                    \
    else if (stype == MI355X_TYPE_F32 && dtype == T)                                                                       \
        hipLaunchKernelGGL((cpy_f32_block_kernel<T>), dim3(g8), dim3(256), 0, stream, a);                                 \
    else if (stype == T && dtype == MI355X_TYPE_F32)                                                                       \
        hipLaunchKernelGGL((cpy_block_f32_kernel<T>), dim3((unsigned)((a.n * 4 + 255) / 256)), dim3(256), 0, stream, a);  \
    else if (stype == T && dtype == T)                                                                                     \
        hipLaunchKernelGGL((cpy_block_block_kernel<T>), dim3((unsigned)((a.n * (BlockFormat<T>::BYTES / 2) + 255) / 256)), dim3(256), 0, stream, a);
    BLOCK_CASES(MI355X_TYPE_Q8_0)
    BLOCK_CASES(MI355X_TYPE_Q4_0)
    BLOCK_CASES(MI355X_TYPE_Q4_1)
    BLOCK_CASES(MI355X_TYPE_Q5_0)
    BLOCK_CASES(MI355X_TYPE_Q5_1)
#undef BLOCK_CASES
    else
        return (int)hipErrorInvalidValue;
    return (int)hipGetLastError();
}

int set_rows_launch(const CpyArgs & a, int dtype, hipStream_t stream) {
    if (a.n == 0) return 0;
    if (a.n > ((int64_t)1 << 38)) return (int)hipErrorInvalidValue;
    const dim3 gb((unsigned)((a.n + 7) / 8));
    if (dtype == MI355X_TYPE_Q8_0)      hipLaunchKernelGGL((set_rows_kernel<MI355X_TYPE_Q8_0>), gb, dim3(256), 0, stream, a);
    else if (dtype == MI355X_TYPE_Q4_0) hipLaunchKernelGGL((set_rows_kernel<MI355X_TYPE_Q4_0>), gb, dim3(256), 0, stream, a);
    else if (dtype == MI355X_TYPE_Q4_1) hipLaunchKernelGGL((set_rows_kernel<MI355X_TYPE_Q4_1>), gb, dim3(256), 0, stream, a);
    else if (dtype == MI355X_TYPE_Q5_0) hipLaunchKernelGGL((set_rows_kernel<MI355X_TYPE_Q5_0>), gb, dim3(256), 0, stream, a);
    else if (dtype == MI355X_TYPE_Q5_1) hipLaunchKernelGGL((set_rows_kernel<MI355X_TYPE_Q5_1>), gb, dim3(256), 0, stream, a);
    else if (dtype == MI355X_TYPE_F16)
        hipLaunchKernelGGL((set_rows_kernel<MI355X_TYPE_F16>), dim3((unsigned)((a.n + 255) / 256)), dim3(256), 0, stream, a);
    else if (dtype == MI355X_TYPE_F32)
        hipLaunchKernelGGL((set_rows_kernel<MI355X_TYPE_F32>), dim3((unsigned)((a.n + 255) / 256)), dim3(256), 0, stream, a);
    else
        return (int)hipErrorInvalidValue;
    return (int)hipGetLastError();
}
