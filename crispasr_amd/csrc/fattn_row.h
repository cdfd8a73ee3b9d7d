// One query row of GGML_OP_FLASH_ATTN_EXT with the CPU op's exact rule for excluded keys: a key whose mask value is
// -inf is skipped, so that neither its K nor its V bytes reach any arithmetic (ggml-cpu: "if (mv == -INFINITY) continue").
// The reference depends on that: cache slots that were never written are masked out, not cleared
// (src/core/attention.h:680-683, fixed_kv_len; src/voxtral.cpp:1137-1145 allocates its cache without clearing it).
//
// The vector kernel is built on this loop.  The MFMA kernels multiply excluded keys by a probability of exactly zero
// instead, which gives the same result for every finite K/V and a non-finite one otherwise (0 * NaN, 0 * inf, or a
// score of inf - inf); they look at their result before they store it and send the rows that came out non-finite
// through attn_row_redo below: the same row again, by this loop.
#pragma once

#include "fattn_common.h"

// 8 consecutive elements of a K/V row starting at element d0, as f32 (exact for all types); of a row that ends inside
// them (head sizes that are multiples of 4 only: aligned16 is false then) the first nvalid, zeros behind
template <int TYPE>
static __device__ __forceinline__ void row_load8(const char * row, int d0, bool aligned16, int nvalid, float (&out)[8]) {
    if constexpr (TYPE == MI355X_TYPE_F16) {
        const char * p = row + (size_t)d0 * 2;
        if (aligned16) {
            const uint4 u = *(const uint4 *)p;
            const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
            for (int i = 0; i < 4; i++) {
                out[2 * i]     = h2f_bits((uint16_t)(w[i] & 0xffffu));
                out[2 * i + 1] = h2f_bits((uint16_t)(w[i] >> 16));
            }
        } else {
            const uint16_t * h = (const uint16_t *)p;
#pragma unroll
            for (int i = 0; i < 8; i++) out[i] = i < nvalid ? h2f_bits(h[i]) : 0.0f;
        }
    } else if constexpr (TYPE == MI355X_TYPE_F32) {
        const char * p = row + (size_t)d0 * 4;
        if (aligned16) {
            const float4 a = *(const float4 *)p;
            const float4 b = *(const float4 *)(p + 16);
            out[0] = a.x; out[1] = a.y; out[2] = a.z; out[3] = a.w;
            out[4] = b.x; out[5] = b.y; out[6] = b.z; out[7] = b.w;
        } else {
            const float * f = (const float *)p;
#pragma unroll
            for (int i = 0; i < 8; i++) out[i] = i < nvalid ? f[i] : 0.0f;
        }
    } else {  // block-32 types: blocks are only 2-byte aligned
        dequant8<TYPE>(row + (size_t)(d0 / FATTN_QK8_0) * fattn_block_bytes(TYPE), d0 % FATTN_QK8_0, out);
    }
}

// online-softmax state of the lanes that share 8 elements of d: running maximum, sum, unnormalised accumulators
struct RowPartial {
    float m, l;
    float acc[8];
};

static __device__ __forceinline__ void row_partial_merge(RowPartial & a, const RowPartial & b) {
    const float mn = fmaxf(a.m, b.m);
    // a state that has seen no key has m = -inf and l = 0: its factor must be 0, not NaN
    const float fa = a.m == -INFINITY ? 0.0f : __expf(a.m - mn);
    const float fb = b.m == -INFINITY ? 0.0f : __expf(b.m - mn);
    a.l = a.l * fa + b.l * fb;
#pragma unroll
    for (int e = 0; e < 8; e++) a.acc[e] = a.acc[e] * fa + b.acc[e] * fb;
    a.m = mn;
}

constexpr int ROW_UNROLL = 4;

// what the loop below needs to know about a call
struct RowScanArgs {
    int32_t D;
    float   scale, softcap;    // scale already divided by the soft cap when that is non-zero
    int64_t nbk1, nbv1;        // row pitches of K and V in bytes
    bool    aligned16;         // K and V rows may be read with 128-bit loads
};
static __device__ __forceinline__ RowScanArgs row_scan_args(const FattnArgs & a) {
    RowScanArgs r;
    r.D = a.Dv; r.scale = a.scale; r.softcap = a.softcap; r.nbk1 = a.nbk1; r.nbv1 = a.nbv1;
    r.aligned16 = a.aligned16 != 0 && a.Dv % 8 == 0;       // (a 16-byte load of a row's last 4 elements would run past the row)
    return r;
}

// The additive mask of one (query, head, batch) as a tensor row: F16 values times the head's ALiBi slope.
struct RowMaskTensor {
    const uint16_t * row;      // nullptr: no mask
    float            slope;
    __device__ __forceinline__ bool present() const { return row != nullptr; }
    // value added to key j's score; every lane of a group calls this with the same j
    __device__ __forceinline__ float operator()(int j) const { return slope * h2f_bits(row[j]); }
};

// Keys [k_begin, k_end) of one row, visited by NWAVES waves: a K or V row is spread over LPR lanes (8 elements each), so a
// wave takes 64 / LPR rows per load; every group of LPR lanes keeps its own state over the keys it visits.  q holds the
// lane's 8 query elements (zeros where d0 is past D).  All 64 lanes must be active (DPP reductions).
template <int TYPE_K, int TYPE_V, int LPR, int NWAVES, typename MaskFn>
static __device__ __forceinline__ void row_scan(const RowScanArgs & a, const float (&q)[8], const char * kbase, const char * vbase,
                                                const MaskFn & mask_at, int k_begin, int k_end, int wave, int lane, RowPartial & st) {
    constexpr int G = 64 / LPR;                 // key rows per wave per load
    const int  grp    = lane / LPR;
    const int  d0     = (lane % LPR) * 8;
    const int  d0c    = d0 < a.D ? d0 : 0;
    const int  nv     = a.D - d0c;               // 8 or more, but for the last lane of a head size that is 4 modulo 8
    const bool al     = a.aligned16;
    const int  stride = NWAVES * G * ROW_UNROLL;
    // every lane runs the same trip count so that the DPP reductions see full groups
    for (int j0 = k_begin; j0 < k_end; j0 += stride) {
        float kf[ROW_UNROLL][8];
        float vf[ROW_UNROLL][8];
        float s[ROW_UNROLL];
        bool  ex[ROW_UNROLL];
        int   jj[ROW_UNROLL];
#pragma unroll
        for (int u = 0; u < ROW_UNROLL; u++) {
            jj[u] = j0 + (u * NWAVES + wave) * G + grp;
            const int jc = min(jj[u], k_end - 1);
            row_load8<TYPE_K>(kbase + (size_t)jc * a.nbk1, d0c, al, nv, kf[u]);
        }
#pragma unroll
        for (int u = 0; u < ROW_UNROLL; u++) {
            const int jc = min(jj[u], k_end - 1);
            row_load8<TYPE_V>(vbase + (size_t)jc * a.nbv1, d0c, al, nv, vf[u]);
        }
        float mloc = -INFINITY;
#pragma unroll
        for (int u = 0; u < ROW_UNROLL; u++) {
            float dot = 0.0f;
#pragma unroll
            for (int e = 0; e < 8; e++) dot = fmaf(q[e], kf[u][e], dot);
            dot = group_sum<LPR>(dot);
            float sc = dot * a.scale;
            if (a.softcap != 0.0f) sc = a.softcap * tanhf(sc);
            ex[u] = jj[u] >= k_end;
            if (mask_at.present()) {
                const float mv = mask_at(min(jj[u], k_end - 1));
                ex[u] = ex[u] || mv == -INFINITY;
                sc += mv;
            }
            // an excluded key is not looked at: whatever its K row made of the score, it is replaced, not added to
            s[u] = ex[u] ? -INFINITY : sc;
            // (a visible key with a NaN score makes the row NaN, as it does on the CPU: the maximum must not ignore it)
            mloc = fmaxf(mloc, s[u] == s[u] ? s[u] : INFINITY);
        }
        if (mloc > st.m) {                       // uniform within a group
            const float alpha = __expf(st.m - mloc);   // exp(-inf) = 0 on the first hit
            st.l *= alpha;
#pragma unroll
            for (int e = 0; e < 8; e++) st.acc[e] *= alpha;
            st.m = mloc;
        }
        if (st.m > -INFINITY) {
#pragma unroll
            for (int u = 0; u < ROW_UNROLL; u++) {
                if (ex[u]) continue;             // nor is its V row: 0 * NaN would not be 0
                const float p = __expf(s[u] - st.m);
                st.l += p;
#pragma unroll
                for (int e = 0; e < 8; e++) st.acc[e] = fmaf(p, vf[u][e], st.acc[e]);
            }
        }
    }
    // merge the G groups of this wave (lanes with equal position in their group)
#pragma unroll
    for (int off = LPR; off < 64; off <<= 1) {
        RowPartial o;
        o.m = xor_shuffle(st.m, off);
        o.l = xor_shuffle(st.l, off);
#pragma unroll
        for (int e = 0; e < 8; e++) o.acc[e] = xor_shuffle(st.acc[e], off);
        row_partial_merge(st, o);
    }
}

// lanes 0 .. LPR-1 hold the row's final state: write dst, or this split's partial for the merge (natural-log units).
// COHERENT: the partial goes out by device-coherent stores, for a merge by another workgroup of the same launch.
template <int LPR, bool COHERENT = false>
static __device__ __forceinline__ void row_store(const FattnArgs & a, const RowPartial & st, int64_t row, int split, int lane) {
    const int d0 = lane * 8;
    if (lane >= LPR || d0 >= a.Dv) return;           // (Dv < D: a head zero-padded to D; partial rows are D apart, dst rows Dv)
    if (a.n_splits == 1) {
        const float inv = st.l > 0.0f ? 1.0f / st.l : (st.l == st.l ? 0.0f : st.l);      // a NaN sum stays NaN, as on the CPU
        float * out = a.dst + row * a.Dv + d0;
#pragma unroll
        for (int e = 0; e < 8; e++)
            if (e < 4 || d0 + e < a.Dv) out[e] = st.acc[e] * inv;       // (the head size is a multiple of 4)
    } else {
        float * pa = a.part_acc + (row * a.n_splits + split) * a.D + d0;
#pragma unroll
        for (int e = 0; e < 8; e++)
            if (e < 4 || d0 + e < a.D) {
                if (COHERENT) device_store(pa + e, st.acc[e]);
                else          pa[e] = st.acc[e];
            }
        if (lane == 0) {
            float * pm = a.part_ml + (row * a.n_splits + split) * 2;
            if (COHERENT) {
                device_store(pm, st.m);
                device_store(pm + 1, st.l);
            } else {
                pm[0] = st.m;
                pm[1] = st.l;
            }
        }
    }
}

// The whole of one row by one wave: what an MFMA kernel calls, with every lane of the wave active, for a row whose result
// came out non-finite.  Writes what that kernel would have written for (row, split).
template <int TYPE, int D>
static __device__ __forceinline__ void attn_row_redo(const FattnArgs & a, int iq1, int h, int b, int split, int k_begin, int k_end) {
    constexpr int LPR = D / 8;
    const int lane = threadIdx.x & 63;
    const int d0   = (lane % LPR) * 8;
    float q[8];
    {
        const float * qrow = (const float *)(a.q + (int64_t)iq1 * a.nbq1 + (int64_t)h * a.nbq2 + (int64_t)b * a.nbq3);
#pragma unroll
        for (int e = 0; e < 8; e++) q[e] = d0 + e < a.Dv ? qrow[d0 + e] : 0.0f;      // (zero-padded head: Dv < D)
    }
    const int hk = h / a.gqa, bk = b / a.bq;
    RowMaskTensor mask;
    mask.row   = a.mask ? (const uint16_t *)(a.mask + (int64_t)iq1 * a.nbm1 + (int64_t)(h % a.Hm) * a.nbm2 + (int64_t)(b % a.Bm) * a.nbm3) : nullptr;
    mask.slope = fattn_slope(a, h);
    RowPartial st;
    st.m = -INFINITY;
    st.l = 0.0f;
#pragma unroll
    for (int e = 0; e < 8; e++) st.acc[e] = 0.0f;
    row_scan<TYPE, TYPE, LPR, 1>(row_scan_args(a), q, a.k + (int64_t)hk * a.nbk2 + (int64_t)bk * a.nbk3, a.v + (int64_t)hk * a.nbv2 + (int64_t)bk * a.nbv3,
                                 mask, k_begin, k_end, 0, lane, st);
    row_store<LPR>(a, st, ((int64_t)b * a.Nq + iq1) * a.Hq + h, split, lane);
}

// true when x is NaN or +-inf
static __device__ __forceinline__ bool not_finite(float x) { return !(fabsf(x) < INFINITY); }

// The mask of FastConformer's relative-position attention for one query, computed as it is needed:
// f16(scale * <q_v[i], r[Nq-1+j-i]> + add[j, i]) with f16-rounded factors, f32 sum - what fattn_relpos_kernel adds.
template <int LPR>
struct RowMaskRelpos {
    const char * rrow0;        // table row of key 0 for this query (f16, contiguous d)
    int64_t      nbr1;
    const char * addrow;       // this query's row of the additive mask, or nullptr
    bool         add_f16;
    float        scale;
    float        qv[8];        // the lane's 8 elements of q_v, rounded to f16
    int          d0;
    __device__ __forceinline__ bool present() const { return true; }
    __device__ __forceinline__ float operator()(int j) const {
        float r[8];
        row_load8<MI355X_TYPE_F16>(rrow0 + (int64_t)j * nbr1, d0, true, 8, r);
        float dot = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; e++) dot = fmaf(qv[e], r[e], dot);
        dot = group_sum<LPR>(dot);
        float mk = dot * scale;
        if (addrow) mk = mul_then_add(dot, scale, add_f16 ? h2f_bits(((const uint16_t *)addrow)[j]) : ((const float *)addrow)[j]);
        return (float)(_Float16)mk;
    }
};

template <int D>
static __device__ __forceinline__ void attn_row_redo_relpos(const FattnRelposArgs & a, int iq, int h, int b) {
    constexpr int LPR = D / 8;
    const int lane = threadIdx.x & 63;
    const int d0   = (lane % LPR) * 8;
    float q[8];
    RowMaskRelpos<LPR> mask;
    {
        const float * pu = (const float *)(a.qu + (int64_t)iq * a.nbu1 + (int64_t)h * a.nbu2 + (int64_t)b * a.nbu3);
        const float * pv = (const float *)(a.qv + (int64_t)iq * a.nbw1 + (int64_t)h * a.nbw2 + (int64_t)b * a.nbw3);
#pragma unroll
        for (int e = 0; e < 8; e++) {
            q[e] = pu[d0 + e];
            mask.qv[e] = (float)(_Float16)pv[d0 + e];
        }
    }
    mask.rrow0   = a.r + (int64_t)(h % a.Hr) * a.nbr2 + (int64_t)(b % a.Br) * a.nbr3 + (int64_t)(a.Nq - 1 - iq) * a.nbr1;
    mask.nbr1    = a.nbr1;
    mask.addrow  = a.add ? a.add + (int64_t)iq * a.nba1 + (int64_t)(h % a.Ha) * a.nba2 + (int64_t)(b % a.Ba) * a.nba3 : nullptr;
    mask.add_f16 = a.add_f16 != 0;
    mask.scale   = a.scale;
    mask.d0      = d0;
    RowScanArgs r;
    r.D = D; r.scale = a.scale; r.softcap = 0.0f; r.nbk1 = a.nbk1; r.nbv1 = a.nbv1; r.aligned16 = true;
    RowPartial st;
    st.m = -INFINITY;
    st.l = 0.0f;
#pragma unroll
    for (int e = 0; e < 8; e++) st.acc[e] = 0.0f;
    const int hk = h / a.gqa, bk = b / a.bq;
    row_scan<MI355X_TYPE_F16, MI355X_TYPE_F16, LPR, 1>(r, q, a.k + (int64_t)hk * a.nbk2 + (int64_t)bk * a.nbk3,
                                                       a.v + (int64_t)hk * a.nbv2 + (int64_t)bk * a.nbv3, mask, 0, a.Nkv, 0, lane, st);
    if (lane < LPR) {
        const float inv = st.l > 0.0f ? 1.0f / st.l : (st.l == st.l ? 0.0f : st.l);
        float * out = a.dst + (((int64_t)b * a.Nq + iq) * a.H + h) * D + d0;
#pragma unroll
        for (int e = 0; e < 8; e++) out[e] = st.acc[e] * inv;
    }
}
