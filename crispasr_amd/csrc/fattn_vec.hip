// Split-KV vector attention kernel for gfx950 (wave64) and the merge of its partials.
//
// One workgroup (4 waves) owns one query row (query, head, batch) and one KV split.
// A row of K or V is spread over LPR lanes, 8 elements (one 128-bit load for f16) per
// lane, so a wave reads 64/LPR whole rows per load instruction - contiguous 128- or
// 256-byte segments.  Each group of LPR lanes keeps its own online-softmax state
// (m, l, acc[8] per lane) over the keys it visits; the dot products are reduced across
// the group with DPP butterflies.  Groups are merged with cross-lane shuffles, waves
// through LDS, and splits by fattn_merge_kernel.
//
// Semantics follow GGML_OP_FLASH_ATTN_EXT as the reference's call sites use it
// (src/crispasr.cpp:3208-3222, 3269-3282; src/core/attention.h:992; src/canary.cpp:966-972):
// s = scale*<q,k> [soft-capped] + slope*mask, -inf mask entries exclude a key, GQA by
// h / (Hq/Hkv), mask broadcast by h % Hm and b % Bm, output [D, Hq, Nq, B].
#include "fattn_row.h"

namespace {

constexpr int VEC_WAVES   = 4;
constexpr int VEC_THREADS = VEC_WAVES * 64;

template <int TYPE, int LPR>
__global__ void __launch_bounds__(VEC_THREADS) fattn_vec_kernel(const FattnArgs a) {
    const int tid  = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int d0   = (lane % LPR) * 8;          // the lane's 8 elements of d (D is a multiple of 4: the last lane may hold 4)

    // blockIdx.x = row * n_splits + split, row = (b*Nq + iq1)*Hq + h  (the dst row order)
    const int split = blockIdx.x % a.n_splits;
    const int row   = blockIdx.x / a.n_splits;
    const int h     = row % a.Hq;
    const int iq1   = (row / a.Hq) % a.Nq;
    const int b     = row / (a.Hq * a.Nq);
    const int hk    = h / a.gqa;
    const int bk    = b / a.bq;

    const int k_begin = split * a.keys_per_split;
    const int k_end   = min(a.Nkv, k_begin + a.keys_per_split);

    float q[8];
    {
        const float * qrow = (const float *)(a.q + iq1 * a.nbq1 + h * a.nbq2 + b * a.nbq3);
#pragma unroll
        for (int e = 0; e < 8; e++) q[e] = d0 + e < a.D ? qrow[d0 + e] : 0.0f;
    }
    const char * kbase = a.k + hk * a.nbk2 + bk * a.nbk3;
    const char * vbase = a.v + hk * a.nbv2 + bk * a.nbv3;
    RowMaskTensor mask;
    mask.row   = a.mask ? (const uint16_t *)(a.mask + iq1 * a.nbm1 + (h % a.Hm) * a.nbm2 + (b % a.Bm) * a.nbm3) : nullptr;
    mask.slope = fattn_slope(a, h);

    RowPartial st;
    st.m = -INFINITY;
    st.l = 0.0f;
#pragma unroll
    for (int e = 0; e < 8; e++) st.acc[e] = 0.0f;
    row_scan<TYPE, TYPE, LPR, VEC_WAVES>(row_scan_args(a), q, kbase, vbase, mask, k_begin, k_end, wave, lane, st);

    // merge the waves through LDS
    __shared__ float sh[VEC_WAVES][LPR][10];
    if (lane < LPR) {
        sh[wave][lane][0] = st.m;
        sh[wave][lane][1] = st.l;
#pragma unroll
        for (int e = 0; e < 8; e++) sh[wave][lane][2 + e] = st.acc[e];
    }
    __syncthreads();
    if (wave == 0 && lane < LPR) {
#pragma unroll
        for (int w = 1; w < VEC_WAVES; w++) {
            RowPartial o;
            o.m = sh[w][lane][0];
            o.l = sh[w][lane][1];
#pragma unroll
            for (int e = 0; e < 8; e++) o.acc[e] = sh[w][lane][2 + e];
            row_partial_merge(st, o);
        }
        if (a.counters) row_store<LPR, true>(a, st, row, split, lane);
        else            row_store<LPR>(a, st, row, split, lane);
    }
    // the last of the row's n_splits workgroups merges them: no launch for the merge
    if (a.n_splits > 1 && a.counters) {
        __shared__ int last;
        if (fattn_last_of_set(a, row, a.n_splits, &last, false) && tid < a.D / 4) fattn_merge_row<true>(a, row, tid);
    }
}

// One row per D/4 lanes (a float4 of d each), 64 / (D/4) rows per wave.
__global__ void __launch_bounds__(256) fattn_merge_kernel(const FattnArgs a, int rows) {
    const int lpr  = a.D / 4;                       // lanes per row
    const int rpw  = 64 / lpr;                      // rows per wave
    const int lane = threadIdx.x & 63;
    const int wave = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int row  = wave * rpw + lane / lpr;
    if (lane >= rpw * lpr || row >= rows) return;
    fattn_merge_row<false>(a, row, lane % lpr);
}

template <int TYPE>
int launch_typed(const FattnArgs & a, hipStream_t stream) {
    const int64_t rows = (int64_t)a.Nq * a.Hq * a.B;
    if (rows * a.n_splits > 0x7fffffff) return (int)hipErrorInvalidValue;      // one workgroup per (row, split)
    const dim3 grid((unsigned)(rows * a.n_splits));
    const dim3 block(VEC_THREADS);
    const int  lanes = (a.D + 7) / 8;
    if (lanes <= 4)       hipLaunchKernelGGL((fattn_vec_kernel<TYPE, 4>),  grid, block, 0, stream, a);
    else if (lanes <= 8)  hipLaunchKernelGGL((fattn_vec_kernel<TYPE, 8>),  grid, block, 0, stream, a);
    else if (lanes <= 16) hipLaunchKernelGGL((fattn_vec_kernel<TYPE, 16>), grid, block, 0, stream, a);
    else                  hipLaunchKernelGGL((fattn_vec_kernel<TYPE, 32>), grid, block, 0, stream, a);
    return (int)hipGetLastError();
}

}  // namespace

int fattn_vec_launch(const FattnArgs & a, int ktype, hipStream_t stream) {
    switch (ktype) {
        case MI355X_TYPE_F16:  return launch_typed<MI355X_TYPE_F16>(a, stream);
        case MI355X_TYPE_F32:  return launch_typed<MI355X_TYPE_F32>(a, stream);
        case MI355X_TYPE_Q8_0: return launch_typed<MI355X_TYPE_Q8_0>(a, stream);
        case MI355X_TYPE_Q4_0: return launch_typed<MI355X_TYPE_Q4_0>(a, stream);
        case MI355X_TYPE_Q4_1: return launch_typed<MI355X_TYPE_Q4_1>(a, stream);
        case MI355X_TYPE_Q5_0: return launch_typed<MI355X_TYPE_Q5_0>(a, stream);
        case MI355X_TYPE_Q5_1: return launch_typed<MI355X_TYPE_Q5_1>(a, stream);
        default:               return (int)hipErrorInvalidValue;
    }
}

int fattn_merge_launch(const FattnArgs & a, hipStream_t stream) {
    const int rows = a.Nq * a.Hq * a.B;
    const int rows_per_block = 4 * (64 / (a.D / 4));          // D is a multiple of 8, at most 256
    const dim3 grid((unsigned)((rows + rows_per_block - 1) / rows_per_block));
    hipLaunchKernelGGL(fattn_merge_kernel, grid, dim3(256), 0, stream, a, rows);
    return (int)hipGetLastError();
}
