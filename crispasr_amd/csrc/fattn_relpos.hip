// FastConformer's relative-position attention in one kernel (the flash branch of core_conformer::build_block,
// src/core/fastconformer.h:876-934):
//
//   dst[:, h, i, b] = softmax_j( scale * <q_u[i], k[j]> + mask[j, i] ) . v[j]
//   mask[j, i]      = f16( scale * <q_v[i], r[Nq-1+j-i]> + add[j, i] )         (the graph's rel_shift view, scale, add, cast)
//
// The reference materialises `mask` as an F16 [T, T, H] tensor per sequence and hands it to ggml_flash_attn_ext; here
// the position term is produced tile by tile inside the attention loop and never leaves the CU.
//
// A workgroup of 4 waves owns 128 consecutive queries of one (head, batch), 32 per wave (the N columns of
// v_mfma_f32_32x32x16_f16 accumulators), and walks the keys 32 at a time.  Per step and wave:
//   S^T  = K tile . Q_u^T                       8 (D = 128) MFMAs, A = K rows from LDS, B = Q_u in registers
//   BD   = R block . Q_v^T                      8 MFMAs, A = 32 rows of the table from LDS, B = Q_v in registers.
//          Block n x the wave's 32 queries is one accumulator whose element (row, il) belongs to key
//          j = 32 n + row + il - 31: tile t is the lower-right triangle (row + il >= 31) of block t and the upper-left
//          one of block t + 1, and for one accumulator slot exactly one of the two owns the slot's place in the tile -
//          so the previous block stays in registers, one new block is computed per step and a select per slot gives
//          the tile, each product computed once.
//   un-skew: the selected values sit at key (row + il + 1) mod 32 of their query; they go through a wave-private
//          32 x 32 f32 square in LDS (pitch 36: writes and the 16-byte row reads are both conflict-free) and come back
//          in the layout of S^T.
//   mask = f16(scale * BD + add), s = S + mask in log2 units, online softmax against a reference that is raised
//          only when a row's maximum outgrows it by a factor 256, P -> f16
//   O^T += V^T . P^T                            8 MFMAs, A = V tile through ds_read_b64_tr_b16, B = P from registers
// The four waves need the same table rows one step apart, so the table is staged once per workgroup in a ring of five
// 32-row blocks.  K tiles and table blocks move global -> LDS without passing registers (global_load_lds_dwordx4, the
// 16-byte chunks of a row XOR-swizzled so that the operand reads are conflict-free), requested behind the first barrier
// of a step and waited for before the second; V is fetched one step ahead into registers and written behind the second.  K, V and the table are f16 with 16-byte aligned rows (the caller rounds F32 ones first, as
// the reference's own graph does for the mask product's operands).
#include "fattn_row.h"

#include <stdlib.h>
#include <type_traits>

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float    float2v __attribute__((ext_vector_type(2)));
typedef float    float16v __attribute__((ext_vector_type(16)));
typedef float    float4v __attribute__((ext_vector_type(4)));
typedef short    short4v __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float    float4_a4 __attribute__((ext_vector_type(4), aligned(4)));
typedef _Float16 half4_a2 __attribute__((ext_vector_type(4), aligned(2)));

constexpr int   FR_SQP   = 36;                      // pitch of the un-skew square in floats
constexpr float FR_LOG2E = 1.4426950408889634f;
constexpr float FR_SUM_LIMIT = 4096.0f;               // a tile's 16 probabilities of a lane sum to at most this before the reference is raised

template <int D> constexpr int fr_kp() { return 2 * D; }          // bytes per K / table row in LDS (chunks swizzled, no padding)
template <int D> __device__ __forceinline__ int fr_swz(int r) { return D == 64 ? (r >> 1) & 7 : r & 15; }
template <int D> __device__ __forceinline__ int fr_swz_v(int r) { return D == 64 ? r & 7 : (r & 3) << 2; }
// K tile, V tile, NW + 1 table blocks (NW in use, one being written), one un-skew square per wave
template <int D, int NW> constexpr int fr_lds_bytes() { return (2 + NW + 1) * 32 * fr_kp<D>() + NW * 32 * FR_SQP * 4; }

template <int D, int NW, bool ADD, bool ADD_F16>
__global__ void __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(2, 2))) fattn_relpos_kernel(const FattnRelposArgs a) {
    constexpr int FR_SLOTS = NW + 1;
    constexpr int KS  = D / 16;                     // reduction steps of the two Q products
    constexpr int DBO = D / 32;                     // 32-wide blocks of the output's d
    constexpr int CH  = D / 8;                      // 16-byte chunks per row
    constexpr int KP  = fr_kp<D>();

    extern __shared__ __attribute__((aligned(16))) char fr_lds[];
    char * const kt   = fr_lds;
    char * const vt   = kt + 32 * KP;
    char * const ring = vt + 32 * KP;
    const int tid  = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int il   = lane & 31;
    const int hh   = lane >> 5;
    float * const sq = (float *)(ring + FR_SLOTS * 32 * KP) + wave * 32 * FR_SQP;

    // Workgroups go to the 8 XCDs round-robin, each with its own L2: the query blocks of one (head, batch) are given to
    // one XCD, so that K, V and the table rows they share come from that L2.  The head index runs faster than the batch:
    // an XCD holds all heads of few sequences, which share the sequence's additive mask (2 MB at T = 750 in F32; with the
    // batch running faster every XCD fetched every sequence's mask and the call took 5% longer).
    const int     n_qb = (a.Nq + 32 * NW - 1) / (32 * NW);
    const int64_t G    = (int64_t)n_qb * a.H * a.B;
    const int64_t per  = (G + 7) / 8;
    const int64_t L    = (int64_t)(blockIdx.x & 7) * per + (blockIdx.x >> 3);
    if ((blockIdx.x >> 3) >= per || L >= G) return;
    const int qb = (int)(L % n_qb);
    const int h  = (int)((L / n_qb) % a.H);
    const int b  = (int)(L / ((int64_t)n_qb * a.H));
    const int hk = h / a.gqa, bk = b / a.bq;

    const int q0  = qb * 32 * NW;
    const int i0w = q0 + wave * 32;
    const int iq  = min(i0w + il, a.Nq - 1);        // rows past Nq repeat the last one and are not stored
    const int NT  = (a.Nkv + 31) / 32;
    const int NR  = a.Nq + a.Nkv - 1;
    const int p_base0 = a.Nq - 1 - q0 - 31;         // table row of (block 0, row 0) in wave 0's numbering; wave w's block n is block n - w

    const char * kbase = a.k + (int64_t)hk * a.nbk2 + (int64_t)bk * a.nbk3;
    const char * vbase = a.v + (int64_t)hk * a.nbv2 + (int64_t)bk * a.nbv3;
    const char * rbase = a.r + (int64_t)(h % a.Hr) * a.nbr2 + (int64_t)(b % a.Br) * a.nbr3;

    // ---- staging ------------------------------------------------------------------------------------------------
    // K tiles and table blocks: each wave moves its quarter, 64 x 16 bytes per instruction; LDS slot
    // L = (wave * NDM + j) * 64 + lane holds chunk (L % CH) ^ swizzle of row L / CH.  Rows that stick out (the last key
    // tile, the ends of the table) repeat the nearest valid row: they belong to excluded keys or to no key at all.
    constexpr int TI  = 32 * CH * 16 / 1024;                  // 64-lane instructions per tile
    constexpr int NDM = (TI + NW - 1) / NW;                   // ... per wave: instruction j of wave w is number j * NW + w
    typedef __attribute__((address_space(3))) void * lds_vptr;
    typedef const __attribute__((address_space(1))) void * glb_vptr;
    auto dma_rows = [&](char * dst, const char * base, int64_t nb1, int row0, int last_row, auto is_v) __attribute__((always_inline)) {
        const bool inside = row0 >= 0 && row0 + 31 <= last_row;      // uniform
        const char * p = base + (int64_t)(inside ? row0 : 0) * nb1;
#pragma unroll
        for (int j = 0; j < NDM; j++) {
            const int ins = j * NW + wave;                            // uniform
            if (TI % NW != 0 && ins >= TI) break;
            const int L = ins * 64 + lane, r = L / CH;
            const int c = (L % CH) ^ (decltype(is_v)::value ? fr_swz_v<D>(r) : fr_swz<D>(r));
            const int rr = inside ? r : min(max(row0 + r, 0), last_row);
            __builtin_amdgcn_global_load_lds((glb_vptr)(p + ((uint32_t)rr * (uint32_t)nb1 + (uint32_t)c * 16u)),
                                             (lds_vptr)(dst + ins * 1024), 16, 0, 0);
        }
    };
    typedef std::integral_constant<bool, false> KLayout;
    typedef std::integral_constant<bool, true>  VLayout;
    auto dma_k = [&](int t) __attribute__((always_inline)) { dma_rows(kt, kbase, a.nbk1, 32 * t, a.Nkv - 1, KLayout{}); };
    auto dma_v = [&](int t) __attribute__((always_inline)) { dma_rows(vt, vbase, a.nbv1, 32 * t, a.Nkv - 1, VLayout{}); };
    auto slot_of = [&](int beta) { return ring + ((beta + NW - 1) % FR_SLOTS) * 32 * KP; };   // beta >= 1 - NW
    auto dma_r = [&](int beta) __attribute__((always_inline)) { dma_rows(slot_of(beta), rbase, a.nbr1, p_base0 + 32 * beta, NR - 1, KLayout{}); };

    // ---- prologue: table blocks 1 - NW .. 1, the first K and V tiles, Q_u and Q_v as B operands ---------------------
#pragma unroll 1
    for (int beta = 1 - NW; beta <= 1; beta++) dma_r(beta);
    dma_k(0);
    dma_v(0);
    half8 qu[KS], qv[KS];
    {
        const float * pu = (const float *)(a.qu + (int64_t)iq * a.nbu1 + (int64_t)h * a.nbu2 + (int64_t)b * a.nbu3);
        const float * pv = (const float *)(a.qv + (int64_t)iq * a.nbw1 + (int64_t)h * a.nbw2 + (int64_t)b * a.nbw3);
        const float   qs = a.scale * FR_LOG2E;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            const float4v u0 = *(const float4v *)(pu + ks * 16 + hh * 8), u1 = *(const float4v *)(pu + ks * 16 + hh * 8 + 4);
            const float4v w0 = *(const float4v *)(pv + ks * 16 + hh * 8), w1 = *(const float4v *)(pv + ks * 16 + hh * 8 + 4);
#pragma unroll
            for (int e = 0; e < 4; e++) {
                qu[ks][e] = (_Float16)(u0[e] * qs); qu[ks][e + 4] = (_Float16)(u1[e] * qs);
                qv[ks][e] = (_Float16)w0[e];        qv[ks][e + 4] = (_Float16)w1[e];
            }
        }
    }
    constexpr int AES = ADD_F16 ? 2 : 4;
    const char * addrow = nullptr;                  // the query's row of the additive mask; addp walks it, 32 keys a step
    if (ADD) addrow = a.add + (int64_t)iq * a.nba1 + (int64_t)(h % a.Ha) * a.nba2 + (int64_t)(b % a.Ba) * a.nba3;
    const char * addp = addrow + 4 * hh * AES;
    // Keys beyond the length of a padded sequence carry -inf in the additive mask for every query: tiles that are masked
    // out entirely at the END of the key range add nothing and are not walked at all.  Each wave looks at its queries'
    // last tile while the first blocks are on their way (that is all an unpadded sequence costs) and, if that one is
    // masked, scans backwards four tiles per round trip; the workgroup takes the largest count.
    int NTL = NT;
    if (ADD) {
        auto tile_max = [&](int tt) __attribute__((always_inline)) {
            float v = -INFINITY;
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int key0 = 32 * tt + 8 * g + 4 * hh;
                if (32 * tt + 32 <= a.Nkv) {
                    if (ADD_F16) {
                        const half4_a2 x = *(const half4_a2 *)(addrow + (int64_t)key0 * 2);
                        v = fmaxf(fmaxf(v, fmaxf((float)x[0], (float)x[1])), fmaxf((float)x[2], (float)x[3]));
                    } else {
                        const float4_a4 x = *(const float4_a4 *)(addrow + (int64_t)key0 * 4);
                        v = fmaxf(fmaxf(v, fmaxf(x[0], x[1])), fmaxf(x[2], x[3]));
                    }
                } else {
#pragma unroll
                    for (int c = 0; c < 4; c++) {
                        const int key = min(key0 + c, a.Nkv - 1);
                        v = fmaxf(v, ADD_F16 ? (float)*(const _Float16 *)(addrow + (int64_t)key * 2) : *(const float *)(addrow + (int64_t)key * 4));
                    }
                }
            }
            return v;
        };
        auto any_live = [&](float v) { return __builtin_amdgcn_ballot_w64(v > -INFINITY || v != v) != 0; };
        int live = NT;
        if (!any_live(tile_max(NT - 1))) {
            live = NT - 1;
            while (live > 0) {
                const int t0 = max(live - 4, 0);
                float mx[4];
#pragma unroll
                for (int u = 0; u < 4; u++) mx[u] = tile_max(min(t0 + u, live - 1));
                unsigned bits = 0;
#pragma unroll
                for (int u = 0; u < 4; u++)
                    if (any_live(mx[u])) bits |= 1u << u;
                if (bits) {
                    live = min(t0 + (32 - __builtin_clz(bits)), live);
                    break;
                }
                live = t0;
            }
        }
        // (the four floats behind each row of a square are padding that nothing else writes)
        if (lane == 0) ((int *)(ring + FR_SLOTS * 32 * KP))[32 + wave] = live;
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);               // vmcnt(0): this wave's share of the blocks is in LDS
    __syncthreads();
    if (ADD) {
        NTL = 0;
#pragma unroll
        for (int w = 0; w < NW; w++) NTL = max(NTL, ((const int *)(ring + FR_SLOTS * 32 * KP))[32 + w]);
    }

    // operand reads of a K or table block: lane (il, hh) takes d = 16 ks + 8 hh .. +7 of row il
    uint32_t opaddr[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ks++) opaddr[ks] = (uint32_t)((il * CH + ((ks * 2 + hh) ^ fr_swz<D>(il))) * 16);
    // transposing reads of the V tile: lane j16 of a group of 16 addresses key 4 hh + j16 / 4 (+ 8, + 16 ks) and four
    // values of d from 32 db + 16 (group % 2) + 4 (j16 % 4) on; the swizzle depends on key % 8 only
    uint32_t vaddr[DBO];
    {
        const int j16 = lane & 15, G16 = lane >> 4, kr0 = 4 * (G16 >> 1) + (j16 >> 2);
#pragma unroll
        for (int db = 0; db < DBO; db++) {
            const int c = 4 * db + 2 * (G16 & 1) + ((j16 & 3) >> 1);
            vaddr[db] = (uint32_t)((kr0 * CH + (c ^ fr_swz_v<D>(kr0))) * 16 + 8 * (j16 & 1));
        }
    }

    auto block_times_q = [&](const char * blk, const half8 (&q)[KS]) __attribute__((always_inline)) {
        float16v acc;
#pragma unroll
        for (int r = 0; r < 16; r++) acc[r] = 0.0f;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            const half8 av = *(const half8 *)(blk + opaddr[ks]);
            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(av, q[ks], acc, 0, 0, 0);
        }
        return acc;
    };

    // the wave's block 0 (= block -wave in wave 0's numbering): its lower-right triangle is the first tile's
    float16v bd_prev = block_times_q(slot_of(-wave), qv);

    float16v oacc[DBO];
#pragma unroll
    for (int db = 0; db < DBO; db++)
#pragma unroll
        for (int r = 0; r < 16; r++) oacc[db][r] = 0.0f;
    float m = -INFINITY, l = 0.0f;


    // un-skew constants: slot r of a lane sits at row k_r + 4 hh of its block, i.e. at key (x + k_r) mod 32 with
    // x = il + 4 hh + 1, and belongs to the previous block exactly when that sum reaches 32
    const int x_lane = il + 4 * hh + 1;
    const int sq_new = il * FR_SQP + x_lane, sq_prev = sq_new - 32;

#pragma unroll 1
    for (int t = 0; t < NTL; t++) {
        const bool tail = 32 * t + 32 > a.Nkv;             // uniform
        // the additive mask of this tile: requested first, used after the products.  The values stay as loaded until
        // then (a conversion inside the branch below would have to wait for its load right there, four round trips a step)
        typedef typename std::conditional<ADD_F16, half4_a2, float4_a4>::type araw_t;
        araw_t araw[4];
        if (ADD) {
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int key0 = 32 * t + 8 * g + 4 * hh;
                if (!tail) {
                    araw[g] = *(const araw_t *)(addp + 8 * g * AES);
                } else {
#pragma unroll
                    for (int c = 0; c < 4; c++) {
                        const int key = min(key0 + c, a.Nkv - 1);
                        if constexpr (ADD_F16) araw[g][c] = *(const _Float16 *)(addrow + (int64_t)key * 2);
                        else                   araw[g][c] = *(const float *)(addrow + (int64_t)key * 4);
                    }
                }
            }
        }
        if (ADD) addp += 32 * AES;
        // ---- the position product against this step's table block; select per slot, un-skew through the square ------
        {
            const float16v bd_new = block_times_q(slot_of(t + 1 - wave), qv);
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int  k_r  = 8 * (r >> 2) + (r & 3);
                const bool prev = x_lane + k_r >= 32;
                sq[(prev ? sq_prev : sq_new) + k_r] = prev ? bd_prev[r] : bd_new[r];
            }
            bd_prev = bd_new;
        }
        // ---- the content product against this step's K tile -------------------------------------------------------------
        const float16v s = block_times_q(kt, qu);
        __builtin_amdgcn_s_waitcnt(0x0F70);               // vmcnt(0): this wave's share of the V tile is in LDS
        __syncthreads();                                  // every wave has read the K tile and its table block; the V tile is complete
        if (t + 1 < NTL) {
            dma_k(t + 1);
            dma_r(t + 2);
        }

        // ---- mask = f16(scale * BD + add); scores in log2 units ------------------------------------------------------
        float s2[16];
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const float4v bd = *(const float4v *)&sq[il * FR_SQP + 8 * g + 4 * hh];
#pragma unroll
            for (int c = 0; c < 4; c += 2) {
                float2v mk;
#pragma unroll
                for (int e = 0; e < 2; e++)                    // as the graph: scale, then add
                    mk[e] = ADD ? mul_then_add(bd[c + e], a.scale, (float)araw[g][c + e]) : bd[c + e] * a.scale;
                uint32_t pk;                                   // rounded two at a time (the compiler converts one at a time)
                asm("v_cvt_pk_f16_f32 %0, %1, %2" : "=v"(pk) : "v"(mk[0]), "v"(mk[1]));
                const half2v mh = __builtin_bit_cast(half2v, pk);
#pragma unroll
                for (int e = 0; e < 2; e++) s2[4 * g + c + e] = fmaf((float)mh[e], FR_LOG2E, s[4 * g + c + e]);
            }
        }
        if (tail) {                                        // keys past the end of the last tile
#pragma unroll
            for (int r = 0; r < 16; r++)
                if (32 * t + 8 * (r >> 2) + 4 * hh + (r & 3) >= a.Nkv) s2[r] = -INFINITY;
        }
        __builtin_amdgcn_wave_barrier();

        // ---- online softmax ----------------------------------------------------------------------------------------------
        // P = 2^(s2 - m) in f16 against the row's reference m as it stands; the row sum is taken over the rounded values
        // the MFMA will use.  No maximum is computed on this path: a reference that has fallen too far behind shows up as
        // a large (or infinite, or NaN) tile sum, and only then - and on a row's first step - is the tile done again
        // with the reference raised to the tile's maximum.  Sums and accumulators are f32; a probability stays below
        // FR_SUM_LIMIT in f16.
        half8 p[2];
        float lsum;
        auto exp_tile = [&](float ref) __attribute__((always_inline)) {
            const half2v ones = {(_Float16)1.0f, (_Float16)1.0f};
            float dsum = 0.0f;
#pragma unroll
            for (int r = 0; r < 16; r += 2) {
                half2v p2;
                p2[0] = (_Float16)__builtin_amdgcn_exp2f(s2[r] - ref);
                p2[1] = (_Float16)__builtin_amdgcn_exp2f(s2[r + 1] - ref);
                dsum = __builtin_amdgcn_fdot2(p2, ones, dsum, false);
                p[r >> 3][r & 7]       = p2[0];
                p[r >> 3][(r & 7) + 1] = p2[1];
            }
            lsum = dsum;
        };
        exp_tile(m == -INFINITY ? 0.0f : m);
        if (__builtin_amdgcn_ballot_w64(!(lsum <= FR_SUM_LIMIT) || m == -INFINITY) != 0) {     // wave-uniform; rare after the first step
            float tmax = s2[0];
#pragma unroll
            for (int r = 1; r < 16; r++) tmax = fmaxf(tmax, s2[r]);
            tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));      // both halves of a query must agree
            const float mn = tmax > m ? tmax : m;
            const float f  = mn == -INFINITY ? 1.0f : __builtin_amdgcn_exp2f(m - mn);     // m = -inf: nothing accumulated yet, f = 0
            l *= f;
#pragma unroll
            for (int db = 0; db < DBO; db++) oacc[db] *= f;
            m = mn;
            exp_tile(m == -INFINITY ? 0.0f : m);
        }
        l += lsum;

        // ---- O^T += V^T . P^T -------------------------------------------------------------------------------------------
        {
#pragma unroll
            for (int db = 0; db < DBO; db++) {
#pragma unroll
                for (int ks = 0; ks < 2; ks++) {
                    const char * p0 = vt + vaddr[db] + 16 * ks * KP;
                    const half4 lo = __builtin_bit_cast(half4, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4v *)p0));
                    const half4 hi = __builtin_bit_cast(half4, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4v *)(p0 + 8 * KP)));
                    const half8 va = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                    oacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(va, p[ks], oacc[db], 0, 0, 0);
                }
            }
        }
        __builtin_amdgcn_s_waitcnt(0x0F70);               // vmcnt(0): this wave's share of the next K tile and table block is in LDS
        __syncthreads();                                  // every wave has read the V tile; the next K tile and table block are complete
        if (t + 1 < NTL) dma_v(t + 1);
    }

    // ---- normalise and store: lane (il, hh) holds d = 32 db + 8 g + 4 hh + c of its query -------------------------------
    l += __shfl_xor(l, 32, 64);
    // Excluded keys (add = -inf) were multiplied by probabilities of exactly zero, not skipped: the same for finite K/V, NaN
    // otherwise.  Queries whose result is not finite are computed again below, excluded keys unread, as the CPU op does it.
    uint64_t badbits = 0;
    if constexpr (ADD) {
        float chk = l * 0.0f;
#pragma unroll
        for (int db = 0; db < DBO; db++)
#pragma unroll
            for (int r = 0; r < 16; r++) chk = fmaf(oacc[db][r], 0.0f, chk);
        badbits = __builtin_amdgcn_ballot_w64(chk != 0.0f);
    }
    if (i0w + il < a.Nq) {
        const float inv = l > 0.0f ? 1.0f / l : 0.0f;
        float * orow = a.dst + (((int64_t)b * a.Nq + (i0w + il)) * a.H + h) * D;
#pragma unroll
        for (int db = 0; db < DBO; db++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                float4v o;
#pragma unroll
                for (int c = 0; c < 4; c++) o[c] = oacc[db][4 * g + c] * inv;
                *(float4v *)(orow + 32 * db + 8 * g + 4 * hh) = o;
            }
    }
    if constexpr (ADD) {
        if (badbits != 0) {
            __threadfence();
            uint32_t bits = (uint32_t)badbits | (uint32_t)(badbits >> 32);      // lanes l and l + 32 hold the same query
            while (bits != 0) {
                const int qi = i0w + __builtin_ctz(bits);
                bits &= bits - 1;
                if (qi < a.Nq) attn_row_redo_relpos<D>(a, qi, h, b);
            }
        }
    }
}

template <int D, int NW>
int launch_d(const FattnRelposArgs & a, hipStream_t stream) {
    const int64_t G = (int64_t)((a.Nq + 32 * NW - 1) / (32 * NW)) * a.H * a.B;
    const int64_t grid = (G + 7) / 8 * 8;
    if (grid > 0x7fffffff) return (int)hipErrorInvalidValue;
    constexpr int lds = fr_lds_bytes<D, NW>();
#define FR_LAUNCH(ADD, F16)                                                                                                   \
    do {                                                                                                                      \
        static std::atomic<uint64_t> lds_allowed{0};                                                                          \
        const hipError_t e = fattn_allow_lds((const void *)fattn_relpos_kernel<D, NW, ADD, F16>, lds, lds_allowed);           \
        if (e != hipSuccess) return (int)e;                                                                                   \
        hipLaunchKernelGGL((fattn_relpos_kernel<D, NW, ADD, F16>), dim3((unsigned)grid), dim3(NW * 64), lds, stream, a);    \
    } while (0)
    if (!a.add)          FR_LAUNCH(false, false);
    else if (a.add_f16)  FR_LAUNCH(true, true);
    else                 FR_LAUNCH(true, false);
#undef FR_LAUNCH
    return (int)hipGetLastError();
}

}  // namespace

bool fattn_relpos_supported(const FattnRelposArgs & a) {
    if (a.D != 64 && a.D != 128) return false;
    if (a.Nq < 1 || a.Nkv < 1 || a.H < 1 || a.B < 1) return false;
    // 32-bit tile indices; the table's rows Nq-1+j-i must exist
    if ((int64_t)a.Nq + a.Nkv > (1 << 24)) return false;
    return true;
}

int fattn_relpos_launch(const FattnRelposArgs & a, hipStream_t stream) {
    if (!fattn_relpos_supported(a)) return (int)hipErrorInvalidValue;
    // Workgroups of 2, 3 or 4 waves (32 queries each).  Every workgroup stages all K, V and table tiles of its head and pays
    // a step's barriers and waits whatever its width, so the widest one that the queries fill is taken (measured at
    // 8 heads x 128, T = 750, batch 8: 4 waves, 384 workgroups: 74 us; 3 waves, 512 workgroups: 80 us; 2 waves, 768: 81 us).
    int best = (a.Nq + 31) / 32;
    best = best < 2 ? 2 : best > 4 ? 4 : best;
    static const char * force = getenv("MI355X_RELPOS_WAVES");            // experiments only
    if (force && atoi(force) >= 2 && atoi(force) <= 4) best = atoi(force);
    switch (best) {
        case 2:  return a.D == 64 ? launch_d<64, 2>(a, stream) : launch_d<128, 2>(a, stream);
        case 3:  return a.D == 64 ? launch_d<64, 3>(a, stream) : launch_d<128, 3>(a, stream);
        default: return a.D == 64 ? launch_d<64, 4>(a, stream) : launch_d<128, 4>(a, stream);
    }
}
