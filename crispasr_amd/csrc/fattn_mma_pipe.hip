// Software-pipelined f16-MFMA attention kernel for head size 64 without mask (the Whisper / Voxtral
// encoder shape) on gfx950.
//
// Same tiling and operand layouts as fattn_mma_kernel (transposed products on
// v_mfma_f32_32x32x16_f16, 256 queries per workgroup of 4 waves, 64 queries per wave, keys in blocks of
// 32, K in LDS at a pitch of 16 mod 128 bytes, V^T by ds_read_b64_tr_b16 at a pitch of 64 mod 128
// bytes), but each wave runs a three-deep software pipeline over the key blocks so that, inside ONE
// wave's instruction stream, the matrix pipe and the vector ALU always have independent work:
//
//   iteration b:   S(b+1) = K(b+1).Q^T - m      8 MFMAs      (K operands fetched during iteration b-1)
//                  O     += V(b-1)^T.P(b-1)     8 MFMAs      (V operands and P from iteration b-1)
//                  P(b)   = 2^S(b), row sums    32 v_exp_f32, 16 v_cvt_pk, 16 v_dot2   (S(b) from b-1)
//                  LDS:     V operands of b, K operands of b+2
//
// The kernel runs one wave per SIMD with the whole 512-entry register budget instead of relying on a second
// resident workgroup.  Measured on MI355X it does NOT beat fattn_mma_kernel (568 vs 631 TFLOP/s on the Whisper
// large-v3 encoder shape): a micro-benchmark of exactly this slice pattern (16 MFMAs interleaved with 32
// v_exp_f32 + 16 v_cvt_pk + 16 v_dot2 in one wave) takes 928 cycles against 592 for the MFMAs alone and 476
// for the vector work alone - the two pipes overlap by about 13% only - so the schedule this kernel was built
// to obtain is not available on this part.  It is kept selectable (MI355X_FATTN_MMA_PIPE) and tested, but
// AUTO never picks it.  K/V tiles go through a three-stage LDS ring (one barrier per
// 64 keys); the global loads of tile t+3 are in flight during tile t+1.
//
// The running reference m is the C operand of the first Q.K^T MFMA; a block is only redone (with a
// maximum, a new reference and a rescale of O) when its f16 probabilities sum above SUM_LIMIT or
// no finite score has been seen yet - checked at the end of the iteration, off the pipelined region.
#include "fattn_common.h"

#include <type_traits>

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float    float16v __attribute__((ext_vector_type(16)));
typedef short    short4v __attribute__((ext_vector_type(4)));

constexpr int   D       = 64;
constexpr int   NQB     = 2;
constexpr int   KS      = D / 16;
constexpr int   DB      = D / 32;
constexpr int   WAVES   = 4;
constexpr int   THREADS = WAVES * 64;
constexpr int   BC      = 64;
constexpr int   CH      = D / 8;
constexpr int   RPP     = THREADS / CH;
constexpr int   NP      = BC / RPP;
constexpr int   PK      = D + 8;
constexpr int   PVT     = D + 32;
constexpr int   STAGES  = 3;
constexpr int   BMG     = 32 * NQB * WAVES;
constexpr float LOG2E     = 1.4426950408889634f;
constexpr float SUM_LIMIT = 8192.0f;

struct Raw {
    uint4 a, b;
};

template <int TYPE>
__device__ __forceinline__ Raw load_chunk(const char * row, int c, bool valid) {
    Raw r;
    r.a = make_uint4(0, 0, 0, 0);
    r.b = make_uint4(0, 0, 0, 0);
    if (!valid) return r;
    if (TYPE == MI355X_TYPE_F16) {
        r.a = *(const uint4 *)(row + c * 16);
    } else if (TYPE == MI355X_TYPE_F32) {
        r.a = *(const uint4 *)(row + c * 32);
        r.b = *(const uint4 *)(row + c * 32 + 16);
    } else {
        const char * blk = row + (c >> 2) * FATTN_Q8_0_BYTES;
        const uint16_t * qs = (const uint16_t *)(blk + 2 + (c & 3) * 8);
        r.a.x = (uint32_t)qs[0] | ((uint32_t)qs[1] << 16);
        r.a.y = (uint32_t)qs[2] | ((uint32_t)qs[3] << 16);
        r.a.z = *(const uint16_t *)blk;
    }
    return r;
}

template <int TYPE>
__device__ __forceinline__ half8 to_half8(const Raw & r) {
    half8 h;
    if (TYPE == MI355X_TYPE_F16) {
        h = __builtin_bit_cast(half8, r.a);
    } else if (TYPE == MI355X_TYPE_F32) {
        const float f[8] = {__uint_as_float(r.a.x), __uint_as_float(r.a.y), __uint_as_float(r.a.z), __uint_as_float(r.a.w),
                            __uint_as_float(r.b.x), __uint_as_float(r.b.y), __uint_as_float(r.b.z), __uint_as_float(r.b.w)};
#pragma unroll
        for (int e = 0; e < 8; e++) h[e] = (_Float16)f[e];
    } else {
        const float d = h2f_bits((uint16_t)r.a.z);
        const uint32_t w[2] = {r.a.x, r.a.y};
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const int8_t q = (int8_t)((w[e >> 2] >> (8 * (e & 3))) & 0xff);
            h[e] = (_Float16)((float)q * d);
        }
    }
    return h;
}

__device__ __forceinline__ float max_xor32(float x) { return fmaxf(x, xor_shuffle(x, 32)); }
__device__ __forceinline__ float sum_xor32(float x) { return x + xor_shuffle(x, 32); }

template <int TYPE>
__global__ void __launch_bounds__(THREADS, 1) fattn_mma_pipe_kernel(const FattnArgs a, const int n_qtiles) {
    extern __shared__ __attribute__((aligned(16))) _Float16 lds_raw[];
    _Float16 (*k_lds)[BC * PK]  = (_Float16 (*)[BC * PK])lds_raw;
    _Float16 (*v_lds)[BC * PVT] = (_Float16 (*)[BC * PVT])(lds_raw + STAGES * BC * PK);

    const int tid  = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int l32  = lane & 31;
    const int hh   = lane >> 5;

    // query tiles of one (head, batch) share K/V: keep them on one XCD (workgroups go to XCDs round-robin)
    int bid = blockIdx.x;
    {
        const int per = gridDim.x / 8;
        if (bid < per * 8) bid = (bid % 8) * per + bid / 8;
    }
    const int qt = bid % n_qtiles;
    const int h  = (bid / n_qtiles) % a.Hq;
    const int b  = bid / (n_qtiles * a.Hq);
    const int hk = h / a.gqa;
    const int bk = b / a.bq;
    const int q0 = qt * BMG + wave * 32 * NQB;

    const float qscale = a.scale * LOG2E;
    half8 qreg[NQB][KS];
#pragma unroll
    for (int qb = 0; qb < NQB; qb++) {
        const int qi = min(q0 + qb * 32 + l32, a.Nq - 1);
        const float * qrow = (const float *)(a.q + (int64_t)qi * a.nbq1 + (int64_t)h * a.nbq2 + (int64_t)b * a.nbq3);
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            const float4 x0 = *(const float4 *)(qrow + ks * 16 + hh * 8);
            const float4 x1 = *(const float4 *)(qrow + ks * 16 + hh * 8 + 4);
            half8 v;
            v[0] = (_Float16)(x0.x * qscale); v[1] = (_Float16)(x0.y * qscale);
            v[2] = (_Float16)(x0.z * qscale); v[3] = (_Float16)(x0.w * qscale);
            v[4] = (_Float16)(x1.x * qscale); v[5] = (_Float16)(x1.y * qscale);
            v[6] = (_Float16)(x1.z * qscale); v[7] = (_Float16)(x1.w * qscale);
            qreg[qb][ks] = v;
        }
    }

    const char * kbase = a.k + (int64_t)hk * a.nbk2 + (int64_t)bk * a.nbk3;
    const char * vbase = a.v + (int64_t)hk * a.nbv2 + (int64_t)bk * a.nbv3;
    const int sc = tid % CH;
    const int sr = tid / CH;

    // two register sets: a tile's global loads stay in flight for two tiles before they are written to LDS
    Raw kraw[2][NP], vraw[2][NP];
    auto load_tile = [&](int tile, auto set_tag) {
        constexpr int SET = decltype(set_tag)::value;
#pragma unroll
        for (int p = 0; p < NP; p++) {
            // rows past Nkv re-read the last row: their scores are forced to -inf, so a finite stand-in is
            // all that is needed, and branch-free loads let the waits on them be counted exactly
            const int key = min(tile * BC + sr + p * RPP, a.Nkv - 1);
            kraw[SET][p] = load_chunk<TYPE>(kbase + (int64_t)key * a.nbk1, sc, true);
            vraw[SET][p] = load_chunk<TYPE>(vbase + (int64_t)key * a.nbv1, sc, true);
        }
    };
    auto store_tile = [&](int stage, auto set_tag) {
        constexpr int SET = decltype(set_tag)::value;
#pragma unroll
        for (int p = 0; p < NP; p++) {
            const int row = sr + p * RPP;
            *(half8 *)&k_lds[stage][row * PK + sc * 8]  = to_half8<TYPE>(kraw[SET][p]);
            *(half8 *)&v_lds[stage][row * PVT + sc * 8] = to_half8<TYPE>(vraw[SET][p]);
        }
    };

    // ---- pipeline registers -----------------------------------------------------------------------
    float16v oacc[NQB][DB];
    float16v negm[NQB];
    float16v s[2][NQB];
    half8    preg[2][NQB][2];
    half8    ka[2][KS];
    half8    va[2][2][DB];
    float    m_ref[NQB], l_run[NQB];
    bool     have[NQB];
    const half8 hzero = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int qb = 0; qb < NQB; qb++) {
        m_ref[qb] = 0.0f;
        l_run[qb] = 0.0f;
        have[qb]  = false;
#pragma unroll
        for (int r = 0; r < 16; r++) negm[qb][r] = 0.0f;
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
            for (int r = 0; r < 16; r++) oacc[qb][db][r] = 0.0f;
#pragma unroll
        for (int k2 = 0; k2 < 2; k2++) preg[1][qb][k2] = hzero;      // the "block -1" the first iteration multiplies
    }
#pragma unroll
    for (int k2 = 0; k2 < 2; k2++)
#pragma unroll
        for (int db = 0; db < DB; db++) va[1][k2][db] = hzero;

    // LDS addresses of this lane's operands inside a stage
    const int k_off = l32 * PK + hh * 8;                                        // + kb*32*PK + ks*16
    const int v_off = (hh * 4 + ((lane & 15) >> 2)) * PVT + ((lane >> 4) & 1) * 16 + (lane & 3) * 4;   // + (kb*32 + k2*16 [+8])*PVT + db*32

    const int n_tiles = (a.Nkv + BC - 1) / BC;

    // One pipeline iteration for block (tile t, half CUR).  NEXT_QK: block b+1 exists; NEXT_TILE: tile t+1
    // exists (its K operands are fetched for b+2); TAIL: tile t runs past Nkv.
    auto body = [&](const int t, auto cur_tag, auto next_qk_tag, auto next_tile_tag, auto tail_tag) {
        constexpr int  CUR       = decltype(cur_tag)::value;
        constexpr int  NXT       = 1 - CUR;
        constexpr bool NEXT_QK   = decltype(next_qk_tag)::value;
        constexpr bool NEXT_TILE = decltype(next_tile_tag)::value;
        constexpr bool TAIL      = decltype(tail_tag)::value;
        const int st_cur = t % STAGES;
        const int st_nxt = (t + 1) % STAGES;

        if (TAIL) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int key = t * BC + CUR * 32 + (r >> 2) * 8 + hh * 4 + (r & 3);
                if (key >= a.Nkv) {
#pragma unroll
                    for (int qb = 0; qb < NQB; qb++) s[CUR][qb][r] = -INFINITY;
                }
            }
        }

        float lsum[NQB] = {0.0f, 0.0f};
        const half2v ones = {(_Float16)1.0f, (_Float16)1.0f};
        half4 vlo[2][DB];

        // 16 slices: one MFMA, two exponentials, one pack, one dot2 and (in the first 12) one LDS read each
#pragma unroll
        for (int i = 0; i < 16; i++) {
            // -- matrix pipe: even slices Q.K^T of block b+1, odd slices P.V of block b-1
            if ((i & 1) == 0) {
                if (NEXT_QK) {
                    const int ks = i >> 2, qb = (i >> 1) & 1;
                    s[NXT][qb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ka[NXT][ks], qreg[qb][ks], ks == 0 ? negm[qb] : s[NXT][qb], 0, 0, 0);
                }
            } else {
                const int j = i >> 1, k2 = j >> 2, db = (j >> 1) & 1, qb = j & 1;
                oacc[qb][db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(va[NXT][k2][db], preg[NXT][qb][k2], oacc[qb][db], 0, 0, 0);
            }
            // -- vector ALU: elements 2*(i/2), 2*(i/2)+1 of query block (i&1) of block b
            {
                const int qb = i & 1, r = (i >> 1) * 2;
                half2v p2;
                p2[0] = (_Float16)__builtin_amdgcn_exp2f(s[CUR][qb][r]);
                p2[1] = (_Float16)__builtin_amdgcn_exp2f(s[CUR][qb][r + 1]);
                lsum[qb] = __builtin_amdgcn_fdot2(p2, ones, lsum[qb], false);
                preg[CUR][qb][r >> 3][r & 7]       = p2[0];
                preg[CUR][qb][r >> 3][(r & 7) + 1] = p2[1];
            }
            // -- LDS: V operands of block b (8 transpose reads), then K operands of block b+2 (4 reads)
            if (i < 8) {
                const int k2 = i >> 2, db = (i >> 1) & 1, half = i & 1;
                const _Float16 * p = &v_lds[st_cur][v_off + (CUR * 32 + k2 * 16 + half * 8) * PVT + db * 32];
                const half4 x = __builtin_bit_cast(half4, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4v *)p));
                if (half == 0) vlo[k2][db] = x;
                else           va[CUR][k2][db] = __builtin_shufflevector(vlo[k2][db], x, 0, 1, 2, 3, 4, 5, 6, 7);
            } else if (i < 8 + KS) {
                if (NEXT_TILE) {
                    const int ks = i - 8;
                    ka[CUR][ks] = *(const half8 *)&k_lds[st_nxt][k_off + CUR * 32 * PK + ks * 16];
                }
            }
        }

        // Every LDS read of this iteration has had four slices to land: drain the counter here, so that the next
        // iteration starts with nothing pending and its first MFMAs are not held behind waits on reads they do
        // not use (lgkmcnt(0), other counters untouched).
        __builtin_amdgcn_s_waitcnt(0xC07F);

        // ---- off the pipelined region: did the reference fall behind (or is this the first finite block)? ----
        bool redo = false;
#pragma unroll
        for (int qb = 0; qb < NQB; qb++) redo = redo || !(lsum[qb] <= SUM_LIMIT) || !have[qb];
        if (__builtin_amdgcn_ballot_w64(redo) != 0) {
#pragma unroll
            for (int qb = 0; qb < NQB; qb++) {
                float mx = s[CUR][qb][0];
#pragma unroll
                for (int r = 1; r < 16; r++) mx = fmaxf(mx, s[CUR][qb][r]);
                const float tm = max_xor32(mx);
                float delta = 0.0f;
                if (tm > -INFINITY) {
                    delta = have[qb] ? fmaxf(tm, 0.0f) : tm;
                    have[qb] = true;
                }
                const float f = __builtin_amdgcn_exp2f(-delta);
                m_ref[qb] += delta;
                l_run[qb] *= f;
#pragma unroll
                for (int r = 0; r < 16; r++) negm[qb][r] = -m_ref[qb];
#pragma unroll
                for (int db = 0; db < DB; db++)
#pragma unroll
                    for (int r = 0; r < 16; r++) oacc[qb][db][r] *= f;
                // P(b-1) has been folded into O already (this iteration's P.V), so only S(b) and S(b+1) move
                float acc = 0.0f;
#pragma unroll
                for (int r = 0; r < 16; r += 2) {
                    half2v p2;
                    p2[0] = (_Float16)__builtin_amdgcn_exp2f(s[CUR][qb][r] - delta);
                    p2[1] = (_Float16)__builtin_amdgcn_exp2f(s[CUR][qb][r + 1] - delta);
                    acc = __builtin_amdgcn_fdot2(p2, ones, acc, false);
                    preg[CUR][qb][r >> 3][r & 7]       = p2[0];
                    preg[CUR][qb][r >> 3][(r & 7) + 1] = p2[1];
                }
                lsum[qb] = acc;
                if (NEXT_QK) {
#pragma unroll
                    for (int r = 0; r < 16; r++) s[NXT][qb][r] -= delta;
                }
            }
        }
#pragma unroll
        for (int qb = 0; qb < NQB; qb++) l_run[qb] += lsum[qb];
    };

    typedef std::integral_constant<int, 0>  I0;
    typedef std::integral_constant<int, 1>  I1;
    typedef std::true_type  T;
    typedef std::false_type F;

    // ---- prologue: tiles 0 and 1 into the ring, tiles 2 and 3 into registers, S(0) computed ---------------------
    load_tile(0, I0{});
    store_tile(0, I0{});
    if (n_tiles > 1) {
        load_tile(1, I1{});
        store_tile(1, I1{});
    }
    __syncthreads();
    // (unconditional, with the tile index clamped: a fixed number of loads in flight lets every wait on
    // them be an exact count instead of a drain; a surplus tile lands in a stage nobody reads any more)
    load_tile(min(2, n_tiles - 1), I0{});
    load_tile(min(3, n_tiles - 1), I1{});
#pragma unroll
    for (int ks = 0; ks < KS; ks++) ka[0][ks] = *(const half8 *)&k_lds[0][k_off + ks * 16];
#pragma unroll
    for (int qb = 0; qb < NQB; qb++) {
#pragma unroll
        for (int ks = 0; ks < KS; ks++)
            s[0][qb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ka[0][ks], qreg[qb][ks], ks == 0 ? negm[qb] : s[0][qb], 0, 0, 0);
    }
#pragma unroll
    for (int ks = 0; ks < KS; ks++) ka[1][ks] = *(const half8 *)&k_lds[0][k_off + 32 * PK + ks * 16];

    // ---- steady state: every tile that has a successor.  Tile t+2 goes from register set t&1 into the ring at
    // the end of tile t, and the same set then takes the loads of tile t+4.
#define FATTN_PIPE_STEADY(T_, SET_)                                      \
    do {                                                                 \
        body((T_), I0{}, T{}, T{}, F{});                                 \
        body((T_), I1{}, T{}, T{}, F{});                                 \
        store_tile(((T_) + 2) % STAGES, SET_{});                         \
        __syncthreads();                                                 \
        load_tile(min((T_) + 4, n_tiles - 1), SET_{});                   \
    } while (0)
    int t = 0;
    for (; t + 2 < n_tiles; t += 2) {
        FATTN_PIPE_STEADY(t, I0);
        FATTN_PIPE_STEADY(t + 1, I1);
    }
    if (t + 1 < n_tiles) {
        FATTN_PIPE_STEADY(t, I0);
        t++;
    }
#undef FATTN_PIPE_STEADY
    // ---- last tile (possibly partial), then the P.V that is still owed ------------------------------------------
    {
        if (a.Nkv % BC) {
            body(t, I0{}, T{}, F{}, T{});
            body(t, I1{}, F{}, F{}, T{});
        } else {
            body(t, I0{}, T{}, F{}, F{});
            body(t, I1{}, F{}, F{}, F{});
        }
#pragma unroll
        for (int k2 = 0; k2 < 2; k2++)
#pragma unroll
            for (int db = 0; db < DB; db++)
#pragma unroll
                for (int qb = 0; qb < NQB; qb++)
                    oacc[qb][db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(va[1][k2][db], preg[1][qb][k2], oacc[qb][db], 0, 0, 0);
    }

    // ---- normalise and write dst[D, Hq, Nq, B] ---------------------------------------------------------------------
#pragma unroll
    for (int qb = 0; qb < NQB; qb++) {
        const float ltot = sum_xor32(l_run[qb]);
        const float inv  = ltot > 0.0f ? 1.0f / ltot : 0.0f;
        const int   qi   = q0 + qb * 32 + l32;
        if (qi < a.Nq) {
            float * out = a.dst + (((int64_t)b * a.Nq + qi) * a.Hq + h) * D;
#pragma unroll
            for (int db = 0; db < DB; db++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    float4 o;
                    o.x = oacc[qb][db][g * 4 + 0] * inv;
                    o.y = oacc[qb][db][g * 4 + 1] * inv;
                    o.z = oacc[qb][db][g * 4 + 2] * inv;
                    o.w = oacc[qb][db][g * 4 + 3] * inv;
                    *(float4 *)(out + db * 32 + g * 8 + hh * 4) = o;
                }
        }
    }
}

template <int TYPE>
int launch(const FattnArgs & a, hipStream_t stream) {
    const int n_qtiles = (a.Nq + BMG - 1) / BMG;
    const dim3 grid((unsigned)(n_qtiles * a.Hq * a.B));
    const size_t lds = (size_t)STAGES * BC * (PK + PVT) * sizeof(_Float16);
    static bool attr_set = false;
    if (!attr_set) {
        const hipError_t e = hipFuncSetAttribute((const void *)fattn_mma_pipe_kernel<TYPE>,
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return (int)e;
        attr_set = true;
    }
    hipLaunchKernelGGL((fattn_mma_pipe_kernel<TYPE>), grid, dim3(THREADS), lds, stream, a, n_qtiles);
    return (int)hipGetLastError();
}

}  // namespace

// head size 64, no mask, no soft cap, enough queries to fill 64-query waves
bool fattn_mma_pipe_supported(const FattnArgs & a, int ktype) {
    if (a.D != 64 || a.mask || a.softcap != 0.0f) return false;
    if (a.Nq < 64 || a.Nkv < 1) return false;
    if (ktype != MI355X_TYPE_Q8_0 && !a.aligned16) return false;
    if (ktype == MI355X_TYPE_Q8_0 && !a.q_aligned16) return false;
    return ktype == MI355X_TYPE_F16 || ktype == MI355X_TYPE_F32 || ktype == MI355X_TYPE_Q8_0;
}

int fattn_mma_pipe_launch(const FattnArgs & a, int ktype, hipStream_t stream) {
    switch (ktype) {
        case MI355X_TYPE_F16:  return launch<MI355X_TYPE_F16>(a, stream);
        case MI355X_TYPE_F32:  return launch<MI355X_TYPE_F32>(a, stream);
        case MI355X_TYPE_Q8_0: return launch<MI355X_TYPE_Q8_0>(a, stream);
        default:               return (int)hipErrorInvalidValue;
    }
}
