// f16-MFMA tile kernel for prefill / encoder attention on gfx950 (CDNA4, wave64).
//
// A workgroup of 4 waves owns 4*32*NQB consecutive queries of one (head, batch) and walks
// the keys in tiles of 64.  Both products run on v_mfma_f32_32x32x16_f16 in the transposed
// form, so that a lane keeps one query column for the whole kernel:
//
//   S^T[key, query] = K[key, :] . Q[query, :]^T        A = K tile (LDS),   B = Q (registers)
//   O^T[d,   query] = V[:, d]^T . P^T[:, query]        A = V^T (LDS),      B = P (registers)
//
// With the 32x32 accumulator layout lane l holds query l%32 and keys {8g + 4(l/32) + r},
// which is exactly the B-operand layout the second product needs (after choosing the order
// of its reduction index), so the probabilities never leave registers and the online softmax
// needs one cross-lane exchange (lane l <-> l+32) per tile for the running maximum.
//
// K and V tiles are staged through LDS in their natural [key][d] layout (converted to f16
// when the cache is F32 or Q8_0), double-buffered, with the next tile's global loads in
// flight during the current tile's MFMAs.  K rows are padded to a pitch of 16 mod 128 bytes
// so the 128-bit operand reads of 8 consecutive lanes fall into distinct banks.  V^T
// operands are produced by ds_read_b64_tr_b16 (LDS transpose read): 16 lanes present four
// 32-byte row segments of four keys and each lane receives the four keys' values of its own
// d - V's pitch is 64 mod 128 bytes so that those four segments tile the banks.
//
// F16 caches skip the registers on the way in (DIRECT): global_load_lds_dwordx4 writes each wave's 64 x 16
// bytes straight into LDS.  Such a load fills 1 KiB of consecutive LDS, so rows cannot be padded; instead
// the 16-byte chunks of a row are stored XOR-swizzled (each lane fetches the global chunk that belongs at
// its LDS slot), with one swizzle for K (128-bit operand reads: 16 consecutive rows, one chunk column) and
// one for V (transpose reads: 8 rows x 4 chunk columns), both conflict-free.
//
// The mask of such a kernel takes the same road (MDMA): each wave fetches the 32 keys x its own queries that a
// half tile needs into a private, swizzled LDS block half a tile before they are read, instead of having
// every lane pull 8-byte pieces of 32 different rows through the vector cache.
//
// Softmax runs in base 2: scale*log2(e) is folded into Q when it is converted to f16.
//
// Grids that would leave CUs idle take the key-split form (KSP = 2): a workgroup owns half as many queries and its
// waves pair up, the two waves of a pair walking the same queries over the first and the second 32 keys of every
// tile; the pair's partial results meet in LDS once, after the last tile.  Same LDS traffic and MFMA count in all,
// half the work per wave.
//
// A 32-key block whose mask excludes every key for all of the wave's queries is skipped outright (its probabilities
// would all be exact zeros): the upper triangle of a causal prompt, the keys beyond a padded sequence's length.
#include "fattn_row.h"

#include <stdio.h>
#include <stdlib.h>
#include <type_traits>

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float    float16v __attribute__((ext_vector_type(16)));
typedef float    float4v __attribute__((ext_vector_type(4)));
typedef short    short4v __attribute__((ext_vector_type(4)));
typedef unsigned uint2v __attribute__((ext_vector_type(2)));

constexpr int   MMA_WAVES   = 4;
constexpr int   MMA_THREADS = MMA_WAVES * 64;
constexpr int   BC          = 64;                 // keys per tile
constexpr float LOG2E       = 1.4426950408889634f;

template <int D> struct Pitch {
    static constexpr int K = D + 8;               // halves: (2D + 16) bytes = 16 mod 128
    static constexpr int V = D + 32;              // halves: (2D + 64) bytes = 64 mod 128
};

// raw global data of one 8-element chunk of a K or V row, converted to f16 when written to LDS
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
            h[e] = (_Float16)((float)q * d);       // exact q*d, then one rounding to f16
        }
    }
    return h;
}

// max / sum of a value held by lane l and lane l^32.  Only used off the hot path (reference
// raises, epilogue), so the LDS-crossbar shuffle is good enough.
__device__ __forceinline__ float max_xor32(float x) { return fmaxf(x, xor_shuffle(x, 32)); }
__device__ __forceinline__ float sum_xor32(float x) { return x + xor_shuffle(x, 32); }

// branch-free tanh: 1 - 2/(2^(2x*log2e) + 1); exact limits at +-inf
__device__ __forceinline__ float fast_tanh(float x) {
    const float e = __builtin_amdgcn_exp2f(x * (2.0f * LOG2E));
    return 1.0f - 2.0f * __builtin_amdgcn_rcpf(e + 1.0f);
}

// Running softmax state of one 32-query block, per lane (= per query, mirrored in lane l^32).
// Scores are kept relative to `m`, a reference that may trail the true running maximum by up
// to 13 (in log2 units, see SUM_LIMIT): it enters the Q.K^T MFMA as its C operand, so the
// common block needs no subtraction, no maximum and no rescale of O.
struct RowState {
    float m;        // reference subtracted from the scores (finite)
    float l;        // sum of p over this lane's keys
    bool  have;     // a finite score has been seen
};
// a block of 16 probabilities summing to more than this means the reference is > 9 behind
constexpr float SUM_LIMIT = 8192.0f;

// chunk swizzles of the unpadded DIRECT layout (r = key row inside the tile)
template <int D> __device__ __forceinline__ int swz_k(int r) { return D == 64 ? (r >> 1) & 7 : r & 15; }
template <int D> __device__ __forceinline__ int swz_v(int r) { return D == 64 ? r & 7 : (r & 3) << 2; }

template <int D> __device__ __forceinline__ int swz_m(int r) { return (r >> 2) & 3; }     // mask half tile: 4 chunks per row

// TK: keys per tile.  64, except in the key-split form of 64-wide heads without a mask - the grids where a wave is alone on
// its SIMD: tiles of 128 (each wave two 32-key blocks of its half: half the barriers per key, and the second block's
// operands are on their way while the first is in the softmax), or of 256 when the workgroups number no more than the
// CUs, since four such tiles are 128 KB of LDS and leave room for one workgroup per CU only.
// (two query blocks per wave with 128-key tiles: 240 bytes of scratch per lane in the loop, 110 us instead of 60 on the
//  large-v3 encoder layer)
// PAD: the head is one of a.Dv elements (a multiple of 8 below D) on K/V copies whose rows are zero-padded to D: a.Dv
// elements of every q row are read and a.Dv of every dst row written.  An instantiation of its own, so that the others
// stay the code they were (the guards cost the one-block forms 2% as a run-time branch).
template <int D, int NQB, int KSP, int TYPE, bool MASK, bool SOFTCAP, bool DIRECT, bool MDMA, int TK = BC, bool PAD = false>
__global__ void __launch_bounds__(MMA_THREADS, 2) fattn_mma_kernel(const FattnArgs a, const int n_qtiles) {
    static_assert(!PAD || (DIRECT && NQB == 1), "zero-padded heads: f16 copies, one query block per wave");
    constexpr bool whole_head = !PAD;
    static_assert(!DIRECT || TYPE == MI355X_TYPE_F16, "only f16 rows can go to LDS unconverted");
    static_assert(!MDMA || (DIRECT && MASK), "the mask goes through LDS only beside directly loaded K/V");
    static_assert(KSP == 1 || (KSP == 2 && NQB == 1 && !MDMA), "key-split form: one query block per wave, mask through registers");
    constexpr int NMH   = NQB * 2;                 // MDMA: loads per wave and half tile (16 rows x 64 bytes each)
    constexpr int MHALF = NQB * 32 * 64;           //       bytes of a wave's half-tile block; a wave owns 2 of them
    constexpr int ROWB  = D * 2;                   // DIRECT: bytes per (unpadded) row
    constexpr int BCT   = TK;                      // keys per tile
    static_assert(TK == BC || (KSP == 2 && D == 64 && !MASK && DIRECT), "larger tiles exist for the unmasked key-split form of 64-wide heads");
    constexpr int TILEB = BCT * ROWB;              //         bytes per K or V tile; LDS = K0 K1 V0 V1
    constexpr int NLD   = TILEB / 1024 / MMA_WAVES;   //      global->LDS loads per wave, tile and tensor

    constexpr int KS   = D / 16;                   // reduction steps of Q.K^T
    constexpr int DB   = D / 32;                   // 32-wide blocks of the output's d
    constexpr int CH   = D / 8;                    // 8-element chunks per row
    constexpr int RPP  = MMA_THREADS / CH;         // rows staged per pass
    constexpr int NP   = BC / RPP;                 // passes per tile
    constexpr int PK   = Pitch<D>::K;
    constexpr int PV   = Pitch<D>::V;
    constexpr int BMW  = 32 * NQB;                 // queries per wave
    constexpr int BMG  = BMW * MMA_WAVES / KSP;    // queries per workgroup
    constexpr int NKB  = BCT / 32 / KSP;           // 32-key blocks of a tile that one wave walks
    // Skipping excluded blocks adds a branch round the block's body.  The instantiations that already fill the register
    // file (two query blocks per wave, 128-wide heads without key split) answer it with spills inside the tile loop, so
    // it is left to the others: the key-split form and one query block of 64-wide heads.
    constexpr bool SKIP = MASK && (KSP == 2 || (D == 64 && NQB == 1));

    extern __shared__ __attribute__((aligned(16))) _Float16 lds_raw[];
    _Float16 (*k_lds)[BC * PK] = (_Float16 (*)[BC * PK])lds_raw;
    _Float16 (*v_lds)[BC * PV] = (_Float16 (*)[BC * PV])(lds_raw + 2 * BC * PK);

    const int tid  = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int l32  = lane & 31;
    const int hh   = lane >> 5;                    // which half of the wave

    // Workgroups are handed to the 8 XCDs round-robin; renumber them so that the query tiles
    // of one (head, batch) - which share K/V - sit on one XCD and hit its L2.
    int bid = blockIdx.x;
    {
        const int nb = gridDim.x;
        const int per = nb / 8;
        if (bid < per * 8) bid = (bid % 8) * per + bid / 8;
    }
    // key range of this workgroup: everything, or one of n_splits ranges of whole tiles (few query tiles on many
    // CUs; the partial results then go through fattn_merge_kernel)
    const int split = bid % a.n_splits;
    bid /= a.n_splits;
    const int k_begin = split * a.keys_per_split;
    const int k_end   = min(a.Nkv, k_begin + a.keys_per_split);
    const int qt = bid % n_qtiles;
    const int h  = (bid / n_qtiles) % a.Hq;
    const int b  = bid / (n_qtiles * a.Hq);
    const int hk = h / a.gqa;
    const int bk = b / a.bq;

    // KSP == 2: waves w and w + 2 share their queries; wave w takes keys 0..31 of every tile, wave w + 2 keys 32..63
    const int qgroup = KSP == 2 ? (wave & 1) : wave;
    const int khalf  = KSP == 2 ? (wave >> 1) : 0;
    const int q0 = qt * BMG + qgroup * BMW;        // first query of this wave

    // ---- Q -> f16 B operands, scaled so that the MFMA result is already in log2 units ----
    const float qscale = SOFTCAP ? a.scale : a.scale * LOG2E;   // a.scale is scale/softcap when capped
    // (called after the first K/V tile has been requested, so the two cold misses overlap)
    half8 qreg[NQB][KS];
    auto load_q = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int qb = 0; qb < NQB; qb++) {
        const int qi = min(q0 + qb * 32 + l32, a.Nq - 1);
        const float * qrow = (const float *)(a.q + (int64_t)qi * a.nbq1 + (int64_t)h * a.nbq2 + (int64_t)b * a.nbq3);
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            // (a head zero-padded to D: a lane with nothing to read behind Dv, a multiple of 8, reads the row's first 8
            //  elements instead and scales them by zero - loads under a guard each wait for one another.  A q row with inf
            //  or NaN in it gives NaN either way.)
            const bool    own = whole_head || ks * 16 + hh * 8 < a.Dv;
            const float * q8  = qrow + (own ? ks * 16 + hh * 8 : 0);
            const float   qs  = own ? qscale : 0.0f;
            const float4  x0  = *(const float4 *)q8;
            const float4  x1  = *(const float4 *)(q8 + 4);
            half8 v;
            v[0] = (_Float16)(x0.x * qs); v[1] = (_Float16)(x0.y * qs);
            v[2] = (_Float16)(x0.z * qs); v[3] = (_Float16)(x0.w * qs);
            v[4] = (_Float16)(x1.x * qs); v[5] = (_Float16)(x1.y * qs);
            v[6] = (_Float16)(x1.z * qs); v[7] = (_Float16)(x1.w * qs);
            qreg[qb][ks] = v;
        }
    }
    };

    const char * kbase = a.k + (int64_t)hk * a.nbk2 + (int64_t)bk * a.nbk3;
    const char * vbase = a.v + (int64_t)hk * a.nbv2 + (int64_t)bk * a.nbv3;
    const float  mslope = MASK ? fattn_slope(a, h) * LOG2E : 0.0f;
    const uint16_t * mrow[NQB];
#pragma unroll
    for (int qb = 0; qb < NQB; qb++) {
        const int qi = min(q0 + qb * 32 + l32, a.Nq - 1);
        mrow[qb] = MASK ? (const uint16_t *)(a.mask + (int64_t)(h % a.Hm) * a.nbm2 + (int64_t)(b % a.Bm) * a.nbm3 +
                                             (int64_t)qi * a.nbm1)
                        : nullptr;
    }

    // staging assignment: chunk sc of rows sr + p*RPP
    const int sc = tid % CH;
    const int sr = tid / CH;

    Raw kraw[NP], vraw[NP];
    // Rows past Nkv re-read the last row: their scores are forced to -inf in the tail tile, so any finite
    // stand-in will do, and branch-free loads let the waits on them be exact counts.
    auto load_tile = [&](int j0) {
#pragma unroll
        for (int p = 0; p < NP; p++) {
            const int key = min(j0 + sr + p * RPP, k_end - 1);
            kraw[p] = load_chunk<TYPE>(kbase + (int64_t)key * a.nbk1, sc, true);
            vraw[p] = load_chunk<TYPE>(vbase + (int64_t)key * a.nbv1, sc, true);
        }
    };
    auto store_tile = [&](int buf) {
#pragma unroll
        for (int p = 0; p < NP; p++) {
            const int row = sr + p * RPP;
            *(half8 *)&k_lds[buf][row * PK + sc * 8] = to_half8<TYPE>(kraw[p]);
            *(half8 *)&v_lds[buf][row * PV + sc * 8] = to_half8<TYPE>(vraw[p]);
        }
    };

    // DIRECT: lane's share of a tile is NLD 16-byte chunks per tensor; LDS slot L = (wave*NLD + j)*64 + lane
    // holds chunk (L % CH) ^ swizzle of row L / CH.  Offsets are relative to the tile's first row.
    uint32_t koff[DIRECT ? NLD : 1], voff[DIRECT ? NLD : 1];
    uint32_t kaddr[DIRECT ? KS : 1], vaddr[DIRECT ? DB : 1];      // operand read offsets (bytes) inside a K / V buffer
    if (DIRECT) {
#pragma unroll
        for (int j = 0; j < NLD; j++) {
            const int L = (wave * NLD + j) * 64 + lane;
            const int r = L / CH, c = L % CH;
            koff[j] = (uint32_t)r * (uint32_t)a.nbk1 + (uint32_t)((c ^ swz_k<D>(r)) * 16);
            voff[j] = (uint32_t)r * (uint32_t)a.nbv1 + (uint32_t)((c ^ swz_v<D>(r)) * 16);
        }
#pragma unroll
        for (int ks = 0; ks < KS; ks++) kaddr[ks] = (uint32_t)((l32 * CH + ((ks * 2 + hh) ^ swz_k<D>(l32))) * 16);
        const int i16 = lane & 15;
        const int kr0 = hh * 4 + (i16 >> 2);
#pragma unroll
        for (int db = 0; db < DB; db++) {
            const int c = db * 4 + ((lane >> 4) & 1) * 2 + ((i16 & 3) >> 1);
            vaddr[db] = (uint32_t)((kr0 * CH + (c ^ swz_v<D>(kr0))) * 16 + 8 * (i16 & 1));
        }
    }
    typedef uint32_t u32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));
    typedef uint32_t u32x2_a2 __attribute__((ext_vector_type(2), aligned(2)));
    typedef __attribute__((address_space(3))) void * lds_vptr;
    typedef const __attribute__((address_space(1))) void * glb_vptr;
    // MDMA: slot (row, s) of a half-tile block holds the 8 keys of chunk s ^ swizzle(row) of query q0 + row
    uint32_t moff[MDMA ? NMH : 1], maddr[MDMA ? 4 : 1];
    const char * mhead = nullptr;
    if (MDMA) {
        mhead = a.mask + (int64_t)(h % a.Hm) * a.nbm2 + (int64_t)(b % a.Bm) * a.nbm3;
#pragma unroll
        for (int j = 0; j < NMH; j++) {
            const int row = j * 16 + (lane >> 2);
            moff[j] = (uint32_t)min(q0 + row, a.Nq - 1) * (uint32_t)a.nbm1 + (uint32_t)((((lane & 3) ^ swz_m<D>(row))) * 16);
        }
#pragma unroll
        for (int g = 0; g < 4; g++) maddr[g] = (uint32_t)(l32 * 64 + ((g ^ swz_m<D>(l32)) * 16) + 8 * hh);
    }
    // half tile hf of the tile at key j0 -> this wave's block hf of mb.  `after` is a value the requests must not
    // overtake: the empty asm ties the addresses to it, so the loads issue only once it has been computed.
    auto load_mask_half = [&](int j0, int hf, char * mb, float after) __attribute__((always_inline)) {
        const char * mp = mhead + (int64_t)(j0 + hf * 32) * 2;
        char * lm = mb + wave * (2 * MHALF) + hf * MHALF;
#pragma unroll
        for (int j = 0; j < NMH; j++) {
            uint32_t mo = moff[j];
            asm volatile("" : "+v"(mo) : "v"(after));
            __builtin_amdgcn_global_load_lds((glb_vptr)(mp + mo), (lds_vptr)(lm + j * 1024), 16, 0, 0);
        }
    };

    // The tail tile's mask takes the same LDS layout through registers.  A chunk that would run past Nkv is fetched
    // from the row's last 8 valid keys instead (Nkv is even and >= 64 here, so that address is dword-aligned and
    // in bounds) and shifted down by the difference: branch-free, all loads in flight together, nothing read past
    // Nkv; the positions shifted in from beyond belong to keys that the tail tile excludes.
    auto stage_mask_tail = [&](int j0, char * mb) __attribute__((always_inline)) {
        u32x4_a4 raw[2][NMH];
        int      sh[2][NMH];
#pragma unroll
        for (int hf = 0; hf < 2; hf++)
#pragma unroll
            for (int j = 0; j < NMH; j++) {
                const int row = j * 16 + (lane >> 2);
                const int cg  = (lane & 3) ^ swz_m<D>(row);
                const int s0  = j0 + hf * 32 + 8 * cg;                     // first key of this lane's chunk
                const int sc  = min(s0, k_end - 8);
                sh[hf][j] = min(s0 - sc, 8);                               // halfwords to shift out
                // moff[j] = row offset + 16*cg, relative to key j0 + 32*hf of the head's mask
                raw[hf][j] = *(const u32x4_a4 *)(mhead + (int64_t)(j0 + hf * 32) * 2 + moff[j] - (int64_t)(s0 - sc) * 2);
            }
#pragma unroll
        for (int hf = 0; hf < 2; hf++)
#pragma unroll
            for (int j = 0; j < NMH; j++) {
                const int k = sh[hf][j];
                uint32_t e[6] = {raw[hf][j][0], raw[hf][j][1], raw[hf][j][2], raw[hf][j][3], 0u, 0u};
                if (k & 8) { e[0] = e[1] = e[2] = e[3] = 0u; }
                if (k & 4) { e[0] = e[2]; e[1] = e[3]; e[2] = 0u; e[3] = 0u; }
                if (k & 2) { e[0] = e[1]; e[1] = e[2]; e[2] = e[3]; e[3] = 0u; }
                const uint32_t bs = (k & 1) * 2;                               // bytes
                uint4 val;
                val.x = __builtin_amdgcn_alignbyte(e[1], e[0], bs);
                val.y = __builtin_amdgcn_alignbyte(e[2], e[1], bs);
                val.z = __builtin_amdgcn_alignbyte(e[3], e[2], bs);
                val.w = __builtin_amdgcn_alignbyte(e[4], e[3], bs);
                *(uint4 *)(mb + wave * (2 * MHALF) + hf * MHALF + j * 1024 + lane * 16) = val;
            }
    };
    auto load_direct = [&](int j0, char * wk, char * wv, bool tail) __attribute__((always_inline)) {
        const char * kp = kbase + (int64_t)j0 * a.nbk1;
        const char * vp = vbase + (int64_t)j0 * a.nbv1;
        char * lk = wk + wave * (NLD * 1024);
        char * lv = wv + wave * (NLD * 1024);
#pragma unroll
        for (int j = 0; j < NLD; j++) {
            uint32_t ko = koff[j], vo = voff[j];
            if (tail) {       // rows past Nkv re-read the last row (their scores are excluded)
                const int L = (wave * NLD + j) * 64 + lane;
                const int r = L / CH, c = L % CH, rr = min(r, k_end - 1 - j0);
                ko = (uint32_t)rr * (uint32_t)a.nbk1 + (uint32_t)((c ^ swz_k<D>(r)) * 16);
                vo = (uint32_t)rr * (uint32_t)a.nbv1 + (uint32_t)((c ^ swz_v<D>(r)) * 16);
            }
            __builtin_amdgcn_global_load_lds((glb_vptr)(kp + ko), (lds_vptr)(lk + j * 1024), 16, 0, 0);
            __builtin_amdgcn_global_load_lds((glb_vptr)(vp + vo), (lds_vptr)(lv + j * 1024), 16, 0, 0);
        }
    };

    // Key-split form with the mask in registers: a wave is alone on its SIMD there, so the mask values of a full tile
    // are requested a tile ahead and the check for excluded blocks does not wait on memory.
    constexpr bool MPRE = MASK && DIRECT && !MDMA && KSP == 2;
    uint2 mpre[MPRE ? NQB : 1][4];
    auto load_mask_ahead = [&](int j0) __attribute__((always_inline)) {
#pragma unroll
        for (int qb = 0; qb < NQB; qb++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const u32x2_a2 w = *(const u32x2_a2 *)(mrow[qb] + j0 + khalf * 32 + g * 8 + hh * 4);
                mpre[MPRE ? qb : 0][g].x = w[0];
                mpre[MPRE ? qb : 0][g].y = w[1];
            }
    };

    float16v oacc[NQB][DB];
    // -m in all 16 slots: the C operand of the first Q.K^T MFMA.  The masked form of 128-wide heads has no 16 registers for
    // it (it answered with spills inside the tile loop, whose reloads wait for the tile's loads): it starts from zero and
    // subtracts m with the mask.
    constexpr bool SPLAT = !SOFTCAP && (KSP == 2 || (DIRECT && !MASK) || (NQB == 1 && D == 64));
    float16v negm[SPLAT ? NQB : 1];
    RowState st[NQB];
#pragma unroll
    for (int qb = 0; qb < NQB; qb++) {
        st[qb].m = 0.0f;
        st[qb].l = 0.0f;
        st[qb].have = false;
#pragma unroll
        for (int r = 0; r < 16; r++) negm[SPLAT ? qb : 0][r] = 0.0f;
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
            for (int r = 0; r < 16; r++) oacc[qb][db][r] = 0.0f;
    }

    // One tile of 64 keys.  TAIL: the tile runs past Nkv (keys beyond it are excluded).
    // DIRECT: operands are read from rk / rv while the tile at key jn (if any) is requested into wk / wv.  The four
    // are distinct buffers, and saying so (restrict) is what lets the compiler keep the operand reads from
    // waiting on the loads that have just been issued.
    auto tile = [&](const int j0, const int buf, auto tail_tag, const char * __restrict__ rk, const char * __restrict__ rv,
                    char * __restrict__ wk, char * __restrict__ wv, const int jn, const bool tn, char * __restrict__ mb,
                    const bool mn) __attribute__((always_inline)) {
        constexpr bool TAIL = decltype(tail_tag)::value;
        constexpr bool MLDS = MDMA;                   // this tile's mask is in LDS (mn: so will the next tile's be)
        // mask of keys 32..63 of this tile: its block was last read before the barrier that ended the previous tile
        // (the tail tile's mask is staged whole before the tile starts)
        if (MLDS && !TAIL) load_mask_half(j0, 1, mb, 0.0f);
        if (DIRECT && jn >= 0) load_direct(jn, wk, wv, tn);

        // additive mask values of this lane's 16 (key, query) pairs per query block and 32-key block, fetched early
        uint2 mraw[MLDS ? 1 : NQB][NKB][4];
        if (MPRE && !TAIL) {
#pragma unroll
            for (int qb = 0; qb < NQB; qb++)
#pragma unroll
                for (int g = 0; g < 4; g++) mraw[MLDS ? 0 : qb][0][g] = mpre[MPRE ? qb : 0][g];
            if (mn) load_mask_ahead(j0 + BC);
        } else if (MASK && !MLDS) {
#pragma unroll
            for (int qb = 0; qb < NQB; qb++)
#pragma unroll
                for (int kbi = 0; kbi < NKB; kbi++)
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        const int key = j0 + (KSP == 2 ? khalf * NKB + kbi : kbi) * 32 + g * 8 + hh * 4;
                        // Past Nkv the loads are clamped to the row's last valid pair (or element): branch-free and in
                        // bounds; what they return belongs to keys that the tail tile excludes anyway.
                        if (!TAIL) {
                            // one 8-byte load whether the row starts on 8 bytes, on a dword or only on a halfword (an odd
                            // Nkv): the memory pipeline takes it at any halfword
                            const u32x2_a2 w = *(const u32x2_a2 *)(mrow[qb] + key);
                            mraw[qb][kbi][g].x = w[0];
                            mraw[qb][kbi][g].y = w[1];
                        } else if (a.mask_al4 && !(k_end & 1)) {
                            const int k0 = min(key, k_end - 2), k1 = min(key + 2, k_end - 2);
                            mraw[qb][kbi][g].x = *(const uint32_t *)(mrow[qb] + k0);
                            mraw[qb][kbi][g].y = *(const uint32_t *)(mrow[qb] + k1);
                        } else {
                            uint16_t mv[4];
#pragma unroll
                            for (int e = 0; e < 4; e++) mv[e] = mrow[qb][min(key + e, k_end - 1)];
                            mraw[qb][kbi][g].x = (uint32_t)mv[0] | ((uint32_t)mv[1] << 16);
                            mraw[qb][kbi][g].y = (uint32_t)mv[2] | ((uint32_t)mv[3] << 16);
                        }
                    }
        }

        // K operands of a 32-key block: KS 128-bit reads per lane
        auto load_k = [&](int kb, half8 (&ka)[KS]) {
#pragma unroll
            for (int ks = 0; ks < KS; ks++)
                ka[ks] = DIRECT ? *(const half8 *)(rk + kaddr[ks] + kb * 32 * ROWB)
                                : *(const half8 *)&k_lds[buf][(kb * 32 + l32) * PK + ks * 16 + hh * 8];
        };
        // V^T operands of a 32-key block by transpose reads: lane i of a 16-lane block addresses
        // 4 halves of key (i/4) at d0 + 4*(i%4) and receives 4 keys' values of d0 + i
        auto load_v = [&](int kb, half8 (&va)[2][DB]) {
            const int i16 = lane & 15;
#pragma unroll
            for (int k2 = 0; k2 < 2; k2++)
#pragma unroll
                for (int db = 0; db < DB; db++) {
                    const int d0 = db * 32 + ((lane >> 4) & 1) * 16;
                    const int kr = (kb * 2 + k2) * 16 + hh * 4 + (i16 >> 2);
                    const _Float16 * p0 = DIRECT ? (const _Float16 *)(rv + vaddr[db] + (kb * 2 + k2) * 16 * ROWB)
                                                 : &v_lds[buf][kr * PV + d0 + (i16 & 3) * 4];
                    const _Float16 * p1 = p0 + 8 * (DIRECT ? D : PV);
                    const half4 lo = __builtin_bit_cast(half4, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4v *)p0));
                    const half4 hi = __builtin_bit_cast(half4, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4v *)p1));
                    va[k2][db] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                }
        };

        // with few reduction steps the next block's K operands are requested a block ahead
        constexpr bool K_AHEAD = KS <= 4 && NKB >= 2;
        half8 ka[K_AHEAD ? 2 : 1][KS];
        load_k(KSP == 2 ? khalf * NKB : 0, ka[0]);

        // the tile is consumed in blocks of 32 keys to keep the score registers few
#pragma unroll
        for (int kbi = 0; kbi < NKB; kbi++) {
            const int kb = KSP == 2 ? khalf * NKB + kbi : kbi;      // which 32 keys of the tile
            if (MLDS && kbi == 1 && !TAIL) {
                // the second half was requested when the tile began; younger than it are the next tile's K and V (requested
                // right behind it) and the next tile's first mask half (behind block 0).  Loads return in order, so waiting
                // until no more than those are outstanding is waiting for the half - and not for the K/V tile, which
                // has until the end of this tile to land
                static_assert(!MDMA || 2 * NLD + NMH <= 15, "wait count encoding");
                if (mn)           __builtin_amdgcn_s_waitcnt(0x0F70 | (2 * NLD + NMH));
                else if (jn >= 0) __builtin_amdgcn_s_waitcnt(0x0F70 | (2 * NLD));
                else              __builtin_amdgcn_s_waitcnt(0x0F70);
            }
            // A block that the mask excludes altogether for this wave's queries - every entry -inf - contributes exact
            // zeros: it is skipped (wave-uniform), and the softmax state stays as it is.
            // The block's mask values leave LDS first, in one go and ahead of the operand reads below: LDS answers a wave in
            // order, so a mask read issued behind those would make its consumer wait for all of them (and four reads issued
            // one by one between the additions, as the compiler places them when left to itself, expose four round trips).
            uint2 mval[NQB][4];
            auto read_mask = [&]() __attribute__((always_inline)) {
#pragma unroll
                for (int qb = 0; qb < NQB; qb++)
#pragma unroll
                    for (int g = 0; g < 4; g++)
                        mval[qb][g] = MLDS ? *(const uint2 *)(mb + wave * (2 * MHALF) + kb * MHALF + qb * 2048 + maddr[g])
                                           : mraw[MLDS ? 0 : qb][kbi][g];
                if (MLDS) __builtin_amdgcn_sched_barrier(0);
            };
            if (SKIP) read_mask();          // (needed for the test below; the other forms read behind the score MFMAs)
            bool     excluded = false;
            uint32_t mdiff    = 0;
            if (SKIP) {
#pragma unroll
                for (int qb = 0; qb < NQB; qb++)
#pragma unroll
                    for (int g = 0; g < 4; g++) mdiff |= (mval[qb][g].x ^ 0xFC00FC00u) | (mval[qb][g].y ^ 0xFC00FC00u);
                excluded = __builtin_amdgcn_ballot_w64(mdiff != 0) == 0;
            }
            if (excluded) {
                if (kbi + 1 < NKB) load_k(kb + 1, ka[K_AHEAD ? (kbi + 1) & 1 : 0]);
                if (MLDS && kbi == 0 && !TAIL && mn) load_mask_half(j0 + BC, 0, mb, __uint_as_float(mdiff));
                continue;
            }
            // ---- S^T = K . Q^T - m  (the reference m enters as the C operand of the first MFMA) ----
            float16v s[NQB];
#pragma unroll
            for (int qb = 0; qb < NQB; qb++) {
                if (!SPLAT) {           // (the cap applies to the raw score: m is subtracted afterwards)
#pragma unroll
                    for (int r = 0; r < 16; r++) s[qb][r] = 0.0f;
                } else {
                    s[qb] = negm[qb];
                }
            }
#pragma unroll
            for (int ks = 0; ks < KS; ks++)
#pragma unroll
                for (int qb = 0; qb < NQB; qb++)
                    s[qb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ka[K_AHEAD ? kbi & 1 : 0][ks], qreg[qb][ks], s[qb], 0, 0, 0);
            if (MASK && !SKIP) read_mask();
            // operands needed next are requested now, so their LDS latency hides behind the softmax
            half8 va[2][DB];
            load_v(kb, va);
            if (kbi + 1 < NKB) load_k(kb + 1, ka[K_AHEAD ? (kbi + 1) & 1 : 0]);

            // ---- soft cap (this path subtracts m explicitly), mask, key tail -----------------------------
            if (SOFTCAP) {
                const float c2 = a.softcap * LOG2E;
#pragma unroll
                for (int qb = 0; qb < NQB; qb++)
#pragma unroll
                    for (int r = 0; r < 16; r++) s[qb][r] = c2 * fast_tanh(s[qb][r]);
            }
            if (MASK) {
#pragma unroll
                for (int qb = 0; qb < NQB; qb++)
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        // f16 halves enter the FMA directly (mixed-precision FMA, no separate conversion)
                        const uint2 mv = mval[qb][g];
                        const half2v w[2] = {__builtin_bit_cast(half2v, mv.x), __builtin_bit_cast(half2v, mv.y)};
#pragma unroll
                        for (int e = 0; e < 4; e++)
                            s[qb][g * 4 + e] = fmaf(mslope, (float)w[e >> 1][e & 1], s[qb][g * 4 + e]);
                    }
            }
            if (!SPLAT) {
#pragma unroll
                for (int qb = 0; qb < NQB; qb++)
#pragma unroll
                    for (int r = 0; r < 16; r++) s[qb][r] -= st[qb].m;
            }
            if (TAIL) {
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int key = j0 + kb * 32 + (r >> 2) * 8 + hh * 4 + (r & 3);
                    if (key >= k_end) {
#pragma unroll
                        for (int qb = 0; qb < NQB; qb++) s[qb][r] = -INFINITY;
                    }
                }
            }

            // ---- P = 2^s in f16; the row sum is taken over the rounded values the MFMA will use -----------
            // No maximum is computed on this path: a reference that has fallen too far behind shows up
            // as a large (or infinite) block sum, and only then is the block redone with a new reference.
            half8 preg[NQB][2];
            float lsum[NQB];
            const half2v ones = {(_Float16)1.0f, (_Float16)1.0f};
            // With 64-wide heads the sum goes through the matrix pipe as well: v_mfma_f32_4x4x4_16b_f16 with A = ones
            // adds the four f16 values a lane supplies as B into that lane's own f32 accumulators (16 independent 4x4
            // blocks, lane = (block, column); all four rows of the result are equal) - exact products, f32
            // accumulation, and the VALU, the busier pipe of that loop, has 32 instructions less per tile.  128-wide
            // heads have no registers to spare for the accumulators and keep the packed dot product.
            constexpr bool MFMA_SUMS = D == 64;
            auto exp_block = [&](int qb) {
                float dsum = 0.0f;
#pragma unroll
                for (int r = 0; r < 16; r += 2) {
                    half2v p2;
                    p2[0] = (_Float16)__builtin_amdgcn_exp2f(s[qb][r]);
                    p2[1] = (_Float16)__builtin_amdgcn_exp2f(s[qb][r + 1]);
                    if (!MFMA_SUMS) dsum = __builtin_amdgcn_fdot2(p2, ones, dsum, false);
                    preg[qb][r >> 3][r & 7]       = p2[0];
                    preg[qb][r >> 3][(r & 7) + 1] = p2[1];
                }
                if (MFMA_SUMS) {
                    const half4 ones4 = {(_Float16)1.0f, (_Float16)1.0f, (_Float16)1.0f, (_Float16)1.0f};
                    float4v acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                    for (int h = 0; h < 2; h++) {
                        acc = __builtin_amdgcn_mfma_f32_4x4x4f16(ones4, __builtin_shufflevector(preg[qb][h], preg[qb][h], 0, 1, 2, 3), acc, 0, 0, 0);
                        acc = __builtin_amdgcn_mfma_f32_4x4x4f16(ones4, __builtin_shufflevector(preg[qb][h], preg[qb][h], 4, 5, 6, 7), acc, 0, 0, 0);
                    }
                    dsum = acc[0];
                }
                lsum[qb] = dsum;
            };
            bool redo = false;
#pragma unroll
            for (int qb = 0; qb < NQB; qb++) {
                exp_block(qb);
                redo = redo || !(lsum[qb] <= SUM_LIMIT) || !st[qb].have;
            }
            if (__builtin_amdgcn_ballot_w64(redo) != 0) {        // wave-uniform; rare after the first block
#pragma unroll
                for (int qb = 0; qb < NQB; qb++) {
                    float mx = s[qb][0];
#pragma unroll
                    for (int r = 1; r < 16; r++) mx = fmaxf(mx, s[qb][r]);
                    const float tm = max_xor32(mx);              // both halves of a query must agree
                    float delta = 0.0f;
                    if (tm > -INFINITY) {
                        delta = st[qb].have ? fmaxf(tm, 0.0f) : tm;
                        st[qb].have = true;
                    }
                    const float f = __builtin_amdgcn_exp2f(-delta);
                    st[qb].m += delta;
                    st[qb].l *= f;
#pragma unroll
                    for (int r = 0; r < 16; r++) negm[SPLAT ? qb : 0][r] = -st[qb].m;
#pragma unroll
                    for (int db = 0; db < DB; db++)
#pragma unroll
                        for (int r = 0; r < 16; r++) oacc[qb][db][r] *= f;
#pragma unroll
                    for (int r = 0; r < 16; r++) s[qb][r] -= delta;
                    exp_block(qb);
                }
            }
#pragma unroll
            for (int qb = 0; qb < NQB; qb++) st[qb].l += lsum[qb];
            if (MLDS && kbi == 0 && !TAIL && mn) {
                // block 0's mask has been consumed - the sums below depend on every value of it - so its LDS
                // block can take the next tile's
                load_mask_half(j0 + BC, 0, mb, lsum[0] + lsum[NQB - 1]);
            }

            // ---- O^T += V^T . P^T ------------------------------------------------------------------------------
#pragma unroll
            for (int k2 = 0; k2 < 2; k2++)
#pragma unroll
                for (int db = 0; db < DB; db++)
#pragma unroll
                    for (int qb = 0; qb < NQB; qb++)
                        oacc[qb][db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(va[k2][db], preg[qb][k2], oacc[qb][db], 0, 0, 0);
        }
    };

    const int n_tiles = (k_end - k_begin + BCT - 1) / BCT;
    const int n_full  = (k_end - k_begin) / BCT;
    if (DIRECT) {
        char * const lb = (char *)lds_raw;               // K0 K1 V0 V1 [mask: per wave 2 half-tile blocks]
        char * const mb = lb + 4 * TILEB;
        load_direct(k_begin, lb, lb + 2 * TILEB, n_full == 0);
        if (MDMA && n_full > 0) load_mask_half(k_begin, 0, mb, 0.0f);
        if (MPRE && n_full > 0) load_mask_ahead(k_begin);
        load_q();
        __builtin_amdgcn_s_waitcnt(0x0F70);          // vmcnt(0): this wave's share of the tile is in LDS
        __syncthreads();
        // Two workgroups share a CU, and the SIMD's arbiter prefers the older wave: left alone, the first
        // workgroup runs at full speed and the second finishes its last third alone, at one wave per SIMD.  Waves
        // therefore take the higher priority in alternating time slices (workgroups i and i + n_cus are the ones
        // that meet on a CU), so that both finish together.
        const int  prio_phase = a.n_cus > 0 ? (blockIdx.x / a.n_cus) & 1 : 0;
        const bool shared_cu  = a.n_cus > 0 && (int)gridDim.x > a.n_cus;
        for (int t = 0; t < n_full; t++) {
            if (shared_cu) {
                if (((int)(clock64() >> 12) ^ prio_phase) & 1) __builtin_amdgcn_s_setprio(2);
                else                                            __builtin_amdgcn_s_setprio(0);
            }
            const int  cur = (t & 1) * TILEB, nxt = TILEB - cur;
            const int  jn  = t + 1 < n_tiles ? k_begin + (t + 1) * BCT : -1;
            const bool mn  = (MDMA || MPRE) && t + 1 < n_full;     // the next tile's mask is requested during this one
            tile(k_begin + t * BCT, 0, std::false_type{}, lb + cur, lb + 2 * TILEB + cur, lb + nxt, lb + 2 * TILEB + nxt, jn, t + 1 >= n_full, mb, mn);
            // everything requested during the tile has had at least half a tile to land
            __builtin_amdgcn_s_waitcnt(0x0F70);
            __syncthreads();
        }
        __builtin_amdgcn_s_setprio(0);
        if (n_full < n_tiles) {
            const int cur = (n_full & 1) * TILEB;
            if (MDMA) stage_mask_tail(k_begin + n_full * BCT, mb);
            tile(k_begin + n_full * BCT, 0, std::true_type{}, lb + cur, lb + 2 * TILEB + cur, nullptr, nullptr, -1, false, mb, false);
        }
    } else {
    load_tile(k_begin);
    load_q();
    store_tile(0);
    __syncthreads();

    // full tiles: the steady-state loop carries no tail handling at all
    for (int t = 0; t < n_full; t++) {
        const int  buf  = t & 1;
        const bool more = t + 1 < n_tiles;
        if (more) load_tile(k_begin + (t + 1) * BC);
        tile(k_begin + t * BC, buf, std::false_type{}, nullptr, nullptr, nullptr, nullptr, -1, false, nullptr, false);
        if (more) store_tile(buf ^ 1);
        __syncthreads();
    }
    // at most one partial tile, already staged by the last iteration above (or the prologue)
    if (n_full < n_tiles) tile(k_begin + n_full * BC, n_full & 1, std::true_type{}, nullptr, nullptr, nullptr, nullptr, -1, false, nullptr, false);
    }

    // ---- key-split form: the pair's second wave hands its state to the first through LDS (free now) ---------------
    if (KSP == 2) {
        constexpr int XREGS = DB * 16 + 2;                 // accumulators, reference, sum: one dword per lane each
        __syncthreads();                                   // every wave is done with the tile buffers
        float * xs = (float *)lds_raw + qgroup * (XREGS * 64) + lane;
        if (khalf == 1) {
#pragma unroll
            for (int db = 0; db < DB; db++)
#pragma unroll
                for (int r = 0; r < 16; r++) xs[(db * 16 + r) * 64] = oacc[0][db][r];
            xs[(DB * 16) * 64]     = st[0].have ? st[0].m : -INFINITY;
            xs[(DB * 16 + 1) * 64] = st[0].l;
        }
        __syncthreads();
        if (khalf == 1) return;
        const float mo = xs[(DB * 16) * 64], lo = xs[(DB * 16 + 1) * 64];
        const bool  ho = mo > -INFINITY;
        const float mn = fmaxf(st[0].have ? st[0].m : -INFINITY, mo);
        const float fa = st[0].have ? __builtin_amdgcn_exp2f(st[0].m - mn) : 0.0f;
        const float fo = ho ? __builtin_amdgcn_exp2f(mo - mn) : 0.0f;
        st[0].l = st[0].l * fa + lo * fo;
#pragma unroll
        for (int db = 0; db < DB; db++)
#pragma unroll
            for (int r = 0; r < 16; r++) oacc[0][db][r] = oacc[0][db][r] * fa + xs[(db * 16 + r) * 64] * fo;
        st[0].have = st[0].have || ho;
        st[0].m    = st[0].have ? mn : 0.0f;
    }

    // ---- normalise and write dst[D, Hq, Nq, B], or hand the unnormalised partial to the merge kernel --------------
    // Two query blocks per wave (the large grids, where the output is a third of the launch's bytes) take the rows through
    // LDS; the other forms, whose launches are short, store from the accumulator layout (the detour costs them a
    // barrier and a round trip: the Whisper-base encoder layer 17.5 -> 18.4 us, against 61.4 -> 60.3 us on large-v3's).
    constexpr bool OUT_LDS = NQB == 2;
    // Excluded keys were multiplied by probabilities of exactly zero, not skipped: the same for finite K/V, NaN for a cache
    // slot that holds NaN or inf bits (never written, and masked out for that reason).  A query whose sum or accumulators
    // are not finite is noted here and computed again below the way the CPU op does it.  (x * 0 is 0 for every finite x.)
    uint64_t badbits[NQB];
    if constexpr (MASK) {
#pragma unroll
        for (int qb = 0; qb < NQB; qb++) {
            float chk = st[qb].l * 0.0f;
#pragma unroll
            for (int db = 0; db < DB; db++)
#pragma unroll
                for (int r = 0; r < 16; r++) chk = fmaf(oacc[qb][db][r], 0.0f, chk);
            badbits[qb] = __builtin_amdgcn_ballot_w64(chk != 0.0f);         // NaN != 0
        }
    }
    if constexpr (OUT_LDS) {
        // A lane holds 16-byte pieces of its query's row, 32 bytes apart: stored from there, one instruction scatters 64
        // quarter-lines over 32 rows.  The rows go through LDS instead (free now: 32 x D floats per wave, chunks XOR-swizzled
        // by row), and come back with 16 (D = 64) or 32 adjacent lanes on one row: whole 256- or 512-byte rows per request.
        constexpr int CPR = D / 4;                         // 16-byte chunks per output row
        constexpr int RPI = 64 / CPR;                      // rows per store instruction
        __syncthreads();                                   // every wave is done with the tile buffers
        float * const stg = (float *)lds_raw + qgroup * (32 * D);
        const int64_t row_stride = a.n_splits > 1 ? (int64_t)a.Hq * a.n_splits * D : (int64_t)a.Hq * D;    // floats between queries
#pragma unroll
        for (int qb = 0; qb < NQB; qb++) {
            const float ltot = sum_xor32(st[qb].l);
            const float inv  = a.n_splits > 1 ? 1.0f : (ltot > 0.0f ? 1.0f / ltot : 0.0f);
            const int   qi   = q0 + qb * 32 + l32;
#pragma unroll
            for (int db = 0; db < DB; db++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    float4 o;
                    o.x = oacc[qb][db][g * 4 + 0] * inv;
                    o.y = oacc[qb][db][g * 4 + 1] * inv;
                    o.z = oacc[qb][db][g * 4 + 2] * inv;
                    o.w = oacc[qb][db][g * 4 + 3] * inv;
                    const int c = db * 8 + g * 2 + hh;
                    *(float4 *)(stg + l32 * D + ((c ^ (l32 & (CPR - 1))) * 4)) = o;
                }
            __builtin_amdgcn_wave_barrier();               // (LDS serves a wave's requests in order)
            const int     q_first = q0 + qb * 32;
            const int64_t row0    = ((int64_t)b * a.Nq + q_first) * a.Hq + h;
            float * const out0    = a.n_splits > 1 ? a.part_acc + (row0 * a.n_splits + split) * D : a.dst + row0 * D;
#pragma unroll
            for (int k = 0; k < 32 / RPI; k++) {
                const int row = k * RPI + lane / CPR, c = lane % CPR;
                const float4 o = *(const float4 *)(stg + row * D + ((c ^ (row & (CPR - 1))) * 4));
                // whole rows, written once: marked non-temporal (encoder launch 2% shorter; the scattered quarter-lines of
                // the direct form were 12 us slower with the mark)
                typedef float f32x4 __attribute__((ext_vector_type(4)));
                if (q_first + row < a.Nq) __builtin_nontemporal_store(f32x4{o.x, o.y, o.z, o.w}, (f32x4 *)(out0 + row * row_stride + c * 4));
            }
            __builtin_amdgcn_wave_barrier();               // the next query block reuses the staging rows
            if (a.n_splits > 1 && hh == 0 && qi < a.Nq) {
                // (reference, sum) in natural-log units; a range with no visible key contributes nothing
                const int64_t row = ((int64_t)b * a.Nq + qi) * a.Hq + h;
                float * pm = a.part_ml + (row * a.n_splits + split) * 2;
                pm[0] = st[qb].have ? st[qb].m * 0.6931471805599453f : -INFINITY;
                pm[1] = ltot;
            }
        }
    } else {
#pragma unroll
        for (int qb = 0; qb < NQB; qb++) {
            const float ltot = sum_xor32(st[qb].l);
            const float inv  = a.n_splits > 1 ? 1.0f : (ltot > 0.0f ? 1.0f / ltot : 0.0f);
            const int   qi   = q0 + qb * 32 + l32;
            if (qi < a.Nq) {
                const int64_t row = ((int64_t)b * a.Nq + qi) * a.Hq + h;
                // (a zero-padded head, Dv < D: dst rows are Dv floats apart and end there; partial rows are D apart)
                float * out = a.n_splits > 1 ? a.part_acc + (row * a.n_splits + split) * D : a.dst + row * (PAD ? a.Dv : D);
#pragma unroll
                for (int db = 0; db < DB; db++)
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        float4 o;
                        o.x = oacc[qb][db][g * 4 + 0] * inv;
                        o.y = oacc[qb][db][g * 4 + 1] * inv;
                        o.z = oacc[qb][db][g * 4 + 2] * inv;
                        o.w = oacc[qb][db][g * 4 + 3] * inv;
                        if (whole_head || db * 32 + g * 8 + hh * 4 < a.Dv) *(float4 *)(out + db * 32 + g * 8 + hh * 4) = o;
                    }
                if (a.n_splits > 1 && hh == 0) {
                    // (reference, sum) in natural-log units; a range with no visible key contributes nothing
                    float * pm = a.part_ml + (row * a.n_splits + split) * 2;
                    pm[0] = st[qb].have ? st[qb].m * 0.6931471805599453f : -INFINITY;
                    pm[1] = ltot;
                }
            }
        }
    }
    // the queries noted above, one row at a time by the whole wave (lanes l and l + 32 hold the same query); the wave
    // that stored a row is the one that stores it again
    if constexpr (MASK) {
        uint64_t any = 0;
#pragma unroll
        for (int qb = 0; qb < NQB; qb++) any |= badbits[qb];
        if (any != 0) {
            __threadfence();
#pragma unroll 1
            for (int qb = 0; qb < NQB; qb++) {
                uint32_t bits = (uint32_t)badbits[qb] | (uint32_t)(badbits[qb] >> 32);
                while (bits != 0) {
                    const int qi = q0 + qb * 32 + __builtin_ctz(bits);
                    bits &= bits - 1;
                    if (qi < a.Nq) attn_row_redo<TYPE, D>(a, qi, h, b, split, k_begin, k_end);
                }
            }
        }
    }
}

template <int D, int NQB, int KSP, int TYPE, bool MASK, bool SOFTCAP, bool DIRECT, bool MDMA, int TK, bool PAD>
int launch_kernel(const FattnArgs & a, hipStream_t stream) {
    const int bmg = 32 * NQB * MMA_WAVES / KSP;
    const int n_qtiles = (a.Nq + bmg - 1) / bmg;
    if ((int64_t)n_qtiles * a.Hq * a.B * a.n_splits > 0x7fffffff) return (int)hipErrorInvalidValue;
    const dim3 grid((unsigned)((int64_t)n_qtiles * a.Hq * a.B * a.n_splits));
    const size_t lds = DIRECT ? (size_t)4 * TK * D * sizeof(_Float16) + (MDMA ? (size_t)MMA_WAVES * NQB * 4096 : 0)
                              : (size_t)2 * BC * (Pitch<D>::K + Pitch<D>::V) * sizeof(_Float16);
    static std::atomic<uint64_t> lds_allowed{0};     // per instantiation
    const hipError_t ea = fattn_allow_lds((const void *)fattn_mma_kernel<D, NQB, KSP, TYPE, MASK, SOFTCAP, DIRECT, MDMA, TK, PAD>, (int)lds, lds_allowed);
    if (ea != hipSuccess) return (int)ea;
    static const bool debug = getenv("MI355X_FATTN_DEBUG") != nullptr;
    if (debug) {
        int nb = -1;
        (void)hipOccupancyMaxActiveBlocksPerMultiprocessor(&nb, (const void *)fattn_mma_kernel<D, NQB, KSP, TYPE, MASK, SOFTCAP, DIRECT, MDMA, TK, PAD>, MMA_THREADS, lds);
        fprintf(stderr, "[mi355x] fattn_mma<%d,%d,%d,%d,%d,%d,%d,%d> grid %u lds %zu B, resident workgroups per CU: %d\n",
                D, NQB, KSP, TYPE, (int)MASK, (int)SOFTCAP, (int)DIRECT, (int)MDMA, grid.x, lds, nb);
    }
    hipLaunchKernelGGL((fattn_mma_kernel<D, NQB, KSP, TYPE, MASK, SOFTCAP, DIRECT, MDMA, TK, PAD>), grid, dim3(MMA_THREADS), lds, stream, a, n_qtiles);
    return (int)hipGetLastError();
}

template <int D, int NQB, int KSP, int TYPE, bool MASK, bool SOFTCAP, bool DIRECT, bool MDMA, int TK = BC>
int launch(const FattnArgs & a, hipStream_t stream) {
    if (a.Dv != a.D) {              // a zero-padded head: the forms that exist for it, or none
        if constexpr (DIRECT && NQB == 1) return launch_kernel<D, NQB, KSP, TYPE, MASK, SOFTCAP, DIRECT, MDMA, TK, true>(a, stream);
        return (int)hipErrorInvalidValue;
    }
    return launch_kernel<D, NQB, KSP, TYPE, MASK, SOFTCAP, DIRECT, MDMA, TK, false>(a, stream);
}

template <int D, int NQB, int KSP, int TYPE, bool DIRECT>
int launch_mask(const FattnArgs & a, const FattnMmaVariant & v, hipStream_t stream) {
    const bool mask = a.mask != nullptr;
    if (KSP == 1 && a.softcap != 0.0f)
        return mask ? launch<D, NQB, 1, TYPE, true, true, DIRECT, false>(a, stream) : launch<D, NQB, 1, TYPE, false, true, DIRECT, false>(a, stream);
    if (!mask) {
        if constexpr (KSP == 2 && D == 64 && DIRECT) {
            const int64_t wgs = (int64_t)((a.Nq + 63) / 64) * a.Hq * a.B * a.n_splits;
            if (a.n_cus > 0 && wgs <= a.n_cus) return launch<D, NQB, KSP, TYPE, false, false, DIRECT, false, 4 * BC>(a, stream);
            return launch<D, NQB, KSP, TYPE, false, false, DIRECT, false, 2 * BC>(a, stream);
        } else {
            return launch<D, NQB, KSP, TYPE, false, false, DIRECT, false>(a, stream);
        }
    }
    if (KSP == 1 && DIRECT && v.mask_dma) return launch<D, NQB, 1, TYPE, true, false, DIRECT, DIRECT>(a, stream);
    return launch<D, NQB, KSP, TYPE, true, false, DIRECT, false>(a, stream);
}

template <int D, int NQB, int KSP, int TYPE>
int launch_flags(const FattnArgs & a, const FattnMmaVariant & v, hipStream_t stream) {
    if (TYPE == MI355X_TYPE_F16 && v.direct) return launch_mask<D, NQB, KSP, MI355X_TYPE_F16, true>(a, v, stream);
    return launch_mask<D, NQB, KSP, TYPE, false>(a, v, stream);
}

template <int TYPE>
int launch_type(const FattnArgs & a, const FattnMmaVariant & v, hipStream_t stream) {
    // the key-split form exists for f16 K/V (what F32 and Q8_0 caches have become by now when there are >= 128 queries)
    constexpr bool SPLITTABLE = TYPE == MI355X_TYPE_F16;
    if (a.D == 64) {
        if (v.query_blocks == 2) return launch_flags<64, 2, 1, TYPE>(a, v, stream);
        if (SPLITTABLE && v.key_split == 2) return launch_flags<64, 1, SPLITTABLE ? 2 : 1, TYPE>(a, v, stream);
        return launch_flags<64, 1, 1, TYPE>(a, v, stream);
    }
    if (a.D == 128) {
        if (SPLITTABLE && v.key_split == 2) return launch_flags<128, 1, SPLITTABLE ? 2 : 1, TYPE>(a, v, stream);
        return launch_flags<128, 1, 1, TYPE>(a, v, stream);
    }
    return (int)hipErrorInvalidValue;
}

}  // namespace

// Which instantiation a call takes (also what mi355x_fattn_plan_info reports):
//  - two query blocks per wave (256 queries per workgroup) halve the LDS operand traffic per MFMA; one block keeps
//    more workgroups in flight when there are few queries;
//  - the key-split form (64 queries per workgroup) when 128-query workgroups leave CUs empty or alone;
//  - f16 rows go straight to LDS when a tile's row offsets fit 32 bits;
//  - the mask follows K/V through LDS when its rows start on dwords, Nkv is even (the tail tile's dword-aligned
//    stand-in chunk) and a wave's row offsets fit 32 bits.
void fattn_mma_variant(const FattnArgs & a, int ktype, FattnMmaVariant & v) {
    static const char * force_nqb = getenv("MI355X_FATTN_NQB");               // experiments only
    static const char * force_ksp = getenv("MI355X_FATTN_KSP");
    static const bool   no_direct = getenv("MI355X_FATTN_NO_DIRECT") != nullptr;
    static const bool   no_mdma   = getenv("MI355X_FATTN_NO_MDMA") != nullptr;
    const int64_t heads = (int64_t)a.Hq * a.B;
    const int64_t wg2 = (int64_t)((a.Nq + 255) / 256) * heads;
    const int64_t wg1 = (int64_t)((a.Nq + 127) / 128) * heads;
    const int     cus = a.n_cus > 0 ? a.n_cus : 256;
    const int want_nqb = a.tile_variant ? (a.tile_variant & 15) : force_nqb ? atoi(force_nqb) : 0;
    const int want_ksp = a.tile_variant ? (a.tile_variant >> 4) : force_ksp ? atoi(force_ksp) : 0;
    // Measured over square shapes of 128 .. 2500 tokens x 8 .. 160 heads, with and without a mask: two query blocks pay
    // from one workgroup per CU on, and only where 256-query workgroups cover the queries about as tightly as 128-query
    // ones (300 queries: 512 slots against 384); the key split pays up to about half a workgroup per CU, and up to a
    // whole one when the key loop is long enough to carry its merge.
    const int64_t slots1 = (int64_t)(a.Nq + 127) / 128 * 128, slots2 = (int64_t)(a.Nq + 255) / 256 * 256;
    const bool two_auto = wg2 >= cus && slots2 * 10 <= slots1 * 11;
    // (With a mask the split form, which skips excluded blocks, carries its merge from 512 keys on; and a mask whose rows
    // cannot go through LDS costs the unsplit forms a quarter of their speed: there the split form wins up to 1.6
    // workgroups per CU.)
    // (a zero-padded head exists in the direct forms only: its K/V are the call's own f16 copies)
    const bool direct = ktype == MI355X_TYPE_F16 && (!no_direct || a.Dv != a.D) && a.nbk1 < (1u << 24) && a.nbv1 < (1u << 24);
    const bool mdma_ok = a.masked && a.softcap == 0.0f && direct && !no_mdma && a.mask_al4 && a.Nkv >= 64 && !(a.Nkv & 1) &&
                         (uint64_t)a.Nq * a.nbm1 < (1ull << 31);
    bool ksp_auto;
    if (a.D == 128)           ksp_auto = wg1 * 2 <= cus || (wg1 <= cus && a.Nkv >= 2048);
    else if (!a.masked)       ksp_auto = wg1 <= cus && (wg1 * 5 <= (int64_t)cus * 3 || a.Nkv >= 1024) && a.Nkv > 128;
    else if (!mdma_ok && a.Nkv >= 256) ksp_auto = wg1 * 5 <= (int64_t)cus * 8;
    else                      ksp_auto = wg1 <= cus && (wg1 * 5 <= (int64_t)cus * 3 || a.Nkv >= 512);
    // (a head zero-padded to 64 keeps to one query block: the two-block form stores whole rows of D floats)
    const bool two  = a.D == 64 && a.Dv == a.D && (want_nqb ? want_nqb == 2 : two_auto);
    const bool ksp2 = !two && ktype == MI355X_TYPE_F16 && a.softcap == 0.0f && (want_ksp ? want_ksp == 2 : ksp_auto);
    v.query_blocks = two ? 2 : 1;
    v.key_split    = ksp2 ? 2 : 1;
    v.queries_per_workgroup = 32 * v.query_blocks * MMA_WAVES / v.key_split;
    v.direct   = direct;
    v.mask_dma = mdma_ok && !ksp2;
}

bool fattn_mma_supported(const FattnArgs & a, int ktype) {
    if (a.D != 64 && a.D != 128) return false;
    if (a.Dv != a.D && (a.Dv % 8 || a.Dv > a.D || ktype != MI355X_TYPE_F16)) return false;     // zero-padded heads
    if (a.Nq < 1 || a.Nkv < 1) return false;
    if (ktype != MI355X_TYPE_Q8_0 && !a.aligned16) return false;   // 128-bit K/V loads
    if (ktype == MI355X_TYPE_Q8_0 && !a.q_aligned16) return false;
    return ktype == MI355X_TYPE_F16 || ktype == MI355X_TYPE_F32 || ktype == MI355X_TYPE_Q8_0;
}

int fattn_mma_launch(const FattnArgs & a, int ktype, hipStream_t stream) {
    FattnMmaVariant v;
    fattn_mma_variant(a, ktype, v);
    switch (ktype) {
        case MI355X_TYPE_F16:  return launch_type<MI355X_TYPE_F16>(a, v, stream);
        case MI355X_TYPE_F32:  return launch_type<MI355X_TYPE_F32>(a, v, stream);
        case MI355X_TYPE_Q8_0: return launch_type<MI355X_TYPE_Q8_0>(a, v, stream);
        default:               return (int)hipErrorInvalidValue;
    }
}
