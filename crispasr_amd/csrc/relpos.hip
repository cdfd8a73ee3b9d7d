// FastConformer's relative-position attention mask, produced on the device:
//
//   mask[j, i, h, b] = f16( scale * <Q_v[:, i, h, b], R[:, Nq-1+j-i, h]>  +  add[j, i] )
//
// which is the chain  mul_mat(cont(R), Q_v) -> rel_shift view -> cont -> scale -> (+ local / pad mask) -> cast F16
// of core_conformer::build_block (src/core/fastconformer.h:98-102, 876-918), i.e. the tensor that block hands to
// ggml_flash_attn_ext as its mask.  The products run on v_mfma_f32_32x32x16_f16 (Q_v and R rounded to f16, f32
// accumulation); scale, add and the final rounding are done in f32 exactly as the graph does them.
//
// A wave owns 32 queries of one (head, batch) and a run of 64-key tiles.  It walks R in blocks of 32 rows:
// block n x the 32 queries is one 32x32 accumulator whose element (row, query il) belongs to key
// j = 32n + row + il - 31 (relative to the wave's first query) - a shift that differs per lane, so the block is
// scattered into a wave-private LDS ring [query][key mod 128] and the finished 64-key tile is read back row-wise
// and written out in full 128-byte rows.  Tile t needs blocks 2t, 2t+1, 2t+2; block 2t+2 is also tile t+1's
// first, so each further tile costs two blocks.  Waves never synchronise with each other.
#include "fattn_common.h"

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float    float16v __attribute__((ext_vector_type(16)));

constexpr int RP_WAVES       = 4;
constexpr int RP_CHUNK_TILES = 4;      // 64-key tiles per wave
constexpr int RP_RING        = 128;    // keys per ring row

template <int RTYPE>
__device__ __forceinline__ half8 load_half8(const char * row, int d0) {
    if (RTYPE == MI355X_TYPE_F16) return *(const half8 *)(row + d0 * 2);
    const float4 x0 = *(const float4 *)(row + d0 * 4);
    const float4 x1 = *(const float4 *)(row + d0 * 4 + 16);
    half8 v;
    v[0] = (_Float16)x0.x; v[1] = (_Float16)x0.y; v[2] = (_Float16)x0.z; v[3] = (_Float16)x0.w;
    v[4] = (_Float16)x1.x; v[5] = (_Float16)x1.y; v[6] = (_Float16)x1.z; v[7] = (_Float16)x1.w;
    return v;
}

template <int D, int RTYPE>
__global__ void __launch_bounds__(RP_WAVES * 64) relpos_bias_kernel(const RelposArgs a) {
    constexpr int KS = D / 16;
    __shared__ float ring_all[RP_WAVES][32 * RP_RING];

    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const int l32  = lane & 31;
    const int hh   = lane >> 5;

    int64_t unit = (int64_t)blockIdx.x * RP_WAVES + wave;
    if (unit >= (int64_t)a.n_qblocks * a.n_chunks * a.H * a.B) return;      // waves are independent: no barriers below
    const int qb = (int)(unit % a.n_qblocks); unit /= a.n_qblocks;
    const int ch = (int)(unit % a.n_chunks);  unit /= a.n_chunks;
    const int h  = (int)(unit % a.H);
    const int b  = (int)(unit / a.H);

    const int i0      = qb * 32;
    const int n_tiles = (a.Nkv + 63) / 64;
    const int t_begin = ch * RP_CHUNK_TILES;
    const int t_end   = min(n_tiles, t_begin + RP_CHUNK_TILES);
    const int NR      = a.Nq + a.Nkv - 1;
    const int p_base  = a.Nq - 1 - i0 - 31;            // R row of (block 0, row 0); may be negative

    // B operands: this lane's query, 8 consecutive d per reduction step (rows past Nq re-read the last one and
    // are never stored)
    half8 qv[KS];
    {
        const int qi = min(i0 + l32, a.Nq - 1);
        const char * qrow = a.qv + (int64_t)qi * a.nbq1 + (int64_t)h * a.nbq2 + (int64_t)b * a.nbq3;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) qv[ks] = load_half8<MI355X_TYPE_F32>(qrow, ks * 16 + hh * 8);
    }
    const char * rbase = a.r + (int64_t)(h % a.Hr) * a.nbr2 + (int64_t)(b % a.Br) * a.nbr3;
    const char * abase = a.add ? a.add + (int64_t)(h % a.Ha) * a.nba2 + (int64_t)(b % a.Ba) * a.nba3 : nullptr;
    char *       obase = a.out + (int64_t)h * a.nbo2 + (int64_t)b * a.nbo3;
    float *      ring  = ring_all[wave];

    // A operands of block n: lane's R row, clamped into the table (clamped rows only feed keys outside [0, Nkv))
    auto load_r = [&](int n, half8 (&ra)[KS]) __attribute__((always_inline)) {
        const int p = min(max(p_base + 32 * n + l32, 0), NR - 1);
        const char * row = rbase + (int64_t)p * a.nbr1;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) ra[ks] = load_half8<RTYPE>(row, ks * 16 + hh * 8);
    };
    auto block = [&](int n, const half8 (&ra)[KS]) __attribute__((always_inline)) {
        float16v g;
#pragma unroll
        for (int e = 0; e < 16; e++) g[e] = 0.0f;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) g = __builtin_amdgcn_mfma_f32_32x32x16_f16(ra[ks], qv[ks], g, 0, 0, 0);
        // accumulator slot gg*4+e of lane (l32, hh) = row 8gg + 4hh + e of the block, query l32
        const int c0 = 32 * n + 4 * hh + l32 - 31;
#pragma unroll
        for (int gg = 0; gg < 4; gg++)
#pragma unroll
            for (int e = 0; e < 4; e++) ring[l32 * RP_RING + ((c0 + 8 * gg + e) & (RP_RING - 1))] = g[gg * 4 + e];
    };
    // tile t is complete in the ring: 2 query rows x 64 keys per step, scale / add / round, store
    auto flush = [&](int t) __attribute__((always_inline)) {
        __builtin_amdgcn_wave_barrier();
        const int j = 64 * t + 2 * l32;
#pragma unroll 4
        for (int k = 0; k < 16; k++) {
            const int row = 2 * k + hh;
            const int i   = i0 + row;
            const float2 g2 = *(const float2 *)&ring[row * RP_RING + (j & (RP_RING - 1))];
            if (i < a.Nq && j < a.Nkv) {
                const bool two = j + 1 < a.Nkv;
                float x0 = g2.x * a.scale, x1 = g2.y * a.scale;
                if (abase) {
                    const char * ap = abase + (int64_t)i * a.nba1;
                    if (a.add_f16) {
                        x0 += (float)*(const _Float16 *)(ap + (int64_t)j * 2);
                        if (two) x1 += (float)*(const _Float16 *)(ap + (int64_t)j * 2 + 2);
                    } else {
                        x0 += *(const float *)(ap + (int64_t)j * 4);
                        if (two) x1 += *(const float *)(ap + (int64_t)j * 4 + 4);
                    }
                }
                const _Float16 h0 = (_Float16)x0, h1 = (_Float16)x1;        // round to nearest even, overflow to +-inf
                char * op = obase + (int64_t)i * a.nbo1 + (int64_t)j * 2;
                if (two && a.out_al4) {
                    *(uint32_t *)op = (uint32_t)__builtin_bit_cast(uint16_t, h0) | ((uint32_t)__builtin_bit_cast(uint16_t, h1) << 16);
                } else {
                    *(_Float16 *)op = h0;
                    if (two) *(_Float16 *)(op + 2) = h1;
                }
            }
        }
        __builtin_amdgcn_wave_barrier();
    };

    // blocks 2*t_begin .. 2*t_end, the operands of the next block requested before the current one is used
    const int n0 = 2 * t_begin, n_last = 2 * t_end;
    half8 ra0[KS], ra1[KS];
    load_r(n0, ra0);
    for (int n = n0; n <= n_last; n += 2) {
        const bool odd = n + 1 <= n_last;
        if (odd) load_r(n + 1, ra1);
        block(n, ra0);
        if (n > n0) flush(n / 2 - 1);
        if (odd) {
            if (n + 2 <= n_last) load_r(n + 2, ra0);
            block(n + 1, ra1);
        }
    }
}

template <int D>
int launch_d(const RelposArgs & a, int rtype, hipStream_t stream) {
    const int64_t units = (int64_t)a.n_qblocks * a.n_chunks * a.H * a.B;
    const dim3 grid((unsigned)((units + RP_WAVES - 1) / RP_WAVES));
    if (rtype == MI355X_TYPE_F16) hipLaunchKernelGGL((relpos_bias_kernel<D, MI355X_TYPE_F16>), grid, dim3(RP_WAVES * 64), 0, stream, a);
    else                          hipLaunchKernelGGL((relpos_bias_kernel<D, MI355X_TYPE_F32>), grid, dim3(RP_WAVES * 64), 0, stream, a);
    return (int)hipGetLastError();
}

}  // namespace

int relpos_bias_launch(RelposArgs a, int rtype, hipStream_t stream) {
    if (a.Nq <= 0 || a.Nkv <= 0 || a.H <= 0 || a.B <= 0) return 0;
    a.n_qblocks = (a.Nq + 31) / 32;
    a.n_chunks  = ((a.Nkv + 63) / 64 + RP_CHUNK_TILES - 1) / RP_CHUNK_TILES;
    if ((int64_t)a.n_qblocks * a.n_chunks * a.H * a.B > ((int64_t)1 << 33)) return (int)hipErrorInvalidValue;
    if (a.D == 64)  return launch_d<64>(a, rtype, stream);
    if (a.D == 128) return launch_d<128>(a, rtype, stream);
    return (int)hipErrorInvalidValue;
}
