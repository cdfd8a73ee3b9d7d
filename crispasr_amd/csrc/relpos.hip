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
// first, so each further tile costs two blocks.
//
// MFMA operands want lane = row with 8 consecutive d, which as a global access pattern is 64 scattered 16-byte
// pieces per instruction.  Rows are therefore fetched coalesced (adjacent lanes = adjacent 16 bytes of a row), 64
// values of d at a time, converted to f16 and passed through a wave-private 32 x 64 staging block in LDS
// (16-byte chunks XOR-swizzled so that both the row-wise writes and the operand reads are conflict-free); the next
// block's global loads are in flight while the current one is multiplied and scattered.  Waves never synchronise with each other.
#include "fattn_common.h"

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float    float16v __attribute__((ext_vector_type(16)));

constexpr int RP_WAVES       = 4;
constexpr int RP_CHUNK_TILES = 4;      // 64-key tiles per wave
constexpr int RP_RING        = 128;    // keys per ring row
constexpr int RP_RING_BYTES  = 32 * RP_RING * 4;
constexpr int RP_STAGE_BYTES = 32 * 64 * 2;
constexpr int RP_LDS_BYTES   = RP_WAVES * (RP_RING_BYTES + RP_STAGE_BYTES);

// swizzle of the staging block's eight 16-byte chunks per row
__device__ __forceinline__ int rp_swz(int r) { return (r >> 1) & 7; }

// One slab = 32 rows x 64 consecutive values of d.  Raw<TYPE>: what a lane holds of it between the global loads
// and the LDS writes.  F16: 4 x 16 bytes (slot = j*64 + lane -> row slot/8, chunk slot%8).
// F32: 8 x float4 (slot -> row slot/16, float4 slot%16).
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
template <int TYPE> struct RawSlab { u32x4 v[TYPE == MI355X_TYPE_F16 ? 4 : 8]; };

// rowptr(row) -> address of d = 0 of that row of the slab's tensor; d0 = first d of the slab
template <int TYPE, typename F>
__device__ __forceinline__ void slab_load(RawSlab<TYPE> & raw, int lane, int d0, F rowptr) {
    if (TYPE == MI355X_TYPE_F16) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int slot = j * 64 + lane;
            raw.v[j] = *(const u32x4 *)(rowptr(slot >> 3) + (d0 + (slot & 7) * 8) * 2);
        }
    } else {
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int slot = j * 64 + lane;
            raw.v[j] = *(const u32x4 *)(rowptr(slot >> 4) + (d0 + (slot & 15) * 4) * 4);
        }
    }
}

template <int TYPE>
__device__ __forceinline__ void slab_store(const RawSlab<TYPE> & raw, int lane, char * stage) {
    if (TYPE == MI355X_TYPE_F16) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int slot = j * 64 + lane, row = slot >> 3, c = slot & 7;
            *(u32x4 *)(stage + row * 128 + ((c ^ rp_swz(row)) * 16)) = raw.v[j];
        }
    } else {
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int slot = j * 64 + lane, row = slot >> 4, c4 = slot & 15;
            half4 h;
            h[0] = (_Float16)__uint_as_float(raw.v[j].x); h[1] = (_Float16)__uint_as_float(raw.v[j].y);
            h[2] = (_Float16)__uint_as_float(raw.v[j].z); h[3] = (_Float16)__uint_as_float(raw.v[j].w);
            *(half4 *)(stage + row * 128 + (((c4 >> 1) ^ rp_swz(row)) * 16) + (c4 & 1) * 8) = h;
        }
    }
}

// operand fragments of the staged slab: lane (l32, hh) takes d = 16*ks + 8*hh .. +8 of row l32, ks = 0..3
__device__ __forceinline__ void slab_operands(const char * stage, int l32, int hh, half8 (&op)[4]) {
#pragma unroll
    for (int ks = 0; ks < 4; ks++) op[ks] = *(const half8 *)(stage + l32 * 128 + (((ks * 2 + hh) ^ rp_swz(l32)) * 16));
}

template <int D, int RTYPE>
__global__ void __launch_bounds__(RP_WAVES * 64, 2) relpos_bias_kernel(const RelposArgs a) {
    constexpr int NSLAB = D / 64;                 // slabs per 32-row block
    extern __shared__ __attribute__((aligned(16))) char rp_lds[];

    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const int l32  = lane & 31;
    const int hh   = lane >> 5;

    // Workgroups go to the 8 XCDs round-robin, each with its own L2.  A group of 4 query blocks of one batch entry
    // is given to one XCD, which walks its key chunks and heads back to back: the add mask (shared by the heads)
    // and Q_v (shared by the chunks) then come from that L2 after their first use instead of crossing the fabric
    // once per head and chunk.
    const int per_group = a.n_chunks * a.H;                      // workgroups per (batch entry, 4 query blocks)
    const int n_qgroups = (a.n_qblocks + RP_WAVES - 1) / RP_WAVES;
    const int64_t s_idx = blockIdx.x >> 3;
    const int64_t group = (s_idx / per_group) * 8 + (blockIdx.x & 7);
    if (group >= (int64_t)n_qgroups * a.B) return;                // waves are independent: no barriers below
    const int w  = (int)(s_idx % per_group);
    const int h  = w % a.H;
    const int ch = w / a.H;
    const int b  = (int)(group / n_qgroups);
    const int qb = (int)(group % n_qgroups) * RP_WAVES + wave;
    if (qb >= a.n_qblocks) return;

    const int i0      = qb * 32;
    const int n_tiles = (a.Nkv + 63) / 64;
    const int t_begin = ch * RP_CHUNK_TILES;
    const int t_end   = min(n_tiles, t_begin + RP_CHUNK_TILES);
    const int NR      = a.Nq + a.Nkv - 1;
    const int p_base  = a.Nq - 1 - i0 - 31;            // R row of (block 0, row 0); may be negative

    float * ring  = (float *)(rp_lds + wave * RP_RING_BYTES);
    char *  stage = rp_lds + RP_WAVES * RP_RING_BYTES + wave * RP_STAGE_BYTES;

    const char * qbase = a.qv + (int64_t)h * a.nbq2 + (int64_t)b * a.nbq3;
    const char * rbase = a.r + (int64_t)(h % a.Hr) * a.nbr2 + (int64_t)(b % a.Br) * a.nbr3;
    const char * abase = a.add ? a.add + (int64_t)(h % a.Ha) * a.nba2 + (int64_t)(b % a.Ba) * a.nba3 : nullptr;
    char *       obase = a.out + (int64_t)h * a.nbo2 + (int64_t)b * a.nbo3;

    // Offsets inside one (head, batch) plane of any operand fit 32 bits (checked by the launcher), so addresses are a
    // wave-uniform base plus a 32-bit lane offset.
    // Rows past the ends of Q_v or of the table re-read the nearest valid row: they only feed (query, key) pairs
    // outside [0, Nq) x [0, Nkv), which are never stored.
    auto qrow = [&](int row) { return qbase + (uint32_t)min(i0 + row, a.Nq - 1) * (uint32_t)a.nbq1; };

    // B operands: the wave's 32 queries, all of d, through the staging block (all loads in flight together)
    half8 qv[NSLAB][4];
    {
        RawSlab<MI355X_TYPE_F32> qraw[NSLAB];
#pragma unroll
        for (int sl = 0; sl < NSLAB; sl++) slab_load<MI355X_TYPE_F32>(qraw[sl], lane, sl * 64, qrow);
#pragma unroll
        for (int sl = 0; sl < NSLAB; sl++) {
            slab_store<MI355X_TYPE_F32>(qraw[sl], lane, stage);
            __builtin_amdgcn_wave_barrier();
            slab_operands(stage, l32, hh, qv[sl]);
            __builtin_amdgcn_wave_barrier();
        }
    }

    // accumulator slot gg*4+e of lane (l32, hh) = row 8gg + 4hh + e of the block, query l32.  Byte address in the
    // ring = row base | ((4*column) mod 512): the wave's ring is 512-byte aligned, so the OR is an addition.
    typedef __attribute__((address_space(3))) float lds_float;
    const uint32_t ring_row = (uint32_t)(uintptr_t)(lds_float *)ring + (uint32_t)l32 * (RP_RING * 4);
    auto scatter = [&](int n, const float16v & g) __attribute__((always_inline)) {
        const uint32_t x4 = (uint32_t)(32 * n + 4 * hh + l32 - 31) * 4u;
#pragma unroll
        for (int gg = 0; gg < 4; gg++)
#pragma unroll
            for (int e = 0; e < 4; e++)
                *(lds_float *)(uintptr_t)(ring_row | ((x4 + (uint32_t)(8 * gg + e) * 4u) & (RP_RING * 4 - 1))) = g[gg * 4 + e];
    };

    // A tile is written out in 16 steps of 2 query rows x 64 keys: lane (l32, hh) handles keys 2*l32, 2*l32+1 of
    // row 2k + hh.  Whole tiles of whole query blocks (the common case) take a path without per-element tests.
    const bool rows_full = i0 + 32 <= a.Nq;
    float ad[16][2];               // add values of the next tile to be written, requested a tile ahead
#pragma unroll
    for (int k = 0; k < 16; k++) ad[k][0] = ad[k][1] = 0.0f;
    auto request_add = [&](int t) __attribute__((always_inline)) {
        if (!abase) return;
        const int j = 64 * t + 2 * l32;
        if (rows_full && 64 * t + 64 <= a.Nkv && a.add_vec) {
            uint32_t off = (uint32_t)(i0 + hh) * (uint32_t)a.nba1 + (uint32_t)j * (a.add_f16 ? 2u : 4u);
            const uint32_t step = 2u * (uint32_t)a.nba1;
            if (a.add_f16) {
#pragma unroll
                for (int k = 0; k < 16; k++, off += step) {
                    const half2v w = *(const half2v *)(abase + off);
                    ad[k][0] = (float)w[0]; ad[k][1] = (float)w[1];
                }
            } else {
#pragma unroll
                for (int k = 0; k < 16; k++, off += step) {
                    const float2 w = *(const float2 *)(abase + off);
                    ad[k][0] = w.x; ad[k][1] = w.y;
                }
            }
            return;
        }
        const bool two = j + 1 < a.Nkv;
#pragma unroll
        for (int k = 0; k < 16; k++) {
            ad[k][0] = ad[k][1] = 0.0f;
            const int i = i0 + 2 * k + hh;
            if (i < a.Nq && j < a.Nkv) {
                const char * ap = abase + (uint32_t)i * (uint32_t)a.nba1;
                if (a.add_f16) {
                    ad[k][0] = (float)*(const _Float16 *)(ap + j * 2);
                    if (two) ad[k][1] = (float)*(const _Float16 *)(ap + j * 2 + 2);
                } else {
                    ad[k][0] = *(const float *)(ap + j * 4);
                    if (two) ad[k][1] = *(const float *)(ap + j * 4 + 4);
                }
            }
        }
    };
    // scale, add and the rounding to f16 as the graph's nodes do them: an f32 multiply, an f32 add (not fused), RNE
    auto finish = [&](float g, float add) { return (_Float16)__fadd_rn(__fmul_rn(g, a.scale), add); };
    auto flush = [&](int t) __attribute__((always_inline)) {
        __builtin_amdgcn_wave_barrier();
        const int j = 64 * t + 2 * l32;
        const float * rp = ring + hh * RP_RING + (j & (RP_RING - 1));
        if (rows_full && 64 * t + 64 <= a.Nkv && a.out_al4) {
            uint32_t off = (uint32_t)(i0 + hh) * (uint32_t)a.nbo1 + (uint32_t)j * 2u;
            const uint32_t step = 2u * (uint32_t)a.nbo1;
#pragma unroll
            for (int k = 0; k < 16; k++, off += step) {
                const float2 g2 = *(const float2 *)(rp + k * 2 * RP_RING);
                half2v hv;
                hv[0] = finish(g2.x, ad[k][0]);
                hv[1] = finish(g2.y, ad[k][1]);
                *(half2v *)(obase + off) = hv;
            }
        } else {
            const bool two = j + 1 < a.Nkv;
#pragma unroll
            for (int k = 0; k < 16; k++) {
                const int i = i0 + 2 * k + hh;
                const float2 g2 = *(const float2 *)(rp + k * 2 * RP_RING);
                if (i < a.Nq && j < a.Nkv) {
                    const _Float16 h0 = finish(g2.x, ad[k][0]), h1 = finish(g2.y, ad[k][1]);
                    char * op = obase + (uint32_t)i * (uint32_t)a.nbo1 + (uint32_t)j * 2u;
                    if (two && a.out_al4) {
                        half2v hv = {h0, h1};
                        *(half2v *)op = hv;
                    } else {
                        *(_Float16 *)op = h0;
                        if (two) *(_Float16 *)(op + 2) = h1;
                    }
                }
            }
        }
        __builtin_amdgcn_wave_barrier();
        if (t + 1 < t_end) request_add(t + 1);
    };

    // blocks 2*t_begin .. 2*t_end in order (an even count plus one); the rows of two blocks ahead are in flight
    // while one is multiplied and scattered
    const int n0 = 2 * t_begin, n_last = 2 * t_end;
    // The table's rows are contiguous f16 (the launcher sees to it), so a block that lies inside the table is a
    // wave-uniform base plus a fixed lane offset; only the first and last blocks need their rows clamped.
    const uint32_t lane_roff = (uint32_t)(lane >> 3) * (2u * D) + (uint32_t)(lane & 7) * 16u;
    auto request = [&](int n, RawSlab<RTYPE> (&raw)[NSLAB]) __attribute__((always_inline)) {
        const int p0 = p_base + 32 * n;
        if (p0 >= 0 && p0 + 31 <= NR - 1) {
            const char * bp = rbase + (uint32_t)p0 * (2u * D);
#pragma unroll
            for (int sl = 0; sl < NSLAB; sl++)
#pragma unroll
                for (int j = 0; j < 4; j++) raw[sl].v[j] = *(const u32x4 *)(bp + lane_roff + (uint32_t)(j * 8 * 2 * D + sl * 128));
        } else {
            auto rrow = [&](int row) { return rbase + (uint32_t)min(max(p0 + row, 0), NR - 1) * (2u * D); };
#pragma unroll
            for (int sl = 0; sl < NSLAB; sl++) slab_load<RTYPE>(raw[sl], lane, sl * 64, rrow);
        }
    };
    // stage the block held in raw, refill raw with block n_next (if any), multiply, scatter
    auto block = [&](int n, int n_next, RawSlab<RTYPE> (&raw)[NSLAB]) __attribute__((always_inline)) {
        float16v g;
#pragma unroll
        for (int e = 0; e < 16; e++) g[e] = 0.0f;
#pragma unroll
        for (int sl = 0; sl < NSLAB; sl++) {
            half8 ra[4];
            slab_store<RTYPE>(raw[sl], lane, stage);
            __builtin_amdgcn_wave_barrier();
            slab_operands(stage, l32, hh, ra);
            __builtin_amdgcn_wave_barrier();
            if (sl == NSLAB - 1 && n_next <= n_last) request(n_next, raw);
#pragma unroll
            for (int ks = 0; ks < 4; ks++) g = __builtin_amdgcn_mfma_f32_32x32x16_f16(ra[ks], qv[sl][ks], g, 0, 0, 0);
        }
        scatter(n, g);
    };
    RawSlab<RTYPE> raw_even[NSLAB], raw_odd[NSLAB];
    request(n0, raw_even);
    request(n0 + 1, raw_odd);            // n_last >= n0 + 2: a chunk holds at least one tile
    request_add(t_begin);
    for (int n = n0; n <= n_last; n += 2) {
        block(n, n + 2, raw_even);
        if (n > n0) flush(n / 2 - 1);
        if (n + 1 <= n_last) block(n + 1, n + 3, raw_odd);
    }
}

template <int D, int RTYPE>
int launch_dt(const RelposArgs & a, hipStream_t stream) {
    static bool attr_set = false;     // per instantiation: the dynamic LDS exceeds the 64 KiB default
    if (!attr_set) {
        const hipError_t e = hipFuncSetAttribute((const void *)relpos_bias_kernel<D, RTYPE>,
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, RP_LDS_BYTES);
        if (e != hipSuccess) return (int)e;
        attr_set = true;
    }
    const int64_t groups = (int64_t)((a.n_qblocks + RP_WAVES - 1) / RP_WAVES) * a.B;
    const dim3 grid((unsigned)((groups + 7) / 8 * 8 * a.n_chunks * a.H));
    hipLaunchKernelGGL((relpos_bias_kernel<D, RTYPE>), grid, dim3(RP_WAVES * 64), RP_LDS_BYTES, stream, a);
    return (int)hipGetLastError();
}

template <int D>
int launch_d(const RelposArgs & a, int rtype, hipStream_t stream) {
    // F32 (or strided) tables are turned into f16 with contiguous rows by the caller of this launcher first (one
    // small copy): half the bytes per block, and the whole table then stays in an XCD's L2
    if (rtype != MI355X_TYPE_F16 || a.nbr1 != (size_t)2 * D) return (int)hipErrorInvalidValue;
    return launch_dt<D, MI355X_TYPE_F16>(a, stream);
}

}  // namespace

int relpos_bias_launch(RelposArgs a, int rtype, hipStream_t stream) {
    if (a.Nq <= 0 || a.Nkv <= 0 || a.H <= 0 || a.B <= 0) return 0;
    a.n_qblocks = (a.Nq + 31) / 32;
    a.n_chunks  = ((a.Nkv + 63) / 64 + RP_CHUNK_TILES - 1) / RP_CHUNK_TILES;
    if ((int64_t)a.n_qblocks * a.n_chunks * a.H * a.B > ((int64_t)1 << 33)) return (int)hipErrorInvalidValue;
    // 32-bit offsets inside a (head, batch) plane
    const uint64_t lim = (uint64_t)1 << 31;
    if ((uint64_t)a.Nq * a.nbq1 >= lim || (uint64_t)(a.Nq + a.Nkv) * a.nbr1 >= lim || (uint64_t)a.Nq * a.nbo1 >= lim ||
        (a.add && (uint64_t)a.Nq * a.nba1 >= lim)) return (int)hipErrorInvalidValue;
    if (a.D == 64)  return launch_d<64>(a, rtype, stream);
    if (a.D == 128) return launch_d<128>(a, rtype, stream);
    return (int)hipErrorInvalidValue;
}
