// FastConformer's relative-position attention mask, produced on the device:
//
//   mask[j, i, h, b] = f16( scale * <Q_v[:, i, h, b], R[:, Nq-1+j-i, h]>  +  add[j, i] )
//
// which is the chain  mul_mat(cont(R), Q_v) -> rel_shift view -> cont -> scale -> (+ local / pad mask) -> cast F16
// of core_conformer::build_block (src/core/fastconformer.h:98-102, 876-918), i.e. the tensor that block hands to
// ggml_flash_attn_ext as its mask.  The products run on v_mfma_f32_32x32x16_f16 (Q_v and R rounded to f16, f32
// accumulation); scale, add and the final rounding are done in f32 exactly as the graph does them.
//
// A workgroup of 4 waves owns 128 consecutive queries of one (head, batch) - 32 per wave - and a run of 32-key
// tiles.  R is walked in blocks of 32 rows: block n x a wave's 32 queries is one 32x32 accumulator whose element
// (row, query il) belongs to key j = 32n + row + il - 31 (relative to the wave's first query) - a shift that differs
// per lane.  Tile t (keys 32t .. 32t+31) is made of the lower-right triangle of block t (row + il >= 31) and the
// upper-left triangle of block t+1 (row + il <= 30): for one accumulator slot the two candidate columns differ by
// exactly 32, so exactly one of the two blocks owns that slot's place in the tile.  A wave therefore keeps the
// previous block's accumulator in registers, computes one new block per tile, selects per slot, and writes the
// 32x32 tile into a wave-private LDS square from which it is read back row-wise, scaled, added to the optional mask
// and stored with 128-bit stores.  One block of MFMAs per 32 keys, no result computed twice.
//
// The four waves need the same rows of R one step apart (wave w's block n is wave 0's block n - w), so the table
// blocks are staged once per workgroup: every step all 256 threads fetch one new block coalesced (adjacent lanes =
// adjacent 16 bytes of a row) into a ring of six f16 blocks in LDS (16-byte chunks XOR-swizzled so that the row-wise
// writes and the MFMA operand reads - lane = row, 8 consecutive d - are both conflict-free), one barrier per step;
// each wave reads its operands from the slot that holds its block.  A quarter of the table traffic and of the
// staging work of a wave-private scheme.  Q_v goes through the same slots once, before the loop.
#include "fattn_common.h"

#include <stdlib.h>

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float    float16v __attribute__((ext_vector_type(16)));

constexpr int RP_WAVES       = 4;
constexpr int RP_TILE_BYTES  = 32 * 32 * 4;
constexpr int RP_SLAB_BYTES  = 32 * 64 * 2;            // 32 rows x 64 values of d, f16
constexpr int RP_SLOTS       = 6;                      // table blocks resident per workgroup

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
    constexpr int NSLAB      = D / 64;                 // slabs per 32-row block
    constexpr int SLOT_BYTES = NSLAB * RP_SLAB_BYTES;
    constexpr int NLD        = SLOT_BYTES / 16 / (RP_WAVES * 64);      // 16-byte pieces per thread and block
    extern __shared__ __attribute__((aligned(16))) char rp_lds[];        // RP_SLOTS table blocks, then 2 squares per wave

    const int tid  = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
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
    if (group >= (int64_t)n_qgroups * a.B) return;                // the whole workgroup leaves
    const int w  = (int)(s_idx % per_group);
    const int h  = w % a.H;
    const int ch = w / a.H;
    const int b  = (int)(group / n_qgroups);
    const int qg = (int)(group % n_qgroups);
    // a wave whose query block lies past Nq keeps step with the others (barriers, table loads) and stores nothing
    const int i0      = (qg * RP_WAVES + wave) * 32;
    const int n_tiles = (a.Nkv + 31) / 32;
    const int t_begin = ch * a.chunk_tiles;                       // even: chunk_tiles is
    const int t_end   = min(n_tiles, t_begin + a.chunk_tiles);
    const int NR      = a.Nq + a.Nkv - 1;
    // table row of (block m, row 0) in wave 0's numbering; wave w's block n is block m = n - w.  May be negative.
    const int p_base0 = a.Nq - 1 - qg * RP_WAVES * 32 - 31;
    const int m_first = t_begin - (RP_WAVES - 1);                 // first block the workgroup stages

    typedef __attribute__((address_space(3))) float lds_float;
    char *  slots = rp_lds;
    float * tile  = (float *)(rp_lds + RP_SLOTS * SLOT_BYTES + wave * 2 * RP_TILE_BYTES);      // squares of an even and an odd tile
    auto slot_of = [&](int m) { return slots + ((m - m_first) % RP_SLOTS) * SLOT_BYTES; };

    const char * qbase = a.qv + (int64_t)h * a.nbq2 + (int64_t)b * a.nbq3;
    const char * rbase = a.r + (int64_t)(h % a.Hr) * a.nbr2 + (int64_t)(b % a.Br) * a.nbr3;
    const char * abase = a.add ? a.add + (int64_t)(h % a.Ha) * a.nba2 + (int64_t)(b % a.Ba) * a.nba3 : nullptr;
    char *       obase = a.out + (int64_t)h * a.nbo2 + (int64_t)b * a.nbo3;

    // Offsets inside one (head, batch) plane of any operand fit 32 bits (checked by the launcher), so addresses are a
    // wave-uniform base plus a 32-bit lane offset.
    // Rows past the ends of Q_v or of the table re-read the nearest valid row: they only feed (query, key) pairs
    // outside [0, Nq) x [0, Nkv), which are never stored.
    auto qrow = [&](int row) { return qbase + (uint32_t)min(i0 + row, a.Nq - 1) * (uint32_t)a.nbq1; };

    // Piece j of a block for this thread: 16 bytes = chunk c of row `row` of slab sl (table rows are contiguous f16,
    // the launcher sees to it)
    u32x4 piece[NLD];
    auto request = [&](int m) __attribute__((always_inline)) {
        const int p0 = p_base0 + 32 * m;
#pragma unroll
        for (int j = 0; j < NLD; j++) {
            const int idx = j * (RP_WAVES * 64) + tid;
            const int sl = idx >> 8, row = (idx & 255) >> 3, c = idx & 7;
            const int p = min(max(p0 + row, 0), NR - 1);
            piece[j] = *(const u32x4 *)(rbase + (uint32_t)p * (2u * D) + (uint32_t)(sl * 128 + c * 16));
        }
    };
    // blocks m_first .. t_begin + 1 (what the first step of all four waves needs) are requested right away, together
    // with Q_v: one memory latency for the whole prologue
    u32x4 first[RP_WAVES + 1][NLD];
#pragma unroll
    for (int i = 0; i <= RP_WAVES; i++) {
        request(m_first + i);
#pragma unroll
        for (int j = 0; j < NLD; j++) first[i][j] = piece[j];
    }

    // B operands: the wave's 32 queries, all of d, through the wave's own slot (all loads in flight together)
    half8 qv[NSLAB][4];
    {
        char * mine = slots + wave * SLOT_BYTES;
        RawSlab<MI355X_TYPE_F32> qraw[NSLAB];
#pragma unroll
        for (int sl = 0; sl < NSLAB; sl++) slab_load<MI355X_TYPE_F32>(qraw[sl], lane, sl * 64, qrow);
#pragma unroll
        for (int sl = 0; sl < NSLAB; sl++) slab_store<MI355X_TYPE_F32>(qraw[sl], lane, mine + sl * RP_SLAB_BYTES);
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int sl = 0; sl < NSLAB; sl++) slab_operands(mine + sl * RP_SLAB_BYTES, l32, hh, qv[sl]);
    }

    auto stage = [&](int m) __attribute__((always_inline)) {
        char * dst = slot_of(m);
#pragma unroll
        for (int j = 0; j < NLD; j++) {
            const int idx = j * (RP_WAVES * 64) + tid;
            const int sl = idx >> 8, row = (idx & 255) >> 3, c = idx & 7;
            *(u32x4 *)(dst + sl * RP_SLAB_BYTES + row * 128 + ((c ^ rp_swz(row)) * 16)) = piece[j];
        }
    };
    // this wave's block n (= staged block n - wave) -> accumulator
    auto multiply = [&](int n, float16v & g) __attribute__((always_inline)) {
        const char * src = slot_of(n - wave);
#pragma unroll
        for (int e = 0; e < 16; e++) g[e] = 0.0f;
#pragma unroll
        for (int sl = 0; sl < NSLAB; sl++) {
            half8 ra[4];
            slab_operands(src + sl * RP_SLAB_BYTES, l32, hh, ra);
#pragma unroll
            for (int ks = 0; ks < 4; ks++) g = __builtin_amdgcn_mfma_f32_32x32x16_f16(ra[ks], qv[sl][ks], g, 0, 0, 0);
        }
    };

    // Accumulator slot gg*4+e of lane (l32, hh) is row rho = 8gg + 4hh + e of its block, query l32.  Its place in
    // tile t is column rho + l32 - 31 if that is >= 0 (the value of block t), else that column + 32 (block t+1).
    const uint32_t tile_row = (uint32_t)(uintptr_t)(lds_float *)tile + (uint32_t)l32 * 128u;
    const int      c_lane   = 4 * hh + l32 - 31;
    auto compose = [&](const float16v & g_lo, const float16v & g_hi, int odd) __attribute__((always_inline)) {
#pragma unroll
        for (int gg = 0; gg < 4; gg++)
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int   c = c_lane + 8 * gg + e;
                const float x = c >= 0 ? g_lo[gg * 4 + e] : g_hi[gg * 4 + e];
                *(lds_float *)(uintptr_t)(tile_row + (uint32_t)odd * RP_TILE_BYTES + (((uint32_t)c & 31u) << 2)) = x;
            }
    };

    // Tiles are written out in pairs (an even tile and the odd one after it: 64 keys, whole 128-byte lines when the
    // output rows are padded to lines) in 4 steps of 8 query rows: lane handles keys 8*(lane%8) .. +7 of the pair in
    // row 8k + lane/8 - a 128-bit store and 2 x 128-bit loads of the add mask when all 8 keys exist and the output
    // rows are dword-aligned, element by element otherwise (the end of a row, odd layouts).  Rows past Nq are
    // computed from the clamped last row and not stored.  The add values of a pair are requested a pair ahead.
    typedef float    f32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));
    typedef _Float16 f16x8_a4 __attribute__((ext_vector_type(8), aligned(4)));
    typedef _Float16 f16x8_a2 __attribute__((ext_vector_type(8), aligned(2)));
    const int frow = lane >> 3, fkey = 8 * (lane & 7);               // fkey: key offset inside the pair
    auto keys_left = [&](int t) { return min(max(a.Nkv - (32 * t + fkey), 0), 8); };      // t even; of this lane's 8
    float ad[4][8];
#pragma unroll
    for (int k = 0; k < 4; k++)
#pragma unroll
        for (int e = 0; e < 8; e++) ad[k][e] = 0.0f;
    auto request_add = [&](int t) __attribute__((always_inline)) {
        if (!abase || keys_left(t) < 8) return;                      // partial lanes read theirs element by element
        const uint32_t es = a.add_f16 ? 2u : 4u;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const uint32_t off = (uint32_t)min(i0 + frow + 8 * k, a.Nq - 1) * (uint32_t)a.nba1 + (uint32_t)(32 * t + fkey) * es;
            if (a.add_f16) {
                const f16x8_a2 wv = *(const f16x8_a2 *)(abase + off);
#pragma unroll
                for (int e = 0; e < 8; e++) ad[k][e] = (float)wv[e];
            } else {
                const f32x4_a4 w0 = *(const f32x4_a4 *)(abase + off), w1 = *(const f32x4_a4 *)(abase + off + 16);
#pragma unroll
                for (int e = 0; e < 4; e++) { ad[k][e] = w0[e]; ad[k][4 + e] = w1[e]; }
            }
        }
    };
    // scale, add and the rounding to f16 as the graph's nodes do them: an f32 multiply, an f32 add (not fused), RNE
    auto finish = [&](float g, float add) { return (_Float16)mul_then_add(g, a.scale, add); };
    auto flush = [&](int t) __attribute__((always_inline)) {         // t even: tiles t and t + 1
        __builtin_amdgcn_wave_barrier();
        const int nk = keys_left(t);
        const float * rp = tile + (fkey >> 5) * (RP_TILE_BYTES / 4) + frow * 32 + (fkey & 31);
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const int i = i0 + frow + 8 * k;
            const float4 x0 = *(const float4 *)(rp + k * 8 * 32), x1 = *(const float4 *)(rp + k * 8 * 32 + 4);
            const float x[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
            if (i < a.Nq && nk > 0) {
                char * op = obase + (uint32_t)i * (uint32_t)a.nbo1 + (uint32_t)(32 * t + fkey) * 2u;
                if (nk == 8 && a.out_al4) {
                    f16x8_a4 hv;
#pragma unroll
                    for (int e = 0; e < 8; e++) hv[e] = finish(x[e], ad[k][e]);
                    *(f16x8_a4 *)op = hv;
                } else {
                    const char * ap = abase ? abase + (uint32_t)i * (uint32_t)a.nba1 + (uint32_t)(32 * t + fkey) * (a.add_f16 ? 2u : 4u) : nullptr;
#pragma unroll
                    for (int e = 0; e < 8; e++) {
                        if (e < nk) {
                            float av = 0.0f;
                            if (ap) av = nk == 8 ? ad[k][e] : (a.add_f16 ? (float)((const _Float16 *)ap)[e] : ((const float *)ap)[e]);
                            ((_Float16 *)op)[e] = finish(x[e], av);
                        }
                    }
                }
            }
        }
        __builtin_amdgcn_wave_barrier();
        if (t + 2 < t_end) request_add(t + 2);
    };

    // Prologue: the Q_v slots are free once every wave has its operands; then the blocks requested at the start
    // are staged.
    __syncthreads();
    {
#pragma unroll
        for (int i = 0; i <= RP_WAVES; i++) {
#pragma unroll
            for (int j = 0; j < NLD; j++) piece[j] = first[i][j];
            stage(m_first + i);
        }
    }
    if (t_begin + 2 <= t_end) request(t_begin + 2);
    request_add(t_begin);
    __syncthreads();
    float16v g0, g1;
    multiply(t_begin, g0);
    // Step t: block t + 2 (requested a step ago) goes into the slot whose last readers finished two steps ago - the
    // barrier of the step between makes that safe - and block t + 3 is requested; the wave multiplies its block t + 1,
    // which was staged a step ago and published by that step's barrier.  Unrolled by two so that both accumulators
    // stay in registers.
    auto step = [&](int t, const float16v & g_lo, float16v & g_hi, int odd) __attribute__((always_inline)) {
        if (t + 2 <= t_end) stage(t + 2);
        if (t + 3 <= t_end) request(t + 3);
        __syncthreads();
        multiply(t + 1, g_hi);
        compose(g_lo, g_hi, odd);
    };
    for (int t = t_begin; t < t_end; t += 2) {          // t_begin is even: pairs start on 64-key boundaries
        step(t, g0, g1, 0);
        if (t + 1 < t_end) step(t + 1, g1, g0, 1);
        flush(t);                                       // a missing odd tile lies past Nkv: its lanes store nothing
    }
}

template <int D, int RTYPE>
int launch_dt(const RelposArgs & a, hipStream_t stream) {
    constexpr int LDS = RP_SLOTS * (D / 64) * RP_SLAB_BYTES + RP_WAVES * 2 * RP_TILE_BYTES;
    static std::atomic<uint64_t> lds_allowed{0};     // per instantiation
    const hipError_t ea = fattn_allow_lds((const void *)relpos_bias_kernel<D, RTYPE>, LDS, lds_allowed);
    if (ea != hipSuccess) return (int)ea;
    const int64_t groups = (int64_t)((a.n_qblocks + RP_WAVES - 1) / RP_WAVES) * a.B;
    const dim3 grid((unsigned)((groups + 7) / 8 * 8 * a.n_chunks * a.H));
    hipLaunchKernelGGL((relpos_bias_kernel<D, RTYPE>), grid, dim3(RP_WAVES * 64), LDS, stream, a);
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
    // Keys are cut into chunks of an even number of 32-key tiles, one workgroup per (4 query blocks, head, chunk).
    // A workgroup costs a prologue worth about 6 tiles (Q_v, the first table blocks) plus its tiles, and workgroups run
    // in rounds of `slots` at a time: take the chunk size with the cheapest rounds x (6 + tiles), the longer on a tie
    // (measured at 8 heads x 128, T = 750, batch 8: 24 tiles 50 us, 12: 52, 8: 53, 6: 57, 4: 59).
    {
        const int     n_tiles = (a.Nkv + 31) / 32;
        const int64_t groups  = (int64_t)((a.n_qblocks + RP_WAVES - 1) / RP_WAVES) * a.B * a.H;
        const int64_t slots   = (int64_t)(a.n_cus > 0 ? a.n_cus : 256) * (a.D == 64 ? 3 : 2);
        int64_t best_cost = -1;
        int     best = 2;
        for (int c = 2; c <= ((n_tiles + 1) & ~1); c += 2) {
            const int64_t wgs  = groups * ((n_tiles + c - 1) / c);
            const int64_t cost = ((wgs + slots - 1) / slots) * (6 + c);
            if (best_cost < 0 || cost < best_cost || (cost == best_cost && c > best)) { best_cost = cost; best = c; }
        }
        static const char * force = getenv("MI355X_RELPOS_CHUNK");          // experiments only
        if (force && atoi(force) >= 2) best = atoi(force) & ~1;
        a.chunk_tiles = best;
        a.n_chunks    = (n_tiles + best - 1) / best;
    }
    if ((int64_t)a.n_qblocks * a.n_chunks * a.H * a.B > ((int64_t)1 << 33)) return (int)hipErrorInvalidValue;
    // 32-bit offsets inside a (head, batch) plane
    const uint64_t lim = (uint64_t)1 << 31;
    if ((uint64_t)a.Nq * a.nbq1 >= lim || (uint64_t)(a.Nq + a.Nkv) * a.nbr1 >= lim || (uint64_t)a.Nq * a.nbo1 >= lim ||
        (a.add && (uint64_t)a.Nq * a.nba1 >= lim)) return (int)hipErrorInvalidValue;
    if (a.D == 64)  return launch_d<64>(a, rtype, stream);
    if (a.D == 128) return launch_d<128>(a, rtype, stream);
    return (int)hipErrorInvalidValue;
}
