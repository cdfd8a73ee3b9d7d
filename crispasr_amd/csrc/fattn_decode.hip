// Split-KV MFMA decode kernel for gfx950: few query rows per KV head (beams and/or a GQA group),
// long KV cache, HBM-bound.
//
// A workgroup of 4 waves owns one (KV head, batch, KV split, chunk of 16 query rows); the query rows
// that read this KV head - all queries of all q heads in its GQA group, 16 of them per chunk - are
// the 16 columns of v_mfma_f32_16x16x32_f16 tiles, so K and V are fetched once per KV head and chunk,
// not once per query row (decode steps have one chunk; a short prompt has a few, and each streams the
// head's K/V again).  Each wave walks its share of the split in steps of 32 keys:
//
//   S^T[key, row] = K[key, :] . Q[row, :]^T      A = K from global memory in operand layout
//                                                 (128-bit loads: 16 rows x 64 contiguous bytes)
//   O^T[d,   row] = V[:, d]^T . P^T[:, row]      A = V^T via a wave-private LDS stage written with
//                                                 coalesced 128-bit rows and read back with
//                                                 ds_read_b64_tr_b16; B = P straight from the
//                                                 accumulator registers of the first product
//
// Q8_0 caches are dequantised in registers: the 8 int8 of a lane's chunk are fetched with three
// aligned dword loads and a byte funnel shift (blocks are 34 bytes, so chunks sit at 2 mod 4),
// widened to exact f16 integers with v_perm_b32 + one packed add, and scaled by the block's f16 d
// with one packed multiply (one rounding, = f16(q*d)).  When the rows of a Q8_0 cache are contiguous the
// K bytes of a step are fetched as one coalesced stream of 8- (or 4-)byte units into a wave-private raw
// stage in LDS and the chunks are cut out of LDS instead - three times fewer global load instructions.
// V then skips the f16 stage: it arrives as the same kind of stream, its quants are stored to LDS as bytes - every
// 2-byte piece of a unit written to its place, [key][column] for quants and [block][key] for scales - and read back
// through ds_read_b64_tr_b8, which hands every lane eight consecutive keys of one column - the A operand of the second
// product - to be widened and multiplied by those keys' scales in registers: same values, half the LDS bytes, one
// register stage instead of two.  Q4_0 / Q4_1 / Q5_0 / Q5_1 rows are streamed the same way into raw K and V stages and
// dequantised out of LDS (V into the f16 stage).  Streams and f16 rows are loaded non-temporal: they are read once.
// Loads of the next step are in flight while the current one is consumed.  Waves are merged through LDS, splits by fattn_merge_kernel.
#include "fattn_row.h"

#include <stdlib.h>
#include <type_traits>

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float    float4v __attribute__((ext_vector_type(4)));
typedef short    short4v __attribute__((ext_vector_type(4)));

constexpr int   DEC_WAVES   = 4;
constexpr int   DEC_THREADS = DEC_WAVES * 64;
constexpr int   STEP        = 32;                  // keys per wave step
constexpr float LOG2E       = 1.4426950408889634f;
constexpr float SUM_LIMIT   = 4096.0f;             // 8 probabilities per lane and step

// K and V are read once per launch and loaded with stream_load where a wave instruction takes whole lines once - the
// coalesced row streams and f16 rows (64 sequences x 4096 f16 entries: 169 against 188 us).  Per-lane pieces of block
// rows come back to a line several times: the 8-byte pieces and halfword scales of the int8 V stage lose 3-5% when
// marked, and the strided-row forms stay plain with them.
typedef uint32_t u32x2    __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4    __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_a2 __attribute__((ext_vector_type(2), aligned(2)));

// ---- Q8_0 in registers ------------------------------------------------------------------

// the 8 quants of chunk c (0..3) of block blk of a row whose address is a multiple of 4
__device__ __forceinline__ uint2 q8_load_chunk(const char * row, int blk, int c) {
    const int o  = blk * FATTN_Q8_0_BYTES + 2 + c * 8;
    const int sh = o & 3;                                   // 0 or 2
    const uint32_t * p = (const uint32_t *)(row + (o - sh));
    const uint32_t u0 = p[0];
    const uint32_t u1 = p[1];
    const uint32_t u2 = sh ? p[2] : 0u;                     // never read past the row when aligned
    uint2 r;
    r.x = __builtin_amdgcn_alignbyte(u1, u0, sh);
    r.y = __builtin_amdgcn_alignbyte(u2, u1, sh);
    return r;
}

// the same from a raw copy of the rows in LDS (row_off = byte offset of the row inside the stage)
// (row_off is a multiple of 4, so odd blocks start on a dword; UNIFORM_BLK says blk is the same in every lane)
template <bool UNIFORM_BLK>
__device__ __forceinline__ uint4 q8_lds_chunk(const char * stage, int row_off, int blk, int c) {
    const int o  = row_off + blk * FATTN_Q8_0_BYTES + 2 + c * 8;
    const int sh = (blk & 1) ? 0 : 2;
    const uint32_t * p = (const uint32_t *)(stage + (o - sh));
    const uint32_t u0 = p[0], u1 = p[1], u2 = p[2];         // the stage is padded: p[2] is always inside it
    uint4 r;
    if (UNIFORM_BLK && (blk & 1)) {
        r.x = u0;
        r.y = u1;
    } else {
        r.x = __builtin_amdgcn_alignbyte(u1, u0, sh);
        r.y = __builtin_amdgcn_alignbyte(u2, u1, sh);
    }
    r.z = *(const uint16_t *)(stage + row_off + blk * FATTN_Q8_0_BYTES);
    r.w = 0;
    return r;
}

// 4 int8 packed in a dword -> 4 exact f16 integers: bytes become the low mantissa bits of
// 1024 + (q + 128), then 1152 is subtracted
__device__ __forceinline__ void q8_widen(uint32_t w, half2v & lo, half2v & hi) {
    const uint32_t x = w ^ 0x80808080u;
    const uint32_t a = __builtin_amdgcn_perm(x, 0x64646464u, 0x00050004u);   // {0x64, b1, 0x64, b0}
    const uint32_t b = __builtin_amdgcn_perm(x, 0x64646464u, 0x00070006u);   // {0x64, b3, 0x64, b2}
    const half2v off = {(_Float16)1152.0f, (_Float16)1152.0f};
    lo = __builtin_bit_cast(half2v, a) - off;
    hi = __builtin_bit_cast(half2v, b) - off;
}

__device__ __forceinline__ half8 q8_dequant(uint2 q, uint16_t dbits) {
    const _Float16 d  = __builtin_bit_cast(_Float16, dbits);
    const half2v   d2 = {d, d};
    half2v h0, h1, h2, h3;
    q8_widen(q.x, h0, h1);
    q8_widen(q.y, h2, h3);
    h0 *= d2; h1 *= d2; h2 *= d2; h3 *= d2;
    half8 r;
    r[0] = h0[0]; r[1] = h0[1]; r[2] = h1[0]; r[3] = h1[1];
    r[4] = h2[0]; r[5] = h2[1]; r[6] = h3[0]; r[7] = h3[1];
    return r;
}

// 8 quants of 8 different keys (one column of V) times those keys' scales
__device__ __forceinline__ half8 q8_dequant_keys(uint32_t q0, uint32_t q1, half8 d) {
    half2v h0, h1, h2, h3;
    q8_widen(q0, h0, h1);
    q8_widen(q1, h2, h3);
    half8 r;
    r[0] = h0[0]; r[1] = h0[1]; r[2] = h1[0]; r[3] = h1[1];
    r[4] = h2[0]; r[5] = h2[1]; r[6] = h3[0]; r[7] = h3[1];
    return r * d;
}

// raw global data of one 8-element chunk
struct Chunk {
    uint4 v;         // f16: the 8 halves; q8_0: x,y = quants, z = scale bits
};

// Q4_0 / Q4_1 / Q5_0 / Q5_1: x, y = the 8 bytes that hold the chunk's nibbles, shifted so that they sit in the low halves;
// z = d (low) and m (high halfword); w = the chunk's 8 fifth bits.  q0, q1: the 8 bytes at QS + 8 (c % 2) of the block,
// dm: d in the low halfword (and m in the high one), qh: the block's 32 fifth bits, c: which 8 of the block's 32 elements.
__device__ __forceinline__ Chunk narrow_fields(uint32_t q0, uint32_t q1, uint32_t dm, uint32_t qh, int c) {
    Chunk r;
    const int sh = (c & 2) ? 4 : 0;
    r.v.x = (q0 >> sh) & 0x0F0F0F0Fu;
    r.v.y = (q1 >> sh) & 0x0F0F0F0Fu;
    r.v.z = dm;
    r.v.w = (qh >> (c * 8)) & 0xFFu;
    return r;
}

// the same from the block's first 8 bytes h0, h1
template <int TYPE>
__device__ __forceinline__ Chunk narrow_chunk(uint32_t q0, uint32_t q1, uint32_t h0, uint32_t h1, int c) {
    typedef BlockFormat<TYPE> F;
    const uint32_t qh = !F::QH ? 0u : F::QH == 4 ? h1 : __builtin_amdgcn_alignbyte(h1, h0, 2);
    return narrow_fields(q0, q1, F::HAS_M ? h0 : h0 & 0xFFFFu, qh, c);
}

// the same chunk cut out of a raw copy of the rows in LDS (row_off: byte offset of the row inside the stage, a multiple
// of 4; blocks and their quants start on even bytes) with aligned dword reads.  Whether a block starts on a dword or two
// bytes past one depends on the block's index alone - 18- and 22-byte blocks alternate, 20- and 24-byte ones always start
// on one - so with blk a constant after unrolling, every shift here is decided at compile time.  The stage is padded:
// the dword after a pair is always inside it.
template <int TYPE>
__device__ __forceinline__ Chunk narrow_lds_chunk(const char * stage, int row_off, int blk, int c) {
    typedef BlockFormat<TYPE> F;
    const int mis  = (blk * F::BYTES) & 2;                   // bytes from the dword below to the block
    const int misq = (mis + F::QS) & 2;                      // ... to its quants
    const uint32_t * ph = (const uint32_t *)(stage + row_off + blk * F::BYTES - mis);
    const uint32_t * pq = (const uint32_t *)(stage + row_off + blk * F::BYTES + F::QS + (c & 1) * 8 - misq);
    const uint32_t a0 = ph[0];
    uint32_t q0 = pq[0], q1 = pq[1];
    if (misq) {
        const uint32_t q2 = pq[2];
        q0 = __builtin_amdgcn_alignbyte(q1, q0, 2);
        q1 = __builtin_amdgcn_alignbyte(q2, q1, 2);
    }
    const uint32_t dm = F::HAS_M ? a0 : mis ? a0 >> 16 : a0 & 0xFFFFu;
    uint32_t qh = 0;
    if (F::QH == 4) qh = ph[1];                                                    // fifth bits at byte 4
    if (F::QH == 2) qh = mis ? ph[1] : __builtin_amdgcn_alignbyte(ph[1], a0, 2);   // at byte 2
    return narrow_fields(q0, q1, dm, qh, c);
}

// bytes per block of the types the raw stream carries (Q8_0 for the others: they never instantiate it)
template <int TYPE> constexpr int raw_block_bytes() {
    if constexpr (FATTN_IS_BLOCK_TYPE(TYPE)) return BlockFormat<TYPE>::BYTES;
    else return FATTN_Q8_0_BYTES;
}

template <int TYPE>
__device__ __forceinline__ Chunk load_chunk(const char * row, int c) {
    Chunk r;
    if constexpr (TYPE == MI355X_TYPE_F16) {
        r.v = __builtin_bit_cast(uint4, stream_load<u32x4>(row + c * 16));
    } else if constexpr (TYPE == MI355X_TYPE_Q8_0) {
        const uint2 q = q8_load_chunk(row, c >> 2, c & 3);
        r.v.x = q.x;
        r.v.y = q.y;
        r.v.z = *(const uint16_t *)(row + (c >> 2) * FATTN_Q8_0_BYTES);
        r.v.w = 0;
    } else {
        typedef BlockFormat<TYPE> F;
        const char * blk = row + (c >> 2) * F::BYTES;
        const int    j0  = (c & 3) * 8;                                   // first element of the chunk inside its block
        const u32x2_a2 q = *(const u32x2_a2 *)(blk + F::QS + (j0 & 8));     // elements j and j + 16 share a byte
        const u32x2_a2 h = *(const u32x2_a2 *)blk;                          // the block's first 8 bytes: d [, m] [, fifth bits]
        r = narrow_chunk<TYPE>(q[0], q[1], h[0], h[1], c & 3);
    }
    return r;
}

// 4 unsigned bytes -> 4 exact f16 integers minus `off`: a byte becomes the low mantissa bits of 1024 + b
__device__ __forceinline__ void u8_widen(uint32_t w, float off, half2v & lo, half2v & hi) {
    const uint32_t a = __builtin_amdgcn_perm(w, 0x64646464u, 0x00050004u);   // {0x64, b1, 0x64, b0}
    const uint32_t b = __builtin_amdgcn_perm(w, 0x64646464u, 0x00070006u);   // {0x64, b3, 0x64, b2}
    const _Float16 o = (_Float16)(1024.0f + off);
    const half2v   o2 = {o, o};
    lo = __builtin_bit_cast(half2v, a) - o2;
    hi = __builtin_bit_cast(half2v, b) - o2;
}

template <int TYPE>
__device__ __forceinline__ half8 chunk_to_half8(const Chunk & r) {
    if constexpr (TYPE == MI355X_TYPE_F16) {
        return __builtin_bit_cast(half8, r.v);
    } else if constexpr (TYPE == MI355X_TYPE_Q8_0) {
        return q8_dequant(make_uint2(r.v.x, r.v.y), (uint16_t)r.v.z);
    } else {
        typedef BlockFormat<TYPE> F;
        uint32_t x = r.v.x, y = r.v.y;
        if (F::QH) {       // bit i of the byte of fifth bits -> bit 4 of byte i
            x |= (((r.v.w & 0xFu) * 0x00204081u) & 0x01010101u) << 4;
            y |= (((r.v.w >> 4) * 0x00204081u) & 0x01010101u) << 4;
        }
        half2v h0, h1, h2, h3;
        const float off = F::HAS_M ? 0.0f : (float)(F::LEVELS / 2);
        u8_widen(x, off, h0, h1);
        u8_widen(y, off, h2, h3);
        const _Float16 d = __builtin_bit_cast(_Float16, (uint16_t)(r.v.z & 0xFFFFu));
        const half2v   d2 = {d, d};
        if (F::HAS_M) {    // f16(q * d + m), one rounding
            const _Float16 m = __builtin_bit_cast(_Float16, (uint16_t)(r.v.z >> 16));
            const half2v   m2 = {m, m};
            h0 = __builtin_elementwise_fma(h0, d2, m2); h1 = __builtin_elementwise_fma(h1, d2, m2);
            h2 = __builtin_elementwise_fma(h2, d2, m2); h3 = __builtin_elementwise_fma(h3, d2, m2);
        } else {
            h0 *= d2; h1 *= d2; h2 *= d2; h3 *= d2;
        }
        half8 o;
        o[0] = h0[0]; o[1] = h0[1]; o[2] = h1[0]; o[3] = h1[1];
        o[4] = h2[0]; o[5] = h2[1]; o[6] = h3[0]; o[7] = h3[1];
        return o;
    }
}

// row pitch in bytes of the int8 V stage: the 16 rows one half of a transpose read touches start 4 banks apart
template <int D> constexpr int v8_pitch() { return D == 128 ? 136 : 80; }

// LDS bytes per workgroup: the per-wave f16 V stages, plus per-wave raw K and V stages when RAW; with V8 the V side is
// one int8 stage and the scales of its 32 x D/32 blocks instead
template <int D, int TYPE, bool RAW, bool V8>
constexpr int decode_lds_bytes() {
    constexpr int RS     = D / 32 * raw_block_bytes<TYPE>();
    constexpr int RAWSZ  = (STEP * RS + 511) / 512 * 512 + 64;                      // 9 x 64 units, padded
    constexpr int wave   = V8 ? RAWSZ + STEP * v8_pitch<D>() + D / 32 * STEP * 2
                              : STEP * (D + 32) * 2 + (RAW ? 2 * RAWSZ : 0);
    constexpr int stage  = DEC_WAVES * wave;
    constexpr int red    = DEC_WAVES * 16 * (D + 1 + 2) * 4;
    return stage > red ? stage : red;
}

// Where the 2-byte pieces of a step's 32 Q8_0 rows go in the int8 V stage, as offsets from the wave's LDS block: byte o
// of the step is byte o % RS of row o / RS; byte 0 of a 34-byte block is its scale's (-> f16 [block][key] behind the
// stage), bytes 2.. are its quants' (-> [key][column]).  Indexed by piece o / 2, padded to whole 64-lane loads of units.
template <int D>
struct V8Places {
    static constexpr int RS = D / 32 * FATTN_Q8_0_BYTES, UNIT = RS % 8 == 0 ? 8 : 4;
    static constexpr int UNITS = (STEP * RS / UNIT + 63) / 64 * 64;
    static constexpr int RAWSZ = (STEP * RS + 511) / 512 * 512 + 64;
    uint16_t at[UNITS * UNIT / 2];
};
template <int D>
constexpr V8Places<D> v8_places() {
    typedef V8Places<D> P;
    P t{};
    for (int o = 0; o < STEP * P::RS; o += 2) {
        const int row = o / P::RS, rem = o % P::RS, blk = rem / FATTN_Q8_0_BYTES, ib = rem % FATTN_Q8_0_BYTES;
        t.at[o / 2] = (uint16_t)(ib == 0 ? P::RAWSZ + STEP * v8_pitch<D>() + (blk * STEP + row) * 2
                                         : P::RAWSZ + row * v8_pitch<D>() + blk * 32 + ib - 2);
    }
    return t;
}
template <int D> __device__ const V8Places<D> v8_places_table = v8_places<D>();

// V8 (with RAW): V's quants go to LDS as bytes and come back through ds_read_b64_tr_b8 already in operand layout
// (8 consecutive keys of one column per lane).  The transposing read ignores the low three address bits and the quants
// of block b start at byte 34 b + 2 of a row, so the rows cannot stay as they are in memory: V arrives as the same
// coalesced stream as K, and each 2-byte piece of a unit is written to its place - a pair of quants to [key][column],
// a scale to [block][key] - by one ds_write_b16 whose address depends on the lane alone (read from a table behind the
// first K/V request: computing the 36 of them costs more instructions than a 32-key step).
// PAD: f16 rows of a.Dv elements (a multiple of 8 below D) read in place: the chunks of a row behind Dv are zeros in the
// registers, q is read and dst written up to Dv.  An instantiation of its own: the others stay the code they were.
template <int D, int TYPE, bool MASK, bool RAW, bool V8, bool PAD = false>
__global__ void __launch_bounds__(DEC_THREADS, 2) fattn_decode_kernel(const FattnArgs a) {
    static_assert(!PAD || (TYPE == MI355X_TYPE_F16 && !RAW && !V8), "other head sizes: f16 rows, read per lane");
    static_assert(!V8 || RAW, "the int8 V stage belongs to the streamed Q8_0 path");
    constexpr int KS  = D / 32;                    // reduction steps of Q.K^T (one Q8_0 block each)
    constexpr int DBK = D / 16;                    // 16-wide blocks of the output's d
    constexpr int CH  = D / 8;                     // chunks per row
    constexpr int NV  = STEP * CH / 64;            // V chunks per lane and step
    constexpr int PV  = D + 32;                    // LDS pitch in halves: 64 mod 128 bytes
    // raw streaming of contiguous rows of blocks: UNIT-byte loads, NU per lane and tensor and step
    constexpr int BB    = raw_block_bytes<TYPE>();
    constexpr int RS    = D / 32 * BB;
    constexpr int UNIT  = RS % 8 == 0 ? 8 : 4;
    constexpr int UPS   = STEP * RS / UNIT;        // units per full step
    constexpr int NU    = (UPS + 63) / 64;
    constexpr int RAWSZ = (STEP * RS + 511) / 512 * 512 + 64;
    static_assert(!RAW || FATTN_IS_BLOCK_TYPE(TYPE), "raw streaming is for rows of blocks");
    static_assert(!V8 || TYPE == MI355X_TYPE_Q8_0, "the int8 V stage holds Q8_0 quants");
    static_assert(NU * 64 * UNIT <= RAWSZ, "raw stage too small");

    // the per-wave stages; after the key loop the same memory carries the cross-wave reduction
    extern __shared__ __attribute__((aligned(16))) char smem[];
    constexpr int VP8 = v8_pitch<D>();
    constexpr int PCS = UNIT / 2;                  // (V8) 2-byte pieces per unit
    constexpr bool ONE = V8;                       // one register stage: the next step is requested once this one is in LDS
                                                   // (two stages, as the other forms have: 102-104 against 99 us at 64 x 4096)
    constexpr int WAVE_BYTES = V8 ? RAWSZ + STEP * VP8 + KS * STEP * 2 : STEP * PV * 2 + (RAW ? 2 * RAWSZ : 0);
    char * const wave_mem = smem + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6) * WAVE_BYTES;
    _Float16 * v_stage = (_Float16 *)wave_mem;                          // (!V8)
    char * k_rawst     = V8 ? wave_mem : wave_mem + STEP * PV * 2;
    char * v_rawst     = k_rawst + RAWSZ;                               // (!V8)
    char * v8_stage    = wave_mem + RAWSZ;                              // (V8) [32 keys][VP8]
    char * vsc_stage   = v8_stage + STEP * VP8;                         // (V8) f16 [KS][32 keys]
    float (*red_o)[16][D + 1]      = (float (*)[16][D + 1])smem;
    float (*red_ml)[16][2]         = (float (*)[16][2])(smem + DEC_WAVES * 16 * (D + 1) * 4);

    const int tid  = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);     // uniform: loop control and row bases stay scalar
    const int lane = tid & 63;
    const int j    = lane & 15;                    // query column
    const int g4   = lane >> 4;

    // workgroup = (split, 16-row chunk, KV head, batch), splits fastest.  With more than one chunk of rows per KV head the
    // chunks of one (split, KV head, batch) read the same keys: workgroups go to the 8 XCDs round-robin, each with its own
    // L2, so those chunks are numbered to follow each other on ONE XCD (the grid is rounded up to whole rounds of 8;
    // the spare workgroups leave here, before any barrier, and belong to no set of the merge).
    int     split, chunk, hk, b;
    int64_t set;                                   // index of (chunk, KV head, batch): the merge's counter
    if (a.q_chunks == 1) {
        split = blockIdx.x % a.n_splits;
        chunk = 0;
        hk    = (blockIdx.x / a.n_splits) % a.Hkv;
        b     = blockIdx.x / (a.n_splits * a.Hkv);
        set   = blockIdx.x / a.n_splits;
    } else {
        // (32-bit arithmetic: the grid has fewer than 2^31 workgroups, and 64-bit divisions are loops of a hundred
        //  instructions each - 1 us before the first request leaves)
        const uint32_t w  = blockIdx.x >> 3;
        const uint32_t p  = (w / (uint32_t)a.q_chunks) * 8u + (blockIdx.x & 7u);
        const uint32_t sh = (uint32_t)a.n_splits * (uint32_t)a.Hkv;           // (<= pairs <= the grid)
        if (p >= sh * (uint32_t)a.B) return;
        chunk = (int)(w % (uint32_t)a.q_chunks);
        split = (int)(p % (uint32_t)a.n_splits);
        hk    = (int)((p / (uint32_t)a.n_splits) % (uint32_t)a.Hkv);
        b     = (int)(p / sh);
        set   = ((int64_t)b * a.Hkv + hk) * a.q_chunks + chunk;
    }
    const int bk    = b / a.bq;

    // row r = iq1 * gqa + gg of this KV head  <->  query iq1 of q head hk*gqa + gg; column j is row chunk*16 + j
    const int  R      = a.Nq * a.gqa;
    const int  row0   = chunk * 16;
    const bool col_ok = row0 + j < R;
    const int  jc     = col_ok ? row0 + j : row0;
    const int  iq1    = jc / a.gqa;
    const int  h      = hk * a.gqa + jc % a.gqa;

    const int k_begin = split * a.keys_per_split;
    const int k_end   = min(a.Nkv, k_begin + a.keys_per_split);

    half8 qreg[KS];
    const char * kbase = a.k + (int64_t)hk * a.nbk2 + (int64_t)bk * a.nbk3;
    const char * vbase = a.v + (int64_t)hk * a.nbv2 + (int64_t)bk * a.nbv3;
    const uint16_t * mrow = MASK
        ? (const uint16_t *)(a.mask + (int64_t)iq1 * a.nbm1 + (int64_t)(h % a.Hm) * a.nbm2 + (int64_t)(b % a.Bm) * a.nbm3)
        : nullptr;
    const float mslope = MASK ? fattn_slope(a, h) * LOG2E : 0.0f;

    float4v oacc[DBK];
#pragma unroll
    for (int db = 0; db < DBK; db++) oacc[db] = float4v{0.0f, 0.0f, 0.0f, 0.0f};
    float m = 0.0f, l = 0.0f;
    bool  have = false;

    // loads of one step: K in operand layout (key = kb*16 + j, chunk = ks*4 + g4), V in row order
    Chunk kraw[2][RAW ? 1 : 2][RAW ? 1 : KS];
    Chunk vraw[2][RAW ? 1 : NV];
    typedef typename std::conditional<UNIT == 8, u32x2, uint32_t>::type unit_t;
    // (V8 keeps one register stage: index 0 whatever the step's stage number)
    unit_t kun[2][RAW ? NU : 1], vun[2][RAW ? NU : 1];
    // (V8) LDS offsets from wave_mem of the pieces of this lane's V units, two to a register
    uint32_t vdst[V8 ? NU : 1][V8 ? PCS / 2 : 1];
    // a partial last step: its loads are clamped to the last valid row or unit (branch-free, in bounds) and the
    // keys they stand for are excluded in the step
    auto issue = [&](int it, auto stage) __attribute__((always_inline)) {
        constexpr int s = decltype(stage)::value;
        const int j0 = k_begin + it * STEP;
        if (RAW) {
            // one coalesced stream per tensor
            const int last = min(STEP, k_end - j0) * (RS / UNIT) - 1;
            const char * kp = kbase + (int64_t)j0 * RS;
            const char * vp = vbase + (int64_t)j0 * RS;
#pragma unroll
            for (int i = 0; i < NU; i++) {
                const uint32_t off = (uint32_t)min(i * 64 + lane, last) * UNIT;
                kun[ONE ? 0 : s][i] = stream_load<unit_t>(kp + off);
                vun[ONE ? 0 : s][i] = stream_load<unit_t>(vp + off);
            }
            return;
        }
#pragma unroll
        for (int kb = 0; kb < 2; kb++) {
            const int key = min(j0 + kb * 16 + j, k_end - 1);
            const char * row = kbase + (int64_t)key * a.nbk1;
#pragma unroll
            for (int ks = 0; ks < KS; ks++) {
                if (!PAD || (ks * 4 + g4) * 8 < a.Dv) kraw[s][kb][ks] = load_chunk<TYPE>(row, ks * 4 + g4);
                else                                  kraw[s][kb][ks].v = make_uint4(0u, 0u, 0u, 0u);
            }
        }
#pragma unroll
        for (int i = 0; i < NV; i++) {
            const int flat = i * 64 + lane;
            const int key  = min(j0 + flat / CH, k_end - 1);
            if (!PAD || (flat % CH) * 8 < a.Dv) vraw[s][i] = load_chunk<TYPE>(vbase + (int64_t)key * a.nbv1, flat % CH);
            else                                vraw[s][i].v = make_uint4(0u, 0u, 0u, 0u);
        }
    };

    const int n_steps = k_end > k_begin ? (k_end - k_begin + STEP - 1) / STEP : 0;
    typedef std::integral_constant<int, 0> S0;

    // one step of 32 keys out of register stage s; the following step is requested into the other stage
    auto step = [&](const int it, auto stage) __attribute__((always_inline)) {
        constexpr int s = decltype(stage)::value;
        const int  j0   = k_begin + it * STEP;
        const bool tail = j0 + STEP > k_end;                  // wave-uniform
        // the following step's loads: into the other register stage, or (V8) into this one as soon as it is in LDS
        if (!ONE && it + DEC_WAVES < n_steps) issue(it + DEC_WAVES, std::integral_constant<int, 1 - s>{});

        if (RAW) {
#pragma unroll
            for (int i = 0; i < NU; i++) {
                *(unit_t *)(k_rawst + (i * 64 + lane) * UNIT) = kun[ONE ? 0 : s][i];
                if (!V8) *(unit_t *)(v_rawst + (i * 64 + lane) * UNIT) = vun[s][i];
            }
            if (V8) {
#pragma unroll
                for (int i = 0; i < NU; i++) {
                    if ((i + 1) * 64 > UPS && i * 64 + lane >= UPS) continue;      // past the step's 32 rows
                    uint32_t w[2];
                    if constexpr (UNIT == 8) { w[0] = vun[ONE ? 0 : s][i][0]; w[1] = vun[ONE ? 0 : s][i][1]; }
                    else                     { w[0] = vun[ONE ? 0 : s][i]; w[1] = 0; }
#pragma unroll
                    for (int k = 0; k < PCS; k++) {
                        const uint32_t dst = k % 2 ? vdst[i][k / 2] >> 16 : vdst[i][k / 2] & 0xFFFFu;
                        *(uint16_t *)(wave_mem + dst) = (uint16_t)(k % 2 ? w[k / 2] >> 16 : w[k / 2]);
                    }
                }
                // rows past k_end hold bytes of other rows: a zero scale makes exact zeros of them (the LDS runs a wave's
                // writes in order)
                if (tail) {
#pragma unroll
                    for (int t = 0; t < STEP * KS / 64; t++) {
                        const int idx = t * 64 + lane, row = idx / KS;
                        if (j0 + row >= k_end) *(uint16_t *)(vsc_stage + ((idx % KS) * STEP + row) * 2) = 0;
                    }
                }
            }
            if (ONE && it + DEC_WAVES < n_steps) issue(it + DEC_WAVES, stage);
            if (!V8 && tail) {
                // rows past k_end hold bytes of no row: a zero scale keeps what is made of them finite
#pragma unroll
                for (int t = 0; t < STEP * KS / 64; t++) {
                    const int idx = t * 64 + lane;
                    if (j0 + idx / KS >= k_end) {
                        *(uint16_t *)(v_rawst + (idx / KS) * RS + (idx % KS) * BB) = 0;
                        if (TYPE == MI355X_TYPE_Q4_1 || TYPE == MI355X_TYPE_Q5_1) *(uint16_t *)(v_rawst + (idx / KS) * RS + (idx % KS) * BB + 2) = 0;
                    }
                }
            }
            __builtin_amdgcn_wave_barrier();
        }
        // ---- S^T = K . Q^T ------------------------------------------------------------------
        float4v sc[2];
#pragma unroll
        for (int kb = 0; kb < 2; kb++) {
            sc[kb] = float4v{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int ks = 0; ks < KS; ks++) {
                Chunk c;
                // (V8: row i of tile kb is key (i / 4) * 8 + kb * 4 + i % 4, so that a lane's eight scores are eight
                //  consecutive keys, the order in which the transposing read hands out V)
                if (RAW && TYPE == MI355X_TYPE_Q8_0) c.v = q8_lds_chunk<true>(k_rawst, (V8 ? (j >> 2) * 8 + kb * 4 + (j & 3) : kb * 16 + j) * RS, ks, g4);
                else if (RAW) c = narrow_lds_chunk<RAW ? TYPE : MI355X_TYPE_Q4_0>(k_rawst, (kb * 16 + j) * RS, ks, g4);
                else     c = kraw[s][kb][ks];
                sc[kb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(chunk_to_half8<TYPE>(c), qreg[ks], sc[kb], 0, 0, 0);
            }
        }
        // V rows into this wave's LDS stage (f16, dequantised when the cache is Q8_0)
#pragma unroll
        for (int i = 0; i < (V8 ? 0 : NV); i++) {
            const int flat = i * 64 + lane;
            Chunk c;
            if (RAW && TYPE != MI355X_TYPE_Q8_0) {
                // one block of 16 rows per pass (4 lanes per row), so that the block index is a constant: pass i takes
                // block i % KS of rows 16 (i / KS) ... + 15
                const int row = (i / KS) * 16 + (lane >> 2), ch = (i % KS) * 4 + (lane & 3);
                c = narrow_lds_chunk<RAW ? TYPE : MI355X_TYPE_Q4_0>(v_rawst, row * RS, i % KS, lane & 3);
                *(half8 *)&v_stage[row * PV + ch * 8] = chunk_to_half8<TYPE>(c);
                continue;
            }
            if (RAW) c.v = q8_lds_chunk<false>(v_rawst, (flat / CH) * RS, (flat % CH) >> 2, (flat % CH) & 3);
            else     c = vraw[s][i];
            *(half8 *)&v_stage[(flat / CH) * PV + (flat % CH) * 8] = chunk_to_half8<TYPE>(c);
        }
        __builtin_amdgcn_wave_barrier();      // LDS runs a wave's instructions in order; keep the compiler from reordering

        // lane holds keys j0 + kb*16 + g4*4 + r of column j (V8: j0 + g4*8 + kb*4 + r)
        float sv[8];
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int key = V8 ? j0 + g4 * 8 + kb * 4 + r : j0 + kb * 16 + g4 * 4 + r;
                float x = sc[kb][r];
                if (MASK) x = fmaf(mslope, h2f_bits(mrow[min(key, k_end - 1)]), x);
                if (tail && key >= k_end) x = -INFINITY;
                sv[kb * 4 + r] = x - m;
            }

        // ---- P = 2^(s - m): no maximum unless the step's sum says the reference fell behind -----
        half8 preg;
        float lsum;
        const half2v ones = {(_Float16)1.0f, (_Float16)1.0f};
        auto exp_step = [&]() {
            float acc = 0.0f;
#pragma unroll
            for (int e = 0; e < 8; e += 2) {
                half2v p2;
                p2[0] = (_Float16)__builtin_amdgcn_exp2f(sv[e]);
                p2[1] = (_Float16)__builtin_amdgcn_exp2f(sv[e + 1]);
                acc = __builtin_amdgcn_fdot2(p2, ones, acc, false);
                preg[e] = p2[0];
                preg[e + 1] = p2[1];
            }
            lsum = acc;
        };
        exp_step();
        const bool redo = !(lsum <= SUM_LIMIT) || !have;
        if (__builtin_amdgcn_ballot_w64(redo) != 0) {
            float mx = sv[0];
#pragma unroll
            for (int e = 1; e < 8; e++) mx = fmaxf(mx, sv[e]);
            mx = fmaxf(mx, xor_shuffle(mx, 16));          // the four lanes of a column must agree
            mx = fmaxf(mx, xor_shuffle(mx, 32));
            float delta = 0.0f;
            if (mx > -INFINITY) {
                delta = have ? fmaxf(mx, 0.0f) : mx;
                have = true;
            }
            const float f = __builtin_amdgcn_exp2f(-delta);
            m += delta;
            l *= f;
#pragma unroll
            for (int db = 0; db < DBK; db++) oacc[db] *= f;
#pragma unroll
            for (int e = 0; e < 8; e++) sv[e] -= delta;
            exp_step();
        }
        l += lsum;

        // ---- O^T += V^T . P^T: transpose reads of the stage, 16 d at a time --------------------------
        if (V8) {
            half8 vsc[KS];
#pragma unroll
            for (int ks = 0; ks < KS; ks++) vsc[ks] = *(const half8 *)(vsc_stage + (ks * STEP + g4 * 8) * 2);
            // lane r of a group of 16 addresses key r / 2, columns 8 (r % 2) ..: the group receives keys g4*8 .. +7 x 16 columns
            const char * p0 = v8_stage + (g4 * 8 + (j >> 1)) * VP8 + (j & 1) * 8;
#pragma unroll
            for (int db = 0; db < DBK; db++) {
                typedef int int2v __attribute__((ext_vector_type(2)));
                const int2v q = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) int2v *)(p0 + db * 16));
                const half8 va = q8_dequant_keys((uint32_t)q[0], (uint32_t)q[1], vsc[db >> 1]);
                oacc[db] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va, preg, oacc[db], 0, 0, 0);
            }
        } else {
            const int kr = g4 * 4 + (j >> 2);
#pragma unroll
            for (int db = 0; db < DBK; db++) {
                const _Float16 * p0 = &v_stage[kr * PV + db * 16 + (j & 3) * 4];
                const _Float16 * p1 = p0 + 16 * PV;
                const half4 lo = __builtin_bit_cast(half4, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4v *)p0));
                const half4 hi = __builtin_bit_cast(half4, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4v *)p1));
                const half8 va = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                oacc[db] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va, preg, oacc[db], 0, 0, 0);
            }
        }
        __builtin_amdgcn_wave_barrier();
    };
    if (wave < n_steps) issue(wave, S0{});

    // (V8) where the pieces of this lane's V units go: read behind the first K/V request, needed when that has arrived
    if (V8) {
        static_assert(!V8 || (V8Places<D>::RAWSZ == RAWSZ && V8Places<D>::UNITS == NU * 64 && V8Places<D>::UNIT == UNIT), "table layout");
        const uint32_t * places = (const uint32_t *)v8_places_table<D>.at;
#pragma unroll
        for (int i = 0; i < NU; i++)
#pragma unroll
            for (int k = 0; k < PCS / 2; k++) vdst[i][k] = places[(i * 64 + lane) * (PCS / 2) + k];
    }
    // ---- Q -> f16 B operands in log2 units (after the first K/V request: the two cold misses overlap) ----
    {
        const float * qrow = (const float *)(a.q + (int64_t)iq1 * a.nbq1 + (int64_t)h * a.nbq2 + (int64_t)b * a.nbq3);
        const float   qs   = a.scale * LOG2E;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            half8 v;
            if constexpr (PAD) {
                // every lane reads 8 elements that exist (its own, or the row's first 8 where it has none) and the lanes
                // without scale them by zero: under a guard each, the 8 * KS loads waited for one another - 2 us per call.
                // (A q row with inf or NaN in it gives NaN either way.)
                const bool    own = ks * 32 + g4 * 8 < a.Dv;
                const float * q8  = qrow + (own ? ks * 32 + g4 * 8 : 0);
                const float   qsl = own ? qs : 0.0f;
#pragma unroll
                for (int e = 0; e < 8; e++) v[e] = (_Float16)(q8[e] * qsl);
            } else {
#pragma unroll
                for (int e = 0; e < 8; e++) v[e] = (_Float16)(qrow[ks * 32 + g4 * 8 + e] * qs);
            }
            qreg[ks] = v;
        }
    }
    for (int it = wave; it < n_steps; it += 2 * DEC_WAVES) {
        step(it, S0{});
        if (it + DEC_WAVES < n_steps) step(it + DEC_WAVES, std::integral_constant<int, ONE ? 0 : 1>{});
    }

    // ---- column totals, then the four waves through LDS ----------------------------------------------
    l += xor_shuffle(l, 16);
    l += xor_shuffle(l, 32);
    if (!have) m = -INFINITY;
    __syncthreads();                           // every wave is done with its stage
#pragma unroll
    for (int db = 0; db < DBK; db++)
#pragma unroll
        for (int r = 0; r < 4; r++) red_o[wave][j][db * 16 + g4 * 4 + r] = oacc[db][r];
    if (g4 == 0) {
        red_ml[wave][j][0] = m;
        red_ml[wave][j][1] = l;
    }
    __syncthreads();

    // thread t: column t / 16, a strided set of d
    const int col = tid >> 4;
    bool bad = false;                           // this column's result is not finite
    if (row0 + col < R) {
        float M = -INFINITY;
#pragma unroll
        for (int w = 0; w < DEC_WAVES; w++) M = fmaxf(M, red_ml[w][col][0]);
        float f[DEC_WAVES];
        float L = 0.0f;
#pragma unroll
        for (int w = 0; w < DEC_WAVES; w++) {
            const float mw = red_ml[w][col][0];
            f[w] = mw == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(mw - M);
            L += red_ml[w][col][1] * f[w];
        }
        bad = not_finite(L);
        const int     ciq1 = (row0 + col) / a.gqa;
        const int     ch   = hk * a.gqa + (row0 + col) % a.gqa;
        const int64_t row  = ((int64_t)b * a.Nq + ciq1) * a.Hq + ch;
        const int dv = PAD ? a.Dv : D;              // dst rows are dv floats; partial rows stay D apart
        for (int d = tid & 15; d < dv; d += 16) {
            float acc = 0.0f;
#pragma unroll
            for (int w = 0; w < DEC_WAVES; w++) acc += red_o[w][col][d] * f[w];
            bad = bad || not_finite(acc);
            if (a.n_splits == 1) {
                a.dst[row * dv + d] = L > 0.0f ? acc / L : 0.0f;
            } else if (a.counters) {
                device_store(a.part_acc + (row * a.n_splits + split) * D + d, acc);
            } else {
                a.part_acc[(row * a.n_splits + split) * D + d] = acc;
            }
        }
        if (a.n_splits > 1 && (tid & 15) == 0) {
            // natural-log units, as the merge expects them
            float * pm = a.part_ml + (row * a.n_splits + split) * 2;
            const float mn = M == -INFINITY ? -INFINITY : M * 0.6931471805599453f;
            if (a.counters) {
                device_store(pm, mn);
                device_store(pm + 1, L);
            } else {
                pm[0] = mn;
                pm[1] = L;
            }
        }
    }
    // An excluded key was multiplied by a probability of zero above, not skipped.  For finite K/V that is the same thing; a
    // cache slot that holds NaN or inf bits (never written, and masked out for that reason) turns the products into NaN.
    // Such a row shows in its result, and is computed again the way the CPU op does it - excluded keys not read at all.
    // Without a mask every key is visible and a non-finite result is the answer.  (Columns 4w .. 4w + 3 belong to wave w
    // in both passes: the second store follows the first in the same wave.)
    bool redone = false;
    if constexpr (MASK) {
        const uint64_t badmask = __builtin_amdgcn_ballot_w64(bad);
        if (badmask != 0) {
            redone = true;
            __threadfence();
#pragma unroll 1
            for (int c = 0; c < 4; c++) {
                const int r = row0 + wave * 4 + c;
                if (((badmask >> (16 * c)) & 0xFFFFu) != 0 && r < R)
                    attn_row_redo<TYPE, D>(a, r / a.gqa, hk * a.gqa + r % a.gqa, b, split, k_begin, k_end);
            }
        }
    }
    // the last of the n_splits workgroups of this (chunk, KV head, batch) merges its rows: no launch for the merge
    if (a.n_splits > 1 && a.counters) {
        if (!fattn_last_of_set(a, set, a.n_splits, (int *)smem, redone)) return;
        constexpr int LPR = D / 4;                  // lanes per row: 8 or 4 rows per pass
        for (int c = tid / LPR; c < 16 && row0 + c < R; c += DEC_THREADS / LPR) {
            const int r = row0 + c;
            fattn_merge_row<true>(a, ((int64_t)b * a.Nq + r / a.gqa) * a.Hq + hk * a.gqa + r % a.gqa, tid % LPR);
        }
    }
}

template <int D, int TYPE, bool MASK, bool RAW, bool V8 = false, bool PAD = false>
int launch_one(const FattnArgs & a, hipStream_t stream) {
    const int64_t pairs = (int64_t)a.n_splits * a.Hkv * a.B;
    const int64_t wgs   = a.q_chunks == 1 ? pairs : (pairs + 7) / 8 * 8 * a.q_chunks;      // as the kernel numbers them
    if (wgs > 0x7fffffff || a.q_chunks != (a.Nq * a.gqa + 15) / 16) return (int)hipErrorInvalidValue;
    const dim3 grid((unsigned)wgs);
    constexpr int lds = decode_lds_bytes<D, TYPE, RAW, V8>();
    static std::atomic<uint64_t> lds_allowed{0};
    const hipError_t e = fattn_allow_lds((const void *)fattn_decode_kernel<D, TYPE, MASK, RAW, V8, PAD>, lds, lds_allowed);
    if (e != hipSuccess) return (int)e;
    hipLaunchKernelGGL((fattn_decode_kernel<D, TYPE, MASK, RAW, V8, PAD>), grid, dim3(DEC_THREADS), lds, stream, a);
    return (int)hipGetLastError();
}

template <int D, int TYPE>
int launch(const FattnArgs & a, hipStream_t stream) {
    if (a.Dv != a.D) {              // another head size on f16 rows, or nothing
        if constexpr (TYPE == MI355X_TYPE_F16)
            return a.mask ? launch_one<D, TYPE, true, false, false, true>(a, stream) : launch_one<D, TYPE, false, false, false, true>(a, stream);
        return (int)hipErrorInvalidValue;
    }
    if constexpr (FATTN_IS_BLOCK_TYPE(TYPE)) {
        // contiguous rows, and every step of every (head, batch, split) starts on a unit boundary
        constexpr int RS   = D / 32 * raw_block_bytes<TYPE>();
        constexpr int UNIT = RS % 8 == 0 ? 8 : 4;
        const bool raw = a.nbk1 == RS && a.nbv1 == RS &&
                         !((uintptr_t)a.k % UNIT) && !((uintptr_t)a.v % UNIT) &&
                         !(a.nbk2 % UNIT) && !(a.nbk3 % UNIT) && !(a.nbv2 % UNIT) && !(a.nbv3 % UNIT);
        static const bool no_raw = getenv("MI355X_FATTN_DECODE_NO_STREAM") != nullptr;      // the per-lane path, for comparison runs
        if (raw && !no_raw) {
            if constexpr (TYPE == MI355X_TYPE_Q8_0) {
                static const bool f16_stage = getenv("MI355X_FATTN_DECODE_F16_STAGE") != nullptr;     // the earlier V path, for comparison runs
                if (!f16_stage) return a.mask ? launch_one<D, TYPE, true, true, true>(a, stream) : launch_one<D, TYPE, false, true, true>(a, stream);
            }
            return a.mask ? launch_one<D, TYPE, true, true>(a, stream) : launch_one<D, TYPE, false, true>(a, stream);
        }
    }
    return a.mask ? launch_one<D, TYPE, true, false>(a, stream) : launch_one<D, TYPE, false, false>(a, stream);
}

}  // namespace

bool fattn_decode_supported(const FattnArgs & a, int ktype) {
    if (a.D != 64 && a.D != 128) return false;
    if (a.Dv != a.D && (a.Dv % 8 || a.Dv > a.D || ktype != MI355X_TYPE_F16)) return false;       // other head sizes: f16 rows read in place
    if (a.Nq < 1 || a.Nkv < 1) return false;
    if ((int64_t)a.Nq * a.gqa > ((int64_t)1 << 20)) return false;      // 16-row chunks of the rows that share a KV head
    if (a.softcap != 0.0f) return false;
    if (ktype == MI355X_TYPE_F16) return a.kv_aligned16 != 0;
    if (ktype == MI355X_TYPE_Q8_0) return a.kv_aligned4 != 0;
    if (FATTN_IS_BLOCK_TYPE(ktype)) return a.kv_aligned2 != 0;
    return false;
}

int fattn_decode_launch(const FattnArgs & a, int ktype, hipStream_t stream) {
    if (ktype == MI355X_TYPE_F16) return a.D == 64 ? launch<64, MI355X_TYPE_F16>(a, stream) : launch<128, MI355X_TYPE_F16>(a, stream);
    switch (ktype) {
#define DEC(T) case T: return a.D == 64 ? launch<64, T>(a, stream) : launch<128, T>(a, stream)
        DEC(MI355X_TYPE_Q8_0);
        DEC(MI355X_TYPE_Q4_0);
        DEC(MI355X_TYPE_Q4_1);
        DEC(MI355X_TYPE_Q5_0);
        DEC(MI355X_TYPE_Q5_1);
#undef DEC
        default: return (int)hipErrorInvalidValue;
    }
}
