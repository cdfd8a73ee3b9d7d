/*
 * CPU oracle for GGML_OP_FLASH_ATTN_EXT and the KV-cache copies around it.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing under oracle/ is part of the shipped
 * library: it is the checker that the parity tests, the smoke run and the
 * benchmark's cpu_baseline leg compare the HIP kernels against.
 *
 * The arithmetic restated here lives in a third-party dependency of the
 * reference that is absent from its tree: ggml (CrispStrobe/ggml, branch
 * sync/upstream-v0.17, commit a0f7289d = ggml v0.17.0 + fork patches; pin named
 * in tools/upstream-prs/SYNC-v0.17-CONFLICTS.md:3-7,197).  The restatement is
 * anchored on the reference's own call sites and notes, cited per function.
 *
 * Parity status of each function:
 *   ora_fp32_to_fp16 / ora_fp16_to_fp32 : pinned (IEEE-754 binary16, RNE; checked
 *       exhaustively against numpy.float16).
 *   ora_quantize_row_q8_0 / ora_dequantize_row_q8_0 : pinned by the reference's
 *       description of the format (tools/upstream-prs/09-metal-q8_0-bit-match.md:24-31),
 *       known-answer blocks and the round-trip bound of
 *       tests/test-kv-quant-roundtrip.cpp:193.
 *   ora_flash_attn_ext, mode ORA_MODE_EXACT : pinned by the mathematics (fp64
 *       textbook softmax(scale*QK^T + mask)V written independently in numpy, closed
 *       forms, brute force) and by the layouts the call sites fix.
 *   ora_alibi_slope (max_bias) : pinned at max_bias = 8 by the published ALiBi head-slope construction, for
 *       power-of-two and other head counts; other values of max_bias scale the exponent the same way.
 *   ora_vec_dot_q8_0_q8_0 and the Q-row quantisation ggml-like mode uses for Q8_0 K : pinned by the reference's
 *       description of ggml-cpu's arithmetic (tools/upstream-prs/09-metal-q8_0-bit-match.md:24-36: d = amax/127
 *       kept in f32 for the division, q = rint(x/d), int8 x int8 -> int32 per block, sumf += sumi * d_k * d_q) on
 *       hand-built blocks with integer answers.
 *   ora_flash_attn_ext, mode ORA_MODE_GGML_LIKE (f32 online softmax in key order, Q row quantised to Q8_0 for
 *       Q8_0 K, f32 accumulator) : the recurrence is the reference's own (src/core/cpu_attention.h:53-83, compiled
 *       into oracle/_ref/ and compared where its tree is present); that the op quantises Q for a Q8_0 K is
 *       recalled.  logit_softcap is pinned by its closed form only.
 *   ora_relpos_bias : pinned by the reference's own graph (src/core/fastconformer.h:98-102,
 *       876-918, every node of which is restated literally, the rel_shift view as byte strides)
 *       and by the mathematics: numpy matmul + numpy.lib.stride_tricks.as_strided with the
 *       view's strides, and the closed form BD[j, i] = <Q_v[i], R[T-1+j-i]>, on small shapes.
 */
#ifndef FATTN_ORACLE_H
#define FATTN_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ggml type ids of the types this path meets */
enum { ORA_TYPE_F32 = 0, ORA_TYPE_F16 = 1, ORA_TYPE_Q4_0 = 2, ORA_TYPE_Q4_1 = 3, ORA_TYPE_Q5_0 = 6, ORA_TYPE_Q5_1 = 7, ORA_TYPE_Q8_0 = 8 };

enum { ORA_MODE_EXACT = 0, ORA_MODE_GGML_LIKE = 1 };

/* rounding of x/d in the Q8_0 quantiser */
enum { ORA_ROUND_NEAREST_EVEN = 0, ORA_ROUND_HALF_AWAY = 1 };

#define ORA_QK8_0 32

typedef struct {
    uint16_t d;               /* fp16 scale */
    int8_t   qs[ORA_QK8_0];   /* quants */
} ora_block_q8_0;             /* 34 bytes, no padding */

/* The narrower block-32 cache types the reference's CRISPASR_KV_QUANT accepts (src/core/attention.h:79-105).  ggml is
 * absent from the reference's tree: layouts and arithmetic are ggml's as recalled (quantize_row_q*_ref /
 * dequantize_row_q*), held by the tests to known-answer blocks worked out by hand from these definitions and to the
 * reference's own round-trip bounds (tests/test-kv-quant-roundtrip.cpp:184-199).
 * Element j (< 16) of a block sits in the low nibble of qs[j], element j + 16 in the high nibble; the fifth bit of
 * element e (0..31) is bit e of qh (little-endian 32-bit). */
typedef struct { uint16_t d; uint8_t qs[16]; } ora_block_q4_0;                       /* 18 bytes: x = (q - 8) * d   */
typedef struct { uint16_t d, m; uint8_t qs[16]; } ora_block_q4_1;                    /* 20 bytes: x = q * d + m     */
typedef struct { uint16_t d; uint8_t qh[4]; uint8_t qs[16]; } ora_block_q5_0;        /* 22 bytes: x = (q - 16) * d  */
typedef struct { uint16_t d, m; uint8_t qh[4]; uint8_t qs[16]; } ora_block_q5_1;     /* 24 bytes: x = q * d + m     */

/* a ggml tensor view: ne = elements per dim, nb = byte strides, dim 0 fastest */
typedef struct {
    const void * data;
    int32_t      type;
    int64_t      ne[4];
    int64_t      nb[4];
} ora_tensor;

uint16_t ora_fp32_to_fp16(float f);
float    ora_fp16_to_fp32(uint16_t h);
void     ora_fp32_to_fp16_row(const float * x, uint16_t * y, int64_t n);
void     ora_fp16_to_fp32_row(const uint16_t * x, float * y, int64_t n);

void ora_quantize_row_q8_0(const float * x, ora_block_q8_0 * y, int64_t n, int rounding);
void ora_dequantize_row_q8_0(const ora_block_q8_0 * x, float * y, int64_t n);

/* any block-32 type (Q8_0 with round-to-nearest-even): n values <-> n/32 blocks; 0, or -2 for a type without blocks */
int    ora_quantize_row(int type, const float * x, void * y, int64_t n);
int    ora_dequantize_row(int type, const void * x, float * y, int64_t n);
size_t ora_block_bytes(int type);      /* bytes of one block of 32 (0: not a block type) */

/* deterministic N(0,1): splitmix64 counter -> Box-Muller in fp64 -> float.
 * element i of stream `seed` depends only on (seed, i). */
void ora_randn(uint64_t seed, int64_t n, float * out);
/* uniform integer in [lo, hi] for element i of stream seed */
int64_t ora_randint(uint64_t seed, int64_t i, int64_t lo, int64_t hi);

/* dst: contiguous f32 [DV, Hq, Nq, B].  mask may be NULL (or mask->data NULL).
 * returns 0, or a negative code when the shapes break the op's contract. */
int ora_flash_attn_ext(const ora_tensor * q, const ora_tensor * k, const ora_tensor * v,
                       const ora_tensor * mask, float * dst,
                       float scale, float max_bias, float logit_softcap,
                       int mode, int n_threads);

/* KV-cache writes (ggml_cpy F32 -> F16/F32/block-32 type into a strided view whose rows
 * are contiguous): src and dst have equal ne, src is F32.  rounding applies to Q8_0 only. */
int ora_cpy_f32(const ora_tensor * src, void * dst_data, int32_t dst_type, const int64_t dst_nb[4],
                int rounding);

/* FastConformer's relative-position mask: f16( scale * rel_shift(R^T Q_v) + add ), see the .c file.
 * qv F32 [D, Nq, H, B]; r F32/F16 [D, Nq+n_kv-1, 1|H.., 1|B..]; add NULL or F32/F16 [n_kv, Nq, 1|H, 1|B];
 * dst f16 [n_kv, Nq, H, B] contiguous. */
int ora_relpos_bias(const ora_tensor * qv, const ora_tensor * r, const ora_tensor * add,
                    float scale, int64_t n_kv, uint16_t * dst, int n_threads);

/* pieces of the above, exported so that tests can hold them to known answers */
float ora_alibi_slope(float max_bias, int64_t h, int64_t n_head);
float ora_vec_dot_q8_0_q8_0(const ora_block_q8_0 * x, const ora_block_q8_0 * y, int64_t n);

int ora_max_threads(void);

#ifdef __cplusplus
}
#endif
#endif
