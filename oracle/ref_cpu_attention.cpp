// TEST INFRASTRUCTURE ONLY.  C entry points around the reference's own scalar attention helpers, compiled from
// the header where it lies in the reference tree (src/core/cpu_attention.h: cpu_dot :27-39,
// cpu_online_softmax_accumulate :53-83) into oracle/_ref/.  Nothing of the reference is copied here: the two
// drivers below only call those helpers the way the reference's hand-written CPU backends do, so that the
// oracle's restatements can be held against compiled reference code:
//   ref_mha_f32        - wav2vec2's encoder self-attention loop (src/wav2vec2-ggml.cpp:1908-1924)
//   ref_relpos_mha_f32 - FireRed's conformer attention with the relative-position term, pos_idx = T-1-tq+tk
//                        (src/firered_asr.cpp:1525-1577)
// ggml's FLASH_ATTN_EXT itself cannot be built here (the ggml submodule is empty).
#include "core/cpu_attention.h"

#include <cmath>
#include <vector>

using crispasr::cpu_attn::cpu_dot;
using crispasr::cpu_attn::cpu_online_softmax_accumulate;

extern "C" {

// Q, K, V: [T, H] row-major with H = n_heads * head_dim; head h at column offset h * head_dim.  out: [T, H].
void ref_mha_f32(int T, int n_heads, int head_dim, const float * Q, const float * K, const float * V, float scale,
                 float * out) {
    const int H = n_heads * head_dim;
    for (int h = 0; h < n_heads; h++) {
        for (int tq = 0; tq < T; tq++) {
            const int     off = h * head_dim;
            const float * q   = Q + tq * H + off;
            cpu_online_softmax_accumulate(T, head_dim, V + off, H, out + tq * H + off,
                                          [&](int tk) { return cpu_dot(q, K + tk * H + off, head_dim) * scale; });
        }
    }
}

// Q, K, V: [T, d] row-major, P: [T_pe, d], bu / bv: [nh, hd]; score = ((q + bu).k + (q + bv).p[T-1-tq+tk]) / sqrt(hd)
void ref_relpos_mha_f32(int T, int T_pe, int nh, int hd, const float * Q, const float * K, const float * V,
                        const float * P, const float * bu, const float * bv, float * out) {
    const int   d     = nh * hd;
    const float scale = 1.0f / sqrtf((float)hd);
    std::vector<float> qbu(hd), qbv(hd);
    for (int h = 0; h < nh; h++) {
        for (int tq = 0; tq < T; tq++) {
            const float * q = Q + h * hd + tq * d;
            for (int dd = 0; dd < hd; dd++) {
                qbu[dd] = q[dd] + bu[h * hd + dd];
                qbv[dd] = q[dd] + bv[h * hd + dd];
            }
            cpu_online_softmax_accumulate(T, hd, V + h * hd, d, out + tq * d + h * hd, [&](int tk) -> float {
                const float content  = cpu_dot(qbu.data(), K + h * hd + tk * d, hd);
                float       position = 0.0f;
                const int   pos_idx  = T - 1 - tq + tk;
                if ((unsigned)pos_idx < (unsigned)T_pe) position = cpu_dot(qbv.data(), P + h * hd + pos_idx * d, hd);
                return (content + position) * scale;
            });
        }
    }
}

}  // extern "C"
