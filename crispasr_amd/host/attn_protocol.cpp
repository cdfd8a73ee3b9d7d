// Native host driver above the C ABI: the attention calls of the reference's Whisper benchmark protocol
// (examples/bench/bench.cpp:103-163 - heat twice, then 256 single-token decodes at n_past = i, 64 decodes of 5
// tokens, 16 prompts of 256 tokens) on a large-v3-shaped decoder: 32 layers x (self-attention over the f16 KV
// cache with the causal f16 mask the runtime builds, src/crispasr.cpp:3467-3499, + cross-attention over the
// 1536-row zero-padded encoder memory, :3262-3282).  It links nothing but libmi355x_fattn.so - no HIP headers, no
// torch - and so also shows what a ggml backend's graph_compute pays per FLASH_ATTN_EXT node on the host side.
//
// A small self-check (one masked GQA-free call against a double-precision loop) guards the timings; the parity
// tests proper live in tests/.
//
// usage: mi355x_attn_protocol [n_layers] [hbm|host] [write]
//   host : the KV caches, Q and the result live in host-visible buffers (mi355x_host_buffer_alloc), which is where an
//          unmodified runtime puts them when this library is its GPU backend (src/crispasr.cpp:3942-3971); the caches are
//          filled the way the graphs fill them, by F32 -> F16 copies into cache views (src/crispasr.cpp:2956-2973,
//          3185-3203), so they are mirrored in HBM and attention reads the mirror
//   write: every decode also writes its new K and V rows into the self-attention cache first (two copies per layer)
// -> one JSON line on stdout, exit code 0 when the self-check passes
#include "mi355x_fattn.h"

#include <chrono>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

namespace {

constexpr int D = 64, H = 20, CTX = 448, NENC = 1536, NSTATE = D * H;

#define CHECK(call)                                                                                   \
    do {                                                                                              \
        const int rc_ = (call);                                                                       \
        if (rc_ != MI355X_OK) {                                                                       \
            fprintf(stderr, "%s failed: %s (%s)\n", #call, mi355x_status_string(rc_), mi355x_last_error()); \
            exit(2);                                                                                  \
        }                                                                                             \
    } while (0)

// IEEE binary16 from binary32, round to nearest even
uint16_t f2h(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    x &= 0x7fffffffu;
    if (x >= 0x7f800000u) return (uint16_t)(sign | 0x7c00u | (x > 0x7f800000u ? 0x200u : 0));
    if (x >= 0x47800000u) return (uint16_t)(sign | 0x7c00u);
    if (x < 0x33000001u) return (uint16_t)sign;
    if (x < 0x38800000u) {
        const int shift = 126 - (int)(x >> 23);
        const uint32_t m = (x & 0x7fffffu) | 0x800000u;
        uint32_t h = m >> shift;
        const uint32_t rem = m & ((1u << shift) - 1), halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (h & 1))) h++;
        return (uint16_t)(sign | h);
    }
    uint32_t h = ((x >> 23) - 112) << 10 | ((x >> 13) & 0x3ffu);
    const uint32_t rem = x & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1))) h++;
    return (uint16_t)(sign | h);
}
float h2f(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1f, m = h & 0x3ffu, x;
    if (e == 0) {
        if (m == 0) x = sign;
        else { e = 113; while (!(m & 0x400u)) { m <<= 1; e--; } x = sign | (e << 23) | ((m & 0x3ffu) << 13); }
    } else if (e == 31) x = sign | 0x7f800000u | (m << 13);
    else x = sign | ((e + 112) << 23) | (m << 13);
    float f;
    memcpy(&f, &x, 4);
    return f;
}

uint64_t rng_state = 0x9e3779b97f4a7c15ull;
float rnd() {                                   // uniform in [-1, 1)
    rng_state = rng_state * 6364136223846793005ull + 1442695040888963407ull;
    return (float)((rng_state >> 40) / 8388608.0 - 1.0);
}

bool g_host = false;                            // caches, Q and the result in host-visible buffers

void * dev_alloc(size_t n) {
    void * p = nullptr;
    CHECK(mi355x_buffer_alloc(n, &p));
    return p;
}
void * cache_alloc(size_t n) {
    if (!g_host) return dev_alloc(n);
    void * p = nullptr;
    CHECK(mi355x_host_buffer_alloc(n, &p));
    return p;
}
mi355x_tensor flat(void * data, int type, int64_t n) {
    mi355x_tensor t;
    t.data = data;
    t.type = type;
    t.ne[0] = n; t.ne[1] = t.ne[2] = t.ne[3] = 1;
    t.nb[0] = type == MI355X_TYPE_F32 ? 4 : 2;
    t.nb[1] = t.nb[2] = t.nb[3] = t.nb[0] * (size_t)n;
    return t;
}
// a cache of n f16 values, zeros from zero_from on.  In host mode it is written as the graphs write it: an F32 tensor
// copied (F32 -> F16) into the cache by the library's copy kernel, which is also what gives the buffer its mirror.
void * dev_f16(size_t n, size_t zero_from = (size_t)-1) {
    if (g_host) {
        std::vector<float> f(n);
        for (size_t i = 0; i < n; i++) f[i] = i >= zero_from ? 0.0f : rnd();
        void * src = dev_alloc(n * 4);
        CHECK(mi355x_buffer_set(src, f.data(), n * 4, nullptr));
        void * p = cache_alloc(n * 2);
        const mi355x_tensor s = flat(src, MI355X_TYPE_F32, (int64_t)n), d = flat(p, MI355X_TYPE_F16, (int64_t)n);
        CHECK(mi355x_cpy(&s, &d, nullptr));
        CHECK(mi355x_stream_synchronize(nullptr));
        CHECK(mi355x_buffer_free(src));
        return p;
    }
    std::vector<uint16_t> h(n);
    for (size_t i = 0; i < n; i++) h[i] = i >= zero_from ? 0 : f2h(rnd());
    void * p = dev_alloc(n * 2);
    CHECK(mi355x_buffer_set(p, h.data(), n * 2, nullptr));
    return p;
}

mi355x_tensor view(void * data, int type, int64_t ne0, int64_t ne1, int64_t ne2, size_t nb0, size_t nb1, size_t nb2) {
    mi355x_tensor t;
    t.data = data;
    t.type = type;
    t.ne[0] = ne0; t.ne[1] = ne1; t.ne[2] = ne2; t.ne[3] = 1;
    t.nb[0] = nb0; t.nb[1] = nb1; t.nb[2] = nb2; t.nb[3] = nb2 * (size_t)ne2;
    return t;
}

struct Layer { void *ks, *vs, *kc, *vc; };

// max |gpu - reference| of one self-attention call with the causal mask, reference in double precision
double self_check(void * q_dev, const std::vector<float> & q_host, void * out_dev) {
    const int n_tok = 5, n_past = 37, n_kv = n_past + n_tok;
    std::vector<uint16_t> kh((size_t)n_kv * NSTATE), vh((size_t)n_kv * NSTATE), mh((size_t)n_tok * n_kv);
    for (auto & x : kh) x = f2h(rnd());
    for (auto & x : vh) x = f2h(rnd());
    for (int t = 0; t < n_tok; t++)
        for (int j = 0; j < n_kv; j++) mh[(size_t)t * n_kv + j] = j > n_past + t ? 0xfc00u : 0;      // -inf beyond the token
    void * kd = dev_alloc(kh.size() * 2); void * vd = dev_alloc(vh.size() * 2); void * md = dev_alloc(mh.size() * 2);
    CHECK(mi355x_buffer_set(kd, kh.data(), kh.size() * 2, nullptr));
    CHECK(mi355x_buffer_set(vd, vh.data(), vh.size() * 2, nullptr));
    CHECK(mi355x_buffer_set(md, mh.data(), mh.size() * 2, nullptr));
    const mi355x_tensor q = view(q_dev, MI355X_TYPE_F32, D, n_tok, H, 4, 4 * NSTATE, 4 * D);
    const mi355x_tensor k = view(kd, MI355X_TYPE_F16, D, n_kv, H, 2, 2 * NSTATE, 2 * D);
    const mi355x_tensor v = view(vd, MI355X_TYPE_F16, D, n_kv, H, 2, 2 * NSTATE, 2 * D);
    const mi355x_tensor m = view(md, MI355X_TYPE_F16, n_kv, n_tok, 1, 2, 2 * (size_t)n_kv, 2 * (size_t)n_kv * n_tok);
    const mi355x_tensor o = view(out_dev, MI355X_TYPE_F32, D, H, n_tok, 4, 4 * D, 4 * NSTATE);
    mi355x_fattn_params p;
    memset(&p, 0, sizeof(p));
    p.scale = 0.125f;
    CHECK(mi355x_flash_attn_ext(&q, &k, &v, &m, &o, &p, nullptr));
    std::vector<float> got((size_t)n_tok * NSTATE);
    CHECK(mi355x_buffer_get(got.data(), out_dev, got.size() * 4, nullptr));
    double worst = 0.0;
    std::vector<double> s(n_kv);
    for (int t = 0; t < n_tok; t++)
        for (int h = 0; h < H; h++) {
            double mx = -INFINITY;
            for (int j = 0; j <= n_past + t; j++) {
                double acc = 0.0;
                for (int d = 0; d < D; d++) acc += (double)q_host[((size_t)t * H + h) * D + d] * h2f(kh[((size_t)j * H + h) * D + d]);
                s[j] = acc * 0.125;
                mx = std::fmax(mx, s[j]);
            }
            double l = 0.0;
            for (int j = 0; j <= n_past + t; j++) { s[j] = std::exp(s[j] - mx); l += s[j]; }
            for (int d = 0; d < D; d++) {
                double acc = 0.0;
                for (int j = 0; j <= n_past + t; j++) acc += s[j] * h2f(vh[((size_t)j * H + h) * D + d]);
                worst = std::fmax(worst, std::fabs(acc / l - got[((size_t)t * H + h) * D + d]));
            }
        }
    mi355x_buffer_free(kd); mi355x_buffer_free(vd); mi355x_buffer_free(md);
    return worst;
}

}  // namespace

int main(int argc, char ** argv) {
    const int L = argc > 1 ? atoi(argv[1]) : 32;
    bool with_write = false;
    for (int i = 2; i < argc; i++) {
        if (!strcmp(argv[i], "host")) g_host = true;
        if (!strcmp(argv[i], "write")) with_write = true;
    }
    int n_dev = 0;
    CHECK(mi355x_device_count(&n_dev));
    if (n_dev < 1) { fprintf(stderr, "no device\n"); return 3; }
    CHECK(mi355x_set_device(0));

    std::vector<Layer> layers(L);
    for (auto & l : layers) {
        l.ks = dev_f16((size_t)CTX * NSTATE);
        l.vs = dev_f16((size_t)CTX * NSTATE);
        l.kc = dev_f16((size_t)NENC * NSTATE, (size_t)1500 * NSTATE);
        l.vc = dev_f16((size_t)NENC * NSTATE, (size_t)1500 * NSTATE);
    }
    std::vector<float> qh((size_t)256 * NSTATE);
    for (auto & x : qh) x = rnd();
    void * q_dev = cache_alloc(qh.size() * 4);
    CHECK(mi355x_buffer_set(q_dev, qh.data(), qh.size() * 4, nullptr));
    void * out_dev = cache_alloc(qh.size() * 4);
    // the rows a decode writes into the cache: Kcur / Vcur of the graph, F32 [n_state, n_tok]
    void * kv_new = cache_alloc(qh.size() * 4);
    CHECK(mi355x_buffer_set(kv_new, qh.data(), qh.size() * 4, nullptr));

    const double err = self_check(q_dev, qh, out_dev);

    // causal masks for (n_tok, n_past), built once as the runtime's graph inputs are
    auto make_mask = [&](int n_tok, int n_past) {
        const int n_kv = n_past + n_tok;
        std::vector<uint16_t> mh((size_t)n_tok * n_kv);
        for (int t = 0; t < n_tok; t++)
            for (int j = 0; j < n_kv; j++) mh[(size_t)t * n_kv + j] = j > n_past + t ? 0xfc00u : 0;
        void * d = cache_alloc(mh.size() * 2);          // a graph input: in the backend's compute buffer
        CHECK(mi355x_buffer_set(d, mh.data(), mh.size() * 2, nullptr));
        return d;
    };
    std::vector<void *> mask1(256);
    for (int i = 0; i < 256; i++) mask1[i] = make_mask(1, i);
    void * mask5 = make_mask(5, 0);
    void * mask256 = make_mask(256, 0);

    mi355x_fattn_params ps, pc;
    memset(&ps, 0, sizeof(ps));
    ps.scale = 1.0f;                                   // Q and K are pre-scaled by 64^-0.25 in the self-attention
    pc = ps;
    pc.scale = 0.35355339059327373f;                   // 64^-0.25: only K is pre-scaled in the cross-attention
    auto decode = [&](int n_tok, int n_past, void * mask) {
        const int n_kv = n_past + n_tok;
        const mi355x_tensor q = view(q_dev, MI355X_TYPE_F32, D, n_tok, H, 4, 4 * NSTATE, 4 * D);
        const mi355x_tensor o = view(out_dev, MI355X_TYPE_F32, D, H, n_tok, 4, 4 * D, 4 * NSTATE);
        const mi355x_tensor m = view(mask, MI355X_TYPE_F16, n_kv, n_tok, 1, 2, 2 * (size_t)n_kv, 2 * (size_t)n_kv * n_tok);
        for (const auto & l : layers) {
            if (with_write) {
                // ggml_cpy(Kcur, ggml_view_1d(kv_self.k, n_tokens * n_state, offset of row n_past)), src/crispasr.cpp:3185-3203
                const mi355x_tensor src = flat(kv_new, MI355X_TYPE_F32, (int64_t)n_tok * NSTATE);
                const mi355x_tensor dk = flat((char *)l.ks + (size_t)n_past * NSTATE * 2, MI355X_TYPE_F16, (int64_t)n_tok * NSTATE);
                const mi355x_tensor dv = flat((char *)l.vs + (size_t)n_past * NSTATE * 2, MI355X_TYPE_F16, (int64_t)n_tok * NSTATE);
                CHECK(mi355x_cpy(&src, &dk, nullptr));
                CHECK(mi355x_cpy(&src, &dv, nullptr));
            }
            const mi355x_tensor ks = view(l.ks, MI355X_TYPE_F16, D, n_kv, H, 2, 2 * NSTATE, 2 * D);
            const mi355x_tensor vs = view(l.vs, MI355X_TYPE_F16, D, n_kv, H, 2, 2 * NSTATE, 2 * D);
            const mi355x_tensor kc = view(l.kc, MI355X_TYPE_F16, D, NENC, H, 2, 2 * NSTATE, 2 * D);
            const mi355x_tensor vc = view(l.vc, MI355X_TYPE_F16, D, NENC, H, 2, 2 * NSTATE, 2 * D);
            CHECK(mi355x_flash_attn_ext(&q, &ks, &vs, &m, &o, &ps, nullptr));
            CHECK(mi355x_flash_attn_ext(&q, &kc, &vc, nullptr, &o, &pc, nullptr));
        }
    };
    for (int h = 0; h < 2; h++) {                      // heat, as the protocol does
        decode(256, 0, mask256);
        for (int i = 0; i < 256; i++) decode(1, i, mask1[i]);
        decode(5, 0, mask5);
    }
    CHECK(mi355x_stream_synchronize(nullptr));

    struct Phase { const char * name; int n; double ms; } phases[3] = {{"single_token_x256", 256, 0}, {"batch5_x64", 64, 0}, {"prompt256_x16", 16, 0}};
    for (int ph = 0; ph < 3; ph++) {
        const auto t0 = std::chrono::steady_clock::now();
        for (int i = 0; i < phases[ph].n; i++) {
            if (ph == 0) decode(1, i, mask1[i]);
            else if (ph == 1) decode(5, 0, mask5);
            else decode(256, 0, mask256);
        }
        CHECK(mi355x_stream_synchronize(nullptr));
        phases[ph].ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
    }
    size_t mirror = 0, valid = 0, uploaded = 0;
    if (g_host) CHECK(mi355x_host_buffer_mirror_stats(layers[0].kc, &mirror, &valid, &uploaded));
    printf("{\"layers\": %d, \"buffers\": \"%s\", \"kv_write_per_decode\": %s, \"self_check_max_abs\": %.3e", L, g_host ? "host-visible, caches mirrored in HBM" : "HBM",
           with_write ? "true" : "false", err);
    if (g_host) printf(", \"cross_cache_mirror\": {\"mirror_bytes\": %zu, \"valid_bytes\": %zu, \"uploaded_bytes\": %zu}", mirror, valid, uploaded);
    for (const auto & p : phases)
        printf(", \"%s\": {\"ms_total\": %.3f, \"ms_per_decode\": %.4f, \"us_per_attention_call\": %.2f}", p.name, p.ms, p.ms / p.n,
               p.ms * 1e3 / ((double)p.n * 2 * L));
    printf("}\n");
    return err <= 2e-3 ? 0 : 1;
}
