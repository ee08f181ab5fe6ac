// Host (CPU) share of hybrid layers: the neurons that are not GPU-resident are computed on host threads from the
// same predictor logits and merged into the layer output, as the hybrid variants of llm_build_sparse_mul_mat /
// llm_build_sparse_axpy do (llama.cpp:4581-4593, 4635-4646: CPU part with gpu_idx + GPU part with gpu_bucket +
// ggml_add).  Arithmetic follows the reference's CPU kernels (ggml.c:14030-14282, 14314-14618): activations
// rounded to fp16 (F16 weights) or Q8_0 blocks (Q4_0 weights), fp32 accumulation.  The down projection is split
// over threads by output COLUMN, so no two threads ever add into the same element (the reference splits by row
// and merges the per-thread vectors without a lock, ggml.c:14433-14458).
#include "cold_path.hpp"
#include "engine_internal.hpp"
#include "runtime.hpp"

#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <atomic>
#include <chrono>
#include <condition_variable>
#include <functional>
#include <mutex>
#include <thread>
#include <vector>

#if defined(__AVX2__) && defined(__F16C__) && defined(__FMA__)
#include <immintrin.h>
#define PI_COLD_SIMD 1
#endif

#define PI_TRY(expr) do { int _rc = (expr); if (_rc != PI_OK) return _rc; } while (0)

namespace pi {

namespace {

struct BlockQ4 { uint16_t d; uint8_t qs[16]; } __attribute__((packed));
struct BlockQ8 { uint16_t d; int8_t qs[32]; } __attribute__((packed));

inline float h2f(uint16_t h) {
#ifdef PI_COLD_SIMD
    return _cvtsh_ss(h);
#else
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16, e = (h >> 10) & 0x1F, m = h & 0x3FF, x;
    if (e == 0) { if (!m) x = sign; else { int s = 0; while (!(m & 0x400)) { m <<= 1; s++; } m &= 0x3FF; x = sign | ((uint32_t)(113 - s) << 23) | (m << 13); } }
    else if (e == 31) x = sign | 0x7F800000u | (m << 13);
    else x = sign | ((e + 112) << 23) | (m << 13);
    float f; memcpy(&f, &x, 4); return f;
#endif
}
inline uint16_t f2h(float f) {
#ifdef PI_COLD_SIMD
    return (uint16_t)_cvtss_sh(f, 0);
#else
    uint32_t x; memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u; x &= 0x7FFFFFFFu;
    if (x >= 0x7F800000u) return (uint16_t)(sign | 0x7C00u | (x > 0x7F800000u ? 0x0200u : 0));
    if (x >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u);
    if (x < 0x33000001u) return (uint16_t)sign;
    int e = (int)(x >> 23) - 127; uint32_t m = (x & 0x7FFFFFu) | 0x800000u; int shift; uint32_t base;
    if (e < -14) { shift = 13 + (-14 - e); base = 0; } else { shift = 13; base = (uint32_t)(e + 15) << 10; m &= 0x7FFFFFu; }
    uint32_t q = m >> shift, rem = m & ((1u << shift) - 1), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1))) q++;
    return (uint16_t)(sign | (base + q));
#endif
}

float dot_f16(int n, const uint16_t * w, const uint16_t * x) {
#ifdef PI_COLD_SIMD
    __m256 a0 = _mm256_setzero_ps(), a1 = a0;
    int i = 0;
    for (; i + 16 <= n; i += 16) {
        a0 = _mm256_fmadd_ps(_mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(w + i))), _mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(x + i))), a0);
        a1 = _mm256_fmadd_ps(_mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(w + i + 8))), _mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(x + i + 8))), a1);
    }
    a0 = _mm256_add_ps(a0, a1);
    __m128 r = _mm_add_ps(_mm256_castps256_ps128(a0), _mm256_extractf128_ps(a0, 1));
    r = _mm_hadd_ps(r, r); r = _mm_hadd_ps(r, r);
    float s = _mm_cvtss_f32(r);
    for (; i < n; ++i) s += h2f(w[i]) * h2f(x[i]);
    return s;
#else
    float s = 0.f;
    for (int i = 0; i < n; ++i) s += h2f(w[i]) * h2f(x[i]);
    return s;
#endif
}

// Q4_0 row . Q8_0 activations (ggml_vec_dot_q4_0_q8_0, ggml-quants.c:2512-2650): exact integer dot per block of 32, scaled by
// d4*d8 and accumulated in fp32 (eight lanes with AVX2, each holding four of a block's products, summed at the end)
float dot_q4_q8(int n, const BlockQ4 * w, const BlockQ8 * x) {
#ifdef PI_COLD_SIMD
    __m256 acc = _mm256_setzero_ps();
    const __m256i lowmask = _mm256_set1_epi8(0x0F), eight = _mm256_set1_epi8(8), ones = _mm256_set1_epi16(1);
    for (int b = 0; b < n / 32; ++b) {
        const __m128i q = _mm_loadu_si128((const __m128i *)w[b].qs);
        __m256i bx = _mm256_and_si256(_mm256_set_m128i(_mm_srli_epi16(q, 4), q), lowmask);     // elements 0..15 | 16..31
        bx = _mm256_sub_epi8(bx, eight);
        const __m256i by = _mm256_loadu_si256((const __m256i *)x[b].qs);
        const __m256i prod = _mm256_maddubs_epi16(_mm256_sign_epi8(bx, bx), _mm256_sign_epi8(by, bx));   // |w| * (x * sign(w)), pairs summed
        const __m256 pf = _mm256_cvtepi32_ps(_mm256_madd_epi16(prod, ones));
        acc = _mm256_fmadd_ps(_mm256_set1_ps(h2f(w[b].d) * h2f(x[b].d)), pf, acc);
    }
    __m128 r = _mm_add_ps(_mm256_extractf128_ps(acc, 1), _mm256_castps256_ps128(acc));
    r = _mm_add_ps(r, _mm_movehl_ps(r, r));
    r = _mm_add_ss(r, _mm_movehdup_ps(r));
    return _mm_cvtss_f32(r);
#else
    float acc = 0.f;
    for (int b = 0; b < n / 32; ++b) {
        int sum = 0;
        for (int j = 0; j < 16; ++j) {
            sum += ((int)(w[b].qs[j] & 0x0F) - 8) * (int)x[b].qs[j];
            sum += ((int)(w[b].qs[j] >> 4) - 8) * (int)x[b].qs[j + 16];
        }
        acc = fmaf(h2f(w[b].d) * h2f(x[b].d), (float)sum, acc);
    }
    return acc;
#endif
}

// out[32 b .. 32 b + 32) += float((q4 - 8) * a) * (d4 * sc) for the blocks [b0, b1) of one Q4_0 row
// (ggml_axpy_q4_0_q8_0, ggml-quants.c:2426-2509: integer product, one fp32 multiply, one fp32 add)
void axpy_q4_blocks(const BlockQ4 * row, int b0, int b1, int a, float sc, float * out) {
    for (int b = b0; b < b1; ++b) {
        const float dd = h2f(row[b].d) * sc;
        float * o = out + b * 32;
#ifdef PI_COLD_SIMD
        const __m128i q = _mm_loadu_si128((const __m128i *)row[b].qs);
        const __m128i lowmask = _mm_set1_epi8(0x0F), eight = _mm_set1_epi8(8);
        const __m128i lo = _mm_sub_epi8(_mm_and_si128(q, lowmask), eight), hi = _mm_sub_epi8(_mm_and_si128(_mm_srli_epi16(q, 4), lowmask), eight);
        const __m256i av = _mm256_set1_epi16((short)a);
        const __m256 dv = _mm256_set1_ps(dd);
        const __m256i plo = _mm256_mullo_epi16(_mm256_cvtepi8_epi16(lo), av), phi = _mm256_mullo_epi16(_mm256_cvtepi8_epi16(hi), av);
        const __m256i parts[4] = {_mm256_cvtepi16_epi32(_mm256_castsi256_si128(plo)), _mm256_cvtepi16_epi32(_mm256_extracti128_si256(plo, 1)),
                                  _mm256_cvtepi16_epi32(_mm256_castsi256_si128(phi)), _mm256_cvtepi16_epi32(_mm256_extracti128_si256(phi, 1))};
        for (int k = 0; k < 4; ++k)
            _mm256_storeu_ps(o + 8 * k, _mm256_add_ps(_mm256_loadu_ps(o + 8 * k), _mm256_mul_ps(_mm256_cvtepi32_ps(parts[k]), dv)));
#else
        for (int q = 0; q < 16; ++q) {
            const float p0 = (float)(((int)(row[b].qs[q] & 0x0F) - 8) * a) * dd, p1 = (float)(((int)(row[b].qs[q] >> 4) - 8) * a) * dd;
            o[q]      = o[q] + p0;
            o[q + 16] = o[q + 16] + p1;
        }
#endif
    }
}

// The same sums with the loops exchanged: the 32 outputs of block b stay in registers while every listed row adds its product, in
// list order, so each output sees the additions of axpy_q4_blocks row by row in the same order (bit-identical) without a load and
// a store of the output per row.  rows[k] = start of row k, a[k] != 0 its Q8_0 value of h, sc[k] that block's scale.
void axpy_q4_rows(const BlockQ4 * const * rows, const int * a, const float * sc, int n_rows, int b0, int b1, float * out) {
#ifdef PI_COLD_SIMD
    const __m128i lowmask = _mm_set1_epi8(0x0F), eight = _mm_set1_epi8(8);
    for (int b = b0; b < b1; ++b) {
        __m256 acc[4] = {_mm256_setzero_ps(), _mm256_setzero_ps(), _mm256_setzero_ps(), _mm256_setzero_ps()};
        for (int k = 0; k < n_rows; ++k) {
            const BlockQ4 & blk = rows[k][b];
            const __m256 dv = _mm256_set1_ps(h2f(blk.d) * sc[k]);
            const __m128i q = _mm_loadu_si128((const __m128i *)blk.qs);
            const __m128i lo = _mm_sub_epi8(_mm_and_si128(q, lowmask), eight), hi = _mm_sub_epi8(_mm_and_si128(_mm_srli_epi16(q, 4), lowmask), eight);
            const __m256i av = _mm256_set1_epi16((short)a[k]);
            const __m256i plo = _mm256_mullo_epi16(_mm256_cvtepi8_epi16(lo), av), phi = _mm256_mullo_epi16(_mm256_cvtepi8_epi16(hi), av);
            acc[0] = _mm256_add_ps(acc[0], _mm256_mul_ps(_mm256_cvtepi32_ps(_mm256_cvtepi16_epi32(_mm256_castsi256_si128(plo))), dv));
            acc[1] = _mm256_add_ps(acc[1], _mm256_mul_ps(_mm256_cvtepi32_ps(_mm256_cvtepi16_epi32(_mm256_extracti128_si256(plo, 1))), dv));
            acc[2] = _mm256_add_ps(acc[2], _mm256_mul_ps(_mm256_cvtepi32_ps(_mm256_cvtepi16_epi32(_mm256_castsi256_si128(phi))), dv));
            acc[3] = _mm256_add_ps(acc[3], _mm256_mul_ps(_mm256_cvtepi32_ps(_mm256_cvtepi16_epi32(_mm256_extracti128_si256(phi, 1))), dv));
        }
        for (int i = 0; i < 4; ++i) _mm256_storeu_ps(out + b * 32 + 8 * i, acc[i]);
    }
#else
    for (int i = b0 * 32; i < b1 * 32; ++i) out[i] = 0.f;
    for (int k = 0; k < n_rows; ++k) axpy_q4_blocks(rows[k], b0, b1, a[k], sc[k], out);
#endif
}

// the cold rows live in host DRAM and a token touches each of them once: fetch the next row while this one is used
inline void prefetch_bytes(const void * p, size_t n) {
#ifdef PI_COLD_SIMD
    const char * b = (const char *)p;
    for (size_t o = 0; o < n; o += 64) _mm_prefetch(b + o, _MM_HINT_T0);
#else
    (void)p; (void)n;
#endif
}

// x86 quantize_row_q8_0 semantics (ggml-quants.c:702-760): d = amax/127 stored as fp16, q = rint(x * 127/amax)
void quantize_q8(const float * x, BlockQ8 * y, int n) {
    for (int b = 0; b < n / 32; ++b) {
#ifdef PI_COLD_SIMD
        const __m256 sign = _mm256_set1_ps(-0.0f);
        __m256 v[4], mx = _mm256_setzero_ps();
        for (int k = 0; k < 4; ++k) { v[k] = _mm256_loadu_ps(x + b * 32 + 8 * k); mx = _mm256_max_ps(mx, _mm256_andnot_ps(sign, v[k])); }
        __m128 m4 = _mm_max_ps(_mm256_extractf128_ps(mx, 1), _mm256_castps256_ps128(mx));
        m4 = _mm_max_ps(m4, _mm_movehl_ps(m4, m4));
        m4 = _mm_max_ss(m4, _mm_movehdup_ps(m4));
        const float amax = _mm_cvtss_f32(m4);
        const float d = amax / 127.f, id = amax != 0.f ? 127.f / amax : 0.f;
        y[b].d = f2h(d);
        const __m256 mul = _mm256_set1_ps(id);
        __m256i q[4];
        for (int k = 0; k < 4; ++k) q[k] = _mm256_cvtps_epi32(_mm256_mul_ps(v[k], mul));        // round to nearest even, as rintf
        const __m256i p01 = _mm256_packs_epi32(q[0], q[1]), p23 = _mm256_packs_epi32(q[2], q[3]);   // lanes interleave: fixed below
        __m256i p = _mm256_packs_epi16(p01, p23);
        p = _mm256_permutevar8x32_epi32(p, _mm256_setr_epi32(0, 4, 1, 5, 2, 6, 3, 7));
        _mm256_storeu_si256((__m256i *)y[b].qs, p);
#else
        float amax = 0.f;
        for (int j = 0; j < 32; ++j) amax = fmaxf(amax, fabsf(x[b * 32 + j]));
        const float d = amax / 127.f, id = amax != 0.f ? 127.f / amax : 0.f;
        y[b].d = f2h(d);
        for (int j = 0; j < 32; ++j) y[b].qs[j] = (int8_t)(int)rintf(x[b * 32 + j] * id);
#endif
    }
}

// Fork/join over persistent host threads.  A decode step forks twice per layer with a few microseconds of work each,
// so idle workers spin on the generation counter for a short while (a condition-variable wake-up costs more than the
// work) and only then go to sleep; the caller takes share 0 and spins for the join.
class Pool {
  public:
    explicit Pool(int n) : n_(n) {
        for (int i = 1; i < n_; ++i) threads_.emplace_back([this, i] { loop(i); });
    }
    ~Pool() {
        stop_.store(true);
        gen_.fetch_add(1);
        { std::lock_guard<std::mutex> g(mu_); }
        cv_.notify_all();
        for (auto & t : threads_) t.join();
    }
    int size() const { return n_; }
    void run(const std::function<void(int, int)> & fn) {
        fn_ = &fn;
        pending_.store(n_ - 1, std::memory_order_relaxed);
        gen_.fetch_add(1);                                    // publishes fn_ and pending_
        if (sleepers_.load() > 0) { { std::lock_guard<std::mutex> g(mu_); } cv_.notify_all(); }
        fn(0, n_);
        while (pending_.load(std::memory_order_acquire) != 0) cpu_relax();
    }

  private:
    static void cpu_relax() {
#ifdef PI_COLD_SIMD
        _mm_pause();
#else
        std::this_thread::yield();
#endif
    }
    void loop(int id) {
        uint64_t seen = 0;
        for (;;) {
            auto t0 = std::chrono::steady_clock::now();
            for (int it = 0; gen_.load(std::memory_order_acquire) == seen; ++it) {
                cpu_relax();
                if ((it & 255) == 255 && std::chrono::steady_clock::now() - t0 > std::chrono::microseconds(kSpinUs)) {
                    std::unique_lock<std::mutex> g(mu_);
                    sleepers_.fetch_add(1);
                    cv_.wait(g, [&] { return gen_.load() != seen; });
                    sleepers_.fetch_sub(1);
                }
            }
            seen = gen_.load(std::memory_order_acquire);
            if (stop_.load()) return;
            (*fn_)(id, n_);
            pending_.fetch_sub(1, std::memory_order_release);
        }
    }
    static constexpr int kSpinUs = 500;
    int n_;
    std::vector<std::thread> threads_;
    std::mutex mu_;
    std::condition_variable cv_;
    const std::function<void(int, int)> * fn_ = nullptr;
    std::atomic<int> pending_{0}, sleepers_{0};
    std::atomic<uint64_t> gen_{0};
    std::atomic<bool> stop_{false};
};

}  // namespace

struct ColdLayer {
    std::vector<float> norm_w, norm_b;          // host copies of the FFN-input norm
    std::vector<int32_t> cold_rows;             // neurons with gpu_idx == 0, ascending
    std::vector<uint32_t> cold_words;           // the same as bits: bit j of word w = neuron 32 w + j
};

struct ColdPath {
    Pool * pool = nullptr;
    std::vector<ColdLayer> layers;
    // pinned staging
    float * logits = nullptr, * src = nullptr, * h_gpu = nullptr;      // device -> host, consumed before the layer call returns
    float * h_full[2] = {nullptr, nullptr}, * out[2] = {nullptr, nullptr};   // host -> device, read by the GPU after the call returned: two sets, used in turn
    BlockQ8 * xq8_pin = nullptr;                // Q8_0 blocks of the normalised FFN input, written by the fused Q4_0 kernel
    uint16_t * x16_pin = nullptr;               // fp16 normalised FFN input, written by the fused F16 kernel
    uint32_t * words_pin = nullptr;             // activity words of the layer in flight, written by the split-off Q4_0 predictor launch
    int flip = 0;
    hipEvent_t ev_in = nullptr, ev_h = nullptr;
    std::vector<float> hval;                    // h of the active cold neurons, in the order of act
    std::vector<const BlockQ4 *> dn_rows; std::vector<int> dn_a; std::vector<float> dn_sc;    // the rows of one Q4_0 down projection
    // PI_COLD_TRACE=1: mean host time per phase of a layer call, printed when the model is freed
    bool trace = false;
    double t_phase[6] = {0, 0, 0, 0, 0, 0};
    long long n_calls = 0, n_cold_active = 0;
    std::chrono::steady_clock::time_point t_last_return;
    double t_between = 0;
    std::vector<float> xn;
    std::vector<uint16_t> x16;
    std::vector<BlockQ8> xq8, hq8;
    std::vector<int32_t> act;                   // active cold neurons of the current token
    int d = 0, ff = 0;

    // Q4_0 layers served without the launching thread: the stream carries hand-over kernels (pi_k_host_signal / pi_k_host_wait),
    // a service thread takes the posted layers in order, waits for the device's signal, computes the host share with the pool and
    // answers through two flag words.  Device and host count the hand-overs in step.
    pi_model * model = nullptr;
    bool async = false;
    std::vector<int> async_layers;              // hybrid layers that take this route, ascending
    uint32_t * flags = nullptr;                 // pinned: [0] logits ready, [8] resident h ready (device -> host), [16] h complete, [32] output share complete, [48] stop word
    std::vector<float *> h_async;               // per layer, pinned: h of that variant; the device writes the resident neurons' entries, the host its own
                                                // (one vector per layer, because the resident set differs from layer to layer)
    std::vector<std::vector<int32_t>> prev_act; // per layer: the host's entries that are non-zero from the previous token
    uint32_t * d_seq = nullptr, * d_status = nullptr;    // device words: hand-over count, non-zero once a device-side wait gave up
    std::thread service;
    std::vector<int> ring;                      // posted layer indices, single producer / single consumer
    std::atomic<uint64_t> posted{0}, served{0};
    std::atomic<bool> stop{false}, failed{false};
    std::atomic<int> service_asleep{0};
    std::mutex mu;
    std::condition_variable cv;
};

namespace { void service_loop(ColdPath * c); }

ColdPath * cold_create(pi_model * m) {
    ColdPath * c = new ColdPath();
    const pi_hparams & hp = m->hp;
    c->d = hp.n_embd; c->ff = hp.n_ff;
    int nt = (int)std::thread::hardware_concurrency();
    if (nt > 8) nt = 8;        // the forks are microseconds long and the workers spin between them: more threads only add join latency
    if (const char * e = getenv("PI_COLD_THREADS")) { const int v = atoi(e); if (v > 0) nt = v; }
    if (nt < 1) nt = 1;
    c->pool = new Pool(nt);
    if (const char * e = getenv("PI_COLD_TRACE")) c->trace = e[0] == '1';
    c->layers.resize(hp.n_layer);
    const bool falcon = hp.arch == PI_ARCH_FALCON;
    for (int il = 0; il < hp.n_layer; ++il) {
        if (!m->L(il, PI_T_GPU_BUCKET).dev) continue;
        ColdLayer & cl = c->layers[il];
        Tensor & nw = m->L(il, falcon ? PI_T_ATTN_NORM : PI_T_FFN_NORM);
        cl.norm_w.resize(c->d);
        if (pi_memcpy_d2h(cl.norm_w.data(), nw.dev, sizeof(float) * c->d) != PI_OK) { cold_destroy(c); return nullptr; }
        if (falcon) {
            cl.norm_b.resize(c->d);
            if (pi_memcpy_d2h(cl.norm_b.data(), m->L(il, PI_T_ATTN_NORM_B).dev, sizeof(float) * c->d) != PI_OK) { cold_destroy(c); return nullptr; }
        }
        const int32_t * gid = (const int32_t *)m->L(il, PI_T_GPU_IDX).host;
        cl.cold_words.assign((size_t)(c->ff + 31) / 32, 0u);
        for (int j = 0; j < c->ff; ++j) if (gid[j] != 1) { cl.cold_rows.push_back(j); cl.cold_words[j >> 5] |= 1u << (j & 31); }
    }
    auto pin = [](size_t n) { void * p = nullptr; return hipHostMalloc(&p, n * sizeof(float), hipHostMallocCoherent) == hipSuccess ? (float *)p : nullptr; };
    c->xq8_pin = (BlockQ8 *)pin((size_t)(c->d / 32 + 1) * sizeof(BlockQ8) / sizeof(float) + 1);
    c->x16_pin = (uint16_t *)pin((size_t)c->d / 2 + 8);
    c->words_pin = (uint32_t *)pin((size_t)c->ff / 32 + 8);
    c->logits = pin(c->ff); c->src = pin(c->d); c->h_gpu = pin(c->ff);
    for (int i = 0; i < 2; ++i) { c->h_full[i] = pin(c->ff); c->out[i] = pin(c->d); }
    if (!c->logits || !c->src || !c->h_gpu || !c->h_full[0] || !c->h_full[1] || !c->out[0] || !c->out[1] || !c->xq8_pin || !c->x16_pin || !c->words_pin) { set_error("cold path: pinned host allocation failed"); cold_destroy(c); return nullptr; }
    if (hipEventCreateWithFlags(&c->ev_in, hipEventDisableTiming) != hipSuccess || hipEventCreateWithFlags(&c->ev_h, hipEventDisableTiming) != hipSuccess) {
        set_error("cold path: event creation failed"); cold_destroy(c); return nullptr;
    }
    c->xn.resize(c->d); c->x16.resize(c->d); c->xq8.resize(c->d / 32 + 1); c->hq8.resize(c->ff / 32 + 1);
    c->act.reserve(c->ff); c->hval.resize(c->ff);
    c->model = m;
    const char * sync_only = getenv("PI_COLD_SYNC");
    if (!(sync_only && sync_only[0] == '1')) {
        for (int il = 0; il < hp.n_layer; ++il) {
            Tensor & up = m->L(il, PI_T_FFN_UP);
            if (!m->L(il, PI_T_GPU_BUCKET).dev || m->L(il, PI_T_FC2).type != PI_TYPE_F16 || !m->hot_words[il]) continue;
            const int r = (int)m->L(il, PI_T_FC1).ne1;
            if ((up.type == PI_TYPE_Q4_0 && pi_k_pred_upgate_q4_supported(c->ff, r, c->d)) ||
                (up.type == PI_TYPE_F16 && pi_k_sparse_ffn_two_phase_supported(c->ff, r, c->d)))
                c->async_layers.push_back(il);
        }
    }
    if (!c->async_layers.empty()) {
        void * fl = nullptr;
        if (hipHostMalloc(&fl, 64 * sizeof(uint32_t), hipHostMallocCoherent) != hipSuccess) { set_error("cold path: pinned host allocation failed"); cold_destroy(c); return nullptr; }
        c->flags = (uint32_t *)fl;
        memset(c->flags, 0, 64 * sizeof(uint32_t));
        c->h_async.assign(hp.n_layer, nullptr);
        c->prev_act.resize(hp.n_layer);
        for (int il : c->async_layers) {
            c->h_async[il] = pin(c->ff);
            if (!c->h_async[il]) { set_error("cold path: pinned host allocation failed"); cold_destroy(c); return nullptr; }
            memset(c->h_async[il], 0, sizeof(float) * c->ff);
        }
        c->d_seq = m->alloc<uint32_t>(1); c->d_status = m->alloc<uint32_t>(1);
        if (!c->d_seq || !c->d_status || pi_memset(c->d_seq, 0, 4) != PI_OK || pi_memset(c->d_status, 0, 4) != PI_OK) { cold_destroy(c); return nullptr; }
        c->ring.resize(1 << 16);
        c->async = true;
        c->service = std::thread([c] { service_loop(c); });
    }
    return c;
}

void cold_destroy(ColdPath * c) {
    if (!c) return;
    if (c->trace && c->n_calls) {
        const double n = (double)c->n_calls;
        fprintf(stderr, "cold path, mean us per layer call over %lld calls: between calls %.1f | wait inputs %.1f | norm+list %.1f | up/gate %.1f | wait h + upload %.1f | down %.1f | merge launch %.1f | active cold neurons %.1f\n",
                c->n_calls, c->t_between / n, c->t_phase[0] / n, c->t_phase[1] / n, c->t_phase[2] / n, c->t_phase[3] / n, c->t_phase[4] / n, c->t_phase[5] / n, (double)c->n_cold_active / n);
    }
    // wait kernels that are still queued (a decode that returned early) must not poll a host that is gone for their whole time limit:
    // raise the host's stop word, which every wait kernel checks, let the stream drain, and only then stop the thread and free the flags
    if (c->flags) __atomic_store_n(&c->flags[48], 1u, __ATOMIC_RELEASE);
    if (c->model && c->model->stream) (void)hipStreamSynchronize(c->model->stream);
    if (c->service.joinable()) {
        c->stop.store(true);
        { std::lock_guard<std::mutex> g(c->mu); }
        c->cv.notify_all();
        c->service.join();
    }
    if (c->flags) (void)hipHostFree(c->flags);
    for (float * p : c->h_async) if (p) (void)hipHostFree(p);
    delete c->pool;
    for (float * p : {c->logits, c->src, c->h_gpu, c->h_full[0], c->h_full[1], c->out[0], c->out[1]}) if (p) (void)hipHostFree(p);
    if (c->xq8_pin) (void)hipHostFree(c->xq8_pin);
    if (c->x16_pin) (void)hipHostFree(c->x16_pin);
    if (c->words_pin) (void)hipHostFree(c->words_pin);
    if (c->ev_in) (void)hipEventDestroy(c->ev_in);
    if (c->ev_h) (void)hipEventDestroy(c->ev_h);
    delete c;
}

namespace {
// The host waits for the device twice per layer and the waits are short: poll the event before falling back to a blocking wait.
hipError_t wait_event(hipEvent_t ev) {
    const auto t0 = std::chrono::steady_clock::now();
    for (int it = 0;; ++it) {
        const hipError_t e = hipEventQuery(ev);
        if (e != hipErrorNotReady) return e;
        if ((it & 63) == 63 && std::chrono::steady_clock::now() - t0 > std::chrono::milliseconds(2)) return hipEventSynchronize(ev);
    }
}
}  // namespace

namespace {
// ---- the host share's three steps, shared by the variant that launches between them and the one that answers the stream's signals ----

// neurons of this layer that are not GPU-resident and whose predictor logit reaches the threshold, ascending, into c->act
// the same list from the activity words the predictor launch left in pinned memory: 1.4 KB to read instead of a logit per cold neuron
int list_active_cold_words(ColdPath * c, const ColdLayer & cl) {
    c->act.clear();
    const uint32_t * aw = c->words_pin;
    const int nw = (int)cl.cold_words.size();
    for (int w = 0; w < nw; ++w) {
        const uint32_t all = aw[w];
        if ((all & cl.cold_words[w]) == 0u) continue;
        for (uint32_t bits = all & cl.cold_words[w]; bits; bits &= bits - 1) c->act.push_back(w * 32 + __builtin_ctz(bits));
    }
    return (int)c->act.size();
}

int list_active_cold(ColdPath * c, const ColdLayer & cl, float thr) {
    c->act.clear();
    for (int j : cl.cold_rows) if (!(c->logits[j] < thr)) c->act.push_back(j);
    return (int)c->act.size();
}

// h of the listed neurons into c->hval: up/gate dots on the input the device rounded (Q8_0 blocks for Q4_0 rows, fp16 for F16 rows;
// ggml.c:14030-14282), the next neuron's rows prefetched while this one's are used
void host_upgate(ColdPath * c, pi_model * m, int il, int na) {
    const bool falcon = m->hp.arch == PI_ARCH_FALCON;
    Tensor & up = m->L(il, PI_T_FFN_UP); Tensor & gate = m->L(il, PI_T_FFN_GATE);
    const bool q4 = up.type == PI_TYPE_Q4_0;
    const int d = c->d;
    float * hval = c->hval.data();
    const size_t rb = q4 ? (size_t)(d / 32) * 18 : (size_t)d * 2;
    const unsigned char * wu = (const unsigned char *)up.host;
    const unsigned char * wg = falcon ? nullptr : (const unsigned char *)gate.host;
    const BlockQ8 * xq = c->xq8_pin;
    const uint16_t * x16 = c->x16_pin;
    c->pool->run([&](int t, int nt) {
        for (int k = t; k < na; k += nt) {
            const int j = c->act[k];
            if (k + nt < na) { prefetch_bytes(wu + rb * c->act[k + nt], rb); if (wg) prefetch_bytes(wg + rb * c->act[k + nt], rb); }
            float u, g = 0.f;
            if (q4) {
                u = dot_q4_q8(d, (const BlockQ4 *)(wu + rb * j), xq);
                if (wg) g = dot_q4_q8(d, (const BlockQ4 *)(wg + rb * j), xq);
            } else {
                u = dot_f16(d, (const uint16_t *)(wu + rb * j), x16);
                if (wg) g = dot_f16(d, (const uint16_t *)(wg + rb * j), x16);
            }
            hval[k] = wg ? (g > 0.f ? g : 0.f) * u : (u > 0.f ? u : 0.f);
        }
    });
}

// the listed neurons' share of the down projection into out[d]; threads split the output columns in blocks of 32, so no two threads
// add into the same element.  Q4_0: h goes through the Q8_0 blocks of the completed vector hfull (only the blocks that hold a listed
// neuron are quantised; ggml.c:14465-14618); F16: h rounded to fp16 (ggml.c:14420-14431).
void host_down(ColdPath * c, pi_model * m, int il, int na, const float * hfull, float * out) {
    Tensor & down = m->L(il, PI_T_FFN_DOWN_T);
    const bool q4 = down.type == PI_TYPE_Q4_0;
    const int d = c->d;
    const size_t rb = q4 ? (size_t)(d / 32) * 18 : (size_t)d * 2;
    const unsigned char * wd = (const unsigned char *)down.host;
    const float * hval = c->hval.data();
    if (q4) {
        for (int k = 0, last = -1; k < na; ++k) {               // act is ascending
            const int b = c->act[k] / 32;
            if (b != last) { quantize_q8(hfull + b * 32, c->hq8.data() + b, 32); last = b; }
        }
    }
    const int n_units = d / 32;
    if (q4) {
        // rows whose h rounds to 0 add nothing (skipped, as before); each thread takes a band of column blocks over all rows
        c->dn_rows.clear(); c->dn_a.clear(); c->dn_sc.clear();
        const std::vector<int> & rows_of = c->act;
        for (size_t k = 0; k < rows_of.size(); ++k) {
            const int j = rows_of[k];
            const BlockQ8 & hb = c->hq8[j / 32];
            if (hb.qs[j % 32] == 0) continue;
            c->dn_rows.push_back((const BlockQ4 *)(wd + rb * j)); c->dn_a.push_back(hb.qs[j % 32]); c->dn_sc.push_back(h2f(hb.d));
        }
        const int nr = (int)c->dn_rows.size();
        c->pool->run([&](int t, int nt) {
            const int u0 = (int)((long long)n_units * t / nt), u1 = (int)((long long)n_units * (t + 1) / nt);
            for (int k = 0; k < nr; ++k) prefetch_bytes((const unsigned char *)(c->dn_rows[k] + u0), (size_t)(u1 - u0) * 18);
            axpy_q4_rows(c->dn_rows.data(), c->dn_a.data(), c->dn_sc.data(), nr, u0, u1, out);
        });
        return;
    }
    c->pool->run([&](int t, int nt) {
        const int u0 = (int)((long long)n_units * t / nt), u1 = (int)((long long)n_units * (t + 1) / nt);
        const int c0 = u0 * 32, c1 = u1 * 32;
        for (int i = c0; i < c1; ++i) out[i] = 0.f;
        for (int k = 0; k < na; ++k) {
            const int j = c->act[k];
            if (k + 2 < na) prefetch_bytes(wd + rb * c->act[k + 2] + (q4 ? (size_t)u0 * 18 : (size_t)c0 * 2), q4 ? (size_t)(u1 - u0) * 18 : (size_t)(c1 - c0) * 2);
            if (q4) {
                const BlockQ8 & hb = c->hq8[j / 32];
                const int a = hb.qs[j % 32];
                if (a == 0) continue;
                axpy_q4_blocks((const BlockQ4 *)(wd + rb * j), u0, u1, a, h2f(hb.d), out);
            } else {
                const uint16_t hb = f2h(hval[k]);
                if (hb == 0) continue;
                const float a = h2f(hb);
                const uint16_t * row = (const uint16_t *)(wd + rb * j);
#ifdef PI_COLD_SIMD
                const __m256 av = _mm256_set1_ps(a);
                for (int i = c0; i < c1; i += 8)
                    _mm256_storeu_ps(out + i, _mm256_fmadd_ps(_mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(row + i))), av, _mm256_loadu_ps(out + i)));
#else
                for (int i = c0; i < c1; ++i) out[i] = fmaf(h2f(row[i]), a, out[i]);
#endif
            }
        }
    });
}
}  // namespace

int cold_stage_inputs(ColdPath * c, int il, pi_model * m, hipStream_t st) {
    (void)il;
    const float * ffn_src = m->hp.arch == PI_ARCH_FALCON ? m->x : m->ffn_inp;
    PI_HIP_TRY(hipMemcpyAsync(c->logits, m->pred_logits, sizeof(float) * c->ff, hipMemcpyDeviceToHost, st));
    PI_HIP_TRY(hipMemcpyAsync(c->src, ffn_src, sizeof(float) * c->d, hipMemcpyDeviceToHost, st));
    PI_HIP_TRY(hipEventRecord(c->ev_in, st));
    return PI_OK;
}

int cold_layer_merge(ColdPath * c, int il, pi_model * m, hipStream_t st) {
    const pi_hparams & hp = m->hp;
    const int d = c->d, ff = c->ff;
    const bool falcon = hp.arch == PI_ARCH_FALCON;
    ColdLayer & cl = c->layers[il];
    Tensor & up = m->L(il, PI_T_FFN_UP); Tensor & gate = m->L(il, PI_T_FFN_GATE); Tensor & down = m->L(il, PI_T_FFN_DOWN_T);
    Tensor & bucket = m->L(il, PI_T_GPU_BUCKET);
    const bool q4 = up.type == PI_TYPE_Q4_0;
    const int n_bucket = (int)bucket.ne0;
    const int32_t * bk = (const int32_t *)bucket.dev;
    int32_t * n_act = m->n_active + il;
    const float thr = hp.sparse_threshold;
    const int p = (c->flip ^= 1);
    auto now = [] { return std::chrono::steady_clock::now(); };
    auto us = [](std::chrono::steady_clock::time_point a, std::chrono::steady_clock::time_point b) { return std::chrono::duration<double, std::micro>(b - a).count(); };
    std::chrono::steady_clock::time_point tp = now();
    if (c->trace && c->n_calls) c->t_between += us(c->t_last_return, tp);
    auto lap = [&](int i) { if (c->trace) { const auto t = now(); c->t_phase[i] += us(tp, t); tp = t; } };

    // 1. the GPU share goes on while the host works: Q4_0 sends its h back (the Q8_0 blocks of h mix hot and cold neurons),
    //    F16 needs nothing from the host and queues its down projection right away
    if (q4) {
        PI_HIP_TRY(hipMemcpyAsync(c->h_gpu, m->h_dense, sizeof(float) * ff, hipMemcpyDeviceToHost, st));
        PI_HIP_TRY(hipEventRecord(c->ev_h, st));
    } else {
        const int rc = pi_k_sparse_axpy(down.type, down.dev, d, n_bucket, m->h_c, nullptr, bk, m->list, n_act, PI_EPI_NONE, nullptr, nullptr, m->x2, m->ws, st);
        if (rc != PI_OK) return rc;
    }
    PI_HIP_TRY(wait_event(c->ev_in));           // predictor logits and the FFN input are on the host
    lap(0);

    // 2. norm of the FFN input (llm_build_norm, llama.cpp:4420-4450), then round to the weights' dot type
    {
        const float * x = c->src;
        double s = 0.0;
        float mean = 0.f;
        if (!falcon) { for (int i = 0; i < d; ++i) s += (double)(x[i] * x[i]); }
        else {
            for (int i = 0; i < d; ++i) s += (double)x[i];
            mean = (float)(s / d); s = 0.0;
            for (int i = 0; i < d; ++i) { const float v = x[i] - mean; s += (double)(v * v); }
        }
        const float scale = 1.0f / sqrtf((float)(s / d) + hp.norm_eps);
        for (int i = 0; i < d; ++i) {
            float v = (x[i] - mean) * scale;
            v = v * cl.norm_w[i];
            if (falcon) v = v + cl.norm_b[i];
            c->xn[i] = v;
        }
        if (q4) quantize_q8(c->xn.data(), c->xq8.data(), d);
        else for (int i = 0; i < d; ++i) c->x16[i] = f2h(c->xn[i]);
    }

    // 3. active cold neurons, then up/gate for them
    c->act.clear();
    for (int j : cl.cold_rows) if (!(c->logits[j] < thr)) c->act.push_back(j);
    const int na = (int)c->act.size();
    lap(1);
    float * hval = c->hval.data();
    const size_t rb = q4 ? (size_t)(d / 32) * 18 : (size_t)d * 2;
    const unsigned char * wu = (const unsigned char *)up.host;
    const unsigned char * wg = falcon ? nullptr : (const unsigned char *)gate.host;
    c->pool->run([&](int t, int nt) {
        for (int k = t; k < na; k += nt) {
            const int j = c->act[k];
            float u, g = 0.f;
            if (q4) {
                u = dot_q4_q8(d, (const BlockQ4 *)(wu + rb * j), c->xq8.data());
                if (wg) g = dot_q4_q8(d, (const BlockQ4 *)(wg + rb * j), c->xq8.data());
            } else {
                u = dot_f16(d, (const uint16_t *)(wu + rb * j), c->x16.data());
                if (wg) g = dot_f16(d, (const uint16_t *)(wg + rb * j), c->x16.data());
            }
            hval[k] = wg ? (g > 0.f ? g : 0.f) * u : (u > 0.f ? u : 0.f);
        }
    });

    lap(2);
    // 4. Q4_0: the Q8_0 scales of h span 32 neighbouring neurons, hot and cold alike, so both sides need the merged vector
    float * hfull = c->h_full[p];
    if (q4) {
        PI_HIP_TRY(wait_event(c->ev_h));
        memcpy(hfull, c->h_gpu, sizeof(float) * ff);        // GPU share's h (zero elsewhere): the supports are disjoint
        for (int k = 0; k < na; ++k) hfull[c->act[k]] = hval[k];
        PI_HIP_TRY(hipMemcpyAsync(m->h_dense, hfull, sizeof(float) * ff, hipMemcpyHostToDevice, st));
        const int rc = pi_k_sparse_axpy(down.type, down.dev, d, n_bucket, m->h_c, m->h_dense, bk, m->list, n_act, PI_EPI_NONE, nullptr, nullptr, m->x2, m->ws, st);
        if (rc != PI_OK) return rc;
        quantize_q8(hfull, c->hq8.data(), ff);
    }

    lap(3);
    // 5. cold share of the down projection, threads split the output columns (blocks of 32 for Q4_0)
    const unsigned char * wd = (const unsigned char *)down.host;
    float * out = c->out[p];
    const int unit = 32, n_units = d / unit;
    c->pool->run([&](int t, int nt) {
        const int u0 = (int)((long long)n_units * t / nt), u1 = (int)((long long)n_units * (t + 1) / nt);
        const int c0 = u0 * unit, c1 = u1 * unit;
        for (int i = c0; i < c1; ++i) out[i] = 0.f;
        for (int k = 0; k < na; ++k) {
            const int j = c->act[k];
            if (q4) {
                const BlockQ8 & hb = c->hq8[j / 32];
                const int a = hb.qs[j % 32];
                if (a == 0) continue;
                const float sc = h2f(hb.d);
                axpy_q4_blocks((const BlockQ4 *)(wd + rb * j), u0, u1, a, sc, out);
            } else {
                const uint16_t hb = f2h(hval[k]);
                if (hb == 0) continue;
                const float a = h2f(hb);
                const uint16_t * row = (const uint16_t *)(wd + rb * j);
#ifdef PI_COLD_SIMD
                const __m256 av = _mm256_set1_ps(a);
                for (int i = c0; i < c1; i += 8)
                    _mm256_storeu_ps(out + i, _mm256_fmadd_ps(_mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(row + i))), av, _mm256_loadu_ps(out + i)));
#else
                for (int i = c0; i < c1; ++i) out[i] = fmaf(h2f(row[i]), a, out[i]);
#endif
            }
        }
    });

    // 6. merge: (cold + hot) + residual(s), in the reference's order (ggml_add(cpu, gpu), then the residual adds).  The kernel
    //    reads the cold share straight from the pinned buffer; that buffer and h_full[p] are written again two layers on, after
    //    the host has waited for an event recorded behind this layer's work, so no wait is needed here.
    lap(4);
    const int rc = merge_shares(m->x2, out, m->x2, falcon ? m->attn_out : m->ffn_inp, falcon ? m->x : nullptr,
                                m->capture ? m->cap_ffn + (size_t)il * d : nullptr, d, st);
    lap(5);
    if (c->trace) { ++c->n_calls; c->n_cold_active += na; c->t_last_return = now(); }
    return rc;
}

int cold_layer_q4(ColdPath * c, int il, pi_model * m, hipStream_t st, bool capture) {
    const pi_hparams & hp = m->hp;
    const int d = c->d, ff = c->ff;
    const bool falcon = hp.arch == PI_ARCH_FALCON;
    ColdLayer & cl = c->layers[il];
    Tensor & up = m->L(il, PI_T_FFN_UP); Tensor & gate = m->L(il, PI_T_FFN_GATE); Tensor & down = m->L(il, PI_T_FFN_DOWN_T);
    Tensor & fc1 = m->L(il, PI_T_FC1); Tensor & fc2 = m->L(il, PI_T_FC2);
    const int r = (int)fc1.ne1;
    const float thr = hp.sparse_threshold;
    const int p = (c->flip ^= 1);
    float * hfull = c->h_full[p];
    float * out = c->out[p];
    auto now = [] { return std::chrono::steady_clock::now(); };
    auto us = [](std::chrono::steady_clock::time_point a, std::chrono::steady_clock::time_point b) { return std::chrono::duration<double, std::micro>(b - a).count(); };
    std::chrono::steady_clock::time_point tp = now();
    if (c->trace && c->n_calls) c->t_between += us(c->t_last_return, tp);
    auto lap = [&](int i) { if (c->trace) { const auto t = now(); c->t_phase[i] += us(tp, t); tp = t; } };

    // 1. the kernel writes what the host needs straight into pinned memory: logits, the Q8_0 blocks of the normalised input,
    //    and h (resident active neurons; zero elsewhere) into the vector the host completes below
    pi_norm fn;
    fn.kind = falcon ? 2 : 1; fn.eps = hp.norm_eps;
    fn.w = (const float *)m->L(il, falcon ? PI_T_ATTN_NORM : PI_T_FFN_NORM).dev;
    fn.b = falcon ? (const float *)m->L(il, PI_T_ATTN_NORM_B).dev : nullptr;
    const float * ffn_src = falcon ? m->x : m->ffn_inp;
    int rc = pi_k_pred_upgate_q4(fc2.dev, ff, r, m->hidden, thr, up.dev, falcon ? nullptr : gate.dev, d, ffn_src, &fn,
                                 m->hot_words[il], m->hot_prefix[il], c->logits, hfull, c->xq8_pin, m->ws, st);
    if (rc != PI_OK) return rc;
    PI_HIP_TRY(hipEventRecord(c->ev_in, st));
    if (capture) PI_HIP_TRY(hipMemcpyAsync(m->cap_logits + (size_t)il * ff, c->logits, sizeof(float) * ff, hipMemcpyHostToDevice, st));
    PI_HIP_TRY(wait_event(c->ev_in));
    lap(0);

    // 2. active cold neurons, their up/gate rows against the same Q8_0 input
    const int na = list_active_cold(c, cl, thr);
    lap(1);
    host_upgate(c, m, il, na);
    for (int k = 0; k < na; ++k) hfull[c->act[k]] = c->hval[k];
    lap(2);

    // 3. the GPU's down projection reads the completed vector from the pinned buffer; the host quantises it the same way
    rc = pi_k_axpy_q4_partials(down.dev, d, ff, hfull, m->hot_words[il], m->hot_prefix[il], m->ws, st);
    if (rc != PI_OK) return rc;
    lap(3);
    host_down(c, m, il, na, hfull, out);
    lap(4);

    // 4. (cold + hot) + residual(s), the reference's order (ggml_add(cpu, gpu), then the residual adds): folded into the
    //    reduction of the GPU partials when there is a single residual and nothing to keep
    int32_t * n_act = m->n_active + il;
    if (!falcon && !capture) {
        rc = pi_k_axpy_q4_reduce(ff, d, PI_EPI_ADD2, out, m->ffn_inp, m->x2, n_act, m->ws, st);
    } else {
        rc = pi_k_axpy_q4_reduce(ff, d, PI_EPI_NONE, nullptr, nullptr, m->x2, n_act, m->ws, st);
        if (rc == PI_OK)
            rc = merge_shares(m->x2, out, m->x2, falcon ? m->attn_out : m->ffn_inp, falcon ? m->x : nullptr,
                              capture ? m->cap_ffn + (size_t)il * d : nullptr, d, st);
    }
    lap(5);
    if (c->trace) { ++c->n_calls; c->n_cold_active += na; c->t_last_return = now(); }
    return rc;
}

int cold_layer_f16(ColdPath * c, int il, pi_model * m, hipStream_t st, bool capture) {
    const pi_hparams & hp = m->hp;
    const int d = c->d, ff = c->ff;
    const bool falcon = hp.arch == PI_ARCH_FALCON;
    ColdLayer & cl = c->layers[il];
    Tensor & up = m->L(il, PI_T_FFN_UP); Tensor & gate = m->L(il, PI_T_FFN_GATE); Tensor & down = m->L(il, PI_T_FFN_DOWN_T);
    Tensor & fc1 = m->L(il, PI_T_FC1); Tensor & fc2 = m->L(il, PI_T_FC2);
    const int r = (int)fc1.ne1;
    const float thr = hp.sparse_threshold;
    const int p = (c->flip ^= 1);
    float * out = c->out[p];
    auto now = [] { return std::chrono::steady_clock::now(); };
    auto us = [](std::chrono::steady_clock::time_point a, std::chrono::steady_clock::time_point b) { return std::chrono::duration<double, std::micro>(b - a).count(); };
    std::chrono::steady_clock::time_point tp = now();
    if (c->trace && c->n_calls) c->t_between += us(c->t_last_return, tp);
    auto lap = [&](int i) { if (c->trace) { const auto t = now(); c->t_phase[i] += us(tp, t); tp = t; } };

    // 1. the resident share in one launch; logits and the fp16 input land in pinned memory for the host share
    pi_norm fn;
    fn.kind = falcon ? 2 : 1; fn.eps = hp.norm_eps;
    fn.w = (const float *)m->L(il, falcon ? PI_T_ATTN_NORM : PI_T_FFN_NORM).dev;
    fn.b = falcon ? (const float *)m->L(il, PI_T_ATTN_NORM_B).dev : nullptr;
    const float * ffn_src = falcon ? m->x : m->ffn_inp;
    int rc = pi_k_sparse_ffn_partials_hot(fc2.dev, ff, r, m->hidden, thr, up.dev, falcon ? nullptr : gate.dev, down.dev, d, ffn_src, &fn,
                                          m->hot_words[il], m->hot_prefix[il], c->logits, nullptr, c->x16_pin, m->ws, st);
    if (rc != PI_OK) return rc;
    PI_HIP_TRY(hipEventRecord(c->ev_in, st));
    if (capture) PI_HIP_TRY(hipMemcpyAsync(m->cap_logits + (size_t)il * ff, c->logits, sizeof(float) * ff, hipMemcpyHostToDevice, st));
    PI_HIP_TRY(wait_event(c->ev_in));
    lap(0);

    // 2. active cold neurons: up/gate dots on the fp16 input (ggml.c:14030-14282), h rounded to fp16 for the axpy (ggml.c:14420-14431)
    const int na = list_active_cold(c, cl, thr);
    lap(1);
    host_upgate(c, m, il, na);
    lap(2);
    lap(3);
    host_down(c, m, il, na, nullptr, out);
    lap(4);

    // 3. (cold + hot) + residual(s), folded into the reduction of the GPU partials when there is one residual and nothing to keep
    int32_t * n_act = m->n_active + il;
    if (!falcon && !capture) {
        rc = pi_k_sparse_ffn_reduce_hot(ff, d, PI_EPI_ADD2, out, m->ffn_inp, m->x2, n_act, m->ws, st);
    } else {
        rc = pi_k_sparse_ffn_reduce_hot(ff, d, PI_EPI_NONE, nullptr, nullptr, m->x2, n_act, m->ws, st);
        if (rc == PI_OK)
            rc = merge_shares(m->x2, out, m->x2, falcon ? m->attn_out : m->ffn_inp, falcon ? m->x : nullptr,
                              capture ? m->cap_ffn + (size_t)il * d : nullptr, d, st);
    }
    lap(5);
    if (c->trace) { ++c->n_calls; c->n_cold_active += na; c->t_last_return = now(); }
    return rc;
}


// ---- Q4_0 hybrid layers without the launching thread in the loop -------------------------------------------------------------
namespace {

inline void relax() {
#ifdef PI_COLD_SIMD
    _mm_pause();
#else
    std::this_thread::yield();
#endif
}

// the host share of one posted layer: what cold_layer_q4 does between its launches, started by the device's signal
void serve_q4(ColdPath * c, int il, uint32_t seq) {
    pi_model * m = c->model;
    const pi_hparams & hp = m->hp;
    const int d = c->d;
    const bool falcon = hp.arch == PI_ARCH_FALCON;
    ColdLayer & cl = c->layers[il];
    Tensor & up = m->L(il, PI_T_FFN_UP); Tensor & gate = m->L(il, PI_T_FFN_GATE); Tensor & down = m->L(il, PI_T_FFN_DOWN_T);
    const float thr = hp.sparse_threshold;
    float * hfull = c->h_async[il];
    float * out = c->out[0];
    auto now = [] { return std::chrono::steady_clock::now(); };
    auto us = [](std::chrono::steady_clock::time_point a, std::chrono::steady_clock::time_point b) { return std::chrono::duration<double, std::micro>(b - a).count(); };
    std::chrono::steady_clock::time_point tp = now();
    if (c->trace && c->n_calls) c->t_between += us(c->t_last_return, tp);
    auto lap = [&](int i) { if (c->trace) { const auto t = now(); c->t_phase[i] += us(tp, t); tp = t; } };

    // 1. logits, the Q8_0 blocks of the normalised input and the resident neurons' h are in pinned memory once the device says so
    {
        const auto t0 = now();
        for (int it = 0; (int32_t)(__atomic_load_n(&c->flags[0], __ATOMIC_ACQUIRE) - seq) < 0; ++it) {
            relax();
            if ((it & 1023) == 1023 && (c->stop.load() || now() - t0 > std::chrono::seconds(20))) {
                // the device never got here (a failed launch, a caller that gave up): release the stream's waits and stop serving
                c->failed.store(true);
                __atomic_store_n(&c->flags[48], 1u, __ATOMIC_RELEASE);
                return;
            }
        }
    }
    lap(0);

    // 2. active cold neurons, their up/gate rows against the same Q8_0 input
    for (int j : c->prev_act[il]) hfull[j] = 0.f;        // this side's entries of the shared vector: the device never writes them
    c->prev_act[il].clear();
    const int na = list_active_cold_words(c, cl);
    lap(1);
    host_upgate(c, m, il, na);
    const float * hval = c->hval.data();
    for (int k = 0; k < na; ++k) hfull[c->act[k]] = hval[k];
    c->prev_act[il].assign(c->act.begin(), c->act.end());
    __atomic_store_n(&c->flags[16], seq, __ATOMIC_RELEASE);          // the device's down projection may read the completed vector
    lap(2);
    // the Q8_0 scales of h span resident and non-resident neurons: the resident ones' h must have arrived
    const auto t0 = now();
    for (int it = 0; (int32_t)(__atomic_load_n(&c->flags[8], __ATOMIC_ACQUIRE) - seq) < 0; ++it) {
        relax();
        if ((it & 1023) == 1023 && (c->stop.load() || now() - t0 > std::chrono::seconds(20))) {
            c->failed.store(true);
            __atomic_store_n(&c->flags[48], 1u, __ATOMIC_RELEASE);
            return;
        }
    }

    // 3. the host quantises h the same way and adds its neurons' down rows
    lap(3);
    host_down(c, m, il, na, hfull, out);
    __atomic_store_n(&c->flags[32], seq, __ATOMIC_RELEASE);          // the reduction may add the host share
    lap(4);
    if (c->trace) { ++c->n_calls; c->n_cold_active += na; c->t_last_return = now(); }
}

// the same for an F16 layer: the resident share needs nothing from the host, so there is one hand-over in each direction
void serve_f16(ColdPath * c, int il, uint32_t seq) {
    pi_model * m = c->model;
    const pi_hparams & hp = m->hp;
    const int d = c->d;
    const bool falcon = hp.arch == PI_ARCH_FALCON;
    ColdLayer & cl = c->layers[il];
    Tensor & up = m->L(il, PI_T_FFN_UP); Tensor & gate = m->L(il, PI_T_FFN_GATE); Tensor & down = m->L(il, PI_T_FFN_DOWN_T);
    float * out = c->out[0];
    auto now = [] { return std::chrono::steady_clock::now(); };
    auto us = [](std::chrono::steady_clock::time_point a, std::chrono::steady_clock::time_point b) { return std::chrono::duration<double, std::micro>(b - a).count(); };
    std::chrono::steady_clock::time_point tp = now();
    if (c->trace && c->n_calls) c->t_between += us(c->t_last_return, tp);
    auto lap = [&](int i) { if (c->trace) { const auto t = now(); c->t_phase[i] += us(tp, t); tp = t; } };
    {
        const auto t0 = now();
        for (int it = 0; (int32_t)(__atomic_load_n(&c->flags[0], __ATOMIC_ACQUIRE) - seq) < 0; ++it) {
            relax();
            if ((it & 1023) == 1023 && (c->stop.load() || now() - t0 > std::chrono::seconds(20))) {
                c->failed.store(true);
                __atomic_store_n(&c->flags[48], 1u, __ATOMIC_RELEASE);
                return;
            }
        }
    }
    lap(0);
    const int na = list_active_cold_words(c, cl);
    lap(1);
    host_upgate(c, m, il, na);
    lap(2);
    lap(3);
    host_down(c, m, il, na, nullptr, out);
    __atomic_store_n(&c->flags[32], seq, __ATOMIC_RELEASE);          // the reduction may add the host share
    lap(4);
    if (c->trace) { ++c->n_calls; c->n_cold_active += na; c->t_last_return = now(); }
}

void service_loop(ColdPath * c) {
    uint64_t next = 0;
    uint32_t seq = 0;
    for (;;) {
        const auto t0 = std::chrono::steady_clock::now();
        for (int it = 0; c->posted.load(std::memory_order_acquire) == next; ++it) {
            if (c->stop.load()) return;
            relax();
            if ((it & 255) == 255 && std::chrono::steady_clock::now() - t0 > std::chrono::microseconds(2000)) {
                std::unique_lock<std::mutex> g(c->mu);
                // the producer stores `posted` and then reads `service_asleep`; this side stores `service_asleep` and then reads
                // `posted`: both pairs are sequentially consistent, so at least one side sees the other's store.  The bounded wait is
                // a second line of defence: a wake-up that is lost all the same costs a few milliseconds, not the 5 s of the device's wait.
                c->service_asleep.store(1, std::memory_order_seq_cst);
                while (c->posted.load(std::memory_order_seq_cst) == next && !c->stop.load())
                    c->cv.wait_for(g, std::chrono::milliseconds(2));
                c->service_asleep.store(0, std::memory_order_seq_cst);
            }
        }
        if (c->stop.load()) return;
        const int il = c->ring[next % c->ring.size()];
        ++seq;
        if (!c->failed.load()) {
            if (c->model->L(il, PI_T_FFN_UP).type == PI_TYPE_Q4_0) serve_q4(c, il, seq);
            else serve_f16(c, il, seq);
        }
        c->served.store(++next, std::memory_order_release);
    }
}

}  // namespace

bool cold_async(const ColdPath * c) { return c && c->async; }
bool cold_layer_async(const ColdPath * c, int il) {
    if (!c || !c->async) return false;
    for (int a : c->async_layers) if (a == il) return true;
    return false;
}
bool cold_every_layer_async(const ColdPath * c) {
    if (!c || !c->async) return false;
    size_t hybrid = 0;
    for (int il = 0; il < c->model->hp.n_layer; ++il) hybrid += c->model->L(il, PI_T_GPU_BUCKET).dev != nullptr;
    return hybrid == c->async_layers.size();
}

// one token's hybrid layers, in the order the stream will reach them
int cold_post_token(ColdPath * c) {
    if (c->failed.load()) return fail(PI_E_STATE, "cold path: the host share stopped after a hand-over timed out");
    for (int il : c->async_layers) {
        const uint64_t p = c->posted.load(std::memory_order_relaxed);
        while (p - c->served.load(std::memory_order_acquire) >= c->ring.size()) relax();
        c->ring[p % c->ring.size()] = il;
        c->posted.store(p + 1, std::memory_order_seq_cst);
    }
    if (c->service_asleep.load(std::memory_order_seq_cst)) { { std::lock_guard<std::mutex> g(c->mu); } c->cv.notify_all(); }
    return PI_OK;
}

// the stream has been synchronised: every posted layer has been answered, or something gave up
int cold_drain(ColdPath * c) {
    if (!c->async) return PI_OK;
    const auto t0 = std::chrono::steady_clock::now();
    while (c->served.load(std::memory_order_acquire) != c->posted.load() && !c->failed.load()) {
        relax();
        if (std::chrono::steady_clock::now() - t0 > std::chrono::seconds(30)) { c->failed.store(true); break; }
    }
    uint32_t status = 0;
    if (pi_memcpy_d2h(&status, c->d_status, 4) != PI_OK) return PI_E_HIP;
    if (status != 0 || c->failed.load()) return fail(PI_E_STATE, "cold path: a hand-over between the stream and the host threads timed out");
    return PI_OK;
}

// the device half of such a layer, queued in one go: fc2 + mask + resident up/gate -> signal -> (wait for h) down projection ->
// (wait for the host share) reduction with the merge folded in
int cold_layer_q4_queue(ColdPath * c, int il, pi_model * m, hipStream_t st) {
    const pi_hparams & hp = m->hp;
    const int d = c->d, ff = c->ff;
    const bool falcon = hp.arch == PI_ARCH_FALCON;
    Tensor & up = m->L(il, PI_T_FFN_UP); Tensor & gate = m->L(il, PI_T_FFN_GATE); Tensor & down = m->L(il, PI_T_FFN_DOWN_T);
    Tensor & fc1 = m->L(il, PI_T_FC1); Tensor & fc2 = m->L(il, PI_T_FC2);
    const int r = (int)fc1.ne1;
    float * hfull = c->h_async[il];
    float * out = c->out[0];
    const double limit = 5.0;
    pi_norm fn;
    fn.kind = falcon ? 2 : 1; fn.eps = hp.norm_eps;
    fn.w = (const float *)m->L(il, falcon ? PI_T_ATTN_NORM : PI_T_FFN_NORM).dev;
    fn.b = falcon ? (const float *)m->L(il, PI_T_ATTN_NORM_B).dev : nullptr;
    const float * ffn_src = falcon ? m->x : m->ffn_inp;
    PI_TRY(pi_k_pred_q4_logits(fc2.dev, ff, r, m->hidden, hp.sparse_threshold, d, ffn_src, &fn, nullptr, m->pred_logits, c->xq8_pin, c->words_pin, m->ws, st));
    // the hand-over starts in the first lane of the next launch, and the second signal travels with the wait behind it
    PI_TRY(pi_k_upgate_q4_hot_rows(ff, hp.sparse_threshold, up.dev, falcon ? nullptr : gate.dev, d, ffn_src, &fn, m->hot_words[il], m->hot_prefix[il],
                                   m->pred_logits, hfull, c->d_seq, c->flags, m->ws, st));
    PI_TRY(pi_k_host_signal_wait(c->d_seq, c->flags, 8, 16, c->d_status, limit, st));
    PI_TRY(pi_k_axpy_q4_partials(down.dev, d, ff, hfull, m->hot_words[il], m->hot_prefix[il], m->ws, st));
    PI_TRY(pi_k_host_wait(c->d_seq, c->flags, 32, c->d_status, limit, st));
    int32_t * n_act = m->n_active + il;
    if (!falcon) return pi_k_axpy_q4_reduce(ff, d, PI_EPI_ADD2, out, m->ffn_inp, m->x2, n_act, m->ws, st);
    PI_TRY(pi_k_axpy_q4_reduce(ff, d, PI_EPI_NONE, nullptr, nullptr, m->x2, n_act, m->ws, st));
    return merge_shares(m->x2, out, m->x2, m->attn_out, m->x, nullptr, d, st);
}

// the device half of an F16 hybrid layer: predictor -> signal -> resident rows (gate / up / down partial vectors) -> (wait for the host
// share) reduction with the merge folded in
int cold_layer_f16_queue(ColdPath * c, int il, pi_model * m, hipStream_t st) {
    const pi_hparams & hp = m->hp;
    const int d = c->d, ff = c->ff;
    const bool falcon = hp.arch == PI_ARCH_FALCON;
    Tensor & up = m->L(il, PI_T_FFN_UP); Tensor & gate = m->L(il, PI_T_FFN_GATE); Tensor & down = m->L(il, PI_T_FFN_DOWN_T);
    Tensor & fc1 = m->L(il, PI_T_FC1); Tensor & fc2 = m->L(il, PI_T_FC2);
    const int r = (int)fc1.ne1;
    float * out = c->out[0];
    const double limit = 5.0;
    pi_norm fn;
    fn.kind = falcon ? 2 : 1; fn.eps = hp.norm_eps;
    fn.w = (const float *)m->L(il, falcon ? PI_T_ATTN_NORM : PI_T_FFN_NORM).dev;
    fn.b = falcon ? (const float *)m->L(il, PI_T_ATTN_NORM_B).dev : nullptr;
    const float * ffn_src = falcon ? m->x : m->ffn_inp;
    PI_TRY(pi_k_sparse_ffn_logits_hot(fc2.dev, ff, r, m->hidden, hp.sparse_threshold, d, ffn_src, &fn, m->hot_words[il], m->hot_prefix[il],
                                      nullptr, m->pred_logits, c->x16_pin, c->words_pin, m->ws, st));
    PI_TRY(pi_k_sparse_ffn_rows_hot(ff, hp.sparse_threshold, up.dev, falcon ? nullptr : gate.dev, down.dev, d, ffn_src, &fn, m->hot_words[il], m->hot_prefix[il],
                                    m->pred_logits, nullptr, c->d_seq, c->flags, m->ws, st));             // its first lane starts the hand-over
    PI_TRY(pi_k_host_wait(c->d_seq, c->flags, 32, c->d_status, limit, st));
    int32_t * n_act = m->n_active + il;
    if (!falcon) return pi_k_sparse_ffn_reduce_hot(ff, d, PI_EPI_ADD2, out, m->ffn_inp, m->x2, n_act, m->ws, st);
    PI_TRY(pi_k_sparse_ffn_reduce_hot(ff, d, PI_EPI_NONE, nullptr, nullptr, m->x2, n_act, m->ws, st));
    return merge_shares(m->x2, out, m->x2, m->attn_out, m->x, nullptr, d, st);
}

}  // namespace pi
