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
#include <stdlib.h>
#include <string.h>

#include <atomic>
#include <condition_variable>
#include <functional>
#include <mutex>
#include <thread>
#include <vector>

#if defined(__AVX2__) && defined(__F16C__) && defined(__FMA__)
#include <immintrin.h>
#define PI_COLD_SIMD 1
#endif

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

float dot_q4_q8(int n, const BlockQ4 * w, const BlockQ8 * x) {
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
}

// x86 quantize_row_q8_0 semantics (ggml-quants.c:702-760): d = amax/127 stored as fp16, q = rint(x * 127/amax)
void quantize_q8(const float * x, BlockQ8 * y, int n) {
    for (int b = 0; b < n / 32; ++b) {
        float amax = 0.f;
        for (int j = 0; j < 32; ++j) amax = fmaxf(amax, fabsf(x[b * 32 + j]));
        const float d = amax / 127.f, id = amax != 0.f ? 127.f / amax : 0.f;
        y[b].d = f2h(d);
        for (int j = 0; j < 32; ++j) y[b].qs[j] = (int8_t)(int)rintf(x[b * 32 + j] * id);
    }
}

class Pool {
  public:
    explicit Pool(int n) : n_(n) {
        for (int i = 1; i < n_; ++i) threads_.emplace_back([this, i] { loop(i); });
    }
    ~Pool() {
        { std::lock_guard<std::mutex> g(mu_); stop_ = true; ++gen_; }
        cv_.notify_all();
        for (auto & t : threads_) t.join();
    }
    int size() const { return n_; }
    void run(const std::function<void(int, int)> & fn) {
        { std::lock_guard<std::mutex> g(mu_); fn_ = &fn; pending_ = n_ - 1; ++gen_; }
        cv_.notify_all();
        fn(0, n_);
        std::unique_lock<std::mutex> g(mu_);
        done_.wait(g, [this] { return pending_ == 0; });
        fn_ = nullptr;
    }

  private:
    void loop(int id) {
        uint64_t seen = 0;
        for (;;) {
            const std::function<void(int, int)> * fn;
            {
                std::unique_lock<std::mutex> g(mu_);
                cv_.wait(g, [&] { return gen_ != seen; });
                seen = gen_;
                if (stop_) return;
                fn = fn_;
            }
            (*fn)(id, n_);
            { std::lock_guard<std::mutex> g(mu_); if (--pending_ == 0) done_.notify_one(); }
        }
    }
    int n_;
    std::vector<std::thread> threads_;
    std::mutex mu_;
    std::condition_variable cv_, done_;
    const std::function<void(int, int)> * fn_ = nullptr;
    int pending_ = 0;
    uint64_t gen_ = 0;
    bool stop_ = false;
};

}  // namespace

struct ColdLayer {
    std::vector<float> norm_w, norm_b;          // host copies of the FFN-input norm
    std::vector<int32_t> cold_rows;             // neurons with gpu_idx == 0, ascending
};

struct ColdPath {
    Pool * pool = nullptr;
    std::vector<ColdLayer> layers;
    // pinned staging
    float * logits = nullptr, * src = nullptr, * h_gpu = nullptr, * h_full = nullptr, * out = nullptr;
    std::vector<float> xn;
    std::vector<uint16_t> x16;
    std::vector<BlockQ8> xq8, hq8;
    std::vector<int32_t> act;                   // active cold neurons of the current token
    int d = 0, ff = 0;
};

ColdPath * cold_create(pi_model * m) {
    ColdPath * c = new ColdPath();
    const pi_hparams & hp = m->hp;
    c->d = hp.n_embd; c->ff = hp.n_ff;
    int nt = (int)std::thread::hardware_concurrency();
    if (nt > 16) nt = 16;
    if (const char * e = getenv("PI_COLD_THREADS")) { const int v = atoi(e); if (v > 0) nt = v; }
    if (nt < 1) nt = 1;
    c->pool = new Pool(nt);
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
        for (int j = 0; j < c->ff; ++j) if (gid[j] != 1) cl.cold_rows.push_back(j);
    }
    auto pin = [](size_t n) { void * p = nullptr; return hipHostMalloc(&p, n * sizeof(float), hipHostMallocDefault) == hipSuccess ? (float *)p : nullptr; };
    c->logits = pin(c->ff); c->src = pin(c->d); c->h_gpu = pin(c->ff); c->h_full = pin(c->ff); c->out = pin(c->d);
    if (!c->logits || !c->src || !c->h_gpu || !c->h_full || !c->out) { set_error("cold path: pinned host allocation failed"); cold_destroy(c); return nullptr; }
    c->xn.resize(c->d); c->x16.resize(c->d); c->xq8.resize(c->d / 32 + 1); c->hq8.resize(c->ff / 32 + 1);
    c->act.reserve(c->ff);
    return c;
}

void cold_destroy(ColdPath * c) {
    if (!c) return;
    delete c->pool;
    for (float * p : {c->logits, c->src, c->h_gpu, c->h_full, c->out}) if (p) (void)hipHostFree(p);
    delete c;
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
    const float * ffn_src = falcon ? m->x : m->ffn_inp;
    const float thr = hp.sparse_threshold;

    // 1. what the host needs from the device: predictor logits and the FFN block's input vector
    PI_HIP_TRY(hipMemcpyAsync(c->logits, m->pred_logits, sizeof(float) * ff, hipMemcpyDeviceToHost, st));
    PI_HIP_TRY(hipMemcpyAsync(c->src, ffn_src, sizeof(float) * d, hipMemcpyDeviceToHost, st));
    if (q4) PI_HIP_TRY(hipMemcpyAsync(c->h_gpu, m->h_dense, sizeof(float) * ff, hipMemcpyDeviceToHost, st));   // after the GPU share's up/gate
    if (!q4) {
        // F16: the GPU share needs nothing from the host; queue its down projection now so it overlaps the CPU work
        const int rc = pi_k_sparse_axpy(down.type, down.dev, d, n_bucket, m->h_c, nullptr, bk, m->list, n_act, PI_EPI_NONE, nullptr, nullptr, m->x2, m->ws, st);
        if (rc != PI_OK) return rc;
    }
    PI_HIP_TRY(hipStreamSynchronize(st));

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
    float * hfull = c->h_full;
    if (q4) memcpy(hfull, c->h_gpu, sizeof(float) * ff);        // GPU share's h (zero elsewhere): the supports are disjoint
    else memset(hfull, 0, sizeof(float) * ff);
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
            hfull[j] = wg ? (g > 0.f ? g : 0.f) * u : (u > 0.f ? u : 0.f);
        }
    });

    // 4. Q4_0: the Q8_0 scales of h span 32 neighbouring neurons, hot and cold alike, so both sides need the merged vector
    if (q4) {
        PI_HIP_TRY(hipMemcpyAsync(m->h_dense, hfull, sizeof(float) * ff, hipMemcpyHostToDevice, st));
        const int rc = pi_k_sparse_axpy(down.type, down.dev, d, n_bucket, m->h_c, m->h_dense, bk, m->list, n_act, PI_EPI_NONE, nullptr, nullptr, m->x2, m->ws, st);
        if (rc != PI_OK) return rc;
        quantize_q8(hfull, c->hq8.data(), ff);
    }

    // 5. cold share of the down projection, threads split the output columns (blocks of 32 for Q4_0)
    const unsigned char * wd = (const unsigned char *)down.host;
    float * out = c->out;
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
                const BlockQ4 * row = (const BlockQ4 *)(wd + rb * j);
                for (int b = u0; b < u1; ++b) {
                    const float dd = h2f(row[b].d) * sc;
                    float * o = out + b * 32;
                    for (int q = 0; q < 16; ++q) {
                        o[q]      = o[q]      + (float)(((int)(row[b].qs[q] & 0x0F) - 8) * a) * dd;
                        o[q + 16] = o[q + 16] + (float)(((int)(row[b].qs[q] >> 4) - 8) * a) * dd;
                    }
                }
            } else {
                const uint16_t hb = f2h(hfull[j]);
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

    // 6. merge: (cold + hot) + residual(s), in the reference's order (ggml_add(cpu, gpu), then the residual adds)
    PI_HIP_TRY(hipMemcpyAsync(m->cold_out, out, sizeof(float) * d, hipMemcpyHostToDevice, st));
    int rc = add_vec(m->cold_out, m->x2, d, st);                 // cold_out = cold + hot
    if (rc != PI_OK) return rc;
    PI_HIP_TRY(hipMemcpyAsync(m->x2, m->cold_out, sizeof(float) * d, hipMemcpyDeviceToDevice, st));
    if (m->capture) PI_HIP_TRY(hipMemcpyAsync(m->cap_ffn + (size_t)il * d, m->cold_out, sizeof(float) * d, hipMemcpyDeviceToDevice, st));
    rc = add_vec(m->x2, falcon ? m->attn_out : m->ffn_inp, d, st);
    if (rc != PI_OK) return rc;
    if (falcon) { rc = add_vec(m->x2, m->x, d, st); if (rc != PI_OK) return rc; }
    // the pinned buffers are reused by the next layer: wait for the upload to be consumed
    PI_HIP_TRY(hipStreamSynchronize(st));
    return PI_OK;
}

}  // namespace pi
