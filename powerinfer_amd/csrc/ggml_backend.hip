// The reference's accelerator-backend entry points (ggml-cuda.h:21-60) implemented on this library's kernels, so
// that a host built against the reference's ggml.h / ggml-cuda.h links to libpowerinfer_hip.so instead of
// ggml-cuda.cu.  Per-node dispatch as ggml_cuda_compute_forward does it (ggml-cuda.cu:9218-9346); the hot
// operators (MUL_MAT at one token, MUL_MAT_SPARSE, AXPY) go to the tuned launchers, everything else to small
// generic kernels.  Device addresses live in tensor->extra.  Errors are fatal, as in the reference
// (CUDA_CHECK -> exit(1), ggml-cuda.cu:192-229).
#include "runtime.hpp"
#include "device_utils.hpp"
#include "../../include/ggml_backend_abi.h"
#include "../../include/powerinfer_hip.h"

#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <mutex>
#include <vector>

namespace {

struct Extra {
    void * data_device[GGML_CUDA_MAX_DEVICES];     // [0] is the only one used (single GPU)
    bool   owned;
    bool   outside_scratch;                        // address computed from a host offset that does not lie in the scratch: never dereferenced
};

bool   g_loaded = false;
float  g_threshold = 0.0f;
char * g_scratch = nullptr;
size_t g_scratch_size = 0, g_scratch_offset = 0;
pi_workspace * g_ws = nullptr;
int    g_ws_ff = 0, g_ws_d = 0;
std::mutex g_mu;
// Per-evaluation extras come from a ring, as in the reference (ggml-cuda.cu:9030-9044): a host rebuilds its graph for every
// token and never hands these back, so they must not be heap objects of their own.
constexpr size_t kMaxNodes = 8192;
Extra * g_ring = nullptr;
size_t  g_ring_next = 0;
Extra * ring_extra(void * p) {
    if (!g_ring) g_ring = new Extra[kMaxNodes];
    Extra * e = &g_ring[g_ring_next];
    g_ring_next = (g_ring_next + 1) % kMaxNodes;
    memset(e, 0, sizeof *e);
    e->data_device[0] = p;
    return e;
}
bool is_ring(const Extra * e) { return g_ring && e >= g_ring && e < g_ring + kMaxNodes; }

[[noreturn]] void die(const char * what) {
    fprintf(stderr, "powerinfer-hip backend: %s: %s\n", what, pi_last_error());
    exit(1);
}
#define BK_HIP(expr) do { hipError_t _e = (expr); if (_e != hipSuccess) { fprintf(stderr, "powerinfer-hip backend: %s: %s\n", #expr, hipGetErrorString(_e)); exit(1); } } while (0)
#define BK_PI(expr) do { if ((expr) != PI_OK) die(#expr); } while (0)

int blck(int type) { return type == GGML_TYPE_Q4_0 ? 32 : 1; }
size_t tsize(int type) {
    switch (type) {
        case GGML_TYPE_F32: case GGML_TYPE_I32: return 4;
        case GGML_TYPE_F16: case GGML_TYPE_I16: return 2;
        case GGML_TYPE_I8: return 1;
        case GGML_TYPE_Q4_0: return 18;
        default: return 0;
    }
}
size_t row_size(const ggml_tensor * t) { return tsize(t->type) * (size_t)(t->ne[0] / blck(t->type)); }
int64_t nrows(const ggml_tensor * t) { return t->ne[1] * t->ne[2] * t->ne[3]; }
int64_t nelem(const ggml_tensor * t) { return t->ne[0] * nrows(t); }
size_t nbytes(const ggml_tensor * t) {                    // ggml_nbytes (ggml.c:1956-1973): the extent up to the last element, strides honoured
    size_t n;
    if (blck(t->type) == 1) {
        n = tsize(t->type);
        for (int i = 0; i < GGML_MAX_DIMS; ++i) n += (size_t)(t->ne[i] - 1) * t->nb[i];      // a permuted tensor's nb[0] is not the element size
    } else {
        n = (size_t)t->ne[0] * t->nb[0] / blck(t->type);
        for (int i = 1; i < GGML_MAX_DIMS; ++i) n += (size_t)(t->ne[i] - 1) * t->nb[i];
    }
    return n;
}
bool contiguous(const ggml_tensor * t) {
    return t->nb[0] == tsize(t->type) && t->nb[1] == row_size(t) && t->nb[2] == t->nb[1] * (size_t)t->ne[1] && t->nb[3] == t->nb[2] * (size_t)t->ne[2];
}

// Temporaries of one operator call (CPU-resident operands staged on the device, device results bound for the host, index lists).
// They come from one arena that lives as long as the scratch buffer: nodes are computed one after the other on one stream, so the
// next node may reuse the bytes as soon as its own work is queued behind the previous node's.  A call that needs more than the
// arena holds takes plain allocations for the excess (freed when it returns) and the arena grows before the next call.
struct Arena { char * base = nullptr; size_t cap = 0, want = 4u << 20; };
Arena g_arena;
struct Temps {
    std::vector<void *> extra;
    size_t off = 0, need = 0;
    Temps() {
        if (g_arena.want > g_arena.cap) {
            if (g_arena.base) { pi_sync(); pi_free(g_arena.base); }
            g_arena.cap = g_arena.want;
            g_arena.base = (char *)pi_malloc(g_arena.cap);
            if (!g_arena.base) die("temporary arena");
        }
    }
    void * get(size_t n) {
        n = (n + 255) & ~(size_t)255;
        need += n;
        if (off + n <= g_arena.cap) { void * p = g_arena.base + off; off += n; return p; }
        void * p = pi_malloc(n); if (!p) die("temporary allocation");
        extra.push_back(p);
        return p;
    }
    ~Temps() {
        for (void * p : extra) pi_free(p);
        if (need > g_arena.want) g_arena.want = need + (need >> 2);
    }
};

// Small host -> device transfers (a token's position, mask, scale and embedding row arrive this way for every evaluation) go through
// a ring of pinned slots: the bytes are copied into a slot and from there by an asynchronous transfer on the launch stream, so the host
// does not wait for the device (a plain hipMemcpy from pageable memory returns only when the device has the data, after everything
// queued before it).  A slot is reused once the event behind its last transfer has passed.
struct PinRing {
    static constexpr size_t kSlot = 64u << 10;
    static constexpr int kSlots = 32;
    char * base = nullptr;
    hipEvent_t ev[kSlots];
    bool used[kSlots] = {};
    int next = 0;
};
PinRing g_pin;
void h2d(void * dst, const void * src, size_t n) {
    if (n == 0) return;
    if (n > PinRing::kSlot) { BK_PI(pi_memcpy_h2d(dst, src, n)); return; }
    if (!g_pin.base) {
        g_pin.base = (char *)pi_malloc_host(PinRing::kSlot * PinRing::kSlots);
        if (!g_pin.base) die("pinned staging ring");
        for (int i = 0; i < PinRing::kSlots; ++i) BK_HIP(hipEventCreateWithFlags(&g_pin.ev[i], hipEventDisableTiming));
    }
    const int slot = g_pin.next;
    g_pin.next = (g_pin.next + 1) % PinRing::kSlots;
    if (g_pin.used[slot]) BK_HIP(hipEventSynchronize(g_pin.ev[slot]));
    char * stage = g_pin.base + (size_t)slot * PinRing::kSlot;
    memcpy(stage, src, n);
    BK_HIP(hipMemcpyAsync(dst, stage, n, hipMemcpyHostToDevice, nullptr));
    BK_HIP(hipEventRecord(g_pin.ev[slot], nullptr));
    g_pin.used[slot] = true;
}

void * dev_ptr(const ggml_tensor * t) {
    const Extra * e = (const Extra *)t->extra;
    if (!e || !e->data_device[0]) { fprintf(stderr, "powerinfer-hip backend: tensor '%s' is marked GPU but has no device buffer\n", t->name); exit(1); }
    if (e->outside_scratch) { fprintf(stderr, "powerinfer-hip backend: tensor '%s' was given a scratch offset outside the scratch buffer\n", t->name); exit(1); }
    return e->data_device[0];
}
void * dev_in(const ggml_tensor * t, Temps & tmp) {
    if (t->backend != GGML_BACKEND_CPU) return dev_ptr(t);
    const size_t n = nbytes(t);
    void * p = tmp.get(n);
    h2d(p, t->data, n);
    return p;
}
void * dev_out(ggml_tensor * t, Temps & tmp) {
    if (t->backend != GGML_BACKEND_CPU) return dev_ptr(t);
    return tmp.get(nbytes(t));
}
void finish_out(ggml_tensor * t, void * dptr) {
    if (t->backend == GGML_BACKEND_CPU) {          // result wanted on the host: copy back, device idle on return
        BK_PI(pi_sync());
        BK_PI(pi_memcpy_d2h(t->data, dptr, nbytes(t)));
    }
}

// hipBLASLt plans for mat-muls of long token batches (the reference's cuBLAS calls, ggml-cuda.cu:7662-7756); kept until the process ends
pi_gemm_lib * g_gemm = nullptr;
pi_gemm_lib * gemm_lib() {
    if (!g_gemm) {
        g_gemm = pi_gemm_lib_create((size_t)32 << 20);
        if (!g_gemm) die("pi_gemm_lib_create");
    }
    return g_gemm;
}

pi_workspace * workspace(int ff, int d) {
    if (!g_ws || ff > g_ws_ff || d > g_ws_d) {
        if (g_ws) { pi_sync(); pi_workspace_destroy(g_ws); }
        g_ws_ff = ff > g_ws_ff ? ff : g_ws_ff; g_ws_d = d > g_ws_d ? d : g_ws_d;
        g_ws = pi_workspace_create(g_ws_ff, g_ws_d);
        if (!g_ws) die("workspace");
    }
    return g_ws;
}

// ---- generic kernels (correctness-first; the tuned paths are the pi_k_* launchers) -----------------------
__global__ void bin_kernel(const float * a, const float * b, float * y, int64_t n, int64_t nb, int is_mul) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) y[i] = is_mul ? __fmul_rn(a[i], b[i % nb]) : __fadd_rn(a[i], b[i % nb]);
}
__global__ void relu_kernel(const float * a, float * y, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) y[i] = fmaxf(a[i], 0.0f);
}
__global__ void scale_kernel(const float * a, float * y, const float * s, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) y[i] = __fmul_rn(a[i], *s);
}
__global__ void fill_kernel(float * y, float v, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) y[i] = v;
}
// one workgroup per row; kind 0 rms_norm (ggml.c:9238), 1 norm (ggml.c:9169)
__global__ __launch_bounds__(256) void norm_rows_kernel(const float * x, float * y, int n, float eps, int kind) {
    __shared__ double red[4];
    const float * xr = x + (size_t)blockIdx.x * n; float * yr = y + (size_t)blockIdx.x * n;
    auto bsum = [&](double v) {
        v = pi_wave_sum_f64(v);
        __syncthreads();
        if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
        __syncthreads();
        return red[0] + red[1] + red[2] + red[3];
    };
    float mean = 0.0f;
    double s = 0.0;
    if (kind == 0) { for (int i = threadIdx.x; i < n; i += 256) s += (double)__fmul_rn(xr[i], xr[i]); s = bsum(s); }
    else {
        for (int i = threadIdx.x; i < n; i += 256) s += (double)xr[i];
        mean = (float)(bsum(s) / n);
        s = 0.0;
        for (int i = threadIdx.x; i < n; i += 256) { const float v = __fsub_rn(xr[i], mean); s += (double)__fmul_rn(v, v); }
        s = bsum(s);
    }
    const float scale = pi_inv_sqrt((float)(s / n) + eps);
    for (int i = threadIdx.x; i < n; i += 256) yr[i] = __fmul_rn(__fsub_rn(xr[i], mean), scale);
}
// norm -> * w -> (+ b) of one row in one launch (llm_build_norm's three nodes, llama.cpp:4420-4450, when each is computed in place of
// the one before); same arithmetic as the three kernels: double statistics, one fp32 product per step
__global__ __launch_bounds__(1024) void norm_affine_kernel(const float * x, const float * w, const float * b, float * y, int n, float eps, int kind) {
    __shared__ double red[16];
    auto bsum = [&](double v) {
        v = pi_wave_sum_f64(v);
        __syncthreads();
        if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
        __syncthreads();
        double t = 0.0;
        for (int i = 0; i < 16; ++i) t += red[i];
        return t;
    };
    float mean = 0.0f;
    double s = 0.0;
    if (kind == 0) { for (int i = threadIdx.x; i < n; i += 1024) s += (double)__fmul_rn(x[i], x[i]); s = bsum(s); }
    else {
        for (int i = threadIdx.x; i < n; i += 1024) s += (double)x[i];
        mean = (float)(bsum(s) / n);
        s = 0.0;
        for (int i = threadIdx.x; i < n; i += 1024) { const float v = __fsub_rn(x[i], mean); s += (double)__fmul_rn(v, v); }
        s = bsum(s);
    }
    const float scale = pi_inv_sqrt((float)(s / n) + eps);
    for (int i = threadIdx.x; i < n; i += 1024) {
        float v = __fmul_rn(__fmul_rn(__fsub_rn(x[i], mean), scale), w[i]);
        if (b) v = __fadd_rn(v, b[i]);
        y[i] = v;
    }
}
// one workgroup per row; exp through the fp16 rounding of the CPU path's table (ggml.c:10747-10759)
__global__ __launch_bounds__(256) void softmax_rows_kernel(const float * x, float * y, int n) {
    __shared__ double red[4];
    __shared__ float redf[4];
    const float * xr = x + (size_t)blockIdx.x * n; float * yr = y + (size_t)blockIdx.x * n;
    float mx = -INFINITY;
    for (int i = threadIdx.x; i < n; i += 256) mx = fmaxf(mx, xr[i]);
    mx = pi_wave_max(mx);
    if ((threadIdx.x & 63) == 0) redf[threadIdx.x >> 6] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(redf[0], redf[1]), fmaxf(redf[2], redf[3]));
    double s = 0.0;
    for (int i = threadIdx.x; i < n; i += 256) {
        const float v = xr[i] == -INFINITY ? 0.0f : pi_round_f16(expf(pi_round_f16(__fsub_rn(xr[i], mx))));
        yr[i] = v; s += (double)v;
    }
    s = pi_wave_sum_f64(s);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
    __syncthreads();
    const float inv = (float)(1.0 / (red[0] + red[1] + red[2] + red[3]));
    for (int i = threadIdx.x; i < n; i += 256) yr[i] = __fmul_rn(yr[i], inv);
}
// x [hd, n_head, T] with element strides s1 (head) and s2 (token), pos[T]; mode 0 adjacent pairs, 2 NeoX halves (ggml.c:11163-11325 for
// fp32, :11327-11460 for fp16).  fp16 is what the K-shift graph runs in place over a layer's K cache (llama.cpp:4332-4381): the same
// arithmetic with a conversion on either side.  A pair belongs to one thread, so y may be x.  Scaling as rope_yarn does it
// (ggml.c:11124-11146): the angle is freq_scale * theta; with ext != 0 it is mixed with the unscaled angle by a ramp over the pair
// index between corr0 and corr1, and cos / sin carry the magnitude factor mscale.  NeoX mode hands the ramp the rotation fraction
// through an integer parameter in the reference, which is 0 for every pair of a fully rotated head.
struct RopeScale { float freq_scale, ext, mscale, corr0, corr1; };
template <typename E>
__global__ void rope_kernel(const E * x, const int32_t * pos, E * y, size_t s1, size_t s2, size_t d1, size_t d2, int n_dims, int mode, float theta_scale, RopeScale rs) {
    const int t = blockIdx.y, h = blockIdx.x, i = threadIdx.x;         // i = pair index < n_dims/2
    const E * s = x + (size_t)t * s2 + (size_t)h * s1; E * o = y + (size_t)t * d2 + (size_t)h * d1;
    float theta = (float)pos[t];
    if (mode & 2) theta = __fmul_rn(theta, rs.freq_scale);
    for (int j = 0; j < i; ++j) theta = __fmul_rn(theta, theta_scale);
    float th = __fmul_rn(rs.freq_scale, theta);
    if (rs.ext != 0.0f) {
        const float ramp_y = __fdiv_rn(__fsub_rn((float)((mode & 2) ? 0 : i), rs.corr0), fmaxf(0.001f, __fsub_rn(rs.corr1, rs.corr0)));
        const float mix = __fmul_rn(__fsub_rn(1.0f, fminf(1.0f, fmaxf(0.0f, ramp_y))), rs.ext);
        th = __fadd_rn(__fmul_rn(th, __fsub_rn(1.0f, mix)), __fmul_rn(theta, mix));
    }
    const float c = __fmul_rn(cosf(th), rs.mscale), sn = __fmul_rn(sinf(th), rs.mscale);
    const int i0 = (mode & 2) ? i : 2 * i, i1 = (mode & 2) ? i + n_dims / 2 : 2 * i + 1;
    const float x0 = (float)s[i0], x1 = (float)s[i1];
    o[i0] = (E)__fsub_rn(__fmul_rn(x0, c), __fmul_rn(x1, sn));
    o[i1] = (E)__fadd_rn(__fmul_rn(x0, sn), __fmul_rn(x1, c));
}
struct Shape { int64_t ne[4]; size_t nb[4]; };
// element-wise copy with type conversion between two 4-D strided tensors of the same element count (ggml_cpy)
__global__ void cpy_kernel(const char * src, Shape ss, int stype, char * dst, Shape ds, int dtype, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    int64_t r = i; size_t so = 0, dof = 0;
    { int64_t q = r; for (int k = 0; k < 4; ++k) { const int64_t id = q % ss.ne[k]; q /= ss.ne[k]; so += (size_t)id * ss.nb[k]; } }
    { int64_t q = r; for (int k = 0; k < 4; ++k) { const int64_t id = q % ds.ne[k]; q /= ds.ne[k]; dof += (size_t)id * ds.nb[k]; } }
    const float v = stype == GGML_TYPE_F16 ? __half2float(*(const __half *)(src + so)) : *(const float *)(src + so);
    if (dtype == GGML_TYPE_F16) *(__half *)(dst + dof) = __float2half_rn(v); else *(float *)(dst + dof) = v;
}
// generic mat-mul for strided / batched operands (attention K.q and V.p): one wave per output element.
// src0 F16 or F32 [ne00, ne01, ne02, ne03] with strides, src1 F32 [ne00, ne11, ne12, ne13]; activations rounded to fp16
// when src0 is F16, as the CPU path does.
__global__ __launch_bounds__(64) void mul_mat_strided_kernel(const char * w, Shape ws, int wtype, const char * x, Shape xs, float * y, Shape ys) {
    const int64_t r = blockIdx.x, t = blockIdx.y, b = blockIdx.z;
    const int64_t i12 = b % xs.ne[2], i13 = b / xs.ne[2];
    const int64_t i02 = i12 / (xs.ne[2] / ws.ne[2]), i03 = i13 / (xs.ne[3] / ws.ne[3]);
    const char * wr = w + r * ws.nb[1] + i02 * ws.nb[2] + i03 * ws.nb[3];
    const char * xr = x + t * xs.nb[1] + i12 * xs.nb[2] + i13 * xs.nb[3];
    float acc = 0.0f;
    for (int64_t k = threadIdx.x; k < ws.ne[0]; k += 64) {
        const float xv = *(const float *)(xr + k * xs.nb[0]);
        if (wtype == GGML_TYPE_F16) acc = fmaf(__half2float(*(const __half *)(wr + k * ws.nb[0])), pi_round_f16(xv), acc);
        else acc = fmaf(*(const float *)(wr + k * ws.nb[0]), xv, acc);
    }
    acc = pi_wave_sum(acc);
    if (threadIdx.x == 0) *(float *)((char *)y + r * ys.nb[0] + t * ys.nb[1] + i12 * ys.nb[2] + i13 * ys.nb[3]) = acc;
}
__global__ void get_rows_kernel(const char * table, int type, size_t row_bytes, const int32_t * ids, float * y, int cols) {
    const char * row = table + (size_t)ids[blockIdx.y] * row_bytes;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= cols) return;
    float v;
    if (type == GGML_TYPE_F32) v = ((const float *)row)[i];
    else if (type == GGML_TYPE_F16) v = __half2float(((const __half *)row)[i]);
    else {
        const pi_block_q4_0 * blk = (const pi_block_q4_0 *)row + (i >> 5);
        uint16_t d; __builtin_memcpy(&d, &blk->d, 2);
        const int j = i & 31;
        const int q = j < 16 ? (blk->qs[j] & 0x0F) : (blk->qs[j - 16] >> 4);
        v = __fmul_rn((float)(q - 8), pi_f16_from_bits(d));
    }
    y[(size_t)blockIdx.y * cols + i] = v;
}
__global__ void gather_h_kernel(const float * h_dense, const int32_t * list, const int32_t * n_active, const int32_t * bucket, float * h_compact) {
    const int n = *n_active;
    for (int k = blockIdx.x * blockDim.x + threadIdx.x; k < n; k += gridDim.x * blockDim.x) {
        const int row = list[k];
        h_compact[k] = h_dense[bucket ? bucket[row] : row];
    }
}

Shape shape_of(const ggml_tensor * t) { Shape s; for (int i = 0; i < 4; ++i) { s.ne[i] = t->ne[i]; s.nb[i] = t->nb[i]; } return s; }
dim3 grid1(int64_t n) { return dim3((unsigned)((n + 255) / 256)); }

// ---- operators ---------------------------------------------------------------------------------------------
bool op_mul_mat(ggml_tensor * dst) {
    const ggml_tensor * a = dst->src[0]; const ggml_tensor * b = dst->src[1];
    if (b->type != GGML_TYPE_F32 || dst->type != GGML_TYPE_F32) return false;
    Temps tmp;
    const bool weight_like = a->ne[2] == 1 && a->ne[3] == 1 && a->nb[0] == tsize(a->type) && a->nb[1] == row_size(a) && contiguous(b) && contiguous(dst) &&
                             (a->type == GGML_TYPE_F16 || a->type == GGML_TYPE_Q4_0) && a->ne[0] % (a->type == GGML_TYPE_F16 ? 8 : 32) == 0;
    if (!weight_like && a->type != GGML_TYPE_F16 && a->type != GGML_TYPE_F32) return false;
    const char * wa = (const char *)dev_in(a, tmp); const char * xb = (const char *)dev_in(b, tmp); float * y = (float *)dev_out(dst, tmp);
    if (weight_like) {
        const int64_t T = nrows(b);
        if (T > 32 && a->type == GGML_TYPE_F16 && T * a->ne[0] < ((int64_t)1 << 28)) {     // a prompt batch: one library mat-mul over all its tokens
            const int cols = (int)a->ne[0], rows = (int)a->ne[1];
            __half * xn16 = (__half *)tmp.get(sizeof(__half) * (size_t)T * cols);
            BK_PI(pi_k_norm_round_f16((const float *)xb, (int)T, cols, nullptr, xn16, nullptr, nullptr));
            BK_PI(pi_gemm_lib_f16(gemm_lib(), wa, rows, cols, xn16, (int)T, PI_EPI_NONE, nullptr, nullptr, y, nullptr, nullptr));
            finish_out(dst, y);
            return true;
        }
        if (T > 1 && a->type == GGML_TYPE_F16 && a->ne[0] % 128 == 0) {          // the matrix is read once per 16 tokens (matrix cores)
            const int cols = (int)a->ne[0], rows = (int)a->ne[1];
            __half * xn16 = (__half *)tmp.get(sizeof(__half) * 16 * (size_t)cols);
            for (int64_t t0 = 0; t0 < T; t0 += 16) {
                const int tc = (int)(T - t0 < 16 ? T - t0 : 16);
                BK_PI(pi_k_norm_round_f16((const float *)xb + t0 * cols, tc, cols, nullptr, xn16, nullptr, nullptr));
                BK_PI(pi_k_gemm_f16(wa, rows, cols, xn16, tc, PI_EPI_NONE, nullptr, nullptr, y + t0 * rows, nullptr, nullptr));
            }
            finish_out(dst, y);
            return true;
        }
        for (int64_t t = 0; t < T; ++t)
            BK_PI(pi_k_gemv(a->type, wa, (int)a->ne[1], (int)a->ne[0], (const float *)xb + t * b->ne[0], nullptr, PI_EPI_NONE, nullptr, nullptr, y + t * a->ne[1], nullptr));
    } else {
        hipLaunchKernelGGL(mul_mat_strided_kernel, dim3((unsigned)a->ne[1], (unsigned)b->ne[1], (unsigned)(b->ne[2] * b->ne[3])), dim3(64), 0, 0,
                           wa, shape_of(a), (int)a->type, xb, shape_of(b), y, shape_of(dst));
    }
    finish_out(dst, y);
    return true;
}

bool sparse_common(ggml_tensor * dst, bool axpy) {
    const ggml_tensor * w = dst->src[0]; const ggml_tensor * x = dst->src[1]; const ggml_tensor * idx = dst->src[2]; const ggml_tensor * aux = dst->src[3];
    if (!idx || (w->type != GGML_TYPE_F16 && w->type != GGML_TYPE_Q4_0) || x->type != GGML_TYPE_F32 || idx->type != GGML_TYPE_F32) return false;
    if (!contiguous(x) || !contiguous(idx) || !contiguous(dst) || w->nb[1] != row_size(w)) return false;
    Temps tmp;
    const int d = (int)w->ne[0], rows = (int)w->ne[1], ff = (int)idx->ne[0];
    const int64_t T = nrows(x);
    const char * wd = (const char *)dev_in(w, tmp); const float * xd = (const float *)dev_in(x, tmp);
    const float * id = (const float *)dev_in(idx, tmp);
    const int32_t * bk = aux ? (const int32_t *)dev_in(aux, tmp) : nullptr;       // GPU part: gpu_bucket maps rows -> neurons
    const int n_bucket = aux ? (int)aux->ne[0] : 0;
    if (aux && n_bucket != rows) return false;
    if (!aux && rows != ff) return false;
    float * y = (float *)dev_out(dst, tmp);
    pi_workspace * ws = workspace(ff, d);
    int32_t * list = (int32_t *)tmp.get(sizeof(int32_t) * (size_t)rows);
    int32_t * n_act = (int32_t *)tmp.get(sizeof(int32_t));
    float * hc = (float *)tmp.get(sizeof(float) * (size_t)rows);
    const int out_n = (int)dst->ne[0];
    // a step of several tokens with every neuron resident: each weight row is read once for up to 16 tokens at a time (the
    // reference's batch kernels, ggml-cuda.cu:6994-7034, 8787-8814); other layouts go token by token below
    if (T > 1 && !aux && w->type == GGML_TYPE_F16 && d % 256 == 0 && d <= g_ws_d) {
        __half * xn16 = axpy ? nullptr : (__half *)tmp.get(sizeof(__half) * 16 * (size_t)d);
        for (int64_t t0 = 0; t0 < T; t0 += 16) {
            const int tc = (int)(T - t0 < 16 ? T - t0 : 16);
            if (!axpy) {
                BK_PI(pi_k_norm_round_f16(xd + t0 * d, tc, d, nullptr, xn16, nullptr, nullptr));
                BK_PI(pi_k_batch_sparse_mul_mat(wd, ff, d, xn16, tc, id + t0 * ff, g_threshold, y + t0 * out_n, list, n_act, ws, nullptr));
            } else {
                BK_PI(pi_k_batch_sparse_axpy(wd, d, ff, xd + t0 * ff, id + t0 * ff, tc, g_threshold, y + t0 * d, list, n_act, ws, nullptr));
            }
        }
        finish_out(dst, y);
        return true;
    }
    for (int64_t t = 0; t < T; ++t) {
        BK_PI(pi_k_compact_active(id + t * ff, ff, g_threshold, bk, n_bucket, list, n_act, ws, nullptr));
        if (!axpy) {
            // dst[neuron] = W[row] . x for active rows, 0 elsewhere (GGML_OP_MUL_MAT_SPARSE; upscale writes bucket positions only)
            hipLaunchKernelGGL(fill_kernel, grid1(out_n), dim3(256), 0, 0, y + t * out_n, 0.0f, (int64_t)out_n);
            BK_PI(pi_k_sparse_upgate(w->type, wd, nullptr, d, ff, xd + t * d, nullptr, 0, list, n_act, bk, hc, nullptr, y + t * out_n, nullptr, ws, nullptr));
        } else {
            // x is the dense, neuron-indexed h; out[d] = sum over active rows of h[neuron] * Wt[row]
            hipLaunchKernelGGL(gather_h_kernel, dim3(16), dim3(256), 0, 0, xd + t * ff, list, n_act, bk, hc);
            BK_PI(pi_k_sparse_axpy(w->type, wd, d, rows, hc, xd + t * ff, bk, list, n_act, PI_EPI_NONE, nullptr, nullptr, y + t * d, ws, nullptr));
        }
    }
    finish_out(dst, y);
    return true;
}

bool op_elementwise(ggml_tensor * dst) {
    const ggml_tensor * a = dst->src[0]; const ggml_tensor * b = dst->src[1];
    if (a->type != GGML_TYPE_F32 || dst->type != GGML_TYPE_F32 || !contiguous(a) || !contiguous(dst)) return false;
    Temps tmp;
    const int64_t n = nelem(dst);
    if (dst->op == GGML_OP_ADD || dst->op == GGML_OP_MUL) {
        if (!b || b->type != GGML_TYPE_F32 || !contiguous(b) || n % nelem(b)) return false;
        const float * ad = (const float *)dev_in(a, tmp); const float * bd = (const float *)dev_in(b, tmp); float * y = (float *)dev_out(dst, tmp);
        hipLaunchKernelGGL(bin_kernel, grid1(n), dim3(256), 0, 0, ad, bd, y, n, nelem(b), dst->op == GGML_OP_MUL ? 1 : 0);
        finish_out(dst, y);
    } else if (dst->op == GGML_OP_UNARY) {
        const float * ad = (const float *)dev_in(a, tmp); float * y = (float *)dev_out(dst, tmp);
        hipLaunchKernelGGL(relu_kernel, grid1(n), dim3(256), 0, 0, ad, y, n);
        finish_out(dst, y);
    } else if (dst->op == GGML_OP_SCALE) {
        if (!b || b->type != GGML_TYPE_F32) return false;
        const float * ad = (const float *)dev_in(a, tmp); const float * sd = (const float *)dev_in(b, tmp); float * y = (float *)dev_out(dst, tmp);
        hipLaunchKernelGGL(scale_kernel, grid1(n), dim3(256), 0, 0, ad, y, sd, n);       // the factor is a 1-element tensor, read where it lives
        finish_out(dst, y);
    } else if (dst->op == GGML_OP_RMS_NORM || dst->op == GGML_OP_NORM) {
        float eps; memcpy(&eps, dst->op_params, 4);
        const float * ad = (const float *)dev_in(a, tmp); float * y = (float *)dev_out(dst, tmp);
        hipLaunchKernelGGL(norm_rows_kernel, dim3((unsigned)nrows(a)), dim3(256), 0, 0, ad, y, (int)a->ne[0], eps, dst->op == GGML_OP_NORM ? 1 : 0);
        finish_out(dst, y);
    } else if (dst->op == GGML_OP_SOFT_MAX) {
        const float * ad = (const float *)dev_in(a, tmp); float * y = (float *)dev_out(dst, tmp);
        hipLaunchKernelGGL(softmax_rows_kernel, dim3((unsigned)nrows(a)), dim3(256), 0, 0, ad, y, (int)a->ne[0]);
        finish_out(dst, y);
    } else {
        return false;
    }
    return true;
}

bool op_rope(ggml_tensor * dst) {
    const ggml_tensor * a = dst->src[0]; const ggml_tensor * p = dst->src[1];
    if ((a->type != GGML_TYPE_F32 && a->type != GGML_TYPE_F16) || dst->type != a->type || !p || p->type != GGML_TYPE_I32 || a->ne[3] != 1) return false;
    const size_t es = tsize(a->type);
    // rows of one head contiguous; heads and tokens at any stride that is a whole number of elements (views into the KV cache)
    if (a->nb[0] != es || dst->nb[0] != es || a->nb[1] % es || a->nb[2] % es || dst->nb[1] % es || dst->nb[2] % es) return false;
    const int n_dims = dst->op_params[1], mode = dst->op_params[2], n_orig_ctx = dst->op_params[4];
    float freq_base, freq_scale, ext_factor, attn_factor, beta_fast, beta_slow;
    memcpy(&freq_base, dst->op_params + 5, 4); memcpy(&freq_scale, dst->op_params + 6, 4); memcpy(&ext_factor, dst->op_params + 7, 4);
    memcpy(&attn_factor, dst->op_params + 8, 4); memcpy(&beta_fast, dst->op_params + 9, 4); memcpy(&beta_slow, dst->op_params + 10, 4);
    if ((mode != 0 && mode != 2) || n_dims != a->ne[0] || n_dims / 2 > 1024) return false;       // no GLM / xPos / partial rotation here
    // YaRN's correction dimensions and magnitude factor, as the host computes them (ggml_rope_yarn_corr_dims, ggml.c:11148-11161)
    RopeScale rs{freq_scale, ext_factor, attn_factor, 0.0f, 0.0f};
    if (ext_factor != 0.0f) {
        auto corr_dim = [&](float n_rot) { return n_dims * logf(n_orig_ctx / (n_rot * 2 * (float)M_PI)) / (2 * logf(freq_base)); };
        rs.corr0 = fmaxf(0.0f, floorf(corr_dim(beta_fast)));
        rs.corr1 = fminf((float)(n_dims - 1), ceilf(corr_dim(beta_slow)));
        rs.mscale = attn_factor * (1.0f + 0.1f * logf(1.0f / freq_scale));
    }
    if (a->backend == GGML_BACKEND_CPU && !contiguous(a)) return false;                                                // staged operands are copied as one block
    if (dst->backend == GGML_BACKEND_CPU && !contiguous(dst)) return false;
    Temps tmp;
    const void * ad = dev_in(a, tmp); const int32_t * pd = (const int32_t *)dev_in(p, tmp); void * y = dev_out(dst, tmp);
    const float theta_scale = powf(freq_base, -2.0f / n_dims);
    const dim3 grid((unsigned)a->ne[1], (unsigned)a->ne[2]), block(n_dims / 2);
    if (a->type == GGML_TYPE_F32)
        hipLaunchKernelGGL(rope_kernel<float>, grid, block, 0, 0, (const float *)ad, pd, (float *)y, a->nb[1] / es, a->nb[2] / es, dst->nb[1] / es, dst->nb[2] / es,
                           n_dims, mode, theta_scale, rs);
    else
        hipLaunchKernelGGL(rope_kernel<__half>, grid, block, 0, 0, (const __half *)ad, pd, (__half *)y, a->nb[1] / es, a->nb[2] / es, dst->nb[1] / es, dst->nb[2] / es,
                           n_dims, mode, theta_scale, rs);
    finish_out(dst, y);
    return true;
}

bool op_cpy(ggml_tensor * dst) {
    // CPY: src0 -> src1 (a view, e.g. into the KV cache), dst is a view of src1.  CONT / DUP: src0 -> dst.
    const ggml_tensor * a = dst->src[0];
    ggml_tensor * to = dst->op == GGML_OP_CPY ? dst->src[1] : dst;
    if ((a->type != GGML_TYPE_F32 && a->type != GGML_TYPE_F16) || (to->type != GGML_TYPE_F32 && to->type != GGML_TYPE_F16) || nelem(a) != nelem(to)) return false;
    Temps tmp;
    const char * ad = (const char *)dev_in(a, tmp);
    char * td;
    if (to->backend != GGML_BACKEND_CPU) td = (char *)dev_ptr(to);
    else { td = (char *)tmp.get(nbytes(to)); BK_PI(pi_memcpy_h2d(td, to->data, nbytes(to))); }      // strided destination: keep the gaps
    hipLaunchKernelGGL(cpy_kernel, grid1(nelem(a)), dim3(256), 0, 0, ad, shape_of(a), (int)a->type, td, shape_of(to), (int)to->type, nelem(a));
    finish_out(to, td);
    return true;
}

bool op_get_rows(ggml_tensor * dst) {
    const ggml_tensor * a = dst->src[0]; const ggml_tensor * ids = dst->src[1];
    if (!ids || ids->type != GGML_TYPE_I32 || a->nb[1] != row_size(a) || !contiguous(dst) || tsize(a->type) == 0 || a->type == GGML_TYPE_I32) return false;
    Temps tmp;
    const char * ad = (const char *)dev_in(a, tmp); const int32_t * id = (const int32_t *)dev_in(ids, tmp); float * y = (float *)dev_out(dst, tmp);
    hipLaunchKernelGGL(get_rows_kernel, dim3((unsigned)((a->ne[0] + 255) / 256), (unsigned)nelem(ids)), dim3(256), 0, 0, ad, (int)a->type, row_size(a), id, y, (int)a->ne[0]);
    finish_out(dst, y);
    return true;
}

bool run_node(ggml_tensor * tensor) {
    switch (tensor->op) {
        case GGML_OP_MUL_MAT:        return op_mul_mat(tensor);
        case GGML_OP_MUL_MAT_SPARSE: return sparse_common(tensor, false);
        case GGML_OP_AXPY:           return sparse_common(tensor, true);
        case GGML_OP_ROPE:           return op_rope(tensor);
        case GGML_OP_CPY: case GGML_OP_CONT: case GGML_OP_DUP: return op_cpy(tensor);
        case GGML_OP_GET_ROWS:       return op_get_rows(tensor);
        case GGML_OP_RESHAPE: case GGML_OP_VIEW: case GGML_OP_PERMUTE: case GGML_OP_TRANSPOSE: return true;
        default:                     return op_elementwise(tensor);
    }
}

Extra * new_extra(void * p, bool owned) {
    Extra * e = new Extra();
    memset(e, 0, sizeof *e);
    e->data_device[0] = p; e->owned = owned;
    return e;
}

bool view_like(int op) { return op == GGML_OP_RESHAPE || op == GGML_OP_VIEW || op == GGML_OP_PERMUTE || op == GGML_OP_TRANSPOSE; }
char * scratch_base() {
    if (!g_scratch) { g_scratch = (char *)pi_malloc(g_scratch_size); if (!g_scratch) die("scratch"); }
    return g_scratch;
}
// Device address of a tensor that shares its parent's memory (ggml-cuda.cu:9069-9082 and 9132-9141): an operator computed in
// place, a reshape / permute / transpose (same host address as src0) or a VIEW (byte offset in op_params) of a tensor that
// lives on the device takes the parent's device address; nullptr when the rule does not apply.
Extra * inplace_extra(const ggml_tensor * t, bool force_inplace) {
    const ggml_tensor * s0 = t->src[0];
    const bool inplace = (s0 != nullptr && s0->data == t->data) || t->op == GGML_OP_VIEW || force_inplace;
    if (!inplace || !s0 || s0->backend == GGML_BACKEND_CPU || !s0->extra) return nullptr;
    size_t offset = 0;
    if (t->op == GGML_OP_VIEW) memcpy(&offset, t->op_params, sizeof(size_t));
    const Extra * parent = (const Extra *)s0->extra;
    const bool unusable = parent->outside_scratch;
    Extra * e = ring_extra((char *)parent->data_device[0] + offset);      // may recycle the parent's slot only after 8192 newer extras
    e->outside_scratch = unusable;
    return e;
}

// ggml_cuda_assign_buffers_impl (ggml-cuda.cu:9046-9117)
void assign(ggml_tensor * tensor, bool scratch, bool force_inplace, bool no_alloc) {
    if (scratch && g_scratch_size == 0) return;
    tensor->backend = GGML_BACKEND_GPU;
    // a chain of views above a host tensor moves to the device with its consumer, and so does the destination of a copy
    if (tensor->src[0] && tensor->src[0]->backend == GGML_BACKEND_CPU && view_like(tensor->src[0]->op)) assign(tensor->src[0], scratch, force_inplace, no_alloc);
    if (tensor->op == GGML_OP_CPY && tensor->src[1]->backend == GGML_BACKEND_CPU) assign(tensor->src[1], scratch, force_inplace, no_alloc);
    if (scratch && no_alloc) return;
    std::lock_guard<std::mutex> g(g_mu);
    if (Extra * shared = inplace_extra(tensor, force_inplace)) { tensor->extra = shared; return; }
    if (tensor->op == GGML_OP_CPY) {                                    // the result of a copy is its destination
        tensor->extra = ring_extra(dev_ptr(tensor->src[1]));
        return;
    }
    const size_t n = nbytes(tensor);
    if (scratch) {
        if (n > g_scratch_size) { fprintf(stderr, "powerinfer-hip backend: '%s' (%zu bytes) exceeds the scratch buffer (%zu)\n", tensor->name, n, g_scratch_size); exit(1); }
        if (g_scratch_offset + n > g_scratch_size) g_scratch_offset = 0;            // ring, as the reference's scratch buffer
        tensor->extra = ring_extra(scratch_base() + g_scratch_offset);
        g_scratch_offset += n;
    } else {
        void * p = pi_malloc(n); if (!p) die("tensor allocation");
        BK_HIP(hipMemset(p, 0, n));
        tensor->extra = new_extra(p, true);                            // released by ggml_cuda_free_data (the KV cache, llama.cpp:1420-1422)
    }
}

// ---- deferred nodes -----------------------------------------------------------------------------------------
// The host hands over one node at a time, in graph order.  A single-token node that may turn out to be part of a block this library
// computes in one launch is not run when it arrives: it joins a window of pending nodes.  The window only ever holds consecutive
// nodes - the first node that cannot join it either consumes it (the AXPY node that completes llm_build_ffn_sparse's sequence,
// llama.cpp:4652-4757: fc1 -> relu -> fc2 -> sparse up / gate -> relu * mul -> sparse down becomes pi_k_gemv + pi_k_sparse_ffn) or makes
// every pending node run, in order, before it runs itself.  Running a node late but in order, with nothing else in between, is
// the schedule the host's allocator planned for, so buffers it shares between nodes stay valid.
// The fused block does not write the dense up / gate vectors and the predictor's hidden layer: in the reference's graph nothing
// else reads them (they are locals of llm_build_ffn_sparse); the predictor logits and h are still written to their nodes.  When the
// node behind the AXPY node adds the residual to its result (llama.cpp:5063, 5443), that add is the block's epilogue and only the
// sum is written.
// GGML_CUDA_NO_FUSION=1 in the environment turns the window off (every node runs when it arrives).
struct PendingNode { ggml_tensor * t; int op; const ggml_tensor * src[4]; void * extra; };
std::vector<PendingNode> g_pending;
bool g_fuse = true;
pi_ggml_backend_stats g_stats{};
constexpr size_t kMaxPending = 24;

bool is_pending(const ggml_tensor * t) { for (const PendingNode & p : g_pending) if (p.t == t) return true; return false; }
bool on_device(const ggml_tensor * t) { return t && t->backend != GGML_BACKEND_CPU && t->extra != nullptr && !((const Extra *)t->extra)->outside_scratch; }
bool vec1(const ggml_tensor * t) { return t && t->type == GGML_TYPE_F32 && contiguous(t) && nrows(t) == 1; }
bool avail(const ggml_tensor * t) { return vec1(t) && (is_pending(t) || on_device(t)); }
bool weight_on_device(const ggml_tensor * a) {
    return on_device(a) && a->ne[2] == 1 && a->ne[3] == 1 && a->nb[0] == tsize(a->type) && a->nb[1] == row_size(a) &&
           (a->type == GGML_TYPE_F16 || a->type == GGML_TYPE_Q4_0) && a->ne[0] % (a->type == GGML_TYPE_F16 ? 8 : 32) == 0;
}

// through reshapes, permutes, transposes and views to the node that computes the data
const ggml_tensor * base_of(const ggml_tensor * t) { while (t && view_like(t->op) && t->src[0]) t = t->src[0]; return t; }
// an fp32 result of one token: contiguous, at most two dimensions larger than one
bool one_token(const ggml_tensor * t) { return t && t->type == GGML_TYPE_F32 && contiguous(t) && t->ne[3] == 1 && (t->ne[1] == 1 || t->ne[2] == 1); }

// The nodes between the q / k / v projections and the output projection of one token's attention (llm_build_kv_store, llm_build_kqv:
// ROPE, CPY into the cache, K.q, SCALE, + mask, SOFT_MAX, V.p, CONT) join a window that the attention norm opened, so that the block can
// run as three launches when the window is flushed (try_fused_attn); on their own they run as they always did, in order.
bool deferrable_attn(const ggml_tensor * n) {
    // (the node of a copy into the cache is a view of its destination and is never read through its own address)
    if (g_pending.empty() || n->backend != GGML_BACKEND_GPU || (n->op != GGML_OP_CPY && !on_device(n))) return false;
    const ggml_tensor * a = n->src[0]; const ggml_tensor * b = n->src[1];
    if (!a) return false;
    const ggml_tensor * ab = base_of(a);
    switch (n->op) {
        case GGML_OP_ROPE: return one_token(n) && a->type == GGML_TYPE_F32 && is_pending(ab) && b && on_device(b) && !is_pending(b);
        case GGML_OP_CPY:  return b && on_device(b) && is_pending(ab) && nelem(a) == nelem(b) && nelem(a) <= 16384;
        case GGML_OP_MUL_MAT: return one_token(n) && b && is_pending(base_of(b)) && b->type == GGML_TYPE_F32 && on_device(a) && !is_pending(ab) && a->type == GGML_TYPE_F16;
        case GGML_OP_SCALE: return one_token(n) && is_pending(a) && b && on_device(b) && !is_pending(b);
        case GGML_OP_ADD: return one_token(n) && is_pending(a) && b && on_device(b) && !is_pending(b) && b->type == GGML_TYPE_F32 && b->ne[0] == a->ne[0];
        case GGML_OP_SOFT_MAX: return one_token(n) && is_pending(a);
        case GGML_OP_CONT: return one_token(n) && is_pending(ab) && a->type == GGML_TYPE_F32;
        default: return false;
    }
}

bool deferrable(const ggml_tensor * n) {
    if (!g_fuse || g_pending.size() >= kMaxPending) return false;
    if (n->backend != GGML_BACKEND_GPU || !vec1(n) || !on_device(n)) return deferrable_attn(n);
    const ggml_tensor * a = n->src[0]; const ggml_tensor * b = n->src[1];
    switch (n->op) {
        case GGML_OP_RMS_NORM: case GGML_OP_NORM: return vec1(a) && on_device(a) && !is_pending(a) && nelem(a) == nelem(n);
        case GGML_OP_MUL: case GGML_OP_ADD: return is_pending(a) && vec1(a) && avail(b) && nelem(b) == nelem(n) && nelem(a) == nelem(n);
        case GGML_OP_UNARY: return n->op_params[0] == GGML_UNARY_OP_RELU && is_pending(a) && vec1(a);
        case GGML_OP_MUL_MAT: return weight_on_device(a) && avail(b) && b->ne[0] == a->ne[0] && n->ne[0] == a->ne[1];
        case GGML_OP_MUL_MAT_SPARSE:
            return n->src[3] == nullptr && weight_on_device(a) && avail(b) && b->ne[0] == a->ne[0] && avail(n->src[2]) &&
                   n->src[2]->ne[0] == a->ne[1] && n->ne[0] == a->ne[1];
        default: return deferrable_attn(n);
    }
}
void defer(ggml_tensor * n) { ++g_stats.nodes_deferred; g_pending.push_back(PendingNode{n, (int)n->op, {n->src[0], n->src[1], n->src[2], n->src[3]}, n->extra}); }
// a node of an abandoned evaluation (the host rebuilt its graph in the same memory) no longer looks the way it was deferred
bool still_valid(const PendingNode & p) {
    return p.t->op == p.op && p.t->src[0] == p.src[0] && p.t->src[1] == p.src[1] && p.t->src[2] == p.src[2] && p.t->src[3] == p.src[3] && p.t->extra == p.extra;
}

// One token's attention block of build_llama (llama.cpp:4977-5022): attention norm, the q / k / v projections, RoPE, the two copies into
// the KV cache, K.q, scale, + mask, soft-max, V.p, the gather of the heads, the output projection and the residual - seventeen nodes
// (fourteen to sixteen in the first layer, whose norm and residual read the embedding from the host and run on their own).
// When the window holds exactly those, they run as three launches: the three projections with the norm as their prologue
// (pi_k_gemv_multi_f16), the attention on the cache's own layouts (pi_k_attn_ggml), the output projection with the residual as its
// epilogue.  q, k and v pass through a buffer of this library's own (their nodes' buffers may have been handed on by the host's plan
// by the time the attention reads them).  Returns false, with nothing done, for any other window.
bool try_fused_attn(const std::vector<PendingNode> & win) {
    auto in_win = [&](const ggml_tensor * t) -> const ggml_tensor * {
        if (!t) return nullptr;
        for (const PendingNode & p : win) if (p.t == t && still_valid(p)) return t;
        return nullptr;
    };
    auto with_op = [&](const ggml_tensor * t, int op) -> const ggml_tensor * { return (in_win(t) && t->op == op) ? t : nullptr; };
    size_t live = 0;
    const ggml_tensor * sm = nullptr;
    for (const PendingNode & p : win) {
        if (!still_valid(p)) continue;
        ++live;
        if (p.t->op == GGML_OP_SOFT_MAX) { if (sm) return false; sm = p.t; }
    }
    if (!sm || live < 14 || live > 17) return false;
    const ggml_tensor * addm = with_op(sm->src[0], GGML_OP_ADD);
    const ggml_tensor * scl = addm ? with_op(addm->src[0], GGML_OP_SCALE) : nullptr;
    const ggml_tensor * kq = scl ? with_op(scl->src[0], GGML_OP_MUL_MAT) : nullptr;
    if (!kq) return false;
    const ggml_tensor * mask = addm->src[1]; const ggml_tensor * kq_scale = scl->src[1];
    const ggml_tensor * kview = kq->src[0];
    const ggml_tensor * ropeq = with_op(base_of(kq->src[1]), GGML_OP_ROPE);
    const ggml_tensor * kcpy = kview ? with_op(kview->src[1], GGML_OP_CPY) : nullptr;
    const ggml_tensor * ropek = kcpy ? with_op(base_of(kcpy->src[0]), GGML_OP_ROPE) : nullptr;
    if (!ropeq || !ropek || kview->op != GGML_OP_VIEW) return false;
    const ggml_tensor * mmq = with_op(base_of(ropeq->src[0]), GGML_OP_MUL_MAT);
    const ggml_tensor * mmk = with_op(base_of(ropek->src[0]), GGML_OP_MUL_MAT);
    const ggml_tensor * kqv = nullptr; const ggml_tensor * cont = nullptr; const ggml_tensor * mmo = nullptr; const ggml_tensor * addr = nullptr;
    for (const PendingNode & p : win) {
        if (!still_valid(p)) continue;
        if (p.t->op == GGML_OP_MUL_MAT && p.t->src[1] == sm) kqv = p.t;
    }
    if (!mmq || !mmk || !kqv) return false;
    for (const PendingNode & p : win) {
        if (!still_valid(p)) continue;
        if (p.t->op == GGML_OP_CONT && base_of(p.t->src[0]) == kqv) cont = p.t;
    }
    if (!cont) return false;
    for (const PendingNode & p : win) {
        if (!still_valid(p)) continue;
        if (p.t->op == GGML_OP_MUL_MAT && p.t->src[1] == cont) mmo = p.t;
    }
    if (!mmo) return false;
    for (const PendingNode & p : win) {
        if (!still_valid(p)) continue;
        if (p.t->op == GGML_OP_ADD && p.t->src[0] == mmo) addr = p.t;
    }
    const ggml_tensor * vview = kqv->src[0];
    const ggml_tensor * vcpy = vview ? with_op(vview->src[1], GGML_OP_CPY) : nullptr;
    const ggml_tensor * mmv = vcpy ? with_op(base_of(vcpy->src[0]), GGML_OP_MUL_MAT) : nullptr;
    if (!mmv || vview->op != GGML_OP_VIEW) return false;
    const ggml_tensor * X = mmq->src[1];
    if (mmk->src[1] != X || mmv->src[1] != X) return false;
    // the projections' input: norm(F) * w with both nodes in the window (the norm becomes the projections' prologue), or a vector
    // that exists (the first layer's norm reads the embedding from the host and has run already)
    const ggml_tensor * mulw = with_op(X, GGML_OP_MUL);
    const ggml_tensor * nrm = mulw ? in_win(mulw->src[0]) : nullptr;
    const ggml_tensor * F = X;
    if (mulw) {
        if (!nrm || (nrm->op != GGML_OP_RMS_NORM) || !on_device(mulw->src[1]) || in_win(mulw->src[1])) return false;
        F = nrm->src[0];
    } else if (in_win(X)) return false;
    if (!F || !on_device(F) || in_win(F)) return false;
    // 3 projections, 2 rope, 2 cpy, kq, scale, add, soft-max, kqv, cont, wo; the norm's two nodes and the residual add where they are pending
    if (live != (size_t)(14 + (mulw ? 2 : 0) + (addr ? 1 : 0))) return false;
    // ---- shapes, types, layouts ----
    const ggml_tensor * wq = mmq->src[0]; const ggml_tensor * wk = mmk->src[0]; const ggml_tensor * wv = mmv->src[0]; const ggml_tensor * wo = mmo->src[0];
    if (!weight_on_device(wq) || !weight_on_device(wk) || !weight_on_device(wv) || !weight_on_device(wo)) return false;
    if (wq->type != GGML_TYPE_F16 || wk->type != GGML_TYPE_F16 || wv->type != GGML_TYPE_F16) return false;
    const int d = (int)wq->ne[0];
    if ((d != 4096 && d != 5120 && d != 8192) || wk->ne[0] != d || wv->ne[0] != d || F->ne[0] != d || !vec1(F)) return false;
    const int hd = (int)ropeq->ne[0], n_head = (int)ropeq->ne[1], n_head_kv = (int)ropek->ne[1], gqa = n_head_kv * hd;
    if (ropeq->ne[2] != 1 || ropek->ne[2] != 1 || ropek->ne[0] != hd || wq->ne[1] != (int64_t)n_head * hd || wk->ne[1] != gqa || wv->ne[1] != gqa || n_head_kv <= 0 || n_head % n_head_kv) return false;
    if (wo->ne[0] != (int64_t)n_head * hd || nelem(cont) != (int64_t)n_head * hd) return false;
    if (memcmp(ropeq->op_params, ropek->op_params, sizeof(int32_t) * 11) != 0 || ropeq->src[1] != ropek->src[1]) return false;
    const int n_dims = ropeq->op_params[1], mode = ropeq->op_params[2];
    float freq_base, freq_scale, ext_factor, attn_factor;
    memcpy(&freq_base, ropeq->op_params + 5, 4); memcpy(&freq_scale, ropeq->op_params + 6, 4); memcpy(&ext_factor, ropeq->op_params + 7, 4); memcpy(&attn_factor, ropeq->op_params + 8, 4);
    const ggml_tensor * pos = ropeq->src[1];
    if (n_dims != hd || (mode != 0 && mode != 2) || ext_factor != 0.0f || !pos || pos->type != GGML_TYPE_I32 || !on_device(pos) || in_win(pos)) return false;
    // K cells [cell][gqa], V transposed [gqa][n_ctx]; the copies' destinations name the cell
    if (kview->type != GGML_TYPE_F16 || vview->type != GGML_TYPE_F16 || !on_device(kview) || !on_device(vview)) return false;
    const int n_kv = (int)kview->ne[1];
    if (kview->ne[0] != hd || kview->ne[2] != n_head_kv || kview->nb[0] != 2 || kview->nb[1] != (size_t)gqa * 2 || kview->nb[2] != (size_t)hd * 2) return false;
    if (vview->ne[0] != n_kv || vview->ne[1] != hd || vview->ne[2] != n_head_kv || vview->nb[0] != 2 || vview->nb[1] % 2 || vview->nb[2] != vview->nb[1] * hd) return false;
    const int n_ctx = (int)(vview->nb[1] / 2);
    const ggml_tensor * kdst = kcpy->src[1]; const ggml_tensor * vdst = vcpy->src[1];
    if (!kdst || !vdst || kdst->type != GGML_TYPE_F16 || vdst->type != GGML_TYPE_F16 || !on_device(kdst) || !on_device(vdst) || nelem(kdst) != gqa || nelem(vdst) != gqa) return false;
    const ptrdiff_t koff = (char *)dev_ptr(kdst) - (char *)dev_ptr(kview), voff = (char *)dev_ptr(vdst) - (char *)dev_ptr(vview);
    if (koff < 0 || koff % ((ptrdiff_t)gqa * 2) || voff < 0 || voff % 2) return false;
    const int cell = (int)(koff / ((ptrdiff_t)gqa * 2));
    if (cell >= n_kv || voff / 2 != cell || vdst->ne[0] != 1 || vdst->nb[1] != vview->nb[1] || !contiguous(kdst)) return false;
    if (!pi_k_attn_ggml_supported(hd, n_ctx, n_kv)) return false;
    if (!mask || mask->type != GGML_TYPE_F32 || !on_device(mask) || in_win(mask) || mask->ne[0] != n_kv || nrows(mask) != 1 || !contiguous(mask)) return false;
    if (!kq_scale || kq_scale->type != GGML_TYPE_F32 || !on_device(kq_scale) || in_win(kq_scale) || nelem(kq_scale) != 1) return false;
    if (kq->ne[0] != n_kv || kq->ne[2] != n_head || kqv->ne[0] != hd || kqv->ne[2] != n_head) return false;
    const ggml_tensor * resid = addr ? addr->src[1] : nullptr;
    if (addr && (!vec1(resid) || !on_device(resid) || in_win(resid) || nelem(resid) != wo->ne[1] || dev_ptr(resid) == dev_ptr(cont))) return false;
    if ((((uintptr_t)dev_ptr(F) | (uintptr_t)(mulw ? dev_ptr(mulw->src[1]) : nullptr) | (uintptr_t)dev_ptr(kview) | (uintptr_t)dev_ptr(vview)) & 15) != 0) return false;
    // ---- run ----
    ++g_stats.attn_blocks_fused;
    static float * qkv = nullptr;
    static size_t qkv_n = 0;
    const size_t need = (size_t)n_head * hd + 2 * (size_t)gqa;
    if (need > qkv_n) {
        if (qkv) { BK_PI(pi_sync()); pi_free(qkv); }
        qkv = (float *)pi_malloc(sizeof(float) * need);
        if (!qkv) die("attention buffer");
        qkv_n = need;
    }
    pi_norm na{0, 0.0f, nullptr, nullptr};
    if (mulw) { na.kind = 1; na.w = (const float *)dev_ptr(mulw->src[1]); memcpy(&na.eps, nrm->op_params, 4); }
    const void * Ws[3] = {dev_ptr(wq), dev_ptr(wk), dev_ptr(wv)};
    const int rows[3] = {n_head * hd, gqa, gqa};
    float * ys[3] = {qkv, qkv + (size_t)n_head * hd, qkv + (size_t)n_head * hd + gqa};
    BK_PI(pi_k_gemv_multi_f16(Ws, rows, 3, d, (const float *)dev_ptr(F), mulw ? &na : nullptr, ys, nullptr));
    BK_PI(pi_k_attn_ggml(ys[0], ys[1], ys[2], (const int32_t *)dev_ptr(pos), mode, powf(freq_base, -2.0f / n_dims), freq_scale, attn_factor,
                         dev_ptr(kview), dev_ptr(vview), n_head, n_head_kv, hd, n_ctx, n_kv, cell, (const float *)dev_ptr(kq_scale), (const float *)dev_ptr(mask),
                         (float *)dev_ptr(cont), nullptr));
    if (addr) BK_PI(pi_k_gemv(wo->type, dev_ptr(wo), (int)wo->ne[1], (int)wo->ne[0], (const float *)dev_ptr(cont), nullptr, PI_EPI_ADD, (const float *)dev_ptr(resid), nullptr,
                              (float *)dev_ptr(addr), nullptr));
    else      BK_PI(pi_k_gemv(wo->type, dev_ptr(wo), (int)wo->ne[1], (int)wo->ne[0], (const float *)dev_ptr(cont), nullptr, PI_EPI_NONE, nullptr, nullptr, (float *)dev_ptr(mmo), nullptr));
    return true;
}

bool try_fused_ffn(const ggml_tensor * axpy, const ggml_tensor * add, bool axpy_pending, bool execute);

// runs what is pending, in order.  Two peepholes: norm -> * w (-> + b) computed in place of one another is one launch, and a
// mat-vec whose ReLU is computed in place of it takes the ReLU as its epilogue.
void flush_pending() {
    if (g_pending.empty()) return;
    ++g_stats.windows_flushed;
    {   // an FFN block whose AXPY node joined the window, with or without the residual add behind it
        const ggml_tensor * axpy = nullptr; const ggml_tensor * add = nullptr;
        for (const PendingNode & p : g_pending) {
            if (!still_valid(p)) continue;
            if (p.t->op == GGML_OP_AXPY) { axpy = p.t; add = nullptr; }
            else if (axpy && !add && p.t->op == GGML_OP_ADD && p.t->src[0] == axpy) add = p.t;
            else if (axpy) { axpy = nullptr; break; }                 // something else came behind it: no block
        }
        if (axpy && try_fused_ffn(axpy, add, true, true)) {
            if (pi::check_launch("ggml_cuda_compute_forward") != PI_OK) die("kernel launch");
            return;
        }
    }
    std::vector<PendingNode> win;
    win.swap(g_pending);
    if (try_fused_attn(win)) return;
    for (size_t i = 0; i < win.size(); ++i) {
        if (!still_valid(win[i])) continue;
        ggml_tensor * n = win[i].t;
        if ((n->op == GGML_OP_RMS_NORM || n->op == GGML_OP_NORM) && i + 1 < win.size() && still_valid(win[i + 1])) {
            ggml_tensor * m = win[i + 1].t;
            if (m->op == GGML_OP_MUL && m->src[0] == n && on_device(m->src[1]) && dev_ptr(m) == dev_ptr(n)) {
                ggml_tensor * last = m; const float * bias = nullptr; size_t used = 2;
                if (i + 2 < win.size() && still_valid(win[i + 2])) {
                    ggml_tensor * a = win[i + 2].t;
                    if (a->op == GGML_OP_ADD && a->src[0] == m && on_device(a->src[1]) && dev_ptr(a) == dev_ptr(m)) { last = a; bias = (const float *)dev_ptr(a->src[1]); used = 3; }
                }
                float eps; memcpy(&eps, n->op_params, 4);
                hipLaunchKernelGGL(norm_affine_kernel, dim3(1), dim3(1024), 0, 0, (const float *)dev_ptr(n->src[0]), (const float *)dev_ptr(m->src[1]), bias,
                                   (float *)dev_ptr(last), (int)n->ne[0], eps, n->op == GGML_OP_NORM ? 1 : 0);
                i += used - 1;
                continue;
            }
        }
        if (n->op == GGML_OP_MUL_MAT && i + 1 < win.size() && still_valid(win[i + 1])) {
            ggml_tensor * r = win[i + 1].t;
            const ggml_tensor * a = n->src[0];
            if (r->op == GGML_OP_UNARY && r->src[0] == n && dev_ptr(r) == dev_ptr(n)) {
                BK_PI(pi_k_gemv(a->type, dev_ptr(a), (int)a->ne[1], (int)a->ne[0], (const float *)dev_ptr(n->src[1]), nullptr, PI_EPI_RELU, nullptr, nullptr,
                                (float *)dev_ptr(r), nullptr));
                ++i;
                continue;
            }
            // ... + residual, computed in place of the product (the attention output projection, llama.cpp:5022)
            if (r->op == GGML_OP_ADD && r->src[0] == n && dev_ptr(r) == dev_ptr(n) && on_device(r->src[1]) && !is_pending(r->src[1]) && r->src[1] != n->src[1] &&
                dev_ptr(r->src[1]) != dev_ptr(n)) {
                BK_PI(pi_k_gemv(a->type, dev_ptr(a), (int)a->ne[1], (int)a->ne[0], (const float *)dev_ptr(n->src[1]), nullptr, PI_EPI_ADD, (const float *)dev_ptr(r->src[1]), nullptr,
                                (float *)dev_ptr(r), nullptr));
                ++i;
                continue;
            }
        }
        if (!run_node(n)) {
            fprintf(stderr, "powerinfer-hip backend: deferred node '%s' (op %d) has a shape/type/stride this backend does not implement\n", n->name, (int)n->op);
            exit(1);
        }
    }
}

const PendingNode * find_pending(const ggml_tensor * t) { for (const PendingNode & p : g_pending) if (p.t == t && still_valid(p)) return &p; return nullptr; }

// The AXPY node that closes llm_build_ffn_sparse's sequence with every neuron on the device.  Returns false (nothing done) unless the
// pending window is exactly that block.  The node is asked about twice: when it arrives (execute false: does the window before it
// hold the block?  then it joins the window, so that the residual add behind it can follow), and when the window is flushed
// (axpy_pending true, execute true; add: the pending node behind it that adds the residual to its result, or null).
bool try_fused_ffn(const ggml_tensor * axpy, const ggml_tensor * add, bool axpy_pending, bool execute) {
    const ggml_tensor * down = axpy->src[0]; const ggml_tensor * cur = axpy->src[1]; const ggml_tensor * idx = axpy->src[2];
    if (axpy->src[3] != nullptr || !idx || !cur || !weight_on_device(down) || down->type != GGML_TYPE_F16 || !vec1(axpy) || axpy->backend != GGML_BACKEND_GPU || !on_device(axpy)) return false;
    size_t used = 0;
    auto take = [&](const ggml_tensor * t, int op) -> const ggml_tensor * {           // t is pending and has this operator
        if (!t || !find_pending(t) || t->op != op) return nullptr;
        ++used;
        return t;
    };
    // h = relu(gate) * up, or relu(up)
    const ggml_tensor * up_s = nullptr; const ggml_tensor * gate_s = nullptr;
    if (take(cur, GGML_OP_MUL)) {
        const ggml_tensor * ga = take(cur->src[0], GGML_OP_UNARY);
        if (!ga) return false;
        gate_s = take(ga->src[0], GGML_OP_MUL_MAT_SPARSE);
        up_s = take(cur->src[1], GGML_OP_MUL_MAT_SPARSE);
        if (!gate_s || !up_s || gate_s == up_s) return false;
    } else if (take(cur, GGML_OP_UNARY)) {
        up_s = take(cur->src[0], GGML_OP_MUL_MAT_SPARSE);
        if (!up_s) return false;
    } else return false;
    const ggml_tensor * X = up_s->src[1];
    if (up_s->src[2] != idx || (gate_s && (gate_s->src[1] != X || gate_s->src[2] != idx))) return false;
    const ggml_tensor * up = up_s->src[0]; const ggml_tensor * gate = gate_s ? gate_s->src[0] : nullptr;
    if (up->type != GGML_TYPE_F16 || (gate && gate->type != GGML_TYPE_F16)) return false;
    // predictor: idx = fc2 . relu(fc1 . P)
    if (!take(idx, GGML_OP_MUL_MAT)) return false;
    const ggml_tensor * fc2 = idx->src[0];
    const ggml_tensor * hid = take(idx->src[1], GGML_OP_UNARY);
    if (!hid) return false;
    const ggml_tensor * pre = take(hid->src[0], GGML_OP_MUL_MAT);
    if (!pre) return false;
    const ggml_tensor * fc1 = pre->src[0]; const ggml_tensor * P = pre->src[1];
    if (is_pending(P) || !on_device(P) || fc2->type != GGML_TYPE_F16) return false;
    // FFN input: norm(F) * w (+ b) still pending, or a vector that exists
    pi_norm nrm{0, 0.0f, nullptr, nullptr};
    const ggml_tensor * F = X;
    if (is_pending(X)) {
        const ggml_tensor * t = X;
        if (t->op == GGML_OP_ADD) { if (!take(t, GGML_OP_ADD) || !on_device(t->src[1])) return false; nrm.b = (const float *)dev_ptr(t->src[1]); t = t->src[0]; }
        if (!take(t, GGML_OP_MUL) || !on_device(t->src[1]) || is_pending(t->src[1])) return false;
        nrm.w = (const float *)dev_ptr(t->src[1]);
        t = t->src[0];
        if (t->op != GGML_OP_RMS_NORM && t->op != GGML_OP_NORM) return false;
        if (!take(t, t->op)) return false;
        nrm.kind = t->op == GGML_OP_RMS_NORM ? 1 : 2;
        memcpy(&nrm.eps, t->op_params, 4);
        if ((nrm.kind == 1 && nrm.b) || (nrm.kind == 2 && !nrm.b)) return false;
        F = t->src[0];
        if (is_pending(F) || !on_device(F)) return false;
    } else if (!on_device(X)) return false;
    size_t live = 0;
    for (const PendingNode & p : g_pending) live += still_valid(p) ? 1 : 0;
    if (used + (axpy_pending ? 1 : 0) + (add ? 1 : 0) != live) return false;                       // something else is pending: not the block
    const ggml_tensor * resid = add ? add->src[1] : nullptr;
    if (add && (add->src[0] != axpy || !vec1(add) || !on_device(add) || !vec1(resid) || !on_device(resid) || is_pending(resid) || nelem(resid) != nelem(axpy))) return false;
    const int d = (int)down->ne[0], ff = (int)down->ne[1], r = (int)fc1->ne[1];
    if (up->ne[0] != d || up->ne[1] != ff || (gate && (gate->ne[0] != d || gate->ne[1] != ff)) || fc2->ne[0] != r || fc2->ne[1] != ff || fc1->ne[0] != P->ne[0] ||
        X->ne[0] != d || idx->ne[0] != ff || axpy->ne[0] != d || !pi_k_sparse_ffn_supported(ff, r, d)) return false;
    if (!execute) return true;
    g_pending.clear();
    ++g_stats.ffn_blocks_fused;
    pi_workspace * ws = workspace(ff, d);
    // The rectified predictor layer goes to a buffer of this library's own: its node's buffer is dead in the host's plan once fc2 has
    // "run", and the allocator may have handed the same bytes to one of the vectors this launch writes (the logits, h).
    static float * hidden = nullptr;
    static int hidden_n = 0;
    if (r > hidden_n) {
        if (hidden) { BK_PI(pi_sync()); pi_free(hidden); }
        hidden = (float *)pi_malloc(sizeof(float) * (size_t)r);
        if (!hidden) die("predictor buffer");
        hidden_n = r;
    }
    BK_PI(pi_k_gemv(fc1->type, dev_ptr(fc1), r, (int)fc1->ne[0], (const float *)dev_ptr(P), nullptr, PI_EPI_RELU, nullptr, nullptr, hidden, nullptr));
    BK_PI(pi_k_sparse_ffn(dev_ptr(fc2), ff, r, hidden, g_threshold, dev_ptr(up), gate ? dev_ptr(gate) : nullptr, dev_ptr(down), d, (const float *)dev_ptr(F),
                          nrm.kind ? &nrm : nullptr, add ? PI_EPI_ADD : PI_EPI_NONE, add ? (const float *)dev_ptr(resid) : nullptr, nullptr,
                          (float *)dev_ptr(add ? add : axpy), (float *)dev_ptr(idx), (float *)dev_ptr(cur), nullptr, ws, nullptr));
    return true;
}

}  // namespace

extern "C" {

void ggml_init_cublas(void) {
    std::lock_guard<std::mutex> g(g_mu);
    if (g_loaded) return;
    g_loaded = pi_init(0) == PI_OK;
    { const char * nf = getenv("GGML_CUDA_NO_FUSION"); g_fuse = !(nf && nf[0] == '1'); }
    if (!g_loaded) fprintf(stderr, "powerinfer-hip backend: no usable HIP device (%s)\n", pi_last_error());
}
bool ggml_cublas_loaded(void) { return g_loaded; }

void * ggml_cuda_host_malloc(size_t size) {
    if (getenv("GGML_CUDA_NO_PINNED")) return nullptr;
    void * p = nullptr;
    if (hipHostMalloc(&p, size, hipHostMallocDefault) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
    return p;
}
void ggml_cuda_host_free(void * ptr) { if (ptr) BK_HIP(hipHostFree(ptr)); }

bool ggml_cuda_can_mul_mat(const struct ggml_tensor * src0, const struct ggml_tensor * src1, struct ggml_tensor * dst) {
    const int64_t ne10 = src1->ne[0], ne0 = dst->ne[0], ne1 = dst->ne[1];
    return (src0->type == GGML_TYPE_F32 || src0->type == GGML_TYPE_F16 || src0->type == GGML_TYPE_Q4_0) &&
           src1->type == GGML_TYPE_F32 && dst->type == GGML_TYPE_F32 && ne0 >= 32 && ne1 >= 32 && ne10 >= 32;   // ggml-cuda.cu:8714-8727
}
void ggml_cuda_set_tensor_split(const float * tensor_split) { (void)tensor_split; }       // one GPU
void ggml_cuda_set_main_device(int main_device) { if (main_device != 0) fprintf(stderr, "powerinfer-hip backend: single-GPU build, main device stays 0\n"); }
void ggml_cuda_set_mul_mat_q(bool mul_mat_q) { (void)mul_mat_q; }

void ggml_cuda_transform_tensor(void * data, struct ggml_tensor * tensor) {
    const size_t n = nbytes(tensor);
    void * p = pi_malloc(n); if (!p) die("ggml_cuda_transform_tensor");
    BK_PI(pi_memcpy_h2d(p, data, n));
    tensor->extra = new_extra(p, true);
}
void ggml_cuda_alloc_tensor(struct ggml_tensor * tensor) {
    void * p = pi_malloc(nbytes(tensor)); if (!p) die("ggml_cuda_alloc_tensor");
    tensor->extra = new_extra(p, true);
}
void ggml_cuda_free_data(struct ggml_tensor * tensor) {
    if (!tensor || !tensor->extra) return;
    flush_pending();
    Extra * e = (Extra *)tensor->extra;
    tensor->extra = nullptr;
    if (is_ring(e)) return;                        // a per-evaluation address: nothing is owned
    if (e->owned && e->data_device[0]) pi_free(e->data_device[0]);
    delete e;
}
// copies src's host row into dst's current device pointer; the caller then bumps the pointer it got from
// ggml_cuda_get_data_pp to stream the bucket's rows into a compact matrix (llama.cpp:2898-2967)
void ggml_cuda_cpy_1d(struct ggml_tensor * dst, const struct ggml_tensor * src) {
    BK_PI(pi_memcpy_h2d(dev_ptr(dst), src->data, nbytes(src)));
}
void ** ggml_cuda_get_data_pp(struct ggml_tensor * tensor) { return &((Extra *)tensor->extra)->data_device[0]; }

void ggml_cuda_assign_buffers(struct ggml_tensor * tensor) { if (tensor) assign(tensor, true, false, false); }
void ggml_cuda_assign_buffers_no_scratch(struct ggml_tensor * tensor) { assign(tensor, false, false, false); }
void ggml_cuda_assign_buffers_force_inplace(struct ggml_tensor * tensor) { assign(tensor, false, true, false); }
void ggml_cuda_assign_buffers_no_alloc(struct ggml_tensor * tensor) { assign(tensor, true, false, true); }
// ggml-cuda.cu:9119-9146.  The host passes the tensor's offset inside its own compute buffer, whose layout the device scratch
// mirrors.  For a tensor that shares its parent's memory the parent's device address wins: the parent may live outside the
// scratch (a view of the KV cache), where the host-side offset means nothing -- the reference stores such an address without
// looking at it, so an offset beyond the scratch is accepted here as long as no kernel is ever pointed at it (checked at use).
void ggml_cuda_assign_scratch_offset(struct ggml_tensor * tensor, size_t offset) {
    if (g_scratch_size == 0) return;
    std::lock_guard<std::mutex> g(g_mu);
    char * base = scratch_base();
    if (Extra * shared = inplace_extra(tensor, false)) { tensor->extra = shared; return; }
    Extra * e = ring_extra(base + offset);
    e->outside_scratch = offset > g_scratch_size || nbytes(tensor) > g_scratch_size - offset;
    tensor->extra = e;
}
void ggml_cuda_set_scratch_size(size_t scratch_size) {
    if (scratch_size > g_scratch_size) ggml_cuda_free_scratch();
    g_scratch_size = scratch_size;
}
void ggml_cuda_free_scratch(void) {
    flush_pending();
    std::lock_guard<std::mutex> g(g_mu);
    if (g_scratch) { pi_free(g_scratch); g_scratch = nullptr; }
    if (g_arena.base) { pi_sync(); pi_free(g_arena.base); g_arena.base = nullptr; g_arena.cap = 0; }
    g_scratch_offset = 0;
}
void ggml_cuda_copy_to_device(struct ggml_tensor * tensor) {
    flush_pending();
    h2d(dev_ptr(tensor), tensor->data, nbytes(tensor));
}
void ggml_cuda_copy_to_host(struct ggml_tensor * tensor) {
    flush_pending();
    BK_PI(pi_sync());
    BK_PI(pi_memcpy_d2h(tensor->data, dev_ptr(tensor), nbytes(tensor)));
}

int ggml_cuda_get_device_count(void) { int n = 0; if (hipGetDeviceCount(&n) != hipSuccess) { (void)hipGetLastError(); return 0; } return n; }
void ggml_cuda_get_device_description(int device, char * description, size_t description_size) {
    hipDeviceProp_t p;
    if (hipGetDeviceProperties(&p, device) != hipSuccess) { (void)hipGetLastError(); snprintf(description, description_size, "unknown"); return; }
    snprintf(description, description_size, "%s", p.gcnArchName);
}
size_t ggml_cuda_get_free_memory(int device) {
    (void)device;
    size_t f = 0, t = 0;
    BK_HIP(hipMemGetInfo(&f, &t));
    return f;
}
void ggml_cuda_set_device_constants(float sparse_pred_threshold) { g_threshold = sparse_pred_threshold; }

bool ggml_cuda_compute_forward(struct ggml_compute_params * params, struct ggml_tensor * tensor) {
    if (!g_loaded) return false;
    const ggml_tensor * s0 = tensor->src[0];
    const bool src0_on_device = s0 != nullptr && s0->backend != GGML_BACKEND_CPU;
    const bool any_on_device = tensor->backend == GGML_BACKEND_GPU || src0_on_device || (tensor->src[1] != nullptr && tensor->src[1]->backend == GGML_BACKEND_GPU);
    // weights not on the device: the sparse operators run on the CPU with the sparsity (ggml-cuda.cu:9226-9230)
    if ((!src0_on_device && (tensor->op == GGML_OP_MUL_MAT_SPARSE || tensor->op == GGML_OP_AXPY)) || (!any_on_device && tensor->op != GGML_OP_MUL_MAT)) return false;
    if (tensor->op == GGML_OP_MUL_MAT) {
        if (tensor->src[0]->ne[3] != tensor->src[1]->ne[3]) return false;
        // host-resident operands: only a product large enough to pay for the transfer is taken (ggml-cuda.cu:9278-9282)
        if (!any_on_device && !ggml_cuda_can_mul_mat(tensor->src[0], tensor->src[1], tensor)) return false;
    }
    switch (tensor->op) {
        case GGML_OP_MUL_MAT: case GGML_OP_MUL_MAT_SPARSE: case GGML_OP_AXPY: case GGML_OP_ADD: case GGML_OP_MUL:
        case GGML_OP_SCALE: case GGML_OP_RMS_NORM: case GGML_OP_NORM: case GGML_OP_SOFT_MAX: case GGML_OP_ROPE:
        case GGML_OP_CPY: case GGML_OP_CONT: case GGML_OP_DUP: case GGML_OP_GET_ROWS:
        case GGML_OP_RESHAPE: case GGML_OP_VIEW: case GGML_OP_PERMUTE: case GGML_OP_TRANSPOSE:
            break;
        case GGML_OP_UNARY:
            if (tensor->op_params[0] != GGML_UNARY_OP_RELU) return false;
            break;
        default:
            return false;
    }
    if (params->ith != 0) return true;
    if (params->type == GGML_TASK_INIT || params->type == GGML_TASK_FINALIZE) return true;
    const bool view = tensor->op == GGML_OP_RESHAPE || tensor->op == GGML_OP_VIEW || tensor->op == GGML_OP_PERMUTE || tensor->op == GGML_OP_TRANSPOSE;
    if (!view) {                                         // views do nothing and neither join nor break the window
        if (deferrable(tensor)) { defer(tensor); return true; }
        if (!g_pending.empty()) {
            // the AXPY node that completes an FFN block joins the window: the block runs when the window is flushed, with the residual
            // add as its epilogue if that is what comes next
            if (g_fuse && tensor->op == GGML_OP_AXPY && try_fused_ffn(tensor, nullptr, false, false)) { defer(tensor); return true; }
            flush_pending();
            if (deferrable(tensor)) { defer(tensor); return true; }      // its operands exist now: it may open the next window
        }
    }
    const bool ok = run_node(tensor);
    if (!ok) {
        // the phase protocol has no way to hand a node back after INIT was claimed: refuse loudly rather than compute wrongly
        fprintf(stderr, "powerinfer-hip backend: node '%s' (op %d) has a shape/type/stride this backend does not implement\n", tensor->name, (int)tensor->op);
        exit(1);
    }
    if (pi::check_launch("ggml_cuda_compute_forward") != PI_OK) die("kernel launch");
    return true;
}

ggml_backend_t ggml_backend_cuda_init(void) { return nullptr; }

void pi_ggml_backend_get_stats(pi_ggml_backend_stats * out) { if (out) *out = g_stats; }
void pi_ggml_backend_set_fusion(int enable) { flush_pending(); g_fuse = enable != 0; }

}  // extern "C"
