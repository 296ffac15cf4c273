// ESS (per-expert bias-gradient sum) and the elementwise GELU backward for gfx950.
//
// ESS is a gathered column sum and is bound by HBM bandwidth: one 256-thread workgroup owns one
// (expert, strip of 8 x 16-byte columns) and streams that expert's token rows, slot after slot.  In a
// wavefront 8 lanes cover the strip of one row and the 8 lane groups take 8 consecutive rows, so
// every load instruction moves eight 128-byte row pieces.  fp32 partial sums stay in registers; the
// 8 row groups of a wavefront are folded with wavefront shuffles (xor 8, 16, 32), the 4 wavefronts
// through LDS.  Each result is written once, in a fixed order: no atomics, no zero-initialised
// output, bit-reproducible.
//
// Replaces the ESS task of fused_grad_bias_kernel_vectorized_* (kernels/fused_ops_full.cu:372-431).
#include <algorithm>

#include <mutex>

#include "small_bodies.h"

namespace hexa {
namespace {

template <typename T>
__global__ __launch_bounds__(256) void ess_kernel(EssK p) { ess_body<T>(p, blockIdx.x); }

__global__ __launch_bounds__(256) void ess_fold_kernel(EssFoldK p) { ess_fold_body(p, blockIdx.x); }

template <typename T>
int launch_ess_t(const EssArgs& a, hipStream_t st) {
    constexpr int STRIP = 8 * Vec16<T>::N;
    if (a.out_dim % Vec16<T>::N)
        HEXA_FAIL(HEXA_ERR_UNSUPPORTED, "ess: out_dim must be a multiple of %d (got %d)", Vec16<T>::N, a.out_dim);
    EssK p;
    p.dy = a.dy; p.db = a.db; p.token_ids = a.r.token_ids; p.offsets = a.r.offsets;
    p.T = a.r.T; p.k = a.r.k; p.E = a.r.E; p.N = a.out_dim;
    p.dy_slot_rows = a.dy_per_slot ? a.r.T : 0;
    p.accumulate = a.accumulate; p.db_dt = a.db_dt;
    // Long token lists are cut into up to 8 parts that run as separate workgroups (the partial sums go
    // through the caller's scratch and are folded in a fixed order): the kernel is otherwise as slow as
    // the walk over the busiest expert's list.
    const long per_part = (long)a.r.E * a.out_dim;
    const long avg_rows = a.r.E > 0 ? (long)a.r.T * a.r.k / a.r.E : 0;
    int splits = 1;
    if (a.ws && per_part > 0 && avg_rows >= 256) splits = (int)std::min<long>(8, a.ws_floats / per_part);
    if (splits < 2) splits = 1;
    p.ws = a.ws; p.splits = splits;
    p.gx = div_up(a.out_dim, STRIP); p.gy = a.r.E;
    SmallTask t;
    t.kind = TASK_ESS; t.ess = p; t.blocks = p.gx * p.gy * splits;
    if (t.blocks == 0) return HEXA_OK;
    if (!defer_task(defer_targets().ess, t, a.dy_dt)) {
        hipLaunchKernelGGL((ess_kernel<T>), dim3(t.blocks), dim3(256), 0, st, p);
        HEXA_CHECK_LAUNCH("ess");
    }
    if (splits > 1) {
        SmallTask f;
        f.kind = TASK_ESS_FOLD; f.ess_fold = EssFoldK{a.db, a.ws, per_part, splits, a.db_dt, a.accumulate};
        f.blocks = (int)((per_part + 255) / 256);
        if (!defer_task(defer_targets().ess_fold, f)) {
            hipLaunchKernelGGL(ess_fold_kernel, dim3(f.blocks), dim3(256), 0, st, f.ess_fold);
            HEXA_CHECK_LAUNCH("ess_fold");
        }
    }
    return HEXA_OK;
}

// dy1 = dy2 * gelu'(y1),  gelu'(x) = Phi(x) + x * phi(x)
template <typename T>
__global__ __launch_bounds__(256) void gelu_bwd_kernel(T* __restrict__ dy1, const T* __restrict__ dy2,
                                                       const T* __restrict__ y1, int64_t n) {
    constexpr int V = Vec16<T>::N;
    const int64_t nv = n / V;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < nv; i += stride) {
        union { uint4 u; T e[V]; } g, y, o;
        g.u = reinterpret_cast<const uint4*>(dy2)[i];
        y.u = reinterpret_cast<const uint4*>(y1)[i];
#pragma unroll
        for (int j = 0; j < V; ++j) {
            const float x = Cvt<T>::to_f(y.e[j]);
            const float cdf = 0.5f * (1.0f + erff(x * 0.70710678118654752440f));
            const float pdf = 0.39894228040143267794f * __expf(-0.5f * x * x);
            o.e[j] = Cvt<T>::from_f(Cvt<T>::to_f(g.e[j]) * (cdf + x * pdf));
        }
        reinterpret_cast<uint4*>(dy1)[i] = o.u;
    }
    // tail (n not a multiple of the vector width)
    for (int64_t i = nv * V + (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const float x = Cvt<T>::to_f(y1[i]);
        const float cdf = 0.5f * (1.0f + erff(x * 0.70710678118654752440f));
        const float pdf = 0.39894228040143267794f * __expf(-0.5f * x * x);
        dy1[i] = Cvt<T>::from_f(Cvt<T>::to_f(dy2[i]) * (cdf + x * pdf));
    }
}

template <typename T>
int launch_gelu_bwd_t(void* dy1, const void* dy2, const void* y1, int64_t n, hipStream_t st) {
    if (n == 0) return HEXA_OK;
    int64_t blocks = (n / Vec16<T>::N + 255) / 256;
    if (blocks < 1) blocks = 1;
    if (blocks > 256 * 16) blocks = 256 * 16;
    hipLaunchKernelGGL((gelu_bwd_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, st, (T*)dy1, (const T*)dy2,
                       (const T*)y1, n);
    HEXA_CHECK_LAUNCH("gelu_bwd");
    return HEXA_OK;
}

template <typename T>
__global__ __launch_bounds__(256) void sum_slots_kernel(SumSlotsK p) { sum_slots_body<T>(p, blockIdx.x); }

template <typename T>
int launch_sum_slots_t(void* out, const void* ws, int64_t n, int nws, const void* extra, int dt, hipStream_t st) {
    if (n == 0 || (nws == 0 && !extra)) return HEXA_OK;
    if (n % Vec16<T>::N) HEXA_FAIL(HEXA_ERR_UNSUPPORTED, "sum_slots: size must be a multiple of the vector width");
    int64_t blocks = (n / Vec16<T>::N + 255) / 256;
    if (blocks > 256 * 16) blocks = 256 * 16;
    SmallTask t;
    t.kind = TASK_SUM_SLOTS; t.sum_slots = SumSlotsK{out, ws, n, nws, extra, (int)blocks}; t.blocks = (int)blocks;
    if (!defer_task(defer_targets().sum_slots, t, dt)) {
        hipLaunchKernelGGL((sum_slots_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, st, t.sum_slots);
        HEXA_CHECK_LAUNCH("sum_slots");
    }
    return HEXA_OK;
}

}  // namespace

int launch_sum_slots(void* out, const void* ws, int64_t n, int nws, int dt, hipStream_t st, const void* extra) {
    if (dt == HEXA_F32) return launch_sum_slots_t<float>(out, ws, n, nws, extra, dt, st);
    if (dt == HEXA_BF16) return launch_sum_slots_t<__bf16>(out, ws, n, nws, extra, dt, st);
    return launch_sum_slots_t<_Float16>(out, ws, n, nws, extra, dt, st);
}

int launch_ess(const EssArgs& a, hipStream_t st) {
    if (a.dy_dt == HEXA_F32) return launch_ess_t<float>(a, st);
    if (a.dy_dt == HEXA_BF16) return launch_ess_t<__bf16>(a, st);
    return launch_ess_t<_Float16>(a, st);
}

// ---- ESS without any allocation by anyone ---------------------------------------------------------------
// The partial sums of the split walk live in a file-scope device array instead of caller scratch.  Every
// device the library runs on holds its own copy at its own address; the array's name is only a host-side
// handle, so the device address is looked up once per device (with that device current) and kept.
constexpr int64_t ESS_SCRATCH_FLOATS = HEXA_ESS_NOALLOC_MAX_FLOATS;   // 8 MiB per device
constexpr int ESS_MAX_DEVICES = 64;
static __device__ __align__(256) float scratch[ESS_SCRATCH_FLOATS];
static float* g_scratch_ptr[ESS_MAX_DEVICES];
static std::mutex g_scratch_mutex;   // the first calls of several threads on one device look the address up once

int ess_scratch_for_current_device(float** out) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= ESS_MAX_DEVICES)
        HEXA_FAIL(HEXA_ERR_LAUNCH, "hexa_ess_noalloc: cannot identify the current device");
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        float* ptr = nullptr;
        const hipError_t e = hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr)
            HEXA_FAIL(HEXA_ERR_LAUNCH, "hexa_ess_noalloc: hipGetSymbolAddress failed: %s", hipGetErrorString(e));
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return HEXA_OK;
}

int launch_ess_noalloc(EssArgs a, hipStream_t st) {
    const int64_t need = (int64_t)8 * a.r.E * a.out_dim;
    if (need > ESS_SCRATCH_FLOATS)
        HEXA_FAIL(HEXA_ERR_UNSUPPORTED,
                  "hexa_ess_noalloc: 8*num_experts*out_dim = %lld floats exceeds the built-in scratch of %lld floats; "
                  "use hexa_ess with caller scratch", (long long)need, (long long)ESS_SCRATCH_FLOATS);
    float* ptr = nullptr;
    if (int rc = ess_scratch_for_current_device(&ptr)) return rc;
    // every partial sum the fold reads is written by this call's own workgroups: nothing to clear
    a.ws = ptr;
    a.ws_floats = need;
    return launch_ess(a, st);
}

int launch_gelu_bwd(void* dy1, const void* dy2, const void* y1, int64_t n, int dt, hipStream_t st) {
    if (dt == HEXA_F32) return launch_gelu_bwd_t<float>(dy1, dy2, y1, n, st);
    if (dt == HEXA_BF16) return launch_gelu_bwd_t<__bf16>(dy1, dy2, y1, n, st);
    return launch_gelu_bwd_t<_Float16>(dy1, dy2, y1, n, st);
}

}  // namespace hexa
