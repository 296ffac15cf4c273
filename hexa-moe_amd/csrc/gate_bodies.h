// Device code of the gate's backward products (see gate.hip), shared with the kernel that runs several small tasks
// in one launch (batch.hip).
#pragma once
#include "small_tasks.h"

namespace hexa {
namespace {

typedef __attribute__((ext_vector_type(16))) float f32x16;

constexpr int GT = 32;          // tokens per workgroup (forward)
constexpr int FWD_NB = 6;       // chunks of 8 contraction indices a wavefront of the forward kernel loads per trip
constexpr int BWD_TB = 64;      // tokens per chunk of the backward tasks (and per dwg partial sum)

__device__ __forceinline__ f32x16 zero16() {
    f32x16 z;
#pragma unroll
    for (int v = 0; v < 16; ++v) z[v] = 0.f;
    return z;
}

__device__ __attribute__((aligned(32))) unsigned int g_gate_zeros[8];   // stays zero: what masked lanes load

// N consecutive elements (N = 4 or 8) as floats; zeros when !ok.  Masked lanes load from a block of
// zeros instead of branching around the load, so that a run of loads is issued back to back and
// their latencies overlap.
template <typename T, int N> struct LoadN {   // 16-bit types
    static __device__ __forceinline__ void run(const T* p, bool ok, float (&o)[N]) {
        const T* src = ok ? p : reinterpret_cast<const T*>(g_gate_zeros);
        union { unsigned u[N / 2]; T h[N]; } v;
        if (N == 8) {
            const uint4 w = *reinterpret_cast<const uint4*>(src);
            v.u[0] = w.x; v.u[1] = w.y; v.u[N / 2 - 2] = w.z; v.u[N / 2 - 1] = w.w;
        } else {
            const uint2 w = *reinterpret_cast<const uint2*>(src);
            v.u[0] = w.x; v.u[1] = w.y;
        }
#pragma unroll
        for (int i = 0; i < N; ++i) o[i] = (float)v.h[i];
    }
};
template <int N> struct LoadN<float, N> {
    static __device__ __forceinline__ void run(const float* p, bool ok, float (&o)[N]) {
        const float* src = ok ? p : reinterpret_cast<const float*>(g_gate_zeros);
#pragma unroll
        for (int q = 0; q < N; q += 4) {
            const float4 v = *reinterpret_cast<const float4*>(src + q);
            o[q] = v.x; o[q + 1] = v.y; o[q + 2] = v.z; o[q + 3] = v.w;
        }
    }
};
// All of v[] has arrived before anything behind this point runs: keeps the scheduler from sinking each
// load next to its first use (which would pay one memory latency per load instead of one per batch).
typedef __attribute__((ext_vector_type(4))) float f32x4;
template <int N> __device__ __forceinline__ void arrive(float (&v)[N][4]) {
    static_assert(N == 8 || N == 16, "batches of 8 or 16");
    f32x4 w[N];
#pragma unroll
    for (int i = 0; i < N; ++i) { w[i].x = v[i][0]; w[i].y = v[i][1]; w[i].z = v[i][2]; w[i].w = v[i][3]; }
    if constexpr (N == 16)
        asm volatile("" : "+v"(w[0]), "+v"(w[1]), "+v"(w[2]), "+v"(w[3]), "+v"(w[4]), "+v"(w[5]), "+v"(w[6]), "+v"(w[7]),
                          "+v"(w[8]), "+v"(w[9]), "+v"(w[10]), "+v"(w[11]), "+v"(w[12]), "+v"(w[13]), "+v"(w[14]), "+v"(w[15]));
    else
        asm volatile("" : "+v"(w[0]), "+v"(w[1]), "+v"(w[2]), "+v"(w[3]), "+v"(w[4]), "+v"(w[5]), "+v"(w[6]), "+v"(w[7]));
#pragma unroll
    for (int i = 0; i < N; ++i) { v[i][0] = w[i].x; v[i][1] = w[i].y; v[i][2] = w[i].z; v[i][3] = w[i].w; }
}
__device__ __forceinline__ float load1(const float* p, bool ok) {
    return *(ok ? p : reinterpret_cast<const float*>(g_gate_zeros));
}
template <typename T> __device__ __forceinline__ void store4(T* p, float a, float b, float c, float d);
template <> __device__ __forceinline__ void store4<float>(float* p, float a, float b, float c, float d) {
    *reinterpret_cast<float4*>(p) = make_float4(a, b, c, d);
}
template <typename T16> __device__ __forceinline__ void store4(T16* p, float a, float b, float c, float d) {
    union { uint2 u; T16 h[4]; } v;
    v.h[0] = (T16)a; v.h[1] = (T16)b; v.h[2] = (T16)c; v.h[3] = (T16)d;
    *reinterpret_cast<uint2*>(p) = v.u;
}

// ---- backward: one task per WAVEFRONT ---------------------------------------------------------------------
// The fp32 MFMA is slow (64 cycles for 32x32x2), the products are small, and a launch is over when its busiest
// SIMD is: what matters is that every SIMD of the chip gets the same number of MFMAs.  So the work is cut into
// tasks of equal length -- 128 MFMAs at 32 experts -- one per wavefront, four wavefronts (one per SIMD of a CU)
// to a workgroup, nothing shared between them:
//   dx task  (chunk, g): dx[64 tokens of the chunk][columns 128g .. 128g+127], two 32-token blocks one after the
//                        other with the wavefront's slice of wg kept in registers (re-read per block above 32
//                        experts)
//   dwg task (chunk, eb, g): partial dwg[experts 32eb .. 32eb+31][columns 128g ..] over the chunk's 64 tokens
// (with workgroups of three busy wavefronts and a fourth idle, and twice as many half-length dx tasks, the same
// kernel took 28 us instead of 17 at 18432 tokens, d = 384, 32 experts: the MFMAs alone are 6.6 us of the chip).
template <typename T>
__device__ __forceinline__ void gate_dx_task(int chunk, int g, T* __restrict__ dx, const float* __restrict__ dl,
                                             const float* __restrict__ wg, int num_tokens, int d, int E) {
    const int lane = threadIdx.x & 63;
    const int r = lane & 31, h = lane >> 5;
    const bool single = E <= 32;               // one pass over the experts: the wg slice is loaded once
    const int col = g * 128 + 4 * r;
    const bool col_ok = col < d;
    float b[16][4];
    auto load_b = [&](int e0) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int e = e0 + 16 * h + i;
            LoadN<float, 4>::run(wg + (size_t)(e < E ? e : 0) * d + (col_ok ? col : 0), col_ok && e < E, b[i]);
        }
    };
    if (single) load_b(0);
    for (int tb = 0; tb < BWD_TB / 32; ++tb) {
        const int t0 = chunk * BWD_TB + tb * 32;
        if (t0 >= num_tokens) break;
        const bool tok_ok = t0 + r < num_tokens;
        const float* drow = dl + (size_t)(tok_ok ? t0 + r : 0) * E;
        f32x16 acc[4] = {zero16(), zero16(), zero16(), zero16()};
        for (int e0 = 0; e0 < E; e0 += 32) {
            // this lane's contraction indices: experts e0 + 16h + 0..15
            float a[16];
            if ((E & 3) == 0) {   // rows are 16-byte aligned: four float4 loads
#pragma unroll
                for (int i = 0; i < 16; i += 4) {
                    const int e = e0 + 16 * h + i;
                    float v[4];
                    LoadN<float, 4>::run(drow + (e < E ? e : 0), tok_ok && e < E, v);
                    a[i] = v[0]; a[i + 1] = v[1]; a[i + 2] = v[2]; a[i + 3] = v[3];
                }
            } else {
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int e = e0 + 16 * h + i;
                    a[i] = load1(drow + (e < E ? e : 0), tok_ok && e < E);
                }
            }
            if (!single) load_b(e0);
            if (!single || tb == 0) arrive(b);
#pragma unroll
            for (int i = 0; i < 16; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[i][j], acc[j], 0, 0, 0);
        }
        if (col_ok) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int t = t0 + 8 * (v >> 2) + 4 * h + (v & 3);
                if (t < num_tokens) store4<T>(dx + (size_t)t * d + col, acc[0][v], acc[1][v], acc[2][v], acc[3][v]);
            }
        }
    }
}

template <typename T>
__device__ __forceinline__ void gate_dwg_task(int chunk, int e_block, int g, float* __restrict__ part,
                                              const float* __restrict__ dl, const T* __restrict__ x, int num_tokens,
                                              int d, int E) {
    const int lane = threadIdx.x & 63;
    const int r = lane & 31, h = lane >> 5;
    const int t0 = chunk * BWD_TB;
    const int e0 = e_block * 32;
    const bool exp_ok = e0 + r < E;
    float* out = part + (size_t)chunk * E * d;
    constexpr int TRIPS = BWD_TB / 16;      // 8 MFMA steps (16 tokens) per trip
    const int col = g * 128 + 4 * r;
    const bool col_ok = col < d;
    f32x16 acc[4] = {zero16(), zero16(), zero16(), zero16()};
    // two trips of loads in flight: the next trip's loads are issued before this trip's products
    float a[2][8], b[2][8][4];
    auto load_trip = [&](int trip, float (&av)[8], float (&bv)[8][4]) {
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int t = t0 + 2 * (8 * trip + u) + h;    // this lane's contraction index: one token
            const bool ok = t < num_tokens;
            av[u] = load1(dl + (size_t)(ok ? t : 0) * E + (exp_ok ? e0 + r : 0), ok && exp_ok);
            LoadN<T, 4>::run(x + (size_t)(ok ? t : 0) * d + (col_ok ? col : 0), ok && col_ok, bv[u]);
        }
    };
    load_trip(0, a[0], b[0]);
#pragma unroll
    for (int trip = 0; trip < TRIPS; ++trip) {
        if (trip + 1 < TRIPS) load_trip(trip + 1, a[(trip + 1) & 1], b[(trip + 1) & 1]);
        arrive(b[trip & 1]);
#pragma unroll
        for (int u = 0; u < 8; ++u)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[trip & 1][u], b[trip & 1][u][j], acc[j], 0, 0, 0);
    }
    if (col_ok) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int e = e0 + 8 * (v >> 2) + 4 * h + (v & 3);
            if (e < E) store4<float>(out + (size_t)e * d + col, acc[0][v], acc[1][v], acc[2][v], acc[3][v]);
        }
    }
}

// dx (when non-null) and the dwg partial sums (when `part` is non-null): each product alone leaves most of the chip
// waiting on memory latency, and they share nothing but their inputs.  Tasks are numbered chunk by chunk -- the dx
// tasks of 64 tokens, then their dwg tasks -- so the dlogits rows both read are fetched once.  `block` = four tasks.
template <typename T>
__device__ __forceinline__ void gate_bwd_body(const GateBwdK& p, int block) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int task = block * 4 + wave;
    if (task >= p.ntasks) return;
    const int groups = (p.d + 127) >> 7, e_blocks = (p.E + 31) >> 5;
    const int n_dx = p.dx ? groups : 0, n_dwg = p.part ? groups * e_blocks : 0;
    const int chunk = task / (n_dx + n_dwg), role = task - chunk * (n_dx + n_dwg);
    if (role < n_dx) {
        gate_dx_task<T>(chunk, role, reinterpret_cast<T*>(p.dx), p.dl, p.wg, p.T, p.d, p.E);
    } else {
        const int q = role - n_dx;
        gate_dwg_task<T>(chunk, q / groups, q - (q / groups) * groups, p.part, p.dl, reinterpret_cast<const T*>(p.x), p.T, p.d,
                         p.E);
    }
}

// dwg = sum of the partial results, in a fixed order: a workgroup takes 16 float4 columns; each of its
// 16 thread groups sums a contiguous range of the partials, then the 16 group sums are added in order.
__device__ __forceinline__ void dwg_reduce_body(const DwgReduceK& p, int block) {
    __shared__ float4 sums[16][16];
    const int c = threadIdx.x & 15, grp = threadIdx.x >> 4;
    const long i = (long)block * 16 + c;
    const int b0 = (int)((long)p.nparts * grp / 16), b1 = (int)((long)p.nparts * (grp + 1) / 16);
    float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
    if (i < p.n4) {
#pragma unroll 6
        for (int b = b0; b < b1; ++b) {
            const float4 v = reinterpret_cast<const float4*>(p.part)[(size_t)b * p.n4 + i];
            s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
        }
    }
    sums[grp][c] = s;
    __syncthreads();
    if (grp == 0 && i < p.n4) {
        float4 t = sums[0][c];
#pragma unroll
        for (int g = 1; g < 16; ++g) { const float4 v = sums[g][c]; t.x += v.x; t.y += v.y; t.z += v.z; t.w += v.w; }
        reinterpret_cast<float4*>(p.dwg)[i] = t;
    }
}

}  // namespace
}  // namespace hexa
