// The gate's linear layer in fp32 on the matrix cores (v_mfma_f32_32x32x2_f32: fp32 multiply, fp32
// accumulate), forward and backward, for token tensors of any supported type:
//   logits[t][e] = sum_c x[t][c] * wg[e][c]                 (gate_fwd_kernel)
//   dx[t][c]     = sum_e dlogits[t][e] * wg[e][c]           (gate_bwd_kernel, dx tasks)
//   dwg[e][c]    = sum_t dlogits[t][e] * x[t][c]            (gate_bwd_kernel, dwg tasks + gate_dwg_reduce_kernel)
// These are skinny products (E is a few dozen): little memory traffic, and at 64 cycles per fp32 MFMA the matrix
// pipelines are what bounds them -- at 18432 tokens, d = 384 and 32 experts each product is 110592 MFMAs, 3.3 us
// of the whole chip.  Operands go from global memory straight to registers.  The MFMA takes ONE contraction index per lane (lane l: row or
// column l%32, index l/32), and which two indices one MFMA pairs is free as long as both operands
// agree -- so a lane loads 8 (or 16) consecutive contraction indices in one go and feeds them to
// consecutive MFMAs.  Where the fast output dimension is the token/gate row (dx, dwg), lane n owns 4
// consecutive columns of a 128-column group, one accumulator per column offset: loads and stores
// are whole 8- or 16-byte pieces.
//
// Replaces LinearTopKGate.forward with fp32_gate (gates/top.py:17-19: a cast of x to fp32 plus a
// skinny fp32 GEMM) and what autograd derives from it.
#include "gate_bodies.h"

namespace hexa {
namespace {

// ---- forward: 32 tokens per workgroup, the model dimension split over the 4 wavefronts ---------------
template <typename T>
__global__ __launch_bounds__(256) void gate_fwd_kernel(float* __restrict__ logits, const T* __restrict__ x,
                                                       const float* __restrict__ wg, int num_tokens, int d, int E) {
    __shared__ float part[4][16][64];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 31, h = lane >> 5;
    const int t0 = blockIdx.x * GT;
    const int pieces = d >> 3;                       // 8 contraction indices per piece
    const int chunks = (pieces + 1) >> 1;            // a chunk = one piece per half-wavefront
    const int c0 = (chunks * wave) >> 2, c1 = (chunks * (wave + 1)) >> 2;
    const bool tok_ok = t0 + r < num_tokens;
    const T* xrow = x + (size_t)(t0 + r) * d;
    for (int e0 = 0; e0 < E; e0 += 32) {
        const bool exp_ok = e0 + r < E;
        const float* wrow = wg + (size_t)(e0 + r) * d;
        f32x16 acc = zero16();
        // FWD_NB chunks per trip, every load of the trip issued before the first product: one memory latency per
        // trip instead of one per chunk (a wavefront's share of d = 384 is 6 chunks = one trip)
        for (int c = c0; c < c1; c += FWD_NB) {
            float xv[FWD_NB][8], wv[FWD_NB][8];
#pragma unroll
            for (int u = 0; u < FWD_NB; ++u) {
                const int piece = 2 * (c + u) + h;
                const bool ok = c + u < c1 && piece < pieces;
                LoadN<T, 8>::run(xrow + (ok ? piece : 0) * 8, ok && tok_ok, xv[u]);
                LoadN<float, 8>::run(wrow + (ok ? piece : 0) * 8, ok && exp_ok, wv[u]);
            }
#pragma unroll
            for (int u = 0; u < FWD_NB; ++u)
#pragma unroll
                for (int i = 0; i < 8; ++i) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(xv[u][i], wv[u][i], acc, 0, 0, 0);
        }
        __syncthreads();   // the previous expert block's partial sums have been consumed
#pragma unroll
        for (int v = 0; v < 16; ++v) part[wave][v][lane] = acc[v];
        __syncthreads();
        // wavefront w finishes result registers 4w..4w+3: token row 8w + 4h + q, expert column r
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int v = 4 * wave + q;
            const float sum = ((part[0][v][lane] + part[1][v][lane]) + part[2][v][lane]) + part[3][v][lane];
            const int t = t0 + 8 * wave + 4 * h + q;
            if (t < num_tokens && exp_ok) logits[(size_t)t * E + e0 + r] = sum;
        }
    }
}

template <typename T>
__global__ __launch_bounds__(256) void gate_bwd_kernel(GateBwdK p) { gate_bwd_body<T>(p, blockIdx.x); }

__global__ __launch_bounds__(256) void gate_dwg_reduce_kernel(DwgReduceK p) { dwg_reduce_body(p, blockIdx.x); }

template <typename T>
int gate_backward_t(void* dx, float* dwg, const float* dl, const void* x, const float* wg, int T_, int d, int E, float* ws,
                    hipStream_t st) {
    const int nchunks = div_up(T_, BWD_TB), groups = div_up(d, 128), eb = div_up(E, 32);
    const GateBwdK g{dx, dwg ? ws : nullptr, dl, x, wg, T_, d, E, nchunks * ((dx ? groups : 0) + (dwg ? groups * eb : 0))};
    hipLaunchKernelGGL(gate_bwd_kernel<T>, dim3(div_up(g.ntasks, 4)), dim3(256), 0, st, g);
    HEXA_CHECK_LAUNCH("gate_bwd");
    if (dwg) {
        SmallTask r;
        r.kind = TASK_DWG_REDUCE;
        r.dwg_reduce = DwgReduceK{dwg, ws, nchunks, (long)E * d / 4};
        r.blocks = (int)div_up(r.dwg_reduce.n4, 16);
        if (!defer_task(defer_targets().dwg_reduce, r)) {
            hipLaunchKernelGGL(gate_dwg_reduce_kernel, dim3(r.blocks), dim3(256), 0, st, r.dwg_reduce);
            HEXA_CHECK_LAUNCH("gate_dwg_reduce");
        }
    }
    return HEXA_OK;
}

}  // namespace
}  // namespace hexa

using namespace hexa;

extern "C" int hexa_gate_logits(float* logits, const void* x, const float* wg, int T, int d, int E, int x_dt,
                                void* stream) {
    if (T < 0 || d < 1 || E < 1) HEXA_FAIL(HEXA_ERR_ARG, "hexa_gate_logits: bad sizes T=%d d=%d E=%d", T, d, E);
    if (T > 0 && (!logits || !x || !wg)) HEXA_FAIL(HEXA_ERR_ARG, "hexa_gate_logits: null pointer");
    if (d % 8) HEXA_FAIL(HEXA_ERR_UNSUPPORTED, "hexa_gate_logits: model dim must be a multiple of 8 (got %d)", d);
    if (T == 0) return HEXA_OK;
    hipStream_t st = (hipStream_t)stream;
    const dim3 grid(div_up(T, GT)), block(256);
    if (x_dt == HEXA_F32) hipLaunchKernelGGL(gate_fwd_kernel<float>, grid, block, 0, st, logits, (const float*)x, wg, T, d, E);
    else if (x_dt == HEXA_BF16) hipLaunchKernelGGL(gate_fwd_kernel<__bf16>, grid, block, 0, st, logits, (const __bf16*)x, wg, T, d, E);
    else if (x_dt == HEXA_F16) hipLaunchKernelGGL(gate_fwd_kernel<_Float16>, grid, block, 0, st, logits, (const _Float16*)x, wg, T, d, E);
    else HEXA_FAIL(HEXA_ERR_ARG, "hexa_gate_logits: unknown element type");
    HEXA_CHECK_LAUNCH("gate_fwd");
    return HEXA_OK;
}

extern "C" int hexa_gate_ws_floats(int T, int d, int E, int64_t* out) {
    if (!out || T < 0 || d < 1 || E < 1) HEXA_FAIL(HEXA_ERR_ARG, "hexa_gate_ws_floats: bad arguments");
    *out = (int64_t)(T > 0 ? div_up(T, BWD_TB) : 1) * E * d;
    return HEXA_OK;
}

extern "C" int hexa_gate_backward(void* dx, float* dwg, const float* dlogits, const void* x, const float* wg, int T,
                                  int d, int E, int x_dt, float* ws, void* stream) {
    if (T < 0 || d < 1 || E < 1) HEXA_FAIL(HEXA_ERR_ARG, "hexa_gate_backward: bad sizes T=%d d=%d E=%d", T, d, E);
    if (d % 8) HEXA_FAIL(HEXA_ERR_UNSUPPORTED, "hexa_gate_backward: model dim must be a multiple of 8 (got %d)", d);
    if (!dx && !dwg) return HEXA_OK;
    if (T > 0 && (!dlogits || !wg || (dwg && (!x || !ws)))) HEXA_FAIL(HEXA_ERR_ARG, "hexa_gate_backward: null pointer");
    hipStream_t st = (hipStream_t)stream;
    if (T == 0) {   // no tokens: dwg = 0 (a reduction over zero partial sums)
        if (dwg) {
            const long n4 = (long)E * d / 4;
            hipLaunchKernelGGL(gate_dwg_reduce_kernel, dim3((unsigned)div_up(n4, 16)), dim3(256), 0, st, DwgReduceK{dwg, dwg, 0, n4});
            HEXA_CHECK_LAUNCH("gate_dwg_reduce");
        }
        return HEXA_OK;
    }
    if (x_dt == HEXA_F32) return gate_backward_t<float>(dx, dwg, dlogits, x, wg, T, d, E, ws, st);
    if (x_dt == HEXA_BF16) return gate_backward_t<__bf16>(dx, dwg, dlogits, x, wg, T, d, E, ws, st);
    if (x_dt == HEXA_F16) return gate_backward_t<_Float16>(dx, dwg, dlogits, x, wg, T, d, E, ws, st);
    HEXA_FAIL(HEXA_ERR_ARG, "hexa_gate_backward: unknown element type");
}
