// ESMM and ESTMM in true fp32 on gfx950: v_mfma_f32_32x32x2_f32 (fp32 multiply, fp32 accumulate),
// 128x128 output tile per 256-thread workgroup, K step 16.  Unlike the reference, which rounds fp32
// operands to fp16 before its WMMA (kernels/esmm_full.cu:128-130,167-169), nothing is rounded, so
// results agree with an fp32 matmul to ~1e-6.
//
// The fp32 MFMA takes ONE contraction index per lane, so there is no layout constraint on the
// operands: both tiles live in LDS as [contraction index][row of the output] (pitch 132 floats),
// whichever way round they sit in memory.
//
// Replaces esmm_shared_tensor_kernel_vectorized_accum_full (kernels/esmm_full.cu:58-246) and the
// ESMM / ESTMM tasks of fused_grad_*_kernel_vectorized_full (kernels/fused_ops_full.cu:117-371).
#include "hexa_internal.h"

namespace hexa {
namespace {

constexpr int BM = 128, BN = 128, BK = 16;
constexpr int LDP = BM + 4;  // LDS pitch (floats) of one contraction row
constexpr int NT = 256;

typedef __attribute__((ext_vector_type(16))) float f32x16;

__device__ __forceinline__ long logical_tile(int group) {
    const int bid = blockIdx.x;
    const int xcd = bid & 7, loc = bid >> 3;
    const int g = loc / group, r = loc - g * group;
    return ((long)g * 8 + xcd) * group + r;
}

__device__ __forceinline__ void mma_tile(const float* sA, const float* sB, int wm, int wn, int lane,
                                         f32x16 (&acc)[2][2]) {
    const int r = lane & 31, kh = lane >> 5;
#pragma unroll
    for (int kk = 0; kk < BK; kk += 2) {
        float a[2], b[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            a[i] = sA[(kk + kh) * LDP + wm * 64 + i * 32 + r];
            b[i] = sB[(kk + kh) * LDP + wn * 64 + i * 32 + r];
        }
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
    }
}

__device__ __forceinline__ float4 zero4f() { return make_float4(0.f, 0.f, 0.f, 0.f); }

// rows x 4 consecutive contraction indices -> 4 scalars at [k..k+3][row]
__device__ __forceinline__ void store_cols(float* s, int k, int row, const float4& v) {
    s[(k + 0) * LDP + row] = v.x;
    s[(k + 1) * LDP + row] = v.y;
    s[(k + 2) * LDP + row] = v.z;
    s[(k + 3) * LDP + row] = v.w;
}

struct EsmmK {
    const float* x; const float* w; const float* bias; float* out; float* out_act;
    const int32_t* token_ids; const int4* tile_info; const int32_t* tile_count;
    int T, K, N, mt_ub, ntn, slot_begin, nslots;
    int x_slot_rows, out_slot_rows;
    int accumulate, act, group;
    long total;
};

template <bool W_IN_OUT>
__global__ __launch_bounds__(NT, 2) void esmm32_kernel(EsmmK p) {
    __shared__ __attribute__((aligned(16))) float sA[BK * LDP];
    __shared__ __attribute__((aligned(16))) float sB[BK * LDP];
    __shared__ int sTok[BM];

    const long logical = logical_tile(p.group);
    if (logical >= p.total) return;
    const int nt = (int)(logical % p.ntn);
    const int mtg = (int)(logical / p.ntn);
    const int s = p.slot_begin + mtg / p.mt_ub;
    const int mt = mtg % p.mt_ub;
    if (mt >= p.tile_count[s]) return;
    const int4 info = p.tile_info[(size_t)s * p.mt_ub + mt];
    const int e = info.x, row_start = info.y, rows = info.z;
    const int n0 = nt * BN;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, wm = wave >> 1, wn = wave & 1;
    const int K = p.K, N = p.N;

    if (tid < BM) sTok[tid] = tid < rows ? p.token_ids[(size_t)s * p.T + row_start + tid] : -1;
    __syncthreads();

    // direct pieces: row = tid & 127, 4-float piece kc = (tid >> 7) + 2*i  (i = 0, 1)
    const int drow = tid & 127, dkc = tid >> 7;
    const int tok = sTok[drow];
    const float* xa = tok >= 0 ? p.x + ((size_t)p.x_slot_rows * s + tok) * K : nullptr;
    const float* wsrc = p.w + (size_t)e * K * N;
    // transposed-source pieces (w[E][in][out]): k-row = (tid >> 5) + 8*i, 4 columns nc = tid & 31
    const int tk = tid >> 5, tnc = tid & 31;

    float4 ra[2], rb[2];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int k = k0 + (dkc + 2 * i) * 4;
            ra[i] = (xa && k < K) ? *reinterpret_cast<const float4*>(xa + k) : zero4f();
        }
        if (W_IN_OUT) {
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const int k = k0 + tk + 8 * i, n = n0 + tnc * 4;
                rb[i] = (k < K && n < N) ? *reinterpret_cast<const float4*>(wsrc + (size_t)k * N + n) : zero4f();
            }
        } else {
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const int k = k0 + (dkc + 2 * i) * 4, n = n0 + drow;
                rb[i] = (n < N && k < K) ? *reinterpret_cast<const float4*>(wsrc + (size_t)n * K + k) : zero4f();
            }
        }
    };
    auto stash = [&]() {
#pragma unroll
        for (int i = 0; i < 2; ++i) store_cols(sA, (dkc + 2 * i) * 4, drow, ra[i]);
        if (W_IN_OUT) {
#pragma unroll
            for (int i = 0; i < 2; ++i) *reinterpret_cast<float4*>(sB + (tk + 8 * i) * LDP + tnc * 4) = rb[i];
        } else {
#pragma unroll
            for (int i = 0; i < 2; ++i) store_cols(sB, (dkc + 2 * i) * 4, drow, rb[i]);
        }
    };

    f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    const int nk = (K + BK - 1) / BK;
    fetch(0);
    stash();
    __syncthreads();
    for (int kt = 0; kt < nk; ++kt) {
        const bool more = kt + 1 < nk;
        if (more) fetch((kt + 1) * BK);
        mma_tile(sA, sB, wm, wn, lane, acc);
        __syncthreads();
        if (more) {
            stash();
            __syncthreads();
        }
    }

#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int col = n0 + wn * 64 + j * 32 + (lane & 31);
        if (col >= N) continue;
        const float bv = p.bias ? p.bias[(size_t)e * N + col] : 0.f;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = wm * 64 + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                const int t = sTok[row];
                if (t < 0) continue;
                const size_t idx = ((size_t)p.out_slot_rows * s + t) * N + col;
                float val = acc[i][j][v] + bv;
                if (p.act == HEXA_ACT_GELU_BWD) val *= gelu_grad_erf(p.out_act[idx]);
                p.out[idx] = p.accumulate ? p.out[idx] + val : val;
                if (p.act == HEXA_ACT_GELU) p.out_act[idx] = gelu_erf(val);
            }
        }
    }
}

struct EstmmK {
    const float* pm; const float* qm; float* dw;
    const int32_t* token_ids; const int32_t* offsets;
    int T, k, E, M, N, mtn, ntn;
    int p_slot_rows, q_slot_rows;
    int accumulate, group;
    long total;
};

struct SegIter {
    int s, r, end;
};

__global__ __launch_bounds__(NT, 2) void estmm32_kernel(EstmmK p) {
    __shared__ __attribute__((aligned(16))) float sA[BK * LDP];
    __shared__ __attribute__((aligned(16))) float sB[BK * LDP];

    const long logical = logical_tile(p.group);
    if (logical >= p.total) return;
    const int per_e = p.mtn * p.ntn;
    const int e = (int)(logical / per_e);
    const int rem = (int)(logical - (long)e * per_e);
    const int m0 = (rem / p.ntn) * BM, n0 = (rem % p.ntn) * BN;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, wm = wave >> 1, wn = wave & 1;
    const int M = p.M, N = p.N, T = p.T;
    // token row = (tid >> 5) + 8*i (i = 0, 1), 4 columns c4 = tid & 31
    const int tr = tid >> 5, c4 = tid & 31;
    const bool m_ok = m0 + c4 * 4 < M, n_ok = n0 + c4 * 4 < N;

    auto seek = [&](SegIter it) {
        while (it.s < p.k && it.r >= it.end) {
            ++it.s;
            if (it.s < p.k) {
                it.r = p.offsets[(size_t)it.s * (p.E + 1) + e];
                it.end = p.offsets[(size_t)it.s * (p.E + 1) + e + 1];
            }
        }
        return it;
    };
    auto next = [&](SegIter it) { it.r += BK; return seek(it); };
    auto load_tok = [&](const SegIter& it, int (&tk)[2]) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int r = it.r + tr + 8 * i;
            tk[i] = (it.s < p.k && r < it.end) ? p.token_ids[(size_t)it.s * T + r] : -1;
        }
    };
    float4 ra[2], rb[2];
    auto fetch = [&](const SegIter& it, const int (&tk)[2]) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const bool ok = tk[i] >= 0;
            ra[i] = (ok && m_ok) ? *reinterpret_cast<const float4*>(
                                       p.pm + ((size_t)p.p_slot_rows * it.s + tk[i]) * M + m0 + c4 * 4)
                                 : zero4f();
            rb[i] = (ok && n_ok) ? *reinterpret_cast<const float4*>(
                                       p.qm + ((size_t)p.q_slot_rows * it.s + tk[i]) * N + n0 + c4 * 4)
                                 : zero4f();
        }
    };
    auto stash = [&]() {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            *reinterpret_cast<float4*>(sA + (tr + 8 * i) * LDP + c4 * 4) = ra[i];
            *reinterpret_cast<float4*>(sB + (tr + 8 * i) * LDP + c4 * 4) = rb[i];
        }
    };

    f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    SegIter cur;
    cur.s = 0;
    cur.r = p.offsets[e];
    cur.end = p.offsets[e + 1];
    cur = seek(cur);
    if (cur.s < p.k) {
        int tk[2], tkn[2];
        load_tok(cur, tk);
        fetch(cur, tk);
        SegIter nxt = next(cur);
        load_tok(nxt, tkn);
        stash();
        __syncthreads();
        while (true) {
            const bool more = nxt.s < p.k;
            SegIter n2 = nxt;
            if (more) {
                fetch(nxt, tkn);
                n2 = next(nxt);
                load_tok(n2, tkn);
            }
            mma_tile(sA, sB, wm, wn, lane, acc);
            __syncthreads();
            if (!more) break;
            stash();
            __syncthreads();
            nxt = n2;
        }
    } else if (p.accumulate) {
        return;
    }

#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int col = n0 + wn * 64 + j * 32 + (lane & 31);
        if (col >= N) continue;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = m0 + wm * 64 + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                if (row >= M) continue;
                const size_t idx = ((size_t)e * M + row) * N + col;
                p.dw[idx] = p.accumulate ? p.dw[idx] + acc[i][j][v] : acc[i][j][v];
            }
        }
    }
}

int round_up(long v, int m) { return (int)(((v + m - 1) / m) * m); }

}  // namespace

int launch_esmm32(const EsmmArgs& a, hipStream_t st) {
    if ((a.in_dim & 3) || (a.out_dim & 3))
        HEXA_FAIL(HEXA_ERR_UNSUPPORTED, "esmm (fp32): in_dim and out_dim must be multiples of 4 (got %d, %d)",
                  a.in_dim, a.out_dim);
    EsmmK p;
    p.x = (const float*)a.x; p.w = (const float*)a.w; p.bias = (const float*)a.bias;
    p.out = (float*)a.out; p.out_act = (float*)a.out_act;
    p.token_ids = a.r.token_ids; p.tile_info = a.r.tile_info; p.tile_count = a.r.tile_count;
    p.T = a.r.T; p.K = a.in_dim; p.N = a.out_dim; p.mt_ub = a.r.mt_ub;
    p.ntn = div_up(a.out_dim, BN);
    p.x_slot_rows = a.x_per_slot ? a.r.T : 0;
    p.out_slot_rows = a.out_per_slot ? a.r.T : 0;
    p.act = a.act;
    p.group = p.ntn * 4;
    const int launches = a.out_per_slot ? 1 : a.r.k;
    for (int l = 0; l < launches; ++l) {
        p.slot_begin = a.out_per_slot ? 0 : l;
        p.nslots = a.out_per_slot ? a.r.k : 1;
        p.accumulate = (a.accumulate || l > 0) ? 1 : 0;
        p.total = (long)p.nslots * p.mt_ub * p.ntn;
        if (p.total == 0) continue;
        const int grid = round_up(p.total, 8 * p.group);
        if (a.w_layout == HEXA_W_IN_OUT)
            hipLaunchKernelGGL((esmm32_kernel<true>), dim3(grid), dim3(NT), 0, st, p);
        else
            hipLaunchKernelGGL((esmm32_kernel<false>), dim3(grid), dim3(NT), 0, st, p);
        HEXA_CHECK_LAUNCH("esmm32");
    }
    return HEXA_OK;
}

int launch_estmm32(const EstmmArgs& a, hipStream_t st) {
    if ((a.m_dim & 3) || (a.n_dim & 3))
        HEXA_FAIL(HEXA_ERR_UNSUPPORTED, "estmm (fp32): dims must be multiples of 4 (got %d, %d)", a.m_dim, a.n_dim);
    EstmmK p;
    p.pm = (const float*)a.p; p.qm = (const float*)a.q; p.dw = (float*)a.dw;
    p.token_ids = a.r.token_ids; p.offsets = a.r.offsets;
    p.T = a.r.T; p.k = a.r.k; p.E = a.r.E; p.M = a.m_dim; p.N = a.n_dim;
    p.mtn = div_up(a.m_dim, BM); p.ntn = div_up(a.n_dim, BN);
    p.p_slot_rows = a.p_per_slot ? a.r.T : 0;
    p.q_slot_rows = a.q_per_slot ? a.r.T : 0;
    p.accumulate = a.accumulate;
    p.group = p.ntn;
    p.total = (long)a.r.E * p.mtn * p.ntn;
    if (p.total == 0) return HEXA_OK;
    const int grid = round_up(p.total, 8 * p.group);
    hipLaunchKernelGGL(estmm32_kernel, dim3(grid), dim3(NT), 0, st, p);
    HEXA_CHECK_LAUNCH("estmm32");
    return HEXA_OK;
}

}  // namespace hexa
