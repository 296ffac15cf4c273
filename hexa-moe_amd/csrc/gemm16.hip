// ESMM and ESTMM for 16-bit operands (bf16 / fp16) on gfx950: v_mfma_f32_32x32x16 tiles with fp32
// accumulation, 128x128 output tile per 256-thread workgroup (2x2 wavefronts of 64x64), K step 64.
//
// Both MFMA operands must hold 8 consecutive contraction indices per lane, so every tile lives in
// LDS as [row of the output][contraction index] (pitch 72 elements).  Operands whose memory layout
// already has the contraction index fastest (token rows for ESMM, w[E][out][in]) are copied in
// 16-byte pieces; operands whose contraction index is the slow one (w[E][in][out]; token rows of dy
// and x for ESTMM, where tokens are contracted) are transposed on the way in: each thread loads four
// 16-byte rows and writes eight 8-byte columns.  No weight is permuted or copied in HBM.
//
// Tiles never straddle experts: ESMM walks the row-tile records the routing pass wrote (one per 128
// rows of a (slot, expert) segment, ragged tails zero-filled in LDS, nothing padded in HBM); ESTMM
// gives every (expert, 128x128 block of dW) to one workgroup that contracts over that expert's
// token list, slot after slot, so results are written once, without atomics, in a fixed order.
//
// Replaces esmm_shared_tensor_kernel_vectorized_accum_{half,mix} (kernels/esmm_half.cu, esmm_mix.cu)
// and the ESMM / ESTMM tasks of fused_grad_*_kernel_vectorized_{half,mix} (kernels/fused_ops_half.cu,
// fused_ops_mix.cu) of the reference, which use 16x16x16 WMMA tiles of 16 tokens and re-stream the
// expert panel for every 16-token block.
#include "hexa_internal.h"

namespace hexa {
namespace {

constexpr int BM = 128, BN = 128, BK = 64;
constexpr int LDK = BK + 8;  // LDS pitch (elements) of one tile row
constexpr int NT = 256;

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

template <typename TC> struct Mfma;
template <> struct Mfma<__bf16> {
    using V = bf16x8;
    static __device__ __forceinline__ f32x16 run(V a, V b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
};
template <> struct Mfma<_Float16> {
    using V = f16x8;
    static __device__ __forceinline__ f32x16 run(V a, V b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
};

// Eight consecutive source elements as eight TC packed into 16 bytes.
template <typename TC, typename TS> struct Load8;
template <typename TC> struct Load8<TC, TC> {
    static __device__ __forceinline__ uint4 run(const TC* p) { return *reinterpret_cast<const uint4*>(p); }
};
template <typename TC> struct Load8<TC, float> {
    static __device__ __forceinline__ uint4 run(const float* p) {
        const float4 a = reinterpret_cast<const float4*>(p)[0];
        const float4 b = reinterpret_cast<const float4*>(p)[1];
        union { uint4 u; TC e[8]; } r;
        r.e[0] = (TC)a.x; r.e[1] = (TC)a.y; r.e[2] = (TC)a.z; r.e[3] = (TC)a.w;
        r.e[4] = (TC)b.x; r.e[5] = (TC)b.y; r.e[6] = (TC)b.z; r.e[7] = (TC)b.w;
        return r.u;
    }
};

__device__ __forceinline__ uint4 zero4() { return make_uint4(0u, 0u, 0u, 0u); }

// Write a 4(k) x 8(n) register block as 8 columns of 4 consecutive k (8 bytes each) into a
// [n][k] LDS tile: dst points at element (n = first column, k = first row of the block).
template <typename TC>
__device__ __forceinline__ void store_transposed(TC* dst, const uint4 (&r)[4]) {
    const unsigned int w0[4] = {r[0].x, r[0].y, r[0].z, r[0].w};
    const unsigned int w1[4] = {r[1].x, r[1].y, r[1].z, r[1].w};
    const unsigned int w2[4] = {r[2].x, r[2].y, r[2].z, r[2].w};
    const unsigned int w3[4] = {r[3].x, r[3].y, r[3].z, r[3].w};
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        uint2 lo, hi;  // columns 2q and 2q+1
        lo.x = (w0[q] & 0xffffu) | (w1[q] << 16);
        lo.y = (w2[q] & 0xffffu) | (w3[q] << 16);
        hi.x = (w0[q] >> 16) | (w1[q] & 0xffff0000u);
        hi.y = (w2[q] >> 16) | (w3[q] & 0xffff0000u);
        *reinterpret_cast<uint2*>(dst + (2 * q) * LDK) = lo;
        *reinterpret_cast<uint2*>(dst + (2 * q + 1) * LDK) = hi;
    }
}

// Workgroup -> logical tile.  Workgroup ids go round-robin over the 8 XCDs (each with its own L2),
// so runs of `group` consecutive logical tiles (which share token rows and an expert's weights) are
// kept on one XCD.
__device__ __forceinline__ long logical_tile(int group) {
    const int bid = blockIdx.x;
    const int xcd = bid & 7, loc = bid >> 3;
    const int g = loc / group, r = loc - g * group;
    return ((long)g * 8 + xcd) * group + r;
}

// 64x64 per wavefront from the two LDS tiles: 4 sub-steps of K=16, 2x2 MFMA tiles each.
template <typename TC>
__device__ __forceinline__ void mma_tile(const TC* sA, const TC* sB, int wm, int wn, int lane,
                                         f32x16 (&acc)[2][2]) {
    using V = typename Mfma<TC>::V;
    const int r = lane & 31, kq = (lane >> 5) * 8;
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
        V a[2], b[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            a[i] = *reinterpret_cast<const V*>(sA + (wm * 64 + i * 32 + r) * LDK + ks * 16 + kq);
            b[i] = *reinterpret_cast<const V*>(sB + (wn * 64 + i * 32 + r) * LDK + ks * 16 + kq);
        }
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) acc[i][j] = Mfma<TC>::run(a[i], b[j], acc[i][j]);
    }
}

// ------------------------------------------------------------------------------------------------
// ESMM
// ------------------------------------------------------------------------------------------------
struct EsmmK {
    const void* x; const void* w; const void* bias; void* out; void* out_act;
    const int32_t* token_ids; const int4* tile_info; const int32_t* tile_count;
    int T, K, N, mt_ub, ntn, slot_begin, nslots;
    int x_slot_rows, out_slot_rows;  // 0 or T
    int accumulate, bias_dt, out_dt, act, group;
    long total;
};

template <typename TC, typename TW, bool W_IN_OUT>
__global__ __launch_bounds__(NT, 2) void esmm16_kernel(EsmmK p) {
    __shared__ __attribute__((aligned(16))) TC sA[BM * LDK];
    __shared__ __attribute__((aligned(16))) TC sB[BN * LDK];
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

    // ---- per-thread source pointers ----
    const int kc = tid & 7;       // 16-byte piece inside a 64-wide K step (direct copies)
    const int rw = tid >> 3;      // row (0..31) + 32*i
    const TC* xa[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int tok = sTok[rw + 32 * i];
        xa[i] = tok >= 0 ? reinterpret_cast<const TC*>(p.x) + ((size_t)p.x_slot_rows * s + tok) * K + kc * 8
                         : nullptr;
    }
    const TW* wsrc = reinterpret_cast<const TW*>(p.w) + (size_t)e * K * N;
    const int nch = tid & 15, kg = tid >> 4;  // transposed copies: 8 columns, 4 k-rows

    uint4 ra[4], rb[4];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
            ra[i] = (xa[i] && k0 + kc * 8 < K) ? Load8<TC, TC>::run(xa[i] + k0) : zero4();
        if (W_IN_OUT) {
            const int n = n0 + nch * 8;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int kk = k0 + kg * 4 + j;
                rb[j] = (kk < K && n < N) ? Load8<TC, TW>::run(wsrc + (size_t)kk * N + n) : zero4();
            }
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int n = n0 + rw + 32 * i;
                rb[i] = (n < N && k0 + kc * 8 < K) ? Load8<TC, TW>::run(wsrc + (size_t)n * K + k0 + kc * 8)
                                                   : zero4();
            }
        }
    };
    auto stash = [&]() {
#pragma unroll
        for (int i = 0; i < 4; ++i)
            *reinterpret_cast<uint4*>(sA + (rw + 32 * i) * LDK + kc * 8) = ra[i];
        if (W_IN_OUT) {
            store_transposed<TC>(sB + (nch * 8) * LDK + kg * 4, rb);
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i)
                *reinterpret_cast<uint4*>(sB + (rw + 32 * i) * LDK + kc * 8) = rb[i];
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
        mma_tile<TC>(sA, sB, wm, wn, lane, acc);
        __syncthreads();
        if (more) {
            stash();
            __syncthreads();
        }
    }

    // ---- epilogue: bias, optional GELU copy, scatter rows back to their tokens ----
    const bool accumulate = p.accumulate != 0;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int col = n0 + wn * 64 + j * 32 + (lane & 31);
        if (col >= N) continue;
        const float bv = p.bias ? load_as_f(p.bias, (size_t)e * N + col, p.bias_dt) : 0.f;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = wm * 64 + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                const int tok = sTok[row];
                if (tok < 0) continue;
                const size_t idx = ((size_t)p.out_slot_rows * s + tok) * N + col;
                float val = acc[i][j][v] + bv;
                if (p.act == HEXA_ACT_GELU_BWD) val *= gelu_grad_erf(load_as_f(p.out_act, idx, p.out_dt));
                store_out(p.out, idx, val, p.out_dt, accumulate);
                if (p.act == HEXA_ACT_GELU) store_out(p.out_act, idx, gelu_erf(val), p.out_dt, false);
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// ESTMM
// ------------------------------------------------------------------------------------------------
struct EstmmK {
    const void* pm; const void* qm; void* dw;
    const int32_t* token_ids; const int32_t* offsets;
    int T, k, E, M, N, mtn, ntn;
    int p_slot_rows, q_slot_rows;
    int accumulate, dw_dt, group;
    long total;
};

struct SegIter {
    int s, r, end;
};

template <typename TC>
__global__ __launch_bounds__(NT, 2) void estmm16_kernel(EstmmK p) {
    __shared__ __attribute__((aligned(16))) TC sA[BM * LDK];
    __shared__ __attribute__((aligned(16))) TC sB[BN * LDK];

    const long logical = logical_tile(p.group);
    if (logical >= p.total) return;
    const int per_e = p.mtn * p.ntn;
    const int e = (int)(logical / per_e);
    const int rem = (int)(logical - (long)e * per_e);
    const int m0 = (rem / p.ntn) * BM, n0 = (rem % p.ntn) * BN;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, wm = wave >> 1, wn = wave & 1;
    const int M = p.M, N = p.N, T = p.T;
    const int ch = tid & 15, kg = tid >> 4;
    const TC* P = reinterpret_cast<const TC*>(p.pm);
    const TC* Q = reinterpret_cast<const TC*>(p.qm);
    const bool m_ok = m0 + ch * 8 < M, n_ok = n0 + ch * 8 < N;

    auto seek = [&](SegIter it) {  // first non-empty chunk at or after `it`
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
    auto load_tok = [&](const SegIter& it, int (&tk)[4]) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int r = it.r + kg * 4 + j;
            tk[j] = (it.s < p.k && r < it.end) ? p.token_ids[(size_t)it.s * T + r] : -1;
        }
    };

    uint4 ra[4], rb[4];
    auto fetch = [&](const SegIter& it, const int (&tk)[4]) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const bool ok = tk[j] >= 0;
            ra[j] = (ok && m_ok) ? Load8<TC, TC>::run(P + ((size_t)p.p_slot_rows * it.s + tk[j]) * M + m0 + ch * 8)
                                 : zero4();
            rb[j] = (ok && n_ok) ? Load8<TC, TC>::run(Q + ((size_t)p.q_slot_rows * it.s + tk[j]) * N + n0 + ch * 8)
                                 : zero4();
        }
    };
    auto stash = [&]() {
        store_transposed<TC>(sA + (ch * 8) * LDK + kg * 4, ra);
        store_transposed<TC>(sB + (ch * 8) * LDK + kg * 4, rb);
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
        int tk[4], tkn[4];
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
            mma_tile<TC>(sA, sB, wm, wn, lane, acc);
            __syncthreads();
            if (!more) break;
            stash();
            __syncthreads();
            nxt = n2;
        }
    } else if (p.accumulate) {
        return;  // expert without tokens adds nothing
    }

    const bool accumulate = p.accumulate != 0;
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
                store_out(p.dw, ((size_t)e * M + row) * N + col, acc[i][j][v], p.dw_dt, accumulate);
            }
        }
    }
}

int round_up(long v, int m) { return (int)(((v + m - 1) / m) * m); }

template <typename TC>
int launch_esmm16_t(const EsmmArgs& a, hipStream_t st) {
    EsmmK p;
    p.x = a.x; p.w = a.w; p.bias = a.bias; p.out = a.out; p.out_act = a.out_act;
    p.token_ids = a.r.token_ids; p.tile_info = a.r.tile_info; p.tile_count = a.r.tile_count;
    p.T = a.r.T; p.K = a.in_dim; p.N = a.out_dim; p.mt_ub = a.r.mt_ub;
    p.ntn = div_up(a.out_dim, BN);
    p.x_slot_rows = a.x_per_slot ? a.r.T : 0;
    p.out_slot_rows = a.out_per_slot ? a.r.T : 0;
    p.bias_dt = a.bias_dt; p.out_dt = a.out_dt; p.act = a.act;
    p.group = p.ntn * 4;
    // Slots that write distinct rows go in one launch; slots that sum into the same rows run one
    // after the other (a token occurs once per slot, so a launch never writes a row twice).
    const int launches = a.out_per_slot ? 1 : a.r.k;
    for (int l = 0; l < launches; ++l) {
        p.slot_begin = a.out_per_slot ? 0 : l;
        p.nslots = a.out_per_slot ? a.r.k : 1;
        p.accumulate = (a.accumulate || l > 0) ? 1 : 0;
        p.total = (long)p.nslots * p.mt_ub * p.ntn;
        if (p.total == 0) continue;
        const int grid = round_up(p.total, 8 * p.group);
        const bool w32 = a.w_dt == HEXA_F32;
        const bool io = a.w_layout == HEXA_W_IN_OUT;
        if (w32 && io) hipLaunchKernelGGL((esmm16_kernel<TC, float, true>), dim3(grid), dim3(NT), 0, st, p);
        else if (w32) hipLaunchKernelGGL((esmm16_kernel<TC, float, false>), dim3(grid), dim3(NT), 0, st, p);
        else if (io) hipLaunchKernelGGL((esmm16_kernel<TC, TC, true>), dim3(grid), dim3(NT), 0, st, p);
        else hipLaunchKernelGGL((esmm16_kernel<TC, TC, false>), dim3(grid), dim3(NT), 0, st, p);
        HEXA_CHECK_LAUNCH("esmm16");
    }
    return HEXA_OK;
}

template <typename TC>
int launch_estmm16_t(const EstmmArgs& a, hipStream_t st) {
    EstmmK p;
    p.pm = a.p; p.qm = a.q; p.dw = a.dw;
    p.token_ids = a.r.token_ids; p.offsets = a.r.offsets;
    p.T = a.r.T; p.k = a.r.k; p.E = a.r.E; p.M = a.m_dim; p.N = a.n_dim;
    p.mtn = div_up(a.m_dim, BM); p.ntn = div_up(a.n_dim, BN);
    p.p_slot_rows = a.p_per_slot ? a.r.T : 0;
    p.q_slot_rows = a.q_per_slot ? a.r.T : 0;
    p.accumulate = a.accumulate; p.dw_dt = a.dw_dt;
    p.group = p.ntn;
    p.total = (long)a.r.E * p.mtn * p.ntn;
    if (p.total == 0) return HEXA_OK;
    const int grid = round_up(p.total, 8 * p.group);
    hipLaunchKernelGGL((estmm16_kernel<TC>), dim3(grid), dim3(NT), 0, st, p);
    HEXA_CHECK_LAUNCH("estmm16");
    return HEXA_OK;
}

}  // namespace

int launch_esmm16(const EsmmArgs& a, hipStream_t st) {
    if ((a.in_dim & 7) || (a.out_dim & 7))
        HEXA_FAIL(HEXA_ERR_UNSUPPORTED, "esmm (16-bit): in_dim and out_dim must be multiples of 8 (got %d, %d)",
                  a.in_dim, a.out_dim);
    if (a.x_dt == HEXA_BF16) return launch_esmm16_t<__bf16>(a, st);
    return launch_esmm16_t<_Float16>(a, st);
}

int launch_estmm16(const EstmmArgs& a, hipStream_t st) {
    if ((a.m_dim & 7) || (a.n_dim & 7))
        HEXA_FAIL(HEXA_ERR_UNSUPPORTED, "estmm (16-bit): dims must be multiples of 8 (got %d, %d)", a.m_dim,
                  a.n_dim);
    if (a.pq_dt == HEXA_BF16) return launch_estmm16_t<__bf16>(a, st);
    return launch_estmm16_t<_Float16>(a, st);
}

}  // namespace hexa
