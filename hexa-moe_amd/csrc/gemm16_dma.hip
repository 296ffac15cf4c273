// Fast path of ESMM and ESTMM for bf16 / fp16 on gfx950 (CDNA4): tiles stream from HBM straight into
// LDS with the asynchronous global->LDS copy (global_load_lds_dwordx4, 16 bytes per lane, no VGPR
// staging), several stages deep, and are fed to v_mfma_f32_32x32x16 with fp32 accumulation.
//
// Workgroup tile: BM x BN with WR x WF wavefronts of 64x64 each.  Two shapes are instantiated:
//   128 x 128 (4 wavefronts, 4 stages, 64 KiB LDS, 2 workgroups per CU)  -- small problems
//   256 x 128 (8 wavefronts, 3 stages, 72 KiB LDS, 2 workgroups per CU)  -- a third less L2 traffic
//   per flop; with 128x128 tiles these kernels sit on the L2 -> LDS bandwidth, not on the MFMA pipe.
//
// LDS tile formats (per stage an operand tile holds W output rows x 32 contraction indices):
//   KC  "contraction index fastest in memory"  [W rows][32 k]  64 B per row; a wavefront copy
//       (64 lanes x 16 B = 1 KiB, contiguous in LDS) covers 16 rows.  Fragments: ds_read_b128.
//       Token rows of ESMM (gathered through the tile's token ids) and w[E][out][in].
//   KS  "contraction index slowest in memory"   [32 k][W rows] 2W B per k.  Fragments: two
//       ds_read_b64_tr_b16 (the CDNA4 transposing LDS read) per 32x16 fragment.
//       w[E][in][out] of ESMM, and both operands of ESTMM (token rows of dy and x, tokens contracted).
// The copy engine places lane i at LDS offset 16*i, so bank conflicts are avoided by choosing WHICH
// 16-byte piece each lane fetches (an XOR swizzle applied on the global-address side) instead of
// padding.  Lanes that have nothing to fetch (rows past the end of a segment, columns past N) read
// a 16-byte block of zeros, so ragged tails cost no HBM bytes and need no branches.
//
// The MFMA operands are swapped with respect to the usual convention (A = the operand that supplies
// the output's fastest dimension, B = the rows), so every lane ends up with 4 consecutive output
// columns; results leave through LDS so that whole 256- / 512-byte row pieces are stored.
//
// Constraints of this path (anything else runs on the general kernels of gemm16.hip): operands and
// weights of one 16-bit type, in_dim a multiple of 32 for ESMM, out/in dims multiples of 8.
#include <algorithm>

#include "dma_common.h"
#include "small_bodies.h"

namespace hexa {
namespace {

template <typename TC, bool W_IN_OUT, bool OUT32, typename C>
__global__ __launch_bounds__(C::NT, C::MINW) void esmm16_dma_kernel(EsmmK p) {
    constexpr int BM = C::BM, BN = C::BN, STAGES = C::STAGES, NW = C::NW, BK = C::BKC;
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    int* sTok = reinterpret_cast<int*>(smem + C::STAGE_AREA);

    int nt, s, mt;
    if (p.group > 0) {
        const long logical = logical_tile(p.group);
        if (logical >= p.total) return;
        nt = (int)(logical % p.ntn);
        const int mtg = (int)(logical / p.ntn);
        s = p.slot_begin + mtg / p.mt_ub;
        mt = mtg % p.mt_ub;
        if (mt >= p.tile_count[s]) return;
    } else {
        // Every XCD (workgroup ids go round-robin over the 8 of them) walks one contiguous eighth of
        // the list of VALID tiles, column tiles fastest: an expert's weights are then fetched into
        // one L2 (two at a boundary) per slot instead of into all eight.
        int cum[9];
        cum[0] = 0;
#pragma unroll
        for (int q = 0; q < 8; ++q) cum[q + 1] = cum[q] + (q < p.nslots ? min(p.tile_count[p.slot_begin + q], p.mt_ub) : 0);
        const int valid = cum[8] * p.ntn;
        const int per = (valid + 7) >> 3;
        const int xcd = blockIdx.x & 7, loc = blockIdx.x >> 3;
        const int logical = xcd * per + loc;
        if (loc >= per || logical >= valid) return;
        const int mtg = logical / p.ntn;
        nt = logical - mtg * p.ntn;
        int sl = 0;
#pragma unroll
        for (int q = 1; q < 8; ++q) sl += (mtg >= cum[q] && q < p.nslots) ? 1 : 0;
        s = p.slot_begin + sl;
        mt = mtg - cum[sl];
    }
    const int4 info = p.tile_info[(size_t)s * p.mt_ub + mt];
    const int e = info.x, row_start = info.y, rows = info.z;
    const int n0 = nt * BN;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wr = wave / C::WF, wf = wave % C::WF;
    const int K = p.K, N = p.N;

    if (tid < BM) sTok[tid] = tid < rows ? p.token_ids[(size_t)s * p.T + row_start + tid] : -1;
    __syncthreads();

    // ---- sources of this lane's copies: a base every lane shares plus a 32-bit byte offset per lane ----
    // (the copy instruction then reads ONE address register per lane and a scalar pair instead of two registers per
    // lane: next to wavefronts that issue MFMAs back to back, a CU moves 28 B/clk with this form against 10 with
    // 64-bit lane addresses, and the MFMAs themselves run at 80 % instead of 60 % -- the launcher keeps tensors of
    // 4 GiB and more off this kernel).  Lanes that have nothing to fetch (rows past the end of a segment, columns
    // past N) re-read the first bytes of the tensor: what they produce is never stored.
    const char* const xbase = reinterpret_cast<const char*>(p.x);
    const char* const wbase = reinterpret_cast<const char*>(p.w) + (size_t)e * K * N * 2;
    unsigned offR[C::R_CPW]; int stepR[C::R_CPW];
    unsigned offF[C::F_CPW]; int stepF[C::F_CPW];
#pragma unroll
    for (int i = 0; i < C::R_CPW; ++i) {   // token rows, KC
        int row, kc;
        kc_lane<BK>(wave + NW * i, lane, row, kc);
        const int tok = sTok[row];
        const bool ok = tok >= 0;
        offR[i] = ok ? (unsigned)((((size_t)p.x_slot_rows * s + tok) * K + kc * 8) * 2) : 0u;
        stepR[i] = ok ? BK * 2 : 0;
    }
#pragma unroll
    for (int i = 0; i < C::F_CPW; ++i) {
        if (W_IN_OUT) {  // w[e][k][n], KS
            int kk, ch;
            ks_lane<BN>(wave + NW * i, lane, kk, ch);
            const int n = n0 + ch * 8;
            const bool ok = n < N;
            offF[i] = ok ? (unsigned)(((size_t)kk * N + n) * 2) : 0u;
            stepF[i] = ok ? BK * N * 2 : 0;
        } else {         // w[e][n][k], KC
            int row, kc;
            kc_lane<BK>(wave + NW * i, lane, row, kc);
            const int n = n0 + row;
            const bool ok = n < N;
            offF[i] = ok ? (unsigned)(((size_t)n * K + kc * 8) * 2) : 0u;
            stepF[i] = ok ? BK * 2 : 0;
        }
    }
    auto issue = [&](int stage) {
        char* base = smem + stage * C::STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < C::R_CPW; ++i) {
            dma16(xbase + (size_t)offR[i], base + (wave + NW * i) * 1024);
            offR[i] += stepR[i];
        }
#pragma unroll
        for (int i = 0; i < C::F_CPW; ++i) {
            dma16(wbase + (size_t)offF[i], base + C::R_BYTES + (wave + NW * i) * 1024);
            offF[i] += stepF[i];
        }
    };

    f32x16 acc[C::FB][C::RB];
    zero_acc(acc);
    const int nk = K / BK;
#pragma unroll
    for (int st = 0; st < STAGES - 1; ++st)
        if (st < nk) issue(st);
    for (int kt = 0; kt < nk; ++kt) {
        // copies of step kt have landed when at most the copies of the later steps are outstanding
        wait_groups<C::CPW, STAGES - 2>(min(nk - 1 - kt, STAGES - 2));
        barrier_nofence();  // everyone's copies of step kt are in LDS; everyone is done reading step kt-1
        if (kt + STAGES - 1 < nk) issue((kt + STAGES - 1) % STAGES);
        const char* base = smem + (kt % STAGES) * C::STAGE_BYTES;
        mma_stage<TC, C, W_IN_OUT, false>(base, base + C::R_BYTES, wr, wf, lane, acc);
    }

    // ---- epilogue: lane holds, per 32x32 block, token row l%32 and 4 consecutive columns per group ----
    // 16-bit results leave through LDS (PR rows per pass) so that BN/8 lanes write one contiguous row
    // piece; fp32 results are stored from the registers, 16 bytes per lane.
    const bool to_ws = p.ws != nullptr && s > 0;
    void* const outp = to_ws ? p.ws : p.out;
    const bool accumulate = p.accumulate != 0 && !to_ws;
    const bool gelu = p.act == HEXA_ACT_GELU;
    const bool gelu_bwd = p.act == HEXA_ACT_GELU_BWD;
    const size_t out_base = to_ws ? (size_t)p.T * (s - 1) : (size_t)p.out_slot_rows * s;
    constexpr int CP = BN * 2 + 16;  // pitch (bytes) of the staged 16-bit result tile
    constexpr int PR = (BM * CP <= C::STAGE_AREA) ? BM : ((BM / 2) * CP <= C::STAGE_AREA ? BM / 2 : BM / 4);
    static_assert(PR * CP <= C::STAGE_AREA, "the staged result must fit in the stage buffers");
    constexpr int NPASS = OUT32 ? 1 : BM / PR;
    constexpr int RW = 32 * C::RB, FW = 32 * C::FB;
    // column sums of the stored result (the bias gradient of the layer below): a thread of the store loop
    // always handles the same 16-byte piece of a row when the workgroup size is a multiple of the pieces per row
    constexpr bool COLSUM_OK = !OUT32 && C::NT % (BN / 8) == 0 && 64 % (BN / 8) == 0;
    const bool colsum = COLSUM_OK && p.colsum != nullptr;
    float cs[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int pass = 0; pass < NPASS; ++pass) {
        if (!OUT32) { if (pass == 0) barrier_nofence(); else __syncthreads(); }   // staging area is free
#pragma unroll
        for (int j = 0; j < C::FB; ++j) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int nl = wf * FW + j * 32 + 8 * g + 4 * (lane >> 5);
                const int n = n0 + nl;
                float bv[4] = {0.f, 0.f, 0.f, 0.f};
                if (p.bias && n < N) {
                    if (p.bias_dt == HEXA_F32) {
                        const float4 b4 = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(p.bias) + (size_t)e * N + n);
                        bv[0] = b4.x; bv[1] = b4.y; bv[2] = b4.z; bv[3] = b4.w;
                    } else {
                        const uint2 b2 = *reinterpret_cast<const uint2*>(reinterpret_cast<const unsigned short*>(p.bias) + (size_t)e * N + n);
                        bv[0] = from_bits16<TC>(b2.x & 0xffff); bv[1] = from_bits16<TC>(b2.x >> 16);
                        bv[2] = from_bits16<TC>(b2.y & 0xffff); bv[3] = from_bits16<TC>(b2.y >> 16);
                    }
                }
#pragma unroll
                for (int i = 0; i < C::RB; ++i) {
                    const int rl = wr * RW + i * 32 + (lane & 31);
                    if (!OUT32 && (wr * RW + i * 32) / PR != pass) continue;
                    float v[4];
#pragma unroll
                    for (int q = 0; q < 4; ++q) v[q] = acc[j][i][4 * g + q] + bv[q];
                    if (OUT32) {
                        const int tok = sTok[rl];
                        if (tok < 0 || n >= N) continue;
                        const size_t off = (out_base + tok) * N + n;
                        float4* dst = reinterpret_cast<float4*>(reinterpret_cast<float*>(outp) + off);
                        if (gelu_bwd) {
                            const float4 y = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(p.out_act) + off);
                            v[0] *= gelu_grad_fast(y.x); v[1] *= gelu_grad_fast(y.y); v[2] *= gelu_grad_fast(y.z); v[3] *= gelu_grad_fast(y.w);
                        }
                        if (accumulate) { const float4 old = *dst; v[0] += old.x; v[1] += old.y; v[2] += old.z; v[3] += old.w; }
                        *dst = make_float4(v[0], v[1], v[2], v[3]);
                        if (gelu)
                            *reinterpret_cast<float4*>(reinterpret_cast<float*>(p.out_act) + off) =
                                make_float4(gelu_fast(v[0]), gelu_fast(v[1]), gelu_fast(v[2]), gelu_fast(v[3]));
                    } else {
                        *reinterpret_cast<uint2*>(smem + (rl - pass * PR) * CP + nl * 2) = pack4<TC>(v[0], v[1], v[2], v[3]);
                    }
                }
            }
        }
        if (!OUT32) {
            __syncthreads();
            constexpr int LPR = BN / 8;             // 16-byte pieces per row
            {
#pragma unroll 4
                for (int idx = tid; idx < PR * LPR; idx += C::NT) {
                    const int rl = idx / LPR, c = idx - rl * LPR, n = n0 + c * 8;
                    const int tok = sTok[pass * PR + rl];
                    if (tok < 0 || n >= N) continue;
                    const size_t off = (out_base + tok) * N + n;
                    uint4 val = *reinterpret_cast<const uint4*>(smem + rl * CP + c * 16);
                    uint4* dst = reinterpret_cast<uint4*>(reinterpret_cast<unsigned short*>(outp) + off);
                    if (gelu_bwd) {
                        const uint4 yv = *reinterpret_cast<const uint4*>(reinterpret_cast<const unsigned short*>(p.out_act) + off);
                        const unsigned yw[4] = {yv.x, yv.y, yv.z, yv.w};
                        unsigned vw[4] = {val.x, val.y, val.z, val.w};
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            const float lo = from_bits16<TC>(vw[q] & 0xffff) * gelu_grad_fast(from_bits16<TC>(yw[q] & 0xffff));
                            const float hi = from_bits16<TC>(vw[q] >> 16) * gelu_grad_fast(from_bits16<TC>(yw[q] >> 16));
                            vw[q] = pack2<TC>(lo, hi);
                        }
                        val = make_uint4(vw[0], vw[1], vw[2], vw[3]);
                    }
                    if (accumulate) {
                        const uint4 old = *dst;
                        const unsigned ow[4] = {old.x, old.y, old.z, old.w};
                        unsigned vw[4] = {val.x, val.y, val.z, val.w};
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            const float lo = from_bits16<TC>(vw[q] & 0xffff) + from_bits16<TC>(ow[q] & 0xffff);
                            const float hi = from_bits16<TC>(vw[q] >> 16) + from_bits16<TC>(ow[q] >> 16);
                            vw[q] = pack2<TC>(lo, hi);
                        }
                        val = make_uint4(vw[0], vw[1], vw[2], vw[3]);
                    }
                    store16(dst, val, p.stream_out == 1);
                    if (colsum) {
                        const unsigned vw[4] = {val.x, val.y, val.z, val.w};
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            cs[2 * q] += from_bits16<TC>(vw[q] & 0xffff);
                            cs[2 * q + 1] += from_bits16<TC>(vw[q] >> 16);
                        }
                    }
                    if (gelu) {
                        // applied to the value as stored (rounded), like act(y1) on the tensor
                        unsigned vw[4] = {val.x, val.y, val.z, val.w};
#pragma unroll
                        for (int q = 0; q < 4; ++q)
                            vw[q] = pack2<TC>(gelu_fast(from_bits16<TC>(vw[q] & 0xffff)), gelu_fast(from_bits16<TC>(vw[q] >> 16)));
                        store16(reinterpret_cast<uint4*>(reinterpret_cast<unsigned short*>(p.out_act) + off),
                                make_uint4(vw[0], vw[1], vw[2], vw[3]), p.stream_out == 1);
                    }
                }
            }
        }
    }
    if (COLSUM_OK && colsum) {
        constexpr int LPR = BN / 8;
        // the 64 / LPR lanes of a wavefront that hold the same piece, then the wavefronts in order through LDS
#pragma unroll
        for (int q = 0; q < 8; ++q) {
#pragma unroll
            for (int m = 32; m >= LPR; m >>= 1) cs[q] += __shfl_xor(cs[q], m);
        }
        __syncthreads();                          // the staged tile has been stored
        float* red = reinterpret_cast<float*>(smem);
        if (lane < LPR) {
#pragma unroll
            for (int q = 0; q < 8; ++q) red[wave * BN + lane * 8 + q] = cs[q];
        }
        __syncthreads();
        float* dst = p.colsum + (((size_t)s * p.mt_ub + mt) * p.ntn + nt) * BN;
        for (int c = tid; c < BN; c += C::NT) {
            float t = 0.f;
#pragma unroll
            for (int w = 0; w < NW; ++w) t += red[w * BN + c];
            dst[c] = t;
        }
    }
}

__global__ __launch_bounds__(256) void esmm_colsum_fold_kernel(ColsumFoldK p) { colsum_fold_body(p, blockIdx.x); }

template <typename TC, bool IO, bool OUT32, typename C>
int launch_esmm_dma_t(EsmmK& p, int grid, hipStream_t st) {
    auto kernel = esmm16_dma_kernel<TC, IO, OUT32, C>;
    constexpr int bytes = C::STAGE_AREA + C::BM * 4;
    if (int rc = ensure_smem(kernel, bytes)) return rc;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(C::NT), bytes, st, p);
    HEXA_CHECK_LAUNCH("esmm16_dma");
    return HEXA_OK;
}

template <typename TC, typename C>
int launch_esmm_dma_d(EsmmK& p, int grid, bool io, bool o32, hipStream_t st) {
    if (o32) return io ? launch_esmm_dma_t<TC, true, true, C>(p, grid, st) : launch_esmm_dma_t<TC, false, true, C>(p, grid, st);
    return io ? launch_esmm_dma_t<TC, true, false, C>(p, grid, st) : launch_esmm_dma_t<TC, false, false, C>(p, grid, st);
}

// ------------------------------------------------------------------------------------------------
// ESTMM: dw[e][m][n] = sum over the expert's (slot, token) list of P[row][m] * Q[row][n]
// ------------------------------------------------------------------------------------------------
constexpr int MAX_SLOTS = 8;      // routing slots handled by this path
constexpr int TOK_RING = 8;       // steps of token ids kept in LDS (32 ids each)

struct EstmmK {
    const void* pm; const void* qm; void* dw;
    const int32_t* token_ids; const int32_t* offsets;
    int T, k, E, M, N, mtn, ntn;
    int p_slot_rows, q_slot_rows;
    int accumulate, group;
    int stream_dw;       // finished results (not the partial ones of split experts) leave with the non-temporal hint
    int off32;           // both operands below 4 GiB and 2^24 rows: rows may be addressed as base + 32-bit offset
    long total;
    const int* plan;     // non-null: units from estmm_plan_kernel (see there); scratch holds the partial results
    float* scratch;
};

// The work plan (see small_bodies.h) as a launch of its own.
__global__ __launch_bounds__(256) void estmm_plan_kernel(int* __restrict__ plan, const int32_t* __restrict__ offsets,
                                                         int E, int k, int cap, int max_slots) {
    extern __shared__ int sp[];
    estmm_plan_body(sp, plan, offsets, E, k, cap, max_slots);
}

__global__ __launch_bounds__(256) void estmm_fixup_kernel(FixupK p) { estmm_fixup_body(p, blockIdx.x); }

struct Cursor {   // walks the expert's token list in 32-token steps, slot after slot
    int s, r;
};

// fp32 result rows staged per pass, and the LDS area that holds both the stages and that staging
template <typename C> constexpr int estmm_pass_rows() {
    // the largest multiple-of-32 divisor of BM whose staged fp32 rows fit in the stage buffers, or in 34 KB where
    // those are smaller (64 rows of a 128-wide block: two passes instead of four for 2 KB more LDS per workgroup)
    constexpr int room = C::STAGE_AREA > 34 * 1024 ? C::STAGE_AREA : 34 * 1024;
    for (int rows = C::BM; rows > 32; rows /= 2)
        if (rows * (C::BN + 4) * 4 <= room) return rows;
    return 32;
}
template <typename C> constexpr int estmm_stage_area() {
    constexpr int staged = estmm_pass_rows<C>() * (C::BN + 4) * 4;
    return C::STAGE_AREA > staged ? C::STAGE_AREA : staged;
}

template <typename TC, bool OUT32, typename C>
__global__ __launch_bounds__(C::NT, C::MINW) void estmm16_dma_kernel(EstmmK p) {
    constexpr int BM = C::BM, BN = C::BN, STAGES = C::STAGES, NW = C::NW;
    static_assert(C::BKC == 32, "token ids travel 32 per step");
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    int* sIds = reinterpret_cast<int*>(smem + estmm_stage_area<C>());       // [TOK_RING][32]
    __shared__ int sBeg[MAX_SLOTS], sEnd[MAX_SLOTS];
    __shared__ int sExpert;

    const long logical = logical_tile(p.group);
    if (logical >= p.total) return;
    const int per_e = p.mtn * p.ntn;
    const int rank = (int)(logical / per_e);
    const int rem = (int)(logical - (long)rank * per_e);
    const int m0 = (rem / p.ntn) * BM, n0 = (rem % p.ntn) * BN;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wr = wave / C::WF, wf = wave % C::WF;
    const int M = p.M, N = p.N, T = p.T, nslot = p.k;

    // Heaviest experts first: workgroups are dispatched in id order, so giving the long token lists
    // to the first ones shortens the tail.  With a plan, `rank` numbers the plan's units (an expert or
    // one part of a busy expert); without, the expert of this workgroup is the one whose load has rank
    // `rank` (ties broken by index; up to 256 experts, beyond that the order is by index).
    int e = rank, part = 0, nparts = 1, slot = -1;
    if (p.plan) {
        __shared__ int sUnit[4];
        if (rank >= p.plan[4 * p.E]) return;
        for (int r = tid; r < p.E; r += C::NT) {
            const int u0 = p.plan[2 * p.E + r], n = p.plan[p.E + r];
            if (rank >= u0 && rank < u0 + n) { sUnit[0] = p.plan[r]; sUnit[1] = rank - u0; sUnit[2] = n; sUnit[3] = p.plan[3 * p.E + r]; }
        }
        __syncthreads();
        e = sUnit[0]; part = sUnit[1]; nparts = sUnit[2]; slot = sUnit[3];
    } else if (p.E <= 256) {
        __shared__ int sLoad[256];
        if (tid < p.E) {
            int t = 0;
            for (int s = 0; s < nslot; ++s)
                t += p.offsets[(size_t)s * (p.E + 1) + tid + 1] - p.offsets[(size_t)s * (p.E + 1) + tid];
            sLoad[tid] = t;
        }
        __syncthreads();
        if (tid < p.E) {
            const int mine = sLoad[tid];
            int r = 0;
            for (int x = 0; x < p.E; ++x) {
                const int o = sLoad[x];
                r += (o > mine || (o == mine && x < tid)) ? 1 : 0;
            }
            if (r == rank) sExpert = tid;
        }
        __syncthreads();
        e = sExpert;
    }

    if (tid < nslot) {
        sBeg[tid] = p.offsets[(size_t)tid * (p.E + 1) + e];
        sEnd[tid] = p.offsets[(size_t)tid * (p.E + 1) + e + 1];
    }
    __syncthreads();
    int all_steps = 0;
    for (int s = 0; s < nslot; ++s) all_steps += (sEnd[s] - sBeg[s] + BK - 1) / BK;
    // this workgroup's share of the expert's steps (all of them unless the expert was cut into parts)
    const int step0 = (int)((long)all_steps * part / nparts);
    const int nsteps = (int)((long)all_steps * (part + 1) / nparts) - step0;

    auto advance = [&](Cursor c) {
        c.r += BK;
        while (c.s < nslot && c.r >= sEnd[c.s]) { ++c.s; c.r = c.s < nslot ? sBeg[c.s] : 0; }
        return c;
    };
    auto first = [&]() {
        Cursor c; c.s = 0; c.r = sBeg[0];
        while (c.s < nslot && c.r >= sEnd[c.s]) { ++c.s; c.r = c.s < nslot ? sBeg[c.s] : 0; }
        for (int i = 0; i < step0; ++i) c = advance(c);
        return c;
    };

    const char* zero = reinterpret_cast<const char*>(g_zero_block);
    // token ids of one step: lanes 0..31 of every wavefront copy the same 32 ids (4 bytes each)
    auto issue_ids = [&](int step, Cursor c) {
        const int r = c.r + (lane & 31);
        const bool ok = c.s < nslot && r < sEnd[c.s < nslot ? c.s : 0];
        const int32_t* src = ok ? p.token_ids + (size_t)c.s * T + r : reinterpret_cast<const int32_t*>(zero);
        if (lane < 32)
            __builtin_amdgcn_global_load_lds((glb_ptr_t)src, (lds_ptr_t)(sIds + (step % TOK_RING) * 32), 4, 0, 0);
    };
    // operand tiles of one step (token ids of the step are already in LDS).  What does not change from step to step
    // -- which token of the step and which column piece a lane fetches -- is worked out once; a step whose 32 tokens
    // all exist, in a tile that lies inside the result, then costs one LDS read and ONE multiply-add per copy: the
    // row is addressed as (base of the slot's rows: scalar) + token * pitch + column offset in 32 bits (the launcher
    // keeps tensors of 4 GiB and more, and 2^24 rows and more, off this form).  The address arithmetic of the
    // general form (64-bit products, a block of zeros for lanes without a row) was most of this kernel's vector
    // instructions -- three times a plain ESMM's -- and it keeps that form for the last step of a token list and for
    // tiles on the result's edge.
    int kkR[C::R_CPW], chR[C::R_CPW], kkF[C::F_CPW], chF[C::F_CPW];
    unsigned colR[C::R_CPW], colF[C::F_CPW];
#pragma unroll
    for (int i = 0; i < C::R_CPW; ++i) {
        ks_lane<BM>(wave + NW * i, lane, kkR[i], chR[i]);
        colR[i] = (unsigned)(m0 + chR[i] * 8) * 2u;
    }
#pragma unroll
    for (int i = 0; i < C::F_CPW; ++i) {
        ks_lane<BN>(wave + NW * i, lane, kkF[i], chF[i]);
        colF[i] = (unsigned)(n0 + chF[i] * 8) * 2u;
    }
    const bool inner_tile = p.off32 && m0 + BM <= M && n0 + BN <= N;
    const unsigned pitchP = (unsigned)M * 2u, pitchQ = (unsigned)N * 2u;
    auto issue_data = [&](int step, Cursor c) {
        char* base = smem + (step % STAGES) * C::STAGE_BYTES;
        const unsigned ids = lds_addr(sIds + (step % TOK_RING) * 32);
        const int end = sEnd[c.s];
        int tokR[C::R_CPW], tokF[C::F_CPW];
#pragma unroll
        for (int i = 0; i < C::R_CPW; ++i) tokR[i] = lds_read_i32(ids + 4 * kkR[i]);
#pragma unroll
        for (int i = 0; i < C::F_CPW; ++i) tokF[i] = lds_read_i32(ids + 4 * kkF[i]);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (inner_tile && c.r + BK <= end) {
            const char* const pb = reinterpret_cast<const char*>(p.pm) + (size_t)p.p_slot_rows * c.s * pitchP;
            const char* const qb = reinterpret_cast<const char*>(p.qm) + (size_t)p.q_slot_rows * c.s * pitchQ;
#pragma unroll
            for (int i = 0; i < C::R_CPW; ++i) {
                int tok = tokR[i];
                asm volatile("" : "+v"(tok));   // consumed only after the wait above
                dma16(pb + (size_t)(__umul24((unsigned)tok, pitchP) + colR[i]), base + (wave + NW * i) * 1024);
            }
#pragma unroll
            for (int i = 0; i < C::F_CPW; ++i) {
                int tok = tokF[i];
                asm volatile("" : "+v"(tok));
                dma16(qb + (size_t)(__umul24((unsigned)tok, pitchQ) + colF[i]), base + C::R_BYTES + (wave + NW * i) * 1024);
            }
            return;
        }
#pragma unroll
        for (int i = 0; i < C::R_CPW; ++i) {
            int tok = tokR[i];
            asm volatile("" : "+v"(tok));
            const bool ok = (c.r + kkR[i] < end) && (m0 + chR[i] * 8 < M);
            const char* sp = ok ? reinterpret_cast<const char*>(p.pm) + (((size_t)p.p_slot_rows * c.s + tok) * M + m0 + chR[i] * 8) * 2 : zero;
            dma16(sp, base + (wave + NW * i) * 1024);
        }
#pragma unroll
        for (int i = 0; i < C::F_CPW; ++i) {
            int tok = tokF[i];
            asm volatile("" : "+v"(tok));
            const bool ok = (c.r + kkF[i] < end) && (n0 + chF[i] * 8 < N);
            const char* sq = ok ? reinterpret_cast<const char*>(p.qm) + (((size_t)p.q_slot_rows * c.s + tok) * N + n0 + chF[i] * 8) * 2 : zero;
            dma16(sq, base + C::R_BYTES + (wave + NW * i) * 1024);
        }
    };

    f32x16 acc[C::FB][C::RB];
    zero_acc(acc);
    if (nsteps > 0) {
        // Copy groups of CPW+1 per wavefront: { data(step x) [CPW copies], ids(step x + LEAD) [1 copy] }.
        // Group x is issued LEAD steps before step x is consumed, so when group kt has landed the ids
        // needed to issue data(kt + LEAD) are in LDS as well.
        constexpr int LEAD = STAGES - 1;
        Cursor cid = first();
        for (int st = 0; st < LEAD; ++st) { issue_ids(st, cid); cid = advance(cid); }
        wait_vmcnt<0>();
        Cursor cdat = first();
#pragma unroll
        for (int st = 0; st < LEAD; ++st) {
            if (st < nsteps) {
                issue_data(st, cdat); cdat = advance(cdat);
                issue_ids(st + LEAD, cid); cid = advance(cid);
            }
        }
        for (int kt = 0; kt < nsteps; ++kt) {
            wait_groups<C::CPW + 1, LEAD - 1>(min(nsteps - 1 - kt, LEAD - 1));   // groups issued after group kt
            barrier_nofence();
            const int jd = kt + LEAD;
            if (jd < nsteps) {
                issue_data(jd, cdat); cdat = advance(cdat);
                issue_ids(jd + LEAD, cid); cid = advance(cid);
            }
            const char* base = smem + (kt % STAGES) * C::STAGE_BYTES;
            mma_stage<TC, C, true, true>(base, base + C::R_BYTES, wr, wf, lane, acc);
        }
    } else if (p.accumulate && slot < 0) {
        return;
    }

    // ---- epilogue: lane holds row m = l%32 of a block and 4 consecutive n per group ----
    // The block leaves through LDS, PRF rows at a time (pitch BN+4 floats), so that BN/4 lanes write
    // one contiguous row of dw; 16-bit results are packed on the way out.
    const bool accumulate = p.accumulate != 0;
    typedef __attribute__((ext_vector_type(4))) float f4;
    typedef __attribute__((ext_vector_type(2))) unsigned u2;
    float* sC = reinterpret_cast<float*>(smem);
    constexpr int CPF = BN + 4;
    constexpr int PRF = estmm_pass_rows<C>();
    constexpr int LPRF = BN / 4;              // 16-byte (fp32) pieces per row
    constexpr int RW = 32 * C::RB, FW = 32 * C::FB;
#pragma unroll
    for (int h = 0; h < BM / PRF; ++h) {
        if (h == 0) barrier_nofence(); else __syncthreads();   // stage buffers / previous pass are free
#pragma unroll
        for (int i = 0; i < C::RB; ++i) {
            const int mb = wr * RW + i * 32;          // first row of this 32-row block inside the tile
            if (mb / PRF != h) continue;
            const int ml = mb - h * PRF + (lane & 31);
#pragma unroll
            for (int j = 0; j < C::FB; ++j) {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int nl = wf * FW + j * 32 + 8 * g + 4 * (lane >> 5);
                    *reinterpret_cast<float4*>(sC + ml * CPF + nl) =
                        make_float4(acc[j][i][4 * g], acc[j][i][4 * g + 1], acc[j][i][4 * g + 2], acc[j][i][4 * g + 3]);
                }
            }
        }
        __syncthreads();
        {
#pragma unroll 4
            for (int idx = tid; idx < PRF * LPRF; idx += C::NT) {
                const int ml = idx / LPRF, c = idx - ml * LPRF, n = n0 + c * 4;
                const int m = m0 + h * PRF + ml;
                if (m >= M || n >= N) continue;
                float4 v = *reinterpret_cast<const float4*>(sC + ml * CPF + c * 4);
                if (slot >= 0) {   // one part of a busy expert: fp32 partial result into its scratch slot
                    *reinterpret_cast<float4*>(p.scratch + ((size_t)(slot + part) * M + m) * N + n) = v;
                    continue;
                }
                const size_t off = ((size_t)e * M + m) * N + n;
                if (OUT32) {
                    float4* dst = reinterpret_cast<float4*>(reinterpret_cast<float*>(p.dw) + off);
                    if (accumulate) { const float4 old = *dst; v.x += old.x; v.y += old.y; v.z += old.z; v.w += old.w; }
                    if (p.stream_dw) { const f4 w4 = {v.x, v.y, v.z, v.w}; __builtin_nontemporal_store(w4, reinterpret_cast<f4*>(dst)); }
                    else *dst = v;
                } else {
                    uint2* dst = reinterpret_cast<uint2*>(reinterpret_cast<unsigned short*>(p.dw) + off);
                    if (accumulate) {
                        const uint2 old = *dst;
                        v.x += from_bits16<TC>(old.x & 0xffff); v.y += from_bits16<TC>(old.x >> 16);
                        v.z += from_bits16<TC>(old.y & 0xffff); v.w += from_bits16<TC>(old.y >> 16);
                    }
                    const uint2 pk = pack4<TC>(v.x, v.y, v.z, v.w);
                    if (p.stream_dw) { const u2 w2 = {pk.x, pk.y}; __builtin_nontemporal_store(w2, reinterpret_cast<u2*>(dst)); }
                    else *dst = pk;
                }
            }
        }
    }
}

template <typename TC, bool OUT32, typename C>
int launch_estmm_dma_t(EstmmK& p, int grid, hipStream_t st) {
    auto kernel = estmm16_dma_kernel<TC, OUT32, C>;
    constexpr int bytes = estmm_stage_area<C>() + TOK_RING * 32 * 4;
    if (int rc = ensure_smem(kernel, bytes)) return rc;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(C::NT), bytes, st, p);
    HEXA_CHECK_LAUNCH("estmm16_dma");
    return HEXA_OK;
}

template <typename C>
int launch_estmm_dma_c(const EstmmArgs& a, hipStream_t st) {
    EstmmK p;
    p.pm = a.p; p.qm = a.q; p.dw = a.dw;
    p.token_ids = a.r.token_ids; p.offsets = a.r.offsets;
    p.T = a.r.T; p.k = a.r.k; p.E = a.r.E; p.M = a.m_dim; p.N = a.n_dim;
    p.mtn = div_up(a.m_dim, C::BM); p.ntn = div_up(a.n_dim, C::BN);
    p.p_slot_rows = a.p_per_slot ? a.r.T : 0;
    p.q_slot_rows = a.q_per_slot ? a.r.T : 0;
    p.accumulate = a.accumulate;
    p.stream_dw = option(OPT_ESMM_STREAM) != 2;
    p.off32 = (size_t)a.r.T * a.r.k < ((size_t)1 << 24) && (size_t)a.r.T * (a.p_per_slot ? a.r.k : 1) * a.m_dim * 2 < ((size_t)1 << 32) &&
              (size_t)a.r.T * (a.q_per_slot ? a.r.k : 1) * a.n_dim * 2 < ((size_t)1 << 32) && a.m_dim * 2 < (1 << 24) && a.n_dim * 2 < (1 << 24);
    // Runs of `group` tiles per XCD (workgroup ids go round-robin over the 8 XCDs, each with its own L2).  Runs of 3
    // row tiles (with all their column tiles) cut the launch's HBM fetch at the benchmark shape from 340 to 230 MB
    // (1.28x the operands: the Q rows of an expert are then fetched by fewer L2s) at the same time, 97 against 99 us;
    // 4 fetch 202 MB and cost 3 %.  Results with few row tiles keep runs of one.
    p.group = p.ntn * (option(OPT_ESTMM_GROUP) > 0 ? option(OPT_ESTMM_GROUP) : (p.mtn >= 6 ? 3 : 1));
    p.plan = nullptr; p.scratch = nullptr;
    int units = a.r.E;
    const int E = a.r.E;
    const long mn = (long)a.m_dim * a.n_dim;
    if (a.plan && a.scratch && a.max_slots >= 2 && (mn & 3) == 0) {
        p.plan = a.plan;
        p.scratch = a.scratch;
        // a list cut into n parts adds n - 1 units and holds n >= 2 of the slots: at most max_slots - 1 more units
        // (workgroups past the plan's unit count leave at once, but tens of thousands of them are not free)
        units = E + (int)std::min<long>(a.max_slots - 1, (long)E * (PLAN_MAX_PARTS - 1));
    }
    p.total = (long)units * p.mtn * p.ntn;
    if (p.total == 0) return HEXA_OK;
    const int grid = round_up(p.total, 8 * p.group);
    const bool o32 = a.dw_dt == HEXA_F32;
    int rc;
    if (a.pq_dt == HEXA_BF16) rc = o32 ? launch_estmm_dma_t<__bf16, true, C>(p, grid, st) : launch_estmm_dma_t<__bf16, false, C>(p, grid, st);
    else rc = o32 ? launch_estmm_dma_t<_Float16, true, C>(p, grid, st) : launch_estmm_dma_t<_Float16, false, C>(p, grid, st);
    if (rc || !p.plan) return rc;
    return launch_estmm_fixup(a, st);
}

template <typename C>
int launch_esmm_dma_c(const EsmmArgs& a, bool large, hipStream_t st) {
    EsmmK p;
    p.x = a.x; p.w = a.w; p.bias = a.bias; p.out = a.out; p.out_act = a.out_act;
    p.token_ids = a.r.token_ids;
    p.tile_info = large ? a.r.tile_info_l : a.r.tile_info;
    p.tile_count = large ? a.r.tile_count_l : a.r.tile_count;
    p.mt_ub = large ? a.r.mt_ub_l : a.r.mt_ub;
    p.T = a.r.T; p.K = a.in_dim; p.N = a.out_dim;
    p.ntn = div_up(a.out_dim, C::BN);
    p.x_slot_rows = a.x_per_slot ? a.r.T : 0;
    p.out_slot_rows = a.out_per_slot ? a.r.T : 0;
    p.bias_dt = a.bias_dt; p.out_dt = a.out_dt; p.act = a.act;
    p.stream_out = option(OPT_ESMM_STREAM) == 1;
    p.colsum = a.colsum;
    p.group = p.ntn * (option(OPT_ESMM_GROUP) > 0 ? option(OPT_ESMM_GROUP) : (large ? 2 : 4));
    // Summing the slots into one result: with scratch, every slot runs in ONE launch (slot 0 into
    // `out`, the others into the scratch) and a reduction adds them in slot order; without it, one
    // launch per slot, each adding into `out`.
    const bool one_launch = a.out_per_slot || a.r.k == 1 || a.slot_ws != nullptr;
    p.ws = (!a.out_per_slot && a.r.k > 1) ? a.slot_ws : nullptr;
    const int launches = one_launch ? 1 : a.r.k;
    for (int l = 0; l < launches; ++l) {
        p.slot_begin = one_launch ? 0 : l;
        p.nslots = one_launch ? a.r.k : 1;
        p.accumulate = (a.accumulate || l > 0) ? 1 : 0;
        p.total = (long)p.nslots * p.mt_ub * p.ntn;
        if (p.total == 0) continue;
        // default: every XCD walks one contiguous eighth of the valid tiles (least re-fetching of weights and
        // token rows by several L2s); 2 selects runs of `group` tiles per XCD
        const bool contiguous = p.nslots <= 8 && option(OPT_ESMM_MAP) != 2;
        const int grid = round_up(p.total, contiguous ? 8 : 8 * p.group);
        if (contiguous) p.group = 0;
        const bool io = a.w_layout == HEXA_W_IN_OUT;
        const bool o32 = a.out_dt == HEXA_F32;
        const int rc = a.x_dt == HEXA_BF16 ? launch_esmm_dma_d<__bf16, C>(p, grid, io, o32, st)
                                           : launch_esmm_dma_d<_Float16, C>(p, grid, io, o32, st);
        if (rc) return rc;
    }
    if (p.ws) return launch_sum_slots(a.out, a.slot_ws, (int64_t)a.r.T * a.out_dim, a.r.k - 1, a.out_dt, st, a.sum_extra);
    if (a.colsum) return launch_colsum_fold(a, p.mt_ub, large ? HEXA_TILE_ROWS_L : HEXA_TILE_ROWS, p.ntn, C::BN, st);
    return HEXA_OK;
}

// HEXA_MOE_TILE (testing aid, read once): 0 automatic; 1 128x128; 2 256x128 (8 wavefronts); 3 256x128
// (4 wavefronts); 4..6 256x256 (4 / 8 / 16 wavefronts); 7 128x384; 8, 9 128x128 with 4 / 3 workgroups
// per CU; 10, 11 128x128 / 256x128 with 64 contraction indices per stage (ESMM only)
int forced_tile() { return option(OPT_TILE); }

int pick_esmm_tile(long rows, int cols, int in_dim) {
    const int f = forced_tile();
    if (f) return f;
    if (rows / 256 * div_up(cols, 128) >= 512) return 2;      // enough 256-row tiles to fill the chip
    return (in_dim % 64) == 0 ? 10 : 1;                       // whole 128-byte lines per row and stage when possible
}

}  // namespace

int launch_colsum_fold(const EsmmArgs& a, int mt_ub, int tile_rows, int ntn, int bn, hipStream_t st) {
    SmallTask t;
    t.kind = TASK_COLSUM_FOLD;
    t.colsum_fold = ColsumFoldK{a.db, a.colsum, a.r.offsets, a.r.E, mt_ub, tile_rows, ntn, bn, a.out_dim, a.r.k, a.db_dt,
                                a.db_accumulate, div_up(a.out_dim, 256)};
    t.blocks = t.colsum_fold.gx * a.r.E;
    if (!defer_task(defer_targets().colsum_fold, t)) {
        hipLaunchKernelGGL(esmm_colsum_fold_kernel, dim3(t.blocks), dim3(256), 0, st, t.colsum_fold);
        HEXA_CHECK_LAUNCH("esmm_colsum_fold");
    }
    return HEXA_OK;
}

// the task that adds the parts of the experts a plan has cut (a launch of its own unless a batch takes it)
int launch_estmm_fixup(const EstmmArgs& a, hipStream_t st) {
    const long mn = (long)a.m_dim * a.n_dim;
    SmallTask t;
    t.kind = TASK_FIXUP;
    t.fixup = FixupK{a.dw, a.plan, a.scratch, a.r.E, mn, a.dw_dt, a.accumulate, (int)((mn / 4 + 256 * FIXUP_PIECES - 1) / (256 * FIXUP_PIECES))};
    t.blocks = t.fixup.gx * std::min(a.r.E, std::max(1, a.max_slots / 2));   // (result piece, j-th cut expert)
    if (!defer_task(defer_targets().fixup, t)) {
        hipLaunchKernelGGL(estmm_fixup_kernel, dim3(t.blocks), dim3(256), 0, st, t.fixup);
        HEXA_CHECK_LAUNCH("estmm_fixup");
    }
    return HEXA_OK;
}

// The persistent kernel (one workgroup per CU, an item at a time at the CU's full rate) against the one-item-per-
// workgroup kernel (four workgroups per CU).  Alone, with its operands in the memory-side cache, the persistent kernel
// is the faster one (73 against 80 us + fix-up at 1152 rows per expert) and needs no fp32 partial results; inside a
// layer's backward, where every operand row comes from HBM, its two stages of copies in flight per CU (64 KB) do
// not cover the memory latency (a step waits 1900 instead of 1100 cycles for its rows) and it takes 86-89 us against
// 81-85, and with an item only one or two steps long its per-item cost loses outright (0.41 against 0.37 ms per
// layer at 72 rows per expert).  So it runs on request only (option "estmm_pipe" = 1).
bool estmm_pipe_wanted(const RouteView& r) {
    (void)r;
    return option(OPT_ESTMM_PIPE) == 1 && option(OPT_TILE) == 0;   // (a forced tile shape selects the one-item-per-workgroup kernels)
}

// Rows above which an expert's list is cut into parts (out_dim, in_dim = 0: unknown result size).  Both kernels hand
// their items out longest-first (the hardware's workgroup dispatcher does it for the one-item-per-workgroup kernel), so a
// cut only pays when one item would be longer than a workgroup slot's share of the launch: rows of all lists x blocks
// per expert / slots -- 256 for the persistent kernel, 1024 (four workgroups per CU, each at a quarter of the CU's
// rate) and never less than 1.5x the mean load for the other.
int estmm_plan_cap_for(const RouteView& r, int out_dim, int in_dim) {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 8)
        cus = 256;
    const int tiles = (out_dim > 0 && in_dim > 0) ? div_up(out_dim, 128) * div_up(in_dim, 128) : 0;
    if (estmm_pipe_wanted(r)) return estmm_plan_cap(r.T, r.k, r.E, tiles, cus);
    return std::max(estmm_plan_cap(r.T, r.k, r.E), tiles ? estmm_plan_cap(r.T, r.k, r.E, tiles, 4 * cus) : 0);
}

int launch_estmm_plan(int32_t* plan, const RouteView& r, int max_slots, int cap, hipStream_t st) {
    if (r.E > 4096) HEXA_FAIL(HEXA_ERR_UNSUPPORTED, "estmm plan: more than 4096 experts");
    hipLaunchKernelGGL(estmm_plan_kernel, dim3(1), dim3(256), 2 * r.E * sizeof(int), st, plan, r.offsets, r.E, r.k, cap,
                       max_slots);
    HEXA_CHECK_LAUNCH("estmm_plan");
    return HEXA_OK;
}

bool esmm16_dma_supported(const EsmmArgs& a) {
    // the copies address their operands as base + 32-bit byte offset: the row operand and one expert's weights
    // must each stay below 4 GiB
    const size_t x_rows = (size_t)a.r.T * (a.x_per_slot ? a.r.k : 1);
    const bool small = x_rows * a.in_dim * 2 < ((size_t)1 << 32) && (size_t)a.in_dim * a.out_dim * 2 < ((size_t)1 << 32);
    return small && a.w_dt == a.x_dt && (a.in_dim % 32) == 0 && (a.out_dim % 8) == 0 &&
           (a.out_dt == a.x_dt || a.out_dt == HEXA_F32);
}

bool estmm16_dma_supported(const EstmmArgs& a) {
    return a.r.k <= MAX_SLOTS && (a.m_dim % 8) == 0 && (a.n_dim % 8) == 0 && (a.dw_dt == a.pq_dt || a.dw_dt == HEXA_F32);
}

int launch_estmm16_dma(const EstmmArgs& a, hipStream_t st) {
    // a result up to 384 wide is spanned by ONE tile: the tall operand (m_dim columns of every token
    // row) is then fetched once instead of once per column tile
    // (measured: not a gain while the longest expert's token list bounds the kernel, so only on request)
    if (forced_tile() == 7) return launch_estmm_dma_c<CfgW>(a, st);
    switch (forced_tile()) {
        case 2: return launch_estmm_dma_c<CfgL>(a, st);
        case 3: return launch_estmm_dma_c<CfgM>(a, st);
        case 4: return launch_estmm_dma_c<CfgX>(a, st);
        case 5: return launch_estmm_dma_c<CfgX8>(a, st);
        case 6: return launch_estmm_dma_c<CfgX16>(a, st);
        case 8: return launch_estmm_dma_c<CfgS2>(a, st);
        case 9: return launch_estmm_dma_c<CfgS3>(a, st);
        case 1: return launch_estmm_dma_c<CfgS>(a, st);
        // Balanced units (a plan) or short token lists keep 4 workgroups per CU busy (measured at 72 rows per
        // expert, 3072 x 768: 105 -> 77 us); long lists without a plan are bounded by the busiest expert's
        // walk, where deeper staging per workgroup wins.
        default: {
            const long avg_rows = (long)a.r.T * a.r.k / std::max(1, a.r.E);
            return (a.plan || avg_rows < 512) ? launch_estmm_dma_c<CfgS2>(a, st) : launch_estmm_dma_c<CfgS>(a, st);
        }
    }
}

// The column sums ride on the store loop of the per-slot, 16-bit-result kernels (not
// the 128x384 tile, whose rows have 48 pieces); the pipelined kernel has its own.
// The pipelined persistent kernel runs whatever it covers (option "pipe": 2 = never, 1 = also when a tile shape is
// forced); the one-tile kernels run the rest.
// One exception by default: a plain launch (no fused activation) whose tiles come to between one and two per CU.  The
// persistent kernel gives every CU a whole number of tiles, so half the CUs would idle through the second half of
// the launch, while two one-tile workgroups share a CU at little loss (measured at 4608 rows, 3072 -> 768, 32
// experts: 62 against 67 us; below one tile per CU -- 2304 rows -- the persistent kernel wins, 39 against 52 us).
// The tile count is bounded from the host's side only (one partial tile per routing segment).
static bool use_pipe(const EsmmArgs& a) {
    const int o = option(OPT_PIPE);
    if (o == 2 || !(o == 1 || forced_tile() == 0) || !esmm16_pipe_supported(a)) return false;
    if (o == 0 && a.act == HEXA_ACT_NONE && !a.colsum) {
        int dev = 0, cus = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 8)
            cus = 256;
        const long tiles_ub = (long)a.r.k * a.r.mt_ub * div_up(a.out_dim, 128);
        if (4 * tiles_ub > 5 * (long)cus && tiles_ub <= 2 * (long)cus) return false;
    }
    return true;
}

bool esmm16_dma_colsum_supported(const EsmmArgs& a) {
    if (use_pipe(a)) return a.out_per_slot && a.r.k <= 8;
    return esmm16_dma_supported(a) && a.out_dt == a.x_dt && a.out_per_slot && a.r.k <= 8 && forced_tile() != 7;
}

int launch_esmm16_dma(const EsmmArgs& a, hipStream_t st) {
    if (use_pipe(a)) return launch_esmm16_pipe(a, st);
    if (forced_tile() == 7) return launch_esmm_dma_c<CfgW>(a, false, st);
    switch (pick_esmm_tile((long)a.r.T * a.r.k, a.out_dim, a.in_dim)) {
        case 2: return launch_esmm_dma_c<CfgL>(a, true, st);
        case 3: return launch_esmm_dma_c<CfgM>(a, true, st);
        case 4: return launch_esmm_dma_c<CfgX>(a, true, st);
        case 5: return launch_esmm_dma_c<CfgX8>(a, true, st);
        case 6: return launch_esmm_dma_c<CfgX16>(a, true, st);
        case 8: return launch_esmm_dma_c<CfgS2>(a, false, st);
        case 10: return (a.in_dim % 64) ? launch_esmm_dma_c<CfgS>(a, false, st) : launch_esmm_dma_c<CfgS64>(a, false, st);
        case 11: return (a.in_dim % 64) ? launch_esmm_dma_c<CfgL>(a, true, st) : launch_esmm_dma_c<CfgL64>(a, true, st);
        case 12: return (a.in_dim % 64) ? launch_esmm_dma_c<CfgS>(a, false, st) : launch_esmm_dma_c<CfgS64W>(a, false, st);
        case 13: return (a.in_dim % 64) ? launch_esmm_dma_c<CfgS>(a, false, st) : launch_esmm_dma_c<CfgS64H>(a, false, st);
        case 9: return launch_esmm_dma_c<CfgS3>(a, false, st);
        default: return launch_esmm_dma_c<CfgS>(a, false, st);
    }
}

}  // namespace hexa
