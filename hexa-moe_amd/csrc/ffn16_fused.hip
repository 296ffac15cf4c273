// One-kernel forward of the MoE FFN for bf16 / fp16 on gfx950: y = sum over slots of gelu(x . W1[e]^T + b1[e]) . W2[e]
// + b2[e], with the pre-activation y1 and the activation y2 written out for the backward as they are made.
//
// A workgroup owns 64 routed token rows of one (slot, expert) segment and walks the hidden dimension in chunks of
// 128 columns.  Per chunk:
//   A  y1 chunk [64 x 128] = x rows [64 x d_in] . W1[e][chunk][d_in]^T   (MFMA, 64 contraction indices per step;
//      x rows and the W1 chunk stream from L2 through two LDS stages by asynchronous copies)
//   E  + b1, rounded; the chunk goes through LDS once: every lane takes 16-byte row pieces, stores y1, applies
//      GELU, stores y2 and leaves y2 in LDS in the layout of an MFMA row operand
//   B  out [64 x d_out] += y2 chunk [64 x 128] . W2[e][chunk rows][d_out]  (MFMA, 32 contraction indices per step,
//      W2 slices through the same two stages); the output tile stays in accumulators over all chunks
// and at the end + b2, rounded, stored (slot 0 into y, the other slots into scratch that a small kernel adds in
// slot order, as hexa_esmm does).  Against the two-launch form this saves the second launch's read of y2 from
// HBM (T*k*hidden elements), its gather prologue per tile and the launch itself; what it costs is that each 64-row
// tile streams the expert's whole W1 and W2 through the memory pipeline (2.4 MB at d=384, h=1536 -- the tile is
// narrow because a 64 x d_out fp32 output tile plus the chunk's accumulators is what the registers hold).
//
// Covers: x, W1, W2, y* of one 16-bit type; d_in a multiple of 64; hidden a multiple of 128; d_out one of 128, 256,
// 384, 512; up to 8 slots.  Everything else stays on the two-launch path.
//
// Replaces the forward of FusedMoE_Shared_CudaCore for the exact GELU (impls/layers.py:256-274: ESMM, activation,
// ESMM, sum over the slots).
#include <algorithm>
#include <utility>

#include "dma_common.h"

namespace hexa {
namespace {

struct FfnK {
    const void* x; const void* w1; const void* b1; const void* w2; const void* b2;
    void* y1; void* y2; void* y; void* ws;
    const int32_t* token_ids; const int4* tile_info; const int32_t* tile_count;
    int T, d_in, hidden, d_out, mt_ub, nslots, b1_dt, b2_dt;
};

constexpr int FFN_BM = 64, FFN_CH = 128, FFN_NT = 512, FFN_NW = 8;
constexpr int FFN_STAGE_A = (FFN_BM + FFN_CH) * 64 * 2;        // x rows + W1 chunk, 64 contraction indices: 24 KiB

template <int DOUT> struct FfnLds {
    static constexpr int STAGE_B = 32 * DOUT * 2;               // W2 slice: 32 hidden indices x d_out
    static constexpr int STAGE = STAGE_B > FFN_STAGE_A ? STAGE_B : FFN_STAGE_A;
    static constexpr int CP1 = FFN_CH * 2 + 16;                 // pitch of the staged y1 chunk
    static constexpr int CHUNK_AT = 2 * STAGE;                  // staged y1 chunk, then the y2 operand [2][64][64]
    static constexpr int TOK_AT = CHUNK_AT + FFN_BM * CP1;
    static constexpr int BYTES = TOK_AT + FFN_BM * 4;
    static constexpr int CPO = DOUT * 2 + 16;                   // pitch of the staged output tile
    static_assert(FFN_BM * CPO <= TOK_AT, "the staged output tile reuses the stages and the chunk area");
};

template <typename TC, int DOUT>
__global__ __launch_bounds__(FFN_NT, 4) void ffn16_fwd_kernel(FfnK p) {
    using V = typename Mfma<TC>::V;
    using L = FfnLds<DOUT>;
    constexpr int FB2 = DOUT / 128;                             // 32-column blocks per wavefront in step B
    constexpr int B_COPIES = L::STAGE_B / 1024, B_CPW = B_COPIES / FFN_NW;
    static_assert(B_COPIES % FFN_NW == 0, "W2 slice copies must divide over the wavefronts");
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    int* sTok = reinterpret_cast<int*>(smem + L::TOK_AT);

    // ---- this workgroup's rows: half of a 128-row tile record ----
    int cum[9];
    cum[0] = 0;
#pragma unroll
    for (int q = 0; q < 8; ++q) cum[q + 1] = cum[q] + (q < p.nslots ? min(p.tile_count[q], p.mt_ub) : 0);
    const int unit = blockIdx.x;
    const int mtg = unit >> 1, half = unit & 1;
    if (mtg >= cum[8]) return;
    int s = 0;
#pragma unroll
    for (int q = 1; q < 8; ++q) s += (mtg >= cum[q] && q < p.nslots) ? 1 : 0;
    const int4 info = p.tile_info[(size_t)s * p.mt_ub + (mtg - cum[s])];
    const int e = info.x, row_start = info.y + half * FFN_BM, rows = min(FFN_BM, info.z - half * FFN_BM);
    if (rows <= 0) return;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int K1 = p.d_in, H = p.hidden, T = p.T;
    if (tid < FFN_BM) sTok[tid] = tid < rows ? p.token_ids[(size_t)s * T + row_start + tid] : -1;
    __syncthreads();

    const char* zero = reinterpret_cast<const char*>(g_zero_block);
    // ---- copy sources ----
    // step A: x rows (KC, 8 copies: one per wavefront) and the W1 chunk (KC, 16 copies: two per wavefront)
    int rowA, kcA;
    kc_lane<64>(wave, lane, rowA, kcA);
    const int tokA = sTok[rowA];
    const char* srcX0 = tokA >= 0 ? reinterpret_cast<const char*>(p.x) + ((size_t)tokA * K1 + kcA * 8) * 2 : zero;
    const int stepX = tokA >= 0 ? 128 : 0;
    int rowW[2], kcW[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) kc_lane<64>(wave + FFN_NW * i, lane, rowW[i], kcW[i]);
    // step B: W2 slice (KS of width DOUT): [32 hidden indices][DOUT]
    int kkB[B_CPW], chB[B_CPW];
#pragma unroll
    for (int i = 0; i < B_CPW; ++i) ks_lane<DOUT>(wave + FFN_NW * i, lane, kkB[i], chB[i]);

    // wavefront layout: A 2 x 4 wavefronts of 32 x 32; B 2 x 4 wavefronts of 32 x (DOUT / 4)
    const int wr = wave >> 2, wc = wave & 3;
    f32x16 acc2[FB2];
#pragma unroll
    for (int j = 0; j < FB2; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc2[j][v] = 0.f;

    const int nkA = K1 / 64, nchunks = H / FFN_CH;
    const size_t hid_base = ((size_t)T * s) * H;                   // y1 / y2 are [k][T][hidden]
    for (int ch = 0; ch < nchunks; ++ch) {
        const int h0 = ch * FFN_CH;
        // ================= A: y1 chunk =================
        const char* srcX = srcX0;
        const char* srcW[2];
#pragma unroll
        for (int i = 0; i < 2; ++i)
            srcW[i] = reinterpret_cast<const char*>(p.w1) + (((size_t)e * H + h0 + rowW[i]) * K1 + kcW[i] * 8) * 2;
        auto issueA = [&](int stage) {
            char* base = smem + stage * L::STAGE;
            dma16(srcX, base + wave * 1024);
            srcX += stepX;
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                dma16(srcW[i], base + FFN_BM * 128 + (wave + FFN_NW * i) * 1024);
                srcW[i] += 128;
            }
        };
        f32x16 acc1;
#pragma unroll
        for (int v = 0; v < 16; ++v) acc1[v] = 0.f;
        __syncthreads();                                       // the stages (and the chunk area) are free
        issueA(0);
        for (int kt = 0; kt < nkA; ++kt) {
            wait_vmcnt<0>();
            barrier_nofence();
            if (kt + 1 < nkA) issueA((kt + 1) & 1);
            const char* tX = smem + (kt & 1) * L::STAGE;
            const char* tW = tX + FFN_BM * 128;
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
                const V f = frag_kc<V, 64>(tW, wc * 32, ks, lane);   // the fast output dimension: hidden columns
                const V r = frag_kc<V, 64>(tX, wr * 32, ks, lane);   // token rows
                acc1 = Mfma<TC>::run(f, r, acc1);
            }
        }
        // ================= E: bias, rounding, y1 / y2 out, y2 as the next operand =================
        // lane holds token row wr*32 + lane%32 and, per group g, 4 consecutive hidden columns wc*32 + 8g + 4*(lane/32)
        {
            char* chunk = smem + L::CHUNK_AT;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int nl = wc * 32 + 8 * g + 4 * (lane >> 5);
                float bv[4] = {0.f, 0.f, 0.f, 0.f};
                if (p.b1) {
                    if (p.b1_dt == HEXA_F32) {
                        const float4 b4 = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(p.b1) + (size_t)e * H + h0 + nl);
                        bv[0] = b4.x; bv[1] = b4.y; bv[2] = b4.z; bv[3] = b4.w;
                    } else {
                        const uint2 b2 = *reinterpret_cast<const uint2*>(reinterpret_cast<const unsigned short*>(p.b1) + (size_t)e * H + h0 + nl);
                        bv[0] = from_bits16<TC>(b2.x & 0xffff); bv[1] = from_bits16<TC>(b2.x >> 16);
                        bv[2] = from_bits16<TC>(b2.y & 0xffff); bv[3] = from_bits16<TC>(b2.y >> 16);
                    }
                }
                const int rl = wr * 32 + (lane & 31);
                *reinterpret_cast<uint2*>(chunk + rl * L::CP1 + nl * 2) =
                    pack4<TC>(acc1[4 * g] + bv[0], acc1[4 * g + 1] + bv[1], acc1[4 * g + 2] + bv[2], acc1[4 * g + 3] + bv[3]);
            }
        }
        __syncthreads();
        {
            // 64 rows x 16 pieces of 16 bytes = 1024 pieces, two per lane; both are read before the chunk area is rewritten
            const char* chunk = smem + L::CHUNK_AT;
            uint4 val[2]; int rl[2], c[2];
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                const int idx = tid + q * FFN_NT;
                rl[q] = idx >> 4; c[q] = idx & 15;
                val[q] = *reinterpret_cast<const uint4*>(chunk + rl[q] * L::CP1 + c[q] * 16);
            }
            __syncthreads();                                   // everyone holds its pieces: the area can take y2
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                const int tok = sTok[rl[q]];
                unsigned vw[4] = {val[q].x, val[q].y, val[q].z, val[q].w}, aw[4];
#pragma unroll
                for (int u = 0; u < 4; ++u)   // applied to the value as stored (rounded), like act(y1) on the tensor
                    aw[u] = pack2<TC>(gelu_fast(from_bits16<TC>(vw[u] & 0xffff)), gelu_fast(from_bits16<TC>(vw[u] >> 16)));
                const uint4 act = make_uint4(aw[0], aw[1], aw[2], aw[3]);
                if (tok >= 0) {
                    const size_t off = (hid_base + (size_t)tok * H) + h0 + c[q] * 8;
                    store16(reinterpret_cast<uint4*>(reinterpret_cast<unsigned short*>(p.y1) + off), val[q], false);
                    store16(reinterpret_cast<uint4*>(reinterpret_cast<unsigned short*>(p.y2) + off), act, false);
                }
                // y2 as a KC operand: two [64 rows][64 k] sub-tiles; piece c of a row = 8 hidden indices
                const int sub = c[q] >> 3, pc = c[q] & 7;
                const int pos = pc ^ kc_swizzle<64>(rl[q]);
                *reinterpret_cast<uint4*>(smem + L::CHUNK_AT + sub * (FFN_BM * 128) + rl[q] * 128 + pos * 16) =
                    tok >= 0 ? act : make_uint4(0u, 0u, 0u, 0u);
            }
        }
        // ================= B: out += y2 chunk . W2[e][h0 .. h0+128][:] =================
        const char* srcB[B_CPW];
#pragma unroll
        for (int i = 0; i < B_CPW; ++i)
            srcB[i] = reinterpret_cast<const char*>(p.w2) + (((size_t)e * H + h0 + kkB[i]) * DOUT + chB[i] * 8) * 2;
        auto issueB = [&](int stage) {
            char* base = smem + stage * L::STAGE;
#pragma unroll
            for (int i = 0; i < B_CPW; ++i) {
                dma16(srcB[i], base + (wave + FFN_NW * i) * 1024);
                srcB[i] += (size_t)32 * DOUT * 2;
            }
        };
        __syncthreads();                                       // y2 operand complete; the stages are free
        issueB(0);
#pragma unroll 1
        for (int kt = 0; kt < FFN_CH / 32; ++kt) {
            wait_vmcnt<0>();
            barrier_nofence();
            if (kt + 1 < FFN_CH / 32) issueB((kt + 1) & 1);
            const char* tW = smem + (kt & 1) * L::STAGE;
            const char* tY = smem + L::CHUNK_AT + (kt >> 1) * (FFN_BM * 128);   // sub-tile of 64 hidden indices
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                V f[FB2];
#pragma unroll
                for (int j = 0; j < FB2; ++j) f[j] = frag_ks<V, DOUT>(tW, wc * (32 * FB2) + j * 32, ks, lane);
                V r[1];
                r[0] = frag_kc<V, 64>(tY, wr * 32, (kt & 1) * 2 + ks, lane);
                lds_fence_all(f, r);
#pragma unroll
                for (int j = 0; j < FB2; ++j) acc2[j] = Mfma<TC>::run(f[j], r[0], acc2[j]);
            }
        }
    }

    // ================= output tile: + b2, rounded, through LDS, 16-byte row pieces =================
    __syncthreads();
    {
        const bool to_ws = p.ws != nullptr && s > 0;
        unsigned short* outp = reinterpret_cast<unsigned short*>(to_ws ? p.ws : p.y);
        const size_t out_base = to_ws ? (size_t)T * (s - 1) : 0;
#pragma unroll
        for (int j = 0; j < FB2; ++j) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int nl = wc * (32 * FB2) + j * 32 + 8 * g + 4 * (lane >> 5);
                float bv[4] = {0.f, 0.f, 0.f, 0.f};
                if (p.b2) {
                    if (p.b2_dt == HEXA_F32) {
                        const float4 b4 = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(p.b2) + (size_t)e * DOUT + nl);
                        bv[0] = b4.x; bv[1] = b4.y; bv[2] = b4.z; bv[3] = b4.w;
                    } else {
                        const uint2 b2 = *reinterpret_cast<const uint2*>(reinterpret_cast<const unsigned short*>(p.b2) + (size_t)e * DOUT + nl);
                        bv[0] = from_bits16<TC>(b2.x & 0xffff); bv[1] = from_bits16<TC>(b2.x >> 16);
                        bv[2] = from_bits16<TC>(b2.y & 0xffff); bv[3] = from_bits16<TC>(b2.y >> 16);
                    }
                }
                const int rl = wr * 32 + (lane & 31);
                *reinterpret_cast<uint2*>(smem + rl * L::CPO + nl * 2) =
                    pack4<TC>(acc2[j][4 * g] + bv[0], acc2[j][4 * g + 1] + bv[1], acc2[j][4 * g + 2] + bv[2], acc2[j][4 * g + 3] + bv[3]);
            }
        }
        __syncthreads();
        constexpr int LPR = DOUT / 8;
        for (int idx = tid; idx < FFN_BM * LPR; idx += FFN_NT) {
            const int rl = idx / LPR, c = idx - rl * LPR;
            const int tok = sTok[rl];
            if (tok < 0) continue;
            const uint4 val = *reinterpret_cast<const uint4*>(smem + rl * L::CPO + c * 16);
            store16(reinterpret_cast<uint4*>(outp + (out_base + tok) * DOUT + c * 8), val, false);
        }
    }
}

template <typename TC, int DOUT>
int launch_ffn_t(FfnK& p, int grid, hipStream_t st) {
    auto kernel = ffn16_fwd_kernel<TC, DOUT>;
    constexpr int bytes = FfnLds<DOUT>::BYTES;
    if (int rc = ensure_smem(kernel, bytes)) return rc;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(FFN_NT), bytes, st, p);
    HEXA_CHECK_LAUNCH("ffn16_fwd");
    return HEXA_OK;
}

template <typename TC>
int launch_ffn_d(FfnK& p, int grid, hipStream_t st) {
    switch (p.d_out) {
        case 128: return launch_ffn_t<TC, 128>(p, grid, st);
        case 256: return launch_ffn_t<TC, 256>(p, grid, st);
        case 384: return launch_ffn_t<TC, 384>(p, grid, st);
        case 512: return launch_ffn_t<TC, 512>(p, grid, st);
    }
    HEXA_FAIL(HEXA_ERR_UNSUPPORTED, "fused FFN forward: d_out must be 128, 256, 384 or 512 (got %d)", p.d_out);
}

}  // namespace

bool ffn16_fused_supported(int T, int k, int d_in, int hidden, int d_out, int act_dt, int w_dt, int b1_dt, int b2_dt) {
    return T > 0 && k <= 8 && (act_dt == HEXA_BF16 || act_dt == HEXA_F16) && w_dt == act_dt &&
           (b1_dt == HEXA_F32 || b1_dt == act_dt) && (b2_dt == HEXA_F32 || b2_dt == act_dt) && (d_in % 64) == 0 && d_in >= 64 &&
           (hidden % FFN_CH) == 0 && (d_out == 128 || d_out == 256 || d_out == 384 || d_out == 512);
}

// y1, y2 [k][T][hidden]; y [T][d_out]; slot_ws [(k-1)][T][d_out] (needed when k > 1)
int launch_ffn16_fused(void* y1, void* y2, void* y, const void* x, const void* w1, const void* b1, const void* w2,
                       const void* b2, const RouteView& r, int d_in, int hidden, int d_out, int act_dt, int b1_dt,
                       int b2_dt, void* slot_ws, hipStream_t st) {
    if (r.k > 1 && !slot_ws) HEXA_FAIL(HEXA_ERR_ARG, "fused FFN forward: scratch for the slot sum is missing");
    FfnK p;
    p.x = x; p.w1 = w1; p.b1 = b1; p.w2 = w2; p.b2 = b2; p.y1 = y1; p.y2 = y2; p.y = y; p.ws = r.k > 1 ? slot_ws : nullptr;
    p.token_ids = r.token_ids; p.tile_info = r.tile_info; p.tile_count = r.tile_count;
    p.T = r.T; p.d_in = d_in; p.hidden = hidden; p.d_out = d_out; p.mt_ub = r.mt_ub; p.nslots = r.k;
    p.b1_dt = b1_dt; p.b2_dt = b2_dt;
    const long units = 2L * r.k * r.mt_ub;                    // two 64-row halves per 128-row tile record
    if (units == 0) return HEXA_OK;
    const int rc = act_dt == HEXA_BF16 ? launch_ffn_d<__bf16>(p, (int)units, st) : launch_ffn_d<_Float16>(p, (int)units, st);
    if (rc) return rc;
    if (r.k > 1) return launch_sum_slots(y, slot_ws, (int64_t)r.T * d_out, r.k - 1, act_dt, st);
    return HEXA_OK;
}

}  // namespace hexa
