// Pipelined persistent ESMM for bf16 / fp16 on gfx950: one workgroup of 16 wavefronts per CU walks a list of
// tiles, and the three phases a one-tile-per-workgroup kernel runs one after the other -- gathering operands,
// MFMA main loop, activation + store epilogue -- run side by side on different wavefronts:
//
//   * 4 "multiply" wavefronts (2 x 2, 64 x 64 results each, one per SIMD): LDS fragment reads and
//     v_mfma_f32_32x32x16, nothing else.  They never touch global memory, so they never wait for it.
//   * 4 "copy" wavefronts issue every asynchronous global->LDS copy (three stages deep, the pipeline never drains
//     between tiles: the first stages of the next tile are issued during the last steps of the current one; the
//     next tile's token ids and bias arrive by copy a whole tile ahead; the tile records of the workgroup's whole
//     walk sit in LDS from the start).  They issue no stores, so their vmcnt counter only ever sees copies and the
//     waits for a stage are exact.
//   * 8 "store" wavefronts take the previous tile's rounded result out of an LDS staging area, apply the
//     activation (GELU with a second output, or the GELU' factor read from the forward's pre-activation), and
//     store 16-byte row pieces, spread over the main-loop steps of the tile that is being multiplied.
//
// In a one-tile-per-workgroup kernel every wavefront first queues for the memory pipeline to issue its copies
// and then multiplies, with a barrier between steps; measured, a 12-step tile spends about as long issuing
// copies as multiplying, plus a prologue of dependent loads and an epilogue whose GELU arithmetic equals the
// tile's MFMA work.  Here copy issue, MFMAs and epilogue overlap, and a step costs what the slowest of them needs.
//
// The groups meet at one barrier per main-loop step (which publishes a stage) and one more per tile, after which
// the multiply wavefronts hand their accumulators (+ bias, rounded) to the staging area.
//
// LDS accesses outside the MFMA fragment reads are inline assembly: a compiler-visible LDS access next to
// copies in flight may be ordered behind them with s_waitcnt vmcnt(0), which would drain the pipeline.
//
// Covers: 16-bit operands and result, weights of the operands' type, in_dim a multiple of 64 and >= 256,
// out_dim a multiple of 8, per-slot results (with or without activation / column sums; plain ones also
// accumulating) and slot-summed results through scratch.  Everything else stays on esmm16_dma_kernel.
//
// Replaces esmm_shared_tensor_kernel_vectorized_accum_half (kernels/esmm_half.cu) and the ESMM task of the
// fused backward kernels (kernels/fused_ops_half.cu) for the cases above.
#include <algorithm>
#include <type_traits>
#include <utility>

#include "pipe_common.h"

namespace hexa {
namespace {

constexpr int PIPE_MAX_ROUNDS = 256;   // tiles one workgroup may walk (their records are kept in LDS)

#ifndef PIPE_WR
#define PIPE_WR 2
#define PIPE_RB 2
#endif
using CfgP = Cfg<PIPE_WR, 2, PIPE_RB, 2, 3, 3, 64>;   // 128 x 128: 4 multiply wavefronts of 64 x 64, 3 stages of 64 contraction indices

// GELU and GELU' of a value that has been rounded to bf16 are functions of 16 bits.  The store wavefronts look them up
// in a table the workgroup builds at its start instead of evaluating them: every magnitude from LUT_M_LO (2^-17, or
// 2^-14 where LDS is short) up to (not including) 8, both signs, the polynomial's own results (so nothing changes in
// any bit), as bf16 for GELU and as fp32 for GELU' (which is multiplied before rounding).  Entry 2 * (magnitude bits
// - LUT_M_LO) + sign: the two 16-bit values of a 32-bit word are turned into two table addresses with packed 16-bit
// arithmetic (four vector instructions per element instead of nine).  A piece with a value outside that range
// (zeros, |x| >= 8, NaN) takes the polynomial: one wavefront-wide branch per 16-byte piece.
constexpr unsigned LUT_M_HI = 0x4100;
template <typename TC, int ACT, bool COLSUM> constexpr unsigned pipe_lut_lo() {
    // GELU' with column sums: fp32 entries next to the column-sum area leave room for magnitudes from 2^-14 only
    return ACT == HEXA_ACT_GELU_BWD && COLSUM ? 0x3880u : 0x3700u;
}
template <typename TC, int ACT, bool COLSUM> constexpr int pipe_lut_bytes() {
    constexpr int r = (int)(LUT_M_HI - pipe_lut_lo<TC, ACT, COLSUM>());
    return !std::is_same<TC, __bf16>::value ? 0 : ACT == HEXA_ACT_GELU ? 2 * r * 2 : ACT == HEXA_ACT_GELU_BWD ? 2 * r * 4 : 0;
}
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ u16x2 as_u16x2(unsigned w) {
    union { unsigned u; u16x2 v; } c;
    c.u = w;
    return c.v;
}
__device__ __forceinline__ unsigned as_u32(u16x2 v) {
    union { unsigned u; u16x2 v; } c;
    c.v = v;
    return c.u;
}
// The table positions (as byte offsets, entries of 1 << SH bytes) of the two 16-bit values of w, packed in one word;
// `far` collects the largest distance from the table's first magnitude (a magnitude below it wraps to a huge
// one), so far >= the table's length says some value is outside.
template <unsigned LO, int SH> __device__ __forceinline__ unsigned lut_offsets(unsigned w, u16x2& far) {
    const u16x2 lo2 = {(unsigned short)LO, (unsigned short)LO};
    const u16x2 u = as_u16x2(w & 0x7fff7fffu) - lo2;
    far = __builtin_elementwise_max(far, u);
    const u16x2 sh = {(unsigned short)(SH + 1), (unsigned short)(SH + 1)};
    return as_u32(u << sh) | ((w >> (15 - SH)) & ((1u << SH) * 0x00010001u));
}
// (the 16-bit LDS loads that target one half of a register clear the other half on this chip, so two entries
// are read into two registers and joined with one shift-or)
template <int OFF> __device__ __forceinline__ unsigned lds_read_u16_async(unsigned addr) {
    unsigned r;
    asm volatile("ds_read_u16 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF));
    return r;
}

struct PipeK {
    EsmmK e;
    int wg_per_xcd;       // workgroups per XCD (grid = 8 * wg_per_xcd)
};

#ifndef PIPE_CW
#define PIPE_CW 4
#define PIPE_SW 8
#endif
constexpr int PIPE_COPY_WAVES = PIPE_CW, PIPE_STORE_WAVES = PIPE_SW;

// LUT: bytes of the activation table (0 = none).  The table comes first: its entries are addressed with 16-bit
// offsets from the start of the workgroup's LDS.
template <typename C, int LUT = 0, bool COLSUM = true> struct PipeLds {
    static constexpr int CP = C::BN * 2 + 16;                 // pitch of a staged 16-bit result row
    static constexpr int LUT_AT = 0;
    static constexpr int STAGES_AT = (LUT + 1023) / 1024 * 1024;
    static constexpr int STAGING_AT = STAGES_AT + C::STAGE_AREA;
    static constexpr int TOK_AT = STAGING_AT + C::BM * CP;    // 3 x BM token ids
    static constexpr int BIAS_SLOT = 1024;                    // one wavefront copy (64 lanes x 16 bytes) per slot
    static constexpr int BIAS_AT = TOK_AT + 3 * C::BM * 4;    // 3 slots of raw bias elements (BN x 4 bytes used at most)
    static constexpr int INFO_AT = BIAS_AT + 3 * BIAS_SLOT;   // PIPE_MAX_ROUNDS x int4
    static constexpr int RED_AT = INFO_AT + PIPE_MAX_ROUNDS * 16;   // column-sum partials: store wavefronts x BN floats
    static constexpr int SINK_AT = RED_AT + (COLSUM ? PIPE_STORE_WAVES * C::BN * 4 : 0);    // 256 bytes nobody reads (filler copies)
    static constexpr int BYTES = SINK_AT + 256;
    static_assert(BYTES <= 160 * 1024, "LDS of a CU");
    static_assert(C::BN * 4 <= BIAS_SLOT, "bias slot");
    static_assert(LUT < 65536, "table offsets are 16 bits");
};

// ACT: HEXA_ACT_NONE / _GELU / _GELU_BWD.  COLSUM: also per-tile column sums of the stored result.
template <typename TC, bool W_IN_OUT, int ACT, bool COLSUM, typename C>
__global__ __launch_bounds__(C::NT + 64 * (PIPE_COPY_WAVES + PIPE_STORE_WAVES)) void esmm16_pipe_kernel(PipeK pk) {
    const EsmmK& p = pk.e;
    constexpr int BM = C::BM, BN = C::BN, STAGES = C::STAGES, NW = C::NW, BK = C::BKC;
    constexpr int CW = PIPE_COPY_WAVES, SW = PIPE_STORE_WAVES, NTS = 64 * SW, NT_ALL = C::NT + 64 * (CW + SW);
    constexpr int R_CPW = C::R_COPIES / CW, F_CPW = C::F_COPIES / CW, CPW = R_CPW + F_CPW;   // copies per copy wavefront and stage
    static_assert(C::R_COPIES % CW == 0 && C::F_COPIES % CW == 0, "copies must divide evenly over the copy wavefronts");
    static_assert(BM <= 64 * CW, "at most one 64-id copy per copy wavefront");
    constexpr int LUT = pipe_lut_bytes<TC, ACT, COLSUM>();
    constexpr unsigned LUT_LO = pipe_lut_lo<TC, ACT, COLSUM>(), LUT_R = LUT_M_HI - LUT_LO;
    using L = PipeLds<C, LUT, COLSUM>;
    constexpr int CP = L::CP;
    constexpr int LPR = BN / 8;                         // 16-byte pieces per staged row
    constexpr int PIECES = BM * LPR / NTS;              // pieces per store lane and tile
    constexpr int PROWS = NTS / LPR;                    // rows between a lane's consecutive pieces
    static_assert(BM * LPR % NTS == 0 && NTS % LPR == 0 && 64 % LPR == 0 && BN <= 64 * CW, "store lanes must tile the staged result");
    static_assert((PIECES - 1) * PROWS * CP < 65536, "piece offsets must fit the LDS offset field");
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    const unsigned lds0 = lds_addr(smem);

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int K = p.K, N = p.N, nk = K / BK;
    const bool streaming = p.stream_out != 0;           // results leave with the non-temporal hint

    // ---- this workgroup's walk: XCD x owns one contiguous eighth of the valid tiles (column tiles fastest);
    // the workgroups of an XCD take its tiles round-robin, so at any time they share token rows and weights
    int cum[9];
    cum[0] = 0;
#pragma unroll
    for (int q = 0; q < 8; ++q) cum[q + 1] = cum[q] + (q < p.nslots ? min(p.tile_count[p.slot_begin + q], p.mt_ub) : 0);
    const int valid = cum[8] * p.ntn;
    const int per = (valid + 7) >> 3;
    const int xcd = blockIdx.x & 7, wg = blockIdx.x >> 3;
    const int first = xcd * per + wg, lim = min(valid, (xcd + 1) * per);
    const int ntiles = first < lim ? (lim - first + pk.wg_per_xcd - 1) / pk.wg_per_xcd : 0;
    if (ntiles == 0) return;

    int4* sInfo = reinterpret_cast<int4*>(smem + L::INFO_AT);   // {expert, first list position, rows | row tile << 10, slot << 24 | column tile}
    for (int i = tid; i < ntiles; i += NT_ALL) {
        const int logical = first + i * pk.wg_per_xcd;
        const int mtg = logical / p.ntn, nt = logical - mtg * p.ntn;
        int sl = 0;
#pragma unroll
        for (int q = 1; q < 8; ++q) sl += (mtg >= cum[q] && q < p.nslots) ? 1 : 0;
        const int s = p.slot_begin + sl;
        const int4 rec = p.tile_info[(size_t)s * p.mt_ub + (mtg - cum[sl])];
        sInfo[i] = make_int4(rec.x, rec.y, rec.z | ((mtg - cum[sl]) << 10), (s << 24) | nt);
    }
    if constexpr (LUT > 0) {
        // entry 2 * (magnitude bits - LUT_LO) + sign: what the polynomial gives for exactly that bf16 value
        for (unsigned i = tid; i < 2 * LUT_R; i += NT_ALL) {
            const unsigned sign = i & 1u;
            const float xv = from_bits16<TC>((unsigned short)((sign << 15) | (LUT_LO + (i >> 1))));
            if (ACT == HEXA_ACT_GELU) reinterpret_cast<unsigned short*>(smem + L::LUT_AT)[i] = (unsigned short)(pack2<TC>(gelu_poly(xv), 0.f) & 0xffff);
            else reinterpret_cast<float*>(smem + L::LUT_AT)[i] = gelu_grad_poly(xv);
        }
    }
    __syncthreads();

    struct Rec { int e, row_start, rows, mt, s, nt; };
    auto tile_rec = [&](int r) {   // uniform: every lane reads the same record
        u32x4 v = lds_read128_async(lds0 + L::INFO_AT + r * 16);
        lds_wait();
        asm volatile("" : "+v"(v));
        const int z = __builtin_amdgcn_readfirstlane((int)v.z), w = __builtin_amdgcn_readfirstlane((int)v.w);
        Rec o;
        o.e = __builtin_amdgcn_readfirstlane((int)v.x); o.row_start = __builtin_amdgcn_readfirstlane((int)v.y);
        o.rows = z & 1023; o.mt = z >> 10; o.s = w >> 24; o.nt = w & 0xffffff;
        return o;
    };
    const char* zero = reinterpret_cast<const char*>(g_zero_block);
    const int bias_esz = p.bias_dt == HEXA_F32 ? 4 : 2;

    if (wave < NW) {
        // =========================== multiply wavefronts ===========================
        const int wr = wave / C::WF, wf = wave % C::WF;
        __syncthreads();                                 // (P) tile 0's token ids and bias are in LDS
        f32x16 acc[C::FB][C::RB];
        zero_acc(acc);
        int stage = 0;
        for (int r = 0; r < ntiles; ++r) {
            for (int kt = 0; kt < nk; ++kt) {
                barrier_nofence();                       // the copies of this step have landed
                const unsigned base = lds0 + L::STAGES_AT + stage * C::STAGE_BYTES;
                mma_stage_ahead<TC, C, W_IN_OUT>(base, base + C::R_BYTES, wr, wf, lane, acc);
                stage = stage + 1 == STAGES ? 0 : stage + 1;
            }
            barrier_nofence();                           // (A) the store wavefronts are done with the staging area
            // accumulators (+ bias, rounded) -> staging area
            constexpr int RW = 32 * C::RB, FW = 32 * C::FB;
            const int nl0 = wf * FW + 4 * (lane >> 5);            // + j * 32 + 8 * gq
            const unsigned bias_at = lds0 + L::BIAS_AT + (r % 3) * L::BIAS_SLOT + nl0 * bias_esz;
            const unsigned stg = lds0 + L::STAGING_AT + (wr * RW + (lane & 31)) * CP + nl0 * 2;   // + i * 32 * CP
            float bv[C::FB * 4][4];
#pragma unroll
            for (int u = 0; u < C::FB * 4; ++u) { bv[u][0] = 0.f; bv[u][1] = 0.f; bv[u][2] = 0.f; bv[u][3] = 0.f; }
            if (p.bias) {                                // every bias value of this lane in one round of LDS reads
                if (bias_esz == 4) {
                    u32x4 b[C::FB * 4];
                    static_for<C::FB * 4>([&](auto jg) {
                        constexpr int u = decltype(jg)::value;
                        b[u] = lds_read128_async<((u / 4) * 32 + 8 * (u % 4)) * 4>(bias_at);
                    });
                    lds_wait();
#pragma unroll
                    for (int u = 0; u < C::FB * 4; ++u) {
                        asm volatile("" : "+v"(b[u]));
                        bv[u][0] = __uint_as_float(b[u].x); bv[u][1] = __uint_as_float(b[u].y);
                        bv[u][2] = __uint_as_float(b[u].z); bv[u][3] = __uint_as_float(b[u].w);
                    }
                } else {
                    u32x2 b[C::FB * 4];
                    static_for<C::FB * 4>([&](auto jg) {
                        constexpr int u = decltype(jg)::value;
                        b[u] = lds_read64_async<((u / 4) * 32 + 8 * (u % 4)) * 2>(bias_at);
                    });
                    lds_wait();
#pragma unroll
                    for (int u = 0; u < C::FB * 4; ++u) {
                        asm volatile("" : "+v"(b[u]));
                        bv[u][0] = lo16<TC>(b[u].x); bv[u][1] = hi16<TC>(b[u].x);
                        bv[u][2] = lo16<TC>(b[u].y); bv[u][3] = hi16<TC>(b[u].y);
                    }
                }
            }
            static_for<C::FB * 4>([&](auto jg) {
                constexpr int u = decltype(jg)::value, j = u / 4, gq = u % 4;
                static_for<C::RB>([&](auto ic) {
                    constexpr int i = decltype(ic)::value;
                    lds_write64<i * 32 * CP + (j * 32 + 8 * gq) * 2>(
                        stg, pack4<TC>(acc[j][i][4 * gq] + bv[u][0], acc[j][i][4 * gq + 1] + bv[u][1],
                                       acc[j][i][4 * gq + 2] + bv[u][2], acc[j][i][4 * gq + 3] + bv[u][3]));
                });
            });
            lds_wait();
            zero_acc(acc);
        }
        barrier_nofence();                               // (B) the last tile is staged
        if (COLSUM) barrier_nofence();                   // (C) the store wavefronts' last partial sums are in LDS
        return;
    }

    if (wave < NW + CW) {
        // =========================== copy wavefronts ===========================
        const int cw = wave - NW;
        // sources as a base every lane shares plus a 32-bit byte offset per lane: the copy instruction reads one address
        // register per lane instead of two, which matters next to wavefronts that issue MFMAs back to back; lanes with
        // nothing to fetch re-read the first bytes of the tensor (what they produce is never stored)
        const char* const xbase = reinterpret_cast<const char*>(p.x);
        const char* wbase = reinterpret_cast<const char*>(p.w);
        unsigned srcR[R_CPW]; int stepR[R_CPW];
        unsigned srcF[F_CPW]; int stepF[F_CPW];
        auto set_sources = [&](int r) {   // this lane's copy sources for tile r (its token ids are in LDS)
            const Rec rec = tile_rec(r);
            const int e = rec.e, rows = rec.rows, s = rec.s, n0 = rec.nt * BN;
            wbase = reinterpret_cast<const char*>(p.w) + (size_t)e * K * N * 2;
            int rowi[R_CPW], kci[R_CPW], toki[R_CPW];
#pragma unroll
            for (int i = 0; i < R_CPW; ++i) {
                kc_lane<BK>(cw + CW * i, lane, rowi[i], kci[i]);
                toki[i] = lds_read_i32(lds0 + L::TOK_AT + ((r % 3) * BM + rowi[i]) * 4);
            }
            lds_wait();
#pragma unroll
            for (int i = 0; i < R_CPW; ++i) {
                int tok = toki[i];
                asm volatile("" : "+v"(tok));
                const bool ok = rowi[i] < rows;
                srcR[i] = ok ? (unsigned)((((size_t)p.x_slot_rows * s + tok) * K + kci[i] * 8) * 2) : 0u;
                stepR[i] = ok ? BK * 2 : 0;
            }
#pragma unroll
            for (int i = 0; i < F_CPW; ++i) {
                if (W_IN_OUT) {  // w[e][k][n], KS
                    int kk, ch;
                    ks_lane<BN>(cw + CW * i, lane, kk, ch);
                    const int n = n0 + ch * 8;
                    const bool ok = n < N;
                    srcF[i] = ok ? (unsigned)(((size_t)kk * N + n) * 2) : 0u;
                    stepF[i] = ok ? BK * N * 2 : 0;
                } else {         // w[e][n][k], KC
                    int row, kc;
                    kc_lane<BK>(cw + CW * i, lane, row, kc);
                    const int n = n0 + row;
                    const bool ok = n < N;
                    srcF[i] = ok ? (unsigned)(((size_t)n * K + kc * 8) * 2) : 0u;
                    stepF[i] = ok ? BK * 2 : 0;
                }
            }
        };
        auto issue = [&](int stage) {
            char* base = smem + L::STAGES_AT + stage * C::STAGE_BYTES;
#pragma unroll
            for (int i = 0; i < R_CPW; ++i) {
                dma16(xbase + (size_t)srcR[i], base + (cw + CW * i) * 1024);
                srcR[i] += stepR[i];
            }
#pragma unroll
            for (int i = 0; i < F_CPW; ++i) {
                dma16(wbase + (size_t)srcF[i], base + C::R_BYTES + (cw + CW * i) * 1024);
                srcF[i] += stepF[i];
            }
        };
        // token ids and bias of tile r by asynchronous copy.  Every copy wavefront issues the same two copies so
        // that their wait counts agree: 64 token ids (or a filler), then the bias row piece (last wavefront) or a filler.
        auto fetch_meta = [&](int r) {
            const Rec rec = tile_rec(r);
            if (cw < BM / 64) {
                const int row = cw * 64 + lane;
                const void* src = row < rec.rows ? (const void*)(p.token_ids + (size_t)rec.s * p.T + rec.row_start + row) : (const void*)zero;
                __builtin_amdgcn_global_load_lds((glb_ptr_t)src, (lds_ptr_t)(smem + L::TOK_AT + ((r % 3) * BM + cw * 64) * 4), 4, 0, 0);
            } else {
                __builtin_amdgcn_global_load_lds((glb_ptr_t)zero, (lds_ptr_t)(smem + L::SINK_AT), 4, 0, 0);
            }
            if (cw == CW - 1 && p.bias) {
                // BN elements = BN * esz bytes = BN * esz / 16 lanes of 16 bytes
                const int n = rec.nt * BN + lane * (16 / bias_esz);
                const bool ok = lane < BN * bias_esz / 16 && n < N;
                const void* bsrc = ok ? (const void*)(reinterpret_cast<const char*>(p.bias) + ((size_t)rec.e * N + n) * bias_esz) : (const void*)zero;
                __builtin_amdgcn_global_load_lds((glb_ptr_t)bsrc, (lds_ptr_t)(smem + L::BIAS_AT + (r % 3) * L::BIAS_SLOT), 16, 0, 0);
            } else {
                __builtin_amdgcn_global_load_lds((glb_ptr_t)zero, (lds_ptr_t)(smem + L::SINK_AT), 4, 0, 0);
            }
        };

        // tile 0: its token ids and bias with plain loads, then the first stages
        {
            const Rec rec = tile_rec(0);
            const int ct = tid - C::NT;                  // 0 .. 64 * CW - 1
            if (ct < BM) reinterpret_cast<int*>(smem + L::TOK_AT)[ct] = ct < rec.rows ? p.token_ids[(size_t)rec.s * p.T + rec.row_start + ct] : 0;
            if (ct < BN) {
                const int n = rec.nt * BN + ct;
                unsigned raw = 0;
                if (p.bias && n < N) {
                    if (bias_esz == 4) raw = reinterpret_cast<const unsigned*>(p.bias)[(size_t)rec.e * N + n];
                    else raw = reinterpret_cast<const unsigned short*>(p.bias)[(size_t)rec.e * N + n];
                }
                if (bias_esz == 4) reinterpret_cast<unsigned*>(smem + L::BIAS_AT)[ct] = raw;
                else reinterpret_cast<unsigned short*>(smem + L::BIAS_AT)[ct] = (unsigned short)raw;
            }
        }
        __syncthreads();                                 // (P)
        set_sources(0);
        const long total_steps = (long)ntiles * nk;
#pragma unroll
        for (int st = 0; st < STAGES - 1; ++st) issue(st);   // nk >= STAGES is guaranteed by the launcher
        long issued = STAGES - 1, g = 0;                 // steps whose copies have been issued; global step
        for (int r = 0; r < ntiles; ++r) {
            for (int kt = 0; kt < nk; ++kt, ++g) {
                // the copies of step g have landed when at most the groups of the later steps are outstanding
                wait_groups<CPW, STAGES - 2>((int)min(total_steps - 1 - g, (long)(STAGES - 2)));
                // A tile's first step: the stage to refill was read in the previous tile's last step, which barrier
                // (A) has closed, and the ring slots the next tile's token ids and bias go to were last used two tiles
                // ago -- so these copies are issued BEFORE the step's barrier, while the multiply wavefronts are
                // still staging the previous tile's result.
                const bool early = kt == 0;
                if (!early) barrier_nofence();           // publishes stage g; everyone is done reading stage g-1
                if (kt == 0 && r + 1 < ntiles) fetch_meta(r + 1);
                if (issued < total_steps) {
                    if (kt == nk - (STAGES - 1)) set_sources(r + 1);   // the next steps belong to the next tile
                    issue((int)(issued % STAGES));
                    ++issued;
                }
                if (early) barrier_nofence();
            }
            barrier_nofence();                           // (A)
        }
        barrier_nofence();                               // (B)
        if (COLSUM) barrier_nofence();                   // (C)
        return;
    }

    // =========================== store wavefronts ===========================
    const int sw = wave - NW - CW;
    const int et = tid - C::NT - 64 * CW;                // 0 .. NTS-1
    const int c = et % LPR;                              // this lane's 16-byte column piece (the same for every piece)
    const int rl0 = et / LPR;                            // row of piece 0; piece q is PROWS rows further down
    float cs[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    __syncthreads();                                     // (P)

    // one tile's pieces: lane state that does not change over the pieces
    struct TileCtx { int rows, n, s, mt, nt; size_t out_base; unsigned tok_at; bool col_ok, to_ws; };
    auto ctx_of = [&](int q) {
        const Rec rec = tile_rec(q);
        TileCtx t;
        t.rows = rec.rows; t.s = rec.s; t.nt = rec.nt; t.mt = rec.mt;
        t.n = t.nt * BN + c * 8;
        t.col_ok = t.n < N;
        t.to_ws = p.ws != nullptr && t.s > 0;
        t.out_base = t.to_ws ? (size_t)p.T * (t.s - 1) : (size_t)p.out_slot_rows * t.s;
        t.tok_at = lds0 + L::TOK_AT + (q % 3) * BM * 4 + rl0 * 4;
        return t;
    };
    // Piece q of the staged tile.  GELU' variant: all PIECES y1 loads of a tile are issued before its first
    // store, so the operations younger than piece q's load are the PIECES-1-q later loads and the stores of the
    // earlier pieces (a store is skipped when no lane of the wavefront has a valid row, so their number is not
    // fixed): allowing PIECES-1-q outstanding operations waits for that load in every case.
    const unsigned stg_lane = lds0 + L::STAGING_AT + rl0 * CP + c * 16;
    // with the table at the very start of the workgroup's LDS its 16-bit offsets are LDS addresses
    const bool lut_ok = LUT > 0 && lds0 == 0;
    // rows are addressed as (row * 2N + column) in 32 bits; a 24-bit multiply when both factors allow
    const bool mul24 = (size_t)p.T * 8 < ((size_t)1 << 24) && N < (1 << 22);
    const unsigned pitch = (unsigned)N * 2u;
    auto row_offset = [&](const auto& t, int tok) {
        const unsigned row = (unsigned)t.out_base + (unsigned)tok;
        return (mul24 ? __umul24(row, pitch) : row * pitch) + (unsigned)t.n * 2u;
    };
    auto in_table = [&](u16x2 far) {
        return lut_ok && __builtin_amdgcn_ballot_w64(max(far.x, far.y) >= (unsigned short)LUT_R) == 0;
    };
    auto piece = [&](const TileCtx& t, auto qc, u32x4 y1v) {
        constexpr int q = decltype(qc)::value;
        const int rl = rl0 + q * PROWS;
        int tok = lds_read32_async<q * PROWS * 4>(t.tok_at);
        u32x4 val = lds_read128_async<q * PROWS * CP>(stg_lane);
        lds_wait();
        asm volatile("" : "+v"(tok));
        asm volatile("" : "+v"(val));
        if (ACT == HEXA_ACT_GELU_BWD) {
            wait_vmcnt<PIECES - 1 - q>();
            asm volatile("" : "+v"(y1v));
        }
        const bool ok = rl < t.rows && t.col_ok;
        if (!ok) return;
        // results, too, are addressed as a base every lane shares plus a 32-bit byte offset
        const unsigned boff = row_offset(t, tok);
        char* const outb = reinterpret_cast<char*>(t.to_ws ? p.ws : p.out);
        unsigned vw[4] = {val.x, val.y, val.z, val.w};
        if (ACT == HEXA_ACT_NONE && p.accumulate) {   // result += : the rounded product joins what the row piece holds
            const u32x4 old = *reinterpret_cast<const u32x4*>(outb + boff);
            const unsigned ow[4] = {old.x, old.y, old.z, old.w};
#pragma unroll
            for (int u = 0; u < 4; ++u)
                vw[u] = pack2<TC>(lo16<TC>(vw[u]) + lo16<TC>(ow[u]), hi16<TC>(vw[u]) + hi16<TC>(ow[u]));
        }
        if (ACT == HEXA_ACT_GELU_BWD) {
            const unsigned yw[4] = {y1v.x, y1v.y, y1v.z, y1v.w};
            bool looked_up = false;
            if constexpr (LUT > 0) {
                unsigned at[4];
                u16x2 far = {0, 0};
#pragma unroll
                for (int u = 0; u < 4; ++u) at[u] = lut_offsets<LUT_LO, 2>(yw[u], far);
                if (in_table(far)) {   // every value of the wavefront's pieces is in the table
                    unsigned g[8];
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        g[2 * u] = (unsigned)lds_read32_async<L::LUT_AT>(at[u] & 0xffffu);
                        g[2 * u + 1] = (unsigned)lds_read32_async<L::LUT_AT>(at[u] >> 16);
                    }
                    lds_wait();
#pragma unroll
                    for (int j = 0; j < 8; ++j) asm volatile("" : "+v"(g[j]));
#pragma unroll
                    for (int u = 0; u < 4; ++u)
                        vw[u] = pack2<TC>(lo16<TC>(vw[u]) * __uint_as_float(g[2 * u]), hi16<TC>(vw[u]) * __uint_as_float(g[2 * u + 1]));
                    looked_up = true;
                }
            }
            if (!looked_up) {
#pragma unroll
                for (int u = 0; u < 4; ++u)
                    vw[u] = pack2<TC>(lo16<TC>(vw[u]) * gelu_grad_poly(lo16<TC>(yw[u])), hi16<TC>(vw[u]) * gelu_grad_poly(hi16<TC>(yw[u])));
            }
        }
        global_store128(outb, boff, u32x4{vw[0], vw[1], vw[2], vw[3]}, streaming);
        if (COLSUM) {
#pragma unroll
            for (int u = 0; u < 4; ++u) { cs[2 * u] += lo16<TC>(vw[u]); cs[2 * u + 1] += hi16<TC>(vw[u]); }
        }
        if (ACT == HEXA_ACT_GELU) {   // applied to the value as stored (rounded), like act(y1) on the tensor
            unsigned aw[4] = {0u, 0u, 0u, 0u};
            bool looked_up = false;
            if constexpr (LUT > 0) {
                unsigned at[4];
                u16x2 far = {0, 0};
#pragma unroll
                for (int u = 0; u < 4; ++u) at[u] = lut_offsets<LUT_LO, 1>(vw[u], far);
                if (in_table(far)) {
                    unsigned g[8];
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        g[2 * u] = lds_read_u16_async<L::LUT_AT>(at[u] & 0xffffu);
                        g[2 * u + 1] = lds_read_u16_async<L::LUT_AT>(at[u] >> 16);
                    }
                    lds_wait();
#pragma unroll
                    for (int j = 0; j < 8; ++j) asm volatile("" : "+v"(g[j]));
#pragma unroll
                    for (int u = 0; u < 4; ++u) aw[u] = g[2 * u] | (g[2 * u + 1] << 16);
                    looked_up = true;
                }
            }
            if (!looked_up) {
#pragma unroll
                for (int u = 0; u < 4; ++u) aw[u] = pack2<TC>(gelu_poly(lo16<TC>(vw[u])), gelu_poly(hi16<TC>(vw[u])));
            }
            global_store128(p.out_act, boff, u32x4{aw[0], aw[1], aw[2], aw[3]}, streaming);
        }
    };
    auto load_y1 = [&](const TileCtx& t, u32x4 (&y)[PIECES]) {
        int tok[PIECES];
        static_for<PIECES>([&](auto qc) {
            constexpr int q = decltype(qc)::value;
            tok[q] = lds_read32_async<q * PROWS * 4>(t.tok_at);
        });
        lds_wait();
#pragma unroll
        for (int q = 0; q < PIECES; ++q) {
            asm volatile("" : "+v"(tok[q]));
            const bool ok = rl0 + q * PROWS < t.rows && t.col_ok;
            y[q] = global_load128_async(p.out_act, ok ? row_offset(t, tok[q]) : 0u);
        }
    };
    // column sums of the tile just stored: the lanes of a wavefront that hold the same piece, then (after the
    // next barrier) the store wavefronts in order through LDS -- a fixed tree
    auto stash_colsum = [&]() {
#pragma unroll
        for (int u = 0; u < 8; ++u) {
#pragma unroll
            for (int m = 32; m >= LPR; m >>= 1) cs[u] += __shfl_xor(cs[u], m);
        }
        float* red = reinterpret_cast<float*>(smem + L::RED_AT);
        if (lane < LPR) {
#pragma unroll
            for (int u = 0; u < 8; ++u) red[sw * BN + lane * 8 + u] = cs[u];
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) cs[u] = 0.f;
        lds_wait();                                      // the sums are in LDS before this wavefront reaches the barrier
    };
    auto write_colsum = [&](const TileCtx& t) {
        if (et < BN) {
            const float* red = reinterpret_cast<const float*>(smem + L::RED_AT);
            float tsum = 0.f;
#pragma unroll
            for (int w = 0; w < SW; ++w) tsum += red[w * BN + et];
            p.colsum[(((size_t)t.s * p.mt_ub + t.mt) * p.ntn + t.nt) * BN + et] = tsum;
        }
    };

    for (int r = 0; r <= ntiles; ++r) {
        const bool have = r >= 1;                        // tile r-1 is (about to be) in the staging area
        TileCtx t{};
        u32x4 y[PIECES];
#pragma unroll
        for (int q = 0; q < PIECES; ++q) y[q] = u32x4{0u, 0u, 0u, 0u};
        if (have) t = ctx_of(r - 1);
        if (r < ntiles) {
            // the pieces are spread over the main-loop steps of tile r
            int kt = 0;
            barrier_nofence(); ++kt;                     // step 0: the staging area holds tile r-1
            if (have) {
                if (ACT == HEXA_ACT_GELU_BWD) load_y1(t, y);
                static_for<PIECES>([&](auto qc) {
                    constexpr int q = decltype(qc)::value;
                    const int target = (q * nk) / PIECES;             // the step during which piece q is handled
                    while (kt <= target) {
                        barrier_nofence(); ++kt;
                    }
                    piece(t, qc, y[q]);
                });
            }
            while (kt < nk) { barrier_nofence(); ++kt; }
            if (COLSUM && have) stash_colsum();
            barrier_nofence();                           // (A)
            if (COLSUM && have) write_colsum(t);
        } else {
            barrier_nofence();                           // (B)
            if (ACT == HEXA_ACT_GELU_BWD) load_y1(t, y);
            static_for<PIECES>([&](auto qc) { piece(t, qc, y[decltype(qc)::value]); });
            if (COLSUM) {
                stash_colsum();
                barrier_nofence();                       // (C)
                write_colsum(t);
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------------
template <typename TC, bool IO, int ACT, bool COLSUM>
int launch_pipe_t(PipeK& pk, int grid, hipStream_t st) {
    using C = CfgP;
    auto kernel = esmm16_pipe_kernel<TC, IO, ACT, COLSUM, C>;
    constexpr int bytes = PipeLds<C, pipe_lut_bytes<TC, ACT, COLSUM>(), COLSUM>::BYTES;
    if (int rc = ensure_smem(kernel, bytes)) return rc;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(C::NT + 64 * (PIPE_COPY_WAVES + PIPE_STORE_WAVES)), bytes, st, pk);
    HEXA_CHECK_LAUNCH("esmm16_pipe");
    return HEXA_OK;
}

template <typename TC, bool IO>
int launch_pipe_a(PipeK& pk, int grid, int act, bool colsum, hipStream_t st) {
    if (act == HEXA_ACT_GELU) return launch_pipe_t<TC, IO, HEXA_ACT_GELU, false>(pk, grid, st);
    if (act == HEXA_ACT_GELU_BWD)
        return colsum ? launch_pipe_t<TC, IO, HEXA_ACT_GELU_BWD, true>(pk, grid, st)
                      : launch_pipe_t<TC, IO, HEXA_ACT_GELU_BWD, false>(pk, grid, st);
    return launch_pipe_t<TC, IO, HEXA_ACT_NONE, false>(pk, grid, st);
}

int compute_units() {
    static int cus = 0;
    if (!cus) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n < 8)
            n = 256;
        cus = n;
    }
    return cus;
}

}  // namespace

bool esmm16_pipe_supported(const EsmmArgs& a) {
    using C = CfgP;
    if (!(a.w_dt == a.x_dt && a.out_dt == a.x_dt && (a.in_dim % C::BKC) == 0 && a.in_dim >= (2 * C::STAGES - 2) * C::BKC && (a.out_dim % 8) == 0))
        return false;
    if (a.r.k > 8) return false;
    // result += is done by the store wavefronts of the plain launch where every row is written once
    if (a.accumulate && !(a.act == HEXA_ACT_NONE && (a.out_per_slot || a.r.k == 1))) return false;
    // copies address their operands as base + 32-bit byte offset
    if ((size_t)a.r.T * (a.x_per_slot ? a.r.k : 1) * a.in_dim * 2 >= ((size_t)1 << 32) || (size_t)a.in_dim * a.out_dim * 2 >= ((size_t)1 << 32) ||
        (size_t)a.r.T * a.r.k * a.out_dim * 2 >= ((size_t)1 << 32))
        return false;
    if (!(a.out_per_slot || a.r.k == 1 || a.slot_ws != nullptr)) return false;      // every slot in one launch
    if (a.colsum && !(a.act == HEXA_ACT_GELU_BWD)) return false;
    const long total_ub = (long)a.r.k * a.r.mt_ub * div_up(a.out_dim, C::BN);
    const int wg_per_xcd = std::max(1, compute_units() / 8);
    return ((total_ub + 7) / 8 + wg_per_xcd - 1) / wg_per_xcd <= PIPE_MAX_ROUNDS;
}

int launch_esmm16_pipe(const EsmmArgs& a, hipStream_t st) {
    using C = CfgP;
    PipeK pk;
    EsmmK& p = pk.e;
    p.x = a.x; p.w = a.w; p.bias = a.bias; p.out = a.out; p.out_act = a.out_act;
    p.token_ids = a.r.token_ids;
    p.tile_info = a.r.tile_info; p.tile_count = a.r.tile_count; p.mt_ub = a.r.mt_ub;
    p.T = a.r.T; p.K = a.in_dim; p.N = a.out_dim;
    p.ntn = div_up(a.out_dim, C::BN);
    p.x_slot_rows = a.x_per_slot ? a.r.T : 0;
    p.out_slot_rows = a.out_per_slot ? a.r.T : 0;
    p.bias_dt = a.bias_dt; p.out_dt = a.out_dt; p.act = a.act;
    p.stream_out = option(OPT_ESMM_STREAM) != 2; p.colsum = a.colsum; p.group = 0; p.accumulate = a.accumulate;
    p.ws = (!a.out_per_slot && a.r.k > 1) ? a.slot_ws : nullptr;
    p.slot_begin = 0; p.nslots = a.r.k;
    p.total = (long)p.nslots * p.mt_ub * p.ntn;
    if (p.total == 0) return HEXA_OK;
    pk.wg_per_xcd = (int)std::min<long>(std::max(1, compute_units() / 8), (p.total + 7) / 8);
    const int grid = 8 * pk.wg_per_xcd;
    const bool io = a.w_layout == HEXA_W_IN_OUT;
    int rc;
    if (a.x_dt == HEXA_BF16) rc = io ? launch_pipe_a<__bf16, true>(pk, grid, a.act, a.colsum != nullptr, st)
                                     : launch_pipe_a<__bf16, false>(pk, grid, a.act, a.colsum != nullptr, st);
    else rc = io ? launch_pipe_a<_Float16, true>(pk, grid, a.act, a.colsum != nullptr, st)
                 : launch_pipe_a<_Float16, false>(pk, grid, a.act, a.colsum != nullptr, st);
    if (rc) return rc;
    if (p.ws) return launch_sum_slots(a.out, a.slot_ws, (int64_t)a.r.T * a.out_dim, a.r.k - 1, a.out_dt, st, a.sum_extra);
    if (a.colsum) return launch_colsum_fold(a, p.mt_ub, HEXA_TILE_ROWS, p.ntn, C::BN, st);
    return HEXA_OK;
}

}  // namespace hexa
