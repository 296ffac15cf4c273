// Shared device helpers of the asynchronous-copy (global -> LDS) kernels for bf16 / fp16 on gfx950:
// tile shapes, the copy and wait primitives, LDS tile formats and fragment reads, packing and the fast
// GELU.  Everything is internal to one translation unit (anonymous namespace).
#pragma once
#include <stdlib.h>

#include <type_traits>

#include "hexa_internal.h"

namespace hexa {
namespace {

constexpr int BK = 32;

// WR x WF wavefronts, each computing RB x FB blocks of 32x32 (RB blocks along the rows, FB along the
// fast output dimension).  MINW = wavefronts per SIMD the register budget is sized for.
// BKC = contraction indices per stage (32, or 64 for the ESMM kernels: whole 128-byte lines of a row).
template <int WR_, int WF_, int RB_, int FB_, int STAGES_, int MINW_, int BKC_ = 32>
struct Cfg {
    static constexpr int WR = WR_, WF = WF_, RB = RB_, FB = FB_, NW = WR_ * WF_, NT = 64 * NW, MINW = MINW_;
    static constexpr int BM = 32 * RB_ * WR_, BN = 32 * FB_ * WF_, STAGES = STAGES_, BKC = BKC_;
    static constexpr int R_BYTES = BM * BKC * 2, F_BYTES = BN * BKC * 2, STAGE_BYTES = R_BYTES + F_BYTES;
    static constexpr int R_COPIES = R_BYTES / 1024, F_COPIES = F_BYTES / 1024;   // wavefront copies per stage
    static_assert(BKC == 32 || BKC == 64, "32 or 64 contraction indices per stage");
    static constexpr int R_CPW = R_COPIES / NW, F_CPW = F_COPIES / NW, CPW = R_CPW + F_CPW;
    static constexpr int STAGE_AREA = STAGES * STAGE_BYTES;
    static_assert(R_COPIES % NW == 0 && F_COPIES % NW == 0, "copies must divide evenly over the wavefronts");
    static_assert(STAGES >= 2 && STAGES <= 4, "2 to 4 stages");
};
using CfgS = Cfg<2, 2, 2, 2, 4, 2>;   // 128 x 128, 4 wavefronts of 64x64
using CfgL = Cfg<4, 2, 2, 2, 3, 4>;   // 256 x 128, 8 wavefronts of 64x64
using CfgM = Cfg<2, 2, 4, 2, 3, 2>;   // 256 x 128, 4 wavefronts of 128x64
using CfgX = Cfg<2, 2, 4, 4, 3, 1>;   // 256 x 256, 4 wavefronts of 128x128
using CfgX8 = Cfg<2, 4, 4, 2, 3, 2>;  // 256 x 256, 8 wavefronts of 128x64
using CfgX16 = Cfg<4, 4, 2, 2, 3, 4>; // 256 x 256, 16 wavefronts of 64x64
using CfgS2 = Cfg<2, 2, 2, 2, 2, 4>;  // 128 x 128, 2 stages, 4 workgroups per CU (128 registers)
using CfgS3 = Cfg<2, 2, 2, 2, 3, 3>;  // 128 x 128, 3 stages, 3 workgroups per CU (168 registers)
using CfgS64 = Cfg<2, 2, 2, 2, 2, 2, 64>;  // 128 x 128, 64 contraction indices per stage, 2 stages
using CfgL64 = Cfg<4, 2, 2, 2, 2, 4, 64>;  // 256 x 128, 8 wavefronts, 64 per stage, 2 stages
using CfgW = Cfg<2, 4, 2, 3, 3, 2>;   // 128 x 384, 8 wavefronts of 64x96: one tile spans a 384-wide result
using CfgS64W = Cfg<2, 4, 2, 1, 2, 4, 64>;   // 128 x 128, 8 wavefronts of 64x32, 64 per stage, 2 stages, 2 workgroups per CU
using CfgS64H = Cfg<4, 2, 1, 2, 2, 4, 64>;   // 128 x 128, 8 wavefronts of 32x64, 64 per stage, 2 stages, 2 workgroups per CU

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;

__device__ __attribute__((aligned(256))) unsigned int g_zero_block[64];  // stays zero: source of masked lanes

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

typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef const __attribute__((address_space(1))) void* glb_ptr_t;

// One wavefront copy: every lane fetches 16 bytes from `src`; lane i lands at lds_base + 16*i.
__device__ __forceinline__ void dma16(const void* src, char* lds_base) {
    __builtin_amdgcn_global_load_lds((glb_ptr_t)src, (lds_ptr_t)lds_base, 16, 0, 0);
}

// 16-byte store; `streaming` marks the line as not worth keeping in the caches (results that are much
// larger than the L2 would otherwise push the weights and token rows out of it)
__device__ __forceinline__ void store16(uint4* dst, uint4 v, bool streaming) {
    typedef __attribute__((ext_vector_type(4))) unsigned u4;
    u4 w;
    w.x = v.x; w.y = v.y; w.z = v.z; w.w = v.w;
    if (streaming) __builtin_nontemporal_store(w, reinterpret_cast<u4*>(dst));
    else *reinterpret_cast<u4*>(dst) = w;
}

template <int N> __device__ __forceinline__ void wait_vmcnt() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
// `ahead` copy groups of G copies each may still be in flight (ahead <= MAXA)
template <int G, int MAXA> __device__ __forceinline__ void wait_groups(int ahead) {
    if (MAXA >= 2 && ahead >= 2) wait_vmcnt<2 * G>();
    else if (ahead >= 1) wait_vmcnt<G>();
    else wait_vmcnt<0>();
}

// Workgroup barrier WITHOUT the memory fence of __syncthreads(): the fence would wait for every
// outstanding copy (vmcnt(0)) and drain the pipeline.  Ordering is by hand: copies are awaited with
// wait_vmcnt, LDS reads of the previous stage have been consumed by MFMAs before a wavefront arrives.
__device__ __forceinline__ void barrier_nofence() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
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

// ---- fragment reads ---------------------------------------------------------------------------------
// KC tile: 32x16 fragment (rows row0..row0+31, k = 16*ks..16*ks+15): lane holds row l%32, 8 k.
// A row holds KD contraction indices (2*KD bytes, KD/8 pieces of 16 bytes); piece p of row r sits at
// position p ^ kc_swizzle(r): rows that share a 256-byte span of LDS get different bank groups.
template <int KD> __device__ __forceinline__ int kc_swizzle(int row) {
    return KD == 32 ? (row >> 2) & 3 : (row >> 1) & 7;
}
template <typename V, int KD = 32>
__device__ __forceinline__ V frag_kc(const char* tile, int row0, int ks, int lane) {
    const int row = row0 + (lane & 31);
    const int kch = ks * 2 + (lane >> 5);
    const int pos = kch ^ kc_swizzle<KD>(row);
    return *reinterpret_cast<const V*>(tile + row * (2 * KD) + pos * 16);
}

// LDS reads issued as inline assembly: the compiler cannot see that they touch LDS, so it does not
// order them behind the asynchronous copies in flight (it would insert s_waitcnt vmcnt(0) and drain
// the pipeline).  Ordering against the copies is done by hand (wait_vmcnt + barrier); the data
// dependency is closed by lds_fence(), which every consumer of these values must pass through.
__device__ __forceinline__ unsigned lds_addr(const void* p) {
    return (unsigned)(uintptr_t)(__attribute__((address_space(3))) const void*)p;
}
__device__ __forceinline__ s16x4 lds_read_tr16(unsigned addr) {
    s16x4 r;
    asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(r) : "v"(addr));
    return r;
}
__device__ __forceinline__ int lds_read_i32(unsigned addr) {
    int r;
    asm volatile("ds_read_b32 %0, %1" : "=v"(r) : "v"(addr));
    return r;
}

// KS tile of width W: the same fragment from a [k][W] tile through two transposing reads (4 k each).
// Chunk c (8 columns, 16 bytes) of row k sits at position c ^ (4*(k&3)) of the row: the four rows a
// transposing read touches land on different banks.  NOT usable before lds_fence() has been applied.
template <typename V, int W>
__device__ __forceinline__ V frag_ks(const char* tile, int col0, int ks, int lane) {
    const int grp = lane >> 4, s = lane & 15;
    const int col = col0 + (grp & 1) * 16 + (s & 3) * 4;           // 4 consecutive columns = 8 bytes
    const int k = ks * 16 + (grp >> 1) * 8 + (s >> 2);              // + 0 / + 4 for the two reads
    const int ch = col >> 3, sub = (col & 7) * 2;
    const unsigned base = lds_addr(tile);
    union { V v; s16x4 h[2]; } r;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
        const int kk = k + half * 4;
        const int pos = ch ^ ((kk & 3) << 2);
        r.h[half] = lds_read_tr16(base + kk * (2 * W) + pos * 16 + sub);
    }
    return r.v;
}

// ---- copy-source helpers: which global piece does this lane fetch for wavefront copy `c` ------------
// KC operand with KD contraction indices per row: copy c covers 512/KD tile rows.
template <int KD = 32> __device__ __forceinline__ void kc_lane(int c, int lane, int& row, int& kc) {
    constexpr int PPR = KD / 8;              // 16-byte pieces per row
    row = (64 / PPR) * c + lane / PPR;
    kc = (lane % PPR) ^ kc_swizzle<KD>(row);
}
// KS operand of width W: copy c covers 512/W k rows; returns the k row and the column piece.
template <int W> __device__ __forceinline__ void ks_lane(int c, int lane, int& kk, int& ch) {
    constexpr int PPR = W / 8;               // 16-byte pieces per k row (a multiple of 16: the swizzle flips bits 2 and 3)
    const int piece = 64 * c + lane;
    kk = piece / PPR;
    ch = (piece - kk * PPR) ^ ((kk & 3) << 2);
}

template <int A, int B> __device__ __forceinline__ void zero_acc(f32x16 (&acc)[A][B]) {
#pragma unroll
    for (int i = 0; i < A; ++i)
#pragma unroll
        for (int j = 0; j < B; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
}

// acc[j][i]: j = 32-wide block of the fast output dimension (operand "F"), i = 32-row block ("R").
template <typename V, int NA, int NB> __device__ __forceinline__ void lds_fence_all(V (&a)[NA], V (&b)[NB]) {
    // The wait carries no operands; every fragment is then passed through an empty statement placed
    // BEHIND the wait, so a register copy the compiler makes for it reads completed data, and the
    // MFMAs that consume the fragments cannot be scheduled ahead of the wait.
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
    for (int i = 0; i < NA; ++i) asm volatile("" : "+v"(a[i]));
#pragma unroll
    for (int i = 0; i < NB; ++i) asm volatile("" : "+v"(b[i]));
}

template <typename TC, typename C, bool F_KS, bool R_KS>
__device__ __forceinline__ void mma_stage(const char* tileR, const char* tileF, int wr, int wf, int lane,
                                          f32x16 (&acc)[C::FB][C::RB]) {
    using V = typename Mfma<TC>::V;
    constexpr int RW = 32 * C::RB, FW = 32 * C::FB;   // rows / columns per wavefront
#pragma unroll
    for (int ks = 0; ks < C::BKC / 16; ++ks) {
        V f[C::FB], r[C::RB];
#pragma unroll
        for (int j = 0; j < C::FB; ++j)
            f[j] = F_KS ? frag_ks<V, C::BN>(tileF, wf * FW + j * 32, ks, lane) : frag_kc<V, C::BKC>(tileF, wf * FW + j * 32, ks, lane);
#pragma unroll
        for (int i = 0; i < C::RB; ++i)
            r[i] = R_KS ? frag_ks<V, C::BM>(tileR, wr * RW + i * 32, ks, lane) : frag_kc<V, C::BKC>(tileR, wr * RW + i * 32, ks, lane);
        if (F_KS || R_KS) lds_fence_all(f, r);
#pragma unroll
        for (int j = 0; j < C::FB; ++j)
#pragma unroll
            for (int i = 0; i < C::RB; ++i) acc[j][i] = Mfma<TC>::run(f[j], r[i], acc[j][i]);
    }
}

template <typename TC> __device__ __forceinline__ unsigned short bits16(float v) {
    union { TC t; unsigned short u; } c;
    c.t = (TC)v;
    return c.u;
}
template <typename TC> __device__ __forceinline__ float from_bits16(unsigned short u) {
    union { TC t; unsigned short u; } c;
    c.u = u;
    return (float)c.t;
}
// two floats rounded (to nearest even) into one 32-bit word, `a` in the low half: written as a two-element vector
// conversion so that it becomes ONE instruction (v_cvt_pk_bf16_f32 / v_cvt_pk_f16_f32) instead of two conversions,
// a shift and an or -- the epilogues pack every element they produce
template <typename TC> __device__ __forceinline__ unsigned pack2(float a, float b) {
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    typedef TC tcx2_t __attribute__((ext_vector_type(2)));
    f32x2_t v;
    v.x = a; v.y = b;
    union { tcx2_t t; unsigned u; } c;
    c.t = __builtin_convertvector(v, tcx2_t);
    return c.u;
}
template <typename TC> __device__ __forceinline__ uint2 pack4(float a, float b, float c, float d) {
    uint2 o;
    o.x = pack2<TC>(a, b);
    o.y = pack2<TC>(c, d);
    return o;
}

// GELU (erf form) for results that are rounded to 16 bits (or compared at 2e-2), without a transcendental
// instruction.  The epilogue's arithmetic is not free here: a wavefront's VALU instruction occupies its SIMD
// for 4 cycles (16 for a transcendental one), and at a contraction length of a few hundred a tile's GELU costs
// about as many SIMD cycles as its MFMAs.  erf(z) = z * Q(z^2) on |z| <= 3 (clamped beyond: erf(3) = 1 - 2e-5),
// Q of degree 8 fitted to |error| < 3e-5 in fp32 -- bf16 / fp16 round at 4e-3 / 5e-4 relative --: 14 VALU
// operations per element against 12 + two transcendental ones (= 20 issue slots) for the Abramowitz-Stegun
// form with exp and a reciprocal that was used before.  The fp32 kernels keep erff.
__device__ __forceinline__ float erf_poly(float z) {
    const float zc = __builtin_amdgcn_fmed3f(z, -3.0f, 3.0f);
    const float s = zc * zc;
    float q = 4.074186864e-08f;
    q = fmaf(q, s, -1.944813793e-06f);
    q = fmaf(q, s, 4.106038601e-05f);
    q = fmaf(q, s, -5.110357344e-04f);
    q = fmaf(q, s, 4.235422156e-03f);
    q = fmaf(q, s, -2.510284743e-02f);
    q = fmaf(q, s, 1.110793160e-01f);
    q = fmaf(q, s, -3.753148625e-01f);
    q = fmaf(q, s, 1.128268422e+00f);
    return zc * q;
}
__device__ __forceinline__ float gelu_poly(float x) {
    const float hx = 0.5f * x;
    return fmaf(hx, erf_poly(x * 0.70710678118654752440f), hx);
}
__device__ __forceinline__ float gelu_fast(float x) { return gelu_poly(x); }

// gelu'(x) = Phi(x) + x * phi(x) needs exp(-x^2 / 2) anyway, so erf comes from Abramowitz & Stegun 7.1.26
// (|error| < 1.5e-7), which shares that exponential: one exp2, one hardware reciprocal and a degree-5 polynomial
// (measured against the polynomial erf above plus a separate exponential: 127 vs 140 us for the backward launch).
__device__ __forceinline__ float gelu_grad_fast(float x) {
    const float z = fabsf(x) * 0.70710678118654752440f;
    const float t = __builtin_amdgcn_rcpf(1.0f + 0.3275911f * z);
    const float poly = t * (0.254829592f + t * (-0.284496736f + t * (1.421413741f + t * (-1.453152027f + t * 1.061405429f))));
    const float ex = __expf(-z * z);
    const float erf_x = copysignf(1.0f - poly * ex, x);
    return 0.5f * (1.0f + erf_x) + x * 0.39894228040143267794f * ex;
}
__device__ __forceinline__ float gelu_grad_poly(float x) { return gelu_grad_fast(x); }

// ------------------------------------------------------------------------------------------------
// ESMM
// ------------------------------------------------------------------------------------------------
struct EsmmK {
    const void* x; const void* w; const void* bias; void* out; void* out_act;
    const int32_t* token_ids; const int4* tile_info; const int32_t* tile_count;
    int T, K, N, mt_ub, ntn, slot_begin, nslots;
    int x_slot_rows, out_slot_rows;
    int accumulate, bias_dt, out_dt, act, group;
    int stream_out;   // results are stored with the streaming (non-temporal) hint
    long total;
    void* ws;   // slots > 0 write here ([slot-1][T][N]) when set: the slots are summed afterwards
    float* colsum;   // when set: [slot][row tile][column tile][BN] column sums of the stored 16-bit result
};

inline int round_up(long v, int m) { return (int)(((v + m - 1) / m) * m); }

template <typename K> int ensure_smem(K kernel, int bytes) {
    static bool done = false;  // per instantiation
    if (!done) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                bytes) != hipSuccess)
            HEXA_FAIL(HEXA_ERR_LAUNCH, "hipFuncSetAttribute(MaxDynamicSharedMemorySize=%d) failed", bytes);
        done = true;
    }
    return HEXA_OK;
}


}  // namespace
}  // namespace hexa
