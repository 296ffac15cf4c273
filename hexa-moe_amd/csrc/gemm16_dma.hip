// Fast path of ESMM and ESTMM for bf16 / fp16 on gfx950 (CDNA4): tiles stream from HBM straight into
// LDS with the asynchronous global->LDS copy (global_load_lds_dwordx4, 16 bytes per lane, no VGPR
// staging), four stages deep, and are fed to v_mfma_f32_32x32x16 with fp32 accumulation.
//
// LDS tile formats (one operand tile = 128 output rows x 32 contraction indices = 8 KiB per stage):
//   KC  "contraction index fastest in memory"  [128 rows][32 k]  64 B per row; a wavefront copy
//       (64 lanes x 16 B = 1 KiB, contiguous in LDS) covers 16 rows.  Fragments: ds_read_b128.
//       Token rows of ESMM (gathered through the tile's token ids) and w[E][out][in].
//   KS  "contraction index slowest in memory"   [32 k][128 rows] 256 B per k; a wavefront copy covers
//       4 k.  Fragments: two ds_read_b64_tr_b16 (the CDNA4 transposing LDS read) per 32x16 fragment.
//       w[E][in][out] of ESMM, and both operands of ESTMM (token rows of dy and x, tokens contracted).
// The copy engine places lane i at LDS offset 16*i, so bank conflicts are avoided by choosing WHICH
// 16-byte piece each lane fetches (an XOR swizzle applied on the global-address side) instead of
// padding.  Lanes that have nothing to fetch (rows past the end of a segment, columns past N) read
// a 16-byte block of zeros, so ragged tails cost no HBM bytes and need no branches.
//
// The MFMA operands are swapped with respect to the usual convention (A = the operand that supplies
// the output's fastest dimension, B = the rows), so every lane ends up with 4 consecutive output
// columns and stores them with one 8-byte (16-bit results) or 16-byte (fp32 results) store.
//
// Constraints of this path (anything else runs on the general kernels of gemm16.hip): operands and
// weights of one 16-bit type, in_dim a multiple of 32 for ESMM, out/in dims multiples of 8.
#include "hexa_internal.h"

namespace hexa {
namespace {

constexpr int BM = 128, BN = 128, BK = 32, STAGES = 4;
constexpr int NT = 256;
constexpr int TILE_BYTES = 128 * BK * 2;             // one operand tile of one stage
constexpr int STAGE_BYTES = 2 * TILE_BYTES;          // A tile + B tile
constexpr int SMEM_BYTES = STAGES * STAGE_BYTES + BM * 4;

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

template <int N> __device__ __forceinline__ void wait_vmcnt() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// Workgroup barrier WITHOUT the memory fence of __syncthreads(): the fence would wait for every
// outstanding copy (vmcnt(0)) and drain the pipeline.  Ordering is by hand: copies are awaited with
// wait_vmcnt, LDS reads of the previous stage have been consumed by MFMAs before a wavefront arrives.
__device__ __forceinline__ void barrier_nofence() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

__device__ __forceinline__ long logical_tile(int group) {
    const int bid = blockIdx.x;
    const int xcd = bid & 7, loc = bid >> 3;
    const int g = loc / group, r = loc - g * group;
    return ((long)g * 8 + xcd) * group + r;
}

// ---- fragment reads ---------------------------------------------------------------------------------
// KC tile: 32x16 fragment (rows row0..row0+31, k = 16*ks..16*ks+15): lane holds row l%32, 8 k.
template <typename V>
__device__ __forceinline__ V frag_kc(const char* tile, int row0, int ks, int lane) {
    const int row = row0 + (lane & 31);
    const int kch = ks * 2 + (lane >> 5);
    const int pos = kch ^ ((row >> 2) & 3);
    return *reinterpret_cast<const V*>(tile + row * 64 + pos * 16);
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
template <typename V> __device__ __forceinline__ void lds_fence(V& a, V& b, V& c, V& d) {
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d));
}
__device__ __forceinline__ void lds_fence(int& a, int& b) {
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a), "+v"(b));
}

// KS tile: same fragment from a [k][128] tile through two transposing reads (4 k each).
// NOT usable before lds_fence() has been applied to it.
template <typename V>
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
        r.h[half] = lds_read_tr16(base + kk * 256 + pos * 16 + sub);
    }
    return r.v;
}

__device__ __forceinline__ void zero_acc(f32x16 (&acc)[2][2]) {
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
}

// acc[j][i]: j = 32-wide block of the fast output dimension (operand "F"), i = 32-row block ("R").
template <typename TC, bool F_KS, bool R_KS>
__device__ __forceinline__ void mma_stage(const char* tileR, const char* tileF, int wr, int wf, int lane,
                                          f32x16 (&acc)[2][2]) {
    using V = typename Mfma<TC>::V;
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
        V f[2], r[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            f[i] = F_KS ? frag_ks<V>(tileF, wf * 64 + i * 32, ks, lane) : frag_kc<V>(tileF, wf * 64 + i * 32, ks, lane);
            r[i] = R_KS ? frag_ks<V>(tileR, wr * 64 + i * 32, ks, lane) : frag_kc<V>(tileR, wr * 64 + i * 32, ks, lane);
        }
        if (F_KS || R_KS) lds_fence(f[0], f[1], r[0], r[1]);
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int i = 0; i < 2; ++i) acc[j][i] = Mfma<TC>::run(f[j], r[i], acc[j][i]);
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

template <typename TC> __device__ __forceinline__ uint2 pack4(float a, float b, float c, float d) {
    uint2 o;
    o.x = bits16<TC>(a) | ((unsigned)bits16<TC>(b) << 16);
    o.y = bits16<TC>(c) | ((unsigned)bits16<TC>(d) << 16);
    return o;
}

// GELU (erf form) with erf from Abramowitz & Stegun 7.1.26 (|error| < 1.5e-7): one exp, one
// reciprocal and a degree-5 polynomial instead of the library erff.  Used where the result is rounded
// to 16 bits (or compared at 2e-2); the fp32 kernels keep erff.
__device__ __forceinline__ float gelu_fast(float x) {
    const float z = fabsf(x) * 0.70710678118654752440f;
    const float t = __frcp_rn(1.0f + 0.3275911f * z);
    const float poly = t * (0.254829592f + t * (-0.284496736f + t * (1.421413741f + t * (-1.453152027f + t * 1.061405429f))));
    const float erf_abs = 1.0f - poly * __expf(-z * z);
    const float erf_x = copysignf(erf_abs, x);
    return 0.5f * x * (1.0f + erf_x);
}

// ------------------------------------------------------------------------------------------------
// ESMM
// ------------------------------------------------------------------------------------------------
struct EsmmK {
    const void* x; const void* w; const void* bias; void* out; void* out_act;
    const int32_t* token_ids; const int4* tile_info; const int32_t* tile_count;
    int T, K, N, mt_ub, ntn, slot_begin, nslots;
    int x_slot_rows, out_slot_rows;
    int accumulate, bias_dt, out_dt, act, group;
    long total;
    void* ws;   // slots > 0 write here ([slot-1][T][N]) when set: the slots are summed afterwards
};

template <typename TC, bool W_IN_OUT, bool OUT32>
__global__ __launch_bounds__(NT, 2) void esmm16_dma_kernel(EsmmK p) {
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    int* sTok = reinterpret_cast<int*>(smem + STAGES * STAGE_BYTES);

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
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wr = wave >> 1, wf = wave & 1;
    const int K = p.K, N = p.N;

    if (tid < BM) sTok[tid] = tid < rows ? p.token_ids[(size_t)s * p.T + row_start + tid] : -1;
    __syncthreads();

    // ---- source pointers of this lane's copies (two wavefront copies per operand per stage) ----
    const char* zero = reinterpret_cast<const char*>(g_zero_block);
    const char* srcA[2]; int stepA[2];
    const char* srcB[2]; int stepB[2];
#pragma unroll
    for (int c = 0; c < 2; ++c) {
        {   // token rows, KC: chunk (wave + 4c) covers rows 16*chunk .. +15
            const int row = 16 * (wave + 4 * c) + (lane >> 2);
            const int kc = (lane & 3) ^ ((row >> 2) & 3);
            const int tok = sTok[row];
            const bool ok = tok >= 0;
            srcA[c] = ok ? reinterpret_cast<const char*>(p.x) + (((size_t)p.x_slot_rows * s + tok) * K + kc * 8) * 2 : zero;
            stepA[c] = ok ? BK * 2 : 0;
        }
        if (W_IN_OUT) {  // w[e][k][n], KS: chunk covers k rows 4*chunk .. +3, 16 pieces of 8 columns
            const int kk = 4 * (wave + 4 * c) + (lane >> 4);
            const int ch = (lane & 15) ^ ((kk & 3) << 2);
            const int n = n0 + ch * 8;
            const bool ok = n < N;
            srcB[c] = ok ? reinterpret_cast<const char*>(p.w) + (((size_t)e * K + kk) * N + n) * 2 : zero;
            stepB[c] = ok ? BK * N * 2 : 0;
        } else {         // w[e][n][k], KC
            const int row = 16 * (wave + 4 * c) + (lane >> 2);
            const int kc = (lane & 3) ^ ((row >> 2) & 3);
            const int n = n0 + row;
            const bool ok = n < N;
            srcB[c] = ok ? reinterpret_cast<const char*>(p.w) + (((size_t)e * N + n) * K + kc * 8) * 2 : zero;
            stepB[c] = ok ? BK * 2 : 0;
        }
    }
    auto issue = [&](int stage) {   // 4 copies per lane
        char* base = smem + stage * STAGE_BYTES;
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            dma16(srcA[c], base + (wave + 4 * c) * 1024);
            dma16(srcB[c], base + TILE_BYTES + (wave + 4 * c) * 1024);
            srcA[c] += stepA[c];
            srcB[c] += stepB[c];
        }
    };

    f32x16 acc[2][2];
    zero_acc(acc);
    const int nk = K / BK;
    // prologue: STAGES-1 steps in flight (empty groups keep the wait counts uniform)
#pragma unroll
    for (int st = 0; st < STAGES - 1; ++st)
        if (st < nk) issue(st);
    for (int kt = 0; kt < nk; ++kt) {
        // copies of step kt have landed when at most the copies of the later steps are outstanding
        const int ahead = min(nk - 1 - kt, STAGES - 2);
        if (ahead >= 2) wait_vmcnt<8>();
        else if (ahead == 1) wait_vmcnt<4>();
        else wait_vmcnt<0>();
        barrier_nofence();  // everyone's copies of step kt are in LDS; everyone is done reading step kt-1
        if (kt + STAGES - 1 < nk) issue((kt + STAGES - 1) % STAGES);
        const char* base = smem + (kt % STAGES) * STAGE_BYTES;
        mma_stage<TC, W_IN_OUT, false>(base, base + TILE_BYTES, wr, wf, lane, acc);
    }

    // ---- epilogue: lane holds, per 32x32 block, token row l%32 and 4 consecutive columns per group ----
    const bool to_ws = p.ws != nullptr && s > 0;
    void* const outp = to_ws ? p.ws : p.out;
    const bool accumulate = p.accumulate != 0 && !to_ws;
    const bool gelu = p.act == HEXA_ACT_GELU;
    const size_t out_base = to_ws ? (size_t)p.T * (s - 1) : (size_t)p.out_slot_rows * s;
    constexpr int CP = BN * 2 + 16;  // pitch (bytes) of the staged 16-bit result tile
    if (!OUT32) barrier_nofence();   // the stage buffers are reused for the result tile
#pragma unroll
    for (int j = 0; j < 2; ++j) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int nl = wf * 64 + j * 32 + 8 * g + 4 * (lane >> 5);
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
            for (int i = 0; i < 2; ++i) {
                const int rl = wr * 64 + i * 32 + (lane & 31);
                float v[4];
#pragma unroll
                for (int q = 0; q < 4; ++q) v[q] = acc[j][i][4 * g + q] + bv[q];
                if (OUT32) {
                    const int tok = sTok[rl];
                    if (tok < 0 || n >= N) continue;
                    const size_t off = (out_base + tok) * N + n;
                    float4* dst = reinterpret_cast<float4*>(reinterpret_cast<float*>(outp) + off);
                    if (accumulate) { const float4 old = *dst; v[0] += old.x; v[1] += old.y; v[2] += old.z; v[3] += old.w; }
                    *dst = make_float4(v[0], v[1], v[2], v[3]);
                    if (gelu)
                        *reinterpret_cast<float4*>(reinterpret_cast<float*>(p.out_act) + off) =
                            make_float4(gelu_fast(v[0]), gelu_fast(v[1]), gelu_fast(v[2]), gelu_fast(v[3]));
                } else {
                    *reinterpret_cast<uint2*>(smem + rl * CP + nl * 2) = pack4<TC>(v[0], v[1], v[2], v[3]);
                }
            }
        }
    }
    if (!OUT32) {
        // 16-bit results leave through LDS so that 16 lanes write one contiguous 256-byte row piece
        __syncthreads();
        const int c = tid & 15, n = n0 + c * 8;
        if (n < N) {
#pragma unroll
            for (int it = 0; it < BM / 16; ++it) {
                const int rl = it * 16 + (tid >> 4);
                const int tok = sTok[rl];
                if (tok < 0) continue;
                const size_t off = (out_base + tok) * N + n;
                uint4 val = *reinterpret_cast<const uint4*>(smem + rl * CP + c * 16);
                uint4* dst = reinterpret_cast<uint4*>(reinterpret_cast<unsigned short*>(outp) + off);
                if (accumulate) {
                    const uint4 old = *dst;
                    const unsigned ow[4] = {old.x, old.y, old.z, old.w};
                    unsigned vw[4] = {val.x, val.y, val.z, val.w};
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const float lo = from_bits16<TC>(vw[q] & 0xffff) + from_bits16<TC>(ow[q] & 0xffff);
                        const float hi = from_bits16<TC>(vw[q] >> 16) + from_bits16<TC>(ow[q] >> 16);
                        vw[q] = bits16<TC>(lo) | ((unsigned)bits16<TC>(hi) << 16);
                    }
                    val = make_uint4(vw[0], vw[1], vw[2], vw[3]);
                }
                *dst = val;
                if (gelu) {
                    // applied to the value as stored (rounded), like act(y1) on the tensor
                    unsigned vw[4] = {val.x, val.y, val.z, val.w};
#pragma unroll
                    for (int q = 0; q < 4; ++q)
                        vw[q] = bits16<TC>(gelu_fast(from_bits16<TC>(vw[q] & 0xffff))) |
                                ((unsigned)bits16<TC>(gelu_fast(from_bits16<TC>(vw[q] >> 16))) << 16);
                    *reinterpret_cast<uint4*>(reinterpret_cast<unsigned short*>(p.out_act) + off) =
                        make_uint4(vw[0], vw[1], vw[2], vw[3]);
                }
            }
        }
    }
}

int round_up(long v, int m) { return (int)(((v + m - 1) / m) * m); }

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

template <typename TC, bool IO, bool OUT32>
int launch_esmm_dma_t(EsmmK& p, int grid, hipStream_t st) {
    auto kernel = esmm16_dma_kernel<TC, IO, OUT32>;
    if (int rc = ensure_smem(kernel, SMEM_BYTES)) return rc;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(NT), SMEM_BYTES, st, p);
    HEXA_CHECK_LAUNCH("esmm16_dma");
    return HEXA_OK;
}

// ------------------------------------------------------------------------------------------------
// ESTMM: dw[e][m][n] = sum over the expert's (slot, token) list of P[row][m] * Q[row][n]
// ------------------------------------------------------------------------------------------------
constexpr int MAX_SLOTS = 8;      // routing slots handled by this path
constexpr int TOK_RING = 8;       // steps of token ids kept in LDS (32 ids each)
constexpr int ESTMM_STAGE_AREA = 128 * (BN + 4) * 4;   // >= STAGES * STAGE_BYTES: also holds the staged fp32 result
constexpr int ESTMM_SMEM_BYTES = ESTMM_STAGE_AREA + TOK_RING * 32 * 4;
static_assert(ESTMM_STAGE_AREA >= STAGES * STAGE_BYTES, "result staging must cover the stage buffers");

struct EstmmK {
    const void* pm; const void* qm; void* dw;
    const int32_t* token_ids; const int32_t* offsets;
    int T, k, E, M, N, mtn, ntn;
    int p_slot_rows, q_slot_rows;
    int accumulate, group;
    long total;
};

struct Cursor {   // walks the expert's token list in 32-token steps, slot after slot
    int s, r;
};

template <typename TC, bool OUT32>
__global__ __launch_bounds__(NT, 2) void estmm16_dma_kernel(EstmmK p) {
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    int* sIds = reinterpret_cast<int*>(smem + ESTMM_STAGE_AREA);       // [TOK_RING][32]
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
    const int wr = wave >> 1, wf = wave & 1;
    const int M = p.M, N = p.N, T = p.T, nslot = p.k;

    // Heaviest experts first: workgroups are dispatched in id order, so giving the long token lists
    // to the first ones shortens the tail.  The expert of this workgroup is the one whose load has
    // rank `rank` (ties broken by index).  Up to 256 experts; beyond that the order is by index.
    int e = rank;
    if (p.E <= NT) {
        auto load_of = [&](int x) {
            int t = 0;
            for (int s = 0; s < nslot; ++s)
                t += p.offsets[(size_t)s * (p.E + 1) + x + 1] - p.offsets[(size_t)s * (p.E + 1) + x];
            return t;
        };
        if (tid < p.E) {
            const int mine = load_of(tid);
            int r = 0;
            for (int x = 0; x < p.E; ++x) {
                const int o = load_of(x);
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
    int nsteps = 0;
    for (int s = 0; s < nslot; ++s) nsteps += (sEnd[s] - sBeg[s] + BK - 1) / BK;

    auto first = [&]() {
        Cursor c; c.s = 0; c.r = sBeg[0];
        while (c.s < nslot && c.r >= sEnd[c.s]) { ++c.s; c.r = c.s < nslot ? sBeg[c.s] : 0; }
        return c;
    };
    auto advance = [&](Cursor c) {
        c.r += BK;
        while (c.s < nslot && c.r >= sEnd[c.s]) { ++c.s; c.r = c.s < nslot ? sBeg[c.s] : 0; }
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
    // operand tiles of one step (token ids of the step are already in LDS)
    const int ch0 = lane & 15;
    auto issue_data = [&](int step, Cursor c) {
        char* base = smem + (step % STAGES) * STAGE_BYTES;
        const unsigned ids = lds_addr(sIds + (step % TOK_RING) * 32);
        const int end = sEnd[c.s];
        int toks[2];
#pragma unroll
        for (int cc = 0; cc < 2; ++cc) toks[cc] = lds_read_i32(ids + 4 * (4 * (wave + 4 * cc) + (lane >> 4)));
        lds_fence(toks[0], toks[1]);
#pragma unroll
        for (int cc = 0; cc < 2; ++cc) {
            const int kk = 4 * (wave + 4 * cc) + (lane >> 4);
            const int ch = ch0 ^ ((kk & 3) << 2);
            const bool row_ok = c.r + kk < end;
            const int tok = toks[cc];
            const bool okp = row_ok && (m0 + ch * 8 < M), okq = row_ok && (n0 + ch * 8 < N);
            const char* sp = okp ? reinterpret_cast<const char*>(p.pm) + (((size_t)p.p_slot_rows * c.s + tok) * M + m0 + ch * 8) * 2 : zero;
            const char* sq = okq ? reinterpret_cast<const char*>(p.qm) + (((size_t)p.q_slot_rows * c.s + tok) * N + n0 + ch * 8) * 2 : zero;
            dma16(sp, base + (wave + 4 * cc) * 1024);
            dma16(sq, base + TILE_BYTES + (wave + 4 * cc) * 1024);
        }
    };

    f32x16 acc[2][2];
    zero_acc(acc);
    if (nsteps > 0) {
        // Copy groups of 5 per wavefront: { data(step x) [4 copies], ids(step x + LEAD) [1 copy] }.
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
            const int ahead = min(nsteps - 1 - kt, LEAD - 1);   // groups issued after group kt
            if (ahead >= 2) wait_vmcnt<10>();
            else if (ahead == 1) wait_vmcnt<5>();
            else wait_vmcnt<0>();
            barrier_nofence();
            const int jd = kt + LEAD;
            if (jd < nsteps) {
                issue_data(jd, cdat); cdat = advance(cdat);
                issue_ids(jd + LEAD, cid); cid = advance(cid);
            }
            const char* base = smem + (kt % STAGES) * STAGE_BYTES;
            mma_stage<TC, true, true>(base, base + TILE_BYTES, wr, wf, lane, acc);
        }
    } else if (p.accumulate) {
        return;
    }

    // ---- epilogue: lane holds row m = l%32 of a block and 4 consecutive n per group ----
    // The block leaves through LDS (pitch 132 floats) so that 32 lanes write one contiguous 512-byte
    // row of dw; 16-bit results are packed on the way out.
    const bool accumulate = p.accumulate != 0;
    constexpr int CPF = BN + 4;   // floats per staged row
    float* sC = reinterpret_cast<float*>(smem);
    barrier_nofence();            // all wavefronts are done reading the stage buffers
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int ml = wr * 64 + i * 32 + (lane & 31);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int nl = wf * 64 + j * 32 + 8 * g + 4 * (lane >> 5);
                *reinterpret_cast<float4*>(sC + ml * CPF + nl) =
                    make_float4(acc[j][i][4 * g], acc[j][i][4 * g + 1], acc[j][i][4 * g + 2], acc[j][i][4 * g + 3]);
            }
        }
    }
    __syncthreads();
    {
        const int c = tid & 31, n = n0 + c * 4;
        if (n < N) {
#pragma unroll 4
            for (int it = 0; it < BM / 8; ++it) {
                const int ml = it * 8 + (tid >> 5);
                const int m = m0 + ml;
                if (m >= M) break;
                float4 v = *reinterpret_cast<const float4*>(sC + ml * CPF + c * 4);
                const size_t off = ((size_t)e * M + m) * N + n;
                if (OUT32) {
                    float4* dst = reinterpret_cast<float4*>(reinterpret_cast<float*>(p.dw) + off);
                    if (accumulate) { const float4 old = *dst; v.x += old.x; v.y += old.y; v.z += old.z; v.w += old.w; }
                    *dst = v;
                } else {
                    uint2* dst = reinterpret_cast<uint2*>(reinterpret_cast<unsigned short*>(p.dw) + off);
                    if (accumulate) {
                        const uint2 old = *dst;
                        v.x += from_bits16<TC>(old.x & 0xffff); v.y += from_bits16<TC>(old.x >> 16);
                        v.z += from_bits16<TC>(old.y & 0xffff); v.w += from_bits16<TC>(old.y >> 16);
                    }
                    *dst = pack4<TC>(v.x, v.y, v.z, v.w);
                }
            }
        }
    }
}


template <typename TC, bool OUT32>
int launch_estmm_dma_t(EstmmK& p, int grid, hipStream_t st) {
    auto kernel = estmm16_dma_kernel<TC, OUT32>;
    if (int rc = ensure_smem(kernel, ESTMM_SMEM_BYTES)) return rc;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(NT), ESTMM_SMEM_BYTES, st, p);
    HEXA_CHECK_LAUNCH("estmm16_dma");
    return HEXA_OK;
}

}  // namespace

bool esmm16_dma_supported(const EsmmArgs& a) {
    return a.w_dt == a.x_dt && (a.in_dim % BK) == 0 && (a.out_dim % 8) == 0 &&
           (a.out_dt == a.x_dt || a.out_dt == HEXA_F32);
}

bool estmm16_dma_supported(const EstmmArgs& a) {
    return a.r.k <= MAX_SLOTS && (a.m_dim % 8) == 0 && (a.n_dim % 8) == 0 && (a.dw_dt == a.pq_dt || a.dw_dt == HEXA_F32);
}

int launch_estmm16_dma(const EstmmArgs& a, hipStream_t st) {
    EstmmK p;
    p.pm = a.p; p.qm = a.q; p.dw = a.dw;
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
    const bool o32 = a.dw_dt == HEXA_F32;
    if (a.pq_dt == HEXA_BF16) return o32 ? launch_estmm_dma_t<__bf16, true>(p, grid, st) : launch_estmm_dma_t<__bf16, false>(p, grid, st);
    return o32 ? launch_estmm_dma_t<_Float16, true>(p, grid, st) : launch_estmm_dma_t<_Float16, false>(p, grid, st);
}

int launch_esmm16_dma(const EsmmArgs& a, hipStream_t st) {
    EsmmK p;
    p.x = a.x; p.w = a.w; p.bias = a.bias; p.out = a.out; p.out_act = a.out_act;
    p.token_ids = a.r.token_ids; p.tile_info = a.r.tile_info; p.tile_count = a.r.tile_count;
    p.T = a.r.T; p.K = a.in_dim; p.N = a.out_dim; p.mt_ub = a.r.mt_ub;
    p.ntn = div_up(a.out_dim, BN);
    p.x_slot_rows = a.x_per_slot ? a.r.T : 0;
    p.out_slot_rows = a.out_per_slot ? a.r.T : 0;
    p.bias_dt = a.bias_dt; p.out_dt = a.out_dt; p.act = a.act;
    p.group = p.ntn * 4;
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
        const int grid = round_up(p.total, 8 * p.group);
        const bool io = a.w_layout == HEXA_W_IN_OUT;
        const bool o32 = a.out_dt == HEXA_F32;
        int rc;
        if (a.x_dt == HEXA_BF16) {
            if (o32) rc = io ? launch_esmm_dma_t<__bf16, true, true>(p, grid, st) : launch_esmm_dma_t<__bf16, false, true>(p, grid, st);
            else rc = io ? launch_esmm_dma_t<__bf16, true, false>(p, grid, st) : launch_esmm_dma_t<__bf16, false, false>(p, grid, st);
        } else {
            if (o32) rc = io ? launch_esmm_dma_t<_Float16, true, true>(p, grid, st) : launch_esmm_dma_t<_Float16, false, true>(p, grid, st);
            else rc = io ? launch_esmm_dma_t<_Float16, true, false>(p, grid, st) : launch_esmm_dma_t<_Float16, false, false>(p, grid, st);
        }
        if (rc) return rc;
    }
    if (p.ws) return launch_sum_slots(a.out, a.slot_ws, (int64_t)a.r.T * a.out_dim, a.r.k - 1, a.out_dt, st);
    return HEXA_OK;
}

}  // namespace hexa
