// Persistent ESMM for bf16 / fp16 on gfx950: a fixed grid of workgroups (as many as fit on the chip at
// once) walks the list of valid tiles.  What a one-tile-per-workgroup launch pays per tile in exposed
// latency is overlapped here:
//   * the next tile's record, token ids and bias are fetched while the current tile is multiplied;
//   * the next tile's first stages are on their way (asynchronous copies) while the current tile's
//     result is staged and stored;
//   * inside a stage, the fragments of the next 16 contraction indices are read from LDS while the
//     MFMAs of the current ones run.
//
// Asynchronous state never crosses a boundary the compiler can see.  LDS reads are issued inside
// inline-assembly blocks that end with s_waitcnt lgkmcnt(0), so every register a block returns is
// complete; the MFMAs that hide the read latency sit inside the same block.  (A register that is
// still being filled when a block ends could be copied or spilled by the compiler before the data
// arrives -- there is no hardware interlock for that.)  LDS accesses are assembly throughout because
// a compiler-visible transposing LDS read is ordered behind the copies in flight with
// s_waitcnt vmcnt(0), which would serialise the pipeline.  Copies are ordered by vmcnt counts and
// barriers, by hand.
//
// Replaces esmm_shared_tensor_kernel_vectorized_accum_half (kernels/esmm_half.cu) and the ESMM task
// of the fused backward kernels (kernels/fused_ops_half.cu) for the layouts this path supports.
#include "dma_common.h"

namespace hexa {
namespace {

constexpr int PERSIST_MAX_SLOTS = 8;

// shapes (the LDS also holds a result staging area next to the stages)
using CfgPS = Cfg<2, 2, 2, 2, 3, 2>;  // 128 x 128, 4 wavefronts of 64x64, 3 stages, 2 workgroups per CU
using CfgPM = Cfg<2, 2, 4, 2, 2, 2>;  // 256 x 128, 4 wavefronts of 128x64, 2 stages, 2 workgroups per CU
using CfgPL = Cfg<4, 2, 2, 2, 3, 2>;  // 256 x 128, 8 wavefronts of 64x64, 3 stages, 1 workgroup per CU

typedef __attribute__((ext_vector_type(4))) unsigned u32x4;
typedef __attribute__((ext_vector_type(2))) unsigned u32x2;

template <typename TC> constexpr bool is_bf16 = std::is_same<TC, __bf16>::value;

// ---- synchronous LDS helpers: issue, then wait; what they return is complete ----------------------
__device__ __forceinline__ void lds_write_b32(unsigned addr, int v) {
    asm volatile("ds_write_b32 %0, %1" ::"v"(addr), "v"(v) : "memory");
}
__device__ __forceinline__ void lds_write_b64(unsigned addr, uint2 v) {
    u32x2 w;
    w.x = v.x; w.y = v.y;
    asm volatile("ds_write_b64 %0, %1" ::"v"(addr), "v"(w) : "memory");
}
// this wavefront's LDS traffic is complete, then the workgroup meets
__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}
__device__ __forceinline__ void lds_read2_i32_sync(unsigned a0, unsigned a1, int& r0, int& r1) {
    asm volatile("ds_read_b32 %0, %2\n\tds_read_b32 %1, %3\n\ts_waitcnt lgkmcnt(0)"
                 : "=&v"(r0), "=&v"(r1) : "v"(a0), "v"(a1) : "memory");
}
__device__ __forceinline__ u32x4 lds_read_b128_sync(unsigned a) {
    u32x4 r;
    asm volatile("ds_read_b128 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=&v"(r) : "v"(a) : "memory");
    return r;
}
// four (token id, 16-byte value) pairs at constant offsets from two addresses
template <int T0, int T1, int T2, int T3, int V0, int V1, int V2, int V3>
__device__ __forceinline__ void lds_read4_pairs_sync(unsigned at, unsigned av, int (&tok)[4], u32x4 (&val)[4]) {
    asm volatile(
        "ds_read_b32 %0, %8 offset:%10\n\tds_read_b128 %4, %9 offset:%14\n\t"
        "ds_read_b32 %1, %8 offset:%11\n\tds_read_b128 %5, %9 offset:%15\n\t"
        "ds_read_b32 %2, %8 offset:%12\n\tds_read_b128 %6, %9 offset:%16\n\t"
        "ds_read_b32 %3, %8 offset:%13\n\tds_read_b128 %7, %9 offset:%17\n\t"
        "s_waitcnt lgkmcnt(0)"
        : "=&v"(tok[0]), "=&v"(tok[1]), "=&v"(tok[2]), "=&v"(tok[3]), "=&v"(val[0]), "=&v"(val[1]), "=&v"(val[2]), "=&v"(val[3])
        : "v"(at), "v"(av), "n"(T0), "n"(T1), "n"(T2), "n"(T3), "n"(V0), "n"(V1), "n"(V2), "n"(V3)
        : "memory");
}
// four 16-byte values at offsets 0, 32, 64, 96 (+BASE) from one address
template <int BASE, int STEP>
__device__ __forceinline__ void lds_read4_b128_sync(unsigned a, u32x4 (&v)[4]) {
    asm volatile(
        "ds_read_b128 %0, %4 offset:%5\n\tds_read_b128 %1, %4 offset:%6\n\t"
        "ds_read_b128 %2, %4 offset:%7\n\tds_read_b128 %3, %4 offset:%8\n\ts_waitcnt lgkmcnt(0)"
        : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]), "=&v"(v[3])
        : "v"(a), "n"(BASE), "n"(BASE + STEP), "n"(BASE + 2 * STEP), "n"(BASE + 3 * STEP)
        : "memory");
}

// ---- fragment addresses -----------------------------------------------------------------------------
// KC tile: per-lane byte address of block 0 for slice 0 and slice 1 (a[0], a[1]); block b adds 2048 b.
// KS tile of width W: per-lane byte address of block b, slice 0, first half (a[b]); slice ks / half h
// add (16 ks + 4 h) * 2W.
template <int NB> struct FragAddr { unsigned a[NB < 2 ? 2 : NB]; };

template <int NB> __device__ __forceinline__ FragAddr<NB> kc_frag_addr(unsigned tile, int row0, int lane) {
    FragAddr<NB> f;
    const int row = row0 + (lane & 31), h = lane >> 5, swz = (row >> 2) & 3;
    f.a[0] = tile + row * 64 + ((h ^ swz) << 4);
    f.a[1] = tile + row * 64 + (((2 + h) ^ swz) << 4);
    return f;
}
template <int NB, int W> __device__ __forceinline__ FragAddr<NB> ks_frag_addr(unsigned tile, int col0, int lane) {
    FragAddr<NB> f;
    const int grp = lane >> 4, s = lane & 15;
    const int k = (grp >> 1) * 8 + (s >> 2);
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        const int col = col0 + b * 32 + (grp & 1) * 16 + (s & 3) * 4;
        const int pos = (col >> 3) ^ ((k & 3) << 2);
        f.a[b] = tile + k * (2 * W) + pos * 16 + (col & 7) * 2;
    }
    return f;
}

// ---- the multiply blocks ------------------------------------------------------------------------------
// One block = the LDS reads of fragments that are needed NEXT, four MFMAs on fragments that are
// complete, s_waitcnt lgkmcnt(0): the reads are hidden behind the MFMAs and nothing is in flight
// when the block ends.  c{j}{i} += f{j} x r{i} (f: fast output dimension, r: rows).  The trailing
// s_nop covers the MFMA-result-to-VALU wait states a compiler-inserted copy of an accumulator after
// the block would need (the compiler cannot see that the block holds MFMAs); it overlaps with the last
// MFMA's execution.
#define HEXA_MFMA_2x2(T)                                          \
    "v_mfma_f32_32x32x16_" T " %[c00], %[f0], %[r0], %[c00]\n\t" \
    "v_mfma_f32_32x32x16_" T " %[c01], %[f0], %[r1], %[c01]\n\t" \
    "v_mfma_f32_32x32x16_" T " %[c10], %[f1], %[r0], %[c10]\n\t" \
    "v_mfma_f32_32x32x16_" T " %[c11], %[f1], %[r1], %[c11]\n\t" \
    "s_waitcnt lgkmcnt(0)\n\t"                                    \
    "s_nop 15"
#define HEXA_ACC_OPS [c00] "+v"(c00), [c01] "+v"(c01), [c10] "+v"(c10), [c11] "+v"(c11)
#define HEXA_FRAG_OPS [f0] "v"(f0), [f1] "v"(f1), [r0] "v"(r0), [r1] "v"(r1)

// reads: 2 KC fragments of F and 2 KC fragments of R
template <typename TC, int OF0, int OF1, int OR0, int OR1, typename V>
__device__ __forceinline__ void block_kc_kc(V& nf0, V& nf1, V& nr0, V& nr1, f32x16& c00, f32x16& c01, f32x16& c10,
                                            f32x16& c11, const V& f0, const V& f1, const V& r0, const V& r1,
                                            unsigned aF, unsigned aR) {
#define HEXA_B(T)                                                                                               \
    asm volatile("ds_read_b128 %[nf0], %[aF] offset:%[of0]\n\t"                                               \
                 "ds_read_b128 %[nf1], %[aF] offset:%[of1]\n\t"                                               \
                 "ds_read_b128 %[nr0], %[aR] offset:%[or0]\n\t"                                               \
                 "ds_read_b128 %[nr1], %[aR] offset:%[or1]\n\t" HEXA_MFMA_2x2(T)                              \
                 : [nf0] "=&v"(nf0), [nf1] "=&v"(nf1), [nr0] "=&v"(nr0), [nr1] "=&v"(nr1), HEXA_ACC_OPS       \
                 : HEXA_FRAG_OPS, [aF] "v"(aF), [aR] "v"(aR), [of0] "n"(OF0), [of1] "n"(OF1), [or0] "n"(OR0), \
                   [or1] "n"(OR1))
    if constexpr (is_bf16<TC>) HEXA_B("bf16"); else HEXA_B("f16");
#undef HEXA_B
}
// reads: 2 KS fragments of F (two transposing reads each) and 2 KC fragments of R
template <typename TC, int OFA, int OFB, int OR0, int OR1, typename V>
__device__ __forceinline__ void block_ks_kc(s16x4 (&nfh)[4], V& nr0, V& nr1, f32x16& c00, f32x16& c01, f32x16& c10,
                                            f32x16& c11, const V& f0, const V& f1, const V& r0, const V& r1,
                                            unsigned aF0, unsigned aF1, unsigned aR) {
#define HEXA_B(T)                                                                                                \
    asm volatile("ds_read_b64_tr_b16 %[h0], %[aF0] offset:%[ofa]\n\t"                                          \
                 "ds_read_b64_tr_b16 %[h1], %[aF0] offset:%[ofb]\n\t"                                          \
                 "ds_read_b64_tr_b16 %[h2], %[aF1] offset:%[ofa]\n\t"                                          \
                 "ds_read_b64_tr_b16 %[h3], %[aF1] offset:%[ofb]\n\t"                                          \
                 "ds_read_b128 %[nr0], %[aR] offset:%[or0]\n\t"                                                \
                 "ds_read_b128 %[nr1], %[aR] offset:%[or1]\n\t" HEXA_MFMA_2x2(T)                               \
                 : [h0] "=&v"(nfh[0]), [h1] "=&v"(nfh[1]), [h2] "=&v"(nfh[2]), [h3] "=&v"(nfh[3]),             \
                   [nr0] "=&v"(nr0), [nr1] "=&v"(nr1), HEXA_ACC_OPS                                            \
                 : HEXA_FRAG_OPS, [aF0] "v"(aF0), [aF1] "v"(aF1), [aR] "v"(aR), [ofa] "n"(OFA), [ofb] "n"(OFB), \
                   [or0] "n"(OR0), [or1] "n"(OR1))
    if constexpr (is_bf16<TC>) HEXA_B("bf16"); else HEXA_B("f16");
#undef HEXA_B
}
// reads: 2 KC fragments of R only
template <typename TC, int OR0, int OR1, typename V>
__device__ __forceinline__ void block_r_kc(V& nr0, V& nr1, f32x16& c00, f32x16& c01, f32x16& c10, f32x16& c11,
                                           const V& f0, const V& f1, const V& r0, const V& r1, unsigned aR) {
#define HEXA_B(T)                                                                        \
    asm volatile("ds_read_b128 %[nr0], %[aR] offset:%[or0]\n\t"                        \
                 "ds_read_b128 %[nr1], %[aR] offset:%[or1]\n\t" HEXA_MFMA_2x2(T)       \
                 : [nr0] "=&v"(nr0), [nr1] "=&v"(nr1), HEXA_ACC_OPS                    \
                 : HEXA_FRAG_OPS, [aR] "v"(aR), [or0] "n"(OR0), [or1] "n"(OR1))
    if constexpr (is_bf16<TC>) HEXA_B("bf16"); else HEXA_B("f16");
#undef HEXA_B
}
#undef HEXA_MFMA_2x2
#undef HEXA_ACC_OPS
#undef HEXA_FRAG_OPS

// reads without MFMAs (first slice of a tile)
template <int O0, int O1, typename V> __device__ __forceinline__ void read2_kc_sync(V& n0, V& n1, unsigned a) {
    asm volatile("ds_read_b128 %0, %2 offset:%3\n\tds_read_b128 %1, %2 offset:%4\n\ts_waitcnt lgkmcnt(0)"
                 : "=&v"(n0), "=&v"(n1) : "v"(a), "n"(O0), "n"(O1) : "memory");
}
template <int OA, int OB> __device__ __forceinline__ void read2_ks_sync(s16x4 (&h)[4], unsigned a0, unsigned a1) {
    asm volatile("ds_read_b64_tr_b16 %0, %4 offset:%6\n\tds_read_b64_tr_b16 %1, %4 offset:%7\n\t"
                 "ds_read_b64_tr_b16 %2, %5 offset:%6\n\tds_read_b64_tr_b16 %3, %5 offset:%7\n\ts_waitcnt lgkmcnt(0)"
                 : "=&v"(h[0]), "=&v"(h[1]), "=&v"(h[2]), "=&v"(h[3]) : "v"(a0), "v"(a1), "n"(OA), "n"(OB) : "memory");
}
template <typename V> __device__ __forceinline__ V join_halves(s16x4 lo, s16x4 hi) {
    union { V v; s16x4 h[2]; } u;
    u.h[0] = lo; u.h[1] = hi;
    return u.v;
}

template <typename C> struct PersistLds {
    static constexpr int CP = C::BN * 2 + 16;            // pitch (bytes) of a staged 16-bit result row
    static constexpr int PASS_ROWS = 32 * C::WR;         // one 32-row block of every wavefront per pass
    static constexpr int ID_COPIES = C::BM / 64, BIAS_COPIES = C::BN / 64;   // 256-byte wavefront copies
    static constexpr int PCW = (ID_COPIES + BIAS_COPIES + 1 + C::NW - 1) / C::NW; // metadata copies per wavefront
    static constexpr int STAGING = C::STAGE_AREA;        // byte offsets
    static constexpr int TOK = STAGING + PASS_ROWS * CP; // [2][BM] token ids
    static constexpr int BIAS = TOK + 2 * C::BM * 4;     // [2][BN] bias, raw (fp32 or packed 16-bit)
    static constexpr int INFO = BIAS + 2 * C::BN * 4;    // [2] tile records (16 bytes each, 256 apart)
    static constexpr int DUMMY = INFO + 512;             // target of the copies that carry nothing
    static constexpr int TOTAL = DUMMY + 256;
};

// at most groups*G (+ P) asynchronous copies of this wavefront may still be in flight
template <int G, int P> __device__ __forceinline__ void wait_outstanding(int groups, bool plus_p) {
    switch (groups * 2 + (plus_p ? 1 : 0)) {
        case 0: wait_vmcnt<0>(); break;
        case 1: wait_vmcnt<P>(); break;
        case 2: wait_vmcnt<G>(); break;
        case 3: wait_vmcnt<G + P>(); break;
        case 4: wait_vmcnt<2 * G>(); break;
        default: wait_vmcnt<2 * G + P>(); break;
    }
}

template <typename TC, bool W_IN_OUT, bool OUT32, typename C>
__global__ __launch_bounds__(C::NT, C::MINW) void esmm16_persist_kernel(EsmmK p) {
    using V = typename Mfma<TC>::V;
    using L = PersistLds<C>;
    constexpr int BM = C::BM, BN = C::BN, STAGES = C::STAGES, NW = C::NW, RB = C::RB;
    constexpr int RW = 32 * RB, FW = 64;
    static_assert(C::FB == 2 && (RB == 2 || RB == 4), "wavefront tiles of 64 columns x 64 or 128 rows");
    static_assert(2 * C::CPW + L::PCW <= 63, "vmcnt is a 6-bit counter");
    static_assert(BM <= C::NT && BN <= C::NT, "one thread per tile row / column in the metadata steps");
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    const unsigned lds0 = lds_addr(smem);

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wr = wave / C::WF, wf = wave % C::WF;
    const int K = p.K, N = p.N, ntn = p.ntn;
    const int nk = K / BK;
    const bool bias32 = p.bias_dt == HEXA_F32;

    // valid row tiles of the slots handled by this launch, as a running sum
    int cum[PERSIST_MAX_SLOTS + 1];
    cum[0] = 0;
#pragma unroll
    for (int s = 0; s < PERSIST_MAX_SLOTS; ++s)
        cum[s + 1] = cum[s] + (s < p.nslots ? min(p.tile_count[p.slot_begin + s], p.mt_ub) : 0);
    const int total = cum[PERSIST_MAX_SLOTS] * ntn;

    // Workgroup ids go round-robin over the XCDs; per sweep, every XCD takes a run of gridDim/8
    // consecutive tiles (column tiles fastest), which share token rows and weights in its L2.
    const int per_xcd = gridDim.x >> 3;
    const int stride = 8 * per_xcd;
    int tile = (int)(blockIdx.x & 7) * per_xcd + (int)(blockIdx.x >> 3);
    if (tile >= total) return;

    // tile index -> slot, first column and the address of the tile's record {expert, first row, rows, -}
    struct Tile { int s, e, row_start, rows, n0; };
    auto place = [&](int t, Tile& r) {
        const int mtg = t / ntn;
        r.n0 = (t - mtg * ntn) * BN;
        int s = 0;
#pragma unroll
        for (int q = 1; q < PERSIST_MAX_SLOTS; ++q) s += (mtg >= cum[q] && q < p.nslots) ? 1 : 0;
        r.s = p.slot_begin + s;
        return p.tile_info + ((size_t)(p.slot_begin + s) * p.mt_ub + (mtg - cum[s]));
    };
    auto locate = [&](int t) {   // with a load: only before the tile loop
        Tile r;
        const int4 info = *place(t, r);
        r.e = info.x; r.row_start = info.y; r.rows = info.z;
        return r;
    };

    const char* zero = reinterpret_cast<const char*>(g_zero_block);
    // A tile's token ids and bias -- and the record of the tile after it -- travel to LDS as
    // 4-byte-per-lane asynchronous copies, PCW per wavefront (the ones that carry nothing read the
    // zero block into a dummy area), so that they count in vmcnt exactly like the operand copies.
    // (A plain load of the record inside the tile loop would be a vector load -- the stores of the
    // loop rule out the scalar path -- whose wait would drain the copies in flight.)
    auto issue_meta = [&](const Tile& t, int buf, const int4* record, int record_buf) {
#pragma unroll
        for (int i = 0; i < L::PCW; ++i) {
            const int q = wave + NW * i;
            const char* src = zero;
            unsigned dst = L::DUMMY;
            if (q < L::ID_COPIES) {
                const int r = q * 64 + lane;
                if (r < t.rows) src = reinterpret_cast<const char*>(p.token_ids + (size_t)t.s * p.T + t.row_start + r);
                dst = L::TOK + (buf * BM + q * 64) * 4;
            } else if (q < L::ID_COPIES + L::BIAS_COPIES) {
                // fp32 bias: copy b holds columns 64b..64b+63; 16-bit bias: columns 128b..128b+127
                const int b = q - L::ID_COPIES;
                if (p.bias && b * (bias32 ? 64 : 128) < BN) {
                    const int c = bias32 ? b * 64 + lane : 2 * (b * 64 + lane);   // first column of this lane's 4 bytes
                    if (t.n0 + c < N)
                        src = reinterpret_cast<const char*>(p.bias) + ((size_t)t.e * N + t.n0 + c) * (bias32 ? 4 : 2);
                    dst = L::BIAS + buf * BN * 4 + b * 256;
                }
            } else if (q == L::ID_COPIES + L::BIAS_COPIES && record) {
                if (lane < 4) src = reinterpret_cast<const char*>(record) + lane * 4;
                dst = L::INFO + record_buf * 256;
            }
            __builtin_amdgcn_global_load_lds((glb_ptr_t)src, (lds_ptr_t)(smem + dst), 4, 0, 0);
        }
    };

    // ---- operand copies: per-lane sources of a tile ----
    const char* srcR[C::R_CPW]; int stepR[C::R_CPW];
    const char* srcF[C::F_CPW]; int stepF[C::F_CPW];
    static_assert(C::R_CPW % 2 == 0, "token ids are fetched from LDS in pairs");
    auto set_sources = [&](const Tile& t, int buf) {
        int ln = lane;
        asm volatile("" : "+v"(ln));   // per-tile address arithmetic stays inside the tile loop
#pragma unroll
        for (int i = 0; i < C::R_CPW; i += 2) {
            int row[2], kc[2], tk[2];
            kc_lane(wave + NW * i, ln, row[0], kc[0]);
            kc_lane(wave + NW * (i + 1), ln, row[1], kc[1]);
            lds_read2_i32_sync(lds0 + L::TOK + (buf * BM + row[0]) * 4, lds0 + L::TOK + (buf * BM + row[1]) * 4, tk[0], tk[1]);
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const bool ok = row[u] < t.rows;
                srcR[i + u] = ok ? reinterpret_cast<const char*>(p.x) + (((size_t)p.x_slot_rows * t.s + tk[u]) * K + kc[u] * 8) * 2 : zero;
                stepR[i + u] = ok ? BK * 2 : 0;
            }
        }
#pragma unroll
        for (int i = 0; i < C::F_CPW; ++i) {
            if (W_IN_OUT) {  // w[e][k][n], KS
                int kk, ch;
                ks_lane<BN>(wave + NW * i, ln, kk, ch);
                const int n = t.n0 + ch * 8;
                const bool ok = n < N;
                srcF[i] = ok ? reinterpret_cast<const char*>(p.w) + (((size_t)t.e * K + kk) * N + n) * 2 : zero;
                stepF[i] = ok ? BK * N * 2 : 0;
            } else {         // w[e][n][k], KC
                int row, kc;
                kc_lane(wave + NW * i, ln, row, kc);
                const int n = t.n0 + row;
                const bool ok = n < N;
                srcF[i] = ok ? reinterpret_cast<const char*>(p.w) + (((size_t)t.e * N + n) * K + kc * 8) * 2 : zero;
                stepF[i] = ok ? BK * 2 : 0;
            }
        }
    };
    auto issue = [&](int stage) {
        char* base = smem + stage * C::STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < C::R_CPW; ++i) {
            dma16(srcR[i], base + (wave + NW * i) * 1024);
            srcR[i] += stepR[i];
        }
#pragma unroll
        for (int i = 0; i < C::F_CPW; ++i) {
            dma16(srcF[i], base + C::R_BYTES + (wave + NW * i) * 1024);
            srcF[i] += stepF[i];
        }
    };
    auto issue_first_stages = [&]() {
#pragma unroll
        for (int st = 0; st < STAGES - 1; ++st)
            if (st < nk) issue(st);
    };

    // ---- fragments ----
    const FragAddr<RB> faR = kc_frag_addr<RB>(lds0, wr * RW, lane);
    FragAddr<2> faF;
    if (W_IN_OUT) faF = ks_frag_addr<2, BN>(lds0, wf * FW, lane);
    else faF = kc_frag_addr<2>(lds0, wf * FW, lane);
    constexpr int FBASE = C::R_BYTES;              // the F tile follows the R tile in a stage
    constexpr int KSROW = 2 * BN;                  // bytes per contraction index of a KS tile of F

    f32x16 acc[2][RB];   // [column block][row block]
    V f[2], r[RB];       // current slice

    // first slice of stage 0 (nothing to hide it behind)
    auto read_first = [&]() {
        if (W_IN_OUT) {
            s16x4 h[4];
            read2_ks_sync<FBASE, FBASE + 4 * KSROW>(h, faF.a[0], faF.a[1]);
            f[0] = join_halves<V>(h[0], h[1]); f[1] = join_halves<V>(h[2], h[3]);
        } else {
            read2_kc_sync<FBASE, FBASE + 2048>(f[0], f[1], faF.a[0]);
        }
        read2_kc_sync<0, 2048>(r[0], r[1], faR.a[0]);
        if constexpr (RB == 4) read2_kc_sync<4096, 6144>(r[2], r[3], faR.a[0]);
    };
    // multiply the current slice while the fragments of slice NKS of the stage at byte offset `so` are read
    auto step = [&](auto nks_tag, unsigned so) {
        constexpr int NKS = decltype(nks_tag)::value;
        V nf[2], nr[RB];
        const unsigned aR = faR.a[NKS] + so;
        if (W_IN_OUT) {
            s16x4 h[4];
            block_ks_kc<TC, FBASE + NKS * 16 * KSROW, FBASE + (NKS * 16 + 4) * KSROW, 0, 2048>(
                h, nr[0], nr[1], acc[0][0], acc[0][1], acc[1][0], acc[1][1], f[0], f[1], r[0], r[1], faF.a[0] + so, faF.a[1] + so, aR);
            nf[0] = join_halves<V>(h[0], h[1]); nf[1] = join_halves<V>(h[2], h[3]);
        } else {
            block_kc_kc<TC, FBASE, FBASE + 2048, 0, 2048>(nf[0], nf[1], nr[0], nr[1], acc[0][0], acc[0][1], acc[1][0], acc[1][1],
                                                          f[0], f[1], r[0], r[1], faF.a[NKS] + so, aR);
        }
        if constexpr (RB == 4)
            block_r_kc<TC, 4096, 6144>(nr[2], nr[3], acc[0][2], acc[0][3], acc[1][2], acc[1][3], f[0], f[1], r[2], r[3], aR);
        f[0] = nf[0]; f[1] = nf[1];
#pragma unroll
        for (int i = 0; i < RB; ++i) r[i] = nr[i];
    };
    auto multiply_last = [&]() {
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int i = 0; i < RB; ++i) acc[j][i] = Mfma<TC>::run(f[j], r[i], acc[j][i]);
    };
    // accumulators start from the bias of the tile's columns (block j, group g -> 4 consecutive columns)
    auto init_acc = [&](int buf) {
        if (!p.bias) {
            zero_acc(acc);
            return;
        }
        int ln = lane;
        asm volatile("" : "+v"(ln));
        const unsigned biasb = lds0 + L::BIAS + buf * BN * 4;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            u32x4 raw[4];
            float b[4][4];
            if (bias32) {
                lds_read4_b128_sync<0, 32>(biasb + (wf * FW + j * 32 + 4 * (ln >> 5)) * 4, raw);
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    b[g][0] = __uint_as_float(raw[g].x); b[g][1] = __uint_as_float(raw[g].y);
                    b[g][2] = __uint_as_float(raw[g].z); b[g][3] = __uint_as_float(raw[g].w);
                }
            } else {
                // 8 columns (16 bytes) per read; this lane's 4 are the low or the high half
                lds_read4_b128_sync<0, 16>(biasb + (wf * FW + j * 32) * 2, raw);
                const bool hi = (ln >> 5) != 0;
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const unsigned lo2 = hi ? raw[g].z : raw[g].x, hi2 = hi ? raw[g].w : raw[g].y;
                    b[g][0] = from_bits16<TC>(lo2 & 0xffff); b[g][1] = from_bits16<TC>(lo2 >> 16);
                    b[g][2] = from_bits16<TC>(hi2 & 0xffff); b[g][3] = from_bits16<TC>(hi2 >> 16);
                }
            }
#pragma unroll
            for (int i = 0; i < RB; ++i)
#pragma unroll
                for (int g = 0; g < 4; ++g)
#pragma unroll
                    for (int q = 0; q < 4; ++q) acc[j][i][4 * g + q] = b[g][q];
        }
    };

    // ---- first tile (and the record of the second) ----
    Tile cur = locate(tile);
    Tile nxt = cur;
    if (tile + stride < total) nxt = locate(tile + stride);
    int buf = 0;
    issue_meta(cur, 0, nullptr, 0);
    wait_vmcnt<0>();
    barrier_nofence();
    set_sources(cur, 0);
    issue_first_stages();
    init_acc(0);

    const bool gelu = p.act == HEXA_ACT_GELU;
    const bool gelu_bwd = p.act == HEXA_ACT_GELU_BWD;

    while (true) {
        const int next_tile = tile + stride;
        const bool has_next = next_tile < total;
        const bool has_after = next_tile + stride < total;
        Tile aft = nxt;   // the tile after the next one: its record arrives through LDS
        const int4* aft_record = has_after ? place(next_tile + stride, aft) : nullptr;

        // ---- main loop: stage kt is multiplied while stages kt+1 .. kt+STAGES-2 are in flight.
        // Copies in issue order: stages 0..STAGES-2 (issued before the previous tile's epilogue),
        // stage STAGES-1, the next tile's metadata, stage STAGES, ...  Copies return in order, so
        // "at most n outstanding" pins down which ones have landed; the previous tile's stores,
        // which also count, only make a wait stricter.
        wait_outstanding<C::CPW, L::PCW>(min(nk - 1, STAGES - 2), false);
        barrier_nofence();
        if (STAGES - 1 < nk) issue((STAGES - 1) % STAGES);
        if (has_next) issue_meta(nxt, buf ^ 1, aft_record, buf);
        read_first();
        for (int kt = 0; kt < nk; ++kt) {
            step(std::integral_constant<int, 1>{}, (kt % STAGES) * C::STAGE_BYTES);   // slice 0 x, slice 1 read
            if (kt + 1 < nk) {
                // stage kt+1 must have landed; the metadata copies are younger than stage STAGES-1
                wait_outstanding<C::CPW, L::PCW>(min(nk - 2 - kt, STAGES - 2), has_next && kt + 1 <= STAGES - 1);
                barrier_nofence();   // stage kt+1 is in LDS for everyone, nobody reads stage kt any more
                if (kt + STAGES < nk) issue((kt + STAGES) % STAGES);
                step(std::integral_constant<int, 0>{}, ((kt + 1) % STAGES) * C::STAGE_BYTES);   // slice 1 x, next slice 0 read
            } else {
                multiply_last();
            }
        }
        wait_vmcnt<0>();     // the metadata copies (all older copies are long done)
        barrier_nofence();   // every wavefront is done with the stage buffers; the next tile's ids are in LDS
        if (has_after) {
            const u32x4 rec = lds_read_b128_sync(lds0 + L::INFO + buf * 256);
            aft.e = __builtin_amdgcn_readfirstlane(rec.x);
            aft.row_start = __builtin_amdgcn_readfirstlane(rec.y);
            aft.rows = __builtin_amdgcn_readfirstlane(rec.z);
        }

        // ---- the next tile's first stages start ----
        if (has_next) {
            set_sources(nxt, buf ^ 1);
            issue_first_stages();
        }

        // ---- epilogue of the current tile ----
        int ln = lane;
        asm volatile("" : "+v"(ln));   // epilogue address arithmetic stays inside the tile loop
        const int tde = wave * 64 + ln;
        const bool to_ws = p.ws != nullptr && cur.s > 0;
        void* const outp = to_ws ? p.ws : p.out;
        const bool accumulate = p.accumulate != 0 && !to_ws;
        const size_t out_base = to_ws ? (size_t)p.T * (cur.s - 1) : (size_t)p.out_slot_rows * cur.s;
        const unsigned tokb = lds0 + L::TOK + buf * BM * 4;
        if (OUT32) {
            // fp32 results are stored from the registers, 16 bytes per lane
#pragma unroll
            for (int i = 0; i < RB; i += 2) {
                int tok[2];
                const int trow = wr * RW + i * 32 + (ln & 31);
                lds_read2_i32_sync(tokb + trow * 4, tokb + (trow + 32) * 4, tok[0], tok[1]);
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    if (trow + 32 * u >= cur.rows) continue;
#pragma unroll
                    for (int j = 0; j < 2; ++j)
#pragma unroll
                        for (int g = 0; g < 4; ++g) {
                            const int n = cur.n0 + wf * FW + j * 32 + 8 * g + 4 * (ln >> 5);
                            if (n >= N) continue;
                            float v[4];
#pragma unroll
                            for (int q = 0; q < 4; ++q) v[q] = acc[j][i + u][4 * g + q];
                            const size_t off = (out_base + tok[u]) * N + n;
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
                        }
                }
            }
        } else {
            // 16-bit results leave through LDS, one 32-row block of every wavefront per pass, so that
            // BN/8 lanes write one contiguous row piece of 16 bytes each
            constexpr int LPR = BN / 8;                    // lanes per row
            constexpr int RPI = C::NT / LPR;               // rows per iteration
            constexpr int ITERS = L::PASS_ROWS / RPI;
            static_assert(ITERS == 4, "four staged rows per thread and pass");
            static_assert(RPI == 8 || RPI == 16 || RPI == 32, "staged row -> tile row by constant offsets");
            const int c = tde % LPR, n = cur.n0 + c * 8, rsub = tde / LPR;
            // staged row it*RPI + rsub belongs to wavefront row (it*RPI)/32, row ((it*RPI)%32 + rsub) of its block
            auto tile_row = [&](int it, int i) { return ((it * RPI) >> 5) * RW + i * 32 + ((it * RPI) & 31) + rsub; };
#pragma unroll
            for (int i = 0; i < RB; ++i) {
                if (i > 0) lds_barrier();                  // the previous pass has been read
#pragma unroll
                for (int j = 0; j < 2; ++j)
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const int nl = wf * FW + j * 32 + 8 * g + 4 * (ln >> 5);
                        const int srow = wr * 32 + (ln & 31);
                        lds_write_b64(lds0 + L::STAGING + srow * L::CP + nl * 2,
                                      pack4<TC>(acc[j][i][4 * g + 0], acc[j][i][4 * g + 1], acc[j][i][4 * g + 2], acc[j][i][4 * g + 3]));
                    }
                lds_barrier();
                u32x4 val[4];
                int tok[4];
#define HEXA_TROW(it) ((((it) * RPI) >> 5) * RW * 4 + (((it) * RPI) & 31) * 4)
                lds_read4_pairs_sync<HEXA_TROW(0), HEXA_TROW(1), HEXA_TROW(2), HEXA_TROW(3), 0, RPI * L::CP, 2 * RPI * L::CP, 3 * RPI * L::CP>(
                    tokb + (i * 32 + rsub) * 4, lds0 + L::STAGING + rsub * L::CP + c * 16, tok, val);
#undef HEXA_TROW
#pragma unroll
                for (int it = 0; it < ITERS; ++it) {
                    if (tile_row(it, i) >= cur.rows || n >= N) continue;
                    const size_t off = (out_base + tok[it]) * N + n;
                    uint4 v = make_uint4(val[it].x, val[it].y, val[it].z, val[it].w);
                    uint4* dst = reinterpret_cast<uint4*>(reinterpret_cast<unsigned short*>(outp) + off);
                    if (gelu_bwd) {
                        const uint4 yv = *reinterpret_cast<const uint4*>(reinterpret_cast<const unsigned short*>(p.out_act) + off);
                        const unsigned yw[4] = {yv.x, yv.y, yv.z, yv.w};
                        unsigned vw[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            const float lo = from_bits16<TC>(vw[q] & 0xffff) * gelu_grad_fast(from_bits16<TC>(yw[q] & 0xffff));
                            const float hi = from_bits16<TC>(vw[q] >> 16) * gelu_grad_fast(from_bits16<TC>(yw[q] >> 16));
                            vw[q] = bits16<TC>(lo) | ((unsigned)bits16<TC>(hi) << 16);
                        }
                        v = make_uint4(vw[0], vw[1], vw[2], vw[3]);
                    }
                    if (accumulate) {
                        const uint4 old = *dst;
                        const unsigned ow[4] = {old.x, old.y, old.z, old.w};
                        unsigned vw[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            const float lo = from_bits16<TC>(vw[q] & 0xffff) + from_bits16<TC>(ow[q] & 0xffff);
                            const float hi = from_bits16<TC>(vw[q] >> 16) + from_bits16<TC>(ow[q] >> 16);
                            vw[q] = bits16<TC>(lo) | ((unsigned)bits16<TC>(hi) << 16);
                        }
                        v = make_uint4(vw[0], vw[1], vw[2], vw[3]);
                    }
                    *dst = v;
                    if (gelu) {
                        // applied to the value as stored (rounded), like act(y1) on the tensor
                        unsigned vw[4] = {v.x, v.y, v.z, v.w};
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
        if (!has_next) break;
        cur = nxt;
        nxt = aft;
        tile = next_tile;
        buf ^= 1;
        init_acc(buf);
    }
}

// workgroups of `kernel` that fit on the chip at once, rounded down to a multiple of the XCD count
template <typename Kn> int persistent_grid(Kn kernel, int threads, int smem_bytes, int* grid) {
    int dev = 0, cus = 0, per_cu = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, reinterpret_cast<const void*>(kernel), threads, smem_bytes) != hipSuccess ||
        cus <= 0 || per_cu <= 0)
        HEXA_FAIL(HEXA_ERR_LAUNCH, "occupancy query failed (CUs %d, workgroups per CU %d)", cus, per_cu);
    *grid = (cus * per_cu) / 8 * 8;
    if (*grid < 8) *grid = 8;
    return HEXA_OK;
}

template <typename TC, bool IO, bool OUT32, typename C>
int launch_t(EsmmK& p, hipStream_t st) {
    auto kernel = esmm16_persist_kernel<TC, IO, OUT32, C>;
    constexpr int bytes = PersistLds<C>::TOTAL;
    if (int rc = ensure_smem(kernel, bytes)) return rc;
    static int grid = 0;   // per instantiation
    if (grid == 0)
        if (int rc = persistent_grid(kernel, C::NT, bytes, &grid)) return rc;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(C::NT), bytes, st, p);
    HEXA_CHECK_LAUNCH("esmm16_persist");
    return HEXA_OK;
}

template <typename TC, typename C>
int launch_d(EsmmK& p, bool io, bool o32, hipStream_t st) {
    if (o32) return io ? launch_t<TC, true, true, C>(p, st) : launch_t<TC, false, true, C>(p, st);
    return io ? launch_t<TC, true, false, C>(p, st) : launch_t<TC, false, false, C>(p, st);
}

template <typename C>
int launch_c(const EsmmArgs& a, bool large, hipStream_t st) {
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
    p.group = 0; p.total = 0; p.stream_out = 0;
    // Summing the slots into one result: with scratch, every slot runs in ONE launch (slot 0 into
    // `out`, the others into the scratch) and a reduction adds them in slot order; without it, one
    // launch per slot, each adding into `out`.
    const bool one_launch = a.out_per_slot || a.r.k == 1 || a.slot_ws != nullptr;
    p.ws = (!a.out_per_slot && a.r.k > 1) ? a.slot_ws : nullptr;
    const int launches = one_launch ? 1 : a.r.k;
    if (p.mt_ub == 0 || p.ntn == 0) return HEXA_OK;
    for (int l = 0; l < launches; ++l) {
        p.slot_begin = one_launch ? 0 : l;
        p.nslots = one_launch ? a.r.k : 1;
        p.accumulate = (a.accumulate || l > 0) ? 1 : 0;
        const bool io = a.w_layout == HEXA_W_IN_OUT;
        const bool o32 = a.out_dt == HEXA_F32;
        const int rc = a.x_dt == HEXA_BF16 ? launch_d<__bf16, C>(p, io, o32, st) : launch_d<_Float16, C>(p, io, o32, st);
        if (rc) return rc;
    }
    if (p.ws) return launch_sum_slots(a.out, a.slot_ws, (int64_t)a.r.T * a.out_dim, a.r.k - 1, a.out_dt, st, a.sum_extra);
    return HEXA_OK;
}

}  // namespace

bool esmm16_persist_supported(const EsmmArgs& a) {
    const int slots_per_launch = (a.out_per_slot || a.r.k == 1 || a.slot_ws != nullptr) ? a.r.k : 1;
    return esmm16_dma_supported(a) && slots_per_launch <= PERSIST_MAX_SLOTS;
}

// tile: 0 / 1 -> 128x128, 2 -> 256x128 with 8 wavefronts, 3 -> 256x128 with 4 wavefronts
int launch_esmm16_persist(const EsmmArgs& a, int tile, hipStream_t st) {
    switch (tile) {
        case 2: return launch_c<CfgPL>(a, true, st);
        case 3: return launch_c<CfgPM>(a, true, st);
        default: return launch_c<CfgPS>(a, false, st);
    }
}

}  // namespace hexa
