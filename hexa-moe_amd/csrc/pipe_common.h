// Helpers shared by the role-split persistent kernels (gemm16_pipe.hip: ESMM, gemm16_estmm_pipe.hip: ESTMM): LDS
// accesses as inline assembly with immediate offsets, global accesses with a base every lane shares plus a 32-bit
// lane offset, and the multiply wavefronts' software-pipelined stage product.
#pragma once
#include <type_traits>
#include <utility>

#include "dma_common.h"

namespace hexa {
namespace {

typedef __attribute__((ext_vector_type(4))) unsigned u32x4;
typedef __attribute__((ext_vector_type(2))) unsigned u32x2;

// LDS accesses with the constant part of the address as the instruction's immediate offset (0..65535), so
// that one address register serves a whole unrolled group of accesses
template <int OFF = 0> __device__ __forceinline__ void lds_write64(unsigned addr, uint2 v) {
    static_assert(OFF >= 0 && OFF < 65536, "LDS offset field");
    u32x2 w;
    w.x = v.x; w.y = v.y;
    asm volatile("ds_write_b64 %0, %1 offset:%2" ::"v"(addr), "v"(w), "n"(OFF) : "memory");
}
template <int OFF = 0> __device__ __forceinline__ void lds_write128(unsigned addr, u32x4 v) {
    static_assert(OFF >= 0 && OFF < 65536, "LDS offset field");
    asm volatile("ds_write_b128 %0, %1 offset:%2" ::"v"(addr), "v"(v), "n"(OFF) : "memory");
}
template <int OFF = 0> __device__ __forceinline__ u32x4 lds_read128_async(unsigned addr) {
    static_assert(OFF >= 0 && OFF < 65536, "LDS offset field");
    u32x4 r;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF));
    return r;
}
template <int OFF = 0> __device__ __forceinline__ u32x2 lds_read64_async(unsigned addr) {
    static_assert(OFF >= 0 && OFF < 65536, "LDS offset field");
    u32x2 r;
    asm volatile("ds_read_b64 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF));
    return r;
}
template <int OFF = 0> __device__ __forceinline__ int lds_read32_async(unsigned addr) {
    static_assert(OFF >= 0 && OFF < 65536, "LDS offset field");
    int r;
    asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF));
    return r;
}
// f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>): a loop whose index is a constant expression
template <int... I, typename F> __device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F&& f) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F> __device__ __forceinline__ void static_for(F&& f) {
    static_for_impl(std::make_integer_sequence<int, N>{}, f);
}
__device__ __forceinline__ void lds_wait() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }
// 16 bytes from base + off (a scalar base and a 32-bit lane offset: one address register per lane)
// 16-byte store to base + off (a base every lane shares plus a 32-bit byte offset); `streaming` (uniform) adds the
// non-temporal hint
__device__ __forceinline__ void global_store128(void* base, unsigned off, u32x4 v, bool streaming) {
    if (streaming) asm volatile("global_store_dwordx4 %0, %1, %2 nt" ::"v"(off), "v"(v), "s"(base) : "memory");
    else asm volatile("global_store_dwordx4 %0, %1, %2" ::"v"(off), "v"(v), "s"(base) : "memory");
}
__device__ __forceinline__ u32x4 global_load128_async(const void* base, unsigned off) {
    u32x4 r;
    asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(r) : "v"(off), "s"(base));
    return r;
}

// One stage's products for a wavefront that does nothing else: the fragments of contraction step ks+1 are read
// from LDS while the MFMAs of step ks run (with one such wavefront per SIMD there is no neighbour to fill the
// gap between a step's reads and its first MFMA: read-then-multiply keeps the matrix pipeline at about 60 %).
// All reads are inline assembly and return in order: the wait before step ks allows exactly the reads of step
// ks+1 to be outstanding, and every fragment passes through an empty statement behind that wait.
template <int N> __device__ __forceinline__ void lds_wait_but() { asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(N) : "memory"); }
template <typename TC, typename C, bool F_KS, bool R_KS = false>
__device__ __forceinline__ void mma_stage_ahead(unsigned tileR, unsigned tileF, int wr, int wf, int lane, f32x16 (&acc)[C::FB][C::RB]) {
    using V = typename Mfma<TC>::V;
    constexpr int RW = 32 * C::RB, FW = 32 * C::FB, KD = C::BKC, NKS = KD / 16;
    constexpr int READS = (R_KS ? 2 * C::RB : C::RB) + (F_KS ? 2 * C::FB : C::FB);      // LDS read instructions per contraction step
    union Frag { V v; u32x4 q; s16x4 h[2]; };
    Frag f[2][C::FB], r[2][C::RB];
    // what does not depend on the step: the row of a KC fragment and its swizzle, the column part of a KS one
    unsigned rbase[C::RB]; int rsw[C::RB];
    const int grp = lane >> 4, sl = lane & 15;
#pragma unroll
    for (int i = 0; i < C::RB; ++i) {
        if (R_KS) {
            const int col = wr * RW + i * 32 + (grp & 1) * 16 + (sl & 3) * 4;
            rbase[i] = tileR + (col & 7) * 2;
            rsw[i] = col >> 3;
        } else {
            const int row = wr * RW + i * 32 + (lane & 31);
            rbase[i] = tileR + row * (2 * KD);
            rsw[i] = kc_swizzle<KD>(row);
        }
    }
    unsigned fbase[C::FB]; int fsw[C::FB];
#pragma unroll
    for (int j = 0; j < C::FB; ++j) {
        if (F_KS) {
            const int col = wf * FW + j * 32 + (grp & 1) * 16 + (sl & 3) * 4;
            fbase[j] = tileF + (col & 7) * 2;
            fsw[j] = col >> 3;
        } else {
            const int row = wf * FW + j * 32 + (lane & 31);
            fbase[j] = tileF + row * (2 * KD);
            fsw[j] = kc_swizzle<KD>(row);
        }
    }
    auto read_step = [&](int ks, Frag (&fs)[C::FB], Frag (&rs)[C::RB]) {
        const int kch = ks * 2 + (lane >> 5);
#pragma unroll
        for (int j = 0; j < C::FB; ++j) {
            if (F_KS) {
                const int k = ks * 16 + (grp >> 1) * 8 + (sl >> 2);
#pragma unroll
                for (int half = 0; half < 2; ++half) {
                    const int kk = k + half * 4;
                    fs[j].h[half] = lds_read_tr16(fbase[j] + kk * (2 * C::BN) + ((fsw[j] ^ ((kk & 3) << 2)) * 16));
                }
            } else {
                fs[j].q = lds_read128_async(fbase[j] + ((kch ^ fsw[j]) * 16));
            }
        }
#pragma unroll
        for (int i = 0; i < C::RB; ++i) {
            if (R_KS) {
                const int k = ks * 16 + (grp >> 1) * 8 + (sl >> 2);
#pragma unroll
                for (int half = 0; half < 2; ++half) {
                    const int kk = k + half * 4;
                    rs[i].h[half] = lds_read_tr16(rbase[i] + kk * (2 * C::BM) + ((rsw[i] ^ ((kk & 3) << 2)) * 16));
                }
            } else {
                rs[i].q = lds_read128_async(rbase[i] + ((kch ^ rsw[i]) * 16));
            }
        }
    };
    read_step(0, f[0], r[0]);
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
        const int cur = ks & 1;
        if (ks + 1 < NKS) {
            read_step(ks + 1, f[cur ^ 1], r[cur ^ 1]);
            lds_wait_but<READS>();
        } else {
            lds_wait_but<0>();
        }
#pragma unroll
        for (int j = 0; j < C::FB; ++j) asm volatile("" : "+v"(f[cur][j].q));
#pragma unroll
        for (int i = 0; i < C::RB; ++i) asm volatile("" : "+v"(r[cur][i].q));
#pragma unroll
        for (int j = 0; j < C::FB; ++j)
#pragma unroll
            for (int i = 0; i < C::RB; ++i) acc[j][i] = Mfma<TC>::run(f[cur][j].v, r[cur][i].v, acc[j][i]);
    }
}

template <typename TC> __device__ __forceinline__ float lo16(unsigned w) { return from_bits16<TC>(w & 0xffff); }
template <typename TC> __device__ __forceinline__ float hi16(unsigned w) { return from_bits16<TC>(w >> 16); }

}  // namespace
}  // namespace hexa
