// Bodies of two single-workgroup kernels that also run as an extra workgroup of another launch (every launch
// of a small kernel costs 5-7 us of the step here, whatever it computes): the GShard loss from the router's
// per-workgroup partial sums, and the work plan of the balanced ESTMM.  Both are written for any workgroup size.
#pragma once
#include "small_tasks.h"

namespace hexa {

// me[e] = sum_t scores[t][e]; ce[e] = count[e] * E / T; l_aux = sum_e me[e]*ce[e] / T  (losses.py:12-19).
// lds: 2 * nch * E + blockDim.x floats, nch = router_loss_chunks(E).
__host__ __device__ inline int router_loss_chunks(int E) { return E <= 256 ? 32 : (8192 / E > 0 ? 8192 / E : 1); }

__device__ inline void router_loss_body(float* lds, float* __restrict__ l_aux, float* __restrict__ me,
                                        float* __restrict__ ce, const float* __restrict__ part_me,
                                        const float* __restrict__ part_cnt, int nblocks, int num_tokens, int E) {
    // per expert: nch threads sum nch contiguous ranges of the workgroup partials, then the range sums
    // are added in range order -- a fixed tree, independent of scheduling
    const int nch = router_loss_chunks(E), nthr = blockDim.x, tid = threadIdx.x;
    float* s_m = lds;
    float* s_c = lds + nch * E;
    float* red = lds + 2 * nch * E;
    const int per = (nblocks + nch - 1) / nch;
    for (int i = tid; i < nch * E; i += nthr) {
        const int c = i / E, e = i - c * E;
        const int b0 = c * per, b1 = min(nblocks, b0 + per);
        float m = 0.f, n = 0.f;
        for (int b = b0; b < b1; b += 8) {     // eight partials of each kind in flight per trip, added in order
            float pm[8], pc[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const size_t at = (size_t)min(b + u, b1 - 1) * E + e;
                pm[u] = part_me[at];
                pc[u] = part_cnt[at];
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                m += (b + u < b1) ? pm[u] : 0.f;
                n += (b + u < b1) ? pc[u] : 0.f;
            }
        }
        s_m[i] = m;
        s_c[i] = n;
    }
    __syncthreads();
    float local = 0.f;
    for (int e = tid; e < E; e += nthr) {
        float m = 0.f, c = 0.f;
        for (int j = 0; j < nch; ++j) { m += s_m[j * E + e]; c += s_c[j * E + e]; }
        const float cev = c * ((float)E / (float)num_tokens);
        me[e] = m;
        ce[e] = cev;
        local += m * cev;
    }
    red[tid] = local;
    __syncthreads();
    if (tid == 0) {       // E products spread over the threads: their partial sums are added in thread order
        float t = 0.f;
        for (int i = 0; i < nthr; ++i) t += red[i];
        *l_aux = t / (float)num_tokens;
    }
}

// ---- plan of a balanced ESTMM launch ------------------------------------------------------------------
// One workgroup's walk over an expert's token list is serial, so the kernel is as slow as the
// busiest expert.  With scratch memory, experts with more than `cap` tokens are cut into up to
// PLAN_MAX_PARTS parts of equal step counts; a part is a unit of work like a whole small expert, its
// fp32 partial result goes to a scratch slot, and estmm_fixup_kernel adds an expert's slots in order
// (bit-reproducible).  Units are numbered heaviest expert first.  plan = 4 arrays of E ints in rank
// order -- expert, parts, first unit, first scratch slot -- followed by the number of units.
// lds: 2 * E ints.
constexpr int PLAN_MAX_PARTS = 8;
constexpr int PLAN_QUEUE_INTS = 16;    // work counters of the persistent ESTMM kernel behind the plan (8 queues, a finish count)
__host__ __device__ inline int estmm_plan_queue_at(int E) { return 4 * E + 1; }

// An expert's list is cut when it is longer than `cap` rows.  The persistent kernel hands items (an expert's or
// part's list x one 128 x 128 block of the result) longest-first to whichever workgroup is free, so a cut only pays
// when one item would be longer than a workgroup's share of the launch: rows of all lists x blocks per expert /
// workgroups (`tiles` = 0: unknown result size, the rule of the one-item-per-workgroup kernel: 1.5x the mean load).
__host__ __device__ inline int estmm_plan_cap(long T, int k, int E, int tiles = 0, int workgroups = 256) {
    const long avg = T * k / E;
    long c = (3 * avg + 1) / 2;
    if (tiles > 0) c = T * k * tiles / workgroups;
    return (int)(c > 256 ? c : 256);
}

__device__ inline void estmm_plan_from_loads(int* sp, int* __restrict__ plan, int E, int cap, int max_slots);

__device__ inline void estmm_plan_body(int* sp, int* __restrict__ plan, const int32_t* __restrict__ offsets, int E, int k,
                                       int cap, int max_slots) {
    int* load = sp;
    const int nthr = blockDim.x;
    for (int e = threadIdx.x; e < E; e += nthr) {
        int t = 0;
        for (int s = 0; s < k; ++s) t += offsets[(size_t)s * (E + 1) + e + 1] - offsets[(size_t)s * (E + 1) + e];
        load[e] = t;
    }
    __syncthreads();
    estmm_plan_from_loads(sp, plan, E, cap, max_slots);
}

// The plan from sp[0..E) = tokens per expert over all slots (written and published by the caller).
__device__ inline void estmm_plan_from_loads(int* sp, int* __restrict__ plan, int E, int cap, int max_slots) {
    int* load = sp;
    int* expert_of = sp + E;          // the expert at each rank
    const int nthr = blockDim.x;
    for (int e = threadIdx.x; e < E; e += nthr) {
        const int mine = load[e];
        int r = 0;
        for (int x = 0; x < E; ++x) {
            const int o = load[x];
            r += (o > mine || (o == mine && x < e)) ? 1 : 0;
        }
        expert_of[r] = e;
    }
    __syncthreads();
    if (threadIdx.x == 0) {          // E is small: a serial pass hands out units and scratch slots
        int unit = 0, slot = 0;
        for (int r = 0; r < E; ++r) {
            const int e = expert_of[r];
            int n = (load[e] + cap - 1) / cap;
            n = max(1, min(n, PLAN_MAX_PARTS));
            if (n > 1 && slot + n > max_slots) n = 1;
            plan[r] = e;
            plan[E + r] = n;
            plan[2 * E + r] = unit;
            plan[3 * E + r] = n > 1 ? slot : -1;
            unit += n;
            if (n > 1) slot += n;
        }
        plan[4 * E] = unit;
    }
    if (threadIdx.x < PLAN_QUEUE_INTS) plan[estmm_plan_queue_at(E) + threadIdx.x] = 0;
}

// ---- ESS: per-expert column sums of gathered rows (see ess.hip) --------------------------------------------------
template <typename T> struct Vec16;  // 16 bytes of T
template <> struct Vec16<float> { static constexpr int N = 4; };
template <> struct Vec16<__bf16> { static constexpr int N = 8; };
template <> struct Vec16<_Float16> { static constexpr int N = 8; };

template <typename T>
__device__ __forceinline__ void ess_body(const EssK& p, int block) {
    constexpr int V = Vec16<T>::N;
    constexpr int STRIP = 8 * V;  // columns per workgroup
    constexpr int U = 8;          // rows in flight per lane: 256 rows (32 KiB) per workgroup step
    __shared__ float red[4][STRIP];
    const int bx = block % p.gx, by = (block / p.gx) % p.gy, bz = block / (p.gx * p.gy);
    const int e = by;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int cl = lane & 7, rg = lane >> 3;
    const int col = bx * STRIP + cl * V;
    const bool col_ok = col < p.N;
    const T* dy = reinterpret_cast<const T*>(p.dy);

    float acc[V];
#pragma unroll
    for (int i = 0; i < V; ++i) acc[i] = 0.f;

    bool any = false;
    for (int s = 0; s < p.k; ++s) {
        int beg = p.offsets[(size_t)s * (p.E + 1) + e];
        int end = p.offsets[(size_t)s * (p.E + 1) + e + 1];
        any = any || end > beg;
        if (p.splits > 1) {
            const int part = (end - beg + p.splits - 1) / p.splits;
            beg = min(end, beg + bz * part);
            end = min(end, beg + part);
        }
        const int32_t* tok = p.token_ids + (size_t)s * p.T;
        const T* base = dy + (size_t)p.dy_slot_rows * s * p.N + col;
        // this lane's rows: beg + wave*8 + rg + 32*u + 256*step; the token ids of the next step are
        // fetched while the rows of the current one are in flight
        const int r_lane = beg + wave * 8 + rg;
        int ids[U];
#pragma unroll
        for (int u = 0; u < U; ++u) { const int r = r_lane + 32 * u; ids[u] = r < end ? tok[r] : -1; }
        for (int r0 = r_lane; r0 < end; r0 += 32 * U) {
            union { uint4 u; T e[V]; } v[U];
#pragma unroll
            for (int u = 0; u < U; ++u)
                v[u].u = (ids[u] >= 0 && col_ok) ? *reinterpret_cast<const uint4*>(base + (size_t)ids[u] * p.N)
                                                 : make_uint4(0u, 0u, 0u, 0u);
#pragma unroll
            for (int u = 0; u < U; ++u) { const int r = r0 + 32 * U + 32 * u; ids[u] = r < end ? tok[r] : -1; }
#pragma unroll
            for (int u = 0; u < U; ++u)
#pragma unroll
                for (int i = 0; i < V; ++i) acc[i] += Cvt<T>::to_f(v[u].e[i]);
        }
    }
#pragma unroll
    for (int i = 0; i < V; ++i) {
        float a = acc[i];
        a += __shfl_xor(a, 8);
        a += __shfl_xor(a, 16);
        a += __shfl_xor(a, 32);
        acc[i] = a;
    }
    if (rg == 0) {
#pragma unroll
        for (int i = 0; i < V; ++i) red[wave][cl * V + i] = acc[i];
    }
    __syncthreads();
    if (tid < STRIP) {
        const int c = bx * STRIP + tid;
        const float v = red[0][tid] + red[1][tid] + red[2][tid] + red[3][tid];
        if (p.splits > 1) {
            if (c < p.N) p.ws[((size_t)bz * p.E + e) * p.N + c] = v;
        } else if (c < p.N && (any || !p.accumulate)) {
            store_out(p.db, (size_t)e * p.N + c, v, p.db_dt, p.accumulate != 0);
        }
    }
}

// db (+)= ws[0] + ws[1] + ... in that order
__device__ __forceinline__ void ess_fold_body(const EssFoldK& p, int block) {
    const long i = (long)block * 256 + threadIdx.x;
    if (i >= p.n) return;
    // all parts' loads in flight at once (at most 8 parts), added in part order
    float part[8];
#pragma unroll
    for (int z = 0; z < 8; ++z) part[z] = p.ws[(size_t)min(z, p.splits - 1) * p.n + i];
    float v = part[0];
#pragma unroll
    for (int z = 1; z < 8; ++z) v += z < p.splits ? part[z] : 0.f;
    store_out(p.db, (size_t)i, v, p.db_dt, p.accumulate != 0);
}

// out[i] += ws[0][i] + ws[1][i] + ... in fp32, slot order (the deterministic reduction behind the one-launch slot
// sum of ESMM).  `extra` (may be null): one more addend of out's shape, added last (the gate path's share of an
// input gradient)
template <typename T>
__device__ __forceinline__ void sum_slots_body(const SumSlotsK& p, int block) {
    constexpr int V = Vec16<T>::N;
    T* out = reinterpret_cast<T*>(p.out);
    const T* ws = reinterpret_cast<const T*>(p.ws);
    const int64_t nv = p.n / V;
    const int64_t stride = (int64_t)p.blocks * 256;
    for (int64_t i = (int64_t)block * 256 + threadIdx.x; i < nv; i += stride) {
        union { uint4 u; T e[V]; } o, w;
        o.u = reinterpret_cast<const uint4*>(out)[i];
        float acc[V];
#pragma unroll
        for (int j = 0; j < V; ++j) acc[j] = Cvt<T>::to_f(o.e[j]);
        for (int s = 0; s < p.nws; ++s) {
            w.u = reinterpret_cast<const uint4*>(ws + (size_t)s * p.n)[i];
#pragma unroll
            for (int j = 0; j < V; ++j) acc[j] += Cvt<T>::to_f(w.e[j]);
        }
        if (p.extra) {
            w.u = reinterpret_cast<const uint4*>(p.extra)[i];
#pragma unroll
            for (int j = 0; j < V; ++j) acc[j] += Cvt<T>::to_f(w.e[j]);
        }
#pragma unroll
        for (int j = 0; j < V; ++j) o.e[j] = Cvt<T>::from_f(acc[j]);
        reinterpret_cast<uint4*>(out)[i] = o.u;
    }
}

// d l_aux / d logits through the softmax (GShard loss): with c[e] = g * ce[e] / T,
//   dlogits[t][e] = scores[t][e] * (c[e] - sum_e' scores[t][e'] * c[e'])
// One token per thread.  s_c: E floats of LDS.
__device__ __forceinline__ void router_bwd_body(float* s_c, const RouterBwdK& p, int block) {
    const int E = p.E;
    const float g = *p.grad_l / (float)p.T;
    for (int e = threadIdx.x; e < E; e += blockDim.x) s_c[e] = g * p.ce[e];
    __syncthreads();
    const int t = block * blockDim.x + threadIdx.x;
    if (t >= p.T) return;
    const float* sr = p.scores + (size_t)t * E;
    float* dr = p.dlogits + (size_t)t * E;
    float dot = 0.f;
    if ((E & 3) == 0) {
        for (int e = 0; e < E; e += 4) {
            const float4 v = *reinterpret_cast<const float4*>(sr + e);
            dot += v.x * s_c[e] + v.y * s_c[e + 1] + v.z * s_c[e + 2] + v.w * s_c[e + 3];
        }
        for (int e = 0; e < E; e += 4) {
            const float4 v = *reinterpret_cast<const float4*>(sr + e);
            *reinterpret_cast<float4*>(dr + e) = make_float4(v.x * (s_c[e] - dot), v.y * (s_c[e + 1] - dot),
                                                             v.z * (s_c[e + 2] - dot), v.w * (s_c[e + 3] - dot));
        }
    } else {
        for (int e = 0; e < E; ++e) dot += sr[e] * s_c[e];
        for (int e = 0; e < E; ++e) dr[e] = sr[e] * (s_c[e] - dot);
    }
}

// dw[e] (+)= slot[0] + slot[1] + ... for the experts that the ESTMM plan cut into parts
constexpr int FIXUP_PIECES = 4;   // pieces of 1024 results per fix-up workgroup
__device__ __forceinline__ void estmm_fixup_body(const FixupK& p, int block) {
    // Workgroups (bx, j): piece bx of the result of the j-th expert whose list was cut.  A cut expert holds at least
    // two scratch slots, so the launch has max_slots / 2 values of j and not one per expert -- with 32 experts of
    // 3072 x 768 results and no list cut, one per expert was 74 thousand workgroups that only looked and left, 35 us.
    const int bx = block % p.gx, j = block / p.gx;
    const int E = p.E, lane = threadIdx.x & 63;
    int r = -1;
    for (int r0 = 0, seen = 0; r0 < E && r < 0; r0 += 64) {
        const bool cut = r0 + lane < E && p.plan[E + r0 + lane] > 1;
        unsigned long long m = __builtin_amdgcn_ballot_w64(cut);
        const int c = __builtin_popcountll(m);
        if (j < seen + c) {
            for (int q = j - seen; q > 0; --q) m &= m - 1;
            r = r0 + (int)__builtin_ctzll(m);
        }
        seen += c;
    }
    if (r < 0) return;
    const int n = p.plan[E + r];
    const int e = p.plan[r];
    const float* src0 = p.scratch + (size_t)p.plan[3 * E + r] * p.mn;
    // FIXUP_PIECES pieces of 1024 results per workgroup, one after the other
    for (int it = 0; it < FIXUP_PIECES; ++it) {
        const long i = (((long)bx * FIXUP_PIECES + it) * 256 + threadIdx.x) * 4;
        if (i >= p.mn) return;
        const float* src = src0 + i;
        // four parts' loads in flight at once, added in part order
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        for (int c0 = 0; c0 < n; c0 += 4) {
            float4 w[4];
#pragma unroll
            for (int c = 0; c < 4; ++c) w[c] = *reinterpret_cast<const float4*>(src + (size_t)min(c0 + c, n - 1) * p.mn);
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                if (c0 + c < n) {
                    if (c0 + c == 0) v = w[0];
                    else { v.x += w[c].x; v.y += w[c].y; v.z += w[c].z; v.w += w[c].w; }
                }
            }
        }
        const size_t o = (size_t)e * p.mn + i;
        if (!p.accumulate) {   // one store of the four results (mn is a multiple of 4, so the piece is aligned)
            typedef __attribute__((ext_vector_type(4))) float f4;
            typedef __attribute__((ext_vector_type(2))) unsigned u2;
            if (p.dw_dt == HEXA_F32) {
                f4 w4 = {v.x, v.y, v.z, v.w};
                *reinterpret_cast<f4*>(reinterpret_cast<float*>(p.dw) + o) = w4;
            } else {
                union { __bf16 b[4]; _Float16 h[4]; u2 w; } pk;   // the conversions of store_out
                if (p.dw_dt == HEXA_BF16) { pk.b[0] = (__bf16)v.x; pk.b[1] = (__bf16)v.y; pk.b[2] = (__bf16)v.z; pk.b[3] = (__bf16)v.w; }
                else { pk.h[0] = (_Float16)v.x; pk.h[1] = (_Float16)v.y; pk.h[2] = (_Float16)v.z; pk.h[3] = (_Float16)v.w; }
                *reinterpret_cast<u2*>(reinterpret_cast<unsigned short*>(p.dw) + o) = pk.w;
            }
            continue;
        }
        store_out(p.dw, o, v.x, p.dw_dt, true);
        store_out(p.dw, o + 1, v.y, p.dw_dt, true);
        store_out(p.dw, o + 2, v.z, p.dw_dt, true);
        store_out(p.dw, o + 3, v.w, p.dw_dt, true);
    }
}

// db[e][n] (+)= the column sums an ESMM launch left per (slot, row tile, column tile), added in tile order.
// The tiles of a slot are listed expert after expert, so expert e's run starts at the number of tiles of the
// experts before it: every thread of the workgroup adds up ceil(rows / tile_rows) over a share of those experts
// (one round of loads instead of a bisection's chain of dependent ones).
__device__ __forceinline__ void colsum_fold_body(const ColsumFoldK& p, int block) {
    __shared__ int sFirst[8], sCount[8];        // per slot: first tile of expert e, its number of tiles
    __shared__ int red[256];
    const int bx = block % p.gx, e = block / p.gx, tid = threadIdx.x;
    for (int s = 0; s < p.nslots; ++s) {
        const int32_t* off = p.offsets + (size_t)s * (p.E + 1);
        int before = 0;
        for (int x = tid; x < e; x += 256) before += (off[x + 1] - off[x] + p.tile_rows - 1) / p.tile_rows;
        red[tid] = before;
        __syncthreads();
        for (int w = 128; w > 0; w >>= 1) {
            if (tid < w) red[tid] += red[tid + w];
            __syncthreads();
        }
        if (tid == 0) { sFirst[s] = red[0]; sCount[s] = (off[e + 1] - off[e] + p.tile_rows - 1) / p.tile_rows; }
        __syncthreads();
    }
    const int n = bx * 256 + tid;
    if (n >= p.N) return;
    const int nt = n / p.bn, nl = n - nt * p.bn;
    float sum = 0.f;
    for (int s = 0; s < p.nslots; ++s) {
        const int first = sFirst[s], last = min(first + sCount[s], p.mt_ub);
        // eight loads in flight per trip (a busy expert has a dozen tiles; one load per trip would pay the
        // memory latency a dozen times); the additions stay in tile order
        for (int mt = first; mt < last; mt += 8) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = p.colsum[(((size_t)s * p.mt_ub + min(mt + u, last - 1)) * p.ntn + nt) * p.bn + nl];
#pragma unroll
            for (int u = 0; u < 8; ++u) sum += (mt + u < last) ? v[u] : 0.f;
        }
    }
    store_out(p.db, (size_t)e * p.N + n, sum, p.db_dt, p.accumulate != 0);
}

}  // namespace hexa
