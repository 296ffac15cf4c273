// Routing segment pass for gfx950: per-expert token lists without padding, dropping or host sync.
//
// Three small launches over (wavefront unit, slot):
//   1. route_hist    one wavefront per HEXA_ROUTE_UNIT consecutive tokens: LDS histogram
//   2. route_scan    one workgroup per slot: per-expert exclusive prefix over the units, exclusive
//                    scan over experts (wavefront shuffles), row-tile records for the matmul kernels
//   3. route_scatter one wavefront per unit again: stable rank of every token inside its
//                    (unit, expert) group from log2(E) ballots, so a segment lists its tokens in
//                    ascending order -- the result is a stable counting sort and is bit-reproducible.
// Up to 256 experts launches 2 and 3 run as one (route_finish_kernel): every scatter workgroup adds up the counts of
// the units before its own and of all units itself instead of waiting for a scan.
// Replaces launch_count / launch_assign of the reference (kernels/shared_cuda_core.cu:126-182,
// 284-333), which run single-workgroup launches with shared-memory atomics, two blocking copies and
// a host-side prefix per call.
#include <algorithm>

#include "hexa_internal.h"
#include "small_bodies.h"

namespace hexa {
namespace {

constexpr int kUnit = HEXA_ROUTE_UNIT;
constexpr int kWave = 64;

template <typename IdxT>
__global__ __launch_bounds__(kWave) void route_hist_kernel(const IdxT* __restrict__ routing,
                                                           int64_t token_stride, int64_t slot_stride,
                                                           int T, int E, int units,
                                                           int32_t* __restrict__ unit_hist) {
    extern __shared__ int32_t sh[];
    const int lane = threadIdx.x, unit = blockIdx.x, s = blockIdx.y;
    for (int i = lane; i < E; i += kWave) sh[i] = 0;
    __syncthreads();
    const int t0 = unit * kUnit;
    const int t1 = min(T, t0 + kUnit);
    for (int t = t0 + lane; t < t1; t += kWave) {
        long e = (long)routing[(int64_t)t * token_stride + (int64_t)s * slot_stride];
        if (e >= 0 && e < E) atomicAdd(&sh[e], 1);
    }
    __syncthreads();
    int32_t* dst = unit_hist + ((size_t)s * units + unit) * E;
    for (int i = lane; i < E; i += kWave) dst[i] = sh[i];
}

// Exclusive scan of one int per thread over the workgroup (a multiple of 64 threads, at most 1024);
// returns the exclusive prefix and the workgroup total.  tmp: 16 ints of LDS.
__device__ __forceinline__ int block_excl_scan(int v, int* tmp, int& total) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
    int incl = v;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        int o = __shfl_up(incl, d);
        if (lane >= d) incl += o;
    }
    if (lane == 63) tmp[wave] = incl;
    __syncthreads();
    int base = 0, all = 0;
    for (int w = 0; w < nwaves; ++w) {
        if (w < wave) base += tmp[w];
        all += tmp[w];
    }
    total = all;
    __syncthreads();
    return base + incl - v;
}

// Given per-expert totals in LDS (tot[E]), write counts / offsets (exclusive prefix of the totals
// rounded up to `pad`) and, when tile_info != nullptr, one record per kTileRows rows of each
// segment.  LDS: tot[E], off[E+1], tbase[E+1], tmp[16].
// One record per `rows_per_tile` rows of every expert segment (tbase: LDS scratch of E+1 ints).
__device__ void emit_tiles(const int32_t* tot, const int32_t* off, int32_t* tbase, int* tmp, int E, int rows_per_tile,
                           int4* tile_info, int32_t* tile_count, int mt_ub) {
    const int tid = threadIdx.x;
    const int nthr = blockDim.x;
    const int chunk = (E + nthr - 1) / nthr;
    const int e0 = min(E, tid * chunk), e1 = min(E, e0 + chunk);
    int sum_tiles = 0;
    for (int e = e0; e < e1; ++e) sum_tiles += (tot[e] + rows_per_tile - 1) / rows_per_tile;
    int total_tiles;
    int tile_base = block_excl_scan(sum_tiles, tmp, total_tiles);
    for (int e = e0; e < e1; ++e) {
        tbase[e] = tile_base;
        tile_base += (tot[e] + rows_per_tile - 1) / rows_per_tile;
    }
    if (tid == 0) { tbase[E] = total_tiles; *tile_count = total_tiles; }
    __syncthreads();
    const int n = min(total_tiles, mt_ub);
    for (int m = tid; m < n; m += nthr) {
        int lo = 0, hi = E;  // invariant: tbase[lo] <= m < tbase[hi]
        while (hi - lo > 1) {
            int mid = (lo + hi) >> 1;
            if (tbase[mid] <= m) lo = mid; else hi = mid;
        }
        int j = m - tbase[lo];
        int rows = min(rows_per_tile, tot[lo] - j * rows_per_tile);
        tile_info[m] = make_int4(lo, off[lo] + j * rows_per_tile, rows, 0);
    }
    __syncthreads();
}

// off[0..E] (LDS) = exclusive prefix of the totals tot[E] (LDS), each rounded up to `pad`.  tmp: 16 ints of LDS.
__device__ void scan_offsets(const int32_t* tot, int32_t* off, int* tmp, int E, int pad) {
    const int tid = threadIdx.x;
    const int nthr = blockDim.x;
    const int chunk = (E + nthr - 1) / nthr;
    const int e0 = min(E, tid * chunk), e1 = min(E, e0 + chunk);
    int sum_rows = 0;
    for (int e = e0; e < e1; ++e) sum_rows += ((tot[e] + pad - 1) / pad) * pad;
    int total_rows;
    int row_base = block_excl_scan(sum_rows, tmp, total_rows);
    for (int e = e0; e < e1; ++e) {
        off[e] = row_base;
        row_base += ((tot[e] + pad - 1) / pad) * pad;
    }
    if (tid == 0) off[E] = total_rows;
    __syncthreads();
}

__device__ void finish_slot(const int32_t* tot, int32_t* off, int32_t* tbase, int* tmp, int E, int pad,
                            int32_t* counts, int32_t* offsets, int4* tile_info, int32_t* tile_count,
                            int mt_ub, int4* tile_info_l, int32_t* tile_count_l, int mt_ub_l) {
    const int tid = threadIdx.x;
    const int nthr = blockDim.x;
    scan_offsets(tot, off, tmp, E, pad);
    for (int e = tid; e <= E; e += nthr) {
        if (offsets) offsets[e] = off[e];
        if (counts && e < E) counts[e] = tot[e];
    }
    if (tile_info) {
        emit_tiles(tot, off, tbase, tmp, E, kTileRows, tile_info, tile_count, mt_ub);
        emit_tiles(tot, off, tbase, tmp, E, HEXA_TILE_ROWS_L, tile_info_l, tile_count_l, mt_ub_l);
    }
}

// One workgroup per slot.  Turns unit_hist[s][u][e] into the exclusive prefix over u (in place) and
// finishes the slot.  given_offsets != nullptr: legacy TOKEN_ASSIGN, segment starts come from the
// caller and nothing but the unit prefixes is written.
__device__ __forceinline__ void route_scan_body(int32_t* sh, int s, int32_t* __restrict__ unit_hist, int E, int units,
                                                int pad, int32_t* __restrict__ counts, int32_t* __restrict__ offsets,
                                                int4* __restrict__ tile_info, int32_t* __restrict__ tile_count, int mt_ub,
                                                int4* __restrict__ tile_info_l, int32_t* __restrict__ tile_count_l,
                                                int mt_ub_l, int prefix_only) {
    int32_t* tot = sh;
    int32_t* off = tot + E;
    int32_t* tbase = off + (E + 1);
    int* tmp = tbase + (E + 1);
    int32_t* H = unit_hist + (size_t)s * units * E;
    // Exclusive prefix over the units, per expert.  Up to 256 experts: 256/E threads share an expert,
    // each takes a contiguous range of units (sum, then rewrite), and loads go 8 at a time so that the
    // memory latency is paid once per batch, not once per unit.
    __shared__ int32_t part[256];
    const int G = E <= 256 ? 256 / E : 1;
    for (int e0 = 0; e0 < E; e0 += 256) {
        const int tid = threadIdx.x;
        const int e = G > 1 ? tid % E : e0 + tid;
        const int j = G > 1 ? tid / E : 0;
        const bool active = e < E && j < G;
        const int per = (units + G - 1) / G;
        const int u_begin = min(units, j * per), u_end = min(units, u_begin + per);
        // up to SCAN_KEEP units per thread stay in registers between the sum and the rewrite: all of a thread's
        // loads are in flight at once and nothing is read twice
        constexpr int SCAN_KEEP = 40;
        const bool keep = per <= SCAN_KEEP;
        int c[SCAN_KEEP];
        int sum = 0;
        if (active && keep) {
#pragma unroll
            for (int i = 0; i < SCAN_KEEP; ++i) c[i] = u_begin + i < u_end ? H[(size_t)(u_begin + i) * E + e] : 0;
#pragma unroll
            for (int i = 0; i < SCAN_KEEP; ++i) sum += c[i];
        } else if (active) {
            for (int u0 = u_begin; u0 < u_end; u0 += 8) {
                int v[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) v[i] = u0 + i < u_end ? H[(size_t)(u0 + i) * E + e] : 0;
#pragma unroll
                for (int i = 0; i < 8; ++i) sum += v[i];
            }
        }
        if (G > 1) {
            part[tid] = active ? sum : 0;
            __syncthreads();
        }
        int run = 0;
        if (active) {
            for (int q = 0; q < j; ++q) run += part[q * E + e];
            if (G > 1 && j == 0) {
                int t = 0;
                for (int q = 0; q < G; ++q) t += part[q * E + e];
                tot[e] = t;
            } else if (G == 1) {
                tot[e] = sum;
            }
            if (keep) {
#pragma unroll
                for (int i = 0; i < SCAN_KEEP; ++i) {
                    if (u_begin + i < u_end) H[(size_t)(u_begin + i) * E + e] = run;
                    run += c[i];
                }
            } else {
                for (int u0 = u_begin; u0 < u_end; u0 += 8) {
                    int v[8];
#pragma unroll
                    for (int i = 0; i < 8; ++i) v[i] = u0 + i < u_end ? H[(size_t)(u0 + i) * E + e] : 0;
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        if (u0 + i < u_end) H[(size_t)(u0 + i) * E + e] = run;
                        run += v[i];
                    }
                }
            }
        }
        if (G > 1) break;
    }
    __syncthreads();
    if (prefix_only) return;
    finish_slot(tot, off, tbase, tmp, E, pad, counts ? counts + (size_t)s * E : nullptr,
                offsets ? offsets + (size_t)s * (E + 1) : nullptr,
                tile_info ? tile_info + (size_t)s * mt_ub : nullptr, tile_count ? tile_count + s : nullptr,
                mt_ub, tile_info_l ? tile_info_l + (size_t)s * mt_ub_l : nullptr,
                tile_count_l ? tile_count_l + s : nullptr, mt_ub_l);
}

__global__ __launch_bounds__(256) void route_scan_kernel(int32_t* __restrict__ unit_hist, int E, int units,
                                                         int pad, int32_t* __restrict__ counts,
                                                         int32_t* __restrict__ offsets,
                                                         int4* __restrict__ tile_info,
                                                         int32_t* __restrict__ tile_count, int mt_ub,
                                                         int4* __restrict__ tile_info_l,
                                                         int32_t* __restrict__ tile_count_l, int mt_ub_l,
                                                         int prefix_only) {
    extern __shared__ int32_t sh[];
    route_scan_body(sh, blockIdx.x, unit_hist, E, units, pad, counts, offsets, tile_info, tile_count, mt_ub, tile_info_l,
                    tile_count_l, mt_ub_l, prefix_only);
}

// The scan of every slot (workgroups 0..k-1) and, in one more workgroup of the same launch, the GShard loss from
// the router's partial sums: the two do not depend on each other, and a launch of its own for a single small
// workgroup costs as much as the whole scan.
__global__ __launch_bounds__(256) void route_scan_loss_kernel(int32_t* __restrict__ unit_hist, int E, int units, int k,
                                                              int32_t* __restrict__ counts, int32_t* __restrict__ offsets,
                                                              int4* __restrict__ tile_info,
                                                              int32_t* __restrict__ tile_count, int mt_ub,
                                                              int4* __restrict__ tile_info_l,
                                                              int32_t* __restrict__ tile_count_l, int mt_ub_l,
                                                              float* __restrict__ l_aux, float* __restrict__ me,
                                                              float* __restrict__ ce, const float* __restrict__ part_me,
                                                              const float* __restrict__ part_cnt, int nblocks,
                                                              int num_tokens) {
    extern __shared__ int32_t sh[];
    if ((int)blockIdx.x < k)
        route_scan_body(sh, blockIdx.x, unit_hist, E, units, 1, counts, offsets, tile_info, tile_count, mt_ub, tile_info_l,
                        tile_count_l, mt_ub_l, 0);
    else
        router_loss_body(reinterpret_cast<float*>(sh), l_aux, me, ce, part_me, part_cnt, nblocks, num_tokens, E);
}

template <typename IdxT>
__device__ __forceinline__ void route_scatter_loop(int32_t* cursor, bool worker, int unit, int s, int unit_tokens,
                                                   const IdxT* __restrict__ routing, int64_t token_stride,
                                                   int64_t slot_stride, int T, int E, int nbits,
                                                   int32_t* __restrict__ token_ids, int32_t* __restrict__ expert_ids,
                                                   int64_t list_stride);

template <typename IdxT>
__device__ __forceinline__ void route_scatter_body(int32_t* cursor, int unit, int s, int unit_tokens,
                                                   const IdxT* __restrict__ routing, int64_t token_stride,
                                                   int64_t slot_stride, int T, int E, int units, int nbits,
                                                   const int32_t* __restrict__ unit_hist,
                                                   const int32_t* __restrict__ offsets, int64_t offsets_slot_stride,
                                                   int32_t* __restrict__ token_ids, int32_t* __restrict__ expert_ids,
                                                   int64_t list_stride) {
    const int lane = threadIdx.x;
    const int32_t* H = unit_hist + ((size_t)s * units + unit) * E;
    const int32_t* off = offsets + (size_t)s * offsets_slot_stride;
    for (int i = lane; i < E; i += kWave) cursor[i] = off[i] + H[i];
    __syncthreads();
    route_scatter_loop<IdxT>(cursor, true, unit, s, unit_tokens, routing, token_stride, slot_stride, T, E, nbits, token_ids,
                             expert_ids, list_stride);
}

// The stable scatter of one unit's tokens given cursor[e] (LDS) = the list position of the unit's first token of
// expert e.  Every wavefront of the workgroup must call it (it contains barriers); the one with `worker` set (the
// first) does the work.
template <typename IdxT>
__device__ __forceinline__ void route_scatter_loop(int32_t* cursor, bool worker, int unit, int s, int unit_tokens,
                                                   const IdxT* __restrict__ routing, int64_t token_stride,
                                                   int64_t slot_stride, int T, int E, int nbits,
                                                   int32_t* __restrict__ token_ids, int32_t* __restrict__ expert_ids,
                                                   int64_t list_stride) {
    const int lane = threadIdx.x & 63;
    const int t0 = unit * unit_tokens;
    const int t1 = min(T, t0 + unit_tokens);
    const unsigned long long lt_mask = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
    int32_t* tok = token_ids + (size_t)s * list_stride;
    int32_t* exp = expert_ids ? expert_ids + (size_t)s * list_stride : nullptr;
    for (int base = t0; base < t1; base += kWave) {   // trip count is uniform over the wavefront
        const int t = base + lane;
        long e = -1;
        if (worker && t < t1) e = (long)routing[(int64_t)t * token_stride + (int64_t)s * slot_stride];
        const bool valid = (e >= 0 && e < E);
        // lanes holding the same expert id: AND over the id's bits of "lanes that agree on the bit"
        unsigned long long peers = __ballot(valid);
        for (int b = 0; b < nbits; ++b) {
            const bool bit = (e >> b) & 1;
            const unsigned long long m = __ballot(valid && bit);
            peers &= bit ? m : ~m;
        }
        int pos = 0;
        if (valid) pos = cursor[e] + __popcll(peers & lt_mask);
        __syncthreads();
        if (valid) {
            tok[pos] = t;
            if (exp) exp[pos] = (int32_t)e;
            if ((peers & lt_mask) == 0) cursor[e] += __popcll(peers);  // first lane of its group
        }
        __syncthreads();
    }
}

template <typename IdxT>
__global__ __launch_bounds__(kWave) void route_scatter_kernel(const IdxT* __restrict__ routing,
                                                              int64_t token_stride, int64_t slot_stride,
                                                              int T, int E, int units, int nbits,
                                                              const int32_t* __restrict__ unit_hist,
                                                              const int32_t* __restrict__ offsets,
                                                              int64_t offsets_slot_stride,
                                                              int32_t* __restrict__ token_ids,
                                                              int32_t* __restrict__ expert_ids,
                                                              int64_t list_stride) {
    extern __shared__ int32_t cursor[];
    route_scatter_body<IdxT>(cursor, blockIdx.x, blockIdx.y, kUnit, routing, token_stride, slot_stride, T, E, units, nbits,
                             unit_hist, offsets, offsets_slot_stride, token_ids, expert_ids, list_stride);
}

// The scatter over units of `unit_tokens` tokens of a [T][k] int32 routing table and, in one more workgroup of the
// same launch (x = units, y = 0), the work plan of the balanced ESTMM, which needs nothing but the offsets.
__global__ __launch_bounds__(kWave) void route_scatter_plan_kernel(const int32_t* __restrict__ routing, int k, int T, int E,
                                                                   int units, int unit_tokens, int nbits,
                                                                   const int32_t* __restrict__ unit_hist,
                                                                   const int32_t* __restrict__ offsets,
                                                                   int32_t* __restrict__ token_ids,
                                                                   int32_t* __restrict__ expert_ids,
                                                                   int32_t* __restrict__ plan, int plan_cap,
                                                                   int plan_slots) {
    extern __shared__ int32_t cursor[];
    if ((int)blockIdx.x < units) {
        route_scatter_body<int32_t>(cursor, blockIdx.x, blockIdx.y, unit_tokens, routing, k, 1, T, E, units, nbits, unit_hist,
                                    offsets, E + 1, token_ids, expert_ids, T);
    } else if (blockIdx.y == 0 && plan) {
        estmm_plan_body(cursor, plan, offsets, E, k, plan_cap, plan_slots);
    }
}

// Per expert, the raw per-unit counts H[u][e] summed over all units (tot) and over the units before u_split (pre,
// may be null).  E <= 256, 256 threads.  With E a multiple of 4 a thread loads four experts' counts at once and
// 1024 / E thread groups share the units (group j takes the units j, j + G, ...: nine 16-byte loads per thread, all
// in flight, for 288 units of 32 experts); otherwise 256 / E groups load single counts, sixteen in flight at a time.
// The partial sums meet in LDS.  part: 2048 ints, tot / pre: E ints each, all LDS; H 16-byte aligned.
__device__ __forceinline__ void unit_sums(const int32_t* __restrict__ H, int E, int units, int u_split, int32_t* part,
                                          int32_t* tot, int32_t* pre) {
    const int tid = threadIdx.x;
    if ((E & 3) == 0) {
        const int E4 = E >> 2, G = 256 / E4;
        const int e4 = tid % E4, j = tid / E4;
        int4 t = make_int4(0, 0, 0, 0), q = t;
        if (j < G) {
            const int4* H4 = reinterpret_cast<const int4*>(H);
            for (int u0 = j; u0 < units; u0 += 16 * G) {
                int4 v[16];
#pragma unroll
                for (int i = 0; i < 16; ++i)
                    v[i] = u0 + i * G < units ? H4[(size_t)(u0 + i * G) * E4 + e4] : make_int4(0, 0, 0, 0);
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    t.x += v[i].x; t.y += v[i].y; t.z += v[i].z; t.w += v[i].w;
                    if (u0 + i * G < u_split) { q.x += v[i].x; q.y += v[i].y; q.z += v[i].z; q.w += v[i].w; }
                }
            }
        }
        reinterpret_cast<int4*>(part)[tid] = t;            // group j, experts 4 e4 .. 4 e4 + 3 at part[(j E4 + e4) 4 ..]
        reinterpret_cast<int4*>(part)[256 + tid] = q;
        __syncthreads();
        if (tid < E) {
            int a = 0, b = 0;
            for (int g = 0; g < G; ++g) { a += part[g * E + tid]; b += part[1024 + g * E + tid]; }
            tot[tid] = a;
            if (pre) pre[tid] = b;
        }
        __syncthreads();
        return;
    }
    const int G = 256 / E;
    const int e = tid % E, j = tid / E;
    int t = 0, q = 0;
    if (j < G) {
        for (int u0 = j; u0 < units; u0 += 16 * G) {
            int v[16];
#pragma unroll
            for (int i = 0; i < 16; ++i) v[i] = u0 + i * G < units ? H[(size_t)(u0 + i * G) * E + e] : 0;
#pragma unroll
            for (int i = 0; i < 16; ++i) { t += v[i]; q += u0 + i * G < u_split ? v[i] : 0; }
        }
    }
    part[tid] = t;
    part[1024 + tid] = q;
    __syncthreads();
    if (tid < E) {
        int a = 0, b = 0;
        for (int g = 0; g < G; ++g) { a += part[g * E + tid]; b += part[1024 + g * E + tid]; }
        tot[tid] = a;
        if (pre) pre[tid] = b;
    }
    __syncthreads();
}

// Everything behind the router's per-unit histogram (raw counts, hist [k][units][E], E <= 256) in ONE launch of
// 256-thread workgroups:
//   [0, units * k)   scatter of one unit of one slot: the workgroup adds up the counts of the units before its own and
//                    of all units itself (the histogram is a few tens of KB in L2), scans the experts and scatters
//   the next k       one per slot: totals, offsets, counts, row-tile records
//   then             the GShard loss from the router's partial sums (when l_aux is given)
//   then             the ESTMM work plan (when plan is given), from the totals of all slots
// No workgroup reads what another one of the launch writes, and the histogram is left as it was.
template <typename IdxT>
__global__ __launch_bounds__(256) void route_finish_kernel(const IdxT* __restrict__ routing, int64_t token_stride,
                                                           int64_t slot_stride, int k, int T, int E, int units,
                                                           int unit_tokens, int nbits, const int32_t* __restrict__ unit_hist,
                                                           int32_t* __restrict__ counts, int32_t* __restrict__ offsets,
                                                           int4* __restrict__ tile_info, int32_t* __restrict__ tile_count,
                                                           int mt_ub, int4* __restrict__ tile_info_l,
                                                           int32_t* __restrict__ tile_count_l, int mt_ub_l,
                                                           int32_t* __restrict__ token_ids, int32_t* __restrict__ expert_ids,
                                                           float* __restrict__ l_aux, float* __restrict__ me,
                                                           float* __restrict__ ce, const float* __restrict__ part_me,
                                                           const float* __restrict__ part_cnt,
                                                           int32_t* __restrict__ plan, int plan_cap, int plan_slots) {
    extern __shared__ int32_t sh[];
    __shared__ __attribute__((aligned(16))) int32_t part[2048];
    const int b = blockIdx.x, tid = threadIdx.x;
    const int n_scatter = units * k;
    if (b < n_scatter) {
        const int unit = b % units, s = b / units;
        int32_t* tot = sh;                // E
        int32_t* pre = tot + E;           // E
        int32_t* off = pre + E;           // E + 1
        int32_t* cursor = off + (E + 1);  // E
        int* tmp = cursor + E;            // 16
        unit_sums(unit_hist + (size_t)s * units * E, E, units, unit, part, tot, pre);
        scan_offsets(tot, off, tmp, E, 1);
        for (int e = tid; e < E; e += 256) cursor[e] = off[e] + pre[e];
        __syncthreads();
        route_scatter_loop<IdxT>(cursor, tid < kWave, unit, s, unit_tokens, routing, token_stride, slot_stride, T, E, nbits,
                                 token_ids, expert_ids, T);
        return;
    }
    if (b < n_scatter + k) {
        const int s = b - n_scatter;
        int32_t* tot = sh;                // the layout of route_scan_body
        int32_t* off = tot + E;
        int32_t* tbase = off + (E + 1);
        int* tmp = tbase + (E + 1);
        unit_sums(unit_hist + (size_t)s * units * E, E, units, units, part, tot, nullptr);
        finish_slot(tot, off, tbase, tmp, E, 1, counts + (size_t)s * E, offsets + (size_t)s * (E + 1),
                    tile_info + (size_t)s * mt_ub, tile_count + s, mt_ub, tile_info_l + (size_t)s * mt_ub_l, tile_count_l + s,
                    mt_ub_l);
        return;
    }
    if (l_aux && b == n_scatter + k) {
        router_loss_body(reinterpret_cast<float*>(sh), l_aux, me, ce, part_me, part_cnt, units, T, E);
        return;
    }
    if (plan) {
        int32_t* load = sh;               // 2 * E for the plan, then E of totals
        int32_t* tot = sh + 2 * E;
        for (int e = tid; e < E; e += 256) load[e] = 0;
        __syncthreads();
        for (int s = 0; s < k; ++s) {
            unit_sums(unit_hist + (size_t)s * units * E, E, units, units, part, tot, nullptr);
            if (tid < E) load[tid] += tot[tid];
            __syncthreads();
        }
        estmm_plan_from_loads(load, plan, E, plan_cap, plan_slots);
    }
}

// offsets from a list sorted by expert: lower bounds by binary search, then the same finish.
__global__ __launch_bounds__(256) void route_from_lists_kernel(const int32_t* __restrict__ expert_idx_list,
                                                               int T, int E, int32_t* __restrict__ counts,
                                                               int32_t* __restrict__ offsets,
                                                               int4* __restrict__ tile_info,
                                                               int32_t* __restrict__ tile_count, int mt_ub,
                                                               int4* __restrict__ tile_info_l,
                                                               int32_t* __restrict__ tile_count_l, int mt_ub_l) {
    extern __shared__ int32_t sh[];
    int32_t* tot = sh;
    int32_t* off = tot + E;
    int32_t* tbase = off + (E + 1);
    int* tmp = tbase + (E + 1);
    const int s = blockIdx.x;
    const int32_t* L = expert_idx_list + (size_t)s * T;
    for (int e = threadIdx.x; e < E; e += 256) {
        int lo = 0, hi = T;  // first position with L[pos] >= e
        while (lo < hi) { int mid = (lo + hi) >> 1; if (L[mid] < e) lo = mid + 1; else hi = mid; }
        int lb = lo;
        lo = lb; hi = T;     // first position with L[pos] > e
        while (lo < hi) { int mid = (lo + hi) >> 1; if (L[mid] <= e) lo = mid + 1; else hi = mid; }
        tot[e] = lo - lb;
    }
    __syncthreads();
    finish_slot(tot, off, tbase, tmp, E, 1, counts + (size_t)s * E, offsets + (size_t)s * (E + 1),
                tile_info + (size_t)s * mt_ub, tile_count + s, mt_ub, tile_info_l + (size_t)s * mt_ub_l,
                tile_count_l + s, mt_ub_l);
}

// Padded lists -> exact lists.  One workgroup per slot walks the slot's stretch of the concatenated
// lists ([slot_ends[s], slot_ends[s+1]) ) and keeps, in order, every entry whose token id is in range;
// fillers (-1) drop out.  Positions past the last kept entry get token -1 / expert E, which the
// operators never visit (they sit beyond offsets[E]).
__global__ __launch_bounds__(1024) void route_compact_kernel(const int32_t* __restrict__ tok_in,
                                                             const int32_t* __restrict__ exp_in,
                                                             const int32_t* __restrict__ slot_ends, int64_t list_len,
                                                             int T, int E, int32_t* __restrict__ tok_out,
                                                             int32_t* __restrict__ exp_out) {
    __shared__ int wave_tot[16];
    __shared__ int base_sh;
    const int s = blockIdx.x, lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    int64_t begin = slot_ends[s], end = slot_ends[s + 1];
    if (begin < 0) begin = 0;
    if (end > list_len) end = list_len;
    int32_t* to = tok_out + (size_t)s * T;
    int32_t* eo = exp_out + (size_t)s * T;
    if (threadIdx.x == 0) base_sh = 0;
    __syncthreads();
    for (int64_t c = begin; c < end; c += 1024) {
        const int64_t i = c + threadIdx.x;
        int32_t t = -1, e = 0;
        if (i < end) { t = tok_in[i]; e = exp_in[i]; }
        const bool keep = t >= 0 && t < T && e >= 0 && e < E;
        const unsigned long long m = __ballot(keep);
        if (lane == 0) wave_tot[wv] = __popcll(m);
        __syncthreads();
        int before = base_sh;
        for (int w = 0; w < wv; ++w) before += wave_tot[w];
        const int pos = before + __popcll(m & ((1ull << lane) - 1));
        if (keep && pos < T) { to[pos] = t; eo[pos] = e; }
        __syncthreads();
        if (threadIdx.x == 0) { int tot = 0; for (int w = 0; w < 16; ++w) tot += wave_tot[w]; base_sh += tot; }
        __syncthreads();
    }
    for (int p = base_sh + threadIdx.x; p < T; p += 1024) { to[p] = -1; eo[p] = E; }
}

// ---- the whole pass in one launch, for token counts that one workgroup per slot can walk -------------------
// 16 wavefronts per slot; wavefront w owns the w-th contiguous sixteenth of the tokens.  Count (private LDS
// histogram per wavefront), prefix over the wavefronts, the same finish as above, then every wavefront
// scatters its own range with the ballot ranking of route_scatter_kernel and its own cursors.  Loads go
// eight steps at a time so that the memory latency is paid once per batch.
constexpr int kOneWaves = 16;
constexpr int kOneMaxE = 256;
// Measured (E = 32): 10 us against 15 us for the three launches up to 4608 tokens, equal at 9216, slower beyond
// (a wavefront walks T/16 tokens serially).
constexpr int kOneMaxT = 8192;

template <typename IdxT>
__global__ __launch_bounds__(64 * kOneWaves) void route_one_kernel(const IdxT* __restrict__ routing,
                                                                   int64_t token_stride, int64_t slot_stride, int T,
                                                                   int E, int nbits, int32_t* __restrict__ counts,
                                                                   int32_t* __restrict__ offsets,
                                                                   int32_t* __restrict__ token_ids,
                                                                   int32_t* __restrict__ expert_ids,
                                                                   int4* __restrict__ tile_info,
                                                                   int32_t* __restrict__ tile_count, int mt_ub,
                                                                   int4* __restrict__ tile_info_l,
                                                                   int32_t* __restrict__ tile_count_l, int mt_ub_l) {
    extern __shared__ int32_t sh[];
    int32_t* wh = sh;                            // [kOneWaves][E]: counts, then prefixes, then cursors
    int32_t* tot = wh + kOneWaves * E;
    int32_t* off = tot + E;
    int32_t* tbase = off + (E + 1);
    int* tmp = tbase + (E + 1);
    const int s = blockIdx.x, tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int chunk = ((T + kOneWaves - 1) / kOneWaves + 63) & ~63;
    const int t0 = min(T, wave * chunk), t1 = min(T, t0 + chunk);
    const IdxT* src = routing + (int64_t)s * slot_stride;
    int32_t* mine = wh + wave * E;
    for (int i = tid; i < kOneWaves * E; i += blockDim.x) wh[i] = 0;
    __syncthreads();
    for (int base = t0; base < t1; base += 64 * 8) {
        long e[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int t = base + 64 * u + lane;
            e[u] = (long)src[(int64_t)min(t, T - 1) * token_stride];
            if (t >= t1) e[u] = -1;
        }
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (e[u] >= 0 && e[u] < E) atomicAdd(&mine[e[u]], 1);
    }
    __syncthreads();
    for (int x = tid; x < E; x += blockDim.x) {
        int run = 0;
        for (int w = 0; w < kOneWaves; ++w) { const int c = wh[w * E + x]; wh[w * E + x] = run; run += c; }
        tot[x] = run;
    }
    __syncthreads();
    finish_slot(tot, off, tbase, tmp, E, 1, counts + (size_t)s * E, offsets + (size_t)s * (E + 1),
                tile_info + (size_t)s * mt_ub, tile_count + s, mt_ub, tile_info_l + (size_t)s * mt_ub_l,
                tile_count_l + s, mt_ub_l);
    for (int i = tid; i < kOneWaves * E; i += blockDim.x) wh[i] += off[i % E];
    __syncthreads();
    const unsigned long long lt_mask = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
    int32_t* tok = token_ids + (size_t)s * T;
    int32_t* exp = expert_ids + (size_t)s * T;
    for (int base = t0; base < t1; base += 64 * 8) {
        long e[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int t = base + 64 * u + lane;
            e[u] = (long)src[(int64_t)min(t, T - 1) * token_stride];
            if (t >= t1) e[u] = -1;
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            if (base + 64 * u >= t1) break;                      // uniform over the wavefront
            const int t = base + 64 * u + lane;
            const bool valid = e[u] >= 0 && e[u] < E;
            unsigned long long peers = __ballot(valid);
            for (int b = 0; b < nbits; ++b) {
                const bool bit = (e[u] >> b) & 1;
                const unsigned long long m = __ballot(valid && bit);
                peers &= bit ? m : ~m;
            }
            // only this wavefront touches its cursors, and a wavefront's LDS accesses complete in order
            if (valid) {
                const int pos = mine[e[u]] + __popcll(peers & lt_mask);
                tok[pos] = t;
                exp[pos] = (int32_t)e[u];
            }
            __builtin_amdgcn_wave_barrier();
            if (valid && (peers & lt_mask) == 0) mine[e[u]] += __popcll(peers);   // first lane of its group
            __builtin_amdgcn_wave_barrier();
        }
    }
}

size_t one_lds_bytes(int E) { return sizeof(int32_t) * (size_t)(kOneWaves * E + E + 2 * (E + 1) + 16); }

int ceil_log2(int n) { int b = 0; while ((1 << b) < n) ++b; return b; }

size_t scan_lds_bytes(int E) { return sizeof(int32_t) * (size_t)(E + 2 * (E + 1) + 16); }

}  // namespace
}  // namespace hexa

using namespace hexa;

extern "C" int hexa_route_layout_get(int T, int k, int E, hexa_route_layout* out) {
    if (!out) HEXA_FAIL(HEXA_ERR_ARG, "hexa_route_layout_get: null layout");
    if (T < 0 || k < 1 || E < 1) HEXA_FAIL(HEXA_ERR_ARG, "hexa_route_layout_get: bad sizes T=%d k=%d E=%d", T, k, E);
    const int64_t K = k;
    out->mt_ub = T / HEXA_TILE_ROWS + E;
    out->mt_ub_l = T / HEXA_TILE_ROWS_L + E;
    out->reserved = 0;
    out->units = T > 0 ? div_up(T, HEXA_ROUTE_UNIT) : 1;
    int64_t p = 0;
    out->counts = p;      p += K * E;
    out->offsets = p;     p += K * (E + 1);
    out->token_ids = p;   p += K * T;
    out->expert_ids = p;  p += K * T;
    out->tile_count = p;  p += K;
    p = (p + 3) & ~(int64_t)3;  // tile records are 16-byte vectors
    out->tile_info = p;   p += K * out->mt_ub * 4;
    out->tile_count_l = p; p += K;
    p = (p + 3) & ~(int64_t)3;
    out->tile_info_l = p; p += K * out->mt_ub_l * 4;
    out->scratch = p;     p += K * out->units * E;
    out->total_ints = p;
    return HEXA_OK;
}

namespace hexa {
RouteView route_view(const int32_t* route, int T, int k, int E) {
    hexa_route_layout L;
    hexa_route_layout_get(T, k, E, &L);
    RouteView v;
    v.token_ids = route + L.token_ids;
    v.offsets = route + L.offsets;
    v.tile_info = reinterpret_cast<const int4*>(route + L.tile_info);
    v.tile_count = route + L.tile_count;
    v.tile_info_l = reinterpret_cast<const int4*>(route + L.tile_info_l);
    v.tile_count_l = route + L.tile_count_l;
    v.T = T; v.k = k; v.E = E; v.mt_ub = L.mt_ub; v.mt_ub_l = L.mt_ub_l;
    return v;
}
}  // namespace hexa

namespace hexa {
// The routing pass for a [T][k] int32 table whose histogram over units of `unit_tokens` tokens (hist [k][units][E])
// has been counted already: scan (+ the GShard loss, when l_aux is given, from the router's partial sums in
// router_ws) and scatter (+ the ESTMM work plan, when plan is given).
int launch_route_from_hist(const int32_t* idx, int T, int k, int E, int32_t* route, int32_t* hist, int unit_tokens,
                           float* l_aux, float* me, float* ce, const float* router_ws, int32_t* plan, int plan_slots,
                           int plan_cap, hipStream_t st) {
    hexa_route_layout L;
    hexa_route_layout_get(T, k, E, &L);
    const int units = div_up(T, unit_tokens);
    const size_t loss_lds = l_aux ? sizeof(float) * (2 * (size_t)router_loss_chunks(E) * E + 256) : 0;
    if (E <= 256 && (reinterpret_cast<uintptr_t>(hist) & 15) == 0 && option(OPT_ROUTE_KERNELS) != 3) {   // one launch; the histogram stays as counted
        const size_t lds = std::max({sizeof(int32_t) * (size_t)(4 * E + 1 + 16), scan_lds_bytes(E), loss_lds});
        const int grid = units * k + k + (l_aux ? 1 : 0) + (plan ? 1 : 0);
        hipLaunchKernelGGL(route_finish_kernel<int32_t>, dim3(grid), dim3(256), lds, st, idx, (int64_t)k, (int64_t)1, k, T, E, units,
                           unit_tokens, ceil_log2(E),
                           hist, route + L.counts, route + L.offsets, reinterpret_cast<int4*>(route + L.tile_info),
                           route + L.tile_count, L.mt_ub, reinterpret_cast<int4*>(route + L.tile_info_l), route + L.tile_count_l,
                           L.mt_ub_l, route + L.token_ids, route + L.expert_ids, l_aux, me, ce, router_ws,
                           router_ws ? router_ws + (size_t)units * E : nullptr, plan, plan_cap, plan_slots);
        HEXA_CHECK_LAUNCH("route_finish");
        return HEXA_OK;
    }
    hipLaunchKernelGGL(route_scan_loss_kernel, dim3(k + (l_aux ? 1 : 0)), dim3(256), std::max(scan_lds_bytes(E), loss_lds), st,
                       hist, E, units, k, route + L.counts, route + L.offsets, reinterpret_cast<int4*>(route + L.tile_info),
                       route + L.tile_count, L.mt_ub, reinterpret_cast<int4*>(route + L.tile_info_l), route + L.tile_count_l,
                       L.mt_ub_l, l_aux, me, ce, router_ws, router_ws ? router_ws + (size_t)units * E : nullptr, units, T);
    HEXA_CHECK_LAUNCH("route_scan_loss");
    hipLaunchKernelGGL(route_scatter_plan_kernel, dim3(units + (plan ? 1 : 0), k), dim3(kWave), sizeof(int32_t) * 2 * E, st, idx,
                       k, T, E, units, unit_tokens, ceil_log2(E), hist, route + L.offsets, route + L.token_ids,
                       route + L.expert_ids, plan, plan_cap, plan_slots);
    HEXA_CHECK_LAUNCH("route_scatter_plan");
    return HEXA_OK;
}
}  // namespace hexa

static int check_route_sizes(const char* who, int T, int k, int E) {
    if (T < 0 || k < 1 || E < 1) HEXA_FAIL(HEXA_ERR_ARG, "%s: bad sizes T=%d k=%d E=%d", who, T, k, E);
    if (E > 8192) HEXA_FAIL(HEXA_ERR_UNSUPPORTED, "%s: more than 8192 experts (E=%d)", who, E);
    return HEXA_OK;
}

extern "C" int hexa_route_build(const void* routing, int routing_is_i64, int64_t token_stride, int64_t slot_stride,
                                int T, int k, int E, int32_t* route, void* stream) {
    if (int rc = check_route_sizes("hexa_route_build", T, k, E)) return rc;
    if (!route || (T > 0 && !routing)) HEXA_FAIL(HEXA_ERR_ARG, "hexa_route_build: null pointer");
    if (((uintptr_t)route & 15) != 0) HEXA_FAIL(HEXA_ERR_ARG, "hexa_route_build: route blob must be 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    hexa_route_layout L;
    hexa_route_layout_get(T, k, E, &L);
    const int nbits = ceil_log2(E);
    const bool one = option(OPT_ROUTE_KERNELS) == 1 ? T <= kOneWaves * 4096 : (option(OPT_ROUTE_KERNELS) != 3 && T <= kOneMaxT);
    if (T > 0 && one && E <= kOneMaxE) {
        // one workgroup per slot does the whole pass
        int4* ti = reinterpret_cast<int4*>(route + L.tile_info);
        int4* til = reinterpret_cast<int4*>(route + L.tile_info_l);
        if (routing_is_i64)
            hipLaunchKernelGGL(route_one_kernel<int64_t>, dim3(k), dim3(64 * kOneWaves), one_lds_bytes(E), st,
                               (const int64_t*)routing, token_stride, slot_stride, T, E, nbits, route + L.counts,
                               route + L.offsets, route + L.token_ids, route + L.expert_ids, ti, route + L.tile_count,
                               L.mt_ub, til, route + L.tile_count_l, L.mt_ub_l);
        else
            hipLaunchKernelGGL(route_one_kernel<int32_t>, dim3(k), dim3(64 * kOneWaves), one_lds_bytes(E), st,
                               (const int32_t*)routing, token_stride, slot_stride, T, E, nbits, route + L.counts,
                               route + L.offsets, route + L.token_ids, route + L.expert_ids, ti, route + L.tile_count,
                               L.mt_ub, til, route + L.tile_count_l, L.mt_ub_l);
        HEXA_CHECK_LAUNCH("route_one");
        return HEXA_OK;
    }
    int32_t* H = route + L.scratch;
    dim3 grid(L.units, k);
    if (routing_is_i64)
        hipLaunchKernelGGL(route_hist_kernel<int64_t>, grid, dim3(kWave), sizeof(int32_t) * E, st,
                           (const int64_t*)routing, token_stride, slot_stride, T, E, L.units, H);
    else
        hipLaunchKernelGGL(route_hist_kernel<int32_t>, grid, dim3(kWave), sizeof(int32_t) * E, st,
                           (const int32_t*)routing, token_stride, slot_stride, T, E, L.units, H);
    HEXA_CHECK_LAUNCH("route_hist");
    if (E <= 256 && option(OPT_ROUTE_KERNELS) != 3) {
        // scan and scatter in one launch: every scatter workgroup derives its cursors from the raw histogram
        const size_t lds = std::max(sizeof(int32_t) * (size_t)(4 * E + 1 + 16), scan_lds_bytes(E));
        const int nwg = L.units * k + k;
        int4* ti = reinterpret_cast<int4*>(route + L.tile_info);
        int4* til = reinterpret_cast<int4*>(route + L.tile_info_l);
        if (routing_is_i64)
            hipLaunchKernelGGL(route_finish_kernel<int64_t>, dim3(nwg), dim3(256), lds, st, (const int64_t*)routing, token_stride,
                               slot_stride, k, T, E, L.units, kUnit, nbits, H, route + L.counts, route + L.offsets, ti,
                               route + L.tile_count, L.mt_ub, til, route + L.tile_count_l, L.mt_ub_l, route + L.token_ids,
                               route + L.expert_ids, (float*)nullptr, (float*)nullptr, (float*)nullptr, (const float*)nullptr,
                               (const float*)nullptr, (int32_t*)nullptr, 0, 0);
        else
            hipLaunchKernelGGL(route_finish_kernel<int32_t>, dim3(nwg), dim3(256), lds, st, (const int32_t*)routing, token_stride,
                               slot_stride, k, T, E, L.units, kUnit, nbits, H, route + L.counts, route + L.offsets, ti,
                               route + L.tile_count, L.mt_ub, til, route + L.tile_count_l, L.mt_ub_l, route + L.token_ids,
                               route + L.expert_ids, (float*)nullptr, (float*)nullptr, (float*)nullptr, (const float*)nullptr,
                               (const float*)nullptr, (int32_t*)nullptr, 0, 0);
        HEXA_CHECK_LAUNCH("route_finish");
        return HEXA_OK;
    }
    hipLaunchKernelGGL(route_scan_kernel, dim3(k), dim3(256), scan_lds_bytes(E), st, H, E, L.units, 1,
                       route + L.counts, route + L.offsets, reinterpret_cast<int4*>(route + L.tile_info),
                       route + L.tile_count, L.mt_ub, reinterpret_cast<int4*>(route + L.tile_info_l),
                       route + L.tile_count_l, L.mt_ub_l, 0);
    HEXA_CHECK_LAUNCH("route_scan");
    if (routing_is_i64)
        hipLaunchKernelGGL(route_scatter_kernel<int64_t>, grid, dim3(kWave), sizeof(int32_t) * E, st,
                           (const int64_t*)routing, token_stride, slot_stride, T, E, L.units, nbits, H,
                           route + L.offsets, (int64_t)(E + 1), route + L.token_ids, route + L.expert_ids,
                           (int64_t)T);
    else
        hipLaunchKernelGGL(route_scatter_kernel<int32_t>, grid, dim3(kWave), sizeof(int32_t) * E, st,
                           (const int32_t*)routing, token_stride, slot_stride, T, E, L.units, nbits, H,
                           route + L.offsets, (int64_t)(E + 1), route + L.token_ids, route + L.expert_ids,
                           (int64_t)T);
    HEXA_CHECK_LAUNCH("route_scatter");
    return HEXA_OK;
}

extern "C" int hexa_token_count(int32_t* tokens_per_expert, int32_t* expanded, const int32_t* routing, int T, int E,
                                int pad, int32_t* scratch, void* stream) {
    if (int rc = check_route_sizes("hexa_token_count", T, 1, E)) return rc;
    if (!tokens_per_expert || !expanded || !scratch || (T > 0 && !routing))
        HEXA_FAIL(HEXA_ERR_ARG, "hexa_token_count: null pointer");
    if (pad < 1) HEXA_FAIL(HEXA_ERR_ARG, "hexa_token_count: pad must be >= 1 (got %d)", pad);
    hipStream_t st = (hipStream_t)stream;
    const int units = T > 0 ? div_up(T, HEXA_ROUTE_UNIT) : 1;
    hipLaunchKernelGGL(route_hist_kernel<int32_t>, dim3(units, 1), dim3(kWave), sizeof(int32_t) * E, st, routing,
                       (int64_t)1, (int64_t)0, T, E, units, scratch);
    HEXA_CHECK_LAUNCH("route_hist");
    hipLaunchKernelGGL(route_scan_kernel, dim3(1), dim3(256), scan_lds_bytes(E), st, scratch, E, units, pad,
                       tokens_per_expert, expanded, (int4*)nullptr, (int32_t*)nullptr, 0, (int4*)nullptr,
                       (int32_t*)nullptr, 0, 0);
    HEXA_CHECK_LAUNCH("route_scan");
    return HEXA_OK;
}

extern "C" int hexa_token_assign(int32_t* token_idx_list, int32_t* expert_idx_list, const int32_t* expanded,
                                 const int32_t* routing, int T, int E, int32_t* scratch, void* stream) {
    if (int rc = check_route_sizes("hexa_token_assign", T, 1, E)) return rc;
    if (!token_idx_list || !expert_idx_list || !expanded || !scratch || (T > 0 && !routing))
        HEXA_FAIL(HEXA_ERR_ARG, "hexa_token_assign: null pointer");
    hipStream_t st = (hipStream_t)stream;
    const int units = T > 0 ? div_up(T, HEXA_ROUTE_UNIT) : 1;
    hipLaunchKernelGGL(route_hist_kernel<int32_t>, dim3(units, 1), dim3(kWave), sizeof(int32_t) * E, st, routing,
                       (int64_t)1, (int64_t)0, T, E, units, scratch);
    HEXA_CHECK_LAUNCH("route_hist");
    hipLaunchKernelGGL(route_scan_kernel, dim3(1), dim3(256), scan_lds_bytes(E), st, scratch, E, units, 1,
                       (int32_t*)nullptr, (int32_t*)nullptr, (int4*)nullptr, (int32_t*)nullptr, 0, (int4*)nullptr,
                       (int32_t*)nullptr, 0, 1);
    HEXA_CHECK_LAUNCH("route_scan");
    hipLaunchKernelGGL(route_scatter_kernel<int32_t>, dim3(units, 1), dim3(kWave), sizeof(int32_t) * E, st, routing,
                       (int64_t)1, (int64_t)0, T, E, units, ceil_log2(E), scratch, expanded, (int64_t)0,
                       token_idx_list, expert_idx_list, (int64_t)0);
    HEXA_CHECK_LAUNCH("route_scatter");
    return HEXA_OK;
}

extern "C" int hexa_route_from_lists(const int32_t* token_idx_list, const int32_t* expert_idx_list, int T, int k,
                                     int E, int32_t* route, void* stream) {
    if (int rc = check_route_sizes("hexa_route_from_lists", T, k, E)) return rc;
    if (!route || (T > 0 && (!token_idx_list || !expert_idx_list)))
        HEXA_FAIL(HEXA_ERR_ARG, "hexa_route_from_lists: null pointer");
    if (((uintptr_t)route & 15) != 0) HEXA_FAIL(HEXA_ERR_ARG, "hexa_route_from_lists: route blob must be 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    hexa_route_layout L;
    hexa_route_layout_get(T, k, E, &L);
    if (T > 0) {
        hipError_t e1 = hipMemcpyAsync(route + L.token_ids, token_idx_list, sizeof(int32_t) * (size_t)k * T,
                                       hipMemcpyDeviceToDevice, st);
        hipError_t e2 = hipMemcpyAsync(route + L.expert_ids, expert_idx_list, sizeof(int32_t) * (size_t)k * T,
                                       hipMemcpyDeviceToDevice, st);
        if (e1 != hipSuccess || e2 != hipSuccess) HEXA_FAIL(HEXA_ERR_LAUNCH, "hexa_route_from_lists: copy failed");
    }
    hipLaunchKernelGGL(route_from_lists_kernel, dim3(k), dim3(256), scan_lds_bytes(E), st, expert_idx_list, T, E,
                       route + L.counts, route + L.offsets, reinterpret_cast<int4*>(route + L.tile_info),
                       route + L.tile_count, L.mt_ub, reinterpret_cast<int4*>(route + L.tile_info_l),
                       route + L.tile_count_l, L.mt_ub_l);
    HEXA_CHECK_LAUNCH("route_from_lists");
    return HEXA_OK;
}

extern "C" int hexa_route_from_padded_lists(const int32_t* token_idx_list, const int32_t* expert_idx_list,
                                            const int32_t* slot_ends, int64_t list_len, int T, int k, int E,
                                            int32_t* route, void* stream) {
    if (int rc = check_route_sizes("hexa_route_from_padded_lists", T, k, E)) return rc;
    if (!route || !slot_ends || list_len < 0 || (list_len > 0 && (!token_idx_list || !expert_idx_list)))
        HEXA_FAIL(HEXA_ERR_ARG, "hexa_route_from_padded_lists: bad arguments");
    if (((uintptr_t)route & 15) != 0)
        HEXA_FAIL(HEXA_ERR_ARG, "hexa_route_from_padded_lists: route blob must be 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    hexa_route_layout L;
    hexa_route_layout_get(T, k, E, &L);
    hipLaunchKernelGGL(route_compact_kernel, dim3(k), dim3(1024), 0, st, token_idx_list, expert_idx_list, slot_ends,
                       list_len, T, E, route + L.token_ids, route + L.expert_ids);
    HEXA_CHECK_LAUNCH("route_compact");
    hipLaunchKernelGGL(route_from_lists_kernel, dim3(k), dim3(256), scan_lds_bytes(E), st, route + L.expert_ids, T, E,
                       route + L.counts, route + L.offsets, reinterpret_cast<int4*>(route + L.tile_info),
                       route + L.tile_count, L.mt_ub, reinterpret_cast<int4*>(route + L.tile_info_l),
                       route + L.tile_count_l, L.mt_ub_l);
    HEXA_CHECK_LAUNCH("route_from_lists");
    return HEXA_OK;
}
