// Routing front end for gfx950: softmax + top-k + GShard auxiliary loss, and the loss's backward
// through the softmax (the gate projection itself is in gate.hip).  These are small HBM-/latency-bound kernels that replace a
// dozen framework launches per MoE depth (fp32 cast, a skinny fp32 GEMM, softmax, top-k select + sort,
// one-hot scatter, reductions).
//
// Reference: hexa_moe_cuda/hexa_moe/gates/top.py:17-19 (fp32 gate projection),
//            hexa_moe_cuda/hexa_moe/impls/cascaded_moe.py:515-531 (noise, softmax, loss selection),
//            hexa_moe_cuda/hexa_moe/impls/layers.py:476-484 (top-k), impls/losses.py:12-19 (GShard loss).
#include "hexa_internal.h"
#include "small_bodies.h"
#include "gate_bodies.h"

namespace hexa {
namespace {

// ---- softmax + top-k + per-workgroup loss partials ----------------------------------------------------
// One token per lane, three passes over its logits row (max, sum of exp, scores + selection); the row
// is tiny (E floats) and stays in L1/L2.  Ties go to the lower expert index.
constexpr int MAX_TOPK = 8;

constexpr int ROUTER_TB = 64;   // tokens (= lanes) per workgroup of the softmax/top-k kernel

constexpr int ROUTER_LDS_E = 240;   // up to this many experts the workgroup's 64 x E tile is staged in LDS

// insertion of (cv, ci) into a descending list of k entries; strict '>' keeps the lower index on ties
__device__ __forceinline__ void topk_insert(float (&best_v)[MAX_TOPK], int (&best_i)[MAX_TOPK], int k, float cv, int ci) {
#pragma unroll
    for (int j = 0; j < MAX_TOPK; ++j) {
        if (j < k && cv > best_v[j]) {
            const float tv = best_v[j]; const int ti = best_i[j];
            best_v[j] = cv; best_i[j] = ci; cv = tv; ci = ti;
        }
    }
}

// One token per lane for any number of experts: every lane walks its own row in global memory (three passes,
// L1-resident) and the per-expert sums are wavefront reductions.  Used above ROUTER_LDS_E experts.
__global__ __launch_bounds__(ROUTER_TB) void router_fwd_kernel(float* __restrict__ scores, int32_t* __restrict__ idx,
                                                         float* __restrict__ part_me, float* __restrict__ part_cnt,
                                                         const float* __restrict__ logits,
                                                         const float* __restrict__ noise, float noise_scale,
                                                         int num_tokens, int E, int k) {
    extern __shared__ float sh[];          // me[E] column sums of the wavefront, cnt[E]
    float* s_me = sh;
    float* s_cnt = sh + E;
    for (int i = threadIdx.x; i < 2 * E; i += blockDim.x) sh[i] = 0.f;
    const int lane = threadIdx.x;
    const int t = blockIdx.x * ROUTER_TB + lane;
    const bool ok = t < num_tokens;
    __syncthreads();
    // The selection is total: a row of NaN scores (NaN or +Inf logits) beats no entry, so the list starts out
    // as experts 0..k-1 and such a token stays routed (torch.topk also returns valid ids for NaN rows); its
    // NaN then reaches the output through the token's own features and the loss through the score sums.
    float best_v[MAX_TOPK];
    int best_i[MAX_TOPK];
#pragma unroll
    for (int j = 0; j < MAX_TOPK; ++j) { best_v[j] = -INFINITY; best_i[j] = j; }
    const float* lr = logits + (size_t)(ok ? t : 0) * E;
    const float* nr = noise ? noise + (size_t)(ok ? t : 0) * E : nullptr;
    float mx = -INFINITY;
    for (int e = 0; e < E; ++e) mx = fmaxf(mx, nr ? lr[e] + noise_scale * nr[e] : lr[e]);
    float sum = 0.f;
    for (int e = 0; e < E; ++e) sum += expf((nr ? lr[e] + noise_scale * nr[e] : lr[e]) - mx);
    const float inv = 1.0f / sum;
    for (int e = 0; e < E; ++e) {        // uniform trip count: every lane takes part in the reductions
        const float v = nr ? lr[e] + noise_scale * nr[e] : lr[e];
        const float sc = ok ? expf(v - mx) * inv : 0.f;
        if (ok) scores[(size_t)t * E + e] = sc;
        topk_insert(best_v, best_i, k, sc, e);
        // column sum over the wavefront: xor butterfly, a fixed summation tree
        float r = sc;
#pragma unroll
        for (int m = 32; m > 0; m >>= 1) r += __shfl_xor(r, m);
        if (lane == 0) s_me[e] = r;
    }
    if (ok) {
#pragma unroll
        for (int j = 0; j < MAX_TOPK; ++j)
            if (j < k) idx[(size_t)t * k + j] = best_i[j];
        atomicAdd(&s_cnt[best_i[0]], 1.0f);            // exact: at most 64 ones per counter
    }
    __syncthreads();
    for (int e = threadIdx.x; e < E; e += blockDim.x) {
        part_me[(size_t)blockIdx.x * E + e] = s_me[e];
        part_cnt[(size_t)blockIdx.x * E + e] = s_cnt[e];
    }
}

// Up to ROUTER_LDS_E experts: FOUR lanes per token (256 threads for the workgroup's 64 tokens).  One lane per
// token leaves a 64-thread workgroup walking E-long dependent chains (max, exp and sum, selection) on a chip that
// holds a few hundred such workgroups at once -- latency, not work, sets the time (18.8 us against 8.8 us at
// 18432 tokens and 32 experts).  Lane q of a
// token owns the experts e = q, q + 4, ...; maxima, sums and the top-k lists are combined over the four lanes
// with quad shuffles.  The 64 x E tile sits token-major in LDS (pitch 4 x odd: the 64 lanes of a wavefront --
// 16 tokens x 4 -- hit every bank twice, the minimum), is loaded and written back with coalesced 16-byte
// accesses when E is a multiple of 4, and the per-expert sums run over it in token order.
constexpr int ROUTER_G = 4;
__host__ __device__ constexpr int router_pitch(int E) {
    int p = (E + 3) / 4;            // in units of 4 floats
    if ((p & 1) == 0) ++p;
    return 4 * p;
}

// hist (optional): [k][workgroups][E] ints, per slot the number of this workgroup's 64 tokens that chose each expert
// -- the histogram the routing pass starts from (units of 64 tokens), so that pass needs no counting launch.
// LDS of the four-lanes-per-token router: cnt[E], the tile [64][P], then hist[k][E]
struct Router4Lds {
    float* cnt; float* tile; int* hist; int P;
    __device__ __forceinline__ Router4Lds(float* sh, int E) : cnt(sh), tile(sh + ((E + 3) & ~3)), P(router_pitch(E)) {
        hist = reinterpret_cast<int*>(tile + ROUTER_TB * P);
    }
};
__host__ __device__ constexpr size_t router4_lds_floats(int E, int k, bool hist) {
    return (size_t)((E + 3) & ~3) + (size_t)ROUTER_TB * router_pitch(E) + (hist ? (size_t)k * E : 0);
}

// Everything behind the tile of (noisy) logits: softmax, top-k, loss partials, histogram, scores out.  The tile
// holds rows [t0, t0 + rows) of the workgroup; the counters have been cleared; a barrier separates both from here.
// The workgroup has at least ROUTER_TB * ROUTER_G threads.
__device__ __forceinline__ void router4_body(const Router4Lds& L, float* __restrict__ scores, int32_t* __restrict__ idx,
                                             float* __restrict__ part_me, float* __restrict__ part_cnt,
                                             int32_t* __restrict__ hist, int t0, int rows, int E, int k) {
    float* s_cnt = L.cnt;
    float* tile = L.tile;
    int* s_hist = L.hist;
    const int P = L.P;
    const int tid = threadIdx.x;
    const size_t g0 = (size_t)t0 * E;
    const int total = rows * E;
    if (tid < ROUTER_TB * ROUTER_G) {   // four lanes per token; further wavefronts of the workgroup help with the sums only
        const int r = tid >> 2, q = tid & 3;
        const int t = t0 + r;
        const bool ok = r < rows;
        float* row = tile + r * P;
        // The selection is total: a row of NaN scores (NaN or +Inf logits) beats no entry, so the lists start out as
        // the lanes' own experts in index order and such a token ends up with experts 0..k-1 (torch.topk also returns
        // valid ids for NaN rows); its NaN then reaches the output through the token's own features and the loss
        // through the score sums.
        float bv[MAX_TOPK];
        int bi[MAX_TOPK];
    #pragma unroll
        for (int j = 0; j < MAX_TOPK; ++j) { bv[j] = -INFINITY; bi[j] = q + ROUTER_G * j; }
        if (ok) {
            float mx = -INFINITY;
            for (int e = q; e < E; e += ROUTER_G) mx = fmaxf(mx, row[e]);
            mx = fmaxf(mx, __shfl_xor(mx, 1));
            mx = fmaxf(mx, __shfl_xor(mx, 2));
            float sum = 0.f;
            for (int e = q; e < E; e += ROUTER_G) {
                const float ex = expf(row[e] - mx);
                row[e] = ex;
                sum += ex;
            }
            sum += __shfl_xor(sum, 1);         // (s0 + s1) + (s2 + s3) on every lane of the quad
            sum += __shfl_xor(sum, 2);
            const float inv = 1.0f / sum;
            for (int e = q; e < E; e += ROUTER_G) {
                const float sc = row[e] * inv;
                row[e] = sc;
                topk_insert(bv, bi, k, sc, e);  // ascending e, strict '>': the lower index stays ahead on ties
            }
        } else {
            for (int e = q; e < E; e += ROUTER_G) row[e] = 0.f;
        }
        // merge the four lists: k rounds, each takes the best head (greater score; lower index on ties)
        int pick[MAX_TOPK];
    #pragma unroll
        for (int j = 0; j < MAX_TOPK; ++j) {
            pick[j] = 0;
            if (j < k) {
                float hv = bv[0];
                int hi = bi[0];
    #pragma unroll
                for (int m = 1; m <= 2; m <<= 1) {
                    const float ov = __shfl_xor(hv, m);
                    const int oi = __shfl_xor(hi, m);
                    if (ov > hv || (ov == hv && oi < hi)) { hv = ov; hi = oi; }
                }
                pick[j] = hi;
                if (hi == bi[0]) {
    #pragma unroll
                    for (int m = 0; m + 1 < MAX_TOPK; ++m) { bv[m] = bv[m + 1]; bi[m] = bi[m + 1]; }
                    bv[MAX_TOPK - 1] = -INFINITY;
                    bi[MAX_TOPK - 1] = 0x7fffffff;
                }
            }
        }
        if (ok) {
    #pragma unroll
            for (int j = 0; j < MAX_TOPK; ++j)
                if (j < k && (j & 3) == q) {
                    idx[(size_t)t * k + j] = pick[j];
                    if (hist) atomicAdd(&s_hist[j * E + pick[j]], 1);
                }
            if (q == 0) atomicAdd(&s_cnt[pick[0]], 1.0f);   // exact: at most 64 ones per counter
        }
    }
    __syncthreads();
    // per-expert sums over the 64 tokens, in token order; the scores leave coalesced
    for (int e = tid; e < E; e += blockDim.x) {
        float m = 0.f;
#pragma unroll 16
        for (int rr = 0; rr < ROUTER_TB; ++rr) m += tile[rr * P + e];
        part_me[(size_t)blockIdx.x * E + e] = m;
        part_cnt[(size_t)blockIdx.x * E + e] = s_cnt[e];
    }
    if (hist)
        for (int i = tid; i < k * E; i += blockDim.x) {
            const int j = i / E, e = i - j * E;
            hist[((size_t)j * gridDim.x + blockIdx.x) * E + e] = s_hist[i];
        }
    if ((E & 3) == 0) {
        for (int i = tid * 4; i < total; i += blockDim.x * 4) {
            const int rr = i / E, e = i - rr * E;
            *reinterpret_cast<float4*>(scores + g0 + i) = *reinterpret_cast<const float4*>(tile + rr * P + e);
        }
    } else {
        for (int i = tid; i < total; i += blockDim.x) {
            const int rr = i / E, e = i - rr * E;
            scores[g0 + i] = tile[rr * P + e];
        }
    }
}

__global__ __launch_bounds__(ROUTER_TB * ROUTER_G) void router_fwd4_kernel(
    float* __restrict__ scores, int32_t* __restrict__ idx, float* __restrict__ part_me, float* __restrict__ part_cnt,
    const float* __restrict__ logits, const float* __restrict__ noise, float noise_scale, int num_tokens, int E, int k,
    int32_t* __restrict__ hist) {
    extern __shared__ float sh[];
    const Router4Lds L(sh, E);
    const int P = L.P;
    float* tile = L.tile;
    const int tid = threadIdx.x;
    const int t0 = blockIdx.x * ROUTER_TB;
    const int rows = min(ROUTER_TB, num_tokens - t0);
    for (int i = tid; i < E; i += blockDim.x) L.cnt[i] = 0.f;
    if (hist)
        for (int i = tid; i < k * E; i += blockDim.x) L.hist[i] = 0;
    // ---- tile in: element i of the contiguous block [rows][E] ----
    const size_t g0 = (size_t)t0 * E;
    const int total = rows * E;
    if ((E & 3) == 0) {
        for (int i = tid * 4; i < total; i += blockDim.x * 4) {
            float4 v = *reinterpret_cast<const float4*>(logits + g0 + i);
            if (noise) {
                const float4 n = *reinterpret_cast<const float4*>(noise + g0 + i);
                v.x += noise_scale * n.x; v.y += noise_scale * n.y; v.z += noise_scale * n.z; v.w += noise_scale * n.w;
            }
            const int r = i / E, e = i - r * E;
            *reinterpret_cast<float4*>(tile + r * P + e) = v;
        }
    } else {
        for (int i = tid; i < total; i += blockDim.x) {
            float v = logits[g0 + i];
            if (noise) v += noise_scale * noise[g0 + i];
            const int r = i / E, e = i - r * E;
            tile[r * P + e] = v;
        }
    }
    __syncthreads();
    router4_body(L, scores, idx, part_me, part_cnt, hist, t0, rows, E, k);
}

// The gate's projection and the router in one launch for 16-bit or fp32 token tensors and up to GATE_ROUTER_MAX_E
// experts: the workgroup's 64 x E logits go from the matrix cores into the router's LDS tile (and out to `logits`,
// which the backward reads) instead of through a launch boundary.  The arithmetic is that of gate_fwd_kernel, sum
// for sum: a 32-token block's model dimension is cut into the same four quarters, one per wavefront, each
// accumulated by the same sequence of products and added in the same order, so the logits are bit-identical to
// hexa_gate_logits'.  Eight wavefronts (two token blocks) project; the first four then route.
constexpr int GATE_ROUTER_MAX_E = 64;
constexpr int GATE_ROUTER_NT = 2 * ROUTER_TB * ROUTER_G;
template <typename T>
__global__ __launch_bounds__(GATE_ROUTER_NT) void gate_router_kernel(
    float* __restrict__ logits, float* __restrict__ scores, int32_t* __restrict__ idx, float* __restrict__ part_me,
    float* __restrict__ part_cnt, const T* __restrict__ x, const float* __restrict__ wg, const float* __restrict__ noise,
    float noise_scale, int num_tokens, int d, int E, int k, int32_t* __restrict__ hist) {
    extern __shared__ float sh[];
    __shared__ float part[2][4][16][64];             // [token block][quarter of d][result register][lane]
    const Router4Lds L(sh, E);
    const int P = L.P;
    float* tile = L.tile;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int t0 = blockIdx.x * ROUTER_TB;
    const int rows = min(ROUTER_TB, num_tokens - t0);
    for (int i = tid; i < E; i += blockDim.x) L.cnt[i] = 0.f;
    if (hist)
        for (int i = tid; i < k * E; i += blockDim.x) L.hist[i] = 0;
    // ---- the gate: logits of 64 tokens into the tile ----
    const int r = lane & 31, h = lane >> 5;
    const int blk = wave >> 2, quarter = wave & 3;
    const int pieces = d >> 3;                       // 8 contraction indices per piece
    const int chunks = (pieces + 1) >> 1;            // a chunk = one piece per half-wavefront
    const int c0 = (chunks * quarter) >> 2, c1 = (chunks * (quarter + 1)) >> 2;
    const bool tok_ok = t0 + 32 * blk + r < num_tokens;
    const T* xrow = x + (size_t)(tok_ok ? t0 + 32 * blk + r : 0) * d;
    for (int e0 = 0; e0 < E; e0 += 32) {
        const bool exp_ok = e0 + r < E;
        const float* wrow = wg + (size_t)(exp_ok ? e0 + r : 0) * d;
        f32x16 acc = zero16();
        for (int c = c0; c < c1; c += FWD_NB) {
            float xv[FWD_NB][8], wv[FWD_NB][8];
#pragma unroll
            for (int u = 0; u < FWD_NB; ++u) {
                const int piece = 2 * (c + u) + h;
                const bool ok = c + u < c1 && piece < pieces;
                LoadN<T, 8>::run(xrow + (ok ? piece : 0) * 8, ok && tok_ok, xv[u]);
                LoadN<float, 8>::run(wrow + (ok ? piece : 0) * 8, ok && exp_ok, wv[u]);
            }
#pragma unroll
            for (int u = 0; u < FWD_NB; ++u)
#pragma unroll
                for (int i = 0; i < 8; ++i) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(xv[u][i], wv[u][i], acc, 0, 0, 0);
        }
#pragma unroll
        for (int v = 0; v < 16; ++v) part[blk][quarter][v][lane] = acc[v];
        __syncthreads();
        // wavefront (blk, w) finishes result registers 4w .. 4w+3: token row 8w + 4h + q of the block, expert column r
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int v = 4 * quarter + q;
            const float sum = ((part[blk][0][v][lane] + part[blk][1][v][lane]) + part[blk][2][v][lane]) + part[blk][3][v][lane];
            const int row = 32 * blk + 8 * quarter + 4 * h + q;
            if (exp_ok) tile[row * P + e0 + r] = sum;
        }
        __syncthreads();   // the partial sums have been consumed (the next expert block overwrites them)
    }
    // ---- the logits leave as they are; the noise joins the tile only ----
    const size_t g0 = (size_t)t0 * E;
    const int total = rows * E;
    if ((E & 3) == 0) {
        for (int i = tid * 4; i < total; i += blockDim.x * 4) {
            const int rr = i / E, e = i - rr * E;
            float4 v = *reinterpret_cast<const float4*>(tile + rr * P + e);
            *reinterpret_cast<float4*>(logits + g0 + i) = v;
            if (noise) {
                const float4 n = *reinterpret_cast<const float4*>(noise + g0 + i);
                v.x += noise_scale * n.x; v.y += noise_scale * n.y; v.z += noise_scale * n.z; v.w += noise_scale * n.w;
                *reinterpret_cast<float4*>(tile + rr * P + e) = v;
            }
        }
    } else {
        for (int i = tid; i < total; i += blockDim.x) {
            const int rr = i / E, e = i - rr * E;
            const float v = tile[rr * P + e];
            logits[g0 + i] = v;
            if (noise) tile[rr * P + e] = v + noise_scale * noise[g0 + i];
        }
    }
    __syncthreads();
    router4_body(L, scores, idx, part_me, part_cnt, hist, t0, rows, E, k);
}

// The GShard loss from the workgroup partials (see small_bodies.h) as a launch of its own.
__global__ __launch_bounds__(256) void router_loss_kernel(float* __restrict__ l_aux, float* __restrict__ me,
                                                          float* __restrict__ ce, const float* __restrict__ part_me,
                                                          const float* __restrict__ part_cnt, int nblocks,
                                                          int num_tokens, int E) {
    extern __shared__ float sh[];
    router_loss_body(sh, l_aux, me, ce, part_me, part_cnt, nblocks, num_tokens, E);
}

__global__ __launch_bounds__(256) void router_bwd_kernel(RouterBwdK p) {
    extern __shared__ float s_c[];
    router_bwd_body(s_c, p, blockIdx.x);
}


// ---- the same front end with the load-importance loss (impls/losses.py:21-42) ----------------------------
// Per token: top-k of softmax(logits + noise_scale*noise) as above; thr = the k-th choice's noisy LOGIT;
// s = softmax(logits) without noise; importance[e] += s[e]; load[e] += Phi((s[e] - thr) / sigma).  The
// loss is the mean of the squared coefficients of variation (unbiased variance / (mean^2 + 1e-10)) of
// importance and load.  One token per lane; the row (E floats) is walked in place, L1-resident.
__device__ __forceinline__ float normal_cdf(float z) { return 0.5f * erfcf(-z * 0.70710678118654752f); }
__device__ __forceinline__ float normal_pdf(float z) { return 0.3989422804014327f * expf(-0.5f * z * z); }

__global__ __launch_bounds__(ROUTER_TB) void router_li_fwd_kernel(float* __restrict__ scores, int32_t* __restrict__ idx,
                                                                  float* __restrict__ thr_out,
                                                                  float* __restrict__ part_imp,
                                                                  float* __restrict__ part_load,
                                                                  const float* __restrict__ logits,
                                                                  const float* __restrict__ noise, float noise_scale,
                                                                  float inv_sigma, int num_tokens, int E, int k) {
    const int lane = threadIdx.x;
    const int t = blockIdx.x * ROUTER_TB + lane;
    const bool ok = t < num_tokens;
    const float* lr = logits + (size_t)(ok ? t : 0) * E;
    const float* nr = noise ? noise + (size_t)(ok ? t : 0) * E : nullptr;
    float best_v[MAX_TOPK];
    int best_i[MAX_TOPK];
#pragma unroll
    for (int j = 0; j < MAX_TOPK; ++j) { best_v[j] = -INFINITY; best_i[j] = j; }
    // noisy scores: selection only
    float mx = -INFINITY, cmx = -INFINITY;
    for (int e = 0; e < E; ++e) {
        const float c = lr[e];
        cmx = fmaxf(cmx, c);
        mx = fmaxf(mx, nr ? c + noise_scale * nr[e] : c);
    }
    float sum = 0.f, csum = 0.f;
    for (int e = 0; e < E; ++e) {
        const float c = lr[e];
        csum += expf(c - cmx);
        sum += expf((nr ? c + noise_scale * nr[e] : c) - mx);
    }
    const float inv = 1.0f / sum, cinv = 1.0f / csum;
    for (int e = 0; e < E; ++e) {
        const float v = nr ? lr[e] + noise_scale * nr[e] : lr[e];
        topk_insert(best_v, best_i, k, expf(v - mx) * inv, e);
    }
    int last = 0;
#pragma unroll
    for (int j = 0; j < MAX_TOPK; ++j)
        if (j == k - 1) last = best_i[j];
    float thr = 0.f;
    if (ok) {
        thr = nr ? lr[last] + noise_scale * nr[last] : lr[last];
        thr_out[t] = thr;
#pragma unroll
        for (int j = 0; j < MAX_TOPK; ++j)
            if (j < k) idx[(size_t)t * k + j] = best_i[j];
    }
    // clean scores, importance and load; uniform trip count: every lane takes part in the reductions
    for (int e = 0; e < E; ++e) {
        float sc = 0.f, ld = 0.f;
        if (ok) {
            sc = expf(lr[e] - cmx) * cinv;
            scores[(size_t)t * E + e] = sc;
            ld = normal_cdf((sc - thr) * inv_sigma);
        }
#pragma unroll
        for (int m = 32; m > 0; m >>= 1) { sc += __shfl_xor(sc, m); ld += __shfl_xor(ld, m); }
        if (lane == 0) {
            part_imp[(size_t)blockIdx.x * E + e] = sc;
            part_load[(size_t)blockIdx.x * E + e] = ld;
        }
    }
}

// importance / load from the workgroup partials (fixed order), the loss, and its derivative with
// respect to each importance[e] and load[e] (kept for the backward pass):
//   cv2(v) = var(v) / (mean(v)^2 + eps),  var unbiased;  d cv2 / d v[e] =
//   2 (v[e] - mean) / ((E-1)(mean^2 + eps))  -  var * 2 mean / (E (mean^2 + eps)^2)
// With a balanced router every v[e] is close to the mean, so v[e] - mean cancels almost all digits:
// the sums over workgroups and everything after them are carried in double (one workgroup, a few
// thousand operations).
constexpr int ROUTER_LI_MAX_E = 1024;

__global__ __launch_bounds__(256) void router_li_loss_kernel(float* __restrict__ l_aux, float* __restrict__ importance,
                                                             float* __restrict__ load, float* __restrict__ g_imp,
                                                             float* __restrict__ g_load,
                                                             const float* __restrict__ part_imp,
                                                             const float* __restrict__ part_load, int nblocks, int E) {
    extern __shared__ double shd[];        // [nch][E] importance, [nch][E] load, then v_imp[E], v_load[E]
    const int nch = max(1, min(32, 2048 / E));
    double* s_a = shd;
    double* s_b = shd + nch * E;
    double* v_a = shd + 2 * nch * E;
    double* v_b = v_a + E;
    __shared__ double red[2][256];
    const int per = (nblocks + nch - 1) / nch;
    for (int i = threadIdx.x; i < nch * E; i += 256) {
        const int c = i / E, e = i - c * E;
        const int b0 = c * per, b1 = min(nblocks, b0 + per);
        double a = 0., b = 0.;
#pragma unroll 4
        for (int q = b0; q < b1; ++q) { a += part_imp[(size_t)q * E + e]; b += part_load[(size_t)q * E + e]; }
        s_a[i] = a;
        s_b[i] = b;
    }
    __syncthreads();
    double la = 0., lb = 0.;
    for (int e = threadIdx.x; e < E; e += 256) {
        double a = 0., b = 0.;
        for (int j = 0; j < nch; ++j) { a += s_a[j * E + e]; b += s_b[j * E + e]; }
        v_a[e] = a; v_b[e] = b;
        importance[e] = (float)a; load[e] = (float)b;
        la += a; lb += b;
    }
    auto block_sum2 = [&](double x, double y, double& ox, double& oy) {
        red[0][threadIdx.x] = x; red[1][threadIdx.x] = y;
        __syncthreads();
        for (int s = 128; s > 0; s >>= 1) {
            if (threadIdx.x < s) { red[0][threadIdx.x] += red[0][threadIdx.x + s]; red[1][threadIdx.x] += red[1][threadIdx.x + s]; }
            __syncthreads();
        }
        ox = red[0][0]; oy = red[1][0];
        __syncthreads();
    };
    double sa, sb;
    block_sum2(la, lb, sa, sb);
    const double ma = sa / E, mb = sb / E;
    double qa = 0., qb = 0.;
    for (int e = threadIdx.x; e < E; e += 256) {
        const double da = v_a[e] - ma, db = v_b[e] - mb;
        qa += da * da; qb += db * db;
    }
    double ssa, ssb;
    block_sum2(qa, qb, ssa, ssb);
    const double var_a = ssa / (E - 1), var_b = ssb / (E - 1);
    const double den_a = ma * ma + 1e-10, den_b = mb * mb + 1e-10;
    if (threadIdx.x == 0) *l_aux = (float)(0.5 * (var_a / den_a + var_b / den_b));
    for (int e = threadIdx.x; e < E; e += 256) {
        g_imp[e] = (float)(0.5 * (2. * (v_a[e] - ma) / ((E - 1) * den_a) - var_a * 2. * ma / (E * den_a * den_a)));
        g_load[e] = (float)(0.5 * (2. * (v_b[e] - mb) / ((E - 1) * den_b) - var_b * 2. * mb / (E * den_b * den_b)));
    }
}

// d l_aux / d logits:  ds[e] = g_imp[e] + g_load[e] * pdf(z[e]) / sigma,  z[e] = (s[e] - thr) / sigma;
// through the noise-free softmax  dlogits[e] = s[e] (ds[e] - sum_e' s[e'] ds[e']);  and through the
// threshold, which is the k-th choice's own logit:  dlogits[last] -= sum_e g_load[e] pdf(z[e]) / sigma.
__global__ __launch_bounds__(ROUTER_TB) void router_li_bwd_kernel(float* __restrict__ dlogits,
                                                                  const float* __restrict__ scores,
                                                                  const float* __restrict__ thr,
                                                                  const int32_t* __restrict__ idx,
                                                                  const float* __restrict__ g_imp,
                                                                  const float* __restrict__ g_load,
                                                                  const float* __restrict__ grad_l, float inv_sigma,
                                                                  int num_tokens, int E, int k) {
    extern __shared__ float s_g[];         // g_imp[E], g_load[E] scaled by the incoming gradient
    const float g = *grad_l;
    for (int e = threadIdx.x; e < E; e += blockDim.x) { s_g[e] = g * g_imp[e]; s_g[E + e] = g * g_load[e] * inv_sigma; }
    __syncthreads();
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= num_tokens) return;
    const float* sr = scores + (size_t)t * E;
    float* dr = dlogits + (size_t)t * E;
    const float th = thr[t];
    float dot = 0.f, dthr = 0.f;
    for (int e = 0; e < E; ++e) {
        const float sc = sr[e];
        const float w = s_g[E + e] * normal_pdf((sc - th) * inv_sigma);
        dot += sc * (s_g[e] + w);
        dthr -= w;
    }
    const int last = idx[(size_t)t * k + (k - 1)];
    for (int e = 0; e < E; ++e) {
        const float sc = sr[e];
        const float w = s_g[E + e] * normal_pdf((sc - th) * inv_sigma);
        dr[e] = sc * (s_g[e] + w - dot) + (e == last ? dthr : 0.f);
    }
}


}  // namespace
}  // namespace hexa

using namespace hexa;

extern "C" int hexa_router_ws_floats(int T, int E, int64_t* out) {
    if (!out || T < 0 || E < 1) HEXA_FAIL(HEXA_ERR_ARG, "hexa_router_ws_floats: bad arguments");
    *out = (int64_t)2 * (T > 0 ? div_up(T, ROUTER_TB) : 1) * E;
    return HEXA_OK;
}

namespace hexa {
namespace {
// The LDS tile of the four-lanes-per-token router (with the routing histogram behind it) passes 64 KiB for many
// experts and a deep top-k: such a launch needs the kernel's dynamic-LDS limit raised first, once per kernel, to the
// most any supported (E, k) asks for.
template <typename K> int allow_router_lds(K kernel, size_t bytes) {
    static bool done = false;   // per kernel
    if (bytes <= 64 * 1024 || done) return HEXA_OK;
    constexpr size_t most = sizeof(float) * router4_lds_floats(ROUTER_LDS_E, MAX_TOPK, true);
    static_assert(most <= 160 * 1024, "LDS of a CU");
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)most) != hipSuccess)
        HEXA_FAIL(HEXA_ERR_LAUNCH, "router: hipFuncSetAttribute(MaxDynamicSharedMemorySize=%d) failed", (int)most);
    done = true;
    return HEXA_OK;
}
}  // namespace
bool router_hist_supported(int E) { return E <= ROUTER_LDS_E; }
int router_tokens_per_workgroup() { return ROUTER_TB; }

// softmax + top-k + the loss partials (ws: hexa_router_ws_floats() floats); with `hist` (only where
// router_hist_supported) also the routing pass's histogram over units of 64 tokens
int launch_router_fwd(float* scores, int32_t* idx, const float* logits, const float* noise, float noise_scale, int T, int E,
                      int k, float* ws, int32_t* hist, hipStream_t st) {
    const int nb = div_up(T, ROUTER_TB);
    float* part_me = ws;
    float* part_cnt = ws + (size_t)nb * E;
    if (E <= ROUTER_LDS_E) {
        const size_t lds = sizeof(float) * router4_lds_floats(E, k, hist != nullptr);
        if (int rc = allow_router_lds(router_fwd4_kernel, lds)) return rc;
        hipLaunchKernelGGL(router_fwd4_kernel, dim3(nb), dim3(ROUTER_TB * ROUTER_G), lds, st, scores, idx, part_me, part_cnt, logits,
                           noise, noise_scale, T, E, k, hist);
    } else
        hipLaunchKernelGGL(router_fwd_kernel, dim3(nb), dim3(ROUTER_TB), sizeof(float) * 2 * E, st, scores, idx,
                           part_me, part_cnt, logits, noise, noise_scale, T, E, k);
    HEXA_CHECK_LAUNCH("router_fwd");
    return HEXA_OK;
}

// gate projection + router in one launch (see gate_router_kernel); same results as hexa_gate_logits followed by
// launch_router_fwd
bool gate_router_supported(int d, int E, int x_dt) {
    return E <= GATE_ROUTER_MAX_E && (d % 8) == 0 && (x_dt == HEXA_F32 || x_dt == HEXA_BF16 || x_dt == HEXA_F16);
}
int launch_gate_router(float* logits, float* scores, int32_t* idx, const void* x, const float* wg, const float* noise,
                       float noise_scale, int T, int d, int E, int k, int x_dt, float* ws, int32_t* hist, hipStream_t st) {
    const int nb = div_up(T, ROUTER_TB);
    float* part_me = ws;
    float* part_cnt = ws + (size_t)nb * E;
    const size_t lds = sizeof(float) * router4_lds_floats(E, k, hist != nullptr);
    const dim3 grid(nb), block(GATE_ROUTER_NT);
    if (int rc = x_dt == HEXA_F32    ? allow_router_lds(gate_router_kernel<float>, lds)
                 : x_dt == HEXA_BF16 ? allow_router_lds(gate_router_kernel<__bf16>, lds)
                                     : allow_router_lds(gate_router_kernel<_Float16>, lds))
        return rc;
    if (x_dt == HEXA_F32)
        hipLaunchKernelGGL(gate_router_kernel<float>, grid, block, lds, st, logits, scores, idx, part_me, part_cnt, (const float*)x, wg,
                           noise, noise_scale, T, d, E, k, hist);
    else if (x_dt == HEXA_BF16)
        hipLaunchKernelGGL(gate_router_kernel<__bf16>, grid, block, lds, st, logits, scores, idx, part_me, part_cnt, (const __bf16*)x, wg,
                           noise, noise_scale, T, d, E, k, hist);
    else
        hipLaunchKernelGGL(gate_router_kernel<_Float16>, grid, block, lds, st, logits, scores, idx, part_me, part_cnt,
                           (const _Float16*)x, wg, noise, noise_scale, T, d, E, k, hist);
    HEXA_CHECK_LAUNCH("gate_router");
    return HEXA_OK;
}
}  // namespace hexa

static int check_router_forward(int T, int E, int k, bool ptrs_ok) {
    if (T < 1 || E < 1 || k < 1) HEXA_FAIL(HEXA_ERR_ARG, "hexa_router_forward: bad sizes T=%d E=%d k=%d", T, E, k);
    if (k > MAX_TOPK || k > E) HEXA_FAIL(HEXA_ERR_UNSUPPORTED, "hexa_router_forward: top_k must be <= min(E, %d)", MAX_TOPK);
    if (!ptrs_ok) HEXA_FAIL(HEXA_ERR_ARG, "hexa_router_forward: null pointer");
    if (E > 4096) HEXA_FAIL(HEXA_ERR_UNSUPPORTED, "hexa_router_forward: more than 4096 experts");
    return HEXA_OK;
}

namespace hexa {
int router_forward_check(int T, int E, int k, bool ptrs_ok) { return check_router_forward(T, E, k, ptrs_ok); }
}

extern "C" int hexa_router_forward(float* scores, int32_t* idx, float* me, float* ce, float* l_aux,
                                   const float* logits, const float* noise, float noise_scale, int T, int E, int k,
                                   float* ws, void* stream) {
    if (int rc = check_router_forward(T, E, k, scores && idx && me && ce && l_aux && logits && ws)) return rc;
    hipStream_t st = (hipStream_t)stream;
    if (int rc = launch_router_fwd(scores, idx, logits, noise, noise_scale, T, E, k, ws, nullptr, st)) return rc;
    const int nb = div_up(T, ROUTER_TB);
    hipLaunchKernelGGL(router_loss_kernel, dim3(1), dim3(256), sizeof(float) * (2 * router_loss_chunks(E) * E + 256), st,
                       l_aux, me, ce, ws, ws + (size_t)nb * E, nb, T, E);
    HEXA_CHECK_LAUNCH("router_loss");
    return HEXA_OK;
}

extern "C" int hexa_router_backward(float* dlogits, const float* scores, const float* ce, const float* grad_l_aux,
                                    int T, int E, void* stream) {
    if (T < 1 || E < 1) HEXA_FAIL(HEXA_ERR_ARG, "hexa_router_backward: bad sizes");
    if (!dlogits || !scores || !ce || !grad_l_aux) HEXA_FAIL(HEXA_ERR_ARG, "hexa_router_backward: null pointer");
    if (E > 8192) HEXA_FAIL(HEXA_ERR_UNSUPPORTED, "hexa_router_backward: more than 8192 experts");
    SmallTask t;
    t.kind = TASK_ROUTER_BWD; t.router_bwd = RouterBwdK{dlogits, scores, ce, grad_l_aux, T, E}; t.blocks = div_up(T, 256);
    if (!defer_task(E <= BATCH_ROUTER_BWD_MAX_E ? defer_targets().router_bwd : nullptr, t)) {
        hipLaunchKernelGGL(router_bwd_kernel, dim3(t.blocks), dim3(256), sizeof(float) * E, (hipStream_t)stream, t.router_bwd);
        HEXA_CHECK_LAUNCH("router_bwd");
    }
    return HEXA_OK;
}

extern "C" int hexa_router_forward_load_importance(float* scores, int32_t* idx, float* thr, float* importance,
                                                   float* load, float* g_importance, float* g_load, float* l_aux,
                                                   const float* logits, const float* noise, float noise_scale,
                                                   float sigma, int T, int E, int k, float* ws, void* stream) {
    const char* who = "hexa_router_forward_load_importance";
    if (T < 1 || E < 2 || k < 1) HEXA_FAIL(HEXA_ERR_ARG, "%s: bad sizes T=%d E=%d k=%d (E >= 2 for a variance)", who, T, E, k);
    if (k > MAX_TOPK || k > E) HEXA_FAIL(HEXA_ERR_UNSUPPORTED, "%s: top_k must be <= min(E, %d)", who, MAX_TOPK);
    if (!(sigma > 0.f)) HEXA_FAIL(HEXA_ERR_ARG, "%s: sigma must be > 0 (gate_noise / E of the reference)", who);
    if (!scores || !idx || !thr || !importance || !load || !g_importance || !g_load || !l_aux || !logits || !ws)
        HEXA_FAIL(HEXA_ERR_ARG, "%s: null pointer", who);
    if (E > ROUTER_LI_MAX_E) HEXA_FAIL(HEXA_ERR_UNSUPPORTED, "%s: more than %d experts", who, ROUTER_LI_MAX_E);
    hipStream_t st = (hipStream_t)stream;
    const int nb = div_up(T, ROUTER_TB);
    float* part_imp = ws;
    float* part_load = ws + (size_t)nb * E;
    hipLaunchKernelGGL(router_li_fwd_kernel, dim3(nb), dim3(ROUTER_TB), 0, st, scores, idx, thr, part_imp, part_load,
                       logits, noise, noise_scale, 1.0f / sigma, T, E, k);
    HEXA_CHECK_LAUNCH("router_li_fwd");
    const int nch = std::max(1, std::min(32, 2048 / E));
    hipLaunchKernelGGL(router_li_loss_kernel, dim3(1), dim3(256), sizeof(double) * (2 * nch * E + 2 * E), st, l_aux,
                       importance, load, g_importance, g_load, part_imp, part_load, nb, E);
    HEXA_CHECK_LAUNCH("router_li_loss");
    return HEXA_OK;
}

extern "C" int hexa_router_backward_load_importance(float* dlogits, const float* scores, const float* thr,
                                                    const int32_t* idx, const float* g_importance,
                                                    const float* g_load, const float* grad_l_aux, float sigma, int T,
                                                    int E, int k, void* stream) {
    const char* who = "hexa_router_backward_load_importance";
    if (T < 1 || E < 2 || k < 1 || k > E) HEXA_FAIL(HEXA_ERR_ARG, "%s: bad sizes", who);
    if (!(sigma > 0.f)) HEXA_FAIL(HEXA_ERR_ARG, "%s: sigma must be > 0", who);
    if (!dlogits || !scores || !thr || !idx || !g_importance || !g_load || !grad_l_aux)
        HEXA_FAIL(HEXA_ERR_ARG, "%s: null pointer", who);
    if (E > 4096) HEXA_FAIL(HEXA_ERR_UNSUPPORTED, "%s: more than 4096 experts", who);
    hipLaunchKernelGGL(router_li_bwd_kernel, dim3(div_up(T, ROUTER_TB)), dim3(ROUTER_TB), sizeof(float) * 2 * E,
                       (hipStream_t)stream, dlogits, scores, thr, idx, g_importance, g_load, grad_l_aux, 1.0f / sigma,
                       T, E, k);
    HEXA_CHECK_LAUNCH("router_li_bwd");
    return HEXA_OK;
}
