// Internal declarations shared by the HIP translation units of libhexa_moe_hip.so.
// The public C ABI is include/hexa_moe_hip.h; nothing here is exported.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/hexa_moe_hip.h"

namespace hexa {

// ---- error plumbing -----------------------------------------------------------------------
void set_error(const char* fmt, ...);

#define HEXA_FAIL(code, ...)                \
    do {                                    \
        ::hexa::set_error(__VA_ARGS__);     \
        return (code);                      \
    } while (0)

#define HEXA_CHECK_LAUNCH(what)                                                        \
    do {                                                                               \
        hipError_t e__ = hipGetLastError();                                            \
        if (e__ != hipSuccess) HEXA_FAIL(HEXA_ERR_LAUNCH, "%s: launch failed: %s", what, \
                                         hipGetErrorString(e__));                      \
    } while (0)

// ---- tiling constants shared between the routing pass and the matmul kernels ----------------
// Row tile of the gathered-row grouped GEMM (ESMM).  The routing pass emits one tile_info entry
// per HEXA_TILE_ROWS rows of every (slot, expert) segment.
constexpr int kTileRows = HEXA_TILE_ROWS;

static inline int div_up(int a, int b) { return (a + b - 1) / b; }

// ---- routing metadata view (all device pointers) --------------------------------------------
struct RouteView {
    const int32_t* token_ids;   // [k][list_stride]
    const int32_t* offsets;     // [k][E+1]
    const int4* tile_info;      // [k][mt_ub]: {expert, row_start, row_count, 0}
    const int32_t* tile_count;  // [k]
    const int4* tile_info_l;    // the same with HEXA_TILE_ROWS_L rows per tile
    const int32_t* tile_count_l;
    int T, k, E, mt_ub, mt_ub_l;
};

RouteView route_view(const int32_t* route, int T, int k, int E);

// ---- launchers implemented in the kernel files ----------------------------------------------
struct EsmmArgs {
    void* out; const void* x; const void* w; const void* bias; void* out_act; void* slot_ws;
    RouteView r;
    int in_dim, out_dim;
    int x_per_slot, out_per_slot;  // row operand / result indexed [slot][T][*] (1) or [T][*] (0)
    int w_layout;                  // HEXA_W_IN_OUT: [E][in][out]; HEXA_W_OUT_IN: [E][out][in]
    int accumulate;                // result += instead of =
    int x_dt, w_dt, bias_dt, out_dt;
    int act;
    // optional: also db[e][:] (+)= column sums of the expert's stored result rows (ESS of the result), through
    // per-tile partial sums in `colsum` (16-bit per-slot results on the fast path only)
    float* colsum = nullptr; void* db = nullptr; int db_dt = 0, db_accumulate = 0;
    // optional, with slot_ws on the fast path: one more tensor of the result's shape added by the slot sum
    const void* sum_extra = nullptr;
};
struct EstmmArgs {
    void* dw; const void* p; const void* q;   // dw[e][m][n] = sum_rows p[row][m] * q[row][n]
    RouteView r;
    int m_dim, n_dim;
    int p_per_slot, q_per_slot;
    int accumulate;
    int pq_dt, dw_dt;
    const int32_t* plan; int max_slots; float* scratch;   // optional: the busiest experts cut into parts
};
struct EssArgs {
    void* db; const void* dy;
    RouteView r;
    int out_dim, dy_per_slot, accumulate, dy_dt, db_dt;
    float* ws; int64_t ws_floats;   // optional scratch for partial sums
};

int esmm_call(void* out, const void* x, const void* w, const void* bias, const int32_t* route, int m2s, int w_layout,
              int accumulate, int T, int k, int in_dim, int out_dim, int E, int x_dt, int w_dt, int bias_dt, int out_dt,
              int act, void* out_act, void* slot_ws, const void* sum_extra, bool* extra_used, void* stream);
bool esmm_slot_sum_takes_extra(const int32_t* route, int w_layout, int T, int k, int in_dim, int out_dim, int E, int x_dt,
                               int w_dt, int out_dt, const void* slot_ws);
int launch_esmm16(const EsmmArgs& a, hipStream_t s);
int launch_esmm32(const EsmmArgs& a, hipStream_t s);
// Tuning / testing knobs: 0 = automatic.  Each one starts from an environment variable (read once) and
// can be changed at run time with hexa_set_option.
enum Opt {
    OPT_TILE,           // HEXA_MOE_TILE: tile configuration of the 16-bit fast path (see gemm16_dma.hip)
    OPT_PIPE,           // HEXA_MOE_PIPE: the pipelined persistent ESMM kernel (multiply, copy and store wavefronts side by side) runs
                        // whatever it covers; 2 = never, 1 = also when a tile shape is forced
    OPT_GENERAL,        // HEXA_MOE_GENERAL_KERNELS: 1 = general 16-bit kernels instead of the fast path
    OPT_ESMM_MAP,       // HEXA_ESMM_MAP: 2 = runs of tiles per XCD instead of one contiguous eighth of the tiles per XCD
    OPT_ESMM_GROUP,     // HEXA_ESMM_GROUP: row tiles per XCD run
    OPT_ESTMM_GROUP,    // HEXA_ESTMM_GROUP: row tiles per XCD run
    OPT_ESMM_STREAM,    // HEXA_ESMM_STREAM: results stored with the streaming (non-temporal) hint: 0 = by the pipelined ESMM
                        // kernel and ESTMM's finished results, 1 = by the one-tile ESMM kernels as well, 2 = by none
    OPT_ROUTE_KERNELS,  // HEXA_ROUTE_KERNELS: 3 = always the three-launch routing pass (behind the router's histogram: a scan and
                        // a scatter launch instead of one), 1 = one launch up to 65536 tokens
    OPT_BATCH,          // HEXA_MOE_BATCH: 2 = every small kernel of the depth backward in a launch of its own, 1 = four batch launches instead of three
    OPT_FFN_FUSED,      // HEXA_MOE_FFN_FUSED: 1 = hexa_moe_depth_forward runs fc1, GELU and fc2 in one kernel where it is covered
    OPT_GATE_ROUTER,    // HEXA_MOE_GATE_ROUTER: 2 = hexa_moe_depth_forward runs the gate projection and the router as two launches
    OPT_ESTMM_PIPE,     // HEXA_ESTMM_PIPE: 1 = the persistent ESTMM kernel wherever it applies (default: the one-item-per-workgroup kernel)
    OPT_SIDE_STREAM,    // HEXA_MOE_SIDE_STREAM: the small kernels of hexa_moe_depth_backward on a second stream beside the matmul kernels: 1 = yes, 2 = no
    OPT_COUNT
};
int option(int id);

bool esmm16_dma_supported(const EsmmArgs& a);
bool esmm16_dma_colsum_supported(const EsmmArgs& a);
bool esmm16_pipe_supported(const EsmmArgs& a);
int launch_esmm16_pipe(const EsmmArgs& a, hipStream_t st);
bool ffn16_fused_supported(int T, int k, int d_in, int hidden, int d_out, int act_dt, int w_dt, int b1_dt, int b2_dt);
int launch_ffn16_fused(void* y1, void* y2, void* y, const void* x, const void* w1, const void* b1, const void* w2,
                       const void* b2, const RouteView& r, int d_in, int hidden, int d_out, int act_dt, int b1_dt,
                       int b2_dt, void* slot_ws, hipStream_t st);
int launch_colsum_fold(const EsmmArgs& a, int mt_ub, int tile_rows, int ntn, int bn, hipStream_t st);
int estmm_plan_cap_for(const RouteView& r, int out_dim, int in_dim);   // rows above which an expert's list is cut
int launch_estmm_plan(int32_t* plan, const RouteView& r, int max_slots, int cap, hipStream_t st);
int launch_estmm_fixup(const EstmmArgs& a, hipStream_t st);
// whether a routing of this size goes to the persistent ESTMM kernel (the plan is made for the kernel that will run)
bool estmm_pipe_wanted(const RouteView& r);
bool estmm16_pipe_supported(const EstmmArgs& a);
int launch_estmm16_pipe(const EstmmArgs& a, hipStream_t st);
int launch_esmm16_dma(const EsmmArgs& a, hipStream_t s);
bool dma_path_enabled();
bool estmm16_dma_supported(const EstmmArgs& a);
int launch_estmm16_dma(const EstmmArgs& a, hipStream_t s);
int launch_estmm16(const EstmmArgs& a, hipStream_t s);
int launch_estmm32(const EstmmArgs& a, hipStream_t s);
int launch_ess(const EssArgs& a, hipStream_t s);
int launch_ess_noalloc(EssArgs a, hipStream_t s);
int launch_sum_slots(void* out, const void* ws, int64_t n, int nws, int dt, hipStream_t s, const void* extra = nullptr);
// routing front end of the depth call: the router also counts, the counting sort's scan launch also finishes the loss,
// its scatter launch also makes the ESTMM plan (see router.hip, route.hip)
bool router_hist_supported(int E);
int router_tokens_per_workgroup();
int router_forward_check(int T, int E, int k, bool ptrs_ok);
int launch_router_fwd(float* scores, int32_t* idx, const float* logits, const float* noise, float noise_scale, int T, int E,
                      int k, float* ws, int32_t* hist, hipStream_t st);
bool gate_router_supported(int d, int E, int x_dt);
int launch_gate_router(float* logits, float* scores, int32_t* idx, const void* x, const float* wg, const float* noise,
                       float noise_scale, int T, int d, int E, int k, int x_dt, float* ws, int32_t* hist, hipStream_t st);
int launch_route_from_hist(const int32_t* idx, int T, int k, int E, int32_t* route, int32_t* hist, int unit_tokens,
                           float* l_aux, float* me, float* ce, const float* router_ws, int32_t* plan, int plan_slots,
                           int plan_cap, hipStream_t st);
int launch_gelu_bwd(void* dy1, const void* dy2, const void* y1, int64_t n, int dt, hipStream_t s);

// ---- small device helpers -------------------------------------------------------------------
__device__ __forceinline__ float gelu_erf(float x) {
    return 0.5f * x * (1.0f + erff(x * 0.70710678118654752440f));
}

// gelu'(x) = Phi(x) + x * phi(x), erf form
__device__ __forceinline__ float gelu_grad_erf(float x) {
    return 0.5f * (1.0f + erff(x * 0.70710678118654752440f)) + x * 0.39894228040143267794f * expf(-0.5f * x * x);
}

template <typename T> struct Cvt;
template <> struct Cvt<float> {
    static __device__ __forceinline__ float to_f(float v) { return v; }
    static __device__ __forceinline__ float from_f(float v) { return v; }
};
template <> struct Cvt<__bf16> {
    static __device__ __forceinline__ float to_f(__bf16 v) { return (float)v; }
    static __device__ __forceinline__ __bf16 from_f(float v) { return (__bf16)v; }
};
template <> struct Cvt<_Float16> {
    static __device__ __forceinline__ float to_f(_Float16 v) { return (float)v; }
    static __device__ __forceinline__ _Float16 from_f(float v) { return (_Float16)v; }
};

// Store / accumulate one fp32 value into a result buffer whose element type is chosen at run time.
__device__ __forceinline__ void store_out(void* base, size_t idx, float v, int dt, bool accumulate) {
    if (dt == HEXA_F32) {
        float* p = (float*)base + idx;
        *p = accumulate ? (*p + v) : v;
    } else if (dt == HEXA_BF16) {
        __bf16* p = (__bf16*)base + idx;
        *p = (__bf16)(accumulate ? ((float)*p + v) : v);
    } else {
        _Float16* p = (_Float16*)base + idx;
        *p = (_Float16)(accumulate ? ((float)*p + v) : v);
    }
}
__device__ __forceinline__ float load_as_f(const void* base, size_t idx, int dt) {
    if (dt == HEXA_F32) return ((const float*)base)[idx];
    if (dt == HEXA_BF16) return (float)((const __bf16*)base)[idx];
    return (float)((const _Float16*)base)[idx];
}

}  // namespace hexa
