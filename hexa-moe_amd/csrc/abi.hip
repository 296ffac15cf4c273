// C ABI of libhexa_moe_hip.so (declared in include/hexa_moe_hip.h): argument validation, dtype
// dispatch and error reporting around the kernel launchers.  Nothing here allocates device memory
// or waits for the device.
#include <stdlib.h>
#include <string.h>

#include "hexa_internal.h"

namespace hexa {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

namespace {
struct OptEntry { const char* name; const char* env; int value; bool loaded; };
OptEntry g_opts[OPT_COUNT] = {
    {"tile", "HEXA_MOE_TILE", 0, false},          {"pipe", "HEXA_MOE_PIPE", 0, false},
    {"general_kernels", "HEXA_MOE_GENERAL_KERNELS", 0, false}, {"esmm_map", "HEXA_ESMM_MAP", 0, false},
    {"esmm_group", "HEXA_ESMM_GROUP", 0, false},  {"estmm_group", "HEXA_ESTMM_GROUP", 0, false},
    {"esmm_stream", "HEXA_ESMM_STREAM", 0, false}, {"route_kernels", "HEXA_ROUTE_KERNELS", 0, false},
    {"batch", "HEXA_MOE_BATCH", 0, false},
    {"ffn_fused", "HEXA_MOE_FFN_FUSED", 0, false},
    {"gate_router", "HEXA_MOE_GATE_ROUTER", 0, false},
    {"estmm_pipe", "HEXA_ESTMM_PIPE", 0, false},
    {"side_stream", "HEXA_MOE_SIDE_STREAM", 0, false},
};
}  // namespace

int option(int id) {
    OptEntry& o = g_opts[id];
    if (!o.loaded) {
        const char* v = getenv(o.env);
        o.value = v ? atoi(v) : 0;
        o.loaded = true;
    }
    return o.value;
}
bool dma_path_enabled() { return option(OPT_GENERAL) != 1; }

static bool is_dt(int dt) { return dt == HEXA_F32 || dt == HEXA_F16 || dt == HEXA_BF16; }
static bool is_16(int dt) { return dt == HEXA_F16 || dt == HEXA_BF16; }

static int check_sizes(const char* who, int T, int k, int E, int a, int b) {
    if (T < 0 || k < 1 || E < 1 || a < 1 || b < 1)
        HEXA_FAIL(HEXA_ERR_ARG, "%s: bad sizes T=%d k=%d E=%d dims=(%d,%d)", who, T, k, E, a, b);
    return HEXA_OK;
}

}  // namespace hexa

using namespace hexa;

extern "C" int hexa_set_option(const char* name, int value) {
    if (!name) HEXA_FAIL(HEXA_ERR_ARG, "hexa_set_option: null name");
    for (int i = 0; i < OPT_COUNT; ++i)
        if (!strcmp(name, g_opts[i].name)) {
            g_opts[i].value = value;
            g_opts[i].loaded = true;
            return HEXA_OK;
        }
    HEXA_FAIL(HEXA_ERR_ARG, "hexa_set_option: unknown option '%s'", name);
}


extern "C" const char* hexa_last_error(void) { return g_err; }
extern "C" int hexa_abi_version(void) { return HEXA_ABI_VERSION; }

// Whether esmm_call, for a slot-summed (m2s) result of these sizes and types, takes the fast path whose slot sum can
// add one more tensor (`sum_extra`): the same predicate esmm_call applies, for callers that must decide beforehand
// where that addend is written.
bool hexa::esmm_slot_sum_takes_extra(const int32_t* route, int w_layout, int T, int k, int in_dim, int out_dim, int E,
                                     int x_dt, int w_dt, int out_dt, const void* slot_ws) {
    if (T <= 0 || k <= 1 || !slot_ws || x_dt == HEXA_F32 || !dma_path_enabled()) return false;
    EsmmArgs a;
    a.out = nullptr; a.x = nullptr; a.w = nullptr; a.bias = nullptr; a.out_act = nullptr; a.slot_ws = const_cast<void*>(slot_ws);
    a.r = route_view(route, T, k, E);
    a.in_dim = in_dim; a.out_dim = out_dim;
    a.x_per_slot = 1; a.out_per_slot = 0;
    a.w_layout = w_layout; a.accumulate = 0;
    a.x_dt = x_dt; a.w_dt = w_dt; a.bias_dt = HEXA_F32; a.out_dt = out_dt; a.act = HEXA_ACT_NONE;
    return esmm16_dma_supported(a);
}

// The body of hexa_esmm with one more operand: `sum_extra` (may be null) is a tensor of the result's shape that
// the slot sum adds on the fast path (m2s, top_k > 1, slot_ws given); *extra_used says whether it was added.
int hexa::esmm_call(void* out, const void* x, const void* w, const void* bias, const int32_t* route, int m2s,
                    int w_layout, int accumulate, int T, int k, int in_dim, int out_dim, int E, int x_dt, int w_dt,
                    int bias_dt, int out_dt, int act, void* out_act, void* slot_ws, const void* sum_extra,
                    bool* extra_used, void* stream) {
    if (extra_used) *extra_used = false;
    if (int rc = check_sizes("hexa_esmm", T, k, E, in_dim, out_dim)) return rc;
    if (!out || !x || !w || !route) HEXA_FAIL(HEXA_ERR_ARG, "hexa_esmm: null pointer");
    if (w_layout != HEXA_W_IN_OUT && w_layout != HEXA_W_OUT_IN) HEXA_FAIL(HEXA_ERR_ARG, "hexa_esmm: bad w_layout %d", w_layout);
    if (!is_dt(x_dt) || !is_dt(w_dt) || !is_dt(out_dt) || (bias && !is_dt(bias_dt)))
        HEXA_FAIL(HEXA_ERR_ARG, "hexa_esmm: unknown element type");
    if (act != HEXA_ACT_NONE && act != HEXA_ACT_GELU && act != HEXA_ACT_GELU_BWD)
        HEXA_FAIL(HEXA_ERR_ARG, "hexa_esmm: unknown activation %d", act);
    if (act != HEXA_ACT_NONE && (!out_act || m2s || accumulate))
        HEXA_FAIL(HEXA_ERR_ARG, "hexa_esmm: a fused activation needs out_act, m2s == 0 and accumulate == 0");
    if (T == 0) return HEXA_OK;
    EsmmArgs a;
    a.out = out; a.x = x; a.w = w; a.bias = bias; a.out_act = out_act; a.slot_ws = slot_ws;
    a.r = route_view(route, T, k, E);
    a.in_dim = in_dim; a.out_dim = out_dim;
    a.x_per_slot = m2s ? 1 : 0;
    a.out_per_slot = m2s ? 0 : 1;
    a.w_layout = w_layout; a.accumulate = accumulate ? 1 : 0;
    a.x_dt = x_dt; a.w_dt = w_dt; a.bias_dt = bias_dt; a.out_dt = out_dt; a.act = act;
    hipStream_t st = (hipStream_t)stream;
    if (x_dt == HEXA_F32) {
        if (w_dt != HEXA_F32 || out_dt != HEXA_F32 || (bias && bias_dt != HEXA_F32))
            HEXA_FAIL(HEXA_ERR_UNSUPPORTED, "hexa_esmm: fp32 tokens need fp32 weights, bias and result");
        return launch_esmm32(a, st);
    }
    if (w_dt != x_dt && w_dt != HEXA_F32)
        HEXA_FAIL(HEXA_ERR_UNSUPPORTED, "hexa_esmm: weights must be fp32 or the tokens' 16-bit type");
    if (out_dt != x_dt && out_dt != HEXA_F32)
        HEXA_FAIL(HEXA_ERR_UNSUPPORTED, "hexa_esmm: result must be fp32 or the tokens' 16-bit type");
    if (bias && bias_dt != x_dt && bias_dt != HEXA_F32)
        HEXA_FAIL(HEXA_ERR_UNSUPPORTED, "hexa_esmm: bias must be fp32 or the tokens' 16-bit type");
    if (dma_path_enabled() && esmm16_dma_supported(a)) {
        if (sum_extra && !a.out_per_slot && k > 1 && slot_ws) {
            a.sum_extra = sum_extra;
            if (extra_used) *extra_used = true;
        }
        return launch_esmm16_dma(a, st);
    }
    return launch_esmm16(a, st);
}

extern "C" int hexa_esmm(void* out, const void* x, const void* w, const void* bias, const int32_t* route, int m2s,
                         int w_layout, int accumulate, int T, int k, int in_dim, int out_dim, int E, int x_dt,
                         int w_dt, int bias_dt, int out_dt, int act, void* out_act, void* slot_ws,
                         void* stream) {
    return esmm_call(out, x, w, bias, route, m2s, w_layout, accumulate, T, k, in_dim, out_dim, E, x_dt, w_dt, bias_dt,
                     out_dt, act, out_act, slot_ws, nullptr, nullptr, stream);
}

extern "C" int hexa_estmm(void* dw, const void* dy, const void* x, const int32_t* route, int dy_per_slot,
                          int x_per_slot, int accumulate, int T, int k, int out_dim, int in_dim, int E, int dt,
                          int dw_dt, int32_t* plan, int max_slots, float* scratch, void* stream) {
    if (int rc = check_sizes("hexa_estmm", T, k, E, in_dim, out_dim)) return rc;
    if (!dw || !route || !dy || !x) HEXA_FAIL(HEXA_ERR_ARG, "hexa_estmm: null pointer");
    if (!is_dt(dt) || !is_dt(dw_dt)) HEXA_FAIL(HEXA_ERR_ARG, "hexa_estmm: unknown element type");
    if (dw_dt != HEXA_F32 && dw_dt != dt)
        HEXA_FAIL(HEXA_ERR_UNSUPPORTED, "hexa_estmm: dw must be fp32 or the operands' type");
    hipStream_t st = (hipStream_t)stream;
    EstmmArgs a;
    a.dw = dw; a.p = dy; a.q = x;
    a.r = route_view(route, T, k, E);
    a.m_dim = out_dim; a.n_dim = in_dim;
    a.p_per_slot = dy_per_slot ? 1 : 0; a.q_per_slot = x_per_slot ? 1 : 0;
    a.accumulate = accumulate ? 1 : 0; a.pq_dt = dt; a.dw_dt = dw_dt;
    // a plan without scratch (max_slots < 2) cuts no expert: it orders the work and carries the persistent kernel's queue
    a.plan = plan;
    a.max_slots = (plan && scratch && max_slots >= 2) ? max_slots : 0;
    a.scratch = a.max_slots ? scratch : nullptr;
    if (is_16(dt) && dma_path_enabled() && estmm_pipe_wanted(a.r) && estmm16_pipe_supported(a)) return launch_estmm16_pipe(a, st);
    if (!a.max_slots) a.plan = nullptr;
    if (is_16(dt) && dma_path_enabled() && estmm16_dma_supported(a)) return launch_estmm16_dma(a, st);
    return is_16(dt) ? launch_estmm16(a, st) : launch_estmm32(a, st);
}

extern "C" int hexa_estmm_plan(int32_t* plan, const int32_t* route, int T, int k, int E, int max_slots, int out_dim,
                               int in_dim, void* stream) {
    if (int rc = check_sizes("hexa_estmm_plan", T, k, E, 8, 8)) return rc;
    if (!plan || !route || max_slots < 0 || out_dim < 0 || in_dim < 0) HEXA_FAIL(HEXA_ERR_ARG, "hexa_estmm_plan: bad arguments");
    const RouteView r = route_view(route, T, k, E);
    return launch_estmm_plan(plan, r, max_slots, estmm_plan_cap_for(r, out_dim, in_dim), (hipStream_t)stream);
}

extern "C" int hexa_ess(void* db, const void* dy, const int32_t* route, int dy_per_slot, int accumulate, int T, int k,
                        int out_dim, int E, int dt, int db_dt, float* ws, int64_t ws_floats, void* stream) {
    if (int rc = check_sizes("hexa_ess", T, k, E, out_dim, out_dim)) return rc;
    if (!db || !route || !dy) HEXA_FAIL(HEXA_ERR_ARG, "hexa_ess: null pointer");
    if (!is_dt(dt) || !is_dt(db_dt)) HEXA_FAIL(HEXA_ERR_ARG, "hexa_ess: unknown element type");
    hipStream_t st = (hipStream_t)stream;
    EssArgs a;
    a.db = db; a.dy = dy;
    a.r = route_view(route, T, k, E);
    a.out_dim = out_dim; a.dy_per_slot = dy_per_slot ? 1 : 0; a.accumulate = accumulate ? 1 : 0;
    a.dy_dt = dt; a.db_dt = db_dt;
    a.ws = ws; a.ws_floats = ws ? ws_floats : 0;
    return launch_ess(a, st);
}

extern "C" int hexa_ess_noalloc(void* db, const void* dy, const int32_t* route, int dy_per_slot, int accumulate, int T,
                                int k, int out_dim, int E, int dt, int db_dt, void* stream) {
    if (int rc = check_sizes("hexa_ess_noalloc", T, k, E, out_dim, out_dim)) return rc;
    if (!db || !route || !dy) HEXA_FAIL(HEXA_ERR_ARG, "hexa_ess_noalloc: null pointer");
    if (!is_dt(dt) || !is_dt(db_dt)) HEXA_FAIL(HEXA_ERR_ARG, "hexa_ess_noalloc: unknown element type");
    EssArgs a;
    a.db = db; a.dy = dy;
    a.r = route_view(route, T, k, E);
    a.out_dim = out_dim; a.dy_per_slot = dy_per_slot ? 1 : 0; a.accumulate = accumulate ? 1 : 0;
    a.dy_dt = dt; a.db_dt = db_dt;
    a.ws = nullptr; a.ws_floats = 0;
    return launch_ess_noalloc(a, (hipStream_t)stream);
}

extern "C" int hexa_fused_grad(void* j_b, void* j_x, void* j_w, const void* j_y, const void* w, const void* x,
                               const int32_t* route, int m2s, int accumulate, int T, int k, int in_dim, int out_dim,
                               int E, int act_dt, int w_dt, int jx_dt, int jw_dt, int jb_dt, void* slot_ws,
                               int32_t* plan, int max_slots, float* estmm_scratch, float* ess_ws,
                               int64_t ess_ws_floats, void* stream) {
    if (!j_x || !j_w || !j_y || !w || !x || !route) HEXA_FAIL(HEXA_ERR_ARG, "hexa_fused_grad: null pointer");
    // ESMM task: j_x = j_y . w[e] with w [E][out][in] read as an [E][in'=out][out'=in] weight; the
    // slot layout is the mirror image of the forward's (shared j_y -> per-slot j_x and vice versa).
    int rc = hexa_esmm(j_x, j_y, w, nullptr, route, m2s, HEXA_W_IN_OUT, accumulate, T, k, out_dim, in_dim, E, act_dt,
                       w_dt, HEXA_F32, jx_dt, HEXA_ACT_NONE, nullptr, slot_ws, stream);
    if (rc) return rc;
    // ESTMM task: j_w[e][out][in] = sum j_y^T x
    rc = hexa_estmm(j_w, j_y, x, route, m2s ? 1 : 0, m2s ? 0 : 1, accumulate, T, k, out_dim, in_dim, E, act_dt, jw_dt,
                    plan, max_slots, estmm_scratch, stream);
    if (rc) return rc;
    if (j_b)
        rc = hexa_ess(j_b, j_y, route, m2s ? 1 : 0, accumulate, T, k, out_dim, E, act_dt, jb_dt, ess_ws,
                      ess_ws ? ess_ws_floats : 0, stream);
    return rc;
}

extern "C" int hexa_esmm_ess_ws_floats(int T, int k, int out_dim, int E, int64_t* out) {
    if (!out || T < 0 || k < 1 || out_dim < 1 || E < 1) HEXA_FAIL(HEXA_ERR_ARG, "hexa_esmm_ess_ws_floats: bad arguments");
    // one row of column sums per (slot, 128-row tile, column tile); also enough for hexa_ess's 8 parts
    const int64_t tiles = (int64_t)k * (T / HEXA_TILE_ROWS + E);
    const int64_t cols = ((int64_t)out_dim + 255) / 256 * 256;
    const int64_t a = tiles * cols, b = (int64_t)8 * E * out_dim;
    *out = a > b ? a : b;
    return HEXA_OK;
}

extern "C" int hexa_esmm_gelu_bwd_ess(void* out, void* db, const void* x, const void* w, const void* y1,
                                      const int32_t* route, int w_layout, int db_accumulate, int T, int k, int in_dim,
                                      int out_dim, int E, int x_dt, int w_dt, int db_dt, float* ws, int64_t ws_floats,
                                      void* stream) {
    if (int rc = check_sizes("hexa_esmm_gelu_bwd_ess", T, k, E, in_dim, out_dim)) return rc;
    if (!out || !db || !x || !w || !y1 || !route) HEXA_FAIL(HEXA_ERR_ARG, "hexa_esmm_gelu_bwd_ess: null pointer");
    if (!is_dt(x_dt) || !is_dt(w_dt) || !is_dt(db_dt)) HEXA_FAIL(HEXA_ERR_ARG, "hexa_esmm_gelu_bwd_ess: unknown element type");
    int64_t need = 0;
    hexa_esmm_ess_ws_floats(T, k, out_dim, E, &need);
    if (T > 0 && is_16(x_dt) && w_dt == x_dt && ws && ws_floats >= need && dma_path_enabled()) {
        EsmmArgs a;
        a.out = out; a.x = x; a.w = w; a.bias = nullptr; a.out_act = const_cast<void*>(y1); a.slot_ws = nullptr;
        a.r = route_view(route, T, k, E);
        a.in_dim = in_dim; a.out_dim = out_dim;
        a.x_per_slot = 0; a.out_per_slot = 1;
        a.w_layout = w_layout; a.accumulate = 0;
        a.x_dt = x_dt; a.w_dt = w_dt; a.bias_dt = HEXA_F32; a.out_dt = x_dt; a.act = HEXA_ACT_GELU_BWD;
        if (w_layout != HEXA_W_IN_OUT && w_layout != HEXA_W_OUT_IN)
            HEXA_FAIL(HEXA_ERR_ARG, "hexa_esmm_gelu_bwd_ess: bad w_layout %d", w_layout);
        if (esmm16_dma_colsum_supported(a)) {
            a.colsum = ws; a.db = db; a.db_dt = db_dt; a.db_accumulate = db_accumulate ? 1 : 0;
            return launch_esmm16_dma(a, (hipStream_t)stream);
        }
    }
    // any other case: the two operators one after the other (same results up to the order of the sums)
    int rc = hexa_esmm(out, x, w, nullptr, route, 0, w_layout, 0, T, k, in_dim, out_dim, E, x_dt, w_dt, HEXA_F32, x_dt,
                       HEXA_ACT_GELU_BWD, const_cast<void*>(y1), nullptr, stream);
    if (rc) return rc;
    return hexa_ess(db, out, route, 1, db_accumulate, T, k, out_dim, E, x_dt, db_dt, ws, ws ? ws_floats : 0, stream);
}

extern "C" int hexa_gelu_bwd(void* dy1, const void* dy2, const void* y1, int64_t n, int dt, void* stream) {
    if (n < 0 || (n > 0 && (!dy1 || !dy2 || !y1))) HEXA_FAIL(HEXA_ERR_ARG, "hexa_gelu_bwd: bad arguments");
    if (!is_dt(dt)) HEXA_FAIL(HEXA_ERR_ARG, "hexa_gelu_bwd: unknown element type");
    return launch_gelu_bwd(dy1, dy2, y1, n, dt, (hipStream_t)stream);
}
