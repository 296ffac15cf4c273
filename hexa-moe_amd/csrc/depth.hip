// One MoE depth per call: hexa_moe_depth_forward / hexa_moe_depth_backward enqueue every kernel of a depth
// (gate projection, softmax + top-k + auxiliary loss, routing segment pass, the ten steps of the formula table
// with the exact GELU) through the single-operator entry points of this library, in the order the Python layer
// used to call them.  Nothing here allocates: all scratch is carved out of one caller-owned workspace.
//
// Replaces the MoE branch of MoE_Cascaded.forward (hexa_moe_cuda/hexa_moe/impls/cascaded_moe.py:508-568),
// FusedMoE_Shared_CudaCore.forward (impls/layers.py:99-277) and .backward (impls/layers.py:280-474).
#include <algorithm>
#include <mutex>

#include "small_tasks.h"

namespace hexa {
namespace {

constexpr int64_t WS_ALIGN = 256;

int64_t elem_size(int dt) { return dt == HEXA_F32 ? 4 : 2; }
bool known_dt(int dt) { return dt == HEXA_F32 || dt == HEXA_F16 || dt == HEXA_BF16; }

struct Carver {   // hands out aligned pieces of the workspace; with base == nullptr it only measures
    char* base; int64_t used = 0;
    explicit Carver(void* b) : base(static_cast<char*>(b)) {}
    void* take(int64_t bytes) {
        void* p = base ? base + used : nullptr;
        used += (bytes + WS_ALIGN - 1) / WS_ALIGN * WS_ALIGN;
        return p;
    }
};

// ESTMM scratch slots for the partial results of experts whose lists are cut (up to E slots, at most 128 MiB per
// result, only for 16-bit operands with long enough lists)
int estmm_slots(const hexa_moe_depth_desc& d, int out_dim, int in_dim) {
    if (d.act_dt == HEXA_F32 || (int64_t)d.num_tokens * d.top_k < (int64_t)128 * d.num_experts) return 0;
    const int64_t mn = (int64_t)out_dim * in_dim;
    if (mn % 4) return 0;
    const int64_t slots = std::min<int64_t>(d.num_experts, ((int64_t)128 << 20) / (mn * 4));
    return slots >= 2 ? (int)slots : 0;
}

// A second stream and the events that tie it to the caller's, made once per device (default priority; the first call
// on a device must not be under stream capture).  The small kernels of the backward are bound by their latency
// chains, not by the chip: beside the matmul kernels they cost next to nothing.
struct SideStream { hipStream_t st = nullptr; hipEvent_t ev[4] = {nullptr, nullptr, nullptr, nullptr}; bool ok = false, tried = false; };
SideStream* side_stream() {
    static SideStream per_device[64];
    static std::mutex mu;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return nullptr;
    std::lock_guard<std::mutex> lock(mu);
    SideStream& s = per_device[dev];
    if (!s.tried) {
        s.tried = true;
        bool ok = hipStreamCreateWithFlags(&s.st, hipStreamNonBlocking) == hipSuccess;
        for (int i = 0; ok && i < 4; ++i) ok = hipEventCreateWithFlags(&s.ev[i], hipEventDisableTiming) == hipSuccess;
        if (!ok) (void)hipGetLastError();
        s.ok = ok;
    }
    return s.ok ? &s : nullptr;
}

struct FwdWs { float* router; int32_t* hist; void* slot_ws; int64_t bytes; };
struct BwdWs {
    float* dlogits; float* gate; float* ess; float* colsum; int64_t colsum_floats; int32_t* plan; float* estmm; float* estmm2;
    int slots; void* slot_ws; void* dx_gate; int64_t bytes;
};

int carve_forward(const hexa_moe_depth_desc& d, void* ws, FwdWs* out) {
    Carver c(ws);
    int64_t rf = 0;
    if (int rc = hexa_router_ws_floats(d.num_tokens, d.num_experts, &rf)) return rc;
    out->router = static_cast<float*>(c.take(rf * 4));
    // the routing pass's histogram over the router's workgroups (64 tokens each), counted by the router itself
    out->hist = static_cast<int32_t*>(c.take((int64_t)d.top_k * div_up(std::max(d.num_tokens, 1), router_tokens_per_workgroup()) *
                                              d.num_experts * 4));
    out->slot_ws = d.top_k > 1 ? c.take((int64_t)(d.top_k - 1) * d.num_tokens * d.d_out * elem_size(d.act_dt)) : nullptr;
    out->bytes = c.used;
    return HEXA_OK;
}

int carve_backward(const hexa_moe_depth_desc& d, void* ws, BwdWs* out) {
    Carver c(ws);
    const int T = d.num_tokens, k = d.top_k, E = d.num_experts;
    int64_t gf = 0, cf = 0;
    if (int rc = hexa_gate_ws_floats(T, d.d_in, E, &gf)) return rc;
    if (int rc = hexa_esmm_ess_ws_floats(T, k, d.hidden, E, &cf)) return rc;
    out->dlogits = static_cast<float*>(c.take((int64_t)T * E * 4));
    out->gate = static_cast<float*>(c.take(gf * 4));
    out->ess = static_cast<float*>(c.take((int64_t)8 * E * d.d_out * 4));
    out->colsum = static_cast<float*>(c.take(cf * 4));
    out->colsum_floats = cf;
    // one plan serves both ESTMM calls; each has a scratch area of its own (the fix-up of the first may run on the
    // side stream while the second call's kernel writes its partial results)
    const int s2 = estmm_slots(d, d.hidden, d.d_out), s1 = estmm_slots(d, d.hidden, d.d_in);
    out->slots = std::min(s1, s2);
    out->plan = static_cast<int32_t*>(c.take((int64_t)HEXA_ESTMM_PLAN_INTS(E) * 4));
    out->estmm = out->slots >= 2 ? static_cast<float*>(c.take((int64_t)out->slots * d.hidden * d.d_out * 4)) : nullptr;
    out->estmm2 = out->slots >= 2 ? static_cast<float*>(c.take((int64_t)out->slots * d.hidden * d.d_in * 4)) : nullptr;
    out->slot_ws = k > 1 ? c.take((int64_t)(k - 1) * T * d.d_in * elem_size(d.act_dt)) : nullptr;
    out->dx_gate = c.take((int64_t)T * d.d_in * elem_size(d.act_dt));
    out->bytes = c.used;
    return HEXA_OK;
}

int check_desc(const char* who, const hexa_moe_depth_desc* d) {
    if (!d) HEXA_FAIL(HEXA_ERR_ARG, "%s: null descriptor", who);
    if (d->num_tokens < 1 || d->top_k < 1 || d->num_experts < 1 || d->d_in < 1 || d->hidden < 1 || d->d_out < 1)
        HEXA_FAIL(HEXA_ERR_ARG, "%s: bad sizes T=%d k=%d E=%d dims=(%d,%d,%d)", who, d->num_tokens, d->top_k,
                  d->num_experts, d->d_in, d->hidden, d->d_out);
    if (d->top_k > d->num_experts) HEXA_FAIL(HEXA_ERR_ARG, "%s: top_k exceeds the number of experts", who);
    if (!known_dt(d->act_dt) || !known_dt(d->w_dt)) HEXA_FAIL(HEXA_ERR_ARG, "%s: unknown element type", who);
    if (d->loss != 0 && d->loss != 1) HEXA_FAIL(HEXA_ERR_ARG, "%s: loss must be 0 (GShard) or 1 (load-importance)", who);
    return HEXA_OK;
}

struct EventPairs {   // caller-owned events recorded around the major kernels (null handles are skipped)
    void* const* ev; int n; hipStream_t st;
    int begin(int i) const {
        if (ev && 2 * i + 1 < n && ev[2 * i] && hipEventRecord((hipEvent_t)ev[2 * i], st) != hipSuccess)
            HEXA_FAIL(HEXA_ERR_LAUNCH, "hipEventRecord failed");
        return HEXA_OK;
    }
    int end(int i) const {
        if (ev && 2 * i + 1 < n && ev[2 * i + 1] && hipEventRecord((hipEvent_t)ev[2 * i + 1], st) != hipSuccess)
            HEXA_FAIL(HEXA_ERR_LAUNCH, "hipEventRecord failed");
        return HEXA_OK;
    }
};

}  // namespace
}  // namespace hexa

using namespace hexa;

#define RUN(call)                 \
    do {                          \
        if (int rc__ = (call)) return rc__; \
    } while (0)

extern "C" int hexa_moe_depth_ws_bytes(const hexa_moe_depth_desc* d, int64_t* forward_bytes, int64_t* backward_bytes) {
    RUN(check_desc("hexa_moe_depth_ws_bytes", d));
    if (forward_bytes) {
        FwdWs f;
        RUN(carve_forward(*d, nullptr, &f));
        *forward_bytes = std::max<int64_t>(f.bytes, WS_ALIGN);
    }
    if (backward_bytes) {
        BwdWs b;
        RUN(carve_backward(*d, nullptr, &b));
        *backward_bytes = std::max<int64_t>(b.bytes, WS_ALIGN);
    }
    return HEXA_OK;
}

extern "C" int hexa_moe_depth_forward(const hexa_moe_depth_desc* d, const void* x, const float* wg, const float* noise,
                                      const void* fc1_w, const void* fc1_b, const void* fc2_w, const void* fc2_b,
                                      float* logits, float* scores, int32_t* idx, float* thr, float* stats,
                                      int32_t* route, int32_t* plan, void* y1, void* y2, void* y, void* ws,
                                      int64_t ws_bytes, void* const* events, int num_events, void* stream) {
    const char* who = "hexa_moe_depth_forward";
    RUN(check_desc(who, d));
    if (!x || !fc1_w || !fc2_w || !idx || !route || !y1 || !y2 || !y || !ws) HEXA_FAIL(HEXA_ERR_ARG, "%s: null pointer", who);
    if (((uintptr_t)ws & (WS_ALIGN - 1)) != 0) HEXA_FAIL(HEXA_ERR_ARG, "%s: the workspace must be 256-byte aligned", who);
    FwdWs w;
    RUN(carve_forward(*d, ws, &w));
    if (ws_bytes < w.bytes) HEXA_FAIL(HEXA_ERR_ARG, "%s: workspace of %lld bytes, %lld needed", who, (long long)ws_bytes, (long long)w.bytes);
    const int T = d->num_tokens, k = d->top_k, E = d->num_experts;
    const EventPairs ev{events, num_events, (hipStream_t)stream};
    // the work plan of the backward's ESTMM calls depends on the routing only: made here when the caller keeps it
    // (without scratch slots it cuts no expert, but still orders the work and carries the persistent kernel's queue)
    const int plan_slots = std::min(estmm_slots(*d, d->hidden, d->d_out), estmm_slots(*d, d->hidden, d->d_in));
    if (plan && d->act_dt == HEXA_F32) plan = nullptr;
    const int plan_cap = estmm_plan_cap_for(route_view(route, T, k, E), d->hidden, std::min(d->d_in, d->d_out));
    bool routed = false;
    if (wg) {
        if (!logits || !scores || !stats || (d->loss == 1 && !thr)) HEXA_FAIL(HEXA_ERR_ARG, "%s: null router state", who);
        const bool front3 = d->loss == 0 && router_hist_supported(E);
        const bool one_launch = front3 && option(OPT_GATE_ROUTER) != 2 && T > 0 && gate_router_supported(d->d_in, E, d->act_dt);
        if (!one_launch) RUN(hexa_gate_logits(logits, x, wg, T, d->d_in, E, d->act_dt, stream));
        if (front3) {
            // two launches for gate, router, loss, routing pass and plan: the gate's logits go straight into the
            // router's tile (a launch of its own above GATE_ROUTER_MAX_E experts), the router counts its own tokens for
            // the routing pass, whose one launch also carries the loss and the plan (above 256 experts, or with option
            // "route_kernels" = 3: a scan launch with the loss and a scatter launch with the plan)
            RUN(router_forward_check(T, E, k, true));
            if (one_launch)
                RUN(launch_gate_router(logits, scores, idx, x, wg, noise, d->noise_scale, T, d->d_in, E, k, d->act_dt, w.router,
                                       w.hist, (hipStream_t)stream));
            else
                RUN(launch_router_fwd(scores, idx, logits, noise, d->noise_scale, T, E, k, w.router, w.hist, (hipStream_t)stream));
            RUN(launch_route_from_hist(idx, T, k, E, route, w.hist, router_tokens_per_workgroup(), stats + 2 * E, stats,
                                       stats + E, w.router, plan, plan_slots, plan_cap, (hipStream_t)stream));
            routed = true;
        } else if (d->loss == 0) {
            RUN(hexa_router_forward(scores, idx, stats, stats + E, stats + 2 * E, logits, noise, d->noise_scale, T, E, k,
                                    w.router, stream));
        } else {
            RUN(hexa_router_forward_load_importance(scores, idx, thr, stats, stats + E, stats + 2 * E, stats + 3 * E,
                                                    stats + 4 * E, logits, noise, d->noise_scale, d->sigma, T, E, k,
                                                    w.router, stream));
        }
    }
    if (!routed) {
        RUN(hexa_route_build(idx, 0, k, 1, T, k, E, route, stream));
        if (plan) RUN(launch_estmm_plan(plan, route_view(route, T, k, E), plan_slots, plan_cap, (hipStream_t)stream));
    }
    if (option(OPT_FFN_FUSED) == 1 && dma_path_enabled() &&
        ffn16_fused_supported(T, k, d->d_in, d->hidden, d->d_out, d->act_dt, d->w_dt, d->b1_dt, d->b2_dt)) {
        // fc1, GELU and fc2 in one kernel: event pair 0 brackets it (and the slot sum), pair 1 stays empty
        RUN(ev.begin(0));
        RUN(launch_ffn16_fused(y1, y2, y, x, fc1_w, fc1_b, fc2_w, fc2_b, route_view(route, T, k, E), d->d_in, d->hidden,
                               d->d_out, d->act_dt, d->b1_dt, d->b2_dt, w.slot_ws, (hipStream_t)stream));
        RUN(ev.end(0));
        RUN(ev.begin(1));
        RUN(ev.end(1));
        return HEXA_OK;
    }
    RUN(ev.begin(0));
    RUN(hexa_esmm(y1, x, fc1_w, fc1_b, route, 0, HEXA_W_OUT_IN, 0, T, k, d->d_in, d->hidden, E, d->act_dt, d->w_dt,
                  d->b1_dt, d->act_dt, HEXA_ACT_GELU, y2, nullptr, stream));
    RUN(ev.end(0));
    RUN(ev.begin(1));
    RUN(hexa_esmm(y, y2, fc2_w, fc2_b, route, 1, HEXA_W_IN_OUT, 0, T, k, d->hidden, d->d_out, E, d->act_dt, d->w_dt,
                  d->b2_dt, d->act_dt, HEXA_ACT_NONE, nullptr, w.slot_ws, stream));
    RUN(ev.end(1));
    return HEXA_OK;
}

extern "C" int hexa_moe_depth_backward(const hexa_moe_depth_desc* d, const void* dy, const float* grad_l_aux,
                                       const void* x, const float* wg, const void* fc1_w, const void* fc2_w,
                                       const float* scores, const int32_t* idx, const float* thr, const float* stats,
                                       const int32_t* route, int32_t* plan, const void* y1, const void* y2,
                                       void* dx, float* dwg, void* dw1, void* db1, void* dw2, void* db2, void* dy1,
                                       void* ws, int64_t ws_bytes, void* const* events, int num_events, void* stream) {
    const char* who = "hexa_moe_depth_backward";
    RUN(check_desc(who, d));
    if (!dy || !x || !fc1_w || !fc2_w || !route || !y1 || !y2 || !dy1 || !ws) HEXA_FAIL(HEXA_ERR_ARG, "%s: null pointer", who);
    if (((uintptr_t)ws & (WS_ALIGN - 1)) != 0) HEXA_FAIL(HEXA_ERR_ARG, "%s: the workspace must be 256-byte aligned", who);
    BwdWs w;
    RUN(carve_backward(*d, ws, &w));
    if (ws_bytes < w.bytes) HEXA_FAIL(HEXA_ERR_ARG, "%s: workspace of %lld bytes, %lld needed", who, (long long)ws_bytes, (long long)w.bytes);
    const int T = d->num_tokens, k = d->top_k, E = d->num_experts;
    const EventPairs ev{events, num_events, (hipStream_t)stream};
    const bool gate_path = wg && grad_l_aux && (dx || dwg);
    if (gate_path && (!scores || !stats || (d->loss == 1 && (!thr || !idx)))) HEXA_FAIL(HEXA_ERR_ARG, "%s: null router state", who);

    // The second-stage and elementwise kernels of this call are independent of most of what surrounds them, and a
    // launch of its own costs each of them 5-7 us: where the element type has a batch kernel they are collected
    // as tasks and run three launches instead of nine, each placed where the stream order allows:
    //   B  ESS(dy) partial sums, router backward, fix-up of dW2     -- behind ESTMM dW2 (the scratch is reused by dW1)
    //   C  fold of the ESS partial sums, fix-up of dW1, fold of db1's column sums   -- behind ESTMM dW1 and the gate
    //   D  slot sum of dx (+ the gate's share), gate dwg fold       -- behind the dx kernel
    // (option "batch" = 1 keeps ESS(dy) and the router backward in a launch of their own at the start, A, and the ESS
    // fold in B: four launches.)
    // A launcher that cannot put its task into the batch offered (other element type, general kernels) launches it
    // on the spot, which is always in order.
    const bool batching = batch_supported(d->act_dt) && option(OPT_BATCH) != 2;
    const bool early_a = option(OPT_BATCH) == 1;
    SmallBatch A, B, C, D;
    A.dt = B.dt = C.dt = D.dt = d->act_dt;
    struct Guard { ~Guard() { defer_targets() = DeferTargets(); } } guard;
    DeferTargets& tg = defer_targets();
    hipStream_t st = (hipStream_t)stream;
    // With the side stream the batches B and C and the gate's backward run beside the matmul kernels:
    //   caller's stream:  ESTMM dW2 | dy1 kernel | ESTMM dW1 |            dx kernel | D
    //   side stream:                 B | gate backward        | C
    // B waits for ESTMM dW2 (event 0), the dx kernel for the gate's backward (event 1), C for ESTMM dW1 (event 2), the
    // caller's stream for C (event 3) before the call's last launch.
    SideStream* side = batching && !early_a && option(OPT_SIDE_STREAM) == 1 ? side_stream() : nullptr;
    hipStream_t sst = side ? side->st : st;
    auto hand_over = [&](int i, hipStream_t from, hipStream_t to) -> int {   // `to` continues behind what `from` holds now
        if (!side) return HEXA_OK;
        if (hipEventRecord(side->ev[i], from) != hipSuccess || hipStreamWaitEvent(to, side->ev[i], 0) != hipSuccess)
            HEXA_FAIL(HEXA_ERR_LAUNCH, "hexa_moe_depth_backward: event hand-over between the streams failed");
        return HEXA_OK;
    };

    // step 4: db2 = ESS(dy)
    if (db2) {
        if (batching) { tg.ess = early_a ? &A : &B; tg.ess_fold = early_a ? &B : &C; }
        RUN(hexa_ess(db2, dy, route, 0, 0, T, k, d->d_out, E, d->act_dt, d->gb2_dt, w.ess, (int64_t)8 * E * d->d_out, stream));
        tg = DeferTargets();
    }
    // the gate path, part 1: d l_aux / d logits through the softmax (and the threshold)
    if (gate_path) {
        if (batching) tg.router_bwd = early_a ? &A : &B;
        if (d->loss == 0)
            RUN(hexa_router_backward(w.dlogits, scores, stats + E, grad_l_aux, T, E, stream));
        else
            RUN(hexa_router_backward_load_importance(w.dlogits, scores, thr, idx, stats + 2 * E, stats + 3 * E, grad_l_aux,
                                                     d->sigma, T, E, k, stream));
        tg = DeferTargets();
    }
    RUN(batch_flush(A, st));
    const bool planned = d->act_dt != HEXA_F32 && (dw1 || dw2);
    if (planned && !plan)
        RUN(launch_estmm_plan(w.plan, route_view(route, T, k, E), w.slots,
                              estmm_plan_cap_for(route_view(route, T, k, E), d->hidden, std::min(d->d_in, d->d_out)), st));
    if (planned && plan) w.plan = plan;   // made by the forward for the same routing and slot count
    // step 5: dW2 = ESTMM(act(y1), dy): the per-slot operand supplies the rows of dW2 [E][hidden][d_out]
    if (dw2) {
        if (batching) tg.fixup = &B;
        RUN(ev.begin(2));
        RUN(hexa_estmm(dw2, y2, dy, route, 1, 0, 0, T, k, d->hidden, d->d_out, E, d->act_dt, d->gw2_dt,
                       planned ? w.plan : nullptr, planned ? w.slots : 0, planned && w.slots >= 2 ? w.estmm : nullptr, stream));
        RUN(ev.end(2));
        tg = DeferTargets();
    }
    RUN(hand_over(0, st, sst));
    RUN(batch_flush(B, sst));
    if (dx || dw1 || db1) {
        // steps 6-8: dy1 = (dy . W2^T) * gelu'(y1), db1 = ESS(dy1)
        if (batching) tg.colsum_fold = &C;
        RUN(ev.begin(0));
        if (db1)
            RUN(hexa_esmm_gelu_bwd_ess(dy1, db1, dy, fc2_w, y1, route, HEXA_W_OUT_IN, 0, T, k, d->d_out, d->hidden, E,
                                       d->act_dt, d->w_dt, d->gb1_dt, w.colsum, w.colsum_floats, stream));
        else
            RUN(hexa_esmm(dy1, dy, fc2_w, nullptr, route, 0, HEXA_W_OUT_IN, 0, T, k, d->d_out, d->hidden, E, d->act_dt,
                          d->w_dt, HEXA_F32, d->act_dt, HEXA_ACT_GELU_BWD, const_cast<void*>(y1), nullptr, stream));
        RUN(ev.end(0));
        tg = DeferTargets();
        // step 9: dW1 = ESTMM(dy1, x)
        if (dw1) {
            if (batching) tg.fixup = &C;
            RUN(ev.begin(3));
            RUN(hexa_estmm(dw1, dy1, x, route, 1, 0, 0, T, k, d->hidden, d->d_in, E, d->act_dt, d->gw1_dt,
                           planned ? w.plan : nullptr, planned ? w.slots : 0, planned && w.slots >= 2 ? w.estmm2 : nullptr, stream));
            RUN(ev.end(3));
            tg = DeferTargets();
        }
    }
    // the gate path, part 2: through the projection
    bool gate_dx_in_ws = false;
    if (gate_path) {
        // With several slots on the 16-bit fast path the slot sum of step 10 adds the gate's share as one more
        // addend; otherwise the gate's share is written into dx first and step 10 accumulates onto it.
        // (decided with the predicate step 10's call itself applies, so a shape the fast path does not cover --
        // operands of 4 GiB and more, odd dimensions -- falls back instead of failing)
        gate_dx_in_ws = dx && esmm_slot_sum_takes_extra(route, HEXA_W_IN_OUT, T, k, d->hidden, d->d_in, E, d->act_dt, d->w_dt,
                                                        d->act_dt, w.slot_ws);
        if (batching) tg.dwg_reduce = &D;
        RUN(hexa_gate_backward(dx ? (gate_dx_in_ws ? w.dx_gate : dx) : nullptr, dwg, w.dlogits, x, wg, T, d->d_in, E,
                               d->act_dt, w.gate, sst));
        tg = DeferTargets();
    }
    RUN(hand_over(1, sst, st));
    RUN(hand_over(2, st, sst));
    RUN(batch_flush(C, sst));
    // step 10: dx = ESMM(dy1, W1), summed over the slots (+ the gate's share)
    if (dx) {
        if (batching) tg.sum_slots = &D;
        RUN(ev.begin(1));
        bool used = false;
        const int acc = gate_path && !gate_dx_in_ws ? 1 : 0;
        RUN(esmm_call(dx, dy1, fc1_w, nullptr, route, 1, HEXA_W_IN_OUT, acc, T, k, d->hidden, d->d_in, E, d->act_dt,
                      d->w_dt, HEXA_F32, d->act_dt, HEXA_ACT_NONE, nullptr, w.slot_ws, gate_dx_in_ws ? w.dx_gate : nullptr,
                      &used, stream));
        if (gate_dx_in_ws && !used) HEXA_FAIL(HEXA_ERR_LAUNCH, "%s: internal: the gate's input gradient was not added", who);
        RUN(ev.end(1));
        tg = DeferTargets();
    }
    RUN(batch_flush(D, st));
    RUN(hand_over(3, sst, st));
    return HEXA_OK;
}
