// Several independent small kernels in ONE launch.  A batch is a list of up to four tasks (small_tasks.h); the
// batch kernel gives each task a contiguous range of workgroups (256 threads) and runs the task's own device code
// in them.  Only the combinations the backward of a MoE depth uses are instantiated, each with exactly the device
// code it needs, so a batch of elementwise tasks does not inherit the register budget of the gate products:
//   ESS + router backward | ESTMM fix-up + ESS fold | ESTMM fix-up + column-sum fold | slot sum + gate dwg reduction
// (The gate products stay a launch of their own: measured in one batch with the fix-up and the fold, 41.8 us against
// 23.4 + 10.8 + 6.2 apart -- every workgroup of a launch reserves the registers of its hungriest task, and at the
// gate products' 148 the memory-bound tasks no longer have the wavefronts in flight that they need.)
// Any other combination, a full batch or an element type without a batch kernel makes defer_task() return false
// and the task is launched on its own, as without a batch.  No counterpart in the reference.
#include "gate_bodies.h"
#include "small_bodies.h"

namespace hexa {
namespace {

struct BatchK {
    SmallTask t[BATCH_MAX_TASKS];
    int first[BATCH_MAX_TASKS + 1];
    int n;
};

template <typename T, unsigned MASK>
__global__ __launch_bounds__(256) void batch_kernel(BatchK b) {
    __shared__ float s_coef[(MASK & TASK_ROUTER_BWD) ? BATCH_ROUTER_BWD_MAX_E : 1];
    int i = 0;
#pragma unroll
    for (int q = 1; q < BATCH_MAX_TASKS; ++q) i += (q < b.n && (int)blockIdx.x >= b.first[q]) ? 1 : 0;
    const SmallTask& t = b.t[i];
    const int block = blockIdx.x - b.first[i];
    const unsigned kind = t.kind;            // uniform over the workgroup
    if ((MASK & TASK_ESS) && kind == TASK_ESS) ess_body<T>(t.ess, block);
    else if ((MASK & TASK_SUM_SLOTS) && kind == TASK_SUM_SLOTS) sum_slots_body<T>(t.sum_slots, block);
    else if ((MASK & TASK_FIXUP) && kind == TASK_FIXUP) estmm_fixup_body(t.fixup, block);
    else if ((MASK & TASK_ESS_FOLD) && kind == TASK_ESS_FOLD) ess_fold_body(t.ess_fold, block);
    else if ((MASK & TASK_COLSUM_FOLD) && kind == TASK_COLSUM_FOLD) colsum_fold_body(t.colsum_fold, block);
    else if ((MASK & TASK_DWG_REDUCE) && kind == TASK_DWG_REDUCE) dwg_reduce_body(t.dwg_reduce, block);
    else if ((MASK & TASK_ROUTER_BWD) && kind == TASK_ROUTER_BWD) router_bwd_body(s_coef, t.router_bwd, block);
}

constexpr unsigned MASK_A = TASK_ESS | TASK_ROUTER_BWD;
constexpr unsigned MASK_B = TASK_FIXUP | TASK_ESS_FOLD;
constexpr unsigned MASK_C = TASK_FIXUP | TASK_COLSUM_FOLD;
constexpr unsigned MASK_D = TASK_SUM_SLOTS | TASK_DWG_REDUCE;
constexpr unsigned MASK_E = TASK_ESS | TASK_ROUTER_BWD | TASK_FIXUP;          // the three-launch arrangement of the depth backward
constexpr unsigned MASK_F = TASK_ESS_FOLD | TASK_FIXUP | TASK_COLSUM_FOLD;

template <typename T, unsigned MASK>
int launch_batch(const BatchK& b, hipStream_t st) {
    hipLaunchKernelGGL((batch_kernel<T, MASK>), dim3(b.first[b.n]), dim3(256), 0, st, b);
    HEXA_CHECK_LAUNCH("batch");
    return HEXA_OK;
}

template <typename T>
int launch_batch_t(const BatchK& b, unsigned kinds, hipStream_t st) {
    if ((kinds & ~MASK_B) == 0) return launch_batch<T, MASK_B>(b, st);
    if ((kinds & ~MASK_D) == 0) return launch_batch<T, MASK_D>(b, st);
    if ((kinds & ~MASK_A) == 0) return launch_batch<T, MASK_A>(b, st);
    if ((kinds & ~MASK_C) == 0) return launch_batch<T, MASK_C>(b, st);
    if ((kinds & ~MASK_E) == 0) return launch_batch<T, MASK_E>(b, st);
    if ((kinds & ~MASK_F) == 0) return launch_batch<T, MASK_F>(b, st);
    HEXA_FAIL(HEXA_ERR_UNSUPPORTED, "batch: no kernel for the task combination 0x%x", kinds);
}

unsigned kinds_of(const SmallBatch& b) {
    unsigned k = 0;
    for (int i = 0; i < b.n; ++i) k |= b.t[i].kind;
    return k;
}

bool combination_ok(unsigned k) {
    return (k & ~MASK_A) == 0 || (k & ~MASK_B) == 0 || (k & ~MASK_C) == 0 || (k & ~MASK_D) == 0 || (k & ~MASK_E) == 0 || (k & ~MASK_F) == 0;
}

}  // namespace

bool batch_supported(int dt) { return dt == HEXA_BF16 || dt == HEXA_F16; }

DeferTargets& defer_targets() {
    static thread_local DeferTargets t;
    return t;
}

bool defer_task(SmallBatch* b, const SmallTask& t, int dt) {
    if (!b || b->full() || t.blocks <= 0) return false;
    if (dt >= 0 && dt != b->dt) return false;                       // a typed task of another element type
    if (!combination_ok(kinds_of(*b) | t.kind)) return false;
    b->t[b->n++] = t;
    return true;
}

int batch_flush(SmallBatch& sb, hipStream_t st) {
    if (sb.n == 0) return HEXA_OK;
    BatchK b;
    b.n = sb.n;
    b.first[0] = 0;
    for (int i = 0; i < sb.n; ++i) {
        b.t[i] = sb.t[i];
        b.first[i + 1] = b.first[i] + b.t[i].blocks;
    }
    for (int i = sb.n; i < BATCH_MAX_TASKS; ++i) b.first[i + 1] = b.first[sb.n];
    const unsigned kinds = kinds_of(sb);
    const int dt = sb.dt;
    sb.n = 0;
    return dt == HEXA_BF16 ? launch_batch_t<__bf16>(b, kinds, st) : launch_batch_t<_Float16>(b, kinds, st);
}

}  // namespace hexa
