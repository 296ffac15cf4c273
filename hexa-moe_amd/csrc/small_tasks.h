// Small kernels as TASKS: argument blocks of the second-stage and elementwise kernels of a MoE depth, so that
// several independent ones can share one launch (batch.hip).  Every launch of a small kernel costs 5-7 us of the
// step whatever it computes, and the backward of a depth has ten of them.  A launcher that finds a batch
// registered for its kind of task (DeferTargets, per host thread) appends the task there instead of launching;
// whoever registered the batch launches it where the stream order allows.
#pragma once
#include "hexa_internal.h"

namespace hexa {

struct EssK {
    const void* dy; void* db;
    const int32_t* token_ids; const int32_t* offsets;
    int T, k, E, N, dy_slot_rows, accumulate, db_dt;
    float* ws; int splits;   // splits > 1: workgroup z sums the z-th part of every segment into ws[z][E][N]
    int gx, gy;              // grid: (column strips, experts, splits)
};
struct EssFoldK { void* db; const float* ws; long n; int splits, db_dt, accumulate; };
struct RouterBwdK { float* dlogits; const float* scores; const float* ce; const float* grad_l; int T, E; };
struct FixupK { void* dw; const int* plan; const float* scratch; int E; long mn; int dw_dt, accumulate, gx; };
struct ColsumFoldK {
    void* db; const float* colsum; const int32_t* offsets;
    int E, mt_ub, tile_rows, ntn, bn, N, nslots, db_dt, accumulate, gx;
};
struct SumSlotsK { void* out; const void* ws; int64_t n; int nws; const void* extra; int blocks; };
struct GateBwdK { void* dx; float* part; const float* dl; const void* x; const float* wg; int T, d, E, ntasks; };
struct DwgReduceK { float* dwg; const float* part; int nparts; long n4; };

enum SmallKind : unsigned {
    TASK_ESS = 1u, TASK_ESS_FOLD = 2u, TASK_ROUTER_BWD = 4u, TASK_FIXUP = 8u, TASK_COLSUM_FOLD = 16u,
    TASK_SUM_SLOTS = 32u, TASK_DWG_REDUCE = 64u
};

struct SmallTask {
    unsigned kind; int blocks;
    union {
        EssK ess; EssFoldK ess_fold; RouterBwdK router_bwd; FixupK fixup; ColsumFoldK colsum_fold; SumSlotsK sum_slots;
        DwgReduceK dwg_reduce;
    };
};

constexpr int BATCH_MAX_TASKS = 4;
constexpr int BATCH_ROUTER_BWD_MAX_E = 1024;   // LDS the batch kernel sets aside for the router backward's coefficients
struct SmallBatch {
    SmallTask t[BATCH_MAX_TASKS];
    int n = 0;
    int dt = HEXA_BF16;          // element type of the token tensors of the typed tasks (ESS, slot sum)
    bool full() const { return n >= BATCH_MAX_TASKS; }
};
// one launch for the tasks collected so far (none: nothing happens); the batch is empty afterwards
int batch_flush(SmallBatch& b, hipStream_t st);
// which element types / task combinations batch_flush has a kernel for
bool batch_supported(int dt);

// Where the launchers of this host thread put their tasks instead of launching (null: launch as usual).
struct DeferTargets {
    SmallBatch* ess = nullptr; SmallBatch* ess_fold = nullptr; SmallBatch* router_bwd = nullptr;
    SmallBatch* fixup = nullptr; SmallBatch* colsum_fold = nullptr; SmallBatch* sum_slots = nullptr;
    SmallBatch* dwg_reduce = nullptr;
};
DeferTargets& defer_targets();
// appends when a batch is registered, of the right element type and not full; false: the caller launches itself
bool defer_task(SmallBatch* b, const SmallTask& t, int dt = -1);

}  // namespace hexa
