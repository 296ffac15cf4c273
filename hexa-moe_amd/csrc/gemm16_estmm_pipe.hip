// Persistent, role-split ESTMM for bf16 / fp16 on gfx950: dw[e][m][n] = sum over the expert's routed rows of
// P[row][m] * Q[row][n].  One workgroup per CU takes work items -- a 128 x 128 block of one expert's result (or of
// one part of a busy expert) -- from a queue until the queue is empty, and its wavefronts have roles, as in the
// pipelined ESMM kernel (gemm16_pipe.hip):
//
//   * 4 "multiply" wavefronts (2 x 2, 64 x 64 results each): transposing LDS fragment reads and MFMAs only;
//   * 4 "copy" wavefronts issue every asynchronous global->LDS copy: both operands are gathered by token id, 64
//     tokens per stage, three stages deep, and the pipeline never drains between items -- the first stages of the
//     next item are in flight while the current one finishes; the token ids travel through an LDS ring, fetched seven
//     steps before the step they belong to;
//   * 4 "store" wavefronts write the previous item's result (staged in LDS by the multiply wavefronts) while the
//     next item is being multiplied;
//   * 1 "scheduler" wavefront pops the queue up to 24 steps ahead (one atomic per batch of items, its latency hidden
//     behind the steps in between) and publishes item records in LDS for the other roles.
//
// The queue is eight counters, one per XCD: the items (heaviest expert first, as the plan orders them) are dealt to
// the XCDs in runs that share token rows, a workgroup pops its own XCD's counter and moves on to the next XCD's when
// that is used up, so the load balances over the whole chip while an expert's rows stay in few L2s.  Because an
// item is summed by one workgroup in list order, and a split expert's parts are added by the fix-up task in part
// order, the result does not depend on which workgroup took what: bit-reproducible.
//
// With items taken longest-first by whoever is free, an expert only has to be cut into parts when one of its items
// would be longer than a workgroup's share of the whole launch (see estmm_plan_cap); at large shapes no expert is
// cut, nothing is written as an fp32 partial result and the fix-up task has nothing to do.
//
// The counters live behind the plan (hexa_estmm_plan zeroes them); the last workgroup to finish puts them back to
// zero, so launches that share a plan must not overlap.
//
// Replaces the ESTMM task of fused_grad_*_kernel_vectorized_half (kernels/fused_ops_half.cu) where it applies:
// 16-bit operands, a plan, up to 256 experts and 8 slots, operands below 4 GiB.
#include <algorithm>

#include "pipe_common.h"
#include "small_bodies.h"

namespace hexa {
namespace {

using CfgE = Cfg<2, 2, 2, 2, 3, 3, 64>;     // 128 x 128, 4 multiply wavefronts of 64 x 64, 3 stages of 64 tokens
constexpr int EP_MUL = 4, EP_COPY = 4, EP_STORE = 4, EP_WAVES = EP_MUL + EP_COPY + EP_STORE + 1, EP_NT = 64 * EP_WAVES;
constexpr int EP_IDS_RING = 8;              // steps of token ids in LDS
constexpr int EP_IDS_AHEAD = 7;             // steps the ids are fetched ahead of the step they belong to
constexpr int EP_REC_RING = 32;             // item records in LDS
constexpr int EP_REC_INTS = 32;
constexpr int EP_LOOK = 24;                 // steps the scheduler runs ahead of the step being multiplied
constexpr int EP_WAIT = 5;                  // steps after which a memory operation of the scheduler is taken to be back
constexpr int EP_NEED = 9;                  // steps that must be covered by published records at every barrier
constexpr int EP_MAX_E = 256, EP_MAX_K = 8;

// item record: what every role needs to know about one work item
enum { R_E = 0, R_M0, R_N0, R_NSTEPS, R_POS0, R_POS1, R_SLOT, R_F32, R_CUM = 8, R_TB = 16 };
// R_NSTEPS < 0: no more items.  R_SLOT: scratch slot of the partial result (-1: the result itself).  R_F32: the item's
// result leaves as fp32 (partial result or fp32 dw).  R_CUM[s]: rows of the expert's list before slot s.
// R_TB[s]: position p of the list (in slot s) holds token_ids[p + R_TB[s]].

struct EstmmPipeK {
    const void* pm; const void* qm; void* dw;
    const int32_t* token_ids; const int32_t* offsets;
    const int32_t* plan; int32_t* queue; float* scratch;
    int T, k, E, M, N, mtn, ntn, group;
    int p_slot_rows, q_slot_rows, accumulate, stream_dw, wg_per_xcd, out32;
    int batch;       // items per pop of the queue (short lists: several, so that one atomic's latency buys enough steps)
};

struct EpLds {
    using C = CfgE;
    static constexpr int CP = C::BN * 2 + 16;           // pitch of a staged 16-bit row
    static constexpr int CPF = C::BN * 4 + 16;          // pitch of a staged fp32 row (half a tile at a time)
    static constexpr int STAGES_AT = 0;
    static constexpr int STAGING_AT = STAGES_AT + C::STAGE_AREA;
    static constexpr int STAGING_BYTES = C::BM * CP;
    static_assert((C::BM / 2) * CPF <= STAGING_BYTES, "half a tile of fp32 rows fits the staging area");
    static constexpr int IDS_AT = STAGING_AT + STAGING_BYTES;
    static constexpr int REC_AT = IDS_AT + EP_IDS_RING * 64 * 4;
    static constexpr int PLAN_AT = REC_AT + EP_REC_RING * EP_REC_INTS * 4;
    static constexpr int OFFS_AT = PLAN_AT + 4 * EP_MAX_E * 4;
    static constexpr int BYTES = OFFS_AT + EP_MAX_K * (EP_MAX_E + 1) * 4;
    static_assert(BYTES <= 160 * 1024, "LDS of a CU");
};

__device__ __forceinline__ int uni(int v) { return __builtin_amdgcn_readfirstlane(v); }

// KS: upper bound of the number of routing slots (1, 2, 4 or 8): the copy wavefronts find a list position's slot by comparing
// it with the KS - 1 boundaries
template <typename TC, bool OUT32, int KS>
__global__ __launch_bounds__(EP_NT) void estmm16_pipe_kernel(EstmmPipeK p) {
    using C = CfgE;
    using L = EpLds;
    constexpr int BM = C::BM, BN = C::BN, STAGES = C::STAGES, BKT = C::BKC;     // BKT tokens per stage
    constexpr int CW = EP_COPY;
    constexpr int R_CPW = C::R_COPIES / CW, F_CPW = C::F_COPIES / CW, CPW = R_CPW + F_CPW;
    static_assert(R_CPW == F_CPW && BM == BN, "the two operands are copied alike");
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    const unsigned lds0 = lds_addr(smem);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = uni(tid >> 6);
    const int E = p.E, nslot = p.k, M = p.M, N = p.N;
    const int tiles = p.mtn * p.ntn;

    int* sPlan = reinterpret_cast<int*>(smem + L::PLAN_AT);        // [4][E]: expert, parts, first unit, first slot (by rank)
    int* sOffs = reinterpret_cast<int*>(smem + L::OFFS_AT);        // [k][E + 1]
    int* sRec = reinterpret_cast<int*>(smem + L::REC_AT);
    for (int i = tid; i < 4 * E; i += EP_NT) sPlan[i] = p.plan[i];
    for (int i = tid; i < nslot * (E + 1); i += EP_NT) sOffs[i] = p.offsets[i];
    const int units = uni(p.plan[4 * E]);
    const int total = units * tiles;
    __syncthreads();                                     // (P0) the tables are in LDS

    // Record j, the same in every lane.  The reads are inline assembly (a compiler-visible LDS read next to
    // asynchronous copies in flight would be ordered behind them) and share one wait.
    struct Rec { int f[EP_REC_INTS]; };
    auto load_rec = [&](int j) {
        u32x4 v[EP_REC_INTS / 4];
        const unsigned at = lds0 + L::REC_AT + (j % EP_REC_RING) * (EP_REC_INTS * 4);
        static_for<EP_REC_INTS / 4>([&](auto ic) {
            constexpr int i = decltype(ic)::value;
            v[i] = lds_read128_async<i * 16>(at);
        });
        lds_wait();
        Rec r;
#pragma unroll
        for (int i = 0; i < EP_REC_INTS / 4; ++i) {
            asm volatile("" : "+v"(v[i]));
            r.f[4 * i] = uni((int)v[i].x); r.f[4 * i + 1] = uni((int)v[i].y);
            r.f[4 * i + 2] = uni((int)v[i].z); r.f[4 * i + 3] = uni((int)v[i].w);
        }
        return r;
    };

    struct Cur {       // a walk over the global steps: the item it is in and the step inside it
        int rec, kt, nsteps, pos0, pos1, m0, n0;
        int cum[KS], tb[KS];
    };
    auto load_cur = [&](Cur& c) {
        const Rec rc = load_rec(c.rec);
        c.kt = 0;
        c.nsteps = rc.f[R_NSTEPS];
        if (c.nsteps < 0) return;
        c.pos0 = rc.f[R_POS0]; c.pos1 = rc.f[R_POS1];
        c.m0 = rc.f[R_M0]; c.n0 = rc.f[R_N0];
#pragma unroll
        for (int s = 0; s < KS; ++s) { c.cum[s] = rc.f[R_CUM + s]; c.tb[s] = rc.f[R_TB + s]; }
    };
    auto advance = [&](Cur& c) {
        if (c.nsteps < 0) return;
        if (++c.kt == c.nsteps) { ++c.rec; load_cur(c); }
    };

    if (wave == EP_WAVES - 1) {
        // =========================== scheduler wavefront ===========================
        const int xcd = blockIdx.x & 7, wg = blockIdx.x >> 3;
        int written = 0, covered = 0;                    // records published; global steps they cover
        int exhausted = 0;                               // (every piece of state is kept uniform, in scalar registers)
        int queue = xcd, issued_at = 0;
        // item `id` -> record `written`
        auto publish = [&](int id) {
            int* r = sRec + (written % EP_REC_RING) * EP_REC_INTS;
            if (id < 0) {
                if (lane == 0) r[R_NSTEPS] = -1;
            } else {
                const int u = id / tiles, t = id - u * tiles;
                // the rank whose run of units holds u
                int rank = 0;
                for (int r0 = 0; r0 < E; r0 += 64) {
                    const int rr = r0 + lane;
                    const bool hit = rr < E && u >= sPlan[2 * E + rr] && u < sPlan[2 * E + rr] + sPlan[E + rr];
                    const unsigned long long m = __builtin_amdgcn_ballot_w64(hit);
                    if (m) rank = r0 + (int)__builtin_ctzll(m);
                }
                rank = uni(rank);
                // (values read from LDS are the same in every lane; saying so keeps the bookkeeping in scalar registers)
                const int e = uni(sPlan[rank]), nparts = uni(sPlan[E + rank]), part = u - uni(sPlan[2 * E + rank]), slot0 = uni(sPlan[3 * E + rank]);
                int rows = 0;
                int cum[EP_MAX_K], tb[EP_MAX_K];
#pragma unroll
                for (int s = 0; s < EP_MAX_K; ++s) {
                    const int beg = s < nslot ? uni(sOffs[s * (E + 1) + e]) : 0, end = s < nslot ? uni(sOffs[s * (E + 1) + e + 1]) : 0;
                    cum[s] = rows;
                    tb[s] = s * p.T + beg - rows;
                    rows += end - beg;
                }
                const int all_steps = max(1, (rows + BKT - 1) / BKT);
                const int step0 = (int)((long)all_steps * part / nparts), step1 = (int)((long)all_steps * (part + 1) / nparts);
                if (lane == 0) {
                    r[R_E] = e; r[R_M0] = (t / p.ntn) * BM; r[R_N0] = (t % p.ntn) * BN;
                    r[R_NSTEPS] = max(1, step1 - step0);
                    r[R_POS0] = step0 * BKT; r[R_POS1] = min(rows, step1 * BKT);
                    r[R_SLOT] = nparts > 1 ? slot0 + part : -1;
                    r[R_F32] = (OUT32 || nparts > 1) ? 1 : 0;
#pragma unroll
                    for (int s = 0; s < EP_MAX_K; ++s) { r[R_CUM + s] = cum[s]; r[R_TB + s] = tb[s]; }
                }
                covered = uni(covered + max(1, step1 - step0));
            }
            written = uni(written + 1);
        };
        // queue position -> item: runs of `group` items go to the XCDs in turn
        auto item_of = [&](int q, int j) { return ((j / p.group) * 8 + q) * p.group + j % p.group; };
        // items in XCD q's queue
        auto queue_len = [&](int q) {
            const int round = 8 * p.group, full = total / round, rem = total - full * round;
            return full * p.group + min(max(rem - q * p.group, 0), p.group);
        };
        // One memory operation is in flight at most: a pop of `queue` (an atomic by lane 0) or, once this XCD's own
        // queue is used up, a look at all eight counters (lanes 0..7) that says which other queue still has items --
        // so a workgroup at the end of the launch learns that nothing is left from two round trips, not from eight
        // failed pops.  Results are awaited where they are first used.
        enum { IDLE, POP, LOOKUP };
        int op = uni((int)IDLE), mem_value = 0;
        auto issue_pop = [&]() {
            if (lane == 0) mem_value = __hip_atomic_fetch_add(p.queue + queue, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            op = uni((int)POP);
        };
        auto issue_lookup = [&]() {
            mem_value = 0;
            if (lane < 8) mem_value = __hip_atomic_load(p.queue + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            op = uni((int)LOOKUP);
        };
        // the items of one pop: `batch` consecutive positions of a queue; false when the queue is used up
        auto publish_batch = [&](int q, int j0) {
            if (uni(item_of(q, j0)) >= total) return false;
            for (int b = 0; b < p.batch; ++b) {
                const int id = uni(item_of(q, j0 + b));
                if (id < total) publish(id);
            }
            return true;
        };
        auto finish_op = [&]() {
            if (op == POP) {
                const int j0 = (p.wg_per_xcd + uni(mem_value)) * p.batch;
                op = uni((int)IDLE);
                if (publish_batch(queue, j0)) return;
                issue_lookup();                          // this queue is used up: who still has items?
                return;
            }
            // the first queue after this XCD's own whose counter has not passed its length
            const bool left = lane < 8 && (p.wg_per_xcd + mem_value) * p.batch < queue_len(lane);
            const unsigned m = (unsigned)__builtin_amdgcn_ballot_w64(left) & 0xffu;
            op = uni((int)IDLE);
            if (!m) { exhausted = 1; publish(-1); return; }
            const unsigned rot = ((m >> xcd) | (m << (8 - xcd))) & 0xffu;     // bit i: queue (xcd + i) % 8
            queue = uni((xcd + (int)__builtin_ctz(rot)) & 7);
            issue_pop();
        };
        // before barrier g: the records cover step g + EP_NEED (or everything); then look further ahead without waiting
        auto before_barrier = [&](int g) {
            while (!exhausted && covered < g + EP_NEED) {
                if (op == IDLE) issue_pop();
                finish_op();
            }
            if (op != IDLE && g - issued_at >= EP_WAIT) { finish_op(); issued_at = uni(g); }   // long since back: costs no wait
            if (op == IDLE && !exhausted && covered < g + EP_LOOK) { issue_pop(); issued_at = uni(g); }
            lds_wait();
        };
        // Token ids of a step into ring slot `ring`, EP_IDS_AHEAD steps before the step is multiplied: 64 lanes, 4 bytes
        // each (a base every lane shares plus a 32-bit offset; a lane past the end of the list reads the first id of
        // the table -- the rows of such positions are replaced by zeros when they are fetched).  Lane l fetches
        // position (l % 4) * 16 + l / 4 of the step, so that the four tokens a copy lane needs (16 apart) lie side by side.
        Cur ci;
        auto issue_ids = [&](int ring) {
            if (ci.nsteps < 0) return;
            const int pos = ci.pos0 + ci.kt * BKT + (lane & 3) * 16 + (lane >> 2);
            int t = ci.tb[0];
#pragma unroll
            for (int s = 1; s < KS; ++s) t = pos >= ci.cum[s] ? ci.tb[s] : t;
            const unsigned off = pos < ci.pos1 ? (unsigned)(pos + t) * 4u : 0u;
            __builtin_amdgcn_global_load_lds((glb_ptr_t)(reinterpret_cast<const char*>(p.token_ids) + (size_t)off),
                                             (lds_ptr_t)(smem + L::IDS_AT + ring * 256), 4, 0, 0);
            advance(ci);
        };
        publish_batch(xcd, wg * p.batch);               // the first items are this workgroup's position in its XCD's queue: no atomic
        before_barrier(0);
        ci.rec = 0; load_cur(ci);
        for (int x = 0; x < EP_IDS_AHEAD; ++x) issue_ids(x);
        wait_vmcnt<0>();
        __syncthreads();                                 // (P) the first records and the first steps' ids are there
        int g = 0;
        for (int r = 0;; ++r) {
            const Rec rc = load_rec(r);
            const int nsteps = rc.f[R_NSTEPS];
            if (nsteps < 0) break;
            const int f32 = rc.f[R_F32];
            for (int kt = 0; kt < nsteps; ++kt, g = uni(g + 1)) {
                if (g > 0) before_barrier(g);
                // the ids of step g + EP_IDS_AHEAD leave now; those of step g + 3, whose tokens the copy wavefronts read
                // behind this barrier, were issued two steps ago and have landed once at most one copy is outstanding
                issue_ids((g + EP_IDS_AHEAD) % EP_IDS_RING);
                wait_vmcnt<EP_IDS_AHEAD - 4>();
                barrier_nofence();
            }
            before_barrier(g);
            barrier_nofence();                           // (A)
            if (f32) { barrier_nofence(); barrier_nofence(); }   // (S1) (S2)
        }
        barrier_nofence();                               // (B)
        // the last workgroup to get here puts the counters back to zero for the next launch
        if (lane == 0) {
            const int done = __hip_atomic_fetch_add(p.queue + 8, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (done == (int)gridDim.x - 1) {
                for (int q = 0; q < 9; ++q) __hip_atomic_store(p.queue + q, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        return;
    }
    __syncthreads();                                     // (P)

    if (wave < EP_MUL) {
        // =========================== multiply wavefronts ===========================
        const int wr = wave / C::WF, wf = wave % C::WF;
        f32x16 acc[C::FB][C::RB];
        zero_acc(acc);
        int stage = 0;
        constexpr int RW = 32 * C::RB, FW = 32 * C::FB;
        const int nl0 = wf * FW + 4 * (lane >> 5);       // + j * 32 + 8 * gq
        for (int r = 0;; ++r) {
            const Rec rc = load_rec(r);
            const int nsteps = rc.f[R_NSTEPS];
            if (nsteps < 0) break;
            const int f32 = rc.f[R_F32];
            for (int kt = 0; kt < nsteps; ++kt) {
                barrier_nofence();                       // the copies of this step have landed
                const unsigned base = lds0 + L::STAGES_AT + stage * C::STAGE_BYTES;
                mma_stage_ahead<TC, C, true, true>(base, base + C::R_BYTES, wr, wf, lane, acc);
                stage = stage + 1 == STAGES ? 0 : stage + 1;
            }
            barrier_nofence();                           // (A) the store wavefronts are done with the staging area
            if (!f32) {
                const unsigned stg = lds0 + L::STAGING_AT + (wr * RW + (lane & 31)) * L::CP + nl0 * 2;   // + i * 32 * CP
                static_for<C::FB * 4>([&](auto jg) {
                    constexpr int u = decltype(jg)::value, j = u / 4, gq = u % 4;
                    static_for<C::RB>([&](auto ic) {
                        constexpr int i = decltype(ic)::value;
                        lds_write64<i * 32 * L::CP + (j * 32 + 8 * gq) * 2>(
                            stg, pack4<TC>(acc[j][i][4 * gq], acc[j][i][4 * gq + 1], acc[j][i][4 * gq + 2], acc[j][i][4 * gq + 3]));
                    });
                });
                lds_wait();
            } else {
                // fp32 rows: half a tile at a time (wavefront row 0, then wavefront row 1 once the first half has left)
                const unsigned stg = lds0 + L::STAGING_AT + (lane & 31) * L::CPF + nl0 * 4;
                auto write_half = [&]() {
                    static_for<C::FB * 4>([&](auto jg) {
                        constexpr int u = decltype(jg)::value, j = u / 4, gq = u % 4;
                        static_for<C::RB>([&](auto ic) {
                            constexpr int i = decltype(ic)::value;
                            u32x4 v = {__float_as_uint(acc[j][i][4 * gq]), __float_as_uint(acc[j][i][4 * gq + 1]),
                                       __float_as_uint(acc[j][i][4 * gq + 2]), __float_as_uint(acc[j][i][4 * gq + 3])};
                            lds_write128<i * 32 * L::CPF + (j * 32 + 8 * gq) * 4>(stg, v);
                        });
                    });
                    lds_wait();
                };
                if (wr == 0) write_half();
                barrier_nofence();                       // (S1)
                barrier_nofence();                       // (S2) the first half has been read
                if (wr == 1) write_half();
            }
            zero_acc(acc);
        }
        barrier_nofence();                               // (B) the last item is staged
        return;
    }

    if (wave < EP_MUL + EP_COPY) {
        // =========================== copy wavefronts ===========================
        const int cw = wave - EP_MUL;
        const char* zero = reinterpret_cast<const char*>(g_zero_block);
        // what does not change from step to step: which token of the stage and which column piece a lane fetches
        int kkc[R_CPW], chc[R_CPW];
#pragma unroll
        for (int i = 0; i < R_CPW; ++i) ks_lane<BM>(cw + CW * i, lane, kkc[i], chc[i]);
        const unsigned pitchP = (unsigned)M * 2u, pitchQ = (unsigned)N * 2u;

        // this lane's four tokens of the step whose ids are in ring slot `ring` (see the scheduler's issue_ids):
        // issued, not awaited
        const unsigned tok_at = lds0 + L::IDS_AT + (4 * cw + (lane >> 4)) * 16;
        auto read_tokens = [&](int ring) { return lds_read128_async(tok_at + ring * 256); };
        auto settle_tokens = [&](u32x4& t) {
            lds_wait();
            asm volatile("" : "+v"(t));
        };
        // operand rows of the cursor's step into stage `stage`, from the step's tokens
        auto issue_data = [&](const Cur& c, int stage, const u32x4& tk) {
            const int tok[4] = {(int)tk.x, (int)tk.y, (int)tk.z, (int)tk.w};
            char* base = smem + L::STAGES_AT + stage * C::STAGE_BYTES;
            if (c.nsteps < 0) {   // nothing left: the copies are issued all the same, so that the waits stay uniform
#pragma unroll
                for (int i = 0; i < R_CPW + F_CPW; ++i) __builtin_amdgcn_global_load_lds((glb_ptr_t)zero, (lds_ptr_t)(smem + L::IDS_AT), 4, 0, 0);
                return;
            }
            const int pos_b = c.pos0 + c.kt * BKT;
            const bool inner = c.m0 + BM <= M && c.n0 + BN <= N && pos_b + BKT <= c.pos1;
            if (inner) {
                // a row is (the tensor: scalar) + (slot rows * s + token) * pitch + column, in 32 bits
                const char* const pb = reinterpret_cast<const char*>(p.pm) + (size_t)c.m0 * 2;
                const char* const qb = reinterpret_cast<const char*>(p.qm) + (size_t)c.n0 * 2;
#pragma unroll
                for (int i = 0; i < R_CPW; ++i) {
                    const int pos = pos_b + kkc[i];
                    unsigned rowp = (unsigned)tok[i], rowq = (unsigned)tok[i];
#pragma unroll
                    for (int j = 1; j < KS; ++j) {
                        const bool in = pos >= c.cum[j];
                        rowp += in ? (unsigned)p.p_slot_rows : 0u;
                        rowq += in ? (unsigned)p.q_slot_rows : 0u;
                    }
                    dma16(pb + (size_t)(__umul24(rowp, pitchP) + (unsigned)chc[i] * 16u), base + (cw + CW * i) * 1024);
                    dma16(qb + (size_t)(__umul24(rowq, pitchQ) + (unsigned)chc[i] * 16u), base + C::R_BYTES + (cw + CW * i) * 1024);
                }
                return;
            }
            // the last step of a list and blocks on the result's edge: lanes without a row read a block of zeros
#pragma unroll
            for (int i = 0; i < R_CPW; ++i) {
                const int pos = pos_b + kkc[i];
                int s = 0;
#pragma unroll
                for (int j = 1; j < KS; ++j) s += pos >= c.cum[j] ? 1 : 0;
                const bool row_ok = pos < c.pos1;
                const bool okp = row_ok && c.m0 + chc[i] * 8 < M, okq = row_ok && c.n0 + chc[i] * 8 < N;
                const char* sp = okp ? reinterpret_cast<const char*>(p.pm) + (((size_t)p.p_slot_rows * s + tok[i]) * M + c.m0 + chc[i] * 8) * 2 : zero;
                const char* sq = okq ? reinterpret_cast<const char*>(p.qm) + (((size_t)p.q_slot_rows * s + tok[i]) * N + c.n0 + chc[i] * 8) * 2 : zero;
                dma16(sp, base + (cw + CW * i) * 1024);
                dma16(sq, base + C::R_BYTES + (cw + CW * i) * 1024);
            }
        };

        // The tokens of a step are read from the ring one step before its rows are fetched (so no LDS latency sits in the
        // way of the copies) and that read is awaited at the end of the same step, when it is long since back.
        static_assert(R_CPW == 4, "a lane's tokens are one 16-byte read");
        Cur cd;
        cd.rec = 0; load_cur(cd);
        int gd = 0;                                      // next step whose rows are to be fetched
        u32x4 tc, tn;
#pragma unroll
        for (int x = 0; x < STAGES - 1; ++x) {
            tc = read_tokens(gd % EP_IDS_RING); settle_tokens(tc);
            issue_data(cd, gd % STAGES, tc); advance(cd); ++gd;
        }
        tc = read_tokens(gd % EP_IDS_RING); settle_tokens(tc);      // the tokens of step 2
        int g = 0;
        for (int r = 0;; ++r) {
            const Rec rc = load_rec(r);
            const int nsteps = rc.f[R_NSTEPS];
            if (nsteps < 0) break;
            const int f32 = rc.f[R_F32];
            for (int kt = 0; kt < nsteps; ++kt, ++g) {
                wait_vmcnt<CPW>();                       // the rows of step g have landed: only those of step g + 1 may be outstanding
                barrier_nofence();                       // publishes stage g; everyone is done reading stage g - 1
                tn = read_tokens((gd + 1) % EP_IDS_RING);
                issue_data(cd, gd % STAGES, tc); advance(cd); ++gd;
                settle_tokens(tn);
                tc = tn;
            }
            barrier_nofence();                           // (A)
            if (f32) { barrier_nofence(); barrier_nofence(); }
        }
        wait_vmcnt<0>();
        barrier_nofence();                               // (B)
        return;
    }

    // =========================== store wavefronts ===========================
    const int et = tid - 64 * (EP_MUL + EP_COPY);        // 0 .. 255
    constexpr int NTS = 64 * EP_STORE;
    constexpr int LPR = BN / 8, PROWS = NTS / LPR, PIECES = BM * LPR / NTS;             // 16-bit rows: 16-byte pieces
    constexpr int LPRF = BN / 4, PROWSF = NTS / LPRF, PIECESF = (BM / 2) * LPRF / NTS;  // fp32 rows, half a tile
    static_assert(PIECES == PIECESF, "both forms leave in the same number of pieces per lane");
    const bool streaming = p.stream_dw != 0;
    struct Out { int e, m0, n0, slot, f32; };
    auto out_of = [&](const Rec& rc) {
        Out o;
        o.e = rc.f[R_E]; o.m0 = rc.f[R_M0]; o.n0 = rc.f[R_N0]; o.slot = rc.f[R_SLOT]; o.f32 = rc.f[R_F32];
        return o;
    };
    // piece q of the staged rows.  half: which half of the tile the staging area holds (fp32 form only).
    auto piece = [&](const Out& o, int q, int half) {
        if (!o.f32) {
            const int c = et % LPR, row = et / LPR + q * PROWS;
            u32x4 v = lds_read128_async(lds0 + L::STAGING_AT + row * L::CP + c * 16);
            lds_wait();
            asm volatile("" : "+v"(v));
            const int m = o.m0 + row, n = o.n0 + c * 8;
            if (m >= M || n >= N) return;
            char* const outb = reinterpret_cast<char*>(p.dw) + ((size_t)o.e * M + o.m0) * N * 2;
            const unsigned off = (unsigned)(row * N + n) * 2u;
            if (p.accumulate) {
                const u32x4 old = *reinterpret_cast<const u32x4*>(outb + off);
                v.x = pack2<TC>(lo16<TC>(v.x) + lo16<TC>(old.x), hi16<TC>(v.x) + hi16<TC>(old.x));
                v.y = pack2<TC>(lo16<TC>(v.y) + lo16<TC>(old.y), hi16<TC>(v.y) + hi16<TC>(old.y));
                v.z = pack2<TC>(lo16<TC>(v.z) + lo16<TC>(old.z), hi16<TC>(v.z) + hi16<TC>(old.z));
                v.w = pack2<TC>(lo16<TC>(v.w) + lo16<TC>(old.w), hi16<TC>(v.w) + hi16<TC>(old.w));
            }
            global_store128(outb, off, v, streaming);
        } else {
            const int c = et % LPRF, rl = et / LPRF + q * PROWSF, row = half * (BM / 2) + rl;
            u32x4 v = lds_read128_async(lds0 + L::STAGING_AT + rl * L::CPF + c * 16);
            lds_wait();
            asm volatile("" : "+v"(v));
            const int m = o.m0 + row, n = o.n0 + c * 4;
            if (m >= M || n >= N) return;
            const unsigned off = (unsigned)(row * N + n) * 4u;
            if (o.slot >= 0) {   // one part of a busy expert: fp32 partial result into its scratch slot
                char* const outb = reinterpret_cast<char*>(p.scratch) + ((size_t)o.slot * M + o.m0) * N * 4;
                global_store128(outb, off, v, false);
                return;
            }
            if (OUT32) {
                char* const outb = reinterpret_cast<char*>(p.dw) + ((size_t)o.e * M + o.m0) * N * 4;
                if (p.accumulate) {
                    const u32x4 old = *reinterpret_cast<const u32x4*>(outb + off);
                    v.x = __float_as_uint(__uint_as_float(v.x) + __uint_as_float(old.x));
                    v.y = __float_as_uint(__uint_as_float(v.y) + __uint_as_float(old.y));
                    v.z = __float_as_uint(__uint_as_float(v.z) + __uint_as_float(old.z));
                    v.w = __float_as_uint(__uint_as_float(v.w) + __uint_as_float(old.w));
                }
                global_store128(outb, off, v, streaming);
            }
        }
    };

    bool have = false;
    Out prev{};
    for (int r = 0;; ++r) {
        const Rec rc = load_rec(r);
        const int nsteps = rc.f[R_NSTEPS];
        if (nsteps < 0) break;
        const Out cur = out_of(rc);
        // the previous item's staged rows (its second half, if it is an fp32 one) leave during this item's steps
        int done = 0;
        for (int kt = 0; kt < nsteps; ++kt) {
            barrier_nofence();
            if (have) {
                const int upto = ((kt + 1) * PIECES + nsteps - 1) / nsteps;
                for (; done < upto && done < PIECES; ++done) piece(prev, done, 1);
            }
        }
        barrier_nofence();                               // (A)
        if (cur.f32) {
            barrier_nofence();                           // (S1) the first half is staged
            for (int q = 0; q < PIECES; ++q) piece(cur, q, 0);
            barrier_nofence();                           // (S2)
        }
        prev = cur;
        have = true;
    }
    barrier_nofence();                                   // (B)
    if (have) {
        for (int q = 0; q < PIECES; ++q) piece(prev, q, 1);
    }
}

template <typename TC, bool OUT32, int KS>
int launch_estmm_pipe_k(const EstmmPipeK& p, int grid, hipStream_t st) {
    auto kernel = estmm16_pipe_kernel<TC, OUT32, KS>;
    if (int rc = ensure_smem(kernel, EpLds::BYTES)) return rc;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(EP_NT), EpLds::BYTES, st, p);
    HEXA_CHECK_LAUNCH("estmm16_pipe");
    return HEXA_OK;
}
template <typename TC, bool OUT32>
int launch_estmm_pipe_t(const EstmmPipeK& p, int grid, hipStream_t st) {
    if (p.k <= 1) return launch_estmm_pipe_k<TC, OUT32, 1>(p, grid, st);
    if (p.k <= 2) return launch_estmm_pipe_k<TC, OUT32, 2>(p, grid, st);
    if (p.k <= 4) return launch_estmm_pipe_k<TC, OUT32, 4>(p, grid, st);
    return launch_estmm_pipe_k<TC, OUT32, 8>(p, grid, st);
}

int cu_count() {
    static int cus = 0;
    if (!cus) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n < 8)
            n = 256;
        cus = n;
    }
    return cus;
}

}  // namespace

bool estmm16_pipe_supported(const EstmmArgs& a) {
    if (!a.plan || a.r.E > EP_MAX_E || a.r.k > EP_MAX_K) return false;
    if ((a.m_dim % 8) || (a.n_dim % 8) || !(a.dw_dt == a.pq_dt || a.dw_dt == HEXA_F32)) return false;
    if (a.max_slots >= 2 && (!a.scratch || (((long)a.m_dim * a.n_dim) & 3))) return false;
    // rows are addressed as base + (24-bit row) * (24-bit pitch) in 32 bits
    const size_t rows = (size_t)a.r.T * a.r.k;
    return rows < ((size_t)1 << 24) && rows * a.m_dim * 2 < ((size_t)1 << 32) && rows * a.n_dim * 2 < ((size_t)1 << 32) &&
           (size_t)128 * std::max(a.m_dim, a.n_dim) * 4 < ((size_t)1 << 32);
}

int launch_estmm16_pipe(const EstmmArgs& a, hipStream_t st) {
    using C = CfgE;
    EstmmPipeK p;
    p.pm = a.p; p.qm = a.q; p.dw = a.dw;
    p.token_ids = a.r.token_ids; p.offsets = a.r.offsets;
    p.plan = a.plan; p.queue = const_cast<int32_t*>(a.plan) + estmm_plan_queue_at(a.r.E);
    p.scratch = a.max_slots >= 2 ? a.scratch : nullptr;
    p.T = a.r.T; p.k = a.r.k; p.E = a.r.E; p.M = a.m_dim; p.N = a.n_dim;
    p.mtn = div_up(a.m_dim, C::BM); p.ntn = div_up(a.n_dim, C::BN);
    // runs of up to three row tiles (with all their column tiles) per XCD: their items share the rows of Q
    p.group = p.ntn * (option(OPT_ESTMM_GROUP) > 0 ? option(OPT_ESTMM_GROUP) : std::min(3, p.mtn));
    p.p_slot_rows = a.p_per_slot ? a.r.T : 0;
    p.q_slot_rows = a.q_per_slot ? a.r.T : 0;
    p.accumulate = a.accumulate;
    p.stream_dw = option(OPT_ESMM_STREAM) != 2;
    p.wg_per_xcd = std::max(1, cu_count() / 8);
    p.out32 = a.dw_dt == HEXA_F32;
    {   // about a dozen steps per pop, but at least four pops per workgroup
        const long avg_steps = std::max<long>(1, ((long)a.r.T * a.r.k / a.r.E + 63) / 64);
        const long items = (long)a.r.E * p.mtn * p.ntn;
        p.batch = (int)std::max<long>(1, std::min<long>({8, (12 + avg_steps - 1) / avg_steps, items / (32L * p.wg_per_xcd)}));
    }
    const int grid = 8 * p.wg_per_xcd;
    const bool o32 = a.dw_dt == HEXA_F32;
    int rc;
    if (a.pq_dt == HEXA_BF16) rc = o32 ? launch_estmm_pipe_t<__bf16, true>(p, grid, st) : launch_estmm_pipe_t<__bf16, false>(p, grid, st);
    else rc = o32 ? launch_estmm_pipe_t<_Float16, true>(p, grid, st) : launch_estmm_pipe_t<_Float16, false>(p, grid, st);
    if (rc || a.max_slots < 2) return rc;
    return launch_estmm_fixup(a, st);
}

}  // namespace hexa
