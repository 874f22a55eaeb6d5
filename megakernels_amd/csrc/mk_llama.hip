// Batch-1 Llama decode as one persistent kernel for MI355X (gfx950).
//
// Execution model (counterpart of the reference VM runtime, include/megakernel.cuh:15-171,
// include/controller/controller.cuh:24-132, include/util.cuh:260-304, rebuilt for CDNA4):
//   * grid = one workgroup per compute unit; workgroup w executes instructions[w, 0..num_slots)
//     strictly in order.  The LDS request (> half of the CU's 160 KB) keeps a second workgroup
//     off the same CU.
//   * a workgroup is 9 wave64: eight CONSUMER waves stream weight rows (16-byte streaming buffer
//     loads straight into VGPRs, several rows in flight per wave, no LDS staging for weights) and
//     do the dot products; one CONTROLLER wave does everything that is latency-critical and small:
//     it waits on the dependency counters, fetches the activation vector, normalises it and hands
//     it to the consumers through LDS, and after the matvec it runs the epilogue (RoPE, SiLU,
//     residual, stores) and signals the next counter.  The controller never has bulk loads
//     outstanding, so its polls and 4 KB activation loads do not queue behind its own weight
//     traffic (vector memory returns in order per wave).  Consumers request the first rows of an
//     instruction on entry, before its dependency is known: weights never depend on a barrier.
//     (In attention and in the partition merge the consumer waves also store and signal.)
//   * launch arguments and the worker's instruction queue are copied into LDS once; every
//     instruction kind has its own non-inlined handler, so each gets its own register allocation.
//   * cross-CU ordering is only through counters in HBM, with the counts of the reference's
//     Python VM (megakernels/demos/latency/python_vm.py).  The eight XCDs have private L2
//     caches, so everything one CU writes for another (activations, the new KV row, counters)
//     is stored write-through and loaded with agent-scope ("sc1") accesses; no cache-wide
//     write-back / invalidate is ever issued.  A producer waits for its stores (s_waitcnt
//     vmcnt(0)) before it bumps the counter.
//   * the four counters that receive one arrival per worker (barriers[l, 2..5, 0]) are kept
//     as 16 shards in the workspace while the kernel runs (256 atomics on one address cost
//     ~3 us, 16 per shard ~0.2 us); the last workgroup to finish adds the shard totals into
//     `barriers`, so after the launch the tensor holds exactly the reference VM's counts.
//   * a residual projection over several column groups (down; O-proj of 4096-wide models) leaves
//     the groups' partial sums as (value, tag) pairs in the workspace; the job of the last group
//     fetches them until every tag is the current phase's and applies them in group order, the
//     Python VM's order, so the bf16 rounding chain is reproduced without serialising the workers.
//   * every barrier wait is bounded (spin_limit_us): on expiry the worker records a status
//     code and every workgroup leaves its instruction loop, so the grid always drains.
//   * optionally the per-token glue of the reference's decode loop is part of the launch (embedding
//     row of the input token, argmax of the logits, barrier reset), and then a launch can run
//     several decode steps back to back: the last workgroup of a step publishes the step's token,
//     the others wait for that and start over one position further on.
//
// Arithmetic: bit-compatible with a fixed "column order" so results can be compared exactly
// with a CPU restatement of the Python VM.  A matvec dot product over K elements is computed by
// one wave: accumulator c = lane * 4 + d takes the element pairs j*256 + c in order of j, each
// step being the two-element bf16 dot product instruction (four independent chains per lane; its
// arithmetic is written out where the test suite keeps its definition), and the 256 sums are
// combined as a balanced pairwise tree (within the lane, then an xor butterfly over lanes).
// Narrowing to bf16 happens exactly where the Python VM narrows (python_vm.py:29-80,127-274).
#include <hip/hip_runtime.h>

#include <climits>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <type_traits>

#include "../../include/mk_llama.h"
#include "mk_math.h"

namespace {

#ifndef MK_CONSUMER_WAVES
#define MK_CONSUMER_WAVES 8
#endif
constexpr int kConsumerWaves = MK_CONSUMER_WAVES;  // waves that stream weight rows in the matvec instructions
constexpr int kAttnWaves = 8;       // waves that work on an attention partition (the token -> slot mapping is built on 8)
static_assert(kConsumerWaves >= kAttnWaves, "attention runs on the first consumer waves");
constexpr int kConsumerThreads = kConsumerWaves * 64;
constexpr int kAttnThreads = kAttnWaves * 64;
constexpr int kThreads = kConsumerThreads + 64;  // + one controller wave
#ifndef MK_SHARDS
#define MK_SHARDS 16
#endif
constexpr int kShards = MK_SHARDS;   // shards per hot barrier counter
#ifndef MK_REPLICAS
#define MK_REPLICAS 4
#endif
constexpr int kReplicas = MK_REPLICAS;  // copies of every shard: a signal goes to all, a worker polls one
constexpr int kHotRows = 4;         // barrier rows 2..5 are sharded
constexpr int kOutRows = 2048;      // rows staged in LDS between matvec and epilogue
constexpr int kMaxK = 4096;         // longest activation vector handed through LDS
constexpr int kScoreCap = 4096;     // tokens per attention partition (LDS score buffer)
constexpr int kShareLayers = 128;   // layers for which QKV work can be shared between partner workers
constexpr int kQueueSlots = 192;    // instructions of a worker's queue kept in LDS at a time (a longer queue goes through in windows)
constexpr int kMaxHeadDim = 128;
constexpr int kGqa = 4;             // query heads per KV head handled by one attention instruction
constexpr int kStatusInts = 16;
constexpr int kDoneSlot = 8;        // workspace int: workgroups finished, summed over the steps of a launch
constexpr int kStepSlot = 9;        // workspace int: decode steps of this launch completed and published
constexpr int kEpochSlot = 10;      // workspace int: decode steps completed since the workspace was zeroed

// Weight rows in flight per consumer wave, per instruction kind (16 VGPRs per 2048-element row; the
// 9-wave workgroup leaves each lane 168 VGPRs).  The rows requested before the dependency wait are
// the prefetch; rows a wave does not have become no-op requests.  Rows per wave in the usual
// schedules: QKV 2, O-proj 2, up/gate 8, down 4, LM head 63.  The depths come from sweeps of the
// whole decode step: an instruction that everybody enters at the same moment, right after its
// dependency resolves (down, LM head), does best with a shallow queue - deep ones only delay the
// first rows - while up/gate, entered early, takes all the rows the registers hold.
#ifndef MK_PF_QKV
#define MK_PF_QKV 2
#endif
#ifndef MK_PF_OPROJ
#define MK_PF_OPROJ 2
#endif
#ifndef MK_PF_UPGATE
#define MK_PF_UPGATE 5
#endif
#ifndef MK_PF_DOWN
#define MK_PF_DOWN 2
#endif
#ifndef MK_PF_LMHEAD
#define MK_PF_LMHEAD 2
#endif
#ifndef MK_PF_WIDE_OPROJ
#define MK_PF_WIDE_OPROJ 4
#endif
#ifndef MK_PF_WIDE_DOWN
#define MK_PF_WIDE_DOWN 6
#endif
#ifndef MK_WIDE_PARK_QKV
#define MK_WIDE_PARK_QKV 1
#endif
#ifndef MK_WIDE_PARK_UPGATE
#define MK_WIDE_PARK_UPGATE 1
#endif
#ifndef MK_WIDE_PARK_DOWN
#define MK_WIDE_PARK_DOWN 2
#endif
#ifndef MK_WIDE_AHEAD
#define MK_WIDE_AHEAD 1             // such a model's O-proj parks the last row per wave of the up/gate instruction behind it
#endif
#ifndef MK_PF_WIDE_CAP
#define MK_PF_WIDE_CAP 2
#endif
template <int KC>
constexpr int rows_in_flight(int wanted) { return KC <= 4 ? wanted : (wanted < MK_PF_WIDE_CAP ? wanted : MK_PF_WIDE_CAP); }

#ifndef MK_PAIR_OPROJ_UPGATE
#define MK_PAIR_OPROJ_UPGATE 1      // O-proj and a directly following up/gate run as one handler
#endif
#ifndef MK_PARK_UPGATE
#define MK_PARK_UPGATE 1            // long-waiting O-proj + up/gate workers park up/gate's last rows in LDS
#endif
#ifndef MK_PARK_DOWN
#define MK_PARK_DOWN 1              // ... and the last rows per wave of the down projection that follows
#endif
#ifndef MK_PARK_ALL
#define MK_PARK_ALL 0               // 1: also the workers that come to O-proj + up/gate from attention park rows
#endif
#ifndef MK_RUN_JOBS
#define MK_RUN_JOBS 1               // consecutive jointly executed jobs of the same blocks run as one
#endif
#ifndef MK_SHARE_QKV
#define MK_SHARE_QKV 1              // a worker with one QKV block less than its partner takes half of the partner's last block
#endif
#ifndef MK_STAGE_QUERY
#define MK_STAGE_QUERY 1            // attention takes the query and the step's K / V row from their stamped copies
#endif
#ifndef MK_HOLD_NOSLEEP
#define MK_HOLD_NOSLEEP 0
#endif
#ifndef MK_HOLD_LOOKS
#define MK_HOLD_LOOKS 2
#endif
#ifndef MK_HOLD_SHARE
#define MK_HOLD_SHARE 30            // thirty-seconds of the arrivals
#endif
#ifndef MK_WIDE_CONTROLLER_CALL
#define MK_WIDE_CONTROLLER_CALL 1
#endif
#ifndef MK_POLL_SLEEP
#define MK_POLL_SLEEP 10            // units of 64 clocks between two looks at a dependency
#endif
// Weight rows parked in LDS (requested long before their instruction, straight from HBM into LDS) live
// in one region that starts with the attention score buffer and continues behind it.  With eight
// consumer waves the registers hold six of a wave's eight up/gate rows: the other two are parked in the
// score buffer and one row per wave of the following down projection behind it.  With more consumer
// waves all up/gate rows fit the registers, and the region takes rows of the down projection: behind
// the first 16 KB, where the jointly executed down projection keeps its activation vector.
#ifndef MK_PARK_DOWN_ROWS
#define MK_PARK_DOWN_ROWS (MK_CONSUMER_WAVES <= 8 ? 1 : 2)
#endif
constexpr int kParkedUpgateRows = MK_PARK_UPGATE && kConsumerWaves <= 8 ? 2 : 0;  // per wave
constexpr int kParkedDownRows = MK_PARK_DOWN ? MK_PARK_DOWN_ROWS : 0;             // per wave
constexpr int kScoreBytes = kScoreCap * kGqa * 4;
constexpr int kParkDownOffset = kConsumerWaves <= 8 ? kScoreBytes : 16 * 1024;     // into the region
constexpr int kParkRegionBytes = kParkDownOffset + kConsumerWaves * kParkedDownRows * 4096;
constexpr int kParkBytes = kParkRegionBytes > kScoreBytes ? kParkRegionBytes - kScoreBytes : 16;  // behind the score buffer
#define AG __HIP_MEMORY_SCOPE_AGENT

// ---------------------------------------------------------------------------------------------
// workspace layout (ints unless noted)
// ---------------------------------------------------------------------------------------------
struct WsLayout {
    size_t status, shards, argmax, partial, pads, stamped, total_bytes;
};
constexpr int kMaxWorkers = 1024;   // workers that can report an LM-head maximum
constexpr int kPadInts = 32;        // a padded counter owns a 128-byte line
// upper bound of the barrier tensor's columns (query + key + value heads) for a hidden size: heads
// are at least 64 wide and four query heads share a KV head
__host__ __device__ constexpr int pad_cols(int hid) { return hid / 64 + hid / 128; }

__host__ __device__ inline WsLayout ws_layout(int L, int hid, int inter, int R) {
    WsLayout w;
    size_t off = 0;
    w.status = off;   off += kStatusInts;
    off = (off + 31) & ~(size_t)31;  // counters start on a 128-byte line
    w.shards = off;   off += (size_t)kReplicas * kShards * L * kHotRows;
    w.argmax = off;   off += 2 * (size_t)kMaxWorkers;  // per worker: value bits, index + 1 (0: nothing)
    off = (off + 3) & ~(size_t)3;
    w.partial = off;  // (value, tag) pairs of 8 bytes: [max(groups_o, groups_d)][hid]
    int g_o = hid / R, g_d = inter / R;
    off += (size_t)(g_o > g_d ? g_o : g_d) * hid * 2;
    // the per-head counters (barrier rows 0 and 1), one cache line each
    off = (off + 31) & ~(size_t)31;
    w.pads = off;     off += (size_t)L * 2 * pad_cols(hid) * kPadInts;
    // stamped copies of what QKV hands to attention: 8 bytes per bf16 pair (the query, hid / 2 pairs,
    // then the step's K row and V row, at most hid / 8 pairs each)
    off = (off + 31) & ~(size_t)31;
    w.stamped = off;  off += 2 * (size_t)hid;
    w.total_bytes = off * 4;
    return w;
}

// ---------------------------------------------------------------------------------------------
// LDS layout
// ---------------------------------------------------------------------------------------------
// What every instruction needs and no instruction changes: computed once per launch, read from LDS.
struct Consts {
    int *status, *shards, *argmax, *pads;  // regions of the workspace
    uint64_t *partial;              // residual partial sums as (value, tag) pairs
    uint64_t *stamped;              // (bf16 pair, stamp) copies of the query and of the step's K and V rows
    uint32_t epoch;                 // decode steps completed in this workspace before the current one
    int *trace_base;                // this worker's rows of `timings`, or nullptr when tracing is off
    long long spin_ticks;           // limit of a dependency wait, in wall-clock ticks
    int cols;                       // columns of `barriers`: query + key + value heads
    int pad_cols;                   // padded per-head counters per (layer, row)
    int down_jobs, o_jobs;          // arrivals that complete barrier rows 5 and 3
    int shard_stride, replica_stride;  // ints from one shard / one replica of a sharded counter to the next
    int hold_looks;                 // looks at a nearly complete dependency before the consumers' bulk requests are released
};
// A matvec instruction (opcodes 1, 4, 5, 6) decoded once per launch: where its weight rows live.
// ntasks < 0: the instruction is malformed.
struct alignas(16) SlotDesc {
    uint64_t w0_base;               // buffer the rows are addressed in
    long long gate_delta;           // opcode 1: how the last block is shared with the partner worker (0: it is not):
                                    // block << 2 | 1 (rows 0-7 of the own last block only) or 2 (also rows 8-15 of the
                                    // partner's last block);
                                    // opcode 5: byte distance from the up matrix to the gate matrix;
                                    // opcodes 4, 6: joint execution (0: own group only): the number of column groups
                                    // G in bits 0-7, the jobs of the block run in one go (1, 2 or 4) in bits 8-15
    uint32_t w0_bytes, row_bytes;
    int ntasks, first_row;
};
static_assert(sizeof(SlotDesc) == 32, "two 16-byte LDS reads");
// Where an instruction's dependency counter and the counter it signals live (opcodes 1, 4, 5, 6, 7),
// worked out once per launch: the first look at a dependency and the signal after the store
// acknowledgement then need one LDS round trip, not a chain of them.
struct alignas(16) SyncDesc {
    uint64_t poll_base;             // lane l < kShards looks at (int *)poll_base + l * shard_stride; 0: nothing to wait for
    uint64_t bar_word;              // lane kShards looks at the counter's word in `barriers`
    uint64_t signal_base;           // this worker's shard of the counter the instruction signals, first replica
    int target;                     // arrivals that satisfy the dependency
    int pad;
};
static_assert(sizeof(SyncDesc) == 32, "two 16-byte LDS reads");

struct Smem {
    int abort;                      // set once, never cleared during a launch
    int last_flag;
    int token;                      // *token_in, or -1
    int window_base, window_count;  // which slots of the worker's queue are in `queue` / `desc`: [base, base + count)
    Consts k;
    mk_llama_args args;             // the launch arguments, read from here by every instruction
    int flags[16];                  // scratch of the end-of-step reduction
    // QKV instructions per layer of this worker's queue ([0]) and of its partner's ([1]): how many, and of
    // the only one: blocks << 20 | its last block
    int qkv_count[2][kShareLayers];
    int qkv_info[2][kShareLayers];
    // the matvec instructions' hand-over buffers and attention's share their space: an instruction
    // uses one set or the other, and nothing in them outlives an instruction
    union {
        struct {
            alignas(16) uint32_t x[kMaxK / 2];          // activation vector as bf16 pairs, lane layout [chunk][lane][4 dwords]
            alignas(16) float out[kOutRows];            // matvec row results awaiting the epilogue
        };
        struct {
            alignas(16) float wave_max[kAttnWaves][kGqa];
            alignas(16) float wave_l[kAttnWaves][kGqa];
            alignas(16) float wave_o[kAttnWaves][kGqa][kMaxHeadDim];
        };
    };
    alignas(16) float scores[kScoreCap][kGqa];  // attention: one partition's scores, then probabilities
    alignas(16) unsigned char park[kParkBytes];  // the parked rows' region continues here
    int parked_slot;                               // the down projection whose last rows per wave are parked, or -1
    // attention: the four query heads and the step's K and V row of the KV head as bf16 pairs, when the
    // controller took them from their stamped copies (attn_staged != 0)
    int attn_staged;
    alignas(16) uint32_t attn_q[kGqa * kMaxHeadDim / 2];
    alignas(16) uint32_t attn_k[kMaxHeadDim / 2];
    alignas(16) uint32_t attn_v[kMaxHeadDim / 2];
    alignas(16) SlotDesc desc[kQueueSlots];        // the matvec instructions of the window, decoded
    alignas(16) SyncDesc sync[kQueueSlots];        // ... and where their counters live
    alignas(16) int queue[kQueueSlots][MK_INSTRUCTION_WORDS];  // a window of this worker's instructions
};
static_assert(offsetof(Smem, x) % 16 == 0 && offsetof(Smem, wave_max) % 16 == 0 && offsetof(Smem, wave_l) % 16 == 0 &&
                  offsetof(Smem, scores) % 16 == 0,
              "128-bit LDS accesses need 16-byte aligned members");

static_assert(sizeof(Smem) <= 160 * 1024, "LDS budget");
static_assert(offsetof(Smem, park) == offsetof(Smem, scores) + sizeof(Smem::scores), "the parked rows' region is contiguous");
static_assert(sizeof(Smem) > 80 * 1024, "must keep a second workgroup off the CU");

// ---------------------------------------------------------------------------------------------
// agent-coherent memory access (bypass the non-coherent per-XCD L2 contents)
// ---------------------------------------------------------------------------------------------
// Device pointers reach the instruction handlers through LDS, so the compiler cannot tell their
// address space; every access casts to the global address space explicitly.  A generic (flat_*)
// access would count on lgkmcnt as well as vmcnt and couple LDS waits to outstanding weight loads.
#define MK_GLOBAL __attribute__((address_space(1)))
template <class T>
__device__ __forceinline__ MK_GLOBAL T *as_global(T *p) { return (MK_GLOBAL T *)p; }

__device__ __forceinline__ int ld_i32(const int *p) { return __hip_atomic_load(as_global(p), __ATOMIC_RELAXED, AG); }
__device__ __forceinline__ uint32_t ld_u32(const void *p) {
    return __hip_atomic_load(as_global((const uint32_t *)p), __ATOMIC_RELAXED, AG);
}
__device__ __forceinline__ uint64_t ld_u64(const void *p) {
    return __hip_atomic_load(as_global((const uint64_t *)p), __ATOMIC_RELAXED, AG);
}
__device__ __forceinline__ float ld_f32(const float *p) { return mkm::bits_f32(ld_u32(p)); }
__device__ __forceinline__ void st_u32(void *p, uint32_t v) {
    __hip_atomic_store(as_global((uint32_t *)p), v, __ATOMIC_RELAXED, AG);
}
__device__ __forceinline__ void st_u64(void *p, uint64_t v) {
    __hip_atomic_store(as_global((uint64_t *)p), v, __ATOMIC_RELAXED, AG);
}
__device__ __forceinline__ void st_f32(float *p, float v) { st_u32(p, mkm::f32_bits(v)); }
__device__ __forceinline__ void st_i32(int *p, int v) { __hip_atomic_store(as_global(p), v, __ATOMIC_RELAXED, AG); }
__device__ __forceinline__ void add_i32(int *p, int v) { __hip_atomic_fetch_add(as_global(p), v, __ATOMIC_RELAXED, AG); }
__device__ __forceinline__ int add_ret_i32(int *p, int v) {
    return __hip_atomic_fetch_add(as_global(p), v, __ATOMIC_RELAXED, AG);
}
__device__ __forceinline__ uint4 ld_b128(const void *p) {
    uint64_t a = ld_u64(p), b = ld_u64((const char *)p + 8);
    return make_uint4((uint32_t)a, (uint32_t)(a >> 32), (uint32_t)b, (uint32_t)(b >> 32));
}
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
// immutable data (rope tables, old KV rows): ordinary cached 16-byte load
__device__ __forceinline__ uint4 ld_const_b128(const void *p) {
    const u32x4 v = *as_global((const u32x4 *)p);
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ float ld_const_f32(const float *p) { return *as_global(p); }
// plain store of a word nobody else reads during the launch (timing trace)
__device__ __forceinline__ void st_plain_i32(int *p, int v) { *as_global(p) = v; }
// weights: read exactly once per step, so stream them past the caches (the "nt" bit of the
// buffer load's cache policy)
#ifdef MK_NO_NT
#define MK_STREAM_AUX 0
#else
#define MK_STREAM_AUX 2
#endif

// All of this wave's global stores and atomics have been performed.  The "memory" clobber keeps
// the compiler from moving memory operations across it.
__device__ __forceinline__ void wait_stores() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
__device__ __forceinline__ void compiler_fence() { asm volatile("" ::: "memory"); }

// Workgroup barrier that orders LDS traffic only: outstanding global loads (the consumers'
// prefetched weight rows) stay in flight across it.
__device__ __forceinline__ void wg_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// ---------------------------------------------------------------------------------------------
// wave-level reductions.  The canonical order is a pairwise tree in lane order (an xor butterfly
// with ascending offsets).  Additions commute exactly, so any exchange pattern that pairs the same
// partial sums at each level gives the same bits.
// ---------------------------------------------------------------------------------------------
// Exchange with lane (l ^ OFFSET) through the VALU data path (DPP within a row of 16 lanes,
// v_permlane{16,32}_swap across rows) instead of the LDS crossbar, whose ~100-cycle round trip per
// exchange dominated the reduction-heavy instructions.  Returns the pair {own, partner} in
// unspecified order, which is all a commutative combine needs.
struct LanePair {
    uint32_t a, b;
};
template <int OFFSET>
__device__ __forceinline__ LanePair lane_xor_pair(uint32_t v) {
    const int vi = (int)v;
    if constexpr (OFFSET == 1) return {v, (uint32_t)__builtin_amdgcn_update_dpp(0, vi, 0xB1, 0xf, 0xf, false)};
    else if constexpr (OFFSET == 2) return {v, (uint32_t)__builtin_amdgcn_update_dpp(0, vi, 0x4E, 0xf, 0xf, false)};
    else if constexpr (OFFSET == 4) {
        // lanes with bit 2 clear read lane + 4 (row_shl:4, banks 0 and 2), the others lane - 4
        const int r = __builtin_amdgcn_update_dpp(0, vi, 0x104, 0xf, 0x5, false);
        return {v, (uint32_t)__builtin_amdgcn_update_dpp(r, vi, 0x114, 0xf, 0xa, false)};
    } else if constexpr (OFFSET == 8) {
        return {v, (uint32_t)__builtin_amdgcn_update_dpp(0, vi, 0x128, 0xf, 0xf, false)};  // row_ror:8
    } else {
        // a = b = v; the swap exchanges the odd rows (upper half) of a with the even rows (lower
        // half) of b, leaving own and partner values in a and b.  Written in assembly: the
        // compiler's builtin for these instructions returns the first result twice.
        uint32_t a = v, b = v;
        if constexpr (OFFSET == 16) asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
        else asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
        return {a, b};
    }
}
template <int OFFSET>
__device__ __forceinline__ float lane_xor_add(float v) {
    const LanePair p = lane_xor_pair<OFFSET>(__builtin_bit_cast(uint32_t, v));
    return __builtin_bit_cast(float, p.a) + __builtin_bit_cast(float, p.b);
}
template <int OFFSET>
__device__ __forceinline__ float lane_xor_max(float v) {
    const LanePair p = lane_xor_pair<OFFSET>(__builtin_bit_cast(uint32_t, v));
    return fmaxf(__builtin_bit_cast(float, p.a), __builtin_bit_cast(float, p.b));
}

template <int FROM = 1, int TO = 64>
__device__ __forceinline__ float lane_tree_sum(float v) {
    if constexpr (FROM <= 1 && TO > 1) v = lane_xor_add<1>(v);
    if constexpr (FROM <= 2 && TO > 2) v = lane_xor_add<2>(v);
    if constexpr (FROM <= 4 && TO > 4) v = lane_xor_add<4>(v);
    if constexpr (FROM <= 8 && TO > 8) v = lane_xor_add<8>(v);
    if constexpr (FROM <= 16 && TO > 16) v = lane_xor_add<16>(v);
    if constexpr (FROM <= 32 && TO > 32) v = lane_xor_add<32>(v);
    return v;
}
template <int FROM = 1, int TO = 64>
__device__ __forceinline__ float lane_tree_max(float v) {
    if constexpr (FROM <= 1 && TO > 1) v = lane_xor_max<1>(v);
    if constexpr (FROM <= 2 && TO > 2) v = lane_xor_max<2>(v);
    if constexpr (FROM <= 4 && TO > 4) v = lane_xor_max<4>(v);
    if constexpr (FROM <= 8 && TO > 8) v = lane_xor_max<8>(v);
    if constexpr (FROM <= 16 && TO > 16) v = lane_xor_max<16>(v);
    if constexpr (FROM <= 32 && TO > 32) v = lane_xor_max<32>(v);
    return v;
}
template <int OFFSET>
__device__ __forceinline__ int lane_xor_add_i32(int v) {
    const LanePair p = lane_xor_pair<OFFSET>((uint32_t)v);
    return (int)p.a + (int)p.b;
}
__device__ __forceinline__ int lane_sum_i32(int v) {
    v = lane_xor_add_i32<1>(v);
    v = lane_xor_add_i32<2>(v);
    v = lane_xor_add_i32<4>(v);
    v = lane_xor_add_i32<8>(v);
    v = lane_xor_add_i32<16>(v);
    v = lane_xor_add_i32<32>(v);
    return v;
}

// value of another lane through the DPP data path (no LDS round trip); lanes of rows not selected
// by ROW_MASK read 0
template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ float dpp_read(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xf, false));
}
constexpr int kDppXor1 = 0xB1;         // quad_perm [1,0,3,2]
constexpr int kDppXor2 = 0x4E;         // quad_perm [2,3,0,1]
constexpr int kDppHalfMirror = 0x141;  // lane i <- 7 - i within 8: the other quad once quads are uniform
constexpr int kDppMirror = 0x140;      // lane i <- 15 - i within 16: the other half once halves are uniform
constexpr int kDppBcast15 = 0x142;     // lane 15 of each row -> next row
constexpr int kDppBcast31 = 0x143;     // lane 31 -> rows 2 and 3

// Sum over the 64 lanes in the canonical tree order; the result is valid in lane 63 (returned as a
// wave-uniform value).  Levels 1..8 are butterflies inside a row of 16; level 16 adds row 0 into
// row 1 and row 2 into row 3; level 32 adds row 1 into row 3: ((r0+r1)+(r2+r3)).
__device__ __forceinline__ float wave_tree_sum_uniform(float v) {
    v = v + dpp_read<kDppXor1>(v);
    v = v + dpp_read<kDppXor2>(v);
    v = v + dpp_read<kDppHalfMirror>(v);
    v = v + dpp_read<kDppMirror>(v);
    v = v + dpp_read<kDppBcast15, 0xa>(v);
    v = v + dpp_read<kDppBcast31, 0xc>(v);
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
// Sum over each aligned group of N lanes (N = 8 or 16), canonical order, valid in every lane.
template <int N>
__device__ __forceinline__ float group_tree_sum(float v) {
    v = v + dpp_read<kDppXor1>(v);
    v = v + dpp_read<kDppXor2>(v);
    v = v + dpp_read<kDppHalfMirror>(v);
    if (N == 16) v = v + dpp_read<kDppMirror>(v);
    return v;
}

// ---------------------------------------------------------------------------------------------
// per-workgroup context
// ---------------------------------------------------------------------------------------------
// LDS is always addressed through address-space-qualified pointers (ds_* instructions, counted by
// lgkmcnt).  A generic pointer would turn every access into a flat_* instruction, which also counts
// on vmcnt and would make LDS reads wait, in order, behind the consumers' outstanding weight loads.
// The launch arguments and the instruction words live in LDS for the same reason: the instruction
// handlers are separate functions (each gets its own register allocation), and what they need is
// read on demand with ds_read.
#define MK_LDS __attribute__((address_space(3)))
typedef MK_LDS Smem *SmemPtr;
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef const MK_LDS mk_llama_args &ArgsRef;
typedef const MK_LDS int *InsPtr;

// value known to be the same in every lane -> scalar register
__device__ __forceinline__ int uni(int v) { return __builtin_amdgcn_readfirstlane(v); }
template <class T>
__device__ __forceinline__ T *uni(T *p) {
    const uint64_t v = (uint64_t)p;
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32));
    return (T *)(((uint64_t)hi << 32) | lo);
}

struct Ctx {
    SmemPtr sm;
    int tid, wave, lane;
    bool controller;
    int worker, slot, opcode;       // slot: index into the window of the queue that is in LDS
    int *trace;                     // this instruction's timing row, or nullptr when tracing is off
};

// TR: the kernel instance that records timings.  The other instance knows at compile time that
// there is no timing row, so none of the stamping code exists in it.
template <bool TR>
__device__ __forceinline__ Ctx make_ctx(SmemPtr sm, int slot, int opcode) {
    Ctx c;
    c.sm = sm;
    c.tid = (int)threadIdx.x;
    c.wave = c.tid / 64;
    c.lane = c.tid % 64;
    c.controller = c.wave == kConsumerWaves;
    c.worker = (int)blockIdx.x;
    c.slot = slot;
    c.opcode = opcode;
    c.trace = nullptr;
    if constexpr (TR) {
        int *const rows = uni(sm->k.trace_base);
        c.trace = rows ? rows + (size_t)(uni(sm->window_base) + slot) * MK_TIMING_SLOTS : nullptr;
    }
    return c;
}

// workspace regions
__device__ __forceinline__ int *ws_status(const Ctx &c) { return uni(c.sm->k.status); }
__device__ __forceinline__ int *ws_shards(const Ctx &c) { return uni(c.sm->k.shards); }
__device__ __forceinline__ uint64_t *ws_partial(const Ctx &c) { return uni(c.sm->k.partial); }
// stamped copies: the query at pair 0, the K row at pair hidden / 2, the V row behind it
__device__ __forceinline__ uint64_t *ws_stamped_q(const Ctx &c) { return uni(c.sm->k.stamped); }
__device__ __forceinline__ uint64_t *ws_stamped_k(const Ctx &c) { return uni(c.sm->k.stamped) + uni(c.sm->args.hidden_size) / 2; }
__device__ __forceinline__ uint64_t *ws_stamped_v(const Ctx &c) {
    return ws_stamped_k(c) + uni(c.sm->args.num_kv_heads) * uni(c.sm->args.head_dim) / 2;
}
__device__ __forceinline__ long long spin_ticks(const Ctx &c) {
    const long long v = c.sm->k.spin_ticks;
    return ((long long)uni((int)(v >> 32)) << 32) | (uint32_t)uni((int)v);
}

// Timing slots written per instruction by the controller when MK_FLAG_TIMINGS is set (low 32 bits
// of the device's 100 MHz wall clock, the same clock on every compute unit; counterpart of the
// reference's timing events, include/util.cuh:215-246).
enum {
    kEvStart = MK_TIMING_START, kEvDepReady = MK_TIMING_DEPENDENCY_READY, kEvInputReady = MK_TIMING_INPUT_READY,
    kEvComputeDone = MK_TIMING_COMPUTE_DONE, kEvEnd = MK_TIMING_END, kEvOpcode = MK_TIMING_OPCODE
};

// stamp by the controller wave
__device__ __forceinline__ void trace_event(const Ctx &c, int slot) {
    if (c.trace && c.controller && c.lane == 0) st_plain_i32(c.trace + slot, (int)(uint32_t)wall_clock64());
}
// the same moment in two slots (a stage of this kernel that is also one of the reference's events)
__device__ __forceinline__ void trace_event(const Ctx &c, int slot, int also) {
    if (c.trace && c.controller && c.lane == 0) {
        const int now = (int)(uint32_t)wall_clock64();
        st_plain_i32(c.trace + slot, now);
        st_plain_i32(c.trace + also, now);
    }
}
// stamp by whichever wave calls it (the waves that stream rows, or that store in attention)
__device__ __forceinline__ void trace_wave(const Ctx &c, int slot) {
    if (c.trace && c.lane == 0) st_plain_i32(c.trace + slot, (int)(uint32_t)wall_clock64());
}
// a consumer wave starts on its first row / is done with its last (one pair of slots per wave); wave 0
// also stands for the instruction's first and last use of a weight row
__device__ __forceinline__ void trace_consumer_first_use(const Ctx &c) {
    if (c.trace && c.lane == 0 && c.wave < MK_TIMING_CONSUMER_WAVES) {
        const int now = (int)(uint32_t)wall_clock64();
        st_plain_i32(c.trace + MK_TIMING_CONSUMER_START + 2 * c.wave, now);
        if (c.wave == 0) st_plain_i32(c.trace + MK_TIMING_FIRST_USE, now);
    }
}
__device__ __forceinline__ void trace_consumer_last_use(const Ctx &c) {
    if (c.trace && c.lane == 0 && c.wave < MK_TIMING_CONSUMER_WAVES) {
        const int now = (int)(uint32_t)wall_clock64();
        st_plain_i32(c.trace + MK_TIMING_CONSUMER_START + 2 * c.wave + 1, now);
        if (c.wave == 0) st_plain_i32(c.trace + MK_TIMING_LAST_USE, now);
    }
}
// wave 0 requested the instruction's first / its own last weight row
__device__ __forceinline__ void trace_first_load(const Ctx &c) {
    if (c.trace && c.lane == 0 && c.wave == 0) {
        const int now = (int)(uint32_t)wall_clock64();
        st_plain_i32(c.trace + MK_TIMING_LOADER_START, now);
        st_plain_i32(c.trace + MK_TIMING_FIRST_LOAD, now);
    }
}
__device__ __forceinline__ void trace_last_load(const Ctx &c) {
    if (c.trace && c.lane == 0 && c.wave == 0) st_plain_i32(c.trace + MK_TIMING_LAST_LOAD, (int)(uint32_t)wall_clock64());
}
// epilogue stages of the wave that stores and signals
__device__ __forceinline__ void trace_store_issue(const Ctx &c) {
    if (c.trace && c.lane == 0) {
        const int now = (int)(uint32_t)wall_clock64();
        st_plain_i32(c.trace + MK_TIMING_STORER_START, now);
        st_plain_i32(c.trace + MK_TIMING_AT_GMEM_STORE, now);
        st_plain_i32(c.trace + MK_TIMING_FIRST_STORE, now);
    }
}
__device__ __forceinline__ void trace_store_done(const Ctx &c) {
    if (c.trace && c.lane == 0) {
        const int now = (int)(uint32_t)wall_clock64();
        st_plain_i32(c.trace + MK_TIMING_DONE_GMEM_STORE, now);
        st_plain_i32(c.trace + MK_TIMING_LAST_STORE, now);
    }
}
__device__ __forceinline__ void trace_signalled(const Ctx &c) { trace_wave(c, MK_TIMING_OUTPUT_READY); }

__device__ __forceinline__ int *bar_ptr(const Ctx &c, int layer, int row, int col) {
    return uni(c.sm->args.barriers) + ((size_t)layer * MK_BARRIER_ROWS + row) * uni(c.sm->k.cols) + col;
}
// [replica][shard][layer][row]: the shards of one counter lie in different cache lines
// Barrier rows 0 (QKV blocks per head) and 1 (attention partitions per head) while the kernel runs.
// In `barriers` the counters of all heads share two cache lines; hundreds of arrivals within a
// microsecond then queue up behind each other (same-line atomics are served one at a time) and
// the waiting side sees its own head complete late.  Here every counter has a line of its own.
__device__ __forceinline__ int *pad_ptr(const Ctx &c, int layer, int row, int col) {
    return uni(c.sm->k.pads) + ((size_t)(layer * 2 + row) * uni(c.sm->k.pad_cols) + col) * kPadInts;
}
__device__ __forceinline__ int *shard_ptr(const Ctx &c, int replica, int shard, int layer, int row) {
    const int L = uni(c.sm->args.num_layers);
    return ws_shards(c) + (((size_t)replica * kShards + shard) * L + layer) * kHotRows + (row - 2);
}

// first error wins
__device__ void record_status(const Ctx &c, int code) {
    int expected = 0;
    int *status = ws_status(c);
    if (__hip_atomic_compare_exchange_strong(as_global(&status[0]), &expected, code, __ATOMIC_RELAXED, __ATOMIC_RELAXED, AG)) {
        st_i32(&status[1], c.worker);
        st_i32(&status[2], c.sm->window_base + c.slot);
        st_i32(&status[3], c.opcode);
    }
}

// First round of a dependency wait, requested ahead of time: the values this lane saw.
struct PollTicket {
    const int *ptr;
    int value, status;
    int base;  // what the counter's word in `barriers` held when the launch started (it does not move during one)
};
__device__ __forceinline__ PollTicket poll_issue(const Ctx &c, const int *ptr, const int *in_barriers = nullptr) {
    PollTicket t;
    t.ptr = ptr;
    t.value = ptr ? ld_i32(ptr) : 0;
    t.base = in_barriers ? ld_i32(in_barriers) : 0;
    t.status = c.lane == 63 ? ld_i32(ws_status(c)) : 0;
    return t;
}

// Executed by all lanes of the controller wave.  The ticket holds this lane's counter (or nullptr)
// and the first values read from it.
// sum_mode: wait until the sum over lanes reaches target (sharded counter + its base value);
// otherwise wait until every lane's counter reaches target.  Lane 63 watches the global status
// word so that one worker's failure releases everybody.
// `not_yet` is called once if the first look finds the dependency unsatisfied.
template <class NotYet>
__device__ __forceinline__ bool poll_wait(const Ctx &c, PollTicket t, bool sum_mode, int target, NotYet not_yet) {
    const long long t0 = wall_clock64();
    const long long limit = spin_ticks(c);
    const int *status = ws_status(c);
    int v = t.value, st = t.status;
    bool first = true;
    int held = 0;
    const int hold_looks = sum_mode ? uni(c.sm->k.hold_looks) : 0;
    while (true) {
        const int arrived = sum_mode ? lane_sum_i32(v) : 0;
        const bool ok = sum_mode ? (arrived >= target) : (bool)__all(t.ptr == nullptr || v + t.base >= target);
        if (ok) break;
        // Nearly everybody has arrived: the rest is a microsecond away.  The bulk requests that `not_yet`
        // releases would hold up the next looks and the fetch of the vector behind them (a CU serves its
        // requests in order), so they wait for up to two more looks - where the step is a chain of
        // hand-overs (the slowest worker of a phase, which arrives last, sees its dependency 1.5 µs
        // earlier); where the phases are bounded by memory, holding requests back only loses bandwidth.
        const bool hold = first && held < hold_looks && arrived * 32 >= target * MK_HOLD_SHARE;
        if (hold) held++;
        if (first && !hold) {
            not_yet();
            first = false;
        }
        if (__any(st != 0)) return false;
        if (wall_clock64() - t0 > limit) {
            if (c.lane == 0) record_status(c, MK_STATUS_BARRIER_TIMEOUT);
            return false;
        }
        // a quarter microsecond between looks: more looks (or two in flight) only add traffic on
        // the counters' memory channels and make the step slower
        if (!(hold && MK_HOLD_NOSLEEP)) __builtin_amdgcn_s_sleep(MK_POLL_SLEEP);
        v = t.ptr ? ld_i32(t.ptr) : 0;
        st = c.lane == 63 ? ld_i32(status) : 0;
    }
    compiler_fence();  // data loads stay after the successful poll
    return true;
}
__device__ bool poll_counters(const Ctx &c, const int *ptr, const int *in_barriers, bool sum_mode, int target) {
    return poll_wait(c, poll_issue(c, ptr, in_barriers), sum_mode, target, []() {});
}

// Stamp of what one layer writes in one decode step: differs from whatever an entry held before (an
// earlier layer or step, or the zero of a fresh workspace).
__device__ __forceinline__ uint32_t layer_stamp(const Ctx &c, int layer) {
    const uint32_t step = (uint32_t)uni((int)c.sm->k.epoch);
    const uint32_t stamp = step * (uint32_t)uni(c.sm->args.num_layers) + (uint32_t)layer + 1u;
    return stamp ? stamp : 1u;
}
// One bf16 pair of a stamped copy: a single 8-byte store, so whoever sees the stamp sees the value.
__device__ __forceinline__ void st_stamped(uint64_t *vec, int pair, uint32_t value, uint32_t stamp) {
    st_u64(vec + pair, ((uint64_t)stamp << 32) | value);
}

// The decoded counters of the instruction in the context's slot, as scalars.
struct SyncInfo {
    const int *poll_base, *bar_word;
    int *signal_base;
    int target;
};
__device__ __forceinline__ SyncInfo sync_info(const Ctx &c) {
    const MK_LDS u32x4 *src = (const MK_LDS u32x4 *)&c.sm->sync[c.slot];
    const u32x4 lo = src[0], hi = src[1];
    auto ptr = [](uint32_t l, uint32_t h) {
        return (int *)(uintptr_t)(((uint64_t)(uint32_t)uni((int)h) << 32) | (uint32_t)uni((int)l));
    };
    return SyncInfo{ptr(lo.x, lo.y), ptr(lo.z, lo.w), ptr(hi.x, hi.y), uni((int)hi.z)};
}
// first look at a sharded dependency counter: lanes 0 .. kShards - 1 one shard each, lane kShards the
// word in `barriers` (what the counter held before the launch), lane 63 the status word
__device__ __forceinline__ PollTicket poll_issue(const Ctx &c, const SyncInfo &sy) {
    const int *ptr = nullptr;
    if (sy.poll_base) {
        if (c.lane < kShards) ptr = sy.poll_base + c.lane * uni(c.sm->k.shard_stride);
        else if (c.lane == kShards) ptr = sy.bar_word;
    }
    return poll_issue(c, ptr);
}
// one arrival on the counter the instruction signals; the caller has waited for its stores
__device__ __forceinline__ void signal_sharded(const Ctx &c, const SyncInfo &sy, int count) {
    if (c.lane == 0) {
        const int stride = uni(c.sm->k.replica_stride);
#pragma unroll
        for (int r = 0; r < kReplicas; r++) add_i32(sy.signal_base + (size_t)r * stride, count);
    }
}

__device__ __forceinline__ const int *sharded_lane_ptr(const Ctx &c, int layer, int row) {
    // 256 workers reading the same 16 lines every quarter microsecond queue up at those lines'
    // memory channels; with four copies each line has a quarter of the readers
    if (c.lane < kShards) return shard_ptr(c, (c.worker / kShards) % kReplicas, c.lane, layer, row);
    if (c.lane == kShards) return bar_ptr(c, layer, row, 0);
    return nullptr;
}
__device__ __forceinline__ bool poll_sharded(const Ctx &c, int layer, int row, int target) {
    return poll_counters(c, sharded_lane_ptr(c, layer, row), nullptr, true, target);
}

// one arrival on a sharded counter; the caller has waited for its stores
__device__ __forceinline__ void signal_sharded_lane(const Ctx &c, int layer, int row, int count) {
#pragma unroll
    for (int r = 0; r < kReplicas; r++) add_i32(shard_ptr(c, r, c.worker & (kShards - 1), layer, row), count);
}
__device__ __forceinline__ void signal_sharded(const Ctx &c, int layer, int row, int count) {
    if (c.lane == 0) signal_sharded_lane(c, layer, row, count);
}

// Controller: publish the outcome of the dependency wait; everybody: first barrier of the
// instruction.  Returns false when the launch is being abandoned.
__device__ __forceinline__ bool barrier_inputs_ready(const Ctx &c, bool controller_ok) {
    if (c.controller && !controller_ok && c.lane == 0) c.sm->abort = 1;
    wg_barrier();
    return c.sm->abort == 0;
}

// ---------------------------------------------------------------------------------------------
// matvec core
// ---------------------------------------------------------------------------------------------
template <int KC>
struct XVec {
    float v[KC][8];
};

__device__ __forceinline__ void unpack8(const uint4 &r, float (&o)[8]) {
    o[0] = mkm::bf16_lo(r.x); o[1] = mkm::bf16_hi(r.x);
    o[2] = mkm::bf16_lo(r.y); o[3] = mkm::bf16_hi(r.y);
    o[4] = mkm::bf16_lo(r.z); o[5] = mkm::bf16_hi(r.z);
    o[6] = mkm::bf16_lo(r.w); o[7] = mkm::bf16_hi(r.w);
}

// activation vector written earlier in this launch by other CUs: coherent loads
template <int KC>
__device__ __forceinline__ void load_x(XVec<KC> &x, const uint16_t *src, int lane) {
    uint4 raw[KC];
#pragma unroll
    for (int j = 0; j < KC; j++) raw[j] = ld_b128(src + j * 512 + lane * 8);
#pragma unroll
    for (int j = 0; j < KC; j++) unpack8(raw[j], x.v[j]);
}

// Sum of the 8 per-lane column accumulators, pairwise in column order.
__device__ __forceinline__ float fold8(const float (&a)[8]) {
    return ((a[0] + a[1]) + (a[2] + a[3])) + ((a[4] + a[5]) + (a[6] + a[7]));
}

// python_vm.py:50-56: w * bf16(x * rsqrt(mean(x^2) + eps)), statistics in fp32.  Result as bf16 pairs.
// Sum of squares in column order: column c = lane * 8 + e accumulates its elements j * 512 + c in
// order of j, the 512 columns are added as a balanced pairwise tree.
template <int KC>
__device__ __forceinline__ void rms_norm_x(uint4 (&xq)[KC], const uint4 (&xraw)[KC], const uint4 (&wraw)[KC], float eps) {
    // the vector stays packed (bf16 pairs, half the registers) and is widened chunk by chunk, twice
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < KC; j++) {
        float xv[8];
        unpack8(xraw[j], xv);
#pragma unroll
        for (int e = 0; e < 8; e++) acc[e] = fmaf(xv[e], xv[e], acc[e]);
    }
    const float mean = wave_tree_sum_uniform(fold8(acc)) / (float)(KC * 512);
    const float inv = 1.0f / sqrtf(mean + eps);
#pragma unroll
    for (int j = 0; j < KC; j++) {
        float wv[8], xv[8], y[8];
        unpack8(wraw[j], wv);
        unpack8(xraw[j], xv);
#pragma unroll
        for (int e = 0; e < 8; e++) y[e] = wv[e] * mkm::round_bf16(xv[e] * inv);
        xq[j].x = mkm::pack_bf16(y[0], y[1]);
        xq[j].y = mkm::pack_bf16(y[2], y[3]);
        xq[j].z = mkm::pack_bf16(y[4], y[5]);
        xq[j].w = mkm::pack_bf16(y[6], y[7]);
    }
}

// activation vector written earlier in this launch by other CUs, kept as bf16 pairs
template <int KC>
__device__ __forceinline__ void load_xq(uint4 (&xq)[KC], const uint16_t *src, int lane) {
#pragma unroll
    for (int j = 0; j < KC; j++) xq[j] = ld_b128(src + j * 512 + lane * 8);
}

// controller -> consumers hand-over of the activation vector: each lane's 16 bytes of a chunk are
// adjacent to its neighbours', so the 128-bit LDS accesses are free of bank conflicts
template <int KC>
__device__ __forceinline__ void x_to_lds(const uint4 (&xq)[KC], MK_LDS uint32_t *dst, int lane) {
#pragma unroll
    for (int j = 0; j < KC; j++)
        *(MK_LDS u32x4 *)(dst + (j * 64 + lane) * 4) = u32x4{xq[j].x, xq[j].y, xq[j].z, xq[j].w};
}
template <int KC>
__device__ __forceinline__ void x_to_lds(const uint4 (&xq)[KC], SmemPtr sm, int lane) {
    x_to_lds<KC>(xq, (MK_LDS uint32_t *)sm->x, lane);
}
// the consumers keep the vector as it lies in LDS: bf16 pairs, 4 dwords per lane and chunk
template <int KC>
struct XPairs {
    uint4 v[KC];
};
template <int KC>
__device__ __forceinline__ void x_from_lds(XPairs<KC> &x, const MK_LDS uint32_t *src, int lane) {
#pragma unroll
    for (int j = 0; j < KC; j++) {
        const u32x4 r = *(const MK_LDS u32x4 *)(src + (j * 64 + lane) * 4);
        x.v[j] = uint4{r.x, r.y, r.z, r.w};
    }
}
template <int KC>
__device__ __forceinline__ void x_from_lds(XPairs<KC> &x, SmemPtr sm, int lane) {
    x_from_lds<KC>(x, (const MK_LDS uint32_t *)sm->x, lane);
}

// A weight row of an instruction: a buffer resource (uniform) and the row's byte offset in it.
struct WeightBuffer {
    const uint16_t *base;
    uint32_t bytes;
};
struct RowRef {
    WeightBuffer buffer;
    uint32_t offset;
};
__device__ __forceinline__ WeightBuffer weight_buffer(const uint16_t *base, size_t bytes) {
    return WeightBuffer{uni(base), (uint32_t)uni((int)bytes)};
}
constexpr uint32_t kNoRow = 0x80000000u;  // beyond any buffer: the load returns zeros and fetches nothing

// Request one row (KC x 16 bytes per lane), streaming.  `valid` false turns the request into a no-op
// that still counts as KC loads, which keeps the number of outstanding loads independent of the
// data: every lane asks for an address beyond the buffer, which returns zeros and fetches nothing.
// A no-op is not free (it occupies the CU's address path like a real row), so the callers arrange
// for few of them.
template <int KC>
__device__ __forceinline__ void load_row(uint4 (&w)[KC], const RowRef &r, bool valid, int lane) {
    const uint32_t off = valid ? r.offset + lane * 16 : kNoRow;
    // the descriptor lives in scalar registers; which buffer a row comes from is the same for the
    // whole wave, and readfirstlane says so
    const __amdgpu_buffer_rsrc_t rsrc =
        __builtin_amdgcn_make_buffer_rsrc((void *)uni(r.buffer.base), 0, uni((int)r.buffer.bytes), 0x00020000);
#pragma unroll
    for (int j = 0; j < KC; j++) {
        const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, off, j * 1024, MK_STREAM_AUX);
        w[j] = uint4{v.x, v.y, v.z, v.w};
    }
}
// plain row load for the small per-instruction vectors (norm weights)
template <int KC>
__device__ __forceinline__ void load_row(uint4 (&w)[KC], const uint16_t *row, int lane) {
#pragma unroll
    for (int j = 0; j < KC; j++) w[j] = ld_const_b128(row + j * 512 + lane * 8);
}

// acc + w.lo * x.lo + w.hi * x.hi for two bf16 pairs: the two-element dot product instruction.  Its
// arithmetic is not a chain of IEEE operations (the addends are aligned and truncated to a fixed
// window before one final rounding); mk_llama_selftest_dot2 checks the written-out definition against it.
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float dot2_bf16(uint32_t w, uint32_t x, float acc) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, w), __builtin_bit_cast(bf16x2, x), acc, false);
}

// dot(w, x) in pair-column order: pair column c = lane * 4 + d accumulates the element pairs
// j*256 + c (elements 2(j*256+c) and the next) over j with the two-element dot product from 0; the
// 256 pair columns are added as a balanced pairwise tree.
template <int KC>
__device__ __forceinline__ float dot_row(const uint4 (&w)[KC], const XPairs<KC> &x) {
    float acc[4] = {0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < KC; j++) {
        acc[0] = dot2_bf16(w[j].x, x.v[j].x, acc[0]);
        acc[1] = dot2_bf16(w[j].y, x.v[j].y, acc[1]);
        acc[2] = dot2_bf16(w[j].z, x.v[j].z, acc[2]);
        acc[3] = dot2_bf16(w[j].w, x.v[j].w, acc[3]);
    }
    return wave_tree_sum_uniform((acc[0] + acc[1]) + (acc[2] + acc[3]));
}

// One batch of a matvec instruction.
//   consumers : request the first rows, barrier (activation vector ready), stream `ntasks` rows
//               (task t -> wave t % 8, result bf16-rounded into sm->out[t]), barrier (results ready)
//   controller: `prepare` (wait for the dependency, build the activation vector in LDS; returns
//               false to abandon), barrier, `overlap`, barrier, `finish` (epilogue + signal)
// Both barriers are reached by all nine waves whatever the outcome of `prepare`.
// The controller's side of one matvec instruction (or one batch of the LM head).
template <class Ahead, class Prepare, class Overlap, class Finish>
__device__ __forceinline__ bool controller_sequence(const Ctx &c, Ahead ahead, Prepare prepare, Overlap overlap,
                                                    Finish finish) {
    // A CU serves its memory requests in order, and the consumers' first requests are bulky.  So
    // the controller's first requests (first look at the dependency, norm weights) go out before
    // them, and the consumers are released (entry barrier) either when that first look says "not
    // yet" - there is time, prefetch away - or, when the dependency is already satisfied, right
    // after the controller has requested the activation vector.  A worker that arrives late then
    // has its short critical requests ahead of its own prefetch instead of behind it.
    ahead();
    trace_event(c, MK_TIMING_AT_GMEM_WAIT);
    bool released = false;
    auto release = [&]() {
        if (!released) wg_barrier();
        released = true;
    };
    const bool ok = prepare(release);
    release();
    trace_event(c, kEvInputReady, MK_TIMING_LAUNCHER_START);
    if (!barrier_inputs_ready(c, ok)) return false;
    overlap();  // runs while the consumers stream rows: fetch what the epilogue will need
    wg_barrier();
    trace_event(c, kEvComputeDone);
    finish();
    // the consumers hold their next requests back until the results and the signal are on their way
    wg_barrier();
    return true;
}

__device__ __forceinline__ int rows_of_wave(int ntasks, int wave) {
    return ntasks > wave ? (ntasks - wave + kConsumerWaves - 1) / kConsumerWaves : 0;
}

template <int KC, int PF, class RowOf, class Ahead, class Prepare, class Overlap, class Finish>
__device__ __forceinline__ bool matvec_batch(const Ctx &c, int ntasks, bool need_x, RowOf row_ref, Ahead ahead,
                                             Prepare prepare, Overlap overlap, Finish finish) {
    if (c.controller) return controller_sequence(c, ahead, prepare, overlap, finish);
    const int mine = rows_of_wave(ntasks, c.wave);
    uint4 buf[PF][KC];
    // Requests are issued unconditionally wherever rows stream (rows past the end become no-op
    // requests), so the count of outstanding loads at each wait is a compile-time constant: the
    // wait for row i leaves the PF - 1 younger rows in flight.
    auto request = [&](uint4 (&dst)[KC], int i) {
        const bool valid = i < mine;
        load_row<KC>(dst, row_ref(valid ? c.wave + i * kConsumerWaves : 0), valid, c.lane);
    };
    auto consume = [&](const uint4 (&src)[KC], int i, const XPairs<KC> &x) {
        const float y = mkm::round_bf16(dot_row<KC>(src, x));
        if (c.lane == 0) c.sm->out[c.wave + i * kConsumerWaves] = y;
    };
    wg_barrier();  // entry: the controller's first requests are out
    trace_first_load(c);
#pragma unroll
    for (int s = 0; s < PF; s++) request(buf[s], s);
    if (!barrier_inputs_ready(c, true)) return false;
    XPairs<KC> x;
    if (need_x) x_from_lds<KC>(x, c.sm, c.lane);
    trace_consumer_first_use(c);
    int base = 0;
    // rounds that are followed by more rows: every row of the round exists, every slot is refilled
    for (; base + PF < mine; base += PF) {
#pragma unroll
        for (int s = 0; s < PF; s++) {
            consume(buf[s], base + s, x);
            compiler_fence();
            request(buf[s], base + s + PF);
            compiler_fence();
        }
    }
    trace_last_load(c);
    // last round: nothing left to request
#pragma unroll
    for (int s = 0; s < PF; s++)
        if (base + s < mine) consume(buf[s], base + s, x);
    trace_consumer_last_use(c);
    wg_barrier();
    // hold the next instruction's weight requests back until the controller has sent this
    // instruction's results and signal: they would otherwise queue behind the bulk loads
    wg_barrier();
    return true;
}

// malformed instruction: every wave evaluates the same condition and leaves; the controller records it
__device__ __forceinline__ bool bail(const Ctx &c, int code, int *refusal) {
    if (c.controller && c.lane == 0) {
        record_status(c, code);
        c.sm->abort = code;
    }
    *refusal = code;
    return false;
}

// ---------------------------------------------------------------------------------------------
// The four matvec instructions (opcodes 1, 4, 5, 6).
//
// describe_matvec() turns an instruction into what the consumer waves need: how many rows, and
// where each row lives.  control_*() is the controller's side of one instruction: dependency
// wait, activation vector into LDS, epilogue, signal.  op_matvec() is the handler: the consumer
// waves request their first rows on entry (the prefetch that overlaps the dependency wait), then
// stream the rest.  (Requesting rows of the *following* instructions as well - a row stream across
// instruction boundaries, or up/gate, down and QKV rows fetched while attention runs - was built
// and measured: the bulk requests delay the short latency-critical ones of the instructions in
// between, and a decode step got 5 % slower.)
// ---------------------------------------------------------------------------------------------
struct MatvecDesc {
    int opcode, ntasks, first_row;
    WeightBuffer w0;
    long long gate_delta;  // opcode 5: byte distance from the up matrix (w0) to the gate matrix
    uint32_t row_bytes;
    InsPtr ins;
};

// Joint execution of a residual projection's column-group jobs (MK_FLAG_JOINT_RESIDUAL: the caller
// promises that for every row block either all G column groups' jobs are in the instruction tensor
// or none).  The G jobs of a block then share the work by rows instead of by columns: the job of
// group c computes rows [c * 16 / G, (c + 1) * 16 / G) of the block over all G column groups, so it
// holds every group's partial sum of its rows and applies them to the residual itself, in group order
// - no partial sums travel between workers and no job waits for another.  Results and barrier counts
// are those of the instruction-by-instruction execution.  Task t of such a job: block t / 16, row
// (t % 16) / G of the job's rows, column group t % G; a wave's tasks (t = wave mod 8) all have column
// group wave % G, so the wave keeps that group's slice of the activation vector in registers.
//
// A worker often holds several of a block's G jobs one after the other in its queue (round-robin
// assignment of a model with G = 2 gives it both).  Jointly executed they are one piece of work - rows
// [c * 16 / G, (c + n) * 16 / G) of the block for the n jobs from group c on - with one dependency, one
// activation vector and one epilogue: the first of the run executes all of them (n = 1, 2 or 4) and
// signals n arrivals per block, and the others become no-ops when the queue window is decoded.
// Models whose residual projections take several column groups of the hidden width (8B) stream their QKV
// rows in a phase that ends with the workers that hold one block more than the others: those share.
template <class Args>
__device__ __forceinline__ bool shares_qkv_blocks(const Args &a) { return MK_SHARE_QKV && a.hidden_size != a.matvec_reduction_size; }
template <class Args>
__device__ __forceinline__ int qkv_counter_unit(const Args &a) { return shares_qkv_blocks(a) ? 2 : 1; }
constexpr int kAbsorbed = -2;  // SlotDesc::ntasks of a job that an earlier job of its block executes
__host__ __device__ constexpr bool joint_groups(uint32_t flags, int G, int in_dim) {
    return (flags & MK_FLAG_JOINT_RESIDUAL) != 0 && G > 1 && 16 % G == 0 && G <= 4 &&
           (size_t)in_dim * 2 <= sizeof(Smem::scores);
}

// Decodes the matvec instruction in queue slot `slot` (executed once per launch by one thread per
// slot; the launch arguments come from the kernel's argument registers).
__device__ __forceinline__ void decode_matvec(SmemPtr sm, int slot, ArgsRef a) {
    const InsPtr ins = sm->queue[slot];
    const int hid = a.hidden_size, inter = a.intermediate_size;
    const int opcode = ins[0], layer = ins[1];
    SlotDesc d;
    d.w0_base = 0;
    d.gate_delta = 0;
    d.w0_bytes = d.row_bytes = 0;
    d.ntasks = -1;
    d.first_row = 0;
    if (layer >= 0 && layer < a.num_layers) {
        if (opcode == 1) {
            const int start = ins[2], end = ins[3];
            const int total_blocks = (a.num_attention_heads + 2 * a.num_kv_heads) * a.head_dim / 16;
            if (start >= 0 && end <= total_blocks && end - start <= kOutRows / 16) {
                const int nblk = end > start ? end - start : 0;
                d.ntasks = nblk * 16;
                // Sharing with the partner worker (share_setup): both have exactly one QKV instruction for
                // the layer and their block counts differ by one.  The one with more computes rows 0-7 of
                // its last block only, the other rows 8-15 of that block as well.
                if (layer < kShareLayers && sm->qkv_count[0][layer] == 1 && sm->qkv_count[1][layer] == 1 &&
                    (sm->qkv_info[0][layer] >> 20) == nblk) {
                    const int theirs = sm->qkv_info[1][layer], n_p = theirs >> 20, last_p = theirs & 0xfffff;
                    if (n_p == nblk + 1 && last_p < total_blocks && nblk * 16 + 8 <= kOutRows) {
                        d.gate_delta = (last_p << 2) | 2;
                        d.ntasks += 8;
                    } else if (n_p == nblk - 1) {
                        d.gate_delta = ((end - 1) << 2) | 1;
                        d.ntasks -= 8;
                    }
                }
                d.first_row = start * 16;
                d.row_bytes = (uint32_t)hid * 2u;
                d.w0_base = (uint64_t)(uintptr_t)(a.qkv_weights + (size_t)layer * total_blocks * 16 * hid);
                d.w0_bytes = (uint32_t)((size_t)total_blocks * 16 * hid * 2);
            }
        } else if (opcode == 4 || opcode == 6) {
            const bool is_down = opcode == 6;
            const int start = ins[2], end = ins[3], group = ins[4];
            const int R = a.matvec_reduction_size, in_dim = is_down ? inter : hid;
            if (start >= 0 && end <= hid / 16 && group >= 0 && group < in_dim / R && end - start <= kOutRows / 16) {
                const int G = in_dim / R;
                d.ntasks = (end > start ? end - start : 0) * 16;
                d.row_bytes = (uint32_t)in_dim * 2u;
                const uint16_t *matrix = (is_down ? a.down_weights : a.o_weights) + (size_t)layer * hid * in_dim;
                if (joint_groups(a.flags, G, in_dim)) {
                    // joint execution: this job takes 16 / G rows of each of its blocks over all G column groups
                    d.first_row = start * 16 + group * (16 / G);
                    d.w0_base = (uint64_t)(uintptr_t)matrix;
                    d.w0_bytes = (uint32_t)((size_t)hid * in_dim * 2);
                    // The run of jobs of the same blocks, with consecutive groups, that this one is part of:
                    // slots [lo, hi).  It executes in pieces of 4, 2 or 1 jobs from its start; the first
                    // job of a piece does the work.  (Timing records are kept per instruction: none of this
                    // in a launch that takes them.)
                    auto follows = [&](int s) {  // is slot s the job after slot s - 1's?
                        const InsPtr p = sm->queue[s - 1], q = sm->queue[s];
                        return q[0] == p[0] && q[1] == p[1] && q[2] == p[2] && q[3] == p[3] && q[4] == p[4] + 1 && q[4] < G;
                    };
                    int run = 1;
                    if (!(a.flags & MK_FLAG_TIMINGS) && end > start && MK_RUN_JOBS) {
                        const int count = sm->window_count;
                        int lo = slot, hi = slot + 1;
                        while (lo > 0 && slot - lo < G && follows(lo)) lo--;
                        while (hi < count && hi - lo < G && follows(hi)) hi++;
                        for (int at = lo; at < hi;) {
                            // (what a piece computes must fit the result buffer)
                            const int left = hi - at, room = kOutRows / ((end - start) * 16);
                            const int piece = left >= 4 && room >= 4 ? 4 : left >= 2 && room >= 2 ? 2 : 1;
                            if (slot == at) run = piece;
                            else if (slot > at && slot < at + piece) run = 0;
                            at += piece;
                        }
                    }
                    d.gate_delta = G | (run << 8);
                    d.ntasks = run ? d.ntasks * run : kAbsorbed;
                } else {
                    d.first_row = start * 16;
                    // the buffer starts at this column group's first element of the layer's matrix
                    d.w0_base = (uint64_t)(uintptr_t)(matrix + (size_t)group * R);
                    d.w0_bytes = (uint32_t)(((size_t)(hid - 1) * in_dim + R) * 2);
                }
            }
        } else if (opcode == 5) {
            const int n = ins[2];
            bool ok = n >= 0 && n <= MK_INSTRUCTION_WORDS - 3 && n * 32 <= kOutRows;
            for (int i = 0; ok && i < n; i++) ok = ins[3 + i] >= 0 && ins[3 + i] < inter / 16;
            if (ok) {
                d.ntasks = n * 32;
                d.row_bytes = (uint32_t)hid * 2u;
                const uint16_t *up = a.up_weights + (size_t)layer * inter * hid;
                const uint16_t *gate = a.gate_weights + (size_t)layer * inter * hid;
                d.w0_base = (uint64_t)(uintptr_t)up;
                d.w0_bytes = (uint32_t)((size_t)inter * hid * 2);
                d.gate_delta = (long long)((uintptr_t)gate - (uintptr_t)up);
            }
        }
    }
    MK_LDS u32x4 *dst = (MK_LDS u32x4 *)&sm->desc[slot];
    dst[0] = u32x4{(uint32_t)d.w0_base, (uint32_t)(d.w0_base >> 32), (uint32_t)d.gate_delta, (uint32_t)((uint64_t)d.gate_delta >> 32)};
    dst[1] = u32x4{d.w0_bytes, d.row_bytes, (uint32_t)d.ntasks, (uint32_t)d.first_row};
}

// Where the counters of the instruction in queue slot `slot` live (opcodes 1, 4, 5, 6, 7; executed once
// per launch by one thread per slot).  An instruction whose layer is out of range gets no counters; its
// handler refuses it before it looks at them.
__device__ __forceinline__ void decode_sync(SmemPtr sm, int slot, ArgsRef a) {
    const InsPtr ins = sm->queue[slot];
    const int opcode = ins[0], L = a.num_layers;
    const int layer = opcode == 7 ? L - 1 : ins[1];
    int wait_layer = -1, wait_row = 2, target = 0, signal_layer = -1, signal_row = 2;
    if (layer >= 0 && layer < L) {
        const int down_jobs = (a.intermediate_size / a.matvec_reduction_size) * (a.hidden_size / 16);
        switch (opcode) {
        case 1:  // the previous layer's down projection (python_vm.py:176)
            if (layer > 0) { wait_layer = layer - 1; wait_row = 5; target = down_jobs; }
            break;
        case 4:  // all heads' attention output (python_vm.py:88-95); signals row 3
            wait_layer = layer; wait_row = 2; target = a.num_attention_heads;
            signal_layer = layer; signal_row = 3;
            break;
        case 5:  // the O projection (python_vm.py:132); signals row 4
            wait_layer = layer; wait_row = 3; target = (a.hidden_size / a.matvec_reduction_size) * (a.hidden_size / 16);
            signal_layer = layer; signal_row = 4;
            break;
        case 6:  // up / gate (python_vm.py:110); signals row 5
            wait_layer = layer; wait_row = 4; target = a.intermediate_size / 16;
            signal_layer = layer; signal_row = 5;
            break;
        default:  // 7: the last layer's down projection (python_vm.py:255)
            wait_layer = layer; wait_row = 5; target = down_jobs;
            break;
        }
    }
    const WsLayout w = ws_layout(L, a.hidden_size, a.intermediate_size, a.matvec_reduction_size);
    int *const shards = static_cast<int *>(a.workspace) + w.shards;
    const int cols = a.num_attention_heads + 2 * a.num_kv_heads;
    const int replica = ((int)blockIdx.x / kShards) % kReplicas, shard = (int)blockIdx.x & (kShards - 1);
    uint64_t poll_base = 0, bar_word = 0, signal_base = 0;
    if (wait_layer >= 0) {
        poll_base = (uint64_t)(uintptr_t)(shards + ((size_t)replica * kShards * L + wait_layer) * kHotRows + (wait_row - 2));
        bar_word = (uint64_t)(uintptr_t)(a.barriers + ((size_t)wait_layer * MK_BARRIER_ROWS + wait_row) * cols);
    }
    if (signal_layer >= 0)
        signal_base = (uint64_t)(uintptr_t)(shards + ((size_t)shard * L + signal_layer) * kHotRows + (signal_row - 2));
    MK_LDS u32x4 *dst = (MK_LDS u32x4 *)&sm->sync[slot];
    dst[0] = u32x4{(uint32_t)poll_base, (uint32_t)(poll_base >> 32), (uint32_t)bar_word, (uint32_t)(bar_word >> 32)};
    dst[1] = u32x4{(uint32_t)signal_base, (uint32_t)(signal_base >> 32), (uint32_t)target, 0u};
}

// The decoded form of the matvec instruction in `slot`; false: the instruction is malformed.
__device__ __forceinline__ bool describe_matvec(SmemPtr sm, int slot, int opcode, MatvecDesc &d) {
    const MK_LDS u32x4 *src = (const MK_LDS u32x4 *)&sm->desc[slot];
    const u32x4 lo = src[0], hi = src[1];
    d.ins = sm->queue[slot];
    d.opcode = opcode;
    d.w0.base = (const uint16_t *)(uintptr_t)(((uint64_t)(uint32_t)uni((int)lo.y) << 32) | (uint32_t)uni((int)lo.x));
    d.gate_delta = (long long)(((uint64_t)(uint32_t)uni((int)lo.w) << 32) | (uint32_t)uni((int)lo.z));
    d.w0.bytes = (uint32_t)uni((int)hi.x);
    d.row_bytes = (uint32_t)uni((int)hi.y);
    d.ntasks = uni((int)hi.z);
    d.first_row = uni((int)hi.w);
    return d.ntasks >= 0;
}

// row computed by task t of the instruction.  Opcode 5: task t is list entry t / 32, matrix
// (t / 16) & 1 (0 up, 1 gate), row t % 16 of that block.
__device__ __forceinline__ RowRef matvec_row(const MatvecDesc &d, int t) {
    if (d.opcode == 5) {
        const int blk = uni(d.ins[3 + (t >> 5)]);
        // the gate matrix has the up matrix's size; its buffer is the up buffer moved by a distance
        const long long shift = (t >> 4) & 1 ? d.gate_delta : 0;
        const WeightBuffer w = {(const uint16_t *)((uintptr_t)d.w0.base + (uintptr_t)shift), d.w0.bytes};
        return RowRef{w, (uint32_t)(blk * 16 + (t & 15)) * d.row_bytes};
    }
    if (d.opcode == 1) {
        // the last 8 tasks of a worker that helps its partner: rows 8-15 of the partner's last block
        const bool helps = ((int)d.gate_delta & 3) == 2 && t >= d.ntasks - 8;
        const int row = helps ? ((int)d.gate_delta >> 2) * 16 + 8 + (t - (d.ntasks - 8)) : d.first_row + t;
        return RowRef{d.w0, (uint32_t)row * d.row_bytes};
    }
    if (d.gate_delta > 0) {
        // jointly executed column-group jobs: G and the number of jobs are powers of two; a block is
        // 16 tasks per job
        const int G = (int)d.gate_delta & 0xff, shift = __builtin_ctz((unsigned)G);
        const int per_block = (int)(d.gate_delta >> 8) * 16, block_shift = __builtin_ctz((unsigned)per_block);
        const int row = d.first_row + (t >> block_shift) * 16 + ((t & (per_block - 1)) >> shift);
        return RowRef{d.w0, (uint32_t)row * d.row_bytes + (uint32_t)(t & (G - 1)) * (d.row_bytes >> shift)};
    }
    return RowRef{d.w0, (uint32_t)(d.first_row + t) * d.row_bytes};
}

// ---------------------------------------------------------------------------------------------
// opcode 1: RMSNorm + QKV matvec + RoPE + KV append  (python_vm.py:168-248;
// reference device op: demos/low-latency-llama/rms_matvec_rope_append.cu:10-231)
// ---------------------------------------------------------------------------------------------
// SHARE: the model is of the kind whose workers share QKV blocks (share_setup); its per-head counters
// count half blocks.
template <int KC, bool SHARE>
__device__ __forceinline__ bool control_qkv(const Ctx &c) {
    const InsPtr ins = c.sm->queue[c.slot];
    ArgsRef a = c.sm->args;
    const int layer = ins[1], start = ins[2], end = ins[3];
    const int hid = a.hidden_size, D = a.head_dim, H = a.num_attention_heads, KVH = a.num_kv_heads;
    const int nblk = end > start ? end - start : 0;
    const int k_start = H * D, v_start = k_start + KVH * D;
    // half a block shared with the partner worker (see decode_matvec): which, and which half
    const int share = SHARE ? uni((int)((const MK_LDS uint32_t *)&c.sm->desc[c.slot])[2]) : 0;
    const int share_mode = share & 3, share_block = share >> 2;
    const int own_rows = nblk * 16 - (share_mode == 1 ? 8 : 0);
    const int npairs = (own_rows + (share_mode == 2 ? 8 : 0)) / 2;   // one lane per pair of adjacent rows
    auto row0_of = [&](int p) { return p * 2 < own_rows ? start * 16 + p * 2 : share_block * 16 + 8 + (p * 2 - own_rows); };
    constexpr int kPre = 2;
    float rot[kPre][4] = {{1.0f, 1.0f, 0.0f, 0.0f}, {1.0f, 1.0f, 0.0f, 0.0f}};
    const bool prefetched = npairs <= kPre * 64;
    PollTicket ticket = {nullptr, 0, 0};
    const SyncInfo sy = sync_info(c);
    const uint32_t stamp = layer_stamp(c, layer);
    uint4 wraw[KC];
    return controller_sequence(
        c,
        [&]() {
            ticket = poll_issue(c, sy);
            if (npairs > 0) load_row<KC>(wraw, a.attn_norm_weights + (size_t)layer * hid, c.lane);
        },
        [&](auto release) {
            if (layer > 0 && !poll_wait(c, ticket, true, sy.target, release)) return false;
            trace_event(c, kEvDepReady, MK_TIMING_DONE_GMEM_WAIT);
            if (npairs > 0) {
                // layer 0 of a launch that was given a token reads the embedding row itself; the
                // worker holding the first block also makes it the residual stream (every later
                // reader of hidden_states waits, through attention, for this worker's signal)
                const bool from_table = layer == 0 && a.token_in != nullptr;
                const uint16_t *src = from_table ? a.embed_table + (size_t)c.sm->token * hid : a.hidden_states;
                uint4 x[KC];
                load_xq<KC>(x, src, c.lane);
                release();
                if (from_table && start == 0 && nblk > 0) {
#pragma unroll
                    for (int j = 0; j < KC; j++) {
                        uint16_t *dst = a.hidden_states + j * 512 + c.lane * 8;
                        st_u32(dst, x[j].x);
                        st_u32(dst + 2, x[j].y);
                        st_u32(dst + 4, x[j].z);
                        st_u32(dst + 6, x[j].w);
                    }
                }
                uint4 xq[KC];
                rms_norm_x<KC>(xq, x, wraw, a.rms_norm_eps);
                x_to_lds<KC>(xq, c.sm, c.lane);
            }
            return true;
        },
        [&]() {
            // the rotary factors of this lane's row pairs do not depend on the matvec: fetch them while
            // the consumers work
            if (prefetched) {
#pragma unroll
                for (int k = 0; k < kPre; k++) {
                    const int p = c.lane + k * 64;
                    const int row0 = row0_of(p);
                    if (p < npairs && row0 < v_start) {
                        const int d = row0 % D;
                        const float *cs = a.rope_cos + (size_t)a.pos_id * D + d;
                        const float *sn = a.rope_sin + (size_t)a.pos_id * D + d;
                        rot[k][0] = ld_const_f32(cs);
                        rot[k][1] = ld_const_f32(cs + 1);
                        rot[k][2] = ld_const_f32(sn);
                        rot[k][3] = ld_const_f32(sn + 1);
                    }
                }
            }
        },
        [&]() {
            // epilogue: one lane per adjacent row pair
            const size_t kv_row = ((size_t)layer * a.kv_max_len + a.pos_id) * KVH * D;
            auto emit = [&](int p, float c0, float c1, float s0, float s1) {
                const int row0 = row0_of(p);
                const float y0 = c.sm->out[p * 2], y1 = c.sm->out[p * 2 + 1];
                uint32_t packed;
                if (row0 < v_start) {
                    // interleaved rotary embedding (llama.py:136-174): products and sum in fp32, unfused
                    const float even = (y0 * c0) + ((-y1) * s0);
                    const float odd = (y1 * c1) + (y0 * s1);
                    packed = mkm::pack_bf16(even, odd);
                } else {
                    packed = mkm::pack_bf16(y0, y1);
                }
                uint16_t *dst;
                if (row0 < k_start) dst = a.q_post_rope + row0;
                else if (row0 < v_start) dst = a.k_cache + kv_row + (row0 - k_start);
                else dst = a.v_cache + kv_row + (row0 - v_start);
                st_u32(dst, packed);
                // and the stamped copy that attention looks for (query | K row | V row: the order of the rows)
                st_stamped(ws_stamped_q(c), row0 >> 1, packed, stamp);
            };
            if (prefetched) {
#pragma unroll
                for (int k = 0; k < kPre; k++)
                    if (c.lane + k * 64 < npairs) emit(c.lane + k * 64, rot[k][0], rot[k][1], rot[k][2], rot[k][3]);
            } else {
                for (int p = c.lane; p < npairs; p += 64) {
                    const int row0 = row0_of(p);
                    float c0 = 1.0f, c1 = 1.0f, s0 = 0.0f, s1 = 0.0f;
                    if (row0 < v_start) {
                        const int d = row0 % D;
                        const float *cs = a.rope_cos + (size_t)a.pos_id * D + d;
                        const float *sn = a.rope_sin + (size_t)a.pos_id * D + d;
                        c0 = ld_const_f32(cs); c1 = ld_const_f32(cs + 1); s0 = ld_const_f32(sn); s1 = ld_const_f32(sn + 1);
                    }
                    emit(p, c0, c1, s0, s1);
                }
            }
            trace_store_issue(c);
            wait_stores();
            trace_store_done(c);
            // One arrival per block on its head's counter (python_vm.py:248).  Where blocks can be shared the
            // counters count half blocks while the kernel runs: two for a whole block, one each from the two
            // workers that share one.
            for (int b = c.lane; b < nblk + (share_mode == 2 ? 1 : 0); b += 64) {
                const int block = b < nblk ? start + b : share_block;
                add_i32(pad_ptr(c, layer, 0, block / (D / 16)), !SHARE || b >= nblk || (share_mode == 1 && b == nblk - 1) ? 1 : 2);
            }
            trace_signalled(c);
        });
}

// Tag of the residual partial sums of one (decode step, layer, projection): differs from whatever a
// slot of the partial-sum buffer held before (the previous projection that used the group, or zero).
__device__ __forceinline__ uint32_t phase_tag(const Ctx &c, int layer, bool is_down) {
    const uint32_t step = (uint32_t)uni((int)c.sm->k.epoch);
    const uint32_t tag = (step * (uint32_t)uni(c.sm->args.num_layers) + (uint32_t)layer) * 2u + (is_down ? 1u : 0u) + 1u;
    return tag ? tag : 1u;
}

// ---------------------------------------------------------------------------------------------
// opcodes 4 and 6: matvec over one column group + residual add  (python_vm.py:59-124;
// reference device op: demos/low-latency-llama/matvec_adds.cu:10-192).
// With several column groups each (group, block) job leaves its bf16-rounded partial sum in the
// workspace as a tagged pair, and the job of the last group applies them to the residual in group
// order, which is the order the Python VM applies them in.
// ---------------------------------------------------------------------------------------------
template <int KC, bool is_down>
__device__ __forceinline__ bool control_matvec_add(const Ctx &c) {
    const InsPtr ins = c.sm->queue[c.slot];
    ArgsRef a = c.sm->args;
    const int layer = ins[1], start = ins[2], end = ins[3], group = ins[4];
    const int hid = a.hidden_size, R = a.matvec_reduction_size;
    const int in_dim = is_down ? a.intermediate_size : hid;
    const int ngroups = in_dim / R;
    const int nblk = end > start ? end - start : 0;
    // column groups executed jointly by this job (0: its own group only), as decoded
    const int joint_word = uni((int)((const MK_LDS uint32_t *)&c.sm->desc[c.slot])[2]);
    const int joint = joint_word & 0xff;                  // G in joint execution, else 0
    const int run = joint ? joint_word >> 8 : 1;          // jobs of each block that this one executes
    const uint16_t *vec = (is_down ? a.silu_out : a.attn_out) + (joint ? 0 : (size_t)group * R);
    const SyncInfo sy = sync_info(c);
    uint16_t *resid = a.hidden_states;
    // One lane per pair of adjacent residual rows.  Alone, a job owns all 16 rows of its blocks; in
    // joint execution it owns 16 / G rows of each, starting at row group * 16 / G.
    const int rows_per_block = joint ? run * 16 / joint : 16;
    const int pairs_per_block = rows_per_block / 2;
    const int npairs = nblk * pairs_per_block;
    auto row0_of = [&](int p) {
        const int bi = p / pairs_per_block, rp = p % pairs_per_block;
        return (start + bi) * 16 + (joint ? group * (16 / joint) : 0) + rp * 2;
    };
    // index in sm->out of the first partial sum of the pair's first row (joint: G sums per row, adjacent)
    auto out0_of = [&](int p) {
        const int bi = p / pairs_per_block, rp = p % pairs_per_block;
        return joint ? bi * 16 * run + rp * 2 * joint : p * 2;
    };
    // The residual rows this instruction updates were last written before its dependency was
    // satisfied, so the controller can fetch them while the consumers work.
    constexpr int kPre = 2;
    uint32_t pre[kPre] = {0, 0};
    const bool prefetched = npairs <= kPre * 64;
    PollTicket ticket = {nullptr, 0, 0};
    return controller_sequence(
        c,
        [&]() { ticket = poll_issue(c, sy); },
        [&](auto release) {
            if (!poll_wait(c, ticket, true, sy.target, release)) return false;
            trace_event(c, kEvDepReady, MK_TIMING_DONE_GMEM_WAIT);
            if (nblk > 0) {
                if (joint) {
                    // all column groups' slices of the vector, into the attention score buffer (idle here)
                    constexpr int kMaxJoint = 4;
                    uint4 xq[kMaxJoint][KC];
#pragma unroll
                    for (int g = 0; g < kMaxJoint; g++)
                        if (g < joint) load_xq<KC>(xq[g], vec + (size_t)g * R, c.lane);
                    release();
                    MK_LDS uint32_t *dst = (MK_LDS uint32_t *)&c.sm->scores[0][0];
#pragma unroll
                    for (int g = 0; g < kMaxJoint; g++)
                        if (g < joint) x_to_lds<KC>(xq[g], dst + g * (KC * 256), c.lane);
                } else {
                    uint4 xq[KC];
                    load_xq<KC>(xq, vec, c.lane);
                    release();
                    x_to_lds<KC>(xq, c.sm, c.lane);
                }
            }
            return true;
        },
        [&]() {
            if (prefetched) {
#pragma unroll
                for (int k = 0; k < kPre; k++) {
                    const int p = c.lane + k * 64;
                    if (p < npairs) pre[k] = ld_u32(resid + row0_of(p));
                }
            }
        },
        [&]() {
            bool guards_data = true;
            if (ngroups == 1 || joint) {
                // every partial sum of these rows is here: apply them in group order, each addition
                // rounded to bf16 as the Python VM's in-place adds are (python_vm.py:59-80)
                const int sums = joint ? joint : 1;
                for (int p = c.lane; p < npairs; p += 64) {
                    const int row0 = row0_of(p), o0 = out0_of(p);
                    const uint32_t h = prefetched ? (p < 64 ? pre[0] : pre[1]) : ld_u32(resid + row0);
                    float lo = mkm::bf16_lo(h), hi = mkm::bf16_hi(h);
                    for (int g = 0; g < sums; g++) {
                        lo = mkm::round_bf16(lo + c.sm->out[o0 + g]);
                        hi = mkm::round_bf16(hi + c.sm->out[o0 + sums + g]);
                    }
                    st_u32(resid + row0, mkm::pack_bf16(lo, hi));
                }
            } else {
                // Several column groups per block, each job on its own.  Every group's job but the last
                // leaves its bf16-rounded sum as a (value, tag) pair - one 8-byte store, so whoever sees
                // the tag sees the value, and nothing has to be acknowledged or counted.  The job of the
                // last group fetches the others' pairs until all carry this phase's tag and applies them
                // in group order, its own last: the Python VM's order.
                uint64_t *partial = ws_partial(c);
                const uint32_t tag = phase_tag(c, layer, is_down);
                if (group != ngroups - 1) {
                    for (int t = c.lane; t < nblk * 16; t += 64)
                        st_u64(partial + (size_t)group * hid + start * 16 + t, ((uint64_t)tag << 32) | mkm::f32_bits(c.sm->out[t]));
                    guards_data = false;
                } else {
                    const long long t0 = wall_clock64();
                    const long long limit = spin_ticks(c);
                    for (int p0 = 0; p0 < nblk * 8; p0 += 64) {  // wave-uniform trip count
                        const int p = p0 + c.lane;
                        const bool active = p < nblk * 8;
                        const int row0 = start * 16 + (active ? p : 0) * 2;
                        const uint32_t h = prefetched ? (p < 64 ? pre[0] : pre[1]) : (active ? ld_u32(resid + row0) : 0u);
                        float lo = mkm::bf16_lo(h), hi = mkm::bf16_hi(h);
                        const uint64_t *theirs = partial + row0;
                        // four groups' pairs per round trip
                        for (int g0 = 0; g0 < ngroups - 1; g0 += 4) {
                            uint4 v[4];
                            while (true) {
                                bool complete = true;
#pragma unroll
                                for (int k = 0; k < 4; k++)
                                    if (g0 + k < ngroups - 1) {
                                        v[k] = active ? ld_b128(theirs + (size_t)(g0 + k) * hid) : make_uint4(0, tag, 0, tag);
                                        complete &= v[k].y == tag && v[k].w == tag;
                                    }
                                if (__all(complete)) break;
                                if (wall_clock64() - t0 > limit || ld_i32(ws_status(c)) != 0) {
                                    if (c.lane == 0) record_status(c, MK_STATUS_BARRIER_TIMEOUT);
                                    break;
                                }
                                __builtin_amdgcn_s_sleep(2);
                            }
#pragma unroll
                            for (int k = 0; k < 4; k++)
                                if (g0 + k < ngroups - 1) {
                                    lo = mkm::round_bf16(lo + mkm::bits_f32(v[k].x));
                                    hi = mkm::round_bf16(hi + mkm::bits_f32(v[k].z));
                                }
                        }
                        if (active) {
                            lo = mkm::round_bf16(lo + c.sm->out[p * 2]);
                            hi = mkm::round_bf16(hi + c.sm->out[p * 2 + 1]);
                            st_u32(resid + row0, mkm::pack_bf16(lo, hi));
                        }
                    }
                }
            }
            // an arrival that stands for nothing another worker reads (a partial sum carries its own
            // tag) need not wait for its stores
            trace_store_issue(c);
            if (guards_data) wait_stores();
            trace_store_done(c);
            signal_sharded(c, sy, nblk * run);
            trace_signalled(c);
        });
}

// ---------------------------------------------------------------------------------------------
// opcode 5: RMSNorm + up and gate matvecs + SiLU  (python_vm.py:127-165;
// reference device op: demos/low-latency-llama/upgate.cu:10-172)
// ---------------------------------------------------------------------------------------------
template <int KC>
__device__ __forceinline__ bool control_upgate(const Ctx &c) {
    const InsPtr ins = c.sm->queue[c.slot];
    ArgsRef a = c.sm->args;
    const int layer = ins[1], n = ins[2];
    const int hid = a.hidden_size;
    const SyncInfo sy = sync_info(c);
    PollTicket ticket = {nullptr, 0, 0};
    uint4 wraw[KC];
    return controller_sequence(
        c,
        [&]() {
            ticket = poll_issue(c, sy);
            if (n > 0) load_row<KC>(wraw, a.mlp_norm_weights + (size_t)layer * hid, c.lane);
        },
        [&](auto release) {
            if (!poll_wait(c, ticket, true, sy.target, release)) return false;
            trace_event(c, kEvDepReady, MK_TIMING_DONE_GMEM_WAIT);
            if (n > 0) {
                uint4 x[KC];
                load_xq<KC>(x, a.hidden_states, c.lane);
                release();
                uint4 xq[KC];
                rms_norm_x<KC>(xq, x, wraw, a.rms_norm_eps);
                x_to_lds<KC>(xq, c.sm, c.lane);
            }
            return true;
        },
        [&]() {},
        [&]() {
            for (int p = c.lane; p < n * 8; p += 64) {
                const int i = p >> 3, r = (p & 7) * 2;
                const MK_LDS float *up = c.sm->out + i * 32, *gate = up + 16;
                // silu(gate) -> bf16, then times up -> bf16 (python_vm.py:161-163)
                const float s0 = mkm::round_bf16(mkm::silu_exact(gate[r]));
                const float s1 = mkm::round_bf16(mkm::silu_exact(gate[r + 1]));
                st_u32(a.silu_out + ins[3 + i] * 16 + r, mkm::pack_bf16(s0 * up[r], s1 * up[r + 1]));
            }
            trace_store_issue(c);
            wait_stores();
            trace_store_done(c);
            signal_sharded(c, sy, n);
            trace_signalled(c);
        });
}

// ---------------------------------------------------------------------------------------------
// Consumer side of the matvec instructions.  Wave w computes tasks w, w + 8, ... of an instruction.
// Weight rows travel through a pool of row buffers (registers); which buffers an instruction uses,
// in which order, is a compile-time list (BufMap), so all register indexing is static.  Requests are
// issued unconditionally (rows past the end become no-op requests): the count of outstanding loads
// at each wait is then a compile-time constant, also across the instructions that one handler
// executes in a row.
// ---------------------------------------------------------------------------------------------
template <int... IDX>
struct BufMap {
    static constexpr int size = sizeof...(IDX);
    static constexpr int at(int s) {
        constexpr int idx[] = {IDX...};
        return idx[s];
    }
};

// request rows first, first + 1, ... of this wave into the buffers of the list (`present` false:
// the instruction is not there, all requests are no-ops)
template <int KC, class Map, int NBUF>
__device__ __forceinline__ void request_rows(const Ctx &c, uint4 (&pool)[NBUF][KC], const MatvecDesc &d, int first, int mine,
                                             bool present = true) {
#pragma unroll
    for (int s = 0; s < Map::size; s++)
        load_row<KC>(pool[Map::at(s)], matvec_row(d, c.wave + (first + s) * kConsumerWaves), present && first + s < mine, c.lane);
}

// Rows parked in LDS: the data goes from HBM straight into this wave's slice of the attention score
// buffer (no registers involved), 16 bytes per lane and chunk, chunk j of a row at byte j * 1024.
template <int KC, int J = 0>
__device__ __forceinline__ void park_chunks(__amdgpu_buffer_rsrc_t rsrc, MK_LDS unsigned char *dst, uint32_t off) {
    if constexpr (J < KC) {
        // The instruction's own offset - which moves the place in memory and the place in LDS alike - has 12
        // bits: whole groups of four chunks go into the scalar offset and the LDS base instead.
        constexpr int kFar = (J / 4) * 4096;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (MK_LDS void *)(dst + kFar), 16, off, kFar, (J % 4) * 1024, MK_STREAM_AUX);
        park_chunks<KC, J + 1>(rsrc, dst, off);
    }
}
// request rows first, first + 1, ... first + N - 1 of this wave into its LDS slice
template <int KC, int N>
__device__ __forceinline__ void park_rows(const Ctx &c, MK_LDS unsigned char *slice, const MatvecDesc &d, int first, int mine,
                                          bool present) {
#pragma unroll
    for (int r = 0; r < N; r++) {
        const RowRef row = matvec_row(d, c.wave + (first + r) * kConsumerWaves);
        const uint32_t off = present && first + r < mine ? row.offset + c.lane * 16 : kNoRow;
        const __amdgpu_buffer_rsrc_t rsrc =
            __builtin_amdgcn_make_buffer_rsrc((void *)uni(row.buffer.base), 0, uni((int)row.buffer.bytes), 0x00020000);
        park_chunks<KC>(rsrc, slice + r * (KC * 1024), off);
    }
}

// One instruction, its first Map::size rows already requested into the listed buffers: wait for the
// activation vector, stream the rows (Map::size in flight), leave the results in LDS, and wait until
// the controller has sent them.  PARKED > 0: the wave's last PARKED rows were parked in `slice` by an
// earlier request and are taken from there; the rows before them stream as usual.
// where this wave's activation vector lies in LDS: the common buffer, or - for a jointly executed
// column-group job - the slice of the wave's column group in the attention score buffer
// (task t of such a job works on column group t mod G: the same for all tasks of a wave when the
// number of consumer waves is a multiple of G, else the wave fetches the slice per task)
constexpr bool kJointSlicePerTask = kConsumerWaves % 4 != 0;
template <int KC>
__device__ __forceinline__ const MK_LDS uint32_t *x_source(const Ctx &c, const MatvecDesc &d, int task) {
    if ((d.opcode == 4 || d.opcode == 6) && d.gate_delta > 0)
        return (const MK_LDS uint32_t *)&c.sm->scores[0][0] + (task & (((int)d.gate_delta & 0xff) - 1)) * (KC * 256);
    return (const MK_LDS uint32_t *)c.sm->x;
}

template <int KC, class Map, int NBUF, int PARKED = 0>
__device__ __forceinline__ bool consumer_run(const Ctx &c, uint4 (&pool)[NBUF][KC], const MatvecDesc &d, int mine,
                                             MK_LDS const unsigned char *slice = nullptr, int parked_rows = PARKED) {
    constexpr int PF = Map::size;
    if (!barrier_inputs_ready(c, true)) return false;
    XPairs<KC> x;
    const bool per_task = kJointSlicePerTask && (d.opcode == 4 || d.opcode == 6) && d.gate_delta > 0;
    if (d.ntasks > 0 && !per_task) x_from_lds<KC>(x, x_source<KC>(c, d, c.wave), c.lane);
    trace_consumer_first_use(c);
    auto consume = [&](const uint4 (&src)[KC], int i) {
        const int task = c.wave + i * kConsumerWaves;
        if (per_task) x_from_lds<KC>(x, x_source<KC>(c, d, task), c.lane);
        const float y = mkm::round_bf16(dot_row<KC>(src, x));
        if (c.lane == 0) c.sm->out[task] = y;
    };
    const int parked_first = mine > parked_rows ? mine - parked_rows : 0;  // rows from here on are in LDS
    const int streamed = PARKED > 0 ? parked_first : mine;
    int base = 0;
    // rounds that are followed by more rows: every row of the round exists, every buffer is refilled
    for (; base + PF < streamed; base += PF) {
#pragma unroll
        for (int s = 0; s < PF; s++) {
            consume(pool[Map::at(s)], base + s);
            compiler_fence();
            const int i = base + s + PF;
            load_row<KC>(pool[Map::at(s)], matvec_row(d, c.wave + i * kConsumerWaves), i < streamed, c.lane);
            compiler_fence();
        }
    }
    trace_last_load(c);
    // last round: nothing left to request
#pragma unroll
    for (int s = 0; s < PF; s++)
        if (base + s < streamed) consume(pool[Map::at(s)], base + s);
    if constexpr (PARKED > 0) {
        wait_stores();  // the parked rows were requested long ago; this makes their arrival in LDS certain
#pragma unroll
        for (int r = 0; r < PARKED; r++)
            if (parked_first + r < mine) {
                uint4 row[KC];
#pragma unroll
                for (int j = 0; j < KC; j++) {
                    const u32x4 v = *(const MK_LDS u32x4 *)(slice + r * (KC * 1024) + j * 1024 + c.lane * 16);
                    row[j] = uint4{v.x, v.y, v.z, v.w};
                }
                consume(row, parked_first + r);
            }
    }
    trace_consumer_last_use(c);
    wg_barrier();  // results are in LDS
    // hold further weight requests back until the controller has sent this instruction's results and
    // signal: they would otherwise queue behind the bulk loads
    wg_barrier();
    return true;
}

template <int KC, bool WIDE>
__device__ __forceinline__ bool control_matvec(const Ctx &c) {
    switch (c.opcode) {
    case 1: return control_qkv<KC, WIDE && MK_SHARE_QKV>(c);
    case 4: return control_matvec_add<KC, false>(c);
    case 5: return control_upgate<KC>(c);
    default: return control_matvec_add<KC, true>(c);
    }
}

__device__ __forceinline__ constexpr int pf_of(int opcode) {
    return opcode == 1 ? MK_PF_QKV : opcode == 4 ? MK_PF_OPROJ : opcode == 5 ? MK_PF_UPGATE : MK_PF_DOWN;
}
template <int N>
struct FirstBuffers;  // BufMap<0, 1, ..., N - 1>
template <> struct FirstBuffers<1> { typedef BufMap<0> type; };
template <> struct FirstBuffers<2> { typedef BufMap<0, 1> type; };
template <> struct FirstBuffers<3> { typedef BufMap<0, 1, 2> type; };
template <> struct FirstBuffers<4> { typedef BufMap<0, 1, 2, 3> type; };
template <> struct FirstBuffers<5> { typedef BufMap<0, 1, 2, 3, 4> type; };
template <> struct FirstBuffers<6> { typedef BufMap<0, 1, 2, 3, 4, 5> type; };

// The two sides of an instruction.  The controller wave runs its side inlined into the kernel's
// instruction loop: leaving a function with the signal's atomics still on their way would mean
// waiting for them (calls and returns wait for all outstanding memory operations), which is a round
// trip through memory between an instruction's signal and the first look at the next one's
// dependency - on the worker that signals last, the round trip the next phase waits for.  The
// consumer waves, which own the big register allocations, call one function per instruction kind.
enum { kConsumerRole = 0, kControllerRole = 1 };

// One matvec instruction (opcode OP, row width KC chunks).
// PARKED > 0: the wave's last PARKED rows come from LDS.  SELF false: an earlier instruction's handler
// requested them (into the region behind the attention score buffer); SELF true: the instruction
// requests them itself on entry, into the score buffer, after the rows that go to registers - more
// rows are then on their way, or there, when the dependency resolves, at no cost in registers.
// AHEAD > 0 (an O projection): the instruction also parks the last row per wave of the up/gate
// instruction that follows it in the queue, whose rows are AHEAD chunks wide - the O projection waits
// for attention with little to fetch, and memory is idle meanwhile.  (Requesting that instruction's
// first rows into registers as well, as the narrow model's pair handler does, was built and measured:
// 12 % slower - the O projection's own short requests then queue behind 192 KB of rows per CU.)
// Self-parked up/gate rows start kAheadOffset into the score buffer, behind the vector of a jointly
// executed O projection.
constexpr int kAheadOffset = 8192;
template <bool TR, int OP, int KC, int PARKED, int ROLE, int ROWS = 0, bool SELF = false, int AHEAD = 0, bool WIDE = false>
__device__ __forceinline__ bool matvec_impl(SmemPtr lds, int slot, int *refusal) {
    constexpr int kSelfOffset = SELF && OP == 5 ? kAheadOffset : 0;
    static_assert(!SELF || kSelfOffset + (size_t)kConsumerWaves * PARKED * KC * 1024 <= sizeof(Smem::scores) + sizeof(Smem::park),
                  "self-parked rows live in the score buffer and the region behind it (which a model with full-width rows only does not use otherwise)");
    constexpr int PF = ROWS ? ROWS : rows_in_flight<KC>(pf_of(OP));  // rows in flight per wave
    typedef typename FirstBuffers<PF>::type Map;
    const Ctx c = make_ctx<TR>(lds, slot, OP);
    MatvecDesc d;
    if (!describe_matvec(lds, slot, OP, d)) return bail(c, MK_STATUS_BAD_INSTRUCTION, refusal);
    if constexpr (ROLE == kControllerRole) return control_matvec<KC, WIDE>(c);
    const int mine = rows_of_wave(d.ntasks, c.wave);
    uint4 pool[PF][KC];
    wg_barrier();  // entry: the controller's first requests are out
    trace_first_load(c);
    // (a jointly executed job keeps its activation vector in the score buffer: no rows of its own there)
    const int parked = SELF && (OP == 4 || OP == 6) && d.gate_delta > 0 ? 0 : PARKED;
    request_rows<KC, Map>(c, pool, d, 0, mine > parked ? mine - parked : 0);
    MK_LDS unsigned char *slice =
        (MK_LDS unsigned char *)&lds->scores[0][0] + (SELF ? kSelfOffset : kParkDownOffset) + c.wave * (PARKED * KC * 1024);
    if constexpr (SELF && PARKED > 0) {
        // (an up/gate instruction's row may be there already: the O projection before it saw to that)
        const bool ahead = OP == 5 && uni(lds->parked_slot) == slot;
        if (parked > 0 && !ahead) park_rows<KC, PARKED>(c, slice, d, mine > parked ? mine - parked : 0, mine, true);
    }
    if constexpr (AHEAD > 0) {
        static_assert(OP == 4 && (size_t)KC * 2048 <= kAheadOffset && MK_WIDE_PARK_UPGATE == 1, "one up/gate row per wave, behind the O projection's vector");
        // the next instruction of the queue that is not a no-op
        int next = slot + 1;
        const int count = uni(lds->window_count);
        while (next < count && uni(lds->queue[next][0]) == 0) next++;
        MatvecDesc du;
        if (next < count && uni(lds->queue[next][0]) == 5 && describe_matvec(lds, next, 5, du)) {
            const int mine_u = rows_of_wave(du.ntasks, c.wave);
            MK_LDS unsigned char *slice_u = (MK_LDS unsigned char *)&lds->scores[0][0] + kAheadOffset + c.wave * (AHEAD * 1024);
            park_rows<AHEAD, 1>(c, slice_u, du, mine_u > 1 ? mine_u - 1 : 0, mine_u, true);
            if (c.tid == 0) lds->parked_slot = next;
        }
    }
    const bool ok = consumer_run<KC, Map, PF, PARKED>(c, pool, d, mine, slice, parked);
    if constexpr (SELF && OP == 5) {
        if (c.tid == 0) lds->parked_slot = -1;  // (the same slot comes round again in the next step of the launch)
    }
    return ok;
}
template <bool TR, int OP, int KC, int PARKED = 0, int ROWS = 0, bool SELF = false, int AHEAD = 0>
static __device__ __noinline__ bool op_matvec(SmemPtr lds, int slot, int *refusal) {
    return matvec_impl<TR, OP, KC, PARKED, kConsumerRole, ROWS, SELF, AHEAD>(lds, slot, refusal);
}

// O-proj followed directly by up/gate, as one handler.  O-proj is short (two rows per wave in the
// usual schedule) and waits long (for attention); the worker that runs it would otherwise request its
// up/gate rows only after O-proj's epilogue, when up/gate's dependency is about to resolve - half of
// the workers would fetch all of their up/gate rows on the critical path.  Here the first up/gate rows
// are requested together with the O-proj rows, and the two O-proj buffers go to up/gate as soon as
// O-proj is done.  Returns the number of instructions executed (2, or 1 when the second instruction
// is malformed and left to report itself), 0 on failure.
template <bool TR, int KC, bool PARK>
static __device__ __noinline__ int op_oproj_upgate(SmemPtr lds, int slot, int *refusal) {
    constexpr int NBUF = 6;
    // PARK: this worker has a long wait ahead (it came here without attention work) and its up/gate
    // instruction has at most two rows per wave beyond the six buffers: those go to LDS on entry - the
    // attention score buffer is free - and up/gate then needs nothing from HBM once its dependency resolves
    constexpr int kParked = PARK && (size_t)kConsumerWaves * kParkedUpgateRows * KC * 1024 <= sizeof(Smem::scores) ? kParkedUpgateRows : 0;
    typedef BufMap<0, 1> MapO;
    typedef BufMap<2, 3, 4, 5> MapU0;        // requested on entry
    typedef BufMap<0, 1> MapU1;              // requested when O-proj is done
    typedef BufMap<2, 3, 4, 5, 0, 1> MapU;
    const Ctx co = make_ctx<TR>(lds, slot, 4);
    const Ctx cu = make_ctx<TR>(lds, slot + 1, 5);
    MatvecDesc dso, dsu;
    if (!describe_matvec(lds, slot, 4, dso)) {
        bail(co, MK_STATUS_BAD_INSTRUCTION, refusal);
        return 0;
    }
    const bool pair = describe_matvec(lds, slot + 1, 5, dsu);
    // (consumer waves only: the controller wave takes the two instructions one after the other)
    if (!pair) dsu = dso;  // never fetched: the requests below become no-ops
    const int mine_o = rows_of_wave(dso.ntasks, co.wave);
    const int mine_u = pair ? rows_of_wave(dsu.ntasks, co.wave) : 0;
    const int stream_u = mine_u > kParked ? mine_u - kParked : 0;  // up/gate rows that go through the buffers
    uint4 pool[NBUF][KC];
    wg_barrier();  // entry of O-proj: the controller's first requests are out
    trace_first_load(co);
    request_rows<KC, MapO>(co, pool, dso, 0, mine_o);
    if (pair) trace_first_load(cu);
    request_rows<KC, MapU0>(co, pool, dsu, 0, stream_u, pair);
    MK_LDS unsigned char *slice = (MK_LDS unsigned char *)&lds->scores[0][0] + co.wave * (kParked * KC * 1024);
    if constexpr (PARK) {
        if constexpr (kParked > 0) park_rows<KC, kParked>(co, slice, dsu, mine_u > kParked ? mine_u - kParked : 0, mine_u, pair);
        // and the last rows per wave of a down projection that follows directly
        if constexpr (kParkedDownRows > 0 && KC * 1024 == 4096) {
            MatvecDesc dsd;
            const bool down_next = slot + 2 < uni(lds->window_count) && uni(lds->queue[slot + 2][0]) == 6 &&
                                   describe_matvec(lds, slot + 2, 6, dsd);
            if (!down_next) dsd = dso;
            const int mine_d = down_next ? rows_of_wave(dsd.ntasks, co.wave) : 0;
            park_rows<KC, kParkedDownRows>(
                co, (MK_LDS unsigned char *)&lds->scores[0][0] + kParkDownOffset + co.wave * (kParkedDownRows * KC * 1024), dsd,
                mine_d > kParkedDownRows ? mine_d - kParkedDownRows : 0, mine_d, down_next);
            if (co.lane == 0 && co.wave == 0) lds->parked_slot = down_next ? slot + 2 : -1;
        }
    }
    if (!consumer_run<KC, MapO>(co, pool, dso, mine_o)) return 0;
    request_rows<KC, MapU1>(co, pool, dsu, MapU0::size, stream_u, pair);
    if (!pair) return 1;
    wg_barrier();  // entry of up/gate: its first requests went out long ago
    return consumer_run<KC, MapU, NBUF, kParked>(cu, pool, dsu, mine_u, slice) ? 2 : 0;
}

// (value, index) pairs: the larger value wins, the smaller index on equal values - the first maximum,
// as torch.argmax reports it.  NaNs never win.  After the call every lane holds the wave's winner.
__device__ __forceinline__ void argmax_combine_wave(float &v, int &i) {
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const float ov = __shfl_xor(v, off);
        const int oi = __shfl_xor(i, off);
        if (ov > v || (ov == v && oi < i)) {
            v = ov;
            i = oi;
        }
    }
}

// ---------------------------------------------------------------------------------------------
// opcode 7: final RMSNorm + LM head  (python_vm.py:251-274;
// reference device op: demos/low-latency-llama/rms_lm_head.cu:10-117)
// ---------------------------------------------------------------------------------------------
template <bool TR, int KC>
static __device__ __noinline__ bool op_lm_head(SmemPtr lds, int slot, int *refusal) {
    const InsPtr ins = lds->queue[slot];
    const Ctx c = make_ctx<TR>(lds, slot, ins[0]);
    ArgsRef a = c.sm->args;
    const int start = ins[1], end = ins[2];
    const int hid = a.hidden_size;
    if (start < 0 || end > a.vocab_size / 16) return bail(c, MK_STATUS_BAD_INSTRUCTION, refusal);
    const SyncInfo sy = c.controller ? sync_info(c) : SyncInfo{nullptr, nullptr, nullptr, 0};
    const int blocks_per_batch = kOutRows / 16;
    const WeightBuffer W = weight_buffer(a.lm_head_weights, (size_t)a.vocab_size * hid * 2);
    float best_v = -INFINITY;
    int best_i = INT_MAX;
    PollTicket ticket = {nullptr, 0, 0};
    uint4 wraw[KC];
    bool first = true;
    int b0 = start;
    do {
        const int b1 = min(b0 + blocks_per_batch, end);
        const int nblk = b1 > b0 ? b1 - b0 : 0;
        const bool ok = matvec_batch<KC, rows_in_flight<KC>(MK_PF_LMHEAD)>(
            c, nblk * 16, true, [&](int t) { return RowRef{W, (uint32_t)(b0 * 16 + t) * (uint32_t)hid * 2u}; },
            [&]() {
                if (!first) return;
                ticket = poll_issue(c, sy);
                load_row<KC>(wraw, a.lm_head_norm_weights, c.lane);
            },
            [&](auto release) {
                if (!first) return true;  // the activation vector stays in LDS between batches
                if (!poll_wait(c, ticket, true, sy.target, release)) return false;
                trace_event(c, kEvDepReady, MK_TIMING_DONE_GMEM_WAIT);
                uint4 x[KC];
                load_xq<KC>(x, a.hidden_states, c.lane);
                release();
                uint4 xq[KC];
                rms_norm_x<KC>(xq, x, wraw, a.rms_norm_eps);
                x_to_lds<KC>(xq, c.sm, c.lane);
                return true;
            },
            [&]() {},
            [&]() {
                for (int p = c.lane; p < nblk * 8; p += 64) {
                    const float y0 = c.sm->out[p * 2], y1 = c.sm->out[p * 2 + 1];
                    st_u32(a.logits + b0 * 16 + p * 2, mkm::pack_bf16(y0, y1));
                    // running maximum of this lane; rows ascend, so "greater" keeps the first maximum
                    const int row = b0 * 16 + p * 2;
                    if (y0 > best_v) { best_v = y0; best_i = row; }
                    if (y1 > best_v) { best_v = y1; best_i = row + 1; }
                }
                trace_store_issue(c);
            });
        if (!ok) return false;
        first = false;
        b0 = b1;
    } while (b0 < end);
    if (c.controller && a.token_out) {
        // this worker's maximum logit (the values are bf16-exact) and its first index
        argmax_combine_wave(best_v, best_i);
        if (c.lane == 0 && best_i != INT_MAX) {
            int *slot_out = uni(c.sm->k.argmax) + 2 * (size_t)c.worker;
            st_i32(slot_out, __builtin_bit_cast(int, best_v));
            st_i32(slot_out + 1, best_i + 1);
        }
    }
    return true;
}

// One level of a recursive-halving tree sum.  `vals` holds N partial sums; the partner is lane
// (l ^ OFFSET).  The lane whose OFFSET bit is clear keeps the first N/2 entries and sends the second
// half, the other lane the opposite; afterwards vals[0 .. N/2) holds own + partner for the kept half.
template <int OFFSET, int N>
__device__ __forceinline__ void halving_level(float *vals, int lane) {
    const bool upper = (lane & OFFSET) != 0;
#pragma unroll
    for (int k = 0; k < N / 2; k++) {
        const float keep = upper ? vals[N / 2 + k] : vals[k];
        const float send = upper ? vals[k] : vals[N / 2 + k];
        const uint32_t own = __builtin_bit_cast(uint32_t, send);
        const LanePair pr = lane_xor_pair<OFFSET>(own);
        // the pair is {own, partner} in unspecified order; if both are equal either will do
        const uint32_t got = pr.a == own ? pr.b : pr.a;
        vals[k] = keep + __builtin_bit_cast(float, got);
    }
}

// ---------------------------------------------------------------------------------------------
// Log-sum-exp merge of n attention partitions of one head (python_vm.py:349-393), executed by the
// D/2 threads of the head (thread j: output dims 2j and 2j + 1, and the log-sum-exp of list entry
// j).  All 64 lanes of the wave must be active; with D = 64 the wave holds two heads.  `list_at(k)`
// is the partition index of list entry k.  Returns the merged pair and log-sum-exp; the caller stores.
// ---------------------------------------------------------------------------------------------
struct MergedPair {
    float o0, o1, lse;
};
template <int D, class ListAt>
__device__ __forceinline__ MergedPair merge_partitions(const Ctx &c, int head, int j, int n_any, ListAt list_at) {
    constexpr int kMaxList = MK_INSTRUCTION_WORDS - 7;
    constexpr int TPH = D / 2;
    ArgsRef a = c.sm->args;
    const int n = uni(n_any);  // the same for the whole wave: the loops below branch on scalars
    const int MP = uni(a.max_partials), d = j * 2;
    const float *outs = a.attn_out_intermediates + (size_t)head * MP * D + d;
    const float *lses = a.attn_lse_intermediates + (size_t)head * MP;
    // lane j of a head's lane group holds list entry j: its partition index and log-sum-exp
    const int entry = j < n ? list_at(j) : 0;
    const float lse = j < n ? ld_f32(lses + entry) : -INFINITY;
    // every request goes out at once: this thread's two dims of each listed partition
    uint64_t v[kMaxList];
#pragma unroll
    for (int k = 0; k < kMaxList; k++)
        if (k < n) v[k] = ld_u64(outs + (size_t)__builtin_amdgcn_readlane(entry, k) * D);
    // weights 2^(lse_i - max)
    const float m = lane_tree_max<1, TPH>(lse);
    const float wj = j < n ? mkm::exp2f_exact(lse - m) : 0.0f;
    float den = 0.0f, o0 = 0.0f, o1 = 0.0f;
    // accumulate in list order; entry k's weight comes from lane k of this head's group
#pragma unroll
    for (int k = 0; k < kMaxList; k++)
        if (k < n) {
            float w;
            if constexpr (TPH == 64) {
                w = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, wj), k));
            } else {
                const float w_lo = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, wj), k));
                const float w_hi = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, wj), k + 32));
                w = c.lane < 32 ? w_lo : w_hi;
            }
            den = den + w;
            o0 = fmaf(w, mkm::bits_f32((uint32_t)v[k]), o0);
            o1 = fmaf(w, mkm::bits_f32((uint32_t)(v[k] >> 32)), o1);
        }
    // every listed partition empty (a run past the end of the sequence in a reduction tree): the merge
    // of nothing is nothing, as for an empty partition itself
    if (m == -INFINITY) return MergedPair{0.0f, 0.0f, -INFINITY};
    return MergedPair{o0 / den, o1 / den, m + mkm::log2f_exact(den)};
}

// ---------------------------------------------------------------------------------------------
// opcode 2: attention of the 4 query heads of one KV head over one partition of the cache
// (python_vm.py:277-346; reference device op: demos/low-latency-llama/attention_partial.cu).
// Two passes over LDS-resident scores: (1) s = scale * q.k for every token, exact maximum;
// (2) p = exp(s - max), slot sums of p and p*v.  Token r of the partition belongs to slot
// r mod NSLOT, NSLOT = 8 waves * (64 / (D/8)) tokens per wave load; a slot accumulates its
// tokens in increasing order and slots are combined by a pairwise tree (token groups of a wave,
// then waves).  A token's row is spread over D/8 lanes, 8 dims each.
// ---------------------------------------------------------------------------------------------
template <bool TR, int D, int ROLE>
__device__ __forceinline__ bool attention_impl(SmemPtr lds, int slot, int *refusal) {
    const InsPtr ins = lds->queue[slot];
    const Ctx c = make_ctx<TR>(lds, slot, ins[0]);
    constexpr int LPT = D / 8;                   // lanes per token
    constexpr int TPW = 64 / LPT;                // tokens per wave per round
    constexpr int NSLOT = kAttnWaves * TPW;  // tokens per workgroup round
    constexpr int G = kGqa;
    ArgsRef a = c.sm->args;
    const SmemPtr sm = c.sm;
    const int layer = ins[1], kvh = ins[2], P = ins[3], pidx = ins[4];
    const int H = a.num_attention_heads, KVH = a.num_kv_heads;
    const bool skip = a.skip_attn_reduction != 0;
    if (layer < 0 || layer >= a.num_layers || kvh < 0 || kvh >= KVH || P < 1 || pidx < 0 || pidx >= P ||
        (!skip && pidx >= a.max_partials))
        return bail(c, MK_STATUS_BAD_INSTRUCTION, refusal);
    const int seq_len = a.pos_id + 1;
    const int total_blocks = (seq_len + 15) / 16;
    const int bpp = (total_blocks + P - 1) / P;
    const int sb = pidx * bpp;
    const int eb = min(sb + bpp, total_blocks);
    const int t0 = sb * 16;
    const int t1 = min(eb * 16, seq_len);
    const int T = t1 > t0 ? t1 - t0 : 0;
    // a partition longer than the score buffer works without it: its second pass recomputes the scores
    const bool scores_fit = T <= kScoreCap;
    const int h0 = kvh * G;
    const int rounds = (T + NSLOT - 1) / NSLOT;

    if constexpr (ROLE == kControllerRole) {
        // wait: Q heads, K head and V head of this step are complete (python_vm.py:281-290)
        const int col = c.lane < G ? h0 + c.lane : c.lane == G ? H + kvh : H + KVH + kvh;
        const bool mine = c.lane < G + 2;
        // (where QKV blocks can be shared, the counters count half blocks, `barriers` whole ones)
        const int unit = qkv_counter_unit(a);
        PollTicket ticket = poll_issue(c, mine ? pad_ptr(c, layer, 0, col) : nullptr, mine ? bar_ptr(c, layer, 0, col) : nullptr);
        ticket.base *= unit;
        // The QKV instructions leave what attention needs of this step - the query, and the step's K and
        // V row for the partition that holds the newest position - twice: in the tensors, followed by an
        // arrival on the heads' counters once the stores are acknowledged; and as stamped copies in the
        // workspace (8 bytes per bf16 pair: value, stamp of step and layer), which need neither.  The
        // controller looks at both.  Usually the copies complete first and ARE the data - one trip to memory
        // instead of acknowledgement, arrival, look at the counter and fetch - and go to the consumers through
        // LDS; the counters cover arrivals from before the launch, whose data exists in the tensors only.
        // (1 to 2 KB that 17 to 32 workers look at; the same for the 4 to 32 KB vectors between the matvec
        // instructions, which all 256 workers would pull, costs more than it saves.)
        constexpr int NQ = D / 64;  // 16-byte looks per lane that cover the four heads' query
        const bool has_new = uni((int)(a.pos_id >= t0 && a.pos_id < t0 + T)) != 0;
        const bool staging = MK_STAGE_QUERY && H * D == a.hidden_size && KVH * kGqa == H;
        const uint32_t stamp = layer_stamp(c, layer);
        const uint64_t *sq = ws_stamped_q(c) + (size_t)h0 * (D / 2) + c.lane * 2;
        // lanes [0, D/4): two pairs each of the K row; lanes [D/4, D/2): of the V row
        const bool kv_lane = has_new && c.lane < D / 2;
        const uint64_t *skv = (c.lane < D / 4 ? ws_stamped_k(c) : ws_stamped_v(c) - D / 2) + (size_t)kvh * (D / 2) + c.lane * 2;
        uint4 qraw[NQ], kvraw = make_uint4(0, 0, 0, 0);
        auto look = [&]() {
#pragma unroll
            for (int j = 0; j < NQ; j++) qraw[j] = ld_b128(sq + j * 128);
            if (kv_lane) kvraw = ld_b128(skv);
        };
        auto complete = [&]() {
            bool all = !kv_lane || (kvraw.y == stamp && kvraw.w == stamp);
#pragma unroll
            for (int j = 0; j < NQ; j++) all &= qraw[j].y == stamp && qraw[j].w == stamp;
            return __all(all) != 0;
        };
        bool ok = true, staged = false;
        if (staging) {
            look();
            const long long w0 = wall_clock64();
            const long long limit = spin_ticks(c);
            const int *status = ws_status(c);
            int v = ticket.value, st = ticket.status;
            while (true) {
                if (complete()) {
                    staged = true;
                    break;
                }
                if (__all(ticket.ptr == nullptr || v + ticket.base >= unit * (D / 16))) break;
                if (__any(st != 0)) {
                    ok = false;
                    break;
                }
                if (wall_clock64() - w0 > limit) {
                    if (c.lane == 0) record_status(c, MK_STATUS_BARRIER_TIMEOUT);
                    ok = false;
                    break;
                }
                __builtin_amdgcn_s_sleep(MK_POLL_SLEEP);
                v = ticket.ptr ? ld_i32(ticket.ptr) : 0;
                st = c.lane == 63 ? ld_i32(status) : 0;
                look();
            }
            compiler_fence();
        } else {
            ok = poll_wait(c, ticket, false, unit * (D / 16), []() {});
        }
        if (staged) {
#pragma unroll
            for (int j = 0; j < NQ; j++) *(MK_LDS u32x2 *)&sm->attn_q[j * 128 + c.lane * 2] = u32x2{qraw[j].x, qraw[j].z};
            if (kv_lane) {
                MK_LDS uint32_t *dst = c.lane < D / 4 ? &sm->attn_k[c.lane * 2] : &sm->attn_v[(c.lane - D / 4) * 2];
                *(MK_LDS u32x2 *)dst = u32x2{kvraw.x, kvraw.z};
            }
        }
        if (c.lane == 0) sm->attn_staged = staged ? 1 : 0;
        trace_event(c, kEvDepReady, MK_TIMING_DONE_GMEM_WAIT);
        if (!barrier_inputs_ready(c, ok)) return false;
        trace_event(c, kEvInputReady);
        wg_barrier();  // wave maxima
        trace_event(c, MK_TIMING_ATTN_MAXIMA);
        wg_barrier();  // probabilities
        trace_event(c, MK_TIMING_ATTN_PROBABILITIES);
        wg_barrier();  // wave sums
        trace_event(c, kEvComputeDone);
        // the waves that combine the sums store and signal on their own
        return true;
    }

    if (c.wave >= kAttnWaves) {
        // consumer waves beyond the eight that the token -> slot mapping uses: nothing to do but keep
        // the workgroup's barriers in step
        if (!barrier_inputs_ready(c, true)) return false;
        wg_barrier();
        wg_barrier();
        wg_barrier();
        return true;
    }
    const int sub = c.lane % LPT;         // which 8 dims of the head this lane owns
    const int tok_in_wave = c.lane / LPT;
    const size_t tok_stride = (size_t)KVH * D;
    const size_t base = ((size_t)layer * a.kv_max_len) * tok_stride + (size_t)kvh * D + sub * 8;
    const uint16_t *kbase = a.k_cache + base;
    const uint16_t *vbase = a.v_cache + base;
    // relative token handled by this lane in round rd
    auto token_of = [&](int rd) { return rd * NSLOT + c.wave * TPW + tok_in_wave; };
    // rows older than this step are immutable; the row at pos_id was written by another CU a moment
    // ago and needs a coherent load
    // (the controller may have found the query and the step's rows as stamped copies: they are in LDS then, and
    // the tensors' own copies of them are not known to have landed; `staged` is set once the dependency is known)
    bool staged = false;
    auto lds_row = [&](const MK_LDS uint32_t *row) {
        const u32x4 v = *(const MK_LDS u32x4 *)(row + sub * 4);
        return uint4{v.x, v.y, v.z, v.w};
    };
    auto newest_row = [&](const uint16_t *kvb) {
        return staged ? lds_row(kvb == vbase ? sm->attn_v : sm->attn_k) : ld_b128(kvb + (size_t)a.pos_id * tok_stride);
    };
    auto load_kv = [&](const uint16_t *kvb, int r) {
        const int t = t0 + r;
        return t == a.pos_id ? newest_row(kvb) : ld_const_b128(kvb + (size_t)t * tok_stride);
    };

    // Rounds are processed in batches of RU so that RU row loads are in flight per lane.  The first
    // batch of K and V does not depend on this step except for the newest token: request it before
    // the dependency is known.
    constexpr int RU = 4;
    uint4 kraw[RU], vraw[RU];
    trace_first_load(c);
#pragma unroll
    for (int u = 0; u < RU; u++) {
        const int r = token_of(u);
        kraw[u] = vraw[u] = make_uint4(0, 0, 0, 0);
        if (r < T && t0 + r != a.pos_id) {
            kraw[u] = ld_const_b128(kbase + (size_t)(t0 + r) * tok_stride);
            vraw[u] = ld_const_b128(vbase + (size_t)(t0 + r) * tok_stride);
        }
    }
    if (!barrier_inputs_ready(c, true)) return false;

    trace_consumer_first_use(c);
    uint4 q[G];  // this lane's 8 dims of the four query heads, as bf16 pairs
    staged = uni(sm->attn_staged) != 0;
    {
#pragma unroll
        for (int h = 0; h < G; h++)
            q[h] = staged ? lds_row(&sm->attn_q[h * (D / 2)]) : ld_b128(a.q_post_rope + (size_t)(h0 + h) * D + sub * 8);
        // the newest token's rows, if they fall into the first batch
#pragma unroll
        for (int u = 0; u < RU; u++) {
            const int r = token_of(u);
            if (r < T && t0 + r == a.pos_id) {
                kraw[u] = newest_row(kbase);
                vraw[u] = newest_row(vbase);
            }
        }
    }

    // scores of one token against the four heads, valid in all lanes of the token's group
    auto scores_of = [&](const uint4 &krow, float (&sc)[G]) {
#pragma unroll
        for (int h = 0; h < G; h++) {
            float acc = dot2_bf16(krow.x, q[h].x, 0.0f);
            acc = dot2_bf16(krow.y, q[h].y, acc);
            acc = dot2_bf16(krow.z, q[h].z, acc);
            acc = dot2_bf16(krow.w, q[h].w, acc);
            sc[h] = group_tree_sum<LPT>(acc) * a.attn_scale;
        }
    };

    // ---- pass 1: scores (kept as [token][head] in LDS when the partition fits) and maximum ----
    // (Deeper batches were measured and bring nothing; what a long partition needs is the next batch in
    // flight while the current one is worked on, see stream_rows.)
    constexpr int RUB = RU;
    float mx[G];
#pragma unroll
    for (int h = 0; h < G; h++) mx[h] = -INFINITY;
    auto score_round = [&](const uint4 &krow, int r) {
        float sc[G];
        scores_of(krow, sc);
#pragma unroll
        for (int h = 0; h < G; h++) mx[h] = fmaxf(mx[h], sc[h]);
        if (scores_fit && sub == 0) *(MK_LDS f32x4 *)&sm->scores[r][0] = f32x4{sc[0], sc[1], sc[2], sc[3]};
    };
    // Rows beyond the first batch stream through two sets of RUB row buffers: the requests of the batch
    // after next go out before a batch is worked on, so rows are in flight while the wave computes (a
    // long partition is half arithmetic, half waiting when the two alternate).
    // Every lane requests a row (a lane beyond the partition's end asks for the last one and ignores it), and
    // the kind of load is the same for the whole batch - coherent if the batch holds the row written in this
    // step - so the requests are straight-line code and each wait counts exactly the younger ones.
    auto load_batch = [&](const uint16_t *kvb, uint4 (&dst)[RUB], int rb) {
        const int first_token = t0 + rb * NSLOT;
        const bool has_new = uni((int)(a.pos_id >= first_token && a.pos_id < first_token + RUB * NSLOT)) != 0;
        if (has_new) {
#pragma unroll
            for (int u = 0; u < RUB; u++) {
                const int t = t0 + min(token_of(rb + u), T - 1);
                dst[u] = staged && t == a.pos_id ? newest_row(kvb) : ld_b128(kvb + (size_t)t * tok_stride);
            }
        } else {
#pragma unroll
            for (int u = 0; u < RUB; u++) dst[u] = ld_const_b128(kvb + (size_t)(t0 + min(token_of(rb + u), T - 1)) * tok_stride);
        }
    };
    auto stream_rows = [&](const uint16_t *kvb, auto first, auto use) {
        uint4 ba[RUB], bb[RUB];
        // the loop is controlled by scalars: the partition's extent is the same for the whole workgroup
        const int n_rounds = uni(rounds);
        // (a branch-free copy of this for batches that lie inside the partition as a whole is 0.6 % faster
        // on long partitions and 2 % slower on short ones, which never get here: the handler's code doubles)
        auto consume = [&](const uint4 (&src)[RUB], int rb) {
#pragma unroll
            for (int u = 0; u < RUB; u++) {
                const int r = token_of(rb + u);
                if (r < T) use(src[u], r);
            }
        };
        // Inside the loop a batch is requested whether or not it exists (one past the end asks for the
        // partition's last rows again and is dropped): with a request on every path the compiler's wait
        // for a batch leaves the younger one in flight.  The fences keep the requests where they are.
        if (RU >= n_rounds) {
            first();
            return;
        }
        load_batch(kvb, ba, RU);
        compiler_fence();
        first();
        for (int rb = RU;;) {
            load_batch(kvb, bb, rb + RUB);
            compiler_fence();
            consume(ba, rb);
            rb += RUB;
            if (rb >= n_rounds) break;
            compiler_fence();
            load_batch(kvb, ba, rb + RUB);
            compiler_fence();
            consume(bb, rb);
            rb += RUB;
            if (rb >= n_rounds) break;
            compiler_fence();
        }
    };
    stream_rows(
        kbase,
        [&]() {
#pragma unroll
            for (int u = 0; u < RU; u++) {
                const int r = token_of(u);
                if (r < T) score_round(kraw[u], r);  // the LPT lanes of a token share r, so they are active together
            }
        },
        score_round);
    {
        float m[G];
#pragma unroll
        for (int h = 0; h < G; h++) m[h] = lane_tree_max<LPT, 64>(mx[h]);
        if (c.lane == 0) *(MK_LDS f32x4 *)&sm->wave_max[c.wave][0] = f32x4{m[0], m[1], m[2], m[3]};
    }
    wg_barrier();
    float hm[G];
    {
        f32x4 m = *(const MK_LDS f32x4 *)&sm->wave_max[0][0];
#pragma unroll
        for (int w = 1; w < kAttnWaves; w++) {
            const f32x4 o = *(const MK_LDS f32x4 *)&sm->wave_max[w][0];
            m.x = fmaxf(m.x, o.x); m.y = fmaxf(m.y, o.y); m.z = fmaxf(m.z, o.z); m.w = fmaxf(m.w, o.w);
        }
        hm[0] = m.x; hm[1] = m.y; hm[2] = m.z; hm[3] = m.w;
    }
    // p = exp(s - max), once per (token, head), in place
    if (scores_fit) {
        MK_LDS float *flat = &sm->scores[0][0];
        for (int i = c.tid; i < G * T; i += kAttnThreads) {
            const int h = i & (G - 1);
            const float m = h == 0 ? hm[0] : h == 1 ? hm[1] : h == 2 ? hm[2] : hm[3];
            flat[i] = mkm::expf_exact(flat[i] - m);
        }
    }
    wg_barrier();

    // ---- pass 2: slot sums ----
    float acc[G][8], lsum[G];
#pragma unroll
    for (int h = 0; h < G; h++) {
        lsum[h] = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; e++) acc[h][e] = 0.0f;
    }
    auto value_round = [&](const uint4 &vrow, const float (&p)[G]) {
        float vf[8];
        unpack8(vrow, vf);
#pragma unroll
        for (int h = 0; h < G; h++) {
            lsum[h] = lsum[h] + p[h];
#pragma unroll
            for (int e = 0; e < 8; e++) acc[h][e] = fmaf(p[h], vf[e], acc[h][e]);
        }
    };
    if (scores_fit) {
        auto from_buffer = [&](const uint4 &vrow, int r) {
            const f32x4 pv = *(const MK_LDS f32x4 *)&sm->scores[r][0];
            const float p[G] = {pv.x, pv.y, pv.z, pv.w};
            value_round(vrow, p);
        };
        stream_rows(
            vbase,
            [&]() {
#pragma unroll
                for (int u = 0; u < RU; u++) {
                    const int r = token_of(u);
                    if (r < T) from_buffer(vraw[u], r);
                }
            },
            from_buffer);
    } else {
        // the scores were not kept: the same arithmetic on the same K rows gives them again, bit for bit
        constexpr int RUL = RU;
        auto recomputed = [&](const uint4 &krow, const uint4 &vrow) {
            float sc[G], p[G];
            scores_of(krow, sc);
#pragma unroll
            for (int h = 0; h < G; h++) p[h] = mkm::expf_exact(sc[h] - hm[h]);
            value_round(vrow, p);
        };
        // the first batch of K was consumed by pass 1 and is fetched again with the rest
        for (int rb = 0; rb < rounds; rb += RUL) {
            uint4 kb[RUL], vb[RUL];
#pragma unroll
            for (int u = 0; u < RUL; u++) {
                const int r = token_of(rb + u);
                if (r < T) {
                    kb[u] = load_kv(kbase, r);
                    vb[u] = load_kv(vbase, r);
                }
            }
#pragma unroll
            for (int u = 0; u < RUL; u++) {
                const int r = token_of(rb + u);
                if (r < T) recomputed(kb[u], vb[u]);
            }
        }
    }
    // Combine the TPW slots of the wave: a pairwise tree over the token groups (lane bits
    // log2(LPT) .. 5).  Recursive halving: at each level a lane hands half of its partial sums to
    // its partner and keeps the other half, so the 32 sums per lane shrink to 32 / TPW and the
    // number of lane exchanges drops from 32 per level to 16 + 8 + 4.  own + partner is the same
    // addition the butterfly would do.
    {
        float part[G * 8];
#pragma unroll
        for (int h = 0; h < G; h++)
#pragma unroll
            for (int e = 0; e < 8; e++) part[h * 8 + e] = acc[h][e];
        halving_level<LPT, G * 8>(part, c.lane);
        halving_level<LPT * 2, G * 4>(part, c.lane);
        if constexpr (TPW == 8) halving_level<LPT * 4, G * 2>(part, c.lane);
        // the lane now holds the sums with index  tg_bit0 * 16 + tg_bit1 * 8 (+ tg_bit2 * 4) + k
        constexpr int kLeft = G * 8 / TPW;
        const int first = ((tok_in_wave & 1) * 16) + (((tok_in_wave >> 1) & 1) * 8) + (TPW == 8 ? ((tok_in_wave >> 2) & 1) * 4 : 0);
        MK_LDS float *dst = &sm->wave_o[c.wave][0][0];
#pragma unroll
        for (int k = 0; k < kLeft; k++) {
            const int idx = first + k;  // = h * 8 + e
            dst[(idx >> 3) * kMaxHeadDim + sub * 8 + (idx & 7)] = part[k];
        }
        float l[G];
#pragma unroll
        for (int h = 0; h < G; h++) l[h] = lane_tree_sum<LPT, 64>(lsum[h]);
        if (c.lane == 0) *(MK_LDS f32x4 *)&sm->wave_l[c.wave][0] = f32x4{l[0], l[1], l[2], l[3]};
    }
    trace_consumer_last_use(c);
    wg_barrier();

    // ---- combine the 8 waves pairwise, normalise, store: thread -> (head, dim pair).  The threads of
    // one head sit in one wave, which signals for that head once its own stores have landed. ----
    if (c.tid < G * D / 2) {
        const int h = c.tid / (D / 2), d = (c.tid % (D / 2)) * 2;
        float o0[kAttnWaves], o1[kAttnWaves], l[kAttnWaves];
#pragma unroll
        for (int w = 0; w < kAttnWaves; w++) {
            o0[w] = sm->wave_o[w][h][d];
            o1[w] = sm->wave_o[w][h][d + 1];
            l[w] = sm->wave_l[w][h];
        }
#pragma unroll
        for (int st = 1; st < kAttnWaves; st <<= 1)
#pragma unroll
            for (int i = 0; i < kAttnWaves; i += 2 * st) {
                o0[i] = o0[i] + o0[i + st];
                o1[i] = o1[i] + o1[i + st];
                l[i] = l[i] + l[i + st];
            }
        const int head = h0 + h;
        float r0, r1, lse;
        if (T == 0) {  // softmax over nothing
            r0 = r1 = 0.0f;
            lse = -INFINITY;
        } else {
            r0 = o0[0] / l[0];
            r1 = o1[0] / l[0];
            const float m = h == 0 ? hm[0] : h == 1 ? hm[1] : h == 2 ? hm[2] : hm[3];
            lse = (m * 1.44269504088896341f) + mkm::log2f_exact(l[0]);
        }
        if (skip) {
            st_u32(a.attn_out + (size_t)head * D + d, mkm::pack_bf16(r0, r1));
        } else {
            float *dst = a.attn_out_intermediates + ((size_t)head * a.max_partials + pidx) * D + d;
            st_f32(dst, r0);
            st_f32(dst + 1, r1);
            if (d == 0) st_f32(a.attn_lse_intermediates + (size_t)head * a.max_partials + pidx, lse);
        }
        // (the stamps of the storing waves share their slots: the last wave to get there is on record)
        trace_store_issue(c);
        wait_stores();
        trace_store_done(c);
        if (d == 0) {
            if (skip) signal_sharded_lane(c, layer, 2, 1);
            else add_i32(pad_ptr(c, layer, 1, head), 1);
        }
        trace_signalled(c);
    }
    return true;
}
template <bool TR, int D>
static __device__ __noinline__ bool op_attention(SmemPtr lds, int slot, int *refusal) {
    return attention_impl<TR, D, kConsumerRole>(lds, slot, refusal);
}

// ---------------------------------------------------------------------------------------------
// opcode 3: log-sum-exp merge of attention partitions  (python_vm.py:349-393;
// reference device op: demos/low-latency-llama/attention_reduction.cu:18-339)
// ---------------------------------------------------------------------------------------------
template <bool TR, int D, int ROLE>
__device__ __forceinline__ bool reduction_impl(SmemPtr lds, int slot, int *refusal) {
    const InsPtr ins = lds->queue[slot];
    const Ctx c = make_ctx<TR>(lds, slot, ins[0]);
    ArgsRef a = c.sm->args;
    constexpr int kMaxList = MK_INSTRUCTION_WORDS - 7;
    constexpr int TPH = D / 2;  // threads per head, two output dims each; all in one wave
    static_assert(TPH >= kMaxList && TPH <= 64, "a head's threads also fetch one list entry's log-sum-exp each");
    const int layer = uni(ins[1]), hs = uni(ins[2]), P = uni(ins[3]), terminal = uni(ins[4]), n = uni(ins[5]);
    const int R = uni(a.attn_reduction_size), MP = uni(a.max_partials);
    bool bad = layer < 0 || layer >= a.num_layers || n < 1 || n > kMaxList || hs < 0 ||
               hs + R > a.num_attention_heads || R > kGqa || a.head_dim != D;
    // the listed partitions, one per lane
    if (!bad) bad = __any(c.lane < n && (ins[6 + c.lane] < 0 || ins[6 + c.lane] >= MP)) != 0;
    const int out_idx = bad ? 0 : uni(ins[6 + n]);
    bad |= !terminal && (out_idx < 0 || out_idx >= MP);
    if (bad) return bail(c, MK_STATUS_BAD_INSTRUCTION, refusal);

    // The waves that hold the heads' threads wait for their own heads' partitions, merge, store and
    // signal; nobody else has anything to do.  (No weights are streamed here, so a wave's looks at
    // the counters do not queue behind bulk loads of its own.)  Everybody leaves together, after the
    // signal: the next instruction starts with bulk weight requests, and a CU serves its requests in
    // order.
    if (ROLE == kConsumerRole && c.tid < R * TPH) {
        const int h = c.tid / TPH, j = c.tid % TPH, d = j * 2;
        const int head = hs + h;
        const bool leader = j == 0;
        const PollTicket ticket =
            poll_issue(c, leader ? pad_ptr(c, layer, 1, head) : nullptr, leader ? bar_ptr(c, layer, 1, head) : nullptr);
        if (poll_wait(c, ticket, false, P, []() {})) {
            if (c.wave == 0) {
                trace_wave(c, kEvDepReady);
                trace_wave(c, MK_TIMING_DONE_GMEM_WAIT);
            }
            trace_consumer_first_use(c);
            const MergedPair r = merge_partitions<D>(c, head, j, n, [&](int k) { return ins[6 + k]; });
            if (terminal) {
                st_u32(a.attn_out + (size_t)head * D + d, mkm::pack_bf16(r.o0, r.o1));
            } else {
                float *dst = a.attn_out_intermediates + ((size_t)head * MP + out_idx) * D + d;
                st_f32(dst, r.o0);
                st_f32(dst + 1, r.o1);
                if (leader) st_f32(a.attn_lse_intermediates + (size_t)head * MP + out_idx, r.lse);
            }
            trace_consumer_last_use(c);
            trace_store_issue(c);
            wait_stores();
            trace_store_done(c);
            // A terminal merge completes the head for the O projection (barrier row 2).  A merge
            // inside a reduction tree is one more arrival among the head's partial results (row 1):
            // the merge that consumes it waits for the partitions plus the merges below it.
            if (leader) {
                if (terminal) signal_sharded_lane(c, layer, 2, 1);
                else add_i32(pad_ptr(c, layer, 1, head), 1);
            }
            trace_signalled(c);
        } else if (c.lane == 0) {
            c.sm->abort = 1;
        }
    }
    if (c.controller) trace_event(c, MK_TIMING_AT_GMEM_WAIT);
    wg_barrier();
    // (the first merging wave stamped the moment it saw its heads' partitions complete)
    trace_event(c, kEvInputReady);
    trace_event(c, kEvComputeDone);
    return c.sm->abort == 0;
}
template <bool TR, int D>
static __device__ __noinline__ bool op_attention_reduction(SmemPtr lds, int slot, int *refusal) {
    return reduction_impl<TR, D, kConsumerRole>(lds, slot, refusal);
}

// The controller wave's side of the instruction in `slot`.
template <bool TR, int KC_HID, int KC_RED, int D>
__device__ __forceinline__ bool controller_step(SmemPtr sm, int slot, int opcode, int *refusal) {
    switch (opcode) {
    case 1: return matvec_impl<TR, 1, KC_HID, 0, kControllerRole, 0, false, 0, KC_HID != KC_RED>(sm, slot, refusal);
    case 2: return attention_impl<TR, D, kControllerRole>(sm, slot, refusal);
    case 3: return reduction_impl<TR, D, kControllerRole>(sm, slot, refusal);
    case 4: return matvec_impl<TR, 4, KC_RED, 0, kControllerRole>(sm, slot, refusal);
    case 5: return matvec_impl<TR, 5, KC_HID, 0, kControllerRole>(sm, slot, refusal);
    case 6: return matvec_impl<TR, 6, KC_RED, 0, kControllerRole>(sm, slot, refusal);
    case 7: return op_lm_head<TR, KC_HID>(sm, slot, refusal);
    default: return bail(make_ctx<TR>(sm, slot, opcode), MK_STATUS_BAD_OPCODE, refusal);  // reference: trap, include/util.cuh:38
    }
}

// The same with a function of its own per instruction kind: where the activation vector is 4096 wide,
// the controller's side of an instruction needs most of the registers, and inlined in the instruction
// loop (or all kinds in one function) it pushes values into scratch memory.
template <bool TR, int OP, int KC, bool WIDE>
static __device__ __noinline__ bool controller_matvec_call(SmemPtr sm, int slot, int *refusal) {
    return matvec_impl<TR, OP, KC, 0, kControllerRole, 0, false, 0, WIDE>(sm, slot, refusal);
}
template <bool TR, int D>
static __device__ __noinline__ bool controller_attention_call(SmemPtr sm, int slot, int *refusal) {
    return attention_impl<TR, D, kControllerRole>(sm, slot, refusal);
}
template <bool TR, int KC_HID, int KC_RED, int D>
__device__ __forceinline__ bool controller_step_call(SmemPtr sm, int slot, int opcode, int *refusal) {
    switch (opcode) {
    case 1: return controller_matvec_call<TR, 1, KC_HID, true>(sm, slot, refusal);
    case 2: return controller_attention_call<TR, D>(sm, slot, refusal);
    case 3: return reduction_impl<TR, D, kControllerRole>(sm, slot, refusal);
    case 4: return controller_matvec_call<TR, 4, KC_RED, true>(sm, slot, refusal);
    case 5: return controller_matvec_call<TR, 5, KC_HID, true>(sm, slot, refusal);
    case 6: return controller_matvec_call<TR, 6, KC_RED, true>(sm, slot, refusal);
    case 7: return op_lm_head<TR, KC_HID>(sm, slot, refusal);
    default: return bail(make_ctx<TR>(sm, slot, opcode), MK_STATUS_BAD_OPCODE, refusal);
    }
}

// ---------------------------------------------------------------------------------------------
// the persistent kernel
// ---------------------------------------------------------------------------------------------
// Everything the instruction loop needs between two instructions lives in LDS (the launch arguments,
// the queue window, the abort flag): the loop itself keeps a handful of values in registers, nothing
// in scratch memory, so that a handler's return is not followed by a reload from memory - which
// would be a round trip through the vector memory path on the way to every next instruction.

// Instruction fetch (reference: controller warp, include/controller/instruction_fetch.cuh:10-27):
// a window of the worker's queue is copied into LDS and its matvec instructions are decoded, so that
// taking an instruction never waits on HBM.  The usual queue fits the window and is fetched once per
// launch; a longer one goes through window by window, every step.
// Which QKV instructions this worker and its partner (the neighbouring worker: w ^ 1) hold, per layer.
// The reference's schedule deals the 16-row blocks of the QKV projection out evenly up to one block (8B:
// 384 blocks, two for every other worker, one for the rest), and the phase ends with the workers that
// have one more, which fetch their last rows after the dependency has resolved.  Where the two partners'
// instructions of a layer differ by one block, the one with fewer takes rows 8-15 of the other's last
// block: both decide so on their own, from the same two queues.
static __device__ __noinline__ void share_setup(SmemPtr sm) {
    ArgsRef a = sm->args;
    const int tid = (int)threadIdx.x;
    MK_LDS int *tables = &sm->qkv_count[0][0];
    static_assert(offsetof(Smem, qkv_info) == offsetof(Smem, qkv_count) + sizeof(Smem::qkv_count), "cleared as one array");
    for (int i = tid; i < 4 * kShareLayers; i += kThreads) tables[i] = 0;
    wg_barrier();
    const int workers = (int)gridDim.x;
    if (shares_qkv_blocks(a) && workers % 2 == 0 && a.num_layers <= kShareLayers) {
        const int partner = (int)blockIdx.x ^ 1;
        for (int s = tid; s < 2 * a.num_slots; s += kThreads) {
            const int who = s < a.num_slots ? 0 : 1, slot = who ? s - a.num_slots : s;
            const MK_GLOBAL int *ins =
                as_global(a.instructions) + ((size_t)(who ? partner : (int)blockIdx.x) * a.num_slots + slot) * MK_INSTRUCTION_WORDS;
            if (ins[0] != 1) continue;
            const int layer = ins[1], start = ins[2], end = ins[3];
            if (layer < 0 || layer >= a.num_layers) continue;
            const int nblk = end > start ? end - start : 0;
            const bool fine = start >= 0 && end < (1 << 20) && nblk <= kOutRows / 16;
            // (a malformed instruction counts twice: no sharing with it)
            __hip_atomic_fetch_add(&sm->qkv_count[who][layer], fine ? 1 : 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            if (fine) sm->qkv_info[who][layer] = (nblk << 20) | (nblk > 0 ? end - 1 : 0);  // (meaningful when it is the only one)
        }
    }
    wg_barrier();
}

static __device__ __noinline__ void fetch_window(SmemPtr sm, int base) {
    ArgsRef a = sm->args;
    const int tid = (int)threadIdx.x;
    const int count = min(kQueueSlots, a.num_slots - base);
    const MK_GLOBAL int *queue = as_global(a.instructions) + ((size_t)blockIdx.x * a.num_slots + base) * MK_INSTRUCTION_WORDS;
    MK_LDS int *dst = &sm->queue[0][0];
    for (int i = tid; i < count * MK_INSTRUCTION_WORDS; i += kThreads) dst[i] = queue[i];
    if (tid == 0) {
        sm->window_base = base;
        sm->window_count = count;
        sm->parked_slot = -1;
    }
    wg_barrier();
    for (int slot = tid; slot < count; slot += kThreads) {
        const int opcode = sm->queue[slot][0];
        if (opcode == 1 || (opcode >= 4 && opcode <= 6)) decode_matvec(sm, slot, a);
        if (opcode == 1 || (opcode >= 4 && opcode <= 7)) decode_sync(sm, slot, a);
    }
    wg_barrier();
    // the jobs that an earlier job of their block executes become no-ops
    for (int slot = tid; slot < count; slot += kThreads) {
        const int opcode = sm->queue[slot][0];
        if ((opcode == 4 || opcode == 6) && sm->desc[slot].ntasks == kAbsorbed) sm->queue[slot][0] = 0;
    }
    wg_barrier();
}

// End of a step.  The last workgroup to get here folds the sharded counters into `barriers` (or
// zeroes `barriers`), leaves the shards zeroed, and turns the workers' LM-head maxima into the step's
// token.  With more steps to go it then publishes the step, and everybody else waits for that before
// starting on the next token.  Returns whether another step follows.
template <bool TR>
static __device__ __noinline__ bool end_of_step(SmemPtr sm, int step, int steps) {
    ArgsRef a = sm->args;
    const int tid = (int)threadIdx.x;
    const WsLayout wl = ws_layout(a.num_layers, a.hidden_size, a.intermediate_size, a.matvec_reduction_size);
    int *status = static_cast<int *>(a.workspace) + wl.status;
    wait_stores();
    wg_barrier();
    if (tid == 0) {
        const int done = __hip_atomic_fetch_add(as_global(&status[kDoneSlot]), 1, __ATOMIC_RELAXED, AG);
        sm->last_flag = done == (int)gridDim.x * (step + 1) - 1;
    }
    wg_barrier();
    const bool more = step + 1 < steps && sm->abort == 0;
    if (sm->last_flag) {
        // One thread per (counter, shard), two pairs per trip with both loads in flight, and the
        // workers' maxima requested before the fold: the step's token waits for one round trip
        // here, not for a chain of them.
        const int counters = a.num_layers * kHotRows;
        int *shards = static_cast<int *>(a.workspace) + wl.shards;
        const int cols = a.num_attention_heads + 2 * a.num_kv_heads;
        const bool reset = (a.flags & MK_FLAG_RESET_BARRIERS) != 0;
        int *maxima = static_cast<int *>(a.workspace) + wl.argmax;
        int *barriers = a.barriers;
        constexpr int kMaxTrips = (kMaxWorkers + kThreads - 1) / kThreads;
        uint64_t reported[kMaxTrips];
#pragma unroll
        for (int k = 0; k < kMaxTrips; k++) {
            const int w = tid + k * kThreads;
            reported[k] = a.token_out && w < (int)gridDim.x ? ld_u64(maxima + 2 * w) : 0;
        }
        // k = (replica, shard, counter); every copy is zeroed, the first one is what gets counted
        auto shard_at = [&](int k) { return shards + k; };
        auto fold = [&](int k, int v) {
            if (v == 0) return;
            st_i32(shard_at(k), 0);
            const int i = k % counters;
            if (!reset && k < counters * kShards) add_i32(barriers + ((size_t)(i / kHotRows) * MK_BARRIER_ROWS + 2 + i % kHotRows) * cols, v);
        };
        const int pairs = counters * kShards * kReplicas;
        for (int k = tid; k < pairs; k += 2 * kThreads) {
            const int k2 = k + kThreads;
            const int v = ld_i32(shard_at(k));
            const int v2 = k2 < pairs ? ld_i32(shard_at(k2)) : 0;
            fold(k, v);
            if (k2 < pairs) fold(k2, v2);
        }
        {
            // the padded per-head counters, four looks in flight per thread and trip
            int *pads = static_cast<int *>(a.workspace) + wl.pads;
            const int pc = pad_cols(a.hidden_size), npad = a.num_layers * 2 * pc;
            for (int k0 = tid; k0 < npad; k0 += 4 * kThreads) {
                int v[4];
#pragma unroll
                for (int u = 0; u < 4; u++) {
                    const int k = k0 + u * kThreads;
                    v[u] = k < npad ? ld_i32(pads + (size_t)k * kPadInts) : 0;
                }
#pragma unroll
                for (int u = 0; u < 4; u++) {
                    const int k = k0 + u * kThreads;
                    if (v[u] == 0) continue;
                    st_i32(pads + (size_t)k * kPadInts, 0);
                    const int col = k % pc, lr = k / pc;
                    // (row 0, the QKV blocks of a head, is counted in half blocks)
                    if (!reset && col < cols)
                        add_i32(barriers + ((size_t)(lr / 2) * MK_BARRIER_ROWS + lr % 2) * cols + col, lr % 2 == 0 ? v[u] / qkv_counter_unit(a) : v[u]);
                }
            }
        }
        if (reset) {
            const int words = a.num_layers * MK_BARRIER_ROWS * cols;
            for (int i = tid; i < words; i += kThreads) st_i32(barriers + i, 0);
        }
        if (a.token_out) {
            // the workers' LM-head maxima -> the step's token
            float v = -INFINITY;
            int idx = INT_MAX;
#pragma unroll
            for (int k = 0; k < kMaxTrips; k++) {
                const int stored = (int)(reported[k] >> 32);
                if (stored) {
                    const float wv = __builtin_bit_cast(float, (int)(uint32_t)reported[k]);
                    if (wv > v || (wv == v && stored - 1 < idx)) {
                        v = wv;
                        idx = stored - 1;
                    }
                    st_i32(maxima + 2 * (tid + k * kThreads) + 1, 0);
                }
            }
            argmax_combine_wave(v, idx);
            if (tid % 64 == 0) {
                sm->out[2 * (tid / 64)] = v;
                sm->flags[tid / 64] = idx;
            }
            wg_barrier();
            if (tid == 0) {
                for (int w = 1; w < kThreads / 64; w++) {
                    const float wv = sm->out[2 * w];
                    const int wi = sm->flags[w];
                    if (wv > v || (wv == v && wi < idx)) {
                        v = wv;
                        idx = wi;
                    }
                }
                const int token = idx == INT_MAX ? 0 : idx;
                st_u64(a.token_out + step, (uint64_t)token);
                sm->token = token;
            }
        }
        if (tid == 0) st_i32(&status[kEpochSlot], (int)(sm->k.epoch + 1u));
        if (more) {
            // everything the next step relies on (zeroed counters, the token) has landed before
            // the step is published
            wait_stores();
            wg_barrier();
            if (tid == 0) st_i32(&status[kStepSlot], step + 1);
        } else if (tid == 0) {
            st_i32(&status[kDoneSlot], 0);
            st_i32(&status[kStepSlot], 0);
        }
    } else if (more && tid < 64) {
        // one wave watches for the step's publication (and for a failure anywhere)
        const long long t0 = wall_clock64();
        const long long limit = (long long)(a.spin_limit_us ? a.spin_limit_us : 2000000u) * 100;
        bool ok = true;
        while (true) {
            const int published = ld_i32(&status[kStepSlot]);
            const int failure = ld_i32(&status[0]);
            if (failure != 0) {
                ok = false;
                break;
            }
            if (published > step) break;
            if (wall_clock64() - t0 > limit) {
                if (tid == 0) record_status(make_ctx<TR>(sm, 0, 0), MK_STATUS_BARRIER_TIMEOUT);
                ok = false;
                break;
            }
            __builtin_amdgcn_s_sleep(MK_POLL_SLEEP);
        }
        compiler_fence();
        const uint64_t token = ok ? ld_u64(a.token_out + step) : 0;
        if (tid == 0) {
            if (ok) sm->token = (int)token;
            else sm->abort = 1;
        }
    }
    if (!more) return false;
    if (tid == 0) {
        sm->args.pos_id = a.pos_id + 1;
        sm->k.epoch += 1u;
        sm->parked_slot = -1;
    }
    wg_barrier();
    return sm->abort == 0;
}

template <int KC_HID, int KC_RED, int D, bool TR>
__global__ __launch_bounds__(kThreads) void mk_llama_kernel(const mk_llama_args a) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    const SmemPtr sm = (SmemPtr)smem_raw;
    const int tid = (int)threadIdx.x;
    if (tid == 0) {
        sm->abort = 0;
        sm->last_flag = 0;
        sm->parked_slot = -1;
        // the token whose embedding row starts the step (written by the previous launch or the host)
        int token = -1;
        if (a.token_in) {
            const long long t = *as_global(a.token_in);
            if (t >= 0 && t < a.vocab_size) token = (int)t;
        }
        sm->token = token;
    }
    {
        // the launch arguments: kernarg segment -> LDS, one word per thread
        const __attribute__((address_space(4))) int *src =
            (const __attribute__((address_space(4))) int *)__builtin_amdgcn_kernarg_segment_ptr();
        MK_LDS int *dst = (MK_LDS int *)&sm->args;
        static_assert(sizeof(mk_llama_args) % 4 == 0 && sizeof(mk_llama_args) / 4 <= kThreads, "argument block");
        if (tid < (int)(sizeof(mk_llama_args) / 4)) dst[tid] = src[tid];
    }
    if (tid == 0) {
        int *const ws = static_cast<int *>(a.workspace);
        const WsLayout w = ws_layout(a.num_layers, a.hidden_size, a.intermediate_size, a.matvec_reduction_size);
        sm->k.status = ws + w.status;
        sm->k.shards = ws + w.shards;
        sm->k.argmax = ws + w.argmax;
        sm->k.pads = ws + w.pads;
        sm->k.partial = reinterpret_cast<uint64_t *>(ws + w.partial);
        sm->k.stamped = reinterpret_cast<uint64_t *>(ws + w.stamped);
        sm->k.epoch = (uint32_t)ld_i32(ws + w.status + kEpochSlot);
        sm->k.trace_base =
            (a.flags & MK_FLAG_TIMINGS) && a.timings ? a.timings + (size_t)blockIdx.x * a.num_slots * MK_TIMING_SLOTS : nullptr;
        sm->k.spin_ticks = (long long)(a.spin_limit_us ? a.spin_limit_us : 2000000u) * 100;  // 100 MHz wall clock
        sm->k.cols = a.num_attention_heads + 2 * a.num_kv_heads;
        sm->k.pad_cols = pad_cols(a.hidden_size);
        sm->k.down_jobs = (a.intermediate_size / a.matvec_reduction_size) * (a.hidden_size / 16);
        sm->k.o_jobs = (a.hidden_size / a.matvec_reduction_size) * (a.hidden_size / 16);
        sm->k.shard_stride = a.num_layers * kHotRows;
        sm->k.replica_stride = kShards * a.num_layers * kHotRows;
        sm->k.hold_looks = a.hidden_size != a.matvec_reduction_size ? 0 : MK_HOLD_LOOKS;
    }
    // A launch covers one decode step, or `num_steps` of them back to back: the token a step
    // produces starts the next one, at the next position.
    const int steps = a.num_steps > 1 ? a.num_steps : 1;
    wg_barrier();  // the argument block and the token are in LDS
    // a launch that was given a token outside the vocabulary: every workgroup sees the same bad token
    // and skips its queue
    const bool bad_token = a.token_in && uni(sm->token) < 0;
    share_setup(sm);
    fetch_window(sm, 0);
    if (bad_token && tid == kConsumerThreads) {
        record_status(make_ctx<TR>(sm, 0, 0), MK_STATUS_BAD_TOKEN);
        sm->abort = MK_STATUS_BAD_TOKEN;
    }
    // From here on nothing refers to the kernel's arguments: what the loop needs comes from LDS.
    // The handlers get the address of a kernel-local word, into which a handler that refuses its
    // instruction writes why.  Nothing reads the word on the way from one instruction to the next (the
    // handlers' return values say whether to go on); it is there because a call that is handed the
    // address of a local cannot be marked as a tail call, and only then does the compiler drop the
    // callee-saved register traffic (dozens of scratch stores and reloads per instruction) from
    // handlers that only this kernel calls.
    int refusal = 0;
    const bool controller = uni(tid) >= kConsumerThreads;
    // A model whose residual projections take several column groups of the hidden width (8B: 4096 = 2 x 2048)
    // streams in phases that the memory system bounds, not the chain of hand-overs: its narrow rows (one
    // column group: half the registers of a full-width row) then pay to have more of them in flight.
    constexpr bool kWide = KC_HID != KC_RED;
    for (int step = 0; step < steps; step++) {
        bool stop = bad_token;
        const int num_slots = uni(sm->args.num_slots);
        for (int base = 0; base < num_slots && !stop; base += kQueueSlots) {
            if (uni(sm->window_base) != base) {
                wg_barrier();  // nobody is still reading the window that goes
                fetch_window(sm, base);
            }
            const int window_slots = min(kQueueSlots, num_slots - base);
            for (int slot = 0; slot < window_slots; slot++) {
                // (everything the loop branches on is the same in all lanes; saying so keeps the branches
                // scalar and the loop's state in a few scalar registers)
                const int opcode = uni(sm->queue[slot][0]);
                if (opcode == 0) continue;  // NoOp pads the queues (megakernels/scheduler.py:287-289)
                if constexpr (TR) {
                    const Ctx c = make_ctx<TR>(sm, slot, opcode);
                    trace_event(c, kEvStart);
                    if (c.trace && c.controller && c.lane == 0) st_plain_i32(c.trace + kEvOpcode, opcode);
                }
                bool ok = true;
                if (controller) {
                    if constexpr (kWide && MK_WIDE_CONTROLLER_CALL)
                        ok = uni((int)controller_step_call<TR, KC_HID, KC_RED, D>(sm, slot, opcode, &refusal)) != 0;
                    else
                        ok = uni((int)controller_step<TR, KC_HID, KC_RED, D>(sm, slot, opcode, &refusal)) != 0;
                } else switch (opcode) {
                case 1: ok = uni((int)op_matvec<TR, 1, KC_HID, kWide ? MK_WIDE_PARK_QKV : 0, 0, kWide>(sm, slot, &refusal)) != 0; break;
                case 2: ok = uni((int)op_attention<TR, D>(sm, slot, &refusal)) != 0; break;
                case 3: ok = uni((int)op_attention_reduction<TR, D>(sm, slot, &refusal)) != 0; break;
                case 4:
                    if constexpr (KC_HID == KC_RED && MK_PAIR_OPROJ_UPGATE) {
                        if (slot + 1 < window_slots && uni(sm->queue[slot + 1][0]) == 5) {
                            // rows can be parked when the wait is long (no attention just before, and a
                            // partition merge between attention and O-proj: with a single partition per head
                            // the wait is too short for it to pay) and the up/gate instruction is small
                            // enough (two list entries: eight rows per wave)
                            const int entries = uni(sm->queue[slot + 1][2]);
                            const bool park = (kParkedUpgateRows > 0 || kParkedDownRows > 0) && !uni(sm->args.skip_attn_reduction) &&
                                              (MK_PARK_ALL || slot == 0 || uni(sm->queue[slot - 1][0]) != 2) && entries >= 0 &&
                                              (kParkedUpgateRows == 0 || entries <= 2);
                            const int executed = uni(park ? op_oproj_upgate<TR, KC_HID, true>(sm, slot, &refusal)
                                                          : op_oproj_upgate<TR, KC_HID, false>(sm, slot, &refusal));
                            ok = executed > 0;
                            slot += ok ? executed - 1 : 0;
                            break;
                        }
                    }
                    ok = uni((int)op_matvec<TR, 4, KC_RED, 0, kWide ? MK_PF_WIDE_OPROJ : 0, false, kWide && MK_WIDE_AHEAD ? KC_HID : 0>(sm, slot, &refusal)) != 0;
                    break;
                case 5: ok = uni((int)op_matvec<TR, 5, KC_HID, kWide ? MK_WIDE_PARK_UPGATE : 0, 0, kWide>(sm, slot, &refusal)) != 0; break;
                case 6:
                    if constexpr (KC_HID == KC_RED && MK_PAIR_OPROJ_UPGATE && kParkedDownRows > 0) {
                        if (uni(sm->parked_slot) == slot) {
                            ok = uni((int)op_matvec<TR, 6, KC_RED, kParkedDownRows>(sm, slot, &refusal)) != 0;
                            break;
                        }
                    }
                    ok = uni((int)op_matvec<TR, 6, KC_RED, kWide ? MK_WIDE_PARK_DOWN : 0, kWide ? MK_PF_WIDE_DOWN : 0, kWide>(sm, slot, &refusal)) != 0;
                    break;
                case 7: ok = uni((int)op_lm_head<TR, KC_HID>(sm, slot, &refusal)) != 0; break;
                default: ok = bail(make_ctx<TR>(sm, slot, opcode), MK_STATUS_BAD_OPCODE, &refusal);  // reference: trap, include/util.cuh:38
                }
                if (!ok) {
                    stop = true;
                    break;
                }
                if constexpr (TR) trace_event(make_ctx<TR>(sm, slot, sm->queue[slot][0]), kEvEnd);
            }
        }
        if (stop && refusal != 0 && tid == 0) sm->abort = refusal;
        if (!uni((int)end_of_step<TR>(sm, step, steps))) break;
    }
}

// Self test: the one-instruction bf16 conversion against the portable round-to-nearest-even formula
// for every non-NaN binary32 input.  Each thread walks a strided slice of the 2^32 bit patterns.
__global__ void bf16_convert_sweep_kernel(unsigned long long *mismatches) {
    const uint32_t stride = gridDim.x * blockDim.x;
    unsigned long long bad = 0;
    uint32_t bits = blockIdx.x * blockDim.x + threadIdx.x;
    for (uint64_t i = bits; i < (1ull << 32); i += stride) {
        const float f = mkm::bits_f32((uint32_t)i);
        if (f != f) continue;
        bad += mkm::f32_to_bf16(f) != mkm::f32_to_bf16_soft(f);
    }
    if (bad) atomicAdd(mismatches, bad);
}

// ---------------------------------------------------------------------------------------------
// Workspace for callers that cannot allocate (mk_llama_launch_static): one array per GPU, held from
// the moment the library is loaded on that GPU until the process ends.  In host code the array's
// name is only a handle for hipGetSymbolAddress; kernels get the address that call returns.
// ---------------------------------------------------------------------------------------------
constexpr size_t kStaticScratchBytes = 2u << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

// Zeroes `count` 16-byte units.  A kernel rather than a memset: the launch may be recorded into a
// graph by the caller, where memset nodes are best avoided.
__global__ void scratch_clear_kernel(uint4 *dst, size_t count) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += stride) dst[i] = make_uint4(0, 0, 0, 0);
}

// the two-element bf16 dot product instruction applied to caller-supplied operands, for the test that
// compares its written-out definition with it
__global__ void dot2_apply_kernel(const uint32_t *a, const uint32_t *b, const float *acc, float *out, uint64_t n) {
    const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = dot2_bf16(a[i], b[i], acc[i]);
}

// ---------------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------------
thread_local char g_error[512] = "";

int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof g_error, fmt, ap);
    va_end(ap);
    return code;
}

using KernelFn = void (*)(const mk_llama_args);

KernelFn pick_kernel(int hid, int R, int D, bool timings) {
    if (hid == 2048 && R == 2048 && D == 64) return timings ? mk_llama_kernel<4, 4, 64, true> : mk_llama_kernel<4, 4, 64, false>;
    if (hid == 4096 && R == 2048 && D == 128) return timings ? mk_llama_kernel<8, 4, 128, true> : mk_llama_kernel<8, 4, 128, false>;
    if (hid == 512 && R == 512 && D == 64) return timings ? mk_llama_kernel<1, 1, 64, true> : mk_llama_kernel<1, 1, 64, false>;
    return nullptr;
}

}  // namespace

extern "C" {

uint64_t mk_llama_workspace_bytes(int32_t num_layers, int32_t hidden_size, int32_t intermediate_size,
                                  int32_t matvec_reduction_size) {
    if (num_layers <= 0 || hidden_size <= 0 || intermediate_size <= 0 || matvec_reduction_size <= 0) return 0;
    return ws_layout(num_layers, hidden_size, intermediate_size, matvec_reduction_size).total_bytes;
}

const char *mk_llama_last_error(void) { return g_error; }

int mk_llama_query(int what) {
    switch (what) {
    case 0: {
        int dev = 0, cus = 0;
        if (hipGetDevice(&dev) != hipSuccess) return -1;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return -1;
        return cus;
    }
    case 1: return (int)sizeof(Smem);
    case 2: return kThreads;
    case 3: return MK_LLAMA_ABI_VERSION;
    case 4: return kScoreCap;
    default: return -1;
    }
}

}  // extern "C"

namespace {

// validate the arguments against what the kernel assumes and pick the kernel instance
int validate(const mk_llama_args &a, KernelFn *kernel) {
    const void *required[] = {a.barriers, a.instructions, a.qkv_weights, a.attn_norm_weights, a.o_weights,
                              a.mlp_norm_weights, a.up_weights, a.gate_weights, a.down_weights,
                              a.lm_head_norm_weights, a.lm_head_weights, a.k_cache, a.v_cache, a.rope_cos,
                              a.rope_sin, a.hidden_states, a.q_post_rope, a.attn_out, a.attn_lse_intermediates,
                              a.attn_out_intermediates, a.silu_out, a.logits, a.workspace};
    for (const void *p : required) {
        if (!p) return fail(-2, "null device pointer in arguments");
        if ((uintptr_t)p % 16) return fail(-2, "device pointer %p is not 16-byte aligned", p);
    }
    const int hid = a.hidden_size, R = a.matvec_reduction_size, D = a.head_dim;
    if (a.num_layers <= 0 || a.num_workers <= 0 || a.num_slots <= 0) return fail(-3, "empty model or schedule");
    if (a.num_attention_heads != a.num_kv_heads * kGqa)
        return fail(-3, "unsupported head grouping: %d query heads for %d KV heads (need %d per KV head)",
                    a.num_attention_heads, a.num_kv_heads, kGqa);
    if (a.num_attention_heads * D != hid) return fail(-3, "num_attention_heads * head_dim must equal hidden_size");
    if (D < 64) return fail(-3, "head_dim must be at least 64");
    if (a.attn_reduction_size != kGqa) return fail(-3, "attn_reduction_size must be %d", kGqa);
    if (R <= 0 || hid % R || a.intermediate_size % R) return fail(-3, "sizes are not multiples of the reduction width");
    if (a.vocab_size % 16 || a.intermediate_size % 16) return fail(-3, "vocab and intermediate sizes must be multiples of 16");
    if (a.pos_id < 0 || a.pos_id >= a.kv_max_len || a.pos_id >= a.rope_positions)
        return fail(-4, "pos_id %d outside the KV cache (%d) or rope table (%d)", a.pos_id, a.kv_max_len,
                    a.rope_positions);
    if (a.max_partials < 1) return fail(-3, "max_partials must be positive");
    if (a.num_workers > kMaxWorkers) return fail(-3, "at most %d workers", kMaxWorkers);
    if (a.token_in) {
        if (!a.embed_table) return fail(-2, "token_in needs embed_table");
        if ((uintptr_t)a.embed_table % 16 || (uintptr_t)a.token_in % 8)
            return fail(-2, "embed_table must be 16-byte aligned and token_in 8-byte aligned");
    }
    if (a.token_out && (uintptr_t)a.token_out % 8) return fail(-2, "token_out must be 8-byte aligned");
    if (a.num_steps < 0) return fail(-3, "num_steps must not be negative");
    if (a.num_steps > 1) {
        if (!a.token_in || !a.token_out || !(a.flags & MK_FLAG_RESET_BARRIERS))
            return fail(-3, "several steps per launch need token_in, token_out and MK_FLAG_RESET_BARRIERS");
        // K / V rows that an earlier step of the launch wrote are read with ordinary cached loads, which is
        // sound as long as no cache line holds bytes of two (position, head) rows: a row's line must not
        // have been fetched, as a neighbour's, before the step that writes it
        if ((uintptr_t)a.k_cache % 128 || (uintptr_t)a.v_cache % 128)
            return fail(-2, "several steps per launch need k_cache and v_cache aligned to 128 bytes");
        const long long last = (long long)a.pos_id + a.num_steps - 1;
        if (last >= a.kv_max_len || last >= a.rope_positions)
            return fail(-4, "%d steps from position %d run past the KV cache (%d) or rope table (%d)", a.num_steps,
                        a.pos_id, a.kv_max_len, a.rope_positions);
    }
    // weight rows are addressed as 32-bit offsets into one buffer per matrix
    const uint64_t widest = 2ull * hid * (uint64_t)(a.vocab_size > a.intermediate_size ? a.vocab_size : a.intermediate_size);
    if (widest >= (1ull << 31)) return fail(-3, "a weight matrix of %llu bytes exceeds the 2 GiB a buffer can address", (unsigned long long)widest);
    KernelFn fn = pick_kernel(hid, R, D, (a.flags & MK_FLAG_TIMINGS) != 0 && a.timings != nullptr);
    if (!fn) return fail(-5, "no kernel instance for hidden %d, reduction width %d, head_dim %d", hid, R, D);
    const uint64_t need = mk_llama_workspace_bytes(a.num_layers, hid, a.intermediate_size, R);
    if (a.workspace_bytes < need)
        return fail(-6, "workspace has %llu bytes, %llu needed", (unsigned long long)a.workspace_bytes,
                    (unsigned long long)need);
    if ((uintptr_t)a.workspace % 16) return fail(-6, "workspace must be 16-byte aligned");

    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
        return fail(-7, "cannot query the device");
    // all workers must be resident at once or the barrier waits can never be satisfied
    if (a.num_workers > cus)
        return fail(-7, "schedule has %d workers but the device has %d compute units", a.num_workers, cus);

    *kernel = fn;
    return 0;
}

int launch_kernel(KernelFn fn, const mk_llama_args &a, void *hip_stream) {
    // Per kernel instance, once: allow the LDS request, and ask the runtime how many workgroups of
    // this shape the device holds at once.  Every barrier wait assumes that all workers are running
    // (the reference: one block per SM by __launch_bounds__(NUM_THREADS, 1) and grid = SM count,
    // include/megakernel.cuh:166-171), so a grid that cannot be resident as a whole is refused here
    // rather than found out by the waits' time limit.
    struct Configured {
        KernelFn fn;
        int device, resident;
    };
    static thread_local Configured configured[16] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return fail(-7, "cannot query the device");
    int resident = -1;
    for (const Configured &k : configured)
        if (k.fn == fn && k.device == dev) resident = k.resident;
    if (resident < 0) {
        hipError_t e = hipFuncSetAttribute((const void *)fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)sizeof(Smem));
        if (e != hipSuccess) return fail(-8, "hipFuncSetAttribute: %s", hipGetErrorString(e));
        int per_cu = 0, cus = 0;
        e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, (const void *)fn, kThreads, sizeof(Smem));
        if (e != hipSuccess) return fail(-8, "hipOccupancyMaxActiveBlocksPerMultiprocessor: %s", hipGetErrorString(e));
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
            return fail(-7, "cannot query the device");
        resident = per_cu * cus;
        for (Configured &k : configured)
            if (!k.fn) {
                k = Configured{fn, dev, resident};
                break;
            }
    }
    if (a.num_workers > resident)
        return fail(-7, "schedule has %d workers but only %d workgroups of this kernel can be resident at once", a.num_workers,
                    resident);
    hipLaunchKernelGGL(fn, dim3(a.num_workers), dim3(kThreads), sizeof(Smem), (hipStream_t)hip_stream, a);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(-9, "kernel launch: %s", hipGetErrorString(e));
    return 0;
}

// device address of this GPU's copy of `scratch`, looked up once per device
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void *g_scratch_ptr[kMaxDevices] = {};

int static_scratch(void **out) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return fail(-7, "cannot query the device");
    if (dev < 0 || dev >= kMaxDevices) return fail(-7, "device index %d beyond the %d the library keeps scratch addresses for", dev, kMaxDevices);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *ptr = nullptr;
        hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr) return fail(-8, "hipGetSymbolAddress(scratch): %s", hipGetErrorString(e));
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return 0;
}

}  // namespace

extern "C" {

int mk_llama_launch(const mk_llama_args *args, void *hip_stream) {
    g_error[0] = 0;
    if (!args) return fail(-1, "null arguments");
    KernelFn fn = nullptr;
    if (const int rc = validate(*args, &fn)) return rc;
    return launch_kernel(fn, *args, hip_stream);
}

int mk_llama_launch_static(const mk_llama_args *args, void *hip_stream, void **scratch_out) {
    g_error[0] = 0;
    if (!args) return fail(-1, "null arguments");
    mk_llama_args a = *args;
    const uint64_t need = mk_llama_workspace_bytes(a.num_layers, a.hidden_size, a.intermediate_size, a.matvec_reduction_size);
    if (need == 0) return fail(-3, "empty model or schedule");
    if (need > kStaticScratchBytes)
        return fail(-6, "these shapes need %llu bytes of workspace, the library's static scratch holds %llu: use mk_llama_launch with a caller-owned workspace",
                    (unsigned long long)need, (unsigned long long)kStaticScratchBytes);
    void *ptr = nullptr;
    if (const int rc = static_scratch(&ptr)) return rc;
    a.workspace = ptr;
    a.workspace_bytes = kStaticScratchBytes;
    KernelFn fn = nullptr;
    if (const int rc = validate(a, &fn)) return rc;
    if (scratch_out) *scratch_out = ptr;
    // The array keeps whatever the last call left: counters are back at zero after a launch that
    // completed, but the residual partial sums of other shapes may lie where this call's counters
    // go, and a launch that gave up leaves its status behind.  Everything this call uses starts at zero.
    const size_t units = (size_t)((need + 15) / 16);
    hipLaunchKernelGGL(scratch_clear_kernel, dim3((unsigned)((units + 255) / 256)), dim3(256), 0, (hipStream_t)hip_stream,
                       static_cast<uint4 *>(ptr), units);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(-9, "scratch clear launch: %s", hipGetErrorString(e));
    return launch_kernel(fn, a, hip_stream);
}

int mk_llama_selftest_bf16(uint64_t *mismatches_out) {
    g_error[0] = 0;
    if (!mismatches_out) return fail(-1, "null pointer");
    unsigned long long *dev = nullptr;
    hipError_t e = hipMalloc(&dev, sizeof *dev);
    if (e != hipSuccess) return fail(-9, "hipMalloc: %s", hipGetErrorString(e));
    (void)hipMemset(dev, 0, sizeof *dev);
    hipLaunchKernelGGL(bf16_convert_sweep_kernel, dim3(4096), dim3(256), 0, 0, dev);
    unsigned long long host = 0;
    e = hipMemcpy(&host, dev, sizeof host, hipMemcpyDeviceToHost);
    (void)hipFree(dev);
    if (e != hipSuccess) return fail(-9, "self test: %s", hipGetErrorString(e));
    *mismatches_out = host;
    return 0;
}

int mk_llama_selftest_dot2(const void *a, const void *b, const void *acc, void *out, uint64_t n, void *hip_stream) {
    g_error[0] = 0;
    if (!a || !b || !acc || !out) return fail(-1, "null pointer");
    if (n == 0) return 0;
    if (n > ((uint64_t)1 << 31)) return fail(-2, "at most 2^31 cases per call");
    hipLaunchKernelGGL(dot2_apply_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)hip_stream,
                       static_cast<const uint32_t *>(a), static_cast<const uint32_t *>(b), static_cast<const float *>(acc),
                       static_cast<float *>(out), n);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(-9, "dot2 self test launch: %s", hipGetErrorString(e));
    return 0;
}

int mk_llama_read_status(void *workspace, void *hip_stream, int32_t out[4]) {
    g_error[0] = 0;
    if (!workspace || !out) return fail(-1, "null pointer");
    hipError_t e = hipStreamSynchronize((hipStream_t)hip_stream);
    if (e != hipSuccess) return fail(-9, "hipStreamSynchronize: %s", hipGetErrorString(e));
    e = hipMemcpy(out, workspace, 4 * sizeof(int32_t), hipMemcpyDeviceToHost);
    if (e != hipSuccess) return fail(-9, "hipMemcpy: %s", hipGetErrorString(e));
    return 0;
}

}  // extern "C"
