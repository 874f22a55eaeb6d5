// Batch-1 Llama decode as one persistent kernel for MI355X (gfx950).
//
// Execution model (counterpart of the reference VM runtime, include/megakernel.cuh:15-171,
// include/controller/controller.cuh:24-132, include/util.cuh:260-304, rebuilt for CDNA4):
//   * grid = one workgroup per compute unit, 1024 threads = 16 wave64; workgroup w executes
//     instructions[w, 0..num_slots) strictly in order.  An LDS request above half the CU's
//     160 KB keeps a second workgroup off the same CU.
//   * there are no specialised loader / storer / controller wavefronts: every wave issues its
//     own 16-byte global loads and keeps several weight rows in flight in VGPRs.  The first
//     rows of an instruction are requested BEFORE the instruction waits for its dependency,
//     because weights never depend on the barrier.
//   * cross-CU ordering is only through counters in HBM, with the counts of the reference's
//     Python VM (megakernels/demos/latency/python_vm.py).  The eight XCDs have private L2
//     caches, so everything one CU writes for another (activations, the new KV row, counters)
//     is stored write-through and loaded with agent-scope ("sc1") accesses; no cache-wide
//     write-back / invalidate is ever issued.  A producer's stores are complete
//     (s_waitcnt vmcnt(0), part of __syncthreads) before it bumps the counter.
//   * the four counters that receive one arrival per worker (barriers[l, 2..5, 0]) are kept
//     as 16 shards in the workspace while the kernel runs (256 atomics on one address cost
//     ~3 us, 16 per shard ~0.2 us); the last workgroup to finish adds the shard totals into
//     `barriers`, so after the launch the tensor holds exactly the reference VM's counts.
//   * every barrier wait is bounded (spin_limit_us): on expiry the worker records a status
//     code and every workgroup leaves its instruction loop, so the grid always drains.
//
// Arithmetic: bit-compatible with a fixed "lane order" so results can be compared exactly
// with a CPU restatement of the Python VM.  A dot product over K elements is computed by one
// wave: lane l owns elements j*512 + l*8 + e and accumulates them in that order with fmaf,
// the 64 lane sums are combined by an xor butterfly (a balanced pairwise tree).  Narrowing
// to bf16 happens exactly where the Python VM narrows (python_vm.py:29-80,127-274).
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <cstring>

#include "../../include/mk_llama.h"
#include "mk_math.h"

namespace {

constexpr int kThreads = 1024;
constexpr int kWaves = 16;
constexpr int kShards = 16;         // shards per hot barrier counter
constexpr int kHotRows = 4;         // barrier rows 2..5 are sharded
constexpr int kOutRows = 2048;      // rows staged in LDS between matvec and epilogue
constexpr int kScoreCap = 6144;     // tokens per attention partition (LDS score buffer)
constexpr int kMaxHeadDim = 128;
constexpr int kGqaMax = 4;          // query heads per KV head handled by one attention instruction
constexpr int kStatusInts = 16;
constexpr int kDoneSlot = 8;        // workspace int: workgroups finished

// weight rows in flight per wave: bounded by the 128 VGPRs a 1024-thread workgroup leaves each lane
template <int KC>
constexpr int rows_in_flight(int want) { return KC <= 4 ? want : 1; }

#define AG __HIP_MEMORY_SCOPE_AGENT

// ---------------------------------------------------------------------------------------------
// workspace layout (ints unless noted)
// ---------------------------------------------------------------------------------------------
struct WsLayout {
    size_t status, shards, arrive_o, arrive_d, partial, total_bytes;
};

__host__ __device__ inline WsLayout ws_layout(int L, int hid, int inter, int R) {
    WsLayout w;
    size_t off = 0;
    w.status = off;   off += kStatusInts;
    w.shards = off;   off += (size_t)kShards * L * kHotRows;
    w.arrive_o = off; off += hid / 16;
    w.arrive_d = off; off += hid / 16;
    off = (off + 3) & ~(size_t)3;
    w.partial = off;  // floats: [max(groups_o, groups_d)][hid]
    int g_o = hid / R, g_d = inter / R;
    off += (size_t)(g_o > g_d ? g_o : g_d) * hid;
    w.total_bytes = off * 4;
    return w;
}

// ---------------------------------------------------------------------------------------------
// LDS layout
// ---------------------------------------------------------------------------------------------
struct Smem {
    int abort;                      // set once, never cleared during a launch
    int last_flag;
    int pad[2];
    int flags[kOutRows / 16];       // per-block "I was the last arriver" (matvec-add)
    float out[kOutRows];            // matvec row results awaiting the epilogue
    float wave_max[kWaves][kGqaMax];
    float wave_l[kWaves][kGqaMax];
    float head_m[kGqaMax];
    float head_w[kGqaMax][32];      // reduction weights
    float wave_o[kWaves][kGqaMax][kMaxHeadDim];
    float scores[kGqaMax][kScoreCap];
};

// ---------------------------------------------------------------------------------------------
// agent-coherent memory access (bypass the non-coherent per-XCD L2 contents)
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ int ld_i32(const int *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, AG); }
__device__ __forceinline__ uint32_t ld_u32(const void *p) {
    return __hip_atomic_load((const uint32_t *)p, __ATOMIC_RELAXED, AG);
}
__device__ __forceinline__ uint64_t ld_u64(const void *p) {
    return __hip_atomic_load((const uint64_t *)p, __ATOMIC_RELAXED, AG);
}
__device__ __forceinline__ float ld_f32(const float *p) { return mkm::bits_f32(ld_u32(p)); }
__device__ __forceinline__ void st_u32(void *p, uint32_t v) {
    __hip_atomic_store((uint32_t *)p, v, __ATOMIC_RELAXED, AG);
}
__device__ __forceinline__ void st_f32(float *p, float v) { st_u32(p, mkm::f32_bits(v)); }
__device__ __forceinline__ void st_i32(int *p, int v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, AG); }
__device__ __forceinline__ void add_i32(int *p, int v) { __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, AG); }
__device__ __forceinline__ uint4 ld_b128(const void *p) {
    uint64_t a = ld_u64(p), b = ld_u64((const char *)p + 8);
    return make_uint4((uint32_t)a, (uint32_t)(a >> 32), (uint32_t)b, (uint32_t)(b >> 32));
}
// immutable data (weights, rope tables, old KV rows): ordinary cached 16-byte load
__device__ __forceinline__ uint4 ld_const_b128(const void *p) { return *(const uint4 *)p; }

// ---------------------------------------------------------------------------------------------
// wave-level reductions: xor butterfly in ascending offset order = pairwise tree in lane order
// ---------------------------------------------------------------------------------------------
template <int FROM = 1, int TO = 64>
__device__ __forceinline__ float lane_tree_sum(float v) {
#pragma unroll
    for (int o = FROM; o < TO; o <<= 1) v = v + __shfl_xor(v, o);
    return v;
}
template <int FROM = 1, int TO = 64>
__device__ __forceinline__ float lane_tree_max(float v) {
#pragma unroll
    for (int o = FROM; o < TO; o <<= 1) v = fmaxf(v, __shfl_xor(v, o));
    return v;
}
__device__ __forceinline__ int lane_sum_i32(int v) {
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) v += __shfl_xor(v, o);
    return v;
}

// ---------------------------------------------------------------------------------------------
// per-workgroup context
// ---------------------------------------------------------------------------------------------
struct Ctx {
    const mk_llama_args &a;
    Smem *sm;
    int *status;
    int *shards;
    int *arrive_o, *arrive_d;
    float *partial;
    int tid, wave, lane;
    int worker, slot, opcode;
    long long spin_ticks;           // wall-clock ticks (100 MHz) a wait may take
    int barrier_cols;               // H + 2 KVH
};

__device__ __forceinline__ int *bar_ptr(const Ctx &c, int layer, int row, int col) {
    return c.a.barriers + ((size_t)layer * MK_BARRIER_ROWS + row) * c.barrier_cols + col;
}
__device__ __forceinline__ int *shard_ptr(const Ctx &c, int shard, int layer, int row) {
    return c.shards + ((size_t)shard * c.a.num_layers + layer) * kHotRows + (row - 2);
}

// first error wins
__device__ void record_status(const Ctx &c, int code) {
    int expected = 0;
    if (__hip_atomic_compare_exchange_strong(&c.status[0], &expected, code, __ATOMIC_RELAXED, __ATOMIC_RELAXED, AG)) {
        st_i32(&c.status[1], c.worker);
        st_i32(&c.status[2], c.slot);
        st_i32(&c.status[3], c.opcode);
    }
}

// Executed by all lanes of wave 0.  `ptr` is this lane's counter or nullptr.  sum_mode: wait until
// the sum over lanes reaches target (sharded counter + its base value); otherwise wait until every
// lane's counter reaches target.  Lane 63 watches the global status word so that one worker's
// failure releases everybody.
__device__ bool poll_wave0(const Ctx &c, const int *ptr, bool sum_mode, int target) {
    const long long t0 = wall_clock64();
    while (true) {
        const int v = ptr ? ld_i32(ptr) : 0;
        const int st = c.lane == 63 ? ld_i32(c.status) : 0;
        const bool ok = sum_mode ? (lane_sum_i32(v) >= target) : (bool)__all(ptr == nullptr || v >= target);
        if (ok) return true;
        if (__any(st != 0)) return false;
        if (wall_clock64() - t0 > c.spin_ticks) {
            if (c.lane == 0) record_status(c, MK_STATUS_BARRIER_TIMEOUT);
            return false;
        }
        __builtin_amdgcn_s_sleep(2);
    }
}

// Every instruction starts here: wave 0 waits for the dependency, then one workgroup barrier
// publishes the outcome.  The barrier also separates the previous instruction's epilogue reads of
// LDS from this instruction's writes.  Returns false when the launch is being abandoned.
template <class Poll>
__device__ __forceinline__ bool wait_dependency(const Ctx &c, Poll poll) {
    if (c.wave == 0) {
        if (!poll()) c.sm->abort = 1;
    }
    __syncthreads();
    return c.sm->abort == 0;
}

__device__ __forceinline__ bool wait_sharded(const Ctx &c, int layer, int row, int target) {
    return wait_dependency(c, [&]() {
        const int *p = nullptr;
        if (c.lane < kShards) p = shard_ptr(c, c.lane, layer, row);
        else if (c.lane == kShards) p = bar_ptr(c, layer, row, 0);
        return poll_wave0(c, p, true, target);
    });
}
__device__ __forceinline__ bool wait_nothing(const Ctx &c) {
    return wait_dependency(c, [&]() { return true; });
}
// malformed instruction: record it and abandon the launch (all threads of the workgroup call this)
__device__ __forceinline__ bool bail(const Ctx &c, int code) {
    if (c.tid == 0) {
        record_status(c, code);
        c.sm->abort = 1;
    }
    __syncthreads();
    return false;
}

// one arrival on a sharded counter; call from ONE thread after a __syncthreads that followed
// the stores being published
__device__ __forceinline__ void signal_sharded(const Ctx &c, int layer, int row, int count) {
    add_i32(shard_ptr(c, c.worker & (kShards - 1), layer, row), count);
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

// python_vm.py:50-56: w * bf16(x * rsqrt(mean(x^2) + eps)), statistics in fp32.  Every wave
// computes the whole vector for itself (4-8 KB from the memory-side cache), so no LDS and no
// workgroup barrier are involved.
template <int KC>
__device__ __forceinline__ void rms_norm_x(XVec<KC> &x, const uint16_t *hidden, const uint16_t *weight, float eps,
                                           int lane) {
    uint4 wraw[KC];
#pragma unroll
    for (int j = 0; j < KC; j++) wraw[j] = ld_const_b128(weight + j * 512 + lane * 8);
    load_x<KC>(x, hidden, lane);
    float acc = 0.0f;
#pragma unroll
    for (int j = 0; j < KC; j++)
#pragma unroll
        for (int e = 0; e < 8; e++) acc = fmaf(x.v[j][e], x.v[j][e], acc);
    const float mean = lane_tree_sum(acc) / (float)(KC * 512);
    const float inv = 1.0f / sqrtf(mean + eps);
#pragma unroll
    for (int j = 0; j < KC; j++) {
        float wv[8];
        unpack8(wraw[j], wv);
#pragma unroll
        for (int e = 0; e < 8; e++) x.v[j][e] = mkm::round_bf16(wv[e] * mkm::round_bf16(x.v[j][e] * inv));
    }
}

template <int KC>
__device__ __forceinline__ void load_row(uint4 (&w)[KC], const uint16_t *row, int lane) {
#pragma unroll
    for (int j = 0; j < KC; j++) w[j] = ld_const_b128(row + j * 512 + lane * 8);
}

template <int KC>
__device__ __forceinline__ float dot_row(const uint4 (&w)[KC], const XVec<KC> &x) {
    float acc = 0.0f;
#pragma unroll
    for (int j = 0; j < KC; j++) {
        acc = fmaf(mkm::bf16_lo(w[j].x), x.v[j][0], acc);
        acc = fmaf(mkm::bf16_hi(w[j].x), x.v[j][1], acc);
        acc = fmaf(mkm::bf16_lo(w[j].y), x.v[j][2], acc);
        acc = fmaf(mkm::bf16_hi(w[j].y), x.v[j][3], acc);
        acc = fmaf(mkm::bf16_lo(w[j].z), x.v[j][4], acc);
        acc = fmaf(mkm::bf16_hi(w[j].z), x.v[j][5], acc);
        acc = fmaf(mkm::bf16_lo(w[j].w), x.v[j][6], acc);
        acc = fmaf(mkm::bf16_hi(w[j].w), x.v[j][7], acc);
    }
    return lane_tree_sum(acc);
}

// Streams `ntasks` weight rows through the workgroup: task t is handled by wave t % 16 and its
// bf16-rounded dot product lands in sm->out[t].  PF rows per wave are in flight; the first PF are
// requested before `wait` (the dependency) and `make_x` (the activation vector) run.
template <int KC, int PF, class RowPtr, class Wait, class MakeX>
__device__ __forceinline__ bool stream_rows(const Ctx &c, int ntasks, RowPtr row_ptr, Wait wait, MakeX make_x) {
    const int mine = ntasks > c.wave ? (ntasks - c.wave + kWaves - 1) / kWaves : 0;
    uint4 buf[PF][KC];
#pragma unroll
    for (int s = 0; s < PF; s++)
        if (s < mine) load_row<KC>(buf[s], row_ptr(c.wave + s * kWaves), c.lane);
    if (!wait()) return false;
    XVec<KC> x;
    make_x(x);
    for (int base = 0; base < mine; base += PF) {
#pragma unroll
        for (int s = 0; s < PF; s++) {
            const int i = base + s;
            if (i < mine) {
                const float y = mkm::round_bf16(dot_row<KC>(buf[s], x));
                if (i + PF < mine) load_row<KC>(buf[s], row_ptr(c.wave + (i + PF) * kWaves), c.lane);
                if (c.lane == 0) c.sm->out[c.wave + i * kWaves] = y;
            }
        }
    }
    return true;
}

// ---------------------------------------------------------------------------------------------
// opcode 1: RMSNorm + QKV matvec + RoPE + KV append  (python_vm.py:168-248;
// reference device op: demos/low-latency-llama/rms_matvec_rope_append.cu:10-231)
// ---------------------------------------------------------------------------------------------
template <int KC>
__device__ bool op_qkv(const Ctx &c, const int *ins) {
    const mk_llama_args &a = c.a;
    const int layer = ins[1], start = ins[2], end = ins[3];
    const int hid = a.hidden_size, D = a.head_dim, H = a.num_attention_heads, KVH = a.num_kv_heads;
    const int total_blocks = (H + 2 * KVH) * D / 16;
    if (layer < 0 || layer >= a.num_layers || start < 0 || end > total_blocks || end - start > kOutRows / 16) return bail(c, MK_STATUS_BAD_INSTRUCTION);
    const int nblk = end > start ? end - start : 0;
    const uint16_t *W = a.qkv_weights + (size_t)layer * total_blocks * 16 * hid;
    const int down_jobs = (a.intermediate_size / a.matvec_reduction_size) * (hid / 16);

    const bool ok = stream_rows<KC, rows_in_flight<KC>(2)>(
        c, nblk * 16, [&](int t) { return W + (size_t)(start * 16 + t) * hid; },
        [&]() { return layer > 0 ? wait_sharded(c, layer - 1, 5, down_jobs) : wait_nothing(c); },
        [&](XVec<KC> &x) {
            if (nblk > 0)
                rms_norm_x<KC>(x, a.hidden_states, a.attn_norm_weights + (size_t)layer * hid, a.rms_norm_eps, c.lane);
        });
    if (!ok) return false;
    if (nblk == 0) return true;
    __syncthreads();

    // epilogue: one thread per adjacent row pair
    const int k_start = H * D, v_start = k_start + KVH * D;
    if (c.tid < nblk * 8) {
        const int lb = c.tid >> 3, pair = c.tid & 7;
        const int row0 = (start + lb) * 16 + pair * 2;
        const float y0 = c.sm->out[lb * 16 + pair * 2], y1 = c.sm->out[lb * 16 + pair * 2 + 1];
        uint32_t packed;
        if (row0 < v_start) {
            // interleaved rotary embedding (llama.py:136-174): products and sum in fp32, unfused
            const int d = row0 % D;
            const float *cs = a.rope_cos + (size_t)a.pos_id * D + d;
            const float *sn = a.rope_sin + (size_t)a.pos_id * D + d;
            const float even = (y0 * cs[0]) + ((-y1) * sn[0]);
            const float odd = (y1 * cs[1]) + (y0 * sn[1]);
            packed = mkm::pack_bf16(even, odd);
        } else {
            packed = mkm::pack_bf16(y0, y1);
        }
        uint16_t *dst;
        const size_t kv_row = ((size_t)layer * a.kv_max_len + a.pos_id) * KVH * D;
        if (row0 < k_start) dst = a.q_post_rope + row0;
        else if (row0 < v_start) dst = a.k_cache + kv_row + (row0 - k_start);
        else dst = a.v_cache + kv_row + (row0 - v_start);
        st_u32(dst, packed);
    }
    __syncthreads();
    // one arrival per block on the head's counter (python_vm.py:248)
    if (c.tid < nblk) add_i32(bar_ptr(c, layer, 0, (start + c.tid) / (D / 16)), 1);
    return true;
}

// ---------------------------------------------------------------------------------------------
// opcodes 4 and 6: matvec over one column group + residual add  (python_vm.py:59-124;
// reference device op: demos/low-latency-llama/matvec_adds.cu:10-192).
// With several column groups each (group, block) job parks its bf16-rounded partial in the
// workspace; the job that arrives last on the block's counter applies the partials to the
// residual in group order, which is the order the Python VM applies them in, so the bf16
// rounding chain is reproduced without serialising the workers.
// ---------------------------------------------------------------------------------------------
template <int KC>
__device__ bool op_matvec_add(const Ctx &c, const int *ins, bool is_down) {
    const mk_llama_args &a = c.a;
    const int layer = ins[1], start = ins[2], end = ins[3], group = ins[4];
    const int hid = a.hidden_size, R = a.matvec_reduction_size;
    const int in_dim = is_down ? a.intermediate_size : hid;
    const int ngroups = in_dim / R;
    if (layer < 0 || layer >= a.num_layers || start < 0 || end > hid / 16 || group < 0 || group >= ngroups ||
        end - start > kOutRows / 16) return bail(c, MK_STATUS_BAD_INSTRUCTION);
    const int nblk = end > start ? end - start : 0;
    const uint16_t *W = (is_down ? a.down_weights : a.o_weights) + (size_t)layer * hid * in_dim + (size_t)group * R;
    const uint16_t *vec = (is_down ? a.silu_out : a.attn_out) + (size_t)group * R;
    const int wait_row = is_down ? 4 : 2;
    const int wait_target = is_down ? a.intermediate_size / 16 : a.num_attention_heads;

    const bool ok = stream_rows<KC, rows_in_flight<KC>(2)>(
        c, nblk * 16, [&](int t) { return W + (size_t)(start * 16 + t) * in_dim; },
        [&]() { return wait_sharded(c, layer, wait_row, wait_target); },
        [&](XVec<KC> &x) {
            if (nblk > 0) load_x<KC>(x, vec, c.lane);
        });
    if (!ok) return false;
    if (nblk == 0) return true;
    __syncthreads();

    uint16_t *resid = a.hidden_states;
    if (ngroups == 1) {
        if (c.tid < nblk * 8) {
            const int t0 = c.tid * 2;
            const int row0 = start * 16 + t0;
            const uint32_t h = ld_u32(resid + row0);
            const float lo = mkm::bf16_lo(h) + c.sm->out[t0];
            const float hi = mkm::bf16_hi(h) + c.sm->out[t0 + 1];
            st_u32(resid + row0, mkm::pack_bf16(lo, hi));
        }
    } else {
        int *arrive = is_down ? c.arrive_d : c.arrive_o;
        if (c.tid < nblk * 16) st_f32(c.partial + (size_t)group * hid + start * 16 + c.tid, c.sm->out[c.tid]);
        __syncthreads();
        if (c.tid < nblk) {
            const int old = __hip_atomic_fetch_add(&arrive[start + c.tid], 1, __ATOMIC_RELAXED, AG);
            const int last = old == ngroups - 1;
            if (last) st_i32(&arrive[start + c.tid], 0);
            c.sm->flags[c.tid] = last;
        }
        __syncthreads();
        if (c.tid < nblk * 8 && c.sm->flags[c.tid >> 3]) {
            const int row0 = start * 16 + c.tid * 2;
            const uint32_t h = ld_u32(resid + row0);
            float lo = mkm::bf16_lo(h), hi = mkm::bf16_hi(h);
            for (int g = 0; g < ngroups; g++) {
                const uint64_t p = ld_u64(c.partial + (size_t)g * hid + row0);
                lo = mkm::round_bf16(lo + mkm::bits_f32((uint32_t)p));
                hi = mkm::round_bf16(hi + mkm::bits_f32((uint32_t)(p >> 32)));
            }
            st_u32(resid + row0, mkm::pack_bf16(lo, hi));
        }
    }
    __syncthreads();
    if (c.tid == 0) signal_sharded(c, layer, is_down ? 5 : 3, nblk);
    return true;
}

// ---------------------------------------------------------------------------------------------
// opcode 5: RMSNorm + up and gate matvecs + SiLU  (python_vm.py:127-165;
// reference device op: demos/low-latency-llama/upgate.cu:10-172)
// ---------------------------------------------------------------------------------------------
template <int KC>
__device__ bool op_upgate(const Ctx &c, const int *ins) {
    const mk_llama_args &a = c.a;
    const int layer = ins[1], n = ins[2];
    const int hid = a.hidden_size, inter = a.intermediate_size;
    bool bad = layer < 0 || layer >= a.num_layers || n < 0 || n > MK_INSTRUCTION_WORDS - 3 || n * 32 > kOutRows;
    if (!bad)
        for (int i = 0; i < n; i++) bad |= ins[3 + i] < 0 || ins[3 + i] >= inter / 16;
    if (bad) return bail(c, MK_STATUS_BAD_INSTRUCTION);
    const uint16_t *Wu = a.up_weights + (size_t)layer * inter * hid;
    const uint16_t *Wg = a.gate_weights + (size_t)layer * inter * hid;
    const int o_jobs = (hid / a.matvec_reduction_size) * (hid / 16);

    // task t: list entry t / 32, matrix (t / 16) & 1 (0 up, 1 gate), row t % 16
    const bool ok = stream_rows<KC, rows_in_flight<KC>(4)>(
        c, n * 32,
        [&](int t) {
            const int blk = ins[3 + (t >> 5)];
            return ((t >> 4) & 1 ? Wg : Wu) + (size_t)(blk * 16 + (t & 15)) * hid;
        },
        [&]() { return wait_sharded(c, layer, 3, o_jobs); },
        [&](XVec<KC> &x) {
            if (n > 0)
                rms_norm_x<KC>(x, a.hidden_states, a.mlp_norm_weights + (size_t)layer * hid, a.rms_norm_eps, c.lane);
        });
    if (!ok) return false;
    if (n == 0) return true;
    __syncthreads();
    if (c.tid < n * 8) {
        const int i = c.tid >> 3, pair = c.tid & 7;
        const float *up = c.sm->out + i * 32, *gate = up + 16;
        const int r = pair * 2;
        // silu(gate) -> bf16, then times up -> bf16 (python_vm.py:161-163)
        const float s0 = mkm::round_bf16(mkm::silu_exact(gate[r]));
        const float s1 = mkm::round_bf16(mkm::silu_exact(gate[r + 1]));
        st_u32(a.silu_out + ins[3 + i] * 16 + r, mkm::pack_bf16(s0 * up[r], s1 * up[r + 1]));
    }
    __syncthreads();
    if (c.tid == 0) signal_sharded(c, layer, 4, n);
    return true;
}

// ---------------------------------------------------------------------------------------------
// opcode 7: final RMSNorm + LM head  (python_vm.py:251-274;
// reference device op: demos/low-latency-llama/rms_lm_head.cu:10-117)
// ---------------------------------------------------------------------------------------------
template <int KC>
__device__ bool op_lm_head(const Ctx &c, const int *ins) {
    const mk_llama_args &a = c.a;
    const int start = ins[1], end = ins[2];
    const int hid = a.hidden_size;
    if (start < 0 || end > a.vocab_size / 16) return bail(c, MK_STATUS_BAD_INSTRUCTION);
    const int down_jobs = (a.intermediate_size / a.matvec_reduction_size) * (hid / 16);
    const int blocks_per_batch = kOutRows / 16;
    bool first = true;
    int b0 = start;
    do {
        const int b1 = min(b0 + blocks_per_batch, end);
        const int nblk = b1 > b0 ? b1 - b0 : 0;
        const bool ok = stream_rows<KC, rows_in_flight<KC>(4)>(
            c, nblk * 16, [&](int t) { return a.lm_head_weights + (size_t)(b0 * 16 + t) * hid; },
            [&]() { return first ? wait_sharded(c, a.num_layers - 1, 5, down_jobs) : wait_nothing(c); },
            [&](XVec<KC> &x) {
                if (nblk > 0) rms_norm_x<KC>(x, a.hidden_states, a.lm_head_norm_weights, a.rms_norm_eps, c.lane);
            });
        if (!ok) return false;
        __syncthreads();
        for (int p = c.tid; p < nblk * 8; p += kThreads)
            st_u32(a.logits + b0 * 16 + p * 2, mkm::pack_bf16(c.sm->out[p * 2], c.sm->out[p * 2 + 1]));
        first = false;
        b0 = b1;
    } while (b0 < end);
    return true;
}

// ---------------------------------------------------------------------------------------------
// opcode 2: attention of the G query heads of one KV head over one partition of the cache
// (python_vm.py:277-346; reference device op: demos/low-latency-llama/attention_partial.cu).
// Two passes over LDS-resident scores: (1) s = scale * q.k for every token, exact maximum;
// (2) p = exp(s - max), slot sums of p and p*v.  Token r of the partition belongs to slot
// r mod NSLOT with NSLOT = 16 waves * (64 / (D/8)) tokens per wave load; a slot accumulates its
// tokens in increasing order and slots are combined by a pairwise tree (lanes, then waves).
// ---------------------------------------------------------------------------------------------
template <int D>
__device__ bool op_attention(const Ctx &c, const int *ins) {
    constexpr int LPT = D / 8;            // lanes per token
    constexpr int TPW = 64 / LPT;         // tokens per wave per round
    constexpr int NSLOT = kWaves * TPW;   // tokens per workgroup round
    constexpr int G = kGqaMax;
    const mk_llama_args &a = c.a;
    Smem *sm = c.sm;
    const int layer = ins[1], kvh = ins[2], P = ins[3], pidx = ins[4];
    const int H = a.num_attention_heads, KVH = a.num_kv_heads;
    const bool skip = a.skip_attn_reduction != 0;
    if (layer < 0 || layer >= a.num_layers || kvh < 0 || kvh >= KVH || P < 1 || pidx < 0 || pidx >= P ||
        (!skip && pidx >= a.max_partials)) return bail(c, MK_STATUS_BAD_INSTRUCTION);
    const int seq_len = a.pos_id + 1;
    const int total_blocks = (seq_len + 15) / 16;
    const int bpp = (total_blocks + P - 1) / P;
    const int sb = pidx * bpp;
    const int eb = min(sb + bpp, total_blocks);
    const int t0 = sb * 16;
    const int t1 = min(eb * 16, seq_len);
    const int T = t1 > t0 ? t1 - t0 : 0;
    if (T > kScoreCap) return bail(c, MK_STATUS_ATTN_TOO_LONG);
    const int h0 = kvh * G;
    const int sub = c.lane % LPT;         // which 8 dims of the head this lane owns
    const int tok_in_wave = c.lane / LPT;
    const int slot = c.wave * TPW + tok_in_wave;
    const size_t tok_stride = (size_t)KVH * D;
    const size_t base = ((size_t)layer * a.kv_max_len) * tok_stride + (size_t)kvh * D + sub * 8;
    const uint16_t *kbase = a.k_cache + base;
    const uint16_t *vbase = a.v_cache + base;
    const int rounds = (T + NSLOT - 1) / NSLOT;

    // wait: Q heads, K head and V head of this step are complete (python_vm.py:281-290)
    const int per_head = D / 16;
    const bool ok = wait_dependency(c, [&]() {
        const int *p = nullptr;
        if (c.lane < G) p = bar_ptr(c, layer, 0, h0 + c.lane);
        else if (c.lane == G) p = bar_ptr(c, layer, 0, H + kvh);
        else if (c.lane == G + 1) p = bar_ptr(c, layer, 0, H + KVH + kvh);
        return poll_wave0(c, p, false, per_head);
    });
    if (!ok) return false;

    // token row loads: rows older than this step are immutable, the row at pos_id was written by
    // another CU a moment ago and needs a coherent load
    auto load_kv = [&](const uint16_t *kvb, int r) {
        const int t = t0 + r;
        const uint16_t *p = kvb + (size_t)t * tok_stride;
        return t == a.pos_id ? ld_b128(p) : ld_const_b128(p);
    };

    float q[G][8];
#pragma unroll
    for (int h = 0; h < G; h++) {
        float tmp[8];
        unpack8(ld_b128(a.q_post_rope + (size_t)(h0 + h) * D + sub * 8), tmp);
#pragma unroll
        for (int e = 0; e < 8; e++) q[h][e] = tmp[e];
    }

    // ---- pass 1: scores and maximum ----
    float mx[G];
#pragma unroll
    for (int h = 0; h < G; h++) mx[h] = -INFINITY;
    for (int rd = 0; rd < rounds; rd++) {
        const int r = rd * NSLOT + slot;
        if (r < T) {
            float kf[8];
            unpack8(load_kv(kbase, r), kf);
#pragma unroll
            for (int h = 0; h < G; h++) {
                float acc = 0.0f;
#pragma unroll
                for (int e = 0; e < 8; e++) acc = fmaf(q[h][e], kf[e], acc);
                // the LPT lanes of a token share r, so they are active together
                const float s = lane_tree_sum<1, LPT>(acc) * a.attn_scale;
                if (sub == 0) sm->scores[h][r] = s;
                mx[h] = fmaxf(mx[h], s);
            }
        }
    }
#pragma unroll
    for (int h = 0; h < G; h++) {
        const float m = lane_tree_max<LPT, 64>(mx[h]);
        if (c.lane == 0) sm->wave_max[c.wave][h] = m;
    }
    __syncthreads();
    if (c.tid < G) {
        float m = sm->wave_max[0][c.tid];
        for (int w = 1; w < kWaves; w++) m = fmaxf(m, sm->wave_max[w][c.tid]);
        sm->head_m[c.tid] = m;
    }
    __syncthreads();
    // p = exp(s - max), once per (head, token), in place
    for (int i = c.tid; i < G * T; i += kThreads) {
        const int h = i / T, r = i - h * T;
        sm->scores[h][r] = mkm::expf_exact(sm->scores[h][r] - sm->head_m[h]);
    }
    __syncthreads();

    // ---- pass 2: slot sums ----
    float acc[G][8], lsum[G];
#pragma unroll
    for (int h = 0; h < G; h++) {
        lsum[h] = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; e++) acc[h][e] = 0.0f;
    }
    for (int rd = 0; rd < rounds; rd++) {
        const int r = rd * NSLOT + slot;
        if (r < T) {
            float vf[8];
            unpack8(load_kv(vbase, r), vf);
#pragma unroll
            for (int h = 0; h < G; h++) {
                const float p = sm->scores[h][r];
                lsum[h] = lsum[h] + p;
#pragma unroll
                for (int e = 0; e < 8; e++) acc[h][e] = fmaf(p, vf[e], acc[h][e]);
            }
        }
    }
    // combine the TPW slots of this wave (pairwise tree over lane groups), then park per wave
#pragma unroll
    for (int h = 0; h < G; h++) {
        lsum[h] = lane_tree_sum<LPT, 64>(lsum[h]);
#pragma unroll
        for (int e = 0; e < 8; e++) acc[h][e] = lane_tree_sum<LPT, 64>(acc[h][e]);
    }
    if (c.lane < LPT) {
#pragma unroll
        for (int h = 0; h < G; h++) {
#pragma unroll
            for (int e = 0; e < 8; e++) sm->wave_o[c.wave][h][sub * 8 + e] = acc[h][e];
            if (c.lane == 0) sm->wave_l[c.wave][h] = lsum[h];
        }
    }
    __syncthreads();

    // ---- combine the 16 waves pairwise, normalise, store ----
    // thread -> (head, adjacent dim pair)
    if (c.tid < G * D / 2) {
        const int h = c.tid / (D / 2), d = (c.tid % (D / 2)) * 2;
        float o0[kWaves], o1[kWaves], l[kWaves];
#pragma unroll
        for (int w = 0; w < kWaves; w++) {
            o0[w] = sm->wave_o[w][h][d];
            o1[w] = sm->wave_o[w][h][d + 1];
            l[w] = sm->wave_l[w][h];
        }
#pragma unroll
        for (int s = 1; s < kWaves; s <<= 1)
#pragma unroll
            for (int i = 0; i < kWaves; i += 2 * s) {
                o0[i] = o0[i] + o0[i + s];
                o1[i] = o1[i] + o1[i + s];
                l[i] = l[i] + l[i + s];
            }
        const int head = h0 + h;
        float r0, r1, lse;
        if (T == 0) {  // softmax over nothing
            r0 = r1 = 0.0f;
            lse = -INFINITY;
        } else {
            r0 = o0[0] / l[0];
            r1 = o1[0] / l[0];
            lse = (sm->head_m[h] * 1.44269504088896341f) + mkm::log2f_exact(l[0]);
        }
        if (skip) {
            st_u32(a.attn_out + (size_t)head * D + d, mkm::pack_bf16(r0, r1));
        } else {
            float *dst = a.attn_out_intermediates + ((size_t)head * a.max_partials + pidx) * D + d;
            st_f32(dst, r0);
            st_f32(dst + 1, r1);
            if (d == 0) st_f32(a.attn_lse_intermediates + (size_t)head * a.max_partials + pidx, lse);
        }
    }
    __syncthreads();
    if (skip) {
        if (c.tid == 0) signal_sharded(c, layer, 2, G);
    } else {
        if (c.tid < G) add_i32(bar_ptr(c, layer, 1, h0 + c.tid), 1);
    }
    return true;
}

// ---------------------------------------------------------------------------------------------
// opcode 3: log-sum-exp merge of attention partitions  (python_vm.py:349-393;
// reference device op: demos/low-latency-llama/attention_reduction.cu:18-339)
// ---------------------------------------------------------------------------------------------
__device__ bool op_attention_reduction(const Ctx &c, const int *ins) {
    const mk_llama_args &a = c.a;
    Smem *sm = c.sm;
    const int layer = ins[1], hs = ins[2], P = ins[3], terminal = ins[4], n = ins[5];
    const int D = a.head_dim, R = a.attn_reduction_size, MP = a.max_partials;
    bool bad = layer < 0 || layer >= a.num_layers || n < 1 || n > MK_INSTRUCTION_WORDS - 7 || hs < 0 ||
               hs + R > a.num_attention_heads || R > kGqaMax;
    if (!bad)
        for (int i = 0; i < n; i++) bad |= ins[6 + i] < 0 || ins[6 + i] >= MP;
    const int out_idx = bad ? 0 : ins[6 + n];
    bad |= !terminal && (out_idx < 0 || out_idx >= MP);
    if (bad) return bail(c, MK_STATUS_BAD_INSTRUCTION);
    const bool ok = wait_dependency(c, [&]() {
        const int *p = c.lane < R ? bar_ptr(c, layer, 1, hs + c.lane) : nullptr;
        return poll_wave0(c, p, false, P);
    });
    if (!ok) return false;

    // weights 2^(lse_i - max) once per (head, list entry)
    if (c.tid < R) {
        const float *lses = a.attn_lse_intermediates + (size_t)(hs + c.tid) * MP;
        float m = -INFINITY;
        for (int i = 0; i < n; i++) m = fmaxf(m, ld_f32(lses + ins[6 + i]));
        sm->head_m[c.tid] = m;
        for (int i = 0; i < n; i++) sm->head_w[c.tid][i] = mkm::exp2f_exact(ld_f32(lses + ins[6 + i]) - m);
    }
    __syncthreads();
    if (c.tid < R * D / 2) {
        const int h = c.tid / (D / 2), d = (c.tid % (D / 2)) * 2;
        const int head = hs + h;
        const float *outs = a.attn_out_intermediates + (size_t)head * MP * D;
        float den = 0.0f, o0 = 0.0f, o1 = 0.0f;
        for (int i = 0; i < n; i++) {
            const float w = sm->head_w[h][i];
            const uint64_t v = ld_u64(outs + (size_t)ins[6 + i] * D + d);
            den = den + w;
            o0 = fmaf(w, mkm::bits_f32((uint32_t)v), o0);
            o1 = fmaf(w, mkm::bits_f32((uint32_t)(v >> 32)), o1);
        }
        o0 = o0 / den;
        o1 = o1 / den;
        if (terminal) {
            st_u32(a.attn_out + (size_t)head * D + d, mkm::pack_bf16(o0, o1));
        } else {
            float *dst = a.attn_out_intermediates + ((size_t)head * MP + out_idx) * D + d;
            st_f32(dst, o0);
            st_f32(dst + 1, o1);
            if (d == 0)
                st_f32(a.attn_lse_intermediates + (size_t)head * MP + out_idx, sm->head_m[h] + mkm::log2f_exact(den));
        }
    }
    __syncthreads();
    if (c.tid == 0) signal_sharded(c, layer, 2, R);
    return true;
}

// ---------------------------------------------------------------------------------------------
// the persistent kernel
// ---------------------------------------------------------------------------------------------
template <int KC_HID, int KC_RED, int D>
__global__ __launch_bounds__(kThreads) void mk_llama_kernel(const mk_llama_args a) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    Smem *sm = reinterpret_cast<Smem *>(smem_raw);
    const WsLayout wl = ws_layout(a.num_layers, a.hidden_size, a.intermediate_size, a.matvec_reduction_size);
    int *ws = static_cast<int *>(a.workspace);
    Ctx c{a,
          sm,
          ws + wl.status,
          ws + wl.shards,
          ws + wl.arrive_o,
          ws + wl.arrive_d,
          reinterpret_cast<float *>(ws + wl.partial),
          (int)threadIdx.x,
          (int)threadIdx.x / 64,
          (int)threadIdx.x % 64,
          (int)blockIdx.x,
          0,
          0,
          (long long)(a.spin_limit_us ? a.spin_limit_us : 2000000u) * 100,
          a.num_attention_heads + 2 * a.num_kv_heads};
    if (c.tid == 0) {
        sm->abort = 0;
        sm->last_flag = 0;
    }
    __syncthreads();

    const int *queue = a.instructions + (size_t)c.worker * a.num_slots * MK_INSTRUCTION_WORDS;
    for (int slot = 0; slot < a.num_slots; slot++) {
        const int *ins = queue + (size_t)slot * MK_INSTRUCTION_WORDS;
        const int opcode = ins[0];
        c.slot = slot;
        c.opcode = opcode;
        bool ok = true;
        switch (opcode) {
        case 0: break;  // NoOp pads the queues (megakernels/scheduler.py:287-289)
        case 1: ok = op_qkv<KC_HID>(c, ins); break;
        case 2: ok = op_attention<D>(c, ins); break;
        case 3: ok = op_attention_reduction(c, ins); break;
        case 4: ok = op_matvec_add<KC_RED>(c, ins, false); break;
        case 5: ok = op_upgate<KC_HID>(c, ins); break;
        case 6: ok = op_matvec_add<KC_RED>(c, ins, true); break;
        case 7: ok = op_lm_head<KC_HID>(c, ins); break;
        default: ok = bail(c, MK_STATUS_BAD_OPCODE);  // reference: trap, include/util.cuh:38
        }
        if (!ok) break;
    }

    // The last workgroup to get here folds the sharded counters into `barriers` and leaves the
    // shards zeroed for the next launch.
    __syncthreads();  // this workgroup's atomics and stores are complete
    if (c.tid == 0) {
        const int done = __hip_atomic_fetch_add(&c.status[kDoneSlot], 1, __ATOMIC_RELAXED, AG);
        sm->last_flag = done == (int)gridDim.x - 1;
    }
    __syncthreads();
    if (sm->last_flag) {
        const int counters = a.num_layers * kHotRows;
        for (int i = c.tid; i < counters; i += kThreads) {
            int total = 0;
            for (int s = 0; s < kShards; s++) {
                int *p = c.shards + (size_t)s * counters + i;
                const int v = ld_i32(p);
                if (v) {
                    total += v;
                    st_i32(p, 0);
                }
            }
            if (total) add_i32(bar_ptr(c, i / kHotRows, 2 + i % kHotRows, 0), total);
        }
        if (c.tid == 0) st_i32(&c.status[kDoneSlot], 0);
    }
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

KernelFn pick_kernel(int hid, int R, int D) {
    if (hid == 2048 && R == 2048 && D == 64) return mk_llama_kernel<4, 4, 64>;
    if (hid == 4096 && R == 2048 && D == 128) return mk_llama_kernel<8, 4, 128>;
    if (hid == 512 && R == 512 && D == 64) return mk_llama_kernel<1, 1, 64>;
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

int mk_llama_launch(const mk_llama_args *args, void *hip_stream) {
    g_error[0] = 0;
    if (!args) return fail(-1, "null arguments");
    const mk_llama_args &a = *args;
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
    if (a.num_attention_heads != a.num_kv_heads * kGqaMax)
        return fail(-3, "unsupported head grouping: %d query heads for %d KV heads (need %d per KV head)",
                    a.num_attention_heads, a.num_kv_heads, kGqaMax);
    if (a.num_attention_heads * D != hid) return fail(-3, "num_attention_heads * head_dim must equal hidden_size");
    if (a.attn_reduction_size != kGqaMax) return fail(-3, "attn_reduction_size must be %d", kGqaMax);
    if (R <= 0 || hid % R || a.intermediate_size % R) return fail(-3, "sizes are not multiples of the reduction width");
    if (a.vocab_size % 16 || a.intermediate_size % 16) return fail(-3, "vocab and intermediate sizes must be multiples of 16");
    if (a.pos_id < 0 || a.pos_id >= a.kv_max_len || a.pos_id >= a.rope_positions)
        return fail(-4, "pos_id %d outside the KV cache (%d) or rope table (%d)", a.pos_id, a.kv_max_len,
                    a.rope_positions);
    if (a.max_partials < 1) return fail(-3, "max_partials must be positive");
    KernelFn fn = pick_kernel(hid, R, D);
    if (!fn) return fail(-5, "no kernel instance for hidden %d, reduction width %d, head_dim %d", hid, R, D);
    const uint64_t need = mk_llama_workspace_bytes(a.num_layers, hid, a.intermediate_size, R);
    if (a.workspace_bytes < need)
        return fail(-6, "workspace has %llu bytes, %llu needed", (unsigned long long)a.workspace_bytes,
                    (unsigned long long)need);

    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
        return fail(-7, "cannot query the device");
    // all workers must be resident at once or the barrier waits can never be satisfied
    if (a.num_workers > cus)
        return fail(-7, "schedule has %d workers but the device has %d compute units", a.num_workers, cus);

    static thread_local KernelFn configured[8] = {};
    bool seen = false;
    for (KernelFn f : configured) seen |= f == fn;
    if (!seen) {
        hipError_t e = hipFuncSetAttribute((const void *)fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)sizeof(Smem));
        if (e != hipSuccess) return fail(-8, "hipFuncSetAttribute: %s", hipGetErrorString(e));
        for (KernelFn &f : configured)
            if (!f) {
                f = fn;
                break;
            }
    }
    hipLaunchKernelGGL(fn, dim3(a.num_workers), dim3(kThreads), sizeof(Smem), (hipStream_t)hip_stream, a);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(-9, "kernel launch: %s", hipGetErrorString(e));
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
