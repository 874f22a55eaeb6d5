/*
 * C ABI of the MI355X batch-1 decode megakernel (libmk_llama.so).
 *
 * This is the drop-in boundary of the reference's `mk` path: what the
 * reference's Python calls through the pybind module `mk_llama`
 * (megakernels/demos/latency/mk.py:15-49 -> demos/low-latency-llama/llama.cu:26-52
 * -> __global__ mk<...>, include/megakernel.cuh:166-171).  One call launches one
 * persistent HIP kernel - one workgroup per compute unit, workgroup w running
 * instructions[w, 0..num_slots) in order - asynchronously on the given stream.
 *
 * Plain pointers and sizes only; the caller (PyTorch in the shipped host code)
 * owns every buffer.  All tensors are contiguous device memory.  bf16 tensors
 * are passed as uint16_t bit patterns.
 */
#ifndef MK_LLAMA_H
#define MK_LLAMA_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MK_LLAMA_ABI_VERSION 6
#define MK_INSTRUCTION_WORDS 32   /* megakernels/scheduler.py:13, include/config.cuh:14 */
#define MK_TIMING_SLOTS 128       /* megakernels/scheduler.py:14, include/config.cuh:18 */
#define MK_BARRIER_ROWS 10        /* megakernels/demos/latency/scheduler.py:53-61 */

/* args.flags: record per-instruction timings into `timings[worker, slot, :]` - the low 32 bits of
 * the device's 100 MHz wall clock (one clock for all compute units, so records of different workers
 * compare directly; subtract the smallest to get times since the first workgroup started), written
 * by the workgroup's controller wave.  Counterpart
 * of the reference's compile-time TIMING_RECORD_ENABLED (include/config.cuh:46); the word indices
 * are MK_TIMING_* below. */
#define MK_FLAG_TIMINGS 1u
/* args.flags: leave `barriers` all zero after the launch instead of holding the VM's counts, so that
 * the next launch needs no reset (the reference's loop refills the tensor before every launch,
 * megakernels/generators.py:127-128). */
#define MK_FLAG_RESET_BARRIERS 2u
/* args.flags: the caller promises that the residual projections' column-group jobs (opcodes 4 and 6
 * with hidden_size or intermediate_size a multiple of matvec_reduction_size) come in complete sets:
 * for every (opcode, layer, row block) that appears in `instructions`, the jobs of all column groups
 * appear, each exactly once.  The jobs of a set then share their work by rows instead of by columns
 * (the job of group c computes 16 / G of the block's rows over all G groups' columns and applies
 * every group's sum to the residual itself, in group order), so no partial sums travel between
 * workers and no job waits for another.  Results and barrier counts are those of executing each
 * instruction on its own, which is what happens without the flag; with the flag set on an incomplete
 * set, rows of hidden_states miss their update.  Every schedule of
 * megakernels/demos/latency/scheduler.py:167-213,346-352 qualifies.  Used when the group count
 * divides 8; other shapes run each job on its own regardless. */
#define MK_FLAG_JOINT_RESIDUAL 4u

/* Words of one instruction's timing record: the reference's event slots (include/util.cuh:215-246),
 * stamped by the wave that does the thing - the controller wave, the waves that stream weight rows
 * (or K / V rows), the wave that stores and signals - so the reference's tools read measured times.
 * Words 1-3 are instruction fetch done, page allocation done and semaphore set-up in the reference:
 * stages this kernel does not have (the queue is in LDS, there are no pages or semaphores); they
 * hold the controller's view of the stages it has instead.  All times are the low 32 bits of the
 * device-wide 100 MHz clock.  For every executed instruction
 * START <= DEPENDENCY_READY <= INPUT_READY <= COMPUTE_DONE <= END (in attention the waves that store
 * signal on their own, so OUTPUT_READY can follow END there).  Words not listed stay as the
 * caller left them. */
enum {
    MK_TIMING_START = 0,            /* TEVENT_CONTROLLER_START: the controller wave took the instruction */
    MK_TIMING_DEPENDENCY_READY = 1, /* the barrier counters it waits for reached their targets */
    MK_TIMING_INPUT_READY = 2,      /* activation vector normalised and handed to the consumer waves */
    MK_TIMING_COMPUTE_DONE = 3,     /* all rows of the instruction computed */
    MK_TIMING_END = 4,              /* TEVENT_CONTROLLER_END: results stored and signalled, the workgroup moves on */
    MK_TIMING_LOADER_START = 5,     /* TEVENT_LOADER_START: first weight (or K / V) row requested, by wave 0 */
    MK_TIMING_LAUNCHER_START = 7,   /* TEVENT_LAUNCHER_START: = INPUT_READY */
    MK_TIMING_STORER_START = 9,     /* TEVENT_STORER_START: = AT_GMEM_STORE */
    MK_TIMING_CONSUMER_START = 11,  /* TEVENT_CONSUMER_START + 2 w, + 2 w + 1: consumer wave w starts on its
                                       first row / is done with its last, w < MK_TIMING_CONSUMER_WAVES */
    MK_TIMING_AT_GMEM_WAIT = 44,    /* TEVENT_AT_GMEM_WAIT: first look at the dependency counters is on its way */
    MK_TIMING_DONE_GMEM_WAIT = 45,  /* TEVENT_DONE_GMEM_WAIT: = DEPENDENCY_READY */
    MK_TIMING_AT_GMEM_STORE = 46,   /* TEVENT_AT_GMEM_STORE: epilogue computed, result stores issued */
    MK_TIMING_DONE_GMEM_STORE = 47, /* TEVENT_DONE_GMEM_STORE: the stores are acknowledged */
    MK_TIMING_FIRST_LOAD = 48,      /* TEVENT_FIRST_LOAD: = LOADER_START */
    MK_TIMING_FIRST_USE = 49,       /* TEVENT_FIRST_USE: wave 0 starts on its first row */
    MK_TIMING_FIRST_STORE = 50,     /* TEVENT_FIRST_STORE: = AT_GMEM_STORE */
    MK_TIMING_LAST_LOAD = 51,       /* TEVENT_LAST_LOAD: wave 0 has requested its last row */
    MK_TIMING_LAST_USE = 52,        /* TEVENT_LAST_USE: wave 0 is done with its last row */
    MK_TIMING_LAST_STORE = 53,      /* TEVENT_LAST_STORE: = DONE_GMEM_STORE */
    MK_TIMING_OUTPUT_READY = 54,    /* TEVENT_OUTPUT_READY: the barrier counters are signalled */
    MK_TIMING_OPCODE = 55,          /* first free slot of the reference: the instruction's opcode, not a time */
    MK_TIMING_ATTN_MAXIMA = 56,     /* attention: scores and their maxima done */
    MK_TIMING_ATTN_PROBABILITIES = 57  /* attention: exponentials done */
};
#define MK_TIMING_CONSUMER_WAVES 8  /* consumer waves with a slot pair of their own */

/* Status codes written by the kernel into the workspace and returned by
 * mk_llama_read_status(). */
enum {
    MK_STATUS_OK = 0,
    MK_STATUS_BARRIER_TIMEOUT = 1,   /* a barrier wait exceeded spin_limit_us */
    MK_STATUS_BAD_OPCODE = 2,        /* reference: asm trap, include/util.cuh:38 */
    MK_STATUS_ATTN_TOO_LONG = 3,     /* reserved: partitions of any length run since ABI version 5 */
    MK_STATUS_BAD_INSTRUCTION = 4,   /* field out of range for the given shapes */
    MK_STATUS_BAD_TOKEN = 5          /* *token_in outside the vocabulary */
};

/* Arguments of one launch, in the positional order of the reference binding
 * (megakernels/demos/latency/mk.py:17-48), followed by the shapes the
 * reference bakes in at compile time (demos/low-latency-llama/llama.cuh:15-24,149-158). */
typedef struct mk_llama_args {
    /* VM state */
    int32_t *barriers;              /* [L, 10, H + 2 KVH]; read-modify-write */
    const int32_t *instructions;    /* [num_workers, num_slots, 32]; a worker runs its row in order, so no
                                       instruction may sit behind one that (transitively) waits for it - which,
                                       without MK_FLAG_JOINT_RESIDUAL, includes: the job of a residual projection's
                                       last column group waits for the other groups' jobs of its row blocks */
    int32_t *timings;               /* [num_workers, num_slots, 128]; may be NULL */
    /* weights */
    const uint16_t *qkv_weights;          /* [L, (H + 2 KVH) D, hidden] */
    const uint16_t *attn_norm_weights;    /* [L, hidden] */
    const uint16_t *o_weights;            /* [L, hidden, H D] */
    const uint16_t *mlp_norm_weights;     /* [L, hidden] */
    const uint16_t *up_weights;           /* [L, inter, hidden] */
    const uint16_t *gate_weights;         /* [L, inter, hidden] */
    const uint16_t *down_weights;         /* [L, hidden, inter] */
    const uint16_t *lm_head_norm_weights; /* [hidden] */
    const uint16_t *lm_head_weights;      /* [vocab, hidden] */
    uint16_t *k_cache;                    /* [L, kv_max_len, KVH, D]; row pos_id is written */
    uint16_t *v_cache;
    const float *rope_cos;                /* [rope_positions, D], rotary pairs adjacent */
    const float *rope_sin;
    /* activations */
    uint16_t *hidden_states;              /* [hidden]; in: embedding row, out: final hidden state */
    uint16_t *q_post_rope;                /* [H D] */
    uint16_t *attn_out;                   /* [H D] */
    float *attn_lse_intermediates;        /* [H, max_partials] */
    float *attn_out_intermediates;        /* [H, max_partials, D] */
    uint16_t *silu_out;                   /* [inter] */
    uint16_t *logits;                     /* [vocab] */
    /* scalars of the reference call */
    int32_t pos_id;
    float attn_scale;
    float rms_norm_eps;
    int32_t skip_attn_reduction;
    /* shapes */
    int32_t num_layers, hidden_size, intermediate_size;
    int32_t num_attention_heads, num_kv_heads, head_dim, vocab_size;
    int32_t num_workers, num_slots;       /* instruction tensor dims 0 and 1 */
    int32_t kv_max_len, max_partials, rope_positions;
    int32_t matvec_reduction_size;        /* column-group width, 2048 in the reference */
    int32_t attn_reduction_size;          /* heads per reduction instruction, 4 */
    /* runtime */
    void *workspace;                      /* mk_llama_workspace_bytes() bytes, zeroed once by the caller */
    uint64_t workspace_bytes;
    uint32_t spin_limit_us;               /* give up a barrier wait after this long; 0 = default (2 s) */
    uint32_t flags;                       /* MK_FLAG_* */
    /* Optional: the per-token glue of the reference's decode loop folded into the launch
     * (megakernels/generators.py:121-143: embedding row -> hidden_states before the launch,
     * argmax(logits) after it).  All NULL gives exactly the reference call. */
    const uint16_t *embed_table;          /* [vocab, hidden]; needed with token_in */
    const int64_t *token_in;              /* device; hidden_states starts as embed_table[*token_in] */
    int64_t *token_out;                   /* device; receives argmax(logits), first index on ties */
    /* Optional: several decode steps in one launch (no counterpart in the reference, which launches
     * once per token).  num_steps > 1 needs embed_table, token_in, token_out and
     * MK_FLAG_RESET_BARRIERS, and k_cache / v_cache aligned to 128 bytes (rows written by one step are read
     * by the next with cached loads, so no cache line may hold bytes of two rows); step s runs at position
     * pos_id + s, starts from the token of step s - 1 (*token_in for s = 0) and writes its token to
     * token_out[s], so token_out holds num_steps entries.  0 and 1 both mean one step. */
    int32_t num_steps;
    int32_t reserved0;                    /* keep zero */
} mk_llama_args;

/* Bytes of scratch device memory a launch needs for these shapes.  The caller
 * zeroes it once; the kernel leaves it usable for the next launch after every
 * successful one (counters back at zero; a count of completed decode steps and
 * tagged partial sums stay, and later launches rely on both - do not share a
 * workspace between models, and zero it again after a launch that gave up).
 * Holds sharded barrier counters, residual partial sums and the status block. */
uint64_t mk_llama_workspace_bytes(int32_t num_layers, int32_t hidden_size, int32_t intermediate_size,
                                  int32_t matvec_reduction_size);

/* Validates the arguments against what the kernel assumes, then launches on
 * `hip_stream` (a hipStream_t, NULL = default stream) without synchronising.
 * Returns 0 or a negative error; the message is available from
 * mk_llama_last_error().  Replaces the `mk_llama(...)` call of
 * megakernels/demos/latency/mk.py:15-49. */
int mk_llama_launch(const mk_llama_args *args, void *hip_stream);

/* The same launch for callers that cannot allocate device memory and have no workspace to bring:
 * code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  No
 * counterpart in the reference.  `args->workspace` and `args->workspace_bytes` are ignored; the
 * workspace is an array inside the library (2 MiB per GPU, held until the process ends), which is
 * enough for every shape the kernel has an instance for (1B: 296 KB, 8B with 32 layers: 1.04 MiB).
 * Shapes that need more are refused with -6 and a message.  The call allocates nothing: it zeroes
 * the part of the array it is going to use with a small kernel on `hip_stream`, then launches as
 * mk_llama_launch does.  `*scratch_out` (may be NULL) receives the array's device address, which is
 * what mk_llama_read_status() takes as `workspace`.  All calls on one GPU share the array: two
 * launches that overlap in time on one GPU (different streams, different threads) race. */
int mk_llama_launch_static(const mk_llama_args *args, void *hip_stream, void **scratch_out);

/* Synchronises `hip_stream` and copies the 4-word status block
 * {code, worker, slot, opcode} of the workspace to the host.  A non-zero code
 * means the launch gave up; the workspace must then be zeroed again. */
int mk_llama_read_status(void *workspace, void *hip_stream, int32_t out[4]);

/* what = 0: compute units of the current device; 1: LDS bytes the kernel
 * requests per workgroup; 2: threads per workgroup; 3: ABI version; 4: longest
 * attention partition (tokens) whose scores stay on the chip - a longer one is
 * accepted and recomputes its scores in the second pass. */
int mk_llama_query(int what);

/* Self test (no counterpart in the reference): counts the binary32 inputs, over all 2^32 bit
 * patterns except NaNs, for which the kernel's one-instruction bf16 conversion differs from the
 * portable round-to-nearest-even formula.  Synchronous, allocates 8 bytes of device memory; for
 * test suites, not for the decode path.  Must report 0. */
int mk_llama_selftest_bf16(uint64_t *mismatches_out);

/* Self test (no counterpart in the reference): out[i] = acc[i] + a[i].lo * b[i].lo + a[i].hi * b[i].hi
 * computed by the instruction the kernel's matvec dot products are built from (V_DOT2_F32_BF16;
 * a, b: 32-bit words holding two bf16, lo = bits 0-15; acc, out: binary32), over n <= 2^31 cases in
 * device memory, asynchronously on `hip_stream`.  The instruction's arithmetic is not a chain of
 * IEEE operations; test suites compare its results with the written-out definition they check the
 * kernel against.  Allocates nothing. */
int mk_llama_selftest_dot2(const void *a, const void *b, const void *acc, void *out, uint64_t n, void *hip_stream);

const char *mk_llama_last_error(void);

#ifdef __cplusplus
}
#endif
#endif
