/*
 * TEST INFRASTRUCTURE - CPU checker for the batch-1 decode instruction VM.
 * Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may
 * load this; the shipped package never does.
 *
 * A restatement in plain C of the reference's Python VM for the low-latency
 * instruction set: megakernels/demos/latency/python_vm.py (solvers, :83-404)
 * driven over a linear instruction list as megakernels/python_vm.py:83-87 does.
 * Each solver below cites the lines it follows.  Like the reference VM it is
 * also a dependency checker: before running, every solver asserts that the
 * barrier counter of its predecessor holds EXACTLY the expected value, so an
 * instruction order that is not a valid topological order fails.
 *
 * What the reference leaves open and this file pins down
 * ------------------------------------------------------
 * The reference does its arithmetic with torch CPU kernels whose fp32
 * summation order inside a dot product / softmax is a property of the torch
 * build, not of the algorithm.  This checker fixes one order (below) so that a
 * GPU implementation can be compared BIT FOR BIT; the rounding points (where a
 * value is narrowed to bfloat16) are exactly the reference's:
 *
 *   rms_norm      fp32 statistics; normalised value -> bf16; times weight -> bf16   (:50-56)
 *   matvec        fp32 accumulate -> bf16                                          (:29-47)
 *   rope          products and sum in fp32, unfused, -> bf16 on store              (:211-230, llama.py:148-174)
 *   silu*up       silu(gate) -> bf16, product -> bf16                              (:161-163)
 *   residual add  bf16 + bf16 -> bf16, partial sums applied in instruction order   (:59-80)
 *   attention     fp32 throughout; bf16 only when written to attn_out              (:316-330)
 *
 * Canonical summation order ("column order"):
 *   matvec dot product over K elements (K a multiple of 512), both operands bf16:
 *   256 accumulators; accumulator c takes the element pairs j*256 + c (elements
 *   2(j*256 + c) and the next; j = 0..K/512-1) in order of j, each step being the
 *   two-element dot product acc + w0*x0 + w1*x1 of exact_math.h (orc_dot2_bf16:
 *   the arithmetic of the GPU's instruction for it, not a chain of IEEE
 *   operations), starting from 0; the 256 sums are then added (IEEE fp32)
 *   pairwise as a balanced binary tree in index order ((0+1)+(2+3))+... .
 *   The sum of squares of the RMS norm: 512 column accumulators, column c
 *   accumulates elements j*512 + c in order of j with fused multiply-add, same tree.
 *   A head-dimension dot product (query . key, both bf16) uses D/8 lanes; lane l
 *   accumulates its element pairs (l*8, l*8+1) .. (l*8+6, l*8+7) in order with the
 *   two-element dot product and the lanes are added as a balanced binary tree.
 *   Attention over a token range: relative token r goes to slot r mod NSLOT
 *   (NSLOT = 4096/D); each slot accumulates its tokens in increasing order
 *   (fused multiply-add for p*v, plain add for the denominator); the slots
 *   are combined by the same pairwise tree.  The softmax maximum is exact in
 *   any order.  exp / exp2 / log2 are the polynomial kernels of exact_math.h.
 *
 * Deviations from the reference VM that change rounding only (stated so the
 * tolerance tests against a torch restatement make sense): the attention
 * output is (sum p v)/(sum p) rather than sum (p / sum p) v; the log-sum-exp is
 * log2(sum exp(s - max)) + max*log2(e) rather than log2(sum exp(s)) (:323).
 * The non-terminal reduction writes max + log2(denominator); the reference's
 * natural log without the maximum (:382) is inconsistent with its own base-2
 * convention and is never scheduled.
 *
 * Parity pins (see tests/): fp64 brute force of every solver on small inputs,
 * a plain Llama decode step, split-KV invariance, closed-form barrier state,
 * the torch restatement in oracle/pyvm_torch.py within bf16 tolerance.
 */
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>

#include "exact_math.h"
#include "mk_oracle.h"

#ifdef _OPENMP
#include <omp.h>
#endif

static char g_error[512];

const char *mk_oracle_last_error(void) { return g_error; }

static int fail(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof g_error, fmt, ap);
    va_end(ap);
    return -1;
}

int mk_oracle_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ---------------------------------------------------------------------- */
/* canonical reductions                                                    */
/* ---------------------------------------------------------------------- */

static float tree_sum(float *v, int n) { /* n a power of two; destroys v */
    for (int s = 1; s < n; s *= 2)
        for (int i = 0; i < n; i += 2 * s) v[i] = v[i] + v[i + s];
    return v[0];
}

/* dot(w[0..K), x[0..K)), w bf16, x fp32 holding bf16 values (every matvec input of the VM is a
 * bf16 tensor), column order */
static float dot_lanes(const uint16_t *w, const float *x, int K) {
    float acc[256];
    for (int c = 0; c < 256; c++) acc[c] = 0.0f;
    for (int j = 0; j < K; j += 512)
        for (int c = 0; c < 256; c++) {
            const int i = j + 2 * c;
            const uint32_t wp = (uint32_t)w[i] | ((uint32_t)w[i + 1] << 16);
            const uint32_t xp = (orc_f32_bits(x[i]) >> 16) | (orc_f32_bits(x[i + 1]) & 0xffff0000u);
            acc[c] = orc_dot2_bf16(wp, xp, acc[c]);
        }
    return tree_sum(acc, 256);
}

/* python_vm.py:50-56.  out[i] = float(bf16(w[i] * bf16(x[i] * rsqrt(mean(x^2) + eps)))) */
static void rms_norm(const uint16_t *x, const uint16_t *w, float eps, int n, float *out) {
    float acc[512];
    for (int c = 0; c < 512; c++) acc[c] = 0.0f;
    for (int j = 0; j < n; j += 512)
        for (int c = 0; c < 512; c++) {
            float v = orc_bf16_to_f32(x[j + c]);
            acc[c] = fmaf(v, v, acc[c]);
        }
    float mean = tree_sum(acc, 512) / (float)n;
    float inv = 1.0f / sqrtf(mean + eps);
    for (int i = 0; i < n; i++) {
        float normed = orc_round_bf16(orc_bf16_to_f32(x[i]) * inv);
        out[i] = orc_round_bf16(orc_bf16_to_f32(w[i]) * normed);
    }
}

/* ---------------------------------------------------------------------- */
/* helpers                                                                  */
/* ---------------------------------------------------------------------- */

#define BAR(g, layer, row, col) \
    ((g)->barriers[((size_t)(layer) * 10 + (row)) * ((g)->num_attention_heads + 2 * (g)->num_kv_heads) + (col)])

static int expect_barrier(const mk_oracle_globals *g, int layer, int row, int col, int want,
                          const char *who) {
    if (!g->check_barriers) return 0;
    int have = BAR(g, layer, row, col);
    if (have != want)
        return fail("%s: barriers[%d,%d,%d] is %d, expected %d", who, layer, row, col, have, want);
    return 0;
}

static int down_total_jobs(const mk_oracle_globals *g) {
    return (g->intermediate_size / g->matvec_reduction_size) * (g->hidden_size / 16);
}
static int o_total_jobs(const mk_oracle_globals *g) {
    return (g->hidden_size / g->matvec_reduction_size) * (g->hidden_size / 16);
}

/* ---------------------------------------------------------------------- */
/* solvers                                                                  */
/* ---------------------------------------------------------------------- */

/* opcode 1, python_vm.py:168-248 */
static int op_qkv_rope_append(mk_oracle_globals *g, const int32_t *w) {
    const int layer = w[1], start = w[2], end = w[3];
    const int H = g->num_attention_heads, KVH = g->num_kv_heads, D = g->head_dim, hid = g->hidden_size;
    if (layer > 0 && expect_barrier(g, layer - 1, 5, 0, down_total_jobs(g), "qkv")) return -1;
    if (end > (H + 2 * KVH) * D / 16 || start < 0) return fail("qkv: block range out of bounds");
    if (g->pos_id < 0 || g->pos_id >= g->kv_max_len) return fail("qkv: pos_id %d outside the cache", g->pos_id);

    float *xhat = (float *)malloc(sizeof(float) * hid);
    rms_norm(g->hidden_states, g->attn_ln_weights + (size_t)layer * hid, g->rms_norm_eps, hid, xhat);

    const int k_start = H * D, v_start = k_start + KVH * D;
    const int pos = g->pos_id;
    const float *cosr = g->rope_cos + (size_t)pos * D, *sinr = g->rope_sin + (size_t)pos * D;
    const size_t kv_row = ((size_t)layer * g->kv_max_len + pos) * KVH * D; /* batch 1 */
    const uint16_t *W = g->qkv_proj_weights + (size_t)layer * (H + 2 * KVH) * D * hid;

    for (int b = start; b < end; b++) {
        float y[16];
#pragma omp parallel for
        for (int r = 0; r < 16; r++)
            y[r] = orc_round_bf16(dot_lanes(W + (size_t)(b * 16 + r) * hid, xhat, hid));
        const int row0 = b * 16;
        uint16_t out[16];
        if (row0 < v_start) { /* q or k: rotate adjacent pairs (llama.py:136-174) */
            const int d0 = row0 % D;
            for (int r = 0; r < 16; r += 2) {
                float a = y[r], c = y[r + 1];
                float even = (a * cosr[d0 + r]) + ((-c) * sinr[d0 + r]);
                float odd = (c * cosr[d0 + r + 1]) + (a * sinr[d0 + r + 1]);
                out[r] = orc_f32_to_bf16(even);
                out[r + 1] = orc_f32_to_bf16(odd);
            }
        } else {
            for (int r = 0; r < 16; r++) out[r] = orc_f32_to_bf16(y[r]);
        }
        uint16_t *dst;
        if (row0 < k_start) dst = g->post_ln_rope_q + row0;
        else if (row0 < v_start) dst = g->k_cache + kv_row + (row0 - k_start);
        else dst = g->v_cache + kv_row + (row0 - v_start);
        memcpy(dst, out, sizeof out);
        BAR(g, layer, 0, b / (D / 16)) += 1;
    }
    free(xhat);
    return 0;
}

/* opcode 2, python_vm.py:277-346 */
static int op_partial_attention(mk_oracle_globals *g, const int32_t *w) {
    const int layer = w[1], kvh = w[2], P = w[3], pidx = w[4];
    const int H = g->num_attention_heads, KVH = g->num_kv_heads, D = g->head_dim;
    const int G = H / KVH, per_head = D / 16;
    for (int i = 0; i < G; i++)
        if (expect_barrier(g, layer, 0, kvh * G + i, per_head, "attention(q)")) return -1;
    if (expect_barrier(g, layer, 0, H + kvh, per_head, "attention(k)")) return -1;
    if (expect_barrier(g, layer, 0, H + KVH + kvh, per_head, "attention(v)")) return -1;
    if (P < 1 || pidx < 0 || pidx >= P) return fail("attention: bad partition %d of %d", pidx, P);
    if (g->pos_id < 0 || g->pos_id >= g->kv_max_len) return fail("attention: pos_id %d outside the cache", g->pos_id);
    if (!g->skip_attn_reduction && pidx >= g->max_partials)
        return fail("attention: partition %d beyond the %d intermediate slots", pidx, g->max_partials);

    const int seq_len = g->pos_id + 1;
    const int total_blocks = (seq_len + 15) / 16;
    const int bpp = (total_blocks + P - 1) / P;
    const int sb = pidx * bpp;
    int eb = sb + bpp; if (eb > total_blocks) eb = total_blocks;
    const int t0 = sb * 16;
    int t1 = eb * 16; if (t1 > seq_len) t1 = seq_len;
    const int T = t1 > t0 ? t1 - t0 : 0;

    const int LPT = D / 8;            /* lanes per token */
    const int NSLOT = 8 * (64 / LPT);
    const size_t tok_stride = (size_t)KVH * D;
    const uint16_t *kbase = g->k_cache + ((size_t)layer * g->kv_max_len) * tok_stride + (size_t)kvh * D;
    const uint16_t *vbase = g->v_cache + ((size_t)layer * g->kv_max_len) * tok_stride + (size_t)kvh * D;
    const int h0 = kvh * G;

#pragma omp parallel for
    for (int h = 0; h < G; h++) {
        const int head = h0 + h;
        float *scores = (float *)malloc(sizeof(float) * (T > 0 ? T : 1));
        float *lslot = (float *)malloc(sizeof(float) * NSLOT);
        float *oslot = (float *)malloc(sizeof(float) * NSLOT * D);
        float *col = (float *)malloc(sizeof(float) * NSLOT);
        float out[256];
        float lse;
        if (T == 0) { /* softmax over nothing */
            for (int d = 0; d < D; d++) out[d] = 0.0f;
            lse = -INFINITY;
        } else {
            const uint16_t *qb = g->post_ln_rope_q + head * D;
            float m = -INFINITY;
            for (int r = 0; r < T; r++) {
                const uint16_t *k = kbase + (size_t)(t0 + r) * tok_stride;
                float lane[16];
                for (int i = 0; i < LPT; i++) {
                    float a = 0.0f;
                    for (int e = 0; e < 8; e += 2)
                        a = orc_dot2_bf16((uint32_t)k[i * 8 + e] | ((uint32_t)k[i * 8 + e + 1] << 16),
                                          (uint32_t)qb[i * 8 + e] | ((uint32_t)qb[i * 8 + e + 1] << 16), a);
                    lane[i] = a;
                }
                float s = tree_sum(lane, LPT) * g->attn_scale;
                scores[r] = s;
                if (s > m) m = s;
            }
            for (int s = 0; s < NSLOT; s++) lslot[s] = 0.0f;
            for (int i = 0; i < NSLOT * D; i++) oslot[i] = 0.0f;
            for (int r = 0; r < T; r++) {
                const int slot = r % NSLOT;
                const float p = orc_expf(scores[r] - m);
                const uint16_t *v = vbase + (size_t)(t0 + r) * tok_stride;
                lslot[slot] = lslot[slot] + p;
                float *o = oslot + (size_t)slot * D;
                for (int d = 0; d < D; d++) o[d] = fmaf(p, orc_bf16_to_f32(v[d]), o[d]);
            }
            const float l = tree_sum(lslot, NSLOT);
            for (int d = 0; d < D; d++) {
                for (int s = 0; s < NSLOT; s++) col[s] = oslot[(size_t)s * D + d];
                out[d] = tree_sum(col, NSLOT) / l;
            }
            lse = (m * 1.44269504088896341f) + orc_log2f(l);
        }
        if (g->skip_attn_reduction) {
            for (int d = 0; d < D; d++) g->attn_out[head * D + d] = orc_f32_to_bf16(out[d]);
        } else {
            g->attn_lse_intermediates[(size_t)head * g->max_partials + pidx] = lse;
            memcpy(g->attn_out_intermediates + ((size_t)head * g->max_partials + pidx) * D, out,
                   sizeof(float) * D);
        }
        free(scores); free(lslot); free(oslot); free(col);
    }

    if (g->skip_attn_reduction) BAR(g, layer, 2, 0) += G;
    else for (int h = 0; h < G; h++) BAR(g, layer, 1, h0 + h) += 1;
    return 0;
}

/* opcode 3, python_vm.py:349-393 */
static int op_attention_reduction(mk_oracle_globals *g, const int32_t *w) {
    const int layer = w[1], hs = w[2], P = w[3], terminal = w[4], n = w[5];
    const int32_t *list = w + 6;
    const int out_idx = w[6 + n];
    const int D = g->head_dim, R = g->attn_reduction_size;
    /* python_vm.py:354 asserts == num_partials.  In a reduction tree (which the reference never
     * schedules) the counter also counts the finished merges below this one, in whatever order they
     * ran, so the check is "at least". */
    if (g->check_barriers && BAR(g, layer, 1, hs) < P)
        return fail("attention reduction: barriers[%d,1,%d] is %d, expected at least %d", layer, hs, BAR(g, layer, 1, hs), P);
    if (n < 1 || 7 + n > 32) return fail("attention reduction: list of %d entries", n);
    for (int i = 0; i < n; i++)
        if (list[i] < 0 || list[i] >= g->max_partials) return fail("attention reduction: slot %d", list[i]);

    for (int h = hs; h < hs + R; h++) {
        const float *lses = g->attn_lse_intermediates + (size_t)h * g->max_partials;
        const float *outs = g->attn_out_intermediates + (size_t)h * g->max_partials * D;
        float M = -INFINITY;
        for (int i = 0; i < n; i++) if (lses[list[i]] > M) M = lses[list[i]];
        float den = 0.0f, acc[256];
        for (int d = 0; d < D; d++) acc[d] = 0.0f;
        for (int i = 0; i < n; i++) {
            const float wt = orc_exp2f(lses[list[i]] - M);
            den = den + wt;
            const float *o = outs + (size_t)list[i] * D;
            for (int d = 0; d < D; d++) acc[d] = fmaf(wt, o[d], acc[d]);
        }
        /* every listed partition empty (lse -inf: a run past the end of the sequence in a reduction
         * tree): the formula gives NaN (-inf - -inf); the merge of nothing is defined as nothing, like
         * an empty partition itself: zeros and -inf */
        const int nothing = M == -INFINITY;
        if (terminal) {
            for (int d = 0; d < D; d++) g->attn_out[h * D + d] = orc_f32_to_bf16(nothing ? 0.0f : acc[d] / den);
        } else {
            float *dst = g->attn_out_intermediates + ((size_t)h * g->max_partials + out_idx) * D;
            for (int d = 0; d < D; d++) dst[d] = nothing ? 0.0f : acc[d] / den;
            g->attn_lse_intermediates[(size_t)h * g->max_partials + out_idx] = nothing ? -INFINITY : M + orc_log2f(den);
        }
    }
    /* python_vm.py:391-392 adds to row 2 after every reduction, terminal or not ("the dumb way"),
     * which would open the O projection's barrier before a tree is done.  Here a non-terminal merge
     * is one more arrival among its heads' partial results (row 1), and only the terminal merge
     * completes the heads for the O projection. */
    if (terminal) BAR(g, layer, 2, 0) += R;
    else
        for (int h = hs; h < hs + R; h++) BAR(g, layer, 1, h) += 1;
    return 0;
}

/* residual[rows] += bf16(W[rows, group] . vec[group]); python_vm.py:59-80 */
static void matvec_residual(const uint16_t *W, size_t row_stride, const uint16_t *vec, uint16_t *residual,
                            int start_block, int end_block, int R, int group) {
    float *x = (float *)malloc(sizeof(float) * R);
    for (int i = 0; i < R; i++) x[i] = orc_bf16_to_f32(vec[(size_t)group * R + i]);
    const int rows = (end_block - start_block) * 16;
#pragma omp parallel for
    for (int i = 0; i < rows; i++) {
        const int row = start_block * 16 + i;
        float part = orc_round_bf16(dot_lanes(W + (size_t)row * row_stride + (size_t)group * R, x, R));
        residual[row] = orc_f32_to_bf16(orc_bf16_to_f32(residual[row]) + part);
    }
    free(x);
}

/* opcode 4, python_vm.py:83-104.  The reference asserts a single block and
 * column group 0; several groups are allowed here for hidden sizes above the
 * reduction width. */
static int op_o_proj(mk_oracle_globals *g, const int32_t *w) {
    const int layer = w[1], start = w[2], end = w[3], group = w[4];
    const int hid = g->hidden_size, R = g->matvec_reduction_size;
    if (expect_barrier(g, layer, 2, 0, g->num_attention_heads, "o_proj")) return -1;
    if (start < 0 || end > hid / 16 || group < 0 || group >= hid / R) return fail("o_proj: bad range");
    matvec_residual(g->o_proj_weights + (size_t)layer * hid * hid, hid, g->attn_out, g->hidden_states,
                    start, end, R, group);
    BAR(g, layer, 3, 0) += end - start;
    return 0;
}

/* opcode 6, python_vm.py:107-124 */
static int op_down_proj(mk_oracle_globals *g, const int32_t *w) {
    const int layer = w[1], start = w[2], end = w[3], group = w[4];
    const int hid = g->hidden_size, inter = g->intermediate_size, R = g->matvec_reduction_size;
    if (expect_barrier(g, layer, 4, 0, inter / 16, "down_proj")) return -1;
    if (start < 0 || end > hid / 16 || group < 0 || group >= inter / R) return fail("down_proj: bad range");
    matvec_residual(g->down_proj_weights + (size_t)layer * hid * inter, inter, g->silu_out,
                    g->hidden_states, start, end, R, group);
    BAR(g, layer, 5, 0) += end - start;
    return 0;
}

/* opcode 5, python_vm.py:127-165 */
static int op_upgate_silu(mk_oracle_globals *g, const int32_t *w) {
    const int layer = w[1], n = w[2];
    const int32_t *blocks = w + 3;
    const int hid = g->hidden_size, inter = g->intermediate_size;
    if (expect_barrier(g, layer, 3, 0, o_total_jobs(g), "upgate")) return -1;
    if (n < 0 || 3 + n > 32) return fail("upgate: list of %d entries", n);
    for (int i = 0; i < n; i++)
        if (blocks[i] < 0 || blocks[i] >= inter / 16) return fail("upgate: block %d", blocks[i]);

    float *xhat = (float *)malloc(sizeof(float) * hid);
    rms_norm(g->hidden_states, g->mlp_ln_weights + (size_t)layer * hid, g->rms_norm_eps, hid, xhat);
    const uint16_t *Wu = g->up_proj_weights + (size_t)layer * inter * hid;
    const uint16_t *Wg = g->gate_proj_weights + (size_t)layer * inter * hid;
#pragma omp parallel for
    for (int i = 0; i < n * 16; i++) {
        const int row = blocks[i / 16] * 16 + (i % 16);
        const float up = orc_round_bf16(dot_lanes(Wu + (size_t)row * hid, xhat, hid));
        const float gate = orc_round_bf16(dot_lanes(Wg + (size_t)row * hid, xhat, hid));
        const float silu = orc_round_bf16(gate / (1.0f + orc_expf(-gate)));
        g->silu_out[row] = orc_f32_to_bf16(silu * up);
    }
    free(xhat);
    BAR(g, layer, 4, 0) += n;
    return 0;
}

/* opcode 7, python_vm.py:251-274 */
static int op_lm_head(mk_oracle_globals *g, const int32_t *w) {
    const int start = w[1], end = w[2];
    const int hid = g->hidden_size;
    if (expect_barrier(g, g->num_hidden_layers - 1, 5, 0, down_total_jobs(g), "lm_head")) return -1;
    if (start < 0 || end > g->vocab_size / 16) return fail("lm_head: bad range");
    float *xhat = (float *)malloc(sizeof(float) * hid);
    rms_norm(g->hidden_states, g->lm_head_norm_weights, g->rms_norm_eps, hid, xhat);
#pragma omp parallel for
    for (int row = start * 16; row < end * 16; row++)
        g->logits[row] = orc_f32_to_bf16(dot_lanes(g->lm_head_weights + (size_t)row * hid, xhat, hid));
    free(xhat);
    return 0;
}

/* ---------------------------------------------------------------------- */
/* interpreter: megakernels/python_vm.py:83-87                              */
/* ---------------------------------------------------------------------- */

int mk_oracle_run(mk_oracle_globals *g, const int32_t *instructions, int count) {
    g_error[0] = 0;
    if (g->hidden_size % 512 || g->matvec_reduction_size % 512 || g->head_dim % 16 ||
        g->head_dim > 256 || g->hidden_size % g->matvec_reduction_size ||
        g->intermediate_size % g->matvec_reduction_size)
        return fail("unsupported shape");
    for (int i = 0; i < count; i++) {
        const int32_t *w = instructions + (size_t)i * 32;
        int rc;
        switch (w[0]) {
        case 0: rc = 0; break;
        case 1: rc = op_qkv_rope_append(g, w); break;
        case 2: rc = op_partial_attention(g, w); break;
        case 3: rc = op_attention_reduction(g, w); break;
        case 4: rc = op_o_proj(g, w); break;
        case 5: rc = op_upgate_silu(g, w); break;
        case 6: rc = op_down_proj(g, w); break;
        case 7: rc = op_lm_head(g, w); break;
        default: rc = fail("instruction %d: unknown opcode %d", i, w[0]);
        }
        if (rc) {
            char head[64];
            snprintf(head, sizeof head, " (instruction %d)", i);
            strncat(g_error, head, sizeof g_error - strlen(g_error) - 1);
            return rc;
        }
    }
    return 0;
}

/* first index of the maximum of a bf16 vector: torch.argmax semantics used by
 * megakernels/generators.py:140-141 */
int mk_oracle_argmax_bf16(const uint16_t *v, int n) {
    int best = 0;
    float bv = orc_bf16_to_f32(v[0]);
    for (int i = 1; i < n; i++) {
        float x = orc_bf16_to_f32(v[i]);
        if (x > bv) { bv = x; best = i; }
    }
    return best;
}

/* scalar kernels exported for the math pinning tests */
float mk_oracle_expf(float x) { return orc_expf(x); }
float mk_oracle_exp2f(float x) { return orc_exp2f(x); }
float mk_oracle_log2f(float x) { return orc_log2f(x); }
uint16_t mk_oracle_f32_to_bf16(float x) { return orc_f32_to_bf16(x); }
float mk_oracle_dot(const uint16_t *w, const float *x, int K) { return dot_lanes(w, x, K); }
void mk_oracle_dot2(const uint32_t *a, const uint32_t *b, const float *acc, float *out, size_t n) {
#pragma omp parallel for
    for (size_t i = 0; i < n; i++) out[i] = orc_dot2_bf16(a[i], b[i], acc[i]);
}
void mk_oracle_dot2_general(const uint32_t *a, const uint32_t *b, const float *acc, float *out, size_t n) {
#pragma omp parallel for
    for (size_t i = 0; i < n; i++) out[i] = orc_dot2_bf16_general(a[i], b[i], acc[i]);
}
