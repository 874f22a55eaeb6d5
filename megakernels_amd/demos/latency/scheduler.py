"""Buffers and instruction DAG for batch-1 decode.

Follows reference ``megakernels/demos/latency/scheduler.py``:

* :func:`make_globals` (``:38-115``): activation buffers, barrier tensor
  ``int32 [layers, 10, H + 2 KVH]``, block sizes 16, reduction width 2048.
* :func:`schedule_qkv`, :func:`schedule_upgate`, :func:`schedule_downproj`,
  :func:`schedule_lm_head` (``:118-232``): how each operator's output blocks are
  cut into one instruction per worker.
* :func:`make_dag` / :func:`make_dag_layer` (``:235-386``): per layer, in order,
  QKV, attention, O projection, up/gate, down projection; LM head last.

Generalisations beyond the reference (which only runs Llama-3.2-1B on 132 or
148 workers with a single attention partition):

* Worker counts larger than an operator's block count are allowed.  The
  reference asserts more than one block (job) per worker for every operator
  (``:128-129,153-154,184,222-223``), which fails for 192 QKV blocks on 256
  compute units; the same rounding rules are used and some instructions simply
  cover an empty block range, which every interpreter treats as zero
  iterations.
* With ``stop_after_op`` set the LM head is not appended; the reference
  appends it whenever all layers are scheduled (``:256-263``), which leaves
  the LM head waiting on a barrier that a truncated layer never raises.
* Column groups come from ``matvec_reduction_size`` rather than
  ``intermediate_size // hidden_size`` (``:171``) and the O projection gets one
  job per (column group, block) rather than a single group (``:346-352``), so a
  4096-wide hidden state and a 14336-wide MLP are fully covered.
* ``num_attention_partitions > 1`` emits the split-KV schedule that the
  reference's interpreters define but its scheduler never produces
  (``:276-277``): per KV head ``P`` partial-attention instructions, then one
  terminal reduction per group of ``attn_reduction_size`` query heads.  More
  partitions than a reduction can list (25) go through a two-level reduction
  tree (the reference's open TODO, ``:21-35``): non-terminal merges over runs
  of partitions, then the terminal merge over their outputs.
"""

from __future__ import annotations

import math

import torch

from megakernels_amd.demos.latency.instructions import (
    AttentionReduction,
    DownProjResidual,
    Globals,
    Instruction,
    LayerNorm_QKV_MatVecRopeAppend,
    LayerNormDoubleMatVecSiLU,
    O_ProjResidual,
    PartialAttention,
    RMS_LM_Head,
)
from megakernels_amd.instructions import NoOp
from megakernels_amd.scheduler import INTS_PER_INSTRUCTION, DAG_Node, ScheduleBuilder
from megakernels_amd.utils import assert_div, get_sm_count

# A reduction instruction is [op, layer, head, P, terminal, n, list(P)..., out]:
# 7 + P words must fit the 32-word format.
MAX_ATTENTION_PARTITIONS = INTS_PER_INSTRUCTION - 7


def pick_num_attention_partitions(prompt_len: int, ntok: int, device=None, num_kv_heads: int | None = None,
                                  head_dim: int | None = None) -> int:
    """One partition per 256 cached positions, at most 24 (reference ``:21-35``) - or, when the shape of the
    KV heads is given, up to one partition per worker for every KV head (256 workers, 8 KV heads: 32).
    Beyond 25 partitions the merges go through a reduction tree, which costs a few microseconds per layer
    and pays once a partition job would otherwise stream more than 384 KB of K and V rows (8B shapes from
    about 20000 positions; the 1B shape at 16384 positions is faster with 24)."""
    min_chunk_size = 256
    length = prompt_len + ntok
    num_divisions = math.ceil(length / min_chunk_size)
    most = 24
    if num_kv_heads and head_dim:
        job_bytes = math.ceil(length / most) * head_dim * 2 * 2
        if job_bytes > 384 * 1024:
            most = max(most, get_sm_count(device if device is not None else "cuda") // num_kv_heads)
    return max(1, min(num_divisions, most))


def reduction_tree_runs(num_partitions: int) -> list[tuple[int, int]]:
    """How the partitions of a head are merged: one run ``[(0, P)]`` when a single merge can list them
    all, otherwise consecutive runs of near-equal length, one first-level merge each, as few as the
    list length allows (so the terminal merge is short)."""
    P, cap = num_partitions, MAX_ATTENTION_PARTITIONS
    if P <= cap:
        return [(0, P)]
    groups = math.ceil(P / cap)
    bounds = [round(i * P / groups) for i in range(groups + 1)]
    return [(bounds[i], bounds[i + 1]) for i in range(groups)]


def reduction_tree_groups(num_partitions: int) -> int:
    """Intermediate slots the first-level merges of a head need (0 without a tree)."""
    runs = reduction_tree_runs(num_partitions)
    return len(runs) if len(runs) > 1 else 0


def make_globals(model, skip_attn_reduction: bool = True) -> Globals:
    config = model.config
    device = model.device
    dtype = model.dtype

    def make_buffer(shape, buffer_dtype=dtype):
        return torch.zeros(shape, device=device, dtype=buffer_dtype)

    params = model.stacked_params
    max_attn_partitions = get_sm_count(device)
    heads = config.num_attention_heads
    kv_heads = config.num_key_value_heads

    return Globals(
        # parameters
        qkv_proj_weights=params.qkv_proj,
        attn_ln_weights=params.attn_ln_weight,
        o_proj_weights=params.o_proj,
        mlp_ln_weights=params.mlp_ln_weight,
        up_proj_weights=params.up_proj,
        gate_proj_weights=params.gate_proj,
        down_proj_weights=params.down_proj,
        lm_head_norm_weights=model.lm_head.input_norm.weight,
        lm_head_weights=model.lm_head.lm_head.weight,
        k_cache=model.stacked_kv_cache[0],
        v_cache=model.stacked_kv_cache[1],
        rope_cos=model.model.rope_cos,
        rope_sin=model.model.rope_sin,
        # constants
        num_hidden_layers=config.num_hidden_layers,
        num_attention_heads=heads,
        num_kv_heads=kv_heads,
        head_dim=config.head_dim,
        hidden_size=config.hidden_size,
        intermediate_size=config.intermediate_size,
        vocab_size=config.vocab_size,
        attn_scale=1 / math.sqrt(config.head_dim),
        rms_norm_eps=config.rms_norm_eps,
        device=device,
        # activations
        hidden_states=make_buffer(config.hidden_size),
        barriers=make_buffer(
            [config.num_hidden_layers, 10, heads + 2 * kv_heads], torch.int32
        ),
        pos_id=0,
        post_ln_rope_q=make_buffer(heads * config.head_dim),
        attn_out=make_buffer(heads * config.head_dim),
        attn_lse_intermediates=make_buffer([heads, max_attn_partitions], torch.float32),
        attn_out_intermediates=make_buffer(
            [heads, max_attn_partitions, config.head_dim], torch.float32
        ),
        silu_out=make_buffer(config.intermediate_size),
        logits=make_buffer(config.vocab_size),
        skip_attn_reduction=skip_attn_reduction,
        # block sizes
        up_gate_proj_block_size=16,
        down_proj_block_size=16,
        o_proj_block_size=16,
        lm_head_block_size=16,
        matvec_reduction_size=min(2048, config.hidden_size),
        qkv_block_size=16,
        attn_kv_block_size=16,
        attn_reduction_size=4,
    )


def _even_ranges(num_blocks: int, num_workers: int):
    """Worker ``i`` gets blocks ``[round(i*b), round((i+1)*b))`` with
    ``b = num_blocks / num_workers`` and Python's round-half-to-even
    (reference ``:128-133,222-227``)."""
    per_worker = num_blocks / num_workers
    return [
        (round(i * per_worker), round((i + 1) * per_worker)) for i in range(num_workers)
    ]


def schedule_qkv(globs: Globals, layer_idx: int) -> list[Instruction]:
    qkv_outdim = globs.num_total_heads() * globs.head_dim
    num_blocks = assert_div(qkv_outdim, globs.qkv_block_size)
    return [
        LayerNorm_QKV_MatVecRopeAppend(
            layer_idx=layer_idx, start_output_block_idx=s, end_output_block_idx=e
        )
        for s, e in _even_ranges(num_blocks, globs.sm_count())
    ]


def schedule_upgate(globs: Globals, layer_idx: int) -> list[Instruction]:
    """Worker ``i`` gets blocks ``i, i+S, i+2S, ...`` (reference ``:145-164``)."""
    num_blocks = assert_div(globs.intermediate_size, globs.up_gate_proj_block_size)
    workers = globs.sm_count()
    instructions = []
    for w in range(workers):
        block_idxs = list(range(w, num_blocks, workers))
        assert 2 + len(block_idxs) + 1 <= INTS_PER_INSTRUCTION
        instructions.append(LayerNormDoubleMatVecSiLU(layer_idx=layer_idx, block_idxs=block_idxs))
    return instructions


def schedule_downproj(globs: Globals, layer_idx: int) -> list[Instruction]:
    """Jobs ``(column group, block)`` in group-major order are dealt out in
    runs: each worker takes ``round(jobs_left / workers_left)`` consecutive
    jobs, cut at the first column-group boundary (reference ``:167-213``)."""
    num_blocks = assert_div(globs.hidden_size, globs.down_proj_block_size)
    num_groups = globs.down_proj_col_groups()
    workers = globs.sm_count()
    total = num_groups * num_blocks

    instructions: list[Instruction] = []
    assigned = 0
    for w in range(workers):
        if assigned == total:
            break  # fewer jobs than workers (tiny models only)
        per_worker = (total - assigned) / (workers - w)
        take = max(1, round(per_worker))
        group, first_block = divmod(assigned, num_blocks)
        # a run never crosses into the next column group
        take = min(take, num_blocks - first_block, total - assigned)
        instructions.append(
            DownProjResidual(
                layer_idx=layer_idx,
                start_block_idx=first_block,
                end_block_idx=first_block + take,
                reduction_block_idx=group,
            )
        )
        assigned += take
    # The reference does not check this; a run cut at a group boundary on the
    # last worker would silently drop jobs.
    assert assigned == total, f"down projection: {total - assigned} jobs left unassigned"
    return instructions


def schedule_lm_head(globs: Globals) -> list[Instruction]:
    num_blocks = assert_div(globs.vocab_size, globs.lm_head_block_size)
    return [
        RMS_LM_Head(start_output_block_idx=s, end_output_block_idx=e)
        for s, e in _even_ranges(num_blocks, globs.sm_count())
    ]


def make_dag(
    globs: Globals,
    stop_after_op: str | None = None,
    layer_limit: int | None = None,
    num_attention_partitions: int = 1,
):
    nodes: list[DAG_Node] = []
    nlayers = globs.num_hidden_layers if layer_limit is None else layer_limit

    last_outputs: list[DAG_Node] = []
    for layer_idx in range(nlayers):
        new_nodes, last_outputs = make_dag_layer(
            globs=globs,
            layer_idx=layer_idx,
            prev_layer_outputs=last_outputs,
            stop_after_op=stop_after_op,
            num_attention_partitions=num_attention_partitions,
        )
        nodes.extend(new_nodes)

    # the LM head only follows a complete stack (reference ``:256-263``)
    if nlayers == globs.num_hidden_layers and stop_after_op is None:
        lm_head_nodes = [DAG_Node(ins, last_outputs) for ins in schedule_lm_head(globs)]
        nodes.extend(lm_head_nodes)
        last_outputs = lm_head_nodes

    end_node = DAG_Node(NoOp(), last_outputs)
    return nodes, end_node


def make_dag_layer(
    globs: Globals,
    layer_idx: int,
    prev_layer_outputs: list[DAG_Node],
    stop_after_op: str | None = None,
    num_attention_partitions: int = 1,
):
    P = num_attention_partitions
    if P == 1:
        assert globs.skip_attn_reduction
    else:
        assert not globs.skip_attn_reduction, (
            "a split-KV schedule needs skip_attn_reduction=False"
        )
        assert 1 < P <= MAX_ATTENTION_PARTITIONS * MAX_ATTENTION_PARTITIONS
        assert P + reduction_tree_groups(P) <= globs.attn_lse_intermediates.shape[1], (
            "the intermediate buffers hold one slot per partition and per first-level merge"
        )

    new_nodes: list[DAG_Node] = []

    # ---- QKV ------------------------------------------------------------
    qkv_nodes = [DAG_Node(ins, prev_layer_outputs) for ins in schedule_qkv(globs, layer_idx)]
    producer_of_block: dict[int, DAG_Node] = {}
    for node in qkv_nodes:
        for block_idx in node.instruction.block_indices():
            producer_of_block[block_idx] = node
    new_nodes.extend(qkv_nodes)
    if stop_after_op == "qkv":
        return new_nodes, qkv_nodes

    # ---- attention partitions ---------------------------------------------
    blocks_per_head = assert_div(globs.head_dim, globs.qkv_block_size)
    H, KVH = globs.num_attention_heads, globs.num_kv_heads
    partial_nodes: list[DAG_Node] = []
    partials_of_kv_head: dict[int, list[DAG_Node]] = {}
    for kv_head_idx in range(KVH):
        # the K and V blocks of this head (reference ``:311-334``; the Q blocks
        # are guarded by the barrier counters at run time, not by the DAG)
        needed = []
        for head_slot in (H + kv_head_idx, H + KVH + kv_head_idx):
            first = head_slot * blocks_per_head
            needed.extend(range(first, first + blocks_per_head))
        deps: list[DAG_Node] = []
        for block_idx in needed:
            producer = producer_of_block[block_idx]
            if all(producer is not d for d in deps):
                deps.append(producer)
        for partial_idx in range(P):
            ins = PartialAttention(
                layer_idx=layer_idx,
                kv_head_idx=kv_head_idx,
                num_partials=P,
                partial_idx=partial_idx,
            )
            node = DAG_Node(ins, list(deps))
            partial_nodes.append(node)
            partials_of_kv_head.setdefault(kv_head_idx, []).append(node)
    new_nodes.extend(partial_nodes)
    if stop_after_op == "partial":
        return new_nodes, partial_nodes

    # ---- log-sum-exp reduction (split-KV only) -----------------------------
    attention_outputs = partial_nodes
    if P > 1:
        gqa = globs.gqa_ratio()
        group = globs.attn_reduction_size
        reduction_nodes: list[DAG_Node] = []
        # A merge lists at most MAX_ATTENTION_PARTITIONS entries (32-word instruction).  More
        # partitions go through a two-level tree (the reference's "TODO ... better reduction tree",
        # ``:21-35``): first-level merges over consecutive runs of partitions, each written to a slot
        # behind the partitions' own and counted as one more partial result of its heads, then the
        # terminal merge over those slots, which waits for the partitions plus the first-level merges.
        runs = reduction_tree_runs(P)
        for head_start in range(0, H, group):
            kv_heads_touched = sorted({h // gqa for h in range(head_start, head_start + group)})
            partials = [partials_of_kv_head[kv] for kv in kv_heads_touched]
            if len(runs) == 1:
                deps = [n for of_head in partials for n in of_head]
                ins = AttentionReduction(
                    layer_idx=layer_idx,
                    head_start_idx=head_start,
                    num_partials=P,
                    is_terminal=True,
                    reduction_list=list(range(P)),
                    output_partial_idx=None,
                )
                reduction_nodes.append(DAG_Node(ins, deps))
                continue
            first_level: list[DAG_Node] = []
            for k, (lo, hi) in enumerate(runs):
                ins = AttentionReduction(
                    layer_idx=layer_idx,
                    head_start_idx=head_start,
                    num_partials=P,
                    is_terminal=False,
                    reduction_list=list(range(lo, hi)),
                    output_partial_idx=P + k,
                )
                first_level.append(DAG_Node(ins, [of_head[i] for of_head in partials for i in range(lo, hi)]))
            new_nodes.extend(first_level)
            ins = AttentionReduction(
                layer_idx=layer_idx,
                head_start_idx=head_start,
                num_partials=P + len(runs),
                is_terminal=True,
                reduction_list=[P + k for k in range(len(runs))],
                output_partial_idx=None,
            )
            reduction_nodes.append(DAG_Node(ins, first_level))
        new_nodes.extend(reduction_nodes)
        attention_outputs = reduction_nodes
        if stop_after_op == "reduction":
            return new_nodes, reduction_nodes

    # ---- O projection -----------------------------------------------------
    num_o_blocks = assert_div(globs.hidden_size, globs.o_proj_block_size)
    o_proj_nodes: list[DAG_Node] = []
    for group_idx in range(globs.o_proj_col_groups()):
        for o_block_idx in range(num_o_blocks):
            ins = O_ProjResidual(
                layer_idx=layer_idx,
                start_block_idx=o_block_idx,
                end_block_idx=o_block_idx + 1,
                reduction_block_idx=group_idx,
            )
            o_proj_nodes.append(DAG_Node(ins, attention_outputs))
    new_nodes.extend(o_proj_nodes)
    if stop_after_op == "oproj":
        return new_nodes, o_proj_nodes

    # ---- up / gate --------------------------------------------------------
    upgate_nodes = [DAG_Node(ins, o_proj_nodes) for ins in schedule_upgate(globs, layer_idx)]
    new_nodes.extend(upgate_nodes)
    if stop_after_op == "upgate":
        return new_nodes, upgate_nodes

    # ---- down projection ----------------------------------------------------
    downproj_nodes = [DAG_Node(ins, upgate_nodes) for ins in schedule_downproj(globs, layer_idx)]
    new_nodes.extend(downproj_nodes)
    assert stop_after_op in (None, "downproj")
    return new_nodes, downproj_nodes


class LatencyScheduleBuilder(ScheduleBuilder):
    @classmethod
    def make_globals(cls, model, skip_attn_reduction: bool = True):
        return make_globals(model, skip_attn_reduction=skip_attn_reduction)

    @classmethod
    def make_dag(
        cls,
        globs,
        stop_after_op: str | None = None,
        layer_limit: int | None = None,
        num_attention_partitions: int = 1,
    ):
        return make_dag(globs, stop_after_op, layer_limit, num_attention_partitions)

    @classmethod
    def build(
        cls,
        model,
        stop_after_op: str | None = None,
        layer_limit: int | None = None,
        num_attention_partitions: int = 1,
    ):
        """As the base ``build`` plus ``num_attention_partitions``: a value above
        one allocates the buffers with ``skip_attn_reduction=False`` and emits
        the split-KV schedule."""
        from megakernels_amd.scheduler import Schedule

        globs = cls.make_globals(model, skip_attn_reduction=num_attention_partitions == 1)
        nodes, end_node = cls.make_dag(globs, stop_after_op, layer_limit, num_attention_partitions)
        return Schedule(globs, nodes, end_node)

    @classmethod
    def with_new_globals(cls, schedule, model):
        from dataclasses import replace

        return replace(
            schedule,
            globs=cls.make_globals(model, skip_attn_reduction=schedule.globs.skip_attn_reduction),
        )



def check_queues_make_progress(globs: Globals, queues: list[list[Instruction]]) -> None:
    """Raises ``AssertionError`` if the worker queues cannot all run to their ends.

    Every worker executes its queue strictly in order and an instruction starts only when the
    counters it waits for have reached their targets, so an assignment that puts an instruction behind
    one that (transitively) waits for it never finishes - on the device: a wait that runs into its time
    limit.  The waits are those of the Python VM (``python_vm.py:88-95,110,132,176,255,281-290,353-356``)
    plus one that only this build's kernel has: when the column-group jobs of a residual projection run
    each on their own (without ``MK_FLAG_JOINT_RESIDUAL``), the job of the last column group collects the
    other groups' partial sums of its rows and therefore waits for those jobs.  The assignment policies
    of ``megakernels_amd/scheduler.py`` keep the linear instruction order within every queue, which
    satisfies all of it; this check is for hand-made or externally produced queues.

    Targets that the instructions present cannot reach (a schedule that starts in the middle of a
    layer, its earlier counts already in ``barriers``) count as reached by what is present."""
    H, KVH = globs.num_attention_heads, globs.num_kv_heads
    gqa = globs.gqa_ratio()
    blocks_per_head = globs.qkv_blocks_per_head()
    real = [[ins for ins in q if ins.opcode() != 0] for q in queues]

    qkv_block_done: dict[tuple[int, int], bool] = {}
    partial_arrivals: dict[tuple[int, int], int] = {}      # (layer, head group start) -> partitions + merges done
    partial_present: dict[tuple[int, int], int] = {}
    row_arrivals: dict[tuple[int, int], int] = {}          # (layer, barrier row 2..5) -> arrivals
    row_present: dict[tuple[int, int], int] = {}
    group_job_done: dict[tuple[int, int, int, int], bool] = {}   # (opcode, layer, block, group)
    lm_dep_layer = globs.num_hidden_layers - 1

    def arrivals_of(ins):
        """(key, count) pairs this instruction adds when it completes."""
        op = ins.opcode()
        if op == 2:
            if globs.skip_attn_reduction:
                return [((ins.layer_idx, 2), gqa)]
            return [((ins.layer_idx, "p", ins.kv_head_idx * gqa), 1)]
        if op == 3:
            if ins.is_terminal:
                return [((ins.layer_idx, 2), globs.attn_reduction_size)]
            return [((ins.layer_idx, "p", ins.head_start_idx), 1)]
        if op == 4:
            return [((ins.layer_idx, 3), ins.end_block_idx - ins.start_block_idx)]
        if op == 5:
            return [((ins.layer_idx, 4), len(ins.block_idxs))]
        if op == 6:
            return [((ins.layer_idx, 5), ins.end_block_idx - ins.start_block_idx)]
        return []

    def add(table, key, count):
        table[key] = table.get(key, 0) + count

    for q in real:
        for ins in q:
            op = ins.opcode()
            if op == 1:
                for b in ins.block_indices():
                    qkv_block_done[(ins.layer_idx, b)] = False
            for key, count in arrivals_of(ins):
                if len(key) == 3:
                    add(partial_present, (key[0], key[2]), count)
                else:
                    add(row_present, key, count)
            if op in (4, 6):
                for b in range(ins.start_block_idx, ins.end_block_idx):
                    group_job_done[(op, ins.layer_idx, b, ins.reduction_block_idx)] = False

    def reached(table, present, key, target):
        return table.get(key, 0) >= min(target, present.get(key, 0))

    def ready(ins) -> bool:
        op = ins.opcode()
        if op == 1:
            return ins.layer_idx == 0 or reached(row_arrivals, row_present, (ins.layer_idx - 1, 5), globs.down_proj_total_jobs())
        if op == 2:
            heads = list(range(ins.kv_head_idx * gqa, (ins.kv_head_idx + 1) * gqa)) + [H + ins.kv_head_idx, H + KVH + ins.kv_head_idx]
            return all(qkv_block_done.get((ins.layer_idx, h * blocks_per_head + b), True)
                       for h in heads for b in range(blocks_per_head))
        if op == 3:
            return reached(partial_arrivals, partial_present, (ins.layer_idx, ins.head_start_idx), ins.num_partials)
        if op in (4, 6):
            row, target = (2, H) if op == 4 else (4, globs.up_gate_total_blocks())
            if not reached(row_arrivals, row_present, (ins.layer_idx, row), target):
                return False
            groups = globs.o_proj_col_groups() if op == 4 else globs.down_proj_col_groups()
            if ins.reduction_block_idx == groups - 1:
                # the collecting job: the other groups' jobs of its rows, where they are scheduled at all
                return all(group_job_done.get((op, ins.layer_idx, b, g), True)
                           for b in range(ins.start_block_idx, ins.end_block_idx) for g in range(groups - 1))
            return True
        if op == 5:
            return reached(row_arrivals, row_present, (ins.layer_idx, 3), globs.o_proj_total_jobs())
        if op == 7:
            return reached(row_arrivals, row_present, (lm_dep_layer, 5), globs.down_proj_total_jobs())
        return True

    def complete(ins):
        op = ins.opcode()
        if op == 1:
            for b in ins.block_indices():
                qkv_block_done[(ins.layer_idx, b)] = True
        for key, count in arrivals_of(ins):
            if len(key) == 3:
                add(partial_arrivals, (key[0], key[2]), count)
            else:
                add(row_arrivals, key, count)
        if op in (4, 6):
            for b in range(ins.start_block_idx, ins.end_block_idx):
                group_job_done[(op, ins.layer_idx, b, ins.reduction_block_idx)] = True

    at = [0] * len(real)
    progressed = True
    while progressed:
        progressed = False
        for w, q in enumerate(real):
            while at[w] < len(q) and ready(q[at[w]]):
                complete(q[at[w]])
                at[w] += 1
                progressed = True
    stuck = [(w, q[at[w]]) for w, q in enumerate(real) if at[w] < len(q)]
    assert not stuck, (
        f"{len(stuck)} worker queue(s) can never finish: worker {stuck[0][0]} waits at {stuck[0][1]} for instructions "
        "that are queued behind instructions waiting for it")
