"""Instruction DAG, worker assignment policies and tensorisation.

Behavioural mirror of reference ``megakernels/scheduler.py``:

* ``DAG_Node`` / ``Schedule`` / ``ScheduleBuilder`` (``scheduler.py:17-91``)
* assignment policies ``rr``, ``zz``, ``wave``, ``dag``, ``pool`` (``scheduler.py:94-271``)
* ``serialize_and_pad`` and ``tensorize_instructions`` (``scheduler.py:274-308``):
  ``globs.instructions`` is ``int32 [workers, slots, 32]`` and ``globs.timings``
  is ``int32 [workers, slots, 128]``.

"SM" in the names is kept for drop-in compatibility; on MI355X a worker is one
persistent workgroup pinned to one compute unit.
"""

from __future__ import annotations

import heapq
from dataclasses import dataclass, field, replace

import torch

from megakernels_amd.instructions import BaseGlobals, Instruction, NoOp

INTS_PER_INSTRUCTION = 32
TIMING_SLOTS = 128


@dataclass(eq=False)
class DAG_Node:
    instruction: Instruction
    dependencies: list["DAG_Node"]

    children: set["DAG_Node"] = field(default_factory=set)
    start_time: float = float("inf")
    end_time: float = float("inf")
    remaining_dependencies: set["DAG_Node"] = field(default_factory=set)
    priority: float = 0

    # Nodes are hashed by the words of their instruction (reference
    # ``scheduler.py:18-19``); equality stays identity, so two nodes with equal
    # instructions remain distinct members of a set.
    def __hash__(self):
        return hash(tuple(self.instruction.serialize()))

    def earliest_ready_time(self, globs: BaseGlobals):
        if not self.dependencies:
            return 0
        return max(dep.end_time for dep in self.dependencies)

    def register_with_parents(self):
        for dep in self.dependencies:
            dep.children.add(self)

    def calc_priority(self, globs: BaseGlobals):
        for dep in self.dependencies:
            dep.priority = max(self.priority + dep.instruction.cost(globs), dep.priority)
            dep.calc_priority(globs)


@dataclass
class Schedule:
    globs: BaseGlobals
    dag_nodes: list[DAG_Node]
    end_node: DAG_Node

    def get_linear_instructions(self) -> list[Instruction]:
        """Instructions in construction order, which is a topological order of
        the DAG (reference ``scheduler.py:55-57``)."""
        return [node.instruction for node in self.dag_nodes]

    def smart_assign_to_sms(self):
        return assign_dag_to_sms(self)

    def round_robin_assign_to_sms(self):
        return round_robin_assign_to_sms(
            self.get_linear_instructions(), self.globs.sm_count()
        )


class ScheduleBuilder:
    @classmethod
    def make_globals(cls, model):
        raise NotImplementedError

    @classmethod
    def make_dag(cls, globs, stop_after_op: str | None = None, layer_limit: int | None = None):
        raise NotImplementedError

    @classmethod
    def build(cls, model, stop_after_op: str | None = None, layer_limit: int | None = None):
        globs = cls.make_globals(model)
        dag_nodes, end_node = cls.make_dag(globs, stop_after_op, layer_limit)
        return Schedule(globs, dag_nodes, end_node)

    @classmethod
    def with_new_globals(cls, schedule: Schedule, model):
        """Same DAG, fresh activation buffers (weights and KV cache are shared
        with the model; reference ``scheduler.py:89-91``)."""
        return replace(schedule, globs=cls.make_globals(model))


# --------------------------------------------------------------------------
# assignment policies
# --------------------------------------------------------------------------


def round_robin_assign_to_sms(instructions: list[Instruction], sm_count: int):
    """Instruction ``i`` goes to worker ``i mod sm_count`` (reference
    ``scheduler.py:154-161``)."""
    queues: list[list[Instruction]] = [[] for _ in range(sm_count)]
    for i, ins in enumerate(instructions):
        queues[i % sm_count].append(ins)
    return queues


def zig_zag_assign_to_sms(instructions: list[Instruction], sm_count: int):
    """Boustrophedon order: workers 0..S-1 then S-1..0 (reference
    ``scheduler.py:164-176``)."""
    queues: list[list[Instruction]] = [[] for _ in range(sm_count)]
    period = 2 * sm_count
    for i, ins in enumerate(instructions):
        phase = i % period
        worker = phase if phase < sm_count else period - 1 - phase
        queues[worker].append(ins)
    return queues


def collect_into_waves(instructions: list[Instruction]):
    """Maximal runs of consecutive instructions with the same opcode
    (reference ``scheduler.py:179-193``)."""
    waves: list[list[Instruction]] = []
    for ins in instructions:
        if waves and waves[-1][-1].opcode() == ins.opcode():
            waves[-1].append(ins)
        else:
            waves.append([ins])
    return waves


def wave_assign_to_sms(schedule: Schedule):
    """Within each wave hand the most expensive instruction to the least
    loaded worker (reference ``scheduler.py:196-220``)."""
    globs = schedule.globs
    sm_count = globs.sm_count()
    queues: list[list[Instruction]] = [[] for _ in range(sm_count)]
    load = [(0, w) for w in range(sm_count)]
    heapq.heapify(load)
    for wave in collect_into_waves(schedule.get_linear_instructions()):
        # sorted() is stable, so equal costs keep their schedule order
        for ins in sorted(wave, key=lambda x: x.cost(globs), reverse=True):
            total, worker = heapq.heappop(load)
            heapq.heappush(load, (total + ins.cost(globs), worker))
            queues[worker].append(ins)
    return queues


def assign_dag_to_sms(schedule: Schedule):
    """List scheduling over the DAG: repeatedly take the most expensive ready
    instruction (ties: lowest schedule index) and give it to the worker that
    becomes free first (ties: lowest worker index); reference
    ``scheduler.py:94-151``."""
    nodes = schedule.dag_nodes
    globs = schedule.globs

    for node in nodes:
        node.children = set()
    for node in nodes:
        node.register_with_parents()
        node.remaining_dependencies = set(node.dependencies)

    sm_count = globs.sm_count()
    queues: list[list[Instruction]] = [[] for _ in range(sm_count)]
    free_at = [(0, w) for w in range(sm_count)]
    heapq.heapify(free_at)

    index_of = {id(n): i for i, n in enumerate(nodes)}
    ready = [
        (-n.instruction.cost(globs), i) for i, n in enumerate(nodes) if not n.dependencies
    ]
    heapq.heapify(ready)

    while ready:
        _, idx = heapq.heappop(ready)
        node = nodes[idx]
        start, worker = heapq.heappop(free_at)
        node.start_time = start
        node.end_time = start + node.instruction.cost(globs)
        queues[worker].append(node.instruction)
        heapq.heappush(free_at, (node.end_time, worker))
        for child in node.children:
            # every parent is popped exactly once, so this set empties exactly once
            child.remaining_dependencies.remove(node)
            if not child.remaining_dependencies:
                heapq.heappush(
                    ready, (-child.instruction.cost(globs), index_of[id(child)])
                )
    return queues


def pool_assign_to_sms(instructions: list[Instruction], sm_count: int, memory_fraction: float):
    """Split workers into a "memory" pool and a "compute" pool by instruction
    tag and round-robin inside each (reference ``scheduler.py:223-242``)."""
    by_pool: dict[str, list[Instruction]] = {"memory": [], "compute": []}
    for ins in instructions:
        pool = ins.tags()["pool"]
        if pool not in by_pool:
            raise ValueError(f"Unknown pool: {pool}")
        by_pool[pool].append(ins)
    mem_workers = round(sm_count * memory_fraction)
    return round_robin_assign_to_sms(by_pool["memory"], mem_workers) + round_robin_assign_to_sms(
        by_pool["compute"], sm_count - mem_workers
    )


def assign_to_sms(
    mode: str,
    schedule: Schedule | None = None,
    instructions: list[Instruction] | None = None,
    sm_count: int | None = None,
    memory_fraction: float | None = None,
):
    """Dispatch on the policy name (reference ``scheduler.py:245-271``)."""
    if schedule is not None:
        instructions = schedule.get_linear_instructions()
        sm_count = schedule.globs.sm_count()
    if mode == "rr":
        return round_robin_assign_to_sms(instructions, sm_count)
    if mode == "zz":
        return zig_zag_assign_to_sms(instructions, sm_count)
    if mode == "wave":
        return wave_assign_to_sms(schedule)
    if mode == "dag":
        return assign_dag_to_sms(schedule)
    if mode == "pool":
        assert memory_fraction is not None
        return pool_assign_to_sms(instructions, sm_count, memory_fraction=memory_fraction)
    raise ValueError(f"Unknown mode: {mode}")


# --------------------------------------------------------------------------
# tensorisation
# --------------------------------------------------------------------------


def serialize_and_pad(instruction: Instruction) -> list[int]:
    words = instruction.serialize()
    if len(words) > INTS_PER_INSTRUCTION:
        raise AssertionError(
            f"{type(instruction).__name__} needs {len(words)} words, "
            f"the device format holds {INTS_PER_INSTRUCTION}"
        )
    return words + [0] * (INTS_PER_INSTRUCTION - len(words))


def tensorize_instructions(globs: BaseGlobals, instruction_queues: list[list[Instruction]]):
    """Pad every queue with ``NoOp`` to the longest one and upload the word
    tensor and a zeroed timings tensor (reference ``scheduler.py:281-308``).
    As in the reference the queues are padded in place."""
    num_workers = len(instruction_queues)
    if num_workers != globs.sm_count():
        raise AssertionError(
            f"{num_workers} queues for {globs.sm_count()} workers"
        )
    longest = max(len(q) for q in instruction_queues)
    for q in instruction_queues:
        q.extend(NoOp() for _ in range(longest - len(q)))

    rows = [serialize_and_pad(ins) for q in instruction_queues for ins in q]
    words = torch.tensor(rows, dtype=torch.int32).view(
        num_workers, longest, INTS_PER_INSTRUCTION
    )
    globs.instructions = words.to(globs.device)
    globs.timings = torch.zeros(
        (num_workers, longest, TIMING_SLOTS), dtype=torch.int32, device=globs.device
    )
