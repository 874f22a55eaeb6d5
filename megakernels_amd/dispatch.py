"""Setting name -> schedule builder / megakernel interpreter
(reference ``megakernels/dispatch.py:17-42``).  Only the "latency" setting
(batch-1 decode) exists in this build.  The Python reference VM is test
infrastructure and is not reachable from here: asking for it raises."""

from __future__ import annotations

from pathlib import Path

from megakernels_amd.demos.latency.mk import LatencyMK_Interpreter
from megakernels_amd.demos.latency.scheduler import LatencyScheduleBuilder
from megakernels_amd.mk import MK_Interpreter
from megakernels_amd.scheduler import ScheduleBuilder

BUILDER_MAP = {"latency": LatencyScheduleBuilder}
MK_INTERPRETER_MAP = {"latency": LatencyMK_Interpreter}


def _lookup(table: dict, mode: str):
    if mode not in table:
        raise ValueError(
            f"setting {mode!r} is not part of this build (available: {sorted(table)})"
        )
    return table[mode]


def make_schedule_builder(mode: str) -> ScheduleBuilder:
    return _lookup(BUILDER_MAP, mode)()


def make_mk_interpreter(mode: str, mk_dir: Path | str | None = None) -> MK_Interpreter:
    return _lookup(MK_INTERPRETER_MAP, mode)(mk_dir)


def make_pyvm_interpreter(mode: str):
    raise NotImplementedError(
        "the Python VM is a CPU checker that lives with the tests, not a product path; "
        "use mode=mk (HIP megakernel) or mode=torch (plain PyTorch forward)"
    )
