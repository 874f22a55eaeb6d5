"""MI355X-native megakernel decode runtime.

Host-side mirror of the reference's Python surface for the ``mk`` batch-1
decode path (reference ``megakernels/``): instruction dataclasses and their
32-word encoding, the scheduler that turns a Llama layer stack into per-CU
instruction queues, the generators, and the ``mk_llama`` launch boundary.
Everything below that boundary is a hand-written HIP persistent kernel for
gfx950 in ``megakernels_amd/csrc``.
"""

__all__ = [
    "dispatch",
    "generators",
    "instructions",
    "llama",
    "mk",
    "model_types",
    "scheduler",
    "utils",
]
