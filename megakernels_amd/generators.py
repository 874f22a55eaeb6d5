"""Token generation loops (reference ``megakernels/generators.py``).

``MK_Generator.run`` is the per-token hot loop of the ``mk`` path
(``generators.py:121-143``): embedding row into ``hidden_states``, barrier
reset, ``pos_id`` update, one megakernel launch, ``argmax`` over the bf16
logits (first maximum wins).  Nothing in it synchronises with the host.
"""

from __future__ import annotations

import torch
from torch import Tensor

from megakernels_amd.mk import MK_Interpreter
from megakernels_amd.model_types import BatchState
from megakernels_amd.scheduler import Schedule


class Generator:
    def generate(self, output_tokens: Tensor, prompt_len: int, ntok: int, ntok_already_generated: int = 1):
        raise NotImplementedError

    def check(self):
        """Raise if the tokens produced so far cannot be trusted (nothing to check by default)."""

    def generate_with_eos(
        self,
        output_tokens: Tensor,
        prompt_len: int,
        ntok: int,
        eos_token_check_interval: int,
        eos_token_ids: list[int],
    ):
        """Decode in chunks of ``eos_token_check_interval`` tokens and look for
        an end-of-sequence id on the host after each chunk.  Returns
        ``(index of the first eos token or ntok, tokens generated)``
        (reference ``generators.py:21-58``)."""
        assert output_tokens.shape[0] == 1, "batch size must be 1"
        for done in range(1, ntok, eos_token_check_interval):
            chunk = min(eos_token_check_interval, ntok - done)
            self.generate(output_tokens, prompt_len=prompt_len, ntok=chunk, ntok_already_generated=done)
            tokens = output_tokens[0, done : done + chunk].cpu().tolist()  # synchronises
            self.check()  # a chunk whose launch gave up holds garbage: raise instead of returning it
            for j, token in enumerate(tokens):
                if token in eos_token_ids:
                    # the first token came from prefill, hence the -1
                    return done + j, done + chunk - 1
        return ntok, ntok - 1


class PyTorchGenerator(Generator):
    """Plain PyTorch decode, one dense forward per token
    (reference ``generators.py:61-92``)."""

    def __init__(self, model):
        self.model = model

    def generate(self, output_tokens: Tensor, prompt_len: int, ntok: int, ntok_already_generated: int = 1):
        first_seq_len = prompt_len + ntok_already_generated
        for i in range(ntok):
            src = i + ntok_already_generated - 1
            state = BatchState(
                input_ids=output_tokens[:, src : src + 1],
                position_ids=torch.tensor([first_seq_len - 1 + i], device=self.model.device),
                seq_len=first_seq_len + i,
            )
            out = self.model(state)
            output_tokens[:, src + 1] = out.output_ids.squeeze(-1)


class MK_Generator(Generator):
    def __init__(
        self,
        model,
        interpreter: MK_Interpreter,
        schedule: Schedule,
        barrier_fill_val: int = 0,
        skip_mk: bool = False,
        skip_rest: bool = False,
        fused_step: bool | None = None,
        steps_per_launch: int = 0,
    ):
        self.model = model
        self.interpreter = interpreter
        self.schedule = schedule
        self.barrier_fill_val = barrier_fill_val
        self.skip_mk = skip_mk
        self.skip_rest = skip_rest
        # One launch per token when the interpreter can do the embedding lookup, the barrier reset
        # and the argmax itself; otherwise (and on request) the reference's sequence of small
        # kernels around the launch.
        can_fuse = hasattr(interpreter, "interpret_step") and barrier_fill_val == 0 and not skip_mk and not skip_rest
        self.fused_step = can_fuse if fused_step is None else (fused_step and can_fuse)
        # With the glue folded in, consecutive steps need nothing from the host: `generate` hands the
        # interpreter up to this many steps per launch (0: all of them, 1: one launch per token).
        self.steps_per_launch = steps_per_launch if hasattr(interpreter, "interpret_steps") else 1
        self.fill()

    def fill(self):
        self.schedule.globs.barriers.fill_(self.barrier_fill_val)

    def replace_with_noops(self):
        self.schedule.globs.instructions.zero_()

    def check(self):
        """Synchronise and raise if a launch since the last check gave up."""
        check = getattr(self.interpreter, "check_status", None)
        if check is not None and not self.skip_mk:
            check(self.schedule.globs.barriers.device)

    def run(self, input_ids: Tensor, pos_id: int):
        globs = self.schedule.globs
        if not self.skip_rest:
            embedded = self.model.model.embed_tokens(BatchState(input_ids=input_ids))
            globs.hidden_states[:] = embedded.hidden_states.reshape(-1)
        self.fill()
        globs.pos_id = pos_id
        if not self.skip_mk:
            self.interpreter.interpret(globs)
        if self.skip_rest:
            return input_ids
        return torch.argmax(globs.logits, dim=-1)

    def generate(self, output_tokens: Tensor, prompt_len: int, ntok: int, ntok_already_generated: int = 1,
                 check: bool = False):
        """``check``: synchronise at the end and raise if a launch gave up (for callers that are
        about to read the tokens anyway; the reference's loop has no such step)."""
        self._generate(output_tokens, prompt_len, ntok, ntok_already_generated)
        if check:
            self.check()

    def _generate(self, output_tokens: Tensor, prompt_len: int, ntok: int, ntok_already_generated: int = 1):
        if self.fused_step and output_tokens.dtype == torch.int64 and output_tokens.is_contiguous():
            globs = self.schedule.globs
            embed = self.model.model.embed_tokens.weight
            self.fill()
            i = 0
            while i < ntok:
                n = ntok - i if self.steps_per_launch <= 0 else min(self.steps_per_launch, ntok - i)
                src = ntok_already_generated + i - 1
                globs.pos_id = prompt_len + ntok_already_generated + i - 1
                if n == 1:
                    self.interpreter.interpret_step(globs, embed, output_tokens[0, src : src + 1], output_tokens[0, src + 1 : src + 2])
                else:
                    self.interpreter.interpret_steps(globs, embed, output_tokens[0, src : src + 1], output_tokens[0, src + 1 : src + 1 + n])
                    globs.pos_id += n - 1  # the position the launch ended on
                i += n
            return
        for i in range(ntok):
            src = ntok_already_generated + i - 1
            pos_id = prompt_len + ntok_already_generated + i - 1
            output_ids = self.run(output_tokens[:, src : src + 1], pos_id=pos_id)
            output_tokens[:, src + 1] = output_ids.reshape(-1)
