"""Token selection on the GPU: greedy (lowest index of the maximum) or temperature sampling by
inverse CDF with SplitMix64 uniforms, and the log-probability of the chosen token under the
distribution that was used (src/generation.rs:655-664, 732-743, 1148-1165).

Draw numbering follows the reference (src/generation.rs:667-699): every selection over a batch
that started with B rows reserves B draws, finished rows included, so the row that started as
number b uses draw  s * B + b  in step s.
"""

import torch

from ..kernels import library as K

_MASK64 = 2 ** 64 - 1


def splitmix64(seed, index):
    """Output ``index`` of the stream (src/generation/random.rs:232-237); host twin of the kernel."""
    value = (seed + 0x9E3779B97F4A7C15 * ((index + 1) & _MASK64)) & _MASK64
    value = ((value ^ (value >> 30)) * 0xBF58476D1CE4E5B9) & _MASK64
    value = ((value ^ (value >> 27)) * 0x94D049BB133111EB) & _MASK64
    return value ^ (value >> 31)


def interior_unit(bits):
    """The uniform in (0, 1) the kernel derives from 64 mixed bits (random.rs:244-247)."""
    return ((bits >> 41) + 0.5) / float(1 << 23)


class Sampler:
    def __init__(self, config, batch_rows, device):
        self.config, self.batch_rows, self.device = config, batch_rows, device
        self.selections = 0
        # ids and log-probabilities share one buffer so that they come back in one copy
        self.packed = torch.zeros((2, batch_rows), dtype=torch.int32, device=device)
        self.ids, self.logp = self.packed[0], self.packed[1].view(torch.float32)
        self.host = torch.zeros((2, batch_rows), dtype=torch.int32).pin_memory()

    def select(self, logits, rows):
        """One token for each row of ``logits`` (float32 [len(rows), vocab]); ``rows`` are the rows'
        numbers in the batch as it started.  Returns (ids, log-probabilities) as Python lists; this
        is the step's one readback."""
        count = len(rows)
        draw_rows = None
        if self.config.sampling:
            draw_rows = torch.tensor(rows, dtype=torch.int32).to(self.device, non_blocking=True)
        K.sample(logits, self.ids[:count], self.logp[:count],
                 temperature=float(self.config.temperature) if self.config.sampling else None,
                 seed=self.config.seed, first_draw=self.selections * self.batch_rows, draw_rows=draw_rows)
        self.selections += 1
        self.host.copy_(self.packed)                  # synchronous: the kernels above have finished after it
        return self.host[0, :count].tolist(), self.host[1].view(torch.float32)[:count].tolist()
