"""Token-level training examples and the metrics log, as the reference's `train` loop builds them
(ferrotensor-trainer/src/data.rs:34-96; ferrotensor-cli/src/main.rs:1885-1921). Tokenisation itself
is outside this package: examples are built from token ids."""
import json
import time
from dataclasses import dataclass
from typing import List, Optional, Sequence, Tuple


@dataclass
class TrainingExample:
    """`TrainingExample` (data.rs:34-43): inputs, next-token targets and a 0/1 loss mask, all the
    same length; `as_tuple()` is what `Trainer.train_batch` takes."""
    input_ids: List[int]
    target_ids: List[int]
    loss_mask: List[int]

    @staticmethod
    def from_next_token(sequence: Sequence[int]) -> "TrainingExample":
        """Inputs are all but the last token, targets all but the first, every target supervised;
        a sequence shorter than 2 is kept as it is (data.rs:47-66)."""
        seq = [int(t) for t in sequence]
        if len(seq) < 2:
            return TrainingExample(list(seq), list(seq), [1] * len(seq))
        return TrainingExample(seq[:-1], seq[1:], [1] * (len(seq) - 1))

    @staticmethod
    def from_sft_prompt_response(prompt_tokens: Sequence[int], response_tokens: Sequence[int]) -> "TrainingExample":
        """Loss only where the prediction recovers a response token: the first response token sits at
        index len(prompt) of the full sequence, so its target index is len(prompt) - 1 (data.rs:72-96)."""
        prompt = [int(t) for t in prompt_tokens]
        response = [int(t) for t in response_tokens]
        full = prompt + response
        if len(full) < 2:
            return TrainingExample.from_next_token(full)
        target = full[1:]
        if prompt and response:
            first = max(len(prompt) - 1, 0)
            mask = [0] * first + [1] * (len(target) - first)
        else:
            mask = [1] * len(target)
        return TrainingExample(full[:-1], target, mask)

    def as_tuple(self) -> Tuple[List[int], List[int], List[int]]:
        return self.input_ids, self.target_ids, self.loss_mask


class MetricsWriter:
    """`metrics.jsonl` of the `train` command: one object per logging window with step, mean loss per
    supervised token, last gradient norm and rate, supervised tokens and seconds of the window, and
    seconds since the start of the run (main.rs:1905-1921)."""

    def __init__(self, path: str):
        self._f = open(path, "a")
        self._run_start = time.monotonic()
        self._reset()

    def _reset(self):
        self._win_start = time.monotonic()
        self._loss_sum, self._tokens = 0.0, 0

    def add_sequence(self, mean_loss: float, tokens: int):
        """One trained sequence: its mean loss weighs by its supervised tokens (main.rs:1884-1887)."""
        self._loss_sum += float(mean_loss) * tokens
        self._tokens += int(tokens)

    def log(self, step: int, grad_norm: Optional[float], lr: Optional[float]) -> dict:
        now = time.monotonic()
        rec = {"step": int(step), "loss": self._loss_sum / max(self._tokens, 1),
               "grad_norm": grad_norm, "lr": lr, "tokens": self._tokens, "seconds": now - self._win_start,
               "elapsed": now - self._run_start}
        self._f.write(json.dumps(rec) + "\n")
        self._f.flush()
        self._reset()
        return rec

    def close(self):
        self._f.close()
