"""Time and energy of the work outside the partitions: embedding, final norm + output layer, loss.

Same five measurements and the same files as the reference's non-partition profiler
(tests/bayesian/nonpartition/profile_nonpartition.py:92-486): ``preprocess`` (embedding forward),
``preprocess_backward``, ``postprocess`` (concatenate the nanobatches, final RMSNorm, output layer),
``postprocess_backward`` and ``loss``, each written to
``<dir>/nonpartition/<freq>/<name>_energy.csv`` with the header
``time (s),total_energy (J),per_rank_energy (J)`` and one row.  ``read_nonpartition`` turns such a
directory back into the per-frequency table the candidate generator adds to the first and last
pipeline stages (tests/kareus/generate_profile_csv.py:79-113).
"""

from __future__ import annotations

import csv
import os
from typing import Callable, Dict, Iterable, Optional, Tuple

import torch

from ..block import LayerConfig
from ..energy import PowerSampler
from ..model import LanguageModelEmbedding, _CrossEntropy, _Linear, _RMSNorm
from .hardware import Trial, measure

STEP_NAMES = ("preprocess", "preprocess_backward", "postprocess", "postprocess_backward", "loss")
_FILE_TO_KEY = {"preprocess": "forward-embedding", "postprocess": "forward-output", "loss": "loss-func",
                "preprocess_backward": "backward-embedding", "postprocess_backward": "backward-output"}
HEADER = "time (s),total_energy (J),per_rank_energy (J)"


class NonPartitionProfiler:
    """Synthetic inputs as in the reference: random token ids and labels ``[batch, seq]``, N(0,1)
    hidden states of two nanobatches, N(0,1) logits for the loss."""

    def __init__(self, config: LayerConfig, vocab_rows: int, batch_size: int, seq_len: int,
                 device=None, seed: int = 1234) -> None:
        self.config, self.device = config, torch.device(device) if device is not None else torch.device("cpu")
        gen = torch.Generator().manual_seed(seed)
        dt, h = config.params_dtype, config.hidden_size
        n = config.num_nanobatches
        self.embedding = LanguageModelEmbedding(config, vocab_rows, 0, device=self.device, generator=gen)
        self.final_gamma = torch.ones(h, device=self.device, dtype=dt, requires_grad=True)
        self.w_out = (torch.randn(vocab_rows, h, generator=gen) * config.init_method_std).to(self.device, dt).requires_grad_(True)
        rnd = lambda *shape: torch.randn(*shape, generator=gen).to(self.device, dt)
        self.input_ids = torch.randint(0, vocab_rows, (batch_size, seq_len), generator=gen).to(self.device)
        self.labels = torch.randint(0, vocab_rows, (batch_size, seq_len), generator=gen).to(self.device)
        self.hidden_parts = [rnd(seq_len, batch_size // n, h) for _ in range(n)]
        self.grad_hidden = rnd(seq_len, batch_size, h)
        self.logits = rnd(seq_len, batch_size, vocab_rows)
        self.grad_logits = rnd(seq_len, batch_size, vocab_rows)
        self._emb_out: Optional[torch.Tensor] = None
        self._post: Optional[Tuple[torch.Tensor, torch.Tensor]] = None

    def _postprocess(self, x):
        be = self.config.backend
        return _Linear.apply(_RMSNorm.apply(x, self.final_gamma, self.config.layernorm_epsilon, be), self.w_out, be)

    def step(self, name: str) -> Callable[[], object]:
        be = self.config.backend
        if name == "preprocess":
            return lambda: self.embedding(self.input_ids)
        if name == "preprocess_backward":
            def run():
                self.embedding.weight.grad = None
                self.embedding(self.input_ids).backward(self.grad_hidden)
            return run
        if name == "postprocess":
            return lambda: self._postprocess(torch.cat(self.hidden_parts, dim=1))
        if name == "postprocess_backward":
            def run():
                self.final_gamma.grad = self.w_out.grad = None
                x = torch.cat(self.hidden_parts, dim=1).requires_grad_(True)
                self._postprocess(x).backward(self.grad_logits)
            return run
        if name == "loss":
            return lambda: _CrossEntropy.apply(self.logits, self.labels, be)
        raise ValueError(f"unknown step {name!r}; expected one of {STEP_NAMES}")

    def run(self, out_dir: str, freq: int, names: Iterable[str] = STEP_NAMES,
            sampler: Optional[PowerSampler] = None, world_size: int = 1, **measure_kwargs) -> Dict[str, Trial]:
        """Measure the named steps and write one CSV each.  Note that ``preprocess_backward`` and
        ``postprocess_backward`` time forward + backward of their step, as the reference's do."""
        d = os.path.join(out_dir, "nonpartition", str(freq))
        os.makedirs(d, exist_ok=True)
        trials = {}
        for name in names:
            trial = measure(self.step(name), sampler, **measure_kwargs)
            energy = trial.energy_per_iter if trial.energy_per_iter is not None else float("nan")
            with open(os.path.join(d, f"{name}_energy.csv"), "w") as f:
                f.write(HEADER + "\n")
                f.write(f"{trial.time_per_iter},{energy},{energy / world_size}\n")
            trials[name] = trial
        return trials


def read_nonpartition(out_dir: str, freqs: Iterable[int]) -> Dict[int, Dict[str, Tuple[float, float]]]:
    """``{freq: {"forward-embedding": (time_s, per_rank_energy_j), ...}}`` from the CSV files."""
    table: Dict[int, Dict[str, Tuple[float, float]]] = {}
    for freq in freqs:
        entry = {}
        for name, key in _FILE_TO_KEY.items():
            path = os.path.join(out_dir, "nonpartition", str(freq), f"{name}_energy.csv")
            if not os.path.exists(path):
                raise FileNotFoundError(path)
            with open(path) as f:
                rows = list(csv.reader(f))
            if len(rows) < 2 or len(rows[1]) < 3:
                raise RuntimeError(f"Malformed CSV at {path} (need at least 1 row and 3 columns)")
            col = rows[0].index("per_rank_energy (J)") if "per_rank_energy (J)" in rows[0] else 2
            entry[key] = (float(rows[1][0]), float(rows[1][col]))
        table[int(freq)] = entry
    return table
