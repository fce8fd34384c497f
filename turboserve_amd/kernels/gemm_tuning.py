"""Measured choice of the BLAS library's matrix products.

Projections over more than 64 rows go to the BLAS library behind ``torch.mm`` / ``torch.addmm``
(as every linear layer of the reference does, src/turboserve/engine/model/layers.py:142).  The
library picks one of its several hundred kernels per shape by a heuristic, and for this
model family's long, narrow products the pick is often far from its best kernel (a 256 x 256
macro tile that fills under half of the compute units, for instance).  PyTorch's tunable-op
layer can time the library's candidates for a shape once and remember the winner; this
module drives it:

* ``with LibraryGemmTuning(path):`` times every product shape that runs inside the block; the
  winners are kept in memory and appended to ``path`` (read again by the next process);
* after the block the winners stay in use, and shapes that were not timed fall back to the
  library's heuristic at no cost (no timing outside the block, so no surprise stalls);
* a candidate has to reproduce the default kernel's result (within bfloat16 rounding) to be
  eligible, and products too small to be worth timing never leave the default kernel
  (``Ops.library_tuning_min_work``).

An engine runs the block over one dry step of its usual prefill size at start-up when asked to
(``EngineConfig.tune_gemm_tokens``).  The choice changes which library kernel computes a product,
never its precision: bfloat16 operands, 32-bit accumulation.
"""

from __future__ import annotations

import json
import os
import tempfile

import torch


def default_results_file() -> str:
    """A per-user file: under ``$XDG_CACHE_HOME`` or ``~/.cache`` when that is writable, else
    under the temporary folder."""
    roots = []
    if os.environ.get("XDG_CACHE_HOME"):
        roots.append(os.environ["XDG_CACHE_HOME"])
    home = os.path.expanduser("~")
    if home and home != "~" and os.path.isdir(home):
        roots.append(os.path.join(home, ".cache"))
    roots.append(os.path.join(tempfile.gettempdir(), f"turboserve_amd-{os.getuid()}"))
    for root in roots:
        folder = os.path.join(root, "turboserve_amd")
        try:
            os.makedirs(folder, exist_ok=True)
            if os.access(folder, os.W_OK):
                return os.path.join(folder, "gemm_tuning.csv")
        except OSError:
            continue
    return os.path.join(tempfile.gettempdir(), f"turboserve_amd_gemm_tuning_{os.getuid()}.csv")


class LibraryGemmTuning:
    """Context manager: inside, new product shapes are timed; afterwards the winners are used."""

    def __init__(self, results_file: str | None = None, *, max_ms_per_candidate: int = 30,
                 max_iterations: int = 20) -> None:
        self.results_file = results_file or default_results_file()
        self.max_ms_per_candidate = max_ms_per_candidate
        self.max_iterations = max_iterations

    def __enter__(self) -> "LibraryGemmTuning":
        tunable = torch.cuda.tunable
        tunable.enable(True)
        tunable.set_filename(self.results_file)  # winners are appended here as they are found
        if os.path.exists(self.results_file):
            try:
                tunable.read_file(self.results_file)
            except RuntimeError:
                pass  # a file of another library version: its entries are ignored and replaced
        tunable.set_max_tuning_duration(self.max_ms_per_candidate)
        tunable.set_max_tuning_iterations(self.max_iterations)
        # A candidate is only eligible if its result agrees with the library's default kernel up
        # to bfloat16 rounding: the fastest kernel for a shape is of no use if it is a broken one.
        tunable.set_numerical_check_tolerances(True, 2e-2, 2e-2)
        tunable.tuning_enable(True)
        return self

    def __exit__(self, *exc) -> None:
        torch.cuda.tunable.tuning_enable(False)
        torch.cuda.tunable.set_numerical_check_tolerances(False)

    @staticmethod
    def num_results() -> int:
        return len(torch.cuda.tunable.get_results())


class OwnProductChoices:
    """What timing this engine's own product against the library's best kernel found
    (``Ops.wide_choices``, ``Ops.wide_timings``), kept in a file beside the library's results so
    that the next process starts from it: it decides as the one before did (a run under a
    profiler, whose clock is not to be trusted, too) and spends no time on what is known.  The
    file holds for one device and one state of the sources; anything else is ignored and
    replaced."""

    def __init__(self, results_file: str, ops) -> None:
        self.path = results_file + ".own.json"
        self.ops = ops

    def _stamp(self) -> dict[str, str]:
        from turboserve_amd.hwinfo import source_digest

        return {"device": torch.cuda.get_device_name(self.ops.device), "torch": torch.__version__,
                "source": source_digest()}

    def load(self) -> int:
        """Adopt the file's choices for products this process has not timed; how many."""
        try:
            with open(self.path, encoding="utf-8") as handle:
                data = json.load(handle)
        except (OSError, ValueError):
            return 0
        if not isinstance(data, dict) or data.get("stamp") != self._stamp():
            return 0
        adopted = 0
        for entry in data.get("products", []):
            try:
                key = (int(entry["rows"]), int(entry["n"]), int(entry["k"]), str(entry["kind"]))
                own, library = float(entry["own_ms"]), float(entry["library_ms"])
            except (KeyError, TypeError, ValueError):
                continue
            if key not in self.ops.wide_choices:
                self.ops.wide_choices[key] = own <= library
                self.ops.wide_timings[key] = (own, library)
                adopted += 1
        return adopted

    def save(self) -> None:
        products = [{"rows": rows, "n": n, "k": k, "kind": kind, "own_ms": own, "library_ms": library}
                    for (rows, n, k, kind), (own, library) in sorted(self.ops.wide_timings.items())]
        try:
            with open(self.path + ".tmp", "w", encoding="utf-8") as handle:
                json.dump({"stamp": self._stamp(), "products": products}, handle)
            os.replace(self.path + ".tmp", self.path)
        except OSError:
            pass  # a folder that cannot be written: the next process times again
