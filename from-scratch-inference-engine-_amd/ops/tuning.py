"""The library matrix product of the bfloat16 path, with optional selection of the library's kernel.

For many rows (prefill) the engine hands x . W^T to the vendor library through ``torch.mm`` (the
reference's engine calls cuBLAS there).  The library picks one of its kernels by a heuristic; its
other kernels are sometimes a fifth or a quarter faster.  With tuning on,
torch's TunableOp times the library's candidates the first time a shape is seen and keeps the
best (in the process, and in a file under the temporary folder for later ones).  Each new shape
costs seconds (at 16,384 rows, minutes), so only two kinds of row counts are tuned: multiples of 256
up to 4,096 (a full token budget of prefill), multiples of 16 up to 128 and of 32 up to 256 (decode batches, timed in the eager run that precedes the
capture of their graph); never inside a graph capture.  Other shapes use what has been found for
them, or the heuristic.
"""

from __future__ import annotations

import hashlib

import torch

from ..csrc.build import private_tmp_dir

_TUNED_ROWS, _TUNED_MAX_ROWS = 256, 4096
_TUNED_DECODE_ROWS, _TUNED_DECODE_MAX = 16, 64   # decode batches are padded to these row counts ...
_TUNED_LARGE_ROWS, _TUNED_LARGE_MAX = 32, 256    # ... and, beyond 64 rows, to these
_TUNED_TILES_MAX = 128                           # (and to multiples of 16 up to here)
_state = {"on": False}


def enable_library_tuning(max_ms_per_candidate: int = 30, iterations: int = 10) -> None:
    import torch.cuda.tunable as tunable

    tunable.enable(True)
    tunable.tuning_enable(False)
    tunable.set_max_tuning_duration(int(max_ms_per_candidate))
    tunable.set_max_tuning_iterations(int(iterations))
    # torch also keeps the results in a file, from which a later process starts: it goes to a
    # private per-user folder under the temporary directory (the working directory may be
    # read-only), named for the device and the library versions the timings belong to; without
    # such a folder the results stay in the process
    folder = private_tmp_dir("fsie-tunableop")
    if folder is not None:
        what = f"{torch.cuda.get_device_name(0) if torch.cuda.is_available() else 'none'}|{torch.__version__}|{torch.version.hip}"
        tunable.set_filename(str(folder / f"results-{hashlib.sha256(what.encode()).hexdigest()[:12]}.csv"))
    elif hasattr(tunable, "write_file_on_exit"):
        tunable.write_file_on_exit(False)
    _state["on"] = True


def disable_library_tuning() -> None:
    import torch.cuda.tunable as tunable

    tunable.tuning_enable(False)
    tunable.enable(False)
    _state["on"] = False


def library_tuning_enabled() -> bool:
    return _state["on"]


def library_mm(x: torch.Tensor, weight: torch.Tensor, float32_result: bool = False) -> torch.Tensor:
    """x [M, K] . weight [N, K]^T by the library, float32 accumulation; the result in the operands'
    dtype, or in float32 (not rounded in between) with ``float32_result``."""
    if float32_result:
        return torch.mm(x, weight.t(), out_dtype=torch.float32)
    if not _state["on"]:
        return torch.mm(x, weight.t())
    import torch.cuda.tunable as tunable

    rows = x.shape[0]
    tune = (((rows % _TUNED_ROWS == 0 and rows <= _TUNED_MAX_ROWS)
             or (rows <= _TUNED_DECODE_MAX and rows % _TUNED_DECODE_ROWS == 0)
             or (rows <= _TUNED_LARGE_MAX and rows % _TUNED_LARGE_ROWS == 0)
             or (rows <= _TUNED_TILES_MAX and rows % _TUNED_DECODE_ROWS == 0)) and rows > 0
            and not torch.cuda.is_current_stream_capturing())
    if not tune:
        return torch.mm(x, weight.t())
    tunable.tuning_enable(True)
    try:
        return torch.mm(x, weight.t())
    finally:
        tunable.tuning_enable(False)
