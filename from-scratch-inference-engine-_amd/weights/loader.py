"""Loading by tensor name.

An architecture describes what it expects as a list of ``ParamBinding``: "this parameter of
this part is made of these checkpoint tensors (concatenated along dim 0), stored this way".
The loader compares the expectation with the file, reports *all* missing and unexpected tensors,
wrong shapes and wrong stored dtypes (a weight or vector stored as anything but 32- or 16-bit
floating point, an integer table stored as floating point) in one error, then fills the parts.

Storage on the device:
  * ``matrix``  - the run's compute dtype (bfloat16, or float32 in the 32-bit path);
  * ``vector``  - float32 always (norm weights, biases: exact for either stored precision, so
                  a tensor stored in 32-bit stays so);
  * ``int_table`` - int32.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Sequence, Tuple

import torch

from .safetensors_file import SafetensorsFile


class WeightsError(RuntimeError):
    """The checkpoint does not hold what the architecture expects."""

    def __init__(self, message: str, missing=(), unexpected=(), wrong_shape=(), wrong_dtype=()):
        super().__init__(message)
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        self.wrong_dtype = list(wrong_dtype)


@dataclass(frozen=True)
class TensorSpec:
    """One tensor of the checkpoint.  ``init`` names the distribution of the random-weights
    mode: 'weight' N(0, 0.02), 'norm' 1 + N(0, 0.02), 'bias' N(0, 0.02), 'int' uniform ids."""

    name: str
    shape: Tuple[int, ...]
    init: str = "weight"


@dataclass
class ParamBinding:
    """Parameter ``attr`` of ``owner`` = the sources joined along dim 0 ('concat': one after the
    other; 'interleave': row i of every source in turn), kept as ``storage``."""

    owner: Any
    attr: str
    sources: Sequence[TensorSpec]
    storage: str = "matrix"  # matrix | vector | int_table
    layout: str = "concat"   # concat | interleave


def expected_tensors(bindings: Sequence[ParamBinding]) -> Dict[str, TensorSpec]:
    out: Dict[str, TensorSpec] = {}
    for b in bindings:
        for s in b.sources:
            if s.name in out and out[s.name].shape != s.shape:
                raise ValueError(f"tensor {s.name} is expected with two shapes")
            out[s.name] = s
    return out


# What a stored tensor may be for each kind of parameter.  Weights and vectors are numbers the
# model computes with: 32-bit or 16-bit floating point, as the reference's container accepts
# (include/engine/dtype.hpp:68-79 refuses every other dtype, tests/cpp/test_safetensors.cpp:100);
# an integer, boolean or 64-bit tensor under a weight's name is a wrong file, not a value to cast.
_STORED_AS = {
    "matrix": (torch.float32, torch.float16, torch.bfloat16),
    "vector": (torch.float32, torch.float16, torch.bfloat16),
    "int_table": (torch.int64, torch.int32, torch.int16, torch.int8, torch.uint8),
}


def _dtype_name(dtype: torch.dtype) -> str:
    return str(dtype).replace("torch.", "")


def storage_of(bindings: Sequence[ParamBinding]) -> Dict[str, str]:
    """Checkpoint tensor name -> storage kind of the parameter it goes into."""
    return {s.name: b.storage for b in bindings for s in b.sources}


def check_against(bindings: Sequence[ParamBinding], found: Dict[str, Tuple[int, ...]],
                  ignore_unexpected: Sequence[str] = (),
                  found_dtypes: Optional[Dict[str, torch.dtype]] = None) -> None:
    """Raise one ``WeightsError`` that lists everything wrong: missing and unexpected tensors,
    wrong shapes and (where ``found_dtypes`` gives them) tensors stored in a dtype that their
    parameter cannot mean."""
    expect = expected_tensors(bindings)
    missing = sorted(n for n in expect if n not in found)
    unexpected = sorted(n for n in found if n not in expect and n not in ignore_unexpected)
    wrong = sorted((n, expect[n].shape, tuple(found[n])) for n in expect
                   if n in found and tuple(found[n]) != tuple(expect[n].shape))
    kinds = storage_of(bindings)
    wrong_dtype = sorted((n, kinds[n], found_dtypes[n]) for n in expect
                         if found_dtypes is not None and n in found_dtypes
                         and found_dtypes[n] not in _STORED_AS[kinds[n]])
    if not (missing or unexpected or wrong or wrong_dtype):
        return
    lines = ["checkpoint does not match the model:"]
    if missing:
        lines.append(f"  missing tensors ({len(missing)}):")
        lines += [f"    {n}  expected shape {list(expect[n].shape)}" for n in missing]
    if unexpected:
        lines.append(f"  unexpected tensors ({len(unexpected)}):")
        lines += [f"    {n}  shape {list(found[n])}" for n in unexpected]
    if wrong:
        lines.append(f"  wrong shapes ({len(wrong)}):")
        lines += [f"    {n}  expected {list(e)}, found {list(f)}" for n, e, f in wrong]
    if wrong_dtype:
        lines.append(f"  wrong dtypes ({len(wrong_dtype)}):")
        lines += [f"    {n}  stored as {_dtype_name(d)}, a {k.replace('_', ' ')} must be one of "
                  f"{', '.join(_dtype_name(a) for a in _STORED_AS[k])}" for n, k, d in wrong_dtype]
    raise WeightsError("\n".join(lines), missing, unexpected, wrong, wrong_dtype)


def _to_storage(t: torch.Tensor, storage: str, compute_dtype: torch.dtype) -> torch.dtype:
    if storage == "matrix":
        return compute_dtype
    if storage == "vector":
        return torch.float32
    if storage == "int_table":
        return torch.int32
    raise ValueError(f"unknown storage '{storage}'")


def fill_parts(bindings: Sequence[ParamBinding], get_tensor, compute_dtype: torch.dtype,
               device) -> int:
    """Set every bound parameter; returns the bytes placed on the device.  Bindings with the
    same sources and storage share one device tensor (tied embeddings)."""
    shared: Dict[Tuple, torch.Tensor] = {}
    total = 0
    for b in bindings:
        key = (tuple(s.name for s in b.sources), b.storage, b.layout)
        if key not in shared:
            target = _to_storage(None, b.storage, compute_dtype)
            pieces = []
            for s in b.sources:
                t = get_tensor(s.name)
                if t.dtype not in _STORED_AS[b.storage]:
                    # (a caller that did not go through check_against: the same refusal, one tensor)
                    what = "must hold integers" if b.storage == "int_table" else "must hold 32- or 16-bit floating point"
                    raise WeightsError(f"tensor {s.name} {what}, found {_dtype_name(t.dtype)}",
                                       wrong_dtype=[(s.name, b.storage, t.dtype)])
                pieces.append(t.to(device=device, dtype=target, non_blocking=False))
            if len(pieces) == 1:
                value = pieces[0]
            elif b.layout == "interleave":
                if any(p.shape != pieces[0].shape for p in pieces):
                    raise WeightsError(f"{b.attr}: interleaved sources must have equal shapes")
                value = torch.stack(pieces, dim=1).reshape(-1, *pieces[0].shape[1:])
            elif b.layout == "concat":
                value = torch.cat(pieces, dim=0)
            else:
                raise ValueError(f"unknown layout '{b.layout}'")
            value = value.contiguous()
            shared[key] = value
            total += value.numel() * value.element_size()
        setattr(b.owner, b.attr, shared[key])
    return total


class CheckpointFiles:
    """The tensors of a model folder by name: ``model.safetensors``, or, where that file does not
    exist, the files that ``model.safetensors.index.json`` names (``weight_map``: tensor name ->
    file name, the layout in which large checkpoints are published; the reference reads the single
    file only, src/cuda/model.cu:774).  A tensor that the index sends to a file which does not
    hold it, or a file that holds tensors the index does not send there, is an error."""

    def __init__(self, model_dir):
        import json
        from pathlib import Path

        root = Path(model_dir)
        single, index = root / "model.safetensors", root / "model.safetensors.index.json"
        self._where: Dict[str, SafetensorsFile] = {}
        if single.is_file():
            f = SafetensorsFile(single)
            self._where = {n: f for n in f.names()}
            return
        if not index.is_file():
            raise WeightsError(f"{root}: neither model.safetensors nor model.safetensors.index.json")
        try:
            weight_map = json.loads(index.read_text())["weight_map"]
            assert isinstance(weight_map, dict) and all(isinstance(v, str) for v in weight_map.values())
        except (ValueError, KeyError, AssertionError) as e:
            raise WeightsError(f"{index}: not an index of safetensors files ({e!r})") from None
        files: Dict[str, SafetensorsFile] = {}
        for name, fname in weight_map.items():
            if "/" in fname or "\\" in fname or fname.startswith("."):
                raise WeightsError(f"{index}: file name '{fname}' must lie in the model folder")
            if fname not in files:
                if not (root / fname).is_file():
                    raise WeightsError(f"{index}: names {fname}, which does not exist")
                files[fname] = SafetensorsFile(root / fname)
            if name not in files[fname].names():
                raise WeightsError(f"{index}: sends {name} to {fname}, which does not hold it")
            self._where[name] = files[fname]
        for fname, f in files.items():
            stray = sorted(n for n in f.names() if weight_map.get(n) != fname)
            if stray:
                raise WeightsError(f"{fname} holds tensors the index does not send there: {', '.join(stray[:8])}")

    def names(self):
        return self._where.keys()

    def shape(self, name: str):
        return self._where[name].shape(name)

    def dtype(self, name: str) -> torch.dtype:
        return self._where[name].dtype(name)

    def get(self, name: str) -> torch.Tensor:
        return self._where[name].get(name)


def load_weights(path, bindings: Sequence[ParamBinding], compute_dtype: torch.dtype, device,
                 ignore_unexpected: Sequence[str] = ()) -> int:
    """Check ``path`` (a .safetensors file, or a model folder: see ``CheckpointFiles``) against
    ``bindings`` and fill the parts."""
    import os

    f = CheckpointFiles(path) if os.path.isdir(path) else SafetensorsFile(path)
    check_against(bindings, {n: f.shape(n) for n in f.names()}, ignore_unexpected,
                  {n: f.dtype(n) for n in f.names()})
    return fill_parts(bindings, f.get, compute_dtype, device)
