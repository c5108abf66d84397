"""Fills a model's tensors from a folder, by tensor name.

The architecture gives one table from name patterns of the folder to parameter
paths of the model, with ``#`` standing for a layer's name, in the manner of the
reference's ``weight_maps`` (configs/models/llama/checkpoint.py:94-158;
src/halite/transformers/convert.py:10-54).  Unlike the reference, which drops
unmatched names silently, everything that does not fit is collected and raised
once: tensors the model needs and the folder lacks, tensors the folder holds and
the model does not know, and shapes that differ.

Element types: the 32-bit mode widens everything to float32.  In the bfloat16 mode
a tensor stored in 32-bit stays 32-bit, 16-bit floats become bfloat16, and integer
tables become int32.
"""

from __future__ import annotations

import torch

from ..parts.decoder import Decoder
from .safetensors_io import _NAMES, ModelFiles, SafetensorsError

_FLOATS = {"F32", "BF16", "F16", "F64"}
_INTS = {"I64", "I32", "I16", "I8", "U8"}


class WeightError(ValueError):
    def __init__(self, folder, missing=(), unexpected=(), wrong_shape=(), wrong_dtype=(), other=()):
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        self.wrong_dtype = list(wrong_dtype)
        self.other = list(other)
        lines = [f"weights in {folder} do not fit the model:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        for name, want, got in self.wrong_shape:
            lines.append(f"  wrong shape: {name} is {list(got)}, the model needs {list(want)}")
        for name, got in self.wrong_dtype:
            lines.append(f"  unsupported element type: {name} is {got}")
        lines.extend(f"  {o}" for o in self.other)
        super().__init__("\n".join(lines))


def expand_weight_map(table: dict[str, str], layer_names) -> dict[str, str]:
    """``{tensor name in the folder: parameter path}`` with ``#`` replaced by every
    layer name."""
    out = {}
    for src, dst in table.items():
        if dst is None:
            continue
        if "#" in src or "#" in dst:
            for name in layer_names:
                out[src.replace("#", name)] = dst.replace("#", name)
        else:
            out[src] = dst
    return out


def stored_to_target_dtype(stored: str, engine_dtype: torch.dtype, integer: bool) -> torch.dtype | None:
    if integer:
        return torch.int32 if stored in _INTS else None
    if stored not in _FLOATS:
        return None
    if engine_dtype == torch.float32 or stored in ("F32", "F64"):
        return torch.float32
    return torch.bfloat16


class _TensorDict:
    """Tensors in memory behind the interface of ``ModelFiles``."""

    def __init__(self, tensors: dict[str, torch.Tensor]):
        self.tensors = tensors

    def names(self):
        return list(self.tensors)

    def dtype_of(self, name):
        return _NAMES.get(self.tensors[name].dtype, str(self.tensors[name].dtype))

    def shape_of(self, name):
        return tuple(self.tensors[name].shape)

    def tensor(self, name):
        return self.tensors[name]

    def close(self):
        pass


def load_state_dict(model: Decoder, weight_table: dict[str, str], tensors: dict[str, torch.Tensor]) -> None:
    """The same as ``load_weights`` from tensors in memory, named as in a folder (the
    reference's engine takes new weights this way,
    src/halite/transformers/infer/engine/engine.py:48-52)."""
    _fill(model, weight_table, _TensorDict(tensors), "the given tensors")


def load_weights(model: Decoder, weight_table: dict[str, str], folder: str) -> None:
    try:
        files = ModelFiles(folder)
    except SafetensorsError as e:
        raise WeightError(folder, other=[str(e)]) from e
    _fill(model, weight_table, files, folder)


def _fill(model: Decoder, weight_table: dict[str, str], files, folder: str) -> None:
    try:
        name_to_path = expand_weight_map(weight_table, list(model.spec.layers))
        path_to_name = {v: k for k, v in name_to_path.items()}
        slots = model.param_slots()
        have = set(files.names())
        missing, wrong_shape, wrong_dtype = [], [], []
        known = set()
        dtypes_of_part: dict[int, dict[str, torch.dtype]] = {}
        for slot in slots:
            name = path_to_name.get(slot.path)
            if name is None:
                missing.append(f"{slot.path} (the architecture's table names no tensor for it)")
                continue
            known.add(name)
            if name not in have:
                missing.append(name)
                continue
            if tuple(files.shape_of(name)) != tuple(slot.decl.shape):
                wrong_shape.append((name, slot.decl.shape, files.shape_of(name)))
            target = stored_to_target_dtype(files.dtype_of(name), model.dtype, slot.decl.integer)
            if target is None:
                wrong_dtype.append((name, files.dtype_of(name)))
            dtypes_of_part.setdefault(id(slot.part), {})[slot.name] = target
        passed_over = {k for k, v in weight_table.items() if v is None}
        unexpected = sorted(have - known - passed_over)
        if missing or unexpected or wrong_shape or wrong_dtype:
            raise WeightError(folder, missing, unexpected, wrong_shape, wrong_dtype,
                              other=getattr(files, "notes", ()))

        parts = {id(s.part): s.part for s in slots}
        views = {}
        problems = []
        for pid, part in parts.items():
            try:
                views[pid] = part.allocate(dtypes_of_part[pid])
            except ValueError as e:
                problems.append(str(e))
        if problems:
            raise WeightError(folder, other=problems)
        for slot in slots:
            src = files.tensor(path_to_name[slot.path])
            dst = views[id(slot.part)][slot.name]
            dst.copy_(src)  # converts the element type on the way
        model.finalize()
    finally:
        files.close()
