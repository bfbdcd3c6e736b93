"""Weights from safetensors, by tensor name.

File layouts are the reference's: ``model.safetensors``, or
``model.safetensors.index.json`` with ``{"weight_map": {tensor: shard}}``
(src/transformers/modeling_utils.py:3680-3695, src/transformers/utils/hub.py:1071-1085).
Unlike the reference, which only warns about missing and unexpected keys
(modeling_utils.py:4895-4914) and raises on the first class of shape mismatch
(:4884-4893), every problem is collected and raised as one ``WeightsError``.

Kept from the reference: a file saved from the bare base model lacks the
``transformer.`` prefix and still loads (modeling_utils.py:4495-4512); a tied
head may be absent (:4546-4554); stale ``rotary_emb.inv_freq`` buffers are
ignored (:4529-4532).
"""
from __future__ import annotations

import json
import os
from typing import Dict, Iterable, List, Mapping, Optional, Sequence

import torch

from ..engine.spec import INT, MATRIX, VECTOR, TensorSpec

SAFE_WEIGHTS_NAME = "model.safetensors"  # src/transformers/utils/__init__.py:261
SAFE_WEIGHTS_INDEX_NAME = "model.safetensors.index.json"  # :262

_IGNORED_SUFFIXES = ("rotary_emb.inv_freq",)
_FLOAT_DTYPES = (torch.float32, torch.bfloat16, torch.float16, torch.float64)


class WeightsError(RuntimeError):
    """Missing, unexpected, wrongly shaped or wrongly typed tensors, all listed."""

    def __init__(self, folder, missing=(), unexpected=(), wrong_shape=(), wrong_type=()):
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        self.wrong_type = list(wrong_type)
        lines = [f"cannot load weights from {folder!r}:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong_shape:
            lines.append(f"  wrong shapes ({len(self.wrong_shape)}): " + "; ".join(
                f"{n}: file has {tuple(got)}, model needs {tuple(want)}" for n, got, want in self.wrong_shape))
        if self.wrong_type:
            lines.append(f"  wrong types ({len(self.wrong_type)}): " + "; ".join(
                f"{n}: file has {got}, model needs {want}" for n, got, want in self.wrong_type))
        super().__init__("\n".join(lines))


def resolve_files(folder: str) -> Dict[str, str]:
    """tensor name -> file path, for either layout."""
    from safetensors import safe_open

    single = os.path.join(folder, SAFE_WEIGHTS_NAME)
    index = os.path.join(folder, SAFE_WEIGHTS_INDEX_NAME)
    if os.path.isfile(single):
        with safe_open(single, framework="pt") as f:
            _check_metadata(single, f.metadata())
            return {k: single for k in f.keys()}
    if os.path.isfile(index):
        with open(index, "r", encoding="utf-8") as f:
            weight_map = json.load(f)["weight_map"]
        out = {}
        for name, shard in weight_map.items():
            path = os.path.join(folder, shard)
            if not os.path.isfile(path):
                raise FileNotFoundError(f"{index} names shard {shard!r}, which is not in {folder!r}")
            out[name] = path
        return out
    # modeling_utils.py:3716-3740
    raise FileNotFoundError(f"Error no file named {SAFE_WEIGHTS_NAME} or {SAFE_WEIGHTS_INDEX_NAME} found in directory {folder}.")


def _check_metadata(path, metadata) -> None:
    # modeling_utils.py:502-511
    if metadata is not None and metadata.get("format", "pt") not in ("pt", "tf", "flax", "mlx"):
        raise OSError(f"The safetensors archive passed at {path} does not contain the valid metadata.")


def _strip_or_add_prefix(file_names: Iterable[str], wanted: Sequence[str], prefix: str) -> Dict[str, str]:
    """model tensor name -> file tensor name, trying the name with and without ``prefix``."""
    file_names = set(file_names)
    out = {}
    for w in wanted:
        if w in file_names:
            out[w] = w
        elif prefix and w.startswith(prefix) and w[len(prefix):] in file_names:
            out[w] = w[len(prefix):]
    return out


def first_float_dtype(folder: str) -> Optional[torch.dtype]:
    """The type of the first floating-point tensor of the weight files (what ``dtype="auto"`` falls back on,
    src/transformers/modeling_utils.py:4030-4041), read from the files' headers."""
    from safetensors import safe_open

    names = {"F64": torch.float64, "F32": torch.float32, "F16": torch.float16, "BF16": torch.bfloat16}
    files = resolve_files(folder)
    for path in sorted(set(files.values())):
        with safe_open(path, framework="pt") as f:
            for k in f.keys():
                dt = names.get(f.get_slice(k).get_dtype())
                if dt is not None:
                    return dt
    return None


def device_dtype_for(spec: TensorSpec, compute_dtype: torch.dtype) -> torch.dtype:
    if spec.kind == MATRIX:
        return compute_dtype
    if spec.kind == VECTOR:
        return torch.float32
    if spec.kind == INT:
        return torch.int32
    raise ValueError(f"unknown tensor kind {spec.kind!r}")


def place(spec: TensorSpec, t: torch.Tensor, compute_dtype: torch.dtype, device) -> torch.Tensor:
    """Convert a file tensor to how the device holds it (round to nearest even when narrowing)."""
    return t.to(device=device, dtype=device_dtype_for(spec, compute_dtype)).contiguous()


def load_weights(folder: str, specs: Sequence[TensorSpec], compute_dtype: torch.dtype, device,
                 *, base_prefix: str = "", strict: bool = True) -> Dict[str, torch.Tensor]:
    """Read every tensor of ``specs`` from ``folder``; raise one WeightsError naming all problems.  ``base_prefix``
    is what the model's tensor names start with when the whole model was saved; a file saved from the body alone
    lacks it and loads too."""
    from safetensors import safe_open

    files = resolve_files(folder)
    by_name = {s.name: s for s in specs}
    mapping = _strip_or_add_prefix(files.keys(), list(by_name), base_prefix)
    # A tensor that is tied to another one is that other one, whatever the file holds under its name: the reference
    # ties after it has loaded (src/transformers/modeling_utils.py:1858-1884 called from :4368), which overwrites a
    # head that a file of a tied model carries.  The file's copy is neither read nor unexpected.
    tied_in_file = {mapping.pop(s.name) for s in specs if s.tied_to is not None and s.name in mapping}
    # A tensor that the file does not hold under its own name may lie there in pieces
    in_pieces = {s.name: _strip_or_add_prefix(files.keys(), [n for n, _ in s.pieces], base_prefix)
                 for s in specs if s.pieces and s.name not in mapping}

    used_file_names = set(mapping.values()) | {f for found in in_pieces.values() for f in found.values()}
    unexpected = sorted(k for k in files if k not in used_file_names and k not in tied_in_file
                        and not k.endswith(_IGNORED_SUFFIXES))
    missing = []
    for s in specs:
        if s.name in mapping:
            continue
        if s.tied_to is not None and s.tied_to in mapping:
            continue
        if s.name in in_pieces and in_pieces[s.name]:  # some pieces are there: the others are what is missing
            missing.extend(n for n, _ in s.pieces if n not in in_pieces[s.name])
            continue
        missing.append(s.name if not s.pieces else f"{s.name} (or its pieces {', '.join(n for n, _ in s.pieces)})")

    wrong_shape, wrong_type = [], []
    handles = {}
    out: Dict[str, torch.Tensor] = {}

    def read(spec, name, fname, shape):
        """The file tensor ``fname`` if it has ``shape`` and the kind of ``spec``; else None, with the problem noted."""
        path = files[fname]
        if path not in handles:
            handles[path] = safe_open(path, framework="pt")
            _check_metadata(path, handles[path].metadata())
        got = tuple(handles[path].get_slice(fname).get_shape())
        if got != tuple(shape):
            wrong_shape.append((name, got, tuple(shape)))
            return None
        t = handles[path].get_tensor(fname)
        if (spec.kind == INT) == (t.dtype in _FLOAT_DTYPES):
            wrong_type.append((name, str(t.dtype).replace("torch.", ""), "integer" if spec.kind == INT else "floating point"))
            return None
        return t

    try:
        for s in specs:
            fname = mapping.get(s.name)
            if fname is not None:
                t = read(s, s.name, fname, s.shape)
            elif s.name in in_pieces and len(in_pieces[s.name]) == len(s.pieces):
                parts = [read(s, n, in_pieces[s.name][n], shape) for n, shape in s.pieces]
                if any(part is None for part in parts):
                    continue
                t = s.assemble(parts) if s.assemble is not None else torch.cat(parts, dim=0)
                if tuple(t.shape) != tuple(s.shape):
                    raise ValueError(f"the pieces of {s.name} make a tensor of shape {tuple(t.shape)}, the model needs "
                                     f"{tuple(s.shape)}: the model's own description of its pieces is wrong")
            else:
                continue
            if t is None:
                continue
            out[s.name] = place(s, t, compute_dtype, device)
            del t
    finally:
        handles.clear()

    if missing or wrong_shape or wrong_type or (unexpected and strict):
        raise WeightsError(folder, missing, unexpected if strict else (), wrong_shape, wrong_type)
    if unexpected:
        import warnings
        warnings.warn(f"tensors in {folder!r} that the model does not use: {', '.join(unexpected)}")
    for s in specs:  # tied tensors share storage
        if s.name not in out and s.tied_to is not None:
            out[s.name] = out[s.tied_to]
    return out


def save_weights(folder: str, tensors: Mapping[str, torch.Tensor], *, shards: int = 1,
                 skip: Optional[Iterable[str]] = None) -> List[str]:
    """Write ``tensors`` as model.safetensors, or as ``shards`` files plus the index."""
    from safetensors.torch import save_file

    os.makedirs(folder, exist_ok=True)
    skip = set(skip or ())
    items = [(k, v.detach().to("cpu").contiguous()) for k, v in tensors.items() if k not in skip]
    meta = {"format": "pt"}
    if shards <= 1:
        path = os.path.join(folder, SAFE_WEIGHTS_NAME)
        save_file(dict(items), path, metadata=meta)
        return [path]
    per = (len(items) + shards - 1) // shards
    weight_map, paths = {}, []
    for i in range(shards):
        chunk = items[i * per:(i + 1) * per]
        if not chunk:
            continue
        fname = f"model-{i + 1:05d}-of-{shards:05d}.safetensors"
        save_file(dict(chunk), os.path.join(folder, fname), metadata=meta)
        paths.append(os.path.join(folder, fname))
        for k, _ in chunk:
            weight_map[k] = fname
    total = sum(v.numel() * v.element_size() for _, v in items)
    with open(os.path.join(folder, SAFE_WEIGHTS_INDEX_NAME), "w", encoding="utf-8") as f:
        json.dump({"metadata": {"total_size": total}, "weight_map": weight_map}, f, indent=2, sort_keys=True)
    return paths
