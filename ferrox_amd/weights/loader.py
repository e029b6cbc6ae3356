"""Binding checkpoint tensors to a model's parameters by name.

The model says which tensors it wants (name, shape); the source says which it
has.  Everything that does not fit — missing tensors, wrong shapes, unusable
dtypes — is collected into ONE `CheckpointError` (the reference stops at the
first: ferrox-models/src/loader.rs:38-65).  Tensors that the file holds and the
model does not ask for are not an error (the reference never looks at them
either: it fetches by name, loader.rs:564-629); they are listed in one
`UnexpectedTensorsWarning`, and in the error if there is one.
Floating tensors are uploaded in the activation type, except that a tensor the
file stores in 32 bits stays float32 under bfloat16 activations; integer tables
become int32.
"""
from __future__ import annotations

import warnings

import torch


class UnexpectedTensorsWarning(UserWarning):
    """The checkpoint holds tensors that the model does not ask for; `names` lists them."""

    def __init__(self, names, where=""):
        self.names = list(names)
        shown = ", ".join(self.names[:12]) + (f", ... and {len(self.names) - 12} more" if len(self.names) > 12 else "")
        super().__init__(f"checkpoint {where} holds {len(self.names)} tensors that the model does not use: {shown}"
                         .replace("  ", " "))


class CheckpointError(ValueError):
    def __init__(self, missing, unexpected, wrong_shape, wrong_dtype, where=""):
        self.missing, self.unexpected = list(missing), list(unexpected)
        self.wrong_shape, self.wrong_dtype = list(wrong_shape), list(wrong_dtype)
        lines = [f"checkpoint {where} does not fit the model:".replace("  ", " ")]

        def show(title, items, fmt=str, limit=12):
            if items:
                lines.append(f"  {title} ({len(items)}):")
                for it in items[:limit]:
                    lines.append("    " + fmt(it))
                if len(items) > limit:
                    lines.append(f"    ... and {len(items) - limit} more")

        show("missing tensors", self.missing)
        show("unexpected tensors", self.unexpected)
        show("wrong shapes", self.wrong_shape, lambda t: f"{t[0]}: file has {list(t[1])}, model wants {list(t[2])}")
        show("unusable dtypes", self.wrong_dtype, lambda t: f"{t[0]}: {t[1]}")
        super().__init__("\n".join(lines))


FLOATS = (torch.float64, torch.float32, torch.float16, torch.bfloat16)
INTS = (torch.int64, torch.int32, torch.int16, torch.int8, torch.uint8)


def check_names(expected: dict, source, where: str = "") -> list:
    """`expected`: full name -> ParamSpec.  Returns the names that the source holds beyond them (after a warning
    that lists them)."""
    have = set(source.names())
    missing = sorted(n for n in expected if n not in have)
    unexpected = sorted(n for n in have if n not in expected)
    wrong_shape, wrong_dtype = [], []
    for n, spec in expected.items():
        if n not in have:
            continue
        dt, shape = source.info(n)
        if tuple(shape) != tuple(spec.shape):
            wrong_shape.append((n, tuple(shape), tuple(spec.shape)))
        if spec.integer and dt not in INTS:
            wrong_dtype.append((n, f"stored as {dt}, the model wants an integer table"))
        if not spec.integer and dt not in FLOATS:
            wrong_dtype.append((n, f"stored as {dt}, the model wants floating point"))
    if missing or wrong_shape or wrong_dtype:
        raise CheckpointError(missing, unexpected, wrong_shape, wrong_dtype, where)
    if unexpected:
        warnings.warn(UnexpectedTensorsWarning(unexpected, where), stacklevel=2)
    return unexpected


def resident_dtype(stored: torch.dtype, act_dtype: torch.dtype) -> torch.dtype:
    if stored in INTS:
        return torch.int32
    if act_dtype == torch.float32:
        return torch.float32
    return torch.float32 if stored in (torch.float32, torch.float64) else act_dtype


def upload(source, name: str, act_dtype: torch.dtype, device) -> torch.Tensor:
    t = source.tensor(name)
    want = resident_dtype(t.dtype, act_dtype)
    t = t.to(device)                          # as stored; converted on the device
    if t.dtype != want:
        t = t.to(want)
    return t.contiguous()
