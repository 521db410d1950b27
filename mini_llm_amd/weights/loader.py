"""Weights by tensor name: checks a file against what the model's parts expect, reports every
problem in one error, and hands each tensor to its part in the layout and precision it runs in.

The reference reads one raw float32 file per tensor name and fails the whole load on a missing
file or a wrong size (engine/src/tensor_loading.c:8-50, engine/src/gpt2.c:113-152)."""

from __future__ import annotations

import warnings
from pathlib import Path

import torch

from .safetensors_io import SafetensorsError, SafetensorsFile
from .spec import INT_TABLE, MATRIX, TABLE, VECTOR, TensorSpec

WEIGHTS_FILE = "model.safetensors"


class WeightsError(ValueError):
    """Lists everything that is wrong with a weights file at once."""

    def __init__(self, where, missing=(), unexpected=(), wrong_shape=(), other=()):
        self.missing, self.unexpected = sorted(missing), sorted(unexpected)
        self.wrong_shape, self.other = sorted(wrong_shape), list(other)
        lines = [f"weights in {where} do not fit the model:"]
        if self.missing:
            lines.append(f"  missing ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong_shape:
            lines.append(f"  wrong shape ({len(self.wrong_shape)}): " + ", ".join(f"{n} is {list(got)}, expected {list(want)}" for n, got, want in self.wrong_shape))
        lines += [f"  {text}" for text in self.other]
        super().__init__("\n".join(lines))


def check_names(where, expected: dict, found: dict, canonical) -> dict:
    """expected: name -> TensorSpec; found: name in file -> (shape, is_float). Returns
    name -> name in file, or raises one WeightsError with all problems."""
    mapping, unexpected, other = {}, [], []
    for file_name in found:
        name = canonical(file_name)
        if name is None:
            continue  # a tensor the architecture knows and does not need (a mask, a tied copy)
        if name not in expected:
            unexpected.append(file_name)
        elif name in mapping:
            other.append(f"{file_name} and {mapping[name]} both name {name}")
        else:
            mapping[name] = file_name
    missing = [n for n in expected if n not in mapping]
    wrong = []
    for name, file_name in mapping.items():
        shape, is_float = found[file_name]
        spec = expected[name]
        if tuple(shape) != tuple(spec.shape):
            wrong.append((file_name, tuple(shape), tuple(spec.shape)))
        elif (spec.role == INT_TABLE) == is_float:
            other.append(f"{file_name} holds {'floats' if is_float else 'integers'}, which a {spec.role} cannot be")
    if missing or unexpected or wrong or other:
        raise WeightsError(where, missing, unexpected, wrong, other)
    return mapping


def place(tensor: torch.Tensor, spec: TensorSpec, precision, device) -> torch.Tensor:
    """A stored tensor as the part keeps it: on the device, in its role's element type, and
    transposed where the spec says so. Vectors stay (or become) 32-bit; a tensor stored in
    32-bit is only narrowed if it is a matrix or a table of a bfloat16 run."""
    tensor = tensor.to(device)
    if spec.role == INT_TABLE:
        return tensor.to(torch.int32).contiguous()
    if spec.role == VECTOR:
        target = precision.vector
    elif spec.role in (MATRIX, TABLE):
        target = precision.compute
    else:
        raise ValueError(f"unknown tensor role {spec.role!r}")
    if tensor.is_cuda and tensor.dtype in (torch.float32, torch.bfloat16) and tensor.dim() in (1, 2):
        from ..ops import kernels  # on the GPU the conversion and the transpose are this framework's kernels

        if spec.role == MATRIX and tensor.dim() == 2:  # operands of matrix products are kept in the packed layout
            return kernels.pack_matrix(tensor.contiguous(), target, transpose=spec.keep_transposed)
        return kernels.convert(tensor.contiguous(), target, transpose=spec.keep_transposed)
    tensor = tensor.to(target)  # other stored types (F16, F64) and host-only checks of the loader
    if spec.keep_transposed:
        tensor = tensor.t()
    return tensor.contiguous()


def bind_tensors(model, tensors: dict, device) -> None:
    """tensors: canonical name -> stored-layout tensor (any device). Checks and binds them."""
    expected = model.named_tensor_specs()
    found = {n: (tuple(t.shape), t.is_floating_point()) for n, t in tensors.items()}
    mapping = check_names("the given tensors", expected, found, lambda n: n)
    model.bind_named({name: place(tensors[mapping[name]], expected[name], model.precision, device) for name in expected})


def load_weights(model, model_dir, device) -> None:
    """Reads model.safetensors of the folder into the model's parts."""
    path = Path(model_dir) / WEIGHTS_FILE
    try:
        file = SafetensorsFile(path)
    except SafetensorsError as error:
        raise WeightsError(path, other=[str(error)]) from None
    expected = model.named_tensor_specs()
    found = {n: (file.shape(n), file.dtype(n).is_floating_point) for n in file.names()}
    mapping = check_names(path, expected, found, model.canonical_tensor_name)
    placed = {}
    with warnings.catch_warnings():
        warnings.simplefilter("ignore", UserWarning)  # the mapped file is read-only; it is only read
        for name, spec in expected.items():
            placed[name] = place(file.tensor(mapping[name]), spec, model.precision, device)
    model.bind_named(placed)
