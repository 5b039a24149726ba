"""Loaders for the JSON vectors under tests/golden/reference_fixtures.

Three on-disk formats exist (all plain JSON, data only):

* ``{"meta", "inputs", "outputs"}`` with nested lists           (reference goldens)
* a list of ``{"description", "inputs", "outputs"}`` whose tensors are
  ``{"dtype", "shape", "data": flat list}``                      (selective_scan_reference)
* ``{section: {case: {"inputs", "outputs", "gradients"}}}`` whose tensors are
  ``{"shape", "dtype", "data": nested list}``                    (upstream CUDA vectors)
"""

from __future__ import annotations

import functools
import json
from pathlib import Path

import torch

FIXTURE_DIR = Path(__file__).resolve().parent / "golden" / "reference_fixtures"

_DTYPES = {
    "float32": torch.float32, "float16": torch.float16, "bfloat16": torch.bfloat16,
    "float64": torch.float64, "int32": torch.int32, "int64": torch.int64,
    "uint8": torch.uint8, "bool": torch.bool,
    "torch.float32": torch.float32, "torch.float16": torch.float16,
    "torch.bfloat16": torch.bfloat16, "torch.float64": torch.float64,
    "torch.int32": torch.int32, "torch.int64": torch.int64, "torch.uint8": torch.uint8,
}


def _decode(value):
    if isinstance(value, dict) and "shape" in value and "dtype" in value:
        name = str(value["dtype"])
        if "complex" in name:
            return None  # complex-A cases are outside the supported dtype set
        dtype = _DTYPES[name]
        data = value["data"]
        # serialised through float32 lists; rebuild in fp32/int then cast
        base = torch.float64 if dtype.is_floating_point else dtype
        t = torch.tensor(data, dtype=base).reshape(tuple(value["shape"]))
        return t.to(dtype)
    if isinstance(value, dict):
        return {k: _decode(v) for k, v in value.items()}
    return value


@functools.lru_cache(maxsize=None)
def _raw(name: str):
    return json.loads((FIXTURE_DIR / name).read_text())


def nested_case(name: str):
    """Reference golden in nested-list form -> (inputs, outputs) of fp32 tensors."""
    doc = _raw(name + ".json")

    def conv(v):
        if isinstance(v, list):
            return torch.tensor(v, dtype=torch.float32)
        return v

    return ({k: conv(v) for k, v in doc["inputs"].items()},
            {k: conv(v) for k, v in doc["outputs"].items()},
            doc.get("meta", {}))


def flat_cases(name: str = "selective_scan_reference"):
    out = []
    for entry in _raw(name + ".json"):
        def conv(v):
            if isinstance(v, dict) and {"dtype", "shape", "data"} <= v.keys():
                dt = _DTYPES[str(v["dtype"])]
                return torch.tensor(v["data"], dtype=dt).reshape(tuple(v["shape"]))
            return v
        out.append((entry["description"],
                    {k: conv(v) for k, v in entry["inputs"].items()},
                    {k: conv(v) for k, v in entry["outputs"].items()}))
    return out


def upstream(section: str, case: str):
    """Upstream-CUDA vector -> dict with decoded ``inputs``/``outputs``/``gradients``."""
    doc = _raw("mamba_reference_cases.json")[section][case]
    return {k: _decode(v) for k, v in doc.items()}
