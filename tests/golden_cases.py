"""Loader for the committed golden fixtures (tests/golden/*.npz)."""
from __future__ import annotations

import os
from dataclasses import dataclass
from typing import Optional, Tuple

import numpy as np

from cubek_amd.scheme import (ElemType, QuantLevel, QuantParam, QuantScheme, QuantStore,
                              QuantValue)

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
_ELEM = {"f32": ElemType.F32, "f16": ElemType.F16, "bf16": ElemType.BF16}
_PARAM = {"f32": QuantParam.F32, "f16": QuantParam.F16, "bf16": QuantParam.BF16}


@dataclass
class GoldenCase:
    name: str
    elem: ElemType
    scheme: QuantScheme
    shape: Tuple[int, ...]
    scale_strides: Tuple[int, ...]
    x: np.ndarray          # storage bits of the input (float32 view for f32)
    scale: np.ndarray      # scale buffer typed like the input
    words: np.ndarray      # expected packed u32 words (native store: bytes)
    out_scale: np.ndarray  # expected out_scale buffer (param dtype bits)
    deq: np.ndarray        # expected dequantized storage bits


def _as_storage(bits: np.ndarray, elem: ElemType) -> np.ndarray:
    if elem == ElemType.F32:
        return bits.astype(np.uint32).view(np.float32)
    return bits.astype(np.uint16)


def load(file: str):
    z = np.load(os.path.join(GOLDEN, file), allow_pickle=False)
    names = sorted({k.split("/")[0] for k in z.files})
    out = []
    for n in names:
        fmt, value, param, shape, block, strides, *store = [str(s) for s in z[f"{n}/meta"]]
        native = store == ["native"]
        shape = tuple(int(v) for v in shape.split(","))
        level = QuantLevel.Tensor if not block else QuantLevel.block([int(v) for v in block.split(",")])
        scheme = (QuantScheme.default().with_level(level).with_value(QuantValue[value])
                  .with_store(QuantStore.Native if native else QuantStore.U32).with_param(_PARAM[param]))
        elem = _ELEM[fmt]
        out.append(GoldenCase(
            name=n, elem=elem, scheme=scheme, shape=shape,
            scale_strides=tuple(int(v) for v in strides.split(",")),
            x=_as_storage(z[f"{n}/x"], elem), scale=_as_storage(z[f"{n}/scale"], elem),
            words=z[f"{n}/words"].astype(np.uint8 if native else np.uint32),
            out_scale=_as_storage(z[f"{n}/out_scale"], _ELEM[param]),
            deq=_as_storage(z[f"{n}/deq"], elem)))
    return out


def bits_equal(a: np.ndarray, b: np.ndarray) -> bool:
    """Bit-for-bit equality of two storage arrays."""
    a = np.ascontiguousarray(a).reshape(-1)
    b = np.ascontiguousarray(b).reshape(-1)
    if a.dtype == np.float32:
        a = a.view(np.uint32)
    if b.dtype == np.float32:
        b = b.view(np.uint32)
    return a.shape == b.shape and bool(np.array_equal(a, b))
