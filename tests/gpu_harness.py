"""Runs the HIP path through the package API on numpy inputs (GPU tests only).

torch owns the device memory; every compute call goes through the C ABI of
libcubek_quant_hip.so.
"""
from __future__ import annotations

import numpy as np
import torch

import cubek_amd
from cubek_amd import ComputeClient, ElemType, QuantScheme, QuantStore, TensorHandleRef
from cubek_amd import dequantize as cq_dequantize
from cubek_amd import quantize as cq_quantize

DEV = "cuda"
_PARAM_ELEM = {cubek_amd.QuantParam.F32: ElemType.F32, cubek_amd.QuantParam.F16: ElemType.F16,
               cubek_amd.QuantParam.BF16: ElemType.BF16}


def param_elem(scheme: QuantScheme) -> ElemType:
    return _PARAM_ELEM[scheme.param]


def to_dev(a: np.ndarray) -> torch.Tensor:
    """numpy storage array (float32 / uint16 / uint32 / uint8) -> device tensor of equal width."""
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16)).to(DEV)
    if a.dtype == np.uint32:
        return torch.from_numpy(a.view(np.int32)).to(DEV)
    return torch.from_numpy(a).to(DEV)


def to_host(t: torch.Tensor, like=None) -> np.ndarray:
    """device tensor -> numpy storage array (int16 -> uint16 bits, int32 -> uint32 words)."""
    a = t.cpu().numpy()
    if a.dtype == np.int16:
        return a.view(np.uint16)
    if a.dtype == np.int32:
        return a.view(np.uint32)
    return a


def storage_dtype(elem: ElemType) -> torch.dtype:
    return torch.float32 if elem == ElemType.F32 else torch.int16


def handle(t: torch.Tensor, shape=None, strides=None) -> TensorHandleRef:
    h = TensorHandleRef.from_torch(t)
    if shape is not None:
        h = TensorHandleRef(h.handle, tuple(shape), tuple(strides), h.elem_size)
    return h


def contiguous_strides(shape):
    st, acc = [], 1
    for s in reversed(shape):
        st.append(acc)
        acc *= s
    return tuple(reversed(st))


def _check_reach(shape, strides, available: int) -> None:
    """The C ABI trusts its pointers: never hand it a layout that leaves the buffer."""
    reach = 1 + sum((n - 1) * st for n, st in zip(shape, strides))
    assert reach <= available, f"scale buffer of {available} entries, layout reaches {reach}"


def _stored_dtype(scheme: QuantScheme):
    return torch.int32 if scheme.store == QuantStore.U32 else torch.uint8


def quantize(x: np.ndarray, elem: ElemType, shape, scale: np.ndarray, scheme: QuantScheme,
             scale_shape=None, scale_strides=None, out_scale_strides=None):
    """cq_quantize.  ``scale`` is the raw scale buffer (typed ``elem``); strided
    layouts pass the logical shape/strides separately."""
    client = ComputeClient.current()
    dx = to_dev(x.reshape(shape))
    dscale = to_dev(scale.reshape(-1))
    sshape = tuple(scale_shape) if scale_shape is not None else scheme.scales_shape(shape)
    sstr = tuple(scale_strides) if scale_strides is not None else contiguous_strides(sshape)
    ostr = tuple(out_scale_strides) if out_scale_strides is not None else sstr
    _check_reach(sshape, sstr, dscale.numel())
    _check_reach(sshape, ostr, dscale.numel())
    pe = param_elem(scheme)
    dout_scale = torch.zeros(dscale.numel(), dtype=storage_dtype(pe), device=DEV)
    pshape = scheme.packed_shape(shape)
    dout = torch.zeros(pshape, dtype=_stored_dtype(scheme), device=DEV)
    cq_quantize.launch_ref(client, handle(dx), handle(dout), handle(dscale, sshape, sstr),
                           handle(dout_scale, sshape, ostr), scheme, elem)
    torch.cuda.synchronize()
    words = to_host(dout, np.uint32)
    return words, to_host(dout_scale, np.float32 if pe == ElemType.F32 else np.uint16)


def dequantize(values: np.ndarray, shape, params: np.ndarray, elem: ElemType, scheme: QuantScheme,
               scale_shape=None, scale_strides=None) -> np.ndarray:
    client = ComputeClient.current()
    dv = to_dev(values.reshape(scheme.packed_shape(shape)))
    dp = to_dev(params.reshape(-1))
    sshape = tuple(scale_shape) if scale_shape is not None else scheme.scales_shape(shape)
    sstr = tuple(scale_strides) if scale_strides is not None else contiguous_strides(sshape)
    _check_reach(sshape, sstr, dp.numel())
    dout = torch.zeros(tuple(shape), dtype=storage_dtype(elem), device=DEV)
    cq_dequantize.launch_ref(client, handle(dv), handle(dout), handle(dp, sshape, sstr), scheme, elem)
    torch.cuda.synchronize()
    return to_host(dout, np.float32)


def workspace(scheme: QuantScheme, n: int):
    nbytes = cq_quantize.workspace_bytes(scheme, n)
    ws = torch.empty(max(nbytes, 4), dtype=torch.uint8, device=DEV)
    return ws, nbytes


def compute_scales(x: np.ndarray, elem: ElemType, shape, scheme: QuantScheme) -> np.ndarray:
    client = ComputeClient.current()
    dx = to_dev(x.reshape(shape))
    sshape = scheme.scales_shape(shape)
    ds = torch.zeros(sshape, dtype=storage_dtype(elem), device=DEV)
    ws, nbytes = workspace(scheme, int(np.prod(shape)))
    cq_quantize.compute_scales(client, handle(dx), handle(ds), scheme, elem, ws.data_ptr(), nbytes)
    torch.cuda.synchronize()
    return to_host(ds, np.float32)


def quantize_dynamic(x: np.ndarray, elem: ElemType, shape, scheme: QuantScheme):
    client = ComputeClient.current()
    dx = to_dev(x.reshape(shape))
    sshape = scheme.scales_shape(shape)
    pe = param_elem(scheme)
    dos = torch.zeros(sshape, dtype=storage_dtype(pe), device=DEV)
    dout = torch.zeros(scheme.packed_shape(shape), dtype=_stored_dtype(scheme), device=DEV)
    ws, nbytes = workspace(scheme, int(np.prod(shape)))
    cq_quantize.launch_dynamic(client, handle(dx), handle(dout), handle(dos), scheme, elem,
                               ws.data_ptr(), nbytes)
    torch.cuda.synchronize()
    return to_host(dout, np.uint32), to_host(dos, np.float32)
