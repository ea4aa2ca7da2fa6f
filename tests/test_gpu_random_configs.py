"""Seeded random configurations (rank, shape, block, value, store, scale parameter,
float type, memory layout of both value tensors) through every entry point, each
compared with the oracle on the contiguous copy.  Complements the hand-picked cases:
whatever kernel the dispatch picks (flat, fused block, row, per-element) must agree."""
import os
import zlib

import numpy as np
import pytest
from numpy.lib.stride_tricks import as_strided

from cubek_amd import (ComputeClient, ElemType, QuantLevel, QuantParam, QuantScheme, QuantStore, QuantValue)
from cubek_amd import dequantize as dq
from cubek_amd import quantize as qz

pytestmark = pytest.mark.gpu

VALUES_U32 = [QuantValue.Q8F, QuantValue.Q8S, QuantValue.Q4F, QuantValue.Q4S, QuantValue.Q2F, QuantValue.Q2S,
              QuantValue.E2M1, QuantValue.E4M3, QuantValue.E5M2, QuantValue.E2M1_OCP]
VALUES_NATIVE = [QuantValue.Q8F, QuantValue.Q8S, QuantValue.E4M3, QuantValue.E5M2, QuantValue.E2M1, QuantValue.E2M1_OCP]


@pytest.fixture(scope="module")
def gpu():
    import gpu_harness

    return gpu_harness


def reach(shape, strides):
    return 1 + sum((n - 1) * st for n, st in zip(shape, strides))


def view(buf, shape, strides):
    assert reach(shape, strides) <= buf.size
    return as_strided(buf, shape, tuple(st * buf.itemsize for st in strides))


def pick(rng, options):
    return options[int(rng.integers(len(options)))]


def random_layout(rng, shape):
    """Strides for `shape`: contiguous, padded rows, permuted leading dimensions, or fully permuted."""
    rank = len(shape)
    kind = pick(rng, ["contiguous", "contiguous", "pitched", "leading_permuted", "permuted"])
    order = list(range(rank))  # memory order, slowest first
    pad = 0
    if kind == "pitched":
        pad = pick(rng, [4, 8, 16, 3])
    elif kind == "leading_permuted" and rank >= 3:
        lead = order[:-1]
        rng.shuffle(lead)
        order = lead + [rank - 1]
        pad = pick(rng, [0, 8])
    elif kind == "permuted" and rank >= 2:
        rng.shuffle(order)
    strides, acc = [0] * rank, 1
    for i, d in enumerate(reversed(order)):
        strides[d] = acc
        acc *= shape[d] + (pad if i == 0 else 0)
    return kind, tuple(strides)


def random_case(rng):
    store = QuantStore.U32 if rng.random() < 0.7 else QuantStore.Native
    value = pick(rng, VALUES_U32 if store == QuantStore.U32 else VALUES_NATIVE)
    elem = pick(rng, [ElemType.F32, ElemType.BF16, ElemType.F16])
    param = pick(rng, [QuantParam.F32, QuantParam.F32, QuantParam.BF16 if elem != ElemType.F16 else QuantParam.F16])
    scheme = QuantScheme.default().with_value(value).with_store(store).with_param(param)
    nq = scheme.num_quants()
    rank = int(rng.integers(1, 5))
    if rng.random() < 0.25:  # per tensor
        shape = [int(rng.integers(1, 7)) for _ in range(rank - 1)] + [nq * int(rng.integers(1, 40))]
        if rng.random() < 0.2:
            shape[-1] *= 64
        return scheme, elem, tuple(shape)
    # block level: the last block extent is a multiple of the values per stored element and of the
    # line the reference's native kernels would pick (16 bytes of the float type at most)
    unit = max(nq, 16 // (4 if elem == ElemType.F32 else 2)) if store == QuantStore.Native else nq
    block_rank = int(rng.integers(1, min(rank, 3) + 1))
    block = [pick(rng, [1, 2, 3, 4, 8, 16]) for _ in range(block_rank - 1)]
    block.append(unit * pick(rng, [1, 2, 3, 4, 8]))
    block = [min(b, 255) for b in block]
    if block[-1] % unit:
        block[-1] = unit
    padded = [1] * (rank - block_rank) + block
    big = rng.random() < 0.2  # now and then more than one workgroup tile in both directions
    shape = [b * int(rng.integers(1, (5 if i < rank - 1 else 9) * (8 if big and i >= rank - 2 else 1)))
             for i, b in enumerate(padded)]
    while int(np.prod(shape)) > (1 << 21):  # keep the oracle fast
        d = int(np.argmax([s // b for s, b in zip(shape, padded)]))
        shape[d] = max(padded[d], (shape[d] // padded[d] // 2) * padded[d])
    return scheme.with_level(QuantLevel.block(block)), elem, tuple(shape)


def random_long_rows_case(rng):
    """Rows of 256 - 1300 sixteen-byte chunks (or a few short ones) behind one to three leading dimensions, one scale
    per tensor or 1-D power-of-two blocks: the layouts the streaming kernels take over row steps or lane by lane."""
    store = QuantStore.U32 if rng.random() < 0.7 else QuantStore.Native
    value = pick(rng, VALUES_U32 if store == QuantStore.U32 else VALUES_NATIVE)
    elem = pick(rng, [ElemType.F32, ElemType.BF16, ElemType.F16])
    param = pick(rng, [QuantParam.F32, QuantParam.F32, QuantParam.BF16 if elem != ElemType.F16 else QuantParam.F16])
    scheme = QuantScheme.default().with_value(value).with_store(store).with_param(param)
    per_chunk = 4 if elem == ElemType.F32 else 8
    unit = max(scheme.num_quants(), per_chunk)
    block = unit * pick(rng, [1, 2, 4, 8])
    while (block // per_chunk) > 32 or (block // per_chunk) & (block // per_chunk - 1):
        block //= 2
    chunks = int(rng.integers(256, 1300)) if rng.random() < 0.7 else int(rng.integers(1, 64))
    cols = max(block, chunks * per_chunk // block * block)
    lead = [int(rng.integers(1, 6)) for _ in range(int(rng.integers(1, 4)))]
    shape = tuple(lead) + (cols,)
    if rng.random() < 0.25:
        return scheme, elem, shape
    return scheme.with_level(QuantLevel.block([block])), elem, shape


def run_case(gpu, oracle, client, rng, scheme, elem, shape):
    import torch

    pe = gpu.param_elem(scheme)
    per = scheme.num_quants()
    pshape = tuple(shape[:-1]) + (shape[-1] // per,)
    sshape = scheme.scales_shape(shape)
    fkind, fstr = random_layout(rng, shape)
    vkind, vstr = random_layout(rng, pshape)
    stored_np = np.uint32 if scheme.store == QuantStore.U32 else np.uint8
    tag = (scheme.value.name, scheme.store.name, scheme.param.name, elem.name, shape,
           "tensor" if scheme.level.is_tensor else scheme.level.block_size.dims, fkind, fstr, vkind, vstr)

    x32 = rng.normal(0, pick(rng, [1e-3, 1.0, 50.0]), reach(shape, fstr)).astype(np.float32)
    fbuf = oracle.to_bits(x32, elem)
    xc = np.ascontiguousarray(view(fbuf, shape, fstr))
    s_ref = oracle.compute_scales(xc, elem, shape, scheme)
    w_ref, os_ref = oracle.quantize(xc, elem, shape, s_ref, scheme)
    y_ref = oracle.dequantize(w_ref, shape, os_ref, elem, scheme)

    d_f = gpu.to_dev(fbuf)
    h_f = gpu.handle(d_f, shape, fstr)
    sentinel = 0xA5 if stored_np == np.uint8 else 0xA5A5A5A5
    vbuf0 = np.full(reach(pshape, vstr), sentinel, dtype=stored_np)
    ws, nbytes = gpu.workspace(scheme, int(np.prod(shape)))

    d_s = torch.zeros(sshape, dtype=gpu.storage_dtype(elem), device="cuda")
    qz.compute_scales(client, h_f, gpu.handle(d_s), scheme, elem, ws.data_ptr(), nbytes)
    assert np.array_equal(gpu.to_host(d_s).reshape(-1), s_ref.reshape(-1)), tag + ("scales",)

    for what in ("given", "dynamic"):
        d_v = gpu.to_dev(vbuf0)
        h_v = gpu.handle(d_v, pshape, vstr)
        d_os = torch.zeros(sshape, dtype=gpu.storage_dtype(pe), device="cuda")
        if what == "given":
            qz.launch_ref(client, h_f, h_v, gpu.handle(d_s), gpu.handle(d_os), scheme, elem)
        else:
            qz.launch_dynamic(client, h_f, h_v, gpu.handle(d_os), scheme, elem, ws.data_ptr(), nbytes)
        torch.cuda.synchronize()
        got = gpu.to_host(d_v).view(stored_np)
        assert np.array_equal(view(got, pshape, vstr), w_ref.reshape(pshape)), tag + (what,)
        mask = np.ones(got.size, dtype=bool)
        view(mask, pshape, vstr)[...] = False
        assert np.all(got[mask] == sentinel), tag + (what, "wrote outside the view")
        assert np.array_equal(gpu.to_host(d_os).reshape(-1), os_ref.reshape(-1)), tag + (what, "out_scale")

    fill = np.float32(777.0) if elem == ElemType.F32 else np.uint16(0x7777)
    d_y = gpu.to_dev(np.full(fbuf.size, fill, dtype=fbuf.dtype))
    dq.launch_ref(client, h_v, gpu.handle(d_y, shape, fstr), gpu.handle(d_os), scheme, elem)
    torch.cuda.synchronize()
    got = gpu.to_host(d_y).view(fbuf.dtype)
    lhs, rhs = view(got, shape, fstr), y_ref.reshape(shape)
    if elem == ElemType.F32:
        lhs, rhs = lhs.view(np.uint32), rhs.view(np.uint32)
    assert np.array_equal(lhs, rhs), tag + ("dequantize",)
    mask = np.ones(got.size, dtype=bool)
    view(mask, shape, fstr)[...] = False
    assert np.all(got[mask] == fill), tag + ("dequantize wrote outside the view",)


# CQ_RANDOM_SEEDS=N widens the campaign (8 configurations per seed)
@pytest.mark.parametrize("seed", range(int(os.environ.get("CQ_RANDOM_SEEDS", "16"))))
def test_random_configurations(gpu, oracle, seed):
    rng = np.random.default_rng(zlib.crc32(b"random configs") + seed)
    client = ComputeClient.current()
    for _ in range(8):
        scheme, elem, shape = random_case(rng)
        run_case(gpu, oracle, client, rng, scheme, elem, shape)


@pytest.mark.parametrize("seed", range(int(os.environ.get("CQ_RANDOM_SEEDS", "16"))))
def test_random_long_rows(gpu, oracle, seed):
    rng = np.random.default_rng(zlib.crc32(b"long rows") + seed)
    client = ComputeClient.current()
    for _ in range(4):
        scheme, elem, shape = random_long_rows_case(rng)
        run_case(gpu, oracle, client, rng, scheme, elem, shape)
