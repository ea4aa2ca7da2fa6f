"""cq_quantize_dynamic_static (the entry point that allocates nothing and takes no workspace) against
cq_quantize_dynamic with a caller's workspace: codes and scales bit for bit, on two calls in a row on
one stream, the second with a smaller input.  The per-tensor schemes are the ones whose kernels use
the library's built-in scratch array (abs-max partials of the grid reduction); a block scheme, which
needs no scratch, goes through the same entry point."""
import numpy as np
import pytest

from cubek_amd import ComputeClient, ElemType, QuantLevel, QuantScheme, QuantValue, TensorHandleRef
from cubek_amd import quantize as qz

pytestmark = pytest.mark.gpu

CASES = [
    # (elem, value, block, first shape, second (smaller) shape)
    (ElemType.BF16, QuantValue.Q8S, None, (1024, 4096), (96, 512)),     # flat two-pass reduction, 256 then 2 partials
    (ElemType.F32, QuantValue.Q4S, None, (2048, 1024), (3, 40)),        # second call: ragged tail only
    (ElemType.F16, QuantValue.E2M1, None, (8, 512, 640), (1, 8, 64)),
    (ElemType.BF16, QuantValue.Q4S, 32, (512, 2048), (16, 256)),        # block scheme: no scratch in use
]


def _torch_dtype(torch, elem):
    return {ElemType.F32: torch.float32, ElemType.BF16: torch.bfloat16, ElemType.F16: torch.float16}[elem]


@pytest.mark.parametrize("elem,value,block,big,small", CASES,
                         ids=lambda v: getattr(v, "name", None) or str(v).replace(" ", ""))
def test_static_scratch_matches_workspace_entry_point(oracle, elem, value, block, big, small):
    import torch

    level = QuantLevel.Tensor if block is None else QuantLevel.block([block])
    scheme = QuantScheme.default().with_value(value).with_level(level)
    h = TensorHandleRef.from_torch
    client = ComputeClient.current()
    gen = torch.Generator(device="cpu").manual_seed(11)
    dt = _torch_dtype(torch, elem)

    runs = []
    for shape in (big, small):
        x = (torch.randn(shape, generator=gen) * 0.02).to(dt).cuda()
        x.view(-1)[x.numel() // 3] = 3.0  # the abs-max sits inside the tensor, not at its start
        bufs = {}
        for name in ("static", "workspace"):
            words = torch.full(scheme.packed_shape(shape), -1, dtype=torch.int32, device="cuda")
            scales = torch.full(scheme.scales_shape(shape), -1.0, dtype=torch.float32, device="cuda")
            bufs[name] = (words, scales)
        runs.append((shape, x, bufs))

    nbytes = qz.workspace_bytes(scheme, int(np.prod(big)))
    ws = torch.zeros(max(nbytes, 16), dtype=torch.uint8, device="cuda")
    torch.cuda.synchronize()
    # the two calls in a row on one stream, no synchronisation in between
    for shape, x, bufs in runs:
        words, scales = bufs["static"]
        qz.launch_dynamic_static(client, h(x), h(words), h(scales), scheme, elem)
    torch.cuda.synchronize()
    for shape, x, bufs in runs:
        words, scales = bufs["workspace"]
        qz.launch_dynamic(client, h(x), h(words), h(scales), scheme, elem, ws.data_ptr(), nbytes)
        torch.cuda.synchronize()

    for shape, x, bufs in runs:
        got_w, got_s = bufs["static"]
        want_w, want_s = bufs["workspace"]
        assert torch.equal(got_w, want_w), (shape, "codes differ from cq_quantize_dynamic")
        assert torch.equal(got_s.view(torch.int32), want_s.view(torch.int32)), (shape, "scales differ")
        # and both against the CPU oracle
        bits = x.cpu().view(torch.int16).numpy().view(np.uint16) if elem != ElemType.F32 else x.cpu().numpy()
        s_ref = oracle.compute_scales(bits, elem, shape, scheme)
        w_ref, os_ref = oracle.quantize(bits, elem, shape, s_ref, scheme)
        assert np.array_equal(got_w.cpu().numpy().view(np.uint32).reshape(-1), np.asarray(w_ref).reshape(-1))
        assert np.array_equal(got_s.cpu().numpy().view(np.uint32).reshape(-1),
                              np.asarray(os_ref, dtype=np.float32).view(np.uint32).reshape(-1))


def test_static_scratch_rejects_bad_arguments():
    """Same validation as cq_quantize_dynamic; nothing reaches the device."""
    import ctypes

    from cubek_amd import _ffi

    lib = _ffi.lib()
    s = QuantScheme.default().to_c()
    assert lib.cq_quantize_dynamic_static(None, None, None, None, ctypes.byref(s), 0) == _ffi.ERR_INVALID_ARGUMENT
    assert lib.cq_quantize_dynamic_static(None, None, None, None, None, 0) == _ffi.ERR_INVALID_ARGUMENT


def test_static_scratch_on_a_stream_of_its_own():
    """A non-default stream of the current device: the entry point asks the stream for its device before it resolves
    the scratch array (a stream of another device would be refused with an invalid-argument status; one GPU cannot
    show that).  Same codes and scale as on the default stream."""
    import torch

    scheme = QuantScheme.default().with_value(QuantValue.Q8S)
    h = TensorHandleRef.from_torch
    shape = (256, 1024)
    x = (torch.randn(shape, generator=torch.Generator(device="cpu").manual_seed(3)) * 0.02).to(torch.bfloat16).cuda()
    outs = []
    side = torch.cuda.Stream()
    for stream in (None, side):
        words = torch.full(scheme.packed_shape(shape), -1, dtype=torch.int32, device="cuda")
        scales = torch.full((1,), -1.0, dtype=torch.float32, device="cuda")
        torch.cuda.synchronize()
        client = ComputeClient.current() if stream is None else ComputeClient(stream.cuda_stream)
        qz.launch_dynamic_static(client, h(x), h(words), h(scales), scheme, ElemType.BF16)
        torch.cuda.synchronize()
        outs.append((words, scales))
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1].view(torch.int32), outs[1][1].view(torch.int32))
    assert float(outs[0][1][0]) > 0
