"""The entry points only enqueue kernels on the caller's stream (no allocation, no
synchronisation, no memset), so a caller can capture them into a HIP graph.  Capture
quantize_dynamic + dequantize for a block-scaled and a per-tensor scheme, replay the
graph several times on changing inputs with eager work in between, and compare every
replay with the eager result."""
import numpy as np
import pytest

from cubek_amd import ComputeClient, ElemType, QuantLevel, QuantScheme, QuantValue, TensorHandleRef
from cubek_amd import dequantize as dq
from cubek_amd import quantize as qz

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("level", ["block32", "tensor", "block64x64"])
def test_graph_replays_match_eager(level):
    import torch

    scheme = QuantScheme.default().with_value(QuantValue.Q4S)
    if level == "block32":
        scheme = scheme.with_level(QuantLevel.block([32]))
    elif level == "block64x64":  # the pipelined block kernel (looks up its occupancy on first use)
        scheme = scheme.with_level(QuantLevel.block([64, 64]))
    shape = (512, 1024)
    h = TensorHandleRef.from_torch
    gen = torch.Generator(device="cuda").manual_seed(7)
    x = torch.randn(shape, device="cuda", dtype=torch.bfloat16, generator=gen)
    words = torch.zeros(scheme.packed_shape(shape), dtype=torch.int32, device="cuda")
    scales = torch.zeros(scheme.scales_shape(shape), dtype=torch.float32, device="cuda")
    y = torch.zeros(shape, device="cuda", dtype=torch.bfloat16)
    nbytes = qz.workspace_bytes(scheme, x.numel())
    ws = torch.zeros(max(nbytes, 16), dtype=torch.uint8, device="cuda")

    def run():
        client = ComputeClient.current()  # the stream torch is capturing on
        qz.launch_dynamic(client, h(x), h(words), h(scales), scheme, ElemType.BF16, ws.data_ptr(), nbytes)
        dq.launch_ref(client, h(words), h(y), h(scales), scheme, ElemType.BF16)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run()  # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run()

    for it in range(4):
        x.copy_(torch.randn(shape, device="cuda", dtype=torch.bfloat16, generator=gen) * (it + 1))
        graph.replay()
        torch.cuda.synchronize()
        got = (words.clone(), scales.clone(), y.clone())
        words.zero_(), scales.zero_(), y.zero_()
        run()  # eager, same buffers
        torch.cuda.synchronize()
        assert torch.equal(got[0], words) and torch.equal(got[1], scales), (level, it)
        assert torch.equal(got[2].view(torch.int16), y.view(torch.int16)), (level, it)
        assert float(y.float().abs().max()) > 0


_COLD_CAPTURE = r"""
import sys
import torch
from cubek_amd import ComputeClient, ElemType, QuantLevel, QuantScheme, QuantValue, TensorHandleRef
from cubek_amd import dequantize as dq, quantize as qz
scheme = QuantScheme.default().with_value(QuantValue.Q4S).with_level(QuantLevel.block(BLOCK))
shape = (512, 1024)
h = TensorHandleRef.from_torch
x = torch.randn(shape, device="cuda", dtype=torch.bfloat16)
words = torch.zeros(scheme.packed_shape(shape), dtype=torch.int32, device="cuda")
scales = torch.zeros(scheme.scales_shape(shape), dtype=torch.float32, device="cuda")
y = torch.zeros(shape, device="cuda", dtype=torch.bfloat16)
torch.cuda.synchronize()
def run():
    c = ComputeClient.current()
    qz.launch_dynamic(c, h(x), h(words), h(scales), scheme, ElemType.BF16, 0, 0)
    dq.launch_ref(c, h(words), h(y), h(scales), scheme, ElemType.BF16)
g = torch.cuda.CUDAGraph()
with torch.cuda.graph(g):
    run()  # the library's first launches in this process
g.replay()
torch.cuda.synchronize()
got = (words.clone(), scales.clone(), y.clone())
words.zero_(), scales.zero_(), y.zero_()
run()
torch.cuda.synchronize()
ok = torch.equal(got[0], words) and torch.equal(got[1], scales) and torch.equal(got[2].view(torch.int16), y.view(torch.int16))
sys.exit(0 if ok and float(y.float().abs().max()) > 0 else 3)
"""


@pytest.mark.parametrize("block", ["[32]", "[64, 64]"])
def test_a_process_first_calls_can_be_captured(block):
    """No warm-up: the first launch out of a code object (the streaming kernels' are stored as they are, the 2-D block
    kernel's compressed) loads it while the stream is capturing; the replay must match the eager result.  Runs in
    a process of its own, since this one has launched before."""
    import os
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, PYTHONPATH=root + os.pathsep + os.environ.get("PYTHONPATH", ""))
    proc = subprocess.run([sys.executable, "-c", _COLD_CAPTURE.replace("BLOCK", block)], cwd=root, env=env,
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=110)
    assert proc.returncode == 0, proc.stdout[-2000:]
