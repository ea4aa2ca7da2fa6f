"""Layouts served by the row kernels (last dimension contiguous, everything else free):
2-D and N-D blocks, block sizes that are not a power-of-two number of lanes, ragged
tiles, leading dimensions, F16/BF16 scale parameters, native store -- against the oracle,
bit for bit, through cq_compute_scales, cq_quantize, cq_quantize_dynamic, cq_dequantize."""
import numpy as np
import pytest

from cubek_amd import ElemType, QuantLevel, QuantParam, QuantScheme, QuantStore, QuantValue

pytestmark = pytest.mark.gpu

ELEMS = [ElemType.F32, ElemType.BF16, ElemType.F16]
# (shape, block, value, store)
CASES = [
    ((256, 384), (128, 128), QuantValue.Q8S, QuantStore.U32),       # weight-style 128 x 128 blocks
    ((3, 96, 200), (32, 40), QuantValue.Q4S, QuantStore.U32),       # 40 = 5 chunks (bf16), leading dimension
    ((130, 1016), (1, 8), QuantValue.Q8F, QuantStore.U32),          # one chunk per block, ragged tiles
    ((64, 4104), (24,), QuantValue.Q8S, QuantStore.U32),            # 3 chunks per block, rows longer than a tile
    ((2, 3, 10, 160), (5, 32), QuantValue.Q2S, QuantStore.U32),     # rank 4, 2-bit codes
    ((50, 64), (50, 64), QuantValue.E2M1, QuantStore.U32),          # one block = the whole matrix
    ((96, 256), (32, 64), QuantValue.E4M3, QuantStore.U32),
    ((96, 256), (32, 64), QuantValue.Q8S, QuantStore.Native),
    ((96, 256), (16, 128), QuantValue.E4M3, QuantStore.Native),
    ((48, 192), (8, 48), QuantValue.E5M2, QuantStore.Native),
    ((40, 320), (4, 32), QuantValue.E2M1, QuantStore.Native),
    ((96, 256), (32, 64), QuantValue.E2M1_OCP, QuantStore.U32),      # the extension value, both stores
    ((48, 320), (8, 32), QuantValue.E2M1_OCP, QuantStore.Native),
    ((7, 4, 3, 64), (4, 3, 32), QuantValue.Q4F, QuantStore.U32),    # block over three dimensions: scales per element
]


@pytest.fixture(scope="module")
def gpu():
    import gpu_harness

    return gpu_harness


def same_bits(a, b):
    a, b = np.ascontiguousarray(a).reshape(-1), np.ascontiguousarray(b).reshape(-1)
    return a.shape == b.shape and np.array_equal(a.view(np.uint8), b.view(np.uint8))


@pytest.mark.parametrize("elem", ELEMS, ids=lambda e: e.name)
@pytest.mark.parametrize("case", CASES, ids=lambda c: f"{c[2].name}_{c[3].name}_{'x'.join(map(str, c[1]))}")
def test_row_kernels_match_oracle(gpu, oracle, elem, case):
    shape, block, value, store = case
    rng = np.random.default_rng(len(shape) * 100 + sum(block) + int(elem))
    for param in (QuantParam.F32, QuantParam.BF16 if elem != ElemType.F16 else QuantParam.F16):
        scheme = (QuantScheme.default().with_value(value).with_store(store).with_param(param)
                  .with_level(QuantLevel.block(list(block))))
        x32 = rng.normal(0, 1.5, shape).astype(np.float32)
        x32[rng.random(shape) < 0.002] = np.nan
        x = oracle.to_bits(x32, elem)
        s_ref = oracle.compute_scales(x, elem, shape, scheme)
        assert same_bits(gpu.compute_scales(x, elem, shape, scheme), s_ref)
        w_ref, os_ref = oracle.quantize(x, elem, shape, s_ref, scheme)
        w_gpu, os_gpu = gpu.quantize(x, elem, shape, s_ref, scheme)
        assert same_bits(w_gpu, w_ref) and same_bits(os_gpu, os_ref)
        w_dyn, os_dyn = gpu.quantize_dynamic(x, elem, shape, scheme)
        assert same_bits(w_dyn, w_ref) and same_bits(os_dyn, os_ref)
        y_ref = oracle.dequantize(w_ref, shape, os_ref, elem, scheme)
        y_gpu = gpu.dequantize(w_ref, shape, os_ref, elem, scheme)
        ok = ~np.isnan(oracle.from_bits(y_ref, elem)).reshape(-1)
        assert same_bits(y_gpu.reshape(-1)[ok], y_ref.reshape(-1)[ok])
        assert np.isnan(oracle.from_bits(y_gpu, elem)).reshape(-1)[~ok].all()
