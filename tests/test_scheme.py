"""Host logic of the scheme mirror (the option set of cubek_quant::scheme)."""
import pytest

from cubek_amd import BlockSize, QuantLevel, QuantParam, QuantScheme, QuantStore, QuantValue


def test_default_and_builders():
    s = QuantScheme.default()
    assert (s.value, s.param, s.store, s.level.is_tensor) == (QuantValue.Q8F, QuantParam.F32, QuantStore.U32, True)
    s2 = (s.with_level(QuantLevel.block([32])).with_value(QuantValue.Q4S).with_store(QuantStore.U32)
          .with_param(QuantParam.BF16))
    assert s2.level.block_size.as_slice() == (32,) and s2.num_quants() == 8 and s.num_quants() == 4
    assert s.value == QuantValue.Q8F  # builders do not mutate


def test_num_quants_and_sizes():
    expect = {QuantValue.Q8F: 4, QuantValue.Q8S: 4, QuantValue.E4M3: 4, QuantValue.E5M2: 4,
              QuantValue.Q4F: 8, QuantValue.Q4S: 8, QuantValue.E2M1: 8, QuantValue.Q2F: 16, QuantValue.Q2S: 16}
    for v, nq in expect.items():
        assert QuantScheme.default().with_value(v).num_quants() == nq
        assert QuantScheme.default().with_value(v).size_bits_stored() == 32
    native = QuantScheme.default().with_store(QuantStore.Native)
    assert native.with_value(QuantValue.E2M1).num_quants() == 2
    assert native.with_value(QuantValue.E4M3).num_quants() == 1


def test_ranges_give_the_test_scale_divisors():
    # q_max - q_min as used by tests/suite/symmetric.rs:35-37
    widths = {QuantValue.Q8F: 255, QuantValue.Q8S: 254, QuantValue.Q4F: 15, QuantValue.Q4S: 14,
              QuantValue.Q2F: 3, QuantValue.Q2S: 2, QuantValue.E2M1: 12}
    for v, w in widths.items():
        lo, hi = v.range()
        assert hi - lo == w
    assert QuantValue.Q8S.is_symmetric() and not QuantValue.Q8F.is_symmetric()


def test_block_size_padding_and_shapes():
    b = BlockSize((2, 16))
    assert b.to_dim_vec(4) == (1, 1, 2, 16) and b.num_elements() == 32
    s = QuantScheme.default().with_level(QuantLevel.block([2, 16])).with_value(QuantValue.Q4S)
    assert s.scales_shape((3, 4, 64)) == (3, 2, 4)
    assert s.packed_shape((3, 4, 64)) == (3, 4, 8)
    assert QuantScheme.default().scales_shape((3, 4, 64)) == (1,)
    with pytest.raises(ValueError):
        s.scales_shape((3, 5, 64))
    with pytest.raises(ValueError):
        s.packed_shape((3, 4, 60))
    with pytest.raises(ValueError):
        BlockSize((1, 2, 3, 4, 5, 6))
    with pytest.raises(ValueError):
        BlockSize((256,))
    with pytest.raises(ValueError):
        b.to_dim_vec(1)


def test_c_struct_round_trip():
    c = QuantScheme.default().with_level(QuantLevel.block([3, 8])).with_value(QuantValue.E2M1).to_c()
    assert (c.value, c.level, c.block_rank, c.block[0], c.block[1], c.reserved) == (6, 1, 2, 3, 8, 0)
