"""Native gfx950 layout: the oracle's definition round-trips through the reference dequant, and
the library's host repacker (dz_repack_2of4) produces the same bytes."""
import ctypes as C

import numpy as np
import pytest
import torch

from oracle import dz_oracle as o
from deltazip_amd import ops


@pytest.mark.parametrize("bits", [2, 4])
@pytest.mark.parametrize("gs", [-1, 64, 128])
def test_oracle_native_round_trip(bits, gs):
    d = o.make_delta(64, 512, 1e-3, bits, gs, 7)
    ref = o.dequant_gptq(d["qweight"], d["qzeros"], d["scales"], d["g_idx"], bits)      # [K, N]
    codes, meta, sc = o.repack_native(d["qweight"], d["qzeros"], d["scales"], d["g_idx"], bits)
    nat = o.dequant_native(codes, meta, sc, 512, 64, bits)                              # [N, K]
    assert np.array_equal(nat.view(np.uint16), np.ascontiguousarray(ref.T).view(np.uint16))


@pytest.mark.parametrize("bits", [2, 4])
def test_adversarial_all_kept_codes_are_zero_point(bits):
    """A delta that is all zero-point codes (nothing to keep) still repacks and dequantises to 0."""
    k, n = 256, 32
    zp = 2 ** (bits - 1)
    codes = np.full((k, n), zp, dtype=np.uint8)
    codes[5, 3] = zp + 1                      # a single non-zero entry
    qw, qz, sc, gi = o.pack_codes_gptq(codes, np.full((1, n), zp), np.full((1, n), 0.5, np.float16), bits)
    c, m, s = o.repack_native(qw, qz, sc, gi, bits)
    nat = o.dequant_native(c, m, s, k, n, bits)
    expect = np.zeros((n, k), np.float16)
    expect[3, 5] = 0.5
    assert np.array_equal(nat, expect)


@pytest.mark.parametrize("bits", [2, 4])
@pytest.mark.parametrize("gs", [-1, 128])
def test_library_repacker_matches_oracle(dzlib, bits, gs):
    d = o.make_delta(96, 768, 1e-3, bits, gs, 21)
    codes, meta, sc = o.repack_native(d["qweight"], d["qzeros"], d["scales"], d["g_idx"], bits)
    q, m, s = ops.repack_gptq_to_native(torch.from_numpy(d["qweight"]), torch.from_numpy(d["qzeros"]),
                                        torch.from_numpy(d["scales"]), torch.from_numpy(d["g_idx"]), bits)
    assert q.numpy().view(np.uint32).tobytes() == codes.tobytes()
    assert m.numpy().view(np.uint32).tobytes() == meta.tobytes()
    assert np.array_equal(s.numpy().view(np.uint16), sc.view(np.uint16))
    # shapes follow the reference's stacked tensors (layers_marlin.py:311-333)
    pf = 32 // bits
    assert tuple(q.shape) == (768 // (pf * 4), 2 * 96) and tuple(m.shape) == (96, 768 // 16)
    cb, mb, sb = ops.native_sizes(768, 96, bits, gs)
    assert cb == q.numel() * 4 and mb == m.numel() * 2 and sb == s.numel() * 2


def test_repacker_rejects_bad_input(dzlib):
    bits = 4
    d = o.make_delta(32, 256, 1e-3, bits, -1, 5)
    qw = torch.from_numpy(d["qweight"].copy()); qz = torch.from_numpy(d["qzeros"].copy())
    sc = torch.from_numpy(d["scales"].copy()); gi = torch.from_numpy(d["g_idx"].copy())
    # not 2:4: make three entries of one group non-zero
    codes, zeros = o.unpack_gptq(d["qweight"], d["qzeros"], bits)
    codes = codes.astype(np.uint8); codes[0:3, 0] = [9, 10, 11]; codes[3, 0] = 8
    bad_qw, _, _, _ = o.pack_codes_gptq(codes, zeros.astype(np.int32), d["scales"], bits)
    with pytest.raises(ValueError, match="2:4"):
        ops.repack_gptq_to_native(torch.from_numpy(bad_qw), qz, sc, gi, bits)
    with pytest.raises(ValueError):
        o.repack_native(bad_qw, d["qzeros"], d["scales"], d["g_idx"], bits)
    # asymmetric zero-point
    bad_qz = qz.clone(); bad_qz[0, 0] = 0x77777776
    with pytest.raises(ValueError, match="zero-point"):
        ops.repack_gptq_to_native(qw, bad_qz, sc, gi, bits)
    # act-order style g_idx
    bad_gi = gi.clone(); bad_gi[3] = 1
    with pytest.raises(ValueError, match="g_idx"):
        ops.repack_gptq_to_native(qw, qz, sc, bad_gi, bits)
    # unsupported bit width and shapes
    with pytest.raises(NotImplementedError):
        ops.repack_gptq_to_native(qw, qz, sc, gi, 3)
    with pytest.raises(ValueError):
        ops.native_sizes(4096 + 32, 4096, 4)          # K % 256
    with pytest.raises(ValueError):
        ops.native_sizes(4096, 4096 + 16, 4)          # N % 32
    with pytest.raises(ValueError):
        ops.native_sizes(4096, 4096, 4, 100)          # group size
    with pytest.raises(NotImplementedError):
        ops.native_sizes(4096, 4096, 8)
