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


@pytest.mark.parametrize("bits", [2, 4])
@pytest.mark.parametrize("gs", [-1, 128])
def test_gptq_writer_is_the_inverse_of_the_repacker(dzlib, bits, gs):
    """dz_unrepack_2of4 (native -> the reference's qweight/qzeros/scales/g_idx) gives back, byte for
    byte, the GPTQ tensors the native delta was made from (those are what QuantLinear.pack writes for
    a 2:4 delta: pruned columns carry the zero-point code), and repacking them gives the same native
    bytes again."""
    n, k = 96, 768
    d = o.make_delta(n, k, 1e-3, bits, gs, 33)
    q, m, s = ops.repack_gptq_to_native(torch.from_numpy(d["qweight"]), torch.from_numpy(d["qzeros"]),
                                        torch.from_numpy(d["scales"]), torch.from_numpy(d["g_idx"]), bits)
    qw, qz, sc, gi = ops.unrepack_native_to_gptq(q, m, s, k, n, bits)
    assert qw.dtype == torch.int32 and tuple(qw.shape) == d["qweight"].shape
    assert np.array_equal(qw.numpy(), d["qweight"])
    assert np.array_equal(qz.numpy(), d["qzeros"])
    assert np.array_equal(sc.numpy().view(np.uint16), d["scales"].view(np.uint16))
    assert np.array_equal(gi.numpy(), d["g_idx"].astype(np.int32))
    q2, m2, s2 = ops.repack_gptq_to_native(qw, qz, sc, gi, bits)
    assert torch.equal(q2, q) and torch.equal(m2, m) and torch.equal(s2, s)
    # known fields: qzeros holds zero - 1 = 2^(bits-1) - 1 in every field of every word
    field = 2 ** (bits - 1) - 1
    word = sum(field << (bits * f) for f in range(32 // bits))
    assert (qz.numpy().view(np.uint32) == word).all()
    # the written tensors dequantise, the reference's way, to the native dequantisation
    ref = o.dequant_gptq(qw.numpy(), qz.numpy(), sc.numpy(), gi.numpy(), bits)
    qn = q.numpy().view(np.uint32)
    codes = qn.reshape(n // 32, k // 256, 64, 4) if bits == 2 else qn.reshape(n // 32, k // 256, 2, 64, 4)
    nat = o.dequant_native(codes, m.numpy().view(np.uint32).reshape(n // 32, k // 256, 64, 4), s.numpy(), k, n, bits)
    assert np.array_equal(nat.view(np.uint16), np.ascontiguousarray(ref.T).view(np.uint16))


def test_gptq_writer_of_an_all_pruned_delta(dzlib):
    """Nothing kept anywhere: every qweight word is the zero-point pattern (0x88888888 at 4 bits)."""
    bits, n, k = 4, 32, 256
    codes = np.full((k, n), 8, dtype=np.uint8)
    qw0, qz0, sc0, gi0 = o.pack_codes_gptq(codes, np.full((1, n), 8), np.full((1, n), 0.25, np.float16), bits)
    q, m, s = ops.repack_gptq_to_native(*(torch.from_numpy(np.ascontiguousarray(v)) for v in (qw0, qz0, sc0, gi0)), bits)
    qw, qz, sc, gi = ops.unrepack_native_to_gptq(q, m, s, k, n, bits)
    assert (qw.numpy().view(np.uint32) == 0x88888888).all() and (qz.numpy().view(np.uint32) == 0x77777777).all()


def test_gptq_writer_argument_checks(dzlib):
    one = C.c_void_p(0x1000)
    f = dzlib.dz_unrepack_2of4
    assert f(None, one, one, 256, 32, 4, -1, one, one, one, one) == -1
    assert f(one, one, one, 256, 32, 3, -1, one, one, one, one) == -3
    assert f(one, one, one, 200, 32, 4, -1, one, one, one, one) == -2
    assert f(one, one, one, 256, 32, 4, 100, one, one, one, one) == -4
    with pytest.raises(ValueError):
        ops.unrepack_native_to_gptq(torch.zeros(10, dtype=torch.int32), torch.zeros(10, dtype=torch.int16),
                                    torch.zeros((1, 32), dtype=torch.float16), 256, 32, 4)


def test_untile_base_inverts_the_documented_tile_order():
    """ops.untile_base (plain tensor ops, runs anywhere) against the tile formula written out value by
    value: tile (np, kb) of 16 KiB, fragment (s, j, h) of 1 KiB, lane 16*g + i holding
    W[32*np + 16*s + i][256*kb + 64*j + 16*g + 8*h + e], e = 0..7."""
    import torch
    from deltazip_amd import ops
    n, k = 64, 512
    w = (np.arange(n * k, dtype=np.int64) % 30011).astype(np.float16).reshape(n, k)   # exact in fp16, no repeats per row block
    tiled = np.empty(n * k, dtype=np.float16)
    for np_ in range(n // 32):
        for kb in range(k // 256):
            for s in range(2):
                for j in range(4):
                    for h in range(2):
                        for lane in range(64):
                            i, g = lane % 16, lane // 16
                            off = ((np_ * (k // 256) + kb) * 16384 + ((s * 4 + j) * 2 + h) * 1024 + lane * 16) // 2
                            row, col = 32 * np_ + 16 * s + i, 256 * kb + 64 * j + 16 * g + 8 * h
                            tiled[off:off + 8] = w[row, col:col + 8]
    back = ops.untile_base(torch.from_numpy(tiled.reshape(n, k)))
    assert np.array_equal(back.numpy(), w)
    with pytest.raises(ValueError):
        ops.untile_base(torch.zeros(48, 512, dtype=torch.float16))
    with pytest.raises(ValueError):
        ops.untile_base(torch.zeros(64, 512, dtype=torch.float32))
