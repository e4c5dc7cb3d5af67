"""The loader's other K types, Q2_K / Q3_K / Q5_K (src/loader/dequant.rs:150-420; reached through
loader::dequantize, src/loader/dequant.rs:673-700): the oracle against the reference's own unit-test
vectors (src/loader/dequant.rs:440-665, transcribed as byte patterns and expected values) and against
an independent whole-array numpy statement of the three layouts; the GPU decoders bit for bit
against the oracle; the matmul entry points refuse these formats."""
import numpy as np
import pytest

from helpers import assert_bit_exact
from rocmforge_amd import quantize as Q

Q2_K, Q3_K, Q5_K = Q.Q2_K, Q.Q3_K, Q.Q5_K
FORMATS = [Q2_K, Q3_K, Q5_K]


def block(scale0_bits=(0x00, 0x3C)):
    d = np.zeros(256, np.uint8)
    d[0], d[1] = scale0_bits                                              # sub-block 0: f16 1.0
    return d


# ---------------------------------------------------------------- the reference's vectors
def test_q5_k_reference_vectors(oracle):
    d = block()
    assert np.all(oracle.dequantize(Q5_K, d, 256) == 0.0)                 # dequant.rs:440-461
    d[48] = 0x01                                                          # :463-493, first 5 bits = 1
    r = oracle.dequantize(Q5_K, d, 256)
    assert r.shape == (256,) and r[0] == 1.0 and np.all(r[1:16] == 0.0)
    r = oracle.dequantize(Q5_K, block(), 100)                             # :495-512, 100 of 256 elements
    assert r.shape == (100,) and np.all(r == 0.0)
    d = np.zeros(512, np.uint8)                                           # :514-541, two blocks
    d[0:2] = (0x00, 0x3C)
    d[256:258] = (0x00, 0x40)                                             # 2.0
    d[256 + 48], d[256 + 49] = 0xFF, 0x80
    r = oracle.dequantize(Q5_K, d, 512)
    assert np.all(r[:256] == 0.0) and r[256] == 62.0                      # 31 * 2.0


def test_q3_k_reference_vectors(oracle):
    r = oracle.dequantize(Q3_K, block(), 256)                             # dequant.rs:543-560
    assert np.all(r[:16] == -4.0)
    d = block(); d[36] = 0x01                                             # :562-584
    r = oracle.dequantize(Q3_K, d, 256)
    assert r[0] == -3.0 and np.all(r[1:16] == -4.0)
    r = oracle.dequantize(Q3_K, block(), 100)                             # :586-605
    assert r.shape == (100,) and np.all(r[:16] == -4.0)


def test_q2_k_reference_vectors(oracle):
    r = oracle.dequantize(Q2_K, block(), 256)                             # dequant.rs:607-626
    assert np.all(r[:16] == 0.0)
    d = block(); d[68] = 0x01                                             # :628-646
    assert oracle.dequantize(Q2_K, d, 256)[0] == 1.0
    r = oracle.dequantize(Q2_K, block(), 100)                             # :648-665
    assert r.shape == (100,) and np.all(r[:16] == 0.0)


# ---------------------------------------------------------------- an independent statement
def bits_lsb_first(stream, width, count):
    """`count` fields of `width` bits from a [blocks, bytes] array, LSB first (numpy, whole array)."""
    bits = np.unpackbits(stream, axis=-1, bitorder="little")[..., : width * count]
    w = (1 << np.arange(width)).astype(np.int64)
    return (bits.reshape(*stream.shape[:-1], count, width) * w).sum(-1)


def independent(fmt, data, n):
    """float64 evaluation of the three layouts over whole arrays, rounded once to f32 where the
    reference rounds once (the product code * f16 scale is exact in f32)."""
    b = data.reshape(-1, 256)
    nb = b.shape[0]
    scale = b[:, 0:32].copy().view("<f2").astype(np.float64).reshape(nb, 16, 1)
    if fmt == Q5_K:
        mn = b[:, 32:48].view(np.int8).astype(np.float64).reshape(nb, 16, 1)
        q = bits_lsb_first(b[:, 48:208].reshape(nb, 16, 10), 5, 16)
        v = mn + q * scale
    elif fmt == Q3_K:
        hb = b[:, 32:36].astype(np.int64)                                  # two bits per sub-block
        qh = (hb[:, np.arange(16) // 4] >> ((np.arange(16) % 4) * 2)) & 3
        q = bits_lsb_first(b[:, 36:132].reshape(nb, 16, 6), 3, 16)
        q[:, :, 0] |= (qh & 1) << 3
        q[:, :, 1] |= (qh >> 1) << 3
        v = (q - 4.0) * scale
    else:
        mn = b[:, 32:64].copy().view("<f2").astype(np.float64).reshape(nb, 16, 1)
        hb = b[:, 64:66].astype(np.int64)                                  # one bit per sub-block
        qh = (hb[:, np.arange(16) // 8] >> (np.arange(16) % 8)) & 1
        q = bits_lsb_first(b[:, 68:132].reshape(nb, 16, 4), 2, 16)
        q[:, :, 0] |= qh << 2
        v = mn + q * scale
    return v.astype(np.float32).ravel()[:n]


@pytest.mark.parametrize("fmt", FORMATS)
def test_oracle_matches_the_independent_statement(fmt, oracle):
    rng = np.random.Generator(np.random.PCG64(900 + fmt))
    data = Q.random_blocks(fmt, 64, rng)
    n = 64 * 256
    assert_bit_exact(oracle.dequantize(fmt, data, n), independent(fmt, data, n), Q.NAMES[fmt])
    # every code with scale 1 and min 0: the values are the codes themselves (Q3_K: code - 4)
    d = np.zeros(256, np.uint8)
    d[0:32] = np.tile(np.frombuffer(np.float16(1.0).tobytes(), np.uint8), 16)
    d[132 if fmt != Q5_K else 208:] = 0xFF                                  # the bytes no decoder reads
    lo, hi, width = {Q5_K: (48, 208, 5), Q3_K: (36, 132, 3), Q2_K: (68, 132, 2)}[fmt]
    d[lo:hi] = rng.integers(0, 256, hi - lo, dtype=np.uint8)
    want = bits_lsb_first(d[lo:hi].reshape(16, -1), width, 16).astype(np.float32).ravel() - (4.0 if fmt == Q3_K else 0.0)
    assert np.array_equal(oracle.dequantize(fmt, d, 256), want)


@pytest.mark.parametrize("fmt", FORMATS)
def test_short_input_and_ragged_count(fmt, oracle):
    rng = np.random.Generator(np.random.PCG64(910 + fmt))
    data = Q.random_blocks(fmt, 3, rng)
    full = oracle.dequantize(fmt, data, 768)
    r = oracle.dequantize(fmt, data[:700], 768)                             # the third block is incomplete: loop ends
    assert np.array_equal(r[:512], full[:512]) and np.all(r[512:] == 0.0)
    r = oracle.dequantize(fmt, data, 600)                                   # fewer elements than the blocks hold
    assert r.shape == (600,) and np.array_equal(r, full[:600])


def test_the_dispatcher_reaches_them(oracle):
    assert oracle.lib().rf_data_size(10, 300) == 512 and oracle.lib().rf_block_bytes(13) == 256


# ---------------------------------------------------------------- GPU
@pytest.mark.gpu
@pytest.mark.parametrize("fmt", FORMATS)
def test_gpu_dequant_bit_exact(fmt, oracle, cuda):
    import torch
    from rocmforge_amd import ops
    rng = np.random.Generator(np.random.PCG64(920 + fmt))
    for blocks, n, cut in ((300, 300 * 256, 0), (7, 7 * 256 - 37, 0), (5, 5 * 256, 100), (1, 3, 0)):
        data = Q.random_blocks(fmt, blocks, rng)
        if cut:
            data = data[:-cut]                                              # the last block is incomplete
        got = ops.dequant(fmt, torch.from_numpy(data).to(cuda), n).cpu().numpy()
        assert_bit_exact(got, oracle.dequantize(fmt, data, n), f"{Q.NAMES[fmt]} blocks={blocks} n={n} cut={cut}")
    out = torch.zeros(256 + 1, dtype=torch.float32, device=cuda)            # an output that is not 16-byte aligned
    data = Q.random_blocks(fmt, 1, rng)
    ops.dequant(fmt, torch.from_numpy(data).to(cuda), 256, out=out[1:])
    assert_bit_exact(out[1:].cpu().numpy(), oracle.dequantize(fmt, data, 256), "unaligned output")


@pytest.mark.gpu
@pytest.mark.parametrize("fmt", FORMATS)
def test_matmul_paths_refuse_them(fmt, cuda):
    import torch
    from rocmforge_amd import _lib, ops
    w = torch.zeros(4 * 256, dtype=torch.uint8, device=cuda)
    x = torch.zeros(256, dtype=torch.float32, device=cuda)
    with pytest.raises(_lib.RfqError) as e:
        ops.gemv(fmt, w, x, 4, 256)
    assert e.value.status == _lib.E_UNSUPPORTED
    with pytest.raises(_lib.RfqError) as e:
        ops.gemm_f16(fmt, w, torch.zeros((2, 256), dtype=torch.float16, device=cuda), 4, 256)
    assert e.value.status == _lib.E_UNSUPPORTED
