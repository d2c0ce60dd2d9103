"""bf16 codec of the CPU checker against torch's dtypes and the committed fixtures; the workload
quantiser's e4m3fn bytes against the committed decode table."""
import os

import numpy as np
import torch

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def test_bf16_decode_exhaustive(oracle):
    bits = np.arange(1 << 16, dtype=np.uint16)
    got = oracle.bf16_to_f32(bits)
    want = torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16).to(torch.float32).numpy()
    np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))


def test_bf16_encode_fixture(oracle):
    fx = np.load(os.path.join(GOLDEN, "bf16_rne_cases.npz"))
    f = fx["f32_bits"].view(np.float32)
    got = oracle.f32_to_bf16(f)
    want = fx["bf16_bits"]
    nan = np.isnan(f)
    np.testing.assert_array_equal(got[~nan], want[~nan])
    # NaN payloads are not pinned, NaN-ness is.
    assert np.isnan(oracle.bf16_to_f32(got[nan])).all()


def test_bf16_encode_live_vs_torch(oracle):
    rng = np.random.default_rng(11)
    f = (rng.standard_normal(200000) * np.exp(rng.uniform(-30, 30, 200000))).astype(np.float32)
    got = oracle.f32_to_bf16(f)
    want = torch.from_numpy(f).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    np.testing.assert_array_equal(got, want)


def test_bf16_ties_to_even_by_hand(oracle):
    # 1.0 = 0x3F800000; half-way to the next bf16 (0x3F81) is 0x3F808000 -> even (0x3F80);
    # 0x3F818000 is half-way between 0x3F81 and 0x3F82 -> even (0x3F82).
    bits = np.array([0x3F808000, 0x3F808001, 0x3F818000, 0x3F817FFF, 0x7F7FFFFF, 0x00000001],
                    dtype=np.uint32)
    got = oracle.f32_to_bf16(bits.view(np.float32))
    assert got.tolist() == [0x3F80, 0x3F81, 0x3F82, 0x3F81, 0x7F80, 0x0000]


def test_fp8_quantiser_uses_ocp_e4m3fn():
    """OCP e4m3fn: bias 7, max 448, no infinities, NaN = 0x7F / 0xFF."""
    from commbench_amd import workloads as wl
    table = np.load(os.path.join(GOLDEN, "e4m3fn_decode.npy"))
    assert table[0x7E] == 448.0 and table[0xFE] == -448.0
    assert np.isnan(table[0x7F]) and np.isnan(table[0xFF])
    assert table[0x38] == 1.0 and table[0x01] == 2.0 ** -9
    # Closed form of every finite byte.
    for b in range(256):
        s, e, m = b >> 7, (b >> 3) & 15, b & 7
        if e == 15 and m == 7:
            continue
        v = (m / 8.0) * 2.0 ** -6 if e == 0 else (1 + m / 8.0) * 2.0 ** (e - 7)
        assert table[b] == (-v if s else v)

    x = wl.bf16_normal(np.random.Generator(np.random.PCG64(5)), 64, 512)
    x[3, 128:256] = 0                                     # an all-zero block
    q, scales = wl.quantize_fp8_blockwise(x)
    qb = q.view(torch.uint8).numpy()
    assert not np.isin(qb, [0x7F, 0xFF]).any()             # saturating: never NaN
    deq = table[qb].reshape(64, 4, 128) * scales.numpy()[:, :, None]
    xf = x.to(torch.float32).numpy().reshape(64, 4, 128)
    amax = np.abs(xf).max(axis=2)
    assert scales[3, 1] == 1.0
    np.testing.assert_allclose(scales.numpy()[amax > 0], (amax / 448.0)[amax > 0], rtol=1e-6)
    # e4m3 has 3 mantissa bits: relative error <= 2^-4 for normals, absolute 2^-10*scale below.
    err = np.abs(deq - xf)
    bound = np.maximum(np.abs(xf) * 2.0 ** -4, scales.numpy()[:, :, None] * 2.0 ** -10)
    assert (err <= bound * 1.0001).all()
    # The block maximum maps to +-448 exactly.
    assert (np.abs(table[qb].reshape(64, 4, 128)).max(axis=2)[amax > 0] == 448.0).all()
