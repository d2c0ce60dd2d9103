"""Writes the codec fixtures used by tests/test_oracle_codec.py.

Source of truth: torch's own dtypes on the CPU (a library, not reference code).
  bf16_rne_cases.npz   float32 inputs (bit patterns) and torch.bfloat16 bit patterns, covering
                       every exponent, ties, near-ties, subnormals, infinities and NaNs
  e4m3fn_decode.npy    float32 value of each of the 256 OCP e4m3fn bytes (NaN kept)
Run from the repository root:  python tests/golden/make_codec_fixtures.py
"""
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def main():
    rng = np.random.Generator(np.random.PCG64(20240607))
    hi = np.arange(0, 1 << 16, dtype=np.uint32) << 16          # every bf16 value, exact
    lows = np.array([0x0000, 0x0001, 0x7FFF, 0x8000, 0x8001, 0xFFFF], dtype=np.uint32)
    grid = (hi[::37, None] | lows[None, :]).reshape(-1)          # ties and near-ties
    rand = rng.integers(0, 1 << 32, size=6000, dtype=np.uint64).astype(np.uint32)
    bits = np.concatenate([hi[::5], grid, rand]).astype(np.uint32)
    f = torch.from_numpy(bits.view(np.float32).copy())
    out = f.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    np.savez_compressed(os.path.join(HERE, "bf16_rne_cases.npz"), f32_bits=bits, bf16_bits=out)

    b = torch.arange(256, dtype=torch.int32).to(torch.uint8).view(torch.float8_e4m3fn)
    np.save(os.path.join(HERE, "e4m3fn_decode.npy"), b.to(torch.float32).numpy())


if __name__ == "__main__":
    main()
