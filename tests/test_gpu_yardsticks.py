"""GPU checks of the bandwidth yardsticks (16-byte streams, the access width of the reference's
example077_GPU_vectorized_copy_widths, .cu:27-33,126-143): what they write, and only that."""
import numpy as np
import pytest
import torch

from commbench_amd import _lib

from . import gpu_util as gu

pytestmark = pytest.mark.gpu

EINVAL = -22
GUARD = 64          # guard bytes on both sides of every destination
WRITE_PATTERN = np.array([0x01010101, 0x02020202, 0x03030303, 0x04040404], dtype=np.uint32).view(np.uint8)


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _guarded(nbytes):
    """A destination of nbytes with guard bytes before and after, all 0xA5; returns (whole, view)."""
    whole = torch.full((nbytes + 2 * GUARD,), 0xA5, dtype=torch.uint8, device=gu.DEV)
    return whole, whole[GUARD:GUARD + nbytes]


@pytest.mark.parametrize("nbytes", [16, 4096 - 16, (1 << 20) + 48, 1 << 30])
def test_copy_yardstick_reproduces_the_source_and_nothing_more(nbytes):
    print(f"copy {nbytes} bytes", flush=True)
    lib = _lib.load()
    gen = torch.Generator(device=gu.DEV).manual_seed(nbytes % 1000)
    src = torch.randint(0, 256, (nbytes,), dtype=torch.uint8, device=gu.DEV, generator=gen)
    keep = src.clone()
    whole, dst = _guarded(nbytes)
    _lib.check(lib.mi_ep_copy_yardstick(dst.data_ptr(), src.data_ptr(), nbytes, _stream()), "copy yardstick")
    torch.cuda.synchronize()
    assert torch.equal(dst, keep)
    assert torch.equal(src, keep)                                         # the source is only read
    assert bool((whole[:GUARD] == 0xA5).all()) and bool((whole[GUARD + nbytes:] == 0xA5).all())


@pytest.mark.parametrize("nbytes", [16, 4096 - 16, (1 << 20) + 48, 1 << 28])
def test_write_yardstick_fills_exactly_its_bytes(nbytes):
    print(f"write {nbytes} bytes", flush=True)
    lib = _lib.load()
    whole, dst = _guarded(nbytes)
    _lib.check(lib.mi_ep_write_yardstick(dst.data_ptr(), nbytes, _stream()), "write yardstick")
    torch.cuda.synchronize()
    pattern = torch.from_numpy(WRITE_PATTERN.copy()).to(gu.DEV)
    assert torch.equal(dst.view(-1, 16), pattern.expand(nbytes // 16, 16))
    assert bool((whole[:GUARD] == 0xA5).all()) and bool((whole[GUARD + nbytes:] == 0xA5).all())


@pytest.mark.parametrize("nbytes", [16, (1 << 20) + 48, 1 << 28])
def test_read_yardstick_writes_nothing(nbytes):
    print(f"read {nbytes} bytes", flush=True)
    lib = _lib.load()
    gen = torch.Generator(device=gu.DEV).manual_seed(7)
    src = torch.randint(0, 256, (nbytes,), dtype=torch.uint8, device=gu.DEV, generator=gen)
    keep = src.clone()
    sink = torch.full((4,), 0x5A5A5A5A, dtype=torch.int32, device=gu.DEV)
    _lib.check(lib.mi_ep_read_yardstick(src.data_ptr(), nbytes, sink.data_ptr(), _stream()), "read yardstick")
    torch.cuda.synchronize()
    assert torch.equal(src, keep)
    assert bool((sink == 0x5A5A5A5A).all())        # random bytes do not fold to the one value that is stored


def test_yardsticks_check_their_arguments():
    lib = _lib.load()
    buf = torch.zeros(256, dtype=torch.uint8, device=gu.DEV)
    p = buf.data_ptr()
    assert p % 16 == 0
    s = _stream()
    assert lib.mi_ep_copy_yardstick(p, p + 64, 24, s) == EINVAL           # size not a multiple of 16
    assert lib.mi_ep_copy_yardstick(p + 8, p + 64, 32, s) == EINVAL       # destination misaligned
    assert lib.mi_ep_copy_yardstick(p, p + 72, 32, s) == EINVAL           # source misaligned
    assert lib.mi_ep_copy_yardstick(None, p, 32, s) == EINVAL
    assert lib.mi_ep_write_yardstick(p + 4, 32, s) == EINVAL
    assert lib.mi_ep_write_yardstick(p, 40, s) == EINVAL
    assert lib.mi_ep_read_yardstick(p, 32, None, s) == EINVAL             # no sink
    assert lib.mi_ep_read_yardstick(p + 4, 32, p + 128, s) == EINVAL
    assert lib.mi_ep_read_yardstick(p, 20, p + 128, s) == EINVAL
    assert lib.mi_ep_copy_yardstick(p, p + 64, 0, s) == 0                 # nothing to do is not an error
    torch.cuda.synchronize()
    assert not buf.any()
