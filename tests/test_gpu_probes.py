"""The two measurement kernels the library exports for the per-launch ceiling of a device (an empty kernel and a plain
streaming read): they launch, they refuse sizes their grid cannot cover, and they leave the data alone."""
import ctypes as C

import numpy as np
import pytest

from kalosm_amd.fusor import FusorHipError, Tensor, check

pytestmark = pytest.mark.gpu


def test_probe_kernels_launch_and_validate(dev):
    lib = dev._lib
    check(lib.fh_probe_empty(dev._h, 1, 64))
    check(lib.fh_probe_empty(dev._h, 256, 1024))
    data = np.arange(4 * 16384, dtype=np.uint8)
    buf = Tensor.from_slice(dev, data, "u8")
    check(lib.fh_probe_read(dev._h, C.c_void_p(buf.ptr), data.size))
    dev.sync()
    assert np.array_equal(buf.as_slice(), data)
    with pytest.raises(FusorHipError, match="16384"):
        check(lib.fh_probe_read(dev._h, C.c_void_p(buf.ptr), 1000))
    with pytest.raises(FusorHipError):
        check(lib.fh_probe_empty(dev._h, 0, 64))
