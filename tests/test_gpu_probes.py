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


def test_device_probes_measure_and_validate(dev):
    """fh_probe_device: every kind returns plausible positive figures for this device, leaves its source buffer alone and
    refuses arguments outside its ranges with a message."""
    lib = dev._lib
    out = (C.c_double * 4)()
    check(lib.fh_probe_device(dev._h, 0, 2, 2000, None, 0, out))  # dense MFMA
    assert 500.0 < out[0] < 2600.0 and out[1] > 0  # TFLOP/s: above a fifth of the 2.5 PFLOP/s peak, not above it
    check(lib.fh_probe_device(dev._h, 1, 8, 0, None, 0, out))  # LDS, linear
    lin = out[1]
    check(lib.fh_probe_device(dev._h, 1, 8, 1, None, 0, out))  # operand rows without a swizzle: bank conflicts
    assert lin > 64.0 and out[1] < 0.5 * lin
    check(lib.fh_probe_device(dev._h, 1, 8, 3, None, 0, out))  # the tile kernels' swizzle: as good as linear
    assert out[1] > 0.9 * lin
    cus = dev.info()["compute_units"]
    need = (256 << 10) + cus * 16 * (512 << 10)
    buf = Tensor(dev, (need,), "u8")
    check(lib.fh_memset(dev._h, C.c_void_p(buf.ptr), 7, need))
    check(lib.fh_probe_device(dev._h, 2, 2, 0, C.c_void_p(buf.ptr), need, out))
    assert out[0] > out[1] > 5.0  # L2 hits outrun the HBM stream inside the same compute unit
    head = np.empty(4096, np.uint8)
    check(lib.fh_download(dev._h, head.ctypes.data_as(C.c_void_p), C.c_void_p(buf.ptr), head.size))
    assert (head == 7).all()
    with pytest.raises(FusorHipError, match="buffer"):
        check(lib.fh_probe_device(dev._h, 2, 0, 0, C.c_void_p(buf.ptr), 1 << 20, out))
    with pytest.raises(FusorHipError, match="wavefronts"):
        check(lib.fh_probe_device(dev._h, 1, 5, 0, None, 0, out))
    with pytest.raises(FusorHipError, match="kind"):
        check(lib.fh_probe_device(dev._h, 9, 0, 0, None, 0, out))
