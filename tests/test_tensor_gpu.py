"""Tensor::copyFromAsync between host and device with and without a dtype change (Tensor.cpp:731-866 of the reference):
the converting forms stage through a temporary device tensor that a stream callback keeps alive."""
from __future__ import annotations

import numpy as np
import pytest

import oracle
from helpers import cpu_tensor, gpu_tensor
from thor_amd import physical as ph
from thor_amd.dtypes import DataType

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("device_dtype", [DataType.fp16, DataType.bf16, DataType.fp8_e4m3, DataType.fp32], ids=lambda d: d.name)
def test_host_device_round_trip_with_conversion(gpu, device_dtype):
    stream = ph.Stream(0)
    rng = np.random.default_rng(21)
    x = (rng.standard_normal((37, 129)) * 4).astype(np.float32)
    host = cpu_tensor(x.shape, DataType.fp32)
    host.numpy()[...] = x
    for _ in range(3):  # repeated so that tensors kept alive by earlier copies are released in between
        device = gpu_tensor(x.shape, device_dtype)
        device.copy_from_async(host, stream)          # host fp32 -> device dtype (converted on the GPU)
        back = cpu_tensor(x.shape, DataType.fp32)
        back.copy_from_async(device, stream)          # device dtype -> host fp32
        stream.synchronize()
        if device_dtype == DataType.fp32:
            np.testing.assert_array_equal(back.numpy(), x)
        else:
            narrow = oracle.convert(x, oracle.FP32, int(device_dtype))
            want = oracle.convert(narrow, int(device_dtype), oracle.FP32).reshape(x.shape)
            np.testing.assert_array_equal(back.numpy().view(np.uint32), want.view(np.uint32))


def test_device_to_device_and_host_to_host_conversion(gpu):
    stream = ph.Stream(0)
    x = np.linspace(-300, 300, 4097, dtype=np.float32)
    host = cpu_tensor(x.shape, DataType.fp32)
    host.numpy()[...] = x
    d32 = gpu_tensor(x.shape, DataType.fp32)
    d32.copy_from_async(host, stream)
    d16 = gpu_tensor(x.shape, DataType.bf16)
    d16.copy_from_async(d32, stream)
    h16 = cpu_tensor(x.shape, DataType.bf16)
    h16.copy_from_async(d16, stream)
    hh = cpu_tensor(x.shape, DataType.fp16)
    hh.copy_from_async(host, stream)                  # host -> host runs the CPU converter in a stream callback
    stream.synchronize()
    np.testing.assert_array_equal(h16.numpy(), oracle.convert(x, oracle.FP32, oracle.BF16))
    np.testing.assert_array_equal(hh.numpy().view(np.uint16), oracle.convert(x, oracle.FP32, oracle.FP16).view(np.uint16))
    with pytest.raises(ValueError, match="element counts"):
        gpu_tensor([5], DataType.fp32).copy_from_async(host, stream)


def test_alias_view_rejects_strides_that_wrap_around(gpu):
    """A stride large enough for (dim - 1) * stride to wrap past 2^64 must not pass the bounds check of aliasView."""
    t = gpu_tensor([4, 6], DataType.fp32)
    ok = t.alias_view([6, 4], [1, 6])
    assert ok.get_dimensions() == [6, 4]
    huge = (1 << 63) + 3  # 2 * huge wraps to 6
    with pytest.raises(Exception, match="outside the backing allocation"):
        t.alias_view([3, 2], [huge, 1])
    with pytest.raises(Exception, match="outside the backing allocation"):
        t.alias_view([2], [1], (1 << 64) - 1)
    with pytest.raises(Exception, match="outside the backing allocation"):
        t.alias_view([4, 7], [6, 1])


def test_numpy_view_keeps_its_tensor_alive(gpu):
    """The array returned by numpy() must hold the pinned allocation: dropping the tensor first may not free the memory."""
    import gc
    host = cpu_tensor([1024], DataType.fp32)
    view = host.numpy()
    view[...] = np.arange(1024, dtype=np.float32)
    del host
    gc.collect()
    filler = [cpu_tensor([1024], DataType.fp32) for _ in range(8)]  # would reuse the freed block
    for f in filler:
        f.numpy()[...] = -1.0
    np.testing.assert_array_equal(view, np.arange(1024, dtype=np.float32))
