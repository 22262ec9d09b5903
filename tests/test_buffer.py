"""The buffer interface (test/test_buffer.py of the reference) for device buffers backed by torch
tensors on the ROCm device, and argument forms around it (test/test_dict_args.py,
test/test_normalize.py, test/test_copy.py)."""
import numpy as np
import pytest
import torch

import parpy_amd as parpy
from parpy_amd.buffer import DataType
from parpy_amd.operators import float32, sum

HIP = parpy.CompileBackend.Hip
SHAPE = (20, 10, 32)


def opts_for(p):
    o = parpy.par(p)
    o.backend = HIP
    return o


# ---------------------------------------------------------------- no GPU
def test_shape_carrier_and_unknown_backend():
    a = np.ndarray(SHAPE, dtype=np.float32)
    b = parpy.buffer.from_array(a, None)
    assert b.shape == SHAPE and b.dtype == DataType.from_elem_size(parpy.types.F32)
    with pytest.raises(ValueError, match="Cannot convert to buffer of unknown backend 5"):
        parpy.buffer.from_array(np.ndarray((10,), dtype=np.float32), 5)
    assert parpy.types.I16.size() == 2


@parpy.jit
def normalize_rows(t, nrows, ncols):
    parpy.label('i')
    for i in range(nrows):
        parpy.label('j1')
        s = sum(t[i, :])
        parpy.label('j2')
        t[i, :] /= s


def normalize_rows_loops(t, nrows, ncols):
    parpy.label('i')
    for i in range(nrows):
        s = float32(0.0)
        parpy.label('j1')
        for j in range(ncols):
            s = s + t[i, j]
        parpy.label('j2')
        for j in range(ncols):
            t[i, j] = t[i, j] / s


@parpy.jit
def copy(x, y):
    parpy.label('i')
    y[:] = x[:]


NORM_PAR = {"i": parpy.threads(256), "j1": parpy.threads(128).reduce(), "j2": parpy.threads(128)}


def test_normalize_and_copy_compile():
    t = np.ones((256, 1024), dtype=np.float32)
    assert len(parpy.print_compiled(normalize_rows_loops, [t, 256, 1024], opts_for(NORM_PAR))) != 0
    assert len(parpy.print_compiled(normalize_rows, [t, 256, 1024], opts_for(NORM_PAR))) != 0
    x = np.zeros(10, dtype=np.float32)
    assert len(parpy.print_compiled(copy, [x, x.copy()], opts_for({'i': parpy.threads(1024)}))) != 0


# ---------------------------------------------------------------- GPU
@pytest.mark.gpu
def test_allocation_and_views():
    b = parpy.buffer.empty(SHAPE, parpy.types.F32, HIP)
    assert b.numpy().shape == SHAPE
    b2 = parpy.buffer.empty_like(b)
    assert b.shape == b2.shape and b._get_ptr() != b2._get_ptr()
    z = parpy.buffer.zeros(SHAPE, parpy.types.F32, HIP)
    assert np.array_equal(z.numpy(), np.zeros(SHAPE, dtype=np.float32))
    z2 = parpy.buffer.zeros_like(b)
    assert z2.shape == b.shape and z2._get_ptr() != b._get_ptr() and not z2.numpy().any()
    s = parpy.buffer.empty(SHAPE, parpy.types.I16, HIP)
    assert s.size() == 20 * 10 * 32 * 2
    a = parpy.buffer.zeros(SHAPE, parpy.types.I16, HIP).numpy()
    assert a.shape == SHAPE and a.dtype == np.int16 and not a.any()
    t = parpy.buffer.zeros(SHAPE, parpy.types.I16, HIP).torch()
    assert t.shape == SHAPE and t.dtype == torch.int16 and t.is_cuda and not t.any()


@pytest.mark.gpu
def test_conversions():
    a = np.ndarray(SHAPE, dtype=np.float32)
    b = parpy.buffer.from_array(a, HIP)
    assert b.shape == SHAPE and b.dtype == DataType.from_elem_size(parpy.types.F32) and b.src is a
    assert float(parpy.buffer.from_array(np.array(2.5, dtype=np.float32), HIP)) == 2.5
    assert int(parpy.buffer.from_array(np.array(2, dtype=np.int32), HIP)) == 2
    assert bool(parpy.buffer.from_array(torch.tensor(True, dtype=torch.bool), HIP))
    r = np.random.default_rng(1).standard_normal(SHAPE)
    assert np.array_equal(parpy.buffer.from_array(r, HIP).numpy(), r)


@pytest.mark.gpu
def test_reshape_shares_and_counts_references():
    b1 = parpy.buffer.zeros(SHAPE, parpy.types.F32, HIP)
    assert b1.refcount[0] == 1
    b2 = b1.reshape(200, 32)
    assert b1.shape == SHAPE and b2.shape == (200, 32)
    assert b1.refcount[0] == 2 and b2.refcount[0] == 2
    del b2
    assert b1.refcount[0] == 1
    with pytest.raises(ValueError, match="Cannot reshape buffer of shape.*to.*"):
        b1.reshape(20, 10, 32, 2)


@pytest.mark.gpu
def test_element_type_changes():
    b1 = parpy.buffer.zeros(SHAPE, parpy.types.I32, HIP)
    b2 = b1.with_type(parpy.types.U32)
    assert b1.dtype == DataType.from_elem_size(parpy.types.I32) and b2.dtype == DataType.from_elem_size(parpy.types.U32)
    assert b1._get_ptr() == b2._get_ptr()          # same width: a reinterpretation
    b3 = b1.with_type(parpy.types.F64)
    assert b3.dtype == DataType.from_elem_size(parpy.types.F64) and b1._get_ptr() != b3._get_ptr()


@pytest.mark.gpu
def test_dictionary_arguments():
    @parpy.jit
    def add_fields(x, y):
        with parpy.gpu:
            y[0] = x["a"][0] + x["b"][0]
    x = {'a': torch.tensor([4], dtype=torch.int64), 'b': torch.tensor([2], dtype=torch.int64)}
    y = torch.tensor([0], dtype=torch.int32)
    add_fields(x, y, opts=opts_for({}))
    assert y[0] == 6

    @parpy.jit
    def nested(x, y):
        with parpy.gpu:
            y[0] = x['a']['b']
    with pytest.raises(RuntimeError, match=r".*nested dictionary.*"):
        nested({'a': {'b': torch.tensor([3], dtype=torch.int64)}}, y, opts=opts_for({}))


@pytest.mark.gpu
def test_normalize_copy_and_buffers_as_arguments():
    t = torch.ones((1, 1024), dtype=torch.float32)
    out = t.clone()
    normalize_rows(out, 1, 1024, opts=opts_for({"i": parpy.threads(256)}))
    assert torch.allclose(out, torch.nn.functional.normalize(t, p=1, dim=1), 1e-5)
    t = torch.rand((256, 1024), dtype=torch.float32) + 0.5
    out = t.clone()
    normalize_rows(out, 256, 1024, opts=opts_for(NORM_PAR))
    assert torch.allclose(out, torch.nn.functional.normalize(t, p=1, dim=1), 1e-5)
    x = torch.randn(10, dtype=torch.float32)
    y = torch.zeros_like(x)
    copy(x, y, opts=opts_for({'i': parpy.threads(1024)}))
    assert torch.equal(x, y)
    # buffers made by the user are passed as they are and stay on the device
    xb = parpy.buffer.from_array(x.numpy(), HIP)
    yb = parpy.buffer.zeros((10,), parpy.types.F32, HIP)
    copy(xb, yb, opts=opts_for({'i': parpy.threads(1024)}))
    assert np.array_equal(yb.numpy(), x.numpy())
