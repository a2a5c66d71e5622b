"""Host-side tests of libnumba-mlir-python-runtime-hip.so: the unboxer of
objects that carry ``__hip_array_interface__`` and the MemInfo helpers
(counterparts of the reference's python_runtime/lib/Boxing.cpp:45-136 and
PythonRt.cpp:29-47).  No GPU: the addresses are never dereferenced."""

import ctypes

import numpy as np
import pytest

from numba_mlir_amd.mlir import python_rt


class Described:
    def __init__(self, **fields):
        self.__hip_array_interface__ = fields


def _iface(a, strides="elements"):
    s = None
    if strides == "elements" and not a.flags.c_contiguous:
        s = tuple(x // a.itemsize for x in a.strides)
    return dict(data=(a.ctypes.data, False), shape=a.shape, strides=s,
                typestr=a.dtype.str, version=1)


@pytest.mark.parametrize("dtype", ["f4", "f8", "i1", "i8", "c16", "b1"])
@pytest.mark.parametrize("shape", [(), (7,), (3, 5), (2, 3, 4)])
def test_dense_arrays(dtype, shape):
    a = np.zeros(shape, dtype)
    obj = Described(**_iface(a))
    rec = python_rt.unbox(obj)
    assert rec.data == (a.ctypes.data or None) and rec.parent == id(obj)
    assert rec.nitems == a.size and rec.itemsize == a.itemsize
    assert tuple(rec.shape) == a.shape and tuple(rec.strides) == a.strides
    info = python_rt.MemInfo.from_address(rec.meminfo)
    assert info.refct == 1 and info.dtor is None and info.data == rec.data
    assert info.size == a.nbytes


def test_strides_are_given_in_elements():
    base = np.zeros((6, 8), np.float32)
    for view in (base.T, base[::2, 1::3], base[:, ::-1]):
        rec = python_rt.unbox(Described(**_iface(view)))
        assert tuple(rec.shape) == view.shape and tuple(rec.strides) == view.strides
        assert rec.data == view.ctypes.data
    # "strides" may also be left out of the dict altogether
    fields = _iface(base)
    del fields["strides"]
    assert tuple(python_rt.unbox(Described(**fields)).strides) == base.strides


def test_what_is_not_an_array_is_refused_with_a_reason():
    a = np.zeros(4)
    good = _iface(a)
    with pytest.raises(AttributeError):
        python_rt.unbox(object(), ndim=1)
    for change, match in [
            (dict(data=a.ctypes.data), "'data' must be"),
            (dict(data=("0x10", False)), "'data' must be"),
            (dict(shape=[4]), "'shape' must be a tuple"),
            (dict(shape=(4.0,)), "'shape' must hold ints"),
            (dict(shape=(-4,)), "negative extent"),
            (dict(typestr="float64"), "'typestr' must be"),
            (dict(typestr=b"<f8"), "'typestr' must be"),
            (dict(strides=(1, 1)), "'strides' must be None or one int per dimension"),
            (dict(data=(0, False)), "null address"),
    ]:
        fields = dict(good)
        fields.update(change)
        with pytest.raises((TypeError, ValueError), match=match):
            python_rt.unbox(Described(**fields), ndim=1)
    obj = Described()
    obj.__hip_array_interface__ = [1, 2]
    with pytest.raises(TypeError, match="not a dict"):
        python_rt.unbox(obj, ndim=1)
    # an empty array may have no address at all
    fields = dict(good, data=(0, False), shape=(0,))
    assert python_rt.unbox(Described(**fields)).nitems == 0


def test_rank_must_match_the_record():
    """The unboxer writes two integers per dimension of the OBJECT: a record
    typed for fewer dimensions would be overrun."""
    a = np.zeros((3, 5), np.float32)
    obj = Described(**_iface(a))
    for ndim in (0, 1, 3):
        with pytest.raises(TypeError, match="2-dimensional"):
            python_rt.unbox(obj, ndim=ndim)
    assert tuple(python_rt.unbox(obj, ndim=2).shape) == (3, 5)


def test_meminfo_carries_its_destructor():
    seen = []
    dtor_type = ctypes.CFUNCTYPE(None, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p)
    dtor = dtor_type(lambda ptr, size, info: seen.append((ptr, size, info)))
    address = python_rt.runtime_lib.nmrtAllocMemInfo(
        0x1000, 256, ctypes.cast(dtor, ctypes.c_void_p), 0x77)
    info = python_rt.MemInfo.from_address(address)
    assert (info.refct, info.data, info.size, info.dtor_info) == (1, 0x1000, 256, 0x77)
    # what NRT does when the last reference goes
    dtor_type(info.dtor)(info.data, info.size, info.dtor_info)
    assert seen == [(0x1000, 256, 0x77)]
    assert set(python_rt.SYMBOLS) == {"nmrtAllocMemInfo", "nmrtUnboxHipInterface"}
