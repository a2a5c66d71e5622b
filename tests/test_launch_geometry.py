"""Host-only checks of the ``kern[global, local]`` front and of the loader
helpers (behaviour of the reference's numba_mlir/numba_mlir/mlir/kernel_base.py:33-58
and utils.py:17-42, 71-82)."""

import warnings

import pytest

from numba_mlir_amd.mlir import utils
from numba_mlir_amd.mlir.kernel_base import KernelBase


def _kern():
    return KernelBase(lambda a: None)


def test_int_and_tuple_global_sizes():
    k = _kern()
    assert k[7].global_size == (7,)
    assert k[7].local_size == ()
    # kern[(4, 5)] is kern[4, 5] to Python: global 4, local 5
    assert k[(4, 5)].global_size == (4,) and k[(4, 5)].local_size == (5,)
    assert k[(4, 5), ].global_size == (4, 5)
    assert k[[4, 5, 6]].global_size == (4, 5, 6)
    assert k[(8192, 8192), ()].local_size == ()


def test_local_size_is_padded_with_ones():
    k = _kern()
    assert k[(8, 9, 10), (2,)].local_size == (2, 1, 1)
    assert k[(8, 9), (2, 3)].local_size == (2, 3)
    assert k[(8, 9), 4].local_size == (4, 1)


def test_subscript_returns_a_copy():
    k = _kern()
    a, b = k[4], k[(5, 6), (1, 2)]
    assert k.global_size == () and k.local_size == ()
    assert a is not k and a.py_func is k.py_func
    assert (a.global_size, b.global_size) == ((4,), (5, 6))


@pytest.mark.parametrize("bad", [(1, 2, 3, 4), "x", 1.5, None])
def test_bad_global_size(bad):
    with pytest.raises(ValueError):
        _kern()[bad, ()]


def test_bad_subscript_arity_and_rank():
    k = _kern()
    with pytest.raises(ValueError):
        k[4, 4, 4]
    with pytest.raises(ValueError):
        k[(4,), (1, 1)]
    with pytest.raises(ValueError):
        k.check_call_args((), {"x": 1})
    k.check_call_args((1, 2), {})


def test_readenv(monkeypatch):
    monkeypatch.delenv("NMK_TEST_SETTING", raising=False)
    assert utils.readenv("NMK_TEST_SETTING", int, 3) == 3
    assert utils.readenv("NMK_TEST_SETTING", int, lambda: 5) == 5
    monkeypatch.setenv("NMK_TEST_SETTING", "12")
    assert utils.readenv("NMK_TEST_SETTING", int, 3) == 12
    monkeypatch.setenv("NMK_TEST_SETTING", "twelve")
    with warnings.catch_warnings(record=True) as caught:
        warnings.simplefilter("always")
        assert utils.readenv("NMK_TEST_SETTING", int, 3) == 3
    assert any("NMK_TEST_SETTING" in str(w.message) for w in caught)


def test_load_lib_lists_every_attempt(monkeypatch, tmp_path):
    monkeypatch.setenv("PYTHONPATH", str(tmp_path))
    with pytest.raises(ValueError) as err:
        utils.load_lib("no-such-runtime")
    text = str(err.value)
    assert 'load_lib("no-such-runtime") failed' in text
    assert str(tmp_path) in text and str(utils.PACKAGE_DIR) in text
    assert utils.mlir_func_name("f") == "_mlir_ciface_f"
