"""The reference's backend-neutral test bodies (tests/reference_suite.py, tests/layer_suite.py) on
the HIP driver, as test/clj/cortex/compute/cuda/tensor_test.clj runs them on
the CUDA driver.  Needs a GPU."""
import pytest

import reference_suite as rs
import layer_suite as ls
from test_reference_cpu_oracle import ALL_DTYPE_TESTS, FLOAT_TESTS, LAYER_TESTS

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def driver():
    from cortex_amd import capi
    from cortex_amd.driver import HipDriver

    d = HipDriver()
    assert d.get_devices(), "no HIP device visible"
    capi.call("ct_set_debug_sync", 1)
    return d


@pytest.mark.parametrize("datatype", rs.ALL_DTYPES)
@pytest.mark.parametrize("name", ALL_DTYPE_TESTS)
def test_all_dtypes(driver, name, datatype):
    getattr(rs, name)(driver, datatype)


@pytest.mark.parametrize("datatype", rs.FLOAT_DTYPES)
@pytest.mark.parametrize("name", FLOAT_TESTS)
def test_float_double(driver, name, datatype):
    getattr(rs, name)(driver, datatype)


@pytest.mark.parametrize("datatype", rs.FLOAT_DTYPES)
@pytest.mark.parametrize("name", LAYER_TESTS)
def test_layers(driver, name, datatype):
    getattr(ls, name)(driver, datatype)


@pytest.mark.parametrize("datatype", ["int", "long"])
def test_mask(driver, datatype):
    rs.mask(driver, "int")


def test_rand_operator(driver):
    rs.rand_operator(driver, "float")
