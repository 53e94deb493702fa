"""Pins the CPU oracle to the reference's own stored vectors: the reference's
backend-neutral test bodies (tests/reference_suite.py) run on the oracle
driver.  CPU only."""
import pytest

import layer_suite as ls
import reference_suite as rs
from oracle_backend import OracleDriver

ALL_DTYPE_TESTS = ["assign_constant", "assign_marshal", "binary_constant_op", "binary_op", "unary_op", "channel_op",
                   "ternary_op_select", "unary_reduce", "transpose", "select", "select_transpose_interaction",
                   "indexed_tensor", "simple_stream"]
FLOAT_TESTS = ["gemm", "gemv", "activation_forward", "activation_gradient", "softmax", "batch_normalize",
               "batch_normalize_update_and_apply", "batch_normalize_gradients", "convolution_operator", "pooling_operator", "magnitude_and_mag_squared", "constrain_inside_hypersphere", "operations_sugar",
               "adam_trajectory", "sgd_closed_form"]

# tests/layer_suite.py: the layers, loss gradients and regularisers built on the tensor calls
LAYER_TESTS = ["relu_activation", "linear", "activations", "activations_batch", "softmax", "softmax_channels",
               "dropout_bernoulli", "dropout_gaussian", "batch_normalization", "batch_normalization_running",
               "batch_normalization_spatial", "prelu", "basic_conv_layer", "pool_layer_basic", "pool_layer_avg", "pool_layer_avg_exc_pad",
               "concatenate", "split", "join_add", "join_add_ragged", "join_multiply", "loss_gradients",
               "train_small_network"]


@pytest.fixture(scope="module")
def driver():
    return OracleDriver()


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
    # the reference runs the body with :int under both names
    # (test/clj/cortex/compute/cpu/tensor_test.clj:91-92)
    rs.mask(driver, "int")


def test_rand_operator(driver):
    rs.rand_operator(driver, "float")
