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
               "batch_normalize_update_and_apply", "batch_normalize_gradients", "convolution_operator", "pooling_operator", "lrn_operator", "magnitude_and_mag_squared", "constrain_inside_hypersphere", "operations_sugar",
               "adam_trajectory", "sgd_closed_form"]

# tests/layer_suite.py: the layers, loss gradients and regularisers built on the tensor calls
LAYER_TESTS = ["relu_activation", "linear", "activations", "activations_batch", "softmax", "softmax_channels",
               "dropout_bernoulli", "dropout_gaussian", "batch_normalization", "batch_normalization_running",
               "batch_normalization_spatial", "prelu", "basic_conv_layer", "pool_layer_basic", "pool_layer_avg", "pool_layer_avg_exc_pad", "lrn_forward",
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


def test_convolution_and_pooling_front_end_checks(driver):
    """The argument checks of tensor.clj:1320-1551 that run before a backend is reached."""
    import numpy as np
    from cortex_amd import tensor as ct
    with rs.context(driver, "float"):
        desc = ct.convolution_descriptor("float", 3, 4, 3, 3, 0, 0, 1, 1)
        assert ct.get_convolution_output_dimensions(desc, 4, 4) == {"output-width": 2, "output-height": 2}
        algorithms = ct.choose_convolution_algorithms(desc, 4, 4, 2, 1000)
        assert algorithms == {"workspace-size": 2 * 2 * 2 * 36}
        inp, out = ct.new_tensor([2, 4, 4, 4]), ct.new_tensor([2, 3, 2, 2])
        weights, work = ct.new_tensor([3, 36]), ct.new_tensor([algorithms["workspace-size"]])
        ct.convolution_forward(out, 0.0, inp, weights, work, desc, algorithms)
        with pytest.raises(ct.TensorError, match="Output dimensions"):
            ct.convolution_forward(ct.new_tensor([2, 3, 3, 3]), 0.0, inp, weights, work, desc, algorithms)
        with pytest.raises(ct.TensorError, match="Input dimensions"):
            ct.convolution_forward(out, 0.0, ct.new_tensor([2, 5, 4, 4]), weights, work, desc, algorithms)
        with pytest.raises(ct.TensorError, match="nil"):
            ct.convolution_descriptor("float", 3, None, 3, 3, 0, 0, 1, 1)
        with pytest.raises(Exception, match="workspace"):
            ct.convolution_forward(out, 0.0, inp, weights, ct.new_tensor([10]), desc, algorithms)
        # the two rounding rules of the output size (tensor.clj:1351-1365)
        pool = ct.pooling_descriptor("float", 4, 2, 2, 0, 0, 2, 2)
        assert pool["dimension-op"] == "ceil" and pool["pool-op"] == "max"
        assert ct.get_convolution_output_dimensions(pool, 5, 5) == {"output-width": 3, "output-height": 3}
        floor = ct.pooling_descriptor("float", 4, 2, 2, 0, 0, 2, 2, dimension_op="floor")
        assert ct.get_convolution_output_dimensions(floor, 5, 5) == {"output-width": 2, "output-height": 2}
        with pytest.raises(ct.TensorError, match="three possible pool operations"):
            ct.pooling_descriptor("float", 4, 2, 2, 0, 0, 2, 2, pool_op="median")
        with pytest.raises(ct.TensorError, match="Output dimensions"):
            ct.pooling_forward(ct.new_tensor([2, 4, 2, 2]), 0.0, ct.new_tensor([2, 4, 5, 5]), pool)
        ints = ct.new_tensor([2, 4, 5, 5], "int")
        with pytest.raises(ct.TensorError):
            ct.pooling_forward(ct.new_tensor([2, 4, 3, 3], "int"), 0.0, ints, pool)
