"""Lowering of Transform.Elementwise functions to the closed op vocabulary of the C ABI."""
import pytest

from gemmkernels import Transform, ConfigError
from gemmkernels.transform import SCALE, ADD, RELU, NEG, ABS, CLAMP, SQUARE

E = Transform.Elementwise


def test_identity():
    assert E().is_identity and E(lambda x: x).is_identity and E(Transform.identity).ops == ()


def test_recognised_functions():
    assert E(lambda x: x * 0.5).ops == ((SCALE, 0.5, 0.0),)
    assert E(lambda x: 2 * x).ops == ((SCALE, 2.0, 0.0),)
    assert E(lambda x: x / 4).ops == ((SCALE, 0.25, 0.0),)
    assert E(lambda x: x + 1).ops == ((ADD, 1.0, 0.0),)
    assert E(lambda x: x - 1).ops == ((ADD, -1.0, 0.0),)
    assert E(lambda x: 1 - x).ops == ((NEG, 0.0, 0.0), (ADD, 1.0, 0.0))
    assert E(lambda x: -x).ops == ((NEG, 0.0, 0.0),)
    assert E(abs).ops == ((ABS, 0.0, 0.0),)
    assert E(Transform.relu).ops == ((RELU, 0.0, 0.0),)
    assert E(lambda x: Transform.maximum(x, 0)).ops == ((RELU, 0.0, 0.0),)
    assert E(lambda x: Transform.clamp(x, -1, 1)).ops == ((CLAMP, -1.0, 1.0),)
    assert E(lambda x: x * x).ops == ((SQUARE, 0.0, 0.0),) and E(lambda x: x ** 2).ops == ((SQUARE, 0.0, 0.0),)
    assert E(lambda x: Transform.relu(x * 2 + 1)).ops == ((SCALE, 2.0, 0.0), (ADD, 1.0, 0.0), (RELU, 0.0, 0.0))


def test_host_evaluation_matches_the_function():
    f = E(lambda x: Transform.relu(x * 2 - 1))
    assert f(3.0) == 5.0 and f(0.25) == 0.0


def test_unsupported_functions_raise_config_error():
    with pytest.raises(ConfigError):
        E(lambda x: max(x, 0))              # data-dependent control flow
    with pytest.raises(ConfigError):
        E(lambda x: x ** 3)
    with pytest.raises(ConfigError):
        E(lambda x: 1.0)                    # does not depend on its argument
    with pytest.raises(ConfigError):
        E(lambda x: ((((x + 1) * 2) + 3) * 4) + 5)   # more than four ops
    with pytest.raises(ConfigError):
        E(lambda x: x * (x + 1))            # product of two expressions
