"""Pins the CPU oracle (oracle/scn_oracle.cpp) against independent statements:
brute-force dictionaries, dense torch routines and closed-form invariants.
The same checks run on the compiled reference where oracle/_ref exists, which
shows that the statements themselves describe the reference."""
import numpy as np
import pytest

import checks
from oracle import cpu_path


def _flavours():
    out = ["oracle"]
    if cpu_path.available("ref"):
        out.append("ref")
    return out


@pytest.fixture(params=_flavours())
def make(request, oracle_built):
    fl = request.param
    return lambda dim: cpu_path.CpuPath(dim, fl)


@pytest.mark.parametrize("mode", [0, 1, 2, 3, 4])
@pytest.mark.parametrize("dim", [2, 3])
def test_input_layer(make, dim, mode):
    checks.check_input_layer(make, dim, mode, seed=10 * dim + mode)


def test_input_layer_no_batch_column(make):
    checks.check_input_layer(make, 3, 4, seed=5, with_batch_col=False)
    checks.check_input_layer(make, 2, 0, seed=6, with_batch_col=False)


@pytest.mark.parametrize("dim", [1, 2, 3])
def test_input_layer_mode0_repeated_points(make, dim):
    checks.check_mode0_repeated_points(make, dim, seed=40 + dim)
    checks.check_mode0_repeated_points(make, dim, seed=50 + dim, spatial=8)


@pytest.mark.parametrize("mode", [0, 1, 2, 3, 4])
@pytest.mark.parametrize("dim", [2, 3])
def test_bl_input_layer(make, dim, mode):
    checks.check_bl_input_layer(make, dim, mode, seed=20 * dim + mode)


def test_bl_input_layer_edge_cases(make):
    checks.check_bl_input_layer(make, 3, 3, seed=1, empties=False)
    checks.check_bl_input_layer(make, 1, 4, seed=2, batch=1, length=300, spatial=40)
    checks.check_bl_input_layer(make, 2, 1, seed=3, batch=5, length=1)


@pytest.mark.parametrize("dim", [1, 2, 3])
def test_input_batch(make, dim):
    checks.check_input_batch(make, dim, seed=70 + dim)


@pytest.mark.parametrize("dim,size,spatial", [(3, 2, 24), (3, 3, 23), (2, 2, (24, 12)), (2, 3, 47), (1, 2, 40)])
def test_generate_rulebooks(make, dim, size, spatial):
    checks.check_generate_rulebooks(make, dim, size, spatial, seed=80 + dim + size)


@pytest.mark.parametrize("dim", [5, 6])
def test_high_dimensions(make, dim):
    # sparseconvnet_cpu.cpp:14-20 instantiates dimensions 1..6
    checks.check_input_layer(make, dim, 4, seed=90 + dim, spatial=3, n=250)
    checks.check_submanifold(make, dim, 3 if dim == 5 else (3, 1, 3, 1, 3, 1), seed=91 + dim, spatial=3, n=150)
    checks.check_strided(make, dim, 2, 2, seed=92 + dim, out_spatial=2, n=150)
    checks.check_s2d(make, dim, seed=93 + dim, spatial=3, n=80)
    checks.check_input_batch(make, dim, seed=94 + dim, spatial=4)


@pytest.mark.parametrize("dim,size", [(1, 3), (2, 3), (3, 3), (2, (3, 1)), (3, (1, 3, 5)), (3, 2),
                                      (4, 3)])
def test_submanifold(make, dim, size):
    checks.check_submanifold(make, dim, size, seed=7 + dim, spatial=8 if dim < 4 else 5,
                             n=200 if dim < 4 else 250, bias=(dim == 2))


@pytest.mark.parametrize("dim,size,stride", [(3, 2, 2), (3, 3, 2), (2, 3, 2), (2, 2, 2), (1, 3, 2),
                                             (2, (3, 2), (2, 1)), (3, 4, 2), (2, 2, 3), (3, 3, 1)])
def test_strided(make, dim, size, stride):
    checks.check_strided(make, dim, size, stride, seed=3 + dim, bias=(dim == 2))


def test_bn(make):
    checks.check_bn(make, seed=1)


def test_nin(make):
    checks.check_nin(make, seed=4)


@pytest.mark.parametrize("dim", [1, 2, 3])
def test_s2d(make, dim):
    checks.check_s2d(make, dim, seed=2 + dim)


@pytest.mark.parametrize("dim", [1, 2, 3, 4])
def test_active_pooling(make, dim):
    checks.check_active_pooling(make, dim, seed=70 + dim)


def test_level_replacement(make):
    checks.check_level_replacement(make)


def test_special_values(make):
    checks.check_special_values(make)


def test_empty(make):
    checks.check_empty(make)


# ---- backward pass: the same independent checks on the oracle and on the compiled reference ----

@pytest.mark.parametrize("dim,size", [(1, 3), (2, 3), (3, 3), (3, 2), (2, (3, 1)), (4, 3)])
def test_conv_backward(make, dim, size):
    checks.check_conv_backward(make, dim, size, seed=30 + dim, spatial=8 if dim < 4 else 5, bias=(dim != 2))


@pytest.mark.parametrize("dim,size,stride", [(3, 2, 2), (3, 3, 2), (2, 3, 2), (2, 2, 2), (1, 3, 2), (2, (3, 2), (2, 1))])
def test_strided_backward(make, dim, size, stride):
    checks.check_strided_backward(make, dim, size, stride, seed=40 + dim)


def test_bn_train(make):
    checks.check_bn_train(make, seed=50)


@pytest.mark.parametrize("mode", [0, 1, 2, 3, 4])
def test_io_backward(make, mode):
    checks.check_io_backward(make, 3, mode, seed=60 + mode)
    checks.check_bl_backward(make, 2, mode, seed=65 + mode)


def test_misc_backward(make):
    checks.check_misc_backward(make, seed=70)
