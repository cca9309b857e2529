"""Pins the CPU oracle to the reference: every golden output the reference's own tests hold for the
Gemm / Conv / epilogue path is reproduced within the reference's test tolerance (1e-3 absolute,
tests/common/test_helpers.h:22; most agree to 1e-6)."""
import json
import os

import numpy as np
import pytest

from tests import graph_runner as gr

# references printed with 4 decimals
FOUR_DECIMALS = ("Gelu", "GeluTanh", "LinearWithLeakyRelu", "AvgPool", "MaxPool1d", "MaxPool2d", "AvgPoolPad", "AvgPoolCountIncludePad",
                 "Exp", "Log", "Neg", "Elu", "SeluNonDefaultCoeffs", "Softmax3d", "Softmax4d", "LayerNormalization2d", "LayerNormalization4d")


# Inputs AND outputs printed with 4 decimals, the outputs computed from the unrounded inputs: the rounding of an input
# reaches the output multiplied by the operator's slope (1/x^2 = 25 at x = 0.2), so these two are held to the
# tolerance of the reference's own test (DEFAULT_TOLERANCE = 1e-3, tests/alpaka/TestAlpakaCommon.h:10).
INPUT_ROUNDED = ("Reciprocal", "Sqrt")
# The same, for operators whose slope is at most 1: half a unit of the fourth decimal from the input plus half a unit from the output.
INPUT_ROUNDED_GENTLE = ("Tanh", "Erf")


def golden_tolerance(model, expected):
    """Half a unit of the last printed digit of the reference file, plus fp32 rounding of the result."""
    if model in INPUT_ROUNDED:
        return 1e-3
    if model in INPUT_ROUNDED_GENTLE:
        return 1.1e-4
    if model in FOUR_DECIMALS:
        return 0.6e-4
    return 2e-5 + 2e-6 * float(np.abs(expected).max())


MODELS = sorted(json.load(open(os.path.join(gr.GOLDEN, "fixtures.json"))).keys())


@pytest.mark.parametrize("model", MODELS)
def test_oracle_reproduces_reference_golden_output(model):
    g, inputs, expected = gr.load_fixture(model)
    got = gr.run(g, inputs, gr.OracleBackend()).ravel()
    assert got.shape == expected.shape
    assert np.abs(got - expected).max() <= golden_tolerance(model, expected), np.abs(got - expected).max()
