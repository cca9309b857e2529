"""The reference's golden outputs reproduced through the HIP C-ABI, operator by operator."""
import numpy as np
import pytest

from tests import graph_runner as gr
from tests.test_oracle_golden import MODELS, golden_tolerance

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("model", MODELS)
def test_hip_reproduces_reference_golden_output(rt, model):
    g, inputs, expected = gr.load_fixture(model)
    print("golden", model, flush=True)
    got = gr.run(g, inputs, gr.HipBackend(rt)).ravel()
    assert got.shape == expected.shape
    assert np.abs(got - expected).max() <= golden_tolerance(model, expected)
    # and against the oracle on the same inputs: 1e-5 relative to the output scale
    want = gr.run(g, inputs, gr.OracleBackend()).ravel()
    assert np.abs(got - want).max() <= 1e-5 * max(1.0, float(np.abs(want).max()))
