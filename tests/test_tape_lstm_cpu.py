"""The reverse-mode tape on the oracle backend alone (no GPU): the LSTM graph's parameter
gradients against central finite differences of its loss.  Pins the gradient wiring of slice,
elementwise product, sigmoid and tanh that the GPU graph test then relies on."""
import numpy as np
import pytest

from oracle_backend import OracleBackend
from tsplit_amd import graph, workloads


def _run(store, x, y):
    t = graph.Tape(OracleBackend())
    b = workloads.Binder(t, store)
    loss, logits = workloads.lstm(t, b, b.input(x), b.input(y), dim_input=5, dim_hidden=6, classes=4, steps=4, std=0.5)
    return t, b, loss, logits


@pytest.mark.parametrize("name", ["lstm_input_gate_u", "lstm_forget_gate_w", "lstm_tanh_b", "lstm_out_weight",
                                  "lstm_output_gate_u", "lstm_out_bias"])
def test_lstm_gradients_match_finite_differences(name):
    rng = np.random.RandomState(0)
    x = rng.uniform(0, 1, size=(3, 4 * 5)).astype(np.float32)
    y = np.zeros((3, 4), np.float32)
    y[np.arange(3), [0, 2, 1]] = 1
    store = workloads.ParamStore(1)
    t, b, loss, logits = _run(store, x, y)
    assert logits.shape == (3, 4)
    t.backward(loss)
    g = np.asarray(b.grads()[name])
    direction = np.sign(g).astype(np.float32)
    eps, losses = 1e-2, []
    for sgn in (+1, -1):
        st = workloads.ParamStore(1)
        st.values = {k: v.copy() for k, v in store.values.items()}
        st.trainable = dict(store.trainable)
        st.values[name] = st.values[name] + sgn * eps * direction.reshape(st.values[name].shape)
        losses.append(float(np.asarray(_run(st, x, y)[2].value).reshape(-1)[0]))
    fd = (losses[0] - losses[1]) / (2 * eps)
    assert abs(fd - np.abs(g).sum()) <= 2e-3 * np.abs(g).sum() + 1e-6


def test_lstm_untrainable_initial_state_gets_no_gradient():
    rng = np.random.RandomState(0)
    x = rng.uniform(0, 1, size=(2, 20)).astype(np.float32)
    y = np.eye(4, dtype=np.float32)[[1, 3]]
    store = workloads.ParamStore(1)
    t, b, loss, _ = _run(store, x, y)
    t.backward(loss)
    assert "initial_state" not in b.grads()
    assert set(b.grads()) == {k for k, tr in store.trainable.items() if tr}
