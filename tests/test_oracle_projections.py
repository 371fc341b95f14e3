"""Pins oracle/projections.py: against torch's own linear + autograd, and against
a closed form of the whole MultiHeadAttention forward."""
import numpy as np
import torch

from oracle import projections as P


def test_linear_matches_torch_functional_linear_and_autograd():
    rng = np.random.default_rng(3)
    x = rng.standard_normal((37, 24))
    W = rng.standard_normal((40, 24))      # non-square: a transposed operand cannot pass
    b = rng.standard_normal(40)
    dy = rng.standard_normal((37, 40))
    xt = torch.tensor(x, requires_grad=True)
    Wt = torch.tensor(W, requires_grad=True)
    bt = torch.tensor(b, requires_grad=True)
    yt = torch.nn.functional.linear(xt, Wt, bt)
    yt.backward(torch.tensor(dy))
    np.testing.assert_allclose(P.linear_forward(x, W, b), yt.detach().numpy(), rtol=1e-12, atol=1e-12)
    dx, dW, db = P.linear_backward(x, W, dy)
    np.testing.assert_allclose(dx, xt.grad.numpy(), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(dW, Wt.grad.numpy(), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(db, bt.grad.numpy(), rtol=1e-12, atol=1e-12)


def test_linear_known_answer():
    # y[n, o] = sum_i x[n, i] W[o, i] + b[o], by hand
    x = np.array([[1.0, 2.0], [0.0, -1.0]])
    W = np.array([[1.0, 0.0], [0.0, 1.0], [2.0, 3.0]])
    b = np.array([0.5, 0.0, -1.0])
    np.testing.assert_array_equal(P.linear_forward(x, W, b), np.array([[1.5, 2.0, 7.0], [0.5, -1.0, -4.0]]))


def test_module_forward_closed_form_with_zero_query_weights():
    """linear_q = 0 makes every score 0, every edge weight exp(0) = 1, so
    out_i = mean over in-neighbours of v, times deg/(deg + 1e-6); then the output
    linear.  A swapped source/destination, a dropped bias or a transposed weight
    changes the result."""
    rng = np.random.default_rng(11)
    S, hidden, H = 9, 16, 4
    x = rng.standard_normal((1, S, hidden))
    params = {
        "linear_q.weight": np.zeros((hidden, hidden)), "linear_q.bias": np.zeros(hidden),
        "linear_k.weight": rng.standard_normal((hidden, hidden)), "linear_k.bias": rng.standard_normal(hidden),
        "linear_v.weight": rng.standard_normal((hidden, hidden)), "linear_v.bias": rng.standard_normal(hidden),
        "output_layer.weight": rng.standard_normal((hidden, hidden)), "output_layer.bias": rng.standard_normal(hidden),
    }
    src = np.array([0, 1, 2, 3, 3, 4, 5, 0, 8, 8])
    dst = np.array([1, 1, 1, 0, 2, 2, 5, 7, 7, 7])      # nodes 3, 4, 6, 8 receive nothing
    got = P.multi_head_attention_forward(x, params, np.stack([src, dst]), H)
    v = x[0] @ params["linear_v.weight"].T + params["linear_v.bias"]
    agg = np.zeros_like(v)
    for i in range(S):
        nb = src[dst == i]
        if len(nb):
            agg[i] = v[nb].sum(0) / (len(nb) + 1e-6)
    want = agg @ params["output_layer.weight"].T + params["output_layer.bias"]
    np.testing.assert_allclose(got[0], want, rtol=1e-12, atol=1e-12)
    # without an output layer (GT flavour) the aggregate itself comes back
    del params["output_layer.weight"], params["output_layer.bias"]
    np.testing.assert_allclose(P.multi_head_attention_forward(x, params, np.stack([src, dst]), H)[0], agg,
                               rtol=1e-12, atol=1e-12)
