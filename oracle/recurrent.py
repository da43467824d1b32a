"""TEST INFRASTRUCTURE: float64 restatement of the recurrent networks of the reference's examples
(examples/walking.py:40-208).  The GRU cell follows eqx.nn.GRUCell's equations (equinox is a third-party dependency
that is not in the reference tree): gi = W_ih x + b, gh = W_hh h, r = s(gi_r + gh_r), z = s(gi_z + gh_z),
n = tanh(gi_n + r (gh_n + b_n)), h' = n + z (h - n).  Pinned by torch.nn.GRUCell, which computes the same cell when its
hidden bias is (0, 0, b_n), and by hand-checkable limits (tests/test_oracle_recurrent.py).  The LSTM cell
(eqx.nn.LSTMCell, gate order input | forget | cell | output) is pinned by torch.nn.LSTMCell.  GELU is the tanh form,
jax.nn.gelu's default."""
import numpy as np


def sigmoid(x):
    return 1.0 / (1.0 + np.exp(-x))


def gru_cell(x, h, weight_ih, weight_hh, bias=None, bias_n=None):
    """x (N, I), h (N, H) -> h' (N, H)."""
    x, h = np.asarray(x, dtype=np.float64), np.asarray(h, dtype=np.float64)
    H = h.shape[-1]
    gi = x @ np.asarray(weight_ih, dtype=np.float64).T + (0.0 if bias is None else np.asarray(bias, dtype=np.float64))
    gh = h @ np.asarray(weight_hh, dtype=np.float64).T
    bn = 0.0 if bias_n is None else np.asarray(bias_n, dtype=np.float64)
    r = sigmoid(gi[:, :H] + gh[:, :H])
    z = sigmoid(gi[:, H:2 * H] + gh[:, H:2 * H])
    n = np.tanh(gi[:, 2 * H:] + r * (gh[:, 2 * H:] + bn))
    return n + z * (h - n)


def lstm_cell(x, h, c, weight_ih, weight_hh, bias=None):
    """eqx.nn.LSTMCell's equations (gate rows input | forget | cell | output): returns (h', c')."""
    x, h, c = (np.asarray(v, dtype=np.float64) for v in (x, h, c))
    H = h.shape[-1]
    g = x @ np.asarray(weight_ih, dtype=np.float64).T + h @ np.asarray(weight_hh, dtype=np.float64).T
    if bias is not None:
        g = g + np.asarray(bias, dtype=np.float64)
    i, f, gg, o = sigmoid(g[:, :H]), sigmoid(g[:, H:2 * H]), np.tanh(g[:, 2 * H:3 * H]), sigmoid(g[:, 3 * H:])
    cn = f * c + i * gg
    return o * np.tanh(cn), cn


def gelu(x):
    x = np.asarray(x, dtype=np.float64)
    return 0.5 * x * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (x + 0.044715 * x**3)))


def mlp(x, weights, biases, act):
    h = np.asarray(x, dtype=np.float64)
    for i, (w, b) in enumerate(zip(weights, biases)):
        h = h @ np.asarray(w, dtype=np.float64).T + np.asarray(b, dtype=np.float64)
        if i + 1 < len(weights):
            h = act(h)
    return h


def recurrent_network(obs, carry, fresh, input_proj, cells, out_weights, out_biases, act=gelu):
    """One control step (examples/walking.py:124-150): returns (output, new carry (depth, N, H)); envs marked fresh
    start from a zero carry."""
    carry = np.asarray(carry, dtype=np.float64)
    lstm = carry.ndim == 4  # (depth, 2, N, H): hidden then cell state (examples/kbot/train.py:910-913)
    keep = ~np.asarray(fresh, dtype=bool)
    carry = carry * (keep[None, None, :, None] if lstm else keep[None, :, None])
    x = np.asarray(obs, dtype=np.float64) @ np.asarray(input_proj[0], dtype=np.float64).T + input_proj[1]
    new = []
    for c, h in zip(cells, carry):
        if lstm:
            x, cn = lstm_cell(x, h[0], h[1], *c)
            new.append(np.stack([x, cn]))
        else:
            x = gru_cell(x, h, *c)
            new.append(x)
    return mlp(x, out_weights, out_biases, act), np.stack(new)


def elu(x):
    x = np.asarray(x, dtype=np.float64)
    return np.where(x > 0, x, np.expm1(np.minimum(x, 0.0)))


def recurrent_sequence(obs, carry0, fresh, input_proj, cells, out_weights, out_biases, act=elu):
    """The GRU network over a trajectory obs (T, N, in): `recurrent_network` step after step.  Returns (T, N, out)."""
    carry, outs = np.asarray(carry0, dtype=np.float64), []
    for t in range(len(obs)):
        y, carry = recurrent_network(obs[t], carry, fresh[t], input_proj, cells, out_weights, out_biases, act)
        outs.append(y)
    return np.stack(outs)


def torch_sequence(obs, carry0, fresh, wp, bp, cs, ow, ob, act="elu"):
    """`recurrent_sequence` on torch float64 tensors (parameters may require gradients): returns the (T, N, out) tensor."""
    import torch

    f = {"elu": torch.nn.functional.elu, "tanh": torch.tanh, "relu": torch.relu, "none": lambda t: t,
         "gelu": lambda t: torch.nn.functional.gelu(t, approximate="tanh")}[act]
    obs_t = torch.tensor(np.asarray(obs, dtype=np.float64))
    carry = torch.tensor(np.asarray(carry0, dtype=np.float64))
    lstm = carry.ndim == 4
    outs = []
    for t in range(obs_t.shape[0]):
        keep = torch.tensor(1.0 - np.asarray(fresh[t], dtype=np.float64))
        carry = carry * (keep[None, None, :, None] if lstm else keep[None, :, None])
        x = obs_t[t] @ wp.T + bp
        new = []
        for c, h in zip(cs, carry):
            if lstm:  # (weight_ih, weight_hh, bias), carry entry (2, N, H)
                wi, wh, b = c
                H = h.shape[-1]
                g = x @ wi.T + h[0] @ wh.T + b
                cn = torch.sigmoid(g[:, H:2 * H]) * h[1] + torch.sigmoid(g[:, :H]) * torch.tanh(g[:, 2 * H:3 * H])
                x = torch.sigmoid(g[:, 3 * H:]) * torch.tanh(cn)
                new.append(torch.stack([x, cn]))
            else:
                wi, wh, b, bn = c
                H = h.shape[-1]
                gi, gh = x @ wi.T + b, h @ wh.T
                r = torch.sigmoid(gi[:, :H] + gh[:, :H])
                z = torch.sigmoid(gi[:, H:2 * H] + gh[:, H:2 * H])
                n = torch.tanh(gi[:, 2 * H:] + r * (gh[:, 2 * H:] + bn))
                x = n + z * (h - n)
                new.append(x)
        carry = torch.stack(new)
        y = x
        for k, (w, b) in enumerate(zip(ow, ob)):
            y = y @ w.T + b
            if k + 1 < len(ow):
                y = f(y)
        outs.append(y)
    return torch.stack(outs)


def torch_parameters(input_proj, cells, out_weights, out_biases):
    import torch

    t64 = lambda a: torch.tensor(np.asarray(a, dtype=np.float64), requires_grad=True)  # noqa: E731
    return (t64(input_proj[0]), t64(input_proj[1]), [tuple(t64(p) for p in c) for c in cells],
            [t64(w) for w in out_weights], [t64(b) for b in out_biases])


def parameter_gradients(params):
    wp, bp, cs, ow, ob = params
    g = lambda p: p.grad.numpy()  # noqa: E731
    return dict(input_proj=(g(wp), g(bp)), cells=[tuple(g(p) for p in c) for c in cs], out=[(g(w), g(b)) for w, b in zip(ow, ob)])


def recurrent_sequence_gradients(obs, carry0, fresh, input_proj, cells, out_weights, out_biases, d_out, act="elu"):
    """Gradients of sum(d_out * recurrent_sequence(...)) with respect to every parameter: the backward pass through time
    that jax.grad performs through the scan over the trajectory (ksim/task/ppo.py:572-694).  The same equations as
    `recurrent_sequence`, written with torch float64 tensors so that the library's reverse-mode differentiation yields the
    gradients; tests pin the forward value to `recurrent_sequence` and single entries to central differences of it.
    GRU cells are (weight_ih, weight_hh, bias, bias_n) with carry (depth, N, H); LSTM cells (weight_ih, weight_hh, bias)
    with carry (depth, 2, N, H).
    Returns (outputs, dict(input_proj=(dW, db), cells=[one gradient per cell parameter], out=[(dW, db)]))."""
    import torch

    params = torch_parameters(input_proj, cells, out_weights, out_biases)
    out = torch_sequence(obs, carry0, fresh, *params, act=act)
    (out * torch.tensor(np.asarray(d_out, dtype=np.float64))).sum().backward()
    return out.detach().numpy(), parameter_gradients(params)
