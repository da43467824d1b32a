"""Recurrent policy / critic networks for the rollout, and the backward pass through time of the GRU stack.

The shipped examples build their actor and critic as an input projection, a stack of GRU cells and an output MLP
(examples/walking.py:40-208); the carry `(depth, N, hidden)` travels with the env state and is zeroed for envs that
start an episode (ksim/task/rl.py:1072-1080).  Weights use the (out, in) layout and gate order (reset | update |
candidate) of the reference's cells.
"""
from __future__ import annotations

import ctypes
from typing import Sequence

import numpy as np
import torch

from . import _lib
from . import _lib_terms as T
from .mlp import MLP


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a.detach().cpu().numpy() if isinstance(a, torch.Tensor) else a, dtype=np.float32)


class GRUCell:
    """h' = GRU(x, h) for N envs at once (`ks_gru_forward`)."""

    def __init__(self, weight_ih, weight_hh, bias=None, bias_n=None, dtype: str = "bf16"):
        lib = _lib.load()
        if dtype not in ("bf16", "f32"):
            raise _lib.KsError("dtype must be 'bf16' or 'f32'")
        wi, wh = _f32(weight_ih), _f32(weight_hh)
        H = wh.shape[1] if wh.ndim == 2 else -1
        if wi.ndim != 2 or wh.shape != (3 * H, H) or wi.shape[0] != 3 * H:
            raise _lib.KsError("weight_ih must be (3H, input) and weight_hh (3H, H)")
        b = None if bias is None else _f32(bias)
        bn = None if bias_n is None else _f32(bias_n)
        if (b is not None and b.shape != (3 * H,)) or (bn is not None and bn.shape != (H,)):
            raise _lib.KsError("bias must be (3H) and bias_n (H)")
        torch.zeros(1, device="cuda")
        d = T.KsGruDesc()
        d.input_size, d.hidden_size = wi.shape[1], H
        d.dtype = T.MLP_BF16 if dtype == "bf16" else T.MLP_F32
        d.weight_ih, d.weight_hh = wi.ctypes.data, wh.ctypes.data
        d.bias = None if b is None else b.ctypes.data
        d.bias_n = None if bn is None else bn.ctypes.data
        self.input_size, self.hidden_size, self.dtype = int(wi.shape[1]), int(H), dtype
        self._lib = lib
        self._handle = ctypes.c_void_p()
        _lib.check(lib.ks_gru_create(ctypes.byref(d), ctypes.byref(self._handle)))
        self._ws: torch.Tensor | None = None

    def workspace(self, M: int, device) -> torch.Tensor:
        need = int(self._lib.ks_gru_workspace_bytes(self._handle, M))
        if self._ws is None or self._ws.numel() < need or self._ws.device != torch.device(device):
            self._ws = torch.empty(need, dtype=torch.uint8, device=device)
        return self._ws

    def __call__(self, x: torch.Tensor, h: torch.Tensor, fresh: torch.Tensor | None = None,
                 out: torch.Tensor | None = None) -> torch.Tensor:
        _lib.require_cuda(x, dtype=torch.float32)
        _lib.require_cuda(h, dtype=torch.float32)
        M = x.shape[0]
        if tuple(x.shape) != (M, self.input_size) or tuple(h.shape) != (M, self.hidden_size):
            raise _lib.KsError(f"expected x (M, {self.input_size}) and h (M, {self.hidden_size})")
        if fresh is not None:
            _lib.require_cuda(fresh, dtype=torch.uint8)
            if tuple(fresh.shape) != (M,):
                raise _lib.KsError("fresh must be (M,) uint8")
        if out is None:
            out = torch.empty_like(h)
        else:
            _lib.require_cuda(out, dtype=torch.float32)
            if tuple(out.shape) != tuple(h.shape):
                raise _lib.KsError("output has the wrong shape")
        ws = self.workspace(M, x.device)
        _lib.check(self._lib.ks_gru_forward(self._handle, _lib.current_stream(), M, _lib.ptr(x), _lib.ptr(h),
                                            _lib.ptr(fresh), _lib.ptr(out), _lib.ptr(ws)))
        return out

    # ------------------------------------------------------------------ training (ksim/task/ppo.py:572-694)
    def train_init(self) -> None:
        """fp32 master weights, gradients and Adam moments of both projections; afterwards `proj_i` / `proj_h` expose them."""
        _lib.check(self._lib.ks_gru_train_init(self._handle))
        pi, ph = ctypes.c_void_p(), ctypes.c_void_p()
        _lib.check(self._lib.ks_gru_projections(self._handle, ctypes.byref(pi), ctypes.byref(ph)))
        H = self.hidden_size
        self.proj_i = MLP._borrow(self._lib, pi, (self.input_size, 3 * H), self.dtype)
        self.proj_h = MLP._borrow(self._lib, ph, (H, 3 * H), self.dtype)
        self._bws: torch.Tensor | None = None

    def train_forward(self, x, h, fresh, out, saved) -> torch.Tensor:
        """`__call__` that also fills `saved` (M, 5H) = r | z | n | hn | h for `backward_step`."""
        _lib.require_cuda(x, h, out, saved, dtype=torch.float32)
        _lib.require_cuda(fresh, dtype=torch.uint8)
        M, H = x.shape[0], self.hidden_size
        if tuple(x.shape) != (M, self.input_size) or tuple(h.shape) != (M, H) or tuple(out.shape) != (M, H) or tuple(saved.shape) != (M, 5 * H):
            raise _lib.KsError("expected x (M, input), h and out (M, H), saved (M, 5H)")
        _lib.check(self._lib.ks_gru_train_forward(self._handle, _lib.current_stream(), M, _lib.ptr(x), _lib.ptr(h), _lib.ptr(fresh),
                                                  _lib.ptr(out), _lib.ptr(saved), _lib.ptr(self.workspace(M, x.device))))
        return out

    def backward_step(self, dh_out, saved, fresh, d_gi, d_gh, dh_in) -> None:
        """One step of the backward pass through time: dh_out (M, H) -> d_gi, d_gh (M, 3H) and dh_in (M, H)."""
        _lib.require_cuda(dh_out, saved, d_gi, d_gh, dh_in, dtype=torch.float32)
        _lib.require_cuda(fresh, dtype=torch.uint8)
        M, H = dh_out.shape[0], self.hidden_size
        if (tuple(dh_out.shape) != (M, H) or tuple(saved.shape) != (M, 5 * H) or tuple(d_gi.shape) != (M, 3 * H)
                or tuple(d_gh.shape) != (M, 3 * H) or tuple(dh_in.shape) != (M, H)):
            raise _lib.KsError("expected dh_out, dh_in (M, H), saved (M, 5H), d_gi, d_gh (M, 3H)")
        need = int(self._lib.ks_gru_backward_workspace_bytes(self._handle, M))
        if self._bws is None or self._bws.numel() < need or self._bws.device != dh_out.device:
            self._bws = torch.empty(need, dtype=torch.uint8, device=dh_out.device)
        _lib.check(self._lib.ks_gru_backward_step(self._handle, _lib.current_stream(), M, _lib.ptr(dh_out), _lib.ptr(saved),
                                                  _lib.ptr(fresh), _lib.ptr(d_gi), _lib.ptr(d_gh), _lib.ptr(dh_in), _lib.ptr(self._bws)))

    def grad_sqnorm(self, acc: torch.Tensor) -> None:
        _lib.check(self._lib.ks_gru_grad_sqnorm(self._handle, _lib.current_stream(), _lib.ptr(acc)))

    def adam_step(self, params, sqnorm) -> None:
        _lib.check(self._lib.ks_gru_adam_step(self._handle, _lib.current_stream(), ctypes.byref(params), _lib.ptr(sqnorm)))

    def parameters(self, gradients: bool = False) -> dict:
        """Copies of weight_ih, weight_hh, bias (3H) and bias_n (H), or of their gradients."""
        (wi, bi), = self.proj_i.parameters(gradients)
        (wh, bh), = self.proj_h.parameters(gradients)
        return dict(weight_ih=wi, weight_hh=wh, bias=bi, bias_n=bh[2 * self.hidden_size:].clone())

    def __del__(self):
        h = getattr(self, "_handle", None)
        if h:
            self._lib.ks_gru_destroy(h)
            self._handle = None


class LSTMCell:
    """(h', c') = LSTM(x, (h, c)) for N envs at once (`ks_lstm_forward`); gate rows ordered input | forget | cell | output."""

    def __init__(self, weight_ih, weight_hh, bias=None, dtype: str = "bf16"):
        lib = _lib.load()
        if dtype not in ("bf16", "f32"):
            raise _lib.KsError("dtype must be 'bf16' or 'f32'")
        wi, wh = _f32(weight_ih), _f32(weight_hh)
        H = wh.shape[1] if wh.ndim == 2 else -1
        if wi.ndim != 2 or wh.shape != (4 * H, H) or wi.shape[0] != 4 * H:
            raise _lib.KsError("weight_ih must be (4H, input) and weight_hh (4H, H)")
        b = None if bias is None else _f32(bias)
        if b is not None and b.shape != (4 * H,):
            raise _lib.KsError("bias must be (4H)")
        torch.zeros(1, device="cuda")
        d = T.KsLstmDesc()
        d.input_size, d.hidden_size = wi.shape[1], H
        d.dtype = T.MLP_BF16 if dtype == "bf16" else T.MLP_F32
        d.weight_ih, d.weight_hh = wi.ctypes.data, wh.ctypes.data
        d.bias = None if b is None else b.ctypes.data
        self.input_size, self.hidden_size, self.dtype = int(wi.shape[1]), int(H), dtype
        self._lib = lib
        self._handle = ctypes.c_void_p()
        _lib.check(lib.ks_lstm_create(ctypes.byref(d), ctypes.byref(self._handle)))
        self._ws: torch.Tensor | None = None

    def workspace(self, M: int, device) -> torch.Tensor:
        need = int(self._lib.ks_lstm_workspace_bytes(self._handle, M))
        if self._ws is None or self._ws.numel() < need or self._ws.device != torch.device(device):
            self._ws = torch.empty(need, dtype=torch.uint8, device=device)
        return self._ws

    def __call__(self, x: torch.Tensor, h: torch.Tensor, c: torch.Tensor, fresh: torch.Tensor | None = None,
                 out: tuple | None = None) -> tuple[torch.Tensor, torch.Tensor]:
        for t in (x, h, c):
            _lib.require_cuda(t, dtype=torch.float32)
        M = x.shape[0]
        if tuple(x.shape) != (M, self.input_size) or tuple(h.shape) != (M, self.hidden_size) or tuple(c.shape) != tuple(h.shape):
            raise _lib.KsError(f"expected x (M, {self.input_size}) and h, c (M, {self.hidden_size})")
        if fresh is not None:
            _lib.require_cuda(fresh, dtype=torch.uint8)
            if tuple(fresh.shape) != (M,):
                raise _lib.KsError("fresh must be (M,) uint8")
        ho, co = (torch.empty_like(h), torch.empty_like(c)) if out is None else out
        for t in (ho, co):
            _lib.require_cuda(t, dtype=torch.float32)
            if tuple(t.shape) != tuple(h.shape):
                raise _lib.KsError("output has the wrong shape")
        ws = self.workspace(M, x.device)
        _lib.check(self._lib.ks_lstm_forward(self._handle, _lib.current_stream(), M, _lib.ptr(x), _lib.ptr(h), _lib.ptr(c),
                                             _lib.ptr(fresh), _lib.ptr(ho), _lib.ptr(co), _lib.ptr(ws)))
        return ho, co

    # ------------------------------------------------------------------ training (ksim/task/ppo.py:572-694)
    def train_init(self) -> None:
        _lib.check(self._lib.ks_lstm_train_init(self._handle))
        pi, ph = ctypes.c_void_p(), ctypes.c_void_p()
        _lib.check(self._lib.ks_lstm_projections(self._handle, ctypes.byref(pi), ctypes.byref(ph)))
        H = self.hidden_size
        self.proj_i = MLP._borrow(self._lib, pi, (self.input_size, 4 * H), self.dtype)
        self.proj_h = MLP._borrow(self._lib, ph, (H, 4 * H), self.dtype)
        self._bws: torch.Tensor | None = None

    def train_forward(self, x, h, c, fresh, h_out, c_out, saved) -> None:
        """`__call__` that also fills `saved` (M, 7H) = i | f | g | o | tanh(c') | c | h for `backward_step`."""
        _lib.require_cuda(x, h, c, h_out, c_out, saved, dtype=torch.float32)
        _lib.require_cuda(fresh, dtype=torch.uint8)
        M, H = x.shape[0], self.hidden_size
        if tuple(x.shape) != (M, self.input_size) or any(tuple(t.shape) != (M, H) for t in (h, c, h_out, c_out)) or tuple(saved.shape) != (M, 7 * H):
            raise _lib.KsError("expected x (M, input), h, c and outputs (M, H), saved (M, 7H)")
        _lib.check(self._lib.ks_lstm_train_forward(self._handle, _lib.current_stream(), M, _lib.ptr(x), _lib.ptr(h), _lib.ptr(c),
                                                   _lib.ptr(fresh), _lib.ptr(h_out), _lib.ptr(c_out), _lib.ptr(saved),
                                                   _lib.ptr(self.workspace(M, x.device))))

    @property
    def sequence_supported(self) -> bool:
        """Whether this cell has the one-launch-per-trajectory kernels (`ks_lstm_sequence_forward / _backward`)."""
        return bool(self._lib.ks_lstm_sequence_supported(self._handle))

    def sequence_forward(self, x, h0, c0, fresh, hs, cs, saved) -> None:
        """The layer over a whole trajectory: x (T, M, input) -> hs, cs (T, M, H) and `saved` (T, M, 7H), from the carry
        (h0, c0); the input projection is one product over all T M rows, the recurrence one launch."""
        _lib.require_cuda(x, h0, c0, hs, cs, saved, dtype=torch.float32)
        _lib.require_cuda(fresh, dtype=torch.uint8)
        Tn, M, H = x.shape[0], x.shape[1], self.hidden_size
        if (tuple(x.shape) != (Tn, M, self.input_size) or any(tuple(t.shape) != (M, H) for t in (h0, c0))
                or any(tuple(t.shape) != (Tn, M, H) for t in (hs, cs)) or tuple(saved.shape) != (Tn, M, 7 * H)
                or tuple(fresh.shape) != (Tn, M)):
            raise _lib.KsError("expected x (T, M, input), h0, c0 (M, H), hs, cs (T, M, H), saved (T, M, 7H), fresh (T, M)")
        gi = self.proj_i(x.reshape(Tn * M, self.input_size))
        _lib.check(self._lib.ks_lstm_sequence_forward(self._handle, _lib.current_stream(), Tn, M, _lib.ptr(gi), _lib.ptr(h0),
                                                      _lib.ptr(c0), _lib.ptr(fresh), _lib.ptr(hs), _lib.ptr(cs), _lib.ptr(saved)))

    def sequence_backward(self, dH, saved, fresh, d_g) -> None:
        """The reverse sweep over the trajectory: dH (T, M, H), the gradient reaching every h_t from above, -> d_g (T, M, 4H)."""
        _lib.require_cuda(dH, saved, d_g, dtype=torch.float32)
        _lib.require_cuda(fresh, dtype=torch.uint8)
        Tn, M, H = dH.shape[0], dH.shape[1], self.hidden_size
        if (tuple(dH.shape) != (Tn, M, H) or tuple(saved.shape) != (Tn, M, 7 * H) or tuple(d_g.shape) != (Tn, M, 4 * H)
                or tuple(fresh.shape) != (Tn, M)):
            raise _lib.KsError("expected dH (T, M, H), saved (T, M, 7H), d_g (T, M, 4H), fresh (T, M)")
        _lib.check(self._lib.ks_lstm_sequence_backward(self._handle, _lib.current_stream(), Tn, M, _lib.ptr(dH), _lib.ptr(saved),
                                                       _lib.ptr(fresh), _lib.ptr(d_g), None, None))

    def backward_step(self, dh_out, dc_out, saved, fresh, d_g, dh_in, dc_in) -> None:
        """One step of the backward pass through time: (dh_out, dc_out) -> d_g (M, 4H), dh_in, dc_in (M, H)."""
        _lib.require_cuda(dh_out, dc_out, saved, d_g, dh_in, dc_in, dtype=torch.float32)
        _lib.require_cuda(fresh, dtype=torch.uint8)
        M, H = dh_out.shape[0], self.hidden_size
        if (any(tuple(t.shape) != (M, H) for t in (dh_out, dc_out, dh_in, dc_in)) or tuple(saved.shape) != (M, 7 * H)
                or tuple(d_g.shape) != (M, 4 * H)):
            raise _lib.KsError("expected gradients of the states (M, H), saved (M, 7H), d_g (M, 4H)")
        need = int(self._lib.ks_lstm_backward_workspace_bytes(self._handle, M))
        if self._bws is None or self._bws.numel() < need or self._bws.device != dh_out.device:
            self._bws = torch.empty(need, dtype=torch.uint8, device=dh_out.device)
        _lib.check(self._lib.ks_lstm_backward_step(self._handle, _lib.current_stream(), M, _lib.ptr(dh_out), _lib.ptr(dc_out),
                                                   _lib.ptr(saved), _lib.ptr(fresh), _lib.ptr(d_g), _lib.ptr(dh_in),
                                                   _lib.ptr(dc_in), _lib.ptr(self._bws)))

    def grad_sqnorm(self, acc: torch.Tensor) -> None:
        _lib.check(self._lib.ks_lstm_grad_sqnorm(self._handle, _lib.current_stream(), _lib.ptr(acc)))

    def adam_step(self, params, sqnorm) -> None:
        _lib.check(self._lib.ks_lstm_adam_step(self._handle, _lib.current_stream(), ctypes.byref(params), _lib.ptr(sqnorm)))

    def parameters(self, gradients: bool = False) -> dict:
        """Copies of weight_ih, weight_hh and bias (4H), or of their gradients."""
        (wi, bi), = self.proj_i.parameters(gradients)
        (wh, _), = self.proj_h.parameters(gradients)
        return dict(weight_ih=wi, weight_hh=wh, bias=bi)

    def __del__(self):
        h = getattr(self, "_handle", None)
        if h:
            self._lib.ks_lstm_destroy(h)
            self._handle = None


class RecurrentNetwork:
    """input projection -> GRU or LSTM stack -> output MLP (examples/walking.py:124-150, 198-208;
    examples/kbot/train.py:903-915).  The carry is (depth, N, hidden) for GRU layers and (depth, 2, N, hidden), hidden
    state then cell state, for LSTM layers, like the arrays the reference stacks."""

    def __init__(self, input_proj: tuple, cells: Sequence[GRUCell], output_proj: MLP, dtype: str = "bf16"):
        w, b = input_proj
        self.input_proj = MLP([w], [b], activation="none", dtype=dtype)
        self.cells, self.output_proj = tuple(cells), output_proj
        H = self.input_proj.out_dim
        if any(c.input_size != H or c.hidden_size != H for c in self.cells) or output_proj.in_dim != H:
            raise _lib.KsError("the projection, the cells and the output network must share one hidden size")
        if len({type(c) for c in self.cells}) > 1:
            raise _lib.KsError("the recurrent layers must all be of one kind")
        self.lstm = bool(self.cells) and isinstance(self.cells[0], LSTMCell)
        self.hidden_size, self.depth = H, len(self.cells)
        self.in_dim, self.out_dim = self.input_proj.in_dim, output_proj.out_dim
        self._x: torch.Tensor | None = None

    def initial_carry(self, num_envs: int, device="cuda") -> torch.Tensor:
        shape = (self.depth, 2, num_envs, self.hidden_size) if self.lstm else (self.depth, num_envs, self.hidden_size)
        return torch.zeros(*shape, dtype=torch.float32, device=device)

    def __call__(self, obs: torch.Tensor, carry: torch.Tensor, fresh: torch.Tensor | None = None,
                 out: torch.Tensor | None = None) -> torch.Tensor:
        """One control step for every env: `carry` is advanced in place."""
        N = obs.shape[0]
        want = (self.depth, 2, N, self.hidden_size) if self.lstm else (self.depth, N, self.hidden_size)
        if tuple(carry.shape) != want:
            raise _lib.KsError(f"carry must be {want}")
        if self._x is None or self._x.shape[0] != N or self._x.device != obs.device:
            self._x = torch.empty(N, self.hidden_size, dtype=torch.float32, device=obs.device)
        x = self.input_proj(obs, out=self._x)
        for i, cell in enumerate(self.cells):  # the layer's new hidden state is also the next layer's input
            if self.lstm:
                x, _ = cell(x, carry[i, 0], carry[i, 1], fresh, out=(carry[i, 0], carry[i, 1]))
            else:
                x = cell(x, carry[i], fresh, out=carry[i])
        return self.output_proj(x, out=out)

    # ------------------------------------------------------------------ training: backward pass through time
    def train_init(self) -> None:
        self.input_proj.train_init()
        for c in self.cells:
            c.train_init()
        self.output_proj.train_init()

    def train_forward(self, obs: torch.Tensor, carry0: torch.Tensor, fresh: torch.Tensor) -> torch.Tensor:
        """The network over a trajectory, obs (T, M, in), starting from carry0 (the rollout's carry layout); envs flagged
        in fresh (T, M) uint8 start an episode at that step (their carry is zero there).  Returns (T, M, out) and keeps
        what `backward` needs.  This is the scan over time inside the loss of PPOTask._single_step
        (ksim/task/ppo.py:572-694)."""
        T_, M = obs.shape[0], obs.shape[1]
        H, dev = self.hidden_size, obs.device
        _lib.require_cuda(obs, carry0, dtype=torch.float32)
        _lib.require_cuda(fresh, dtype=torch.uint8)
        want = (self.depth, 2, M, H) if self.lstm else (self.depth, M, H)
        if tuple(obs.shape) != (T_, M, self.in_dim) or tuple(carry0.shape) != want or tuple(fresh.shape) != (T_, M):
            raise _lib.KsError(f"expected obs (T, M, in), carry0 {want}, fresh (T, M)")
        obs = obs.contiguous()
        x = self.input_proj(obs.view(T_ * M, self.in_dim)).view(T_, M, H)
        xs, saved = [], []
        for i, cell in enumerate(self.cells):
            hs = torch.empty(T_, M, H, dtype=torch.float32, device=dev)
            sv = torch.empty(T_, M, (7 if self.lstm else 5) * H, dtype=torch.float32, device=dev)
            if self.lstm and getattr(cell, "proj_i", None) is not None and cell.sequence_supported:
                cs = torch.empty(T_, M, H, dtype=torch.float32, device=dev)
                cell.sequence_forward(x, carry0[i, 0], carry0[i, 1], fresh, hs, cs, sv)
            elif self.lstm:
                cs = torch.empty(T_, M, H, dtype=torch.float32, device=dev)
                for t in range(T_):
                    h0, c0 = (carry0[i, 0], carry0[i, 1]) if t == 0 else (hs[t - 1], cs[t - 1])
                    cell.train_forward(x[t], h0, c0, fresh[t], hs[t], cs[t], sv[t])
            else:
                for t in range(T_):
                    cell.train_forward(x[t], carry0[i] if t == 0 else hs[t - 1], fresh[t], hs[t], sv[t])
            xs.append(x)
            saved.append(sv)
            x = hs
        out = self.output_proj.train_forward(x.view(T_ * M, H)).view(T_, M, self.out_dim)
        self._tape = dict(obs=obs, xs=xs, saved=saved, top=x, fresh=fresh.contiguous(), T=T_, M=M)
        return out

    def backward(self, d_out: torch.Tensor) -> None:
        """Gradients of sum(d_out * output) with respect to every parameter, into the handles (the jax.grad through the
        scan).  Per layer, top to bottom: a sweep over the steps, last to first, that carries the gradient of the
        recurrent state, then one pass over all (step, env) rows for the weight gradients and the gradient of the layer's
        inputs."""
        tp = self._tape
        T_, M, H = tp["T"], tp["M"], self.hidden_size
        G = 4 if self.lstm else 3
        dev = d_out.device
        _lib.require_cuda(d_out, dtype=torch.float32)
        if tuple(d_out.shape) != (T_, M, self.out_dim):
            raise _lib.KsError("d_out must have the shape of the output")
        dH = torch.empty(T_, M, H, dtype=torch.float32, device=dev)
        self.output_proj.backward_dx(tp["top"].view(T_ * M, H), d_out.contiguous().view(T_ * M, self.out_dim), dH.view(T_ * M, H))
        for i in range(self.depth - 1, -1, -1):
            cell, sv = self.cells[i], tp["saved"][i]
            d_gi = torch.empty(T_, M, G * H, dtype=torch.float32, device=dev)
            d_gh = d_gi if self.lstm else torch.empty(T_, M, G * H, dtype=torch.float32, device=dev)
            carry = torch.zeros(2, M, H, dtype=torch.float32, device=dev)   # gradient of the hidden state, ping-pong
            ccarry = torch.zeros(2, M, H, dtype=torch.float32, device=dev)  # and of the cell state (LSTM)
            fused = self.lstm and cell.sequence_supported
            if fused:
                cell.sequence_backward(dH, sv, tp["fresh"], d_gi)
            for t in range(T_ - 1, -1, -1) if not fused else ():
                dH[t] += carry[t & 1]
                if self.lstm:
                    cell.backward_step(dH[t], ccarry[t & 1], sv[t], tp["fresh"][t], d_gi[t], carry[(t + 1) & 1], ccarry[(t + 1) & 1])
                else:
                    cell.backward_step(dH[t], sv[t], tp["fresh"][t], d_gi[t], d_gh[t], carry[(t + 1) & 1])
            h_used = sv[:, :, (6 if self.lstm else 4) * H:].contiguous().view(T_ * M, H)
            cell.proj_h.backward(h_used, d_gh.view(T_ * M, G * H))
            dX = torch.empty(T_, M, H, dtype=torch.float32, device=dev)
            cell.proj_i.backward_dx(tp["xs"][i].reshape(T_ * M, H), d_gi.view(T_ * M, G * H), dX.view(T_ * M, H))
            dH = dX
        self.input_proj.backward(tp["obs"].view(T_ * M, self.in_dim), dH.view(T_ * M, H))

    def grad_sqnorm(self, acc: torch.Tensor) -> None:
        for net in (self.input_proj, *self.cells, self.output_proj):
            net.grad_sqnorm(acc)

    def adam_step(self, params, sqnorm) -> None:
        for net in (self.input_proj, *self.cells, self.output_proj):
            net.adam_step(params, sqnorm)
