"""Recurrent policy / critic networks for the rollout (forward only).

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
