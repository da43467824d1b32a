"""MLP forward on the matrix cores (policy / critic / discriminator networks of the rollout path).

The reference leaves the network to the task (``sample_action``, ksim/task/rl.py:892-926); the configs here
use plain MLP stacks.  Weights are given as (out, in) fp32 arrays, like the reference's linear layers.
"""
from __future__ import annotations

import ctypes
from typing import Sequence

import numpy as np
import torch

from . import _lib
from . import _lib_terms as T

_ACT = {None: T.ACT_NONE, "none": T.ACT_NONE, "elu": T.ACT_ELU, "relu": T.ACT_RELU, "tanh": T.ACT_TANH,
        "gelu": T.ACT_GELU}


class MLP:
    def __init__(self, weights: Sequence, biases: Sequence, activation: str = "elu", dtype: str = "bf16"):
        lib = _lib.load()
        if len(weights) != len(biases) or not weights:
            raise _lib.KsError("one bias per weight matrix is required")
        if dtype not in ("bf16", "f32"):
            raise _lib.KsError("dtype must be 'bf16' or 'f32'")
        torch.zeros(1, device="cuda")  # make sure a HIP context exists before the library allocates
        ws = [np.ascontiguousarray(w.detach().cpu().numpy() if isinstance(w, torch.Tensor) else w, dtype=np.float32)
              for w in weights]
        bs = [np.ascontiguousarray(b.detach().cpu().numpy() if isinstance(b, torch.Tensor) else b, dtype=np.float32)
              for b in biases]
        dims = [ws[0].shape[1]]
        for w, b in zip(ws, bs):
            if w.ndim != 2 or w.shape[1] != dims[-1] or b.shape != (w.shape[0],):
                raise _lib.KsError("weight / bias shapes do not chain")
            dims.append(w.shape[0])
        d = T.KsMlpDesc()
        d.n_layers, d.activation = len(ws), _ACT[activation]
        d.dtype = T.MLP_BF16 if dtype == "bf16" else T.MLP_F32
        for i, v in enumerate(dims):
            d.dims[i] = v
        for i, (w, b) in enumerate(zip(ws, bs)):
            d.weights[i] = w.ctypes.data
            d.biases[i] = b.ctypes.data
        self.dims, self.dtype, self.activation = dims, dtype, activation
        self._lib = lib
        self._handle = ctypes.c_void_p()
        _lib.check(lib.ks_mlp_create(ctypes.byref(d), ctypes.byref(self._handle)))
        self._ws: dict | None = None

    @property
    def in_dim(self) -> int:
        return self.dims[0]

    @property
    def out_dim(self) -> int:
        return self.dims[-1]

    def flops_per_row(self) -> int:
        return 2 * sum(a * b for a, b in zip(self.dims[:-1], self.dims[1:]))

    def workspace(self, M: int, device) -> torch.Tensor:
        """Scratch of the per-layer path, one buffer per stream: calls on different streams may overlap on the GPU."""
        need = int(self._lib.ks_mlp_workspace_bytes(self._handle, M))
        key = torch.cuda.current_stream().cuda_stream if need else 0
        if self._ws is None:
            self._ws = {}
        ws = self._ws.get(key)
        if ws is None or ws.numel() < need or ws.device != torch.device(device):
            ws = torch.empty(need, dtype=torch.uint8, device=device)
            self._ws[key] = ws
        return ws

    def __call__(self, x: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
        _lib.require_cuda(x, dtype=torch.float32)
        if x.dim() != 2 or x.shape[1] != self.in_dim:
            raise _lib.KsError(f"expected input (M, {self.in_dim}), got {tuple(x.shape)}")
        M = x.shape[0]
        if out is None:
            out = torch.empty((M, self.out_dim), dtype=torch.float32, device=x.device)
        else:
            _lib.require_cuda(out, dtype=torch.float32)
            if tuple(out.shape) != (M, self.out_dim):
                raise _lib.KsError("output has the wrong shape")
        ws = self.workspace(M, x.device)
        _lib.check(self._lib.ks_mlp_forward(self._handle, _lib.current_stream(), M, _lib.ptr(x), _lib.ptr(out),
                                            _lib.ptr(ws)))
        return out

    def forward_pair(self, x: torch.Tensor, out: torch.Tensor, other: "MLP", x_other: torch.Tensor,
                     out_other: torch.Tensor) -> None:
        """This network on ``x`` and ``other`` on ``x_other`` (same row count), in one launch when the library can."""
        M = x.shape[0]
        for net, a, o in ((self, x, out), (other, x_other, out_other)):
            _lib.require_cuda(a, dtype=torch.float32)
            _lib.require_cuda(o, dtype=torch.float32)
            if tuple(a.shape) != (M, net.in_dim) or tuple(o.shape) != (M, net.out_dim):
                raise _lib.KsError(f"expected input (M, {net.in_dim}) and output (M, {net.out_dim})")
        _lib.check(self._lib.ks_mlp_forward_pair(self._handle, other._handle, _lib.current_stream(), M, _lib.ptr(x),
                                                 _lib.ptr(out), _lib.ptr(x_other), _lib.ptr(out_other),
                                                 _lib.ptr(self.workspace(M, x.device)),
                                                 _lib.ptr(other.workspace(M, x.device))))

    # ------------------------------------------------------------------ training (ksim/task/ppo.py:495-565)
    def train_init(self) -> None:
        """fp32 master weights, gradients and Adam moments beside the working copies."""
        _lib.check(self._lib.ks_mlp_train_init(self._handle))
        self._training = True

    def _train_ws(self, M: int, device) -> torch.Tensor:
        need = int(self._lib.ks_mlp_train_workspace_bytes(self._handle, M))
        ws = getattr(self, "_tws", None)
        if ws is None or ws.numel() < need or ws.device != torch.device(device):
            ws = torch.empty(need, dtype=torch.uint8, device=device)
            self._tws = ws
        return ws

    def train_forward(self, x: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
        """Forward pass that keeps the hidden activations for `backward` (same rows, called next)."""
        _lib.require_cuda(x, dtype=torch.float32)
        if x.dim() != 2 or x.shape[1] != self.in_dim:
            raise _lib.KsError(f"expected input (M, {self.in_dim}), got {tuple(x.shape)}")
        M = x.shape[0]
        if out is None:
            out = torch.empty((M, self.out_dim), dtype=torch.float32, device=x.device)
        _lib.check(self._lib.ks_mlp_train_forward(self._handle, _lib.current_stream(), M, _lib.ptr(x), _lib.ptr(out),
                                                  _lib.ptr(self._train_ws(M, x.device))))
        return out

    def backward(self, x: torch.Tensor, dy: torch.Tensor) -> None:
        """Gradients of sum(dy * net(x)) into the handle; `x` is the input of the preceding `train_forward`."""
        _lib.require_cuda(x, dy, dtype=torch.float32)
        if tuple(dy.shape) != (x.shape[0], self.out_dim):
            raise _lib.KsError("dy must have the shape of the network output")
        _lib.check(self._lib.ks_mlp_train_backward(self._handle, _lib.current_stream(), x.shape[0], _lib.ptr(x),
                                                   _lib.ptr(dy), _lib.ptr(self._train_ws(x.shape[0], x.device))))

    def backward_dx(self, x: torch.Tensor | None, dy: torch.Tensor, dx: torch.Tensor, *, weight_gradients: bool = True,
                    accumulate: bool = False, zero_rows: torch.Tensor | None = None) -> torch.Tensor:
        """`backward` that also writes (or adds) the gradient with respect to the network input into `dx`; without
        `weight_gradients` only that.  Rows flagged in `zero_rows` (uint8) get a zero input gradient."""
        _lib.require_cuda(x, dy, dx, dtype=torch.float32)
        M = dy.shape[0]
        if tuple(dy.shape) != (M, self.out_dim) or tuple(dx.shape) != (M, self.in_dim) or (x is not None and tuple(x.shape) != (M, self.in_dim)):
            raise _lib.KsError("x and dx must be (M, in), dy (M, out)")
        if x is None and weight_gradients:
            raise _lib.KsError("the weight gradients need the input")
        if zero_rows is not None:
            _lib.require_cuda(zero_rows, dtype=torch.uint8)
            if tuple(zero_rows.shape) != (M,):
                raise _lib.KsError("zero_rows must be (M,) uint8")
        _lib.check(self._lib.ks_mlp_train_backward_dx(self._handle, _lib.current_stream(), M, _lib.ptr(x), _lib.ptr(dy),
                                                      _lib.ptr(dx), int(weight_gradients), int(accumulate),
                                                      _lib.ptr(zero_rows), _lib.ptr(self._train_ws(M, dy.device))))
        return dx

    def disc_loss_grad(self, real: torch.Tensor, sim: torch.Tensor, grad_penalty_coef: float) -> torch.Tensor:
        """Gradient of the AMP discriminator loss (ksim/task/amp.py:360-438) into the handle: real (B, T, in) reference
        motions, sim (B2, T2, in) simulated ones; returns the (real, simulated, penalty) terms of the loss, on the device."""
        _lib.require_cuda(real, sim, dtype=torch.float32)
        if real.dim() != 3 or sim.dim() != 3 or real.shape[2] != self.in_dim or sim.shape[2] != self.in_dim:
            raise _lib.KsError(f"motions must be (B, T, {self.in_dim}), got {tuple(real.shape)} and {tuple(sim.shape)}")
        n_real, n_sim = real.shape[0] * real.shape[1], sim.shape[0] * sim.shape[1]
        need = int(self._lib.ks_mlp_disc_workspace_bytes(self._handle, n_real, n_sim))
        ws = getattr(self, "_dws", None)
        if ws is None or ws.numel() < need or ws.device != real.device:
            ws = torch.empty(need, dtype=torch.uint8, device=real.device)
            self._dws = ws
        losses = torch.empty(3, dtype=torch.float32, device=real.device)
        _lib.check(self._lib.ks_mlp_disc_loss_grad(self._handle, _lib.current_stream(), n_real, _lib.ptr(real), n_sim, _lib.ptr(sim),
                                                   float(grad_penalty_coef), max(real.shape[0], 1), _lib.ptr(losses), _lib.ptr(ws)))
        return losses

    @classmethod
    def _borrow(cls, lib, handle, dims, dtype: str) -> "MLP":
        """A view of a network that another object owns (the projections inside a GRU cell): never destroyed here."""
        self = cls.__new__(cls)
        self._lib, self._handle, self.dims, self.dtype, self.activation = lib, handle, list(dims), dtype, "none"
        self._ws = None
        self._borrowed = True
        return self

    def grad_sqnorm(self, acc: torch.Tensor) -> None:
        _lib.require_cuda(acc, dtype=torch.float64)
        _lib.check(self._lib.ks_mlp_grad_sqnorm(self._handle, _lib.current_stream(), _lib.ptr(acc)))

    def adam_step(self, params: "T.KsAdamParams", sqnorm: torch.Tensor | None) -> None:
        _lib.check(self._lib.ks_mlp_adam_step(self._handle, _lib.current_stream(), ctypes.byref(params), _lib.ptr(sqnorm)))

    def parameters(self, gradients: bool = False) -> list[tuple[torch.Tensor, torch.Tensor]]:
        """[(weight (out, in), bias (out))] copies of the fp32 master parameters, or of their gradients."""
        out = []
        for l, (i, o) in enumerate(zip(self.dims[:-1], self.dims[1:])):
            w = torch.empty((o, i), dtype=torch.float32, device="cuda")
            b = torch.empty((o,), dtype=torch.float32, device="cuda")
            _lib.check(self._lib.ks_mlp_get_params(self._handle, _lib.current_stream(), l, _lib.ptr(w), _lib.ptr(b),
                                                   int(gradients)))
            out.append((w, b))
        return out

    def close(self) -> None:
        if getattr(self, "_borrowed", False):
            return
        if self._handle:
            self._lib.ks_mlp_destroy(self._handle)
            self._handle = ctypes.c_void_p()

    def __del__(self):  # pragma: no cover
        try:
            self.close()
        except Exception:
            pass


def random_mlp(dims: Sequence[int], seed: int, activation: str = "elu", dtype: str = "bf16"):
    """Random-init network: W ~ N(0, 1/fan_in), b = 0. Returns (MLP, weights, biases)."""
    rng = np.random.default_rng(seed)
    ws = [rng.normal(scale=1.0 / np.sqrt(i), size=(o, i)).astype(np.float32) for i, o in zip(dims[:-1], dims[1:])]
    bs = [np.zeros(o, dtype=np.float32) for o in dims[1:]]
    return MLP(ws, bs, activation=activation, dtype=dtype), ws, bs
