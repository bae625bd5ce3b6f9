"""Mixers that keep a matrix of state per head and request instead of keys and values, both
delta rules: a token first takes out of the state what it holds along a probe direction, then
writes its own key/value pair, and reads with a query.

Both are instances of one recurrence per head (``ops.delta_scan``; in memory the state lies
transposed, [slot, head, value, key], and only that kernel reads it), with the state S [key, value]
and, per token, five vectors over the key channels and the value v:

    S <- diag(decay) S - removal (probe^T S) + write v^T        (probe^T S: of S as the last token left it)
    o  = S^T read

``general_delta`` (the generalized delta rule): decay w = exp(-c sigmoid(W2 tanh(W1 h) + w0)) per
key channel, removal rate a = sigmoid(W_a h + b_a) per key channel, unit key u = k / sqrt(|k|^2 +
eps): decay = w, probe = u, removal = a u, write = k, read = r.

``gated_delta`` (the gated delta rule): q, k, v pass a short causal convolution per channel and
SiLU; q and k are made unit vectors, q times key_dim^(-1/2); one decay g = exp(-exp(A) softplus(W_a h
+ b)) and one write strength beta = sigmoid(W_b h) per head.  S <- g S; u = beta (v - S^T k); S <- S
+ k u^T is the recurrence above with decay = g, probe = g k, removal = beta k, write = beta k.  The
last ``taps - 1`` inputs of the convolutions are state as well.

Everything between the projections and the output product is float32: the projections leave as
float32, a kernel turns them into the five vectors (gates, exponentials, unit vectors), the scan
keeps S in float32, and the read-out is divided by its root mean square per head and gated before
it is rounded for the output product.  A step's tokens are scanned in order within each request
from the state that the request's slot holds, whatever the cut of the prompt.
"""
from __future__ import annotations

from typing import Dict

import torch

from ..cache.specs import FixedStates
from ..config.registry import MIXERS
from ..kernels import ops
from ..weights.loader import ParamDecl
from .base import BuildContext, Part
from .feed_forward import stack_rows


def _f32(t: torch.Tensor) -> torch.Tensor:
    return t.to(torch.float32).contiguous()


@MIXERS.register("general_delta")
class GeneralDelta(Part):
    graph_safe = True   # launches only kernels whose arguments stay put between steps

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, norm_eps: float,
                 unit_eps: float = 1e-6, decay_scale: float = 0.6065306597126334):
        super().__init__(hidden_size=hidden_size, num_heads=num_heads, head_dim=head_dim, norm_eps=norm_eps,
                         unit_eps=unit_eps, decay_scale=decay_scale)
        self.H, self.nh, self.d = int(hidden_size), int(num_heads), int(head_dim)
        self.norm_eps, self.unit_eps, self.decay_scale = float(norm_eps), float(unit_eps), float(decay_scale)
        ops.check_delta_sizes("general_delta", self.d, self.d)

    def declare(self) -> Dict[str, ParamDecl]:
        n = self.nh * self.d
        # the inner size of the decay's two small matrices is whatever the checkpoint holds
        return {"r": ParamDecl((n, self.H)), "k": ParamDecl((n, self.H)), "v": ParamDecl((n, self.H)),
                "gate": ParamDecl((n, self.H)), "removal": ParamDecl((n, self.H)),
                "removal_bias": ParamDecl((n,), role="vector"),
                "decay_in": ParamDecl((-1, self.H)), "decay_out": ParamDecl((n, -1)),
                "decay_bias": ParamDecl((n,), role="vector"),
                "norm": ParamDecl((n,), role="vector", init="ones_plus_normal"), "o": ParamDecl((self.H, n))}

    def bind(self, tensors, ctx: BuildContext) -> None:
        self.dtype = ctx.dtype
        self.inner = int(tensors["decay_in"].shape[0])
        if tensors["decay_out"].shape[1] != self.inner:
            raise ValueError(f"general_delta: the decay's matrices do not fit each other "
                             f"({tuple(tensors['decay_in'].shape)}, {tuple(tensors['decay_out'].shape)})")
        self.proj = stack_rows([tensors[k] for k in ("r", "k", "v", "gate", "removal", "decay_in")])
        self.decay_out = _f32(tensors["decay_out"])
        self.decay_bias, self.removal_bias = _f32(tensors["decay_bias"]), _f32(tensors["removal_bias"])
        self.norm, self.o = _f32(tensors["norm"]), tensors["o"]

    def cache_need(self):
        return FixedStates(((self.nh, self.d, self.d),))

    def forward(self, x: torch.Tensor, site) -> torch.Tensor:
        batch = site.batch
        (state,) = site.cache
        proj = ops.gemm(x, self.proj, torch.float32)
        coef, v = ops.general_delta_prepare(proj, self.nh, self.d, self.inner, self.decay_out, self.decay_bias,
                                            self.removal_bias, self.unit_eps, self.decay_scale)
        o = ops.delta_scan(coef, v, state, batch.q_offsets, batch.slot_ids, batch.num_requests,
                           self.nh, self.d, self.d)
        n = self.nh * self.d
        y = ops.head_gate_norm(o, proj, 3 * n, self.norm, True, self.norm_eps, "sigmoid", self.nh, self.d,
                               self.dtype)
        return ops.gemm(y, self.o, self.dtype, defer=True)


@MIXERS.register("gated_delta")
class GatedDelta(Part):
    graph_safe = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, key_dim: int, value_dim: int,
                 conv_taps: int, norm_eps: float, unit_eps: float = 1e-6):
        super().__init__(hidden_size=hidden_size, num_heads=num_heads, num_kv_heads=num_kv_heads, key_dim=key_dim,
                         value_dim=value_dim, conv_taps=conv_taps, norm_eps=norm_eps, unit_eps=unit_eps)
        if num_heads % num_kv_heads:
            raise ValueError(f"gated_delta: {num_heads} heads are not a multiple of {num_kv_heads} kv heads")
        self.H, self.nh, self.nkv = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.dk, self.dv, self.taps = int(key_dim), int(value_dim), int(conv_taps)
        self.norm_eps, self.unit_eps = float(norm_eps), float(unit_eps)
        self.channels = 2 * self.nkv * self.dk + self.nh * self.dv       # what passes the convolutions
        ops.check_delta_sizes("gated_delta", self.dk, self.dv, self.taps)

    def declare(self) -> Dict[str, ParamDecl]:
        nk, nv = self.nkv * self.dk, self.nh * self.dv
        return {"q": ParamDecl((nk, self.H)), "q_conv": ParamDecl((nk, self.taps), role="vector"),
                "k": ParamDecl((nk, self.H)), "k_conv": ParamDecl((nk, self.taps), role="vector"),
                "v": ParamDecl((nv, self.H)), "v_conv": ParamDecl((nv, self.taps), role="vector"),
                "beta": ParamDecl((self.nh, self.H)), "rate": ParamDecl((self.nh, self.H)),
                "rate_log": ParamDecl((self.nh,), role="vector"), "rate_bias": ParamDecl((self.nh,), role="vector"),
                "norm": ParamDecl((self.dv,), role="vector", init="ones_plus_normal"),
                "gate": ParamDecl((nv, self.H)), "o": ParamDecl((self.H, nv))}

    def bind(self, tensors, ctx: BuildContext) -> None:
        self.dtype = ctx.dtype
        self.proj = stack_rows([tensors[k] for k in ("q", "k", "v", "gate", "beta", "rate")])
        self.conv = torch.cat([_f32(tensors[k]) for k in ("q_conv", "k_conv", "v_conv")], dim=0).contiguous()
        self.rate_log, self.rate_bias = _f32(tensors["rate_log"]), _f32(tensors["rate_bias"])
        self.norm, self.o = _f32(tensors["norm"]), tensors["o"]

    def cache_need(self):
        return FixedStates(((self.nh, self.dv, self.dk), (max(self.taps - 1, 0), self.channels)))

    def forward(self, x: torch.Tensor, site) -> torch.Tensor:
        batch = site.batch
        state, tail = site.cache
        proj = ops.gemm(x, self.proj, torch.float32)
        coef, v = ops.gated_delta_prepare(proj, tail, self.conv, self.rate_log, self.rate_bias, self.nh, self.nkv,
                                          self.dk, self.dv, self.taps, self.unit_eps, batch.tok_req,
                                          batch.q_offsets, batch.slot_ids)
        ops.conv_tail_update(proj, tail, self.channels, self.taps, batch.q_offsets, batch.slot_ids,
                             batch.num_requests)
        o = ops.delta_scan(coef, v, state, batch.q_offsets, batch.slot_ids, batch.num_requests,
                           self.nh, self.dk, self.dv)
        y = ops.head_gate_norm(o, proj, self.channels, self.norm, False, self.norm_eps, "silu", self.nh, self.dv,
                               self.dtype)
        return ops.gemm(y, self.o, self.dtype, defer=True)
