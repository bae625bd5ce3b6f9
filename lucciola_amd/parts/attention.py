"""Grouped-query attention over the paged cache, as a part.

Order of operations as in the reference's layer (src/qwen.cc:592-738): q, k, v projections
(one product here, the weights are stacked at load) -> RMSNorm over head_dim on every q and k
head with one [d] weight each -> rotary embedding of q and k -> k, v written to the cache ->
causal attention over all cached keys (kv head = h / (nh / nkv), scale 1/sqrt(d)) -> output
projection.  Sizes, the scale, the norm, the position encoding and an optional window are
parameters; nh * d need not equal the hidden size.

Beyond the reference: values of another size than the keys (``value_dim``), a learned factor on
every head's scores (``head_temperature``), and a layer without keys and values of its own
(``shared_kv``: it reads the cache of the site that the run order names as ``cache_of``, with its
own queries).  With any of these the part prepares q, k and v with a kernel of its own: the norm
is taken over the key size, the temperature is folded into the normed queries, and keys and
values lie in the cache in head slots of one size (the larger of the two, zeros behind the
shorter), so that the attention kernels serve them as they are.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..cache.specs import PagedKV
from ..config.registry import MIXERS, NORMS, POSITION_ENCODINGS
from ..config.specs import PartSpec
from ..kernels import ops
from ..weights.loader import ParamDecl
from .base import BuildContext, Part, build_part
from .feed_forward import stack_rows


@MIXERS.register("attention")
class Attention(Part):
    graph_safe = True   # launches only kernels whose arguments stay put between steps
    takes_scaled_rows = True   # x may be ops.ScaledRows; the output may be an ops.PendingProduct

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 scale: Optional[float] = None, qk_norm: Optional[PartSpec] = None,
                 position: Optional[PartSpec] = None, window: Optional[int] = None,
                 value_dim: Optional[int] = None, head_temperature: bool = False, shared_kv: bool = False):
        super().__init__(hidden_size=hidden_size, num_heads=num_heads, num_kv_heads=num_kv_heads,
                         head_dim=head_dim, scale=scale, qk_norm=qk_norm, position=position,
                         window=window, value_dim=value_dim, head_temperature=head_temperature,
                         shared_kv=shared_kv)
        if num_heads % num_kv_heads:
            raise ValueError(f"attention: {num_heads} heads are not a multiple of "
                             f"{num_kv_heads} kv heads")
        self.H, self.nh, self.nkv, self.d = int(hidden_size), int(num_heads), int(num_kv_heads), int(head_dim)
        self.scale = float(scale) if scale is not None else self.d ** -0.5
        self.window = int(window) if window else None
        self.dv = int(value_dim) if value_dim else self.d
        self.head_temperature, self.shared_kv = bool(head_temperature), bool(shared_kv)
        # the head slot of the cache and of the attention kernels: the key size itself, or, on the
        # part's own path, the size that holds the longer of key and value
        self.own_prologue = self.dv != self.d or self.head_temperature or self.shared_kv
        self.slot = ops.attention_head_slot(max(self.d, self.dv)) if self.own_prologue else self.d
        if self.own_prologue and position is not None:
            raise ValueError("attention: value_dim, head_temperature and shared_kv go without a position encoding")
        self.fused_qk_norm = True
        self.q_norm = build_part(NORMS, qk_norm) if qk_norm else None
        self.k_norm = build_part(NORMS, qk_norm) if qk_norm else None
        self.position = build_part(POSITION_ENCODINGS, position) if position else None
        if getattr(self.position, "pairing", "half") != "half":
            raise ValueError("attention: its kernels rotate entry i with entry i + rot/2 only "
                             "(pairing 'half')")

    def declare(self) -> Dict[str, ParamDecl]:
        out = {"q_proj": ParamDecl((self.nh * self.d, self.H)),
               "o_proj": ParamDecl((self.H, self.nh * self.dv))}
        if not self.shared_kv:
            out["k_proj"] = ParamDecl((self.nkv * self.d, self.H))
            out["v_proj"] = ParamDecl((self.nkv * self.dv, self.H))
        if self.head_temperature:
            out["head_temperature"] = ParamDecl((self.nh,), role="vector", init="ones_plus_normal")
        if self.q_norm is not None:
            for name, decl in self.q_norm.declare().items():
                out["q_norm." + name] = decl
            if not self.shared_kv:
                for name, decl in self.k_norm.declare().items():
                    out["k_norm." + name] = decl
        return out

    def bind(self, tensors, ctx: BuildContext) -> None:
        self.dtype = ctx.dtype
        if self.own_prologue:
            self._bind_own(tensors, ctx)
            return
        self.qkv = stack_rows([tensors["q_proj"], tensors["k_proj"], tensors["v_proj"]])
        self.o = tensors["o_proj"]
        if self.q_norm is not None:
            self.q_norm.bind({k[7:]: v for k, v in tensors.items() if k.startswith("q_norm.")}, ctx)
            self.k_norm.bind({k[7:]: v for k, v in tensors.items() if k.startswith("k_norm.")}, ctx)
            # a norm that the fused kernel cannot apply (no fused_rms()) is applied through its
            # own ``apply`` on the heads, one kernel more a step
            fused = getattr(self.q_norm, "fused_rms", None)
            self.fused_qk_norm = fused is not None and fused() is not None
            if not self.fused_qk_norm and not hasattr(self.q_norm, "apply"):
                raise NotImplementedError("attention: the q/k norm must offer fused_rms() or apply()")
        if self.position is not None:
            self.position.bind({}, ctx)

    def _norm_heads(self, qkv: torch.Tensor) -> None:
        """The q and k heads of ``qkv`` [T, (nh + 2 nkv) d] through the norms' own ``apply``."""
        T = qkv.shape[0]
        for norm, first, heads in ((self.q_norm, 0, self.nh), (self.k_norm, self.nh, self.nkv)):
            cols = slice(first * self.d, (first + heads) * self.d)
            x = qkv[:, cols].contiguous().view(T * heads, self.d)
            qkv[:, cols] = norm.apply(x).view(T, heads * self.d)

    def _bind_own(self, tensors, ctx: BuildContext) -> None:
        """The part's own path: q (and k, v) stacked as they are; the output projection takes
        heads in slots (zero columns behind a value shorter than its slot)."""
        mats = [tensors["q_proj"]] + ([] if self.shared_kv else [tensors["k_proj"], tensors["v_proj"]])
        self.qkv = stack_rows(mats)
        o = tensors["o_proj"]
        if self.slot != self.dv:
            wide = o.new_zeros((self.H, self.nh, self.slot))
            wide[:, :, :self.dv] = o.view(self.H, self.nh, self.dv)
            o = wide.view(self.H, self.nh * self.slot).contiguous()
        self.o = o
        self.q_weight = self.k_weight = None
        self.norm_eps = 0.0
        if self.q_norm is not None:
            self.q_norm.bind({k[7:]: v for k, v in tensors.items() if k.startswith("q_norm.")}, ctx)
            fused = self.q_norm.fused_rms() if hasattr(self.q_norm, "fused_rms") else None
            if fused is None:
                raise NotImplementedError("attention: on this path the q/k norm must be an RMS norm")
            self.q_weight, self.norm_eps = fused
            if not self.shared_kv:
                self.k_norm.bind({k[7:]: v for k, v in tensors.items() if k.startswith("k_norm.")}, ctx)
                self.k_weight, _ = self.k_norm.fused_rms()
        self.temperature = tensors["head_temperature"].to(torch.float32).contiguous() \
            if self.head_temperature else None

    def _forward_own(self, x, site) -> torch.Tensor:
        attn = ops.attention_batch(site.batch, site.pages, site.batch.plans.get(ops.ATTENTION_PLAN))
        page_size = site.pages.page_size
        proj = ops.gemm(x, self.qkv, self.dtype)
        k_cache, v_cache = site.cache
        writes = site.writes_cache and not self.shared_kv
        q = ops.head_norm_write(proj, self.nh, 0 if self.shared_kv else self.nkv, self.d, self.dv, self.slot,
                                self.q_weight, self.k_weight, self.norm_eps, self.temperature,
                                k_cache if writes else None, v_cache if writes else None,
                                attn.slots if writes else None, page_size)
        o = ops.attention(q, attn, k_cache, v_cache, self.nh, self.nkv, self.slot, page_size,
                          self.scale, self.window or 0, None)
        return ops.gemm(o, self.o, self.dtype, defer=True)

    def cache_need(self):
        return PagedKV(self.nkv, self.slot, self.window, granule=ops.attention_page_granule())

    def batch_planner(self):
        return ops.ATTENTION_PLAN, ops.plan_attention

    def tables_epoch(self) -> int:
        return self.position.tables_epoch() if self.position is not None else 0

    def ready(self, position: int) -> bool:
        return self.position.ready(position) if self.position is not None else True

    def forward(self, x: torch.Tensor, site) -> torch.Tensor:
        if self.own_prologue:
            return self._forward_own(x, site)
        # the attention kernels' record of the step: made once a step for the page group, from
        # the batch, the group's pages and the work lists of this part's planner
        attn = ops.attention_batch(site.batch, site.pages, site.batch.plans.get(ops.ATTENTION_PLAN))
        page_size = site.pages.page_size
        q_w = k_w = None
        eps = 0.0
        own_norm = self.q_norm is not None and not self.fused_qk_norm
        if self.q_norm is not None and self.fused_qk_norm:
            q_w, eps = self.q_norm.fused_rms()
            k_w, _ = self.k_norm.fused_rms()
        table = None
        if self.position is not None:
            table = self.position.rotary_table(site.batch.max_position)
        # where the q/k/v product is cut along K and the attention kernel can sum its shares
        # as it reads them, the kernel that would sum them is saved
        rows = x.x.shape[0] if isinstance(x, ops.ScaledRows) else x.shape[0]
        as_shares = ((table is not None or self.position is None) and not own_norm
                     and ops.attention_takes_shares(attn, rows, self.nh, self.nkv, self.d, page_size,
                                                    self.dtype, table.shape[1] if table is not None else 0))
        qkv = ops.gemm(x, self.qkv, self.dtype, shares=as_shares)
        if own_norm:
            self._norm_heads(qkv)
        if self.position is not None and table is None:
            self.position.apply(qkv, self.nh, self.nkv, self.d, attn.positions)
        k_cache, v_cache = site.cache
        prologue = ops.QKPrologue(q_w, k_w, eps, table, attn.slots if site.writes_cache else None)
        o = ops.attention(qkv, attn, k_cache, v_cache, self.nh, self.nkv, self.d, page_size,
                          self.scale, self.window or 0, prologue)
        return ops.gemm(o, self.o, self.dtype, defer=True)
