"""Grouped-query softmax attention over a paged key/value cache.

Order of operations follows engine/nn/attention.py:171-198: q/k/v projections,
per-head RMSNorm on q and k (one weight vector shared by all heads, :178-182)
before the position encoding (:184), keys and values written to the cache after
both (:186-188), causal attention with scale head_dim^-0.5 where query head j reads
key/value head j // (nq/nkv) (engine/nn/sdpa.py:56,85-102), output projection.
The three projections run as one product over row-concatenated weights.
"""

from __future__ import annotations

import torch

from tokensprint_amd.kernels.stream import StreamProducts, fused_rmsnorm_of
from tokensprint_amd.parts.base import MIXERS, Mixer, PagedKVNeed, TensorDecl, register


@register(MIXERS, "gqa_attention")
class GroupedQueryAttention(StreamProducts, Mixer):
    """params: prefix, num_heads, num_kv_heads, head_dim, qk_norm (bool), qk_norm_eps,
    position (name of a shared position encoding or None), window (None = all keys),
    own_kv (False: the layer has no k/v weights and only reads another run's cache).
    """

    def __init__(self, params, ctx):
        super().__init__(params, ctx)
        p = params
        self.prefix = p["prefix"]
        self.nq, self.nkv, self.hd = int(p["num_heads"]), int(p["num_kv_heads"]), int(p["head_dim"])
        self.qk_norm = bool(p.get("qk_norm", False))
        self.eps = float(p.get("qk_norm_eps", 0.0))
        self.window = p.get("window")
        self.own_kv = bool(p.get("own_kv", True))
        self.scale = float(self.hd) ** -0.5
        self.position = ctx.positions[p["position"]] if p.get("position") else None
        if self.nq % self.nkv:
            raise ValueError(f"num_heads={self.nq} is not a multiple of num_kv_heads={self.nkv}")
        self.w_qkv = self.w_o = self.w_qnorm = self.w_knorm = None

    # -- weights
    def tensors(self):
        H, pre = self.ctx.width, self.prefix
        t = {pre + "q_proj.weight": TensorDecl((self.nq * self.hd, H)),
             pre + "o_proj.weight": TensorDecl((H, self.nq * self.hd))}
        if self.own_kv:
            t[pre + "k_proj.weight"] = TensorDecl((self.nkv * self.hd, H))
            t[pre + "v_proj.weight"] = TensorDecl((self.nkv * self.hd, H))
        if self.qk_norm:
            t[pre + "q_norm.weight"] = TensorDecl((self.hd,), role="vector")
            if self.own_kv:
                t[pre + "k_norm.weight"] = TensorDecl((self.hd,), role="vector")
        return t

    def load(self, get):
        pre = self.prefix
        rows = [get(pre + "q_proj.weight")]
        if self.own_kv:
            rows += [get(pre + "k_proj.weight"), get(pre + "v_proj.weight")]
        if len({r.dtype for r in rows}) != 1:
            raise ValueError(f"{pre}: q/k/v projection weights are stored in different dtypes")
        self.w_qkv = torch.cat(rows, dim=0).contiguous() if len(rows) > 1 else rows[0]
        self.w_o = get(pre + "o_proj.weight")
        if self.qk_norm:
            self.w_qnorm = get(pre + "q_norm.weight")
            self.w_knorm = get(pre + "k_norm.weight") if self.own_kv else None

    def cache_need(self):
        return PagedKVNeed(self.nkv, self.hd, self.window)

    # -- step
    def stream_hint(self, norm):
        return self.first_product_hint(norm, self.w_qkv)

    def forward_from_stream(self, resid, delta, norm, batch, cache, write_cache, hint=None):
        fused = fused_rmsnorm_of(norm)
        if fused is None:
            return super().forward_from_stream(resid, delta, norm, batch, cache, write_cache)
        qkv, resid = self.ops.norm_linear(resid, delta, fused[0], fused[1], self.w_qkv,
                                          self.ctx.dtype)
        o = self._attend(qkv, batch, cache, write_cache)
        return self.last_product(o, self.w_o, resid, hint), resid

    def forward(self, h, batch, cache, write_cache):
        o = self._attend(self.ops.linear(h, self.w_qkv, self.ctx.dtype), batch, cache, write_cache)
        return self.ops.linear(o, self.w_o, self.ctx.dtype)

    def _attend(self, qkv, batch, cache, write_cache):
        if cache is None:
            raise RuntimeError("gqa_attention needs a paged key/value cache")
        if write_cache and not self.own_kv:
            raise RuntimeError(f"{self.prefix}: a layer without k/v weights cannot own a cache")
        ops, T = self.ops, qkv.shape[0]
        nkv_here = self.nkv if self.own_kv else 0
        table = batch.tables[cache.group]
        tables = self.position.rotary_tables() if self.position is not None else None
        fused = self.position is None or tables is not None
        if fused:
            o = ops.attend(
                qkv, batch, table, cache, write_cache, num_heads=self.nq,
                num_kv_heads=self.nkv, kv_in_row=nkv_here, head_dim=self.hd,
                q_weight=self.w_qnorm, k_weight=self.w_knorm, eps=self.eps,
                cos_sin=tables, scale=self.scale, window=self.window,
                # the result goes into the output projection, a product of the same provider,
                # which may then finish attention's last stage itself: it may come back as
                # a handle (kernels.stream.UnmergedRows) in place of a tensor
                defer_merge=True)
        else:
            # the encoding has no rotary table: norm only, let it encode, then store
            q, k, v = ops.qk_norm_split(
                qkv, num_heads=self.nq, num_kv_heads=nkv_here, head_dim=self.hd,
                q_weight=self.w_qnorm, k_weight=self.w_knorm, eps=self.eps)
            self.position.apply(q, k, batch.positions)
            if write_cache:
                ops.kv_store(k, v, batch, table, cache)
            o = ops.paged_attention(q, batch, table, cache, num_heads=self.nq,
                                    num_kv_heads=self.nkv, head_dim=self.hd,
                                    scale=self.scale, window=self.window)
        return o.view(T, self.nq * self.hd)
