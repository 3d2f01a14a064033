"""Plain torch reference of every kernel, one function per kernel, same signatures
as the HIP operations (`tokensprint_amd.kernels.hip_ops.HipOps`).

Two uses: each HIP kernel is compared with its function here, at sizes of the test's
choosing; and, as an operations provider handed to the engine by a test, it lets the
cache manager, batch builder, step function and scheduler be checked on a machine
without a GPU.  The product never imports this file.
"""

from __future__ import annotations

import torch


class TorchOps:
    name = "torch-reference"

    # ---------------------------------------------------------------- rows
    def embed(self, table, token_ids):
        return table[token_ids.long()].float()

    def gather_rows(self, x, rows):
        return x[rows.long()].contiguous()

    def rmsnorm(self, x, weight, eps, out_dtype):
        xf = x.float()
        rstd = torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
        return (xf * rstd * weight.float()).to(out_dtype)

    def add_rmsnorm(self, resid, delta, weight, eps, out_dtype):
        resid.add_(delta.float())
        return self.rmsnorm(resid, weight, eps, out_dtype)

    def linear(self, x, weight, out_dtype):
        return (x.float() @ weight.float().T).to(out_dtype)

    def norm_linear(self, resid, delta, norm_weight, eps, weight, out_dtype, silu_mul=False):
        act = torch.bfloat16 if weight.dtype == torch.bfloat16 else torch.float32
        h = self.rmsnorm(resid, norm_weight, eps, act) if delta is None \
            else self.add_rmsnorm(resid, delta, norm_weight, eps, act)
        out = self.linear_silu_mul(h, weight, out_dtype) if silu_mul \
            else self.linear(h, weight, out_dtype)
        return out, resid

    def linear_silu_mul(self, x, weight, out_dtype):
        return self.silu_mul(self.linear(x, weight, out_dtype))

    def silu_mul(self, gate_up):
        inner = gate_up.shape[-1] // 2
        g, u = gate_up[:, :inner].float(), gate_up[:, inner:].float()
        return (g * torch.sigmoid(g) * u).to(gate_up.dtype)

    # ---------------------------------------------------------------- q/k preparation
    @staticmethod
    def _head_norm(x, weight, eps):
        if weight is None:
            return x.float()
        xf = x.float()
        return xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * weight.float()

    @staticmethod
    def _rotate(xf, positions, cos, sin):
        half = xf.shape[-1] // 2
        c, s = cos[positions.long()][:, None, :], sin[positions.long()][:, None, :]
        re, im = xf[..., :half], xf[..., half:]
        return torch.cat((re * c - im * s, im * c + re * s), dim=-1)

    def rope_inplace(self, x, positions, cos, sin):
        x.copy_(self._rotate(x.float(), positions, cos, sin).to(x.dtype))

    def qk_norm_split(self, qkv, *, num_heads, num_kv_heads, head_dim, q_weight, k_weight, eps):
        T = qkv.shape[0]
        nq, nkv, hd = num_heads, num_kv_heads, head_dim
        q = qkv[:, :nq * hd].view(T, nq, hd)
        q = self._head_norm(q, q_weight, eps).to(qkv.dtype).contiguous()
        if nkv == 0:
            return q, None, None
        k = qkv[:, nq * hd:(nq + nkv) * hd].view(T, nkv, hd)
        v = qkv[:, (nq + nkv) * hd:].view(T, nkv, hd)
        return q, self._head_norm(k, k_weight, eps).to(qkv.dtype).contiguous(), v.contiguous()

    def kv_store(self, k, v, batch, table, cache):
        P = cache.page_size
        pos = batch.positions.long()
        page = table[batch.entry_of_token.long(), pos // P].long()
        if (page < 0).any():
            raise RuntimeError("store to a position whose page was given back")
        cache.k_pages[page, :, pos % P] = k.to(cache.k_pages.dtype)
        cache.v_pages[page, :, :, pos % P] = v.to(cache.v_pages.dtype)

    def qk_norm_rope_store(self, qkv, batch, table, cache, *, num_heads, num_kv_heads,
                           head_dim, q_weight, k_weight, eps, cos_sin):
        T = qkv.shape[0]
        nq, nkv, hd = num_heads, num_kv_heads, head_dim
        q = self._head_norm(qkv[:, :nq * hd].view(T, nq, hd), q_weight, eps)
        if cos_sin is not None:
            q = self._rotate(q, batch.positions, *cos_sin)
        q = q.to(qkv.dtype).contiguous()
        if nkv and cache is not None:
            k = self._head_norm(qkv[:, nq * hd:(nq + nkv) * hd].view(T, nkv, hd), k_weight, eps)
            if cos_sin is not None:
                k = self._rotate(k, batch.positions, *cos_sin)
            v = qkv[:, (nq + nkv) * hd:].view(T, nkv, hd)
            self.kv_store(k.to(qkv.dtype), v, batch, table, cache)
        return q

    def attend(self, qkv, batch, table, cache, write_cache, *, num_heads, num_kv_heads,
               kv_in_row, head_dim, q_weight, k_weight, eps, cos_sin, scale, window,
               defer_merge=False):
        q = self.qk_norm_rope_store(
            qkv, batch, table, cache if write_cache else None, num_heads=num_heads,
            num_kv_heads=kv_in_row, head_dim=head_dim, q_weight=q_weight, k_weight=k_weight,
            eps=eps, cos_sin=cos_sin)
        return self.paged_attention(q, batch, table, cache, num_heads=num_heads,
                                    num_kv_heads=num_kv_heads, head_dim=head_dim,
                                    scale=scale, window=window)

    # ---------------------------------------------------------------- attention
    def paged_attention(self, q, batch, table, cache, *, num_heads, num_kv_heads, head_dim,
                        scale, window, only=None):
        """`only`: compute just these flat tokens (a test's choice; the other rows of the
        result are left unset)."""
        T = q.shape[0]
        P = cache.page_size
        group = num_heads // num_kv_heads
        out = torch.empty(T, num_heads, head_dim, dtype=torch.float32, device=q.device)
        for t in (range(T) if only is None else only):
            b = int(batch.entry_of_token[t])
            p = int(batch.positions[t])
            lo = 0 if window is None else max(0, p - window + 1)
            keys = torch.arange(lo, p + 1, device=q.device)
            pages = table[b, keys // P].long()
            if (pages < 0).any():
                raise RuntimeError("attention reads a position whose page was given back")
            k = cache.k_pages[pages, :, keys % P].float()       # [n, nkv, hd]
            v = cache.v_pages[pages, :, :, keys % P].float()
            for j in range(num_heads):
                s = (k[:, j // group] @ q[t, j].float()) * scale
                out[t, j] = torch.softmax(s, dim=0) @ v[:, j // group]
        return out.to(q.dtype)

    # ---------------------------------------------------------------- sampling
    def argmax(self, logits):
        return logits.float().argmax(dim=-1).to(torch.int32)
