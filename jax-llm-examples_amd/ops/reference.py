"""Plain PyTorch statements of every op the engine's kernels implement.

These functions define what each hand-written kernel computes.  They are what
the kernel tests compare against, and they let the cache manager, the step
function and the scheduler be exercised on a machine without a GPU.  They are
*not* a serving path: the engine refuses to run on a GPU without the compiled
kernels, and its entry points refuse a CPU device unless a test asks for these
ops by name.  All arithmetic is float32 inside; results are cast to the dtype
the kernel would write.
"""
from __future__ import annotations

import math
from typing import Optional

import torch


def retention_start(retention: tuple, pos: torch.Tensor) -> torch.Tensor:
    """First key position a query at ``pos`` may read (vectorised)."""
    kind = retention[0]
    if kind == "all":
        return torch.zeros_like(pos)
    if kind == "chunk":
        c = int(retention[1])
        return (pos // c) * c
    if kind == "window":
        return (pos - int(retention[1]) + 1).clamp_min(0)
    raise ValueError(f"unknown retention rule {retention!r}")


def values_t(kv_cache: torch.Tensor) -> torch.Tensor:
    """The value planes of the pages as ``[pages, kv_heads, head_dim, page_size]`` (how they lie in memory)."""
    p, _, hk, ps, dh = kv_cache.shape
    return kv_cache[:, 1].view(p, hk, dh, ps)  # a view: writes through it land in the cache


class ReferenceOps:
    name = "reference"

    # ------------------------------------------------------------------ embedding
    def embed(self, token_ids: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
        return table[token_ids.long()].float()

    # ------------------------------------------------------------------ norms
    def add_rmsnorm(self, x, delta, weight, eps: float, out_dtype, want32: bool = False):
        """``x += delta`` (in place, float32), then ``h = x / sqrt(mean(x^2) + eps) * weight``."""
        if delta is not None:
            x.add_(delta.float())
        h = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)
        if weight is not None:
            h = h * weight.float()
        return h.to(out_dtype), (h if want32 else None)

    def add_residual(self, x, delta) -> None:
        x.add_(delta.float())

    def gather_rows(self, x, idx):
        return x[idx.long()]

    # ------------------------------------------------------------------ matrix products
    def linear(self, h, w, out_dtype=None):
        out = h.float() @ w.float().t()
        return out.to(out_dtype or h.dtype)

    def lm_head(self, h, w, tiled: bool = False):
        assert not tiled, "the plain ops read row-major weights"
        return h.float() @ w.float().t()

    def swiglu_linear(self, h, w_gate_up):
        return self.silu_mul(self.linear(h, w_gate_up))

    def materialize(self, delta):
        return delta

    def silu_mul(self, gate_up):
        f = gate_up.shape[-1] // 2
        g, u = gate_up[..., :f].float(), gate_up[..., f:].float()
        return (torch.nn.functional.silu(g) * u).to(gate_up.dtype)

    # ------------------------------------------------------------------ attention
    def qk_prepare_kv_write(self, qkv, num_heads: int, num_kv_heads: int, head_dim: int, positions, prep,
                            kv_cache: Optional[torch.Tensor], slot_mapping: Optional[torch.Tensor]):
        """Splits fused q|k|v rows and prepares q and k as ``prep`` (a
        :class:`~..parts.base.QKPreparation`) says: the rotation turns element pairs by the angle
        ``pos * inv_freq[j]`` (float32) - adjacent pairs ``(x[2j], x[2j+1])`` or half-split pairs
        ``(x[j], x[j + rotary_dim/2])`` of the leading ``rotary_dim`` elements; the RMS norm over the
        head (``x / sqrt(mean(x^2) + eps)``, times a weight if there is one) comes after the rotation,
        or before it with ``norm_first``; ``query_scale = (floor_scale, attn_scale)`` multiplies q by
        ``1 + attn_scale * ln(1 + floor((pos + 1) / floor_scale))``.  Then k and v are written into
        their page at ``slot = page * page_size + offset``.  ``kv_cache`` is ``[pages, 2, kv_heads,
        page_size * head_dim]`` in memory: plane 0 holds keys as ``[page_size, head_dim]``, plane 1
        holds values transposed, ``[head_dim, page_size]``.  Returns q ``[N, num_heads, head_dim]``."""
        n = qkv.shape[0]
        dt = qkv.dtype
        hq, hk, dh = num_heads, num_kv_heads, head_dim
        q = qkv[:, : hq * dh].float().reshape(n, hq, dh)
        k = qkv[:, hq * dh : (hq + hk) * dh].float().reshape(n, hk, dh)
        v = qkv[:, (hq + hk) * dh :].float().reshape(n, hk, dh)

        def norm(x, w):
            x = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + prep.norm_eps)
            return x if w is None else x * w.float()

        if prep.norm_eps is not None and prep.norm_first:
            q, k = norm(q, prep.norm_weight_q), norm(k, prep.norm_weight_k)
        rot = prep.rotation
        if rot is not None:
            rd = int(rot.rotary_dim) or dh
            ang = positions.float()[:, None] * rot.inv_freq.float()[None, :]
            sin, cos = torch.sin(ang)[:, None, :], torch.cos(ang)[:, None, :]

            def turn(x):
                head, rest = x[..., :rd], x[..., rd:]
                if rot.pairing == "adjacent":
                    pairs = head.reshape(n, -1, rd // 2, 2)
                    a, b = pairs[..., 0], pairs[..., 1]
                    head = torch.stack([a * cos - b * sin, b * cos + a * sin], dim=-1).reshape(n, -1, rd)
                else:
                    a, b = head[..., : rd // 2], head[..., rd // 2:]
                    head = torch.cat([a * cos - b * sin, b * cos + a * sin], dim=-1)
                return torch.cat([head, rest], dim=-1)

            q, k = turn(q), turn(k)
        if prep.norm_eps is not None and not prep.norm_first:
            q, k = norm(q, prep.norm_weight_q), norm(k, prep.norm_weight_k)
        if prep.query_scale is not None:
            floor_scale, attn_scale = prep.query_scale
            s = 1.0 + attn_scale * torch.log1p(torch.floor((positions.float() + 1.0) / floor_scale))
            q = q * s[:, None, None]
        if kv_cache is not None:
            ps = kv_cache.shape[3]
            page = (slot_mapping // ps).long()
            off = (slot_mapping % ps).long()
            kv_cache[page, 0, :, off] = k.to(kv_cache.dtype)
            values_t(kv_cache)[page, :, :, off] = v.to(kv_cache.dtype)
        return q.to(dt)

    def attention_from_qkv(self, qkv, num_heads, num_kv_heads, head_dim, positions, token_segment, prep, kv_cache,
                           writes: bool, slot_mapping, block_table, retention, scale: float, meta=None):
        """q and k prepared, k and v written (if this run writes its cache), attention over the pages."""
        q = self.qk_prepare_kv_write(qkv, num_heads, num_kv_heads, head_dim, positions, prep,
                                     kv_cache if writes else None, slot_mapping)
        return self.paged_attention(q, kv_cache, block_table, positions, token_segment, retention, scale, meta)

    def paged_attention(self, q, kv_cache, block_table, positions, token_segment, retention, scale: float, meta=None):
        """For each token: softmax over the keys of its own request at positions
        ``[start(pos), pos]``, read from the pages its block table names."""
        n, hq, dh = q.shape
        hk, ps = kv_cache.shape[2], kv_cache.shape[3]
        g = hq // hk
        out = torch.empty(n, hq * dh, dtype=q.dtype, device=q.device)
        starts = retention_start(retention, positions)
        for i in range(n):
            p = int(positions[i])
            s = int(starts[i])
            kpos = torch.arange(s, p + 1, device=q.device)
            pages = block_table[int(token_segment[i])][(kpos // ps).long()].long()
            if bool((pages < 0).any()):
                raise RuntimeError(f"token {i} at position {p} reads a page that was given back")
            off = (kpos % ps).long()
            k = kv_cache[pages, 0, :, off].float()  # [T, hk, dh]
            v = values_t(kv_cache)[pages, :, :, off].float()
            qi = q[i].float().reshape(hk, g, dh)
            sc = torch.einsum("hgd,thd->hgt", qi, k) * scale
            pr = torch.softmax(sc, dim=-1)
            out[i] = torch.einsum("hgt,thd->hgd", pr, v).reshape(-1).to(q.dtype)
        return out

    # ------------------------------------------------------------------ routed experts
    def moe_route(self, h32, router, top_k: int, group: bool = False):
        """Router logits in float32, the ``top_k`` largest per token (lowest index
        first among equals), gate = sigmoid of the chosen logit.  ``group``: a third result, the
        grouping of the choices by expert for ``moe_experts`` (none here: these ops do not group)."""
        logits = h32.float() @ router.float().t()
        # stable sort by (-logit, index): lowest index wins ties
        order = torch.sort(logits, dim=-1, descending=True, stable=True).indices[:, :top_k]
        vals = torch.gather(logits, 1, order)
        ids, gates = order.to(torch.int32), torch.sigmoid(vals)
        return (ids, gates, None) if group else (ids, gates)

    def moe_experts(self, h, expert_ids, gates, w_gate_up, w_down, shared=None, tiled: bool = False, grouping=None,
                    shared_weights=None):
        """``sum_j  W_down[e_j] (silu(g_j W_gate[e_j] h) * (g_j W_up[e_j] h))`` per token,
        plus ``shared`` if given; float32 result.  ``w_gate_up`` is ``[E, 2F, D]`` (gate rows then
        up rows), ``w_down`` ``[E, D, F]``.  Activations between the two products are
        rounded to the run dtype, as the kernels store them."""
        assert not tiled, "the plain ops read row-major weights"
        if shared is None and shared_weights is not None:
            shared = self.linear(self.swiglu_linear(h, shared_weights[0]), shared_weights[1])
        n, d = h.shape
        f = w_down.shape[2]
        out = torch.zeros(n, d, dtype=torch.float32, device=h.device)
        hf = h.float()
        for j in range(expert_ids.shape[1]):
            for e in torch.unique(expert_ids[:, j]).tolist():
                rows = (expert_ids[:, j] == e).nonzero().squeeze(-1)
                gu = (hf[rows] @ w_gate_up[e].float().t()) * gates[rows, j : j + 1]
                act = (torch.nn.functional.silu(gu[:, :f]) * gu[:, f:]).to(h.dtype).float()
                out[rows] += (act @ w_down[e].float().t()).to(h.dtype).float()
        if shared is not None:
            out += shared.float()
        return out

    # ------------------------------------------------------------------ sampling
    def sample(self, logits, temperature, top_k, seeds, counters, any_top_k: bool = True):
        """Greedy where ``temperature == 0`` (lowest index among equals); otherwise
        Gumbel-max over ``logits / temperature`` restricted to the ``top_k`` largest
        (0 = all), with noise that depends only on (seed, counter, token id)."""
        m, v = logits.shape
        out = torch.empty(m, dtype=torch.int32, device=logits.device)
        ids = torch.arange(v, device=logits.device, dtype=torch.int64)
        for i in range(m):
            row = logits[i].float()
            t = float(temperature[i])
            if t <= 0.0:
                out[i] = int(torch.argmax(row))  # first maximal index
                continue
            z = row / t
            k = int(top_k[i])
            if 0 < k < v:
                kth = torch.topk(z, k).values[-1]
                z = torch.where(z >= kth, z, torch.full_like(z, -math.inf))
            u = uniform_from_hash(int(seeds[i]), int(counters[i]), ids)
            gumbel = -torch.log(-torch.log(u))
            out[i] = int(torch.argmax(z + gumbel))
        return out


def uniform_from_hash(seed: int, counter: int, ids: torch.Tensor) -> torch.Tensor:
    """A uniform in (0, 1) for every token id from a 32-bit mix of (seed, counter, id).
    The kernel computes the same integers; float32 result."""
    M = 0xFFFFFFFF

    def mix(x):
        x = x & M
        x = ((x ^ (x >> 16)) * 0x7FEB352D) & M
        x = ((x ^ (x >> 15)) * 0x846CA68B) & M
        return (x ^ (x >> 16)) & M

    s = mix(torch.tensor((seed * 0x9E3779B1 + 0x85EBCA6B) & M, dtype=torch.int64))
    c = mix(torch.tensor(((counter + 1) * 0xC2B2AE35) & M, dtype=torch.int64) ^ s)
    x = mix((ids.to(torch.int64) * 0x27D4EB2F + c) & M)
    x = mix(x ^ s)
    # 24 high bits -> (0, 1)
    return ((x >> 8).to(torch.float32) + 0.5) * (1.0 / 16777216.0)
