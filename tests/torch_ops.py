"""Plain torch stand-ins for the HIP kernels, one per kernel, with the kernels' interface.

Two uses, both in tests only (the package itself has no such path and refuses to run without
its HIP library):
- the reference each kernel is compared with on the GPU;
- a way to run the host side of the engine (cache manager, step function, scheduler, replay)
  on a machine without GPU, by handing this object to the Runtime in place of the kernels.

Everything computes in float32 and rounds to the storage dtype at the end, like the kernels.
"""
import math

import numpy as np
import torch


# ---------------------------------------------------------------- counter-based noise (same as sampling.hip)

def _philox_first(c0, c1, k0, k1, c2=0, c3=0):
    """First output word of Philox4x32-10 for counters (c0, c1, c2, c3) and key (k0, k1); numpy uint64 maths."""
    M0, M1 = np.uint64(0xD2511F53), np.uint64(0xCD9E8D57)
    mask = np.uint64(0xFFFFFFFF)
    c0 = c0.astype(np.uint64)
    c1 = np.full_like(c0, c1, dtype=np.uint64)
    c2 = np.full_like(c0, c2, dtype=np.uint64)
    c3 = np.full_like(c0, c3, dtype=np.uint64)
    k0 = np.uint64(k0)
    k1 = np.uint64(k1)
    for _ in range(10):
        p0 = M0 * c0
        p1 = M1 * c2
        hi0, lo0 = p0 >> np.uint64(32), p0 & mask
        hi1, lo1 = p1 >> np.uint64(32), p1 & mask
        c0, c1, c2, c3 = (hi1 ^ c1 ^ k0) & mask, lo1, (hi0 ^ c3 ^ k1) & mask, lo0
        k0 = (k0 + np.uint64(0x9E3779B9)) & mask
        k1 = (k1 + np.uint64(0xBB67AE85)) & mask
    return c0


def gumbel_noise(seed, draw, V):
    """float32 [V]: -log(-log(u_i)), u_i = ((r_i >> 9) + 0.5) / 2^23, strictly inside (0, 1)."""
    seed = int(seed) & 0xFFFFFFFFFFFFFFFF
    r = _philox_first(np.arange(V, dtype=np.uint64), int(draw) & 0xFFFFFFFF, seed & 0xFFFFFFFF, seed >> 32)
    u = ((r >> np.uint64(9)).astype(np.float32) + np.float32(0.5)) * np.float32(1.0 / 8388608.0)
    assert u.min() > 0.0 and u.max() < 1.0
    return torch.from_numpy(-np.log(-np.log(u))).to(torch.float32)


def _order_key(x):
    """Order-preserving uint32 image of float32 values (as int64 tensor)."""
    b = x.contiguous().view(torch.int32).to(torch.int64) & 0xFFFFFFFF
    b = torch.where(b == 0x80000000, torch.zeros_like(b), b)      # -0 and +0 are one value
    neg = (b & 0x80000000) != 0
    return torch.where(neg, (~b) & 0xFFFFFFFF, b | 0x80000000)


class TorchOps:
    name = "torch-standin"

    # ------------------------------------------------------------ embedding / norm
    def embedding(self, ids, table, scale=1.0):
        return table[ids.long()].to(torch.float32) * scale

    def bad_token_seen(self):
        return False

    def patch_tokens(self, ids, src, prev):
        take = src[:ids.numel()] >= 0
        ids[take] = prev[src[:ids.numel()][take].long()].to(ids.dtype)

    def add_rms_norm(self, branch, residual, weight, eps, out_dtype, rows=None, weight_offset=0.0, defer_ok=False):
        x = None
        if branch is not None:
            x = branch.to(torch.float32)
        if residual is not None:
            x = residual if x is None else x + residual
        if branch is not None and residual is not None and rows is None:
            residual.copy_(x)
        if rows is not None:
            x = x[rows.long()]
        var = (x * x).mean(dim=-1, keepdim=True)
        y = x * torch.rsqrt(var + eps) * (weight.to(torch.float32) + weight_offset)
        return y.to(out_dtype)

    # ------------------------------------------------------------ rotary + cache write
    def rope_cache_write(self, qkv, nh, nkv, d, positions, table, rot_dim, neox, slots, k_pages, v_pages):
        N = qkv.shape[0]
        q = qkv[:, :nh * d].reshape(N, nh, d)
        k = qkv[:, nh * d:(nh + nkv) * d].reshape(N, nkv, d)
        v = qkv[:, (nh + nkv) * d:(nh + 2 * nkv) * d].reshape(N, nkv, d)
        if table is not None:
            half = rot_dim // 2
            cs = table[positions.long()]
            cos, sin = cs[:, None, :half], cs[:, None, half:]

            def rot(x):
                x32 = x.to(torch.float32)
                out = x32.clone()
                if neox:
                    a, b = x32[..., :half], x32[..., half:rot_dim]
                    out[..., :half] = a * cos - b * sin
                    out[..., half:rot_dim] = b * cos + a * sin
                else:
                    a, b = x32[..., 0:rot_dim:2], x32[..., 1:rot_dim:2]
                    out[..., 0:rot_dim:2] = a * cos - b * sin
                    out[..., 1:rot_dim:2] = b * cos + a * sin
                return out.to(x.dtype)

            q, k = rot(q), rot(k)
            qkv[:, :nh * d] = q.reshape(N, nh * d)
            qkv[:, nh * d:(nh + nkv) * d] = k.reshape(N, nkv * d)
        if slots is not None:
            ps = k_pages.shape[2]
            sl = slots.long()
            ok = sl >= 0
            page, off = sl[ok] // ps, sl[ok] % ps
            k_pages[page, :, off, :] = k[ok]
            v_pages[page, :, :, off] = v[ok]

    def qkv_rope_cache(self, x, weight, bias, nh, nkv, d, positions, table, rot_dim, neox, slots, k_pages, v_pages):
        y = self.linear(x, weight, bias)
        if table is not None or slots is not None:
            self.rope_cache_write(y, nh, nkv, d, positions, table, rot_dim, neox, slots, k_pages, v_pages)
        return y

    # ------------------------------------------------------------ attention
    def paged_attention(self, q, k_pages, v_pages, block_tables, seg, pos, nh, nkv, d, scale, window=0, batch=None):
        N = q.shape[0]
        ps = k_pages.shape[2]
        out = torch.empty((N, nh * d), dtype=q.dtype, device=q.device)
        rep = nh // nkv
        for t in range(N):
            s, p = int(seg[t]), int(pos[t])
            lo = max(0, p - window + 1) if window and window > 0 else 0
            js = torch.arange(lo, p + 1, device=q.device)
            pages = block_tables[s].long()[js // ps]
            keys = k_pages[pages, :, js % ps, :].to(torch.float32)      # [n, nkv, d]
            vals = v_pages[pages, :, :, js % ps].to(torch.float32)      # [n, nkv, d]
            qt = q[t, :nh * d].to(torch.float32).reshape(nh, d)
            keys = keys.repeat_interleave(rep, dim=1)                    # [n, nh, d]
            vals = vals.repeat_interleave(rep, dim=1)
            sc = torch.einsum("hd,nhd->hn", qt, keys) * scale
            pr = torch.softmax(sc, dim=-1)
            out[t] = torch.einsum("hn,nhd->hd", pr, vals).reshape(nh * d).to(q.dtype)
        return out

    # ------------------------------------------------------------ feed-forward / linear
    def gated_act(self, gu, kind="silu"):
        I = gu.shape[1] // 2
        g, u = gu[:, :I].to(torch.float32), gu[:, I:].to(torch.float32)
        if kind == "silu":
            a = g / (1.0 + torch.exp(-g))
        elif kind == "gelu":
            a = 0.5 * g * (1.0 + torch.erf(g / math.sqrt(2.0)))
        else:
            raise ValueError(kind)
        return (a * u).to(gu.dtype)

    def linear_gated(self, x, weight, bias=None, kind="silu"):
        return self.gated_act(self.linear(x, weight, bias), kind)

    def linear(self, x, weight, bias=None, out_dtype=None, pending_ok=False, out=None):
        y = x.to(torch.float32) @ weight.to(torch.float32).t()
        if bias is not None:
            y = y + bias.to(torch.float32)
        y = y.to(out_dtype or x.dtype)
        return y if out is None else out.copy_(y)

    def materialize(self, y):
        return y

    # ------------------------------------------------------------ sampling
    def sample(self, logits, temperature=None, top_k=None, top_p=None, min_p=None, seeds=None, draws=None):
        R, V = logits.shape
        out = torch.empty(R, dtype=torch.int32, device=logits.device)
        for r in range(R):
            T = float(temperature[r]) if temperature is not None else 0.0
            row = logits[r].to(torch.float32).cpu()
            if T < 1e-5:
                out[r] = int(torch.argmax(row))      # first maximum
                continue
            x = row * np.float32(1.0 / np.float32(T))
            keys = _order_key(x)
            mx = x.max()
            cut = 0
            k = int(top_k[r]) if top_k is not None else -1
            if 0 < k < V:
                cut = int(torch.sort(keys, descending=True).values[k - 1])
            p = float(top_p[r]) if top_p is not None else 1.0
            if p < 1.0:
                e = torch.where(keys >= cut, torch.exp(x - mx), torch.zeros_like(x))
                target = np.float32(p) * e.sum()
                order = torch.argsort(keys, descending=True)
                csum = torch.cumsum(e[order], dim=0)
                # largest key whose mass of keys >= it reaches the target (ties counted together)
                sk = keys[order]
                group_end = torch.cat([sk[1:] != sk[:-1], torch.ones(1, dtype=torch.bool)])
                hit = torch.nonzero(group_end & (csum >= target))
                best = max(cut, int(sk[int(hit[0])])) if hit.numel() else cut
                cut = best
            mp = float(min_p[r]) if min_p is not None else 0.0
            if mp > 0.0:
                c = int(_order_key((mx + np.float32(math.log(mp))).reshape(1))[0])
                cut = max(cut, c)
            cut = min(cut, int(_order_key(mx.reshape(1))[0]))
            seed = int(seeds[r]) if seeds is not None else 0
            draw = int(draws[r]) if draws is not None else 0
            y = x + gumbel_noise(seed, draw, V)
            y = torch.where(keys >= cut, y, torch.full_like(y, float("-inf")))
            out[r] = int(torch.argmax(y))
        return out

    def apply_penalties(self, logits, tokens, offsets, prompt_lens, presence, frequency, repetition):
        R, V = logits.shape
        for r in range(R):
            b, e, np_ = int(offsets[r]), int(offsets[r + 1]), int(prompt_lens[r])
            toks = tokens[b:e].long()
            seen = torch.zeros(V, dtype=torch.bool, device=logits.device)
            seen[toks] = True
            counts = torch.zeros(V, dtype=torch.float32, device=logits.device)
            counts.index_add_(0, toks[np_:], torch.ones(e - b - np_, device=logits.device))
            x = logits[r]
            rep = torch.where(seen, repetition[r], torch.ones_like(x))
            x = torch.where(x > 0, x / rep, x * rep)
            x = x - frequency[r] * counts
            x = x - presence[r] * (counts > 0).to(torch.float32)
            logits[r] = x
