"""The kernel set in plain PyTorch, for tests only.

Two uses: the per-kernel reference that each HIP kernel is compared with on the
GPU, and a stand-in kernel set that lets the step function, the cache and the
scheduler run on a CPU in the ``not gpu`` tests. Nothing in ``socrates_amd``
imports this file. Statistics, softmax, angles and sums are float32 (float64 if
the set is built with it) and results are rounded once to the compute dtype, as
the HIP kernels do.
"""

import numpy as np
import torch


def splitmix64(x: int) -> int:
    """One step of the splitmix64 generator: a counter-based hash on 64 bits."""
    m = (1 << 64) - 1
    x = (x + 0x9E3779B97F4A7C15) & m
    x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & m
    x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & m
    return x ^ (x >> 31)


def uniform_of(seed: int, draw: int) -> float:
    """The uniform number in [0, 1) that request stream ``seed`` yields at draw ``draw``."""
    h = splitmix64(splitmix64(int(seed)) ^ ((int(draw) * 0xD1342543DE82EF95) & ((1 << 64) - 1)))
    return (h >> 40) * (1.0 / (1 << 24))


class TorchKernels:
    def __init__(self, dtype=torch.float32, device="cpu", acc=torch.float32):
        self.dtype, self.device, self.acc = dtype, torch.device(device), acc

    # -- elementwise and norms ---------------------------------------------------------------
    def embedding(self, ids, table):
        return table[ids.long()].to(torch.float32 if self.acc == torch.float32 else self.acc)

    def _norm(self, x, weight, eps):
        x = x.to(self.acc)
        var = x.pow(2).mean(-1, keepdim=True)
        return x / torch.sqrt(var + eps) * weight.to(self.acc)

    def add_rmsnorm(self, residual, delta, weight, eps, rows=None):
        if delta is not None and delta.dim() == 3:            # split-K partial sums
            delta = delta.sum(0)
        if rows is not None:
            r = residual[rows.long()].to(self.acc)
            if delta is not None:
                r = r + delta[rows.long()].to(self.acc)
            return self._norm(r, weight, eps).to(self.dtype)
        if delta is not None:
            residual += delta.to(residual.dtype)
        return self._norm(residual, weight, eps).to(self.dtype)

    def rmsnorm(self, x, weight, eps):
        return self._norm(x, weight, eps).to(x.dtype)

    def scale_softcap_(self, x, scale=1.0, softcap=None):
        x.mul_(scale)
        if softcap is not None:
            x.copy_(softcap * torch.tanh(x / softcap))
        return x

    def swiglu(self, gate_up, interleave=0):
        ff = gate_up.shape[-1] // 2
        if interleave:
            blocks = gate_up.reshape(*gate_up.shape[:-1], ff // interleave, 2, interleave)
            g, u = blocks[..., 0, :].reshape(*gate_up.shape[:-1], ff), blocks[..., 1, :].reshape(*gate_up.shape[:-1], ff)
        else:
            g, u = gate_up[..., :ff], gate_up[..., ff:]
        g, u = g.to(self.acc), u.to(self.acc)
        return (u * (g * torch.sigmoid(g))).to(self.dtype)

    def linear_swiglu(self, x, w_gate_up, interleave=0):
        return self.swiglu(self.linear(x, w_gate_up), interleave)

    def linear(self, x, w, out_dtype=None, allow_partial=False):
        y = x.to(self.acc) @ w.to(self.acc).T
        return y.to(out_dtype or self.dtype)

    # -- attention pieces --------------------------------------------------------------------
    def _rotate(self, x, positions, inv_freq, rotary_dim):
        """x: [N, H, D] in acc dtype."""
        ang = positions.to(torch.float32)[:, None] * inv_freq.to(torch.float32)[None, :]
        cos, sin = ang.cos().to(self.acc)[:, None, :], ang.sin().to(self.acc)[:, None, :]
        h = rotary_dim // 2
        x1, x2 = x[..., :h], x[..., h:rotary_dim]
        out = x.clone()
        out[..., :h] = x1 * cos - x2 * sin
        out[..., h:rotary_dim] = x2 * cos + x1 * sin
        return out

    def qk_norm_split(self, qkv, Hq, Hkv, D, q_gain, k_gain, eps):
        N = qkv.shape[0]
        q = qkv[:, :Hq * D].reshape(N, Hq, D)
        k = qkv[:, Hq * D:(Hq + Hkv) * D].reshape(N, Hkv, D)
        v = qkv[:, (Hq + Hkv) * D:(Hq + 2 * Hkv) * D].reshape(N, Hkv, D).contiguous()
        if q_gain is not None:
            q = self._norm(q, q_gain, eps).to(self.dtype)
            k = self._norm(k, k_gain, eps).to(self.dtype)
        return q.contiguous(), k.contiguous(), v

    def rope(self, x, positions, inv_freq, rotary_dim):
        x.copy_(self._rotate(x.to(self.acc), positions, inv_freq, rotary_dim).to(x.dtype))

    def kv_write(self, k, v, positions, token_rows, slot):
        bs = slot.block_size
        pos = positions.long()
        page = slot.block_table[token_rows.long(), pos // bs].long()
        slot.k[page, :, pos % bs] = k.to(slot.k.dtype)
        slot.v[page, :, pos % bs] = v.to(slot.v.dtype)

    def qk_norm_rope_write(self, qkv, Hq, Hkv, D, q_gain, k_gain, eps, inv_freq, rotary_dim,
                           positions, token_rows, slot):
        N = qkv.shape[0]
        q = qkv[:, :Hq * D].reshape(N, Hq, D).to(self.acc)
        k = qkv[:, Hq * D:(Hq + Hkv) * D].reshape(N, Hkv, D).to(self.acc)
        v = qkv[:, (Hq + Hkv) * D:(Hq + 2 * Hkv) * D].reshape(N, Hkv, D)
        if q_gain is not None:
            q, k = self._norm(q, q_gain, eps), self._norm(k, k_gain, eps)
        if inv_freq is not None:
            q = self._rotate(q, positions, inv_freq, rotary_dim)
            k = self._rotate(k, positions, inv_freq, rotary_dim)
        if slot is not None:
            self.kv_write(k, v, positions, token_rows, slot)
        return q.to(self.dtype).contiguous()

    def paged_attention(self, q, slot, ctx, scale, window, terms=None):
        """Token by token: gather the row's keys 0..p through the table, mask the window.
        ``terms``: a bias by distance (``slopes`` [Hq]), a soft cap of the scores, one more
        logit per head in the softmax's sum (``sinks`` [Hq])."""
        terms = terms or {}
        N, Hq, D = q.shape
        Hkv, bs = slot.k.shape[1], slot.block_size
        G = Hq // Hkv
        out = torch.empty((N, Hq * D), dtype=self.dtype, device=q.device)
        table = slot.block_table.cpu().numpy()
        positions = ctx.positions.cpu().numpy()
        rows = ctx.token_rows.cpu().numpy()
        for t in range(N):
            p, row = int(positions[t]), int(rows[t])
            lo = 0 if window is None else max(0, p - window + 1)
            idx = np.arange(lo, p + 1)
            pages = torch.as_tensor(table[row, idx // bs].astype(np.int64), device=q.device)
            offs = torch.as_tensor(idx % bs, device=q.device)
            k = slot.k[pages, :, offs].to(self.acc)          # [n, Hkv, D]
            v = slot.v[pages, :, offs].to(self.acc)
            qt = q[t].to(self.acc).view(Hkv, G, D)
            s = torch.einsum("hgd,nhd->hgn", qt, k) * scale
            if terms.get("slopes") is not None:
                dist = torch.as_tensor(idx - p, device=q.device).to(self.acc)
                s = s + terms["slopes"].to(self.acc).view(Hkv, G, 1) * dist
            if terms.get("softcap"):
                s = terms["softcap"] * torch.tanh(s / terms["softcap"])
            if terms.get("sinks") is not None:
                s = torch.cat([s, terms["sinks"].to(self.acc).view(Hkv, G, 1)], dim=-1)
                a = torch.softmax(s, dim=-1)[..., :-1]
            else:
                a = torch.softmax(s, dim=-1)
            out[t] = torch.einsum("hgn,nhd->hgd", a, v).reshape(Hq * D).to(self.dtype)
        return out

    # -- sampling ----------------------------------------------------------------------------
    def argmax(self, logits):
        return logits.argmax(dim=-1).to(torch.int32)

    def sample(self, logits, temperature, seed, draws):
        """Greedy where temperature is 0; else the inverse-CDF draw of softmax(logits / T)
        at the uniform number of (seed, draw)."""
        out = []
        for i in range(logits.shape[0]):
            T = float(temperature[i])
            if T <= 0.0:
                out.append(int(logits[i].argmax()))
                continue
            u = uniform_of(int(seed[i]), int(draws[i]))
            p = torch.softmax(logits[i].double() / T, dim=-1)
            cdf = torch.cumsum(p, dim=-1)
            tok = int(torch.searchsorted(cdf, torch.tensor(u * float(cdf[-1]), dtype=cdf.dtype, device=cdf.device), right=True))
            out.append(min(tok, logits.shape[1] - 1))
        return torch.tensor(out, dtype=torch.int32, device=logits.device)
