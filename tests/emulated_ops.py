"""A host stand-in for the kernel library, for tests only.

It implements the kernel library's Python interface (``prefixserve_amd.kernels.ops.HipOps``)
with plain torch on the CPU, reading and writing the same buffers in the same layouts, so
that everything on the host side of a step (batch packing, block tables, page reuse, the
scheduler, replay) can be tested without a GPU. The package itself never uses it: without
the compiled kernels and a GPU the engine raises.
"""

from __future__ import annotations

import contextlib

import torch

PAGE = 16


class EmulatedOps:
    PREFILL_TILE_Q = 64
    name = "emulated"

    def __init__(self, device: torch.device | str = "cpu", workspace=None) -> None:
        self.device = torch.device(device)
        self.ws = workspace

    def step_scope(self):
        return contextlib.nullcontext()

    def prepare_matrix(self, w: torch.Tensor, rt) -> torch.Tensor:
        return w.to(device=rt.device, dtype=rt.dtype).contiguous()

    def embed(self, ids, table, out) -> None:
        out.copy_(table[ids.long()].float())

    def add_rmsnorm(self, residual, delta, weight, eps, out) -> None:
        if delta is not None:
            residual.add_(delta.float())
        x = residual
        out.copy_((weight.float() * x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps)).to(out.dtype))

    def add_rmsnorm_rows(self, residual, delta, rows, weight, eps, out) -> None:
        x = residual[rows.long()]
        if delta is not None:
            x = x + delta[rows.long()].float()
        out.copy_((weight.float() * x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps)).to(out.dtype))

    def linear(self, x, w, out) -> None:
        out.copy_((x.float() @ w.float().T).to(out.dtype))

    def linear_to_residual(self, x, w, name, residual=None):
        out = self.ws.get(name, (x.shape[0], w.shape[0]), x.dtype)
        self.linear(x, w, out)
        return out

    def linear_swiglu(self, x, w_gate_up, out) -> None:
        gu = x.float() @ w_gate_up.float().T
        inter = gu.shape[1] // 2
        out.copy_((torch.nn.functional.silu(gu[:, :inter]) * gu[:, inter:]).to(out.dtype))

    def qkv_rope_append(self, x, w_qkv, qkv, hq, hkv, d, positions, table, kv, write_slot) -> None:
        self.linear(x, w_qkv, qkv)
        self.rope_kv_append(qkv, hq, hkv, d, positions, table, kv, write_slot)

    def rope_kv_append(self, qkv, hq, hkv, d, positions, table, kv, write_slot) -> None:
        t = qkv.shape[0]
        q = qkv[:, : hq * d].view(t, hq, d)
        k = qkv[:, hq * d: (hq + hkv) * d].view(t, hkv, d)
        v = qkv[:, (hq + hkv) * d:].view(t, hkv, d)
        if table is not None:
            cs = table[positions.long()]  # [t, d/2, 2]
            cos, sin = cs[..., 0][:, None, :], cs[..., 1][:, None, :]
            for x in (q, k):
                x1, x2 = x[..., : d // 2].float().clone(), x[..., d // 2:].float().clone()
                x[..., : d // 2] = (x1 * cos - x2 * sin).to(x.dtype)
                x[..., d // 2:] = (x2 * cos + x1 * sin).to(x.dtype)
        if kv is not None:
            page = (write_slot // PAGE).long()
            off = (write_slot % PAGE).long()
            kpages = kv[:, 0].view(kv.shape[0], hkv, PAGE, d)
            vpages = kv[:, 1].view(kv.shape[0], hkv, d, PAGE)
            kpages[page, :, off, :] = k
            vpages[page, :, :, off] = v

    def expand_kv(self, x, rep):
        """[keys, kv_heads, d] -> [keys, heads, d]: query head h reads kv head h // rep."""
        return x.repeat_interleave(rep, dim=1)

    def paged_attention(self, qkv, out, kv, ctx, group, hq, hkv, d, scale, window) -> None:
        g = ctx.groups[group]
        t = qkv.shape[0]
        q = qkv[:, : hq * d].view(t, hq, d).float()
        o = out.view(t, hq, d)
        rep = hq // hkv
        starts = ctx.item_start.tolist()
        offs = g.table_off.tolist()
        for i in range(ctx.num_items):
            t0, t1 = starts[i], starts[i + 1]
            pos0, end = int(ctx.item_pos0[i]), int(ctx.item_end[i])
            pages = g.block_ids[offs[i]: offs[i] + -(-end // PAGE)].long()
            keys = kv[pages, 0].view(-1, hkv, PAGE, d).permute(0, 2, 1, 3).reshape(-1, hkv, d)[:end].float()
            vals = kv[pages, 1].view(-1, hkv, d, PAGE).permute(0, 3, 1, 2).reshape(-1, hkv, d)[:end].float()
            keys = self.expand_kv(keys, rep)
            vals = self.expand_kv(vals, rep)
            qi = q[t0:t1].transpose(0, 1)                                  # [hq, n, d]
            scores = torch.matmul(qi, keys.permute(1, 2, 0)) * scale        # [hq, n, end]
            qpos = torch.arange(pos0, end)[:, None]
            kpos = torch.arange(end)[None, :]
            hidden = kpos > qpos
            if window is not None:
                hidden = hidden | (qpos - kpos >= window)
            scores = scores.masked_fill(hidden, float("-inf"))
            probs = torch.softmax(scores, dim=-1)
            o[t0:t1] = torch.matmul(probs, vals.transpose(0, 1)).transpose(0, 1).to(out.dtype)

    def argmax(self, logits, out) -> None:
        out.copy_(torch.argmax(logits, dim=-1).to(out.dtype))

    def sample(self, logits, temperatures, uniforms, out) -> None:
        for i in range(logits.shape[0]):
            temp = float(temperatures[i])
            if temp <= 0.0:
                out[i] = int(torch.argmax(logits[i]))
                continue
            z = logits[i].double() / temp
            p = torch.exp(z - z.max())
            c = torch.cumsum(p, 0)
            idx = int(torch.searchsorted(c, float(uniforms[i]) * float(c[-1]), right=True))
            out[i] = min(idx, logits.shape[1] - 1)
