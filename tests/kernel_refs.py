"""Plain torch versions of every kernel op, with the signatures of `tokenizer_amd.kernels.Ops`.

They serve two purposes: the GPU tests compare each HIP kernel with its function here, and the
CPU tests hand an instance to the engine in place of the kernel library so that the host-side
orchestration (tables, slots, scheduling) can be checked without a GPU.  This is a test double,
not a product path: the package itself has no CPU fallback.
"""
from __future__ import annotations

import torch


class PlainOps:
    """Every op computes in float32 (float64 if asked) and rounds to the output's dtype at the end."""

    def __init__(self, work=torch.float32):
        self.work = work

    def embedding(self, ids, table, out):
        out.copy_(table[ids.long()].to(torch.float32))
        return out

    def add_rmsnorm(self, residual, delta, weight, eps, out, rows=None, store_residual=True):
        x = residual if rows is None else residual[rows.long()]
        x = x.to(self.work)
        if delta is not None:
            d = delta if rows is None else delta[rows.long()]
            x = x + d.to(self.work)
        if store_residual:
            assert rows is None
            residual.copy_(x.to(torch.float32))
            x = residual.to(self.work)
        y = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * weight.to(self.work)
        out.copy_(y.to(out.dtype))
        return out

    def silu_gate(self, gate_up, out):
        inner = gate_up.shape[1] // 2
        g, u = gate_up[:, :inner].to(self.work), gate_up[:, inner:].to(self.work)
        out.copy_((g * torch.sigmoid(g) * u).to(out.dtype))
        return out

    def rope_store(self, qkv, bias, positions, cos_sin, slots, k_pages, v_pages, n_q, n_kv, head_dim):
        n_tokens = qkv.shape[0]
        x = qkv.to(self.work)
        if bias is not None:
            x = x + bias.to(self.work)
        x = x.reshape(n_tokens, n_q + 2 * n_kv, head_dim).clone()
        if cos_sin is not None:
            half = head_dim // 2
            cs = cos_sin[positions.long()].to(self.work)
            cos, sin = cs[:, None, :half], cs[:, None, half:]
            rot = x[:, :n_q + n_kv]
            x1, x2 = rot[..., :half], rot[..., half:]
            x[:, :n_q + n_kv] = torch.cat([x1 * cos - x2 * sin, x2 * cos + x1 * sin], dim=-1)
        qkv.copy_(x.reshape(n_tokens, -1).to(qkv.dtype))
        if slots is not None:
            page_size = k_pages.shape[2]
            stored = qkv.reshape(n_tokens, n_q + 2 * n_kv, head_dim)
            for t in range(n_tokens):
                slot = int(slots[t])
                if slot < 0:
                    continue
                page, off = divmod(slot, page_size)
                k_pages[page, :, off, :] = stored[t, n_q:n_q + n_kv]
                v_pages[page, :, :, off] = stored[t, n_q + n_kv:]       # values lie transposed in a page

    def paged_attention(self, qkv, out, k_pages, v_pages, positions, entry_of_token, block_table,
                        n_q, n_kv, head_dim, window, scale, max_position=None, batch=None):
        page_size = k_pages.shape[2]
        group = n_q // n_kv
        for t in range(qkv.shape[0]):
            if int(entry_of_token[t]) < 0:                   # a token that only fills the batch up
                continue
            pos = int(positions[t])
            table = block_table[int(entry_of_token[t])]
            lo = max(0, pos - window) if window is not None else 0
            keys = list(range(lo, pos + 1))
            pages = [int(table[j // page_size]) for j in keys]
            assert all(p >= 0 for p in pages), "attention reads a page that was given back"
            offs = [j % page_size for j in keys]
            k = k_pages[pages, :, offs, :].to(self.work)     # [keys, n_kv, d]
            v = v_pages[pages, :, :, offs].to(self.work)      # [keys, n_kv, d]
            q = qkv[t, :n_q * head_dim].reshape(n_q, head_dim).to(self.work)
            k = k.repeat_interleave(group, dim=1)            # [keys, n_q, d]
            v = v.repeat_interleave(group, dim=1)
            scores = torch.einsum("hd,khd->hk", q, k) * scale
            probs = torch.softmax(scores, dim=-1)
            out[t] = torch.einsum("hk,khd->hd", probs, v).reshape(-1).to(out.dtype)
        return out

    def linear(self, x, weight, bias=None, out=None, out_dtype=None):
        y = x.to(self.work) @ weight.to(self.work).t()
        if bias is not None:
            y = y + bias.to(self.work)
        if out_dtype is None:
            out_dtype = x.dtype if out is None else out.dtype
        y = y.to(out_dtype)
        if out is not None:
            out.copy_(y)
            return out
        return y

    def linear_silu_gate(self, x, weight, out=None):
        inner = weight.shape[0] // 2
        result = torch.empty((x.shape[0], inner), dtype=x.dtype, device=x.device) if out is None else out
        return self.silu_gate(self.linear(x, weight), result)

    # The fused decode products, as compositions of the ops above.
    fuse_rows = 16

    def can_fuse_decode(self, rows, dtype, hidden=0):
        return 0 < rows <= self.fuse_rows

    def can_rope_store(self, rows, dtype, weight_elements=0):
        return self.fuse_rows < rows <= 64

    def fold_norm(self, hidden):
        return hidden <= 80          # so that the CPU tests of the engine take both routes

    def fused_norm_qkv_rope(self, residual, norm_weight, eps, weight, bias, positions, cos_sin, slots,
                            k_pages, v_pages, n_q, n_kv, head_dim):
        if norm_weight is None:                                  # the rows are normalised already
            x = residual
        else:
            x = torch.empty(residual.shape, dtype=weight.dtype, device=residual.device)
            self.add_rmsnorm(residual.clone(), None, norm_weight, eps, x)
        qkv = (x.to(self.work) @ weight.to(self.work).t())
        if bias is not None:
            qkv = qkv + bias.to(self.work)
        # The fused kernel rotates the float accumulators and rounds once.
        holder = qkv.to(self.work).clone()
        work_k = None if slots is None else k_pages.to(self.work)
        work_v = None if slots is None else v_pages.to(self.work)
        PlainOps(self.work).rope_store(holder, None, positions, cos_sin, slots, work_k, work_v, n_q, n_kv, head_dim)
        if slots is not None:
            k_pages.copy_(work_k.to(k_pages.dtype))
            v_pages.copy_(work_v.to(v_pages.dtype))
        return holder[:, :n_q * head_dim].to(weight.dtype).contiguous()

    def fused_norm_gated(self, residual, norm_weight, eps, weight):
        if norm_weight is None:
            x = residual
        else:
            x = torch.empty(residual.shape, dtype=weight.dtype, device=residual.device)
            self.add_rmsnorm(residual.clone(), None, norm_weight, eps, x)
        gate_up = x.to(self.work) @ weight.to(self.work).t()
        inner = weight.shape[0] // 2
        g, u = gate_up[:, :inner], gate_up[:, inner:]
        return (g * torch.sigmoid(g) * u).to(weight.dtype)

    def linear_add(self, x, weight, bias, residual):
        y = x.to(self.work) @ weight.to(self.work).t()
        if bias is not None:
            y = y + bias.to(self.work)
        residual.add_(y.to(torch.float32))

    def sample(self, logits, temperature, top_p, uniform, out=None, any_cut=True):
        from plain import qwen2_plain as plain
        result = torch.empty(logits.shape[0], dtype=torch.int32, device=logits.device) if out is None else out
        for row in range(logits.shape[0]):
            result[row] = plain.sample_token(logits[row].float().cpu().numpy(), float(temperature[row]),
                                             float(top_p[row]), float(uniform[row]))
        return result

    def argmax(self, logits, out=None):
        result = torch.empty(logits.shape[0], dtype=torch.int32, device=logits.device) if out is None else out
        for row in range(logits.shape[0]):
            values = logits[row]
            best = values.max()
            hit = torch.nonzero(values == best)
            result[row] = int(hit[0]) if hit.numel() else 0
        return result
