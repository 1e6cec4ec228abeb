"""Plain torch twins of the device kernels, one per kernel, with the kernels' signatures.

Two uses, both in tests only:

* on the GPU, each HIP kernel is compared alone with its twin;
* on the CPU, where the HIP kernels cannot run, a ``TwinKernels`` object is handed to
  the engine in place of the kernel library, so that the cache manager, the step
  function, the scheduler and trace replay can be tested without a GPU.

The engine itself has no such path: without its compiled kernels it refuses to start.
"""

from __future__ import annotations

import torch


class TwinKernels:
    name = "torch-twins"

    # -- embedding ---------------------------------------------------------
    def place_tokens(self, token_ids, dst_rows, src_tokens, src_rows):
        token_ids[dst_rows.long()] = src_tokens[src_rows.long()]

    def embed(self, token_ids, table):
        return table[token_ids.long()].float()

    # -- residual add + rms norm ---------------------------------------------
    def add_rmsnorm(self, residual, delta, weight, eps, out_dtype, rows=None):
        if rows is None:
            if delta is not None:
                residual.add_(delta.float())
            x = residual
        else:
            x = residual[rows.long()]
            if delta is not None:
                x = x + delta[rows.long()].float()
        var = x.pow(2).mean(-1, keepdim=True)
        return (x * torch.rsqrt(var + eps) * weight.float()).to(out_dtype)

    # -- matrix product ------------------------------------------------------
    def linear(self, x, w, out_float32=False):
        y = x.float() @ w.float().T
        return y if out_float32 else y.to(x.dtype)

    pending_linear = linear   # computed at once: the twin's norm always has a kernel of its own

    def gated_linear(self, x, w_gate_up):
        return self.swiglu(self.linear(x, w_gate_up))

    # -- feed-forward activation --------------------------------------------
    def swiglu(self, gu):
        inter = gu.shape[-1] // 2
        g, u = gu[:, :inter].float(), gu[:, inter:].float()
        return (g * torch.sigmoid(g) * u).to(gu.dtype)

    def qkv_to_cache(self, x, w_qkv, n_heads, n_kv_written, head_dim, rotary_dim, cos, sin, ctx, cache):
        qkv = self.linear(x, w_qkv)
        self.rope_kv_write(qkv, n_heads, n_kv_written, head_dim, rotary_dim, cos, sin, ctx, cache)
        return qkv

    # -- rotation + cache write ----------------------------------------------
    def rope_kv_write(self, qkv, n_heads, n_kv_written, head_dim, rotary_dim, cos, sin, ctx, cache):
        N = qkv.shape[0]
        pos = ctx.positions.long()
        q = qkv[:, :n_heads * head_dim].view(N, n_heads, head_dim)

        def rotate(x):
            if rotary_dim == 0:
                return x
            half = rotary_dim // 2
            c = cos[pos][:, None, :]
            s = sin[pos][:, None, :]
            xf = x.float()
            a, b = xf[..., :half], xf[..., half:rotary_dim]
            out = xf.clone()
            out[..., :half] = a * c - b * s
            out[..., half:rotary_dim] = b * c + a * s
            return out.to(x.dtype)

        q.copy_(rotate(q))
        if n_kv_written == 0:
            return
        kv0 = n_heads * head_dim
        k = qkv[:, kv0:kv0 + n_kv_written * head_dim].view(N, n_kv_written, head_dim)
        v = qkv[:, kv0 + n_kv_written * head_dim:kv0 + 2 * n_kv_written * head_dim].view(N, n_kv_written, head_dim)
        k = rotate(k)
        ps = cache.page_size
        seq = ctx.seq_of_token.long()
        page = cache.block_table.long()[seq, pos // ps]
        off = pos % ps
        cache.k_pages[page, :, off, :] = k
        cache.v_pages[page, :, :, off] = v

    # -- attention over the pages --------------------------------------------
    def paged_attention(self, qkv, n_heads, n_kv_heads, head_dim, scale, window, ctx, cache):
        N = qkv.shape[0]
        q = qkv[:, :n_heads * head_dim].view(N, n_heads, head_dim).float()
        out = torch.zeros(N, n_heads, head_dim, dtype=torch.float32, device=qkv.device)
        ps = cache.page_size
        group = n_heads // n_kv_heads
        cu = ctx.cu_q.tolist()
        kv_len = ctx.kv_len.tolist()
        table = cache.block_table.long()
        for s in range(ctx.n_seqs):
            L = kv_len[s]
            lo = 0
            first = kv_len[s] - (cu[s + 1] - cu[s])
            if window is not None:
                lo = max(0, first - window + 1)
            idx = torch.arange(lo, L, device=qkv.device)
            pages = table[s, idx // ps]
            k = cache.k_pages[pages, :, idx % ps, :].float()          # [T, Hkv, D]
            v = cache.v_pages[pages, :, :, idx % ps].float()          # [T, Hkv, D]
            qs = q[cu[s]:cu[s + 1]]
            qpos = torch.arange(first, L, device=qkv.device)
            visible = idx[None, :] <= qpos[:, None]
            if window is not None:
                visible &= idx[None, :] > qpos[:, None] - window
            for h in range(n_heads):
                sc = (qs[:, h] @ k[:, h // group].T) * scale
                sc = sc.masked_fill(~visible, float("-inf"))
                out[cu[s]:cu[s + 1], h] = torch.softmax(sc, -1) @ v[:, h // group]
        return out.view(N, n_heads * head_dim).to(qkv.dtype)

    # -- sampling --------------------------------------------------------------
    def sample(self, logits, temperature, top_k, top_p, uniform, all_greedy=False, filters=None):
        if all_greedy:
            return torch.argmax(logits.double(), dim=-1).to(torch.int32)
        out = []
        for r in range(logits.shape[0]):
            row = logits[r].double()
            t = float(temperature[r])
            if t == 0.0:
                out.append(int(torch.argmax(row)))
                continue
            row = row / t
            k = int(top_k[r])
            V = row.shape[0]
            if 0 < k < V:
                kth = torch.sort(row, descending=True).values[k - 1]
                row = torch.where(row < kth, torch.full_like(row, float("-inf")), row)
            p = float(top_p[r])
            if p < 1.0:
                srt, idx = torch.sort(row, descending=True)
                cum = torch.softmax(srt, -1).cumsum(-1)
                rem = torch.zeros_like(cum, dtype=torch.bool)
                if p > 0.0:
                    rem[1:] = cum[:-1] > p
                else:
                    rem[1:] = True
                row = row.masked_fill(torch.zeros_like(rem).scatter(0, idx, rem), float("-inf"))
            cdf = torch.softmax(row, -1).cumsum(-1)
            out.append(min(int((cdf <= float(uniform[r]) * cdf[-1]).sum()), V - 1))
        return torch.tensor(out, dtype=torch.int32, device=logits.device)
