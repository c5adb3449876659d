"""A stand-in for the kernels that runs on the CPU with torch, for tests of the engine's logic
(cache, batching, schedule, generation) on a machine without a GPU.  It is a test double with the
same method signatures as ``libllm_amd.hip.ops.HipOps``; the library itself never uses it.
"""
import numpy as np
import torch

from libllm_amd.parts import kv_pages as layout


class CpuOps:
    supports_graphs = False

    def __init__(self):
        self.device = torch.device("cpu")
        self.calls = []

    def upload_int32(self, arr):
        return torch.from_numpy(np.ascontiguousarray(arr, dtype=np.int32)).clone()

    def embed(self, table, ids, scale=1.0):
        return table[ids.long()].float() * scale

    def add_rmsnorm(self, res, delta, weight, eps, out_dtype, rows=None):
        if delta is not None:
            for part in (delta if delta.dim() == 3 else [delta]):      # a stack is added in its order
                res += part.float()
        x = res if rows is None else res[rows.long()]
        inv = torch.rsqrt((x * x).mean(dim=-1, keepdim=True) + eps)
        return (x * weight * inv).to(out_dtype)

    def linear(self, x, w, bias, out_dtype, residual=None):
        y = x.float() @ w.float().t()
        if bias is not None:
            y = y + bias
        if x.dtype == torch.bfloat16 and out_dtype == torch.bfloat16:
            return y.to(torch.bfloat16)
        return y.to(out_dtype)

    def linear_swiglu(self, x, w, dtype=None, activation="silu"):
        return self.silu_mul(self.linear(x, w, None, x.dtype), activation)

    def silu_mul(self, gu, activation="silu"):
        i = gu.shape[1] // 2
        g, u = gu[:, :i].float(), gu[:, i:].float()
        act = {"silu": lambda t: t / (1.0 + torch.exp(-t)), "relu": torch.relu,
               "gelu_tanh": lambda t: torch.nn.functional.gelu(t, approximate="tanh")}[activation]
        return (u * act(g)).to(gu.dtype)

    def rope_kv_write(self, qkv, bias, n_heads, n_kv, hd, cos, sin, rot_dim, ctx, kv, write):
        m = qkv.shape[0]
        n_rot = n_heads + (n_kv if write else 0)
        x = qkv.float()
        if bias is not None:
            x = x + bias[:x.shape[1]]
        heads = x[:, :n_rot * hd].reshape(m, n_rot, hd).clone()
        if rot_dim:
            pos = ctx.tok_pos.long()
            c, s = cos[pos][:, None, :], sin[pos][:, None, :]
            h2 = rot_dim // 2
            x1, x2 = heads[..., :h2].clone(), heads[..., h2:rot_dim].clone()
            heads[..., :h2] = x1 * c - x2 * s
            heads[..., h2:rot_dim] = x2 * c + x1 * s
        qkv[:, :n_heads * hd] = heads[:, :n_heads].reshape(m, -1).to(qkv.dtype)
        if write:
            k = heads[:, n_heads:]
            v = x[:, (n_heads + n_kv) * hd:(n_heads + 2 * n_kv) * hd].reshape(m, n_kv, hd)
            slots = ctx.seq_slot.long()[ctx.tok_seq.long()]
            pos = ctx.tok_pos.long()
            pages = kv.block_table.long()[slots, pos // kv.page_size]
            layout.write_keys(kv.plane("k"), pages, pos % kv.page_size, k.to(kv.plane("k").dtype))
            layout.write_values(kv.plane("v"), pages, pos % kv.page_size, v.to(kv.plane("v").dtype))

    def attention(self, qkv, n_heads, n_kv, hd, ctx, kv, scale, window):
        m = qkv.shape[0]
        out = torch.empty((m, n_heads * hd), dtype=qkv.dtype)
        group = n_heads // n_kv
        page = kv.page_size
        for t in range(m):
            pos = int(ctx.tok_pos[t])
            slot = int(ctx.seq_slot[int(ctx.tok_seq[t])])
            first = max(0, pos - window + 1) if window else 0
            keys = torch.arange(first, pos + 1)
            pages = kv.block_table[slot].long()[keys // page]
            k = layout.read_keys(kv.plane("k"), pages, keys % page, hd).float()       # [L, n_kv, hd]
            v = layout.read_values(kv.plane("v"), pages, keys % page).float()
            q = qkv[t, :n_heads * hd].float().reshape(n_heads, hd)
            k = k.repeat_interleave(group, dim=1)
            v = v.repeat_interleave(group, dim=1)
            s = torch.einsum("hd,lhd->hl", q, k) * scale
            p = torch.softmax(s, dim=-1)
            out[t] = torch.einsum("hl,lhd->hd", p, v).reshape(-1).to(qkv.dtype)
        return out

    def argmax(self, logits):
        return torch.argmax(logits, dim=-1).to(torch.int32)

    def sample(self, logits, temperature, top_k, top_p, seed, streams, counters):
        from plain import sampling
        out = []
        for r in range(logits.shape[0]):
            u = sampling.uniform(seed, streams[r], counters[r])
            out.append(sampling.sample(logits[r].double().numpy(), temperature, top_k, top_p, u))
        return torch.tensor(out, dtype=torch.int32)
