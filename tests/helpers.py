"""Shared helpers of the GPU tests: step contexts and paged caches built by hand, error metrics."""
import numpy as np
import torch

from libllm_amd.parts import CacheNeed, KVView, StepContext

PAGE = 64

# Bounds on max|out - ref| / mean|ref| (the reference's metric, src/libllm/llama_test.cc:109-130).
# float32: only the order of additions differs from the float64 oracle.
TOL_F32 = 1e-4
# bfloat16 keeps 8 bits of mantissa where the reference's half keeps 11, so its own bound for half
# (0.02, src/libllm/llama_test.cc:49) scales by 2^3.
TOL_BF16 = 0.16
# Per position, the relative L2 error of the logits row.  A bfloat16 rounding is 2^-9 relative and
# a logit has passed some tens of them, so a row is off by about one percent; a lost key, a wrong
# page or a position off by one moves the affected rows by far more.
ROW_F32 = 2e-5
ROW_BF16 = 0.05


def rel_err(out, ref):
    out = np.asarray(out, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    return float(np.abs(out - ref).max() / max(np.abs(ref).mean(), 1e-30))


def row_err(out, ref):
    """Largest relative L2 error of a row."""
    out = np.asarray(out, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    return float((np.linalg.norm(out - ref, axis=-1) / np.maximum(np.linalg.norm(ref, axis=-1), 1e-30)).max())


def tol_for(dtype):
    return TOL_F32 if dtype in ("float32", torch.float32) else TOL_BF16


def row_tol_for(dtype):
    return ROW_F32 if dtype in ("float32", torch.float32) else ROW_BF16


def assert_logits_close(out, ref, dtype, what=""):
    e, r = rel_err(out, ref), row_err(out, ref)
    assert e < tol_for(dtype) and r < row_tol_for(dtype), "%s: max error %.3g, row error %.3g" % (what, e, r)
    return e, r


def make_ctx(ops, dtype, seqs):
    """seqs: list of (slot, pos0, n_new).  Tokens are zeros; parts under test do not read them."""
    b = len(seqs)
    lens = [n for _, _, n in seqs]
    m = sum(lens)
    starts = np.zeros(b + 1, dtype=np.int64)
    starts[1:] = np.cumsum(lens)
    tok_seq = np.repeat(np.arange(b), lens)
    pos0 = np.array([p for _, p, _ in seqs])
    tok_pos = np.arange(m) - starts[tok_seq] + pos0[tok_seq]
    ctx = StepContext(ops, dtype, m, b)
    ctx.tokens = ops.upload_int32(np.zeros(m))
    ctx.tok_pos = ops.upload_int32(tok_pos)
    ctx.tok_seq = ops.upload_int32(tok_seq)
    ctx.seq_start = ops.upload_int32(starts)
    ctx.seq_slot = ops.upload_int32(np.array([s for s, _, _ in seqs]))
    ctx.seq_pos0 = ops.upload_int32(pos0)
    ctx.seq_lens = lens
    ctx.seq_pos0_host = list(pos0)
    ctx.seq_slot_host = [s for s, _, _ in seqs]
    ctx.max_new = max(lens)
    ctx.max_ctx = int(max(p + n for _, p, n in seqs))
    ctx.decode = all(n == 1 for n in lens)
    return ctx


def make_kv(device, dtype, n_slots, pages_per_seq, n_kv, hd, seed=0, window=0):
    """A cache entry whose page table is a random permutation, so that a kernel that ignores the
    table reads the wrong page."""
    g = torch.Generator().manual_seed(seed)
    n_pages = n_slots * pages_per_seq
    perm = torch.randperm(n_pages, generator=g).reshape(n_slots, pages_per_seq).to(torch.int32)
    k = torch.zeros((n_pages + 1, n_kv, PAGE, hd), dtype=dtype, device=device)
    v = torch.zeros((n_pages + 1, n_kv, hd, PAGE), dtype=dtype, device=device)
    need = CacheNeed("window" if window else "full", n_kv, hd, window)
    return KVView(k, v, perm.to(device), PAGE, need)


def fill_kv(kv, slot, keys, values):
    """keys, values: [L, n_kv, hd] (any float dtype) written at positions 0..L-1 of the slot."""
    length = keys.shape[0]
    pos = torch.arange(length)
    pages = kv.block_table[slot].cpu().long()[pos // PAGE].to(kv.k_pages.device)
    off = (pos % PAGE).to(kv.k_pages.device)
    kv.k_pages[pages, :, off, :] = keys.to(kv.k_pages.device, kv.k_pages.dtype)
    kv.v_pages[pages, :, :, off] = values.to(kv.v_pages.device, kv.v_pages.dtype)


def read_kv(kv, slot, length):
    pos = torch.arange(length)
    pages = kv.block_table[slot].cpu().long()[pos // PAGE].to(kv.k_pages.device)
    off = (pos % PAGE).to(kv.k_pages.device)
    return kv.k_pages[pages, :, off, :].float().cpu(), kv.v_pages[pages, :, :, off].float().cpu()


def attention_oracle(q, keys, values, pos, scale, window=0):
    """q [n_heads, hd], keys/values [L, n_kv, hd] (float64): the query at position ``pos`` sees
    keys max(0, pos - window + 1) .. pos; softmax(q k / sqrt) v with grouped heads."""
    n_heads = q.shape[0]
    n_kv = keys.shape[1]
    group = n_heads // n_kv
    first = max(0, pos - window + 1) if window else 0
    k = keys[first:pos + 1].repeat_interleave(group, dim=1)
    v = values[first:pos + 1].repeat_interleave(group, dim=1)
    s = torch.einsum("hd,lhd->hl", q, k) * scale
    p = torch.softmax(s, dim=-1)
    return torch.einsum("hl,lhd->hd", p, v)
