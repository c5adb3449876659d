"""How the attention mixer's keys and values lie inside a page of the cache.

The cache hands a mixer pages of whatever shape it asked for and never looks inside them; this
module is the attention part's own knowledge.  A page holds ``page`` = 64 positions of every kv
head.  Per (page, kv head):

* keys, layout ``K_LAYOUT``: ``[ceil(head_dim / 16), 64, 16]``: blocks of 16 dims, each holding
  all 64 positions (a head size that is no multiple of 16 pads its last block);
* values, layout ``V_LAYOUT``: ``[2, head_dim, 32]``: halves of 32 positions.

The attention kernels load 16-byte pieces, 8 dims of a key or 8 positions of a value dim, in the
pattern the matrix cores want them; in this layout the pieces of one load instruction fill whole
128-byte lines (4 consecutive keys of a block; 16 consecutive dims of a half), so a line is
fetched once and not in two halves by two instructions.
"""
from typing import Tuple

from ..errors import ConfigError
from .base import CacheNeed, Plane

PAGE = 64
DIM_BLOCK = 16
HALF = 32
K_LAYOUT = "k: blocks of 16 dims x 64 positions"
V_LAYOUT = "v: halves of 32 positions"


def key_page_shape(n_kv_heads: int, head_dim: int) -> Tuple[int, ...]:
    return (n_kv_heads, -(-head_dim // DIM_BLOCK), PAGE, DIM_BLOCK)


def value_page_shape(n_kv_heads: int, head_dim: int) -> Tuple[int, ...]:
    return (n_kv_heads, PAGE // HALF, head_dim, HALF)


def key_pages_shape(n_pages: int, n_kv_heads: int, head_dim: int) -> Tuple[int, ...]:
    return (n_pages,) + key_page_shape(n_kv_heads, head_dim)


def value_pages_shape(n_pages: int, n_kv_heads: int, head_dim: int) -> Tuple[int, ...]:
    return (n_pages,) + value_page_shape(n_kv_heads, head_dim)


def kv_need(n_kv_heads: int, head_dim: int, window: int, page: int) -> CacheNeed:
    """What grouped-query attention keeps per token: the planes "k" and "v" in the layouts above."""
    if page != PAGE:
        raise ConfigError("the attention kernels read pages of %d positions, the cache has pages of %d" % (PAGE, page))
    return CacheNeed("window" if window else "full",
                     (Plane("k", key_page_shape(n_kv_heads, head_dim), K_LAYOUT),
                      Plane("v", value_page_shape(n_kv_heads, head_dim), V_LAYOUT)), window)


def write_keys(k_pages, pages, offsets, keys) -> None:
    """k_pages[page, :, position] = keys[i] for every i: ``pages`` and ``offsets`` (position in
    the page) are index tensors of length L, ``keys`` is ``[L, n_kv_heads, head_dim]``."""
    n, n_kv, hd = keys.shape
    blocks = k_pages.shape[2]
    padded = keys.new_zeros((n, n_kv, blocks * DIM_BLOCK))
    padded[..., :hd] = keys
    k_pages[pages, :, :, offsets, :] = padded.reshape(n, n_kv, blocks, DIM_BLOCK).to(k_pages.dtype)


def write_values(v_pages, pages, offsets, values) -> None:
    """The same for values ``[L, n_kv_heads, head_dim]``."""
    v_pages[pages, :, offsets // HALF, :, offsets % HALF] = values.to(v_pages.dtype)


def read_keys(k_pages, pages, offsets, head_dim: int):
    """``[L, n_kv_heads, head_dim]``: the keys at (pages[i], offsets[i])."""
    got = k_pages[pages, :, :, offsets, :]                   # [L, n_kv, blocks, 16]
    return got.reshape(got.shape[0], got.shape[1], -1)[..., :head_dim]


def read_values(v_pages, pages, offsets):
    """``[L, n_kv_heads, head_dim]``: the values at (pages[i], offsets[i])."""
    return v_pages[pages, :, offsets // HALF, :, offsets % HALF]
