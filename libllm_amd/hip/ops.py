"""Host side of the kernels: checks every operand, then launches on the current HIP stream.

This is the only implementation of the operations on the product path.  It needs a GPU and the
built kernel library; without either it raises KernelError.  Matrix products in bfloat16 with many
rows go to the vendor library through ``torch.matmul`` (the reference uses its vendor's library
for them as well, src/flint/cuda/gemm_cublas.cc:160-197); every other operation is a kernel of
``csrc``.
"""
import ctypes
import gc
import os
from typing import List, Optional

import numpy as np
import torch

from ..parts.kv_pages import K_LAYOUT, V_LAYOUT, key_pages_shape, value_pages_shape
from ..errors import KernelError, ReplayMismatch
from . import build

_F32, _BF16 = 0, 1
_vp, _i, _f = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
_u64 = ctypes.c_ulonglong


def _code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return _F32
    if dtype == torch.bfloat16:
        return _BF16
    raise KernelError("unsupported storage dtype %s (float32 and bfloat16 only)" % dtype)


_SIGNATURES = {
    "llm_embed": [_vp, _i, _vp, _vp, _i, _i, _i, _f, _vp],
    "llm_embed_norm": [_vp, _i, _vp, _vp, _i, _i, _i, _f, _vp, _vp, _vp, _vp],
    "llm_add_rmsnorm": [_vp, _vp, _i, _i, ctypes.c_size_t, _vp, _f, _vp, _i, _vp, _i, _i, _vp],
    "llm_silu_mul": [_vp, _vp, _i, _i, _i, _i, _vp],
    "llm_add_bias": [_vp, _i, _vp, _i, _i, _vp],
    "llm_rope_kv_write": [_vp, _i, _i, _vp, _i, _i, _i, _vp, _vp, _i, _vp, _vp, _vp, _vp, _i, _vp,
                          _vp, _i, _i, _i, _i, _vp],
    "llm_gemm_skinny_rope_bf16": [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp, _vp, _i,
                                  _vp, _vp, _vp, _vp, _i, _vp, _vp, _i, _i, _vp, _i, _f, _vp],
    "llm_pack_weight": [_vp, _vp, _i, _i, _i, _vp],
    "llm_gemm_f32": [_vp, _vp, _vp, _i, _i, _i, _vp],
    "llm_attention_ref": [_vp, _i, _i, _vp, _vp, _vp, _i, _i, _vp, _vp, _vp, _vp, _i, _i, _i, _i,
                          _f, _i, _vp],
    "llm_gemm_skinny_bf16": [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp],
    "llm_gemm_mid_bf16": [_vp, _i, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp],
    "llm_gemm_wide_bf16": [_vp, _i, _vp, _i, _vp, _i, _i, _i, _i, _i, _vp],
    "llm_gemm_skinny_norm_bf16": [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _i, _f, _vp],
    "llm_attention_mfma_supported": [_i],
    "llm_attention_prefill_bf16": [_vp, _i, _vp, _vp, _vp, _i, _i, _vp, _vp, _vp, _vp, _i, _i, _i,
                                   _i, _i, _f, _i, _i, _vp],
    "llm_attention_decode_bf16": [_vp, _i, _vp, _vp, _vp, _i, _i, _vp, _vp, _vp, _vp, _vp, _i,
                                  _i, _i, _i, _f, _i, _i, _i, _vp],
    "llm_attention_decode_waves": [_i],
    "llm_argmax": [_vp, _vp, _vp, _vp, _i, _i, _vp],
    "llm_argmax_parts": [_i],
    "llm_sample": [_vp, _vp, _i, _i, _f, _i, _f, _u64, _vp, _vp, _vp, _vp, _vp, _vp],
    "llm_sample_parts": [_i],
    "llm_sample_k_part": [_i, _i],
    "llm_peak_sink_words": [],
    "llm_peak_read": [_vp, ctypes.c_size_t, _vp, _i, _i, _vp],
    "llm_peak_copy": [_vp, _vp, ctypes.c_size_t, _i, _vp],
    "llm_peak_mfma_bf16": [_vp, _i, ctypes.POINTER(ctypes.c_double), _vp],
    "llm_peak_fma_f32": [_vp, _i, ctypes.POINTER(ctypes.c_double), _vp],
}


class Prenormed:
    """What a product that added into the stream leaves for the norm with ``weight`` and ``eps``
    that reads the stream next: ``raw`` = bfloat16(stream * weight) and ``ssq[M, width / 16]``, the
    sums of squares of the stream's rows over tiles of 16 columns.  The product after that norm
    takes ``raw`` as its rows and multiplies its sums by rsqrt(sum(ssq[m]) / width + eps)."""

    def __init__(self, raw, ssq, weight, eps):
        self.raw, self.ssq, self.weight, self.eps = raw, ssq, weight, eps


class NormedRows:
    """Rows ``rows`` (all, if None) of the float32 matrix ``res``, to be RMS-normalised with
    ``weight`` and ``eps``: what ``HipOps.normed`` returns.  ``pre``: what the product before
    left for this norm, if it did."""

    def __init__(self, res, weight, eps, rows=None, pre=None):
        self.res, self.weight, self.eps, self.rows, self.pre = res, weight, eps, rows, pre
        self.n_rows = res.shape[0] if rows is None else rows.shape[0]


class PreparedWeight:
    """A weight matrix ``w`` and its copy ``tiled`` for the matrix cores: what
    ``HipOps.prepare_weight`` returns and every product takes in place of the matrix."""

    def __init__(self, w, tiled):
        self.w, self.tiled = w, tiled
        self.shape, self.dtype = w.shape, w.dtype


class HipOps:
    """The operations of the model on the GPU: the only implementation there is.  Every method
    checks its operands on the host before a kernel is launched."""

    supports_graphs = True
    folds_norms = True      # ``linear`` takes ``then_norm`` and may return a ``Prenormed``

    # Launch decisions, each measured with variants side by side in one process:
    SKINNY_ROWS = 64        # most rows the streaming matrix product takes at once; beyond, the library's
    ACCUM_ROWS = 16         # most rows for which a product adds into the stream itself
    SPLIT_ROWS = 64         # beyond those and up to here it goes in slices of K that the next norm adds; then the library's
    # MID_FROM to MID_ROWS rows: a streaming product of their own for weights with a tiled copy; beyond,
    # the library's.  Whole engines compared in one process, prompt steps of 128 tokens: 3.27
    # against 4.18 ms at the 3B shape, 5.57 against 7.07 at 8B, 1.62 against 1.66 at 1B; decode
    # batches of 96: 3.56 against 4.34, 5.84 against 7.10, 1.72 against 1.82.  For the small o
    # weight of the 1B shape the library's product is as fast (10.2 against 10.4 us): hence the limit.
    MID_ROWS = 128
    # From 33 rows on it also beats the product for few rows, which stages the rows of X anew for
    # every 16 to 64 rows of the weight (decode steps of whole engines in one process, batches of
    # 48 and 64: 2.04 against 2.09 and 2.38 against 2.46 ms at the 1B shape, 4.02 against 4.11 and
    # 4.69 against 4.83 at 3B, 5.58 against 5.74 and 6.17 against 6.45 at 8B).
    MID_FROM = 33
    MID_HEAD = True         # logits of 65 rows and more by it too (beyond its most rows in passes)
    # With ``mid_two``, 129 to MID_TWO_ROWS rows go to the same product in two slabs of rows, a
    # block each for every tile of W, neighbours on one chiplet, so that W still comes from memory
    # once.  Where it is taken, by the product (us a product with the norm that follows, at 160 / 256
    # rows, against the library's): down 1B 20.8 / 24.5 against 30.1 / 32.5, 3B 30.0 / 33.9 against
    # 33.6 / 39.7, 8B 49.7 / 56.8 against 89.1 / 70.2, a 8,192 x 28,672 weight 172 / 197 against 221 /
    # 323; output 3B 18.5 / 20.6 against 21.2 / 22.9, 8B 22.1 / 25.8 against 33.0 / 28.9 (1B 13.7 /
    # 16.0 against 13.3 / 14.2: a tie at best); half as many slices of K as up to 128 rows, for as
    # many blocks.  Whole engines with the rules below (ms): decode at batch 160 / 256, context 1,024:
    # 1B 2.48 / 3.08 against 2.81 / 3.29, 3B 6.38 / 8.30 against 6.79 / 9.02, 8B 9.06 / 11.8 against
    # 10.9 / 12.9; prompts of 170 / 256 tokens: 1B 1.58 / 1.74 against 1.93 / 1.96, 3B 3.71 / 4.01
    # against 4.05 / 4.70, 8B 6.20 / 6.89 against 7.00 / 7.87.
    MID_TWO_ROWS = 256
    MID_PLAIN_FILL = 0.6    # a product that does not add into the stream goes to it in two slabs if its blocks fill this share of one round of the units
    # Beyond MID_ROWS rows the gate/up product with its SwiGLU is a kernel of ours where its tiles
    # (256 or 128 rows by 128 outputs) would be filled, over whole rounds of the compute units, to
    # at least WIDE_FILL: there it beats the library's product followed by the SiLU-mul kernel, which reads
    # gate and up again (the two timed in turns, 1B shape: 105 against 121 us at 2,048 rows, 56
    # against 69 at 1,024, 206 against 234 at 4,096, 817 against 927 at 16,384, and with 128 rows a
    # block 35 against 42 at 512 and 32 against 36 at 384; 3B: 152 against 163, 79 against 90, 297
    # against 315, 1,195 against 1,269, and 52 against 55 at 512; 8B: 95 against 112 at 512, 191
    # against 207 at 1,024, the same from 2,048 on).  With half-empty rounds the library's stays
    # (1B, 256 rows: a tile of 128 rows fills half a round, 31 against 33; some such steps would
    # gain, others lose 10 %).  It gains up to WIDE_MAX_K elements of K (width 5,120, feed-forward
    # 13,824, whole prompt steps: 10.07 against 10.31 ms at 2,048 rows, 19.65 against 20.85 at 4,096)
    # and loses beyond (width 8,192, feed-forward 28,672: 16.97 against 16.59 ms and 34.6 against
    # 33.4), so there the library's stays.
    WIDE_FILL = 0.75
    WIDE_MAX_K = 5120
    # Launch sizes below are in blocks per compute unit; ``__init__`` multiplies them by the
    # device's number of units (the figures in the comments were measured on 256 units).
    MID_BLOCKS_PER_UNIT = 1.0       # blocks that the slices of K of the product for 33 to 128 rows aim at (half and twice as many lose 8 to 10 % of a prompt step of 128 tokens at the 3B and 8B shapes: fewer blocks, or more matrices for the norm to add)
    MID_FILL = 0.75                 # it takes a product that adds into the stream only if slices of at least MID_MIN_SLICE elements of K give it blocks for this share of the units (a 2,048 x 2,048 weight gets 128 blocks: the library's product is as fast, 10.2 against 10.4 us; 3,072 x 3,072 gets 192 and gains)
    MID_MIN_SLICE = 512
    DECODE_BLOCKS_PER_UNIT = 3      # blocks of the decode attention grid beyond which sequences are not split further
    DECODE_BLOCKS_AHEAD_PER_UNIT = 2    # the same where a wave would get DECODE_AHEAD_PAGES pages or more and the sequences
    DECODE_AHEAD_PAGES = 6              # fill such a grid: two blocks a compute unit, at which the kernel overlaps a wave's pages
    # New rows of the step's longest sequence from which a wave of prompt attention takes two
    # tiles of rows: heads up to 64 wide, up to 128 (wider ones never: one wave a unit would be
    # left).  A block's walk over the pages of its rows is what a short prompt waits for, and two
    # tiles make every walk longer; from here on the pages staged half as often outweigh that
    # (head size 64: 67.3 against 68.6 us at 3,072 rows, 109.4 against 104.0 at 4,096; head size
    # 128: 59.7 against 64.2 at 2,048, 124.9 against 108.1 at 3,072).  More sequences of the same
    # lengths do not move the crossing (4 x 1,024 rows: 39.1 against 43.0).
    PROMPT_TILE_ROWS = (3584, 2560)
    _EPI_NONE, _EPI_SWIGLU, _EPI_ACCUM = 0, 1, 2
    # activations of the gate in a gated feed-forward (csrc/common.h); a gated epilogue takes the
    # code above its own: epilogue | act << 4
    ACTIVATIONS = {"silu": 0, "gelu_tanh": 1, "relu": 2}

    def __init__(self, device: Optional[str] = None):
        if not torch.cuda.is_available():
            raise KernelError("no GPU is visible: this library runs on an AMD GPU only")
        self.device = torch.device(device or "cuda:0")
        if self.device.type != "cuda":
            raise KernelError("device %s is not a GPU" % (self.device,))
        self.lib = build.load()
        for name, argtypes in _SIGNATURES.items():
            try:
                fn = getattr(self.lib, name)
            except AttributeError:
                raise KernelError("the kernel library lacks %s; rebuild it" % name)
            fn.argtypes = argtypes
            fn.restype = _i
        torch.backends.cuda.matmul.allow_tf32 = False
        self.units = torch.cuda.get_device_properties(self.device).multi_processor_count
        self.MID_BLOCKS = max(1, int(self.MID_BLOCKS_PER_UNIT * self.units))
        self.DECODE_BLOCKS = self.DECODE_BLOCKS_PER_UNIT * self.units
        self.DECODE_BLOCKS_AHEAD = self.DECODE_BLOCKS_AHEAD_PER_UNIT * self.units
        # switches for tests and measurements; the product runs with all three on
        self.fast_attention = True      # bfloat16 attention on the matrix cores (else the plain kernel, as for float32)
        self.pack_weights = True        # keep a tiled copy of every weight for the skinny product
        self.fast_gemm = True           # the skinny product for few rows (else the library's for every product)
        self.wide_gemm = True           # the gate/up product with SwiGLU for many rows (else the library's and the SiLU-mul kernel)
        self.mid_gemm = True            # the product for 33 to 128 rows (else the one for few rows and the library's)
        self.mid_two = True             # the same for 129 to 256 rows, in two slabs (else the library's)
        if not build.trusted("gemm_mid.hip"):
            # its loads are invisible to the compiler: with a spilled register it would be wrong
            self.mid_gemm = False
            build._say("the product for 33 to 128 rows spills registers in this build: the one for few rows and the library's run instead")
        self.fold_norms = True          # up to ACCUM_ROWS rows, a norm between two products gets no kernel of its own
        self.prompt_tiles = 0           # tiles of rows a wave of prompt attention takes (1 or 2; 0: by the number of blocks)
        self.timing = False
        self._warming = False           # inside the run that precedes a capture
        if os.environ.get("LIBLLM_AMD_TIME", "") not in ("", "0"):
            self.start_timing()

    # ---- time per operation, behind a switch
    _TIMED = ("embed", "embed_prepared", "add_rmsnorm", "linear", "linear_swiglu", "silu_mul", "qkv_rope", "rope_kv_write",
              "attention", "argmax", "sample")

    def start_timing(self) -> None:
        """From now on every operation is bracketed by two events on its stream, and
        ``timing_report`` says where the time went (the reference has LOG_TIME around blocks and a
        build that waits after every kernel, src/lutil/log.h:39-42, src/flint/cuda/common.h:50-54).
        Also switched on by the environment variable LIBLLM_AMD_TIME=1.  Engines built on these
        operations then queue every step kernel by kernel: a captured graph would hide the
        operations from the clock."""
        if self.timing:
            return
        self.timing, self._timed, self._depth = True, {}, 0
        for name in self._TIMED:
            setattr(self, name, self._timed_call(name, getattr(self, name)))

    def _timed_call(self, name, fn):
        def call(*args, **kwargs):
            if self._depth or torch.cuda.is_current_stream_capturing():
                return fn(*args, **kwargs)                 # an operation inside another counts once
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            self._depth += 1
            try:
                start.record()
                out = fn(*args, **kwargs)
                end.record()
            finally:
                self._depth -= 1
            self._timed.setdefault(name, []).append((start, end))
            return out
        return call

    def timing_report(self, reset: bool = True):
        """[(operation, calls, milliseconds)] since the last report, the longest first."""
        torch.cuda.synchronize(self.device)
        rows = [(name, len(ev), sum(a.elapsed_time(b) for a, b in ev)) for name, ev in self._timed.items()]
        if reset:
            self._timed = {}
        return sorted(rows, key=lambda r: -r[2])

    # ---- helpers
    def _stream(self):
        return torch.cuda.current_stream(self.device).cuda_stream

    @staticmethod
    def _check(status: int, what: str):
        if status != 0:
            raise KernelError("%s: %s" % (what, {1: "the kernel refuses these operands",
                                                 2: "the launch failed",
                                                 3: "the operands exceed the fixed buffer of this entry point"
                                                 }.get(status, "error %d" % status)))

    def _weight(self, w: torch.Tensor, what: str):
        """A weight matrix: on the device, rows contiguous; rows may lie further apart than
        their length (a view of some columns of a wider matrix)."""
        if w.device != self.device:
            raise KernelError("%s lies on %s, not on %s" % (what, w.device, self.device))
        if w.dim() != 2 or w.stride(1) != 1 or w.stride(0) < w.shape[1]:
            raise KernelError("%s must be a matrix with contiguous rows" % what)
        return w.data_ptr()

    def _dev(self, t: torch.Tensor, what: str, dtype=None, shape=None):
        if t.device != self.device:
            raise KernelError("%s lies on %s, not on %s" % (what, t.device, self.device))
        if not t.is_contiguous():
            raise KernelError("%s is not contiguous" % what)
        if dtype is not None and t.dtype != dtype:
            raise KernelError("%s has dtype %s, expected %s" % (what, t.dtype, dtype))
        if shape is not None and tuple(t.shape) != tuple(shape):
            raise KernelError("%s has shape %s, expected %s" % (what, tuple(t.shape), tuple(shape)))
        return t.data_ptr()

    def upload_int32(self, arr: np.ndarray) -> torch.Tensor:
        """The array on the device, sent through pinned memory without waiting for the stream."""
        host = torch.from_numpy(np.ascontiguousarray(arr, dtype=np.int32)).pin_memory()
        return host.to(self.device, non_blocking=True)

    def capture(self, body):
        """Runs ``body`` once to warm up, then captures it into a HIP graph.  A product of the
        vendor library that ``body`` holds is first tried alone (``_library_product``); if it
        does not replay, ReplayMismatch is raised and nothing is captured.

        The capture is in global mode: runtime calls that free or query device resources are
        errors anywhere in the process while it lasts, and a finaliser that makes one (of a graph,
        a pinned buffer, an event) ends the process.  So whatever is dead and waits for the
        collector goes before the capture begins, and the collector does not run during it."""
        side = torch.cuda.Stream(self.device)
        side.wait_stream(torch.cuda.current_stream(self.device))
        warming, self._warming = self._warming, True
        try:
            with torch.cuda.stream(side):
                body()
        finally:
            self._warming = warming
        torch.cuda.current_stream(self.device).wait_stream(side)
        torch.cuda.synchronize(self.device)
        gc.collect()
        collecting = gc.isenabled()
        gc.disable()
        try:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                body()
        finally:
            if collecting:
                gc.enable()
        return graph

    # ---- operations
    def embed(self, table, ids, scale=1.0):
        v, h = table.shape
        m = ids.shape[0]
        out = torch.empty((m, h), dtype=torch.float32, device=self.device)
        self._check(self.lib.llm_embed(self._dev(table, "embedding table"), _code(table.dtype),
                                       self._dev(ids, "token ids", torch.int32), out.data_ptr(),
                                       m, h, v, float(scale), self._stream()), "embed")
        return out

    def embed_prepared(self, table, ids, scale, weight, eps, dtype):
        """The embedding, and in the same kernel what the RMS norm with ``weight`` and ``eps`` that
        reads these rows first needs (a ``Prenormed``, as ``linear(..., then_norm=)`` returns):
        (rows, record), or None where that does not apply (more than ``ACCUM_ROWS`` rows, another
        activation dtype than bfloat16, a width that is no multiple of 16)."""
        v, h = table.shape
        m = ids.shape[0]
        if not (self.fold_norms and self.fast_gemm and dtype == torch.bfloat16 and m <= self.ACCUM_ROWS and h % 16 == 0):
            return None
        self._dev(weight, "norm weight", torch.float32, (h,))
        out = torch.empty((m, h), dtype=torch.float32, device=self.device)
        raw = torch.empty((m, h), dtype=torch.bfloat16, device=self.device)
        ssq = torch.empty((m, h // 16), dtype=torch.float32, device=self.device)
        self._check(self.lib.llm_embed_norm(self._dev(table, "embedding table"), _code(table.dtype),
                                            self._dev(ids, "token ids", torch.int32), out.data_ptr(), m, h, v,
                                            float(scale), weight.data_ptr(), raw.data_ptr(), ssq.data_ptr(),
                                            self._stream()), "embed_norm")
        return out, Prenormed(raw, ssq, weight, float(eps))

    def add_rmsnorm(self, res, delta, weight, eps, out_dtype, rows=None):
        m, h = res.shape
        self._dev(res, "residual stream", torch.float32)
        self._dev(weight, "norm weight", torch.float32, (h,))
        dptr, dcode, n_delta = None, _code(out_dtype), 1
        if delta is not None:
            if delta.dim() == 3:                     # several float32 matrices, added in their order
                n_delta = delta.shape[0]
                dptr = self._dev(delta, "delta", torch.float32, (n_delta, m, h))
            else:
                dptr = self._dev(delta, "delta", shape=(m, h))
            dcode = _code(delta.dtype)
        n_out = m
        rptr = None
        if rows is not None:
            rptr = self._dev(rows, "row indices", torch.int32)
            n_out = rows.shape[0]
        out = torch.empty((n_out, h), dtype=out_dtype, device=self.device)
        self._check(self.lib.llm_add_rmsnorm(res.data_ptr(), dptr, dcode, n_delta, m * h, weight.data_ptr(),
                                             float(eps), out.data_ptr(), _code(out_dtype), rptr,
                                             n_out, h, self._stream()), "add_rmsnorm")
        return out

    def prepare_weight(self, w: torch.Tensor, like=None):
        """Called once for a weight matrix that products will stream many times.  Returns what
        the products take in place of ``w``: ``w`` itself, or a record that holds, beside ``w``,
        a copy tiled for the matrix cores, which the products for few rows read instead (a wave
        then loads 1 KiB in a row rather than 16 pieces of 64 bytes); the library product for
        many rows goes on reading ``w``.  ``like``: the record of a matrix of which ``w`` is the
        leading rows (a multiple of 16 of them); its tiled copy then serves ``w`` too."""
        if isinstance(like, PreparedWeight) and w.shape[0] % 16 == 0 and w.data_ptr() == like.w.data_ptr() \
                and w.shape[1] == like.w.shape[1] and w.shape[0] <= like.w.shape[0]:
            return PreparedWeight(w, like.tiled)
        if (not self.pack_weights or w.dtype != torch.bfloat16 or w.dim() != 2 or w.shape[1] % 8
                or w.stride(1) != 1 or w.stride(0) % 8 or w.data_ptr() % 16 or w.device != self.device):
            return w
        n, k = w.shape
        tiled = torch.empty((-(-n // 16) * -(-k // 32) * 512,), dtype=torch.bfloat16, device=self.device)
        self._check(self.lib.llm_pack_weight(w.data_ptr(), tiled.data_ptr(), n, k, w.stride(0),
                                             self._stream()), "pack_weight")
        return PreparedWeight(w, tiled)

    @staticmethod
    def _plain(w):
        return w.w if isinstance(w, PreparedWeight) else w

    @staticmethod
    def _streamed(w):
        """(pointer, row stride) the skinny product reads a weight through: its tiled copy if it
        has one (row stride 0 says so), else the matrix itself."""
        if isinstance(w, PreparedWeight):
            return w.tiled.data_ptr(), 0
        return w.data_ptr(), w.stride(0)

    def normed(self, res, weight, eps, rows=None, pre=None):
        """Rows of the float32 stream ``res`` that are to be RMS-normalised: a record that
        ``linear``, ``linear_swiglu`` and ``qkv_rope`` take in place of a matrix: they run the
        norm kernel on just these rows, in the dtype they need, or, with ``pre`` (what
        ``linear(..., then_norm=)`` returned when it added into ``res``, nothing having touched
        ``res`` since), take the rows the product before has left.  (The norm computed inside the
        product itself was measured and lost: every block then normalises the rows again.)"""
        if pre is not None and (rows is not None or pre.weight is not weight or pre.eps != float(eps)
                                or pre.raw.shape != res.shape):
            pre = None
        return NormedRows(res, weight, float(eps), rows, pre)

    def _materialise(self, x, dtype):
        if isinstance(x, NormedRows):
            return self.add_rmsnorm(x.res, None, x.weight, x.eps, dtype, x.rows)
        return x

    def _skinny_ok(self, x, w, m, k):
        w = self._plain(w)
        if not (self.fast_gemm and w.dtype == torch.bfloat16 and k % 8 == 0 and w.data_ptr() % 16 == 0
                and w.stride(0) % 8 == 0):
            return False
        if isinstance(x, NormedRows):
            # rows left by the product before go straight in; else the norm kernel runs first
            return x.pre is not None and m <= self.ACCUM_ROWS
        return x.dtype == torch.bfloat16 and x.data_ptr() % 16 == 0

    @staticmethod
    def _k_split(n, k):
        """Slices of K for a product of 17 to 64 rows with a weight of ``n`` rows: enough for about
        a block a compute unit at 64 weight rows a block, each at least 512 long and a multiple of 32."""
        ks = max(1, min(8, 256 // max(1, -(-n // 64))))
        while ks > 1 and (k % (ks * 32) or k // ks < 512):
            ks -= 1
        return ks

    def _mid_rows(self):
        return self.MID_TWO_ROWS if self.mid_two else self.MID_ROWS

    def _mid_ok(self, x, w, m, k):
        return (self.fast_gemm and self.mid_gemm and isinstance(w, PreparedWeight)
                and self.MID_FROM <= m <= self._mid_rows() and not isinstance(x, NormedRows)
                and x.dtype == torch.bfloat16 and x.dim() == 2 and x.stride(1) == 1 and x.stride(0) >= k
                and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0 and k % 128 == 0)

    def _wide_ok(self, x, w, m, k, inter):
        """The rows of X a block takes (256 or 128) if the gate/up product of ``m`` rows goes to
        the kernel for many rows, else 0."""
        if not (self.fast_gemm and self.wide_gemm and m > self.MID_ROWS and not isinstance(x, NormedRows)):
            return 0
        wp = self._plain(w)
        if not (x.dtype == torch.bfloat16 and wp.dtype == torch.bfloat16 and x.dim() == 2 and x.stride(1) == 1
                and x.stride(0) >= k and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0
                and wp.stride(1) == 1 and wp.stride(0) >= k and wp.stride(0) % 8 == 0 and wp.data_ptr() % 16 == 0
                and k % 64 == 0 and k <= self.WIDE_MAX_K and inter % 16 == 0):
            return 0
        for block_rows in (256, 128):
            tiles = -(-m // block_rows) * -(-inter // 128)
            rounds = -(-tiles // self.units)
            # the share of the rounds' tiles that the step's rows and outputs really fill
            if m * inter >= self.WIDE_FILL * rounds * self.units * block_rows * 128:
                return block_rows
        return 0

    def _wide(self, x, w, out, epilogue, block_rows=256):
        wp = self._plain(w)
        n, k = wp.shape
        self._check(self.lib.llm_gemm_wide_bf16(
            x.data_ptr(), x.stride(0), wp.data_ptr(), wp.stride(0), out.data_ptr(), epilogue, block_rows,
            x.shape[0], n, k, self._stream()), "gemm_wide_bf16")
        return out

    def _k_split_mid(self, n, k, slabs=1):
        """Slices of K for a product of 33 to 256 rows whose result the next norm adds: enough for
        about MID_BLOCKS blocks at 64 weight rows a block and slab of rows, each at least
        MID_MIN_SLICE long and a multiple of 128."""
        ks = max(1, min(16, self.MID_BLOCKS // max(1, -(-n // 64) * slabs)))
        while ks > 1 and (k % (ks * 128) or k // ks < self.MID_MIN_SLICE):
            ks -= 1
        return ks

    def _mid(self, x, w, out, epilogue, k_split=1):
        n, k = w.shape
        self._check(self.lib.llm_gemm_mid_bf16(
            x.data_ptr(), x.stride(0), w.tiled.data_ptr(), out.data_ptr(), epilogue, _code(out.dtype),
            x.shape[0], n, k, k_split, self._stream()), "gemm_mid_bf16")
        return out

    def _skinny(self, x, w, out, epilogue, m0=0, mm=None, k_split=1):
        """Launches the skinny kernel on rows m0 .. m0+mm of the bfloat16 matrix x; with ``k_split``
        the products over that many slices of K go to ``out[k_split, mm, n]``."""
        n, k = w.shape
        width = n // 2 if (epilogue & 15) == self._EPI_SWIGLU else n
        wptr, ldw = self._streamed(w)
        if isinstance(x, NormedRows):           # rows that lack their norm's scale: see Prenormed
            pre = x.pre
            self._check(self.lib.llm_gemm_skinny_norm_bf16(
                pre.raw.data_ptr(), wptr, out.data_ptr(), epilogue, _code(out.dtype), mm, n, k, ldw,
                None, None, None, pre.ssq.data_ptr(), pre.ssq.shape[1], pre.eps, self._stream()),
                "gemm_skinny_norm_bf16")
            return
        xp = x.data_ptr() + m0 * k * 2
        self._check(self.lib.llm_gemm_skinny_bf16(
            xp, wptr, out.data_ptr() + m0 * width * out.element_size(),
            epilogue, _code(out.dtype), mm, n, k, ldw, k_split, self._stream()), "gemm_skinny_bf16")

    def linear(self, x, w, bias, out_dtype, residual=None, then_norm=None):
        """x W^T (+ bias) as ``out_dtype``.  ``x`` is a matrix or a ``normed`` record.  With
        ``residual`` (the float32 stream, same shape as the result) the product is added into it
        where the kernel can do that, and None is returned; otherwise the result is returned and
        the caller adds it.  ``then_norm`` = (weight, eps) says that an RMS norm with these reads
        ``residual`` next, before anything else touches it: where the product adds into the
        stream at up to ``ACCUM_ROWS`` rows it then returns a ``Prenormed`` for ``normed``."""
        lazy = isinstance(x, NormedRows)
        m, k = (x.n_rows, x.res.shape[1]) if lazy else x.shape
        n, k2 = w.shape
        if k != k2:
            raise KernelError("linear: x is [%d, %d] but the weight is [%d, %d]" % (m, k, n, k2))
        self._weight(self._plain(w), "linear weight")
        if lazy:
            self._dev(x.res, "residual stream", torch.float32)
            self._dev(x.weight, "norm weight", torch.float32, (k,))
        else:
            self._dev(x, "linear input")
        if (m <= self.SKINNY_ROWS and residual is not None and bias is None and self._mid_ok(x, w, m, k)
                and (ks := self._k_split_mid(n, k)) * -(-n // 64) >= self.MID_FILL * self.units):
            return self._mid(x, w, torch.empty((ks, m, n), dtype=torch.float32, device=self.device),
                             self._EPI_NONE, ks)
        if (self.MID_HEAD and out_dtype == torch.float32 and residual is None and bias is None
                and self.SKINNY_ROWS < m and not lazy):
            # float32 results (logits) for 65 to 128 rows in one pass over the weight, where the
            # product for few rows would take two, and for more rows in passes of up to 128
            passes = -(-m // self._mid_rows())
            # the rows dealt out evenly, each pass starting at a multiple of 16 rows (which keeps
            # its rows of the result aligned): passes of at least 49 rows
            cuts = [min(m, -(-(i * m) // (passes * 16)) * 16) for i in range(passes)] + [m]
            if self._mid_ok(x[:cuts[1]], w, cuts[1], k):
                out = torch.empty((m, n), dtype=torch.float32, device=self.device)
                for m0, m1 in zip(cuts, cuts[1:]):
                    self._mid(x[m0:m1], w, out[m0:m1].view(1, m1 - m0, n), self._EPI_NONE, 1)
                return out
        if (self._skinny_ok(x, w, m, k) and bias is None and residual is not None
                and self.ACCUM_ROWS < m <= self.SPLIT_ROWS and (ks := self._k_split(n, k)) > 1):
            # K in slices, one block for 64 rows of the weight and a slice: each slice of X is staged
            # for four times the rows; the norm kernel that follows adds the slices, in order
            parts = torch.empty((ks, m, n), dtype=torch.float32, device=self.device)
            self._skinny(x, w, parts, self._EPI_NONE, 0, m, k_split=ks)
            return parts
        if self._skinny_ok(x, w, m, k) and bias is None and not (residual is not None and m > self.ACCUM_ROWS):
            if residual is not None and m <= self.SKINNY_ROWS:
                self._dev(residual, "residual stream", torch.float32, (m, n))
                if then_norm is not None and self.fold_norms and n % 16 == 0 and not lazy:
                    weight, eps = then_norm
                    self._dev(weight, "norm weight", torch.float32, (n,))
                    raw = torch.empty((m, n), dtype=torch.bfloat16, device=self.device)
                    ssq = torch.empty((m, n // 16), dtype=torch.float32, device=self.device)
                    wptr, ldw = self._streamed(w)
                    self._check(self.lib.llm_gemm_skinny_norm_bf16(
                        x.data_ptr(), wptr, residual.data_ptr(), self._EPI_ACCUM, _code(torch.float32),
                        m, n, k, ldw, weight.data_ptr(), raw.data_ptr(), ssq.data_ptr(), None, 0, 0.0,
                        self._stream()), "gemm_skinny_norm_bf16")
                    return Prenormed(raw, ssq, weight, float(eps))
                self._skinny(x, w, residual, self._EPI_ACCUM, 0, m)
                return None
            if m <= self.SKINNY_ROWS or (out_dtype == torch.float32 and not lazy):
                # float32 results for many rows (logits of whole prompts) go through the same kernel
                # 64 rows at a time: a row's logits are then the same bits whatever the batch holds
                odt = torch.float32 if out_dtype == torch.float32 else torch.bfloat16
                out = torch.empty((m, n), dtype=odt, device=self.device)
                for m0 in range(0, m, self.SKINNY_ROWS):
                    self._skinny(x, w, out, self._EPI_NONE, m0, min(self.SKINNY_ROWS, m - m0))
                return out
        if lazy:
            x = self._materialise(x, torch.float32 if w.dtype == torch.float32 else torch.bfloat16)
            if self._skinny_ok(x, w, m, k) and bias is None:
                return self.linear(x, w, None, out_dtype, residual)
        if self._mid_ok(x, w, m, k) and bias is None and out_dtype != torch.float32:
            slabs = 2 if m > self.MID_ROWS else 1
            tiles = -(-n // 64) * slabs
            if residual is not None and (ks := self._k_split_mid(n, k, slabs)) * tiles >= self.MID_FILL * self.units:
                # K in slices for enough blocks; the norm kernel that follows adds them, in order
                return self._mid(x, w, torch.empty((ks, m, n), dtype=torch.float32, device=self.device),
                                 self._EPI_NONE, ks)
            # Without slices of K, for a product that does not add into the stream (q|k|v), it has
            # too few blocks up to 128 rows and loses to the library (16.7 against 13.0 us at 128
            # rows of the 1B shape).  In two slabs it has twice as many and wins where they make
            # one round of the units that is well filled (us at 160 / 256 rows: 3B, 160 blocks,
            # 19.3 / 21.6 against 24.0 / 32.3; 8B, 192 blocks, 24.7 / 28.0 against 29.2 / 41.3; but
            # 1B, 96 blocks, 13.5 / 15.3 against 9.5 / 10.9, and a weight of 10,240 x 8,192, 320
            # blocks, 85 / 99 against 72 / 94).
            if (residual is None and slabs == 2
                    and self.MID_PLAIN_FILL * self.units <= tiles <= self.units):
                return self._mid(x, w, torch.empty((m, n), dtype=torch.bfloat16, device=self.device), self._EPI_NONE)
        w = self._plain(w)
        if w.dtype == torch.float32:
            if w.stride(0) != k:
                raise KernelError("linear: a float32 weight must be contiguous")
            xf = x if x.dtype == torch.float32 else x.float()
            out = torch.empty((m, n), dtype=torch.float32, device=self.device)
            self._check(self.lib.llm_gemm_f32(xf.data_ptr(), w.data_ptr(), out.data_ptr(), m, n, k,
                                              self._stream()), "gemm_f32")
        elif w.dtype == torch.bfloat16 and x.dtype == torch.bfloat16:
            out = self._library_product(x, w)
        else:
            raise KernelError("linear: input %s with weight %s is not supported" % (x.dtype, w.dtype))
        if bias is not None:
            self._dev(bias, "bias", torch.float32, (n,))
            self._check(self.lib.llm_add_bias(out.data_ptr(), _code(out.dtype), bias.data_ptr(), m, n,
                                              self._stream()), "add_bias")
        return out if out.dtype == out_dtype else out.to(out_dtype)

    REPLAY_TRIALS = 3
    _replayable = {}                # (device, shape of a library product) -> whether it replays from a graph; one for the process

    def _library_product(self, x, w):
        """x W^T by the vendor library.  The library chooses a kernel by the shape, and some of
        its kernels clear a scratch buffer first by a fill that, recorded into a graph, has been
        seen here to take effect on the first replay only.  So the first time a shape is about
        to be captured (in the run that precedes the capture) the product alone is recorded
        into a graph of its own and replayed ``REPLAY_TRIALS`` times over new rows, with the
        same product queued directly beside it; a shape whose replays differ by one bit raises
        ReplayMismatch, now and whenever it is about to be captured again."""
        if self._warming and not torch.cuda.is_current_stream_capturing():
            key = (x.shape[0], w.shape[0], w.shape[1], x.stride(0), w.stride(0), self.device.index or 0)
            if key not in self._replayable:
                self._replayable[key] = self._product_replays(x, w)
            if not self._replayable[key]:
                raise ReplayMismatch("the library's product of %d x %d rows over %d elements does not replay from a "
                                     "captured graph" % key[:3])
        return torch.matmul(x, w.t())

    def _product_replays(self, x, w) -> bool:
        rows = torch.empty_strided(x.shape, x.stride(), dtype=x.dtype, device=self.device).normal_()
        held = {}

        def body():
            held["out"] = torch.matmul(rows, w.t())
        warming, self._warming = self._warming, False        # (the capture below warms up too)
        try:
            graph = self.capture(body)
        finally:
            self._warming = warming
        same = True
        for trial in range(self.REPLAY_TRIALS):
            rows.normal_()
            direct = torch.matmul(rows, w.t())
            graph.replay()
            same = same and torch.equal(held["out"].view(torch.int16), direct.view(torch.int16))
        return same

    def _act(self, activation):
        if activation not in self.ACTIVATIONS:
            raise KernelError("unknown activation %r (known: %s)" % (activation, ", ".join(sorted(self.ACTIVATIONS))))
        return self.ACTIVATIONS[activation]

    def linear_swiglu(self, x, w, dtype=None, activation="silu"):
        """act(x Wg^T) * (x Wu^T) for the stacked weight ``w = [Wg; Wu]``, ``act`` being SiLU or
        another of ``ACTIVATIONS``: one kernel where a product of ours takes the rows, else the
        library's product followed by the kernel that gates.  ``x`` is a matrix or a ``normed``
        record; ``dtype`` is the activation dtype (needed for a record)."""
        gated = self._EPI_SWIGLU | (self._act(activation) << 4)
        lazy = isinstance(x, NormedRows)
        m, k = (x.n_rows, x.res.shape[1]) if lazy else x.shape
        dtype = dtype or (x.dtype if not lazy else None)
        two_i = w.shape[0]
        if two_i % 2:
            raise KernelError("linear_swiglu: the stacked weight has an odd number of rows")
        inter = two_i // 2
        if k != w.shape[1]:
            raise KernelError("linear_swiglu: x is [%d, %d] but the weight is %s" % (m, k, tuple(w.shape)))
        if (self._skinny_ok(x, w, m, k) and m <= self.SKINNY_ROWS and inter % 16 == 0
                and dtype == torch.bfloat16 and not self._mid_ok(x, w, m, k)):
            self._weight(self._plain(w), "linear weight")
            out = torch.empty((m, inter), dtype=torch.bfloat16, device=self.device)
            self._skinny(x, w, out, gated, 0, m)
            return out
        if lazy:
            if dtype is None:
                raise KernelError("linear_swiglu: a normed record needs the activation dtype")
            x = self._materialise(x, dtype)
            return self.linear_swiglu(x, w, dtype, activation)
        # (in two slabs of rows only where all its blocks run at once: us at 160 / 256 rows against
        # the library's product and the gating kernel: 1B 30.0 / 36.3 against 32.7 / 36.5, 3B 41.3 /
        # 48.1 against 40.8 / 50.3, but 8B, 1,792 blocks, 93 / 105 against 67 / 80)
        if (self._mid_ok(x, w, m, k) and inter % 16 == 0 and dtype == torch.bfloat16
                and (m <= self.MID_ROWS or -(-inter // 32) <= self.units)):
            self._weight(self._plain(w), "linear weight")
            return self._mid(x, w, torch.empty((m, inter), dtype=torch.bfloat16, device=self.device), gated)
        if dtype == torch.bfloat16 and (block_rows := self._wide_ok(x, w, m, k, inter)):
            self._weight(self._plain(w), "linear weight")
            self._dev(x, "linear input")
            return self._wide(x, w, torch.empty((m, inter), dtype=torch.bfloat16, device=self.device),
                              gated, block_rows)
        return self.silu_mul(self.linear(x, w, None, x.dtype), activation)

    def silu_mul(self, gu, activation="silu"):
        """act(first half of each row) * second half; ``act`` is SiLU unless said otherwise."""
        m, two_i = gu.shape
        if two_i % 2:
            raise KernelError("silu_mul: the input width %d is odd" % two_i)
        out = torch.empty((m, two_i // 2), dtype=gu.dtype, device=self.device)
        self._check(self.lib.llm_silu_mul(self._dev(gu, "gate_up"), out.data_ptr(), _code(gu.dtype),
                                          m, two_i // 2, self._act(activation), self._stream()), "silu_mul")
        return out

    # rotating pairs side by side (2j, 2j+1) let the projection's epilogue rotate them: a mixer
    # that reorders its projection's rows accordingly may pass adjacent=True
    prefers_adjacent_pairs = True

    def qkv_rope(self, x, w, bias, n_heads, n_kv, hd, cos, sin, rot_dim, ctx, kv, write, adjacent,
                 dtype):
        """The stacked q|k|v projection (q alone if not ``write``), bias, rotation of q and k at
        the tokens' positions, and k and v into the cache.  Returns rows whose first
        ``n_heads * hd`` columns are the rotated queries.  For few rows in bfloat16 with pairs
        side by side this is one kernel; otherwise the product and the rotation kernel."""
        lazy = isinstance(x, NormedRows)
        m, k = (x.n_rows, x.res.shape[1]) if lazy else x.shape
        n = (n_heads + (2 * n_kv if write else 0)) * hd
        if tuple(w.shape) != (n, k):
            raise KernelError("qkv_rope: the weight is %s, expected %s" % (tuple(w.shape), (n, k)))
        fused = (dtype == torch.bfloat16 and (adjacent or rot_dim == 0) and hd % 16 == 0
                 and m <= self.SKINNY_ROWS and m == ctx.n_tokens
                 and (not write or (kv is not None and "k" in kv.planes and kv.planes["k"].dtype == torch.bfloat16)))
        pre = x.pre if lazy and fused and self._skinny_ok(x, w, m, k) else None
        if pre is not None:
            x, lazy = pre.raw, False             # rows that lack their norm's scale: see Prenormed
        elif fused and lazy:
            x, lazy = self._materialise(x, dtype), False
        if fused and self._skinny_ok(x, w, m, k):
            self._weight(self._plain(w), "qkv weight")
            cptr = sptr = None
            if rot_dim:
                if cos is None or cos.shape[1] != rot_dim // 2 or cos.shape != sin.shape:
                    raise KernelError("qkv_rope: rotary tables do not match rot_dim %d" % rot_dim)
                if not ctx.captured and ctx.max_ctx > cos.shape[0]:
                    raise KernelError("qkv_rope: position %d exceeds the rotary table of %d rows"
                                      % (ctx.max_ctx - 1, cos.shape[0]))
                cptr, sptr = self._dev(cos, "cos", torch.float32), self._dev(sin, "sin", torch.float32)
            bptr = None
            if bias is not None:
                bptr = self._dev(bias, "qkv bias", torch.float32)
                if bias.shape[0] < n:
                    raise KernelError("qkv_rope: the bias is shorter than a row")
            kptr = vptr = tptr = None
            stride = 0
            if write:
                k_pages, v_pages = self._kv_planes(kv, n_kv, hd, torch.bfloat16)
                kptr, vptr, tptr = k_pages.data_ptr(), v_pages.data_ptr(), kv.block_table.data_ptr()
                stride = kv.block_table.shape[1]
            xp = self._dev(x, "qkv input", torch.bfloat16)
            q = torch.empty((m, n_heads * hd), dtype=torch.bfloat16, device=self.device)
            wptr, ldw = self._streamed(w)
            self._check(self.lib.llm_gemm_skinny_rope_bf16(
                xp, wptr, bptr, q.data_ptr(), m, k, ldw, n_heads, n_kv, hd,
                cptr, sptr, rot_dim, ctx.tok_pos.data_ptr(), ctx.tok_seq.data_ptr(),
                ctx.seq_slot.data_ptr(), tptr, stride, kptr, vptr, 64, 1 if write else 0,
                pre.ssq.data_ptr() if pre is not None else None, pre.ssq.shape[1] if pre is not None else 0,
                pre.eps if pre is not None else 0.0, self._stream()), "gemm_skinny_rope_bf16")
            return q
        qkv = self.linear(x, w, None, dtype)
        self.rope_kv_write(qkv, bias, n_heads, n_kv, hd, cos, sin, rot_dim, ctx, kv, write, adjacent)
        return qkv

    def rope_kv_write(self, qkv, bias, n_heads, n_kv, hd, cos, sin, rot_dim, ctx, kv, write,
                      adjacent=False):
        m, width = qkv.shape
        need = (n_heads + (2 * n_kv if write else 0)) * hd
        if width != need:
            raise KernelError("rope_kv_write: rows are %d wide, expected %d" % (width, need))
        self._dev(qkv, "qkv")
        if m != ctx.n_tokens:
            raise KernelError("rope_kv_write: %d rows for a step of %d tokens" % (m, ctx.n_tokens))
        cptr = sptr = None
        if rot_dim:
            if cos is None or cos.shape[1] != rot_dim // 2 or cos.shape != sin.shape:
                raise KernelError("rope_kv_write: rotary tables do not match rot_dim %d" % rot_dim)
            if not ctx.captured and ctx.max_ctx > cos.shape[0]:
                raise KernelError("rope_kv_write: position %d exceeds the rotary table of %d rows"
                                  % (ctx.max_ctx - 1, cos.shape[0]))
            cptr, sptr = self._dev(cos, "cos", torch.float32), self._dev(sin, "sin", torch.float32)
        bptr = None
        if bias is not None:
            bptr = self._dev(bias, "qkv bias", torch.float32)
            if bias.shape[0] < need:
                raise KernelError("rope_kv_write: the bias is shorter than a row")
        kptr = vptr = tptr = None
        stride = 0
        if write:
            k_pages, v_pages = self._kv_planes(kv, n_kv, hd, qkv.dtype)
            kptr, vptr, tptr = k_pages.data_ptr(), v_pages.data_ptr(), kv.block_table.data_ptr()
            stride = kv.block_table.shape[1]
        self._check(self.lib.llm_rope_kv_write(
            qkv.data_ptr(), _code(qkv.dtype), width, bptr, n_heads, n_kv, hd, cptr, sptr, rot_dim,
            ctx.tok_pos.data_ptr(), ctx.tok_seq.data_ptr(), ctx.seq_slot.data_ptr(), tptr, stride,
            kptr, vptr, 64, 1 if write else 0, 1 if adjacent else 0, m, self._stream()), "rope_kv_write")

    def _kv_planes(self, kv, n_kv, hd, dtype):
        """The planes of keys and values that the attention kernels read and write, checked: the
        cache entry holds planes "k" and "v" in the layouts of ``parts/kv_pages.py``, for these
        head counts and sizes, in the activations' dtype, with a page table beside them."""
        if kv is None:
            raise KernelError("this layer has no cache entry")
        for name, layout in (("k", K_LAYOUT), ("v", V_LAYOUT)):
            plane = kv.need.plane(name) if kv.need is not None else None
            if name not in kv.planes or plane is None:
                raise KernelError("attention needs a cache entry with planes \"k\" and \"v\"; this one has: %s"
                                  % (", ".join(sorted(kv.planes)) or "none"))
            if plane.layout != layout:
                raise KernelError("plane %r is laid out as %r, the attention kernels read %r" % (name, plane.layout, layout))
        if kv.page_size != 64:
            raise KernelError("the attention kernels read pages of 64 positions, not %d" % kv.page_size)
        k_pages, v_pages = kv.planes["k"], kv.planes["v"]
        shape, vshape = tuple(k_pages.shape), tuple(v_pages.shape)
        want = key_pages_shape(shape[0] if shape else 0, n_kv, hd)
        vwant = value_pages_shape(shape[0] if shape else 0, n_kv, hd)
        if shape != want or vshape != vwant:
            raise KernelError("cache pages have shapes %s / %s, expected %s and %s" % (shape, vshape, want, vwant))
        if k_pages.dtype != dtype or v_pages.dtype != dtype:
            raise KernelError("cache dtype %s differs from the activations' %s" % (k_pages.dtype, dtype))
        self._dev(k_pages, "key pages")
        self._dev(v_pages, "value pages")
        self._dev(kv.block_table, "page table", torch.int32)
        return k_pages, v_pages

    def attention(self, qkv, n_heads, n_kv, hd, ctx, kv, scale, window):
        m, width = qkv.shape
        if width < n_heads * hd:
            raise KernelError("attention: rows are %d wide, queries need %d" % (width, n_heads * hd))
        if n_heads % n_kv:
            raise KernelError("attention: %d heads are not a multiple of %d kv heads" % (n_heads, n_kv))
        if hd > 256:
            raise KernelError("attention: head_dim %d above 256 is not supported" % hd)
        k_pages, v_pages = self._kv_planes(kv, n_kv, hd, qkv.dtype)
        out = torch.empty((m, n_heads * hd), dtype=qkv.dtype, device=self.device)
        table = kv.block_table
        if (self.fast_attention and qkv.dtype == torch.bfloat16 and width % 8 == 0
                and self.lib.llm_attention_mfma_supported(hd)):
            if ctx.decode:
                if m != ctx.n_seqs:
                    raise KernelError("attention: a decode step has one row per sequence")
                pages = (ctx.max_ctx + 63) // 64
                if window:
                    pages = min(pages, window // 64 + 2)
                waves = self.lib.llm_attention_decode_waves(hd)
                # a page for each wave, as long as the grid stays within two or three blocks a
                # compute unit; the kernel gives every wave ceil(pages / waves) pages in a row, so
                # blocks beyond ceil(pages / (that * waves)) would get none: they are not launched
                budget = self.DECODE_BLOCKS
                ahead = self.DECODE_BLOCKS_AHEAD // (m * n_kv) * (m * n_kv)      # blocks the smaller grid would have
                if (hd <= 128 and pages * m * n_kv >= self.DECODE_AHEAD_PAGES * self.DECODE_BLOCKS_AHEAD * waves
                        and ahead * 16 >= self.DECODE_BLOCKS_AHEAD * 15):
                    budget = self.DECODE_BLOCKS_AHEAD
                n_blocks = max(1, min(-(-pages // waves), max(1, budget // (m * n_kv))))
                per_wave = -(-pages // (n_blocks * waves))
                n_blocks = -(-pages // (per_wave * waves))
                by_length = 0
                if getattr(ctx, "unequal", False) and m > 1:
                    # lengths that differ widely: the kernel deals the pages out by the lengths it
                    # finds in device memory, within so many blocks (and one more a pair at most)
                    by_length, n_blocks = self.DECODE_BLOCKS, 1
                    chunks = by_length + m * n_kv
                    part_o = torch.empty((chunks, n_heads // n_kv, hd), dtype=torch.float32, device=self.device)
                    part_ml = torch.empty((chunks, n_heads // n_kv, 2), dtype=torch.float32, device=self.device)
                else:
                    part_o = torch.empty((m, n_heads, n_blocks, hd), dtype=torch.float32, device=self.device)
                    part_ml = torch.empty((m, n_heads, n_blocks, 2), dtype=torch.float32, device=self.device)
                self._check(self.lib.llm_attention_decode_bf16(
                    qkv.data_ptr(), width, k_pages.data_ptr(), v_pages.data_ptr(),
                    table.data_ptr(), table.shape[1], 64, ctx.seq_slot.data_ptr(),
                    ctx.seq_pos0.data_ptr(), part_o.data_ptr(), part_ml.data_ptr(), out.data_ptr(), m, n_heads, n_kv, hd, float(scale),
                    int(window), n_blocks, by_length, self._stream()), "attention_decode_bf16")
            else:
                tiles = self.prompt_tiles
                if not tiles:
                    tiles = 2 if hd <= 128 and ctx.max_new >= self.PROMPT_TILE_ROWS[0 if hd <= 64 else 1] else 1
                self._check(self.lib.llm_attention_prefill_bf16(
                    qkv.data_ptr(), width, k_pages.data_ptr(), v_pages.data_ptr(),
                    table.data_ptr(), table.shape[1], 64, ctx.seq_start.data_ptr(),
                    ctx.seq_slot.data_ptr(), ctx.seq_pos0.data_ptr(), out.data_ptr(), ctx.n_seqs,
                    ctx.max_new, n_heads, n_kv, hd, float(scale), int(window), tiles, self._stream()),
                    "attention_prefill_bf16")
            return out
        self._check(self.lib.llm_attention_ref(
            qkv.data_ptr(), _code(qkv.dtype), width, k_pages.data_ptr(), v_pages.data_ptr(),
            kv.block_table.data_ptr(), kv.block_table.shape[1], 64, ctx.tok_pos.data_ptr(),
            ctx.tok_seq.data_ptr(), ctx.seq_slot.data_ptr(), out.data_ptr(), m, n_heads, n_kv, hd,
            float(scale), int(window), self._stream()), "attention")
        return out

    def measured_peaks(self, nbytes: int = 2 << 30, reps: int = 5):
        """What this GPU reaches at most, by kernels of this library timed with events (the best of
        ``reps`` runs after one to warm up, and for the memory kernels the best of several grid
        sizes): {"read_GBs": a read of ``nbytes``, "copy_GBs": a copy of them (bytes read plus
        bytes written), "bf16_TFs": a loop of matrix-core instructions on registers, "fp32_TFs": a
        loop of float32 multiply-adds in the vector units}."""
        src = torch.empty(nbytes, dtype=torch.uint8, device=self.device).fill_(1)
        dst = torch.empty_like(src)
        sink = torch.empty(self.lib.llm_peak_sink_words(), dtype=torch.int32, device=self.device)
        flops = ctypes.c_double(0.0)

        def best(launch):
            times = []
            for r in range(reps + 1):
                t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                t0.record()
                self._check(launch(), "peak measurement")
                t1.record()
                t1.synchronize()
                if r:
                    times.append(t0.elapsed_time(t1) * 1e-3)
            return min(times)
        out = {}
        grids = (2, 3, 4, 6, 16)        # blocks for every two compute units
        t = min(best(lambda g=g, nt=nt: self.lib.llm_peak_read(src.data_ptr(), nbytes, sink.data_ptr(), g, nt,
                                                               self._stream()))
                for g in grids for nt in (0, 1))
        out["read_GBs"] = nbytes / t / 1e9
        t = min(best(lambda g=g: self.lib.llm_peak_copy(src.data_ptr(), dst.data_ptr(), nbytes, g, self._stream()))
                for g in grids)
        out["copy_GBs"] = 2 * nbytes / t / 1e9
        t = best(lambda: self.lib.llm_peak_mfma_bf16(sink.data_ptr(), 20000, ctypes.byref(flops), self._stream()))
        out["bf16_TFs"] = flops.value / t / 1e12
        t = best(lambda: self.lib.llm_peak_fma_f32(sink.data_ptr(), 20000, ctypes.byref(flops), self._stream()))
        out["fp32_TFs"] = flops.value / t / 1e12
        return out

    def argmax(self, logits):
        r, v = logits.shape
        self._dev(logits, "logits", torch.float32)
        out = torch.empty((r,), dtype=torch.int32, device=self.device)
        parts = self.lib.llm_argmax_parts(v)
        part_val = torch.empty((r * parts,), dtype=torch.float32, device=self.device)
        part_idx = torch.empty((r * parts,), dtype=torch.int32, device=self.device)
        self._check(self.lib.llm_argmax(logits.data_ptr(), out.data_ptr(), part_val.data_ptr(),
                                        part_idx.data_ptr(), r, v, self._stream()), "argmax")
        return out

    def sample(self, logits, temperature, top_k, top_p, seed, streams: List[int], counters: List[int]):
        r, v = logits.shape
        self._dev(logits, "logits", torch.float32)
        if len(streams) != r or len(counters) != r:
            raise KernelError("sample: one stream and counter per row are needed")
        # through pinned memory and without waiting: a copy from pageable memory holds the host
        # until the stream gets to it, and the step after this one could not be queued meanwhile
        keys = torch.tensor([streams, counters], dtype=torch.int64).pin_memory().to(self.device, non_blocking=True)
        out = torch.empty((r,), dtype=torch.int32, device=self.device)
        parts = self.lib.llm_sample_parts(v)
        # (no limit on the candidates and top_p below 1: the kernel first tries the most probable 1,024)
        k_part = self.lib.llm_sample_k_part(v, int(top_k) if (top_k or top_p >= 1.0) else min(v, 1024))
        part_max = torch.empty((r * parts,), dtype=torch.float32, device=self.device)
        part_sum = torch.empty((r * parts,), dtype=torch.float32, device=self.device)
        cand = torch.empty((max(1, r * parts * k_part),), dtype=torch.int64, device=self.device)
        self._check(self.lib.llm_sample(logits.data_ptr(), out.data_ptr(), r, v, float(temperature),
                                        int(top_k), float(top_p), int(seed) & (2**64 - 1),
                                        keys[0].data_ptr(), keys[1].data_ptr(), part_max.data_ptr(),
                                        part_sum.data_ptr(), cand.data_ptr(), self._stream()), "sample")
        return out
