"""The kernel library as Python calls on torch tensors.

Every method checks shapes and dtypes on the host, then enqueues hand-written
gfx950 kernels from the HIP library on torch's current stream. There is no
other implementation behind these calls: if the library cannot be built or
loaded, `load_ops` raises.
"""
from __future__ import annotations

import ctypes
import weakref
from typing import Optional

import torch

from .build import ensure_built

_c_int_p = ctypes.c_void_p
_DT = {torch.float32: 0, torch.bfloat16: 1}


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


class KernelError(RuntimeError):
    """The kernel library refused a call (bad size, dtype or launch)."""


class _GemmArgs(ctypes.Structure):
    _fields_ = [("A", ctypes.c_void_p), ("W", ctypes.c_void_p), ("C", ctypes.c_void_p),
                ("bias", ctypes.c_void_p), ("offsets", ctypes.c_void_p),
                ("a_index", ctypes.c_void_p), ("c_index", ctypes.c_void_p),
                ("tiles16", ctypes.c_void_p), ("tiles_big", ctypes.c_void_p),
                ("tile_counts", ctypes.c_void_p), ("w_group_stride", ctypes.c_int64),
                ("M", ctypes.c_int), ("N", ctypes.c_int), ("K", ctypes.c_int),
                ("lda", ctypes.c_int), ("ldc", ctypes.c_int), ("groups", ctypes.c_int),
                ("a_div", ctypes.c_int), ("in_dtype", ctypes.c_int), ("out_dtype", ctypes.c_int),
                ("epilogue", ctypes.c_int),
                ("k_parts", ctypes.c_int), ("workspace", ctypes.c_void_p),
                ("workspace_floats", ctypes.c_int64), ("split_min_bytes", ctypes.c_int64),
                ("force_kernel", ctypes.c_int), ("skinny_two", ctypes.c_int),
                ("act_limit", ctypes.c_float), ("act_alpha", ctypes.c_float)]


class _RouteArgs(ctypes.Structure):
    _fields_ = [("ids", ctypes.c_void_p), ("wts", ctypes.c_void_p), ("offsets", ctypes.c_void_p),
                ("order", ctypes.c_void_p), ("tiles16", ctypes.c_void_p),
                ("tiles_big", ctypes.c_void_p), ("tile_counts", ctypes.c_void_p),
                ("choice_bias", ctypes.c_void_p), ("parts", ctypes.c_void_p),
                ("E", ctypes.c_int), ("k", ctypes.c_int), ("renorm", ctypes.c_int),
                ("score", ctypes.c_int), ("scale", ctypes.c_float), ("n_group", ctypes.c_int),
                ("topk_group", ctypes.c_int), ("group_top", ctypes.c_int),
                ("renorm_eps", ctypes.c_float), ("weightless", ctypes.c_int)]


BIG_TILE_ROWS = 256   # rows of a tall tile of the grouped products (the library's kGroupedTileRows)
ROUTE_ROWS_PER_BLOCK = 1024  # the library's kAlignRowsPerBlock
# rows (tokens) from which the grouping runs as several blocks side by side: 12.5 against 13 us
# at 2,048 rows of 60 experts top-4 (11 against 10 at 1,024), 19 against 37 at 8,192, 46 against 127
# at 32,768
ROUTE_MANY_MIN_ROWS = 2048
_SCORES = {"softmax": 0, "sigmoid": 1}
# activations of a gated product, by the names config.json gives them -> the library's epilogue
# ('clamped_swish': g sigmoid(alpha g) (u + 1) with g cut at a limit from above and u to
# [-limit, limit]; the limit and alpha travel with the call)
GATE_ACTS = {"silu": 1, "gelu_pytorch_tanh": 2, "clamped_swish": 4}
# ... and of a plain product: none, or the square of relu on every output
UNGATED_ACTS = {None: 0, "relu2": 3}


class _AttnArgs(ctypes.Structure):
    _fields_ = [("q", ctypes.c_void_p), ("kpool", ctypes.c_void_p), ("vpool", ctypes.c_void_p),
                ("out", ctypes.c_void_p), ("block_table", ctypes.c_void_p),
                ("positions", ctypes.c_void_p), ("row_seq", ctypes.c_void_p),
                ("seq_row_start", ctypes.c_void_p), ("seq_qlen", ctypes.c_void_p),
                ("seq_pos0", ctypes.c_void_p), ("workspace", ctypes.c_void_p),
                ("workspace_floats", ctypes.c_int64),
                ("q_stride", ctypes.c_int), ("bt_stride", ctypes.c_int), ("T", ctypes.c_int),
                ("S", ctypes.c_int), ("Hq", ctypes.c_int), ("Hkv", ctypes.c_int),
                ("D", ctypes.c_int), ("page_size", ctypes.c_int), ("window", ctypes.c_int),
                ("scale", ctypes.c_float), ("dtype", ctypes.c_int), ("max_qlen", ctypes.c_int),
                ("max_kv_len", ctypes.c_int), ("single_rows", ctypes.c_int),
                ("slopes", ctypes.c_void_p), ("Dv", ctypes.c_int), ("sink", ctypes.c_int)]


class _QkvConvArgs(ctypes.Structure):
    _fields_ = [("u", ctypes.c_void_p), ("w", ctypes.c_void_p), ("wt", ctypes.c_void_p),
                ("state", ctypes.c_void_p),
                ("state_stride", ctypes.c_int64), ("q_out", ctypes.c_void_p),
                ("kpool", ctypes.c_void_p), ("vpool", ctypes.c_void_p),
                ("block_table", ctypes.c_void_p), ("positions", ctypes.c_void_p),
                ("row_seq", ctypes.c_void_p), ("seq_row_start", ctypes.c_void_p),
                ("seq_slots", ctypes.c_void_p), ("q_gain", ctypes.c_void_p),
                ("k_gain", ctypes.c_void_p), ("inv_freq", ctypes.c_void_p),
                ("bt_stride", ctypes.c_int), ("T", ctypes.c_int), ("S", ctypes.c_int),
                ("Hq", ctypes.c_int), ("Hkv", ctypes.c_int), ("dim", ctypes.c_int),
                ("vdim", ctypes.c_int), ("taps", ctypes.c_int), ("rot_dim", ctypes.c_int),
                ("interleaved", ctypes.c_int), ("page_size", ctypes.c_int),
                ("dtype", ctypes.c_int), ("eps", ctypes.c_float), ("all_single", ctypes.c_int),
                ("force_plain", ctypes.c_int)]


class _QkvRopeArgs(ctypes.Structure):
    _fields_ = [("x", ctypes.c_void_p), ("w", ctypes.c_void_p), ("bias", ctypes.c_void_p),
                ("qkv", ctypes.c_void_p), ("positions", ctypes.c_void_p),
                ("row_seq", ctypes.c_void_p), ("inv_freq", ctypes.c_void_p),
                ("kpool", ctypes.c_void_p), ("vpool", ctypes.c_void_p),
                ("block_table", ctypes.c_void_p), ("T", ctypes.c_int), ("K", ctypes.c_int),
                ("lda", ctypes.c_int), ("Hq", ctypes.c_int), ("Hkv", ctypes.c_int),
                ("D", ctypes.c_int), ("bt_stride", ctypes.c_int), ("page_size", ctypes.c_int),
                ("write_kv", ctypes.c_int)]


class _LatentArgs(ctypes.Structure):
    _fields_ = [("dkv", ctypes.c_void_p), ("q", ctypes.c_void_p), ("q_abs", ctypes.c_void_p),
                ("pool", ctypes.c_void_p), ("out", ctypes.c_void_p), ("gate", ctypes.c_void_p),
                ("norm_w", ctypes.c_void_p), ("freq", ctypes.c_void_p),
                ("block_table", ctypes.c_void_p), ("positions", ctypes.c_void_p),
                ("row_seq", ctypes.c_void_p), ("seq_row_start", ctypes.c_void_p),
                ("seq_pos0", ctypes.c_void_p), ("workspace", ctypes.c_void_p),
                ("workspace_floats", ctypes.c_longlong), ("S", ctypes.c_int),
                ("max_kv_len", ctypes.c_int), ("max_qlen", ctypes.c_int),
                ("force_plain", ctypes.c_int),
                ("dkv_stride", ctypes.c_int),
                ("gate_stride", ctypes.c_int), ("bt_stride", ctypes.c_int), ("T", ctypes.c_int),
                ("Hq", ctypes.c_int), ("dim", ctypes.c_int), ("R", ctypes.c_int),
                ("rd", ctypes.c_int), ("rot_n", ctypes.c_int), ("page_size", ctypes.c_int),
                ("window", ctypes.c_int), ("write_kv", ctypes.c_int), ("dtype", ctypes.c_int),
                ("eps", ctypes.c_float), ("magnitude", ctypes.c_float), ("scale", ctypes.c_float),
                ("interleaved", ctypes.c_int)]


class _DiffAttnArgs(ctypes.Structure):
    _fields_ = [("qkv", ctypes.c_void_p), ("kpool", ctypes.c_void_p), ("vpool", ctypes.c_void_p),
                ("out", ctypes.c_void_p), ("block_table", ctypes.c_void_p),
                ("positions", ctypes.c_void_p), ("row_seq", ctypes.c_void_p),
                ("seq_row_start", ctypes.c_void_p), ("workspace", ctypes.c_void_p),
                ("workspace_floats", ctypes.c_int64), ("q_stride", ctypes.c_int),
                ("bt_stride", ctypes.c_int), ("T", ctypes.c_int), ("S", ctypes.c_int),
                ("Hq", ctypes.c_int), ("Hkv", ctypes.c_int), ("dim", ctypes.c_int),
                ("vdim", ctypes.c_int), ("page_size", ctypes.c_int), ("dtype", ctypes.c_int),
                ("max_qlen", ctypes.c_int), ("max_kv_len", ctypes.c_int),
                ("force_plain", ctypes.c_int), ("single_rows", ctypes.c_int),
                ("scale", ctypes.c_float), ("cap", ctypes.c_float),
                ("t_coef", ctypes.c_float), ("t_every", ctypes.c_int), ("lam", ctypes.c_float),
                ("eps", ctypes.c_float), ("out_scale", ctypes.c_float)]


class _SigAttnArgs(ctypes.Structure):
    _fields_ = [("qkv", ctypes.c_void_p), ("kpool", ctypes.c_void_p), ("vpool", ctypes.c_void_p),
                ("out", ctypes.c_void_p), ("block_table", ctypes.c_void_p),
                ("positions", ctypes.c_void_p), ("row_seq", ctypes.c_void_p),
                ("seq_row_start", ctypes.c_void_p), ("head_bias", ctypes.c_void_p),
                ("mix", ctypes.c_void_p), ("workspace", ctypes.c_void_p),
                ("workspace_floats", ctypes.c_int64),
                ("q_stride", ctypes.c_int), ("bt_stride", ctypes.c_int), ("T", ctypes.c_int),
                ("S", ctypes.c_int), ("Hq", ctypes.c_int), ("Hkv", ctypes.c_int),
                ("dim", ctypes.c_int), ("vdim", ctypes.c_int), ("page_size", ctypes.c_int),
                ("dtype", ctypes.c_int), ("max_qlen", ctypes.c_int), ("max_kv_len", ctypes.c_int),
                ("chunk", ctypes.c_int), ("force_plain", ctypes.c_int),
                ("single_rows", ctypes.c_int), ("scale", ctypes.c_float)]


class _GatedSumArgs(ctypes.Structure):
    _fields_ = [("residual", ctypes.c_void_p), ("a", ctypes.c_void_p), ("g1", ctypes.c_void_p),
                ("b1", ctypes.c_void_p), ("dense", ctypes.c_void_p), ("y", ctypes.c_void_p),
                ("w", ctypes.c_void_p), ("ids", ctypes.c_void_p), ("xin", ctypes.c_void_p),
                ("g2", ctypes.c_void_p), ("b2", ctypes.c_void_p),
                ("T", ctypes.c_int), ("H", ctypes.c_int), ("k", ctypes.c_int),
                ("real", ctypes.c_int), ("dtype", ctypes.c_int), ("mult", ctypes.c_float)]


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelError(msg)


def _dev(t: torch.Tensor, name: str, dtype=None, dims: Optional[int] = None) -> None:
    if t.is_cuda and t.is_contiguous() and (dtype is None or t.dtype == dtype) \
            and (dims is None or t.dim() == dims):
        return   # (a step makes about a thousand of these checks: the good case is one test)
    _need(t.is_cuda, f"{name} must be on the GPU")
    _need(t.is_contiguous(), f"{name} must be contiguous")
    if dtype is not None:
        _need(t.dtype == dtype, f"{name} must be {dtype}, is {t.dtype}")
    if dims is not None:
        _need(t.dim() == dims, f"{name} must have {dims} dimensions, has {t.dim()}")


class _Together:
    def __init__(self, ops):
        self.ops = ops

    def __enter__(self):
        if self.ops._held is not None:
            raise KernelError("together(): already inside one")
        self.ops._held = []
        self.ops._held_route = None
        return self

    def __exit__(self, exc_type, exc, tb):
        held, self.ops._held = self.ops._held, None
        route, self.ops._held_route = self.ops._held_route, None
        if exc_type is None:
            self.ops._launch_held(held, route)
        return False


class _Beside:
    """Work on a second stream that starts after everything the current stream has been
    given so far; `HipOps.join()` makes the current stream wait for it. The two events are
    made once and recorded again every time (an event's earlier waits keep their meaning);
    a record and its wait are one call into the library (with torch's event and stream
    objects a block cost the host some 100 us, half of a layer's launches).

    Memory: tensors made inside the block come from the second stream's part of torch's
    allocator and are read on the main stream after `join()` without `record_stream`. That
    holds because the second stream is used inside such blocks only, and every block begins
    by waiting for an event recorded on the main stream at its entry: a tensor of an earlier
    block that the main stream has been told to read is read before any later block's work
    can write into memory the allocator has handed out again."""

    def __init__(self, ops):
        self.ops = ops

    def __enter__(self):
        ops = self.ops
        if ops._side is None:
            ops._side = torch.cuda.Stream()   # default priority
            ops._side_events = (ops._new_event(), ops._new_event())
        raw = ops._stream().value or 0
        if ops._main is None or ops._main.cuda_stream != raw:
            ops._main = torch.cuda.current_stream()   # the object is kept: making one costs
        if ops._side_open:   # a block that nobody joined (a step that failed half-way): join it now
            ops.join()
        ops._ok(ops.lib.ninfer_stream_after(ops._side.cuda_stream, raw, ops._side_events[0]))
        torch.cuda.set_stream(ops._side)
        return self

    def __exit__(self, exc_type, exc, tb):
        # nothing is given to the second stream outside such blocks: the event that marks the
        # block's end is recorded by `join()`, together with the wait for it
        torch.cuda.set_stream(self.ops._main)
        self.ops._side_open = True
        return False


class _Tuned:
    def __init__(self, ops, values):
        self.ops, self.values = ops, values

    def __enter__(self):
        self.saved = dict(self.ops._tune)
        self.ops._tune.update(self.values)
        return self.ops

    def __exit__(self, *exc):
        self.ops._tune = self.saved
        return False


class HipOps:
    def __init__(self, lib_path: Optional[str] = None):
        self.lib_path = lib_path or ensure_built()
        self.lib = ctypes.CDLL(self.lib_path)
        self.lib.ninfer_last_error.restype = ctypes.c_char_p
        self.lib.ninfer_attention_workspace_floats.restype = ctypes.c_longlong
        self.lib.ninfer_event_create.restype = ctypes.c_void_p
        self.lib.ninfer_stream_after.argtypes = [ctypes.c_void_p] * 3
        self.lib.ninfer_sample_few_places.restype = ctypes.c_longlong
        self.lib.ninfer_latent_attention_workspace_floats.restype = ctypes.c_longlong
        self.lib.ninfer_diff_attention_workspace_floats.restype = ctypes.c_longlong
        self.lib.ninfer_sigmoid_attention_workspace_floats.restype = ctypes.c_longlong
        self.force_generic = False  # tests: run the plain kernels whatever the shape
        self._device_index = None   # the one GPU's index, asked for at the first launch
        self._held = None           # products held back inside `together()`
        self._held_route = None     # ... and a routing by the logits one of them writes
        self._side = None           # the second stream of `beside()`, made at first use
        self._side_events = None    # (start, end) of the `beside()` block
        self._side_open = False     # a `beside()` block that `join()` has not waited for
        self._main = None           # the stream that the last `beside()` block left and returns to
        # rows from which independent work is worth a second stream (with fewer rows the
        # products on it lose more by sharing the units than the step gains: the smaller
        # model's portion of 256 tokens 7.6 ms with it, 6.6 without; 512 tokens 7.5 against 7.8,
        # 1,024 9.5 against 10.3, 2,048 13.6 against 15.0; the two waits between the streams
        # alone cost 0.1 to 0.2 ms a step)
        self.beside_min_rows = 512
        # ... and from far fewer rows where the work on the second stream reads a lot of
        # weights, so that it is long whatever the rows (a shared expert of 440 MB beside 64
        # experts of 55 MB: 64 rows 20.8 against 21.0 ms, 128 rows 21.6 against 22.6, 256 rows
        # 23.4 against 25.1, 448 rows 26.2 against 29.8; the smaller model's 69 MB beside 60
        # experts of 17 MB: 128 to 448 rows 7.6 to 7.8 ms with it, 5.6 to 7.5 without)
        # (65: a decode step of up to 64 rows takes the same kernels run eagerly and captured)
        self.beside_heavy_min_rows = 65
        self.beside_heavy_bytes = 256 << 20
        self.conv_pieces_always = False     # tests: qkv_conv's kernel of whole pieces at every row count
        self.gla_chunk_min_rows = 8         # the same for gated linear attention
        self.lightning_chunk_min_rows = 8   # a step's longest portion from which lightning attention runs in chunks
        self.library_min_rows = 32  # dense bf16 products with more rows go to the library
        self.rows_kernel_max = 64   # ... unless the kernel for 33 to 64 rows takes them
        self.rows_kernel_features = (4096, 32768)   # (gemm_skinny_rows.hip: where it beats the library)
        # ... but never a SwiGLU's gate/up product: the tile kernels here have the activation in
        # their epilogue, which beats the library's product followed by a kernel for the
        # activation at every row count (70 against 98 us at 64 rows of 40960 x 3584; whole
        # prompt portions of 256 to 8,192 tokens 2 to 4% faster at 2048 -> 2 x 5632, the same
        # within 1% at 3584 -> 2 x 20480)
        self.split_max_rows = 512   # most rows of a product that may be cut along K (gemm_split)
        # a plain product of at most this many rows runs on the tile kernel here when it is on
        # the second stream: the library's product there took the 512-token portion 7.25 ms in
        # some processes and 8.2 in others (7.5 to 7.8 with the tile kernel in all of them),
        # 576 tokens 8.17 against 7.9, 640 tokens 8.05 to 8.2 against 8.0; from 704 rows the same.
        # That product's weights are 23 MB; with 147 MB (3584 x 20480) the library's is the
        # faster one there too (64 to 640 rows: steps up to 3% shorter), hence the second bound
        self.side_own_max_rows = 640
        self.side_own_max_bytes = 64 << 20
        self._attn_ws = None
        self._outgrown = []     # workspaces that captured graphs may still point to
        self._split_ws = None   # 32 MB of 32-bit scratch for products cut along K, made at first use
        # what tests and measurements ask of the product kernels (see `tuned`); all 0: the
        # library chooses
        self._tune = {"force_kernel": 0, "split_min_bytes": 0, "skinny_two": 0}
        # runners whose captured graphs may hold workspace addresses (held weakly: a runner
        # that is simply dropped leaves the set by itself)
        self._graph_holders = weakref.WeakSet()

    def graph_holder_new(self, runner) -> None:
        self._graph_holders.add(runner)

    def graph_holder_gone(self, runner) -> None:
        """A runner with captured graphs has dropped them. When no other is left, nothing can
        replay into the workspaces any more: they are given back (the next call that needs
        one makes it anew)."""
        self._graph_holders.discard(runner)
        if len(self._graph_holders) == 0:
            self._outgrown = []
            self._attn_ws = None
            self._split_ws = None

    def tuned(self, **values):
        """Context manager for tests and measurements: inside it every product call carries
        these choices (force_kernel: 1, 2, 3 = many-row tiles of 64, 128, 256 rows;
        split_min_bytes: least bytes of weights for a cut along K;
        skinny_two: 1 / -1 = two feature sets per block whenever possible / never). They
        travel with each call; the library keeps no such state."""
        unknown = set(values) - set(self._tune)
        if unknown:
            raise KernelError(f"tuned(): unknown choices {sorted(unknown)}")
        return _Tuned(self, values)

    # ---- helpers ----------------------------------------------------------------
    def _stream(self) -> ctypes.c_void_p:
        # the current stream's handle, asked for with every launch: torch's own short way to it
        # where this build has one (a tenth of the time of making a Stream object)
        if _raw_stream is not None:
            if self._device_index is None:
                self._device_index = torch.cuda.current_device()
            return ctypes.c_void_p(_raw_stream(self._device_index))
        return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def _ok(self, rc: int) -> None:
        if rc != 0:
            raise KernelError(self.lib.ninfer_last_error().decode())

    def device_info(self):
        cu, lds = ctypes.c_int(), ctypes.c_int()
        arch = ctypes.create_string_buffer(128)
        self._ok(self.lib.ninfer_device_info(ctypes.byref(cu), ctypes.byref(lds), arch, 128))
        return {"cu_count": cu.value, "lds_bytes": lds.value, "arch": arch.value.decode()}

    # ---- fills --------------------------------------------------------------------
    def fill_nan_pages(self, pool, pages):
        """NaN into every number of the given pages of a pool [pages, ...] (debugging:
        pages that were given back)."""
        _dev(pool, "pool")
        _dev(pages, "pages", torch.int32, 1)
        _need(pool.dtype in _DT, f"fill_nan_pages: pool of {pool.dtype}")
        per_page = pool.numel() // pool.shape[0]
        self._ok(self.lib.ninfer_fill_nan_pages(
            ctypes.c_void_p(pool.data_ptr()), ctypes.c_void_p(pages.data_ptr()), pages.shape[0],
            pool.shape[0], ctypes.c_longlong(per_page), _DT[pool.dtype], self._stream()))

    def fill_random(self, out, key, std, mean=0.0):
        """out[i] = mean + std * z(key, i), z an approximately normal number that is a pure
        function of the 64-bit key and the flat index (see weights/counter_random.py, which
        computes the same bits on the host)."""
        _dev(out, "out")
        _need(out.dtype in _DT, f"fill_random: tensor of {out.dtype}")
        self._ok(self.lib.ninfer_fill_random(
            ctypes.c_void_p(out.data_ptr()), ctypes.c_longlong(out.numel()),
            ctypes.c_ulonglong(key & ((1 << 64) - 1)), ctypes.c_float(std), ctypes.c_float(mean),
            _DT[out.dtype], self._stream()))

    def read_probe(self, t):
        """Streams the tensor's bytes through a kernel that only reads (measurements: the rate
        of a plain read of HBM)."""
        _dev(t, "t")
        self._ok(self.lib.ninfer_read_probe(ctypes.c_void_p(t.data_ptr()),
                                            ctypes.c_longlong(t.numel() * t.element_size()),
                                            self._stream()))

    # ---- row-wise ---------------------------------------------------------------
    def embed(self, tokens, table, out, positions=None, pos_table=None):
        """out[t] = table[tokens[t]] (+ pos_table[positions[t]]: learned absolute positions),
        in 32-bit."""
        _dev(tokens, "tokens", torch.int32, 1)
        _dev(table, "table", dims=2)
        _dev(out, "out", torch.float32, 2)
        _need(out.shape == (tokens.shape[0], table.shape[1]), "embed: out has the wrong shape")
        if pos_table is not None:
            _dev(pos_table, "pos_table", table.dtype, 2)
            _need(positions is not None, "embed: a table of positions needs the rows' positions")
            _dev(positions, "positions", torch.int32, 1)
            _need(pos_table.shape[1] == table.shape[1] and positions.shape[0] == tokens.shape[0],
                  "embed: the table of positions or the positions have the wrong shape")
        self._ok(self.lib.ninfer_embed(
            ctypes.c_void_p(tokens.data_ptr()), ctypes.c_void_p(table.data_ptr()),
            ctypes.c_void_p(out.data_ptr()), tokens.shape[0], table.shape[1], _DT[table.dtype],
            ctypes.c_void_p(_ptr(positions) if pos_table is not None else None),
            ctypes.c_void_p(_ptr(pos_table)), 0 if pos_table is None else pos_table.shape[0],
            self._stream()))

    def rmsnorm(self, x, gain, eps, out, delta=None, rows=None, rows_sum=None, center=False):
        """out = norm(x [+ delta] [+ rows_sum]); `rows_sum` is a weighted sum of
        rows (an object with y, weights, shared, gate) added on the fly. norm(v) =
        v rsqrt(mean(v^2) + eps) gain, or with `center` the layer norm without a bias,
        (v - mean(v)) rsqrt(mean((v - mean(v))^2) + eps) gain."""
        _dev(x, "x", torch.float32, 2)
        _dev(gain, "gain", torch.float32, 1)
        _dev(out, "out", dims=2)
        h = x.shape[1]
        _need(gain.shape[0] == h and out.shape[1] == h, "rmsnorm: widths differ")
        if delta is not None:
            _dev(delta, "delta", out.dtype, 2)
            _need(delta.shape == x.shape, "rmsnorm: delta has the wrong shape")
        if rows is not None:
            _dev(rows, "rows", torch.int32, 1)
            _need(out.shape[0] == rows.shape[0], "rmsnorm: out has the wrong number of rows")
        else:
            _need(out.shape[0] == x.shape[0], "rmsnorm: out has the wrong number of rows")
        my, mw, msh, mg, mgs, mk = None, None, None, None, 0, 0
        if rows_sum is not None:
            mk, mgs = self._check_rows_sum(rows_sum, x.shape[0], h, out.dtype)
            my, mw = rows_sum.y.data_ptr(), rows_sum.weights.data_ptr()
            msh, mg = _ptr(rows_sum.shared), _ptr(rows_sum.gate)
        self._ok(self.lib.ninfer_rmsnorm(
            ctypes.c_void_p(x.data_ptr()), ctypes.c_void_p(_ptr(delta)),
            ctypes.c_void_p(gain.data_ptr()), ctypes.c_void_p(out.data_ptr()),
            ctypes.c_void_p(_ptr(rows)), out.shape[0], h, ctypes.c_float(eps), _DT[out.dtype],
            ctypes.c_void_p(my), ctypes.c_void_p(mw), ctypes.c_void_p(msh), ctypes.c_void_p(mg),
            mgs, mk, 1 if center else 0, self._stream()))

    @staticmethod
    def _check_rows_sum(rs, t, h, dtype):
        _need(getattr(rs, "ids", None) is None, "row sum: rows of experts that hand their input "
              "back are added by gated_sum_add only")
        _dev(rs.y, "y", dtype, 2)
        _dev(rs.weights, "weights", torch.float32, 2)
        k = rs.weights.shape[1]
        _need(rs.weights.shape[0] == t and rs.y.shape == (t * k, h), "row sum: shapes differ")
        stride = 0
        if rs.shared is not None:
            _dev(rs.shared, "shared", dtype, 2)
            _need(rs.shared.shape == (t, h), "row sum: shared has the wrong shape")
        if rs.gate is not None:
            _need(rs.gate.is_cuda and rs.gate.dtype == torch.float32 and rs.gate.dim() == 1
                  and rs.gate.shape[0] == t, "row sum: gate must be 32-bit [rows] on the GPU")
            stride = rs.gate.stride(0)
        return k, stride

    def rope_kv_write(self, qkv, bias, positions, row_seq, inv_freq, rot_dim, n_q, n_kv, head_dim,
                      k_pool, v_pool, block_table, page_size, write_kv=True, interleaved=False,
                      q_norm=None, k_norm=None, norm_eps=0.0):
        """Bias, rotation of q and k, and the write of k and v into pages. Pair i of the
        first `rot_dim` dims of a head turns by pos * inv_freq[i]; the pairs are
        (i, i + rot_dim / 2), or the neighbours (2i, 2i + 1) when `interleaved`. `q_norm`,
        `k_norm` [head_dim] (32-bit gains, both or neither): every query and key head is
        normed over its dims (x rsqrt(mean(x^2) + norm_eps) gain) after the bias and before it
        turns."""
        _dev(qkv, "qkv", dims=2)
        t = qkv.shape[0]
        width = (n_q + 2 * n_kv) * head_dim
        _need(qkv.shape[1] == width, f"rope_kv_write: qkv width {qkv.shape[1]} != {width}")
        if bias is not None:
            _dev(bias, "bias", torch.float32, 1)
            _need(bias.shape[0] == width, "rope_kv_write: bias has the wrong size")
        _dev(positions, "positions", torch.int32, 1)
        _dev(row_seq, "row_seq", torch.int32, 1)
        _need(positions.shape[0] == t and row_seq.shape[0] == t, "rope_kv_write: index sizes")
        if rot_dim:
            _dev(inv_freq, "inv_freq", torch.float32, 1)
            _need(inv_freq.shape[0] == rot_dim // 2, "rope_kv_write: table size != rot_dim / 2")
        _dev(k_pool, "k_pool", qkv.dtype, 4)
        _dev(v_pool, "v_pool", qkv.dtype, 4)
        _need(k_pool.shape == v_pool.shape and k_pool.shape[1:] == (n_kv, page_size, head_dim),
              f"rope_kv_write: pools {tuple(k_pool.shape)} do not fit (kv heads {n_kv}, page "
              f"{page_size}, head {head_dim})")
        _dev(block_table, "block_table", torch.int32, 2)
        _need((q_norm is None) == (k_norm is None), "rope_kv_write: both heads' norms or neither")
        if q_norm is not None:
            _dev(q_norm, "q_norm", torch.float32, 1)
            _dev(k_norm, "k_norm", torch.float32, 1)
            _need(q_norm.shape[0] == head_dim and k_norm.shape[0] == head_dim,
                  "rope_kv_write: a head's norm has one gain per dim of a head")
        self._ok(self.lib.ninfer_rope_kv_write(
            ctypes.c_void_p(qkv.data_ptr()), ctypes.c_void_p(_ptr(bias)),
            ctypes.c_void_p(positions.data_ptr()), ctypes.c_void_p(row_seq.data_ptr()),
            ctypes.c_void_p(_ptr(inv_freq) if rot_dim else None), rot_dim, n_q, n_kv, head_dim,
            ctypes.c_void_p(k_pool.data_ptr()), ctypes.c_void_p(v_pool.data_ptr()),
            ctypes.c_void_p(block_table.data_ptr()), block_table.shape[1], page_size,
            1 if write_kv else 0, 1 if interleaved else 0, t, _DT[qkv.dtype],
            ctypes.c_void_p(_ptr(q_norm)), ctypes.c_void_p(_ptr(k_norm)), ctypes.c_float(norm_eps),
            self._stream()))

    def qkv_rope(self, x, w_qkv, bias, qkv, positions, row_seq, inv_freq, rot_dim, n_q, n_kv,
                 head_dim, k_pool, v_pool, block_table, page_size, write_kv=True,
                 interleaved=False, q_norm=None, k_norm=None, norm_eps=0.0):
        """qkv = x w_qkv^T, then what `rope_kv_write` does. Few bf16 rows with a full
        rotation in half-split pairs and no norm of the heads run as one kernel (its blocks
        hold parts of heads); everything else as the product and the rotation kernel one after
        the other."""
        t = x.shape[0]
        fused = (not self.force_generic and not interleaved and x.dtype == torch.bfloat16
                 and x.dim() == 2 and q_norm is None
                 and self.lib.ninfer_qkv_rope_takes(t, x.shape[1], x.shape[1], head_dim, rot_dim))
        if not fused:
            self.linear(x, w_qkv, qkv)
            self.rope_kv_write(qkv, bias, positions, row_seq, inv_freq, rot_dim, n_q, n_kv,
                               head_dim, k_pool, v_pool, block_table, page_size, write_kv,
                               interleaved, q_norm, k_norm, norm_eps)
            return
        width = (n_q + 2 * n_kv) * head_dim
        _dev(x, "x", torch.bfloat16, 2)
        _dev(w_qkv, "w_qkv", torch.bfloat16, 2)
        _dev(qkv, "qkv", torch.bfloat16, 2)
        _need(w_qkv.shape == (width, x.shape[1]) and qkv.shape == (t, width), "qkv_rope: shapes")
        if bias is not None:
            _dev(bias, "bias", torch.float32, 1)
            _need(bias.shape[0] == width, "qkv_rope: bias has the wrong size")
        _dev(positions, "positions", torch.int32, 1)
        _dev(row_seq, "row_seq", torch.int32, 1)
        _need(positions.shape[0] == t and row_seq.shape[0] == t, "qkv_rope: index sizes")
        _dev(inv_freq, "inv_freq", torch.float32, 1)
        _need(inv_freq.shape[0] == head_dim // 2, "qkv_rope: table size != head_dim / 2")
        _dev(k_pool, "k_pool", torch.bfloat16, 4)
        _dev(v_pool, "v_pool", torch.bfloat16, 4)
        _need(k_pool.shape == v_pool.shape and k_pool.shape[1:] == (n_kv, page_size, head_dim),
              "qkv_rope: pools do not fit the head layout")
        _dev(block_table, "block_table", torch.int32, 2)
        args = _QkvRopeArgs(x.data_ptr(), w_qkv.data_ptr(), _ptr(bias), qkv.data_ptr(),
                            positions.data_ptr(), row_seq.data_ptr(), inv_freq.data_ptr(),
                            k_pool.data_ptr(), v_pool.data_ptr(), block_table.data_ptr(), t,
                            x.shape[1], x.shape[1], n_q, n_kv, head_dim, block_table.shape[1],
                            page_size, 1 if write_kv else 0)
        self._ok(self.lib.ninfer_qkv_rope(ctypes.byref(args), self._stream()))

    def moe_combine(self, residual, y, wts, shared=None, gate=None):
        _dev(residual, "residual", torch.float32, 2)
        _dev(y, "y", dims=2)
        _dev(wts, "wts", torch.float32, 2)
        t, h = residual.shape
        k = wts.shape[1]
        _need(wts.shape[0] == t and y.shape == (t * k, h), "moe_combine: shapes differ")
        if shared is not None:
            _dev(shared, "shared", y.dtype, 2)
            _need(shared.shape == (t, h), "moe_combine: shared has the wrong shape")
        stride = 1
        if gate is not None:
            _need(gate.is_cuda and gate.dtype == torch.float32 and gate.numel() == t,
                  "moe_combine: gate must be 32-bit with one value per row, on the GPU")
            gate = gate.reshape(t)
            stride = gate.stride(0)
        self._ok(self.lib.ninfer_moe_combine(
            ctypes.c_void_p(residual.data_ptr()), ctypes.c_void_p(y.data_ptr()),
            ctypes.c_void_p(wts.data_ptr()), ctypes.c_void_p(_ptr(shared)),
            ctypes.c_void_p(_ptr(gate)), stride, t, h, k, _DT[y.dtype], self._stream()))

    # ---- products ---------------------------------------------------------------
    def _gemm(self, a, w, c, *, n, k, m, bias=None, offsets=None, a_index=None, c_index=None,
              a_div=1, groups=1, epilogue=0, w_group_stride=0, tiles=None, only_if_split=False,
              act_limit=0.0, act_alpha=1.0):
        t16 = t64 = tc = None
        if tiles is not None and tiles.tiles16 is not None:
            t16, t64, tc = tiles.tiles16.data_ptr(), tiles.tiles_big.data_ptr(), \
                tiles.tile_counts.data_ptr()
        args = _GemmArgs(a.data_ptr(), w.data_ptr(), c.data_ptr(), _ptr(bias), _ptr(offsets),
                         _ptr(a_index), _ptr(c_index), t16, t64, tc, w_group_stride, m, n, k,
                         a.shape[1],
                         c.shape[1], groups, a_div, _DT[a.dtype], _DT[c.dtype], epilogue)
        args.force_kernel = self._tune["force_kernel"]
        args.split_min_bytes = self._tune["split_min_bytes"]
        args.skinny_two = self._tune["skinny_two"]
        args.act_limit, args.act_alpha = float(act_limit), float(act_alpha)
        if only_if_split:
            # a dense product of few dozen rows: the library's unless the kernels here cut it
            # along K (its output tiles alone would not fill the GPU). The one workspace of
            # the cut belongs to the main stream: on the second stream nothing is cut (the
            # library's product runs instead).
            if self._on_side():
                return False
            if self._split_ws is None:
                self._split_ws = torch.empty(1 << 23, dtype=torch.float32, device=a.device)
            args.workspace = self._split_ws.data_ptr()
            args.workspace_floats = self._split_ws.numel()
            if self.lib.ninfer_gemm_split_parts(ctypes.byref(args)) < 2:
                return False
            self._ok(self.lib.ninfer_gemm(ctypes.byref(args), 0, self._stream()))
            return True
        if self._held is not None:
            self._held.append((args, (a, w, c, bias, offsets, a_index, c_index, tiles)))
            return
        self._ok(self.lib.ninfer_gemm(ctypes.byref(args), 1 if self.force_generic else 0,
                                      self._stream()))

    def _on_side(self) -> bool:
        return self._side is not None and (self._stream().value or 0) == self._side.cuda_stream

    def _new_event(self) -> ctypes.c_void_p:
        ev = self.lib.ninfer_event_create()
        _need(ev, "no event: " + self.lib.ninfer_last_error().decode())
        return ctypes.c_void_p(ev)

    def together(self):
        """Context manager for products that do not depend on each other: the
        hand-written ones called inside are held back and launched when it ends,
        two at a time as one launch where such a pair has a kernel (few rows: a
        launch's fixed time is paid once), otherwise one after the other. Outputs
        are valid after the block, not inside it."""
        return _Together(self)

    def wants_beside(self, rows: int, weight_bytes: int = 0) -> bool:
        """Is independent work of this many rows, which reads this many bytes of weights, worth
        the second stream? Not while a graph is being captured: its steps have few rows each,
        and a fork inside a capture is one more thing a replay would have to get right."""
        if rows < self.beside_min_rows and (rows < self.beside_heavy_min_rows
                                            or weight_bytes < self.beside_heavy_bytes):
            return False
        return not torch.cuda.is_current_stream_capturing()

    def beside(self):
        """Context manager for work that nothing on the current stream waits for until
        `join()`: it runs on a second stream, so that the device can fill with its blocks
        the units that the current stream's kernels leave empty (the last, partly filled
        round of a kernel whose blocks run one per CU). Memory made inside may be read on
        the current stream after `join()`; what it reads must have been given to the
        current stream before the block."""
        return _Beside(self)

    def join(self) -> None:
        """The current stream waits for the `beside()` block before."""
        if self._side_open:
            self._ok(self.lib.ninfer_stream_after(self._stream(), self._side.cuda_stream,
                                                  self._side_events[1]))
            self._side_open = False

    def _launch_held(self, held, route=None):
        force = 1 if self.force_generic else 0
        if route is not None:
            logits, rargs, keep = route
            if len(held) == 1 and held[0][1][2] is logits:
                # the router's logits and the routing by them: one block does both for few rows
                self._ok(self.lib.ninfer_gemm_route(ctypes.byref(held[0][0]), ctypes.byref(rargs),
                                                    force, self._stream()))
                return
            if len(held) == 2 and held[0][1][2] is logits:
                # the router's logits, a product beside them, and the routing: one launch
                # where the library has a kernel for the three, else it runs them in turn
                self._ok(self.lib.ninfer_gemm_pair_route(
                    ctypes.byref(held[0][0]), ctypes.byref(held[1][0]), ctypes.byref(rargs), force,
                    self._stream()))
                return
        i = 0
        while i < len(held):
            if i + 1 < len(held):
                self._ok(self.lib.ninfer_gemm_pair(ctypes.byref(held[i][0]),
                                                   ctypes.byref(held[i + 1][0]), force,
                                                   self._stream()))
                i += 2
            else:
                self._ok(self.lib.ninfer_gemm(ctypes.byref(held[i][0]), force, self._stream()))
                i += 1
        if route is not None:
            self._route_now(*route[2])

    def linear(self, x, w, out, bias=None, act=None):
        """out = x w^T (+ bias); out may be 32-bit whatever the inputs are. `act` 'relu2': the
        square of relu on every element of out."""
        # (an activation runs in the product's epilogue, on the kernels here at every row count)
        _need(act in UNGATED_ACTS, f"linear: activation {act!r} is not one of {sorted(map(str, UNGATED_ACTS))}")
        _dev(x, "x", dims=2)
        _dev(w, "w", x.dtype, 2)
        _dev(out, "out", dims=2)
        _need(x.shape[1] == w.shape[1], f"linear: x has {x.shape[1]} columns, w has {w.shape[1]}")
        _need(out.shape == (x.shape[0], w.shape[0]), "linear: out has the wrong shape")
        _need(out.dtype in (x.dtype, torch.float32), "linear: bad out dtype")
        if bias is not None:
            _dev(bias, "bias", torch.float32, 1)
            _need(bias.shape[0] == w.shape[0], "linear: bias has the wrong size")
        if act is None and self._use_library(x, out, w) and bias is None and not (
                x.shape[0] <= self.side_own_max_rows
                and w.numel() * w.element_size() <= self.side_own_max_bytes and self._on_side()):
            if x.shape[0] > self.split_max_rows or not self._gemm(
                    x, w, out, m=x.shape[0], n=w.shape[0], k=x.shape[1], only_if_split=True):
                torch.matmul(x, w.t(), out=out)
            return
        self._gemm(x, w, out, m=x.shape[0], n=w.shape[0], k=x.shape[1], bias=bias,
                   epilogue=UNGATED_ACTS[act])

    def _use_library(self, x, out, w) -> bool:
        """Plain dense products of many bf16 rows go to the vendor library, as
        the reference sends every multi-row product to rocBLAS
        (src/ops/linear.hip:21-35); few rows, 32-bit, grouped and fused products
        run on the hand-written kernels, and so do products of up to `rows_kernel_max` rows
        whose sizes the kernel for them takes (gemm_skinny_rows.hip)."""
        if self.force_generic or x.dtype != torch.bfloat16 or out.dtype != x.dtype:
            return False
        rows = x.shape[0]
        if rows <= self.rows_kernel_max and w.shape[0] % 32 == 0 and w.shape[1] % 128 == 0 \
                and self.rows_kernel_features[0] <= w.shape[0] <= self.rows_kernel_features[1]:
            return False
        return rows > self.library_min_rows

    @staticmethod
    def _gate_epilogue(act: str) -> int:
        _need(act in GATE_ACTS, f"gated product: activation {act!r} is not one of {sorted(GATE_ACTS)}")
        return GATE_ACTS[act]

    def swiglu_linear(self, x, w_gate_up, out, act="silu", bias=None, limit=0.0, alpha=1.0):
        """out = act(x Wg^T [+ bg]) * (x Wu^T [+ bu]), Wg = rows [0, I), Wu = rows [I, 2I); act
        is SiLU or the tanh form of GELU (`GATE_ACTS`); `bias` [2I] (32-bit) holds bg, then bu."""
        _dev(x, "x", dims=2)
        _dev(w_gate_up, "w_gate_up", x.dtype, 2)
        _dev(out, "out", x.dtype, 2)
        inner = w_gate_up.shape[0] // 2
        _need(w_gate_up.shape == (2 * inner, x.shape[1]), "swiglu_linear: weight shape")
        _need(out.shape == (x.shape[0], inner), "swiglu_linear: out has the wrong shape")
        if bias is not None:
            _dev(bias, "bias", torch.float32, 1)
            _need(bias.shape[0] == 2 * inner, "swiglu_linear: bias has the wrong size")
        self._gemm(x, w_gate_up, out, m=x.shape[0], n=inner, k=x.shape[1],
                   epilogue=self._gate_epilogue(act), bias=bias, act_limit=limit, act_alpha=alpha)

    def grouped_swiglu(self, x, w_gate_up, offsets, order, top_k, out, tiles=None, act="silu",
                       limit=0.0, alpha=1.0):
        """out[r] = the gated product (see `swiglu_linear`) of row order[r] // top_k of x by
        the expert that owns sorted position r. `offsets` may go on beyond the experts that
        `w_gate_up` holds (experts without weights, sorted last): their rows are passed over."""
        _dev(x, "x", dims=2)
        _dev(w_gate_up, "w_gate_up", x.dtype, 3)
        _dev(out, "out", x.dtype, 2)
        _dev(offsets, "offsets", torch.int32, 1)
        _dev(order, "order", torch.int32, 1)
        e, two_i, h = w_gate_up.shape
        inner = two_i // 2
        n = order.shape[0]
        _need(h == x.shape[1] and two_i == 2 * inner, "grouped_swiglu: weight shape")
        _need(offsets.shape[0] >= e + 1, "grouped_swiglu: offsets size")
        _need(n == x.shape[0] * top_k and out.shape == (n, inner), "grouped_swiglu: row counts")
        self._gemm(x, w_gate_up, out, m=n, n=inner, k=h, offsets=offsets, a_index=order,
                   a_div=top_k, groups=e, epilogue=self._gate_epilogue(act),
                   w_group_stride=two_i * h, tiles=tiles, act_limit=limit, act_alpha=alpha)

    def grouped_down(self, h, w_down, offsets, order, out, tiles=None):
        """out[order[r]] = h[r] Wd_e^T for the expert e that owns sorted position r."""
        _dev(h, "h", dims=2)
        _dev(w_down, "w_down", h.dtype, 3)
        _dev(out, "out", h.dtype, 2)
        _dev(offsets, "offsets", torch.int32, 1)
        _dev(order, "order", torch.int32, 1)
        e, hidden, inner = w_down.shape
        n = order.shape[0]
        _need(inner == h.shape[1] and h.shape[0] == n, "grouped_down: input shape")
        _need(out.shape == (n, hidden) and offsets.shape[0] >= e + 1, "grouped_down: shapes")
        self._gemm(h, w_down, out, m=n, n=hidden, k=inner, offsets=offsets, c_index=order,
                   groups=e, w_group_stride=hidden * inner, tiles=tiles)

    # ---- routing ------------------------------------------------------------------
    def _route_args(self, experts, top_k, renorm, ids, wts, r=None, score="softmax",
                    choice_bias=None, scale=1.0, n_group=0, topk_group=0, group_top=1,
                    renorm_eps=0.0, weightless=0):
        """The router's parameters and the places routing writes, as the library takes them.
        `weightless`: the last so many experts have no weights (no tiles are listed for them).
        `score`: 'softmax' over all experts or 'sigmoid' of each logit; `choice_bias` [experts]
        is added to the scores for the choice of experts only (the weights are the scores);
        `scale` multiplies every weight, after the renormalisation if there is one; with
        `n_group` > 1 only the experts of the `topk_group` groups (of experts / n_group
        neighbours each) with the largest best score (+ bias) are candidates (`group_top` > 1:
        with the largest sum of their group_top best); `renorm_eps` is added to the sum the
        chosen scores are divided by."""
        _need(score in _SCORES, f"routing: score {score!r} is not one of {sorted(_SCORES)}")
        _need(1 <= top_k <= experts, f"routing: top_k {top_k} not in [1, {experts}]")
        if choice_bias is not None:
            _dev(choice_bias, "choice_bias", torch.float32, 1)
            _need(choice_bias.shape[0] == experts, "routing: one bias per expert")
        t16 = t64 = tc = offsets = order = parts = None
        if r is not None:
            offsets, order = r.offsets.data_ptr(), r.order.data_ptr()
            t16, t64, tc = self._tile_ptrs(r, r.order.shape[0], experts)
            if ids.shape[0] >= ROUTE_MANY_MIN_ROWS:
                # many rows: the grouping runs as several blocks, which meet through counts
                # per block of rows (scratch that lives with the routing record)
                n_parts = -(-ids.shape[0] // ROUTE_ROWS_PER_BLOCK)
                if getattr(r, "parts", None) is None or r.parts.numel() < n_parts * experts:
                    r.parts = torch.empty(n_parts * experts, dtype=torch.int32, device=ids.device)
                parts = r.parts.data_ptr()
        args = _RouteArgs(ids.data_ptr(), wts.data_ptr(), offsets, order, t16, t64, tc,
                          _ptr(choice_bias), parts, experts, top_k, 1 if renorm else 0,
                          _SCORES[score], float(scale), int(n_group), int(topk_group),
                          int(group_top), float(renorm_eps), int(weightless))
        return args

    def router_topk(self, logits, experts, top_k, renorm, ids, wts, score="softmax",
                    choice_bias=None, scale=1.0, n_group=0, topk_group=0, group_top=1,
                    renorm_eps=0.0):
        _dev(logits, "logits", torch.float32, 2)
        _dev(ids, "ids", torch.int32, 2)
        _dev(wts, "wts", torch.float32, 2)
        t = logits.shape[0]
        _need(ids.shape == (t, top_k) and wts.shape == (t, top_k), "router_topk: output shapes")
        args = self._route_args(experts, top_k, renorm, ids, wts, None, score, choice_bias, scale,
                                n_group, topk_group, group_top, renorm_eps)
        self._ok(self.lib.ninfer_router_topk(
            ctypes.c_void_p(logits.data_ptr()), logits.shape[1], t, ctypes.byref(args),
            self._stream()))

    def _tile_ptrs(self, tiles, n, experts):
        if tiles is None or tiles.tiles16 is None:
            return None, None, None
        _dev(tiles.tiles16, "tiles16", torch.int32, 2)
        _dev(tiles.tiles_big, "tiles_big", torch.int32, 2)
        _dev(tiles.tile_counts, "tile_counts", torch.int32, 1)
        _need(tiles.tiles16.shape == (min(n, n // 16 + experts), 4)
              and tiles.tiles_big.shape == (n // BIG_TILE_ROWS + experts, 4)
              and tiles.tile_counts.shape[0] == 2, "routing: tile lists have the wrong sizes")
        return tiles.tiles16.data_ptr(), tiles.tiles_big.data_ptr(), tiles.tile_counts.data_ptr()

    def moe_align(self, ids, experts, offsets, order, tiles=None, weightless=0):
        _dev(ids, "ids", torch.int32)
        _dev(offsets, "offsets", torch.int32, 1)
        _dev(order, "order", torch.int32, 1)
        _need(offsets.shape[0] == experts + 1 and order.shape[0] == ids.numel(),
              "moe_align: output sizes")
        t16, t64, tc = self._tile_ptrs(tiles, ids.numel(), experts)
        self._ok(self.lib.ninfer_moe_align(
            ctypes.c_void_p(ids.data_ptr()), ids.numel(), experts,
            ctypes.c_void_p(offsets.data_ptr()), ctypes.c_void_p(order.data_ptr()),
            ctypes.c_void_p(t16), ctypes.c_void_p(t64), ctypes.c_void_p(tc), int(weightless),
            self._stream()))

    def moe_route(self, logits, experts, top_k, renorm, r, score="softmax", choice_bias=None,
                  scale=1.0, n_group=0, topk_group=0, group_top=1, renorm_eps=0.0, weightless=0):
        """Scores + top-k per row (see `_route_args` for the router's parameters) and the
        grouping by expert, into the routing record `r` (ids, weights, offsets, order, tile
        lists): one launch for up to 16 rows (one block does both), two for more (top-k by
        one wave per row in parallel, then the grouping). Inside `together()`, after the
        product that writes `logits`, it is held back with the products and launched with
        them (for few rows: by the block that computes the logits)."""
        t = logits.shape[0]
        _dev(logits, "logits", torch.float32, 2)
        _dev(r.ids, "ids", torch.int32, 2)
        _dev(r.weights, "weights", torch.float32, 2)
        _dev(r.offsets, "offsets", torch.int32, 1)
        _dev(r.order, "order", torch.int32, 1)
        _need(logits.shape[1] >= experts, "moe_route: fewer logits than experts")
        _need(r.ids.shape == (t, top_k) and r.weights.shape == (t, top_k)
              and r.offsets.shape[0] == experts + 1 and r.order.shape[0] == t * top_k,
              "moe_route: output sizes")
        rargs = self._route_args(experts, top_k, renorm, r.ids, r.weights, r, score, choice_bias,
                                 scale, n_group, topk_group, group_top, renorm_eps, weightless)
        if self._held is not None:
            _need(self._held_route is None, "together(): one routing at most")
            self._held_route = (logits, rargs, (logits, rargs, r, choice_bias))
            return
        self._route_now(logits, rargs, r)

    def _route_now(self, logits, rargs, r, keep=None):
        t = logits.shape[0]
        if t > 16 and rargs.parts:
            self._ok(self.lib.ninfer_moe_route_many(
                ctypes.c_void_p(logits.data_ptr()), logits.shape[1], t, ctypes.byref(rargs),
                self._stream()))
            return
        if t > 16:
            self._ok(self.lib.ninfer_router_topk(
                ctypes.c_void_p(logits.data_ptr()), logits.shape[1], t, ctypes.byref(rargs),
                self._stream()))
            self.moe_align(r.ids, rargs.E, r.offsets, r.order, tiles=r, weightless=rargs.weightless)
            return
        self._ok(self.lib.ninfer_moe_route_small(
            ctypes.c_void_p(logits.data_ptr()), logits.shape[1], t, ctypes.byref(rargs),
            self._stream()))

    # ---- attention ------------------------------------------------------------------
    def paged_attention(self, qkv, k_pool, v_pool, block_table, ctx, n_q, n_kv, head_dim,
                        page_size, window, scale, out, plan_only=False, slopes=None, vdim=None,
                        sink=False):
        """Attention of the rows' query heads (the first n_q * head_dim columns
        of `qkv`) over their requests' cached keys and values. `slopes` [n_q] (32-bit): head
        h's scores get slopes[h] * (key's position - row's position) added before the softmax
        (a distance-based position bias; negative distances, so a positive slope favours near
        keys). `vdim`: numbers of a value head when they differ from a key head's (`v_pool` and
        `out` are that wide). `sink`: the softmax's denominator has one more term, exp(0), that
        belongs to no key. `plan_only`: launch
        nothing and say how a step of single-token rows of this shape would run
        (which split-context kernel, keys per chunk, chunks)."""
        vdim = head_dim if vdim is None else int(vdim)
        _dev(qkv, "qkv", dims=2)
        _dev(k_pool, "k_pool", qkv.dtype, 4)
        _dev(v_pool, "v_pool", qkv.dtype, 4)
        _dev(out, "out", qkv.dtype, 2)
        _dev(block_table, "block_table", torch.int32, 2)
        t = qkv.shape[0]
        _need(out.shape == (t, n_q * vdim), "paged_attention: out has the wrong shape")
        _need(k_pool.shape[0] == v_pool.shape[0] and k_pool.shape[1:] == (n_kv, page_size, head_dim)
              and v_pool.shape[1:] == (n_kv, page_size, vdim),
              "paged_attention: pools do not fit the head layout")
        _need(block_table.shape[0] == ctx.S, "paged_attention: block table rows != requests")
        _need(ctx.positions.shape[0] == t, "paged_attention: positions size")
        if slopes is not None:
            _dev(slopes, "slopes", torch.float32, 1)
            _need(slopes.shape[0] == n_q, "paged_attention: one slope per query head")
        ws, ws_floats = None, 0
        single = int(getattr(ctx, "single_rows", 0))
        if (ctx.max_qlen == 1 or single > 0) and qkv.dtype == torch.bfloat16 \
                and not self.force_generic:
            ws_floats = int(self.lib.ninfer_attention_workspace_floats(
                t if ctx.max_qlen == 1 else single, n_q, max(head_dim, vdim), ctx.max_kv_len))
            if self._attn_ws is None or self._attn_ws.numel() < ws_floats:
                # A captured graph may hold the address of the workspace it was recorded
                # with: an outgrown one is kept, never given back (a replay would write
                # into whatever took its place), and growth at least doubles, which bounds
                # what is kept to the size of the largest.
                if self._attn_ws is not None:
                    self._outgrown.append(self._attn_ws)
                    ws_floats = max(ws_floats, 2 * self._attn_ws.numel())
                self._attn_ws = torch.empty(ws_floats, dtype=torch.float32, device=qkv.device)
            ws_floats = self._attn_ws.numel()
            ws = self._attn_ws.data_ptr()
        args = _AttnArgs(
            qkv.data_ptr(), k_pool.data_ptr(), v_pool.data_ptr(), out.data_ptr(),
            block_table.data_ptr(), ctx.positions.data_ptr(), ctx.row_seq.data_ptr(),
            ctx.seq_row_start.data_ptr(), ctx.seq_qlen.data_ptr(), ctx.seq_pos0.data_ptr(),
            ws, ws_floats, qkv.shape[1], block_table.shape[1], t, ctx.S, n_q, n_kv, head_dim, page_size,
            int(window or 0), float(scale), _DT[qkv.dtype], ctx.max_qlen, ctx.max_kv_len, single,
            _ptr(slopes), vdim, 1 if sink else 0)
        if plan_only:
            kernel, chunk, n_chunks = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
            self._ok(self.lib.ninfer_attention_decode_plan(
                ctypes.byref(args), ctypes.byref(kernel), ctypes.byref(chunk),
                ctypes.byref(n_chunks)))
            return {"kernel": ("plain", "scalar", "heads")[kernel.value], "chunk": chunk.value,
                    "chunks": n_chunks.value}
        self._ok(self.lib.ninfer_paged_attention(ctypes.byref(args),
                                                 1 if self.force_generic else 0, self._stream()))

    def qkv_conv(self, u, w_conv, state, ctx, q_out, heads, kv_heads, dim, vdim, k_pool, v_pool,
                 block_table, page_size, q_norm=None, k_norm=None, norm_eps=0.0, inv_freq=None,
                 rot_dim=0, interleaved=False, w_conv_t=None):
        """Projected rows u [T, heads * dim + kv_heads * (dim + vdim)] on their way to attention:
        a causal convolution over time per channel (`w_conv` [channels, taps], None: none; the
        taps - 1 projected rows before a step's first row come from `state` [slots, >= (taps - 1)
        * channels] 32-bit, which is moved on), then query and key heads normed over their `dim`
        numbers (gains `q_norm`, `k_norm` [dim], None: no norm) and turned by their position
        (`inv_freq`, `rot_dim`, pairing as in `rope_kv_write`); queries to `q_out` [T, heads *
        dim], keys and values to the requests' pages of `k_pool` [pages, kv_heads, page_size,
        dim] and `v_pool` [.., vdim]. kv_heads 0: the rows hold queries only. `w_conv_t`: the
        convolution's weights once more, transposed [taps, channels], for the kernel that moves
        whole pieces of 8 channels (without it the kernel of a wave per head runs)."""
        _dev(u, "u", dims=2)
        _dev(q_out, "q_out", u.dtype, 2)
        t = ctx.T
        channels = heads * dim + kv_heads * (dim + vdim)
        _need(u.dtype in _DT and u.shape == (t, channels) and q_out.shape == (t, heads * dim),
              f"qkv_conv: rows of {tuple(u.shape)} for {channels} channels")
        a = _QkvConvArgs()
        a.u, a.q_out = u.data_ptr(), q_out.data_ptr()
        taps = 0
        if w_conv is not None:
            _dev(w_conv, "w_conv", torch.float32, 2)
            taps = w_conv.shape[1]
            _need(w_conv.shape[0] == channels and taps >= 1, "qkv_conv: one row of taps per channel")
            a.w = w_conv.data_ptr()
            if w_conv_t is not None:
                _dev(w_conv_t, "w_conv_t", torch.float32, 2)
                _need(w_conv_t.shape == (taps, channels), "qkv_conv: the transposed weights' shape")
                a.wt = w_conv_t.data_ptr()
        if taps > 1:
            _need(state is not None and state.is_cuda and state.dtype == torch.float32
                  and state.dim() == 2 and state.stride(1) == 1
                  and state.shape[1] >= (taps - 1) * channels,
                  "qkv_conv: the state must be 32-bit rows of at least (taps - 1) * channels numbers")
            a.state, a.state_stride = state.data_ptr(), state.stride(0)
        if kv_heads:
            _dev(k_pool, "k_pool", u.dtype, 4)
            _dev(v_pool, "v_pool", u.dtype, 4)
            _dev(block_table, "block_table", torch.int32, 2)
            _need(k_pool.shape[0] == v_pool.shape[0]
                  and k_pool.shape[1:] == (kv_heads, page_size, dim)
                  and v_pool.shape[1:] == (kv_heads, page_size, vdim) and block_table.shape[0] == ctx.S,
                  "qkv_conv: pools or block table do not fit the head layout")
            a.kpool, a.vpool, a.block_table = k_pool.data_ptr(), v_pool.data_ptr(), block_table.data_ptr()
            a.bt_stride = block_table.shape[1]
        for g, name in ((q_norm, "q_norm"), (k_norm, "k_norm")):
            if g is not None:
                _dev(g, name, torch.float32, 1)
                _need(g.shape[0] == dim, f"qkv_conv: {name} has one gain per number of a head")
        _need(kv_heads == 0 or (q_norm is None) == (k_norm is None), "qkv_conv: both heads' norms or neither")
        a.q_gain, a.k_gain = _ptr(q_norm), _ptr(k_norm)
        if rot_dim:
            _dev(inv_freq, "inv_freq", torch.float32, 1)
            _need(inv_freq.shape[0] == rot_dim // 2 and rot_dim <= dim, "qkv_conv: table size != rot_dim / 2")
            a.inv_freq = inv_freq.data_ptr()
        a.positions, a.row_seq = ctx.positions.data_ptr(), ctx.row_seq.data_ptr()
        a.seq_row_start, a.seq_slots = ctx.seq_row_start.data_ptr(), ctx.seq_slots.data_ptr()
        a.T, a.S, a.Hq, a.Hkv, a.dim, a.vdim, a.taps = t, ctx.S, heads, kv_heads, dim, vdim, taps
        a.rot_dim, a.interleaved, a.page_size = rot_dim, 1 if interleaved else 0, page_size
        a.dtype, a.eps = _DT[u.dtype], norm_eps
        a.all_single = 1 if ctx.max_qlen == 1 else 0
        a.force_plain = 1 if self.force_generic else 2 if self.conv_pieces_always else 0
        self._ok(self.lib.ninfer_qkv_conv(ctypes.byref(a), self._stream()))

    # ---- sublayers with the norm on their output -----------------------------------
    def short_conv(self, x, w, state, ctx, out):
        """out = x + conv(x): per channel, conv(x)_t = sum_j w[:, j] x_(t - taps + 1 + j) over
        the rows of each request; the taps - 1 inputs before a step's first row come from
        `state` ([slots, >= (taps - 1) * H] 32-bit, a view whose rows may lie apart), which is
        moved on to the step's last inputs. x: the 32-bit rows [T, H]; w: [H, taps] 32-bit."""
        _dev(x, "x", torch.float32, 2)
        _dev(w, "w", torch.float32, 2)
        _dev(out, "out", dims=2)
        t, h = x.shape
        taps = w.shape[1]
        _need(w.shape[0] == h and out.shape == (t, h), "short_conv: shapes")
        _need(out.dtype in _DT, f"short_conv: out of {out.dtype}")
        if taps == 1 and state is None:   # one tap keeps nothing
            state_ptr, state_stride = None, 0
        else:
            _need(state is not None and state.is_cuda and state.dtype == torch.float32
                  and state.dim() == 2 and state.stride(1) == 1
                  and state.shape[1] >= (taps - 1) * h,
                  "short_conv: the state must be 32-bit rows of at least (taps - 1) * H numbers")
            state_ptr, state_stride = state.data_ptr(), state.stride(0)
        _need(ctx.T == t, "short_conv: rows differ from the step's")
        self._ok(self.lib.ninfer_short_conv(
            ctypes.c_void_p(x.data_ptr()), ctypes.c_void_p(w.data_ptr()),
            ctypes.c_void_p(state_ptr), ctypes.c_longlong(state_stride),
            ctypes.c_void_p(out.data_ptr()), ctypes.c_void_p(ctx.row_seq.data_ptr()),
            ctypes.c_void_p(ctx.seq_row_start.data_ptr()), ctypes.c_void_p(ctx.seq_slots.data_ptr()),
            t, ctx.S, h, taps, 1 if ctx.max_qlen == 1 else 0, _DT[out.dtype], self._stream()))

    def norm_add(self, residual, y, gain, eps, center=False, weights=None):
        """residual += y rsqrt(mean(y^2) + eps) gain; gain holds one number or one per column.
        `center`: the layer norm instead, (y - mean(y)) rsqrt(mean((y - mean(y))^2) + eps) gain.
        `weights` [T, k] (32-bit): y holds T * k rows and stands for the rows
        sum_j weights[t, j] y[t * k + j], formed in 32-bit (a sparse feed-forward's output)."""
        _dev(residual, "residual", torch.float32, 2)
        _dev(y, "y", dims=2)
        _dev(gain, "gain", torch.float32, 1)
        k = 0
        if weights is not None:
            _dev(weights, "weights", torch.float32, 2)
            k = weights.shape[1]
            _need(weights.shape[0] == residual.shape[0] and y.shape == (residual.shape[0] * k,
                  residual.shape[1]), "norm_add: the weighted rows do not fit the residual")
        else:
            _need(y.shape == residual.shape, "norm_add: y does not fit the residual")
        _need(y.dtype in _DT, "norm_add: y's dtype")
        _need(gain.shape[0] in (1, y.shape[1]), "norm_add: one gain, or one per column")
        self._ok(self.lib.ninfer_norm_add(
            ctypes.c_void_p(residual.data_ptr()), ctypes.c_void_p(y.data_ptr()),
            ctypes.c_void_p(gain.data_ptr()), gain.shape[0], residual.shape[0], y.shape[1],
            ctypes.c_float(eps), _DT[y.dtype], 1 if center else 0,
            ctypes.c_void_p(_ptr(weights)), k, self._stream()))

    def gated_rmsnorm(self, o, gate, weight, eps, out, group=0, gate_act="sigmoid"):
        """out = o rsqrt(mean(o^2) + eps) weight sigmoid(gate), the mean over the whole row, or
        with `group` over every group of so many neighbouring columns by itself (`weight` then
        has `group` numbers, shared by the groups). `gate_act` 'silu': gate sigmoid(gate) in
        place of sigmoid(gate). o: [T, N] 32-bit; gate: [T, N] columns of a wider row-major
        tensor (a view)."""
        _dev(o, "o", torch.float32, 2)
        _dev(weight, "weight", torch.float32, 1)
        _dev(out, "out", dims=2)
        t, n = o.shape
        _need(gate_act in ("sigmoid", "silu"), f"gated_rmsnorm: gate activation {gate_act!r}")
        _need(group >= 0 and (group == 0 or n % group == 0), "gated_rmsnorm: groups do not fill the rows")
        _need(out.shape == (t, n) and weight.shape[0] == (group or n) and out.dtype in _DT,
              "gated_rmsnorm: shapes")
        _need(gate.is_cuda and gate.dtype == out.dtype and gate.shape == (t, n)
              and gate.stride(1) == 1, "gated_rmsnorm: the gate must be [T, N] columns of rows")
        self._ok(self.lib.ninfer_gated_rmsnorm(
            ctypes.c_void_p(o.data_ptr()), ctypes.c_void_p(gate.data_ptr()),
            gate.stride(0) if t > 1 else max(n, gate.stride(0)),
            ctypes.c_void_p(weight.data_ptr()), ctypes.c_void_p(out.data_ptr()), t, n,
            ctypes.c_float(eps), _DT[out.dtype], int(group), 1 if gate_act == "silu" else 0,
            self._stream()))

    def lightning_attention(self, qkv, q_off, k_off, v_off, heads, dim, vdim, decay, state, ctx,
                            out):
        """Linear attention with a decay per head over the rows of each request:
        S <- decay_h S + k v^T, out = S^T q with q, k, v = silu of the columns of `qkv` at
        q_off, k_off (heads x dim) and v_off (heads x vdim). `state` ([slots, >= heads * dim *
        vdim] 32-bit view) holds every request's S between steps. out: [T, heads * vdim] 32-bit."""
        _dev(qkv, "qkv", dims=2)
        _dev(decay, "decay", torch.float32, 1)
        _dev(out, "out", torch.float32, 2)
        t = qkv.shape[0]
        _need(qkv.dtype in _DT, f"lightning_attention: rows of {qkv.dtype}")
        _need(decay.shape[0] == heads and out.shape == (t, heads * vdim) and ctx.T == t,
              "lightning_attention: shapes")
        for off, n in ((q_off, heads * dim), (k_off, heads * dim), (v_off, heads * vdim)):
            _need(0 <= off and off + n <= qkv.shape[1], "lightning_attention: columns outside the rows")
        _need(state.is_cuda and state.dtype == torch.float32 and state.dim() == 2
              and state.stride(1) == 1 and state.shape[1] >= heads * dim * vdim,
              "lightning_attention: the state must be 32-bit rows of heads * dim * vdim numbers")
        args = (ctypes.c_void_p(qkv.data_ptr()), qkv.shape[1], q_off, k_off, v_off,
                ctypes.c_void_p(decay.data_ptr()), ctypes.c_void_p(state.data_ptr()),
                ctypes.c_longlong(state.stride(0)), ctypes.c_void_p(out.data_ptr()),
                ctypes.c_void_p(ctx.seq_row_start.data_ptr()), ctypes.c_void_p(ctx.seq_slots.data_ptr()),
                t, ctx.S, heads, dim, vdim, _DT[qkv.dtype], self._stream())
        # bfloat16 steps that bring prompt portions: chunks of 64 rows on the matrix cores (the
        # sums of a chunk are ordered otherwise than token by token, so the 32-bit path, whose
        # logits do not depend on the cut to the bit, stays on the token-by-token kernel)
        if qkv.dtype == torch.bfloat16 and ctx.max_qlen >= self.lightning_chunk_min_rows \
                and not self.force_generic:
            rc = self.lib.ninfer_lightning_attention_chunks(*args)
            if rc == 0:
                return
            if rc < 0:
                self._ok(rc)
        self._ok(self.lib.ninfer_lightning_attention(*args))

    def _latent_args(self, ctx, pool, block_table, heads, dim, rank, rot_dim, rot_n, page_size,
                     dtype):
        _dev(pool, "pool", dtype, 3)
        _need(pool.shape[1:] == (page_size, rank + rot_dim),
              f"latent attention: pool {tuple(pool.shape)} does not fit pages of {page_size} rows "
              f"of {rank + rot_dim}")
        _dev(block_table, "block_table", torch.int32, 2)
        _need(block_table.shape[0] == ctx.S, "latent attention: block table rows != requests")
        a = _LatentArgs()
        a.pool, a.block_table = pool.data_ptr(), block_table.data_ptr()
        a.positions, a.row_seq = ctx.positions.data_ptr(), ctx.row_seq.data_ptr()
        a.seq_row_start, a.seq_pos0 = ctx.seq_row_start.data_ptr(), ctx.seq_pos0.data_ptr()
        a.S, a.max_kv_len, a.max_qlen = ctx.S, ctx.max_kv_len, ctx.max_qlen
        a.force_plain = 1 if self.force_generic else 2 if self.conv_pieces_always else 0
        a.bt_stride, a.T, a.Hq, a.dim, a.R, a.rd, a.rot_n = \
            block_table.shape[1], ctx.T, heads, dim, rank, rot_dim, rot_n
        a.page_size, a.dtype = page_size, _DT[dtype]
        return a

    def latent_kv_write(self, dkv, q, q_abs, pool, block_table, ctx, heads, dim, rank, rot_dim,
                        norm_w, eps, freq, rot_n, magnitude, page_size, write_kv=True,
                        interleaved=False):
        """Per row: the first `rank` columns of `dkv` normed (x rsqrt(mean(x^2) + eps) norm_w)
        and the next `rot_dim`, turned by the row's position, go to the request's page of
        `pool` [pages, page_size, rank + rot_dim]; the rotated part of every head of `q`
        ([T, heads * (dim + rot_dim)]) is turned and written behind the first `rank` numbers of
        the head's row of `q_abs` [T, heads, rank + rot_dim] (32-bit). Pair (i, i + rot_n / 2)
        (with `interleaved`: pair (2i, 2i + 1)) of the first rot_n rotated numbers turns by
        pos * freq[i]; cos and sin times `magnitude`."""
        _need(dkv.is_cuda and dkv.dim() == 2 and dkv.stride(1) == 1 and dkv.shape[1] >= rank + rot_dim,
              "latent_kv_write: dkv must be rows of at least rank + rot_dim columns")
        _dev(q, "q", dkv.dtype, 2)
        _dev(q_abs, "q_abs", torch.float32, 3)
        _dev(norm_w, "norm_w", torch.float32, 1)
        t = ctx.T
        _need(dkv.shape[0] == t and q.shape == (t, heads * (dim + rot_dim))
              and q_abs.shape == (t, heads, rank + rot_dim) and norm_w.shape[0] == rank,
              "latent_kv_write: shapes")
        a = self._latent_args(ctx, pool, block_table, heads, dim, rank, rot_dim, rot_n, page_size,
                              dkv.dtype)
        if rot_n:
            _dev(freq, "freq", torch.float32, 1)
            _need(freq.shape[0] == rot_n // 2, "latent_kv_write: table size != rot_n / 2")
            a.freq = freq.data_ptr()
        a.dkv, a.q, a.q_abs, a.norm_w = dkv.data_ptr(), q.data_ptr(), q_abs.data_ptr(), norm_w.data_ptr()
        a.dkv_stride = dkv.stride(0) if t > 1 else max(dkv.shape[1], dkv.stride(0))
        a.eps, a.magnitude, a.scale, a.write_kv = eps, magnitude, 1.0, 1 if write_kv else 0
        a.interleaved = 1 if interleaved else 0
        self._ok(self.lib.ninfer_latent_kv_write(ctypes.byref(a), self._stream()))

    def latent_attention(self, q_abs, pool, block_table, ctx, heads, rank, rot_dim, page_size,
                         scale, out, gate=None, window=None):
        """Softmax attention of q_abs [T, heads, rank + rot_dim] (32-bit) over the rows of the
        requests' pages of `pool` (every head reads the same rows): scores (q . row) * scale
        over positions <= the row's own (within `window` if given), out[t, h] = sum_j p_j
        row_j[:rank], times sigmoid(gate[t, h]) when `gate` ([T, heads] columns of a wider
        tensor, a view) is given. out: [T, heads * rank]."""
        _dev(q_abs, "q_abs", torch.float32, 3)
        _dev(out, "out", pool.dtype, 2)
        t = ctx.T
        _need(q_abs.shape == (t, heads, rank + rot_dim) and out.shape == (t, heads * rank),
              "latent_attention: shapes")
        a = self._latent_args(ctx, pool, block_table, heads, 0, rank, rot_dim, 0, page_size,
                              pool.dtype)
        a.q_abs, a.out, a.scale, a.window = q_abs.data_ptr(), out.data_ptr(), scale, int(window or 0)
        if gate is not None:
            _need(gate.is_cuda and gate.dtype == pool.dtype and gate.shape == (t, heads)
                  and gate.stride(1) == 1, "latent_attention: the gate must be [T, heads] columns")
            a.gate = gate.data_ptr()
            a.gate_stride = gate.stride(0) if t > 1 else max(heads, gate.stride(0))
        need = int(self.lib.ninfer_latent_attention_workspace_floats(ctypes.byref(a)))
        if need:   # contexts cut into chunks: partial sums, merged by a second kernel
            ws = self._workspace(need, q_abs.device)
            a.workspace, a.workspace_floats = ws.data_ptr(), ws.numel()
        self._ok(self.lib.ninfer_latent_attention(ctypes.byref(a), self._stream()))

    def _workspace(self, floats: int, device) -> torch.Tensor:
        """The attention kernels' 32-bit scratch, grown when a step needs more. A captured graph
        may hold the address of the one it was recorded with: an outgrown one is kept, never
        given back, and growth at least doubles, which bounds what is kept."""
        if self._attn_ws is None or self._attn_ws.numel() < floats:
            if self._attn_ws is not None:
                self._outgrown.append(self._attn_ws)
                floats = max(floats, 2 * self._attn_ws.numel())
            self._attn_ws = torch.empty(floats, dtype=torch.float32, device=device)
        return self._attn_ws

    def head_index(self, ctx, heads):
        """(offsets [heads + 1], index [T * heads]) for products that every head runs with
        weights of its own on its own columns of the rows: with the rows viewed as [T * heads,
        columns of a head], group h owns the sorted rows h * T .. (h + 1) * T - 1, and sorted
        row h * T + t is row t * heads + h. Made once per step and kept in its scratch."""
        key = ("head_index", heads)
        if key not in ctx.scratch:
            t = ctx.T
            offsets = torch.arange(0, (heads + 1) * t, t, dtype=torch.int32, device=ctx.device)
            index = (torch.arange(t, dtype=torch.int32, device=ctx.device)[None, :] * heads
                     + torch.arange(heads, dtype=torch.int32, device=ctx.device)[:, None]).reshape(-1)
            ctx.scratch[key] = (offsets, index.contiguous())
        return ctx.scratch[key]

    def per_head_linear(self, x, w, out, ctx, k, n):
        """out[t, h, :n] = x[t, h, :k] w[h]^T for every head: x [T, heads, >= k], w [heads, n, k],
        out [T, heads, >= n] (32-bit or x's dtype); columns beyond k and n are left alone. Runs
        as one grouped product (the groups are the heads)."""
        _dev(x, "x", dims=3)
        _dev(w, "w", x.dtype, 3)
        _dev(out, "out", dims=3)
        t, heads = x.shape[0], x.shape[1]
        _need(w.shape == (heads, n, k) and x.shape[2] >= k and out.shape[:2] == (t, heads)
              and out.shape[2] >= n, "per_head_linear: shapes")
        _need(out.dtype in (x.dtype, torch.float32), "per_head_linear: bad out dtype")
        offsets, index = self.head_index(ctx, heads)
        self._gemm(x.view(t * heads, x.shape[2]), w, out.view(t * heads, out.shape[2]),
                   m=t * heads, n=n, k=k, offsets=offsets, a_index=index, c_index=index,
                   groups=heads, w_group_stride=n * k)

    # ---- parallel sublayers, hashed pairs, differential attention ------------------------
    def embed_pairs(self, ctx, table, out, scale=1.0, pair_table=None, buckets=0, mul_prev=0,
                    mul_cur=0, state=None):
        """out[t] = table[token[t]] scale (+ pair_table[row]) in 32-bit, row = (previous token x
        mul_prev + token x mul_cur) mod buckets, or `buckets` (the table's last row) for a
        request's first token. The token before a step's first row comes from `state` ([slots,
        >= 1] 32-bit view: previous token + 1 as an integer, 0 for none), which is moved on to
        the step's last token."""
        _dev(table, "table", dims=2)
        _dev(out, "out", torch.float32, 2)
        _need(out.shape == (ctx.T, table.shape[1]), "embed_pairs: out has the wrong shape")
        state_ptr, stride = None, 0
        if pair_table is not None:
            _dev(pair_table, "pair_table", table.dtype, 2)
            _need(pair_table.shape == (buckets + 1, table.shape[1]) and buckets > 0,
                  "embed_pairs: the table of pairs must have buckets + 1 rows")
            _need(state is not None and state.is_cuda and state.dtype == torch.float32
                  and state.dim() == 2 and state.shape[1] >= 1,
                  "embed_pairs: the state must be 32-bit rows of at least one number")
            state_ptr, stride = state.data_ptr(), state.stride(0)
        self._ok(self.lib.ninfer_embed_pairs(
            ctypes.c_void_p(ctx.tokens.data_ptr()), ctypes.c_void_p(table.data_ptr()),
            ctypes.c_void_p(out.data_ptr()), ctx.T, table.shape[1], _DT[table.dtype],
            ctypes.c_float(scale), ctypes.c_void_p(_ptr(pair_table)), int(buckets), int(mul_prev),
            int(mul_cur), ctypes.c_void_p(ctx.row_seq.data_ptr()),
            ctypes.c_void_p(ctx.seq_row_start.data_ptr()), ctypes.c_void_p(ctx.seq_slots.data_ptr()),
            ctx.S, ctypes.c_void_p(state_ptr), ctypes.c_longlong(stride), self._stream()))

    def concat_rows(self, a, b, out):
        """out[:, :H] = a, out[:, H:] = b (a, b: 32-bit [T, H]; out: [T, 2H] of any dtype)."""
        _dev(a, "a", torch.float32, 2)
        _dev(b, "b", torch.float32, 2)
        _dev(out, "out", dims=2)
        _need(a.shape == b.shape and out.shape == (a.shape[0], 2 * a.shape[1])
              and out.dtype in _DT, "concat_rows: shapes")
        self._ok(self.lib.ninfer_concat_rows(
            ctypes.c_void_p(a.data_ptr()), ctypes.c_void_p(b.data_ptr()),
            ctypes.c_void_p(out.data_ptr()), a.shape[0], a.shape[1], _DT[out.dtype], self._stream()))

    def scaled_sum_add(self, residual, a, s1, f, s2):
        """residual += s1 a + s2 f in 32-bit: a rows [T, H] or None; f rows [T, H], a weighted
        sum of rows (an object with y, weights, shared, gate) or None; s1, s2 [H] 32-bit or
        None (factor 1)."""
        _dev(residual, "residual", torch.float32, 2)
        t, h = residual.shape
        dtype = None
        if a is not None:
            _dev(a, "a", dims=2)
            _need(a.shape == (t, h) and a.dtype in _DT, "scaled_sum_add: a does not fit")
            dtype = a.dtype
        for name, sc in (("s1", s1), ("s2", s2)):
            if sc is not None:
                _dev(sc, name, torch.float32, 1)
                _need(sc.shape[0] == h, f"scaled_sum_add: {name} has the wrong size")
        dense = y = w = shared = gate = None
        k = gs = 0
        if f is not None and hasattr(f, "weights"):
            dtype = dtype or f.y.dtype
            k, gs = self._check_rows_sum(f, t, h, dtype)
            y, w, shared, gate = f.y.data_ptr(), f.weights.data_ptr(), _ptr(f.shared), _ptr(f.gate)
        elif f is not None:
            dtype = dtype or f.dtype
            _dev(f, "f", dtype, 2)
            _need(f.shape == (t, h), "scaled_sum_add: f does not fit")
            dense = f.data_ptr()
        if dtype is None:
            return
        self._ok(self.lib.ninfer_scaled_sum_add(
            ctypes.c_void_p(residual.data_ptr()), ctypes.c_void_p(_ptr(a)), ctypes.c_void_p(_ptr(s1)),
            ctypes.c_void_p(dense), ctypes.c_void_p(y), ctypes.c_void_p(w), k,
            ctypes.c_void_p(shared), ctypes.c_void_p(gate), gs, ctypes.c_void_p(_ptr(s2)), t, h,
            _DT[dtype], self._stream()))

    def tanh_cap(self, x, cap):
        """x <- cap tanh(x / cap) in place (32-bit numbers)."""
        _dev(x, "x", torch.float32)
        self._ok(self.lib.ninfer_tanh_cap(ctypes.c_void_p(x.data_ptr()),
                                          ctypes.c_longlong(x.numel()), ctypes.c_float(cap),
                                          self._stream()))

    def relu_square(self, x):
        """x <- max(x, 0)^2 in place."""
        _dev(x, "x")
        _need(x.dtype in _DT, f"relu_square: tensor of {x.dtype}")
        self._ok(self.lib.ninfer_relu_square(ctypes.c_void_p(x.data_ptr()),
                                             ctypes.c_longlong(x.numel()), _DT[x.dtype],
                                             self._stream()))

    def diff_attention(self, qkv, k_pool, v_pool, block_table, ctx, heads, kv_heads, dim, vdim,
                       page_size, scale, cap, temp_coef, temp_every, lam, eps, out_scale, out,
                       write_kv=True):
        """Differential attention of the rows of `qkv` ([T, heads x 2 dim | kv_heads x 2 dim |
        kv_heads x vdim]: two queries and two keys per head, [map 1 | map 2], and one value):
        k and v go into the requests' pages (`write_kv`), then every query head forms
        a1 - lam a2 from its two causal softmax attentions over the same values, divides it by
        its root mean square over vdim (eps inside the root; eps < 0: no norm) and multiplies
        by out_scale. Scores: (q . k) scale (1 + temp_coef ln(floor((p + 1) / temp_every) + 1))
        at the row's position p, then cap tanh(. / cap) when cap > 0. out: [T, heads x vdim]."""
        _dev(qkv, "qkv", dims=2)
        _need(qkv.dtype in _DT, f"diff_attention: rows of {qkv.dtype}")
        _dev(k_pool, "k_pool", qkv.dtype, 4)
        _dev(v_pool, "v_pool", qkv.dtype, 4)
        _dev(out, "out", qkv.dtype, 2)
        _dev(block_table, "block_table", torch.int32, 2)
        t = qkv.shape[0]
        _need(t == ctx.T and qkv.shape[1] == (heads + kv_heads) * 2 * dim + kv_heads * vdim,
              "diff_attention: qkv has the wrong shape")
        _need(out.shape == (t, heads * vdim), "diff_attention: out has the wrong shape")
        _need(k_pool.shape[1:] == (kv_heads, page_size, 2 * dim)
              and v_pool.shape[1:] == (kv_heads, page_size, vdim)
              and k_pool.shape[0] == v_pool.shape[0],
              "diff_attention: pools do not fit the head layout")
        _need(block_table.shape[0] == ctx.S, "diff_attention: block table rows != requests")
        a = _DiffAttnArgs()
        a.qkv, a.kpool, a.vpool, a.out = qkv.data_ptr(), k_pool.data_ptr(), v_pool.data_ptr(), out.data_ptr()
        a.block_table, a.positions = block_table.data_ptr(), ctx.positions.data_ptr()
        a.row_seq, a.seq_row_start = ctx.row_seq.data_ptr(), ctx.seq_row_start.data_ptr()
        a.q_stride, a.bt_stride, a.T, a.S = qkv.shape[1], block_table.shape[1], t, ctx.S
        a.Hq, a.Hkv, a.dim, a.vdim, a.page_size = heads, kv_heads, dim, vdim, page_size
        a.dtype, a.max_qlen, a.max_kv_len = _DT[qkv.dtype], ctx.max_qlen, ctx.max_kv_len
        a.force_plain = 1 if self.force_generic else 2 if self.conv_pieces_always else 0
        a.single_rows = int(getattr(ctx, "single_rows", 0))
        a.scale, a.cap, a.t_coef, a.t_every = scale, cap, temp_coef, int(temp_every)
        a.lam, a.eps, a.out_scale = lam, eps, out_scale
        if write_kv:
            self._ok(self.lib.ninfer_diff_kv_write(ctypes.byref(a), self._stream()))
        need = int(self.lib.ninfer_diff_attention_workspace_floats(ctypes.byref(a)))
        if need:   # contexts cut into chunks: partial sums, merged by a second kernel
            ws = self._workspace(need, qkv.device)
            a.workspace, a.workspace_floats = ws.data_ptr(), ws.numel()
        self._ok(self.lib.ninfer_diff_attention(ctypes.byref(a), self._stream()))

    def gated_sum_add(self, residual, a, g1, b1, f, g2, b2, mult=1.0):
        """residual += mult (c1 a + c2 f) in 32-bit: a rows [T, H] or None; f rows [T, H], a
        weighted sum of rows (an object with y, weights and, where some chosen experts hand
        their input back, ids, real and rows) or None; c = sigmoid(g + b) per row and column
        from a gate's logits g [T, H] and bias b [H] (32-bit), or 1 where g is None."""
        _dev(residual, "residual", torch.float32, 2)
        t, h = residual.shape
        p = _GatedSumArgs()
        p.residual, p.T, p.H, p.mult = residual.data_ptr(), t, h, float(mult)
        dtype = None
        keep = [residual, a, g1, b1, f, g2, b2]
        if a is not None:
            _dev(a, "a", dims=2)
            _need(a.shape == (t, h) and a.dtype in _DT, "gated_sum_add: a does not fit")
            dtype = a.dtype
            p.a = a.data_ptr()
        if f is not None and hasattr(f, "weights"):
            dtype = dtype or f.y.dtype
            _need(getattr(f, "shared", None) is None, "gated_sum_add: no shared expert's rows")
            k = f.weights.shape[1]
            _dev(f.y, "y", dtype, 2)
            _dev(f.weights, "weights", torch.float32, 2)
            _need(f.y.shape == (t * k, h) and f.weights.shape == (t, k), "gated_sum_add: weighted rows do not fit")
            p.y, p.w, p.k = f.y.data_ptr(), f.weights.data_ptr(), k
            if getattr(f, "ids", None) is not None:
                _dev(f.ids, "ids", torch.int32, 2)
                _dev(f.rows, "rows", dtype, 2)
                _need(f.ids.shape == (t, k) and f.rows.shape == (t, h), "gated_sum_add: ids or rows do not fit")
                p.ids, p.xin, p.real = f.ids.data_ptr(), f.rows.data_ptr(), int(f.real)
        elif f is not None:
            dtype = dtype or f.dtype
            _dev(f, "f", dtype, 2)
            _need(f.shape == (t, h), "gated_sum_add: f does not fit")
            p.dense = f.data_ptr()
        if dtype is None:
            return
        for g, b, name in ((g1, b1, "1"), (g2, b2, "2")):
            if g is None:
                continue
            _dev(g, "g" + name, dtype, 2)
            _need(g.shape == (t, h), f"gated_sum_add: gate {name} does not fit")
            setattr(p, "g" + name, g.data_ptr())
            if b is not None:
                _dev(b, "b" + name, torch.float32, 1)
                _need(b.shape[0] == h, f"gated_sum_add: bias {name} has the wrong size")
                setattr(p, "b" + name, b.data_ptr())
        p.dtype = _DT[dtype]
        self._ok(self.lib.ninfer_gated_sum_add(ctypes.byref(p), self._stream()))
        del keep

    def gla_work_floats(self, qkv_dtype, ctx, heads, dim):
        """The size of the workspace with which `gated_linear_attention` runs this step in
        chunks, per row; 0 if the step runs token by token."""
        if qkv_dtype != torch.bfloat16 or ctx.max_qlen < self.gla_chunk_min_rows or self.force_generic \
                or dim > 128 or dim % 4:
            return 0
        return 3 * heads * dim + 16 * heads

    def gated_linear_attention(self, qkv, q_off, k_off, v_off, z, heads, dim, vdim, tau, q_scale,
                               state, ctx, out, work=None):
        """Linear attention with a decay per key channel and token over the rows of each
        request: S <- diag(alpha) S + k v^T, out = S^T (q q_scale) with alpha =
        sigmoid(z)^(1 / tau), q, k at the columns q_off, k_off (heads x dim) and v at v_off
        (heads x vdim) of `qkv`; z: [T, heads * dim] 32-bit. `state` ([slots, >= heads * dim *
        vdim] 32-bit view) holds every request's S between steps. out: [T, heads * vdim] 32-bit.
        `work` ([T, gla_work_floats(..)] 32-bit, or None): with it a bfloat16 step that brings
        prompt portions runs in chunks of 16 rows on the matrix cores (the sums of a chunk are
        ordered otherwise than token by token, so the 32-bit path, whose logits do not depend
        on the cut to the bit, stays on the token-by-token kernel)."""
        _dev(qkv, "qkv", dims=2)
        _dev(z, "z", torch.float32, 2)
        _dev(out, "out", torch.float32, 2)
        t = qkv.shape[0]
        _need(qkv.dtype in _DT, f"gated_linear_attention: rows of {qkv.dtype}")
        _need(z.shape == (t, heads * dim) and out.shape == (t, heads * vdim) and ctx.T == t,
              "gated_linear_attention: shapes")
        for off, n in ((q_off, heads * dim), (k_off, heads * dim), (v_off, heads * vdim)):
            _need(0 <= off and off + n <= qkv.shape[1], "gated_linear_attention: columns outside the rows")
        _need(state.is_cuda and state.dtype == torch.float32 and state.dim() == 2
              and state.stride(1) == 1 and state.shape[1] >= heads * dim * vdim,
              "gated_linear_attention: the state must be 32-bit rows of heads * dim * vdim numbers")
        if work is not None and self.gla_work_floats(qkv.dtype, ctx, heads, dim):
            _dev(work, "work", torch.float32, 2)
            _need(work.is_contiguous() and work.shape[0] == t
                  and work.shape[1] >= 3 * heads * dim + 16 * heads,
                  "gated_linear_attention: the workspace is too small")
            rc = self.lib.ninfer_gated_linear_attention_chunks(
                ctypes.c_void_p(qkv.data_ptr()), qkv.shape[1], q_off, k_off, v_off,
                ctypes.c_void_p(z.data_ptr()), ctypes.c_float(tau), ctypes.c_float(q_scale),
                ctypes.c_void_p(state.data_ptr()), ctypes.c_longlong(state.stride(0)),
                ctypes.c_void_p(out.data_ptr()), ctypes.c_void_p(ctx.seq_row_start.data_ptr()),
                ctypes.c_void_p(ctx.seq_slots.data_ptr()), ctypes.c_void_p(work.data_ptr()),
                t, ctx.S, heads, dim, vdim, _DT[qkv.dtype], self._stream())
            if rc == 0:
                return
            if rc < 0:
                self._ok(rc)
        self._ok(self.lib.ninfer_gated_linear_attention(
            ctypes.c_void_p(qkv.data_ptr()), qkv.shape[1], q_off, k_off, v_off,
            ctypes.c_void_p(z.data_ptr()), ctypes.c_float(tau), ctypes.c_float(q_scale),
            ctypes.c_void_p(state.data_ptr()), ctypes.c_longlong(state.stride(0)),
            ctypes.c_void_p(out.data_ptr()), ctypes.c_void_p(ctx.seq_row_start.data_ptr()),
            ctypes.c_void_p(ctx.seq_slots.data_ptr()), t, ctx.S, heads, dim, vdim, _DT[qkv.dtype],
            self._stream()))

    def sigmoid_attention(self, qkv, k_pool, v_pool, block_table, ctx, heads, kv_heads, dim, vdim,
                          page_size, scale, chunk, head_bias, mix, out, write_kv=True):
        """Attention without a softmax over the rows of `qkv` ([T, heads x dim] queries,
        followed by kv_heads x dim keys and kv_heads x vdim values when `write_kv`: those go
        into the requests' pages first). The weight of key j for row i of head a is
        sigmoid((q . k) scale + head_bias[a]) where j <= i and, with chunk > 0,
        floor(i / chunk) == floor(j / chunk), else 0; with `mix` [heads, heads] the heads'
        weights are mixed (w'_a = sum_b mix[a, b] w_b); head a applies its weights to the
        values of kv head a // (heads / kv_heads). out: [T, heads x vdim]."""
        _dev(qkv, "qkv", dims=2)
        _need(qkv.dtype in _DT, f"sigmoid_attention: rows of {qkv.dtype}")
        _dev(k_pool, "k_pool", qkv.dtype, 4)
        _dev(v_pool, "v_pool", qkv.dtype, 4)
        _dev(out, "out", qkv.dtype, 2)
        _dev(block_table, "block_table", torch.int32, 2)
        t = qkv.shape[0]
        width = heads * dim + (kv_heads * (dim + vdim) if write_kv else 0)
        _need(t == ctx.T and qkv.shape[1] == width, "sigmoid_attention: qkv has the wrong shape")
        _need(out.shape == (t, heads * vdim), "sigmoid_attention: out has the wrong shape")
        _need(k_pool.shape[1:] == (kv_heads, page_size, dim)
              and v_pool.shape[1:] == (kv_heads, page_size, vdim)
              and k_pool.shape[0] == v_pool.shape[0],
              "sigmoid_attention: pools do not fit the head layout")
        _need(block_table.shape[0] == ctx.S, "sigmoid_attention: block table rows != requests")
        a = _SigAttnArgs()
        a.qkv, a.kpool, a.vpool, a.out = qkv.data_ptr(), k_pool.data_ptr(), v_pool.data_ptr(), out.data_ptr()
        a.block_table, a.positions = block_table.data_ptr(), ctx.positions.data_ptr()
        a.row_seq, a.seq_row_start = ctx.row_seq.data_ptr(), ctx.seq_row_start.data_ptr()
        if head_bias is not None:
            _dev(head_bias, "head_bias", torch.float32, 1)
            _need(head_bias.shape[0] == heads, "sigmoid_attention: one bias per head")
            a.head_bias = head_bias.data_ptr()
        if mix is not None:
            _dev(mix, "mix", torch.float32, 2)
            _need(mix.shape == (heads, heads), "sigmoid_attention: the mixing matrix is [heads, heads]")
            a.mix = mix.data_ptr()
        a.q_stride, a.bt_stride, a.T, a.S = qkv.shape[1], block_table.shape[1], t, ctx.S
        a.Hq, a.Hkv, a.dim, a.vdim, a.page_size = heads, kv_heads, dim, vdim, page_size
        a.dtype, a.max_qlen, a.max_kv_len = _DT[qkv.dtype], ctx.max_qlen, ctx.max_kv_len
        a.chunk, a.scale = int(chunk), float(scale)
        a.force_plain = 1 if self.force_generic else 2 if self.conv_pieces_always else 0
        a.single_rows = int(getattr(ctx, "single_rows", 0))
        if write_kv:
            self._ok(self.lib.ninfer_sigmoid_kv_write(ctypes.byref(a), self._stream()))
        need = int(self.lib.ninfer_sigmoid_attention_workspace_floats(ctypes.byref(a)))
        if need:   # the visible keys cut into parts: partial outputs, added up by a second kernel
            ws = self._workspace(need, qkv.device)
            a.workspace, a.workspace_floats = ws.data_ptr(), ws.numel()
        self._ok(self.lib.ninfer_sigmoid_attention(ctypes.byref(a), self._stream()))

    # ---- sampling -------------------------------------------------------------------
    FEW_TOKENS = 64   # most tokens a row may keep (top_k) for the two-launch sampling path

    def sample(self, logits, temperature, uniform, out, top_k=None, top_p=None, rep_penalty=None,
               pen_tokens=None, pen_counts=None, pen_offsets=None, few=False):
        """One token per row. `few`: the caller asserts that every row is greedy
        (temperature <= 0) or has 1 <= top_k <= FEW_TOKENS; same result, much faster."""
        _dev(logits, "logits", torch.float32, 2)
        r, v = logits.shape
        _dev(temperature, "temperature", torch.float32, 1)
        _dev(uniform, "uniform", torch.float32, 1)
        _dev(out, "out", torch.int32, 1)
        _need(temperature.shape[0] == r and uniform.shape[0] == r and out.shape[0] == r,
              "sample: per-row arrays have the wrong size")
        for name, t, dt in (("top_k", top_k, torch.int32), ("top_p", top_p, torch.float32),
                            ("rep_penalty", rep_penalty, torch.float32)):
            if t is not None:
                _dev(t, name, dt, 1)
                _need(t.shape[0] == r, f"sample: {name} has the wrong size")
        if pen_offsets is not None:
            _dev(pen_offsets, "pen_offsets", torch.int32, 1)
            _dev(pen_tokens, "pen_tokens", torch.int32, 1)
            _dev(pen_counts, "pen_counts", torch.int32, 1)
            _need(pen_offsets.shape[0] == r + 1, "sample: pen_offsets has the wrong size")
        if few:
            # every row keeps few tokens (the caller knows its rows' options): candidates from
            # the whole GPU first, then the same selection and draw on those
            _need(top_k is not None, "sample: rows that keep few tokens need top_k")
            places = int(self.lib.ninfer_sample_few_places(v))
            cand_val = torch.empty((r, places), dtype=torch.float32, device=logits.device)
            cand_idx = torch.empty((r, places), dtype=torch.int32, device=logits.device)
            work = torch.empty((r, places), dtype=torch.float32, device=logits.device)
            self._ok(self.lib.ninfer_sample_few(
                ctypes.c_void_p(logits.data_ptr()), logits.stride(0), v, r,
                ctypes.c_void_p(cand_val.data_ptr()), ctypes.c_void_p(cand_idx.data_ptr()),
                ctypes.c_void_p(work.data_ptr()), ctypes.c_void_p(temperature.data_ptr()),
                ctypes.c_void_p(top_k.data_ptr()), ctypes.c_void_p(_ptr(top_p)),
                ctypes.c_void_p(_ptr(rep_penalty)), ctypes.c_void_p(_ptr(pen_tokens)),
                ctypes.c_void_p(_ptr(pen_counts)), ctypes.c_void_p(_ptr(pen_offsets)),
                ctypes.c_void_p(uniform.data_ptr()), ctypes.c_void_p(out.data_ptr()),
                self._stream()))
            return
        work = torch.empty((r, v), dtype=torch.float32, device=logits.device)
        self._ok(self.lib.ninfer_sample(
            ctypes.c_void_p(logits.data_ptr()), logits.stride(0), v, r,
            ctypes.c_void_p(work.data_ptr()), ctypes.c_void_p(temperature.data_ptr()),
            ctypes.c_void_p(_ptr(top_k)), ctypes.c_void_p(_ptr(top_p)),
            ctypes.c_void_p(_ptr(rep_penalty)), ctypes.c_void_p(_ptr(pen_tokens)),
            ctypes.c_void_p(_ptr(pen_counts)), ctypes.c_void_p(_ptr(pen_offsets)),
            ctypes.c_void_p(uniform.data_ptr()), ctypes.c_void_p(out.data_ptr()), self._stream()))
