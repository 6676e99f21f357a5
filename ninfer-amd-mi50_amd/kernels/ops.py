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
                ("force_kernel", ctypes.c_int), ("skinny_two", ctypes.c_int)]


class _RouteArgs(ctypes.Structure):
    _fields_ = [("ids", ctypes.c_void_p), ("wts", ctypes.c_void_p), ("offsets", ctypes.c_void_p),
                ("order", ctypes.c_void_p), ("tiles16", ctypes.c_void_p),
                ("tiles_big", ctypes.c_void_p), ("tile_counts", ctypes.c_void_p),
                ("choice_bias", ctypes.c_void_p), ("parts", ctypes.c_void_p),
                ("E", ctypes.c_int), ("k", ctypes.c_int), ("renorm", ctypes.c_int),
                ("score", ctypes.c_int), ("scale", ctypes.c_float), ("n_group", ctypes.c_int),
                ("topk_group", ctypes.c_int)]


BIG_TILE_ROWS = 256   # rows of a tall tile of the grouped products (the library's kGroupedTileRows)
ROUTE_ROWS_PER_BLOCK = 1024  # the library's kAlignRowsPerBlock
# rows (tokens) from which the grouping runs as several blocks side by side: 12.5 against 13 us
# at 2,048 rows of 60 experts top-4 (11 against 10 at 1,024), 19 against 37 at 8,192, 46 against 127
# at 32,768
ROUTE_MANY_MIN_ROWS = 2048
_SCORES = {"softmax": 0, "sigmoid": 1}
# activations of a gated product, by the names config.json gives them -> the library's epilogue
GATE_ACTS = {"silu": 1, "gelu_pytorch_tanh": 2}


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
                ("slopes", ctypes.c_void_p)]


class _QkvRopeArgs(ctypes.Structure):
    _fields_ = [("x", ctypes.c_void_p), ("w", ctypes.c_void_p), ("bias", ctypes.c_void_p),
                ("qkv", ctypes.c_void_p), ("positions", ctypes.c_void_p),
                ("row_seq", ctypes.c_void_p), ("inv_freq", ctypes.c_void_p),
                ("kpool", ctypes.c_void_p), ("vpool", ctypes.c_void_p),
                ("block_table", ctypes.c_void_p), ("T", ctypes.c_int), ("K", ctypes.c_int),
                ("lda", ctypes.c_int), ("Hq", ctypes.c_int), ("Hkv", ctypes.c_int),
                ("D", ctypes.c_int), ("bt_stride", ctypes.c_int), ("page_size", ctypes.c_int),
                ("write_kv", ctypes.c_int)]


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

    def rmsnorm(self, x, gain, eps, out, delta=None, rows=None, rows_sum=None):
        """out = norm(x [+ delta] [+ rows_sum]); `rows_sum` is a weighted sum of
        rows (an object with y, weights, shared, gate) added on the fly."""
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
            mgs, mk, self._stream()))

    @staticmethod
    def _check_rows_sum(rs, t, h, dtype):
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
              a_div=1, groups=1, epilogue=0, w_group_stride=0, tiles=None, only_if_split=False):
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

    def linear(self, x, w, out, bias=None):
        """out = x w^T (+ bias); out may be 32-bit whatever the inputs are."""
        _dev(x, "x", dims=2)
        _dev(w, "w", x.dtype, 2)
        _dev(out, "out", dims=2)
        _need(x.shape[1] == w.shape[1], f"linear: x has {x.shape[1]} columns, w has {w.shape[1]}")
        _need(out.shape == (x.shape[0], w.shape[0]), "linear: out has the wrong shape")
        _need(out.dtype in (x.dtype, torch.float32), "linear: bad out dtype")
        if bias is not None:
            _dev(bias, "bias", torch.float32, 1)
            _need(bias.shape[0] == w.shape[0], "linear: bias has the wrong size")
        if self._use_library(x, out, w) and bias is None and not (
                x.shape[0] <= self.side_own_max_rows
                and w.numel() * w.element_size() <= self.side_own_max_bytes and self._on_side()):
            if x.shape[0] > self.split_max_rows or not self._gemm(
                    x, w, out, m=x.shape[0], n=w.shape[0], k=x.shape[1], only_if_split=True):
                torch.matmul(x, w.t(), out=out)
            return
        self._gemm(x, w, out, m=x.shape[0], n=w.shape[0], k=x.shape[1], bias=bias)

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

    def swiglu_linear(self, x, w_gate_up, out, act="silu", bias=None):
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
                   epilogue=self._gate_epilogue(act), bias=bias)

    def grouped_swiglu(self, x, w_gate_up, offsets, order, top_k, out, tiles=None, act="silu"):
        """out[r] = the gated product (see `swiglu_linear`) of row order[r] // top_k of x by
        the expert that owns sorted position r."""
        _dev(x, "x", dims=2)
        _dev(w_gate_up, "w_gate_up", x.dtype, 3)
        _dev(out, "out", x.dtype, 2)
        _dev(offsets, "offsets", torch.int32, 1)
        _dev(order, "order", torch.int32, 1)
        e, two_i, h = w_gate_up.shape
        inner = two_i // 2
        n = order.shape[0]
        _need(h == x.shape[1] and two_i == 2 * inner, "grouped_swiglu: weight shape")
        _need(offsets.shape[0] == e + 1, "grouped_swiglu: offsets size")
        _need(n == x.shape[0] * top_k and out.shape == (n, inner), "grouped_swiglu: row counts")
        self._gemm(x, w_gate_up, out, m=n, n=inner, k=h, offsets=offsets, a_index=order,
                   a_div=top_k, groups=e, epilogue=self._gate_epilogue(act),
                   w_group_stride=two_i * h, tiles=tiles)

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
        _need(out.shape == (n, hidden) and offsets.shape[0] == e + 1, "grouped_down: shapes")
        self._gemm(h, w_down, out, m=n, n=hidden, k=inner, offsets=offsets, c_index=order,
                   groups=e, w_group_stride=hidden * inner, tiles=tiles)

    # ---- routing ------------------------------------------------------------------
    def _route_args(self, experts, top_k, renorm, ids, wts, r=None, score="softmax",
                    choice_bias=None, scale=1.0, n_group=0, topk_group=0):
        """The router's parameters and the places routing writes, as the library takes them.
        `score`: 'softmax' over all experts or 'sigmoid' of each logit; `choice_bias` [experts]
        is added to the scores for the choice of experts only (the weights are the scores);
        `scale` multiplies every weight, after the renormalisation if there is one; with
        `n_group` > 1 only the experts of the `topk_group` groups (of experts / n_group
        neighbours each) with the largest best score (+ bias) are candidates."""
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
                          _SCORES[score], float(scale), int(n_group), int(topk_group))
        return args

    def router_topk(self, logits, experts, top_k, renorm, ids, wts, score="softmax",
                    choice_bias=None, scale=1.0, n_group=0, topk_group=0):
        _dev(logits, "logits", torch.float32, 2)
        _dev(ids, "ids", torch.int32, 2)
        _dev(wts, "wts", torch.float32, 2)
        t = logits.shape[0]
        _need(ids.shape == (t, top_k) and wts.shape == (t, top_k), "router_topk: output shapes")
        args = self._route_args(experts, top_k, renorm, ids, wts, None, score, choice_bias, scale,
                                n_group, topk_group)
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

    def moe_align(self, ids, experts, offsets, order, tiles=None):
        _dev(ids, "ids", torch.int32)
        _dev(offsets, "offsets", torch.int32, 1)
        _dev(order, "order", torch.int32, 1)
        _need(offsets.shape[0] == experts + 1 and order.shape[0] == ids.numel(),
              "moe_align: output sizes")
        t16, t64, tc = self._tile_ptrs(tiles, ids.numel(), experts)
        self._ok(self.lib.ninfer_moe_align(
            ctypes.c_void_p(ids.data_ptr()), ids.numel(), experts,
            ctypes.c_void_p(offsets.data_ptr()), ctypes.c_void_p(order.data_ptr()),
            ctypes.c_void_p(t16), ctypes.c_void_p(t64), ctypes.c_void_p(tc), self._stream()))

    def moe_route(self, logits, experts, top_k, renorm, r, score="softmax", choice_bias=None,
                  scale=1.0, n_group=0, topk_group=0):
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
                                 scale, n_group, topk_group)
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
            self.moe_align(r.ids, rargs.E, r.offsets, r.order, tiles=r)
            return
        self._ok(self.lib.ninfer_moe_route_small(
            ctypes.c_void_p(logits.data_ptr()), logits.shape[1], t, ctypes.byref(rargs),
            self._stream()))

    # ---- attention ------------------------------------------------------------------
    def paged_attention(self, qkv, k_pool, v_pool, block_table, ctx, n_q, n_kv, head_dim,
                        page_size, window, scale, out, plan_only=False, slopes=None):
        """Attention of the rows' query heads (the first n_q * head_dim columns
        of `qkv`) over their requests' cached keys and values. `slopes` [n_q] (32-bit): head
        h's scores get slopes[h] * (key's position - row's position) added before the softmax
        (a distance-based position bias; negative distances, so a positive slope favours near
        keys). `plan_only`: launch
        nothing and say how a step of single-token rows of this shape would run
        (which split-context kernel, keys per chunk, chunks)."""
        _dev(qkv, "qkv", dims=2)
        _dev(k_pool, "k_pool", qkv.dtype, 4)
        _dev(v_pool, "v_pool", qkv.dtype, 4)
        _dev(out, "out", qkv.dtype, 2)
        _dev(block_table, "block_table", torch.int32, 2)
        t = qkv.shape[0]
        _need(out.shape == (t, n_q * head_dim), "paged_attention: out has the wrong shape")
        _need(k_pool.shape == v_pool.shape and k_pool.shape[1:] == (n_kv, page_size, head_dim),
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
                t if ctx.max_qlen == 1 else single, n_q, head_dim, ctx.max_kv_len))
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
            _ptr(slopes))
        if plan_only:
            kernel, chunk, n_chunks = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
            self._ok(self.lib.ninfer_attention_decode_plan(
                ctypes.byref(args), ctypes.byref(kernel), ctypes.byref(chunk),
                ctypes.byref(n_chunks)))
            return {"kernel": ("plain", "scalar", "heads")[kernel.value], "chunk": chunk.value,
                    "chunks": n_chunks.value}
        self._ok(self.lib.ninfer_paged_attention(ctypes.byref(args),
                                                 1 if self.force_generic else 0, self._stream()))

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
