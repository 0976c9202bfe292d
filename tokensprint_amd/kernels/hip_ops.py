"""The HIP kernels as Python operations: argument checks on the host, then one C call.

Every method checks shapes, dtypes, devices and contiguity before a pointer reaches a
kernel, because a kernel handed a wrong shape would read or write out of bounds.  There
is no other implementation behind these methods: without a GPU or without the built
library, construction raises.
"""

from __future__ import annotations

import ctypes
from ctypes import Structure, byref, c_float, c_int, c_int64, c_void_p

import numpy as np
import torch

from tokensprint_amd.kernels.build import build, find_library
from tokensprint_amd.kernels.dispatch import default_dispatch
from tokensprint_amd.kernels.stream import PreparedRows, UnmergedRows

ABI_VERSION = 1
_TYPE_CODE = {torch.float32: 0, torch.bfloat16: 1}


class KernelError(RuntimeError):
    pass


class QkPrepareArgs(Structure):
    _fields_ = [
        ("qkv", c_void_p), ("q_out", c_void_p), ("k_dst", c_void_p), ("v_dst", c_void_p),
        ("q_weight", c_void_p), ("k_weight", c_void_p), ("cos", c_void_p), ("sin", c_void_p),
        ("positions", c_void_p), ("entry_of_token", c_void_p), ("table", c_void_p),
        ("table_width", c_int), ("num_tokens", c_int), ("nq", c_int), ("nkv", c_int),
        ("hd", c_int), ("page_size", c_int), ("max_pos", c_int), ("paged", c_int),
        ("store_kv", c_int), ("eps", c_float), ("row_extra", c_int),
    ]


class AttentionMfmaArgs(Structure):
    pass


class AttentionArgs(Structure):
    _fields_ = [
        ("q", c_void_p), ("out", c_void_p), ("k_pages", c_void_p), ("v_pages", c_void_p),
        ("positions", c_void_p), ("entry_of_token", c_void_p), ("q_start", c_void_p),
        ("ctx_len", c_void_p), ("table", c_void_p),
        ("table_width", c_int), ("num_tokens", c_int), ("num_entries", c_int), ("nq", c_int),
        ("nkv", c_int), ("hd", c_int), ("page_size", c_int), ("num_pages", c_int),
        ("window", c_int), ("scale", c_float), ("sink", c_void_p),
        ("chunk", c_int), ("softcap", c_float), ("slopes", c_void_p), ("temp_coef", c_float),
        ("temp_every", c_int),
    ]


AttentionMfmaArgs._fields_ = [
    ("base", AttentionArgs), ("tiles", c_void_p), ("partial_o", c_void_p),
    ("partial_ml", c_void_p), ("num_tiles", c_int), ("rows_per_token", c_int),
    ("head_blocks", c_int), ("num_splits", c_int), ("cooperative", c_int),
    ("tiles_per_wave", c_int),
]


class AttentionDecodeArgs(Structure):
    _fields_ = [
        ("m", AttentionMfmaArgs), ("qkv", c_void_p), ("q_weight", c_void_p),
        ("k_weight", c_void_p), ("cos", c_void_p), ("sin", c_void_p), ("eps", c_float),
        ("kv_in_row", c_int), ("defer_merge", c_int), ("arrivals", c_void_p),
        ("row_extra", c_int),
    ]


def _load_library() -> ctypes.CDLL:
    path = find_library()
    if path is None:
        path = build()
    lib = ctypes.CDLL(str(path))
    lib.ts_last_error.restype = ctypes.c_char_p
    if lib.ts_abi_version() != ABI_VERSION:
        raise KernelError(f"{path} has interface version {lib.ts_abi_version()}, "
                          f"this package needs {ABI_VERSION}")
    return lib


def _ptr(t: torch.Tensor | None):
    return c_void_p(t.data_ptr()) if t is not None else c_void_p(0)


class _PendingMerge:
    """A decode step's attention output that still lies in the partial results of its key
    splits: `out` is where the merge puts it.  Holds the partial results alive."""

    def __init__(self, ops, out, args, partial_o, partial_ml, positions, window):
        self.ops, self.out, self.args = ops, out, args       # args: AttentionMfmaArgs
        self.partial_o, self.partial_ml = partial_o, partial_ml
        self.positions, self.window = positions, window
        self.done = False

    def merge(self) -> None:
        if not self.done:
            self.ops._call(self.ops.lib.ts_attention_merge, byref(self.args), self.ops._stream())
            self.done = True


class HipOps:
    name = "hip-gfx950"

    def __init__(self, device) -> None:
        self.device = torch.device(device)
        if self.device.type != "cuda" or not torch.cuda.is_available():
            raise KernelError(
                "the HIP kernels need an AMD GPU (device 'cuda:N'); there is no CPU path")
        self.lib = _load_library()
        self._device_index = self.device.index if self.device.index is not None \
            else torch.cuda.current_device()
        self._raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None) or (
            lambda index: torch.cuda.current_stream(index).cuda_stream)
        self._attn_chunk = self.lib.ts_attention_mfma_chunk()
        self._units = torch.cuda.get_device_properties(self.device).multi_processor_count
        # which kernel takes what: every threshold in one table (kernels/dispatch.py)
        self.dispatch = default_dispatch()
        # for the vendor library's algorithms that want scratch memory during a product
        self._library_workspace = torch.empty(64 << 20, dtype=torch.uint8, device=self.device)
        self._timed_plans = False
        self._staging, self._staging_turn = [None] * 4, -1      # pinned buffers of _upload_ints
        # products of few rows with large weights: ours or the library's, per weight shape
        # (see large_weight_choices)
        self._large_rows, self._large_undecided, self._large_trial = {}, set(), None
        self.merged_rows = self.lib.ts_gemm_tail_merged_rows()   # rows up to which that pays
        # Above those rows the decode kernel merges its key splits itself: the workgroups of
        # an item count themselves in here and the last one merges.  The kernel leaves every
        # count at zero, so one zeroed array serves every launch (of one stream); a launch
        # that did not run to its end may leave counts behind, so the array is zeroed again
        # after every failed call and before warm-up and capture (`reset_scratch`).
        # `fold_merge = False` gives the merge a kernel of its own again.
        self.fold_merge = True
        self._arrivals = torch.zeros(4096, dtype=torch.int32, device=self.device)

    # ------------------------------------------------------------ helpers
    def _stream(self):
        # the current stream's handle, by the short way: this runs before every kernel
        return c_void_p(self._raw_stream(self._device_index))

    def _call(self, fn, *args):
        if fn(*args) != 0:
            message = self.lib.ts_last_error().decode()
            self.reset_scratch()
            raise KernelError(message)

    def reset_scratch(self) -> None:
        """Put what this provider keeps between calls back to its start: the arrival counts
        of the decode kernel's own merge at zero.  Called after a failed call, and by the
        engine before its warm-up step and before graphs are captured."""
        self._arrivals.zero_()

    def _check(self, name, t, dtype=None, shape=None, ndim=None):
        # (written for the case that all is well, which is every call of a working engine:
        # this runs several times before every kernel)
        try:
            ok = t.device == self.device and t.is_contiguous()
        except AttributeError:
            if isinstance(t, UnmergedRows):
                raise TypeError(f"{name}: an unmerged attention output; this call does not "
                                "take one (merged() gives the tensor)") from None
            raise TypeError(f"{name}: expected a tensor, got {type(t)}") from None
        if ok and dtype is not None:
            ok = t.dtype is dtype or (dtype.__class__ is tuple and t.dtype in dtype)
        if ok and ndim is not None:
            ok = t.dim() == ndim
        if ok and shape is not None:
            ok = t.shape == tuple(shape)
        if ok:
            return t
        if t.device != self.device:
            raise ValueError(f"{name}: on {t.device}, kernels run on {self.device}")
        if not t.is_contiguous():
            raise ValueError(f"{name}: must be contiguous, strides {t.stride()}")
        if dtype is not None:
            dtypes = dtype if isinstance(dtype, (tuple, list)) else (dtype,)
            if t.dtype not in dtypes:
                raise TypeError(f"{name}: dtype {t.dtype}, expected one of {dtypes}")
        if ndim is not None and t.dim() != ndim:
            raise ValueError(f"{name}: {t.dim()} dimensions, expected {ndim}")
        raise ValueError(f"{name}: shape {tuple(t.shape)}, expected {tuple(shape)}")

    _FLOATS = (torch.float32, torch.bfloat16)

    # ------------------------------------------------------------ deferred merge
    # A decode step's attention whose keys were split over workgroups ends in a merge of the
    # splits' partial results.  `attend(defer_merge=True)` may leave that merge undone and
    # return an `UnmergedRows` handle instead of a tensor; handed to `linear_into_stream`
    # (the output projection in its tail form), that product's kernel merges the rows itself
    # and a layer has one dependent kernel less.  The other calls that take activation rows
    # merge first (`_rows`); nothing else can read the rows by mistake, the handle being no
    # tensor.
    @staticmethod
    def _rows(x):
        return x.merged() if x.__class__ is UnmergedRows else x

    # ------------------------------------------------------------ rows
    def embed(self, table, token_ids, scale=1.0):
        """Rows of `table` as float32, times `scale`."""
        self._check("embedding table", table, self._FLOATS, ndim=2)
        self._check("token ids", token_ids, torch.int32, ndim=1)
        T, (V, H) = token_ids.shape[0], table.shape
        out = torch.empty(T, H, dtype=torch.float32, device=self.device)
        self._call(self.lib.ts_embed, _ptr(table), _TYPE_CODE[table.dtype], V, _ptr(token_ids),
                   _ptr(out), T, H, c_float(scale), self._stream())
        return out

    def add_bias(self, x, bias):
        """In place: bias (float32 [n]) is added to the first n columns of float32 rows."""
        self._check("x", x, torch.float32, ndim=2)
        self._check("bias", bias, torch.float32, ndim=1)
        if bias.shape[0] > x.shape[1]:
            raise ValueError(f"add_bias: {bias.shape[0]} biases for rows of {x.shape[1]}")
        self._call(self.lib.ts_add_bias, _ptr(x), _ptr(bias), x.shape[0], bias.shape[0],
                   x.shape[1], self._stream())

    def finish_projection(self, rows, bias, *, q_cols, k_cols, extra, values_from_keys, q_norm,
                          k_norm, q_count, k_count, eps, out_dtype):
        """A q/k/v projection's float32 sums [T, q | k | v | extra] (no v with
        `values_from_keys`) -> [T, q | k | v | extra] in `out_dtype`: `bias` (float32 over the
        row's first columns, or None) added; q, and k, divided by the root of (their sum of
        squares over `q_count`, `k_count`, plus eps) and weighed by `q_norm`, `k_norm`
        (float32 [q_cols], [k_cols]; None: left as they are); with `values_from_keys` the
        keys as they were before their norm stand where the values do."""
        self._check("projection rows", rows, torch.float32, ndim=2)
        T, ld = rows.shape
        v_cols = k_cols if values_from_keys else ld - q_cols - k_cols - extra
        if v_cols < 0 or (values_from_keys and ld != q_cols + k_cols + extra):
            raise ValueError(f"finish_projection: rows of {ld} for q={q_cols} k={k_cols} "
                             f"extra={extra}")
        if bias is not None:
            self._check("bias", bias, torch.float32, ndim=1)
            if bias.shape[0] > ld:
                raise ValueError("finish_projection: more biases than columns")
        if q_norm is not None:
            self._check("q norm weight", q_norm, torch.float32, shape=(q_cols,))
        if k_norm is not None:
            self._check("k norm weight", k_norm, torch.float32, shape=(k_cols,))
        out = torch.empty(T, q_cols + k_cols + v_cols + extra, dtype=out_dtype,
                          device=self.device)
        self._call(self.lib.ts_finish_projection, _ptr(rows), _ptr(bias),
                   bias.shape[0] if bias is not None else 0, _ptr(q_norm), _ptr(k_norm),
                   _ptr(out), _TYPE_CODE[out_dtype], T, int(q_cols), int(k_cols), int(v_cols),
                   int(extra), int(bool(values_from_keys)), int(q_count), int(k_count),
                   c_float(eps), self._stream())
        return out

    def take_tokens(self, token_ids, sources, drawn):
        """In place: token_ids[i] = drawn[sources[i]] where 0 <= sources[i] < len(drawn)."""
        self._check("token ids", token_ids, torch.int32, ndim=1)
        self._check("sources", sources, torch.int32, shape=token_ids.shape)
        self._check("drawn", drawn, torch.int32, ndim=1)
        self._call(self.lib.ts_take_tokens, _ptr(token_ids), _ptr(sources), _ptr(drawn),
                   token_ids.shape[0], drawn.shape[0], self._stream())

    def gather_rows(self, x, rows):
        x = self._rows(x)
        self._check("x", x, self._FLOATS, ndim=2)
        self._check("rows", rows, torch.int32, ndim=1)
        out = torch.empty(rows.shape[0], x.shape[1], dtype=x.dtype, device=self.device)
        self._call(self.lib.ts_gather_rows, _ptr(x), _TYPE_CODE[x.dtype], _ptr(rows), _ptr(out),
                   rows.shape[0], x.shape[1], self._stream())
        return out

    def rmsnorm(self, x, weight, eps, out_dtype):
        x = self._rows(x)
        self._check("x", x, self._FLOATS, ndim=2)
        self._check("norm weight", weight, torch.float32, shape=(x.shape[1],))
        out = torch.empty(x.shape, dtype=out_dtype, device=self.device)
        self._call(self.lib.ts_rmsnorm, _ptr(x), _TYPE_CODE[x.dtype], _ptr(weight), _ptr(out),
                   _TYPE_CODE[out_dtype], x.shape[0], x.shape[1], c_float(eps), self._stream())
        return out

    def add_rmsnorm(self, resid, delta, weight, eps, out_dtype):
        delta = self._rows(delta)
        self._check("resid", resid, torch.float32, ndim=2)
        self._check("delta", delta, self._FLOATS, shape=resid.shape)
        self._check("norm weight", weight, torch.float32, shape=(resid.shape[1],))
        out = torch.empty(resid.shape, dtype=out_dtype, device=self.device)
        self._call(self.lib.ts_add_rmsnorm, _ptr(resid), _ptr(delta), _TYPE_CODE[delta.dtype],
                   _ptr(weight), _ptr(out), _TYPE_CODE[out_dtype], resid.shape[0],
                   resid.shape[1], c_float(eps), self._stream())
        return out

    def silu_mul(self, gate_up):
        self._check("gate_up", gate_up, self._FLOATS, ndim=2)
        rows, two_inner = gate_up.shape
        if two_inner % 2:
            raise ValueError("gate_up needs an even row width (gate half, up half)")
        out = torch.empty(rows, two_inner // 2, dtype=gate_up.dtype, device=self.device)
        self._call(self.lib.ts_silu_mul, _ptr(gate_up), _ptr(out), _TYPE_CODE[gate_up.dtype],
                   rows, two_inner // 2, self._stream())
        return out

    # ------------------------------------------------------------ matrix product
    def linear(self, x, weight, out_dtype):
        """x [M, K] times weight [N, K] transposed -> [M, N] in out_dtype."""
        x = self._rows(x)
        self._check("x", x, self._FLOATS, ndim=2)
        self._check("weight", weight, self._FLOATS, ndim=2)
        M, K = x.shape
        N = weight.shape[0]
        if weight.shape[1] != K:
            raise ValueError(f"linear: x has {K} columns, weight has {weight.shape[1]}")
        if self._tiled_plain_ok(M, N, K, x.dtype, weight.dtype, out_dtype):
            # a prompt's portion at small weights: as fast as the library's product on the
            # GPU and a fifth of its cost on the host (which a step's first layer waits for)
            return self.gemm_tiled(x, weight, out_dtype)
        if self._library_ok(x, weight):
            # the library's float32 sums leave in the type asked for: bfloat16 activations,
            # float32 logits at the output head (not rounded to bfloat16 and widened, so
            # that logits are of one precision on both sides of the row count at which
            # the library takes over)
            out = torch.empty(M, N, dtype=out_dtype, device=self.device)
            self._call(self.lib.ts_gemm_library_bf16, _ptr(x), _ptr(weight), _ptr(out),
                       _TYPE_CODE[out_dtype], M, N, K, _ptr(self._library_workspace),
                       ctypes.c_size_t(self._library_workspace.numel()), self._stream())
            return out
        out = torch.empty(M, N, dtype=out_dtype, device=self.device)
        if self._mfma_ok(x, weight):
            self._call(self.lib.ts_gemm_mfma_bf16, _ptr(x), _ptr(weight), _ptr(out),
                       _TYPE_CODE[out_dtype], M, N, K, 0, self._stream())
        else:
            self._call(self.lib.ts_gemm_fma, _ptr(x), _TYPE_CODE[x.dtype], _ptr(weight),
                       _TYPE_CODE[weight.dtype], _ptr(out), _TYPE_CODE[out_dtype], M, N, K,
                       self._stream())
        return out

    def timed_plans(self, on: bool) -> bool:
        """While on, the library products that are met for the first time have their
        algorithm chosen by timing the first entries of the library's list instead of
        taking the first (ten to a hundred milliseconds a shape: for shapes that will be
        used for the rest of the run, i.e. the warm-up's largest step and the decode
        steps that are captured).  Returns what it was before."""
        before = self._timed_plans
        self._timed_plans = bool(on)
        self.lib.ts_gemm_library_candidates(8 if on else 1)
        return before

    def gemm_tiled(self, x, weight, out_dtype, pair=False, tile=0):
        """The LDS-tiled product for many rows: x [M, K] bfloat16, weight [N, K] bfloat16
        (with `pair` [2 N, K], gate rows then up rows, and the result is silu(gate) * up).
        `tile` 0 lets the sizes choose the tile; another names one (the result is the same
        to the bit)."""
        self._check("x", x, torch.bfloat16, ndim=2)
        self._check("weight", weight, torch.bfloat16, ndim=2)
        M, K = x.shape
        N = weight.shape[0] // 2 if pair else weight.shape[0]
        if weight.shape[1] != K or (pair and weight.shape[0] % 2):
            raise ValueError(f"gemm_tiled: x {tuple(x.shape)}, weight {tuple(weight.shape)}")
        out = torch.empty(M, N, dtype=out_dtype, device=self.device)
        self._call(self.lib.ts_gemm_tiled_bf16, _ptr(x), _ptr(weight), _ptr(out),
                   _TYPE_CODE[out_dtype], M, N, K, int(pair), tile, self._stream())
        return out

    # Which rows and sizes go to the vendor library, to the LDS-tiled kernel or stay with
    # the weight-streaming kernels is `self.dispatch`'s (kernels/dispatch.py: every
    # threshold with the shapes it was measured on).  The library accumulates in float32
    # and stores the type asked for: bfloat16 activations, and float32 logits at the output
    # head (the reference's logits are bfloat16).

    def _tiled_pair_ok(self, x, weight, out_dtype):
        M, K = x.shape
        inner = weight.shape[0] // 2
        return (x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16
                and out_dtype == torch.bfloat16 and weight.numel() <= self.dispatch.tiled_pair_weight
                and self._library_rows(M, weight.shape[0], K)
                and self.lib.ts_gemm_tiled_fits(M, inner, K, 1) == 1)

    def _tiled_plain_ok(self, M, N, K, x_dtype, w_dtype, out_dtype):
        d = self.dispatch
        return (x_dtype == torch.bfloat16 and w_dtype == torch.bfloat16
                and out_dtype in (torch.bfloat16, torch.float32)
                and M >= d.tiled_stream_rows and N * K <= d.tiled_stream_weight
                and self.lib.ts_gemm_tiled_fits(M, N, K, 0) == 1)

    def _library_ok(self, x, weight, out_dtype=None):
        if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
            return False
        return self._library_rows(x.shape[0], weight.shape[0], weight.shape[1])

    def large_weight_choices(self):
        """Row counts from which products with a large weight may go to the library, for the
        warm-up to try in a captured decode step, the default first; empty unless a large
        weight of a shape that has no choice yet has been met.  At the Qwen3-8B shapes the
        kernels here are ahead below sixteen rows (a decode step of one row 3.45 against
        4.07 ms), at the 32B shapes (a hidden size of 5,120: 320 or 640 workgroups for 256
        compute units, and a K that the loads' steps divide less well) the library is, by 15
        to 20 %, norm kernels and all.  A choice is kept per weight shape (N, K), so that
        models of other shapes in the same process get their own."""
        if not self._large_undecided:
            return ()
        return (self.dispatch.library_rows_large, 1)

    def try_large_weight_rows(self, rows) -> None:
        """For the shapes without a choice: `rows` for now (None: the default again)."""
        self._large_trial = rows

    def keep_large_weight_rows(self, rows: int) -> None:
        """The shapes met so far without a choice get `rows` for good."""
        for shape in self._large_undecided:
            self._large_rows[shape] = int(rows)
        self._large_undecided = set()
        self._large_trial = None

    def _library_rows(self, M, N, K):
        """Whether a bfloat16 product of M rows with a weight [N, K] is the library's."""
        d = self.dispatch
        if M >= d.library_rows:
            return True
        if M >= d.library_rows_head and N >= d.head_columns:
            return True
        if N * K > d.large_weight:
            rows = self._large_rows.get((N, K))
            if rows is None:
                self._large_undecided.add((N, K))
                rows = d.library_rows_large if self._large_trial is None else self._large_trial
            if M >= rows:
                return True
        return M >= d.library_rows_wide and self.lib.ts_gemm_mfma_layout(N, K) == 2

    @staticmethod
    def _mfma_ok(x, weight):
        """The matrix-core product takes bfloat16 operands with K a multiple of 8;
        everything else (float32 anywhere) goes to the float32 multiply-add kernel."""
        return (x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16
                and x.shape[1] % 8 == 0)

    def linear_into_stream(self, x, weight, resid, hint):
        """The product that ends a sub-layer, told what follows (`hint`, a NormHint).
        Where one kernel can do it (bfloat16, up to 64 rows, both products among those
        this provider keeps from the library): resid += bf16(x W^T) in place, and the
        PreparedRows for the hinted norm and product are returned, to be passed on as
        the stream's delta.  Otherwise None, and nothing has been done: the caller runs
        `linear` and passes its result on."""
        if hint is None or x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16 \
                or hint.weight.dtype != torch.bfloat16:
            return None
        if x.__class__ is UnmergedRows:
            if not x.is_merged:
                prepared = self._merged_into_stream(x._pending, x, weight, resid, hint)
                if prepared is not None:
                    return prepared
            x = x.merged()
        self._check("x", x, torch.bfloat16, ndim=2)
        self._check("weight", weight, torch.bfloat16, ndim=2)
        M, K = x.shape
        N = weight.shape[0]
        if weight.shape[1] != K:
            raise ValueError(f"linear_into_stream: x has {K} columns, weight has {weight.shape[1]}")
        next_n = hint.weight.shape[0] // 2 if hint.silu_mul else hint.weight.shape[0]
        if self._tiled_stream_ok(M, N, K, hint):
            # a prompt's portion: the LDS-tiled product in its tail form
            self._check("resid", resid, torch.float32, shape=(M, N))
            self._check("norm weight", hint.norm_weight, torch.float32, shape=(N,))
            rows = torch.empty(M, N, dtype=torch.bfloat16, device=self.device)
            sumsq = torch.empty(self.lib.ts_gemm_tiled_tail_parts(N), M, dtype=torch.float32,
                                device=self.device)
            self._call(self.lib.ts_gemm_tiled_tail_bf16, _ptr(x), _ptr(weight), _ptr(resid),
                       _ptr(hint.norm_weight), _ptr(rows), _ptr(sumsq), M, N, K, 0,
                       self._stream())
            return PreparedRows(rows, sumsq, sumsq.shape[0], hint)
        parts = self.lib.ts_gemm_tail_parts(M, N)
        if hint.weight.shape[1] != N or self._library_rows(M, N, K) \
                or self._library_rows(M, next_n, N) \
                or self.lib.ts_gemm_tail_fits(M, N, K) != 1 \
                or self.lib.ts_gemm_scaled_fits(M, next_n, N, int(hint.silu_mul), parts) != 1:
            return None
        self._check("resid", resid, torch.float32, shape=(M, N))
        self._check("norm weight", hint.norm_weight, torch.float32, shape=(N,))
        rows = torch.empty(M, N, dtype=torch.bfloat16, device=self.device)
        sumsq = torch.empty(M, -(-parts // 4) * 4, dtype=torch.float32, device=self.device)
        self._call(self.lib.ts_gemm_tail_bf16, _ptr(x), _ptr(weight), _ptr(resid),
                   _ptr(hint.norm_weight), _ptr(rows), _ptr(sumsq), M, N, K, self._stream())
        return PreparedRows(rows, sumsq, parts, hint)

    def _tiled_stream_ok(self, M, N, K, hint):
        """Whether the product [M, K] x [N, K] that ends a sub-layer, and the hinted norm
        and product behind it, are the LDS-tiled kernel's tail and scaled forms."""
        d = self.dispatch
        if M < d.tiled_stream_rows or hint.weight.shape[1] != N \
                or N * K > d.tiled_stream_weight or hint.weight.numel() > d.tiled_pair_weight:
            return False
        next_n = hint.weight.shape[0] // 2 if hint.silu_mul else hint.weight.shape[0]
        return (self.lib.ts_gemm_tiled_tail_fits(M, N, K) == 1
                and self.lib.ts_gemm_tiled_scaled_fits(
                    M, next_n, N, int(hint.silu_mul), self.lib.ts_gemm_tiled_tail_parts(N)) == 1)

    def _merged_into_stream(self, unmerged, x, weight, resid, hint):
        """`linear_into_stream` over an attention output that is still unmerged: one kernel
        merges the rows and multiplies, if it takes the sizes; else None, nothing done."""
        a = unmerged.args.base
        M, K = x.shape
        N = weight.shape[0]
        if len(x.shape) != 2 or K != a.nq * a.hd or weight.shape[1] != K or M != a.num_tokens \
                or hint.weight.shape[1] != N or M > self.merged_rows:
            return None
        next_n = hint.weight.shape[0] // 2 if hint.silu_mul else hint.weight.shape[0]
        parts = self.lib.ts_gemm_tail_parts(M, N)
        if self._library_rows(M, N, K) or self._library_rows(M, next_n, N) \
                or self.lib.ts_gemm_tail_merged_fits(M, N, a.nq, a.hd) != 1 \
                or self.lib.ts_gemm_scaled_fits(M, next_n, N, int(hint.silu_mul), parts) != 1:
            return None
        self._check("weight", weight, torch.bfloat16, ndim=2)
        self._check("resid", resid, torch.float32, shape=(M, N))
        self._check("norm weight", hint.norm_weight, torch.float32, shape=(N,))
        rows = torch.empty(M, N, dtype=torch.bfloat16, device=self.device)
        sumsq = torch.empty(M, -(-parts // 4) * 4, dtype=torch.float32, device=self.device)
        self._call(self.lib.ts_gemm_tail_merged_bf16, _ptr(unmerged.partial_o),
                   _ptr(unmerged.partial_ml), _ptr(unmerged.positions),
                   unmerged.args.num_splits, a.nq, a.nkv, a.hd,
                   0 if unmerged.window is None else int(unmerged.window), _ptr(weight),
                   _ptr(resid), _ptr(hint.norm_weight), _ptr(rows), _ptr(sumsq), M, N,
                   self._stream())
        return PreparedRows(rows, sumsq, parts, hint)

    def _prepared_linear(self, resid, prepared, norm_weight, eps, weight, out_dtype, silu_mul):
        hint = prepared.hint
        if hint.norm_weight is not norm_weight or hint.eps != eps or hint.weight is not weight \
                or hint.silu_mul != silu_mul:
            raise ValueError("norm_linear: the rows were prepared for another norm or product")
        M, K = prepared.rows.shape
        if resid.shape != (M, K):
            raise ValueError("norm_linear: prepared rows and stream differ in shape")
        N = weight.shape[0] // 2 if silu_mul else weight.shape[0]
        if out_dtype not in (torch.bfloat16, torch.float32) or (silu_mul and out_dtype != torch.bfloat16):
            raise ValueError(f"norm_linear: prepared rows cannot give {out_dtype}")
        out = torch.empty(M, N, dtype=out_dtype, device=self.device)
        if M >= self.dispatch.tiled_stream_rows:      # prepared by the tiled tail form
            self._call(self.lib.ts_gemm_tiled_scaled_bf16, _ptr(prepared.rows),
                       _ptr(prepared.sumsq), prepared.slices, c_float(eps), _ptr(weight),
                       _ptr(out), _TYPE_CODE[out_dtype], M, N, K, int(silu_mul), 0, self._stream())
            return out, resid
        self._call(self.lib.ts_gemm_scaled_bf16, _ptr(prepared.rows), _ptr(prepared.sumsq),
                   prepared.slices, c_float(eps), _ptr(weight), _ptr(out), _TYPE_CODE[out_dtype], M, N, K,
                   int(silu_mul), self._stream())
        return out, resid

    def norm_linear(self, resid, delta, norm_weight, eps, weight, out_dtype, silu_mul=False):
        """(RMSNorm(resid + delta) W^T, resid + delta): the residual add, the norm and
        the product in one kernel where it can be (bfloat16 weights, at most 16 rows);
        otherwise the same from separate kernels.  `delta` may be None.  With `silu_mul`
        the weight is [Wg; Wu] and the result silu(h Wg^T) * (h Wu^T).  The returned
        residual stream may or may not be the tensor passed in."""
        self._check("resid", resid, torch.float32, ndim=2)
        if isinstance(delta, PreparedRows):     # already added in, by linear_into_stream
            return self._prepared_linear(resid, delta, norm_weight, eps, weight, out_dtype,
                                         silu_mul)
        delta = self._rows(delta)
        M, K = resid.shape
        self._check("weight", weight, self._FLOATS, ndim=2)
        if weight.shape[1] != K:
            raise ValueError(f"norm_linear: stream width {K}, weight has {weight.shape[1]} columns")
        N = weight.shape[0] // 2 if silu_mul else weight.shape[0]
        fused = (weight.dtype == torch.bfloat16
                 and self.lib.ts_norm_gemm_mfma_fits(M, N, K) == 1
                 and (delta is None or delta.dtype == torch.bfloat16
                      or self.lib.ts_gemm_mfma_layout(N, K) == 2)
                 and (out_dtype == torch.bfloat16 or not silu_mul)
                 and out_dtype in (torch.bfloat16, torch.float32))
        if not fused:
            act = torch.bfloat16 if weight.dtype == torch.bfloat16 else torch.float32
            h = self.rmsnorm(resid, norm_weight, eps, act) if delta is None \
                else self.add_rmsnorm(resid, delta, norm_weight, eps, act)
            out = self.linear_silu_mul(h, weight, out_dtype) if silu_mul \
                else self.linear(h, weight, out_dtype)
            return out, resid
        self._check("norm weight", norm_weight, torch.float32, shape=(K,))
        if delta is not None:
            self._check("delta", delta, self._FLOATS, shape=resid.shape)
        if silu_mul and weight.shape[0] % 2:
            raise ValueError("norm_linear: stacked gate/up weight needs an even row count")
        out = torch.empty(M, N, dtype=out_dtype, device=self.device)
        resid_out = torch.empty_like(resid)
        self._call(self.lib.ts_norm_gemm_mfma_bf16, _ptr(resid), _ptr(delta),
                   _TYPE_CODE[delta.dtype] if delta is not None else 0,
                   1 if delta is not None else 0, _ptr(norm_weight), c_float(eps),
                   _ptr(resid_out), _ptr(weight), _ptr(out), _TYPE_CODE[out_dtype], M, N, K,
                   int(silu_mul), self._stream())
        return out, resid_out

    def linear_silu_mul(self, x, weight, out_dtype):
        """silu(x Wg^T) * (x Wu^T) for weight = [Wg; Wu] stacked by rows -> [M, N/2]."""
        x = self._rows(x)
        self._check("x", x, self._FLOATS, ndim=2)
        self._check("weight", weight, self._FLOATS, ndim=2)
        M, K = x.shape
        if weight.shape[1] != K or weight.shape[0] % 2:
            raise ValueError(f"linear_silu_mul: x {tuple(x.shape)}, weight {tuple(weight.shape)}")
        inner = weight.shape[0] // 2
        if self._tiled_pair_ok(x, weight, out_dtype):
            return self.gemm_tiled(x, weight, out_dtype, pair=True)
        if (self._mfma_ok(x, weight) and out_dtype == torch.bfloat16
                and not self._library_ok(x, weight, out_dtype)):
            out = torch.empty(M, inner, dtype=out_dtype, device=self.device)
            self._call(self.lib.ts_gemm_mfma_bf16, _ptr(x), _ptr(weight), _ptr(out),
                       _TYPE_CODE[out_dtype], M, inner, K, 1, self._stream())
            return out
        return self.silu_mul(self.linear(x, weight, out_dtype))

    # ------------------------------------------------------------ q/k preparation
    def _qk_args(self, qkv, batch, *, num_heads, kv_in_row, head_dim, q_weight, k_weight, eps,
                 cos_sin, row_extra=0):
        T = qkv.shape[0]
        if row_extra < 0 or row_extra % 8:
            raise ValueError(f"row_extra={row_extra} must be a multiple of 8")
        self._check("qkv", qkv, self._FLOATS,
                    shape=(T, (num_heads + 2 * kv_in_row) * head_dim + row_extra))
        if head_dim % 2:
            raise ValueError(f"head_dim={head_dim} must be even")
        a = QkPrepareArgs()
        a.qkv = qkv.data_ptr()
        a.num_tokens, a.nq, a.nkv, a.hd = T, num_heads, kv_in_row, head_dim
        a.eps, a.row_extra = eps, row_extra
        if q_weight is not None:
            a.q_weight = self._check("q norm weight", q_weight, torch.float32,
                                     shape=(head_dim,)).data_ptr()
        if k_weight is not None:
            a.k_weight = self._check("k norm weight", k_weight, torch.float32,
                                     shape=(head_dim,)).data_ptr()
        if cos_sin is not None:
            cos, sin = cos_sin
            self._check("cos", cos, torch.float32, ndim=2)
            self._check("sin", sin, torch.float32, shape=cos.shape)
            if cos.shape[1] != head_dim // 2:
                raise ValueError(f"rotary table has {cos.shape[1]} columns, "
                                 f"head_dim/2 is {head_dim // 2}")
            if batch.max_ctx_len > cos.shape[0]:
                raise ValueError(f"position {batch.max_ctx_len - 1} is beyond the rotary "
                                 f"table's {cos.shape[0]} rows")
            a.cos, a.sin, a.max_pos = cos.data_ptr(), sin.data_ptr(), cos.shape[0]
        self._check("positions", batch.positions, torch.int32, shape=(T,))
        self._check("entry_of_token", batch.entry_of_token, torch.int32, shape=(T,))
        a.positions = batch.positions.data_ptr()
        a.entry_of_token = batch.entry_of_token.data_ptr()
        return a

    def _check_cache(self, cache, table, batch, nkv, head_dim):
        P = cache.page_size
        self._check("k_pages", cache.k_pages, self._FLOATS,
                    shape=(cache.num_pages, nkv, P, head_dim))
        self._check("v_pages", cache.v_pages, cache.k_pages.dtype,
                    shape=(cache.num_pages, nkv, head_dim, P))
        self._check("block table", table, torch.int32, ndim=2)
        if table.shape[0] != batch.num_entries:
            raise ValueError("block table rows differ from the batch's entries")
        if table.shape[1] * P < batch.max_ctx_len:
            raise ValueError(
                f"block table of width {table.shape[1]} (page size {P}) cannot cover "
                f"{batch.max_ctx_len} positions")

    def qk_norm_rope_store(self, qkv, batch, table, cache, *, num_heads, num_kv_heads,
                           head_dim, q_weight, k_weight, eps, cos_sin, row_extra=0):
        """`row_extra`: further columns of a qkv row behind the heads (another product's
        results in the same rows), a multiple of 8."""
        a = self._qk_args(qkv, batch, num_heads=num_heads, kv_in_row=num_kv_heads,
                          head_dim=head_dim, q_weight=q_weight, k_weight=k_weight, eps=eps,
                          cos_sin=cos_sin, row_extra=row_extra)
        q = torch.empty(qkv.shape[0], num_heads, head_dim, dtype=qkv.dtype, device=self.device)
        a.q_out = q.data_ptr()
        cache_type = _TYPE_CODE[qkv.dtype]
        if cache is not None and num_kv_heads:
            self._check_cache(cache, table, batch, num_kv_heads, head_dim)
            a.k_dst, a.v_dst = cache.k_pages.data_ptr(), cache.v_pages.data_ptr()
            a.table, a.table_width = table.data_ptr(), table.shape[1]
            a.page_size, a.paged, a.store_kv = cache.page_size, 1, 1
            cache_type = _TYPE_CODE[cache.k_pages.dtype]
        self._call(self.lib.ts_qk_prepare, byref(a), _TYPE_CODE[qkv.dtype], cache_type,
                   self._stream())
        return q

    def qk_norm_split(self, qkv, *, num_heads, num_kv_heads, head_dim, q_weight, k_weight, eps):
        T = qkv.shape[0]

        class _B:   # positions are not used without a rotation or a paged store
            positions = torch.zeros(T, dtype=torch.int32, device=self.device)
            entry_of_token = positions
            max_ctx_len = 0
        a = self._qk_args(qkv, _B, num_heads=num_heads, kv_in_row=num_kv_heads,
                          head_dim=head_dim, q_weight=q_weight, k_weight=k_weight, eps=eps,
                          cos_sin=None)
        q = torch.empty(T, num_heads, head_dim, dtype=qkv.dtype, device=self.device)
        a.q_out = q.data_ptr()
        k = v = None
        if num_kv_heads:
            k = torch.empty(T, num_kv_heads, head_dim, dtype=qkv.dtype, device=self.device)
            v = torch.empty_like(k)
            a.k_dst, a.v_dst, a.paged, a.store_kv = k.data_ptr(), v.data_ptr(), 0, 1
        self._call(self.lib.ts_qk_prepare, byref(a), _TYPE_CODE[qkv.dtype],
                   _TYPE_CODE[qkv.dtype], self._stream())
        return q, k, v

    def rope_inplace(self, x, positions, cos, sin):
        self._check("x", x, self._FLOATS, ndim=3)
        T, heads, hd = x.shape
        self._check("positions", positions, torch.int32, shape=(T,))
        self._check("cos", cos, torch.float32, ndim=2)
        self._check("sin", sin, torch.float32, shape=cos.shape)
        if hd % 2 or cos.shape[1] != hd // 2:
            raise ValueError(f"rotary table has {cos.shape[1]} columns for head_dim {hd}")
        self._call(self.lib.ts_rope_inplace, _ptr(x), _TYPE_CODE[x.dtype], _ptr(positions),
                   _ptr(cos), _ptr(sin), T, heads, hd, self._stream())

    def kv_store(self, k, v, batch, table, cache):
        self._check("k", k, self._FLOATS, ndim=3)
        self._check("v", v, k.dtype, shape=k.shape)
        T, nkv, hd = k.shape
        self._check_cache(cache, table, batch, nkv, hd)
        self._check("positions", batch.positions, torch.int32, shape=(T,))
        self._call(self.lib.ts_kv_store, _ptr(k), _ptr(v), _TYPE_CODE[k.dtype],
                   _ptr(cache.k_pages), _ptr(cache.v_pages), _TYPE_CODE[cache.k_pages.dtype],
                   _ptr(batch.positions), _ptr(batch.entry_of_token), _ptr(table),
                   table.shape[1], T, nkv, hd, cache.page_size, self._stream())

    # ------------------------------------------------------------ attention
    def paged_attention(self, q, batch, table, cache, *, num_heads, num_kv_heads, head_dim,
                        scale, window, sink=None, chunk=None, softcap=None, slopes=None,
                        q_temp=None):
        """`sink`: float32 [num_heads] or None: a score per query head that joins the
        softmax's denominator once (not scaled, no key, no value).  `chunk`: a query sees
        the earlier keys of its own stretch of `chunk` positions, counted from position 0.
        Scores beyond scale times the product: `softcap` c (score <- c tanh(score / c)),
        `slopes` (float32 [num_heads]: slope times the distance to the key comes off),
        `q_temp` (coef, every): the query at position p counts 1 + coef ln(floor((p + 1) /
        every) + 1) times."""
        T = q.shape[0]
        self._check("q", q, self._FLOATS, shape=(T, num_heads, head_dim))
        self._check_cache(cache, table, batch, num_kv_heads, head_dim)
        if T != batch.num_tokens:
            raise ValueError("q rows differ from the batch's tokens")
        out = torch.empty_like(q)
        a = AttentionArgs()
        self._fill_attention_args(a, q, out, batch, table, cache, num_heads, num_kv_heads,
                                  head_dim, scale, window, sink, chunk, softcap, slopes, q_temp)
        extras = softcap is not None or slopes is not None or q_temp is not None
        if (q.dtype == torch.bfloat16 and cache.k_pages.dtype == torch.bfloat16
                and head_dim % 16 == 0 and head_dim <= 256 and cache.page_size % 4 == 0):
            # (scores with extras: the decode kernel and the kernel for short portions and
            # mixed steps know them, the LDS-tiled kernels for long portions do not)
            if self._decode_fits(batch, num_kv_heads, num_heads // num_kv_heads, head_dim,
                                 cache.page_size, False):
                self._attention_decode(a, batch, num_heads // num_kv_heads)
            else:
                self._attention_mfma(a, batch, num_heads // num_kv_heads, extras)
        else:
            self._call(self.lib.ts_attention_generic, byref(a), _TYPE_CODE[q.dtype],
                       _TYPE_CODE[cache.k_pages.dtype], self._stream())
        return out

    def attend(self, qkv, batch, table, cache, write_cache, *, num_heads, num_kv_heads,
               kv_in_row, head_dim, q_weight, k_weight, eps, cos_sin, scale, window,
               defer_merge=False, sink=None, row_extra=0, chunk=None, softcap=None,
               slopes=None, q_temp=None):
        """Everything between the q/k/v projection and the output projection: per-head
        norm of q and k, rotation, the write of k and v into `cache` (if `write_cache`;
        the row then brings `kv_in_row` = `num_kv_heads` key and value heads) and attention
        over the cache -> [T, num_heads, head_dim].  A decode step (one token per entry)
        in bfloat16 is one kernel; anything else is the preparation kernel and
        paged_attention.  With `defer_merge` the result may be an `UnmergedRows` handle of
        that shape instead of a tensor (the caller hands it to `linear_into_stream` or
        `linear`, or asks it for the tensor with `merged()`)."""
        T = qkv.shape[0]
        fused = (qkv.dtype == torch.bfloat16 and cache.k_pages.dtype == torch.bfloat16
                 and bool(write_cache) == bool(kv_in_row)
                 and self._decode_fits(batch, num_kv_heads, num_heads // num_kv_heads,
                                       head_dim, cache.page_size, True))
        if not fused:
            q = self.qk_norm_rope_store(
                qkv, batch, table, cache if write_cache else None, num_heads=num_heads,
                num_kv_heads=kv_in_row, head_dim=head_dim, q_weight=q_weight,
                k_weight=k_weight, eps=eps, cos_sin=cos_sin, row_extra=row_extra)
            return self.paged_attention(q, batch, table, cache, num_heads=num_heads,
                                        num_kv_heads=num_kv_heads, head_dim=head_dim,
                                        scale=scale, window=window, sink=sink, chunk=chunk,
                                        softcap=softcap, slopes=slopes, q_temp=q_temp)
        # the same argument checks as the preparation kernel's
        qa = self._qk_args(qkv, batch, num_heads=num_heads, kv_in_row=kv_in_row,
                           head_dim=head_dim, q_weight=q_weight, k_weight=k_weight, eps=eps,
                           cos_sin=cos_sin, row_extra=row_extra)
        self._check_cache(cache, table, batch, num_kv_heads, head_dim)
        if T != batch.num_tokens or T != batch.num_entries:
            raise ValueError("a decode step brings one token per entry")
        out = torch.empty(T, num_heads, head_dim, dtype=qkv.dtype, device=self.device)
        a = AttentionArgs()
        self._fill_attention_args(a, None, out, batch, table, cache, num_heads, num_kv_heads,
                                  head_dim, scale, window, sink, chunk, softcap, slopes, q_temp)
        if sink is not None or chunk is not None:
            defer_merge = False        # the product that merges for itself knows neither
        d = AttentionDecodeArgs()
        d.qkv, d.q_weight, d.k_weight = qa.qkv, qa.q_weight, qa.k_weight
        d.cos, d.sin, d.eps, d.kv_in_row = qa.cos, qa.sin, eps, kv_in_row
        d.row_extra = row_extra
        pending = self._attention_decode(a, batch, num_heads // num_kv_heads, d,
                                         out if defer_merge else None, window)
        return out if pending is None else UnmergedRows(pending, out.shape)

    def _attention_decode(self, a, batch, group, d=None, defer_out=None, window=None):
        """One token per entry: workgroups per (entry, key/value head, share of the keys).
        `defer_out`: the output tensor, if the merge of the splits may be left undone; then
        the pending merge is returned (else None)."""
        d = d or AttentionDecodeArgs()
        m = d.m
        m.base = a
        m.rows_per_token, m.head_blocks = min(group, 16), -(-group // 16)
        m.num_tiles = batch.num_entries
        items = m.num_tiles * a.nkv * m.head_blocks
        reach = self._reach(a)
        span = batch.max_ctx_len if reach == 0 else min(batch.max_ctx_len,
                                                        reach + self._attn_chunk)
        m.num_splits = self._decode_splits(items, span)
        if m.num_splits > 1:
            po = torch.empty(items * m.num_splits * 16 * a.hd, dtype=torch.float32,
                             device=self.device)
            pml = torch.empty(items * m.num_splits * 16 * 2, dtype=torch.float32,
                              device=self.device)
            m.partial_o, m.partial_ml = po.data_ptr(), pml.data_ptr()
            if defer_out is not None and batch.num_entries <= self.merged_rows:
                d.defer_merge = 1
            elif self.fold_merge and items <= self._arrivals.numel():
                d.arrivals = self._arrivals.data_ptr()
        self._call(self.lib.ts_attention_decode, byref(d), self._stream())
        if d.defer_merge:
            kept = AttentionMfmaArgs.from_buffer_copy(m)
            return _PendingMerge(self, defer_out, kept, po, pml, batch.positions, window)
        return None

    def _decode_fits(self, batch, num_kv_heads, group, head_dim, page_size, fused):
        items = batch.num_entries * num_kv_heads * -(-group // 16)
        return (batch.max_q_len == 1 and items <= self.dispatch.decode_items
                and self.lib.ts_attention_decode_fits(head_dim, page_size, int(fused)) == 1)

    def _decode_splits(self, items, span):
        """Workgroups per tile: enough to give every compute unit one, never more than the
        context has 128-key chunks (a split without chunks costs an idle workgroup and a
        line of the merge).  Measured in decode steps of 8 to 32 entries at 16 query / 8
        key heads of 128: a workgroup per unit is as good as three quarters of that at 800
        tokens of context and better beyond (16 entries at 4,096 tokens: 2.04 against
        2.33 ms a step); half as many again, twice or three times as many are slower
        everywhere."""
        max_chunks = max(1, -(-span // self._attn_chunk))
        return min(max_chunks, max(1, self._units // items))

    @staticmethod
    def _reach(a):
        """How many keys a query sees at most (0: all earlier ones), by window and chunk."""
        if a.window and a.chunk:
            return min(a.window, a.chunk)
        return a.window or a.chunk

    def _attention_mfma(self, a, batch, group, extras=False):
        """Tile the batch's queries (16 rows of q heads x tokens per wavefront), choose how
        many waves share a tile's keys, and launch."""
        rows_per_token = min(group, 16)
        head_blocks = -(-group // 16)
        tokens_per_tile = 16 // rows_per_token
        m = AttentionMfmaArgs()
        m.base = a
        m.rows_per_token, m.head_blocks = rows_per_token, head_blocks
        # long portions of prompts: a wavefront takes several query tiles and walks alone
        # (scores with extras: those of these kernels that know them take pages of a power of
        # two from 16)
        page16 = a.page_size >= 16 and a.page_size & (a.page_size - 1) == 0
        if (not extras or page16) and self._prefill_tiles(batch, a.nkv, group) is not None:
            tiles16 = sum(-(-n // tokens_per_tile) for n in batch.q_lens)
            tpw = self.lib.ts_attention_prefill_tiles(a.hd, a.page_size, tiles16,
                                                      a.nkv * head_blocks)
            tiles_dev, num_tiles = self._attention_tiles(batch, tokens_per_tile * tpw,
                                                         longest_first=True)
            m.tiles, m.num_tiles, m.tiles_per_wave = tiles_dev.data_ptr(), num_tiles, tpw
            m.num_splits = 1
            self._call(self.lib.ts_attention_prefill, byref(m), self._stream())
            return
        if batch.max_q_len == 1:           # decode: tile i is entry i, no list needed
            tiles_dev, num_tiles = None, batch.num_entries
        else:
            tiles_dev, num_tiles = self._attention_tiles(batch, tokens_per_tile)
        items = num_tiles * a.nkv * head_blocks
        chunk = self._attn_chunk
        reach = self._reach(a)
        span = batch.max_ctx_len if reach == 0 else min(batch.max_ctx_len,
                                                        reach + batch.max_q_len + chunk)
        max_chunks = max(1, -(-span // chunk))
        # few tiles (decode): a workgroup per tile and chunk, its waves share the chunk;
        # many tiles (prompts): a wavefront per tile walks its keys
        d = self.dispatch
        cooperative = items <= d.cooperative_items
        splits = min(max_chunks, max(1, (d.cooperative_workgroups if cooperative
                                         else d.per_wave_workgroups) // items))
        m.cooperative = int(cooperative)
        m.tiles = tiles_dev.data_ptr() if tiles_dev is not None else None
        m.num_tiles = num_tiles
        m.num_splits = splits
        if splits > 1:
            po = torch.empty(items * splits * 16 * a.hd, dtype=torch.float32, device=self.device)
            pml = torch.empty(items * splits * 16 * 2, dtype=torch.float32, device=self.device)
            m.partial_o, m.partial_ml = po.data_ptr(), pml.data_ptr()
        self._call(self.lib.ts_attention_mfma, byref(m), self._stream())

    def _prefill_tiles(self, batch, num_kv_heads, group):
        """Tokens per 16-row tile if the step goes to the kernel for long portions (enough
        16-row wave tiles for the kernel whose waves share key/value blocks through LDS;
        the counts and what they were measured on: kernels/dispatch.py), else None."""
        tokens_per_tile = 16 // min(group, 16)
        tiles16 = sum(-(-n // tokens_per_tile) for n in batch.q_lens)
        waves = tiles16 * num_kv_heads * -(-group // 16)
        d = self.dispatch
        enough = d.portion_tiles if batch.max_q_len >= d.portion_tokens else d.single_token_tiles
        return tokens_per_tile if waves >= enough else None

    def _attention_tiles(self, batch, tokens, longest_first=False):
        """Device list of (entry, first flat token, tokens) cutting every entry of the batch
        into runs of at most `tokens` consecutive tokens; made once per step and size.
        `longest_first`: sorted by the number of keys a run's last token sees, most first
        (the kernels for long portions pair runs from both ends of that order)."""
        key = ("attn_tiles", tokens, longest_first)
        if key not in batch.plans and batch.max_q_len == 1:
            # a step of single tokens: tile i is entry i.  No order: the host's `starts` of a
            # captured decode batch are placeholders, and the order is a hint for the
            # kernel's balance only, never for what it computes (it reads positions and
            # lengths on the device).
            tiles = [(entry, entry, 1) for entry in range(batch.num_entries)]
            batch.plans[key] = (self._upload_ints(tiles), len(tiles))
        if key not in batch.plans:
            tiles, keys = [], []
            first = 0
            for entry, (n, start) in enumerate(zip(batch.q_lens, batch.starts)):
                for t0 in range(0, n, tokens):
                    m = min(tokens, n - t0)
                    tiles.append((entry, first + t0, m))
                    keys.append(start + t0 + m)
                first += n
            if longest_first:
                order = sorted(range(len(tiles)), key=lambda i: -keys[i])
                tiles = [tiles[i] for i in order]
            batch.plans[key] = (self._upload_ints(tiles), len(tiles))
        return batch.plans[key]

    def _upload_ints(self, rows):
        """A list of equally long int tuples as an int32 device tensor, copied out of pinned
        memory (a copy out of pageable memory holds the host until it is done, and the step's
        first attention call, which the GPU is waiting for, makes this list).  Four buffers
        in turn, each free again once its last copy has been made."""
        host = np.asarray(rows, dtype=np.int32)
        if self.device.type != "cuda":
            return torch.from_numpy(host).to(self.device)
        turn = self._staging_turn = (self._staging_turn + 1) % len(self._staging)
        slot = self._staging[turn]
        if slot is None or slot[0].numel() < host.size:
            slot = (torch.empty(max(host.size, 1 << 14), dtype=torch.int32, pin_memory=True),
                    torch.cuda.Event())
            self._staging[turn] = slot
        else:
            slot[1].synchronize()
        # (written through numpy: the buffer may have been made under inference mode, which
        # forbids a tensor's own in-place copy outside it)
        slot[0].numpy()[:host.size] = host.reshape(-1)
        dev = slot[0][:host.size].view(host.shape).to(self.device, non_blocking=True)
        slot[1].record()
        return dev

    def _fill_attention_args(self, a, q, out, batch, table, cache, num_heads, num_kv_heads,
                             head_dim, scale, window, sink=None, chunk=None, softcap=None,
                             slopes=None, q_temp=None):
        T = out.shape[0]
        if chunk is not None:
            if int(chunk) < 1:
                raise ValueError(f"chunk={chunk} must be positive")
            a.chunk = int(chunk)
        if softcap is not None:
            if not softcap > 0:
                raise ValueError(f"softcap={softcap} must be positive")
            a.softcap = float(softcap)
        if slopes is not None:
            a.slopes = self._check("slopes", slopes, torch.float32, shape=(num_heads,)).data_ptr()
        if q_temp is not None:
            coef, every = q_temp
            if int(every) < 1:
                raise ValueError(f"q_temp: every={every} must be positive")
            a.temp_coef, a.temp_every = float(coef), int(every)
        if sink is not None:
            a.sink = self._check("sink", sink, torch.float32, shape=(num_heads,)).data_ptr()
        a.q, a.out = (q.data_ptr() if q is not None else None), out.data_ptr()
        a.k_pages, a.v_pages = cache.k_pages.data_ptr(), cache.v_pages.data_ptr()
        a.positions, a.entry_of_token = batch.positions.data_ptr(), batch.entry_of_token.data_ptr()
        a.q_start, a.ctx_len = batch.q_start.data_ptr(), batch.ctx_len.data_ptr()
        a.table, a.table_width = table.data_ptr(), table.shape[1]
        a.num_tokens, a.num_entries = T, batch.num_entries
        a.nq, a.nkv, a.hd = num_heads, num_kv_heads, head_dim
        a.page_size, a.num_pages = cache.page_size, cache.num_pages
        a.window = 0 if window is None else int(window)
        a.scale = scale

    # ------------------------------------------------------------ sampling
    def argmax(self, logits):
        self._check("logits", logits, torch.float32, ndim=2)
        R, V = logits.shape
        out = torch.empty(R, dtype=torch.int32, device=self.device)
        part_v, part_i = self._pick_scratch(R, V)
        self._call(self.lib.ts_argmax, _ptr(logits), _ptr(out), _ptr(part_v), _ptr(part_i), R, V,
                   self._stream())
        return out

    def _pick_scratch(self, rows, vocab):
        slices = self.lib.ts_pick_slices(vocab)
        return (torch.empty(rows * slices, dtype=torch.float32, device=self.device),
                torch.empty(rows * slices, dtype=torch.int32, device=self.device))

    def sample(self, logits, temperatures, keys, out=None):
        """Row r: greedy if temperatures[r] <= 1e-10, else a draw from
        softmax(logits[r] / T) with noise keyed by keys[r] (int64 bit pattern).  Into
        `out` (int32, one per row) if given."""
        self._check("logits", logits, torch.float32, ndim=2)
        R = logits.shape[0]
        self._check("temperatures", temperatures, torch.float32, shape=(R,))
        self._check("keys", keys, torch.int64, shape=(R,))
        if out is None:
            out = torch.empty(R, dtype=torch.int32, device=self.device)
        else:
            self._check("out", out, torch.int32, shape=(R,))
        part_v, part_i = self._pick_scratch(R, logits.shape[1])
        self._call(self.lib.ts_sample, _ptr(logits), _ptr(temperatures), _ptr(keys), _ptr(out),
                   _ptr(part_v), _ptr(part_i), R, logits.shape[1], self._stream())
        return out

    # ------------------------------------------------------------ sandwich-norm rows
    def _batch_ptrs(self, batch, T):
        self._check("positions", batch.positions, torch.int32, shape=(T,))
        self._check("entry_of_token", batch.entry_of_token, torch.int32, shape=(T,))
        self._check("q_start", batch.q_start, torch.int32, shape=(batch.num_entries + 1,))
        self._check("slot_ids", batch.slot_ids, torch.int32, shape=(batch.num_entries,))
        if T != batch.num_tokens:
            raise ValueError(f"{T} rows for a batch of {batch.num_tokens} tokens")
        return (_ptr(batch.positions), _ptr(batch.entry_of_token), _ptr(batch.q_start),
                _ptr(batch.slot_ids))

    def _check_state(self, name, state, shape, dtype=torch.float32):
        self._check(name, state, dtype, ndim=len(shape) + 1)
        if tuple(state.shape[1:]) != tuple(shape):
            raise ValueError(f"{name}: shape {tuple(state.shape)}, expected [slots, "
                             f"{', '.join(str(s) for s in shape)}]")

    def bigram_embed(self, table, bigram, norm_w, batch, prev_state, *, scale, buckets,
                     mul_prev, mul_cur, eps):
        """norm(table[id] * scale + bigram[row]) -> float32 [T, width]; row hashes the
        previous and the current token (`prev_state` [slots, 1] int32 keeps a request's
        last token between steps), the last row serves a sequence's first token."""
        self._check("embedding table", table, self._FLOATS, ndim=2)
        W = table.shape[1]
        self._check("bigram table", bigram, table.dtype, shape=(buckets + 1, W))
        self._check("norm weight", norm_w, torch.float32, shape=(W,))
        self._check("token ids", batch.token_ids, torch.int32, ndim=1)
        T = batch.token_ids.shape[0]
        pos, eot, qs, slots = self._batch_ptrs(batch, T)
        self._check_state("previous tokens", prev_state, (1,), torch.int32)
        out = torch.empty(T, W, dtype=torch.float32, device=self.device)
        self._call(self.lib.ts_bigram_embed, _ptr(table), _ptr(bigram), _TYPE_CODE[table.dtype],
                   _ptr(norm_w), _ptr(batch.token_ids), pos, eot, qs, slots, _ptr(prev_state),
                   _ptr(out), T, W, c_float(scale), int(buckets), int(mul_prev), int(mul_cur),
                   c_float(eps), self._stream())
        return out

    def postnorm_add(self, resid, delta, post_w, eps):
        """resid += delta / rms(delta) * post_w, in place (float32)."""
        self._postnorm(resid, delta, post_w, eps, None, 0.0, None)

    def postnorm_add_norm(self, resid, delta, post_w, post_eps, norm_w, norm_eps, out_dtype):
        """The same, and the norm (norm_w, norm_eps) of the new resid in `out_dtype`."""
        return self._postnorm(resid, delta, post_w, post_eps, norm_w, norm_eps, out_dtype)

    def _postnorm(self, resid, delta, post_w, post_eps, norm_w, norm_eps, out_dtype):
        delta = self._rows(delta)
        self._check("resid", resid, torch.float32, ndim=2)
        self._check("delta", delta, torch.float32, shape=resid.shape)
        W = resid.shape[1]
        self._check("post-norm weight", post_w, torch.float32, shape=(W,))
        out = None
        if norm_w is not None:
            self._check("norm weight", norm_w, torch.float32, shape=(W,))
            out = torch.empty(resid.shape, dtype=out_dtype, device=self.device)
        self._call(self.lib.ts_postnorm_add, _ptr(resid), _ptr(delta), _ptr(post_w),
                   c_float(post_eps), _ptr(norm_w), c_float(norm_eps), _ptr(out),
                   _TYPE_CODE[out_dtype] if out is not None else 0, resid.shape[0], W,
                   self._stream())
        return out

    def norm_token_shift(self, resid, norm_w, eps, shift_w, batch, state, out_dtype):
        """h = norm(resid); out_t = h_t + (h_(t-1) - h_t) * shift_w.  `state` [slots, width]
        float32 carries a request's last h from step to step."""
        self._check("resid", resid, torch.float32, ndim=2)
        T, W = resid.shape
        self._check("norm weight", norm_w, torch.float32, shape=(W,))
        self._check("shift weight", shift_w, torch.float32, shape=(W,))
        self._check_state("shift state", state, (W,))
        pos, eot, qs, slots = self._batch_ptrs(batch, T)
        out = torch.empty(T, W, dtype=out_dtype, device=self.device)
        self._call(self.lib.ts_norm_token_shift, _ptr(resid), _ptr(norm_w), c_float(eps),
                   _ptr(shift_w), _ptr(state), _ptr(out), _TYPE_CODE[out_dtype], pos, eot, qs,
                   slots, T, W, self._stream())
        return out

    def polynorm(self, z, coef, eps, out_dtype):
        """a N(z) + b N(z^2) + c N(z^3) + e with N(v) = v / rms(v) per row; coef = (a, b, c, e)."""
        self._check("z", z, torch.float32, ndim=2)
        self._check("coefficients", coef, torch.float32, shape=(4,))
        out = torch.empty(z.shape, dtype=out_dtype, device=self.device)
        self._call(self.lib.ts_polynorm, _ptr(z), _ptr(coef), _ptr(out), _TYPE_CODE[out_dtype],
                   z.shape[0], z.shape[1], c_float(eps), self._stream())
        return out

    # ------------------------------------------------------------ state-space mixer
    def conv_silu(self, proj, col, channels, weight, bias, batch, state, in_bias=None,
                  plain=False):
        """Causal convolution per channel over columns [col, col + channels) of `proj`
        (float32 [T, ld]), bias, SiLU -> float32 [T, channels].  weight [channels, taps]
        (the last tap is the current token's); `state` [slots, taps - 1, channels] carries
        a request's last inputs.  `in_bias` [channels]: added to every input of the sequence
        before the convolution (the zeros in front of a sequence stay zeros); `plain`: no
        activation behind it."""
        self._check("proj", proj, torch.float32, ndim=2)
        T, ld = proj.shape
        self._check("conv weight", weight, torch.float32, ndim=2)
        taps = weight.shape[1]
        if weight.shape[0] != channels or col < 0 or col + channels > ld:
            raise ValueError(f"conv_silu: {channels} channels from column {col} of {ld}, "
                             f"weight {tuple(weight.shape)}")
        if bias is not None:
            self._check("conv bias", bias, torch.float32, shape=(channels,))
        if in_bias is not None:
            self._check("conv input bias", in_bias, torch.float32, shape=(channels,))
        self._check_state("conv state", state, (taps - 1, channels))
        pos, eot, qs, slots = self._batch_ptrs(batch, T)
        out = torch.empty(T, channels, dtype=torch.float32, device=self.device)
        self._call(self.lib.ts_conv_silu, _ptr(proj), ld, col, channels, taps, _ptr(weight),
                   _ptr(bias), _ptr(state), _ptr(out), pos, eot, qs, slots, T,
                   batch.num_entries, int(batch.max_q_len), _ptr(in_bias), int(bool(plain)),
                   self._stream())
        return out

    def ssm_scan(self, xbc, proj, dt_col, dt_bias, a_log, d_skip, batch, state, *, heads, vdim,
                 state_rows, groups):
        """The recurrence S <- exp(-exp(A_log) d) S + d B x^T, y = S^T C + D x per head,
        d = softplus(dt + dt_bias), over each entry's tokens in order -> float32
        [T, heads * vdim].  xbc [T, heads*vdim + 2*groups*state_rows]; dt is `heads`
        columns of `proj` from `dt_col`; `state` [slots, heads, state_rows, vdim]."""
        inner, N = heads * vdim, state_rows
        self._check("xbc", xbc, torch.float32, ndim=2)
        T = xbc.shape[0]
        if xbc.shape[1] != inner + 2 * groups * N:
            raise ValueError(f"ssm_scan: xbc has {xbc.shape[1]} columns, expected "
                             f"{inner + 2 * groups * N}")
        self._check("proj", proj, torch.float32, ndim=2)
        if proj.shape[0] != T or dt_col < 0 or dt_col + heads > proj.shape[1]:
            raise ValueError("ssm_scan: dt columns outside the projection")
        for name, v in (("dt_bias", dt_bias), ("A_log", a_log), ("D", d_skip)):
            self._check(name, v, torch.float32, shape=(heads,))
        self._check_state("recurrent state", state, (heads, N, vdim))
        pos, eot, qs, slots = self._batch_ptrs(batch, T)
        y = torch.empty(T, inner, dtype=torch.float32, device=self.device)
        # a step with a long portion runs its entries in chunks side by side (the lists are
        # the step's: every recurrent layer of the model uses the same)
        chunks, entry_chunks, num_chunks = self._scan_chunks(batch)
        scratch = decays = None
        if num_chunks:
            scratch = torch.empty(num_chunks, heads, N, vdim, dtype=torch.float32,
                                  device=self.device)
            decays = torch.empty(num_chunks, heads, dtype=torch.float32, device=self.device)
        self._call(self.lib.ts_ssm_scan, _ptr(xbc), _ptr(proj), proj.shape[1], dt_col,
                   _ptr(dt_bias), _ptr(a_log), _ptr(d_skip), _ptr(state), _ptr(y), pos, eot, qs,
                   slots, T, batch.num_entries, heads, vdim, N, groups, _ptr(chunks),
                   _ptr(entry_chunks), num_chunks, _ptr(scratch), _ptr(decays), self._stream())
        return y

    def _scan_chunks(self, batch):
        """(chunk list, chunks of each entry, number of chunks) for a step with a portion long
        enough to run in chunks side by side, else (None, None, 0).  The lists are the
        step's: every recurrent layer of the model uses the same."""
        if batch.max_q_len <= self.dispatch.scan_whole_tokens:
            return None, None, 0
        if "scan_chunks" not in batch.plans:
            size, rows, firsts, t0 = self.lib.ts_ssm_scan_chunk(), [], [0], 0
            for e, n in enumerate(batch.q_lens):
                rows += [(t0 + c, min(t0 + c + size, t0 + n), e) for c in range(0, n, size)]
                firsts.append(len(rows))
                t0 += n
            batch.plans["scan_chunks"] = (self._upload_ints(rows), self._upload_ints(firsts),
                                          len(rows))
        return batch.plans["scan_chunks"]

    def gated_group_norm(self, y, proj, norm_w, groups, eps, out_dtype):
        """(y * silu(z)) normalised in `groups` equal parts, times norm_w; z is the first
        y.shape[1] columns of `proj`."""
        self._check("y", y, torch.float32, ndim=2)
        T, inner = y.shape
        self._check("proj", proj, torch.float32, ndim=2)
        if proj.shape[0] != T or proj.shape[1] < inner or inner % groups:
            raise ValueError("gated_group_norm: shapes do not fit")
        self._check("norm weight", norm_w, torch.float32, shape=(inner,))
        out = torch.empty(T, inner, dtype=out_dtype, device=self.device)
        self._call(self.lib.ts_gated_group_norm, _ptr(y), _ptr(proj), proj.shape[1], _ptr(norm_w),
                   _ptr(out), _TYPE_CODE[out_dtype], T, inner, groups, c_float(eps),
                   self._stream())
        return out

    # ------------------------------------------------------------ matrix-state mixers
    def delta_gates(self, qkv, proj, beta_col, z, z_col, a_log, dt_bias, *, heads, kv_heads, dim,
                    per_channel):
        """The gated delta rule's operands.  In place on `qkv` (float32 [T, q | k | v]): every
        q and k head of `dim` columns becomes a unit vector (eps 1e-6 inside the root), q also
        times dim^-1/2.  Returns float32 [T, heads + n]: beta = sigmoid(proj[:, beta_col + h]),
        then g = exp(-exp(a_log[h]) softplus(z[:, z_col + j] + dt_bias[j])) for j over the
        heads (n = heads) or, `per_channel`, over heads x dim."""
        self._check("qkv", qkv, torch.float32, ndim=2)
        T = qkv.shape[0]
        self._check("proj", proj, torch.float32, ndim=2)
        self._check("z", z, torch.float32, ndim=2)
        n = heads * dim if per_channel else heads
        self._check("A_log", a_log, torch.float32, shape=(heads,))
        self._check("dt_bias", dt_bias, torch.float32, shape=(n,))
        if proj.shape[0] != T or z.shape[0] != T:
            raise ValueError("delta_gates: row counts differ")
        gates = torch.empty(T, heads + n, dtype=torch.float32, device=self.device)
        self._call(self.lib.ts_delta_gates, _ptr(qkv), qkv.shape[1], _ptr(proj), proj.shape[1],
                   int(beta_col), _ptr(z), z.shape[1], int(z_col), _ptr(a_log), _ptr(dt_bias),
                   _ptr(gates), heads + n, T, heads, kv_heads, dim, int(bool(per_channel)),
                   self._stream())
        return gates

    def linear_recurrence(self, x, q_col, k_col, v_col, batch, state, *, heads, kv_heads, dim,
                          vdim, silu_inputs, decay=None, gates=None, per_channel=False,
                          delta=False):
        """Per head and entry, a token at a time: S <- g S; u = v, or (`delta`)
        u = beta (v - S^T k); S <- S + k u^T; o = S^T q -> float32 [T, heads * vdim].
        `x` (float32 [T, ld]) holds q and k (kv_heads x dim; head h reads q/k head
        h // (heads / kv_heads)) and v (heads x vdim) from the given columns, their SiLU taken
        on the way if `silu_inputs`.  g is `decay` [heads] (fixed), or comes with beta from
        `gates` ([T, heads + n] as `delta_gates` lays it out, `per_channel`: one g per row of
        S).  `state` [slots, heads, dim, vdim] float32 carries S from step to step."""
        self._check("x", x, torch.float32, ndim=2)
        T, ld = x.shape
        self._check_state("recurrent state", state, (heads, dim, vdim))
        if decay is not None:
            self._check("decay", decay, torch.float32, shape=(heads,))
        ldg = 0
        if gates is not None:
            ldg = heads + (heads * dim if per_channel else heads)
            self._check("gates", gates, torch.float32, shape=(T, ldg))
        pos, eot, qs, slots = self._batch_ptrs(batch, T)
        out = torch.empty(T, heads * vdim, dtype=torch.float32, device=self.device)
        # without the delta rule a long portion runs in chunks side by side
        chunks = entry_chunks = scratch = decays = None
        num_chunks = 0
        if not delta and dim <= 128:
            chunks, entry_chunks, num_chunks = self._scan_chunks(batch)
        if num_chunks:
            scratch = torch.empty(num_chunks, heads, dim, vdim, dtype=torch.float32,
                                  device=self.device)
            decays = torch.empty(num_chunks, heads, dtype=torch.float32, device=self.device)
        self._call(self.lib.ts_linear_recurrence, _ptr(x), ld, int(q_col), int(k_col), int(v_col),
                   _ptr(decay), _ptr(gates), ldg, _ptr(state), _ptr(out), pos, eot, qs, slots, T,
                   batch.num_entries, int(batch.max_q_len), heads, kv_heads, dim, vdim,
                   int(bool(silu_inputs)), int(bool(delta)), int(bool(per_channel)),
                   _ptr(chunks), _ptr(entry_chunks), num_chunks, _ptr(scratch), _ptr(decays),
                   self._stream())
        return out

    def norm_gate(self, y, gate_rows, gate_col, norm_w, *, groups, gate, eps, out_dtype):
        """Each of `groups` equal parts of a row of y (float32) over its root mean square,
        times norm_w (one value per column of a part, shared by the parts, or one per column
        of the row), times sigmoid or SiLU (`gate`) of columns [gate_col, gate_col + width) of
        `gate_rows` (float32)."""
        self._check("y", y, torch.float32, ndim=2)
        T, inner = y.shape
        self._check("gate rows", gate_rows, torch.float32, ndim=2)
        self._check("norm weight", norm_w, torch.float32, ndim=1)
        if gate not in ("sigmoid", "silu"):
            raise ValueError(f"norm_gate: gate {gate!r}; built are sigmoid and silu")
        if gate_rows.shape[0] != T:
            raise ValueError("norm_gate: row counts differ")
        out = torch.empty(T, inner, dtype=out_dtype, device=self.device)
        self._call(self.lib.ts_norm_gate, _ptr(y), _ptr(gate_rows), gate_rows.shape[1],
                   int(gate_col), _ptr(norm_w), norm_w.shape[0], _ptr(out), _TYPE_CODE[out_dtype],
                   T, inner, int(groups), 0 if gate == "sigmoid" else 1, c_float(eps),
                   self._stream())
        return out

    # ------------------------------------------------------------ routed experts
    def route_experts(self, logits, *, top, group_count=1, group_keep=1, scores="softmax",
                      normalize=True, correction=None, weight_scale=1.0):
        """Router logits (float32 [T, experts]) -> float32 [T, experts]: a token's weight for
        each of its `top` experts (softmax score over the chosen scores' sum), zero elsewhere.
        Only experts of the `group_keep` best of `group_count` groups of neighbours can be
        chosen (a group's score: its best expert's).  `scores` "sigmoid": an expert's score is
        the sigmoid of its logit; `normalize` False: the weights are the chosen scores as
        they are.  `correction` (float32 [experts]): groups and experts are ranked by score +
        correction (softmax scores), the weights stay the scores; `weight_scale`: a factor on
        the weights."""
        if scores not in ("softmax", "sigmoid"):
            raise ValueError(f"route_experts: scores={scores!r}")
        self._check("router logits", logits, torch.float32, ndim=2)
        T, E = logits.shape
        if correction is not None:
            self._check("correction", correction, torch.float32, shape=(E,))
        weights = torch.empty(T, E, dtype=torch.float32, device=self.device)
        self._call(self.lib.ts_route_experts, _ptr(logits), _ptr(weights), T, E, int(top),
                   int(group_count), int(group_keep), int(scores == "sigmoid"),
                   int(bool(normalize)), _ptr(correction), c_float(weight_scale), self._stream())
        return weights

    def expert_activation(self, gate_up, weights, inner, limit, out_dtype, weighted_input=False,
                          form=None, experts=None, shared_inner=0):
        """gate_up [T, experts x (gate | up)] -> [T, experts x inner]: with g = min(gate,
        limit), u = clamp(up, -limit, limit): g sigmoid(1.702 g) (u + 1) times the token's
        weight for the expert (zeros where it is zero).  `weighted_input`: the expert is a
        plain gated unit that read the token times its weight w: silu(w gate) (w up).
        `form` "silu": silu(gate) up times the weight; the weights' first `experts` columns
        are the experts' (further columns belong to experts without weights), and behind the
        experts' columns gate_up holds `shared_inner` gate and as many up columns of a unit
        that every token uses with the weight one -> [T, experts x inner + shared_inner]."""
        gate_up = self._rows(gate_up)
        self._check("gate_up", gate_up, self._FLOATS, ndim=2)
        T = gate_up.shape[0]
        self._check("expert weights", weights, torch.float32, ndim=2)
        if form == "silu":
            E = weights.shape[1] if experts is None else int(experts)
            width = E * inner + int(shared_inner)
            if weights.shape[0] != T or E > weights.shape[1] or gate_up.shape[1] != 2 * width \
                    or out_dtype != gate_up.dtype:
                raise ValueError(f"expert_activation: gate_up {tuple(gate_up.shape)} for {E} "
                                 f"experts of {inner} and {shared_inner} shared columns")
            out = torch.empty(T, width, dtype=out_dtype, device=self.device)
            self._call(self.lib.ts_expert_silu, _ptr(gate_up), _ptr(weights), _ptr(out),
                       _TYPE_CODE[out_dtype], T, E, int(inner), int(shared_inner),
                       weights.shape[1], self._stream())
            return out
        if form is not None:
            raise ValueError(f"expert_activation: form={form!r}")
        E = weights.shape[1]
        if weights.shape[0] != T or gate_up.shape[1] != E * 2 * inner or out_dtype != gate_up.dtype:
            raise ValueError(f"expert_activation: gate_up {tuple(gate_up.shape)} for {E} experts "
                             f"of {inner} columns, out {out_dtype}")
        out = torch.empty(T, E * inner, dtype=out_dtype, device=self.device)
        self._call(self.lib.ts_expert_activation, _ptr(gate_up), _ptr(weights), _ptr(out),
                   _TYPE_CODE[out_dtype], T, E, int(inner), c_float(limit),
                   int(bool(weighted_input)), self._stream())
        return out

    # ------------------------------------------------------------ gated diagonal recurrence
    def rglru_gates(self, u, w_a, w_i, b_a, b_i, rate):
        """The recurrence's operands from its input u (float32 [T, width]): per block of
        channels r = sigmoid(w_a[b] u_b + b_a), i = sigmoid(w_i[b] u_b + b_i) (w [blocks, bw,
        bw], [out, in] per block), log a = rate * r -> (a, sqrt(1 - a^2) i u), float32 each."""
        self._check("u", u, torch.float32, ndim=2)
        T, width = u.shape
        self._check("gate weight", w_a, self._FLOATS, ndim=3)
        blocks, bw = w_a.shape[0], w_a.shape[1]
        if blocks * bw != width or w_a.shape[2] != bw:
            raise ValueError(f"rglru_gates: weights {tuple(w_a.shape)} for {width} channels")
        self._check("gate weight", w_i, w_a.dtype, shape=w_a.shape)
        for name, v in (("gate bias", b_a), ("gate bias", b_i), ("decay rate", rate)):
            self._check(name, v, torch.float32, shape=(width,))
        a = torch.empty(T, width, dtype=torch.float32, device=self.device)
        x = torch.empty(T, width, dtype=torch.float32, device=self.device)
        self._call(self.lib.ts_rglru_gates, _ptr(u), _ptr(w_a), _ptr(w_i), _TYPE_CODE[w_a.dtype],
                   _ptr(b_a), _ptr(b_i), _ptr(rate), _ptr(a), _ptr(x), T, width, blocks,
                   self._stream())
        return a, x

    def rglru_scan(self, a, x, proj, y_col, y_bias, batch, state, out_dtype):
        """S_t = a_t S_(t-1) + x_t per channel over each entry's tokens in order, from the
        request's `state` [slots, width] (zero where a portion starts at position 0), which
        receives the last S -> S_t * gelu_tanh(y_t + y_bias) in `out_dtype`, y being `width`
        columns of `proj` (float32) from `y_col`."""
        self._check("a", a, torch.float32, ndim=2)
        T, width = a.shape
        self._check("x", x, torch.float32, shape=(T, width))
        self._check("proj", proj, torch.float32, ndim=2)
        if proj.shape[0] != T or y_col < 0 or y_col + width > proj.shape[1]:
            raise ValueError("rglru_scan: gate columns outside the projection")
        if y_bias is not None:
            self._check("y bias", y_bias, torch.float32, shape=(width,))
        self._check_state("recurrent state", state, (width,))
        pos, eot, qs, slots = self._batch_ptrs(batch, T)
        out = torch.empty(T, width, dtype=out_dtype, device=self.device)
        chunks, entry_chunks, num_chunks = self._scan_chunks(batch)
        scratch = decays = None
        if num_chunks:
            scratch = torch.empty(num_chunks, width, dtype=torch.float32, device=self.device)
            decays = torch.empty(num_chunks, width, dtype=torch.float32, device=self.device)
        self._call(self.lib.ts_rglru_scan, _ptr(a), _ptr(x), _ptr(proj), proj.shape[1],
                   int(y_col), _ptr(y_bias), _ptr(state), _ptr(out), _TYPE_CODE[out_dtype], pos,
                   eot, qs, slots, T, batch.num_entries, width, _ptr(chunks), _ptr(entry_chunks),
                   num_chunks, _ptr(scratch), _ptr(decays), self._stream())
        return out

    # ------------------------------------------------------------ activations of rows
    def relu_squared(self, x, out_dtype):
        """relu(x)^2, element by element."""
        x = self._rows(x)
        self._check("x", x, self._FLOATS, ndim=2)
        out = torch.empty(x.shape, dtype=out_dtype, device=self.device)
        self._call(self.lib.ts_relu_squared, _ptr(x), _TYPE_CODE[x.dtype], _ptr(out),
                   _TYPE_CODE[out_dtype], c_int64(x.numel()), self._stream())
        return out

    def sigmoid_gate(self, x, gate_rows, gate_col, out_dtype, group=1):
        """x [T, n] times the sigmoid of columns [gate_col, gate_col + n / group) of
        `gate_rows`: every `group` neighbouring columns of x share a gate."""
        x = self._rows(x)
        self._check("x", x, self._FLOATS, ndim=2)
        self._check("gate", gate_rows, self._FLOATS, ndim=2)
        T, n = x.shape
        if group < 1 or n % group or gate_rows.shape[0] != T or gate_col < 0 \
                or gate_col + n // group > gate_rows.shape[1]:
            raise ValueError("sigmoid_gate: gate columns outside their rows")
        out = torch.empty(T, n, dtype=out_dtype, device=self.device)
        self._call(self.lib.ts_sigmoid_gate, _ptr(x), _TYPE_CODE[x.dtype], _ptr(gate_rows),
                   _TYPE_CODE[gate_rows.dtype], gate_rows.shape[1], int(gate_col), _ptr(out),
                   _TYPE_CODE[out_dtype], T, n, int(group), self._stream())
        return out

    def add_weighted_rows(self, out, h, weights, col, count):
        """In place on float32 `out` [T, width]: out[t] += h[t] times the sum of columns
        [col, col + count) of `weights` [T, n]."""
        self._check("out", out, torch.float32, ndim=2)
        h = self._rows(h)
        self._check("h", h, self._FLOATS, shape=out.shape)
        self._check("weights", weights, torch.float32, ndim=2)
        if weights.shape[0] != out.shape[0] or col < 0 or col + count > weights.shape[1]:
            raise ValueError("add_weighted_rows: columns outside the weights")
        self._call(self.lib.ts_add_weighted_rows, _ptr(out), _ptr(h), _TYPE_CODE[h.dtype],
                   _ptr(weights), out.shape[0], out.shape[1], weights.shape[1], int(col),
                   int(count), self._stream())

    # ------------------------------------------------------------ sums around the stream
    def stream_add(self, resid, a, b, row):
        """In place on the float32 stream: resid += (a + b), then resid += row (float32
        [width], or [T, width]: a row for every token); each may be None (b only with a)."""
        self._check("resid", resid, torch.float32, ndim=2)
        codes = []
        for name, t in (("a", a), ("b", b)):
            if t is not None:
                t = self._rows(t)
                self._check(name, t, self._FLOATS, shape=resid.shape)
            codes.append(t)
        a, b = codes
        self._call(self.lib.ts_stream_add, _ptr(resid), _ptr(a),
                   _TYPE_CODE[a.dtype] if a is not None else 0, _ptr(b),
                   _TYPE_CODE[b.dtype] if b is not None else 0, _ptr(row),
                   self._row_stride(row, resid), resid.shape[0], resid.shape[1], self._stream())

    def _row_stride(self, row, resid):
        """0 for a row that every row of the stream gets, the width for rows of their own."""
        if row is None:
            return 0
        if row.dim() == 2:
            self._check("rows", row, torch.float32, shape=resid.shape)
            return resid.shape[1]
        self._check("row", row, torch.float32, shape=(resid.shape[1],))
        return 0

    def stream_add_norm(self, resid, a, b, row, norm_w, eps, out_dtype):
        """`stream_add(resid, a, b, row)` (b and row may be None), and the RMS norm (norm_w,
        eps) of the new stream in `out_dtype`."""
        self._check("resid", resid, torch.float32, ndim=2)
        a = self._rows(a)
        self._check("a", a, self._FLOATS, shape=resid.shape)
        if b is not None:
            b = self._rows(b)
            self._check("b", b, self._FLOATS, shape=resid.shape)
        stride = self._row_stride(row, resid)
        self._check("norm weight", norm_w, torch.float32, shape=(resid.shape[1],))
        out = torch.empty(resid.shape, dtype=out_dtype, device=self.device)
        self._call(self.lib.ts_stream_add_norm, _ptr(resid), _ptr(a), _TYPE_CODE[a.dtype], _ptr(b),
                   _TYPE_CODE[b.dtype] if b is not None else 0, _ptr(row), stride, _ptr(norm_w),
                   _ptr(out),
                   _TYPE_CODE[out_dtype], resid.shape[0], resid.shape[1], c_float(eps),
                   self._stream())
        return out

    def scaled_sum(self, a, scale_a, b, scale_b):
        """scale_a * a + scale_b * b -> float32."""
        a, b = self._rows(a), self._rows(b)
        self._check("a", a, self._FLOATS, ndim=2)
        self._check("b", b, self._FLOATS, shape=a.shape)
        out = torch.empty(a.shape, dtype=torch.float32, device=self.device)
        self._call(self.lib.ts_scaled_sum, _ptr(a), _TYPE_CODE[a.dtype], c_float(scale_a), _ptr(b),
                   _TYPE_CODE[b.dtype], c_float(scale_b), _ptr(out), a.shape[0], a.shape[1],
                   self._stream())
        return out

    def take_columns(self, x, col, count, out_dtype):
        """Columns [col, col + count) of float32 rows as rows of their own in `out_dtype`."""
        self._check("x", x, torch.float32, ndim=2)
        out = torch.empty(x.shape[0], count, dtype=out_dtype, device=self.device)
        self._call(self.lib.ts_take_columns, _ptr(x), x.shape[1], int(col), int(count), _ptr(out),
                   _TYPE_CODE[out_dtype], x.shape[0], self._stream())
        return out

    # ------------------------------------------------------------ latent attention
    def _check_latent(self, cache, table, batch, dl):
        self._check("latent pages", cache.k_pages, self._FLOATS,
                    shape=(cache.num_pages, cache.page_size, dl))
        self._check("block table", table, torch.int32, ndim=2)
        if table.shape[0] != batch.num_entries:
            raise ValueError("block table rows differ from the batch's entries")

    def latent_prepare(self, proj, batch, table, cache, *, q_rank, kv_rank, rot_dim, q_norm,
                       kv_norm, eps, freqs, rot_dims, out_dtype):
        """Rows [q latent | kv latent | shared key part] (float32): the normalised q latent
        comes back in `out_dtype`; the normalised kv latent and the rotated key part are
        written to the tokens' rows of the latent pages."""
        self._check("proj", proj, torch.float32, ndim=2)
        T = proj.shape[0]
        dl = kv_rank + rot_dim
        if proj.shape[1] != q_rank + dl:
            raise ValueError(f"latent_prepare: rows of {proj.shape[1]}, expected {q_rank + dl}")
        self._check("q norm", q_norm, torch.float32, shape=(q_rank,))
        self._check("kv norm", kv_norm, torch.float32, shape=(kv_rank,))
        self._check("frequencies", freqs, torch.float32, shape=(rot_dims // 2,))
        self._check_latent(cache, table, batch, dl)
        pos, eot, _, _ = self._batch_ptrs(batch, T)
        cq = torch.empty(T, q_rank, dtype=out_dtype, device=self.device)
        self._call(self.lib.ts_latent_prepare, _ptr(proj), _ptr(q_norm), _ptr(kv_norm),
                   _ptr(freqs), _ptr(cq), _TYPE_CODE[out_dtype], _ptr(cache.k_pages),
                   _TYPE_CODE[cache.k_pages.dtype], pos, eot, _ptr(table), table.shape[1],
                   cache.page_size, T, q_rank, kv_rank, rot_dim, rot_dims, c_float(eps),
                   self._stream())
        return cq

    def rotate_interleaved_inplace(self, x, positions, freqs, dims, offset=0):
        """x [T, heads, width]: the pairs (offset + 2i, offset + 2i + 1), i < dims / 2, of
        every head's vector turned by positions[t] * freqs[i], in place."""
        self._check("x", x, self._FLOATS, ndim=3)
        T, heads, width = x.shape
        self._check("positions", positions, torch.int32, shape=(T,))
        self._check("frequencies", freqs, torch.float32, shape=(dims // 2,))
        if dims % 2 or offset < 0 or offset + dims > width:
            raise ValueError(f"rotate_interleaved: {dims} dimensions from {offset} of {width}")
        self._call(self.lib.ts_rotate_interleaved, _ptr(x), _TYPE_CODE[x.dtype], _ptr(positions),
                   _ptr(freqs), T, heads, width, offset, dims, self._stream())

    def latent_attention(self, qa, batch, table, cache, *, heads, kv_rank, rot_dim, scale,
                         window, out_dtype=torch.float32):
        """Softmax attention of qa [T, heads, kv_rank+rot_dim] (float32) over the latent
        pages -> sum_t p_t c_t, [T, heads, kv_rank] in `out_dtype`."""
        dl = kv_rank + rot_dim
        self._check("qa", qa, torch.float32, ndim=3)
        T = qa.shape[0]
        if tuple(qa.shape[1:]) != (heads, dl):
            raise ValueError("latent_attention: query shape does not fit")
        self._check_latent(cache, table, batch, dl)
        pos, eot, _, _ = self._batch_ptrs(batch, T)
        out = torch.empty(T, heads, kv_rank, dtype=out_dtype, device=self.device)
        if cache.k_pages.dtype == torch.bfloat16 and self.latent_mfma and \
                self.lib.ts_latent_attention_mfma_fits(kv_rank, rot_dim) == 1:
            self._latent_attention_mfma(qa, out, batch, table, cache, heads, kv_rank, rot_dim,
                                        scale, window)
            return out
        self._call(self.lib.ts_latent_attention, _ptr(qa), _ptr(cache.k_pages),
                   _TYPE_CODE[cache.k_pages.dtype], _ptr(out), _TYPE_CODE[out_dtype], pos, eot,
                   _ptr(table),
                   table.shape[1], cache.page_size, T, heads, kv_rank, rot_dim,
                   int(window) if window else 0, c_float(scale), self._stream())
        return out

    #: False sends bfloat16 pages to the float32 multiply-add kernel as well
    latent_mfma = True

    def _latent_attention_mfma(self, qa, out, batch, table, cache, heads, kv_rank, rot_dim,
                               scale, window):
        """The matrix-core kernel: tiles of 16 (token, head) rows of one entry, made on the
        host once a step and head count; where they are few, each tile's keys are shared out
        over several wavefronts and merged."""
        d = self.dispatch
        counts = [-(-n * heads // 16) for n in batch.q_lens]
        # many tiles: four of one entry to a workgroup, which walk their keys together; few:
        # one tile a workgroup (and three empty ones), every tile's keys shared out
        waves = 1 if sum(counts) < d.latent_full_tiles else 4
        key = ("latent_tiles", heads, waves)
        if key not in batch.plans:
            tiles, row = [], 0
            for e, n in enumerate(batch.q_lens):
                rows = n * heads
                for i in range(0, rows, 16):
                    tiles.append((row + i, min(16, rows - i), e))
                    while waves == 1 and len(tiles) % 4:
                        tiles.append((row, 0, e))       # empty tiles fill the workgroup
                while len(tiles) % 4:
                    tiles.append((row, 0, e))
                row += rows
            batch.plans[key] = (self._upload_ints(tiles), len(tiles))
        tiles, num_tiles = batch.plans[key]
        # the longest run of keys a workgroup can have: the window and its own tokens, or
        # the longest context
        span = batch.max_ctx_len if not window else min(batch.max_ctx_len, window + 16 * waves)
        # shares start at an absolute multiple of 32 at or below the first visible key, so
        # up to 31 keys more than the span have to be covered
        splits, per = 1, 1 << 30
        if waves == 1:
            most = max(1, d.latent_full_tiles // (num_tiles // 4))
            per = -(-max(d.latent_split_keys, -(-(span + 31) // most)) // 32) * 32
            splits = -(-(span + 31) // per)
            if splits == 1:
                per = 1 << 30
        part_o = part_ml = None
        if splits > 1:
            part_o = torch.empty(num_tiles, splits, 16, kv_rank, dtype=torch.float32,
                                 device=self.device)
            part_ml = torch.empty(num_tiles, splits, 16, 2, dtype=torch.float32,
                                  device=self.device)
        self._call(self.lib.ts_latent_attention_mfma, _ptr(qa), _ptr(cache.k_pages), _ptr(out),
                   _TYPE_CODE[out.dtype], _ptr(tiles), num_tiles, 4, _ptr(batch.positions),
                   _ptr(table), table.shape[1], cache.page_size, heads, kv_rank, rot_dim,
                   int(window) if window else 0, c_float(scale), per, splits, _ptr(part_o),
                   _ptr(part_ml), self._stream())
