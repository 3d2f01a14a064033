"""The HIP kernels as Python operations: argument checks on the host, then one C call.

Every method checks shapes, dtypes, devices and contiguity before a pointer reaches a
kernel, because a kernel handed a wrong shape would read or write out of bounds.  There
is no other implementation behind these methods: without a GPU or without the built
library, construction raises.
"""

from __future__ import annotations

import ctypes
from ctypes import Structure, byref, c_float, c_int, c_void_p

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
        ("store_kv", c_int), ("eps", c_float),
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
        ("window", c_int), ("scale", c_float),
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
    def embed(self, table, token_ids):
        self._check("embedding table", table, self._FLOATS, ndim=2)
        self._check("token ids", token_ids, torch.int32, ndim=1)
        T, (V, H) = token_ids.shape[0], table.shape
        out = torch.empty(T, H, dtype=torch.float32, device=self.device)
        self._call(self.lib.ts_embed, _ptr(table), _TYPE_CODE[table.dtype], V, _ptr(token_ids),
                   _ptr(out), T, H, self._stream())
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
                 cos_sin):
        T = qkv.shape[0]
        self._check("qkv", qkv, self._FLOATS, shape=(T, (num_heads + 2 * kv_in_row) * head_dim))
        if head_dim % 2:
            raise ValueError(f"head_dim={head_dim} must be even")
        a = QkPrepareArgs()
        a.qkv = qkv.data_ptr()
        a.num_tokens, a.nq, a.nkv, a.hd = T, num_heads, kv_in_row, head_dim
        a.eps = eps
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
                           head_dim, q_weight, k_weight, eps, cos_sin):
        a = self._qk_args(qkv, batch, num_heads=num_heads, kv_in_row=num_kv_heads,
                          head_dim=head_dim, q_weight=q_weight, k_weight=k_weight, eps=eps,
                          cos_sin=cos_sin)
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
                        scale, window):
        T = q.shape[0]
        self._check("q", q, self._FLOATS, shape=(T, num_heads, head_dim))
        self._check_cache(cache, table, batch, num_kv_heads, head_dim)
        if T != batch.num_tokens:
            raise ValueError("q rows differ from the batch's tokens")
        out = torch.empty_like(q)
        a = AttentionArgs()
        self._fill_attention_args(a, q, out, batch, table, cache, num_heads, num_kv_heads,
                                  head_dim, scale, window)
        if (q.dtype == torch.bfloat16 and cache.k_pages.dtype == torch.bfloat16
                and head_dim % 16 == 0 and head_dim <= 256 and cache.page_size % 4 == 0):
            if self._decode_fits(batch, num_kv_heads, num_heads // num_kv_heads, head_dim,
                                 cache.page_size, False):
                self._attention_decode(a, batch, num_heads // num_kv_heads)
            else:
                self._attention_mfma(a, batch, num_heads // num_kv_heads)
        else:
            self._call(self.lib.ts_attention_generic, byref(a), _TYPE_CODE[q.dtype],
                       _TYPE_CODE[cache.k_pages.dtype], self._stream())
        return out

    def attend(self, qkv, batch, table, cache, write_cache, *, num_heads, num_kv_heads,
               kv_in_row, head_dim, q_weight, k_weight, eps, cos_sin, scale, window,
               defer_merge=False):
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
                k_weight=k_weight, eps=eps, cos_sin=cos_sin)
            return self.paged_attention(q, batch, table, cache, num_heads=num_heads,
                                        num_kv_heads=num_kv_heads, head_dim=head_dim,
                                        scale=scale, window=window)
        # the same argument checks as the preparation kernel's
        qa = self._qk_args(qkv, batch, num_heads=num_heads, kv_in_row=kv_in_row,
                           head_dim=head_dim, q_weight=q_weight, k_weight=k_weight, eps=eps,
                           cos_sin=cos_sin)
        self._check_cache(cache, table, batch, num_kv_heads, head_dim)
        if T != batch.num_tokens or T != batch.num_entries:
            raise ValueError("a decode step brings one token per entry")
        out = torch.empty(T, num_heads, head_dim, dtype=qkv.dtype, device=self.device)
        a = AttentionArgs()
        self._fill_attention_args(a, None, out, batch, table, cache, num_heads, num_kv_heads,
                                  head_dim, scale, window)
        d = AttentionDecodeArgs()
        d.qkv, d.q_weight, d.k_weight = qa.qkv, qa.q_weight, qa.k_weight
        d.cos, d.sin, d.eps, d.kv_in_row = qa.cos, qa.sin, eps, kv_in_row
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
        span = batch.max_ctx_len if a.window == 0 else min(batch.max_ctx_len,
                                                           a.window + self._attn_chunk)
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

    def _attention_mfma(self, a, batch, group):
        """Tile the batch's queries (16 rows of q heads x tokens per wavefront), choose how
        many waves share a tile's keys, and launch."""
        rows_per_token = min(group, 16)
        head_blocks = -(-group // 16)
        tokens_per_tile = 16 // rows_per_token
        m = AttentionMfmaArgs()
        m.base = a
        m.rows_per_token, m.head_blocks = rows_per_token, head_blocks
        # long portions of prompts: a wavefront takes several query tiles and walks alone
        if self._prefill_tiles(batch, a.nkv, group) is not None:
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
        span = batch.max_ctx_len if a.window == 0 else min(batch.max_ctx_len,
                                                           a.window + batch.max_q_len + chunk)
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
                             head_dim, scale, window):
        T = out.shape[0]
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
