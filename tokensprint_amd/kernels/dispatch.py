"""The row counts and sizes at which the kernel provider changes from one kernel to
another, in one table, each entry with what it was measured on.

None of these decides what is computed, only by which kernel; every one was found by
timing captured steps on an MI355X at the shapes named below.  A model of other shapes
runs correctly with them and may be faster with others: `HipOps.dispatch` is an ordinary
attribute, `dataclasses.replace(ops.dispatch, decode_items=...)` gives a changed copy, and
`MEASURED` is where a table measured on other shapes is added.
"""

from __future__ import annotations

from dataclasses import dataclass


@dataclass(frozen=True)
class Dispatch:
    # ---- plain bfloat16 products: from how many rows the vendor library (hipBLASLt)
    # takes them, as the reference sends every linear layer to its vendor library
    # (engine/nn/base_layers.py:7-10).  Measured inside captured graphs at the Qwen3-0.6B
    # layer shapes (K = 1,024 to 3,072, N = 1,024 to 6,144).
    #: up to 64 rows the weight-streaming kernels here are faster at the layer products
    #: and fuse the norm before and the SwiGLU after
    library_rows: int = 65
    #: in the wide layout (a short K: four waves along N) the library is ahead from 17 rows
    library_rows_wide: int = 17
    #: at the output head (N from `head_columns`: every one of thousands of workgroups
    #: reads all rows of x) from 5 rows; measured at N = 151,936, K = 1,024
    library_rows_head: int = 5
    head_columns: int = 16384
    #: weights above `large_weight` elements (the layer shapes of the 8B and 32B models:
    #: products bound by bandwidth, not latency): every workgroup's reading of the rows of
    #: x costs as much as the weights from 16 rows on, and the library is ahead from there
    #: (a decode step of the 8B shape with 12 requests 4.13 ms here against 4.37 with the
    #: library, with 16 requests 4.47 against 4.43, with 32 5.59 against 4.92); whether it
    #: also takes the rows below is decided per weight shape by the warm-up
    library_rows_large: int = 16
    large_weight: int = 1 << 23

    # ---- gate/up product of many rows with the SiLU-multiply in its epilogue: stacked
    # weights up to this many elements take the LDS-tiled kernel.  Against the library's
    # product followed by the SiLU-multiply kernel: at the 0.6B shape (2 x 3,072 x 1,024)
    # 0.56 to 0.87 of their time from 128 to 8,192 rows, because the [M, 2 I] intermediate
    # is neither written nor read; at the 8B shape 0.85 to 1.07, at the 32B shape 1.02 to
    # 1.20, the library's product itself being 10 to 20 % ahead at large sizes.
    tiled_pair_weight: int = 1 << 23
    #: rows from which, and elements of a weight [N, K] up to which, the product that ends a
    #: sub-layer is the LDS-tiled kernel's tail form (it adds itself into the float32 stream
    #: and prepares the rows for the norm behind it, whose product then takes the scaled
    #: form) instead of the library's product and a norm kernel.  Plain products of such
    #: sizes (a model's first layer, whose norm nothing prepares) take the tiled kernel too:
    #: the same time on the GPU (22.5 against 22.4 us for qkv at 2,048 rows) and a fifth of
    #: the library call's 20 to 30 us on the host, which the GPU waits for at a step's start.
    tiled_stream_rows: int = 512
    tiled_stream_weight: int = 1 << 23

    # ---- attention.  Measured at 16 query / 8 key-value heads of 128, page size 16.
    #: workgroups (entries x key/value heads) up to which a decode step takes the decode
    #: kernel; with more, the chip is full anyway and the smaller workgroups of the
    #: general kernel do better
    decode_items: int = 512
    #: a step that holds a portion of at least `portion_tokens` tokens takes the kernel
    #: for long portions from this many 16-row wave tiles (one portion of 256 tokens 11.0
    #: against the general kernel's 16.6 us, 1,024 tokens 21.5 against 34.4, 1,536 tokens
    #: 34.0 against 96.8; below that the two are equal)
    portion_tiles: int = 256
    portion_tokens: int = 32
    #: a step of single tokens only takes it where the chip is full without splitting
    #: keys: from 1,024 wave tiles (128 entries at 8 key/value heads) it is ahead of the
    #: general kernel at every context length tried (136 entries: 34 against 41 us at 300
    #: tokens each, 130 against 150 at 100 to 2,000, 426 against 445 at 4,000; 200
    #: entries: 46 / 51, 180 / 223, 608 / 653), at 576 to 768 it is level or behind
    single_token_tiles: int = 1024
    #: the general kernel: up to this many tiles a workgroup per tile and chunk whose
    #: waves share the chunk (decode), above it a wavefront per tile walks its keys
    #: (prompts); and the workgroups each mode spreads a tile's key chunks over
    cooperative_items: int = 1024
    cooperative_workgroups: int = 512
    per_wave_workgroups: int = 4096


#: what each table was measured on -> the table
MEASURED: dict[str, Dispatch] = {
    "gfx950 (MI355X, 256 compute units); Qwen3 dense at the 0.6B, 8B and 32B layer shapes: "
    "16 to 64 query heads over 8 key/value heads of 128, page size 16": Dispatch(),
}


def default_dispatch() -> Dispatch:
    """The table for this build's one target."""
    return next(iter(MEASURED.values()))
