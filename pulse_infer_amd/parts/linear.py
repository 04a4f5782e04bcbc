"""y = x W^T for a weight stored [out, in] (reference: src/layer/linear.cpp:213).

Three products stand behind it:

* few rows (decoding, short portions) of bfloat16: this package's weight-streaming
  matrix-core kernel, which can also add into the float32 residual or apply SwiGLU;
* many rows of bfloat16: the vendor library's product (torch.matmul / torch.mm,
  i.e. hipBLASLt/rocBLAS, float32 accumulation, bfloat16 or float32 output), as
  the reference uses cuBLAS (src/ops/kernels/cuda/matmul_kernel.cu:132-154), or this
  package's product in output tiles of 256 x 256, which can apply SwiGLU on the way
  out or leave float32 results of shares of the inner dimension (``OWN_MANY_ROWS``
  says which products go there);
* the float32 run, and any weight kept in 32-bit: this package's own
  fused-multiply-add kernel, with no reduced-precision mode anywhere.
"""
from __future__ import annotations

import os
from typing import Optional

import torch

from ..ops import kernels, timing
from ..ops.device import compute_units
from .base import LazyNorm, RowStats, Workspace


# Which products of many rows (256 and more) run as this package's tiled product instead of the library's: "none";
# "swiglu": gate and up with SwiGLU inside, which saves the pass over twice the feed-forward's width; "all": every
# product of bfloat16 (a step then makes no library call).  PULSE_OWN_PRODUCTS sets it.  Measured through the
# serving loop: a prompt of 2,048 tokens of the 8B shape 73.9K tokens/s with "none", 72.9K with "swiglu", 71.6K with
# "all" (alone and with the chip warm, gate+up with SwiGLU inside takes 310 us against the library's 328 + 30 for
# the pass; between the other kernels of a step the library's product takes 278); serving of the 8B shape 4,334 /
# 4,313 / 4,248 tokens/s, of the 14B shape 2,695 / 2,688 (means of two runs each, "none" and "swiglu"), of the 32B shape
# 1,258 / 1,264.  So the library stays the default.
OWN_MANY_ROWS = os.environ.get("PULSE_OWN_PRODUCTS", "none")
if OWN_MANY_ROWS not in ("none", "swiglu", "all"):
    raise ValueError(f"PULSE_OWN_PRODUCTS must be none, swiglu or all, not '{OWN_MANY_ROWS}'")

library_calls = 0   # products that went to the vendor library so far (a step that made none can be recorded as a graph)


class Linear:
    def __init__(self, weight: torch.Tensor, mode: str):
        if weight.dim() != 2:
            raise ValueError(f"a linear weight must be a matrix, got shape {tuple(weight.shape)}")
        self.weight = weight
        self.out_features, self.in_features = weight.shape
        self.mode = mode
        self.library = mode == "bfloat16" and weight.dtype == torch.bfloat16

    def takes_lazy(self, x: LazyNorm, rows: Optional[int] = None) -> bool:
        """Whether the product can take rows that have not been normalised yet and scale its result instead."""
        n = self.out_features if rows is None else rows
        return (self.library and kernels.gemm_skinny_fusable(x.shape[0], n, self.in_features)
                and x.x.dtype == torch.bfloat16 and kernels.gemm_skinny_ok(x.x, self.weight))

    def forward(self, x, out: torch.Tensor, rows: Optional[int] = None, swiglu: bool = False,
                own: bool = True) -> torch.Tensor:
        """``out`` [M, out_features] receives the product; its storage type is bfloat16 or float32.  ``x`` may be a
        ``LazyNorm`` that ``takes_lazy`` accepted.  ``swiglu``: few rows of a slab-interleaved gate/up weight only.
        ``own=False``: 17 to 64 rows go to the library although this package has a product for them (a caller that
        measured the library faster for its shape)."""
        w = self.weight if rows is None else self.weight[:rows]
        if isinstance(x, LazyNorm):
            kernels.gemm_skinny(x.x, w, out, swiglu=swiglu, row_scale=(x.sumsq, x.eps))
            return out
        if swiglu:
            if x.shape[0] > self.MID_ROWS[1]:
                kernels.gemm_tile(x, w, out, swiglu=True)
            elif x.shape[0] > kernels.SKINNY_FAST_ROWS:
                kernels.gemm_mid(x, w, out, swiglu=True, waves=self.swiglu_waves_for(x.shape[0]) or 4)
            else:
                kernels.gemm_skinny(x, w, out, swiglu=True)
            return out
        if self.library and x.dtype == torch.bfloat16:
            few = x.shape[0] <= kernels.SKINNY_FAST_ROWS
            if few and kernels.gemm_skinny_ok(x, w):
                kernels.gemm_skinny(x, w, out)
                return out
            if own and self.takes_own_rows(x, w, out):
                # 17 to 64 rows: X through LDS, 16 weight rows a wavefront.  A float32 result (logits) is the "parts"
                # output with one share; many weight rows take wide workgroups, few take narrow ones so that there
                # are enough of them (measured: logits of a 152K vocabulary 212 to 237 us against the library's 276 to
                # 281; 6,144 rows of qkv 17 to 21 us against 15 to 18, which a step without a library call, recorded
                # and replayed as a whole, makes up several times over).
                if self.takes_shared_k(x, w, out):
                    # few weight rows (qkv): a workgroup owns two 16-row slabs and all of K, which its wavefronts
                    # share out among themselves (6,144 weight rows of 4,096: 14.1 / 15.0 / 18.7 us at 24 / 32 / 64
                    # rows against 17.2 / 17.1 / 22.2 with a wavefront a slab; the library 14.7 / 15.1 / 17.8)
                    kernels.gemm_rows(x, w, out, slabs=2)
                    return out
                waves = 10 if w.shape[0] >= 64 * compute_units() else 2
                kernels.gemm_mid(x, w, out.view(1, *out.shape) if out.dtype == torch.float32 else out, waves=waves)
                return out
            if own and out.dtype == torch.bfloat16 and self.takes_tiles(x, w) and out.stride(1) == 1 \
                    and out.stride(0) % 8 == 0 and out.data_ptr() % 16 == 0:
                kernels.gemm_tile(x, w, out)
                return out
            global library_calls
            library_calls += 1
            if out.dtype == torch.bfloat16:
                with timing.region("library matmul"):
                    torch.matmul(x, w.t(), out=out)
                return out
            if out.dtype == torch.float32 and out.is_contiguous():
                # float32 results of many rows (logits): the library's product with a float32 output
                with timing.region("library matmul (float32 out)"):
                    torch.mm(x, w.t(), out_dtype=torch.float32, out=out)
                return out
            if w.shape[1] % 8 == 0:  # otherwise the few-rows kernel, 64 rows at a time
                for r0 in range(0, x.shape[0], kernels.SKINNY_MAX_ROWS):
                    kernels.gemm_skinny(x[r0:r0 + kernels.SKINNY_MAX_ROWS], w, out[r0:r0 + kernels.SKINNY_MAX_ROWS])
                return out
        kernels.gemm_f32(x, w, out)
        return out

    def add_into(self, x: torch.Tensor, residual: torch.Tensor, scratch: torch.Tensor,
                 workspace: Optional[Workspace] = None, next_scale: Optional[torch.Tensor] = None):
        """residual += x W^T, in one of five ways.  Few rows: the kernel adds into the residual itself and None is
        returned, or, given a workspace and a shape the fused kernel takes, the ``RowStats`` of the updated rows (their
        sums of squares and a rounded copy, multiplied column by column by ``next_scale``, the weight of the norm that
        reads the residual next: with these the next product can do without a norm kernel before it).  17 to
        192 rows, given a workspace: the product's inner dimension is shared out over workgroups and the shares' float32
        results [parts, rows, out] are returned as the update, which the next norm adds up in order; more rows of a
        product with a wide inner dimension and a narrow output: the same through the library's batched product.
        Otherwise the product is written to ``scratch`` and returned for the caller to add."""
        splits, waves = self.shares_and_waves_for(x) if workspace is not None else (0, 0)
        if splits:
            rows = x.shape[0]
            parts = workspace.buffer(f"linear.parts.{self.out_features}.{self.in_features}", splits * rows,
                                     self.out_features, torch.float32).view(splits, rows, self.out_features)
            kernels.gemm_mid(x, self.weight, parts, splits=splits, waves=waves)
            return parts
        splits = self.tile_shares_for(x) if workspace is not None else 0
        if splits:
            rows = x.shape[0]
            parts = workspace.buffer(f"linear.parts.{self.out_features}.{self.in_features}", splits * rows,
                                     self.out_features, torch.float32).view(splits, rows, self.out_features)
            kernels.gemm_tile(x, self.weight, parts)
            return parts
        splits = self.library_shares_for(x) if workspace is not None else 0
        if splits:
            # Many rows but few output tiles (down: a wide inner dimension, a narrow output): the library's product
            # leaves most compute units idle (14B shape, 544 rows: 179 us), so it runs as a batch over shares of the
            # inner dimension (102 us) whose float32 results the next norm adds up in order.
            rows, share = x.shape[0], self.in_features // splits
            parts = workspace.buffer(f"linear.parts.{self.out_features}.{self.in_features}", splits * rows,
                                     self.out_features, torch.float32).view(splits, rows, self.out_features)
            xa = x.view(rows, splits, share).transpose(0, 1)
            wb = self.weight.view(self.out_features, splits, share).permute(1, 2, 0)
            global library_calls
            library_calls += 1
            with timing.region("library batched matmul"):
                torch.bmm(xa, wb, out_dtype=torch.float32, out=parts)
            return parts
        if (self.library and x.dtype == torch.bfloat16 and x.shape[0] <= kernels.SKINNY_FAST_ROWS
                and kernels.gemm_skinny_ok(x, self.weight)):
            if (workspace is not None
                    and kernels.gemm_skinny_fusable(x.shape[0], self.out_features, self.in_features)):
                sums = workspace.buffer(f"linear.sumsq.{self.out_features}", x.shape[0], (self.out_features + 15) // 16,
                                        torch.float32)
                rounded = workspace.buffer(f"linear.rounded.{self.out_features}", x.shape[0], self.out_features,
                                           torch.bfloat16)
                scaled = next_scale is not None and next_scale.dtype == torch.bfloat16 \
                    and next_scale.numel() == self.out_features and next_scale.is_contiguous()
                kernels.gemm_skinny(x, self.weight, residual, add=True, sumsq_out=sums, copy_out=rounded,
                                    copy_scale=next_scale if scaled else None)
                return RowStats(sums, rounded, next_scale if scaled else None)
            kernels.gemm_skinny(x, self.weight, residual, add=True)
            return None
        return self.forward(x, scratch)

    MID_ROWS = (17, 64)          # where the product with X shared through LDS and SwiGLU inside beats the library's
                                 # product followed by the SwiGLU kernel
    SHARES_ROWS = (17, 192)      # where a product that adds into the residual has its inner dimension shared out over
                                 # workgroups (measured on the 8B shape: 1% of a decoding step at 17 to 32 rows, 4% at
                                 # 48, 6% at 64; at 96 to 192 rows the library takes 22 to 33 us for o and 55 to 90 us
                                 # for down, the shared-out product 16 to 22 and 33 to 47.  Up to 16 rows the few-rows
                                 # kernel stands: it leaves what the next product needs to do without a norm kernel,
                                 # and a step of 13 rows is 3% faster with it, one of 16 rows as fast)

    LIBRARY_SHARES_MIN_K = 8192  # inner dimensions from here on are worth sharing out in the library's product
    LIBRARY_TILE = 256           # its output tiles are about this large in both directions

    def library_shares_for(self, x: torch.Tensor) -> int:
        """Into how many shares the library's product of more than 192 rows is cut; 0: not at all.  Measured (8B,
        14B and 32B shapes of down, 272 to 2,048 rows): 4 shares win up to about 50 output tiles, 2 shares up to
        about 140 (8B shape at 2,048 rows: 182 -> 157 us, which the wider update costs again in the norm that adds
        it up, so the rule stops at 100 tiles), none beyond; products with an inner dimension of 4,096 to 8,192 (o)
        gain 5 us at most."""
        rows = x.shape[0]
        if not (self.library and x.dtype == torch.bfloat16 and rows > self.SHARES_ROWS[1]
                and self.in_features >= self.LIBRARY_SHARES_MIN_K and x.is_contiguous()
                and self.weight.is_contiguous() and self.out_features % 4 == 0):
            return 0
        tile = self.LIBRARY_TILE
        tiles = ((rows + tile - 1) // tile) * ((self.out_features + tile - 1) // tile)
        splits = 4 if tiles <= 50 else (2 if tiles <= 100 else 0)
        while splits > 1 and (self.in_features % splits or (self.in_features // splits) % 64):
            splits //= 2
        return splits if splits > 1 else 0

    def operands_ok(self, x: torch.Tensor) -> bool:
        """Contiguous, aligned bfloat16 rows of a length the kernels' 16-byte loads take."""
        w = self.weight
        return (x.dim() == 2 and x.shape[1] % 8 == 0 and x.stride(1) == 1 and w.stride(1) == 1
                and (x.shape[0] <= 1 or x.stride(0) % 8 == 0) and (w.shape[0] <= 1 or w.stride(0) % 8 == 0)
                and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)

    def takes_own_rows(self, x: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> bool:
        """Whether a plain product of this many rows (bfloat16 or float32 result) runs as this package's product for
        17 to 64 rows instead of the library's."""
        rows = x.shape[0]
        if not (self.MID_ROWS[0] <= rows <= self.MID_ROWS[1] and self.operands_ok(x) and w.stride(1) == 1
                and kernels.gemm_mid_takes(rows, w.shape[0], w.shape[1])):
            return False
        if out.dtype == torch.float32:
            return out.is_contiguous() and out.data_ptr() % 16 == 0 and w.shape[0] % 4 == 0
        return out.dtype == torch.bfloat16 and out.stride(1) == 1 and out.stride(0) % 4 == 0 and out.data_ptr() % 16 == 0

    TILE_MIN_ROWS = 256          # from here on the tiled product for many rows is a candidate

    def takes_tiles(self, x: torch.Tensor, w: Optional[torch.Tensor] = None, swiglu: bool = False) -> bool:
        """Whether a product of this many rows runs as this package's tiled product (``OWN_MANY_ROWS`` allowing)."""
        w = self.weight if w is None else w
        if OWN_MANY_ROWS == "none" or (OWN_MANY_ROWS == "swiglu" and not swiglu):
            return False
        return (self.library and x.dtype == torch.bfloat16 and x.shape[0] >= self.TILE_MIN_ROWS and self.operands_ok(x)
                and kernels.gemm_tile_takes(x.shape[0], w.shape[0], w.shape[1], swiglu=swiglu))

    def tile_shares_for(self, x: torch.Tensor) -> int:
        """Into how many shares of the inner dimension the tiled product of many rows is cut when it adds into the
        residual (float32 results that the next norm adds up); 0: not this product.  As many shares as bring the
        tiles to the number of compute units, at most 8."""
        if OWN_MANY_ROWS != "all" or not self.takes_tiles(x) or self.out_features % 4:
            return 0
        tile = kernels.TILE_ROWS
        tiles = ((x.shape[0] + tile - 1) // tile) * ((self.out_features + tile - 1) // tile)
        splits = max(1, min(8, compute_units() // tiles))
        while splits > 1 and self.in_features % (splits * kernels.TILE_K):
            splits -= 1
        return splits

    def takes_shared_k(self, x: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> bool:
        """Whether a bfloat16 product of 17 to 64 rows runs with the inner dimension shared out inside a workgroup:
        weights of so few rows that a wavefront a slab leaves most of the chip's wavefront slots empty."""
        return (out.dtype == torch.bfloat16 and w.shape[0] <= 32 * compute_units()
                and kernels.gemm_rows_takes(x.shape[0], w.shape[0], w.shape[1]))

    def takes_mid(self, x: torch.Tensor) -> bool:
        return (self.library and x.dtype == torch.bfloat16 and self.MID_ROWS[0] <= x.shape[0] <= self.MID_ROWS[1]
                and self.operands_ok(x) and self.swiglu_waves_for(x.shape[0]) > 0)

    def swiglu_waves_for(self, rows: int) -> int:
        """Wavefronts a workgroup of the product for 17 to 64 rows with SwiGLU inside (no sharing out of the inner
        dimension there), or 0 where the library's product followed by the SwiGLU kernel is faster.

        The estimate is again the fullest compute unit's: workgroups on it x (weight rows a workgroup + half the
        rows of X, which every workgroup fetches).  Measured at 32 rows: 8B shape (24,576 weight rows) 96 rows a
        workgroup 37.9 us (one workgroup a unit), 64 rows 43.6; 14B shape (34,816) 160 rows 68.8 us, 96 rows 80.5
        (363 workgroups: two on some units); 32B shape (51,200) 64 rows 117 us, the best of all shapes, against
        the library's 100 + 5: no shape shares 200 rows a unit out evenly, so the library takes that one (the rule:
        this product's estimate must stay below 1.5 x the weight rows a unit)."""
        n = self.out_features
        units = compute_units()
        if n <= 32 * units:
            return 2    # too few weight rows to fill the chip in any shape: the most workgroups
        best = None
        for waves in (2, 4, 6, 10):
            on_a_unit = ((n + 16 * waves - 1) // (16 * waves) + units - 1) // units
            cost = on_a_unit * (16 * waves + rows // 2)
            if best is None or cost < best[0]:
                best = (cost, waves)
        if n <= 64 * units:
            return best[1]    # (12,288 weight rows: 64 rows a workgroup 12 to 15 us, the library 15 to 18 + 5)
        return best[1] if best[0] * units < 1.5 * n else 0

    def shares_for(self, x: torch.Tensor) -> int:
        """Into how many shares the inner dimension is cut for an update in parts; 0: not this product."""
        return self.shares_and_waves_for(x)[0]

    def shares_and_waves_for(self, x: torch.Tensor):
        """(shares of the inner dimension, wavefronts a workgroup) of the product for 17 to 192 rows whose float32
        partial results the next norm adds up; (0, 0): not this product.

        The pair with the least estimated time of the fullest compute unit is taken: workgroups on it (all of them
        over the compute units, rounded up) x weight rows a workgroup x (length of a share + 280, what a workgroup costs
        beside its walk), plus half a microsecond a share for the norm that adds them up.  Measured at 64 rows: down
        of the 8B shape 4 shares of 64 rows (256 workgroups) 23.8 us, 8 shares 24.9, 6 shares (384 workgroups, two on
        half the units) 28.6; down of the 14B shape 4 shares of 96 rows (216 workgroups) 40.9 us, 8 shares of 64 rows
        (640 workgroups) 46.9."""
        if not (self.library and x.dtype == torch.bfloat16 and self.SHARES_ROWS[0] <= x.shape[0] <= self.SHARES_ROWS[1]
                and self.operands_ok(x)) or self.out_features % 4:
            return 0, 0
        best = None
        units = compute_units()
        for waves in (4, 6):
            rows = 16 * waves
            tiles = (self.out_features + rows - 1) // rows
            for splits in range(1, 17):
                if self.in_features % splits or (self.in_features // splits) % 128:
                    continue
                share = self.in_features // splits
                on_a_unit = (tiles * splits + units - 1) // units
                cost = on_a_unit * rows * (share + 280) + 8000 * splits
                if best is None or cost < best[0]:
                    best = (cost, splits, waves)
        return (best[1], best[2]) if best else (0, 0)

