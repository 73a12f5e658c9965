"""The device side that parts share: which GPU, which precision, how a tensor
is placed, and the matrix product.

dtype "bfloat16": weights stay as stored (bfloat16; a tensor stored in 32-bit
stays 32-bit), activations between kernels are bfloat16, while the residual
stream, norms, softmax, rotation and every accumulation are float32.
dtype "float32": everything is widened to float32 and every product is a true
32-bit one (no matrix-core or reduced-precision mode).
"""
from __future__ import annotations

import os

import torch

from .csrc import ops

DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32}


def device_dtype(stored: torch.dtype, kind: str, compute: str) -> torch.dtype:
    """Type a tensor has on the device, from its type in the file: integer
    tables are int32; under float32 every real tensor is widened; under bfloat16
    a bfloat16 tensor stays bfloat16, a tensor stored in 32-bit stays 32-bit and
    float16 is widened (exactly) to float32."""
    if kind == "int":
        return torch.int32
    if compute == "float32":
        return torch.float32
    if stored == torch.bfloat16:
        return torch.bfloat16
    return torch.float32


class Weight:
    """A matrix [N, K] as the products want it: `rows` as stored, for the library
    product and the 32-bit kernels, and `tiles`, the same values in the layout
    that the few-rows kernels stream fastest (None where that layout does not
    apply).  `pairs`: the matrix is [gate; up] and its tiles hold 8 gate rows over
    the 8 matching up rows each (for the product that ends in SwiGLU)."""
    __slots__ = ("rows", "tiles", "pairs")

    def __init__(self, rows: torch.Tensor, tiles: torch.Tensor | None = None, pairs: bool = False):
        self.rows, self.tiles, self.pairs = rows, tiles, pairs

    @property
    def shape(self):
        return self.rows.shape

    @property
    def dtype(self):
        return self.rows.dtype


class ScaledRows:
    """Rows of an RMS norm that still lack their scale: `rows` = bfloat16(x * norm
    weight) and `sumsq` [M, >= parts], `parts` partial sums of x^2 a row whose total gives
    row t's scale rsqrt(sum(sumsq[t, :parts]) / width + eps).  A row's scale commutes with a product over
    the row, so `Runtime.linear` applies it to the product's rows; any other
    consumer asks `Runtime.rows_of` for the finished rows.  `steps_major`: `rows` holds its values as
    [width / 32][M][32] (what the few-rows products read fastest, `ops.steps_major`), not as [M][width]."""
    __slots__ = ("rows", "sumsq", "parts", "eps", "steps_major")

    def __init__(self, rows: torch.Tensor, sumsq: torch.Tensor, parts: int, eps: float, steps_major: bool = False):
        self.rows, self.sumsq, self.parts, self.eps, self.steps_major = rows, sumsq, parts, eps, steps_major

    @property
    def scale(self):
        """What the products' `row_scale` takes."""
        return (self.sumsq, self.parts, self.eps)

    @property
    def shape(self):
        return self.rows.shape

    @property
    def dtype(self):
        return self.rows.dtype


class Deferred:
    """A product `x . w^T` that `Runtime.linear(..., defer=True)` has not launched
    yet: the delta of a mixer or a feed-forward, which a norm that follows may
    launch together with the residual add (`Runtime.product_add_norm`); `run()`
    launches it as it is.  `x_steps_major`: x holds its values in the order of `ops.steps_major`."""
    __slots__ = ("rt", "x", "w", "slabs", "x_steps_major")

    def __init__(self, rt, x, w, slabs, x_steps_major=False):
        self.rt, self.x, self.w, self.slabs, self.x_steps_major = rt, x, w, slabs, x_steps_major

    def run(self) -> torch.Tensor:
        return self.rt.linear(self.x, self.w, slabs=self.slabs, x_steps_major=self.x_steps_major)


class Runtime:
    FUSE_NORM_X_BYTES = 40e6    # most bytes of X the workgroups of an unsplit product may read together for the fused norm to pay

    def __init__(self, dtype: str = "bfloat16", device: str = "cuda:0", stream_layout: bool = True):
        if dtype not in DTYPES:
            raise ValueError(f"dtype must be one of {sorted(DTYPES)}, got {dtype!r}")
        if not torch.cuda.is_available():
            raise RuntimeError("no GPU visible: kipp_amd runs on a gfx950 GPU only and has no CPU path")
        self.dtype = dtype
        self.device = torch.device(device)
        self.act_dtype = DTYPES[dtype]
        self.cache_dtype = DTYPES[dtype]
        self.ops = ops
        self.stream_layout = stream_layout   # keep a second copy of bfloat16 matrices in the streaming layout
        self._mm_out_f32 = None
        self.library_products = 0   # calls that went to the library (they stay out of HIP graphs)
        self.generic_attention_launches = 0   # bfloat16 attention that fell to the generic kernel (geometry the matrix-core kernels refuse)
        self.fuse_norms = True      # few rows: residual add and norm ride on the products around them
        # Where one kernel hands over to the next, measured at the 4B shape on an MI355X; another width or device may
        # move them, so they are the runtime's and can be set on it
        self.few_rows = int(os.environ.get("KIPP_AMD_FEW_ROWS", ops.SKINNY_BEST_ROWS))   # rows up to which every wave reads its rows of x itself (the kernel with the fused ends)
        self.staged_rows = ops.ROWS_BEST_ROWS       # rows up to which x is staged through LDS; beyond, the product built for hundreds of rows
        self.fused_decode_rows = 16                 # single tokens up to which decode attention starts from the QKV product ...
        self.fused_decode_keys = 8192               # ... while their contexts are shorter than this
        self.fuse_norm_x_bytes = float(os.environ.get("KIPP_AMD_FUSE_NORM_X_BYTES", self.FUSE_NORM_X_BYTES))
        # rows that one few-rows product writes for the next (a norm's rows, the activation) in the order that product
        # reads fastest, [width / 32][rows][32]: half the memory requests for x at 8 rows (3 % of a decode step at batch 8)
        self.steps_major_rows = os.environ.get("KIPP_AMD_STEPS_MAJOR", "1") != "0"
        # products of more than about 200 rows: True (the default): our own matrix-core kernel, in the fastest of the
        # cuts that give the planned cut's bits, so that every process computes the same bits; "auto": the fastest of
        # all our cuts and the library's product, timed once in a process at a shape's first use (another process
        # may choose otherwise, and its results then differ in their last bits); False: always the library's.
        # KIPP_AMD_PRODUCTS=own|auto|library sets it from outside.
        self.own_prompt_products = {"own": True, "auto": "auto", "library": False}.get(os.environ.get("KIPP_AMD_PRODUCTS", "own"), True)
        self.prompt_product_choices = {}     # shape -> "library", "plan" (our kernel, cut as planned) or a forced cut of ours
        self.tile_products = 0      # products of many rows that ran on our own kernel
        # decode attention: the splits of a head are merged by whichever of their workgroups finishes last (one launch
        # fewer a layer; ordered by device-scope stores, one device-scope counter a head and device-scope loads); False,
        # or KIPP_AMD_DECODE_MERGE=launch, merges them in a launch of its own, which needs no ordering between workgroups
        self.merge_in_kernel = os.environ.get("KIPP_AMD_DECODE_MERGE", "kernel") != "launch"
        self.for_a_graph = False    # set around a step of single tokens that is, or is to be, recorded as a HIP graph
        torch.backends.cuda.matmul.allow_tf32 = False

    # -- placement -----------------------------------------------------------
    def stored_dtype(self, stored: torch.dtype, kind: str) -> torch.dtype:
        return device_dtype(stored, kind, self.dtype)

    def place(self, t: torch.Tensor, kind: str = "float", force: torch.dtype | None = None) -> torch.Tensor:
        target = force or self.stored_dtype(t.dtype, kind)
        return t.to(device=self.device, dtype=target).contiguous()

    def empty(self, shape, dtype) -> torch.Tensor:
        return torch.empty(shape, dtype=dtype, device=self.device)

    def weight(self, w: torch.Tensor, gate_up: bool = False) -> Weight:
        """A matrix on the device, made ready for `linear`.  A bfloat16 matrix whose
        K is a multiple of 32 gets a copy in the streaming layout: decode reads every
        weight once a step and is bound by that read, which is a fifth faster from
        that layout; many-row products go to the library, which needs the rows.
        The price is the matrix held twice.  `gate_up`: w is [gate; up] and feeds
        SwiGLU; its tiles pair gate rows with their up rows."""
        tiles = None
        if self.stream_layout and w.dtype == torch.bfloat16 and w.dim() == 2 and w.shape[1] % 32 == 0:
            tiles = self.ops.tile_weight_pairs(w) if gate_up else self.ops.tile_weight(w)
        return Weight(w, tiles, gate_up and tiles is not None)

    # -- matrix product ------------------------------------------------------
    def _few_rows(self, m: int, k: int, w) -> bool:
        """The product goes to the few-rows kernel (the one with the fused ends, which take up to 16 rows)."""
        return w.dtype == torch.bfloat16 and self.ops.gemm_rows_ok(m, k) and m <= min(self.few_rows, 16)

    def settle(self, delta):
        """The tensor of a delta, launched now if it was deferred."""
        return delta.run() if isinstance(delta, Deferred) else delta

    def rows_of(self, h):
        """The tensor of norm output, scaled now if the scale was left to a product."""
        if not isinstance(h, ScaledRows):
            return h
        return self.ops.scale_rows(h.rows, h.sumsq, h.parts, h.eps, self.empty(h.rows.shape, torch.bfloat16), steps_major=h.steps_major)

    def product_add_norm(self, delta: Deferred, x: torch.Tensor, norm_weight: torch.Tensor, eps: float):
        """x += delta's product, in the product's own kernel, which also prepares the
        RMS norm of the new x: returns ScaledRows (None if this product has no such
        kernel: the caller then runs it and norms as usual)."""
        w = delta.w
        rows, k = delta.x.shape
        if not (self.fuse_norms and isinstance(w, Weight) and not w.pairs and delta.x.dtype == torch.bfloat16
                and self._few_rows(rows, k, w) and x.dtype == torch.float32 and x.is_contiguous()
                and norm_weight.dtype == torch.float32):
            return None
        # That kernel is not split over workgroups.  Where the product alone would be, each of its N / 16
        # workgroups reads all of delta.x instead of a part of it, which costs more than the norm's kernel
        # once that is some tens of megabytes (measured: 5120 x 8192 and 5120 x 25600 at 8 rows, +5.6 us
        # each against 4.6 saved; at 4 rows and for narrower weights the fused form wins).
        most = 1 if delta.slabs is False else (8 if delta.slabs is True else int(delta.slabs))
        n_out = w.shape[0]
        if self.ops.gemm_skinny_parts(n_out, k, most) > 1 and ((n_out + 15) // 16) * rows * k * 2 > self.fuse_norm_x_bytes:
            return None
        major = self.steps_major_rows and n_out % 32 == 0 and rows > 1       # one row is one run either way
        rows_out, sumsq = self.ops.gemm_skinny(delta.x, w.rows, tiles=w.tiles, add_norm=(x, norm_weight),
                                               x_steps_major=delta.x_steps_major, out_steps_major=major)
        return ScaledRows(rows_out, sumsq, (w.shape[0] + 15) // 16, eps, steps_major=major)

    # -- products of prompt portions ------------------------------------------------------------
    def streams(self, m: int, k: int, n: int) -> bool:
        """Whether a bfloat16 product of m rows takes the kernels that stream the weight once (few rows, or a
        shape the product for many rows does not take)."""
        return self.ops.gemm_rows_ok(m, k) and (m <= self.staged_rows or not self.ops.gemm_tiles_ok(m, k, n))

    @staticmethod
    def _rows_class(m: int) -> int:
        """Rows of a prompt product, in classes of a factor of two (193-256, 257-512, 513-1024, ...): one decision a class."""
        return 1 << (max(m, 1) - 1).bit_length()

    # Cuts of our kernel that are timed beside the planned one: 100 x (wave tile rows / 32) + 10 x (wave tile
    # columns / 32) + parts of K (+ 1000: workgroups of 8 waves, two a SIMD, on the same 256 x 256 tile; + 2000: those for
    # the whole rounds of 256 tiles and smaller tiles for the columns that are left, + 30000: the smallest for those).  The
    # plan's cost model is linear; the GPU under its power limit is not (a round that leaves compute units idle
    # clocks the others higher), so the plan is not always the fastest.  An output element is summed over K in
    # the same order whatever the tile, so cuts with the same parts of K give the same bits.
    _choices_of_process: dict = {}
    TILE_CUTS_SLABS = (441, 442, 444, 431, 432, 421, 422, 1421, 1422, 1424)
    TILE_CUTS_BF16 = (441, 421, 241, 1421, 2421, 32421)

    def _fastest(self, key, ways: dict, same_bits, extra_ms=None):
        """Which of several ways to compute one product is taken for the shape `key`: decided once, by timing
        them on the operands at hand (three runs each after a first one).  `ways`: name -> callable, "library"
        and "plan" among them; `same_bits`: the names whose results are those of "plan" bit for bit;
        `extra_ms`: name -> milliseconds that a way costs its consumer beyond its own kernel (the slabs of a split
        product are read by the kernel that adds them).
        `own_prompt_products` True: only those are timed, so the choice changes how long a
        product takes and never what it gives; "auto" (the default): all of them (the library's product and other parts of K
        round differently: two runs of one program may then differ in their last bits); False: the library's."""
        if self.for_a_graph:
            # a step that is to be recorded keeps to our own kernels (the library's calls stay out of HIP graphs)
            key = key + ("for a graph",)
            ways = {name: run for name, run in ways.items() if name != "library"}
        choice = self.prompt_product_choices.get(key)
        if choice is None:
            choice = self._choices_of_process.get((self.own_prompt_products, key))      # every engine of a process decides alike
        if choice is not None:
            self.prompt_product_choices[key] = choice
        if choice is None:
            if self.own_prompt_products is False:
                choice = "library" if "library" in ways else "plan"
            else:
                # The chip is at its power limit while products follow each other, and a product that wins from
                # a standing start need not win then: every candidate runs a few times first, then they are
                # timed in turn, twice round, without a pause between them
                runs = {}
                for name, run in ways.items():
                    if self.own_prompt_products != "auto" and name not in same_bits:
                        continue
                    try:
                        for _ in range(3):
                            run()
                    except self.ops.KernelError:
                        continue                      # a cut this shape does not take
                    runs[name] = run
                marks = []
                for _ in range(2):
                    for name, run in runs.items():
                        begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                        begin.record()
                        for _ in range(4):
                            run()
                        end.record()
                        marks.append((name, begin, end))
                torch.cuda.current_stream().synchronize()
                took = {}
                for name, begin, end in marks:
                    took[name] = took.get(name, 0.0) + begin.elapsed_time(end) / 4
                for name in took:
                    took[name] += 2 * (extra_ms or {}).get(name, 0.0)
                choice = min(took, key=took.get) if took else "plan"
            self.prompt_product_choices[key] = choice
            self._choices_of_process[(self.own_prompt_products, key)] = choice
        return choice

    def _library_product(self, x, w):
        """bfloat16 x bfloat16 with float32 accumulation and a float32 result by the library (hipBLASLt through torch.mm)."""
        if self._mm_out_f32 is None:
            try:
                torch.mm(x[:1], w[:1].t(), out_dtype=torch.float32)
                self._mm_out_f32 = True
            except (RuntimeError, TypeError):
                self._mm_out_f32 = False
        if self._mm_out_f32:
            return torch.mm(x, w.t(), out_dtype=torch.float32)
        # a torch without float32 results from bfloat16 products would round deltas of the residual stream
        raise RuntimeError("this torch cannot return float32 from a bfloat16 product; the library product is not used then")

    def gated(self, x, w: "Weight", act: torch.Tensor) -> torch.Tensor:
        """act [M, I] (bfloat16) = silu(x . gate^T) * (x . up^T) for many rows, w = [gate; up]: our kernel
        computes both products and the activation in one pass; after the library's product (float32, so
        that either way rounds once, after the activation) the activation is a kernel of its own."""
        m, k = x.shape
        rows = w.rows

        def ours(force=0):
            return self.ops.gemm_tiles(x, rows, end="swiglu", force=force)

        def library():
            return self.ops.swiglu(self._library_product(x, rows), act)
        if self.ops.gemm_tiles_ok(m, k, rows.shape[0]):
            ways = {"library": library, "plan": ours}
            ways.update({cut: (lambda cut=cut: ours(cut)) for cut in self.TILE_CUTS_BF16})
            choice = self._fastest(("gated", self._rows_class(m), rows.shape[0], k), ways, ("plan",) + self.TILE_CUTS_BF16)
            if choice != "library":
                self.tile_products += 1
                return ours(0 if choice == "plan" else choice)
        self.library_products += 1
        return library()

    def linear(self, x, w, slabs: bool = False, defer: bool = False, x_steps_major: bool = False):
        """float32 [M, N] = x [M, K] . w [N, K]^T.  With `slabs` the result may come
        as [parts, M, N] whose sum over parts is the product (few rows against a
        weight with few output rows: the contraction is split over workgroups and
        the consumer adds the slabs in order); an integer is the most slabs the
        consumer takes.  `x` may be ScaledRows.  With
        `defer` the product may come back as a `Deferred` (for a delta of the
        residual stream, which the next norm launches or `settle` does).  `x_steps_major`: a plain x
        holds its values in the order of `ops.steps_major` (few rows only)."""
        if defer and self.fuse_norms and not isinstance(x, ScaledRows) and self._few_rows(x.shape[0], x.shape[1], w):
            return Deferred(self, x, w, slabs, x_steps_major)
        row_scale = None
        if isinstance(x, ScaledRows):
            if self._few_rows(x.shape[0], x.shape[1], w):
                row_scale, x_steps_major, x = x.scale, x.steps_major, x.rows
            else:
                x = self.rows_of(x)
        if x_steps_major and not (isinstance(w, Weight) and self._few_rows(x.shape[0], x.shape[1], w) and self.streams(x.shape[0], x.shape[1], w.shape[0])):
            x, x_steps_major = self.ops.from_steps_major(x), False       # only the few-rows kernel reads that order
        tiles = None
        if isinstance(w, Weight):
            # paired tiles give the columns in another order: only the feed-forward asks for that
            w, tiles = w.rows, (None if w.pairs else w.tiles)
        m = x.shape[0]
        n = w.shape[0]
        if w.dtype == torch.float32:
            if x.dtype != torch.float32:
                x = self.ops.cast(x, self.empty(x.shape, torch.float32))
            return self.ops.gemm_f32(x, w, self.empty((m, n), torch.float32))
        if x.dtype != torch.bfloat16:
            x = self.ops.cast(x, self.empty(x.shape, torch.bfloat16))
        if self.streams(m, x.shape[1], n):
            # up to about 200 rows: our own kernels stream the weight once
            most = 0 if slabs is False else (None if slabs is True else int(slabs))
            if m <= self.few_rows:
                y = self.ops.gemm_skinny(x, w, max_parts=1 if most == 0 else (most or 8), tiles=tiles, row_scale=row_scale,
                                         x_steps_major=x_steps_major)
            else:
                y = self.ops.gemm_rows(x, w, max_parts=1 if most == 0 else (most or 12), tiles=tiles)
            return y if y.shape[0] > 1 else y[0]
        # more rows (prompt portions): our matrix-core kernel, or the library's product
        if self.ops.gemm_tiles_ok(m, x.shape[1], n):
            most = 1 if slabs is False else (4 if slabs is True else max(1, min(4, int(slabs))))

            def ours(force=0):
                y = self.ops.gemm_tiles(x, w, end="slabs", max_parts=most, force=force)
                return y if y.shape[0] > 1 else y[0]

            def library():
                return self._library_product(x, w)
            ways = {"library": library, "plan": ours}
            ways.update({cut: (lambda cut=cut: ours(cut)) for cut in self.TILE_CUTS_SLABS if cut % 10 <= most})
            planned = self.ops.gemm_tiles_parts(m, n, x.shape[1], "slabs", most)
            same = ("plan",) + tuple(cut for cut in self.TILE_CUTS_SLABS if cut % 10 == planned)
            # every slab beyond the first is read once more by the kernel that adds them (at about 5 TB/s)
            slab_ms = m * n * 4 / 5e12 * 1e3
            extra = {name: ((planned if name == "plan" else name % 10) - 1) * slab_ms for name in ways if name != "library"}
            choice = self._fastest(("linear", self._rows_class(m), n, x.shape[1], most), ways, same, extra)
            if choice != "library":
                self.tile_products += 1
                return ours(0 if choice == "plan" else choice)
        self.library_products += 1
        return self._library_product(x, w)
