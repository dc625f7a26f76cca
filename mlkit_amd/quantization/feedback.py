"""Hessian error feedback in LDL form: GPTQ (one column at a time) and LDLQ (blocks).

With the damped Hessian factored as ``H = R R^T`` (``R`` upper triangular), column block
``k`` is rounded after adding ``sum_{j<k} d_j R_jk R_kk^-1`` to its weights, ``d = w - q``.
``feedback_coefficients`` returns ``A = R blockdiag(R)^-1`` once; the sweep then needs no
inverse.  Mirrors /root/reference/src/mlkit/quantization/algorithms/error_feedback.py
(:37-83 feedback_coefficients, :107-233 CodecAccumulator, :236-467 ErrorFeedback,
:473-489 ldlq / gptq) and operations/losses.py:9-15 (proxy_loss).

On a HIP device, scalar grids with ``step == 1`` run entirely in kernels: per region one
triangular solve (``mk_feedback_pending``), one scale fit, then per tile the column sweep
(``mk_feedback_round_tile``) and the trailing update on the matrix cores
(``mk_feedback_block_update``).  Vector grids (codebooks of 2-, 4-, 8- or 16-dimensional
codewords, the E8P lattice) with ``step`` equal to their dimension run the same way with
``mk_feedback_round_vector_tile``.  Other rounders take the block-by-block tensor path.
"""

import math
from collections.abc import Callable
from typing import Any

import torch
from torch import Tensor

from mlkit_amd.quantization.codecs import decode_feedback, decode_vector_scaled
from mlkit_amd.quantization.core import (Ctx, FittedRounder, Q, Quantizer, ScalarRounding, VectorRounding, as_q,
                                         fit_quantizer)

FUSED_CODEBOOK_LIMIT = 256
FUSED_VECTOR_DIMENSIONS = {2, 4, 8, 16}
FUSED_VECTOR_CODEBOOK_LIMIT = 65536
UPPER_FACTORIZATION_WIDTH = 4096
MAXIMUM_FUSED_TILE = 1024
MAXIMUM_FUSED_VECTOR_TILE = 256
DEFERRED_TILES = 4  # tiles whose far-column updates are applied in one pass on the device


BLOCKED_FACTORIZATION_WIDTH = 1024  # narrower matrices go to the library factorisation
FACTORIZATION_BLOCK = 128           # one workgroup factors a diagonal block of this size
FACTORIZATION_PANEL = 1024          # rank of the trailing updates of the whole matrix
TRAILING_BAND = 1024                # rows per product of a trailing update (only the upper triangle is needed)
LOOK_AHEAD_WIDTH = 8192             # from here on the far part of a trailing update runs on a second stream


def _factor_in_place(matrix: Tensor, status: Tensor, factored: Tensor) -> None:
    """``matrix = U^T U`` for a symmetric positive definite FP32 matrix on a HIP device, factored
    in place (``status``: an int32 device scalar holding zero; ``factored``: scratch for the
    diagonal blocks, ``[ceil(width / 128), 128, 128]``).

    Two levels of blocking.  Panels of 1024 columns update the rest of the matrix, right-looking (a
    rank-1024 product reads and writes the trailing matrix an eighth as often as rank-128 ones
    would).  Inside a panel 128-column blocks are factored left-looking: a block's rows first take
    the updates of all earlier blocks of the panel in one product, then ``mk_cholesky_block``
    factors the diagonal block and carries the rest of its rows, to the last column, through the
    same elimination, which makes them the factor's block row; no triangular solve is left.  (The
    chain block kernel -> product -> block kernel is what bounds the run time; right-looking blocks
    with the far rows of each update on a stream of their own made it 7 % longer: every block then
    waited for two products.)  The factored diagonal blocks themselves are needed by nobody before
    the end (updates read block rows only): they wait in ``factored`` and go into the matrix in one
    copy.

    Look-ahead between panels: only the band of rows the next panel consists of is updated on the
    current stream; the rest runs on a second stream while the next panel is factored.  Events fix
    the order in which updates reach every entry, so results do not depend on timing (and are the
    same with all work on one stream).

    ``status`` stays zero, or becomes one plus the first column whose pivot is not positive (as
    ``torch.linalg.cholesky_ex`` reports it).  Nothing here allocates device memory or reads
    anything back, so the whole sequence can be captured in a HIP graph."""
    from mlkit_amd import native

    width = matrix.shape[0]
    device = matrix.device
    library = native.library()
    main = torch.cuda.current_stream(device)
    look_ahead = width >= LOOK_AHEAD_WIDTH   # narrower: the event traffic costs more than it hides
    side = torch.cuda.Stream(device) if look_ahead else None    # far rows of a panel's update

    def subtract_outer_product(start: int, stop: int, first_row: int, last_row: int, limit: int, after_first_band=None):
        """A[r, c] -= sum_k U[k, r] U[k, c] for k in start:stop, rows first_row:last_row, columns from
        the row band's first column to ``limit``: bands of rows, so that little below the diagonal
        is computed (what is, is never read).  ``after_first_band`` (a stream): returns an event
        recorded on it behind the first band."""
        event = None
        for band_start in range(first_row, last_row, TRAILING_BAND):
            band_stop = min(last_row, band_start + TRAILING_BAND)
            matrix[band_start:band_stop, band_start:limit].addmm_(
                matrix[start:stop, band_start:band_stop].T, matrix[start:stop, band_start:limit], alpha=-1.0)
            if after_first_band is not None and event is None:
                event = after_first_band.record_event()
        return event

    side_done = band_done = None
    for panel_start in range(0, width, FACTORIZATION_PANEL):
        panel_stop = min(width, panel_start + FACTORIZATION_PANEL)
        raw_stream = native.current_stream(device)
        for start in range(panel_start, panel_stop, FACTORIZATION_BLOCK):
            stop = min(panel_stop, start + FACTORIZATION_BLOCK)
            if start > panel_start:
                # the block's rows take the updates of every earlier block of the panel at once: one
                # product of rank start - panel_start, over all columns to the right (what a triangular
                # solve with the panel's whole diagonal block would otherwise do for them)
                matrix[start:stop, start:width].addmm_(matrix[panel_start:start, start:stop].T,
                                                       matrix[panel_start:start, start:width], alpha=-1.0)
            # the block kernel also carries the rest of rows start:stop, to the matrix's last column,
            # through the elimination (their block row of the factor); the factored block goes to
            # `factored`, since every workgroup of that launch reads the block itself
            beside = width - stop
            slot = factored[start // FACTORIZATION_BLOCK]
            native.check(library.mk_cholesky_block(matrix[start, start:].data_ptr(), width, stop - start, start, beside,
                                                   slot.data_ptr() if beside else None, status.data_ptr(), raw_stream))
        # the diagonal block's lower triangle holds leftovers of the products above
        matrix[panel_start:panel_stop, panel_start:panel_stop].triu_()
        if panel_stop == width:
            break
        if not look_ahead:
            subtract_outer_product(panel_start, panel_stop, panel_stop, width, width)
            continue
        row_ready = main.record_event()
        # the rows of the next panel: here, after the second stream's earlier update of them (its
        # first band: the stream works through the bands from the top, and through the panels in
        # order, so that band being done means every earlier update of these rows is)
        next_panel_stop = min(width, panel_stop + FACTORIZATION_PANEL)
        if band_done is not None:
            main.wait_event(band_done)
        subtract_outer_product(panel_start, panel_stop, panel_stop, next_panel_stop, width)
        if next_panel_stop < width:
            side.wait_event(row_ready)
            with torch.cuda.stream(side):
                band_done = subtract_outer_product(panel_start, panel_stop, next_panel_stop, width, width, after_first_band=side)
                side_done = side.record_event()
    if side_done is not None:
        main.wait_event(side_done)
    # the factored diagonal blocks (all but a last block that has no columns beside it, factored in place)
    whole = (width - 1) // FACTORIZATION_BLOCK
    if whole:
        diagonal = matrix.as_strided((whole, FACTORIZATION_BLOCK, FACTORIZATION_BLOCK),
                                     (FACTORIZATION_BLOCK * (width + 1), width, 1))
        diagonal.copy_(factored[:whole])


def _factor_scratch(width: int, device: torch.device) -> Tensor:
    return torch.empty((-(-width // FACTORIZATION_BLOCK), FACTORIZATION_BLOCK, FACTORIZATION_BLOCK), dtype=torch.float32,
                       device=device)


class _FactorGraph:
    """The launches of ``_factor_in_place`` for one width, captured once: several hundred small
    launches cost more to issue from Python than to run, and they are the same for every matrix
    of that width.  The graph owns the buffer it factors in."""

    def __init__(self, width: int, device: torch.device) -> None:
        self.matrix = torch.empty((width, width), dtype=torch.float32, device=device)
        self.status = torch.zeros((), dtype=torch.int32, device=device)
        self.factored = _factor_scratch(width, device)
        current = torch.cuda.current_stream(device)
        torch.cuda.synchronize(device)
        stream = torch.cuda.Stream(device)
        stream.wait_stream(current)
        with torch.cuda.stream(stream):
            try:
                self.graph = self._captured()
            except RuntimeError as error:
                # The random generator's capture state belongs to the mode in which the process made its first
                # capture.  If that was inference mode (a compiled model's first call under it), beginning a
                # capture writes that state in place, which only inference mode may do: capture there.  The
                # refused capture had not begun; its graph object is dropped.
                if "nference tensor" not in str(error):
                    raise
                with torch.inference_mode():
                    self.graph = self._captured()
        current.wait_stream(stream)

    def _captured(self) -> "torch.cuda.CUDAGraph":
        graph = torch.cuda.CUDAGraph()
        graph.capture_begin()
        try:
            self.status.zero_()   # a fill kernel
            _factor_in_place(self.matrix, self.status, self.factored)
        finally:
            graph.capture_end()
        return graph

    def __call__(self, fill: Callable[[Tensor], None]) -> tuple[Tensor, Tensor]:
        fill(self.matrix)
        self.graph.replay()
        return self.matrix, self.status


FACTOR_GRAPHS = True        # capture the factorisation of a width the second time it is asked for
FACTOR_GRAPH_LIMIT = 2      # graphs (and their width x width buffers) kept per process
_factor_graphs: dict[tuple[int, int], "_FactorGraph | None"] = {}


def clear_factor_graphs() -> None:
    """Drop the captured factorisations and their buffers (up to FACTOR_GRAPH_LIMIT graphs, each holding a
    width x width fp32 matrix plus scratch: about 0.5 GB at 11008 columns).  ``mk.quantize`` calls this at
    the end of a pass; callers that drive ``mk.gptq`` layer by layer themselves call it when they are done."""
    _factor_graphs.clear()


def _blocked_upper_factor(fill: Callable[[Tensor], None], width: int, device: torch.device) -> tuple[Tensor, Tensor]:
    """``(U, status)`` with ``U^T U`` = the matrix that ``fill(target)`` writes into a
    ``[width, width]`` FP32 tensor.  The first matrix of a width is factored launch by launch
    (which also warms every kernel up); from the second on the captured graph of that width
    runs.  The result may live in the graph's own buffer: it is valid until the next call."""
    key = (torch.cuda.current_device() if device.index is None else device.index, width)
    if FACTOR_GRAPHS and key in _factor_graphs and not torch.cuda.is_current_stream_capturing():
        graph = _factor_graphs[key]
        if graph is None:
            while sum(entry is not None for entry in _factor_graphs.values()) >= FACTOR_GRAPH_LIMIT:
                oldest = next(k for k, entry in _factor_graphs.items() if entry is not None)
                del _factor_graphs[oldest]
            graph = _factor_graphs[key] = _FactorGraph(width, device)
        return graph(fill)
    _factor_graphs.setdefault(key, None)   # seen once
    matrix = torch.empty((width, width), dtype=torch.float32, device=device)
    fill(matrix)
    status = torch.zeros((), dtype=torch.int32, device=device)
    _factor_in_place(matrix, status, _factor_scratch(width, device))
    return matrix, status




def feedback_coefficients(hessian: Tensor, step: int, *, damp: float = 0.01,
                          permutation: Tensor | None = None) -> tuple[Tensor, int]:
    """``(A, status)``: ``A = R blockdiag(R)^-1`` for the damped ``H = R R^T``, row-major;
    only entries above the block diagonal are meaningful.  ``status != 0``: H is indefinite.

    Zero diagonal entries (channels never activated) become one before damping by
    ``damp * mean(diag)``.  The lower Cholesky factor of the index-reversed matrix,
    reversed back, is the upper factor ``R``.
    """
    width = hessian.shape[0]
    if width >= BLOCKED_FACTORIZATION_WIDTH and hessian.is_cuda and hessian.dtype == torch.float32:
        return _coefficients_on_kernels(hessian, step, damp, permutation)
    if permutation is None:
        flipped = hessian.flip(0, 1)
    else:
        order = permutation.flip(0)
        flipped = hessian[order][:, order]
    diagonal = flipped.diagonal()
    diagonal.masked_fill_(diagonal == 0, 1)
    diagonal.add_(damp * diagonal.mean().clamp_min(1e-12))
    if width >= UPPER_FACTORIZATION_WIDTH:
        # column-major solvers factor the upper triangle faster; its transpose is the lower factor
        factor, status = torch.linalg.cholesky_ex(flipped, upper=True)
        lower = factor.T
    else:
        lower, status = torch.linalg.cholesky_ex(flipped)
    return _coefficients_of(lower, status, step)


def _coefficients_on_kernels(hessian: Tensor, step: int, damp: float, permutation: Tensor | None) -> tuple[Tensor, int]:
    """The same on a HIP device for matrices of 1024 columns and more: one pass writes the
    reversed, damped matrix where it is factored (``mk_hessian_reversed``), the blocked
    factorisation runs, and for ``step == 1`` one pass turns the factor into the coefficients
    (``mk_unit_upper_from_factor``)."""
    from mlkit_amd import native

    width, device = hessian.shape[0], hessian.device
    source = hessian.contiguous()
    order = None if permutation is None else permutation.flip(0).to(torch.int64).contiguous()
    ones_for_zeros = source.diagonal().clone()
    ones_for_zeros.masked_fill_(ones_for_zeros == 0, 1)
    addend = (damp * ones_for_zeros.mean().clamp_min(1e-12)).reshape(1).float()
    library = native.library()

    def fill(target: Tensor) -> None:
        native.check(library.mk_hessian_reversed(source.data_ptr(), target.data_ptr(), width, native.pointer(order),
                                                 addend.data_ptr(), native.current_stream(device)))

    factor, status = _blocked_upper_factor(fill, width, device)
    if step == 1 and int(status.item()) == 0:
        coefficients = torch.empty_like(factor)
        native.check(library.mk_unit_upper_from_factor(factor.data_ptr(), coefficients.data_ptr(), width,
                                                       native.current_stream(device)))
        return coefficients, 0
    return _coefficients_of(factor.T, status, step)


def _coefficients_of(lower: Tensor, status: Tensor, step: int) -> tuple[Tensor, int]:
    """``R blockdiag(R)^-1`` from the lower factor of the index-reversed matrix."""
    width = lower.shape[0]
    if int(status.item()) != 0:
        return lower.clone(), int(status.item())
    if step == 1:
        lower = lower / lower.diagonal().clone()
        return lower.flip(0, 1).contiguous(), 0
    upper = lower.flip(0, 1).contiguous()
    blocks = width // step
    pick = torch.arange(blocks, device=upper.device)
    diagonal_blocks = upper.reshape(blocks, step, blocks, step)[pick, :, pick, :]
    block_columns = upper.reshape(width, blocks, step).transpose(0, 1)
    solved = torch.linalg.solve_triangular(diagonal_blocks, block_columns, upper=True, left=False)
    return solved.transpose(0, 1).reshape(width, width).contiguous(), 0


def proxy_loss(weight: Tensor, reconstruction: Tensor, hessian: Tensor) -> Tensor:
    """``tr(E H E^T) / rows`` with ``E = W - W_hat``: the layer-output error the sweep minimises."""
    error = (weight - reconstruction).float()
    return ((error @ hessian.float()) * error).sum() / weight.shape[0]


class _PermutedStatistics:
    """Calibration statistics in the column order of permuted weights."""

    def __init__(self, ctx: Ctx, permutation: Tensor) -> None:
        self.ctx, self.permutation, self.seen = ctx, permutation, {}

    def __call__(self, name: str, function: Callable | None, reduction: str) -> Tensor:
        if name not in self.seen:
            value = self.ctx.stat(name, function, reduction)
            if name == "H":
                value = value[self.permutation][:, self.permutation]
            elif name == "X":
                value = value[:, self.permutation]
            elif name in {"act_absmean", "act_absmax"}:
                value = value[self.permutation]
            self.seen[name] = value
        return self.seen[name]


class _Collected:
    """Codes and fitted parameters of all regions, so the result stays a portable codec."""

    def __init__(self, rows: int, width: int, device: torch.device) -> None:
        self.rows, self.width, self.device = rows, width, device
        self.codes: Tensor | None = None
        self.shared: dict[str, Any] = {}
        self.metadata: dict[str, Any] = {}
        self.scales: list[Tensor] = []
        self.zeros: list[Tensor] = []
        self.portable = True
        self.bits: float | None = 0.0

    def count(self, bits: float | None) -> None:
        self.bits = None if self.bits is None or bits is None else self.bits + bits

    def open_scalar_region(self, scalar: ScalarRounding) -> Tensor:
        if self.codes is None:
            self.codes = torch.empty((self.rows, self.width), dtype=torch.uint8, device=self.device)
            self.shared = {"values": scalar.values, "group": scalar.group}
            self.metadata = scalar.metadata
        self.scales.append(scalar.scales)
        if scalar.zero is not None:
            self.zeros.append(scalar.zero)
        self.count(scalar.bits)
        return self.codes

    def open_vector_region(self, vector: VectorRounding) -> Tensor:
        dimension = vector.grid.dim
        if self.codes is None:
            self.codes = torch.empty((self.rows, self.width // dimension), dtype=torch.int32, device=self.device)
            self.shared = {"values": None if vector.lattice else vector.codebook, "group": vector.group,
                           "dim": dimension}
            self.metadata = vector.metadata
        self.scales.append(vector.scales)
        self.count(vector.bits)
        return self.codes

    def add_block(self, quantized: Q, column: int, stop: int, region_start: int) -> None:
        self.count(quantized.bits)
        if not self.portable:
            return
        if quantized.codec not in {"scaled", "vector_scaled"} or quantized.codes is None:
            self.portable = False
            return
        dimension = quantized.params.get("dim", 1)
        if self.codes is None:
            self.codes = torch.empty((self.rows, self.width // dimension), dtype=quantized.codes.dtype,
                                     device=self.device)
            self.shared = quantized.params
            self.metadata = quantized.metadata
        self.codes[:, column // dimension:stop // dimension] = quantized.codes
        if column == region_start:
            self.scales.append(quantized.params["scales"])
            if quantized.params["zero"] is not None:
                self.zeros.append(quantized.params["zero"])

    def result(self, output: Tensor, permutation: Tensor | None, refit_width: int, ctx: Ctx) -> Q:
        if self.portable and self.codes is not None:
            if permutation is not None:
                ctx.add_bits(self.width * math.ceil(math.log2(self.width)))
            params = {"scales": torch.cat(self.scales, dim=1), "values": self.shared["values"],
                      "group": self.shared["group"], "refit": refit_width,
                      "zero": torch.cat(self.zeros, dim=1) if self.zeros else None, "permutation": permutation}
            dimension = self.shared.get("dim")
            if dimension is not None:
                params["dim"] = dimension
                return Q(codes=self.codes, bits=self.bits, codec="vector_feedback", decode=decode_vector_scaled,
                         params=params, metadata=self.metadata)
            return Q(codes=self.codes, bits=self.bits, codec="feedback", decode=decode_feedback, params=params,
                     metadata=self.metadata)
        if permutation is not None:
            output = output[:, permutation.argsort()]
        return Q(output, bits=self.bits)


class ErrorFeedback(Quantizer):
    """LDL error feedback around an inner quantizer, with per-region refits of its format."""

    def __init__(self, inner: Callable[..., "Q | Tensor"], *, step: int = 8, refit: int | None = None,
                 damp: float = 0.01, order: str = "natural", block_size: int = 128, backend: str = "auto") -> None:
        if step < 1 or block_size < step or block_size % step:
            raise ValueError("block_size must be a positive multiple of step")
        if refit is not None and (refit < step or refit % step):
            raise ValueError("refit must be a positive multiple of step or None")
        if damp < 0 or order not in {"natural", "activation"}:
            raise ValueError("damp must be nonnegative and order must be natural or activation")
        if backend not in {"auto", "torch", "hip", "triton"}:
            raise ValueError("error-feedback backend must be auto, torch, or hip")
        self.inner, self.step, self.refit, self.damp = inner, step, refit, damp
        self.order, self.block_size = order, block_size
        self.backend = "hip" if backend == "triton" else backend

    @property
    def row_separable(self) -> bool:  # type: ignore[override]
        return bool(getattr(self.inner, "row_separable", False))

    def __repr__(self) -> str:
        return f"ldlq({self.inner!r}, step={self.step}, refit={self.refit})"

    # -- pieces --------------------------------------------------------------------------

    def _kernel_state(self, rounder: Callable[[Tensor, slice], Q],
                      device: torch.device) -> ScalarRounding | VectorRounding | None:
        """The fitted state when the HIP kernels can round this region: scalar grids go column
        by column, vector grids in blocks, which needs a step equal to the grid's dimension."""
        fitted = rounder if isinstance(rounder, FittedRounder) and device.type == "cuda" and self.backend != "torch" else None
        scalar = None if fitted is None else fitted.scalar
        if (scalar is not None and self.step == 1 and scalar.grid.bits <= 8
                and 1 <= scalar.values.numel() <= FUSED_CODEBOOK_LIMIT and self.block_size <= MAXIMUM_FUSED_TILE):
            return scalar
        vector = None if fitted is None else fitted.vector
        if (vector is not None and self.step == vector.grid.dim and vector.grid.dim in FUSED_VECTOR_DIMENSIONS
                and vector.codebook_size <= FUSED_VECTOR_CODEBOOK_LIMIT and vector.scales.dtype == torch.float32
                and self.block_size <= MAXIMUM_FUSED_VECTOR_TILE):
            return vector
        if self.backend == "hip":
            raise ValueError("fused error feedback requires a HIP device and a native scalar rounder with step=1, "
                             "or a native vector rounder with step equal to its dimension")
        return None

    def _whole_sweep(self, original: Tensor, feedback: Tensor, output: Tensor, coefficients: Tensor,
                     collected: "_Collected") -> bool:
        """Run every region in one call into the library when the inner format is a scaled
        scalar grid with range-fitted scales (no search, no user scale rule)."""
        from mlkit_amd.quantization.scaled import SCALE_FORMAT_BITS, Scaled

        inner = self.inner
        rows, width = original.shape
        refit = width if self.refit is None else self.refit
        usable = (type(inner) is Scaled and self.step == 1 and self.backend != "torch" and inner.scale == "absmax"
                  and isinstance(inner.scale_fmt, str) and inner.scale_fmt in SCALE_FORMAT_BITS
                  and inner.grid.values is not None and inner.grid.bits <= 8
                  and inner.grid.values.numel() <= FUSED_CODEBOOK_LIMIT and self.block_size <= MAXIMUM_FUSED_TILE
                  and (refit >= width or refit <= MAXIMUM_FUSED_TILE))
        if not usable:
            return False
        from mlkit_amd.kernels import error_feedback as kernel

        group = width if inner.group is None else inner.group
        values = inner.values_on(original.device)
        encoded = torch.empty((rows, width), dtype=torch.uint8, device=original.device)
        scales, zeros = kernel.sweep(
            original, feedback, output, encoded, coefficients, values=values, group=group, refit=refit,
            block=self.block_size, integer_grid=inner.grid.integer, code_minimum=inner._value_minimum,
            code_maximum=inner._value_maximum, asym=inner.asym,
            reciprocal=inner._range_reciprocal if inner.asym else inner._magnitude_reciprocal,
            value_minimum=inner._value_minimum, scale_format=inner.scale_fmt, deferred_tiles=DEFERRED_TILES)
        if not bool(torch.isfinite(scales).all()):
            raise ValueError("scaled requires a finite floating-point weight matrix")
        collected.codes = encoded
        collected.shared = {"values": values, "group": min(group, min(refit, width))}
        collected.metadata = {"code_bits": inner.grid.bits, "scale_fmt": inner.scale_fmt,
                              "trainable": ["scales"] + (["zero"] if inner.asym else [])}
        collected.scales = [scales]
        collected.zeros = [] if zeros is None else [zeros]
        side_bits = scales.numel() * SCALE_FORMAT_BITS[inner.scale_fmt] * (2 if inner.asym else 1)
        collected.count(inner.grid.bits * rows * width + side_bits)
        return True

    @staticmethod
    def _pending_continuation(feedback: Tensor, coefficients: Tensor, start: int, stop: int) -> Tensor:
        """The adjustment the region's columns would take if nothing more were rounded:
        accumulated feedback is that adjustment times the region's unit-triangular block."""
        if feedback.is_cuda and stop - start <= MAXIMUM_FUSED_TILE:
            from mlkit_amd.kernels import error_feedback as kernel

            return kernel.pending_continuation(feedback, coefficients, start, stop)
        return torch.linalg.solve_triangular(coefficients[start:stop, start:stop], feedback[:, start:stop],
                                             upper=True, left=False, unitriangular=True)

    def _round_tile_by_blocks(self, rounder, original, feedback, coefficients, output, collected,
                              region_start: int, tile_start: int, tile_stop: int) -> None:
        corrections = feedback[:, tile_start:tile_stop].clone()
        for column in range(tile_start, tile_stop, self.step):
            stop = column + self.step
            local = slice(column - tile_start, stop - tile_start)
            weights = original[:, column:stop]
            quantized = as_q(rounder(weights + corrections[:, local], slice(column - region_start, stop - region_start)))
            restored = quantized.w
            if restored.shape != weights.shape:
                raise ValueError("inner quantizer changed the shape of a column slice")
            output[:, column:stop] = restored
            collected.add_block(quantized, column, stop, region_start)
            if stop < tile_stop:
                deviation = weights - restored
                later = coefficients[column:stop, stop:tile_stop]
                if self.step == 1:
                    corrections[:, local.stop:] += deviation * later
                else:
                    corrections[:, local.stop:] += deviation @ later

    # -- the sweep -----------------------------------------------------------------------

    def __call__(self, w: Tensor, ctx: Ctx | None = None) -> Q:
        ctx = ctx or Ctx(device=w.device)
        rows, width = w.shape
        hessian = ctx.H.to(device=w.device, dtype=torch.float32).detach()
        if hessian.shape != (width, width):
            raise ValueError("Hessian dimensions must match the weight input width")
        if width % self.step:
            raise ValueError("weight input width must be divisible by the error-feedback step")
        dead = hessian.diagonal() == 0
        original = w.detach().to(torch.float32, copy=True)
        original[:, dead] = 0
        permutation = None
        if self.order == "activation":
            permutation = hessian.diagonal().masked_fill(dead, 1).argsort(descending=True)
            original = original[:, permutation].contiguous()
        coefficients, status = feedback_coefficients(hessian.clone(), self.step, damp=self.damp, permutation=permutation)
        if status != 0:
            raise ValueError(f"calibration Hessian for {ctx.name!r} is not positive definite; increase damp")
        del hessian
        statistics = None if permutation is None else _PermutedStatistics(ctx, permutation)
        feedback = torch.zeros_like(original)
        output = torch.empty_like(original)
        collected = _Collected(rows, width, w.device)
        refit_width = width if self.refit is None else self.refit
        on_device = w.is_cuda
        if on_device:
            from mlkit_amd.kernels import error_feedback as kernel
        # On the device the update of far columns is deferred: after a tile, only columns up to
        # `limit` are updated at once; the tiles in `deferred` reach the columns beyond it in
        # one pass when the super-block ends (or when a region needs those columns).  Every
        # column still receives the tiles' sums one by one in tile order, so nothing changes
        # in the result.
        fused = self._whole_sweep(original, feedback, output, coefficients, collected) if on_device else False
        if fused:
            return collected.result(output, permutation, refit_width, ctx)
        deferred: list[tuple[int, int]] = []
        limit = 0

        def flush() -> None:
            index = 0
            while index < len(deferred):  # runs of equally wide consecutive tiles
                run = index + 1
                chain = deferred[index][1] - deferred[index][0]
                while run < len(deferred) and deferred[run][1] - deferred[run][0] == chain:
                    run += 1
                kernel.block_update_range(feedback, original, output, coefficients, deferred[index][0], chain,
                                          run - index, limit, width)
                index = run
            deferred.clear()

        for region_start in range(0, width, refit_width):
            region_stop = min(width, region_start + refit_width)
            if deferred and region_stop > limit:
                flush()
            if not deferred:
                limit = min(width, max(region_start + DEFERRED_TILES * self.block_size, region_stop))
            targets = original[:, region_start:region_stop]
            if region_start:
                if on_device and region_stop - region_start <= MAXIMUM_FUSED_TILE:
                    targets = kernel.pending_continuation(feedback, coefficients, region_start, region_stop,
                                                          original=original)
                else:
                    targets = targets + self._pending_continuation(feedback, coefficients, region_start, region_stop)
            fitted_ctx = ctx if statistics is None else ctx.derive(statistics)
            rounder = fit_quantizer(self.inner, targets, fitted_ctx)
            del targets
            if fitted_ctx is not ctx:
                ctx.add_bits(fitted_ctx.additional_bits)
            state = self._kernel_state(rounder, w.device)
            scalar = state if isinstance(state, ScalarRounding) else None
            vector = state if isinstance(state, VectorRounding) else None
            encoded = None
            if scalar is not None:
                encoded = collected.open_scalar_region(scalar)
            elif vector is not None:
                encoded = collected.open_vector_region(vector)
            for tile_start in range(region_start, region_stop, self.block_size):
                tile_stop = min(region_stop, tile_start + self.block_size)
                if scalar is not None:
                    kernel.round_tile(original, feedback, coefficients, scalar.scales.contiguous(),
                                      None if scalar.zero is None else scalar.zero.contiguous(), output, encoded,
                                      region_start=region_start, tile_start=tile_start,
                                      tile_width=tile_stop - tile_start, group=scalar.group, bits=scalar.grid.bits,
                                      values=scalar.values, integer_grid=scalar.grid.integer)
                elif vector is not None:
                    kernel.round_vector_tile(original, feedback, coefficients, vector.scales.contiguous(),
                                             vector.codebook, output, encoded, region_start=region_start,
                                             tile_start=tile_start, tile_width=tile_stop - tile_start,
                                             group=vector.group, dimension=vector.grid.dim,
                                             codebook_size=vector.codebook_size, lattice=vector.lattice)
                else:
                    self._round_tile_by_blocks(rounder, original, feedback, coefficients, output, collected,
                                               region_start, tile_start, tile_stop)
                if tile_stop >= width:
                    continue
                if not on_device:
                    deviations = original[:, tile_start:tile_stop] - output[:, tile_start:tile_stop]
                    feedback[:, tile_stop:].addmm_(deviations, coefficients[tile_start:tile_stop, tile_stop:])
                    continue
                if tile_stop < limit:
                    kernel.block_update_range(feedback, original, output, coefficients, tile_start,
                                              tile_stop - tile_start, 1, tile_stop, limit)
                if limit < width:
                    deferred.append((tile_start, tile_stop))
                    if tile_stop >= limit:
                        flush()
        return collected.result(output, permutation, refit_width, ctx)


def ldlq(inner: Callable[..., "Q | Tensor"], **options: Any) -> ErrorFeedback:
    return ErrorFeedback(inner, **options)


def gptq(inner: Callable[..., "Q | Tensor"], refit: int | None = 128, act_order: bool = False,
         **options: Any) -> ErrorFeedback:
    return ldlq(inner, step=1, refit=refit, order="activation" if act_order else "natural", **options)
