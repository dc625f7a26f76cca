"""Orthogonal structured transforms of ordinary transformer widths.

Mirrors /root/reference/src/mlkit/quantization/operations/orthogonal_transforms.py:
  :12-31     hadamard                 :34-67    prime, paley_matrix
  :70-98     transform_factor         :101-109  structured_transform
  :112-122   randomized_transform, rht
FP32 / FP16 / BF16 tensors on a HIP device run ``mk_fwht`` (one launch per tensor) and
``mk_basis_mix``; ``rotate`` additionally fuses the sign flips into those launches.
Host tensors and tensors that track gradients use the stage-by-stage tensor operations.
"""

import functools
import math

import torch
from torch import Tensor

_KERNEL_DTYPES = {torch.float32, torch.float16, torch.bfloat16}
MAXIMUM_KERNEL_WIDTH = 32768
MAXIMUM_KERNEL_ORDER = 256


def _on_kernel(value: Tensor) -> bool:
    tracked = torch.is_grad_enabled() and value.requires_grad
    return value.is_cuda and value.dtype in _KERNEL_DTYPES and not tracked and value.shape[-1] <= MAXIMUM_KERNEL_WIDTH


def hadamard(value: Tensor, *, normalize: bool = True) -> Tensor:
    """Fast Walsh-Hadamard transform along the final dimension (natural order)."""
    width = value.shape[-1]
    if width <= 0 or width & (width - 1):
        raise ValueError("hadamard currently requires a power-of-two final dimension")
    if _on_kernel(value):
        from mlkit_amd.kernels import hadamard as kernel

        return kernel.transform(value.contiguous(), normalize=normalize)
    out = value.clone()
    stride = 1
    while stride < width:
        pairs = out.reshape(*value.shape[:-1], -1, 2, stride)
        low, high = pairs[..., 0, :], pairs[..., 1, :]
        out = torch.stack((low + high, low - high), dim=-2).reshape_as(value)
        stride *= 2
    return out / math.sqrt(width) if normalize else out


def prime(value: int) -> bool:
    return value >= 2 and all(value % divisor for divisor in range(2, math.isqrt(value) + 1))


def _quadratic_characters(field: int) -> Tensor:
    """chi(i - j) over the prime field: +1 for nonzero squares, -1 for non-squares, 0 on the diagonal."""
    index = torch.arange(field)
    is_square = torch.zeros(field)
    is_square[(index[1:] ** 2) % field] = 1
    difference = (index[:, None] - index[None, :]) % field
    return torch.where(difference == 0, 0.0, 2 * is_square[difference] - 1)


@functools.lru_cache(maxsize=32)
def paley_matrix(order: int) -> Tensor:
    """An orthonormal Hadamard matrix of a Paley order: q + 1 (q = 3 mod 4) or 2(q + 1) (q = 1 mod 4)."""
    if prime(order - 1) and (order - 1) % 4 == 3:
        field = order - 1
        matrix = torch.ones(order, order)
        matrix[1:, 0] = -1
        matrix[1:, 1:] = _quadratic_characters(field) + torch.eye(field)
        return matrix / math.sqrt(order)
    field = order // 2 - 1
    if order % 2 == 0 and prime(field) and field % 4 == 1:
        conference = torch.ones(field + 1, field + 1)
        conference[0, 0] = 0
        conference[1:, 1:] = _quadratic_characters(field)
        eye = torch.eye(field + 1)
        top = torch.cat((conference + eye, conference - eye), dim=1)
        bottom = torch.cat((conference - eye, -conference - eye), dim=1)
        return torch.cat((top, bottom), dim=0) / math.sqrt(order)
    raise ValueError(f"no prime-field Paley construction for order {order}")


@functools.lru_cache(maxsize=128)
def transform_factor(width: int) -> tuple[int, int, Tensor | None]:
    """``(order, power, basis)`` with ``width = order * power``: a dense orthonormal basis of
    ``order`` and a Hadamard power of two.  Widths without a Paley construction keep their
    odd factor as an orthonormal DCT-II basis."""
    if width < 1:
        raise ValueError("transform width must be positive")
    if width & (width - 1) == 0:
        return 1, width, None
    odd = width
    while odd % 2 == 0:
        odd //= 2
    power = width // odd
    for multiplier in (1, 2, 4, 8, 16):
        if power % multiplier:
            continue
        try:
            return odd * multiplier, power // multiplier, paley_matrix(odd * multiplier)
        except ValueError:
            continue
    index = torch.arange(odd, dtype=torch.float64)
    matrix = torch.cos(math.pi / odd * (index[None, :] + 0.5) * index[:, None])
    matrix[0] *= 1 / math.sqrt(odd)
    matrix[1:] *= math.sqrt(2 / odd)
    return odd, power, matrix.float()


@functools.lru_cache(maxsize=64)
def _basis_on(width: int, device: torch.device) -> Tensor:
    basis = transform_factor(width)[2]
    assert basis is not None
    return basis.to(device).contiguous()


ONE_LAUNCH_ROWS = 256
ROW_KERNEL_ROWS = 64   # activation rows the per-block rotation kernel takes (mk_rotate_rows)


def _rotate_blocks_separately(value: Tensor, block: int, inverse: bool, signs: Tensor | None) -> Tensor:
    """The final dimension as blocks of ``block`` values (a power of two), each
    Walsh-Hadamard-transformed for itself: ``(I (x) H_block) / sqrt(block)``, its own inverse."""
    width = value.shape[-1]
    if block < 2 or block & (block - 1) or width % block:
        raise ValueError(f"blocks of {block} values do not tile a width of {width} as powers of two")
    before, after = (None, signs) if inverse else (signs, None)
    blocks = value.reshape(*value.shape[:-1], width // block, block)
    if _on_kernel(value) and block <= MAXIMUM_KERNEL_WIDTH:
        from mlkit_amd.kernels import hadamard as kernel

        def as_kernel_signs(vector):
            return None if vector is None else vector.to(device=value.device, dtype=torch.float32).contiguous()

        out = kernel.transform(blocks.contiguous(), signs_before=as_kernel_signs(before), signs_after=as_kernel_signs(after))
        return out.reshape(value.shape)
    if before is not None:
        blocks = (value * before).reshape(blocks.shape)
    out = hadamard(blocks).reshape(value.shape)
    return out * after if after is not None else out


def rotate(value: Tensor, *, inverse: bool = False, signs: Tensor | None = None, block: int | None = None) -> Tensor:
    """``structured_transform`` with optional fused sign flips: forward ``T(value * signs)``,
    inverse ``T^-1(value) * signs``.  Two launches at most on a HIP device.  ``block``: T
    transforms blocks of that many values one by one instead (no counterpart in the reference,
    whose T always spans the row; a row of whole 2048-value blocks is what a packed layer can
    rotate inside its own matvec launch)."""
    if block is not None:
        return _rotate_blocks_separately(value, block, inverse, signs)
    order, power, basis = transform_factor(value.shape[-1])
    if not (_on_kernel(value) and power <= MAXIMUM_KERNEL_WIDTH and order <= MAXIMUM_KERNEL_ORDER):
        if signs is not None and not inverse:
            value = value * signs
        out = _structured_on_host(value, order, power, basis, inverse)
        return out * signs if signs is not None and inverse else out
    from mlkit_amd.kernels import hadamard as kernel

    if signs is not None:
        signs = signs.to(device=value.device, dtype=torch.float32).contiguous()
    before, after = (None, signs) if inverse else (signs, None)
    value = value.contiguous()
    if basis is None:
        return kernel.transform(value, signs_before=before, signs_after=after)
    blocks = value.reshape(*value.shape[:-1], order, power)
    # Activations (few rows) take the one-launch kernel that works in LDS; weight-sized tensors
    # take the one-pass kernel that transforms in registers where it applies, and stream through
    # the two kernels otherwise (measured at 4096 x 14336: 0.20 ms in two launches, 0.27 ms
    # through the LDS kernel).
    outer_rows = blocks.numel() // (order * power)
    if ((outer_rows <= ONE_LAUNCH_ROWS and kernel.fits_one_launch(order, power))
            or (outer_rows > ONE_LAUNCH_ROWS and kernel.streams_in_one_pass(blocks, order, power))):
        mixed = kernel.rotate_blocks(blocks, _basis_on(value.shape[-1], value.device), transpose=inverse,
                                     signs_before=before, signs_after=after)
        return mixed.reshape(value.shape)
    staged = torch.empty(blocks.shape, device=value.device, dtype=torch.float32)
    kernel.transform(blocks, signs_before=before, out=staged)
    mixed = kernel.mix_blocks(staged, _basis_on(value.shape[-1], value.device), transpose=inverse, signs_after=after)
    return mixed.reshape(value.shape).to(value.dtype)


def _structured_on_host(value: Tensor, order: int, power: int, basis: Tensor | None, inverse: bool) -> Tensor:
    if basis is None:
        return hadamard(value)
    blocks = hadamard(value.reshape(*value.shape[:-1], order, power)).transpose(-1, -2)
    basis = basis.to(device=value.device, dtype=value.dtype)
    mixed = blocks @ (basis if inverse else basis.T)
    return mixed.transpose(-1, -2).reshape_as(value)


def structured_transform(value: Tensor, *, inverse: bool = False) -> Tensor:
    """``(basis (x) H_power)`` along the final dimension; ``inverse`` applies its transpose."""
    return rotate(value, inverse=inverse)


@functools.lru_cache(maxsize=256)
def _cached_signs(width: int, seed: int, device: torch.device) -> Tensor:
    generator = torch.Generator(device=device).manual_seed(seed)
    return torch.randint(2, (width,), generator=generator, device=device).float() * 2 - 1


def random_signs(width: int, seed: int, device: torch.device | str, dtype: torch.dtype = torch.float32) -> Tensor:
    """The +-1 vector ``randomized_transform`` draws for ``seed`` on ``device`` (drawn once per
    width, seed and device: an online rotation reuses it on every call)."""
    return _cached_signs(width, seed, torch.device(device)).to(dtype)


def randomized_transform(value: Tensor, *, seed: int = 0, inverse: bool = False, block: int | None = None) -> Tensor:
    # the cached FP32 vector itself: +-1 is exact in every dtype and the kernels take FP32 signs
    signs = _cached_signs(value.shape[-1], seed, value.device)
    if not _on_kernel(value):
        signs = signs.to(value.dtype)
    return rotate(value, inverse=inverse, signs=signs, block=block)


class OnlineRotation:
    """``rht(value, seed=seed)`` for the forward pre-hook of a rotated layer: the same result
    with the per-call work reduced to one allocation and one library call (the launch
    arguments of a width, device and dtype are prepared once)."""

    def __init__(self, seed: int, block: int | None = None):
        self.seed = seed
        self.block = block   # None: the transform spans the row; else blocks of that many values, one by one
        self._plans: dict = {}

    def __getstate__(self) -> dict:
        """Prepared plans are closures over raw device addresses: a copy prepares its own."""
        return {"seed": self.seed, "block": self.block, "_plans": {}}

    def __deepcopy__(self, memo: dict) -> "OnlineRotation":
        return OnlineRotation(self.seed, self.block)

    def __call__(self, value: Tensor) -> Tensor:
        key = (value.shape[-1], value.device, value.dtype)
        plan = self._plans.get(key)
        if plan is None:
            plan = self._plans[key] = self._prepare(value)
        return plan(value)

    def launch_arguments(self, width: int, device: torch.device) -> tuple | None:
        """``(order, power, basis pointer or None, signs pointer, scale, keep)`` for
        ``mk_rotate_rows`` / ``mk_rotated_packed_matvec``, or None when the row-rotation kernel
        does not take this width (``keep`` holds the tensors the pointers belong to).  A plain
        power-of-two width is ``(1, width, None, ...)``."""
        from mlkit_amd.kernels import hadamard as kernel

        signs = _cached_signs(width, self.seed, device)
        if self.block is not None:   # no basis and several blocks: each block for itself
            block = self.block
            if block < 32 or block & (block - 1) or width % block or block > MAXIMUM_KERNEL_WIDTH or width == block:
                return None
            return width // block, block, None, signs.data_ptr(), kernel.normaliser(block), (signs,)
        order, power, basis = transform_factor(width)
        if basis is None:
            if width < 32 or width > MAXIMUM_KERNEL_WIDTH:
                return None
            return 1, width, None, signs.data_ptr(), kernel.normaliser(width), (signs,)
        if not 32 <= power <= 1024 or order > 65535:
            return None
        basis_on_device = _basis_on(width, device)
        return order, power, basis_on_device.data_ptr(), signs.data_ptr(), kernel.normaliser(power), (signs, basis_on_device)

    def _prepare(self, value: Tensor):
        """The callable for tensors of this width, device and dtype.  Up to ROW_KERNEL_ROWS rows
        (decode-time activations) go to ``mk_rotate_rows``: one short workgroup per output block
        and row.  Taller inputs take the transform-then-mix kernels of ``rotate``."""
        seed = self.seed
        width = value.shape[-1]

        block = self.block

        def general(tensor: Tensor) -> Tensor:
            return randomized_transform(tensor, seed=seed, block=block)

        arguments = self.launch_arguments(width, value.device) if _on_kernel(value) and block is None else None
        if arguments is None:
            return general
        from mlkit_amd import native

        order, power, basis, signs, scale, keep = arguments
        if order == 1:  # H_width = H_blocks (x) H_points, about sqrt(width) points per block
            points = 32
            while points * points < width and points < 1024:
                points *= 2
            order, power = width // points, points
        device = value.device
        code = native.dtype_code(value)
        launch = native.library().mk_rotate_rows

        def by_rows(tensor: Tensor) -> Tensor:
            rows = tensor.numel() // width
            if rows > ROW_KERNEL_ROWS or rows == 0:
                return general(tensor)
            if not tensor.is_contiguous():
                tensor = tensor.contiguous()
            output = torch.empty_like(tensor)
            native.check(launch(tensor.data_ptr(), code, output.data_ptr(), code, rows, order, power, basis, signs, scale,
                                native.current_stream(device)))
            return output

        by_rows.keeps = keep
        return by_rows


def rht(value: Tensor, *, seed: int = 0, inverse: bool = False, block: int | None = None) -> Tensor:
    return randomized_transform(value, seed=seed, inverse=inverse, block=block)
