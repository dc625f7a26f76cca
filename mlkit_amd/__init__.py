"""mlkit's packed-inference and fused-quantization path on MI355X (gfx950).

The public names are the reference's (``import mlkit_amd as mk``): ``mk.scaled`` /
``mk.int`` / ``mk.nf4`` / ``mk.mxfp4``, ``mk.grid``, ``mk.codec``, ``mk.gptq`` / ``mk.ldlq``,
``mk.pack`` / ``mk.unpack``, ``mk.hadamard`` / ``mk.rht``, ``mk.snap`` / ``mk.nearest``, ``mk.proxy_loss``,
``mk.PackedLinear``, ``mk.optimize``, ``mk.capabilities``, ``mk.Q`` / ``mk.Ctx`` /
``mk.Quantizer`` / ``mk.quantizer``, ``mk.save`` / ``mk.load_checkpoint``.  Every fused path
runs a hand-written HIP kernel from ``libmlkit_amd.so`` (``python -m mlkit_amd.build``) and
raises if that library is missing.
"""

from mlkit_amd.checkpoints import load_checkpoint, save
from mlkit_amd.conversion import Rotate, install_transform, rotate
from mlkit_amd.evaluation.capabilities import Capabilities, capabilities
from mlkit_amd.inference.optimization import optimize
from mlkit_amd.inference.packed_linear import PackedEmbedding, PackedLinear, packed_compatible
from mlkit_amd.models import Model, QModel, quantize
from mlkit_amd.quantization.bitstream import pack, unpack
from mlkit_amd.quantization.codecs import codec, concatenate_rows, deterministic_signs
from mlkit_amd.quantization.core import Ctx, Q, Quantizer, layer_seed, quantizer
from mlkit_amd.quantization.feedback import clear_factor_graphs, feedback_coefficients, gptq, ldlq, proxy_loss
from mlkit_amd.quantization.grids import NF4_VALUES, Grid, grid
from mlkit_amd.quantization.incoherence import Incoherent, incoherent
from mlkit_amd.quantization.scaled import Scaled, int, mxfp4, nf4, scaled, store_scale  # noqa: A004
from mlkit_amd.quantization.search import nearest, snap
from mlkit_amd.quantization.transforms import hadamard, paley_matrix, rht, structured_transform, transform_factor

__version__ = "0.1.0"


@quantizer
def rtn(w, ctx=None, *, fmt=None):
    """Round to nearest with ``fmt`` (default ``mk.int(4)``): the reference's ``mk.rtn``."""
    return (fmt or int(4))(w, ctx)


__all__ = [
    "Capabilities", "Ctx", "Grid", "Model", "NF4_VALUES", "PackedEmbedding", "PackedLinear", "Q", "QModel",
    "Quantizer", "Rotate", "Scaled", "capabilities", "clear_factor_graphs", "codec", "concatenate_rows", "deterministic_signs",
    "feedback_coefficients", "gptq", "grid", "hadamard", "incoherent", "install_transform", "int", "layer_seed", "ldlq", "load_checkpoint", "mxfp4",
    "nearest", "nf4", "optimize", "pack", "packed_compatible", "paley_matrix", "proxy_loss", "quantize", "quantizer", "rht",
    "rotate", "rtn", "save", "scaled", "snap", "store_scale", "structured_transform", "transform_factor", "unpack",
]
