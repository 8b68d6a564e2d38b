"""ixrun_amd: the INT8-X fused decode+GEMV path of dfytensor/ixrun for MI355X.

Hand-written gfx950 HIP kernels behind a C ABI (``include/ixhip.h``,
``ixrun_amd/csrc``) with the reference's Python surface on top:

=====================  =====================================================
``ixrun_amd.config``   level scheme and code-offset tables
``ixrun_amd.bitpack``  bit-stream layout (host packer / unpacker)
``ixrun_amd.quantize`` ``int8x_quantize`` and the torch scatter decoder
``ixrun_amd.triton_kernels``  device decode (name kept for import compatibility)
``ixrun_amd.fused``    ``fused_gemv``, ``compute_row_prefixes``
``ixrun_amd.linear``   ``Int8XLinear``, ``deploy_model``
``ixrun_amd.engine``   ``StreamingLinear``, ``GraphLinear``, ``Int8XEngine``
=====================  =====================================================
"""
from .config import BIT_TO_THRESHOLD, DEFAULT_LEVELS
from .quantize import int8x_quantize, decode_to_weight, compute_positions
from .bitpack import pack_bits_stream, unpack_bits_stream, pack_bitmap
from .fused import fused_gemv, compute_row_prefixes, FUSED_TILE
from .triton_kernels import decode_weight_triton, decode_weight_scatter, precompute_block_offsets
from .linear import Int8XLinear, deploy_model, iter_quantizable_linears
from .engine import Int8XEngine, StreamingLinear, GraphLinear, ResourceScheduler

__version__ = "0.1.0"
