"""MI355X (gfx950) FlashOmni sparse-attention engine.

Same public names as the reference package (flashomni/__init__.py:17-28); every op runs in
hand-written HIP kernels through the C ABI of include/flashomni_hip.h."""
from .attention import BatchFlashOmniFAWithRaggedKVWrapper, DecodedWorkList  # noqa: F401
from .gemm import flashomni_gemm, flashomni_gemm_reduction  # noqa: F401
from .quantization import packbits, quant_fp8_block, segment_packbits, token_blocks  # noqa: F401
from .symbols import sparse_symbols_from_scores  # noqa: F401
from . import ops  # noqa: F401  (registers torch.ops.flashomni_kernels.*)

__version__ = "0.1.0"
