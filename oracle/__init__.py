"""CPU oracle for the FlashOmni sparse-attention hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package may import this
module: it exists so that tests, the smoke entry point and the benchmark's
CPU-baseline leg can check (or time) a plain restatement of what the
reference computes.  Every function cites the reference lines it follows.

Pinning status (what each restatement is checked against, see tests/):

* packbits / segment_packbits  -- numpy.packbits + the two docstring
  known-answer vectors of flashomni/quantization.py:90-93,133-138.  pinned.
* indptr helpers               -- closed forms.  pinned.
* prefill planner              -- closed forms / brute force on tiny inputs.  pinned.
* symbol decoder               -- independent per-bit python loop on hand-written
  fixtures (tests/golden/decoder_cases.json).  pinned.
* dense masked attention       -- torch scaled_dot_product_attention special
  cases, single-block softmax, permutation invariance.  pinned.
* masked GEMM-Q / GEMM-O       -- F.linear special cases, cache+final identity.  pinned.
* fp8 block quantizer, fp8 attention -- NOT in the reference (it has no absmax
  quantizer and up-casts fp8 to fp16 before its MMA): parity unpinned against
  the reference; pinned only by closed forms (scale = absmax/448, torch's own
  float8_e4m3fn cast) and by the fp32 dense masked reference at rel-L2 3e-2.
* symbol producer (producer.py) -- the reference holds no vectors for it (its script
  prints); pinned by hand-worked rows with exactly representable probabilities, by a
  remove-the-smallest brute force, by the script's own consistency checks
  (benchmark/test_attn_score.py:155-160) and by mass invariants.  The order of equal
  scores and rows whose cumulative mass meets the threshold within fp32 rounding are
  left open by the reference (torch.sort / torch.cumsum): parity unpinned there.
"""
from .symbols import (  # noqa: F401
    get_bit, packbits, segment_packbits, sparse_info_indptr_bits,
    sparse_kv_info_indptr_bits, decode_rows, decode_kv_csr, decode_head_csr,
)
from .planner import prefill_plan  # noqa: F401
from .attention import sparse_attention  # noqa: F401
from .gemm import gemm_q, gemm_o  # noqa: F401
from .quant import quant_fp8_block, dequant_fp8_block  # noqa: F401
from . import producer  # noqa: F401
