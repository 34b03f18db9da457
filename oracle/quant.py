"""Per-(head, token-block) absmax fp8 e4m3fn quantiser.  Test infrastructure only.

There is NO counterpart in the reference (its quantization.cuh only packs bits, and its
prefill kernel up-casts fp8 storage to fp16: include/flashomni/attention/prefill.cuh:602-612).
parity unpinned against the reference; the definition below is the closed form
scale = absmax / 448 (448 = largest finite e4m3fn), x8 = round_to_nearest_even(x / scale),
all-zero block -> scale 1.  The optional residual term is the same rounding applied to what the
first term left: x8_lo = round_to_nearest_even(x / scale - x8)."""
import torch

FP8_MAX = 448.0


def quant_fp8_block(x, indptr, block=128, residual=False):
    """x [nnz,H,D] -> (x8 float8_e4m3fn [nnz,H,D], scale fp32 [H, total_blocks]) and, with
    residual=True, x8_lo = e4m3(x / scale - x8) as a third result.
    Blocks never straddle requests: request r owns ceil(len_r/block) consecutive blocks."""
    nnz, H, D = x.shape
    spans = []
    for r in range(len(indptr) - 1):
        a, b = int(indptr[r]), int(indptr[r + 1])
        t = a
        while t < b:
            spans.append((t, min(b, t + block)))
            t += block
    scale = torch.ones(H, len(spans), dtype=torch.float32)
    x8 = torch.empty(nnz, H, D, dtype=torch.float8_e4m3fn)
    x8_lo = torch.empty(nnz, H, D, dtype=torch.float8_e4m3fn)
    for j, (a, b) in enumerate(spans):
        blk = x[a:b].float()
        amax = blk.abs().amax(dim=(0, 2))
        s = torch.where(amax > 0, amax / FP8_MAX, torch.ones_like(amax))
        scale[:, j] = s
        scaled = (blk / s[None, :, None]).clamp(-FP8_MAX, FP8_MAX)
        x8[a:b] = scaled.to(torch.float8_e4m3fn)
        x8_lo[a:b] = (scaled - x8[a:b].float()).to(torch.float8_e4m3fn)
    return (x8, scale, x8_lo) if residual else (x8, scale)


def dequant_fp8_block(x8, scale, indptr, block=128):
    out = torch.empty(x8.shape, dtype=torch.float32)
    j = 0
    for r in range(len(indptr) - 1):
        a, b = int(indptr[r]), int(indptr[r + 1])
        t = a
        while t < b:
            e = min(b, t + block)
            out[t:e] = x8[t:e].float() * scale[:, j][None, :, None]
            j += 1
            t += block
    return out
