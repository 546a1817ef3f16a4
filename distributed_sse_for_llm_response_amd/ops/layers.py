"""Layer-mechanism ops for configuration-driven designs: HIP kernels on GPU tensors, ``layers_reference`` on CPU tensors.

Dispatch follows ``ops/__init__.py``: a GPU tensor always takes the HIP kernel (the call raises when the kernel library
is missing), a CPU tensor the PyTorch reference.  The element type (bf16, or fp32 for the exact mode) comes with the
tensors; sizes and constants are arguments, so another design reuses the same ops with its own numbers.
"""
from __future__ import annotations

import torch

from . import layers_reference as lref


def _hip(t: torch.Tensor) -> bool:
    if t.is_cuda:
        from . import load_library

        load_library(required=True)
        return True
    return False


def gemm_rm(x, w, out, bias=None, act: int = 0):
    """out = act(x · wᵀ + bias) for row-major w [N, K]; any sizes; 3-D operands are batched over dim 0 (strided views
    of wider buffers are fine: only the innermost stride must be 1).  act: 0 none, 1 gelu (tanh form)."""
    if _hip(x):
        torch.ops.dsse.gemm_rm(x, w, out, bias, act)
    else:
        lref.gemm_rm(x, w, out, bias, act)


def scalar_norm(y, g, resid, xb, eps: float, nsum: int = 1):
    """y given: resid += y / rms(y) · g (one number g), xb = resid rounded; y [M · nsum, W] holds each row in nsum
    consecutive parts that are summed first (the grouped experts' slots).  y None: xb = resid / rms(resid) · g."""
    if _hip(resid):
        torch.ops.dsse.scalar_norm(y, g, resid, xb, eps, nsum)
    else:
        lref.scalar_norm(y, g, resid, xb, eps, nsum)


def embed_rows(ids, embed, resid, xb):
    """resid (fp32) = xb = embed[ids]."""
    if _hip(resid):
        torch.ops.dsse.embed_rows(ids, embed, resid, xb)
    else:
        lref.embed_rows(ids, embed, resid, xb)


def latent_kv_write(ckr, norm_w, positions, slots, rope, cache, eps: float, vt=None):
    """cache[slot] = [rms-norm(ckr[:, :rk]) · norm_w | rot(ckr[:, rk:])] for rows with slot >= 0; vt (optional,
    [pages, rk, 32]) receives the latent once more in transposed pages (the MFMA attention's value operand)."""
    if _hip(ckr):
        torch.ops.dsse.latent_kv_write(ckr, norm_w, positions, slots, rope, cache, eps, vt)
    else:
        lref.latent_kv_write(ckr, norm_w, positions, slots, rope, cache, eps, vt)


def latent_flash_ok(dtype, rk: int, dr: int) -> bool:
    """Shapes the MFMA form of latent_attention covers (everything else takes the row kernel)."""
    return dtype == torch.bfloat16 and rk in (64, 128, 256, 512) and dr % 32 == 0


def latent_flash_part_floats(items: int, heads: int, hp: int, nparts: int, rk: int) -> int:
    """fp32 words of the key-split scratch of latent_attention's MFMA form."""
    return items * (-(-heads // hp)) * nparts * 16 * (rk + 2)


def latent_attention(q, q_abs, cache, block_tables, q_start, q_len, ctx_len, work_seq, work_tile, rope, out,
                     window: int, scale: float, qt: int, vt=None, hp: int = 1, part=None, nparts: int = 1):
    """Sliding-window multi-query attention over the latent cache (folded form), `qt` query rows per work item.
    With vt (transposed latent pages, latent_flash_ok shapes): the MFMA form, qt rows x hp heads = 16 columns per
    item, the item's keys optionally split over `nparts` partitions (fp32 scratch `part`, latent_flash_part_floats)
    and merged by a combine kernel; without vt: the row kernel (any sizes, both element types)."""
    if _hip(q):
        torch.ops.dsse.latent_attention(q, q_abs, cache, block_tables, q_start, q_len, ctx_len, work_seq, work_tile,
                                        rope, out, window, scale, qt, vt, hp, part, nparts)
    else:
        lref.latent_attention(q, q_abs, cache, block_tables, q_start, q_len, ctx_len, work_seq, work_tile, rope, out,
                              window, scale, qt, vt)


def conv_state(inp, taps, bias, tail, q_start, q_len, ctx_len, state_slot, out, out_b, in_bias=None):
    """Per-channel causal convolution continued from each sequence's slot tail (and the tail's update); in_bias is
    added to every input (the bias of the projection that made `inp`)."""
    if _hip(inp):
        torch.ops.dsse.conv_state(inp, taps, bias, tail, q_start, q_len, ctx_len, state_slot, out, out_b, in_bias)
    else:
        lref.conv_state(inp, taps, bias, tail, q_start, q_len, ctx_len, state_slot, out, out_b, in_bias)


def lru_scan(u, gates, y, lam, state, q_start, q_len, ctx_len, state_slot, out, c: float, y_bias=None,
             coeff: bool = True, scratch=None):
    """Real-gated linear recurrence continued from each sequence's slot state; out = state · gelu(y + y_bias).
    coeff: turn the gate pre-activations of ALL rows into the recurrence's coefficients first (in place); pass False
    for a further sequence group of the same step.  scratch (fp32 [2, rows / 32 + sequences + 1, C]): steps of 128 rows
    or more walk in three phases over 32-row chunks instead of one thread per sequence and channel."""
    if _hip(u):
        torch.ops.dsse.lru_scan(u, gates, y, lam, state, q_start, q_len, ctx_len, state_slot, out, c, y_bias, coeff,
                                scratch)
    else:
        lref.lru_scan(u, gates, y, lam, state, q_start, q_len, ctx_len, state_slot, out, c, y_bias, coeff)


def moe_topk(logits, topk_idx, topk_w):
    """The top-k experts of fp32 router logits [M, E] and the softmax over the chosen logits."""
    if _hip(logits):
        torch.ops.dsse.moe_topk(logits, topk_idx, topk_w)
    else:
        lref.moe_topk(logits, topk_idx, topk_w)


def moe_router(x, w, b, topk_idx, topk_w):
    """fp32 router logits, the top-k experts per row and the softmax over the chosen logits."""
    if _hip(x):
        torch.ops.dsse.moe_router(x, w, b, topk_idx, topk_w)
    else:
        lref.moe_router(x, w, b, topk_idx, topk_w)


def moe_ffn(x, topk_idx, topk_w, gate, up, down, sgate, sup, sdown, out):
    """out (fp32) = sum_k w_k · expert_k(x) + shared(x), experts of the gated-SiLU form."""
    if _hip(x):
        torch.ops.dsse.moe_ffn(x, topk_idx, topk_w, gate, up, down, sgate, sup, sdown, out)
    else:
        lref.moe_ffn(x, topk_idx, topk_w, gate, up, down, sgate, sup, sdown, out)


def moe_grouped(x, topk_idx, topk_w, gate, up, down, sgate, sup, sdown, sorted_ids, tile_expert, num_tiles, h, o):
    """Grouped form of the routed experts: rows sorted by expert, 16-row MFMA tiles of one expert each.  o [M · S, W]
    (fp32) = weight · expert output per (row, slot), S = top (+ 1: the shared expert's slot); scalar_norm(nsum=S) sums
    them.  sorted_ids / tile_expert / num_tiles / h are scratch."""
    if _hip(x):
        torch.ops.dsse.moe_grouped(x, topk_idx, topk_w, gate, up, down, sgate, sup, sdown, sorted_ids, tile_expert,
                                   num_tiles, h, o)
    else:
        lref.moe_grouped(x, topk_idx, topk_w, gate, up, down, sgate, sup, sdown, o)
