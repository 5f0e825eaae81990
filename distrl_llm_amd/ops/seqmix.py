"""Sequence-mixing ops for layer-list models: dispatch to the gfx950
kernels of ``csrc_seqmix`` on a GPU, to ``seqmix_reference`` on the CPU.

A GPU tensor requires the compiled extension: a missing build raises, it
never falls back to eager torch. Matrix products stay with the vendor
GEMM (``F.linear`` / ``torch.bmm``); everything between them runs here.
Every op takes its sizes and constants as arguments, so a new design
combines them freely.
"""

from __future__ import annotations

import torch

from . import seqmix_reference as R
from .build import get_seqmix_extension


def _ext(op: str):
    ext = get_seqmix_extension()
    if ext is None:
        raise RuntimeError(
            f"seqmix op '{op}' called on a GPU tensor but the gfx950 "
            f"extension is not built/loadable (python -m distrl_llm_amd.ops.build)")
    return ext


def _bf16(dtype) -> bool:
    if dtype not in (torch.bfloat16, torch.float32):
        raise ValueError(f"seqmix ops run in bfloat16 or float32, not {dtype}")
    return dtype == torch.bfloat16


def offset_rmsnorm(x, w, eps, out_dtype):
    if x.is_cuda:
        return _ext("offset_rmsnorm").offset_rmsnorm(x.contiguous(), w, eps,
                                                     _bf16(out_dtype))
    return R.offset_rmsnorm(x, w, eps, out_dtype)


def causal_tap_conv(h, w, tails, cu, tok_seq, slots, out_dtype):
    if h.is_cuda:
        return _ext("causal_tap_conv").causal_tap_conv(
            h, w, tails, cu, tok_seq, slots, _bf16(out_dtype))
    return R.causal_tap_conv(h, w, tails, cu, slots, out_dtype)


def latent_prepare(proj, heads, dim, rot_dim, kv_rank, own_cache, norm_w, eps,
                   positions, rope_base, rope_dims, page_slot, cache):
    if proj.is_cuda:
        return _ext("latent_prepare").latent_prepare(
            proj, heads, dim, rot_dim, kv_rank, own_cache, norm_w, eps,
            positions, rope_base, rope_dims, page_slot, cache)
    return R.latent_prepare(proj, heads, dim, rot_dim, kv_rank, own_cache,
                            norm_w, eps, positions, rope_base, rope_dims,
                            page_slot, cache)


QUERY_TILE = 16   # most queries of one sequence the tiled kernel takes at once
WIDE_QUERY_TILE = 64   # the same for the K/V attention kernel (four waves x 16)


def query_tiles(row_lengths, tile=QUERY_TILE):
    """Cut each batch row's tokens into tiles of up to ``tile`` consecutive
    queries: [(batch row, first flat token, queries)], and the largest
    tile."""
    tiles, at = [], 0
    for b, n in enumerate(row_lengths):
        for k in range(0, n, tile):
            tiles.append((b, at + k, min(tile, n - k)))
        at += n
    return tiles, max((t[2] for t in tiles), default=1)


def latent_window_attention(q_lat, q_rot, cache, kv_rank, block_tables,
                            block_size, cu, tok_seq, positions, window, scale,
                            out_dtype, tiles=None, max_tile=0):
    """``tiles`` (int32 [n, 3] from :func:`query_tiles`, with ``max_tile``)
    selects the tiled MFMA kernel for bf16; without it, or in fp32, the
    one-wave-per-query kernel runs."""
    if q_lat.is_cuda:
        return _ext("latent_window_attention").latent_window_attention(
            q_lat.contiguous(), q_rot, cache, kv_rank, block_tables,
            block_size, tok_seq, positions, window, scale, tiles, max_tile)
    return R.latent_window_attention(q_lat, q_rot, cache, kv_rank, block_tables,
                                     block_size, cu, positions, window, scale,
                                     out_dtype)


SCAN_CHUNK = 64    # tokens per parallel chunk of a long row's recurrence


def scan_chunks(row_lengths):
    """Chunks of up to SCAN_CHUNK consecutive tokens per batch row, for the
    parallel form of the recurrence: ([(row, first flat token, tokens)],
    per-row chunk offsets). Empty when no row is longer than one chunk."""
    if max(row_lengths, default=0) <= SCAN_CHUNK:
        return [], []
    chunks, cu, at = [], [0], 0
    for b, n in enumerate(row_lengths):
        for k in range(0, n, SCAN_CHUNK):
            chunks.append((b, at + k, min(SCAN_CHUNK, n - k)))
        cu.append(len(chunks))
        at += n
    return chunks, cu


def mingru_scan(zxg, bias, state, cu, slots, out_dtype, chunks=None,
                chunk_cu=None):
    """``chunks``/``chunk_cu`` (from :func:`scan_chunks`) select the
    three-pass chunk-parallel kernels; without them each (row, channel)
    walks its tokens in order."""
    if zxg.is_cuda:
        if chunks is not None and chunks.numel() == 0:
            chunks = chunk_cu = None
        return _ext("mingru_scan").mingru_scan(zxg, bias, state, cu, slots,
                                               chunks, chunk_cu)
    return R.mingru_scan(zxg, bias, state, cu, slots, out_dtype)


def moe_route(h, router_w, router_b, top):
    if h.is_cuda:
        return _ext("moe_route").moe_route(h, router_w, router_b, top)
    return R.moe_route(h, router_w, router_b, top)


def moe_experts(h, idx, wts, exp_gu, exp_down):
    if h.is_cuda:
        return _ext("moe_experts").moe_experts(h, idx, wts, exp_gu, exp_down)
    return R.moe_experts(h, idx, wts, exp_gu, exp_down)


def gated_residual_add(x, mix, ff, gates, gate_b, mult):
    if x.is_cuda:
        _ext("gated_residual_add").gated_residual_add(x, mix, ff, gates,
                                                      gate_b, mult)
        return x
    return R.gated_residual_add(x, mix, ff, gates, gate_b, mult)


def gated_residual_norm(x, mix, ff, gates, gate_b, mult, next_w, eps,
                        out_dtype):
    """Fused layer tail: the gated residual update followed by the next
    layer's offset RMS norm of the new residual. Returns (fp32, out_dtype)
    normed rows; x is updated in place."""
    if x.is_cuda:
        return _ext("gated_residual_norm").gated_residual_norm(
            x, mix, ff, gates, gate_b, mult, next_w, eps, _bf16(out_dtype))
    R.gated_residual_add(x, mix, ff, gates, gate_b, mult)
    return R.offset_rmsnorm(x, next_w, eps, out_dtype)


# ------------------------------------------------- sandwich-block mechanisms

def sandwich_residual_norm(x, y, y2, post_w, next_w, eps, out_dtype):
    """Fused sublayer tail: x += rms_unit(y [+ y2]) * (1 + post_w) on the
    fp32 residual (in place), then, with ``next_w``, the next offset RMS
    norm of the new residual in ``out_dtype``; None without."""
    if x.is_cuda:
        return _ext("sandwich_residual_norm").sandwich_residual_norm(
            x, y.contiguous(), None if y2 is None else y2.contiguous(), post_w,
            next_w, eps, _bf16(out_dtype))
    return R.sandwich_residual_norm(x, y, y2, post_w, next_w, eps, out_dtype)


def rope_kv_write(proj, heads, kv_heads, dim, vdim, positions, rope_base,
                  rope_dims, page_slot, cache, vmix=None, v_first=None):
    if proj.is_cuda:
        return _ext("rope_kv_write").rope_kv_write(
            proj, heads, kv_heads, dim, vdim, positions, rope_base, rope_dims,
            page_slot, cache, vmix, v_first)
    return R.rope_kv_write(proj, heads, kv_heads, dim, vdim, positions,
                           rope_base, rope_dims, page_slot, cache, vmix, v_first)


def sink_attention(q, cache, heads, kv_heads, dim, vdim, block_tables,
                   block_size, cu, tok_seq, positions, scale, softcap, sink,
                   talk, out_dtype, tiles=None, max_tile=0):
    """``tiles`` (from :func:`query_tiles` with ``WIDE_QUERY_TILE``) selects
    the tiled MFMA kernel for bf16 prompt portions; decode steps and fp32
    models run one wave per (token, head)."""
    if q.is_cuda:
        return _ext("sink_attention").sink_attention(
            q, cache, heads, kv_heads, dim, vdim, block_tables, block_size,
            tok_seq, positions, scale, softcap, sink, talk, tiles, max_tile)
    return R.sink_attention(q, cache, heads, kv_heads, dim, vdim, block_tables,
                            block_size, cu, positions, scale, softcap, sink,
                            talk, out_dtype)


def tap_conv_silu(x, w, tails, cu, tok_seq, slots, out_dtype):
    """``x`` may be a column slice of a wider row-major matrix. Every row of
    the step holds at least one token (a step whose rows all hold exactly
    one runs conv and tail update as one kernel)."""
    if x.is_cuda:
        return _ext("tap_conv_silu").tap_conv_silu(x, w, tails, cu, tok_seq,
                                                   slots, _bf16(out_dtype))
    return R.tap_conv_silu(x, w, tails, cu, slots, out_dtype)


def gated_delta_rule(qkv, gate, ab, a_log, dt_bias, onorm_w, eps, state, cu,
                     slots, heads, kv_heads, dim, vdim, out_dtype, h=None,
                     ab_w=None):
    """``ab`` None: the [strength | step] inputs are projected inside the op
    from the mixer input ``h`` with the fp32 matrix ``ab_w`` [2H, D]."""
    if qkv.is_cuda:
        return _ext("gated_delta_rule").gated_delta_rule(
            qkv, gate, ab, h, ab_w, a_log, dt_bias, onorm_w, eps, state, cu,
            slots, heads, kv_heads, dim, vdim)
    if ab is None:
        ab = torch.nn.functional.linear(h.float(), ab_w.float())
    return R.gated_delta_rule(qkv, gate, ab, a_log, dt_bias, onorm_w, eps,
                              state, cu, slots, heads, kv_heads, dim, vdim,
                              out_dtype)


def capped_glu(gu, limit):
    if gu.is_cuda:
        return _ext("capped_glu").capped_glu(gu, limit)
    return R.capped_glu(gu, limit)


def moe_route_all(h, router_w, correction, top, scale):
    if h.is_cuda:
        return _ext("moe_route_all").moe_route_all(h, router_w, correction,
                                                   top, scale)
    return R.moe_route_all(h, router_w, correction, top, scale)


def moe_experts_glu(h, idx, wts, exp_gu, exp_down, limit):
    if h.is_cuda:
        return _ext("moe_experts_glu").moe_experts_glu(h, idx, wts, exp_gu,
                                                       exp_down, limit)
    return R.moe_experts_glu(h, idx, wts, exp_gu, exp_down, limit)
