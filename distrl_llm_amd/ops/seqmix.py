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


def offset_rmsnorm(x, w, eps, out_dtype, offset=1.0, groups=1):
    """x / rms(x) * (offset + w) -> (fp32, out_dtype) rows; ``groups`` > 1:
    the root mean square of each of that many equal parts of the row."""
    if x.is_cuda:
        return _ext("offset_rmsnorm").offset_rmsnorm(
            x if x.stride(-1) == 1 else x.contiguous(), w, eps,
            _bf16(out_dtype), offset, groups)
    return R.offset_rmsnorm(x, w, eps, out_dtype, offset, groups)


def causal_tap_conv(h, w, tails, cu, tok_seq, slots, out_dtype):
    if h.is_cuda:
        return _ext("causal_tap_conv").causal_tap_conv(
            h, w, tails, cu, tok_seq, slots, _bf16(out_dtype))
    return R.causal_tap_conv(h, w, tails, cu, slots, out_dtype)


def latent_prepare(q, dkv, heads, dim, rot_dim, kv_rank, norm_w, eps,
                   positions, rope_base, rope_dims, page_slot, cache,
                   freqs=None, mag=1.0, pairs=False):
    """``q`` and ``dkv`` may be column slices of wider row-major matrices;
    ``dkv`` None: the layer reads another layer's cache. ``freqs`` (fp32
    [rope_dims / 2]) with ``mag`` and ``pairs`` selects a tabulated rotation
    (rescaled frequencies, cos/sin factor, (2i, 2i+1) pairs)."""
    if q.is_cuda:
        return _ext("latent_prepare").latent_prepare(
            q, dkv, heads, dim, rot_dim, kv_rank, norm_w, eps, positions,
            rope_base, rope_dims, page_slot, cache, freqs, mag, pairs)
    return R.latent_prepare(q, dkv, heads, dim, rot_dim, kv_rank, norm_w, eps,
                            positions, rope_base, rope_dims, page_slot, cache,
                            freqs, mag, pairs)


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
                            out_dtype, tiles=None, max_tile=0, sink=None,
                            gate=None):
    """``tiles`` (int32 [n, 3] from :func:`query_tiles`, with ``max_tile``)
    selects the tiled MFMA kernel for bf16; without it, or in fp32, the
    one-wave-per-query kernel runs. ``sink`` (fp32 [H]) joins the softmax
    denominator; ``gate`` ([T, H] pre-activations, may be a column slice)
    scales head h's result by its sigmoid."""
    if q_lat.is_cuda:
        return _ext("latent_window_attention").latent_window_attention(
            q_lat.contiguous(), q_rot, cache, kv_rank, block_tables,
            block_size, tok_seq, positions, window, scale, tiles, max_tile,
            sink, gate)
    return R.latent_window_attention(q_lat, q_rot, cache, kv_rank, block_tables,
                                     block_size, cu, positions, window, scale,
                                     out_dtype, sink, gate)


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

def sandwich_residual_norm(x, y, y2, post_w, next_w, eps, out_dtype,
                           offset=1.0, y_scale=1.0, y2_scale=1.0,
                           cast_next=False, groups=1):
    """Fused sublayer tail: x += rms_unit(y_scale y [+ y2_scale y2]) *
    (offset + post_w) on the fp32 residual (in place; ``post_w`` None: the
    sum is added without a closing norm), then, with ``next_w``, the next
    offset RMS norm of the new residual (over ``groups`` equal parts) in
    ``out_dtype``; with ``cast_next`` instead the new residual itself in
    ``out_dtype`` (x when that is fp32); None without either."""
    if x.is_cuda:
        h = _ext("sandwich_residual_norm").sandwich_residual_norm(
            x, y.contiguous(), None if y2 is None else y2.contiguous(), post_w,
            next_w, eps, _bf16(out_dtype), offset, y_scale, y2_scale,
            cast_next and next_w is None and _bf16(out_dtype), groups)
        if h is None and cast_next and next_w is None:
            return x
        return h
    return R.sandwich_residual_norm(x, y, y2, post_w, next_w, eps, out_dtype,
                                    offset, y_scale, y2_scale, cast_next, groups)


def residual_add_norm(x, y, next_w, eps, out_dtype, offset=1.0, groups=1):
    """Pre-norm sublayer tail: x += y on the fp32 residual (in place), then,
    with ``next_w``, the next norm of the new residual in ``out_dtype``."""
    return sandwich_residual_norm(x, y, None, None, next_w, eps, out_dtype,
                                  offset, groups=groups)


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
                     ab_w=None, decay_up=None, gate_sigmoid=False):
    """``ab`` None: the [strength | decay input] rows are projected inside
    the op from the mixer input ``h`` with the fp32 matrix ``ab_w``.
    ``decay_up`` (fp32 [H dim, R]): a decay per head and key channel from the
    R low-rank decay inputs, ``dt_bias`` [H dim]; else one decay per head.
    ``gate_sigmoid``: sigmoid output gate instead of SiLU."""
    if qkv.is_cuda:
        return _ext("gated_delta_rule").gated_delta_rule(
            qkv, gate, ab, h, ab_w, a_log, dt_bias, onorm_w, eps, state, cu,
            slots, heads, kv_heads, dim, vdim, decay_up, gate_sigmoid)
    if ab is None:
        ab = torch.nn.functional.linear(h.float(), ab_w.float())
    return R.gated_delta_rule(qkv, gate, ab, a_log, dt_bias, onorm_w, eps,
                              state, cu, slots, heads, kv_heads, dim, vdim,
                              out_dtype, decay_up, gate_sigmoid)


def capped_glu(gu, limit):
    if gu.is_cuda:
        return _ext("capped_glu").capped_glu(gu, limit)
    return R.capped_glu(gu, limit)


def silu_glu(gu):
    """Rows [gate | up] -> silu(gate) * up."""
    if gu.is_cuda:
        return _ext("silu_glu").silu_glu(gu)
    return R.silu_glu(gu)


def qk_norm_kv_write(proj, heads, kv_heads, dim, vdim, q_norm_w, k_norm_w, eps,
                     page_slot, cache):
    """``proj`` rows [q | k | v] may be a column slice of a wider matrix."""
    if proj.is_cuda:
        return _ext("qk_norm_kv_write").qk_norm_kv_write(
            proj, heads, kv_heads, dim, vdim, q_norm_w, k_norm_w, eps,
            page_slot, cache)
    return R.qk_norm_kv_write(proj, heads, kv_heads, dim, vdim, q_norm_w,
                              k_norm_w, eps, page_slot, cache)


def sigmoid_attention(q, cache, heads, kv_heads, dim, vdim, block_tables,
                      block_size, cu, tok_seq, positions, scale, window,
                      keep_first, slopes, pos_bias, out_dtype, tiles=None,
                      max_tile=0):
    """``tiles`` (from :func:`query_tiles` with ``WIDE_QUERY_TILE``) selects
    the tiled MFMA kernel for bf16 prompt portions; other steps and fp32
    models run one wave per (token, head)."""
    if q.is_cuda:
        return _ext("sigmoid_attention").sigmoid_attention(
            q, cache, heads, kv_heads, dim, vdim, block_tables, block_size,
            tok_seq, positions, scale, window, keep_first, slopes, pos_bias,
            tiles, max_tile)
    return R.sigmoid_attention(q, cache, heads, kv_heads, dim, vdim,
                               block_tables, block_size, cu, positions, scale,
                               window, keep_first, slopes, pos_bias, out_dtype)


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


# ------------------------------------------- windowed softmax attention, MLP

def qk_prepare_kv_write(proj, heads, kv_heads, dim, vdim, q_norm_w, k_norm_w,
                        eps, positions, freqs, mag, mix, page_slot, cache):
    """``proj`` rows [q | k | v | ...] may be a column slice of a wider
    matrix. ``q_norm_w``/``k_norm_w`` None: no q/k norm; ``freqs`` None: no
    rotation; ``mix`` (fp32 [H, H]): the returned queries are folded with
    the score-mixing matrix and span every kv head's key columns."""
    if proj.is_cuda:
        return _ext("qk_prepare_kv_write").qk_prepare_kv_write(
            proj, heads, kv_heads, dim, vdim, q_norm_w, k_norm_w, eps,
            positions, freqs, mag, mix, page_slot, cache)
    return R.qk_prepare_kv_write(proj, heads, kv_heads, dim, vdim, q_norm_w,
                                 k_norm_w, eps, positions, freqs, mag, mix,
                                 page_slot, cache)


def window_attention(q, cache, heads, kv_heads, dim, vdim, whole_key,
                     block_tables, block_size, cu, tok_seq, positions, scale,
                     window, keep_first, r1, r2, gate, out_dtype, tiles=None,
                     max_tile=0):
    """``tiles`` (from :func:`query_tiles` with ``WIDE_QUERY_TILE``) selects
    the tiled MFMA kernel for bf16 prompt portions; steps of few tokens per
    row run one workgroup per (token, kv head, share of the keys), fp32
    models and odd sizes one wave per (token, head). ``gate`` may be a
    column slice of a wider matrix."""
    if q.is_cuda:
        return _ext("window_attention").window_attention(
            q, cache, heads, kv_heads, dim, vdim, whole_key, block_tables,
            block_size, tok_seq, positions, scale, window, keep_first, r1, r2,
            gate, tiles, max_tile)
    return R.window_attention(q, cache, heads, kv_heads, dim, vdim, whole_key,
                              block_tables, block_size, cu, positions, scale,
                              window, keep_first, r1, r2, gate, out_dtype)


def gelu_tanh(x):
    if x.is_cuda:
        return _ext("gelu_tanh").gelu_tanh(x)
    return R.gelu_tanh(x)


def moe_route_sigmoid(h, router_w, top):
    if h.is_cuda:
        return _ext("moe_route_sigmoid").moe_route_sigmoid(h, router_w, top)
    return R.moe_route_sigmoid(h, router_w, top)


def moe_experts_scaled_input(h, idx, wts, exp_gu, exp_down):
    """SiLU-gated experts whose routing weight multiplies their input."""
    if h.is_cuda:
        return _ext("moe_experts_scaled_input").moe_experts_scaled_input(
            h, idx, wts, exp_gu, exp_down)
    return R.moe_experts_scaled_input(h, idx, wts, exp_gu, exp_down)
