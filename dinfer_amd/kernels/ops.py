"""Typed Python wrappers around the HIP kernels.

Each wrapper checks on the host what the kernel assumes about its operands
(device, dtype, strides, sizes) and launches on torch's current HIP stream, so
the calls can be captured into a HIP graph like any other stream work.
"""
from __future__ import annotations

import ctypes

import numpy as np
import torch

from . import lib

F32, BF16 = 0, 1


def dtype_code(dt: torch.dtype) -> int:
    if dt == torch.float32:
        return F32
    if dt == torch.bfloat16:
        return BF16
    raise TypeError(f"kernels take float32 or bfloat16 storage, not {dt}")


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    """The current HIP stream of the current device (also under graph capture, which switches it)."""
    if _raw_stream is not None:  # the handle alone: a tenth of the cost of building a Stream object per launch
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _need_gpu(*tensors) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise lib.KernelError("kernel operands must live on the GPU; there is no CPU path")


def _ptr(t) -> int:
    return 0 if t is None else t.data_ptr()


def _rows(t: torch.Tensor) -> int:
    """Row stride of a 2-D tensor whose rows are contiguous."""
    if t.dim() != 2 or t.stride(1) != 1:
        raise ValueError(f"expected a 2-D tensor with contiguous rows, got shape {tuple(t.shape)} stride {t.stride()}")
    return t.stride(0)


def _is_param_f32(w: torch.Tensor, act_dtype: torch.dtype) -> int:
    if w.dtype == torch.float32:
        return 1
    if w.dtype != act_dtype:
        raise TypeError(f"a parameter vector must be float32 or the activation dtype {act_dtype}, not {w.dtype}")
    return 0


def embedding(ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor, src: torch.Tensor | None = None,
              last: torch.Tensor | None = None) -> torch.Tensor:
    """out[t] = table[ids[t]]; ids int32 [T], table [V, W], out [T, W]. src, last (int32, both or neither): where
    src[t] >= 0 the id is last[src[t]], a token the step before sampled, which only the device knows so far."""
    _need_gpu(ids, table, out, src, last)
    assert ids.dtype == torch.int32 and ids.is_contiguous()
    assert (src is None) == (last is None)
    if src is not None:
        assert src.dtype == last.dtype == torch.int32 and src.numel() >= ids.numel()
    assert table.is_contiguous() and out.is_contiguous() and table.dtype == out.dtype
    T = ids.numel()
    V, W = table.shape
    assert out.shape[0] >= T and out.shape[1] == W
    lib.call("dinfer_embedding", dtype_code(table.dtype), ids.data_ptr(), table.data_ptr(), out.data_ptr(), T, V, W,
             _ptr(src), _ptr(last), _stream())
    return out


GATED_ACTS = {"silu": 0}   # activations the gated kernels know -> their code in the C interface
MAX_HEAD_DIM = 512         # the largest head the norm / rotation / plain attention kernels hold in registers


def gated_act(gate_up: torch.Tensor, out: torch.Tensor, tokens: int, act: str = "silu") -> torch.Tensor:
    """out[t, i] = act(gate_up[t, i]) * gate_up[t, I + i]."""
    _need_gpu(gate_up, out)
    if act not in GATED_ACTS:
        raise lib.KernelError(f"gated activation {act!r} has no kernel (known: {sorted(GATED_ACTS)})")
    inter = out.shape[1]
    assert gate_up.shape[1] == 2 * inter and gate_up.dtype == out.dtype and out.is_contiguous()
    assert gate_up.shape[0] >= tokens and out.shape[0] >= tokens
    lib.call("dinfer_gated_act", dtype_code(out.dtype), GATED_ACTS[act], gate_up.data_ptr(), out.data_ptr(), tokens, inter,
             _rows(gate_up), _stream())
    return out


def add_inplace(dst: torch.Tensor, src: torch.Tensor, n: int | None = None) -> None:
    """dst[:n] += src[:n] (flat), summed in float and rounded once."""
    _need_gpu(dst, src)
    assert dst.dtype == src.dtype and dst.is_contiguous() and src.is_contiguous()
    n = dst.numel() if n is None else n
    assert n <= dst.numel() and n <= src.numel()
    lib.call("dinfer_add_inplace", dtype_code(dst.dtype), dst.data_ptr(), src.data_ptr(), n, _stream())


def scale_softcap(x: torch.Tensor, rows: int, scale: float = 1.0, cap: float | None = None) -> None:
    """In place on the first `rows` rows of x: x *= scale, then x = cap * tanh(x / cap) where a cap is given."""
    _need_gpu(x)
    assert x.shape[0] >= rows
    lib.call("dinfer_scale_softcap", dtype_code(x.dtype), x.data_ptr(), _rows(x), rows, x.shape[1], float(scale),
             float(cap) if cap else 0.0, _stream())


def widen(src: torch.Tensor, dst: torch.Tensor, n: int | None = None) -> None:
    _need_gpu(src, dst)
    assert dst.dtype == torch.float32 and dst.is_contiguous() and src.is_contiguous()
    n = src.numel() if n is None else n
    lib.call("dinfer_widen", dtype_code(src.dtype), src.data_ptr(), dst.data_ptr(), n, _stream())


def fill_zero(t: torch.Tensor) -> None:
    """Zero-fills a tensor with a kernel (safe inside a captured graph)."""
    _need_gpu(t)
    nbytes = t.numel() * t.element_size()
    assert t.is_contiguous() and nbytes % 4 == 0 and t.data_ptr() % 4 == 0
    lib.call("dinfer_fill_u32", t.data_ptr(), 0, nbytes // 4, _stream())


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, out: torch.Tensor, eps: float, n_rows: int, *,
            residual: torch.Tensor | None = None, rows: torch.Tensor | None = None,
            weight_offset: float = 0.0) -> torch.Tensor:
    """out[r] = rmsnorm(x[src(r)]) * (weight + weight_offset).

    residual: updated in place to round(x + residual) first, and that sum is normed.
    rows: int32 indices of the n_rows source rows (gather); default identity.
    """
    _need_gpu(x, weight, out, residual, rows)
    width = out.shape[1]
    assert x.shape[1] == width and weight.numel() == width and weight.is_contiguous() and out.is_contiguous()
    assert x.dtype == out.dtype and out.shape[0] >= n_rows
    if rows is None:
        assert x.shape[0] >= n_rows
    else:
        assert rows.dtype == torch.int32 and rows.is_contiguous() and rows.numel() >= n_rows
    if residual is not None:
        assert residual.dtype == x.dtype and residual.shape == x.shape
    lib.call("dinfer_rmsnorm", dtype_code(x.dtype), x.data_ptr(), _ptr(residual), _ptr(rows), weight.data_ptr(),
             _is_param_f32(weight, x.dtype), out.data_ptr(), n_rows, width, _rows(x),
             _rows(residual) if residual is not None else 0, float(eps), float(weight_offset), _stream())
    return out


# ---- cache page layouts ------------------------------------------------------------------------
# K pages [blocks, kv_heads, D / 8, page, 8]: the 8-element pieces of consecutive keys are contiguous,
# so the rows of an MFMA operand (consecutive keys, one piece) are read as contiguous memory.
# V pages [blocks, kv_heads, D, page]: transposed, a row holds one dimension of a page's keys.
def k_cache_shape(blocks: int, kv_heads: int, page_size: int, head_dim: int) -> tuple:
    if head_dim % 8 != 0:
        raise ValueError(f"head_dim {head_dim}: the cache stores keys in pieces of 8 elements")
    return (blocks, kv_heads, head_dim // 8, page_size, 8)


def v_cache_shape(blocks: int, kv_heads: int, page_size: int, head_dim: int) -> tuple:
    return (blocks, kv_heads, head_dim, page_size)


def k_cache_pack(rows: torch.Tensor) -> torch.Tensor:
    """[blocks, kv_heads, page, D] (one row per key) -> the layout of K pages."""
    nb, hkv, page, d = rows.shape
    return rows.view(nb, hkv, page, d // 8, 8).permute(0, 1, 3, 2, 4).contiguous()


def k_cache_rows(pages: torch.Tensor) -> torch.Tensor:
    """The layout of K pages -> [blocks, kv_heads, page, D] (one row per key)."""
    nb, hkv, pieces, page, _ = pages.shape
    return pages.permute(0, 1, 3, 2, 4).reshape(nb, hkv, page, pieces * 8)


def _check_pages(k_cache, v_cache, kv_heads, head_dim, page_size) -> None:
    nb = k_cache.shape[0]
    assert tuple(k_cache.shape) == k_cache_shape(nb, kv_heads, page_size, head_dim) and k_cache.is_contiguous()
    assert tuple(v_cache.shape) == v_cache_shape(nb, kv_heads, page_size, head_dim) and v_cache.is_contiguous()


def qkv_post(qkv: torch.Tensor, tokens: int, *, heads: int, kv_heads: int, head_dim: int, q_off: int, k_off: int,
             v_off: int, q_gain: torch.Tensor | None, k_gain: torch.Tensor | None, eps: float, gain_offset: float,
             positions: torch.Tensor, cos_sin: torch.Tensor | None, rotary_dim: int, rope_style: int,
             k_cache: torch.Tensor | None, v_cache: torch.Tensor | None, slot_mapping: torch.Tensor | None,
             page_size: int, token_runs: bool = True) -> None:
    """Per-head q/k norm, rotation, q written back in place, k and v written to the cache pages.

    k_cache and v_cache in the page layouts above; slot_mapping int64 [T] (None: nothing is written
    to the cache and k is written back in place, as q is). token_runs: the tokens come in runs of consecutive positions (prompt portions, not
    single decoded tokens); it only chooses the faster of two ways of writing V.
    """
    _need_gpu(qkv, q_gain, k_gain, positions, cos_sin, k_cache, v_cache, slot_mapping)
    ld = _rows(qkv)
    assert qkv.shape[0] >= tokens
    assert max(q_off + heads * head_dim, k_off + kv_heads * head_dim, v_off + kv_heads * head_dim) <= qkv.shape[1]
    assert positions.dtype == torch.int32 and positions.numel() >= tokens
    wf32 = 0
    if q_gain is not None:
        assert q_gain.numel() == head_dim and k_gain is not None and k_gain.numel() == head_dim
        wf32 = _is_param_f32(q_gain, qkv.dtype)
        assert _is_param_f32(k_gain, qkv.dtype) == wf32
    if cos_sin is not None:
        assert cos_sin.dtype == torch.float32 and cos_sin.is_contiguous() and cos_sin.shape[1] == rotary_dim
    if slot_mapping is not None:
        assert slot_mapping.dtype == torch.int64 and slot_mapping.numel() >= tokens
        assert k_cache is not None and v_cache is not None
        _check_pages(k_cache, v_cache, kv_heads, head_dim, page_size)
        assert k_cache.dtype == qkv.dtype and v_cache.dtype == qkv.dtype
    lib.call("dinfer_qkv_post", dtype_code(qkv.dtype), qkv.data_ptr(), tokens, ld, q_off, k_off, v_off,
             _ptr(q_gain), _ptr(k_gain), wf32, float(eps), float(gain_offset), positions.data_ptr(), _ptr(cos_sin),
             rotary_dim, rope_style, _ptr(k_cache), _ptr(v_cache), _ptr(slot_mapping), heads, kv_heads, head_dim,
             page_size, int(token_runs), _stream())


def attn_paged_ref(q: torch.Tensor, out: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                   block_table: torch.Tensor, cu_seqlens: torch.Tensor, seq_lens: torch.Tensor, num_reqs: int,
                   tokens: int, *, scale: float, window: int, heads: int, kv_heads: int, head_dim: int,
                   page_size: int) -> torch.Tensor:
    """Plain paged attention (any head size); q is a view whose row t holds the heads at columns h*D."""
    _need_gpu(q, out, k_cache, v_cache, block_table, cu_seqlens, seq_lens)
    assert q.dtype == out.dtype == k_cache.dtype == v_cache.dtype
    assert block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous()
    assert block_table.shape[0] >= num_reqs
    assert cu_seqlens.dtype == torch.int32 and cu_seqlens.numel() >= num_reqs + 1
    assert seq_lens.dtype == torch.int32 and seq_lens.numel() >= num_reqs
    _check_pages(k_cache, v_cache, kv_heads, head_dim, page_size)
    assert q.shape[1] >= heads * head_dim and out.shape[1] >= heads * head_dim
    assert q.shape[0] >= tokens and out.shape[0] >= tokens
    lib.call("dinfer_attn_paged_ref", dtype_code(q.dtype), q.data_ptr(), _rows(q), out.data_ptr(), _rows(out),
             k_cache.data_ptr(), v_cache.data_ptr(), block_table.data_ptr(), block_table.shape[1],
             cu_seqlens.data_ptr(), seq_lens.data_ptr(), num_reqs, tokens, float(scale), int(window), heads,
             kv_heads, head_dim, page_size, _stream())
    return out


def attn_mfma_supports(head_dim: int, page_size: int, heads: int, kv_heads: int) -> bool:
    return bool(lib.get("dinfer_attn_mfma_supports")(head_dim, page_size, heads, kv_heads))


def _check_paged(q, out, k_cache, v_cache, block_table, seq_lens, num_reqs, heads, kv_heads, head_dim, page_size):
    assert q.dtype == out.dtype == k_cache.dtype == v_cache.dtype == torch.bfloat16
    assert block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous()
    assert block_table.shape[0] >= num_reqs and seq_lens.dtype == torch.int32 and seq_lens.numel() >= num_reqs
    _check_pages(k_cache, v_cache, kv_heads, head_dim, page_size)
    assert q.shape[1] >= heads * head_dim and out.shape[1] >= heads * head_dim


def attn_flash(q, out, k_cache, v_cache, block_table, cu_seqlens, seq_lens, num_reqs: int, tokens: int,
               max_q_len: int, *, scale: float, window: int, heads: int, kv_heads: int, head_dim: int,
               page_size: int, skip_single: bool = False):
    """MFMA flash attention over the pages: rows with or without history, causal, optional window."""
    _need_gpu(q, out, k_cache, v_cache, block_table, cu_seqlens, seq_lens)
    _check_paged(q, out, k_cache, v_cache, block_table, seq_lens, num_reqs, heads, kv_heads, head_dim, page_size)
    assert cu_seqlens.dtype == torch.int32 and cu_seqlens.numel() >= num_reqs + 1
    assert q.shape[0] >= tokens and out.shape[0] >= tokens
    lib.call("dinfer_attn_flash", q.data_ptr(), _rows(q), out.data_ptr(), _rows(out), k_cache.data_ptr(),
             v_cache.data_ptr(), block_table.data_ptr(), block_table.shape[1], cu_seqlens.data_ptr(),
             seq_lens.data_ptr(), num_reqs, max_q_len, float(scale), int(window), heads, kv_heads, head_dim,
             page_size, 1 if skip_single else 0, _stream())
    return out


def attn_decode(q, out, part, k_cache, v_cache, block_table, cu_seqlens, seq_lens, num_reqs: int, splits: int, *,
                scale: float, window: int, heads: int, kv_heads: int, head_dim: int, page_size: int):
    """Split-K attention for requests that bring one row. cu_seqlens None: row b is request b;
    given: only the requests with one row are served (mixed batches). Each request's keys are cut
    into `splits` equal parts on the device, so the launch shape does not depend on the lengths."""
    _need_gpu(q, out, part, k_cache, v_cache, block_table, cu_seqlens, seq_lens)
    _check_paged(q, out, k_cache, v_cache, block_table, seq_lens, num_reqs, heads, kv_heads, head_dim, page_size)
    assert part.dtype == torch.float32 and part.is_contiguous()
    lib.call("dinfer_attn_decode", q.data_ptr(), _rows(q), out.data_ptr(), _rows(out), part.data_ptr(),
             part.numel(), k_cache.data_ptr(), v_cache.data_ptr(), block_table.data_ptr(), block_table.shape[1],
             _ptr(cu_seqlens), seq_lens.data_ptr(), num_reqs, splits, float(scale), int(window), heads, kv_heads,
             head_dim, page_size, _stream())
    return out


def attn_decode_post_supports(head_dim: int) -> bool:
    return bool(lib.get("dinfer_attn_decode_post_supports")(head_dim))


def attn_decode_post(qkv, out, part, k_cache, v_cache, block_table, seq_lens, num_reqs: int, splits: int, *,
                     scale: float, window: int, heads: int, kv_heads: int, head_dim: int, page_size: int, q_off: int,
                     k_off: int, v_off: int, q_gain, k_gain, eps: float, gain_offset: float, positions, cos_sin,
                     slot_mapping):
    """attn_decode for a step in which every request brings one row, straight from the q|k|v product: the per-head
    norms, the rotation (pairs (i, i + head_dim/2), the whole head) and the write of the new key and value into their
    pages happen inside the attention kernel. qkv stays as the product left it. slot_mapping None: nothing is written."""
    _need_gpu(qkv, out, part, k_cache, v_cache, block_table, seq_lens, q_gain, k_gain, positions, cos_sin, slot_mapping)
    _check_paged(qkv, out, k_cache, v_cache, block_table, seq_lens, num_reqs, heads, kv_heads, head_dim, page_size)
    assert part.dtype == torch.float32 and part.is_contiguous() and qkv.shape[0] >= num_reqs
    assert max(q_off + heads * head_dim, k_off + kv_heads * head_dim, v_off + kv_heads * head_dim) <= qkv.shape[1]
    assert q_off % 8 == 0 and k_off % 8 == 0 and v_off % 8 == 0
    assert positions.dtype == torch.int32 and positions.numel() >= num_reqs
    if q_gain is not None:   # (gains kept in 32-bit go through qkv_post)
        assert k_gain is not None and q_gain.numel() == k_gain.numel() == head_dim
        assert q_gain.dtype == k_gain.dtype == torch.bfloat16
    if cos_sin is not None:
        assert cos_sin.dtype == torch.float32 and cos_sin.is_contiguous() and cos_sin.shape[1] == head_dim
    if slot_mapping is not None:
        assert slot_mapping.dtype == torch.int64 and slot_mapping.numel() >= num_reqs
    base, es = qkv.data_ptr(), qkv.element_size()
    lib.call("dinfer_attn_decode_post", base + q_off * es, base + k_off * es, base + v_off * es, _rows(qkv),
             out.data_ptr(), _rows(out), part.data_ptr(), part.numel(), k_cache.data_ptr(), v_cache.data_ptr(),
             block_table.data_ptr(), block_table.shape[1], seq_lens.data_ptr(), num_reqs, splits, float(scale),
             int(window), heads, kv_heads, head_dim, page_size, _ptr(q_gain), _ptr(k_gain), float(eps),
             float(gain_offset), positions.data_ptr(), _ptr(cos_sin), _ptr(slot_mapping), _stream())
    return out


def gemm_ref(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, m: int) -> torch.Tensor:
    """out[:m] = a[:m] @ w.T on the vector ALUs with float accumulation (true 32-bit for float operands)."""
    _need_gpu(a, w, out)
    n, k = w.shape
    assert a.shape[1] == k and out.shape[1] == n and a.dtype == w.dtype
    assert a.shape[0] >= m and out.shape[0] >= m
    out_f32 = 1 if out.dtype == torch.float32 else 0
    if not out_f32:
        assert out.dtype == a.dtype
    lib.call("dinfer_gemm_ref", dtype_code(a.dtype), out_f32, a.data_ptr(), _rows(a), w.data_ptr(), _rows(w),
             out.data_ptr(), _rows(out), m, n, k, _stream())
    return out


def gemm_small_m(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, m: int, *, row_tiles: int = 0,
                 waves: int = 0) -> torch.Tensor:
    """out[:m] = a[:m] @ w.T for m <= 64, bf16 operands, weight streamed once (MFMA, split-K in the workgroup)."""
    _need_gpu(a, w, out)
    n, k = w.shape
    assert a.dtype == w.dtype == torch.bfloat16 and a.shape[1] == k and out.shape[1] == n
    assert a.shape[0] >= m and out.shape[0] >= m and out.dtype in (torch.bfloat16, torch.float32)
    lib.call("dinfer_gemm_small_m", 1 if out.dtype == torch.float32 else 0, a.data_ptr(), _rows(a), w.data_ptr(),
             _rows(w), out.data_ptr(), _rows(out), m, n, k, row_tiles, waves, _stream())
    return out


def gemm_small_m_gated(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, m: int, *, waves: int = 0) -> torch.Tensor:
    """out[:m] = silu(a @ wg.T) * (a @ wu.T) for w = [wg; wu] stacked [2N, K], m <= 32, bf16: both
    projections of a gated feed-forward and the activation in one weight-streaming kernel."""
    _need_gpu(a, w, out)
    k = w.shape[1]
    n = w.shape[0] // 2
    assert w.shape[0] == 2 * n and a.dtype == w.dtype == out.dtype == torch.bfloat16
    assert a.shape[1] == k and out.shape[1] == n and a.shape[0] >= m and out.shape[0] >= m
    lib.call("dinfer_gemm_small_m_gated", a.data_ptr(), _rows(a), w.data_ptr(), _rows(w), out.data_ptr(), _rows(out),
             m, n, k, waves, _stream())
    return out


def gemm_small_m_sink(a: torch.Tensor, w: torch.Tensor, stream_: torch.Tensor, xg: torch.Tensor, gain: torch.Tensor,
                      stats: torch.Tensor, m: int, *, gain_offset: float = 0.0) -> int:
    """stream_[:m] += a[:m] @ w.T in place (the residual stream: summed in float, rounded once), and what the RMSNorm
    that reads it next needs: xg[:m] = stream_ * (gain + gain_offset), stats[r, j] = sum of squares of stream_[r] over
    columns g j .. g j + g - 1, g being 16 or 8 as the kernel for these sizes has it. Returns how many of them a token
    has (ceil(n / g)). m <= 32, bf16."""
    _need_gpu(a, w, stream_, xg, gain, stats)
    n, k = w.shape
    assert a.dtype == w.dtype == stream_.dtype == xg.dtype == torch.bfloat16 and stats.dtype == torch.float32
    assert a.shape[1] == k and stream_.shape[1] == n and xg.shape[1] == n and gain.numel() == n and gain.is_contiguous()
    cols = -(-n // lib.get("dinfer_gemm_small_m_sink_stats_columns")(m, n, k))
    assert min(a.shape[0], stream_.shape[0], xg.shape[0], stats.shape[0]) >= m and stats.shape[1] >= cols
    lib.call("dinfer_gemm_small_m_sink", a.data_ptr(), _rows(a), w.data_ptr(), _rows(w), stream_.data_ptr(), _rows(stream_),
             xg.data_ptr(), _rows(xg), gain.data_ptr(), _is_param_f32(gain, torch.bfloat16), float(gain_offset),
             stats.data_ptr(), _rows(stats), m, n, k, _stream())
    return cols


def gemm_small_m_scaled(xg: torch.Tensor, w: torch.Tensor, out: torch.Tensor, m: int, stats: torch.Tensor, cols: int,
                        eps: float, width: int, *, gated: bool = False) -> torch.Tensor:
    """out[:m] = (xg[:m] @ w.T) * rsqrt(sum(stats[r, :cols]) / width + eps) per row r: with xg and stats from
    gemm_small_m_sink, the product of the RMS-normed stream with w. gated: w = [wg; wu] stacked and
    out = silu(scaled gate) * scaled up. m <= 32, bf16."""
    _need_gpu(xg, w, out, stats)
    k = w.shape[1]
    n = w.shape[0] // 2 if gated else w.shape[0]
    assert xg.dtype == w.dtype == out.dtype == torch.bfloat16 and stats.dtype == torch.float32
    assert xg.shape[1] == k and out.shape[1] == n and min(xg.shape[0], out.shape[0], stats.shape[0]) >= m
    assert 0 < cols <= stats.shape[1]
    lib.call("dinfer_gemm_small_m_scaled", xg.data_ptr(), _rows(xg), w.data_ptr(), _rows(w), out.data_ptr(), _rows(out),
             m, n, k, 1 if gated else 0, stats.data_ptr(), _rows(stats), cols, float(eps), width, _stream())
    return out


def gemm_mid_m_workspace(m: int, n: int, k: int, *, gated: bool = False, ks: int = 0, rt: int = 0) -> int:
    """Bytes of float workspace gemm_mid_m needs for these sizes (0: the product is stored directly)."""
    need = ctypes.c_int64(0)
    lib.call("dinfer_gemm_mid_m_workspace", m, n, k, 1 if gated else 0, ks, rt, ctypes.addressof(need))
    return need.value


def gemm_mid_m(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, m: int, workspace: torch.Tensor | None = None, *,
               gated: bool = False, ks: int = 0, rt: int = 0) -> torch.Tensor:
    """out[:m] = a[:m] @ w.T for m <= 64 (made for 17 to 64), bf16 operands; gated: w = [wg; wu] stacked
    [2N, K] and out = silu(a @ wg.T) * (a @ wu.T). A narrow weight is cut into slices of k whose float
    partial sums go through `workspace` and are added in slice order by a second kernel."""
    _need_gpu(a, w, out, workspace)
    k = w.shape[1]
    n = w.shape[0] // 2 if gated else w.shape[0]
    assert a.dtype == w.dtype == torch.bfloat16 and a.shape[1] == k and out.shape[1] == n
    assert a.shape[0] >= m and out.shape[0] >= m and out.dtype in (torch.bfloat16, torch.float32)
    assert workspace is None or workspace.is_contiguous()
    lib.call("dinfer_gemm_mid_m", 1 if out.dtype == torch.float32 else 0, a.data_ptr(), _rows(a), w.data_ptr(), _rows(w),
             out.data_ptr(), _rows(out), m, n, k, 1 if gated else 0, ks, rt, _ptr(workspace),
             workspace.numel() * workspace.element_size() if workspace is not None else 0, _stream())
    return out


GEMM_MID_SINK_MAX_N = 8192   # columns a workgroup of gemm_mid_m_sink's second kernel holds in registers


def gemm_mid_m_sink(a: torch.Tensor, w: torch.Tensor, stream_: torch.Tensor, out: torch.Tensor, gain: torch.Tensor,
                    gain_offset: float, eps: float, m: int, workspace: torch.Tensor, *, ks: int = 0, rt: int = 0) -> None:
    """stream_[:m] += a[:m] @ w.T in place (the float sum of the slices and the stream, rounded once) and out[:m] = the
    RMSNorm of the new rows (gain + gain_offset, eps): gemm_mid_m's product with a second kernel that is also the add
    and the norm. bf16, m <= 64, N <= GEMM_MID_SINK_MAX_N."""
    _need_gpu(a, w, stream_, out, gain, workspace)
    n, k = w.shape
    assert a.dtype == w.dtype == stream_.dtype == out.dtype == torch.bfloat16 and a.shape[1] == k
    assert stream_.shape[1] == n and out.shape[1] == n and gain.numel() == n and gain.is_contiguous()
    assert a.shape[0] >= m and stream_.shape[0] >= m and out.shape[0] >= m and workspace.is_contiguous()
    assert gain.dtype in (torch.bfloat16, torch.float32)
    lib.call("dinfer_gemm_mid_m_sink", a.data_ptr(), _rows(a), w.data_ptr(), _rows(w), stream_.data_ptr(), _rows(stream_),
             out.data_ptr(), _rows(out), gain.data_ptr(), 1 if gain.dtype == torch.float32 else 0, float(gain_offset),
             float(eps), m, n, k, ks, rt, workspace.data_ptr(), workspace.numel() * workspace.element_size(), _stream())


def gemm_wide_supports(m: int, n: int, k: int) -> bool:
    """Whether gemm_wide takes a product of m rows with a weight of n rows (gated: n of each half) and k columns."""
    return bool(lib.get("dinfer_gemm_wide_supports")(m, n, k))


def gemm_wide(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, m: int, *, gated: bool = False,
              stats: torch.Tensor | None = None, cols: int = 0, eps: float = 0.0, width: int = 0) -> torch.Tensor:
    """out[:m] = a[:m] @ w.T for m <= 64 and a weight of many rows (96 of them a workgroup), bf16 operands, out bf16 or
    float32; gated: w = [wg; wu] stacked [2N, K] and out = silu(a @ wg.T) * (a @ wu.T). stats [m, >= cols] float32:
    row r of the result is multiplied by rsqrt(sum(stats[r, :cols]) / width + eps) first (a norm carried by the
    product before this one). K a multiple of 512, N of 16."""
    _need_gpu(a, w, out, stats)
    k = w.shape[1]
    n = w.shape[0] // 2 if gated else w.shape[0]
    assert a.dtype == w.dtype == torch.bfloat16 and a.shape[1] == k and out.shape[1] == n
    assert a.shape[0] >= m and out.shape[0] >= m and out.dtype in (torch.bfloat16, torch.float32)
    if stats is not None:
        assert stats.dtype == torch.float32 and stats.shape[0] >= m and stats.shape[1] >= cols > 0 and width > 0
    lib.call("dinfer_gemm_wide", 1 if out.dtype == torch.float32 else 0, a.data_ptr(), _rows(a), w.data_ptr(), _rows(w),
             out.data_ptr(), _rows(out), m, n, k, 1 if gated else 0, _ptr(stats), _rows(stats) if stats is not None else 0,
             int(cols), float(eps), int(width), _stream())
    return out


def argmax_scratch(rows: int, vocab: int, device) -> torch.Tensor:
    """The scratch with which argmax spreads each of up to `rows` rows over many workgroups."""
    n = ctypes.c_int64(0)
    lib.call("dinfer_argmax_scratch_bytes", rows, vocab, ctypes.addressof(n))
    return torch.empty(n.value, dtype=torch.uint8, device=device)


def argmax(logits: torch.Tensor, out: torch.Tensor, rows: int, scratch: torch.Tensor | None = None) -> torch.Tensor:
    """out[r] = the index of the largest of logits[r] (the lowest such index). scratch (argmax_scratch): a long row
    is spread over many workgroups instead of taken by one."""
    _need_gpu(logits, out, scratch)
    assert logits.dtype == torch.float32 and out.dtype == torch.int32 and out.numel() >= rows
    assert scratch is None or (scratch.dtype == torch.uint8 and scratch.is_contiguous())
    lib.call("dinfer_argmax", logits.data_ptr(), _rows(logits), out.data_ptr(), rows, logits.shape[1], _ptr(scratch),
             0 if scratch is None else scratch.numel(), _stream())
    return out


def sample(logits: torch.Tensor, work: torch.Tensor | None, out: torch.Tensor, rows: int, *,
           temperature: torch.Tensor | None, top_k: torch.Tensor | None = None, top_p: torch.Tensor | None = None,
           min_p: torch.Tensor | None = None, seeds: torch.Tensor | None = None,
           offsets: torch.Tensor | None = None) -> torch.Tensor:
    """One token per row. temperature None: all rows greedy. seeds/offsets are int64 holding the uint64 bits."""
    _need_gpu(logits, work, out, temperature, top_k, top_p, min_p, seeds, offsets)
    vocab = logits.shape[1]
    assert logits.dtype == torch.float32 and out.dtype == torch.int32 and out.numel() >= rows
    if temperature is not None:
        assert temperature.dtype == torch.float32 and temperature.numel() >= rows
        assert work is not None and work.dtype == torch.float32 and work.is_contiguous()
        assert work.numel() >= rows * vocab
        assert seeds is not None and offsets is not None
        assert seeds.dtype == torch.int64 and offsets.dtype == torch.int64
        assert seeds.numel() >= rows and offsets.numel() >= rows
    for t, dt in ((top_k, torch.int32), (top_p, torch.float32), (min_p, torch.float32)):
        assert t is None or (t.dtype == dt and t.numel() >= rows)
    lib.call("dinfer_sample", logits.data_ptr(), _rows(logits), _ptr(work), _ptr(temperature), _ptr(top_k),
             _ptr(top_p), _ptr(min_p), _ptr(seeds), _ptr(offsets), out.data_ptr(), rows, vocab, _stream())
    return out


# One row of dinfer_sample_rows: what to do with a row of logits.
SAMPLE_ROW = np.dtype([("temperature", "<f4"), ("top_k", "<i4"), ("top_p", "<f4"), ("min_p", "<f4"),
                       ("seed", "<u8"), ("offset", "<u8")])


def sample_scratch_bytes(rows: int, vocab: int) -> int:
    n = ctypes.c_int64(0)
    lib.call("dinfer_sample_scratch_bytes", rows, vocab, ctypes.addressof(n))
    return n.value


def sample_rows(logits: torch.Tensor, work: torch.Tensor, scratch: torch.Tensor, packed: torch.Tensor,
                out: torch.Tensor, rows: int, any_filter: bool = True, force_generic: bool = False) -> torch.Tensor:
    """One token per row by the rule of `sample`, a row spread over many workgroups. packed: uint8 device
    tensor holding `rows` records of SAMPLE_ROW; work [rows, vocab] float32 and scratch (uint8,
    sample_scratch_bytes) are the kernels' own memory between their launches. any_filter=False promises
    that no row has top-k or top-p."""
    _need_gpu(logits, work, scratch, packed, out)
    vocab = logits.shape[1]
    assert logits.dtype == torch.float32 and out.dtype == torch.int32 and out.numel() >= rows
    assert work.dtype == torch.float32 and work.is_contiguous() and work.numel() >= rows * vocab
    assert packed.dtype == torch.uint8 and packed.is_contiguous() and packed.numel() >= rows * SAMPLE_ROW.itemsize
    assert scratch.dtype == torch.uint8 and scratch.is_contiguous()
    lib.call("dinfer_sample_rows", logits.data_ptr(), _rows(logits), work.data_ptr(), scratch.data_ptr(),
             scratch.numel(), packed.data_ptr(), out.data_ptr(), rows, vocab, int(any_filter), int(force_generic), _stream())
    return out


# One row of penalties_dense: which history slot a row of logits takes its penalties from (< 0: none).
PENALTY_ROW = np.dtype([("slot", "<i4"), ("repetition", "<f4"), ("frequency", "<f4"), ("presence", "<f4")])


def history_add(history: torch.Tensor, entries: torch.Tensor) -> None:
    """history [slots, vocab] int32; entries [n, 3] int32 = (slot, token, kind): kind 0 marks a token of the
    prompt, kind 1 counts one more occurrence among the outputs."""
    _need_gpu(history, entries)
    assert history.dtype == torch.int32 and history.is_contiguous() and history.dim() == 2
    assert entries.dtype == torch.int32 and entries.is_contiguous() and entries.dim() == 2 and entries.shape[1] == 3
    lib.call("dinfer_history_add", history.data_ptr(), history.shape[0], history.shape[1], entries.data_ptr(),
             entries.shape[0], _stream())


def penalties_dense(logits: torch.Tensor, rows: int, history: torch.Tensor, packed: torch.Tensor) -> None:
    """In place on logits: row r takes repetition / frequency / presence penalties from history[slot_r]
    (packed: uint8 device tensor of `rows` PENALTY_ROW records; slot < 0 leaves the row alone)."""
    _need_gpu(logits, history, packed)
    assert logits.dtype == torch.float32 and history.dtype == torch.int32 and history.is_contiguous()
    assert history.shape[1] == logits.shape[1]
    assert packed.dtype == torch.uint8 and packed.is_contiguous() and packed.numel() >= rows * PENALTY_ROW.itemsize
    lib.call("dinfer_penalties_dense", logits.data_ptr(), _rows(logits), history.data_ptr(), history.shape[0],
             packed.data_ptr(), rows, logits.shape[1], _stream())


MAX_TOP_LOGPROBS = 32


def logit_bias(logits: torch.Tensor, rows: int, entries: torch.Tensor, values: torch.Tensor) -> None:
    """In place: logits[row, token] += value for entries [n, 2] int32 = (row, token) and values [n] float32.
    A (row, token) pair occurs once."""
    _need_gpu(logits, entries, values)
    assert logits.dtype == torch.float32 and entries.dtype == torch.int32 and values.dtype == torch.float32
    assert entries.is_contiguous() and entries.dim() == 2 and entries.shape[1] == 2
    assert values.is_contiguous() and values.numel() == entries.shape[0] and logits.shape[0] >= rows
    lib.call("dinfer_logit_bias", logits.data_ptr(), _rows(logits), entries.data_ptr(), values.data_ptr(),
             entries.shape[0], rows, logits.shape[1], _stream())


def logprobs(logits: torch.Tensor, chosen: torch.Tensor, top: torch.Tensor, out_ids: torch.Tensor,
             out_lp: torch.Tensor, rank: torch.Tensor, rows: int) -> None:
    """Per row r with top[r] >= 0, from the log-softmax of logits[r]: out_ids[r, 0], out_lp[r, 0] = chosen[r] and its
    log-probability; columns 1..top[r] the most probable tokens, falling (equal values: lower index first);
    rank[r] = how many tokens have a larger logit than the chosen one. out_ids / out_lp are [>= rows, stride] with
    stride <= MAX_TOP_LOGPROBS + 1; top[r] is cut to stride - 1."""
    _need_gpu(logits, chosen, top, out_ids, out_lp, rank)
    assert logits.dtype == torch.float32 and out_lp.dtype == torch.float32
    assert chosen.dtype == top.dtype == out_ids.dtype == rank.dtype == torch.int32
    assert out_ids.is_contiguous() and out_lp.is_contiguous() and out_ids.shape == out_lp.shape and out_ids.dim() == 2
    assert min(logits.shape[0], chosen.numel(), top.numel(), rank.numel(), out_ids.shape[0]) >= rows
    lib.call("dinfer_logprobs", logits.data_ptr(), _rows(logits), chosen.data_ptr(), top.data_ptr(),
             out_ids.shape[1], out_ids.data_ptr(), out_lp.data_ptr(), rank.data_ptr(), rows, logits.shape[1],
             _stream())


# ---- measured ceilings ---------------------------------------------------------------------------
def measured_hbm_read(device, nbytes: int = 4 << 30, repeats: int = 3) -> float:
    """Bytes per second a kernel that only reads reaches on `nbytes` of device memory (far beyond the caches):
    the best of `repeats` runs."""
    buf = torch.empty(nbytes // 4, dtype=torch.float32, device=device)
    buf.zero_()
    blocks = 256
    out = torch.empty(blocks * 8, dtype=torch.float32, device=device)
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    best = float("inf")
    for _ in range(repeats + 1):      # the first run loads the kernel
        start.record()
        lib.call("dinfer_stream_read", buf.data_ptr(), buf.numel() * 4, blocks, out.data_ptr(), _stream())
        end.record()
        end.synchronize()
        best = min(best, start.elapsed_time(end) * 1e-3)
    del buf
    return nbytes / best


def measured_mfma_bf16(device, repeats: int = 3) -> float:
    """Flops per second of chains of independent bf16 MFMAs on registers, every SIMD busy: the best of `repeats` runs."""
    blocks, iters = 256 * 8, 2048
    out = torch.empty(blocks * 256, dtype=torch.float32, device=device)
    flops = ctypes.c_int64(0)
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    best = float("inf")
    for _ in range(repeats + 1):
        start.record()
        lib.call("dinfer_mfma_loop", iters, blocks, out.data_ptr(), ctypes.addressof(flops), _stream())
        end.record()
        end.synchronize()
        best = min(best, start.elapsed_time(end) * 1e-3)
    return flops.value / best
