"""Tensor-level wrappers over the C ABI (one function per entry point).

Each wrapper checks what the kernels assume (device, dtype, contiguity of the
innermost dimension), allocates outputs / workspaces through torch's caching
allocator (so calls are graph-capturable), and launches on torch's current
stream.  bf16 only: the operator path has no other precision.
"""
from __future__ import annotations

import torch

from . import _hip

BF16 = torch.bfloat16
KV_PAGE = 256


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _gpu_bf16(*tensors):
    for t in tensors:
        if not (t.is_cuda and t.dtype == BF16):
            raise TypeError(f"expected a bf16 GPU tensor, got {t.dtype} on {t.device}")


def _p(t):
    return 0 if t is None else t.data_ptr()


# ---------------------------------------------------------------- norms
def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor | None = None) -> torch.Tensor:
    """x [..., dim] -> normalised copy (a strided view, e.g. q inside the fused qkv buffer, is
    compacted first; the model's own forward uses the fused qknorm_rope_store_ instead)."""
    _gpu_bf16(x, weight)
    dim = x.shape[-1]
    if not x.is_contiguous():
        x = x.contiguous()
    if out is None:
        out = torch.empty_like(x)
    rows = x.numel() // dim
    _hip.call("nvh_rmsnorm", x.data_ptr(), dim, weight.data_ptr(), out.data_ptr(), dim, rows, dim, float(eps), _stream())
    return out


def add_rmsnorm(x: torch.Tensor | None, residual: torch.Tensor, weight: torch.Tensor, eps: float,
                partials: torch.Tensor | None = None) -> tuple[torch.Tensor, torch.Tensor]:
    """(y, residual): residual is updated IN PLACE to bf16(x + residual).  With ``partials``
    (fp32 [S, rows, dim] split-K slabs) x is bf16(sum of slabs)."""
    _gpu_bf16(residual, weight)
    dim = residual.shape[-1]
    rows = residual.numel() // dim
    assert residual.is_contiguous()
    y = torch.empty_like(residual)
    if partials is not None:
        assert partials.dtype == torch.float32 and partials.is_contiguous() and partials.shape[-2:] == (rows, dim)
        _hip.call("nvh_add_rmsnorm", 0, residual.data_ptr(), weight.data_ptr(), y.data_ptr(), rows, dim, float(eps),
                  partials.data_ptr(), partials.shape[0], _stream())
    else:
        _gpu_bf16(x)
        if not x.is_contiguous():
            x = x.contiguous()
        _hip.call("nvh_add_rmsnorm", x.data_ptr(), residual.data_ptr(), weight.data_ptr(), y.data_ptr(), rows, dim,
                  float(eps), 0, 0, _stream())
    return y, residual


# ---------------------------------------------------------------- rotary / fused qkv epilogue
def rope_(positions: torch.Tensor, q: torch.Tensor, k: torch.Tensor, cos_sin: torch.Tensor) -> None:
    """In-place rotation of q [T,Hq,D] and k [T,Hkv,D] (views with head stride D allowed)."""
    _gpu_bf16(q, k)
    assert positions.dtype == torch.int64 and cos_sin.dtype == torch.float32 and cos_sin.is_contiguous()
    t, hq, d = q.shape
    hkv = k.shape[1]
    assert q.stride(2) == 1 and q.stride(1) == d and k.stride(2) == 1 and k.stride(1) == d
    _hip.call("nvh_rope", positions.data_ptr(), q.data_ptr(), q.stride(0), hq, k.data_ptr(), k.stride(0), hkv,
              cos_sin.data_ptr(), cos_sin.shape[0], t, d, _stream())


def qknorm_rope_store_(qkv: torch.Tensor, num_q_heads: int, num_kv_heads: int, q_weight, k_weight, eps: float,
                       positions, cos_sin, k_cache, v_cache, slot_mapping) -> None:
    """Fused per-head RMSNorm + RoPE on the q/k parts of qkv [T, (Hq+2Hkv)*128] in place,
    and K/V scatter into the caches (skipped when the caches are None)."""
    _gpu_bf16(qkv, q_weight, k_weight)
    assert qkv.stride(1) == 1 and positions.dtype == torch.int64
    store = k_cache is not None and k_cache.numel() > 0 and slot_mapping is not None and slot_mapping.numel() > 0
    _hip.call("nvh_qknorm_rope_store", qkv.data_ptr(), qkv.stride(0), num_q_heads, num_kv_heads, q_weight.data_ptr(),
              k_weight.data_ptr(), float(eps), positions.data_ptr(), cos_sin.data_ptr(), cos_sin.shape[0],
              k_cache.data_ptr() if store else 0, v_cache.data_ptr() if store else 0,
              slot_mapping.data_ptr() if store else 0, qkv.shape[0], _stream())


def linear_qkv_rope_store(x, w, num_q_heads: int, num_kv_heads: int, q_weight, k_weight, eps: float, positions, cos_sin,
                          k_cache=None, v_cache=None, slot_mapping=None, raw_rows: int = 0) -> torch.Tensor:
    """qkv [T, (Hq+2Hkv)*128] = x w^T with the q/k epilogue and KV store of rows raw_rows.. applied (in the GEMM's
    epilogue where the shape allows, as two launches otherwise; same bits)."""
    _gpu_bf16(x, w, q_weight, k_weight)
    t, k = x.shape
    n = (num_q_heads + 2 * num_kv_heads) * 128
    assert w.shape == (n, k) and w.is_contiguous() and x.stride(1) == 1 and positions.dtype == torch.int64
    store = k_cache is not None and k_cache.numel() > 0 and slot_mapping is not None and slot_mapping.numel() > 0
    qkv = torch.empty(t, n, dtype=BF16, device=x.device)
    _hip.call("nvh_gemm_qkv_rope_store", x.data_ptr(), x.stride(0), w.data_ptr(), qkv.data_ptr(), n, t, k, num_q_heads,
              num_kv_heads, 128, q_weight.data_ptr(), k_weight.data_ptr(), float(eps), positions.data_ptr(), cos_sin.data_ptr(),
              cos_sin.shape[0], k_cache.data_ptr() if store else 0, v_cache.data_ptr() if store else 0,
              slot_mapping.data_ptr() if store else 0, raw_rows, _stream())
    return qkv


# ---------------------------------------------------------------- RMSNorm as a row scale (prefill-sized steps)
def residual_rowsq_parts(m: int, n: int, k: int) -> int:
    """Partial sums of squares per row that `linear_add_residual_` leaves for this shape; 0: shape not supported."""
    return int(_hip.lib().nvh_gemm_residual_rowsq_parts(m, n, k))


def fold_norm_weight(weight: torch.Tensor, norm_weight: torch.Tensor) -> torch.Tensor:
    """w[n][k] * norm[k] rounded to bf16: the projection weight the row-scaled entry points take."""
    return (weight.float() * norm_weight.float()[None, :]).to(weight.dtype)


def linear_add_residual_(x: torch.Tensor, weight: torch.Tensor, residual: torch.Tensor) -> torch.Tensor:
    """residual += x weight^T in place (product rounded to bf16, sum in fp32, rounded to bf16); returns the fp32 partial
    sums of squares of the un-rounded sums, [M, parts]."""
    _gpu_bf16(x, weight, residual)
    m, k = x.shape
    n = weight.shape[0]
    parts = residual_rowsq_parts(m, n, k)
    assert parts > 0 and residual.shape == (m, n) and residual.is_contiguous() and weight.is_contiguous() and x.stride(1) == 1
    rowsq = torch.empty(m, parts, dtype=torch.float32, device=x.device)
    _hip.call("nvh_gemm_residual_rowsq_bf16_nt", x.data_ptr(), x.stride(0), weight.data_ptr(), residual.data_ptr(), rowsq.data_ptr(),
              m, n, k, _stream())
    return rowsq


def linear_swiglu_rowscaled(x: torch.Tensor, weight_folded_interleaved: torch.Tensor, rowsq: torch.Tensor, eps: float) -> torch.Tensor:
    """silu(g) * u of (x w^T) * 1/sqrt(sum(rowsq[m]) / K + eps): RMSNorm + gate/up projection + SwiGLU over the
    un-normalised rows, the norm weight folded into `weight_folded_interleaved`."""
    _gpu_bf16(x, weight_folded_interleaved)
    m, k = x.shape
    n = weight_folded_interleaved.shape[0]
    assert rowsq.dtype == torch.float32 and rowsq.shape[0] == m and rowsq.is_contiguous() and x.stride(1) == 1
    y = torch.empty(m, n // 2, dtype=BF16, device=x.device)
    _hip.call("nvh_gemm_swiglu_rowscaled_bf16_nt", x.data_ptr(), x.stride(0), weight_folded_interleaved.data_ptr(), y.data_ptr(), n // 2,
              m, n, k, rowsq.data_ptr(), rowsq.shape[1], float(eps), _stream())
    return y


def linear_qkv_rope_store_rowscaled(x, w_folded, num_q_heads: int, num_kv_heads: int, q_weight, k_weight, eps: float, positions, cos_sin,
                                    rowsq: torch.Tensor, norm_eps: float, k_cache=None, v_cache=None, slot_mapping=None,
                                    raw_rows: int = 0) -> torch.Tensor:
    """`linear_qkv_rope_store` over un-normalised rows (see linear_swiglu_rowscaled); only for shapes whose epilogue runs
    inside the GEMM (HipError otherwise)."""
    _gpu_bf16(x, w_folded, q_weight, k_weight)
    t, k = x.shape
    n = (num_q_heads + 2 * num_kv_heads) * 128
    assert w_folded.shape == (n, k) and w_folded.is_contiguous() and x.stride(1) == 1 and positions.dtype == torch.int64
    assert rowsq.dtype == torch.float32 and rowsq.shape[0] == t and rowsq.is_contiguous()
    store = k_cache is not None and k_cache.numel() > 0 and slot_mapping is not None and slot_mapping.numel() > 0
    qkv = torch.empty(t, n, dtype=BF16, device=x.device)
    _hip.call("nvh_gemm_qkv_rope_store_rowscaled", x.data_ptr(), x.stride(0), w_folded.data_ptr(), qkv.data_ptr(), n, t, k, num_q_heads,
              num_kv_heads, 128, q_weight.data_ptr(), k_weight.data_ptr(), float(eps), positions.data_ptr(), cos_sin.data_ptr(),
              cos_sin.shape[0], k_cache.data_ptr() if store else 0, v_cache.data_ptr() if store else 0,
              slot_mapping.data_ptr() if store else 0, raw_rows, rowsq.data_ptr(), rowsq.shape[1], float(norm_eps), _stream())
    return qkv


def store_kvcache(key, value, k_cache, v_cache, slot_mapping) -> None:
    _gpu_bf16(key, value, k_cache, v_cache)
    n, h, d = key.shape
    assert key.stride(-1) == 1 and value.stride(-1) == 1 and key.stride(1) == d and value.stride(1) == d
    assert k_cache.is_contiguous() and v_cache.is_contiguous() and slot_mapping.dtype == torch.int32
    assert slot_mapping.numel() == n
    _hip.call("nvh_store_kvcache", key.data_ptr(), key.stride(0), value.data_ptr(), value.stride(0), k_cache.data_ptr(),
              v_cache.data_ptr(), slot_mapping.data_ptr(), n, h * d, _stream())


# ---------------------------------------------------------------- activation / gathers
def silu_mul(x: torch.Tensor) -> torch.Tensor:
    _gpu_bf16(x)
    if not x.is_contiguous():
        x = x.contiguous()
    inter = x.shape[-1] // 2
    rows = x.numel() // (2 * inter)
    y = torch.empty(*x.shape[:-1], inter, dtype=BF16, device=x.device)
    _hip.call("nvh_silu_mul", x.data_ptr(), y.data_ptr(), rows, inter, _stream())
    return y


def embedding(ids: torch.Tensor, table: torch.Tensor, vocab_start: int = 0) -> torch.Tensor:
    _gpu_bf16(table)
    assert ids.dtype == torch.int64 and ids.is_cuda and table.is_contiguous()
    out = torch.empty(ids.numel(), table.shape[1], dtype=BF16, device=table.device)
    _hip.call("nvh_embedding", ids.data_ptr(), table.data_ptr(), out.data_ptr(), ids.numel(), table.shape[1],
              vocab_start, table.shape[0], _stream())
    return out


def feed_token_ids(input_ids: torch.Tensor, dst_index: torch.Tensor, sampled: torch.Tensor, src_index: torch.Tensor) -> None:
    """input_ids[dst_index[i]] = sampled[src_index[i]], in place (ids a step takes from the previous step's sampler
    output before the host has read them)."""
    assert input_ids.dtype == torch.int64 and sampled.dtype == torch.int64 and input_ids.is_cuda and sampled.is_cuda
    assert dst_index.dtype == torch.int32 and src_index.dtype == torch.int32 and dst_index.numel() == src_index.numel()
    assert input_ids.is_contiguous() and sampled.is_contiguous()
    _hip.call("nvh_feed_token_ids", input_ids.data_ptr(), dst_index.data_ptr(), sampled.data_ptr(), src_index.data_ptr(),
              dst_index.numel(), _stream())


def gather_last_rows(hidden: torch.Tensor, cu_seqlens_q: torch.Tensor, need: torch.Tensor | None, num_rows: int) -> torch.Tensor:
    _gpu_bf16(hidden)
    assert hidden.is_contiguous() and cu_seqlens_q.dtype == torch.int32
    out = torch.empty(num_rows, hidden.shape[1], dtype=BF16, device=hidden.device)
    _hip.call("nvh_gather_last_rows", hidden.data_ptr(), cu_seqlens_q.data_ptr(), _p(need), out.data_ptr(), num_rows,
              hidden.shape[1], _stream())
    return out


# ---------------------------------------------------------------- GEMM
def suggest_split_k(m: int, n: int, k: int) -> int:
    return _hip.lib().nvh_gemm_suggest_split_k(m, n, k)


def linear(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
    """y = x @ W^T (+ bias); x [..., K] with contiguous rows, W [N, K]."""
    _gpu_bf16(x, weight)
    k = x.shape[-1]
    n = weight.shape[0]
    assert weight.is_contiguous() and weight.shape[1] == k
    x2 = x.reshape(-1, k)
    if x2.stride(1) != 1:
        x2 = x2.contiguous()
    m = x2.shape[0]
    y = torch.empty(m, n, dtype=BF16, device=x.device)
    _hip.call("nvh_gemm_bf16_nt", x2.data_ptr(), x2.stride(0), weight.data_ptr(), _p(bias), y.data_ptr(), n, m, n, k, 1,
              0, _stream())
    return y.view(*x.shape[:-1], n)


def linear_splitk(x: torch.Tensor, weight: torch.Tensor, split_k: int) -> torch.Tensor:
    """fp32 partial slabs [split_k, M, N]; the consumer (add_rmsnorm / splitk_reduce) sums them."""
    _gpu_bf16(x, weight)
    k = x.shape[-1]
    n = weight.shape[0]
    x2 = x.reshape(-1, k)
    if x2.stride(1) != 1:
        x2 = x2.contiguous()
    m = x2.shape[0]
    ws = torch.empty(split_k, m, n, dtype=torch.float32, device=x.device)
    _hip.call("nvh_gemm_bf16_nt", x2.data_ptr(), x2.stride(0), weight.data_ptr(), 0, 0, n, m, n, k, split_k,
              ws.data_ptr(), _stream())
    return ws


def interleave_gate_up(weight: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    """[gate (I rows) | up (I rows)] -> blocks of 16 gate rows followed by their 16 up rows (for linear_swiglu)."""
    _gpu_bf16(weight)
    assert weight.is_contiguous() and weight.shape[0] % 32 == 0
    if out is None:
        out = torch.empty_like(weight)
    assert out.shape == weight.shape and out.is_contiguous() and out.data_ptr() != weight.data_ptr()
    _hip.call("nvh_interleave_gate_up", weight.data_ptr(), out.data_ptr(), weight.shape[0] // 2, weight.shape[1], _stream())
    return out


def linear_swiglu(x: torch.Tensor, weight_interleaved: torch.Tensor) -> torch.Tensor:
    """silu(x Wg^T) * (x Wu^T) in one kernel; bit-identical to silu_mul(linear(x, W))."""
    _gpu_bf16(x, weight_interleaved)
    k = x.shape[-1]
    n = weight_interleaved.shape[0]
    x2 = x.reshape(-1, k)
    if x2.stride(1) != 1:
        x2 = x2.contiguous()
    m = x2.shape[0]
    y = torch.empty(m, n // 2, dtype=BF16, device=x.device)
    _hip.call("nvh_gemm_swiglu_bf16_nt", x2.data_ptr(), x2.stride(0), weight_interleaved.data_ptr(), y.data_ptr(), n // 2,
              m, n, k, _stream())
    return y.view(*x.shape[:-1], n // 2)


def add_rmsnorm_linear(x: torch.Tensor | None, residual: torch.Tensor, norm_weight: torch.Tensor, eps: float, weight: torch.Tensor,
                       partials: torch.Tensor | None = None, swiglu: bool = False) -> tuple[torch.Tensor, torch.Tensor]:
    """(y, new_residual) of add_rmsnorm followed by linear (or linear_swiglu over an interleaved weight) in ONE launch:
    decode batches of 1..64 rows with rows of at most 1024 elements.  ``residual`` is NOT modified; bit-identical to the
    two calls.  ``fused_add_rmsnorm_linear`` tells whether the step executor would take it."""
    _gpu_bf16(residual, norm_weight, weight)
    k = residual.shape[-1]
    m = residual.numel() // k
    n = weight.shape[0]
    assert residual.is_contiguous() and weight.is_contiguous() and weight.shape[1] == k
    new_res = torch.empty_like(residual)
    y = torch.empty(m, n // 2 if swiglu else n, dtype=BF16, device=residual.device)
    if partials is not None:
        assert partials.dtype == torch.float32 and partials.is_contiguous() and partials.shape[-2:] == (m, k)
        prev, slabs, ns = 0, partials.data_ptr(), partials.shape[0]
    else:
        _gpu_bf16(x)
        x = x.contiguous()
        prev, slabs, ns = x.data_ptr(), 0, 0
    _hip.call("nvh_add_rmsnorm_gemm_bf16_nt", prev, slabs, ns, residual.data_ptr(), new_res.data_ptr(), norm_weight.data_ptr(),
              float(eps), weight.data_ptr(), y.data_ptr(), y.shape[1], m, n, k, 1 if swiglu else 0, _stream())
    return y, new_res


def fused_add_rmsnorm_linear(m: int, n: int, k: int, num_partials: int = 0, swiglu: bool = False) -> bool:
    return _hip.lib().nvh_add_rmsnorm_gemm_fused(m, n, k, num_partials, 1 if swiglu else 0) == 1


def splitk_reduce(partials: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
    s, m, n = partials.shape
    y = torch.empty(m, n, dtype=BF16, device=partials.device)
    _hip.call("nvh_splitk_reduce", partials.data_ptr(), s, _p(bias), y.data_ptr(), n, m, n, _stream())
    return y


# ---------------------------------------------------------------- attention
def attn_varlen(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q: int, scale: float, block_tables=None,
                max_seqlen_k: int | None = None, num_splits: int = 0) -> torch.Tensor:
    """q [T,Hq,128]; (k, v) packed [Tk,Hkv,128] or page pools [P,256,Hkv,128] with block_tables [B,W] int32."""
    _gpu_bf16(q, k, v)
    t, hq, d = q.shape
    assert q.stride(2) == 1 and q.stride(1) == d
    if block_tables is None:
        hkv = k.shape[1]
        assert k.stride(2) == 1 and k.stride(1) == d and v.stride(1) == d and k.stride(0) == v.stride(0)
        kv_stride, tbl, tbl_stride = k.stride(0), 0, 0
    else:
        hkv = k.shape[2]
        assert k.is_contiguous() and v.is_contiguous() and k.shape[1] == KV_PAGE
        assert block_tables.dtype == torch.int32 and block_tables.stride(1) == 1
        kv_stride, tbl, tbl_stride = hkv * d, block_tables.data_ptr(), block_tables.stride(0)
    out = torch.empty(t, hq, d, dtype=BF16, device=q.device)
    batch = cu_seqlens_q.numel() - 1
    if max_seqlen_k is None:        # upper bound: every key of the pool / packed buffer
        max_seqlen_k = block_tables.shape[1] * KV_PAGE if block_tables is not None else k.shape[0]
    lib = _hip.lib()
    if num_splits <= 0:
        num_splits = lib.nvh_attn_varlen_suggest_splits(t, batch, hq, hkv, max_seqlen_k)
    ws = 0
    if num_splits > 1:
        ws_t = torch.empty(lib.nvh_attn_varlen_workspace_bytes(t, hq, d, num_splits) // 4, dtype=torch.float32, device=q.device)
        ws = ws_t.data_ptr()
    _hip.call("nvh_attn_varlen", q.data_ptr(), q.stride(0), k.data_ptr(), v.data_ptr(), kv_stride,
              cu_seqlens_q.data_ptr(), cu_seqlens_k.data_ptr(), tbl, tbl_stride, batch,
              max_seqlen_q, max_seqlen_k, t, hq, hkv, d, float(scale), out.data_ptr(), num_splits, ws, _stream())
    return out


def suggest_decode_splits(batch: int, num_kv_heads: int, max_context: int) -> int:
    return _hip.lib().nvh_attn_decode_suggest_splits(batch, num_kv_heads, max_context)


def plan_decode_items(context_lens, max_ranges: int = 32, range_keys: int = 0, capacity: int = 0) -> dict:
    """Work list of the decode attention for a batch of uneven context lengths (host side, numpy): one item per
    key range, where only sequences that hold at least two ranges' worth of keys are cut into ranges.  A range
    is `range_keys` keys (0: total keys / 512, kept within 512..2048) and a sequence has at most `max_ranges`;
    `capacity` > 0 fixes the list length (unused slots -1) and widens the ranges until the list fits it.
    Returns int32 arrays item_seq, item_range [items], seq_active, seq_chunk [B] and max_ranges."""
    import numpy as np
    ctx = np.maximum(np.asarray(context_lens, dtype=np.int64), 0)
    b = ctx.size
    assert capacity <= 0 or capacity >= b
    if range_keys <= 0:
        range_keys = min(2048, max(512, (-(-int(ctx.sum()) // 512) + 63) // 64 * 64))
    while True:
        active = np.clip(ctx // range_keys, 1, max_ranges)
        if capacity <= 0 or int(active.sum()) <= capacity:
            break
        range_keys *= 2
    chunk = np.maximum(64, (-(-ctx // active) + 63) // 64 * 64)
    active = np.maximum(1, -(-ctx // chunk))              # rounding the range up to 64 keys can empty the last one
    n = capacity if capacity > 0 else int(active.sum())
    # longest items first: workgroups are dispatched in list order, and a long range started last would run on alone
    order = np.argsort(-chunk * (active > 1), kind="stable")
    reps = active[order]
    total = int(reps.sum())
    item_seq, item_range = np.full(n, -1, np.int32), np.zeros(n, np.int32)
    item_seq[:total] = np.repeat(order, reps)
    item_range[:total] = np.arange(total) - np.repeat(np.cumsum(reps) - reps, reps)
    return {"item_seq": item_seq, "item_range": item_range, "seq_active": active.astype(np.int32),
            "seq_chunk": chunk.astype(np.int32), "max_ranges": max_ranges}


def upload_decode_items(plan: dict, device, out: torch.Tensor | None = None) -> dict:
    """The plan's four arrays in one int32 device tensor (one copy); `out` reuses a buffer of the right length."""
    import numpy as np
    packed = np.concatenate([plan["item_seq"], plan["item_range"], plan["seq_active"], plan["seq_chunk"]])
    host = torch.from_numpy(packed)
    if out is None:
        out = host.to(device, non_blocking=False)
    else:
        assert out.numel() == packed.size and out.dtype == torch.int32
        out.copy_(host, non_blocking=False)
    n, b = plan["item_seq"].size, plan["seq_active"].size
    return {"item_seq": out[:n], "item_range": out[n:2 * n], "seq_active": out[2 * n:2 * n + b],
            "seq_chunk": out[2 * n + b:2 * n + 2 * b], "max_ranges": plan["max_ranges"]}


def _items_args(items, batch):
    assert all(items[k].dtype == torch.int32 and items[k].is_cuda and items[k].is_contiguous()
               for k in ("item_seq", "item_range", "seq_active", "seq_chunk"))
    assert items["item_seq"].numel() == items["item_range"].numel() >= batch
    assert items["seq_active"].numel() == items["seq_chunk"].numel() == batch
    return (items["item_seq"].data_ptr(), items["item_range"].data_ptr(), items["seq_active"].data_ptr(),
            items["seq_chunk"].data_ptr(), items["item_seq"].numel(), items["max_ranges"])


def attn_decode(q, k_cache, v_cache, context_lens, block_tables, scale: float, num_splits: int = 0,
                max_context: int | None = None, min_range: int = 0, items: dict | None = None) -> torch.Tensor:
    """q [B,Hq,128] (token stride free); caches [P,256,Hkv,128]; one query per sequence.  `num_splits` key ranges
    are offered to every sequence, of at least `min_range` keys each (0 = 64); or `items`, an uploaded
    plan_decode_items work list, names the ranges one by one."""
    _gpu_bf16(q, k_cache, v_cache)
    b, hq, d = q.shape
    hkv = k_cache.shape[2]
    assert q.stride(2) == 1 and q.stride(1) == d and k_cache.is_contiguous() and v_cache.is_contiguous()
    assert context_lens.dtype == torch.int32 and block_tables.dtype == torch.int32 and block_tables.stride(1) == 1
    if items is not None:
        num_splits = items["max_ranges"]
    elif num_splits <= 0:
        mc = max_context if max_context is not None else block_tables.shape[1] * KV_PAGE
        num_splits = suggest_decode_splits(b, hkv, mc)
    out = torch.empty(b, hq, d, dtype=BF16, device=q.device)
    ws = 0
    if num_splits > 1:
        nbytes = _hip.lib().nvh_attn_decode_workspace_bytes(b, hq, d, num_splits)
        ws_t = torch.empty(nbytes // 4, dtype=torch.float32, device=q.device)
        ws = ws_t.data_ptr()
    if items is not None:
        _hip.call("nvh_attn_decode_items", q.data_ptr(), q.stride(0), k_cache.data_ptr(), v_cache.data_ptr(),
                  context_lens.data_ptr(), block_tables.data_ptr(), block_tables.stride(0), b, hq, hkv, d, float(scale),
                  out.data_ptr(), *_items_args(items, b), ws, _stream())
        return out
    _hip.call("nvh_attn_decode", q.data_ptr(), q.stride(0), k_cache.data_ptr(), v_cache.data_ptr(),
              context_lens.data_ptr(), block_tables.data_ptr(), block_tables.stride(0), b, hq, hkv, d, float(scale),
              out.data_ptr(), num_splits, min_range, ws, _stream())
    return out


def attn_decode_fused_qkv(qkv, num_q_heads: int, num_kv_heads: int, q_weight, k_weight, eps: float, positions, cos_sin,
                          k_cache, v_cache, context_lens, block_tables, scale: float, num_splits: int = 0,
                          max_context: int | None = None, min_range: int = 0, items: dict | None = None) -> torch.Tensor:
    """Decode attention straight from the raw fused qkv rows [B, (Hq+2Hkv)*128]: q/k norm + RoPE + KV store +
    attention in one launch."""
    _gpu_bf16(qkv, q_weight, k_weight, k_cache, v_cache)
    b, d = qkv.shape[0], 128
    assert qkv.stride(1) == 1 and k_cache.is_contiguous() and v_cache.is_contiguous() and positions.dtype == torch.int64
    if items is not None:
        num_splits = items["max_ranges"]
    elif num_splits <= 0:
        mc = max_context if max_context is not None else block_tables.shape[1] * KV_PAGE
        num_splits = suggest_decode_splits(b, num_kv_heads, mc)
    out = torch.empty(b, num_q_heads, d, dtype=BF16, device=qkv.device)
    ws = 0
    if num_splits > 1:
        ws_t = torch.empty(_hip.lib().nvh_attn_decode_workspace_bytes(b, num_q_heads, d, num_splits) // 4,
                           dtype=torch.float32, device=qkv.device)
        ws = ws_t.data_ptr()
    if items is not None:
        _hip.call("nvh_attn_decode_fused_qkv_items", qkv.data_ptr(), qkv.stride(0), q_weight.data_ptr(), k_weight.data_ptr(),
                  float(eps), positions.data_ptr(), cos_sin.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                  context_lens.data_ptr(), block_tables.data_ptr(), block_tables.stride(0), b, num_q_heads, num_kv_heads, d,
                  float(scale), out.data_ptr(), *_items_args(items, b), ws, _stream())
        return out
    _hip.call("nvh_attn_decode_fused_qkv", qkv.data_ptr(), qkv.stride(0), q_weight.data_ptr(), k_weight.data_ptr(), float(eps),
              positions.data_ptr(), cos_sin.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), context_lens.data_ptr(),
              block_tables.data_ptr(), block_tables.stride(0), b, num_q_heads, num_kv_heads, d, float(scale), out.data_ptr(),
              num_splits, min_range, ws, _stream())
    return out


# ---------------------------------------------------------------- sampling
def _logits_args(logits):
    assert logits.is_cuda and logits.dim() == 2 and logits.stride(1) == 1
    if logits.dtype == torch.float32:
        return 1
    if logits.dtype == BF16:
        return 0
    raise TypeError(f"logits dtype {logits.dtype} unsupported")


def _sample_ws(logits):
    n = _hip.lib().nvh_sample_workspace_bytes(logits.shape[0], logits.shape[1])
    return torch.empty(n, dtype=torch.uint8, device=logits.device) if n else None


def argmax(logits: torch.Tensor) -> torch.Tensor:
    f = _logits_args(logits)
    out = torch.empty(logits.shape[0], dtype=torch.int64, device=logits.device)
    ws = _sample_ws(logits)
    _hip.call("nvh_argmax", logits.data_ptr(), f, logits.stride(0), out.data_ptr(), logits.shape[0], logits.shape[1],
              _p(ws), _stream())
    return out


def sample(logits: torch.Tensor, temperatures: torch.Tensor, seed: int, offset: int) -> torch.Tensor:
    f = _logits_args(logits)
    assert temperatures.dtype == torch.float32 and temperatures.numel() == logits.shape[0]
    out = torch.empty(logits.shape[0], dtype=torch.int64, device=logits.device)
    ws = _sample_ws(logits)
    _hip.call("nvh_sample", logits.data_ptr(), f, logits.stride(0), temperatures.data_ptr(), out.data_ptr(),
              logits.shape[0], logits.shape[1], seed, offset, _p(ws), _stream())
    return out


def lm_head_sample_fused(m: int, n: int, k: int) -> bool:
    """Whether `lm_head_sample` covers an [m, k] x [n, k]^T projection (it takes the 256 x 256 GEMM tile)."""
    return bool(_hip.lib().nvh_lm_head_sample_fused(m, n, k))


def lm_head_sample(x: torch.Tensor, weight: torch.Tensor, temperatures: torch.Tensor, seed: int, offset: int) -> torch.Tensor:
    """sample(x @ W^T, temperatures, seed, offset) in one GEMM launch + a pick: the logits are never written."""
    _gpu_bf16(x, weight)
    m, k = x.shape
    n = weight.shape[0]
    assert x.stride(1) == 1 and weight.is_contiguous() and weight.shape[1] == k
    assert temperatures.dtype == torch.float32 and temperatures.numel() == m
    out = torch.empty(m, dtype=torch.int64, device=x.device)
    ws = torch.empty(_hip.lib().nvh_lm_head_sample_workspace_bytes(m, n), dtype=torch.uint8, device=x.device)
    _hip.call("nvh_lm_head_sample", x.data_ptr(), x.stride(0), weight.data_ptr(), temperatures.data_ptr(), out.data_ptr(), m, n, k,
              seed, offset, ws.data_ptr(), _stream())
    return out


def sample_shard(logits: torch.Tensor, temperatures: torch.Tensor, seed: int, offset: int, col_offset: int, rank: int,
                 world: int) -> torch.Tensor:
    """Best candidate of every row of a vocabulary shard [rows, shard_vocab] (columns col_offset.. of the full row), as
    bf16 bytes in this rank's segment of a [world, rows, 8] tensor (zeros elsewhere): sum it over the ranks, then
    `sample_pick`."""
    f = _logits_args(logits)
    rows, vocab = logits.shape
    assert temperatures.dtype == torch.float32 and temperatures.numel() == rows
    enc = torch.empty(world, rows, 8, dtype=BF16, device=logits.device)
    ws = torch.empty(max(16, _hip.lib().nvh_sample_shard_workspace_bytes(rows, vocab)), dtype=torch.uint8, device=logits.device)
    _hip.call("nvh_sample_shard", logits.data_ptr(), f, logits.stride(0), temperatures.data_ptr(), enc.data_ptr(), rows, vocab,
              col_offset, rank, world, seed, offset, ws.data_ptr(), _stream())
    return enc


def sample_pick(enc: torch.Tensor) -> torch.Tensor:
    """The winner per row among the ranks' candidates (`sample_shard` summed over the ranks): int64 [rows]."""
    world, rows, _ = enc.shape
    assert enc.dtype == BF16 and enc.is_contiguous()
    out = torch.empty(rows, dtype=torch.int64, device=enc.device)
    _hip.call("nvh_sample_pick", enc.data_ptr(), out.data_ptr(), rows, world, _stream())
    return out


def sample_with_noise(logits: torch.Tensor, temperatures: torch.Tensor, noise: torch.Tensor) -> torch.Tensor:
    f = _logits_args(logits)
    assert noise.dtype == torch.float32 and noise.is_contiguous() and noise.shape == logits.shape
    out = torch.empty(logits.shape[0], dtype=torch.int64, device=logits.device)
    ws = _sample_ws(logits)
    _hip.call("nvh_sample_with_noise", logits.data_ptr(), f, logits.stride(0), temperatures.data_ptr(), noise.data_ptr(),
              out.data_ptr(), logits.shape[0], logits.shape[1], _p(ws), _stream())
    return out


# ---------------------------------------------------------------- fp32 residual stream, free head sizes, bf16 or fp32 activations
F32 = torch.float32


def _act_flag(*tensors) -> int:
    """0 for bf16 activations, 1 for fp32; every tensor must be on the GPU and of the one type."""
    dt = tensors[0].dtype
    for t in tensors:
        if not t.is_cuda or t.dtype != dt:
            raise TypeError(f"expected GPU tensors of one activation type, got {t.dtype} on {t.device} beside {dt}")
    if dt not in (BF16, F32):
        raise TypeError(f"activation type {dt} unsupported (bf16 or fp32)")
    return int(dt == F32)


def linear_any(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None, out_f32: bool = False) -> torch.Tensor:
    """y = x @ W^T (+ bias) for any sizes: bf16 shapes the tuned GEMM takes (K % 64 == 0, N % 4 == 0, 16-byte rows) go
    there, everything else - ragged sizes, fp32 operands, an fp32 result of bf16 operands - to the any-shape kernel.  The
    route depends on (N, K) and the types only, never on the number of rows."""
    f = _act_flag(x, weight)
    k, n = x.shape[-1], weight.shape[0]
    assert weight.is_contiguous() and weight.shape[1] == k and x.stride(-1) == 1
    x2 = x.reshape(-1, k)
    m = x2.shape[0]
    if not f and not out_f32 and k % 64 == 0 and n % 4 == 0 and x2.stride(0) % 8 == 0 and x2.data_ptr() % 16 == 0:
        y = torch.empty(m, n, dtype=BF16, device=x.device)
        if m:
            _hip.call("nvh_gemm_bf16_nt", x2.data_ptr(), x2.stride(0), weight.data_ptr(), _p(bias), y.data_ptr(), n, m, n, k, 1, 0, _stream())
        return y
    out_f32 = bool(out_f32 or f)
    y = torch.empty(m, n, dtype=F32 if out_f32 else BF16, device=x.device)
    _hip.call("nvh_gemm_any_nt", x2.data_ptr(), x2.stride(0), weight.data_ptr(), _p(bias), y.data_ptr(), n, m, n, k, f, int(out_f32), _stream())
    return y


def embedding_stream(ids: torch.Tensor, table: torch.Tensor, x0: torch.Tensor | None = None) -> torch.Tensor:
    """fp32 rows table[ids]; `x0` (a view [T, dim] of the table's type, row stride free) receives the same rows."""
    f = _act_flag(table)
    assert ids.dtype == torch.int64 and table.is_contiguous()
    t, dim = ids.numel(), table.shape[1]
    x = torch.empty(t, dim, dtype=F32, device=table.device)
    assert x0 is None or (x0.dtype == table.dtype and x0.shape == (t, dim) and x0.stride(1) == 1)
    _hip.call("nvh_embedding_stream", ids.data_ptr(), table.data_ptr(), x.data_ptr(), _p(x0), x0.stride(0) if x0 is not None else 0,
              t, dim, table.shape[0], f, _stream())
    return x


def residual_dyt(x: torch.Tensor, y: torch.Tensor | None = None, post=None, bias: torch.Tensor | None = None, accumulate: bool = True,
                 nxt=None, out: torch.Tensor | None = None) -> torch.Tensor | None:
    """x <- (x if accumulate else 0) + post(y) + bias in place (fp32 rows); returns next(x) in the activation type, or None
    without `nxt`.  post / nxt are (alpha, weight, bias) triples of a Dynamic-Tanh norm."""
    assert x.dtype == F32 and x.is_contiguous() and x.dim() == 2
    rows, dim = x.shape
    ref = nxt[1] if nxt is not None else (post[1] if post is not None else (y if y is not None else bias))
    f = _act_flag(ref)
    h = None
    if nxt is not None:
        h = out if out is not None else torch.empty(rows, dim, dtype=ref.dtype, device=x.device)
        assert h.stride(1) == 1 and h.shape == (rows, dim)
    assert y is None or (y.shape == (rows, dim) and y.stride(1) == 1 and y.dtype == ref.dtype)
    pa, pw, pb = post if post is not None else (None, None, None)
    na, nw, nb = nxt if nxt is not None else (None, None, None)
    _hip.call("nvh_residual_dyt", _p(y), y.stride(0) if y is not None else 0, _p(pa), _p(pw), _p(pb), _p(bias), x.data_ptr(), int(accumulate),
              _p(na), _p(nw), _p(nb), _p(h), h.stride(0) if h is not None else 0, rows, dim, f, _stream())
    return h


def stream_cast_(x: torch.Tensor, out: torch.Tensor) -> None:
    """out[:, :dim] = x in out's type (out may be wider: its other columns stay)."""
    f = _act_flag(out)
    assert x.dtype == F32 and x.is_contiguous() and out.stride(1) == 1 and out.shape[0] == x.shape[0] and out.shape[1] >= x.shape[1]
    _hip.call("nvh_stream_cast", x.data_ptr(), out.data_ptr(), out.stride(0), x.shape[0], x.shape[1], f, _stream())


def gelu_tanh_mul(gate_up: torch.Tensor) -> torch.Tensor:
    f = _act_flag(gate_up)
    assert gate_up.dim() == 2 and gate_up.stride(1) == 1
    rows, inter = gate_up.shape[0], gate_up.shape[1] // 2
    y = torch.empty(rows, inter, dtype=gate_up.dtype, device=gate_up.device)
    _hip.call("nvh_gelu_tanh_mul", gate_up.data_ptr(), gate_up.stride(0), y.data_ptr(), rows, inter, f, _stream())
    return y


def gather_rows_f32(x: torch.Tensor, index: torch.Tensor) -> torch.Tensor:
    assert x.dtype == F32 and x.is_contiguous() and index.dtype == torch.int32 and x.is_cuda and index.is_cuda
    out = torch.empty(index.numel(), x.shape[1], dtype=F32, device=x.device)
    if index.numel() == 0:
        return out
    _hip.call("nvh_gather_rows_f32", x.data_ptr(), index.data_ptr(), out.data_ptr(), index.numel(), x.shape[1], _stream())
    return out


def logit_softcap(logits: torch.Tensor, cap: float) -> torch.Tensor:
    """fp32 cap * tanh(logits / cap); cap <= 0: the logits in fp32."""
    f = _act_flag(logits)
    assert logits.dim() == 2 and logits.stride(1) == 1
    out = torch.empty(logits.shape, dtype=F32, device=logits.device)
    _hip.call("nvh_logit_softcap", logits.data_ptr(), logits.stride(0), out.data_ptr(), logits.shape[0], logits.shape[1], float(cap or 0.0), f, _stream())
    return out


def attn_rotary_prep(proj, q_norm, k_norm, eps: float, positions, qk_freq, qk_mag: float, rot_dims: int, v_freq, k_cache, v_cache,
                     slot_mapping, heads: int, kv_heads: int, dim: int, vdim: int, gated: bool = True, qk_interleaved: bool = False,
                     v_interleaved: bool = False, norm_per_head: bool = False):
    """(q [T, H*dim], sigmoid gate fp32 [T, H] | None) from the fused projection rows [q | k | v | gate]; k and v go to their
    cache rows (see nvh_attn_rotary_prep).  q_norm / k_norm None: no norm; rot_dims 0: no rotary.  `norm_per_head`: the norm runs
    over every head by itself, with weights [dim] that the heads share (else over the whole projection, weights of its size)."""
    f = _act_flag(proj, k_cache, v_cache) if q_norm is None else _act_flag(proj, q_norm, k_norm, k_cache, v_cache)
    t = proj.shape[0]
    assert proj.stride(1) == 1 and positions.dtype == torch.int64 and slot_mapping.dtype == torch.int32 and slot_mapping.numel() == t
    assert qk_freq is None or (qk_freq.dtype == F32 and qk_freq.numel() * 2 == rot_dims)
    assert v_freq is None or (v_freq.dtype == F32 and v_freq.numel() * 2 == vdim)
    assert (q_norm is None and k_norm is None) or (q_norm.numel() == k_norm.numel() == dim if norm_per_head else
                                                    (q_norm.numel() == heads * dim and k_norm.numel() == kv_heads * dim))
    assert k_cache.is_contiguous() and v_cache.is_contiguous()
    q = torch.empty(t, heads * dim, dtype=proj.dtype, device=proj.device)
    gate = torch.empty(t, heads, dtype=F32, device=proj.device) if gated else None
    _hip.call("nvh_attn_rotary_prep", proj.data_ptr(), proj.stride(0), _p(q_norm), _p(k_norm), float(eps), positions.data_ptr(),
              _p(qk_freq), float(qk_mag), rot_dims, int(qk_interleaved), _p(v_freq), int(v_interleaved), q.data_ptr(), _p(gate),
              k_cache.data_ptr(), v_cache.data_ptr(), slot_mapping.data_ptr(), k_cache.shape[1], t, heads, kv_heads, dim, vdim,
              int(norm_per_head and q_norm is not None), f, _stream())
    return q, gate


def attn_paged_any(q, k_cache, v_cache, cu_seqlens_q, context_lens, block_tables, scale: float, heads: int, kv_heads: int, dim: int,
                   vdim: int, gate=None, v_freq=None, v_interleaved: bool = False, slopes=None, window: int = 0, keep_first: int = 0,
                   chunk: int = 0, sinks=None) -> torch.Tensor:
    """Causal attention of the packed queries q [T, H*dim] over paged caches, keys [pages, page, G, dim] and values
    [pages, G, vdim, page] (transposed within a page, as attn_rotary_prep stores them); out [T, H*vdim].  `slopes` (fp32 [H]):
    score -= slope * distance; `window` > 0: a query sees the last `window` positions and the first `keep_first`; `chunk` > 0: a
    query sees only the keys of its own block of `chunk` positions (counted from the sequence's start); `sinks` (fp32 [H]): a logit
    per head whose exponential is one more term of the softmax's denominator (it stands for no token and carries no value)."""
    f = _act_flag(q, k_cache, v_cache)
    t = q.shape[0]
    batch = context_lens.numel()
    assert q.is_contiguous() and k_cache.is_contiguous() and v_cache.is_contiguous() and k_cache.dim() == 4
    assert tuple(v_cache.shape) == (k_cache.shape[0], kv_heads, vdim, k_cache.shape[1])
    assert context_lens.dtype == torch.int32 and block_tables.dtype == torch.int32 and block_tables.stride(1) == 1
    assert cu_seqlens_q is None or (cu_seqlens_q.dtype == torch.int32 and cu_seqlens_q.numel() == batch + 1)
    assert cu_seqlens_q is not None or t == batch
    assert gate is None or (gate.dtype == F32 and gate.shape == (t, heads) and gate.is_contiguous())
    assert slopes is None or (slopes.dtype == F32 and slopes.numel() == heads and slopes.is_contiguous() and slopes.is_cuda)
    assert sinks is None or (sinks.dtype == F32 and sinks.numel() == heads and sinks.is_contiguous() and sinks.is_cuda)
    out = torch.empty(t, heads * vdim, dtype=q.dtype, device=q.device)
    # one-query steps that would leave most of the chip idle spread a sequence's key tiles over several workgroups: scratch for their rows
    ws_bytes = int(_hip.lib().nvh_attn_paged_any_parts_bytes(batch, t, heads, kv_heads, dim, vdim, k_cache.shape[1], int(v_freq is not None), f))
    ws = torch.empty(ws_bytes // 4, dtype=F32, device=q.device) if ws_bytes else None
    _hip.call("nvh_attn_paged_any", q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), _p(cu_seqlens_q), context_lens.data_ptr(),
              block_tables.data_ptr(), block_tables.stride(0), batch, t, k_cache.shape[1], heads, kv_heads, dim, vdim, float(scale),
              _p(gate), _p(v_freq), int(v_interleaved), _p(slopes), int(window), int(keep_first), int(chunk), _p(sinks), out.data_ptr(), _p(ws), ws_bytes,
              f, _stream())
    return out


def delta_rule(r, k, v, a_raw, lowrank, w2, w0, a_bias, state, slots, cu_seqlens_q, context_lens, heads: int, dk: int,
               decay_scale: float) -> torch.Tensor:
    """One step of the generalized delta rule over the packed tokens: fp32 outputs [T, H*dk]; `state` [slots, H, dk, dk] fp32 is
    read (unless the sequence starts in this step) and left updated.  r, k, v, a_raw, lowrank: column views of the fused
    projection output (row stride free)."""
    f = _act_flag(r, k, v, a_raw, lowrank, w2, w0, a_bias)
    t = r.shape[0]
    batch = context_lens.numel()
    for x in (r, k, v, a_raw, lowrank):
        assert x.stride(1) == 1 and x.shape[0] == t
    assert state.dtype == F32 and state.is_contiguous() and tuple(state.shape[1:]) == (heads, dk, dk) and slots.dtype == torch.int32
    assert w2.is_contiguous() and w2.shape[0] == heads * dk and (cu_seqlens_q is None or cu_seqlens_q.dtype == torch.int32)
    rank = w2.shape[1]
    pack = torch.empty(t, heads, 6, dk, dtype=F32, device=r.device)
    _hip.call("nvh_delta_prep", r.data_ptr(), r.stride(0), k.data_ptr(), k.stride(0), v.data_ptr(), v.stride(0), a_raw.data_ptr(),
              a_raw.stride(0), lowrank.data_ptr(), lowrank.stride(0), w2.data_ptr(), w0.data_ptr(), a_bias.data_ptr(), pack.data_ptr(),
              t, heads, dk, rank, float(decay_scale), f, _stream())
    out = torch.empty(t, heads * dk, dtype=F32, device=r.device)
    _hip.call("nvh_delta_scan", pack.data_ptr(), state.data_ptr(), slots.data_ptr(), _p(cu_seqlens_q), context_lens.data_ptr(),
              out.data_ptr(), batch, heads, dk, dk, _stream())
    return out


def gated_delta_rule(qkv, b, a, conv_w, dt_bias, a_log, conv_state, state, slots, cu_seqlens_q, context_lens, heads: int, qk_heads: int,
                     dk: int, dv: int) -> torch.Tensor:
    """One step of the gated delta rule over the packed tokens: fp32 outputs [T, H*dv].  `qkv`: the column view q | k | v of the
    projection rows (qk_heads*dk, qk_heads*dk, heads*dv channels), convolved over time with `conv_w` [C, taps] (continued from
    `conv_state` [slots, taps - 1, C] fp32, then brought up to date) and passed through silu; `b`, `a`: column views [T, H] of the
    write-strength and decay logits.  `state` [slots, H, dk, dv] fp32 is read (unless the sequence starts in this step) and left
    updated."""
    f = _act_flag(qkv, b, a, conv_w, dt_bias, a_log)
    t, c = qkv.shape[0], 2 * qk_heads * dk + heads * dv
    taps = conv_w.shape[1]
    batch = context_lens.numel()
    assert qkv.shape[1] == c and qkv.stride(1) == 1 and b.shape == (t, heads) and a.shape == (t, heads) and b.stride(1) == 1 and a.stride(1) == 1
    assert conv_w.shape == (c, taps) and conv_w.is_contiguous() and dt_bias.numel() == heads and a_log.numel() == heads and heads % qk_heads == 0
    assert taps == 1 or (conv_state.dtype == F32 and conv_state.is_contiguous() and tuple(conv_state.shape[1:]) == (taps - 1, c))
    assert state.dtype == F32 and state.is_contiguous() and tuple(state.shape[1:]) == (heads, dk, dv) and slots.dtype == torch.int32
    assert context_lens.dtype == torch.int32 and (cu_seqlens_q is None or cu_seqlens_q.dtype == torch.int32)
    pack = torch.empty(t, heads, 5 * dk + dv, dtype=F32, device=qkv.device)
    _hip.call("nvh_gated_delta_prep", qkv.data_ptr(), qkv.stride(0), b.data_ptr(), b.stride(0), a.data_ptr(), a.stride(0), conv_w.data_ptr(),
              dt_bias.data_ptr(), a_log.data_ptr(), _p(conv_state), slots.data_ptr(), _p(cu_seqlens_q), context_lens.data_ptr(), pack.data_ptr(),
              batch, t, taps, heads, qk_heads, dk, dv, f, _stream())
    _hip.call("nvh_conv_state_update", qkv.data_ptr(), qkv.stride(0), _p(conv_state), slots.data_ptr(), _p(cu_seqlens_q), context_lens.data_ptr(), batch,
              taps, c, f, _stream())
    out = torch.empty(t, heads * dv, dtype=F32, device=qkv.device)
    _hip.call("nvh_delta_scan", pack.data_ptr(), state.data_ptr(), slots.data_ptr(), _p(cu_seqlens_q), context_lens.data_ptr(),
              out.data_ptr(), batch, heads, dk, dv, _stream())
    return out


def delta_post(o: torch.Tensor, norm_weight: torch.Tensor, gate: torch.Tensor | None, heads: int, dv: int, eps: float) -> torch.Tensor:
    """o / rms_head(o) * norm_weight * sigmoid(gate) in norm_weight's type; gate: a column view of the projection output."""
    f = _act_flag(norm_weight) if gate is None else _act_flag(norm_weight, gate)
    assert o.dtype == F32 and o.is_contiguous() and o.shape[1] == heads * dv and (gate is None or gate.stride(1) == 1)
    y = torch.empty(o.shape, dtype=norm_weight.dtype, device=o.device)
    _hip.call("nvh_delta_post", o.data_ptr(), norm_weight.data_ptr(), _p(gate), gate.stride(0) if gate is not None else 0, y.data_ptr(),
              y.stride(0), o.shape[0], heads, dv, float(eps), f, _stream())
    return y


# ---------------------------------------------------------------- layer norm / RMS norm around the fp32 stream, plain activations
NORM_KINDS = {None: 0, "layer": 1, "rms": 2}
ACTS = {"silu": 0, "gelu_tanh": 1, "relu2": 2}


def embedding_pos_stream(ids: torch.Tensor, positions: torch.Tensor, table: torch.Tensor, pos_table: torch.Tensor | None, scale: float = 1.0) -> torch.Tensor:
    """fp32 rows table[ids] * scale + pos_table[positions]."""
    f = _act_flag(table) if pos_table is None else _act_flag(table, pos_table)
    assert ids.dtype == torch.int64 and positions.dtype == torch.int64 and table.is_contiguous() and (pos_table is None or pos_table.is_contiguous())
    t, dim = ids.numel(), table.shape[1]
    assert pos_table is None or pos_table.shape[1] == dim
    x = torch.empty(t, dim, dtype=F32, device=table.device)
    _hip.call("nvh_embedding_pos_stream", ids.data_ptr(), positions.data_ptr(), table.data_ptr(), _p(pos_table), float(scale), x.data_ptr(), t, dim,
              table.shape[0], pos_table.shape[0] if pos_table is not None else 0, f, _stream())
    return x


def residual_norm(x: torch.Tensor, a=None, a_weight=None, b=None, b_weight=None, branch_scale: float = 1.0, branch_eps: float = 0.0, c=None, c32=None,
                  norm: str | None = None, weight=None, bias=None, eps: float = 0.0) -> torch.Tensor | None:
    """x <- x + branch_scale * (unit(a) a_weight + unit(b) b_weight) + c + c32 in place (fp32 rows; a branch without a weight
    is added as it is, absent terms are skipped); returns norm(x) in the activation type, or None without `norm`."""
    assert x.dtype == F32 and x.is_contiguous() and x.dim() == 2
    rows, dim = x.shape
    typed = [t for t in (a, a_weight, b, b_weight, c, weight, bias) if t is not None]
    assert typed, "nothing to add and nothing to normalise"
    f = _act_flag(*typed)
    for t in (a, b, c):
        assert t is None or (t.shape == (rows, dim) and t.stride(1) == 1)
    for t in (a_weight, b_weight, weight, bias):
        assert t is None or (t.numel() == dim and t.is_contiguous())
    assert c32 is None or (c32.dtype == F32 and c32.shape == (rows, dim) and c32.stride(1) == 1)
    h = torch.empty(rows, dim, dtype=weight.dtype, device=x.device) if norm is not None else None
    _hip.call("nvh_residual_norm", _p(a), a.stride(0) if a is not None else 0, _p(a_weight), _p(b), b.stride(0) if b is not None else 0, _p(b_weight),
              float(branch_scale), float(branch_eps), _p(c), c.stride(0) if c is not None else 0, _p(c32), c32.stride(0) if c32 is not None else 0,
              x.data_ptr(), NORM_KINDS[norm], _p(weight), _p(bias), float(eps), _p(h), dim, rows, dim, f, _stream())
    return h


def residual_postnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, y=None, y32=None, layer_scale=None, alpha: float = 1.0,
                      weight_offset: float = 0.0, want_h: bool = True, in_place: bool = True) -> torch.Tensor | None:
    """x <- rms_norm(alpha x + layer_scale (y + y32)) * (weight_offset + weight) in place (fp32 rows; y of the activation type and
    y32 fp32 may each be absent); returns the new x in the activation type (the input of the next sublayer).  `in_place` False:
    x is only read."""
    assert x.dtype == F32 and x.is_contiguous() and x.dim() == 2
    rows, dim = x.shape
    typed = [t for t in (weight, y, layer_scale) if t is not None]
    f = _act_flag(*typed)
    assert weight.numel() == dim and weight.is_contiguous() and (layer_scale is None or (layer_scale.numel() == dim and layer_scale.is_contiguous()))
    assert y is None or (y.shape == (rows, dim) and y.stride(1) == 1)
    assert y32 is None or (y32.dtype == F32 and y32.shape == (rows, dim) and y32.stride(1) == 1)
    h = torch.empty(rows, dim, dtype=weight.dtype, device=x.device) if want_h else None
    _hip.call("nvh_residual_postnorm", _p(y), y.stride(0) if y is not None else 0, _p(y32), y32.stride(0) if y32 is not None else 0, _p(layer_scale),
              float(alpha), x.data_ptr(), int(in_place), weight.data_ptr(), float(weight_offset), float(eps), _p(h), dim, rows, dim, f, _stream())
    return h


def residual_subnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, mult: float = 1.0, a=None, a_scale: float = 1.0, b=None, b_scale: float = 1.0,
                     c32=None, want_h: bool = True):
    """x <- x + mult * weight * y / sqrt(mean(y^2) + eps) in place (fp32 rows), y = a_scale a + b_scale b + c32: a sublayer's result is
    normed before it joins the stream.  a, b: rows of the activation type, c32: fp32 rows (any may be absent); weight: one number or
    one per column.  Returns the new x in the activation type (the next sublayer's input), or None."""
    assert x.dtype == F32 and x.is_contiguous() and x.dim() == 2 and (a is not None or b is not None or c32 is not None)
    rows, dim = x.shape
    typed = [t for t in (a, b, weight) if t is not None]
    f = _act_flag(*typed)
    for t in (a, b, c32):
        assert t is None or (t.shape == (rows, dim) and t.stride(1) == 1)
    assert c32 is None or (c32.dtype == F32 and c32.is_cuda)
    assert weight.numel() in (1, dim) and weight.is_contiguous()
    h = torch.empty(rows, dim, dtype=weight.dtype, device=x.device) if want_h else None
    _hip.call("nvh_residual_subnorm", _p(a), a.stride(0) if a is not None else 0, float(a_scale), _p(b), b.stride(0) if b is not None else 0, float(b_scale),
              _p(c32), c32.stride(0) if c32 is not None else 0, float(mult), weight.data_ptr(), weight.numel(), float(eps), x.data_ptr(), _p(h), dim, rows, dim,
              f, _stream())
    return h


def stream_conv(x: torch.Tensor, weight: torch.Tensor, state: torch.Tensor | None, slots, cu_seqlens_q, context_lens) -> torch.Tensor:
    """h_t = x_t + sum_k weight[:, k] x_(t - taps + 1 + k) over the fp32 stream x [T, dim] (the last tap on the token itself), in weight's
    type.  Rows before this step come from `state` [slots, taps - 1, dim] fp32 (zeros at a sequence's start), which is then brought up
    to date with this step's rows."""
    f = _act_flag(weight)
    t, dim = x.shape
    taps = weight.shape[1]
    batch = context_lens.numel()
    assert x.dtype == F32 and x.is_contiguous() and weight.shape == (dim, taps) and weight.is_contiguous()
    assert taps == 1 or (state.dtype == F32 and state.is_contiguous() and tuple(state.shape[1:]) == (taps - 1, dim))
    assert slots.dtype == torch.int32 and context_lens.dtype == torch.int32 and (cu_seqlens_q is None or cu_seqlens_q.dtype == torch.int32)
    h = torch.empty(t, dim, dtype=weight.dtype, device=x.device)
    _hip.call("nvh_stream_conv", x.data_ptr(), weight.data_ptr(), _p(state), slots.data_ptr(), _p(cu_seqlens_q), context_lens.data_ptr(), h.data_ptr(), dim,
              batch, t, taps, dim, f, _stream())
    _hip.call("nvh_conv_state_update", x.data_ptr(), dim, _p(state), slots.data_ptr(), _p(cu_seqlens_q), context_lens.data_ptr(), batch, taps, dim, 1, _stream())
    return h


def act_mul(x: torch.Tensor, act: str, gated: bool) -> torch.Tensor:
    """act(x) for plain rows, act(x[:, :I]) * x[:, I:] for a merged [gate | up] projection; act: silu, gelu_tanh, relu2."""
    f = _act_flag(x)
    assert x.dim() == 2 and x.stride(1) == 1
    rows, inter = x.shape[0], x.shape[1] // 2 if gated else x.shape[1]
    y = torch.empty(rows, inter, dtype=x.dtype, device=x.device)
    _hip.call("nvh_act_mul", x.data_ptr(), x.stride(0), y.data_ptr(), inter, rows, inter, ACTS[act], int(gated), f, _stream())
    return y


def logits_scale(logits: torch.Tensor, scale: float, cap: float = 0.0) -> torch.Tensor:
    """fp32 scale * logits (softcapped when cap > 0)."""
    f = _act_flag(logits)
    assert logits.dim() == 2 and logits.stride(1) == 1
    out = torch.empty(logits.shape, dtype=F32, device=logits.device)
    _hip.call("nvh_logits_scale", logits.data_ptr(), logits.stride(0), out.data_ptr(), logits.shape[0], logits.shape[1], float(scale), float(cap or 0.0), f, _stream())
    return out


# ---------------------------------------------------------------- linear recurrences with a diagonal decay
def _f32_rows(t, *tensors):
    for x in tensors:
        assert x.dtype == F32 and x.is_cuda and x.stride(-1) == 1 and x.shape[0] == t


SCAN_SEGMENT_MIN_TOKENS = 256      # a sequence that brings at least this many tokens to a step is scanned in segments ...
SCAN_SEGMENT_MAX_BATCH = 8         # ... in steps of at most this many sequences (the segments' records are scratch per sequence)


def gated_linear_scan(q, k, w, v, state, slots, cu_seqlens_q, context_lens, heads: int, dk: int, dv: int, qk_groups: int | None = None,
                      kscale=None, skip=None, max_seqlen_q: int = 0, read_first: bool = False, bonus=None) -> torch.Tensor:
    """S <- diag(w) S + (kscale k) v^T, o = S^T q + skip v over the packed tokens; fp32 operands q, k [T, qk_groups * dk],
    w [T, H * dk] or [T, H] (one decay per head), kscale [T, H] | None, v [T, H * dv], skip [H] | None; `state`
    [slots, H, dv, dk] fp32 (S transposed: a column's rows lie together) is read (unless the sequence starts in this step) and
    left updated.  Returns fp32 [T, H * dv].  `read_first`: o = (S + diag(bonus) (kscale k) v^T)^T q + skip v is taken BEFORE the
    token is written and the state decayed (bonus fp32 [H, dk] | None)."""
    t = v.shape[0]
    g = qk_groups or heads
    _f32_rows(t, q, k, w, v)
    assert q.shape[1] == g * dk and k.shape[1] == g * dk and v.shape[1] == heads * dv and w.shape[1] in (heads, heads * dk)
    w_scalar = w.shape[1] == heads and dk != 1
    assert kscale is None or (kscale.dtype == F32 and kscale.shape == (t, heads) and kscale.stride(1) == 1)
    assert skip is None or (skip.dtype == F32 and skip.numel() == heads and skip.is_contiguous())
    assert bonus is None or (read_first and bonus.dtype == F32 and bonus.numel() == heads * dk and bonus.is_contiguous() and bonus.is_cuda)
    assert state.dtype == F32 and state.is_contiguous() and tuple(state.shape[1:]) == (heads, dv, dk) and slots.dtype == torch.int32
    assert context_lens.dtype == torch.int32 and (cu_seqlens_q is None or cu_seqlens_q.dtype == torch.int32)
    batch = context_lens.numel()
    assert cu_seqlens_q is not None or t == batch
    out = torch.empty(t, heads * dv, dtype=F32, device=v.device)
    # Long portions (prompt chunks) in small batches: segments walked side by side, joined in a second launch.  The choice
    # depends on the step's longest portion, so a position's result may differ between schedules - within fp32 rounding.
    segments, ws_l, ws_d = 1, None, None
    if (cu_seqlens_q is not None and batch <= SCAN_SEGMENT_MAX_BATCH and max_seqlen_q >= SCAN_SEGMENT_MIN_TOKENS
            and _hip.lib().nvh_scan_segmentable(dk)):
        segments = 8 if max_seqlen_q >= 2 * SCAN_SEGMENT_MIN_TOKENS else 4
        ws_l = torch.empty(batch * heads * segments * dv * dk, dtype=F32, device=v.device)
        ws_d = torch.empty(batch * heads * segments * dk, dtype=F32, device=v.device)
    _hip.call("nvh_gated_linear_scan", q.data_ptr(), q.stride(0), k.data_ptr(), k.stride(0), g, w.data_ptr(), w.stride(0), int(w_scalar),
              _p(kscale), kscale.stride(0) if kscale is not None else 0, v.data_ptr(), v.stride(0), _p(skip), state.data_ptr(), slots.data_ptr(),
              _p(cu_seqlens_q), context_lens.data_ptr(), out.data_ptr(), batch, heads, dk, dv, segments, SCAN_SEGMENT_MIN_TOKENS, _p(ws_l), _p(ws_d),
              int(read_first), _p(bonus), _stream())
    return out


def hgrn2_prep(q, f, v, f_bias, lower):
    """fp32 (q, k, w, v) of the HGRN2 recurrence from projection columns: silu(q), 1 - g, g = lower + (1 - lower) sigmoid(f + f_bias), v."""
    fl = _act_flag(q, f, v, f_bias, lower)
    t, nk, nv = q.shape[0], q.shape[1], v.shape[1]
    assert q.stride(1) == 1 and f.stride(1) == 1 and v.stride(1) == 1 and f.shape == (t, nk) and f_bias.numel() == nk and lower.numel() == nk
    oq, ok, ow = (torch.empty(t, nk, dtype=F32, device=q.device) for _ in range(3))
    ov = torch.empty(t, nv, dtype=F32, device=q.device)
    _hip.call("nvh_hgrn2_prep", q.data_ptr(), q.stride(0), f.data_ptr(), f.stride(0), v.data_ptr(), v.stride(0), f_bias.data_ptr(), lower.data_ptr(),
              oq.data_ptr(), ok.data_ptr(), ow.data_ptr(), ov.data_ptr(), t, nk, nv, fl, _stream())
    return oq, ok, ow, ov


def gla_prep(q, k, v, decay_logits, q_scale: float, tau: float):
    """fp32 (q * q_scale, k, sigmoid(decay_logits)^(1/tau), v) from projection columns and fp32 decay logits."""
    fl = _act_flag(q, k, v)
    t, nk, nv = q.shape[0], q.shape[1], v.shape[1]
    assert q.stride(1) == 1 and k.stride(1) == 1 and v.stride(1) == 1 and k.shape == (t, nk)
    assert decay_logits.dtype == F32 and decay_logits.shape == (t, nk) and decay_logits.stride(1) == 1
    oq, ok, ow = (torch.empty(t, nk, dtype=F32, device=q.device) for _ in range(3))
    ov = torch.empty(t, nv, dtype=F32, device=q.device)
    _hip.call("nvh_gla_prep", q.data_ptr(), q.stride(0), k.data_ptr(), k.stride(0), v.data_ptr(), v.stride(0), decay_logits.data_ptr(),
              decay_logits.stride(0), float(q_scale), float(tau), oq.data_ptr(), ok.data_ptr(), ow.data_ptr(), ov.data_ptr(), t, nk, nv, fl, _stream())
    return oq, ok, ow, ov


def wkv_prep(r, k, v, lowrank, w2, w0):
    """fp32 (r, k, w, v) of the RWKV time mix from projection columns: w = exp(-exp(w0 + w2 @ tanh(lowrank))) per key channel, the
    rank-sized product formed in fp32 inside the launch."""
    fl = _act_flag(r, k, v, lowrank, w2, w0)
    t, nk, nv = r.shape[0], r.shape[1], v.shape[1]
    rank = lowrank.shape[1]
    assert r.stride(1) == 1 and k.stride(1) == 1 and v.stride(1) == 1 and lowrank.stride(1) == 1 and k.shape == (t, nk) and lowrank.shape[0] == t
    assert w2.is_contiguous() and tuple(w2.shape) == (nk, rank) and w0.is_contiguous() and w0.numel() == nk
    oq, ok, ow = (torch.empty(t, nk, dtype=F32, device=r.device) for _ in range(3))
    ov = torch.empty(t, nv, dtype=F32, device=r.device)
    _hip.call("nvh_wkv_prep", r.data_ptr(), r.stride(0), k.data_ptr(), k.stride(0), v.data_ptr(), v.stride(0), lowrank.data_ptr(), lowrank.stride(0),
              w2.data_ptr(), w0.data_ptr(), oq.data_ptr(), ok.data_ptr(), ow.data_ptr(), ov.data_ptr(), t, nk, nv, rank, fl, _stream())
    return oq, ok, ow, ov


def token_shift_mix(h: torch.Tensor, mu: torch.Tensor, state: torch.Tensor, slots, cu_seqlens_q, context_lens) -> torch.Tensor:
    """out[s] = h + (previous token's h - h) * mu[s] for every row s of mu [n, dim]: [n, T, dim] in h's type.  The token before a
    step's first comes from `state` fp32 [slots, 1, dim] (zeros when the sequence starts in this step), which is then left
    holding the step's last h of every sequence."""
    f = _act_flag(h, mu)
    t, dim = h.shape
    n = mu.shape[0]
    assert h.stride(1) == 1 and mu.is_contiguous() and mu.shape[1] == dim
    assert state.dtype == F32 and state.is_contiguous() and state.numel() == state.shape[0] * dim
    assert slots.dtype == torch.int32 and context_lens.dtype == torch.int32 and (cu_seqlens_q is None or cu_seqlens_q.dtype == torch.int32)
    batch = context_lens.numel()
    out = torch.empty(n, t, dim, dtype=h.dtype, device=h.device)
    _hip.call("nvh_token_shift_mix", h.data_ptr(), h.stride(0), state.data_ptr(), slots.data_ptr(), _p(cu_seqlens_q), context_lens.data_ptr(), batch,
              mu.data_ptr(), out.data_ptr(), t, n, dim, f, _stream())
    _hip.call("nvh_conv_state_update", h.data_ptr(), h.stride(0), state.data_ptr(), slots.data_ptr(), _p(cu_seqlens_q), context_lens.data_ptr(), batch,
              2, dim, f, _stream())
    return out


def rotary_qkv_prep(q, k, v, positions, freq, mag: float, rot_dims: int, interleaved: bool, heads: int, dim: int, vdim: int,
                    q_scale: float = 1.0, k_scale: float = 1.0):
    """fp32 (q, k, v) operands of a recurrence from projection columns, with rotary positions on the first `rot_dims` dimensions of
    every q / k head (freq fp32 [rot_dims / 2]; pairs interleaved or in halves) and q, k scaled after the rotation."""
    fl = _act_flag(q, k, v)
    t = q.shape[0]
    assert q.stride(1) == 1 and k.stride(1) == 1 and v.stride(1) == 1 and q.shape[1] == heads * dim and k.shape[1] == heads * dim and v.shape[1] == heads * vdim
    assert positions.dtype == torch.int64 and (rot_dims == 0 or (freq.dtype == F32 and freq.numel() * 2 == rot_dims and freq.is_cuda))
    oq, ok = (torch.empty(t, heads * dim, dtype=F32, device=q.device) for _ in range(2))
    ov = torch.empty(t, heads * vdim, dtype=F32, device=q.device)
    _hip.call("nvh_rotary_qkv_prep", q.data_ptr(), q.stride(0), k.data_ptr(), k.stride(0), v.data_ptr(), v.stride(0), positions.data_ptr(), _p(freq),
              float(mag), rot_dims, int(interleaved), float(q_scale), float(k_scale), oq.data_ptr(), ok.data_ptr(), ov.data_ptr(), t, heads, dim, vdim,
              fl, _stream())
    return oq, ok, ov


def ssd_conv_prep(xbc, dt, conv_w, conv_b, dt_bias, a_log, conv_state, slots, cu_seqlens_q, context_lens, heads: int, inner: int, gn: int):
    """Causal convolution + silu over the channels x | B | C of the in-projection (continued from `conv_state`
    [slots, taps - 1, C] fp32, which is then brought up to date), dt = softplus(dt + dt_bias), decay = exp(-exp(a_log) dt):
    fp32 (x [T, inner], B [T, gn], C [T, gn], dt [T, H], decay [T, H])."""
    fl = _act_flag(xbc, dt, conv_w, dt_bias, a_log)
    t, c = xbc.shape[0], inner + 2 * gn
    taps = conv_w.shape[1]
    assert xbc.shape[1] == c and xbc.stride(1) == 1 and dt.shape == (t, heads) and dt.stride(1) == 1 and conv_w.shape == (c, taps) and conv_w.is_contiguous()
    assert conv_b is None or (conv_b.numel() == c and conv_b.dtype == conv_w.dtype)
    assert taps == 1 or (conv_state.dtype == F32 and conv_state.is_contiguous() and tuple(conv_state.shape[1:]) == (taps - 1, c))
    assert slots.dtype == torch.int32 and context_lens.dtype == torch.int32 and (cu_seqlens_q is None or cu_seqlens_q.dtype == torch.int32)
    batch = context_lens.numel()
    ox = torch.empty(t, inner, dtype=F32, device=xbc.device)
    ob, oc = (torch.empty(t, gn, dtype=F32, device=xbc.device) for _ in range(2))
    odt, odecay = (torch.empty(t, heads, dtype=F32, device=xbc.device) for _ in range(2))
    _hip.call("nvh_ssd_conv_prep", xbc.data_ptr(), xbc.stride(0), dt.data_ptr(), dt.stride(0), conv_w.data_ptr(), _p(conv_b), dt_bias.data_ptr(),
              a_log.data_ptr(), _p(conv_state), slots.data_ptr(), _p(cu_seqlens_q), context_lens.data_ptr(), batch, t, taps, heads, inner, gn,
              ox.data_ptr(), ob.data_ptr(), oc.data_ptr(), odt.data_ptr(), odecay.data_ptr(), fl, _stream())
    _hip.call("nvh_conv_state_update", xbc.data_ptr(), xbc.stride(0), _p(conv_state), slots.data_ptr(), _p(cu_seqlens_q), context_lens.data_ptr(), batch,
              taps, c, fl, _stream())
    return ox, ob, oc, odt, odecay


def group_rmsnorm_gate(o: torch.Tensor, weight: torch.Tensor | None, group_size: int, eps: float, gate=None, gate_act: str | None = None,
                       gate_first: bool = False, out_dtype=None) -> torch.Tensor:
    """RMS norm of fp32 rows over groups of `group_size` columns, times `weight` ([group_size], shared by the groups, or one per
    column), with an optional gate (columns of the activation type; "sigmoid" or "silu") applied before or after the norm."""
    typed = [t for t in (weight, gate) if t is not None]
    assert typed or out_dtype is not None, "without a weight and a gate the result's type must be named"
    f = _act_flag(*typed) if typed else int(out_dtype == F32)
    rows, n = o.shape
    assert o.dtype == F32 and o.is_contiguous() and n % group_size == 0
    assert weight is None or (weight.numel() in (group_size, n) and weight.is_contiguous())
    assert gate is None or (gate.shape == (rows, n) and gate.stride(1) == 1 and gate_act in ("sigmoid", "silu"))
    y = torch.empty(rows, n, dtype=typed[0].dtype if typed else out_dtype, device=o.device)
    _hip.call("nvh_group_rmsnorm_gate", o.data_ptr(), _p(weight), int(weight is not None and weight.numel() == n and n != group_size), _p(gate),
              gate.stride(0) if gate is not None else 0, {None: 0, "sigmoid": 1, "silu": 2}[gate_act if gate is not None else None], int(gate_first),
              y.data_ptr(), n, rows, n // group_size, group_size, float(eps), f, _stream())
    return y


# ---------------------------------------------------------------- mixture of experts
def moe_route(logits: torch.Tensor, top: int):
    """(ids int32 [T, top], weights fp32 [T, top]): the `top` largest fp32 router logits per token, softmax over them alone."""
    assert logits.dtype == F32 and logits.dim() == 2 and logits.stride(1) == 1 and logits.is_cuda
    t, e = logits.shape
    ids = torch.empty(t, top, dtype=torch.int32, device=logits.device)
    weights = torch.empty(t, top, dtype=F32, device=logits.device)
    _hip.call("nvh_moe_route", logits.data_ptr(), logits.stride(0), ids.data_ptr(), weights.data_ptr(), t, e, top, _stream())
    return ids, weights


def moe_route_linear(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None, top: int, want_logits: bool = False, sigmoid_scores: bool = False):
    """moe_route of the fp32 logits x @ weight^T + bias, formed inside the same launch: (ids, weights[, logits]).  `sigmoid_scores`: the
    weights are the picked experts' own sigmoid(logit), not renormalised."""
    f = _act_flag(x, weight) if bias is None else _act_flag(x, weight, bias)
    t, k = x.shape
    e = weight.shape[0]
    assert x.stride(1) == 1 and weight.is_contiguous() and weight.shape[1] == k and (bias is None or bias.numel() == e)
    ids = torch.empty(t, top, dtype=torch.int32, device=x.device)
    weights = torch.empty(t, top, dtype=F32, device=x.device)
    logits = torch.empty(t, e, dtype=F32, device=x.device) if want_logits else None
    _hip.call("nvh_moe_route_linear", x.data_ptr(), x.stride(0), weight.data_ptr(), _p(bias), ids.data_ptr(), weights.data_ptr(), _p(logits), t, e, k, top,
              int(sigmoid_scores), f, _stream())
    return (ids, weights, logits) if want_logits else (ids, weights)


def moe_align(ids: torch.Tensor, experts: int) -> dict:
    """The (token, choice) pairs ordered by expert, as device arrays (see nvh_moe_align): src_token, pos_of_pair, and the tile list."""
    assert ids.dtype == torch.int32 and ids.is_contiguous() and ids.is_cuda
    t, top = ids.shape
    pairs = t * top
    max_tiles = int(_hip.lib().nvh_moe_max_tiles(pairs, experts))
    buf = torch.empty(2 * pairs + 3 * max_tiles, dtype=torch.int32, device=ids.device)
    src, pos = buf[:pairs], buf[pairs:2 * pairs]
    te, t0, tr = (buf[2 * pairs + i * max_tiles:2 * pairs + (i + 1) * max_tiles] for i in range(3))
    _hip.call("nvh_moe_align", ids.data_ptr(), t, experts, top, src.data_ptr(), pos.data_ptr(), te.data_ptr(), t0.data_ptr(), tr.data_ptr(), max_tiles, _stream())
    return dict(src_token=src, pos_of_pair=pos, tile_expert=te, tile_row0=t0, tile_rows=tr, max_tiles=max_tiles, pairs=pairs)


def linear_grouped(x: torch.Tensor, weight: torch.Tensor, plan: dict, gather: bool, out_f32: bool = False) -> torch.Tensor:
    """y[pos] = x[src_token[pos] if gather else pos] @ weight[expert of pos]^T for every position of the plan; weight [E, N, K]."""
    f = _act_flag(x, weight)
    e, n, k = weight.shape
    assert weight.is_contiguous() and x.dim() == 2 and x.shape[1] == k and x.stride(1) == 1 and (gather or x.shape[0] == plan["pairs"])
    out_f32 = bool(out_f32 or f)
    y = torch.empty(plan["pairs"], n, dtype=F32 if out_f32 else BF16, device=x.device)
    _hip.call("nvh_gemm_grouped_any_nt", x.data_ptr(), x.stride(0), plan["src_token"].data_ptr() if gather else 0, weight.data_ptr(), y.data_ptr(), n,
              plan["tile_expert"].data_ptr(), plan["tile_row0"].data_ptr(), plan["tile_rows"].data_ptr(), plan["max_tiles"], n, k, f, int(out_f32), _stream())
    return y


def glu_clamp_pairs(gate_up: torch.Tensor, plan: dict, weights: torch.Tensor | None, limit: float, alpha: float = 1.702) -> torch.Tensor:
    """The experts' activation over the rows [G | U] of the first grouped product where a pair's routing weight w (fp32 [T, top]; None:
    1) multiplies the expert's input: g = min(w G, limit), u = clamp(w U, -limit, limit), y = g sigmoid(alpha g) (u + 1)."""
    f = _act_flag(gate_up)
    pairs, inter = gate_up.shape[0], gate_up.shape[1] // 2
    assert gate_up.dim() == 2 and gate_up.stride(1) == 1 and pairs == plan["pairs"] and (weights is None or (weights.dtype == F32 and weights.is_contiguous() and weights.numel() == pairs))
    y = torch.empty(pairs, inter, dtype=gate_up.dtype, device=gate_up.device)
    _hip.call("nvh_glu_clamp_pairs", gate_up.data_ptr(), gate_up.stride(0), plan["pos_of_pair"].data_ptr(), _p(weights), y.data_ptr(), inter, pairs, inter,
              float(limit), float(alpha), f, _stream())
    return y


def moe_combine(y: torch.Tensor, plan: dict, weights: torch.Tensor | None, shared: torch.Tensor | None = None, shared_gate: torch.Tensor | None = None,
                top: int | None = None) -> torch.Tensor:
    """fp32 [T, dim]: every token's weighted sum of its choices' rows of y (in choice order), plus `shared` [T, dim], which is
    multiplied by sigmoid(shared_gate[t]) when a gate logit per token (fp32 [T] or a column view) is given.  weights None (then
    `top` says how many choices a token has): a plain sum."""
    f = _act_flag(y) if shared is None else _act_flag(y, shared)
    t, top = weights.shape if weights is not None else (plan["pairs"] // top, top)
    dim = y.shape[1]
    assert y.stride(1) == 1 and (weights is None or (weights.dtype == F32 and weights.is_contiguous())) and y.shape[0] == t * top
    assert shared is None or (shared.shape == (t, dim) and shared.stride(1) == 1)
    assert shared_gate is None or (shared is not None and shared_gate.dtype == F32 and shared_gate.numel() == t and shared_gate.is_cuda)
    out = torch.empty(t, dim, dtype=F32, device=y.device)
    _hip.call("nvh_moe_combine", y.data_ptr(), y.stride(0), plan["pos_of_pair"].data_ptr(), _p(weights), _p(shared),
              shared.stride(0) if shared is not None else 0, _p(shared_gate), shared_gate.reshape(t, -1).stride(0) if shared_gate is not None else 0,
              out.data_ptr(), t, dim, top, f, _stream())
    return out


def moe_route_scored(x: torch.Tensor, weight: torch.Tensor, top: int, correction: torch.Tensor | None = None, groups: int = 1, keep: int = 1,
                     scale: float = 1.0, aux: torch.Tensor | None = None, want_scores: bool = False):
    """Routing by softmax scores over all experts of the fp32 logits x @ weight^T: the `top` experts with the largest score +
    correction among the `keep` best of `groups` equal groups of neighbouring experts (a group's score: its largest corrected
    score), weighted by their uncorrected scores times `scale`.  `aux` [n, K]: more rows over the same input, returned as fp32
    products [T, n].  Returns (ids int32 [T, top], weights fp32 [T, top], aux products | None[, scores fp32 [T, E]])."""
    typed = [t_ for t_ in (x, weight, correction, aux) if t_ is not None]
    f = _act_flag(*typed)
    t, k = x.shape
    e = weight.shape[0]
    assert x.stride(1) == 1 and weight.is_contiguous() and weight.shape[1] == k and (correction is None or (correction.numel() == e and correction.is_contiguous()))
    assert aux is None or (aux.is_contiguous() and aux.dim() == 2 and aux.shape[1] == k)
    n_aux = 0 if aux is None else aux.shape[0]
    ids = torch.empty(t, top, dtype=torch.int32, device=x.device)
    weights = torch.empty(t, top, dtype=F32, device=x.device)
    aux_out = torch.empty(t, n_aux, dtype=F32, device=x.device) if n_aux else None
    scores = torch.empty(t, e, dtype=F32, device=x.device) if want_scores else None
    _hip.call("nvh_moe_route_scored", x.data_ptr(), x.stride(0), weight.data_ptr(), _p(correction), _p(aux), _p(aux_out), n_aux, ids.data_ptr(),
              weights.data_ptr(), _p(scores), t, e, k, top, int(groups), int(keep), float(scale), f, _stream())
    return (ids, weights, aux_out, scores) if want_scores else (ids, weights, aux_out)


# ---------------------------------------------------------------- attention through a low-rank latent
def latent_prep(proj, q_rank: int, kv_rank: int, rot_dim: int, heads: int, q_norm, kv_norm, eps: float, positions, freq, mag: float,
                interleaved: bool, k_cache, v_cache, slot_mapping, gated: bool = True):
    """(normed query latent [T, q_rank], sigmoid gate fp32 [T, H] | None) from the fused projection rows [dq | dkv | gate]; with caches given
    (a layer that owns its latent) the normed key/value latent and the rotated shared key part go to the tokens' slots: keys
    [pages, page, 1, kv_rank + rot_dim], values [pages, 1, kv_rank, page].  Without caches the row is [dq | gate]."""
    own = k_cache is not None
    typed = [x for x in (proj, q_norm, kv_norm, k_cache, v_cache) if x is not None]
    f = _act_flag(*typed)
    t = proj.shape[0]
    assert proj.stride(1) == 1 and positions.dtype == torch.int64 and q_norm.numel() == q_rank
    page = 1
    if own:
        assert slot_mapping.dtype == torch.int32 and slot_mapping.numel() == t and kv_norm.numel() == kv_rank
        assert k_cache.is_contiguous() and v_cache.is_contiguous() and k_cache.dim() == 4 and tuple(k_cache.shape[2:]) == (1, kv_rank + rot_dim)
        assert tuple(v_cache.shape) == (k_cache.shape[0], 1, kv_rank, k_cache.shape[1])
        assert rot_dim == 0 or (freq.dtype == F32 and freq.numel() * 2 == rot_dim)
        page = k_cache.shape[1]
    cq = torch.empty(t, q_rank, dtype=proj.dtype, device=proj.device)
    gate = torch.empty(t, heads, dtype=F32, device=proj.device) if gated else None
    _hip.call("nvh_latent_prep", proj.data_ptr(), proj.stride(0), q_rank, kv_rank, rot_dim, heads, int(own), q_norm.data_ptr(), _p(kv_norm), float(eps),
              positions.data_ptr(), _p(freq), float(mag), int(interleaved), cq.data_ptr(), _p(gate), _p(k_cache), _p(v_cache), _p(slot_mapping), page,
              t, f, _stream())
    return cq, gate


def linear_heads(x: torch.Tensor, weight: torch.Tensor, x_head_stride: int, out: torch.Tensor | None = None, out_head_stride: int | None = None) -> torch.Tensor:
    """y[t, h, :] = x[t, h x_head_stride : + K] @ weight[h]^T for every head; weight [H, N, K].  `out` (rows of at least H heads of
    `out_head_stride` elements; default a new [T, H * N]) receives head h's N results at column h * out_head_stride."""
    f = _act_flag(x, weight)
    heads, n, k = weight.shape
    t = x.shape[0]
    assert weight.is_contiguous() and x.dim() == 2 and x.stride(1) == 1 and x.shape[1] >= (heads - 1) * x_head_stride + k
    if out is None:
        out, out_head_stride = torch.empty(t, heads * n, dtype=x.dtype, device=x.device), n
    assert out.dtype == x.dtype and out.stride(1) == 1 and out.shape[0] == t and out.shape[1] >= (heads - 1) * out_head_stride + n
    _hip.call("nvh_gemm_heads_nt", x.data_ptr(), x.stride(0), x_head_stride, weight.data_ptr(), out.data_ptr(), out.stride(0), out_head_stride, t, heads, n, k,
              f, _stream())
    return out


def latent_q_rotary(q: torch.Tensor, positions, freq, mag: float, interleaved: bool, out: torch.Tensor, heads: int, dim: int, rot_dim: int,
                    out_head: int, out_offset: int) -> None:
    """out[t, h, out_offset + d] = rotary(q[t, h, dim + d]) for d < rot_dim; q rows [H, dim + rot_dim], out rows [H, out_head]."""
    f = _act_flag(q, out)
    assert q.stride(1) == 1 and out.stride(1) == 1 and positions.dtype == torch.int64 and (rot_dim == 0 or (freq.dtype == F32 and freq.numel() * 2 == rot_dim))
    _hip.call("nvh_latent_q_rotary", q.data_ptr(), q.stride(0), positions.data_ptr(), _p(freq), float(mag), int(interleaved), out.data_ptr(), out.stride(0),
              q.shape[0], heads, dim, rot_dim, out_head, out_offset, f, _stream())
