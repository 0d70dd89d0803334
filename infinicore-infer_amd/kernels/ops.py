"""Python face of the HIP kernels: one function per kernel.  Each checks on the
host that shapes, dtypes and strides are what the kernel and its grid assume,
then launches on torch's current stream.  Nothing here computes on the CPU.
"""
import torch

from .lib import IcResidualNorm, IcRowFactor, KernelError, check, get_lib

F32, BF16 = 0, 1
_DT = {torch.float32: F32, torch.bfloat16: BF16}


def dtype_code(dt) -> int:
    try:
        return _DT[dt]
    except KeyError:
        raise KernelError("dtype %s is not supported by the kernels (float32, bfloat16)" % dt)


_scoped_stream = None


class stream_scope:
    """Looks torch's current stream up once and uses it for every launch inside the ``with`` block
    (the lookup costs about as much as a launch).  Do not switch streams inside the block."""

    def __enter__(self):
        global _scoped_stream
        self._outer = _scoped_stream
        _scoped_stream = torch.cuda.current_stream().cuda_stream
        return self

    def __exit__(self, *exc):
        global _scoped_stream
        _scoped_stream = self._outer
        return False


def _stream():
    return _scoped_stream if _scoped_stream is not None else torch.cuda.current_stream().cuda_stream


def current_stream():
    """The stream the kernels launch on (the scoped one inside ``stream_scope``)."""
    return _stream()


def _need(cond, what):
    if not cond:
        raise KernelError(what)


def _dev(*ts):
    for t in ts:
        if t is not None and not t.is_cuda:
            raise KernelError("kernel operands must be on the GPU (got a %s tensor)" % t.device)


def _i32(t, name):
    _need(t.dtype == torch.int32 and t.is_contiguous(), "%s must be a contiguous int32 tensor" % name)


def embed(tokens, table, out, scale: float):
    """out[t, :] = table[tokens[t], :] * scale; out is float32 [T, d]."""
    _dev(tokens, table, out)
    _i32(tokens, "tokens")
    T, d = out.shape
    _need(tokens.numel() == T and table.dim() == 2 and table.shape[1] == d, "embed: shape mismatch")
    _need(out.dtype == torch.float32 and out.is_contiguous() and table.is_contiguous(), "embed: layout")
    check(get_lib().ic_embed(tokens.data_ptr(), table.data_ptr(), dtype_code(table.dtype), out.data_ptr(),
                             T, d, float(scale), _stream()), "embed")
    return out


def rmsnorm(x, weight, out, eps: float, out_scale: float = 1.0, rows=None):
    """out[r] = x[rows[r] or r] * rsqrt(mean(x^2) + eps) * weight * out_scale.  x is float32."""
    _dev(x, weight, out, rows)
    d = x.shape[-1]
    n = out.shape[0]
    _need(x.dtype == torch.float32 and x.is_contiguous() and out.is_contiguous(), "rmsnorm: layout")
    _need(weight.dtype == torch.float32 and weight.numel() == d and out.shape[-1] == d, "rmsnorm: shape mismatch")
    if rows is not None:
        _i32(rows, "rows")
        _need(rows.numel() == n, "rmsnorm: rows/out mismatch")
    else:
        _need(x.shape[0] == n, "rmsnorm: x/out mismatch")
    check(get_lib().ic_rmsnorm(x.data_ptr(), rows.data_ptr() if rows is not None else None, weight.data_ptr(),
                               out.data_ptr(), dtype_code(out.dtype), n, d, float(eps), float(out_scale),
                               _stream()), "rmsnorm")
    return out


def add_rmsnorm(x, y, alpha: float, weight, out, eps: float):
    """x += alpha * y (x float32, in place); out = rmsnorm(x) * weight."""
    _dev(x, y, weight, out)
    T, d = x.shape
    _need(x.dtype == torch.float32 and x.is_contiguous() and y.is_contiguous() and out.is_contiguous(),
          "add_rmsnorm: layout")
    _need(tuple(y.shape) == (T, d) and tuple(out.shape) == (T, d) and weight.numel() == d
          and weight.dtype == torch.float32, "add_rmsnorm: shape mismatch")
    check(get_lib().ic_add_rmsnorm(x.data_ptr(), y.data_ptr(), dtype_code(y.dtype), float(alpha),
                                   weight.data_ptr(), out.data_ptr(), dtype_code(out.dtype), T, d,
                                   float(eps), _stream()), "add_rmsnorm")
    return out


def residual_add(x, y, alpha: float):
    """x += alpha * y; x float32."""
    _dev(x, y)
    _need(x.dtype == torch.float32 and x.is_contiguous() and y.is_contiguous() and x.shape == y.shape,
          "residual_add: layout")
    check(get_lib().ic_residual_add(x.data_ptr(), y.data_ptr(), dtype_code(y.dtype), float(alpha),
                                    x.numel(), _stream()), "residual_add")
    return x


def swiglu(gate_up, out):
    """out[t, j] = up * silu(gate), gate = gate_up[t, j], up = gate_up[t, di + j]."""
    _dev(gate_up, out)
    T, di = out.shape
    _need(tuple(gate_up.shape) == (T, 2 * di) and gate_up.is_contiguous() and out.is_contiguous()
          and gate_up.dtype == out.dtype, "swiglu: layout")
    check(get_lib().ic_swiglu(gate_up.data_ptr(), out.data_ptr(), dtype_code(out.dtype), T, di, _stream()),
          "swiglu")
    return out


def glu_clamped(gate_up, out, limit: float, alpha: float):
    """out[t, j] = g * sigmoid(alpha * g) * (u + 1) with g = min(gate_up[t, j], limit) and
    u = clamp(gate_up[t, di + j], -limit, limit)."""
    _dev(gate_up, out)
    T, di = out.shape
    _need(tuple(gate_up.shape) == (T, 2 * di) and gate_up.is_contiguous() and out.is_contiguous()
          and gate_up.dtype == out.dtype, "glu_clamped: layout")
    _need(limit > 0, "glu_clamped: the limit must be positive")
    check(get_lib().ic_glu_clamped(gate_up.data_ptr(), out.data_ptr(), dtype_code(out.dtype), T, di, float(limit),
                                   float(alpha), _stream()), "glu_clamped")
    return out


def copy_pages(planes, src, dst):
    """planes[..., dst[i], :, :, :] = planes[..., src[i], :, :, :] for a cache group's planes
    [slots, planes, pages, kv_heads, page_size, head_dim] (contiguous); src, dst: int32 page ids on the device."""
    _dev(planes, src, dst)
    _i32(src, "src")
    _i32(dst, "dst")
    _need(planes.dim() == 6 and planes.is_contiguous() and src.numel() == dst.numel(), "copy_pages: layout")
    n_pages = planes.shape[2]
    page_bytes = planes.shape[3] * planes.shape[4] * planes.shape[5] * planes.element_size()
    check(get_lib().ic_copy_pages(planes.data_ptr(), planes.shape[0] * planes.shape[1], n_pages, page_bytes,
                                  src.data_ptr(), dst.data_ptr(), src.numel(), _stream()), "copy_pages")


def rope_kv_write(qkv, positions, cos, sin, kcache, vcache, slots, n_heads, n_kv_heads, head_dim,
                  rot_dim, page_size):
    """Rotate the q heads of qkv[T, H] in place; rotate the k heads and copy the
    v heads into cache slot ``slots[t]``.  n_kv_heads == 0: q only, no cache write."""
    _dev(qkv, positions, cos, sin, kcache, vcache, slots)
    T = qkv.shape[0]
    _i32(positions, "positions")
    _need(qkv.dim() == 2 and qkv.stride(1) == 1, "rope: qkv must be [T, H] with unit inner stride")
    _need(qkv.shape[1] >= (n_heads + 2 * n_kv_heads) * head_dim, "rope: qkv row too short")
    _need(positions.numel() == T, "rope: positions/qkv mismatch")
    half = rot_dim // 2
    if rot_dim > 0:
        _need(cos.dtype == torch.float32 and sin.dtype == torch.float32 and cos.is_contiguous()
              and sin.is_contiguous() and cos.shape[-1] == half and sin.shape == cos.shape,
              "rope: cos/sin must be float32 [max_pos, rot/2]")
    if n_kv_heads > 0:
        _i32(slots, "slots")
        _need(slots.numel() == T, "rope: slots/qkv mismatch")
        _need(kcache.dtype == qkv.dtype and vcache.dtype == qkv.dtype, "rope: cache dtype differs from qkv")
        _need(kcache.is_contiguous() and vcache.is_contiguous()
              and tuple(kcache.shape[1:]) == (n_kv_heads, page_size, head_dim)
              and kcache.shape == vcache.shape, "rope: cache must be [pages, kv_heads, page_size, head_dim]")
    check(get_lib().ic_rope_kv_write(
        qkv.data_ptr(), dtype_code(qkv.dtype), positions.data_ptr(),
        cos.data_ptr() if rot_dim > 0 else None, sin.data_ptr() if rot_dim > 0 else None,
        kcache.data_ptr() if n_kv_heads > 0 else None, vcache.data_ptr() if n_kv_heads > 0 else None,
        slots.data_ptr() if n_kv_heads > 0 else None,
        T, qkv.stride(0), n_heads, n_kv_heads, head_dim, rot_dim, page_size, _stream()), "rope_kv_write")


def _attn_common(q, out, kcache, vcache, block_tables, n_heads, n_kv_heads, head_dim, page_size):
    _dev(q, out, kcache, vcache, block_tables)
    _need(q.dim() == 2 and q.stride(1) == 1 and q.shape[1] >= n_heads * head_dim, "attention: q layout")
    _need(out.dim() == 2 and out.stride(1) == 1 and out.shape[1] >= n_heads * head_dim, "attention: out layout")
    _need(q.dtype == out.dtype == kcache.dtype == vcache.dtype, "attention: dtypes differ")
    _need(kcache.is_contiguous() and vcache.is_contiguous() and kcache.shape == vcache.shape
          and tuple(kcache.shape[1:]) == (n_kv_heads, page_size, head_dim),
          "attention: cache must be [pages, kv_heads, page_size, head_dim]")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.stride(1) == 1,
          "attention: block_tables must be int32 [R, max_blocks]")
    _need(n_heads % n_kv_heads == 0, "attention: heads not a multiple of kv heads")


def attention_generic(q, out, kcache, vcache, block_tables, token_req, positions, n_heads, n_kv_heads,
                      head_dim, page_size, scale: float, window: int = 0):
    """out[t, h] = softmax over keys <= positions[t] (within the window) of q[t, h] . K, times V."""
    _attn_common(q, out, kcache, vcache, block_tables, n_heads, n_kv_heads, head_dim, page_size)
    _i32(token_req, "token_req")
    _i32(positions, "positions")
    T = q.shape[0]
    _need(token_req.numel() == T and positions.numel() == T and out.shape[0] == T, "attention: T mismatch")
    _need(head_dim <= 512, "attention: head size above 512")
    check(get_lib().ic_attn_generic(
        q.data_ptr(), q.stride(0), out.data_ptr(), out.stride(0), dtype_code(q.dtype), kcache.data_ptr(),
        vcache.data_ptr(), block_tables.data_ptr(), block_tables.stride(0), token_req.data_ptr(),
        positions.data_ptr(), T, n_heads, n_kv_heads, head_dim, page_size, float(scale), int(window or 0),
        _stream()), "attention_generic")


def attention_decode_supported(dtype, head_dim: int) -> bool:
    return bool(get_lib().ic_attn_decode_supported(dtype_code(dtype), head_dim))


def attention_decode_on_matrix_cores(dtype, n_heads: int, n_kv_heads: int) -> bool:
    """True when attention_decode runs its grouped-query kernel (bfloat16, several query heads per
    kv head): that kernel wants fewer key splits than the one-head-per-wave kernel (the library's rule)."""
    return bool(get_lib().ic_attn_decode_on_matrix_cores(dtype_code(dtype), int(n_heads), int(n_kv_heads)))


def attention_decode_splits(n_rows: int, n_heads: int, n_kv_heads: int, head_dim: int, elem_bytes: int, window: int,
                            max_context: int, matrix_cores: int, compute_units: int) -> int:
    """Ways to split the keys of ``n_rows`` single-token rows that see up to ``max_context`` keys (the library's
    cost model of its two kernels, fitted to sweeps)."""
    return int(get_lib().ic_attn_decode_splits(int(n_rows), int(n_heads), int(n_kv_heads), int(head_dim), int(elem_bytes),
                                               int(window or 0), int(max_context), int(bool(matrix_cores)),
                                               int(compute_units)))


def attention_decode(q, out, kcache, vcache, block_tables, tok_list, n_tok, token_req, positions, part_acc,
                     part_ml, n_heads, n_kv_heads, head_dim, page_size, scale: float, window: int, n_split: int):
    """Split-key attention of the single tokens listed in tok_list (None: rows 0..n_tok-1)."""
    _attn_common(q, out, kcache, vcache, block_tables, n_heads, n_kv_heads, head_dim, page_size)
    _i32(token_req, "token_req")
    _i32(positions, "positions")
    if tok_list is not None:
        _i32(tok_list, "tok_list")
        _need(tok_list.numel() >= n_tok, "attention_decode: tok_list too short")
    else:
        _need(q.shape[0] >= n_tok, "attention_decode: fewer rows than tokens")
    _need(part_acc.dtype == torch.float32 and part_acc.is_contiguous()
          and part_acc.numel() >= n_tok * n_heads * n_split * head_dim, "attention_decode: part_acc too small")
    _need(part_ml.dtype == torch.float32 and part_ml.is_contiguous()
          and part_ml.numel() >= n_tok * n_heads * n_split * 2, "attention_decode: part_ml too small")
    check(get_lib().ic_attn_decode(
        q.data_ptr(), q.stride(0), out.data_ptr(), out.stride(0), dtype_code(q.dtype), kcache.data_ptr(),
        vcache.data_ptr(), block_tables.data_ptr(), block_tables.stride(0),
        tok_list.data_ptr() if tok_list is not None else None, token_req.data_ptr(), positions.data_ptr(),
        part_acc.data_ptr(), part_ml.data_ptr(), n_tok, n_heads, n_kv_heads, head_dim, page_size,
        float(scale), int(window or 0), int(n_split), _stream()), "attention_decode")


def attention_prefill_supported(dtype, head_dim: int, page_size: int) -> bool:
    return bool(get_lib().ic_attn_prefill_supported(dtype_code(dtype), head_dim, page_size))


def attention_prefill_tile_rows() -> int:
    return get_lib().ic_attn_prefill_tile_rows()


def attention_prefill_parts(n_tiles: int, n_heads: int, head_dim: int, max_keys: int, compute_units: int):
    """(parts, part_len): into how many blocks of their own to cut the query tiles' walks over the keys when the longest
    tile of the step sees ``max_keys`` keys (1: no cut), and how many key tiles of 64 a part holds at least."""
    import ctypes
    part_len = ctypes.c_int(0)
    parts = get_lib().ic_attn_prefill_parts(int(n_tiles), int(n_heads), int(head_dim), int(max_keys), int(compute_units),
                                            ctypes.byref(part_len))
    return int(parts), int(part_len.value)


def attention_prefill_parts_of_step(dtype, n_tiles: int, n_heads: int, head_dim: int, max_position: int, window: int, compute_units: int):
    """(parts, part_len) for a step whose largest position is ``max_position`` under a mixer's ``window`` (0: none);
    float32 walks are never cut."""
    import ctypes
    part_len = ctypes.c_int(0)
    parts = get_lib().ic_attn_prefill_parts_of_step(dtype_code(dtype), int(n_tiles), int(n_heads), int(head_dim), int(max_position), int(window or 0),
                                                    int(compute_units), ctypes.byref(part_len))
    return int(parts), int(part_len.value)


def attention_prefill_counter_ints() -> int:
    return int(get_lib().ic_attn_prefill_counter_ints())


def attention_prefill_scratch_floats(n_tiles: int, n_heads: int, head_dim: int, parts: int) -> int:
    return int(get_lib().ic_attn_prefill_scratch_floats(int(n_tiles), int(n_heads), int(head_dim), int(parts)))


def attention_prefill(q, out, kcache, vcache, block_tables, tiles, n_tiles, n_heads, n_kv_heads, head_dim,
                      page_size, scale: float, window: int = 0, groups: int = 0, parts: int = 1, part_len: int = 0,
                      scratch=None, counters=None):
    """Matrix-core attention of prompt portions.  tiles: int32 [n, 4] rows of
    (request row in block_tables, first token row, rows <= tile_rows, first position).
    groups: wave groups per query tile (1 or 2); 0 lets the kernel choose from the number of blocks.
    parts > 1: every tile's walk over the keys is cut into up to ``parts`` blocks of at least ``part_len`` key tiles
    that meet through ``scratch`` (float32, attention_prefill_scratch_floats(...) elements) and count themselves in at
    ``counters`` (int32, attention_prefill_counter_ints() elements, zero before the first launch; every launch leaves them
    zero; launches that overlap in time need counters of their own)."""
    _need(groups in (0, 1, 2), "attention_prefill: groups must be 0, 1 or 2")
    _attn_common(q, out, kcache, vcache, block_tables, n_heads, n_kv_heads, head_dim, page_size)
    _need(tiles.dtype == torch.int32 and tiles.is_contiguous() and tiles.dim() == 2 and tiles.shape[1] == 4
          and tiles.shape[0] >= n_tiles, "attention_prefill: tiles must be int32 [n, 4]")
    if parts > 1:
        _dev(scratch)
        _dev(counters)
        _need(scratch is not None and scratch.dtype == torch.float32 and scratch.is_contiguous(),
              "attention_prefill: a cut walk needs float32 scratch memory")
        _need(counters is not None and counters.dtype == torch.int32 and counters.is_contiguous()
              and counters.numel() >= attention_prefill_counter_ints(), "attention_prefill: a cut walk needs its int32 arrival counters")
    check(get_lib().ic_attn_prefill_split(
        q.data_ptr(), q.stride(0), out.data_ptr(), out.stride(0), dtype_code(q.dtype), kcache.data_ptr(),
        vcache.data_ptr(), block_tables.data_ptr(), block_tables.stride(0), tiles.data_ptr(), n_tiles,
        n_heads, n_kv_heads, head_dim, page_size, float(scale), int(window or 0), int(groups), int(parts), int(part_len),
        scratch.data_ptr() if parts > 1 else None, scratch.numel() if parts > 1 else 0,
        counters.data_ptr() if parts > 1 else None, _stream()),
        "attention_prefill")


def sample(logits, out, temperature=None, top_k=None, top_p=None, uniform=None):
    """out[r] = token sampled from logits[r] (float32 [R, V]).  temperature None: argmax."""
    _dev(logits, out, temperature, top_k, top_p, uniform)
    R, V = logits.shape
    _need(logits.dtype == torch.float32 and logits.stride(1) == 1, "sample: logits must be float32 rows")
    _i32(out, "out")
    _need(out.numel() >= R, "sample: out too short")
    if temperature is not None:
        _need(temperature.dtype == torch.float32 and top_p.dtype == torch.float32
              and uniform.dtype == torch.float32 and top_k.dtype == torch.int32, "sample: parameter dtypes")
        _need(min(temperature.numel(), top_k.numel(), top_p.numel(), uniform.numel()) >= R,
              "sample: parameter arrays too short")
    p = lambda t: t.data_ptr() if t is not None else None
    check(get_lib().ic_sample(logits.data_ptr(), logits.stride(0), R, V, p(temperature), p(top_k), p(top_p),
                              p(uniform), out.data_ptr(), _stream()), "sample")
    return out


def argmax(logits, out, scratch_val, scratch_idx):
    """out[r] = index of the largest logit of row r (the lowest index among equals), in two
    stages; scratch_val float32 and scratch_idx int32 of at least 64 * rows elements."""
    _dev(logits, out, scratch_val, scratch_idx)
    R, V = logits.shape
    _need(logits.dtype == torch.float32 and logits.stride(1) == 1, "argmax: logits must be float32 rows")
    _i32(out, "out")
    _i32(scratch_idx, "scratch_idx")
    _need(out.numel() >= R and scratch_val.dtype == torch.float32 and scratch_val.is_contiguous()
          and scratch_val.numel() >= 64 * R and scratch_idx.numel() >= 64 * R, "argmax: buffers too small")
    check(get_lib().ic_argmax(logits.data_ptr(), logits.stride(0), R, V, scratch_val.data_ptr(),
                              scratch_idx.data_ptr(), out.data_ptr(), _stream()), "argmax")
    return out


def argmax_static(logits, out):
    """argmax with the library's own static scratch memory: allocates nothing, takes at most
    ``get_lib().ic_argmax_static_max_rows()`` rows; calls that overlap on one GPU race."""
    _dev(logits, out)
    R, V = logits.shape
    _need(logits.dtype == torch.float32 and logits.stride(1) == 1, "argmax_static: logits must be float32 rows")
    _i32(out, "out")
    _need(out.numel() >= R, "argmax_static: out too short")
    check(get_lib().ic_argmax_static(logits.data_ptr(), logits.stride(0), R, V, out.data_ptr(), _stream()),
          "argmax_static")
    return out


def gemm_nt_supported(a_dtype, w_dtype, c_dtype) -> bool:
    try:
        return bool(get_lib().ic_gemm_nt_supported(dtype_code(a_dtype), dtype_code(w_dtype), dtype_code(c_dtype)))
    except KernelError:
        return False


# ---- which kernel takes what: the library's rules, shared with its native step function ----------------------------
TAIL_PLAIN, TAIL_SPLIT_NORM, TAIL_SLICES = 0, 1, 2
ATTN_GENERAL, ATTN_SINGLE_TOKENS, ATTN_PORTIONS = 0, 1, 2


def _code_or_none(dt):
    return _DT.get(dt)


def rule_own_product(a_dtype, w_dtype, c_dtype, rows: int) -> bool:
    """True when a plain product of ``rows`` rows runs in the package's own kernel (gemm_nt), not in the library."""
    codes = (_code_or_none(a_dtype), _code_or_none(w_dtype), _code_or_none(c_dtype))
    return None not in codes and bool(get_lib().ic_rule_own_product(codes[0], codes[1], codes[2], int(rows)))


def rule_qkv_fused(dtype, rows: int, a, w, head_dim: int, rot_dim: int, kv_heads_written: int, row_factors_owed: bool) -> bool:
    """True when the QKV projection of a[rows, K] with w runs with rotary and cache write in its epilogue."""
    code = _code_or_none(dtype)
    return code is not None and bool(get_lib().ic_rule_qkv_fused(code, int(rows), int(a.shape[1]), int(a.stride(0)), int(w.stride(0)),
                                                                 int(head_dim), int(rot_dim), int(kv_heads_written),
                                                                 int(bool(row_factors_owed))))


def rule_gate_up_fused(dtype, rows: int, a, w, row_factors_owed: bool) -> bool:
    """True when the gate/up projection of a[rows, K] with w runs with SwiGLU in its epilogue."""
    code = _code_or_none(dtype)
    return code is not None and bool(get_lib().ic_rule_gate_up_fused(code, int(rows), int(a.shape[1]), int(a.stride(0)),
                                                                     int(w.stride(0)), int(bool(row_factors_owed))))


def rule_tail(dtype, a, w) -> int:
    """How the projection a w^T into the residual stream, followed by a norm, runs: TAIL_PLAIN, TAIL_SPLIT_NORM or TAIL_SLICES."""
    code = _code_or_none(dtype)
    if code is None or a.dtype != dtype or w.dtype != dtype:
        return TAIL_PLAIN
    return int(get_lib().ic_rule_tail(code, int(a.shape[0]), int(w.shape[0]), int(a.shape[1]), int(a.stride(0)), int(w.stride(0))))


def rule_attention(dtype, head_dim: int, page_size: int, n_decode_rows: int, n_tiles: int) -> int:
    """ATTN_GENERAL, or the bits ATTN_SINGLE_TOKENS and ATTN_PORTIONS: which attention kernels a step takes."""
    return int(get_lib().ic_rule_attention(dtype_code(dtype), int(head_dim), int(page_size), int(n_decode_rows), int(n_tiles)))


def rule_context_bucket(n_keys: int) -> int:
    """The key count that the key split of single-token rows is chosen for (rounded up, so that a recorded step
    serves a range of lengths and splits as an eager one does)."""
    return int(get_lib().ic_rule_context_bucket(int(n_keys)))


def max_sumsq_parts() -> int:
    """Column blocks of sums of squares a product can take as row factors."""
    return int(get_lib().ic_rule_sumsq_parts_max())


def residual_parts(n: int) -> int:
    """Column blocks of sums of squares that gemm_nt(..., residual=...) writes for an n wide product."""
    return int(get_lib().ic_gemm_nt_residual_parts(int(n)))


def _row_factor(row_factor, M, what):
    """row_factor = (sumsq float32 [n_parts, 16], width, eps) -> the C struct (or None)."""
    if row_factor is None:
        return None
    sumsq, width, eps = row_factor
    _dev(sumsq)
    _need(M <= 16, what + ": row factors need at most 16 rows")
    _need(sumsq.dtype == torch.float32 and sumsq.is_contiguous() and sumsq.dim() == 2 and sumsq.shape[1] == 16
          and 0 < sumsq.shape[0] <= max_sumsq_parts(), what + ": sums of squares must be float32 [<= 256, 16]")
    _need(width > 0, what + ": width")
    return IcRowFactor(sumsq.data_ptr(), sumsq.shape[0], int(width), float(eps))


def gemm_epilogue_rows(kind: str, a, w) -> int:
    """Rows that the product with the ``kind`` epilogue ("swiglu", or "rope" for gemm_qkv_rope) takes for these operands: 32
    where the weights can be read in whole cache lines, 16 otherwise (and above 16 rows without row factors)."""
    return int(get_lib().ic_gemm_nt_epilogue_rows({"swiglu": 1, "rope": 2}[kind], int(a.shape[1]), int(a.stride(0)), int(w.stride(0))))


def gemm_nt(a, w, out, alpha: float = 1.0, swiglu_output: bool = False, row_factor=None, residual=None, whole_lines: bool = True,
            activation=None, glu_clamped=None):
    """out[M, N] = alpha * a[M, K] @ w[N, K]^T (bfloat16 operands, float32 accumulation).
    swiglu_output (M <= gemm_epilogue_rows("swiglu", a, w)): w = [gate rows; up rows] and out[M, N/2] = up * silu(gate).
    row_factor = (sumsq [n_parts, 16], width, eps), M <= 16: row m of the product is first multiplied by
    rsqrt(sumsq[:, m].sum() / width + eps), the factor an RMS norm of a's rows still owes.
    residual = (x float32 [M, N], weight float32 [N], beta, sumsq_out float32 [residual_parts(N), 16]),
    M <= 16, bfloat16 out: x += beta * (the product rounded to bfloat16); out = x * weight;
    sumsq_out[b, m] = sum of x[m]^2 over columns 16 b .. 16 b + 15.
    whole_lines False (tests): the weights are loaded in operand layout also where whole cache lines would apply.
    activation ("relu2", "gelu_tanh", "silu"; not with the other epilogues): out = act(the product as rounded to out's dtype).
    glu_clamped = (limit, slope), with swiglu_output: out = g sigmoid(slope g) (u + 1), g = min(gate, limit), u = clamp(up, -limit, limit)."""
    import ctypes
    _dev(a, w, out)
    M, K = a.shape
    N = w.shape[0]
    _need(w.shape[1] == K and tuple(out.shape) == (M, N // 2 if swiglu_output else N), "gemm_nt: shape mismatch")
    _need(not swiglu_output or (M <= 32 and N % 2 == 0), "gemm_nt: fused activation needs M <= 32 and even N")
    _need(a.stride(1) == 1 and w.stride(1) == 1 and out.stride(1) == 1, "gemm_nt: inner strides must be 1")
    rf = _row_factor(row_factor, M, "gemm_nt")
    rn = None
    mode = 1 if swiglu_output else 0
    if residual is not None:
        x, weight, beta, sumsq_out = residual
        _dev(x, weight, sumsq_out)
        _need(not swiglu_output and M <= 16 and out.dtype == torch.bfloat16, "gemm_nt: residual epilogue needs M <= 16 and bfloat16 out")
        _need(x.dtype == torch.float32 and tuple(x.shape) == (M, N) and x.stride(1) == 1, "gemm_nt: residual stream must be float32 [M, N]")
        _need(weight.dtype == torch.float32 and weight.is_contiguous() and weight.numel() == N, "gemm_nt: norm weight must be float32 [N]")
        _need(sumsq_out.dtype == torch.float32 and sumsq_out.is_contiguous()
              and tuple(sumsq_out.shape) == (residual_parts(N), 16) and residual_parts(N) <= max_sumsq_parts(),
              "gemm_nt: sumsq_out must be float32 [residual_parts(N) <= 256, 16]")
        rn = IcResidualNorm(x.data_ptr(), x.stride(0), weight.data_ptr(), float(beta), sumsq_out.data_ptr(), sumsq_out.shape[0])
        mode = 2
    if activation is not None:
        _need(mode == 0 and activation in ACTIVATIONS, "gemm_nt: an activation goes with the plain product only (have %s)" % ", ".join(sorted(ACTIVATIONS)))
        mode = 3 + ACTIVATIONS[activation]
    if glu_clamped is not None:
        _need(swiglu_output and whole_lines and alpha == 1.0, "gemm_nt: the bounded gated unit is an epilogue of the gate/up product")
        check(get_lib().ic_gemm_nt_glu_clamped(a.data_ptr(), dtype_code(a.dtype), w.data_ptr(), dtype_code(w.dtype),
                                               out.data_ptr(), dtype_code(out.dtype), M, N, K, a.stride(0), w.stride(0),
                                               out.stride(0), float(glu_clamped[0]), float(glu_clamped[1]),
                                               ctypes.byref(rf) if rf else None, _stream()), "gemm_nt")
        return out
    if not whole_lines:
        check(get_lib().ic_gemm_nt_variant(a.data_ptr(), dtype_code(a.dtype), w.data_ptr(), dtype_code(w.dtype),
                                           out.data_ptr(), dtype_code(out.dtype), M, N, K, a.stride(0), w.stride(0),
                                           out.stride(0), float(alpha), mode, ctypes.byref(rf) if rf else None,
                                           ctypes.byref(rn) if rn else None, 0, _stream()), "gemm_nt")
        return out
    check(get_lib().ic_gemm_nt(a.data_ptr(), dtype_code(a.dtype), w.data_ptr(), dtype_code(w.dtype),
                               out.data_ptr(), dtype_code(out.dtype), M, N, K, a.stride(0), w.stride(0),
                               out.stride(0), float(alpha), mode, ctypes.byref(rf) if rf else None,
                               ctypes.byref(rn) if rn else None, _stream()), "gemm_nt")
    return out


_matmul_workspace = {}
MATMUL_WORKSPACE_BYTES = 64 << 20


def _workspace(device):
    """The library's scratch memory: one buffer per device and stream, since products that run at the
    same time on different streams must not share it (some algorithms keep flags and partial sums there)."""
    key = (device, _stream())
    ws = _matmul_workspace.get(key)
    if ws is None:
        ws = _matmul_workspace[key] = torch.empty(MATMUL_WORKSPACE_BYTES, dtype=torch.uint8, device=device)
    return ws


def library_workspace(device):
    """The library products' scratch memory for the current stream on ``device``."""
    return _workspace(device)


class NoLibraryAlgorithm(KernelError):
    """The library proposes no algorithm for a product."""


_matmul_types = {}      # (operand dtype, result dtype) -> (codes) or None: asked of the library once


def _matmul_args(a, w, out, what):
    """Checks a product's operands and returns (M, N, K, operand code, result code, row strides of a, w, out).
    Written for few attribute lookups: this runs four times a layer."""
    if not (a.is_cuda and w.is_cuda and out.is_cuda):
        _dev(a, w, out)
    M, K = a.shape
    N, Kw = w.shape
    Mo, No = out.shape
    sa, sa1 = a.stride()
    sw, sw1 = w.stride()
    so, so1 = out.stride()
    if Kw != K or Mo != M or No != N:
        raise KernelError(what + ": shape mismatch")
    if sa1 != 1 or sw1 != 1 or so1 != 1:
        raise KernelError(what + ": layout")
    key = (a.dtype, w.dtype, out.dtype)
    codes = _matmul_types.get(key, False)
    if codes is False:
        codes = None
        if a.dtype == w.dtype and a.dtype in _DT and out.dtype in _DT and \
                get_lib().ic_matmul_supported(_DT[a.dtype], _DT[out.dtype]):
            codes = (_DT[a.dtype], _DT[out.dtype])
        _matmul_types[key] = codes
    if codes is None:
        raise KernelError(what + ": unsupported types")
    return M, N, K, codes[0], codes[1], sa, sw, so


def matmul_library(a, w, out, alpha: float = 1.0):
    """out[M, N] = alpha * a[M, K] @ w[N, K]^T through the library (hipBLASLt), any number of rows.
    bfloat16 operands with a bfloat16 or float32 result, or all float32."""
    M, N, K, ca, cc, sa, sw, so = _matmul_args(a, w, out, "matmul_library")
    stream = _stream()
    ws = _matmul_workspace.get((a.device, stream))
    if ws is None:
        ws = _workspace(a.device)
    st = get_lib().ic_matmul(a.data_ptr(), ca, w.data_ptr(), out.data_ptr(), cc, M, N, K, sa, sw, so, alpha,
                        ws.data_ptr(), MATMUL_WORKSPACE_BYTES, stream)
    if st == 0:
        return out
    if st == -4:
        raise NoLibraryAlgorithm("matmul_library: no algorithm for %d x %d x %d" % (M, N, K))
    if st == -3:
        raise KernelError("matmul_library: the library refused the product %d x %d x %d" % (M, N, K))
    check(st, "matmul_library")
    return out


def matmul_library_tune(a, w, out, reps: int = 5, flush=None) -> int:
    """Times the library's algorithms for this product's shape and keeps the fastest; returns how many it tried.
    flush: a device tensor larger than the chip's caches; it is overwritten before every timed launch, so that the
    algorithms are compared with operands that come from memory, as a model's weights do."""
    M, N, K, ca, cc, sa, sw, so = _matmul_args(a, w, out, "matmul_library_tune")
    ws = _workspace(a.device)
    if flush is not None:
        _dev(a, flush)
        _need(flush.is_contiguous(), "matmul_library_tune: flush must be contiguous")
    n = get_lib().ic_matmul_tune(a.data_ptr(), ca, w.data_ptr(), out.data_ptr(), cc, M, N, K, sa, sw, so,
                                 ws.data_ptr(), ws.numel(),
                                 flush.data_ptr() if flush is not None else None,
                                 flush.numel() * flush.element_size() if flush is not None else 0, int(reps), _stream())
    if n < 0:
        raise KernelError("matmul_library_tune failed with %d for %d x %d x %d" % (n, M, N, K))
    return n


def gemm_qkv_rope_supported(dtype, head_dim: int) -> bool:
    try:
        return bool(get_lib().ic_gemm_qkv_rope_supported(dtype_code(dtype), head_dim))
    except KernelError:
        return False


def gemm_qkv_rope(a, w, qkv, positions, slots, cos, sin, kcache, vcache, n_heads, n_kv_heads, head_dim, page_size,
                  row_factor=None, tile_rows: int = 0):
    """For M <= gemm_epilogue_rows("rope", a, w) rows: qkv = a @ w^T with the rotary encoding and the cache write in the epilogue.
    The q heads of qkv[M, >= n_heads * head_dim] hold rotated queries afterwards; rotated keys and
    the values are in cache slot ``slots[m]``.  Full rotary, bfloat16.  row_factor: as in gemm_nt.
    tile_rows (tests): used weight rows per tile, 16, 8 or 4; 0: chosen from the number of heads."""
    import ctypes
    _dev(a, w, qkv, positions, slots, cos, sin, kcache, vcache)
    M, K = a.shape
    _i32(positions, "positions")
    _i32(slots, "slots")
    _need(M <= 32 and positions.numel() == M and slots.numel() == M, "gemm_qkv_rope: at most 32 rows, one position and slot each")
    rf = _row_factor(row_factor, M, "gemm_qkv_rope")
    _need(tuple(w.shape) == ((n_heads + 2 * n_kv_heads) * head_dim, K), "gemm_qkv_rope: weight shape")
    _need(qkv.shape[0] == M and qkv.shape[1] >= n_heads * head_dim and qkv.stride(1) == 1
          and a.stride(1) == 1 and w.stride(1) == 1, "gemm_qkv_rope: layout")
    _need(a.dtype == w.dtype == qkv.dtype == kcache.dtype == vcache.dtype == torch.bfloat16, "gemm_qkv_rope: bfloat16 only")
    _need(cos.dtype == torch.float32 and sin.dtype == torch.float32 and cos.is_contiguous() and sin.is_contiguous()
          and cos.shape[-1] == head_dim // 2 and sin.shape == cos.shape, "gemm_qkv_rope: cos/sin must be float32 [max_pos, dh/2]")
    _need(kcache.is_contiguous() and vcache.is_contiguous() and kcache.shape == vcache.shape
          and tuple(kcache.shape[1:]) == (n_kv_heads, page_size, head_dim), "gemm_qkv_rope: cache layout")
    args = (a.data_ptr(), w.data_ptr(), qkv.data_ptr(), M, K, a.stride(0), w.stride(0), qkv.stride(0), positions.data_ptr(),
            slots.data_ptr(), cos.data_ptr(), sin.data_ptr(), kcache.data_ptr(), vcache.data_ptr(), n_heads, n_kv_heads,
            head_dim, page_size, ctypes.byref(rf) if rf else None)
    if tile_rows:
        check(get_lib().ic_gemm_qkv_rope_variant(*args, int(tile_rows), _stream()), "gemm_qkv_rope")
    else:
        check(get_lib().ic_gemm_qkv_rope(*args, _stream()), "gemm_qkv_rope")
    return qkv


# ---- products of 17..64 rows as slices over K, and what follows them -------------------------------------------
def gemm_splitk_supported(a, w) -> bool:
    return bool(a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and a.dim() == 2 and w.dim() == 2
                and a.stride(1) == 1 and w.stride(1) == 1 and a.shape[1] == w.shape[1]
                and get_lib().ic_gemm_splitk_supported(a.shape[0], w.shape[0], a.shape[1], a.stride(0), w.stride(0)))


def gemm_splitk_pays(m: int, n: int, k: int) -> bool:
    """True when the sliced product beats the library's for an m x n x k product (17..64 rows, enough blocks)."""
    return bool(get_lib().ic_gemm_splitk_pays(int(m), int(n), int(k)))


def gemm_splitk_slices(n: int, k: int) -> int:
    return int(get_lib().ic_gemm_splitk_slices(int(n), int(k)))


def gemm_splitk(a, w, parts, n_slices=None):
    """parts[s, m, n] (float32) = a[m, K_s] . w[n, K_s] for the slices K_s of K; 1..64 rows, bfloat16 operands.
    ``parts`` must hold n_slices * M * N floats; returns its [n_slices, M, N] view."""
    _dev(a, w, parts)
    M, K = a.shape
    N = w.shape[0]
    _need(gemm_splitk_supported(a, w), "gemm_splitk: at most 64 bfloat16 rows, K a multiple of 8, rows 16-byte aligned")
    S = int(n_slices) if n_slices else gemm_splitk_slices(N, K)
    _need(parts.dtype == torch.float32 and parts.is_contiguous() and parts.numel() >= S * M * N, "gemm_splitk: parts too small")
    check(get_lib().ic_gemm_splitk(a.data_ptr(), w.data_ptr(), parts.data_ptr(), M, N, K, a.stride(0), w.stride(0), S, _stream()),
          "gemm_splitk")
    return parts.view(-1)[:S * M * N].view(S, M, N)


def splitk_add_rmsnorm(parts, x, alpha: float, weight, out, eps: float):
    """x += alpha * (the product given as slices parts [S, M, d], rounded to bfloat16); out = rmsnorm(x) * weight."""
    _dev(parts, x, weight, out)
    S, M, d = parts.shape
    _need(parts.dtype == torch.float32 and parts.is_contiguous() and x.dtype == torch.float32 and x.is_contiguous()
          and tuple(x.shape) == (M, d) and weight.dtype == torch.float32 and weight.numel() == d and weight.is_contiguous()
          and out.dtype == torch.bfloat16 and out.is_contiguous() and tuple(out.shape) == (M, d), "splitk_add_rmsnorm: layout")
    check(get_lib().ic_splitk_add_rmsnorm(parts.data_ptr(), S, M, x.data_ptr(), float(alpha), weight.data_ptr(), out.data_ptr(),
                                          d, float(eps), _stream()), "splitk_add_rmsnorm")
    return out


# ---- decoders whose sublayers read the residual stream and are normalised on the way back -------------------------
ACTIVATIONS = {"relu2": 0, "gelu_tanh": 1, "silu": 2}


def embed_sinusoid(tokens, positions, table, freq, out, copy=None, scale: float = 1.0):
    """out[t, 2i] = table[tokens[t], 2i] * scale + sin(positions[t] * f_i), out[t, 2i+1] = .. + cos(..);
    ``freq`` is float32 [2, ceil(d/2)]: f_i rounded, and what the rounding left (zeros: the rounded value alone).
    out is float32 [T, d]; ``copy`` (optional, [T, d]) receives out rounded to its dtype."""
    _dev(tokens, positions, table, freq, out, copy)
    _i32(tokens, "tokens")
    _i32(positions, "positions")
    T, d = out.shape
    _need(tokens.numel() == T and positions.numel() == T and table.dim() == 2 and table.shape[1] == d,
          "embed_sinusoid: shape mismatch")
    _need(out.dtype == torch.float32 and out.is_contiguous() and table.is_contiguous(), "embed_sinusoid: layout")
    _need(freq.dtype == torch.float32 and freq.is_contiguous() and tuple(freq.shape) == (2, (d + 1) // 2),
          "embed_sinusoid: freq must be float32 [2, ceil(d/2)]")
    if copy is not None:
        _need(tuple(copy.shape) == (T, d) and copy.is_contiguous(), "embed_sinusoid: copy layout")
    check(get_lib().ic_embed_sinusoid(tokens.data_ptr(), positions.data_ptr(), table.data_ptr(), dtype_code(table.dtype),
                                      freq.data_ptr(), out.data_ptr(), copy.data_ptr() if copy is not None else None,
                                      dtype_code(copy.dtype) if copy is not None else 0, T, d, float(scale), _stream()),
          "embed_sinusoid")
    return out


def norm_into_stream(y, weight, x, eps: float, bias=None, copy=None):
    """x += rmsnorm(y + bias) * weight, row by row (x float32, in place); ``copy`` (optional) receives the new x
    rounded to its dtype."""
    _dev(y, weight, x, bias, copy)
    T, d = x.shape
    _need(x.dtype == torch.float32 and x.is_contiguous() and y.is_contiguous() and tuple(y.shape) == (T, d),
          "norm_into_stream: layout")
    _need(weight.dtype == torch.float32 and weight.numel() == d and weight.is_contiguous(), "norm_into_stream: weight must be float32 [d]")
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.numel() == d and bias.is_contiguous(), "norm_into_stream: bias must be float32 [d]")
    if copy is not None:
        _need(tuple(copy.shape) == (T, d) and copy.is_contiguous(), "norm_into_stream: copy layout")
    check(get_lib().ic_norm_into_stream(y.data_ptr(), dtype_code(y.dtype), bias.data_ptr() if bias is not None else None,
                                        weight.data_ptr(), x.data_ptr(), copy.data_ptr() if copy is not None else None,
                                        dtype_code(copy.dtype) if copy is not None else 0, T, d, float(eps), _stream()),
          "norm_into_stream")
    return x


def qk_norm_store(rows, bias, q_weight, k_weight, norm_mode: int, eps: float, mix_mode: int, mix_lambda, v_keep, q_out,
                  kcache, vcache, slots, n_heads: int, n_kv_heads: int, key_dim: int, value_dim: int, page_size: int):
    """One pass over the projected rows [q | k | v | ..]: bias, query/key norm (0 none, 1 per head, with weights or with
    both None to unit root mean square alone, 2 whole row), value
    mixing (0 none, 1 keep the values in ``v_keep``, 2 mix with ``v_keep`` by ``mix_lambda``), q to ``q_out``, k and v
    into the cache planes at ``slots`` (None: no cache write)."""
    _dev(rows, bias, q_weight, k_weight, mix_lambda, v_keep, q_out, kcache, vcache, slots)
    T = rows.shape[0]
    nq, nk, nv = n_heads * key_dim, n_kv_heads * key_dim, n_kv_heads * value_dim
    _need(rows.dim() == 2 and rows.stride(1) == 1 and rows.shape[1] >= nq + nk + nv, "qk_norm_store: rows too short")
    _need(tuple(q_out.shape) == (T, nq) and q_out.is_contiguous() and q_out.dtype == rows.dtype, "qk_norm_store: q_out layout")
    for v, n, what in ((bias, nq + nk + nv, "bias"), (q_weight, (key_dim, nq)[norm_mode == 2], "q weight"),
                       (k_weight, (key_dim, nk)[norm_mode == 2], "k weight"), (mix_lambda, 1, "lambda")):
        if v is not None:
            _need(v.dtype == torch.float32 and v.is_contiguous() and v.numel() == n, "qk_norm_store: %s must be float32 [%d]" % (what, n))
    _need((q_weight is None) == (k_weight is None), "qk_norm_store: the query and key norms have weights both or neither")
    _need(norm_mode != 2 or q_weight is not None, "qk_norm_store: the whole-row norm needs its weights")
    if mix_mode:
        _need(v_keep is not None and v_keep.dtype == torch.float32 and v_keep.is_contiguous() and v_keep.numel() == T * nv,
              "qk_norm_store: v_keep must be float32 [T, kv_heads * value_dim]")
        _need(mix_mode == 1 or mix_lambda is not None, "qk_norm_store: lambda missing")
    if slots is not None:
        _i32(slots, "slots")
        _need(slots.numel() == T, "qk_norm_store: slots/rows mismatch")
        _need(kcache.dtype == rows.dtype and vcache.dtype == rows.dtype and kcache.is_contiguous() and vcache.is_contiguous()
              and tuple(kcache.shape[1:]) == (n_kv_heads, page_size, key_dim)
              and tuple(vcache.shape[1:]) == (n_kv_heads, page_size, value_dim) and kcache.shape[0] == vcache.shape[0],
              "qk_norm_store: cache must be K [pages, kv_heads, page_size, key_dim], V [.., value_dim]")
    p = lambda t: t.data_ptr() if t is not None else None
    check(get_lib().ic_qk_norm_store(rows.data_ptr(), rows.stride(0), dtype_code(rows.dtype), p(bias), p(q_weight), p(k_weight),
                                     int(norm_mode), float(eps), int(mix_mode), p(mix_lambda), p(v_keep), q_out.data_ptr(),
                                     p(kcache) if slots is not None else None, p(vcache) if slots is not None else None,
                                     p(slots), T, n_heads, n_kv_heads, key_dim, value_dim, page_size, _stream()),
          "qk_norm_store")


def activation(x, out, kind: str):
    """out = act(x) element by element (relu2: relu(z)^2, gelu_tanh, silu)."""
    _dev(x, out)
    _need(x.is_contiguous() and out.is_contiguous() and x.shape == out.shape and x.dtype == out.dtype, "activation: layout")
    _need(kind in ACTIVATIONS, "activation: kind %r (have %s)" % (kind, ", ".join(sorted(ACTIVATIONS))))
    check(get_lib().ic_activation(x.data_ptr(), out.data_ptr(), dtype_code(x.dtype), x.numel(), ACTIVATIONS[kind], _stream()),
          "activation")
    return out


def _span_common(q, out, gate, kcache, vcache, block_tables, n_heads, n_kv_heads, key_dim, value_dim, page_size):
    _dev(q, out, gate, kcache, vcache, block_tables)
    _need(q.dim() == 2 and q.stride(1) == 1 and q.shape[1] >= n_heads * key_dim, "span attention: q layout")
    _need(out.dim() == 2 and out.stride(1) == 1 and out.shape[1] >= n_heads * value_dim and out.shape[0] == q.shape[0],
          "span attention: out layout")
    _need(q.dtype == out.dtype == kcache.dtype == vcache.dtype, "span attention: dtypes differ")
    if gate is not None:
        _need(gate.dim() == 2 and gate.stride(1) == 1 and gate.shape[1] >= n_heads * value_dim and gate.shape[0] == q.shape[0]
              and gate.dtype == q.dtype, "span attention: gate layout")
    _need(kcache.is_contiguous() and vcache.is_contiguous() and kcache.shape[0] == vcache.shape[0]
          and tuple(kcache.shape[1:]) == (n_kv_heads, page_size, key_dim)
          and tuple(vcache.shape[1:]) == (n_kv_heads, page_size, value_dim),
          "span attention: cache must be K [pages, kv_heads, page_size, key_dim], V [.., value_dim]")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.stride(1) == 1,
          "span attention: block_tables must be int32 [R, max_blocks]")
    _need(n_heads % n_kv_heads == 0, "span attention: heads not a multiple of kv heads")


def _sink_args(sink, n_heads: int):
    """``sink``: False (none), True (the term exp(0)) or a float32 tensor [heads] of learned sinks (the term exp(sink_h))."""
    if isinstance(sink, torch.Tensor):
        _dev(sink)
        _need(sink.dtype == torch.float32 and sink.is_contiguous() and sink.numel() == n_heads,
              "span attention: learned sinks must be float32 [%d]" % n_heads)
        return 1, sink.data_ptr()
    return int(bool(sink)), None


def attention_span_generic(q, out, gate, kcache, vcache, block_tables, token_req, positions, n_heads, n_kv_heads, key_dim,
                           value_dim, page_size, scale: float, window: int = 0, keep_first: int = 0, sink=False,
                           softcap: float = 0.0):
    """out[t, h] = sum_j p_j V_j over the keys j <= positions[t] with positions[t] - j < window or j < keep_first
    (window 0: all), p = softmax of s_j = scale * q . K_j (``softcap`` c > 0: s_j <- c tanh(s_j / c)) with the sink's
    term added to the denominator (``sink``: see ``_sink_args``); times sigmoid(gate)."""
    sink_flag, sink_ptr = _sink_args(sink, n_heads)
    _span_common(q, out, gate, kcache, vcache, block_tables, n_heads, n_kv_heads, key_dim, value_dim, page_size)
    _i32(token_req, "token_req")
    _i32(positions, "positions")
    T = q.shape[0]
    _need(token_req.numel() == T and positions.numel() == T, "span attention: T mismatch")
    _need(key_dim <= 512 and value_dim <= 512, "span attention: head size above 512")
    check(get_lib().ic_attn_span_generic(
        q.data_ptr(), q.stride(0), out.data_ptr(), out.stride(0), gate.data_ptr() if gate is not None else None,
        gate.stride(0) if gate is not None else 0, dtype_code(q.dtype), kcache.data_ptr(), vcache.data_ptr(),
        block_tables.data_ptr(), block_tables.stride(0), token_req.data_ptr(), positions.data_ptr(), T, n_heads, n_kv_heads,
        key_dim, value_dim, page_size, float(scale), int(window or 0), int(keep_first or 0), sink_flag, sink_ptr,
        float(softcap or 0.0), _stream()),
        "attention_span_generic")


def attention_span_decode_supported(dtype, key_dim: int, value_dim: int) -> bool:
    code = _code_or_none(dtype)
    return code is not None and bool(get_lib().ic_attn_span_decode_supported(code, key_dim, value_dim))


def attention_span_decode_splits(n_rows: int, n_kv_heads: int, max_keys: int, compute_units: int) -> int:
    return int(get_lib().ic_attn_span_decode_splits(n_rows, n_kv_heads, max_keys, compute_units))


def attention_span_decode(q, out, gate, kcache, vcache, block_tables, tok_list, n_tok, token_req, positions, part_acc,
                          part_ml, n_heads, n_kv_heads, key_dim, value_dim, page_size, scale: float, window: int = 0,
                          keep_first: int = 0, sink=False, softcap: float = 0.0, n_split: int = 1):
    """The rows ``tok_list`` (None: rows 0..n_tok-1) of q, each a request's single new token, split ``n_split`` ways
    over their visible keys.  part_acc / part_ml: float32 scratch of n_tok * heads * n_split * (value_dim / 2) elements."""
    _span_common(q, out, gate, kcache, vcache, block_tables, n_heads, n_kv_heads, key_dim, value_dim, page_size)
    _i32(token_req, "token_req")
    _i32(positions, "positions")
    if tok_list is not None:
        _i32(tok_list, "tok_list")
        _need(tok_list.numel() >= n_tok, "span decode: tok_list shorter than n_tok")
    else:
        _need(n_tok <= q.shape[0], "span decode: more tokens than rows")
    _need(1 <= n_split <= 32, "span decode: 1..32 splits")
    sink_flag, sink_ptr = _sink_args(sink, n_heads)
    if n_split > 1:
        _dev(part_acc, part_ml)
        _need(part_acc.dtype == torch.float32 and part_ml.dtype == torch.float32
              and part_acc.numel() >= n_tok * n_heads * n_split * value_dim
              and part_ml.numel() >= n_tok * n_heads * n_split * 2, "span decode: scratch too small")
    check(get_lib().ic_attn_span_decode(
        q.data_ptr(), q.stride(0), out.data_ptr(), out.stride(0), gate.data_ptr() if gate is not None else None,
        gate.stride(0) if gate is not None else 0, dtype_code(q.dtype), kcache.data_ptr(), vcache.data_ptr(),
        block_tables.data_ptr(), block_tables.stride(0), tok_list.data_ptr() if tok_list is not None else None,
        token_req.data_ptr(), positions.data_ptr(), part_acc.data_ptr() if n_split > 1 else None,
        part_ml.data_ptr() if n_split > 1 else None, n_tok, n_heads, n_kv_heads, key_dim, value_dim, page_size,
        float(scale), int(window or 0), int(keep_first or 0), sink_flag, sink_ptr, float(softcap or 0.0), int(n_split),
        _stream()),
        "attention_span_decode")


def attention_span_prefill_supported(dtype, key_dim: int, value_dim: int) -> bool:
    code = _code_or_none(dtype)
    return code is not None and bool(get_lib().ic_attn_span_prefill_supported(code, key_dim, value_dim))


def attention_span_prefill(q, out, gate, kcache, vcache, block_tables, tiles, n_tiles, n_heads, n_kv_heads, key_dim,
                           value_dim, page_size, scale: float, window: int = 0, keep_first: int = 0, sink=False,
                           softcap: float = 0.0):
    """Prompt portions listed as tiles int32 [n_tiles, 4] (request row, first token row, rows, first position)."""
    sink_flag, sink_ptr = _sink_args(sink, n_heads)
    _span_common(q, out, gate, kcache, vcache, block_tables, n_heads, n_kv_heads, key_dim, value_dim, page_size)
    _dev(tiles)
    _need(tiles.dtype == torch.int32 and tiles.is_contiguous() and tiles.numel() >= 4 * n_tiles, "span prefill: tiles layout")
    _need(scale > 0, "span prefill: the scale must be positive")
    check(get_lib().ic_attn_span_prefill(
        q.data_ptr(), q.stride(0), out.data_ptr(), out.stride(0), gate.data_ptr() if gate is not None else None,
        gate.stride(0) if gate is not None else 0, dtype_code(q.dtype), kcache.data_ptr(), vcache.data_ptr(),
        block_tables.data_ptr(), block_tables.stride(0), tiles.data_ptr(), n_tiles, n_heads, n_kv_heads, key_dim, value_dim,
        page_size, float(scale), int(window or 0), int(keep_first or 0), sink_flag, sink_ptr, float(softcap or 0.0),
        _stream()),
        "attention_span_prefill")


# ---- several residual streams, the embedding with a pair table -----------------------------------------------
def _ptr(t):
    return t.data_ptr() if t is not None else None


def pair_rows(tokens, positions, token_req, state_slots, prev_state, rows, buckets: int, mul_prev: int, mul_cur: int):
    """rows[t] = (prev * mul_prev + tokens[t] * mul_cur) mod buckets, prev the token before in the same sequence (the
    request's remembered token for a step's first row); ``buckets`` itself at position 0."""
    _dev(tokens, positions, token_req, state_slots, prev_state, rows)
    for t, n in ((tokens, "tokens"), (positions, "positions"), (token_req, "token_req"), (state_slots, "state_slots"),
                 (prev_state, "prev_state"), (rows, "rows")):
        _i32(t, n)
    T = tokens.numel()
    _need(positions.numel() == T and token_req.numel() == T and rows.numel() >= T, "pair_rows: T mismatch")
    check(get_lib().ic_pair_rows(tokens.data_ptr(), positions.data_ptr(), token_req.data_ptr(), state_slots.data_ptr(),
                                 prev_state.data_ptr(), rows.data_ptr(), T, int(buckets), int(mul_prev), int(mul_cur),
                                 _stream()), "pair_rows")
    return rows


def embed_streams(tokens, table, out, rows=None, pair_table=None, token_req=None, state_slots=None, prev_state=None):
    """out[s, t] = table[tokens[t]] + pair_table[rows[t]] for every stream s of out [S, T, d] (float32); with
    ``prev_state`` the last token of every request's share of the step is remembered there."""
    _dev(tokens, table, out, rows, pair_table, token_req, state_slots, prev_state)
    _i32(tokens, "tokens")
    _need(out.dim() == 3 and out.dtype == torch.float32 and out.is_contiguous(), "embed_streams: out is float32 [S, T, d]")
    S, T, d = out.shape
    _need(tokens.numel() == T and table.dim() == 2 and table.shape[1] == d and table.is_contiguous(), "embed_streams: table")
    if pair_table is not None:
        _i32(rows, "rows")
        _need(pair_table.dtype == table.dtype and pair_table.shape[1] == d and pair_table.is_contiguous()
              and rows.numel() >= T, "embed_streams: pair table")
    if prev_state is not None:
        for t, n in ((token_req, "token_req"), (state_slots, "state_slots"), (prev_state, "prev_state")):
            _i32(t, n)
    check(get_lib().ic_embed_streams(tokens.data_ptr(), _ptr(rows) if pair_table is not None else None, table.data_ptr(),
                                     _ptr(pair_table), dtype_code(table.dtype), out.data_ptr(), S, T, d, _ptr(token_req),
                                     _ptr(state_slots), _ptr(prev_state), _stream()), "embed_streams")
    return out


def hc_step(x, y=None, mix=None, out_w=None, in_w=None, norm_w=None, eps: float = 0.0, h=None):
    """x [S, T, d] float32 streams.  With ``y`` [T, d]: x_t <- sum_s mix[s, t] x_s + out_w[t] y, all streams at once.
    With ``in_w``: h = sum_s in_w[s] x_s (after the write), times rsqrt(mean + eps) * norm_w when ``norm_w`` is given."""
    _dev(x, y, mix, out_w, in_w, norm_w, h)
    _need(x.dim() == 3 and x.dtype == torch.float32 and x.is_contiguous(), "hc_step: x is float32 [S, T, d]")
    S, T, d = x.shape
    for v, n, shape in ((mix, "mix", (S, S)), (out_w, "out_w", (S,)), (in_w, "in_w", (S,)), (norm_w, "norm_w", (d,))):
        if v is not None:
            _need(v.dtype == torch.float32 and v.is_contiguous() and tuple(v.shape) == shape, "hc_step: %s is float32 %s" % (n, shape))
    if y is not None:
        _need(tuple(y.shape) == (T, d) and y.is_contiguous() and mix is not None and out_w is not None, "hc_step: y")
    if in_w is not None:
        _need(h is not None and tuple(h.shape) == (T, d) and h.is_contiguous(), "hc_step: h")
    check(get_lib().ic_hc_step(x.data_ptr(), S, T, d, _ptr(y), dtype_code(y.dtype) if y is not None else 0, _ptr(mix),
                               _ptr(out_w), _ptr(in_w), _ptr(norm_w), float(eps), _ptr(h),
                               dtype_code(h.dtype) if h is not None else 0, _stream()), "hc_step")
    return h


# ---- mixers with a fixed-size state ------------------------------------------------------------------------------
def _state_part(state, offset: int):
    _need(state.dtype == torch.float32 and state.dim() == 2 and state.is_contiguous(), "state is float32 [slots, n]")
    return state.data_ptr() + 4 * int(offset), state.shape[1]


def causal_conv(xin, w, b, out, state, state_offset: int, token_req, req_start, state_slots, n_requests: int,
                in_bias=None, out_copy=None, act: str = "none"):
    """out[t, c] = act(b[c] + sum_k w[c, k] in(t - (taps-1-k), c)), in = xin + in_bias, rows before a request's first
    one from its state (the last taps-1 inputs at ``state_offset``, [taps-1, C]), which is then moved on."""
    _dev(xin, w, b, out, state, token_req, req_start, state_slots, in_bias, out_copy)
    T, C = out.shape
    taps = w.shape[1]
    _need(xin.shape[0] == T and xin.shape[1] == C and xin.stride(1) == 1, "causal_conv: xin")
    _need(out.dtype == torch.float32 and out.is_contiguous() and w.dtype == torch.float32 and w.is_contiguous()
          and tuple(w.shape) == (C, taps), "causal_conv: layout")
    for v in (b, in_bias):
        if v is not None:
            _need(v.dtype == torch.float32 and v.numel() == C and v.is_contiguous(), "causal_conv: bias")
    if out_copy is not None:
        _need(out_copy.dtype == xin.dtype and tuple(out_copy.shape) == (T, C) and out_copy.stride(1) == 1, "causal_conv: copy")
    for t, n in ((token_req, "token_req"), (req_start, "req_start"), (state_slots, "state_slots")):
        _i32(t, n)
    _need(token_req.numel() >= T and req_start.numel() >= n_requests + 1 and state_slots.numel() >= n_requests, "causal_conv: lists")
    sp, stride = _state_part(state, state_offset)
    _need(state_offset + (taps - 1) * C <= stride, "causal_conv: state too small")
    check(get_lib().ic_causal_conv(xin.data_ptr(), xin.stride(0), dtype_code(xin.dtype), _ptr(in_bias), w.data_ptr(), _ptr(b),
                                   taps, C, out.data_ptr(), _ptr(out_copy), out_copy.stride(0) if out_copy is not None else 0,
                                   {"none": 0, "silu": 1}[act], sp, stride, token_req.data_ptr(), req_start.data_ptr(),
                                   state_slots.data_ptr(), T, n_requests, _stream()), "causal_conv")
    return out


def _chunk_scratch(chunks, n_state: int, n_factors: int, n_requests: int, what: str):
    """(chunk_len, max_chunks, scratch for states, scratch for factors) of a recurrence run in chunks side by side, or
    zeros and None for the single pass.  ``chunks`` = (chunk_len, max_chunks, float32 states, float32 factors)."""
    if not chunks or chunks[1] <= 1:
        return 0, 1, None, None
    chunk_len, max_chunks, scr_s, scr_a = chunks
    _dev(scr_s, scr_a)
    _need(chunk_len > 0 and scr_s.dtype == torch.float32 and scr_a.dtype == torch.float32
          and scr_s.numel() >= n_requests * max_chunks * n_state and scr_a.numel() >= n_requests * max_chunks * n_factors,
          what + ": scratch for the chunks too small")
    return int(chunk_len), int(max_chunks), scr_s.data_ptr(), scr_a.data_ptr()


def rglru_scan(gates, gate_bias, u, yb, y_bias, decay, block_width: int, out, state, state_offset: int, req_start,
               state_slots, n_requests: int, chunks=None):
    """The gated diagonal recurrence over every request's rows (see csrc/recurrent.hip); out = S * gelu_tanh(yb + y_bias).
    ``chunks``: (chunk_len, max_chunks, scratch, scratch) to run every request's rows as chunks side by side (every
    request must fit max_chunks chunks of chunk_len rows)."""
    _dev(gates, gate_bias, u, yb, y_bias, decay, out, state, req_start, state_slots)
    T, width = u.shape
    for v, shape in ((gates, (T, 2 * width)), (u, (T, width))):
        _need(v.dtype == torch.float32 and v.is_contiguous() and tuple(v.shape) == shape, "rglru_scan: float32 operands")
    for v, n in ((gate_bias, 2 * width), (decay, width), (y_bias, width)):
        _need(v is None or (v.dtype == torch.float32 and v.numel() == n and v.is_contiguous()), "rglru_scan: vectors")
    _need(tuple(yb.shape) == (T, width) and yb.stride(1) == 1 and out.dtype == yb.dtype and tuple(out.shape) == (T, width)
          and out.is_contiguous(), "rglru_scan: branches")
    _i32(req_start, "req_start")
    _i32(state_slots, "state_slots")
    sp, stride = _state_part(state, state_offset)
    _need(state_offset + width <= stride, "rglru_scan: state too small")
    check(get_lib().ic_rglru_scan(gates.data_ptr(), gate_bias.data_ptr(), u.data_ptr(), yb.data_ptr(), yb.stride(0),
                                  dtype_code(yb.dtype), _ptr(y_bias), decay.data_ptr(), width, int(block_width), out.data_ptr(),
                                  sp, stride, req_start.data_ptr(), state_slots.data_ptr(), n_requests,
                                  *_chunk_scratch(chunks, width, width, n_requests, "rglru_scan"), _stream()), "rglru_scan")
    return out


def ssm_scan(xbc, dt_raw, dt_bias, neg_a, d_skip, heads: int, head_dim: int, state_dim: int, groups: int, y, state,
             state_offset: int, req_start, state_slots, n_requests: int, chunks=None, in_act=None):
    """The state-space recurrence over every request's rows (see csrc/recurrent.hip): y float32 [T, heads * head_dim].
    ``xbc`` [T, >= inner + 2 groups state_dim] holds x, B, C of every token, float32 or y's compute dtype (rows may be
    strided: a projection's own columns); ``in_act`` "silu": applied as they are read.  ``dt_raw`` None: no step sizes,
    ``neg_a`` is then the fixed decay per head and every step is one (linear attention with keys B, values x, queries
    C); ``dt_bias`` and ``d_skip`` may be None."""
    _dev(xbc, dt_raw, dt_bias, neg_a, d_skip, y, state, req_start, state_slots)
    T = xbc.shape[0]
    inner = heads * head_dim
    _need(xbc.dim() == 2 and xbc.stride(1) == 1 and xbc.shape[1] >= inner + 2 * groups * state_dim
          and xbc.stride(0) >= inner + 2 * groups * state_dim, "ssm_scan: xbc")
    _need(y.dtype == torch.float32 and y.is_contiguous() and tuple(y.shape) == (T, inner), "ssm_scan: y")
    _need(in_act in (None, "silu"), "ssm_scan: in_act is None or 'silu'")
    if dt_raw is not None:
        _need(tuple(dt_raw.shape) == (T, heads) and dt_raw.stride(1) == 1, "ssm_scan: dt")
        _need(xbc.dtype in (torch.float32, dt_raw.dtype), "ssm_scan: xbc is float32 or of the step sizes' dtype")
    for v in (dt_bias, neg_a, d_skip):
        _need(v is None or (v.dtype == torch.float32 and v.numel() == heads and v.is_contiguous()), "ssm_scan: per-head vectors")
    _need(neg_a is not None, "ssm_scan: the decays are missing")
    _i32(req_start, "req_start")
    _i32(state_slots, "state_slots")
    sp, stride = _state_part(state, state_offset)
    _need(state_offset + inner * state_dim <= stride, "ssm_scan: state too small")
    dt_code = dtype_code(dt_raw.dtype) if dt_raw is not None else dtype_code(xbc.dtype)
    check(get_lib().ic_ssm_scan(xbc.data_ptr(), xbc.stride(0), dtype_code(xbc.dtype), 1 if in_act else 0, _ptr(dt_raw),
                                dt_raw.stride(0) if dt_raw is not None else 0, dt_code, _ptr(dt_bias),
                                neg_a.data_ptr(), _ptr(d_skip), heads, head_dim, state_dim, groups, y.data_ptr(), sp, stride,
                                req_start.data_ptr(), state_slots.data_ptr(), n_requests,
                                *_chunk_scratch(chunks, inner * state_dim, heads, n_requests, "ssm_scan"), _stream()), "ssm_scan")
    return y


def gated_group_norm(y, z, weight, groups: int, eps: float, out, gate_after: bool = False):
    """out = rms_in_groups(y * silu(z)) * weight, or with ``gate_after`` rms_in_groups(y) * weight * sigmoid(z);
    y float32 [T, n], z (rows may be strided) and out the compute dtype."""
    _dev(y, z, weight, out)
    T, n = y.shape
    _need(y.dtype == torch.float32 and y.is_contiguous() and tuple(z.shape) == (T, n) and z.stride(1) == 1
          and out.dtype == z.dtype and tuple(out.shape) == (T, n) and out.is_contiguous(), "gated_group_norm: layout")
    _need(weight.dtype == torch.float32 and weight.numel() == n and weight.is_contiguous(), "gated_group_norm: weight")
    check(get_lib().ic_gated_group_norm(y.data_ptr(), z.data_ptr(), z.stride(0), dtype_code(z.dtype), weight.data_ptr(), n,
                                        int(groups), float(eps), out.data_ptr(), T, 1 if gate_after else 0, _stream()),
          "gated_group_norm")
    return out


def blocked_product(a, w, out, gate=None):
    """out[m, b, n] = sum_k a[m, b, k] w[b, n, k] (times sigmoid(gate[m, b, n])): a [M, B, K] and out [M, B, N] may be
    views whose rows are strided; w [B, N, K] contiguous.  out may be float32 under bfloat16 operands."""
    _dev(a, w, out, gate)
    M, B, K = a.shape
    N = w.shape[1]
    _need(tuple(w.shape) == (B, N, K) and w.is_contiguous() and w.dtype == a.dtype, "blocked_product: w")
    _need(tuple(out.shape) == (M, B, N) and a.stride(2) == 1 and out.stride(2) == 1, "blocked_product: shapes")
    if gate is not None:
        _need(tuple(gate.shape) == (M, B, N) and gate.dtype == a.dtype and gate.stride(2) == 1 and gate.stride(1) == out.stride(1),
              "blocked_product: gate")
    check(get_lib().ic_blocked_product(a.data_ptr(), a.stride(0), a.stride(1), w.data_ptr(), dtype_code(a.dtype), out.data_ptr(),
                                       dtype_code(out.dtype), out.stride(0), out.stride(1), _ptr(gate),
                                       gate.stride(0) if gate is not None else 0, M, N, K, B, _stream()), "blocked_product")
    return out


# ---- attention through a latent -------------------------------------------------------------------------------------
def latent_prep(rows, q_rank: int, kv_rank: int, rot_dim: int, qn_w, kvn_w, eps: float, freq, rot_dims: int, positions,
                cq, cache, slots):
    """cq = rms(rows[:, :q_rank]) * qn_w; cache[slots[t]] = [rms(next kv_rank columns) * kvn_w | the next rot_dim rotated]."""
    _dev(rows, qn_w, kvn_w, freq, positions, cq, cache, slots)
    T = rows.shape[0]
    _need(rows.stride(1) == 1 and rows.shape[1] >= q_rank + kv_rank + rot_dim, "latent_prep: rows")
    _need(cq.dtype == rows.dtype and tuple(cq.shape) == (T, q_rank) and cq.is_contiguous(), "latent_prep: cq")
    for v, n in ((qn_w, q_rank), (kvn_w, kv_rank), (freq, rot_dims // 2)):
        _need(v.dtype == torch.float32 and v.numel() >= n and v.is_contiguous(), "latent_prep: vectors")
    _i32(positions, "positions")
    if slots is not None:
        _i32(slots, "slots")
        _need(cache.dtype == rows.dtype and cache.is_contiguous() and cache.shape[-1] == kv_rank + rot_dim and cache.shape[1] == 1,
              "latent_prep: cache plane")
    check(get_lib().ic_latent_prep(rows.data_ptr(), rows.stride(0), dtype_code(rows.dtype), q_rank, kv_rank, rot_dim,
                                   qn_w.data_ptr(), kvn_w.data_ptr(), float(eps), freq.data_ptr(), int(rot_dims),
                                   positions.data_ptr(), cq.data_ptr(), _ptr(cache), _ptr(slots), T, _stream()), "latent_prep")


def latent_q_rotate(q, dim: int, rot_dim: int, kv_rank: int, heads: int, freq, rot_dims: int, positions, qa):
    """qa[t, h, kv_rank:] = the rotated part q[t, h, dim:] turned by its position's angles."""
    _dev(q, freq, positions, qa)
    T = q.shape[0]
    _need(q.shape[1] == heads * (dim + rot_dim) and q.stride(1) == 1 and qa.dtype == q.dtype
          and tuple(qa.shape) == (T, heads * (kv_rank + rot_dim)) and qa.stride(1) == 1, "latent_q_rotate: layout")
    _i32(positions, "positions")
    check(get_lib().ic_latent_q_rotate(q.data_ptr(), q.stride(0), dtype_code(q.dtype), dim, rot_dim, kv_rank, heads,
                                       freq.data_ptr(), int(rot_dims), positions.data_ptr(), qa.data_ptr(), qa.stride(0), T,
                                       _stream()), "latent_q_rotate")


LATENT_MAX_RANK = 512


def attention_latent_on_matrix_cores(dtype, kv_rank: int, rot_dim: int) -> bool:
    """True when ``attention_latent`` runs its matrix-core kernel for these sizes."""
    code = _code_or_none(dtype)
    return code is not None and bool(get_lib().ic_attn_latent_on_matrix_cores(code, kv_rank, rot_dim))


def attention_latent(qa, out, cache, block_tables, token_req, positions, heads: int, kv_rank: int, rot_dim: int,
                     page_size: int, scale: float, n_split: int = 1, part_acc=None, part_ml=None, row_list=None, n_rows=None,
                     vector_units: bool = False):
    """out[t, h, :kv_rank] = sum_j p_j c_j over the cached rows [c | k_rot] j <= positions[t] of the token's request,
    p = softmax(scale * qa[t, h] . row_j): every head walks the same rows.  ``row_list`` (int32, ``n_rows`` of them): the
    rows t to compute; None: all.  bfloat16 with a latent of 64..512 and a rotated part of 16..64 values runs on the
    matrix cores unless ``vector_units`` asks for the general kernel."""
    _dev(qa, out, cache, block_tables, token_req, positions, part_acc, part_ml, row_list)
    T = qa.shape[0]
    n_launch = T
    if row_list is not None:
        _i32(row_list, "row_list")
        n_launch = int(n_rows)
        _need(0 <= n_launch <= row_list.numel(), "attention_latent: row list shorter than n_rows")
    D = kv_rank + rot_dim
    _need(tuple(qa.shape) == (T, heads * D) and qa.stride(1) == 1 and out.dtype == qa.dtype
          and tuple(out.shape) == (T, heads * kv_rank) and out.stride(1) == 1, "attention_latent: q / out")
    _need(cache.dtype == qa.dtype and cache.is_contiguous() and cache.shape[-1] == D and cache.shape[1] == 1
          and cache.shape[2] == page_size, "attention_latent: cache plane")
    for t, n in ((block_tables, "block_tables"), (token_req, "token_req"), (positions, "positions")):
        _need(t.dtype == torch.int32, n + " must be int32")
    _need(block_tables.stride(1) == 1 and token_req.numel() >= T and positions.numel() >= T, "attention_latent: lists")
    if n_split > 1:
        _need(part_acc is not None and part_ml is not None and part_acc.dtype == torch.float32 and part_ml.dtype == torch.float32
              and part_acc.numel() >= T * heads * n_split * kv_rank and part_ml.numel() >= T * heads * n_split * 2,
              "attention_latent: scratch too small")
    check(get_lib().ic_attn_latent(qa.data_ptr(), qa.stride(0), out.data_ptr(), out.stride(0), dtype_code(qa.dtype),
                                   cache.data_ptr(), block_tables.data_ptr(), block_tables.stride(0), token_req.data_ptr(),
                                   positions.data_ptr(), _ptr(row_list), n_launch, heads, kv_rank, rot_dim, page_size,
                                   float(scale), int(n_split), _ptr(part_acc), _ptr(part_ml), int(bool(vector_units)), _stream()),
          "attention_latent")
    return out


def latent_gather(cache, table_row, n_keys: int, n_padded: int, page_size: int, kv_rank: int, rows, rows_t):
    """rows[j] = the cached row of key j of the request whose block-table row is ``table_row`` (zeros from n_keys to
    n_padded); rows_t[c, j] = rows[j, c] for the first kv_rank columns."""
    _dev(cache, table_row, rows, rows_t)
    D = cache.shape[-1]
    _need(table_row.dtype == torch.int32 and table_row.stride(-1) == 1 and table_row.numel() * page_size >= n_keys,
          "latent_gather: block table")
    _need(cache.is_contiguous() and cache.shape[1] == 1 and cache.shape[2] == page_size, "latent_gather: cache plane")
    _need(rows.dtype == cache.dtype and rows_t.dtype == cache.dtype and tuple(rows.shape) == (n_padded, D) and rows.is_contiguous()
          and tuple(rows_t.shape) == (kv_rank, n_padded) and rows_t.is_contiguous() and n_padded >= n_keys, "latent_gather: outputs")
    check(get_lib().ic_latent_gather(cache.data_ptr(), dtype_code(cache.dtype), table_row.data_ptr(), page_size, D, kv_rank,
                                     int(n_keys), int(n_padded), rows.data_ptr(), rows_t.data_ptr(), _stream()), "latent_gather")


def latent_softmax(scores, probs, heads: int, first_limit: int, scale: float):
    """probs[m] = softmax(scale * scores[m, :n]) with n = first_limit + m // heads + 1 visible keys, zeros beyond."""
    _dev(scores, probs)
    M, n_cols = scores.shape
    _need(scores.dtype == torch.float32 and scores.stride(1) == 1 and tuple(probs.shape) == (M, n_cols) and probs.stride(1) == 1,
          "latent_softmax: layout")
    check(get_lib().ic_latent_softmax(scores.data_ptr(), scores.stride(0), probs.data_ptr(), probs.stride(0), dtype_code(probs.dtype),
                                      M, heads, n_cols, int(first_limit), float(scale), _stream()), "latent_softmax")
    return probs


# ---- attention over a window of tokens plus the means of the blocks before it (csrc/attn_pooled.hip) -----------------------
def rope_pairs_store(rows, positions, freq, rot_dims: int, q_out, kcache, vcache, slots, n_heads: int, n_kv_heads: int,
                     key_dim: int, value_dim: int, page_size: int):
    """rows [T, >= q | k | v]: adjacent pairs of the first ``rot_dims`` entries of every query and key head turn by
    position * f_i (``freq`` float32 [2, rot_dims / 2]: f_i rounded, and what the rounding left); q -> ``q_out``
    [T, heads * key_dim], k and v -> the cache planes at ``slots`` (None: queries only)."""
    _dev(rows, positions, freq, q_out, kcache, vcache, slots)
    T = rows.shape[0]
    nq, nk, nv = n_heads * key_dim, n_kv_heads * key_dim, n_kv_heads * value_dim
    _need(rows.dim() == 2 and rows.stride(1) == 1 and rows.shape[1] >= nq + nk + nv, "rope_pairs_store: rows too short")
    _need(tuple(q_out.shape) == (T, nq) and q_out.is_contiguous() and q_out.dtype == rows.dtype, "rope_pairs_store: q_out layout")
    _need(0 <= rot_dims <= key_dim and rot_dims % 2 == 0, "rope_pairs_store: rot_dims must be even and at most the key size")
    if rot_dims:
        _need(freq is not None and freq.dtype == torch.float32 and freq.is_contiguous() and tuple(freq.shape) == (2, rot_dims // 2),
              "rope_pairs_store: freq must be float32 [2, rot_dims / 2]")
    _i32(positions, "positions")
    _need(positions.numel() == T, "rope_pairs_store: positions/rows mismatch")
    if slots is not None:
        _i32(slots, "slots")
        _need(slots.numel() == T, "rope_pairs_store: slots/rows mismatch")
        _need(kcache.dtype == rows.dtype and vcache.dtype == rows.dtype and kcache.is_contiguous() and vcache.is_contiguous()
              and tuple(kcache.shape[1:]) == (n_kv_heads, page_size, key_dim)
              and tuple(vcache.shape[1:]) == (n_kv_heads, page_size, value_dim) and kcache.shape[0] == vcache.shape[0],
              "rope_pairs_store: cache must be K [pages, kv_heads, page_size, key_dim], V [.., value_dim]")
    check(get_lib().ic_rope_pairs_store(rows.data_ptr(), rows.stride(0), dtype_code(rows.dtype), positions.data_ptr(), _ptr(freq),
                                        int(rot_dims), q_out.data_ptr(), _ptr(kcache) if slots is not None else None,
                                        _ptr(vcache) if slots is not None else None, _ptr(slots), T, n_heads, n_kv_heads,
                                        key_dim, value_dim, page_size, _stream()), "rope_pairs_store")
    return q_out


def _pooled_planes(kcache, vcache, kpool, vpool, n_kv_heads, key_dim, value_dim, page_size, what):
    for k, v in ((kcache, vcache), (kpool, vpool)):
        if k is None and v is None:
            continue
        _need(k is not None and v is not None and k.dtype == kcache.dtype and v.dtype == kcache.dtype and k.is_contiguous()
              and v.is_contiguous() and tuple(k.shape[1:]) == (n_kv_heads, page_size, key_dim)
              and tuple(v.shape[1:]) == (n_kv_heads, page_size, value_dim) and k.shape[0] == v.shape[0], what + ": cache planes")


def pool_blocks(kcache, vcache, kpool, vpool, block_tables, pool_tables, req_rows, positions, n_requests: int, most_tokens: int,
                block: int, n_kv_heads: int, key_dim: int, value_dim: int, page_size: int):
    """For every block of ``block`` tokens that a request's portion completes (its last position lies in the portion): the
    means of the block's keys and values, read from the token cache, into row b of the request's block-mean cache.
    ``req_rows``: first token row of every request, then T; ``most_tokens``: the longest portion of the step."""
    _dev(kcache, vcache, kpool, vpool, block_tables, pool_tables, req_rows, positions)
    _pooled_planes(kcache, vcache, kpool, vpool, n_kv_heads, key_dim, value_dim, page_size, "pool_blocks")
    for t, n in ((block_tables, "block_tables"), (pool_tables, "pool_tables"), (req_rows, "req_rows"), (positions, "positions")):
        _need(t.dtype == torch.int32 and t.stride(-1) == 1, "pool_blocks: %s must be int32" % n)
    _need(block > 0 and req_rows.numel() >= n_requests + 1 and block_tables.dim() == 2 and pool_tables.dim() == 2
          and block_tables.shape[0] >= n_requests and pool_tables.shape[0] >= n_requests and most_tokens >= 1, "pool_blocks: lists")
    check(get_lib().ic_pool_blocks(kcache.data_ptr(), vcache.data_ptr(), kpool.data_ptr(), vpool.data_ptr(), dtype_code(kcache.dtype),
                                   block_tables.data_ptr(), block_tables.stride(0), pool_tables.data_ptr(), pool_tables.stride(0),
                                   req_rows.data_ptr(), positions.data_ptr(), int(n_requests), int(most_tokens) // int(block) + 1,
                                   int(block), n_kv_heads, key_dim, value_dim, page_size, _stream()), "pool_blocks")


def attention_pooled_generic(q, out, kcache, vcache, kpool, vpool, block_tables, pool_tables, token_req, positions, bias,
                             n_heads: int, n_kv_heads: int, key_dim: int, value_dim: int, page_size: int, scale: float,
                             window: int, block: int):
    """out[t, h] = sum over what position p sees of sigmoid(scale q.k + bias[h]) v: tokens j with 0 <= p - j < window
    and blocks b with (b + 1) * block <= p - window + 1 (window 0: every earlier token, no blocks).  Any sizes up to 512."""
    _dev(q, out, kcache, vcache, kpool, vpool, block_tables, pool_tables, token_req, positions, bias)
    T = q.shape[0]
    _need(q.dim() == 2 and q.stride(1) == 1 and q.shape[1] == n_heads * key_dim and out.dtype == q.dtype and out.stride(1) == 1
          and tuple(out.shape) == (T, n_heads * value_dim) and kcache.dtype == q.dtype, "attention_pooled: q/out layout")
    _pooled_planes(kcache, vcache, kpool, vpool, n_kv_heads, key_dim, value_dim, page_size, "attention_pooled")
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.stride(1) == 1, "attention_pooled: block tables")
    pooled = bool(window and block)
    if pooled:
        _need(pool_tables is not None and kpool is not None and pool_tables.dtype == torch.int32 and pool_tables.dim() == 2
              and pool_tables.stride(1) == 1, "attention_pooled: the block means' planes and tables are missing")
    _i32(token_req, "token_req")
    _i32(positions, "positions")
    _need(bias is None or (bias.dtype == torch.float32 and bias.numel() == n_heads and bias.is_contiguous()), "attention_pooled: bias")
    check(get_lib().ic_attn_pooled_generic(q.data_ptr(), q.stride(0), out.data_ptr(), out.stride(0), dtype_code(q.dtype),
                                           kcache.data_ptr(), vcache.data_ptr(), _ptr(kpool) if pooled else None,
                                           _ptr(vpool) if pooled else None, block_tables.data_ptr(), block_tables.stride(0),
                                           _ptr(pool_tables) if pooled else None, pool_tables.stride(0) if pooled else 0,
                                           token_req.data_ptr(), positions.data_ptr(), _ptr(bias), T, n_heads, n_kv_heads, key_dim,
                                           value_dim, page_size, float(scale), int(window or 0), int(block or 0), _stream()),
          "attention_pooled_generic")
    return out


def _pooled_common(q, out, kcache, vcache, kpool, vpool, block_tables, pool_tables, n_heads, n_kv_heads, key_dim, value_dim,
                   page_size, window, block, bias, what):
    T = q.shape[0]
    _need(q.dim() == 2 and q.stride(1) == 1 and q.shape[1] == n_heads * key_dim and out.dtype == q.dtype and out.stride(1) == 1
          and tuple(out.shape) == (T, n_heads * value_dim) and kcache.dtype == q.dtype, what + ": q/out layout")
    _pooled_planes(kcache, vcache, kpool, vpool, n_kv_heads, key_dim, value_dim, page_size, what)
    _need(block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.stride(1) == 1, what + ": block tables")
    pooled = bool(window and block)
    if pooled:
        _need(pool_tables is not None and kpool is not None and pool_tables.dtype == torch.int32 and pool_tables.dim() == 2
              and pool_tables.stride(1) == 1, what + ": the block means' planes and tables are missing")
    _need(bias is None or (bias.dtype == torch.float32 and bias.numel() == n_heads and bias.is_contiguous()), what + ": bias")
    return pooled


def attention_pooled_decode_supported(dtype, key_dim: int, value_dim: int) -> bool:
    return dtype in _DT and bool(get_lib().ic_attn_pooled_decode_supported(_DT[dtype], int(key_dim), int(value_dim)))


def attention_pooled_decode(q, out, kcache, vcache, kpool, vpool, block_tables, pool_tables, tok_list, n_tok: int, token_req,
                            positions, parts, bias, n_heads: int, n_kv_heads: int, key_dim: int, value_dim: int, page_size: int,
                            scale: float, window: int, block: int, n_split: int = 1):
    """As ``attention_pooled_generic`` for rows that are a request's single token (``tok_list``: their rows, None: rows
    0 .. n_tok - 1), what each sees split ``n_split`` ways over blocks of threads; ``parts``: float32 scratch of
    n_split * n_tok * heads * value_dim when n_split > 1."""
    _dev(q, out, kcache, vcache, kpool, vpool, block_tables, pool_tables, tok_list, token_req, positions, parts, bias)
    pooled = _pooled_common(q, out, kcache, vcache, kpool, vpool, block_tables, pool_tables, n_heads, n_kv_heads, key_dim,
                            value_dim, page_size, window, block, bias, "attention_pooled_decode")
    _i32(token_req, "token_req")
    _i32(positions, "positions")
    if tok_list is not None:
        _i32(tok_list, "tok_list")
        _need(tok_list.numel() >= n_tok, "attention_pooled_decode: tok_list")
    else:
        _need(n_tok <= q.shape[0], "attention_pooled_decode: more rows than q holds")
    if n_split > 1:
        _need(parts is not None and parts.dtype == torch.float32 and parts.is_contiguous()
              and parts.numel() >= n_split * n_tok * n_heads * value_dim, "attention_pooled_decode: scratch for the splits")
    check(get_lib().ic_attn_pooled_decode(q.data_ptr(), q.stride(0), out.data_ptr(), out.stride(0), dtype_code(q.dtype),
                                          kcache.data_ptr(), vcache.data_ptr(), _ptr(kpool) if pooled else None,
                                          _ptr(vpool) if pooled else None, block_tables.data_ptr(), block_tables.stride(0),
                                          _ptr(pool_tables) if pooled else None, pool_tables.stride(0) if pooled else 0,
                                          _ptr(tok_list), token_req.data_ptr(), positions.data_ptr(), _ptr(bias), _ptr(parts),
                                          int(n_tok), n_heads, n_kv_heads, key_dim, value_dim, page_size, float(scale),
                                          int(window or 0), int(block or 0), int(n_split), _stream()), "attention_pooled_decode")
    return out


def attention_pooled_prefill_supported(dtype, key_dim: int, value_dim: int, page_size: int = 16) -> bool:
    return dtype in _DT and bool(get_lib().ic_attn_pooled_prefill_supported(_DT[dtype], int(key_dim), int(value_dim)))


def attention_pooled_prefill(q, out, kcache, vcache, kpool, vpool, block_tables, pool_tables, tiles, n_tiles: int, bias,
                             n_heads: int, n_kv_heads: int, key_dim: int, value_dim: int, page_size: int, scale: float,
                             window: int, block: int):
    """As ``attention_pooled_generic`` for prompt portions listed as tiles (int32 [n_tiles, 4]: request row, first token
    row, rows <= 128, first position), on the matrix cores (bfloat16)."""
    _dev(q, out, kcache, vcache, kpool, vpool, block_tables, pool_tables, tiles, bias)
    pooled = _pooled_common(q, out, kcache, vcache, kpool, vpool, block_tables, pool_tables, n_heads, n_kv_heads, key_dim,
                            value_dim, page_size, window, block, bias, "attention_pooled_prefill")
    _need(tiles.dtype == torch.int32 and tiles.is_contiguous() and tiles.numel() >= 4 * n_tiles and tiles.data_ptr() % 16 == 0,
          "attention_pooled_prefill: tiles must be int32 [n, 4], 16-byte aligned")
    check(get_lib().ic_attn_pooled_prefill(q.data_ptr(), q.stride(0), out.data_ptr(), out.stride(0), dtype_code(q.dtype),
                                           kcache.data_ptr(), vcache.data_ptr(), _ptr(kpool) if pooled else None,
                                           _ptr(vpool) if pooled else None, block_tables.data_ptr(), block_tables.stride(0),
                                           _ptr(pool_tables) if pooled else None, pool_tables.stride(0) if pooled else 0,
                                           tiles.data_ptr(), int(n_tiles), _ptr(bias), n_heads, n_kv_heads, key_dim, value_dim,
                                           page_size, float(scale), int(window or 0), int(block or 0), _stream()),
          "attention_pooled_prefill")
    return out


# ---- routed experts (csrc/moe.hip) ----------------------------------------------------------------------------------------
def moe_route(logits, top: int, ids, weights, mode: str = "sigmoid", renormalize: bool = False):
    """ids[t, k], weights[t, k]: the ``top`` experts with the largest scores of float32 ``logits`` [T, E] and their scores
    (sigmoid of the logit, or the softmax over all experts), renormalised over the chosen ones if asked."""
    _dev(logits, ids, weights)
    T, E = logits.shape
    _need(logits.dtype == torch.float32 and logits.stride(1) == 1, "moe_route: float32 logits")
    _need(ids.dtype == torch.int32 and ids.is_contiguous() and tuple(ids.shape) == (T, top) and weights.dtype == torch.float32
          and weights.is_contiguous() and tuple(weights.shape) == (T, top), "moe_route: outputs")
    check(get_lib().ic_moe_route(logits.data_ptr(), logits.stride(0), T, E, int(top), {"sigmoid": 0, "softmax": 1}[mode],
                                 1 if renormalize else 0, ids.data_ptr(), weights.data_ptr(), _stream()), "moe_route")


def moe_sort(ids, n_experts: int, offsets, order, place):
    """The (token, choice) pairs in expert order, stable: offsets [E + 1], order [n] (sorted place -> pair), place [n]."""
    _dev(ids, offsets, order, place)
    n = ids.numel()
    for t, m in ((ids, n), (offsets, n_experts + 1), (order, n), (place, n)):
        _need(t.dtype == torch.int32 and t.is_contiguous() and t.numel() == m, "moe_sort: int32 lists")
    check(get_lib().ic_moe_sort(ids.data_ptr(), n, int(n_experts), offsets.data_ptr(), order.data_ptr(), place.data_ptr(), _stream()),
          "moe_sort")


def moe_gather(h, order, weights, top: int, out):
    """out[s] = h[order[s] // top] * weights[order[s]] (weights None: as it is)."""
    _dev(h, order, weights, out)
    n, d = out.shape
    _need(h.stride(1) == 1 and h.shape[1] == d and out.is_contiguous() and out.dtype == h.dtype and order.numel() == n,
          "moe_gather: layout")
    _i32(order, "order")
    _need(weights is None or (weights.dtype == torch.float32 and weights.is_contiguous() and weights.numel() == n), "moe_gather: weights")
    check(get_lib().ic_moe_gather(h.data_ptr(), h.stride(0), dtype_code(h.dtype), order.data_ptr(), _ptr(weights), n, int(top), d,
                                  out.data_ptr(), _stream()), "moe_gather")
    return out


def moe_expert_product(a, w, offsets, out, glu: bool = False, compute_units: int = 256):
    """out[s] = a[s] W_e^T for the sorted rows s of every expert e (``offsets`` [E + 1]); ``w`` [E, N or 2N, K].  ``glu``: w
    holds gate rows then up rows, out = silu(gate) * up.  For few rows: every row chunk streams its expert's matrix."""
    _dev(a, w, offsets, out)
    E, rows, K = w.shape
    N = rows // 2 if glu else rows
    _need(w.is_contiguous() and a.stride(1) == 1 and a.shape[1] == K and out.stride(1) == 1 and out.shape[1] == N
          and out.shape[0] == a.shape[0] and a.dtype == w.dtype == out.dtype and (not glu or rows % 2 == 0), "moe_expert_product: layout")
    _i32(offsets, "offsets")
    _need(offsets.numel() == E + 1, "moe_expert_product: offsets")
    check(get_lib().ic_moe_expert_product(a.data_ptr(), a.stride(0), w.data_ptr(), rows * K, dtype_code(a.dtype), offsets.data_ptr(),
                                          out.data_ptr(), out.stride(0), E, N, K, 1 if glu else 0, int(compute_units), _stream()),
          "moe_expert_product")
    return out


def moe_combine(y, place, weights, shared, top: int, out):
    """out[t] = sum_k y[place[t * top + k]] * (weights[t * top + k] or 1) + (shared[t] or 0)."""
    _dev(y, place, weights, shared, out)
    T, d = out.shape
    _need(y.stride(1) == 1 and y.shape[1] == d and out.stride(1) == 1 and y.dtype == out.dtype and place.numel() == T * top
          and y.shape[0] == T * top, "moe_combine: layout")
    _i32(place, "place")
    _need(shared is None or (tuple(shared.shape) == (T, d) and shared.stride(1) == 1 and shared.dtype == out.dtype), "moe_combine: shared")
    _need(weights is None or (weights.dtype == torch.float32 and weights.is_contiguous() and weights.numel() == T * top), "moe_combine: weights")
    check(get_lib().ic_moe_combine(y.data_ptr(), y.stride(0), dtype_code(y.dtype), place.data_ptr(), _ptr(weights), _ptr(shared),
                                   shared.stride(0) if shared is not None else 0, T, int(top), d, out.data_ptr(), out.stride(0),
                                   _stream()), "moe_combine")
    return out


# ---- a gate on a sublayer's result; a gate on a slice of a token table (csrc/stream_rows.hip) ------------------------------
def gated_norm_into_stream(y, gate, gate_bias, weight, x, eps: float, copy=None):
    """x += rmsnorm(y * sigmoid(gate + gate_bias)) * weight, row by row (x float32, in place; ``gate`` None: no gate);
    ``copy`` (optional) receives the new x rounded to its dtype."""
    _dev(y, gate, gate_bias, weight, x, copy)
    T, d = x.shape
    _need(x.dtype == torch.float32 and x.is_contiguous() and y.is_contiguous() and tuple(y.shape) == (T, d), "gated_norm_into_stream: layout")
    _need(weight.dtype == torch.float32 and weight.numel() == d and weight.is_contiguous(), "gated_norm_into_stream: weight must be float32 [d]")
    if gate is not None:
        _need(tuple(gate.shape) == (T, d) and gate.stride(1) == 1 and gate.dtype == y.dtype, "gated_norm_into_stream: gate layout")
    _need(gate_bias is None or (gate is not None and gate_bias.dtype == torch.float32 and gate_bias.numel() == d and gate_bias.is_contiguous()),
          "gated_norm_into_stream: gate bias must be float32 [d]")
    if copy is not None:
        _need(tuple(copy.shape) == (T, d) and copy.is_contiguous() and copy.dtype == y.dtype, "gated_norm_into_stream: copy layout")
    check(get_lib().ic_gated_norm_into_stream(y.data_ptr(), _ptr(gate), gate.stride(0) if gate is not None else 0, dtype_code(y.dtype),
                                              _ptr(gate_bias), weight.data_ptr(), x.data_ptr(), _ptr(copy),
                                              dtype_code(copy.dtype) if copy is not None else 0, T, d, float(eps), _stream()),
          "gated_norm_into_stream")
    return x


def token_gate(z, table, tokens, col0: int, out):
    """out[t, j] = gelu_tanh(z[t, j]) * table[tokens[t], col0 + j]."""
    _dev(z, table, tokens, out)
    T, n = out.shape
    _need(tuple(z.shape) == (T, n) and z.stride(1) == 1 and out.is_contiguous() and table.dim() == 2 and table.stride(1) == 1
          and z.dtype == table.dtype == out.dtype and 0 <= col0 and col0 + n <= table.shape[1], "token_gate: layout")
    _i32(tokens, "tokens")
    _need(tokens.numel() == T, "token_gate: tokens/rows mismatch")
    check(get_lib().ic_token_gate(z.data_ptr(), z.stride(0), table.data_ptr(), table.stride(0), dtype_code(z.dtype), tokens.data_ptr(),
                                  int(col0), n, out.data_ptr(), T, _stream()), "token_gate")
    return out
