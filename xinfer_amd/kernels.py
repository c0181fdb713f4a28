"""Python bindings of the gfx950 kernel library (csrc/kernels/*.hip) through ctypes.

Every function checks on the host that operand shapes, types, devices and layouts match
what the kernel and its grid assume, and raises `KernelError` otherwise: a kernel is
never launched on operands it was not written for.  Kernels run on torch's current HIP
stream.  There is no other implementation behind these functions: if the library
cannot be built or loaded, importing fails loudly.
"""
from __future__ import annotations

import ctypes
import functools
from typing import Optional

import torch

from .csrc.build import load_kernels


class KernelError(RuntimeError):
    pass


F32, BF16 = 0, 1
_CODE = {torch.float32: F32, torch.bfloat16: BF16}

_lib = None


def lib():
    global _lib
    if _lib is None:
        l = load_kernels()
        l.xi_last_error.restype = ctypes.c_char_p
        _lib = l
    return _lib


def _code(t: torch.Tensor, what: str) -> int:
    try:
        return _CODE[t.dtype]
    except KeyError:
        raise KernelError(f"{what}: dtype {t.dtype} is not supported (float32 or bfloat16)") from None


def _dev(*tensors: Optional[torch.Tensor]) -> None:
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise KernelError("kernel operands must live on the GPU (there is no CPU path)")
        if not t.is_contiguous():
            raise KernelError(f"kernel operand of shape {tuple(t.shape)} is not contiguous")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise KernelError("kernel operands live on different devices")


def _p(t: Optional[torch.Tensor]) -> ctypes.c_void_p:
    return ctypes.c_void_p(t.data_ptr() if t is not None else 0)


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> ctypes.c_void_p:
    """The current HIP stream of the current device (asked for at every launch: the runner
    records graphs on a side stream)."""
    if _raw_stream is not None:
        return ctypes.c_void_p(_raw_stream(torch.cuda.current_device()))
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ok(rc: int) -> None:
    if rc != 0:
        raise KernelError(lib().xi_last_error().decode())


def _want(t: torch.Tensor, dtype: torch.dtype, what: str) -> None:
    if t.dtype != dtype:
        raise KernelError(f"{what} must be {dtype}, got {t.dtype}")


# ---------------------------------------------------------------------------------------
def embed(table: torch.Tensor, ids: torch.Tensor, out: Optional[torch.Tensor] = None, scale: float = 1.0) -> torch.Tensor:
    """out[t] = float32(table[ids[t]]) * scale.  ids: int32 [T], values in [0, rows) (caller checks)."""
    _dev(table, ids, out)
    _want(ids, torch.int32, "embed: ids")
    if table.dim() != 2 or ids.dim() != 1:
        raise KernelError("embed: table must be [V, H] and ids [T]")
    T, H = ids.shape[0], table.shape[1]
    if out is None:
        out = torch.empty((T, H), dtype=torch.float32, device=table.device)
    elif out.shape != (T, H) or out.dtype != torch.float32:
        raise KernelError("embed: out must be float32 [T, H]")
    _ok(lib().xi_embed(_p(table), _code(table, "embed"), _p(ids), _p(out), T, H, ctypes.c_float(scale), _stream()))
    return out


def counter_normal_(out: torch.Tensor, key: int, scale: float = 1.0, shift: float = 0.0, first: int = 0) -> torch.Tensor:
    """out.flat[i] = normal(key, first + i) * scale + shift, rounded once to out's type (float32 or
    bfloat16): seeded normal values that depend on (key, index) alone, bit for bit those of
    `weights.counter_normal.counter_normal` on the CPU."""
    _dev(out)
    if not (0 <= key < 1 << 64) or first < 0:
        raise KernelError("counter_normal: the key is a 64-bit number and the first index is not negative")
    _ok(lib().xi_counter_normal(_p(out), ctypes.c_uint64(out.numel()), ctypes.c_uint64(first), ctypes.c_uint64(key),
                                ctypes.c_float(scale), ctypes.c_float(shift), _code(out, "counter_normal"), _stream()))
    return out


def stream_read(t: torch.Tensor, workgroups: int = 2048, chunk_bytes: int = 1 << 18) -> None:
    """Reads all of a tensor's memory and keeps nothing: the plain read-only stream that the
    weight-streaming kernels are measured against.  A workgroup reads whole chunks of
    `chunk_bytes` (a multiple of 8 KB)."""
    _dev(t)
    _ok(lib().xi_stream_read(_p(t), ctypes.c_int64(t.numel() * t.element_size()), int(workgroups),
                             ctypes.c_int64(chunk_bytes), _stream()))


def lane_xor_probe(values: torch.Tensor) -> torch.Tensor:
    """values [64] float32 -> [8, 64]: row i < 6 holds values[l ^ (1 << i)] as the kernels' exchange
    between lanes gives it, row 6 the wave's sum and row 7 its maximum in every lane (for tests)."""
    _dev(values)
    _want(values, torch.float32, "lane_xor_probe: values")
    if values.shape != (64,):
        raise KernelError("lane_xor_probe: 64 values, one a lane")
    out = torch.empty((8, 64), dtype=torch.float32, device=values.device)
    _ok(lib().xi_lane_xor_probe(_p(values), _p(out), _stream()))
    return out


def softcap_(logits: torch.Tensor, cap: float) -> torch.Tensor:
    """logits = cap * tanh(logits / cap), in place, float32."""
    _dev(logits)
    _want(logits, torch.float32, "softcap: logits")
    if not cap > 0:
        raise KernelError(f"softcap: the cap must be positive, got {cap}")
    _ok(lib().xi_softcap(_p(logits), ctypes.c_int64(logits.numel()), ctypes.c_float(cap), _stream()))
    return logits


def add_rmsnorm(resid: torch.Tensor, y: Optional[torch.Tensor], weight: torch.Tensor, eps: float,
                out_dtype: torch.dtype, rows: Optional[torch.Tensor] = None,
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """s = resid (+ y); out = rms(s) * weight in `out_dtype`.  Without `rows` every row is
    normed and the sum is written back into resid; with `rows` (int32 indices) only those
    rows are produced and resid is left alone.  y may be a stack [P, T, H] of float32 partial
    sums, which are added in order."""
    _dev(resid, y, weight, rows, out)
    _want(resid, torch.float32, "add_rmsnorm: residual stream")
    _want(weight, torch.float32, "add_rmsnorm: weight")
    if resid.dim() != 2 or weight.shape != (resid.shape[1],):
        raise KernelError(f"add_rmsnorm: resid {tuple(resid.shape)} and weight {tuple(weight.shape)} do not match")
    parts = 1
    if y is not None and y.dim() == 3:
        if y.dtype != torch.float32 or tuple(y.shape[1:]) != tuple(resid.shape):
            raise KernelError(f"add_rmsnorm: partial sums {tuple(y.shape)} {y.dtype} must be float32 [P, T, H]")
        parts = int(y.shape[0])
    elif y is not None and y.shape != resid.shape:
        raise KernelError(f"add_rmsnorm: y {tuple(y.shape)} differs from resid {tuple(resid.shape)}")
    H = resid.shape[1]
    if rows is not None:
        _want(rows, torch.int32, "add_rmsnorm: rows")
        n = rows.shape[0]
    else:
        n = resid.shape[0]
    if out is None:
        out = torch.empty((n, H), dtype=out_dtype, device=resid.device)
    elif out.shape != (n, H) or out.dtype != out_dtype:
        raise KernelError("add_rmsnorm: out has the wrong shape or dtype")
    _ok(lib().xi_add_rmsnorm(_p(resid), _p(y), _code(y, "add_rmsnorm") if y is not None else F32, parts,
                             int(resid.shape[0]), _p(weight), ctypes.c_float(eps), _p(out),
                             _code(out, "add_rmsnorm"), _p(rows), n, H, _stream()))
    return out


def silu_mul(gate_up: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out = silu(gate_up[:, :I]) * gate_up[:, I:]"""
    _dev(gate_up, out)
    if gate_up.dim() != 2 or gate_up.shape[1] % 2:
        raise KernelError("silu_mul: input must be [T, 2I]")
    T, I = gate_up.shape[0], gate_up.shape[1] // 2
    if out is None:
        out = torch.empty((T, I), dtype=gate_up.dtype, device=gate_up.device)
    elif out.shape != (T, I) or out.dtype != gate_up.dtype:
        raise KernelError("silu_mul: out has the wrong shape or dtype")
    _ok(lib().xi_silu_mul(_p(gate_up), _p(out), _code(gate_up, "silu_mul"), T, I, _stream()))
    return out


def qk_norm_rope_kv(qkv: torch.Tensor, q_weight: Optional[torch.Tensor],
                    k_weight: Optional[torch.Tensor], eps: float, cos: torch.Tensor,
                    sin: torch.Tensor, rotary_dim: int, interleaved: bool,
                    positions: torch.Tensor, slots: torch.Tensor, k_cache: torch.Tensor,
                    v_cache: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int,
                    q_out: Optional[torch.Tensor] = None, v_grouped: bool = False,
                    vector_min_tokens: int = 128, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Per-head RMSNorm of q and k (if weights are given), rotation by position, q to q_out
    [T, nq, d], k and v into the paged cache [pages, nkv, page_size, d] at `slots`; with
    `v_grouped` the V pool is [pages, nkv, page_size / 8, d, 8] (eight keys side by side for every
    dim: what the matrix-core attention reads).  From `vector_min_tokens` tokens
    on, bfloat16 with the grouped pool runs the vectorized kernel.  `bias` (float32, one
    value per element of a packed row) is added to the rows first, in float32.  `qkv` may be a
    stack [slices, T, width] of float32 partial sums (`linear_mid`), added here in slice order;
    q and the cache then have the cache's dtype and the form of one wave per head runs."""
    _dev(qkv, q_weight, k_weight, cos, sin, positions, slots, k_cache, v_cache, q_out, bias)
    nq, nkv, d = num_heads, num_kv_heads, head_dim
    slices, dtype = 0, qkv.dtype
    if qkv.dim() == 3:            # float32 partial sums [slices, T, width] of a product cut along K
        _want(qkv, torch.float32, "qk_norm_rope_kv: partial sums")
        slices, dtype = int(qkv.shape[0]), k_cache.dtype
        if not (0 < slices <= 64) or not qkv.is_contiguous():
            raise KernelError(f"qk_norm_rope_kv: partial sums {tuple(qkv.shape)} must be contiguous [1..64, T, width]")
    T = qkv.shape[-2]
    if qkv.dim() not in (2, 3) or qkv.shape[-1] != (nq + 2 * nkv) * d:
        raise KernelError(f"qk_norm_rope_kv: qkv {tuple(qkv.shape)} is not [T, {(nq + 2 * nkv) * d}]")
    _want(positions, torch.int32, "qk_norm_rope_kv: positions")
    _want(slots, torch.int64, "qk_norm_rope_kv: slots")
    _want(cos, torch.float32, "qk_norm_rope_kv: cos")
    _want(sin, torch.float32, "qk_norm_rope_kv: sin")
    if positions.shape != (T,) or slots.shape != (T,):
        raise KernelError("qk_norm_rope_kv: positions and slots must be [T]")
    if cos.dim() != 2 or cos.shape[1] != rotary_dim // 2 or sin.shape != cos.shape:
        raise KernelError(f"qk_norm_rope_kv: cos/sin {tuple(cos.shape)} are not [positions, {rotary_dim // 2}]")
    for w in (q_weight, k_weight):
        if w is not None:
            _want(w, torch.float32, "qk_norm_rope_kv: norm weight")
            if w.shape != (d,):
                raise KernelError("qk_norm_rope_kv: norm weight must be [head_dim]")
    if bias is not None:
        _want(bias, torch.float32, "qk_norm_rope_kv: bias")
        if bias.shape != (qkv.shape[-1],):
            raise KernelError(f"qk_norm_rope_kv: bias {tuple(bias.shape)} is not [{qkv.shape[-1]}]")
    _check_cache(k_cache, v_cache, nkv, d, dtype, v_grouped, "qk_norm_rope_kv")
    if q_out is None:
        q_out = torch.empty((T, nq, d), dtype=dtype, device=qkv.device)
    elif q_out.shape != (T, nq, d) or q_out.dtype != dtype:
        raise KernelError("qk_norm_rope_kv: q_out has the wrong shape or dtype")
    _ok(lib().xi_qk_norm_rope_kv(
        _p(qkv), _code(q_out, "qk_norm_rope_kv"), slices, _p(bias), _p(q_weight), _p(k_weight), ctypes.c_float(eps),
        _p(cos), _p(sin), int(rotary_dim), int(bool(interleaved)), _p(positions), _p(slots),
        _p(q_out), _p(k_cache), _p(v_cache), int(k_cache.shape[2]), T, nq, nkv, d,
        int(bool(v_grouped)), int(vector_min_tokens), _stream()))
    return q_out


def _check_cache(k_cache, v_cache, nkv, d, dtype, v_grouped, what):
    """K pool [pages, nkv, page, d]; V pool the same, or [pages, nkv, page / 8, d, 8] if in groups of eight keys."""
    if k_cache.dim() != 4 or k_cache.shape[1] != nkv or k_cache.shape[3] != d or k_cache.dtype != dtype:
        raise KernelError(f"{what}: K pool {tuple(k_cache.shape)} {k_cache.dtype} does not match "
                          f"[pages, {nkv}, page_size, {d}] {dtype}")
    pages, _, page, _ = k_cache.shape
    if v_grouped and page % 8:
        raise KernelError(f"{what}: V in groups of eight keys needs pages of a multiple of 8 tokens, not {page}")
    want = (pages, nkv, page // 8, d, 8) if v_grouped else (pages, nkv, page, d)
    if tuple(v_cache.shape) != want or v_cache.dtype != dtype:
        raise KernelError(f"{what}: V pool {tuple(v_cache.shape)} {v_cache.dtype} does not match {want} {dtype}")


def attention_generic(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                      block_tables: torch.Tensor, tok_seq: torch.Tensor, positions: torch.Tensor,
                      scale: float, window: int = 0, out: Optional[torch.Tensor] = None,
                      v_grouped: bool = False) -> torch.Tensor:
    """Causal paged GQA attention for any mix of tokens.  q [T, nq, d]; caches
    [pages, nkv, page_size, d]; block_tables int32 [B, max_pages]; tok_seq / positions
    int32 [T] name each token's row of block_tables and its absolute position.
    window = 0 keeps all keys, w > 0 the last w (the query's own key included)."""
    _dev(q, k_cache, v_cache, block_tables, tok_seq, positions, out)
    if q.dim() != 3:
        raise KernelError("attention: q must be [T, nq, d]")
    T, nq, d = q.shape
    if k_cache.dim() != 4:
        raise KernelError("attention: the K pool must be [pages, nkv, page_size, d]")
    nkv, page = k_cache.shape[1], k_cache.shape[2]
    _check_cache(k_cache, v_cache, nkv, d, q.dtype, v_grouped, "attention")
    for t, name in ((block_tables, "block_tables"), (tok_seq, "tok_seq"), (positions, "positions")):
        _want(t, torch.int32, f"attention: {name}")
    if block_tables.dim() != 2 or tok_seq.shape != (T,) or positions.shape != (T,):
        raise KernelError("attention: block_tables must be [B, max_pages], tok_seq and positions [T]")
    if out is None:
        out = torch.empty((T, nq * d), dtype=q.dtype, device=q.device)
    elif out.shape != (T, nq * d) or out.dtype != q.dtype:
        raise KernelError("attention: out has the wrong shape or dtype")
    _ok(lib().xi_attention_generic(
        _p(q), _p(k_cache), _p(v_cache), _code(q, "attention"), _p(block_tables),
        int(block_tables.shape[1]), _p(tok_seq), _p(positions), _p(out), ctypes.c_float(scale),
        int(window), int(page), T, nq, nkv, d, int(bool(v_grouped)), _stream()))
    return out


def gemm_tn(x: torch.Tensor, w: torch.Tensor, out_dtype: Optional[torch.dtype] = None,
            out: Optional[torch.Tensor] = None, accumulate: bool = False) -> torch.Tensor:
    """y = x @ w.T with x [M, K], w [N, K]; float32 accumulation in ascending k.
    `accumulate` adds the product to `out` instead of overwriting it."""
    _dev(x, w, out)
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1]:
        raise KernelError(f"gemm: x {tuple(x.shape)} and w {tuple(w.shape)} do not match")
    if x.dtype != w.dtype:
        raise KernelError(f"gemm: x is {x.dtype} but w is {w.dtype}")
    M, K = x.shape
    N = w.shape[0]
    if out is None:
        if accumulate:
            raise KernelError("gemm: accumulate needs an output to add to")
        out = torch.empty((M, N), dtype=out_dtype or x.dtype, device=x.device)
    elif out.shape != (M, N) or (out_dtype is not None and out.dtype != out_dtype):
        raise KernelError("gemm: out has the wrong shape or dtype")
    _ok(lib().xi_gemm_tn(_p(x), _p(w), _p(out), M, N, K, _code(x, "gemm"), _code(out, "gemm"),
                         int(bool(accumulate)), _stream()))
    return out


DECODE_WORKGROUPS = 512             # workgroups of the split-K decode kernel a launch of mixed lengths aims at: two a compute unit
DECODE_KEYS_LEAST = 128             # keys of a workgroup: from one 32-key step a wave
DECODE_KEYS_MOST = 512              # to four, in batches of mixed lengths
DECODE_WORKGROUP_KEYS = 32          # what a workgroup costs beyond its keys (start, page numbers, merge, partial results), in keys
DECODE_SPLITS_MOST = 1024           # splits of a sequence that the search below tries
DECODE_WHOLE_KEYS = 2048            # mixed lengths, one and a half pairs a compute unit and more: a workgroup's keys at most


def decode_keys_per_workgroup(pairs: int, span: int, similar: bool = False) -> int:
    return _decode_keys_per_workgroup(int(pairs), int(span), bool(similar))


@functools.lru_cache(maxsize=4096)
def _decode_keys_per_workgroup(pairs: int, span: int, similar: bool) -> int:
    """Keys per workgroup of the split-K decode kernel for `pairs` (sequence, kv head) pairs of
    up to `span` keys (a multiple of 128; more than `span`: a workgroup takes a whole sequence and
    there is no second kernel).

    `similar` (the sequences are about equally long): the number of splits s that makes the least
    of rounds(s) * (keys of a split + DECODE_WORKGROUP_KEYS), rounds(s) = ceil(pairs * s /
    compute units): the compute units take the workgroups in turn, so the launch lasts as long
    as the unit with the most of them, and a workgroup costs about 32 keys' time beyond its keys.
    One round of large chunks wins where it exists (8 sequences of 4,096 keys on 8 kv heads: 4
    splits, 31.7 us against 32.2 at 8 and 33.8 at 16; 16 sequences of 8,500 keys, 64 query heads:
    2 splits, 104 us against 121 at 17; one sequence of 4,096: 32 splits of 128 keys, 11.2 us
    against 13.0 at 16), whole sequences from 256 pairs on.

    Otherwise (mixed lengths): 128, 256 or 512 keys, whichever makes about DECODE_WORKGROUPS
    workgroups: larger chunks lose there (64 sequences of 256 to 2,304 keys: 75 us at 512, 81 at
    1,024), since the short sequences' workgroups end early and the long ones' run on.  From one
    and a half pairs a compute unit on there are enough workgroups to even that out (the scheduler
    puts the long sequences first), and a workgroup's start and end cost more than the chunks'
    balance gains: whole sequences up to DECODE_WHOLE_KEYS keys, chunks of that many beyond (192
    sequences of 100 to 768 keys, longest first: 64 us against 72 in chunks of 512, and 80 in chunks
    of 512 in random order; 64 of 256 to 2,304: 64 against 68; 48 of 100 to 768: 20.5 against 21.9);
    from one pair a compute unit on chunks of 1,024 (32 sequences of 500 to 4,000: 60 us against 65
    at 512 and 63 whole)."""
    if similar:
        chunks = max(1, -(-int(span) // 128))
        plans = []
        for s in range(1, min(chunks, DECODE_SPLITS_MOST) + 1):
            kpw = -(-chunks // s) * 128
            splits = -(-chunks * 128 // kpw)
            cost = -(-pairs * splits // COMPUTE_UNITS) * (kpw + DECODE_WORKGROUP_KEYS)
            plans.append((cost, kpw, splits))
        # a workgroup alone on its compute unit does not draw the unit's share of the memory
        # bandwidth: with workgroups for fewer than seven eighths of the units more, smaller ones are
        # ahead (one sequence of 8,704 keys: 16.8 us in 544 workgroups of 128 keys, 18.9 in 184 of
        # 384; three of them: 27.4 us in 240 workgroups of 896 keys, 30.5 in 408 of 512)
        filling = [p for p in plans if pairs * p[2] >= COMPUTE_UNITS * 7 // 8]
        best = min(filling or [max(plans, key=lambda p: p[2])], key=lambda p: (p[0], -p[1]))
        if best[2] == 1:
            return (span + 128) // 128 * 128          # more than span: one split
        return best[1]
    if 2 * pairs >= 3 * COMPUTE_UNITS:
        return (span + 128) // 128 * 128 if span <= DECODE_WHOLE_KEYS else DECODE_WHOLE_KEYS
    if pairs >= COMPUTE_UNITS and span > 1024:
        return 1024
    kpw = DECODE_KEYS_LEAST
    while kpw < DECODE_KEYS_MOST and pairs * span >= 2 * kpw * DECODE_WORKGROUPS:
        kpw *= 2
    return kpw


def mfma_attention_supported(nq: int, nkv: int, d: int, page: int) -> bool:
    return bool(lib().xi_attention_mfma_supported(nq, nkv, d, page))


def decode_attention_takes(nq: int, nkv: int, d: int) -> bool:
    """Whether the split-K decode kernel takes these head counts and this head size: up to 16 query
    heads per kv head (the columns of one tile), and the waves' partial results of a group must
    fit the LDS through which they are merged."""
    g = nq // nkv
    return g <= 16 and (4 * g * d + 8 * g) * 4 <= 64 * 1024


def attention_prefill_bf16(q, k_cache, vt_cache, block_tables, tiles, cu_q, ctx_lens, scale, window=0, out=None,
                           small=False):
    """MFMA attention for any mix of portions.  tiles int32 [n, 2] = (sequence, first query
    token of a block of `prefill_block(d, nq // nkv, small)` tokens within the sequence's
    portion); `small` selects the workgroup shape (see `prefill_tiles`): 0 eight waves, 1 four
    waves and half the block, 2 (head sizes 32, 64, 128, 256) eight waves in two groups that split
    a tile's keys, the block of shape 1."""
    _dev(q, k_cache, vt_cache, block_tables, tiles, cu_q, ctx_lens, out)
    T, nq, d = q.shape
    nkv, page = k_cache.shape[1], k_cache.shape[2]
    _want(q, torch.bfloat16, "attention_prefill: q")
    _check_cache(k_cache, vt_cache, nkv, d, torch.bfloat16, True, "attention_prefill")
    for t, name in ((block_tables, "block_tables"), (tiles, "tiles"), (cu_q, "cu_q"), (ctx_lens, "ctx_lens")):
        _want(t, torch.int32, f"attention_prefill: {name}")
    B = ctx_lens.shape[0]
    if block_tables.shape[0] != B or cu_q.shape != (B + 1,) or tiles.dim() != 2 or tiles.shape[1] != 2:
        raise KernelError("attention_prefill: block_tables [B, pages], cu_q [B+1], ctx_lens [B], tiles [n, 2] expected")
    if out is None:
        out = torch.empty((T, nq * d), dtype=q.dtype, device=q.device)
    # head sizes 32, 64, 128, 256: the kernel whose tiles reach LDS through a ring of direct loads
    ring = PREFILL_RING and prefill_ring_supported(d)
    if int(small) == 2 and not ring:
        raise KernelError(f"attention_prefill: the shape of two groups of waves needs a head size of 32, 64, 128 or 256, got {d}")
    entry = lib().xi_attention_prefill_ring_bf16 if ring else lib().xi_attention_prefill_bf16
    _ok(entry(
        _p(q), _p(k_cache), _p(vt_cache), _p(block_tables), int(block_tables.shape[1]), _p(tiles),
        int(tiles.shape[0]), _p(cu_q), _p(ctx_lens), _p(out), ctypes.c_float(scale), int(window), int(page),
        nq, nkv, d, int(small), _stream()))
    return out


PREFILL_RING = True       # False: every head size goes to the kernel that copies tiles through registers


def prefill_ring_supported(d: int) -> bool:
    return bool(lib().xi_attention_prefill_ring_supported(int(d)))


def prefill_block(d: int, group: int = 1, small: bool = False) -> int:
    """Query positions per workgroup of the prefill kernel for a head size, a number of
    query heads per kv head and a workgroup shape."""
    return int(lib().xi_attention_prefill_block(int(d), int(group), int(small)))


COMPUTE_UNITS = 256
MIXED_DECODE_FROM = 4          # single-token sequences at the head of a mixed batch from which they may go to the decode
MIXED_DECODE_WORK = 40_000     # kernel: where sequences x longest context x reads of a kv head's keys reach this,
MIXED_DECODE_CONTEXT = 4096    # or the longest context this (measured on MI355X beside a portion of 2,000 tokens:
                               # 40 query heads on 8 kv heads, 64 sequences at 1,500 keys: 450 -> 155 us a layer)


def prefill_tiles(q_lens, ctx_lens, d: int, nq: int, nkv: int, small=None, first_seq: int = 0):
    """The query blocks of a batch of portions for the prefill kernel: (rows, shape).
    rows = [(sequence, first query of the block)] in launch order.  A block's work grows
    with the keys it sees, and the compute units take workgroups in launch order, so the
    blocks are sorted by work and laid out in a zigzag over rounds of one workgroup per
    compute unit.  The shape (chosen here unless given) is 0, eight waves and the full block,
    where that makes two workgroups a compute unit or more; with fewer blocks 1, four waves and
    half the block: twice the workgroups, two of them resident on a compute unit, and the
    zigzag gives a unit that got a long block in the first round a short one in the second; and
    with so few blocks that even those leave compute units with one workgroup (a prompt of 2,048
    tokens on 8 kv heads) 2, where the head size allows: eight waves in two groups that split a
    tile's keys, so that the longest block, which ends up alone on its unit, walks its keys with
    twice the waves (2,048 tokens, 32 query heads: 60 -> 56 us; 1,024: 31 -> 28).  Shape 0 has one
    workgroup per unit at a time: longest first."""
    g = nq // nkv
    heads = nkv * (g // (4 if g % 4 == 0 else 2 if g % 2 == 0 else 1))     # workgroups per query block
    big = prefill_block(d, g, False)
    if small is None:
        blocks = sum(-(-n // big) for n in q_lens[first_seq:])
        small = 0 if blocks * heads >= 2 * COMPUTE_UNITS else 1
        if small and PREFILL_RING and prefill_ring_supported(d):
            half = prefill_block(d, g, 1)
            if sum(-(-n // half) for n in q_lens[first_seq:]) * heads <= 2 * COMPUTE_UNITS:
                small = 2
    small = int(small)
    qb = prefill_block(d, g, small)
    rows = [(b, q0) for b, n in enumerate(q_lens) if b >= first_seq for q0 in range(0, n, qb)]
    rows.sort(key=lambda t: -(ctx_lens[t[0]] - q_lens[t[0]] + t[1]))
    per_round = max(1, COMPUTE_UNITS // heads)
    out = []
    for i in range(0, len(rows), per_round):
        chunk = rows[i:i + per_round]
        out += chunk if (small != 1 or (i // per_round) % 2 == 0) else chunk[::-1]
    return out, small


def attention_decode_bf16(q, k_cache, vt_cache, block_tables, ctx_lens, max_ctx_len, scale, window=0, out=None,
                          keys_per_workgroup=None, similar=False):
    """Split-K MFMA attention for a batch in which every sequence has one token (q [B, nq, d]).
    `keys_per_workgroup` (a multiple of 128) is chosen from the batch if not given (`similar`:
    see `decode_keys_per_workgroup`)."""
    _dev(q, k_cache, vt_cache, block_tables, ctx_lens, out)
    B, nq, d = q.shape
    nkv, page = k_cache.shape[1], k_cache.shape[2]
    _want(q, torch.bfloat16, "attention_decode: q")
    _check_cache(k_cache, vt_cache, nkv, d, torch.bfloat16, True, "attention_decode")
    _want(block_tables, torch.int32, "attention_decode: block_tables")
    _want(ctx_lens, torch.int32, "attention_decode: ctx_lens")
    if block_tables.shape[0] != B or ctx_lens.shape != (B,):
        raise KernelError("attention_decode: one block table row and one context length per sequence")
    span = min(int(max_ctx_len), int(window) + 31) if window > 0 else int(max_ctx_len)
    kpw = int(keys_per_workgroup or decode_keys_per_workgroup(B * nkv, span, similar))
    max_splits = span // kpw + 1
    part_o = torch.empty((B, nq, max_splits, d), dtype=torch.float32, device=q.device)
    part_ml = torch.empty((B, nq, max_splits, 2), dtype=torch.float32, device=q.device)
    if out is None:
        out = torch.empty((B, nq * d), dtype=q.dtype, device=q.device)
    _ok(lib().xi_attention_decode_bf16(
        _p(q), _p(k_cache), _p(vt_cache), _p(block_tables), int(block_tables.shape[1]), _p(ctx_lens), _p(out),
        _p(part_o), _p(part_ml), max_splits, kpw, ctypes.c_float(scale), int(window), int(page), B, nq, nkv, d,
        _stream()))
    return out


def attention_decode_packed_bf16(qkv, q_weight, k_weight, eps, cos, sin, rotary_dim, interleaved, positions, slots,
                                 k_cache, vt_cache, block_tables, ctx_lens, max_ctx_len, num_heads, scale, window=0,
                                 bias=None, out=None, keys_per_workgroup=None, similar=False):
    """What `qk_norm_rope_kv` and `attention_decode_bf16` do one after the other for a batch in which
    every sequence has one token, in one launch less: `qkv` is the packed projection
    [B, (nq + 2 nkv) d] in bfloat16, or a stack [slices, B, width] of float32 partial sums; the new
    keys and values go into the cache at `slots` on the way (the same bits as the other kernel's)."""
    _dev(qkv, q_weight, k_weight, cos, sin, positions, slots, k_cache, vt_cache, block_tables, ctx_lens, out, bias)
    nq, nkv, page, d = int(num_heads), k_cache.shape[1], k_cache.shape[2], k_cache.shape[3]
    slices = 0
    if qkv.dim() == 3:
        _want(qkv, torch.float32, "attention_decode_packed: partial sums")
        slices = int(qkv.shape[0])
        if not (0 < slices <= 64):
            raise KernelError(f"attention_decode_packed: {slices} slices of partial sums, at most 64")
    else:
        _want(qkv, torch.bfloat16, "attention_decode_packed: qkv")
    if qkv.dim() not in (2, 3) or qkv.shape[-1] != (nq + 2 * nkv) * d:
        raise KernelError(f"attention_decode_packed: qkv {tuple(qkv.shape)} is not [B, {(nq + 2 * nkv) * d}]")
    B = int(qkv.shape[-2])
    _check_cache(k_cache, vt_cache, nkv, d, torch.bfloat16, True, "attention_decode_packed")
    _want(block_tables, torch.int32, "attention_decode_packed: block_tables")
    _want(ctx_lens, torch.int32, "attention_decode_packed: ctx_lens")
    _want(positions, torch.int32, "attention_decode_packed: positions")
    _want(slots, torch.int64, "attention_decode_packed: slots")
    _want(cos, torch.float32, "attention_decode_packed: cos")
    _want(sin, torch.float32, "attention_decode_packed: sin")
    if block_tables.shape[0] != B or ctx_lens.shape != (B,) or positions.shape != (B,) or slots.shape != (B,):
        raise KernelError("attention_decode_packed: one block table row, context length, position and slot per sequence")
    if cos.dim() != 2 or cos.shape[1] != rotary_dim // 2 or sin.shape != cos.shape:
        raise KernelError(f"attention_decode_packed: cos/sin {tuple(cos.shape)} are not [positions, {rotary_dim // 2}]")
    for w in (q_weight, k_weight):
        if w is not None:
            _want(w, torch.float32, "attention_decode_packed: norm weight")
            if w.shape != (d,):
                raise KernelError("attention_decode_packed: norm weight must be [head_dim]")
    if bias is not None:
        _want(bias, torch.float32, "attention_decode_packed: bias")
        if bias.shape != (qkv.shape[-1],):
            raise KernelError(f"attention_decode_packed: bias {tuple(bias.shape)} is not [{qkv.shape[-1]}]")
    span = min(int(max_ctx_len), int(window) + 31) if window > 0 else int(max_ctx_len)
    kpw = int(keys_per_workgroup or decode_keys_per_workgroup(B * nkv, span, similar))
    max_splits = span // kpw + 1
    part_o = torch.empty((B, nq, max_splits, d), dtype=torch.float32, device=qkv.device)
    part_ml = torch.empty((B, nq, max_splits, 2), dtype=torch.float32, device=qkv.device)
    if out is None:
        out = torch.empty((B, nq * d), dtype=torch.bfloat16, device=qkv.device)
    elif out.shape != (B, nq * d) or out.dtype != torch.bfloat16 or not out.is_contiguous():
        raise KernelError("attention_decode_packed: out has the wrong shape or dtype")
    _ok(lib().xi_attention_decode_packed_bf16(
        _p(qkv), slices, _p(bias), _p(q_weight), _p(k_weight), ctypes.c_float(eps), _p(cos), _p(sin), int(rotary_dim),
        int(bool(interleaved)), _p(positions), _p(slots), _p(k_cache), _p(vt_cache), _p(block_tables),
        int(block_tables.shape[1]), _p(ctx_lens), _p(out), _p(part_o), _p(part_ml), max_splits, kpw,
        ctypes.c_float(scale), int(window), int(page), B, nq, nkv, d, _stream()))
    return out


def attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, ctx, group: int,
              scale: float, window: int = 0, v_grouped: bool = False) -> torch.Tensor:
    """Attention of one step's tokens over the paged cache of `group`; chooses the kernel
    from the precision and the shape of the batch: float32, or sizes the matrix-core
    kernels do not take, go to the generic kernel; bfloat16 batches of single tokens to
    the split-K decode kernel; everything else to the prefill kernel."""
    T, nq, d = q.shape
    nkv, page = k_cache.shape[1], k_cache.shape[2]
    bt = ctx.block_tables[group]
    if q.dtype == torch.bfloat16 and v_grouped and mfma_attention_supported(nq, nkv, d, page):
        g = nq // nkv
        if ctx.max_q_len == 1 and decode_attention_takes(nq, nkv, d):
            return attention_decode_bf16(q, k_cache, v_cache, bt, ctx.ctx_lens, ctx.max_ctx_len, scale, window,
                                         similar=getattr(ctx, "similar_lengths", False))
        key = ("attention_tiles", d, nq, nkv)
        cached = ctx.scratch.get(key)
        if cached is None:
            q_lens = [ctx.cu_q_host[b + 1] - ctx.cu_q_host[b] for b in range(ctx.num_seqs)]
            # The sequences at the head of the batch that bring one token (the scheduler puts the
            # decoding requests first) go to the decode kernel, which reads a kv head's keys once
            # for all its query heads and splits a context over workgroups; the prefill kernel
            # would give each of them a 16-row tile with one row in use.
            # The two kernels run one after the other, so it pays only where the prefill kernel
            # would have much to do for those sequences: keys times the times it reads them (once
            # per group of query heads it takes together), or a long context for one workgroup to walk.
            lead = 0
            while lead < len(q_lens) and q_lens[lead] == 1:
                lead += 1
            lead_ctx = max(ctx.ctx_lens_host[:lead]) if lead else 0
            reads = g // (4 if g % 4 == 0 else 2 if g % 2 == 0 else 1)
            if (lead < MIXED_DECODE_FROM or not decode_attention_takes(nq, nkv, d)
                    or not (lead * lead_ctx * reads >= MIXED_DECODE_WORK or lead_ctx >= MIXED_DECODE_CONTEXT)):
                lead = 0
            rows, small = prefill_tiles(q_lens, ctx.ctx_lens_host, d, nq, nkv, first_seq=lead)
            cached = (torch.tensor(rows, dtype=torch.int32, device=q.device).reshape(-1, 2), small, lead,
                      lead_ctx if lead else 0)
            ctx.scratch[key] = cached
        tiles, small, lead, lead_ctx = cached
        out = None
        if lead:
            out = torch.empty((T, nq * d), dtype=q.dtype, device=q.device)
            attention_decode_bf16(q[:lead], k_cache, v_cache, bt[:lead], ctx.ctx_lens[:lead], lead_ctx, scale, window,
                                  out=out[:lead])
        return attention_prefill_bf16(q, k_cache, v_cache, bt, tiles, ctx.cu_q, ctx.ctx_lens, scale, window,
                                      out=out, small=small)
    return attention_generic(q, k_cache, v_cache, bt, ctx.tok_seq, ctx.positions, scale, window,
                             v_grouped=v_grouped)


SKINNY_MAX_ROWS = 64      # most rows the streaming kernel takes
SKINNY_ROWS = 8           # up to this many rows it is faster than the vendor library (measured)
SKINNY_SPLIT_ROWS = 64    # the same where the consumer takes partial sums over slices of K,
SKINNY_SPLIT_FROM = 17    # which pays from this many rows on (fewer rows: the unsplit product)
SKINNY_GATED_ROWS = 32    # the same for the fused gate/up/silu form, which also saves a kernel


def linear_skinny(x: torch.Tensor, w: torch.Tensor, out_dtype: Optional[torch.dtype] = None,
                  gated: bool = False, out: Optional[torch.Tensor] = None, allow_split: bool = False,
                  row_tiles: int = 0, waves: int = 0) -> torch.Tensor:
    """bfloat16 x [M, K] @ w [N, K]^T for M <= 64 rows with the streaming matrix-core kernel.
    `gated`: w is [2N, K] = [gate; up] and the result is silu(x @ gate^T) * (x @ up^T), [M, N].
    `allow_split`: for narrow outputs the kernel may cut K into slices across workgroups and
    return float32 partial sums [slices, M, N] for the consumer to add in order (the fused
    add + RMSNorm does).  `row_tiles`, `waves`: 0 = chosen from the sizes."""
    _dev(x, w, out)
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise KernelError("linear_skinny: operands must be bfloat16")
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1]:
        raise KernelError(f"linear_skinny: x {tuple(x.shape)} and w {tuple(w.shape)} do not match")
    M, K = x.shape
    N = w.shape[0]
    if gated:
        if N % 2:
            raise KernelError("linear_skinny: a gated weight must be [2N, K]")
        N //= 2
    if M > SKINNY_MAX_ROWS or K % 8:
        raise KernelError(f"linear_skinny: M={M} must be <= {SKINNY_MAX_ROWS} and K={K} a multiple of 8")
    assert SKINNY_MAX_ROWS == int(lib().xi_linear_skinny_max_rows())
    slices = int(lib().xi_linear_skinny_slices(N, K, int(bool(gated)), int(bool(allow_split))))
    if slices > 1:
        out_dtype, shape = torch.float32, (slices, M, N)
    else:
        out_dtype, shape = out_dtype or torch.bfloat16, (M, N)
    if out is None:
        out = torch.empty(shape, dtype=out_dtype, device=x.device)
    elif tuple(out.shape) != shape or out.dtype != out_dtype:
        raise KernelError("linear_skinny: out has the wrong shape or dtype")
    _ok(lib().xi_linear_skinny(_p(x), _p(w), _p(out), M, N, K, _code(out, "linear_skinny"), int(bool(gated)),
                               int(bool(allow_split)), int(row_tiles), int(waves), _stream()))
    return out


def linear_skinny_plan(M: int, N: int, K: int, gated: bool = False, allow_split: bool = False):
    """What `linear_skinny` chooses for these sizes: (slices of K, row tiles per workgroup, output
    features per workgroup, workgroups).  Only the slices change a sum's order."""
    L = lib()
    ks = int(L.xi_linear_skinny_slices(N, K, int(bool(gated)), int(bool(allow_split))))
    rt = int(L.xi_linear_skinny_row_tiles(M, N, K, int(bool(gated)), int(bool(allow_split))))
    rows = int(L.xi_linear_skinny_rows(M, N, K, int(bool(gated)), int(bool(allow_split))))
    return ks, rt, rows, -(-N // rows) * ks


MID_ROTATE = 1            # workgroup tile t of the tiled products starts t * this many k tiles into its slice and
MID_GATED_ROTATE = 1      # wraps around (0: all start at the slice's first tile, which measured 5% slower in a
                          # decode step: every workgroup then asks for the same offset of its rows at the same time)
MID_ROWS = 256            # most rows of the tiled product for narrow outputs (`linear_mid`)
MID_WIDE_FROM = 4         # rows from which it is ahead of the streaming kernel on an output so wide that it needs no
                          # slices (the head: 215 against 242 us at 8 rows, 238 against 349 at 64, vocabulary 151936)
MID_FROM = 17             # from this many rows on it is used, where the caller takes partial sums,
MID_WIDEST = 12288        # for outputs up to this wide (N = 10240, K = 5120: 21 / 23 / 30 us at 17 / 64 / 128 rows against
                          # 24 / 31 / 39 in the library), and above 128 rows (two passes over w) for weights from
MID_BLOCK = 128           # (rows of one pass)
MID_TWO_BLOCKS = 32 << 20  # this many bytes on (below, the library is ahead: 8 MB at 256 rows, 16 against 9 us)


def linear_mid_slices(N: int, K: int) -> int:
    """The slices of K in which `linear_mid` answers for an output of N features; 0 if it does
    not take the sizes."""
    return int(lib().xi_linear_mid_slices(int(N), int(K)))


def linear_mid(x: torch.Tensor, w: torch.Tensor, depth: int = 0) -> torch.Tensor:
    """bfloat16 x [M, K] @ w [N, K]^T for up to MID_ROWS rows as float32 partial sums
    [slices, M, N], to be added in order (the fused add + RMSNorm does): the tiled kernel for
    decode batches too large for `linear_skinny` and outputs too narrow for the library.
    `depth`: tiles of loads a thread keeps in flight, 0 = the default; the result does not depend on it."""
    _dev(x, w)
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise KernelError("linear_mid: operands must be bfloat16")
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1]:
        raise KernelError(f"linear_mid: x {tuple(x.shape)} and w {tuple(w.shape)} do not match")
    M, K = x.shape
    N = w.shape[0]
    slices = linear_mid_slices(N, K)
    if not (0 < M <= MID_ROWS) or slices < 1:
        raise KernelError(f"linear_mid: M={M} must be 1..{MID_ROWS} and K={K} a multiple of 64")
    y = torch.empty((slices, M, N), dtype=torch.float32, device=x.device)
    _ok(lib().xi_linear_mid(_p(x), _p(w), _p(y), M, N, K, int(depth), int(MID_ROTATE), _stream()))
    return y


TILE_SPLIT_ROWS = 1024        # most rows of a product that the many-row tiled kernel takes with K cut into slices
TILE_SPLIT_K = 512            # least K of a slice
TILE_SPLIT_BYTES = 8 << 20    # a weight up to this size is left to the library (level there, measured at Qwen3-0.6B sizes)
TILE_SHAPES = ((128, 256), (256, 128), (256, 256))     # rows of x by rows of w a workgroup, by `shape` of `linear_tile`
TILE_FILL_RATE = 58e9         # bytes a second that one compute unit's loads bring into its LDS
TILE_STREAM_RATE = 5e12       # bytes a second that the chip streams from memory


def tile_split_plan(M: int, N: int, K: int):
    """(slices, tile shape) of x [M, K] @ w [N, K]^T in the many-row tiled kernel (`linear_tile`) for a
    narrow output at 129 to 1,024 rows, slices 1 = it is not used.  A narrow output gives too few
    tiles for the chip's 256 compute units (256 rows by 4,096 features: 32 tiles of 256 x 128), so K
    is cut into slices, each a workgroup's own, with float32 partial sums [slices, M, N] for the
    caller to add in order.  Slices (2 to 16, whole tiles of 64 k, a slice at least 512 long) and tile shape are
    those with the least cost in a model of two terms that fits what was measured on MI355X within a
    tenth: a workgroup brings (rows of x + rows of w of its tile) x its slice of K into LDS at 58 GB/s
    (that, not the matrix cores, bounds these shapes: x is fetched again by every workgroup, so
    tiles with as many rows of w as of x are ahead where x is a whole tile's rows), rounds of 256
    workgroups one after the other, never faster than the weight streams from memory; and the
    partial sums are written and read again, 8 bytes an element and slice.  256 rows of N = 5120,
    K = 17408: 4 slices of 256 x 128 tiles 71 us, 8 slices of 256 x 256 tiles 55.  Beyond 256 rows
    only for K >= 2 N (the down projection): the reader of the partial sums reads `slices` float32
    values for every bfloat16 one, which a smaller gain does not pay for.  Up to 128 rows the tiled
    kernel of few rows (`linear_mid`) is level or ahead."""
    if not (MID_BLOCK < M <= TILE_SPLIT_ROWS) or (M > MID_ROWS and K < 2 * N) or N % 4 or K % 64 \
            or N * K * 2 <= TILE_SPLIT_BYTES:
        return 1, 0
    best = None
    k_tiles = K // 64
    for shape in ((1, 0, 2) if M <= 256 else (0, 1, 2)):      # (among equals: every row of w in one workgroup)
        bm, bn = TILE_SHAPES[shape]
        tiles = -(-M // bm) * -(-N // bn)
        for slices in range(2, 17):
            longest = -(-k_tiles // slices) * 64               # the slices differ by a tile at most
            if longest < TILE_SPLIT_K:
                break
            rounds = -(-tiles * slices // COMPUTE_UNITS)
            fill = rounds * (bm + bn) * longest * 2 / TILE_FILL_RATE
            cost = max(fill, N * K * 2 / TILE_STREAM_RATE) + slices * M * N * 8 / TILE_STREAM_RATE
            if best is None or cost < best[0] - 1e-9:
                best = (cost, slices, shape)
    return (best[1], best[2]) if best is not None else (1, 0)


def linear_tile_takes(M: int, N: int, K: int, slices: int = 1) -> bool:
    """Whether the many-row tiled product takes a shape: K in whole tiles of 64, a tile a slice at least, N in fours."""
    return bool(lib().xi_linear_tile_takes(int(M), int(N), int(K), int(slices)))


def linear_tile(x: torch.Tensor, w: torch.Tensor, slices: int = 1, partial: bool = False,
                shape: Optional[int] = None) -> torch.Tensor:
    """bfloat16 x [M, K] @ w [N, K]^T on the matrix cores for many rows: bfloat16 [M, N], or with
    `partial` (needed for more than one slice) float32 partial sums [slices, M, N] over slices of K
    (whole tiles of 64, equal but for one tile).  `shape` 0: workgroup tiles of 128 rows by 256 features, 1: 256 by 128; None: the
    one that makes fewer tiles (128 by 256 at equal numbers); 2: 256 by 256."""
    _dev(x, w)
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise KernelError("linear_tile: operands must be bfloat16")
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1]:
        raise KernelError(f"linear_tile: x {tuple(x.shape)} and w {tuple(w.shape)} do not match")
    M, K = x.shape
    N = w.shape[0]
    partial = bool(partial) or slices > 1
    if not linear_tile_takes(M, N, K, slices):
        raise KernelError(f"linear_tile: M={M} N={N} K={K} in {slices} slices is not taken")
    if shape is None:
        shape = 1 if -(-M // 256) * -(-N // 128) < -(-M // 128) * -(-N // 256) else 0
    if partial:
        y = torch.empty((slices, M, N), dtype=torch.float32, device=x.device)
    else:
        y = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    _ok(lib().xi_linear_tile(_p(x), _p(w), _p(y), M, N, K, int(slices), int(partial), int(shape), _stream()))
    return y


MID_GATED_ROWS = 128      # most rows of the gated form of the tiled product
MID_GATED_FEATURES = 0    # features a workgroup of it owns; 0: chosen from N (the fewest workgroups that are a multiple of 256)
MID_GATED_UP_TO = 64      # it is used up to this many rows (more: its reads of x from L2 outweigh the library's
                          # weakness); measured on MI355X at the gate/up sizes of Qwen3-8B, 14B and 32B, it is
MID_GATED_FROM = 2        # ahead of the streaming kernel from this many rows on, and from the first row where
MID_GATED_BIG = 300 << 20  # the weight has this many bytes (the streaming kernel falls behind on large weights)


def gated_uses_mid(M: int, w: torch.Tensor) -> bool:
    """Whether the gated product of M rows with w [2N, K] goes to `linear_mid_gated`."""
    if w.dtype != torch.bfloat16 or w.shape[1] % 64 or w.shape[1] < 64 or w.shape[0] % 2:
        return False
    return (MID_GATED_FROM <= M <= MID_GATED_UP_TO) or (0 < M < MID_GATED_FROM and w.numel() * 2 >= MID_GATED_BIG)


def linear_mid_gated(x: torch.Tensor, w: torch.Tensor, ss: Optional[torch.Tensor] = None, eps: float = 0.0,
                     features: Optional[int] = None) -> torch.Tensor:
    """silu(x @ gate^T) * (x @ up^T) in bfloat16 for w = [gate; up] [2N, K] and up to MID_GATED_ROWS
    rows with the tiled kernel: one pass over w whatever the number of rows.  `ss` [M, parts]
    float32 (up to FOLD_ROWS rows): x is the first half of a folded RMSNorm (`linear_fold_out`)
    and the rows of the products are multiplied by rsqrt(sum(ss[row]) / K + eps) first.
    `features`: the features a workgroup owns (up to 64, up to 128 for up to 64 rows), for
    measurements and tests; chosen from the sizes if not given."""
    _dev(x, w, ss)
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise KernelError("linear_mid_gated: operands must be bfloat16")
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1] or w.shape[0] % 2:
        raise KernelError(f"linear_mid_gated: x {tuple(x.shape)} and w {tuple(w.shape)} ([2N, K]) do not match")
    M, K = x.shape
    N = w.shape[0] // 2
    if not (0 < M <= MID_GATED_ROWS) or K % 64 or K < 64:
        raise KernelError(f"linear_mid_gated: M={M} must be 1..{MID_GATED_ROWS} and K={K} a multiple of 64")
    parts = 0
    if ss is not None:
        _want(ss, torch.float32, "linear_mid_gated: ss")
        if M > FOLD_ROWS or ss.dim() != 2 or ss.shape[0] != M or not (0 < ss.shape[1] <= FOLD_PARTS):
            raise KernelError(f"linear_mid_gated: a folded norm takes up to {FOLD_ROWS} rows and ss [M, up to "
                              f"{FOLD_PARTS} parts], got M={M}, ss {tuple(ss.shape)}")
        parts = int(ss.shape[1])
    y = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    _ok(lib().xi_linear_mid_gated(_p(x), _p(w), _p(y), M, N, K, _p(ss), parts, ctypes.c_float(eps), int(MID_GATED_ROTATE),
                                  int(features if features is not None else MID_GATED_FEATURES), _stream()))
    return y


FOLD_ROWS = 16            # most rows of the products that carry a folded norm between them
FOLD_PARTS = 512          # most parts of a row's sum of squares the product after the norm adds up


def linear_fold_parts(M: int, N: int, K: int) -> int:
    """The parts in which `linear_fold_out` hands on each row's sum of squares for these sizes."""
    return int(lib().xi_linear_skinny_fold_parts(int(M), int(N), int(K)))


def linear_fold_out(x: torch.Tensor, w: torch.Tensor, resid: torch.Tensor, norm_weight: torch.Tensor):
    """The product before an RMSNorm, for up to FOLD_ROWS rows: resid [M, N] float32 += x [M, K] @
    w [N, K]^T in place; returns (xg, ss): xg [M, N] bfloat16 = round(resid * norm_weight), ss
    [M, parts] float32 the sums of squares of the rows of resid in parts.  `linear_fold_in` is the
    product after the norm; between them no norm kernel runs."""
    _dev(x, w, resid, norm_weight)
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise KernelError("linear_fold_out: operands must be bfloat16")
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1]:
        raise KernelError(f"linear_fold_out: x {tuple(x.shape)} and w {tuple(w.shape)} do not match")
    M, K = x.shape
    N = w.shape[0]
    if not (0 < M <= FOLD_ROWS) or K % 8:
        raise KernelError(f"linear_fold_out: M={M} must be 1..{FOLD_ROWS} and K={K} a multiple of 8")
    _want(resid, torch.float32, "linear_fold_out: resid")
    _want(norm_weight, torch.float32, "linear_fold_out: norm weight")
    if tuple(resid.shape) != (M, N) or tuple(norm_weight.shape) != (N,) or not resid.is_contiguous():
        raise KernelError(f"linear_fold_out: resid {tuple(resid.shape)} / norm weight {tuple(norm_weight.shape)} "
                          f"do not match [M={M}, N={N}]")
    parts = linear_fold_parts(M, N, K)
    xg = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    ss = torch.empty((M, parts), dtype=torch.float32, device=x.device)
    _ok(lib().xi_linear_skinny_fold_out(_p(x), _p(w), M, N, K, _p(resid), _p(norm_weight), _p(xg), _p(ss), _stream()))
    return xg, ss


def linear_fold_in(xg: torch.Tensor, ss: torch.Tensor, eps: float, w: torch.Tensor,
                   out_dtype: Optional[torch.dtype] = None, gated: bool = False) -> torch.Tensor:
    """The product after an RMSNorm whose first half `linear_fold_out` did: (xg @ w^T) with each
    row multiplied by rsqrt(sum(ss[row]) / K + eps), one rounding; `gated` as in `linear_skinny`."""
    _dev(xg, ss, w)
    if xg.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise KernelError("linear_fold_in: operands must be bfloat16")
    if xg.dim() != 2 or w.dim() != 2 or xg.shape[1] != w.shape[1]:
        raise KernelError(f"linear_fold_in: x {tuple(xg.shape)} and w {tuple(w.shape)} do not match")
    M, K = xg.shape
    N = w.shape[0]
    if gated:
        if N % 2:
            raise KernelError("linear_fold_in: a gated weight must be [2N, K]")
        N //= 2
    _want(ss, torch.float32, "linear_fold_in: ss")
    if not (0 < M <= FOLD_ROWS) or K % 8 or ss.dim() != 2 or ss.shape[0] != M or not (0 < ss.shape[1] <= FOLD_PARTS) \
            or not ss.is_contiguous():
        raise KernelError(f"linear_fold_in: M={M} (1..{FOLD_ROWS}), K={K} (multiple of 8), ss {tuple(ss.shape)} "
                          f"([M, up to {FOLD_PARTS} parts])")
    out_dtype = out_dtype or torch.bfloat16
    if gated and out_dtype != torch.bfloat16:
        raise KernelError("linear_fold_in: the gated form writes bfloat16")
    y = torch.empty((M, N), dtype=out_dtype, device=xg.device)
    _ok(lib().xi_linear_skinny_fold_in(_p(xg), _p(w), _p(y), M, N, K, _code(y, "linear_fold_in"), int(bool(gated)),
                                       _p(ss), int(ss.shape[1]), ctypes.c_float(eps), _stream()))
    return y


THIN_ROTATE = 0           # workgroup b of the thin product starts b * this many k tiles into K (see MID_ROTATE;
                          # here it measured no gain: 0)


def thin_ahead(M: int, w: torch.Tensor) -> bool:
    """Whether a product of M <= FOLD_ROWS rows with whole sums goes to the thin kernel: wherever it
    takes the sizes (K a multiple of 256).  Measured in decode steps at Qwen3-8B, 14B and 32B sizes
    against the streaming kernel: level at one row, 1 to 3% of a step ahead from two rows on."""
    if w.dtype != torch.bfloat16 or not (0 < M <= FOLD_ROWS):
        return False
    return 0 < linear_thin_parts(w.shape[0], w.shape[1]) <= FOLD_PARTS


def linear_thin_parts(N: int, K: int) -> int:
    """Workgroups of the thin product for an output of N features (the parts in which
    `linear_thin_fold_out` hands on a row's sum of squares); 0 if it does not take the sizes."""
    return int(lib().xi_linear_thin_parts(int(N), int(K)))


def _thin_operands(what: str, x: torch.Tensor, w: torch.Tensor):
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise KernelError(f"{what}: operands must be bfloat16")
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1]:
        raise KernelError(f"{what}: x {tuple(x.shape)} and w {tuple(w.shape)} do not match")
    M, K = x.shape
    N = w.shape[0]
    if not (0 < M <= FOLD_ROWS) or linear_thin_parts(N, K) < 1:
        raise KernelError(f"{what}: M={M} must be 1..{FOLD_ROWS} and K={K} a multiple of 256")
    return M, N, K


def linear_thin(x: torch.Tensor, w: torch.Tensor, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """bfloat16 x [M, K] @ w [N, K]^T for up to FOLD_ROWS rows, whole sums (no slices of K) with few
    output features per workgroup, loaded as whole lines through LDS: the shape of the products
    around a folded norm."""
    _dev(x, w)
    M, N, K = _thin_operands("linear_thin", x, w)
    y = torch.empty((M, N), dtype=out_dtype or torch.bfloat16, device=x.device)
    _ok(lib().xi_linear_thin(_p(x), _p(w), _p(y), M, N, K, _code(y, "linear_thin"), int(THIN_ROTATE), _stream()))
    return y


def linear_thin_fold_out(x: torch.Tensor, w: torch.Tensor, resid: torch.Tensor, norm_weight: torch.Tensor):
    """`linear_fold_out` with the thin kernel: resid [M, N] float32 += x @ w^T in place; returns
    (xg, ss) with ss [M, linear_thin_parts(N, K)]."""
    _dev(x, w, resid, norm_weight)
    M, N, K = _thin_operands("linear_thin_fold_out", x, w)
    _want(resid, torch.float32, "linear_thin_fold_out: resid")
    _want(norm_weight, torch.float32, "linear_thin_fold_out: norm weight")
    if tuple(resid.shape) != (M, N) or tuple(norm_weight.shape) != (N,):
        raise KernelError(f"linear_thin_fold_out: resid {tuple(resid.shape)} / norm weight {tuple(norm_weight.shape)} "
                          f"do not match [M={M}, N={N}]")
    xg = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    ss = torch.empty((M, linear_thin_parts(N, K)), dtype=torch.float32, device=x.device)
    _ok(lib().xi_linear_thin_fold_out(_p(x), _p(w), M, N, K, _p(resid), _p(norm_weight), _p(xg), _p(ss),
                                      int(THIN_ROTATE), _stream()))
    return xg, ss


def linear_thin_fold_in(xg: torch.Tensor, ss: torch.Tensor, eps: float, w: torch.Tensor,
                        out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """`linear_fold_in` (plain form) with the thin kernel."""
    _dev(xg, ss, w)
    M, N, K = _thin_operands("linear_thin_fold_in", xg, w)
    _want(ss, torch.float32, "linear_thin_fold_in: ss")
    if ss.dim() != 2 or ss.shape[0] != M or not (0 < ss.shape[1] <= FOLD_PARTS):
        raise KernelError(f"linear_thin_fold_in: ss {tuple(ss.shape)} is not [M={M}, up to {FOLD_PARTS} parts]")
    y = torch.empty((M, N), dtype=out_dtype or torch.bfloat16, device=xg.device)
    _ok(lib().xi_linear_thin_fold_in(_p(xg), _p(w), _p(y), M, N, K, _code(y, "linear_thin_fold_in"), _p(ss),
                                     int(ss.shape[1]), ctypes.c_float(eps), int(THIN_ROTATE), _stream()))
    return y


def linear_bf16(x: torch.Tensor, w: torch.Tensor, out_dtype: Optional[torch.dtype] = None,
                skinny_rows: int = SKINNY_ROWS, allow_split: bool = False) -> torch.Tensor:
    """bfloat16 x @ w.T with float32 accumulation, rounded once to `out_dtype` (bfloat16 or
    float32).  Up to `skinny_rows` rows (decode): the hand-written streaming kernel, which with
    `allow_split` may answer with float32 partial sums [slices, M, N] for a narrow output.  More
    rows: the vendor library (hipBLASLt through torch), which the reference's engine also
    uses for its matrix products."""
    _dev(x, w)
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise KernelError("linear_bf16: operands must be bfloat16")
    out_dtype = out_dtype or torch.bfloat16
    if out_dtype == torch.float32 and MID_WIDE_FROM <= x.shape[0] <= MID_GATED_ROWS \
            and linear_mid_slices(w.shape[0], w.shape[1]) == 1:
        return linear_mid(x, w)[0]           # a wide output in float32 (the head): one slice is the result
    if allow_split and MID_BLOCK < x.shape[0] <= TILE_SPLIT_ROWS:
        slices, shape = tile_split_plan(x.shape[0], w.shape[0], w.shape[1])
        if slices > 1:
            return linear_tile(x, w, slices, partial=True, shape=shape)
    if allow_split and MID_FROM <= x.shape[0] <= MID_ROWS and linear_mid_slices(w.shape[0], w.shape[1]) > 0 \
            and w.shape[0] <= MID_WIDEST and (x.shape[0] <= MID_BLOCK or w.numel() * 2 >= MID_TWO_BLOCKS):
        return linear_mid(x, w)
    if (allow_split and x.shape[1] % 8 == 0 and x.shape[0] >= SKINNY_SPLIT_FROM
            and int(lib().xi_linear_skinny_slices(w.shape[0], w.shape[1], 0, 1)) > 1):
        skinny_rows = max(skinny_rows, SKINNY_SPLIT_ROWS)
    else:
        allow_split = False
    if not allow_split and thin_ahead(x.shape[0], w):
        return linear_thin(x, w, out_dtype)
    if 0 < x.shape[0] <= min(skinny_rows, SKINNY_MAX_ROWS) and x.shape[1] % 8 == 0:
        return linear_skinny(x, w, out_dtype, allow_split=allow_split)
    if out_dtype == torch.float32:
        return torch.mm(x, w.t(), out_dtype=torch.float32)
    return torch.nn.functional.linear(x, w)
