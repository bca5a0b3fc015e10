"""Checked wrappers around the HIP entry points.  Each takes torch tensors that
live on the GPU, checks on the host that shapes, strides and element types are
what the kernel and its grid assume, and launches on torch's current stream.
Nothing here computes on the CPU and nothing falls back to a library."""
from __future__ import annotations

import math
import os
from typing import Optional

import torch

from . import lib as _lib
from .packing import PackedWeight

F32, BF16, I32 = 0, 1, 2
_CODES = {torch.float32: F32, torch.bfloat16: BF16, torch.int32: I32}


def _code(t: torch.Tensor) -> int:
    try:
        return _CODES[t.dtype]
    except KeyError:
        raise TypeError(f"element type {t.dtype} is not handled by the kernels (float32, bfloat16, int32)") from None


def _stream() -> int:
    """The current HIP stream's handle (the raw call: `torch.cuda.current_stream()` builds an object each time)."""
    return torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice())


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise ValueError(msg)


def _gpu(*ts: Optional[torch.Tensor]) -> None:
    for t in ts:
        if t is not None and not t.is_cuda:
            raise ValueError("kernel operands must live on the GPU (there is no CPU path)")


def _rows(t: torch.Tensor, what: str) -> int:
    """A [rows, cols] view with unit column stride; returns its row stride."""
    if not (t.dim() == 2):
        raise ValueError(f"{what}: expected 2 dimensions, got shape {tuple(t.shape)}")
    if not (t.shape[1] == 0 or t.stride(1) == 1):
        raise ValueError(f"{what}: columns must be contiguous")
    return t.stride(0) if t.shape[0] > 1 else max(t.stride(0), t.shape[1])


def _i32(t: Optional[torch.Tensor], n: int, what: str) -> int:
    if t is None:
        return 0
    if not (t.dtype == torch.int32 and t.is_contiguous() and t.numel() >= n):
        raise ValueError(f"{what}: need >= {n} contiguous int32")
    return t.data_ptr()


# --------------------------------------------------------------------------- plain library
def embed_rows(table, tokens: torch.Tensor, out: torch.Tensor) -> None:
    """out[t] = table[tokens[t]]; the table is a [vocab, dim] matrix or its tiled form (`PackedWeight`)."""
    T = tokens.numel()
    ldo = _rows(out, "embed out")
    if isinstance(table, PackedWeight):
        _gpu(table.data, tokens, out)
        _need(out.shape == (T, table.K), "embed out must be [tokens, dim]")
        L = _lib.load("plain")
        _lib.check(L.apc_embed_rows_tiled(table.data.data_ptr(), table.chunks, _i32(tokens, T, "tokens"),
                                          out.data_ptr(), _code(out), T, table.K, ldo, _stream()), "embed_rows_tiled")
        return
    _gpu(table, tokens, out)
    _need(table.dim() == 2 and table.is_contiguous(), "embedding table must be a contiguous [vocab, dim] matrix")
    _need(out.shape[0] == T and out.shape[1] == table.shape[1], "embed out must be [tokens, dim]")
    L = _lib.load("plain")
    _lib.check(L.apc_embed_rows(table.data_ptr(), _code(table), _i32(tokens, T, "tokens"), out.data_ptr(), _code(out),
                                T, table.shape[1], ldo, _stream()), "embed_rows")


def gather_rows(x: torch.Tensor, rows: torch.Tensor, out: torch.Tensor) -> None:
    _gpu(x, rows, out)
    R = rows.numel()
    ldx, ldo = _rows(x, "gather x"), _rows(out, "gather out")
    _need(out.shape == (R, x.shape[1]) and out.dtype == x.dtype, "gather out must be [rows, dim] of x's type")
    L = _lib.load("plain")
    _lib.check(L.apc_gather_rows(x.data_ptr(), _code(x), ldx, _i32(rows, R, "rows"), out.data_ptr(), ldo, R, x.shape[1],
                                 _stream()), "gather_rows")


def rmsnorm_rows(x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor,
                 rows: Optional[torch.Tensor] = None) -> None:
    _gpu(x, weight, out, rows)
    ldx, ldo = _rows(x, "rmsnorm x"), _rows(out, "rmsnorm out")
    R = out.shape[0]
    D = x.shape[1]
    if not (weight.dtype == torch.float32 and weight.is_contiguous() and weight.numel() == D):
        raise ValueError(f"rmsnorm weight must be float32 [{D}]")
    _need(out.shape[1] == D, "rmsnorm out width differs from x")
    _need(rows is not None or x.shape[0] == R, "rmsnorm: out rows differ from x rows")
    L = _lib.load("plain")
    _lib.check(L.apc_rmsnorm_rows(x.data_ptr(), _code(x), ldx, _i32(rows, R, "rows"), weight.data_ptr(), float(eps),
                                  out.data_ptr(), _code(out), ldo, R, D, _stream()), "rmsnorm_rows")


def add_into(acc: torch.Tensor, y: torch.Tensor) -> None:
    _gpu(acc, y)
    lda, ldy = _rows(acc, "add acc"), _rows(y, "add y")
    _need(acc.dtype == torch.float32, "the residual sum is kept in float32")
    _need(acc.shape == y.shape, "add_into: shapes differ")
    L = _lib.load("plain")
    _lib.check(L.apc_add_into(acc.data_ptr(), lda, y.data_ptr(), _code(y), ldy, acc.shape[0], acc.shape[1], _stream()),
               "add_into")


def silu_mul(gate_up: torch.Tensor, out: torch.Tensor) -> None:
    _gpu(gate_up, out)
    ldg, ldo = _rows(gate_up, "silu_mul in"), _rows(out, "silu_mul out")
    T, F = out.shape
    _need(gate_up.shape == (T, 2 * F), "silu_mul: input must be [rows, 2*F] (gate columns, then up columns)")
    L = _lib.load("plain")
    for r0 in range(0, T, 32768):
        n = min(32768, T - r0)
        _lib.check(L.apc_silu_mul(gate_up[r0:].data_ptr(), _code(gate_up), ldg, out[r0:].data_ptr(), _code(out), ldo,
                                  n, F, _stream()), "silu_mul")


def cast(src: torch.Tensor, dst: torch.Tensor) -> None:
    _gpu(src, dst)
    _need(src.is_contiguous() and dst.is_contiguous() and src.numel() == dst.numel(), "cast: contiguous, same count")
    L = _lib.load("plain")
    _lib.check(L.apc_cast(src.data_ptr(), _code(src), dst.data_ptr(), _code(dst), src.numel(), _stream()), "cast")


def rope_kv_write(qkv: torch.Tensor, q_off: int, k_off: int, v_off: int, n_heads: int, n_kv_heads: int, head_dim: int,
                  rot: int, cos_sin: Optional[torch.Tensor], positions: torch.Tensor,
                  row_seg: Optional[torch.Tensor] = None, block_table: Optional[torch.Tensor] = None,
                  cache: Optional[torch.Tensor] = None, page_tokens: int = 0) -> None:
    """Rotate q (and k) of every row by its position; with `cache`, write rotated k and v into the pages."""
    _gpu(qkv, cos_sin, positions, row_seg, block_table, cache)
    ld = _rows(qkv, "qkv")
    T = qkv.shape[0]
    width = qkv.shape[1]
    _need(q_off + n_heads * head_dim <= width and k_off + n_kv_heads * head_dim <= width
          and v_off + n_kv_heads * head_dim <= width, "qkv: head ranges exceed the row")
    _need(rot % 2 == 0 and 0 <= rot <= head_dim, "rotated width must be even and at most head_dim")
    if rot:
        _need(cos_sin is not None and cos_sin.dtype == torch.float32 and cos_sin.is_contiguous()
              and cos_sin.dim() == 3 and cos_sin.shape[1] == 2 and cos_sin.shape[2] == rot // 2,
              "cos/sin table must be float32 [positions, 2, rot/2]")
    max_blocks = 0
    if cache is not None:
        _need(block_table is not None and row_seg is not None, "cache write needs a block table and row segments")
        if not (cache.dim() == 5 and cache.is_contiguous()
                and tuple(cache.shape[1:]) == (2, n_kv_heads, page_tokens, head_dim)):
            raise ValueError(f"cache must be [pages, 2, {n_kv_heads}, {page_tokens}, {head_dim}], "
                             f"got {tuple(cache.shape)}")
        _need(block_table.dim() == 2 and block_table.dtype == torch.int32 and block_table.is_contiguous(),
              "block table must be contiguous int32 [segments, blocks]")
        max_blocks = block_table.shape[1]
    if (not FORCE_PLAIN and qkv.dtype == torch.bfloat16 and (cache is None or cache.dtype == torch.bfloat16)
            and head_dim % 8 == 0 and rot % 16 == 0 and ld % 8 == 0 and q_off % 8 == 0 and k_off % 8 == 0
            and v_off % 8 == 0 and qkv.data_ptr() % 16 == 0):
        # the same operation 16 bytes a lane (library `tuned`)
        _lib.check(_lib.load("tuned").apc_rope_kv_write_bf16(
            qkv.data_ptr(), ld, q_off, k_off, v_off, T, n_heads, n_kv_heads, head_dim, rot,
            cos_sin.data_ptr() if rot else 0, _i32(positions, T, "positions"),
            _i32(row_seg, T, "row_seg") if row_seg is not None else 0,
            block_table.data_ptr() if block_table is not None else 0, max_blocks,
            cache.data_ptr() if cache is not None else 0, page_tokens, _stream()), "rope_kv_write_bf16")
        return
    L = _lib.load("plain")
    _lib.check(L.apc_rope_kv_write(
        qkv.data_ptr(), _code(qkv), ld, q_off, k_off, v_off, T, n_heads, n_kv_heads, head_dim, rot,
        cos_sin.data_ptr() if rot else 0, _i32(positions, T, "positions"),
        _i32(row_seg, T, "row_seg") if row_seg is not None else 0,
        block_table.data_ptr() if block_table is not None else 0, max_blocks,
        cache.data_ptr() if cache is not None else 0, _code(cache) if cache is not None else 0, page_tokens,
        _stream()), "rope_kv_write")


def gemm_plain(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, accumulate: bool = False) -> None:
    """out = a . w^T, or out += a . w^T (out float32), in true 32-bit arithmetic."""
    _gpu(a, w, out)
    lda, ldw, ldc = _rows(a, "gemm a"), _rows(w, "gemm w"), _rows(out, "gemm out")
    M, K = a.shape
    N = w.shape[0]
    if not (w.shape[1] == K):
        raise ValueError(f"gemm: a is [*, {K}] but w is {tuple(w.shape)}")
    if not (out.shape == (M, N)):
        raise ValueError(f"gemm: out must be [{M}, {N}], got {tuple(out.shape)}")
    _need(not accumulate or out.dtype == torch.float32, "gemm: accumulation needs a float32 destination")
    L = _lib.load("plain")
    for r0 in range(0, M, 1 << 21):  # grid.y limit: 65535 tiles of 64 rows
        n = min(1 << 21, M - r0)
        _lib.check(L.apc_gemm_plain(a[r0:].data_ptr(), _code(a), lda, w.data_ptr(), _code(w), ldw,
                                    out[r0:].data_ptr(), _code(out), ldc, n, N, K, 1 if accumulate else 0, _stream()),
                   "gemm_plain")


def paged_attention_plain(q: torch.Tensor, q_off: int, out: torch.Tensor, n_heads: int, n_kv_heads: int,
                          head_dim: int, cache: torch.Tensor, page_tokens: int, block_table: torch.Tensor,
                          positions: torch.Tensor, row_seg: torch.Tensor, window: int = 0,
                          scale: Optional[float] = None) -> None:
    _gpu(q, out, cache, block_table, positions, row_seg)
    ldq, ldo = _rows(q, "attention q"), _rows(out, "attention out")
    T = q.shape[0]
    _need(q_off + n_heads * head_dim <= q.shape[1], "attention: q heads exceed the row")
    _need(out.shape == (T, n_heads * head_dim), "attention out must be [rows, heads*head_dim]")
    _need(n_heads % n_kv_heads == 0, "heads must be a multiple of kv heads")
    _need(head_dim <= 256, "plain attention handles head_dim <= 256")
    if not (cache.dim() == 5 and cache.is_contiguous()
            and tuple(cache.shape[1:]) == (2, n_kv_heads, page_tokens, head_dim)):
        raise ValueError(f"cache must be [pages, 2, {n_kv_heads}, {page_tokens}, {head_dim}], got {tuple(cache.shape)}")
    _need(block_table.dim() == 2 and block_table.dtype == torch.int32 and block_table.is_contiguous(),
          "block table must be contiguous int32 [segments, blocks]")
    L = _lib.load("plain")
    sc = (1.0 / math.sqrt(head_dim)) if scale is None else float(scale)
    _lib.check(L.apc_paged_attention_plain(
        q.data_ptr(), _code(q), ldq, q_off, out.data_ptr(), _code(out), ldo, T, n_heads, n_kv_heads, head_dim,
        cache.data_ptr(), _code(cache), page_tokens, block_table.data_ptr(), block_table.shape[1],
        _i32(positions, T, "positions"), _i32(row_seg, T, "row_seg"), int(window), sc, _stream()),
        "paged_attention_plain")


def argmax_rows(logits: torch.Tensor, out: torch.Tensor) -> None:
    _gpu(logits, out)
    ld = _rows(logits, "logits")
    R, V = logits.shape
    _need(logits.dtype == torch.float32, "logits are float32")
    L = _lib.load("plain")
    scratch = torch.empty(2 * R * 64, dtype=torch.int32, device=logits.device) if V >= 8192 else None
    _lib.check(L.apc_argmax_rows(logits.data_ptr(), ld, R, V, _i32(out, R, "argmax out"),
                                 scratch.data_ptr() if scratch is not None else 0, _stream()), "argmax_rows")


def sample_rows(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
                uniform: torch.Tensor, out: torch.Tensor, any_top_k: bool = True, any_top_p: bool = True,
                few_after_top_k: bool = False, one_block: bool = False) -> None:
    """One token a row by temperature / top-k / top-p with the row's uniform number.  `any_top_k`, `any_top_p`: whether
    some row may ask for that cut; `few_after_top_k`: every row that samples has 0 < top-k <= 1,024.  A caller that
    knows its rows saves the launches that none of them needs; a row for which its word is wrong still gets its
    token, slowly.  `one_block`: the kernel without working memory, one block a row."""
    _gpu(logits, temperature, top_k, top_p, uniform, out)
    ld = _rows(logits, "logits")
    R, V = logits.shape
    _need(logits.dtype == torch.float32, "logits are float32")
    for t, name in ((temperature, "temperature"), (top_p, "top_p"), (uniform, "uniform")):
        if not (t.dtype == torch.float32 and t.is_contiguous() and t.numel() >= R):
            raise ValueError(f"{name}: float32 [{R}]")
    L = _lib.load("plain")
    kib = 0 if one_block else L.apc_sample_rows_scratch_kib(R)
    scratch = torch.empty(kib * 1024, dtype=torch.uint8, device=logits.device) if kib else None
    _lib.check(L.apc_sample_rows(logits.data_ptr(), ld, R, V, temperature.data_ptr(), _i32(top_k, R, "top_k"),
                                 top_p.data_ptr(), uniform.data_ptr(), _i32(out, R, "sample out"),
                                 scratch.data_ptr() if scratch is not None else 0, kib * 1024,
                                 (1 if any_top_k else 0) | (2 if any_top_p else 0) | (4 if few_after_top_k else 0),
                                 _stream()),
               "sample_rows")


# --------------------------------------------------------------------------- dispatch
# With FORCE_PLAIN every step runs on the plain kernels whatever the element type
# (used by tests to check one tuned kernel at a time against the same model).
FORCE_PLAIN = os.environ.get("ALLPACA_AMD_PLAIN", "0") == "1"


def _tuned_ok(*ts: torch.Tensor) -> bool:
    return (not FORCE_PLAIN) and all(t.dtype == torch.bfloat16 for t in ts)


def prepare_matrix(w: torch.Tensor, run_dtype: torch.dtype):
    """How a weight matrix [out, in] is kept on the GPU: a bfloat16 matrix of a bfloat16 run in the tiled layout
    of the MFMA kernels (if its width is a multiple of 8), anything else as it is."""
    from .packing import can_pack, pack_mfma
    if run_dtype == torch.bfloat16 and not FORCE_PLAIN and w.is_cuda and can_pack(w):
        return pack_mfma(w)
    return w.contiguous()


def linear(a: torch.Tensor, w, out: torch.Tensor, accumulate: bool = False, emit=None) -> None:
    """out = a . w^T (or out += ..., out float32).  A tiled bfloat16 weight runs on the MFMA kernels.
    `emit` (with accumulate): an object with `weight` (an RMS norm's) whose `raw` and `ss` are filled with what
    that norm's next product needs, where there is a kernel for these sizes; else it is left as it is."""
    if isinstance(w, PackedWeight):
        from . import tuned
        if emit is not None and accumulate:
            left = tuned.gemm_emit_bf16(a, w, out, emit.weight)
            if left is not None:
                emit.raw, emit.ss = left
                return
        tuned.gemm_bf16(a, w, out, accumulate)
    else:
        gemm_plain(a, w, out, accumulate)


def swiglu(h: torch.Tensor, w_gate_up, out: torch.Tensor) -> None:
    """out[t, f] = silu(h . Wg[f]) * (h . Wu[f]); w_gate_up is [Wg; Wu] of shape [2F, D], or the pair of
    their tiled forms."""
    if isinstance(w_gate_up, tuple):
        from . import tuned
        tuned.swiglu_bf16(h, w_gate_up[0], w_gate_up[1], out)
        return
    T, F = out.shape
    gu = torch.empty((T, 2 * F), dtype=torch.float32 if h.dtype == torch.float32 else out.dtype, device=h.device)
    gemm_plain(h, w_gate_up, gu)
    silu_mul(gu, out)


def linear_pre(raw: torch.Tensor, ss: torch.Tensor, eps: float, w, out: torch.Tensor) -> bool:
    """The product of a normalised row from what `linear(..., emit=...)` left; False if there is no kernel for
    these sizes (nothing is done then)."""
    if isinstance(w, PackedWeight) and not FORCE_PLAIN:
        from . import tuned
        return tuned.gemm_pre_bf16(raw, ss, eps, w, out)
    return False


def qkv_rope_write(a: torch.Tensor, pre, w, q_out: torch.Tensor, n_heads: int, n_kv_heads: int, head_dim: int,
                   cos_sin: torch.Tensor, positions: torch.Tensor, row_seg: torch.Tensor, block_table: torch.Tensor,
                   cache: torch.Tensor, page_tokens: int) -> bool:
    """The product for q, k and v, the rotation of whole q and k heads and the write of k and v into the pages in
    one kernel (few rows; `pre` = (ss, eps) if `a` is a row that `linear(..., emit=...)` left, else None).  False if
    there is no such kernel for these sizes (nothing is done then)."""
    if isinstance(w, PackedWeight) and not FORCE_PLAIN:
        from . import tuned
        return tuned.qkv_rope_bf16(a, pre, w, q_out, n_heads, n_kv_heads, head_dim, cos_sin, positions, row_seg,
                                   block_table, cache, page_tokens)
    return False


def swiglu_pre(raw: torch.Tensor, ss: torch.Tensor, eps: float, w_gate_up, out: torch.Tensor) -> bool:
    if isinstance(w_gate_up, tuple) and not FORCE_PLAIN:
        from . import tuned
        return tuned.swiglu_pre_bf16(raw, ss, eps, w_gate_up[0], w_gate_up[1], out)
    return False


def attention_tile_rows(run_dtype: torch.dtype = torch.bfloat16) -> int:
    """Rows of a tile of the attention kernel that takes segments of several rows: the step packer cuts segments into
    such tiles (`StepInfo.tile_row0`, `tile_rows`).  The kernel's library says how many; the plain kernel, which
    32-bit runs use, does not look at tiles."""
    if run_dtype != torch.bfloat16 or FORCE_PLAIN:
        return 64
    return int(_lib.load("tuned").apc_attention_prefill_tile_rows())


def paged_attention(q: torch.Tensor, q_off: int, out: torch.Tensor, n_heads: int, n_kv_heads: int, head_dim: int,
                    cache: torch.Tensor, page_tokens: int, block_table: torch.Tensor, step, window: int = 0,
                    scale: Optional[float] = None) -> None:
    if _tuned_ok(q, cache, out):
        from . import tuned
        if tuned.attention_bf16(q, q_off, out, n_heads, n_kv_heads, head_dim, cache, page_tokens, block_table, step,
                                window, scale):
            return
    paged_attention_plain(q, q_off, out, n_heads, n_kv_heads, head_dim, cache, page_tokens, block_table,
                          step.positions, step.row_seg, window, scale)


# --------------------------------------------------------------------------- mechanisms beside the llama layer
MASKS = {"causal": 0, "window": 1, "chunk": 2}


def _f32(t: Optional[torch.Tensor], n: int, what: str) -> int:
    if t is None:
        return 0
    if not (t.dtype == torch.float32 and t.is_contiguous() and t.numel() >= n):
        raise ValueError(f"{what}: need >= {n} contiguous float32")
    return t.data_ptr()


def _split_pages(cache: torch.Tensor, kv_heads: int, key_dim: int, value_dim: int, page_tokens: int) -> None:
    if not (cache.dim() == 3 and cache.is_contiguous()
            and tuple(cache.shape[1:]) == (kv_heads, page_tokens * (key_dim + value_dim))):
        raise ValueError(f"cache must be [pages, {kv_heads}, {page_tokens} * ({key_dim} + {value_dim})], "
                         f"got {tuple(cache.shape)}")


def conv_heads(proj: torch.Tensor, q_off: int, k_off: int, v_off: int, n_heads: int, n_kv_heads: int, key_dim: int,
               value_dim: int, bias: Optional[torch.Tensor], conv_w: Optional[torch.Tensor],
               state: Optional[torch.Tensor], step, slots: Optional[torch.Tensor], unit_norm: bool, eps: float,
               q_out: torch.Tensor, block_table: Optional[torch.Tensor] = None, cache: Optional[torch.Tensor] = None,
               page_tokens: int = 0, norm_dim: int = 0, q_norm_w: Optional[torch.Tensor] = None,
               k_norm_w: Optional[torch.Tensor] = None, norm_rows: bool = False, q_temp_coef: float = 0.0,
               q_temp_every: int = 0) -> None:
    """Bias, short causal convolution over time (taps = conv_w.shape[1]; the inputs of the positions ahead of a
    segment come from `state` [slots + 1, taps - 1, width], which is moved on), unit RMS norm of q and k heads,
    q to `q_out` [rows, heads * key_dim], k and v into the pages.  `n_kv_heads` = 0: the row holds q only.
    `norm_dim` (divides key_dim; 0: key_dim): the norm is taken over every piece of that many elements of a head;
    `q_norm_w`, `k_norm_w` float32 [norm_dim]: weights the normed pieces are multiplied with.
    `norm_rows`: the norm is taken over all heads of q (of k) at once, and the weights are float32
    [heads * key_dim] ([kv heads * key_dim]).  `q_temp_every` > 0: q of a row at position p is multiplied by
    1 + q_temp_coef * ln(floor((p + 1) / q_temp_every) + 1)."""
    _gpu(proj, bias, conv_w, state, slots, q_out, block_table, cache, q_norm_w, k_norm_w)
    nd = int(norm_dim) or key_dim
    _need(nd > 0 and key_dim % nd == 0, "conv_heads: norm_dim must divide key_dim")
    _need((q_norm_w is None and k_norm_w is None) or unit_norm, "conv_heads: norm weights need the norm")
    _need(not norm_rows or (unit_norm and nd == key_dim), "conv_heads: a norm over the whole projection has no pieces")
    _need(int(q_temp_every) >= 0, "conv_heads: q_temp_every must not be negative")
    nq, nk = (n_heads * key_dim, int(n_kv_heads) * key_dim) if norm_rows else (nd, nd)
    ld, ldq = _rows(proj, "projected rows"), _rows(q_out, "q out")
    T, width = proj.shape
    G = int(n_kv_heads)
    _need(q_off + n_heads * key_dim <= width and (G == 0 or (k_off + G * key_dim <= width and
                                                             v_off + G * value_dim <= width)),
          "conv_heads: head ranges exceed the row")
    _need(q_out.shape == (T, n_heads * key_dim), "conv_heads: q out must be [rows, heads * key_dim]")
    taps = 1
    if conv_w is not None:
        _need(conv_w.dim() == 2 and conv_w.shape[0] == width, "conv_heads: conv weights must be [width, taps]")
        taps = int(conv_w.shape[1])
    if taps > 1:
        _need(state is not None and slots is not None and state.dim() == 3 and state.is_contiguous()
              and state.dtype == torch.float32 and tuple(state.shape[1:]) == (taps - 1, width),
              f"conv_heads: state must be float32 [slots, {taps - 1}, {width}]")
    max_blocks = 0
    if G:
        _need(cache is not None and block_table is not None, "conv_heads: keys and values need pages and a block table")
        _split_pages(cache, G, key_dim, value_dim, page_tokens)
        _need(block_table.dim() == 2 and block_table.dtype == torch.int32 and block_table.is_contiguous(),
              "block table must be contiguous int32 [segments, blocks]")
        max_blocks = block_table.shape[1]
    S = step.n_segs
    L = _lib.load("plain")
    if (_tuned_ok(proj, q_out) and (cache is None or cache.dtype == torch.bfloat16) and q_off == 0
            and (G == 0 or (k_off == n_heads * key_dim and v_off == (n_heads + G) * key_dim))):
        LT = _lib.load("tuned")
        if (LT.apc_conv_heads_bf16_takes(ld, width, n_heads, G, key_dim, value_dim, taps, ldq) and nd % 8 == 0
                and all(w is None or w.data_ptr() % 16 == 0 for w in (q_norm_w, k_norm_w))
                and proj.data_ptr() % 16 == 0 and q_out.data_ptr() % 16 == 0
                and (cache is None or cache.data_ptr() % 16 == 0) and (state is None or state.data_ptr() % 16 == 0)
                and (conv_w is None or (conv_w.data_ptr() % 16 == 0 and width % 4 == 0))):
            # the same on 16 bytes a thread (library `tuned`); the plain kernel then moves the state on, unless every
            # segment is a single row (decoded tokens): then the kernel does that too
            fold = taps > 1 and bool(getattr(step, "decode_only", False))
            _lib.check(LT.apc_conv_heads_bf16(
                proj.data_ptr(), ld, T, n_heads, G, key_dim, value_dim, _f32(bias, width, "bias"),
                _f32(conv_w, width * taps, "conv weights"), taps,
                state.data_ptr() if taps > 1 else 0, 1 if fold else 0, width, _i32(step.row_seg, T, "row_seg"),
                _i32(step.seg_row0, S, "seg_row0"), _i32(slots, S, "slots") if taps > 1 else 0,
                _i32(step.positions, T, "positions"), 1 if unit_norm else 0, float(eps), nd,
                _f32(q_norm_w, nq, "q norm weight"), _f32(k_norm_w, nk, "k norm weight"), 1 if norm_rows else 0,
                float(q_temp_coef), int(q_temp_every), q_out.data_ptr(), ldq,
                block_table.data_ptr() if G else 0, max_blocks, cache.data_ptr() if G else 0, page_tokens, _stream()),
                "conv_heads_bf16")
            if taps > 1 and not fold:
                _lib.check(L.apc_conv_state(proj.data_ptr(), _code(proj), ld, _f32(bias, width, "bias"), taps,
                                            state.data_ptr(), width, S, _i32(step.seg_row0, S, "seg_row0"),
                                            _i32(step.seg_rows, S, "seg_rows"), _i32(slots, S, "slots"), _stream()),
                           "conv_state")
            return
    _lib.check(L.apc_conv_heads(
        proj.data_ptr(), _code(proj), ld, q_off, k_off, v_off, T, S, n_heads, G, key_dim, value_dim,
        _f32(bias, width, "bias"), _f32(conv_w, width * taps, "conv weights"), taps,
        state.data_ptr() if taps > 1 else 0, width, _i32(step.row_seg, T, "row_seg"), _i32(step.seg_row0, S, "seg_row0"),
        _i32(step.seg_rows, S, "seg_rows"), _i32(slots, S, "slots") if taps > 1 else 0,
        _i32(step.positions, T, "positions"), 1 if unit_norm else 0, float(eps), nd,
        _f32(q_norm_w, nq, "q norm weight"), _f32(k_norm_w, nk, "k norm weight"), 1 if norm_rows else 0,
        float(q_temp_coef), int(q_temp_every), q_out.data_ptr(), _code(q_out), ldq,
        block_table.data_ptr() if G else 0, max_blocks, cache.data_ptr() if G else 0, _code(cache) if G else 0,
        page_tokens, _stream()), "conv_heads")


def masked_attention_plain(q: torch.Tensor, out: torch.Tensor, n_heads: int, n_kv_heads: int, key_dim: int,
                           value_dim: int, cache: torch.Tensor, page_tokens: int, block_table: torch.Tensor,
                           positions: torch.Tensor, row_seg: torch.Tensor, mask: str, mask_size: int, sink: bool,
                           scale: float, key_parts: int = 1, sinks: Optional[torch.Tensor] = None,
                           gate: Optional[torch.Tensor] = None, softcap: float = 0.0,
                           distance_bias: Optional[tuple] = None) -> None:
    _gpu(q, out, cache, block_table, positions, row_seg, sinks, gate)
    r1, r2 = distance_bias if distance_bias is not None else (None, None)
    _gpu(r1, r2)
    _need(float(softcap) >= 0.0, "attention: the soft cap must not be negative")
    ldq, ldo = _rows(q, "attention q"), _rows(out, "attention out")
    T = q.shape[0]
    _check_key_parts(n_heads, n_kv_heads, key_dim, key_parts)
    _check_sinks_gate(sink, sinks, gate, T, n_heads)
    _need(q.shape[1] == n_heads * (key_dim // key_parts), "attention: q must be [rows, heads * key_dim / key_parts]")
    _need(out.shape == (T, n_heads * value_dim), "attention out must be [rows, heads * value_dim]")
    _split_pages(cache, n_kv_heads, key_dim, value_dim, page_tokens)
    _need(block_table.dim() == 2 and block_table.dtype == torch.int32 and block_table.is_contiguous(),
          "block table must be contiguous int32 [segments, blocks]")
    L = _lib.load("plain")
    _lib.check(L.apc_masked_attention_plain(
        q.data_ptr(), _code(q), ldq, out.data_ptr(), _code(out), ldo, T, n_heads, n_kv_heads, key_dim, value_dim,
        cache.data_ptr(), _code(cache), page_tokens, block_table.data_ptr(), block_table.shape[1],
        _i32(positions, T, "positions"), _i32(row_seg, T, "row_seg"), MASKS[mask], int(mask_size), 1 if sink else 0,
        _f32(sinks, n_heads, "sinks"), gate.data_ptr() if gate is not None else 0,
        _code(gate) if gate is not None else 0, _rows(gate, "head gate") if gate is not None else 0,
        float(scale), int(key_parts), float(softcap), _f32(r1, n_heads, "distance bias r1"),
        _f32(r2, n_heads, "distance bias r2"), _stream()), "masked_attention_plain")


def _check_sinks_gate(sink: bool, sinks, gate, T: int, n_heads: int) -> None:
    _need(sinks is None or sink, "attention: learned sink scores need the sink")
    _need(gate is None or (gate.dim() == 2 and gate.shape[0] == T and gate.shape[1] >= n_heads),
          "attention: the head gate's logits must be [rows, >= heads]")


def _check_key_parts(n_heads: int, n_kv_heads: int, key_dim: int, key_parts: int) -> None:
    _need(key_parts >= 1 and key_dim % key_parts == 0 and n_heads % n_kv_heads == 0
          and (n_heads // n_kv_heads) % key_parts == 0,
          "attention: key_parts must divide key_dim and the query heads of a kv head")


def masked_attention(q: torch.Tensor, out: torch.Tensor, n_heads: int, n_kv_heads: int, key_dim: int, value_dim: int,
                     cache: torch.Tensor, page_tokens: int, block_table: torch.Tensor, step, mask: str = "causal",
                     mask_size: int = 0, sink: bool = False, scale: float = 1.0, key_parts: int = 1,
                     sinks: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None, softcap: float = 0.0,
                     distance_bias: Optional[tuple] = None) -> None:
    """`key_parts` = M > 1: a cached key of `key_dim` elements is M keys of key_dim / M side by side, one for each of M
    softmax maps over the same values; q holds `n_heads` heads of key_dim / M, head j uses part j % M (M consecutive
    heads are the maps of one head), and `out` holds n_heads heads of value_dim (float32 or the run's type).
    `sinks` float32 [heads]: the sink's score per head (0 without).  `gate` [rows, >= heads] logits: head h of a row
    leaves multiplied by sigmoid(gate[row][h]).  `softcap` c > 0: a score s becomes c * tanh(s / c).  `distance_bias`
    (r1, r2), float32 [heads] each: the score of a key d positions back is lowered by r1[h] * ln(1 + r2[h] * d)."""
    if _tuned_ok(q, cache) and out.dtype in (torch.bfloat16, torch.float32):
        from . import tuned
        if tuned.masked_attention_bf16(q, out, n_heads, n_kv_heads, key_dim, value_dim, cache, page_tokens,
                                       block_table, step, mask, mask_size, sink, scale, key_parts, sinks, gate,
                                       softcap, distance_bias):
            return
    masked_attention_plain(q, out, n_heads, n_kv_heads, key_dim, value_dim, cache, page_tokens, block_table,
                           step.positions, step.row_seg, mask, mask_size, sink, scale, key_parts, sinks, gate,
                           softcap, distance_bias)


def rotary_pages(q: torch.Tensor, q_off: int, n_heads: int, q_dim: int, q_rot0: int, q_out: torch.Tensor,
                 ka: torch.Tensor, ka_off: int, a_dim: int, kb: Optional[torch.Tensor], kb_off: int, b_dim: int,
                 kb_shared: bool, k_rot0: int, v: torch.Tensor, v_off: int, value_dim: int, n_kv_heads: int, rot: int,
                 cos_sin: Optional[torch.Tensor], step, block_table: torch.Tensor, cache: torch.Tensor,
                 page_tokens: int, q_norm_w: Optional[torch.Tensor] = None, k_norm_w: Optional[torch.Tensor] = None,
                 norm_eps: float = 0.0) -> None:
    """Heads put together, rotated and cached.  Query head h: q[:, q_off + h * q_dim ...], its elements
    [q_rot0, q_rot0 + rot) rotated by the row's position, to q_out [rows, heads * q_dim] (q_out may be q).  Key of kv
    head g: a_dim elements of ka (column ka_off + g * a_dim) followed by b_dim elements of kb (column kb_off, the same
    for every head if `kb_shared`, else + g * b_dim); elements [k_rot0, k_rot0 + rot) of the whole rotated; into the
    pages.  Value of kv head g: v[:, v_off + g * value_dim ...] as it is (it may be the key's own columns).  Pairs are
    (i, i + rot/2) of the rotated range; cos_sin float32 [positions, 2, rot/2].  `q_norm_w` float32 [q_dim],
    `k_norm_w` float32 [a_dim + b_dim]: the head is first divided by its root mean square (`norm_eps` inside the root)
    and multiplied with these weights, which all heads share; values are taken as they are."""
    _gpu(q, q_out, ka, kb, v, cos_sin, block_table, cache, q_norm_w, k_norm_w)
    T = q.shape[0]
    H, G, dq, da, db, dv = int(n_heads), int(n_kv_heads), int(q_dim), int(a_dim), int(b_dim), int(value_dim)
    ldq, ldqo, ldka, ldv = _rows(q, "q"), _rows(q_out, "q out"), _rows(ka, "keys"), _rows(v, "values")
    ldkb = _rows(kb, "shared key part") if kb is not None else 0
    _need(q_off + H * dq <= q.shape[1] and q_out.shape == (T, H * dq), "rotary_pages: q heads exceed the row")
    _need(ka.shape[0] == T and v.shape[0] == T and ka_off + G * da <= ka.shape[1] and v_off + G * dv <= v.shape[1],
          "rotary_pages: key or value heads exceed the row")
    _need(db == 0 or (kb is not None and kb.shape[0] == T and kb_off + (1 if kb_shared else G) * db <= kb.shape[1]),
          "rotary_pages: the second key part exceeds its row")
    _need(rot % 2 == 0 and 0 <= q_rot0 and q_rot0 + rot <= dq and 0 <= k_rot0 and k_rot0 + rot <= da + db,
          "rotary_pages: the rotated range must lie inside a head")
    if rot:
        _need(cos_sin is not None and cos_sin.dtype == torch.float32 and cos_sin.is_contiguous()
              and cos_sin.dim() == 3 and cos_sin.shape[1] == 2 and cos_sin.shape[2] == rot // 2,
              "cos/sin table must be float32 [positions, 2, rot/2]")
    _split_pages(cache, G, da + db, dv, page_tokens)
    _need(block_table.dim() == 2 and block_table.dtype == torch.int32 and block_table.is_contiguous(),
          "block table must be contiguous int32 [segments, blocks]")
    if _tuned_ok(q, q_out, ka, v, cache):
        from . import tuned
        if tuned.rotary_pages_bf16(q, ldq, q_off, H, dq, q_rot0, q_out, ldqo, ka, ldka, ka_off, da, kb, ldkb, kb_off,
                                   db, kb_shared, k_rot0, v, ldv, v_off, dv, G, rot, cos_sin, step, block_table, cache,
                                   page_tokens, q_norm_w, k_norm_w, norm_eps):
            return
    L = _lib.load("plain")
    _lib.check(L.apc_rotary_pages(
        q.data_ptr(), _code(q), ldq, q_off, H, dq, q_rot0, q_out.data_ptr(), _code(q_out), ldqo,
        ka.data_ptr(), _code(ka), ldka, ka_off, da, kb.data_ptr() if kb is not None else 0,
        _code(kb) if kb is not None else 0, ldkb, kb_off, db, 1 if kb_shared else 0, k_rot0,
        v.data_ptr(), _code(v), ldv, v_off, dv, G, rot, cos_sin.data_ptr() if rot else 0,
        _i32(step.positions, T, "positions"), _i32(step.row_seg, T, "row_seg"), block_table.data_ptr(),
        block_table.shape[1], cache.data_ptr(), _code(cache), page_tokens, T, _f32(q_norm_w, dq, "q norm weight"),
        _f32(k_norm_w, da + db, "k norm weight"), float(norm_eps), _stream()), "rotary_pages")


def streams_step(x: torch.Tensor, n_streams: int, y: Optional[torch.Tensor] = None,
                 mix: Optional[torch.Tensor] = None, out_w: Optional[torch.Tensor] = None,
                 in_w: Optional[torch.Tensor] = None, norm_w: Optional[torch.Tensor] = None, eps: float = 0.0,
                 h: Optional[torch.Tensor] = None, rows: Optional[torch.Tensor] = None) -> None:
    """x [T, S * D] float32, S residual copies a row.  With y [T, D]: copy b <- sum_a mix[a][b] copy a + out_w[b] y.
    With in_w: h = rms_norm(sum_a in_w[a] copy a) * norm_w (of the new copies, if both are asked for).  `rows`: h[r]
    from x[rows[r]] (reading only)."""
    _gpu(x, y, mix, out_w, in_w, norm_w, h, rows)
    S = int(n_streams)
    _need(x.dim() == 2 and x.dtype == torch.float32 and x.is_contiguous() and x.shape[1] % S == 0,
          "streams: x must be contiguous float32 [rows, streams * width]")
    T, D = x.shape[0], x.shape[1] // S
    ldy = ldh = 0
    if y is not None:
        ldy = _rows(y, "streams y")
        _need(y.shape == (T, D) and rows is None, "streams: y must be [rows, width]")
    n_out = T
    if in_w is not None:
        ldh = _rows(h, "streams h")
        n_out = rows.numel() if rows is not None else T
        _need(h.shape == (n_out, D), "streams: h must be [rows, width]")
    L = _lib.load("plain")
    _lib.check(L.apc_streams_step(
        x.data_ptr(), n_out, S, D, y.data_ptr() if y is not None else 0, _code(y) if y is not None else 0, ldy,
        _f32(mix, S * S, "mix") if y is not None else 0, _f32(out_w, S, "out weights") if y is not None else 0,
        _f32(in_w, S, "in weights"), _f32(norm_w, D, "norm weight"), float(eps),
        h.data_ptr() if in_w is not None else 0, _code(h) if in_w is not None else 0, ldh,
        _i32(rows, n_out, "rows") if rows is not None else 0, _stream()), "streams_step")


def embed_streams(table: torch.Tensor, tokens: torch.Tensor, norm_w: Optional[torch.Tensor], eps: float,
                  x: torch.Tensor, n_streams: int) -> None:
    """x[t] = S copies of rms_norm(table[tokens[t]]) * norm_w (of the bare row without norm_w)."""
    _gpu(table, tokens, norm_w, x)
    T = tokens.numel()
    _need(table.dim() == 2 and table.is_contiguous(), "embedding table must be a contiguous [vocab, width] matrix")
    D = table.shape[1]
    _need(x.dtype == torch.float32 and x.is_contiguous() and x.shape == (T, n_streams * D),
          "embed_streams: x must be contiguous float32 [tokens, streams * width]")
    L = _lib.load("plain")
    _lib.check(L.apc_embed_streams(table.data_ptr(), _code(table), _i32(tokens, T, "tokens"),
                                   _f32(norm_w, D, "norm weight"), float(eps), x.data_ptr(), T, int(n_streams), D,
                                   _stream()), "embed_streams")


def clamped_glu_mul(gate_up: torch.Tensor, out: torch.Tensor, alpha: float, limit: float) -> None:
    _gpu(gate_up, out)
    ldg, ldo = _rows(gate_up, "clamped_glu in"), _rows(out, "clamped_glu out")
    T, F = out.shape
    _need(gate_up.shape == (T, 2 * F), "clamped_glu: input must be [rows, 2*F] (gate columns, then up columns)")
    L = _lib.load("plain")
    for r0 in range(0, T, 32768):
        n = min(32768, T - r0)
        _lib.check(L.apc_clamped_glu(gate_up[r0:].data_ptr(), _code(gate_up), ldg, out[r0:].data_ptr(), _code(out),
                                     ldo, n, F, float(alpha), float(limit), _stream()), "clamped_glu")


def clamped_glu(h: torch.Tensor, w_gate_up, out: torch.Tensor, alpha: float, limit: float) -> None:
    """out[t, f] = g * sigmoid(alpha g) * (u + 1), g = min(h . Wg[f], limit), u = clamp(h . Wu[f], -limit, limit);
    w_gate_up is [Wg; Wu] of shape [2F, D] (row-major or tiled): one product for both branches (in the run's element
    type: 16 bits in a bfloat16 run), then the activation."""
    T, F = out.shape
    packed = isinstance(w_gate_up, PackedWeight)
    gu = torch.empty((T, 2 * F), dtype=h.dtype if packed else torch.float32, device=h.device)
    linear(h, w_gate_up, gu)
    clamped_glu_mul(gu, out, alpha, limit)


def scale_(x: torch.Tensor, s: float) -> None:
    _gpu(x)
    _need(x.dtype == torch.float32 and x.is_contiguous(), "scale_: contiguous float32")
    L = _lib.load("plain")
    _lib.check(L.apc_scale(x.data_ptr(), float(s), x.numel(), _stream()), "scale")


# --------------------------------------------------------------------------- embedding with positions, normed residual sum
def embed_positions(table: torch.Tensor, tokens: torch.Tensor, pos_table: torch.Tensor, positions: torch.Tensor,
                    scale: float, out: torch.Tensor) -> None:
    """out[t] = table[tokens[t]] * scale + pos_table[positions[t]]  (float32 out; the caller has checked that every
    position has a row in `pos_table`)."""
    _gpu(table, tokens, pos_table, positions, out)
    T = tokens.numel()
    _need(table.dim() == 2 and table.is_contiguous() and pos_table.dim() == 2 and pos_table.is_contiguous()
          and pos_table.shape[1] == table.shape[1], "embedding and position tables must be contiguous [n, width]")
    D = table.shape[1]
    ldo = _rows(out, "embed out")
    _need(out.dtype == torch.float32 and out.shape == (T, D), "embed out must be float32 [tokens, width]")
    L = _lib.load("plain")
    _lib.check(L.apc_embed_positions(table.data_ptr(), _code(table), _i32(tokens, T, "tokens"), pos_table.data_ptr(),
                                     _code(pos_table), _i32(positions, T, "positions"), float(scale), out.data_ptr(),
                                     ldo, T, D, _stream()), "embed_positions")


def rmsnorm_add(y: torch.Tensor, weight: torch.Tensor, eps: float, mult: float, x: torch.Tensor,
                copy: Optional[torch.Tensor] = None) -> None:
    """x += mult * rms_norm(y) * weight, in 32-bit; `copy` (if given) receives the new x in its own element type."""
    _gpu(y, weight, x, copy)
    ldy, ldx = _rows(y, "rmsnorm_add y"), _rows(x, "rmsnorm_add x")
    T, D = x.shape
    _need(x.dtype == torch.float32 and y.shape == (T, D), "rmsnorm_add: x float32 [rows, width], y of the same shape")
    _need(copy is None or copy.shape == (T, D), "rmsnorm_add: the copy must have x's shape")
    L = _lib.load("plain")
    _lib.check(L.apc_rmsnorm_add(y.data_ptr(), _code(y), ldy, _f32(weight, D, "norm weight"), float(eps), float(mult),
                                 x.data_ptr(), ldx, copy.data_ptr() if copy is not None else 0,
                                 _code(copy) if copy is not None else 0,
                                 _rows(copy, "rmsnorm_add copy") if copy is not None else 0, T, D, _stream()),
               "rmsnorm_add")


# --------------------------------------------------------------------------- linear attention with a decay
def linear_attention(proj: torch.Tensor, q_off: int, k_off: int, v_off: int, n_heads: int, key_dim: int,
                     value_dim: int, silu: bool, decay: torch.Tensor, state: torch.Tensor, step, slots: torch.Tensor,
                     out: torch.Tensor, powers: Optional[torch.Tensor] = None, rot: int = 0,
                     cos_sin: Optional[torch.Tensor] = None, k_scale: float = 1.0) -> None:
    """Per head S <- decay * S + k_t v_t^T, o_t = S^T q_t over the rows of every segment in order, S float32
    [slots + 1, heads, key_dim, value_dim] per request; q, k, v (through silu if asked) from the projected rows;
    `out` float32 [rows, heads * value_dim].  `powers` (optional): `tuned.decay_powers` of the same decay, kept by the
    caller for the kernel that walks prompt portions in chunks.  `rot` > 0: the first rot elements of every q and k
    head are rotated by the row's position (pairs i, i + rot/2; cos_sin float32 [positions, 2, rot/2]); `k_scale`
    multiplies k behind the rotation.  (A bfloat16 step of prompt portions rotates q and k of `proj` where they lie.)"""
    _gpu(proj, decay, state, slots, out, powers, cos_sin)
    rot = int(rot)
    _need(rot % 2 == 0 and 0 <= rot <= int(key_dim), "linear attention: the rotated width must be even and at most key_dim")
    if rot:
        _need(cos_sin is not None and cos_sin.dtype == torch.float32 and cos_sin.is_contiguous()
              and cos_sin.dim() == 3 and cos_sin.shape[1] == 2 and cos_sin.shape[2] == rot // 2,
              "cos/sin table must be float32 [positions, 2, rot/2]")
    ld, ldo = _rows(proj, "projected rows"), _rows(out, "linear attention out")
    T, width = proj.shape
    H, dk, dv = int(n_heads), int(key_dim), int(value_dim)
    _need(q_off + H * dk <= width and k_off + H * dk <= width and v_off + H * dv <= width,
          "linear attention: head ranges exceed the row")
    _need(out.dtype == torch.float32 and out.shape == (T, H * dv), "linear attention: out float32 [rows, heads * value_dim]")
    _need(state.dtype == torch.float32 and state.is_contiguous() and tuple(state.shape[1:]) == (H, dk, dv),
          f"linear attention: state must be float32 [slots, {H}, {dk}, {dv}]")
    S = step.n_segs
    if _tuned_ok(proj):
        from . import tuned
        if tuned.linear_attention_bf16(proj, q_off, k_off, v_off, H, dk, dv, silu, decay, state, step, slots, out,
                                       powers, rot, cos_sin, k_scale):
            return
    L = _lib.load("plain")
    _lib.check(L.apc_linear_attention(proj.data_ptr(), _code(proj), ld, q_off, k_off, v_off, H, dk, dv,
                                      1 if silu else 0, _f32(decay, H, "decay"), state.data_ptr(), S,
                                      _i32(step.seg_row0, S, "seg_row0"), _i32(step.seg_rows, S, "seg_rows"),
                                      _i32(slots, S, "slots"), out.data_ptr(), ldo, rot,
                                      cos_sin.data_ptr() if rot else 0, _i32(step.positions, T, "positions") if rot else 0,
                                      float(k_scale), _stream()), "linear_attention")


GATES = {"sigmoid": 0, "silu": 1}


def gated_rmsnorm(o: torch.Tensor, weight: Optional[torch.Tensor], eps: float, gate: Optional[torch.Tensor],
                  out: torch.Tensor, group: int = 0, gate_act: str = "sigmoid") -> None:
    """out = rms_norm(o) * weight * sigmoid(gate), the norm over the whole row; o float32, gate (logits) and out any.
    `group` > 0: the norm is taken over every `group` consecutive elements (a head) for itself; `weight` may be None;
    `gate_act` "silu": times gate * sigmoid(gate)."""
    _gpu(o, weight, gate, out)
    T, N = o.shape
    _need(gate_act in GATES and int(group) >= 0 and (not group or N % int(group) == 0),
          "gated_rmsnorm: the gate is 'sigmoid' or 'silu', and a group must divide the row")
    _need(o.dtype == torch.float32 and out.shape == (T, N) and (gate is None or gate.shape == (T, N)),
          "gated_rmsnorm: o float32 [rows, n], gate and out of the same shape")
    L = _lib.load("plain")
    _lib.check(L.apc_gated_rmsnorm(o.data_ptr(), _rows(o, "o"), _f32(weight, N, "norm weight"), float(eps),
                                   gate.data_ptr() if gate is not None else 0, _code(gate) if gate is not None else 0,
                                   _rows(gate, "gate") if gate is not None else 0, out.data_ptr(), _code(out),
                                   _rows(out, "out"), T, N, int(group), GATES[gate_act], _stream()), "gated_rmsnorm")


def diff_combine(a: torch.Tensor, lam: float, post: float, eps: float, gate: Optional[torch.Tensor],
                 out: torch.Tensor, n_heads: int, value_dim: int) -> None:
    """a float32 [rows, heads * 2 * value_dim] (per head: map 1, map 2): o = a1 - lam * a2, divided by its root mean
    square over the head, times `post` and sigmoid(gate[row][head]) (gate logits [rows, heads], or None)."""
    _gpu(a, gate, out)
    T = a.shape[0]
    H, dv = int(n_heads), int(value_dim)
    _need(a.dtype == torch.float32 and a.shape == (T, 2 * H * dv) and out.shape == (T, H * dv),
          "diff_combine: a float32 [rows, heads * 2 * value_dim], out [rows, heads * value_dim]")
    _need(gate is None or gate.shape == (T, H), "diff_combine: gate must be [rows, heads]")
    L = _lib.load("plain")
    _lib.check(L.apc_diff_combine(a.data_ptr(), _rows(a, "a"), float(lam), float(post), float(eps),
                                  gate.data_ptr() if gate is not None else 0, _code(gate) if gate is not None else 0,
                                  _rows(gate, "gate") if gate is not None else 0, out.data_ptr(), _code(out),
                                  _rows(out, "out"), T, H, dv, _stream()), "diff_combine")


# --------------------------------------------------------------------------- routed experts
ROUTER_SCORES = {"softmax": 0, "sigmoid": 1}


def route_topk(z: torch.Tensor, correction: Optional[torch.Tensor], top: int, ids: torch.Tensor,
               weights: torch.Tensor, renormalize: bool = False, score: str = "softmax") -> None:
    """s = softmax(z) over a row (`score` "sigmoid": s = sigmoid(z), every output for itself); the `top` largest of s + correction are chosen (the lower index wins a tie);
    weights = s of the chosen (divided by their sum with `renormalize`).  z float32 [rows, n]."""
    _gpu(z, correction, ids, weights)
    T, N = z.shape
    _need(z.dtype == torch.float32 and weights.dtype == torch.float32 and weights.is_contiguous()
          and weights.numel() >= T * top, "route_topk: z float32, weights contiguous float32 [rows, top]")
    _need(score in ROUTER_SCORES, f"route_topk: score {score!r} is not one of {sorted(ROUTER_SCORES)}")
    L = _lib.load("plain")
    _lib.check(L.apc_route_topk(z.data_ptr(), _rows(z, "router logits"), _f32(correction, N, "correction"), T, N,
                                int(top), 1 if renormalize else 0, ROUTER_SCORES[score], _i32(ids, T * top, "ids"),
                                weights.data_ptr(), _stream()), "route_topk")


def prepare_experts(gate_up: torch.Tensor, down: torch.Tensor, run_dtype: torch.dtype):
    """How the experts' matrices [experts, 2 ff, width] and [experts, width, ff] are kept on the GPU: in the tiled
    layout of the MFMA kernels for a bfloat16 run whose sizes they take, else as they are."""
    if run_dtype == torch.bfloat16 and not FORCE_PLAIN and gate_up.is_cuda and gate_up.dtype == torch.bfloat16:
        from . import tuned
        packed = tuned.pack_experts(gate_up, down)
        if packed is not None:
            return packed
    return gate_up.contiguous(), down.contiguous()


EXPERT_ACTIVATIONS = {"silu": 0, "clamped": 1}


def routed_experts(h: torch.Tensor, w_gate_up, w_down, n_experts: int, ff: int, ids: torch.Tensor,
                   weights: torch.Tensor, top: int, y: torch.Tensor, activation: str = "silu", alpha: float = 1.0,
                   limit: float = 0.0, weight_input: bool = False) -> None:
    """y[t] = sum_k weights[t][k] * expert ids[t][k] (h[t]); experts 0 .. n_experts-1 are gated units
    Wd a(Wg h, Wu h) with w_gate_up [n_experts, 2 * ff, width] (gate rows, then up rows) and w_down
    [n_experts, width, ff]; ids from n_experts on are identity experts.  y float32 [rows, width].
    `activation` "silu": a(g, u) = silu(g) * u; "clamped": g' * sigmoid(alpha g') * (u' + 1) with g' = min(g, limit),
    u' = clamp(u, -limit, limit).  `weight_input`: the weight multiplies the expert's input instead of its output,
    y[t] = sum_k expert(weights[t][k] * h[t]) (identity experts then return the weighted row as well)."""
    T, D = h.shape
    E, F, K = int(n_experts), int(ff), int(top)
    _gpu(h, ids, weights, y)
    _need(y.dtype == torch.float32 and y.shape == (T, D), "routed_experts: y float32 [rows, width]")
    _need(activation in EXPERT_ACTIVATIONS, f"routed_experts: activation {activation!r} is not one of {sorted(EXPERT_ACTIVATIONS)}")
    kind = EXPERT_ACTIVATIONS[activation]
    if not isinstance(w_gate_up, torch.Tensor) and w_gate_up is not None:
        from . import tuned
        tuned.routed_experts_bf16(h, w_gate_up, w_down, E, F, ids, weights, K, y, kind, alpha, limit, weight_input)
        return
    act = torch.empty((T * K, F), dtype=h.dtype, device=h.device)
    L = _lib.load("plain")
    if E:
        _gpu(w_gate_up, w_down)
        _need(w_gate_up.is_contiguous() and tuple(w_gate_up.shape) == (E, 2 * F, D) and w_down.is_contiguous()
              and tuple(w_down.shape) == (E, D, F), "routed_experts: matrices [experts, 2 ff, width] and [experts, width, ff]")
        _lib.check(L.apc_routed_glu(h.data_ptr(), _code(h), _rows(h, "h"), w_gate_up.data_ptr(), _code(w_gate_up), E, F,
                                    D, _i32(ids, T * K, "ids"), K, act.data_ptr(), _code(act), T, kind, float(alpha),
                                    float(limit), _f32(weights, T * K, "weights") if weight_input else 0, _stream()),
                   "routed_glu")
    _lib.check(L.apc_routed_down(act.data_ptr(), _code(act), w_down.data_ptr() if E else 0,
                                 _code(w_down) if E else 0, E, F, D, _i32(ids, T * K, "ids"),
                                 _f32(weights, T * K, "weights"), K, h.data_ptr(), _code(h), _rows(h, "h"),
                                 y.data_ptr(), _rows(y, "y"), T, 1 if weight_input else 0, _stream()), "routed_down")


# --------------------------------------------------------------------------- selective scan, activations, biases
ACTIVATIONS = {"none": 0, "silu": 1, "relu2": 2, "gelu_tanh": 3}


def conv_channels(x: torch.Tensor, channels: int, conv_w: torch.Tensor, bias: Optional[torch.Tensor],
                  state: Optional[torch.Tensor], step, slots: Optional[torch.Tensor], activation: str,
                  out: torch.Tensor) -> None:
    """A short causal convolution over time on the first `channels` columns of x, the bias behind it, then the
    activation: out[t][c] = act(sum_j conv_w[c][j] * x[t - (taps - 1) + j][c] + bias[c]) inside a segment; the inputs
    of the positions ahead of a segment come from `state` float32 [slots + 1, taps - 1, channels], which is moved on to
    the segment's last inputs."""
    _gpu(x, conv_w, bias, state, slots, out)
    ldx, ldo = _rows(x, "conv input"), _rows(out, "conv out")
    T, C = x.shape[0], int(channels)
    _need(activation in ACTIVATIONS, f"conv_channels: activation {activation!r} is not one of {sorted(ACTIVATIONS)}")
    _need(C <= x.shape[1] and out.shape == (T, C), "conv_channels: out must be [rows, channels]")
    _need(conv_w.dim() == 2 and conv_w.shape[0] == C and conv_w.dtype == torch.float32 and conv_w.is_contiguous(),
          "conv_channels: weights must be float32 [channels, taps]")
    taps = int(conv_w.shape[1])
    S = step.n_segs
    if taps > 1:
        _need(state is not None and slots is not None and state.dim() == 3 and state.is_contiguous()
              and state.dtype == torch.float32 and tuple(state.shape[1:]) == (taps - 1, C),
              f"conv_channels: state must be float32 [slots, {taps - 1}, {C}]")
    L = _lib.load("plain")
    _lib.check(L.apc_conv_channels(x.data_ptr(), _code(x), ldx, T, C, conv_w.data_ptr(), _f32(bias, C, "bias"), taps,
                                   state.data_ptr() if taps > 1 else 0, _i32(step.row_seg, T, "row_seg"),
                                   _i32(step.seg_row0, S, "seg_row0"), _i32(slots, S, "slots") if taps > 1 else 0,
                                   ACTIVATIONS[activation], out.data_ptr(), _code(out), ldo, _stream()),
               "conv_channels")
    if taps > 1:
        _lib.check(L.apc_conv_state(x.data_ptr(), _code(x), ldx, 0, taps, state.data_ptr(), C, S,
                                    _i32(step.seg_row0, S, "seg_row0"), _i32(step.seg_rows, S, "seg_rows"),
                                    _i32(slots, S, "slots"), _stream()), "conv_state")


def selective_scan(x: torch.Tensor, dt: torch.Tensor, dt_bias: Optional[torch.Tensor], A: torch.Tensor,
                   bc: torch.Tensor, D: Optional[torch.Tensor], z: torch.Tensor, state: torch.Tensor, step,
                   slots: torch.Tensor, out: torch.Tensor) -> None:
    """Per channel c with N states, over the rows of every segment in order:
      d = softplus(dt[t][c] + dt_bias[c]);  S[c][n] <- exp(d A[c][n]) S[c][n] + d x[t][c] B[t][n]
      out[t][c] = (sum_n S[c][n] C[t][n] + D[c] x[t][c]) * silu(z[t][c])
    x, z, out [rows, channels] (any element type), dt float32 [rows, channels], bc float32 [rows, 2 N] (B, then C),
    A float32 [channels, N], state float32 [slots + 1, channels, N]."""
    _gpu(x, dt, dt_bias, A, bc, D, z, state, slots, out)
    T, C = out.shape
    N = int(A.shape[1])
    _need(x.shape == (T, C) and z.shape == (T, C) and dt.shape == (T, C) and dt.dtype == torch.float32
          and bc.shape == (T, 2 * N) and bc.dtype == torch.float32, "selective_scan: x, z, dt [rows, channels], bc float32 [rows, 2 N]")
    _need(A.dtype == torch.float32 and A.is_contiguous() and tuple(A.shape) == (C, N), "selective_scan: A float32 [channels, N]")
    _need(state.dtype == torch.float32 and state.is_contiguous() and tuple(state.shape[1:]) == (C, N),
          f"selective_scan: state must be float32 [slots, {C}, {N}]")
    S = step.n_segs
    if _tuned_ok(x, z, out):
        from . import tuned
        if tuned.selective_scan_bf16(x, dt, dt_bias, A, bc, D, z, state, step, slots, out):
            return
    L = _lib.load("plain")
    _lib.check(L.apc_selective_scan(x.data_ptr(), _code(x), _rows(x, "x"), dt.data_ptr(), _rows(dt, "dt"),
                                    _f32(dt_bias, C, "dt bias"), A.data_ptr(), bc.data_ptr(), _rows(bc, "B and C"),
                                    _f32(D, C, "D"), z.data_ptr(), _code(z), _rows(z, "z"), state.data_ptr(), C, N, S,
                                    _i32(step.seg_row0, S, "seg_row0"), _i32(step.seg_rows, S, "seg_rows"),
                                    _i32(slots, S, "slots"), out.data_ptr(), _code(out), _rows(out, "out"), _stream()),
               "selective_scan")


def act_rows(x: torch.Tensor, out: torch.Tensor, activation: str) -> None:
    """out = act(x) element by element: "silu", "relu2" (the square of max(x, 0)), "gelu_tanh", "none"."""
    _gpu(x, out)
    _need(activation in ACTIVATIONS, f"act_rows: activation {activation!r} is not one of {sorted(ACTIVATIONS)}")
    _need(x.shape == out.shape, "act_rows: shapes differ")
    ldi, ldo = _rows(x, "act in"), _rows(out, "act out")
    T, n = x.shape
    L = _lib.load("plain")
    _lib.check(L.apc_act_rows(x.data_ptr(), _code(x), ldi, out.data_ptr(), _code(out), ldo, T, n,
                              ACTIVATIONS[activation], _stream()), "act_rows")


def bias_rows(x: torch.Tensor, bias: torch.Tensor) -> None:
    """x[t] += bias (x float32 [rows, n], bias float32 [n])."""
    _gpu(x, bias)
    ldx = _rows(x, "bias x")
    T, n = x.shape
    _need(x.dtype == torch.float32, "bias_rows: x float32")
    L = _lib.load("plain")
    _lib.check(L.apc_bias_rows(x.data_ptr(), ldx, _f32(bias, n, "bias"), T, n, _stream()), "bias_rows")


def weighted_pair(u: torch.Tensor, a: float, v: torch.Tensor, b: float, out: torch.Tensor) -> None:
    """out = a * u + b * v (float32 rows; out may be u)."""
    _gpu(u, v, out)
    T, n = out.shape
    _need(u.shape == (T, n) and v.shape == (T, n) and all(t.dtype == torch.float32 for t in (u, v, out)),
          "weighted_pair: three float32 [rows, n]")
    L = _lib.load("plain")
    _lib.check(L.apc_weighted_pair(out.data_ptr(), _rows(out, "out"), u.data_ptr(), _rows(u, "u"), float(a),
                                   v.data_ptr(), _rows(v, "v"), float(b), T, n, _stream()), "weighted_pair")


def linear_act(a: torch.Tensor, w, out: torch.Tensor, activation: str) -> None:
    """out = act(a . w^T): the product's sums are 32-bit, the activation is applied to them before they are stored in
    `out`'s element type."""
    _need(activation in ACTIVATIONS, f"linear_act: activation {activation!r} is not one of {sorted(ACTIVATIONS)}")
    T, n = out.shape
    sums = torch.empty((T, n), dtype=torch.float32, device=a.device)
    linear(a, w, sums)
    act_rows(sums, out, activation)
